"""MoE grouped GEMMs over the preshuffled weight layout (the reference's ``kernels/moe/moe_gemm_2stage`` call shapes)."""
