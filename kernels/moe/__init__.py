"""Import path of the reference's ``kernels.moe`` package; only the 2-stage fp8 / int8 grouped GEMMs live here."""
