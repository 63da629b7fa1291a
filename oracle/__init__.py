"""CPU oracle for the preshuffle quantized GEMM path -- test infrastructure, never shipped."""
