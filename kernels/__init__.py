"""Import path of the reference's pre-built kernel library (``kernels.gemm.*``), so that callers of
``kernels.gemm.preshuffle_gemm.compile_preshuffle_gemm`` and ``kernels.gemm.mxfp4_preshuffle.launch_gemm``
need no change.  Only the preshuffle GEMM lives here."""
