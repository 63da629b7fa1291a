// Instantiations of the tiled MFMA mainloop (gemm_tiled.h, gemm_tiled8.h) for int8 operands; one translation unit per operand
// type so that the instantiations compile in parallel.
#include "gemm_tiled8.h"

hipError_t psg_launch_tiled_int8(const A8W8Params& p, int store, int tile_m, int tile_n, hipStream_t stream) {
    if (store == STORE_ACC) return launch_shape<KIND_INT8, STORE_ACC>(p, tile_m, tile_n, stream);
    if (store == STORE_C_GENERIC) return launch_shape<KIND_INT8, STORE_C_GENERIC>(p, tile_m, tile_n, stream);
    return launch_shape<KIND_INT8, STORE_C>(p, tile_m, tile_n, stream);
}
