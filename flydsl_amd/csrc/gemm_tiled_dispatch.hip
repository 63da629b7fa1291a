// Host entry of the tiled MFMA mainloop used by the C-ABI layer.  kind: KIND_INT8 / KIND_FP8 / KIND_FP16 / KIND_BF16 /
// KIND_MXFP4 / KIND_MXFP8.  tile_m x tile_n must be one of the instantiated shapes: 256x256, 128x512, 128x256, 64x256, 32x256, then
// 128x128 and 64x64 (8- and 16-bit) or 64x128 and 32x128 (MXFP4, MXFP8).
#include "psg_common.h"
#include "tile_order.h"

hipError_t psg_launch_tiled_int8(const A8W8Params& p, int store, int tile_m, int tile_n, hipStream_t stream);
hipError_t psg_launch_tiled_fp8(const A8W8Params& p, int store, int tile_m, int tile_n, hipStream_t stream);
hipError_t psg_launch_tiled_fp16(const A8W8Params& p, int store, int tile_m, int tile_n, hipStream_t stream);
hipError_t psg_launch_tiled_bf16(const A8W8Params& p, int store, int tile_m, int tile_n, hipStream_t stream);
hipError_t psg_launch_tiled_mxfp4(const A8W8Params& p, int store, int tile_m, int tile_n, hipStream_t stream);
hipError_t psg_launch_tiled_mxfp8(const A8W8Params& p, int store, int tile_m, int tile_n, hipStream_t stream);

hipError_t psg_launch_a8w8_tiled(const A8W8Params& p, int kind, int store, int tile_m, int tile_n, hipStream_t stream) {
    // the plain bf16 store without bias/activation has its own instantiation; everything else is the generic epilogue
    if (store == STORE_C && (p.epi != EPI_NONE || p.out != OUT_BF16)) store = STORE_C_GENERIC;
    switch (kind) {
        case KIND_INT8: return psg_launch_tiled_int8(p, store, tile_m, tile_n, stream);
        case KIND_FP8: return psg_launch_tiled_fp8(p, store, tile_m, tile_n, stream);
        case KIND_FP16: return psg_launch_tiled_fp16(p, store, tile_m, tile_n, stream);
        case KIND_BF16: return psg_launch_tiled_bf16(p, store, tile_m, tile_n, stream);
        case KIND_MXFP4: return psg_launch_tiled_mxfp4(p, store, tile_m, tile_n, stream);
        case KIND_MXFP8: return psg_launch_tiled_mxfp8(p, store, tile_m, tile_n, stream);
    }
    return hipErrorInvalidValue;
}

// Writes, for every workgroup id of a tiles_m x tiles_n launch, the tile (tm, tn) the tiled kernel would work on:
// out[2*id] = tm, out[2*id+1] = tn.  Lets a test compare the device's tile order with the host function.
namespace {
__global__ void __launch_bounds__(64) k_tile_order(int tiles_m, int tiles_n, int group_m, int32_t* out) {
    if (threadIdx.x != 0) return;
    int tm, tn;
    psg_tile_order((int)blockIdx.x, tiles_m, tiles_n, group_m, &tm, &tn);
    out[2 * blockIdx.x] = tm;
    out[2 * blockIdx.x + 1] = tn;
}
}  // namespace

hipError_t psg_launch_tile_order(int tiles_m, int tiles_n, int group_m, int32_t* out, hipStream_t stream) {
    hipLaunchKernelGGL(k_tile_order, dim3(tiles_m * tiles_n), dim3(64), 0, stream, tiles_m, tiles_n, group_m, out);
    return hipGetLastError();
}
