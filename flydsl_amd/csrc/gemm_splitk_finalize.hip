// Second pass of the split-K tiled path: sums the per-split accumulator slices in a fixed order (deterministic)
// and applies the same epilogue as the single-pass kernels.  One thread per four consecutive columns.
#include "psg_common.h"

namespace {

template <int IS_INT>
__global__ void __launch_bounds__(256) k_splitk_finalize(A8W8Params p, const void* partial, int scaled) {
    const size_t quads = (size_t)p.M * (size_t)(p.N >> 2);
    const size_t q = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (q >= quads) return;
    const int m = (int)(q / (size_t)(p.N >> 2));
    const int n = (int)(q % (size_t)(p.N >> 2)) << 2;
    const size_t idx = (size_t)m * (size_t)p.N + (size_t)n;
    const size_t slice = (size_t)p.M * (size_t)p.N;
    v4f x;
    if constexpr (IS_INT) {
        v4i sum = *reinterpret_cast<const v4i*>(static_cast<const int*>(partial) + idx);
        for (int s = 1; s < p.splits; s++) sum += *reinterpret_cast<const v4i*>(static_cast<const int*>(partial) + s * slice + idx);
        x = (v4f){(float)sum[0], (float)sum[1], (float)sum[2], (float)sum[3]};
    } else {
        v4f sum = *reinterpret_cast<const v4f*>(static_cast<const float*>(partial) + idx);
        for (int s = 1; s < p.splits; s++) sum += *reinterpret_cast<const v4f*>(static_cast<const float*>(partial) + s * slice + idx);
        x = sum;
    }
    if (scaled) {
        const float sa = p.sa[m];
        const v4f sb = *reinterpret_cast<const v4f*>(p.sb + n);
        x = (v4f){(x[0] * sa) * sb[0], (x[1] * sa) * sb[1], (x[2] * sa) * sb[2], (x[3] * sa) * sb[3]};
    }
    store_c4(p, idx, n, x);
}

}  // namespace

// p.c / p.sa / p.sb / p.bias / p.epi / p.out describe the final output; p.splits slices of [M,N] accumulators at `partial`
hipError_t psg_launch_splitk_finalize(const A8W8Params& p, const void* partial, int is_int, int scaled, hipStream_t stream) {
    const size_t quads = (size_t)p.M * (size_t)(p.N >> 2);
    const unsigned grid = (unsigned)((quads + 255) / 256);
    if (is_int) hipLaunchKernelGGL((k_splitk_finalize<1>), dim3(grid), dim3(256), 0, stream, p, partial, scaled);
    else hipLaunchKernelGGL((k_splitk_finalize<0>), dim3(grid), dim3(256), 0, stream, p, partial, scaled);
    return hipGetLastError();
}
