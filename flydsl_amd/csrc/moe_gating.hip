// Router gating in front of the MoE expert sorter: softmax over the experts, top-k, optional renormalisation.
// One group of L lanes per token (L * VPT >= experts, VPT <= 16 values per lane), 256 / L tokens per workgroup, no LDS:
// every reduction is a butterfly inside the group.  The launch reads tokens * experts logits and writes 12 bytes per
// (token, slot), so it is bound by launch latency for decode and by HBM for prefill.
#include "moe_gating.h"

namespace {

template <typename T, int VPT>
__global__ void __launch_bounds__(256) k_topk_gating(MoeGatingParams p) {
    const int L = p.lanes, sh = __builtin_ctz(L);
    const int gl = threadIdx.x & (L - 1);
    const int t = (int)blockIdx.x * (256 >> sh) + (int)(threadIdx.x >> sh);
    const bool live = t < p.tokens;
    const T* row = static_cast<const T*>(p.gating) + (size_t)(live ? t : 0) * p.experts;
    float keep[GATE_KEEP];
    const float f = gate_row<T, VPT>(row, p.experts, p.topk, p.renorm != 0, L, gl, p.vec != 0, keep, [&](int k, int index) {
        if (live && gl == 0) {
            p.indices[(size_t)t * p.topk + k] = index;
            if (p.tei) p.tei[(size_t)t * p.topk + k] = k * p.tokens + t;
        }
    });
    // lane k % L holds the weight of winner k
    if (live) {
#pragma unroll
        for (int j = 0; j < GATE_KEEP; j++) {
            const int k = (j << sh) + gl;
            if (k < p.topk) p.weights[(size_t)t * p.topk + k] = keep[j] * f;
        }
    }
}

template <typename T>
hipError_t launch_t(const MoeGatingParams& p, int vpt, hipStream_t stream) {
    const int tpb = 256 / p.lanes;
    const dim3 grid((p.tokens + tpb - 1) / tpb), block(256);
    switch (vpt) {
        case 1: hipLaunchKernelGGL((k_topk_gating<T, 1>), grid, block, 0, stream, p); break;
        case 2: hipLaunchKernelGGL((k_topk_gating<T, 2>), grid, block, 0, stream, p); break;
        case 4: hipLaunchKernelGGL((k_topk_gating<T, 4>), grid, block, 0, stream, p); break;
        case 8: hipLaunchKernelGGL((k_topk_gating<T, 8>), grid, block, 0, stream, p); break;
        default: hipLaunchKernelGGL((k_topk_gating<T, 16>), grid, block, 0, stream, p); break;
    }
    return hipGetLastError();
}

}  // namespace

int psg_gate_max_experts() { return GATE_MAX_EXPERTS; }
int psg_gate_max_topk() { return GATE_MAX_TOPK; }

// dtype: 0 fp32, 1 bf16, 2 fp16.  Fills p.lanes / p.vec.
hipError_t psg_launch_moe_gating(MoeGatingParams p, int dtype, hipStream_t stream) {
    int vpt, lanes;
    gate_layout(p.experts, &vpt, &lanes);
    const int esz = dtype == 0 ? 4 : 2;
    const int chunk = vpt * esz;  // bytes a lane fetches; needs that alignment (at most 16 matter: wider loads are split)
    const int need = chunk < 16 ? chunk : 16;
    p.lanes = lanes;
    p.vec = p.experts % vpt == 0 && reinterpret_cast<uintptr_t>(p.gating) % need == 0 && ((size_t)p.experts * esz) % need == 0;
    switch (dtype) {
        case 0: return launch_t<float>(p, vpt, stream);
        case 1: return launch_t<uint16_t>(p, vpt, stream);
        case 2: return launch_t<_Float16>(p, vpt, stream);
    }
    return hipErrorInvalidValue;
}
