// Softmax + top-k of one token's router logits by a group of L lanes (L a power of two <= 64), shared by the stand-alone
// gating kernel and the fused gating + sorting launch.
//
// Arithmetic (the reference's kernels/moe/topk_gating_softmax_kernel.py:545-630): fp32 throughout; p = exp2((x - max) *
// log2(e)) * (1 / sum); top-k by k rounds of arg-max over p with the lower expert index winning ties, the winner masked
// with -inf; optional renormalisation w * (1 / max(sum of the k winners, 1e-20)).
#pragma once
#include "psg_common.h"

constexpr int GATE_MAX_TOPK = 32;
constexpr int GATE_MAX_EXPERTS = 1024;  // 64 lanes x 16 values

template <typename T>
__device__ __forceinline__ float gate_to_f32(T v);
template <>
__device__ __forceinline__ float gate_to_f32<float>(float v) { return v; }
template <>
__device__ __forceinline__ float gate_to_f32<_Float16>(_Float16 v) { return (float)v; }
template <>
__device__ __forceinline__ float gate_to_f32<uint16_t>(uint16_t v) { return __builtin_bit_cast(float, (uint32_t)v << 16); }  // bf16 bits

// Exchange step S of a butterfly over a group of 2, 4, 8, 16, 32 or 64 lanes: every lane gets the value of lane ^ mask with
// masks 1, 2, 7, 15 (DPP: quad permutes, half-row mirror, row mirror; any masks that span the group make a butterfly), then
// 16 and 32 through the LDS crossbar.  Steps 0 .. log2(L)-1 cover a group of L lanes.
template <int S>
__device__ __forceinline__ int gate_xchg(int v) {
    if constexpr (S == 0) return __builtin_amdgcn_update_dpp(v, v, 0xB1, 0xF, 0xF, false);   // quad_perm [1,0,3,2]
    else if constexpr (S == 1) return __builtin_amdgcn_update_dpp(v, v, 0x4E, 0xF, 0xF, false);  // quad_perm [2,3,0,1]
    else if constexpr (S == 2) return __builtin_amdgcn_update_dpp(v, v, 0x141, 0xF, 0xF, false); // row_half_mirror
    else if constexpr (S == 3) return __builtin_amdgcn_update_dpp(v, v, 0x140, 0xF, 0xF, false); // row_mirror
    else if constexpr (S == 4) return __shfl_xor(v, 16);
    else return __shfl_xor(v, 32);
}
template <int S>
__device__ __forceinline__ float gate_xchg(float v) { return __builtin_bit_cast(float, gate_xchg<S>(__builtin_bit_cast(int, v))); }

constexpr int GATE_KEEP = 16;  // winners a lane may have to keep: topk <= experts <= 16 * lanes

// Lane gl of the group owns the columns [gl * VPT, gl * VPT + VPT) of `row`; columns >= E count as -inf.  `vec`: every
// lane's columns can be fetched as one aligned vector (E % VPT == 0, base and row pitch aligned).  All L lanes of the
// group must call this together.  Winner k (k = 0 .. K-1, descending weight) is reported through found(k, index) on every
// lane, and its weight stays with lane k % L in keep[k / L]; the return value is the factor to apply to the weights
// (1 without renormalisation), the same on every lane.
template <typename T, int VPT, class F>
__device__ __forceinline__ float gate_row(const T* row, int E, int K, bool renorm, int L, int gl, bool vec, float (&keep)[GATE_KEEP], F&& found) {
    struct alignas(sizeof(T) * VPT) Vec {
        T v[VPT];
    };
    const int sh = __builtin_ctz(L);
    const int c0 = gl * VPT;
    float x[VPT];
    if (vec) {
        if (c0 < E) {
            const Vec raw = *reinterpret_cast<const Vec*>(row + c0);
#pragma unroll
            for (int v = 0; v < VPT; v++) x[v] = gate_to_f32<T>(raw.v[v]);
        } else {
#pragma unroll
            for (int v = 0; v < VPT; v++) x[v] = -INFINITY;
        }
    } else {
#pragma unroll
        for (int v = 0; v < VPT; v++) x[v] = c0 + v < E ? gate_to_f32<T>(row[c0 + v]) : -INFINITY;
    }
    float mx = -INFINITY;
#pragma unroll
    for (int v = 0; v < VPT; v++) mx = fmaxf(mx, x[v]);
    static_for<6>([&](auto S) {
        if (decltype(S)::value < sh) mx = fmaxf(mx, gate_xchg<decltype(S)::value>(mx));
    });
    float sum = 0.f;
#pragma unroll
    for (int v = 0; v < VPT; v++) {
        x[v] = __builtin_amdgcn_exp2f((x[v] - mx) * 1.4426950408889634f);  // the hardware exp2 (the reference's is fast-math too); exp2(-inf) = 0
        sum += x[v];
    }
    static_for<6>([&](auto S) {
        if (decltype(S)::value < sh) sum += gate_xchg<decltype(S)::value>(sum);
    });
    const float inv = __builtin_amdgcn_rcpf(sum);  // sum >= 1 (the maximum contributes exp2(0))
#pragma unroll
    for (int v = 0; v < VPT; v++) x[v] = c0 + v < E ? x[v] * inv : -INFINITY;
    float picked = 0.f;
    for (int k = 0; k < K; k++) {
        // arg-max of the lane's values as a tree (short dependency chains: one wavefront per SIMD has nothing else to
        // issue); the higher column of a pair wins only when strictly greater, so the lowest column of equal values stays
        float tv[VPT];
        int ti[VPT];
#pragma unroll
        for (int v = 0; v < VPT; v++) {
            tv[v] = x[v];
            ti[v] = c0 + v;
        }
#pragma unroll
        for (int w = 1; w < VPT; w <<= 1)
#pragma unroll
            for (int v = 0; v + w < VPT; v += 2 * w) {
                const bool hi = tv[v + w] > tv[v];
                tv[v] = hi ? tv[v + w] : tv[v];
                ti[v] = hi ? ti[v + w] : ti[v];
            }
        float bv = tv[0];
        int bi = tv[0] == -INFINITY ? -1 : ti[0];
        static_for<6>([&](auto S) {
            if (decltype(S)::value < sh) {
                const float pv = gate_xchg<decltype(S)::value>(bv);
                const int pi = gate_xchg<decltype(S)::value>(bi);
                const bool take = pv > bv || (pv == bv && pi < bi);
                bv = take ? pv : bv;
                bi = take ? pi : bi;
            }
        });
        found(k, bi);
        const int slot = k >> sh;
        const bool mine = gl == (k & (L - 1));
#pragma unroll
        for (int j = 0; j < GATE_KEEP; j++)
            if (j == slot) keep[j] = mine ? bv : keep[j];  // (slot is uniform: one predicated move per round)
        picked += bv;
#pragma unroll
        for (int v = 0; v < VPT; v++) x[v] = c0 + v == bi ? -INFINITY : x[v];
    }
    return renorm ? 1.0f / fmaxf(picked, 1e-20f) : 1.0f;
}

// (values per lane, lanes per token) for E experts: 16 values per lane from 16 experts on, lanes a power of two
inline void gate_layout(int E, int* vpt, int* lanes) {
    int v = 1;
    while (v < 16 && v < E) v <<= 1;
    int l = 1;
    while (l * v < E) l <<= 1;
    *vpt = v;
    *lanes = l;
}

struct MoeGatingParams {
    const void* gating;   // [tokens, experts] fp32 / bf16 / fp16
    float* weights;       // [tokens, topk]
    int32_t* indices;     // [tokens, topk]
    int32_t* tei;         // [tokens, topk] = k * tokens + token, or nullptr
    int tokens, experts, topk, renorm;
    int lanes;            // lanes per token
    int vec;              // 1: aligned vector loads
};
