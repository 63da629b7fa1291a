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

// Lane gl of the group owns the columns [gl * VPT, gl * VPT + VPT) of `row`; columns >= E count as -inf.  `vec`: every
// lane's columns can be fetched as one aligned vector (E % VPT == 0, base and row pitch aligned).  All L lanes of the
// group must call this together; all of them return the same winners in sel_w / sel_i (entries 0 .. K-1) and the
// factor to apply to the weights (1 without renormalisation).
template <typename T, int VPT>
__device__ __forceinline__ float gate_row(const T* row, int E, int K, bool renorm, int L, int gl, bool vec,
                                          float (&sel_w)[GATE_MAX_TOPK], int (&sel_i)[GATE_MAX_TOPK]) {
    struct alignas(sizeof(T) * VPT) Vec {
        T v[VPT];
    };
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
    for (int o = L >> 1; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    float sum = 0.f;
#pragma unroll
    for (int v = 0; v < VPT; v++) {
        x[v] = exp2f((x[v] - mx) * 1.4426950408889634f);  // exp2(-inf) = 0 for the columns past E
        sum += x[v];
    }
    for (int o = L >> 1; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
    const float inv = 1.0f / sum;
#pragma unroll
    for (int v = 0; v < VPT; v++) x[v] = c0 + v < E ? x[v] * inv : -INFINITY;
    float picked = 0.f;
    for (int k = 0; k < K; k++) {
        float bv = -INFINITY;
        int bi = -1;
#pragma unroll
        for (int v = 0; v < VPT; v++) {
            const bool better = x[v] > bv;  // strict: the lowest column of equal values stays
            bv = better ? x[v] : bv;
            bi = better ? c0 + v : bi;
        }
        for (int o = L >> 1; o > 0; o >>= 1) {
            const float pv = __shfl_xor(bv, o);
            const int pi = __shfl_xor(bi, o);
            const bool take = pv > bv || (pv == bv && pi < bi);
            bv = take ? pv : bv;
            bi = take ? pi : bi;
        }
#pragma unroll
        for (int j = 0; j < GATE_MAX_TOPK; j++) {
            sel_w[j] = j == k ? bv : sel_w[j];
            sel_i[j] = j == k ? bi : sel_i[j];
        }
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
