// Shared device helpers for the preshuffle GEMM kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

enum { KIND_INT8 = 0, KIND_FP8 = 1, KIND_FP16 = 2, KIND_BF16 = 3, KIND_MXFP4 = 4, KIND_MXFP8 = 5, KIND_INT8W4 = 6 };
enum { OUT_BF16 = 0, OUT_FP16 = 1 };
enum { EPI_NONE = 0, EPI_BIAS = 1, EPI_BIAS_RELU = 2, EPI_BIAS_SILU = 3, EPI_BIAS_GELU = 4 };
// what a kernel writes: the scaled/activated C, or the raw accumulators
enum { STORE_C = 0, STORE_ACC = 1, STORE_C_GENERIC = 2 };

// Raw buffer resource over [base, base+bytes): loads past the end return 0, stores past it are dropped.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint64_t bytes) {
    uint32_t n = bytes > 0xFFFFFFFFull ? 0xFFFFFFFFu : (uint32_t)bytes;
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)n, 0x00020000);
}

__device__ __forceinline__ v4i buf_load16(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
    return (v4i)__builtin_amdgcn_raw_buffer_load_b128(r, (int)voff, (int)soff, 0);
}

// non-temporal variant for data that is streamed exactly once
__device__ __forceinline__ v4i buf_load16_nt(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
    return (v4i)__builtin_amdgcn_raw_buffer_load_b128(r, (int)voff, (int)soff, 2);
}

__device__ __forceinline__ v2i buf_load8(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
    return (v2i)__builtin_amdgcn_raw_buffer_load_b64(r, (int)voff, (int)soff, 0);
}

__device__ __forceinline__ int buf_load4(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
    return (int)__builtin_amdgcn_raw_buffer_load_b32(r, (int)voff, (int)soff, 0);
}

__device__ __forceinline__ int wave_id() { return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)); }

template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1>{});
    }
}

// bias / activation of the fused epilogue, fp32 in, fp32 out
template <int EPI>
__device__ __forceinline__ float epi_act(float v, float bias) {
    if constexpr (EPI != EPI_NONE) v = v + bias;
    if constexpr (EPI == EPI_BIAS_RELU) v = fmaxf(v, 0.0f);
    if constexpr (EPI == EPI_BIAS_SILU) {
        float e = __expf(-v);
        v = v * (1.0f / (1.0f + e));
    }
    if constexpr (EPI == EPI_BIAS_GELU) {
        float x3 = v * v * v;
        float y = 0.7978845608f * (v + 0.044715f * x3);
        float e = __expf(-2.0f * fabsf(y));
        float num = y > 0.0f ? 2.0f : 2.0f * e;
        v = 0.5f * v * (num * (1.0f / (1.0f + e)));
    }
    return v;
}

template <int OUT>
__device__ __forceinline__ uint16_t to_out16(float v) {
    if constexpr (OUT == OUT_BF16) {
        __bf16 h = (__bf16)v;
        return __builtin_bit_cast(uint16_t, h);
    } else {
        _Float16 h = (_Float16)v;
        return __builtin_bit_cast(uint16_t, h);
    }
}

template <int OUT>
__device__ __forceinline__ float from_out16(uint16_t b) {
    if constexpr (OUT == OUT_BF16) {
        return __builtin_bit_cast(float, (uint32_t)b << 16);
    } else {
        return (float)__builtin_bit_cast(_Float16, b);
    }
}

// four fp32 -> four 16-bit outputs packed into 8 bytes; two values per conversion instruction (v_cvt_pk_bf16_f32 /
// v_cvt_pk_f16_f32, round to nearest even like the scalar conversions)
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
template <int OUT>
__device__ __forceinline__ int pack2_out16(float a, float b) {
    const v2f x = {a, b};
    if constexpr (OUT == OUT_BF16) {
        return __builtin_bit_cast(int, __builtin_convertvector(x, v2bf));
    } else {
        return __builtin_bit_cast(int, __builtin_convertvector(x, v2h));
    }
}
template <int OUT>
__device__ __forceinline__ v2i pack4_out16(float a, float b, float c, float d) {
    v2i r;
    r[0] = pack2_out16<OUT>(a, b);
    r[1] = pack2_out16<OUT>(c, d);
    return r;
}

// compute units of the current device (host; defined next to psg_init, read once)
int psg_cu_count();

// Arguments shared by the 8-bit kernels.  Plain data, passed by value.
struct A8W8Params {
    void* c;             // [M,N] out16, or raw accumulators when STORE_ACC
    const uint8_t* a;    // [M,K]
    const uint8_t* b;    // preshuffled [N,K]
    const float* sa;     // [M]
    const float* sb;     // [N]
    const uint16_t* bias;  // [N] out16
    int M, N, K;
    int group_m;  // M-tiles per group of the XCD-aware tile order (tiled kernel)
    int ksplit;   // K splits per n-block (small-M kernel)
    int splits;   // tiled kernel: workgroups along K per tile (> 1 only with STORE_ACC into a partials buffer)
    int wave_layout;  // tiled kernel: 2 = 2x2 wavefronts for the 256x256 tile, else 1x4
    int epi;      // EPI_*
    int out;      // OUT_*
    int b_rowmajor;  // 0: W preshuffled (1 KB fragment blocks); 1: W plain row-major [N,K] (8- and 16-bit kinds only)
    const uint8_t* mx_sa;  // MXFP4 only: shuffled e8m0 [ceil(M/32)*32, K/32]
    const uint8_t* mx_sb;  // MXFP4 only: shuffled e8m0 [N, K/32]
};

struct MxParams {
    void* c;
    const uint8_t* a;    // [M,K/2]
    const uint8_t* b;    // preshuffled [N,K/2]
    const uint8_t* sa;   // shuffled e8m0 [ceil(M/32)*32, K/32]
    const uint8_t* sb;   // shuffled e8m0 [N, K/32]
    int M, N, K;
    int group_m;
    int ksplit;
    int out;  // OUT_*
};

// Arguments of the general MX kernel: any of fp4 / fp6 / fp8 A against fp4 / fp8 W, strided-batched.
enum { MXF_FP4 = 0, MXF_FP6 = 1, MXF_FP8 = 2 };
struct MxGenParams {
    void* c;
    const uint8_t* a;    // A rows: fp4 K/2 bytes; fp8 K bytes; fp6 K bytes (per 32 elements 24 packed bytes + 8 of padding)
    const uint8_t* b;    // preshuffled W: K/2 bytes per row (fp4) or K (fp8)
    const uint8_t* sa;   // shuffled e8m0, 32-row chunks of (K/256)*256 bytes
    const uint8_t* sb;
    int M, N, K;
    int out;             // OUT_*
    int splits;          // workgroups along K per tile (> 1 only with STORE_ACC into a partials buffer, batch 1)
    int64_t a_row_stride;      // bytes between rows of A
    int64_t c_row_stride;      // ELEMENTS between rows of C
    int64_t sa_chunk_stride;   // bytes between 32-row chunks of scale_a
    int64_t a_batch, b_batch, c_batch, sa_batch, sb_batch;  // bytes between batches
};

// Arguments of the MoE grouped GEMMs (gate-up stage and down stage) over sorted token blocks.
constexpr int OUT_F32 = 2;
struct MoeParams {
    void* out;
    const uint8_t* x;           // stage 1: [tokens, K]; stage 2: [tokens*topk, K]
    const uint8_t* w;           // preshuffled [experts * rows_per_expert, K] (rows_per_expert = 2*inter or model_dim); K/2 bytes
                                // per row for packed int4
    const float* sx;            // one scale per row of x
    const float* sw;            // [experts * rows_per_expert]
    const int32_t* sorted_ids;  // (slot << 24) | token per sorted row; padding rows hold token >= tokens
    const int32_t* expert_ids;  // expert of each block of block_m sorted rows
    const float* sorted_w;      // routing weight per sorted row
    const int32_t* num_valid;   // [0] = number of sorted rows in use (a multiple of block_m)
    int tokens, topk, experts;
    int n_out;                  // inter_dim (stage 1) or model_dim (stage 2)
    int K;                      // model_dim (stage 1) or inter_dim (stage 2)
    int sorted_size;            // entries of sorted_ids / sorted_w
    int out_dtype;              // OUT_BF16 / OUT_FP16 / OUT_F32 (stage 2 with accumulate only)
    int doweight;               // multiply by the routing weight in this stage
    int accumulate;             // stage 2: atomic add into out[token] (else one row per (token, slot))
    int x_slot_major;           // stage 1: x / sx hold one row per (slot, token) at slot*tokens + token
    int pair_blocks;            // blocks of 16 / 32 rows: multiply two consecutive blocks of one expert in one workgroup
};

// Arguments of the MX (fp4 weights, e8m0 scales per 32 K elements) MoE grouped GEMMs over sorted token blocks.
struct MoeMxParams {
    void* out;                  // stage 1: packed fp4 codes [sorted_size, inter/2]; stage 2: 16-bit [tokens, model_dim] (atomic) or
                                // [sorted_size, model_dim] (one row per sorted position, unweighted)
    uint8_t* out_scale;         // stage 1: e8m0 scales of `out` over sorted rows, shuffled: per (32 rows, 256 columns) 64 dwords
    const uint8_t* a;           // stage 1: [tokens, K/2] fp4 or [tokens, K] fp8 (gathered by token id); stage 2: [sorted_size, K/2] fp4
    const uint8_t* a_scale;     // shuffled e8m0 over SORTED rows: 32-row chunks of (K/256)*256 bytes
    const uint8_t* w;           // preshuffled fp4 [experts * rows_per_expert, K/2] (rows_per_expert = 2*inter: gate rows then up
                                // rows; or model_dim)
    const uint8_t* w_scale;     // shuffled e8m0 over the experts * rows_per_expert rows of w
    const int32_t* sorted_ids;  // (slot << 24) | token per sorted row; padding rows hold token >= tokens
    const int32_t* expert_ids;  // expert of each block of block_m sorted rows
    const float* sorted_w;      // routing weight per sorted row (stage 2, atomic)
    const int32_t* num_valid;   // [0] = number of sorted rows in use (a multiple of block_m)
    int tokens, experts;
    int n_out;                  // inter_dim (stage 1) or model_dim (stage 2)
    int K;                      // model_dim (stage 1) or inter_dim (stage 2)
    int sorted_size;
    int out_dtype;              // stage 2: OUT_BF16 / OUT_FP16
    int atomic;                 // stage 2: weighted atomic add into out[token]
    int eshift;                 // set by the launcher: log2(sorter block rows / rows per workgroup)
    int n_tiles, n_groups;      // set by the launcher: column tiles of the output, and groups of 8 of them
    int by_expert;              // set by the launcher: workgroup ids are mapped to XCDs by (expert, column tile)
    int quad_tiles;             // set by the launcher: workgroup ids are mapped to XCDs by (row block parity, column tile % 4)
    int blocks;                 // set by the launcher: entries of expert_ids (a workgroup id past the last block leaves at once)
};

// Arguments of the device-side expert sorter (the step in front of the MoE grouped GEMMs).
struct MoeSortParams {
    const int32_t* topk_ids;     // [tokens, topk]
    const float* topk_weights;   // [tokens, topk]
    const int32_t* expert_mask;  // [experts] or nullptr: experts with mask 0 are dropped, the others renumbered densely
    int32_t* sorted_ids;         // [sorted_size]
    float* sorted_weights;       // [sorted_size]
    int32_t* sorted_expert_ids;  // [blocks]
    int32_t* num_valid;          // [2] = {padded rows in use, tokens}
    v4i* zero_buf;               // nullptr or a buffer to clear
    int64_t zero_vec;            // 16-byte vectors of zero_buf
    int tokens, topk, experts, block_m, sorted_size, blocks;
};

// bias + activation + 16-bit conversion of four consecutive columns.  The variant is chosen at run time
// (the epilogue is a vanishing part of any launch, so it is not worth a kernel instantiation per variant).
template <int OUT, int EPI>
__device__ __forceinline__ v2i finish4(v4f x, const uint16_t* bias_n) {
    float b0 = 0.f, b1 = 0.f, b2 = 0.f, b3 = 0.f;
    if constexpr (EPI != EPI_NONE) {
        const v2i braw = *reinterpret_cast<const v2i*>(bias_n);
        b0 = from_out16<OUT>((uint16_t)(braw[0] & 0xFFFF));
        b1 = from_out16<OUT>((uint16_t)((uint32_t)braw[0] >> 16));
        b2 = from_out16<OUT>((uint16_t)(braw[1] & 0xFFFF));
        b3 = from_out16<OUT>((uint16_t)((uint32_t)braw[1] >> 16));
    }
    return pack4_out16<OUT>(epi_act<EPI>(x[0], b0), epi_act<EPI>(x[1], b1), epi_act<EPI>(x[2], b2), epi_act<EPI>(x[3], b3));
}

template <int OUT>
__device__ __forceinline__ v2i finish4_rt(v4f x, const uint16_t* bias_n, int epi) {
    switch (epi) {
        case EPI_BIAS: return finish4<OUT, EPI_BIAS>(x, bias_n);
        case EPI_BIAS_RELU: return finish4<OUT, EPI_BIAS_RELU>(x, bias_n);
        case EPI_BIAS_SILU: return finish4<OUT, EPI_BIAS_SILU>(x, bias_n);
        case EPI_BIAS_GELU: return finish4<OUT, EPI_BIAS_GELU>(x, bias_n);
        default: return finish4<OUT, EPI_NONE>(x, bias_n);
    }
}

// store four consecutive columns of row-major 16-bit C starting at element index idx (column n)
template <class P>
__device__ __forceinline__ void store_c4(const P& p, size_t idx, int n, v4f x) {
    const v2i r = p.out == OUT_BF16 ? finish4_rt<OUT_BF16>(x, p.bias + n, p.epi) : finish4_rt<OUT_FP16>(x, p.bias + n, p.epi);
    *reinterpret_cast<v2i*>(reinterpret_cast<uint16_t*>(p.c) + idx) = r;
}
