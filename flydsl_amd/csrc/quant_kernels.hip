// On-device activation quantisers that feed the preshuffle GEMM (gfx950).  HBM-bound elementwise work: each
// input element is read once and each output byte written once.
//
//   psg_launch_quant_pertoken : per-row symmetric quantisation to int8 / OCP e4m3fn + fp32 scale per row
//                               (same results as the host utility: NaN -> 0, +-Inf -> +-dtypeMax, scale = max|row| /
//                               dtypeMax, 1 for an all-zero row, y = x / scale, int8 truncates toward zero, fp8 rounds
//                               to nearest even)
//   psg_launch_quant_mxfp4    : OCP-MX fp4: one e8m0 scale per 32 consecutive K elements (scale byte =
//                               exponent of amax/4 rounded up when its mantissa is >= 1.5), e2m1 codes by nearest
//                               value with ties to the even mantissa, two codes per byte (even k low), scales
//                               written either row-major [R, K/32] or in the shuffled layout the GEMM reads
#include "psg_common.h"

namespace {

enum { X_F32 = 0, X_BF16 = 1, X_F16 = 2 };

template <int XT>
__device__ __forceinline__ void load8(const void* base, size_t elem, float* v) {
    if constexpr (XT == X_F32) {
        const v4f a = *reinterpret_cast<const v4f*>(static_cast<const float*>(base) + elem);
        const v4f b = *reinterpret_cast<const v4f*>(static_cast<const float*>(base) + elem + 4);
        v[0] = a[0]; v[1] = a[1]; v[2] = a[2]; v[3] = a[3]; v[4] = b[0]; v[5] = b[1]; v[6] = b[2]; v[7] = b[3];
    } else {
        const v4i raw = *reinterpret_cast<const v4i*>(static_cast<const uint16_t*>(base) + elem);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t w = (uint32_t)raw[i];
            if constexpr (XT == X_BF16) {
                v[2 * i] = __builtin_bit_cast(float, w << 16);
                v[2 * i + 1] = __builtin_bit_cast(float, w & 0xFFFF0000u);
            } else {
                v[2 * i] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xFFFF));
                v[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16));
            }
        }
    }
}

// fp32 -> e4m3fn bits, round to nearest even; anything that rounds past 448 gives NaN (0x7F), as torch's cast does
__device__ __forceinline__ uint32_t f32_to_e4m3fn(float x) {
    const uint32_t u = __builtin_bit_cast(uint32_t, x);
    const uint32_t sign = (u >> 24) & 0x80u;
    const uint32_t a = u & 0x7FFFFFFFu;
    if (a >= 0x43F00000u) return sign | 0x7Fu;       // >= 480 (and Inf / NaN)
    if (a < 0x3C800000u) {                            // < 2^-6: subnormal target, spacing 2^-9
        const float q = __builtin_bit_cast(float, a) * 512.0f;   // exact (power of two)
        return sign | (uint32_t)__builtin_rintf(q);              // round half to even; 8 = smallest normal
    }
    // normal: keep 3 mantissa bits, round to nearest even on the 20 dropped bits (464 ties down to 448,
    // anything above rounds to the 0x7F pattern by itself)
    const uint32_t r = a + 0x7FFFFu + ((a >> 20) & 1u);
    return sign | (((r >> 23) - 120u) << 3) | ((r >> 20) & 7u);
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

// NaN -> 0, +-Inf -> +-dtypeMax, finite values untouched
__device__ __forceinline__ float clean(float t, float dmax) {
    if (t != t) return 0.0f;
    if (__builtin_isinf(t)) return t > 0.0f ? dmax : -dmax;
    return t;
}

template <int OUT_FP8>
__device__ __forceinline__ void quant_store8(const float* v, float s, uint8_t* dst) {
    float q[8];
#pragma unroll
    for (int e = 0; e < 8; e++) q[e] = v[e] / s;  // correctly rounded fp32 division
    v2i o;
    if constexpr (OUT_FP8) {
        // v_cvt_pk_fp8_f32: two fp32 -> two OCP e4m3 bytes, round to nearest even (|q| <= 448 here, so its
        // saturation never comes into play)
        unsigned w0 = 0, w1 = 0;
        w0 = __builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], w0, false);
        w0 = __builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], w0, true);
        w1 = __builtin_amdgcn_cvt_pk_fp8_f32(q[4], q[5], w1, false);
        w1 = __builtin_amdgcn_cvt_pk_fp8_f32(q[6], q[7], w1, true);
        o[0] = (int)w0;
        o[1] = (int)w1;
    } else {
        uint32_t b[8];
#pragma unroll
        for (int e = 0; e < 8; e++) b[e] = (uint32_t)(int32_t)q[e] & 0xFFu;  // float -> int truncates toward zero
        o[0] = (int)(b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24));
        o[1] = (int)(b[4] | (b[5] << 8) | (b[6] << 16) | (b[7] << 24));
    }
    *reinterpret_cast<v2i*>(dst) = o;
}

// one workgroup of 256 threads per row; the first 8192 elements of the row stay in registers between the two
// passes (rows longer than that re-read their tail, which is then still in L2)
template <int XT, int OUT_FP8>
__global__ void __launch_bounds__(256) k_quant_pertoken(const void* x, uint8_t* y, float* scale, int M, int K) {
    constexpr int KEEP = 4;  // 8-element vectors kept per thread
    __shared__ float red[4];
    const int row = blockIdx.x;
    const int tid = threadIdx.x;
    const float dmax = OUT_FP8 ? 448.0f : 127.0f;
    const size_t base = (size_t)row * (size_t)K;
    const int nvec = K >> 3;  // K % 8 == 0
    float keep[KEEP][8];
    float amax = 0.0f;
#pragma unroll
    for (int it = 0; it < KEEP; it++) {
        const int vi = tid + it * 256;
        if (vi < nvec) {
            load8<XT>(x, base + (size_t)vi * 8, keep[it]);
#pragma unroll
            for (int e = 0; e < 8; e++) {
                keep[it][e] = clean(keep[it][e], dmax);
                amax = fmaxf(amax, fabsf(keep[it][e]));
            }
        }
    }
    for (int vi = tid + KEEP * 256; vi < nvec; vi += 256) {
        float v[8];
        load8<XT>(x, base + (size_t)vi * 8, v);
#pragma unroll
        for (int e = 0; e < 8; e++) amax = fmaxf(amax, fabsf(clean(v[e], dmax)));
    }
    amax = wave_max(amax);
    if ((tid & 63) == 0) red[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    float s = amax / dmax;
    if (s == 0.0f) s = 1.0f;
    if (tid == 0) scale[row] = s;
#pragma unroll
    for (int it = 0; it < KEEP; it++) {
        const int vi = tid + it * 256;
        if (vi < nvec) quant_store8<OUT_FP8>(keep[it], s, y + base + (size_t)vi * 8);
    }
    for (int vi = tid + KEEP * 256; vi < nvec; vi += 256) {
        float v[8];
        load8<XT>(x, base + (size_t)vi * 8, v);
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] = clean(v[e], dmax);
        quant_store8<OUT_FP8>(v, s, y + base + (size_t)vi * 8);
    }
}

// Four consecutive lanes share one 32-element block (8 elements each, so a wavefront reads fully coalesced 16- or
// 32-byte pieces); the block maximum is combined with two lane exchanges.  Rows in [M, R) (padding up to a multiple
// of 32 rows) get scale byte 0 and no codes.
template <int XT>
__global__ void __launch_bounds__(256) k_quant_mxfp4(const void* x, uint8_t* packed, uint8_t* scales, int M, int R, int K,
                                                      int shuffled) {
    const int KB = K >> 5;
    const size_t piece = (size_t)blockIdx.x * 256 + threadIdx.x;  // 8-element piece index over R x K
    const size_t blk = piece >> 2;
    const int sub = (int)(piece & 3);
    const bool live = blk < (size_t)R * KB;
    const int r = live ? (int)(blk / KB) : 0, kb = live ? (int)(blk % KB) : 0;
    float v[8];
    float amax = 0.0f;
    if (live && r < M) {
        load8<XT>(x, (size_t)r * K + (size_t)kb * 32 + sub * 8, v);
#pragma unroll
        for (int e = 0; e < 8; e++) amax = fmaxf(amax, fabsf(v[e]));
    } else {
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] = 0.0f;
    }
    amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
    amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
    if (!live) return;
    // scale byte: biased exponent of amax/4, +1 when bit 22 is set and (lower mantissa bits or a normal exponent)
    const uint32_t u = __builtin_bit_cast(uint32_t, amax / 4.0f);
    uint32_t e = (u >> 23) & 0xFFu;
    const bool up = (u & 0x400000u) && ((u & 0x3FFFFFu) || e > 0);
    if (e != 0xFFu && up) e = (e + 1) & 0xFFu;
    const float sf = e == 0 ? __builtin_bit_cast(float, 0x00400000u)
                            : (e == 0xFF ? __builtin_bit_cast(float, 0x7F800001u) : __builtin_bit_cast(float, e << 23));
    if (r < M) {
        // v_cvt_scalef32_pk_fp4_f32: (a, b) / scale -> two e2m1 codes (a in the low nibble) into one byte of the word
        unsigned word = 0;
        word = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(word, v[0], v[1], sf, 0);
        word = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(word, v[2], v[3], sf, 1);
        word = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(word, v[4], v[5], sf, 2);
        word = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(word, v[6], v[7], sf, 3);
        *reinterpret_cast<unsigned*>(packed + (size_t)r * (K >> 1) + (size_t)kb * 16 + sub * 4) = word;
    }
    if (sub == 0) {
        size_t off;
        if (shuffled) {
            off = (size_t)(r >> 5) * (32u * (size_t)KB) + (size_t)(kb >> 3) * 256 + (size_t)(kb & 3) * 64 + (size_t)(r & 15) * 4 +
                  (size_t)((kb & 7) >> 2) * 2 + (size_t)((r & 31) >> 4);
        } else {
            off = (size_t)r * KB + kb;
        }
        scales[off] = (uint8_t)e;
    }
}

}  // namespace

hipError_t psg_launch_quant_pertoken(const void* x, int x_dtype, void* y, float* scale, int M, int K, int out_fp8,
                                     hipStream_t stream) {
#define PSG_Q(XT_)                                                                                                      \
    if (out_fp8) hipLaunchKernelGGL((k_quant_pertoken<XT_, 1>), dim3(M), dim3(256), 0, stream, x, (uint8_t*)y, scale, M, K); \
    else hipLaunchKernelGGL((k_quant_pertoken<XT_, 0>), dim3(M), dim3(256), 0, stream, x, (uint8_t*)y, scale, M, K);
    if (x_dtype == X_F32) { PSG_Q(X_F32) } else if (x_dtype == X_BF16) { PSG_Q(X_BF16) } else if (x_dtype == X_F16) { PSG_Q(X_F16) } else return hipErrorInvalidValue;
#undef PSG_Q
    return hipGetLastError();
}

hipError_t psg_launch_quant_mxfp4(const void* x, int x_dtype, void* packed, void* scales, int M, int R, int K, int shuffled,
                                  hipStream_t stream) {
    const size_t blocks = ((size_t)R * (K / 32) * 4 + 255) / 256;  // four threads per 32-element block
    if (x_dtype == X_F32) hipLaunchKernelGGL((k_quant_mxfp4<X_F32>), dim3(blocks), dim3(256), 0, stream, x, (uint8_t*)packed, (uint8_t*)scales, M, R, K, shuffled);
    else if (x_dtype == X_BF16) hipLaunchKernelGGL((k_quant_mxfp4<X_BF16>), dim3(blocks), dim3(256), 0, stream, x, (uint8_t*)packed, (uint8_t*)scales, M, R, K, shuffled);
    else if (x_dtype == X_F16) hipLaunchKernelGGL((k_quant_mxfp4<X_F16>), dim3(blocks), dim3(256), 0, stream, x, (uint8_t*)packed, (uint8_t*)scales, M, R, K, shuffled);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}
