/*
 * CPU oracle, C restatement.  TEST INFRASTRUCTURE ONLY: nothing shipped links or loads this file;
 * only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg do, as the checker.
 *
 * Unlike the numpy oracle (which multiplies the UN-shuffled quantised operands the way the
 * reference's run_torch does), these routines consume the WIRE FORMAT the kernels consume:
 * preshuffled B bytes and shuffled e8m0 scale bytes, addressed through the closed-form offsets.
 * Agreement of the two oracles therefore pins the offset formulas against the view/permute chains.
 *
 * Reference lines followed:
 *   preshuffled B addressing      kernels/gemm/preshuffle_gemm.py:765-780 (strides 16 / 256 / 1024 / (K/64)*1024)
 *                                 tests/utils.py:82-94
 *   epilogue order                kernels/gemm/preshuffle_gemm.py:694-714  ((f32(acc)*sa)*sb, +bias, act, ->bf16)
 *   activations                   kernels/gemm/preshuffle_gemm.py:672-692
 *   MX scale addressing / opsel   kernels/gemm/mxfp4_preshuffle.py:125-126,315-318,340-369,388
 *                                 tests/kernels/utils/gemm_common_utils.py:645-672
 *   fp4 / e8m0 decode             tests/kernels/utils/gemm_common_utils.py:23-50,63-71
 *
 * Build: gcc -O2 -fopenmp -shared -fPIC psg_oracle_c.c -o libpsg_oracle.so -lm   (see oracle/Makefile)
 */
#include <math.h>
#ifdef _OPENMP
#include <omp.h>
#endif
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

enum { KIND_INT8 = 0, KIND_FP8 = 1 };
enum { ACT_NONE = 0, ACT_BIAS = 1, ACT_BIAS_RELU = 2, ACT_BIAS_SILU = 3, ACT_BIAS_GELU = 4 };

static float e4m3fn_decode(uint8_t c) {
    int s = c >> 7, e = (c >> 3) & 15, m = c & 7;
    float v;
    if (e == 15 && m == 7) v = NAN;
    else if (e == 0) v = ldexpf((float)m / 8.0f, -6);
    else v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
    return s ? -v : v;
}

static uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if (isnan(f)) return (uint16_t)((u >> 16) | 0x40);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static float bf16_to_f32(uint16_t b) {
    uint32_t u = (uint32_t)b << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* byte offset of W[n,k] (1-byte elements) inside the preshuffled buffer */
static inline size_t bshuf_off(size_t n, size_t k, size_t K) {
    return (n / 16) * (16 * K) + (k / 64) * 1024 + ((k % 64) / 16) * 256 + (n % 16) * 16 + (k % 16);
}

/* byte offset of scale S[r,kb] inside the shuffled e8m0 buffer; KB = K/32 */
static inline size_t sshuf_off(size_t r, size_t kb, size_t KB) {
    return (r / 32) * (32 * KB) + (kb / 8) * 256 + (kb % 4) * 64 + (r % 16) * 4 + ((kb % 8) / 4) * 2 + ((r % 32) / 16);
}

static float activation(float v, int epi) {
    if (epi == ACT_BIAS_RELU) return v > 0.0f ? v : 0.0f;
    if (epi == ACT_BIAS_SILU) {
        float e = expf(-v);
        return v * (1.0f / (1.0f + e));
    }
    if (epi == ACT_BIAS_GELU) {
        float x3 = v * v * v;
        float y = 0.7978845608f * (v + 0.044715f * x3);
        float ay = fabsf(y);
        float e = expf(-2.0f * ay);
        float num = y > 0.0f ? 2.0f : 2.0f * e;
        return 0.5f * v * (num * (1.0f / (1.0f + e)));
    }
    return v;
}

/*
 * 8-bit GEMM from the wire format.  a: [M,K] bytes row-major; b_shuf: preshuffled [N,K] bytes;
 * sa [M], sb [N] fp32; bias [N] bf16 bits or NULL.
 * acc_i32 (int8 only, may be NULL): exact int32 accumulators [M,N].
 * acc_f32 (may be NULL): fp32 value the epilogue starts from ([M,N]); for fp8 it is the float64
 *   sum of exact products rounded once to fp32.
 * c_bf16 (may be NULL): bf16 bits of ((acc*sa)*sb + bias) after the activation.
 */
int psg_oracle_a8w8(const uint8_t *a, const uint8_t *b_shuf, const float *sa, const float *sb, const uint16_t *bias,
                    int64_t M, int64_t N, int64_t K, int kind, int epi, int32_t *acc_i32, float *acc_f32,
                    uint16_t *c_bf16) {
    if (N % 16 || K % 64) return -1;
    float lut[256];
    for (int i = 0; i < 256; i++) lut[i] = e4m3fn_decode((uint8_t)i);
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; n++) {
        /* gather row n of W out of the fragment order once */
        uint8_t *wrow = (uint8_t *)malloc((size_t)K);
        for (int64_t k = 0; k < K; k++) wrow[k] = b_shuf[bshuf_off((size_t)n, (size_t)k, (size_t)K)];
        for (int64_t m = 0; m < M; m++) {
            const uint8_t *arow = a + m * K;
            float accf;
            if (kind == KIND_INT8) {
                int64_t s = 0;
                for (int64_t k = 0; k < K; k++) s += (int32_t)(int8_t)arow[k] * (int32_t)(int8_t)wrow[k];
                if (acc_i32) acc_i32[m * N + n] = (int32_t)s;
                accf = (float)(int32_t)s;
            } else {
                double s = 0.0;
                for (int64_t k = 0; k < K; k++) s += (double)lut[arow[k]] * (double)lut[wrow[k]];
                accf = (float)s;
            }
            if (acc_f32) acc_f32[m * N + n] = accf;
            if (c_bf16) {
                float v = (accf * sa[m]) * sb[n];
                if (epi != ACT_NONE) v = v + bf16_to_f32(bias[n]);
                v = activation(v, epi);
                c_bf16[m * N + n] = f32_to_bf16(v);
            }
        }
        free(wrow);
    }
    return 0;
}

static const float E2M1[16] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f,
                               -0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};

static double e8m0_decode(uint8_t b) {
    if (b == 0xFF) return NAN;
    return ldexp(1.0, (int)b - 127); /* byte 0 -> 2^-127, same value as bits 0x00400000 */
}

/*
 * MXFP4 GEMM from the wire format.  a: [M, K/2] packed row-major (even k in the low nibble);
 * b_shuf: preshuffled packed [N, K/2]; sa_shuf: shuffled e8m0 over ceil(M/32)*32 rows x K/32;
 * sb_shuf: shuffled e8m0 over N rows (N % 32 == 0) x K/32.
 * out_f32 (may be NULL): float64 block-scaled sum rounded once to fp32; c_bf16 (may be NULL): bf16 bits of it.
 */
int psg_oracle_mxfp4(const uint8_t *a, const uint8_t *b_shuf, const uint8_t *sa_shuf, const uint8_t *sb_shuf,
                     int64_t M, int64_t N, int64_t K, float *out_f32, uint16_t *c_bf16) {
    if (N % 32 || K % 256) return -1;
    const int64_t KP = K / 2, KB = K / 32;
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; n++) {
        uint8_t *wrow = (uint8_t *)malloc((size_t)KP);
        for (int64_t kb = 0; kb < KP; kb++) wrow[kb] = b_shuf[bshuf_off((size_t)n, (size_t)kb, (size_t)KP)];
        for (int64_t m = 0; m < M; m++) {
            const uint8_t *arow = a + m * KP;
            double s = 0.0;
            for (int64_t blk = 0; blk < KB; blk++) {
                double bs = 0.0;
                for (int64_t j = 0; j < 16; j++) {
                    uint8_t av = arow[blk * 16 + j], wv = wrow[blk * 16 + j];
                    bs += (double)E2M1[av & 15] * (double)E2M1[wv & 15];
                    bs += (double)E2M1[av >> 4] * (double)E2M1[wv >> 4];
                }
                double sca = e8m0_decode(sa_shuf[sshuf_off((size_t)m, (size_t)blk, (size_t)KB)]);
                double scb = e8m0_decode(sb_shuf[sshuf_off((size_t)n, (size_t)blk, (size_t)KB)]);
                s += bs * sca * scb;
            }
            float f = (float)s;
            if (out_f32) out_f32[m * N + n] = f;
            if (c_bf16) c_bf16[m * N + n] = f32_to_bf16(f);
        }
        free(wrow);
    }
    return 0;
}

/* The reference's CPU path as plain C for the cpu_baseline timing: dequantise both operands to fp32
 * (tests/kernels/test_preshuffle_gemm.py:105-106), then a blocked fp32 matmul a32 @ b32.T (:110).
 * b is UN-shuffled here, as in run_torch.  Not used for parity. */
int psg_oracle_run_torch_f32(const uint8_t *a, const uint8_t *b, const float *sa, const float *sb, int64_t M,
                             int64_t N, int64_t K, int kind, float *c) {
    float lut[256];
    for (int i = 0; i < 256; i++) lut[i] = kind == KIND_INT8 ? (float)(int8_t)(uint8_t)i : e4m3fn_decode((uint8_t)i);
    float *a32 = (float *)malloc(sizeof(float) * (size_t)M * (size_t)K);
    float *b32 = (float *)malloc(sizeof(float) * (size_t)N * (size_t)K);
    if (!a32 || !b32) { free(a32); free(b32); return -2; }
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; m++)
        for (int64_t k = 0; k < K; k++) a32[m * K + k] = lut[a[m * K + k]] * sa[m];
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; n++)
        for (int64_t k = 0; k < K; k++) b32[n * K + k] = lut[b[n * K + k]] * sb[n];
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; n++) {
        const float *br = b32 + n * K;
        for (int64_t m = 0; m < M; m++) {
            const float *ar = a32 + m * K;
            float s = 0.0f;
            for (int64_t k = 0; k < K; k++) s += ar[k] * br[k];
            c[m * N + n] = s;
        }
    }
    free(a32);
    free(b32);
    return 0;
}

int psg_oracle_num_threads(void) {
    int n = 1;
#ifdef _OPENMP
#pragma omp parallel
    {
#pragma omp master
        n = omp_get_num_threads();
    }
#endif
    return n;
}
