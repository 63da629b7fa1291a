/*
 * psgemm.h -- C ABI of the MI355X-native preshuffle quantized GEMM library (libpsgemm.so).
 *
 *   C[M,N] = A[M,K] * B[N,K]^T      B preshuffled into MFMA-fragment order on the host
 *
 * Plain pointers and sizes only; no framework types.  Every pointer is a DEVICE pointer owned by
 * the caller and only borrowed for the duration of the (asynchronous) launch.  Every launch goes to
 * the caller's stream and nothing else touches the device: no allocation, no synchronisation, no
 * default-stream work, so calls may be recorded into a HIP graph.  Entry points are re-entrant.
 *
 * Return value of every int function: 0 = ok, negative = argument validation failed (PSG_E_*),
 * positive = hipError_t of a failed HIP call.  psg_last_error() returns a thread-local message.
 *
 * What each entry point replaces in the reference (paths relative to the reference tree):
 *   psg_gemm_a8w8       the compiled launcher returned by compile_preshuffle_gemm()
 *                       kernels/gemm/preshuffle_gemm.py:717-806 (launch_gemm) + :220-714 (kernel_gemm),
 *                       reached through the JIT host stub -> mgpuLaunchKernel
 *                       lib/Runtime/ROCm/FlyRocmRuntimeWrappers.cpp:58-64
 *   psg_gemm_a8w8_acc   no counterpart: the reference never exposes accumulators; this dumps them
 *                       (int32 for int8, fp32 for fp8) so parity tests can check them bit-exactly
 *   psg_gemm_mxfp4      kernels/gemm/mxfp4_preshuffle.py:57-488 (launch_gemm / kernel_gemm): fp4/fp6/fp8 A x fp4/fp8 W,
 *                       caller strides, batch over grid.z
 *   psg_gemm_mxfp4_acc  no counterpart: fp32 accumulators of the MXFP4 mainloop, for parity tests
 *   psg_workspace_bytes no counterpart (the reference's preshuffle GEMM has no split-K path)
 *   psg_tile_coords     the workgroup-id -> tile remap xcd_remap_bx_by
 *                       kernels/common/mma/mfma_preshuffle_pipeline.py:685-729 (host evaluation of the function the
 *                       tiled kernel uses); psg_debug_tile_order runs the same function on the device
 *   psg_gemm_a8w8_static, psg_init, psg_static_scratch_bytes
 *                       no counterpart in the reference: for callers that cannot allocate (see below)
 *   psg_moe_gemm        kernels/moe/moe_gemm_2stage/gemm1.py, gemm2.py (launch_moe_gemm1 / launch_moe_gemm2), fp8 and int8
 *   psg_moe_reduce      kernels/moe/moe_gemm_2stage/moe_reduce.py:164 (compile_moe_reduction)
 *   psg_quant_pertoken  device version of the host quantiser tests/utils.py:29-73
 *   psg_quant_mxfp4     device version of tests/kernels/utils/gemm_common_utils.py:675-704 (+ :645-672)
 */
#ifndef PSGEMM_H
#define PSGEMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PSG_ABI_VERSION 7

/* input element types of A and B */
enum psg_in_dtype { PSG_IN_INT8 = 0, PSG_IN_FP8_E4M3FN = 1, PSG_IN_FP16 = 2, PSG_IN_BF16 = 3,
                    PSG_IN_INT8_W4 = 6 /* psg_moe_gemm only: int8 activations, packed int4 weights */ };
/* output element types of C */
enum psg_out_dtype { PSG_OUT_BF16 = 0, PSG_OUT_FP16 = 1, PSG_OUT_F32 = 2 /* psg_moe_gemm stage 2 with accumulate only */ };
/* fused epilogue, as the reference's `epilogue` keyword (kernels/gemm/preshuffle_gemm.py:118) */
enum psg_epilogue {
    PSG_EPI_NONE = 0,
    PSG_EPI_BIAS = 1,
    PSG_EPI_BIAS_RELU = 2,
    PSG_EPI_BIAS_SILU = 3,
    PSG_EPI_BIAS_GELU = 4
};

/* validation errors (negative return values) */
enum psg_error {
    PSG_E_NULL = -1,        /* a required pointer is NULL */
    PSG_E_SHAPE = -2,       /* M/N/K violate the layout's divisibility or range rules */
    PSG_E_DTYPE = -3,       /* unsupported dtype / epilogue combination */
    PSG_E_WORKSPACE = -4,   /* workspace missing or too small for this call */
    PSG_E_UNSUPPORTED = -5, /* valid in the reference but not built here (says which in the message) */
    PSG_E_ALIGN = -6        /* a pointer is not 16-byte aligned */
};

/*
 * Arguments of the 8-bit (and 16-bit) preshuffle GEMM.
 *   c        [M,N] row-major, out_dtype; rows >= M of the allocation are never written
 *   a        [M,K] row-major, 1 byte/element (int8 or e4m3fn) or 2 bytes/element (fp16 / bf16); rows >= M are never read
 *   b        preshuffle of W[N,K]: byte of W[n,k] at
 *            (n/16)*16K + (k/64)*1024 + ((k%64)/16)*256 + (n%16)*16 + k%16      (tests/utils.py:76-96)
 *            (2-byte elements: element (n,k) at (n/16)*16K + (k/32)*512 + ((k%32)/8)*128 + (n%16)*8 + k%8, in elements)
 *   scale_a  [M] fp32 per-token scales; scale_b [N] fp32 per-channel scales; ignored (may be NULL) for fp16 / bf16
 *   bias     [N] out_dtype, read only when epilogue != PSG_EPI_NONE
 *   N % 16 == 0, K*bytes_per_element % 64 == 0, 1 <= M <= 65536 (kernels/gemm/preshuffle_gemm.py:783-785)
 *   workspace / workspace_bytes: scratch for the split-K plan of the tiled path (32 < M, few tiles, long K):
 *            psg_workspace_bytes() bytes, no initialisation needed.  May always be NULL/0: the library then
 *            runs the problem unsplit.  Two launches that may overlap in time must not share one workspace.
 *   tile_m/tile_n/tile_k, xcd_swizzle: the reference's tuning keywords; accepted as hints
 *            (0 = library's choice).  The library picks its own tiling per regime.  xcd_swizzle > 0 is the number
 *            of M-tiles per group of the tile order (psg_tile_coords); 0, which switches the remap off in the
 *            reference, here means the library's default group of 8 (results do not depend on the tile order).
 */
typedef struct psg_a8w8_args {
    void *c;
    const void *a;
    const void *b;
    const float *scale_a;
    const float *scale_b;
    const void *bias;
    void *workspace;
    uint64_t workspace_bytes;
    int32_t M, N, K;
    int32_t in_dtype;  /* enum psg_in_dtype */
    int32_t out_dtype; /* enum psg_out_dtype */
    int32_t epilogue;  /* enum psg_epilogue */
    int32_t tile_m, tile_n, tile_k;
    int32_t xcd_swizzle;
    int32_t force_path; /* 0 = auto, 1 = tiled MFMA mainloop, 2 = small-M streaming kernel, M <= 64 (tests/benchmarks) */
    int32_t reserved;   /* 0; tuning knob for a forced 256x256 tile: 2 = 2x2 wavefronts, 8 = eight wavefronts 1x8 (default 1x4) */
    int32_t b_layout;   /* 0 = b is preshuffled (above); 1 = b is plain row-major W[N,K], the b_preshuffled=False call
                           shape of the reference's row-scale fp8 GEMMs (kernels/gemm/fp8_gemm_8wave.py:148) */
    int32_t pad0;       /* 0 */
} psg_a8w8_args;

/* Element formats of the MX GEMM's operands (kernels/gemm/mxfp4_preshuffle.py:70-72, a_dtype / b_dtype). */
enum psg_mx_dtype { PSG_MX_FP4 = 0, PSG_MX_FP6 = 1, PSG_MX_FP8 = 2,
                    PSG_MX_BF16_QUANT = 3 /* psg_moe_mx_gemm stage 1 only: bf16 activations, quantised to fp4 by the kernel */ };

/*
 * Arguments of the MX preshuffle GEMM: A in fp4 (e2m1), fp6 (e2m3) or fp8 (e4m3fn), W in fp4 or fp8, one e8m0 scale
 * per 32 K elements on both sides, optionally strided-batched (kernels/gemm/mxfp4_preshuffle.py:57-91).
 *   c        [M,N] out_dtype, rows c_row_stride elements apart
 *   a        rows a_row_stride bytes apart; a row is
 *              fp4: K/2 bytes of packed e2m1, even k in the low nibble
 *              fp8: K bytes of e4m3fn
 *              fp6: K bytes: per 32 elements 24 bytes of packed e2m3 (element j at bits [6j, 6j+6) of the 192-bit
 *                   little-endian group) followed by 8 bytes that are not read
 *                   (tests/kernels/utils/gemm_common_utils.py pack_fp6_e2m3 + the fp8-sized padding of
 *                   tests/kernels/test_preshuffle_gemm.py test_mfma_a6w4_preshuffle)
 *   b        fp4: shuffle_weight_w4 of packed W[N,K/2]; fp8: shuffle_weight of W[N,K] (same 16x16-byte block map as
 *            the 8-bit GEMM, K bytes per row)
 *   scale_a  shuffle_scale_w4 of e8m0 [ceil(M/32)*32, K/32], 32-row chunks scale_a_chunk_stride bytes apart;
 *            scale_b the same over [N, K/32], dense
 *            byte of S[r,kb] at (r/32)*32*(K/32) + (kb/8)*256 + (kb%4)*64 + (r%16)*4 + ((kb%8)/4)*2 + (r%32)/16
 *            (tests/kernels/utils/gemm_common_utils.py:645-672)
 *   N % 32 == 0, K % 256 == 0, 1 <= M <= 65536, 1 <= batch <= 65535 (0 is read as 1)
 * Strides and batch: a stride of 0 means dense (a_row_stride = bytes of a row, c_row_stride = N,
 * scale_a_chunk_stride = (K/256)*256, batch strides = the dense size of one batch: [B,M,*] for a / c,
 * ceil(M/32) chunks for scale_a).  W and scale_b are always batch-dense (mxfp4_preshuffle.py:177-193).  Batch z reads
 * a + z*a_batch_stride etc. (bytes) and all batches run in ONE launch (grid.z = batch).
 * Which kernel runs: fp4 x fp4 with batch 1 and dense strides takes the tuned fp4 kernels (tiled mainloop, small-M
 * split-K; workspace / tile_* / force_path 1, 2 apply to them only); everything else, or force_path 3, takes the
 * general kernel, which ignores the tile arguments and uses workspace (psg_workspace_bytes(M, N, K, 5) bytes) for
 * split-K when batch is 1 and C is dense.
 */
typedef struct psg_mxfp4_args {
    void *c;
    const void *a;
    const void *b;
    const void *scale_a;
    const void *scale_b;
    void *workspace;
    uint64_t workspace_bytes;
    int32_t M, N, K;
    int32_t out_dtype; /* enum psg_out_dtype */
    int32_t tile_m, tile_n, tile_k;
    int32_t xcd_swizzle;
    int32_t force_path; /* 0 = auto, 1 = tiled (fp4 x fp4), 2 = small-M (fp4 x fp4), 3 = general kernel */
    int32_t reserved;
    int32_t a_dtype;    /* enum psg_mx_dtype */
    int32_t b_dtype;    /* PSG_MX_FP4 or PSG_MX_FP8 */
    int32_t batch;      /* 0 or 1 = a single GEMM */
    int32_t pad0;       /* 0 */
    int64_t a_row_stride;         /* bytes; 0 = dense */
    int64_t c_row_stride;         /* ELEMENTS; 0 = N */
    int64_t scale_a_chunk_stride; /* bytes between 32-row chunks; 0 = dense */
    int64_t a_batch_stride;       /* bytes; 0 = dense */
    int64_t c_batch_stride;       /* bytes; 0 = dense */
    int64_t scale_a_batch_stride; /* bytes; 0 = dense */
} psg_mxfp4_args;

/* ABI version of the loaded library (PSG_ABI_VERSION it was built with). */
int psg_abi_version(void);

/* Thread-local text of the last error returned on this thread ("" if none). */
const char *psg_last_error(void);

/* Bytes of workspace the split-K plan would use for this problem (0 when the chosen plan needs none).
 * in_dtype: enum psg_in_dtype, 4 for psg_gemm_mxfp4 on its fp4 x fp4 kernels, 5 for psg_gemm_mxfp4 on the general MX
 * kernel (any other format pair, or force_path 3; batch 1 and dense C only, otherwise it runs unsplit). */
uint64_t psg_workspace_bytes(int32_t M, int32_t N, int32_t K, int32_t in_dtype);

/* C = epilogue((acc * scale_a[m]) * scale_b[n]) on `stream` (a hipStream_t passed as void*). */
int psg_gemm_a8w8(const psg_a8w8_args *args, void *stream);

/*
 * psg_gemm_a8w8 for callers that cannot allocate device memory: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  It computes exactly what
 * psg_gemm_a8w8 computes (same plan, same kernels, same bits) but ignores args->workspace: the split-K partial sums
 * go to a scratch array that is part of the library's device image (psg_static_scratch_bytes() bytes, 32 MiB, one
 * copy per GPU, held until the process ends).  The call allocates and frees nothing.  A problem whose split-K plan
 * wants more than that is rejected with PSG_E_WORKSPACE (use psg_gemm_a8w8 with a caller workspace, or none).
 * All calls on one GPU share that GPU's array: two calls that may overlap in time on one GPU (different streams)
 * race; calls on one stream, or ordered by events, are safe.  Nothing needs clearing between calls: every partial
 * that is read was written by the same call.
 * psg_init() looks up the array's device address for the current device (otherwise done by the first call on that
 * device); call it once per device before a graph capture that records psg_gemm_a8w8_static.
 */
int psg_init(void);
uint64_t psg_static_scratch_bytes(void);
int psg_gemm_a8w8_static(const psg_a8w8_args *args, void *stream);

/* Tile (tm, tn) that workgroup `id` of a tiles_m x tiles_n launch of the tiled kernel works on, groups of `group_m`
 * M-tiles; the reference's xcd_remap_bx_by with linear id = bx*gx + by, gx = tiles_n, gy = tiles_m,
 * xcd_swizzle = group_m (kernels/common/mma/mfma_preshuffle_pipeline.py:685-729).  Host function, no GPU needed. */
void psg_tile_coords(int32_t id, int32_t tiles_m, int32_t tiles_n, int32_t group_m, int32_t *tm, int32_t *tn);

/* Evaluates the same function on the device for every id: out[2*id] = tm, out[2*id+1] = tn (int32 [tiles_m*tiles_n*2]). */
int psg_debug_tile_order(int32_t tiles_m, int32_t tiles_n, int32_t group_m, int32_t *out, void *stream);

/* Same mainloop, but writes the raw accumulators [M,N] (int32 for int8, fp32 for fp8) to `acc`
 * instead of C.  c, scale_a, scale_b, bias are ignored. */
int psg_gemm_a8w8_acc(const psg_a8w8_args *args, void *acc, void *stream);

/* C = bf16/fp16( sum over 32-blocks of 2^(ea-127) * 2^(eb-127) * dot32(A4, B4) ) on `stream`. */
int psg_gemm_mxfp4(const psg_mxfp4_args *args, void *stream);

/* Same mainloop, but writes the fp32 accumulators [M,N] to `acc` instead of C (no counterpart in the
 * reference; parity tests use it to look at the sum before the 16-bit rounding). */
int psg_gemm_mxfp4_acc(const psg_mxfp4_args *args, void *acc, void *stream);

/*
 * On-device activation quantisers (the step before the GEMM).  The reference quantises on the host with
 * tests/utils.py:29-73 (pertoken_quant) and tests/kernels/utils/gemm_common_utils.py:675-704 (per_1x32_f4_quant)
 * followed by :645-672 (shuffle_scale_w4); these produce the same bytes on the device.
 *   x_dtype: 0 fp32, 1 bf16, 2 fp16.  x is [M,K] row-major.
 *   psg_quant_pertoken treats NaN / Inf like the reference (nan_to_num, then the row maximum).  psg_quant_mxfp4 is
 *   defined for FINITE inputs only: a NaN or Inf inside a 32-element block does not produce the reference's 0xFF
 *   scale byte (the block maximum is taken with fmaxf, which drops NaN).
 */

/* y [M,K] int8 (out_dtype PSG_IN_INT8) or e4m3fn (PSG_IN_FP8_E4M3FN); scale [M] fp32 = max|row| / dtypeMax. K % 8 == 0. */
int psg_quant_pertoken(const void *x, int32_t x_dtype, void *y, float *scale, int32_t M, int32_t K, int32_t out_dtype,
                       void *stream);

/* packed [M,K/2] e2m1 pairs; scales: e8m0 bytes over ceil(M/32)*32 rows x K/32, row-major (shuffled = 0) or in the
 * shuffle_scale_w4 layout the GEMM reads (shuffled = 1, needs K % 256 == 0).  K % 32 == 0. */
int psg_quant_mxfp4(const void *x, int32_t x_dtype, void *packed, void *scales, int32_t M, int32_t K, int32_t shuffled,
                    void *stream);

/*
 * MoE grouped GEMMs over expert-sorted token blocks: the two stages of the reference's 2-stage MoE
 * (kernels/moe/moe_gemm_2stage/gemm1.py:367-381,502-537 launch_moe_gemm1; gemm2.py launch_moe_gemm2), int8 or e4m3fn
 * operands with one fp32 scale per row of x and per weight row.
 *   stage 1: out[t, slot, n] = silu(g) * u (* routing weight when doweight), g = x[t] . W1[e, n], u = x[t] . W1[e, inter + n];
 *            x [tokens, model_dim], w = shuffle_weight of W1 [experts * 2*inter_dim, model_dim], out [tokens, topk, inter_dim]
 *   stage 2: y = x[t*topk + slot] . W2[e, n] (* routing weight when doweight); accumulate = 1 adds y atomically into
 *            out[t, n] (out [tokens, model_dim], bf16 / fp16 / fp32, zeroed by the caller; the order of the additions is
 *            not fixed), accumulate = 0 writes out[t*topk + slot, n] (bf16 / fp16) for psg_moe_reduce;
 *            x [tokens*topk, inter_dim], w = shuffle_weight of W2 [experts * model_dim, inter_dim]
 *   sorted_token_ids  (slot << 24) | token for every sorted row, experts in ascending order, every expert padded to
 *                     whole blocks of block_m rows with entries whose token is >= tokens (tests/kernels/
 *                     test_moe_gemm_2stage.py:99-137); sorted_weights the routing weight of each sorted row;
 *                     sorted_expert_ids one expert per block (entries < 0 are skipped); num_valid_ids[0] = sorted rows
 *                     in use (read on the device, so the grid does not depend on the routing)
 *   block_m in {16, 32, 64, 128}; model_dim % 128 == 0 and inter_dim % 128 == 0 for the K side of each stage;
 *   the output width of each stage a multiple of 16; tokens < 2^24; rows of x times K below 4 GiB.
 */
typedef struct psg_moe_args {
    void *out;
    const void *x;
    const void *w;
    const float *scale_x;
    const float *scale_w;
    const int32_t *sorted_token_ids;
    const int32_t *sorted_expert_ids;
    const float *sorted_weights;
    const int32_t *num_valid_ids;
    int32_t tokens, topk, experts;
    int32_t model_dim, inter_dim;
    int32_t sorted_size; /* entries of sorted_token_ids / sorted_weights */
    int32_t blocks;      /* entries of sorted_expert_ids = grid size along the sorted rows */
    int32_t block_m;
    int32_t in_dtype;    /* PSG_IN_INT8, PSG_IN_FP8_E4M3FN, or PSG_IN_INT8_W4: x int8 and w the preshuffled int8 bytes (values in
                            [-8, 7]) with every 8 consecutive values v0..v7 packed into 4 bytes, byte j = (v_j & 15) | (v_{j+4} << 4)
                            (W4A8; tests/kernels/test_moe_gemm_2stage.py:64-80, kernels/moe/moe_gemm_2stage/layout_helpers.py:146-189) */
    int32_t out_dtype;   /* enum psg_out_dtype */
    int32_t stage;       /* 1 or 2 */
    int32_t doweight;
    int32_t accumulate;  /* stage 2 only */
    int32_t x_slot_major; /* stage 1 only: 1 = x and scale_x hold one row per (slot, token), row slot*tokens + token (the
                             reference's int8smooth inputs, kernels/moe/moe_gemm_2stage/gemm1.py:100-101,321-328); 0 = one row per token */
    int32_t no_pairing;  /* 0: in stage 1 with one-byte weights and block_m 16 or 32, two consecutive blocks of the same expert are multiplied by one workgroup,
                            so that an expert with up to 2*block_m routed rows streams its weights once (same results: the
                            rows of a block never mix); 1: every block gets its own workgroup (tests, tuning) */
    int32_t pad0;        /* 0 */
} psg_moe_args;

int psg_moe_gemm(const psg_moe_args *args, void *stream);

/*
 * MoE grouped GEMMs with MX operands over expert-sorted token blocks: the two stages of the reference's fused MX-FP4 MoE
 * (kernels/moe/mxfp_moe/host.py:87-165 flydsl_mxfp4_gemm1, :168-231 flydsl_mxfp4_gemm2).  Weights are fp4 (e2m1 pairs, even
 * column in the low nibble) in the shuffle_weight order with e8m0 scales per 32 K elements in the e8m0_shuffle order
 * (tests/kernels/utils/gemm_common_utils.py:114-136), both over all experts * rows.
 *   stage 1: y[r, n] = silu(g) * u, g = a[t_r] . W1[e, n], u = a[t_r] . W1[e, inter + n] for every sorted row r of token t_r;
 *            y is quantised per 32 columns as the reference's kernel does (kernels/moe/mxfp_moe/mxfp4_gemm_common.py:221-230: scale byte =
 *            exponent of the smallest power of two >= amax / 6, at most 254; codes = nearest-even e2m1 of y / 2^(byte-127))
 *            and written BY SORTED POSITION: out [sorted_size, inter_dim/2] packed codes, out_scale the scales of those
 *            rows in the e8m0_shuffle order over ceil(sorted_size/256)*256 rows x inter_dim/32 columns.
 *            a [tokens, model_dim/2] fp4 (a_dtype PSG_MX_FP4) or [tokens, model_dim] e4m3fn (PSG_MX_FP8); a_scale the e8m0 scales
 *            of the rows of a gathered by sorted position, in the same shuffled order (moe_mxfp4_sort,
 *            gemm_common_utils.py:464-598); w = W1 [experts * 2*inter_dim, model_dim/2].
 *   stage 2: y[r, n] = a[r] . W2[e, n] over the sorted rows stage 1 wrote (a = its out, a_scale = its out_scale);
 *            atomic = 1: out[t_r, n] += y * sorted_weights[r] (out [tokens, model_dim] bf16 / fp16, zeroed by the caller, order
 *            of the additions not fixed: the reference's "atomic" epilogue); atomic = 0: out[r, n] = y, out [sorted_size,
 *            model_dim] (its "nonatomic" epilogue: the caller applies the weights); w = W2 [experts * model_dim, inter_dim/2].
 *            With a_dtype PSG_MX_BF16_QUANT (the reference's inline_quant variant, gemm1.py:324-412; block_m 16 only) a is
 *            [tokens, model_dim] bf16 and every 32 elements are quantised to fp4 inside the kernel with the same scale rule as
 *            the output; a_scale is not read.
 *   block_m in {32, 64, 128}, or 16 (stage 1: only with PSG_MX_BF16_QUANT); model_dim % 256 == 0 and inter_dim % 256 == 0;
 *   tokens < 2^24; every operand below 4 GiB.
 *   sorted_token_ids, sorted_expert_ids, sorted_weights, num_valid_ids as for psg_moe_gemm.
 */
typedef struct psg_moe_mx_args {
    void *out;
    void *out_scale;     /* stage 1 only */
    const void *a;
    const void *a_scale;
    const void *w;
    const void *w_scale;
    const int32_t *sorted_token_ids;
    const int32_t *sorted_expert_ids;
    const float *sorted_weights; /* stage 2 with atomic = 1 only */
    const int32_t *num_valid_ids;
    int32_t tokens, experts;
    int32_t model_dim, inter_dim;
    int32_t sorted_size; /* entries of sorted_token_ids / sorted_weights = rows of the sorted intermediate */
    int32_t blocks;      /* entries of sorted_expert_ids = grid size along the sorted rows */
    int32_t block_m;
    int32_t a_dtype;     /* stage 1: PSG_MX_FP4, PSG_MX_FP8 or PSG_MX_BF16_QUANT; stage 2: PSG_MX_FP4 */
    int32_t out_dtype;   /* stage 2: PSG_OUT_BF16 / PSG_OUT_FP16 */
    int32_t stage;       /* 1 or 2 */
    int32_t atomic;      /* stage 2 only */
    int32_t pad0;        /* 0 */
} psg_moe_mx_args;

int psg_moe_mx_gemm(const psg_moe_mx_args *args, void *stream);

/* a_scale of psg_moe_mx_gemm stage 1 from the scales of the quantised activations: the reference's moe_mxfp4_sort
 * (tests/kernels/utils/gemm_common_utils.py:464-598).  scale [tokens, cols] e8m0 bytes (topk = 1) or [tokens, topk, cols] (then the
 * row of a sorted id is token * topk + slot); out: ceil(sorted_size/32)*32 rows x cols bytes in the shuffled order, row i = the scale
 * row of sorted_token_ids[i]; rows of padding ids and rows from num_valid_ids[0] on are zero (every byte of out is written; the
 * reference leaves the rows past num_valid_ids[0] untouched).  cols % 8 == 0. */
int psg_moe_mx_scale_sort(const void *scale, const int32_t *sorted_token_ids, const int32_t *num_valid_ids, void *out, int32_t tokens,
                          int32_t topk, int32_t cols, int32_t sorted_size, void *stream);

/* y[t, :] = sum over the topk slots of x[t, slot, :] (fp32 sum in slot order), the pass after stage 2 with accumulate = 0
 * (kernels/moe/moe_gemm_2stage/moe_reduce.py:164-203 with use_mask = False).  dtype: PSG_OUT_BF16 / PSG_OUT_FP16 / PSG_OUT_F32,
 * the type of both x and y (the reference's dense variants, :57-61); model_dim % 4 == 0. */
int psg_moe_reduce(const void *x, void *y, int32_t tokens, int32_t topk, int32_t model_dim, int32_t dtype, void *stream);

/* The same sum with the reference's expert mask (moe_reduce.py:100-103,147-148): slot k of token t only counts when
 * expert_mask[topk_ids[t*topk + k]] != 0 (ids outside [0, experts) count as masked).  With expert parallelism the sorter
 * drops the masked experts, stage 2 never writes their rows of x, and this pass must not read them.
 * expert_mask [experts] int32, topk_ids [tokens, topk] int32. */
int psg_moe_reduce_masked(const void *x, void *y, const int32_t *expert_mask, const int32_t *topk_ids, int32_t tokens, int32_t topk,
                          int32_t model_dim, int32_t experts, int32_t dtype, void *stream);

/*
 * Expert sorting of the routed (token, slot) pairs on the device: what the reference's moe_sorting_flydsl
 * (kernels/moe/moe_sorting_kernel.py:2070-2215, the aiter moe_sorting_fwd call shape) produces, in the layout
 * psg_moe_gemm reads.  Same results as the reference's host restatements (tests/kernels/test_moe_sorting.py:74-110,
 * tests/kernels/test_moe_gemm_2stage.py:99-137): experts ascending, the pairs of an expert in (token, slot) order,
 * every expert padded to whole blocks of block_m rows with (topk << 24) | tokens, one expert id per block.
 *   topk_ids [tokens, topk] int32 (ids outside [0, experts) are dropped), topk_weights [tokens, topk] fp32;
 *   expert_mask NULL or [experts] int32: experts with 0 are dropped and the others numbered densely (test_moe_sorting.py:88-105);
 *   sorted_size >= tokens*topk + experts*block_m - topk entries of sorted_ids / sorted_weights, blocks >=
 *   ceil(sorted_size / block_m) entries of sorted_expert_ids; rows and blocks past the ones in use are written too
 *   (padding value, weight 0, expert -1); num_valid_ids = {padded rows in use, tokens};
 *   zero_buf NULL or a 16-byte aligned buffer of zero_bytes (a multiple of 16) that is cleared in the same launch (the
 *   reference clears moe_buf, the accumulate target of stage 2, in its sorter).
 *   workspace NULL or psg_moe_sorting_workspace_bytes(tokens, topk, experts) bytes of device memory (4-byte aligned;
 *   nothing in it has to be initialised): routings of more than 4096 pairs are then sorted by three launches
 *   (histograms per slice of the pairs, offsets, scatter) instead of one; without it they still sort correctly in one
 *   launch, several times slower.  The reference's sorter takes a workspace in the same place (moe_sorting_kernel.py:2030).
 * No atomics on global memory and a stable order: the output does not depend on timing.  experts <= 4096, topk <= experts
 * (PSG_E_SHAPE otherwise: the padded total can reach tokens*topk + experts*(block_m - 1), which the bound on sorted_size above
 * only covers when a token's slots go to distinct experts).
 */
typedef struct psg_moe_sort_args {
    const int32_t *topk_ids;
    const float *topk_weights;
    const int32_t *expert_mask;
    int32_t *sorted_ids;
    float *sorted_weights;
    int32_t *sorted_expert_ids;
    int32_t *num_valid_ids;
    void *zero_buf;
    int64_t zero_bytes;
    void *workspace;
    uint64_t workspace_bytes;
    int32_t tokens, topk, experts, block_m;
    int32_t sorted_size;
    int32_t blocks;
} psg_moe_sort_args;

uint64_t psg_moe_sorting_workspace_bytes(int32_t tokens, int32_t topk, int32_t experts);
int psg_moe_sorting(const psg_moe_sort_args *args, void *stream);

/* Router gating in front of the sorter: softmax over the experts, top-k, optional renormalisation.  Replaces the
 * launcher returned by build_topk_gating_softmax_module (kernels/moe/topk_gating_softmax_kernel.py:392-686; call shape
 * (gating, weights, indices, tei, num_tokens, stream) :656-663; tests/kernels/test_topk_gating_softmax.py).
 *   gating [tokens, experts] row-major, dtype 0 = fp32, 1 = bf16, 2 = fp16 (the x_dtype numbering of the quantisers);
 *   p = exp2((x - max) * log2 e) / sum in fp32; top-k = k rounds of arg-max over p, the LOWER expert index winning ties,
 *   the winner masked (:585-618); renormalize = 1 multiplies the k weights by 1 / max(their sum, 1e-20) (:623-625);
 *   weights [tokens, topk] fp32, indices [tokens, topk] int32 in the order found (descending weight),
 *   token_expert_indices NULL or [tokens, topk] int32 = k * tokens + token (:648-650).
 * experts <= 1024 (any value, not only the reference's power-of-two splits), topk <= min(32, experts). */
typedef struct psg_moe_gating_args {
    const void *gating;
    float *weights;
    int32_t *indices;
    int32_t *token_expert_indices;
    int32_t tokens, experts, topk;
    int32_t dtype;
    int32_t renormalize; /* 0 or 1 */
    int32_t pad0;        /* 0 */
} psg_moe_gating_args;

int psg_moe_topk_gating(const psg_moe_gating_args *args, void *stream);

/* Gating followed by sorting: the reference's moe_softmax_sort_flydsl (kernels/moe/moe_sorting_kernel.py:2250-2400).
 * tokens / topk / experts of both structs must agree.  psg_moe_softmax_sorting_fused(tokens, topk, experts) = 1 says that
 * this routing runs as ONE launch (tokens <= 32, tokens*topk <= 1024 and all tokens in one pass of a workgroup's 256
 * lanes, i.e. tokens <= 256 / lanes-per-token: 16 tokens for 256 experts, 32 for up to 128; every sorting workgroup repeats
 * the gating of all tokens into LDS; the reference fuses up to 16 tokens, :2313-2320): then sort->topk_ids / topk_weights are not
 * read, and gating->weights / indices / token_expert_indices are optional outputs (written when non-NULL).  Otherwise
 * the gating kernel runs first and the sorter reads its outputs: sort->topk_ids must be gating->indices and
 * sort->topk_weights gating->weights (both non-NULL). */
int psg_moe_softmax_sorting_fused(int32_t tokens, int32_t topk, int32_t experts);
int psg_moe_softmax_sorting(const psg_moe_gating_args *gating, const psg_moe_sort_args *sort, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* PSGEMM_H */
