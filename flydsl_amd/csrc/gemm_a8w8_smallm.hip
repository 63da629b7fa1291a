// Memory-bound small-M (M <= 32) path of the 8-bit preshuffle GEMM for gfx950.
//
// The whole cost is streaming W once (N*K bytes), so the kernel is organised around the 1 KB preshuffled
// blocks [N/16][K/64]: a wavefront owns one 16-column n-block and a contiguous slice of K, issues the block
// loads of a chunk of K steps up front (one fully coalesced 1 KB load per block, 16 bytes per lane) and
// feeds the registers straight into MFMA.  A workgroup is NW (4 or 8) wavefronts = (NW/ksplit) n-blocks x ksplit
// K-slices; the K-slices of one n-block always sit in one workgroup, so the split-K reduction happens in LDS
// in a fixed order (deterministic, single launch, no workspace).
//
// A (at most 32 x K bytes, L2 resident after first touch) is needed in fragment order: lane
// (i = lane%16, g = lane/16) wants bytes [16g,16g+16) and [64+16g, 64+16g+16) of row i per K step, i.e. 16
// different rows per load instruction.  Reading it that way from global memory costs more address
// processing than the whole W stream, so each wavefront instead reads its slice of A with row-contiguous
// loads (32 or 16 lanes per row) into a private 8 KB LDS patch (XOR-swizzled 16-byte chunks) and picks the
// fragments up from there.  The patch is private to the wavefront: no barrier is involved.
// Rows >= M and bytes >= K read as zero through the buffer descriptor bound.
//
// Operands are swapped like in the tiled kernel (src0 = W fragment, src1 = A fragment): a lane holds
// C[m = i][n = nblk*16 + g*4 + 0..3].
#include "psg_common.h"

namespace {

constexpr int UNROLL = 4;   // 128-byte K steps per chunk when 16 rows of A are staged (2 when 32 rows are)

template <int KIND>
struct Acc {
    using type = v4f;
};
template <>
struct Acc<KIND_INT8> {
    using type = v4i;
};

// NB = n-blocks per wavefront: with two, the A slice a wavefront stages is shared by twice as much of W.
// NW = wavefronts per workgroup (4 or 8): four with longer K slices leave fewer partial sums to reduce and smaller
// workgroups to place; eight give more, shorter slices when K is short.
template <int KIND, int MB, int NB, int NW, int STORE>
__global__ void __launch_bounds__(NW * 64) k_a8w8_smallm(A8W8Params p) {
    using acc_t = typename Acc<KIND>::type;
    constexpr int ROWS = 16 * MB;          // A rows staged
    constexpr int SPS = UNROLL / MB;       // K steps per staging pass (patch = ROWS x SPS*128 bytes = 8 KB)
    constexpr int CPR = SPS * 8;           // 16-byte chunks per staged row (32 or 16)
    __shared__ __attribute__((aligned(16))) v4i patch[NW][512];
    __shared__ __attribute__((aligned(16))) acc_t red[NW][NB * MB][64];

    const int tid = threadIdx.x;
    const int wave = wave_id();
    const int lane = tid & 63;
    const int li = lane & 15;
    const int lg = lane >> 4;
    constexpr bool IS16 = KIND == KIND_FP16 || KIND == KIND_BF16;
    const int K = IS16 ? (p.K << 1) : p.K;   // BYTES per operand row from here on
    const int ks = p.ksplit;           // 1, 2, 4 or 8
    const int nbw = NW / ks;           // wavefront groups (K-slice sets) per workgroup, NB n-blocks each
    const int my_ks = wave % ks;
    const int my_nb = ((int)blockIdx.x * nbw + wave / ks) * NB;
    const int n_blocks = p.N >> 4;
    const int steps = (K + 127) >> 7;                    // 128-byte K steps
    const int per = (steps + ks - 1) / ks;               // steps per K-slice
    const int s_begin = my_ks * per;
    const int s_end = (s_begin + per) < steps ? (s_begin + per) : steps;

    acc_t acc[NB][MB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
#pragma unroll
        for (int mb = 0; mb < MB; mb++) acc[nb][mb] = (acc_t){0, 0, 0, 0};

    // The scales of the outputs this thread will finish are fetched early (right behind the first chunk's loads),
    // so that their latency does not sit behind the reduction barrier at the very end of the kernel.  Finishing
    // work item t = tid (+ NW*64): (n-block t/(MB*64) of the workgroup, m-block, lane).
    constexpr int FIN = (NB * MB * NW * 64 + NW * 64 - 1) / (NW * 64);  // items per thread at ksplit 1
    float fin_sa[FIN];
    v4f fin_sb[FIN];
    auto fetch_scales = [&]() {
        if constexpr (STORE != STORE_ACC && !IS16) {
#pragma unroll
            for (int f = 0; f < FIN; f++) {
                const int t = tid + f * NW * 64;
                const int nbq = (int)blockIdx.x * nbw * NB + t / (MB * 64);
                const int m = ((t / 64) % MB) * 16 + li;
                const bool live = t < nbw * NB * MB * 64 && nbq < n_blocks && m < p.M;
                // clamp the ADDRESS for dead items instead of selecting the loaded value (a select would force
                // a wait for these cold loads right here)
                fin_sa[f] = p.sa[live ? m : 0];
                fin_sb[f] = *reinterpret_cast<const v4f*>(p.sb + (live ? nbq * 16 + lg * 4 : 0));
            }
        }
    };
    bool scales_fetched = false;

    if (my_nb < n_blocks) {
        // this wavefront's NB n-blocks; a block past N/16 (odd block count) reads as zero
        const uint64_t b_left = (uint64_t)(n_blocks - my_nb) * 16ull * (uint64_t)K;
        const uint64_t b_mine = (uint64_t)NB * 16ull * (uint64_t)K;
        __amdgpu_buffer_rsrc_t rb = make_rsrc(p.b + (uint64_t)my_nb * 16ull * (uint64_t)K, b_left < b_mine ? b_left : b_mine);
        __amdgpu_buffer_rsrc_t ra = make_rsrc(p.a, (uint64_t)p.M * (uint64_t)K);
        v4i* my_patch = patch[wave];
        // staging geometry: item = pass*64 + lane -> (row = item / CPR, chunk = item % CPR)
        const int st_c = lane % CPR;
        const int st_r0 = lane / CPR;                   // + pass * (64 / CPR)
        const uint32_t slice_end = (uint32_t)(s_end * 128 < K ? s_end * 128 : K);

        for (int s0 = s_begin; s0 < s_end; s0 += SPS) {
            // 1. A first: it comes from L2 and must not queue behind the W stream (loads return in order)
            const uint32_t kbase = (uint32_t)s0 * 128u;
            v4i tmp[8];
#pragma unroll
            for (int ps = 0; ps < 8; ps++) {
                const int r = st_r0 + ps * (64 / CPR);
                const uint32_t kbyte = kbase + (uint32_t)st_c * 16u;
                tmp[ps] = buf_load16(ra, kbyte < slice_end ? (uint32_t)r * (uint32_t)K + kbyte : 0xFFFFFFF0u, 0);
            }
            // (the fences keep the machine scheduler from sinking loads below their first use to save registers,
            // which would serialise two memory latencies)
            __builtin_amdgcn_sched_barrier(0);
            // 2. the W blocks of this chunk, all in flight at once
            v4i blo[NB][SPS], bhi[NB][SPS];
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
#pragma unroll
                for (int u = 0; u < SPS; u++) {
                    const int s = s0 + u;
                    const bool has_lo = s < s_end;                       // wave-uniform
                    const bool has_hi = has_lo && (s * 128 + 64) < K;    // K % 128 == 64: last step has no upper half
                    const uint32_t boff = has_lo ? (uint32_t)s * 2048u : 0u;
                    const uint32_t voff = (uint32_t)lane * 16u + (uint32_t)nb * 16u * (uint32_t)K;
                    blo[nb][u] = buf_load16_nt(rb, has_lo ? voff : 0xFFFFFFF0u, boff);
                    bhi[nb][u] = buf_load16_nt(rb, has_hi ? voff : 0xFFFFFFF0u, has_hi ? boff + 1024u : 0u);
                }
            if (!scales_fetched) {  // first chunk only (wave-uniform)
                fetch_scales();
                scales_fetched = true;
            }
            __builtin_amdgcn_sched_barrier(0);
            // 3. A through the private LDS patch into fragment order while W is still on its way
#pragma unroll
            for (int ps = 0; ps < 8; ps++) {
                const int r = st_r0 + ps * (64 / CPR);
                my_patch[r * CPR + (st_c ^ (r & 15))] = tmp[ps];
            }
            v4i alo[SPS][MB], ahi[SPS][MB];
#pragma unroll
            for (int t = 0; t < SPS; t++)
#pragma unroll
                for (int mb = 0; mb < MB; mb++) {
                    const int r = mb * 16 + li;
                    alo[t][mb] = my_patch[r * CPR + ((t * 8 + lg) ^ (r & 15))];
                    ahi[t][mb] = my_patch[r * CPR + ((t * 8 + 4 + lg) ^ (r & 15))];
                }
            // 4. MFMA as W arrives
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
#pragma unroll
                for (int t = 0; t < SPS; t++)
#pragma unroll
                    for (int mb = 0; mb < MB; mb++) {
                        if constexpr (KIND == KIND_INT8) {
                            acc[nb][mb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(blo[nb][t], alo[t][mb], acc[nb][mb], 0, 0, 0);
                            acc[nb][mb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(bhi[nb][t], ahi[t][mb], acc[nb][mb], 0, 0, 0);
                        } else if constexpr (KIND == KIND_BF16) {
                            acc[nb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, blo[nb][t]), __builtin_bit_cast(v8bf, alo[t][mb]), acc[nb][mb], 0, 0, 0);
                            acc[nb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, bhi[nb][t]), __builtin_bit_cast(v8bf, ahi[t][mb]), acc[nb][mb], 0, 0, 0);
                        } else if constexpr (KIND == KIND_FP16) {
                            acc[nb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, blo[nb][t]), __builtin_bit_cast(v8h, alo[t][mb]), acc[nb][mb], 0, 0, 0);
                            acc[nb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, bhi[nb][t]), __builtin_bit_cast(v8h, ahi[t][mb]), acc[nb][mb], 0, 0, 0);
                        } else {
                            const v8i bf = {blo[nb][t][0], blo[nb][t][1], blo[nb][t][2], blo[nb][t][3],
                                            bhi[nb][t][0], bhi[nb][t][1], bhi[nb][t][2], bhi[nb][t][3]};
                            const v8i af = {alo[t][mb][0], alo[t][mb][1], alo[t][mb][2], alo[t][mb][3],
                                            ahi[t][mb][0], ahi[t][mb][1], ahi[t][mb][2], ahi[t][mb][3]};
                            acc[nb][mb] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf, af, acc[nb][mb], 0, 0, 0, 0, 0, 0);
                        }
                    }
        }
    }

    if (!scales_fetched) fetch_scales();  // wavefronts without an n-block still finish outputs

    // split-K reduction through LDS, fixed order
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
#pragma unroll
        for (int mb = 0; mb < MB; mb++) red[wave][nb * MB + mb][lane] = acc[nb][mb];
    __syncthreads();

#pragma unroll
    for (int f = 0; f < FIN; f++) {
        const int t = tid + f * NW * 64;
        if (t < nbw * NB * MB * 64) {
            const int nbi = t / (MB * 64);  // n-block of the workgroup: wavefront group nbi / NB, its block nbi % NB
            const int mb = (t / 64) % MB;
            const int grp = nbi / NB, frag = (nbi % NB) * MB + mb;
            const int nbq = (int)blockIdx.x * nbw * NB + nbi;
            acc_t sum = red[grp * ks][frag][lane];
            for (int j = 1; j < ks; j++) sum += red[grp * ks + j][frag][lane];
            const int m = mb * 16 + li;
            const int n = nbq * 16 + lg * 4;
            if (nbq < n_blocks && m < p.M) {
                const size_t idx = (size_t)m * (size_t)p.N + (size_t)n;
                if constexpr (STORE == STORE_ACC) {
                    *reinterpret_cast<acc_t*>(reinterpret_cast<uint8_t*>(p.c) + idx * 4) = sum;
                } else {
                    v4f x;
                    if constexpr (IS16) {
                        x = (v4f){(float)sum[0], (float)sum[1], (float)sum[2], (float)sum[3]};
                    } else {
                        const float sa = fin_sa[f];
                        const v4f sb = fin_sb[f];
                        x = (v4f){((float)sum[0] * sa) * sb[0], ((float)sum[1] * sa) * sb[1], ((float)sum[2] * sa) * sb[2],
                                  ((float)sum[3] * sa) * sb[3]};
                    }
                    store_c4(p, idx, n, x);
                }
            }
        }
    }
}

template <int KIND, int MB, int NB, int NW, int STORE>
hipError_t launch_one(const A8W8Params& p, hipStream_t stream) {
    const int per_wg = (NW / p.ksplit) * NB;  // n-blocks per workgroup
    const int n_blocks = p.N / 16;
    const int grid = (n_blocks + per_wg - 1) / per_wg;
    hipLaunchKernelGGL((k_a8w8_smallm<KIND, MB, NB, NW, STORE>), dim3(grid), dim3(NW * 64), 0, stream, p);
    return hipGetLastError();
}

template <int KIND, int STORE>
hipError_t launch_kind(const A8W8Params& p, int nb, int nw, hipStream_t stream) {
    const int mb = p.M <= 16 ? 1 : 2;
#define PSG_GO(MB_, NB_)                                                                                   \
    return nw == 4 ? launch_one<KIND, MB_, NB_, 4, STORE>(p, stream) : launch_one<KIND, MB_, NB_, 8, STORE>(p, stream);
    if (mb == 1) {
        if (nb == 2) { PSG_GO(1, 2) } else { PSG_GO(1, 1) }
    }
    if (nb == 2) { PSG_GO(2, 2) } else { PSG_GO(2, 1) }
#undef PSG_GO
}

}  // namespace

// Host entry used by the C-ABI layer.  Requires 1 <= M <= 32, nw (wavefronts per workgroup) in {4,8}, p.ksplit a power of
// two <= nw, nb (n-blocks per wavefront) in {1,2}.
hipError_t psg_launch_a8w8_smallm(const A8W8Params& p, int kind, int store, int nb, int nw, hipStream_t stream) {
    if (kind == KIND_INT8)
        return store == STORE_ACC ? launch_kind<KIND_INT8, STORE_ACC>(p, nb, nw, stream) : launch_kind<KIND_INT8, STORE_C>(p, nb, nw, stream);
    if (kind == KIND_FP8)
        return store == STORE_ACC ? launch_kind<KIND_FP8, STORE_ACC>(p, nb, nw, stream) : launch_kind<KIND_FP8, STORE_C>(p, nb, nw, stream);
    if (kind == KIND_BF16)
        return store == STORE_ACC ? launch_kind<KIND_BF16, STORE_ACC>(p, nb, nw, stream) : launch_kind<KIND_BF16, STORE_C>(p, nb, nw, stream);
    if (kind == KIND_FP16)
        return store == STORE_ACC ? launch_kind<KIND_FP16, STORE_ACC>(p, nb, nw, stream) : launch_kind<KIND_FP16, STORE_C>(p, nb, nw, stream);
    return hipErrorInvalidValue;
}
