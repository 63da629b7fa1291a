// Memory-bound small-M (M <= 32) path of the 8-bit preshuffle GEMM for gfx950.
//
// The whole cost is streaming W once (N*K bytes), so the kernel is organised around the 1 KB preshuffled
// blocks [N/16][K/64]: a wavefront owns one 16-column n-block and a contiguous slice of K, issues every
// block load of its slice up front (one fully coalesced 1 KB load per block, 16 bytes per lane, marked
// non-temporal), and feeds the registers straight into MFMA.  A workgroup is 8 wavefronts =
// (8/ksplit) n-blocks x ksplit K-slices; the K-slices of one n-block always sit in one workgroup, so the
// split-K reduction happens in LDS in a fixed order (deterministic, single launch, no workspace).
//
// A (at most 32 x K bytes, L2 resident after first touch) is read directly in fragment order:
// lane (i = lane%16, g = lane/16) needs bytes [16g,16g+16) and [64+16g, 64+16g+16) of row i per 128-byte K step.
// Rows >= M read as zero through the buffer descriptor bound.
//
// Operands are swapped like in the tiled kernel (src0 = W fragment, src1 = A fragment): a lane holds
// C[m = i][n = nblk*16 + g*4 + 0..3].
#include "psg_common.h"

namespace {

constexpr int NW = 8;       // wavefronts per workgroup
constexpr int UNROLL = 4;   // 128-byte K steps in flight per wavefront

template <int KIND>
struct Acc {
    using type = v4f;
};
template <>
struct Acc<KIND_INT8> {
    using type = v4i;
};

template <int KIND, int MB, int STORE>
__global__ void __launch_bounds__(NW * 64) k_a8w8_smallm(A8W8Params p) {
    using acc_t = typename Acc<KIND>::type;
    __shared__ __attribute__((aligned(16))) acc_t red[NW][MB][64];

    const int tid = threadIdx.x;
    const int wave = wave_id();
    const int lane = tid & 63;
    const int li = lane & 15;
    const int lg = lane >> 4;
    const int K = p.K;
    const int ks = p.ksplit;           // 1, 2, 4 or 8
    const int nbw = NW / ks;           // n-blocks per workgroup
    const int my_ks = wave % ks;
    const int my_nb = (int)blockIdx.x * nbw + wave / ks;
    const int n_blocks = p.N >> 4;
    const int steps = (K + 127) >> 7;                    // 128-byte K steps
    const int per = (steps + ks - 1) / ks;               // steps per K-slice
    const int s_begin = my_ks * per;
    const int s_end = (s_begin + per) < steps ? (s_begin + per) : steps;

    acc_t acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++) acc[mb] = (acc_t){0, 0, 0, 0};

    if (my_nb < n_blocks) {
        __amdgpu_buffer_rsrc_t rb = make_rsrc(p.b + (uint64_t)my_nb * 16ull * (uint64_t)K, 16ull * (uint64_t)K);
        __amdgpu_buffer_rsrc_t ra = make_rsrc(p.a, (uint64_t)p.M * (uint64_t)K);
        const uint32_t a_voff = (uint32_t)li * (uint32_t)K + (uint32_t)lg * 16u;

        for (int s0 = s_begin; s0 < s_end; s0 += UNROLL) {
            v4i blo[UNROLL], bhi[UNROLL], alo[UNROLL][MB], ahi[UNROLL][MB];
#pragma unroll
            for (int u = 0; u < UNROLL; u++) {
                const int s = s0 + u;
                blo[u] = bhi[u] = (v4i){0, 0, 0, 0};
#pragma unroll
                for (int mb = 0; mb < MB; mb++) alo[u][mb] = ahi[u][mb] = (v4i){0, 0, 0, 0};
                if (s < s_end) {  // wave-uniform
                    const bool has_hi = (s * 128 + 64) < K;
                    const uint32_t kb = (uint32_t)s * 128u;
                    const uint32_t boff = (uint32_t)s * 2048u;
                    blo[u] = buf_load16_nt(rb, (uint32_t)lane * 16u, boff);
                    if (has_hi) bhi[u] = buf_load16_nt(rb, (uint32_t)lane * 16u, boff + 1024u);
#pragma unroll
                    for (int mb = 0; mb < MB; mb++) {
                        // row select in the bounds-checked VGPR offset: rows >= M read as zero
                        const uint32_t voff = a_voff + (uint32_t)mb * 16u * (uint32_t)K;
                        alo[u][mb] = buf_load16(ra, voff, kb);
                        if (has_hi) ahi[u][mb] = buf_load16(ra, voff, kb + 64u);
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < UNROLL; u++) {
#pragma unroll
                for (int mb = 0; mb < MB; mb++) {
                    if constexpr (KIND == KIND_INT8) {
                        acc[mb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(blo[u], alo[u][mb], acc[mb], 0, 0, 0);
                        acc[mb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(bhi[u], ahi[u][mb], acc[mb], 0, 0, 0);
                    } else {
                        const v8i bf = {blo[u][0], blo[u][1], blo[u][2], blo[u][3], bhi[u][0], bhi[u][1], bhi[u][2], bhi[u][3]};
                        const v8i af = {alo[u][mb][0], alo[u][mb][1], alo[u][mb][2], alo[u][mb][3],
                                        ahi[u][mb][0], ahi[u][mb][1], ahi[u][mb][2], ahi[u][mb][3]};
                        acc[mb] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf, af, acc[mb], 0, 0, 0, 0, 0, 0);
                    }
                }
            }
        }
    }

    // split-K reduction through LDS, fixed order
#pragma unroll
    for (int mb = 0; mb < MB; mb++) red[wave][mb][lane] = acc[mb];
    __syncthreads();

    // work item t < nbw*MB*64 finishes (n-block t/(MB*64), m-block, lane); up to 1024 items for 512 threads
    for (int t = tid; t < nbw * MB * 64; t += NW * 64) {
        const int nbi = t / (MB * 64);
        const int mb = (t / 64) % MB;
        const int nb = (int)blockIdx.x * nbw + nbi;
        acc_t sum = red[nbi * ks][mb][lane];
        for (int j = 1; j < ks; j++) sum += red[nbi * ks + j][mb][lane];
        const int m = mb * 16 + li;
        const int n = nb * 16 + lg * 4;
        if (nb < n_blocks && m < p.M) {
            const size_t idx = (size_t)m * (size_t)p.N + (size_t)n;
            if constexpr (STORE == STORE_ACC) {
                *reinterpret_cast<acc_t*>(reinterpret_cast<uint8_t*>(p.c) + idx * 4) = sum;
            } else {
                const float sa = p.sa[m];
                const v4f sb = *reinterpret_cast<const v4f*>(p.sb + n);
                const v4f x = {((float)sum[0] * sa) * sb[0], ((float)sum[1] * sa) * sb[1], ((float)sum[2] * sa) * sb[2],
                               ((float)sum[3] * sa) * sb[3]};
                store_c4(p, idx, n, x);
            }
        }
    }
}

template <int KIND, int MB, int STORE>
hipError_t launch_one(const A8W8Params& p, hipStream_t stream) {
    const int nbw = NW / p.ksplit;
    const int n_blocks = p.N / 16;
    const int grid = (n_blocks + nbw - 1) / nbw;
    hipLaunchKernelGGL((k_a8w8_smallm<KIND, MB, STORE>), dim3(grid), dim3(NW * 64), 0, stream, p);
    return hipGetLastError();
}

}  // namespace

// Host entry used by the C-ABI layer.  Requires 1 <= M <= 32 and p.ksplit in {1,2,4,8}.
hipError_t psg_launch_a8w8_smallm(const A8W8Params& p, int kind, int store, hipStream_t stream) {
    const int mb = p.M <= 16 ? 1 : 2;
#define PSG_GO(KIND_, MB_)                                                                    \
    return store == STORE_ACC ? launch_one<KIND_, MB_, STORE_ACC>(p, stream) : launch_one<KIND_, MB_, STORE_C>(p, stream);
    if (kind == KIND_INT8) {
        if (mb == 1) { PSG_GO(KIND_INT8, 1) } else { PSG_GO(KIND_INT8, 2) }
    }
    if (kind == KIND_FP8) {
        if (mb == 1) { PSG_GO(KIND_FP8, 1) } else { PSG_GO(KIND_FP8, 2) }
    }
#undef PSG_GO
    return hipErrorInvalidValue;
}
