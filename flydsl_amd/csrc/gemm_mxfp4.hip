// MXFP4 (e2m1 x e2m1, one e8m0 scale per 32 K elements) preshuffle GEMM for gfx950.
//
// v_mfma_scale_f32_16x16x128_f8f6f4 with both operand formats = fp4: a lane supplies 32 consecutive K
// elements (16 bytes) of one row plus one e8m0 scale byte that applies to exactly those 32 elements.
//   * W operand: one preshuffled 1 KB block [n/16][kbyte/64] is exactly one MFMA operand
//     (lane l = 16*klane + nlane reads bytes [16l, 16l+16)).
//   * Scales: the shuffled layout stores, per (32-row chunk, 256-K chunk), 64 dwords; lane l's dword holds
//     the four bytes (128-K half kh, 16-row half h) -> byte kh*2 + h, selected with the MFMA's opsel.
//   * Operands are swapped (src0 = W, src1 = A) so a lane ends up with 4 consecutive N columns.
//
// This file holds the small-M kernel (M <= 32, wavefront = one 32-column n-pair x a K slice, LDS split-K
// reduction in a fixed order); the tiled MFMA mainloop shares its source with the 8-bit kernels.
#include "psg_common.h"

namespace {

constexpr int TKB = 128;  // bytes of packed K per mainloop step (= 256 K elements = one scale chunk)

// fp4 operands occupy the low four dwords of the eight-dword MFMA operand
__device__ __forceinline__ v8i widen(v4i x) { return __builtin_shufflevector(x, x, 0, 1, 2, 3, -1, -1, -1, -1); }

template <int OPSEL_W, int OPSEL_A>
__device__ __forceinline__ v4f mx_mfma(v4i w, v4i a, v4f c, int scale_w, int scale_a) {
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(widen(w), widen(a), c, 4, 4, OPSEL_W, scale_w, OPSEL_A, scale_a);
}

template <class P>
__device__ __forceinline__ void store_mx4(const P& p, int store, size_t idx, v4f v) {
    if (store == STORE_ACC) {
        *reinterpret_cast<v4f*>(reinterpret_cast<float*>(p.c) + idx) = v;
    } else {
        v2i r = p.out == OUT_BF16 ? pack4_out16<OUT_BF16>(v[0], v[1], v[2], v[3]) : pack4_out16<OUT_FP16>(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<v2i*>(reinterpret_cast<uint16_t*>(p.c) + idx) = r;
    }
}

// ------------------------------------------------------------------------------------------------
// small-M kernel: M <= 64; wavefront = (n-pair of 32 columns, K slice of 256-K steps)
// ------------------------------------------------------------------------------------------------
constexpr int UNROLL = 2;

// NW = wavefronts per workgroup (4 or 8), as in the 8-bit streaming kernel
template <int MB, int NW, int STORE>
__global__ void __launch_bounds__(NW * 64) k_mxfp4_smallm(MxParams p) {
    __shared__ __attribute__((aligned(16))) v4f red[NW][MB * 2][64];

    const int tid = threadIdx.x;
    const int wave = wave_id();
    const int lane = tid & 63;
    const int li = lane & 15;
    const int lg = lane >> 4;
    const int KP = p.K >> 1;
    const int KT = p.K >> 8;
    // four wavefronts are always four K slices: a compile-time constant spares the run-time divisions in front of the loads
    const int ks = NW == 4 ? 4 : p.ksplit;
    const int npw = NW / ks;  // n-pairs per workgroup
    const int my_ks = wave % ks;
    // workgroups go round-robin over the 8 XCDs: give each XCD one contiguous range of n-pairs, so the 128-byte lines of C
    // that two neighbouring n-pairs share are completed in one L2
    const int bid = (gridDim.x & 7) == 0 ? (int)((blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3)) : (int)blockIdx.x;
    const int my_np = bid * npw + wave / ks;
    const int n_pairs = p.N >> 5;
    const int per = (KT + ks - 1) / ks;
    const int s_begin = my_ks * per;
    const int s_end = (s_begin + per) < KT ? (s_begin + per) : KT;

    v4f acc[MB][2];
#pragma unroll
    for (int mb = 0; mb < MB; mb++) acc[mb][0] = acc[mb][1] = (v4f){0.f, 0.f, 0.f, 0.f};

    if (my_np < n_pairs) {
        __amdgpu_buffer_rsrc_t rb = make_rsrc(p.b + (uint64_t)my_np * 32ull * (uint64_t)KP, 32ull * (uint64_t)KP);
        __amdgpu_buffer_rsrc_t ra = make_rsrc(p.a, (uint64_t)p.M * (uint64_t)KP);
        const uint64_t chunk_bytes = (uint64_t)KT * 256ull;
        constexpr int MC = (MB + 1) / 2;  // 32-row chunks of A scales
        __amdgpu_buffer_rsrc_t rsa = make_rsrc(p.sa, (uint64_t)((p.M + 31) >> 5) * chunk_bytes);
        __amdgpu_buffer_rsrc_t rsb = make_rsrc(p.sb + (uint64_t)my_np * chunk_bytes, chunk_bytes);
        const uint32_t a_voff = (uint32_t)li * (uint32_t)KP + (uint32_t)lg * 16u;

        for (int s0 = s_begin; s0 < s_end; s0 += UNROLL) {
            v4i bq[UNROLL][2][2], aq[UNROLL][MB][2];
            int sav[UNROLL][(MB + 1) / 2], sbv[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; u++) {
                const int s = s0 + u;
                sbv[u] = 0;
#pragma unroll
                for (int mc = 0; mc < (MB + 1) / 2; mc++) sav[u][mc] = 0;
#pragma unroll
                for (int nb = 0; nb < 2; nb++) bq[u][nb][0] = bq[u][nb][1] = (v4i){0, 0, 0, 0};
#pragma unroll
                for (int mb = 0; mb < MB; mb++) aq[u][mb][0] = aq[u][mb][1] = (v4i){0, 0, 0, 0};
                if (s < s_end) {  // wave-uniform
#pragma unroll
                    for (int nb = 0; nb < 2; nb++) {
                        const uint32_t voff = (uint32_t)lane * 16u + (uint32_t)nb * 16u * (uint32_t)KP;
                        bq[u][nb][0] = buf_load16_nt(rb, voff, (uint32_t)s * 2048u);
                        bq[u][nb][1] = buf_load16_nt(rb, voff, (uint32_t)s * 2048u + 1024u);
                    }
#pragma unroll
                    for (int mb = 0; mb < MB; mb++) {
                        const uint32_t voff = a_voff + (uint32_t)mb * 16u * (uint32_t)KP;
                        aq[u][mb][0] = buf_load16(ra, voff, (uint32_t)s * TKB);
                        aq[u][mb][1] = buf_load16(ra, voff, (uint32_t)s * TKB + 64u);
                    }
#pragma unroll
                    for (int mc = 0; mc < MC; mc++) sav[u][mc] = buf_load4(rsa, (uint32_t)mc * (uint32_t)chunk_bytes + (uint32_t)lane * 4u, (uint32_t)s * 256u);
                    sbv[u] = buf_load4(rsb, (uint32_t)lane * 4u, (uint32_t)s * 256u);
                }
            }
            // keep every load of the chunk ahead of the first MFMA (the scheduler would otherwise sink some)
            __builtin_amdgcn_sched_barrier(0);
            static_for<UNROLL>([&](auto U) {
                constexpr int u = decltype(U)::value;
                static_for<2>([&](auto KH) {
                    constexpr int kh = decltype(KH)::value;
                    static_for<2>([&](auto NB) {
                        constexpr int nb = decltype(NB)::value;
                        static_for<MB>([&](auto MBI) {
                            constexpr int mb = decltype(MBI)::value;
                            acc[mb][nb] = mx_mfma<kh * 2 + nb, kh * 2 + (mb & 1)>(bq[u][nb][kh], aq[u][mb][kh], acc[mb][nb], sbv[u], sav[u][mb / 2]);
                        });
                    });
                });
            });
        }
    }

#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
        red[wave][mb * 2 + 0][lane] = acc[mb][0];
        red[wave][mb * 2 + 1][lane] = acc[mb][1];
    }
    __syncthreads();

    // work item t < npw*MB*2*64 finishes (n-pair, m-block, n-block of the pair, lane)
    for (int t = tid; t < npw * MB * 2 * 64; t += NW * 64) {
        const int npi = t / (MB * 2 * 64);
        const int f = (t / 64) % (MB * 2);
        const int mb = f >> 1, nb = f & 1;
        const int np = bid * npw + npi;
        // all partial sums are read in one batch (no wait between them), then added in slice order
        v4f part[NW];
#pragma unroll
        for (int j = 0; j < NW; j++) part[j] = red[npi * ks + (j < ks ? j : 0)][f][lane];
        v4f sum = part[0];
#pragma unroll
        for (int j = 1; j < NW; j++)
            if (j < ks) sum += part[j];
        const int m = mb * 16 + li;
        const int n = np * 32 + nb * 16 + lg * 4;
        if (np < n_pairs && m < p.M) store_mx4(p, STORE, (size_t)m * (size_t)p.N + (size_t)n, sum);
    }
}

template <int MB, int NW, int STORE>
hipError_t launch_smallm(const MxParams& p, hipStream_t stream) {
    const int npw = NW / p.ksplit;
    const int n_pairs = p.N / 32;
    hipLaunchKernelGGL((k_mxfp4_smallm<MB, NW, STORE>), dim3((n_pairs + npw - 1) / npw), dim3(NW * 64), 0, stream, p);
    return hipGetLastError();
}

}  // namespace

// requires 1 <= M <= 64, nw (wavefronts per workgroup) in {4,8} and p.ksplit a power of two <= nw
hipError_t psg_launch_mxfp4_smallm(const MxParams& p, int store, int nw, hipStream_t stream) {
#define PSG_GO(MB_)                                                                                             \
    if (nw == 4) return store == STORE_ACC ? launch_smallm<MB_, 4, STORE_ACC>(p, stream) : launch_smallm<MB_, 4, STORE_C>(p, stream); \
    return store == STORE_ACC ? launch_smallm<MB_, 8, STORE_ACC>(p, stream) : launch_smallm<MB_, 8, STORE_C>(p, stream);
    if (p.M <= 16) { PSG_GO(1) }
    if (p.M <= 32) { PSG_GO(2) }
    if (p.M <= 48) { PSG_GO(3) }
    PSG_GO(4)
#undef PSG_GO
}
