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
// Two kernels: a tiled one (A staged through swizzled LDS, 4 wavefronts along N) and a small-M one
// (M <= 32, wavefront = one 32-column n-pair x a K slice, LDS split-K reduction in a fixed order).
#include "psg_common.h"

namespace {

constexpr int TKB = 128;  // bytes of packed K per mainloop step (= 256 K elements = one scale chunk)

__device__ __forceinline__ int lds_off(int row, int kc) { return row * TKB + ((kc ^ ((row >> 1) & 7)) << 4); }

__device__ __forceinline__ void tile_coords(int id, int tiles_m, int tiles_n, int group_m, int& tm, int& tn) {
    const int num = tiles_m * tiles_n;
    const int q = num >> 3, r = num & 7;
    const int xcd = id & 7, in_xcd = id >> 3;
    const int wg = xcd * q + (xcd < r ? xcd : r) + in_xcd;
    const int per_group = group_m * tiles_n;
    const int g = wg / per_group;
    const int first_m = g * group_m;
    const int size_m = (tiles_m - first_m) < group_m ? (tiles_m - first_m) : group_m;
    const int in_g = wg - g * per_group;
    tm = first_m + in_g % size_m;
    tn = in_g / size_m;
}

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
// tiled kernel: tile (16*MR) x (64*NR) x 256 K; MR and NR even (scale chunks cover 32 rows)
// ------------------------------------------------------------------------------------------------
template <int MR, int NR, int STORE>
__global__ void __launch_bounds__(256) k_mxfp4_tiled(MxParams p) {
    constexpr int TM = 16 * MR;
    constexpr int TN = 64 * NR;
    constexpr int A_LOADS = TM / 32;
    constexpr int MP = MR / 2, NP = NR / 2;
    static_assert(MR % 2 == 0 && NR % 2 == 0, "scale chunks cover 32 rows");

    __shared__ __attribute__((aligned(16))) uint8_t lds[2][TM * TKB];

    const int tid = threadIdx.x;
    const int wave = wave_id();
    const int lane = tid & 63;
    const int li = lane & 15;
    const int lg = lane >> 4;

    const int tiles_m = (p.M + TM - 1) / TM;
    const int tiles_n = (p.N + TN - 1) / TN;
    int tm, tn;
    tile_coords((int)blockIdx.x, tiles_m, tiles_n, p.group_m, tm, tn);
    const int m0 = tm * TM;
    const int n0 = tn * TN;
    const int KP = p.K >> 1;   // packed bytes per row
    const int KT = p.K >> 8;   // 256-K steps

    __amdgpu_buffer_rsrc_t ra = make_rsrc(p.a + (uint64_t)m0 * KP, (uint64_t)(p.M - m0) * (uint64_t)KP);
    const int nb0 = (n0 >> 4) + wave * NR;
    const uint64_t b_off = (uint64_t)nb0 * 16ull * (uint64_t)KP;
    const uint64_t b_total = (uint64_t)p.N * (uint64_t)KP;
    __amdgpu_buffer_rsrc_t rb = make_rsrc(p.b + (b_off < b_total ? b_off : b_total), b_off < b_total ? b_total - b_off : 0);
    // scales: 256 bytes per (32-row chunk, 256-K chunk)
    const uint64_t chunk_bytes = (uint64_t)KT * 256ull;
    const uint64_t sa_chunks = (uint64_t)((p.M + 31) >> 5);
    const uint64_t sa_first = (uint64_t)(m0 >> 5);
    __amdgpu_buffer_rsrc_t rsa = make_rsrc(p.sa + sa_first * chunk_bytes, (sa_chunks - sa_first) * chunk_bytes);
    const uint64_t sb_chunks = (uint64_t)(p.N >> 5);
    const uint64_t sb_first = (uint64_t)((n0 >> 5) + wave * NP);
    __amdgpu_buffer_rsrc_t rsb = make_rsrc(p.sb + (sb_first < sb_chunks ? sb_first : sb_chunks) * chunk_bytes,
                                           sb_first < sb_chunks ? (sb_chunks - sb_first) * chunk_bytes : 0);

    const int a_row0 = tid >> 3;
    const int a_kc = tid & 7;
    const uint32_t a_goff0 = (uint32_t)a_row0 * (uint32_t)KP + (uint32_t)a_kc * 16u;

    v4f acc[MR][NR];
#pragma unroll
    for (int mi = 0; mi < MR; mi++)
#pragma unroll
        for (int ni = 0; ni < NR; ni++) acc[mi][ni] = (v4f){0.f, 0.f, 0.f, 0.f};

    v4i areg[A_LOADS];
    v4i bq[2][NR][2];
    int sav[2][MP], sbv[2][NP];

    // Loads never sit under control flow: a K step past the end (prefetch of the last iteration) is
    // redirected past the descriptor bounds, where the hardware returns zero without touching memory.
    auto load_a = [&](int kt) {
        const bool valid = kt < KT;
#pragma unroll
        for (int j = 0; j < A_LOADS; j++) {
            const uint32_t off = a_goff0 + (uint32_t)j * 32u * (uint32_t)KP + (uint32_t)kt * TKB;
            areg[j] = buf_load16(ra, valid ? off : 0xFFFFFFF0u, 0);
        }
    };
    auto store_a = [&](int stage) {
#pragma unroll
        for (int j = 0; j < A_LOADS; j++)
            *reinterpret_cast<v4i*>(&lds[stage][lds_off(a_row0 + 32 * j, a_kc)]) = areg[j];
    };
    auto load_b = [&](int kt, auto ST) {
        constexpr int st = decltype(ST)::value;
        const bool valid = kt < KT;
        const uint32_t koff = valid ? (uint32_t)kt * 2048u : 0u;
        const uint32_t soff = valid ? (uint32_t)kt * 256u : 0u;
#pragma unroll
        for (int ni = 0; ni < NR; ni++) {
            const uint32_t voff = valid ? (uint32_t)lane * 16u + (uint32_t)ni * 16u * (uint32_t)KP : 0xFFFFFFF0u;
            bq[st][ni][0] = buf_load16(rb, voff, koff);
            bq[st][ni][1] = buf_load16(rb, voff, valid ? koff + 1024u : 0u);
        }
#pragma unroll
        for (int mp = 0; mp < MP; mp++)
            sav[st][mp] = buf_load4(rsa, valid ? (uint32_t)mp * (uint32_t)chunk_bytes + (uint32_t)lane * 4u : 0xFFFFFFF0u, soff);
#pragma unroll
        for (int np = 0; np < NP; np++)
            sbv[st][np] = buf_load4(rsb, valid ? (uint32_t)np * (uint32_t)chunk_bytes + (uint32_t)lane * 4u : 0xFFFFFFF0u, soff);
    };
    // A fragments (m-block, 128-K half) are read one step ahead of the MFMAs that use them
    auto compute = [&](auto ST) {
        constexpr int st = decltype(ST)::value;
        v4i af[2];
        af[0] = *reinterpret_cast<const v4i*>(&lds[st][lds_off(li, lg)]);
        static_for<MR * 2>([&](auto IDX) {
            constexpr int idx = decltype(IDX)::value;
            constexpr int mi = idx / 2, kh = idx % 2;
            if constexpr (idx + 1 < MR * 2) {
                constexpr int mi1 = (idx + 1) / 2, kh1 = (idx + 1) % 2;
                af[(idx + 1) & 1] = *reinterpret_cast<const v4i*>(&lds[st][lds_off(mi1 * 16 + li, kh1 * 4 + lg)]);
            }
            __builtin_amdgcn_sched_barrier(0);
            static_for<NR>([&](auto NI) {
                constexpr int ni = decltype(NI)::value;
                acc[mi][ni] = mx_mfma<kh * 2 + (ni & 1), kh * 2 + (mi & 1)>(bq[st][ni][kh], af[idx & 1], acc[mi][ni],
                                                                               sbv[st][ni / 2], sav[st][mi / 2]);
            });
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    load_a(0);
    load_b(0, S0{});
    store_a(0);
    __syncthreads();

    // two K steps per iteration (ping-pong); an odd step count ends with one step on zero operands
    for (int kt = 0; kt < KT; kt += 2) {
        load_a(kt + 1);
        load_b(kt + 1, S1{});
        compute(S0{});
        store_a(1);
        __syncthreads();

        load_a(kt + 2);
        load_b(kt + 2, S0{});
        compute(S1{});
        store_a(0);
        __syncthreads();
    }

    static_for<MR>([&](auto MI) {
        constexpr int mi = decltype(MI)::value;
        const int m = m0 + mi * 16 + li;
        if (m < p.M) {
            static_for<NR>([&](auto NI) {
                constexpr int ni = decltype(NI)::value;
                const int n = n0 + (wave * NR + ni) * 16 + lg * 4;
                if (n < p.N) store_mx4(p, STORE, (size_t)m * (size_t)p.N + (size_t)n, acc[mi][ni]);
            });
        }
    });
}

// ------------------------------------------------------------------------------------------------
// small-M kernel: M <= 32; wavefront = (n-pair of 32 columns, K slice of 256-K steps)
// ------------------------------------------------------------------------------------------------
constexpr int NW = 8;
constexpr int UNROLL = 2;

template <int MB, int STORE>
__global__ void __launch_bounds__(NW * 64) k_mxfp4_smallm(MxParams p) {
    __shared__ __attribute__((aligned(16))) v4f red[NW][MB * 2][64];

    const int tid = threadIdx.x;
    const int wave = wave_id();
    const int lane = tid & 63;
    const int li = lane & 15;
    const int lg = lane >> 4;
    const int KP = p.K >> 1;
    const int KT = p.K >> 8;
    const int ks = p.ksplit;
    const int npw = NW / ks;  // n-pairs per workgroup
    const int my_ks = wave % ks;
    const int my_np = (int)blockIdx.x * npw + wave / ks;
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
        __amdgpu_buffer_rsrc_t rsa = make_rsrc(p.sa, chunk_bytes);  // M <= 32: one chunk
        __amdgpu_buffer_rsrc_t rsb = make_rsrc(p.sb + (uint64_t)my_np * chunk_bytes, chunk_bytes);
        const uint32_t a_voff = (uint32_t)li * (uint32_t)KP + (uint32_t)lg * 16u;

        for (int s0 = s_begin; s0 < s_end; s0 += UNROLL) {
            v4i bq[UNROLL][2][2], aq[UNROLL][MB][2];
            int sav[UNROLL], sbv[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; u++) {
                const int s = s0 + u;
                sav[u] = sbv[u] = 0;
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
                    sav[u] = buf_load4(rsa, (uint32_t)lane * 4u, (uint32_t)s * 256u);
                    sbv[u] = buf_load4(rsb, (uint32_t)lane * 4u, (uint32_t)s * 256u);
                }
            }
            static_for<UNROLL>([&](auto U) {
                constexpr int u = decltype(U)::value;
                static_for<2>([&](auto KH) {
                    constexpr int kh = decltype(KH)::value;
                    static_for<2>([&](auto NB) {
                        constexpr int nb = decltype(NB)::value;
                        static_for<MB>([&](auto MBI) {
                            constexpr int mb = decltype(MBI)::value;
                            acc[mb][nb] = mx_mfma<kh * 2 + nb, kh * 2 + mb>(bq[u][nb][kh], aq[u][mb][kh], acc[mb][nb], sbv[u], sav[u]);
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
        const int np = (int)blockIdx.x * npw + npi;
        v4f sum = red[npi * ks][f][lane];
        for (int j = 1; j < ks; j++) sum += red[npi * ks + j][f][lane];
        const int m = mb * 16 + li;
        const int n = np * 32 + nb * 16 + lg * 4;
        if (np < n_pairs && m < p.M) store_mx4(p, STORE, (size_t)m * (size_t)p.N + (size_t)n, sum);
    }
}

template <int MR, int NR, int STORE>
hipError_t launch_tiled(const MxParams& p, hipStream_t stream) {
    constexpr int TM = 16 * MR, TN = 64 * NR;
    const int tiles_m = (p.M + TM - 1) / TM, tiles_n = (p.N + TN - 1) / TN;
    hipLaunchKernelGGL((k_mxfp4_tiled<MR, NR, STORE>), dim3(tiles_m * tiles_n), dim3(256), 0, stream, p);
    return hipGetLastError();
}

template <int MB, int STORE>
hipError_t launch_smallm(const MxParams& p, hipStream_t stream) {
    const int npw = NW / p.ksplit;
    const int n_pairs = p.N / 32;
    hipLaunchKernelGGL((k_mxfp4_smallm<MB, STORE>), dim3((n_pairs + npw - 1) / npw), dim3(NW * 64), 0, stream, p);
    return hipGetLastError();
}

}  // namespace

// tile_m x tile_n in {256x256, 128x256, 64x256, 32x256, 64x128, 32x128}
hipError_t psg_launch_mxfp4_tiled(const MxParams& p, int store, int tile_m, int tile_n, hipStream_t stream) {
#define PSG_CASE(MR_, NR_)                                                                         \
    if (tile_m == 16 * MR_ && tile_n == 64 * NR_)                                                  \
        return store == STORE_ACC ? launch_tiled<MR_, NR_, STORE_ACC>(p, stream) : launch_tiled<MR_, NR_, STORE_C>(p, stream);
    PSG_CASE(16, 4)
    PSG_CASE(8, 4)
    PSG_CASE(4, 4)
    PSG_CASE(2, 4)
    PSG_CASE(4, 2)
    PSG_CASE(2, 2)
#undef PSG_CASE
    return hipErrorInvalidConfiguration;
}

// requires 1 <= M <= 32 and p.ksplit in {1,2,4,8}
hipError_t psg_launch_mxfp4_smallm(const MxParams& p, int store, hipStream_t stream) {
    if (p.M <= 16) return store == STORE_ACC ? launch_smallm<1, STORE_ACC>(p, stream) : launch_smallm<1, STORE_C>(p, stream);
    return store == STORE_ACC ? launch_smallm<2, STORE_ACC>(p, stream) : launch_smallm<2, STORE_C>(p, stream);
}
