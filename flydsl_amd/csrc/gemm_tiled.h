// Compute-bound mainloop of the preshuffle GEMM for gfx950: int8, OCP fp8, MXFP4 and fp16/bf16 operands.
//
//   C[M,N] = A[M,K] * W[N,K]^T, W preshuffled into 1 KB fragment blocks [N/16][K/64][klane 4][nlane 16][16 B].
//
// One workgroup = 4 wavefronts arranged WM x WN (1x4: side by side along N, or 2x2); each wavefront owns MR x NR
// MFMA blocks, so the tile is (16*MR*WM) x (16*NR*WN) x 128 bytes of K.  The 1x4 layout reads every W fragment
// from memory once but makes every wavefront read the whole A tile from LDS; the 2x2 layout halves the LDS reads
// and loads every W fragment twice (the second time from L1).
//   * A tile: global -> VGPR -> LDS (XOR-swizzled 128-byte rows), double buffered, read back as
//     MFMA fragments with ds_read_b128.
//   * B fragments: each wave loads its own 1 KB blocks straight from global memory into the MFMA
//     operand registers (lane l reads bytes [16l, 16l+16) of a block: one fully coalesced 1 KB load).
//   * MFMA: operands are swapped (B fragment = src0, A fragment = src1) so that a lane ends up with
//     four CONSECUTIVE N columns of one M row: the epilogue stores 8 bytes per lane per fragment.
//       fp8 : v_mfma_f32_16x16x128_f8f6f4 (unscaled form), 32 bytes of K per lane, taken as
//             bytes [16g,16g+16) and [64+16g, 64+16g+16) of the 128-byte K step (g = lane/16) so that
//             each half is exactly one preshuffled block; A uses the same K order.
//       int8: two v_mfma_i32_16x16x64_i8 per K step (one per 64-byte half), int32 accumulate (exact).
//       fp16/bf16: 2-byte elements are preshuffled as [N/16][K/32][4][16][8 elements], i.e. again 1 KB blocks of
//             16 rows x 64 bytes; two v_mfma_f32_16x16x32_{f16,bf16} per 128-byte K step (64 elements), no scales.
//       mxfp4: K is packed two elements per byte, so a 128-byte K step is 256 elements = one chunk of the
//             shuffled e8m0 scale layout; two v_mfma_scale_f32_16x16x128_f8f6f4 per step (one per 64-byte
//             half = one preshuffled block), each lane's 16 bytes are 32 consecutive K elements sharing one
//             scale byte, selected from the lane's scale dword with op_sel (byte = 2*half + 16-row half).
//       mxfp8: e4m3fn x e4m3fn with one e8m0 scale per 32 K elements: the data path of fp8 (one 16x16x128 MFMA per
//             128-byte step, both 64-byte halves), the scale path of mxfp4 with two K steps per 256-element scale
//             chunk (op_sel byte = 2*(step parity) + 16-row half; a lane's scale applies to elements [32g, 32g+32)
//             while its data are [16g, 16g+16) and [64+16g, 64+16g+16): the hardware pairs them up by K index).
//   * Workgroup ids are remapped so that the ids the hardware deals to one XCD cover a compact
//     group_m x tiles_n patch of tiles (A and B panels stay in that XCD's L2).
#pragma once
#include "psg_common.h"
#include "tile_order.h"

namespace {

constexpr int TK = 128;  // bytes of K per mainloop step

template <int KIND>
struct Acc {
    using type = v4f;
};
template <>
struct Acc<KIND_INT8> {
    using type = v4i;
};

// MFMA through inline assembly with the accumulator constrained to the AGPR file ("+a").  With the builtin
// the register allocator is free to place accumulators in either file; at 256 accumulator registers per lane
// it then shuffles them between the files inside the main loop.  The accumulator of each call is both vDst
// and SrcC (in-place accumulate); the compiler does not know these are MFMAs, so the kernel itself provides the
// wait states between the last MFMA of a K step and anything else that may read an accumulator.
__device__ __forceinline__ void mfma_f8(v4f& c, const v8i& a, const v8i& b) {
    asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma_i8(v4i& c, const v4i& a, const v4i& b) {
    asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma_bf16(v4f& c, const v4i& a, const v4i& b) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma_f16(v4f& c, const v4i& a, const v4i& b) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}
// fp4 x fp4 with per-lane e8m0 scales: scale byte of src0 = 2*HI + LO0 of dword s0, of src1 = 2*HI + LO1 of s1
template <int HI, int LO0, int LO1>
__device__ __forceinline__ void mfma_mx(v4f& c, const v4i& a, const v4i& b, int s0, int s1) {
    asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel:[%5,%6,0] op_sel_hi:[%7,%7,0] cbsz:4 blgp:4"
                 : "+a"(c)
                 : "v"(a), "v"(b), "v"(s0), "v"(s1), "n"(LO0), "n"(LO1), "n"(HI));
}

// fp8 x fp8 with per-lane e8m0 scales (MXFP8): one MFMA covers the whole 128-element step; HI = its parity in the
// 256-element scale chunk
template <int HI, int LO0, int LO1>
__device__ __forceinline__ void mfma_mx8(v4f& c, const v8i& a, const v8i& b, int s0, int s1) {
    asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel:[%5,%6,0] op_sel_hi:[%7,%7,0]"
                 : "+a"(c)
                 : "v"(a), "v"(b), "v"(s0), "v"(s1), "n"(LO0), "n"(LO1), "n"(HI));
}

// LDS byte offset of 16-byte chunk `kc` (0..7) of row `row` inside one A stage
__device__ __forceinline__ int lds_off(int row, int kc) { return row * TK + ((kc ^ ((row >> 1) & 7)) << 4); }

__device__ __forceinline__ void tile_coords(int id, int tiles_m, int tiles_n, int group_m, int& tm, int& tn) {
    psg_tile_order(id, tiles_m, tiles_n, group_m, &tm, &tn);
}

// Two workgroups per CU are asked for where 128 + 128 registers per lane suffice; the 128x256 tile of the MX kinds
// (scale dwords on top of the operands) does not fit that and is left to the register allocator (it spilled 172 bytes per
// lane into the K loop when forced: MXFP4 4096x7168x2048 82 us).
// STORE: STORE_ACC dumps raw accumulators; STORE_C writes bf16 with no bias/activation (the common case, kept
// free of run-time epilogue switches); STORE_C_GENERIC handles fp16 output and the fused bias/activation variants.
// OCC > 0 overrides that rule: the 128x256 tile of the 8- and 16-bit kinds spills 20-50 bytes per lane when held to two
// workgroups per CU, which only pays when there are more tiles than CUs (fp8 8192x4096x4096: 127 us against 150 with one
// workgroup per CU); with at most one tile per CU the unconstrained build is faster (int8 1024x8192x8192: 68 us against
// 106, fp8 67 against 76), so the launcher picks per problem.
// PFW = K steps the W fragments are fetched ahead of their MFMAs (PFW + 1 register sets).  1 for problems that fill the GPU
// (the MFMAs of a step hide one memory latency).  3 for the few-tile / split-K regime, where a workgroup's MFMAs take no time
// and the launch is bound by the bytes of W in flight: one 128x128 tile per CU with one step ahead keeps 16 KB per CU on
// its way, far from what HBM needs (fp8 M=128, N=K=8192: 27 us for a 67 MB weight).
template <int KIND, int MR, int NR, int WM, int STORE, int WAVES = 4, int OCC = 0, int PFW = 1>
__global__ void __launch_bounds__(WAVES * 64, (OCC > 0 ? OCC : (WAVES == 4 && MR * NR <= 32 && !((KIND == KIND_MXFP4 || KIND == KIND_MXFP8) && MR * NR == 32) ? 2 : 1)))
k_a8w8_tiled(A8W8Params p) {
    using acc_t = typename Acc<KIND>::type;
    constexpr int WN = WAVES / WM;
    constexpr int TM = 16 * MR * WM;
    constexpr int TN = 16 * NR * WN;
    constexpr int RPP = WAVES * 8;        // A rows one pass of the whole workgroup copies (8 threads x 16 bytes per row)
    constexpr int A_LOADS = TM / RPP;     // 16-byte chunks of the A tile per thread
    static_assert(TM % RPP == 0, "the A tile must be a whole number of copy passes");

    __shared__ __attribute__((aligned(16))) uint8_t lds[2][TM * TK];

    const int tid = threadIdx.x;
    const int wave = wave_id();
    const int wm = wave / WN, wn = wave % WN;  // this wavefront's place in the workgroup
    const int lane = tid & 63;
    const int li = lane & 15;
    const int lg = lane >> 4;

    const int tiles_m = (p.M + TM - 1) / TM;
    const int tiles_n = (p.N + TN - 1) / TN;
    int tm, tn;
    tile_coords((int)blockIdx.x, tiles_m, tiles_n, p.group_m, tm, tn);
    const int m0 = tm * TM;
    const int n0 = tn * TN;
    // K counts BYTES of one operand row from here on (two fp4 elements per byte)
    constexpr bool IS16 = KIND == KIND_FP16 || KIND == KIND_BF16;
    constexpr bool SCALED = KIND == KIND_INT8 || KIND == KIND_FP8;  // per-token x per-channel fp32 scales in the epilogue
    constexpr bool MX = KIND == KIND_MXFP4 || KIND == KIND_MXFP8;   // e8m0 scales applied by the MFMA
    const int K = KIND == KIND_MXFP4 ? (p.K >> 1) : (IS16 ? (p.K << 1) : p.K);
    const int KT = (K + TK - 1) / TK;
    // split-K: workgroup blockIdx.y of p.splits covers K steps [kt_begin, kt_end) and (STORE_ACC only) writes its
    // accumulators to slice blockIdx.y of the partials buffer
    const int kt_per = (KT + p.splits - 1) / p.splits;
    const int kt_begin = (int)blockIdx.y * kt_per;
    const int kt_end = (kt_begin + kt_per) < KT ? (kt_begin + kt_per) : KT;

    // A: this tile's rows; rows >= M read as zero through the descriptor bound
    const uint64_t a_rows = (uint64_t)(p.M - m0);
    __amdgpu_buffer_rsrc_t ra = make_rsrc(p.a + (uint64_t)m0 * K, a_rows * (uint64_t)K);
    // B: this wave's NR n-blocks; blocks >= N/16 read as zero
    const int nb0 = (n0 >> 4) + wn * NR;
    const uint64_t b_off = (uint64_t)nb0 * 16ull * (uint64_t)K;
    const uint64_t b_total = (uint64_t)p.N * (uint64_t)K;
    __amdgpu_buffer_rsrc_t rb = make_rsrc(p.b + (b_off < b_total ? b_off : b_total), b_off < b_total ? b_total - b_off : 0);

    // MXFP4 scales: 256 bytes per (32-row chunk, 256-K chunk); this tile's / this wave's chunks; chunks past the
    // end read as zero (scale byte 0 = 2^-127, multiplied by operands that are zero too)
    constexpr int MP = MR / 2 > 0 ? MR / 2 : 1, NP = NR / 2 > 0 ? NR / 2 : 1;
    __amdgpu_buffer_rsrc_t rsa = ra, rsb = ra;
    uint32_t chunk_bytes = 0;
    if constexpr (MX) {
        static_assert(!MX || (MR % 2 == 0 && NR % 2 == 0), "scale chunks cover 32 rows");
        // one 256-byte block of scale dwords per 256 K elements: every K step for mxfp4, every second one for mxfp8
        chunk_bytes = KIND == KIND_MXFP4 ? (uint32_t)KT * 256u : (uint32_t)(p.K >> 8) * 256u;
        const uint64_t sa_chunks = (uint64_t)((p.M + 31) >> 5), sa_first = (uint64_t)((m0 >> 5) + wm * MP);
        rsa = make_rsrc(p.mx_sa + (sa_first < sa_chunks ? sa_first : sa_chunks) * chunk_bytes,
                        sa_first < sa_chunks ? (sa_chunks - sa_first) * chunk_bytes : 0);
        const uint64_t sb_chunks = (uint64_t)(p.N >> 5), sb_first = (uint64_t)((n0 >> 5) + wn * NP);
        rsb = make_rsrc(p.mx_sb + (sb_first < sb_chunks ? sb_first : sb_chunks) * chunk_bytes,
                        sb_first < sb_chunks ? (sb_chunks - sb_first) * chunk_bytes : 0);
    }
    int sav[2][MP], sbv[2][NP];

    // per-thread A copy geometry: chunk c = tid + 256*j -> (row = c/8, kc = c%8)
    const int a_row0 = tid >> 3;
    const int a_kc = tid & 7;
    const uint32_t a_goff0 = (uint32_t)a_row0 * (uint32_t)K + (uint32_t)a_kc * 16u;

    acc_t acc[MR][NR];
#pragma unroll
    for (int mi = 0; mi < MR; mi++)
#pragma unroll
        for (int ni = 0; ni < NR; ni++) acc[mi][ni] = (acc_t){0, 0, 0, 0};

    // Register sets: areg holds the A tile of the next K step on its way to LDS (each register is written to
    // LDS and immediately reloaded for the step after); blo/bhi[q] hold the W fragments of the steps with kt % NB == q.
    constexpr int NB = PFW + 1;
    static_assert(NB == 2 || (NB == 4 && !MX), "W register sets: 2, or 4 for the kinds without MX scale dwords");
    // With four W sets the A tile is fetched just as far ahead (loads return in order: a wait for A of the next step would
    // otherwise also wait for every W fragment requested before it): four A register sets, A(j) in set j % 4, loaded five
    // steps before its MFMAs and written to LDS one step before them.
    constexpr int NA = NB == 4 ? 4 : 1;
    v4i areg[NA][A_LOADS];
    v4i blo[NB][NR], bhi[NB][NR];

    // Loads never sit under control flow: a K step past the end (prefetch of the last iterations) and an A
    // chunk past K (only when K % 128 == 64) are redirected past the descriptor bound, where the hardware
    // returns zero without touching memory.  Selecting on the ADDRESS keeps the loaded registers untouched
    // until they are used, so no wait is forced early.
    auto load_a1 = [&](int kt, int j, v4i& dst) {
        const uint32_t k0 = (uint32_t)kt * TK;
        const bool in_k = kt < kt_end && (k0 + (uint32_t)a_kc * 16u) < (uint32_t)K;
        const uint32_t off = a_goff0 + (uint32_t)j * (uint32_t)RPP * (uint32_t)K + k0;
        dst = buf_load16(ra, in_k ? off : 0xFFFFFFF0u, 0);
    };
    auto store_a1 = [&](int stage, int j, const v4i& src) {
        *reinterpret_cast<v4i*>(&lds[stage][lds_off(a_row0 + RPP * j, a_kc)]) = src;
    };
    // W fragment load number idx of a K step: n-block idx/2, 64-byte half idx%2.  The n-block select sits in
    // the bounds-checked VGPR offset (blocks >= N/16 read as zero), the K position in the scalar offset.
    // MXFP4: load number 2*NR + q fetches scale dword q of the step (A-side chunks first, then W-side)
    auto load_sc1 = [&](int kt, int q, int* sa_dst, int* sb_dst) {
        const bool has = kt < kt_end;
        const uint32_t soff = has ? (uint32_t)(KIND == KIND_MXFP8 ? (kt >> 1) : kt) * 256u : 0u;
        if (q < MP) {
            sa_dst[q] = buf_load4(rsa, has ? (uint32_t)q * chunk_bytes + (uint32_t)lane * 4u : 0xFFFFFFF0u, soff);
        } else {
            sb_dst[q - MP] = buf_load4(rsb, has ? (uint32_t)(q - MP) * chunk_bytes + (uint32_t)lane * 4u : 0xFFFFFFF0u, soff);
        }
    };
    // W addressing.  Preshuffled: lane l reads bytes [16l, 16l+16) of the 1 KB block (n-block, 64-byte K block).
    // Row-major [N,K] (the row-scale fp8 GEMM's plain-B call shape): the same fragment is 16 rows x 64 bytes, lane
    // (row li, 16-byte K group lg) reads row li of the n-block at K offset 16*lg; 16 segments of 64 bytes per load
    // instead of one contiguous KB.  Either way an n-block of 16 rows is 16*K bytes, so the descriptor is the same.
    const uint32_t b_lane_off = p.b_rowmajor ? (uint32_t)li * (uint32_t)K + (uint32_t)lg * 16u : (uint32_t)lane * 16u;
    const uint32_t b_step = p.b_rowmajor ? 128u : 2048u, b_half = p.b_rowmajor ? 64u : 1024u;
    auto load_b1 = [&](int kt, int idx, v4i* lo, v4i* hi) {
        const int ni = idx >> 1;
        const bool has = kt < kt_end && (kt * TK + (idx & 1) * 64) < K;
        const uint32_t voff = b_lane_off + (uint32_t)ni * 16u * (uint32_t)K;
        const v4i v = buf_load16(rb, has ? voff : 0xFFFFFFF0u, has ? (uint32_t)kt * b_step + (uint32_t)(idx & 1) * b_half : 0u);
        if (idx & 1) hi[ni] = v; else lo[ni] = v;
    };
    auto read_frag = [&](int stage, int mi, v4i& flo, v4i& fhi) {
        const int row = (wm * MR + mi) * 16 + li;
        flo = *reinterpret_cast<const v4i*>(&lds[stage][lds_off(row, lg)]);
        fhi = *reinterpret_cast<const v4i*>(&lds[stage][lds_off(row, 4 + lg)]);
    };

    // One K step (tile kt, parity S): MFMAs on LDS stage S and W set S, with the memory work of the next
    // steps dealt out between the m-blocks so that no instruction queue (texture addresser, LDS) ever holds
    // up MFMA issue:
    //   first half of the m-blocks : the W fragment loads of step kt+1 -> W set S^1
    //   second half                : A tile of step kt+1 (in registers, loaded one step ago) -> LDS stage S^1,
    //                                each register reloaded at once with its part of the A tile of step kt+2
    //   every m-block              : LDS read of the next m-block's A fragment (register double buffer)
    auto step = [&](int kt, auto SP) {
        constexpr int SB = decltype(SP)::value;  // W register set of this step
        constexpr int S = SB & 1;                // LDS stage (and MX scale set) of this step
        constexpr int SN = (SB + PFW) % NB;      // W register set the loads of this step fill
        constexpr int HALF = MR / 2;
        constexpr int N_LOADS = 2 * NR + (MX ? MP + NP : 0);  // W fragments (+ scale dwords)
        constexpr int B_PER = (N_LOADS + HALF - 1) / HALF;
        // A fragments are read FRAG_AHEAD m-blocks ahead of the MFMAs that use them (register ring buffer)
        // (one block ahead for the int8 128x256 tile held to two workgroups per CU: with two the build spilled 48 bytes per
        // lane, int8 5120x2048x8320 123 us against 95; the fp8 build of the same tile is the other way round)
        constexpr int FRAG_AHEAD = (MR >= 4 && !(KIND == KIND_INT8 && WAVES == 4 && MR * NR == 32 && OCC == 0)) ? 2 : 1;
        constexpr int FRAG_BUFS = FRAG_AHEAD + 1;
        v4i flo[FRAG_BUFS], fhi[FRAG_BUFS];
        static_for<FRAG_AHEAD>([&](auto I) {
            constexpr int i = decltype(I)::value;
            if constexpr (i < MR) read_frag(S, i, flo[i % FRAG_BUFS], fhi[i % FRAG_BUFS]);
        });
        static_for<MR>([&](auto MI) {
            constexpr int mi = decltype(MI)::value;
            if constexpr (mi + FRAG_AHEAD < MR)
                read_frag(S, mi + FRAG_AHEAD, flo[(mi + FRAG_AHEAD) % FRAG_BUFS], fhi[(mi + FRAG_AHEAD) % FRAG_BUFS]);
            if constexpr (mi < HALF) {
                static_for<B_PER>([&](auto Q) {
                    constexpr int idx = mi * B_PER + decltype(Q)::value;
                    if constexpr (idx < 2 * NR) load_b1(kt + PFW, idx, blo[SN], bhi[SN]);
                    else if constexpr (idx < N_LOADS) load_sc1(kt + 1, idx - 2 * NR, sav[S ^ 1], sbv[S ^ 1]);
                });
            } else {
                constexpr int A_PER = (A_LOADS + (MR - HALF) - 1) / (MR - HALF);
                static_for<A_PER>([&](auto Q) {
                    constexpr int j = (mi - HALF) * A_PER + decltype(Q)::value;
                    if constexpr (j < A_LOADS) {
                        constexpr int AS = NA == 4 ? (SB + 1) % 4 : 0;  // set of A(kt + 1)
                        store_a1(S ^ 1, j, areg[AS][j]);
                        load_a1(kt + (NA == 4 ? 5 : 2), j, areg[AS][j]);
                    }
                });
            }
            // keep the memory instructions above ahead of this block's MFMAs (the machine scheduler would
            // otherwise cluster them at the top of the step)
            __builtin_amdgcn_sched_barrier(0);
            const v4i alo = flo[mi % FRAG_BUFS], ahi = fhi[mi % FRAG_BUFS];
            if constexpr (KIND == KIND_INT8) {
#pragma unroll
                for (int ni = 0; ni < NR; ni++) mfma_i8(acc[mi][ni], blo[SB][ni], alo);
#pragma unroll
                for (int ni = 0; ni < NR; ni++) mfma_i8(acc[mi][ni], bhi[SB][ni], ahi);
            } else if constexpr (IS16) {
#pragma unroll
                for (int ni = 0; ni < NR; ni++) {
                    if constexpr (KIND == KIND_BF16) mfma_bf16(acc[mi][ni], blo[SB][ni], alo); else mfma_f16(acc[mi][ni], blo[SB][ni], alo);
                }
#pragma unroll
                for (int ni = 0; ni < NR; ni++) {
                    if constexpr (KIND == KIND_BF16) mfma_bf16(acc[mi][ni], bhi[SB][ni], ahi); else mfma_f16(acc[mi][ni], bhi[SB][ni], ahi);
                }
            } else if constexpr (KIND == KIND_MXFP4) {
                static_for<NR>([&](auto NI) {
                    constexpr int ni = decltype(NI)::value;
                    mfma_mx<0, ni & 1, mi & 1>(acc[mi][ni], blo[SB][ni], alo, sbv[S][ni / 2], sav[S][mi / 2]);
                });
                static_for<NR>([&](auto NI) {
                    constexpr int ni = decltype(NI)::value;
                    mfma_mx<1, ni & 1, mi & 1>(acc[mi][ni], bhi[SB][ni], ahi, sbv[S][ni / 2], sav[S][mi / 2]);
                });
            } else if constexpr (KIND == KIND_MXFP8) {
                // step parity S = 128-element half of the scale chunk: K ranges start at even steps (no split-K here)
                const v8i af = {alo[0], alo[1], alo[2], alo[3], ahi[0], ahi[1], ahi[2], ahi[3]};
                static_for<NR>([&](auto NI) {
                    constexpr int ni = decltype(NI)::value;
                    const v8i bf = {blo[SB][ni][0], blo[SB][ni][1], blo[SB][ni][2], blo[SB][ni][3],
                                    bhi[SB][ni][0], bhi[SB][ni][1], bhi[SB][ni][2], bhi[SB][ni][3]};
                    mfma_mx8<S, ni & 1, mi & 1>(acc[mi][ni], bf, af, sbv[S][ni / 2], sav[S][mi / 2]);
                });
            } else {
                const v8i af = {alo[0], alo[1], alo[2], alo[3], ahi[0], ahi[1], ahi[2], ahi[3]};
#pragma unroll
                for (int ni = 0; ni < NR; ni++) {
                    const v8i bf = {blo[SB][ni][0], blo[SB][ni][1], blo[SB][ni][2], blo[SB][ni][3],
                                    bhi[SB][ni][0], bhi[SB][ni][1], bhi[SB][ni][2], bhi[SB][ni][3]};
                    mfma_f8(acc[mi][ni], bf, af);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        // The compiler does not know that the asm statements above are MFMAs, so it inserts none of the wait
        // states a non-MFMA read of an accumulator needs after the last MFMA that wrote it (11 for an 8-pass
        // MFMA).  Nothing inside the loop reads accumulators, but the code after the loop does, and the compiler may
        // place such a read (even a plain register copy) first thing after the loop.  Wait states directly behind
        // the last MFMA of every step cover that: volatile asm statements keep their order, and code after the
        // loop cannot move up across the barrier below.
        asm volatile("s_nop 15" ::: "memory");
        __syncthreads();
    };

    // prologue: A(0) -> LDS stage 0, A(1) -> registers, W(0) -> set 0
#pragma unroll
    for (int j = 0; j < A_LOADS; j++) load_a1(kt_begin, j, areg[0][j]);
    static_for<PFW>([&](auto I) {
        constexpr int i = decltype(I)::value;
#pragma unroll
        for (int idx = 0; idx < 2 * NR; idx++) load_b1(kt_begin + i, idx, blo[i], bhi[i]);
        if constexpr (NA == 4) {
#pragma unroll
            for (int j = 0; j < A_LOADS; j++) load_a1(kt_begin + 1 + i, j, areg[1 + i][j]);
        }
    });
    if constexpr (MX) {
#pragma unroll
        for (int q = 0; q < MP + NP; q++) load_sc1(kt_begin, q, sav[0], sbv[0]);
    }
#pragma unroll
    for (int j = 0; j < A_LOADS; j++) {
        store_a1(0, j, areg[0][j]);
        if constexpr (NA == 4) {
            load_a1(kt_begin + 4, j, areg[0][j]);
        } else {
            load_a1(kt_begin + 1, j, areg[0][j]);
        }
    }
    __syncthreads();

    // Two K steps per iteration (LDS / register ping-pong).  When the step count is odd the last "odd" step
    // multiplies zero operands (its loads were redirected past the bounds): harmless, and the loop body stays
    // free of control flow, which the software pipeline needs.
    if constexpr (NB == 2) {
        for (int kt = kt_begin; kt < kt_end; kt += 2) {
            step(kt, std::integral_constant<int, 0>{});
            step(kt + 1, std::integral_constant<int, 1>{});
        }
    } else {
        // four register sets: steps past the end are skipped (the condition is uniform over the workgroup) instead of run on
        // zero operands; with 16 steps per workgroup three idle steps would be a fifth of the loop
        for (int kt = kt_begin; kt < kt_end; kt += 4) {
            step(kt, std::integral_constant<int, 0>{});
            if (kt + 1 < kt_end) step(kt + 1, std::integral_constant<int, 1>{});
            if (kt + 2 < kt_end) step(kt + 2, std::integral_constant<int, 2>{});
            if (kt + 3 < kt_end) step(kt + 3, std::integral_constant<int, 3>{});
        }
    }

    // epilogue operands, fetched in one batch (one memory latency for the whole tile, not one per fragment)
    float sa_v[MR];
    v4f sb_v[NR];
    if constexpr (STORE != STORE_ACC && SCALED) {
#pragma unroll
        for (int mi = 0; mi < MR; mi++) {
            const int m = m0 + (wm * MR + mi) * 16 + li;
            sa_v[mi] = p.sa[m < p.M ? m : p.M - 1];
        }
#pragma unroll
        for (int ni = 0; ni < NR; ni++) {
            const int n = n0 + (wn * NR + ni) * 16 + lg * 4;
            sb_v[ni] = *reinterpret_cast<const v4f*>(p.sb + (n < p.N ? n : 0));
        }
    }

    // epilogue: lane owns C[m0 + mi*16 + li][n0 + (wave*NR + ni)*16 + lg*4 + 0..3].  Compile-time indices only,
    // so the accumulators are never addressed dynamically.
    if constexpr (STORE == STORE_ACC) {
        static_for<MR>([&](auto MI) {
            constexpr int mi = decltype(MI)::value;
            const int m = m0 + (wm * MR + mi) * 16 + li;
            if (m < p.M) {
                static_for<NR>([&](auto NI) {
                    constexpr int ni = decltype(NI)::value;
                    const int n = n0 + (wn * NR + ni) * 16 + lg * 4;
                    if (n < p.N) {
                        const size_t idx = (size_t)m * (size_t)p.N + (size_t)n;
                        const size_t slice = (size_t)blockIdx.y * (size_t)p.M * (size_t)p.N;
                        *reinterpret_cast<acc_t*>(reinterpret_cast<uint8_t*>(p.c) + (slice + idx) * 4) = acc[mi][ni];
                    }
                });
            }
        });
    } else {
        // 16-bit C goes through LDS (free after the loop's last barrier) so that every store instruction writes
        // whole rows of the tile: a lane's own fragment is 8 bytes wide and a wavefront's store of it touches 16
        // rows x 32 bytes, which reaches 3.6 TB/s of HBM writes; rows of 128 bytes and more reach 5.7 TB/s (measured
        // with store-only kernels over 64 MiB).  The tile is written in passes of CH_ROWS rows (what the A stages
        // hold); 16-byte granules are XOR-swizzled by the row so that neither side has LDS bank conflicts.
        constexpr int ROWB = TN * 2;                      // bytes of one tile row of C
        constexpr int GR = ROWB / 16;                     // 16-byte granules per row
        constexpr int XM = (GR < 16 ? GR : 16) - 1;
        constexpr int CH_FIT = (2 * TM * TK) / ROWB;      // rows the LDS array holds
        constexpr int CH_ROWS = CH_FIT < TM ? CH_FIT : TM;
        constexpr int NCH = TM / CH_ROWS;
        constexpr int CH_BLK = CH_ROWS / 16;              // 16-row blocks per pass
        constexpr int NT = WAVES * 64;
        static_assert(CH_ROWS % 16 == 0 && TM % CH_ROWS == 0 && (CH_ROWS * GR) % NT == 0, "epilogue passes must tile the C tile");
        uint8_t* stage = &lds[0][0];
        static_for<NCH>([&](auto CI) {
            constexpr int ci = decltype(CI)::value;
            static_for<MR>([&](auto MI) {
                constexpr int mi = decltype(MI)::value;
                const int blk = wm * MR + mi;             // 16-row block of the tile (uniform over the wavefront)
                if (blk / CH_BLK == ci) {
                    const int rl = (blk - ci * CH_BLK) * 16 + li;  // row within the pass
                    float sa = 0.f;
                    if constexpr (SCALED) sa = sa_v[mi];
                    static_for<NR>([&](auto NI) {
                        constexpr int ni = decltype(NI)::value;
                        const int n = n0 + (wn * NR + ni) * 16 + lg * 4;
                        if (n < p.N) {
                            const acc_t r = acc[mi][ni];
                            v4f x;
                            if constexpr (!SCALED) {
                                x = (v4f){(float)r[0], (float)r[1], (float)r[2], (float)r[3]};  // no epilogue scales (MX: applied by the MFMA)
                            } else {
                                const v4f sb = sb_v[ni];
                                x = (v4f){((float)r[0] * sa) * sb[0], ((float)r[1] * sa) * sb[1], ((float)r[2] * sa) * sb[2],
                                          ((float)r[3] * sa) * sb[3]};
                            }
                            v2i out;
                            if constexpr (STORE == STORE_C) {
                                out = finish4<OUT_BF16, EPI_NONE>(x, nullptr);
                            } else {
                                out = p.out == OUT_BF16 ? finish4_rt<OUT_BF16>(x, p.bias + n, p.epi) : finish4_rt<OUT_FP16>(x, p.bias + n, p.epi);
                            }
                            const int g = (wn * NR + ni) * 2 + (lg >> 1);
                            *reinterpret_cast<v2i*>(stage + rl * ROWB + ((g ^ (rl & XM)) << 4) + (lg & 1) * 8) = out;
                        }
                    });
                }
            });
            __syncthreads();
#pragma unroll
            for (int q0 = 0; q0 < CH_ROWS * GR; q0 += NT) {
                const int q = q0 + tid, rl = q / GR, g = q % GR;
                const int m = m0 + ci * CH_ROWS + rl, n = n0 + g * 8;
                if (m < p.M && n < p.N) {
                    const v4i v = *reinterpret_cast<const v4i*>(stage + rl * ROWB + ((g ^ (rl & XM)) << 4));
                    *reinterpret_cast<v4i*>(reinterpret_cast<uint16_t*>(p.c) + (size_t)m * (size_t)p.N + (size_t)n) = v;
                }
            }
            if constexpr (ci + 1 < NCH) __syncthreads();
        });
    }
}

template <int KIND, int MR, int NR, int WM, int STORE, int WAVES = 4, int OCC = 0, int PFW = 1>
hipError_t launch_one(const A8W8Params& p, hipStream_t stream) {
    constexpr int TM = 16 * MR * WM, TN = 16 * NR * (WAVES / WM);
    const int tiles_m = (p.M + TM - 1) / TM, tiles_n = (p.N + TN - 1) / TN;
    const int splits = STORE == STORE_ACC && p.splits > 1 ? p.splits : 1;
    A8W8Params q = p;
    q.splits = splits;
    hipLaunchKernelGGL((k_a8w8_tiled<KIND, MR, NR, WM, STORE, WAVES, OCC, PFW>), dim3(tiles_m * tiles_n, splits), dim3(WAVES * 64), 0, stream, q);
    return hipGetLastError();
}

// the 256x256 tile of eight wavefronts has a kernel of its own (gemm_tiled8.h, which includes this file)
template <int KIND, int STORE>
hipError_t launch_tiled8(const A8W8Params& p, hipStream_t stream);
template <int KIND, int STORE>
hipError_t launch_tiled_deep(const A8W8Params& p, hipStream_t stream);

// p.wave_layout selects the wavefront layout of the 256x256 tile: 2 = 2x2 wavefronts, 8 = eight wavefronts along N, anything
// else = 1x4
template <int KIND, int STORE>
hipError_t launch_shape(const A8W8Params& p, int tile_m, int tile_n, hipStream_t stream) {
#define PSG_CASE(MR_, NR_, WM_) \
    if (tile_m == 16 * MR_ * WM_ && tile_n == 16 * NR_ * (4 / WM_)) return launch_one<KIND, MR_, NR_, WM_, STORE>(p, stream);
    if (p.wave_layout == 2) {
        PSG_CASE(8, 8, 2)
    }
    if (p.wave_layout == 8) {  // eight wavefronts side by side along N: 256x256 tile, every W fragment loaded once
        if (tile_m == 256 && tile_n == 256) return launch_tiled8<KIND, STORE>(p, stream);
    }
    if constexpr (KIND != KIND_MXFP4 && KIND != KIND_MXFP8) {
        // few tiles (p.ksplit = 3: the planner's mark for launches of at most two workgroups per CU): W fetched three steps ahead
        if (p.ksplit == 3) {
            // 128x128 with a deep ring of stages (gemm_tiled8.h); wave_layout 4 keeps the older build with W three steps ahead
            if (tile_m == 128 && tile_n == 128) {
                // one workgroup per CU at most (its LDS ring fills the CU), and only above 256 rows (measured: no gain below);
                // everything else keeps the register-ring build
                const long wgs = (long)((p.M + 127) / 128) * (long)((p.N + 127) / 128) * (STORE == STORE_ACC && p.splits > 1 ? p.splits : 1);
                return p.wave_layout == 4 || wgs > psg_cu_count() || p.M <= 256 ? launch_one<KIND, 8, 2, 1, STORE, 4, 1, 3>(p, stream) : launch_tiled_deep<KIND, STORE>(p, stream);
            }
            if (tile_m == 64 && tile_n == 64) return launch_one<KIND, 4, 1, 1, STORE, 4, 0, 3>(p, stream);
        }
    }
    PSG_CASE(16, 4, 1)
    PSG_CASE(8, 8, 1)
    if constexpr (KIND != KIND_MXFP4 && KIND != KIND_MXFP8) {
        // 128x256 with at most one tile per CU: the build that is not held to two workgroups per CU
        if (tile_m == 128 && tile_n == 256) {
            const long tiles = (long)((p.M + 127) / 128) * (long)((p.N + 255) / 256) * (STORE == STORE_ACC && p.splits > 1 ? p.splits : 1);
            if (tiles <= 256) return launch_one<KIND, 8, 4, 1, STORE, 4, 1>(p, stream);
        }
    }
    PSG_CASE(8, 4, 1)
    PSG_CASE(4, 4, 1)
    PSG_CASE(2, 4, 1)
    if constexpr (KIND == KIND_MXFP4 || KIND == KIND_MXFP8) {
        PSG_CASE(4, 2, 1)
        PSG_CASE(2, 2, 1)
    } else {
        PSG_CASE(8, 2, 1)
        PSG_CASE(4, 1, 1)
    }
#undef PSG_CASE
    return hipErrorInvalidConfiguration;
}

}  // namespace
