// Tiles of the compute-bound mainloop whose A operand travels global -> LDS by DMA (gfx950): the 256x256 tile of eight
// wavefronts side by side along N, and a 128x128 tile of four wavefronts with a deep ring of stages for launches with few
// tiles and a long K.
//
// Same operand paths as gemm_tiled.h (W fragments straight from memory into MFMA operand registers, every fragment read
// from memory once per workgroup; the A tile shared through LDS and read by all eight wavefronts), with a different way
// of moving A and of synchronising:
//   * A goes global -> LDS by DMA (buffer_load_dwordx4 ... lds): no staging registers, no ds_write.  A DMA instruction
//     writes 64 x 16 bytes to consecutive LDS addresses (M0 + 16*lane), i.e. eight 128-byte rows of the stage, so the XOR
//     swizzle of the 16-byte chunks is applied to the SOURCE address of each lane (lane l of a 1 KB block fills physical
//     chunk l%8 of row l/8 and therefore fetches logical chunk (l%8) ^ ((row/2)%8) of that row).  Lanes redirected past
//     the descriptor bound (rows >= M, K tail, steps past the end) write zeros.
//   * NS LDS stages (four of 32 KB for the 256-row tile): the A tile of step kt+NS-1 is requested during step kt, is waited
//     for (vmcnt, by the wavefront that requested it) before the barrier that ends step kt+NS-3, and is therefore complete
//     for everybody one whole step before its MFMAs.  That lets every wavefront read the first A fragments of step kt+1 BEFORE the barrier
//     that ends step kt, so the MFMAs continue right behind the barrier instead of waiting for LDS.  The one barrier per
//     step that is left only keeps a stage from being overwritten while a slower wavefront still reads it.
//   * The DMA is issued from inline assembly: the compiler does not know that it writes LDS (it would otherwise put a
//     full vmcnt wait in front of every LDS read that follows), so the kernel does that bookkeeping itself.  Loads
//     return in order, and the compiler counts only the W loads it knows about, so within a step the DMAs are issued
//     before the W loads and only behind the first MFMAs (where the compiler waits for this step's W fragments): a
//     compiler-made vmcnt then never covers a DMA that was issued a moment ago.
//   * MX scale dwords take the same road (4-byte DMAs into a slot per stage, read back one step ahead): as register
//     loads the compiler had to wait for all of them, i.e. for every load in flight, at the top of every step.
//   * Every descriptor an instruction of the loop uses is built from values forced into scalar registers
//     (make_rsrc_uniform): left to the compiler, the W descriptor of some builds lived in vector registers and every W load
//     paid four v_readfirstlane (350 core cycles per fp8 K step).
//   * In steady state no load is predicated: the selects and compares that redirect loads past the K range run only in
//     the last steps (a second copy of the loop), not in front of the MFMAs of every step.
//   * C leaves through LDS as whole rows, in two halves: the stores of rows 0..127 are under way while rows 128..255 are
//     converted.  Epilogue scales wait in LDS since the prologue.
#pragma once
#include "gemm_tiled.h"

namespace {

// descriptor built from values forced into scalar registers (an inline-asm "s" operand must not end up in vector registers)
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc_uniform(const void* base, uint64_t bytes) {
    const uint64_t b = (uint64_t)(uintptr_t)base;
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32));
    const uint32_t n = (uint32_t)__builtin_amdgcn_readfirstlane((int)(bytes > 0xFFFFFFFFull ? 0xFFFFFFFFu : (uint32_t)bytes));
    return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>((uintptr_t)(((uint64_t)hi << 32) | lo)), 0, (int)n, 0x00020000);
}

// one DMA instruction: 64 lanes x 16 bytes from (descriptor, voff + soff) to LDS [lds_addr, lds_addr + 1024)
__device__ __forceinline__ void dma16(__amdgpu_buffer_rsrc_t r, uint32_t lds_addr, uint32_t voff, uint32_t soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds" ::"s"(__builtin_amdgcn_readfirstlane((int)lds_addr)), "v"(voff), "s"(r), "s"(__builtin_amdgcn_readfirstlane((int)soff))
                 : "memory");
}

// 4 bytes per lane: 64 lanes x 4 bytes to LDS [lds_addr, lds_addr + 256)
__device__ __forceinline__ void dma4(__amdgpu_buffer_rsrc_t r, uint32_t lds_addr, uint32_t voff, uint32_t soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds" ::"s"(__builtin_amdgcn_readfirstlane((int)lds_addr)), "v"(voff), "s"(r), "s"(__builtin_amdgcn_readfirstlane((int)soff))
                 : "memory");
}

// Built with -DT8_TIMING (a measuring harness, never the library) thread 0 of every workgroup records the core clock and the
// 10 ns wall clock at: 0 start, 1 loop begin, 2 loop end, 4 C staged, 5 behind the barrier, 6 stores issued, 3 stores done.
#ifdef T8_TIMING
__device__ unsigned long long* t8_dbg;
#define T8_STAMP(i) do { if (threadIdx.x == 0) { t8_dbg[blockIdx.x * 16 + 2 * (i)] = clock64(); t8_dbg[blockIdx.x * 16 + 2 * (i) + 1] = wall_clock64(); } } while (0)
#else
#define T8_STAMP(i) do { } while (0)
#endif

// Tile = (16 MR) x (32 WAVES) x 128 bytes of K: WAVES wavefronts side by side along N with two 16-column blocks each, every
// one of them multiplying all MR 16-row blocks of the A tile.  NS = LDS stages of the A tile, PFW = K steps the W fragments
// are fetched ahead of their MFMAs (PFW + 1 register sets; NS must be a multiple of that).
//   <16, 8, 4, 1>: 256x256, one workgroup per CU with two wavefronts per SIMD; for problems that fill the GPU.  (Measured on it
//       and not kept, fp8 8192x4096x4096, core cycles per K step / us per launch: the memory instructions of the two
//       wavefronts of a SIMD two m-blocks apart 2,354 / 115.5 and the same with s_setprio 1 around the MFMAs 2,425 / 115.4,
//       against 2,311 / 114.5 as built; 2,048 cycles is the issue limit of the 64 MFMAs per SIMD.  W three steps ahead, four
//       register sets: the same time, and no room left for the allocator.  A fragments read one or three m-blocks ahead
//       instead of two: the same cycles for fp8 and fp4.  The row passes of the upper half of C alternating with the
//       conversion of the lower half: fp8 104.83 against 104.82 us, MXFP4 4096x7168x2048 40.71 against 40.34.  The eight
//       A-side MX scale dwords of a step stored lane-major and read with two 16-byte reads instead of eight 4-byte reads:
//       40.43 against 40.47 us.)
//   <8, 4, 8, 7>: 128x128, one wavefront per SIMD, seven steps of A (DMA) and W (registers) on their way: for launches with
//       few tiles and a long K.  Against the build that keeps W three steps ahead in registers (fp8, N = K = 8192, split-K
//       pair, us): M=512 42.9 / 45.4, M=384 (5120x13824) 44.1 / 45.8, M=256 35.2 / 34.9, M=128 27.8 / 26.6, so the launcher takes
//       it above 256 rows only: more bytes in flight per CU is not what these launches lack.  Nor is it wavefronts per SIMD: the same
//       tile with eight wavefronts as 2 x 4 (four m-blocks each, W three steps ahead) took 53.1 against 48.3 us at M=512 and 77.6
//       against 69.2 at 384x5120x13824 (every W fragment is then loaded by two wavefronts).
template <int KIND, int STORE, int MR, int WAVES, int NS, int PFW>
__global__ void __launch_bounds__(WAVES * 64, 1) k_tiled_dma(A8W8Params p) {
    using acc_t = typename Acc<KIND>::type;
    constexpr int NR = 2;
    constexpr int TM = 16 * MR, TN = 16 * NR * WAVES;
    constexpr int NB = PFW + 1;
    constexpr int STAGE = TM * TK;                   // bytes of one A stage
    constexpr int A_DMA = STAGE / 1024 / WAVES;      // 1 KB blocks of a stage this wavefront fills
    static_assert(NS % NB == 0 && MR % 4 == 0 && A_DMA >= 1 && A_DMA % 2 == 0 && STAGE % (1024 * WAVES) == 0, "tile geometry");
    constexpr bool IS16 = KIND == KIND_FP16 || KIND == KIND_BF16;
    constexpr bool SCALED = KIND == KIND_INT8 || KIND == KIND_FP8;
    constexpr bool MX = KIND == KIND_MXFP4 || KIND == KIND_MXFP8;
    static_assert(!MX || (MR == 16 && NS == 4), "MX scale slots are laid out for the 256-row tile");

    // LDS: the A stages; behind them NS slots of MX scale dwords (per slot 8 A-side chunks + 8 W-side chunks of 256 bytes)
    // or the per-token / per-channel scales of the epilogue (TM + TN floats)
    constexpr int SC_SLOT = 4096;
    constexpr int LDS_EXTRA = MX ? NS * SC_SLOT : (TM + TN) * 4;
    __shared__ __attribute__((aligned(1024))) uint8_t lds[NS * STAGE + LDS_EXTRA];
    uint8_t* const lds_x = lds + NS * STAGE;

    T8_STAMP(0);
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
    const int K = KIND == KIND_MXFP4 ? (p.K >> 1) : (IS16 ? (p.K << 1) : p.K);  // BYTES of one operand row
    const int KT = (K + TK - 1) / TK;
    const int kt_per = (KT + p.splits - 1) / p.splits;
    const int kt_begin = (int)blockIdx.y * kt_per;
    const int kt_end = (kt_begin + kt_per) < KT ? (kt_begin + kt_per) : KT;

    const uint64_t a_rows = (uint64_t)(p.M - m0);
    __amdgpu_buffer_rsrc_t ra = make_rsrc_uniform(p.a + (uint64_t)m0 * K, a_rows * (uint64_t)K);
    const int nb0 = (n0 >> 4) + wave * NR;
    const uint64_t b_off = (uint64_t)nb0 * 16ull * (uint64_t)K;
    const uint64_t b_total = (uint64_t)p.N * (uint64_t)K;
    __amdgpu_buffer_rsrc_t rb = make_rsrc_uniform(p.b + (b_off < b_total ? b_off : b_total), b_off < b_total ? b_total - b_off : 0);

    // MX scales: per (32-row chunk, 256-element K chunk) 64 dwords, one per lane.  Wavefront w brings A-side chunk w of the
    // tile and its own W-side chunk (32 columns) into the slot of the step by two 4-byte DMAs; chunks past the end read
    // as zero (scale byte 0 = 2^-127, multiplied by operands that are zero too).
    constexpr int MP = MR / 2, NP = 1;
    __amdgpu_buffer_rsrc_t rsa = ra, rsb = ra;
    if constexpr (MX) {
        const uint32_t chunk_bytes = KIND == KIND_MXFP4 ? (uint32_t)KT * 256u : (uint32_t)(p.K >> 8) * 256u;
        const uint64_t sa_chunks = (uint64_t)((p.M + 31) >> 5), sa_mine = (uint64_t)((m0 >> 5) + wave);
        rsa = make_rsrc_uniform(p.mx_sa + (sa_mine < sa_chunks ? sa_mine : sa_chunks) * chunk_bytes, sa_mine < sa_chunks ? chunk_bytes : 0);
        const uint64_t sb_chunks = (uint64_t)(p.N >> 5), sb_mine = (uint64_t)((n0 >> 5) + wave);
        rsb = make_rsrc_uniform(p.mx_sb + (sb_mine < sb_chunks ? sb_mine : sb_chunks) * chunk_bytes, sb_mine < sb_chunks ? chunk_bytes : 0);
    }
    int sav[2][MP], sbv[2][NP];

    acc_t acc[MR][NR];
#pragma unroll
    for (int mi = 0; mi < MR; mi++)
#pragma unroll
        for (int ni = 0; ni < NR; ni++) acc[mi][ni] = (acc_t){0, 0, 0, 0};

    v4i blo[NB][NR], bhi[NB][NR];

    // A by DMA: this wavefront fills the 1 KB blocks A_DMA*wave + j (rows 8*(A_DMA*wave + j) .. + 7) of a stage
    const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
    uint32_t a_voff[A_DMA];
    int a_kc[2];  // logical 16-byte chunk this lane fetches, by the parity of the block
#pragma unroll
    for (int j = 0; j < A_DMA; j++) {
        const int row = (wave * A_DMA + j) * 8 + (lane >> 3);
        const int kc = (lane & 7) ^ ((row >> 1) & 7);
        a_voff[j] = (uint32_t)row * (uint32_t)K + (uint32_t)kc * 16u;
        a_kc[j & 1] = kc;
    }
    // CHK = false: the step is known to lie inside [kt_begin, kt_end) and not to be the K tail, so nothing is redirected (the
    // selects and compares of the checked form are ten instructions per load in front of the MFMAs of both wavefronts of a SIMD)
    auto dma_a1 = [&](int kt, int stage, int j, auto CHK) __attribute__((always_inline)) {
        const uint32_t dst = lds_base + (uint32_t)(stage * STAGE + (wave * A_DMA + j) * 1024);
        if constexpr (decltype(CHK)::value) {
            const bool in_k = kt < kt_end && (uint32_t)(kt * TK + a_kc[j & 1] * 16) < (uint32_t)K;
            dma16(ra, dst, in_k ? a_voff[j] : 0xFFFFFFF0u, kt < kt_end ? (uint32_t)kt * TK : 0u);
        } else {
            dma16(ra, dst, a_voff[j], (uint32_t)kt * TK);
        }
    };

    // scale dwords of step kt -> slot (two DMAs per wavefront), and slot -> registers
    auto dma_sc = [&](int kt, int slot, int which) __attribute__((always_inline)) {
        const bool has = kt < kt_end;
        const uint32_t dst = lds_base + (uint32_t)(NS * STAGE + slot * SC_SLOT + which * 2048 + wave * 256);
        dma4(which ? rsb : rsa, dst, has ? (uint32_t)lane * 4u : 0xFFFFFFF0u, has ? (uint32_t)(KIND == KIND_MXFP8 ? (kt >> 1) : kt) * 256u : 0u);
    };
    auto read_sc = [&](int slot, int q, int* sa_dst, int* sb_dst) __attribute__((always_inline)) {
        if (q < MP) sa_dst[q] = *reinterpret_cast<const int*>(lds_x + slot * SC_SLOT + q * 256 + lane * 4);
        else sb_dst[0] = *reinterpret_cast<const int*>(lds_x + slot * SC_SLOT + 2048 + wave * 256 + lane * 4);
    };
    const uint32_t b_lane_off = p.b_rowmajor ? (uint32_t)li * (uint32_t)K + (uint32_t)lg * 16u : (uint32_t)lane * 16u;
    const uint32_t b_step = p.b_rowmajor ? 128u : 2048u, b_half = p.b_rowmajor ? 64u : 1024u;
    auto load_b1 = [&](int kt, int idx, v4i* lo, v4i* hi, auto CHK) __attribute__((always_inline)) {
        const int ni = idx >> 1;
        const bool has = !decltype(CHK)::value || (kt < kt_end && (kt * TK + (idx & 1) * 64) < K);
        const uint32_t voff = b_lane_off + (uint32_t)ni * 16u * (uint32_t)K;
        const v4i v = buf_load16(rb, has ? voff : 0xFFFFFFF0u, has ? (uint32_t)kt * b_step + (uint32_t)(idx & 1) * b_half : 0u);
        if (idx & 1) hi[ni] = v; else lo[ni] = v;
    };
    // fragment (16 rows x 2 x 16 bytes of K) of m-block mi from a stage: row mi*16 + li, chunks lg and 4 + lg; the swizzle
    // term (row/2)%8 = (li/2)%8 does not depend on mi
    const int f_lo = li * TK + ((lg ^ ((li >> 1) & 7)) << 4);
    const int f_hi = li * TK + (((4 + lg) ^ ((li >> 1) & 7)) << 4);
    auto read_frag = [&](int stage, int mi, v4i& flo, v4i& fhi) __attribute__((always_inline)) {
        flo = *reinterpret_cast<const v4i*>(&lds[stage * STAGE + mi * 16 * TK + f_lo]);
        fhi = *reinterpret_cast<const v4i*>(&lds[stage * STAGE + mi * 16 * TK + f_hi]);
    };

    constexpr int FRAG_AHEAD = 2, FRAG_BUFS = 4;  // MR is a multiple of 4: buffer mi % 4 lines up across steps
    v4i flo[FRAG_BUFS], fhi[FRAG_BUFS];

    // One K step: MFMAs on LDS stage S and W set S % NB.  m-block 0 only multiplies (the compiler waits for this step's W
    // fragments there); the memory instructions follow from m-block 1 on, dealt out evenly: the DMAs of the A tile of step
    // kt+NS-1 (MX: and two of its scale chunks), then the four W loads of step kt+PFW.  Every m-block reads the A fragment two
    // m-blocks ahead, the last two those of step kt+1.
    // (always_inline: with many call sites the inliner would otherwise leave this lambda a function of its own, with the
    // accumulators and descriptors passed through memory)
    constexpr int N_DMA = A_DMA + (MX ? 2 : 0);  // DMAs per wavefront per step
    constexpr int N_W = 2 * NR;                  // W fragment loads per wavefront per step
    constexpr int N_OPS = A_DMA + (MX ? 1 : 0) + N_W;          // slots: the two scale DMAs share one
    constexpr int OPS_PER = (N_OPS + MR - 2) / (MR - 1);       // slots per m-block (m-blocks 1 .. MR-1)
    auto step = [&](int kt, auto SP, auto CHK) __attribute__((always_inline)) {
        constexpr int S = decltype(SP)::value;   // LDS stage of this step (kt % NS)
        constexpr int SB = S % NB;               // W register set of this step
        constexpr int SN = (SB + PFW) % NB;      // W register set the loads of this step fill
        constexpr int SS = S & 1;                // MX scale set of this step
        static_for<MR>([&](auto MI) {
            constexpr int mi = decltype(MI)::value;
            if constexpr (mi + FRAG_AHEAD < MR)
                read_frag(S, mi + FRAG_AHEAD, flo[(mi + FRAG_AHEAD) % FRAG_BUFS], fhi[(mi + FRAG_AHEAD) % FRAG_BUFS]);
            else
                read_frag((S + 1) % NS, mi + FRAG_AHEAD - MR, flo[(mi + FRAG_AHEAD) % FRAG_BUFS], fhi[(mi + FRAG_AHEAD) % FRAG_BUFS]);
            if constexpr (mi >= 1) {
                static_for<OPS_PER>([&](auto Q) {
                    constexpr int op = (mi - 1) * OPS_PER + decltype(Q)::value;
                    if constexpr (op < A_DMA) {
                        dma_a1(kt + NS - 1, (S + NS - 1) % NS, op, CHK);
                    } else if constexpr (MX && op == A_DMA) {
                        dma_sc(kt + NS - 1, (S + NS - 1) % NS, 0);
                        dma_sc(kt + NS - 1, (S + NS - 1) % NS, 1);
                    } else if constexpr (op < N_OPS) {
                        load_b1(kt + PFW, op - (N_OPS - N_W), blo[SN], bhi[SN], CHK);
                    }
                });
            }
            // MX: the scale dwords of step kt+1 leave their slot for the other register set, one per m-block
            if constexpr (MX && mi >= MR - (MP + NP)) read_sc((S + 1) % NS, mi - (MR - (MP + NP)), sav[SS ^ 1], sbv[SS ^ 1]);
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
                    mfma_mx<0, ni & 1, mi & 1>(acc[mi][ni], blo[SB][ni], alo, sbv[SS][ni / 2], sav[SS][mi / 2]);
                });
                static_for<NR>([&](auto NI) {
                    constexpr int ni = decltype(NI)::value;
                    mfma_mx<1, ni & 1, mi & 1>(acc[mi][ni], bhi[SB][ni], ahi, sbv[SS][ni / 2], sav[SS][mi / 2]);
                });
            } else if constexpr (KIND == KIND_MXFP8) {
                const v8i af = {alo[0], alo[1], alo[2], alo[3], ahi[0], ahi[1], ahi[2], ahi[3]};
                static_for<NR>([&](auto NI) {
                    constexpr int ni = decltype(NI)::value;
                    const v8i bf = {blo[SB][ni][0], blo[SB][ni][1], blo[SB][ni][2], blo[SB][ni][3],
                                    bhi[SB][ni][0], bhi[SB][ni][1], bhi[SB][ni][2], bhi[SB][ni][3]};
                    mfma_mx8<SS, ni & 1, mi & 1>(acc[mi][ni], bf, af, sbv[SS][ni / 2], sav[SS][mi / 2]);
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
        // The DMAs this wavefront issued NS-3 steps ago (A tile of step kt+2) must have landed before the barrier: behind them
        // it has issued the W loads of that step and everything of the steps since.
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(N_W + (NS - 3) * (N_DMA + N_W)) : "memory");
    };
    static_assert(N_W + (NS - 3) * (N_DMA + N_W) <= 63 && PFW * N_W <= 63, "vmcnt holds six bits");

    // prologue: the epilogue's scales into LDS, A(0) .. A(NS-2) (and their MX scales) by DMA, W(0..PFW-1) into registers
    float ep_sa = 0.f, ep_sb = 0.f;
    if constexpr (SCALED && STORE != STORE_ACC) {
        if (tid < TM) {
            const int m = m0 + tid;
            ep_sa = p.sa[m < p.M ? m : p.M - 1];
        }
        if (tid < TN) {
            const int n = n0 + tid;
            ep_sb = p.sb[n < p.N ? n : p.N - 1];
        }
    }
#pragma unroll
    for (int s = 0; s < NS - 1; s++) {
#pragma unroll
        for (int j = 0; j < A_DMA; j++) dma_a1(kt_begin + s, s, j, std::true_type{});
        if constexpr (MX) {
            dma_sc(kt_begin + s, s, 0);
            dma_sc(kt_begin + s, s, 1);
        }
    }
    static_for<PFW>([&](auto I) {
        constexpr int i = decltype(I)::value;
#pragma unroll
        for (int idx = 0; idx < 2 * NR; idx++) load_b1(kt_begin + i, idx, blo[i], bhi[i], std::true_type{});
    });
    if constexpr (SCALED && STORE != STORE_ACC) {
        if (tid < TM) reinterpret_cast<float*>(lds_x)[tid] = ep_sa;
        if (tid < TN) reinterpret_cast<float*>(lds_x)[TM + tid] = ep_sb;
    }
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(PFW * N_W) : "memory");
    static_for<FRAG_AHEAD>([&](auto I) {
        constexpr int i = decltype(I)::value;
        read_frag(0, i, flo[i], fhi[i]);
    });
    if constexpr (MX) {
#pragma unroll
        for (int q = 0; q < MP + NP; q++) read_sc(0, q, sav[0], sbv[0]);
    }

    T8_STAMP(1);
    // NS K steps per iteration (LDS stages and register sets are compile-time).  The loop bodies have no branches: the
    // compiler's count of outstanding loads at the loop head is then the same on every path and its waits for W stay exact
    // (with skipped steps inside the loop it assumed the worst case and waited for every load once per iteration).
    // The first loop runs while every load it issues (NS-1 steps ahead at most) lies inside the K range and before the
    // K tail, so it issues them unchecked; the second one finishes the range with checked loads; the steps that are left
    // run behind it.
    const int kt_full = (K % TK) ? kt_end - 1 : kt_end;  // steps before this one have all 128 bytes
    int kt = kt_begin;
    for (; kt + 2 * NS - 1 <= kt_full; kt += NS)
        static_for<NS>([&](auto I) { step(kt + decltype(I)::value, I, std::false_type{}); });
    for (; kt + NS <= kt_end; kt += NS)
        static_for<NS>([&](auto I) { step(kt + decltype(I)::value, I, std::true_type{}); });
    static_for<NS - 1>([&](auto I) {
        if (kt + decltype(I)::value < kt_end) step(kt + decltype(I)::value, I, std::true_type{});
    });
    // wait states between the last MFMA and the first ordinary read of an accumulator (the compiler does not know that the
    // asm statements are MFMAs), and every DMA still on its way (redirected past the bounds) must be done before the
    // stages are reused for C
    asm volatile("s_nop 15\n\ts_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    T8_STAMP(2);

    // The epilogue derives its thread indices afresh (lane id from the execution mask, wavefront id from a scalar register): the
    // ones of the prologue would otherwise be kept alive through the loops, where no register is free for them (they were
    // spilled to scratch memory: 16 bytes per thread written and read back once per tile).
    int lane_e;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane_e));
    const int tid_e = wave * 64 + lane_e, li_e = lane_e & 15, lg_e = lane_e >> 4;

    float sa_v[MR];
    v4f sb_v[NR];
    if constexpr (STORE != STORE_ACC && SCALED) {
#pragma unroll
        for (int mi = 0; mi < MR; mi++) sa_v[mi] = reinterpret_cast<const float*>(lds_x)[mi * 16 + li_e];
#pragma unroll
        for (int ni = 0; ni < NR; ni++) sb_v[ni] = *reinterpret_cast<const v4f*>(lds_x + (TM + (wave * NR + ni) * 16 + lg_e * 4) * 4);
    }

    // raw accumulators of this workgroup -> slice blockIdx.y of `dst` ([splits][M][N] of 4-byte values)
    auto store_partial = [&](void* dst) __attribute__((always_inline)) {
        static_for<MR>([&](auto MI) {
            constexpr int mi = decltype(MI)::value;
            const int m = m0 + mi * 16 + li_e;
            if (m < p.M) {
                static_for<NR>([&](auto NI) {
                    constexpr int ni = decltype(NI)::value;
                    const int n = n0 + (wave * NR + ni) * 16 + lg_e * 4;
                    if (n < p.N) {
                        const size_t idx = (size_t)m * (size_t)p.N + (size_t)n;
                        const size_t slice = (size_t)blockIdx.y * (size_t)p.M * (size_t)p.N;
                        *reinterpret_cast<acc_t*>(reinterpret_cast<uint8_t*>(dst) + (slice + idx) * 4) = acc[mi][ni];
                    }
                });
            }
        });
    };
    if constexpr (STORE == STORE_ACC) {
        store_partial(p.c);
    } else {
        // The whole 16-bit C tile (TM rows of 2 TN bytes) is staged in the A stages and written as whole rows.
        // Nothing here is conditional: columns past N are staged like the others (their scales were clamped) and dropped by the
        // store pass.  Row mi*16 + li keeps the swizzle term li for every mi, so a lane's staging addresses are two bases
        // (one per n-block) plus compile-time offsets.
        constexpr int ROWB = TN * 2, GR = ROWB / 16, XM = 15, NT = WAVES * 64;
        static_assert(TM * ROWB <= NS * STAGE && NT / GR == 16 && GR >= 16, "C staging");
        uint8_t* st_base[NR];
#pragma unroll
        for (int ni = 0; ni < NR; ni++) st_base[ni] = lds + li_e * ROWB + (((((wave * NR + ni) * 2 + (lg_e >> 1)) ^ li_e) & (GR - 1)) << 4) + (lg_e & 1) * 8;
        const int g = tid_e & (GR - 1), r0 = tid_e / GR;  // store pass: thread -> granule tid_e % GR of rows tid_e / GR + 16 i
        const int n_st = n0 + g * 8;
        // stores go through a descriptor over the rows of C from m0 on: rows >= M fall behind its bound and are dropped; a
        // granule past N is redirected there
        __amdgpu_buffer_rsrc_t rc = make_rsrc(reinterpret_cast<uint16_t*>(p.c) + (size_t)m0 * (size_t)p.N, (uint64_t)(p.M - m0) * (uint64_t)p.N * 2ull);
        const uint32_t c_off = ((uint32_t)r0 * (uint32_t)p.N + (uint32_t)n_st) * 2u;
        const uint32_t c_step = 16u * (uint32_t)p.N * 2u;
        const uint8_t* src = lds + r0 * ROWB + ((g ^ (r0 & XM)) << 4);
        static_for<2>([&](auto HALF) {
            constexpr int half = decltype(HALF)::value;
            static_for<MR / 2>([&](auto MI) {
                constexpr int mi = half * (MR / 2) + decltype(MI)::value;
                float sa = 0.f;
                if constexpr (SCALED) sa = sa_v[mi];
                static_for<NR>([&](auto NI) {
                    constexpr int ni = decltype(NI)::value;
                    const acc_t r = acc[mi][ni];
                    v4f x;
                    if constexpr (!SCALED) {
                        x = (v4f){(float)r[0], (float)r[1], (float)r[2], (float)r[3]};
                    } else {
                        const v4f sb = sb_v[ni];
                        x = (v4f){((float)r[0] * sa) * sb[0], ((float)r[1] * sa) * sb[1], ((float)r[2] * sa) * sb[2], ((float)r[3] * sa) * sb[3]};
                    }
                    v2i out;
                    if constexpr (STORE == STORE_C) {
                        out = finish4<OUT_BF16, EPI_NONE>(x, nullptr);
                    } else {
                        const int n = n0 + (wave * NR + ni) * 16 + lg_e * 4;
                        const uint16_t* bias_n = p.bias + (n < p.N ? n : 0);
                        out = p.out == OUT_BF16 ? finish4_rt<OUT_BF16>(x, bias_n, p.epi) : finish4_rt<OUT_FP16>(x, bias_n, p.epi);
                    }
                    *reinterpret_cast<v2i*>(st_base[ni] + mi * 16 * ROWB) = out;
                });
            });
            if constexpr (half == 1) T8_STAMP(4);
            __syncthreads();
            if constexpr (half == 1) T8_STAMP(5);
#pragma unroll
            for (int i = half * (TM / 32); i < (half + 1) * (TM / 32); i++) {
                const v4i v = *reinterpret_cast<const v4i*>(src + i * 16 * ROWB);
                __builtin_amdgcn_raw_buffer_store_b128((v4u)v, rc, (int)(n_st < p.N ? c_off + (uint32_t)i * c_step : 0xFFFFFFF0u), 0, 0);
            }
        });
    }
#ifdef T8_TIMING
    T8_STAMP(6);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    T8_STAMP(3);
#endif
}

template <int KIND, int STORE, int MR, int WAVES, int NS, int PFW>
hipError_t launch_tiled_dma(const A8W8Params& p, hipStream_t stream) {
    constexpr int TM = 16 * MR, TN = 32 * WAVES;
    const int tiles_m = (p.M + TM - 1) / TM, tiles_n = (p.N + TN - 1) / TN;
    const int splits = STORE == STORE_ACC && p.splits > 1 ? p.splits : 1;
    A8W8Params q = p;
    q.splits = splits;
    hipLaunchKernelGGL((k_tiled_dma<KIND, STORE, MR, WAVES, NS, PFW>), dim3(tiles_m * tiles_n, splits), dim3(WAVES * 64), 0, stream, q);
    return hipGetLastError();
}

// 256x256, eight wavefronts
template <int KIND, int STORE>
hipError_t launch_tiled8(const A8W8Params& p, hipStream_t stream) {
    return launch_tiled_dma<KIND, STORE, 16, 8, 4, 1>(p, stream);
}

// 128x128, four wavefronts, seven K steps in flight (the 8- and 16-bit kinds)
template <int KIND, int STORE>
hipError_t launch_tiled_deep(const A8W8Params& p, hipStream_t stream) {
    return launch_tiled_dma<KIND, STORE, 8, 4, 8, 7>(p, stream);
}

}  // namespace
