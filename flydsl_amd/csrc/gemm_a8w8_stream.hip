// Memory-bound small-M (M <= 32) path of the 8-bit / 16-bit preshuffle GEMM for gfx950.
//
// The whole cost is streaming W once (N*K bytes), so the launch is shaped by the memory system, not by the MFMAs:
//   * The columns are dealt out in units of 8 (half a preshuffled 16-row block), evenly over one workgroup per CU:
//     for N = 6144 that is 768 units = exactly 3 per workgroup on 256 CUs (whole 16-column blocks would give 1.5
//     blocks per CU, i.e. half the CUs twice the work of the others).  A wavefront group covers its (up to 4) units
//     with one or two 16-column MFMA windows that start at a multiple of 8 columns; lanes of a window that fall
//     outside the group's columns read nothing (their loads are redirected past the buffer bound) and store nothing.
//   * The 8 wavefronts of a workgroup are ks K-slices x (8/ks) column groups; K is never split across workgroups, so
//     the split-K reduction happens in LDS in a fixed order (deterministic, one launch, no workspace).
//   * Each wavefront walks its K slice in chunks of CH 128-byte steps: every load of a chunk (A rows, then the W
//     blocks of both windows) is issued before anything waits.  Chunks are NOT prefetched across: with all 256 CUs
//     streaming, more than about 100 KB of requests per CU only deepens the queues of the memory system (measured:
//     keeping two chunks in flight per wavefront is 4 % slower than one), so the chunk size sets the depth.
//   * A (at most 64 rows, L2 resident after first touch) is needed in fragment order (16 different rows per load
//     instruction, which costs the texture addresser more than the whole W stream), so each wavefront brings its K
//     slice of A row-contiguously into a private LDS patch (XOR-swizzled 16-byte chunks, no barrier) and picks the
//     fragments up from there.  The rows travel global -> LDS by DMA (buffer_load_dwordx4 ... lds: 64 lanes x 16 bytes to
//     consecutive LDS addresses, so the swizzle is applied to the source address of each lane): no staging registers, no
//     ds_write.  A is requested before W in every chunk: loads return in order and A comes from L2, so one
//     s_waitcnt vmcnt(number of W loads) is the wait for A.
// Operands are swapped like in the tiled kernel (src0 = W fragment, src1 = A fragment): a lane holds
// C[m = lane%16][n = window + (lane/16)*4 + 0..3].
#include "psg_common.h"

namespace {

constexpr uint32_t OOB = 0xFFFFFFF0u;  // byte offset past every buffer bound: the load returns 0 without a memory access

template <int KIND>
struct Acc {
    using type = v4f;
};
template <>
struct Acc<KIND_INT8> {
    using type = v4i;
};

// descriptor built from values forced into scalar registers (an inline-asm "s" operand must not end up in vector registers)
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc_uniform(const void* base, uint64_t bytes) {
    const uint64_t b = (uint64_t)(uintptr_t)base;
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32));
    const uint32_t n = (uint32_t)__builtin_amdgcn_readfirstlane((int)(bytes > 0xFFFFFFFFull ? 0xFFFFFFFFu : (uint32_t)bytes));
    return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>((uintptr_t)(((uint64_t)hi << 32) | lo)), 0, (int)n, 0x00020000);
}

// one DMA instruction: 64 lanes x 16 bytes from (descriptor, voff) to LDS [lds_addr, lds_addr + 1024).  Issued from inline
// assembly: the compiler does not know that it writes LDS (it would put a full vmcnt wait in front of every LDS read that
// follows), so the kernel waits for it itself.
__device__ __forceinline__ void dma16(__amdgpu_buffer_rsrc_t r, uint32_t lds_addr, uint32_t voff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" ::"s"(__builtin_amdgcn_readfirstlane((int)lds_addr)), "v"(voff), "s"(r)
                 : "memory");
}

// MB = 16-row blocks of A (1 to 4); NWIN = 16-column windows per wavefront group (1 or 2).
// CH = 128-byte K steps per chunk; NWAVES = wavefronts per workgroup.
template <int KIND, int MB, int NWIN, int NWAVES, int CH, int STORE>
__global__ void __launch_bounds__(NWAVES * 64) k_a8w8_stream(A8W8Params p) {
    using acc_t = typename Acc<KIND>::type;
    constexpr bool IS16 = KIND == KIND_FP16 || KIND == KIND_BF16;
    constexpr int ROWS = 16 * MB;
    constexpr int CPR = CH * 8;                 // 16-byte chunks per staged row (256 bytes)
    constexpr int PASSES = ROWS * CPR / 64;     // staging loads (or DMA instructions) per chunk, 1 KB of the patch each
    constexpr int RPP = 64 / CPR;               // rows per staging pass
    // A by DMA from two 16-row blocks on: fp8 N=6144 K=4096, us per launch, registers + ds_write against DMA: M=32 8.50 / 8.28,
    // M=16 6.67 / 6.84, M=1 6.33 / 6.46 (one block moves too little for the DMA's extra wait and issue cost to pay)
    constexpr bool ADMA = MB >= 2;
    __shared__ __attribute__((aligned(16))) v4i patch[NWAVES][ROWS * CPR];
    // the partial sums of the split-K reduction reuse the wavefront's own patch (it is done with it by then): with 64 rows
    // patch and a separate array would not fit the LDS together
    static_assert(ROWS * CPR >= NWIN * MB * 64, "the partial sums of a wavefront must fit its A patch");
    auto red = [&](int w) { return reinterpret_cast<acc_t*>(patch[w]); };

    const int tid = threadIdx.x;
    const int wave = wave_id();
    const int lane = tid & 63;
    const int li = lane & 15;
    const int lg = lane >> 4;
    const int K = IS16 ? (p.K << 1) : p.K;   // BYTES per operand row from here on
    const int ks = p.ksplit;                 // K slices per workgroup: 1, 2, 4 or 8 (a power of two: shifts, no divisions,
    const int ksh = __builtin_ctz(ks);       // which cost tens of instructions each in front of the first load)
    const int gpw = NWAVES >> ksh;           // column groups per workgroup
    const int tg = p.splits;                 // column groups in the whole launch
    // 8-column units are dealt out evenly: group g starts at unit g*uq + min(g, ur) (the first ur groups hold one more)
    const int uq = p.group_m, ur = p.wave_layout;
    auto unit_begin = [&](int g) { return g * uq + (g < ur ? g : ur); };
    const int my_ks = wave & (ks - 1);
    // Workgroups go round-robin over the 8 XCDs, so workgroup b of a grid that is a multiple of 8 takes the column groups
    // of position (b % 8) * grid/8 + b / 8: each XCD then owns one contiguous range of columns and the partial lines of
    // C that neighbouring workgroups share are merged in one L2 instead of being written back from several.
    const int bid = (gridDim.x & 7) == 0 ? (int)((blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3)) : (int)blockIdx.x;
    const int grp = bid * gpw + (wave >> ksh);
    const int steps = (K + 127) >> 7;
    const int per = (steps + ks - 1) >> ksh;
    const int s_begin = my_ks * per;
    const int s_end = (s_begin + per) < steps ? (s_begin + per) : steps;
    const int nchunks = s_end > s_begin ? (s_end - s_begin + CH - 1) / CH : 0;

    // this group's columns [n_begin, n_end): units dealt out evenly, at most 4 per group (host guarantees it)
    const bool has_cols = grp < tg;
    const int n_begin = has_cols ? unit_begin(grp) << 3 : 0;
    const int n_end = has_cols ? unit_begin(grp + 1) << 3 : 0;

    acc_t acc[NWIN][MB];
#pragma unroll
    for (int w = 0; w < NWIN; w++)
#pragma unroll
        for (int mb = 0; mb < MB; mb++) acc[w][mb] = (acc_t){0, 0, 0, 0};

    // Finishing work item t = tid (+ 512 per extra item): (group of the workgroup, window, m-block, lane).  Its scales
    // are fetched early (right behind the first loads) so their latency does not sit behind the reduction barrier.
    constexpr int FIN = NWIN * MB;  // items per thread when every wavefront is its own column group
    float fin_sa[FIN];
    v4f fin_sb[FIN];
    auto item_coords = [&](int t, int& g, int& frag, int& m, int& n, bool& live) {
        g = (t >> 6) / (NWIN * MB);
        frag = (t >> 6) % (NWIN * MB);
        const int gq = bid * gpw + g;
        const int nb = gq < tg ? unit_begin(gq) << 3 : 0;
        const int ne = gq < tg ? unit_begin(gq + 1) << 3 : 0;
        m = (frag % MB) * 16 + li;
        n = nb + (frag / MB) * 16 + lg * 4;
        live = g < gpw && n < ne && m < p.M;
    };
    auto fetch_scales = [&]() {
        if constexpr (STORE != STORE_ACC && !IS16) {
#pragma unroll
            for (int f = 0; f < FIN; f++) {
                int g, frag, m, n;
                bool live;
                item_coords(tid + f * NWAVES * 64, g, frag, m, n, live);
                // clamp the ADDRESS of dead items instead of selecting the loaded value (a select would wait here)
                fin_sa[f] = p.sa[live ? m : 0];
                fin_sb[f] = *reinterpret_cast<const v4f*>(p.sb + (live ? n : 0));
            }
        }
    };

    if (nchunks > 0 && n_end > n_begin) {
        __amdgpu_buffer_rsrc_t rb = make_rsrc(p.b, (uint64_t)p.N * (uint64_t)K);
        __amdgpu_buffer_rsrc_t ra = ADMA ? make_rsrc_uniform(p.a, (uint64_t)p.M * (uint64_t)K) : make_rsrc(p.a, (uint64_t)p.M * (uint64_t)K);
        v4i* my_patch = patch[wave];
        const uint32_t patch_lds = (uint32_t)(uintptr_t)my_patch;
        // per-window W offset of this lane: row n of the window, 16-byte K group lg of a 1 KB block
        uint32_t wvoff[NWIN];
#pragma unroll
        for (int w = 0; w < NWIN; w++) {
            const int n = n_begin + w * 16 + li;
            // preshuffled: 16-byte piece (K group lg, row n%16) of the 1 KB block; row-major [N,K]: row n, K offset 16*lg
            const uint32_t off = p.b_rowmajor ? (uint32_t)n * (uint32_t)K + (uint32_t)lg * 16u
                                              : (uint32_t)(n >> 4) * 16u * (uint32_t)K + (uint32_t)lg * 256u + (uint32_t)(n & 15) * 16u;
            wvoff[w] = n < n_end ? off : OOB;
        }
        const uint32_t w_step = p.b_rowmajor ? 128u : 2048u, w_half = p.b_rowmajor ? 64u : 1024u;
        // DMA instruction ps fills patch chunks [64 ps, 64 ps + 64): lane l writes physical chunk (64 ps + l) % CPR of row
        // (64 ps + l) / CPR and therefore fetches that row's logical chunk physical ^ (row & 15).  (row & 15) repeats every
        // 16 / RPP instructions, so a lane needs that many source offsets; the others follow by adding whole rows.
        constexpr int NVAR = 16 / RPP < PASSES ? 16 / RPP : PASSES;
        uint32_t a_src[NVAR];
#pragma unroll
        for (int v = 0; v < NVAR; v++) {
            const int r = v * RPP + lane / CPR;
            a_src[v] = (uint32_t)r * (uint32_t)K + (uint32_t)(((lane % CPR) ^ (r & 15)) << 4);
        }
        const uint32_t slice_end = (uint32_t)(s_end * 128 < K ? s_end * 128 : K);

        // chunk c of this wavefront's K slice: A rows first (they come from L2 and must not queue behind W), then W
        const int st_c = lane % CPR;
        const int st_r0 = lane / CPR;
        constexpr int NAT = ADMA ? 1 : PASSES;
        auto load_chunk = [&](int c, v4i (&at)[NAT], v4i (&wlo)[NWIN][CH], v4i (&whi)[NWIN][CH]) __attribute__((always_inline)) {
            const int s0 = s_begin + c * CH;
            const uint32_t kbyte0 = (uint32_t)s0 * 128u;
            if constexpr (ADMA) {
#pragma unroll
                for (int ps = 0; ps < PASSES; ps++) {
                    const uint32_t src = a_src[ps % NVAR] + (uint32_t)((ps / NVAR) * 16) * (uint32_t)K;
                    // rows >= M lie behind the descriptor's bound; a chunk past the K slice (or a chunk that does not exist) is
                    // redirected there too: both write zeros
                    const uint32_t kb = kbyte0 + ((((uint32_t)(lane % CPR)) ^ (uint32_t)(((ps % NVAR) * RPP + lane / CPR) & 15)) << 4);
                    const bool a_ok = c < nchunks && kb < slice_end;
                    dma16(ra, patch_lds + (uint32_t)ps * 1024u, a_ok ? src + kbyte0 : OOB);
                }
            } else {
                const uint32_t kbyte = kbyte0 + (uint32_t)st_c * 16u;
                const bool a_ok = c < nchunks && kbyte < slice_end;
#pragma unroll
                for (int ps = 0; ps < PASSES; ps++) {
                    const int r = st_r0 + ps * RPP;
                    at[ps] = buf_load16(ra, a_ok ? (uint32_t)r * (uint32_t)K + kbyte : OOB, 0);
                }
            }
#pragma unroll
            for (int w = 0; w < NWIN; w++)
#pragma unroll
                for (int u = 0; u < CH; u++) {
                    const int s = s0 + u;
                    const bool has_lo = c < nchunks && s < s_end;      // wave-uniform
                    const bool has_hi = has_lo && (s * 128 + 64) < K;  // K % 128 == 64: the last step has no upper half
                    wlo[w][u] = buf_load16_nt(rb, has_lo ? wvoff[w] : OOB, has_lo ? (uint32_t)s * w_step : 0u);
                    whi[w][u] = buf_load16_nt(rb, has_hi ? wvoff[w] : OOB, has_hi ? (uint32_t)s * w_step + w_half : 0u);
                }
            // keep the machine scheduler from sinking these loads below later code to save registers
            __builtin_amdgcn_sched_barrier(0);
        };
        // A through the private patch into fragment order, then the chunk's MFMAs as W arrives
        auto compute_chunk = [&](const v4i (&at)[NAT], const v4i (&wlo)[NWIN][CH], const v4i (&whi)[NWIN][CH], auto FIRST) __attribute__((always_inline)) {
            if constexpr (ADMA) {
                // the chunk's A has landed once only what was requested behind its DMAs is still on its way: its W loads
                // and, for the first chunk, the epilogue scales
                constexpr int BEHIND = NWIN * CH * 2 + (decltype(FIRST)::value && STORE != STORE_ACC && !IS16 ? 2 * FIN : 0);
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"(BEHIND) : "memory");
            } else {
#pragma unroll
                for (int ps = 0; ps < PASSES; ps++) {
                    const int r = st_r0 + ps * RPP;
                    my_patch[r * CPR + (st_c ^ (r & 15))] = at[ps];
                }
            }
            // one K step's MFMAs on fragments alo / ahi (per 16-row block) and W registers wlo / whi (per window) of step t
            auto mfma_step = [&](int t, const v4i (&alo_t)[MB], const v4i (&ahi_t)[MB], int w) {
#pragma unroll
                for (int mb = 0; mb < MB; mb++) {
                    if constexpr (KIND == KIND_INT8) {
                        acc[w][mb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wlo[w][t], alo_t[mb], acc[w][mb], 0, 0, 0);
                        acc[w][mb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(whi[w][t], ahi_t[mb], acc[w][mb], 0, 0, 0);
                    } else if constexpr (KIND == KIND_BF16) {
                        acc[w][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, wlo[w][t]), __builtin_bit_cast(v8bf, alo_t[mb]), acc[w][mb], 0, 0, 0);
                        acc[w][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, whi[w][t]), __builtin_bit_cast(v8bf, ahi_t[mb]), acc[w][mb], 0, 0, 0);
                    } else if constexpr (KIND == KIND_FP16) {
                        acc[w][mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, wlo[w][t]), __builtin_bit_cast(v8h, alo_t[mb]), acc[w][mb], 0, 0, 0);
                        acc[w][mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, whi[w][t]), __builtin_bit_cast(v8h, ahi_t[mb]), acc[w][mb], 0, 0, 0);
                    } else {
                        const v8i bf = {wlo[w][t][0], wlo[w][t][1], wlo[w][t][2], wlo[w][t][3],
                                        whi[w][t][0], whi[w][t][1], whi[w][t][2], whi[w][t][3]};
                        const v8i af = {alo_t[mb][0], alo_t[mb][1], alo_t[mb][2], alo_t[mb][3],
                                        ahi_t[mb][0], ahi_t[mb][1], ahi_t[mb][2], ahi_t[mb][3]};
                        acc[w][mb] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf, af, acc[w][mb], 0, 0, 0, 0, 0, 0);
                    }
                }
            };
            if constexpr (MB <= 2) {
                // all fragments of the chunk are read first, then window by window
                v4i alo[CH][MB], ahi[CH][MB];
#pragma unroll
                for (int t = 0; t < CH; t++)
#pragma unroll
                    for (int mb = 0; mb < MB; mb++) {
                        const int r = mb * 16 + li;
                        alo[t][mb] = my_patch[r * CPR + ((t * 8 + lg) ^ (r & 15))];
                        ahi[t][mb] = my_patch[r * CPR + ((t * 8 + 4 + lg) ^ (r & 15))];
                    }
#pragma unroll
                for (int w = 0; w < NWIN; w++)
#pragma unroll
                    for (int t = 0; t < CH; t++) mfma_step(t, alo[t], ahi[t], w);
            } else {
                // three and four 16-row blocks: step by step, so that only one step's fragments are live (the order of the
                // additions into every accumulator is the same; all fragments at once spilled registers at 64 rows)
#pragma unroll
                for (int t = 0; t < CH; t++) {
                    v4i alo[MB], ahi[MB];
#pragma unroll
                    for (int mb = 0; mb < MB; mb++) {
                        const int r = mb * 16 + li;
                        alo[mb] = my_patch[r * CPR + ((t * 8 + lg) ^ (r & 15))];
                        ahi[mb] = my_patch[r * CPR + ((t * 8 + 4 + lg) ^ (r & 15))];
                    }
#pragma unroll
                    for (int w = 0; w < NWIN; w++) mfma_step(t, alo, ahi, w);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        };

        v4i at[NAT];
        v4i wlo[NWIN][CH], whi[NWIN][CH];
        load_chunk(0, at, wlo, whi);
        fetch_scales();
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (ADMA) {
            // the first chunk apart: its wait for A counts the scale loads too
            compute_chunk(at, wlo, whi, std::true_type{});
            if (1 < nchunks) load_chunk(1, at, wlo, whi);
            for (int c = 1; c < nchunks; c++) {
                compute_chunk(at, wlo, whi, std::false_type{});
                if (c + 1 < nchunks) load_chunk(c + 1, at, wlo, whi);
            }
        } else {
            for (int c = 0; c < nchunks; c++) {
                compute_chunk(at, wlo, whi, std::false_type{});
                if (c + 1 < nchunks) load_chunk(c + 1, at, wlo, whi);
            }
        }
    } else {
        fetch_scales();  // wavefronts without work still finish outputs
    }

    // split-K reduction through LDS, fixed order
#pragma unroll
    for (int w = 0; w < NWIN; w++)
#pragma unroll
        for (int mb = 0; mb < MB; mb++) red(wave)[(w * MB + mb) * 64 + lane] = acc[w][mb];
    __syncthreads();

#pragma unroll
    for (int f = 0; f < FIN; f++) {
        int g, frag, m, n;
        bool live;
        item_coords(tid + f * NWAVES * 64, g, frag, m, n, live);
        if (live) {
            // all partial sums are read in one batch (no wait between them), then added in slice order
            acc_t part[NWAVES];
#pragma unroll
            for (int j = 0; j < NWAVES; j++) part[j] = red(g * ks + (j < ks ? j : 0))[frag * 64 + lane];
            acc_t sum = part[0];
#pragma unroll
            for (int j = 1; j < NWAVES; j++)
                if (j < ks) sum += part[j];
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

template <int KIND, int NWAVES, int CH, int STORE>
hipError_t launch_kind(const A8W8Params& p, int nwin, int grid, hipStream_t stream) {
    const int mb = (p.M + 15) / 16;
#define PSG_GO(MB_, NWIN_)                                                                                                   \
    {                                                                                                                        \
        hipLaunchKernelGGL((k_a8w8_stream<KIND, MB_, NWIN_, NWAVES, CH, STORE>), dim3(grid), dim3(NWAVES * 64), 0, stream, p); \
        return hipGetLastError();                                                                                            \
    }
    if (mb == 1) {
        if (nwin == 2) PSG_GO(1, 2) else PSG_GO(1, 1)
    }
    if (mb == 2) {
        if (nwin == 2) PSG_GO(2, 2) else PSG_GO(2, 1)
    }
    if (mb == 3) {
        if (nwin == 2) PSG_GO(3, 2) else PSG_GO(3, 1)
    }
    if (nwin == 2) PSG_GO(4, 2) else PSG_GO(4, 1)
#undef PSG_GO
}

template <int KIND, int STORE>
hipError_t launch_planned(const A8W8Params& p0, int kbytes, hipStream_t stream) {
    A8W8Params p = p0;
    const int steps = (kbytes + 127) / 128;
    // long rows: 8 wavefronts x chunks of 2 steps (96 KB of requests per CU at a time); short rows: 4 wavefronts x
    // chunks of 4 steps, which start faster and leave fewer partial sums to reduce
    const int nwaves = steps >= 32 ? 8 : 4;
    int ks = nwaves;  // K slices per workgroup: every slice holds at least two K steps
    while (ks > 1 && ks * 2 > steps) ks >>= 1;
    const int gpw = nwaves / ks;
    const long units = p.N / 8;
    const long cus = psg_cu_count();
    const long rounds = (units + 4 * cus * gpw - 1) / (4 * cus * gpw);
    long tg = cus * gpw * rounds;  // column groups: a whole number of workgroups per CU ...
    if (tg > units) tg = units;    // ... but never less than one 8-column unit per group
    const int max_units = (int)((units + tg - 1) / tg);
    const int nwin = max_units > 2 ? 2 : 1;
    p.ksplit = ks;
    p.splits = (int)tg;
    p.group_m = (int)(units / tg);      // units per group ...
    p.wave_layout = (int)(units % tg);  // ... and how many groups hold one more
    const int grid = (int)((tg + gpw - 1) / gpw);
    return nwaves == 8 ? launch_kind<KIND, 8, 2, STORE>(p, nwin, grid, stream) : launch_kind<KIND, 4, 4, STORE>(p, nwin, grid, stream);
}

}  // namespace

// Host entry used by the C-ABI layer.  Requires 1 <= M <= 64.  Plans the launch: wavefronts per workgroup by the
// row length, K slices per workgroup so that a slice holds at least two K steps, then column groups dealt out
// evenly over a multiple of the CU count (at most four 8-column units per group, at least one).
hipError_t psg_launch_a8w8_stream(const A8W8Params& p, int kind, int store, hipStream_t stream) {
    const int kbytes = (kind == KIND_FP16 || kind == KIND_BF16) ? p.K * 2 : p.K;
    switch (kind) {
        case KIND_INT8: return store == STORE_ACC ? launch_planned<KIND_INT8, STORE_ACC>(p, kbytes, stream) : launch_planned<KIND_INT8, STORE_C>(p, kbytes, stream);
        case KIND_FP8: return store == STORE_ACC ? launch_planned<KIND_FP8, STORE_ACC>(p, kbytes, stream) : launch_planned<KIND_FP8, STORE_C>(p, kbytes, stream);
        case KIND_BF16: return store == STORE_ACC ? launch_planned<KIND_BF16, STORE_ACC>(p, kbytes, stream) : launch_planned<KIND_BF16, STORE_C>(p, kbytes, stream);
        case KIND_FP16: return store == STORE_ACC ? launch_planned<KIND_FP16, STORE_ACC>(p, kbytes, stream) : launch_planned<KIND_FP16, STORE_C>(p, kbytes, stream);
    }
    return hipErrorInvalidValue;
}
