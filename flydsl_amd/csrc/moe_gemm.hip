// MoE grouped GEMMs for gfx950 over expert-sorted token blocks, int8 or OCP fp8 operands with per-row fp32 scales, or int8
// activations against packed int4 weights (W4A8).
//
// The sorted row list (one entry per routed (token, slot), padded per expert to whole blocks of BM rows) says which
// row of x each tile row reads; one expert id per block says which slab of the preshuffled weights it multiplies.
//   stage 1 (gate-up): y[t, slot, n] = silu(g) * u with g = x[t] . W1[e, n], u = x[t] . W1[e, inter + n]
//   stage 2 (down):    y[n] = a2[t, slot] . W2[e, n] (* routing weight); added atomically into out[t] or written to
//                      out[t*topk + slot]
// Workgroup = four wavefronts side by side along N, tile BM x 64*NR, 128 bytes of K per step.  The A rows are
// gathered (per-row offsets through a bounds-checked buffer descriptor: padding rows read zeros) into a two-stage
// XOR-swizzled LDS tile; W fragments go straight from the expert's slab into MFMA operand registers (lane l reads
// bytes [16l, 16l+16) of a 1 KB block, the same wire format as the plain GEMM).  Stage 1 keeps two accumulators per
// fragment (gate and up) so silu(g)*u happens in registers.
// W4A8: the weights are the preshuffled int8 bytes with every 8 consecutive values v0..v7 packed into 4 bytes, byte j =
// (v_j & 15) | (v_{j+4} << 4) (tests/kernels/test_moe_gemm_2stage.py:64-80 of the reference), so a lane's 16-byte piece
// of a fragment is 8 bytes at half the offset; it is unpacked with the reference's sign-extending mask-and-multiply
// (kernels/common/mma/mfma_preshuffle_pipeline.py:225-238) into the same int8 fragment and multiplied by the int8 MFMA.
#include "psg_common.h"

namespace {

typedef __fp16 v2h __attribute__((ext_vector_type(2)));
typedef __bf16 v2b __attribute__((ext_vector_type(2)));

template <int KIND>
struct MoeAcc {
    using type = v4f;
};
template <>
struct MoeAcc<KIND_INT8> {
    using type = v4i;
};
template <>
struct MoeAcc<KIND_INT8W4> {
    using type = v4i;
};

// 8 packed int4 (one dword) -> two dwords of int8: the low nibbles of the four bytes, then the high nibbles
__device__ __forceinline__ void unpack_int4(int packed, int& even, int& odd) {
    even = (packed & 0x0F0F0F0F) | ((packed & 0x08080808) * 0x1E);
    const int t = (int)((unsigned)packed >> 4);
    odd = (t & 0x0F0F0F0F) | ((t & 0x08080808) * 0x1E);
}
__device__ __forceinline__ v4i unpack_int4x16(v2i packed) {
    int e0, o0, e1, o1;
    unpack_int4(packed[0], e0, o0);
    unpack_int4(packed[1], e1, o1);
    return (v4i){e0, o0, e1, o1};
}

__device__ __forceinline__ int moe_lds_off(int row, int kc) { return row * 128 + ((kc ^ ((row >> 1) & 7)) << 4); }

__device__ __forceinline__ float silu(float g) { return g / (1.0f + __expf(-g)); }

// CO = 2: the workgroup's BM rows are TWO consecutive blocks of the sorted list when both belong to the same expert (blocks
// of 16 or 32 rows: an expert with 17 to 32 routed rows would otherwise stream its weights once per block).  Blocks pair up
// from the start of each run of equal expert ids: the workgroup of the second block of a pair ends at once, and the
// first one treats the second half of its tile as padding when the run ends there.
template <int KIND, int MR, int NR, int STAGE, int CO = 1>
__global__ void __launch_bounds__(256) k_moe_gemm(MoeParams p) {
    using acc_t = typename MoeAcc<KIND>::type;
    constexpr int BM = 16 * MR, TN = 64 * NR;
    constexpr int BLK = BM / CO;                        // rows of one block of the sorted list
    constexpr int NSET = STAGE == 1 ? 2 : 1;           // gate and up
    constexpr int A_LOADS = (BM * 8 + 255) / 256;      // 16-byte chunks of the A tile per thread
    constexpr bool W4 = KIND == KIND_INT8W4;           // packed int4 weights
    constexpr int WSH = W4 ? 1 : 0;                    // weight byte offsets are halved
    __shared__ __attribute__((aligned(16))) uint8_t lds[2][BM * 128];
    __shared__ int ids[BM];
    __shared__ float s_sx[BM], s_rw[BM];  // per tile row: scale of its x row and routing weight, fetched before the K loop

    const int tid = threadIdx.x;
    const int wave = wave_id();
    const int lane = tid & 63, li = lane & 15, lg = lane >> 4;
    const int blk = (int)blockIdx.y;
    const int n0 = (int)blockIdx.x * TN;
    const int used = p.num_valid[0];
    if (blk * BLK >= used) return;                     // uniform: blocks past the sorted rows in use
    const int e = p.expert_ids[blk];
    if (e < 0 || e >= p.experts) return;               // uniform: a block without an expert
    int rows_live = BLK;                               // rows of the tile that belong to this workgroup's expert
    if constexpr (CO == 2) {
        // position of this block in its run of equal expert ids: 64 earlier ids at a time, one per lane
        int before = 0;
        for (int base = blk - 1; base >= 0; base -= 64) {
            const int j = base - lane;
            const unsigned long long same = __ballot(j >= 0 && p.expert_ids[j] == e);
            const int run = same == ~0ull ? 64 : __builtin_ctzll(~same);
            before += run;
            if (run < 64) break;
        }
        before = __builtin_amdgcn_readfirstlane(before);
        if (before & 1) return;                        // uniform: the second block of a pair
        if (blk + 1 < (int)gridDim.y && (blk + 1) * BLK < used && p.expert_ids[blk + 1] == e) rows_live = BM;  // (gridDim.y = entries of expert_ids)
    }

    const int K = p.K, KT = K >> 7;
    const int rows_x = (STAGE == 1 && !p.x_slot_major) ? p.tokens : p.tokens * p.topk;
    const int rows_e = STAGE == 1 ? 2 * p.n_out : p.n_out;            // weight rows per expert
    __amdgpu_buffer_rsrc_t ra = make_rsrc(p.x, (uint64_t)rows_x * (uint64_t)K);
    const uint8_t* w_e = p.w + (((uint64_t)e * (uint64_t)rows_e * (uint64_t)K) >> WSH);
    __amdgpu_buffer_rsrc_t rb = make_rsrc(w_e, ((uint64_t)rows_e * (uint64_t)K) >> WSH);

    // n-blocks of this wavefront inside the expert's slab: set 0 = gate (or the only set), set 1 = up
    uint32_t b_voff[NSET][NR];
#pragma unroll
    for (int s = 0; s < NSET; s++)
#pragma unroll
        for (int ni = 0; ni < NR; ni++) {
            const int n = n0 + (ni * 4 + wave) * 16;                  // first column of the block: the four wavefronts of pass ni
                                                                      // cover 64 consecutive columns
            const int nb = (n + s * p.n_out) >> 4;
            b_voff[s][ni] = n < p.n_out ? ((uint32_t)nb * 16u * (uint32_t)K + (uint32_t)lane * 16u) >> WSH : 0xFFFFFFF0u;
        }

    uint32_t a_voff[A_LOADS];
    int a_ldsoff[A_LOADS];
    v4i areg[A_LOADS];
    auto load_a = [&](int kt) {
#pragma unroll
        for (int j = 0; j < A_LOADS; j++) {
            const bool ok = kt < KT;
            areg[j] = buf_load16(ra, ok ? a_voff[j] : 0xFFFFFFF0u, ok ? (uint32_t)kt * 128u : 0u);
        }
    };
    auto store_a = [&](int stage) {
#pragma unroll
        for (int j = 0; j < A_LOADS; j++)
            if (a_ldsoff[j] >= 0) *reinterpret_cast<v4i*>(&lds[stage][a_ldsoff[j]]) = areg[j];
    };
    using wreg_t = typename std::conditional<W4, v2i, v4i>::type;  // a lane's piece of a W fragment as it is loaded
    // W register sets: the fragments of step kt live in set kt % NWS and are requested WPF steps ahead.  Stage-1 tiles of up
    // to 32 rows (decode) are bound by the bytes of W a workgroup keeps in flight (64 tokens x top-8 on 32 experts: 86 -> 80 us
    // with three steps ahead); stage 2 (34 -> 36 us) and packed int4 weights (36 -> 38) are not and stay one step ahead
    constexpr int WPF = (MR <= 2 && STAGE == 1 && !W4) ? 3 : 1;
    constexpr int NWS = WPF + 1;
    wreg_t blo[NWS][NSET][NR], bhi[NWS][NSET][NR];
    auto load_b = [&](int kt, int set) {
#pragma unroll
        for (int s = 0; s < NSET; s++)
#pragma unroll
            for (int ni = 0; ni < NR; ni++) {
                const bool ok = kt < KT;
                if constexpr (W4) {
                    blo[set][s][ni] = buf_load8(rb, ok ? b_voff[s][ni] : 0xFFFFFFF0u, ok ? (uint32_t)kt * 1024u : 0u);
                    bhi[set][s][ni] = buf_load8(rb, ok ? b_voff[s][ni] + 512u : 0xFFFFFFF0u, ok ? (uint32_t)kt * 1024u : 0u);
                } else {
                    blo[set][s][ni] = buf_load16(rb, ok ? b_voff[s][ni] : 0xFFFFFFF0u, ok ? (uint32_t)kt * 2048u : 0u);
                    bhi[set][s][ni] = buf_load16(rb, ok ? b_voff[s][ni] + 1024u : 0xFFFFFFF0u, ok ? (uint32_t)kt * 2048u : 0u);
                }
            }
    };

    // the weight scales of the lane's columns (pass ni: columns ni*64 + wave*16 + lg*4 + 0..3), also ahead of the K loop
    v4f swa_[NR], swb_[STAGE == 1 ? NR : 1];
#pragma unroll
    for (int ni = 0; ni < NR; ni++) {
        const int ncol = n0 + ni * 64 + wave * 16 + lg * 4;
        const bool in = ncol < p.n_out;
        swa_[ni] = in ? *reinterpret_cast<const v4f*>(p.sw + (size_t)e * rows_e + ncol) : (v4f){0.f, 0.f, 0.f, 0.f};
        if constexpr (STAGE == 1) swb_[ni] = in ? *reinterpret_cast<const v4f*>(p.sw + (size_t)e * rows_e + p.n_out + ncol) : (v4f){0.f, 0.f, 0.f, 0.f};
    }

    acc_t acc[MR][NSET][NR];
#pragma unroll
    for (int mi = 0; mi < MR; mi++)
#pragma unroll
        for (int s = 0; s < NSET; s++)
#pragma unroll
            for (int ni = 0; ni < NR; ni++) acc[mi][s][ni] = (acc_t){0, 0, 0, 0};

    auto step = [&](int kt, auto SP, auto WP) __attribute__((always_inline)) {
        constexpr int S = decltype(SP)::value;    // LDS stage of this step's A tile
        constexpr int WS = decltype(WP)::value;   // register set of this step's W fragments
        load_a(kt + 1);
        load_b(kt + WPF, (WS + WPF) % NWS);
        // packed int4: this step's fragments unpacked once, in front of the row blocks that share them
        v4i ulo[W4 ? NSET : 1][W4 ? NR : 1], uhi[W4 ? NSET : 1][W4 ? NR : 1];
        if constexpr (W4) {
#pragma unroll
            for (int s = 0; s < NSET; s++)
#pragma unroll
                for (int ni = 0; ni < NR; ni++) {
                    ulo[s][ni] = unpack_int4x16(blo[WS][s][ni]);
                    uhi[s][ni] = unpack_int4x16(bhi[WS][s][ni]);
                }
        }
        static_for<MR>([&](auto MI) {
            constexpr int mi = decltype(MI)::value;
            const int row = mi * 16 + li;
            const v4i alo = *reinterpret_cast<const v4i*>(&lds[S][moe_lds_off(row, lg)]);
            const v4i ahi = *reinterpret_cast<const v4i*>(&lds[S][moe_lds_off(row, 4 + lg)]);
            static_for<NSET>([&](auto SI) {
                constexpr int s = decltype(SI)::value;
                static_for<NR>([&](auto NI) {
                    constexpr int ni = decltype(NI)::value;
                    if constexpr (W4) {
                        acc[mi][s][ni] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ulo[s][ni], alo, acc[mi][s][ni], 0, 0, 0);
                        acc[mi][s][ni] = __builtin_amdgcn_mfma_i32_16x16x64_i8(uhi[s][ni], ahi, acc[mi][s][ni], 0, 0, 0);
                    } else if constexpr (KIND == KIND_INT8) {
                        acc[mi][s][ni] = __builtin_amdgcn_mfma_i32_16x16x64_i8(blo[WS][s][ni], alo, acc[mi][s][ni], 0, 0, 0);
                        acc[mi][s][ni] = __builtin_amdgcn_mfma_i32_16x16x64_i8(bhi[WS][s][ni], ahi, acc[mi][s][ni], 0, 0, 0);
                    } else {
                        const v8i w8 = __builtin_shufflevector(blo[WS][s][ni], bhi[WS][s][ni], 0, 1, 2, 3, 4, 5, 6, 7);
                        const v8i a8 = __builtin_shufflevector(alo, ahi, 0, 1, 2, 3, 4, 5, 6, 7);
                        acc[mi][s][ni] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(w8, a8, acc[mi][s][ni], 0, 0, 0, 0, 0, 0);
                    }
                });
            });
        });
        store_a(S ^ 1);
        __syncthreads();
    };

    // W first: its addresses need only the expert, so these requests are in flight while the sorted row list is fetched
    static_for<WPF>([&](auto I) { load_b(decltype(I)::value, decltype(I)::value); });
    if (tid < BM) {
        const int q = blk * BLK + tid;
        ids[tid] = (tid < rows_live && q < p.sorted_size) ? p.sorted_ids[q] : p.tokens;  // past the list or the pair = a padding row
    }
    __syncthreads();

    // row of x (and of its scale) a tile row reads, or -1 for a padding row
    auto x_row = [&](int r) {
        const uint32_t sid = (uint32_t)ids[r];
        const int t = (int)(sid & 0xFFFFFFu), s = (int)(sid >> 24);
        if (t >= p.tokens || s >= p.topk) return -1;
        if constexpr (STAGE == 1) return p.x_slot_major ? s * p.tokens + t : t;
        return t * p.topk + s;
    };
    // the epilogue's per-row factors now, so that their memory latency runs under the K loop (whose barriers also make them
    // visible to every wavefront)
    if (tid < BM) {
        const int xr = x_row(tid);
        s_sx[tid] = xr >= 0 ? p.sx[xr] : 0.f;
        s_rw[tid] = (p.doweight && xr >= 0) ? p.sorted_w[blk * BLK + tid] : 1.0f;
    }

#pragma unroll
    for (int j = 0; j < A_LOADS; j++) {
        const int c = tid + 256 * j, row = c >> 3, kc = c & 7;
        const int xr = row < BM ? x_row(row) : -1;
        a_voff[j] = xr >= 0 ? (uint32_t)xr * (uint32_t)K + (uint32_t)kc * 16u : 0xFFFFFFF0u;
        a_ldsoff[j] = row < BM ? moe_lds_off(row, kc) : -1;
    }
    load_a(0);
    store_a(0);
    __syncthreads();
    // unrolled over lcm(2 LDS stages, NWS register sets) steps so that both indices are compile-time
    constexpr int UN = NWS % 2 == 0 ? NWS : 2 * NWS;
    for (int kt0 = 0; kt0 < KT; kt0 += UN) {
        static_for<UN>([&](auto I) {
            constexpr int i = decltype(I)::value;
            if (kt0 + i < KT) step(kt0 + i, std::integral_constant<int, i & 1>{}, std::integral_constant<int, i % NWS>{});
        });
    }

    // Epilogue, one pass per ni (64 consecutive columns of the tile): every lane finishes its own fragments (rows
    // mi*16 + li, columns ni*64 + wave*16 + lg*4 + 0..3) into an LDS tile of BM rows (free after the loop's last
    // barrier; 16-byte granules XOR-swizzled by the row), then the workgroup walks the tile row by row so that one
    // store or atomic instruction covers whole 128- or 256-byte rows of the output instead of 16 rows x 16 bytes.
    const bool f32_out = p.out_dtype == OUT_F32;
    const int esize = f32_out ? 4 : 2;
    const int row_bytes = 64 * esize;                  // one pass's row in LDS: 128 or 256 bytes (both stages hold BM*256)
    const int gmask = (row_bytes >> 4) - 1;            // granules per row - 1 (7 or 15)
    uint8_t* stage = &lds[0][0];
    static_for<NR>([&](auto NI) {
        constexpr int ni = decltype(NI)::value;
        const int ncol = n0 + ni * 64 + wave * 16 + lg * 4;   // first of the lane's four columns
        const v4f swa = swa_[ni], swb = swb_[STAGE == 1 ? ni : 0];
        static_for<MR>([&](auto MI) {
            constexpr int mi = decltype(MI)::value;
            const int r = mi * 16 + li;
            const float sx = s_sx[r];
            const float rw = s_rw[r];
            v4f y;
            if constexpr (STAGE == 1) {
                const acc_t ag = acc[mi][0][ni], au = acc[mi][NSET - 1][ni];
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const float g = ((float)ag[v] * sx) * swa[v], u = ((float)au[v] * sx) * swb[v];
                    y[v] = silu(g) * u * rw;
                }
            } else {
                const acc_t a = acc[mi][0][ni];
#pragma unroll
                for (int v = 0; v < 4; v++) y[v] = (((float)a[v] * sx) * swa[v]) * rw;
            }
            const int cb = (wave * 16 + lg * 4) * esize;      // byte column inside the pass's row
            uint8_t* dst = stage + r * row_bytes + ((((cb >> 4) ^ r) & gmask) << 4) + (cb & 15);
            if (f32_out) {
                *reinterpret_cast<v4f*>(dst) = y;
            } else {
                *reinterpret_cast<v2i*>(dst) = p.out_dtype == OUT_BF16 ? pack4_out16<OUT_BF16>(y[0], y[1], y[2], y[3]) : pack4_out16<OUT_FP16>(y[0], y[1], y[2], y[3]);
            }
        });
        __syncthreads();
        const bool atomic = STAGE == 2 && p.accumulate;
        const int unit = atomic ? 4 : 16;                      // bytes one thread moves per trip
        const int upr = row_bytes / unit;                      // units per row
        for (int q = tid; q < BM * upr; q += 256) {
            const int r = q / upr, cb = (q % upr) * unit;
            const int n = n0 + ni * 64 + cb / esize;
            const uint32_t sid = (uint32_t)ids[r];
            const int t = (int)(sid & 0xFFFFFFu), slot = (int)(sid >> 24);
            if (t < p.tokens && slot < p.topk && n < p.n_out) {
                const uint8_t* src = stage + r * row_bytes + ((((cb >> 4) ^ r) & gmask) << 4) + (cb & 15);
                const size_t orow = atomic ? (size_t)t : (size_t)t * p.topk + slot;
                uint8_t* o = static_cast<uint8_t*>(p.out) + (orow * (size_t)p.n_out + n) * esize;
                if (!atomic) {
                    *reinterpret_cast<v4i*>(o) = *reinterpret_cast<const v4i*>(src);
                } else if (f32_out) {
                    unsafeAtomicAdd(reinterpret_cast<float*>(o), *reinterpret_cast<const float*>(src));
                } else if (p.out_dtype == OUT_FP16) {
                    __builtin_amdgcn_global_atomic_fadd_v2f16((__attribute__((address_space(1))) v2h*)o, *reinterpret_cast<const v2h*>(src));
                } else {
                    __builtin_amdgcn_global_atomic_fadd_v2bf16((__attribute__((address_space(1))) v2b*)o, *reinterpret_cast<const v2b*>(src));
                }
            }
        }
        if constexpr (ni + 1 < NR) __syncthreads();
    });
}

template <int KIND, int STAGE, int NR>
hipError_t launch_nr(const MoeParams& p, int block_m, int blocks, bool pair, hipStream_t stream) {
    const dim3 grid((p.n_out + 64 * NR - 1) / (64 * NR), blocks, 1);
#define PSG_MOE(MR_, CO_)                                                                                \
    {                                                                                                    \
        hipLaunchKernelGGL((k_moe_gemm<KIND, MR_, NR, STAGE, CO_>), grid, dim3(256), 0, stream, p);     \
        return hipGetLastError();                                                                        \
    }
    if (pair && block_m == 16) PSG_MOE(2, 2)
    if (pair && block_m == 32) PSG_MOE(4, 2)
    if (block_m == 16) PSG_MOE(1, 1)
    if (block_m == 32) PSG_MOE(2, 1)
    if (block_m == 64) PSG_MOE(4, 1)
    if (block_m == 128) PSG_MOE(8, 1)
#undef PSG_MOE
    return hipErrorInvalidValue;
}

template <int KIND, int STAGE>
hipError_t launch_kind(const MoeParams& p, int block_m, int blocks, hipStream_t stream) {
    // Stage 1 with one-byte weights multiplies blocks of 16 and 32 rows two at a time where they share an expert (64 tokens x
    // top-8 on 32 experts, blocks of 16: 107 -> 92 us).  Measured and left alone: stage 2 (34 -> 37 us: its second pass over an
    // expert's smaller slab already hits in L2, and pairing halves the workgroups in flight) and packed int4 weights (49 -> 50).
    const bool pair = block_m <= 32 && p.pair_blocks != 0 && STAGE == 1 && KIND != KIND_INT8W4;
    const int tile_m = pair ? 2 * block_m : block_m;
    // 128 columns per workgroup when they divide the output; stage 1 (two accumulator sets) only for tiles of up to 32
    // rows: measured at 4096 tokens x top-8, blocks of 128: stage 1 488 us with 64 columns against 800 with 128, stage 2
    // 442 against 412 (stage 2 with 256 columns: 805 with one workgroup per CU, 492 when held to two)
    // ... and only when that still leaves several workgroups per CU: a workgroup streams its slab at the pace its loads in
    // flight allow, so a decode-sized stage 1 (64 tokens x top-8 on 32 experts: at most 63 blocks x 12 column tiles) is faster
    // with twice as many workgroups of half the width
    const long wgs128 = (long)blocks / (pair ? 2 : 1) * (long)(p.n_out / 128);
    if (p.n_out % 128 == 0 && (STAGE == 2 || (tile_m <= 32 && wgs128 >= 1024))) return launch_nr<KIND, STAGE, 2>(p, block_m, blocks, pair, stream);
    return launch_nr<KIND, STAGE, 1>(p, block_m, blocks, pair, stream);
}

}  // namespace

// kind: KIND_INT8 / KIND_FP8 / KIND_INT8W4; stage 1 or 2; block_m in {16, 32, 64, 128}; blocks = entries of expert_ids
hipError_t psg_launch_moe_gemm(const MoeParams& p, int kind, int stage, int block_m, int blocks, hipStream_t stream) {
    if (kind == KIND_INT8) return stage == 1 ? launch_kind<KIND_INT8, 1>(p, block_m, blocks, stream) : launch_kind<KIND_INT8, 2>(p, block_m, blocks, stream);
    if (kind == KIND_INT8W4) return stage == 1 ? launch_kind<KIND_INT8W4, 1>(p, block_m, blocks, stream) : launch_kind<KIND_INT8W4, 2>(p, block_m, blocks, stream);
    return stage == 1 ? launch_kind<KIND_FP8, 1>(p, block_m, blocks, stream) : launch_kind<KIND_FP8, 2>(p, block_m, blocks, stream);
}

// sum over the topk slots: y[t, :] = sum_s x[t, s, :] (bf16, fp16 or fp32, the same type in and out; fp32 sum in slot order)
namespace {
// mask != nullptr: slot k of token t only counts when mask[ids[t*topk + k]] != 0 (expert parallelism: the rows of experts
// that live elsewhere were never written by stage 2)
__global__ void __launch_bounds__(256) k_moe_reduce(const uint16_t* x, uint16_t* y, int tokens, int topk, int dim, int out_dtype,
                                                    const int32_t* mask, const int32_t* ids, int experts) {
    const size_t q = (size_t)blockIdx.x * 256 + threadIdx.x;   // one thread per 4 columns
    const size_t quads = (size_t)tokens * (size_t)(dim >> 2);
    if (q >= quads) return;
    const size_t t = q / (size_t)(dim >> 2), c = (q % (size_t)(dim >> 2)) << 2;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    for (int k = 0; k < topk; k++) {
        if (mask) {
            const int e = ids[t * topk + k];
            if ((unsigned)e >= (unsigned)experts || mask[e] == 0) continue;
        }
        if (out_dtype == OUT_F32) {
            const v4f v = *reinterpret_cast<const v4f*>(reinterpret_cast<const float*>(x) + (t * topk + k) * (size_t)dim + c);
            s0 += v[0]; s1 += v[1]; s2 += v[2]; s3 += v[3];
            continue;
        }
        const v2i v = *reinterpret_cast<const v2i*>(x + (t * topk + k) * (size_t)dim + c);
        const uint16_t h0 = (uint16_t)(v[0] & 0xFFFF), h1 = (uint16_t)((uint32_t)v[0] >> 16), h2 = (uint16_t)(v[1] & 0xFFFF), h3 = (uint16_t)((uint32_t)v[1] >> 16);
        if (out_dtype == OUT_BF16) {
            s0 += from_out16<OUT_BF16>(h0); s1 += from_out16<OUT_BF16>(h1); s2 += from_out16<OUT_BF16>(h2); s3 += from_out16<OUT_BF16>(h3);
        } else {
            s0 += from_out16<OUT_FP16>(h0); s1 += from_out16<OUT_FP16>(h1); s2 += from_out16<OUT_FP16>(h2); s3 += from_out16<OUT_FP16>(h3);
        }
    }
    if (out_dtype == OUT_F32) {
        *reinterpret_cast<v4f*>(reinterpret_cast<float*>(y) + t * (size_t)dim + c) = (v4f){s0, s1, s2, s3};
        return;
    }
    const v2i o = out_dtype == OUT_BF16 ? pack4_out16<OUT_BF16>(s0, s1, s2, s3) : pack4_out16<OUT_FP16>(s0, s1, s2, s3);
    *reinterpret_cast<v2i*>(y + t * (size_t)dim + c) = o;
}
}  // namespace

hipError_t psg_launch_moe_reduce(const void* x, void* y, int tokens, int topk, int dim, int out_dtype, const int32_t* mask,
                                 const int32_t* ids, int experts, hipStream_t stream) {
    const size_t quads = (size_t)tokens * (size_t)(dim >> 2);
    hipLaunchKernelGGL(k_moe_reduce, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, stream, static_cast<const uint16_t*>(x),
                       static_cast<uint16_t*>(y), tokens, topk, dim, out_dtype, mask, ids, experts);
    return hipGetLastError();
}
