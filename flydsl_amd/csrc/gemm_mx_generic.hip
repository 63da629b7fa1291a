// General MX preshuffle GEMM for gfx950: A in fp4 (e2m1), fp6 (e2m3) or fp8 (e4m3), W in fp4 or fp8, one e8m0 scale per
// 32 K elements on both sides, strided-batched over blockIdx.z with caller-chosen row / batch strides.  This is the
// path for everything the fp4 x fp4 kernels (gemm_tiled.h, gemm_mxfp4.hip) do not cover; it favours generality over
// the last bit of speed (4 wavefronts side by side along N, one 128-element K step per iteration, A through LDS).
//
// v_mfma_scale_f32_16x16x128_f8f6f4, lane (i = lane%16, g = lane/16), one 128-element K step:
//   fp4 / fp6 operands: the lane supplies row i's 32 elements [32g, 32g+32) (4 or 6 dwords).
//   fp8 operands:       the lane supplies row i's elements [16g, 16g+16) (dwords 0-3) and [64+16g, 64+16g+16)
//                       (dwords 4-7).
//   scales:             the lane's scale byte is row i's scale for elements [32g, 32g+32), whatever the format.
//   A fp4: 16 bytes at byte 16g of the row's 64-byte step; fp6: the 32-byte group g of its 128-byte step, of which
//          the first 24 bytes hold the 32 packed 6-bit codes; fp8: the 16-byte pieces g and 4+g of its 128-byte step.
//   W fp4: one preshuffled 1 KB block (n-block, 64-byte K block kt) is one operand (lane l reads bytes [16l, 16l+16)).
//   W fp8: the 128-byte step is two 1 KB blocks (64-byte K blocks 2kt, 2kt+1); the lane reads bytes [16l, 16l+16) of
//          each.
//   Scales: the shuffled layout stores per (32-row chunk, 256-K chunk) 64 dwords; lane l's dword holds the bytes
//          (128-K half kh, 16-row half h) -> byte 2*kh + h, selected with the MFMA's op_sel; kh = K step parity.
// Operands are swapped (src0 = W, src1 = A) so a lane ends up with 4 consecutive N columns of one row.
#include "psg_common.h"

namespace {

template <int F>
struct MxCode {  // cbsz / blgp format code of the MFMA
    static constexpr int value = F == MXF_FP4 ? 4 : (F == MXF_FP6 ? 2 : 0);
};

template <int AF, int BF, int MR, int NR, int STORE>
__global__ void __launch_bounds__(256) k_mx_generic(MxGenParams p) {
    static_assert(MR % 2 == 0 && NR % 2 == 0, "scale chunks cover 32 rows");
    constexpr int TM = 16 * MR, TN = 64 * NR;
    constexpr int AB = AF == MXF_FP4 ? 64 : 128;   // bytes of an A row per K step
    constexpr int CPR = AB / 16;                   // 16-byte chunks per staged row
    constexpr int A_LOADS = (TM * CPR + 255) / 256;
    constexpr int BW = BF == MXF_FP4 ? 1 : 2;      // 16-byte loads per W operand
    __shared__ __attribute__((aligned(16))) uint8_t lds[2][TM * AB];

    const int tid = threadIdx.x;
    const int wave = wave_id();
    const int lane = tid & 63, li = lane & 15, lg = lane >> 4;
    const int tiles_n = (p.N + TN - 1) / TN;
    const int m0 = ((int)blockIdx.x / tiles_n) * TM, n0 = ((int)blockIdx.x % tiles_n) * TN;
    const uint64_t z = blockIdx.z;
    const int KT = p.K >> 7;                                   // 128-element steps (even: K % 256 == 0)
    // split-K: workgroup blockIdx.y of p.splits covers the steps [kt_begin, kt_end), a whole number of 256-K scale chunks,
    // and (STORE_ACC only) writes its accumulators to slice blockIdx.y of the partials buffer
    const int kt_per = (((KT >> 1) + p.splits - 1) / p.splits) << 1;
    const int kt_begin = (int)blockIdx.y * kt_per;
    const int kt_end = (kt_begin + kt_per) < KT ? (kt_begin + kt_per) : KT;
    const uint32_t a_row_bytes = AF == MXF_FP4 ? (uint32_t)p.K >> 1 : (uint32_t)p.K;
    const uint32_t b_row_bytes = BF == MXF_FP4 ? (uint32_t)p.K >> 1 : (uint32_t)p.K;
    const uint32_t a_rs = (uint32_t)p.a_row_stride;
    const uint32_t chunk_bytes = (uint32_t)(p.K >> 8) * 256u;  // one 32-row chunk of shuffled scales

    // A: this tile's rows, bounded to the last valid row (rows >= M read as zero)
    const int rows_left = p.M - m0;
    __amdgpu_buffer_rsrc_t ra = make_rsrc(p.a + z * (uint64_t)p.a_batch + (uint64_t)m0 * a_rs,
                                          rows_left > 0 ? (uint64_t)(rows_left - 1) * a_rs + a_row_bytes : 0);
    // W: this wavefront's NR n-blocks; blocks >= N/16 read as zero
    const int nb0 = (n0 >> 4) + wave * NR;
    const uint64_t b_total = (uint64_t)p.N * b_row_bytes, b_off = (uint64_t)nb0 * 16ull * b_row_bytes;
    __amdgpu_buffer_rsrc_t rb = make_rsrc(p.b + z * (uint64_t)p.b_batch + (b_off < b_total ? b_off : b_total), b_off < b_total ? b_total - b_off : 0);
    // scales: A-side chunks of the tile, W-side chunks of this wavefront; chunks past the end read as zero (2^-127,
    // multiplied by operands that are zero too)
    const int sa_chunks = (p.M + 31) >> 5, sa_first = m0 >> 5;
    const uint32_t sa_cs = (uint32_t)p.sa_chunk_stride;
    __amdgpu_buffer_rsrc_t rsa = make_rsrc(p.sa + z * (uint64_t)p.sa_batch + (uint64_t)(sa_first < sa_chunks ? sa_first : sa_chunks) * sa_cs,
                                           sa_first < sa_chunks ? (uint64_t)(sa_chunks - sa_first - 1) * sa_cs + chunk_bytes : 0);
    const int sb_chunks = p.N >> 5, sb_first = (n0 >> 5) + wave * (NR / 2);
    __amdgpu_buffer_rsrc_t rsb = make_rsrc(p.sb + z * (uint64_t)p.sb_batch + (uint64_t)(sb_first < sb_chunks ? sb_first : sb_chunks) * chunk_bytes,
                                           sb_first < sb_chunks ? (uint64_t)(sb_chunks - sb_first) * chunk_bytes : 0);

    // LDS: row-major AB-byte rows, the 16-byte chunk index XORed with row / 2: eight consecutive lanes of a 16-byte access then
    // cover eight different 16-byte slots of a 128-byte bank row, for 64-byte rows too (with row / 4 the rows r and r + 2 met in
    // one slot: 16.2 M conflict cycles per launch of the 4096-token MoE stage 1 against 2.9 M)
    auto lds_off = [&](int row, int c) { return row * AB + ((c ^ ((row >> 1) & (CPR - 1))) << 4); };
    // Operands are requested PF steps ahead of their MFMAs in rings of RING register sets (small tiles: a K step is a few hundred
    // MFMA cycles per wavefront, far below the latency of a load; the 128 x 256 tile needs its registers for accumulators)
    constexpr int RING = MR * NR <= 8 ? 4 : 2, PF = RING - 1;
    v4i areg[RING][A_LOADS];
    auto load_a = [&](int kt, v4i* dst) {
#pragma unroll
        for (int j = 0; j < A_LOADS; j++) {
            const int c = tid + 256 * j, row = c / CPR, kc = c % CPR;
            const bool ok = row < TM && kt < kt_end;
            dst[j] = buf_load16(ra, ok ? (uint32_t)row * a_rs + (uint32_t)kc * 16u : 0xFFFFFFF0u, ok ? (uint32_t)kt * AB : 0u);
        }
    };
    auto store_a = [&](int stage, const v4i* src) {
#pragma unroll
        for (int j = 0; j < A_LOADS; j++) {
            const int c = tid + 256 * j, row = c / CPR, kc = c % CPR;
            if (row < TM) *reinterpret_cast<v4i*>(&lds[stage][lds_off(row, kc)]) = src[j];
        }
    };
    // W operand of n-block ni for step kt -> 8 dwords (fp4 uses the low four)
    v8i bw[RING][NR];
    auto load_b = [&](int kt, v8i* dst) {
#pragma unroll
        for (int ni = 0; ni < NR; ni++) {
            const bool ok = kt < kt_end;
            v8i v = {0, 0, 0, 0, 0, 0, 0, 0};
            if constexpr (BF == MXF_FP4) {
                const v4i x = buf_load16(rb, ok ? (uint32_t)lane * 16u + (uint32_t)ni * 16u * b_row_bytes : 0xFFFFFFF0u, ok ? (uint32_t)kt * 1024u : 0u);
                v = __builtin_shufflevector(x, x, 0, 1, 2, 3, -1, -1, -1, -1);
            } else {
                const uint32_t voff = (uint32_t)lane * 16u + (uint32_t)ni * 16u * b_row_bytes;
                const v4i x0 = buf_load16(rb, ok ? voff : 0xFFFFFFF0u, ok ? (uint32_t)kt * 2048u : 0u);
                const v4i x1 = buf_load16(rb, ok ? voff + 1024u : 0xFFFFFFF0u, ok ? (uint32_t)kt * 2048u : 0u);
                v = __builtin_shufflevector(x0, x1, 0, 1, 2, 3, 4, 5, 6, 7);
            }
            dst[ni] = v;
        }
    };
    // scale dwords of a 256-K chunk kc: MR/2 on the A side, NR/2 on the W side
    int sav[2][MR / 2], sbv[2][NR / 2];
    auto load_sc = [&](int kc, int* sa_dst, int* sb_dst) {
        const bool ok = kc < (kt_end >> 1);
#pragma unroll
        for (int q = 0; q < MR / 2; q++) sa_dst[q] = buf_load4(rsa, ok ? (uint32_t)q * sa_cs + (uint32_t)lane * 4u : 0xFFFFFFF0u, ok ? (uint32_t)kc * 256u : 0u);
#pragma unroll
        for (int q = 0; q < NR / 2; q++) sb_dst[q] = buf_load4(rsb, ok ? (uint32_t)q * chunk_bytes + (uint32_t)lane * 4u : 0xFFFFFFF0u, ok ? (uint32_t)kc * 256u : 0u);
    };
    auto read_frag = [&](int stage, int mi) {
        const int row = mi * 16 + li;
        v8i v = {0, 0, 0, 0, 0, 0, 0, 0};
        if constexpr (AF == MXF_FP4) {
            const v4i x = *reinterpret_cast<const v4i*>(&lds[stage][lds_off(row, lg)]);
            v = __builtin_shufflevector(x, x, 0, 1, 2, 3, -1, -1, -1, -1);
        } else {
            constexpr bool F8 = AF == MXF_FP8;
            const v4i x0 = *reinterpret_cast<const v4i*>(&lds[stage][lds_off(row, F8 ? lg : 2 * lg)]);
            const v4i x1 = *reinterpret_cast<const v4i*>(&lds[stage][lds_off(row, F8 ? 4 + lg : 2 * lg + 1)]);
            v = __builtin_shufflevector(x0, x1, 0, 1, 2, 3, 4, 5, 6, 7);  // fp6 uses the first six dwords
        }
        return v;
    };

    v4f acc[MR][NR];
#pragma unroll
    for (int mi = 0; mi < MR; mi++)
#pragma unroll
        for (int ni = 0; ni < NR; ni++) acc[mi][ni] = (v4f){0.f, 0.f, 0.f, 0.f};

    // One K step of parity KH (= 128-K half of the current scale chunk): MFMAs on LDS stage KH, W set WS = step % RING and the
    // scale set SET (scale chunks alternate between the two sets); requests the operands of step kt + PF and, in the first half of
    // a chunk, the scales of the next one; stages the A rows of step kt + 1
    auto step = [&](int kt, auto KHP, auto SETP, auto WSP) __attribute__((always_inline)) {
        constexpr int KH = decltype(KHP)::value, SET = decltype(SETP)::value, WS = decltype(WSP)::value;
        load_a(kt + PF, areg[(WS + PF) % RING]);
        load_b(kt + PF, bw[(WS + PF) % RING]);
        if constexpr (KH == 0) load_sc((kt >> 1) + 1, sav[SET ^ 1], sbv[SET ^ 1]);
        const int* sa_cur = sav[SET];
        const int* sb_cur = sbv[SET];
        static_for<MR>([&](auto MI) {
            constexpr int mi = decltype(MI)::value;
            const v8i af = read_frag(KH, mi);
            static_for<NR>([&](auto NI) {
                constexpr int ni = decltype(NI)::value;
                acc[mi][ni] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bw[WS][ni], af, acc[mi][ni], MxCode<BF>::value, MxCode<AF>::value,
                                                                              KH * 2 + (ni & 1), sb_cur[ni / 2], KH * 2 + (mi & 1), sa_cur[mi / 2]);
            });
        });
        store_a(KH ^ 1, areg[(WS + 1) % RING]);
        __syncthreads();
    };

    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2 % RING>;
    using I3 = std::integral_constant<int, 3 % RING>;
#pragma unroll
    for (int i = 0; i < PF; i++) {
        load_a(kt_begin + i, areg[i]);
        load_b(kt_begin + i, bw[i]);
    }
    load_sc(kt_begin >> 1, sav[0], sbv[0]);
    store_a(0, areg[0]);
    __syncthreads();
    for (int kt = kt_begin; kt < kt_end; kt += 4) {  // two scale chunks per trip, so every register index is a constant
        step(kt, I0{}, I0{}, I0{});
        step(kt + 1, I1{}, I0{}, I1{});
        if (kt + 2 < kt_end) {
            step(kt + 2, I0{}, I1{}, I2{});
            step(kt + 3, I1{}, I1{}, I3{});
        }
    }

    const int64_t c_rs = p.c_row_stride;
    uint8_t* cbase = static_cast<uint8_t*>(p.c) + z * (uint64_t)p.c_batch;
#pragma unroll
    for (int mi = 0; mi < MR; mi++) {
        const int m = m0 + mi * 16 + li;
#pragma unroll
        for (int ni = 0; ni < NR; ni++) {
            const int n = n0 + (wave * NR + ni) * 16 + lg * 4;
            if (m < p.M && n < p.N) {
                const v4f v = acc[mi][ni];
                if constexpr (STORE == STORE_ACC) {
                    const size_t slice = (size_t)blockIdx.y * (size_t)p.M * (size_t)p.N;
                    *reinterpret_cast<v4f*>(reinterpret_cast<float*>(cbase) + slice + (size_t)m * (size_t)p.N + (size_t)n) = v;
                } else {
                    const v2i r = p.out == OUT_BF16 ? pack4_out16<OUT_BF16>(v[0], v[1], v[2], v[3]) : pack4_out16<OUT_FP16>(v[0], v[1], v[2], v[3]);
                    *reinterpret_cast<v2i*>(reinterpret_cast<uint16_t*>(cbase) + (int64_t)m * c_rs + n) = r;
                }
            }
        }
    }
}

template <int AF, int BF, int STORE>
hipError_t launch_fmt(const MxGenParams& p, int batch, hipStream_t stream) {
    // 32x128 tiles for M <= 32, 128x256 when those alone give every CU a workgroup, else 64x128
    const int splits = STORE == STORE_ACC && p.splits > 1 ? p.splits : 1;
    if (p.M <= 32) {
        const int tiles = ((p.M + 31) / 32) * ((p.N + 127) / 128);
        hipLaunchKernelGGL((k_mx_generic<AF, BF, 2, 2, STORE>), dim3(tiles, splits, batch), dim3(256), 0, stream, p);
    } else if ((long)((p.M + 127) / 128) * (long)((p.N + 255) / 256) * batch >= 256 && splits == 1) {
        const int tiles = ((p.M + 127) / 128) * ((p.N + 255) / 256);
        hipLaunchKernelGGL((k_mx_generic<AF, BF, 8, 4, STORE>), dim3(tiles, 1, batch), dim3(256), 0, stream, p);
    } else {
        const int tiles = ((p.M + 63) / 64) * ((p.N + 127) / 128);
        hipLaunchKernelGGL((k_mx_generic<AF, BF, 4, 2, STORE>), dim3(tiles, splits, batch), dim3(256), 0, stream, p);
    }
    return hipGetLastError();
}

template <int STORE>
hipError_t launch_store(const MxGenParams& p, int af, int bf, int batch, hipStream_t stream) {
    if (bf == MXF_FP4) {
        if (af == MXF_FP4) return launch_fmt<MXF_FP4, MXF_FP4, STORE>(p, batch, stream);
        if (af == MXF_FP6) return launch_fmt<MXF_FP6, MXF_FP4, STORE>(p, batch, stream);
        return launch_fmt<MXF_FP8, MXF_FP4, STORE>(p, batch, stream);
    }
    if (af == MXF_FP4) return launch_fmt<MXF_FP4, MXF_FP8, STORE>(p, batch, stream);
    if (af == MXF_FP6) return launch_fmt<MXF_FP6, MXF_FP8, STORE>(p, batch, stream);
    return launch_fmt<MXF_FP8, MXF_FP8, STORE>(p, batch, stream);
}

}  // namespace

// af: MXF_FP4 / MXF_FP6 / MXF_FP8; bf: MXF_FP4 / MXF_FP8; batch >= 1 (grid.z <= 65535)
hipError_t psg_launch_mx_generic(const MxGenParams& p, int af, int bf, int store, int batch, hipStream_t stream) {
    return store == STORE_ACC ? launch_store<STORE_ACC>(p, af, bf, batch, stream) : launch_store<STORE_C>(p, af, bf, batch, stream);
}
