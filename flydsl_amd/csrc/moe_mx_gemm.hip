// MoE grouped GEMMs with MX operands for gfx950: activations in fp4 (e2m1) or fp8 (e4m3), expert weights in fp4, one e8m0
// scale per 32 K elements on both sides (v_mfma_scale_f32_16x16x128_f8f6f4), over blocks of sorted token rows that all
// belong to one expert.
//   stage 1 (gate-up): g = a[t] . W1[e, n], u = a[t] . W1[e, inter + n]; y = silu(g) * u; y is quantised again per 32 columns
//                      (scale byte = exponent of the smallest power of two >= amax / 6, e2m1 codes by nearest-even) and
//                      written by SORTED position: codes row-major, scales in the shuffled layout stage 2 reads.
//   stage 2 (down):    y[n] = a2[sorted row] . W2[e, n]; times the routing weight and added atomically into out[token], or
//                      written unweighted to one row per sorted position.
// Operand layouts (lane l = 16 g + i of a wavefront, one 128-element K step):
//   A fp4: row i's 16 bytes at byte 16 g of its 64-byte step; fp8: the 16-byte pieces g and 4 + g of its 128-byte step.
//   W: one preshuffled 1 KB block (16 rows x 64 bytes) is one operand: lane l reads bytes [16 l, 16 l + 16).
//   Scales: per (32-row chunk, 256-K chunk) 64 dwords; lane l's dword holds the bytes (128-K half kh, 16-row half h) at
//           byte 2 kh + h, selected with the MFMA's op_sel.  The A-side chunks count SORTED rows.
// Operands are swapped (src0 = W, src1 = A) so a lane ends up with 4 consecutive columns of one row.  Four wavefronts side
// by side along N; each covers 64 W rows: in stage 1 32 gate rows and the 32 up rows of the same columns, so a wavefront
// owns whole 32-column quantisation groups.
#include "psg_common.h"

namespace {

typedef __fp16 v2h __attribute__((ext_vector_type(2)));
typedef __bf16 v2b __attribute__((ext_vector_type(2)));

// adds the two 16-bit values packed in `bits` to o[0], o[1]
template <int OUT>
__device__ __forceinline__ void atomic_add2(uint16_t* o, int bits) {
    if constexpr (OUT == OUT_BF16) __builtin_amdgcn_global_atomic_fadd_v2bf16((__attribute__((address_space(1))) v2b*)o, __builtin_bit_cast(v2b, bits));
    else __builtin_amdgcn_global_atomic_fadd_v2f16((__attribute__((address_space(1))) v2h*)o, __builtin_bit_cast(v2h, bits));
}

// Scale byte of a 32-element group with maximum amax: exponent of the smallest power of two >= amax / 6, at most 254
__device__ __forceinline__ uint32_t scale_byte(float amax) {
    const uint32_t b = ((__float_as_uint(amax * (1.0f / 6.0f)) + 0x7FFFFFu) >> 23) & 0xFFu;
    return b < 254u ? b : 254u;
}

// Eight values of a group -> their e2m1 codes (first value in the lowest nibble) at the group's scale
__device__ __forceinline__ int codes8(const float* x, uint32_t bexp) {
    const float sf = bexp ? __uint_as_float(bexp << 23) : 1.0f;
    int word = 0;
    word = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(word, x[0], x[1], sf, 0);
    word = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(word, x[2], x[3], sf, 1);
    word = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(word, x[4], x[5], sf, 2);
    word = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(word, x[6], x[7], sf, 3);
    return word;
}

// Eight bf16 of a 32-element group that four neighbouring lanes hold together -> this lane's codes, the group's scale byte
__device__ __forceinline__ int quant_group_bf16(const v4i src, uint32_t& bexp) {
    float x[8];
    float amax = 0.f;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        x[2 * j] = __uint_as_float((uint32_t)src[j] << 16);
        x[2 * j + 1] = __uint_as_float((uint32_t)src[j] & 0xFFFF0000u);
        amax = fmaxf(amax, fmaxf(fabsf(x[2 * j]), fabsf(x[2 * j + 1])));
    }
    amax = fmaxf(amax, __uint_as_float(__builtin_amdgcn_update_dpp(0, __float_as_uint(amax), 0xB1, 0xF, 0xF, true)));
    amax = fmaxf(amax, __uint_as_float(__builtin_amdgcn_update_dpp(0, __float_as_uint(amax), 0x4E, 0xF, 0xF, true)));
    bexp = scale_byte(amax);
    return codes8(x, bexp);
}

// silu(gate) * up of this lane's eight columns of a 32-column group spread over the lanes l, l^16, l^32, l^48 -> codes, scale byte
__device__ __forceinline__ int quant_silu_mul(const v4f g0, const v4f g1, const v4f u0, const v4f u1, uint32_t& bexp) {
    float y[8];
    float amax = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const float g = j < 4 ? g0[j & 3] : g1[j & 3], u = j < 4 ? u0[j & 3] : u1[j & 3];
        const float sig = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g * -1.4426950408889634f));
        y[j] = g * sig * u;
        amax = fmaxf(amax, fabsf(y[j]));
    }
    amax = fmaxf(amax, __shfl_xor(amax, 16));
    amax = fmaxf(amax, __shfl_xor(amax, 32));
    bexp = scale_byte(amax);
    return codes8(y, bexp);
}

// IQ (stage 1, 16-row blocks): `a` holds bf16 activations [tokens, K]; every 32 of them are quantised to fp4 on their way into
// LDS with the same scale rule as the output (kernels/moe/mxfp_moe/gemm1.py:324-412), and no A-side scales are read.  (A variant
// that first quantised all K elements of the 16 rows into LDS and then ran the K loop without barriers measured slower: 16 tokens
// x top-8 on 32 experts 38.9 us against 35.4, 64 tokens 42.2 against 41.)
template <int AF, int MR, int STAGE, bool IQ = false>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(MR <= 4 ? 2 : 1))) k_moe_mx(MoeMxParams p) {
    static_assert(MR % 2 == 0 || MR == 1, "scale chunks cover 32 rows; a single 16-row block picks its half at run time");
    static_assert(!IQ || (MR == 1 && STAGE == 1 && AF == MXF_FP4), "inline quantisation: 16-row blocks of stage 1");
    constexpr int NR = 4;
    constexpr int TM = 16 * MR;
    constexpr int TN = STAGE == 1 ? 128 : 256;     // output columns per workgroup
    constexpr int AB = AF == MXF_FP4 ? 64 : 128;   // bytes of an A row per K step
    constexpr int CPR = AB / 16;                   // 16-byte chunks per staged row
    constexpr int A_LOADS = IQ ? 1 : (TM * CPR + 255) / 256;
    constexpr int SC = (MR + 1) / 2;               // A-side scale dwords per 256-K chunk
    constexpr int ACODE = AF == MXF_FP4 ? 4 : 0;
    constexpr int EPI_BYTES = TM * (STAGE == 1 ? 64 : 512);  // the epilogue's tile: TM rows of 64 code bytes or 256 16-bit values
    constexpr int LDS_BYTES = 2 * TM * AB > EPI_BYTES ? 2 * TM * AB : EPI_BYTES;
    __shared__ __attribute__((aligned(16))) uint8_t lds_raw[LDS_BYTES];
    __shared__ uint8_t iq_scale[2][IQ ? 64 : 1];   // IQ: scale byte of (row, 32-element group) of each LDS stage
    uint8_t(*lds)[TM * AB] = reinterpret_cast<uint8_t(*)[TM * AB]>(lds_raw);

    // Workgroup id -> (row block, column tile).  Consecutive ids go to the 8 XCDs in turn, each with an L2 of its own.
    // by_expert: slice (expert e, column tile t) of the weights belongs to XCD (e * n_tiles + t) % 8, so the few row blocks of an
    // expert read it through the same L2 (ids whose column tile does not exist leave at once); else ids simply count the tiles
    // row block by row block (a slice then alternates between 8 / gcd(8, n_tiles) XCDs).
    int blk, n_tile;
    if (p.by_expert) {
        const int wg_slot = (int)blockIdx.x >> 3;
        blk = wg_slot / p.n_groups;
        n_tile = wg_slot % p.n_groups * 8;
    } else if (p.quad_tiles) {
        // XCD x = id % 8 takes the row blocks of parity x / 4 and the column tiles t with t % 4 == x % 4: the tiles of a block meet in
        // four L2s instead of eight, a slice of the weights alternates between two
        const int x = (int)blockIdx.x & 7, s = (int)blockIdx.x >> 3, nq = p.n_tiles >> 2;
        blk = 2 * (s / nq) + (x >> 2);
        n_tile = (x & 3) + 4 * (s % nq);
    } else {
        blk = (int)blockIdx.x / p.n_tiles;  // block of TM sorted rows; the sorter's blocks hold TM << eshift rows
        n_tile = (int)blockIdx.x % p.n_tiles;
    }
    // the quad order rounds the row blocks up to an even number: the odd one out has no entry in expert_ids
    if ((blk >> p.eshift) >= p.blocks || blk * TM >= p.num_valid[0]) return;
    const int e = p.expert_ids[blk >> p.eshift];
    if ((unsigned)e >= (unsigned)p.experts) return;
    if (p.by_expert) n_tile += ((int)blockIdx.x - e * p.n_tiles) & 7;
    if (n_tile >= p.n_tiles) return;
    const int tid = threadIdx.x;
    const int wave = wave_id();
    const int lane = tid & 63, li = lane & 15, lg = lane >> 4;
    const int n0 = n_tile * TN;
    const int KT = p.K >> 7;  // 128-element steps (even: K % 256 == 0)
    const uint32_t a_row_bytes = AF == MXF_FP4 ? (uint32_t)p.K >> 1 : (uint32_t)p.K;
    const uint32_t b_row_bytes = (uint32_t)p.K >> 1;
    const uint32_t chunk_bytes = (uint32_t)(p.K >> 8) * 256u;  // one 32-row chunk of shuffled scales
    const int w_rows = STAGE == 1 ? 2 * p.n_out : p.n_out;     // rows of one expert's matrix

    // A: stage 1 gathers token rows, stage 2 reads the block's sorted rows; rows without a token read as zero
    const int a_rows = STAGE == 1 ? p.tokens : p.sorted_size;
    const uint32_t a_src_bytes = IQ ? (uint32_t)p.K * 2u : a_row_bytes;  // bytes of a row of `a`
    constexpr uint32_t A_STEP = IQ ? 256u : (uint32_t)AB;                // ... and of one K step of it
    __amdgpu_buffer_rsrc_t ra = make_rsrc(p.a, (uint64_t)a_rows * a_src_bytes);
    uint32_t arow[A_LOADS];
    // W and its scales: this expert's matrix; the wavefront's four n-blocks
    __amdgpu_buffer_rsrc_t rb = make_rsrc(p.w + (uint64_t)e * (uint64_t)w_rows * b_row_bytes, (uint64_t)w_rows * b_row_bytes);
    __amdgpu_buffer_rsrc_t rsb = make_rsrc(p.w_scale + (uint64_t)e * (uint64_t)(w_rows >> 5) * chunk_bytes, (uint64_t)(w_rows >> 5) * chunk_bytes);
    uint32_t boff[NR], sboff[NR / 2];
#pragma unroll
    for (int ni = 0; ni < NR; ni++) {
        const int nb = STAGE == 1 ? (ni >> 1) * (p.n_out >> 4) + (n0 >> 4) + wave * 2 + (ni & 1) : (n0 >> 4) + wave * 4 + ni;
        boff[ni] = (uint32_t)nb * 16u * b_row_bytes + (uint32_t)lane * 16u;
    }
#pragma unroll
    for (int q = 0; q < NR / 2; q++) {
        const int ch = STAGE == 1 ? q * (p.n_out >> 5) + (n0 >> 5) + wave : (n0 >> 5) + wave * 2 + q;
        sboff[q] = (uint32_t)ch * chunk_bytes + (uint32_t)lane * 4u;
    }
    __amdgpu_buffer_rsrc_t rsa = make_rsrc(IQ ? p.w_scale : p.a_scale + (uint64_t)((blk * TM) >> 5) * chunk_bytes, IQ ? 0 : (uint64_t)SC * chunk_bytes);
    const int sa_shift = MR == 1 ? ((blk * TM) >> 4 & 1) * 8 : 0;  // a 16-row block in the upper half of its 32-row scale chunk

    // LDS: row-major AB-byte rows, the 16-byte chunk index XORed with row / 2: eight consecutive lanes of a 16-byte access then
    // cover eight different 16-byte slots of a 128-byte bank row, for 64-byte rows too (with row / 4 the rows r and r + 2 met in
    // one slot: 16.2 M conflict cycles per launch of the 4096-token MoE stage 1 against 2.9 M)
    auto lds_off = [&](int row, int c) { return row * AB + ((c ^ ((row >> 1) & (CPR - 1))) << 4); };
    // Loads run PF steps ahead of the MFMAs in rings of RING register sets: one step of a 64-row tile is 256 MFMA cycles per
    // wavefront, far less than the latency of a load from HBM
    constexpr int RING = AF == MXF_FP4 ? 4 : 2, PF = RING - 1;
    v4i areg[RING][A_LOADS];
    auto load_a = [&](int kt, v4i* dst) {
        const bool ok = kt < KT;
#pragma unroll
        for (int j = 0; j < A_LOADS; j++) dst[j] = buf_load16(ra, ok ? arow[j] : 0xFFFFFFF0u, ok ? (uint32_t)kt * A_STEP : 0u);
    };
    auto store_a = [&](int stage, const v4i* src) {
        if constexpr (IQ) {
            // 8 bf16 -> block maximum over the four lanes of the group -> scale byte -> 8 fp4 codes = one dword of the row's step
            uint32_t bexp;
            const int word = quant_group_bf16(src[0], bexp);
            const int row = tid >> 4, grp = (tid >> 2) & 3, q = tid & 3;
            *reinterpret_cast<int*>(&lds[stage][lds_off(row, grp) + q * 4]) = word;
            if (q == 0) iq_scale[stage][row * 4 + grp] = (uint8_t)bexp;
            return;
        }
#pragma unroll
        for (int j = 0; j < A_LOADS; j++) {
            const int c = tid + 256 * j, row = c / CPR, kc = c % CPR;
            if (row < TM) *reinterpret_cast<v4i*>(&lds[stage][lds_off(row, kc)]) = src[j];
        }
    };
    v4i bw[RING][NR];
    auto load_b = [&](int kt, v4i* dst) {
        const bool ok = kt < KT;
#pragma unroll
        for (int ni = 0; ni < NR; ni++) dst[ni] = buf_load16(rb, ok ? boff[ni] : 0xFFFFFFF0u, ok ? (uint32_t)kt * 1024u : 0u);
    };
    int sav[2][SC], sbv[2][NR / 2];
    auto load_sc = [&](int kc, int* sa_dst, int* sb_dst) {
        const bool ok = kc < (KT >> 1);
#pragma unroll
        for (int q = 0; q < SC; q++)
            sa_dst[q] = IQ ? 0 : buf_load4(rsa, ok ? (uint32_t)q * chunk_bytes + (uint32_t)lane * 4u : 0xFFFFFFF0u, ok ? (uint32_t)kc * 256u : 0u) >> sa_shift;
#pragma unroll
        for (int q = 0; q < NR / 2; q++) sb_dst[q] = buf_load4(rsb, ok ? sboff[q] : 0xFFFFFFF0u, ok ? (uint32_t)kc * 256u : 0u);
    };
    auto read_frag = [&](int stage, int mi) {
        const int row = mi * 16 + li;
        v8i v = {0, 0, 0, 0, 0, 0, 0, 0};
        if constexpr (AF == MXF_FP4) {
            const v4i x = *reinterpret_cast<const v4i*>(&lds[stage][lds_off(row, lg)]);
            v = __builtin_shufflevector(x, x, 0, 1, 2, 3, -1, -1, -1, -1);
        } else {
            const v4i x0 = *reinterpret_cast<const v4i*>(&lds[stage][lds_off(row, lg)]);
            const v4i x1 = *reinterpret_cast<const v4i*>(&lds[stage][lds_off(row, 4 + lg)]);
            v = __builtin_shufflevector(x0, x1, 0, 1, 2, 3, 4, 5, 6, 7);
        }
        return v;
    };

    v4f acc[MR][NR];
#pragma unroll
    for (int mi = 0; mi < MR; mi++)
#pragma unroll
        for (int ni = 0; ni < NR; ni++) acc[mi][ni] = (v4f){0.f, 0.f, 0.f, 0.f};

    // One K step of parity KH (= 128-K half of the current scale chunk): MFMAs on LDS stage KH, W set WS = kt % RING and scale
    // set SET; requests the operands of step kt + PF and the scales of the next chunk, stages the A rows of step kt + 1
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
            // A-side scale: IQ keeps the byte of (row, group) of this stage in LDS; a single 16-row block has shifted its half down
            const int sa_op = IQ ? (int)iq_scale[KH][li * 4 + lg] : sa_cur[mi / 2];
            constexpr int sa_sel = IQ ? 0 : KH * 2 + (MR == 1 ? 0 : (mi & 1));
            static_for<NR>([&](auto NI) {
                constexpr int ni = decltype(NI)::value;
                const v4i w4 = bw[WS][ni];
                const v8i wf = __builtin_shufflevector(w4, w4, 0, 1, 2, 3, -1, -1, -1, -1);
                acc[mi][ni] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, af, acc[mi][ni], 4, ACODE, KH * 2 + (ni & 1), sb_cur[ni / 2], sa_sel, sa_op);
            });
        });
        store_a(KH ^ 1, areg[(WS + 1) % RING]);
        __syncthreads();
    };

    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2 % RING>;
    using I3 = std::integral_constant<int, 3 % RING>;
    // the first W fragments are requested before the list of sorted rows is fetched: they only depend on the expert
#pragma unroll
    for (int i = 0; i < PF; i++) load_b(i, bw[i]);
#pragma unroll
    for (int j = 0; j < A_LOADS; j++) {
        // IQ: thread t takes 8 bf16 (16 bytes) of row t / 16: four neighbouring lanes hold one 32-element group
        const int c = tid + 256 * j, row = IQ ? c >> 4 : c / CPR, kc = IQ ? c & 15 : c % CPR;
        arow[j] = 0xFFFFFFF0u;
        if (row < TM) {
            const int src = STAGE == 1 ? (p.sorted_ids[blk * TM + row] & 0xFFFFFF) : blk * TM + row;
            if (src < a_rows) arow[j] = (uint32_t)src * a_src_bytes + (uint32_t)kc * 16u;
        }
    }
#pragma unroll
    for (int i = 0; i < PF; i++) load_a(i, areg[i]);
    load_sc(0, sav[0], sbv[0]);
    store_a(0, areg[0]);
    __syncthreads();
    for (int kt = 0; kt < KT; kt += 4) {  // two scale chunks per trip, so every register index is a constant
        step(kt, I0{}, I0{}, I0{});
        step(kt + 1, I1{}, I0{}, I1{});
        if (kt + 2 < KT) {
            step(kt + 2, I0{}, I1{}, I2{});
            step(kt + 3, I1{}, I1{}, I3{});
        }
    }

    if constexpr (STAGE == 1) {
        // lane (i, g) holds, for row mi*16 + i, gate and up of the columns n0 + wave*32 + ni*16 + 4g + [0, 4), ni = 0, 1:
        // the 32-column group of this wavefront is spread over the four lanes i, i+16, i+32, i+48
        const uint32_t out_row_bytes = (uint32_t)p.n_out >> 1;
        const uint32_t sc_chunk = (uint32_t)(p.n_out >> 8) * 256u;
        const int c32 = (n0 >> 5) + wave;  // scale column
        uint8_t* codes = static_cast<uint8_t*>(p.out);
#pragma unroll
        for (int mi = 0; mi < MR; mi++) {
            uint32_t bexp;
            const int word = quant_silu_mul(acc[mi][0], acc[mi][1], acc[mi][2], acc[mi][3], bexp);
            const int r = mi * 16 + li;
            const size_t sr = (size_t)blk * TM + r;
            // the tile's codes go through LDS (64 bytes per row, free after the loop's last barrier) so that they leave in 16-byte pieces
            uint8_t* dst = lds_raw + r * 64 + wave * 16 + lg * 2;
            *reinterpret_cast<uint16_t*>(dst) = (uint16_t)(word & 0xFFFF);
            *reinterpret_cast<uint16_t*>(dst + 8) = (uint16_t)((uint32_t)word >> 16);
            if (lg == 0) {
                const size_t off = ((sr >> 5) * (size_t)sc_chunk) + (size_t)(c32 >> 3) * 256u + (size_t)((c32 & 3) * 16 + li) * 4u + (size_t)(((c32 >> 2) & 1) * 2 + ((sr >> 4) & 1));
                p.out_scale[off] = (uint8_t)bexp;
            }
        }
        __syncthreads();
        for (int q = tid; q < TM * 4; q += 256) {
            const int r = q >> 2, c = q & 3;
            *reinterpret_cast<v4i*>(codes + ((size_t)blk * TM + r) * out_row_bytes + (uint32_t)((n0 >> 1) + c * 16)) = *reinterpret_cast<const v4i*>(lds_raw + r * 64 + c * 16);
        }
    } else {
        // The tile goes through LDS as 16-bit values (512 bytes per row, 16-byte granules XOR-swizzled by the row; the A stages are
        // free after the loop's last barrier); then the workgroup walks it row by row, so that one store or atomic instruction
        // covers 256 or 1024 contiguous bytes of the output instead of 16 rows x 8 bytes.
        const size_t N = (size_t)p.n_out;
        uint16_t* out = static_cast<uint16_t*>(p.out);
#pragma unroll
        for (int mi = 0; mi < MR; mi++) {
            const int r = mi * 16 + li;
            const float wgt = p.atomic ? p.sorted_w[blk * TM + r] : 1.0f;
#pragma unroll
            for (int ni = 0; ni < NR; ni++) {
                const int cb = ((wave * NR + ni) * 16 + lg * 4) * 2;
                const v4f v = acc[mi][ni] * wgt;
                const v2i pk = p.out_dtype == OUT_BF16 ? pack4_out16<OUT_BF16>(v[0], v[1], v[2], v[3]) : pack4_out16<OUT_FP16>(v[0], v[1], v[2], v[3]);
                *reinterpret_cast<v2i*>(lds_raw + r * 512 + ((((cb >> 4) ^ r) & 31) << 4) + (cb & 15)) = pk;
            }
        }
        __syncthreads();
        if (p.atomic) {
            for (int q = tid; q < TM * 128; q += 256) {
                const int r = q >> 7, cb = (q & 127) * 4;
                const int t = p.sorted_ids[blk * TM + r] & 0xFFFFFF;
                if (t >= p.tokens) continue;
                const int bits = *reinterpret_cast<const int*>(lds_raw + r * 512 + ((((cb >> 4) ^ r) & 31) << 4) + (cb & 15));
                uint16_t* o = out + (size_t)t * N + n0 + (cb >> 1);
                if (p.out_dtype == OUT_BF16) atomic_add2<OUT_BF16>(o, bits);
                else atomic_add2<OUT_FP16>(o, bits);
            }
        } else {
            for (int q = tid; q < TM * 32; q += 256) {
                const int r = q >> 5, g = q & 31;
                *reinterpret_cast<v4i*>(out + ((size_t)blk * TM + r) * N + n0 + g * 8) = *reinterpret_cast<const v4i*>(lds_raw + r * 512 + (((g ^ r) & 31) << 4));
            }
        }
    }
}

// Blocks of 128 sorted rows run as two workgroups of 64 rows each: a 128-row tile needs every register of the wavefront for its
// accumulators, so one workgroup per CU would run with nothing to overlap its loads and its epilogue with (measured, 4096
// tokens x top-8 on 32 experts, 4096 x 1536, operands three steps ahead in both: stage 1 364 us with 128-row tiles against 292 with
// 64-row tiles, stage 2 with the atomic epilogue 655 against 393, one row per sorted position 271 against 225).
template <int AF, int STAGE>
hipError_t launch_rows(MoeMxParams p, int block_m, int blocks, hipStream_t stream) {
    p.eshift = block_m == 128 ? 1 : 0;
    p.blocks = blocks;
    p.n_tiles = p.n_out / (STAGE == 1 ? 128 : 256);
    p.n_groups = (p.n_tiles + 7) / 8;
    // Keyed by expert while an expert has few rows (then sharing an L2 is what saves re-reads: 256 tokens x top-8 on 32 experts,
    // blocks of 32, stage 1 66 -> 49 us; blocks of 16: 84 -> 71); from about 200 sorted rows per expert on the other orders measured
    // better (1024 tokens, blocks of 64: 93 us against 103; 4096 tokens: 297 against 330)
    p.by_expert = p.n_tiles % 8 != 0 && (long)p.sorted_size <= 192L * p.experts;
    p.quad_tiles = !p.by_expert && p.n_tiles % 4 == 0 && p.n_tiles % 8 != 0;
    const unsigned row_blocks = (unsigned)(blocks << p.eshift);
    const dim3 grid((unsigned)(p.by_expert ? p.n_groups * 8 : p.n_tiles) * (p.quad_tiles ? (row_blocks + 1) / 2 * 2 : row_blocks));
    if (block_m == 16) {
        if constexpr (STAGE == 2) hipLaunchKernelGGL((k_moe_mx<MXF_FP4, 1, 2>), grid, dim3(256), 0, stream, p);
        else if constexpr (AF == MXF_FP4) hipLaunchKernelGGL((k_moe_mx<MXF_FP4, 1, 1, true>), grid, dim3(256), 0, stream, p);
        else return hipErrorInvalidValue;
    } else if (block_m == 32) hipLaunchKernelGGL((k_moe_mx<AF, 2, STAGE>), grid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((k_moe_mx<AF, 4, STAGE>), grid, dim3(256), 0, stream, p);
    return hipGetLastError();
}

}  // namespace

// Scales of the sorted rows in the shuffled order stage 1 reads: one thread per output dword = the scale bytes of the rows r16 and
// r16 + 16 of a 32-row chunk at the columns c4 and c4 + 4 of an 8-column chunk (byte = 2 * column half + row half).
__global__ void __launch_bounds__(256) k_moe_mx_scale_sort(const uint8_t* scale, const int32_t* sorted_ids, const int32_t* num_valid, uint32_t* out,
                                                            int tokens, int topk, int cols, int sorted_size, int dwords) {
    const int d = (int)blockIdx.x * 256 + (int)threadIdx.x;
    if (d >= dwords) return;
    const int r16 = d & 15, c4 = (d >> 4) & 3, blk = d >> 6;  // blk = chunk * (cols / 8) + column chunk
    const int ncc = cols >> 3, chunk = blk / ncc, cc = blk % ncc;
    const int nv = num_valid[0];
    uint32_t word = 0;
#pragma unroll
    for (int rh = 0; rh < 2; rh++) {
        const int i = chunk * 32 + rh * 16 + r16;
        if (i >= sorted_size || i >= nv) continue;
        const uint32_t id = (uint32_t)sorted_ids[i];
        const int tok = (int)(id & 0xFFFFFFu), slot = (int)(id >> 24);
        if (tok >= tokens || (topk > 1 && slot >= topk)) continue;
        const uint8_t* row = scale + (size_t)(topk > 1 ? tok * topk + slot : tok) * (size_t)cols + cc * 8 + c4;
        word |= (uint32_t)row[0] << (8 * rh);
        word |= (uint32_t)row[4] << (8 * (2 + rh));
    }
    out[d] = word;
}

// a_format: MXF_FP4 / MXF_FP8 (stage 1 only; stage 2 reads the fp4 rows stage 1 wrote); block_m: 32 / 64 / 128, or 16: stage 1 then
// takes bf16 activations in p.a and quantises them itself (a_format MXF_FP4); blocks: blocks of
// block_m sorted rows the launch covers (blocks past num_valid[0] exit at once)
hipError_t psg_launch_moe_mx_gemm(const MoeMxParams& p, int a_format, int stage, int block_m, int blocks, hipStream_t stream) {
    if (stage == 1) return a_format == MXF_FP8 ? launch_rows<MXF_FP8, 1>(p, block_m, blocks, stream) : launch_rows<MXF_FP4, 1>(p, block_m, blocks, stream);
    return launch_rows<MXF_FP4, 2>(p, block_m, blocks, stream);
}

// out: ceil(sorted_size / 32) * 32 rows x cols bytes, every byte written
hipError_t psg_launch_moe_mx_scale_sort(const void* scale, const int32_t* sorted_ids, const int32_t* num_valid, void* out, int tokens, int topk, int cols,
                                        int sorted_size, hipStream_t stream) {
    const int dwords = (sorted_size + 31) / 32 * 8 * cols;
    hipLaunchKernelGGL(k_moe_mx_scale_sort, dim3((dwords + 255) / 256), dim3(256), 0, stream, static_cast<const uint8_t*>(scale), sorted_ids, num_valid,
                       static_cast<uint32_t*>(out), tokens, topk, cols, sorted_size, dwords);
    return hipGetLastError();
}
