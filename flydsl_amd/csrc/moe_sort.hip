// Expert sorting of routed (token, slot) pairs on the device: the step in front of the MoE grouped GEMMs.
//
// Output layout (the one the MoE stage kernels read): experts in ascending order, each expert's pairs in row-major
// (token, slot) order, padded to whole blocks of block_m rows with (topk << 24) | tokens; one expert id per block.
// No atomics on global memory and a stable order inside every expert, so the output never depends on timing.
//
// Small routings (decode): ONE launch, one workgroup per expert.
//   1. every workgroup builds the whole histogram of expert ids in LDS (4 bytes per routed pair, read from L2), which
//      gives it its own start row (padded rows of all experts below it), the total and, with an expert mask, its local
//      expert number;
//   2. it walks the pairs again in order and compacts those of its expert with wavefront ballots and a prefix over the
//      wavefronts of the workgroup;
//   3. it fills its padding rows, its block ids and its share of the unused tails.
// Large routings (prefill) with a caller workspace: THREE launches, because E workgroups that each count all pairs
// spend their time in LDS atomics (4096 tokens x top-8 on 32 experts: 109 us in one launch).
//   1. the pairs are cut into slices; one workgroup per slice writes the slice's histogram to the workspace;
//   2. one workgroup turns the histograms into per-(slice, expert) offsets, the start row and local number of every
//      expert, the total, the block ids;
//   3. one workgroup per slice moves the slice's pairs straight to their final rows (lanes with the same expert find each
//      other with ballots and share a running base in LDS).
// Either way extra workgroups of the first launch clear the caller's accumulate buffer at full memory bandwidth.
#include "moe_gating.h"

namespace {

constexpr int SORT_THREADS = 256;
constexpr int SORT_WAVES = SORT_THREADS / 64;
constexpr int SORT_MAX_EXPERTS = 4096;
constexpr int SORT_ONESHOT_PAIRS = 4096;   // routings up to this many pairs always take the single launch
constexpr int SORT_SLICE = 1024;           // pairs per slice of the three-launch path (more when there would be > 64 slices)
constexpr int SORT_MAX_SLICES = 64;
constexpr int FUSE_MAX_TOKENS = 32;        // the gating + sorting launch: every sorting workgroup repeats the gating of all tokens
constexpr int FUSE_MAX_PAIRS = 1024;

__device__ __forceinline__ int pack_id(int slot, int token) { return (int)(((unsigned)slot << 24) | (unsigned)token); }

// workgroups past the sorting ones clear the caller's buffer, 16 bytes per lane, grid-stride
__device__ __forceinline__ void clear_share(const MoeSortParams& p, int wg, int wgs) {
    for (int64_t i = (int64_t)wg * SORT_THREADS + threadIdx.x; i < p.zero_vec; i += (int64_t)wgs * SORT_THREADS)
        p.zero_buf[i] = (v4i){0, 0, 0, 0};
}

// rows [total, sorted_size) and blocks [total / block_m, blocks): padding value, weight 0, expert -1; share `wg` of `wgs`
__device__ __forceinline__ void fill_tails(const MoeSortParams& p, int total, int wg, int wgs) {
    const int sentinel = pack_id(p.topk, p.tokens);
    const int tail = p.sorted_size - total, per = (tail + wgs - 1) / wgs;
    const int lo = total + wg * per, hi = lo + per < p.sorted_size ? lo + per : p.sorted_size;
    for (int i = lo + (int)threadIdx.x; i < hi; i += SORT_THREADS) {
        p.sorted_ids[i] = sentinel;
        p.sorted_weights[i] = 0.f;
    }
    const int used = total / p.block_m, btail = p.blocks - used, bper = (btail + wgs - 1) / wgs;
    const int blo = used + wg * bper, bhi = blo + bper < p.blocks ? blo + bper : p.blocks;
    for (int i = blo + (int)threadIdx.x; i < bhi; i += SORT_THREADS) p.sorted_expert_ids[i] = -1;
}

// Stable compaction of the pairs [q_begin, q_end) whose expert is e into rows dst, dst + 1, ...: every wavefront takes a
// contiguous quarter, counts its matches, and after one barrier writes them behind the wavefronts before it.
__device__ __forceinline__ void compact_range(const MoeSortParams& p, const int* ids, const float* wts, int e, int q_begin, int q_end, int dst, int (&wcount)[SORT_WAVES]) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int len = q_end - q_begin, per = ((len + SORT_WAVES - 1) / SORT_WAVES + 63) & ~63;
    const int lo = q_begin + wave * per, hi = lo + per < q_end ? lo + per : q_end;
    int mine = 0;
#pragma unroll 4
    for (int q0 = lo; q0 < hi; q0 += 64) {
        const int q = q0 + lane;
        mine += __popcll(__ballot(q < hi && ids[q] == e));
    }
    if (lane == 0) wcount[wave] = mine;
    __syncthreads();
    int row = dst;
    for (int w = 0; w < wave; w++) row += wcount[w];
    for (int q0 = lo; q0 < hi; q0 += 64) {
        const int q = q0 + lane;
        const bool hit = q < hi && ids[q] == e;
        const unsigned long long ballot = __ballot(hit);
        if (hit) {
            const int r = row + __popcll(ballot & ((1ull << lane) - 1ull));
            const int token = q / p.topk, slot = q - token * p.topk;
            p.sorted_ids[r] = pack_id(slot, token);
            p.sorted_weights[r] = wts[q];
        }
        row += __popcll(ballot);
    }
}

__device__ __forceinline__ void fill_padding(const MoeSortParams& p, int start, int cnt, int local) {
    const int B = p.block_m, padded = (cnt + B - 1) / B * B, sentinel = pack_id(p.topk, p.tokens);
    for (int i = cnt + (int)threadIdx.x; i < padded; i += SORT_THREADS) {
        p.sorted_ids[start + i] = sentinel;
        p.sorted_weights[start + i] = 0.f;
    }
    for (int b = threadIdx.x; b < padded / B; b += SORT_THREADS) p.sorted_expert_ids[start / B + b] = local;
}

// ---- single launch: grid = experts sorting workgroups + clearing workgroups ----
// the work of sorting workgroup e on the routing (ids, wts), which lies in global memory or in LDS
__device__ __forceinline__ void sort_one_expert(const MoeSortParams& p, const int* ids, const float* wts, int e) {
    __shared__ int hist[SORT_MAX_EXPERTS];
    __shared__ int wcount[SORT_WAVES];
    __shared__ int red[3][SORT_WAVES];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int P = p.tokens * p.topk, B = p.block_m;
    for (int i = tid; i < p.experts; i += SORT_THREADS) hist[i] = 0;
    __syncthreads();
    for (int q = tid; q < P; q += SORT_THREADS) {
        const int id = ids[q];
        if ((unsigned)id < (unsigned)p.experts) atomicAdd(&hist[id], 1);  // ids outside [0, experts) are dropped
    }
    __syncthreads();
    // padded rows of the enabled experts below e, of all enabled experts, and the number of enabled experts below e
    int below = 0, total = 0, local = 0;
    for (int j = tid; j < p.experts; j += SORT_THREADS) {
        const bool on = !p.expert_mask || p.expert_mask[j] != 0;
        const int padded = on ? (hist[j] + B - 1) / B * B : 0;
        total += padded;
        if (j < e) {
            below += padded;
            local += on ? 1 : 0;
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        below += __shfl_xor(below, o);
        total += __shfl_xor(total, o);
        local += __shfl_xor(local, o);
    }
    if (lane == 0) {
        red[0][wave] = below;
        red[1][wave] = total;
        red[2][wave] = local;
    }
    __syncthreads();
    below = total = local = 0;
#pragma unroll
    for (int w = 0; w < SORT_WAVES; w++) {
        below += red[0][w];
        total += red[1][w];
        local += red[2][w];
    }
    const bool enabled = !p.expert_mask || p.expert_mask[e] != 0;
    const int cnt = enabled ? hist[e] : 0;
    if (cnt > 0) compact_range(p, ids, wts, e, 0, P, below, wcount);  // cnt is uniform over the workgroup
    fill_padding(p, below, cnt, local);
    fill_tails(p, total, e, p.experts);
    if (e == 0 && tid == 0) {
        p.num_valid[0] = total;
        p.num_valid[1] = p.tokens;
    }
}

__global__ void __launch_bounds__(SORT_THREADS) k_moe_sort(MoeSortParams p) {
    const int e = (int)blockIdx.x;
    if (e >= p.experts) {
        clear_share(p, e - p.experts, (int)gridDim.x - p.experts);
        return;
    }
    sort_one_expert(p, p.topk_ids, p.topk_weights, e);
}

// ---- gating + sorting in one launch (decode): every sorting workgroup first computes the routing of all tokens from the
// router logits into LDS (a few KB of logits from L2 per workgroup, cheaper than a launch), then sorts from there.
// Workgroup 0 also writes the routing to g.weights / g.indices / g.tei where those are given.
template <typename T, int VPT>
__global__ void __launch_bounds__(SORT_THREADS) k_moe_gate_sort(MoeSortParams p, MoeGatingParams g) {
    __shared__ int s_ids[FUSE_MAX_PAIRS];
    __shared__ float s_w[FUSE_MAX_PAIRS];
    const int e = (int)blockIdx.x;
    if (e >= p.experts) {
        clear_share(p, e - p.experts, (int)gridDim.x - p.experts);
        return;
    }
    const int L = g.lanes, sh = __builtin_ctz(L), tpb = SORT_THREADS >> sh;
    const int gl = threadIdx.x & (L - 1);
    for (int t0 = 0; t0 < p.tokens; t0 += tpb) {
        const int t = t0 + (int)(threadIdx.x >> sh);
        const bool live = t < p.tokens;
        const T* row = static_cast<const T*>(g.gating) + (size_t)(live ? t : 0) * p.experts;
        float keep[GATE_KEEP];
        const float f = gate_row<T, VPT>(row, p.experts, p.topk, g.renorm != 0, L, gl, g.vec != 0, keep, [&](int k, int index) {
            if (live && gl == 0) {
                const int q = t * p.topk + k;
                s_ids[q] = index;
                if (e == 0) {
                    if (g.indices) g.indices[q] = index;
                    if (g.tei) g.tei[q] = k * p.tokens + t;
                }
            }
        });
        if (live) {
#pragma unroll
            for (int j = 0; j < GATE_KEEP; j++) {
                const int k = (j << sh) + gl;
                if (k < p.topk) {
                    const int q = t * p.topk + k;
                    s_w[q] = keep[j] * f;
                    if (e == 0 && g.weights) g.weights[q] = keep[j] * f;
                }
            }
        }
    }
    __syncthreads();
    sort_one_expert(p, s_ids, s_w, e);
}

// ---- three launches.  Workspace (ints): off[(slices + 1) * experts] | start[experts] | local[experts] | total ----
struct SortPlan {
    int slices, slice_len;
};

// launch 1: histogram of one slice -> off[g][*]; clearing workgroups behind the slices
__global__ void __launch_bounds__(SORT_THREADS) k_moe_sort_count(MoeSortParams p, SortPlan plan, int* ws) {
    __shared__ int hist[SORT_MAX_EXPERTS];
    const int tid = threadIdx.x, g = (int)blockIdx.x;
    if (g >= plan.slices) {
        clear_share(p, g - plan.slices, (int)gridDim.x - plan.slices);
        return;
    }
    const int P = p.tokens * p.topk;
    for (int i = tid; i < p.experts; i += SORT_THREADS) hist[i] = 0;
    __syncthreads();
    const int lo = g * plan.slice_len, hi = lo + plan.slice_len < P ? lo + plan.slice_len : P;
    for (int q = lo + tid; q < hi; q += SORT_THREADS) {
        const int id = p.topk_ids[q];
        if ((unsigned)id < (unsigned)p.experts) atomicAdd(&hist[id], 1);
    }
    __syncthreads();
    for (int i = tid; i < p.experts; i += SORT_THREADS) ws[g * p.experts + i] = hist[i];
}

// launch 2 (one workgroup): counts per slice -> running offsets per expert; start row, local number, block ids, total
__global__ void __launch_bounds__(1024) k_moe_sort_plan(MoeSortParams p, SortPlan plan, int* ws) {
    __shared__ int padded[SORT_MAX_EXPERTS];
    __shared__ int on[SORT_MAX_EXPERTS];
    __shared__ int s_start[SORT_MAX_EXPERTS];
    __shared__ int s_local[SORT_MAX_EXPERTS];
    const int tid = threadIdx.x, E = p.experts, B = p.block_m;
    int* off = ws;
    int* start = ws + (plan.slices + 1) * E;
    int* local = start + E;
    for (int j = tid; j < E; j += 1024) {
        // the counts of the column in batches of independent loads (one memory latency per batch, not one per slice), then the running sums;
        // neighbouring threads walk neighbouring columns: coalesced
        int acc = 0;
        for (int g0 = 0; g0 < plan.slices; g0 += 16) {  // 16 at a time: the registers of 1024 threads allow no more
            int c[16];
#pragma unroll
            for (int g = 0; g < 16; g++) c[g] = g0 + g < plan.slices ? off[(g0 + g) * E + j] : 0;
#pragma unroll
            for (int g = 0; g < 16; g++)
                if (g0 + g < plan.slices) {
                    off[(g0 + g) * E + j] = acc;
                    acc += c[g];
                }
        }
        const int enabled = !p.expert_mask || p.expert_mask[j] != 0;
        off[plan.slices * E + j] = enabled ? acc : 0;  // row `slices` = pairs of the expert that are kept
        on[j] = enabled;
        padded[j] = enabled ? (acc + B - 1) / B * B : 0;
    }
    __syncthreads();
    // exclusive prefix sums of padded[] (start rows) and on[] (local expert numbers): a Hillis-Steele scan over the experts in LDS,
    // up to four entries per thread, log2(E) rounds
    for (int j = tid; j < E; j += 1024) {
        s_start[j] = padded[j];
        s_local[j] = on[j];
    }
    __syncthreads();
    for (int d = 1; d < E; d <<= 1) {
        int add_p[SORT_MAX_EXPERTS / 1024], add_o[SORT_MAX_EXPERTS / 1024];
#pragma unroll
        for (int q = 0; q < SORT_MAX_EXPERTS / 1024; q++) {
            const int j = tid + q * 1024;
            const bool take = j < E && j >= d;
            add_p[q] = take ? s_start[j - d] : 0;
            add_o[q] = take ? s_local[j - d] : 0;
        }
        __syncthreads();
#pragma unroll
        for (int q = 0; q < SORT_MAX_EXPERTS / 1024; q++) {
            const int j = tid + q * 1024;
            if (j < E) {
                s_start[j] += add_p[q];
                s_local[j] += add_o[q];
            }
        }
        __syncthreads();
    }
    if (tid == 0) {
        const int total = s_start[E - 1];
        start[2 * E] = total;  // behind start[] and local[]
        p.num_valid[0] = total;
        p.num_valid[1] = p.tokens;
    }
    for (int j = tid; j < E; j += 1024) {
        const int st = s_start[j] - padded[j], lo = s_local[j] - on[j];
        start[j] = st;
        local[j] = lo;
        for (int b = 0; b < padded[j] / B; b++) p.sorted_expert_ids[st / B + b] = lo;
    }
}

// launch 3: one workgroup per slice moves the slice's pairs straight to their final rows (work proportional to the pairs,
// whatever the expert count); one more workgroup fills the tails.  Every wavefront owns a contiguous quarter of the slice:
//   pass 1  histogram of the quarter in a row of LDS counters of its own;
//   then    the counters become running bases: rows of the expert taken by earlier slices (launch 2) + by earlier wavefronts;
//   pass 2  64 pairs at a time, in order: the lanes with the same expert find each other with one ballot per bit of the
//           expert id, rank themselves by lane, read the running base, and the first of them advances it.
// Stable by construction (slices, wavefronts, chunks and lanes all in pair order) and free of global atomics.
__global__ void __launch_bounds__(SORT_THREADS) k_moe_sort_scatter(MoeSortParams p, SortPlan plan, const int* ws) {
    __shared__ int base[SORT_WAVES][SORT_MAX_EXPERTS];
    const int g = (int)blockIdx.x, E = p.experts, B = p.block_m;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int* off = ws;
    const int* start = ws + (plan.slices + 1) * E;
    if (g == plan.slices) {
        fill_tails(p, start[2 * E], 0, 1);
        return;
    }
    // padding rows: one thread per expert (independent loads; an expert has fewer than block_m padding rows)
    const int sentinel = pack_id(p.topk, p.tokens);
    for (int e = g * SORT_THREADS + tid; e < E; e += plan.slices * SORT_THREADS) {
        const int kept = off[plan.slices * E + e], padded = (kept + B - 1) / B * B, st = start[e];
        for (int i = kept; i < padded; i++) {
            p.sorted_ids[st + i] = sentinel;
            p.sorted_weights[st + i] = 0.f;
        }
    }
    const int P = p.tokens * p.topk;
    const int lo_s = g * plan.slice_len, hi_s = lo_s + plan.slice_len < P ? lo_s + plan.slice_len : P;
    const int per = ((hi_s - lo_s + SORT_WAVES - 1) / SORT_WAVES + 63) & ~63;
    const int lo = lo_s + wave * per, hi = lo + per < hi_s ? lo + per : hi_s;
    for (int i = lane; i < E; i += 64) base[wave][i] = 0;
    __syncthreads();
    constexpr int G = 8;  // chunks of 64 pairs whose loads are issued together (one memory latency per group, not per chunk)
    for (int q0 = lo; q0 < hi; q0 += 64 * G) {
        int id[G];
#pragma unroll
        for (int c = 0; c < G; c++) {
            const int q = q0 + c * 64 + lane;
            id[c] = q < hi ? p.topk_ids[q] : -1;
        }
#pragma unroll
        for (int c = 0; c < G; c++)
            if ((unsigned)id[c] < (unsigned)E) atomicAdd(&base[wave][id[c]], 1);
    }
    __syncthreads();
    for (int e = tid; e < E; e += SORT_THREADS) {
        int run = start[e] + off[g * E + e];
#pragma unroll
        for (int w = 0; w < SORT_WAVES; w++) {
            const int c = base[w][e];
            base[w][e] = run;
            run += c;
        }
    }
    __syncthreads();
    int bits = 1;
    while ((1 << bits) < E) bits++;
    for (int q0 = lo; q0 < hi; q0 += 64 * G) {  // uniform per wavefront
        int id[G];
        float wt[G];
        bool ok[G];
#pragma unroll
        for (int c = 0; c < G; c++) {
            const int q = q0 + c * 64 + lane;
            id[c] = q < hi ? p.topk_ids[q] : -1;
            wt[c] = q < hi ? p.topk_weights[q] : 0.f;
        }
#pragma unroll
        for (int c = 0; c < G; c++) ok[c] = (unsigned)id[c] < (unsigned)E && (!p.expert_mask || p.expert_mask[id[c]] != 0);
#pragma unroll
        for (int c = 0; c < G; c++) {
            if (q0 + c * 64 >= hi) break;  // uniform
            const int q = q0 + c * 64 + lane;
            unsigned long long peers = __ballot(ok[c]);
            for (int b = 0; b < bits; b++) {
                const unsigned long long set = __ballot((id[c] >> b) & 1);
                peers &= ((id[c] >> b) & 1) ? set : ~set;
            }
            const unsigned long long below = peers & ((1ull << lane) - 1ull);
            if (ok[c]) {
                const int row = base[wave][id[c]] + __popcll(below);
                const int token = q / p.topk, slot = q - token * p.topk;
                p.sorted_ids[row] = pack_id(slot, token);
                p.sorted_weights[row] = wt[c];
            }
            // every lane has read its base: now the first lane of each expert advances it (LDS operations of a wavefront complete in order)
            if (ok[c] && below == 0) base[wave][id[c]] += __popcll(peers);
        }
    }
}

int clear_wgs(const MoeSortParams& p) {
    if (!p.zero_buf || p.zero_vec <= 0) return 0;
    const int64_t want = (p.zero_vec * 16 + (128 << 10) - 1) / (128 << 10);  // 128 KB per workgroup, at most 4 per CU
    return (int)(want < 1 ? 1 : (want > 1024 ? 1024 : want));
}

SortPlan make_plan(int64_t pairs) {
    SortPlan plan;
    int64_t slices = (pairs + SORT_SLICE - 1) / SORT_SLICE;
    if (slices > SORT_MAX_SLICES) slices = SORT_MAX_SLICES;
    plan.slices = (int)slices;
    plan.slice_len = (int)(((pairs + slices - 1) / slices + 63) / 64 * 64);
    return plan;
}

}  // namespace

int psg_moe_sort_max_experts() { return SORT_MAX_EXPERTS; }

// whether gating + sorting of this routing runs as one launch
bool psg_moe_gate_sort_fuses(int tokens, int topk, int experts) {
    if (experts > GATE_MAX_EXPERTS || topk > GATE_MAX_TOPK || (int64_t)tokens * topk > FUSE_MAX_PAIRS) return false;
    int vpt, lanes;
    gate_layout(experts, &vpt, &lanes);
    // one pass of the workgroup's 256 lanes over the tokens: a second pass costs more than the launch it saves
    return tokens <= FUSE_MAX_TOKENS && tokens <= SORT_THREADS / lanes;
}

namespace {
template <typename T>
hipError_t launch_gate_sort_t(const MoeSortParams& p, const MoeGatingParams& g, int vpt, int grid, hipStream_t stream) {
    switch (vpt) {
        case 1: hipLaunchKernelGGL((k_moe_gate_sort<T, 1>), dim3(grid), dim3(SORT_THREADS), 0, stream, p, g); break;
        case 2: hipLaunchKernelGGL((k_moe_gate_sort<T, 2>), dim3(grid), dim3(SORT_THREADS), 0, stream, p, g); break;
        case 4: hipLaunchKernelGGL((k_moe_gate_sort<T, 4>), dim3(grid), dim3(SORT_THREADS), 0, stream, p, g); break;
        case 8: hipLaunchKernelGGL((k_moe_gate_sort<T, 8>), dim3(grid), dim3(SORT_THREADS), 0, stream, p, g); break;
        default: hipLaunchKernelGGL((k_moe_gate_sort<T, 16>), dim3(grid), dim3(SORT_THREADS), 0, stream, p, g); break;
    }
    return hipGetLastError();
}
}  // namespace

// One launch: gating of g (dtype 0 fp32, 1 bf16, 2 fp16) feeding the sort of p; p.topk_ids / p.topk_weights are not read.
// Requires psg_moe_gate_sort_fuses(tokens, topk, experts).
hipError_t psg_launch_moe_gate_sort(const MoeSortParams& p, MoeGatingParams g, int dtype, hipStream_t stream) {
    int vpt, lanes;
    gate_layout(p.experts, &vpt, &lanes);
    const int esz = dtype == 0 ? 4 : 2;
    const int chunk = vpt * esz, need = chunk < 16 ? chunk : 16;
    g.lanes = lanes;
    g.vec = p.experts % vpt == 0 && reinterpret_cast<uintptr_t>(g.gating) % need == 0 && ((size_t)p.experts * esz) % need == 0;
    const int grid = p.experts + clear_wgs(p);
    switch (dtype) {
        case 0: return launch_gate_sort_t<float>(p, g, vpt, grid, stream);
        case 1: return launch_gate_sort_t<uint16_t>(p, g, vpt, grid, stream);
        case 2: return launch_gate_sort_t<_Float16>(p, g, vpt, grid, stream);
    }
    return hipErrorInvalidValue;
}

// bytes of workspace the three-launch path wants for this routing (0: the single launch is used anyway)
uint64_t psg_moe_sort_workspace(int64_t pairs, int experts) {
    if (pairs <= SORT_ONESHOT_PAIRS) return 0;
    const SortPlan plan = make_plan(pairs);
    return ((uint64_t)(plan.slices + 1) * experts + 2ull * experts + 4) * sizeof(int);
}

hipError_t psg_launch_moe_sort(const MoeSortParams& p, void* workspace, uint64_t workspace_bytes, hipStream_t stream) {
    const int64_t pairs = (int64_t)p.tokens * p.topk;
    const uint64_t want = psg_moe_sort_workspace(pairs, p.experts);
    const int zwgs = clear_wgs(p);
    if (want == 0 || !workspace || workspace_bytes < want) {
        hipLaunchKernelGGL(k_moe_sort, dim3(p.experts + zwgs), dim3(SORT_THREADS), 0, stream, p);
        return hipGetLastError();
    }
    const SortPlan plan = make_plan(pairs);
    int* ws = static_cast<int*>(workspace);
    hipLaunchKernelGGL(k_moe_sort_count, dim3(plan.slices + zwgs), dim3(SORT_THREADS), 0, stream, p, plan, ws);
    hipLaunchKernelGGL(k_moe_sort_plan, dim3(1), dim3(1024), 0, stream, p, plan, ws);
    hipLaunchKernelGGL(k_moe_sort_scatter, dim3(plan.slices + 1), dim3(SORT_THREADS), 0, stream, p, plan, (const int*)ws);
    return hipGetLastError();
}
