// C ABI of libpsgemm.so: argument validation, regime selection and launch on the caller's stream.
// Nothing here allocates, synchronises or touches any stream but the caller's.
#include "../../include/psgemm.h"

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>

#include "psg_common.h"
#include "moe_gating.h"
#include "tile_order.h"

hipError_t psg_launch_a8w8_tiled(const A8W8Params& p, int kind, int store, int tile_m, int tile_n, hipStream_t stream);
hipError_t psg_launch_a8w8_stream(const A8W8Params& p, int kind, int store, hipStream_t stream);
hipError_t psg_launch_moe_gemm(const MoeParams& p, int kind, int stage, int block_m, int blocks, hipStream_t stream);
hipError_t psg_launch_moe_mx_gemm(const MoeMxParams& p, int a_format, int stage, int block_m, int blocks, hipStream_t stream);
hipError_t psg_launch_moe_mx_scale_sort(const void* scale, const int32_t* sorted_ids, const int32_t* num_valid, void* out, int tokens, int topk, int cols,
                                        int sorted_size, hipStream_t stream);
hipError_t psg_launch_moe_sort(const MoeSortParams& p, void* workspace, uint64_t workspace_bytes, hipStream_t stream);
uint64_t psg_moe_sort_workspace(int64_t pairs, int experts);
int psg_moe_sort_max_experts();
hipError_t psg_launch_moe_gating(MoeGatingParams p, int dtype, hipStream_t stream);
hipError_t psg_launch_moe_gate_sort(const MoeSortParams& p, MoeGatingParams g, int dtype, hipStream_t stream);
bool psg_moe_gate_sort_fuses(int tokens, int topk, int experts);
hipError_t psg_launch_moe_reduce(const void* x, void* y, int tokens, int topk, int dim, int out_dtype, const int32_t* mask,
                                 const int32_t* ids, int experts, hipStream_t stream);
hipError_t psg_launch_mx_generic(const MxGenParams& p, int af, int bf, int store, int batch, hipStream_t stream);
hipError_t psg_launch_mxfp4_smallm(const MxParams& p, int store, int nw, hipStream_t stream);
hipError_t psg_launch_splitk_finalize(const A8W8Params& p, const void* partial, int is_int, int scaled, hipStream_t stream);
hipError_t psg_launch_tile_order(int tiles_m, int tiles_n, int group_m, int32_t* out, hipStream_t stream);
hipError_t psg_launch_quant_pertoken(const void* x, int x_dtype, void* y, float* scale, int M, int K, int out_fp8, hipStream_t stream);
hipError_t psg_launch_quant_mxfp4(const void* x, int x_dtype, void* packed, void* scales, int M, int R, int K, int shuffled,
                                  hipStream_t stream);

// Scratch of the entry point that allocates nothing (psg_gemm_a8w8_static): the split-K partial sums of the tiled
// path live here instead of in a caller-supplied workspace.  Every GPU the library runs on holds its own copy of the
// array at its own address until the process ends.  In host code the name below is only a stand-in for the symbol:
// the device address is looked up once per device with hipGetSymbolAddress and that pointer is what kernels get.
#define PSG_STATIC_SCRATCH_BYTES (32u << 20)
static __device__ __align__(256) unsigned char scratch[PSG_STATIC_SCRATCH_BYTES];

// Compute units of the current device, read once (the planners deal workgroups out per CU).  Without a device (host-only use of
// the planning entry points) the MI355X's 256.
int psg_cu_count() {
    static const int n = [] {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) {
            (void)hipGetLastError();
            cus = 256;
        }
        return cus;
    }();
    return n;
}

namespace {

thread_local char g_err[512] = "";

constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {};  // device address of `scratch` on each device, filled on first use
std::mutex g_scratch_mu;

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int hip_fail(hipError_t e, const char* what) {
    snprintf(g_err, sizeof(g_err), "%s: %s", what, hipGetErrorString(e));
    return (int)e;
}

bool aligned(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

constexpr int kSmallM = 32;      // rows the split-K path covers
constexpr int kStreamMaxM = 64;  // rows the small-M kernels can hold (four 16-row blocks)

// Which regime an fp4 x fp4 problem takes: the small-M kernel up to 32 rows; up to 64 rows while the weight is at most 40 MB
// and K at least 2048 (measured, us small-M / tiled plan: M=33 7168x2048 4.9 / 6.5, 8192x8192 10.9 / 14.6, 1024x2048 4.3 / 5.3,
// 4096x1024 4.8 / 4.1, 28672x4096 16.5 / 17.0; M=64 5.9 / 6.7, 13.2 / 15.8, 5.4 / 5.3, 5.8 / 4.2, 22.0 / 17.8).
bool mx_takes_small(int M, int N, int K) {
    if (M <= kSmallM) return true;
    return M <= kStreamMaxM && K >= 2048 && (long)N * (K / 2) <= (40L << 20);
}

// Which regime an 8- / 16-bit problem takes when the caller does not force one.  Up to 32 rows always the streaming
// kernel.  Above that every workgroup of the streaming kernel still reads all of A (M x K bytes through its texture
// path), so it only wins while the weight is small enough that the split-K pair of the tiled kernel is bound by its
// two launches and its partial sums rather than by bandwidth (measured, fp8, us streaming / tiled+split-K: M=33 1024x2048
// 4.3 / 8.0, 6144x4096 9.2 / 14.1, 8192x8192 15.3 / 19.6, 28672x4096 31.7 / 32.3, 2048x16384 15.5 / 16.0; M=48 9.7 / 14.4,
// 16.5 / 20.4, 33.0 / 31.3, 17.3 / 16.3; M=64 1024x2048 5.5 / 8.2, 6144x4096 11.3 / 15.0, 8192x8192 18.3 / 22.2,
// 5120x8192 15.8 / 19.0, 28672x4096 37.5 / 32.7, 2048x16384 20.0 / 15.6).
bool takes_stream(int M, int N, int kbytes) {
    if (M <= kSmallM) return true;
    if (M > kStreamMaxM) return false;
    const long w = (long)N * kbytes, a = (long)M * kbytes;
    return a <= (512L << 10) && w <= (80L << 20);
}
constexpr int kTargetWaves = 1536;  // wavefronts wanted in flight for the streaming path (6 per CU)

int pick_ksplit(int units, int steps) {
    int ks = 1;
    while (ks < 8 && units * ks < kTargetWaves && ks * 2 <= steps) ks *= 2;
    return ks;
}

struct Tile {
    int m, n;
    int waves;  // wavefronts per workgroup: 4 (side by side along N, or 2x2) or 8 (side by side along N)
};

// Tile choice for the MFMA mainloop.  Each shape has a measured relative efficiency at full occupancy.  The 256x256
// tile of eight wavefronts side by side along N loads every W fragment once per CU and moves the least data per flop:
// on real data the chip is power-limited, so that is what decides (fp8 8192x4096x4096: 117 us against 134 us for
// the 128x256 tile that runs two workgroups per CU; int8 4096x28672x8192: 775 against 940).  MXFP4 4096x7168x2048:
// 46 us with eight wavefronts against 52 with four, 58 for the 128x256 tile (one workgroup per CU: with two it spilled) and
// 48 for 64x256; MXFP4 1024x8192x8192, where 256x256 gives only 128 tiles: 40 us with 128x256 against 59.  The MX efficiencies of the 64x128
// and 32x128 tiles come from timing every forced tile next to the automatic plan (M 96-5120 on five N x K pairs: 256x8192x8192 21.3 us
// with 64x128 tiles against 25.0 with 32x256; 96x7168x2048 5.7 with 32x128 against 6.7 with 64x128).  The score multiplies the efficiency by
// how evenly the tiles fill the CUs' workgroup slots and by the fraction of each tile that is not padding.
Tile pick_tile(int M, int N, bool mx, int hint_m, int hint_n) {
    struct Shape {
        int m, n, waves, per_cu;
        double eff;
    };
    static const Shape shapes8[] = {{256, 256, 8, 1, 1.17}, {128, 256, 4, 2, 1.00}, {64, 256, 4, 2, 0.62}, {32, 256, 4, 3, 0.36},
                                    {128, 128, 4, 2, 0.70}, {64, 64, 4, 5, 0.25}};
    static const Shape shapesx[] = {{256, 256, 8, 1, 1.00}, {128, 256, 4, 1, 0.80}, {64, 256, 4, 2, 0.75}, {32, 256, 4, 3, 0.40},
                                    {64, 128, 4, 3, 0.60}, {32, 128, 4, 4, 0.34}};
    const Shape* shapes = mx ? shapesx : shapes8;
    if (hint_m > 0 && hint_n > 0) return {hint_m, hint_n, 4};  // forced by the caller; the launcher rejects unknown shapes
    double best = -1.0;
    Tile t = {shapes[0].m, shapes[0].n, shapes[0].waves};
    for (int i = 0; i < 6; i++) {
        const int tm = shapes[i].m, tn = shapes[i].n;
        const long tiles_m = (M + tm - 1) / tm, tiles_n = (N + tn - 1) / tn;
        const long tiles = tiles_m * tiles_n;
        const long cus = psg_cu_count();
        const long slots = cus * shapes[i].per_cu;
        const long rounds = (tiles + slots - 1) / slots;
        // a partly filled last round still costs a full tile time on the CUs it touches
        const double fill = (double)tiles / (double)(rounds * slots);
        // between one workgroup per CU and a full set of slots the CUs that hold one more than the others finish last (scored
        // for the MX kinds, whose 64x128 and 64x256 tiles meet that case: 1024x5120x5120 24.7 us with 640 tiles of 64x128
        // against 27.7 with 320 of 64x256; the 8- and 16-bit kinds have the rule behind the loop instead)
        const double between = (double)tiles / (double)(((tiles + cus - 1) / cus) * cus);
        const double busy = tiles >= slots ? fill : (tiles <= cus ? (double)tiles / (double)cus : (mx ? between : 1.0));
        const double pad = ((double)M / (double)(tiles_m * tm)) * ((double)N / (double)(tiles_n * tn));
        const double score = busy * pad * shapes[i].eff;
        if (score > best) {
            best = score;
            t = {tm, tn, shapes[i].waves};
        }
    }
    // The score counts workgroup slots, two per CU for 128x256, so between one and two such tiles per CU it sees one round where
    // the CUs that hold two take twice as long.  When the 256x256 tiles of the same problem make one round that fills more
    // than half of the CUs, they are faster (fp8, us 256x256 / 128x256: 5120x2048x8320 86 / 96; 1536x8192x8192 89 / 103;
    // 2048x5120x5120 60 / 71; 3072x4096x4096 52 / 56; with only half of the CUs filled they are not: 2048x4096x4096 47 / 38).
    if (!mx && t.m == 128 && t.n == 256) {
        const long cus = psg_cu_count();
        const long t256 = (long)((M + 255) / 256) * (long)((N + 255) / 256), t128 = (long)((M + 127) / 128) * (long)((N + 255) / 256);
        if (t128 > cus && t256 <= cus && t256 * 20 > cus * 11) t = {256, 256, 8};
    }
    return t;
}

// Split-K for the regime between the streaming kernel (M <= 32) and problems with enough tiles to fill the GPU:
// with few tiles every workgroup walks all of K behind a one-step prefetch and the launch is latency-bound.
// Splitting K over `splits` workgroups per tile multiplies the loads in flight; the price is one fp32 slice of
// [M,N] per split written and read back, so the split count is capped where that traffic reaches 1.25 W, and where the
// workgroups would no longer all be resident at once.
// Returns 1 when splitting does not pay.  kbytes = bytes of one operand row.
int pick_splits(int M, int N, int kbytes, Tile t) {
    const long tiles = (long)((M + t.m - 1) / t.m) * (long)((N + t.n - 1) / t.n);
    const int steps = (kbytes + 127) / 128;
    const long cus = psg_cu_count();
    // a CU holds one workgroup of a 128x128 tile (or larger), two of a 64x64 tile on long rows
    const bool pairs = t.m == 64 && t.n == 64 && steps >= 48;
    if (tiles >= (pairs ? 2 * cus : cus) * 3 / 4 || steps < 32) return 1;
    // Measured on operands that do not fit the last-level cache (fp8, 128x128 tiles): the best split count is the largest one
    // that still gives every workgroup a CU of its own, powers of two or not (us for 2/3/4/5/6/7/8 splits: 256x2304x14336,
    // 36 tiles, 40/32/27/25/24/23.5/30; 384x1664x10240, 39 tiles, 32/26/23/22/21.7/24.5/27; 256x3072x14336, 48 tiles,
    // 43/34/30/27.6/35/35/33; 512x2112x7168, 68 tiles, 24.8/22.1 for 2/3; one workgroup more than there are CUs costs a second
    // round).  64x64 tiles on long rows may also come two to a CU, but then (nearly) all CUs should have two: between one and one
    // and a half workgroups per CU the doubled CUs finish last (64x6144x16384, 96 tiles, us for 2/3/4/5/8 splits: 34/35/31/29/29;
    // 48x5120x13824, 80 tiles, 3/6/8 splits: 23.3/21.4/22.7; 48x2304x14336, 36 tiles, 7/8 splits: 14.9/16.6).  Bounds: at least
    // 8 K steps per workgroup (12 on rows shorter than 48 steps), partial sums at most 1.25 W.
    const int min_steps = steps >= 48 ? 8 : 12;
    int s = 1;
    for (int c = 2; c <= 8; c++) {
        const long wgs = tiles * c;
        const bool fits = wgs <= cus || (pairs && 2 * wgs >= 3 * cus && wgs <= 2 * cus);
        if (fits && steps / c >= min_steps && (long)c * M * 16 <= (long)kbytes * 5) s = c;
    }
    return s;
}

// Split-K for the general MX kernel: its tiles are 64x128 (32x128 for M <= 32), so decode-like shapes launch few
// workgroups; K is split until about two workgroups per CU exist, every split keeps at least eight 128-element steps
// and the fp32 partials (written and read back once) stay below a quarter of the bytes of an fp4 W.
int mx_general_splits(int M, int N, int K) {
    const uint64_t w_bytes = (uint64_t)N * (uint64_t)K / 2;  // of fp4 W; fp8 W gets the same plan
    const long tiles = (long)((M + (M <= 32 ? 31 : 63)) / (M <= 32 ? 32 : 64)) * (long)((N + 127) / 128);
    const int steps = K / 128;
    int s = 1;
    while (s < 8 && tiles * (s * 2) <= 2L * psg_cu_count() && steps / (s * 2) >= 8 && (uint64_t)(s * 2) * (uint64_t)M * (uint64_t)N * 8ull <= w_bytes / 4) s *= 2;
    return s;
}

// Tile + split plan of the tiled path.  With few tiles and a long K (the regime between the streaming kernel and
// GPU-filling problems) small square-ish tiles with split-K measured best: 64x64 up to M=64, 128x128 above.
struct Plan {
    Tile t;
    int splits;
};
Plan plan_tiled(int M, int N, int kbytes, bool mx) {
    Tile t = pick_tile(M, N, mx, 0, 0);
    const long tiles_big = (long)((M + 127) / 128) * (long)((N + 255) / 256);
    const int steps = (kbytes + 127) / 128;
    const long tiles64 = (long)((M + 63) / 64) * (long)((N + 63) / 64);
    // long rows, few tiles: 128x128 tiles with split-K; 64x64 tiles up to 64 rows, and above that while the whole problem is small
    // (tiles x steps, i.e. M N K / 2^19, up to 11,000: then twice as many workgroups count for more than the W fragments that are
    // loaded twice; fp8, us, 64x64 plan against 128x128 plan: 256x2112x7168 14.8 / 16.8; 320x2112x7168 15.6 / 18.4; 320x1664x10240
    // 18.3 / 20.2; 128x2048x16384 19.2 / 21.2; but 256x2304x14336 27.1 / 23.9; 320x2048x16384 30.0 / 26.3; 65x5120x13824 25.8 / 23.4)
    if (!mx && tiles_big < psg_cu_count() * 3L / 4 && steps >= 48) t = M <= 64 || tiles64 * steps <= 11000 ? Tile{64, 64, 4} : Tile{128, 128, 4};
    // Shorter rows (8..47 steps; K = 4096 one-byte elements is 32): while at most about 600 of them exist, 64x64 tiles beat
    // every larger shape, with or without split-K: many small workgroups keep more bytes of W in flight than a few large ones
    // (fp8, weights not cache-resident: M=128, N=K=4096 14.0 us against 19.4 with 128x128 tiles and two K splits; M=256,
    // N=8192 22.0 against 23.7; M=384, N=8192, 768 tiles: 28.0 against 26.5, so the larger tile is kept there)
    if (!mx && steps >= 8 && steps < 48 && tiles64 <= 600) t = Tile{64, 64, 4};
    return {t, pick_splits(M, N, kbytes, t)};
}

uint64_t splitk_bytes(int M, int N, int splits) { return splits > 1 ? (uint64_t)splits * M * N * 4ull : 0; }

int validate_a8w8(const psg_a8w8_args* a, bool acc_only, const void* acc) {
    if (!a) return fail(PSG_E_NULL, "args is NULL");
    if (!a->a || !a->b) return fail(PSG_E_NULL, "a and b must be non-NULL");
    const bool is16 = a->in_dtype == PSG_IN_FP16 || a->in_dtype == PSG_IN_BF16;
    const int64_t eb = is16 ? 2 : 1;
    if (acc_only) {
        if (!acc) return fail(PSG_E_NULL, "acc must be non-NULL");
    } else {
        if (!a->c) return fail(PSG_E_NULL, "c must be non-NULL");
        if (!is16 && (!a->scale_a || !a->scale_b)) return fail(PSG_E_NULL, "scale_a and scale_b must be non-NULL for 8-bit inputs");
        if (a->epilogue != PSG_EPI_NONE && !a->bias) return fail(PSG_E_NULL, "bias must be non-NULL when epilogue != none");
    }
    if (a->in_dtype < PSG_IN_INT8 || a->in_dtype > PSG_IN_BF16) return fail(PSG_E_DTYPE, "in_dtype %d unknown", a->in_dtype);
    if (a->out_dtype != PSG_OUT_BF16 && a->out_dtype != PSG_OUT_FP16) return fail(PSG_E_DTYPE, "out_dtype %d unknown", a->out_dtype);
    if (a->epilogue < PSG_EPI_NONE || a->epilogue > PSG_EPI_BIAS_GELU) return fail(PSG_E_DTYPE, "epilogue %d unknown", a->epilogue);
    if (a->M < 1 || a->M > 65536) return fail(PSG_E_SHAPE, "M=%d outside [1, 65536]", a->M);
    if (a->N < 16 || a->N % 16) return fail(PSG_E_SHAPE, "N=%d must be a positive multiple of 16", a->N);
    if (a->K < 64 / eb || (a->K * eb) % 64) return fail(PSG_E_SHAPE, "K=%d must be a positive multiple of %d", a->K, (int)(64 / eb));
    if ((uint64_t)a->N * (uint64_t)a->K * (uint64_t)eb > 0xFFFFFFFFull) return fail(PSG_E_SHAPE, "N*K bytes exceed the 4 GiB descriptor range");
    if (!aligned(a->a, 16) || !aligned(a->b, 16)) return fail(PSG_E_ALIGN, "a and b must be 16-byte aligned");
    if (acc_only) {
        if (!aligned(acc, 16)) return fail(PSG_E_ALIGN, "acc must be 16-byte aligned");
    } else {
        if (!aligned(a->c, 16)) return fail(PSG_E_ALIGN, "c must be 16-byte aligned");
        if (!is16 && !aligned(a->scale_b, 16)) return fail(PSG_E_ALIGN, "scale_b must be 16-byte aligned");
        if (!is16 && !aligned(a->scale_a, 4)) return fail(PSG_E_ALIGN, "scale_a must be 4-byte aligned");
        if (a->epilogue != PSG_EPI_NONE && !aligned(a->bias, 8)) return fail(PSG_E_ALIGN, "bias must be 8-byte aligned");
    }
    if (a->workspace && !aligned(a->workspace, 16)) return fail(PSG_E_ALIGN, "workspace must be 16-byte aligned");
    if (a->b_layout != 0 && a->b_layout != 1) return fail(PSG_E_DTYPE, "b_layout=%d unknown (0 preshuffled, 1 row-major)", a->b_layout);
    if (a->force_path < 0 || a->force_path > 2) return fail(PSG_E_SHAPE, "force_path=%d unknown", a->force_path);
    if (a->force_path == 2 && a->M > kStreamMaxM) return fail(PSG_E_SHAPE, "small-M path needs M <= %d, got %d", kStreamMaxM, a->M);
    return 0;
}

// Device address of `scratch` on the current device (looked up once per device, then cached).
int static_scratch(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
    if (dev < 0 || dev >= kMaxDevices) return fail(PSG_E_UNSUPPORTED, "device index %d outside [0, %d)", dev, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress(scratch)");
        if (!ptr) return fail(PSG_E_WORKSPACE, "hipGetSymbolAddress returned a null address for the static scratch");
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return 0;
}

// Argument checks of the expert sorter; `need_routing`: topk_ids / topk_weights are read (not with the fused gating).
int check_moe_sort(const psg_moe_sort_args* a, bool need_routing, MoeSortParams* out) {
    if (!a) return fail(PSG_E_NULL, "args is NULL");
    if ((need_routing && (!a->topk_ids || !a->topk_weights)) || !a->sorted_ids || !a->sorted_weights || !a->sorted_expert_ids || !a->num_valid_ids)
        return fail(PSG_E_NULL, "topk_ids, topk_weights, sorted_ids, sorted_weights, sorted_expert_ids, num_valid_ids must be non-NULL");
    if (a->tokens < 1 || a->tokens >= (1 << 24)) return fail(PSG_E_SHAPE, "tokens=%d outside [1, 2^24)", a->tokens);
    if (a->topk < 1 || a->topk > 255) return fail(PSG_E_SHAPE, "topk=%d outside [1, 255]", a->topk);
    if (a->experts < 1 || a->experts > psg_moe_sort_max_experts()) return fail(PSG_E_SHAPE, "experts=%d outside [1, %d]", a->experts, psg_moe_sort_max_experts());
    if (a->block_m < 1 || a->block_m > 4096) return fail(PSG_E_SHAPE, "block_m=%d outside [1, 4096]", a->block_m);
    // the bound below (the reference's) counts at most one partly filled block per expert and at least topk rows routed: with
    // more slots than experts a token repeats an expert and the padded total can exceed it
    if (a->topk > a->experts) return fail(PSG_E_SHAPE, "topk=%d exceeds experts=%d", a->topk, a->experts);
    const int64_t pairs = (int64_t)a->tokens * a->topk;
    const int64_t need = pairs + (int64_t)a->experts * a->block_m - a->topk;
    if (need > 0x7FFFFFFF) return fail(PSG_E_SHAPE, "tokens*topk + experts*block_m must stay below 2^31");
    if (a->sorted_size < need) return fail(PSG_E_SHAPE, "sorted_size=%d is below tokens*topk + experts*block_m - topk = %lld", a->sorted_size, (long long)need);
    if ((int64_t)a->blocks * a->block_m < a->sorted_size)
        return fail(PSG_E_SHAPE, "blocks=%d must cover sorted_size=%d rows in blocks of %d", a->blocks, a->sorted_size, a->block_m);
    if (a->zero_buf && (a->zero_bytes < 0 || a->zero_bytes % 16 || !aligned(a->zero_buf, 16)))
        return fail(PSG_E_ALIGN, "zero_buf must be 16-byte aligned and zero_bytes a multiple of 16");
    if (a->workspace && !aligned(a->workspace, 4)) return fail(PSG_E_ALIGN, "workspace must be 4-byte aligned");
    MoeSortParams p;
    p.topk_ids = a->topk_ids;
    p.topk_weights = a->topk_weights;
    p.expert_mask = a->expert_mask;
    p.sorted_ids = a->sorted_ids;
    p.sorted_weights = a->sorted_weights;
    p.sorted_expert_ids = a->sorted_expert_ids;
    p.num_valid = a->num_valid_ids;
    p.zero_buf = a->zero_bytes > 0 ? static_cast<v4i*>(a->zero_buf) : nullptr;
    p.zero_vec = a->zero_buf ? a->zero_bytes / 16 : 0;
    p.tokens = a->tokens;
    p.topk = a->topk;
    p.experts = a->experts;
    p.block_m = a->block_m;
    p.sorted_size = a->sorted_size;
    p.blocks = a->blocks;
    *out = p;
    return 0;
}

// Argument checks of the router gating; `need_outputs`: weights / indices must be given (optional with the fused sorting).
int check_moe_gating(const psg_moe_gating_args* a, bool need_outputs, MoeGatingParams* out) {
    if (!a) return fail(PSG_E_NULL, "args is NULL");
    if (!a->gating) return fail(PSG_E_NULL, "gating must be non-NULL");
    if (need_outputs && (!a->weights || !a->indices)) return fail(PSG_E_NULL, "weights and indices must be non-NULL");
    if (a->dtype < 0 || a->dtype > 2) return fail(PSG_E_DTYPE, "dtype %d unknown (0 fp32, 1 bf16, 2 fp16)", a->dtype);
    if (a->tokens < 1 || a->tokens >= (1 << 24)) return fail(PSG_E_SHAPE, "tokens=%d outside [1, 2^24)", a->tokens);
    if (a->experts < 1 || a->experts > GATE_MAX_EXPERTS) return fail(PSG_E_SHAPE, "experts=%d outside [1, %d]", a->experts, GATE_MAX_EXPERTS);
    if (a->topk < 1 || a->topk > GATE_MAX_TOPK || a->topk > a->experts)
        return fail(PSG_E_SHAPE, "topk=%d outside [1, min(%d, experts=%d)]", a->topk, GATE_MAX_TOPK, a->experts);
    if (a->renormalize != 0 && a->renormalize != 1) return fail(PSG_E_SHAPE, "renormalize=%d must be 0 or 1", a->renormalize);
    if (!aligned(a->gating, a->dtype == 0 ? 4 : 2) || (a->weights && !aligned(a->weights, 4)) || (a->indices && !aligned(a->indices, 4)) ||
        (a->token_expert_indices && !aligned(a->token_expert_indices, 4)))
        return fail(PSG_E_ALIGN, "gating must be aligned to its element size, the outputs to 4 bytes");
    MoeGatingParams g;
    g.gating = a->gating;
    g.weights = a->weights;
    g.indices = a->indices;
    g.tei = a->token_expert_indices;
    g.tokens = a->tokens;
    g.experts = a->experts;
    g.topk = a->topk;
    g.renorm = a->renormalize;
    g.lanes = 1;
    g.vec = 0;
    *out = g;
    return 0;
}

int run_a8w8(const psg_a8w8_args* a, void* out, int store, void* stream) {
    A8W8Params p{};
    p.c = out;
    p.a = static_cast<const uint8_t*>(a->a);
    p.b = static_cast<const uint8_t*>(a->b);
    p.sa = a->scale_a;
    p.sb = a->scale_b;
    p.bias = static_cast<const uint16_t*>(a->bias);
    p.M = a->M;
    p.N = a->N;
    p.K = a->K;
    p.epi = a->epilogue;
    p.out = a->out_dtype;
    p.b_rowmajor = a->b_layout;
    // M-tiles per group of the XCD-aware tile order: 8 makes the set of tiles one XCD works on at a time roughly
    // square in bytes (A rows vs W rows), which minimises what its L2 has to fetch
    p.group_m = a->xcd_swizzle > 0 ? a->xcd_swizzle : 8;
    const int kinds[4] = {KIND_INT8, KIND_FP8, KIND_FP16, KIND_BF16};
    const int kind = kinds[a->in_dtype];
    const int kbytes = (kind == KIND_FP16 || kind == KIND_BF16) ? a->K * 2 : a->K;
    const bool small = a->force_path == 2 || (a->force_path == 0 && takes_stream(a->M, a->N, kbytes));
    hipError_t e;
    if (small) {
        e = psg_launch_a8w8_stream(p, kind, store, static_cast<hipStream_t>(stream));
    } else {
        const bool forced = a->force_path == 1 && a->tile_m > 0 && a->tile_n > 0;
        const Plan plan = plan_tiled(a->M, a->N, kbytes, false);
        const Tile t = forced ? Tile{a->tile_m, a->tile_n, 4} : plan.t;
        p.ksplit = 1;
        // wavefront layout of the 256x256 tile: the planner's choice, or forced (2 = 2x2, 8 = 1x8) by tests / tuning
        p.wave_layout = a->reserved >= 2 ? a->reserved : (!forced && t.waves == 8 ? 8 : 1);
        // forced launches take the split count from tile_k (1..16); otherwise the planner decides
        int splits = forced ? (a->tile_k >= 1 && a->tile_k <= 16 ? a->tile_k : 1) : plan.splits;
        if (store != STORE_C || !a->workspace || a->workspace_bytes < splitk_bytes(a->M, a->N, splits)) splits = 1;
        p.splits = splits;
        // at most two workgroups per CU: the launch is bound by the bytes of W in flight, so the builds that fetch W three
        // steps ahead run (ksplit doubles as that mark for the tiled kernel); reserved = 7 keeps the one-step builds (tests)
        const long wgs = (long)((a->M + t.m - 1) / t.m) * (long)((a->N + t.n - 1) / t.n) * splits;
        const int steps_per_wg = ((kbytes + 127) / 128 + splits - 1) / splits;
        if (wgs <= 512 && steps_per_wg >= 6 && a->reserved != 7) p.ksplit = 3;
        if (splits > 1) {
            A8W8Params part = p;
            part.c = a->workspace;
            e = psg_launch_a8w8_tiled(part, kind, STORE_ACC, t.m, t.n, static_cast<hipStream_t>(stream));
            if (e == hipSuccess)
                e = psg_launch_splitk_finalize(p, a->workspace, kind == KIND_INT8, kind == KIND_INT8 || kind == KIND_FP8,
                                               static_cast<hipStream_t>(stream));
        } else {
            e = psg_launch_a8w8_tiled(p, kind, store, t.m, t.n, static_cast<hipStream_t>(stream));
        }
    }
    if (e != hipSuccess) return hip_fail(e, "psg_gemm_a8w8 launch");
    g_err[0] = 0;
    return 0;
}

}  // namespace

extern "C" {

int psg_abi_version(void) { return PSG_ABI_VERSION; }

const char* psg_last_error(void) { return g_err; }

uint64_t psg_workspace_bytes(int32_t M, int32_t N, int32_t K, int32_t in_dtype) {
    // Only the split-K variant of the tiled path (few tiles, long K) uses global scratch: one fp32 / int32 slice of
    // [M,N] per split.  Without it (NULL or too small) the library runs the same problem unsplit.
    if (in_dtype == 5) return M >= 1 && N >= 32 && K >= 256 ? splitk_bytes(M, N, mx_general_splits(M, N, K)) : 0;  // general MX kernel
    if (M <= kSmallM || M < 1 || N < 16 || K < 64) return 0;
    const bool mx = in_dtype == 4;  // MXFP4 (psg_gemm_mxfp4)
    const int kbytes = mx ? K / 2 : ((in_dtype == PSG_IN_FP16 || in_dtype == PSG_IN_BF16) ? K * 2 : K);
    if (mx ? mx_takes_small(M, N, K) : takes_stream(M, N, kbytes)) return 0;  // the small-M kernels reduce inside their workgroups
    return splitk_bytes(M, N, plan_tiled(M, N, kbytes, mx).splits);
}

int psg_gemm_a8w8(const psg_a8w8_args* args, void* stream) {
    if (int rc = validate_a8w8(args, false, nullptr)) return rc;
    return run_a8w8(args, args->c, STORE_C, stream);
}

int psg_init(void) {
    (void)psg_cu_count();
    void* ptr = nullptr;
    if (int rc = static_scratch(&ptr)) return rc;
    g_err[0] = 0;
    return 0;
}

uint64_t psg_static_scratch_bytes(void) { return PSG_STATIC_SCRATCH_BYTES; }

int psg_gemm_a8w8_static(const psg_a8w8_args* args, void* stream) {
    if (int rc = validate_a8w8(args, false, nullptr)) return rc;
    // what the same problem's plan would want as workspace; forced tiles take their split count from tile_k
    uint64_t need = psg_workspace_bytes(args->M, args->N, args->K, args->in_dtype);
    if (args->force_path == 1 && args->tile_m > 0 && args->tile_n > 0)
        need = splitk_bytes(args->M, args->N, args->tile_k >= 1 && args->tile_k <= 16 ? args->tile_k : 1);
    if (args->force_path == 2) need = 0;  // (psg_workspace_bytes is already 0 for what the streaming kernel takes by itself)
    if (need > PSG_STATIC_SCRATCH_BYTES)
        return fail(PSG_E_WORKSPACE, "this problem's split-K plan needs %llu bytes of scratch, the static scratch holds %u; use "
                    "psg_gemm_a8w8 with a caller workspace", (unsigned long long)need, PSG_STATIC_SCRATCH_BYTES);
    psg_a8w8_args local = *args;
    local.workspace = nullptr;
    local.workspace_bytes = 0;
    if (need) {
        void* ptr = nullptr;
        if (int rc = static_scratch(&ptr)) return rc;
        local.workspace = ptr;  // the per-device address, never the symbol's host-side name
        local.workspace_bytes = PSG_STATIC_SCRATCH_BYTES;
    }
    return run_a8w8(&local, local.c, STORE_C, stream);
}

void psg_tile_coords(int32_t id, int32_t tiles_m, int32_t tiles_n, int32_t group_m, int32_t* tm, int32_t* tn) {
    int a = 0, b = 0;
    psg_tile_order(id, tiles_m, tiles_n, group_m, &a, &b);
    *tm = a;
    *tn = b;
}

int psg_debug_tile_order(int32_t tiles_m, int32_t tiles_n, int32_t group_m, int32_t* out, void* stream) {
    if (!out) return fail(PSG_E_NULL, "out must be non-NULL");
    if (tiles_m < 1 || tiles_n < 1 || group_m < 1 || (int64_t)tiles_m * tiles_n > (1 << 24))
        return fail(PSG_E_SHAPE, "need tiles_m, tiles_n, group_m >= 1 and at most 2^24 tiles");
    const hipError_t e = psg_launch_tile_order(tiles_m, tiles_n, group_m, out, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, "psg_debug_tile_order launch");
    g_err[0] = 0;
    return 0;
}

int psg_gemm_a8w8_acc(const psg_a8w8_args* args, void* acc, void* stream) {
    if (int rc = validate_a8w8(args, true, acc)) return rc;
    return run_a8w8(args, acc, STORE_ACC, stream);
}

static int mx_common(const psg_mxfp4_args* a, void* out, int store, void* stream) {
    if (!a) return fail(PSG_E_NULL, "args is NULL");
    if (!out || !a->a || !a->b || !a->scale_a || !a->scale_b) return fail(PSG_E_NULL, "c, a, b, scale_a, scale_b must be non-NULL");
    if (a->out_dtype != PSG_OUT_BF16 && a->out_dtype != PSG_OUT_FP16) return fail(PSG_E_DTYPE, "out_dtype %d unknown", a->out_dtype);
    if (a->a_dtype < PSG_MX_FP4 || a->a_dtype > PSG_MX_FP8) return fail(PSG_E_DTYPE, "a_dtype %d unknown (0 fp4, 1 fp6, 2 fp8)", a->a_dtype);
    if (a->b_dtype != PSG_MX_FP4 && a->b_dtype != PSG_MX_FP8) return fail(PSG_E_DTYPE, "b_dtype %d must be 0 (fp4) or 2 (fp8)", a->b_dtype);
    if (a->M < 1 || a->M > 65536) return fail(PSG_E_SHAPE, "M=%d outside [1, 65536]", a->M);
    if (a->N < 32 || a->N % 32) return fail(PSG_E_SHAPE, "N=%d must be a positive multiple of 32", a->N);
    if (a->K < 256 || a->K % 256) return fail(PSG_E_SHAPE, "K=%d must be a positive multiple of 256", a->K);
    if (a->batch < 0 || a->batch > 65535) return fail(PSG_E_SHAPE, "batch=%d outside [0, 65535]", a->batch);
    if (a->pad0 != 0) return fail(PSG_E_SHAPE, "pad0 must be 0");
    const int batch = a->batch > 1 ? a->batch : 1;
    const uint64_t a_row = a->a_dtype == PSG_MX_FP4 ? (uint64_t)a->K / 2 : (uint64_t)a->K;
    const uint64_t b_row = a->b_dtype == PSG_MX_FP4 ? (uint64_t)a->K / 2 : (uint64_t)a->K;
    const uint64_t chunk = (uint64_t)(a->K / 256) * 256;
    if ((uint64_t)a->N * b_row > 0xFFFFFFFFull) return fail(PSG_E_SHAPE, "one batch of W exceeds the 4 GiB descriptor range");
    if (a->a_row_stride < 0 || a->c_row_stride < 0 || a->scale_a_chunk_stride < 0 || a->a_batch_stride < 0 || a->c_batch_stride < 0 ||
        a->scale_a_batch_stride < 0)
        return fail(PSG_E_SHAPE, "strides must be >= 0 (0 = dense)");
    const uint64_t a_rs = a->a_row_stride ? (uint64_t)a->a_row_stride : a_row;
    const uint64_t c_rs = a->c_row_stride ? (uint64_t)a->c_row_stride : (uint64_t)a->N;
    const uint64_t sa_cs = a->scale_a_chunk_stride ? (uint64_t)a->scale_a_chunk_stride : chunk;
    if (a_rs < a_row || a_rs % 16) return fail(PSG_E_SHAPE, "a_row_stride=%lld must be a multiple of 16 and at least the %llu bytes of a row",
                                               (long long)a_rs, (unsigned long long)a_row);
    if (c_rs < (uint64_t)a->N || c_rs % 4) return fail(PSG_E_SHAPE, "c_row_stride=%lld must be a multiple of 4 elements and at least N", (long long)c_rs);
    if (sa_cs < chunk || sa_cs % 4) return fail(PSG_E_SHAPE, "scale_a_chunk_stride=%lld must be a multiple of 4 and at least %llu", (long long)sa_cs,
                                                (unsigned long long)chunk);
    if ((uint64_t)a->M * a_rs > 0xFFFFFFFFull || (uint64_t)((a->M + 31) / 32) * sa_cs > 0xFFFFFFFFull)
        return fail(PSG_E_SHAPE, "one batch of A or scale_a exceeds the 4 GiB descriptor range");
    if (a->a_batch_stride % 16 || a->c_batch_stride % 8 || a->scale_a_batch_stride % 4)
        return fail(PSG_E_ALIGN, "batch strides must keep a 16-byte, c 8-byte and scale_a 4-byte aligned");
    if (!aligned(a->a, 16) || !aligned(a->b, 16)) return fail(PSG_E_ALIGN, "a and b must be 16-byte aligned");
    if (!aligned(a->scale_a, 4) || !aligned(a->scale_b, 4)) return fail(PSG_E_ALIGN, "scales must be 4-byte aligned");
    if (!aligned(out, 16)) return fail(PSG_E_ALIGN, "output must be 16-byte aligned");
    if (a->force_path < 0 || a->force_path > 3) return fail(PSG_E_SHAPE, "force_path=%d unknown", a->force_path);
    const bool dense = a_rs == a_row && c_rs == (uint64_t)a->N && sa_cs == chunk;
    const bool fp4_fast = a->a_dtype == PSG_MX_FP4 && a->b_dtype == PSG_MX_FP4 && batch == 1 && dense;
    // fp8 x fp8 (MXFP8) also runs on the tiled mainloop when the problem has enough 128x256 tiles to fill the GPU (that
    // kernel has no split-K for this format; decode-like shapes go to the general kernel and its split-K plan)
    const bool fp8_pair = a->a_dtype == PSG_MX_FP8 && a->b_dtype == PSG_MX_FP8 && batch == 1 && dense;
    const bool fp8_tiled = fp8_pair && a->force_path != 3 &&
                           (a->force_path == 1 || (a->M > kSmallM && (long)((a->M + 127) / 128) * (long)((a->N + 255) / 256) >= 192));
    if (a->force_path == 2 && !fp4_fast) return fail(PSG_E_SHAPE, "force_path=2 is for dense, unbatched fp4 x fp4 only");
    if (a->force_path == 1 && !fp4_fast && !fp8_pair)
        return fail(PSG_E_SHAPE, "force_path=1 is for dense, unbatched fp4 x fp4 or fp8 x fp8 only");
    if (a->force_path == 2 && a->M > kStreamMaxM) return fail(PSG_E_SHAPE, "small-M path needs M <= %d, got %d", kStreamMaxM, a->M);
    if (fp8_tiled) {
        const bool forced = a->force_path == 1 && a->tile_m > 0 && a->tile_n > 0;
        const Tile t = forced ? Tile{a->tile_m, a->tile_n, 4} : pick_tile(a->M, a->N, true, 0, 0);
        A8W8Params q{};
        q.c = out;
        q.a = static_cast<const uint8_t*>(a->a);
        q.b = static_cast<const uint8_t*>(a->b);
        q.mx_sa = static_cast<const uint8_t*>(a->scale_a);
        q.mx_sb = static_cast<const uint8_t*>(a->scale_b);
        q.M = a->M;
        q.N = a->N;
        q.K = a->K;
        q.group_m = a->xcd_swizzle > 0 ? a->xcd_swizzle : 8;
        q.ksplit = 1;
        q.wave_layout = a->reserved >= 2 ? a->reserved : 1;  // four wavefronts: 8192x4096x4096 117 us against 130 with eight
        q.splits = 1;
        q.epi = EPI_NONE;
        q.out = a->out_dtype;
        const hipError_t te = psg_launch_a8w8_tiled(q, KIND_MXFP8, store, t.m, t.n, static_cast<hipStream_t>(stream));
        if (te != hipSuccess) return hip_fail(te, "psg_gemm_mxfp4 launch");
        g_err[0] = 0;
        return 0;
    }
    if (a->force_path == 3 || !fp4_fast) {
        MxGenParams g;
        g.c = out;
        g.a = static_cast<const uint8_t*>(a->a);
        g.b = static_cast<const uint8_t*>(a->b);
        g.sa = static_cast<const uint8_t*>(a->scale_a);
        g.sb = static_cast<const uint8_t*>(a->scale_b);
        g.M = a->M;
        g.N = a->N;
        g.K = a->K;
        g.out = a->out_dtype;
        g.splits = 1;
        g.a_row_stride = (int64_t)a_rs;
        g.c_row_stride = (int64_t)c_rs;
        g.sa_chunk_stride = (int64_t)sa_cs;
        g.a_batch = a->a_batch_stride ? a->a_batch_stride : (int64_t)((uint64_t)a->M * a_rs);
        g.b_batch = (int64_t)((uint64_t)a->N * b_row);
        g.c_batch = store == STORE_ACC ? (int64_t)a->M * a->N * 4 : (a->c_batch_stride ? a->c_batch_stride : (int64_t)((uint64_t)a->M * c_rs * 2));
        g.sa_batch = a->scale_a_batch_stride ? a->scale_a_batch_stride : (int64_t)((uint64_t)((a->M + 31) / 32) * sa_cs);
        g.sb_batch = (int64_t)((uint64_t)(a->N / 32) * chunk);
        hipError_t ge;
        const int splits = batch == 1 && c_rs == (uint64_t)a->N && store == STORE_C ? mx_general_splits(a->M, a->N, a->K) : 1;
        if (splits > 1 && a->workspace && aligned(a->workspace, 16) && a->workspace_bytes >= splitk_bytes(a->M, a->N, splits)) {
            MxGenParams part = g;
            part.c = a->workspace;
            part.splits = splits;
            ge = psg_launch_mx_generic(part, a->a_dtype, a->b_dtype, STORE_ACC, 1, static_cast<hipStream_t>(stream));
            A8W8Params q{};
            q.c = out;
            q.M = a->M;
            q.N = a->N;
            q.K = a->K;
            q.splits = splits;
            q.epi = EPI_NONE;
            q.out = a->out_dtype;
            if (ge == hipSuccess) ge = psg_launch_splitk_finalize(q, a->workspace, 0, 0, static_cast<hipStream_t>(stream));
        } else {
            ge = psg_launch_mx_generic(g, a->a_dtype, a->b_dtype, store, batch, static_cast<hipStream_t>(stream));
        }
        if (ge != hipSuccess) return hip_fail(ge, "psg_gemm_mxfp4 launch");
        g_err[0] = 0;
        return 0;
    }
    MxParams p;
    p.c = out;
    p.a = static_cast<const uint8_t*>(a->a);
    p.b = static_cast<const uint8_t*>(a->b);
    p.sa = static_cast<const uint8_t*>(a->scale_a);
    p.sb = static_cast<const uint8_t*>(a->scale_b);
    p.M = a->M;
    p.N = a->N;
    p.K = a->K;
    p.out = a->out_dtype;
    p.group_m = a->xcd_swizzle > 0 ? a->xcd_swizzle : 8;
    const bool small = a->force_path == 2 || (a->force_path == 0 && mx_takes_small(a->M, a->N, a->K));
    hipError_t e;
    if (small) {
        // four wavefronts x four K slices per workgroup when every slice still holds two 256-K steps, else eight
        const int kt = a->K / 256;
        const int nw = kt >= 8 ? 4 : 8;
        p.ksplit = pick_ksplit(a->N / 32, kt);
        if (p.ksplit > nw) p.ksplit = nw;
        if (nw == 4 && p.ksplit < 4) p.ksplit = 4;
        e = psg_launch_mxfp4_smallm(p, store, nw, static_cast<hipStream_t>(stream));
    } else {
        const bool forced = a->force_path == 1 && a->tile_m > 0 && a->tile_n > 0;
        const Plan plan = plan_tiled(a->M, a->N, a->K / 2, true);
        const Tile t = forced ? Tile{a->tile_m, a->tile_n, 4} : plan.t;
        int splits = forced ? (a->tile_k >= 1 && a->tile_k <= 16 ? a->tile_k : 1) : plan.splits;
        if (store != STORE_C || !a->workspace || !aligned(a->workspace, 16) || a->workspace_bytes < splitk_bytes(a->M, a->N, splits)) splits = 1;
        A8W8Params q{};
        q.c = p.c;
        q.a = p.a;
        q.b = p.b;
        q.mx_sa = p.sa;
        q.mx_sb = p.sb;
        q.M = p.M;
        q.N = p.N;
        q.K = p.K;
        q.group_m = p.group_m;
        q.ksplit = 1;
        q.wave_layout = a->reserved >= 2 ? a->reserved : (!forced && t.waves == 8 ? 8 : 1);
        q.splits = splits;
        q.epi = EPI_NONE;
        q.out = p.out;
        if (splits > 1) {
            A8W8Params part = q;
            part.c = a->workspace;
            e = psg_launch_a8w8_tiled(part, KIND_MXFP4, STORE_ACC, t.m, t.n, static_cast<hipStream_t>(stream));
            if (e == hipSuccess) e = psg_launch_splitk_finalize(q, a->workspace, 0, 0, static_cast<hipStream_t>(stream));
        } else {
            e = psg_launch_a8w8_tiled(q, KIND_MXFP4, store, t.m, t.n, static_cast<hipStream_t>(stream));
        }
    }
    if (e != hipSuccess) return hip_fail(e, "psg_gemm_mxfp4 launch");
    g_err[0] = 0;
    return 0;
}

int psg_gemm_mxfp4(const psg_mxfp4_args* args, void* stream) { return mx_common(args, args ? args->c : nullptr, STORE_C, stream); }

int psg_gemm_mxfp4_acc(const psg_mxfp4_args* args, void* acc, void* stream) { return mx_common(args, acc, STORE_ACC, stream); }

int psg_moe_gemm(const psg_moe_args* a, void* stream) {
    if (!a) return fail(PSG_E_NULL, "args is NULL");
    if (!a->out || !a->x || !a->w || !a->scale_x || !a->scale_w || !a->sorted_token_ids || !a->sorted_expert_ids || !a->num_valid_ids)
        return fail(PSG_E_NULL, "out, x, w, scale_x, scale_w, sorted_token_ids, sorted_expert_ids, num_valid_ids must be non-NULL");
    if (a->doweight && !a->sorted_weights) return fail(PSG_E_NULL, "sorted_weights must be non-NULL when doweight is set");
    if (a->stage != 1 && a->stage != 2) return fail(PSG_E_SHAPE, "stage=%d must be 1 or 2", a->stage);
    if (a->in_dtype != PSG_IN_INT8 && a->in_dtype != PSG_IN_FP8_E4M3FN && a->in_dtype != PSG_IN_INT8_W4)
        return fail(PSG_E_DTYPE, "in_dtype %d must be int8, fp8 or int8 with int4 weights", a->in_dtype);
    if (a->out_dtype < PSG_OUT_BF16 || a->out_dtype > PSG_OUT_F32) return fail(PSG_E_DTYPE, "out_dtype %d unknown", a->out_dtype);
    if (a->out_dtype == PSG_OUT_F32 && !(a->stage == 2 && a->accumulate))
        return fail(PSG_E_DTYPE, "fp32 output exists only for stage 2 with accumulate (kernels/moe/moe_gemm_2stage/gemm2.py:629)");
    if (a->x_slot_major != 0 && !(a->x_slot_major == 1 && a->stage == 1))
        return fail(PSG_E_SHAPE, "x_slot_major=%d must be 0, or 1 for stage 1", a->x_slot_major);
    if ((a->no_pairing != 0 && a->no_pairing != 1) || a->pad0 != 0) return fail(PSG_E_SHAPE, "no_pairing must be 0 or 1 and pad0 0");
    if (a->tokens < 1 || a->tokens >= (1 << 24)) return fail(PSG_E_SHAPE, "tokens=%d outside [1, 2^24)", a->tokens);
    if (a->topk < 1 || a->topk > 255) return fail(PSG_E_SHAPE, "topk=%d outside [1, 255]", a->topk);
    if (a->experts < 1) return fail(PSG_E_SHAPE, "experts=%d must be positive", a->experts);
    if (a->block_m != 16 && a->block_m != 32 && a->block_m != 64 && a->block_m != 128) return fail(PSG_E_SHAPE, "block_m=%d must be 16, 32, 64 or 128", a->block_m);
    if (a->blocks < 1 || a->blocks > 65535) return fail(PSG_E_SHAPE, "blocks=%d outside [1, 65535]", a->blocks);
    if (a->sorted_size < 1) return fail(PSG_E_SHAPE, "sorted_size=%d must be positive", a->sorted_size);
    const int K = a->stage == 1 ? a->model_dim : a->inter_dim, n_out = a->stage == 1 ? a->inter_dim : a->model_dim;
    if (K < 128 || K % 128) return fail(PSG_E_SHAPE, "K=%d of stage %d must be a positive multiple of 128", K, a->stage);
    if (n_out < 16 || n_out % 16) return fail(PSG_E_SHAPE, "output width %d of stage %d must be a positive multiple of 16", n_out, a->stage);
    const uint64_t rows_x = (a->stage == 1 && !a->x_slot_major) ? (uint64_t)a->tokens : (uint64_t)a->tokens * (uint64_t)a->topk;
    const uint64_t rows_e = a->stage == 1 ? 2ull * (uint64_t)n_out : (uint64_t)n_out;
    if (rows_x * (uint64_t)K > 0xFFFFFFF0ull) return fail(PSG_E_SHAPE, "x exceeds the 4 GiB descriptor range");
    if (rows_e * (uint64_t)K > 0xFFFFFFF0ull) return fail(PSG_E_SHAPE, "one expert's weights exceed the 4 GiB descriptor range");
    if (!aligned(a->x, 16) || !aligned(a->w, 16) || !aligned(a->scale_w, 16) || !aligned(a->out, 16))
        return fail(PSG_E_ALIGN, "x, w, scale_w and out must be 16-byte aligned");
    MoeParams p;
    p.out = a->out;
    p.x = static_cast<const uint8_t*>(a->x);
    p.w = static_cast<const uint8_t*>(a->w);
    p.sx = a->scale_x;
    p.sw = a->scale_w;
    p.sorted_ids = a->sorted_token_ids;
    p.expert_ids = a->sorted_expert_ids;
    p.sorted_w = a->sorted_weights;
    p.num_valid = a->num_valid_ids;
    p.x_slot_major = a->x_slot_major;
    p.pair_blocks = a->no_pairing ? 0 : 1;
    p.tokens = a->tokens;
    p.topk = a->topk;
    p.experts = a->experts;
    p.n_out = n_out;
    p.K = K;
    p.sorted_size = a->sorted_size;
    p.out_dtype = a->out_dtype;
    p.doweight = a->doweight ? 1 : 0;
    p.accumulate = a->stage == 2 && a->accumulate ? 1 : 0;
    const hipError_t e = psg_launch_moe_gemm(p, a->in_dtype == PSG_IN_INT8 ? KIND_INT8 : a->in_dtype == PSG_IN_INT8_W4 ? KIND_INT8W4 : KIND_FP8, a->stage, a->block_m, a->blocks, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, "psg_moe_gemm launch");
    g_err[0] = 0;
    return 0;
}

namespace {
int moe_reduce_common(const void* x, void* y, const int32_t* mask, const int32_t* ids, int32_t tokens, int32_t topk, int32_t model_dim,
                      int32_t experts, int32_t dtype, void* stream) {
    if (!x || !y) return fail(PSG_E_NULL, "x and y must be non-NULL");
    if (dtype != PSG_OUT_BF16 && dtype != PSG_OUT_FP16 && dtype != PSG_OUT_F32) return fail(PSG_E_DTYPE, "dtype %d must be bf16, fp16 or fp32", dtype);
    if (tokens < 1 || topk < 1 || model_dim < 4 || model_dim % 4) return fail(PSG_E_SHAPE, "need tokens, topk >= 1 and model_dim a positive multiple of 4");
    const int al = dtype == PSG_OUT_F32 ? 16 : 8;
    if (!aligned(x, al) || !aligned(y, al)) return fail(PSG_E_ALIGN, "x and y must be %d-byte aligned", al);
    if (mask && (!ids || experts < 1)) return fail(PSG_E_NULL, "an expert mask needs topk_ids and experts >= 1");
    const hipError_t e = psg_launch_moe_reduce(x, y, tokens, topk, model_dim, dtype, mask, ids, experts, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, "psg_moe_reduce launch");
    g_err[0] = 0;
    return 0;
}
}  // namespace

int psg_moe_mx_scale_sort(const void* scale, const int32_t* sorted_token_ids, const int32_t* num_valid_ids, void* out, int32_t tokens, int32_t topk,
                          int32_t cols, int32_t sorted_size, void* stream) {
    if (!scale || !sorted_token_ids || !num_valid_ids || !out) return fail(PSG_E_NULL, "scale, sorted_token_ids, num_valid_ids and out must be non-NULL");
    if (tokens < 1 || tokens >= (1 << 24)) return fail(PSG_E_SHAPE, "tokens=%d outside [1, 2^24)", tokens);
    if (topk < 1 || topk > 255) return fail(PSG_E_SHAPE, "topk=%d outside [1, 255]", topk);
    if (cols < 8 || cols % 8) return fail(PSG_E_SHAPE, "cols=%d must be a positive multiple of 8", cols);
    if (sorted_size < 1) return fail(PSG_E_SHAPE, "sorted_size=%d must be positive", sorted_size);
    if (((int64_t)sorted_size + 31) / 32 * 8 * (int64_t)cols > 0x7FFFFFFFll) return fail(PSG_E_SHAPE, "sorted_size * cols exceeds 2^33 bytes");
    if (!aligned(out, 4)) return fail(PSG_E_ALIGN, "out must be 4-byte aligned");
    const hipError_t e = psg_launch_moe_mx_scale_sort(scale, sorted_token_ids, num_valid_ids, out, tokens, topk, cols, sorted_size, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, "psg_moe_mx_scale_sort launch");
    g_err[0] = 0;
    return 0;
}

int psg_moe_mx_gemm(const psg_moe_mx_args* a, void* stream) {
    if (!a) return fail(PSG_E_NULL, "args is NULL");
    const bool inline_quant = a->stage == 1 && a->a_dtype == PSG_MX_BF16_QUANT;
    if (!a->out || !a->a || (!a->a_scale && !inline_quant) || !a->w || !a->w_scale || !a->sorted_token_ids || !a->sorted_expert_ids || !a->num_valid_ids)
        return fail(PSG_E_NULL, "out, a, a_scale, w, w_scale, sorted_token_ids, sorted_expert_ids and num_valid_ids must be non-NULL");
    if (a->stage != 1 && a->stage != 2) return fail(PSG_E_SHAPE, "stage=%d must be 1 or 2", a->stage);
    if (a->stage == 1 && !a->out_scale) return fail(PSG_E_NULL, "out_scale must be non-NULL in stage 1");
    if (a->stage == 2 && a->atomic && !a->sorted_weights) return fail(PSG_E_NULL, "sorted_weights must be non-NULL for the atomic epilogue");
    if (a->pad0 != 0) return fail(PSG_E_SHAPE, "pad0 must be 0");
    if (a->stage == 1 ? (a->a_dtype != PSG_MX_FP4 && a->a_dtype != PSG_MX_FP8 && a->a_dtype != PSG_MX_BF16_QUANT) : a->a_dtype != PSG_MX_FP4)
        return fail(PSG_E_DTYPE, "a_dtype %d: stage 1 takes 0 (fp4), 2 (fp8) or 3 (bf16, quantised by the kernel), stage 2 takes 0 (fp4)", a->a_dtype);
    if (a->stage == 2 && a->out_dtype != PSG_OUT_BF16 && a->out_dtype != PSG_OUT_FP16) return fail(PSG_E_DTYPE, "out_dtype %d unknown", a->out_dtype);
    if (a->block_m != 16 && a->block_m != 32 && a->block_m != 64 && a->block_m != 128) return fail(PSG_E_SHAPE, "block_m=%d must be 16, 32, 64 or 128", a->block_m);
    if (a->stage == 1 && (a->block_m == 16) != inline_quant)
        return fail(PSG_E_SHAPE, "stage 1: blocks of 16 rows go with a_dtype 3 (bf16 activations quantised by the kernel) and only with it, got block_m=%d a_dtype=%d", a->block_m, a->a_dtype);
    if (a->tokens < 1 || a->tokens >= (1 << 24)) return fail(PSG_E_SHAPE, "tokens=%d outside [1, 2^24)", a->tokens);
    if (a->experts < 1) return fail(PSG_E_SHAPE, "experts=%d must be positive", a->experts);
    if (a->model_dim < 256 || a->model_dim % 256) return fail(PSG_E_SHAPE, "model_dim=%d must be a positive multiple of 256", a->model_dim);
    if (a->inter_dim < 256 || a->inter_dim % 256) return fail(PSG_E_SHAPE, "inter_dim=%d must be a positive multiple of 256", a->inter_dim);
    if (a->sorted_size < a->block_m) return fail(PSG_E_SHAPE, "sorted_size=%d is below one block of %d rows", a->sorted_size, a->block_m);
    if (a->blocks < 1) return fail(PSG_E_SHAPE, "blocks=%d must be positive", a->blocks);
    if ((int64_t)a->blocks * a->block_m > (int64_t)a->sorted_size)
        return fail(PSG_E_SHAPE, "blocks=%d of %d rows exceed sorted_size=%d", a->blocks, a->block_m, a->sorted_size);
    const int K = a->stage == 1 ? a->model_dim : a->inter_dim;
    const int n_out = a->stage == 1 ? a->inter_dim : a->model_dim;
    const uint64_t a_row = inline_quant ? 2ull * (uint64_t)K : a->a_dtype == PSG_MX_FP8 ? (uint64_t)K : (uint64_t)K / 2;
    const uint64_t a_rows = a->stage == 1 ? (uint64_t)a->tokens : (uint64_t)a->sorted_size;
    const uint64_t rows_e = a->stage == 1 ? 2ull * (uint64_t)n_out : (uint64_t)n_out;
    if (a_rows * a_row > 0xFFFFFFF0ull) return fail(PSG_E_SHAPE, "a exceeds the 4 GiB descriptor range");
    if (rows_e * (uint64_t)(K / 2) > 0xFFFFFFF0ull) return fail(PSG_E_SHAPE, "one expert's weights exceed the 4 GiB descriptor range");
    if (!aligned(a->a, 16) || !aligned(a->w, 16) || (!inline_quant && !aligned(a->a_scale, 4)) || !aligned(a->w_scale, 4) || !aligned(a->out, 16))
        return fail(PSG_E_ALIGN, "a, w and out must be 16-byte aligned, a_scale and w_scale 4-byte aligned");
    MoeMxParams p;
    p.out = a->out;
    p.out_scale = static_cast<uint8_t*>(a->out_scale);
    p.a = static_cast<const uint8_t*>(a->a);
    p.a_scale = static_cast<const uint8_t*>(a->a_scale);
    p.w = static_cast<const uint8_t*>(a->w);
    p.w_scale = static_cast<const uint8_t*>(a->w_scale);
    p.sorted_ids = a->sorted_token_ids;
    p.expert_ids = a->sorted_expert_ids;
    p.sorted_w = a->sorted_weights;
    p.num_valid = a->num_valid_ids;
    p.tokens = a->tokens;
    p.experts = a->experts;
    p.n_out = n_out;
    p.K = K;
    p.sorted_size = a->sorted_size;
    p.out_dtype = a->out_dtype;
    p.atomic = a->stage == 2 && a->atomic ? 1 : 0;
    p.eshift = 0;
    p.n_tiles = p.n_groups = p.by_expert = p.quad_tiles = 0;
    if (((int64_t)a->blocks << 1) * (int64_t)((n_out / 128 + 7) / 8 * 8) > 0x7FFFFFFFll) return fail(PSG_E_SHAPE, "blocks=%d times the column tiles exceed the grid", a->blocks);
    const hipError_t e = psg_launch_moe_mx_gemm(p, a->a_dtype == PSG_MX_FP8 ? MXF_FP8 : MXF_FP4, a->stage, a->block_m, a->blocks, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, "psg_moe_mx_gemm launch");
    g_err[0] = 0;
    return 0;
}

int psg_moe_reduce(const void* x, void* y, int32_t tokens, int32_t topk, int32_t model_dim, int32_t dtype, void* stream) {
    return moe_reduce_common(x, y, nullptr, nullptr, tokens, topk, model_dim, 0, dtype, stream);
}

int psg_moe_reduce_masked(const void* x, void* y, const int32_t* expert_mask, const int32_t* topk_ids, int32_t tokens, int32_t topk,
                          int32_t model_dim, int32_t experts, int32_t dtype, void* stream) {
    if (!expert_mask || !topk_ids) return fail(PSG_E_NULL, "expert_mask and topk_ids must be non-NULL");
    return moe_reduce_common(x, y, expert_mask, topk_ids, tokens, topk, model_dim, experts, dtype, stream);
}

uint64_t psg_moe_sorting_workspace_bytes(int32_t tokens, int32_t topk, int32_t experts) {
    if (tokens < 1 || topk < 1 || experts < 1) return 0;
    return psg_moe_sort_workspace((int64_t)tokens * topk, experts);
}

int psg_moe_sorting(const psg_moe_sort_args* a, void* stream) {
    MoeSortParams p;
    if (int rc = check_moe_sort(a, true, &p)) return rc;
    const hipError_t e = psg_launch_moe_sort(p, a->workspace, a->workspace ? a->workspace_bytes : 0, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, "psg_moe_sorting launch");
    g_err[0] = 0;
    return 0;
}

int psg_moe_topk_gating(const psg_moe_gating_args* a, void* stream) {
    MoeGatingParams g;
    if (int rc = check_moe_gating(a, true, &g)) return rc;
    const hipError_t e = psg_launch_moe_gating(g, a->dtype, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, "psg_moe_topk_gating launch");
    g_err[0] = 0;
    return 0;
}

int psg_moe_softmax_sorting_fused(int32_t tokens, int32_t topk, int32_t experts) {
    return tokens >= 1 && topk >= 1 && experts >= 1 && psg_moe_gate_sort_fuses(tokens, topk, experts) ? 1 : 0;
}

int psg_moe_softmax_sorting(const psg_moe_gating_args* ga, const psg_moe_sort_args* sa, void* stream) {
    if (!ga || !sa) return fail(PSG_E_NULL, "args is NULL");
    if (ga->tokens != sa->tokens || ga->topk != sa->topk || ga->experts != sa->experts)
        return fail(PSG_E_SHAPE, "gating (tokens=%d topk=%d experts=%d) and sorting (tokens=%d topk=%d experts=%d) disagree", ga->tokens,
                    ga->topk, ga->experts, sa->tokens, sa->topk, sa->experts);
    const bool fused = ga->tokens >= 1 && ga->topk >= 1 && ga->experts >= 1 && psg_moe_gate_sort_fuses(ga->tokens, ga->topk, ga->experts);
    MoeGatingParams g;
    MoeSortParams p;
    if (int rc = check_moe_gating(ga, !fused, &g)) return rc;
    if (int rc = check_moe_sort(sa, false, &p)) return rc;
    hipError_t e;
    if (fused) {
        e = psg_launch_moe_gate_sort(p, g, ga->dtype, static_cast<hipStream_t>(stream));
    } else {
        // two steps: the sorter reads what the gating kernel wrote
        if ((const void*)sa->topk_ids != (const void*)ga->indices || (const void*)sa->topk_weights != (const void*)ga->weights)
            return fail(PSG_E_NULL, "beyond the fused range the sorter's topk_ids / topk_weights must be the gating's indices / weights");
        e = psg_launch_moe_gating(g, ga->dtype, static_cast<hipStream_t>(stream));
        if (e == hipSuccess) e = psg_launch_moe_sort(p, sa->workspace, sa->workspace ? sa->workspace_bytes : 0, static_cast<hipStream_t>(stream));
    }
    if (e != hipSuccess) return hip_fail(e, "psg_moe_softmax_sorting launch");
    g_err[0] = 0;
    return 0;
}

int psg_quant_pertoken(const void* x, int32_t x_dtype, void* y, float* scale, int32_t M, int32_t K, int32_t out_dtype, void* stream) {
    if (!x || !y || !scale) return fail(PSG_E_NULL, "x, y and scale must be non-NULL");
    if (x_dtype < 0 || x_dtype > 2) return fail(PSG_E_DTYPE, "x_dtype %d unknown (0 fp32, 1 bf16, 2 fp16)", x_dtype);
    if (out_dtype != PSG_IN_INT8 && out_dtype != PSG_IN_FP8_E4M3FN) return fail(PSG_E_DTYPE, "out_dtype must be int8 or fp8");
    if (M < 1 || K < 8 || K % 8) return fail(PSG_E_SHAPE, "need M >= 1 and K a positive multiple of 8 (got M=%d K=%d)", M, K);
    if (!aligned(x, 16) || !aligned(y, 8)) return fail(PSG_E_ALIGN, "x must be 16-byte and y 8-byte aligned");
    const hipError_t e = psg_launch_quant_pertoken(x, x_dtype, y, scale, M, K, out_dtype == PSG_IN_FP8_E4M3FN, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, "psg_quant_pertoken launch");
    g_err[0] = 0;
    return 0;
}

int psg_quant_mxfp4(const void* x, int32_t x_dtype, void* packed, void* scales, int32_t M, int32_t K, int32_t shuffled, void* stream) {
    if (!x || !packed || !scales) return fail(PSG_E_NULL, "x, packed and scales must be non-NULL");
    if (x_dtype < 0 || x_dtype > 2) return fail(PSG_E_DTYPE, "x_dtype %d unknown (0 fp32, 1 bf16, 2 fp16)", x_dtype);
    if (M < 1 || K < 32 || K % 32) return fail(PSG_E_SHAPE, "need M >= 1 and K a positive multiple of 32 (got M=%d K=%d)", M, K);
    if (shuffled && K % 256) return fail(PSG_E_SHAPE, "the shuffled scale layout needs K %% 256 == 0 (got K=%d)", K);
    if (!aligned(x, 16) || !aligned(packed, 16)) return fail(PSG_E_ALIGN, "x and packed must be 16-byte aligned");
    const int R = (M + 31) / 32 * 32;  // scales cover whole 32-row chunks; the padding rows get scale byte 0
    const hipError_t e = psg_launch_quant_mxfp4(x, x_dtype, packed, scales, M, R, K, shuffled, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, "psg_quant_mxfp4 launch");
    g_err[0] = 0;
    return 0;
}

}  // extern "C"
