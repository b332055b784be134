// C ABI of libfp8bs.so (declared in include/fp8bs.h): argument checking, the shape-family planner
// and kernel launches.  Host code only; the device code is in fp8bs_kernels.hip.
//
// This layer stands where the reference has its launcher `fp8_mm(...)`
// (1-amd-fp8-mm/amd-fp8-mm-submission.py:514-579).  Differences by design: it is stream-aware,
// returns a status instead of void, never writes the inputs, and picks kernels by shape family
// instead of an exact-shape table.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include <stdlib.h>
#include <unistd.h>
#include <atomic>
#include <chrono>

#include "fp8bs.h"
#include "fp8bs_kernels.h"

namespace {

constexpr int KBLK = 128;

struct VariantInfo { int bm, bn, threads; };

bool variant_info(int variant, VariantInfo* out) {
    switch (variant) {
        case FP8BS_VARIANT_GENERIC:  *out = {16, 16, 256}; return true;
        case FP8BS_VARIANT_T256x256: *out = {256, 256, 512}; return true;
        case FP8BS_VARIANT_T128x128: *out = {128, 128, 256}; return true;
        case FP8BS_VARIANT_T64x128:  *out = {64, 128, 256}; return true;
        case FP8BS_VARIANT_T256x128: *out = {256, 128, 512}; return true;
        case FP8BS_VARIANT_SKINNY64x144: *out = {64, 144, 256}; return true;
        case FP8BS_VARIANT_SKINNY64x256: *out = {64, 256, 256}; return true;
        case FP8BS_VARIANT_SKINNY64x288: *out = {64, 288, 256}; return true;
        case FP8BS_VARIANT_T256x192: *out = {256, 192, 512}; return true;
        case FP8BS_VARIANT_T256x128S3: *out = {256, 128, 512}; return true;
        case FP8BS_VARIANT_T192x192S3: *out = {192, 192, 512}; return true;
        case FP8BS_VARIANT_T64x256S3: *out = {64, 256, 512}; return true;
        default: return false;
    }
}

inline long cdiv(long a, long b) { return (a + b - 1) / b; }

// Workgroups of a call that deals K blocks instead of tiles: one per place on the chip (what the tile's LDS
// and thread count let a CU hold), never more than there are (tile, K block) pairs.
int streamk_grid(int variant, int m, int n, int k, int num_cus) {
    VariantInfo vi{};
    if (!variant_info(variant, &vi) || variant == FP8BS_VARIANT_GENERIC || k < KBLK) return 0;
    const int lds = fp8bs::variant_lds_bytes(variant);
    if (lds <= 0 || lds > 163840) return 0;
    if (num_cus <= 0) num_cus = 256;
    const long by_lds = 163840 / lds, by_threads = 2048 / vi.threads;
    long g = (long)num_cus * (by_lds < by_threads ? by_lds : by_threads);
    const long pairs = cdiv(m, vi.bm) * cdiv(n, vi.bn) * (k / KBLK);
    if (pairs >= (1L << 31)) return 0;                  // the kernel counts the pairs in 32 bits
    g = g < pairs ? g : pairs;
    return (int)(g < fp8bs::StreamK::MAX_GRID ? g : fp8bs::StreamK::MAX_GRID);
}

bool is_streaming_variant(int v) { return v == FP8BS_VARIANT_SKINNY64x144 || v == FP8BS_VARIANT_SKINNY64x256 || v == FP8BS_VARIANT_SKINNY64x288; }

// The fp32 partial planes of a K split followed by the reduce kernel.
uint64_t planes_bytes(int m, int n, int split_k) { return split_k > 1 ? (uint64_t)split_k * (uint64_t)m * (uint64_t)n * 4u : 0u; }

// Can the partial tiles of a K split of this tile shape be summed in the kernel that writes them (one counter per
// tile in the head of the workspace, the partition count in the counter's low 16 bits)?
bool can_sum_in_kernel(int m, int n, int variant, int split_k) {
    VariantInfo vi{};
    if (variant == FP8BS_VARIANT_GENERIC || is_streaming_variant(variant) || !variant_info(variant, &vi)) return false;
    return split_k >= 2 && split_k <= 255 && cdiv(m, vi.bm) * cdiv(n, vi.bn) <= fp8bs::StreamK::MAX_GRID;
}

// Fill a plan for a given variant and split count.  in_kernel: the split's partial tiles are summed by the last
// workgroup to finish each tile (where the shape allows it, see above; else the reduce kernel follows).
void fill_plan(int m, int n, int k, int variant, int split_k, fp8bs_plan_t* out, int stream_k = 0, bool in_kernel = false) {
    VariantInfo vi{};
    variant_info(variant, &vi);
    int kbt = k / KBLK;
    if (variant == FP8BS_VARIANT_GENERIC) { split_k = 1; stream_k = 0; }
    if (stream_k > 0) split_k = 1;
    if (split_k < 1) split_k = 1;
    if (split_k > kbt) split_k = kbt > 0 ? kbt : 1;
    out->variant = variant;
    out->tile_m = vi.bm;
    out->tile_n = vi.bn;
    out->split_k = split_k;
    out->block_threads = vi.threads;
    out->lds_bytes = fp8bs::variant_lds_bytes(variant);
    out->stream_k = stream_k > 0 ? stream_k : 0;
    out->sum_in_kernel = in_kernel && stream_k <= 0 && can_sum_in_kernel(m, n, variant, split_k) ? 1 : 0;
    out->reserved = 0;
    if (variant == FP8BS_VARIANT_GENERIC) {
        out->grid_x = (int)cdiv(n, 16); out->grid_y = (int)cdiv(m, 16); out->grid_z = 1;
    } else {
        out->grid_x = stream_k > 0 ? stream_k : (int)(cdiv(m, vi.bm) * cdiv(n, vi.bn) * split_k); out->grid_y = 1; out->grid_z = 1;
    }
    if (stream_k > 0) out->workspace_bytes = (uint64_t)fp8bs::StreamK::bytes(stream_k, vi.bm, vi.bn);
    else if (out->sum_in_kernel)   // the counters, then one fp32 tile per (tile, K partition)
        out->workspace_bytes = (uint64_t)fp8bs::StreamK::SLOTS_OFF + (uint64_t)(cdiv(m, vi.bm) * cdiv(n, vi.bn)) * (uint64_t)split_k * (uint64_t)vi.bm * (uint64_t)vi.bn * 4u;
    else out->workspace_bytes = planes_bytes(m, n, split_k);
}

// Rows of c (n bf16) that keep 16-byte stores aligned: what the streaming kernels need (forced variants only;
// the tiled kernels take any m and n in every mode: they repair the last bytes of a and b themselves, store a
// row's last chunk of c in pieces and write the partial planes of a K split element by element where rows do not
// end on a group of four).
bool vector_shape(int n) { return (n % 8) == 0; }

// At most 64 rows against a b of 24 MB or more: the call streams b from HBM once and everything else is small.
bool skinny_shape(int m, int n, int k) { return m <= 64 && (double)n * (double)k >= 24.0e6; }

// The tile shape and K split of the tiled MFMA kernel that finish soonest (any m, any n).
void choose_tiled(int m, int n, int k, int num_cus, fp8bs_plan_t* out, bool may_split = true) {
    if (num_cus <= 0) num_cus = 256;
    int kbt = k / KBLK;
    // The tile shape and K split that finish soonest under a cost model in microseconds.  A workgroup advances one
    // K block in max(t_alone x f(r), t_power x w / CUs): t_alone is the tile's time per block at the full clock
    // (f(r) = 1, 1.30, 1.71 with r = 1, 2, 3 workgroups sharing a CU), t_power what the board's power limit allows
    // when every CU runs one such workgroup - with w workgroups running together the limit is shared by w, so fewer
    // busy CUs clock higher until the full clock is reached.  A round of workgroups (CUs x the most that fit a CU; a
    // last partial round with fewer) costs a fixed time for the first copies' latency, the output and the drain.  A
    // K split adds the fp32 partial planes (written and read back, mostly through the 256 MB cache) and the reduce
    // launch.  The constants are a least-squares fit (of logarithms) of this model to the measured time of every
    // (tile, split) pair on 38 shapes on MI355X - the 18 of the upstream benchmark and 20 others, M 96 .. 16384,
    // N 1024 .. 28672, K 1024 .. 14336 - (rms error 10 %; picking by the model costs 1.2 % against picking the
    // measured best, geometric mean over the shapes, worst shape +13 %).
    struct Cand { int variant; int rmax; double t_alone, t_power, t_fixed; };
    const Cand cands[7] = {
        {FP8BS_VARIANT_T256x256, 1, 1.181, 1.462, 6.75},
        {FP8BS_VARIANT_T256x192, 1, 1.011, 1.163, 5.51},
        {FP8BS_VARIANT_T192x192S3, 1, 0.881, 1.059, 4.11},
        {FP8BS_VARIANT_T256x128S3, 1, 0.783, 0.906, 3.70},
        {FP8BS_VARIANT_T128x128, 2, 0.797, 0.570, 2.86},
        {FP8BS_VARIANT_T64x128, 3, 0.645, 0.400, 1.91},
        // the 64x256 three-stage tile: many small tiles and a deep copy ring; what shapes of a few hundred rows, or
        // with few K blocks per tile, finish soonest on (1536 x 1536 x 4096: 21.4 us against 25.0 with the best of the others)
        {FP8BS_VARIANT_T64x256S3, 1, 0.576, 0.618, 2.03},
    };
    const double shared[3] = {1.0, 1.30, 1.71};
    const int splits[6] = {1, 2, 3, 4, 6, 8};
    int best_variant = 0, best_split = 1; double best_cost = 0; bool best_fused = false;
    for (const Cand& c : cands) {
        VariantInfo vi{};
        variant_info(c.variant, &vi);
        const long tiles = cdiv(m, vi.bm) * cdiv(n, vi.bn);
        auto t_block = [&](long w) {          // w workgroups running together
            const long r = cdiv(w, num_cus) < c.rmax ? cdiv(w, num_cus) : c.rmax;
            const double alone = c.t_alone * shared[r - 1], power = c.t_power * (double)w / (double)num_cus;
            return alone > power ? alone : power;
        };
        for (int s : splits) {
            // keep at least 4 K blocks per workgroup - 8 with the 64x256 tile, whose short blocks leave a workgroup's
            // first copies and its partial plane as most of its time (1024 x 512 x 7168: split 8 20.9 us, split 4 18.6)
            if (s > 1 && (kbt / s < (c.variant == FP8BS_VARIANT_T64x256S3 ? 8 : 4) || !may_split)) continue;
            const long wgs = tiles * s, per_round = (long)num_cus * c.rmax;
            const long full = wgs / per_round, rem = wgs % per_round;
            const double kb = (double)cdiv(kbt, s);
            double cost = (double)full * (c.t_fixed + kb * t_block(per_round));
            if (rem) cost += c.t_fixed + kb * t_block(rem);
            // the planes and the reduce launch; or, with two or three partitions, the sum in the kernel: no second
            // launch and no pass over whole planes, but the last workgroup of a tile reads s - 1 partial tiles alone
            // (measured on the same 38 shapes: two partitions 1-50 us faster than with the reduce launch, median 4.7;
            // three: median 2.3 faster; four and more: the serial sums cost more than the launch)
            const double planes = 4.85 + 1.10e-6 * s * (double)m * (double)n;
            const double in_kernel = 3.77 + 0.752e-6 * s * (double)m * (double)n
                                     + 5.90 * (s - 1) * (vi.bm * vi.bn * 4e-6) * (double)cdiv(wgs, num_cus);
            const bool fuse = (s == 2 || s == 3) && can_sum_in_kernel(m, n, c.variant, s) && in_kernel < planes;
            if (s > 1) cost += fuse ? in_kernel : planes;
            if (best_variant == 0 || cost < best_cost) { best_variant = c.variant; best_split = s; best_cost = cost; best_fused = fuse; }
        }
    }
    fill_plan(m, n, k, best_variant, best_split, out, 0, best_fused);
}

// Skinny shapes: the 64 x 256 tile with three LDS stages (two K blocks of b, 64 KB, in flight per workgroup) and
// the K split that finishes soonest under a model in microseconds: a workgroup advances one K block in the time
// the workgroups running together need to pull their 32 KB of b each from HBM at 5.5 TB/s, and never faster than
// the 1.05 us a block's copies take to arrive; 2 us per round for the first block and the output; the partial
// planes and the reduce launch as for the other tiles, with 4 us for the launch (the main kernel is short).
// Measured with b streamed from HBM (inputs rotated through more than the 256 MB cache) against the 64 x 144
// streaming kernel and the 64 x 128 tile: 64 x 18432 x 7168 34.3 us (split 3) against 37.7 and 38.4;
// 64 x 7168 x 7168 20.4 against 32.4 and 21.0; 1 x 18432 x 7168 29.2 against 31.8 and 34.1;
// 1 x 28672 x 4096 26.7 against 34.6 and 30.6.
void choose_skinny(int m, int n, int k, int num_cus, fp8bs_plan_t* out, bool may_split = true) {
    if (num_cus <= 0) num_cus = 256;
    const int kbt = k / KBLK;
    const long tiles = cdiv(m, 64) * cdiv(n, 256);
    int best_s = 1; double best = 0; bool best_fused = false;
    for (int s = 1; s <= 8 && s <= kbt; s++) {
        if (s > 1 && !may_split) break;
        const long wgs = tiles * s;
        const double together = (double)(wgs < num_cus ? wgs : num_cus);
        double t_block = together * 32768.0 / 5.5e6;
        if (t_block < 1.05) t_block = 1.05;
        double cost = (double)cdiv(wgs, num_cus) * (2.0 + (double)cdiv(kbt, s) * t_block);
        if (s > 1) cost += 4.0 + 0.24 * s + 1.19e-6 * s * (double)m * (double)n;
        // Two or three partitions in one round of workgroups are summed in the kernel where the planes are large
        // enough for the reduce launch to cost more than the chain of round trips that replaces it (the partial
        // tile's acknowledged stores, the count, the last workgroup's reads).  b from HBM, three partitions of
        // 18432 x 7168: 64 rows 33.7 us against 34.4 with the reduce launch, 16 rows 30.3 against 29.3, one row 31.0
        // against 29.0; two partitions of 64 rows 37.4 against 38.6, four 52.8 against 49.6.
        const double in_kernel = 2.05 - 0.78e-6 * s * (double)m * (double)n;
        const bool fuse = (s == 2 || s == 3) && wgs <= num_cus && in_kernel < 0 && can_sum_in_kernel(m, n, FP8BS_VARIANT_T64x256S3, s);
        if (fuse) cost += in_kernel;
        if (s == 1 || cost < best) { best = cost; best_s = s; best_fused = fuse; }
    }
    fill_plan(m, n, k, FP8BS_VARIANT_T64x256S3, best_s, out, 0, best_fused);
}

// Shape-family rule.  A few rows against a large b -> the 64 x 256 three-stage tile.  Everything else -> the
// tile and K split that the cost model of the tiled kernel picks.
void choose(int m, int n, int k, int num_cus, fp8bs_plan_t* out, bool may_split = true) {
    if (skinny_shape(m, n, k)) choose_skinny(m, n, k, num_cus, out, may_split);
    else choose_tiled(m, n, k, num_cus, out, may_split);
}

// Order of the tiles of a grouped call (the row counts themselves are on the device).  With a tile or more of
// rows per expert on average the tiles go expert by expert: the tile that holds an expert's last rows then runs
// beside the full tiles that read the same weights (32 experts of 1040 rows x 4096 x 7168: 956 us against 1014;
// configuration 5: 2-3 % faster).  With fewer rows every expert is one tile row and the call streams the weights;
// the order across the experts is then 0.7-1.2 % ahead (8 or 100 rows per expert), so it is kept there.
int group_order(int total_rows, int num_experts) { return (long)total_rows >= 256L * num_experts ? 1 : 0; }

// The value a flag takes in one call that deals K blocks: never zero, different from call to call (and, through
// the clock and the process id, from run to run), so that whatever an earlier call or an uninitialised workspace
// left in a flag is not mistaken for this call's.
unsigned long long next_nonce() {
    static std::atomic<unsigned long long> counter{0};
    static const unsigned long long seed = ((unsigned long long)std::chrono::steady_clock::now().time_since_epoch().count() * 0x9E3779B97F4A7C15ull)
                                           ^ ((unsigned long long)getpid() << 32);
    unsigned long long x = seed + (counter.fetch_add(1, std::memory_order_relaxed) + 1) * 0xD1342543DE82EF95ull;
    return x ? x : 1ull;
}

// Polls of one flag before a workgroup's wait gives up (each poll is a round trip to memory plus a short sleep,
// about a microsecond: the default is a quarter of a second or so).  FP8BS_STREAMK_SPIN overrides it; a negative
// value makes every such wait give up at once, which exercises the error path without a kernel that hangs.
int streamk_spin_limit() {
    static const int limit = [] {
        const char* e = getenv("FP8BS_STREAMK_SPIN");
        return e && *e ? atoi(e) : (1 << 18);
    }();
    return limit;
}


int check_common(const void* a, const void* b, const float* as, const float* bs, void* c, int m, int n, int k) {
    if (m < 0 || n < 0 || k < 0 || (k % KBLK) != 0) return FP8BS_ERR_BAD_SHAPE;
    if (m == 0 || n == 0) return FP8BS_OK;   // nothing to write
    if (!a || !b || !as || !bs || !c) {
        if (k == 0 && c) return FP8BS_OK;
        return FP8BS_ERR_NULL_POINTER;
    }
    if ((uint64_t)m * (uint64_t)k >= (1ull << 32) || (uint64_t)n * (uint64_t)k >= (1ull << 32)) return FP8BS_ERR_TOO_LARGE;
    if ((((uintptr_t)as | (uintptr_t)bs) & 3) != 0 || ((uintptr_t)c & 1) != 0) return FP8BS_ERR_BAD_SHAPE;   // element alignment
    return FP8BS_OK;
}

// Operands and output on 16-byte boundaries: what the streaming kernels need (aligned 8- and 16-byte stores
// of c, aligned copies).
bool vector_aligned(const void* a, const void* b, const void* c) {
    return ((((uintptr_t)a | (uintptr_t)b | (uintptr_t)c) & 15) == 0);
}

}  // namespace

// ---- built-in K-split scratch of fp8bs_gemm_noalloc ---------------------------------------------------
// Device memory that belongs to the library's code object: every GPU the library runs on holds its own
// copy, at its own address, until the process ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress; the address it yields (looked up once per device, with that device current) is what
// kernels, copies and fills are given.
static __device__ __align__(256) unsigned char scratch[FP8BS_NOALLOC_SCRATCH_BYTES];
static void* scratch_ptr[fp8bs::MAX_DEVICES];

static int scratch_address(void** out, hipStream_t stream) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= fp8bs::MAX_DEVICES) return FP8BS_ERR_LAUNCH;
    void* p = __atomic_load_n(&scratch_ptr[dev], __ATOMIC_ACQUIRE);
    if (!p) {
        // the lookup is no stream operation: it must not fall into a capture (the caller makes one eager call first)
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &cap) != hipSuccess) { (void)hipGetLastError(); cap = hipStreamCaptureStatusNone; }
        if (cap != hipStreamCaptureStatusNone) return FP8BS_ERR_CAPTURE;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return FP8BS_ERR_LAUNCH;
        __atomic_store_n(&scratch_ptr[dev], p, __ATOMIC_RELEASE);     // the same value from every thread
    }
    *out = p;
    return FP8BS_OK;
}

extern "C" {

int fp8bs_version(void) { return 300; }      // 0.3.0: fp8bs_plan_t grew (sum_in_kernel)

const char* fp8bs_strerror(int status) {
    switch (status) {
        case FP8BS_OK: return "success";
        case FP8BS_ERR_NULL_POINTER: return "a required pointer is NULL";
        case FP8BS_ERR_BAD_SHAPE: return "bad shape: m, n, k must be non-negative and k a multiple of 128 (or a pointer is not aligned to its element type)";
        case FP8BS_ERR_WORKSPACE: return "workspace missing or smaller than fp8bs_workspace_bytes()";
        case FP8BS_ERR_TOO_LARGE: return "operand exceeds the 4 GiB buffer-addressing limit (m*k or n*k >= 2^32)";
        case FP8BS_ERR_LAUNCH: return "kernel launch failed";
        case FP8BS_ERR_BAD_OFFSETS: return "grouped: num_experts must be positive";
        case FP8BS_ERR_BAD_VARIANT: return "unknown or inapplicable kernel variant";
        case FP8BS_ERR_CAPTURE: return "fp8bs_gemm_noalloc: the first call on a device looks up the built-in scratch and must be made outside stream capture";
        case FP8BS_ERR_TIMEOUT: return "a workgroup gave up waiting for another workgroup's partial tile (status word of the workspace); the output of that call is not valid";
        case FP8BS_ERR_SCRATCH_LIMIT: return "fp8bs_gemm_noalloc: the K split planned for this shape needs more than the built-in scratch (FP8BS_NOALLOC_SCRATCH_BYTES); use fp8bs_gemm with a caller workspace";
        default: return "unknown fp8bs status";
    }
}

int fp8bs_plan(int m, int n, int k, int num_cus, fp8bs_plan_t* out) {
    if (!out) return FP8BS_ERR_NULL_POINTER;
    if (m <= 0 || n <= 0 || k <= 0 || (k % KBLK) != 0) return FP8BS_ERR_BAD_SHAPE;
    if (num_cus <= 0) num_cus = fp8bs::device_cus();     // the current device's, 256 where there is none
    choose(m, n, k, num_cus, out);
    return FP8BS_OK;
}

size_t fp8bs_workspace_bytes(int m, int n, int k) {
    fp8bs_plan_t p{};
    if (fp8bs_plan(m, n, k, fp8bs::device_cus(), &p) != FP8BS_OK) return 0;
    return (size_t)p.workspace_bytes;
}

int fp8bs_gemm_ex(const void* a, const void* b, const float* a_scale, const float* b_scale,
                  void* c, void* ws, size_t ws_bytes, int m, int n, int k,
                  int variant, int split_k, void* stream) {
    int st = check_common(a, b, a_scale, b_scale, c, m, n, k);
    if (st != FP8BS_OK) return st;
    if (m == 0 || n == 0) return FP8BS_OK;
    hipStream_t s = (hipStream_t)stream;
    fp8bs_plan_t plan{};
    if (k == 0) variant = FP8BS_VARIANT_GENERIC;   // empty sum: the generic kernel writes zeros
    // Operands off the 16-byte grid and n off the 8-column grid: the tiled kernels take them in every mode
    // (the same instantiation as for rows of a, b and c that start anywhere); only the streaming kernels are
    // left out.  A workspace that starts off the 16-byte grid is used from its first 16-byte boundary on.
    const bool aligned = vector_aligned(a, b, c);
    if (ws && ((uintptr_t)ws & 15) != 0) {
        const size_t skip = 16 - ((uintptr_t)ws & 15);
        if (ws_bytes > skip) { ws = (char*)ws + skip; ws_bytes -= skip; }
        else { ws = nullptr; ws_bytes = 0; }
    }
    const bool simple = aligned && vector_shape(n);      // streaming kernels possible
    const int cus = fp8bs::device_cus();
    if (variant == FP8BS_VARIANT_AUTO) {
        choose(m, n, k, cus, &plan);
        if (split_k > 0) fill_plan(m, n, k, plan.variant, split_k & ~FP8BS_SPLIT_SUM_IN_KERNEL, &plan, 0, (split_k & FP8BS_SPLIT_SUM_IN_KERNEL) != 0);
        else if (split_k < 0) fill_plan(m, n, k, plan.variant, 1, &plan, streamk_grid(plan.variant, m, n, k, cus));
        // the plan needs a workspace the caller did not bring: the best plan that needs none
        else if (plan.workspace_bytes > 0 && (!ws || ws_bytes < plan.workspace_bytes)) {
            // too small for the partial tiles of a sum in the kernel but not for the planes (tiles that overhang
            // the matrix): the same split with the reduce kernel
            if (plan.sum_in_kernel && ws && ws_bytes >= planes_bytes(m, n, plan.split_k)) fill_plan(m, n, k, plan.variant, plan.split_k, &plan);
            else choose(m, n, k, cus, &plan, false);
        }
    } else {
        VariantInfo vi{};
        if (!variant_info(variant, &vi)) return FP8BS_ERR_BAD_VARIANT;
        if (is_streaming_variant(variant) && !simple) return FP8BS_ERR_BAD_VARIANT;
        if (is_streaming_variant(variant) && variant != FP8BS_VARIANT_SKINNY64x144 && (m % 4) != 0) return FP8BS_ERR_BAD_VARIANT;   // only the planner's width repairs a
        if (split_k < 0) {
            if (is_streaming_variant(variant) || variant == FP8BS_VARIANT_GENERIC) return FP8BS_ERR_BAD_VARIANT;   // K blocks are dealt by the tiled kernel only
            fill_plan(m, n, k, variant, 1, &plan, streamk_grid(variant, m, n, k, cus));
        } else {
            const bool in_kernel = split_k > 0 && (split_k & FP8BS_SPLIT_SUM_IN_KERNEL) != 0;
            if (in_kernel && (is_streaming_variant(variant) || variant == FP8BS_VARIANT_GENERIC)) return FP8BS_ERR_BAD_VARIANT;   // the tiled kernel only
            fill_plan(m, n, k, variant, split_k > 0 ? (split_k & ~FP8BS_SPLIT_SUM_IN_KERNEL) : 1, &plan, 0, in_kernel);
        }
    }
    if (plan.workspace_bytes > 0 && (!ws || ws_bytes < plan.workspace_bytes)) return FP8BS_ERR_WORKSPACE;

    fp8bs::GemmArgs g{};
    g.a = (const uint8_t*)a; g.b = (const uint8_t*)b; g.as = a_scale; g.bs = b_scale;
    g.c = (uint16_t*)c; g.ws = (float*)ws; g.row_offsets = nullptr;
    g.m = m; g.n = n; g.k = k; g.lda = m; g.nb = (n + 127) / 128;
    g.split_k = plan.split_k;
    g.kb_per_split = (int)cdiv(k / KBLK, plan.split_k);
    g.band_h = 4;
    g.num_experts = 0;
    int mode = plan.split_k > 1 ? 1 : 0;
    if (plan.sum_in_kernel && plan.split_k > 1) {
        mode = 4;
        g.sk_nonce = next_nonce();
    } else if (plan.stream_k > 0) {
        mode = 3;
        g.sk_grid = plan.stream_k;
        g.sk_nonce = next_nonce();
        g.sk_spin = streamk_spin_limit();
    }
    if (fp8bs::launch_gemm(plan.variant, mode, g, s) != hipSuccess) return FP8BS_ERR_LAUNCH;
    if (mode == 1) {
        if (fp8bs::launch_splitk_reduce(g.ws, g.c, (size_t)m * n, plan.split_k, s) != hipSuccess) return FP8BS_ERR_LAUNCH;
    }
    return FP8BS_OK;
}

int fp8bs_gemm(const void* a, const void* b, const float* a_scale, const float* b_scale,
               void* c, void* ws, size_t ws_bytes, int m, int n, int k, void* stream) {
    return fp8bs_gemm_ex(a, b, a_scale, b_scale, c, ws, ws_bytes, m, n, k, FP8BS_VARIANT_AUTO, 0, stream);
}

int fp8bs_gemm_noalloc(const void* a, const void* b, const float* a_scale, const float* b_scale,
                       void* c, int m, int n, int k, void* stream) {
    int st = check_common(a, b, a_scale, b_scale, c, m, n, k);
    if (st != FP8BS_OK) return st;
    if (m == 0 || n == 0) return FP8BS_OK;
    // the plan fp8bs_gemm would follow; its partial planes must fit the built-in array
    fp8bs_plan_t plan{};
    if (k > 0) {
        choose(m, n, k, fp8bs::device_cus(), &plan);
        uint64_t need = plan.workspace_bytes;
        if (plan.sum_in_kernel && planes_bytes(m, n, plan.split_k) < need) need = planes_bytes(m, n, plan.split_k);   // fp8bs_gemm_ex falls back to the planes
        if (need > (uint64_t)FP8BS_NOALLOC_SCRATCH_BYTES) return FP8BS_ERR_SCRATCH_LIMIT;
    }
    void* ws = nullptr;
    st = scratch_address(&ws, (hipStream_t)stream);
    if (st != FP8BS_OK) return st;
    // Every partial element that the sum reads is written by this call first, and a tile's counter in the head
    // of the array counts only arrivals that carry this call's tag, so nothing in the array has to start at zero.
    return fp8bs_gemm_ex(a, b, a_scale, b_scale, c, ws, (size_t)FP8BS_NOALLOC_SCRATCH_BYTES, m, n, k, FP8BS_VARIANT_AUTO, 0, stream);
}

int fp8bs_gemm_grouped_ex(const void* a, const void* b, const float* a_scale, const float* b_scale,
                          void* c, const int32_t* row_offsets, int num_experts, int total_rows,
                          int n, int k, int variant, void* stream) {
    if (num_experts <= 0) return FP8BS_ERR_BAD_OFFSETS;
    if (!row_offsets) return FP8BS_ERR_NULL_POINTER;
    int st = check_common(a, b, a_scale, b_scale, c, total_rows, n, k);
    if (st != FP8BS_OK) return st;
    if (total_rows == 0 || n == 0) return FP8BS_OK;
    hipStream_t s = (hipStream_t)stream;
    fp8bs::GemmArgs g{};
    g.a = (const uint8_t*)a; g.b = (const uint8_t*)b; g.as = a_scale; g.bs = b_scale;
    g.c = (uint16_t*)c; g.ws = nullptr; g.row_offsets = row_offsets;
    g.m = total_rows; g.n = n; g.k = k; g.lda = total_rows; g.nb = (n + 127) / 128;
    g.split_k = 1; g.kb_per_split = k / KBLK; g.band_h = 4; g.num_experts = num_experts;
    g.by_expert = group_order(total_rows, num_experts);
    if (variant == FP8BS_VARIANT_AUTO) {
        // The 256x256 tile for every routing with more than 32 rows per expert on average: measured with 32
        // experts of 8 .. 1024 rows each (even and random counts, n x k = 4096 x 7168 and 7168 x 2048) it is the
        // fastest of the two-stage tiles throughout - the waves without rows only copy, and the widest tile moves
        // the fewest bytes of a per byte of b.  With 32 rows or fewer per expert the call streams every expert's
        // weights once and little else: the 64 x 256 tile with three stages keeps two K blocks of b in flight per
        // workgroup (32 experts x 4096 x 7168: 1 / 8 / 32 rows each 165 / 167 / 173 us against 181 / 185 / 186;
        // from 100 rows on an expert needs a second row of its tiles and the 256x256 tile wins).  Any n and any
        // operand alignment (the instantiation that repairs every expert's last bytes of b).
        variant = k == 0 ? FP8BS_VARIANT_GENERIC : ((long)total_rows <= 32L * num_experts ? FP8BS_VARIANT_T64x256S3 : FP8BS_VARIANT_T256x256);
    } else {
        VariantInfo vi{};
        if (!variant_info(variant, &vi) || is_streaming_variant(variant)) return FP8BS_ERR_BAD_VARIANT;   // no grouped mode in the streaming kernels
        if (variant != FP8BS_VARIANT_GENERIC && k == 0) return FP8BS_ERR_BAD_VARIANT;
    }
    if (fp8bs::launch_gemm(variant, 2, g, s) != hipSuccess) return FP8BS_ERR_LAUNCH;
    return FP8BS_OK;
}

int fp8bs_gemm_grouped(const void* a, const void* b, const float* a_scale, const float* b_scale,
                       void* c, const int32_t* row_offsets, int num_experts, int total_rows,
                       int n, int k, void* stream) {
    return fp8bs_gemm_grouped_ex(a, b, a_scale, b_scale, c, row_offsets, num_experts, total_rows, n, k, FP8BS_VARIANT_AUTO, stream);
}

int fp8bs_gemm_silu_mul(const void* a, const void* b, const float* a_scale, const float* b_scale, void* h,
                        const int32_t* row_offsets, int num_experts, int rows, int n, int k, void* stream) {
    if (row_offsets && num_experts <= 0) return FP8BS_ERR_BAD_OFFSETS;
    if ((n & 1) != 0) return FP8BS_ERR_BAD_SHAPE;
    int st = check_common(a, b, a_scale, b_scale, h, rows, n, k);
    if (st != FP8BS_OK) return st;
    if (rows == 0 || n == 0) return FP8BS_OK;
    fp8bs::GemmArgs g{};
    g.a = (const uint8_t*)a; g.b = (const uint8_t*)b; g.as = a_scale; g.bs = b_scale;
    g.c = (uint16_t*)h; g.ws = nullptr; g.row_offsets = row_offsets;
    g.m = rows; g.n = n; g.k = k; g.lda = rows; g.nb = (n + 127) / 128;
    g.split_k = 1; g.kb_per_split = k / KBLK; g.band_h = 4; g.num_experts = row_offsets ? num_experts : 0;
    g.epi = 1;
    g.by_expert = row_offsets ? group_order(rows, num_experts) : 0;
    // any even n and any operand alignment: rows of h that do not keep 16-byte stores aligned are stored in pieces
    int variant = k == 0 ? FP8BS_VARIANT_GENERIC : FP8BS_VARIANT_T256x256;
    if (fp8bs::launch_gemm(variant, row_offsets ? 2 : 0, g, (hipStream_t)stream) != hipSuccess) return FP8BS_ERR_LAUNCH;
    return FP8BS_OK;
}

}  // extern "C"
