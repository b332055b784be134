/*
 * fp8bs.h - C ABI of libfp8bs.so: FP8 (OCP e4m3fn) block-scaled GEMM for gfx950 (MI355X).
 *
 *   C[m][n] (bf16) = sum_kb ( sum_{kk in block kb} A[m][kk] * B[n][kk] ) * a_scale[m][kb] * b_scale[n/128][kb]
 *
 * This header is the drop-in boundary for the host launcher of the reference
 * (1-amd-fp8-mm/amd-fp8-mm-submission.py:8 and :514-579, `void fp8_mm(torch::Tensor a, b, as, bs,
 * c, c_tmp)`), re-cut as plain pointers and sizes so that any host language can bind it.
 *
 * Physical layouts (the reference's, 1-amd-fp8-mm/amd-fp8-mm-submission.py:66-75, 307-316, 364):
 *   a        : K rows of M bytes       a[kk * M + i]                 e4m3fn
 *   b        : K rows of N bytes       b[kk * N + j]                 e4m3fn
 *   a_scale  : K/128 rows of M floats  a_scale[(kk/128) * M + i]
 *   b_scale  : K/128 rows of NB floats b_scale[(kk/128) * NB + j/128],  NB = ceil(N/128)
 *   c        : M rows of N bf16        c[i * N + j]
 * All pointers are device pointers. The library never allocates or frees device memory and writes
 * nothing but `c` and the caller's workspace `ws`. Calls are asynchronous on `stream`
 * (a hipStream_t passed as void*; NULL = the null stream). K must be a multiple of 128.
 */
#ifndef FP8BS_H
#define FP8BS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes (0 = success). The reference launcher returns void and never reads launch errors
 * (1-amd-fp8-mm/amd-fp8-mm-submission.py:514-579); this boundary reports them. */
enum {
    FP8BS_OK = 0,
    FP8BS_ERR_NULL_POINTER = 1,   /* a required pointer is NULL                             */
    FP8BS_ERR_BAD_SHAPE = 2,      /* m,n,k <= 0 where not allowed, k % 128 != 0, or a pointer
                                     not aligned to its element type                          */
    FP8BS_ERR_WORKSPACE = 3,      /* ws is NULL / smaller than fp8bs_workspace_bytes(...)    */
    FP8BS_ERR_TOO_LARGE = 4,      /* an operand exceeds the 4 GiB buffer-addressing limit    */
    FP8BS_ERR_LAUNCH = 5,         /* hipGetLastError() after launch was not hipSuccess       */
    FP8BS_ERR_BAD_OFFSETS = 6,    /* grouped: bad expert count                               */
    FP8BS_ERR_BAD_VARIANT = 7,    /* forced variant id unknown or not applicable             */
    FP8BS_ERR_SCRATCH_LIMIT = 8,  /* fp8bs_gemm_noalloc: the shape's K split needs more than
                                     FP8BS_NOALLOC_SCRATCH_BYTES of partial planes            */
    FP8BS_ERR_TIMEOUT = 9,        /* never returned by a call (calls do not wait for the GPU): the value a
                                     kernel leaves in the first word of the workspace when a workgroup's
                                     bounded wait for another workgroup's partial tile gave up     */
    FP8BS_ERR_CAPTURE = 10        /* fp8bs_gemm_noalloc: first call on this device made under stream capture */
};

/* Kernel variants the planner chooses from. */
enum {
    FP8BS_VARIANT_AUTO = 0,
    FP8BS_VARIANT_GENERIC = 1,    /* scalar kernel, any m/n: the planner uses it for k = 0 only */
    FP8BS_VARIANT_T256x256 = 2,   /* compute-bound: 256x256 tile, 8 waves                    */
    FP8BS_VARIANT_T128x128 = 3,   /* mid-size: 128x128 tile, 4 waves                         */
    FP8BS_VARIANT_T64x128 = 4,    /* skinny-M: 64(m) x 128(n) tile, 4 waves, split-K         */
    FP8BS_VARIANT_T256x128 = 5,   /* 256(m) x 128(n) tile, 8 waves                           */
    FP8BS_VARIANT_SKINNY64x144 = 6, /* streaming kernel: 64(m) x 144(n) tile, 4-stage copy ring (forced only: needs m <= 64
                                       per tile row to pay, n % 8 == 0 and operands on 16-byte boundaries) */
    FP8BS_VARIANT_SKINNY64x256 = 7, /* same, 256-wide tile (whole 128-byte lines), 3 stages      */
    FP8BS_VARIANT_SKINNY64x288 = 8, /* same, 288-wide tile, 3 stages                             */
    FP8BS_VARIANT_T256x192 = 9,   /* 256(m) x 192(n) tile, 8 waves: fills more CUs when n/256 rounds up badly */
    FP8BS_VARIANT_T256x128S3 = 10, /* 256 x 128 tile, three LDS stages (a copy has two K blocks' time to land) */
    FP8BS_VARIANT_T192x192S3 = 11, /* 192 x 192 tile, 8 waves of 48 x 96, three LDS stages     */
    FP8BS_VARIANT_T64x256S3 = 12,  /* 64(m) x 256(n) tile, 8 waves of 32 x 64, three LDS stages: few rows against much of b */
    FP8BS_VARIANT_COUNT = 13
};

/* What fp8bs_plan() decides for a shape. Replaces the exact-(m,n,k) if-ladder of the reference
 * (1-amd-fp8-mm/amd-fp8-mm-submission.py:528-578) with a shape-family rule. */
typedef struct fp8bs_plan_t {
    int32_t variant;        /* FP8BS_VARIANT_*                                   */
    int32_t tile_m, tile_n; /* workgroup tile                                    */
    int32_t split_k;        /* number of K partitions (1 = no workspace needed)  */
    int32_t grid_x, grid_y, grid_z;
    int32_t block_threads;
    int32_t lds_bytes;
    int32_t stream_k;       /* > 0: K blocks, not tiles, are dealt to this many workgroups (one launch;
                               partial tiles meet in the workspace); split_k is 1 then           */
    int32_t sum_in_kernel;  /* 1 (with split_k > 1): one launch - the workgroups of a tile's K partitions leave fp32
                               partial tiles in the workspace and the last one to finish adds them in ascending K and
                               writes c; 0: partial planes and a reduce kernel (two launches)      */
    int32_t reserved;
    uint64_t workspace_bytes;
} fp8bs_plan_t;

/* Or'ed into a positive split_k of fp8bs_gemm_ex: sum the K partitions in the kernel (see sum_in_kernel). */
#define FP8BS_SPLIT_SUM_IN_KERNEL (1 << 30)

/* Library version (major*10000 + minor*100 + patch). */
int fp8bs_version(void);

/* Human-readable text of a status code. Never NULL. */
const char* fp8bs_strerror(int status);

/* Host-only planning: no GPU needed. Replaces the dispatch of
 * 1-amd-fp8-mm/amd-fp8-mm-submission.py:528-578. `num_cus` <= 0 means the CU count of the current device, as fp8bs_gemm, fp8bs_gemm_noalloc and
 * fp8bs_workspace_bytes use it (256, MI355X's, where no device can be asked).  The plan is the one
 * fp8bs_gemm follows with a workspace of workspace_bytes; without the workspace of a planned K split
 * fp8bs_gemm runs the best plan that needs none (slower, same result up to the summation order). */
int fp8bs_plan(int m, int n, int k, int num_cus, fp8bs_plan_t* out);

/* Bytes of device workspace fp8bs_gemm needs for this shape (0 when split_k == 1; the partial planes, or the
 * counters and partial tiles of a split summed in the kernel). Replaces the
 * per-call `torch.empty(m*n*4)` of 1-amd-fp8-mm/amd-fp8-mm-submission.py:600: the caller owns and
 * reuses the workspace. */
size_t fp8bs_workspace_bytes(int m, int n, int k);

/* Dense GEMM. Replaces `fp8_mm(a,b,as,bs,c,c_tmp)`,
 * 1-amd-fp8-mm/amd-fp8-mm-submission.py:514-579. Inputs are never modified (the reference's
 * pre-transpose branch, :570-571, overwrites a and b; this one does not).
 * Any m and n, a and b on any byte, c on any bf16 element: the tiled kernels read a and b with their
 * true row lengths, repair their last one to three bytes in LDS and, with n not a multiple of 8 or c off
 * the 16-byte grid, store c (and the partial planes of a K split) without assuming any alignment of its
 * rows; a workspace off the 16-byte grid is used from its first 16-byte boundary on.  a_scale and b_scale
 * must be 4-byte aligned, c 2-byte aligned (FP8BS_ERR_BAD_SHAPE otherwise). */
int fp8bs_gemm(const void* a, const void* b, const float* a_scale, const float* b_scale,
               void* c, void* ws, size_t ws_bytes, int m, int n, int k, void* stream);

/* Same as fp8bs_gemm with the variant and split-K forced (testing and benchmarking the shape
 * families against each other). variant = FP8BS_VARIANT_AUTO and split_k = 0 reproduce fp8bs_gemm.
 * Workspace requirement for a forced split_k > 1: split_k * m * n * 4 bytes.
 * split_k | FP8BS_SPLIT_SUM_IN_KERNEL: the same K partitions in ONE launch - the role of the reference's split
 * kernel plus merge kernel (1-amd-fp8-mm/amd-fp8-mm-submission.py:371-511) without the second launch, and what
 * fp8bs_plan chooses for splits in two or three (sum_in_kernel of the plan).  Every workgroup writes its fp32
 * partial tile to the workspace and then counts itself in at the tile's counter there; the one that finds all
 * the others counted in adds the partial tiles in ascending K, its own from its registers - the order of the
 * reduce kernel, so c holds the same bits as with two launches - and writes c.  Nobody waits for anybody.  The
 * tiled variants only (else FP8BS_ERR_BAD_VARIANT); with more than 2016 tiles or more than 255 partitions the
 * call takes the two-launch form.  Workspace: 16384 + tiles * split_k * tile_m * tile_n * 4 bytes
 * (FP8BS_ERR_WORKSPACE if smaller), contents unspecified on entry (a counter carries the call's own tag, so
 * whatever an earlier use left there counts as zero), one call at a time per workspace.
 * split_k < 0: another one-launch form, K BLOCKS instead of tiles dealt to
 * the workgroups (one per place on the chip, G = min(places, tiles * K/128); the tiled variants only, else
 * FP8BS_ERR_BAD_VARIANT); a workgroup whose run of K blocks ends inside a tile leaves an fp32 partial tile in the
 * workspace and raises a flag there, the workgroup that holds the tile's last K block waits for the flags (a
 * bounded number of polls), adds the partial tiles in ascending K to its own accumulators - a fixed order, so the
 * result is the same from run to run - and writes c.  Workspace: 16384 + G * tile_m * tile_n * 4 bytes
 * (FP8BS_ERR_WORKSPACE if smaller; at most 64 MiB + 16 KiB on 256 CUs), contents unspecified on entry, one
 * call at a time per workspace.  Its first word is a status: a wait that gives up stores FP8BS_ERR_TIMEOUT there
 * and the kernel still runs to its end (c is then not valid); nothing else ever writes that word, so a caller
 * that means to read it zeroes it once after allocating.  The environment variable FP8BS_STREAMK_SPIN, read once,
 * sets the polls per flag (default 262144, about a quarter of a second; negative: every wait gives up at once).
 * Measured on MI355X this form is not faster than the planned K split, so fp8bs_plan never chooses it
 * (stream_k of a plan is 0). */
int fp8bs_gemm_ex(const void* a, const void* b, const float* a_scale, const float* b_scale,
                  void* c, void* ws, size_t ws_bytes, int m, int n, int k,
                  int variant, int split_k, void* stream);

/* fp8bs_gemm for callers that cannot allocate device memory or hand over a workspace: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference
 * (its split-K path allocates a tensor per call, 1-amd-fp8-mm/amd-fp8-mm-submission.py:600).  Same
 * arguments, plan, kernels and results as fp8bs_gemm, but the fp32 partial planes or tiles of a K split live in an
 * array of FP8BS_NOALLOC_SCRATCH_BYTES that is part of the library's device code (every GPU the library
 * runs on holds it until the process ends).  Calls no hipMalloc / hipFree or any allocating routine.
 * A shape whose planned K split needs more workspace than that returns FP8BS_ERR_SCRATCH_LIMIT
 * and launches nothing.  All calls on one GPU share the one array: calls that overlap on a GPU (two
 * streams, two threads) race on it; calls on one stream are ordered and safe.  Nothing in the array has to
 * be cleared between calls (every partial element read was written by the same call).
 * Under HIP graph capture: make one eager call per device and shape first.  The first call on a device looks the
 * array's address up (hipGetSymbolAddress) and the first launch of every kernel instantiation raises that kernel's
 * dynamic-LDS limit (hipFuncSetAttribute); neither is a stream operation that a capture could record.  A first
 * call that finds its stream capturing returns FP8BS_ERR_CAPTURE and launches nothing. */
#define FP8BS_NOALLOC_SCRATCH_BYTES (32u * 1024u * 1024u)
int fp8bs_gemm_noalloc(const void* a, const void* b, const float* a_scale, const float* b_scale,
                       void* c, int m, int n, int k, void* stream);

/* Grouped (MoE expert) GEMM. Row-offset convention of 2-amd-moe/3-amd-fp8-moe-hip-myhgemm.py:142-148
 * and :328-336 (expert_offset = exclusive prefix sum of per-expert row counts), with the total
 * appended: row_offsets has num_experts+1 int32 entries on the device, row_offsets[0] = 0,
 * row_offsets[num_experts] = total_rows. Expert e owns rows [row_offsets[e], row_offsets[e+1]).
 *   a        : K rows of total_rows bytes (permuted, expert-contiguous rows), a_scale likewise
 *   b        : num_experts matrices, each K rows of N bytes;  b_scale: num_experts x (K/128) x NB
 *   c        : total_rows rows of N bf16
 * No host synchronisation (the reference needs one to size its grid, :595, :607-610). */
int fp8bs_gemm_grouped(const void* a, const void* b, const float* a_scale, const float* b_scale,
                       void* c, const int32_t* row_offsets, int num_experts, int total_rows,
                       int n, int k, void* stream);

/* Same with the tile forced: one of the FP8BS_VARIANT_T* tiles or FP8BS_VARIANT_GENERIC (the streaming
 * variants have no grouped mode: FP8BS_ERR_BAD_VARIANT).  FP8BS_VARIANT_AUTO reproduces
 * fp8bs_gemm_grouped (the 256x256 tile, or the 64x256 three-stage tile when total_rows <= 32 * num_experts, for any n
 * and any operand alignment; the scalar kernel only for k = 0). */
int fp8bs_gemm_grouped_ex(const void* a, const void* b, const float* a_scale, const float* b_scale,
                          void* c, const int32_t* row_offsets, int num_experts, int total_rows,
                          int n, int k, int variant, void* stream);

/* ---- Quantisers (the step in front of the GEMM) -------------------------------------------------
 * The reference has no counterpart: its operands arrive already quantised from the harness
 * (1-amd-fp8-mm/0-amd-fp8-mm-new-begins.py:66-77).  These produce exactly those operands, in the
 * storage layouts above, from a row-major fp32 or bf16 matrix.  Rule per block, bit for bit:
 *   scale = max(max|x| / 448, 1e-12) (fp32),  q = e4m3fn(round to nearest even) of clamp(x / scale, +-448).
 * `ldx` is the distance between input rows in elements (>= k; rows must start 16-byte aligned for
 * fp32, 8-byte for bf16). */
enum { FP8BS_DTYPE_F32 = 0, FP8BS_DTYPE_BF16 = 1 };

/* Activations: x [m or src_rows][k] -> a (K rows of m bytes) and a_scale (K/128 rows of m floats), one
 * scale per row and 128-wide K block.  If row_map is not NULL (device pointer, m int32 entries), output
 * row i is quantised from input row row_map[i] (0 <= row_map[i] < src_rows; out-of-range entries give
 * zero rows): the expert-contiguous gather of MoE tokens
 * (2-amd-moe/3-amd-fp8-moe-hip-myhgemm.py:174-191) fused into the quantiser. */
int fp8bs_quantize_a(const void* x, int x_dtype, int64_t ldx, const int32_t* row_map, int src_rows,
                     void* a, float* a_scale, int m, int k, void* stream);

/* Row gather of quantised activations: a[kk][i] = a_src[kk][row_map[i]] and a_scale[kb][i] =
 * a_scale_src[kb][row_map[i]] for i < m (a_src: K rows of src_rows bytes, a_scale_src: K/128 rows of
 * src_rows floats; entries of row_map outside [0, src_rows) give zero bytes and the scale 1e-12, what
 * fp8bs_quantize_a writes for a zero row).  Quantising the tokens once and gathering gives the same
 * bytes as fp8bs_quantize_a with the same row_map at an eighth of the arithmetic when every token is
 * routed to 8 experts; the reference copies rows into expert order the same way
 * (2-amd-moe/3-amd-fp8-moe-hip-myhgemm.py:174-191).  Fast path: src_rows and m multiples of 4,
 * src_rows <= 40960, row_map and a_scale 16-byte aligned; anything else takes a byte-wise kernel. */
int fp8bs_gather_a(const void* a_src, const float* a_scale_src, int src_rows, const int32_t* row_map,
                   void* a, float* a_scale, int m, int k, void* stream);

/* Weights: w [n][k] -> b (K rows of n bytes) and b_scale (K/128 rows of ceil(n/128) floats), one scale
 * per 128x128 block; a partial last block of rows takes its maximum over the rows that exist. */
int fp8bs_quantize_b(const void* w, int w_dtype, int64_t ldw, void* b, float* b_scale, int n, int k,
                     void* stream);

/* e4m3fnuz bytes (the gfx942 type of the reference, 1-amd-fp8-mm/amd-fp8-mm-submission.py:20-21: bias 8,
 * max 240, NaN 0x80) -> e4m3fn bytes of the same value, so that operands quantised for the reference's
 * hardware can be fed to this library unchanged in scale.  Exact except for the 16 smallest magnitudes
 * (below 2^-6), which land on e4m3fn's coarser subnormal grid with round-to-nearest-even.  src and dst
 * must be 16-byte aligned and may be the same buffer. */
int fp8bs_convert_fnuz_to_fn(const void* src, void* dst, size_t nbytes, void* stream);

/* ---- MoE routing (the caller of the grouped GEMM) ------------------------------------------------
 * Top-k selection with the reference's rule (2-amd-moe/amd-moe-submission.py:32-56, 58-105): per token,
 * k times the strictly greatest score not yet taken, lowest index first among equals, best first; NaN
 * and -inf are never selected (index -1, as in the reference).  scores: [tokens][experts] fp32
 * row-major; top_idx: [tokens][topk] int32. */
int fp8bs_moe_topk(const float* scores, int tokens, int experts, int topk, int32_t* top_idx, void* stream);

/* Bytes of device workspace fp8bs_moe_route needs. */
size_t fp8bs_moe_route_workspace_bytes(int tokens, int experts);

/* From top_idx [tokens][topk] (entries outside [0, experts) are ignored) build, on the device and with
 * no host synchronisation (the reference synchronises and reads the counts on the host, :230-234):
 *   row_offsets [experts+1]   exclusive prefix of the rows per expert, total appended
 *                              (2-amd-moe/3-amd-fp8-moe-hip-myhgemm.py:142-148) - what fp8bs_gemm_grouped takes
 *   row_map     [tokens*topk] row_map[row] = token that fills that row; rows of an expert are ordered by
 *                              token id (the reference hands positions out by atomicAdd, :107-156, so its
 *                              order varies between runs) - what fp8bs_quantize_a takes as its gather list;
 *                              entries beyond row_offsets[experts] are set to -1
 *   slot_of     [tokens][topk] row of every (token, choice), -1 for ignored entries; may be NULL
 * experts <= 1024, topk <= 16. */
int fp8bs_moe_route(const int32_t* top_idx, int tokens, int experts, int topk, int32_t* row_offsets,
                    int32_t* row_map, int32_t* slot_of, void* ws, size_t ws_bytes, void* stream);

/* ---- Expert FFN pieces behind the grouped GEMM ---------------------------------------------------
 * Gate/up projection with the activation fused into the GEMM's epilogue.  b holds the gate and up
 * weights interleaved by row: row 2i = gate_i, row 2i+1 = up_i (n = 2 x intermediate size, even);
 * h[row][i] = bf16( silu(C[row][2i]) * C[row][2i+1] ) with C the fp32 block-scaled product, h has n/2
 * columns.  Role of re_silu_mul_kernel (2-amd-moe/amd-moe-submission.py:366-407; fp16 there, rounding
 * silu to fp16 before the product) fused as in 2-amd-moe/5-amd-fp8-moe-hip-fuse.py:366-408.
 * row_offsets NULL: dense (one weight matrix); else grouped as fp8bs_gemm_grouped. */
int fp8bs_gemm_silu_mul(const void* a, const void* b, const float* a_scale, const float* b_scale, void* h,
                        const int32_t* row_offsets, int num_experts, int rows, int n, int k, void* stream);

/* Weighted un-permute: out[t][:] = sum_j weights[t][j] * y[slot_of[t][j]][:]  (y bf16 [rows][d], out bf16
 * [tokens][d], d % 8 == 0, y and out 16-byte aligned; fp32 accumulation in the order j = 0..topk-1, one rounding; a slot outside
 * [0, rows) is skipped).  Role of pack_output (2-amd-moe/amd-moe-submission.py:239-301; fp16
 * accumulation there). */
int fp8bs_moe_combine(const void* y, int rows, const int32_t* slot_of, const float* weights, void* out,
                      int tokens, int topk, int d, void* stream);

/* ---- Measurement aid -------------------------------------------------------------------------------
 * No counterpart in the reference and no part of any GEMM call: runs, `iters` times per wave, the
 * instruction mix of one K block of the 256x256 tile's wave (32 FP8 MFMAs on random operands, 8 waves per
 * workgroup) with the parts selected by the bits of `mix` (0 .. 23): 1 = the scale fold (4 v_fma per MFMA),
 * 2 = the transposing LDS reads (48 per 32 MFMAs), 4 = the global->LDS copies (8 KiB per wave per 32 MFMAs;
 * the 8 workgroups an XCD runs side by side share a stream, the streams walk src cyclically), 8 = the same
 * multiply-accumulates as 16 MFMAs of the 32x32x64 form, 16 (with bit 2 only) = the LDS reads spread evenly
 * over the K block into a second set of A registers instead of the GEMM's bursts - without barriers, waits or
 * output; `iters` must be even (the loop body is two K blocks, one per LDS stage, all LDS addresses immediate).  One iteration is 2048 clocks of matrix-core work per SIMD, so
 * iters * 2048 / 2.4e9 / time is the fraction of the nominal FP8 peak the mix reaches on `workgroups` CUs.
 * src: device buffer of src_bytes (a power of two >= 4 MiB, 16-byte aligned) whose first 64 KiB hold e4m3fn
 * codes used as operands; sink: 4 writable device bytes (never written in practice).  bench.py
 * --mfma-ceiling drives it. */
int fp8bs_diag_mfma_mix(int mix, int workgroups, int iters, const void* src, size_t src_bytes, void* sink, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FP8BS_H */
