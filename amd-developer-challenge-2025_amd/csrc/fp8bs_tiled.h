// FP8 (OCP e4m3fn) block-scaled GEMM kernels for gfx950 (CDNA4, MI355X).
//
// Computes, per 128-wide K block kb,   P_kb[m][n] = sum_{kk in kb} A[m][kk] * B[n][kk]   on the FP8
// matrix cores (v_mfma_f32_16x16x128_f8f6f4, one instruction = one whole scale block of one 16x16
// tile), then folds   C[m][n] += P_kb[m][n] * (a_scale[m][kb] * b_scale[n/128][kb])   into fp32
// accumulators on the vector ALU, and finally rounds to bf16.  Semantics follow the reference's
// dequantise-then-multiply statement (1-amd-fp8-mm/0-amd-fp8-mm-new-begins.py:17-49, 85-89) and the
// per-block fold of its shipped kernel (1-amd-fp8-mm/amd-fp8-mm-submission.py:333, 350-352).
//
// Memory layouts are the reference's (amd-fp8-mm-submission.py:66-75, 307-316): both operands arrive
// with K as the strided dimension, a[kk*M + i], b[kk*N + j].  The K<->M/N transpose the matrix cores
// need is fused into the LDS read: tiles are copied to LDS untransposed ([k][m] rows, 16-byte chunks,
// asynchronous global->LDS loads that bypass registers) and the operands are fetched with the CDNA4
// transposing read ds_read_b64_tr_b8, which hands every lane 8 consecutive-k bytes of one row.
//
// Layout facts used below were measured on the chip with one-hot operands:
//  * ds_read_b64_tr_b8: inside each group of 16 lanes, source lanes 2r and 2r+1 address the low and
//    high 8 bytes of "k row" r (r = 0..7); result lane i receives, as byte r, column i of row r.
//  * v_mfma_f32_16x16x128_f8f6f4: lane l supplies 32 bytes of row l%16 for k group l/16; operand A
//    and operand B use the same (group, byte) -> k map, so any k order inside the block is valid as
//    long as both operands use the same one.  D[i][j] (i from src0 rows, j from src1 rows) lives in
//    lane 16*(i/4) + j, register i%4.
// The kernel feeds B rows (n) as src0 and A rows (m) as src1, so a lane owns four consecutive n of
// one output row m: one a_scale value per lane per 16x16 tile and 8-byte contiguous bf16 stores.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include <type_traits>
#include <utility>

#include "fp8bs_kernels.h"

namespace fp8bs {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef unsigned short v4us __attribute__((ext_vector_type(4)));

#define LDS_V2I(p) ((__attribute__((address_space(3))) v2i*)(p))
#define LDS_VOID(p) ((__attribute__((address_space(3))) void*)(p))

static constexpr int KBLK = 128;  // scale block along K == K extent of one MFMA
static constexpr int GROUP_TABLE_MAX = 264;   // grouped walk: up to 263 experts have their row ranges kept in LDS (4.1 KiB)

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    v2f f = {lo, hi};
    v2bf h = __builtin_convertvector(f, v2bf);   // v_cvt_pk_bf16_f32: round to nearest even
    return __builtin_bit_cast(uint32_t, h);
}

// 16 bytes per lane, global -> LDS without passing through registers (buffer_load_dwordx4 ... lds):
// lane l's bytes land at lds_base + 16*l; lds_base and wave_offset must be wave-uniform (SGPRs), the
// address is buffer base + lane_offset + wave_offset.
// M0 (the LDS base of such a load) is written inside the statement.  The compiler reserves M0 and warns
// when it sees it among the clobbers; nothing it generates for these kernels reads M0 (LDS instructions
// need no M0 on gfx9, and there are no indirect register moves, GWS or message instructions here).
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void copy16_global_to_lds(__amdgpu_buffer_rsrc_t rsrc, uint32_t lds_base, uint32_t lane_offset, uint32_t wave_offset) {
    asm volatile("s_mov_b32 m0, %2\n\tbuffer_load_dwordx4 %0, %1, %3 offen lds"
                 :: "v"(lane_offset), "s"(rsrc), "s"(lds_base), "s"(wave_offset) : "memory", "m0");
}
// same with 4 bytes per lane: lane l's dword lands at lds_base + 4*l
__device__ __forceinline__ void copy4_global_to_lds(__amdgpu_buffer_rsrc_t rsrc, uint32_t lds_base, uint32_t lane_offset, uint32_t wave_offset) {
    asm volatile("s_mov_b32 m0, %2\n\tbuffer_load_dword %0, %1, %3 offen lds"
                 :: "v"(lane_offset), "s"(rsrc), "s"(lds_base), "s"(wave_offset) : "memory", "m0");
}
#pragma clang diagnostic pop

// ---------------------------------------------------------------------------------------------------
// Tile -> workgroup mapping.  Workgroups are dealt round-robin to the 8 XCDs (each with its own L2),
// so workgroup w lives on XCD w%8.  Give every XCD a contiguous run of "virtual" ids, and lay the
// virtual ids over the tile grid in bands of GH tile rows walked column by column, so the tiles that
// share an L2 form a compact block and re-use each other's A and B panels.
// ---------------------------------------------------------------------------------------------------
__device__ __forceinline__ int xcd_virtual_id(int wg, int total) {
    const int NX = 8;
    int x = wg % NX, idx = wg / NX;
    int q = total / NX, r = total % NX;
    return x * q + (x < r ? x : r) + idx;
}

__device__ __forceinline__ void band_tile(int v, int tiles_m, int tiles_n, int gh, int& tm, int& tn) {
    int per_band = gh * tiles_n;
    int band = v / per_band;
    int rem = v - band * per_band;
    int rows = tiles_m - band * gh;           // rows in this band (last band may be short)
    rows = rows < gh ? rows : gh;
    tn = rem / rows;
    tm = band * gh + (rem - tn * rows);
}

// ---------------------------------------------------------------------------------------------------
// Main kernel.
//   BM x BN : workgroup tile (rows of A x rows of B), WM x WN : wave tile, 64*(BM/WM)*(BN/WN) threads.
//   MODE 0  : dense, bf16 output
//   MODE 1  : dense split-K, fp32 partial planes to the workspace
//   MODE 2  : grouped (row_offsets), bf16 output
//   MODE 3  : dense, K blocks instead of tiles dealt to the workgroups, partial tiles through the workspace, bf16 output
//   MODE 4  : dense split-K, partial tiles to the workspace, summed by the last workgroup to finish a tile, bf16 output
// LDS: 2 stages, each [128 k][BM] bytes of A then [128 k][BN] bytes of B, 16-byte chunks XOR-swizzled
// so that the 16 k rows touched by half a wave in one transposing read fall on 16 different 16-byte
// bank groups, then the k block's a_scale row and b_scale values.
// ---------------------------------------------------------------------------------------------------
template <int BM, int BN, int WM, int WN, int MODE, int NSTAGE_ = 2>
struct TileCfg {
    static constexpr int NSTAGE = NSTAGE_;                           // LDS stages of one K block each
    static constexpr int WAVES_M = BM / WM, WAVES_N = BN / WN;
    static constexpr int NWAVES = WAVES_M * WAVES_N;
    static constexpr int NTHREADS = NWAVES * 64;
    static constexpr int MT = WM / 16, NT = WN / 16;
    static constexpr int CPR_A = BM / 16, CPR_B = BN / 16;          // 16-byte chunks per k row
    static constexpr int A_BYTES = KBLK * BM, B_BYTES = KBLK * BN;
    static constexpr int AS_BYTES = BM * 4;                          // the k block's a_scale row
    static constexpr int AS_AREA = AS_BYTES < 1024 ? 1024 : AS_BYTES;
    static constexpr int BS_AREA = 256;                              // the k block's b_scale values of the tile's n blocks
    static constexpr int STAGE_BYTES = A_BYTES + B_BYTES + AS_AREA + BS_AREA;
    static constexpr int LDS_BYTES = NSTAGE * STAGE_BYTES;
    static_assert(NSTAGE == 2 || NSTAGE == 3, "two or three stages");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS");
    static constexpr int A_LOADS = A_BYTES / 16 / NTHREADS;         // 16-byte loads per thread per block
    static constexpr int B_LOADS = B_BYTES / 16 / NTHREADS;
    static_assert(A_BYTES % (16 * NTHREADS) == 0 && B_BYTES % (16 * NTHREADS) == 0, "tile/threads");
    // A wave's n range lies inside one b_scale block when the tile starts on a block boundary and the
    // wave width divides 128.  Otherwise (BN = 192, WN = 96) it may cross one boundary, at an n tile that
    // depends on the tile and the wave: the K loop is instantiated per boundary position.
    static constexpr bool SPLIT_SCALES = !(BN % 128 == 0 && 128 % WN == 0);
    static_assert(WN <= 128, "a wave's n range crosses at most one b_scale block boundary");
    static_assert(!SPLIT_SCALES || (BN == 192 && WN == 96), "boundary positions are enumerated for the 192-wide tile only");
    static_assert(CPR_A <= 16 && CPR_B <= 16, "swizzle assumes a k row spans at most 256 bytes");
};

template <int N> __device__ __forceinline__ void wait_vmcnt() {
    // s_waitcnt with only vmcnt constrained: vmcnt is split over bits [3:0] and [15:14]
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

// same, and all LDS and scalar-memory results back (lgkmcnt(0))
template <int N> __device__ __forceinline__ void wait_vmcnt_lgkm0() {
    __builtin_amdgcn_s_waitcnt(0x0070 | (N & 15) | ((N >> 4) << 14));
}

template <int CPR>
__device__ __forceinline__ int swz_of_krow(int krow) {
    if constexpr (CPR != 12) {
        // rows per 256-byte bank sweep = 16/CPR; consecutive sweeps get consecutive XOR masks
        constexpr int ROWS_PER_SWEEP = CPR <= 16 ? 16 / CPR : 1;      // (wider rows are never swizzled)
        return (krow / ROWS_PER_SWEEP) % CPR;
    } else {
        // 12 chunks per k row (192 bytes): four consecutive rows start on the four different quarters of
        // a 256-byte bank sweep, the next four repeat them; rotating the chunks of each group of four
        // rows by one more position puts any 16 consecutive rows of one chunk column on 16 different
        // 16-byte bank groups.
        return (krow >> 2) & 3;
    }
}
// position of logical chunk `ch` inside its k row, and back
template <int CPR>
__device__ __forceinline__ int chunk_to_stored(int ch, int swz) {
    if constexpr ((CPR & (CPR - 1)) == 0) return ch ^ swz;
    else { int x = ch + swz; return x >= CPR ? x - CPR : x; }
}
template <int CPR>
__device__ __forceinline__ int stored_to_chunk(int st, int swz) {
    if constexpr ((CPR & (CPR - 1)) == 0) return st ^ swz;
    else { int x = st - swz; return x < 0 ? x + CPR : x; }
}

// Repair of the last bytes of a or b (see the main kernel).  cand[i]: bit 31 = the byte is lost, bits
// 29-30 = its k row inside the last K block minus 125, bits 0-28 = its row (of a) or column (of b); bits
// 8-31 of `last` = the bytes themselves.  tile: the operand's tile of the tile's last K block, x0 its first
// row / column, spare: a byte of LDS nobody reads.  No control flow: a store that does not apply goes to
// the spare byte.  (A branch at this place, in the middle of a K block's step sequence, makes the compiler
// move the folds of the MFMAs before it below it, which costs some thirty registers.)
template <int BX, int CPR>
__device__ __forceinline__ void patch_tail_bytes(unsigned char* tile, unsigned char* spare, bool enable, int x0,
                                                 uint32_t cand0, uint32_t cand1, uint32_t cand2, uint32_t last, int tid) {
    const uint32_t cand[3] = {cand0, cand1, cand2};
#pragma unroll
    for (int c = 0; c < 3; c++) {
        const int xt = (int)(cand[c] & 0x1FFFFFFFu) - x0;                 // row / column inside the tile
        const int kl = KBLK - 3 + (int)((cand[c] >> 29) & 3u);            // k row inside the last block
        int xc = xt < 0 ? 0 : xt;                                         // in range whatever xt is
        xc = xc < BX ? xc : BX - 1;
        unsigned char* dst = tile + kl * BX + (chunk_to_stored<CPR>(xc >> 4, swz_of_krow<CPR>(kl)) << 4) + (xc & 15);
        int apply = (enable && (cand[c] >> 31) != 0 && xt >= 0 && xt < BX && tid == 0) ? 1 : 0;
        asm volatile("" : "+v"(apply));       // opaque to the optimiser: a select follows, never a branch
        *(apply != 0 ? dst : spare) = (unsigned char)(last >> (8 * (c + 1)));
    }
}
// The last four bytes of an operand, which may start on any byte.
__device__ __forceinline__ uint32_t load_last_dword(const uint8_t* q) {
    return (uint32_t)q[0] | ((uint32_t)q[1] << 8) | ((uint32_t)q[2] << 16) | ((uint32_t)q[3] << 24);
}
// The three candidates of an operand whose k rows are ld bytes long and whose buffer ends at `end`.
__device__ __forceinline__ uint32_t tail_candidate(uint32_t o, uint32_t ld, uint32_t end, uint32_t k) {
    const uint32_t krow = o / ld, x = o - krow * ld;
    const bool lost = krow * ld + (x & ~3u) + 4u > end;                   // its dword crosses the end
    return lost ? (0x80000000u | ((krow - (k - 3u)) << 29) | x) : 0u;
}

// EPI 0: plain bf16 output.  EPI 1: gate/up pairs - column 2i is gate_i, column 2i+1 is up_i - are
// combined to silu(gate_i) * up_i in fp32 and the output has n/2 columns (role of the fp16 layer's
// re_silu_mul_kernel, 2-amd-moe/amd-moe-submission.py:366-407, fused into the GEMM as in
// 2-amd-moe/5-amd-fp8-moe-hip-fuse.py:366-408).
__device__ __forceinline__ float silu_mul(float gate, float up) {
    // gate / (1 + exp(-gate)) * up; exp2 and rcp are the hardware approximations (~1 ulp)
    return gate * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504088896341f * gate)) * up;
}

// TAILS: lda is not a multiple of four or n not a multiple of eight; the kernel then repairs the last
// bytes of a and b in LDS (one more barrier per tile) and stores a row's last, partial 16-byte chunk of c
// in pieces, see below.
// Waves per SIMD when as many workgroups as LDS and thread count allow share a CU.  The modes that exchange partial
// tiles must keep their registers within that (their sums would otherwise take registers the K loop does not need
// and halve the number of workgroups per CU); the other modes fit without being told.
template <int BM, int BN, int WM, int WN, int MODE, int NSTAGE>
constexpr int waves_per_simd() {
    using C = TileCfg<BM, BN, WM, WN, MODE, NSTAGE>;
    const int by_lds = 163840 / C::LDS_BYTES, by_threads = 2048 / C::NTHREADS;
    const int w = C::NWAVES * (by_lds < by_threads ? by_lds : by_threads) / 4;
    return MODE >= 3 && w > 1 ? w : 1;
}

template <int BM, int BN, int WM, int WN, int MODE, int EPI = 0, int NSTAGE = 2, bool TAILS = false>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * 64) __attribute__((amdgpu_waves_per_eu(waves_per_simd<BM, BN, WM, WN, MODE, NSTAGE>())))
void gemm_tr_kernel(const GemmArgs p) {
    using C = TileCfg<BM, BN, WM, WN, MODE, NSTAGE>;
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];

    // global store instructions per wave and tile in the bf16 epilogue (always this many: lanes without
    // a valid element are switched off by an out-of-range buffer offset, not by a branch)
    constexpr int EPI_WNO = EPI == 1 ? WN / 2 : WN;
    constexpr int EPI_ROW_CHUNKS = EPI_WNO * 2 / 16;
    constexpr int EPI_ROWS_PER_PASS = (EPI_ROW_CHUNKS & (EPI_ROW_CHUNKS - 1)) == 0 ? 64 / EPI_ROW_CHUNKS : 4;
    constexpr int EPI_PARTS = (WM / 16) % 2 == 0 ? 2 : WM / 16;       // the wave tile is staged in parts of whole m tiles
    constexpr int EPI_STORES = MODE == 1 ? 0 : EPI_PARTS * ((WM / EPI_PARTS) / EPI_ROWS_PER_PASS);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 4, i16 = lane & 15;
    // Waves w and w+4 share a SIMD.  With 4 x 2 waves they get m positions two apart, so that in a tile
    // whose valid rows end at half height (the last tile of an expert, of M) every SIMD keeps one wave
    // with work instead of two SIMDs keeping both.
    const int wave_n = wave / C::WAVES_M;
    const int wave_m = (C::WAVES_M == 4 && C::NWAVES == 8) ? ((wave + 2 * wave_n) & 3) : wave % C::WAVES_M;

    // ---- tiles ---------------------------------------------------------------------------------
    // The workgroup is persistent: it walks the tiles  blockIdx.x, blockIdx.x + gridDim.x, ...  and
    // issues the first K block of the next tile before it converts and stores the current one, so a
    // tile's output and the next tile's first loads overlap (with K = 2048 the per-tile prologue and
    // epilogue are a third of a tile's time otherwise).
    struct Tile {
        int valid, m0, n0, kb_begin, kb_end, split_z, row_lo, row_hi;
        int sk_contrib, sk_first;             // MODE 3: the segment ends before the tile's last K block; first workgroup of the tile's earlier segments (-1: none)
        const uint8_t* bptr;
        const float* bsptr;
    };
    int total_slots = 0;                      // grouped: m-tile slots that exist (from row_offsets)
    // Grouped, fewer than GROUP_TABLE_MAX experts: a table in LDS, one entry per expert - first row of its first
    // tile (row_offsets[e] rounded down to 16), its row range, and the number of slots before it - built once
    // by wave 0.  Finding a tile's expert is then one LDS read per lane and a count of the lanes whose experts
    // start at or before the tile's slot; as a loop over row_offsets in scalar code it took 1.5-2 us per tile,
    // between the last K block of one tile and the first copies of the next.  More experts: that loop.
    [[maybe_unused]] v4i* gtable = nullptr;
    bool use_table = false;
    if constexpr (MODE == 2) {
        __shared__ v4i gtable_store[GROUP_TABLE_MAX];        // entry [num_experts]: the slots before the end = all of them
        gtable = gtable_store;
        use_table = p.num_experts < GROUP_TABLE_MAX;
        if (use_table) {
            if (wave == 0) {
                int carry = 0;
                for (int base = 0; base < p.num_experts; base += 64) {
                    const int x = base + lane;
                    int lo = 0, hi = 0;
                    if (x < p.num_experts) { lo = p.row_offsets[x]; hi = p.row_offsets[x + 1]; }
                    lo = lo < 0 ? 0 : lo; hi = hi > p.m ? p.m : hi;       // a malformed table must not reach beyond the matrix
                    const int s = lo & ~15;
                    const int nt = (hi > lo) ? (hi - s + BM - 1) / BM : 0;
                    int incl = nt;                                        // inclusive prefix sum over the 64 lanes
#pragma unroll
                    for (int d = 1; d < 64; d <<= 1) {
                        const int y = __shfl_up(incl, d, 64);
                        if (lane >= d) incl += y;
                    }
                    if (x < p.num_experts) gtable_store[x] = (v4i){s, lo, hi, carry + incl - nt};
                    carry += __shfl(incl, 63, 64);
                }
                if (lane == 0) gtable_store[p.num_experts] = (v4i){0, 0, 0, carry};
            }
            __syncthreads();
            total_slots = __builtin_amdgcn_readfirstlane(gtable_store[p.num_experts][3]);
        } else {
            for (int x = 0; x < p.num_experts; x++) {
                int lo = p.row_offsets[x], hi = p.row_offsets[x + 1];
                lo = lo < 0 ? 0 : lo; hi = hi > p.m ? p.m : hi;
                total_slots += (hi > lo) ? (hi - (lo & ~15) + BM - 1) / BM : 0;
            }
        }
    }
    [[maybe_unused]] const int sk_self = xcd_virtual_id(blockIdx.x, gridDim.x);
    auto pick_tile = [&](int it) -> Tile {
        Tile t;
        t.valid = 0; t.m0 = 0; t.n0 = 0; t.kb_begin = 0; t.kb_end = 0; t.split_z = 0; t.row_lo = 0; t.row_hi = p.m;
        t.sk_contrib = 0; t.sk_first = -1;
        t.bptr = p.b; t.bsptr = p.bs;
        const int G = gridDim.x;
        if (MODE == 3) {
            // K blocks, not tiles, are dealt to the workgroups: the (tile, K block) pairs of the whole product
            // form one sequence - tiles in the band order of the dense walk, K ascending inside a tile - and
            // workgroup v takes a run of total/G pairs (the first total%G runs hold one more), G <= total.  A run
            // covers the end of one tile, whole tiles, and the beginning of another; the workgroup walks its tiles
            // from the last to the first.  A segment that ends before its tile's last K block is stored as an fp32 partial tile in
            // the workgroup's slot of the workspace (only the first segment a workgroup works on can be one);
            // the segment that holds the tile's last K block belongs to the tile's owner, who adds the
            // partial tiles of the workgroups before it in ascending order of K, then its own accumulators,
            // and writes the output.  The owner works on that segment last and every workgroup it waits for
            // has a lower index, started no later and worked on its partial tile first.
            const int tiles_m = (p.m + BM - 1) / BM, tiles_n = (p.n + BN - 1) / BN;
            const uint32_t kbt = (uint32_t)(p.k / KBLK);
            const uint32_t total = (uint32_t)tiles_m * (uint32_t)tiles_n * kbt;           // < 2^31 (checked by the launcher)
            // runs of q or q+1 pairs, the longer ones first
            const uint32_t q = total / (uint32_t)G, r = total - q * (uint32_t)G;
            auto run_start = [&](uint32_t w) -> uint32_t { return w * q + (w < r ? w : r); };
            const uint32_t v = (uint32_t)sk_self;
            const uint32_t s = run_start(v), e = run_start(v + 1);
            if (e <= s) return t;
            const int t_first = (int)(s / kbt), t_last = (int)((e - 1) / kbt);
            const int tile = t_last - it;
            if (tile < t_first) return t;
            t.valid = 1;
            int tm, tn;
            band_tile(tile, tiles_m, tiles_n, p.band_h, tm, tn);
            const uint32_t x0 = (uint32_t)tile * kbt;                                      // the tile's first pair
            int kb0 = tile == t_first ? (int)(s - x0) : 0;
            int kb1 = tile == t_last ? (int)(e - x0) : (int)kbt;
            int first = -1;
            if (kb1 == (int)kbt && kb0 > 0)                                               // the workgroup whose run holds x0
                first = (int)(x0 < r * (q + 1) ? x0 / (q + 1) : r + (x0 - r * (q + 1)) / q);
            // (uniform values that went through the vector ALU's division sequences: back to scalar registers)
            t.m0 = __builtin_amdgcn_readfirstlane(tm * BM); t.n0 = __builtin_amdgcn_readfirstlane(tn * BN);
            t.kb_begin = __builtin_amdgcn_readfirstlane(kb0);
            t.kb_end = __builtin_amdgcn_readfirstlane(kb1);
            t.sk_contrib = t.kb_end < (int)kbt;
            t.sk_first = __builtin_amdgcn_readfirstlane(first);
        } else if (MODE == 2) {
            // grouped: m-tile slots are laid over the experts in order; expert e's tiles start at
            // row_offsets[e] rounded down to 16 so that global 16-byte loads stay aligned; rows outside
            // [row_offsets[e], row_offsets[e+1]) are computed but never stored.  The gridDim.x tiles in
            // flight together are dealt to the XCDs in contiguous runs.  Two orders of the tiles.  Across
            // the experts: the (slot, n tile) grid of all slots in bands of band_h slots, as in the dense case.
            // Expert by expert (p.by_expert): inside an expert's own grid in bands, an expert of up to eight
            // slots being one band, so that the tiles sharing an L2 form a compact block of few A panels and
            // few B panels of one expert and the tile that holds an expert's last rows runs beside the full
            // tiles that read the same panel of the expert's weights.
            const int tiles_n = (p.n + BN - 1) / BN;
            const int total = total_slots * tiles_n;
            const int v = it * G + xcd_virtual_id(blockIdx.x, G);
            if (v >= total) return t;
            const bool by_expert = p.by_expert != 0;
            int slot_all = 0, tn = 0;
            if (!by_expert) band_tile(v, total_slots, tiles_n, p.band_h, slot_all, tn);
            int e = 0, found = 0, start = 0, cnt_lo = 0, cnt_hi = 0;
            if (use_table) {
                // the expert whose slots hold slot `key`: the last one that starts at or before it (experts
                // without rows start where the next one starts, and are never the last such)
                const int key = by_expert ? v / tiles_n : slot_all;
                int cnt = 0;
                for (int base = 0; base < p.num_experts; base += 64) {
                    const int x = base + lane;
                    const int before = x < p.num_experts ? gtable[x][3] : 0x7FFFFFFF;
                    cnt += __popcll(__ballot(before <= key));
                }
                cnt = __builtin_amdgcn_readfirstlane(cnt);
                if (cnt > 0) {
                    e = cnt - 1;
                    const v4i row = gtable[e];
                    const int s = __builtin_amdgcn_readfirstlane(row[0]), before = __builtin_amdgcn_readfirstlane(row[3]);
                    cnt_lo = __builtin_amdgcn_readfirstlane(row[1]); cnt_hi = __builtin_amdgcn_readfirstlane(row[2]);
                    const int nt = (cnt_hi > cnt_lo) ? (cnt_hi - s + BM - 1) / BM : 0;
                    int slot = slot_all - before;
                    if (by_expert) band_tile(v - before * tiles_n, nt, tiles_n, nt <= 8 ? nt : p.band_h, slot, tn);
                    found = slot < nt;
                    start = s + slot * BM;
                }
            } else {
                int acc_slots = 0;
                for (int x = 0; x < p.num_experts; x++) {
                    int lo = p.row_offsets[x], hi = p.row_offsets[x + 1];
                    lo = lo < 0 ? 0 : lo; hi = hi > p.m ? p.m : hi;
                    int s = lo & ~15;
                    int nt = (hi > lo) ? (hi - s + BM - 1) / BM : 0;
                    if (!found && (by_expert ? v < (acc_slots + nt) * tiles_n : slot_all < acc_slots + nt)) {
                        int slot = slot_all - acc_slots;
                        if (by_expert) band_tile(v - acc_slots * tiles_n, nt, tiles_n, nt <= 8 ? nt : p.band_h, slot, tn);
                        found = 1; e = x; start = s + slot * BM; cnt_lo = lo; cnt_hi = hi;
                    }
                    acc_slots += nt;
                }
            }
            if (!found) return t;                      // uniform for the whole workgroup
            t.valid = 1;
            t.m0 = start; t.n0 = tn * BN;
            t.row_lo = cnt_lo; t.row_hi = cnt_hi;
            t.bptr = p.b + (size_t)e * (size_t)p.k * (size_t)p.n;
            t.bsptr = p.bs + (size_t)e * (size_t)(p.k / KBLK) * (size_t)p.nb;
            t.kb_begin = 0; t.kb_end = p.k / KBLK;
        } else {
            const int tiles_m = (p.m + BM - 1) / BM, tiles_n = (p.n + BN - 1) / BN;
            const int per_split = tiles_m * tiles_n, total = per_split * p.split_k;
            // the gridDim.x tiles in flight together: every XCD takes a contiguous run of them
            const int first = it * G;
            const int here = total - first < G ? total - first : G;
            if (here <= 0) return t;
            const int v = first + xcd_virtual_id(blockIdx.x, G);
            if (v >= total) return t;
            (void)here;
            t.valid = 1;
            t.split_z = v / per_split;
            int tm, tn;
            band_tile(v - t.split_z * per_split, tiles_m, tiles_n, p.band_h, tm, tn);
            if (MODE == 4) t.sk_first = v - t.split_z * per_split;        // the tile's number: its counter and its slots
            t.m0 = tm * BM; t.n0 = tn * BN;
            const int kbt = p.k / KBLK;
            t.kb_begin = t.split_z * p.kb_per_split;
            t.kb_end = t.kb_begin + p.kb_per_split;
            t.kb_end = t.kb_end < kbt ? t.kb_end : kbt;
        }
        return t;
    };

    // ---- buffer resources: out-of-range lanes read zeros instead of faulting -------------------
    const uint32_t a_bytes = (uint32_t)p.k * (uint32_t)p.lda;
    const uint32_t b_bytes = (uint32_t)p.k * (uint32_t)p.n;
    __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)p.a, 0, a_bytes, 0x00020000);

    // ---- global -> LDS copy plan of a tile -------------------------------------------------------
    // Wave w, copy q fills the 1 KiB of LDS that starts at chunk slot (q*NWAVES + w)*64; lane l fills
    // slot P = that + l, which holds k row P/CPR, stored chunk P%CPR = logical chunk (P%CPR) ^ swz(k row).
    // The XOR mask of a lane does not depend on q, so a lane's global offset is one constant (k row of
    // copy 0, chunk column) plus a wave-uniform term (k block and q), which travels in an SGPR.
    // A chunk that starts beyond the matrix is pointed at the tile's first chunk (its rows are never
    // stored).  A chunk that starts inside and ends beyond it (m a multiple of 4 but not of 16) runs on
    // into the next k row, or, in the last k row, past the end of the buffer, where the per-dword range
    // check of the buffer load returns zeros: the rows that exist are always read from where they are.
    // Scales of a k block ride along in the tail of the stage: the a_scale row (BM floats, 64 per wave,
    // waves 0 .. BM/64-1) and the b_scale values of the tile's n blocks (the remaining waves, all the same
    // copy to the same place).  Every wave issues exactly one such 4-byte-per-lane copy, with its source
    // and destination in scalar registers: a branch here would split the K loop's straight-line block and
    // the compiler would sink the folds of the first MFMAs below it, away from the MFMAs they are meant
    // to overlap.  With the scales in LDS the K loop has no loads of its own that the compiler would have
    // to order against the output stores of the previous tile.
    constexpr int ROWS_PER_COPY_A = C::NWAVES * 64 / C::CPR_A, ROWS_PER_COPY_B = C::NWAVES * 64 / C::CPR_B;
    // With 12 chunks per k row of B one copy of the workgroup (NWAVES*64 chunks) does not end on a row
    // boundary: a lane's (k row, chunk) then differs from copy to copy and it keeps one offset per copy.
    constexpr bool B_ROWS_WHOLE = (C::NWAVES * 64) % C::CPR_B == 0;
    constexpr bool A_ROWS_WHOLE = (C::NWAVES * 64) % C::CPR_A == 0;
    constexpr int AS_COPIES = BM / 64;
    static_assert(C::NWAVES > AS_COPIES, "some wave must be left to copy the b_scale values");
    const bool sc_is_b = wave >= AS_COPIES;                       // this wave's scale copy is the b_scale one
    const uint32_t sc_dst = C::A_BYTES + C::B_BYTES + (sc_is_b ? C::AS_AREA : wave * 256);
    const uint32_t sc_kstep = (sc_is_b ? (uint32_t)p.nb : (uint32_t)p.lda) * 4u;
    struct CopyPlan {
        uint32_t a_voff, b_voff, sc_voff;
        uint32_t b_voffq[C::B_LOADS];           // only without B_ROWS_WHOLE
        uint32_t a_voffq[C::A_LOADS];           // only without A_ROWS_WHOLE
        int kb_begin;
        __amdgpu_buffer_rsrc_t b_rsrc, sc_rsrc;
    };
    auto copy_plan = [&](const Tile& t) -> CopyPlan {
        CopyPlan c;
        int P = wave * 64 + lane;
        int krow = P / C::CPR_A, ch = stored_to_chunk<C::CPR_A>(P % C::CPR_A, swz_of_krow<C::CPR_A>(krow));
        int col = t.m0 + 16 * ch;
        // A chunk of rows that all lie beyond the matrix, or that all belong to a later expert, is not fetched at
        // all.  Its lanes get an offset at the end of the buffer, for which the range check of the load returns
        // zeros without a memory access: one token row against a 64-row tile then moves one chunk of a per k row
        // instead of four, a tile that holds an expert's last few rows a few instead of sixteen.
        const bool skip = col >= t.row_hi && a_bytes < 0x80000000u;
        col = col < p.lda ? col : t.m0;
        c.a_voff = skip ? a_bytes : (uint32_t)krow * (uint32_t)p.lda + (uint32_t)col;
#pragma unroll
        for (int q = 0; q < C::A_LOADS; q++) {
            c.a_voffq[q] = 0;
            if constexpr (!A_ROWS_WHOLE) {
                const int Pq = q * C::NWAVES * 64 + P;
                const int kr = Pq / C::CPR_A;
                int cl = t.m0 + 16 * stored_to_chunk<C::CPR_A>(Pq % C::CPR_A, swz_of_krow<C::CPR_A>(kr));
                const bool skipq = cl >= t.row_hi && a_bytes < 0x80000000u;
                cl = cl < p.lda ? cl : t.m0;
                c.a_voffq[q] = skipq ? a_bytes : (uint32_t)kr * (uint32_t)p.lda + (uint32_t)cl;
            }
        }
        krow = P / C::CPR_B; ch = stored_to_chunk<C::CPR_B>(P % C::CPR_B, swz_of_krow<C::CPR_B>(krow));
        col = t.n0 + 16 * ch;
        const bool skip_b = col >= p.n && b_bytes < 0x80000000u;      // columns beyond the matrix: not fetched either
        col = col < p.n ? col : t.n0;
        c.b_voff = skip_b ? b_bytes : (uint32_t)krow * (uint32_t)p.n + (uint32_t)col;
#pragma unroll
        for (int q = 0; q < C::B_LOADS; q++) {
            c.b_voffq[q] = 0;
            if constexpr (!B_ROWS_WHOLE) {
                const int Pq = q * C::NWAVES * 64 + P;
                const int kr = Pq / C::CPR_B;
                int cl = t.n0 + 16 * stored_to_chunk<C::CPR_B>(Pq % C::CPR_B, swz_of_krow<C::CPR_B>(kr));
                const bool skipq = cl >= p.n && b_bytes < 0x80000000u;
                cl = cl < p.n ? cl : t.n0;
                c.b_voffq[q] = skipq ? b_bytes : (uint32_t)kr * (uint32_t)p.n + (uint32_t)cl;
            }
        }
        int r = sc_is_b ? t.n0 / 128 + lane : t.m0 + wave * 64 + lane;      // n block or row of a
        const int last = (sc_is_b ? p.nb : p.lda) - 1;
        r = r < last ? r : last;
        c.sc_voff = (uint32_t)r * 4u;
        c.kb_begin = t.kb_begin;
        c.b_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)t.bptr, 0, b_bytes, 0x00020000);
        c.sc_rsrc = __builtin_amdgcn_make_buffer_rsrc(sc_is_b ? (void*)t.bsptr : (void*)p.as, 0,
                                                      sc_is_b ? (uint32_t)(p.k / KBLK) * (uint32_t)p.nb * 4u
                                                              : (uint32_t)(p.k / KBLK) * (uint32_t)p.lda * 4u, 0x00020000);
        return c;
    };
    const uint32_t a_kstep = (uint32_t)KBLK * (uint32_t)p.lda, b_kstep = (uint32_t)KBLK * (uint32_t)p.n;

    // The copies are issued from inline assembly so that the compiler's hazard tracking does not see
    // them: it cannot tell that a copy into one stage never aliases the transposing reads of the other
    // stage and would otherwise make every LDS read wait for all outstanding copies.  Completion is
    // enforced by hand: s_waitcnt vmcnt(0) + workgroup barrier before the first read of a stage.
    const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char*)lds;
    constexpr int NLOADS = C::A_LOADS + C::B_LOADS + 1;     // + the scales
    // the counted waits below name up to two blocks of copies and a tile's output stores; the counter has six bits
    static_assert(2 * NLOADS + EPI_STORES <= 63, "vmcnt wait thresholds must fit the counter");
    // copy q (compile-time) of k block `blk` (relative to the tile's first) into `stage`
    auto issue_one = [&](const CopyPlan& cp, int stage, int blk, auto q_tag) {
        constexpr int q = decltype(q_tag)::value;
        const uint32_t sa = lds_base + stage * C::STAGE_BYTES + wave * 1024;
        const uint32_t kb = (uint32_t)(cp.kb_begin + blk);
        if constexpr (q < C::A_LOADS) {
            if constexpr (A_ROWS_WHOLE)
                copy16_global_to_lds(a_rsrc, sa + q * C::NWAVES * 1024, cp.a_voff, kb * a_kstep + (uint32_t)(q * ROWS_PER_COPY_A) * (uint32_t)p.lda);
            else
                copy16_global_to_lds(a_rsrc, sa + q * C::NWAVES * 1024, cp.a_voffq[q], kb * a_kstep);
        } else if constexpr (q < C::A_LOADS + C::B_LOADS) {
            constexpr int qb = q - C::A_LOADS;
            if constexpr (B_ROWS_WHOLE)
                copy16_global_to_lds(cp.b_rsrc, sa + C::A_BYTES + qb * C::NWAVES * 1024, cp.b_voff, kb * b_kstep + (uint32_t)(qb * ROWS_PER_COPY_B) * (uint32_t)p.n);
            else
                copy16_global_to_lds(cp.b_rsrc, sa + C::A_BYTES + qb * C::NWAVES * 1024, cp.b_voffq[qb], kb * b_kstep);
        } else {
            copy4_global_to_lds(cp.sc_rsrc, lds_base + stage * C::STAGE_BYTES + sc_dst, cp.sc_voff, kb * sc_kstep);
        }
    };
    auto issue_all = [&](const CopyPlan& cp, int stage, int blk) {
        [&]<int... Q>(std::integer_sequence<int, Q...>) {
            (issue_one(cp, stage, blk, std::integral_constant<int, Q>{}), ...);
        }(std::make_integer_sequence<int, NLOADS>{});
    };

    // ---- per-lane LDS read addresses -----------------------------------------------------------
    // transposing read j of a 16-row tile: k rows 32j + 8g + (i16>>1), byte half (i16&1)
    const int krow_lane = 8 * g + (i16 >> 1);
    const int swz_a = swz_of_krow<C::CPR_A>(krow_lane);     // independent of j (32j is a multiple of 16)
    const int swz_b = swz_of_krow<C::CPR_B>(krow_lane);
    const int a_lane_off = krow_lane * BM + (i16 & 1) * 8;
    const int b_lane_off = C::A_BYTES + krow_lane * BN + (i16 & 1) * 8;
    const int a_chunk0 = wave_m * (WM / 16), b_chunk0 = wave_n * (WN / 16);

    auto read_a = [&](v8i& dst, int t, const unsigned char* sbase) {
        const unsigned char* q = sbase + a_lane_off + (chunk_to_stored<C::CPR_A>(a_chunk0 + t, swz_a) << 4);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            v2i x = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_V2I(q + j * 32 * BM));
            dst[2 * j] = x[0]; dst[2 * j + 1] = x[1];
        }
    };
    auto read_b = [&](v8i& dst, int u, const unsigned char* sbase) {
        const unsigned char* q = sbase + b_lane_off + (chunk_to_stored<C::CPR_B>(b_chunk0 + u, swz_b) << 4);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            v2i x = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_V2I(q + j * 32 * BN));
            dst[2 * j] = x[0]; dst[2 * j + 1] = x[1];
        }
    };

    const int as_lane_off = C::A_BYTES + C::B_BYTES + (wave_m * WM + i16) * 4;
    const int bs_base = C::A_BYTES + C::B_BYTES + C::AS_AREA;     // slot i: b_scale of n block n0/128 + i

    // ---- rows of a that are not a multiple of four, columns of b that are not ------------------------
    // The buffer of a ends on a dword boundary (K is a multiple of 128), but with lda % 4 != 0 the copies
    // fetch its last one to three bytes in dwords that start inside and end beyond it; the range check
    // of a buffer load works on whole dwords and hands back zeros for those.  Every other byte of a
    // arrives intact (a dword that crosses the end of a k row just runs on into the next one).  The
    // workgroup whose tile holds those bytes writes them into LDS itself once the last K block has
    // landed: they all lie in the last aligned dword of a.  The same holds for b with n % 4 != 0.
    // The three candidates (byte offsets end-3 .. end-1) are worked out once, here, where registers are
    // plentiful, and kept in scalar registers.
    const bool a_tail = TAILS && (p.lda & 3) != 0 && p.k > 0;
    const bool b_tail = TAILS && (p.n & 3) != 0 && p.k > 0;
    uint32_t acand0 = 0, acand1 = 0, acand2 = 0, a_last = 0, bcand0 = 0, bcand1 = 0, bcand2 = 0, b_last = 0;
    if (a_tail) {
        const uint32_t end = (uint32_t)p.k * (uint32_t)p.lda;
        acand0 = tail_candidate(end - 3, (uint32_t)p.lda, end, (uint32_t)p.k);
        acand1 = tail_candidate(end - 2, (uint32_t)p.lda, end, (uint32_t)p.k);
        acand2 = tail_candidate(end - 1, (uint32_t)p.lda, end, (uint32_t)p.k);
        a_last = load_last_dword(p.a + (end - 4));
    }
    if (b_tail) {
        const uint32_t end = (uint32_t)p.k * (uint32_t)p.n;
        bcand0 = tail_candidate(end - 3, (uint32_t)p.n, end, (uint32_t)p.k);
        bcand1 = tail_candidate(end - 2, (uint32_t)p.n, end, (uint32_t)p.k);
        bcand2 = tail_candidate(end - 1, (uint32_t)p.n, end, (uint32_t)p.k);
        if (MODE != 2) b_last = load_last_dword(p.b + (end - 4));     // grouped: every expert's matrix has last bytes of its own, read per tile
    }
    // (the loads are consumed here, not inside the K loop)
    acand0 = __builtin_amdgcn_readfirstlane(acand0); acand1 = __builtin_amdgcn_readfirstlane(acand1);
    acand2 = __builtin_amdgcn_readfirstlane(acand2); a_last = __builtin_amdgcn_readfirstlane(a_last);
    bcand0 = __builtin_amdgcn_readfirstlane(bcand0); bcand1 = __builtin_amdgcn_readfirstlane(bcand1);
    bcand2 = __builtin_amdgcn_readfirstlane(bcand2); b_last = __builtin_amdgcn_readfirstlane(b_last);
    // stage: the tile's last K block; called by every wave right behind the barrier that publishes that
    // block; ends with a second barrier
#define FP8BS_PATCH_TAILS(stage, spare_stage)                                                                                              \
    do {                                                                                                                                   \
        patch_tail_bytes<BM, C::CPR_A>(lds + (stage) * C::STAGE_BYTES, lds + (spare_stage) * C::STAGE_BYTES + C::STAGE_BYTES - 1,          \
                                       patch_tile && a_tail, m0, acand0, acand1, acand2, a_last, tid);                                     \
        patch_tail_bytes<BN, C::CPR_B>(lds + (stage) * C::STAGE_BYTES + C::A_BYTES, lds + (spare_stage) * C::STAGE_BYTES + C::STAGE_BYTES - 1, \
                                       patch_tile && b_tail, n0, bcand0, bcand1, bcand2, b_last, tid);                                     \
        __syncthreads();                                                                                                                   \
    } while (0)

    Tile cur = pick_tile(0);
    if (!cur.valid) return;
    CopyPlan cp = copy_plan(cur);
    bool prefetched = false;                // block 0 of `cur` is already on its way into stage 0
    bool stores_behind = false;             // ... and this wave's output stores of the previous tile were issued after it
    for (int it = 0;; it++) {
    const int m0 = cur.m0, n0 = cur.n0, kb_begin = cur.kb_begin, kb_end = cur.kb_end, split_z = cur.split_z;
    const int row_lo = cur.row_lo, row_hi = cur.row_hi;
    [[maybe_unused]] const int sk_contrib = cur.sk_contrib, sk_first = cur.sk_first;
    if constexpr (TAILS && MODE == 2) {
        if (b_tail) b_last = __builtin_amdgcn_readfirstlane(load_last_dword(cur.bptr + ((uint32_t)p.k * (uint32_t)p.n - 4u)));
    }
    // a_scale: lane's output row of m-tile t is tile row wave_m*WM + 16t + i16, read from the stage's
    // copy of the a_scale row.
    // does any element of this wave's tile get stored?  (rows of the expert / matrix, columns of the matrix)
    const bool wave_active = __builtin_amdgcn_readfirstlane((m0 + wave_m * WM < row_hi && m0 + wave_m * WM + WM > row_lo &&
                                                             n0 + wave_n * WN < p.n) ? 1 : 0) != 0;
    // b_scale of the wave's n tiles: slot bs_off for n tiles [0, ub), the next slot for [ub, NT)
    const int wave_col = (C::SPLIT_SCALES ? (n0 & 127) : 0) + wave_n * WN;               // from the start of the tile's first n block
    const int bs_off = bs_base + (wave_col >> 7) * 4;
    const int ub = C::SPLIT_SCALES ? (128 - (wave_col & 127)) >> 4 : C::NT;

    v4f acc[C::MT][C::NT];
#pragma unroll
    for (int t = 0; t < C::MT; t++)
#pragma unroll
        for (int u = 0; u < C::NT; u++) acc[t][u] = (v4f){0.f, 0.f, 0.f, 0.f};

    const int nkb = kb_end - kb_begin;
    const bool patch_tile = TAILS && kb_end * KBLK == p.k;        // this tile's last K block is the last of a and b
    if (nkb > 0) {
        constexpr int STEPS = C::MT * C::NT;
        constexpr int LAG = 3, RING = 4;      // fold the result of step s-LAG while step s runs
        // Copies of block j+2 start right behind the barrier of block j (NL_LATE of them, one per
        // trailing step) and continue one every DMA_EVERY steps of block j+1: a burst would block this
        // wave's instruction issue until the texture unit has taken it, and the MFMAs queued behind.
        constexpr int NL_LATE = C::MT < 2 ? C::MT : 2;
        constexpr int NL_EARLY = NLOADS - NL_LATE;
        // (the 192-wide tile is the exception, measured: one copy per step gives it 0.92 us per K block on
        // one CU against 1.02, while the 256-wide tile loses 4 % that way)
        constexpr int DMA_EVERY = BN == 192 ? 1 : ((STEPS - C::MT) / NL_EARLY >= 2 ? 2 : 1), DMA_FIRST = DMA_EVERY - 1;
        static_assert(NL_EARLY * DMA_EVERY <= STEPS - C::MT, "not enough steps to issue the copies before the barrier");

        // ---- prologue: blocks 0 .. NSTAGE-2 -> stages 0 .. NSTAGE-2 (unless the previous tile already
        //      sent them), wait for block 0; first copies of block NSTAGE-1 -> the last stage.  The
        //      barrier also ends the previous tile's use of the last stage as the staging area of its
        //      output ----
        // The vector memory counter retires loads and stores in the order they were issued.  If block 0
        // was sent ahead of the previous tile's NSTORES output stores, "at most NSTORES outstanding" means
        // the block has landed, and the stores are left to finish under the first K block.  With three
        // stages block 1 (NLOADS copies) sits between block 0 and the stores.
        if (!prefetched) {
            issue_all(cp, 0, 0);
            if constexpr (NSTAGE == 3) { if (nkb > 1) issue_all(cp, 1, 1); }
        }
        if constexpr (NSTAGE == 2) {
            if (prefetched && stores_behind) wait_vmcnt<EPI_STORES>();
            else wait_vmcnt<0>();
        } else {
            const bool sb = prefetched && stores_behind;
            if (nkb > 1) { if (sb) wait_vmcnt<NLOADS + EPI_STORES>(); else wait_vmcnt<NLOADS>(); }
            else { if (sb) wait_vmcnt<EPI_STORES>(); else wait_vmcnt<0>(); }
        }
        __syncthreads();
        if (TAILS && nkb == 1) FP8BS_PATCH_TAILS(0, 1);
        if (nkb > NSTAGE - 1) {
            [&]<int... Q>(std::integer_sequence<int, Q...>) {
                (issue_one(cp, NSTAGE - 1, NSTAGE - 1, std::integral_constant<int, Q>{}), ...);
            }(std::make_integer_sequence<int, NL_LATE>{});
        }

        v8i areg[C::MT], breg[2];
        if (wave_active) {
#pragma unroll
            for (int t = 0; t < C::MT; t++) read_a(areg[t], t, lds);
            read_b(breg[0], 0, lds);
        }

        // All K blocks of the tile.  UB: the wave's n tiles [UB, NT) belong to the next b_scale block
        // (UB = NT: none does).
        auto run_blocks = [&](auto ub_tag) {
        constexpr int UB = decltype(ub_tag)::value;
        // One K block (index j, in stage j&1).  The flags are compile-time so that the step sequence
        // is one straight-line block for the instruction scheduler.
        // Block j lives in stage j % NSTAGE.  While it is multiplied, the rest of block j+NSTAGE-1 is
        // copied into the stage that the barrier of block j-1 freed; behind the barrier of block j the
        // first copies of block j+NSTAGE go into the stage just read.  With two stages a copy has one
        // block's time to land, with three stages two.
        auto k_block = [&](int j, auto h1_tag, auto h2_tag, auto h3_tag) {
            constexpr bool HAS_NEXT = decltype(h1_tag)::value;                                              // block j+1 exists
            constexpr bool HAS_EARLY = NSTAGE == 2 ? decltype(h1_tag)::value : decltype(h2_tag)::value;    // block j+NSTAGE-1 exists
            constexpr bool HAS_LATE = NSTAGE == 2 ? decltype(h2_tag)::value : decltype(h3_tag)::value;     // block j+NSTAGE exists
            constexpr bool LANDS_LAST = decltype(h1_tag)::value && !decltype(h2_tag)::value;               // block j+1 is the tile's last
            const int cur_stage = NSTAGE == 2 ? (j & 1) : j % NSTAGE;
            const int next_stage = cur_stage + 1 == NSTAGE ? 0 : cur_stage + 1;
            const int early_stage = NSTAGE == 2 ? next_stage : (next_stage + 1 == NSTAGE ? 0 : next_stage + 1);
            // what must have landed at the barrier is block j+1; with three stages the NLOADS copies of
            // block j+2 were all issued after it and may stay in flight
            auto wait_next_block = [&]() {
                if constexpr (NSTAGE == 3 && HAS_EARLY) wait_vmcnt_lgkm0<NLOADS>();
                else __builtin_amdgcn_s_waitcnt(0x0070);   // vmcnt(0) lgkmcnt(0)
            };
            if (!wave_active) {
                // none of this wave's rows is stored: it only does its share of the copies, in the
                // same order and around the same single barrier as the waves that compute
                if constexpr (HAS_EARLY) {
                    [&]<int... Q>(std::integer_sequence<int, Q...>) {
                        (issue_one(cp, early_stage, j + NSTAGE - 1, std::integral_constant<int, NL_LATE + Q>{}), ...);
                    }(std::make_integer_sequence<int, NL_EARLY>{});
                }
                wait_next_block();
                __syncthreads();
                if constexpr (TAILS && LANDS_LAST) FP8BS_PATCH_TAILS(next_stage, cur_stage);
                if constexpr (HAS_LATE) {
                    [&]<int... Q>(std::integer_sequence<int, Q...>) {
                        (issue_one(cp, cur_stage, j + NSTAGE, std::integral_constant<int, Q>{}), ...);
                    }(std::make_integer_sequence<int, NL_LATE>{});
                }
                return;
            }
            const unsigned char* sbase = lds + cur_stage * C::STAGE_BYTES;
            const unsigned char* snext = lds + next_stage * C::STAGE_BYTES;
            float sc[C::MT], sc1[C::MT];
            const float bsv = *(const float*)(sbase + bs_off);
            const float bsv1 = UB < C::NT ? *(const float*)(sbase + bs_off + 4) : 0.f;
#pragma unroll
            for (int t = 0; t < C::MT; t++) {
                const float asv = *(const float*)(sbase + as_lane_off + t * 64);
                sc[t] = asv * bsv;
                sc1[t] = UB < C::NT ? asv * bsv1 : 0.f;
            }
            v4f ring[RING];
            auto step = [&](auto s_tag) {
                constexpr int s = decltype(s_tag)::value;
                if constexpr (s < STEPS) {
                    constexpr int u = s / C::MT, t = s % C::MT;
                    if constexpr (HAS_EARLY && s % DMA_EVERY == DMA_FIRST && s / DMA_EVERY < NL_EARLY)
                        issue_one(cp, early_stage, j + NSTAGE - 1, std::integral_constant<int, NL_LATE + s / DMA_EVERY>{});
                    if constexpr (t == 0 && u + 1 < C::NT) read_b(breg[(u + 1) & 1], u + 1, sbase);
                    if constexpr (t == 0 && u == C::NT - 1) {
                        // All reads of this stage are issued.  Wait for them and for this wave's part
                        // of the next block, then meet the other waves: after the barrier the next
                        // block is complete in the other stage and this stage may be overwritten.
                        wait_next_block();
                        __syncthreads();
                        if constexpr (TAILS && LANDS_LAST) FP8BS_PATCH_TAILS(next_stage, cur_stage);
                    }
                    const v4f z = {0.f, 0.f, 0.f, 0.f};
                    ring[s % RING] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(breg[u & 1], areg[t], z, 0, 0, 0, 0, 0, 0);
                    if constexpr (u == C::NT - 1 && HAS_NEXT) {
                        // operands of the next block, fetched while the last MFMAs of this one run
                        read_a(areg[t], t, snext);
                        if constexpr (t == 0) read_b(breg[0], 0, snext);
                    }
                    if constexpr (u == C::NT - 1 && HAS_LATE && t < NL_LATE)
                        issue_one(cp, cur_stage, j + NSTAGE, std::integral_constant<int, t>{});
                }
                if constexpr (s >= LAG) {
                    constexpr int sp = s - LAG, u = sp / C::MT, t = sp % C::MT;
#pragma unroll
                    for (int r = 0; r < 4; r++) acc[t][u][r] = __builtin_fmaf(ring[sp % RING][r], u < UB ? sc[t] : sc1[t], acc[t][u][r]);
                }
                __builtin_amdgcn_sched_barrier(0);
            };
            [&]<int... S>(std::integer_sequence<int, S...>) {
                (step(std::integral_constant<int, S>{}), ...);
            }(std::make_integer_sequence<int, STEPS + LAG>{});
        };

        constexpr std::true_type T{};
        constexpr std::false_type F{};
        int j = 0;
        if constexpr (NSTAGE == 2) {
            for (; j + 2 < nkb; j++) k_block(j, T, T, F);
            if (j + 1 < nkb) { k_block(j, T, F, F); j++; }
        } else {
            for (; j + 3 < nkb; j++) k_block(j, T, T, T);
            if (j + 2 < nkb) { k_block(j, T, T, F); j++; }
            if (j + 1 < nkb) { k_block(j, T, F, F); j++; }
        }
        k_block(j, F, F, F);
        };   // run_blocks
        if constexpr (C::SPLIT_SCALES) {
            // 96-column wave tiles of a 192-column tile start 0, 96, 64 or 160 columns into a block
            if (ub == 2) run_blocks(std::integral_constant<int, 2>{});
            else if (ub == 4) run_blocks(std::integral_constant<int, 4>{});
            else run_blocks(std::integral_constant<int, C::NT>{});
        } else {
            run_blocks(std::integral_constant<int, C::NT>{});
        }
    }

    else if (it > 0) {
        __syncthreads();                    // nothing to multiply: still let the previous tile's staging reads finish
    }

    // ---- the next tile's first K blocks (all stages but the last) start now: after the last barrier
    //      above no wave reads a stage any more, and the output below is staged in the last stage only ----
    Tile nxt = pick_tile(it + 1);
    CopyPlan ncp = cp;
    prefetched = false;
    if (nxt.valid) {
        ncp = copy_plan(nxt);
        if (nxt.kb_end > nxt.kb_begin) {
            issue_all(ncp, 0, 0);
            if constexpr (NSTAGE == 3) { if (nxt.kb_end - nxt.kb_begin > 1) issue_all(ncp, 1, 1); }
            prefetched = true;
        }
    }

    // ---- K blocks dealt to the workgroups: partial tiles travel through the workspace ---------------
    // Partial tiles are written and read with agent-scope accesses (sc1: written through to, and read from,
    // the memory side of the eight L2s), in the order of the lanes: the two sides run the same tile shape, so
    // accumulator (t, u) of wave w is the 1 KiB piece number w*MT*NT + t*NT + u of the slot.
    bool store_output = true;
    if constexpr (MODE == 3) {
        constexpr uint32_t SLOT_BYTES = (uint32_t)BM * (uint32_t)BN * 4u;
        constexpr int NG = C::MT * C::NT;
        constexpr int AUX_AGENT = 16;                                           // sc1
        unsigned char* const ws_base = (unsigned char*)p.ws;
        unsigned long long* const flags = (unsigned long long*)(ws_base + StreamK::FLAGS_OFF);
        unsigned char* const slots = ws_base + StreamK::SLOTS_OFF;
        if (sk_contrib) {
            store_output = false;
            if (wave_active) {
                // (the accumulators are next written after the wait below: nothing follows these stores closely)
                __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)(slots + (size_t)sk_self * SLOT_BYTES), 0, SLOT_BYTES, 0x00020000);
                const uint32_t voff = (uint32_t)(wave * NG) * 1024u + (uint32_t)lane * 16u;
#pragma unroll
                for (int t = 0; t < C::MT; t++)
#pragma unroll
                    for (int u = 0; u < C::NT; u++)
                        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, acc[t][u]), rs, voff + (uint32_t)(t * C::NT + u) * 1024u, 0, AUX_AGENT);
            }
            // A store with sc1 is written through to the agent's point of coherence and is counted by vmcnt
            // until it is acknowledged from there, so after this wait every wave's part of the tile can be
            // seen by any CU that reads it with sc1; the barrier then lets one lane raise the flag for all.
            // (An agent-scope release fence in its place writes the whole L2 back once per wave: 4096 x 2112
            // x 7168 took 131 us with it against 81 us, 64 x 18432 x 7168 76 us against 30 us.)
            wait_vmcnt<0>();
            __syncthreads();
            if (tid == 0) __hip_atomic_store(&flags[sk_self], p.sk_nonce, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else if (sk_first >= 0) {
            // The tile's owner: wait, a bounded number of polls, for the flags of the workgroups that hold the
            // tile's earlier K blocks (one lane per flag, all polled together), take the flags down again (so
            // that a replay of the same launch starts clean), then add the partial tiles to the accumulators in
            // ascending order of K: ((own + P_first) + P_next) + ...  A wait that gives up leaves the status
            // word set and the kernel runs on to its end with whatever the slots hold.
            if (wave == 0) {
                bool ok = p.sk_spin >= 0;
                for (int base = sk_first; ok && base < sk_self; base += 64) {
                    const int u = base + lane;
                    const bool mine = u < sk_self;
                    int spins = p.sk_spin;
                    for (;;) {
                        const unsigned long long f = mine ? __hip_atomic_load(&flags[u], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : p.sk_nonce;
                        if (__ballot(f != p.sk_nonce) == 0) break;
                        if (--spins < 0) { ok = false; break; }
                        __builtin_amdgcn_s_sleep(2);
                    }
                    if (ok && mine) __hip_atomic_store(&flags[u], 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                if (!ok && lane == 0) __hip_atomic_store((unsigned int*)ws_base, StreamK::STATUS_TIMEOUT, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            __syncthreads();
            if (wave_active) {
                // loads in flight at a time: what the registers beside the accumulators hold
                constexpr int BATCH = NG <= 8 ? NG : (NG % 4 == 0 ? 4 : (NG % 3 == 0 ? 3 : 1));
                __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)slots, 0, (uint32_t)gridDim.x * SLOT_BYTES, 0x00020000);
                const uint32_t voff = (uint32_t)(wave * NG) * 1024u + (uint32_t)lane * 16u;
#pragma unroll
                for (int base = 0; base < NG; base += BATCH) {
#pragma unroll 2
                    for (int u = sk_first; u < sk_self; u++) {
                        const uint32_t soff = (uint32_t)u * SLOT_BYTES + (uint32_t)base * 1024u;
                        v4f part[BATCH];
#pragma unroll
                        for (int i = 0; i < BATCH; i++)
                            part[i] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rs, voff, soff + i * 1024u, AUX_AGENT));
#pragma unroll
                        for (int i = 0; i < BATCH; i++)
                            acc[(base + i) / C::NT][(base + i) % C::NT] += part[i];
                    }
                    __builtin_amdgcn_sched_barrier(0);      // the registers hold the whole tile already: one batch at a time
                }
            }
        }
    } else if constexpr (MODE == 4) {
        // K split in one launch, nobody waits: every workgroup leaves its partial tile in the slot
        // (tile, K partition) and then counts itself in at the tile's counter; the one that finds all others
        // counted in before it adds the partial tiles in ascending order of K - ((P0 + P1) + P2) + ..., its own
        // from the registers, the order of the separate reduce kernel - and writes the bf16 tile.  The counter
        // carries the call's tag in its upper 48 bits, so whatever an earlier use of the workspace left there
        // counts as zero; the last workgroup puts it back to zero for a replay of the same launch.
        constexpr uint32_t SLOT_BYTES = (uint32_t)BM * (uint32_t)BN * 4u;
        constexpr int NG = C::MT * C::NT;
        constexpr int AUX_AGENT = 16;                                           // sc1
        __shared__ int last_in;
        unsigned char* const ws_base = (unsigned char*)p.ws;
        unsigned long long* const counters = (unsigned long long*)(ws_base + StreamK::FLAGS_OFF);
        unsigned char* const tile_slots = ws_base + StreamK::SLOTS_OFF + (size_t)sk_first * (size_t)p.split_k * SLOT_BYTES;
        const uint32_t voff = (uint32_t)(wave * NG) * 1024u + (uint32_t)lane * 16u;
        // (the counter is read ahead of the stores: the value only seeds the exchange below, which finds out if it is stale)
        unsigned long long seen = 0;
        if (tid == 0) seen = __hip_atomic_load(&counters[sk_first], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // Lanes whose row or columns lie outside the matrix neither store nor load their piece (an offset beyond the
        // slot drops a store and makes a load return zeros): one row against 18432 columns leaves 1 KB per workgroup
        // in the workspace instead of 32 KB (31.6 us with every lane storing, against 29.1 as two launches).
        uint32_t rows_in = 0, cols_in = 0;                 // bit t: the lane's row of m tile t exists; bit u: its columns of n tile u
#pragma unroll
        for (int t = 0; t < C::MT; t++) rows_in |= (m0 + wave_m * WM + 16 * t + i16 < row_hi ? 1u : 0u) << t;
#pragma unroll
        for (int u = 0; u < C::NT; u++) cols_in |= (n0 + wave_n * WN + 16 * u + 4 * g < p.n ? 1u : 0u) << u;
        auto piece = [&](int x) -> uint32_t {               // x = t * NT + u, a compile-time number at every use
            return ((rows_in >> (x / C::NT)) & (cols_in >> (x % C::NT)) & 1u) ? voff + (uint32_t)x * 1024u : 0xFFFFFFFFu;
        };
        if (wave_active) {
            __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)(tile_slots + (size_t)split_z * SLOT_BYTES), 0, SLOT_BYTES, 0x00020000);
#pragma unroll
            for (int t = 0; t < C::MT; t++)
#pragma unroll
                for (int u = 0; u < C::NT; u++)
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, acc[t][u]), rs, piece(t * C::NT + u), 0, AUX_AGENT);
        }
        wait_vmcnt<0>();                                    // acknowledged from the agent's point of coherence
        __syncthreads();
        if (tid == 0) {
            const unsigned long long tag = (p.sk_nonce | 0x10000ull) & ~0xFFFFull;       // never zero
            unsigned long long count;
            for (;;) {
                count = (seen & ~0xFFFFull) == tag ? (seen & 0xFFFFull) : 0ull;
                if (__hip_atomic_compare_exchange_strong(&counters[sk_first], &seen, tag | (count + 1), __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) break;
            }
            const int last = (int)(count + 1) == p.split_k;
            if (last) __hip_atomic_store(&counters[sk_first], 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            last_in = last;
        }
        __syncthreads();
        store_output = __builtin_amdgcn_readfirstlane(last_in) != 0;
        if (store_output && wave_active) {
            auto slot_of = [&](int z) { return __builtin_amdgcn_make_buffer_rsrc((void*)(tile_slots + (size_t)z * SLOT_BYTES), 0, SLOT_BYTES, 0x00020000); };
            // S partitions known at compile time: the loads of all other partitions' pieces of a batch are in flight
            // together (up to 16 of 16 bytes per lane); S = 0: any number, one partition at a time
            [[maybe_unused]] auto sum_planes = [&]<int S>() {
                constexpr int WANT = S > 1 ? (16 / (S - 1) > 0 ? 16 / (S - 1) : 1) : 4;
                constexpr int BATCH = WANT >= NG ? NG : (WANT >= 4 && NG % 4 == 0 ? 4 : (WANT >= 3 && NG % 3 == 0 ? 3 : (WANT >= 2 && NG % 2 == 0 ? 2 : 1)));
                const int nz = S > 0 ? S : p.split_k;
#pragma unroll
                for (int base = 0; base < NG; base += BATCH) {
                    if constexpr (S > 0) {
                        v4f part[S - 1][BATCH];                              // the other partitions, ascending
#pragma unroll
                        for (int j = 0; j < S - 1; j++) {
                            __amdgpu_buffer_rsrc_t rs = slot_of(j + (j >= split_z ? 1 : 0));
#pragma unroll
                            for (int i = 0; i < BATCH; i++)
                                part[j][i] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rs, piece(base + i), 0, AUX_AGENT));
                        }
#pragma unroll
                        for (int i = 0; i < BATCH; i++) {
                            v4f& own = acc[(base + i) / C::NT][(base + i) % C::NT];
                            v4f sum = part[0][i];
                            if (split_z == 0) sum = own + sum;                  // (the same bits as sum + own)
#pragma unroll
                            for (int j = 1; j < S - 1; j++) {
                                if (j == split_z) sum += own;
                                sum += part[j][i];
                            }
                            if (split_z == S - 1) sum += own;
                            own = sum;
                        }
                    } else {
                        v4f sum[BATCH];
                        for (int z = 0; z < nz; z++) {
                            v4f part[BATCH];
                            if (z == split_z) {
#pragma unroll
                                for (int i = 0; i < BATCH; i++) part[i] = acc[(base + i) / C::NT][(base + i) % C::NT];
                            } else {
                                __amdgpu_buffer_rsrc_t rs = slot_of(z);
#pragma unroll
                                for (int i = 0; i < BATCH; i++)
                                    part[i] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rs, piece(base + i), 0, AUX_AGENT));
                            }
#pragma unroll
                            for (int i = 0; i < BATCH; i++) sum[i] = z == 0 ? part[i] : sum[i] + part[i];
                        }
#pragma unroll
                        for (int i = 0; i < BATCH; i++) acc[(base + i) / C::NT][(base + i) % C::NT] = sum[i];
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            };
            if constexpr (NG > 16) {
                // 72 to 128 accumulator registers leave room for one partition's batch of three or four (the loop of
                // the S = 0 case above, written out: called through the lambda it cost the 256x256 tile ~40 spilled registers)
                constexpr int GB = NG % 4 == 0 ? 4 : (NG % 3 == 0 ? 3 : (NG % 2 == 0 ? 2 : 1));
#pragma unroll
                for (int base = 0; base < NG; base += GB) {
                    v4f sum[GB];
                    for (int z = 0; z < p.split_k; z++) {
                        v4f part[GB];
                        if (z == split_z) {
#pragma unroll
                            for (int i = 0; i < GB; i++) part[i] = acc[(base + i) / C::NT][(base + i) % C::NT];
                        } else {
                            __amdgpu_buffer_rsrc_t rs = slot_of(z);
#pragma unroll
                            for (int i = 0; i < GB; i++)
                                part[i] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rs, piece(base + i), 0, AUX_AGENT));
                        }
#pragma unroll
                        for (int i = 0; i < GB; i++) sum[i] = z == 0 ? part[i] : sum[i] + part[i];
                    }
#pragma unroll
                    for (int i = 0; i < GB; i++) acc[(base + i) / C::NT][(base + i) % C::NT] = sum[i];
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
                switch (p.split_k) {
                    case 2: sum_planes.template operator()<2>(); break;
                    case 3: sum_planes.template operator()<3>(); break;
                    case 4: sum_planes.template operator()<4>(); break;
                    case 5: sum_planes.template operator()<5>(); break;
                    case 6: sum_planes.template operator()<6>(); break;
                    default: sum_planes.template operator()<0>(); break;
                }
            }
        }
    }

    // ---- epilogue (a wave without valid rows has nothing to store; no barrier in here) -----------
    if (!wave_active || !store_output) {
    } else if (MODE == 1) {
        // split-K: fp32 partial tile, 16 bytes per lane
#pragma unroll
        for (int t = 0; t < C::MT; t++) {
            const int row = m0 + wave_m * WM + 16 * t + i16;
            if (row >= row_hi) continue;
#pragma unroll
            for (int u = 0; u < C::NT; u++) {
                const int col = n0 + wave_n * WN + 16 * u + 4 * g;
                if (col >= p.n) continue;
                float* dst = p.ws + ((size_t)split_z * p.m + row) * (size_t)p.n + col;
                if constexpr (!TAILS) {
                    *(v4f*)dst = acc[t][u];
                } else {
                    // rows of the plane start on any 4-byte boundary and may end inside the lane's four columns
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        if (col + r < p.n) dst[r] = acc[t][u][r];
                }
            }
        }
    } else {
        // bf16 through LDS so that the global stores are 16 bytes per lane and every store
        // instruction writes whole rows of the wave tile (WNO*2 contiguous bytes each).  (Measured against the
        // route through the registers alone - v_permlane16_swap pairing the 8-byte pieces of neighbouring lane
        // groups into 16-byte ones, a rotation by 8 lanes so that an instruction writes 128-byte lines, no LDS:
        // 4096^3 59.9-60.1 us against 60.2-60.5 with this staging on the same box, but 6144 x 7168 x 256 29.5
        // against 27.5, 1024 x 7168 x 2048 19.4 against 18.9, the grouped configuration 915 against 901; with
        // 64-byte pieces per row, no rotation, 58.1 against 56.1 on 4096^3.  Rows of 256 bytes per instruction
        // are what the write path takes best, and the staging costs less than the narrower stores.)  The last
        // stage is free (after the barrier of the last K block no wave reads it and no copy into it is in
        // flight); the stages before it already receive the next tile.  Each wave stages its tile in two halves of
        // WM/2 rows in its own region; 16-byte chunks are XOR-swizzled by row so that neither the
        // writes (16 rows per instruction) nor the 16-byte reads conflict.
        constexpr int WNO = EPI == 1 ? WN / 2 : WN;                   // output columns of the wave tile
        constexpr int ROW_CHUNKS = WNO * 2 / 16;                      // 16-byte chunks per tile row
        constexpr int ROWS_PER_SWEEP = 16 / ROW_CHUNKS > 0 ? 16 / ROW_CHUNKS : 1;
        constexpr int HALF_ROWS = WM / EPI_PARTS, HALF_MT = C::MT / EPI_PARTS;    // a "half" is one of EPI_PARTS parts: two, or one per m tile if their number is odd
        // A row of 12 chunks is staged with one chunk of padding instead of the XOR swizzle: with 13
        // chunks from row to row, 16 consecutive rows of one chunk column fall on 16 different bank groups.
        constexpr bool ROW_POW2 = (ROW_CHUNKS & (ROW_CHUNKS - 1)) == 0;
        constexpr int RSTRIDE = ROW_POW2 ? WNO * 2 : WNO * 2 + 16;    // bytes from row to row in the staging area
        static_assert(C::MT % EPI_PARTS == 0 && C::NWAVES * HALF_ROWS * RSTRIDE <= C::STAGE_BYTES, "output staging must fit one stage");
        unsigned char* region = lds + (NSTAGE - 1) * C::STAGE_BYTES + wave * (HALF_ROWS * RSTRIDE);
        const int ldc = EPI == 1 ? p.n / 2 : p.n;
        // Stores go through buffer descriptors: an offset of 0xFFFFFFFF drops the lane's store, so the
        // instruction count does not depend on the data.  Each store gets a descriptor based at the first
        // element of its group of rows (scalar arithmetic only); the scalar-offset operand is not used:
        // with it, the vector ALU instruction that follows a 16-byte store was seen to overwrite the
        // store's data register before the store had read it (the compiler pads that case only for
        // stores without a scalar offset).
        const int col0 = EPI == 1 ? n0 / 2 : n0;
        uint16_t* const c_tile = p.c + (size_t)m0 * ldc + col0;
        const bool c_lines = p.c_whole_lines != 0;          // uniform: a kernel argument
#pragma unroll
        for (int half = 0; half < EPI_PARTS; half++) {
#pragma unroll
            for (int th = 0; th < HALF_MT; th++) {
                const int t = half * HALF_MT + th;
                const int r = 16 * th + i16;
                const int sw = ROW_POW2 ? (r / ROWS_PER_SWEEP) % ROW_CHUNKS : 0;
                if constexpr (EPI == 0 && C::NT % 2 == 0) {
                    // The lane's 8 bytes of n tile u and of n tile u+1 become 16 consecutive bytes of one of them:
                    // v_permlane16_swap exchanges lanes 16-31 / 48-63 of its first operand with lanes 0-15 / 32-47 of
                    // its second, so after swapping the low and the high dwords lane group g holds columns
                    // 16*(u + g%2) + 8*(g/2) .. +7 - one whole 16-byte chunk, written to LDS in one instruction
                    // instead of two (half the LDS cycles of the staging: 4096^3 59.3 against 59.6 us, 8192 x 8192 x 2048
                    // 124.7 against 126.3, 4096 x 4096 x 16384 213.0 against 214.9; 6144 x 7168 x 256 28.1 against 27.8).
#pragma unroll
                    for (int u = 0; u < C::NT; u += 2) {
                        const uint32_t lo0 = pack_bf16x2(acc[t][u][0], acc[t][u][1]), hi0 = pack_bf16x2(acc[t][u][2], acc[t][u][3]);
                        const uint32_t lo1 = pack_bf16x2(acc[t][u + 1][0], acc[t][u + 1][1]), hi1 = pack_bf16x2(acc[t][u + 1][2], acc[t][u + 1][3]);
                        const auto sl = __builtin_amdgcn_permlane16_swap(lo0, lo1, false, false);
                        const auto sh = __builtin_amdgcn_permlane16_swap(hi0, hi1, false, false);
                        const v4i o = {(int)sl[0], (int)sh[0], (int)sl[1], (int)sh[1]};
                        const int chunk = 2 * (u + (g & 1)) + (g >> 1);
                        *(v4i*)(region + r * RSTRIDE + ((chunk ^ sw) << 4)) = o;
                    }
                } else {
#pragma unroll
                for (int u = 0; u < C::NT; u++) {
                    if (EPI == 1) {
                        // the lane's four columns are two (gate, up) pairs -> two outputs, 4 bytes
                        const uint32_t o = pack_bf16x2(silu_mul(acc[t][u][0], acc[t][u][1]), silu_mul(acc[t][u][2], acc[t][u][3]));
                        *(uint32_t*)(region + r * RSTRIDE + ((u ^ sw) << 4) + g * 4) = o;
                    } else {
                        v2i o;
                        o[0] = (int)pack_bf16x2(acc[t][u][0], acc[t][u][1]);
                        o[1] = (int)pack_bf16x2(acc[t][u][2], acc[t][u][3]);
                        const int chunk = 2 * u + (g >> 1);
                        *(v2i*)(region + r * RSTRIDE + ((chunk ^ sw) << 4) + (g & 1) * 8) = o;
                    }
                }
                }
            }
            // A pass = one 16-byte store per lane.  With 12 chunks per row a pass covers 4 rows with 48 lanes
            // (the other 16 are switched off like out-of-range ones), so that, as in the power-of-two
            // case, a lane keeps its row-in-pass and chunk over all passes.
            constexpr int ROWS_PER_PASS = ROW_POW2 ? 64 / ROW_CHUNKS : 4, PASSES = HALF_ROWS / ROWS_PER_PASS;
            static_assert(HALF_ROWS % ROWS_PER_PASS == 0 && ROWS_PER_PASS * ROW_CHUNKS <= 64, "a half tile is a whole number of passes");
            static_assert(MODE == 1 || EPI_STORES == EPI_PARTS * PASSES, "store count used by the next tile's wait");
            // lane -> (row inside the pass, chunk); everything else about a store's address is uniform
            // and sits in the descriptor, so the 16 stores need one address register, not 16
            const int lane_r = lane / ROW_CHUNKS, lane_chunk = lane % ROW_CHUNKS;
            const bool lane_live = ROW_POW2 || lane_r < ROWS_PER_PASS;
            const int wave_row0 = wave_m * WM, wave_col0 = wave_n * WNO;              // inside the tile, output columns
            const bool col_ok = lane_live && col0 + wave_col0 + lane_chunk * 8 < ldc;
            const uint32_t lane_off = ((uint32_t)(wave_row0 + lane_r) * (uint32_t)ldc + (uint32_t)(wave_col0 + lane_chunk * 8)) * 2u;
#pragma unroll
            for (int q = 0; q < PASSES; q++) {
                const int r = q * ROWS_PER_PASS + (lane_live ? lane_r : 0);
                const int sw = ROW_POW2 ? (r / ROWS_PER_SWEEP) % ROW_CHUNKS : 0;
                const v4i val = *(const v4i*)(region + r * RSTRIDE + ((lane_chunk ^ sw) << 4));
                const int pass_row0 = half * HALF_ROWS + q * ROWS_PER_PASS;            // compile-time
                const int row = m0 + wave_row0 + pass_row0 + lane_r;
                const bool ok = col_ok && row >= row_lo && row < row_hi;
                __amdgpu_buffer_rsrc_t c_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)(c_tile + (size_t)pass_row0 * ldc), 0, 0xFFFFFFF0u, 0x00020000);
                if constexpr (!TAILS) {
                    // Written once and not read again here: nontemporal where rows of c are whole 128-byte lines.
                    // Where they are not, a tile's row segment begins and ends inside lines that it shares with
                    // the neighbouring tiles; plain stores let the L2 put those lines together before they leave
                    // (4096 x 4088 x 4096: 61 us against 65 us with the hint; with whole lines the hint gains 1 us).
                    if (c_lines) __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, val), c_rsrc, ok ? lane_off : 0xFFFFFFFFu, 0, 2);
                    else __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, val), c_rsrc, ok ? lane_off : 0xFFFFFFFFu, 0, 0);
                } else {
                    // n not a multiple of eight: the chunk that holds a row's last columns is stored in
                    // pieces of 4, 2 and 1 elements (the bits of the number of columns left), every piece
                    // its own instruction that the other lanes sit out; rows then start on 2-, 4- or
                    // 8-byte boundaries only, which the stores take in their stride (plain stores: the lines a
                    // row segment shares with the neighbouring tiles are put together in the L2)
                    int left = ldc - (col0 + wave_col0 + lane_chunk * 8);                  // columns from this chunk's first to the row's end
                    left = left < 0 ? 0 : (left > 8 ? 8 : left);
                    const bool part = ok && left < 8;
                    const v4u v = __builtin_bit_cast(v4u, val);
                    __builtin_amdgcn_raw_buffer_store_b128(v, c_rsrc, ok && left == 8 ? lane_off : 0xFFFFFFFFu, 0, 0);
                    const v2i lo = {val[0], val[1]};
                    __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(v2u, lo), c_rsrc, part && (left & 4) ? lane_off : 0xFFFFFFFFu, 0, 0);
                    const uint32_t d2 = (left & 4) ? v[2] : v[0];                          // elements (left & 4), +1
                    __builtin_amdgcn_raw_buffer_store_b32(d2, c_rsrc, part && (left & 2) ? lane_off + (uint32_t)(left & 4) * 2u : 0xFFFFFFFFu, 0, 0);
                    const int e1 = left & 6;                                               // element (left & 6)
                    const uint32_t d1 = e1 == 0 ? v[0] : e1 == 2 ? v[1] : e1 == 4 ? v[2] : v[3];
                    __builtin_amdgcn_raw_buffer_store_b16((unsigned short)(d1 & 0xFFFFu), c_rsrc, part && (left & 1) ? lane_off + (uint32_t)e1 * 2u : 0xFFFFFFFFu, 0, 0);
                }
            }
        }
    }
    if (!nxt.valid) break;
    stores_behind = prefetched && wave_active && MODE != 1 && !TAILS && store_output;   // (with TAILS the store count is four times EPI_STORES: plain wait)
    cur = nxt; cp = ncp;
    }   // tiles
}

#undef FP8BS_PATCH_TAILS

// ---------------------------------------------------------------------------------------------------
// Launchers
// ---------------------------------------------------------------------------------------------------
template <int BM, int BN, int WM, int WN, int MODE, int EPI = 0, int NSTAGE = 2>
static inline hipError_t launch_tr(const GemmArgs& a, dim3 grid, hipStream_t stream) {
    using C = TileCfg<BM, BN, WM, WN, MODE, NSTAGE>;
    // rows of a that are not a multiple of four, columns that are not a multiple of eight, operands that
    // start off the 16-byte grid: the instantiation that repairs the last bytes of a and b and stores c
    // without assuming any alignment of its rows
    // (with the fused epilogue the rows of the output have n/2 columns: 16-byte stores need n/2 on the 8-column grid)
    const int out_cols = EPI == 1 ? a.n / 2 : a.n;
    const bool tails = (a.lda & 3) != 0 || (a.n & 7) != 0 || (out_cols & 7) != 0 || (((uintptr_t)a.a | (uintptr_t)a.b | (uintptr_t)a.c) & 15) != 0;
    GemmArgs args = a;
    args.c_whole_lines = ((size_t)out_cols * 2u) % 128u == 0 && ((uintptr_t)a.c & 127) == 0;
    void (*kern)(const GemmArgs) = tails ? gemm_tr_kernel<BM, BN, WM, WN, MODE, EPI, NSTAGE, true> : gemm_tr_kernel<BM, BN, WM, WN, MODE, EPI, NSTAGE, false>;
    static int raised[2][MAX_DEVICES];
    hipError_t e = raise_lds_limit((const void*)kern, C::LDS_BYTES, raised[tails ? 1 : 0]);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, grid, dim3(C::NTHREADS), C::LDS_BYTES, stream, args);
    return hipGetLastError();
}

template <int BM, int BN, int WM, int WN, bool WITH_EPI = false, int NSTAGE = 2>
static inline hipError_t launch_shape(const GemmArgs& a, int mode, hipStream_t stream) {
    using C = TileCfg<BM, BN, WM, WN, 0, NSTAGE>;
    // persistent workgroups: as many as fit the chip at once (LDS and thread limits), each walks
    // tiles  blockIdx.x, blockIdx.x + grid, ...
    const int by_lds = 163840 / (C::LDS_BYTES + (mode == 2 ? GROUP_TABLE_MAX * 16 : 0)), by_threads = 2048 / C::NTHREADS;   // (grouped: + the table of the experts)
    const long resident = (long)device_cus() * (by_lds < by_threads ? by_lds : by_threads);
    const int tiles_n = (a.n + BN - 1) / BN;
    long total;
    if (mode == 2) {
        // upper bound on m-tile slots: every expert can waste up to 15 rows (aligned-down start)
        // plus one partial tile; workgroups beyond the real count find no tile and leave
        total = (((long)a.m + BM - 1) / BM + 2L * a.num_experts) * tiles_n;
    } else {
        total = (long)((a.m + BM - 1) / BM) * tiles_n * a.split_k;
    }
    if (mode == 3) {
        // K blocks dealt to the workgroups: one workgroup per place on the chip, never more than there are
        // (tile, K block) pairs, so that every workgroup's run holds at least one
        if (a.epi != 0 || a.k < KBLK) return hipErrorInvalidValue;
        const long pairs = (long)((a.m + BM - 1) / BM) * tiles_n * (a.k / KBLK);
        if (a.sk_grid < 1 || a.sk_grid > resident || a.sk_grid > pairs || a.sk_grid > StreamK::MAX_GRID) return hipErrorInvalidValue;
        return launch_tr<BM, BN, WM, WN, 3, 0, NSTAGE>(a, dim3((unsigned)a.sk_grid), stream);
    }
    const dim3 grid((unsigned)(total < resident ? total : resident));
    if (mode == 4) {
        // K split summed by the last workgroup of every tile: one counter per tile in the workspace's head
        const long tiles = total / a.split_k;
        if (a.epi != 0 || a.split_k < 2 || a.split_k > 0xFFFF || tiles > StreamK::MAX_GRID || (long)a.split_k * BM * BN * 4 >= (1L << 32)) return hipErrorInvalidValue;
        return launch_tr<BM, BN, WM, WN, 4, 0, NSTAGE>(a, grid, stream);
    }
    if (a.epi != 0) {
        // the fused silu-mul epilogue exists for the 256x256 tile, dense or grouped, without K split
        if constexpr (WITH_EPI) {
            if (a.epi != 1 || mode == 1) return hipErrorInvalidValue;
            if (mode == 2) return launch_tr<BM, BN, WM, WN, 2, 1>(a, grid, stream);
            return launch_tr<BM, BN, WM, WN, 0, 1>(a, grid, stream);
        } else {
            return hipErrorInvalidValue;
        }
    }
    if (mode == 2) return launch_tr<BM, BN, WM, WN, 2, 0, NSTAGE>(a, grid, stream);
    if (mode == 1) return launch_tr<BM, BN, WM, WN, 1, 0, NSTAGE>(a, grid, stream);
    return launch_tr<BM, BN, WM, WN, 0, 0, NSTAGE>(a, grid, stream);
}

}  // namespace fp8bs
