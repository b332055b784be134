// MoE routing in front of the grouped FP8 GEMM, for gfx950 (MI355X): top-k expert selection, the
// row_offsets table and the expert-contiguous row order, all on the device and without a host sync.
//
// Roles in the reference (fp16 MoE layer, 2-amd-moe/amd-moe-submission.py):
//   topk / top4_nre32            :32-56, :58-105    per token, k times: the strictly greatest score not yet
//                                                   taken, lowest index first among equals, best first
//   calculate_index(_nre32_ept4) :107-117, :119-156 position of every (token, choice) inside its expert,
//                                                   handed out by atomicAdd (order varies from run to run)
//   calculate_offset             2-amd-moe/3-amd-fp8-moe-hip-myhgemm.py:142-148   exclusive prefix of the counts
//   host read of the counts      :230-234           hipDeviceSynchronize + loop, to size the next launch
// Here the positions are deterministic: rows of an expert are ordered by token id (then choice), which
// is what a stable sort by expert gives and what inputs.make_grouped builds.  Counting is done per block
// of 256 tokens in LDS (integer atomics: the totals do not depend on the order), a one-block scan turns
// the per-block counts into bases and the expert totals into row_offsets[E+1] (total appended), and a
// third kernel ranks every choice inside its block from LDS bitmaps and writes
//   row_map[row] = token   (the gather list fp8bs_quantize_a takes)   and   slot_of[token][choice] = row.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

#include "fp8bs.h"

namespace fp8bs {

static constexpr int RB = 256;            // tokens per block
static constexpr int MAX_EXPERTS = 1024;  // LDS: 32 bytes of bitmap per expert
static constexpr int MAX_TOPK = 16;       // a token's choices are held in registers

// the choices of token t, all loads in flight at once; absent entries are -1; an expert repeated by the
// token is kept at its first occurrence only (later ones become -1 as well)
__device__ __forceinline__ void load_choices(const int32_t* __restrict__ top_idx, int t, int tokens, int experts, int topk, int (&ch)[MAX_TOPK]) {
#pragma unroll
    for (int j = 0; j < MAX_TOPK; j++) ch[j] = (t < tokens && j < topk) ? top_idx[(size_t)t * topk + j] : -1;
#pragma unroll
    for (int j = 0; j < MAX_TOPK; j++) {
        bool keep = ch[j] >= 0 && ch[j] < experts;
#pragma unroll
        for (int l = 0; l < j; l++) keep &= ch[l] != ch[j];
        ch[j] = keep ? ch[j] : -1;
    }
}

// one thread per token; scores row-major [tokens][experts].  "Not yet taken" needs no list: the picks
// come out in the strict order (score descending, index ascending), so a candidate is eligible exactly
// when it lies behind the previous pick in that order.
__global__ __launch_bounds__(RB)
void moe_topk_kernel(const float* __restrict__ scores, int tokens, int experts, int topk, int32_t* __restrict__ top_idx) {
    const int t = blockIdx.x * RB + threadIdx.x;
    if (t >= tokens) return;
    const float* row = scores + (size_t)t * experts;
    int32_t* out = top_idx + (size_t)t * topk;
    float prev = __builtin_inff();
    int prev_j = -1;
    bool none = false;
    for (int i = 0; i < topk; i++) {
        float best = -__builtin_inff();
        int best_j = -1;
        if (!none)
            for (int j = 0; j < experts; j++) {
                const float v = row[j];
                const bool eligible = i == 0 || v < prev || (v == prev && j > prev_j);
                if (eligible && v > best) { best = v; best_j = j; }     // strictly greater: lowest index wins a tie, NaN never wins
            }
        out[i] = best_j;
        none = best_j < 0;
        prev = best; prev_j = best_j;
    }
}

// same rule for experts <= 64, one wave per token, lane j = expert j.  Scores are mapped to unsigned
// keys that order like the floats (0 = "never selected": NaN, -inf, lanes beyond the experts); a pick is
// the wave-wide maximum key, its lowest lane among equals; the picked lane then drops out.
__device__ __forceinline__ uint32_t umax32(uint32_t a, uint32_t b) { return a > b ? a : b; }
__global__ __launch_bounds__(RB)
void moe_topk64_kernel(const float* __restrict__ scores, int tokens, int experts, int topk, int32_t* __restrict__ top_idx) {
    const int lane = threadIdx.x & 63;
    const int wave = blockIdx.x * (RB / 64) + (threadIdx.x >> 6), nwaves = gridDim.x * (RB / 64);
    for (int t = wave; t < tokens; t += nwaves) {
        const float v = lane < experts ? scores[(size_t)t * experts + lane] : -__builtin_inff();
        uint32_t u = __builtin_bit_cast(uint32_t, v);
        u = u == 0x80000000u ? 0u : u;              // -0.0 and +0.0 compare equal: one key, the lowest index wins
        uint32_t key = v > -__builtin_inff() ? ((u & 0x80000000u) ? ~u : (u | 0x80000000u)) : 0u;
        int mine = -1;                              // lane i keeps pick i
        for (int i = 0; i < topk; i++) {
            uint32_t m = key;
            m = umax32(m, (uint32_t)__builtin_amdgcn_mov_dpp((int)m, 0xB1, 0xF, 0xF, true));    // quad_perm [1,0,3,2]
            m = umax32(m, (uint32_t)__builtin_amdgcn_mov_dpp((int)m, 0x4E, 0xF, 0xF, true));    // quad_perm [2,3,0,1]
            m = umax32(m, (uint32_t)__builtin_amdgcn_mov_dpp((int)m, 0x141, 0xF, 0xF, true));   // row_half_mirror
            m = umax32(m, (uint32_t)__builtin_amdgcn_mov_dpp((int)m, 0x140, 0xF, 0xF, true));   // row_mirror
            const uint32_t best = umax32(umax32((uint32_t)__builtin_amdgcn_readlane((int)m, 0), (uint32_t)__builtin_amdgcn_readlane((int)m, 16)),
                                         umax32((uint32_t)__builtin_amdgcn_readlane((int)m, 32), (uint32_t)__builtin_amdgcn_readlane((int)m, 48)));
            int pick = -1;
            if (best != 0u) {                       // wave-uniform
                const uint64_t hit = __builtin_amdgcn_ballot_w64(key == best);
                pick = __builtin_ctzll(hit);
                if (lane == pick) key = 0u;
            }
            if (lane == i) mine = pick;
        }
        if (lane < topk) top_idx[(size_t)t * topk + lane] = mine;
    }
}

// block_counts[b][e] = number of choices of expert e among the tokens of block b
__global__ __launch_bounds__(RB)
void route_count_kernel(const int32_t* __restrict__ top_idx, int tokens, int experts, int topk, int32_t* __restrict__ block_counts) {
    __shared__ int hist[MAX_EXPERTS];
    for (int e = threadIdx.x; e < experts; e += RB) hist[e] = 0;
    __syncthreads();
    const int t = blockIdx.x * RB + threadIdx.x;
    int ch[MAX_TOPK];
    load_choices(top_idx, t, tokens, experts, topk, ch);
#pragma unroll
    for (int j = 0; j < MAX_TOPK; j++)
        if (ch[j] >= 0) atomicAdd(&hist[ch[j]], 1);
    __syncthreads();
    for (int e = threadIdx.x; e < experts; e += RB) block_counts[(size_t)blockIdx.x * experts + e] = hist[e];
}

// one block: per expert an exclusive prefix over the blocks (in place), then an exclusive prefix over
// the experts into row_offsets[0..E]
__global__ __launch_bounds__(RB)
void route_scan_kernel(int32_t* __restrict__ block_counts, int nblocks, int experts, int32_t* __restrict__ row_offsets) {
    __shared__ int total[MAX_EXPERTS];
    for (int e = threadIdx.x; e < experts; e += RB) {
        int run = 0;
        for (int b = 0; b < nblocks; b++) {
            const int c = block_counts[(size_t)b * experts + e];
            block_counts[(size_t)b * experts + e] = run;
            run += c;
        }
        total[e] = run;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int run = 0;
        for (int e = 0; e < experts; e++) { row_offsets[e] = run; run += total[e]; }
        row_offsets[experts] = run;
    }
}

// rank of every choice among the choices of the same expert in its block (by token id), from one
// 256-bit bitmap per expert; a token's choices are distinct experts, a repeated expert keeps one row.
// SCAN_HERE: block_base holds the raw per-block counts and every block derives its own bases and the
// row offsets from them (few blocks: cheaper than a launch of its own); block 0 writes row_offsets.
template <bool SCAN_HERE>
__global__ __launch_bounds__(RB)
void route_assign_kernel(const int32_t* __restrict__ top_idx, int tokens, int experts, int topk,
                         const int32_t* __restrict__ block_base, int32_t* __restrict__ row_offsets,
                         int32_t* __restrict__ row_map, int32_t* __restrict__ slot_of) {
    __shared__ uint32_t bits[MAX_EXPERTS * (RB / 32)];
    __shared__ int first_row[MAX_EXPERTS];       // first row of this block's tokens inside expert e's segment
    __shared__ int part[RB];
    __shared__ int tot_s[SCAN_HERE ? MAX_EXPERTS : 1], base_s[SCAN_HERE ? MAX_EXPERTS : 1];
    int row_offsets_total;                       // row_offsets[experts]: rows that belong to some expert
    for (int i = threadIdx.x; i < experts * (RB / 32); i += RB) bits[i] = 0;
    if (SCAN_HERE) {
        // totals over all blocks and bases over the blocks before this one, summed in LDS (integer
        // atomics: order-independent) with all loads of a sweep in flight at once; then thread x owns
        // experts 4x .. 4x+3 for the prefix over the experts
        const int nblocks = gridDim.x;
        for (int e = threadIdx.x; e < experts; e += RB) { tot_s[e] = 0; base_s[e] = 0; }
        __syncthreads();
        for (int idx = threadIdx.x; idx < nblocks * experts; idx += RB) {
            const int b = idx / experts, e = idx - b * experts;
            const int c = block_base[idx];
            atomicAdd(&tot_s[e], c);
            if (b < (int)blockIdx.x) atomicAdd(&base_s[e], c);
        }
        __syncthreads();
        int tot[4], base[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int e = 4 * threadIdx.x + i;
            tot[i] = e < experts ? tot_s[e] : 0;
            base[i] = e < experts ? base_s[e] : 0;
        }
        part[threadIdx.x] = tot[0] + tot[1] + tot[2] + tot[3];
        __syncthreads();
        for (int off = 1; off < RB; off <<= 1) {           // inclusive scan of the 256 partial sums
            const int v = threadIdx.x >= off ? part[threadIdx.x - off] : 0;
            __syncthreads();
            part[threadIdx.x] += v;
            __syncthreads();
        }
        int run = part[threadIdx.x] - (tot[0] + tot[1] + tot[2] + tot[3]);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int e = 4 * threadIdx.x + i;
            if (e < experts) {
                first_row[e] = run + base[i];
                if (blockIdx.x == 0) row_offsets[e] = run;
            }
            run += tot[i];
        }
        if (blockIdx.x == 0 && threadIdx.x == RB - 1) row_offsets[experts] = part[RB - 1];
        row_offsets_total = part[RB - 1];
    } else {
        for (int e = threadIdx.x; e < experts; e += RB) first_row[e] = row_offsets[e] + block_base[(size_t)blockIdx.x * experts + e];
        row_offsets_total = row_offsets[experts];
    }
    __syncthreads();
    const int t = blockIdx.x * RB + threadIdx.x;
    const int w = threadIdx.x >> 5, bit = threadIdx.x & 31;
    int ch[MAX_TOPK];
    load_choices(top_idx, t, tokens, experts, topk, ch);
#pragma unroll
    for (int j = 0; j < MAX_TOPK; j++)
        if (ch[j] >= 0) atomicOr(&bits[ch[j] * (RB / 32) + w], 1u << bit);
    __syncthreads();
    // rows beyond the last expert's (they exist only if some choices were outside [0, experts)) map to no token
    for (int r = row_offsets_total + blockIdx.x * RB + threadIdx.x; r < tokens * topk; r += gridDim.x * RB) row_map[r] = -1;
    if (t >= tokens) return;
#pragma unroll
    for (int j = 0; j < MAX_TOPK; j++) {
        if (j < topk) {
            int dest = -1;
            if (ch[j] >= 0) {
                const uint32_t* bm = bits + ch[j] * (RB / 32);
                int rank = __builtin_popcount(bm[w] & ((1u << bit) - 1u));
#pragma unroll
                for (int x = 0; x < RB / 32; x++) rank += x < w ? __builtin_popcount(bm[x]) : 0;
                dest = first_row[ch[j]] + rank;
                row_map[dest] = t;
            }
            if (slot_of) slot_of[(size_t)t * topk + j] = dest;
        }
    }
}

// out[t][d] = sum_j weights[t][j] * y[slot_of[t][j]][d], fp32 accumulation in the order j = 0..topk-1,
// one rounding to bf16 (role of pack_output, 2-amd-moe/amd-moe-submission.py:239-301, which accumulates
// in fp16).  One block per token, 8 columns (16 bytes) per thread and step; entries whose slot is not a
// row of y (-1 or beyond) are skipped.
typedef int cv4i __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(RB)
void moe_combine_kernel(const uint16_t* __restrict__ y, const int32_t* __restrict__ slot_of, const float* __restrict__ weights,
                        uint16_t* __restrict__ out, int rows, int topk, int d) {
    const int t = blockIdx.x;
    for (int c = threadIdx.x * 8; c < d; c += RB * 8) {
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        // four rows at a time, all four loads issued before the first is used (one after the other a step costs
        // one memory latency per choice); a choice that is skipped enters as weight 0 times zeros, which leaves
        // the sum as it is
        for (int j0 = 0; j0 < topk; j0 += 4) {
            cv4i v[4];
            float w[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int j = j0 + i;
                const int slot = j < topk ? slot_of[(size_t)t * topk + j] : -1;
                const bool ok = slot >= 0 && slot < rows;
                w[i] = ok ? weights[(size_t)t * topk + j] : 0.f;
                v[i] = (cv4i){0, 0, 0, 0};
                if (ok) v[i] = __builtin_nontemporal_load((const cv4i*)(y + (size_t)slot * d + c));
            }
#pragma unroll
            for (int i = 0; i < 4; i++) {
#pragma unroll
                for (int x = 0; x < 4; x++) {
                    acc[2 * x] = __builtin_fmaf(w[i], __builtin_bit_cast(float, (uint32_t)v[i][x] << 16), acc[2 * x]);
                    acc[2 * x + 1] = __builtin_fmaf(w[i], __builtin_bit_cast(float, (uint32_t)v[i][x] & 0xFFFF0000u), acc[2 * x + 1]);
                }
            }
        }
        cv4i o;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            typedef float cv2f __attribute__((ext_vector_type(2)));
            typedef __bf16 cv2bf __attribute__((ext_vector_type(2)));
            cv2f f = {acc[2 * i], acc[2 * i + 1]};
            o[i] = (int)__builtin_bit_cast(uint32_t, __builtin_convertvector(f, cv2bf));
        }
        *(cv4i*)(out + (size_t)t * d + c) = o;
    }
}

}  // namespace fp8bs

extern "C" int fp8bs_moe_topk(const float* scores, int tokens, int experts, int topk, int32_t* top_idx, void* stream) {
    if (tokens < 0 || experts <= 0 || topk <= 0 || topk > experts) return FP8BS_ERR_BAD_SHAPE;
    if (tokens == 0) return FP8BS_OK;
    if (!scores || !top_idx) return FP8BS_ERR_NULL_POINTER;
    if (experts <= 64)
        hipLaunchKernelGGL(fp8bs::moe_topk64_kernel, dim3(tokens < 4096 ? (tokens + 3) / 4 : 1024), dim3(fp8bs::RB), 0, (hipStream_t)stream,
                           scores, tokens, experts, topk, top_idx);
    else
        hipLaunchKernelGGL(fp8bs::moe_topk_kernel, dim3((tokens + fp8bs::RB - 1) / fp8bs::RB), dim3(fp8bs::RB), 0, (hipStream_t)stream,
                           scores, tokens, experts, topk, top_idx);
    return hipGetLastError() == hipSuccess ? FP8BS_OK : FP8BS_ERR_LAUNCH;
}

extern "C" size_t fp8bs_moe_route_workspace_bytes(int tokens, int experts) {
    if (tokens <= 0 || experts <= 0) return 0;
    return (size_t)((tokens + fp8bs::RB - 1) / fp8bs::RB) * (size_t)experts * sizeof(int32_t);
}

extern "C" int fp8bs_moe_route(const int32_t* top_idx, int tokens, int experts, int topk, int32_t* row_offsets,
                               int32_t* row_map, int32_t* slot_of, void* ws, size_t ws_bytes, void* stream) {
    if (tokens < 0 || experts <= 0 || topk <= 0 || topk > fp8bs::MAX_TOPK) return FP8BS_ERR_BAD_SHAPE;
    if (experts > fp8bs::MAX_EXPERTS) return FP8BS_ERR_BAD_OFFSETS;
    if (!row_offsets) return FP8BS_ERR_NULL_POINTER;
    if ((size_t)tokens * (size_t)topk > 0x7FFFFFFFull) return FP8BS_ERR_TOO_LARGE;
    hipStream_t s = (hipStream_t)stream;
    const int nblocks = (tokens + fp8bs::RB - 1) / fp8bs::RB;
    if (tokens == 0) {
        hipLaunchKernelGGL(fp8bs::route_scan_kernel, dim3(1), dim3(fp8bs::RB), 0, s, (int32_t*)ws, 0, experts, row_offsets);
        return hipGetLastError() == hipSuccess ? FP8BS_OK : FP8BS_ERR_LAUNCH;
    }
    if (!top_idx || !row_map) return FP8BS_ERR_NULL_POINTER;
    if (!ws || ws_bytes < fp8bs_moe_route_workspace_bytes(tokens, experts)) return FP8BS_ERR_WORKSPACE;
    hipLaunchKernelGGL(fp8bs::route_count_kernel, dim3(nblocks), dim3(fp8bs::RB), 0, s, top_idx, tokens, experts, topk, (int32_t*)ws);
    if (hipGetLastError() != hipSuccess) return FP8BS_ERR_LAUNCH;
    if (nblocks <= 64) {
        // few blocks: every block of the assign kernel scans the counts itself
        hipLaunchKernelGGL(fp8bs::route_assign_kernel<true>, dim3(nblocks), dim3(fp8bs::RB), 0, s, top_idx, tokens, experts, topk,
                           (const int32_t*)ws, row_offsets, row_map, slot_of);
    } else {
        hipLaunchKernelGGL(fp8bs::route_scan_kernel, dim3(1), dim3(fp8bs::RB), 0, s, (int32_t*)ws, nblocks, experts, row_offsets);
        if (hipGetLastError() != hipSuccess) return FP8BS_ERR_LAUNCH;
        hipLaunchKernelGGL(fp8bs::route_assign_kernel<false>, dim3(nblocks), dim3(fp8bs::RB), 0, s, top_idx, tokens, experts, topk,
                           (const int32_t*)ws, row_offsets, row_map, slot_of);
    }
    return hipGetLastError() == hipSuccess ? FP8BS_OK : FP8BS_ERR_LAUNCH;
}

extern "C" int fp8bs_moe_combine(const void* y, int rows, const int32_t* slot_of, const float* weights, void* out,
                                 int tokens, int topk, int d, void* stream) {
    if (tokens < 0 || rows < 0 || topk <= 0 || d < 0 || (d % 8) != 0) return FP8BS_ERR_BAD_SHAPE;
    if (tokens == 0 || d == 0) return FP8BS_OK;
    if (!y || !slot_of || !weights || !out) return FP8BS_ERR_NULL_POINTER;
    if ((((uintptr_t)y | (uintptr_t)out) & 15) != 0) return FP8BS_ERR_BAD_SHAPE;      // 16-byte row accesses
    hipLaunchKernelGGL(fp8bs::moe_combine_kernel, dim3(tokens), dim3(fp8bs::RB), 0, (hipStream_t)stream,
                       (const uint16_t*)y, slot_of, weights, (uint16_t*)out, rows, topk, d);
    return hipGetLastError() == hipSuccess ? FP8BS_OK : FP8BS_ERR_LAUNCH;
}
