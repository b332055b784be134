// Streaming (skinny-M) kernel, split-K reduction, scalar kernel and the dispatch over the kernel variants.
// The tiled MFMA kernel is a template in fp8bs_tiled.h, instantiated per tile shape in fp8bs_tile_*.hip
// (one translation unit each, so that they compile side by side).
#include "fp8bs_tiled.h"

namespace fp8bs {

// ---------------------------------------------------------------------------------------------------
// Skinny-M streaming kernel (bandwidth-bound shapes: a few rows of A against a long B).
//
// One workgroup = 64 rows of A x 144 columns of B over a K range; 4 waves.  The work per K block is
// tiny, the time goes into streaming B from HBM once, so the design is a deep ring of LDS stages kept
// full by asynchronous global->LDS copies: NSTAGE = 4 stages of (A 8 KiB + B 18 KiB + scales), three K
// blocks in flight per workgroup, one barrier per K block (a fifth stage measured slower: workgroups
// drift further apart in K and evict the 128-byte lines they share with their neighbours from L2).
// Split-K partial planes are summed by a separate small kernel: an in-kernel last-arriver reduction
// was measured 1.5x slower overall, because exchanging the planes between XCDs needs either an L2
// write-back + invalidate per workgroup (which evicts the B lines still in use) or device-coherent
// 4-byte accesses.  144 = 9 sixteen-byte chunks: with an odd
// number of chunks per k row the 16 k rows a transposing read touches already fall on 16 different bank
// groups, so the B tile needs no swizzle; and 18432 / 144 = 128 tiles x split-K 2 fills 256 CUs exactly.
// Every wave issues the same number of copies per block (7), which makes "block j has landed" a fixed
// s_waitcnt vmcnt threshold.  The scales of the block (a_scale row, the <= 3 b_scale values the 144
// columns span) ride the same ring.
//   MODE 0: bf16 output      MODE 1: fp32 split-K partial planes
// ---------------------------------------------------------------------------------------------------
// Tile widths: 144 (9 chunks: odd, no swizzle needed), 288 (18 chunks: the 8 k rows one 16-lane group
// reads are still 8 different bank groups), 256 (16 chunks: XOR swizzle as in the main kernel; rows are
// whole 128-byte lines, the cheapest for the texture path).  The copies of a block are padded with
// repeats of the last one to the same number per wave, which makes "block j has landed" a fixed
// s_waitcnt vmcnt threshold.
template <int BN_, int NSTAGE_>
struct SkinnyCfg {
    static constexpr int BM = 64, BN = BN_, CPR_A = 4, CPR_B = BN / 16, NWAVES = 4, NTHREADS = 256;
    static constexpr bool SWZ_B = (CPR_B % 2 == 0) && (CPR_B != 18);
    static constexpr int A_BYTES = KBLK * BM, B_BYTES = KBLK * BN, SC_BYTES = 1024;
    static constexpr int STAGE_BYTES = A_BYTES + B_BYTES + SC_BYTES;
    static constexpr int NSTAGE = NSTAGE_;
    static constexpr int LDS_BYTES = NSTAGE * STAGE_BYTES;
    static constexpr int A_COPIES = A_BYTES / 1024, B_COPIES = B_BYTES / 1024;
    static constexpr int COPIES = (A_COPIES + B_COPIES + 2 + NWAVES - 1) / NWAVES;     // per wave per K block
    static constexpr int MT = BM / 16, NT_MAX = (CPR_B + NWAVES - 1) / NWAVES;        // n tiles per wave
    static_assert(!SWZ_B || CPR_B == 16, "the XOR swizzle is written for 256-byte rows");
    static_assert((NSTAGE - 2) * COPIES <= 63, "vmcnt has 6 bits");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS");
};


// MTV: the 16-row m tiles that get multiplied, 1..4.  Fewer than 4 only when the whole matrix has at
// most 16*MTV rows (a decode step has one to a few): a compile-time count, because a run-time test per
// m tile put branches between the MFMAs and their folds, and results read back too early were seen.
// TAILS: lda is not a multiple of four; the last bytes of a are repaired in LDS as in the tiled kernel.
template <int BN_, int NSTAGE_, int MODE, int MTV, bool TAILS = false>
__global__ __launch_bounds__(256)
void gemm_skinny_kernel(const GemmArgs p) {
    using C = SkinnyCfg<BN_, NSTAGE_>;
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 4, i16 = lane & 15;

    const int tiles_n = (p.n + C::BN - 1) / C::BN;
    // neighbouring n tiles can share 128-byte lines of every k row of B: give each XCD a contiguous
    // run of tiles so that the shared lines are fetched into one L2 only
    const int bid = xcd_virtual_id(blockIdx.x, gridDim.x);
    const int tn = bid % tiles_n, split_z = (bid / tiles_n) % p.split_k, tm = bid / (tiles_n * p.split_k);
    const int m0 = tm * C::BM, n0 = tn * C::BN;
    const int kbt = p.k / KBLK;
    const int kb_begin = split_z * p.kb_per_split;
    int kb_end = kb_begin + p.kb_per_split;
    kb_end = kb_end < kbt ? kb_end : kbt;
    const int nkb = kb_end - kb_begin;
    const int nb0 = n0 / 128;

    const uint32_t a_bytes = (uint32_t)p.k * (uint32_t)p.lda, b_bytes = (uint32_t)p.k * (uint32_t)p.n;
    const uint32_t as_bytes = (uint32_t)kbt * (uint32_t)p.lda * 4u, bs_bytes = (uint32_t)kbt * (uint32_t)p.nb * 4u;

    // ---- copy plan.  The one-KiB copies of a block are numbered I = 4q + wave, q = 0..COPIES-1:
    //      I < A_COPIES the A tile, then B_COPIES of the B tile (copy Ib fills B chunks 64*Ib ..), then the
    //      a_scale row, then the b_scale values (repeated as padding).  Lane offsets are fixed for the
    //      whole kernel; the K block enters through the wave-uniform offset.  Chunks that start beyond
    //      the matrix re-read the tile's first chunk (never stored).
    uint32_t voff[C::COPIES];
#pragma unroll
    for (int q = 0; q < C::COPIES; q++) {
        const int I = 4 * q + wave;
        uint32_t v;
        if (I < C::A_COPIES) {
            int krow = 16 * I + lane / 4;
            int c = (lane % 4) ^ swz_of_krow<C::CPR_A>(krow);
            int col = m0 + 16 * c;
            col = col < p.lda ? col : m0;
            v = (uint32_t)krow * (uint32_t)p.lda + (uint32_t)col;
        } else if (I < C::A_COPIES + C::B_COPIES) {
            int P = 64 * (I - C::A_COPIES) + lane;
            int kr = P / C::CPR_B, cc = P % C::CPR_B;
            if (C::SWZ_B) cc ^= swz_of_krow<C::CPR_B>(kr);
            int cl = n0 + 16 * cc;
            cl = cl < p.n ? cl : n0;
            v = (uint32_t)kr * (uint32_t)p.n + (uint32_t)cl;
        } else if (I == C::A_COPIES + C::B_COPIES) {
            int r = m0 + lane; r = r < p.lda - 1 ? r : p.lda - 1;
            v = (uint32_t)r * 4u;
        } else {
            int x = nb0 + lane; x = x < p.nb - 1 ? x : p.nb - 1;
            v = (uint32_t)x * 4u;
        }
        voff[q] = v;
    }
    const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char*)lds;
    // All copies of K block `blk` (relative to kb_begin).  Beyond the last block the same number of
    // copies is issued against empty buffers (every lane out of range: zeros land in a free stage and no
    // memory is read), which keeps the count of outstanding copies per wave the same in every iteration.
    auto issue_block = [&](auto wave_tag, int blk) {
        constexpr int W = decltype(wave_tag)::value;
        const uint32_t st = lds_base + (uint32_t)(blk % C::NSTAGE) * C::STAGE_BYTES;
        const bool live = blk < nkb;
        const uint32_t kb = (uint32_t)(kb_begin + (live ? blk : 0));
        __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)p.a, 0, live ? a_bytes : 0u, 0x00020000);
        __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)p.b, 0, live ? b_bytes : 0u, 0x00020000);
        __amdgpu_buffer_rsrc_t as_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)p.as, 0, live ? as_bytes : 0u, 0x00020000);
        __amdgpu_buffer_rsrc_t bs_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)p.bs, 0, live ? bs_bytes : 0u, 0x00020000);
        const uint32_t a_k = kb * (uint32_t)KBLK * (uint32_t)p.lda, b_k = kb * (uint32_t)KBLK * (uint32_t)p.n;
        [&]<int... Q>(std::integer_sequence<int, Q...>) {
            ([&] {
                constexpr int I = 4 * Q + W;
                if constexpr (I < C::A_COPIES) copy16_global_to_lds(a_rsrc, st + I * 1024, voff[Q], a_k);
                else if constexpr (I < C::A_COPIES + C::B_COPIES) copy16_global_to_lds(b_rsrc, st + C::A_BYTES + (I - C::A_COPIES) * 1024, voff[Q], b_k);
                else if constexpr (I == C::A_COPIES + C::B_COPIES) copy4_global_to_lds(as_rsrc, st + C::A_BYTES + C::B_BYTES, voff[Q], kb * (uint32_t)p.lda * 4u);
                else copy4_global_to_lds(bs_rsrc, st + C::A_BYTES + C::B_BYTES + 256, voff[Q], kb * (uint32_t)p.nb * 4u);
            }(), ...);
        }(std::make_integer_sequence<int, C::COPIES>{});
    };

    // ---- LDS read addresses ----
    const int krow_lane = 8 * g + (i16 >> 1);
    const int swz_a = swz_of_krow<C::CPR_A>(krow_lane);
    const int swz_b = C::SWZ_B ? swz_of_krow<C::CPR_B>(krow_lane) : 0;
    const int a_lane_off = krow_lane * C::BM + (i16 & 1) * 8;
    const int b_lane_off = C::A_BYTES + krow_lane * C::BN + (i16 & 1) * 8;

    v4f acc[C::MT][C::NT_MAX];
#pragma unroll
    for (int t = 0; t < C::MT; t++)
#pragma unroll
        for (int x = 0; x < C::NT_MAX; x++) acc[t][x] = (v4f){0.f, 0.f, 0.f, 0.f};

    // rows of a that are not a multiple of four: see the tiled kernel
    const bool a_tail = TAILS && (p.lda & 3) != 0 && p.k > 0 && kb_end == kbt && nkb > 0;
    uint32_t acand0 = 0, acand1 = 0, acand2 = 0, a_last = 0;
    if (a_tail) {
        const uint32_t end = (uint32_t)p.k * (uint32_t)p.lda;
        acand0 = tail_candidate(end - 3, (uint32_t)p.lda, end, (uint32_t)p.k);
        acand1 = tail_candidate(end - 2, (uint32_t)p.lda, end, (uint32_t)p.k);
        acand2 = tail_candidate(end - 1, (uint32_t)p.lda, end, (uint32_t)p.k);
        a_last = load_last_dword(p.a + (end - 4));
    }
    acand0 = __builtin_amdgcn_readfirstlane(acand0); acand1 = __builtin_amdgcn_readfirstlane(acand1);
    acand2 = __builtin_amdgcn_readfirstlane(acand2); a_last = __builtin_amdgcn_readfirstlane(a_last);

    // The loop is instantiated once per wave index: which copies a wave issues and which n tiles it
    // multiplies then are compile-time facts, and the loop body has no branches.
    auto k_loop = [&](auto wave_tag) {
    constexpr int W = decltype(wave_tag)::value;
    // ---- prologue: NSTAGE-1 blocks in flight ----
    for (int b = 0; b < C::NSTAGE - 1; b++) issue_block(wave_tag, b);

    for (int j = 0; j < nkb; j++) {
        // the NSTAGE-2 blocks issued after block j may still be on their way
        wait_vmcnt<(C::NSTAGE - 2) * C::COPIES>();
        __syncthreads();      // block j complete in LDS; everyone is done with the stage of block j-1
        if constexpr (TAILS) {
            if (j == nkb - 1) {   // the last block of a has landed: its last bytes, then a second barrier
                unsigned char* st = lds + (j % C::NSTAGE) * C::STAGE_BYTES;
                patch_tail_bytes<C::BM, C::CPR_A>(st, st + C::STAGE_BYTES - 1, a_tail, m0, acand0, acand1, acand2, a_last, tid);
                __syncthreads();
            }
        }
        issue_block(wave_tag, j + C::NSTAGE - 1);

        const unsigned char* sbase = lds + (j % C::NSTAGE) * C::STAGE_BYTES;
        const unsigned char* sc = sbase + C::A_BYTES + C::B_BYTES;
        float asv[C::MT];
        v8i areg[C::MT];
#pragma unroll
        for (int t = 0; t < C::MT; t++) {
            if (t < MTV) {                               // m tiles beyond the matrix do no work
                asv[t] = *(const float*)(sc + (16 * t + i16) * 4);
                const unsigned char* q = sbase + a_lane_off + ((t ^ swz_a) << 4);
#pragma unroll
                for (int jj = 0; jj < 4; jj++) {
                    v2i x = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_V2I(q + jj * 32 * C::BM));
                    areg[t][2 * jj] = x[0]; areg[t][2 * jj + 1] = x[1];
                }
            }
        }
        [&]<int... X>(std::integer_sequence<int, X...>) {
            ([&] {
            constexpr int x = X, u = W + 4 * X;
            if constexpr (u < C::CPR_B) {
                v8i breg;
                const unsigned char* q = sbase + b_lane_off + ((u ^ swz_b) << 4);
#pragma unroll
                for (int jj = 0; jj < 4; jj++) {
                    v2i y = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_V2I(q + jj * 32 * C::BN));
                    breg[2 * jj] = y[0]; breg[2 * jj + 1] = y[1];
                }
                int bi = ((n0 + 16 * u) >> 7) - nb0;     // which of the staged b_scale values
                const float bsv = *(const float*)(sc + 256 + bi * 4);
#pragma unroll
                for (int t = 0; t < C::MT; t++) {
                    if (t < MTV) {
                        const v4f z = {0.f, 0.f, 0.f, 0.f};
                        v4f d = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(breg, areg[t], z, 0, 0, 0, 0, 0, 0);
                        const float s = asv[t] * bsv;
#pragma unroll
                        for (int r = 0; r < 4; r++) acc[t][x][r] = __builtin_fmaf(d[r], s, acc[t][x][r]);
                    }
                }
            }
            }(), ...);
        }(std::make_integer_sequence<int, C::NT_MAX>{});
    }
    };   // k_loop
    switch (wave) {
        case 0: k_loop(std::integral_constant<int, 0>{}); break;
        case 1: k_loop(std::integral_constant<int, 1>{}); break;
        case 2: k_loop(std::integral_constant<int, 2>{}); break;
        default: k_loop(std::integral_constant<int, 3>{}); break;
    }

    wait_vmcnt<0>();          // the trailing empty copies still target this workgroup's LDS

    // ---- epilogue ----
#pragma unroll
    for (int t = 0; t < C::MT; t++) {
        const int row = m0 + 16 * t + i16;
        if (row >= p.m) continue;
#pragma unroll
        for (int x = 0; x < C::NT_MAX; x++) {
            const int u = wave + 4 * x;
            const int col = n0 + 16 * u + 4 * g;
            if (u >= C::CPR_B || col >= p.n) continue;
            if (MODE == 1) {
                *(v4f*)(p.ws + ((size_t)split_z * p.m + row) * (size_t)p.n + col) = acc[t][x];
            } else {
                v2i o;
                o[0] = (int)pack_bf16x2(acc[t][x][0], acc[t][x][1]);
                o[1] = (int)pack_bf16x2(acc[t][x][2], acc[t][x][3]);
                *(v2i*)(p.c + (size_t)row * p.n + col) = o;
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// Split-K reduction: sums `split_k` fp32 planes in a fixed order and rounds to bf16, 8 outputs per
// thread with one 16-byte store (role of fp8_mm_128x128_ft2_split4_merge,
// 1-amd-fp8-mm/amd-fp8-mm-submission.py:485-511, for any split count).  The planes and c are walked as flat
// arrays of m*n elements, so the row length plays no part.  VEC: m*n is a multiple of 8 and c starts on a
// 16-byte boundary; otherwise the same sums, element by element, with the last group cut at m*n.
// ---------------------------------------------------------------------------------------------------
// SPLIT > 0: the number of planes is a compile-time fact, so all of a thread's loads are issued before the first add
// (with a run-time count the compiler keeps the loop and every plane's load waits for the previous plane's add: the
// kernel then takes one memory latency per plane); SPLIT == 0: any count.  The sum is taken in ascending order of
// the planes either way.
template <bool VEC, int SPLIT>
__global__ __launch_bounds__(256)
void splitk_reduce_kernel(const float* __restrict__ ws, uint16_t* __restrict__ c, size_t mn, int split_k) {
    size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 8;
    if (i >= mn) return;
    if constexpr (VEC) {
        v4f s0, s1;
        if constexpr (SPLIT > 0) {
            v4f p0[SPLIT], p1[SPLIT];
#pragma unroll
            for (int z = 0; z < SPLIT; z++) {
                p0[z] = __builtin_nontemporal_load((const v4f*)(ws + (size_t)z * mn + i));
                p1[z] = __builtin_nontemporal_load((const v4f*)(ws + (size_t)z * mn + i + 4));
            }
            s0 = p0[0]; s1 = p1[0];
#pragma unroll
            for (int z = 1; z < SPLIT; z++) { s0 += p0[z]; s1 += p1[z]; }
        } else {
            s0 = *(const v4f*)(ws + i); s1 = *(const v4f*)(ws + i + 4);
            for (int z = 1; z < split_k; z++) {
                s0 += *(const v4f*)(ws + (size_t)z * mn + i);
                s1 += *(const v4f*)(ws + (size_t)z * mn + i + 4);
            }
        }
        v4i o;
        o[0] = (int)pack_bf16x2(s0[0], s0[1]); o[1] = (int)pack_bf16x2(s0[2], s0[3]);
        o[2] = (int)pack_bf16x2(s1[0], s1[1]); o[3] = (int)pack_bf16x2(s1[2], s1[3]);
        *(v4i*)(c + i) = o;
    } else {
        const int cnt = mn - i < 8 ? (int)(mn - i) : 8;
        for (int j = 0; j < cnt; j++) {
            float s = ws[i + j];
            for (int z = 1; z < split_k; z++) s += ws[(size_t)z * mn + i + j];
            c[i + j] = (uint16_t)(pack_bf16x2(s, 0.f) & 0xFFFFu);
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// Generic kernel: any m, n (no alignment requirement), one output element per thread, scalar decode, fp32
// accumulation.  The planner uses it for K = 0 only (an empty sum: zeros); the parity tests use it, dense and
// grouped (row_offsets != nullptr), as the fp32-accurate HIP statement of the product.
// ---------------------------------------------------------------------------------------------------
__device__ __forceinline__ float e4m3fn_to_float(uint32_t v) {
    uint32_t s = (v & 0x80u) << 24, e = (v >> 3) & 15u, m = v & 7u;
    float f;
    if (e == 0) f = (float)m * 0.001953125f;                         // subnormal: m * 2^-9
    else if (e == 15 && m == 7) f = __builtin_nanf("");
    else f = __builtin_bit_cast(float, ((e + 120u) << 23) | (m << 20));
    return __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, f) | s);
}

__device__ __forceinline__ float generic_dot(const GemmArgs& p, const uint8_t* b, const float* bs, int row, int col) {
    float accum = 0.f;
    for (int kb = 0; kb < p.k / KBLK; kb++) {
        float part = 0.f;
        for (int kk = kb * KBLK; kk < (kb + 1) * KBLK; kk++)
            part = __builtin_fmaf(e4m3fn_to_float(p.a[(size_t)kk * p.lda + row]), e4m3fn_to_float(b[(size_t)kk * p.n + col]), part);
        accum = __builtin_fmaf(part, p.as[(size_t)kb * p.lda + row] * bs[(size_t)kb * p.nb + col / 128], accum);
    }
    return accum;
}

__global__ __launch_bounds__(256)
void gemm_generic_kernel(const GemmArgs p) {
    int col = blockIdx.x * 16 + (threadIdx.x & 15);            // output column (epi 1: pair index)
    int row = blockIdx.y * 16 + (threadIdx.x >> 4);
    const int ncols = p.epi == 1 ? p.n / 2 : p.n;
    if (row >= p.m || col >= ncols) return;
    const uint8_t* b = p.b;
    const float* bs = p.bs;
    if (p.row_offsets) {
        int e = 0;
        while (e + 1 < p.num_experts && row >= p.row_offsets[e + 1]) e++;
        b += (size_t)e * p.k * p.n;
        bs += (size_t)e * (p.k / KBLK) * p.nb;
    }
    float accum;
    if (p.epi == 1) {
        const float gate = generic_dot(p, b, bs, row, 2 * col), up = generic_dot(p, b, bs, row, 2 * col + 1);
        accum = gate / (1.0f + __expf(-gate)) * up;
    } else {
        accum = generic_dot(p, b, bs, row, col);
    }
    v2f f = {accum, 0.f};
    v2bf h = __builtin_convertvector(f, v2bf);
    p.c[(size_t)row * ncols + col] = __builtin_bit_cast(uint32_t, h) & 0xFFFFu;
}

template <int BN, int NSTAGE, int MODE, bool TAILS>
static void (*skinny_kernel_for(int mtv))(const GemmArgs) {
    if constexpr (BN == 144) {
        if (mtv == 1) return gemm_skinny_kernel<BN, NSTAGE, MODE, 1, TAILS>;
        if (mtv == 2) return gemm_skinny_kernel<BN, NSTAGE, MODE, 2, TAILS>;
        if (mtv == 3) return gemm_skinny_kernel<BN, NSTAGE, MODE, 3, TAILS>;
    }
    return gemm_skinny_kernel<BN, NSTAGE, MODE, 4, TAILS>;
}

template <int BN, int NSTAGE>
static hipError_t launch_skinny(const GemmArgs& a, int mode, hipStream_t stream) {
    if (mode == 2 || a.epi != 0) return hipErrorInvalidValue;
    using C = SkinnyCfg<BN, NSTAGE>;
    // m tiles with rows: fewer than 4 only for the planner's tile width and a matrix of at most 48 rows
    const int mtv = (BN == 144 && a.m <= 48) ? (a.m + 15) / 16 : 4;
    const bool tails = (a.lda & 3) != 0;      // the instantiation that repairs the last bytes of a: planner's tile width only
    void (*kern)(const GemmArgs) = mode == 1 ? skinny_kernel_for<BN, NSTAGE, 1, false>(mtv) : skinny_kernel_for<BN, NSTAGE, 0, false>(mtv);
    if (tails) {
        if constexpr (BN == 144) kern = mode == 1 ? skinny_kernel_for<BN, NSTAGE, 1, true>(mtv) : skinny_kernel_for<BN, NSTAGE, 0, true>(mtv);
        else return hipErrorInvalidValue;
    }
    static int raised[16][MAX_DEVICES];
    hipError_t e = raise_lds_limit((const void*)kern, C::LDS_BYTES, raised[(tails ? 8 : 0) + (mode == 1 ? 4 : 0) + mtv - 1]);
    if (e != hipSuccess) return e;
    int tiles = ((a.n + C::BN - 1) / C::BN) * a.split_k * ((a.m + C::BM - 1) / C::BM);
    hipLaunchKernelGGL(kern, dim3(tiles), dim3(C::NTHREADS), C::LDS_BYTES, stream, a);
    return hipGetLastError();
}

hipError_t launch_gemm(int variant, int mode, const GemmArgs& a, hipStream_t stream) {
    switch (variant) {
        case 1: {
            dim3 grid(((a.epi == 1 ? a.n / 2 : a.n) + 15) / 16, (a.m + 15) / 16);
            hipLaunchKernelGGL(gemm_generic_kernel, grid, dim3(256), 0, stream, a);
            return hipGetLastError();
        }
        case 2: return launch_tile_256x256(a, mode, stream);
        case 3: return launch_tile_128x128(a, mode, stream);
        case 4: return launch_tile_64x128(a, mode, stream);
        case 5: return launch_tile_256x128(a, mode, stream);
        case 6: return launch_skinny<144, 4>(a, mode, stream);
        case 7: return launch_skinny<256, 3>(a, mode, stream);
        case 8: return launch_skinny<288, 3>(a, mode, stream);
        case 9: return launch_tile_256x192(a, mode, stream);
        case 10: return launch_tile_256x128s3(a, mode, stream);
        case 11: return launch_tile_192x192s3(a, mode, stream);
        case 12: return launch_tile_64x256s3(a, mode, stream);
        default: return hipErrorInvalidValue;
    }
}

hipError_t launch_splitk_reduce(const float* ws, uint16_t* c, size_t mn, int split_k, hipStream_t stream) {
    size_t threads = (mn + 7) / 8;
    unsigned blocks = (unsigned)((threads + 255) / 256);
    if ((mn & 7) == 0 && ((uintptr_t)c & 15) == 0 && ((uintptr_t)ws & 15) == 0) {
        void (*kern)(const float*, uint16_t*, size_t, int) = splitk_reduce_kernel<true, 0>;
        switch (split_k) {
            case 2: kern = splitk_reduce_kernel<true, 2>; break;
            case 3: kern = splitk_reduce_kernel<true, 3>; break;
            case 4: kern = splitk_reduce_kernel<true, 4>; break;
            case 5: kern = splitk_reduce_kernel<true, 5>; break;
            case 6: kern = splitk_reduce_kernel<true, 6>; break;
            case 7: kern = splitk_reduce_kernel<true, 7>; break;
            case 8: kern = splitk_reduce_kernel<true, 8>; break;
            default: break;
        }
        hipLaunchKernelGGL(kern, dim3(blocks), dim3(256), 0, stream, ws, c, mn, split_k);
    } else {
        hipLaunchKernelGGL((splitk_reduce_kernel<false, 0>), dim3(blocks), dim3(256), 0, stream, ws, c, mn, split_k);
    }
    return hipGetLastError();
}

int variant_lds_bytes(int variant) {
    switch (variant) {
        case 2: return TileCfg<256, 256, 64, 128, 0>::LDS_BYTES;
        case 3: return TileCfg<128, 128, 64, 64, 0>::LDS_BYTES;
        case 4: return TileCfg<64, 128, 32, 64, 0>::LDS_BYTES;
        case 5: return TileCfg<256, 128, 64, 64, 0>::LDS_BYTES;
        case 6: return SkinnyCfg<144, 4>::LDS_BYTES;
        case 7: return SkinnyCfg<256, 3>::LDS_BYTES;
        case 8: return SkinnyCfg<288, 3>::LDS_BYTES;
        case 9: return TileCfg<256, 192, 64, 96, 0>::LDS_BYTES;
        case 10: return TileCfg<256, 128, 64, 64, 0, 3>::LDS_BYTES;
        case 11: return TileCfg<192, 192, 48, 96, 0, 3>::LDS_BYTES;
        case 12: return TileCfg<64, 256, 32, 64, 0, 3>::LDS_BYTES;
        default: return 0;
    }
}

}  // namespace fp8bs
