// Block quantisers that produce the operands of the FP8 block-scaled GEMM directly in its storage
// layout, for gfx950 (MI355X).
//
// The reference has no quantiser: its operands arrive quantised from the harness
// (1-amd-fp8-mm/0-amd-fp8-mm-new-begins.py:66-77 describes what arrives).  These kernels are the step
// in front of the GEMM, turning a row-major [rows][K] fp32 or bf16 matrix into
//   q      : e4m3fn, K rows of `rows` bytes      q[kk * rows + i]          (the layout of a and b,
//   scale  : fp32                                                           amd-fp8-mm-submission.py:66-75)
//     per row and 128-wide K block (activations, a_scale[(kk/128) * rows + i]), or
//     per 128x128 block           (weights,     b_scale[(kk/128) * NB + i/128], NB = ceil(rows/128)).
// Rule, bit for bit: scale = max(max|x| / 448, 1e-12) in fp32, q = round-to-nearest-even e4m3fn of
// clamp(x / scale, -448, 448) with a correctly rounded fp32 division.
//
// One workgroup = 128 rows x 128 k (one K block).  Every lane loads four k of four rows (16-byte
// loads along k, 32 lanes cover a row's block), the per-row maxima are reduced across those 32 lanes,
// the four rows' bytes are transposed 4x4 in registers (v_perm_b32) so that a dword holds four
// consecutive rows of one k, and the tile is staged in LDS ([128 k][128 rows], rows padded to 132
// bytes) so that the global stores are 16 bytes per lane, 128 contiguous bytes per k row.
// An optional row map gathers input rows (out row i = in row row_map[i]): the expert-contiguous
// permutation of MoE tokens (2-amd-moe/3-amd-fp8-moe-hip-myhgemm.py:174-191 does it as a copy of its
// own) then costs nothing extra.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

#include "fp8bs.h"
#include "fp8bs_kernels.h"

namespace fp8bs {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));

struct QuantArgs {
    const void* x;
    const int32_t* row_map;   // may be null
    uint8_t* q;
    float* scale;
    int64_t ldx;              // elements between input rows
    int rows, k, src_rows;    // output rows, K, rows of the input matrix (row_map targets)
    int nb;                   // per-block mode: ceil(rows/128)
};

static constexpr int TM = 128, TK = 128, LD = 132;   // LDS row pitch in bytes (33 dwords: spreads banks)

__device__ __forceinline__ v4f cvt4(v4i r, const float*) { return __builtin_bit_cast(v4f, r); }
__device__ __forceinline__ v4f cvt4(v2i r, const uint16_t*) {      // four bf16
    v4f o;
    o[0] = __builtin_bit_cast(float, (uint32_t)r[0] << 16);
    o[1] = __builtin_bit_cast(float, (uint32_t)r[0] & 0xFFFF0000u);
    o[2] = __builtin_bit_cast(float, (uint32_t)r[1] << 16);
    o[3] = __builtin_bit_cast(float, (uint32_t)r[1] & 0xFFFF0000u);
    return o;
}
// four k of one row; an offset of 0xFFFFFFFF is out of range for the buffer and reads zeros
__device__ __forceinline__ v4f load4(__amdgpu_buffer_rsrc_t rsrc, uint32_t byte_off, const float* tag) {
    return cvt4(__builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc, byte_off, 0, 0)), tag);
}
__device__ __forceinline__ v4f load4(__amdgpu_buffer_rsrc_t rsrc, uint32_t byte_off, const uint16_t* tag) {
    return cvt4(__builtin_bit_cast(v2i, __builtin_amdgcn_raw_buffer_load_b64(rsrc, byte_off, 0, 0)), tag);
}

// max over the 32 lanes that share a row, on the bit patterns of |x|: for non-negative floats the
// integer order is the float order, and every NaN pattern is above every number, so a NaN in the row
// comes out as the maximum (torch.amax propagates NaN the same way).  Steps 1, 2 (quad permutes), 4, 8
// (mirrors: all lanes of a reduced group already agree) are DPP modifiers, step 16 a swizzle.
__device__ __forceinline__ uint32_t umax(uint32_t a, uint32_t b) { return a > b ? a : b; }
__device__ __forceinline__ uint32_t rowmax32(uint32_t v) {
    v = umax(v, (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0xB1, 0xF, 0xF, true));    // quad_perm [1,0,3,2]
    v = umax(v, (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x4E, 0xF, 0xF, true));    // quad_perm [2,3,0,1]
    v = umax(v, (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x141, 0xF, 0xF, true));   // row_half_mirror
    v = umax(v, (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x140, 0xF, 0xF, true));   // row_mirror
    v = umax(v, (uint32_t)__builtin_amdgcn_ds_swizzle((int)v, 0x401F));               // lane ^ 16
    return v;
}

// Correctly rounded x / s for finite s >= 1e-12 and |x / s| < 2^96: the arithmetic of the IEEE
// division sequence (reciprocal refined once, quotient corrected twice, all by fused multiply-add)
// without its range scaling, which only acts on quotients or operands at the ends of the exponent
// range; there the result is a zero after conversion to e4m3fn either way.  `y` is refine_rcp(s).
__device__ __forceinline__ float refine_rcp(float s) {
    float y = __builtin_amdgcn_rcpf(s);
    float e = __builtin_fmaf(-s, y, 1.0f);
    return __builtin_fmaf(e, y, y);
}
__device__ __forceinline__ float div_by(float x, float s, float y) {
    float q = x * y;
    float r = __builtin_fmaf(-s, q, x);
    q = __builtin_fmaf(r, y, q);
    r = __builtin_fmaf(-s, q, x);
    q = __builtin_fmaf(r, y, q);
    return __builtin_copysignf(q, x);          // keeps -0 (the residuals above turn it into +0)
}
// scale of a block from the bit pattern of its max |x|
__device__ __forceinline__ float scale_of(uint32_t amax_bits) {
    const float amax = __builtin_bit_cast(float, amax_bits);
    float s = div_by(amax, 448.f, refine_rcp(448.f));
    s = s < 1e-12f ? 1e-12f : s;
    return amax_bits >= 0x7F800000u ? amax : s;            // inf stays inf, NaN stays NaN
}

__device__ __forceinline__ float clamp448(float v) {
    // NaN stays NaN (becomes the e4m3fn NaN code), like clamp_ followed by the cast in torch
    return v != v ? v : __builtin_fminf(__builtin_fmaxf(v, -448.f), 448.f);
}

// four fp32 -> four e4m3fn codes in one dword (byte j = value j), round to nearest even
__device__ __forceinline__ uint32_t cvt4_e4m3fn(v4f v) {
    int w = __builtin_amdgcn_cvt_pk_fp8_f32(v[0], v[1], 0, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(v[2], v[3], w, true);
    return (uint32_t)w;
}

// PER_BLOCK false: one scale per row and K block (activations); true: one per 128x128 block (weights)
template <typename T, bool PER_BLOCK, bool HAS_MAP>
__global__ __launch_bounds__(256)
void quantize_kernel(const QuantArgs p) {
    __shared__ __attribute__((aligned(16))) unsigned char tile[TK * LD];
    __shared__ float row_scale[TM];
    __shared__ uint32_t wave_max[4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int g = lane >> 5, l = lane & 31;
    const int kb = blockIdx.x, m0 = blockIdx.y * TM;
    __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void*)p.x, 0, (uint32_t)((size_t)p.src_rows * (size_t)p.ldx * sizeof(T)), 0x00020000);

    // ---- load: iteration it, row group rg = it*8 + wave*2 + g holds rows 4rg .. 4rg+3 ----
    v4f v[4][4];
    uint32_t rmax[4][4];
    const uint32_t col_off = (uint32_t)((kb * TK + 4 * l) * sizeof(T));
    const uint32_t row_pitch = (uint32_t)(p.ldx * sizeof(T));
    int src[4][4];
    // all row-map entries first, then all data loads: neither waits for the other one by one
#pragma unroll
    for (int it = 0; it < 4; it++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int row = m0 + 4 * (it * 8 + wave * 2 + g) + r;
            if (HAS_MAP) src[it][r] = p.row_map[row < p.rows ? row : p.rows - 1];
            else src[it][r] = row;
        }
#pragma unroll
    for (int it = 0; it < 4; it++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int row = m0 + 4 * (it * 8 + wave * 2 + g) + r;
            const bool ok = row < p.rows && (uint32_t)src[it][r] < (uint32_t)p.src_rows;
            const uint32_t off = ok ? (uint32_t)src[it][r] * row_pitch + col_off : 0xFFFFFFFFu;
            v[it][r] = load4(rsrc, off, (const T*)nullptr);
        }
    // ---- per-row max |x| ----
#pragma unroll
    for (int it = 0; it < 4; it++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const v4i b = __builtin_bit_cast(v4i, v[it][r]) & 0x7FFFFFFF;
            rmax[it][r] = rowmax32(umax(umax((uint32_t)b[0], (uint32_t)b[1]), umax((uint32_t)b[2], (uint32_t)b[3])));
        }
    float bscale = 0.f;
    if (PER_BLOCK) {
        uint32_t mx = 0;
#pragma unroll
        for (int it = 0; it < 4; it++)
#pragma unroll
            for (int r = 0; r < 4; r++) mx = umax(mx, rmax[it][r]);
        mx = umax(mx, (uint32_t)__shfl_xor((int)mx, 32, 64));
        if (lane == 0) wave_max[wave] = mx;
        __syncthreads();
        bscale = scale_of(umax(umax(wave_max[0], wave_max[1]), umax(wave_max[2], wave_max[3])));
        if (tid == 0) p.scale[(size_t)kb * p.nb + blockIdx.y] = bscale;
    }
    // ---- quantise, transpose 4x4 bytes, stage in LDS ----
    const float bscale_rcp = refine_rcp(bscale);
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const int rg = it * 8 + wave * 2 + g;
        uint32_t rw[4];
#pragma unroll
        for (int r = 0; r < 4; r++) {
            float s, y;
            if (PER_BLOCK) { s = bscale; y = bscale_rcp; }
            else {
                s = scale_of(rmax[it][r]);
                y = refine_rcp(s);
                if (l == 0) row_scale[4 * rg + r] = s;
            }
            const v4f a = v[it][r];
            v4f qf;
            if (__builtin_expect(__builtin_bit_cast(uint32_t, s) >= 0x7F800000u, 0)) {
                // an inf or NaN in the block: the plain division has the IEEE special cases
#pragma unroll
                for (int j = 0; j < 4; j++) qf[j] = clamp448(a[j] / s);
            } else {
#pragma unroll
                for (int j = 0; j < 4; j++) qf[j] = __builtin_amdgcn_fmed3f(div_by(a[j], s, y), -448.f, 448.f);
            }
            rw[r] = cvt4_e4m3fn(qf);
        }
        // rw[r] = bytes (k0..k3) of row r  ->  c[j] = bytes (row0..row3) of k j
        const uint32_t lo01 = __builtin_amdgcn_perm(rw[1], rw[0], 0x05010400u), hi01 = __builtin_amdgcn_perm(rw[1], rw[0], 0x07030602u);
        const uint32_t lo23 = __builtin_amdgcn_perm(rw[3], rw[2], 0x05010400u), hi23 = __builtin_amdgcn_perm(rw[3], rw[2], 0x07030602u);
        const uint32_t c0 = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u), c1 = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
        const uint32_t c2 = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u), c3 = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
        unsigned char* t = tile + (4 * l) * LD + 4 * rg;
        *(uint32_t*)(t) = c0;
        *(uint32_t*)(t + LD) = c1;
        *(uint32_t*)(t + 2 * LD) = c2;
        *(uint32_t*)(t + 3 * LD) = c3;
    }
    __syncthreads();
    // ---- scales of the 128 rows: 512 contiguous bytes ----
    if (!PER_BLOCK && tid < TM && m0 + tid < p.rows) p.scale[(size_t)kb * p.rows + m0 + tid] = row_scale[tid];
    // ---- store: 1024 chunks of 16 rows x 1 k, 4 per thread; 8 consecutive lanes write one k row ----
    const bool wide = (p.rows & 15) == 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int id = i * 256 + tid;
        const int krow = id >> 3, c = id & 7;
        const unsigned char* s = tile + krow * LD + 16 * c;
        const int row = m0 + 16 * c;
        if (row >= p.rows) continue;
        uint8_t* dst = p.q + ((size_t)kb * TK + krow) * (size_t)p.rows + row;
        const uint32_t w0 = *(const uint32_t*)s, w1 = *(const uint32_t*)(s + 4), w2 = *(const uint32_t*)(s + 8), w3 = *(const uint32_t*)(s + 12);
        if (wide) {
            *(v4i*)dst = (v4i){(int)w0, (int)w1, (int)w2, (int)w3};
        } else {
            const uint32_t w[4] = {w0, w1, w2, w3};
            for (int b = 0; b < 16 && row + b < p.rows; b++) dst[b] = (uint8_t)(w[b >> 2] >> (8 * (b & 3)));
        }
    }
}

template <typename T, bool PER_BLOCK>
static hipError_t launch_quant(const QuantArgs& a, hipStream_t stream) {
    dim3 grid((unsigned)(a.k / TK), (unsigned)((a.rows + TM - 1) / TM));
    if (a.row_map) hipLaunchKernelGGL((quantize_kernel<T, PER_BLOCK, true>), grid, dim3(256), 0, stream, a);
    else hipLaunchKernelGGL((quantize_kernel<T, PER_BLOCK, false>), grid, dim3(256), 0, stream, a);
    return hipGetLastError();
}

// e4m3fnuz (gfx942: bias 8, max 240, NaN = 0x80, no -0) -> e4m3fn (bias 7) with the same value.
// Normal fnuz codes with exponent field >= 2 are the fn code with the exponent field one lower, exactly.
// The 16 smallest magnitudes (fnuz subnormals and exponent field 1, steps of 2^-10) fall on fn's
// subnormal grid of 2^-9: magnitude code x becomes x/2 rounded to nearest even.  16 bytes per thread.
__device__ __forceinline__ uint32_t fnuz_to_fn_byte(uint32_t b) {
    const uint32_t mag = b & 0x7Fu;
    const uint32_t out = mag >= 16u ? mag - 8u : (mag + ((mag >> 1) & 1u)) >> 1;
    return b == 0x80u ? 0x7Fu : ((b & 0x80u) | out);
}
__global__ __launch_bounds__(256)
void fnuz_to_fn_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, size_t n) {
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 16;
    if (i + 16 <= n) {
        const v4i v = *(const v4i*)(src + i);
        v4i o;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const uint32_t x = (uint32_t)v[w];
            o[w] = (int)(fnuz_to_fn_byte(x & 0xFFu) | (fnuz_to_fn_byte((x >> 8) & 0xFFu) << 8) |
                         (fnuz_to_fn_byte((x >> 16) & 0xFFu) << 16) | (fnuz_to_fn_byte(x >> 24) << 24));
        }
        *(v4i*)(dst + i) = o;
    } else {
        for (size_t j = i; j < n; j++) dst[j] = (uint8_t)fnuz_to_fn_byte(src[j]);
    }
}


// ---------------------------------------------------------------------------------------------------
// Row gather of an already quantised activation matrix: out row i = source row row_map[i], bytes and
// scales, in the K-major storage layout (a[kk * rows + i]).  With top-k routing every token appears
// top-k times in the expert-contiguous order (2-amd-moe/3-amd-fp8-moe-hip-myhgemm.py:174-191 copies
// rows the same way); quantising the tokens once and gathering bytes costs an eighth of the arithmetic
// of quantising every copy.
//
// In this layout the gather runs along the contiguous dimension (one byte per row), so it goes through
// LDS: a workgroup takes KC consecutive k rows of the source (KC * src_rows bytes), transposes them in
// registers (v_perm_b32, 4x4 bytes) to token-major order - LDS slot of token t holds its KC bytes - and
// then every lane produces four consecutive output rows: one LDS read of KC bytes per row, the
// transpose back, and KC dword stores (a wave writes 256 contiguous bytes of one k row per store).
// Slot of token t is (t % 4) * ceil(src_rows / 4) + t / 4, which makes the LDS writes of phase 1
// contiguous across lanes.
// ---------------------------------------------------------------------------------------------------
struct GatherArgs {
    const uint8_t* src;       // [k][src_rows]
    const float* src_scale;   // [k/128][src_rows]
    const int32_t* row_map;   // [rows]
    uint8_t* dst;             // [k][rows]
    float* dst_scale;         // [k/128][rows]
    int rows, k, src_rows;
    int rows_per_wg;          // multiple of 4
};

// rw[r] = bytes (c0..c3) of line r  ->  out[j] = bytes (line0..line3) of column j
__device__ __forceinline__ void transpose4x4(const uint32_t rw[4], uint32_t out[4]) {
    const uint32_t lo01 = __builtin_amdgcn_perm(rw[1], rw[0], 0x05010400u), hi01 = __builtin_amdgcn_perm(rw[1], rw[0], 0x07030602u);
    const uint32_t lo23 = __builtin_amdgcn_perm(rw[3], rw[2], 0x05010400u), hi23 = __builtin_amdgcn_perm(rw[3], rw[2], 0x07030602u);
    out[0] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u); out[1] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
    out[2] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u); out[3] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
}

template <int KC>
__global__ __launch_bounds__(256)
void gather_a_kernel(const GatherArgs p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char slots[];     // [4 * quarter][KC]
    constexpr int KG = KC / 4;
    const int tid = threadIdx.x;
    const int k0 = blockIdx.x * KC;
    const int quarter = (p.src_rows + 3) / 4;
    // ---- phase 1: KC source rows -> token-major slots ----
    __amdgpu_buffer_rsrc_t src_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)p.src, 0, (uint32_t)p.k * (uint32_t)p.src_rows, 0x00020000);
    for (int task = tid; task < quarter; task += 256) {
        uint32_t tok[4][KG];                       // tok[j][kg]: bytes (k rows 4kg..4kg+3) of token 4*task + j
#pragma unroll
        for (int kg = 0; kg < KG; kg++) {
            uint32_t rw[4], c[4];
#pragma unroll
            for (int r = 0; r < 4; r++)
                rw[r] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(src_rsrc, (uint32_t)(k0 + 4 * kg + r) * (uint32_t)p.src_rows + 4u * (uint32_t)task, 0, 0);
            transpose4x4(rw, c);
#pragma unroll
            for (int j = 0; j < 4; j++) tok[j][kg] = c[j];
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            unsigned char* d = slots + (size_t)(j * quarter + task) * KC;
#pragma unroll
            for (int kg = 0; kg < KG; kg++) *(uint32_t*)(d + 4 * kg) = tok[j][kg];
        }
    }
    __syncthreads();
    // ---- phase 2: four consecutive output rows per lane ----
    const int row_begin = blockIdx.y * p.rows_per_wg;
    int row_end = row_begin + p.rows_per_wg;
    row_end = row_end < p.rows ? row_end : p.rows;
    for (int i0 = row_begin + 4 * tid; i0 < row_end; i0 += 1024) {
        const v4i map = *(const v4i*)(p.row_map + i0);
        uint32_t tok[4][KG];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t t = (uint32_t)map[j];
            const bool ok = t < (uint32_t)p.src_rows;
            const unsigned char* sp = slots + (size_t)((t & 3u) * (uint32_t)quarter + (t >> 2)) * KC;
#pragma unroll
            for (int kg = 0; kg < KG; kg++) tok[j][kg] = ok ? *(const uint32_t*)(sp + 4 * kg) : 0u;
        }
#pragma unroll
        for (int kg = 0; kg < KG; kg++) {
            uint32_t rw[4], c[4];
#pragma unroll
            for (int j = 0; j < 4; j++) rw[j] = tok[j][kg];
            transpose4x4(rw, c);                   // c[r] = bytes (rows i0..i0+3) of k row 4kg + r
#pragma unroll
            for (int r = 0; r < 4; r++)
                __builtin_nontemporal_store(c[r], (uint32_t*)(p.dst + (size_t)(k0 + 4 * kg + r) * (size_t)p.rows + i0));
        }
        // the scales of a K block travel with its first k rows
        if ((k0 & 127) == 0) {
            v4f sc;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint32_t t = (uint32_t)map[j];
                sc[j] = t < (uint32_t)p.src_rows ? p.src_scale[(size_t)(k0 >> 7) * p.src_rows + t] : 1e-12f;
            }
            *(v4f*)(p.dst_scale + (size_t)(k0 >> 7) * p.rows + i0) = sc;
        }
    }
}

// any alignment, any size: one output byte per thread
__global__ __launch_bounds__(256)
void gather_a_bytes_kernel(const GatherArgs p) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= p.rows) return;
    const uint32_t t = (uint32_t)p.row_map[i];
    const bool ok = t < (uint32_t)p.src_rows;
    for (int kk = blockIdx.y; kk < p.k; kk += gridDim.y) {
        p.dst[(size_t)kk * p.rows + i] = ok ? p.src[(size_t)kk * p.src_rows + t] : (uint8_t)0;
        if ((kk & 127) == 0) p.dst_scale[(size_t)(kk >> 7) * p.rows + i] = ok ? p.src_scale[(size_t)(kk >> 7) * p.src_rows + t] : 1e-12f;
    }
}

template <int KC>
static hipError_t launch_gather(const GatherArgs& a, hipStream_t stream) {
    const int quarter = (a.src_rows + 3) / 4;
    const int lds = 4 * quarter * KC;
    auto kern = gather_a_kernel<KC>;
    static int raised[MAX_DEVICES];
    if (lds > 65536) {
        hipError_t e = raise_lds_limit((const void*)kern, lds, raised);
        if (e != hipSuccess) return e;
    }
    dim3 grid((unsigned)(a.k / KC), (unsigned)((a.rows + a.rows_per_wg - 1) / a.rows_per_wg));
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, a);
    return hipGetLastError();
}

}  // namespace fp8bs

extern "C" int fp8bs_convert_fnuz_to_fn(const void* src, void* dst, size_t nbytes, void* stream) {
    if (nbytes == 0) return FP8BS_OK;
    if (!src || !dst) return FP8BS_ERR_NULL_POINTER;
    if ((((uintptr_t)src | (uintptr_t)dst) & 15) != 0) return FP8BS_ERR_BAD_SHAPE;
    const size_t threads = (nbytes + 15) / 16;
    hipLaunchKernelGGL(fp8bs::fnuz_to_fn_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const uint8_t*)src, (uint8_t*)dst, nbytes);
    return hipGetLastError() == hipSuccess ? FP8BS_OK : FP8BS_ERR_LAUNCH;
}

namespace {
int quantize_common(const void* x, int dtype, int64_t ldx, const int32_t* row_map, int src_rows, void* q, float* scale,
                    int rows, int k, bool per_block, void* stream) {
    if (rows < 0 || k < 0 || (k % 128) != 0) return FP8BS_ERR_BAD_SHAPE;
    if (dtype != FP8BS_DTYPE_F32 && dtype != FP8BS_DTYPE_BF16) return FP8BS_ERR_BAD_SHAPE;
    if (rows == 0 || k == 0) return FP8BS_OK;
    if (!x || !q || !scale) return FP8BS_ERR_NULL_POINTER;
    if (ldx < k) return FP8BS_ERR_BAD_SHAPE;
    // 16-byte loads along k: rows must start on a 16-byte boundary
    const int64_t esz = dtype == FP8BS_DTYPE_F32 ? 4 : 2;
    if (((uintptr_t)x & 15) != 0 || ((ldx * esz) & (dtype == FP8BS_DTYPE_F32 ? 15 : 7)) != 0) return FP8BS_ERR_BAD_SHAPE;
    if ((size_t)rows * (size_t)k > 0xFFFFFFFFull) return FP8BS_ERR_TOO_LARGE;
    if ((size_t)(row_map ? src_rows : rows) * (size_t)ldx * (size_t)esz > 0xFFFFFFFFull) return FP8BS_ERR_TOO_LARGE;   // buffer addressing
    fp8bs::QuantArgs a{x, row_map, (uint8_t*)q, scale, ldx, rows, k, row_map ? src_rows : rows, (rows + 127) / 128};
    hipStream_t s = (hipStream_t)stream;
    hipError_t e;
    if (dtype == FP8BS_DTYPE_F32) e = per_block ? fp8bs::launch_quant<float, true>(a, s) : fp8bs::launch_quant<float, false>(a, s);
    else e = per_block ? fp8bs::launch_quant<uint16_t, true>(a, s) : fp8bs::launch_quant<uint16_t, false>(a, s);
    return e == hipSuccess ? FP8BS_OK : FP8BS_ERR_LAUNCH;
}
}  // namespace

extern "C" int fp8bs_quantize_a(const void* x, int x_dtype, int64_t ldx, const int32_t* row_map, int src_rows,
                                void* a, float* a_scale, int m, int k, void* stream) {
    return quantize_common(x, x_dtype, ldx, row_map, src_rows, a, a_scale, m, k, false, stream);
}

extern "C" int fp8bs_quantize_b(const void* w, int w_dtype, int64_t ldw, void* b, float* b_scale, int n, int k, void* stream) {
    return quantize_common(w, w_dtype, ldw, nullptr, 0, b, b_scale, n, k, true, stream);
}

extern "C" int fp8bs_gather_a(const void* a_src, const float* a_scale_src, int src_rows, const int32_t* row_map,
                              void* a, float* a_scale, int m, int k, void* stream) {
    if (m < 0 || k < 0 || src_rows < 0 || (k % 128) != 0) return FP8BS_ERR_BAD_SHAPE;
    if (m == 0 || k == 0) return FP8BS_OK;
    if (!row_map || !a || !a_scale || (src_rows > 0 && (!a_src || !a_scale_src))) return FP8BS_ERR_NULL_POINTER;
    if ((size_t)src_rows * (size_t)k > 0xFFFFFFFFull) return FP8BS_ERR_TOO_LARGE;       // buffer addressing
    fp8bs::GatherArgs g{(const uint8_t*)a_src, a_scale_src, row_map, (uint8_t*)a, a_scale, m, k, src_rows, 8192};
    hipStream_t s = (hipStream_t)stream;
    // dword loads of source rows, dword stores of output rows, 16-byte loads of the map and stores of
    // the scales: everything must sit on those boundaries, and the KC source rows must fit the LDS
    const bool aligned = (src_rows % 4) == 0 && (m % 4) == 0 && src_rows > 0 &&
                         ((((uintptr_t)a_src | (uintptr_t)a) & 3) == 0) && ((((uintptr_t)row_map | (uintptr_t)a_scale) & 15) == 0);
    hipError_t e;
    if (aligned && src_rows <= 4096) e = fp8bs::launch_gather<16>(g, s);
    else if (aligned && src_rows <= 8192) e = fp8bs::launch_gather<8>(g, s);
    else if (aligned && src_rows <= 40960) e = fp8bs::launch_gather<4>(g, s);
    else {
        hipLaunchKernelGGL(fp8bs::gather_a_bytes_kernel, dim3((unsigned)((m + 255) / 256), (unsigned)(k < 4096 ? k : 4096)), dim3(256), 0, s, g);
        e = hipGetLastError();
    }
    return e == hipSuccess ? FP8BS_OK : FP8BS_ERR_LAUNCH;
}
