// Measurement aid, not part of the GEMM path: the instruction mix of one K block of the 256x256 tile's wave
// (32 v_mfma_f32_16x16x128_f8f6f4 on random operands) in a register-only loop, to which the other parts of
// the real K block can be added one by one - the scale fold (4 v_fma per MFMA), the transposing LDS reads
// (48 ds_read_b64_tr_b8 per 32 MFMAs) and the global->LDS copies (8 one-KiB copies per wave per 32 MFMAs) -
// with no barriers, no waits for the copies and no output.  Timing it on one workgroup and on a full grid
// separates what the instruction mix costs from what the schedule of the real kernel adds, and what the
// chip's power management takes (bench.py --mfma-ceiling).  The reference has nothing comparable.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

#include "fp8bs.h"
#include "fp8bs_tiled.h"

namespace {

using fp8bs::v8i;
using fp8bs::v2i;
using fp8bs::v4f;
#define DIAG_LDS_V2I(p) ((__attribute__((address_space(3))) v2i*)(p))

constexpr int DIAG_LDS_BYTES = 128 * 1024;      // 64 KiB read by the transposing reads, 64 KiB filled by the copies

// src: at least 64 KiB of e4m3fn codes (no NaN codes) followed by whatever the copies walk; src_mask + 1 = bytes walked
// M32: the same multiply-accumulates as 16 v_mfma_f32_32x32x64_f8f6f4 (64 clocks each, half the operand
// register reads per multiply-accumulate) instead of 32 v_mfma_f32_16x16x128_f8f6f4
// SPREAD: the LDS reads spread evenly over the K block - one B read per step, and one A read per two steps into a
// second set of A registers (32 more VGPRs than the GEMM's wave has left) - instead of the GEMM's pattern: the next n
// tile's B operand as 4 reads every 4 steps, the next block's 4 A operands as 16 reads behind the last 4 MFMAs
// The loop body is two K blocks (one per LDS stage), so that every LDS address is an immediate offset.
template <int FOLD, int LDSR, int DMA, int M32, int SPREAD>
__global__ __launch_bounds__(512) void mfma_mix_kernel(int iters, const unsigned char* src, size_t src_mask, float* sink) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
    const int t = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(t >> 6), lane = t & 63;
    const int* in = (const int*)src;
    for (int i = t; i < 16384; i += 512) ((int*)smem)[i] = in[i];
    __syncthreads();
    v8i a[2][4], b[2];
    for (int h = 0; h < 2; h++) for (int j = 0; j < 4; j++) for (int i = 0; i < 8; i++) a[h][j][i] = in[(t * 8 + i + j * 131 + h * 7) & 4095];
    for (int j = 0; j < 2; j++) for (int i = 0; i < 8; i++) b[j][i] = in[(t * 8 + i + 77 + j * 57) & 4095];
    constexpr int NACC = 32;
    v4f acc[NACC];
    for (int i = 0; i < NACC; i++) acc[i] = (v4f){0, 0, 0, 0};
    const float sc = __builtin_bit_cast(float, in[t & 4095]) * 1e-30f + 1.0f;
    v4f ring[4];
    for (int i = 0; i < 4; i++) ring[i] = (v4f){0, 0, 0, 0};
    const v4f z = {0, 0, 0, 0};
    typedef float v16f __attribute__((ext_vector_type(16)));
    v16f ring32[2];
    for (int i = 0; i < 2; i++) for (int r = 0; r < 16; r++) ring32[i][r] = 0.f;
    v16f z32;
    for (int r = 0; r < 16; r++) z32[r] = 0.f;
    // the 256-wide tile's [k][m] layout and XOR swizzle: lane reads k row 8*(lane/16) + (lane%16)/2, byte half lane%2
    const int krow = 8 * (lane >> 4) + ((lane & 15) >> 1);
    const unsigned char* rbase = smem + krow * 256 + (lane & 1) * 8;
    // the 8 workgroups that an XCD runs side by side in a tile row share one stream of copies (an A panel)
    // (issued like the GEMM's, from inline assembly: the compiler would make every LDS read wait for all copies in flight)
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)src, 0, (uint32_t)src_mask + 1u, 0x00020000);
    const uint32_t lds_copy_base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char*)smem + 65536 + wave * 8192;
    uint32_t goff = 65536 + (uint32_t)((blockIdx.x % 8) * 4 + (blockIdx.x / 8) % 4) * 65536u + wave * 8192;
    // one K block; H: the LDS stage it reads and the A register set it multiplies (the other set is filled)
    auto block = [&](auto h_tag) {
        constexpr int H = decltype(h_tag)::value;
#pragma unroll
        for (int s = 0; s < 32; s++) {
            if (LDSR && !SPREAD && (s & 3) == 0) {
                // the B operand of the next n tile: 4 reads of 8 k rows each, 32 k rows apart
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    v2i v = __builtin_amdgcn_ds_read_tr8_b64_v2i32(DIAG_LDS_V2I(rbase + ((((wave + (s >> 2)) & 15) ^ (krow & 15)) << 4) + j * 8192 + H * 32768));
                    b[((s >> 2) + 1) & 1][2 * j] = v[0]; b[((s >> 2) + 1) & 1][2 * j + 1] = v[1];
                }
            }
            if (LDSR && !SPREAD && s >= 28) {
                // the A operands of the next K block, behind the last MFMAs of this one
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    v2i v = __builtin_amdgcn_ds_read_tr8_b64_v2i32(DIAG_LDS_V2I(rbase + ((((wave >> 1) * 4 + (s & 3)) ^ (krow & 15)) << 4) + j * 8192 + (1 - H) * 32768));
                    a[1 - H][s & 3][2 * j] = v[0]; a[1 - H][s & 3][2 * j + 1] = v[1];
                }
            }
            if (LDSR && SPREAD) {
                const int j = s & 3;
                v2i v = __builtin_amdgcn_ds_read_tr8_b64_v2i32(DIAG_LDS_V2I(rbase + ((((wave + (s >> 2)) & 15) ^ (krow & 15)) << 4) + j * 8192 + H * 32768));
                b[((s >> 2) + 1) & 1][2 * j] = v[0]; b[((s >> 2) + 1) & 1][2 * j + 1] = v[1];
                if ((s & 1) == 0) {
                    const int ja = (s >> 1) & 3, ta = s >> 3;
                    v2i w = __builtin_amdgcn_ds_read_tr8_b64_v2i32(DIAG_LDS_V2I(rbase + ((((wave >> 1) * 4 + ta) ^ (krow & 15)) << 4) + ja * 8192 + (1 - H) * 32768));
                    a[1 - H][ta][2 * ja] = w[0]; a[1 - H][ta][2 * ja + 1] = w[1];
                }
            }
            if (DMA && (s & 3) == 0) {
                fp8bs::copy16_global_to_lds(rsrc, lds_copy_base + (s >> 2) * 1024, lane * 16, __builtin_amdgcn_readfirstlane(goff & (uint32_t)src_mask));
                goff += 1024;
            }
            if (!LDSR && (s & 3) == 0) b[((s >> 2) + 1) & 1][(s >> 2) & 7] += 0x01010101;   // operands change from step to step
            constexpr int HA = LDSR ? H : 0;                   // without LDS reads there is one A set
            if (M32) {
                if ((s & 1) == 0) ring32[(s >> 1) & 1] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b[(s >> 2) & 1], a[HA][s & 3], z32, 0, 0, 0, 0, 0, 0);
                if (FOLD) {
                    // half of the previous instruction's sixteen results per step
#pragma unroll
                    for (int r = 0; r < 8; r++) acc[(2 * s + r / 4) % NACC][r & 3] = __builtin_fmaf(ring32[((s >> 1) + 1) & 1][(s & 1) * 8 + r], sc, acc[(2 * s + r / 4) % NACC][r & 3]);
                } else if ((s & 1) == 0) {
                    asm volatile("" :: "v"(ring32[(s >> 1) & 1]));
                }
                __builtin_amdgcn_sched_barrier(0);
                continue;
            }
            ring[s & 3] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b[(s >> 2) & 1], a[HA][s & 3], z, 0, 0, 0, 0, 0, 0);
            if (FOLD) {
                const v4f p = ring[(s + 1) & 3];          // the result of three steps ago
#pragma unroll
                for (int r = 0; r < 4; r++) acc[s % NACC][r] = __builtin_fmaf(p[r], sc, acc[s % NACC][r]);
            } else {
                asm volatile("" :: "v"(ring[s & 3]));
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (DMA) goff += 32u * 65536u - 8192u;           // next K block of the stream
    };
    for (int it = 0; it < iters; it += 2) {
        block(std::integral_constant<int, 0>{});
        block(std::integral_constant<int, 1>{});
    }
    if (DMA) __builtin_amdgcn_s_waitcnt(0x0F70);          // vmcnt(0): the copies target this workgroup's LDS
    float s = 0;
    for (int i = 0; i < 4; i++) s += ring[i][0];
    for (int i = 0; i < 2; i++) s += ring32[i][0] + ring32[i][9];
    for (int h = 0; h < 2; h++) for (int j = 0; j < 4; j++) s += __builtin_bit_cast(float, a[h][j][0]) * 0.f;
    for (int i = 0; i < NACC; i++) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
    if (s == 1.2345f) sink[0] = s;
}

template <int FOLD, int LDSR, int DMA, int M32 = 0, int SPREAD = 0>
hipError_t launch_mix(int workgroups, int iters, const unsigned char* src, size_t src_mask, float* sink, hipStream_t stream) {
    static int raised[fp8bs::MAX_DEVICES];
    hipError_t e = fp8bs::raise_lds_limit((const void*)mfma_mix_kernel<FOLD, LDSR, DMA, M32, SPREAD>, DIAG_LDS_BYTES, raised);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((mfma_mix_kernel<FOLD, LDSR, DMA, M32, SPREAD>), dim3(workgroups), dim3(512), DIAG_LDS_BYTES, stream, iters, src, src_mask, sink);
    return hipGetLastError();
}

}  // namespace

extern "C" int fp8bs_diag_mfma_mix(int mix, int workgroups, int iters, const void* src, size_t src_bytes, void* sink, void* stream) {
    if (!src || !sink) return FP8BS_ERR_NULL_POINTER;
    if (workgroups <= 0 || iters < 0 || (iters & 1) != 0 || mix < 0 || mix > 23 || (mix >= 16 && (mix & 2) == 0)) return FP8BS_ERR_BAD_SHAPE;
    // the walked range is a power of two of at least 4 MiB (the 32 streams of one pass are 64 KiB apart, 2 MiB each way)
    if (src_bytes < (4u << 20) || src_bytes > (1u << 31) || (src_bytes & (src_bytes - 1)) != 0 || ((uintptr_t)src & 15) != 0) return FP8BS_ERR_BAD_SHAPE;
    const unsigned char* p = (const unsigned char*)src;
    const size_t mask = src_bytes - 1;
    float* sk = (float*)sink;
    hipStream_t s = (hipStream_t)stream;
    hipError_t e;
    switch (mix) {
        case 0: e = launch_mix<0, 0, 0>(workgroups, iters, p, mask, sk, s); break;
        case 1: e = launch_mix<1, 0, 0>(workgroups, iters, p, mask, sk, s); break;
        case 2: e = launch_mix<0, 1, 0>(workgroups, iters, p, mask, sk, s); break;
        case 3: e = launch_mix<1, 1, 0>(workgroups, iters, p, mask, sk, s); break;
        case 4: e = launch_mix<0, 0, 1>(workgroups, iters, p, mask, sk, s); break;
        case 5: e = launch_mix<1, 0, 1>(workgroups, iters, p, mask, sk, s); break;
        case 6: e = launch_mix<0, 1, 1>(workgroups, iters, p, mask, sk, s); break;
        case 7: e = launch_mix<1, 1, 1>(workgroups, iters, p, mask, sk, s); break;
        case 8: e = launch_mix<0, 0, 0, 1>(workgroups, iters, p, mask, sk, s); break;
        case 9: e = launch_mix<1, 0, 0, 1>(workgroups, iters, p, mask, sk, s); break;
        case 10: e = launch_mix<0, 1, 0, 1>(workgroups, iters, p, mask, sk, s); break;
        case 11: e = launch_mix<1, 1, 0, 1>(workgroups, iters, p, mask, sk, s); break;
        case 12: e = launch_mix<0, 0, 1, 1>(workgroups, iters, p, mask, sk, s); break;
        case 13: e = launch_mix<1, 0, 1, 1>(workgroups, iters, p, mask, sk, s); break;
        case 14: e = launch_mix<0, 1, 1, 1>(workgroups, iters, p, mask, sk, s); break;
        case 15: e = launch_mix<1, 1, 1, 1>(workgroups, iters, p, mask, sk, s); break;
        case 18: e = launch_mix<0, 1, 0, 0, 1>(workgroups, iters, p, mask, sk, s); break;
        case 19: e = launch_mix<1, 1, 0, 0, 1>(workgroups, iters, p, mask, sk, s); break;
        case 22: e = launch_mix<0, 1, 1, 0, 1>(workgroups, iters, p, mask, sk, s); break;
        default: e = launch_mix<1, 1, 1, 0, 1>(workgroups, iters, p, mask, sk, s); break;
    }
    return e == hipSuccess ? FP8BS_OK : FP8BS_ERR_LAUNCH;
}
