// Test infrastructure, not part of the product: what the FP8 MFMA of the reference's kernel returns on gfx950.
//
// The reference multiplies with v_mfma_f32_16x16x32_fp8_fp8, four chained per 128-wide K block with the fp32
// accumulator carried through (1-amd-fp8-mm/amd-fp8-mm-submission.py:345-352; 32 = 4 lane groups x 8 bytes).
// The product's kernels use v_mfma_f32_16x16x128_f8f6f4, whose accumulation drops low product bits
// (oracle/mfma_model.c).  This probe feeds the same committed vector pairs to the reference's instruction so
// that the two can be compared on the hardware: pair i is row i of A and column i of B of a 16x16 tile, the
// answer is the diagonal of D.  Lane l supplies the 8 bytes k = 8*(l/16) .. 8*(l/16)+7 of row l%16 of its chunk
// of 32 for both operands (the same map on both sides, so the sum is over matching k whatever the hardware's
// own order inside a chunk is).  Only tests/ may load the library built from this file.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef float v4f __attribute__((ext_vector_type(4)));

// a, b: count x 128 e4m3fn codes, k ascending; out: count floats.  One wave per 16 pairs.
__global__ __launch_bounds__(64) void chain_16x16x32_kernel(const uint8_t* a, const uint8_t* b, int count, float* out) {
    const int lane = threadIdx.x, r = lane & 15, g = lane >> 4;
    const int pair = blockIdx.x * 16 + r;
    v4f acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < 4; c++) {
        long av = 0, bv = 0;
        if (pair < count) {
            av = *(const long*)(a + (size_t)pair * 128 + 32 * c + 8 * g);
            bv = *(const long*)(b + (size_t)pair * 128 + 32 * c + 8 * g);
        }
        acc = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(av, bv, acc, 0, 0, 0);
    }
    // D[i][j] sits in lane j + 16*(i/4), register i%4: the diagonal element of pair r in lane r + 16*(r/4)
    if (g == r / 4 && pair < count) out[pair] = acc[r & 3];
}

extern "C" int mfma_probe_chain_16x16x32(const void* a, const void* b, int count, float* out, void* stream) {
    if (count <= 0) return 0;
    hipLaunchKernelGGL(chain_16x16x32_kernel, dim3((count + 15) / 16), dim3(64), 0, (hipStream_t)stream,
                       (const uint8_t*)a, (const uint8_t*)b, count, out);
    return hipGetLastError() == hipSuccess ? 0 : 1;
}
