// Internal interface between the C-ABI layer (fp8bs_api.hip) and the device code (fp8bs_kernels.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace fp8bs {

// Kernel arguments. Layouts as in include/fp8bs.h. In grouped mode `m` and `lda` are the total row
// count and `b`/`bs` carry a leading expert dimension.
struct GemmArgs {
    const uint8_t* a;
    const uint8_t* b;
    const float* as;
    const float* bs;
    uint16_t* c;            // bf16 bits
    float* ws;              // split-K partial planes [split_k][m][n]
    const int32_t* row_offsets;
    int m, n, k;
    int lda;                // bytes per k row of a (the row count of the whole matrix)
    int nb;                 // ceil(n / 128)
    int split_k, kb_per_split;
    int band_h;             // tile rows per band of the tile walk
    int num_experts;
    int epi;                // 0: bf16 of the product; 1: silu(column 2i) * column 2i+1, n/2 output columns
    int c_whole_lines;      // set by the launcher: rows of c start and end on 128-byte lines
    int by_expert;          // grouped: order of the tiles, 0 across the experts, 1 expert by expert (see the tile walk)
    // K blocks dealt to the workgroups (MODE 3 of the tiled kernel): `ws` then holds a header (a status word, one
    // 8-byte flag per workgroup) and one fp32 partial tile per workgroup, see StreamK below
    unsigned long long sk_nonce;   // value a flag takes when its workgroup's partial tile is complete: differs from call to call
    int sk_grid;            // workgroups of such a call: at most the places on the chip and the number of (tile, K block) pairs
    int sk_spin;            // polls of a flag before the wait gives up (< 0: give up at once - tests of the error path)
};

// Workspace of a call that deals K blocks (all offsets from the 16-byte aligned workspace base):
//   [0, 4)                          status word: set to FP8BS_ERR_TIMEOUT by a workgroup whose bounded wait gave up
//   [SK_FLAGS_OFF, + 8 * grid)      one flag per workgroup
//   [SK_SLOTS_OFF, + grid * slot)   one partial tile per workgroup, slot = tile_m * tile_n * 4 bytes, in lane order
struct StreamK {
    static constexpr size_t FLAGS_OFF = 256, SLOTS_OFF = 16384;
    static constexpr int MAX_GRID = (int)((SLOTS_OFF - FLAGS_OFF) / 8);
    static constexpr unsigned STATUS_TIMEOUT = 9;        // FP8BS_ERR_TIMEOUT
    static size_t bytes(int grid, int tile_m, int tile_n) { return SLOTS_OFF + (size_t)grid * (size_t)tile_m * (size_t)tile_n * 4u; }
};

// Per-device bookkeeping of the launchers.  A kernel's dynamic-LDS limit is a property of the kernel
// on one device, so "already raised" is remembered per device; devices beyond the table just set the
// attribute on every launch.  Races between threads are harmless (the call is idempotent).
static constexpr int MAX_DEVICES = 64;
inline int device_slot() {
    int d = 0;
    return (hipGetDevice(&d) == hipSuccess && d >= 0 && d < MAX_DEVICES) ? d : -1;
}
// `raised[slot]` holds the largest limit set so far for this kernel on that device.
inline hipError_t raise_lds_limit(const void* kernel, int bytes, int* raised) {
    const int slot = device_slot();
    if (slot >= 0 && raised[slot] >= bytes) return hipSuccess;
    hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess && slot >= 0) raised[slot] = bytes;
    return e;
}

// CUs of the current device, asked once per device (256, MI355X's count, if the runtime does not say)
inline int device_cus() {
    static int cus[MAX_DEVICES];
    const int slot = device_slot();
    if (slot >= 0 && cus[slot] > 0) return cus[slot];
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    if (slot >= 0) cus[slot] = n;
    return n;
}

// mode: 0 dense bf16, 1 dense split-K partials, 2 grouped.  variant: FP8BS_VARIANT_* (not AUTO).
hipError_t launch_gemm(int variant, int mode, const GemmArgs& args, hipStream_t stream);
// one per tile shape of the tiled kernel, each in a translation unit of its own
hipError_t launch_tile_256x256(const GemmArgs& args, int mode, hipStream_t stream);
hipError_t launch_tile_256x192(const GemmArgs& args, int mode, hipStream_t stream);
hipError_t launch_tile_256x128(const GemmArgs& args, int mode, hipStream_t stream);
hipError_t launch_tile_256x128s3(const GemmArgs& args, int mode, hipStream_t stream);
hipError_t launch_tile_128x128(const GemmArgs& args, int mode, hipStream_t stream);
hipError_t launch_tile_64x128(const GemmArgs& args, int mode, hipStream_t stream);
hipError_t launch_tile_192x192s3(const GemmArgs& args, int mode, hipStream_t stream);
hipError_t launch_tile_64x256s3(const GemmArgs& args, int mode, hipStream_t stream);
hipError_t launch_splitk_reduce(const float* ws, uint16_t* c, size_t mn, int split_k, hipStream_t stream);
int variant_lds_bytes(int variant);

}  // namespace fp8bs
