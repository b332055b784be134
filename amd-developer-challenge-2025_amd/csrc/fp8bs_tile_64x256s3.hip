// The tiled MFMA kernel of fp8bs_tiled.h for one tile shape (all modes, both tail instantiations).
#include "fp8bs_tiled.h"

namespace fp8bs {
hipError_t launch_tile_64x256s3(const GemmArgs& a, int mode, hipStream_t stream) { return launch_shape<64, 256, 32, 64, false, 3>(a, mode, stream); }
}  // namespace fp8bs
