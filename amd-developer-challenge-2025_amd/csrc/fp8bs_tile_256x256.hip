// The tiled MFMA kernel of fp8bs_tiled.h for one tile shape (all modes, both tail instantiations).
#include "fp8bs_tiled.h"

namespace fp8bs {
hipError_t launch_tile_256x256(const GemmArgs& a, int mode, hipStream_t stream) { return launch_shape<256, 256, 64, 128, true>(a, mode, stream); }
}  // namespace fp8bs
