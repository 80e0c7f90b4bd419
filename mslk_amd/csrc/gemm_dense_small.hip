// The tile shapes of the dense GEMM below 128 x 256 on row-major weights, in a translation unit of their own so that they
// compile beside the large ones; which shape a problem gets is decided in launch_dense_tiled() (gemm_dense.hip).
// The last template argument of each launcher says when the weights are fetched with non-temporal loads: 2 always (shapes
// that are only picked for a single row of tiles), 1 when the problem is one row of tiles, 0 never.
#include "gemm_dense_shapes.h"

namespace mslk_amd {

hipError_t launch_dense_small_tile(int shape, const GemmProblem& p, hipStream_t s) {
  switch (shape) {
    case kTile32x32: return launch_tiled_shape<TileShape<32, 32, 2, 1, 8>, false, 2>(p, s);
    case kTile64x32: return launch_tiled_shape<TileShape<64, 32, 4, 1, 6>, false, 2>(p, s);
    case kTile64x64: return launch_tiled_shape<TileShape<64, 64, 4, 1, 5>, false, 1>(p, s);
    case kTile128x32: return launch_tiled_shape<TileShape<128, 32, 4, 1, 8>, false, 1>(p, s);
    case kTile128x64: return launch_tiled_shape<TileShape<128, 64, 4, 1, 6>, false, 1>(p, s);
    case kTile96x128: return launch_tiled_shape<TileShape<96, 128, 2, 2, 5>, false, 1>(p, s);
    case kTile128x128Ring: return launch_tiled_shape<TileShape<128, 128, 2, 2, 5>, false, 1>(p, s);
    case kTile128x128: return launch_tiled_shape<TileShape<128, 128>, false>(p, s);
    case kTile192x128: return launch_tiled_shape<TileShape<192, 128, 2, 2, 3>, false>(p, s);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace mslk_amd
