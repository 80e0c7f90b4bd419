// The tile-shape kernels of the dense GEMM on pre-shuffled (blocked) weights: the instances and their shape dispatch, in a
// translation unit of their own so that they compile beside the row-major ones.
#include "gemm_dense_shapes.h"

namespace mslk_amd {

// Same tile-count thresholds as the row-major dispatch in launch_dense_tiled(), written as fractions of `cus`, the CU count
// of the device: 256 x 256 tiles once they give most CUs work (persistent when there are more tiles than CUs), 128-row
// tiles of 128, 64 or 32 columns below that, so that the weight stream is spread over as many CUs as there are.
hipError_t launch_dense_tiled_preshuffled(const GemmProblem& p, int cus, hipStream_t s) {
  const int64_t big_tiles = (int64_t)((p.M + 255) / 256) * ((p.N + 255) / 256);
  const int64_t small_tiles = (int64_t)((p.M + 127) / 128) * ((p.N + 127) / 128);
  if (big_tiles > cus) return launch_persistent_shape<TileShape<256, 256>, true>(p, cus, s);
  // the two 192-row shapes of the row-major dispatch, under the same conditions: 192 x 256 where more than half a CU
  // count of 256 x 256 tiles still leaves CUs idle, 192 x 128 where the 128 x 128 tiles would need a second pass
  if (big_tiles > cus / 2 && p.K >= 2048 && (int64_t)((p.M + 191) / 192) * ((p.N + 255) / 256) <= cus)
    return launch_tiled_shape<TileShape<192, 256>, true>(p, s);
  if (big_tiles >= cus * 3 / 4) return launch_tiled_shape<TileShape<256, 256>, true>(p, s);
  if (small_tiles <= cus / 4 && p.N >= 64) return launch_tiled_shape<TileShape<128, 32, 4, 1, 8>, true>(p, s);
  if (small_tiles <= cus / 2 && p.N >= 128) return launch_tiled_shape<TileShape<128, 64, 4, 1, 6>, true>(p, s);
  if (small_tiles <= cus) {   // 96-row tiles where they fit one per CU as well: more tiles, never more work per tile
    if ((int64_t)((p.M + 95) / 96) * ((p.N + 127) / 128) <= cus) return launch_tiled_shape<TileShape<96, 128, 2, 2, 5>, true>(p, s);
    return launch_tiled_shape<TileShape<128, 128, 2, 2, 5>, true>(p, s);
  }
  if (big_tiles <= cus / 2 && (int64_t)((p.M + 191) / 192) * ((p.N + 127) / 128) <= cus)
    return launch_tiled_shape<TileShape<192, 128, 2, 2, 3>, true>(p, s);
  return launch_tiled_shape<TileShape<128, 128>, true>(p, s);
}

}  // namespace mslk_amd
