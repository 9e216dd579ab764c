// Launch geometry of the kernels whose grids follow the problem size in more
// than one dimension. Plain host arithmetic, kept apart from the kernels so
// that its bounds can be tested without a device.
#ifndef RUY_AMD_CSRC_KERNELS_LAUNCH_GEOMETRY_H_
#define RUY_AMD_CSRC_KERNELS_LAUNCH_GEOMETRY_H_

#include <cstdint>

namespace ruyamd {

// HIP limits: grid.x < 2^31, grid.y and grid.z <= 65535.
constexpr unsigned kMaxGridX = 0x7fffffffu;
constexpr unsigned kMaxGridY = 65535u;

struct Grid2D {
  unsigned x = 1;
  unsigned y = 1;
};

// Generic kernel: tiles of kGenericTile x kGenericTile destination elements,
// x along the destination's contiguous dimension (`fast` elements), y along
// the other (`slow` elements). The kernel walks tile rows blockIdx.y,
// blockIdx.y + gridDim.y, ... so y may be capped.
constexpr int kGenericTile = 16;
inline Grid2D GenericGrid(int fast, int slow) {
  Grid2D g;
  const int64_t bx = (int64_t(fast) + kGenericTile - 1) / kGenericTile;
  const int64_t by = (int64_t(slow) + kGenericTile - 1) / kGenericTile;
  g.x = static_cast<unsigned>(bx < 1 ? 1 : bx);  // at most 2^27 for an int dimension
  g.y = static_cast<unsigned>(by < 1 ? 1 : (by > int64_t(kMaxGridY) ? int64_t(kMaxGridY) : by));
  return g;
}

// Element-wise kernels: `threads` elements per workgroup, grid-stride loop, so
// the block count may be capped as well.
inline unsigned ElementwiseBlocks(int64_t n, int threads) {
  const int64_t b = (n + threads - 1) / threads;
  return static_cast<unsigned>(b < 1 ? 1 : (b > int64_t(kMaxGridX) ? int64_t(kMaxGridX) : b));
}

}  // namespace ruyamd

#endif  // RUY_AMD_CSRC_KERNELS_LAUNCH_GEOMETRY_H_
