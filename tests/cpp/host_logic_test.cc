// Host-only tests of launch arithmetic that the device kernels rely on.
//
// Launch geometry: the generic kernel serves every type tuple ruy::Mul accepts
// (ruy/kernel.h:174-241 is the reference's counterpart), so its grid must be
// legal for every int-sized destination, including tall row-major ones whose
// tile-row count exceeds HIP's 65535 limit on grid.y.
#include <cstdint>
#include <cstdio>

#include "kernels/launch_geometry.h"

static int g_failures = 0;
#define EXPECT(cond)                                                          \
  do {                                                                        \
    if (!(cond)) {                                                            \
      std::fprintf(stderr, "%s:%d: EXPECT failed: %s\n", __FILE__, __LINE__, #cond); \
      ++g_failures;                                                           \
    }                                                                         \
  } while (0)

// Every (fast, slow) element must be visited exactly once by a kernel that
// walks tile rows blockIdx.y, blockIdx.y + gridDim.y, ...
static void CheckGenericCoverage(int fast, int slow) {
  const ruyamd::Grid2D g = ruyamd::GenericGrid(fast, slow);
  EXPECT(g.x >= 1 && g.x <= ruyamd::kMaxGridX);
  EXPECT(g.y >= 1 && g.y <= ruyamd::kMaxGridY);
  EXPECT(int64_t(g.x) * ruyamd::kGenericTile >= fast);
  // Tile rows: block row b handles rows b, b + g.y, ... < tile_rows.
  const int64_t tile_rows = (int64_t(slow) + ruyamd::kGenericTile - 1) / ruyamd::kGenericTile;
  int64_t visited = 0;
  for (unsigned b = 0; b < g.y; ++b)
    for (int64_t r = b; r < tile_rows; r += g.y) ++visited;
  EXPECT(visited == tile_rows);
}

static void TestGenericGrid() {
  CheckGenericCoverage(1, 1);
  CheckGenericCoverage(16, 16);
  CheckGenericCoverage(17, 15);
  CheckGenericCoverage(4, 2000000);        // f64 2M x 4 row-major: 125000 tile rows
  CheckGenericCoverage(2, 1048561);        // one past the old limit
  CheckGenericCoverage(2, 2147483647);     // the largest int dimension
  CheckGenericCoverage(2147483647, 1);
  const ruyamd::Grid2D tall = ruyamd::GenericGrid(4, 2000000);
  EXPECT(tall.y == 65535);
}

static void TestElementwiseBlocks() {
  EXPECT(ruyamd::ElementwiseBlocks(1, 256) == 1);
  EXPECT(ruyamd::ElementwiseBlocks(256, 256) == 1);
  EXPECT(ruyamd::ElementwiseBlocks(257, 256) == 2);
  EXPECT(ruyamd::ElementwiseBlocks(int64_t(1) << 40, 256) == ruyamd::kMaxGridX);
}

int main() {
  TestGenericGrid();
  TestElementwiseBlocks();
  if (g_failures) {
    std::fprintf(stderr, "host_logic_test: %d failure(s)\n", g_failures);
    return 1;
  }
  std::printf("host_logic_test: all passed\n");
  return 0;
}
