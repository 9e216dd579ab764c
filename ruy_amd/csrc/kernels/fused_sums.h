// Row sums of the `a` operand formed inside the launch of the largest int8
// tile (what the reference does in Pack, in the pass that touches the data
// anyway: ruy/pack.h:105-132), instead of by a kernel of their own in front
// of it. The arithmetic that kernel, planner and a host-only test share:
// which workgroups form the sums of a tile row, and which depth steps each of
// their waves takes.
//
// A wave of the 256x256 tile holds, for every depth step, the fragments of its
// 128 rows of `a` in registers; the same fragments sit in every workgroup of
// the tile row. So the sums of a tile row are dealt out: a few workgroups of
// the row (the contributors: those that the hardware starts first) each add up
// a share of the depth steps, from the fragments they hold anyway, one
// v_dot4 per register between two ring steps, and add their shares to the
// row's sums in global memory with atomic adds. Every workgroup of the row
// fetches the finished sums shortly before its write-back.
//
// uint8 data used in place is flipped to int8 in the fragment registers at
// its first use in a ring step, so at the point between two ring steps where
// the registers are added up, the fragments of the step just done are flipped
// and those of the step to come are not yet: the latter get the flip applied
// to the dot product's operand (one more v_xor per register), and the sums
// are those of the int8 values either way.
//
// Every workgroup walks the depth forwards, so the share of the last depth
// steps is only added when the main loops of the contributors end, which is
// when they themselves need the sums: the workgroups of the first round wait a
// few microseconds there, once per launch. (Letting half of the contributors
// walk the depth backwards, so that every step has been seen by somebody when
// the loops are half way through, was built and measured: the workgroups that
// walk the other way share no operand panel in L2 with their neighbours and
// fetch in descending address order, and the launch lost 10 us by it, three
// times what the wait costs.)
//
// Protocol. Every row has one 64-bit word, zero when the launch starts. A
// contributing wave adds, with one atomic add per row, its share of the row's
// sum plus 2^40: the word then holds the sum so far in its low 40 bits (as a
// signed number) and the number of contributions above them, and a reader of
// the word knows from that one read whether the sum is complete - there is no
// second location whose order with the first would matter. Every wave asks
// for the words of its 128 rows two or three ring steps before the end of its
// depth (they land in LDS while the last steps run). If a word is not
// complete then, the wave reads again after its main loop, a bounded number
// of times, and if the contributions still have not arrived (their workgroups
// never became resident: a device shared with somebody else's kernels) it
// forms the sums of its rows itself from global memory. No wave waits without
// bound, so a launch cannot hang. All of these accesses are agent-scope atomic
// operations (relaxed) or loads with the same cache policy, performed where
// all XCDs of the device agree (see depth_split.h).
//
// The words must be zero when a launch starts. There are two sets: a launch
// uses one and zeroes the other for the launch after it (the planner
// alternates them and tells the kernel how many rows the launch before last
// left dirty). A launch that is recorded into a graph and replayed would meet
// its own leftovers, so recorded calls keep the separate kernel.
//
// The same words serve the other way of forming sums inside a launch: the
// rows of an operand shared out over the workgroups of the grid's first round,
// each of which adds up its share from global memory in its prologue and
// contributes once per row (the tiles of 128 and 64 rows, either operand; the
// largest tile, the rows of `b`, whose words stand behind those of a's rows).
#ifndef RUY_AMD_CSRC_KERNELS_FUSED_SUMS_H_
#define RUY_AMD_CSRC_KERNELS_FUSED_SUMS_H_

#include "depth_split.h"  // RUYAMD_HOST_DEVICE

namespace ruyamd {
namespace fused_sums {

constexpr int kTileRows = 256;          // of the tile that forms sums this way
constexpr int kMaxRows = 65536;         // rows of `a` a launch may have
constexpr int kMaxContributorTiles = 8;
constexpr int kMinDepthSteps = 8;       // fewer ring steps than this: not worth it
constexpr int kBandRows = 4;            // tile rows per band of the kernel's tile order
constexpr int kXcds = 8;

// What a contributor adds to a row's word, and what a reader makes of the word.
constexpr int kCountShift = 40;
RUYAMD_HOST_DEVICE inline long long Contribution(int share_of_sum) {
  return static_cast<long long>(share_of_sum) + (1ll << kCountShift);
}
RUYAMD_HOST_DEVICE inline int ContributionsIn(long long word) {
  return static_cast<int>((word + (1ll << (kCountShift - 1))) >> kCountShift);
}
RUYAMD_HOST_DEVICE inline int SumIn(long long word) {
  return static_cast<int>(word - (static_cast<long long>(ContributionsIn(word)) << kCountShift));
}

// Position of tile (tile_m, tile_n) in the kernel's tile order: bands of four
// tile rows, walked column by column.
RUYAMD_HOST_DEVICE inline int TileOrder(int tiles_m, int tiles_n, int tile_m, int tile_n) {
  const int band = tile_m / kBandRows;
  const int rows_left = tiles_m - band * kBandRows;
  const int band_rows = rows_left < kBandRows ? rows_left : kBandRows;
  return band * kBandRows * tiles_n + tile_n * band_rows + (tile_m - band * kBandRows);
}

// The kernel gives each XCD a contiguous run of the tile order, and the
// hardware starts an XCD's workgroups in that order: a tile's place in the
// queue of its XCD.
RUYAMD_HOST_DEVICE inline int PlaceInQueue(int tiles_m, int tiles_n, int order) {
  const int per_xcd = (tiles_m * tiles_n + kXcds - 1) / kXcds;
  return order % per_xcd;
}

struct Contributors {
  int first_tile_n;  // the contributors of a tile row are tile columns first_tile_n .. first_tile_n + count - 1
  int count;
};

// The contributors of tile row tile_m: up to eight workgroups of the row that
// sit next to each other at the front of an XCD's queue, so that nobody who
// needs the sums runs a whole round ahead of those who form them. A band that
// starts in the middle of one XCD's queue and goes on at the head of the next
// one's has its contributors there, at the head.
RUYAMD_HOST_DEVICE inline Contributors ContributorsOfRow(int tiles_m, int tiles_n, int tile_m) {
  const int per_xcd = (tiles_m * tiles_n + kXcds - 1) / kXcds;
  const int band = tile_m / kBandRows;
  const int rows_left = tiles_m - band * kBandRows;
  const int band_rows = rows_left < kBandRows ? rows_left : kBandRows;
  const int row_in_band = tile_m - band * kBandRows;
  const int band_first = band * kBandRows * tiles_n;
  const int band_end = band_first + band_rows * tiles_n;
  int first = 0;
  if (band_first % per_xcd != 0) {
    const int next_queue = (band_first / per_xcd + 1) * per_xcd;
    if (next_queue < band_end) {
      // First tile column of this row at or behind the head of that queue.
      const int from = next_queue - band_first - row_in_band;
      const int n = from <= 0 ? 0 : (from + band_rows - 1) / band_rows;
      if (n < tiles_n) first = n;
    }
  }
  const int left = tiles_n - first;
  return Contributors{first, left < kMaxContributorTiles ? left : kMaxContributorTiles};
}

// What one wave of a workgroup does for the sums of its rows.
struct WaveShare {
  bool contributes;
  int first_step;    // its share: depth steps first_step .. end_step - 1
  int end_step;
  int expected;      // contributions a row's word shows when its sum is complete
};

// Depth steps per contributing wave when `contributor_tiles` workgroups of a
// tile row contribute.
RUYAMD_HOST_DEVICE inline int StepsPerWave(int depth_steps, int contributor_tiles) {
  return (depth_steps + 2 * contributor_tiles - 1) / (2 * contributor_tiles);
}

// `wave_n`: which of the workgroup's two waves that hold the same rows.
// `depth_steps`: ring steps of the whole depth. `uniform_run`: not 0 if the
// caller knows that the contributors of every tile row of this grid start at
// tile column 0 (FirstContributorIsZero), and then StepsPerWave of the grid,
// which saves the divisions that finding both takes. The contributing waves take consecutive runs of the depth
// steps, the two waves of a workgroup neighbouring runs: a workgroup is busy
// with the sums during one short stretch of its main loop.
RUYAMD_HOST_DEVICE inline WaveShare ShareOfWave(int tiles_m, int tiles_n, int tile_m, int tile_n, int wave_n,
                                               int depth_steps, int uniform_run = 0) {
  const Contributors c =
      uniform_run ? Contributors{0, tiles_n < kMaxContributorTiles ? tiles_n : kMaxContributorTiles}
                  : ContributorsOfRow(tiles_m, tiles_n, tile_m);
  WaveShare s;
  const int index = tile_n - c.first_tile_n;
  s.contributes = index >= 0 && index < c.count;
  s.expected = 2 * c.count;
  const int run = uniform_run ? uniform_run : StepsPerWave(depth_steps, c.count);
  const int first = (2 * index + wave_n) * run;
  const int end = first + run;
  s.first_step = first < depth_steps ? first : depth_steps;
  s.end_step = end < depth_steps ? end : depth_steps;
  return s;
}

// Whether the contributors of every tile row of a grid start at tile column 0
// (host side; true for grids whose bands of tile rows start at the head of an
// XCD's queue or do not reach the next one).
inline bool FirstContributorIsZero(int tiles_m, int tiles_n) {
  for (int tile_m = 0; tile_m < tiles_m; ++tile_m)
    if (ContributorsOfRow(tiles_m, tiles_n, tile_m).first_tile_n != 0) return false;
  return true;
}

}  // namespace fused_sums
}  // namespace ruyamd

#endif  // RUY_AMD_CSRC_KERNELS_FUSED_SUMS_H_
