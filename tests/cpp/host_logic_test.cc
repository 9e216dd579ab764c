// Host-only tests of launch arithmetic that the device kernels rely on.
//
// Launch geometry: the generic kernel serves every type tuple ruy::Mul accepts
// (ruy/kernel.h:174-241 is the reference's counterpart), so its grid must be
// legal for every int-sized destination, including tall row-major ones whose
// tile-row count exceeds HIP's 65535 limit on grid.y.
//
// Depth split: the arrival-counter protocol of the tiled kernels, modelled
// with host threads in place of workgroups (one thread per part of a tile).
// The model uses the same arithmetic header as the kernels and checks what
// does not depend on the hardware: the parts cover every depth step exactly
// once whatever the remainder, exactly one workgroup per tile elects itself,
// it sees every part, the sum is taken in part order, and the counters are
// back at zero for the next launch.
//
// The same for the split of the 256x256 int8 tile, whose parts also share the
// adding up and the write-back by waiting for each other a bounded time.
//
// Row sums formed inside the launch of the largest int8 tile: which
// workgroups of a tile row add up which depth steps (kernels/fused_sums.h).
// Checked for every grid up to 48 x 48 tiles and several depths: the shares of
// a row's contributing waves cover every depth step exactly once for each of
// the two groups of 128 rows, the number of contributions everybody waits for
// is the number of contributing waves, and the contributors are among the
// tiles of their row that the hardware starts first; and a row's 64-bit word
// gives back the sum and the number of contributions whatever the signs and
// the order of the shares.
#include <atomic>
#include <cstdint>
#include <cstdio>
#include <thread>
#include <vector>

#include "kernels/depth_split.h"
#include "kernels/fused_sums.h"
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

namespace ds = ruyamd::depth_split;

static void TestDepthPartsCoverEveryStepOnce() {
  for (int steps = 1; steps <= 300; ++steps) {
    for (int wanted = 1; wanted <= 40; ++wanted) {
      const int parts = ds::PartsWithoutEmpty(steps, wanted);
      EXPECT(parts >= 1 && parts <= wanted);
      EXPECT(ds::NoEmptyPart(steps, parts));
      std::vector<int> covered(steps, 0);
      for (int z = 0; z < parts; ++z) {
        const int first = ds::FirstStep(steps, parts, z), count = ds::StepCount(steps, parts, z);
        EXPECT(count >= 1);
        for (int k = first; k < first + count; ++k) {
          EXPECT(k < steps);
          if (k < steps) ++covered[k];
        }
      }
      for (int k = 0; k < steps; ++k) EXPECT(covered[k] == 1);
      // A part index past the last part walks nothing (what a kernel launched
      // with more grid rows than parts would see).
      EXPECT(ds::StepCount(steps, parts, parts) == 0);
    }
  }
  EXPECT(!ds::NoEmptyPart(10, 7));  // 7 parts of 2 steps: parts 5 and 6 would be empty
  EXPECT(ds::PartsWithoutEmpty(10, 7) == 5);
}

// One "launch": tiles x parts threads. Thread (t, z) computes the partial sum
// of its depth steps of tile t (step k of tile t contributes value(t, k)),
// stores it to its slice, counts itself in, and if it was the last to arrive
// resets the counter, adds the slices up in part order and writes the result.
// fetch_add is acq_rel here: on the device the same ordering comes from
// waiting for the slice stores before the add and issuing the slice loads
// after it (see depth_split.h).
struct SplitModel {
  int tiles, steps;
  std::vector<std::atomic<unsigned>> counters;
  std::vector<double> slices;  // [tile][part]
  std::vector<double> result;  // [tile]
  std::vector<std::atomic<int>> finishers;
  SplitModel(int tiles_, int steps_, int max_parts)
      : tiles(tiles_), steps(steps_), counters(tiles_), slices(size_t(tiles_) * max_parts), result(tiles_),
        finishers(tiles_) {
    for (auto& c : counters) c.store(0);
  }
  static double Value(int tile, int k) { return 1.0 / (1 + tile + 3 * k); }  // order of summation matters
  void Launch(int parts, unsigned shuffle) {
    for (auto& f : finishers) f.store(0);
    std::vector<std::thread> threads;
    const int total = tiles * parts;
    for (int n = 0; n < total; ++n) {
      // A different arrival order every launch.
      const int id = int((n * 7919u + shuffle * 104729u) % unsigned(total));
      threads.emplace_back([this, id, parts] {
        const int t = id / parts, z = id % parts;
        double part = 0;
        const int first = ds::FirstStep(steps, parts, z);
        for (int k = first; k < first + ds::StepCount(steps, parts, z); ++k) part += Value(t, k);
        slices[size_t(t) * parts + z] = part;
        const unsigned previous = counters[t].fetch_add(1u, std::memory_order_acq_rel);
        if (!ds::IsLastArrival(previous, parts)) return;
        counters[t].store(0u, std::memory_order_relaxed);
        double sum = 0;
        for (int p = 0; p < parts; ++p) sum += slices[size_t(t) * parts + p];
        result[t] = sum;
        finishers[t].fetch_add(1);
      });
    }
    for (auto& th : threads) th.join();
  }
};

static void TestDepthSplitArrivalProtocol() {
  const int tiles = 6, steps = 37, max_parts = 8;
  SplitModel model(tiles, steps, max_parts);
  for (int launch = 0; launch < 24; ++launch) {
    const int parts = ds::PartsWithoutEmpty(steps, 2 + launch % (max_parts - 1));
    model.Launch(parts, unsigned(launch));
    for (int t = 0; t < tiles; ++t) {
      EXPECT(model.finishers[t].load() == 1);      // exactly one workgroup did the write-back
      EXPECT(model.counters[t].load() == 0);       // left at zero for the next launch
      // Reference: the same parts, summed in part order by one thread.
      double want = 0;
      for (int z = 0; z < parts; ++z) {
        double part = 0;
        const int first = ds::FirstStep(steps, parts, z);
        for (int k = first; k < first + ds::StepCount(steps, parts, z); ++k) part += SplitModel::Value(t, k);
        want += part;
      }
      EXPECT(model.result[t] == want);  // bit for bit: the order does not depend on who arrived last
    }
  }
}

// The split of the largest int8 tile (depth_split.h, second half): the parts
// of a tile also share the adding up and the write-back. One host thread per
// workgroup runs the kernel's protocol on the tile's three words - count in,
// look for the others a bounded number of times, claim one's own columns, the
// last one to arrive claims what is left, count out, last one out clears the
// words - with every kind of patience (no look at all, a few, many) and small
// random delays. Checked: every block column of every tile is finished exactly
// once, from all parts' values; the words are zero again after every launch;
// with no patience at all the last arriver does everything.
struct LargeSplitModel {
  int tiles, steps;
  std::vector<std::atomic<unsigned>> words;  // kLargeWordsPerTile per tile
  std::vector<long long> slices;             // [tile][part][block column]
  std::vector<std::atomic<int>> finished;    // [tile][block column]: how often
  std::vector<long long> result;             // [tile][block column]
  std::vector<std::atomic<int>> columns_by_last;  // [tile]: columns the last arriver finished
  LargeSplitModel(int tiles, int steps)
      : tiles(tiles), steps(steps), words(size_t(tiles) * ds::kLargeWordsPerTile),
        slices(size_t(tiles) * ds::kLargeMaxParts * ds::kLargeBlockColumns),
        finished(size_t(tiles) * ds::kLargeBlockColumns), result(size_t(tiles) * ds::kLargeBlockColumns),
        columns_by_last(tiles) {
    for (auto& w : words) w.store(0);
  }
  static long long Value(int t, int k, int column) { return (t + 1) * 1000003ll + k * 7919ll - column * 31ll; }
  void Launch(int parts, int looks, unsigned seed) {
    for (auto& f : finished) f.store(0);
    for (auto& c : columns_by_last) c.store(0);
    std::vector<std::thread> threads;
    for (int t = 0; t < tiles; ++t)
      for (int z = 0; z < parts; ++z)
        threads.emplace_back([this, t, z, parts, looks, seed] {
          unsigned rng = seed * 2654435761u + unsigned(t * 131 + z * 17 + 1);
          auto pause = [&rng] {
            rng = rng * 1664525u + 1013904223u;
            if ((rng >> 28) < 6) std::this_thread::yield();
          };
          std::atomic<unsigned>* w = &words[size_t(t) * ds::kLargeWordsPerTile];
          // The part's accumulators: all block columns go to memory.
          const int first = ds::FirstStep(steps, parts, z);
          for (int c = 0; c < ds::kLargeBlockColumns; ++c) {
            long long sum = 0;
            for (int k = first; k < first + ds::StepCount(steps, parts, z); ++k) sum += Value(t, k, c);
            slices[(size_t(t) * ds::kLargeMaxParts + z) * ds::kLargeBlockColumns + c] = sum;
          }
          pause();
          const unsigned before = w[ds::kArrivals].fetch_add(1, std::memory_order_acq_rel);
          const bool last = ds::IsLastArrival(before, parts);
          bool all = last;
          for (int look = 0; !all && look < looks; ++look) {
            pause();
            all = w[ds::kArrivals].load(std::memory_order_acquire) == unsigned(parts);
          }
          const int columns = ds::LargeColumnsPerPart(parts);
          for (int turn = 0; turn < parts; ++turn) {
            if (turn == 0 ? !all : !last) break;
            const int owner = z + turn < parts ? z + turn : z + turn - parts;
            const unsigned claims = w[ds::kClaims].fetch_or(ds::ClaimBit(owner), std::memory_order_acq_rel);
            if (!ds::ClaimSucceeded(claims, owner)) continue;
            for (int c = owner * columns; c < (owner + 1) * columns; ++c) {
              long long sum = 0;
              for (int p = 0; p < parts; ++p)
                sum += slices[(size_t(t) * ds::kLargeMaxParts + p) * ds::kLargeBlockColumns + c];
              result[size_t(t) * ds::kLargeBlockColumns + c] = sum;
              finished[size_t(t) * ds::kLargeBlockColumns + c].fetch_add(1);
              if (last) columns_by_last[t].fetch_add(1);
              pause();
            }
          }
          if (ds::IsLastArrival(w[ds::kExits].fetch_add(1, std::memory_order_acq_rel), parts)) {
            w[ds::kArrivals].store(0);
            w[ds::kClaims].store(0);
            w[ds::kExits].store(0);
          }
        });
    for (auto& th : threads) th.join();
  }
};

// Every (tile, part) of a split launch of the large tile is some workgroup's
// work exactly once, an XCD sees one part only, and its tiles are a run of the
// tile order.
static void TestLargeTileSplitWork() {
  for (int total = 1; total <= 256; ++total) {
    const int grid = (total + 7) / 8 * 8;
    for (int parts = 2; parts <= 8; parts *= 2) {
      std::vector<int> taken(size_t(total) * parts, 0);
      int part_of_xcd[8], first_of_xcd[8], count_of_xcd[8] = {};
      bool ok = true;
      for (int linear = 0; linear < grid * parts; ++linear) {
        const ds::LargeSplitWork w = ds::LargeSplitWorkOf(linear, total, parts);
        ok = ok && w.part >= 0 && w.part < parts && w.tile >= 0 && w.tile <= total;
        if (!ok || w.tile == total) continue;
        ++taken[size_t(w.tile) * parts + w.part];
        const int xcd = linear & 7;
        if (count_of_xcd[xcd] == 0) {
          part_of_xcd[xcd] = w.part;
          first_of_xcd[xcd] = w.tile;
        }
        ok = ok && part_of_xcd[xcd] == w.part && w.tile == first_of_xcd[xcd] + count_of_xcd[xcd];
        ++count_of_xcd[xcd];
      }
      for (int x : taken) ok = ok && x == 1;
      EXPECT(ok);
      if (!ok) return;
    }
  }
}

static void TestLargeTileSplitProtocol() {
  const int tiles = 5, steps = 40;
  LargeSplitModel model(tiles, steps);
  EXPECT(ds::LargeParts(steps, 8) == 8 && ds::LargeParts(steps, 7) == 4 && ds::LargeParts(steps, 3) == 2 &&
         ds::LargeParts(steps, 1) == 1 && ds::LargeParts(3, 8) == 2 && ds::LargeParts(1, 8) == 1 &&
         ds::LargeParts(7, 8) == 4 &&
         ds::LargeParts(41, 8) == 4);  // (41 steps in 8 parts of 6 would leave the last one empty)
  for (int launch = 0; launch < 60; ++launch) {
    const int parts = 2 << (launch % 3);
    const int looks = launch % 4 == 0 ? 0 : (launch % 4 == 1 ? 3 : 100000);
    EXPECT(ds::LargePartsAllowed(parts) && ds::NoEmptyPart(steps, parts));
    model.Launch(parts, looks, unsigned(launch));
    for (int t = 0; t < tiles; ++t) {
      for (int c = 0; c < ds::kLargeBlockColumns; ++c) {
        EXPECT(model.finished[size_t(t) * ds::kLargeBlockColumns + c].load() == 1);
        long long want = 0;
        for (int k = 0; k < steps; ++k) want += LargeSplitModel::Value(t, k, c);
        EXPECT(model.result[size_t(t) * ds::kLargeBlockColumns + c] == want);
      }
      for (int i = 0; i < ds::kLargeWordsPerTile; ++i)
        EXPECT(model.words[size_t(t) * ds::kLargeWordsPerTile + i].load() == 0);
      if (looks == 0) EXPECT(model.columns_by_last[t].load() == ds::kLargeBlockColumns);
    }
  }
}

namespace fs = ruyamd::fused_sums;

static void CheckRowSumShares(int tiles_m, int tiles_n, int depth_steps) {
  for (int tile_m = 0; tile_m < tiles_m; ++tile_m) {
    const fs::Contributors c = fs::ContributorsOfRow(tiles_m, tiles_n, tile_m);
    EXPECT(c.count >= 1 && c.count <= fs::kMaxContributorTiles);
    EXPECT(c.first_tile_n >= 0 && c.first_tile_n + c.count <= tiles_n);
    // The first contributor is in the round of workgroups (32 to an XCD) in
    // which the first tile of the row is started, and the contributors follow
    // each other in the tile order.
    int first_place = 1 << 30;
    for (int n = 0; n < tiles_n; ++n) {
      const int place = fs::PlaceInQueue(tiles_m, tiles_n, fs::TileOrder(tiles_m, tiles_n, tile_m, n));
      if (place < first_place) first_place = place;
    }
    const int order0 = fs::TileOrder(tiles_m, tiles_n, tile_m, c.first_tile_n);
    EXPECT(fs::PlaceInQueue(tiles_m, tiles_n, order0) / 32 == first_place / 32);
    const int order_last = fs::TileOrder(tiles_m, tiles_n, tile_m, c.first_tile_n + c.count - 1);
    EXPECT(order_last - order0 <= (fs::kMaxContributorTiles - 1) * fs::kBandRows);
    // Coverage: every depth step once, by the waves that hold the same rows
    // (wave_n 0 and 1 of every contributing workgroup).
    std::vector<int> seen(depth_steps, 0);
    int contributing = 0, expected = -1;
    for (int n = 0; n < tiles_n; ++n) {
      for (int wave_n = 0; wave_n < 2; ++wave_n) {
        const fs::WaveShare s = fs::ShareOfWave(tiles_m, tiles_n, tile_m, n, wave_n, depth_steps);
        EXPECT(expected < 0 || expected == s.expected);
        expected = s.expected;
        EXPECT(s.contributes == (n >= c.first_tile_n && n < c.first_tile_n + c.count));
        // The same with the hint that saves the search for the contributors.
        if (fs::FirstContributorIsZero(tiles_m, tiles_n)) {
          const int run = fs::StepsPerWave(depth_steps, tiles_n < fs::kMaxContributorTiles ? tiles_n : fs::kMaxContributorTiles);
          const fs::WaveShare h = fs::ShareOfWave(tiles_m, tiles_n, tile_m, n, wave_n, depth_steps, run);
          EXPECT(h.contributes == s.contributes && h.first_step == s.first_step && h.end_step == s.end_step &&
                 h.expected == s.expected);
        }
        if (!s.contributes) continue;
        ++contributing;
        EXPECT(s.first_step >= 0 && s.first_step <= s.end_step && s.end_step <= depth_steps);
        for (int step = s.first_step; step < s.end_step; ++step) ++seen[step];
      }
    }
    EXPECT(contributing == expected);
    for (int k = 0; k < depth_steps; ++k) EXPECT(seen[k] == 1);
  }
}

static void TestRowSumWords() {
  // Shares of every sign and size that a depth of up to 2^23 bytes can
  // produce, added in any order, 1 to 16 of them.
  uint64_t state = 12345;
  auto next = [&]() {
    state = state * 6364136223846793005ull + 1442695040888963407ull;
    return state >> 33;
  };
  const int extremes[] = {0, 1, -1, 127 * (1 << 23), -128 * (1 << 23), 2147483647, -2147483647 - 1};
  for (int trial = 0; trial < 20000; ++trial) {
    const int n = 1 + int(next() % 16);
    long long word = 0;
    int64_t sum = 0;
    for (int i = 0; i < n; ++i) {
      int share = trial < 2000 ? extremes[next() % 7] / n : int(int64_t(next() % (1ull << 31)) - (1ll << 30)) / n;
      word += fs::Contribution(share);
      sum += share;
      EXPECT(fs::ContributionsIn(word) == i + 1);
      EXPECT(fs::SumIn(word) == int(sum));
    }
  }
  EXPECT(fs::ContributionsIn(0) == 0 && fs::SumIn(0) == 0);
}

static void TestRowSumShares() {
  const int before = g_failures;
  for (int tiles_m = 1; tiles_m <= 48 && g_failures == before; ++tiles_m)
    for (int tiles_n = 1; tiles_n <= 48 && g_failures == before; ++tiles_n)
      for (int depth_steps : {16, 17, 33, 64}) CheckRowSumShares(tiles_m, tiles_n, depth_steps);
  CheckRowSumShares(32, 32, 64);   // 8192^3
  CheckRowSumShares(256, 3, 128);  // the most rows a launch may have
  CheckRowSumShares(5, 200, 20);
  if (g_failures != before) std::fprintf(stderr, "(row-sum shares: stopped at the first failing grid)\n");
}

int main() {
  TestRowSumWords();
  TestRowSumShares();
  TestGenericGrid();
  TestElementwiseBlocks();
  TestDepthPartsCoverEveryStepOnce();
  TestDepthSplitArrivalProtocol();
  TestLargeTileSplitProtocol();
  TestLargeTileSplitWork();
  if (g_failures) {
    std::fprintf(stderr, "host_logic_test: %d failure(s)\n", g_failures);
    return 1;
  }
  std::printf("host_logic_test: all passed\n");
  return 0;
}
