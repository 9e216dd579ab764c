// Host-only model of the ring of the largest int8 tile (the "paired" schedule
// of kernels/mfma_gemm.h). The kernel takes the position of every matrix
// instruction, fragment read, load and barrier of a ring step from
// kernels/paired_schedule.h; this test builds the instruction stream of a wave
// from the same header and checks, without a GPU, what the schedule must
// guarantee whatever the timing of the four waves:
//
//   registers  every matrix instruction of depth step t finds the fragments of
//              step t in both of its operand registers (no register is read
//              anew before its last use, none is used before it is read), and
//              uint8 data is flipped exactly once between read and first use;
//   LDS, read after write   a fragment is read from a ring slot only when the
//              loads that fill those rows have been awaited by the wave that
//              issued them AND a workgroup barrier has been passed since;
//   LDS, write after read   a ring slot's rows are loaded anew only after a
//              barrier that every wave passes behind its last read of them;
//   coverage   a step issues each of the 64 blocks once per depth half and
//              each of the 16 loads once.
//
// What the model knows of the hardware: a direct-to-LDS load may write its
// rows at any moment between its issue and the wait that covers it (loads
// complete in order; a wait for "at most n outstanding" covers all but the n
// most recent); a barrier orders everything a wave did in front of it (its LDS
// reads included: the compiler puts the wait for them in front of every
// barrier) against everything any wave does behind it. All four waves run the
// same stream, so the barriers cut it into epochs that the waves pass
// together: two events of different waves are ordered only if they lie in
// different epochs. Every fragment's rows come from two loads that mostly
// another wave issued (paired_schedule::FirstRowOfLoad, FirstRowOfFragment),
// so the model holds every read against the cross-wave rule.
//
// The test then alters the constants, one alteration at a time (barriers moved,
// the two load trains exchanged, a shorter wait, ...), and expects the model to
// object to every one of them: a model that accepts everything checks nothing.
#include <cstdio>
#include <string>
#include <vector>

#include "kernels/paired_schedule.h"

namespace ps = ruyamd::paired_schedule;

static int g_failures = 0;
#define EXPECT(cond)                                                          \
  do {                                                                        \
    if (!(cond)) {                                                            \
      std::fprintf(stderr, "%s:%d: EXPECT failed: %s\n", __FILE__, __LINE__, #cond); \
      ++g_failures;                                                           \
    }                                                                         \
  } while (0)

namespace {

enum Kind { kLoad, kOtherMemoryOp, kWaitLoads, kBarrier, kRead, kMma };

struct Event {
  Kind kind;
  int step;      // kLoad: the depth step fetched; kMma: the step computed
  bool is_a;     // kLoad, kRead
  int half;      // kRead, kMma
  int index;     // kLoad: load number; kRead: block row / column; kMma: block row
  int col;       // kMma: block column
  int slot;      // kRead: ring slot read
  int left;      // kWaitLoads: loads that may stay outstanding
  bool first_a, first_b;  // kMma: where uint8 data would be flipped
  int instruction;        // the matrix instruction it stands at (for messages)
};

// The stream of one wave over `depth_steps` ring steps. `other_memory_ops`:
// between two steps the wave issues memory operations of its own that count
// like loads (the atomic adds and the fetch of the row sums, see
// kernels/fused_sums.h); they must not weaken any wait.
std::vector<Event> StreamOfWave(int depth_steps, const ps::Timing& t, int other_memory_ops) {
  std::vector<Event> s;
  auto load = [&](int step, bool is_a, int index, int n) {
    s.push_back(Event{kLoad, step, is_a, 0, index, 0, step % 2, 0, false, false, n});
  };
  auto read = [&](int slot, bool is_a, int half, int index, int n) {
    s.push_back(Event{kRead, 0, is_a, half, index, 0, slot, 0, false, false, n});
  };
  // In front of the first step (mfma_gemm.h, "the largest int8 tile").
  for (int step = 0; step < 2; ++step) {
    for (int l = 0; l < ps::kLoads; ++l) load(step, false, l, -1);
    for (int l = 0; l < ps::kLoads; ++l) load(step, true, l, -1);
  }
  s.push_back(Event{kWaitLoads, 0, false, 0, 0, 0, 0, ps::kLoadsLeftBeforeFirstStep, false, false, -1});
  s.push_back(Event{kBarrier, 0, false, 0, 0, 0, 0, 0, false, false, -1});
  for (int i = 0; i < ps::kRowsReadAhead; ++i)
    for (int half = 0; half < 2; ++half) read(0, true, half, i, -1);
  for (int cp = 0; cp < ps::kColumnsReadAhead; ++cp)
    for (int half = 0; half < 2; ++half) read(0, false, half, ps::ColumnAt(0, 0, cp), -1);
  for (int kt = 0; kt < depth_steps; ++kt) {
    const int parity = kt % 2;
    for (int n = 0; n < ps::kInstructions; ++n) {
      if (n == t.barrier1) s.push_back(Event{kBarrier, 0, false, 0, 0, 0, 0, 0, false, false, n});
      if (n == t.barrier2) {
        s.push_back(Event{kWaitLoads, 0, false, 0, 0, 0, 0, t.loads_left_at_barrier2, false, false, n});
        s.push_back(Event{kBarrier, 0, false, 0, 0, 0, 0, 0, false, false, n});
      }
      const ps::Mma m = ps::MmaAt(parity, n);
      s.push_back(Event{kMma, kt, false, m.half, m.row, m.col, 0, 0, m.first_use_of_a, m.first_use_of_b, n});
      const ps::Read r = ps::ReadBehind(parity, n, t);
      if (r.valid) read(r.of_next_step ? parity ^ 1 : parity, r.is_a, r.half, r.index, n);
      const ps::Load l = ps::LoadBehind(n, t);
      // Steps past the end of the depth are fetched, too (as zeros): the
      // number of loads in flight never depends on the depth.
      if (l.valid) load(kt + 2, !l.is_b, l.index, n);
    }
    for (int i = 0; i < other_memory_ops; ++i)
      s.push_back(Event{kOtherMemoryOp, 0, false, 0, 0, 0, 0, 0, false, false, ps::kInstructions});
  }
  // Behind the last step, before the ring's LDS is used for something else.
  s.push_back(Event{kWaitLoads, 0, false, 0, 0, 0, 0, 0, false, false, ps::kInstructions});
  s.push_back(Event{kBarrier, 0, false, 0, 0, 0, 0, 0, false, false, ps::kInstructions});
  return s;
}

struct LoadWindow {
  int step;
  int issue_epoch;
  int covered_epoch;  // epoch of the wait that covers it; visible to all from the next epoch on
};

std::string Where(const Event& e, int position) {
  char buffer[96];
  std::snprintf(buffer, sizeof buffer, " (event %d, at matrix instruction %d)", position, e.instruction);
  return buffer;
}

// Returns the first objection, or an empty string. `flip`: model the uint8
// path, where a fragment is flipped in its registers at its first use.
std::string Check(int depth_steps, const ps::Timing& t, int other_memory_ops, bool flip, int* min_read_ahead) {
  const std::vector<Event> s = StreamOfWave(depth_steps, t, other_memory_ops);
  const int count = static_cast<int>(s.size());

  // Pass 1: epochs, and for every load the epoch of the wait that covers it.
  std::vector<int> epoch(count);
  // windows[is_a][slot][load index]: the loads into those rows, in issue order.
  std::vector<LoadWindow> windows[2][2][ps::kLoads];
  {
    struct Outstanding {
      bool is_load;
      int is_a, slot, index, entry;
    };
    std::vector<Outstanding> in_flight;
    int barriers = 0;
    for (int p = 0; p < count; ++p) {
      const Event& e = s[p];
      epoch[p] = barriers;
      if (e.kind == kBarrier) ++barriers;
      if (e.kind == kLoad) {
        auto& w = windows[e.is_a][e.slot][e.index];
        w.push_back(LoadWindow{e.step, barriers, -1});
        in_flight.push_back(Outstanding{true, e.is_a, e.slot, e.index, static_cast<int>(w.size()) - 1});
      }
      if (e.kind == kOtherMemoryOp) in_flight.push_back(Outstanding{false, 0, 0, 0, 0});
      if (e.kind == kWaitLoads) {
        while (static_cast<int>(in_flight.size()) > e.left) {
          const Outstanding o = in_flight.front();
          in_flight.erase(in_flight.begin());
          if (o.is_load) windows[o.is_a][o.slot][o.index][o.entry].covered_epoch = barriers;
        }
      }
    }
    if (!in_flight.empty()) return "loads still in flight when the ring is given up";
  }
  // Loads into the same rows must not overlap each other either.
  for (int a = 0; a < 2; ++a)
    for (int slot = 0; slot < 2; ++slot)
      for (int l = 0; l < ps::kLoads; ++l) {
        const auto& w = windows[a][slot][l];
        for (size_t i = 0; i + 1 < w.size(); ++i) {
          if (w[i + 1].step != w[i].step + 2) return "a ring slot's rows are not loaded with every second step in turn";
          if (w[i + 1].issue_epoch <= w[i].covered_epoch) return "two loads into the same rows may be in flight at once";
        }
      }

  // What step the rows of load (is_a, slot, index) hold for a reader in epoch
  // e, whichever wave it is: -1 if a load into them may be in flight.
  auto content = [&](bool is_a, int slot, int index, int e) {
    int step = -1;
    for (const LoadWindow& w : windows[is_a][slot][index]) {
      if (w.covered_epoch < e) {
        step = w.step;  // arrived, and a barrier has been passed since
      } else if (w.issue_epoch <= e) {
        return -1;  // may be writing while this reader reads
      }
    }
    return step;
  };

  // Pass 2: registers.
  struct Register {
    int step = -2;  // -2 never read, -1 read while its rows were in flux
    bool flipped = false;
    int read_at = -1;   // number of matrix instructions issued before its read
    bool used = false;  // since that read
  };
  Register fa[2][ps::kBlocks], fb[2][ps::kBlocks];
  int mmas = 0;
  int last_mma = -1;
  int step_of_counts = -1;
  int block_count[2][ps::kBlocks][ps::kBlocks] = {};
  int load_count[2][ps::kLoads] = {};
  auto close_step = [&]() -> std::string {
    for (int h = 0; h < 2; ++h)
      for (int i = 0; i < ps::kBlocks; ++i)
        for (int j = 0; j < ps::kBlocks; ++j) {
          if (block_count[h][i][j] != 1) return "a step does not issue every block once per depth half";
          block_count[h][i][j] = 0;
        }
    for (int a = 0; a < 2; ++a)
      for (int l = 0; l < ps::kLoads; ++l) {
        if (load_count[a][l] != 1) return "a step does not issue each of its 16 loads once";
        load_count[a][l] = 0;
      }
    return "";
  };
  for (int p = 0; p < count; ++p) {
    const Event& e = s[p];
    if (e.kind == kLoad && e.instruction >= 0) ++load_count[e.is_a][e.index];
    if (e.kind == kRead) {
      // A fragment's 16 rows are those of two loads, whichever wave reads
      // (the loads' numbers are the same for all four; their waves differ).
      Register& r = (e.is_a ? fa : fb)[e.half][e.index];
      r.step = -3;
      for (int wave = 0; wave < ps::kWaves; ++wave) {
        const int first_row = ps::FirstRowOfFragment(wave, e.is_a, e.index);
        for (int row = first_row; row < first_row + ps::kRowsPerBlock; row += ps::kRowsPerLoad) {
          const int loader = row / ps::kRowsPerLoad / ps::kLoads;
          const int index = row / ps::kRowsPerLoad % ps::kLoads;
          if (loader < 0 || loader >= ps::kWaves || ps::FirstRowOfLoad(loader, index) != row)
            return "a fragment's rows are not those of whole loads";
          const int c = content(e.is_a, e.slot, index, epoch[p]);
          r.step = r.step == -3 || r.step == c ? c : -1;
        }
      }
      r.flipped = false;
      r.read_at = e.instruction < 0 ? -1 : mmas;  // (the reads in front of the first step are used at once)
      r.used = false;
    }
    if (e.kind == kMma) {
      if (e.step != step_of_counts) {
        if (step_of_counts >= 0) {
          const std::string objection = close_step();
          if (!objection.empty()) return objection;
        }
        step_of_counts = e.step;
      }
      ++block_count[e.half][e.index][e.col];
      // (Reads and loads may stand between the two; another matrix instruction may not.)
      if (e.half == 1 && (last_mma < 0 || s[last_mma].step != e.step || s[last_mma].index != e.index ||
                          s[last_mma].col != e.col || s[last_mma].half != 0))
        return "the two depth halves of a block are not consecutive matrix instructions" + Where(e, p);
      last_mma = p;
      if (flip && e.half == 0) {
        for (int h = 0; h < 2; ++h) {
          if (e.first_a) {
            if (fa[h][e.index].flipped) return "an A fragment is flipped twice" + Where(e, p);
            if (fa[h][e.index].step != e.step) return "an A fragment is flipped before it is read" + Where(e, p);
            fa[h][e.index].flipped = true;
          }
          if (e.first_b) {
            if (fb[h][e.col].flipped) return "a B fragment is flipped twice" + Where(e, p);
            if (fb[h][e.col].step != e.step) return "a B fragment is flipped before it is read" + Where(e, p);
            fb[h][e.col].flipped = true;
          }
        }
      }
      Register* operands[2] = {&fa[e.half][e.index], &fb[e.half][e.col]};
      for (Register* r : operands) {
        if (r->step == -2) return "a matrix instruction uses a register that was never read" + Where(e, p);
        if (r->step == -1)
          return "a matrix instruction uses a fragment that was read while its rows could be written" + Where(e, p);
        if (r->step != e.step) {
          char buffer[160];
          std::snprintf(buffer, sizeof buffer, "a matrix instruction of step %d finds the fragment of step %d",
                        e.step, r->step);
          return buffer + Where(e, p);
        }
        if (flip && !r->flipped) return "a matrix instruction uses uint8 data that was not flipped" + Where(e, p);
        if (!r->used) {
          r->used = true;
          const int ahead = mmas - r->read_at;
          if (min_read_ahead && r->read_at >= 0 && ahead < *min_read_ahead) *min_read_ahead = ahead;
        }
      }
      ++mmas;
    }
  }
  if (step_of_counts >= 0) {
    const std::string objection = close_step();
    if (!objection.empty()) return objection;
  }
  return "";
}

void TestScheduleOfTheKernel() {
  int min_read_ahead = 1 << 30;
  for (int depth_steps = 1; depth_steps <= 9; ++depth_steps)
    for (int other = 0; other <= 3; ++other)
      for (int flip = 0; flip < 2; ++flip) {
        const std::string objection = Check(depth_steps, ps::kTiming, other, flip != 0, &min_read_ahead);
        if (!objection.empty()) {
          std::fprintf(stderr, "%d steps, %d other memory operations, flip %d: %s\n", depth_steps, other, flip,
                       objection.c_str());
          ++g_failures;
          return;
        }
      }
  std::printf("paired schedule: every fragment is read at least %d matrix instructions ahead of its first use\n",
              min_read_ahead);
  EXPECT(min_read_ahead >= ps::kMinInstructionsFromReadToUse);
}

void ExpectObjection(const char* what, const ps::Timing& t) {
  bool objected = false;
  std::string first;
  for (int depth_steps = 1; depth_steps <= 6 && !objected; ++depth_steps) {
    first = Check(depth_steps, t, 0, false, nullptr);
    objected = !first.empty();
  }
  if (!objected) {
    std::fprintf(stderr, "the model accepts a schedule it must not accept: %s\n", what);
    ++g_failures;
  } else {
    std::printf("  altered (%s): %s\n", what, first.c_str());
  }
}

void TestAlteredSchedulesAreRefused() {
  const ps::Timing k = ps::kTiming;
  ps::Timing t;
  t = k; t.barrier1 = 8;
  ExpectObjection("barrier 1 in front of the step's last B reads", t);
  t = k; t.barrier1 = k.load_b0; t.load_b0 = k.barrier1;
  ExpectObjection("barrier 1 and the first B load exchanged", t);
  t = k; t.barrier2 = 60;
  ExpectObjection("barrier 2 (and the reads behind it) before the first half is over", t);
  t = k; t.barrier2 = 48;
  ExpectObjection("barrier 2 in the middle of the B loads", t);
  t = k; t.barrier1 = k.barrier2; t.barrier2 = k.barrier1;
  ExpectObjection("the two barriers exchanged", t);
  t = k; t.loads_left_at_barrier2 = 2 * ps::kLoads;
  ExpectObjection("the wait at barrier 2 leaves the next step's A loads outstanding", t);
  t = k; t.loads_left_at_barrier2 = ps::kLoads + 1;
  ExpectObjection("the wait at barrier 2 leaves one load too many outstanding", t);
  t = k; t.load_b0 = k.load_a0; t.load_a0 = k.load_b0;
  ExpectObjection("the A and B loads exchange their places", t);
  t = k; t.load_b_stride = k.load_a_stride; t.load_a_stride = k.load_b_stride;
  ExpectObjection("the A and B loads exchange their strides", t);
  t = k; t.load_b0 = k.barrier1 - 2;
  ExpectObjection("the first B load in front of barrier 1", t);
  t = k; t.load_a0 = k.barrier2 - 2;
  ExpectObjection("the first A load in front of barrier 2", t);
  t = k; t.load_a_stride = 9;
  ExpectObjection("the A loads do not fit the step", t);
  t = k; t.barrier1 = 44; t.load_b0 = 46; t.load_b_stride = 2;
  ExpectObjection("barrier 1 so late that A rows 4-7 are still being read when their slot is refilled", t);
}

}  // namespace

int main() {
  TestScheduleOfTheKernel();
  TestAlteredSchedulesAreRefused();
  if (g_failures) {
    std::fprintf(stderr, "paired_schedule_test: %d failure(s)\n", g_failures);
    return 1;
  }
  std::printf("paired_schedule_test: all passed\n");
  return 0;
}
