// The instruction schedule of one ring step of the largest int8 tile (the
// "paired" schedule of mfma_gemm.h), as compile-time arithmetic that the
// kernel and a host-only model test share: which accumulator block and which
// fragment registers matrix instruction n uses, which fragment is read from
// LDS behind it, which direct-to-LDS load is issued behind it, where the two
// workgroup barriers and the wait for the loads stand.
//
// A wave holds 8 x 8 accumulator blocks of 16x16 and, of a 128-byte ring step,
// the fragments of both 64-byte depth halves at once: fa[half][block row] and
// fb[half][block column], 16 registers of four dwords each. A ring step is 64
// pairs of matrix instructions (the two depth halves on one accumulator block,
// back to back). There is no second set of fragment registers, so a register
// can only be read anew once the last pair that needs its old value has been
// issued, and the new value must be there when the first pair of the next
// step that needs it comes up. The walk over the blocks that makes room for
// that: two halves of four block rows, each half column by column (four pairs
// a column, down one column and up the next), the second half in the opposite
// column order of the first, and the next ring step's first half in the column
// order of this one's second half.
//
// The ring has two slots; the slot of step kt is kt mod 2 and is refilled with
// step kt + 2 during step kt: the B half behind barrier 1 (every wave has read
// the step's last B fragments by then), the A half behind barrier 2 (A rows
// 4-7 have been read). In front of barrier 2 every wave waits for all its loads
// but the eight it has just issued: everything of step kt + 1 is in LDS when
// the barrier opens, and the reads of step kt + 1 start behind it.
#ifndef RUY_AMD_CSRC_KERNELS_PAIRED_SCHEDULE_H_
#define RUY_AMD_CSRC_KERNELS_PAIRED_SCHEDULE_H_

namespace ruyamd {
namespace paired_schedule {

constexpr int kBlocks = 8;          // block rows and block columns of a wave
constexpr int kInstructions = 128;  // matrix instructions of a ring step
constexpr int kHalf = kInstructions / 2;
constexpr int kLoads = 8;           // direct-to-LDS loads per operand, wave and ring step

// Who fills and who reads which part of a ring slot. An operand's half of a
// slot is 256 tile rows of 128 bytes. Load `index` of wave w fills the eight
// rows from FirstRowOfLoad(w, index); wave w = 2 * wave_m + wave_n reads its A
// fragments from rows 128 * wave_m on and its B fragments from rows 128 *
// wave_n on, 16 rows a block: every fragment a wave reads was brought in by
// two loads, mostly of another wave.
constexpr int kWaves = 4;
constexpr int kRowsPerLoad = 8;
constexpr int kRowsPerBlock = 16;
constexpr int FirstRowOfLoad(int wave, int index) { return (wave * kLoads + index) * kRowsPerLoad; }
constexpr int FirstRowOfFragment(int wave, bool is_a, int index) {
  return (is_a ? wave / 2 : wave % 2) * kBlocks * kRowsPerBlock + index * kRowsPerBlock;
}

// Where in a ring step the barriers and the loads stand.
struct Timing {
  // Barrier 1 stands in front of this instruction.
  int barrier1;
  // Barrier 2 stands in front of this one, behind a wait that leaves this many
  // of the wave's most recent loads outstanding.
  int barrier2;
  int loads_left_at_barrier2;
  // The loads of step kt + 2: B load l behind instruction load_b0 + l *
  // load_b_stride, A load l behind load_a0 + l * load_a_stride (a
  // direct-to-LDS load keeps the CU's address unit busy for 16 cycles, so they
  // must not bunch).
  int load_b0, load_b_stride;
  int load_a0, load_a_stride;
};
constexpr Timing kTiming{/*barrier1=*/24, /*barrier2=*/64, /*loads_left_at_barrier2=*/8,
                         /*load_b0=*/26,  /*load_b_stride=*/5,
                         /*load_a0=*/66,  /*load_a_stride=*/6};

// The block column at position `cp` (0..7) of half `h` of a ring step of the given parity.
constexpr int ColumnAt(int parity, int h, int cp) { return (parity ^ h) == 0 ? cp : kBlocks - 1 - cp; }

struct Mma {
  int half;       // depth half: fa[half][row], fb[half][col]
  int row, col;   // accumulator block
  // The step's first pair on fa[.][row] / on fb[.][col] (where uint8 data is
  // flipped to int8 in the registers, both depth halves at once).
  bool first_use_of_a;
  bool first_use_of_b;
};
constexpr Mma MmaAt(int parity, int n) {
  const int pair = n / 2;
  const int h = pair / 32;
  const int cp = pair % 32 / 4;
  const int rp = pair % 4;
  return Mma{n % 2, 4 * h + (cp % 2 == 0 ? rp : 3 - rp), ColumnAt(parity, h, cp), cp == 0, h == 0 && rp == 0};
}

// The fragment read that is issued behind instruction n (at most one).
struct Read {
  bool valid;
  bool is_a;
  bool of_next_step;  // from the other ring slot: the step to come
  int half;
  int index;          // block row (A) or block column (B)
};
constexpr Read ReadBehind(int parity, int n, Timing t = kTiming) {
  // The last four columns of this step's first half (needed from instruction 32 on).
  if (n < 16 && n % 2 == 0) return Read{true, false, false, n / 2 % 2, ColumnAt(parity, 0, 4 + n / 4)};
  // A rows 4-7 of this step (needed from instruction 64 on), behind barrier 1.
  if (n > t.barrier1 && n < t.barrier1 + 25 && (n - t.barrier1) % 3 == 1)
    return Read{true, true, false, (n - t.barrier1 - 1) / 3 % 2, 4 + (n - t.barrier1 - 1) / 6};
  // A rows 0-3 of the next step, behind barrier 2.
  if (n > t.barrier2 && n < t.barrier2 + 17 && (n - t.barrier2) % 2 == 1)
    return Read{true, true, true, (n - t.barrier2 - 1) / 2 % 2, (n - t.barrier2 - 1) / 4};
  // The first four columns of the next step's first half, as this step's
  // second half is done with them, one column every eight instructions.
  if (n >= kHalf + 8 && n < kHalf + 40 && (n % 8 == 0 || n % 8 == 2))
    return Read{true, false, true, n % 8 / 2, ColumnAt(parity, 1, (n - kHalf - 8) / 8)};
  return Read{false, false, false, 0, 0};
}

// The load of step kt + 2 that is issued behind instruction n.
struct Load {
  bool valid;
  bool is_b;
  int index;  // 0 .. kLoads - 1
};
constexpr Load LoadBehind(int n, Timing t = kTiming) {
  if (n >= t.load_b0 && n < t.barrier2 && (n - t.load_b0) % t.load_b_stride == 0 &&
      (n - t.load_b0) / t.load_b_stride < kLoads)
    return Load{true, true, (n - t.load_b0) / t.load_b_stride};
  if (n >= t.load_a0 && n < kInstructions && (n - t.load_a0) % t.load_a_stride == 0 &&
      (n - t.load_a0) / t.load_a_stride < kLoads)
    return Load{true, false, (n - t.load_a0) / t.load_a_stride};
  return Load{false, false, 0};
}

// What is in the fragment registers before the first ring step: both depth
// halves of A rows 0-3 and of the first four B columns of step 0 (positions
// 0-3 of ColumnAt(0, 0, .)). In front of these reads the loads of steps 0 and
// 1 have been issued (B then A, step by step), all but the last
// kLoadsLeftBeforeFirstStep of them awaited, and a barrier passed.
constexpr int kRowsReadAhead = 4;
constexpr int kColumnsReadAhead = 4;
constexpr int kLoadsLeftBeforeFirstStep = 2 * kLoads;

// A fragment register is read at least this many matrix instructions ahead of
// the first one that uses it (an LDS read of 16 bytes a lane takes a few
// hundred cycles to come back when all four waves read at once; a matrix
// instruction takes 16 on its own and 8 as the second of a pair).
constexpr int kMinInstructionsFromReadToUse = 24;

}  // namespace paired_schedule
}  // namespace ruyamd

#endif  // RUY_AMD_CSRC_KERNELS_PAIRED_SCHEDULE_H_
