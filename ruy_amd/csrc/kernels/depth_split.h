// The arithmetic of the depth split, shared by the kernels, the host-side
// planner and a host-only model test: which depth steps a part walks, when a
// split has no empty part, and who does the write-back.
//
// Protocol (the small tiles; the largest int8 tile adds to it, see below). A launch carries `parts`
// workgroups per destination tile. Each walks its part of the depth steps,
// stores its raw accumulators to its slice of a scratch buffer, waits until
// those stores have been performed, and then adds 1 to the tile's arrival
// counter; the workgroup whose add returns parts - 1 is the last to arrive: it
// sets the counter back to 0 for the next launch, reads all slices in the order
// of the parts (so a floating-point sum does not depend on who was last) and
// runs the write-back. Nobody waits for anybody, so a launch cannot hang.
//
// What orders the accesses on the device. The slices and the counter are
// accessed with agent-scope atomic operations only (relaxed): on gfx942/gfx950
// those are performed at the point where all XCDs of the device agree (they
// carry the sc1 bit and do not linger in an XCD's L2). A workgroup issues its
// counter add only after s_waitcnt vmcnt(0) has returned for its slice stores,
// i.e. after they have been performed there, and after a workgroup barrier, so
// every wave's stores are covered; the last arriver issues its slice loads
// only after the add has returned its value (the loads depend on it through
// the branch and are issued behind it in program order). These are the two
// properties the compiler's own agent-scope release and acquire sequences
// rest on (release: write back, s_waitcnt vmcnt(0), then the atomic; acquire:
// the atomic, then invalidate): the kernel uses per-access sc1 operations
// where those sequences write back and invalidate whole caches.
#ifndef RUY_AMD_CSRC_KERNELS_DEPTH_SPLIT_H_
#define RUY_AMD_CSRC_KERNELS_DEPTH_SPLIT_H_

#if defined(__HIPCC__)
#define RUYAMD_HOST_DEVICE __host__ __device__
#else
#define RUYAMD_HOST_DEVICE
#endif

namespace ruyamd {
namespace depth_split {

// Depth steps per part when `steps` steps are dealt to `parts` parts.
RUYAMD_HOST_DEVICE inline int StepsPerPart(int steps, int parts) { return (steps + parts - 1) / parts; }

// First step of part `index`.
RUYAMD_HOST_DEVICE inline int FirstStep(int steps, int parts, int index) {
  return index * StepsPerPart(steps, parts);
}

// Number of steps of part `index` (0 if the part lies past the end).
RUYAMD_HOST_DEVICE inline int StepCount(int steps, int parts, int index) {
  const int per = StepsPerPart(steps, parts);
  const int left = steps - index * per;
  return left < 0 ? 0 : (left < per ? left : per);
}

// Every part has at least one step (what a launch requires).
RUYAMD_HOST_DEVICE inline bool NoEmptyPart(int steps, int parts) {
  return parts >= 1 && (parts - 1) * StepsPerPart(steps, parts) < steps;
}

// The largest number of parts <= `wanted` that leaves no part empty with
// the steps dealt as above.
RUYAMD_HOST_DEVICE inline int PartsWithoutEmpty(int steps, int wanted) {
  if (wanted < 1 || steps < 1) return 1;
  const int per = StepsPerPart(steps, wanted);
  return (steps + per - 1) / per;
}

// `previous`: what this workgroup's add on the tile's arrival counter returned.
RUYAMD_HOST_DEVICE inline bool IsLastArrival(unsigned previous, int parts) {
  return previous == static_cast<unsigned>(parts - 1);
}

// ---- The split of the largest int8 tile (256x256, 8 x 8 blocks of 16x16 a wave) ----
//
// Adding up the parts costs in proportion to the tile's area, and here a part
// is 256 KiB: one workgroup that reads all the others' parts and then writes
// the whole tile back is busy for longer than the split saves. So the parts
// share that work as well. Every workgroup stores its accumulators as above
// and counts itself in; then it waits, a bounded number of looks at the
// counter, until all parts of its tile have arrived. The tile's destination
// columns are dealt to the parts (block columns index * 8 / parts ...: every
// wave of the workgroup owns those of its 8 block columns): a workgroup that
// has seen everybody arrive claims its columns (one bit per part in a word of
// claims, set with an atomic OR whose return value says who was first), adds
// the other parts' accumulators of those columns to its own and writes those
// columns back. Parts of a tile take the same time, so the wait is short and
// all parts read and write side by side.
//
// Nobody may wait without bound (the other parts' workgroups may not be
// running: a device shared with somebody else's kernels, a grid larger than
// the device). A workgroup whose looks are used up leaves without claiming. The
// last one to arrive never waits; after its own columns it claims whatever
// nobody has claimed and finishes those columns too: every part's full set of
// accumulators is in memory, its own are still in its registers. With a limit
// of zero looks this is the plain protocol above.
//
// Every workgroup counts itself out when it leaves; the last one out sets the
// tile's three words back to zero (nobody reads them any more).
constexpr int kLargeWordsPerTile = 4;  // arrivals, claims, exits, one unused
constexpr int kArrivals = 0, kClaims = 1, kExits = 2;
constexpr int kLargeBlockColumns = 8;
constexpr int kLargeMaxParts = 8;

// The parts must deal out the block columns evenly.
RUYAMD_HOST_DEVICE inline bool LargePartsAllowed(int parts) { return parts == 2 || parts == 4 || parts == 8; }
// The largest allowed number of parts <= wanted that leaves no part without a
// depth step (1: no split).
RUYAMD_HOST_DEVICE inline int LargeParts(int steps, int wanted) {
  for (int parts = kLargeMaxParts; parts >= 2; parts /= 2)
    if (parts <= wanted && NoEmptyPart(steps, parts)) return parts;
  return 1;
}
RUYAMD_HOST_DEVICE inline int LargeColumnsPerPart(int parts) { return kLargeBlockColumns / parts; }
// Whether the claim of part `index` succeeded: `claims_before` is what the
// atomic OR of ClaimBit(index) into the tile's claims returned.
RUYAMD_HOST_DEVICE inline unsigned ClaimBit(int index) { return 1u << index; }
RUYAMD_HOST_DEVICE inline bool ClaimSucceeded(unsigned claims_before, int index) {
  return (claims_before & ClaimBit(index)) == 0;
}

// Which tile and part a workgroup of such a launch takes. The hardware deals
// workgroups to the device's 8 XCDs round-robin by their linear number, and
// every XCD has an L2 of its own: an XCD gets workgroups of one depth part
// only, and a contiguous run of the tile order, so that the operand panels in
// its L2 serve all of them. (Parts of one tile share no operand bytes.)
// `tile` == total_tiles: a workgroup without work (the grid is rounded up).
struct LargeSplitWork {
  int tile;
  int part;
};
RUYAMD_HOST_DEVICE inline LargeSplitWork LargeSplitWorkOf(int linear_workgroup, int total_tiles, int parts) {
  const int xcd = linear_workgroup & 7, place = linear_workgroup >> 3;
  const int xcds_per_part = 8 / parts;
  const int tiles_per_xcd = (total_tiles + xcds_per_part - 1) / xcds_per_part;
  LargeSplitWork w;
  w.part = xcd % parts;
  w.tile = place < tiles_per_xcd ? (xcd / parts) * tiles_per_xcd + place : total_tiles;
  if (w.tile > total_tiles) w.tile = total_tiles;
  return w;
}

}  // namespace depth_split
}  // namespace ruyamd

#endif  // RUY_AMD_CSRC_KERNELS_DEPTH_SPLIT_H_
