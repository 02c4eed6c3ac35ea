// Window logic of the decoupled look-back scan, free of device intrinsics so that a CPU
// build can test it.  A wavefront looks at the 64 tiles before its own at once: lane L
// reads the status word of tile base - L (lane 0 is the nearest predecessor; tiles before
// tile 0 read as "inclusive prefix 0").  `inc` has bit L set when that word carries an
// inclusive prefix, `inv` when it is not published yet; every other word carries the
// tile's own sum.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define LMI_HD __host__ __device__
#else
#define LMI_HD
#endif

namespace lmi {

struct LookbackWindow {
  int first_inc;   // nearest lane whose word is an inclusive prefix; 63 when none is
  uint64_t take;   // lanes whose values this step adds up: 0 .. first_inc
  bool wait;       // one of those lanes has not published yet: read the window again
  bool done;       // an inclusive prefix was reached: the sum is complete after this step
};

LMI_HD inline LookbackWindow lookback_window(uint64_t inc, uint64_t inv) {
  LookbackWindow w;
  w.first_inc = inc ? __builtin_ctzll(inc) : 63;
  w.take = (w.first_inc >= 63) ? ~0ull : ((1ull << (w.first_inc + 1)) - 1ull);
  w.wait = (inv & w.take) != 0;
  w.done = inc != 0;
  return w;
}

// Which pipe a block of a launch that serves n pipes works on, and which of that pipe's blocks it
// is.  Each aligned run of n blocks holds one block of every pipe (block b is its pipe's block
// b / n), so every pipe's blocks are dispatched in step and in ascending order, which the
// look-back relies on.  The pipe a place in the run serves rotates from run to run: workgroups
// go to the 8 XCDs round robin (block b to XCD b % 8), so a plain b % n would pin a pipe to 8 / n
// of them when n divides 8 (one XCD per pipe at n = 8) and the pipes would finish unevenly.
// Rotating by the octet (n | 8) or by the run (otherwise) takes every pipe over all the XCDs.
struct GridRow {
  int row;  // pipe
  int bx;   // the pipe's own block index
};

LMI_HD inline GridRow grid_row(unsigned block, unsigned n) {
  const unsigned rot = (8u % n == 0) ? block / 8u : block / n;
  return GridRow{(int)((block % n + rot) % n), (int)(block / n)};
}

}  // namespace lmi
