// CPU build of the look-back window logic (legion-ibp_amd/csrc/lookback.hpp) for
// tests/test_lookback.py: what wavefront 0 of tile `tile` computes from a frozen array of
// status words.  Returns 1 with the exclusive prefix of the tile, or 0 when a word it needs
// has not been published (the device code would read the window again).
#include "../legion-ibp_amd/csrc/lookback.hpp"

extern "C" int lookback_prefix(const uint64_t *status, int tile, int64_t *prefix_out, int *windows_out) {
  int64_t prefix = 0;
  int base = tile - 1, windows = 0;
  while (tile > 0) {
    uint64_t word[64], inc = 0, inv = 0;
    for (int lane = 0; lane < 64; ++lane) {
      const int j = base - lane;
      word[lane] = j >= 0 ? status[j] : (2ull << 32);  // before tile 0: an inclusive prefix of 0
      const unsigned flag = (unsigned)(word[lane] >> 32);
      if (flag == 2u) inc |= 1ull << lane;
      if (flag == 0u) inv |= 1ull << lane;
    }
    ++windows;
    const lmi::LookbackWindow w = lmi::lookback_window(inc, inv);
    if (w.wait) return 0;
    for (int lane = 0; lane < 64; ++lane)
      if ((w.take >> lane) & 1ull) prefix += (uint32_t)word[lane];
    if (w.done) break;
    base -= 64;
  }
  *prefix_out = prefix;
  if (windows_out) *windows_out = windows;
  return 1;
}

// The block -> (pipe, block of that pipe) mapping of launches that serve n pipes.
extern "C" void grid_row_of(unsigned block, unsigned n, int *row, int *bx) {
  const lmi::GridRow g = lmi::grid_row(block, n);
  *row = g.row;
  *bx = g.bx;
}
