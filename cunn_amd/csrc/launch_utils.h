// Host-side launch policy shared by the tiled kernels.
#pragma once

#include <algorithm>
#include <cstddef>
#include <cstdint>

namespace launch {

// LDS per workgroup the band chooser aims for: with 160 KB of LDS per CU this
// keeps at least 6 workgroups (24 wavefronts) resident so that the load phase of
// one overlaps the compute/store phase of the others.
constexpr size_t kLdsBudget = 24 * 1024;
// Largest dynamic LDS a launch may ask for without opting in.
constexpr size_t kLdsMax = 64 * 1024;
// Workgroups wanted per launch: 256 CUs x 8 resident workgroups.
constexpr long kMinBlocks = 2048;

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
inline int roundUp(int a, int b) { return (a + b - 1) / b * b; }
inline int ceilDiv(int a, int b) { return (a + b - 1) / b; }

// Splits `produced` rows of a plane into equal bands. bytes(rows) is the LDS a
// band of that many rows needs. Returns false when a one-row band exceeds the
// LDS limit or the grid would not fit an int.
//
// The staging loaders keep kLoadBatch 16-byte loads per lane in flight; a band
// that needs one load more than a whole number of batches pays a full extra
// memory round trip for it. stagedFloats(rows) (optional) is the number of
// floats a band stages: bands are shrunk until they fit one batch of a
// 256-lane workgroup (4096 floats) when that still leaves >= 4 rows.
constexpr int kBatchFloats = 4 * 4 * 256;

template <typename BytesFn, typename StagedFn>
bool pickBand(int produced, long planes, BytesFn bytes, int *tileRows, int *tilesPerPlane, StagedFn stagedFloats,
              size_t budget = kLdsBudget) {
  if (produced < 1 || bytes(1) > kLdsMax) return false;
  int rows = produced;
  while (rows > 1 && bytes(rows) > budget) rows = (rows + 1) / 2;
  {
    int r = rows;
    while (r > 4 && stagedFloats(r) > (size_t)kBatchFloats) --r;
    if (stagedFloats(r) <= (size_t)kBatchFloats) rows = r;
  }
  while (rows > 4 && planes * ceilDiv(produced, rows) < kMinBlocks) rows = (rows + 1) / 2;
  int t = ceilDiv(produced, rows);
  rows = ceilDiv(produced, t);
  if (planes * t >= 0x7fffffffL) return false;
  *tileRows = rows;
  *tilesPerPlane = t;
  return true;
}

template <typename BytesFn>
bool pickBand(int produced, long planes, BytesFn bytes, int *tileRows, int *tilesPerPlane) {
  return pickBand(produced, planes, bytes, tileRows, tilesPerPlane, [](int) { return (size_t)0; });
}

// Work items of the kernels that convolve or pool staged planes from LDS: an item produces `rw` consecutive
// outputs of a row (7 or 4), `lp` lanes share a plane of LH rows, the window rows of output row r start at
// staged row r * CS. Chooses rw and the LDS row pitch (base .. base + 8, at most maxPitch): the pair with
// the fewest LDS read cycles = lane-steps (rounds over the lanes that share a plane x the columns of an
// item's window, (rw - 1) * CS + KS) x the most lanes of the first wave that read the same of the 64 banks at one
// window column. splitRagged: the items that end past the row run in a pass of their own. The last choice
// is kept per slot (0..7) and thread: the search costs a few microseconds.
struct ItemChoice {
  int rw, LW;
};
inline ItemChoice pickItem(int slot, int oW, int rows, int lp, int lpShift, int LH, int CS, int base, int maxPitch,
                           bool splitRagged, int KS = 3) {
  struct Key {
    int oW, rows, lp, LH, CS, base, maxPitch, split, KS, rw, LW;
  };
  static thread_local Key last[8] = {};
  Key &ch = last[slot & 7];
  if (ch.rw != 0 && ch.oW == oW && ch.rows == rows && ch.lp == lp && ch.LH == LH && ch.CS == CS && ch.base == base &&
      ch.maxPitch == maxPitch && ch.split == (int)splitRagged && ch.KS == KS)
    return ItemChoice{ch.rw, ch.LW};
  ch = Key{oW, rows, lp, LH, CS, base, maxPitch, (int)splitRagged, KS, 0, 0};
  long best = 0;
  for (int LW = base; LW <= std::min(base + 8, std::max(maxPitch, base)); ++LW)
    for (int r : {7, 4}) {
      const bool split = splitRagged && oW % r != 0 && oW > r;
      const int nseg = split ? oW / r : ceilDiv(oW, r), items = rows * nseg;
      unsigned char lanes[64] = {};
      int worst = 1;
      for (int tid = 0; tid < 64; ++tid) {
        const int pl = tid >> lpShift, it = tid & (lp - 1);
        if (it >= items) continue;
        const int row = it / nseg, c0 = (it - row * nseg) * r;
        worst = std::max(worst, (int)++lanes[(pl * LH * LW + row * CS * LW + c0 * CS) & 63]);
      }
      const long cost = (long)(ceilDiv(items, lp) + (split ? ceilDiv(rows, lp) : 0)) * ((r - 1) * CS + KS) * worst;  // window columns
      if (ch.rw == 0 || cost < best) best = cost, ch.rw = r, ch.LW = LW;
    }
  return ItemChoice{ch.rw, ch.LW};
}

inline unsigned directGrid(long total, int block) {
  long b = (total + block - 1) / block;
  return (unsigned)(b > 262144 ? 262144 : (b < 1 ? 1 : b));
}

}  // namespace launch
