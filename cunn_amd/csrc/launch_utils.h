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

inline unsigned directGrid(long total, int block) {
  long b = (total + block - 1) / block;
  return (unsigned)(b > 262144 ? 262144 : (b < 1 ? 1 : b));
}

}  // namespace launch
