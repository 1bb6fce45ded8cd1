// Shared machinery of the "strip" kernels (depthwise convolution and pooling):
// a lane produces 4 consecutive outputs of a row from a compile-time window of
// input columns held in LDS.
#pragma once

#include "device_utils.h"

namespace dev {

constexpr int kStripPadL = 4;  // fill cells in front of staged rows (>= pad, keeps rows 16-byte aligned)

// Offsets q = (d + PAD - k) / ST over positions d in [0, ND) and taps k in
// [0, KS) with (d + PAD - k) divisible by ST: the rows/columns of the strided
// (output-side) tensor, relative to floor(position / ST), whose windows cover
// input-side positions d. Used by the backward gathers.
template <int KS, int ST, int ND, int PAD>
struct TapSpan {
  static constexpr int lo() {
    int m = 1 << 20;
    for (int d = 0; d < ND; ++d)
      for (int k = 0; k < KS; ++k) {
        int t = d + PAD - k;
        if (t % ST == 0 && t / ST < m) m = t / ST;
      }
    return m;
  }
  static constexpr int hi() {
    int m = -(1 << 20);
    for (int d = 0; d < ND; ++d)
      for (int k = 0; k < KS; ++k) {
        int t = d + PAD - k;
        if (t % ST == 0 && t / ST > m) m = t / ST;
      }
    return m;
  }
};

// How the input band of a strip kernel is laid out in LDS and how a lane reads
// the NW = 3*ST + KS consecutive input columns its 4 outputs need.
//   ST == 1: plain rows, pitch W + 4, element (r, col) at r*pitch + 4 + col.
//   ST == 2: rows split into even and odd columns (loadRowsSplit), so the window
//            becomes two unit-stride runs; the pitch is skewed to 16 (mod 32)
//            floats so that consecutive output rows (2 input rows apart) start
//            32 banks apart.
// Cells outside the image hold `fill`. Requires W % 4 == 0 (ST == 1) or
// W % 8 == 0 (ST == 2) and PAD <= 4.
template <int KS, int ST, int PAD>
struct Strip {
  static constexpr int NW = 3 * ST + KS;
  __host__ __device__ static int pitch(int W) {
    return ST == 1 ? W + kStripPadL : (W + 8 - 16 + 31) / 32 * 32 + 16;
  }
  __host__ __device__ static size_t floats(int rows, int W) { return (size_t)rows * pitch(W) + kStripPadL; }
  __device__ static void stage(float *dst, const float *plane, int H, int W, int r0, int nRows, float fill = 0.f) {
    if (ST == 1)
      loadRowsPadded<true>(dst, plane, H, W, r0, nRows, pitch(W), kStripPadL, fill);
    else
      loadRowsSplit(dst, plane, H, W, r0, nRows, pitch(W), fill);
  }
  // The same staging in two halves: issue() starts the (at most kLoadBatch per lane) 16-byte
  // loads of a band into registers, commit() parks them in LDS in the layout stage() produces
  // (zero fill). Whatever else a workgroup needs before it can compute (taps, bias, derived
  // indices) is fetched between the two, while the band is in flight.
  // One batch only: nRows * W / 4 <= kLoadBatch * blockDim.x.
  struct InFlight {
    float4 v[kLoadBatch];
    int off[kLoadBatch];
  };
  __device__ static void issue(InFlight &f, const float *plane, int H, int W, int r0, int nRows) {
    const int tid = threadIdx.x, nt = blockDim.x;
    const int W4 = W >> 2, total = nRows * W4;
    const unsigned magic = magicOf(W4);
    const int p = pitch(W);
    const __amdgpu_buffer_rsrc_t rs = makeRsrc(plane, (long)H * W * 4);
#pragma unroll
    for (int u = 0; u < kLoadBatch; ++u) {
      const int i = u * nt + tid;
      const int r = fastDiv(i, magic), c4 = i - r * W4;
      const int gr = r0 + r;
      const bool ok = i < total && (unsigned)gr < (unsigned)H;
      f.off[u] = (i < total) ? r * p + kStripPadL + (ST == 1 ? (c4 << 2) : (c4 << 1)) : -1;
      f.v[u] = bufLoad4(rs, ok ? (gr * W + (c4 << 2)) * 4 : kBufOob);
    }
  }
  __device__ static void commit(float *dst, const InFlight &f, int W, int nRows) {
    const int tid = threadIdx.x, nt = blockDim.x;
    const int p = pitch(W);
    if (ST == 1) {
      for (int i = tid; i < (nRows + 1) * kStripPadL; i += nt) dst[(i >> 2) * p + (i & 3)] = 0.f;
#pragma unroll
      for (int u = 0; u < kLoadBatch; ++u)
        if (f.off[u] >= 0) *reinterpret_cast<float4 *>(dst + f.off[u]) = f.v[u];
    } else {
      const int oddOff = (W >> 1) + 8;
      for (int i = tid; i < nRows * 8 + 4; i += nt) {
        const int r = i >> 3, k = i & 7;
        dst[r * p + (k < 4 ? k : (W >> 1) + k)] = 0.f;
      }
#pragma unroll
      for (int u = 0; u < kLoadBatch; ++u)
        if (f.off[u] >= 0) {
          *reinterpret_cast<float2 *>(dst + f.off[u]) = make_float2(f.v[u].x, f.v[u].z);
          *reinterpret_cast<float2 *>(dst + f.off[u] + oddOff - 4) = make_float2(f.v[u].y, f.v[u].w);
        }
    }
  }
  // window element j is input column 4*ST*b4 - PAD + j
  static constexpr int half(int j) { return (j - PAD) % 2 == 0 ? (j - PAD) / 2 : (j - PAD - 1) / 2; }
  static constexpr bool even(int j) { return (j - PAD) % 2 == 0; }
  static constexpr int lo(bool e) {
    int m = 1 << 20;
    for (int j = 0; j < NW; ++j)
      if (even(j) == e && half(j) < m) m = half(j);
    return m;
  }
  static constexpr int hi(bool e) {
    int m = -(1 << 20);
    for (int j = 0; j < NW; ++j)
      if (even(j) == e && half(j) > m) m = half(j);
    return m;
  }
  __device__ static void loadWin(const float *__restrict__ row, int b4, int W, float (&win)[NW]) {
    if constexpr (ST == 1) {
      readWindow<0, NW, (kStripPadL - PAD) & 3, 4>(row + (kStripPadL - PAD) + b4 * 4, win);
    } else {
      constexpr int ELO = lo(true), EHI = hi(true), OLO = lo(false), OHI = hi(false);
      constexpr int NE = EHI - ELO + 1, NO = OHI - OLO + 1;
      float ew[NE], ow[NO];
      readWindow<0, NE, ((ELO % 4) + 4) % 4, 4>(row + 4 + b4 * 4 + ELO, ew);
      readWindow<0, NO, ((OLO % 4) + 4) % 4, 4>(row + (W >> 1) + 8 + b4 * 4 + OLO, ow);
#pragma unroll
      for (int j = 0; j < NW; ++j) win[j] = even(j) ? ew[half(j) - ELO] : ow[half(j) - OLO];
    }
  }
};

}  // namespace dev
