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

// Window of a stride-1 item: columns 4*b4 - PAD .. 4*b4 + 3 + PAD of a staged row, p pointing at column 4*b4.
// For loops in which the lanes of a wave hold consecutive items (b4, then the next row): the window is the
// lane's own 4 columns (one aligned 16-byte read) plus PAD columns on either side, and those are the last /
// first columns of the neighbouring lanes' reads - they come over the wave shift of the DPP unit instead of
// 4-byte LDS reads, which hit only 16 of the 64 banks (stride of 4 floats between lanes). The first and
// last group of a row take the zero border instead; lanes 0 and 63 of a wave have no neighbour on one
// side and read LDS (the cells around a row hold the border or the neighbouring group).
template <int PAD>
__device__ __forceinline__ void loadWindowShared(const float *__restrict__ p, int b4, int W4, float (&win)[4 + 2 * PAD]) {
  static_assert(PAD >= 1 && PAD <= 2, "kernel 3 or 5");
  const float4 c = *reinterpret_cast<const float4 *>(p);
  const int lane = threadIdx.x % kWave;
  auto fromLeft = [](float v) {   // value of lane - 1
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x138, 0xF, 0xF, true));
  };
  auto fromRight = [](float v) {  // value of lane + 1
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x130, 0xF, 0xF, true));
  };
  float l[2] = {fromLeft(c.z), fromLeft(c.w)};
  float r[2] = {fromRight(c.x), fromRight(c.y)};
  if (lane == 0) l[0] = p[-2], l[1] = p[-1];
  if (lane == kWave - 1) r[0] = p[4], r[1] = p[5];
  if (b4 == 0) l[0] = l[1] = 0.f;
  if (b4 == W4 - 1) r[0] = r[1] = 0.f;
#pragma unroll
  for (int j = 0; j < PAD; ++j) win[j] = l[2 - PAD + j], win[PAD + 4 + j] = r[j];
  win[PAD] = c.x, win[PAD + 1] = c.y, win[PAD + 2] = c.z, win[PAD + 3] = c.w;
}

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
  template <bool STREAM = false>
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
      f.v[u] = STREAM ? bufLoadStream4(rs, ok ? (gr * W + (c4 << 2)) * 4 : kBufOob)
                      : bufLoad4(rs, ok ? (gr * W + (c4 << 2)) * 4 : kBufOob);
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
  // The same window with its edge columns taken from the neighbouring lanes (see loadWindowShared), for rows
  // whose border cells hold zeros: a lane reads its own 4 columns (ST == 1) or its 4 even and 4 odd columns
  // (ST == 2) with aligned 16-byte reads only. nb4 = groups per row.
  __device__ static void loadWinShared(const float *__restrict__ row, int b4, int nb4, int W, float (&win)[NW]) {
    if constexpr (ST == 1) {
      static_assert(NW == 4 + 2 * PAD, "stride 1");
      loadWindowShared<PAD>(row + kStripPadL + b4 * 4, b4, nb4, win);
    } else {
      constexpr int ELO = lo(true), EHI = hi(true), OLO = lo(false), OHI = hi(false);
      static_assert(ELO >= -2 && OLO >= -2 && EHI <= 5 && OHI <= 5, "at most two columns from a neighbour");
      const float *pe = row + 4 + b4 * 4, *po = row + (W >> 1) + 8 + b4 * 4;
      const float4 e = *reinterpret_cast<const float4 *>(pe), o = *reinterpret_cast<const float4 *>(po);
      const int lane = threadIdx.x % kWave;
      const bool first = b4 == 0, last = b4 == nb4 - 1;
      // half-index k of the even (odd) columns: 0..3 own, negative from lane - 1, above 3 from lane + 1
      auto pick = [&](const float4 &v, const float *p, int k) -> float {
        const float own[4] = {v.x, v.y, v.z, v.w};
        if (k >= 0 && k < 4) return own[k];
        if (k < 0) {
          float t = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, own[4 + k]), 0x138, 0xF, 0xF, true));
          if (lane == 0) t = p[k];
          return first ? 0.f : t;
        }
        float t = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, own[k - 4]), 0x130, 0xF, 0xF, true));
        if (lane == kWave - 1) t = p[k];
        return last ? 0.f : t;
      };
#pragma unroll
      for (int j = 0; j < NW; ++j) win[j] = even(j) ? pick(e, pe, half(j)) : pick(o, po, half(j));
    }
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
