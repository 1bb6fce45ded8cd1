// Pooling on runs of memory (plane_runs.h): square windows of compile-time size KS, stride ST and padding
// PAD without dilation, planes of any width. Included by pooling.hip inside its anonymous namespace.
//
//   forward  : the input run is parked in LDS as planes with a border of -FLT_MAX (max) or 0 (average), so
//              a window is scanned without bounds tests in the reference's order (rows outer, columns inner,
//              strict '>': lib/THCUNN/SpatialDilatedMaxPooling.cu:18-40; SpatialAveragePooling.cu:24-38);
//              a work item produces RW consecutive outputs of a row; values and (32-bit) argmax positions go
//              through linear LDS buffers and leave as 16-byte stores
//   backward : the gradOutput run (average: each element already divided by its window's divisor; max: with
//              the argmax positions beside it) is parked compactly with a border; a work item produces 4
//              consecutive gradInput elements of a row as the gather over the windows that reach them
//              (SpatialDilatedMaxPooling.cu:45-80, SpatialAveragePooling.cu:41-82), windows outer-to-inner
//              in the reference's order. Which window columns reach which of the 4 elements is known at
//              compile time (items start at multiples of 4, strides are 1 or 2).
#pragma once

#include "plane_runs.h"

// Divisor of the window at (ph, pw): its extent clipped to the padded image (count_include_pad) or to the
// image (lib/THCUNN/SpatialAveragePooling.cu:18-23, 35-37).
template <int KS, int ST, int PAD>
__device__ __forceinline__ float poolRunDivisor(int ph, int pw, int H, int W, bool includePad) {
  int hs = ph * ST - PAD, ws = pw * ST - PAD;
  int he = min(hs + KS, H + PAD), we = min(ws + KS, W + PAD);
  const int pool = (he - hs) * (we - ws);
  hs = max(hs, 0), ws = max(ws, 0), he = min(he, H), we = min(we, W);
  return includePad ? (float)pool : (float)((he - hs) * (we - ws));
}

// g: source = input plane (sH, sW), produced = pooled plane (oH, oW). LDS: staged planes | values | argmax.
template <int KS, int ST, int PAD, bool MAX, int RW>
__global__ void __launch_bounds__(dev::kBlock)
poolRunFwd(const float *__restrict__ in, float *__restrict__ out, long *__restrict__ indices, SmallGeom g, int secondFloats,
           bool includePad) {
  constexpr int NWIN = (RW - 1) * ST + KS;
  extern __shared__ float smem[];
  float *xs = smem, *os = smem + g.xsFloats;
  int *is = reinterpret_cast<int *>(os + secondFloats);
  const int tid = threadIdx.x;
  const SmallBand b = smallBand<KS, ST, 1, PAD>(g);
  const int oPlane = g.oH * g.oW;
  SmallRun run;
  smallIssue(run, in, (long)b.q0 * g.sH * g.sW + b.rLo * g.sW, b.np * b.nr * g.sW, g.srcFloats);
  smallFill(xs, g.xsFloats, MAX ? -FLT_MAX : 0.f);
  __syncthreads();
  smallScatter<1, PAD>(xs, run, b, g);
  __syncthreads();

  const int pl = tid >> g.lpShift, it0 = tid & (g.lp - 1);
  const long outFirst = (long)b.q0 * oPlane + b.o0 * g.oW;
  if (pl < b.np) {
    const float *xp = xs + pl * (g.LH * g.LW);
    float *op = os + (int)(outFirst & 3) + pl * oPlane;
    int *ip = is + (int)(outFirst & 1) + pl * oPlane;
    const int items = b.nOut * g.nseg;
    for (int it = it0; it < items; it += g.lp) {
      const int r = dev::fastDiv(it, g.magicSeg), c0 = (it - r * g.nseg) * RW;
      const int ph = b.o0 + r;
      float acc[RW];
      int code[RW];
#pragma unroll
      for (int q = 0; q < RW; ++q) acc[q] = MAX ? -FLT_MAX : 0.f, code[q] = -1;
#pragma unroll
      for (int kh = 0; kh < KS; ++kh) {
        const float *row = xp + (r * ST + kh) * g.LW + c0 * ST;
        float win[NWIN];
#pragma unroll
        for (int j = 0; j < NWIN; ++j) win[j] = row[j];
#pragma unroll
        for (int kw = 0; kw < KS; ++kw)
#pragma unroll
          for (int q = 0; q < RW; ++q) {
            const float v = win[q * ST + kw];
            if (MAX) {
              if (v > acc[q]) acc[q] = v, code[q] = kh * KS + kw;
            } else {
              acc[q] += v;
            }
          }
      }
#pragma unroll
      for (int q = 0; q < RW; ++q)
        if (c0 + q < g.oW) {
          if (MAX) {
            const int kh = code[q] / KS, kw = code[q] - kh * KS;
            op[r * g.oW + c0 + q] = acc[q];
            ip[r * g.oW + c0 + q] =
                (code[q] < 0 ? -1 : (ph * ST - PAD + kh) * g.sW + (c0 + q) * ST - PAD + kw) + TH_INDEX_BASE;
          } else {
            op[r * g.oW + c0 + q] = acc[q] / poolRunDivisor<KS, ST, PAD>(ph, c0 + q, g.sH, g.sW, includePad);
          }
        }
    }
  }
  __syncthreads();
  const int produced = b.np * b.nOut * g.oW;
  smallStoreRun(out, outFirst, os, produced);
  if (MAX) smallStoreIdxRun(indices, outFirst, is, produced);
}

// Backward geometry: gradInput element h receives from the windows ph with ph * ST - PAD <= h < ph * ST - PAD + KS,
// at most NC = ceil(KS / ST) of them, the first one floor((h + PAD - KS) / ST) + 1 >= -BT.
template <int KS, int ST, int PAD>
struct PoolReach {
  static constexpr int NC = (KS + ST - 1) / ST;
  static constexpr int BT = (KS - PAD + ST - 1) / ST - 1;   // border in front of window 0
  static constexpr int kShift = PAD - KS + (BT + 1) * ST;  // >= 0
  // first window that can reach element h, counted from window -BT
  static __host__ __device__ constexpr int first(int h) { return (h + kShift) / ST; }
  // does the window `first(h) + j` (of an element h with h % ST == phase % ST) reach it?
  static __host__ __device__ constexpr bool reaches(int phase, int j) {
    return ((phase + kShift) / ST + j - BT) * ST <= phase + PAD;
  }
};

// What one workgroup of the backward kernel works on: gradInput rows [o0, o0 + nOut) of planes q0 .. q0 + np - 1;
// gradOutput rows [rLo, rLo + nr) are loaded; window ph sits in LDS row ph + BT - R0.
struct PoolBwdBand {
  int q0, np, o0, nOut, rLo, nr, R0;
};
template <int KS, int ST, int PAD>
__device__ __forceinline__ PoolBwdBand poolBwdBand(const SmallGeom &g) {
  using R = PoolReach<KS, ST, PAD>;
  PoolBwdBand b;
  if (g.P > 1) {
    b.q0 = blockIdx.x * g.P, b.np = min(g.P, g.planes - b.q0);
    b.o0 = 0, b.nOut = g.oH, b.rLo = 0, b.nr = g.sH, b.R0 = 0;
  } else {
    b.q0 = dev::fastDiv(blockIdx.x, g.magicBands), b.np = 1;
    const int band = blockIdx.x - b.q0 * g.bands;
    b.o0 = band * g.rowsPerBand, b.nOut = min(g.rowsPerBand, g.oH - b.o0);
    b.R0 = R::first(b.o0);
    b.rLo = max(0, b.R0 - R::BT);
    const int rHi = min(g.sH - 1, R::first(b.o0 + b.nOut - 1) + R::NC - 1 - R::BT);
    b.nr = max(0, rHi - b.rLo + 1);
  }
  return b;
}

// g: source = gradOutput plane (sH, sW), produced = gradInput plane (oH, oW); (LH, LW): staged plane with
// its border. LDS: staged gradOutput | staged argmax (max only) | gradInput run.
template <int KS, int ST, int PAD, bool MAX>
__global__ void __launch_bounds__(dev::kBlock)
poolRunBwd(const float *__restrict__ gradOut, const long *__restrict__ indices, float *__restrict__ gradIn, SmallGeom g,
           bool includePad) {
  using R = PoolReach<KS, ST, PAD>;
  constexpr int NC = R::NC, BT = R::BT;
  // element q of an item (columns c0 .. c0 + 3, c0 % 4 == 0) is first reached by window column c0 / ST - BT + O(q)
  constexpr int O0 = R::first(0), O3 = R::first(3);
  constexpr int NWIN = O3 - O0 + NC;
  extern __shared__ float smem[];
  float *gs = smem;
  int *is = reinterpret_cast<int *>(smem + g.xsFloats);
  float *os = smem + (MAX ? 2 : 1) * g.xsFloats;
  const int tid = threadIdx.x;
  const PoolBwdBand b = poolBwdBand<KS, ST, PAD>(g);
  const int sPlane = b.nr * g.sW, lPlane = g.LH * g.LW;
  const long srcFirst = (long)b.q0 * g.sH * g.sW + b.rLo * g.sW;
  const int srcCount = b.np * b.nr * g.sW;
  SmallRun run;
  SmallIdxRun irun;
  smallIssue(run, gradOut, srcFirst, srcCount, g.srcFloats);
  if (MAX) smallIssueIdx<true>(irun, indices, srcFirst, srcCount, g.srcFloats);  // their only use
  smallZero(gs, g.xsFloats);
  if (MAX) smallFill(reinterpret_cast<float *>(is), g.xsFloats, __int_as_float(-1));
  __syncthreads();
  // park the run: source (p, r, c) at plane p, LDS row r + BT - R0, column c + BT
  const int rowBase = b.rLo + BT - b.R0;
#pragma unroll
  for (int u = 0; u < dev::kLoadBatch; ++u) {
    const int e = (u * dev::kBlock + tid) * 4;
    if (e < run.lead + run.count) {
      const int skip = max(run.lead - e, 0);
      const int i0 = e + skip - run.lead;
      int p = g.P > 1 ? dev::fastDiv(i0, g.magicSPlane) : 0;
      const int rem = i0 - p * sPlane;
      int h = dev::fastDiv(rem, g.magicSW);
      int w = rem - h * g.sW;
      const float vals[4] = {run.v[u].x, run.v[u].y, run.v[u].z, run.v[u].w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if (k >= skip && i0 + k - skip < run.count) {
          float v = vals[k];
          if (!MAX) v = v / poolRunDivisor<KS, ST, PAD>(b.rLo + h, w, g.oH, g.oW, includePad);
          gs[p * lPlane + (h + rowBase) * g.LW + w + BT] = v;
          if (++w == g.sW) {
            w = 0;
            if (++h == b.nr) h = 0, ++p;
          }
        }
      }
    }
  }
  if (MAX) {
#pragma unroll
    for (int u = 0; u < 2 * dev::kLoadBatch; ++u) {
      const int e = (u * dev::kBlock + tid) * 2;
      if (e < irun.lead + irun.count) {
        const long vals[2] = {irun.v[u].x, irun.v[u].y};
#pragma unroll
        for (int k = 0; k < 2; ++k) {
          const int i = e + k - irun.lead;
          if (i >= 0 && i < irun.count) {
            const int p = g.P > 1 ? dev::fastDiv(i, g.magicSPlane) : 0;
            const int rem = i - p * sPlane;
            const int h = dev::fastDiv(rem, g.magicSW), w = rem - h * g.sW;
            is[p * lPlane + (h + rowBase) * g.LW + w + BT] = (int)(vals[k] - TH_INDEX_BASE);
          }
        }
      }
    }
  }
  __syncthreads();

  const int pl = tid >> g.lpShift, it0 = tid & (g.lp - 1);
  const int oPlane = g.oH * g.oW;
  const long outFirst = (long)b.q0 * oPlane + b.o0 * g.oW;
  if (pl < b.np) {
    const float *gp = gs + pl * lPlane;
    const int *ixp = is + pl * lPlane;
    float *op = os + (int)(outFirst & 3) + pl * oPlane;
    const int items = b.nOut * g.nseg;  // nseg = ceil(oW / 4)
    for (int it = it0; it < items; it += g.lp) {
      const int r = dev::fastDiv(it, g.magicSeg), c0 = (it - r * g.nseg) * 4;
      const int h = b.o0 + r;
      const int row0 = R::first(h) - b.R0;
      const int col0 = c0 / ST + O0;  // first LDS column of the item
      const int target = h * g.oW + c0;
      float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < NC; ++j) {
        // windows beyond the last one that reaches row h hold other rows' values (or the border)
        const bool rowReached = (R::first(h) + j - BT) * ST <= h + PAD;
        float gw[NWIN];
        int iw[NWIN];
#pragma unroll
        for (int k = 0; k < NWIN; ++k) {
          gw[k] = gp[(row0 + j) * g.LW + col0 + k];
          if (MAX) iw[k] = ixp[(row0 + j) * g.LW + col0 + k];
        }
#pragma unroll
        for (int jc = 0; jc < NC; ++jc)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            if (!R::reaches(q, jc)) continue;  // compile time: c0 is a multiple of ST
            const int k = R::first(q) - O0 + jc;
            if (MAX)
              acc[q] += iw[k] == target + q ? gw[k] : 0.f;
            else
              acc[q] += rowReached ? gw[k] : 0.f;
          }
      }
#pragma unroll
      for (int q = 0; q < 4; ++q)
        if (c0 + q < g.oW) op[r * g.oW + c0 + q] = acc[q];
    }
  }
  __syncthreads();
  smallStoreRun(gradIn, outFirst, os, b.np * b.nOut * g.oW);
}
