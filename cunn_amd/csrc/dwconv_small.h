// Depthwise convolution on runs of memory: several whole small planes (the 28x28 / 14x14 / 7x7 stages
// of a network) or a band of rows of one larger plane of any width per workgroup. Included by dwconv.hip
// inside its anonymous namespace.
//
// Planes are contiguous in memory and so are the rows of a band, so what a workgroup reads is one
// contiguous run of floats: it is fetched with 16-byte loads in memory order (from the 16-byte boundary
// at or below its first element - no alignment or multiple-of-4 requirement on the extents), scattered
// into zero-bordered planes in LDS, convolved from LDS with no bounds test, and the results go through a
// linear LDS buffer so that they leave as 16-byte streaming stores in memory order as well.
//
//   forward            : source = input,      staged 1:1,            compute stride = conv stride
//   gradInput          : source = gradOutput, staged zero-dilated by the conv stride, compute stride 1,
//                        taps flipped - the transpose of a strided convolution as a stride-1 convolution
//   accGradParameters  : input staged 1:1, gradOutput linear; k*k+1 sums reduced over the lanes of a
//                        plane, one partial per (plane, band, tap) for the second-stage fold
//
// With several planes per workgroup the lanes are dealt to planes in fixed groups of kBlock / P (a power
// of two), so a lane keeps the taps of one channel in registers. Depth multiplier 1, square kernel 3 or
// 5, stride 1 or 2, padding k / 2.
#pragma once

#include "plane_runs.h"

// dst planes = bias + conv(src planes): CS = stride of the computation, DS = dilation of the staging,
// FLIP = taps reversed (gradInput), RW = consecutive outputs of a row per work item.
template <int KS, int CS, int DS, bool FLIP, int RW>
__global__ void __launch_bounds__(dev::kBlock)
dwSmallConv(const float *__restrict__ src, const float *__restrict__ weight, Strides4 ws, const float *__restrict__ bias,
            Strides2 bs, float *__restrict__ dst, SmallGeom g) {
  constexpr int PAD = KS / 2, NWIN = (RW - 1) * CS + KS;
  extern __shared__ float smem[];
  float *xs = smem, *os = smem + g.xsFloats;
  const int tid = threadIdx.x;
  const SmallBand b = smallBand<KS, CS, DS>(g);
  const int oPlane = g.oH * g.oW;
  SmallRun run;
  smallIssue(run, src, (long)b.q0 * g.sH * g.sW + b.rLo * g.sW, b.np * b.nr * g.sW, g.srcFloats);

  // this lane's plane and its taps, fetched while the run is in flight
  const int pl = tid >> g.lpShift, it0 = tid & (g.lp - 1);
  const bool live = pl < b.np;
  float w[KS * KS];
  float bv = 0.f;
  {
    const int q = b.q0 + (live ? pl : 0);
    const int c = q - dev::fastDiv(q, g.magicC) * g.C;
    const float *wp = weight + c * ws.s1;
#pragma unroll
    for (int kh = 0; kh < KS; ++kh)
#pragma unroll
      for (int kw = 0; kw < KS; ++kw)
        w[FLIP ? (KS - 1 - kh) * KS + (KS - 1 - kw) : kh * KS + kw] = wp[kh * ws.s2 + kw * ws.s3];
    if (bias) bv = bias[c * bs.s1];
  }
  smallZero(xs, g.xsFloats);
  __syncthreads();
  smallScatter<DS, PAD>(xs, run, b, g);
  __syncthreads();

  const long outFirst = (long)b.q0 * oPlane + b.o0 * g.oW;  // first element of the produced run
  if (live) {
    const float *xp = xs + pl * (g.LH * g.LW);
    float *op = os + (int)(outFirst & 3) + pl * oPlane;  // (several planes: whole planes, o0 = 0)
    const int items = b.nOut * g.nseg;
    for (int it = it0; it < items; it += g.lp) {
      const int r = dev::fastDiv(it, g.magicSeg), c0 = (it - r * g.nseg) * RW;
      float acc[RW];
#pragma unroll
      for (int q = 0; q < RW; ++q) acc[q] = bv;
#pragma unroll
      for (int kh = 0; kh < KS; ++kh) {
        const float *row = xp + (r * CS + kh) * g.LW + c0 * CS;
        float win[NWIN];
#pragma unroll
        for (int j = 0; j < NWIN; ++j) win[j] = row[j];
#pragma unroll
        for (int kw = 0; kw < KS; ++kw)
#pragma unroll
          for (int q = 0; q < RW; ++q) acc[q] = fmaf(win[q * CS + kw], w[kh * KS + kw], acc[q]);
      }
#pragma unroll
      for (int q = 0; q < RW; ++q)
        if (c0 + q < g.oW) op[r * g.oW + c0 + q] = acc[q];
    }
  }
  __syncthreads();
  smallStoreRun(dst, outFirst, os, b.np * b.nOut * g.oW);
}

// partial[((n * bands + band) * C + c) * TP + t] = sum over the band of plane (n, c) of gradOutput * input
// window element t (t = kh * KS + kw; t = KS * KS: the bias, sum of gradOutput), T = KS * KS + 1, TP = T rounded
// up to 16: the sums of one (plane, band) are one aligned run, written as 16-byte groups (padding zero).
template <int KS, int ST, int RW>
__global__ void __launch_bounds__(dev::kBlock)
dwSmallAccGrad(const float *__restrict__ in, const float *__restrict__ gradOut, float *__restrict__ partial, SmallGeom g) {
  constexpr int PAD = KS / 2, NWIN = (RW - 1) * ST + KS, T = KS * KS + 1;
  extern __shared__ float smem[];
  __shared__ float red[dev::kBlock / dev::kWave][T];
  float *xs = smem, *gs = smem + g.xsFloats;
  const int tid = threadIdx.x;
  const SmallBand b = smallBand<KS, ST, 1>(g);
  const int oPlane = g.oH * g.oW;
  const long gFirst = (long)b.q0 * oPlane + b.o0 * g.oW;
  SmallRun run, grun;
  // (both tensors are read here for the last time in a training step)
  smallIssue<true>(run, in, (long)b.q0 * g.sH * g.sW + b.rLo * g.sW, b.np * b.nr * g.sW, g.srcFloats);
  smallIssue<true>(grun, gradOut, gFirst, b.np * b.nOut * g.oW, g.outFloats);
  smallZero(xs, g.xsFloats);
  __syncthreads();
  smallScatter<1, PAD>(xs, run, b, g);
#pragma unroll
  for (int u = 0; u < dev::kLoadBatch; ++u) {
    const int i = u * dev::kBlock + tid;
    if (i * 4 < grun.lead + grun.count) reinterpret_cast<float4 *>(gs)[i] = grun.v[u];  // element i of the run at gs[lead + i]
  }
  __syncthreads();

  const int pl = tid >> g.lpShift, it0 = tid & (g.lp - 1);
  const bool live = pl < b.np;
  float acc[T];
#pragma unroll
  for (int t = 0; t < T; ++t) acc[t] = 0.f;
  if (live) {
    const float *xp = xs + pl * (g.LH * g.LW);
    const float *gp = gs + grun.lead + pl * oPlane;
    // An item whose outputs all exist needs no masking; the last item of a row may (MASK): a masked output
    // must not multiply whatever lies past the row, which may not be finite. The two kinds run in loops of
    // their own, so that no wave has to execute both bodies.
    auto item = [&](auto masked, int r, int c0) {
      constexpr bool MASK = decltype(masked)::value;
      float gv[RW];
#pragma unroll
      for (int q = 0; q < RW; ++q) {
        gv[q] = !MASK || c0 + q < g.oW ? gp[r * g.oW + (MASK ? min(c0 + q, g.oW - 1) : c0 + q)] : 0.f;
        acc[T - 1] += gv[q];
      }
#pragma unroll
      for (int kh = 0; kh < KS; ++kh) {
        const float *row = xp + (r * ST + kh) * g.LW + c0 * ST;
        float win[NWIN];
#pragma unroll
        for (int j = 0; j < NWIN; ++j) win[j] = row[j];
#pragma unroll
        for (int q = 0; q < RW; ++q) {
          const bool ok = !MASK || c0 + q < g.oW;
#pragma unroll
          for (int kw = 0; kw < KS; ++kw) acc[kh * KS + kw] = fmaf(gv[q], ok ? win[q * ST + kw] : 0.f, acc[kh * KS + kw]);
        }
      }
    };
    const int items = b.nOut * g.nfull;
    for (int it = it0; it < items; it += g.lp) {
      const int r = dev::fastDiv(it, g.magicFull);
      item(std::false_type{}, r, (it - r * g.nfull) * RW);
    }
    // the ragged items, one per row, dealt from the last lane down: those lanes did the fewest items above
    if (g.nfull != g.nseg)
      for (int r = g.lp - 1 - it0; r < b.nOut; r += g.lp) item(std::true_type{}, r, g.nfull * RW);
  }
  // fold over the lanes of the plane, fixed association: inside the wave on the VALU; a plane that has
  // two or all four waves of the workgroup (lp = 128, 256) adds the wave sums through LDS
#pragma unroll
  for (int t = 0; t < T; ++t) acc[t] = dev::groupSum(acc[t], min(g.lp, dev::kWave));
  if (g.lp > dev::kWave) {
    const int lane = tid % dev::kWave, wave = tid / dev::kWave;
    if (lane == 0) {
#pragma unroll
      for (int t = 0; t < T; ++t) red[wave][t] = acc[t];
    }
    __syncthreads();
    const int w0 = pl << (g.lpShift - 6);  // first wave of this lane's plane
#pragma unroll
    for (int t = 0; t < T; ++t) {
      acc[t] = red[w0][t] + red[w0 + 1][t];
      if (g.lp == dev::kBlock) acc[t] += red[2][t] + red[3][t];
    }
  }
  if (live && it0 == 0) {
    const int q = b.q0 + pl;
    const int n = dev::fastDiv(q, g.magicC), c = q - n * g.C;
    constexpr int TP = (T + 15) & ~15;
    float4 *dst = reinterpret_cast<float4 *>(partial + (((long)n * g.bands + b.band) * g.C + c) * TP);
#pragma unroll
    for (int t4 = 0; t4 < (T + 3) / 4; ++t4)
      dst[t4] = make_float4(acc[t4 * 4], t4 * 4 + 1 < T ? acc[t4 * 4 + 1] : 0.f, t4 * 4 + 2 < T ? acc[t4 * 4 + 2] : 0.f,
                            t4 * 4 + 3 < T ? acc[t4 * 4 + 3] : 0.f);
  }
}
