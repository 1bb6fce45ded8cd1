// Depthwise convolution on small planes (the 28x28 / 14x14 / 7x7 stages of a network): several whole
// (n, c) planes per workgroup. Included by dwconv.hip inside its anonymous namespace.
//
// Planes are contiguous in memory, so a workgroup's P planes are one contiguous run of floats: it is
// fetched with 16-byte loads in memory order, scattered into zero-bordered planes in LDS (any width:
// no multiple-of-4 requirement), convolved from LDS with no bounds test, and the results go through a
// linear LDS buffer so that they leave as 16-byte streaming stores in memory order as well.
//
//   forward            : source = input,      staged 1:1,            compute stride = conv stride
//   gradInput          : source = gradOutput, staged zero-dilated by the conv stride, compute stride 1,
//                        taps flipped - the transpose of a strided convolution as a stride-1 convolution
//   accGradParameters  : input staged 1:1, gradOutput linear; k*k+1 sums per plane reduced over the
//                        lanes of the plane, one partial per (plane, tap) for the second-stage fold
//
// Lanes are dealt to planes in fixed groups of kBlock / P (a power of two), so a lane keeps the taps of
// one channel in registers. Depth multiplier 1, square kernel 3 or 5, stride 1 or 2, padding k / 2.
#pragma once

#include <type_traits>

struct SmallGeom {
  int C, planes;          // channels, N * C
  int P, lp, lpShift;     // planes per workgroup, lanes per plane (kBlock / P), log2(lp)
  int sH, sW;             // plane of the tensor that is read and staged
  int oH, oW;             // plane of the tensor that is produced (accGrad: gradOutput, read linear)
  int LH, LW;             // staged plane in LDS (zero border included); LW is the row pitch (odd, >= the bordered width)
  int xsFloats;           // floats of the P staged planes incl. slack, a multiple of 4
  int nseg;               // segments of RW outputs per row
  unsigned magicC, magicSPlane, magicSW, magicSeg;
};

// Issues the 16-byte loads of `count` floats at `chunk` (16-byte aligned; count <= 4 * kLoadBatch * kBlock).
// A float4 that would straddle the end of the run is fetched element by element.
struct SmallRun {
  float4 v[dev::kLoadBatch];
};
__device__ __forceinline__ void smallIssue(SmallRun &r, const float *__restrict__ chunk, int count) {
  const __amdgpu_buffer_rsrc_t rs = dev::makeRsrc(chunk, (long)(count & ~3) * 4);
#pragma unroll
  for (int u = 0; u < dev::kLoadBatch; ++u) {
    const int e = (u * dev::kBlock + (int)threadIdx.x) * 4;
    r.v[u] = dev::bufLoad4(rs, e + 4 <= count ? e * 4 : dev::kBufOob);
    if (e < count && e + 4 > count) {  // the last, partial group of the tensor
      r.v[u].x = chunk[e];
      r.v[u].y = e + 1 < count ? chunk[e + 1] : 0.f;
      r.v[u].z = e + 2 < count ? chunk[e + 2] : 0.f;
    }
  }
}

// Parks a fetched run in LDS as zero-bordered planes: element (p, h, w) at p * LH * LW + (h * DS + PAD) * LW + w * DS + PAD.
// The planes must have been zeroed (and a barrier passed) before.
template <int DS, int PAD>
__device__ __forceinline__ void smallScatter(float *__restrict__ xs, const SmallRun &r, int count, const SmallGeom &g) {
  const int sPlane = g.sH * g.sW, lPlane = g.LH * g.LW;
#pragma unroll
  for (int u = 0; u < dev::kLoadBatch; ++u) {
    const int e = (u * dev::kBlock + (int)threadIdx.x) * 4;
    if (e < count) {
      int p = dev::fastDiv(e, g.magicSPlane);
      const int rem = e - p * sPlane;
      int h = dev::fastDiv(rem, g.magicSW);
      int w = rem - h * g.sW;
      const float vals[4] = {r.v[u].x, r.v[u].y, r.v[u].z, r.v[u].w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if (e + k < count) xs[p * lPlane + (h * DS + PAD) * g.LW + w * DS + PAD] = vals[k];
        if (++w == g.sW) {
          w = 0;
          if (++h == g.sH) h = 0, ++p;
        }
      }
    }
  }
}

__device__ __forceinline__ void smallZero(float *__restrict__ xs, int floats) {
  for (int i = threadIdx.x; i * 4 < floats; i += dev::kBlock) reinterpret_cast<float4 *>(xs)[i] = make_float4(0.f, 0.f, 0.f, 0.f);
}

// Stores `count` floats from LDS (16-byte aligned) to `dst` (16-byte aligned) in memory order.
__device__ __forceinline__ void smallStoreRun(float *__restrict__ dst, const float *__restrict__ os, int count) {
  for (int i = threadIdx.x; i * 4 < count; i += dev::kBlock) {
    const int e = i * 4;
    if (e + 4 <= count) {
      dev::storeStream4(dst + e, reinterpret_cast<const float4 *>(os)[i]);
    } else {
      for (int k = e; k < count; ++k) dst[k] = os[k];
    }
  }
}

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
  const int q0 = blockIdx.x * g.P;
  const int np = min(g.P, g.planes - q0);
  const int sPlane = g.sH * g.sW, oPlane = g.oH * g.oW;
  const int count = np * sPlane;
  SmallRun run;
  smallIssue(run, src + (long)q0 * sPlane, count);

  // this lane's plane and its taps, fetched while the run is in flight
  const int pl = tid >> g.lpShift, it0 = tid & (g.lp - 1);
  const bool live = pl < np;
  float w[KS * KS];
  float b = 0.f;
  {
    const int q = q0 + (live ? pl : 0);
    const int c = q - dev::fastDiv(q, g.magicC) * g.C;
    const float *wp = weight + c * ws.s1;
#pragma unroll
    for (int kh = 0; kh < KS; ++kh)
#pragma unroll
      for (int kw = 0; kw < KS; ++kw)
        w[FLIP ? (KS - 1 - kh) * KS + (KS - 1 - kw) : kh * KS + kw] = wp[kh * ws.s2 + kw * ws.s3];
    if (bias) b = bias[c * bs.s1];
  }
  smallZero(xs, g.xsFloats);
  __syncthreads();
  smallScatter<DS, PAD>(xs, run, count, g);
  __syncthreads();

  if (live) {
    const float *xp = xs + pl * (g.LH * g.LW);
    float *op = os + pl * oPlane;
    const int items = g.oH * g.nseg;
    for (int it = it0; it < items; it += g.lp) {
      const int r = dev::fastDiv(it, g.magicSeg), c0 = (it - r * g.nseg) * RW;
      float acc[RW];
#pragma unroll
      for (int q = 0; q < RW; ++q) acc[q] = b;
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
  smallStoreRun(dst + (long)q0 * oPlane, os, np * oPlane);
}

// partial[(c * T + t) * N + n] = sum over the plane (n, c) of gradOutput * input window element t
// (t = kh * KS + kw; t = KS * KS: the bias, sum of gradOutput), T = KS * KS + 1.
template <int KS, int ST, int RW>
__global__ void __launch_bounds__(dev::kBlock)
dwSmallAccGrad(const float *__restrict__ in, const float *__restrict__ gradOut, float *__restrict__ partial, SmallGeom g,
               int N) {
  constexpr int PAD = KS / 2, NWIN = (RW - 1) * ST + KS, T = KS * KS + 1;
  extern __shared__ float smem[];
  float *xs = smem, *gs = smem + g.xsFloats;
  const int tid = threadIdx.x;
  const int q0 = blockIdx.x * g.P;
  const int np = min(g.P, g.planes - q0);
  const int sPlane = g.sH * g.sW, oPlane = g.oH * g.oW;
  const int count = np * sPlane, gcount = np * oPlane;
  SmallRun run, grun;
  smallIssue(run, in + (long)q0 * sPlane, count);
  smallIssue(grun, gradOut + (long)q0 * oPlane, gcount);
  smallZero(xs, g.xsFloats);
  __syncthreads();
  smallScatter<1, PAD>(xs, run, count, g);
#pragma unroll
  for (int u = 0; u < dev::kLoadBatch; ++u) {
    const int i = u * dev::kBlock + tid;
    if (i * 4 < gcount) reinterpret_cast<float4 *>(gs)[i] = grun.v[u];  // floats past the run are never read
  }
  __syncthreads();

  const int pl = tid >> g.lpShift, it0 = tid & (g.lp - 1);
  const bool live = pl < np;
  float acc[T];
#pragma unroll
  for (int t = 0; t < T; ++t) acc[t] = 0.f;
  if (live) {
    const float *xp = xs + pl * (g.LH * g.LW);
    const float *gp = gs + pl * oPlane;
    const int items = g.oH * g.nseg;
    // an item whose outputs all exist needs no masking; the last item of a row may (MASK): a masked output
    // must not multiply whatever lies past the row, which may not be finite
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
    for (int it = it0; it < items; it += g.lp) {
      const int r = dev::fastDiv(it, g.magicSeg), c0 = (it - r * g.nseg) * RW;
      if (c0 + RW <= g.oW)
        item(std::false_type{}, r, c0);
      else
        item(std::true_type{}, r, c0);
    }
  }
  // fold over the lanes of the plane, returned in each of them, fixed association
#pragma unroll
  for (int t = 0; t < T; ++t) acc[t] = dev::groupSum(acc[t], g.lp);
  if (live && it0 == 0) {
    const int q = q0 + pl;
    const int n = dev::fastDiv(q, g.magicC), c = q - n * g.C;
#pragma unroll
    for (int t = 0; t < T; ++t) partial[((long)c * T + t) * N + n] = acc[t];
  }
}
