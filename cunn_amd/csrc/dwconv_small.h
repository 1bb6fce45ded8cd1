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

#include <type_traits>

struct SmallGeom {
  int C, planes;           // channels, N * C
  int P, lp, lpShift;      // planes per workgroup (1 when the planes are cut into bands), lanes per plane, log2(lp)
  int bands, rowsPerBand;  // bands per plane, produced rows per band (bands == 1: the whole plane)
  int sH, sW;              // plane of the tensor that is read and staged
  int oH, oW;              // plane of the tensor that is produced (accGrad: gradOutput, read linear)
  int LH, LW;              // staged plane (or band) in LDS incl. its zero border; LW is the row pitch (odd)
  int xsFloats;            // floats of the staged planes incl. slack, a multiple of 4
  int nseg;                // segments of RW outputs per row
  int nfull;               // those of them with all RW outputs inside the row (nseg or nseg - 1)
  long srcFloats, outFloats;  // elements of the source / produced tensor (bounds of the 16-byte accesses)
  unsigned magicC, magicSPlane, magicSW, magicSeg, magicFull, magicBands;
};

// What one workgroup works on.
struct SmallBand {
  int q0, np;      // first plane, planes
  int band;        // band of the plane (0 when bands == 1)
  int o0, nOut;    // produced rows [o0, o0 + nOut) of each plane
  int rLo, nr;     // source rows [rLo, rLo + nr) of each plane are loaded
  int rowBase;     // LDS row of source row rLo: source (r, c) sits at LDS (rowBase + (r - rLo) * DS, PAD + c * DS)
};

template <int KS, int CS, int DS>
__device__ __forceinline__ SmallBand smallBand(const SmallGeom &g) {
  constexpr int PAD = KS / 2;
  SmallBand b;
  if (g.bands == 1) {
    b.q0 = blockIdx.x * g.P, b.np = min(g.P, g.planes - b.q0), b.band = 0;
    b.o0 = 0, b.nOut = g.oH, b.rLo = 0, b.nr = g.sH, b.rowBase = PAD;
  } else {
    b.q0 = dev::fastDiv(blockIdx.x, g.magicBands), b.np = 1, b.band = blockIdx.x - b.q0 * g.bands;
    b.o0 = b.band * g.rowsPerBand, b.nOut = min(g.rowsPerBand, g.oH - b.o0);
    // LDS row j holds bordered-plane row y0 + j; source row r is bordered-plane row r * DS + PAD
    const int y0 = b.o0 * CS, y1 = y0 + (b.nOut - 1) * CS + KS - 1;
    b.rLo = max(0, dev::ceilDivPos(y0 - PAD, DS));
    const int rHi = min(g.sH - 1, (y1 - PAD) / DS);  // y1 >= PAD
    b.nr = max(0, rHi - b.rLo + 1);
    b.rowBase = b.rLo * DS + PAD - y0;
  }
  return b;
}

// A contiguous run of `count` floats of a tensor, fetched with 16-byte loads from the 16-byte boundary at
// or below its first element: float4 i of the fetch holds run elements 4i - lead .. 4i + 3 - lead.
// lead + count <= 4 * kLoadBatch * kBlock.
struct SmallRun {
  float4 v[dev::kLoadBatch];
  int lead, count;
};
// tensor: first element of the tensor (16-byte aligned); first: index of the run's first element; total: elements of the tensor
__device__ __forceinline__ void smallIssue(SmallRun &r, const float *__restrict__ tensor, long first, int count, long total) {
  r.lead = (int)(first & 3), r.count = count;
  const float *base = tensor + (first - r.lead);
  const long avail = total - (first - r.lead);  // floats from the aligned start to the end of the tensor
  const int span = r.lead + count;
  const __amdgpu_buffer_rsrc_t rs = dev::makeRsrc(base, (long)(span & ~3) * 4);
#pragma unroll
  for (int u = 0; u < dev::kLoadBatch; ++u) {
    const int e = (u * dev::kBlock + (int)threadIdx.x) * 4;
    r.v[u] = dev::bufLoad4(rs, e + 4 <= span ? e * 4 : dev::kBufOob);
    if (e < span && e + 4 > span) {  // the last, partial group of the run: whole if the tensor goes on, else by element
      if (e + 4 <= avail) {
        r.v[u] = *reinterpret_cast<const float4 *>(base + e);
      } else {
        r.v[u].x = base[e];
        r.v[u].y = e + 1 < span ? base[e + 1] : 0.f;
        r.v[u].z = e + 2 < span ? base[e + 2] : 0.f;
      }
    }
  }
}

// Parks a fetched source run in LDS as zero-bordered planes (see SmallBand). The planes must have been
// zeroed (and a barrier passed) before.
template <int DS, int PAD>
__device__ __forceinline__ void smallScatter(float *__restrict__ xs, const SmallRun &r, const SmallBand &b, const SmallGeom &g) {
  const int sPlane = b.nr * g.sW, lPlane = g.LH * g.LW;
#pragma unroll
  for (int u = 0; u < dev::kLoadBatch; ++u) {
    const int e = (u * dev::kBlock + (int)threadIdx.x) * 4;
    if (e < r.lead + r.count) {
      const int skip = max(r.lead - e, 0);  // elements of this group in front of the run (first group only)
      const int i0 = e + skip - r.lead;     // run index of the first element taken from this group
      int p = g.bands == 1 ? dev::fastDiv(i0, g.magicSPlane) : 0;
      const int rem = i0 - p * sPlane;
      int h = dev::fastDiv(rem, g.magicSW);
      int w = rem - h * g.sW;
      const float vals[4] = {r.v[u].x, r.v[u].y, r.v[u].z, r.v[u].w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if (k >= skip && i0 + k - skip < r.count) {
          xs[p * lPlane + (h * DS + b.rowBase) * g.LW + w * DS + PAD] = vals[k];
          if (++w == g.sW) {
            w = 0;
            if (++h == b.nr) h = 0, ++p;
          }
        }
      }
    }
  }
}

__device__ __forceinline__ void smallZero(float *__restrict__ xs, int floats) {
  for (int i = threadIdx.x; i * 4 < floats; i += dev::kBlock) reinterpret_cast<float4 *>(xs)[i] = make_float4(0.f, 0.f, 0.f, 0.f);
}

// Stores the run of `count` floats that starts at element `first` of `tensor` (16-byte aligned) from LDS,
// where element i of the run sits at os[(first & 3) + i]: 16-byte streaming stores for the groups that lie
// inside the run, single stores for its ragged ends.
__device__ __forceinline__ void smallStoreRun(float *__restrict__ tensor, long first, const float *__restrict__ os, int count) {
  const int lead = (int)(first & 3);
  float *base = tensor + (first - lead);
  for (int i = threadIdx.x; i * 4 < lead + count; i += dev::kBlock) {
    const int e = i * 4;
    if (e >= lead && e + 4 <= lead + count) {
      dev::storeStream4(base + e, reinterpret_cast<const float4 *>(os)[i]);
    } else {
      for (int k = max(e, lead); k < min(e + 4, lead + count); ++k) base[k] = os[k];
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

// partial[(c * T + t) * nslots + n * bands + band] = sum over the band of plane (n, c) of gradOutput * input
// window element t (t = kh * KS + kw; t = KS * KS: the bias, sum of gradOutput), T = KS * KS + 1, nslots = N * bands.
template <int KS, int ST, int RW>
__global__ void __launch_bounds__(dev::kBlock)
dwSmallAccGrad(const float *__restrict__ in, const float *__restrict__ gradOut, float *__restrict__ partial, SmallGeom g,
               int N) {
  constexpr int PAD = KS / 2, NWIN = (RW - 1) * ST + KS, T = KS * KS + 1;
  extern __shared__ float smem[];
  __shared__ float red[dev::kBlock / dev::kWave][T];
  float *xs = smem, *gs = smem + g.xsFloats;
  const int tid = threadIdx.x;
  const SmallBand b = smallBand<KS, ST, 1>(g);
  const int oPlane = g.oH * g.oW;
  const long gFirst = (long)b.q0 * oPlane + b.o0 * g.oW;
  SmallRun run, grun;
  smallIssue(run, in, (long)b.q0 * g.sH * g.sW + b.rLo * g.sW, b.np * b.nr * g.sW, g.srcFloats);
  smallIssue(grun, gradOut, gFirst, b.np * b.nOut * g.oW, g.outFloats);
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
    const long nslots = (long)N * g.bands;
#pragma unroll
    for (int t = 0; t < T; ++t) partial[((long)c * T + t) * nslots + n * g.bands + b.band] = acc[t];
  }
}
