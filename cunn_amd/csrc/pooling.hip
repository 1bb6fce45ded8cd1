// SpatialMaxPooling / SpatialDilatedMaxPooling / SpatialAveragePooling for gfx950.
//
// All four kernels are pure streaming: a workgroup owns a band of rows of one
// (n,c) plane, stages the rows of the other tensor that the band depends on in
// LDS with one contiguous (16-byte where aligned) copy, and produces its band
// with coalesced stores. Window scans keep the reference's order (rows outer,
// columns inner, strict '>' for max) so ties resolve identically
// (lib/THCUNN/SpatialDilatedMaxPooling.cu:7-42) and float sums associate
// identically (lib/THCUNN/SpatialAveragePooling.cu:6-82). The backward passes are
// gathers per input pixel, as in the reference, hence deterministic.
#include <cfloat>
#include <cmath>

#include "device_utils.h"
#include "launch_utils.h"
#include "strip.h"
#include "thc_internal.h"

using namespace thc;

namespace {

struct PoolGeom {
  int H, W, oH, oW;
  int kH, kW, dH, dW, padH, padW, dilH, dilW;
  int tileRows, tilesPerPlane, nblk;
  int maxStageRows;  // rows of the staged tensor per band (upper bound)
  unsigned magicTiles;  // dev::magicOf(tilesPerPlane), used by the strip kernels
  int constDiv;         // average pooling: every window has the divisor kH*kW (no window is clipped)
  unsigned magicDH, magicDW;  // dev::magicOf(dH), dev::magicOf(dW): the backward gathers divide by the strides
};

// (plane, tile) of a workgroup of the strip kernels
__device__ __forceinline__ void blockPos(const PoolGeom &g, int &plane, int &tile) {
  const int bid = blockIdx.x;  // consecutive workgroups work on neighbouring planes
  plane = g.tilesPerPlane == 1 ? bid : dev::fastDiv(bid, g.magicTiles);
  tile = bid - plane * g.tilesPerPlane;
}

// ----------------------------------------------------------- max: forward ----
template <int KS, int ST, bool VEC>
__global__ void __launch_bounds__(dev::kBlock)
maxPoolFwdTiled(const float *__restrict__ in, float *__restrict__ out, long *__restrict__ indices, PoolGeom g) {
  extern __shared__ float smem[];
  const int kH = KS ? KS : g.kH, kW = KS ? KS : g.kW;
  const int dH = ST ? ST : g.dH, dW = ST ? ST : g.dW;
  const int dilH = KS ? 1 : g.dilH, dilW = KS ? 1 : g.dilW;
  const int bid = dev::xcdRemap(blockIdx.x, g.nblk);
  const int plane = bid / g.tilesPerPlane, tile = bid - plane * g.tilesPerPlane;
  const int ph0 = tile * g.tileRows;
  const int nOut = min(g.tileRows, g.oH - ph0);
  const int hLo = max(0, ph0 * dH - g.padH);
  const int hHi = min(g.H, (ph0 + nOut - 1) * dH - g.padH + (kH - 1) * dilH + 1);
  dev::loadFlat<VEC>(smem, in + ((long)plane * g.H + hLo) * g.W, max(0, hHi - hLo) * g.W);
  __syncthreads();

  const long obase = ((long)plane * g.oH + ph0) * g.oW;
  const int total = nOut * g.oW;
  for (int i = threadIdx.x; i < total; i += blockDim.x) {
    int r = i / g.oW, pw = i - r * g.oW;
    int hstart = (ph0 + r) * dH - g.padH;
    int wstart = pw * dW - g.padW;
    float maxval = -FLT_MAX;
    int maxidx = -1;
    if (KS) {
#pragma unroll
      for (int kh = 0; kh < KS; ++kh) {
        int h = hstart + kh;
        bool hv = h >= 0 && h < g.H;
#pragma unroll
        for (int kw = 0; kw < KS; ++kw) {
          int w = wstart + kw;
          if (hv && w >= 0 && w < g.W) {
            float v = smem[(h - hLo) * g.W + w];
            if (v > maxval) {
              maxval = v;
              maxidx = h * g.W + w;
            }
          }
        }
      }
    } else {
      int hend = min(hstart + (kH - 1) * dilH + 1, g.H);
      int wend = min(wstart + (kW - 1) * dilW + 1, g.W);
      while (hstart < 0) hstart += dilH;
      while (wstart < 0) wstart += dilW;
      for (int h = hstart; h < hend; h += dilH)
        for (int w = wstart; w < wend; w += dilW) {
          float v = smem[(h - hLo) * g.W + w];
          if (v > maxval) {
            maxval = v;
            maxidx = h * g.W + w;
          }
        }
    }
    out[obase + i] = maxval;
    indices[obase + i] = (long)maxidx + TH_INDEX_BASE;
  }
}

__global__ void __launch_bounds__(dev::kBlock)
maxPoolFwdDirect(const float *__restrict__ in, float *__restrict__ out, long *__restrict__ indices, PoolGeom g,
                 long total) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    int pw = (int)(i % g.oW);
    long t = i / g.oW;
    int ph = (int)(t % g.oH);
    long plane = t / g.oH;
    const float *ip = in + plane * g.H * g.W;
    int hstart = ph * g.dH - g.padH, wstart = pw * g.dW - g.padW;
    int hend = min(hstart + (g.kH - 1) * g.dilH + 1, g.H);
    int wend = min(wstart + (g.kW - 1) * g.dilW + 1, g.W);
    while (hstart < 0) hstart += g.dilH;
    while (wstart < 0) wstart += g.dilW;
    float maxval = -FLT_MAX;
    int maxidx = -1;
    for (int h = hstart; h < hend; h += g.dilH)
      for (int w = wstart; w < wend; w += g.dilW) {
        float v = ip[(long)h * g.W + w];
        if (v > maxval) {
          maxval = v;
          maxidx = h * g.W + w;
        }
      }
    out[i] = maxval;
    indices[i] = (long)maxidx + TH_INDEX_BASE;
  }
}

// ---------------------------------------------------------- max: backward ----
// Band of gradInput rows; the gradOutput rows and indices (narrowed to 32 bits,
// base removed) of every window that can reach the band are staged in LDS.
template <bool VEC>
__global__ void __launch_bounds__(dev::kBlock)
maxPoolBwdTiled(const float *__restrict__ gradOut, const long *__restrict__ indices, float *__restrict__ gradIn,
                PoolGeom g) {
  extern __shared__ float smem[];
  const int extH = (g.kH - 1) * g.dilH + 1, extW = (g.kW - 1) * g.dilW + 1;
  const int bid = dev::xcdRemap(blockIdx.x, g.nblk);
  const int plane = bid / g.tilesPerPlane, tile = bid - plane * g.tilesPerPlane;
  const int h0 = tile * g.tileRows;
  const int nRows = min(g.tileRows, g.H - h0);
  const int phLo = max(0, dev::ceilDivPos(h0 + g.padH - extH + 1, g.dH));
  const int phHi = min(g.oH - 1, (h0 + nRows - 1 + g.padH) / g.dH);
  const int nPh = max(0, phHi - phLo + 1);
  float *gs = smem;
  int *is = reinterpret_cast<int *>(smem + (size_t)g.maxStageRows * g.oW);
  const long sbase = ((long)plane * g.oH + phLo) * g.oW;
  const int cnt = nPh * g.oW;
  dev::loadFlat<VEC>(gs, gradOut + sbase, cnt);
  for (int i = threadIdx.x; i < cnt; i += blockDim.x) is[i] = (int)(indices[sbase + i] - TH_INDEX_BASE);
  __syncthreads();

  float *o = gradIn + ((long)plane * g.H + h0) * g.W;
  const int total = nRows * g.W;
  for (int i = threadIdx.x; i < total; i += blockDim.x) {
    int r = i / g.W, w = i - r * g.W;
    int h = h0 + r;
    int phstart = (h + g.padH < extH) ? 0 : (h + g.padH - extH) / g.dH + 1;
    int phend = min((h + g.padH) / g.dH + 1, g.oH);
    int pwstart = (w + g.padW < extW) ? 0 : (w + g.padW - extW) / g.dW + 1;
    int pwend = min((w + g.padW) / g.dW + 1, g.oW);
    const int me = h * g.W + w;
    float grad = 0.f;
    for (int ph = phstart; ph < phend; ++ph)
      for (int pw = pwstart; pw < pwend; ++pw) {
        int k = (ph - phLo) * g.oW + pw;
        if (is[k] == me) grad += gs[k];
      }
    o[i] = grad;
  }
}

__global__ void __launch_bounds__(dev::kBlock)
maxPoolBwdDirect(const float *__restrict__ gradOut, const long *__restrict__ indices, float *__restrict__ gradIn,
                 PoolGeom g, long total) {
  const int extH = (g.kH - 1) * g.dilH + 1, extW = (g.kW - 1) * g.dilW + 1;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    int w = (int)(i % g.W);
    long t = i / g.W;
    int h = (int)(t % g.H);
    long plane = t / g.H;
    int phstart = (h + g.padH < extH) ? 0 : (h + g.padH - extH) / g.dH + 1;
    int phend = min((h + g.padH) / g.dH + 1, g.oH);
    int pwstart = (w + g.padW < extW) ? 0 : (w + g.padW - extW) / g.dW + 1;
    int pwend = min((w + g.padW) / g.dW + 1, g.oW);
    const float *gp = gradOut + plane * g.oH * g.oW;
    const long *ix = indices + plane * g.oH * g.oW;
    float grad = 0.f;
    for (int ph = phstart; ph < phend; ++ph)
      for (int pw = pwstart; pw < pwend; ++pw)
        if (ix[ph * g.oW + pw] - TH_INDEX_BASE == (long)h * g.W + w) grad += gp[ph * g.oW + pw];
    gradIn[i] = grad;
  }
}

// ------------------------------------------------------- average: forward ----
template <bool INCLUDE_PAD>
__device__ __forceinline__ float avgDivisor(int ph, int pw, const PoolGeom &g, int &hs, int &he, int &ws, int &we) {
  hs = ph * g.dH - g.padH;
  ws = pw * g.dW - g.padW;
  he = min(hs + g.kH, g.H + g.padH);
  we = min(ws + g.kW, g.W + g.padW);
  const int pool = (he - hs) * (we - ws);
  hs = max(hs, 0);
  ws = max(ws, 0);
  he = min(he, g.H);
  we = min(we, g.W);
  return INCLUDE_PAD ? (float)pool : (float)((he - hs) * (we - ws));
}

template <bool INCLUDE_PAD, bool VEC>
__global__ void __launch_bounds__(dev::kBlock)
avgPoolFwdTiled(const float *__restrict__ in, float *__restrict__ out, PoolGeom g) {
  extern __shared__ float smem[];
  const int bid = dev::xcdRemap(blockIdx.x, g.nblk);
  const int plane = bid / g.tilesPerPlane, tile = bid - plane * g.tilesPerPlane;
  const int ph0 = tile * g.tileRows;
  const int nOut = min(g.tileRows, g.oH - ph0);
  const int hLo = max(0, ph0 * g.dH - g.padH);
  const int hHi = min(g.H, (ph0 + nOut - 1) * g.dH - g.padH + g.kH);
  dev::loadFlat<VEC>(smem, in + ((long)plane * g.H + hLo) * g.W, max(0, hHi - hLo) * g.W);
  __syncthreads();
  const long obase = ((long)plane * g.oH + ph0) * g.oW;
  const int total = nOut * g.oW;
  for (int i = threadIdx.x; i < total; i += blockDim.x) {
    int r = i / g.oW, pw = i - r * g.oW;
    int hs, he, ws, we;
    float div = avgDivisor<INCLUDE_PAD>(ph0 + r, pw, g, hs, he, ws, we);
    float s = 0.f;
    for (int h = hs; h < he; ++h)
      for (int w = ws; w < we; ++w) s += smem[(h - hLo) * g.W + w];
    out[obase + i] = s / div;
  }
}

template <bool INCLUDE_PAD>
__global__ void __launch_bounds__(dev::kBlock)
avgPoolFwdDirect(const float *__restrict__ in, float *__restrict__ out, PoolGeom g, long total) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    int pw = (int)(i % g.oW);
    long t = i / g.oW;
    int ph = (int)(t % g.oH);
    long plane = t / g.oH;
    const float *ip = in + plane * g.H * g.W;
    int hs, he, ws, we;
    float div = avgDivisor<INCLUDE_PAD>(ph, pw, g, hs, he, ws, we);
    float s = 0.f;
    for (int h = hs; h < he; ++h)
      for (int w = ws; w < we; ++w) s += ip[(long)h * g.W + w];
    out[i] = s / div;
  }
}

// ------------------------------------------------------ average: backward ----
template <bool INCLUDE_PAD>
__device__ __forceinline__ float avgGather(const float *__restrict__ gp, int rowOff, int h, int w, const PoolGeom &g) {
  const int hp = h + g.padH, wp = w + g.padW;
  const int phstart = (hp < g.kH) ? 0 : dev::fastDiv(hp - g.kH, g.magicDH) + 1;
  const int phend = min(dev::fastDiv(hp, g.magicDH) + 1, g.oH);
  const int pwstart = (wp < g.kW) ? 0 : dev::fastDiv(wp - g.kW, g.magicDW) + 1;
  const int pwend = min(dev::fastDiv(wp, g.magicDW) + 1, g.oW);
  float grad = 0.f;
  for (int ph = phstart; ph < phend; ++ph)
    for (int pw = pwstart; pw < pwend; ++pw) {
      int hs, he, ws, we;
      float div = avgDivisor<INCLUDE_PAD>(ph, pw, g, hs, he, ws, we);
      grad += gp[(ph - rowOff) * g.oW + pw] / div;
    }
  return grad;
}

template <bool INCLUDE_PAD, bool VEC>
__global__ void __launch_bounds__(dev::kBlock)
avgPoolBwdTiled(const float *__restrict__ gradOut, float *__restrict__ gradIn, PoolGeom g) {
  extern __shared__ float smem[];
  const int bid = dev::xcdRemap(blockIdx.x, g.nblk);
  const int plane = bid / g.tilesPerPlane, tile = bid - plane * g.tilesPerPlane;
  const int h0 = tile * g.tileRows;
  const int nRows = min(g.tileRows, g.H - h0);
  const int phLo = max(0, dev::ceilDivPos(h0 + g.padH - g.kH + 1, g.dH));
  const int phHi = min(g.oH - 1, (h0 + nRows - 1 + g.padH) / g.dH);
  const int nPh = max(0, phHi - phLo + 1);
  dev::loadFlat<VEC>(smem, gradOut + ((long)plane * g.oH + phLo) * g.oW, nPh * g.oW);
  __syncthreads();
  float *o = gradIn + ((long)plane * g.H + h0) * g.W;
  const int total = nRows * g.W;
  for (int i = threadIdx.x; i < total; i += blockDim.x) {
    int r = i / g.W, w = i - r * g.W;
    o[i] = avgGather<INCLUDE_PAD>(smem, phLo, h0 + r, w, g);
  }
}

template <bool INCLUDE_PAD>
__global__ void __launch_bounds__(dev::kBlock)
avgPoolBwdDirect(const float *__restrict__ gradOut, float *__restrict__ gradIn, PoolGeom g, long total) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    int w = (int)(i % g.W);
    long t = i / g.W;
    int h = (int)(t % g.H);
    long plane = t / g.H;
    gradIn[i] = avgGather<INCLUDE_PAD>(gradOut + plane * g.oH * g.oW, 0, h, w, g);
  }
}

// ===================================================== small planes, any geometry ==
// Planes of at most 1024 elements (the 28x28 / 14x14 / 7x7 stages) that the strip kernels do not take:
// a plane per workgroup would leave most lanes idle, so a workgroup takes P consecutive planes - one
// contiguous run of memory - stages what it reads in LDS and produces its results in memory order
// (a lane per output element forward, 4 consecutive gradInput elements backward), so every global
// access of a wave is one contiguous run. Window geometry is run-time (the reference's loops).
struct SmallPool {
  int planes, P;          // N * C, planes per workgroup
  unsigned magicHW, magicW, magicOHW, magicOW;
  bool vec;               // runs start on 16-byte boundaries: 16-byte accesses allowed
};

template <bool MAX, bool INCLUDE_PAD>
__global__ void __launch_bounds__(dev::kBlock)
poolFwdSmall(const float *__restrict__ in, float *__restrict__ out, long *__restrict__ indices, PoolGeom g, SmallPool sp) {
  extern __shared__ float smem[];
  const int HW = g.H * g.W, oHW = g.oH * g.oW;
  const int q0 = blockIdx.x * sp.P;
  const int np = min(sp.P, sp.planes - q0);
  const int nIn = np * HW, nOut = np * oHW;
  const float *src = in + (long)q0 * HW;
  if (sp.vec) {
    for (int i = threadIdx.x * 4; i < nIn; i += dev::kBlock * 4) {
      if (i + 4 <= nIn) {
        *reinterpret_cast<float4 *>(smem + i) = *reinterpret_cast<const float4 *>(src + i);
      } else {
        for (int k = i; k < nIn; ++k) smem[k] = src[k];
      }
    }
  } else {
    for (int i = threadIdx.x; i < nIn; i += dev::kBlock) smem[i] = src[i];
  }
  __syncthreads();
  float *o = out + (long)q0 * oHW;
  long *ix = MAX ? indices + (long)q0 * oHW : nullptr;
  for (int i = threadIdx.x; i < nOut; i += dev::kBlock) {
    const int pl = dev::fastDiv(i, sp.magicOHW), r = i - pl * oHW;
    const int ph = dev::fastDiv(r, sp.magicOW), pw = r - ph * g.oW;
    const float *ip = smem + pl * HW;
    if (MAX) {
      int hstart = ph * g.dH - g.padH, wstart = pw * g.dW - g.padW;
      const int hend = min(hstart + (g.kH - 1) * g.dilH + 1, g.H);
      const int wend = min(wstart + (g.kW - 1) * g.dilW + 1, g.W);
      while (hstart < 0) hstart += g.dilH;
      while (wstart < 0) wstart += g.dilW;
      float maxval = -FLT_MAX;
      int maxidx = -1;
      for (int h = hstart; h < hend; h += g.dilH)
        for (int w = wstart; w < wend; w += g.dilW) {
          const float v = ip[h * g.W + w];
          if (v > maxval) maxval = v, maxidx = h * g.W + w;
        }
      o[i] = maxval;
      ix[i] = (long)maxidx + TH_INDEX_BASE;
    } else {
      int hs, he, ws, we;
      const float div = avgDivisor<INCLUDE_PAD>(ph, pw, g, hs, he, ws, we);
      float sum = 0.f;
      for (int h = hs; h < he; ++h)
        for (int w = ws; w < we; ++w) sum += ip[h * g.W + w];
      o[i] = sum / div;
    }
  }
}

template <bool MAX, bool INCLUDE_PAD>
__global__ void __launch_bounds__(dev::kBlock)
poolBwdSmall(const float *__restrict__ gradOut, const long *__restrict__ indices, float *__restrict__ gradIn, PoolGeom g,
             SmallPool sp) {
  extern __shared__ float smem[];
  const int HW = g.H * g.W, oHW = g.oH * g.oW;
  const int q0 = blockIdx.x * sp.P;
  const int np = min(sp.P, sp.planes - q0);
  const int nIn = np * HW, nOut = np * oHW;
  float *gs = smem;
  int *is = reinterpret_cast<int *>(smem + sp.P * oHW);  // max: argmax positions inside their plane, 0-based
  for (int i = threadIdx.x; i < nOut; i += dev::kBlock) {
    gs[i] = gradOut[(long)q0 * oHW + i];
    if (MAX) is[i] = (int)(indices[(long)q0 * oHW + i] - TH_INDEX_BASE);
  }
  __syncthreads();
  const int extH = (g.kH - 1) * g.dilH + 1, extW = (g.kW - 1) * g.dilW + 1;
  float *o = gradIn + (long)q0 * HW;
  for (int i4 = threadIdx.x * 4; i4 < nIn; i4 += dev::kBlock * 4) {
    float v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int i = i4 + k;
      v[k] = 0.f;
      if (i < nIn) {
        const int pl = dev::fastDiv(i, sp.magicHW), r = i - pl * HW;
        const int h = dev::fastDiv(r, sp.magicW), w = r - h * g.W;
        if (MAX) {
          const int phstart = (h + g.padH < extH) ? 0 : dev::fastDiv(h + g.padH - extH, g.magicDH) + 1;
          const int phend = min(dev::fastDiv(h + g.padH, g.magicDH) + 1, g.oH);
          const int pwstart = (w + g.padW < extW) ? 0 : dev::fastDiv(w + g.padW - extW, g.magicDW) + 1;
          const int pwend = min(dev::fastDiv(w + g.padW, g.magicDW) + 1, g.oW);
          float grad = 0.f;
          for (int ph = phstart; ph < phend; ++ph)
            for (int pw = pwstart; pw < pwend; ++pw)
              if (is[pl * oHW + ph * g.oW + pw] == r) grad += gs[pl * oHW + ph * g.oW + pw];
          v[k] = grad;
        } else {
          v[k] = avgGather<INCLUDE_PAD>(gs + pl * oHW, 0, h, w, g);
        }
      }
    }
    if (sp.vec && i4 + 4 <= nIn) {
      dev::storeStream4(o + i4, make_float4(v[0], v[1], v[2], v[3]));
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if (i4 + k < nIn) o[i4 + k] = v[k];
    }
  }
}

#include "pooling_runs.h"

// ============================================================ strip kernels ==
// Fast paths for square windows without dilation whose geometry (KS, ST, PAD) is
// known at compile time and whose rows are multiples of 4 (see strip.h). A lane
// produces 4 consecutive outputs (forward) or an ST x 4 patch (backward); cells
// outside the image hold a neutral fill (-FLT_MAX for max, 0 for sums), so the
// scans run without bounds tests while visiting elements in the reference's
// order (rows outer, columns inner).

template <int KS, int ST, int PAD>
__global__ void __launch_bounds__(dev::kBlock)
maxPoolFwdStrip(const float *__restrict__ in, float *__restrict__ out, long *__restrict__ indices, PoolGeom g) {
  using S = dev::Strip<KS, ST, PAD>;
  constexpr int NW = S::NW;
  extern __shared__ float smem[];
  int plane, tile;
  blockPos(g, plane, tile);
  const int ph0 = tile * g.tileRows;
  const int nOut = min(g.tileRows, g.oH - ph0);
  const int nIn = (nOut - 1) * ST + KS;
  const int pitch = S::pitch(g.W);
  S::stage(smem, in + (long)plane * g.H * g.W, g.H, g.W, ph0 * ST - PAD, nIn, -FLT_MAX);
  __syncthreads();
  const int oW4 = g.oW >> 2;
  const unsigned magicOw4 = dev::magicOf(oW4);
  const int total = nOut * oW4;
  const long obase = ((long)plane * g.oH + ph0) * g.oW;
  for (int i = threadIdx.x; i < total; i += blockDim.x) {
    const int r = dev::fastDiv(i, magicOw4), b4 = i - r * oW4;
    const float *p = smem + r * ST * pitch;
    float mv[4] = {-FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX};
    int mi[4] = {-1, -1, -1, -1};
    const int idx0 = ((ph0 + r) * ST - PAD) * g.W + b4 * 4 * ST - PAD;  // flat index of window element (kh=0, j=0)
#pragma unroll
    for (int kh = 0; kh < KS; ++kh) {
      float win[NW];
      S::loadWin(p + kh * pitch, b4, g.W, win);
#pragma unroll
      for (int kw = 0; kw < KS; ++kw)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          if (win[q * ST + kw] > mv[q]) {
            mv[q] = win[q * ST + kw];
            mi[q] = idx0 + kh * g.W + q * ST + kw;
          }
    }
    const long o = obase + (long)r * g.oW + b4 * 4;
    dev::storeStream4(out + o, make_float4(mv[0], mv[1], mv[2], mv[3]));
    long2 i01, i23;
    i01.x = (long)mi[0] + TH_INDEX_BASE, i01.y = (long)mi[1] + TH_INDEX_BASE;
    i23.x = (long)mi[2] + TH_INDEX_BASE, i23.y = (long)mi[3] + TH_INDEX_BASE;
    dev::storeStream2(indices + o, i01.x, i01.y);
    dev::storeStream2(indices + o + 2, i23.x, i23.y);
  }
}

template <int KS, int ST, int PAD, bool INCLUDE_PAD>
__global__ void __launch_bounds__(dev::kBlock)
avgPoolFwdStrip(const float *__restrict__ in, float *__restrict__ out, PoolGeom g) {
  using S = dev::Strip<KS, ST, PAD>;
  constexpr int NW = S::NW;
  extern __shared__ float smem[];
  int plane, tile;
  blockPos(g, plane, tile);
  const int ph0 = tile * g.tileRows;
  const int nOut = min(g.tileRows, g.oH - ph0);
  const int nIn = (nOut - 1) * ST + KS;
  const int pitch = S::pitch(g.W);
  S::stage(smem, in + (long)plane * g.H * g.W, g.H, g.W, ph0 * ST - PAD, nIn, 0.f);
  __syncthreads();
  const int oW4 = g.oW >> 2;
  const unsigned magicOw4 = dev::magicOf(oW4);
  const int total = nOut * oW4;
  const long obase = ((long)plane * g.oH + ph0) * g.oW;
  for (int i = threadIdx.x; i < total; i += blockDim.x) {
    const int r = dev::fastDiv(i, magicOw4), b4 = i - r * oW4;
    const float *p = smem + r * ST * pitch;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kh = 0; kh < KS; ++kh) {
      float win[NW];
      S::loadWin(p + kh * pitch, b4, g.W, win);
#pragma unroll
      for (int kw = 0; kw < KS; ++kw)
#pragma unroll
        for (int q = 0; q < 4; ++q) acc[q] += win[q * ST + kw];
    }
    float res[4];
    if (g.constDiv) {
#pragma unroll
      for (int q = 0; q < 4; ++q) res[q] = acc[q] / (float)(KS * KS);
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        int hs, he, ws, we;
        res[q] = acc[q] / avgDivisor<INCLUDE_PAD>(ph0 + r, b4 * 4 + q, g, hs, he, ws, we);
      }
    }
    dev::storeStream4(out + obase + (long)r * g.oW + b4 * 4, make_float4(res[0], res[1], res[2], res[3]));
  }
}

// Global average pooling (one window = the whole plane, no padding; the last layer of most
// classification networks, with planes of 49 elements). Forward: a wave sums one plane at a time,
// four planes in flight, lanes over the plane's elements in memory order. Backward: a lane writes
// elements of gradInput in memory order, each the plane's gradOutput over the plane size.
__global__ void __launch_bounds__(dev::kBlock)
avgPoolGlobalFwd(const float *__restrict__ in, float *__restrict__ out, long planes, int S) {
  const int lane = threadIdx.x % dev::kWave;
  const long nWaves = (long)gridDim.x * (dev::kBlock / dev::kWave);
  const float div = (float)S;
  for (long q = ((long)blockIdx.x * (dev::kBlock / dev::kWave) + threadIdx.x / dev::kWave) * 4; q < planes; q += nWaves * 4) {
    float a[4] = {0.f, 0.f, 0.f, 0.f};
    for (int i = lane; i < S; i += dev::kWave) {
#pragma unroll
      for (int u = 0; u < 4; ++u) a[u] += q + u < planes ? in[(q + u) * S + i] : 0.f;
    }
    float r = 0.f;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const float v = dev::waveSum(a[u]);
      if (lane == u) r = v;
    }
    if (lane < 4 && q + lane < planes) out[q + lane] = r / div;
  }
}

__global__ void __launch_bounds__(dev::kBlock)
avgPoolGlobalBwd(const float *__restrict__ gradOut, float *__restrict__ gradIn, unsigned total, int S, unsigned magicS) {
  const float div = (float)S;
  for (unsigned e = blockIdx.x * dev::kBlock + threadIdx.x; e < total; e += gridDim.x * dev::kBlock)
    gradIn[e] = gradOut[dev::fastDiv((int)e, magicS)] / div;
}

// Non-overlapping average pooling (window = stride = KS, no padding, H = KS*oH, W = KS*oW): no
// input element is shared between windows, so nothing is staged. With these extents the planes
// of the batch form one tall image of planes*oH output rows; a lane owns 4 consecutive outputs
// of one of those rows and streams its KS x 4*KS input patch through registers with 16-byte
// loads (forward), or expands 4 gradOutput values into that patch (backward).
template <int KS>
__global__ void __launch_bounds__(dev::kBlock)
avgPoolFwdFlat(const float *__restrict__ in, float *__restrict__ out, int oW4, unsigned magicOw4, int W, unsigned total) {
  const unsigned i = blockIdx.x * dev::kBlock + threadIdx.x;
  if (i >= total) return;
  const unsigned R = dev::fastDiv((int)i, magicOw4), b = i - R * oW4;
  const float4 *p = reinterpret_cast<const float4 *>(in + (size_t)R * KS * W) + b * KS;
  const int W4 = W >> 2;
  float4 v[KS][KS];
#pragma unroll
  for (int kh = 0; kh < KS; ++kh)
#pragma unroll
    for (int k = 0; k < KS; ++k) v[kh][k] = p[kh * W4 + k];
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int kh = 0; kh < KS; ++kh) {
    float row[4 * KS];
#pragma unroll
    for (int k = 0; k < KS; ++k) row[4 * k] = v[kh][k].x, row[4 * k + 1] = v[kh][k].y, row[4 * k + 2] = v[kh][k].z, row[4 * k + 3] = v[kh][k].w;
#pragma unroll
    for (int kw = 0; kw < KS; ++kw)
#pragma unroll
      for (int q = 0; q < 4; ++q) acc[q] += row[q * KS + kw];
  }
  dev::storeStream4(out + (size_t)i * 4, make_float4(acc[0] / (float)(KS * KS), acc[1] / (float)(KS * KS),
                                                    acc[2] / (float)(KS * KS), acc[3] / (float)(KS * KS)));
}

// total = float4s of every KS-th gradInput row; a lane reads the up to 4 gradOutput values above float4 b of
// the KS gradInput rows under one gradOutput row once and writes that float4 to each of the rows (a wave's
// store is one contiguous run; KS stores in flight per lane, gradOutput crosses the memory system once).
template <int KS>
__global__ void __launch_bounds__(dev::kBlock)
avgPoolBwdFlat(const float *__restrict__ gradOut, float *__restrict__ gradIn, int W4, unsigned magicW4, int oW, unsigned total) {
  const unsigned i = blockIdx.x * dev::kBlock + threadIdx.x;
  if (i >= total) return;
  const unsigned R = dev::fastDiv((int)i, magicW4), b = i - R * W4;  // row of the tall gradOutput image, float4 within the rows under it
  const float *gp = gradOut + (size_t)R * oW;
  float v[4];
  if constexpr (KS == 2) {
    typedef float f32x2v __attribute__((ext_vector_type(2)));
    const f32x2v g2 = __builtin_nontemporal_load(reinterpret_cast<const f32x2v *>(gp) + b);
    v[0] = v[1] = g2.x / 4.f, v[2] = v[3] = g2.y / 4.f;
  } else if constexpr (KS == 4) {
    v[0] = v[1] = v[2] = v[3] = __builtin_nontemporal_load(gp + b) / 16.f;
  } else {
#pragma unroll
    for (int q = 0; q < 4; ++q) v[q] = gp[(b * 4 + q) / KS] / (float)(KS * KS);
  }
  float *o = gradIn + ((size_t)R * KS * W4 + b) * 4;
#pragma unroll
  for (int k = 0; k < KS; ++k) dev::storeStream4(o + (size_t)k * W4 * 4, make_float4(v[0], v[1], v[2], v[3]));
}

// Backward gathers. MAX: gradOutput and the argmax (narrowed to int32, base
// removed, -2 outside) are staged with a 4-cell fill in front of every row; a
// patch element adds the gradOutput of each covering window whose argmax is that
// element. Otherwise (average): gradOutput / divisor(window) is staged and the
// covering windows are summed.
template <int KS, int ST, int PAD, bool MAX, bool INCLUDE_PAD>
__global__ void __launch_bounds__(dev::kBlock)
poolBwdStrip(const float *__restrict__ gradOut, const long *__restrict__ indices, float *__restrict__ gradIn,
             PoolGeom g, int stageRows) {
  constexpr int QH0 = dev::TapSpan<KS, ST, ST, PAD>::lo(), QH1 = dev::TapSpan<KS, ST, ST, PAD>::hi();
  constexpr int QW0 = dev::TapSpan<KS, ST, 4, PAD>::lo(), QW1 = dev::TapSpan<KS, ST, 4, PAD>::hi();
  constexpr int NW = QW1 - QW0 + 1;
  constexpr int CPB = 4 / ST;
  constexpr int OFF = ((dev::kStripPadL + QW0) % 4 + 4) % 4;
  constexpr int ALIGN = (CPB % 4 == 0) ? 4 : 2;
  extern __shared__ float smem[];
  int plane, tile;
  blockPos(g, plane, tile);
  const int h0 = tile * g.tileRows;  // multiple of ST
  const int nRows = min(g.tileRows, g.H - h0);
  const int pitch = g.oW + dev::kStripPadL;
  const int region = stageRows * pitch + dev::kStripPadL;
  float *gs = smem;
  float *is = smem + region;  // int32 bit patterns (MAX only)
  const int ph0 = h0 / ST + QH0;
  const float *gp = gradOut + (long)plane * g.oH * g.oW;
  if (MAX) {
    dev::loadRowsPadded<true>(gs, gp, g.oH, g.oW, ph0, stageRows, pitch, dev::kStripPadL, 0.f);
    const long *ip = indices + (long)plane * g.oH * g.oW;
    const int cnt = stageRows * pitch + dev::kStripPadL;
    const unsigned magicPitch = dev::magicOf(pitch);
    for (int i = threadIdx.x; i < cnt; i += blockDim.x) {
      int r = dev::fastDiv(i, magicPitch), cc = i - r * pitch - dev::kStripPadL;
      int ph = ph0 + r;
      int v = -2;
      if (cc >= 0 && r < stageRows && ph >= 0 && ph < g.oH) v = (int)(__builtin_nontemporal_load(ip + (long)ph * g.oW + cc) - TH_INDEX_BASE);
      is[i] = __int_as_float(v);
    }
  } else {
    const int cnt = stageRows * pitch + dev::kStripPadL;
    const unsigned magicPitch = dev::magicOf(pitch);
    for (int i = threadIdx.x; i < cnt; i += blockDim.x) {
      int r = dev::fastDiv(i, magicPitch), cc = i - r * pitch - dev::kStripPadL;
      int ph = ph0 + r;
      float v = 0.f;
      if (cc >= 0 && r < stageRows && ph >= 0 && ph < g.oH) {
        int hs, he, ws, we;
        const float gyv = gp[(long)ph * g.oW + cc];
        v = g.constDiv ? gyv / (float)(KS * KS) : gyv / avgDivisor<INCLUDE_PAD>(ph, cc, g, hs, he, ws, we);
      }
      gs[i] = v;
    }
  }
  __syncthreads();
  const int W4 = g.W >> 2;
  const unsigned magicW4 = dev::magicOf(W4);
  // A lane produces the 4 elements i*4 .. i*4+3 of the band in memory order (a wave's store is one
  // contiguous 1 KB run). Its row h0 + hl = ST*a + dy is covered by staged window row qh iff
  // kh = dy + PAD - qh*ST lies inside the window; dy is a run-time value. For max pooling the argmax
  // test alone decides (a window that does not cover the element cannot point at it).
  const int total = nRows * W4;
  const __amdgpu_buffer_rsrc_t orr = dev::makeRsrc(gradIn + ((long)plane * g.H + h0) * g.W, (long)total * 16);
  for (int i = threadIdx.x; i < total; i += blockDim.x) {
    const int hl = dev::fastDiv(i, magicW4), b = i - hl * W4;
    const int a = ST == 1 ? hl : hl / ST, dy = hl - a * ST;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    const int me0 = (h0 + hl) * g.W + b * 4;  // flat index of element 0
    const int woff = dev::kStripPadL + QW0 + b * CPB;
#pragma unroll
    for (int qh = QH0; qh <= QH1; ++qh) {
      float gw[NW], iw[NW];
      dev::readWindow<0, NW, OFF, ALIGN>(gs + (a + qh - QH0) * pitch + woff, gw);
      if (MAX) dev::readWindow<0, NW, OFF, ALIGN>(is + (a + qh - QH0) * pitch + woff, iw);
      bool covers = false;
#pragma unroll
      for (int dyc = 0; dyc < ST; ++dyc) {
        const int kh = dyc + PAD - qh * ST;
        if (kh >= 0 && kh < KS) covers = covers || dy == dyc;
      }
#pragma unroll
      for (int dx = 0; dx < 4; ++dx)
#pragma unroll
        for (int kw = KS - 1; kw >= 0; --kw) {  // descending kw = ascending window column
          const int t = dx + PAD - kw;
          if (t % ST != 0) continue;
          if (MAX) {
            if (__float_as_int(iw[t / ST - QW0]) == me0 + dx) acc[dx] += gw[t / ST - QW0];
          } else {
            acc[dx] += covers ? gw[t / ST - QW0] : 0.f;
          }
        }
    }
    dev::bufStoreStream4(orr, i * 16, make_float4(acc[0], acc[1], acc[2], acc[3]));
  }
}

// -------------------------------------------------------------- host side ----
using launch::aligned16;

// 1: shape-agnostic direct kernels, 2: generic LDS-tiled kernels (no strip fast path).
int forcedPath() { return g_switches.poolForce; }
bool forceDirect() { return forcedPath() == 1; }

// 1 when no window of the average pooling is clipped, i.e. every divisor is kH*kW:
// windows inside the padded extent (count_include_pad) or inside the image itself.
int avgConstDivisor(const PoolGeom &g, bool include_pad) {
  int lastH = (g.oH - 1) * g.dH - g.padH + g.kH, lastW = (g.oW - 1) * g.dW - g.padW + g.kW;  // one past the last window
  if (include_pad) return lastH <= g.H + g.padH && lastW <= g.W + g.padW;
  return g.padH == 0 && g.padW == 0 && lastH <= g.H && lastW <= g.W;
}

// (KS, ST, PAD) combinations the strip kernels are instantiated for
#define POOL_STRIP_COMBOS(X) X(3, 2, 1) X(2, 2, 0) X(3, 2, 0) X(3, 1, 1)

bool stripCombo(const PoolGeom &g) {
  if (g.kH != g.kW || g.dH != g.dW || g.padH != g.padW || g.dilH != 1 || g.dilW != 1) return false;
#define X(K, S, P) \
  if (g.kH == K && g.dH == S && g.padH == P) return true;
  POOL_STRIP_COMBOS(X)
#undef X
  return false;
}

// Forward strips read 4 fill cells beyond a row at most (and, in the split
// stride-2 layout, only even columns may overhang).
// Geometry of the flat average-pooling kernels: window = stride in {2, 3, 4}, no padding, extents
// that the windows tile exactly, rows of 4-output groups, and item indices that keep the reciprocal
// division exact.
bool avgFlatOk(const PoolGeom &g, long planes) {
  const bool sq = g.kH == g.kW && g.dH == g.kH && g.dW == g.kW && g.padH == 0 && g.padW == 0;
  const long total = planes * g.oH * (g.oW / 4);
  return forcedPath() == 0 && sq && g.kH >= 2 && g.kH <= 4 && g.H == g.oH * g.kH && g.W == g.oW * g.kW && g.oW % 4 == 0 &&
         total > 0 && total * (g.oW / 4) < 0xffffffffL && total < 0x7fffffffL;
}

// Plans the small-plane kernels: planes of at most 1024 elements; `staged` = elements per plane held in LDS
// (forward: the input plane; backward: gradOutput and, for max pooling, its indices), `produced` = elements
// per plane written. P planes per workgroup: about 8192 produced elements, at most 32 KB of LDS.
bool smallPoolPlan(const PoolGeom &g, long planes, bool backward, bool max, const void *a, const void *b, SmallPool *sp,
                   size_t *lds) {
  const long HW = (long)g.H * g.W, oHW = (long)g.oH * g.oW;
  // forward: measured faster than the band kernels up to about 20x20 planes; backward up to 32x32
  if (forcedPath() != 0 || HW > (backward ? 1024 : 400) || HW < 1 || oHW < 1 || oHW > 4096 || planes >= 0x7fffffffL)
    return false;
  const long ldsPerPlane = backward ? oHW * (max ? 8 : 4) : HW * 4;
  const long produced = backward ? HW : oHW;
  long P = std::max<long>(1, std::min<long>(8192 / std::max<long>(produced, 1), (32 * 1024) / ldsPerPlane));
  P = std::min(P, planes);
  if (P < 1 || P * ldsPerPlane > (long)launch::kLdsMax) return false;
  // enough workgroups to occupy the chip
  while (P > 1 && planes / P < launch::kMinBlocks) P = (P + 1) / 2;
  sp->planes = (int)planes, sp->P = (int)P;
  sp->magicHW = dev::magicOf((int)HW), sp->magicW = dev::magicOf(g.W);
  sp->magicOHW = dev::magicOf((int)oHW), sp->magicOW = dev::magicOf(g.oW);
  sp->vec = (P * HW) % 4 == 0 && aligned16(a) && aligned16(b);
  *lds = (size_t)(P * ldsPerPlane);
  return true;
}

// One window that is exactly the plane; total elements small enough for the reciprocal division.
bool avgGlobalOk(const PoolGeom &g, long planes) {
  return forcedPath() == 0 && g.oH == 1 && g.oW == 1 && g.padH == 0 && g.padW == 0 && g.kH == g.H && g.kW == g.W &&
         planes * g.H * g.W < 0x7fffffffL && planes * g.H * g.W * ((long)g.H * g.W) < 0xffffffffL;
}

bool stripFwdOk(const PoolGeom &g) {
  if (forcedPath() != 0 || !stripCombo(g) || g.oW % 4 != 0) return false;
  if (g.W % (4 * g.dW) != 0) return false;
  int cmax = (g.oW - 1) * g.dW - g.padW + g.kW - 1;  // last column any window touches
  if (g.dW == 1) return cmax <= g.W + 3;
  int emax = cmax % 2 == 0 ? cmax : cmax - 1, omax = cmax % 2 == 1 ? cmax : cmax - 1;
  return emax <= g.W + 6 && omax <= g.W - 1;
}
bool stripBwdOk(const PoolGeom &g) { return forcedPath() == 0 && stripCombo(g) && g.oW % 4 == 0 && g.W % 4 == 0; }

int bwdExtraRows(const PoolGeom &g) {
#define X(K, S, P) \
  if (g.kH == K && g.dH == S && g.padH == P) return dev::TapSpan<K, S, S, P>::hi() - dev::TapSpan<K, S, S, P>::lo();
  POOL_STRIP_COMBOS(X)
#undef X
  return 0;
}
size_t fwdStripFloats(const PoolGeom &g, int rows) {
#define X(K, S, P) \
  if (g.kH == K && g.dH == S && g.padH == P) return dev::Strip<K, S, P>::floats(rows, g.W);
  POOL_STRIP_COMBOS(X)
#undef X
  return 0;
}

// ---- runs of memory (pooling_runs.h) ------------------------------------------------
// The strip kernels' window geometries on planes of any width: several whole planes per workgroup
// (planes of at most 2048 elements) or a band of rows of a larger plane. Test switch
// THCUNN_POOL_RUNS: 0 never, 1 also where the strip kernels would be chosen.
struct PoolRunPlan {
  SmallGeom sg;
  int rw, secondFloats;
  size_t lds;
};

template <int KS, int ST, int PAD>
bool poolRunPlanFor(const PoolGeom &g, long planes, bool backward, bool max, PoolRunPlan *out) {
  using R = PoolReach<KS, ST, PAD>;
  using launch::ceilDiv;
  using launch::roundUp;
  const int HW = g.H * g.W, oHW = g.oH * g.oW;
  if (planes >= 0x7fffffffL / 64 || HW < 1 || oHW < 1) return false;
  SmallGeom sg{};
  sg.C = 1, sg.planes = (int)planes;
  if (backward)
    sg.sH = g.oH, sg.sW = g.oW, sg.oH = g.H, sg.oW = g.W;
  else
    sg.sH = g.H, sg.sW = g.W, sg.oH = g.oH, sg.oW = g.oW;
  sg.srcFloats = planes * sg.sH * sg.sW, sg.outFloats = planes * sg.oH * sg.oW;
  const int kRun = launch::kBatchFloats - 3;  // a run and up to 3 floats in front of it are one batch of 16-byte loads
  const int nIdx = max ? 2 : 1;               // max pooling keeps a 32-bit plane of argmax positions beside the values
  auto fetched = [&](int n) { return n + (n % 4 ? 3 : 0); };  // runs of whole planes start on 16-byte boundaries if P planes do
  const int kSlack = backward ? 4 : 7 * ST + KS;  // floats the widest forward item may read past the last staged row
  // staged plane (or band of `rows` produced rows) with its border
  const int LW0 = backward ? std::max(R::BT + sg.sW, (4 * (ceilDiv(g.W, 4) - 1)) / ST + R::first(3) + R::NC) | 1
                           : std::max(PAD + g.W, (g.oW - 1) * ST + KS) | 1;
  const int LHplanes = backward ? std::max(R::BT + sg.sH, R::first(g.H - 1) + R::NC) : std::max(PAD + g.H, (g.oH - 1) * ST + KS);
  auto LHband = [&](int rows) { return backward ? (rows + ST - 2) / ST + R::NC : (rows - 1) * ST + KS; };
  // LDS floats: forward staged planes | values | argmax; backward staged gradOutput | staged argmax | gradInput run
  auto ldsFloats = [&](int P, int LH, int producedPerPlane) {
    const int staged = roundUp(P * LH * LW0 + kSlack, 4), second = roundUp(P * producedPerPlane + 4, 4);
    return (size_t)(backward ? nIdx * staged + second : staged + nIdx * second);
  };
  const int producedPlane = sg.oH * sg.oW, srcPlane = sg.sH * sg.sW;
  if (std::max(HW, oHW) <= 2048) {
    auto fits = [&](int P) {
      return fetched(P * srcPlane) <= launch::kBatchFloats && fetched(P * producedPlane) <= launch::kBatchFloats &&
             ldsFloats(P, LHplanes, producedPlane) * sizeof(float) <= launch::kLdsMax;
    };
    int P = 64;
    while (P > 2 && !fits(P)) P >>= 1;
    if (fits(P)) {
      sg.P = P, sg.bands = 1, sg.rowsPerBand = sg.oH, sg.LH = LHplanes;
    }
  }
  if (sg.P == 0) {
    auto fits = [&](int rows) {
      const int srcRows = std::min(sg.sH, LHband(rows));
      return srcRows * sg.sW <= kRun && rows * sg.oW <= kRun &&
             ldsFloats(1, LHband(rows), rows * sg.oW) * sizeof(float) <= 48 * 1024;
    };
    if (!fits(1)) return false;
    int rows = 1;
    while (rows < sg.oH && fits(rows + 1)) ++rows;
    sg.P = 1, sg.bands = ceilDiv(sg.oH, rows);
    sg.rowsPerBand = ceilDiv(sg.oH, sg.bands);
    if (planes * sg.bands >= 0x7fffffffL) return false;
    sg.LH = LHband(sg.rowsPerBand);
  }
  sg.lp = dev::kBlock / sg.P;
  for (sg.lpShift = 0; (1 << sg.lpShift) < sg.lp; ++sg.lpShift) {
  }
  const int second = roundUp(sg.P * sg.rowsPerBand * sg.oW + 4, 4);
  sg.LW = LW0;
  int rw = 4;
  if (!backward) {
    const int room = (int)((launch::kLdsMax / sizeof(float) - nIdx * second - kSlack - 4) / ((size_t)sg.P * sg.LH));
    const launch::ItemChoice ch = launch::pickItem(3 + (max ? 1 : 0), sg.oW, sg.rowsPerBand, sg.lp, sg.lpShift, sg.LH, ST,
                                                   LW0 & ~1, std::max(room, LW0), false, KS);
    rw = ch.rw, sg.LW = std::max(ch.LW, std::max(PAD + g.W, (g.oW - 1) * ST + KS));
  }
  sg.xsFloats = roundUp(sg.P * sg.LH * sg.LW + kSlack, 4);
  sg.nseg = ceilDiv(sg.oW, rw), sg.nfull = sg.oW / rw;
  sg.magicC = dev::magicOf(1), sg.magicSPlane = dev::magicOf(srcPlane), sg.magicSW = dev::magicOf(sg.sW);
  sg.magicSeg = dev::magicOf(sg.nseg), sg.magicFull = dev::magicOf(std::max(sg.nfull, 1)), sg.magicBands = dev::magicOf(sg.bands);
  out->sg = sg, out->rw = rw, out->secondFloats = second;
  out->lds = (size_t)(backward ? nIdx * sg.xsFloats + second : sg.xsFloats + nIdx * second) * sizeof(float);
  return out->lds <= launch::kLdsMax;
}

int runSwitch() { return g_switches.poolRuns; }
// Where both families apply (widths that are multiples of 4), measured on 8x8 ... 224x224 planes: the run
// kernels' max forward wins up to 112x112 (16x16: 44 -> 12 us, 112x112: 64 -> 62 us; at 224x224 the strip
// kernels are 5-15 % faster); the average forward wins up to 28x28 and the backward passes up to about 36x36
// (a plane per workgroup leaves the strip kernels' lanes idle there), beyond that the strip kernels'
// backward is 10-20 % faster.
bool runsFirst(const PoolGeom &g, bool backward, bool max) {
  if (runSwitch() >= 0) return runSwitch() == 1;
  const long plane = std::max((long)g.H * g.W, (long)g.oH * g.oW);
  if (backward) return plane <= 2048;
  return plane <= (max ? 112 * 112 : 1024);
}

bool poolRunPlan(const PoolGeom &g, long planes, bool backward, bool max, PoolRunPlan *out) {
  if (forcedPath() != 0 || runSwitch() == 0 || !stripCombo(g)) return false;
#define X(K, S, P) \
  if (g.kH == K && g.dH == S && g.padH == P) return poolRunPlanFor<K, S, P>(g, planes, backward, max, out);
  POOL_STRIP_COMBOS(X)
#undef X
  return false;
}

inline unsigned poolRunGrid(const SmallGeom &sg) {
  return sg.bands == 1 ? (unsigned)launch::ceilDiv(sg.planes, sg.P) : (unsigned)((long)sg.planes * sg.bands);
}

template <bool MAX>
void launchPoolRunFwd(hipStream_t s, const PoolGeom &g, const PoolRunPlan &pl, const float *in, float *out, long *indices,
                      bool includePad) {
  const dim3 grid(poolRunGrid(pl.sg));
#define X(K, S, P)                                                                                                        \
  if (g.kH == K && g.dH == S && g.padH == P) {                                                                            \
    if (pl.rw == 7)                                                                                                       \
      poolRunFwd<K, S, P, MAX, 7><<<grid, dev::kBlock, pl.lds, s>>>(in, out, indices, pl.sg, pl.secondFloats, includePad); \
    else                                                                                                                  \
      poolRunFwd<K, S, P, MAX, 4><<<grid, dev::kBlock, pl.lds, s>>>(in, out, indices, pl.sg, pl.secondFloats, includePad); \
  }
  POOL_STRIP_COMBOS(X)
#undef X
}

template <bool MAX>
void launchPoolRunBwd(hipStream_t s, const PoolGeom &g, const PoolRunPlan &pl, const float *gradOut, const long *indices,
                      float *gradIn, bool includePad) {
  const dim3 grid(poolRunGrid(pl.sg));
#define X(K, S, P)                            \
  if (g.kH == K && g.dH == S && g.padH == P) \
    poolRunBwd<K, S, P, MAX><<<grid, dev::kBlock, pl.lds, s>>>(gradOut, indices, gradIn, pl.sg, includePad);
  POOL_STRIP_COMBOS(X)
#undef X
}

// Output extent rule shared by max and average pooling
// (lib/THCUNN/generic/SpatialDilatedMaxPooling.cu:47-64,
//  lib/THCUNN/generic/SpatialAveragePooling.cu:41-58): float division,
// floor/ceil, +1, then - only when padded - drop a last window that would start
// beyond the input plus its leading pad.
long poolExtent(long in, int k, int d, int pad, int dil, bool ceil_mode) {
  float q = float(in - (dil * (k - 1) + 1) + 2 * pad) / float(d);
  return (long)(ceil_mode ? ceilf(q) : floorf(q)) + 1;
}

struct PoolCall {
  PoolGeom g;
  long N, C;
  bool batch;
};

// lib/THCUNN/generic/SpatialDilatedMaxPooling.cu:7-82 / generic/SpatialAveragePooling.cu:7-70
PoolCall poolSetup(THCudaTensor *input, THCudaTensor *gradOutput, THCudaLongTensor *indices, int kH, int kW, int dH,
                   int dW, int padH, int padW, int dilH, int dilW, bool ceil_mode, bool isMax) {
  THC_ARG_CHECK(input != nullptr, 2, "input tensor expected");
  THC_ARG_CHECK(kW > 0 && kH > 0, 5, "kernel size should be greater than zero, but got kH: %d kW: %d", kH, kW);
  THC_ARG_CHECK(dW > 0 && dH > 0, 8, "stride should be greater than zero, but got dH: %d dW: %d", dH, dW);
  if (isMax)
    THC_ARG_CHECK(dilH > 0 && dilW > 0, 12,
                  "dilation should be greater than zero, but got dilationH: %d dilationW: %d", dilH, dilW);
  int ndim = input->nDimension;
  int dimf = 0, dimh = 1, dimw = 2;
  long batchSize = 1;
  THC_ARG_CHECK(ndim == 3 || ndim == 4, 2, "3D or 4D input tensor expected but got: %s",
                sizeDesc(erase(input)).c_str());
  if (ndim == 4) {
    batchSize = input->size[0];
    dimf++;
    dimh++;
    dimw++;
  }
  THC_ARG_CHECK(kW / 2 >= padW && kH / 2 >= padH, 2,
                "pad should be smaller than half of kernel size, but got padW = %d, padH = %d, kW = %d, kH = %d",
                padW, padH, kW, kH);
  long nInputPlane = input->size[dimh - 1];
  long nInputRows = input->size[dimh], nInputCols = input->size[dimw];
  long nOutputCols = poolExtent(nInputCols, kW, dW, padW, dilW, ceil_mode);
  long nOutputRows = poolExtent(nInputRows, kH, dH, padH, dilH, ceil_mode);
  if (padW || padH) {
    if ((nOutputRows - 1) * dH >= nInputRows + padH) --nOutputRows;
    if ((nOutputCols - 1) * dW >= nInputCols + padW) --nOutputCols;
  }
  if (nOutputCols < 1 || nOutputRows < 1)
    error("Given input size: (%ldx%ldx%ld). Calculated output size: (%ldx%ldx%ld). Output size is too small",
          nInputPlane, nInputRows, nInputCols, nInputPlane, nOutputRows, nOutputCols);
  if (gradOutput) {
    checkDimSize(erase(gradOutput), "gradOutput", ndim, dimf, nInputPlane);
    checkDimSize(erase(gradOutput), "gradOutput", ndim, dimh, nOutputRows);
    checkDimSize(erase(gradOutput), "gradOutput", ndim, dimw, nOutputCols);
  }
  if (indices) {
    checkDimSize(erase(indices), "indices", 4, 0, batchSize);
    checkDimSize(erase(indices), "indices", 4, 1, nInputPlane);
    checkDimSize(erase(indices), "indices", 4, 2, nOutputRows);
    checkDimSize(erase(indices), "indices", 4, 3, nOutputCols);
  }
  if (nInputRows * nInputCols >= 0x7fffffffL) error("input planes of 2^31 or more elements are not supported");
  PoolCall c;
  c.batch = ndim == 4;
  c.N = batchSize;
  c.C = nInputPlane;
  PoolGeom &g = c.g;
  g.H = (int)nInputRows, g.W = (int)nInputCols, g.oH = (int)nOutputRows, g.oW = (int)nOutputCols;
  g.kH = kH, g.kW = kW, g.dH = dH, g.dW = dW, g.padH = padH, g.padW = padW, g.dilH = dilH, g.dilW = dilW;
  g.tileRows = g.tilesPerPlane = g.nblk = g.maxStageRows = 0;
  g.magicTiles = 0;
  g.constDiv = 0;
  g.magicDH = dev::magicOf(dH), g.magicDW = dev::magicOf(dW);
  return c;
}

template <bool VEC>
void launchMaxFwd(hipStream_t s, size_t lds, const float *in, float *out, long *idx, const PoolGeom &g) {
  dim3 grid(g.nblk), block(dev::kBlock);
  bool sq = g.kH == g.kW && g.dH == g.dW && g.dilH == 1 && g.dilW == 1;
  if (sq && g.kH == 3 && g.dH == 2)
    maxPoolFwdTiled<3, 2, VEC><<<grid, block, lds, s>>>(in, out, idx, g);
  else if (sq && g.kH == 2 && g.dH == 2)
    maxPoolFwdTiled<2, 2, VEC><<<grid, block, lds, s>>>(in, out, idx, g);
  else if (sq && g.kH == 3 && g.dH == 1)
    maxPoolFwdTiled<3, 1, VEC><<<grid, block, lds, s>>>(in, out, idx, g);
  else
    maxPoolFwdTiled<0, 0, VEC><<<grid, block, lds, s>>>(in, out, idx, g);
}

void maxPoolUpdateOutput(THCState *state, THCudaTensor *input, THCudaTensor *output, THCudaLongTensor *indices,
                         int kW, int kH, int dW, int dH, int padW, int padH, int dilW, int dilH, bool ceil_mode) {
  THC_ARG_CHECK(output != nullptr, 3, "output tensor expected");
  THC_ARG_CHECK(indices != nullptr, 4, "indices tensor expected");
  PoolCall call = poolSetup(input, nullptr, nullptr, kH, kW, dH, dW, padH, padW, dilH, dilW, ceil_mode, true);
  PoolGeom &g = call.g;
  Contiguous in(state, input);
  resize(state, output, {call.N, call.C, g.oH, g.oW});
  resize(state, indices, {call.N, call.C, g.oH, g.oW});  // always 4-D (:140-141)
  if (!isContiguous(erase(output)) || !isContiguous(erase(indices)))
    error("output and indices tensors have to be contiguous");
  hipStream_t s = state->stream;
  const long planes = call.N * call.C;
  if (planes > 0) {
    bool vec = g.W % 4 == 0 && aligned16(in.ptr());
    auto stageRows = [&](int rows) { return std::min(g.H, (rows - 1) * g.dH + (g.kH - 1) * g.dilH + 1); };
    auto bytes = [&](int rows) { return (size_t)stageRows(rows) * g.W * sizeof(float); };
    auto sbytes = [&](int rows) { return fwdStripFloats(g, (rows - 1) * g.dH + g.kH) * sizeof(float); };
    auto staged = [&](int rows) { return (size_t)((rows - 1) * g.dH + g.kH) * g.W; };
    SmallPool sp;
    PoolRunPlan rp;
    size_t slds;
    const bool haveRuns = aligned16(in.ptr()) && aligned16(data(output)) && aligned16(data(indices)) &&
                          poolRunPlan(g, planes, false, true, &rp);
    if (stripFwdOk(g) && !(haveRuns && runsFirst(g, false, true)) && vec && aligned16(data(output)) && aligned16(data(indices)) &&
        launch::pickBand(g.oH, planes, sbytes, &g.tileRows, &g.tilesPerPlane, staged)) {
      g.nblk = (int)(planes * g.tilesPerPlane);
      g.magicTiles = dev::magicOf(g.tilesPerPlane);
      dim3 grid(g.nblk), block(dev::kBlock);
      size_t lds = sbytes(g.tileRows);
#define X(K, S, P)                                  \
  if (g.kH == K && g.dH == S && g.padH == P)       \
    maxPoolFwdStrip<K, S, P><<<grid, block, lds, s>>>(in.ptr(), data(output), data(indices), g);
      POOL_STRIP_COMBOS(X)
#undef X
    } else if (haveRuns) {
      launchPoolRunFwd<true>(s, g, rp, in.ptr(), data(output), data(indices), false);
    } else if (smallPoolPlan(g, planes, false, true, in.ptr(), in.ptr(), &sp, &slds)) {
      poolFwdSmall<true, false><<<launch::ceilDiv(sp.planes, sp.P), dev::kBlock, slds, s>>>(in.ptr(), data(output),
                                                                                           data(indices), g, sp);
    } else if (!forceDirect() && launch::pickBand(g.oH, planes, bytes, &g.tileRows, &g.tilesPerPlane)) {
      g.nblk = (int)(planes * g.tilesPerPlane);
      g.magicTiles = dev::magicOf(g.tilesPerPlane);
      if (vec)
        launchMaxFwd<true>(s, bytes(g.tileRows), in.ptr(), data(output), data(indices), g);
      else
        launchMaxFwd<false>(s, bytes(g.tileRows), in.ptr(), data(output), data(indices), g);
    } else {
      long total = planes * g.oH * g.oW;
      maxPoolFwdDirect<<<launch::directGrid(total, dev::kBlock), dev::kBlock, 0, s>>>(in.ptr(), data(output),
                                                                                      data(indices), g, total);
    }
    THC_HIP_CHECK(hipGetLastError());
  }
  if (!call.batch) resize(state, output, {call.C, g.oH, g.oW});
}

void maxPoolUpdateGradInput(THCState *state, THCudaTensor *input, THCudaTensor *gradOutput, THCudaTensor *gradInput,
                            THCudaLongTensor *indices, int kW, int kH, int dW, int dH, int padW, int padH, int dilW,
                            int dilH, bool ceil_mode) {
  THC_ARG_CHECK(gradOutput != nullptr, 3, "gradOutput tensor expected");
  THC_ARG_CHECK(gradInput != nullptr, 4, "gradInput tensor expected");
  THC_ARG_CHECK(indices != nullptr, 5, "indices tensor expected");
  PoolCall call = poolSetup(input, gradOutput, indices, kH, kW, dH, dW, padH, padW, dilH, dilW, ceil_mode, true);
  PoolGeom &g = call.g;
  Contiguous go(state, gradOutput);
  if (!isContiguous(erase(indices))) error("indices tensor has to be contiguous");
  if (call.batch)
    resize(state, gradInput, {call.N, call.C, g.H, g.W});
  else
    resize(state, gradInput, {call.C, g.H, g.W});
  if (!isContiguous(erase(gradInput))) error("gradInput tensor has to be contiguous");
  hipStream_t s = state->stream;
  const long planes = call.N * call.C;
  if (planes == 0) return;
  const int extH = (g.kH - 1) * g.dilH + 1;
  bool vec = g.oW % 4 == 0 && aligned16(go.ptr());
  auto stageRows = [&](int rows) { return std::min(g.oH, (rows + extH - 2) / g.dH + 2); };
  auto bytes = [&](int rows) { return (size_t)stageRows(rows) * g.oW * (sizeof(float) + sizeof(int)); };
  const int extra = bwdExtraRows(g);
  const int spitch = g.oW + dev::kStripPadL;
  auto sbytes = [&](int units) { return 2 * ((size_t)(units + extra) * spitch + dev::kStripPadL) * sizeof(float); };
  int units = 0;
  SmallPool sp;
    PoolRunPlan rp;
  size_t slds;
  const bool haveRuns = aligned16(go.ptr()) && aligned16(data(gradInput)) && aligned16(data(indices)) &&
                        poolRunPlan(g, planes, true, true, &rp);
  if (stripBwdOk(g) && !(haveRuns && runsFirst(g, true, true)) && vec && aligned16(data(gradInput)) &&
      launch::pickBand(launch::ceilDiv(g.H, g.dH), planes, sbytes, &units, &g.tilesPerPlane)) {
    g.tileRows = units * g.dH;
    g.nblk = (int)(planes * g.tilesPerPlane);
      g.magicTiles = dev::magicOf(g.tilesPerPlane);
    dim3 grid(g.nblk), block(dev::kBlock);
    size_t lds = sbytes(units);
#define X(K, S, P)                            \
  if (g.kH == K && g.dH == S && g.padH == P) \
    poolBwdStrip<K, S, P, true, true><<<grid, block, lds, s>>>(go.ptr(), data(indices), data(gradInput), g, units + extra);
    POOL_STRIP_COMBOS(X)
#undef X
  } else if (haveRuns) {
    launchPoolRunBwd<true>(s, g, rp, go.ptr(), data(indices), data(gradInput), false);
  } else if (smallPoolPlan(g, planes, true, true, data(gradInput), data(gradInput), &sp, &slds)) {
    poolBwdSmall<true, false><<<launch::ceilDiv(sp.planes, sp.P), dev::kBlock, slds, s>>>(go.ptr(), data(indices),
                                                                                         data(gradInput), g, sp);
  } else if (!forceDirect() && launch::pickBand(g.H, planes, bytes, &g.tileRows, &g.tilesPerPlane)) {
    g.nblk = (int)(planes * g.tilesPerPlane);
      g.magicTiles = dev::magicOf(g.tilesPerPlane);
    g.maxStageRows = stageRows(g.tileRows);
    dim3 grid(g.nblk), block(dev::kBlock);
    if (vec)
      maxPoolBwdTiled<true><<<grid, block, bytes(g.tileRows), s>>>(go.ptr(), data(indices), data(gradInput), g);
    else
      maxPoolBwdTiled<false><<<grid, block, bytes(g.tileRows), s>>>(go.ptr(), data(indices), data(gradInput), g);
  } else {
    long total = planes * g.H * g.W;
    maxPoolBwdDirect<<<launch::directGrid(total, dev::kBlock), dev::kBlock, 0, s>>>(go.ptr(), data(indices),
                                                                                    data(gradInput), g, total);
  }
  THC_HIP_CHECK(hipGetLastError());
}

}  // namespace

extern "C" {

void THNN_CudaSpatialDilatedMaxPooling_updateOutput(THCState *state, THCudaTensor *input, THCudaTensor *output,
                                                    THCudaLongTensor *indices, int kW, int kH, int dW, int dH,
                                                    int padW, int padH, int dilationW, int dilationH,
                                                    bool ceil_mode) {
  THNN_ENTER
  maxPoolUpdateOutput(state, input, output, indices, kW, kH, dW, dH, padW, padH, dilationW, dilationH, ceil_mode);
  THNN_LEAVE
}

void THNN_CudaSpatialDilatedMaxPooling_updateGradInput(THCState *state, THCudaTensor *input,
                                                       THCudaTensor *gradOutput, THCudaTensor *gradInput,
                                                       THCudaLongTensor *indices, int kW, int kH, int dW, int dH,
                                                       int padW, int padH, int dilationW, int dilationH,
                                                       bool ceil_mode) {
  THNN_ENTER
  maxPoolUpdateGradInput(state, input, gradOutput, gradInput, indices, kW, kH, dW, dH, padW, padH, dilationW,
                         dilationH, ceil_mode);
  THNN_LEAVE
}

// lib/THCUNN/generic/SpatialMaxPooling.cu:7-38: dilation 1
void THNN_CudaSpatialMaxPooling_updateOutput(THCState *state, THCudaTensor *input, THCudaTensor *output,
                                             THCudaLongTensor *indices, int kW, int kH, int dW, int dH, int padW,
                                             int padH, bool ceil_mode) {
  THNN_ENTER
  maxPoolUpdateOutput(state, input, output, indices, kW, kH, dW, dH, padW, padH, 1, 1, ceil_mode);
  THNN_LEAVE
}

void THNN_CudaSpatialMaxPooling_updateGradInput(THCState *state, THCudaTensor *input, THCudaTensor *gradOutput,
                                                THCudaTensor *gradInput, THCudaLongTensor *indices, int kW, int kH,
                                                int dW, int dH, int padW, int padH, bool ceil_mode) {
  THNN_ENTER
  maxPoolUpdateGradInput(state, input, gradOutput, gradInput, indices, kW, kH, dW, dH, padW, padH, 1, 1, ceil_mode);
  THNN_LEAVE
}

void THNN_CudaSpatialAveragePooling_updateOutput(THCState *state, THCudaTensor *input, THCudaTensor *output, int kW,
                                                 int kH, int dW, int dH, int padW, int padH, bool ceil_mode,
                                                 bool count_include_pad) {
  THNN_ENTER
  THC_ARG_CHECK(output != nullptr, 3, "output tensor expected");
  PoolCall call = poolSetup(input, nullptr, nullptr, kH, kW, dH, dW, padH, padW, 1, 1, ceil_mode, false);
  PoolGeom &g = call.g;
  g.constDiv = avgConstDivisor(g, count_include_pad);
  Contiguous in(state, input);
  resize(state, output, {call.N, call.C, g.oH, g.oW});
  if (!isContiguous(erase(output))) error("output tensor has to be contiguous");
  hipStream_t s = state->stream;
  const long planes = call.N * call.C;
  if (planes > 0) {
    bool vec = g.W % 4 == 0 && aligned16(in.ptr());
    auto stageRows = [&](int rows) { return std::min(g.H, (rows - 1) * g.dH + g.kH); };
    auto bytes = [&](int rows) { return (size_t)stageRows(rows) * g.W * sizeof(float); };
    auto sbytes = [&](int rows) { return fwdStripFloats(g, (rows - 1) * g.dH + g.kH) * sizeof(float); };
    auto staged = [&](int rows) { return (size_t)((rows - 1) * g.dH + g.kH) * g.W; };
    SmallPool sp;
    PoolRunPlan rp;
    size_t slds;
    const bool haveRuns = aligned16(in.ptr()) && aligned16(data(output)) && poolRunPlan(g, planes, false, false, &rp);
    if (avgGlobalOk(g, planes)) {
      const long waves = std::min<long>((planes + 3) / 4, 8192);
      avgPoolGlobalFwd<<<(unsigned)((waves + 3) / 4), dev::kBlock, 0, s>>>(in.ptr(), data(output), planes, g.H * g.W);
    } else if (avgFlatOk(g, planes) && vec && aligned16(data(output))) {
      const unsigned total = (unsigned)(planes * g.oH * (g.oW / 4));
      const unsigned grid = (total + dev::kBlock - 1) / dev::kBlock;
      const unsigned magic = dev::magicOf(g.oW / 4);
      if (g.kH == 2) avgPoolFwdFlat<2><<<grid, dev::kBlock, 0, s>>>(in.ptr(), data(output), g.oW / 4, magic, g.W, total);
      if (g.kH == 3) avgPoolFwdFlat<3><<<grid, dev::kBlock, 0, s>>>(in.ptr(), data(output), g.oW / 4, magic, g.W, total);
      if (g.kH == 4) avgPoolFwdFlat<4><<<grid, dev::kBlock, 0, s>>>(in.ptr(), data(output), g.oW / 4, magic, g.W, total);
    } else if (stripFwdOk(g) && !(haveRuns && runsFirst(g, false, false)) && vec && aligned16(data(output)) &&
        launch::pickBand(g.oH, planes, sbytes, &g.tileRows, &g.tilesPerPlane, staged)) {
      g.nblk = (int)(planes * g.tilesPerPlane);
      g.magicTiles = dev::magicOf(g.tilesPerPlane);
      dim3 grid(g.nblk), block(dev::kBlock);
      size_t lds = sbytes(g.tileRows);
#define X(K, S, P)                                                                        \
  if (g.kH == K && g.dH == S && g.padH == P) {                                           \
    if (count_include_pad)                                                               \
      avgPoolFwdStrip<K, S, P, true><<<grid, block, lds, s>>>(in.ptr(), data(output), g);  \
    else                                                                                 \
      avgPoolFwdStrip<K, S, P, false><<<grid, block, lds, s>>>(in.ptr(), data(output), g); \
  }
      POOL_STRIP_COMBOS(X)
#undef X
    } else if (haveRuns) {
      launchPoolRunFwd<false>(s, g, rp, in.ptr(), data(output), nullptr, count_include_pad);
    } else if (smallPoolPlan(g, planes, false, false, in.ptr(), in.ptr(), &sp, &slds)) {
      const unsigned grid = launch::ceilDiv(sp.planes, sp.P);
      if (count_include_pad)
        poolFwdSmall<false, true><<<grid, dev::kBlock, slds, s>>>(in.ptr(), data(output), nullptr, g, sp);
      else
        poolFwdSmall<false, false><<<grid, dev::kBlock, slds, s>>>(in.ptr(), data(output), nullptr, g, sp);
    } else if (!forceDirect() && launch::pickBand(g.oH, planes, bytes, &g.tileRows, &g.tilesPerPlane)) {
      g.nblk = (int)(planes * g.tilesPerPlane);
      g.magicTiles = dev::magicOf(g.tilesPerPlane);
      dim3 grid(g.nblk), block(dev::kBlock);
      size_t lds = bytes(g.tileRows);
      if (count_include_pad) {
        if (vec)
          avgPoolFwdTiled<true, true><<<grid, block, lds, s>>>(in.ptr(), data(output), g);
        else
          avgPoolFwdTiled<true, false><<<grid, block, lds, s>>>(in.ptr(), data(output), g);
      } else {
        if (vec)
          avgPoolFwdTiled<false, true><<<grid, block, lds, s>>>(in.ptr(), data(output), g);
        else
          avgPoolFwdTiled<false, false><<<grid, block, lds, s>>>(in.ptr(), data(output), g);
      }
    } else {
      long total = planes * g.oH * g.oW;
      unsigned grid = launch::directGrid(total, dev::kBlock);
      if (count_include_pad)
        avgPoolFwdDirect<true><<<grid, dev::kBlock, 0, s>>>(in.ptr(), data(output), g, total);
      else
        avgPoolFwdDirect<false><<<grid, dev::kBlock, 0, s>>>(in.ptr(), data(output), g, total);
    }
    THC_HIP_CHECK(hipGetLastError());
  }
  if (!call.batch) resize(state, output, {call.C, g.oH, g.oW});
  THNN_LEAVE
}

void THNN_CudaSpatialAveragePooling_updateGradInput(THCState *state, THCudaTensor *input, THCudaTensor *gradOutput,
                                                    THCudaTensor *gradInput, int kW, int kH, int dW, int dH,
                                                    int padW, int padH, bool ceil_mode, bool count_include_pad) {
  THNN_ENTER
  THC_ARG_CHECK(gradOutput != nullptr, 3, "gradOutput tensor expected");
  THC_ARG_CHECK(gradInput != nullptr, 4, "gradInput tensor expected");
  PoolCall call = poolSetup(input, gradOutput, nullptr, kH, kW, dH, dW, padH, padW, 1, 1, ceil_mode, false);
  PoolGeom &g = call.g;
  g.constDiv = avgConstDivisor(g, count_include_pad);
  Contiguous go(state, gradOutput);
  if (call.batch)
    resize(state, gradInput, {call.N, call.C, g.H, g.W});
  else
    resize(state, gradInput, {call.C, g.H, g.W});
  if (!isContiguous(erase(gradInput))) error("gradInput tensor has to be contiguous");
  hipStream_t s = state->stream;
  const long planes = call.N * call.C;
  if (planes == 0) return;
  bool vec = g.oW % 4 == 0 && aligned16(go.ptr());
  auto stageRows = [&](int rows) { return std::min(g.oH, (rows + g.kH - 2) / g.dH + 2); };
  auto bytes = [&](int rows) { return (size_t)stageRows(rows) * g.oW * sizeof(float); };
  const int extra = bwdExtraRows(g);
  const int spitch = g.oW + dev::kStripPadL;
  auto sbytes = [&](int units) { return ((size_t)(units + extra) * spitch + dev::kStripPadL) * sizeof(float); };
  int units = 0;
  SmallPool sp;
    PoolRunPlan rp;
  size_t slds;
  const bool haveRuns = aligned16(go.ptr()) && aligned16(data(gradInput)) && poolRunPlan(g, planes, true, false, &rp);
  if (avgGlobalOk(g, planes)) {
    const unsigned total = (unsigned)(planes * g.H * g.W);
    avgPoolGlobalBwd<<<launch::directGrid(total, dev::kBlock), dev::kBlock, 0, s>>>(go.ptr(), data(gradInput), total,
                                                                                    g.H * g.W, dev::magicOf(g.H * g.W));
  } else if (avgFlatOk(g, planes) && vec && aligned16(data(gradInput)) && planes * g.H * (g.W / 4) * (g.W / 4) < 0xffffffffL) {
    const unsigned total = (unsigned)(planes * g.oH * (g.W / 4));
    const unsigned grid = (total + dev::kBlock - 1) / dev::kBlock;
    const unsigned magic = dev::magicOf(g.W / 4);
    if (g.kH == 2) avgPoolBwdFlat<2><<<grid, dev::kBlock, 0, s>>>(go.ptr(), data(gradInput), g.W / 4, magic, g.oW, total);
    if (g.kH == 3) avgPoolBwdFlat<3><<<grid, dev::kBlock, 0, s>>>(go.ptr(), data(gradInput), g.W / 4, magic, g.oW, total);
    if (g.kH == 4) avgPoolBwdFlat<4><<<grid, dev::kBlock, 0, s>>>(go.ptr(), data(gradInput), g.W / 4, magic, g.oW, total);
  } else if (stripBwdOk(g) && !(haveRuns && runsFirst(g, true, false)) && vec && aligned16(data(gradInput)) &&
      launch::pickBand(launch::ceilDiv(g.H, g.dH), planes, sbytes, &units, &g.tilesPerPlane)) {
    g.tileRows = units * g.dH;
    g.nblk = (int)(planes * g.tilesPerPlane);
      g.magicTiles = dev::magicOf(g.tilesPerPlane);
    dim3 grid(g.nblk), block(dev::kBlock);
    size_t lds = sbytes(units);
#define X(K, S, P)                                                                                                    \
  if (g.kH == K && g.dH == S && g.padH == P) {                                                                       \
    if (count_include_pad)                                                                                           \
      poolBwdStrip<K, S, P, false, true><<<grid, block, lds, s>>>(go.ptr(), nullptr, data(gradInput), g, units + extra);  \
    else                                                                                                             \
      poolBwdStrip<K, S, P, false, false><<<grid, block, lds, s>>>(go.ptr(), nullptr, data(gradInput), g, units + extra); \
  }
    POOL_STRIP_COMBOS(X)
#undef X
  } else if (haveRuns) {
    launchPoolRunBwd<false>(s, g, rp, go.ptr(), nullptr, data(gradInput), count_include_pad);
  } else if (smallPoolPlan(g, planes, true, false, data(gradInput), data(gradInput), &sp, &slds)) {
    const unsigned grid = launch::ceilDiv(sp.planes, sp.P);
    if (count_include_pad)
      poolBwdSmall<false, true><<<grid, dev::kBlock, slds, s>>>(go.ptr(), nullptr, data(gradInput), g, sp);
    else
      poolBwdSmall<false, false><<<grid, dev::kBlock, slds, s>>>(go.ptr(), nullptr, data(gradInput), g, sp);
  } else if (!forceDirect() && launch::pickBand(g.H, planes, bytes, &g.tileRows, &g.tilesPerPlane)) {
    g.nblk = (int)(planes * g.tilesPerPlane);
      g.magicTiles = dev::magicOf(g.tilesPerPlane);
    dim3 grid(g.nblk), block(dev::kBlock);
    size_t lds = bytes(g.tileRows);
    if (count_include_pad) {
      if (vec)
        avgPoolBwdTiled<true, true><<<grid, block, lds, s>>>(go.ptr(), data(gradInput), g);
      else
        avgPoolBwdTiled<true, false><<<grid, block, lds, s>>>(go.ptr(), data(gradInput), g);
    } else {
      if (vec)
        avgPoolBwdTiled<false, true><<<grid, block, lds, s>>>(go.ptr(), data(gradInput), g);
      else
        avgPoolBwdTiled<false, false><<<grid, block, lds, s>>>(go.ptr(), data(gradInput), g);
    }
  } else {
    long total = planes * g.H * g.W;
    unsigned grid = launch::directGrid(total, dev::kBlock);
    if (count_include_pad)
      avgPoolBwdDirect<true><<<grid, dev::kBlock, 0, s>>>(go.ptr(), data(gradInput), g, total);
    else
      avgPoolBwdDirect<false><<<grid, dev::kBlock, 0, s>>>(go.ptr(), data(gradInput), g, total);
  }
  THC_HIP_CHECK(hipGetLastError());
  THNN_LEAVE
}

}  // extern "C"
