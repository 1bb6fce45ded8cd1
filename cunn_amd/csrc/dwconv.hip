// SpatialDepthWiseConvolution for gfx950: one fused, bandwidth-bound kernel per
// entry point instead of the reference's 2-3 launches per (image, channel)
// (lib/THCUNN/generic/SpatialDepthWiseConvolution.cu:150-226, 350-395, 531-615).
//
// Data layout: input (N,C,H,W), output/gradOutput (N,C*M,oH,oW) with
// out-channel c*M+j (:121,244), weight (M,C,kH,kW) read through its strides,
// bias (M,C). A workgroup owns a band of rows of one (n,c) plane: the band
// (plus halo, zero padded) is staged once in LDS with 16-byte transfers, every
// tap is then an LDS read, and results leave through coalesced stores, so each
// input byte crosses HBM once. Weight gradients are reduced without atomics:
// per-lane partial sums -> 64-lane shuffle tree -> cross-wave LDS -> one partial
// per workgroup in scratch, then a second small kernel folds the partials in a
// fixed order (deterministic) and accumulates into gradWeight/gradBias.
#include "device_utils.h"
#include "launch_utils.h"
#include "strip.h"
#include "thc_internal.h"

#include <atomic>
#include <mutex>

using namespace thc;

namespace {

struct Strides4 {
  long s0, s1, s2, s3;
};
struct Strides2 {
  long s0, s1;
};

struct DwGeom {
  int N, C, M, H, W, oH, oW;
  int kH, kW, dH, dW, padH, padW;
  int tileRows;       // rows of the tiled tensor one workgroup produces
  int tilesPerPlane;  // workgroups per (n,c) plane
  int pitch, padL;    // LDS row pitch / left zero pad of the staged input band
  int nblk;           // grid size
  int nslots;         // N * tilesPerPlane (accGradParameters partials per (c,j) and tap)
  unsigned magicTiles, magicC;  // dev::magicOf(tilesPerPlane), dev::magicOf(C): used by the strip kernels
  unsigned magicOW4, magicW4;   // dev::magicOf(oW / 4), dev::magicOf(W / 4)
};

// (plane, tile, channel) of a workgroup of the strip kernels
struct BlockPos {
  int plane, tile, c;
};
__device__ __forceinline__ BlockPos blockPos(const DwGeom &g) {
  const int bid = blockIdx.x;  // consecutive workgroups work on neighbouring planes: one compact window of memory in flight
  BlockPos b;
  b.plane = g.tilesPerPlane == 1 ? bid : dev::fastDiv(bid, g.magicTiles);
  b.tile = bid - b.plane * g.tilesPerPlane;
  b.c = b.plane - dev::fastDiv(b.plane, g.magicC) * g.C;
  return b;
}

// The KS*KS taps of (multiplier j, channel c) into registers; one wide scalar
// load when the kernel plane is contiguous.
template <int KS>
__device__ __forceinline__ void loadTaps(const float *__restrict__ weight, const Strides4 &ws, int j, int c,
                                         float (&w)[KS * KS]) {
  const float *wp = weight + j * ws.s0 + c * ws.s1;
  if (ws.s3 == 1 && ws.s2 == KS) {
#pragma unroll
    for (int t = 0; t < KS * KS; ++t) w[t] = wp[t];
  } else {
#pragma unroll
    for (int kh = 0; kh < KS; ++kh)
#pragma unroll
      for (int kw = 0; kw < KS; ++kw) w[kh * KS + kw] = wp[kh * ws.s2 + kw * ws.s3];
  }
}

#include "dwconv_small.h"

// ------------------------------------------------------------------ forward --
// KS/ST > 0: square kernel / stride known at compile time (taps in registers,
// fully unrolled); 0: runtime geometry.
template <int KS, int ST, bool VEC>
__global__ void __launch_bounds__(dev::kBlock)
dwFwdTiled(const float *__restrict__ in, const float *__restrict__ weight, Strides4 ws,
           const float *__restrict__ bias, Strides2 bs, float *__restrict__ out, DwGeom g) {
  extern __shared__ float smem[];
  const int kH = KS ? KS : g.kH, kW = KS ? KS : g.kW;
  const int dH = ST ? ST : g.dH, dW = ST ? ST : g.dW;
  const int bid = dev::xcdRemap(blockIdx.x, g.nblk);
  const int plane = bid / g.tilesPerPlane, tile = bid - plane * g.tilesPerPlane;
  const int c = plane % g.C;
  const int oh0 = tile * g.tileRows;
  const int nOut = min(g.tileRows, g.oH - oh0);
  const int nIn = (nOut - 1) * dH + kH;
  float *xs = smem;
  float *wsm = smem + (size_t)((g.tileRows - 1) * dH + kH) * g.pitch + g.padL;  // M*kH*kW taps

  dev::loadRowsPadded<VEC>(xs, in + (long)plane * g.H * g.W, g.H, g.W, oh0 * dH - g.padH, nIn, g.pitch, g.padL);
  const int nTap = kH * kW;
  for (int i = threadIdx.x; i < g.M * nTap; i += blockDim.x) {
    int j = i / nTap, t = i - j * nTap;
    int kh = t / kW, kw = t - kh * kW;
    wsm[i] = weight[j * ws.s0 + c * ws.s1 + kh * ws.s2 + kw * ws.s3];
  }
  __syncthreads();

  const int colOff = g.padL - g.padW;
  const int total = nOut * g.oW;
  for (int j = 0; j < g.M; ++j) {
    const float b = bias ? bias[j * bs.s0 + c * bs.s1] : 0.f;
    float *o = out + (((long)plane * g.M + j) * g.oH + oh0) * g.oW;
    const float *wj = wsm + j * nTap;
    if (KS) {
      float w[KS ? KS * KS : 1];
#pragma unroll
      for (int t = 0; t < KS * KS; ++t) w[t] = wj[t];
      for (int i = threadIdx.x; i < total; i += blockDim.x) {
        int r = i / g.oW, ow = i - r * g.oW;
        const float *p = xs + r * dH * g.pitch + ow * dW + colOff;
        float acc = b;
#pragma unroll
        for (int kh = 0; kh < KS; ++kh)
#pragma unroll
          for (int kw = 0; kw < KS; ++kw) acc = fmaf(p[kh * g.pitch + kw], w[kh * KS + kw], acc);
        o[i] = acc;
      }
    } else {
      for (int i = threadIdx.x; i < total; i += blockDim.x) {
        int r = i / g.oW, ow = i - r * g.oW;
        const float *p = xs + r * dH * g.pitch + ow * dW + colOff;
        float acc = b;
        for (int kh = 0; kh < kH; ++kh)
          for (int kw = 0; kw < kW; ++kw) acc = fmaf(p[kh * g.pitch + kw], wj[kh * kW + kw], acc);
        o[i] = acc;
      }
    }
  }
}

// Any geometry, no LDS: one lane per output element, taps read through the cache.
__global__ void __launch_bounds__(dev::kBlock)
dwFwdDirect(const float *__restrict__ in, const float *__restrict__ weight, Strides4 ws,
            const float *__restrict__ bias, Strides2 bs, float *__restrict__ out, DwGeom g, long total) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    int ow = (int)(i % g.oW);
    long t = i / g.oW;
    int oh = (int)(t % g.oH);
    t /= g.oH;
    int j = (int)(t % g.M);
    long plane = t / g.M;
    int c = (int)(plane % g.C);
    const float *ip = in + plane * g.H * g.W;
    float acc = bias ? bias[j * bs.s0 + c * bs.s1] : 0.f;
    for (int kh = 0; kh < g.kH; ++kh) {
      int h = oh * g.dH - g.padH + kh;
      if (h < 0 || h >= g.H) continue;
      for (int kw = 0; kw < g.kW; ++kw) {
        int w = ow * g.dW - g.padW + kw;
        if (w < 0 || w >= g.W) continue;
        acc = fmaf(ip[(long)h * g.W + w], weight[j * ws.s0 + c * ws.s1 + kh * ws.s2 + kw * ws.s3], acc);
      }
    }
    out[i] = acc;
  }
}

// ---------------------------------------------------------------- gradInput --
// A workgroup produces rows [h0, h0+nRows) of one gradInput plane from the
// gradOutput rows that reach them (all M multipliers), staged in LDS.
template <int KS, int ST, bool VEC>
__global__ void __launch_bounds__(dev::kBlock)
dwGradInputTiled(const float *__restrict__ gradOut, const float *__restrict__ weight, Strides4 ws,
                 float *__restrict__ gradIn, DwGeom g, int maxOhRows) {
  extern __shared__ float smem[];
  const int kH = KS ? KS : g.kH, kW = KS ? KS : g.kW;
  const int dH = ST ? ST : g.dH, dW = ST ? ST : g.dW;
  const int bid = dev::xcdRemap(blockIdx.x, g.nblk);
  const int plane = bid / g.tilesPerPlane, tile = bid - plane * g.tilesPerPlane;
  const int c = plane % g.C;
  const int h0 = tile * g.tileRows;
  const int nRows = min(g.tileRows, g.H - h0);
  // gradOutput rows touching input rows [h0, h0+nRows)
  const int ohLo = max(0, dev::ceilDivPos(h0 + g.padH - kH + 1, dH));
  const int ohHi = min(g.oH - 1, (h0 + nRows - 1 + g.padH) / dH);
  const int nOh = max(0, ohHi - ohLo + 1);
  float *gs = smem;                                   // [M][maxOhRows][oW]
  float *wsm = smem + (size_t)g.M * maxOhRows * g.oW;  // [M][kH*kW]
  const int nTap = kH * kW;
  const long L = (long)g.oH * g.oW;
  for (int j = 0; j < g.M; ++j)
    dev::loadFlat<VEC>(gs + (size_t)j * maxOhRows * g.oW,
                       gradOut + ((long)plane * g.M + j) * L + (long)ohLo * g.oW, nOh * g.oW);
  for (int i = threadIdx.x; i < g.M * nTap; i += blockDim.x) {
    int j = i / nTap, t = i - j * nTap;
    int kh = t / kW, kw = t - kh * kW;
    wsm[i] = weight[j * ws.s0 + c * ws.s1 + kh * ws.s2 + kw * ws.s3];
  }
  __syncthreads();

  float *o = gradIn + ((long)plane * g.H + h0) * g.W;
  const int total = nRows * g.W;
  for (int i = threadIdx.x; i < total; i += blockDim.x) {
    int r = i / g.W, w = i - r * g.W;
    int hp = h0 + r + g.padH, wp = w + g.padW;
    int ohs = (hp < kH) ? 0 : (hp - kH) / dH + 1;
    int ohe = min(hp / dH + 1, g.oH);
    int ows = (wp < kW) ? 0 : (wp - kW) / dW + 1;
    int owe = min(wp / dW + 1, g.oW);
    float acc = 0.f;
    for (int j = 0; j < g.M; ++j) {
      const float *gj = gs + (size_t)j * maxOhRows * g.oW;
      const float *wj = wsm + j * nTap;
      for (int oh = ohs; oh < ohe; ++oh) {
        int kh = hp - oh * dH;
        for (int ow = ows; ow < owe; ++ow) {
          int kw = wp - ow * dW;
          acc = fmaf(gj[(oh - ohLo) * g.oW + ow], wj[kh * kW + kw], acc);
        }
      }
    }
    o[i] = acc;
  }
}

__global__ void __launch_bounds__(dev::kBlock)
dwGradInputDirect(const float *__restrict__ gradOut, const float *__restrict__ weight, Strides4 ws,
                  float *__restrict__ gradIn, DwGeom g, long total) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    int w = (int)(i % g.W);
    long t = i / g.W;
    int h = (int)(t % g.H);
    long plane = t / g.H;
    int c = (int)(plane % g.C);
    int hp = h + g.padH, wp = w + g.padW;
    int ohs = (hp < g.kH) ? 0 : (hp - g.kH) / g.dH + 1;
    int ohe = min(hp / g.dH + 1, g.oH);
    int ows = (wp < g.kW) ? 0 : (wp - g.kW) / g.dW + 1;
    int owe = min(wp / g.dW + 1, g.oW);
    float acc = 0.f;
    for (int j = 0; j < g.M; ++j) {
      const float *gj = gradOut + (plane * g.M + j) * g.oH * g.oW;
      for (int oh = ohs; oh < ohe; ++oh) {
        int kh = hp - oh * g.dH;
        for (int ow = ows; ow < owe; ++ow) {
          int kw = wp - ow * g.dW;
          acc = fmaf(gj[(long)oh * g.oW + ow], weight[j * ws.s0 + c * ws.s1 + kh * ws.s2 + kw * ws.s3], acc);
        }
      }
    }
    gradIn[i] = acc;
  }
}

// -------------------------------------------------------- accGradParameters --
// floats between the partial runs of neighbouring (slot, c, j): the T sums rounded up to whole 64-byte groups
__host__ __device__ constexpr int partialPitch(int T) { return (T + 15) & ~15; }

// Stage 1: per workgroup, partial sums over its band of one (n,c) plane of
//   gw[tap] = sum gy[oh,ow] * x[oh*d-p+kh, ow*d-p+kw]   and   gb = sum gy
// written to partial[(slot * C*M + c*M+j) * TP + tap], T = KS*KS + 1, TP = T rounded up to 16 (partialPitch):
// what a workgroup leaves is one aligned run of 64 or 128 bytes.
template <int KS, int ST, bool VEC, bool VECG>
__global__ void __launch_bounds__(dev::kBlock)
dwAccGradStage1(const float *__restrict__ in, const float *__restrict__ gradOut, float *__restrict__ partial,
                DwGeom g) {
  extern __shared__ float smem[];
  constexpr int T = KS * KS + 1;
  constexpr int nWaves = dev::kBlock / dev::kWave;
  const int bid = dev::xcdRemap(blockIdx.x, g.nblk);
  const int plane = bid / g.tilesPerPlane, tile = bid - plane * g.tilesPerPlane;
  const int n = plane / g.C, c = plane - n * g.C;
  const int oh0 = tile * g.tileRows;
  const int nOut = min(g.tileRows, g.oH - oh0);
  const int nIn = (nOut - 1) * ST + KS;
  float *xs = smem;
  float *gs = smem + (((g.tileRows - 1) * ST + KS) * g.pitch + g.padL + 3) / 4 * 4;  // [tileRows*oW]
  __shared__ float red[nWaves][T];

  dev::loadRowsPadded<VEC>(xs, in + (long)plane * g.H * g.W, g.H, g.W, oh0 * ST - g.padH, nIn, g.pitch, g.padL);
  const int colOff = g.padL - g.padW;
  const int total = nOut * g.oW;
  const int slot = n * g.tilesPerPlane + tile;
  const int lane = threadIdx.x % dev::kWave, wave = threadIdx.x / dev::kWave;

  for (int j = 0; j < g.M; ++j) {
    if (j > 0) __syncthreads();  // previous multiplier's gs / red still being read
    dev::loadFlat<VECG>(gs, gradOut + (((long)plane * g.M + j) * g.oH + oh0) * g.oW, total);
    __syncthreads();
    float acc[T];
#pragma unroll
    for (int t = 0; t < T; ++t) acc[t] = 0.f;
    for (int i = threadIdx.x; i < total; i += blockDim.x) {
      int r = i / g.oW, ow = i - r * g.oW;
      const float *p = xs + r * ST * g.pitch + ow * ST + colOff;
      const float gy = gs[i];
#pragma unroll
      for (int kh = 0; kh < KS; ++kh)
#pragma unroll
        for (int kw = 0; kw < KS; ++kw) acc[kh * KS + kw] = fmaf(gy, p[kh * g.pitch + kw], acc[kh * KS + kw]);
      acc[T - 1] += gy;
    }
#pragma unroll
    for (int t = 0; t < T; ++t) {
      float v = dev::waveSum(acc[t]);
      if (lane == 0) red[wave][t] = v;
    }
    __syncthreads();
    if (threadIdx.x < partialPitch(T)) {  // the whole run, padding included: stage 2 reads whole runs, also from scratch that is reused
      float v = 0.f;
      if (threadIdx.x < T) {
#pragma unroll
        for (int w = 0; w < nWaves; ++w) v += red[w][threadIdx.x];
      }
      partial[((long)slot * (g.C * g.M) + c * g.M + j) * partialPitch(T) + threadIdx.x] = v;
    }
  }
}

// Stage 2: one wave per (c, j) folds the partials of all slots in a fixed order and accumulates
// scale * sum into the caller's tensors. A lane owns four taps (one 16-byte group of a run, lane % Q) and every
// PH-th slot (PH = 64 / Q slot phases, lane / Q): a load instruction of the wave reads PH whole runs as the
// stage-1 workgroups wrote them, and up to 8 of them are in flight before the first add, so a batch of 64 images
// is one memory round trip. The phases are then added in a fixed association. The old values are requested before
// the partials so that the read-modify-write costs no second round trip.
template <int TP>
__global__ void __launch_bounds__(dev::kWave)
dwAccGradStage2(const float *__restrict__ partial, float *__restrict__ gradWeight, Strides4 gs,
                float *__restrict__ gradBias, Strides2 bs, int M, int kW, int T, int nslots, float scale, int CJ) {
  constexpr int Q = TP / 4, PH = dev::kWave / Q;
  constexpr int U = 8;  // loads in flight per lane
  const int cj = blockIdx.x;
  const int q = threadIdx.x % Q, ph = threadIdx.x / Q;
  const int c = cj / M, j = cj - c * M;
  float *dst[4];
  float old[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int t = q * 4 + e;
    dst[e] = nullptr;
    if (ph == 0 && t < T - 1) {
      const int kh = t / kW, kw = t - kh * kW;
      dst[e] = gradWeight + j * gs.s0 + c * gs.s1 + kh * gs.s2 + kw * gs.s3;
    } else if (ph == 0 && t == T - 1 && gradBias) {
      dst[e] = gradBias + j * bs.s0 + c * bs.s1;
    }
    old[e] = dst[e] ? *dst[e] : 0.f;
  }
  const long step = (long)CJ * TP;  // floats between the runs of consecutive slots
  const float *p = partial + (long)cj * TP + q * 4;
  float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int s0 = ph; s0 < nslots; s0 += U * PH) {
    float4 a[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int sl = s0 + u * PH;
      a[u] = sl < nslots ? *reinterpret_cast<const float4 *>(p + (long)sl * step) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) v.x += a[u].x, v.y += a[u].y, v.z += a[u].z, v.w += a[u].w;
  }
  float r[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int e = 0; e < 4; ++e) {
#pragma unroll
    for (int m = dev::kWave / 2; m >= Q; m >>= 1) r[e] += __shfl_down(r[e], m);
    if (dst[e]) *dst[e] = old[e] + scale * r[e];
  }
}

// Any geometry: one workgroup per (c, j, tap) - tap == kH*kW is the bias - that
// walks the whole batch. Slow (re-reads gradOutput per tap) but shape-agnostic.
__global__ void __launch_bounds__(dev::kBlock)
dwAccGradDirect(const float *__restrict__ in, const float *__restrict__ gradOut, float *__restrict__ gradWeight,
                Strides4 gs, float *__restrict__ gradBias, Strides2 bs, DwGeom g, float scale) {
  __shared__ float red[dev::kBlock / dev::kWave];
  const int T = g.kH * g.kW + 1;
  const int t = blockIdx.x % T;
  const int cj = blockIdx.x / T;
  const int c = cj / g.M, j = cj - c * g.M;
  if (t == T - 1 && !gradBias) return;
  const int kh = t / g.kW, kw = t - kh * g.kW;
  const long L = (long)g.oH * g.oW;
  float acc = 0.f;
  for (long i = threadIdx.x; i < (long)g.N * L; i += blockDim.x) {
    int n = (int)(i / L);
    int l = (int)(i - (long)n * L);
    float gy = gradOut[(((long)n * g.C + c) * g.M + j) * L + l];
    if (t == T - 1) {
      acc += gy;
    } else {
      int oh = l / g.oW, ow = l - oh * g.oW;
      int h = oh * g.dH - g.padH + kh, w = ow * g.dW - g.padW + kw;
      if (h >= 0 && h < g.H && w >= 0 && w < g.W)
        acc = fmaf(gy, in[(((long)n * g.C + c) * g.H + h) * g.W + w], acc);
    }
  }
  acc = dev::waveSum(acc);
  if (threadIdx.x % dev::kWave == 0) red[threadIdx.x / dev::kWave] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    float v = 0.f;
    for (int w = 0; w < (int)(blockDim.x / dev::kWave); ++w) v += red[w];
    if (t < T - 1)
      gradWeight[j * gs.s0 + c * gs.s1 + kh * gs.s2 + kw * gs.s3] += scale * v;
    else
      gradBias[j * bs.s0 + c * bs.s1] += scale * v;
  }
}

// ============================================================ strip kernels ==
// Fast paths for the geometries depthwise layers actually use: square odd
// kernel KS with "same" padding KS/2, stride ST in {1,2}, row lengths that are
// multiples of 4. A lane produces 4 consecutive outputs (one 16-byte store);
// the taps it needs form a (3*ST+KS)-wide window per input row which is read
// from LDS with 16/8-byte loads at compile-time-known alignment, and every
// index inside the window is a compile-time constant, so the inner loops are
// straight-line FMAs on registers.

// ONE: depth multiplier 1 and the band is a single load batch (at most kLoadBatch 16-byte loads
// per lane) - its loads are issued before anything else and the taps and bias are fetched while
// they are in flight.
template <int KS, int ST, bool ONE>
__global__ void __launch_bounds__(dev::kBlock)
dwFwdStrip(const float *__restrict__ in, const float *__restrict__ weight, Strides4 ws,
           const float *__restrict__ bias, Strides2 bs, float *__restrict__ out, DwGeom g) {
  using S = dev::Strip<KS, ST, KS / 2>;
  constexpr int PAD = KS / 2, NW = S::NW;
  extern __shared__ float smem[];
  const BlockPos bp = blockPos(g);
  const int plane = bp.plane, tile = bp.tile, c = bp.c;
  const int oh0 = tile * g.tileRows;
  const int nOut = min(g.tileRows, g.oH - oh0);
  const int nIn = (nOut - 1) * ST + KS;
  const int pitch = S::pitch(g.W);
  typename S::InFlight fl;
  // Stride 2 reads four bytes for every byte it writes, and its input is read with the non-temporal hint: after a
  // kernel that has just written that input the pass measures 22 us with the hint and 23-28 us without
  // (N 64, 128 x 56 x 56); only a caller that runs this pass again on an input still resident in the Infinity
  // Cache, or the weight-gradient pass right behind it, would gain from plain loads. At stride 1 the two forms
  // measure the same behind a producer, and plain loads keep a resident input resident.
  if (ONE) S::template issue<(ST == 2)>(fl, in + (long)plane * g.H * g.W, g.H, g.W, oh0 * ST - PAD, nIn);
  float w[KS * KS];
  loadTaps<KS>(weight, ws, 0, c, w);
  float b = bias ? bias[c * bs.s1] : 0.f;
  if (ONE)
    S::commit(smem, fl, g.W, nIn);
  else
    S::stage(smem, in + (long)plane * g.H * g.W, g.H, g.W, oh0 * ST - PAD, nIn);
  __syncthreads();
  const int oW4 = g.oW >> 2;
  const int total = nOut * oW4;
  const int nMul = ONE ? 1 : g.M;
  for (int j = 0; j < nMul; ++j) {
    if (!ONE && j > 0) {
      loadTaps<KS>(weight, ws, j, c, w);
      b = bias ? bias[j * bs.s0 + c * bs.s1] : 0.f;
    }
    const __amdgpu_buffer_rsrc_t orr = dev::makeRsrc(out + (((long)plane * nMul + j) * g.oH + oh0) * g.oW, (long)total * 16);
    for (int i = threadIdx.x; i < total; i += blockDim.x) {
      const int r = dev::fastDiv(i, g.magicOW4), b4 = i - r * oW4;
      const float *p = smem + r * ST * pitch;
      float acc[4] = {b, b, b, b};
#pragma unroll
      for (int kh = 0; kh < KS; ++kh) {
        float win[NW];
        S::loadWinShared(p + kh * pitch, b4, oW4, g.W, win);
#pragma unroll
        for (int kw = 0; kw < KS; ++kw)
#pragma unroll
          for (int q = 0; q < 4; ++q) acc[q] = fmaf(win[q * ST + kw], w[kh * KS + kw], acc[q]);
      }
      // Stride 2 writes a fifth of what it moves: plain stores cost this pass nothing (a 4:1 stream measures the
      // same with either kind), and they leave the output in the Infinity Cache for the layer that reads it next
      // (BatchNormalization behind this pass: 11.8 -> 10.0 us at N 64, 128 x 28 x 28). At stride 1 half of the
      // traffic is stores and streaming stores are 8 % faster.
      if (ST == 2)
        dev::bufStore4(orr, i * 16, make_float4(acc[0], acc[1], acc[2], acc[3]));
      else
        dev::bufStoreStream4(orr, i * 16, make_float4(acc[0], acc[1], acc[2], acc[3]));  // r * oW + b4 * 4 = 4 i
    }
  }
}

// gradInput: a lane produces an ST x 4 patch (rows ST*a .. ST*a+ST-1, columns
// 4b .. 4b+3). The gradOutput rows are staged zero-padded, so no tap needs a
// bounds test, and which (kh, kw) reaches which patch element is resolved at
// compile time: only the K*K/(ST*ST) taps that really contribute are executed.
// M1: depth multiplier 1 - the taps are fetched once, before the band, and stay in scalar registers.
template <int KS, int ST, bool M1>
__global__ void __launch_bounds__(dev::kBlock)
dwGradInputStrip(const float *__restrict__ gradOut, const float *__restrict__ weight, Strides4 ws,
                 float *__restrict__ gradIn, DwGeom g, int stageRows) {
  constexpr int PAD = KS / 2;
  constexpr int QH0 = dev::TapSpan<KS, ST, ST, KS / 2>::lo(), QH1 = dev::TapSpan<KS, ST, ST, KS / 2>::hi();
  constexpr int QW0 = dev::TapSpan<KS, ST, 4, KS / 2>::lo(), QW1 = dev::TapSpan<KS, ST, 4, KS / 2>::hi();
  constexpr int NW = QW1 - QW0 + 1;
  constexpr int CPB = 4 / ST;  // gradOutput columns a patch advances per b
  constexpr int OFF = ((dev::kStripPadL + QW0) % 4 + 4) % 4;
  constexpr int ALIGN = (CPB % 4 == 0) ? 4 : 2;
  extern __shared__ float smem[];
  const BlockPos bp = blockPos(g);
  const int plane = bp.plane, tile = bp.tile, c = bp.c;
  const int h0 = tile * g.tileRows;  // multiple of ST
  const int nRows = min(g.tileRows, g.H - h0);
  const int pitch = g.oW + dev::kStripPadL;
  const long L = (long)g.oH * g.oW;
  // the taps of the first multiplier are requested before the band, so that they arrive in its shadow
  float w[KS * KS];
  loadTaps<KS>(weight, ws, 0, c, w);
  const int nMul = M1 ? 1 : g.M;
  for (int j = 0; j < nMul; ++j)
    dev::loadRowsPadded<true>(smem + (size_t)j * (stageRows * pitch + dev::kStripPadL),
                              gradOut + ((long)plane * nMul + j) * L, g.oH, g.oW, h0 / ST + QH0, stageRows, pitch,
                              dev::kStripPadL);
  __syncthreads();
  const int W4 = g.W >> 2;
  const unsigned magicW4 = g.magicW4;
  // A lane produces the 4 outputs i*4 .. i*4+3 of the band in memory order, so that a wave's store is one
  // contiguous 1 KB run (full cache lines: what the streaming stores need to run at full rate). Its row
  // h0 + hl = ST*a + dy picks, per staged gradOutput row qh, the kernel row kh = dy + PAD - qh*ST; dy is
  // a run-time value, so those taps are selected into per-lane weights instead of being resolved at compile time.
  const int total = nRows * W4;
  const __amdgpu_buffer_rsrc_t orr = dev::makeRsrc(gradIn + ((long)plane * g.H + h0) * g.W, (long)total * 16);
  constexpr int kUnroll = ST == 1 ? 1 : 2;  // the wave shifts of the stride-1 window do not unroll
#pragma unroll kUnroll
  for (int i = threadIdx.x; i < total; i += blockDim.x) {
    const int hl = dev::fastDiv(i, magicW4), b = i - hl * W4;
    const int a = ST == 1 ? hl : hl >> (ST == 2 ? 1 : 0), dy = hl - a * ST;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int j = 0; j < nMul; ++j) {
      if (!M1) loadTaps<KS>(weight, ws, j, c, w);
      const float *gj = smem + (size_t)j * (stageRows * pitch + dev::kStripPadL) + dev::kStripPadL + QW0 + b * CPB;
#pragma unroll
      for (int qh = QH0; qh <= QH1; ++qh) {
        float wq[KS];
#pragma unroll
        for (int kw = 0; kw < KS; ++kw) {
          wq[kw] = 0.f;
#pragma unroll
          for (int dyc = 0; dyc < ST; ++dyc) {
            const int kh = dyc + PAD - qh * ST;
            if (kh >= 0 && kh < KS) wq[kw] = (dy == dyc) ? w[kh * KS + kw] : wq[kw];
          }
        }
        float win[NW];
        if constexpr (ST == 1)
          dev::loadWindowShared<PAD>(gj - QW0 + (a + qh - QH0) * pitch, b, W4, win);  // NW = 4 + 2 PAD, QW0 = -PAD
        else
          dev::readWindow<0, NW, OFF, ALIGN>(gj + (a + qh - QH0) * pitch, win);
#pragma unroll
        for (int dx = 0; dx < 4; ++dx)
#pragma unroll
          for (int kw = 0; kw < KS; ++kw) {
            const int t = dx + PAD - kw;
            if (t % ST != 0) continue;
            acc[dx] = fmaf(win[t / ST - QW0], wq[kw], acc[dx]);
          }
      }
    }
    dev::bufStoreStream4(orr, i * 16, make_float4(acc[0], acc[1], acc[2], acc[3]));
  }
}

// accGradParameters stage 1 with the same 4-wide windows as the forward pass.
// ONE: depth multiplier 1 and both bands (input, gradOutput) are a single load batch: all their
// loads are issued back to back before the first wait, one memory round trip per workgroup.
template <int KS, int ST, bool ONE>
__global__ void __launch_bounds__(dev::kBlock)
dwAccGradStrip(const float *__restrict__ in, const float *__restrict__ gradOut, float *__restrict__ partial,
               DwGeom g) {
  using S = dev::Strip<KS, ST, KS / 2>;
  constexpr int PAD = KS / 2, NW = S::NW;
  constexpr int T = KS * KS + 1;
  constexpr int nWaves = dev::kBlock / dev::kWave;
  extern __shared__ float smem[];
  __shared__ float red[nWaves * 4][T];  // one sum per row of 16 lanes
  const BlockPos bp = blockPos(g);
  const int plane = bp.plane, tile = bp.tile, c = bp.c;
  const int n = dev::fastDiv(plane, g.magicC);
  const int oh0 = tile * g.tileRows;
  const int nOut = min(g.tileRows, g.oH - oh0);
  const int nIn = (nOut - 1) * ST + KS;
  const int pitch = S::pitch(g.W);
  float *gs = smem + S::floats((g.tileRows - 1) * ST + KS, g.W);  // multiple of 4 floats (staged gradOutput band: !ONE only)
  const int nMul = ONE ? 1 : g.M;
  const int oW4 = g.oW >> 2;
  const int total = nOut * oW4;
  // ONE: item i of the band (4 consecutive outputs, memory order) is float4 i of the gradOutput band, and the lane
  // that loads float4 u * kBlock + tid is the lane that works on item u * kBlock + tid: gradOutput never leaves
  // the registers it was loaded into (no LDS copy, 3 KB less LDS per workgroup at 28 x 28 outputs).
  float4 gv[dev::kLoadBatch];
  if (ONE) {
    typename S::InFlight fl;
    S::template issue<true>(fl, in + (long)plane * g.H * g.W, g.H, g.W, oh0 * ST - PAD, nIn);
    const __amdgpu_buffer_rsrc_t rs = dev::makeRsrc(gradOut + ((long)plane * g.oH + oh0) * g.oW, (long)total * 16);
#pragma unroll
    for (int u = 0; u < dev::kLoadBatch; ++u) gv[u] = dev::bufLoadStream4(rs, (u * dev::kBlock + threadIdx.x) * 16);  // past the end reads 0
    S::commit(smem, fl, g.W, nIn);
  } else {
    S::stage(smem, in + (long)plane * g.H * g.W, g.H, g.W, oh0 * ST - PAD, nIn);
  }
  const int slot = n * g.tilesPerPlane + tile;
  const int lane = threadIdx.x % dev::kWave, wave = threadIdx.x / dev::kWave;
  for (int j = 0; j < nMul; ++j) {
    if (!ONE) {
      if (j > 0) __syncthreads();
      dev::loadFlat<true>(gs, gradOut + (((long)plane * g.M + j) * g.oH + oh0) * g.oW, nOut * g.oW);
    }
    __syncthreads();
    float acc[T];
#pragma unroll
    for (int t = 0; t < T; ++t) acc[t] = 0.f;
    auto item = [&](int i, const float4 gy4) {
      const int r = dev::fastDiv(i, g.magicOW4), b4 = i - r * oW4;
      const float *p = smem + r * ST * pitch;
      const float gy[4] = {gy4.x, gy4.y, gy4.z, gy4.w};
#pragma unroll
      for (int kh = 0; kh < KS; ++kh) {
        float win[NW];
        S::loadWinShared(p + kh * pitch, b4, oW4, g.W, win);
#pragma unroll
        for (int kw = 0; kw < KS; ++kw)
#pragma unroll
          for (int q = 0; q < 4; ++q) acc[kh * KS + kw] = fmaf(gy[q], win[q * ST + kw], acc[kh * KS + kw]);
      }
      acc[T - 1] += (gy[0] + gy[1]) + (gy[2] + gy[3]);
    };
    if constexpr (ONE) {
#pragma unroll
      for (int u = 0; u < dev::kLoadBatch; ++u) {
        const int i = u * dev::kBlock + (int)threadIdx.x;
        if (i < total) item(i, gv[u]);
      }
    } else {
      for (int i = threadIdx.x; i < total; i += blockDim.x) item(i, *reinterpret_cast<const float4 *>(gs + i * 4));
    }
    // rows of 16 lanes are folded on the VALU (4 DPP steps per sum), the 16 row sums of the workgroup through LDS
#pragma unroll
    for (int t = 0; t < T; ++t) {
      const float v = dev::groupSum(acc[t], 16);
      if ((lane & 15) == 0) red[wave * 4 + (lane >> 4)][t] = v;
    }
    __syncthreads();
    if (threadIdx.x < partialPitch(T)) {  // the whole run, padding included, leaves in one store instruction
      float v = 0.f;
      if (threadIdx.x < T) {
#pragma unroll
        for (int w = 0; w < nWaves * 4; ++w) v += red[w][threadIdx.x];
      }
      partial[((long)slot * (g.C * nMul) + c * nMul + j) * partialPitch(T) + threadIdx.x] = v;
    }
  }
}

// -------------------------------------------------------------- host helpers --
using launch::aligned16;
using launch::ceilDiv;
using launch::roundUp;

// lib/THCUNN/generic/SpatialDepthWiseConvolution.cu:5-56
void dwShapeCheck(THCudaTensor *input, THCudaTensor *gradOutput, THCudaTensor *weight, THCudaTensor *bias,
                  int kH, int kW, int dH, int dW, int padH, int padW) {
  THC_ARG_CHECK(kW > 0 && kH > 0, 9, "kernel size should be greater than zero, but got kH: %d kW: %d", kH, kW);
  THC_ARG_CHECK(dW > 0 && dH > 0, 11, "stride should be greater than zero, but got dH: %d dW: %d", dH, dW);
  THC_ARG_CHECK(weight->nDimension == 4, 5, "2D or 4D weight tensor expected, but got: %s",
                sizeDesc(erase(weight)).c_str());
  if (bias) {
    checkDimSize(erase(bias), "bias", 2, 0, weight->size[0]);
    checkDimSize(erase(bias), "bias", 2, 1, weight->size[1]);
  }
  int ndim = input->nDimension;
  int dimf = 0, dimh = 1, dimw = 2;
  if (ndim == 4) {
    dimf++;
    dimh++;
    dimw++;
  }
  THC_ARG_CHECK(ndim == 3 || ndim == 4, 2, "3D or 4D input tensor expected but got: %s",
                sizeDesc(erase(input)).c_str());
  long nInputPlane = weight->size[1];
  long inputHeight = input->size[dimh], inputWidth = input->size[dimw];
  long nOutputPlane = weight->size[0];
  long outputHeight = (inputHeight + 2 * padH - kH) / dH + 1;
  long outputWidth = (inputWidth + 2 * padW - kW) / dW + 1;
  if (outputWidth < 1 || outputHeight < 1)
    error("Given input size: (%ld x %ld x %ld). Calculated output size: (%ld x %ld x %ld). Output size is too small",
          nInputPlane, inputHeight, inputWidth, nOutputPlane * nInputPlane, outputHeight, outputWidth);
  checkDimSize(erase(input), "input", ndim, dimf, nInputPlane);
  if (gradOutput) {
    // the reference checks a (.., C, M, oH, oW) view of gradOutput (:285-297); here the
    // caller's (.., C*M, oH, oW) tensor is checked against the same extents
    const Tensor *go = erase(gradOutput);
    bool ok = go->nDimension == ndim && go->size[dimf] == nInputPlane * nOutputPlane &&
              go->size[dimh] == outputHeight && go->size[dimw] == outputWidth &&
              (ndim == 3 || go->size[0] == input->size[0]);
    if (!ok)
      error("Need gradOutput of dimension %d and gradOutput.size[%d] == %ld, gradOutput.size[%d] == %ld, "
            "gradOutput.size[%d] == %ld but got gradOutput to be of shape: %s",
            ndim, dimf, nInputPlane * nOutputPlane, dimh, outputHeight, dimw, outputWidth, sizeDesc(go).c_str());
  }
}

struct DwCall {
  DwGeom g;
  bool batch;
};

// Reads the geometry off the tensors; reshapes a 2-D weight to 4-D in place as
// the reference does on the caller's tensor (:76-80, :439-443).
DwCall dwSetup(THCState *state, THCudaTensor *input, THCudaTensor *gradOutput, THCudaTensor *weight,
               THCudaTensor *bias, int kW, int kH, int dW, int dH, int padW, int padH) {
  THC_ARG_CHECK(input && weight, 2, "input and weight tensors expected");
  THC_ARG_CHECK(weight->nDimension == 2 || weight->nDimension == 4, 5,
                "2D or 4D weight tensor expected, but got: %s", sizeDesc(erase(weight)).c_str());
  THC_ARG_CHECK(kW > 0 && kH > 0, 9, "kernel size should be greater than zero, but got kH: %d kW: %d", kH, kW);
  int nInputPlane = weight->nDimension == 2 ? (int)(weight->size[1] / (kH * kW)) : (int)weight->size[1];
  int nOutputPlane = (int)weight->size[0];
  if (weight->nDimension == 2) resize(state, weight, {nOutputPlane, nInputPlane, kH, kW});
  dwShapeCheck(input, gradOutput, weight, bias, kH, kW, dH, dW, padH, padW);
  DwCall call;
  DwGeom &g = call.g;
  call.batch = input->nDimension == 4;
  int o = call.batch ? 1 : 0;
  g.N = call.batch ? (int)input->size[0] : 1;
  g.C = nInputPlane;
  g.M = nOutputPlane;
  g.H = (int)input->size[o + 1];
  g.W = (int)input->size[o + 2];
  g.kH = kH, g.kW = kW, g.dH = dH, g.dW = dW, g.padH = padH, g.padW = padW;
  g.oH = (g.H + 2 * padH - kH) / dH + 1;
  g.oW = (g.W + 2 * padW - kW) / dW + 1;
  g.tileRows = g.tilesPerPlane = g.pitch = g.padL = g.nblk = g.nslots = 0;
  g.magicTiles = g.magicC = 0;
  return call;
}

Strides4 strides4(const THCudaTensor *t) { return {t->stride[0], t->stride[1], t->stride[2], t->stride[3]}; }
Strides2 strides2(const THCudaTensor *t) { return t ? Strides2{t->stride[0], t->stride[1]} : Strides2{0, 0}; }

template <bool VEC>
void launchFwd(hipStream_t s, size_t lds, const float *in, const float *w, Strides4 ws, const float *b,
               Strides2 bs, float *out, const DwGeom &g) {
  dim3 grid(g.nblk), block(dev::kBlock);
  bool sq = g.kH == g.kW && g.dH == g.dW;
  if (sq && g.kH == 3 && g.dH == 1)
    dwFwdTiled<3, 1, VEC><<<grid, block, lds, s>>>(in, w, ws, b, bs, out, g);
  else if (sq && g.kH == 3 && g.dH == 2)
    dwFwdTiled<3, 2, VEC><<<grid, block, lds, s>>>(in, w, ws, b, bs, out, g);
  else if (sq && g.kH == 5 && g.dH == 1)
    dwFwdTiled<5, 1, VEC><<<grid, block, lds, s>>>(in, w, ws, b, bs, out, g);
  else if (sq && g.kH == 5 && g.dH == 2)
    dwFwdTiled<5, 2, VEC><<<grid, block, lds, s>>>(in, w, ws, b, bs, out, g);
  else
    dwFwdTiled<0, 0, VEC><<<grid, block, lds, s>>>(in, w, ws, b, bs, out, g);
}

template <bool VEC>
void launchGradInput(hipStream_t s, size_t lds, const float *go, const float *w, Strides4 ws, float *gi,
                     const DwGeom &g, int maxOh) {
  dim3 grid(g.nblk), block(dev::kBlock);
  bool sq = g.kH == g.kW && g.dH == g.dW;
  if (sq && g.kH == 3 && g.dH == 1)
    dwGradInputTiled<3, 1, VEC><<<grid, block, lds, s>>>(go, w, ws, gi, g, maxOh);
  else if (sq && g.kH == 3 && g.dH == 2)
    dwGradInputTiled<3, 2, VEC><<<grid, block, lds, s>>>(go, w, ws, gi, g, maxOh);
  else if (sq && g.kH == 5 && g.dH == 1)
    dwGradInputTiled<5, 1, VEC><<<grid, block, lds, s>>>(go, w, ws, gi, g, maxOh);
  else if (sq && g.kH == 5 && g.dH == 2)
    dwGradInputTiled<5, 2, VEC><<<grid, block, lds, s>>>(go, w, ws, gi, g, maxOh);
  else
    dwGradInputTiled<0, 0, VEC><<<grid, block, lds, s>>>(go, w, ws, gi, g, maxOh);
}

template <int KS, int ST>
void launchAcc1(hipStream_t s, size_t lds, bool vec, bool vecg, const float *in, const float *go, float *partial,
                const DwGeom &g) {
  dim3 grid(g.nblk), block(dev::kBlock);
  if (vec && vecg)
    dwAccGradStage1<KS, ST, true, true><<<grid, block, lds, s>>>(in, go, partial, g);
  else if (vec)
    dwAccGradStage1<KS, ST, true, false><<<grid, block, lds, s>>>(in, go, partial, g);
  else if (vecg)
    dwAccGradStage1<KS, ST, false, true><<<grid, block, lds, s>>>(in, go, partial, g);
  else
    dwAccGradStage1<KS, ST, false, false><<<grid, block, lds, s>>>(in, go, partial, g);
}

void launchStage2(hipStream_t s, int TP, const float *partial, float *gw, Strides4 gs, float *gb, Strides2 bs, int M, int kW,
                  int T, int nslots, float scale, int CJ) {
  if (TP == 16)
    dwAccGradStage2<16><<<CJ, dev::kWave, 0, s>>>(partial, gw, gs, gb, bs, M, kW, T, nslots, scale, CJ);
  else
    dwAccGradStage2<32><<<CJ, dev::kWave, 0, s>>>(partial, gw, gs, gb, bs, M, kW, T, nslots, scale, CJ);
}

// Switch used by the tests (THCUNN_setSwitch) to exercise the shape-agnostic kernels on
// shapes the tiled ones would otherwise take.
// 1: shape-agnostic direct kernels, 2: generic LDS-tiled kernels (no strip fast path).
int forcedPath() { return g_switches.dwForce; }
bool forceDirect() { return forcedPath() == 1; }

// Geometry the strip kernels are compiled for.
bool stripGeometry(const DwGeom &g) {
  bool sq = g.kH == g.kW && g.dH == g.dW && g.padH == g.padW;
  return forcedPath() == 0 && sq && (g.kH == 3 || g.kH == 5) && (g.dH == 1 || g.dH == 2) && g.padH == g.kH / 2 &&
         g.W % 4 == 0 && g.oW % 4 == 0;
}

#define DW_STRIP_DISPATCH1(KERNEL, FLAG, ...)                                            \
  do {                                                                                   \
    if (g.kH == 3 && g.dH == 1) KERNEL<3, 1, FLAG><<<grid, block, lds, s>>>(__VA_ARGS__); \
    if (g.kH == 3 && g.dH == 2) KERNEL<3, 2, FLAG><<<grid, block, lds, s>>>(__VA_ARGS__); \
    if (g.kH == 5 && g.dH == 1) KERNEL<5, 1, FLAG><<<grid, block, lds, s>>>(__VA_ARGS__); \
    if (g.kH == 5 && g.dH == 2) KERNEL<5, 2, FLAG><<<grid, block, lds, s>>>(__VA_ARGS__); \
  } while (0)

#define DW_STRIP_DISPATCH(KERNEL, ...)                                           \
  do {                                                                           \
    if (g.kH == 3 && g.dH == 1) KERNEL<3, 1><<<grid, block, lds, s>>>(__VA_ARGS__); \
    if (g.kH == 3 && g.dH == 2) KERNEL<3, 2><<<grid, block, lds, s>>>(__VA_ARGS__); \
    if (g.kH == 5 && g.dH == 1) KERNEL<5, 1><<<grid, block, lds, s>>>(__VA_ARGS__); \
    if (g.kH == 5 && g.dH == 2) KERNEL<5, 2><<<grid, block, lds, s>>>(__VA_ARGS__); \
  } while (0)

// LDS floats of a staged input band of `rows` rows in the strip layout
size_t stripFloats(const DwGeom &g, int rows) {
  if (g.dH == 1) return g.kH == 3 ? dev::Strip<3, 1, 1>::floats(rows, g.W) : dev::Strip<5, 1, 2>::floats(rows, g.W);
  return g.kH == 3 ? dev::Strip<3, 2, 1>::floats(rows, g.W) : dev::Strip<5, 2, 2>::floats(rows, g.W);
}

// rows of gradOutput staged beyond the h/ST rows of a gradInput band
int gradInputExtraRows(int ks, int st) {
  if (ks == 3 && st == 1) return dev::TapSpan<3, 1, 1, 1>::hi() - dev::TapSpan<3, 1, 1, 1>::lo();
  if (ks == 3 && st == 2) return dev::TapSpan<3, 2, 2, 1>::hi() - dev::TapSpan<3, 2, 2, 1>::lo();
  if (ks == 5 && st == 1) return dev::TapSpan<5, 1, 1, 2>::hi() - dev::TapSpan<5, 1, 1, 2>::lo();
  return dev::TapSpan<5, 2, 2, 2>::hi() - dev::TapSpan<5, 2, 2, 2>::lo();
}

// ---- small planes: several planes per workgroup (dwconv_small.h) ----------------------------
enum SmallPass { kSmallFwd, kSmallGradInput, kSmallAccGrad };

// Planes of at most 1024 elements take these kernels, several per workgroup (measured faster than the strip
// kernels up to 28x28), and so do larger planes whose width or output width is not a multiple of 4 (which
// the strip kernels need): two per workgroup up to 2048 elements, a band of rows per workgroup beyond. Test switch THCUNN_DW_SMALL: 0 never, 1 also for
// the larger planes that the strip kernels could take.
int smallSwitch() { return g_switches.dwSmall; }

constexpr int kSmallPlane = 1024;

// Plans a small-plane launch; false when the geometry is outside what those kernels are compiled for.
bool smallPlan(const DwGeom &g, SmallPass pass, SmallGeom *out, int *rw, size_t *lds) {
  const bool sq = g.kH == g.kW && g.dH == g.dW && g.padH == g.padW;
  if (forcedPath() != 0 || smallSwitch() == 0 || !sq || g.M != 1 || (g.kH != 3 && g.kH != 5) || (g.dH != 1 && g.dH != 2) ||
      g.padH != g.kH / 2)
    return false;
  const int HW = g.H * g.W, oHW = g.oH * g.oW;
  if (oHW < 1 || (long)g.N * g.C >= 0x7fffffffL / 64) return false;
  const int PAD = g.kH / 2, KS = g.kH, st = g.dH;
  SmallGeom sg{};
  sg.C = g.C, sg.planes = g.N * g.C;
  if (pass == kSmallGradInput)
    sg.sH = g.oH, sg.sW = g.oW, sg.oH = g.H, sg.oW = g.W;
  else
    sg.sH = g.H, sg.sW = g.W, sg.oH = g.oH, sg.oW = g.oW;
  sg.srcFloats = (long)sg.planes * sg.sH * sg.sW, sg.outFloats = (long)sg.planes * sg.oH * sg.oW;
  sg.LW = (g.W + 2 * PAD) | 1;  // row pitch for sizing; the final one (up to 8 more) is chosen below
  const int CS = pass == kSmallGradInput ? 1 : st, DS = pass == kSmallGradInput ? st : 1;  // compute stride, staging dilation
  const int kRun = launch::kBatchFloats - 3;  // floats of a run (one batch of 16-byte loads, incl. up to 3 in front of it)
  const int kSlack = 7 * 2 + KS;              // LDS floats the widest work item may read past the last staged row
  int secondFloats = 0;                       // second LDS buffer: output run (forward, gradInput) / gradOutput run (accGrad)
  if (HW <= kSmallPlane || (HW <= 2 * kSmallPlane && !stripGeometry(g))) {
    // several whole planes per workgroup, at least 2
    sg.bands = 1, sg.rowsPerBand = sg.oH;
    sg.LH = g.H + 2 * PAD;
    const int second = pass == kSmallGradInput ? HW : oHW;
    auto bytes = [&](int P) { return (size_t)(roundUp(P * sg.LH * sg.LW + kSlack, 4) + roundUp(P * second + 4, 4)) * sizeof(float); };
    // a workgroup's runs start at multiples of P planes: on a 16-byte boundary if P planes are a multiple of 4 floats
    auto fetched = [&](int n) { return n + (n % 4 ? 3 : 0); };
    auto fits = [&](int P) { return fetched(P * HW) <= launch::kBatchFloats && fetched(P * oHW) <= launch::kBatchFloats && bytes(P) <= launch::kLdsMax; };
    int P = 64;
    while (P > 2 && !fits(P)) P >>= 1;
    if (fits(P)) {
      sg.P = P;
      sg.xsFloats = roundUp(P * sg.LH * sg.LW + kSlack, 4);
      secondFloats = roundUp(P * second + 4, 4);
    }
  }
  if (sg.P == 0) {
    // a band of rows of one plane per workgroup: for the widths the strip kernels do not take
    if (smallSwitch() != 1 && stripGeometry(g)) return false;
    sg.P = 1;
    // produced rows per band: the source rows behind them and the produced rows themselves are one run each
    auto srcRows = [&](int rows) { return ((rows - 1) * CS + KS - 1) / DS + 1; };
    auto fits = [&](int rows) {
      const int LHb = (rows - 1) * CS + KS;
      const size_t b = (size_t)(roundUp(LHb * sg.LW + kSlack, 4) + roundUp(rows * sg.oW + 4, 4)) * sizeof(float);
      return srcRows(rows) * sg.sW <= kRun && rows * sg.oW <= kRun && b <= 48 * 1024;
    };
    if (!fits(1)) return false;
    int rows = 1;
    while (rows < sg.oH && fits(rows + 1)) ++rows;
    sg.bands = ceilDiv(sg.oH, rows);
    sg.rowsPerBand = ceilDiv(sg.oH, sg.bands);
    if ((long)sg.planes * sg.bands >= 0x7fffffffL) return false;
    sg.LH = (sg.rowsPerBand - 1) * CS + KS;
    sg.xsFloats = roundUp(sg.LH * sg.LW + kSlack, 4);
    secondFloats = roundUp(sg.rowsPerBand * sg.oW + 4, 4);
  }
  sg.lp = dev::kBlock / sg.P;
  for (sg.lpShift = 0; (1 << sg.lpShift) < sg.lp; ++sg.lpShift) {
  }
  const int base = g.W + 2 * PAD;
  const int room = (int)((launch::kLdsMax / sizeof(float) - secondFloats - kSlack - 4) / ((size_t)sg.P * sg.LH));  // widest pitch that fits
  const launch::ItemChoice ch = launch::pickItem(pass, sg.oW, sg.rowsPerBand, sg.lp, sg.lpShift, sg.LH, CS, base,
                                                 std::max(room, sg.LW), pass == kSmallAccGrad, KS);
  *rw = ch.rw;
  sg.LW = ch.LW;
  sg.xsFloats = roundUp(sg.P * sg.LH * sg.LW + kSlack, 4);
  sg.nseg = ceilDiv(sg.oW, *rw), sg.nfull = sg.oW / *rw;
  sg.magicC = dev::magicOf(g.C), sg.magicSPlane = dev::magicOf(sg.sH * sg.sW), sg.magicSW = dev::magicOf(sg.sW);
  sg.magicSeg = dev::magicOf(sg.nseg), sg.magicFull = dev::magicOf(std::max(sg.nfull, 1)), sg.magicBands = dev::magicOf(sg.bands);
  *out = sg;
  *lds = (size_t)(sg.xsFloats + secondFloats) * sizeof(float);
  return true;
}

// workgroups of a small-plane launch
inline unsigned smallGrid(const SmallGeom &sg) {
  return sg.bands == 1 ? (unsigned)ceilDiv(sg.planes, sg.P) : (unsigned)((long)sg.planes * sg.bands);
}

#define DW_SMALL_CONV(CS, DS, FLIP, ...)                                                                          \
  do {                                                                                                            \
    if (g.kH == 3 && rw == 4) dwSmallConv<3, CS, DS, FLIP, 4><<<grid, dev::kBlock, lds, s>>>(__VA_ARGS__);        \
    if (g.kH == 3 && rw == 7) dwSmallConv<3, CS, DS, FLIP, 7><<<grid, dev::kBlock, lds, s>>>(__VA_ARGS__);        \
    if (g.kH == 5 && rw == 4) dwSmallConv<5, CS, DS, FLIP, 4><<<grid, dev::kBlock, lds, s>>>(__VA_ARGS__);        \
    if (g.kH == 5 && rw == 7) dwSmallConv<5, CS, DS, FLIP, 7><<<grid, dev::kBlock, lds, s>>>(__VA_ARGS__);        \
  } while (0)

#define DW_SMALL_ACC(ST, ...)                                                                                     \
  do {                                                                                                            \
    if (g.kH == 3 && rw == 4) dwSmallAccGrad<3, ST, 4><<<grid, dev::kBlock, lds, s>>>(__VA_ARGS__);               \
    if (g.kH == 3 && rw == 7) dwSmallAccGrad<3, ST, 7><<<grid, dev::kBlock, lds, s>>>(__VA_ARGS__);               \
    if (g.kH == 5 && rw == 4) dwSmallAccGrad<5, ST, 4><<<grid, dev::kBlock, lds, s>>>(__VA_ARGS__);               \
    if (g.kH == 5 && rw == 7) dwSmallAccGrad<5, ST, 7><<<grid, dev::kBlock, lds, s>>>(__VA_ARGS__);               \
  } while (0)

// ---- fixed scratch of the entry point that allocates nothing ----------------------------------
// accGradParameters needs device memory beyond its inputs and outputs: the per-workgroup partial sums that
// its second kernel folds. The regular entry point takes it from the caller's `columns` tensor (growing it)
// or from a stream-ordered temporary; the no-allocation variant takes it from this array, which each GPU the
// library runs on holds (4 MiB) until the process ends. In host code the array's name is only a handle for
// hipGetSymbolAddress, never a device address: the address is looked up once per device and kept.
constexpr long kNoAllocScratchFloats = 1L << 20;
static __device__ __align__(256) float scratch[kNoAllocScratchFloats];

constexpr int kMaxDevices = 64;
std::mutex g_scratchMutex;
float *g_scratchPtr[kMaxDevices];  // per device: that GPU's copy of `scratch`
std::atomic<int> g_scratchBusy[kMaxDevices];  // per device: a host thread is inside the no-allocation entry point

// Address of the current device's copy of the array; `device` must be the current device.
float *noAllocScratch(int device) {
  if (device < 0 || device >= kMaxDevices) error("device ordinal %d out of range", device);
  std::lock_guard<std::mutex> lock(g_scratchMutex);
  if (!g_scratchPtr[device]) {
    void *p = nullptr;
    THC_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    g_scratchPtr[device] = static_cast<float *>(p);
  }
  return g_scratchPtr[device];
}

// Where accGradParameters puts its partial sums.
struct DwScratch {
  THCudaTensor *columns = nullptr;  // the caller's buffer tensor (resized), or NULL: a stream-ordered temporary
  float *fixed = nullptr;           // no-allocation variant: the device's fixed array
  bool noAlloc = false;
  Temp tmp;

  // `rows` x `nslots` floats of scratch
  float *get(THCState *state, long rows, long nslots) {
    if (noAlloc) {
      if (rows * nslots > kNoAllocScratchFloats)
        error("SpatialDepthWiseConvolution_accGradParameters_noAlloc: this shape needs %ld floats of scratch "
              "(%ld workgroup slots of %ld floats), the fixed scratch holds %ld; use "
              "SpatialDepthWiseConvolution_accGradParameters",
              rows * nslots, rows, nslots, kNoAllocScratchFloats);
      return fixed;
    }
    if (columns) {
      resize(state, columns, {rows, nslots});
      if (!isContiguous(erase(columns))) error("columns tensor has to be contiguous");
      if (launch::aligned16(data(columns))) return data(columns);  // the runs are written as 16-byte groups
    }
    tmp = Temp(state->stream, (size_t)(rows * nslots) * sizeof(float));
    return (float *)tmp.get();
  }
};

}  // namespace

extern "C" {

void THNN_CudaSpatialDepthWiseConvolution_updateOutput(THCState *state, THCudaTensor *input, THCudaTensor *output,
                                                       THCudaTensor *weight, THCudaTensor *bias,
                                                       THCudaTensor *columns, THCudaTensor *ones, int kW, int kH,
                                                       int dW, int dH, int padW, int padH) {
  THNN_ENTER
  (void)columns;  // the fused kernel never materialises im2col columns or a ones vector;
  (void)ones;     // both buffers are left as the caller passed them
  THC_ARG_CHECK(output != nullptr, 3, "output tensor expected");
  DwCall call = dwSetup(state, input, nullptr, weight, bias, kW, kH, dW, dH, padW, padH);
  DwGeom &g = call.g;
  Contiguous in(state, input);
  if (call.batch)
    resize(state, output, {g.N, (long)g.C * g.M, g.oH, g.oW});
  else
    resize(state, output, {(long)g.C * g.M, g.oH, g.oW});
  if (!isContiguous(erase(output))) error("output tensor has to be contiguous");
  hipStream_t s = state->stream;
  const long planes = (long)g.N * g.C;
  if (planes == 0) return;
  const float *bptr = bias ? data(bias) : nullptr;

  {
    SmallGeom sg;
    int rw;
    size_t lds;
    if (aligned16(in.ptr()) && aligned16(data(output)) && smallPlan(g, kSmallFwd, &sg, &rw, &lds)) {
      const dim3 grid(smallGrid(sg));
      if (g.dH == 1)
        DW_SMALL_CONV(1, 1, false, in.ptr(), data(weight), strides4(weight), bptr, strides2(bias), data(output), sg);
      else
        DW_SMALL_CONV(2, 1, false, in.ptr(), data(weight), strides4(weight), bptr, strides2(bias), data(output), sg);
      THC_HIP_CHECK(hipGetLastError());
      return;
    }
  }
  bool vec = (g.W % 4 == 0) && aligned16(in.ptr());
  g.padL = vec ? roundUp(g.padW, 4) : g.padW;
  g.pitch = g.W + g.padL;
  auto bytes = [&](int rows) {
    return ((size_t)((rows - 1) * g.dH + g.kH) * g.pitch + g.padL + (size_t)g.M * g.kH * g.kW) * sizeof(float);
  };
  if (stripGeometry(g) && vec && aligned16(data(output))) {
    auto sbytes = [&](int rows) { return stripFloats(g, (rows - 1) * g.dH + g.kH) * sizeof(float); };
    auto staged = [&](int rows) { return (size_t)((rows - 1) * g.dH + g.kH) * g.W; };
    if (launch::pickBand(g.oH, planes, sbytes, &g.tileRows, &g.tilesPerPlane, staged)) {
      g.nblk = (int)(planes * g.tilesPerPlane);
      size_t lds = sbytes(g.tileRows);
      dim3 grid(g.nblk), block(dev::kBlock);
      g.magicTiles = dev::magicOf(g.tilesPerPlane), g.magicC = dev::magicOf(g.C);
      g.magicOW4 = dev::magicOf(g.oW / 4), g.magicW4 = dev::magicOf(g.W / 4);
      if (g.M == 1 && staged(g.tileRows) <= (size_t)launch::kBatchFloats)
        DW_STRIP_DISPATCH1(dwFwdStrip, true, in.ptr(), data(weight), strides4(weight), bptr, strides2(bias), data(output), g);
      else
        DW_STRIP_DISPATCH1(dwFwdStrip, false, in.ptr(), data(weight), strides4(weight), bptr, strides2(bias), data(output), g);
      THC_HIP_CHECK(hipGetLastError());
      return;
    }
  }
  if (!forceDirect() && launch::pickBand(g.oH, planes, bytes, &g.tileRows, &g.tilesPerPlane)) {
    g.nblk = (int)(planes * g.tilesPerPlane);
    size_t lds = bytes(g.tileRows);
    if (vec)
      launchFwd<true>(s, lds, in.ptr(), data(weight), strides4(weight), bptr, strides2(bias), data(output), g);
    else
      launchFwd<false>(s, lds, in.ptr(), data(weight), strides4(weight), bptr, strides2(bias), data(output), g);
  } else {
    long total = planes * g.M * g.oH * g.oW;
    dwFwdDirect<<<launch::directGrid(total, dev::kBlock), dev::kBlock, 0, s>>>(
        in.ptr(), data(weight), strides4(weight), bptr, strides2(bias), data(output), g, total);
  }
  THC_HIP_CHECK(hipGetLastError());
  THNN_LEAVE
}

void THNN_CudaSpatialDepthWiseConvolution_updateGradInput(THCState *state, THCudaTensor *input,
                                                          THCudaTensor *gradOutput, THCudaTensor *gradInput,
                                                          THCudaTensor *weight, THCudaTensor *gradColumns,
                                                          THCudaTensor *ones, int kW, int kH, int dW, int dH,
                                                          int padW, int padH) {
  THNN_ENTER
  (void)gradColumns;
  (void)ones;
  THC_ARG_CHECK(gradOutput != nullptr, 3, "gradOutput tensor expected");
  THC_ARG_CHECK(gradInput != nullptr, 4, "gradInput tensor expected");
  DwCall call = dwSetup(state, input, gradOutput, weight, nullptr, kW, kH, dW, dH, padW, padH);
  DwGeom &g = call.g;
  Contiguous go(state, gradOutput);
  if (call.batch)
    resize(state, gradInput, {g.N, g.C, g.H, g.W});
  else
    resize(state, gradInput, {g.C, g.H, g.W});
  if (!isContiguous(erase(gradInput))) error("gradInput tensor has to be contiguous");
  hipStream_t s = state->stream;
  const long planes = (long)g.N * g.C;
  if (planes == 0) return;

  {
    SmallGeom sg;
    int rw;
    size_t lds;
    if (aligned16(go.ptr()) && aligned16(data(gradInput)) && smallPlan(g, kSmallGradInput, &sg, &rw, &lds)) {
      const dim3 grid(smallGrid(sg));
      const Strides2 nob{0, 0};
      if (g.dH == 1)
        DW_SMALL_CONV(1, 1, true, go.ptr(), data(weight), strides4(weight), nullptr, nob, data(gradInput), sg);
      else
        DW_SMALL_CONV(1, 2, true, go.ptr(), data(weight), strides4(weight), nullptr, nob, data(gradInput), sg);
      THC_HIP_CHECK(hipGetLastError());
      return;
    }
  }
  // a band of `rows` gradInput rows is reached by at most (rows + kH - 2) / dH + 2 gradOutput rows
  bool vec = (g.oW % 4 == 0) && aligned16(go.ptr());
  auto ohRows = [&](int rows) { return std::min(g.oH, (rows + g.kH - 2) / g.dH + 2); };
  auto bytes = [&](int rows) {
    return ((size_t)g.M * ohRows(rows) * g.oW + (size_t)g.M * g.kH * g.kW) * sizeof(float);
  };
  if (stripGeometry(g) && vec && aligned16(data(gradInput))) {
    const int extra = gradInputExtraRows(g.kH, g.dH);
    const int pitch = g.oW + dev::kStripPadL;
    auto sbytes = [&](int units) { return (size_t)g.M * ((size_t)(units + extra) * pitch + dev::kStripPadL) * sizeof(float); };
    int units = 0;
    if (launch::pickBand(ceilDiv(g.H, g.dH), planes, sbytes, &units, &g.tilesPerPlane)) {
      g.tileRows = units * g.dH;
      g.nblk = (int)(planes * g.tilesPerPlane);
      size_t lds = sbytes(units);
      dim3 grid(g.nblk), block(dev::kBlock);
      g.magicTiles = dev::magicOf(g.tilesPerPlane), g.magicC = dev::magicOf(g.C);
      g.magicOW4 = dev::magicOf(g.oW / 4), g.magicW4 = dev::magicOf(g.W / 4);
      if (g.M == 1)
        DW_STRIP_DISPATCH1(dwGradInputStrip, true, go.ptr(), data(weight), strides4(weight), data(gradInput), g, units + extra);
      else
        DW_STRIP_DISPATCH1(dwGradInputStrip, false, go.ptr(), data(weight), strides4(weight), data(gradInput), g, units + extra);
      THC_HIP_CHECK(hipGetLastError());
      return;
    }
  }
  if (!forceDirect() && launch::pickBand(g.H, planes, bytes, &g.tileRows, &g.tilesPerPlane)) {
    g.nblk = (int)(planes * g.tilesPerPlane);
    int maxOh = ohRows(g.tileRows);
    size_t lds = bytes(g.tileRows);
    if (vec)
      launchGradInput<true>(s, lds, go.ptr(), data(weight), strides4(weight), data(gradInput), g, maxOh);
    else
      launchGradInput<false>(s, lds, go.ptr(), data(weight), strides4(weight), data(gradInput), g, maxOh);
  } else {
    long total = planes * g.H * g.W;
    dwGradInputDirect<<<launch::directGrid(total, dev::kBlock), dev::kBlock, 0, s>>>(
        go.ptr(), data(weight), strides4(weight), data(gradInput), g, total);
  }
  THC_HIP_CHECK(hipGetLastError());
  THNN_LEAVE
}

}  // extern "C"

namespace {

// lib/THCUNN/generic/SpatialDepthWiseConvolution.cu:418-650; `sc` says where the partial sums go
void dwAccGradParameters(THCState *state, THCudaTensor *input, THCudaTensor *gradOutput, THCudaTensor *gradWeight,
                         THCudaTensor *gradBias, DwScratch &sc, int kW, int kH, int dW, int dH, int padW, int padH,
                         float scale) {
  THC_ARG_CHECK(gradOutput != nullptr, 3, "gradOutput tensor expected");
  THC_ARG_CHECK(gradWeight != nullptr, 4, "gradWeight tensor expected");
  if (sc.noAlloc) {
    // everything that would allocate in the regular entry point is refused up front
    THC_ARG_CHECK(input != nullptr, 2, "input tensor expected");
    if (gradWeight->nDimension != 4)
      error("SpatialDepthWiseConvolution_accGradParameters_noAlloc: 4D gradWeight tensor expected, but got: %s",
            sizeDesc(erase(gradWeight)).c_str());
    if (!isContiguous(erase(input)) || !isContiguous(erase(gradOutput)))
      error("SpatialDepthWiseConvolution_accGradParameters_noAlloc: input and gradOutput have to be contiguous "
            "(packing them would allocate)");
  }
  DwCall call = dwSetup(state, input, gradOutput, gradWeight, gradBias, kW, kH, dW, dH, padW, padH);
  DwGeom &g = call.g;
  Contiguous in(state, input);  // contiguous tensors are used in place
  Contiguous go(state, gradOutput);
  hipStream_t s = state->stream;
  const long planes = (long)g.N * g.C;
  if (planes == 0) return;
  float *gbPtr = gradBias ? data(gradBias) : nullptr;

  {
    SmallGeom sg;
    int rw;
    size_t lds;
    if (aligned16(in.ptr()) && aligned16(go.ptr()) && smallPlan(g, kSmallAccGrad, &sg, &rw, &lds)) {
      const int T = g.kH * g.kW + 1;
      // one partial per (channel, tap, image); scratch as in the general case below
      const long nslots = (long)g.N * sg.bands;
      if (nslots >= 0x7fffffffL) error("SpatialDepthWiseConvolution: batch too large");
      const int TP = partialPitch(T);
      float *partial = sc.get(state, nslots, (long)g.C * TP);
      const dim3 grid(smallGrid(sg));
      if (g.dH == 1)
        DW_SMALL_ACC(1, in.ptr(), go.ptr(), partial, sg);
      else
        DW_SMALL_ACC(2, in.ptr(), go.ptr(), partial, sg);
      THC_HIP_CHECK(hipGetLastError());
      launchStage2(s, TP, partial, data(gradWeight), strides4(gradWeight), gbPtr, strides2(gradBias), 1, g.kW, T, (int)nslots,
                   scale, g.C);
      THC_HIP_CHECK(hipGetLastError());
      return;
    }
  }
  bool sq = g.kH == g.kW && g.dH == g.dW;
  int ks = sq ? g.kH : 0, st = sq ? g.dH : 0;
  bool haveKernel = (ks == 3 || ks == 5) && (st == 1 || st == 2);
  bool vec = (g.W % 4 == 0) && aligned16(in.ptr());
  const bool useStrip = stripGeometry(g) && vec && aligned16(go.ptr());
  g.padL = vec ? roundUp(g.padW, 4) : g.padW;
  g.pitch = g.W + g.padL;
  // staged input band (rounded up so the gradOutput band behind it stays 16-byte aligned) + gradOutput band
  auto bytes = [&](int rows) {
    size_t band = useStrip ? stripFloats(g, (rows - 1) * g.dH + g.kH)
                           : (size_t)roundUp(((rows - 1) * g.dH + g.kH) * g.pitch + g.padL, 4);
    return (band + (size_t)rows * g.oW) * sizeof(float);
  };
  auto staged = [&](int rows) { return useStrip ? (size_t)((rows - 1) * g.dH + g.kH) * g.W : (size_t)0; };
  // Two bands are staged here (input and gradOutput), and every workgroup pays a fixed reduction epilogue: a
  // budget of 34 KB (4 workgroups per CU) keeps a one-batch input band and its gradOutput rows in one workgroup.
  if (haveKernel && !forceDirect() &&
      launch::pickBand(g.oH, planes, bytes, &g.tileRows, &g.tilesPerPlane, staged, useStrip ? 34 * 1024 : launch::kLdsBudget)) {
    g.nblk = (int)(planes * g.tilesPerPlane);
    g.nslots = g.N * g.tilesPerPlane;
    size_t lds = bytes(g.tileRows);
    const int T = ks * ks + 1;
    // per-workgroup partials: the caller's `columns` buffer is the scratch the ABI
    // provides for this call (the reference resizes it as well, :528); fall back to a
    // stream-ordered temporary when none is passed
    const int TP = partialPitch(T);
    float *partial = sc.get(state, g.nslots, (long)g.C * g.M * TP);
    // a band of gradOutput rows starts at ((plane*M+j)*oH + oh0) * oW
    bool vecg = aligned16(go.ptr()) && (g.oW % 4 == 0 || (g.tilesPerPlane == 1 && ((long)g.oH * g.oW) % 4 == 0));
    if (useStrip) {
      dim3 grid(g.nblk), block(dev::kBlock);
      g.magicTiles = dev::magicOf(g.tilesPerPlane), g.magicC = dev::magicOf(g.C);
      g.magicOW4 = dev::magicOf(g.oW / 4), g.magicW4 = dev::magicOf(g.W / 4);
      if (g.M == 1 && staged(g.tileRows) <= (size_t)launch::kBatchFloats && aligned16(go.ptr())) {
        lds = stripFloats(g, (g.tileRows - 1) * g.dH + g.kH) * sizeof(float);  // gradOutput stays in registers
        DW_STRIP_DISPATCH1(dwAccGradStrip, true, in.ptr(), go.ptr(), partial, g);
      } else
        DW_STRIP_DISPATCH1(dwAccGradStrip, false, in.ptr(), go.ptr(), partial, g);
    } else {
      if (ks == 3 && st == 1) launchAcc1<3, 1>(s, lds, vec, vecg, in.ptr(), go.ptr(), partial, g);
      if (ks == 3 && st == 2) launchAcc1<3, 2>(s, lds, vec, vecg, in.ptr(), go.ptr(), partial, g);
      if (ks == 5 && st == 1) launchAcc1<5, 1>(s, lds, vec, vecg, in.ptr(), go.ptr(), partial, g);
      if (ks == 5 && st == 2) launchAcc1<5, 2>(s, lds, vec, vecg, in.ptr(), go.ptr(), partial, g);
    }
    THC_HIP_CHECK(hipGetLastError());
    launchStage2(s, TP, partial, data(gradWeight), strides4(gradWeight), gbPtr, strides2(gradBias), g.M, g.kW, T, g.nslots,
                 scale, g.C * g.M);
  } else {
    int T = g.kH * g.kW + 1;
    dwAccGradDirect<<<g.C * g.M * T, dev::kBlock, 0, s>>>(in.ptr(), go.ptr(), data(gradWeight),
                                                          strides4(gradWeight), gbPtr, strides2(gradBias), g, scale);
  }
  THC_HIP_CHECK(hipGetLastError());
}

}  // namespace

namespace thc {
void dwNoAllocInit(int device) { (void)noAllocScratch(device); }
}  // namespace thc

extern "C" {

void THNN_CudaSpatialDepthWiseConvolution_accGradParameters(THCState *state, THCudaTensor *input,
                                                            THCudaTensor *gradOutput, THCudaTensor *gradWeight,
                                                            THCudaTensor *gradBias, THCudaTensor *columns,
                                                            THCudaTensor *ones, int kW, int kH, int dW, int dH,
                                                            int padW, int padH, float scale) {
  THNN_ENTER
  (void)ones;
  DwScratch sc;
  sc.columns = columns;
  dwAccGradParameters(state, input, gradOutput, gradWeight, gradBias, sc, kW, kH, dW, dH, padW, padH, scale);
  THNN_LEAVE
}

// No counterpart in the reference: the same pass for callers that cannot allocate device memory (HIP graph
// capture, serving loops). Same kernels; the partial sums go to the device's fixed scratch array.
void THNN_CudaSpatialDepthWiseConvolution_accGradParameters_noAlloc(THCState *state, THCudaTensor *input,
                                                                    THCudaTensor *gradOutput,
                                                                    THCudaTensor *gradWeight, THCudaTensor *gradBias,
                                                                    int kW, int kH, int dW, int dH, int padW,
                                                                    int padH, float scale) {
  THNN_ENTER
  int device = -1;
  THC_HIP_CHECK(hipGetDevice(&device));
  if (device != state->device)
    error("SpatialDepthWiseConvolution_accGradParameters_noAlloc: the state was made on device %d but device %d "
          "is current", state->device, device);
  DwScratch sc;
  sc.noAlloc = true;
  sc.fixed = noAllocScratch(device);  // looked up when the state was made; a table read here
  // All calls on a GPU share that array. Two host threads inside this entry point for the same GPU at once are
  // refused; calls that overlap only on the GPU (one thread, two streams) cannot be seen from here without a
  // synchronising or allocating call and remain the caller's to order.
  struct Busy {
    std::atomic<int> &f;
    bool mine;
    explicit Busy(std::atomic<int> &flag) : f(flag), mine(flag.exchange(1) == 0) {}
    ~Busy() {
      if (mine) f.store(0);
    }
  } busy(g_scratchBusy[device]);
  if (!busy.mine)
    error("SpatialDepthWiseConvolution_accGradParameters_noAlloc: another thread is inside this entry point on "
          "device %d; the calls share one scratch array per GPU and must not overlap", device);
  dwAccGradParameters(state, input, gradOutput, gradWeight, gradBias, sc, kW, kH, dW, dH, padW, padH, scale);
  THNN_LEAVE
}

}  // extern "C"
