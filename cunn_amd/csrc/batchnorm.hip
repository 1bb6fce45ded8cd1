// BatchNormalization (1-D/2-D/3-D share it: the input is viewed as N x C x L,
// lib/THCUNN/generic/BatchNormalization.cu:8-32) for gfx950.
//
// The reference gives one workgroup a whole channel and walks the batch
// serially three times (lib/THCUNN/BatchNormalization.cu:166-212). With 256 CUs
// and typically a few hundred channels that leaves the chip idle, so here a
// channel is cut into chunks (a few whole planes, or a segment of a large
// plane) and every pass is a grid of C x chunks workgroups streaming 16-byte
// loads:
//   statistics:  per chunk (count, mean, M2) from shifted sums, reduced with a
//                64-lane shuffle tree + LDS; chunks are merged with Chan's
//                formula in double, in a fixed order, by every workgroup of
//                the channel (no atomics, no extra launch, deterministic)
//   apply:       y = gamma * (x - mean) * invStd + beta on the same chunking.
// Backward mirrors it with the fused (sum gy, sum gy*(x-mean)) reduction of
// lib/THCUNN/BatchNormalization.cu:214-283.
#include <cmath>

#include <atomic>

#include <type_traits>

#include "device_utils.h"
#include "launch_utils.h"
#include "thc_internal.h"

using namespace thc;

namespace {

struct BnGeom {
  int N, C, L;
  int planesPerChunk;  // whole planes a chunk covers (1 when planes are segmented)
  int segsPerPlane;    // segments a plane is cut into
  int segLen;          // elements per segment (multiple of 4 when vectorised)
  int chunks;          // chunks per channel = ceil(N / planesPerChunk) * segsPerPlane
};

struct Chunk {
  int n0, nN;  // planes [n0, n0 + nN)
  int l0, lN;  // elements [l0, l0 + lN) of each plane
};

__device__ __forceinline__ Chunk chunkOf(const BnGeom &g, int chunk) {
  int nb = chunk / g.segsPerPlane, sg = chunk - nb * g.segsPerPlane;
  Chunk c;
  c.n0 = nb * g.planesPerChunk;
  c.nN = min(g.planesPerChunk, g.N - c.n0);
  c.l0 = sg * g.segLen;
  c.lN = min(g.segLen, g.L - c.l0);
  return c;
}

// Visits every element of a chunk of channel `ch`: f(offset, width) is called with the flat offset into the
// (N,C,L) tensor of `width` (W4 or W1) consecutive elements. MODE 1: plane segments start on 16-byte
// boundaries and are multiples of 4 long (16-byte accesses only); MODE 2: any plane size in a 16-byte aligned
// tensor - per plane segment the elements in front of the first boundary, the 16-byte groups, and the
// elements behind the last boundary are three kinds of work items; MODE 0: element by element.
using W1 = std::integral_constant<int, 1>;
using W4 = std::integral_constant<int, 4>;
template <int MODE, typename F>
__device__ __forceinline__ void forChunk(const BnGeom &g, int ch, const Chunk &c, F f) {
  if (MODE == 1) {
    const int seg4 = c.lN >> 2;
    const int total = c.nN * seg4;
    for (int i = threadIdx.x; i < total; i += blockDim.x) {
      int n = i / seg4, l4 = i - n * seg4;
      f(((long)(c.n0 + n) * g.C + ch) * g.L + c.l0 + (l4 << 2), W4{});
    }
  } else if (MODE == 2) {
    const int slots = (c.lN >> 2) + 2;  // head, at most lN / 4 groups, tail
    const int total = c.nN * slots;
    for (int i = threadIdx.x; i < total; i += blockDim.x) {
      const int n = i / slots, k = i - n * slots;
      const long off0 = ((long)(c.n0 + n) * g.C + ch) * g.L + c.l0;
      const int head = min((int)(-off0 & 3), c.lN);
      const int body4 = (c.lN - head) >> 2, tail = (c.lN - head) & 3;
      if (k == 0) {
        for (int j = 0; j < head; ++j) f(off0 + j, W1{});
      } else if (k <= body4) {
        f(off0 + head + ((k - 1) << 2), W4{});
      } else if (k == body4 + 1) {
        for (int j = 0; j < tail; ++j) f(off0 + head + (body4 << 2) + j, W1{});
      }
    }
  } else {
    const int total = c.nN * c.lN;
    for (int i = threadIdx.x; i < total; i += blockDim.x) {
      int n = i / c.lN, l = i - n * c.lN;
      f(((long)(c.n0 + n) * g.C + ch) * g.L + c.l0 + l, W1{});
    }
  }
}

template <int NV>
__device__ __forceinline__ void blockSum(float (&v)[NV], float (*red)[NV]) {
  const int lane = threadIdx.x % dev::kWave, wave = threadIdx.x / dev::kWave;
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    v[k] = dev::waveSum(v[k]);
    if (lane == 0) red[wave][k] = v[k];
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < dev::kBlock / dev::kWave; ++w) s += red[w][k];
    v[k] = s;
  }
}

// One normalised element, y = gamma * (x - mean) * invStd + beta, in a fixed sequence of fp32 operations: the
// forward kernels store it and the fused ReLU backward re-derives its sign from x, so both must round alike.
__device__ __forceinline__ float bnAffine(float x, float mean, float invStd, float gamma, float beta) {
  return __builtin_fmaf(gamma * (x - mean), invStd, beta);
}
// Threshold(0, 0) of lib/THCUNN/Threshold.cu:6-20 on top of it when `relu` is set: v > 0 ? v : 0 (NaN -> 0)
__device__ __forceinline__ float bnAct(float v, int relu) { return (relu && !(v > 0.f)) ? 0.f : v; }

// ------------------------------------------------------ forward statistics ----
// partial[(ch * chunks + chunk) * 3 + {0,1,2}] = count, mean, M2 of the chunk
template <int VEC>
__global__ void __launch_bounds__(dev::kBlock)
bnStatsKernel(const float *__restrict__ x, float *__restrict__ partial, BnGeom g) {
  __shared__ float red[dev::kBlock / dev::kWave][2];
  const int ch = blockIdx.x / g.chunks, chunk = blockIdx.x - ch * g.chunks;
  const Chunk c = chunkOf(g, chunk);
  // sums are taken about the chunk's first element so that E[d^2] - E[d]^2 does
  // not cancel when |mean| >> sigma
  const float shift = x[((long)c.n0 * g.C + ch) * g.L + c.l0];
  float v[2] = {0.f, 0.f};
  forChunk<VEC>(g, ch, c, [&](long off, auto width) {
    if constexpr (decltype(width)::value == 4) {
      float4 q = *reinterpret_cast<const float4 *>(x + off);
      float d0 = q.x - shift, d1 = q.y - shift, d2 = q.z - shift, d3 = q.w - shift;
      v[0] += (d0 + d1) + (d2 + d3);
      v[1] += (d0 * d0 + d1 * d1) + (d2 * d2 + d3 * d3);
    } else {
      float d = x[off] - shift;
      v[0] += d;
      v[1] += d * d;
    }
  });
  blockSum<2>(v, red);
  if (threadIdx.x == 0) {
    float cnt = (float)c.nN * (float)c.lN;
    float *p = partial + ((long)ch * g.chunks + chunk) * 3;
    p[0] = cnt;
    p[1] = shift + v[0] / cnt;
    p[2] = fmaxf(v[1] - v[0] * v[0] / cnt, 0.f);
  }
}

// Chan et al. pairwise merge of (n, mean, M2), lanes of wave 0 stride the chunk
// list, then a shuffle tree; every lane ends with the channel totals.
__device__ __forceinline__ void mergeStats(const float *__restrict__ p, int chunks, double &n, double &mean,
                                           double &m2) {
  const int lane = threadIdx.x % dev::kWave;
  n = 0.0, mean = 0.0, m2 = 0.0;
  for (int k = lane; k < chunks; k += dev::kWave) {
    double nb = p[k * 3], mb = p[k * 3 + 1], qb = p[k * 3 + 2];
    double tot = n + nb, d = mb - mean;
    mean += d * (nb / tot);
    m2 += qb + d * d * (n * nb / tot);
    n = tot;
  }
#pragma unroll
  for (int o = dev::kWave / 2; o > 0; o >>= 1) {
    double nb = __shfl_xor(n, o, dev::kWave), mb = __shfl_xor(mean, o, dev::kWave),
           qb = __shfl_xor(m2, o, dev::kWave);
    double tot = n + nb;
    if (tot > 0.0) {
      // symmetric form so that both partners compute bit-identical results
      double ma = mean, d = mb - ma;
      mean = (ma * n + mb * nb) / tot;
      m2 = m2 + qb + d * d * (n * nb / tot);
      n = tot;
    }
  }
}

// ------------------------------------------------------------ forward apply ----
// TRAIN: merges the chunk statistics, publishes saveMean/saveStd/running stats
// (chunk 0 only) and normalises; otherwise uses the running statistics.
template <bool TRAIN, int VEC>
__global__ void __launch_bounds__(dev::kBlock)
bnApplyKernel(const float *__restrict__ x, float *__restrict__ y, const float *__restrict__ partial,
              const float *__restrict__ weight, const float *__restrict__ bias, float *__restrict__ runningMean,
              float *__restrict__ runningVar, float *__restrict__ saveMean, float *__restrict__ saveStd, BnGeom g,
              float momentum, float eps, int relu) {
  __shared__ float bc[2];
  // the statistics pass went through the tensor front to back: going back to front meets what it read last
  // while that is still in the last-level cache
  const int bid = gridDim.x - 1 - blockIdx.x;
  const int ch = bid / g.chunks, chunk = bid - ch * g.chunks;
  float mean, invStd;
  if (TRAIN) {
    if (threadIdx.x < dev::kWave) {
      double n, m, m2;
      mergeStats(partial + (long)ch * g.chunks * 3, g.chunks, n, m, m2);
      if (threadIdx.x == 0) {
        // lib/THCUNN/BatchNormalization.cu:181-200, in the Cuda type's float accreal
        float meanF = (float)m, varN = (float)m2, norm = 1.f / (float)n;
        float inv = 0.f;
        if (varN != 0.f || eps != 0.f) inv = 1.f / sqrtf(varN * norm + eps);
        bc[0] = meanF;
        bc[1] = inv;
        if (chunk == 0) {
          float unbiased = varN / ((float)n - 1.f);
          saveMean[ch] = meanF;
          saveStd[ch] = inv;
          runningMean[ch] = (1.f - momentum) * runningMean[ch] + momentum * meanF;
          runningVar[ch] = (1.f - momentum) * runningVar[ch] + momentum * unbiased;
        }
      }
    }
    __syncthreads();
    mean = bc[0];
    invStd = bc[1];
  } else {
    mean = runningMean[ch];
    invStd = 1.f / sqrtf(runningVar[ch] + eps);
  }
  const float gamma = weight ? weight[ch] : 1.f, beta = bias ? bias[ch] : 0.f;
  const Chunk c = chunkOf(g, chunk);
  forChunk<VEC>(g, ch, c, [&](long off, auto width) {
    if constexpr (decltype(width)::value == 4) {
      float4 q = *reinterpret_cast<const float4 *>(x + off), r;
      r.x = bnAct(bnAffine(q.x, mean, invStd, gamma, beta), relu);
      r.y = bnAct(bnAffine(q.y, mean, invStd, gamma, beta), relu);
      r.z = bnAct(bnAffine(q.z, mean, invStd, gamma, beta), relu);
      r.w = bnAct(bnAffine(q.w, mean, invStd, gamma, beta), relu);
      dev::storeStream4(y + off, r);  // written once, read by another kernel: keeps x in the caches for the two-pass re-read
    } else {
      y[off] = bnAct(bnAffine(x[off], mean, invStd, gamma, beta), relu);
    }
  });
}

// ------------------------------------------------- fused ReLU in the backward ----
// With the fused activation the gradient that reaches the normalisation is gradOutput where the forward
// output was positive and 0 elsewhere (lib/THCUNN/Threshold.cu:42-56). The output is not an operand of
// the backward pass: its sign is re-derived from x with the forward's own arithmetic (bnAffine).
struct ReluMask {
  int relu;             // 0: plain batch normalisation, nothing is masked
  int train;            // which statistics stdSrc holds: 1/sigma of the batch, or the running variance
  const float *weight;  // gamma (NULL: 1)
  const float *bias;    // beta (NULL: 0)
  const float *stdSrc;
  float eps;
};
struct ChannelMask {
  int relu;
  float mean, invStd, gamma, beta;
  __device__ ChannelMask(const ReluMask &rm, int ch, float mean_) : relu(rm.relu), mean(mean_), invStd(0.f), gamma(1.f), beta(0.f) {
    if (relu) {
      invStd = rm.train ? rm.stdSrc[ch] : 1.f / sqrtf(rm.stdSrc[ch] + rm.eps);
      gamma = rm.weight ? rm.weight[ch] : 1.f;
      beta = rm.bias ? rm.bias[ch] : 0.f;
    }
  }
  __device__ __forceinline__ float apply(float d, float x) const {
    return (relu && !(bnAffine(x, mean, invStd, gamma, beta) > 0.f)) ? 0.f : d;
  }
  __device__ __forceinline__ void apply(float4 &d, const float4 &q) const {
    d.x = apply(d.x, q.x), d.y = apply(d.y, q.y), d.z = apply(d.z, q.z), d.w = apply(d.w, q.w);
  }
};

// ----------------------------------------------------------- backward sums ----
// partial[(ch * chunks + chunk) * 2 + {0,1}] = sum gy, sum gy * (x - mean)
template <int VEC>
__global__ void __launch_bounds__(dev::kBlock)
bnGradSumsKernel(const float *__restrict__ x, const float *__restrict__ gy, float *__restrict__ partial,
                 const float *__restrict__ meanSrc, BnGeom g, ReluMask rm) {
  __shared__ float red[dev::kBlock / dev::kWave][2];
  const int ch = blockIdx.x / g.chunks, chunk = blockIdx.x - ch * g.chunks;
  const Chunk c = chunkOf(g, chunk);
  const float mean = meanSrc[ch];
  const ChannelMask m(rm, ch, mean);
  float v[2] = {0.f, 0.f};
  forChunk<VEC>(g, ch, c, [&](long off, auto width) {
    if constexpr (decltype(width)::value == 4) {
      float4 q = *reinterpret_cast<const float4 *>(x + off);
      float4 d = *reinterpret_cast<const float4 *>(gy + off);
      m.apply(d, q);
      v[0] += (d.x + d.y) + (d.z + d.w);
      v[1] += (d.x * (q.x - mean) + d.y * (q.y - mean)) + (d.z * (q.z - mean) + d.w * (q.w - mean));
    } else {
      float d = m.apply(gy[off], x[off]);
      v[0] += d;
      v[1] += d * (x[off] - mean);
    }
  });
  blockSum<2>(v, red);
  if (threadIdx.x == 0) {
    float *p = partial + ((long)ch * g.chunks + chunk) * 2;
    p[0] = v[0];
    p[1] = v[1];
  }
}

__device__ __forceinline__ void mergeSums(const float *__restrict__ p, int chunks, double &s0, double &s1) {
  const int lane = threadIdx.x % dev::kWave;
  s0 = 0.0, s1 = 0.0;
  for (int k = lane; k < chunks; k += dev::kWave) {
    s0 += p[k * 2];
    s1 += p[k * 2 + 1];
  }
#pragma unroll
  for (int o = dev::kWave / 2; o > 0; o >>= 1) {
    s0 += __shfl_xor(s0, o, dev::kWave);
    s1 += __shfl_xor(s1, o, dev::kWave);
  }
}

// ---------------------------------------------------------- backward apply ----
// lib/THCUNN/BatchNormalization.cu:253-282. HAVE_SUMS: partial holds the chunk
// sums (needed for train-mode gradInput and for gradWeight/gradBias).
template <bool TRAIN, int VEC>
__global__ void __launch_bounds__(dev::kBlock)
bnBackwardKernel(const float *__restrict__ x, const float *__restrict__ gy, float *__restrict__ gx,
                 const float *__restrict__ partial, float *__restrict__ gradWeight, float *__restrict__ gradBias,
                 const float *__restrict__ weight, const float *__restrict__ meanSrc,
                 const float *__restrict__ stdSrc, BnGeom g, float scale, float eps, ReluMask rm) {
  __shared__ float bc[2];
  const int bid = gridDim.x - 1 - blockIdx.x;  // back to front, see bnApplyKernel
  const int ch = bid / g.chunks, chunk = bid - ch * g.chunks;
  const float mean = meanSrc[ch];
  const ChannelMask m(rm, ch, mean);
  const float stdVal = TRAIN ? stdSrc[ch] : 1.f / sqrtf(stdSrc[ch] + eps);
  const float weightVal = weight ? weight[ch] : 1.f;
  float gradOutputSum = 0.f, dotP = 0.f;
  if (partial) {
    if (threadIdx.x < dev::kWave) {
      double s0, s1;
      mergeSums(partial + (long)ch * g.chunks * 2, g.chunks, s0, s1);
      if (threadIdx.x == 0) {
        bc[0] = (float)s0;
        bc[1] = (float)s1;
      }
    }
    __syncthreads();
    gradOutputSum = bc[0];
    dotP = bc[1];
  }
  const float norm = 1.f / ((float)g.N * (float)g.L);
  const float gradMean = gradOutputSum * norm;
  const float projScale = dotP * norm * stdVal * stdVal;
  const float gradScale = stdVal * weightVal;
  if (gx) {
    const Chunk c = chunkOf(g, chunk);
    forChunk<VEC>(g, ch, c, [&](long off, auto width) {
      if constexpr (decltype(width)::value == 4) {
        float4 d = *reinterpret_cast<const float4 *>(gy + off), r;
        if (TRAIN) {
          float4 q = *reinterpret_cast<const float4 *>(x + off);
          m.apply(d, q);
          r.x = (d.x - (q.x - mean) * projScale - gradMean) * gradScale;
          r.y = (d.y - (q.y - mean) * projScale - gradMean) * gradScale;
          r.z = (d.z - (q.z - mean) * projScale - gradMean) * gradScale;
          r.w = (d.w - (q.w - mean) * projScale - gradMean) * gradScale;
        } else {
          if (m.relu) m.apply(d, *reinterpret_cast<const float4 *>(x + off));
          r.x = d.x * gradScale, r.y = d.y * gradScale, r.z = d.z * gradScale, r.w = d.w * gradScale;
        }
        dev::storeStream4(gx + off, r);
      } else {
        if (TRAIN)
          gx[off] = (m.apply(gy[off], x[off]) - (x[off] - mean) * projScale - gradMean) * gradScale;
        else
          gx[off] = (m.relu ? m.apply(gy[off], x[off]) : gy[off]) * gradScale;
      }
    });
  }
  if (chunk == 0 && threadIdx.x == 0) {
    if (gradWeight) gradWeight[ch] += scale * dotP * stdVal;
    if (gradBias) gradBias[ch] += scale * gradOutputSum;
  }
}

// ============================================================ resident path ==
// When a channel's N*L elements fit the register file of one CU, a single
// 1024-lane workgroup per channel loads them once (R 16-byte loads in flight
// per lane), derives the statistics from registers with the reference's exact
// two-pass formulas (mean first, then sum (x - mean)^2,
// lib/THCUNN/BatchNormalization.cu:181-191) and writes the result: every byte
// crosses HBM exactly once. Needs C of the order of the CU count to fill the chip.
constexpr int kResBlock = 1024;
constexpr int kResWaves = kResBlock / dev::kWave;

__device__ __forceinline__ float blockSum1024(float v, float *red) {
  const int lane = threadIdx.x % dev::kWave, wave = threadIdx.x / dev::kWave;
  v = dev::waveSum(v);
  __syncthreads();  // red may still be read from a previous reduction
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float s = 0.f;
#pragma unroll
  for (int w = 0; w < kResWaves; ++w) s += red[w];
  return s;
}

// Walks the float4s tid, tid + 1024, tid + 2048, ... of channel ch (numbered
// n-major over the channel's N planes of L/4 float4s) without a division per
// step. Offsets are 32-bit byte offsets from the channel's first plane (the
// host checks that the tensor is smaller than 2 GiB).
struct ResWalker {
  int off, l4, stepOff, stepL, L4, wrapOff;
  // fresh: the walk is derived again from a lane index the compiler cannot relate to an earlier walk, so
  // that it recomputes the offsets (one add and a compare per step) instead of keeping one register per
  // step of the earlier walk alive.
  __device__ ResWalker(int L, int C, bool fresh = false) : L4(L >> 2) {
    int tid = threadIdx.x;
    if (fresh) __asm__ volatile("" : "+v"(tid));
    const int n = tid / L4;
    l4 = tid - n * L4;
    const int stepN = kResBlock / L4;
    stepL = kResBlock - stepN * L4;
    off = (n * C * L + (l4 << 2)) * 4;
    stepOff = (stepN * C * L + (stepL << 2)) * 4;
    wrapOff = (C * L - L) * 4;
  }
  __device__ int offset() const { return off; }
  __device__ void next() {
    off += stepOff;
    l4 += stepL;
    if (l4 >= L4) {
      l4 -= L4;
      off += wrapOff;
    }
  }
};

template <int R>
__global__ void __launch_bounds__(kResBlock)
bnFwdResident(const float *__restrict__ x, float *__restrict__ y, const float *__restrict__ weight,
              const float *__restrict__ bias, float *__restrict__ runningMean, float *__restrict__ runningVar,
              float *__restrict__ saveMean, float *__restrict__ saveStd, int N, int C, int L, float momentum,
              float eps, int relu) {
  __shared__ float red[kResWaves];
  const int ch = blockIdx.x;
  const int total4 = N * (L >> 2);
  const long span = ((long)(N - 1) * C * L + L) * 4;  // bytes from the channel's first to past its last element
  const __amdgpu_buffer_rsrc_t xr = dev::makeRsrc(x + (long)ch * L, span), yr = dev::makeRsrc(y + (long)ch * L, span);
  float4 v[R];
  {
    ResWalker wk(L, C);
#pragma unroll
    for (int u = 0; u < R; ++u) {
      v[u] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (u * kResBlock + (int)threadIdx.x < total4) v[u] = dev::bufLoad4(xr, wk.offset());
      wk.next();
    }
  }
  const float cnt = (float)N * (float)L, norm = 1.f / cnt;
  float s = 0.f;
#pragma unroll
  for (int u = 0; u < R; ++u) s += (v[u].x + v[u].y) + (v[u].z + v[u].w);
  const float mean = blockSum1024(s, red) * norm;
  float q = 0.f;
#pragma unroll
  for (int u = 0; u < R; ++u)
    if (u * kResBlock + (int)threadIdx.x < total4) {
      float a = v[u].x - mean, b = v[u].y - mean, c = v[u].z - mean, d = v[u].w - mean;
      q += (a * a + b * b) + (c * c + d * d);
    }
  const float varN = blockSum1024(q, red);
  float invStd = 0.f;
  if (varN != 0.f || eps != 0.f) invStd = 1.f / sqrtf(varN * norm + eps);
  if (threadIdx.x == 0) {
    float unbiased = varN / (cnt - 1.f);
    saveMean[ch] = mean;
    saveStd[ch] = invStd;
    runningMean[ch] = (1.f - momentum) * runningMean[ch] + momentum * mean;
    runningVar[ch] = (1.f - momentum) * runningVar[ch] + momentum * unbiased;
  }
  const float gamma = weight ? weight[ch] : 1.f, beta = bias ? bias[ch] : 0.f;
  ResWalker wk(L, C);
#pragma unroll
  for (int u = 0; u < R; ++u) {
    if (u * kResBlock + (int)threadIdx.x < total4) {
      float4 r;
      r.x = bnAct(bnAffine(v[u].x, mean, invStd, gamma, beta), relu);
      r.y = bnAct(bnAffine(v[u].y, mean, invStd, gamma, beta), relu);
      r.z = bnAct(bnAffine(v[u].z, mean, invStd, gamma, beta), relu);
      r.w = bnAct(bnAffine(v[u].w, mean, invStd, gamma, beta), relu);
      dev::bufStoreStream4(yr, wk.offset(), r);
    }
    wk.next();
  }
}

// Backward with gradOutput resident in registers. KEEPX: (x - mean) stays in
// registers as well (2R float4 per lane). Otherwise x is consumed in batches; XL > 0: the first XL float4
// of x per lane wait in LDS for the apply phase and the other R - XL in registers, so that x crosses HBM
// once as well; XL == 0: nothing of x is kept (no apply phase, or one that does not need x).
// x and gradOutput are read with the non-temporal hint: the backward pass is the last reader of both in a training
// step (cfg3, N 64, 256 x 28 x 28: 27.0 -> 25.9 us per call, forward + backward step 46.0 -> 44.5 us).
template <int R, bool TRAIN, bool KEEPX, int XL = 0>
__global__ void __launch_bounds__(kResBlock)
bnBwdResident(const float *__restrict__ x, const float *__restrict__ gy, float *__restrict__ gx,
              float *__restrict__ gradWeight, float *__restrict__ gradBias, const float *__restrict__ weight,
              const float *__restrict__ meanSrc, const float *__restrict__ stdSrc, int N, int C, int L, float scale,
              float eps, ReluMask rm) {
  __shared__ float red[kResWaves];
  extern __shared__ float4 xpark[];  // XL float4 of x per lane
  constexpr int XK = XL > 0 ? R - XL : 0;
  static_assert(!KEEPX || XL == 0, "either everything of x in registers or the split");
  float4 xk[XK > 0 ? XK : 1];
  const int ch = blockIdx.x;
  const int total4 = N * (L >> 2);
  const float mean = meanSrc[ch];
  const float stdVal = TRAIN ? stdSrc[ch] : 1.f / sqrtf(stdSrc[ch] + eps);
  const float weightVal = weight ? weight[ch] : 1.f;
  const ChannelMask m(rm, ch, mean);
  const long span = ((long)(N - 1) * C * L + L) * 4;
  const __amdgpu_buffer_rsrc_t xr = dev::makeRsrc(x + (long)ch * L, span), gr = dev::makeRsrc(gy + (long)ch * L, span);
  const __amdgpu_buffer_rsrc_t or_ = dev::makeRsrc(gx ? gx + (long)ch * L : x, gx ? span : 0);
  constexpr int XB = (R > 8 && XL == 0) ? 8 : 4;  // x float4 per lane requested together when x is not kept in registers
  float4 d[R], xc[KEEPX ? R : 1];
  float s0 = 0.f, s1 = 0.f;
  {
    ResWalker wk(L, C);
    if (KEEPX) {
#pragma unroll
      for (int u = 0; u < R; ++u) {
        d[u] = make_float4(0.f, 0.f, 0.f, 0.f);
        xc[KEEPX ? u : 0] = make_float4(mean, mean, mean, mean);
        if (u * kResBlock + (int)threadIdx.x < total4) {
          const int off = wk.offset();
          d[u] = dev::bufLoadStream4(gr, off);
          xc[KEEPX ? u : 0] = dev::bufLoadStream4(xr, off);
        }
        wk.next();
      }
#pragma unroll
      for (int u = 0; u < R; ++u) {
        float4 &q = xc[KEEPX ? u : 0];
        m.apply(d[u], q);
        q.x -= mean, q.y -= mean, q.z -= mean, q.w -= mean;
        s0 += (d[u].x + d[u].y) + (d[u].z + d[u].w);
        s1 += (d[u].x * q.x + d[u].y * q.y) + (d[u].z * q.z + d[u].w * q.w);
      }
    } else {
      // gy for the whole channel first (kept), x in batches of 4 (consumed)
      ResWalker wx = wk;
#pragma unroll
      for (int u = 0; u < R; ++u) {
        d[u] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (u * kResBlock + (int)threadIdx.x < total4) d[u] = dev::bufLoadStream4(gr, wk.offset());
        wk.next();
      }
#pragma unroll
      for (int u0 = 0; u0 < R; u0 += XB) {
        float4 q[XB];
#pragma unroll
        for (int k = 0; k < XB; ++k) {
          q[k] = make_float4(mean, mean, mean, mean);
          if (u0 + k < R) {
            if ((u0 + k) * kResBlock + (int)threadIdx.x < total4) q[k] = dev::bufLoadStream4(xr, wx.offset());
            wx.next();
          }
        }
#pragma unroll
        for (int k = 0; k < XB; ++k)
          if (u0 + k < R) {
            if (u0 + k < XL)
              xpark[(u0 + k) * kResBlock + threadIdx.x] = q[k];
            else if (XL > 0)
              xk[XK > 0 ? u0 + k - XL : 0] = q[k];
          }
#pragma unroll
        for (int k = 0; k < XB; ++k)
          if (u0 + k < R) {
            m.apply(d[u0 + k], q[k]);
            const float4 &g4 = d[u0 + k];
            s0 += (g4.x + g4.y) + (g4.z + g4.w);
            s1 += (g4.x * (q[k].x - mean) + g4.y * (q[k].y - mean)) + (g4.z * (q[k].z - mean) + g4.w * (q[k].w - mean));
          }
        __asm__ volatile("" ::: "memory");  // keep the batches apart: XB loads in flight, not R
      }
    }
  }
  const float gradOutputSum = blockSum1024(s0, red);
  const float dotP = blockSum1024(s1, red);
  const float norm = 1.f / ((float)N * (float)L);
  const float gradMean = gradOutputSum * norm;
  const float projScale = dotP * norm * stdVal * stdVal;
  const float gradScale = stdVal * weightVal;
  if (gx) {
    ResWalker wk(L, C, XL > 0);
    if (KEEPX || !TRAIN) {
#pragma unroll
      for (int u = 0; u < R; ++u) {
        if (u * kResBlock + (int)threadIdx.x < total4) {
          float4 r;
          const float4 q = xc[KEEPX ? u : 0];
          if (TRAIN) {
            r.x = (d[u].x - q.x * projScale - gradMean) * gradScale;
            r.y = (d[u].y - q.y * projScale - gradMean) * gradScale;
            r.z = (d[u].z - q.z * projScale - gradMean) * gradScale;
            r.w = (d[u].w - q.w * projScale - gradMean) * gradScale;
          } else {
            r.x = d[u].x * gradScale, r.y = d[u].y * gradScale, r.z = d[u].z * gradScale, r.w = d[u].w * gradScale;
          }
          dev::bufStoreStream4(or_, wk.offset(), r);
        }
        wk.next();
      }
    } else {
#pragma unroll
      for (int u0 = 0; u0 < R; u0 += XB) {
        float4 q[XB];
        int off[XB];
#pragma unroll
        for (int k = 0; k < XB; ++k) {
          off[k] = -1;
          q[k] = make_float4(mean, mean, mean, mean);
          if (u0 + k < R) {
            if ((u0 + k) * kResBlock + (int)threadIdx.x < total4) {
              off[k] = wk.offset();
              if (XL == 0)
                q[k] = dev::bufLoad4(xr, off[k]);
              else if (u0 + k < XL)
                q[k] = xpark[(u0 + k) * kResBlock + threadIdx.x];
              else
                q[k] = xk[XK > 0 ? u0 + k - XL : 0];
            }
            wk.next();
          }
        }
#pragma unroll
        for (int k = 0; k < XB; ++k)
          if (u0 + k < R && off[k] >= 0) {
            const float4 &g4 = d[u0 + k];
            float4 r;
            r.x = (g4.x - (q[k].x - mean) * projScale - gradMean) * gradScale;
            r.y = (g4.y - (q[k].y - mean) * projScale - gradMean) * gradScale;
            r.z = (g4.z - (q[k].z - mean) * projScale - gradMean) * gradScale;
            r.w = (g4.w - (q[k].w - mean) * projScale - gradMean) * gradScale;
            dev::bufStoreStream4(or_, off[k], r);
          }
        __asm__ volatile("" ::: "memory");
      }
    }
  }
  if (threadIdx.x == 0) {
    if (gradWeight) gradWeight[ch] += scale * dotP * stdVal;
    if (gradBias) gradBias[ch] += scale * gradOutputSum;
  }
}

// ---- resident path for small channels of any plane size -----------------------------------
// The last stages of a network have planes of 49 elements (7x7): not a multiple of 4, so the 16-byte
// walkers above do not apply, and a channel holds only N*L of the order of 3000 elements. One 256-lane
// workgroup per channel keeps them in registers, RS scalar elements per lane (element e = tid + 256 u is
// image e / L, position e % L: the lanes of a wave read runs of L consecutive floats); the formulas
// are those of the 1024-lane kernels.
constexpr int kSmallBlock = 256;  // channels of up to 32 * 256 elements; up to 32 * 1024 take 1024 lanes

template <int BS>
__device__ __forceinline__ float blockSumSmall(float v, float *red) {
  const int lane = threadIdx.x % dev::kWave, wave = threadIdx.x / dev::kWave;
  v = dev::waveSum(v);
  __syncthreads();  // red may still be read from a previous reduction
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float s = 0.f;
#pragma unroll
  for (int w = 0; w < BS / dev::kWave; w += 4) s += (red[w] + red[w + 1]) + (red[w + 2] + red[w + 3]);
  return s;
}

// element offsets (in floats, from the channel's first plane) of this lane; -1 past the channel
template <int RS, int BS>
__device__ __forceinline__ void smallOffsets(int (&off)[RS], int N, int C, int L, unsigned magicL) {
#pragma unroll
  for (int u = 0; u < RS; ++u) {
    const int e = u * BS + (int)threadIdx.x;
    const int n = dev::fastDiv(e, magicL);
    off[u] = e < N * L ? n * C * L + (e - n * L) : -1;
  }
}

template <int RS, int BS>
__global__ void __launch_bounds__(BS)
bnFwdSmall(const float *__restrict__ x, float *__restrict__ y, const float *__restrict__ weight,
           const float *__restrict__ bias, float *__restrict__ runningMean, float *__restrict__ runningVar,
           float *__restrict__ saveMean, float *__restrict__ saveStd, int N, int C, int L, unsigned magicL,
           float momentum, float eps, int relu) {
  __shared__ float red[BS / dev::kWave];
  const int ch = blockIdx.x;
  const float *xc = x + (long)ch * L;
  float *yc = y + (long)ch * L;
  int off[RS];
  smallOffsets<RS, BS>(off, N, C, L, magicL);
  float v[RS];
#pragma unroll
  for (int u = 0; u < RS; ++u) v[u] = off[u] >= 0 ? xc[off[u]] : 0.f;
  const float cnt = (float)N * (float)L, norm = 1.f / cnt;
  float s = 0.f;
#pragma unroll
  for (int u = 0; u < RS; ++u) s += v[u];
  const float mean = blockSumSmall<BS>(s, red) * norm;
  float q = 0.f;
#pragma unroll
  for (int u = 0; u < RS; ++u)
    if (off[u] >= 0) q += (v[u] - mean) * (v[u] - mean);
  const float varN = blockSumSmall<BS>(q, red);
  float invStd = 0.f;
  if (varN != 0.f || eps != 0.f) invStd = 1.f / sqrtf(varN * norm + eps);
  if (threadIdx.x == 0) {
    float unbiased = varN / (cnt - 1.f);
    saveMean[ch] = mean;
    saveStd[ch] = invStd;
    runningMean[ch] = (1.f - momentum) * runningMean[ch] + momentum * mean;
    runningVar[ch] = (1.f - momentum) * runningVar[ch] + momentum * unbiased;
  }
  const float gamma = weight ? weight[ch] : 1.f, beta = bias ? bias[ch] : 0.f;
#pragma unroll
  for (int u = 0; u < RS; ++u)
    if (off[u] >= 0) yc[off[u]] = bnAct(bnAffine(v[u], mean, invStd, gamma, beta), relu);
}

template <int RS, bool TRAIN, int BS>
__global__ void __launch_bounds__(BS)
bnBwdSmall(const float *__restrict__ x, const float *__restrict__ gy, float *__restrict__ gx,
           float *__restrict__ gradWeight, float *__restrict__ gradBias, const float *__restrict__ weight,
           const float *__restrict__ meanSrc, const float *__restrict__ stdSrc, int N, int C, int L, unsigned magicL,
           float scale, float eps, ReluMask rm) {
  __shared__ float red[BS / dev::kWave];
  const int ch = blockIdx.x;
  const float *xc = x + (long)ch * L, *gc = gy + (long)ch * L;
  const float mean = meanSrc[ch];
  const ChannelMask m(rm, ch, mean);
  const float stdVal = TRAIN ? stdSrc[ch] : 1.f / sqrtf(stdSrc[ch] + eps);
  const float weightVal = weight ? weight[ch] : 1.f;
  int off[RS];
  smallOffsets<RS, BS>(off, N, C, L, magicL);
  float d[RS], xm[RS];
#pragma unroll
  for (int u = 0; u < RS; ++u) {
    d[u] = off[u] >= 0 ? gc[off[u]] : 0.f;
    xm[u] = off[u] >= 0 ? xc[off[u]] : mean;
  }
  float s0 = 0.f, s1 = 0.f;
#pragma unroll
  for (int u = 0; u < RS; ++u) {
    d[u] = m.apply(d[u], xm[u]);
    xm[u] -= mean;
    s0 += d[u];
    s1 += d[u] * xm[u];
  }
  const float gradOutputSum = blockSumSmall<BS>(s0, red);
  const float dotP = blockSumSmall<BS>(s1, red);
  const float norm = 1.f / ((float)N * (float)L);
  const float gradMean = gradOutputSum * norm;
  const float projScale = dotP * norm * stdVal * stdVal;
  const float gradScale = stdVal * weightVal;
  if (gx) {
    float *oc = gx + (long)ch * L;
#pragma unroll
    for (int u = 0; u < RS; ++u)
      if (off[u] >= 0) oc[off[u]] = TRAIN ? (d[u] - xm[u] * projScale - gradMean) * gradScale : d[u] * gradScale;
  }
  if (threadIdx.x == 0) {
    if (gradWeight) gradWeight[ch] += scale * dotP * stdVal;
    if (gradBias) gradBias[ch] += scale * gradOutputSum;
  }
}

// -------------------------------------------------------------- host side ----
struct BnView {
  BnGeom g;
  bool vec;  // plane size a multiple of 4 and every tensor 16-byte aligned
  int mode;  // forChunk: 1 = vec, 2 = 16-byte accesses around unaligned plane starts, 0 = element by element
};

// N x C x L view of the input (lib/THCUNN/generic/BatchNormalization.cu:8-32)
// and the chunking policy.
BnView bnView(const THCudaTensor *t, std::initializer_list<const void *> ptrs) {
  const Tensor *e = erase(t);
  THC_ARG_CHECK(e->nDimension >= 2, 2, "input of at least 2 dimensions (batch x features) expected, got: %s",
                sizeDesc(e).c_str());
  BnView v;
  BnGeom &g = v.g;
  long L = 1;
  for (int i = 2; i < e->nDimension; ++i) L *= e->size[i];
  if (e->size[0] >= 0x7fffffffL || e->size[1] >= 0x7fffffffL || L >= 0x7fffffffL)
    error("BatchNormalization: dimensions of 2^31 or more elements are not supported");
  g.N = (int)e->size[0], g.C = (int)e->size[1], g.L = (int)L;
  v.vec = g.L % 4 == 0;
  bool aligned = true;
  for (const void *p : ptrs) aligned = aligned && (p == nullptr || launch::aligned16(p));
  v.vec = v.vec && aligned;
  v.mode = v.vec ? 1 : (aligned && g.L >= 8 ? 2 : 0);
  // ~8K elements (32 KB) per workgroup: 8 x 16-byte loads per lane
  const int target = 8192;
  if (g.L >= target) {
    g.planesPerChunk = 1;
    g.segsPerPlane = launch::ceilDiv(g.L, target);
    g.segLen = launch::roundUp(launch::ceilDiv(g.L, g.segsPerPlane), 4);
    g.segsPerPlane = launch::ceilDiv(g.L, g.segLen);
  } else {
    g.segsPerPlane = 1;
    g.segLen = g.L;
    g.planesPerChunk = std::max(1, std::min(g.N, target / std::max(g.L, 1)));
    // keep at least ~2048 workgroups in flight when the batch allows it
    while (g.planesPerChunk > 1 && (long)g.C * launch::ceilDiv(g.N, g.planesPerChunk) < launch::kMinBlocks)
      g.planesPerChunk = (g.planesPerChunk + 1) / 2;
  }
  g.chunks = launch::ceilDiv(g.N, g.planesPerChunk) * g.segsPerPlane;
  return v;
}

void checkVector(const THCudaTensor *t, const char *name, int C, bool required) {
  if (!t) {
    if (required) error("%s tensor expected", name);
    return;
  }
  const Tensor *e = erase(t);
  if (numel(e) != C || !isContiguous(e))
    error("%s must be a contiguous vector of %d elements, got: %s", name, C, sizeDesc(e).c_str());
}

inline float *dataOrNull(const THCudaTensor *t) { return t ? data(t) : nullptr; }

constexpr int kMaxDevices = 64;
inline int currentDevice() {
  int dv = 0;
  THC_HIP_CHECK(hipGetDevice(&dv));
  if (dv < 0 || dv >= kMaxDevices) error("BatchNormalization: device ordinal %d not supported", dv);
  return dv;
}

// The resident kernels hold a channel in the registers of one 1024-lane
// workgroup: at most maxR float4 per lane, and enough channels to occupy the chip.
int residentR(const BnView &v, int maxR) {
  if (g_switches.bnChunked == 1) return 0;
  const BnGeom &g = v.g;
  if (!v.vec || g.C < 96 || g.L / 4 > kResBlock || (long)g.N * g.C * g.L * 4 >= 0x7fffffffL) return 0;
  long total4 = (long)g.N * (g.L / 4);
  int need = (int)((total4 + kResBlock - 1) / kResBlock);
  const int sizes[] = {2, 4, 8, 12, 13, 14};
  for (int r : sizes)
    if (need <= r && r <= maxR) return r;
  return 0;
}

// Elements per lane and lanes per workgroup of the small-channel kernels (rs 0: not applicable): planes whose
// size is not a multiple of 4 (the 16-byte kernels take the others), channels of at most 32 * 1024 elements,
// enough channels to occupy the chip.
struct SmallChoice {
  int rs, bs;
};
SmallChoice smallR(const BnView &v) {
  if (g_switches.bnChunked == 1) return {0, 0};
  const BnGeom &g = v.g;
  const long NL = (long)g.N * g.L;
  if (g.L % 4 == 0 || g.C < 96 || NL > 32 * kResBlock || (long)g.N * g.C * g.L >= 0x7fffffffL) return {0, 0};
  const int bs = NL <= 32 * kSmallBlock ? kSmallBlock : kResBlock;
  const int need = (int)((NL + bs - 1) / bs);
  const int sizes[] = {4, 8, 16, 32};
  for (int r : sizes)
    if (need <= r) return {r, bs};
  return {0, 0};
}

// lib/THCUNN/generic/BatchNormalization.cu:34-66; relu: Threshold(0, 0) applied to every element before it is stored
void bnUpdateOutput(THCState *state, THCudaTensor *input_, THCudaTensor *output_, THCudaTensor *weight_,
                    THCudaTensor *bias_, THCudaTensor *runningMean_, THCudaTensor *runningVar_,
                    THCudaTensor *saveMean_, THCudaTensor *saveStd_, bool train, double momentum, double eps,
                    int relu) {
  THC_ARG_CHECK(input_ != nullptr, 2, "input tensor expected");
  THC_ARG_CHECK(output_ != nullptr, 3, "output tensor expected");
  tensorResize(state, erase(output_), input_->nDimension, input_->size, sizeof(float));  // resizeAs (:40)
  if (!isContiguous(erase(output_))) error("output tensor has to be contiguous");
  Contiguous in(state, input_);
  BnView v = bnView(input_, {in.ptr(), data(output_)});
  const BnGeom &g = v.g;
  checkVector(weight_, "weight", g.C, false);
  checkVector(bias_, "bias", g.C, false);
  checkVector(runningMean_, "runningMean", g.C, true);
  checkVector(runningVar_, "runningVar", g.C, true);
  if (train) {
    checkVector(saveMean_, "saveMean", g.C, true);
    checkVector(saveStd_, "saveStd", g.C, true);
  }
  if ((long)g.N * g.C * g.L == 0) return;
  if ((long)g.C * g.chunks >= 0x7fffffffL) error("BatchNormalization: grid too large");
  hipStream_t s = state->stream;
  dim3 grid((unsigned)(g.C * g.chunks)), block(dev::kBlock);
  if (int R = train ? residentR(v, 14) : 0) {
#define BN_FWD_RES(RR)                                                                                              \
  if (R == RR)                                                                                                      \
    bnFwdResident<RR><<<g.C, kResBlock, 0, s>>>(in.ptr(), data(output_), dataOrNull(weight_), dataOrNull(bias_),    \
                                                data(runningMean_), data(runningVar_), data(saveMean_),             \
                                                data(saveStd_), g.N, g.C, g.L, (float)momentum, (float)eps, relu);
    BN_FWD_RES(2) BN_FWD_RES(4) BN_FWD_RES(8) BN_FWD_RES(12) BN_FWD_RES(13) BN_FWD_RES(14)
#undef BN_FWD_RES
    THC_HIP_CHECK(hipGetLastError());
    return;
  }
  if (const SmallChoice sc = train ? smallR(v) : SmallChoice{0, 0}; sc.rs) {
#define BN_FWD_SMALL(RR, BS)                                                                                        \
  if (sc.rs == RR && sc.bs == BS)                                                                                   \
    bnFwdSmall<RR, BS><<<g.C, BS, 0, s>>>(in.ptr(), data(output_), dataOrNull(weight_), dataOrNull(bias_),          \
                                          data(runningMean_), data(runningVar_), data(saveMean_), data(saveStd_),   \
                                          g.N, g.C, g.L, dev::magicOf(g.L), (float)momentum, (float)eps, relu);
    BN_FWD_SMALL(4, kSmallBlock) BN_FWD_SMALL(8, kSmallBlock) BN_FWD_SMALL(16, kSmallBlock) BN_FWD_SMALL(32, kSmallBlock)
    BN_FWD_SMALL(16, kResBlock) BN_FWD_SMALL(32, kResBlock)
#undef BN_FWD_SMALL
    THC_HIP_CHECK(hipGetLastError());
    return;
  }
  if (train) {
    // chunk statistics: BatchNormalization has no buffer argument, they live in the stream's scratch space
    float *p = (float *)streamScratch(state, (size_t)g.C * g.chunks * 3 * sizeof(float));
#define BN_FWD_TRAIN(MODE)                                                                                        \
  {                                                                                                               \
    bnStatsKernel<MODE><<<grid, block, 0, s>>>(in.ptr(), p, g);                                                   \
    bnApplyKernel<true, MODE><<<grid, block, 0, s>>>(in.ptr(), data(output_), p, dataOrNull(weight_),             \
                                                     dataOrNull(bias_), data(runningMean_), data(runningVar_),    \
                                                     data(saveMean_), data(saveStd_), g, (float)momentum,         \
                                                     (float)eps, relu);                                           \
  }
    if (v.mode == 1) BN_FWD_TRAIN(1) else if (v.mode == 2) BN_FWD_TRAIN(2) else BN_FWD_TRAIN(0)
#undef BN_FWD_TRAIN
  } else {
#define BN_FWD_EVAL(MODE)                                                                                         \
  bnApplyKernel<false, MODE><<<grid, block, 0, s>>>(in.ptr(), data(output_), nullptr, dataOrNull(weight_),        \
                                                    dataOrNull(bias_), data(runningMean_), data(runningVar_),     \
                                                    nullptr, nullptr, g, (float)momentum, (float)eps, relu);
    if (v.mode == 1) BN_FWD_EVAL(1) else if (v.mode == 2) BN_FWD_EVAL(2) else BN_FWD_EVAL(0)
#undef BN_FWD_EVAL
  }
  THC_HIP_CHECK(hipGetLastError());
}

// lib/THCUNN/generic/BatchNormalization.cu:68-94; relu: gradOutput counts only where the fused forward output was
// positive (bias_ is needed to re-derive that sign from the input)
void bnBackward(THCState *state, THCudaTensor *input_, THCudaTensor *gradOutput_, THCudaTensor *gradInput_,
                THCudaTensor *gradWeight_, THCudaTensor *gradBias_, THCudaTensor *weight_, THCudaTensor *bias_,
                THCudaTensor *runningMean_, THCudaTensor *runningVar_, THCudaTensor *saveMean_,
                THCudaTensor *saveStd_, bool train, double scale, double eps, int relu) {
  THC_ARG_CHECK(input_ != nullptr, 2, "input tensor expected");
  THC_ARG_CHECK(gradOutput_ != nullptr, 3, "gradOutput tensor expected");
  if (!sameSize(erase(input_), erase(gradOutput_)))  // THCUNN_check_shape (:74)
    error("input_ and gradOutput_ shapes do not match: input_ %s, gradOutput_ %s", sizeDesc(erase(input_)).c_str(),
          sizeDesc(erase(gradOutput_)).c_str());
  if (gradInput_) {
    // the reference writes through gradInput as it finds it; a tensor of another
    // shape would be written out of bounds there, here it is an error
    if (!sameSize(erase(input_), erase(gradInput_)))
      error("input_ and gradInput_ shapes do not match: input_ %s, gradInput_ %s", sizeDesc(erase(input_)).c_str(),
            sizeDesc(erase(gradInput_)).c_str());
    if (!isContiguous(erase(gradInput_))) error("gradInput tensor has to be contiguous");
  }
  Contiguous in(state, input_);
  Contiguous go(state, gradOutput_);
  BnView v = bnView(input_, {in.ptr(), go.ptr(), gradInput_ ? data(gradInput_) : nullptr});
  const BnGeom &g = v.g;
  checkVector(gradWeight_, "gradWeight", g.C, false);
  checkVector(gradBias_, "gradBias", g.C, false);
  checkVector(weight_, "weight", g.C, false);
  if (relu) checkVector(bias_, "bias", g.C, false);
  if (train) {
    checkVector(saveMean_, "saveMean", g.C, true);
    checkVector(saveStd_, "saveStd", g.C, true);
  } else {
    checkVector(runningMean_, "runningMean", g.C, true);
    checkVector(runningVar_, "runningVar", g.C, true);
  }
  if ((long)g.N * g.C * g.L == 0) return;
  if (!gradInput_ && !gradWeight_ && !gradBias_) return;
  if ((long)g.C * g.chunks >= 0x7fffffffL) error("BatchNormalization: grid too large");
  hipStream_t s = state->stream;
  dim3 grid((unsigned)(g.C * g.chunks)), block(dev::kBlock);
  const float *meanSrc = train ? data(saveMean_) : data(runningMean_);
  const float *stdSrc = train ? data(saveStd_) : data(runningVar_);
  const ReluMask rm{relu, train ? 1 : 0, dataOrNull(weight_), relu ? dataOrNull(bias_) : nullptr, stdSrc, (float)eps};
  const bool needSums = (train && gradInput_) || gradWeight_ || gradBias_;
  if (int R = needSums ? residentR(v, 13) : 0) {
    float *gxp = gradInput_ ? data(gradInput_) : nullptr;
#define BN_BWD_RES(RR)                                                                                             \
  if (R == RR) {                                                                                                   \
    /* x between the two phases: 9 of the up to 13 float4 per lane in LDS (144 KB of the CU's 160 KB), the rest   \
       in registers */                                                                                             \
    constexpr int XL = RR > 8 ? 9 : 0;                                                                             \
    constexpr size_t lds = (size_t)XL * kResBlock * sizeof(float4);                                                \
    if (train && gxp && XL > 0) {                                                                                  \
      /* once per kernel instance and device: allow more than 64 KB of dynamic LDS */                             \
      static std::atomic<bool> ldsRaised[kMaxDevices];                                                             \
      const int dv = currentDevice();                                                                              \
      if (!ldsRaised[dv].load()) {                                                                                 \
        THC_HIP_CHECK(hipFuncSetAttribute((const void *)bnBwdResident<RR, true, false, XL>,                        \
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));                  \
        ldsRaised[dv].store(true);                                                                                 \
      }                                                                                                            \
      bnBwdResident<RR, true, false, XL><<<g.C, kResBlock, lds, s>>>(in.ptr(), go.ptr(), gxp,                      \
                                                        dataOrNull(gradWeight_), dataOrNull(gradBias_),            \
                                                        dataOrNull(weight_), meanSrc, stdSrc, g.N, g.C, g.L,       \
                                                        (float)scale, (float)eps, rm);                             \
    } else if (train) {                                                                                            \
      bnBwdResident<RR, true, (RR <= 8)><<<g.C, kResBlock, 0, s>>>(in.ptr(), go.ptr(), gxp, dataOrNull(gradWeight_), \
                                                        dataOrNull(gradBias_), dataOrNull(weight_), meanSrc,       \
                                                        stdSrc, g.N, g.C, g.L, (float)scale, (float)eps, rm);      \
    } else {                                                                                                       \
      bnBwdResident<RR, false, (RR <= 8)><<<g.C, kResBlock, 0, s>>>(in.ptr(), go.ptr(), gxp, dataOrNull(gradWeight_), \
                                                         dataOrNull(gradBias_), dataOrNull(weight_), meanSrc,      \
                                                         stdSrc, g.N, g.C, g.L, (float)scale, (float)eps, rm);     \
    }                                                                                                              \
  }
    BN_BWD_RES(2) BN_BWD_RES(4) BN_BWD_RES(8) BN_BWD_RES(12) BN_BWD_RES(13)
#undef BN_BWD_RES
    THC_HIP_CHECK(hipGetLastError());
    return;
  }
  if (const SmallChoice sc = needSums ? smallR(v) : SmallChoice{0, 0}; sc.rs) {
    float *gxp = gradInput_ ? data(gradInput_) : nullptr;
#define BN_BWD_SMALL(RR, BS)                                                                                      \
  if (sc.rs == RR && sc.bs == BS) {                                                                               \
    if (train)                                                                                                    \
      bnBwdSmall<RR, true, BS><<<g.C, BS, 0, s>>>(in.ptr(), go.ptr(), gxp, dataOrNull(gradWeight_),               \
                                                  dataOrNull(gradBias_), dataOrNull(weight_), meanSrc, stdSrc,    \
                                                  g.N, g.C, g.L, dev::magicOf(g.L), (float)scale, (float)eps, rm); \
    else                                                                                                          \
      bnBwdSmall<RR, false, BS><<<g.C, BS, 0, s>>>(in.ptr(), go.ptr(), gxp, dataOrNull(gradWeight_),              \
                                                   dataOrNull(gradBias_), dataOrNull(weight_), meanSrc, stdSrc,   \
                                                   g.N, g.C, g.L, dev::magicOf(g.L), (float)scale, (float)eps, rm); \
  }
    BN_BWD_SMALL(4, kSmallBlock) BN_BWD_SMALL(8, kSmallBlock) BN_BWD_SMALL(16, kSmallBlock) BN_BWD_SMALL(32, kSmallBlock)
    BN_BWD_SMALL(16, kResBlock) BN_BWD_SMALL(32, kResBlock)
#undef BN_BWD_SMALL
    THC_HIP_CHECK(hipGetLastError());
    return;
  }
  float *p = nullptr;
  if (needSums) {
    p = (float *)streamScratch(state, (size_t)g.C * g.chunks * 2 * sizeof(float));
    if (v.mode == 1)
      bnGradSumsKernel<1><<<grid, block, 0, s>>>(in.ptr(), go.ptr(), p, meanSrc, g, rm);
    else if (v.mode == 2)
      bnGradSumsKernel<2><<<grid, block, 0, s>>>(in.ptr(), go.ptr(), p, meanSrc, g, rm);
    else
      bnGradSumsKernel<0><<<grid, block, 0, s>>>(in.ptr(), go.ptr(), p, meanSrc, g, rm);
    THC_HIP_CHECK(hipGetLastError());
  }
  BnGeom ga = g;
  dim3 gridApply = grid;
  float *gx = gradInput_ ? data(gradInput_) : nullptr;
  float *gw = dataOrNull(gradWeight_), *gb = dataOrNull(gradBias_);
  const float *w = dataOrNull(weight_);
#define BN_BWD(TRAIN, VEC)                                                                                   \
  bnBackwardKernel<TRAIN, VEC><<<gridApply, block, 0, s>>>(in.ptr(), go.ptr(), gx, p, gw, gb, w, meanSrc, stdSrc, ga, \
                                                           (float)scale, (float)eps, rm)
  if (train) {
    if (v.mode == 1)
      BN_BWD(true, 1);
    else if (v.mode == 2)
      BN_BWD(true, 2);
    else
      BN_BWD(true, 0);
  } else {
    if (v.mode == 1)
      BN_BWD(false, 1);
    else if (v.mode == 2)
      BN_BWD(false, 2);
    else
      BN_BWD(false, 0);
  }
#undef BN_BWD
  THC_HIP_CHECK(hipGetLastError());
}

}  // namespace

extern "C" {

void THNN_CudaBatchNormalization_updateOutput(THCState *state, THCudaTensor *input_, THCudaTensor *output_,
                                              THCudaTensor *weight_, THCudaTensor *bias_,
                                              THCudaTensor *runningMean_, THCudaTensor *runningVar_,
                                              THCudaTensor *saveMean_, THCudaTensor *saveStd_, bool train,
                                              double momentum, double eps) {
  THNN_ENTER
  bnUpdateOutput(state, input_, output_, weight_, bias_, runningMean_, runningVar_, saveMean_, saveStd_, train, momentum,
                 eps, 0);
  THNN_LEAVE
}

void THNN_CudaBatchNormalization_backward(THCState *state, THCudaTensor *input_, THCudaTensor *gradOutput_,
                                          THCudaTensor *gradInput_, THCudaTensor *gradWeight_,
                                          THCudaTensor *gradBias_, THCudaTensor *weight_,
                                          THCudaTensor *runningMean_, THCudaTensor *runningVar_,
                                          THCudaTensor *saveMean_, THCudaTensor *saveStd_, bool train, double scale,
                                          double eps) {
  THNN_ENTER
  bnBackward(state, input_, gradOutput_, gradInput_, gradWeight_, gradBias_, weight_, nullptr, runningMean_, runningVar_,
             saveMean_, saveStd_, train, scale, eps, 0);
  THNN_LEAVE
}

// No counterpart in the reference's C ABI: BatchNormalization followed by Threshold(0, 0) - the conv -> BN -> ReLU
// step of a residual or depthwise block - in one pass over the tensor (include/THCUNN_fused.h).
void THNN_CudaBatchNormalizationReLU_updateOutput(THCState *state, THCudaTensor *input_, THCudaTensor *output_,
                                                  THCudaTensor *weight_, THCudaTensor *bias_,
                                                  THCudaTensor *runningMean_, THCudaTensor *runningVar_,
                                                  THCudaTensor *saveMean_, THCudaTensor *saveStd_, bool train,
                                                  double momentum, double eps) {
  THNN_ENTER
  bnUpdateOutput(state, input_, output_, weight_, bias_, runningMean_, runningVar_, saveMean_, saveStd_, train, momentum,
                 eps, 1);
  THNN_LEAVE
}

void THNN_CudaBatchNormalizationReLU_backward(THCState *state, THCudaTensor *input_, THCudaTensor *gradOutput_,
                                              THCudaTensor *gradInput_, THCudaTensor *gradWeight_,
                                              THCudaTensor *gradBias_, THCudaTensor *weight_, THCudaTensor *bias_,
                                              THCudaTensor *runningMean_, THCudaTensor *runningVar_,
                                              THCudaTensor *saveMean_, THCudaTensor *saveStd_, bool train,
                                              double scale, double eps) {
  THNN_ENTER
  bnBackward(state, input_, gradOutput_, gradInput_, gradWeight_, gradBias_, weight_, bias_, runningMean_, runningVar_,
             saveMean_, saveStd_, train, scale, eps, 1);
  THNN_LEAVE
}

}  // extern "C"
