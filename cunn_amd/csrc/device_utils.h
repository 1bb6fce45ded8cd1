// Device-side building blocks shared by the gfx950 kernels: 64-lane wavefront
// reductions, the XCD-aware block remap and the row-tile loaders that stage a
// band of rows of one NCHW plane into LDS.
#pragma once

#include <hip/hip_runtime.h>

namespace dev {

constexpr int kWave = 64;     // CDNA wavefront width
constexpr int kXcds = 8;      // MI355X: 8 XCDs, each with its own L2
constexpr int kBlock = 256;   // 4 wavefronts per workgroup

__device__ __forceinline__ float waveSum(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}

// Workgroups are handed to the XCDs round-robin (block b runs on XCD b % 8).
// Remapping so that each XCD works on one contiguous range of logical tiles
// keeps the tiles that share halo rows (and the planes that are neighbours in
// memory) behind the same L2.
__device__ __forceinline__ int xcdRemap(int bid, int nblk) {
  int q = nblk / kXcds, r = nblk % kXcds;
  int xcd = bid % kXcds, idx = bid / kXcds;
  return xcd * q + (xcd < r ? xcd : r) + idx;
}

__device__ __forceinline__ int ceilDivPos(int a, int b) {  // ceil(a / b) for b > 0, any sign of a
  return (a >= 0) ? (a + b - 1) / b : -((-a) / b);
}

// Copies rows [r0, r0 + nRows) of a (H x W) plane into LDS at
//   dst[r * pitch + padL + col],  r = 0 .. nRows-1, col = 0 .. W-1
// Rows outside the plane are zero-filled and so are the padL cells in front of
// every row plus padL cells after the last one, so that a reader may run up to
// padL columns off either side of a row and see zeros (the right overhang of
// row r is the left pad of row r+1). VEC: W % 4 == 0, pitch % 4 == 0,
// padL % 4 == 0 and a 16-byte aligned plane, which makes every transfer a
// 16-byte global load and a 16-byte LDS store.
template <bool VEC>
__device__ __forceinline__ void loadRowsPadded(float *__restrict__ dst, const float *__restrict__ plane,
                                               int H, int W, int r0, int nRows, int pitch, int padL) {
  const int tid = threadIdx.x, nt = blockDim.x;
  if (VEC) {
    const int W4 = W >> 2;
    const int total = nRows * W4;
    for (int i = tid; i < total; i += nt) {
      int r = i / W4, c4 = i - r * W4;
      int gr = r0 + r;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (gr >= 0 && gr < H) v = reinterpret_cast<const float4 *>(plane + (long)gr * W)[c4];
      *reinterpret_cast<float4 *>(dst + r * pitch + padL + (c4 << 2)) = v;
    }
  } else {
    const int total = nRows * W;
    for (int i = tid; i < total; i += nt) {
      int r = i / W, c = i - r * W;
      int gr = r0 + r;
      dst[r * pitch + padL + c] = (gr >= 0 && gr < H) ? plane[(long)gr * W + c] : 0.f;
    }
  }
  if (padL > 0) {
    const int totalPad = (nRows + 1) * padL;
    for (int i = tid; i < totalPad; i += nt) {
      int r = i / padL, k = i - r * padL;
      dst[r * pitch + k] = 0.f;
    }
  }
}

// Copies the contiguous run of `count` elements starting at src into LDS.
// VEC: src 16-byte aligned and count % 4 == 0.
template <bool VEC, typename T>
__device__ __forceinline__ void loadFlat(T *__restrict__ dst, const T *__restrict__ src, int count) {
  const int tid = threadIdx.x, nt = blockDim.x;
  if (VEC && sizeof(T) == 4) {
    const int n4 = count >> 2;
    for (int i = tid; i < n4; i += nt)
      reinterpret_cast<float4 *>(dst)[i] = reinterpret_cast<const float4 *>(src)[i];
  } else {
    for (int i = tid; i < count; i += nt) dst[i] = src[i];
  }
}

}  // namespace dev
