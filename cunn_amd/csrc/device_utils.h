// Device-side building blocks shared by the gfx950 kernels: 64-lane wavefront
// reductions, the XCD-aware block remap and the row-tile loaders that stage a
// band of rows of one NCHW plane into LDS.
#pragma once

#include <hip/hip_runtime.h>

namespace dev {

constexpr int kWave = 64;     // CDNA wavefront width
constexpr int kXcds = 8;      // MI355X: 8 XCDs, each with its own L2
constexpr int kBlock = 256;   // 4 wavefronts per workgroup

// v + (v of the lane selected by the DPP control), computed on the VALU: no LDS
// crossbar traffic, unlike ds_bpermute-based shuffles.
template <int CTRL>
__device__ __forceinline__ float dppAdd(float v) {
  return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

// Sum over the 64 lanes of a wavefront, returned in every lane (wave-uniform).
// Four DPP steps fold each row of 16 lanes (quad xor 1, quad xor 2, half-row
// mirror, row mirror), then the four row sums are read as scalars and added.
__device__ __forceinline__ float waveSum(float v) {
  v = dppAdd<0xB1>(v);   // quad_perm [1,0,3,2]
  v = dppAdd<0x4E>(v);   // quad_perm [2,3,0,1]
  v = dppAdd<0x141>(v);  // row_half_mirror
  v = dppAdd<0x140>(v);  // row_mirror
  const int b = __builtin_bit_cast(int, v);
  float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0));
  float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
  float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32));
  float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
  return (r0 + r1) + (r2 + r3);
}

// Sum over each aligned group of `lanes` lanes (4, 8, 16, 32 or 64; wave-uniform), returned in
// every lane of the group; the same DPP steps as waveSum, stopped where the group is complete.
__device__ __forceinline__ float groupSum(float v, int lanes) {
  v = dppAdd<0xB1>(v);
  v = dppAdd<0x4E>(v);
  if (lanes >= 8) v = dppAdd<0x141>(v);
  if (lanes >= 16) v = dppAdd<0x140>(v);
  if (lanes >= 32) {
    const int b = __builtin_bit_cast(int, v);
    const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0));
    const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
    const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32));
    const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
    v = lanes >= 64 ? (r0 + r1) + (r2 + r3) : ((threadIdx.x & 32) ? r2 + r3 : r0 + r1);
  }
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

// Division of a non-negative int by a positive runtime divisor d through its
// reciprocal magic = floor(2^32 / d) + 1 (magicOf): exact while i * d < 2^32, which
// holds for every in-tile index here. A few integer instructions instead of the
// ~25 of a generic 32-bit division. d == 1 has no 32-bit magic (it would be 2^32)
// and is encoded as 0.
__host__ __device__ __forceinline__ unsigned magicOf(int d) { return d == 1 ? 0u : 0xFFFFFFFFu / (unsigned)d + 1u; }
__device__ __forceinline__ int fastDiv(int i, unsigned magic) {
  return magic ? (int)__umulhi((unsigned)i, magic) : i;
}

// Buffer-addressed 16-byte accesses: the base lives in a scalar resource
// descriptor, an access carries a 32-bit byte offset, and an offset at or beyond
// the descriptor's size reads as 0 - out-of-image elements need no branch.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
constexpr int kBufOob = 0x7fffffff;
__device__ __forceinline__ __amdgpu_buffer_rsrc_t makeRsrc(const void *base, long bytes) {
  return __builtin_amdgcn_make_buffer_rsrc((void *)base, 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ float4 bufLoad4(__amdgpu_buffer_rsrc_t r, int byteOff) {
  u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(r, byteOff, 0, 0);
  return make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
}
// the same with the non-temporal hint: for the last reader of a tensor
__device__ __forceinline__ float4 bufLoadStream4(__amdgpu_buffer_rsrc_t r, int byteOff) {
  u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(r, byteOff, 0, 2);
  return make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
}
__device__ __forceinline__ void bufStore4(__amdgpu_buffer_rsrc_t r, int byteOff, float4 f) {
  u32x4 v = {__float_as_uint(f.x), __float_as_uint(f.y), __float_as_uint(f.z), __float_as_uint(f.w)};
  __builtin_amdgcn_raw_buffer_store_b128(v, r, byteOff, 0, 0);
}

// the same as a streaming store (see storeStream4): cache-policy bits nt (2) and sc1 (16). Of the eight
// combinations of a store's policy bits, "sc1 nt" measured fastest on a 1:4 read:write stream: 6.79 TB/s
// against 6.76 (nt alone) and 5.2 (plain) while the buffers a program cycles through stay under about
// 1.3 GB, 5.95 against 5.75 and 5.2 TB/s beyond.
__device__ __forceinline__ void bufStoreStream4(__amdgpu_buffer_rsrc_t r, int byteOff, float4 f) {
  u32x4 v = {__float_as_uint(f.x), __float_as_uint(f.y), __float_as_uint(f.z), __float_as_uint(f.w)};
  __builtin_amdgcn_raw_buffer_store_b128(v, r, byteOff, 0, 2 | 16);
}

// two 64-bit values as one streaming 16-byte store
__device__ __forceinline__ void bufStoreStream2L(__amdgpu_buffer_rsrc_t r, int byteOff, long a, long b) {
  u32x4 v = {(unsigned)a, (unsigned)((unsigned long)a >> 32), (unsigned)b, (unsigned)((unsigned long)b >> 32)};
  __builtin_amdgcn_raw_buffer_store_b128(v, r, byteOff, 0, 2 | 16);
}

__device__ __forceinline__ int ceilDivPos(int a, int b) {  // ceil(a / b) for b > 0, any sign of a
  return (a >= 0) ? (a + b - 1) / b : -((-a) / b);
}

// 16-byte store of data that is not read again soon (an output tensor written once): the
// non-temporal hint keeps it from displacing tensors that the next kernels re-read from the
// last-level cache. (The builtin sets the nt bit only; bufStoreStream4 sets sc1 as well, which measured a
// little faster still - it takes a wave-uniform base, so kernels whose stores have one use that form.)
typedef float f32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void storeStream4(float *p, float4 v) {
  f32x4 q = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(q, reinterpret_cast<f32x4 *>(p));
}

typedef long i64x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void storeStream2(long *p, long a, long b) {
  i64x2 q = {a, b};
  __builtin_nontemporal_store(q, reinterpret_cast<i64x2 *>(p));
}

// Number of independent 16-byte (or 4-byte) global loads a lane keeps in flight
// before it starts storing to LDS: the loads of one batch are issued back to
// back, so a band costs ceil(per-lane loads / kLoadBatch) memory round trips
// instead of one round trip per load.
constexpr int kLoadBatch = 4;

// Copies rows [r0, r0 + nRows) of a (H x W) plane into LDS at
//   dst[r * pitch + padL + col],  r = 0 .. nRows-1, col = 0 .. W-1
// Rows outside the plane are filled with `fill` (0 for sums, -FLT_MAX for max
// scans) and so are the padL cells in front of every row plus padL cells after
// the last one, so that a reader may run up to padL columns off either side of
// a row and see the fill value (the right overhang of row r is the left pad of
// row r+1). VEC: W % 4 == 0, pitch % 4 == 0,
// padL % 4 == 0 and a 16-byte aligned plane, which makes every transfer a
// 16-byte global load and a 16-byte LDS store.
template <bool VEC>
__device__ __forceinline__ void loadRowsPadded(float *__restrict__ dst, const float *__restrict__ plane,
                                               int H, int W, int r0, int nRows, int pitch, int padL,
                                               float fill = 0.f) {
  const int tid = threadIdx.x, nt = blockDim.x;
  if (VEC) {
    const int W4 = W >> 2;
    const int total = nRows * W4;
    const unsigned magic = magicOf(W4);
    const __amdgpu_buffer_rsrc_t rs = makeRsrc(plane, (long)H * W * 4);
    for (int base = 0; base < total; base += kLoadBatch * nt) {
      float4 v[kLoadBatch];
      int off[kLoadBatch];
#pragma unroll
      for (int u = 0; u < kLoadBatch; ++u) {
        const int i = base + u * nt + tid;
        const int r = fastDiv(i, magic), c4 = i - r * W4;
        const int gr = r0 + r;
        const bool ok = i < total && (unsigned)gr < (unsigned)H;
        off[u] = (i < total) ? r * pitch + padL + (c4 << 2) : -1;
        v[u] = bufLoad4(rs, ok ? (gr * W + (c4 << 2)) * 4 : kBufOob);
        if (fill != 0.f && !ok) v[u] = make_float4(fill, fill, fill, fill);
      }
#pragma unroll
      for (int u = 0; u < kLoadBatch; ++u)
        if (off[u] >= 0) *reinterpret_cast<float4 *>(dst + off[u]) = v[u];
    }
  } else {
    const int total = nRows * W;
    for (int base = 0; base < total; base += kLoadBatch * nt) {
      float v[kLoadBatch];
      int off[kLoadBatch];
#pragma unroll
      for (int u = 0; u < kLoadBatch; ++u) {
        int i = base + u * nt + tid;
        int r = i / W, c = i - r * W;
        int gr = r0 + r;
        off[u] = (i < total) ? r * pitch + padL + c : -1;
        v[u] = (i < total && gr >= 0 && gr < H) ? plane[(long)gr * W + c] : fill;
      }
#pragma unroll
      for (int u = 0; u < kLoadBatch; ++u)
        if (off[u] >= 0) dst[off[u]] = v[u];
    }
  }
  if (padL > 0) {
    const int totalPad = (nRows + 1) * padL;
    for (int i = tid; i < totalPad; i += nt) {
      int r = i / padL, k = i - r * padL;
      dst[r * pitch + k] = fill;
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
    const __amdgpu_buffer_rsrc_t rs = makeRsrc(src, (long)count * 4);
    for (int base = 0; base < n4; base += kLoadBatch * nt) {
      float4 v[kLoadBatch];
#pragma unroll
      for (int u = 0; u < kLoadBatch; ++u) v[u] = bufLoad4(rs, (base + u * nt + tid) * 16);  // past the end reads 0
#pragma unroll
      for (int u = 0; u < kLoadBatch; ++u) {
        int i = base + u * nt + tid;
        if (i < n4) reinterpret_cast<float4 *>(dst)[i] = v[u];
      }
    }
  } else {
    for (int base = 0; base < count; base += kLoadBatch * nt) {
      T v[kLoadBatch];
#pragma unroll
      for (int u = 0; u < kLoadBatch; ++u) {
        int i = base + u * nt + tid;
        v[u] = T(0);
        if (i < count) v[u] = src[i];
      }
#pragma unroll
      for (int u = 0; u < kLoadBatch; ++u) {
        int i = base + u * nt + tid;
        if (i < count) dst[i] = v[u];
      }
    }
  }
}

// De-interleaving variant for stride-2 consumers: row r of the band is stored as
//   dst[r * pitch + 4 + m]           = x[r][2m]      (even columns)
//   dst[r * pitch + oddOff + m]      = x[r][2m + 1]  (odd columns), oddOff = W/2 + 8
// with 4 fill cells in front of each half and 4 after the last row, so that a
// lane reading 4 consecutive even (or odd) columns issues one 16-byte LDS read at
// unit stride across lanes instead of a 32-byte-strided one (which maps 64 lanes
// onto 8 banks). Requires W % 8 == 0, pitch % 4 == 0, 16-byte aligned plane.
__device__ __forceinline__ void loadRowsSplit(float *__restrict__ dst, const float *__restrict__ plane, int H, int W,
                                              int r0, int nRows, int pitch, float fill = 0.f) {
  const int tid = threadIdx.x, nt = blockDim.x;
  const int W4 = W >> 2;
  const int oddOff = (W >> 1) + 8;
  const int total = nRows * W4;
  const unsigned magic = magicOf(W4);
  const __amdgpu_buffer_rsrc_t rs = makeRsrc(plane, (long)H * W * 4);
  for (int base = 0; base < total; base += kLoadBatch * nt) {
    float4 v[kLoadBatch];
    int off[kLoadBatch];
#pragma unroll
    for (int u = 0; u < kLoadBatch; ++u) {
      const int i = base + u * nt + tid;
      const int r = fastDiv(i, magic), c4 = i - r * W4;
      const int gr = r0 + r;
      const bool ok = i < total && (unsigned)gr < (unsigned)H;
      off[u] = (i < total) ? r * pitch + 4 + (c4 << 1) : -1;
      v[u] = bufLoad4(rs, ok ? (gr * W + (c4 << 2)) * 4 : kBufOob);
      if (fill != 0.f && !ok) v[u] = make_float4(fill, fill, fill, fill);
    }
#pragma unroll
    for (int u = 0; u < kLoadBatch; ++u)
      if (off[u] >= 0) {
        *reinterpret_cast<float2 *>(dst + off[u]) = make_float2(v[u].x, v[u].z);
        *reinterpret_cast<float2 *>(dst + off[u] + oddOff - 4) = make_float2(v[u].y, v[u].w);
      }
  }
  // zero cells: [0,4) and [4 + W/2, 8 + W/2) of every row, [0,4) after the last row
  const int totalPad = nRows * 8 + 4;
  for (int i = tid; i < totalPad; i += nt) {
    int r = i >> 3, k = i & 7;
    dst[r * pitch + (k < 4 ? k : (W >> 1) + k)] = fill;
  }
}

// Reads N consecutive floats starting at p into w[], using the widest LDS reads
// the known alignment allows. OFF = element offset of p from an ALIGN-element
// aligned address (ALIGN is 4, 2 or 1), both compile-time.
template <int J, int N, int OFF, int ALIGN>
__device__ __forceinline__ void readWindow(const float *__restrict__ p, float (&w)[N]) {
  if constexpr (J < N) {
    if constexpr (ALIGN >= 4 && ((OFF + J) % 4 == 0) && (J + 4 <= N)) {
      float4 v = *reinterpret_cast<const float4 *>(p + J);
      w[J] = v.x, w[J + 1] = v.y, w[J + 2] = v.z, w[J + 3] = v.w;
      readWindow<J + 4, N, OFF, ALIGN>(p, w);
    } else if constexpr (ALIGN >= 2 && ((OFF + J) % 2 == 0) && (J + 2 <= N)) {
      float2 v = *reinterpret_cast<const float2 *>(p + J);
      w[J] = v.x, w[J + 1] = v.y;
      readWindow<J + 2, N, OFF, ALIGN>(p, w);
    } else {
      w[J] = p[J];
      readWindow<J + 1, N, OFF, ALIGN>(p, w);
    }
  }
}

}  // namespace dev
