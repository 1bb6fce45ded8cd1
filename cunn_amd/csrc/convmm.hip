// SpatialConvolutionMM for gfx950: im2col/col2im + fp32 MFMA GEMM.
//
// The reference loops over the batch and per image launches im2col, an SGEMM
// and (for the bias) a k=1 SGEMM, writing a (Cin*kH*kW) x (oH*oW) column
// buffer to memory and reading it back
// (lib/THCUNN/generic/SpatialConvolutionMM.cu:129-194, 272-308, 396-470).
// Here each entry point is one batched GEMM over the whole mini-batch built on
// v_mfma_f32_32x32x2_f32 with LDS-staged 128x128x16 tiles:
//   updateOutput       C[o][n,l]  = bias[o] + sum_k W[o][k] * col[k][n,l]
//                      col is never stored: the B-tile loader gathers it from
//                      the NCHW input on the fly (implicit im2col, zero padded)
//   accGradParameters  gW[o][k]  += scale * sum_{n,l} gy[n][o][l] * col[k][n,l]
//                      split over groups of images; partial products go to the
//                      caller's `columns` scratch and are folded in a fixed
//                      order (deterministic, no atomics); gradBias is a
//                      separate 64-lane shuffle reduction
//   updateGradInput    gradCol[k][n,l] = sum_o W[o][k] * gy[n][o][l] for a group
//                      of images into `gradColumns`, then the col2im gather of
//                      lib/THCUNN/im2col.h:63-102 over the group.
#include <atomic>
#include <cstring>
#include <map>
#include <mutex>
#include <numeric>
#include <type_traits>

#include "device_utils.h"
#include "launch_utils.h"
#include "thc_internal.h"

using namespace thc;

namespace {

typedef float float16v __attribute__((ext_vector_type(16)));

constexpr int BM = 128, BN = 128, BK = 16;
constexpr int PITCH = 132;  // 8 * PITCH % 64 == 32: the two k-halves of a transposing store hit disjoint banks

struct ConvGeom {
  int N, Cin, Cout, H, W, oH, oW;
  int kH, kW, dH, dW, padH, padW;
  int dilH, dilW;  // tap spacing (1 = ordinary convolution)
  int K;  // Cin * kH * kW
  int L;  // oH * oW
};

enum GemmMode { kForward = 0, kGradCol = 1, kGradWeight = 2 };

struct GemmArgs {
  const float *a;   // forward: W (Cout x K); gradCol: W; gradWeight: gy
  const float *b;   // forward: x; gradCol: gy; gradWeight: x
  float *c;         // forward: out; gradCol: gradCol of the group; gradWeight: partials
  const float *bias;
  int M, Ncols, R;  // GEMM extents: C is M x Ncols, reduction length R (per split)
  int n0;           // first image of the group (gradCol) / reduction tiles (of BK positions) per split (gradWeight)
  int nImages;      // images covered by this launch
  int mTiles;
  bool vecA;        // A rows may be fetched with 16-byte loads (extent % 4 == 0, aligned base)
};

// Decomposition of a flat output position lg = n*L + oh*oW + ow.
struct Pos {
  int n, oh, ow;
};

// ---- the MFMA core: one 128x128 tile, 4 waves of 64x64 -----------------------
__device__ __forceinline__ void mfmaTile(const float (*As)[PITCH], const float (*Bs)[PITCH], float16v (&acc)[2][2],
                                         int wm, int wn, int lane) {
  const int kk = lane >> 5, idx = lane & 31;
#pragma unroll
  for (int k = 0; k < BK; k += 2) {
    float a0 = As[k + kk][wm * 64 + idx], a1 = As[k + kk][wm * 64 + 32 + idx];
    float b0 = Bs[k + kk][wn * 64 + idx], b1 = Bs[k + kk][wn * 64 + 32 + idx];
    acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
    acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
    acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
    acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
  }
}

// Element (r, col) of the implicit im2col matrix for image base xb:
// x[c][oh*dH - padH + kh][ow*dW - padW + kw] or 0 (lib/THCUNN/im2col.h:24-36).
__device__ __forceinline__ float gatherCol(const float *__restrict__ xb, const ConvGeom &g, int c, int kh, int kw,
                                           int ih0, int iw0) {
  int ih = ih0 + kh * g.dilH, iw = iw0 + kw * g.dilW;
  return (ih >= 0 && ih < g.H && iw >= 0 && iw < g.W) ? xb[((long)c * g.H + ih) * g.W + iw] : 0.f;
}

template <int MODE>
__global__ void __launch_bounds__(dev::kBlock)
convGemmKernel(GemmArgs p, ConvGeom g) {
  __shared__ float As[2][BK][PITCH];
  __shared__ float Bs[2][BK][PITCH];
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int mTile = blockIdx.x % p.mTiles, nTile = blockIdx.x / p.mTiles;
  const int m0 = mTile * BM, j0 = nTile * BN;
  const int split = blockIdx.y;
  const int KK = g.kH * g.kW;

  float16v acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  float ra[8], rb[8];

  // ---- per-thread loader state ------------------------------------------------
  // "col-major" mapping: one tile column, 8 consecutive reduction rows
  const int colA = t & 127, rowA8 = (t >> 7) * 8;
  // "row-major" mapping: one tile row/column pair (t >> 1), 8 consecutive reduction elements
  const int rowT = t >> 1, redT8 = (t & 1) * 8;

  // forward / gradCol: B column = output position lg (fixed per thread)
  Pos bp = {0, 0, 0};
  bool bValid = false;
  const float *bBase = nullptr;
  int ih0 = 0, iw0 = 0;
  if (MODE == kForward || MODE == kGradCol) {
    long lg = (long)j0 + colA;
    bValid = lg < (long)p.Ncols;
    if (bValid) {
      bp.n = (int)(lg / g.L);
      int l = (int)(lg - (long)bp.n * g.L);
      bp.oh = l / g.oW;
      bp.ow = l - bp.oh * g.oW;
      if (MODE == kForward) {
        bBase = p.b + (long)(p.n0 + bp.n) * g.Cin * g.H * g.W;
        ih0 = bp.oh * g.dH - g.padH;
        iw0 = bp.ow * g.dW - g.padW;
      } else {
        bBase = p.b + (long)(p.n0 + bp.n) * g.Cout * g.L + l;  // + o * L
      }
    }
  }
  // gradWeight: B column = k index (c, kh, kw), 16-lane groups walk consecutive positions
  const int gwR = t & 15, gwJ = t >> 4;  // reduction row within the tile, first of 8 columns (stride 16)
  // gradWeight: split `split` reduces positions [rBegin, rEnd) of the N*L positions of the batch
  const long rBegin = (MODE == kGradWeight) ? (long)split * p.n0 * BK : 0;
  const long rEnd = (MODE == kGradWeight) ? min(rBegin + (long)p.n0 * BK, (long)p.nImages * g.L) : (long)p.R;
  const int nkt = (int)((rEnd - rBegin + BK - 1) / BK);

  auto loadTiles = [&](int kt) {
    const int r0 = kt * BK;
    if (MODE == kForward) {
      // A: W[o][k], k contiguous
      {
        int o = m0 + rowT, k = r0 + redT8;
        const float *src = p.a + (long)o * g.K + k;
        bool rowOk = o < p.M;
        if (p.vecA && rowOk && k + 8 <= g.K) {
          float4 v0 = reinterpret_cast<const float4 *>(src)[0], v1 = reinterpret_cast<const float4 *>(src)[1];
          ra[0] = v0.x, ra[1] = v0.y, ra[2] = v0.z, ra[3] = v0.w;
          ra[4] = v1.x, ra[5] = v1.y, ra[6] = v1.z, ra[7] = v1.w;
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i) ra[i] = (rowOk && k + i < g.K) ? src[i] : 0.f;
        }
      }
      // B: implicit im2col, rows k = r0 + rowA8 + i
      {
        int k = r0 + rowA8;
        int c = k / KK, rem = k - c * KK;
        int kh = rem / g.kW, kw = rem - kh * g.kW;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          rb[i] = (bValid && k + i < g.K) ? gatherCol(bBase, g, c, kh, kw, ih0, iw0) : 0.f;
          if (++kw == g.kW) {
            kw = 0;
            if (++kh == g.kH) {
              kh = 0;
              ++c;
            }
          }
        }
      }
    } else if (MODE == kGradCol) {
      // A[m = k][r = o] = W[o][k]: contiguous along m
      {
        int k = m0 + colA;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          int o = r0 + rowA8 + i;
          ra[i] = (k < p.M && o < p.R) ? p.a[(long)o * g.K + k] : 0.f;
        }
      }
      // B[r = o][lg] = gy[n][o][l]
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        int o = r0 + rowA8 + i;
        rb[i] = (bValid && o < p.R) ? bBase[(long)o * g.L] : 0.f;
      }
    } else {
      // gradWeight. A[m = o][r = (n,l)] = gy[n][o][l]: contiguous along r inside an image
      {
        int o = m0 + rowT;
        long r = rBegin + r0 + redT8;
        bool rowOk = o < p.M;
        int n = (int)(r / g.L);
        int l = (int)(r - (long)n * g.L);
        if (p.vecA && rowOk && r + 8 <= rEnd) {
          // with L % 4 == 0 a group of 4 never straddles an image
          const float *s0 = p.a + ((long)n * g.Cout + o) * g.L + l;
          float4 v0 = *reinterpret_cast<const float4 *>(s0);
          int l2 = l + 4, n2 = n;
          if (l2 >= g.L) {
            l2 -= g.L;
            ++n2;
          }
          const float *s1 = p.a + ((long)n2 * g.Cout + o) * g.L + l2;
          float4 v1 = *reinterpret_cast<const float4 *>(s1);
          ra[0] = v0.x, ra[1] = v0.y, ra[2] = v0.z, ra[3] = v0.w;
          ra[4] = v1.x, ra[5] = v1.y, ra[6] = v1.z, ra[7] = v1.w;
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            ra[i] = (rowOk && r + i < rEnd) ? p.a[((long)n * g.Cout + o) * g.L + l] : 0.f;
            if (++l == g.L) {
              l = 0;
              ++n;
            }
          }
        }
      }
      // B[r = (n,l)][j = k] = col[k][n,l]; lanes 0..15 of a group walk consecutive l
      {
        long r = rBegin + r0 + gwR;
        bool rOk = r < rEnd;
        int n = rOk ? (int)(r / g.L) : 0;
        int l = rOk ? (int)(r - (long)n * g.L) : 0;
        int oh = l / g.oW, ow = l - oh * g.oW;
        const float *xb = p.b + (long)n * g.Cin * g.H * g.W;
        int ih0g = oh * g.dH - g.padH, iw0g = ow * g.dW - g.padW;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          int k = j0 + gwJ + 16 * i;
          float v = 0.f;
          if (rOk && k < p.Ncols) {
            int c = k / KK, rem = k - c * KK;
            int kh = rem / g.kW, kw = rem - kh * g.kW;
            v = gatherCol(xb, g, c, kh, kw, ih0g, iw0g);
          }
          rb[i] = v;
        }
      }
    }
  };

  auto storeTiles = [&](int buf) {
    if (MODE == kForward) {
#pragma unroll
      for (int i = 0; i < 8; ++i) As[buf][redT8 + i][rowT] = ra[i];
#pragma unroll
      for (int i = 0; i < 8; ++i) Bs[buf][rowA8 + i][colA] = rb[i];
    } else if (MODE == kGradCol) {
#pragma unroll
      for (int i = 0; i < 8; ++i) As[buf][rowA8 + i][colA] = ra[i];
#pragma unroll
      for (int i = 0; i < 8; ++i) Bs[buf][rowA8 + i][colA] = rb[i];
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) As[buf][redT8 + i][rowT] = ra[i];
#pragma unroll
      for (int i = 0; i < 8; ++i) Bs[buf][gwR][gwJ + 16 * i] = rb[i];
    }
  };

  if (nkt > 0) {
    loadTiles(0);
    storeTiles(0);
  }
  __syncthreads();
  for (int kt = 0; kt < nkt; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < nkt) loadTiles(kt + 1);
    mfmaTile(As[buf], Bs[buf], acc, wm, wn, lane);
    if (kt + 1 < nkt) storeTiles(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue ----------------------------------------------------------------
  // 32x32 accumulator layout: lane holds column (lane & 31) and rows
  // 8*(v/4) + 4*(lane/32) + v%4, v = 0..15.
  const int colInTile = lane & 31, rowHalf = (lane >> 5) * 4;
#pragma unroll
  for (int tj = 0; tj < 2; ++tj) {
    const long col = (long)j0 + wn * 64 + tj * 32 + colInTile;
    if (col >= p.Ncols) continue;
    long cOff;  // offset of (row 0, col) and row stride
    long rowStride;
    if (MODE == kForward) {
      int n = (int)(col / g.L);
      int l = (int)(col - (long)n * g.L);
      cOff = (long)(p.n0 + n) * g.Cout * g.L + l;
      rowStride = g.L;
    } else if (MODE == kGradCol) {
      int n = (int)(col / g.L);
      int l = (int)(col - (long)n * g.L);
      cOff = (long)n * g.K * g.L + l;
      rowStride = g.L;
    } else {
      cOff = (long)split * p.M * p.Ncols + col;
      rowStride = p.Ncols;
    }
#pragma unroll
    for (int ti = 0; ti < 2; ++ti) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        int row = m0 + wm * 64 + ti * 32 + 8 * (v >> 2) + rowHalf + (v & 3);
        if (row < p.M) {
          float val = acc[ti][tj][v];
          if (MODE == kForward && p.bias) val += p.bias[row];
          p.c[cOff + (long)row * rowStride] = val;
        }
      }
    }
  }
}

// ---- forward implicit GEMM, second generation ---------------------------------
// Same 128x128x16 tiling as convGemmKernel<kForward>, with the two costs that
// kept the MFMA pipe at ~40 % removed:
//  * operands sit in LDS as float4 groups of 4 consecutive k
//    (As[kg][row], Bs[kg][col]); a lane fetches the operands of four MFMAs with
//    one ds_read_b128 and the loaders store with ds_write_b128. Lane group
//    g = lane / 32 of super-step s consumes k-group 2s + g, i.e. MFMA j contracts
//    k = 8s + j (g = 0) with k = 8s + 4 + j (g = 1) - any pairing is valid as long
//    as A and B agree.
//  * the im2col gather is a buffer load: the image base is a scalar resource,
//    the lane's position (n, oh, ow) is a fixed 32-bit byte offset, and the tap
//    (c, kh, kw) of each k is wave-uniform, so it lives in scalar registers.
//    A tap outside the image gets an out-of-range offset, for which the buffer
//    unit returns 0 - the zero padding costs no branch.
constexpr int FPITCH = BM + 8;  // float4 per k-group row: +8 keeps the 2 k-groups a lane pair writes in disjoint banks

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

struct FwdArgs {
  const float *w;     // (M x K) row-major
  const float *x;     // images n0 .. n0 + nImages - 1 of (N, Cin, H, W)
  float *out;         // element (n, row, oh, ow) at out[n * outImg + row * outRow + oh * outSH + ow * outSW]
  long outImg;        // dense output (nImages, M, oH, oW): M * L, L, oW, 1
  int outRow, outSH, outSW;
  // != 0 (outSW == 2, outSH == 2 * row length): every element is the top-left corner of a 2 x 2 block of out
  // whose other three elements get the bias (or 0) - the gradInput of a 1x1 convolution with stride 2
  int dilate;
  const float *bias;  // M or null
  int M, Ncols;       // Ncols = nImages * L
  int mTiles;
  int bm, bn;         // rows and columns of an output tile: 128 x 128, or 64 x 256 (padded kernel only)
  int xBytes;         // bytes of the nImages input images (< 2^31)
  int wBytes;         // padded kernel: bytes of the weights (< 2^31)
  bool vecA;
  // tail launch: tiles tile0 .. are each reduced by nSplit workgroups over ktPerSplit k-tiles;
  // their 128x128 partial tiles go to `partial` and fwdTailFixupKernel folds them
  int tile0, nSplit, ktPerSplit;
  // padded kernel, one launch for both: workgroups 0 .. full - 1 reduce tiles 0 .. full - 1 over all of K,
  // workgroup full + split * tail + i reduces split `split` of tile tile0 + i (tile0 = full)
  int full, tail;
  float *partial;
  int relu;           // != 0: the stored value is v > 0 ? v : 0 (Threshold(0, 0) applied to the output)
  // padded kernel: the output spans fewer than 2^31 bytes (outBytes) - whole row tiles are then stored with a
  // per-lane column offset and a scalar row offset, no address arithmetic on the vector ALU
  int outBytes;       // 0: not applicable
  unsigned magicL, magicOW;  // reciprocals of L and oW (dev::magicOf), 0: divide
  const int *taps;    // padded kernel: byte offset of tap (c, kh, kw) inside a (zero-padded) image, per k
  int tapStride;      // > 0 (1x1 windows): tap k sits at byte offset k * tapStride, no table is read
};

// Epilogue shared by the forward kernels: a lane holds column (lane & 31) and rows
// 8*(v/4) + 4*(lane/32) + v%4 of each 32x32 accumulator tile. Split workgroups store their
// partial tile, the others add the bias and store to out(n, row, l).
// biasLds: the tile's bias values in LDS (index = row - m0, zeros where there is no bias or row), or null.
// column (n, l) -> (n, oh, ow): through the reciprocals when the launch provides them
__device__ __forceinline__ void splitColumn(const FwdArgs &p, const ConvGeom &g, unsigned col, int &n, int &oh, int &ow) {
  n = p.magicL ? dev::fastDiv((int)col, p.magicL) : (int)(col / (unsigned)g.L);
  const int l = (int)col - n * g.L;
  oh = p.magicOW ? dev::fastDiv(l, p.magicOW) : l / g.oW;
  ow = l - oh * g.oW;
}

// biasDone: the accumulators started from the bias (whole tiles of the padded kernel)
template <int TBN = BN, int TI = 2>
__device__ __forceinline__ void fwdEpilogue(const FwdArgs &p, const ConvGeom &g, const float16v (&acc)[TI][2], int bx,
                                            int by, int m0, int j0, int wm, int wn, int grp, int idx,
                                            const float *biasLds = nullptr, int toPartial = -1, bool biasDone = false) {
  const int rowHalf = grp * 4;
  if (toPartial < 0 ? p.nSplit > 1 : toPartial != 0) {
    float *dst = p.partial + ((long)bx * p.nSplit + by) * (BM * BN);  // both tile shapes hold BM * BN elements
#pragma unroll
    for (int tj = 0; tj < 2; ++tj)
#pragma unroll
      for (int ti = 0; ti < TI; ++ti)
#pragma unroll
        for (int v = 0; v < 16; ++v)
          dst[(wm * 64 + ti * 32 + 8 * (v >> 2) + rowHalf + (v & 3)) * TBN + wn * 64 + tj * 32 + idx] = acc[ti][tj][v];
    return;
  }
  if (biasDone && p.outBytes > 0 && m0 + wm * 64 + TI * 32 <= p.M) {
    // every row of the wave exists: 64 stores of (per-lane column offset, scalar row offset); a column past the
    // batch is an offset out of range
    const __amdgpu_buffer_rsrc_t orr = dev::makeRsrc(p.out, p.outBytes);
    const int rowBase = __builtin_amdgcn_readfirstlane(m0 + wm * 64);
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) {
      const unsigned col = (unsigned)j0 + wn * 64 + tj * 32 + idx;
      int n, oh, ow;
      splitColumn(p, g, min(col, (unsigned)p.Ncols - 1), n, oh, ow);
      const int voff = col < (unsigned)p.Ncols
                           ? (int)(((long)n * p.outImg + (long)oh * p.outSH + ow * p.outSW + (long)rowHalf * p.outRow) * 4)
                           : dev::kBufOob;
#pragma unroll
      for (int ti = 0; ti < TI; ++ti)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          float o = acc[ti][tj][v];
          if (p.relu) o = o > 0.f ? o : 0.f;
          const int soff = (rowBase + ti * 32 + 8 * (v >> 2) + (v & 3)) * p.outRow * 4;
          if (p.dilate) {
            // the element and its right neighbour, then the two below: 8-byte stores, a wave covers whole rows
            const float z = biasLds ? biasLds[wm * 64 + ti * 32 + 8 * (v >> 2) + rowHalf + (v & 3)] : 0.f;
            const u32x2 top = {__float_as_uint(o), __float_as_uint(z)}, bottom = {__float_as_uint(z), __float_as_uint(z)};
            const int below = col < (unsigned)p.Ncols ? voff + (p.outSH >> 1) * 4 : dev::kBufOob;
            __builtin_amdgcn_raw_buffer_store_b64(top, orr, voff, soff, 0);
            __builtin_amdgcn_raw_buffer_store_b64(bottom, orr, below, soff, 0);
          } else {
            __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(o), orr, voff, soff, 0);
          }
        }
    }
    return;
  }
  auto store = [&](auto withBias) {
    constexpr bool BIAS = decltype(withBias)::value;
    // the lane's 32 bias values first: a load between the stores would wait for each store before it
    // (the compiler must assume that out and bias overlap)
    float bv[TI][16];
    if (BIAS) {
#pragma unroll
      for (int ti = 0; ti < TI; ++ti)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          if (biasLds) {  // 4 consecutive rows: one 16-byte LDS read
            const float4 b4 = *reinterpret_cast<const float4 *>(biasLds + wm * 64 + ti * 32 + 8 * q + rowHalf);
            bv[ti][4 * q] = b4.x, bv[ti][4 * q + 1] = b4.y, bv[ti][4 * q + 2] = b4.z, bv[ti][4 * q + 3] = b4.w;
          } else {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const int row = m0 + wm * 64 + ti * 32 + 8 * q + rowHalf + r;
              bv[ti][4 * q + r] = row < p.M ? p.bias[row] : 0.f;
            }
          }
        }
    }
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) {
      const unsigned col = (unsigned)j0 + wn * 64 + tj * 32 + idx;  // Ncols < 2^31
      if (col >= (unsigned)p.Ncols) continue;
      int n, oh, ow;
      splitColumn(p, g, col, n, oh, ow);
      float *dst = p.out + (long)n * p.outImg + (long)oh * p.outSH + ow * p.outSW;
#pragma unroll
      for (int ti = 0; ti < TI; ++ti)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int row = m0 + wm * 64 + ti * 32 + 8 * (v >> 2) + rowHalf + (v & 3);
          float o = BIAS ? acc[ti][tj][v] + bv[ti][v] : acc[ti][tj][v];
          if (p.relu) o = o > 0.f ? o : 0.f;
          if (row < p.M) {
            float *q = dst + (long)row * p.outRow;
            q[0] = o;
            if (p.dilate) {
              const float z = p.bias ? p.bias[row] : 0.f;
              q[1] = z, q[p.outSH >> 1] = z, q[(p.outSH >> 1) + 1] = z;
            }
          }
        }
    }
  };
  if (p.bias && !biasDone)
    store(std::true_type{});
  else
    store(std::false_type{});
}

// taps[k] = ((c*H + kh*dilH)*W + kw*dilW) * 4 for k = (c*kH + kh)*kW + kw; g is the geometry of the padded images.
// Entries beyond Cin*kH*kW (rows padded to a multiple of BK, spare entries) point at the position's own
// first element: valid memory, and their weights are zero or they are never used.
// byte offset of tap k = (c, kh, kw) inside a (zero-bordered) image of g.H x g.W; 0 beyond the last tap
__device__ __forceinline__ int tapOffset(int k, const ConvGeom &g) {
  const int KK = g.kH * g.kW;
  const int c = k / KK, rem = k - c * KK;
  const int kh = rem / g.kW, kw = rem - kh * g.kW;
  return c < g.Cin ? ((c * g.H + kh * g.dilH) * g.W + kw * g.dilW) * 4 : 0;
}

__global__ void __launch_bounds__(dev::kBlock)
buildTapTableKernel(int *taps, int entries, ConvGeom g) {
  for (int k = blockIdx.x * blockDim.x + threadIdx.x; k < entries; k += gridDim.x * blockDim.x) taps[k] = tapOffset(k, g);
}

// wp(rows x Kp) = w(rows x K) with zeros in columns K .. Kp-1
__global__ void __launch_bounds__(dev::kBlock)
padRowsKernel(const float *__restrict__ w, float *__restrict__ wp, int rows, int K, int Kp) {
  const long total = (long)rows * Kp;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    const int k = (int)(i % Kp);
    const long r = i / Kp;
    wp[i] = k < K ? w[r * K + k] : 0.f;
  }
}

// Wf[c][(o, kh', kw')] = W[o][(c, kH-1-kh', kW-1-kw')]: with these weights the stride-1 gradInput is a plain forward
// convolution of gradOutput (padding k-1-pad). The job rides along with the bordered copy of gradOutput (a few more
// workgroups of that launch) instead of costing a launch of its own: both are short, and their latencies would add.
__global__ void flipWeightKernel(const float *__restrict__ w, float *__restrict__ wf, int Cout, int Cin, int kH, int kW);
struct FlipJob {
  const float *w;
  float *wf;
  int Cout, Cin, kH, kW;
};
constexpr int kFlipBlocks = 4096;  // a lane per element up to a million weights: a lane that walks several is bound by their latencies
__device__ __forceinline__ void flipWeights(const FlipJob &f, int block, int blocks) {
  const int KK = f.kH * f.kW;
  const long total = (long)f.Cout * f.Cin * KK;
  for (long i = (long)block * dev::kBlock + threadIdx.x; i < total; i += (long)blocks * dev::kBlock) {
    const int t = (int)(i % KK);
    const long r = i / KK;
    const int o = (int)(r % f.Cout), c = (int)(r / f.Cout);
    f.wf[i] = f.w[((long)o * f.Cin + c) * KK + (KK - 1 - t)];
  }
}

// xp(nc, Hp, Wp) = x(nc, H, W) at row padTop, column padLeft inside zeros. grid = (planes, chunks of a plane);
// VEC: a lane produces 4 consecutive floats of the bordered plane with one 16-byte store
// (plane size a multiple of 4 floats, 16-byte aligned destination).
template <bool VEC>
__global__ void __launch_bounds__(dev::kBlock)
padPlanesKernel(const float *__restrict__ x, float *__restrict__ xp, int H, int W, int padTop, int padLeft, int Hp, int Wp,
                int planes, int *taps, int tapEntries, ConvGeom tg) {
  if ((int)blockIdx.x == planes) {  // one more column of workgroups builds the tap table of the convolution that follows
    for (int k = blockIdx.y * dev::kBlock + threadIdx.x; k < tapEntries; k += gridDim.y * dev::kBlock) taps[k] = tapOffset(k, tg);
    return;
  }
  const unsigned magic = dev::magicOf(Wp);
  const float *src = x + (long)blockIdx.x * H * W;
  float *dst = xp + (long)blockIdx.x * Hp * Wp;
  auto fetch = [&](int j) {
    const int hp = dev::fastDiv(j, magic), wp = j - hp * Wp;
    const int h = hp - padTop, w = wp - padLeft;
    return (((unsigned)h < (unsigned)H) & ((unsigned)w < (unsigned)W)) ? src[h * W + w] : 0.f;
  };
  const int i = blockIdx.y * dev::kBlock + threadIdx.x;
  if (VEC) {
    if (i * 4 < Hp * Wp)
      *reinterpret_cast<float4 *>(dst + i * 4) = make_float4(fetch(i * 4), fetch(i * 4 + 1), fetch(i * 4 + 2), fetch(i * 4 + 3));
  } else {
    if (i < Hp * Wp) dst[i] = fetch(i);
  }
}

// The same for small planes (7x7 ... 28x28 stages: a workgroup per plane would leave most lanes idle): a lane per
// 16-byte group of the whole destination. Workgroups past copyBlocks build the tap table.
// ANY: planes of any size (9x9 = a bordered 7x7 plane): a group may straddle two planes and the last elements of
// the destination may not fill a group.
// The copy of padPlanesFlatKernel for planes of a multiple of 4 floats: workgroups 0 .. copyBlocks - 1 of a launch, a
// lane per 16-byte group of the bordered planes.
__device__ __forceinline__ void padFlatVecBody(const float *__restrict__ x, float *__restrict__ xp, int H, int W, int padTop,
                                               int padLeft, int Hp, int Wp, long total4, int copyBlocks) {
  const int plane4 = (Hp * Wp) >> 2;
  const unsigned magicPlane = dev::magicOf(plane4), magicW = dev::magicOf(Wp);
  for (long i = (long)blockIdx.x * dev::kBlock + threadIdx.x; i < total4; i += (long)copyBlocks * dev::kBlock) {
    const int pl = dev::fastDiv((int)i, magicPlane), j = ((int)i - pl * plane4) * 4;
    const float *src = x + (long)pl * H * W;
    float v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int hp = dev::fastDiv(j + k, magicW), wp = j + k - hp * Wp;
      const int h = hp - padTop, w = wp - padLeft;
      v[k] = (((unsigned)h < (unsigned)H) & ((unsigned)w < (unsigned)W)) ? src[h * W + w] : 0.f;
    }
    reinterpret_cast<float4 *>(xp)[i] = make_float4(v[0], v[1], v[2], v[3]);
  }
}

template <bool ANY>
__global__ void __launch_bounds__(dev::kBlock)
padPlanesFlatKernel(const float *__restrict__ x, float *__restrict__ xp, int H, int W, int padTop, int padLeft, int Hp, int Wp,
                    long total4, int copyBlocks, int *taps, int tapEntries, ConvGeom tg, int tapBlocks, FlipJob flip) {
  if ((int)blockIdx.x >= copyBlocks + tapBlocks) {  // the weights of the convolution that follows, flipped
    flipWeights(flip, blockIdx.x - copyBlocks - tapBlocks, gridDim.x - copyBlocks - tapBlocks);
    return;
  }
  if ((int)blockIdx.x >= copyBlocks) {
    for (int k = (blockIdx.x - copyBlocks) * dev::kBlock + threadIdx.x; k < tapEntries; k += tapBlocks * dev::kBlock)
      taps[k] = tapOffset(k, tg);
    return;
  }
  if (ANY) {
    // total4 counts elements here
    const int plane = Hp * Wp;
    const unsigned magicPlane = dev::magicOf(plane), magicW = dev::magicOf(Wp);
    auto fetch = [&](unsigned e) {
      const int pl = dev::fastDiv((int)e, magicPlane), j = (int)e - pl * plane;
      const int hp = dev::fastDiv(j, magicW), wp = j - hp * Wp;
      const int h = hp - padTop, w = wp - padLeft;
      return (((unsigned)h < (unsigned)H) & ((unsigned)w < (unsigned)W)) ? x[(long)pl * H * W + h * W + w] : 0.f;
    };
    const long groups = (total4 + 3) >> 2;
    for (long i = (long)blockIdx.x * dev::kBlock + threadIdx.x; i < groups; i += (long)copyBlocks * dev::kBlock) {
      const unsigned e = (unsigned)(i * 4);
      if (e + 4 <= (unsigned long)total4) {
        reinterpret_cast<float4 *>(xp)[i] = make_float4(fetch(e), fetch(e + 1), fetch(e + 2), fetch(e + 3));
      } else {
        for (unsigned q = e; q < (unsigned long)total4; ++q) xp[q] = fetch(q);
      }
    }
    return;
  }
  padFlatVecBody(x, xp, H, W, padTop, padLeft, Hp, Wp, total4, copyBlocks);
}

// taps != nullptr: the same launch also builds the tap table (tapEntries entries) of geometry tg
// flip != nullptr: and flips the weights of *flip (the flat kernels take the job along; otherwise a launch of its own)
void launchPadPlanes(hipStream_t s, const float *x, float *xp, long planes, int H, int W, int padTop, int padLeft, int Hp,
                     int Wp, int *taps = nullptr, int tapEntries = 0, const ConvGeom *tg = nullptr, const FlipJob *flip = nullptr) {
  const int plane = Hp * Wp;
  const FlipJob fj = flip ? *flip : FlipJob{};
  const int flipBlocks = flip ? (int)std::min<long>(kFlipBlocks, ((long)fj.Cout * fj.Cin * fj.kH * fj.kW + dev::kBlock - 1) / dev::kBlock) : 0;
  auto flipAlone = [&]() {
    if (!flip) return;
    flipWeightKernel<<<launch::directGrid((long)fj.Cout * fj.Cin * fj.kH * fj.kW, dev::kBlock), dev::kBlock, 0, s>>>(
        fj.w, fj.wf, fj.Cout, fj.Cin, fj.kH, fj.kW);
  };
  if (launch::ceilDiv(plane, dev::kBlock) > 65535) error("SpatialConvolutionMM: image plane too large");
  const unsigned gx = (unsigned)planes + (taps ? 1 : 0);
  const ConvGeom g = tg ? *tg : ConvGeom{};
  const long total4 = planes * (plane / 4);
  // (the reciprocal division of a group index by the groups per plane is exact while index * divisor < 2^32)
  if (plane % 4 == 0 && plane < 4096 && launch::aligned16(xp) && total4 * (plane / 4) < 0xffffffffL) {
    const int copyBlocks = (int)std::min<long>((total4 + dev::kBlock - 1) / dev::kBlock, 16384);
    const int tapBlocks = taps ? std::max(1, std::min(16, launch::ceilDiv(tapEntries, dev::kBlock))) : 0;
    padPlanesFlatKernel<false><<<copyBlocks + tapBlocks + flipBlocks, dev::kBlock, 0, s>>>(
        x, xp, H, W, padTop, padLeft, Hp, Wp, total4, copyBlocks, taps, tapEntries, g, tapBlocks, fj);
  } else if (plane < 1024 && launch::aligned16(xp) && planes * plane * (long)plane < 0xffffffffL) {
    // small planes of any size (a bordered 7x7 or 13x13 plane): a workgroup per plane would leave most of its lanes idle
    const long total = planes * plane;
    const int copyBlocks = (int)std::min<long>(((total + 3) / 4 + dev::kBlock - 1) / dev::kBlock, 16384);
    const int tapBlocks = taps ? std::max(1, std::min(16, launch::ceilDiv(tapEntries, dev::kBlock))) : 0;
    padPlanesFlatKernel<true><<<copyBlocks + tapBlocks + flipBlocks, dev::kBlock, 0, s>>>(
        x, xp, H, W, padTop, padLeft, Hp, Wp, total, copyBlocks, taps, tapEntries, g, tapBlocks, fj);
  } else if (plane % 4 == 0 && launch::aligned16(xp)) {
    flipAlone();
    padPlanesKernel<true><<<dim3(gx, launch::ceilDiv(plane / 4, dev::kBlock)), dev::kBlock, 0, s>>>(
        x, xp, H, W, padTop, padLeft, Hp, Wp, (int)planes, taps, tapEntries, g);
  } else {
    flipAlone();
    padPlanesKernel<false><<<dim3(gx, launch::ceilDiv(plane, dev::kBlock)), dev::kBlock, 0, s>>>(
        x, xp, H, W, padTop, padLeft, Hp, Wp, (int)planes, taps, tapEntries, g);
  }
  THC_HIP_CHECK(hipGetLastError());
}
inline void launchPadPlanes(hipStream_t s, const float *x, float *xp, long planes, int H, int W, int padH, int padW,
                            int *taps = nullptr, int tapEntries = 0, const ConvGeom *tg = nullptr, const FlipJob *flip = nullptr) {
  launchPadPlanes(s, x, xp, planes, H, W, padH, padW, H + 2 * padH, W + 2 * padW, taps, tapEntries, tg, flip);
}

// ---- gradInput by output phase ------------------------------------------------------------------
// gi[h] receives gy[oh] * w[kh] where h + pad = oh * stride + kh * dil. For the positions
// h = ph + stride * i of one phase only the taps with kh * dil = ph + pad (mod stride) contribute,
// they form an arithmetic sequence kh = k0 + a * kStep, and tap a reads gy row i + q0 - a * qStep:
// per phase a stride-1 convolution of gy with a sub-kernel, written to a strided sub-grid of gi.
struct PhaseAxis {
  int n;                // gi positions of the phase along the axis
  int k0, kStep, nk;    // contributing taps
  int q0, qStep;        // gy index of tap a at position i: i + q0 - a * qStep
};
struct Phase {
  PhaseAxis h, w;
  int h0, w0;           // first gi row / column of the phase
  int K, Kp;            // Cout * h.nk * w.nk, rounded up to a positive multiple of BK
  int tapOfs;           // ints from the start of the tap tables
  long wOfs;            // floats from the start of the phase weights
};
constexpr int kMaxPhases = 16;
struct PhaseSet {
  Phase ph[kMaxPhases];
  int count;
};

// Phase weights Wp(Cin x Kp): Wp[c][(o, a, b)] = w[o][c][h.k0 + a*h.kStep][w.k0 + b*w.kStep], zero from K to Kp, and the
// tap table of each phase: entry k = (o, a, b) is the byte offset of gy element (o, q0h - a*qStepH, q0w - b*qStepW) of
// the bordered image, 0 from K on.
// grid = (chunks of a weight row, Cin + 1, phases): blocks with blockIdx.y == Cin write the tap table.
// (bx of gx, by, bz) = the workgroup's position in that grid
__device__ __forceinline__ void phaseSetupBody(const float *__restrict__ w, float *__restrict__ dst, int *__restrict__ taps,
                                               const PhaseSet &set, int Cin, int kH, int kW, int Hp, int Wp, int top, int left,
                                               int bx, int gx, int by, int bz) {
  const Phase &P = set.ph[bz];
  const int tp = P.h.nk * P.w.nk;
  const unsigned magicTp = dev::magicOf(tp), magicNk = dev::magicOf(P.w.nk);
  const int c = by;
  if (c == Cin) {
    const int entries = P.Kp + 2 * BK;
    int *d = taps + P.tapOfs;
    for (int k = bx * dev::kBlock + threadIdx.x; k < entries; k += gx * dev::kBlock) {
      int v = 0;
      if (k < P.K) {
        const int o = dev::fastDiv(k, magicTp), r = k - o * tp;
        const int a = dev::fastDiv(r, magicNk), b = r - a * P.w.nk;
        v = ((o * Hp + top + P.h.q0 - a * P.h.qStep) * Wp + left + P.w.q0 - b * P.w.qStep) * 4;
      }
      d[k] = v;
    }
    return;
  }
  float *d = dst + P.wOfs + (long)c * P.Kp;
  const long oStride = (long)Cin * kH * kW;
  const float *src = w + ((long)c * kH + P.h.k0) * kW + P.w.k0;
  for (int k = bx * dev::kBlock + threadIdx.x; k < P.Kp; k += gx * dev::kBlock) {
    float v = 0.f;
    if (k < P.K) {
      const int o = dev::fastDiv(k, magicTp), r = k - o * tp;
      const int a = dev::fastDiv(r, magicNk), b = r - a * P.w.nk;
      v = src[o * oStride + (a * P.h.kStep) * kW + b * P.w.kStep];
    }
    d[k] = v;
  }
}

__global__ void __launch_bounds__(dev::kBlock)
phaseSetupKernel(const float *__restrict__ w, float *__restrict__ dst, int *__restrict__ taps, PhaseSet set, int Cin, int kH,
                 int kW, int Hp, int Wp, int top, int left) {
  phaseSetupBody(w, dst, taps, set, Cin, kH, kW, Hp, Wp, top, left, blockIdx.x, gridDim.x, blockIdx.y, blockIdx.z);
}

// The bordered copy of gradOutput and the phase set-up in one launch (both are short: as two launches their latencies
// add): workgroups 0 .. copyBlocks - 1 copy (planes of a multiple of 4 floats), the others are the set-up's grid
// (chunks, Cin + 1, phases) laid out flat.
__global__ void __launch_bounds__(dev::kBlock)
padPlanesPhaseSetupKernel(const float *__restrict__ x, float *__restrict__ xp, int H, int W, int Hp, int Wp, int top, int left,
                          long total4, int copyBlocks, const float *__restrict__ w, float *__restrict__ dst,
                          int *__restrict__ taps, PhaseSet set, int Cin, int kH, int kW, int chunks) {
  if ((int)blockIdx.x < copyBlocks) {
    padFlatVecBody(x, xp, H, W, top, left, Hp, Wp, total4, copyBlocks);
    return;
  }
  const int l = blockIdx.x - copyBlocks;
  const int r = l / chunks, bx = l - r * chunks;
  const int bz = r / (Cin + 1), by = r - bz * (Cin + 1);
  phaseSetupBody(w, dst, taps, set, Cin, kH, kW, Hp, Wp, top, left, bx, chunks, by, bz);
}

// Generic forward kernel: any K, any alignment; taps and bounds resolved in the loop.
__global__ void __launch_bounds__(dev::kBlock)
convFwdImplicitKernel(FwdArgs p, ConvGeom g) {
  __shared__ float4 As[2][BK / 4][FPITCH];
  __shared__ float4 Bs[2][BK / 4][FPITCH];
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tileIdx = p.tile0 + blockIdx.x;
  const int mTile = tileIdx % p.mTiles, nTile = tileIdx / p.mTiles;
  const int m0 = mTile * BM, j0 = nTile * BN;
  const int KK = g.kH * g.kW;

  float16v acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  // A loader: row (t >> 1), k = 8 * (t & 1) .. + 7
  const int rowA = t >> 1, kA = (t & 1) * 8;
  const bool rowOk = m0 + rowA < p.M;
  const float *aSrc = p.w + (long)(m0 + rowA) * g.K + kA;
  // B loader: column (t & 127) = one output position, k = 8 * (t >> 7) .. + 7 (wave-uniform)
  const int colB = t & 127;
  const int kB = __builtin_amdgcn_readfirstlane((t >> 7) * 8);
  const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc((void *)p.x, 0, p.xBytes, 0x00020000);
  const int kOob = 0x7fffffff;  // beyond num_records: the load returns 0
  int ih0 = 0, iw0 = 0, posOff = kOob;
  {
    long lg = (long)j0 + colB;
    if (lg < (long)p.Ncols) {
      int n = (int)(lg / g.L);
      int l = (int)(lg - (long)n * g.L);
      int oh = l / g.oW, ow = l - oh * g.oW;
      ih0 = oh * g.dH - g.padH;
      iw0 = ow * g.dW - g.padW;
      posOff = ((n * g.Cin * g.H + ih0) * g.W + iw0) * 4;  // may be "negative": only used when the tap is inside
    } else {
      ih0 = -(1 << 28);  // every tap fails the bounds test
    }
  }

  float4 ra0, ra1, rb0, rb1;
  const int nktAll = (g.K + BK - 1) / BK;
  const int ktBegin = blockIdx.y * p.ktPerSplit;
  const int nkt = min(nktAll, ktBegin + p.ktPerSplit);  // this workgroup reduces k-tiles [ktBegin, nkt)

  auto loadTiles = [&](int kt) {
    const int k0 = kt * BK;
    // ---- A
    if (p.vecA && rowOk && k0 + kA + 8 <= g.K) {
      ra0 = reinterpret_cast<const float4 *>(aSrc + k0)[0];
      ra1 = reinterpret_cast<const float4 *>(aSrc + k0)[1];
    } else {
      float tmp[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) tmp[i] = (rowOk && k0 + kA + i < g.K) ? aSrc[k0 + i] : 0.f;
      ra0 = make_float4(tmp[0], tmp[1], tmp[2], tmp[3]);
      ra1 = make_float4(tmp[4], tmp[5], tmp[6], tmp[7]);
    }
    // ---- B: scalar walk over the 8 taps of this wave
    int k = k0 + kB;  // scalar
    int c = k / KK, rem = k - c * KK;
    int kh = rem / g.kW, kw = rem - kh * g.kW;
    float tmp[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int ih = ih0 + kh * g.dilH, iw = iw0 + kw * g.dilW;
      const bool ok = (unsigned)ih < (unsigned)g.H && (unsigned)iw < (unsigned)g.W && (k + i) < g.K;
      const int soff = ((c * g.H + kh * g.dilH) * g.W + kw * g.dilW) * 4;  // scalar
      const int off = ok ? posOff + soff : kOob;
      tmp[i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xr, off, 0, 0));
      if (++kw == g.kW) {
        kw = 0;
        if (++kh == g.kH) {
          kh = 0;
          ++c;
        }
      }
    }
    rb0 = make_float4(tmp[0], tmp[1], tmp[2], tmp[3]);
    rb1 = make_float4(tmp[4], tmp[5], tmp[6], tmp[7]);
  };
  auto storeTiles = [&](int buf) {
    As[buf][(t & 1) * 2][rowA] = ra0;
    As[buf][(t & 1) * 2 + 1][rowA] = ra1;
    Bs[buf][(t >> 7) * 2][colB] = rb0;
    Bs[buf][(t >> 7) * 2 + 1][colB] = rb1;
  };

  loadTiles(ktBegin);
  storeTiles(ktBegin & 1);
  __syncthreads();
  const int grp = lane >> 5, idx = lane & 31;
  for (int kt = ktBegin; kt < nkt; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < nkt) loadTiles(kt + 1);
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const float4 a0 = As[buf][2 * s + grp][wm * 64 + idx], a1 = As[buf][2 * s + grp][wm * 64 + 32 + idx];
      const float4 b0 = Bs[buf][2 * s + grp][wn * 64 + idx], b1 = Bs[buf][2 * s + grp][wn * 64 + 32 + idx];
      const float av0[4] = {a0.x, a0.y, a0.z, a0.w}, av1[4] = {a1.x, a1.y, a1.z, a1.w};
      const float bv0[4] = {b0.x, b0.y, b0.z, b0.w}, bv1[4] = {b1.x, b1.y, b1.z, b1.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av0[j], bv0[j], acc[0][0], 0, 0, 0);
        acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av0[j], bv1[j], acc[0][1], 0, 0, 0);
        acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av1[j], bv0[j], acc[1][0], 0, 0, 0);
        acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av1[j], bv1[j], acc[1][1], 0, 0, 0);
      }
    }
    if (kt + 1 < nkt) storeTiles(buf ^ 1);
    __syncthreads();
  }
  fwdEpilogue(p, g, acc, blockIdx.x, blockIdx.y, m0, j0, wm, wn, grp, idx);
}

// One half of a k-tile for one wave: 4 ds_read_b128 (two k-groups... one per lane group) and 16 MFMAs.
// aSrc / bSrc point at the lane's operands of k-group (lane / 32) in buffer 0; OA / OB are the float4
// offsets of the buffer and super-step, compile-time so that they fold into the LDS instruction.
template <int OA, int OB>
__device__ __forceinline__ void mfmaHalf(const float4 *aSrc, const float4 *bSrc, float16v (&acc)[2][2]) {
  const float4 a0 = aSrc[OA], a1 = aSrc[OA + 32];
  const float4 b0 = bSrc[OB], b1 = bSrc[OB + 32];
  const float av0[4] = {a0.x, a0.y, a0.z, a0.w}, av1[4] = {a1.x, a1.y, a1.z, a1.w};
  const float bv0[4] = {b0.x, b0.y, b0.z, b0.w}, bv1[4] = {b1.x, b1.y, b1.z, b1.w};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av0[j], bv0[j], acc[0][0], 0, 0, 0);
    acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av0[j], bv1[j], acc[0][1], 0, 0, 0);
    acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av1[j], bv0[j], acc[1][0], 0, 0, 0);
    acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av1[j], bv1[j], acc[1][1], 0, 0, 0);
  }
}
// the same for a wave that multiplies 32 rows: 3 ds_read_b128 and 8 MFMAs
template <int OA, int OB>
__device__ __forceinline__ void mfmaHalf(const float4 *aSrc, const float4 *bSrc, float16v (&acc)[1][2]) {
  const float4 a0 = aSrc[OA];
  const float4 b0 = bSrc[OB], b1 = bSrc[OB + 32];
  const float av0[4] = {a0.x, a0.y, a0.z, a0.w};
  const float bv0[4] = {b0.x, b0.y, b0.z, b0.w}, bv1[4] = {b1.x, b1.y, b1.z, b1.w};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av0[j], bv0[j], acc[0][0], 0, 0, 0);
    acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av0[j], bv1[j], acc[0][1], 0, 0, 0);
  }
}

// Forward kernel for images that carry their zero border in memory (padH = padW = 0 in g,
// K % BK == 0, 16-byte loadable weight rows). On this part every ordinary vector-ALU
// instruction takes issue time away from the MFMA pipe, so the main loop has none:
//  * a lane's output position is a fixed byte offset in a VGPR, the tap (c, kh, kw) of each k
//    is a byte offset read from a table with scalar loads and handed to the buffer load as its
//    scalar offset; every tap of every position is inside the padded image - no bounds test
//  * weight rows are addressed as fixed VGPR offset + scalar k offset
//  * the loop is unrolled over the two LDS buffers, so every LDS address is base + immediate
// Rows past M and columns past the batch are clamped to valid ones and dropped in the epilogue.
// WM = 2: 128 x 128 tiles, the four waves as 2 x 2; WM = 1: 64 x 256 tiles, the four waves side by side,
// for row counts whose last 128-row tile would be at most half full; a wave multiplies 64 x 64 either way.
// WM = 0: 32 x 256 tiles, a wave multiplies 32 x 64, for 32 rows or fewer left over (32-plane layers).
// (bx, by): position among the tiles that start at tile0 and split; whole: the workgroup reduces all of K
// of tile bx and writes the output itself
// LINEAR: 1x1 windows - the tap offsets are an arithmetic sequence, computed by the scalar unit instead of
// read from the table
template <int WM, bool LINEAR = false>
__device__ __forceinline__ void fwdPaddedBody(const FwdArgs &p, const ConvGeom &g, int bx, int by, bool whole) {
  constexpr int TBM = WM == 0 ? 32 : 64 * WM, TBN = WM == 2 ? 128 : 256;
  constexpr int TI = WM == 0 ? 1 : 2;         // 32-row blocks of a wave
  constexpr int NA = WM == 2 ? 2 : 1;         // 16-byte groups of weights a lane loads per k-tile
  constexpr int AP = TBM + 8, BP = TBN + 8;  // float4 per k-group row
  constexpr int NB = WM == 2 ? 8 : 16;        // image elements a lane gathers per k-tile
  __shared__ float4 As[2][BK / 4][AP];
  __shared__ float4 Bs[2][BK / 4][BP];
  __shared__ __attribute__((aligned(16))) float biasS[TBM];  // the tile's bias values: the epilogue reads them from here
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wm = WM == 2 ? wave >> 1 : 0, wn = WM == 2 ? wave & 1 : wave;
  const int tileIdx = whole ? bx : p.tile0 + bx;
  const int mTile = tileIdx % p.mTiles, nTile = tileIdx / p.mTiles;
  const int m0 = mTile * TBM, j0 = nTile * TBN;
  if (t < TBM) biasS[t] = p.bias && m0 + t < p.M ? p.bias[m0 + t] : 0.f;  // visible after the first barrier

  float16v acc[TI][2];

  const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc((void *)p.w, 0, p.wBytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc((void *)p.x, 0, p.xBytes, 0x00020000);
  // weights: WM = 2 - a lane loads 8 consecutive k of row t / 2; WM = 1 - 4 consecutive k of row t / 4;
  //          WM = 0 - the same of row (t / 4) % 32: both halves of the workgroup fetch and park the same values
  // image:   WM = 2 - a lane gathers 8 taps of column t % 128; WM < 2 - all 16 taps of column t
  const int rowA = WM == 2 ? t >> 1 : WM == 1 ? t >> 2 : (t >> 2) & 31;
  const int kgA = WM == 2 ? (t & 1) * 2 : t & 3;
  const int colB = WM == 2 ? t & 127 : t;
  const int kgB = WM == 2 ? (t >> 7) * 2 : 0;
  const int aOff = (min(m0 + rowA, p.M - 1) * g.K + kgA * 4) * 4;
  const int kB = __builtin_amdgcn_readfirstlane(kgB * 4);
  int posOff;
  {
    const unsigned lg = min((unsigned)j0 + colB, (unsigned)p.Ncols - 1);  // Ncols < 2^31
    int n, oh, ow;
    splitColumn(p, g, lg, n, oh, ow);
    posOff = ((n * g.Cin * g.H + oh * g.dH) * g.W + ow * g.dW) * 4;
  }
  const int ktBegin = by * p.ktPerSplit;  // by == 0 for whole tiles
  const int nkt = whole ? g.K / BK : min(g.K / BK, ktBegin + p.ktPerSplit);  // this workgroup reduces k-tiles [ktBegin, nkt)

  u32x4 ra[NA];
  unsigned rb[NB];
  // The tap offsets of a wave and k-tile are fetched with scalar loads one tile ahead of their use,
  // so that no wave waits on the scalar cache inside the loop (the table has spare entries at its end).
  const int4 *tapBase = reinterpret_cast<const int4 *>(p.taps + kB);
  int4 e[NB / 4];
  auto loadTaps = [&](int kt) {
#pragma unroll
    for (int i = 0; i < NB / 4; ++i) {
      if (LINEAR) {
        const int b = __builtin_amdgcn_readfirstlane((int)((unsigned)(kt * BK + kB + 4 * i) * (unsigned)p.tapStride));
        e[i] = make_int4(b, b + p.tapStride, b + 2 * p.tapStride, b + 3 * p.tapStride);
      } else {
        e[i] = tapBase[kt * (BK / 4) + i];
      }
    }
  };
  auto loadTiles = [&](int kt) {
    const int k0 = __builtin_amdgcn_readfirstlane(kt * BK);
#pragma unroll
    for (int i = 0; i < NA; ++i) ra[i] = __builtin_amdgcn_raw_buffer_load_b128(wr, aOff + 16 * i, k0 * 4, 0);
#pragma unroll
    for (int i = 0; i < NB / 4; ++i) {
      rb[4 * i + 0] = __builtin_amdgcn_raw_buffer_load_b32(xr, posOff, e[i].x, 0);
      rb[4 * i + 1] = __builtin_amdgcn_raw_buffer_load_b32(xr, posOff, e[i].y, 0);
      rb[4 * i + 2] = __builtin_amdgcn_raw_buffer_load_b32(xr, posOff, e[i].z, 0);
      rb[4 * i + 3] = __builtin_amdgcn_raw_buffer_load_b32(xr, posOff, e[i].w, 0);
    }
  };
  u32x4 *aDst = reinterpret_cast<u32x4 *>(&As[0][kgA][rowA]);
  u32x4 *bDst = reinterpret_cast<u32x4 *>(&Bs[0][kgB][colB]);
  constexpr int BUFA = (BK / 4) * AP, BUFB = (BK / 4) * BP;  // float4 per LDS buffer
  auto storeTiles = [&](auto bufc) {
    constexpr int b = decltype(bufc)::value;
#pragma unroll
    for (int i = 0; i < NA; ++i) aDst[b * BUFA + i * AP] = ra[i];
#pragma unroll
    for (int i = 0; i < NB / 4; ++i) bDst[b * BUFB + i * BP] = u32x4{rb[4 * i], rb[4 * i + 1], rb[4 * i + 2], rb[4 * i + 3]};
  };
  const int grp = lane >> 5, idx = lane & 31;
  const float4 *aSrc = &As[0][grp][wm * 64 + idx];
  const float4 *bSrc = &Bs[0][grp][wn * 64 + idx];
  using Buf0 = std::integral_constant<int, 0>;
  using Buf1 = std::integral_constant<int, 1>;

  // Software pipeline. While tile kt is multiplied out of one LDS buffer, tile kt + 1 waits in
  // registers and tile kt + 2 is requested from memory:
  //   first 16 MFMAs of kt | registers (kt + 1) -> other LDS buffer, global loads of kt + 2 |
  //   last 16 MFMAs of kt | barrier
  // The LDS stores and the load issue sit between the two MFMA halves, so the matrix pipe has
  // queued work while they run and the only stall left at the barrier is the LDS read latency.
  // The scheduling fences pin that order.
  auto step = [&](auto cur, auto nxt, int kt, bool store, bool load) {
    constexpr int C = decltype(cur)::value;
    mfmaHalf<C * BUFA, C * BUFB>(aSrc, bSrc, acc);
    __builtin_amdgcn_sched_barrier(0);
    if (store) storeTiles(nxt);
    if (load) {
      loadTiles(kt + 2);
      loadTaps(kt + 3);
    }
    __builtin_amdgcn_sched_barrier(0);
    mfmaHalf<C * BUFA + 2 * AP, C * BUFB + 2 * BP>(aSrc, bSrc, acc);
    __syncthreads();
  };

  loadTaps(ktBegin);
  loadTiles(ktBegin);
  loadTaps(ktBegin + 1);
  storeTiles(Buf0{});
  if (ktBegin + 1 < nkt) {
    loadTiles(ktBegin + 1);
    loadTaps(ktBegin + 2);
  }
  __syncthreads();
  // the accumulators of a whole tile start from the bias (in LDS since the barrier): no addition in the epilogue
  {
    const int grpRow = (lane >> 5) * 4;
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float4 b4 = make_float4(0.f, 0.f, 0.f, 0.f);
        if (whole) b4 = *reinterpret_cast<const float4 *>(biasS + wm * 64 + i * 32 + 8 * q + grpRow);
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j][4 * q] = b4.x, acc[i][j][4 * q + 1] = b4.y, acc[i][j][4 * q + 2] = b4.z, acc[i][j][4 * q + 3] = b4.w;
      }
  }
  int kt = ktBegin;
  for (; kt + 3 < nkt; kt += 2) {  // tile kt sits in buffer 0, tile kt + 1 in registers
    step(Buf0{}, Buf1{}, kt, true, true);
    step(Buf1{}, Buf0{}, kt + 1, true, true);
  }
  // one to three tiles left
  step(Buf0{}, Buf1{}, kt, kt + 1 < nkt, kt + 2 < nkt);
  if (kt + 1 < nkt) step(Buf1{}, Buf0{}, kt + 1, kt + 2 < nkt, false);
  if (kt + 2 < nkt) step(Buf0{}, Buf1{}, kt + 2, false, false);
  fwdEpilogue<TBN, TI>(p, g, acc, bx, by, m0, j0, wm, wn, grp, idx, biasS, whole ? 0 : 1, whole);
}

template <int WM, bool LINEAR = false>
__global__ void __launch_bounds__(dev::kBlock, 3)
convFwdPaddedKernel(FwdArgs p, ConvGeom g) {
  int bx = blockIdx.x, by = 0;
  const bool whole = bx < p.full;
  if (!whole) {
    const int u = bx - p.full;
    by = u / p.tail;
    bx = u - by * p.tail;
  }
  fwdPaddedBody<WM, LINEAR>(p, g, bx, by, whole);
}

// Several independent GEMMs of the same tile shape in one launch (the phases of a strided gradInput). An item's
// first p.full tiles are reduced by one workgroup each, its other p.tail tiles by p.nSplit workgroups. One flat
// grid: the whole tiles of all items in item order, then the splits of all items (split-major within an item) -
// the splits fill the slots that the last whole tiles free.
struct FwdBatchItem {
  FwdArgs p;
  ConvGeom g;
  int wholeEnd, splitEnd;  // running totals of p.full and of p.tail * p.nSplit up to and including this item
};
constexpr int kMaxBatch = 16;
struct FwdBatch {
  FwdBatchItem item[kMaxBatch];
  int count, wholeTotal;
};
static_assert(sizeof(FwdBatch) <= 4096, "kernel arguments are limited to 4 KB");

template <int WM>
__global__ void __launch_bounds__(dev::kBlock, 3)
convFwdPaddedBatchKernel(FwdBatch b) {
  int bx = blockIdx.x, by = 0, i = 0;
  const bool whole = bx < b.wholeTotal;
  if (whole) {
    while (i + 1 < b.count && bx >= b.item[i].wholeEnd) ++i;
    bx -= i > 0 ? b.item[i - 1].wholeEnd : 0;
  } else {
    bx -= b.wholeTotal;
    while (i + 1 < b.count && bx >= b.item[i].splitEnd) ++i;
    bx -= i > 0 ? b.item[i - 1].splitEnd : 0;
    const int tail = b.item[i].p.tail;
    by = bx / tail;
    bx -= by * tail;
  }
  fwdPaddedBody<WM>(b.item[i].p, b.item[i].g, bx, by, whole);
}

// 16-byte load of data that is read exactly once (non-temporal hint: it does not displace what the caches hold)
__device__ __forceinline__ float4 loadOnce4(const float4 *p) {
  typedef float f32x4v __attribute__((ext_vector_type(4)));
  const f32x4v v = __builtin_nontemporal_load(reinterpret_cast<const f32x4v *>(p));
  return make_float4(v.x, v.y, v.z, v.w);
}

// out tile = bias + sum over the nSplit partial tiles (ascending split order).
// grid = (tail tiles, BM*BN / 1024): a workgroup folds 1024 consecutive tile elements, 4 per lane.
__device__ __forceinline__ void fwdTailFixupBody(const FwdArgs &p, const ConvGeom &g) {
  const int tileIdx = p.tile0 + blockIdx.x;
  const int mTile = tileIdx % p.mTiles, nTile = tileIdx / p.mTiles;
  const float *src = p.partial + (long)blockIdx.x * p.nSplit * (BM * BN);
  const int e = (blockIdx.y * dev::kBlock + threadIdx.x) * 4;  // tile width % 4 == 0: the 4 elements share a row
  float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
  // the partials are requested eight (then four) at a time and added in ascending split order: one memory round trip
  // per batch instead of one per split, the same sum bit for bit
  int sp = 0;
  auto batch = [&](auto nc) {
    constexpr int NQ = decltype(nc)::value;
    float4 q[NQ];
#pragma unroll
    for (int i = 0; i < NQ; ++i) q[i] = loadOnce4(reinterpret_cast<const float4 *>(src + (long)(sp + i) * (BM * BN) + e));
#pragma unroll
    for (int i = 0; i < NQ; ++i) v.x += q[i].x, v.y += q[i].y, v.z += q[i].z, v.w += q[i].w;
    sp += NQ;
  };
  while (sp + 8 <= p.nSplit) batch(std::integral_constant<int, 8>{});
  if (sp + 4 <= p.nSplit) batch(std::integral_constant<int, 4>{});
  while (sp < p.nSplit) batch(std::integral_constant<int, 1>{});
  const int r = e / p.bn, c = e - r * p.bn;
  const int row = mTile * p.bm + r;
  if (r >= p.bm || row >= p.M) return;  // 32 x 256 tiles fill half of a partial
  const float b = p.bias ? p.bias[row] : 0.f;
  float vals[4] = {v.x + b, v.y + b, v.z + b, v.w + b};
  if (p.relu) {
#pragma unroll
    for (int i = 0; i < 4; ++i) vals[i] = vals[i] > 0.f ? vals[i] : 0.f;
  }
  // (n, oh, ow) of the first of the four columns by one division (through the reciprocals when the launch provides
  // them), the others by stepping
  const long col0 = (long)nTile * p.bn + c;
  if (col0 >= p.Ncols) return;
  int n, oh, ow;
  if (col0 + 3 < 0x7fffffffL) {
    splitColumn(p, g, (unsigned)col0, n, oh, ow);
  } else {
    n = (int)(col0 / g.L);
    const int l = (int)(col0 - (long)n * g.L);
    oh = l / g.oW, ow = l - oh * g.oW;
  }
  if (p.dilate) {
    // four neighbouring columns of one output row: their 2 x 2 blocks are 8 consecutive floats of two rows of out
    float *q = p.out + (long)n * p.outImg + (long)row * p.outRow + (long)oh * p.outSH + ow * 2;
    if (col0 + 3 < p.Ncols && ow + 3 < g.oW && ((uintptr_t)q & 15) == 0 && (p.outSH & 7) == 0) {
      float4 *top = reinterpret_cast<float4 *>(q), *bottom = reinterpret_cast<float4 *>(q + (p.outSH >> 1));
      top[0] = make_float4(vals[0], b, vals[1], b), top[1] = make_float4(vals[2], b, vals[3], b);
      bottom[0] = bottom[1] = make_float4(b, b, b, b);
      return;
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (col0 + i >= p.Ncols) break;
    float *q = p.out + (long)n * p.outImg + (long)row * p.outRow + (long)oh * p.outSH + ow * p.outSW;
    if (p.dilate) {  // the block's rows start on 8-byte boundaries (even extents, 8-byte aligned tensor)
      *reinterpret_cast<float2 *>(q) = make_float2(vals[i], b);
      *reinterpret_cast<float2 *>(q + (p.outSH >> 1)) = make_float2(b, b);
    } else {
      q[0] = vals[i];
    }
    if (++ow == g.oW) {
      ow = 0;
      if (++oh == g.oH) oh = 0, ++n;
    }
  }
}

__global__ void __launch_bounds__(dev::kBlock)
fwdTailFixupKernel(FwdArgs p, ConvGeom g) {
  fwdTailFixupBody(p, g);
}

// the fold for the split tiles of a batch; grid = (most split tiles of an item, BM*BN / 1024, items)
__global__ void __launch_bounds__(dev::kBlock)
fwdTailFixupBatchKernel(FwdBatch b) {
  const FwdBatchItem &it = b.item[blockIdx.z];
  if ((int)blockIdx.x >= it.p.tail) return;
  fwdTailFixupBody(it.p, it.g);
}

// ---- weight gradient, second generation ------------------------------------------
// partial[split][o][k] = sum over the split's positions r = (n, l) of gy[n][o][l] * col[k][n,l].
// Same MFMA core and float4 operand layout as the forward kernels, with the reduction
// running over positions: 4 consecutive l of one gradOutput row are already a float4
// in memory (L % 4 == 0), so the A tile goes from 16-byte buffer loads to
// ds_write_b128 without a transpose. For the B tile a lane owns one position of the
// k-tile and 8 columns k; the columns never change, so their tap offsets are resolved
// once into registers, the images carry their zero border in memory (no bounds test)
// and a gather costs one add per element on top of one position update per k-tile.
// 16 consecutive lanes gather 16 consecutive positions (64-byte runs of x).
// L16: L % 16 == 0 - a k-tile never crosses an image, so the gradOutput offsets are a
// fixed VGPR part plus a scalar part.
struct GradWeightArgs {
  const float *gy;  // (N, M, L)
  const float *x;   // (N, Cin, H, W) of g: images with their zero border
  float *partial;   // (splits, M, Ncols)
  float *biasPartial;  // (splits, M) row sums of gy per split, or null: the bias gradient comes out of the same pass
  int M, Ncols;     // Cout, K
  int mTiles, nTiles;
  int totalKt, ktPerSplit;  // k-tiles of BK positions over the N*L positions; per split
  int gyBytes, xBytes;      // < 2^31
  unsigned magicOW;
  unsigned magicKK, magicKW;  // reciprocals of kH * kW and kW (dev::magicOf)
  int Lvalid;               // positions of an image (g.L may count the padding of the gradOutput rows)
};

// WM = 2: 128 x 128 tiles of gradWeight (Cout x K), WM = 1: 64 x 256 tiles (as in the forward kernel).
// WM = 0: 64 x 64 tiles for small gradWeights (first layers, narrow 1x1 convolutions), where the large tiles
// would spend most of their multiplications on padding: the four waves all own the whole tile and take one
// position group (4 of the 16 positions) of every k-tile each, i.e. a wave is a split of its own - it stores
// its partial under split index 4 * split + wave and the fold adds them like any other splits.
template <int OA, int OB, int TI, int TJ>
__device__ __forceinline__ void mfmaGroupPair(const float *aSrc, const float *bSrc, float16v (&acc)[TI][TJ]) {
  // lanes 0-31 hold position OA / OB of the group, lanes 32-63 the next one (aSrc / bSrc already point there)
  float a[TI], b[TJ];
#pragma unroll
  for (int i = 0; i < TI; ++i) a[i] = aSrc[OA + i * 32 * 4];
#pragma unroll
  for (int j = 0; j < TJ; ++j) b[j] = bSrc[OB + j * 32 * 4];
#pragma unroll
  for (int i = 0; i < TI; ++i)
#pragma unroll
    for (int j = 0; j < TJ; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
}

// (TI, TJ): 32-row and 32-column blocks of a small tile (WMODE = 0 only): 64 x 64, 32 x 64, 32 x 128, 64 x 32 ...
// B4: 4 consecutive positions of a column are 4 consecutive floats of the image (unit stride along the row, and the
// 4 positions never straddle two output rows - or the rows follow each other without a gap): a lane then fetches
// one such group for each of its columns with one 16-byte load (any 4-byte alignment) and parks it with one
// ds_write_b128, a quarter of the instructions of the element-wise gather.
template <bool L16, int WMODE, int TI = 2, int TJ = 2, bool B4 = false>
__global__ void __launch_bounds__(dev::kBlock, 3)
convGradWeightKernel(GradWeightArgs p, ConvGeom g) {
  constexpr bool TINY = WMODE == 0;
  static_assert(TINY || (TI == 2 && TJ == 2), "block counts are a parameter of the small tiles only");
  static_assert(!(TINY && B4), "the small tiles gather element by element");
  constexpr int WM = TINY ? 1 : WMODE;  // loader layout: 64 rows as in the 64 x 256 shape
  constexpr int TBM = TINY ? 32 * TI : 64 * WM, TBN = TINY ? 32 * TJ : 256 / WM;
  constexpr int AP = TBM + 8;   // float4 per position-group row of As
  constexpr int GP = TBN + 4;   // of Bs: the 4 groups of a wave's scalar stores hit disjoint banks
  constexpr int NB = B4 ? TBN / 64 : TBN / 16;  // columns a lane gathers per k-tile
  constexpr int CS = B4 ? 64 : 16;              // distance between a lane's columns
  __shared__ float4 As[2][BK / 4][AP];
  __shared__ float4 Bs[2][BK / 4][GP];
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wm = WM == 2 ? wave >> 1 : 0, wn = TINY ? 0 : (WM == 2 ? wave & 1 : wave);
  // workgroups that reduce the same positions (one split) are neighbours in the remapped order: same XCD, same L2
  const int tilesPerSplit = p.mTiles * p.nTiles;
  const int bid = dev::xcdRemap(blockIdx.x, gridDim.x);
  const int split = bid / tilesPerSplit, tileIdx = bid - split * tilesPerSplit;
  const int mTile = tileIdx % p.mTiles, nTile = tileIdx / p.mTiles;
  const int m0 = mTile * TBM, j0 = nTile * TBN;
  const int ktBegin = split * p.ktPerSplit;
  const int ktEnd = min(p.totalKt, ktBegin + p.ktPerSplit);
  const int kOob = 0x7fffffff;

  float16v acc[TI][TJ];
#pragma unroll
  for (int i = 0; i < TI; ++i)
#pragma unroll
    for (int j = 0; j < TJ; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  // ---- A loader. WM = 2: row o = t >> 1, positions 8 * (t & 1) .. + 7 of the k-tile as two float4;
  //                WM = 1: row o = t >> 2, positions 4 * (t & 3) .. + 3 as one float4 (32-row tiles: both halves
  //                of the workgroup fetch and park the same rows)
  const __amdgpu_buffer_rsrc_t gr = __builtin_amdgcn_make_buffer_rsrc((void *)p.gy, 0, p.gyBytes, 0x00020000);
  const int rowA = WM == 2 ? t >> 1 : (t >> 2) & (TBM - 1);
  const int pgA = WM == 2 ? (t & 1) * 2 : t & 3;  // first position group (of 4 positions) of the lane
  const int rowOffA = min(m0 + rowA, p.M - 1) * g.L * 4;  // rows past M are clamped and dropped in the epilogue
  const int imgStrideA = p.M * g.L * 4;
  int nA, lA;  // L16: scalar image and position of the k-tile; else: of this lane's first group
  {
    const unsigned r = (unsigned)ktBegin * BK + (L16 ? 0 : pgA * 4);  // N * L < 2^31
    nA = (int)(r / (unsigned)g.L);
    lA = (int)(r - (unsigned)nA * (unsigned)g.L);
  }
  // ---- B loader: position t & 15 of the k-tile, columns (t >> 4) + 16 i
  //      (B4: positions 4 * (t & 3) .. + 3, columns (t >> 2) + 64 i)
  const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc((void *)p.x, 0, p.xBytes, 0x00020000);
  const int rB = B4 ? (t & 3) * 4 : t & 15, cB = B4 ? t >> 2 : t >> 4;
  int tapOff[NB];
  {
    const int KK = g.kH * g.kW;
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int k = min(j0 + cB + CS * i, p.Ncols - 1);  // columns past K are dropped in the epilogue
      const int c = dev::fastDiv(k, p.magicKK), rem = k - c * KK;
      const int kh = dev::fastDiv(rem, p.magicKW), kw = rem - kh * g.kW;
      tapOff[i] = ((c * g.H + kh * g.dilH) * g.W + kw * g.dilW) * 4;
    }
  }
  const int imgStrideB = g.Cin * g.H * g.W * 4;
  const int rowStepB = g.dH * g.W * 4, colStepB = g.dW * 4;
  int lB, nOffB;  // position inside the image, byte offset of the image (>= xBytes past the batch: loads return 0)
  {
    const unsigned r = (unsigned)ktBegin * BK + rB;
    const int n = (int)(r / (unsigned)g.L);
    lB = (int)(r - (unsigned)n * (unsigned)g.L);
    nOffB = n * imgStrideB;
  }

  u32x4 ra[WM];
  unsigned rb[B4 ? 1 : NB];
  u32x4 rb4[B4 ? NB : 1];
  // loads the k-tile the position counters stand on, then advances them by BK (L >= BK: one wrap at most)
  auto loadTiles = [&]() {
    if constexpr (L16) {
      // N*L is a multiple of BK here, so every k-tile lies inside the batch (the scalar offset is not range-checked)
      const int so = __builtin_amdgcn_readfirstlane(nA * imgStrideA + lA * 4);
#pragma unroll
      for (int i = 0; i < WM; ++i) ra[i] = __builtin_amdgcn_raw_buffer_load_b128(gr, rowOffA + pgA * 16 + 16 * i, so, 0);
      lA += BK;
      if (lA >= g.L) lA -= g.L, ++nA;
    } else {
      const int o0 = nA < g.N ? nA * imgStrideA + rowOffA + lA * 4 : kOob;
      ra[0] = __builtin_amdgcn_raw_buffer_load_b128(gr, o0, 0, 0);
      if constexpr (WM == 2) {
        int n1 = nA, l1 = lA + 4;
        if (l1 >= g.L) l1 -= g.L, ++n1;
        const int o1 = n1 < g.N ? n1 * imgStrideA + rowOffA + l1 * 4 : kOob;
        ra[WM - 1] = __builtin_amdgcn_raw_buffer_load_b128(gr, o1, 0, 0);
      }
      lA += BK;
      if (lA >= g.L) lA -= g.L, ++nA;
    }
    {
      // (positions behind the image's last one exist when the gradOutput rows were padded to a multiple of 4:
      // their gradOutput is zero, they read the image at position 0)
      const int lq = lB < p.Lvalid ? lB : 0;
      const int oh = dev::fastDiv(lq, p.magicOW), ow = lq - oh * g.oW;
      const int posOff = nOffB + oh * rowStepB + ow * colStepB;
#pragma unroll
      for (int i = 0; i < NB; ++i) {
        if constexpr (B4)
          rb4[i] = __builtin_amdgcn_raw_buffer_load_b128(xr, (int)((unsigned)posOff + (unsigned)tapOff[i]), 0, 0);
        else
          rb[i] = __builtin_amdgcn_raw_buffer_load_b32(xr, (int)((unsigned)posOff + (unsigned)tapOff[i]), 0, 0);
      }
      lB += BK;
      if (lB >= g.L) lB -= g.L, nOffB += imgStrideB;
    }
  };
  u32x4 *aDst = reinterpret_cast<u32x4 *>(&As[0][pgA][rowA]);
  unsigned *bDst = reinterpret_cast<unsigned *>(&Bs[0][rB >> 2][cB]) + (rB & 3);
  u32x4 *bDst4 = reinterpret_cast<u32x4 *>(&Bs[0][rB >> 2][cB]);
  constexpr int BUFA = (BK / 4) * AP, BUFB = (BK / 4) * GP;  // float4 per LDS buffer
  // The workgroups of the first column tile also sum the gradOutput elements they pass on (each element of a
  // row is loaded by exactly one lane of exactly one of them): the bias gradient without a second pass over gy.
  const bool rowSums = nTile == 0 && p.biasPartial != nullptr;
  float rowSum = 0.f;
  auto storeTiles = [&](auto bufc) {
    constexpr int buf = decltype(bufc)::value;
#pragma unroll
    for (int i = 0; i < WM; ++i) aDst[buf * BUFA + i * AP] = ra[i];
    if (rowSums) {
#pragma unroll
      for (int i = 0; i < WM; ++i)
      {
        // (element by element: a bit cast applied to a vector element expression reads element 0 here)
        const unsigned ex = ra[i].x, ey = ra[i].y, ez = ra[i].z, ew = ra[i].w;
        rowSum += (__uint_as_float(ex) + __uint_as_float(ey)) + (__uint_as_float(ez) + __uint_as_float(ew));
      }
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      if constexpr (B4)
        bDst4[buf * BUFB + 64 * i] = rb4[i];
      else
        bDst[buf * BUFB * 4 + 64 * i] = rb[i];  // column + 16 = 16 float4 further
    }
  };
  const int grp = lane >> 5, idx = lane & 31;
  const float4 *aSrc = &As[0][grp][wm * 64 + idx];
  const float4 *bSrc = &Bs[0][grp][wn * 64 + idx];
  // small tiles: this wave's position group, element grp (then grp + 2) of its float4
  const float *aTiny = reinterpret_cast<const float *>(&As[0][wave][idx]) + grp;
  const float *bTiny = reinterpret_cast<const float *>(&Bs[0][wave][idx]) + grp;
  using Buf0 = std::integral_constant<int, 0>;
  using Buf1 = std::integral_constant<int, 1>;

  // same software pipeline as the forward kernel: tile kt in LDS, kt + 1 in registers, kt + 2 requested
  auto step = [&](auto cur, auto nxt, bool store, bool load) {
    constexpr int C = decltype(cur)::value;
    if constexpr (TINY)
      mfmaGroupPair<C * BUFA * 4, C * BUFB * 4, TI, TJ>(aTiny, bTiny, acc);
    else
      mfmaHalf<C * BUFA, C * BUFB>(aSrc, bSrc, acc);
    __builtin_amdgcn_sched_barrier(0);
    if (store) storeTiles(nxt);
    if (load) loadTiles();
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (TINY)
      mfmaGroupPair<C * BUFA * 4 + 2, C * BUFB * 4 + 2, TI, TJ>(aTiny, bTiny, acc);
    else
      mfmaHalf<C * BUFA + 2 * AP, C * BUFB + 2 * GP>(aSrc, bSrc, acc);
    __syncthreads();
  };
  if (ktBegin < ktEnd) {
    loadTiles();
    storeTiles(Buf0{});
    if (ktBegin + 1 < ktEnd) loadTiles();
    __syncthreads();
    int kt = ktBegin;
    for (; kt + 3 < ktEnd; kt += 2) {  // tile kt sits in buffer 0, tile kt + 1 in registers
      step(Buf0{}, Buf1{}, true, true);
      step(Buf1{}, Buf0{}, true, true);
    }
    // one to three tiles left
    step(Buf0{}, Buf1{}, kt + 1 < ktEnd, kt + 2 < ktEnd);
    if (kt + 1 < ktEnd) step(Buf1{}, Buf0{}, kt + 2 < ktEnd, false);
    if (kt + 2 < ktEnd) step(Buf0{}, Buf1{}, false, false);
  }

  // lane holds column (lane & 31), rows 8*(v/4) + 4*(lane/32) + v%4 of each 32x32 tile
  float *dst = p.partial + (long)(TINY ? split * 4 + wave : split) * p.M * p.Ncols;
#pragma unroll
  for (int tj = 0; tj < TJ; ++tj) {
    const int col = j0 + wn * 64 + tj * 32 + idx;
    if (col >= p.Ncols) continue;
#pragma unroll
    for (int ti = 0; ti < TI; ++ti)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = m0 + wm * 64 + ti * 32 + 8 * (v >> 2) + grp * 4 + (v & 3);
        if (row < p.M) dst[(long)row * p.Ncols + col] = acc[ti][tj][v];
      }
  }
  if (rowSums) {
    // the 2 (WM = 2) or 4 (WM = 1) lanes that loaded parts of a row are neighbours inside a quad
    rowSum = dev::dppAdd<0xB1>(rowSum);
    if (WM == 1) rowSum = dev::dppAdd<0x4E>(rowSum);
    if ((t & (WM == 2 ? 1 : 3)) == 0 && m0 + rowA < p.M && (t >> 2) < TBM) {
      if (TINY) {  // four partial slots per workgroup: the row sums go to the first, the others add nothing
        float *bp = p.biasPartial + (long)split * 4 * p.M + m0 + rowA;
        bp[0] = rowSum, bp[p.M] = 0.f, bp[2 * (long)p.M] = 0.f, bp[3 * (long)p.M] = 0.f;
      } else {
        p.biasPartial[(long)split * p.M + m0 + rowA] = rowSum;
      }
    }
  }
}

// gW[i] += scale * sum_s partial[s][i] in a fixed association: a workgroup owns 64 consecutive float4
// of gW; its 4 lane groups each sum the splits s = group, group + 4, ... with 4 independent
// accumulators (16 16-byte loads in flight per lane), then the groups are added in order through
// LDS. With few elements and hundreds of splits (1x1 convolutions) a one-lane-per-element loop is
// latency bound; this form keeps enough bytes in flight to run at memory speed.
// Blocks past the last float4 of gW do the same for the bias partials (biasPartial(splits, M), M % 4 == 0), when given.
// E: float4 of gW a workgroup owns (64, 16 or 4); its 256 / E lane groups share the splits. Small
// gradWeights with thousands of splits take small E: more workgroups, more loads in flight.
template <int E>
__global__ void __launch_bounds__(dev::kBlock)
foldPartials4Kernel(const float *__restrict__ partial, float *__restrict__ dst, long count4, int splits, float scale,
                    const float *__restrict__ biasPartial, float *__restrict__ gradBias, int M, int gwBlocks) {
  constexpr int G = dev::kBlock / E;
  __shared__ float4 part[G][E];
  int blk = blockIdx.x;
  if (blk >= gwBlocks) blk -= gwBlocks, partial = biasPartial, dst = gradBias, count4 = M >> 2;
  const int e = threadIdx.x % E, grp = threadIdx.x / E;
  const long i = (long)blk * E + e;
  float4 a[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) a[u] = make_float4(0.f, 0.f, 0.f, 0.f);
  if (i < count4) {
    const float4 *p = reinterpret_cast<const float4 *>(partial) + i;
    int s = grp;
    for (; s + 3 * G < splits; s += 4 * G) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const float4 v = loadOnce4(p + (long)(s + G * u) * count4);  // the partials' only reader
        a[u].x += v.x, a[u].y += v.y, a[u].z += v.z, a[u].w += v.w;
      }
    }
    for (; s < splits; s += G) {
      const float4 v = loadOnce4(p + (long)s * count4);
      a[0].x += v.x, a[0].y += v.y, a[0].z += v.z, a[0].w += v.w;
    }
  }
  part[grp][e] = make_float4((a[0].x + a[1].x) + (a[2].x + a[3].x), (a[0].y + a[1].y) + (a[2].y + a[3].y),
                             (a[0].z + a[1].z) + (a[2].z + a[3].z), (a[0].w + a[1].w) + (a[2].w + a[3].w));
  __syncthreads();
  if (grp == 0 && i < count4) {
    float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll 4
    for (int q = 0; q < G; q += 4) {
      const float4 p0 = part[q][e], p1 = part[q + 1][e], p2 = part[q + 2][e], p3 = part[q + 3][e];
      t.x += (p0.x + p1.x) + (p2.x + p3.x), t.y += (p0.y + p1.y) + (p2.y + p3.y);
      t.z += (p0.z + p1.z) + (p2.z + p3.z), t.w += (p0.w + p1.w) + (p2.w + p3.w);
    }
    float4 d = reinterpret_cast<float4 *>(dst)[i];
    d.x += scale * t.x, d.y += scale * t.y, d.z += scale * t.z, d.w += scale * t.w;
    reinterpret_cast<float4 *>(dst)[i] = d;
  }
}

// the same for any count / alignment: gW[i] += scale * sum_s partial[s][i], s ascending
__global__ void __launch_bounds__(dev::kBlock)
foldPartialsKernel(const float *__restrict__ partial, float *__restrict__ dst, long count, int splits, float scale) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (long)gridDim.x * blockDim.x) {
    float s = 0.f;
    for (int k = 0; k < splits; ++k) s += partial[(long)k * count + i];
    dst[i] += scale * s;
  }
}

// gradBias[o] += scale * sum_{n,l} gy[n][o][l]   (lib/THCUNN/generic/SpatialConvolutionMM.cu:440-455)
// One 1024-lane workgroup per output plane o streams its N runs of L floats.
constexpr int kBiasBlock = 1024;
template <bool VEC>
__global__ void __launch_bounds__(kBiasBlock)
gradBiasKernel(const float *__restrict__ gy, float *__restrict__ gradBias, int N, int Cout, int L, float scale) {
  __shared__ float red[kBiasBlock / dev::kWave];
  const int o = blockIdx.x;
  float acc = 0.f;
  if (VEC) {
    const int L4 = L >> 2;
    const int total4 = N * L4;
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    for (int i = threadIdx.x; i < total4; i += kBiasBlock) {
      int n = i / L4, l4 = i - n * L4;
      float4 v = *reinterpret_cast<const float4 *>(gy + ((long)n * Cout + o) * L + (l4 << 2));
      a0 += v.x, a1 += v.y, a2 += v.z, a3 += v.w;
    }
    acc = (a0 + a1) + (a2 + a3);
  } else {
    const long total = (long)N * L;
    for (long i = threadIdx.x; i < total; i += kBiasBlock) {
      int n = (int)(i / L);
      int l = (int)(i - (long)n * L);
      acc += gy[((long)n * Cout + o) * L + l];
    }
  }
  acc = dev::waveSum(acc);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    float s = 0.f;
    for (int w = 0; w < kBiasBlock / dev::kWave; ++w) s += red[w];
    gradBias[o] += scale * s;
  }
}

// wt[k][o] = w[o][k] for w (rows x cols)
__global__ void __launch_bounds__(dev::kBlock)
transposeKernel(const float *__restrict__ w, float *__restrict__ wt, int rows, int cols) {
  const long total = (long)rows * cols;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    const int o = (int)(i % rows);
    const long k = i / rows;
    wt[i] = w[(long)o * cols + k];
  }
}

// Wf[c][(o, kh', kw')] = W[o][(c, kH-1-kh', kW-1-kw')]: with these weights the
// stride-1 gradInput is a plain forward convolution of gradOutput (padding k-1-pad).
__global__ void __launch_bounds__(dev::kBlock)
flipWeightKernel(const float *__restrict__ w, float *__restrict__ wf, int Cout, int Cin, int kH, int kW) {
  const int KK = kH * kW;
  const long total = (long)Cout * Cin * KK;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    int t = (int)(i % KK);
    long r = i / KK;
    int o = (int)(r % Cout);
    int c = (int)(r / Cout);
    wf[i] = w[((long)o * Cin + c) * KK + (KK - 1 - t)];
  }
}

// ---- im2col / col2im (lib/THCUNN/im2col.h) -----------------------------------
// One lane per column entry; consecutive lanes write consecutive addresses.
__global__ void __launch_bounds__(dev::kBlock)
im2colKernel(const float *__restrict__ im, float *__restrict__ col, int nImg, int C, int H, int W, int kH, int kW,
             int padH, int padW, int dH, int dW, int dilH, int dilW, int oH, int oW) {
  const long L = (long)oH * oW;
  const long perImg = (long)C * kH * kW * L;
  const long total = perImg * nImg;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    long n = i / perImg;
    long r = i - n * perImg;
    int ow = (int)(r % oW);
    r /= oW;
    int oh = (int)(r % oH);
    r /= oH;
    int kw = (int)(r % kW);
    r /= kW;
    int kh = (int)(r % kH);
    int c = (int)(r / kH);
    int h = oh * dH - padH + kh * dilH, w = ow * dW - padW + kw * dilW;
    col[i] = (h >= 0 && w >= 0 && h < H && w < W) ? im[((n * C + c) * H + h) * W + w] : 0.f;
  }
}

// One lane per image pixel gathers every column entry that maps onto it
// (lib/THCUNN/im2col.h:63-102); float accumulation in the reference's order.
__global__ void __launch_bounds__(dev::kBlock)
col2imKernel(const float *__restrict__ col, float *__restrict__ im, int nImg, int C, int H, int W, int kH, int kW,
             int padH, int padW, int dH, int dW, int dilH, int dilW, int oH, int oW, const float *__restrict__ bias) {
  const long total = (long)nImg * C * H * W;
  const int extW = (kW - 1) * dilW + 1, extH = (kH - 1) * dilH + 1;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    int w_im = (int)(i % W) + padW;
    int h_im = (int)((i / W) % H) + padH;
    long nc = i / ((long)W * H);  // n * C + c
    int ws = (w_im < extW) ? 0 : (w_im - extW) / dW + 1;
    int we = min(w_im / dW + 1, oW);
    int hs = (h_im < extH) ? 0 : (h_im - extH) / dH + 1;
    int he = min(h_im / dH + 1, oH);
    float val = bias ? bias[(int)(nc % C)] : 0.f;  // per-plane bias of the transposed convolution, else 0
    for (int hc = hs; hc < he; ++hc)
      for (int wc = ws; wc < we; ++wc) {
        int hk = h_im - hc * dH, wk = w_im - wc * dW;
        if (hk % dilH == 0 && wk % dilW == 0) {
          hk /= dilH;
          wk /= dilW;
          val += col[(((nc * kH + hk) * kW + wk) * oH + hc) * oW + wc];
        }
      }
    im[i] = val;
  }
}

#include "conv_pointwise.h"
#include "conv_fewplanes.h"

// ---- host side -----------------------------------------------------------------
struct ConvCall {
  ConvGeom g;
  bool batch;
};

ConvGeom makeGeom(int N, int Cin, int Cout, int H, int W, int oH, int oW, int kH, int kW, int dH, int dW, int padH,
                  int padW, int dilH, int dilW) {
  ConvGeom g{};
  g.N = N, g.Cin = Cin, g.Cout = Cout, g.H = H, g.W = W, g.oH = oH, g.oW = oW;
  g.kH = kH, g.kW = kW, g.dH = dH, g.dW = dW, g.padH = padH, g.padW = padW, g.dilH = dilH, g.dilW = dilW;
  g.K = g.Cin * kH * kW;
  g.L = g.oH * g.oW;
  if ((long)g.Cin * g.H * g.W >= 0x7fffffffL || (long)g.Cout * g.L >= 0x7fffffffL || (long)g.K * g.L >= 0x7fffffffL * 8L)
    error("spatial convolution: image too large");
  return g;
}

// Shape rules of lib/THCUNN/generic/SpatialConvolutionMM.cu:5-56 (kConvMM: `weight` 2-D
// (Cout, Cin*kH*kW) or 4-D) and of generic/SpatialDilatedConvolution.cu:5-67 (kDilated: 4-D weight,
// dilation > 0); only the extents of `weight` are read here.
enum ConvFlavor { kConvMM, kDilated };
ConvCall convSetup(THCudaTensor *input, THCudaTensor *gradOutput, THCudaTensor *weight, THCudaTensor *bias,
                   const char *weightName, int kH, int kW, int dH, int dW, int padH, int padW, int dilH = 1,
                   int dilW = 1, ConvFlavor flavor = kConvMM) {
  THC_ARG_CHECK(input && weight, 2, "input and weight tensors expected");
  if (flavor == kDilated)
    THC_ARG_CHECK(weight->nDimension == 4, 4,
                  "4D weight tensor (nOutputPlane,nInputPlane,kH,kW) expected, but got: %s",
                  sizeDesc(erase(weight)).c_str());
  else
    THC_ARG_CHECK(isContiguous(erase(weight)), 4, "%s tensor has to be contiguous", weightName);
  THC_ARG_CHECK(kW > 0 && kH > 0, 9, "kernel size should be greater than zero, but got kH: %d kW: %d", kH, kW);
  THC_ARG_CHECK(dW > 0 && dH > 0, 11, "stride should be greater than zero, but got dH: %d dW: %d", dH, dW);
  if (flavor == kDilated)
    THC_ARG_CHECK(isContiguous(erase(weight)), 4, "%s tensor has to be contiguous", weightName);
  THC_ARG_CHECK(!bias || isContiguous(erase(bias)), 5, "bias tensor has to be contiguous");
  if (flavor == kDilated)
    THC_ARG_CHECK(dilW > 0 && dilH > 0, 14, "dilation should be greater than 0, but got dilationH: %d dilationW: %d",
                  dilH, dilW);
  else
    THC_ARG_CHECK(weight->nDimension == 2 || weight->nDimension == 4, 5,
                  "2D or 4D weight tensor expected, but got: %s", sizeDesc(erase(weight)).c_str());
  long nOutputPlane = weight->size[0];
  long wcols = weight->nDimension == 2 ? weight->size[1] : weight->size[1] * weight->size[2] * weight->size[3];
  if (bias) checkDimSize(erase(bias), "bias", 1, 0, nOutputPlane);
  int ndim = input->nDimension;
  int dimf = 0, dimh = 1, dimw = 2;
  if (ndim == 4) {
    dimf++;
    dimh++;
    dimw++;
  }
  THC_ARG_CHECK(ndim == 3 || ndim == 4, 2, "3D or 4D input tensor expected but got: %s",
                sizeDesc(erase(input)).c_str());
  long nInputPlane = flavor == kDilated ? weight->size[1] : wcols / (kH * kW);
  long inputHeight = input->size[dimh], inputWidth = input->size[dimw];
  long outputHeight = (inputHeight + 2 * padH - (dilH * (kH - 1) + 1)) / dH + 1;
  long outputWidth = (inputWidth + 2 * padW - (dilW * (kW - 1) + 1)) / dW + 1;
  if (outputWidth < 1 || outputHeight < 1)
    error("Given input size: (%ld x %ld x %ld). Calculated output size: (%ld x %ld x %ld). Output size is too small",
          nInputPlane, inputHeight, inputWidth, nOutputPlane, outputHeight, outputWidth);
  checkDimSize(erase(input), "input", ndim, dimf, nInputPlane);
  if (gradOutput) {
    checkDimSize(erase(gradOutput), "gradOutput", ndim, dimf, nOutputPlane);
    checkDimSize(erase(gradOutput), "gradOutput", ndim, dimh, outputHeight);
    checkDimSize(erase(gradOutput), "gradOutput", ndim, dimw, outputWidth);
    if (ndim == 4 && gradOutput->size[0] != input->size[0])
      error("input and gradOutput batch sizes do not match: input %s, gradOutput %s", sizeDesc(erase(input)).c_str(),
            sizeDesc(erase(gradOutput)).c_str());
  }
  if (wcols != nInputPlane * kH * kW)
    error("%s of shape %s does not match a %d x %d kernel", weightName, sizeDesc(erase(weight)).c_str(), kH, kW);
  ConvCall call;
  call.batch = ndim == 4;
  call.g = makeGeom(call.batch ? (int)input->size[0] : 1, (int)nInputPlane, (int)nOutputPlane, (int)inputHeight,
                    (int)inputWidth, (int)outputHeight, (int)outputWidth, kH, kW, dH, dW, padH, padW, dilH, dilW);
  return call;
}

inline unsigned tiles(long n, int b) { return (unsigned)((n + b - 1) / b); }

// Workgroups of `kernel` (256 lanes, static LDS) the whole device holds at once.
// kernel == nullptr: the number of CUs.
int residentSlots(const void *kernel) {
  static std::mutex mu;
  static std::map<std::pair<int, const void *>, int> cache;  // per (device, kernel)
  int dev = 0, cus = 0, perCu = 1;
  THC_HIP_CHECK(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(mu);
  auto it = cache.find({dev, kernel});
  if (it != cache.end()) return it->second;
  THC_HIP_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  if (kernel) THC_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&perCu, kernel, dev::kBlock, 0));
  int v = std::max(1, cus) * std::max(1, perCu);
  cache[{dev, kernel}] = v;
  return v;
}

// Test switch: "1" routes the forward pass (and the stride-1 gradInput that
// reuses it) through the first-generation kernels.
bool forceGeneric() { return g_switches.convGeneric == 1; }

// Plan of one implicit-GEMM forward launch. The 128x128 tiles are dealt to the
// CUs in rounds; a last partial round would leave most CUs idle while a few
// finish one more tile, so the tiles of that round are instead split along K
// over all CUs (partials in scratch, folded by fwdTailFixupKernel in a fixed order).
// Whole tiles and splits are workgroups of one launch: the splits take the slots
// that the last whole tiles free.
struct FwdPlan {
  int bm, bn;          // tile shape: 128 x 128, or 64 x 256 when that wastes fewer rows (padded kernel only)
  int mTiles, total, full, tail, nSplit, ktPerSplit;
  int tapEntries;      // > 0: the padded kernel applies; entries of the tap table at the start of the scratch
  long paddedFloats;   // floats of the zero-bordered copy of the images (0: no border needed, or generic kernel)
  long weightFloats;   // floats of the copy of the weights with rows padded to a multiple of BK (0: not needed)
  long scratchFloats;  // tap table, tail partials, padded images
};
// Tiles of an M x Ncols output reduced over nkt k-tiles; wideOk: the 64 x 256 tile shape may be used.
void planTiles(FwdPlan &pl, int M, long Ncols, int nkt, bool wideOk) {
  const bool wide = wideOk && tiles(M, 64) * 64 < tiles(M, BM) * BM;
  // 32-row tiles when they cut the padded rows by a quarter or more (a wave then issues half the MFMAs per
  // element it gathers)
  const bool low = wideOk && tiles(M, 32) * 32 * 4 <= tiles(M, 64) * 64 * 3;
  pl.bm = low ? 32 : wide ? 64 : BM, pl.bn = low || wide ? 256 : BN;
  pl.mTiles = (int)tiles(M, pl.bm);
  pl.total = pl.mTiles * (int)tiles(Ncols, pl.bn);
  const int cus = residentSlots(nullptr);
  // Which tiles to split along K, and how finely: the workgroups go to the CUs in launch order (up to three
  // share a CU), so a CU's time is the sum over what it is dealt. In units of one k-tile of one workgroup alone
  // on its CU: a workgroup costs its k-tiles + 4 (prologue, epilogue), a split tile 0.006 more per partial
  // (written, then read by the fold), and a CU that only ever holds one workgroup runs at 0.85 of the rate
  // (nothing covers its barriers) - constants fitted to measured sweeps over S on 14x14 ... 56x56 layers.
  // Candidates: no split; the last, partial round split S ways; every tile split S ways (S <= 16, >= 4 k-tiles
  // per split). E.g. 196 tiles on 256 CUs: 5 splits (980 workgroups, 4 per CU at most) beat 2 (392: 136 CUs
  // carry two halves, 120 one) by 15 %; 136 tiles left over after a full round: 3 splits, not 1.
  const int maxS = std::max(1, std::min(nkt / 4, 16));
  const int q = pl.total / cus, r = pl.total % cus;
  auto perWg = [&](int S) { return (double)launch::ceilDiv(nkt, S) + 4.0; };
  // a split has to promise 5 % before it is taken: the model is coarse and the fold is one more launch
  double best = 0.95 * launch::ceilDiv(pl.total, cus) * perWg(1) / (pl.total <= cus ? 0.85 : 1.0);
  int nSplit = 1;
  pl.tail = 0;
  for (int S = 2; S <= maxS; ++S) {
    if (launch::ceilDiv(nkt, launch::ceilDiv(nkt, S)) != S) continue;  // the same pieces as a smaller S
    if (q > 0 && r > 0) {
      const double t = q * perWg(1) + launch::ceilDiv(r * S, cus) * perWg(S) + 0.006 * r * S;
      if (t < best) best = t, nSplit = S, pl.tail = r;
    }
    if (pl.total <= 2 * cus) {
      const int n = launch::ceilDiv(pl.total * S, cus);
      const double t = n * perWg(S) / (n == 1 ? 0.85 : 1.0) + 0.006 * pl.total * S;
      if (t < best) best = t, nSplit = S, pl.tail = pl.total;
    }
  }
  pl.full = pl.total - pl.tail;
  pl.ktPerSplit = launch::ceilDiv(nkt, nSplit);
  pl.nSplit = launch::ceilDiv(nkt, pl.ktPerSplit);
}
inline long partialFloats(const FwdPlan &pl) { return pl.tail ? (long)pl.tail * pl.nSplit * BM * BN : 0; }

// wAligned: the weights start on a 16-byte boundary (else the padded kernel works on an aligned copy)
FwdPlan planFwdImplicit(int M, int nImages, const ConvGeom &g, bool wAligned = true) {
  FwdPlan pl{};
  const int nkt = launch::ceilDiv(g.K, BK);
  const long padded = (long)nImages * g.Cin * (g.H + 2 * g.padH) * (g.W + 2 * g.padW);
  // K that is not a multiple of BK (first layers: Cin = 3) runs on the same kernel with the weight rows
  // copied into rows of Kp = nkt * BK floats, zero beyond K
  const int Kp = nkt * BK;
  const bool fast = !forceGeneric() && padded * 4 < 0x7fffffffL && (long)M * Kp * 4 < 0x7fffffffL;
  planTiles(pl, M, (long)nImages * g.L, nkt, fast);
  pl.tapEntries = fast ? Kp + 2 * BK : 0;  // spare entries: the kernel reads tap offsets up to two k-tiles ahead
  pl.paddedFloats = fast && (g.padH > 0 || g.padW > 0) ? padded : 0;
  pl.weightFloats = fast && (Kp != g.K || !wAligned) ? (long)M * Kp : 0;
  pl.scratchFloats = pl.tapEntries + partialFloats(pl) + (pl.paddedFloats + 3) / 4 * 4 + pl.weightFloats;
  return pl;
}

// The launches of one planned forward GEMM: full rounds, then the K-split tail and its fold. `p` carries the
// operands, the output addressing, M, Ncols and the byte sizes; gk is the geometry the kernels see.
void launchFwdKernels(hipStream_t s, const FwdPlan &pl, FwdArgs p, float *partial, const ConvGeom &gk, bool fast) {
  p.mTiles = pl.mTiles;
  p.bm = pl.bm, p.bn = pl.bn;
  p.full = pl.full, p.tail = pl.tail;
  if (fast) {
    // one launch: the tiles reduced by one workgroup first, then the splits of the tail tiles, which fill
    // the slots that the last whole tiles leave
    p.tile0 = pl.full;
    p.nSplit = pl.tail > 0 ? pl.nSplit : 1;
    p.ktPerSplit = pl.tail > 0 ? pl.ktPerSplit : launch::ceilDiv(gk.K, BK);
    p.partial = partial;
    const dim3 grid(pl.full + pl.tail * p.nSplit);
    if (p.tapStride > 0) {
      if (pl.bm == 32)
        convFwdPaddedKernel<0, true><<<grid, dev::kBlock, 0, s>>>(p, gk);
      else if (pl.bm == 64)
        convFwdPaddedKernel<1, true><<<grid, dev::kBlock, 0, s>>>(p, gk);
      else
        convFwdPaddedKernel<2, true><<<grid, dev::kBlock, 0, s>>>(p, gk);
    } else if (pl.bm == 32) {
      convFwdPaddedKernel<0><<<grid, dev::kBlock, 0, s>>>(p, gk);
    } else if (pl.bm == 64) {
      convFwdPaddedKernel<1><<<grid, dev::kBlock, 0, s>>>(p, gk);
    } else {
      convFwdPaddedKernel<2><<<grid, dev::kBlock, 0, s>>>(p, gk);
    }
    THC_HIP_CHECK(hipGetLastError());
    if (pl.tail > 0) {
      fwdTailFixupKernel<<<dim3(pl.tail, BM * BN / (4 * dev::kBlock)), dev::kBlock, 0, s>>>(p, gk);
      THC_HIP_CHECK(hipGetLastError());
    }
    return;
  }
  p.tile0 = 0;
  p.nSplit = 1;
  p.ktPerSplit = launch::ceilDiv(gk.K, BK);
  if (pl.full > 0) {
    convFwdImplicitKernel<<<dim3(pl.full), dev::kBlock, 0, s>>>(p, gk);
    THC_HIP_CHECK(hipGetLastError());
  }
  if (pl.tail > 0) {
    p.tile0 = pl.full;
    p.ktPerSplit = pl.ktPerSplit;
    p.nSplit = pl.nSplit;
    p.partial = partial;
    convFwdImplicitKernel<<<dim3(pl.tail, pl.nSplit), dev::kBlock, 0, s>>>(p, gk);
    THC_HIP_CHECK(hipGetLastError());
    fwdTailFixupKernel<<<dim3(pl.tail, BM * BN / (4 * dev::kBlock)), dev::kBlock, 0, s>>>(p, gk);
    THC_HIP_CHECK(hipGetLastError());
  }
}

// out(nImages, M, L) = bias + W(M x K) * im2col(x); `scratch` holds plan.scratchFloats floats
// Where the output elements go when not into a dense (nImages, M, oH, oW) tensor.
struct OutMap {
  long outImg;
  int outRow, outSH, outSW;
  int dilate;  // FwdArgs::dilate
};

void launchFwdImplicit(hipStream_t s, const FwdPlan &pl, float *scratch, const float *w, const float *x, float *out,
                       const float *bias, int M, int nImages, const ConvGeom &g, bool relu = false,
                       const OutMap *om = nullptr, const FlipJob *flip = nullptr) {
  const bool fast = pl.tapEntries > 0;
  if (flip && !(fast && pl.paddedFloats > 0)) {  // no bordered copy to ride along with
    flipWeightKernel<<<launch::directGrid((long)flip->Cout * flip->Cin * flip->kH * flip->kW, dev::kBlock), dev::kBlock, 0, s>>>(
        flip->w, flip->wf, flip->Cout, flip->Cin, flip->kH, flip->kW);
    THC_HIP_CHECK(hipGetLastError());
    flip = nullptr;
  }
  if (fast && !(launch::aligned16(scratch) && (pl.weightFloats > 0 || launch::aligned16(w))))
    error("SpatialConvolutionMM: internal error, convolution scratch or weights not 16-byte aligned");
  float *partial = scratch + pl.tapEntries;
  ConvGeom gk = g;  // geometry the kernel sees
  FwdArgs p{};
  p.x = x;
  if (fast) {
    gk.H = g.H + 2 * g.padH, gk.W = g.W + 2 * g.padW, gk.padH = gk.padW = 0;
    float *xp = partial + partialFloats(pl);
    // 1x1 windows over a whole number of k-tiles: tap k is plane k of the image, no table needed
    const bool linear = g.kH == 1 && g.kW == 1 && g.K % BK == 0;
    if (pl.paddedFloats > 0) {  // the copy into the bordered layout builds the tap table on the side
      launchPadPlanes(s, x, xp, (long)nImages * g.Cin, g.H, g.W, g.padH, g.padW, linear ? nullptr : reinterpret_cast<int *>(scratch),
                      pl.tapEntries, &gk, flip);
      p.x = xp;
    }
    if (linear) {
      p.tapStride = gk.H * gk.W * (int)sizeof(float);
    } else if (pl.paddedFloats <= 0) {
      buildTapTableKernel<<<launch::directGrid(pl.tapEntries, dev::kBlock), dev::kBlock, 0, s>>>(
          reinterpret_cast<int *>(scratch), pl.tapEntries, gk);
      THC_HIP_CHECK(hipGetLastError());
    }
    if (pl.weightFloats > 0) {
      float *wp = xp + (pl.paddedFloats + 3) / 4 * 4;
      gk.K = (int)(pl.weightFloats / M);
      padRowsKernel<<<launch::directGrid(pl.weightFloats, dev::kBlock), dev::kBlock, 0, s>>>(w, wp, M, g.K, gk.K);
      THC_HIP_CHECK(hipGetLastError());
      w = wp;
    }
  }
  p.taps = reinterpret_cast<const int *>(scratch);
  p.w = w;
  p.out = out;
  p.bias = bias;
  p.relu = relu ? 1 : 0;
  p.M = M;
  p.Ncols = nImages * g.L;
  p.outImg = (long)M * g.L, p.outRow = g.L, p.outSH = g.oW, p.outSW = 1;
  if (om) p.outImg = om->outImg, p.outRow = om->outRow, p.outSH = om->outSH, p.outSW = om->outSW, p.dilate = om->dilate;
  if (fast) {
    const long span = ((long)(nImages - 1) * p.outImg + (long)(M - 1) * p.outRow + (long)(g.oH - 1) * p.outSH +
                       (long)(g.oW - 1) * p.outSW + 1 + (p.dilate ? p.outSH / 2 + 1 : 0)) * 4;
    p.outBytes = span < 0x7fffffffL ? (int)span : 0;
    // (the reciprocal division is exact while dividend * divisor < 2^32)
    p.magicL = (long)p.Ncols * g.L < 0xffffffffL ? dev::magicOf(g.L) : 0;
    p.magicOW = (long)g.L * g.oW < 0xffffffffL ? dev::magicOf(g.oW) : 0;
  }
  p.xBytes = (int)((long)nImages * gk.Cin * gk.H * gk.W * sizeof(float));
  p.wBytes = (int)((long)M * gk.K * sizeof(float));
  p.vecA = (gk.K % 4 == 0) && launch::aligned16(w);
  launchFwdKernels(s, pl, p, partial, gk, fast);
}

// Scratch of `floats` floats: the caller's buffer tensor (resized) or a stream-ordered temporary.
float *scratchFloats(THCState *state, THCudaTensor *buffer, long floats, Temp &tmp, const char *name) {
  if (floats <= 0) return nullptr;
  if (buffer) {
    resize(state, buffer, {floats});
    if (!isContiguous(erase(buffer))) error("%s tensor has to be contiguous", name);
    if (launch::aligned16(data(buffer))) return data(buffer);
    // a buffer tensor at an odd storage offset: its contents are unspecified anyway, work in a temporary
  }
  tmp = Temp(state->stream, (size_t)floats * sizeof(float));
  return (float *)tmp.get();
}

// ---- pointwise forward -------------------------------------------------------------------------
// Launch shape of convPointwiseKernel for an M x K weight matrix: rows per wave, waves along the rows, column
// tiles per chunk, waves per workgroup.
struct PwShape {
  int mr, wr, ct, nw;
};
// K: 32 / 64 / 128. One workgroup of 8 waves per CU; a chunk of positions is 64 KB of x (CT = 512 / K column
// tiles), two of them in LDS. Measured against the tiled GEMM on the 1x1 layers of MobileNet-v1 and ResNet-50
// (N = 32 ... 64): 10-20 % faster at 56 x 56 and 112 x 112 (128 -> 128: 84 -> 70 us, 64 -> 128: 55 -> 45 us,
// 64 -> 256: 53 -> 43 us), level at 28 x 28. Left to the tiled GEMM because they measured slower here: K = 256
// (128 registers of weights per lane leave one wave per SIMD) and outputs of 32 rows or fewer.
bool pwShape(int M, int K, PwShape *sh) {
  if (K != 32 && K != 64 && K != 128) return false;
  const int ct = 512 / K;
  if (M >= 256 && K <= 64)
    *sh = {2, 4, ct, 8};  // 256 rows per workgroup, K registers of weights per lane (beyond K = 64 they would spill)
  else if (M > 64)
    *sh = {1, 4, ct, 8};  // 128 rows, two waves along the positions
  else if (M > 32)
    *sh = {1, 2, ct, 8};  // 64 rows, four waves along the positions
  else
    return false;
  return true;
}

template <int K, int MR, int WR, int CT, int NW, bool RELU, bool TRANS>
void launchPointwiseShape(hipStream_t s, PwArgs p, int device) {
  constexpr size_t lds = (size_t)pwLdsFloats(K, MR, WR, CT) * sizeof(float);
  auto kernel = convPointwiseKernel<K, MR, WR, CT, NW, RELU, TRANS>;
  if (lds > 64 * 1024) {  // once per kernel instance and device: allow more than 64 KB of dynamic LDS
    static std::atomic<bool> raised[64];
    if (!raised[device].load()) {
      THC_HIP_CHECK(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
      raised[device].store(true);
    }
  }
  const int rowsPerWg = 32 * MR * WR;
  const int rowBlocks = launch::ceilDiv(p.M, rowsPerWg);
  // one workgroup per CU (two of the 4-wave shapes), shared between the row blocks; each streams a run of column tiles
  int slots = std::max(1, residentSlots(nullptr) / rowBlocks);  // every shape fills a CU with one workgroup
  if (g_switches.convPointwise > 1) slots = std::min(slots, g_switches.convPointwise);  // tests: long runs of tiles per workgroup
  p.tilesPerWg = launch::ceilDiv(p.nTiles, std::min(slots, p.nTiles));
  const int gx = launch::ceilDiv(p.nTiles, p.tilesPerWg);
  kernel<<<dim3(gx, rowBlocks), 64 * NW, lds, s>>>(p);
  THC_HIP_CHECK(hipGetLastError());
}

// out(N, M, L) = bias + W(M x K) x(N, K, L) on the weight-stationary kernel; false: the shape is not one of its.
// transW: w holds (K x M) and its transpose is what multiplies (the gradInput pass hands over the layer's weights).
bool convPointwise(THCState *state, const ConvGeom &g, const float *x, const float *w, const float *bias, float *out,
                   bool relu = false, bool transW = false) {
  if (forceGeneric() || g_switches.convPointwise == 0) return false;
  if (g.kH != 1 || g.kW != 1 || g.dH != 1 || g.dW != 1 || g.padH != 0 || g.padW != 0) return false;
  const long P = (long)g.N * g.L;
  PwShape sh;
  if (g.L % 4 != 0 || g.Cout % 8 != 0 || P < 32 || !pwShape(g.Cout, g.K, &sh)) return false;
  // Short runs: with fewer than three chunks per workgroup the pipeline (chunk c multiplied, c + 1 in registers,
  // c + 2 in flight) never fills; chunks of half the size do better there (128 -> 128 at 28 x 28, N = 64, 7 column
  // tiles per workgroup: 28.2 -> 24.7 us, the tiled GEMM 25.8; at 56 x 56, 25 tiles per workgroup: 70 -> 76 us).
  if (g.K == 128 && sh.wr == 4) {
    const int rowBlocks = launch::ceilDiv(g.Cout, 32 * sh.mr * sh.wr);
    const int slots = std::max(1, residentSlots(nullptr) / rowBlocks);
    const long perWg = (((P + 31) / 32) + slots - 1) / slots;
    if (perWg < 5 * sh.ct) sh.ct = 2;
  }
  if (!launch::aligned16(x) || !launch::aligned16(w) || !launch::aligned16(out)) return false;
  // 32-bit byte offsets into x and out; the reciprocal division of a position by L is exact while P * L < 2^32
  if (P * g.K * 4 >= 0x7fffffffL || P * g.Cout * 4 >= 0x7fffffffL || P * g.L >= 0xffffffffL) return false;
  int device = 0;
  THC_HIP_CHECK(hipGetDevice(&device));
  if (device < 0 || device >= 64) return false;
  PwArgs p{};
  p.w = w, p.x = x, p.out = out, p.bias = bias;
  p.M = g.Cout, p.L = g.L, p.P = (int)P;
  p.nTiles = (int)((P + 31) / 32);
  p.magicL = dev::magicOf(g.L);
  p.xBytes = (int)(P * g.K * 4), p.outBytes = (int)(P * g.Cout * 4);
  hipStream_t s = state->stream;
#define PW_CASE(KK, MRR, WRR, CTT, NWW)                                              \
  if (g.K == KK && sh.mr == MRR && sh.wr == WRR && sh.ct == CTT && sh.nw == NWW) {   \
    if (transW)                                                                      \
      launchPointwiseShape<KK, MRR, WRR, CTT, NWW, false, true>(s, p, device);       \
    else if (relu)                                                                   \
      launchPointwiseShape<KK, MRR, WRR, CTT, NWW, true, false>(s, p, device);       \
    else                                                                             \
      launchPointwiseShape<KK, MRR, WRR, CTT, NWW, false, false>(s, p, device);      \
    return true;                                                                     \
  }
  PW_CASE(32, 2, 4, 16, 8) PW_CASE(32, 1, 4, 16, 8) PW_CASE(32, 1, 2, 16, 8)
  PW_CASE(64, 2, 4, 8, 8) PW_CASE(64, 1, 4, 8, 8) PW_CASE(64, 1, 2, 8, 8)
  PW_CASE(128, 1, 4, 4, 8) PW_CASE(128, 1, 2, 4, 8) PW_CASE(128, 1, 4, 2, 8)
#undef PW_CASE
  return false;
}

// ---- the three passes on raw device pointers -------------------------------------------------
// `scratchBuf` is the caller's buffer tensor (columns / gradColumns) or null; its contents are
// unspecified afterwards.

// out(N, Cout, oH, oW) = bias + conv(x(N, Cin, H, W), w(Cout, K))
// relu: out = Threshold(0, 0) of that, applied as the values are stored
void convForward(THCState *state, const ConvGeom &g, const float *x, const float *w, const float *bias, float *out,
                 THCudaTensor *scratchBuf, const char *bufName, bool relu = false) {
  if ((long)g.N * g.Cout == 0) return;
  if (convPointwise(state, g, x, w, bias, out, relu)) return;
  hipStream_t s = state->stream;
  // images per launch so that the flat column index n*L + l fits an int
  int group = (int)std::min<long>(g.N, std::max<long>(1, 0x7fffffffL / 2 / g.L));
  const long imgBytes = (long)g.Cin * (g.H + 2 * g.padH) * (g.W + 2 * g.padW) * sizeof(float);  // with its zero border
  const bool implicit2 = !forceGeneric() && imgBytes < (1L << 30);
  if (implicit2) group = (int)std::min<long>(group, std::max<long>(1, ((1L << 31) - 1 - 4096) / imgBytes));
  if (implicit2) {
    FwdPlan pl = planFwdImplicit(g.Cout, std::min(group, g.N), g, launch::aligned16(w));
    long need = pl.scratchFloats;  // the last, smaller group may split differently
    if (g.N % group != 0) need = std::max(need, planFwdImplicit(g.Cout, g.N % group, g, launch::aligned16(w)).scratchFloats);
    Temp tmp;
    float *scratch = scratchFloats(state, scratchBuf, need, tmp, bufName);
    for (int n0 = 0; n0 < g.N; n0 += group) {
      int cnt = std::min(group, g.N - n0);
      if (cnt != std::min(group, g.N)) pl = planFwdImplicit(g.Cout, cnt, g, launch::aligned16(w));
      launchFwdImplicit(s, pl, scratch, w, x + (long)n0 * g.Cin * g.H * g.W, out + (long)n0 * g.Cout * g.L, bias, g.Cout,
                        cnt, g, relu);
    }
    return;
  }
  for (int n0 = 0; n0 < g.N; n0 += group) {
    int cnt = std::min(group, g.N - n0);
    GemmArgs p{};
    p.a = w;
    p.b = x;
    p.c = out;
    p.bias = bias;
    p.M = g.Cout;
    p.Ncols = cnt * g.L;
    p.R = g.K;
    p.n0 = n0;
    p.nImages = cnt;
    p.mTiles = (int)tiles(p.M, BM);
    p.vecA = (g.K % 4 == 0) && launch::aligned16(p.a);
    dim3 grid(p.mTiles * tiles(p.Ncols, BN), 1);
    convGemmKernel<kForward><<<grid, dev::kBlock, 0, s>>>(p, g);
    THC_HIP_CHECK(hipGetLastError());
  }
  if (relu) reluInPlace(s, out, (long)g.N * g.Cout * g.L);  // the first-generation kernel has no such epilogue
}

// Taps and gy indices of phase ph along one axis (see PhaseAxis).
PhaseAxis phaseAxis(int ph, int size, int pad, int k, int dil, int stride) {
  PhaseAxis a{};
  a.n = ph < size ? (size - ph + stride - 1) / stride : 0;
  const int d = std::gcd(dil, stride);
  a.kStep = stride / d, a.qStep = dil / d;
  for (int kk = 0; kk < std::min(k, a.kStep); ++kk) {  // kk * dil = ph + pad (mod stride) has period stride / d in kk
    const int v = ph + pad - kk * dil;
    if (((v % stride) + stride) % stride == 0) {
      a.k0 = kk, a.nk = (k - 1 - kk) / a.kStep + 1, a.q0 = v / stride;
      break;
    }
  }
  return a;
}

// gradInput (and the transposed convolution's forward pass) for any stride, padding and dilation:
// per phase of gi a stride-1 convolution of the zero-bordered gradOutput with the phase's sub-kernel,
// on the forward kernels. No gradient columns reach memory and no multiply is spent on the zeros a
// strided convolution's transpose is full of. Returns false when the geometry is outside the 32-bit
// offsets of those kernels (the caller then takes the column path).
bool gradInputByPhase(THCState *state, const ConvGeom &g, const float *gy, const float *w, float *gi,
                      THCudaTensor *scratchBuf, const char *bufName, const float *bias) {
  if ((long)g.dH * g.dW > kMaxPhases) return false;
  hipStream_t s = state->stream;
  PhaseSet set{};
  int lowH = 0, highH = g.oH - 1, lowW = 0, highW = g.oW - 1;  // gy rows / columns the phases touch
  long wTotal = 0, tapTotal = 0, maxL = 1;
  for (int ph = 0; ph < g.dH; ++ph)
    for (int pw = 0; pw < g.dW; ++pw) {
      Phase P{};
      P.h = phaseAxis(ph, g.H, g.padH, g.kH, g.dilH, g.dH);
      P.w = phaseAxis(pw, g.W, g.padW, g.kW, g.dilW, g.dW);
      if (P.h.n == 0 || P.w.n == 0) continue;
      P.h0 = ph, P.w0 = pw;
      const long K = (long)g.Cout * P.h.nk * P.w.nk;
      if (K >= 0x7fffffffL / 8) return false;
      P.K = (int)K;
      P.Kp = std::max(BK, launch::ceilDiv(P.K, BK) * BK);
      if (P.K > 0) {
        lowH = std::min(lowH, P.h.q0 - (P.h.nk - 1) * P.h.qStep), highH = std::max(highH, P.h.n - 1 + P.h.q0);
        lowW = std::min(lowW, P.w.q0 - (P.w.nk - 1) * P.w.qStep), highW = std::max(highW, P.w.n - 1 + P.w.q0);
      }
      maxL = std::max(maxL, (long)P.h.n * P.w.n);
      set.ph[set.count++] = P;
    }
  if (set.count == 0) return true;  // gi has no elements
  // heaviest phase first: its workgroups are dispatched first
  std::stable_sort(set.ph, set.ph + set.count, [](const Phase &a, const Phase &b) { return a.Kp > b.Kp; });
  for (int i = 0; i < set.count; ++i) {
    Phase &P = set.ph[i];
    P.tapOfs = (int)tapTotal, tapTotal += P.Kp + 2 * BK;
    P.wOfs = wTotal, wTotal += (long)g.Cin * P.Kp;
  }
  const int top = -lowH, left = -lowW;
  const long Hp = (long)highH + 1 + top, Wp = (long)highW + 1 + left;
  const long imgFloats = (long)g.Cout * Hp * Wp;
  if (imgFloats * 4 >= (1L << 30) || wTotal * 4 >= 0x7fffffffL || tapTotal >= 0x7fffffffL / 8 ||
      launch::ceilDiv(Hp * Wp, (long)dev::kBlock) > 65535)
    return false;
  const bool copy = top > 0 || left > 0 || Hp != g.oH || Wp != g.oW || !launch::aligned16(gy);
  int group = (int)std::min<long>(g.N, std::max<long>(1, 0x7fffffffL / 2 / maxL));
  group = (int)std::min<long>(group, std::max<long>(1, ((1L << 31) - 1 - 4096) / (imgFloats * 4)));

  // All phases of a group of images run as one batched launch. The phases differ in K; the heavier ones are
  // split along K so that a workgroup reduces about the same number of k-tiles whatever its phase and the
  // grid holds about two workgroups per CU. Split phases leave partial tiles for the batched fold.
  const bool wide = tiles(g.Cin, 64) * 64 < tiles(g.Cin, BM) * BM;
  const bool low = tiles(g.Cin, 32) * 32 * 4 <= tiles(g.Cin, 64) * 64 * 3;  // as in planTiles
  const int bm = low ? 32 : wide ? 64 : BM, bn = low || wide ? 256 : BN;
  const int mTiles = (int)tiles(g.Cin, bm);
  struct Split {
    int tiles, tail, nSplit, ktPerSplit;  // the last `tail` of the item's tiles are split nSplit ways
    long partialOfs;
  } split[kMaxPhases];
  long partialTotal = 0;
  auto planAll = [&](int cnt) {
    const int cus = residentSlots(nullptr);
    long units = 0, wgs = 0;
    for (int i = 0; i < set.count; ++i) {
      const Phase &P = set.ph[i];
      split[i].tiles = mTiles * (int)tiles((long)cnt * P.h.n * P.w.n, bn);
      units += (long)split[i].tiles * (P.Kp / BK);
    }
    const long target = std::max<long>(4, units / (2L * cus));  // k-tiles per workgroup
    bool anySplit = false;
    for (int i = 0; i < set.count; ++i) {
      const int nkt = set.ph[i].Kp / BK;
      const int n = (int)std::max<long>(1, std::min<long>(nkt / 4, (nkt + target / 2) / target));
      split[i].ktPerSplit = launch::ceilDiv(nkt, n);
      split[i].nSplit = launch::ceilDiv(nkt, split[i].ktPerSplit);
      split[i].tail = split[i].nSplit > 1 ? split[i].tiles : 0;
      anySplit = anySplit || split[i].nSplit > 1;
      wgs += split[i].tiles;
    }
    // No phase is heavy enough to be split by that rule, and the whole tiles fill the CUs once or more with a
    // partial round left over (4 equal phases of a 4x4 stride-2 layer: 392 tiles on 256 CUs): the tiles of that
    // last round - the end of the launch order - are split along K like the tail of a single forward pass
    // (planTiles: same cost model, the k-tiles of the heaviest phase in the tail).
    const int q = (int)(wgs / cus), r = (int)(wgs % cus);
    if (!anySplit && q > 0 && r > 0) {
      int first = set.count - 1;  // first item with tiles in the tail
      for (int left = r; first > 0 && left > split[first].tiles; --first) left -= split[first].tiles;
      const int nktTail = set.ph[first].Kp / BK, nktHead = set.ph[0].Kp / BK;
      auto perWg = [&](int nkt, int S) { return (double)launch::ceilDiv(nkt, S) + 4.0; };
      double best = 0.95 * (q + 1) * perWg(nktHead, 1);
      int S = 1;
      for (int c = 2; c <= std::max(1, std::min(nktTail / 4, 16)); ++c) {
        if (launch::ceilDiv(nktTail, launch::ceilDiv(nktTail, c)) != c) continue;
        const double t = q * perWg(nktHead, 1) + launch::ceilDiv(r * c, cus) * perWg(nktTail, c) + 0.006 * r * c;
        if (t < best) best = t, S = c;
      }
      if (S > 1) {
        int left = r;
        for (int i = set.count - 1; i >= 0 && left > 0; --i) {
          const int nkt = set.ph[i].Kp / BK;
          split[i].tail = std::min(left, split[i].tiles);
          left -= split[i].tail;
          split[i].ktPerSplit = launch::ceilDiv(nkt, std::min(S, std::max(1, nkt / 4)));
          split[i].nSplit = launch::ceilDiv(nkt, split[i].ktPerSplit);
          if (split[i].nSplit <= 1) split[i].tail = 0;
        }
      }
    }
    long total = 0;
    for (int i = 0; i < set.count; ++i) {
      split[i].partialOfs = total;
      total += (long)split[i].tail * split[i].nSplit * BM * BN;
    }
    partialTotal = std::max(partialTotal, total);
  };
  if (g.N % group != 0) planAll(g.N % group);  // the last, smaller group may split differently
  planAll(std::min(group, g.N));
  const long paddedFloats = copy ? (group * imgFloats + 3) / 4 * 4 : 0;
  Temp tmp;
  float *buf = scratchFloats(state, scratchBuf, tapTotal + wTotal + partialTotal + paddedFloats, tmp, bufName);
  int *taps = reinterpret_cast<int *>(buf);
  float *wph = buf + tapTotal;
  float *partial = wph + wTotal;
  float *gyp = partial + partialTotal;
  int maxKp = 0;
  for (int i = 0; i < set.count; ++i) maxKp = std::max(maxKp, set.ph[i].Kp);
  if (g.Cin + 1 > 65535) return false;
  const int chunks = std::max(1, std::min(8, launch::ceilDiv(maxKp + 2 * BK, 4 * dev::kBlock)));
  // the set-up rides along with the first group's bordered copy when that copy has the flat 16-byte form
  const long plane = Hp * Wp, firstTotal4 = (long)std::min(group, g.N) * g.Cout * (plane / 4);
  const long setupBlocks = (long)chunks * (g.Cin + 1) * set.count;
  const bool together = copy && plane % 4 == 0 && plane < 4096 && launch::aligned16(gyp) &&
                        firstTotal4 * (plane / 4) < 0xffffffffL && setupBlocks < (1L << 24);
  if (!together) {
    phaseSetupKernel<<<dim3(chunks, g.Cin + 1, set.count), dev::kBlock, 0, s>>>(w, wph, taps, set, g.Cin, g.kH, g.kW, (int)Hp,
                                                                              (int)Wp, top, left);
    THC_HIP_CHECK(hipGetLastError());
  }
  for (int n0 = 0; n0 < g.N; n0 += group) {
    const int cnt = std::min(group, g.N - n0);
    if (cnt != std::min(group, g.N)) planAll(cnt);
    const float *src = gy + (long)n0 * g.Cout * g.L;
    if (copy && together && n0 == 0) {
      const int copyBlocks = (int)std::min<long>((firstTotal4 + dev::kBlock - 1) / dev::kBlock, 16384);
      padPlanesPhaseSetupKernel<<<(unsigned)(copyBlocks + setupBlocks), dev::kBlock, 0, s>>>(
          src, gyp, g.oH, g.oW, (int)Hp, (int)Wp, top, left, firstTotal4, copyBlocks, w, wph, taps, set, g.Cin, g.kH, g.kW, chunks);
      THC_HIP_CHECK(hipGetLastError());
      src = gyp;
    } else if (copy) {
      launchPadPlanes(s, src, gyp, (long)cnt * g.Cout, g.oH, g.oW, top, left, (int)Hp, (int)Wp);
      src = gyp;
    }
    FwdBatch batch{};
    batch.count = set.count;
    int maxTail = 0, wholeTotal = 0, splitTotal = 0;
    for (int i = 0; i < set.count; ++i) {
      const Phase &P = set.ph[i];
      FwdBatchItem &it = batch.item[i];
      ConvGeom &gk = it.g;  // what the forward kernel sees: a stride-1 pass over the bordered gy
      gk.N = cnt, gk.Cin = g.Cout, gk.Cout = g.Cin;
      gk.H = (int)Hp, gk.W = (int)Wp, gk.oH = P.h.n, gk.oW = P.w.n;
      gk.kH = gk.kW = gk.dH = gk.dW = gk.dilH = gk.dilW = 1;
      gk.K = P.Kp, gk.L = P.h.n * P.w.n;
      FwdArgs &a = it.p;
      a.w = wph + P.wOfs;
      a.x = src;
      a.taps = taps + P.tapOfs;
      a.bias = bias;
      a.M = g.Cin;
      a.Ncols = cnt * gk.L;
      a.out = gi + (long)n0 * g.Cin * g.H * g.W + (long)P.h0 * g.W + P.w0;
      a.outImg = (long)g.Cin * g.H * g.W, a.outRow = g.H * g.W, a.outSH = g.dH * g.W, a.outSW = g.dW;
      {
        const long span = ((long)(cnt - 1) * a.outImg + (long)(g.Cin - 1) * a.outRow + (long)(P.h.n - 1) * a.outSH +
                           (long)(P.w.n - 1) * a.outSW + 1) * 4;
        a.outBytes = span < 0x7fffffffL ? (int)span : 0;
        a.magicL = (long)a.Ncols * gk.L < 0xffffffffL ? dev::magicOf(gk.L) : 0;
        a.magicOW = (long)gk.L * gk.oW < 0xffffffffL ? dev::magicOf(gk.oW) : 0;
      }
      a.xBytes = (int)(cnt * imgFloats * 4);
      a.wBytes = (int)((long)g.Cin * P.Kp * 4);
      a.vecA = true;
      a.mTiles = mTiles, a.bm = bm, a.bn = bn;
      a.tail = split[i].tail, a.full = split[i].tiles - split[i].tail;
      a.tile0 = a.full;
      a.nSplit = a.tail > 0 ? split[i].nSplit : 1;
      a.ktPerSplit = a.tail > 0 ? split[i].ktPerSplit : P.Kp / BK;
      a.partial = partial + split[i].partialOfs;
      wholeTotal += a.full, splitTotal += a.tail * a.nSplit;
      it.wholeEnd = wholeTotal, it.splitEnd = splitTotal;
      maxTail = std::max(maxTail, a.tail);
    }
    batch.wholeTotal = wholeTotal;
    const dim3 grid(wholeTotal + splitTotal);
    if (low)
      convFwdPaddedBatchKernel<0><<<grid, dev::kBlock, 0, s>>>(batch);
    else if (wide)
      convFwdPaddedBatchKernel<1><<<grid, dev::kBlock, 0, s>>>(batch);
    else
      convFwdPaddedBatchKernel<2><<<grid, dev::kBlock, 0, s>>>(batch);
    THC_HIP_CHECK(hipGetLastError());
    if (maxTail > 0) {
      fwdTailFixupBatchKernel<<<dim3(maxTail, BM * BN / (4 * dev::kBlock), set.count), dev::kBlock, 0, s>>>(batch);
      THC_HIP_CHECK(hipGetLastError());
    }
  }
  return true;
}

// ---- gradInput with one to four input planes (conv_fewplanes.h) ----
template <int S, int T, int KC, int PADC>
void launchFewPlanes(hipStream_t s, FpArgs a, const FpTaps &tp, const ConvGeom &g) {
  using Sh = FpShape<S, T, KC, PADC>;
  const int PR = (g.H + S - 1) / S, PC = (g.W + S - 1) / S;  // phase positions per image
  a.tilesR = (int)tiles(PR, 4 * T), a.tilesC = (int)tiles(PC, 16);
  a.magicTiles = dev::magicOf(a.tilesR * a.tilesC), a.magicTilesC = dev::magicOf(a.tilesC);
  const int RR = Sh::CT ? Sh::RR : a.RR;
  const int KKP = (g.kH * g.kW + 3) / 4 * 4;
  convFewPlanesGradInputKernel<S, T, KC, PADC>
      <<<g.N * a.tilesR * a.tilesC, 64 * kFpWaves, Sh::ldsBytes(RR, KKP), s>>>(a, tp);
  THC_HIP_CHECK(hipGetLastError());
}

// false: not a shape for this kernel (the caller goes on to the other routes)
bool convFewPlanesGradInput(THCState *state, const ConvGeom &g, const float *gy, const float *w, float *gi,
                            const float *bias, bool runtimeOnly) {
  const int S = g.dH;
  if (g.Cin > 4 || g.dilH != 1 || g.dilW != 1 || g.dH != g.dW || S > 4 || g.padH < 0 || g.padW < 0) return false;
  if ((long)g.Cout * g.L * 4 >= (1L << 31) || (long)g.Cin * g.H * g.W * 4 >= (1L << 31) || (long)g.Cout * g.K * 4 >= (1L << 31))
    return false;
  FpArgs a{};
  FpTaps tp{};
  a.gy = gy, a.w = w, a.bias = bias, a.gi = gi;
  a.Cin = g.Cin, a.Cout = g.Cout, a.H = g.H, a.W = g.W, a.oH = g.oH, a.oW = g.oW, a.kH = g.kH, a.kW = g.kW;
  a.magicCK = dev::magicOf(g.Cin * g.kH * g.kW), a.magicKK = dev::magicOf(g.kH * g.kW);
  const int PR = (g.H + S - 1) / S, PC = (g.W + S - 1) / S;
  const int Tg = S <= 2 ? 4 : S == 3 ? 2 : 1;  // rows per lane of the run-time variant
  {  // block numbering: n * tiles + tile must divide back exactly
    const long tl = tiles(PR, 4) * tiles(PC, 16);  // at most this many blocks per image (T >= 1)
    if ((long)g.N * tl >= (1L << 31) || (double)g.N * tl * tl >= 4294967296.0) return false;
  }
  hipStream_t s = state->stream;
  const bool square = g.kH == g.kW && g.padH == g.padW;
  const int k = g.kH, pad = g.padH;
  if (square && !runtimeOnly) {
#define FEW_PLANES_SHAPE(S_, T_, K_, P_)                  \
  if (S == S_ && k == K_ && pad == P_) {                  \
    launchFewPlanes<S_, T_, K_, P_>(s, a, tp, g);         \
    return true;                                          \
  }
    FEW_PLANES_SHAPE(2, 4, 7, 3)   // 7x7 stride 2: the first layer of ResNet / Inception-v1
    FEW_PLANES_SHAPE(2, 4, 3, 1)   // 3x3 stride 2: MobileNet
    FEW_PLANES_SHAPE(2, 4, 3, 0)   // 3x3 stride 2, unpadded: Inception-v3
    FEW_PLANES_SHAPE(1, 8, 3, 1)   // 3x3: VGG
    FEW_PLANES_SHAPE(1, 8, 5, 2)   // 5x5
    FEW_PLANES_SHAPE(2, 4, 4, 1)   // 4x4 stride 2: the transposed convolutions of a generator
    FEW_PLANES_SHAPE(4, 2, 11, 2)  // 11x11 stride 4: AlexNet
#undef FEW_PLANES_SHAPE
  }
  // any other kernel size / padding: tap loops with run-time bounds
  if (g.kH * g.kW > kFpMaxTaps) return false;
  auto fill = [&](FpDim &d, int kk, int pd) {
    d.lo = fpLo(pd, S, kk), d.hi = fpHi(pd, S, kk);
    for (int ph = 0; ph < S; ++ph) d.rem[ph] = fpRem(ph, pd, S), d.q0[ph] = fpQ0(ph, pd, S), d.taps[ph] = fpTaps(ph, pd, S, kk);
  };
  fill(a.dh, g.kH, g.padH);
  fill(a.dw, g.kW, g.padW);
  a.RR = 4 * Tg + a.dh.hi - a.dh.lo, a.CC = 16 + a.dw.hi - a.dw.lo;
  a.magicCC = dev::magicOf(a.CC);
  const int pitch = Tg == 4 ? 28 : Tg == 2 ? 24 : 48;
  if (a.CC > pitch || a.RR * a.CC > 64 * kFpMaxLoads || 2 * g.Cin * g.kH * g.kW > 64 * kFpMaxWLoads ||
      a.RR * pitch >= 65536)
    return false;
  int cnt = 0;
  for (int ph = 0; ph < S; ++ph)
    for (int pw = 0; pw < S; ++pw) {
      tp.first[ph * S + pw] = cnt;
      for (int ta = 0; ta < a.dh.taps[ph]; ++ta)
        for (int tb = 0; tb < a.dw.taps[pw]; ++tb) {
          const unsigned tap = (a.dh.rem[ph] + ta * S) * g.kW + a.dw.rem[pw] + tb * S;
          const unsigned off = (a.dh.q0[ph] - ta - a.dh.lo) * pitch + (a.dw.q0[pw] - tb - a.dw.lo);
          tp.e[cnt++] = tap | off << 16;
        }
    }
  for (int q = S * S; q <= 16; ++q) tp.first[q] = cnt;
  switch (S) {
    case 1: launchFewPlanes<1, 4, 0, 0>(s, a, tp, g); break;
    case 2: launchFewPlanes<2, 4, 0, 0>(s, a, tp, g); break;
    case 3: launchFewPlanes<3, 2, 0, 0>(s, a, tp, g); break;
    default: launchFewPlanes<4, 1, 0, 0>(s, a, tp, g); break;
  }
  return true;
}

// gi(N, Cin, H, W) = conv^T(gy(N, Cout, oH, oW), w(Cout, K))
// + bias[c] per plane of gi when bias != null (the transposed convolution's forward pass)
void convGradInput(THCState *state, const ConvGeom &g, const float *gy, const float *w, float *gi,
                   THCudaTensor *scratchBuf, const char *bufName, const float *bias = nullptr) {
  if ((long)g.N * g.Cin == 0) return;
  hipStream_t s = state->stream;
  // Stride 1: gradInput is a forward convolution of gradOutput with the flipped,
  // transposed weights and padding dil*(k-1)-pad, so it runs on the implicit-GEMM
  // forward kernel and no gradient columns ever reach memory.
  const int tpH = g.dilH * (g.kH - 1) - g.padH, tpW = g.dilW * (g.kW - 1) - g.padW;
  const long goImgBytes = (long)g.Cout * (g.oH + 2 * std::max(tpH, 0)) * (g.oW + 2 * std::max(tpW, 0)) * sizeof(float);  // with its zero border
  // (with stride 1 the extents correspond exactly unless a transposed convolution asks for output padding)
  const bool exact = g.H == g.oH + 2 * tpH - g.dilH * (g.kH - 1) && g.W == g.oW + 2 * tpW - g.dilW * (g.kW - 1);
  // (one to four input planes - the first layer of a network - would fill a sixteenth of the 64-row tiles of that
  // GEMM: 1.08 ms for 3 -> 64 planes 3x3 at 224x224, N = 32; the column GEMM below has K = Cin * kH * kW rows)
  const bool sliver = g.Cin <= 4 && g.kH * g.kW > 1;
  const int route = g_switches.convGradInput;  // 1: phases, 2: columns, 3: few-plane kernel with run-time tap loops
  if (g.Cin <= 4 && (g.kH * g.kW > 1 || g.dH > 1 || g.dW > 1) && !forceGeneric() && (route == 0 || route == 3) &&
      convFewPlanesGradInput(state, g, gy, w, gi, bias, route == 3))
    return;
  // 1x1 window, stride 2, no padding, even extents (the shortcut and reduction layers of a residual network):
  // gradInput is W^T gradOutput at the even positions and the bias (or 0) everywhere else. One pointwise pass of
  // the forward kernels over gradOutput whose epilogue writes each element's whole 2 x 2 block - contiguous
  // 8-byte stores - instead of four phases that each write every other element of every other row.
  if (g.kH == 1 && g.kW == 1 && g.dH == 2 && g.dW == 2 && g.padH == 0 && g.padW == 0 && g.H == 2 * g.oH && g.W == 2 * g.oW &&
      route == 0 && !forceGeneric() && ((uintptr_t)gi & 7) == 0 && (long)g.Cout * g.oH * g.oW * 4 < (1L << 30) &&
      (long)g.Cout * g.K < 0x7fffffffL / 4) {
    ConvGeom t = g;
    t.Cin = g.Cout, t.Cout = g.Cin;
    t.H = t.oH = g.oH, t.W = t.oW = g.oW;
    t.dH = t.dW = 1;
    t.K = g.Cout;
    t.L = g.oH * g.oW;
    OutMap om{(long)g.Cin * g.H * g.W, g.H * g.W, 2 * g.W, 2, 1};
    int group = (int)std::min<long>(g.N, std::max<long>(1, 0x7fffffffL / 2 / t.L));
    group = (int)std::min<long>(group, std::max<long>(1, ((1L << 31) - 1 - 4096) / ((long)g.Cout * t.L * 4)));
    FwdPlan pl = planFwdImplicit(t.Cout, std::min(group, g.N), t);
    long need = pl.scratchFloats;
    if (g.N % group != 0) need = std::max(need, planFwdImplicit(t.Cout, g.N % group, t).scratchFloats);
    const long wfFloats = ((long)g.Cout * g.K + 3) / 4 * 4;
    Temp tmp;
    float *buf = scratchFloats(state, scratchBuf, wfFloats + need, tmp, bufName);
    flipWeightKernel<<<launch::directGrid((long)g.Cout * g.K, dev::kBlock), dev::kBlock, 0, s>>>(w, buf, g.Cout, g.Cin, 1, 1);
    THC_HIP_CHECK(hipGetLastError());
    for (int n0 = 0; n0 < g.N; n0 += group) {
      int cnt = std::min(group, g.N - n0);
      if (cnt != std::min(group, g.N)) pl = planFwdImplicit(t.Cout, cnt, t);
      launchFwdImplicit(s, pl, buf + wfFloats, buf, gy + (long)n0 * g.Cout * g.L, gi + (long)n0 * g.Cin * g.H * g.W, bias,
                        t.Cout, cnt, t, false, &om);
    }
    return;
  }
  if (g.dH == 1 && g.dW == 1 && tpH >= 0 && tpW >= 0 && exact && !sliver && !forceGeneric() && goImgBytes < (1L << 30) &&
      (long)g.Cout * g.K < 0x7fffffffL / 4) {
    ConvGeom t = g;  // the transposed problem
    t.Cin = g.Cout, t.Cout = g.Cin;
    t.H = g.oH, t.W = g.oW, t.oH = g.H, t.oW = g.W;
    t.padH = tpH, t.padW = tpW;
    t.K = g.Cout * g.kH * g.kW;
    t.L = g.H * g.W;
    int group = (int)std::min<long>(g.N, std::max<long>(1, 0x7fffffffL / 2 / t.L));
    group = (int)std::min<long>(group, std::max<long>(1, ((1L << 31) - 1 - 4096) / goImgBytes));
    FwdPlan pl = planFwdImplicit(t.Cout, std::min(group, g.N), t);
    long need = pl.scratchFloats;
    if (g.N % group != 0) need = std::max(need, planFwdImplicit(t.Cout, g.N % group, t).scratchFloats);
    // 1x1: gradInput = W^T gradOutput, a pointwise pass itself, which reads the weights as they are
    if (convPointwise(state, t, gy, w, bias, gi, false, true)) return;
    const long wfFloats = ((long)g.Cout * g.K + 3) / 4 * 4;
    Temp tmp;
    float *buf = scratchFloats(state, scratchBuf, wfFloats + need, tmp, bufName);
    const FlipJob flip{w, buf, g.Cout, g.Cin, g.kH, g.kW};  // done by the first group's bordered copy, or by a launch of its own
    for (int n0 = 0; n0 < g.N; n0 += group) {
      int cnt = std::min(group, g.N - n0);
      if (cnt != std::min(group, g.N)) pl = planFwdImplicit(t.Cout, cnt, t);
      launchFwdImplicit(s, pl, buf + wfFloats, buf, gy + (long)n0 * g.Cout * g.L, gi + (long)n0 * g.Cin * g.H * g.W,
                        bias, t.Cout, cnt, t, false, nullptr, n0 == 0 ? &flip : nullptr);
    }
    return;
  }
  // Every other geometry goes phase by phase (with 32-row tiles that measured faster than the gradient columns
  // below down to 8 input planes: 8 -> 16 3x3 stride 2 at 128x128, N = 32: 37 against 62 us); the columns remain for
  // what that route refuses and for the test switch THCUNN_CONV_GRADINPUT = "columns".
  const bool tryPhases = route != 2;
  if (!forceGeneric() && tryPhases && gradInputByPhase(state, g, gy, w, gi, scratchBuf, bufName, bias)) return;
  // Gradient columns of a group of images at a time (<= 128 MB so the buffer stays cache resident), then
  // the col2im gather. gradCol[n][k][l] = sum_o W[o][k] * gy[n][o][l] is itself a 1x1 convolution of gy
  // with the transposed weights, so it runs on the forward kernels as well.
  const long perImg = (long)g.K * g.L;
  int group = (int)std::max<long>(1, std::min<long>(g.N, (128L << 20) / 4 / perImg));
  group = (int)std::min<long>(group, std::max<long>(1, 0x7fffffffL / 2 / g.L));
  const long gyImgBytes = (long)g.Cout * g.L * sizeof(float);
  const bool viaForward = !forceGeneric() && gyImgBytes < (1L << 30) && (long)g.Cout * g.K < 0x7fffffffL / 4;
  if (viaForward) group = (int)std::min<long>(group, std::max<long>(1, ((1L << 31) - 1 - 4096) / gyImgBytes));
  ConvGeom q{};  // the 1x1 convolution: (N, Cout, oH, oW) -> (N, K, oH, oW)
  q.N = g.N, q.Cin = g.Cout, q.Cout = g.K, q.H = q.oH = g.oH, q.W = q.oW = g.oW;
  q.kH = q.kW = q.dH = q.dW = q.dilH = q.dilW = 1;
  q.K = g.Cout, q.L = g.L;
  FwdPlan pl{};
  long wtFloats = 0;
  if (viaForward) {
    pl = planFwdImplicit(q.Cout, std::min(group, g.N), q);
    wtFloats = ((long)g.Cout * g.K + 3) / 4 * 4;
  }
  long need = pl.scratchFloats;
  if (viaForward && g.N % group != 0) need = std::max(need, planFwdImplicit(q.Cout, g.N % group, q).scratchFloats);
  const long fwdFloats = (need + 3) / 4 * 4;
  Temp tmp;
  float *buf = scratchFloats(state, scratchBuf, wtFloats + fwdFloats + (long)group * perImg, tmp, bufName);
  float *gcol = buf + wtFloats + fwdFloats;
  if (viaForward) {
    transposeKernel<<<launch::directGrid((long)g.Cout * g.K, dev::kBlock), dev::kBlock, 0, s>>>(w, buf, g.Cout, g.K);
    THC_HIP_CHECK(hipGetLastError());
  }
  for (int n0 = 0; n0 < g.N; n0 += group) {
    int cnt = std::min(group, g.N - n0);
    if (viaForward) {
      if (cnt != std::min(group, g.N)) pl = planFwdImplicit(q.Cout, cnt, q);
      launchFwdImplicit(s, pl, buf + wtFloats, buf, gy + (long)n0 * g.Cout * g.L, gcol, nullptr, q.Cout, cnt, q);
    } else {
      GemmArgs p{};
      p.a = w;
      p.b = gy;
      p.c = gcol;
      p.M = g.K;
      p.Ncols = cnt * g.L;
      p.R = g.Cout;
      p.n0 = n0;
      p.nImages = cnt;
      p.mTiles = (int)tiles(p.M, BM);
      dim3 grid(p.mTiles * tiles(p.Ncols, BN), 1);
      convGemmKernel<kGradCol><<<grid, dev::kBlock, 0, s>>>(p, g);
      THC_HIP_CHECK(hipGetLastError());
    }
    long total = (long)cnt * g.Cin * g.H * g.W;
    col2imKernel<<<launch::directGrid(total, dev::kBlock), dev::kBlock, 0, s>>>(
        gcol, gi + (long)n0 * g.Cin * g.H * g.W, cnt, g.Cin, g.H, g.W, g.kH, g.kW, g.padH, g.padW, g.dH, g.dW, g.dilH,
        g.dilW, g.oH, g.oW, bias);
    THC_HIP_CHECK(hipGetLastError());
  }
}

// gB[o] += scale * sum_{n,l} gy[n][o][l] over a (N, C, L) tensor
void convGradBias(hipStream_t s, const float *gy, float *gB, int N, int C, int L, float scale) {
  if ((long)N * C * L == 0) return;
  if (L % 4 == 0 && launch::aligned16(gy) && (long)N * (L / 4) < 0x7fffffffL)
    gradBiasKernel<true><<<C, kBiasBlock, 0, s>>>(gy, gB, N, C, L, scale);
  else
    gradBiasKernel<false><<<C, kBiasBlock, 0, s>>>(gy, gB, N, C, L, scale);
  THC_HIP_CHECK(hipGetLastError());
}

// gW(Cout, K) += scale * sum_n gy_n(Cout x L) * im2col(x_n)^T
// gB(Cout) += scale * sum_{n,l} gy when gB is given (the bias gradient of the ordinary convolution)
void convGradWeight(THCState *state, const ConvGeom &g, const float *x, const float *gy, float *gW,
                    THCudaTensor *scratchBuf, float scale, float *gB = nullptr) {
  if ((long)g.N * g.Cout * g.K == 0) return;
  hipStream_t s = state->stream;

  // Split the reduction over the N*L positions so that the grid fills the
  // resident workgroup slots of the chip exactly once: with fewer, fatter
  // splits some CUs would carry one workgroup more than others for the whole
  // kernel.
  // The second-generation kernel loads 4 consecutive positions of a gradOutput row as one 16-byte group. Rows
  // whose length is not a multiple of 4 (7x7, 13x13, 27x27 ... planes) or that start off a 16-byte boundary are
  // first copied into rows padded with zeros to a multiple of 4: the added positions contribute nothing (the
  // kernel lets them read position 0 of the image).
  const int Lp = launch::roundUp(g.L, 4);
  const bool padGy = !forceGeneric() && (g.L % 4 != 0 || !launch::aligned16(gy)) && Lp >= BK;
  const int Lk = padGy ? Lp : g.L;  // positions per image as the kernel sees them
  if ((long)g.N * Lk >= 0x7fffffffL) error("spatial convolution: batch too large");
  const int totalKt = launch::ceilDiv(g.N * Lk, BK);
  const int HpX = g.H + 2 * g.padH;
  // second-generation kernel: gradOutput rows loadable as float4 groups, 32-bit byte offsets into both operands
  const bool bordered = g.padH > 0 || g.padW > 0;
  const long gyBytes = (long)g.N * g.Cout * Lk * 4;
  const long xpFloats = (long)g.N * g.Cin * HpX * (g.W + 2 * g.padW);
  const long gypFloats = padGy ? (long)g.N * g.Cout * Lp : 0;
  const bool fast = !forceGeneric() && Lk % 4 == 0 && Lk >= BK && (padGy || launch::aligned16(gy)) &&
                    gyBytes < 0x7fffffffL && xpFloats * 4 < 0x7fffffffL - 65536 && (long)Lk * g.oW < 0x7fffffffL;
  const bool l16 = Lk % BK == 0;
  // tile shape: 64 x 256 where it covers gradWeight (Cout x K) with less padding than 128 x 128
  const bool wide = fast && tiles(g.Cout, 64) * 64 * tiles(g.K, 256) * 256 < tiles(g.Cout, BM) * BM * tiles(g.K, BN) * BN;
  // Small tiles (the waves of a workgroup split the positions instead of the tile; blocks of 32 rows x 32 columns:
  // 1x1, 1x2, 1x4, 2x1, 2x2) where the large shapes would mostly multiply padding. The shape is the one with
  // the least tiles x cost per tile and k-tile; the costs are measured (first layers, 32- and 64-plane layers at
  // 56x56 ... 149x149): the gather of the image patch weighs more than the matrix instructions, so a tile is not
  // cheaper in proportion to its area.
  struct Shape {
    int ti, tj, cost;
  };
  static const Shape kSmall[] = {{2, 2, 88}, {1, 4, 90}, {1, 2, 50}, {2, 1, 50}, {1, 1, 33}};
  const int kBigCost = 260;  // a 128 x 128 or 64 x 256 tile
  long bestCost = std::min(tiles(g.Cout, 64) * tiles(g.K, 256), tiles(g.Cout, BM) * tiles(g.K, BN)) * (long)kBigCost;
  int tI = 0, tJ = 0;
  if (fast)
    for (const Shape &sh : kSmall) {
      const long c = (long)tiles(g.Cout, 32 * sh.ti) * tiles(g.K, 32 * sh.tj) * sh.cost;
      if (c < bestCost) bestCost = c, tI = sh.ti, tJ = sh.tj;
    }
  const bool tiny = tI > 0;
  const int mT = (int)tiles(g.Cout, tiny ? 32 * tI : wide ? 64 : BM), nT = (int)tiles(g.K, tiny ? 32 * tJ : wide ? 256 : BN);
  struct TinyKernel {
    const void *fn;
    void (*launch)(dim3, hipStream_t, const GradWeightArgs &, const ConvGeom &);
  };
  auto tinyKernel = [&](auto l16c, auto tic, auto tjc) {
    constexpr bool L = decltype(l16c)::value;
    constexpr int I = decltype(tic)::value, J = decltype(tjc)::value;
    return TinyKernel{(const void *)convGradWeightKernel<L, 0, I, J>,
                      [](dim3 grid, hipStream_t st, const GradWeightArgs &q, const ConvGeom &gk) {
                        convGradWeightKernel<L, 0, I, J><<<grid, dev::kBlock, 0, st>>>(q, gk);
                      }};
  };
  auto pickTiny = [&](auto l16c) {
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I4 = std::integral_constant<int, 4>;
    if (tI == 1 && tJ == 1) return tinyKernel(l16c, I1{}, I1{});
    if (tI == 1 && tJ == 2) return tinyKernel(l16c, I1{}, I2{});
    if (tI == 1 && tJ == 4) return tinyKernel(l16c, I1{}, I4{});
    if (tI == 2 && tJ == 1) return tinyKernel(l16c, I2{}, I1{});
    return tinyKernel(l16c, I2{}, I2{});
  };
  const TinyKernel tk = l16 ? pickTiny(std::true_type{}) : pickTiny(std::false_type{});
  // 16-byte gathers of the image: unit stride along a row, and groups of 4 positions that stay inside an output row
  // (or output rows that follow each other in the image without a gap: kW = 1, no padding, unit stride down too)
  const bool b4 = fast && !tiny && !padGy && g.dW == 1 &&
                  (g.oW % 4 == 0 || (g.dH == 1 && g.W + 2 * g.padW == g.oW));
  struct BigKernel {
    const void *fn;
    void (*launch)(dim3, hipStream_t, const GradWeightArgs &, const ConvGeom &);
  };
  auto bigKernel = [](auto l16c, auto wmc, auto b4c) {
    constexpr bool L = decltype(l16c)::value, B = decltype(b4c)::value;
    constexpr int W = decltype(wmc)::value;
    return BigKernel{(const void *)convGradWeightKernel<L, W, 2, 2, B>,
                     [](dim3 grid, hipStream_t st, const GradWeightArgs &q, const ConvGeom &gk) {
                       convGradWeightKernel<L, W, 2, 2, B><<<grid, dev::kBlock, 0, st>>>(q, gk);
                     }};
  };
  auto pickBig = [&](auto l16c, auto wmc) { return b4 ? bigKernel(l16c, wmc, std::true_type{}) : bigKernel(l16c, wmc, std::false_type{}); };
  auto pickBigW = [&](auto l16c) {
    return wide ? pickBig(l16c, std::integral_constant<int, 1>{}) : pickBig(l16c, std::integral_constant<int, 2>{});
  };
  const BigKernel bk = l16 ? pickBigW(std::true_type{}) : pickBigW(std::false_type{});
  const void *kern = !fast ? (const void *)convGemmKernel<kGradWeight> : tiny ? tk.fn : bk.fn;
  // Every split leaves a partial copy of gradWeight (64 KB per tile) for the fold: three workgroups per CU
  // measured better than the four that fit (less partial traffic for the same matrix-pipe load), two when
  // gradWeight is one or two tiles and the partials are most of the traffic. The small tiles stream: as many
  // workgroups as fit, to have enough loads in flight.
  // A split should keep at least about 20 k-tiles (short reductions at 14x14 and 7x7: with 8 k-tiles per split the
  // partial copies and the pipeline fill cost more than the third workgroup per CU gains).
  int perCu = mT * nT <= 2 ? 2 : tiny ? 4 : 3;
  auto splitsAt = [&](int wgPerCu) {
    const int slots = std::min(residentSlots(kern), residentSlots(nullptr) * wgPerCu);
    return std::max(1, std::min(totalKt, slots / (mT * nT)));
  };
  while (perCu > 1 && totalKt / splitsAt(perCu) < 20) --perCu;
  int splits = splitsAt(perCu);
  const int perSplit = launch::ceilDiv(totalKt, splits);
  splits = launch::ceilDiv(totalKt, perSplit);
  const int wgSplits = splits;       // splits of the positions over workgroups
  if (tiny) splits *= 4;             // partial copies of gradWeight: one per wave
  const long count = (long)g.Cout * g.K;
  // scratch: the splits' partial products, then (second-generation kernel) the images with their zero border
  const long partialFloats = (splits * count + 3) / 4 * 4;
  // the bias gradient rides along when the fold below has the 16-byte form; else it is a pass of its own
  const bool fold4 = count % 4 == 0 && launch::aligned16(gW);
  const bool fusedBias = gB && fast && fold4 && g.Cout % 4 == 0 && launch::aligned16(gB);
  const long biasFloats = fusedBias ? ((long)splits * g.Cout + 3) / 4 * 4 : 0;
  Temp tmp;
  const long xpScratch = fast && bordered ? (xpFloats + 3) / 4 * 4 : 0;
  float *partial = scratchFloats(state, scratchBuf, partialFloats + biasFloats + xpScratch + (fast ? gypFloats : 0), tmp, "columns");
  float *biasPartial = fusedBias ? partial + partialFloats : nullptr;
  if (fast) {
    ConvGeom gk = g;
    const float *xk = x, *gyk = gy;
    if (bordered) {
      float *xp = partial + partialFloats + biasFloats;
      launchPadPlanes(s, x, xp, (long)g.N * g.Cin, g.H, g.W, g.padH, g.padW, HpX, g.W + 2 * g.padW);
      gk.H = HpX, gk.W = g.W + 2 * g.padW, gk.padH = gk.padW = 0;
      xk = xp;
    }
    if (padGy) {  // rows of L floats -> rows of Lp floats, zeros behind
      float *gyp = partial + partialFloats + biasFloats + xpScratch;
      launchPadPlanes(s, gy, gyp, (long)g.N * g.Cout, 1, g.L, 0, 0, 1, Lp);
      gk.L = Lp;
      gyk = gyp;
    }
    GradWeightArgs q{};
    q.gy = gyk;
    q.x = xk;
    q.partial = partial;
    q.biasPartial = biasPartial;
    q.M = g.Cout;
    q.Ncols = g.K;
    q.mTiles = mT;
    q.nTiles = nT;
    q.totalKt = totalKt;
    q.ktPerSplit = perSplit;
    q.gyBytes = (int)gyBytes;
    q.xBytes = (int)(xpFloats * 4);
    q.magicOW = dev::magicOf(g.oW);
    q.magicKK = dev::magicOf(g.kH * g.kW), q.magicKW = dev::magicOf(g.kW);
    q.Lvalid = g.L;
    const dim3 grid(mT * nT * wgSplits);
    if (tiny)
      tk.launch(grid, s, q, gk);
    else
      bk.launch(grid, s, q, gk);
  } else {
    GemmArgs p{};
    p.a = gy;
    p.b = x;
    p.c = partial;
    p.M = g.Cout;
    p.Ncols = g.K;
    p.R = 0;
    p.n0 = perSplit;
    p.nImages = g.N;
    p.mTiles = mT;
    p.vecA = (g.L % 4 == 0) && launch::aligned16(p.a);
    dim3 grid(mT * nT, splits);
    convGemmKernel<kGradWeight><<<grid, dev::kBlock, 0, s>>>(p, g);
  }
  THC_HIP_CHECK(hipGetLastError());
  if (fold4) {  // (the scratch starts on a 16-byte boundary)
    // elements per workgroup: the fewest (most lane groups over the splits) that still give 128 workgroups
    const int E = count / 4 >= 128 * 64 ? 64 : count / 4 >= 128 * 16 ? 16 : 4;
    const int gwBlocks = (int)((count / 4 + E - 1) / E);
    const int biasBlocks = fusedBias ? launch::ceilDiv(g.Cout / 4, E) : 0;
    if (E == 64)
      foldPartials4Kernel<64><<<gwBlocks + biasBlocks, dev::kBlock, 0, s>>>(partial, gW, count / 4, splits, scale, biasPartial,
                                                                           gB, g.Cout, gwBlocks);
    else if (E == 16)
      foldPartials4Kernel<16><<<gwBlocks + biasBlocks, dev::kBlock, 0, s>>>(partial, gW, count / 4, splits, scale, biasPartial,
                                                                           gB, g.Cout, gwBlocks);
    else
      foldPartials4Kernel<4><<<gwBlocks + biasBlocks, dev::kBlock, 0, s>>>(partial, gW, count / 4, splits, scale, biasPartial,
                                                                          gB, g.Cout, gwBlocks);
  } else {
    foldPartialsKernel<<<launch::directGrid(count, dev::kBlock), dev::kBlock, 0, s>>>(partial, gW, count, splits, scale);
  }
  THC_HIP_CHECK(hipGetLastError());
  if (gB && !fusedBias) convGradBias(s, gy, gB, g.N, g.Cout, g.L, scale);
}

// ---- entry-point bodies shared by SpatialConvolutionMM and SpatialDilatedConvolution --------
void convUpdateOutput(THCState *state, THCudaTensor *input, THCudaTensor *output, THCudaTensor *weight,
                      THCudaTensor *bias, THCudaTensor *columns, int kW, int kH, int dW, int dH, int padW, int padH,
                      int dilW, int dilH, ConvFlavor flavor, bool relu = false) {
  THC_ARG_CHECK(output != nullptr, 3, "output tensor expected");
  ConvCall call = convSetup(input, nullptr, weight, bias, "weight", kH, kW, dH, dW, padH, padW, dilH, dilW, flavor);
  ConvGeom &g = call.g;
  Contiguous in(state, input);
  if (call.batch)
    resize(state, output, {g.N, g.Cout, g.oH, g.oW});
  else
    resize(state, output, {g.Cout, g.oH, g.oW});
  if (!isContiguous(erase(output))) error("output tensor has to be contiguous");
  convForward(state, g, in.ptr(), data(weight), bias ? data(bias) : nullptr, data(output), columns, "columns", relu);
}

void convUpdateGradInput(THCState *state, THCudaTensor *input, THCudaTensor *gradOutput, THCudaTensor *gradInput,
                         THCudaTensor *weight, THCudaTensor *gradColumns, int kW, int kH, int dW, int dH, int padW,
                         int padH, int dilW, int dilH, ConvFlavor flavor) {
  THC_ARG_CHECK(gradOutput != nullptr, 3, "gradOutput tensor expected");
  THC_ARG_CHECK(gradInput != nullptr, 4, "gradInput tensor expected");
  ConvCall call = convSetup(input, gradOutput, weight, nullptr, "weight", kH, kW, dH, dW, padH, padW, dilH, dilW, flavor);
  ConvGeom &g = call.g;
  Contiguous go(state, gradOutput);
  if (call.batch)
    resize(state, gradInput, {g.N, g.Cin, g.H, g.W});
  else
    resize(state, gradInput, {g.Cin, g.H, g.W});
  if (!isContiguous(erase(gradInput))) error("gradInput tensor has to be contiguous");
  convGradInput(state, g, go.ptr(), data(weight), data(gradInput), gradColumns, "gradColumns");
}

void convAccGradParameters(THCState *state, THCudaTensor *input, THCudaTensor *gradOutput, THCudaTensor *gradWeight,
                           THCudaTensor *gradBias, THCudaTensor *columns, int kW, int kH, int dW, int dH, int padW,
                           int padH, int dilW, int dilH, float scale, ConvFlavor flavor) {
  THC_ARG_CHECK(gradOutput != nullptr, 3, "gradOutput tensor expected");
  THC_ARG_CHECK(gradWeight != nullptr, 4, "gradWeight tensor expected");
  ConvCall call = convSetup(input, gradOutput, gradWeight, gradBias, "weight", kH, kW,
                            dH, dW, padH, padW, dilH, dilW, flavor);
  ConvGeom &g = call.g;
  Contiguous in(state, input);
  Contiguous go(state, gradOutput);
  convGradWeight(state, g, in.ptr(), go.ptr(), data(gradWeight), columns, scale, gradBias ? data(gradBias) : nullptr);
}

// ---- transposed ("full") convolution -----------------------------------------------------------
// SpatialFull(Dilated)Convolution maps the (N, Cin, H, W) input to (N, Cout, oH, oW) with
// oH = (H-1)*dH - 2*padH + dilH*(kH-1) + 1 + adjH; its weight is (Cin, Cout, kH, kW). It is the
// ordinary convolution C with input (N, Cout, oH, oW), output (N, Cin, H, W) and weight
// (Cin, Cout*kH*kW) run backwards: updateOutput = C's gradInput pass (+ bias), updateGradInput =
// C's forward pass, accGradParameters = C's weight-gradient pass with the roles of input and
// gradOutput swapped (lib/THCUNN/generic/SpatialFullDilatedConvolution.cu:141-165, 268-298, 385-414).
// The geometry returned here is C's.
ConvCall fullSetup(THCudaTensor *input, THCudaTensor *gradOutput, THCudaTensor *weight, THCudaTensor *bias, int kH,
                   int kW, int dH, int dW, int padH, int padW, int dilH, int dilW, int adjH, int adjW) {
  // lib/THCUNN/generic/SpatialFullDilatedConvolution.cu:5-66
  THC_ARG_CHECK(input && weight, 2, "input and weight tensors expected");
  THC_ARG_CHECK(kW > 0 && kH > 0, 9, "kernel size should be greater than zero, but got kH: %d kW: %d", kH, kW);
  THC_ARG_CHECK(dW > 0 && dH > 0, 11, "stride should be greater than zero, but got dH: %d dW: %d", dH, dW);
  THC_ARG_CHECK(dilW > 0 && dilH > 0, 15, "dilation should be greater than zero, but got dilationH: %d, dilationW: %d",
                dilH, dilW);
  THC_ARG_CHECK((adjW < dW || adjW < dilW) && (adjH < dH || adjH < dilH), 15,
                "output padding must be smaller than either stride or dilation, but got adjH: %d adjW: %d dH: %d dW: %d "
                "dilationH: %d dilationW: %d",
                adjH, adjW, dH, dW, dilH, dilW);
  THC_ARG_CHECK(isContiguous(erase(weight)), 4, "weight tensor has to be contiguous");
  THC_ARG_CHECK(!bias || isContiguous(erase(bias)), 5, "bias tensor has to be contiguous");
  THC_ARG_CHECK(weight->nDimension == 2 || weight->nDimension == 4, 5, "2D or 4D weight tensor expected, but got: %s",
                sizeDesc(erase(weight)).c_str());
  if (bias) checkDimSize(erase(bias), "bias", 1, 0, weight->size[1]);
  int ndim = input->nDimension;
  int dimf = 0, dimh = 1, dimw = 2;
  if (ndim == 4) {
    dimf++;
    dimh++;
    dimw++;
  }
  THC_ARG_CHECK(ndim == 3 || ndim == 4, 2, "3D or 4D input tensor expected but got: %s",
                sizeDesc(erase(input)).c_str());
  if (weight->nDimension != 4) error("transposed convolution: 4D weight tensor (nInputPlane,nOutputPlane,kH,kW) expected");
  long nInputPlane = weight->size[0], nOutputPlane = weight->size[1];
  long inputHeight = input->size[dimh], inputWidth = input->size[dimw];
  long outputHeight = (inputHeight - 1) * dH - 2 * padH + (dilH * (kH - 1) + 1) + adjH;
  long outputWidth = (inputWidth - 1) * dW - 2 * padW + (dilW * (kW - 1) + 1) + adjW;
  if (outputWidth < 1 || outputHeight < 1)
    error("Given input size: (%ld x %ld x %ld). Calculated output size: (%ld x %ld x %ld). Output size is too small",
          nInputPlane, inputHeight, inputWidth, nOutputPlane, outputHeight, outputWidth);
  checkDimSize(erase(input), "input", ndim, dimf, nInputPlane);
  if (gradOutput) {
    checkDimSize(erase(gradOutput), "gradOutput", ndim, dimf, nOutputPlane);
    checkDimSize(erase(gradOutput), "gradOutput", ndim, dimh, outputHeight);
    checkDimSize(erase(gradOutput), "gradOutput", ndim, dimw, outputWidth);
    if (ndim == 4 && gradOutput->size[0] != input->size[0])
      error("input and gradOutput batch sizes do not match: input %s, gradOutput %s", sizeDesc(erase(input)).c_str(),
            sizeDesc(erase(gradOutput)).c_str());
  }
  if (weight->size[2] != kH || weight->size[3] != kW)
    error("weight of shape %s does not match a %d x %d kernel", sizeDesc(erase(weight)).c_str(), kH, kW);
  ConvCall call;
  call.batch = ndim == 4;
  call.g = makeGeom(call.batch ? (int)input->size[0] : 1, (int)nOutputPlane, (int)nInputPlane, (int)outputHeight,
                    (int)outputWidth, (int)inputHeight, (int)inputWidth, kH, kW, dH, dW, padH, padW, dilH, dilW);
  return call;
}

void fullUpdateOutput(THCState *state, THCudaTensor *input, THCudaTensor *output, THCudaTensor *weight,
                      THCudaTensor *bias, THCudaTensor *columns, int kW, int kH, int dW, int dH, int padW, int padH,
                      int dilW, int dilH, int adjW, int adjH) {
  THC_ARG_CHECK(output != nullptr, 3, "output tensor expected");
  ConvCall call = fullSetup(input, nullptr, weight, bias, kH, kW, dH, dW, padH, padW, dilH, dilW, adjH, adjW);
  ConvGeom &g = call.g;
  Contiguous in(state, input);
  if (call.batch)
    resize(state, output, {g.N, g.Cin, g.H, g.W});
  else
    resize(state, output, {g.Cin, g.H, g.W});
  if (!isContiguous(erase(output))) error("output tensor has to be contiguous");
  convGradInput(state, g, in.ptr(), data(weight), data(output), columns, "columns", bias ? data(bias) : nullptr);
}

void fullUpdateGradInput(THCState *state, THCudaTensor *input, THCudaTensor *gradOutput, THCudaTensor *gradInput,
                         THCudaTensor *weight, THCudaTensor *gradColumns, int kW, int kH, int dW, int dH, int padW,
                         int padH, int dilW, int dilH, int adjW, int adjH) {
  THC_ARG_CHECK(gradOutput != nullptr, 3, "gradOutput tensor expected");
  THC_ARG_CHECK(gradInput != nullptr, 4, "gradInput tensor expected");
  ConvCall call = fullSetup(input, gradOutput, weight, nullptr, kH, kW, dH, dW, padH, padW, dilH, dilW, adjH, adjW);
  ConvGeom &g = call.g;
  Contiguous go(state, gradOutput);
  if (call.batch)
    resize(state, gradInput, {g.N, g.Cout, g.oH, g.oW});
  else
    resize(state, gradInput, {g.Cout, g.oH, g.oW});
  if (!isContiguous(erase(gradInput))) error("gradInput tensor has to be contiguous");
  convForward(state, g, go.ptr(), data(weight), nullptr, data(gradInput), gradColumns, "gradColumns");
}

void fullAccGradParameters(THCState *state, THCudaTensor *input, THCudaTensor *gradOutput, THCudaTensor *gradWeight,
                           THCudaTensor *gradBias, THCudaTensor *columns, int kW, int kH, int dW, int dH, int padW,
                           int padH, int dilW, int dilH, int adjW, int adjH, float scale) {
  THC_ARG_CHECK(gradOutput != nullptr, 3, "gradOutput tensor expected");
  THC_ARG_CHECK(gradWeight != nullptr, 4, "gradWeight tensor expected");
  ConvCall call = fullSetup(input, gradOutput, gradWeight, gradBias, kH, kW, dH, dW, padH, padW, dilH, dilW, adjH, adjW);
  ConvGeom &g = call.g;
  Contiguous in(state, input);
  Contiguous go(state, gradOutput);
  convGradWeight(state, g, go.ptr(), in.ptr(), data(gradWeight), columns, scale);
  if (gradBias) convGradBias(state->stream, go.ptr(), data(gradBias), g.N, g.Cin, g.H * g.W, scale);
}

}  // namespace

extern "C" {

void THNN_CudaSpatialConvolutionMM_updateOutput(THCState *state, THCudaTensor *input, THCudaTensor *output,
                                                THCudaTensor *weight, THCudaTensor *bias, THCudaTensor *columns,
                                                THCudaTensor *ones, int kW, int kH, int dW, int dH, int padW,
                                                int padH) {
  THNN_ENTER
  (void)ones;  // never read; `columns` is used (and resized) only as scratch
  convUpdateOutput(state, input, output, weight, bias, columns, kW, kH, dW, dH, padW, padH, 1, 1, kConvMM);
  THNN_LEAVE
}

// No counterpart in the reference (include/THCUNN_fused.h): SpatialConvolutionMM_updateOutput followed by
// Threshold_updateOutput(0, 0), the clamp applied as the convolution stores its values.
void THNN_CudaSpatialConvolutionMMReLU_updateOutput(THCState *state, THCudaTensor *input, THCudaTensor *output,
                                                    THCudaTensor *weight, THCudaTensor *bias, THCudaTensor *columns,
                                                    THCudaTensor *ones, int kW, int kH, int dW, int dH, int padW,
                                                    int padH) {
  THNN_ENTER
  (void)ones;
  convUpdateOutput(state, input, output, weight, bias, columns, kW, kH, dW, dH, padW, padH, 1, 1, kConvMM, true);
  THNN_LEAVE
}

void THNN_CudaSpatialConvolutionMM_updateGradInput(THCState *state, THCudaTensor *input, THCudaTensor *gradOutput,
                                                   THCudaTensor *gradInput, THCudaTensor *weight,
                                                   THCudaTensor *gradColumns, THCudaTensor *ones, int kW, int kH,
                                                   int dW, int dH, int padW, int padH) {
  THNN_ENTER
  (void)ones;
  convUpdateGradInput(state, input, gradOutput, gradInput, weight, gradColumns, kW, kH, dW, dH, padW, padH, 1, 1, kConvMM);
  THNN_LEAVE
}

void THNN_CudaSpatialConvolutionMM_accGradParameters(THCState *state, THCudaTensor *input, THCudaTensor *gradOutput,
                                                     THCudaTensor *gradWeight, THCudaTensor *gradBias,
                                                     THCudaTensor *columns, THCudaTensor *ones, int kW, int kH,
                                                     int dW, int dH, int padW, int padH, float scale) {
  THNN_ENTER
  (void)ones;
  convAccGradParameters(state, input, gradOutput, gradWeight, gradBias, columns, kW, kH, dW, dH, padW, padH, 1, 1, scale,
                        kConvMM);
  THNN_LEAVE
}

// SpatialDilatedConvolution (lib/THCUNN/generic/SpatialDilatedConvolution.cu:69-190, 192-293, 295-432):
// the same three GEMMs with taps dilationH/W apart.
void THNN_CudaSpatialDilatedConvolution_updateOutput(THCState *state, THCudaTensor *input, THCudaTensor *output,
                                                     THCudaTensor *weight, THCudaTensor *bias, THCudaTensor *columns,
                                                     THCudaTensor *ones, int kW, int kH, int dW, int dH, int padW,
                                                     int padH, int dilationW, int dilationH) {
  THNN_ENTER
  (void)ones;
  convUpdateOutput(state, input, output, weight, bias, columns, kW, kH, dW, dH, padW, padH, dilationW, dilationH,
                   kDilated);
  THNN_LEAVE
}

void THNN_CudaSpatialDilatedConvolution_updateGradInput(THCState *state, THCudaTensor *input,
                                                        THCudaTensor *gradOutput, THCudaTensor *gradInput,
                                                        THCudaTensor *weight, THCudaTensor *gradColumns, int kW,
                                                        int kH, int dW, int dH, int padW, int padH, int dilationW,
                                                        int dilationH) {
  THNN_ENTER
  convUpdateGradInput(state, input, gradOutput, gradInput, weight, gradColumns, kW, kH, dW, dH, padW, padH, dilationW,
                      dilationH, kDilated);
  THNN_LEAVE
}

void THNN_CudaSpatialDilatedConvolution_accGradParameters(THCState *state, THCudaTensor *input,
                                                          THCudaTensor *gradOutput, THCudaTensor *gradWeight,
                                                          THCudaTensor *gradBias, THCudaTensor *columns,
                                                          THCudaTensor *ones, int kW, int kH, int dW, int dH,
                                                          int padW, int padH, int dilationW, int dilationH,
                                                          float scale) {
  THNN_ENTER
  (void)ones;
  convAccGradParameters(state, input, gradOutput, gradWeight, gradBias, columns, kW, kH, dW, dH, padW, padH, dilationW,
                        dilationH, scale, kDilated);
  THNN_LEAVE
}

// SpatialFullDilatedConvolution / SpatialFullConvolution
// (lib/THCUNN/generic/SpatialFullDilatedConvolution.cu:68-204, 206-312, 314-465; generic/SpatialFullConvolution.cu:5-59)
void THNN_CudaSpatialFullDilatedConvolution_updateOutput(THCState *state, THCudaTensor *input, THCudaTensor *output,
                                                         THCudaTensor *weight, THCudaTensor *bias,
                                                         THCudaTensor *columns, THCudaTensor *ones, int kW, int kH,
                                                         int dW, int dH, int padW, int padH, int dilationW,
                                                         int dilationH, int adjW, int adjH) {
  THNN_ENTER
  (void)ones;
  fullUpdateOutput(state, input, output, weight, bias, columns, kW, kH, dW, dH, padW, padH, dilationW, dilationH, adjW,
                   adjH);
  THNN_LEAVE
}

void THNN_CudaSpatialFullDilatedConvolution_updateGradInput(THCState *state, THCudaTensor *input,
                                                            THCudaTensor *gradOutput, THCudaTensor *gradInput,
                                                            THCudaTensor *weight, THCudaTensor *gradColumns, int kW,
                                                            int kH, int dW, int dH, int padW, int padH,
                                                            int dilationW, int dilationH, int adjW, int adjH) {
  THNN_ENTER
  fullUpdateGradInput(state, input, gradOutput, gradInput, weight, gradColumns, kW, kH, dW, dH, padW, padH, dilationW,
                      dilationH, adjW, adjH);
  THNN_LEAVE
}

void THNN_CudaSpatialFullDilatedConvolution_accGradParameters(THCState *state, THCudaTensor *input,
                                                              THCudaTensor *gradOutput, THCudaTensor *gradWeight,
                                                              THCudaTensor *gradBias, THCudaTensor *columns,
                                                              THCudaTensor *ones, int kW, int kH, int dW, int dH,
                                                              int padW, int padH, int dilationW, int dilationH,
                                                              int adjW, int adjH, float scale) {
  THNN_ENTER
  (void)ones;
  fullAccGradParameters(state, input, gradOutput, gradWeight, gradBias, columns, kW, kH, dW, dH, padW, padH, dilationW,
                        dilationH, adjW, adjH, scale);
  THNN_LEAVE
}

void THNN_CudaSpatialFullConvolution_updateOutput(THCState *state, THCudaTensor *input, THCudaTensor *output,
                                                  THCudaTensor *weight, THCudaTensor *bias, THCudaTensor *columns,
                                                  THCudaTensor *ones, int kW, int kH, int dW, int dH, int padW,
                                                  int padH, int adjW, int adjH) {
  THNN_ENTER
  (void)ones;
  fullUpdateOutput(state, input, output, weight, bias, columns, kW, kH, dW, dH, padW, padH, 1, 1, adjW, adjH);
  THNN_LEAVE
}

void THNN_CudaSpatialFullConvolution_updateGradInput(THCState *state, THCudaTensor *input, THCudaTensor *gradOutput,
                                                     THCudaTensor *gradInput, THCudaTensor *weight,
                                                     THCudaTensor *gradColumns, int kW, int kH, int dW, int dH,
                                                     int padW, int padH, int adjW, int adjH) {
  THNN_ENTER
  fullUpdateGradInput(state, input, gradOutput, gradInput, weight, gradColumns, kW, kH, dW, dH, padW, padH, 1, 1, adjW,
                      adjH);
  THNN_LEAVE
}

void THNN_CudaSpatialFullConvolution_accGradParameters(THCState *state, THCudaTensor *input, THCudaTensor *gradOutput,
                                                       THCudaTensor *gradWeight, THCudaTensor *gradBias,
                                                       THCudaTensor *columns, THCudaTensor *ones, int kW, int kH,
                                                       int dW, int dH, int padW, int padH, int adjW, int adjH,
                                                       float scale) {
  THNN_ENTER
  (void)ones;
  fullAccGradParameters(state, input, gradOutput, gradWeight, gradBias, columns, kW, kH, dW, dH, padW, padH, 1, 1, adjW,
                        adjH, scale);
  THNN_LEAVE
}

// Stand-alone im2col / col2im over a batch of images with the semantics of
// lib/THCUNN/im2col.h:40-61 and :104-121 (the reference keeps them as C++
// templates inside the library; they are exported here so that their parity
// can be checked on their own).
void THNN_Cuda_im2col(THCState *state, const float *im, int nImages, int channels, int height, int width, int kH,
                      int kW, int padH, int padW, int dH, int dW, int dilH, int dilW, float *col) {
  THNN_ENTER
  int oH = (height + 2 * padH - (dilH * (kH - 1) + 1)) / dH + 1;
  int oW = (width + 2 * padW - (dilW * (kW - 1) + 1)) / dW + 1;
  long total = (long)nImages * channels * kH * kW * oH * oW;
  if (total <= 0) return;
  im2colKernel<<<launch::directGrid(total, dev::kBlock), dev::kBlock, 0, state->stream>>>(
      im, col, nImages, channels, height, width, kH, kW, padH, padW, dH, dW, dilH, dilW, oH, oW);
  THC_HIP_CHECK(hipGetLastError());
  THNN_LEAVE
}

void THNN_Cuda_col2im(THCState *state, const float *col, int nImages, int channels, int height, int width, int kH,
                      int kW, int padH, int padW, int dH, int dW, int dilH, int dilW, float *im) {
  THNN_ENTER
  int oH = (height + 2 * padH - (dilH * (kH - 1) + 1)) / dH + 1;
  int oW = (width + 2 * padW - (dilW * (kW - 1) + 1)) / dW + 1;
  long total = (long)nImages * channels * height * width;
  if (total <= 0) return;
  col2imKernel<<<launch::directGrid(total, dev::kBlock), dev::kBlock, 0, state->stream>>>(
      col, im, nImages, channels, height, width, kH, kW, padH, padW, dH, dW, dilH, dilW, oH, oW, nullptr);
  THC_HIP_CHECK(hipGetLastError());
  THNN_LEAVE
}

}  // extern "C"
