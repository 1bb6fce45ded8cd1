// Runs of memory for kernels that work on small planes: several whole planes (the 28x28 / 14x14 / 7x7
// stages of a network) or a band of rows of one larger plane of any width per workgroup. Planes are
// contiguous in memory and so are the rows of a band, so what a workgroup reads is one contiguous run
// of floats: it is fetched with 16-byte loads in memory order (from the 16-byte boundary at or below its
// first element - no alignment or multiple-of-4 requirement on the extents), scattered into bordered
// planes in LDS, and what the workgroup produces goes through a linear LDS buffer so that it leaves as
// 16-byte streaming stores in memory order as well. Included inside an anonymous namespace after
// device_utils.h.
#pragma once

#include <type_traits>

struct SmallGeom {
  int C, planes;           // channels (where the kernel needs the channel of a plane), N * C
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

// KS: window, CS: stride of the computation, DS: dilation of the staging, PAD: border in front of source row 0
template <int KS, int CS, int DS, int PAD = KS / 2>
__device__ __forceinline__ SmallBand smallBand(const SmallGeom &g) {
  SmallBand b;
  if (g.P > 1) {
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
// STREAM: with the non-temporal hint (the run's last reader)
template <bool STREAM = false>
__device__ __forceinline__ void smallIssue(SmallRun &r, const float *__restrict__ tensor, long first, int count, long total) {
  r.lead = (int)(first & 3), r.count = count;
  const float *base = tensor + (first - r.lead);
  const long avail = total - (first - r.lead);  // floats from the aligned start to the end of the tensor
  const int span = r.lead + count;
  const __amdgpu_buffer_rsrc_t rs = dev::makeRsrc(base, (long)(span & ~3) * 4);
#pragma unroll
  for (int u = 0; u < dev::kLoadBatch; ++u) {
    const int e = (u * dev::kBlock + (int)threadIdx.x) * 4;
    r.v[u] = STREAM ? dev::bufLoadStream4(rs, e + 4 <= span ? e * 4 : dev::kBufOob)
                    : dev::bufLoad4(rs, e + 4 <= span ? e * 4 : dev::kBufOob);
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
      int p = g.P > 1 ? dev::fastDiv(i0, g.magicSPlane) : 0;
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

__device__ __forceinline__ void smallFill(float *__restrict__ xs, int floats, float v) {
  for (int i = threadIdx.x; i * 4 < floats; i += dev::kBlock) reinterpret_cast<float4 *>(xs)[i] = make_float4(v, v, v, v);
}
__device__ __forceinline__ void smallZero(float *__restrict__ xs, int floats) { smallFill(xs, floats, 0.f); }

// Stores the run of `count` floats that starts at element `first` of `tensor` (16-byte aligned) from LDS,
// where element i of the run sits at os[(first & 3) + i]: 16-byte streaming stores for the groups that lie
// inside the run, single stores for its ragged ends.
__device__ __forceinline__ void smallStoreRun(float *__restrict__ tensor, long first, const float *__restrict__ os, int count) {
  const int lead = (int)(first & 3);
  float *base = tensor + (first - lead);
  const __amdgpu_buffer_rsrc_t br = dev::makeRsrc(base, (long)(lead + count) * 4);
  for (int i = threadIdx.x; i * 4 < lead + count; i += dev::kBlock) {
    const int e = i * 4;
    if (e >= lead && e + 4 <= lead + count) {
      dev::bufStoreStream4(br, e * 4, reinterpret_cast<const float4 *>(os)[i]);
    } else {
      for (int k = max(e, lead); k < min(e + 4, lead + count); ++k) base[k] = os[k];
    }
  }
}


// The same for a run of 64-bit indices (16-byte loads of two): index i of the run sits in group
// (lead + i) / 2, lead = first & 1. Two batches cover the 4 * kLoadBatch * kBlock elements of a float run.
struct SmallIdxRun {
  long2 v[2 * dev::kLoadBatch];
  int lead, count;
};
typedef long i64x2v __attribute__((ext_vector_type(2)));
template <bool STREAM = false>
__device__ __forceinline__ void smallIssueIdx(SmallIdxRun &r, const long *__restrict__ tensor, long first, int count, long total) {
  r.lead = (int)(first & 1), r.count = count;
  const long *base = tensor + (first - r.lead);
  const long avail = total - (first - r.lead);
  const int span = r.lead + count;
#pragma unroll
  for (int u = 0; u < 2 * dev::kLoadBatch; ++u) {
    const int e = (u * dev::kBlock + (int)threadIdx.x) * 2;
    r.v[u] = make_long2(0, 0);
    if (e + 2 <= span || (e < span && e + 2 <= avail)) {
      if (STREAM) {
        const i64x2v q = __builtin_nontemporal_load(reinterpret_cast<const i64x2v *>(base + e));
        r.v[u] = make_long2(q.x, q.y);
      } else {
        r.v[u] = *reinterpret_cast<const long2 *>(base + e);
      }
    }
    else if (e < span)
      r.v[u].x = base[e];
  }
}

// Stores a run of `count` 64-bit indices from 32-bit values in LDS (element i of the run at is[(first & 1) + i]).
__device__ __forceinline__ void smallStoreIdxRun(long *__restrict__ tensor, long first, const int *__restrict__ is, int count) {
  const int lead = (int)(first & 1);
  long *base = tensor + (first - lead);
  const __amdgpu_buffer_rsrc_t br = dev::makeRsrc(base, (long)(lead + count) * 8);
  for (int i = threadIdx.x; i * 2 < lead + count; i += dev::kBlock) {
    const int e = i * 2;
    if (e >= lead && e + 2 <= lead + count) {
      const int2 v = reinterpret_cast<const int2 *>(is)[i];
      dev::bufStoreStream2L(br, e * 8, (long)v.x, (long)v.y);
    } else {
      for (int k = max(e, lead); k < min(e + 2, lead + count); ++k) base[k] = is[k];
    }
  }
}
