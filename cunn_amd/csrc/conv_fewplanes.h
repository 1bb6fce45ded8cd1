// updateGradInput of a convolution with one to four input planes (the first layer of a network; the last layer of a
// generator when run as a transposed convolution's forward pass):
//   gi(n, c, h, w) = bias(c) + sum_{o, kh, kw} gy(n, o, oh, ow) * W(o, c, kh, kw),   oh * s + kh - pad = h  (same for w)
// lib/THCUNN/generic/SpatialConvolutionMM.cu:272-308 does this as a (Cin*kH*kW x Cout) x (Cout x L) SGEMM into gradient
// columns followed by the col2im gather (lib/THCUNN/im2col.h:63-102): K*L floats per image written and read again.
//
// A GEMM tile with Cin rows would be all padding, so the matrix cores are fed the other way round, with
// v_mfma_f32_4x4x1_16B_f32: 16 independent 4x4 outer products per instruction, same peak rate as the large shapes.
// The 4 rows are the input planes, the 64 lanes are 64 gradInput positions, and one instruction adds one
// (o, kh, kw) term to 4 planes x 64 positions. Nothing goes through memory in between:
//  * gradInput is computed phase by phase (h = s*i + ph): for the positions of one phase only the taps with
//    kh = (ph + pad) mod s (+ s, + 2s ...) contribute, and tap number a reads gradOutput row i + q0 - a - no
//    multiplication is spent on the zeros of a dilated gradOutput;
//  * a wave owns a block of phase positions (4*T rows x 16 columns, all s*s phases: a 4T*s x 16*s patch of
//    gradInput) and walks over the output planes in chunks of 4: the gradOutput patch with its halo and the chunk's
//    weights are parked in wave-private LDS (no workgroup barrier anywhere), the next chunk is in flight meanwhile;
//  * lane (lr, lc) works on rows lr*T + t, t = 0..T-1, of the block: tiles that are neighbours in t read the same
//    gradOutput rows for neighbouring taps, so with a compile-time kernel size every LDS value is fetched once per
//    output plane and used by up to (k/s)^2 * ... instructions.
// Sums run over o, then taps, in a fixed order: results do not depend on the grid.
#pragma once

__host__ __device__ constexpr int fpRem(int ph, int pad, int s) { return (ph + pad) % s; }
__host__ __device__ constexpr int fpQ0(int ph, int pad, int s) { return (ph + pad) / s; }
__host__ __device__ constexpr int fpTaps(int ph, int pad, int s, int k) {
  return fpRem(ph, pad, s) < k ? (k - fpRem(ph, pad, s) + s - 1) / s : 0;
}
// lowest / highest gradOutput row, relative to the phase row, that any phase reads
__host__ __device__ constexpr int fpLo(int pad, int s, int k) {
  int lo = 1 << 20;
  for (int ph = 0; ph < s; ++ph)
    if (fpTaps(ph, pad, s, k) > 0 && fpQ0(ph, pad, s) - fpTaps(ph, pad, s, k) + 1 < lo)
      lo = fpQ0(ph, pad, s) - fpTaps(ph, pad, s, k) + 1;
  return lo;
}
__host__ __device__ constexpr int fpHi(int pad, int s, int k) {
  int hi = -(1 << 20);
  for (int ph = 0; ph < s; ++ph)
    if (fpTaps(ph, pad, s, k) > 0 && fpQ0(ph, pad, s) > hi) hi = fpQ0(ph, pad, s);
  return hi;
}
// LDS row pitch: the four 16-lane rows of a wave sit T rows apart and must fall on different groups of 16 banks
__host__ __device__ constexpr int fpPitch(int T, int cols) {
  int p = cols;
  while ((T * p) % 32 != 16) ++p;
  return p;
}

constexpr int kFpWaves = 4;       // waves per workgroup: they share a block and split the output planes
constexpr int kFpGroup = 4;       // output planes are dealt to the waves in groups of 4
constexpr int kFpMaxLoads = 13;   // run-time variant: patch elements per lane and output plane
constexpr int kFpMaxWLoads = 12;  // run-time variant: weight elements per lane and chunk
constexpr int kFpMaxTaps = 128;   // run-time variant: kH * kW
constexpr int kFpRedQ = 8;        // accumulators (of 4 floats) per lane that cross LDS in one pass of the final sum

struct FpDim {
  int rem[4], q0[4], taps[4];  // per phase
  int lo, hi;
};

struct FpArgs {
  const float *gy;    // (N, Cout, oH, oW)
  const float *w;     // (Cout, Cin * kH * kW)
  const float *bias;  // Cin or null
  float *gi;          // (N, Cin, H, W)
  int Cin, Cout, H, W, oH, oW, kH, kW;
  int tilesR, tilesC;  // blocks per image
  unsigned magicTiles, magicTilesC, magicCK, magicKK, magicCC;  // dev::magicOf of tilesR*tilesC, tilesC, Cin*kH*kW, kH*kW, CC
  FpDim dh, dw;        // run-time variant
  int RR, CC;          // run-time variant: rows / columns of the parked patch
};

// Run-time variant: the taps of every phase pair (ph, pw), in (a, b) order: weight index kh * kW + kw in the low
// half, offset of the gradOutput value in the parked patch (floats, relative to the lane's corner) in the high half.
struct FpTaps {
  int first[17];  // phase pair q = ph * S + pw owns entries first[q] .. first[q + 1] - 1
  unsigned e[kFpMaxTaps];
};

typedef float float4v __attribute__((ext_vector_type(4)));

// S: stride (both directions). T: rows per lane. KC > 0: kH = kW = KC and padH = padW = PADC at compile time.
template <int S, int T, int KC, int PADC>
struct FpShape {
  static constexpr bool CT = KC > 0;
  static constexpr int OC = CT ? 4 : 2;  // output planes per LDS chunk
  static constexpr int LO = CT ? fpLo(PADC, S, CT ? KC : 1) : 0, HI = CT ? fpHi(PADC, S, CT ? KC : 1) : 0;
  static constexpr int SPAN = HI - LO;
  static constexpr int RR = 4 * T + SPAN, CC = 16 + SPAN;  // compile-time variant
  // run-time variant: fixed pitch, spans up to pitch - 16
  static constexpr int PITCH = CT ? fpPitch(T, CC) : (T == 4 ? 28 : T == 2 ? 24 : 48);
  static constexpr int NLG = CT ? (RR * CC + 63) / 64 : kFpMaxLoads;
  static constexpr int KK = CT ? KC * KC : 0;
  static constexpr int KKP = (KK + 3) / 4 * 4;
  static constexpr int NLW = CT ? (OC * 4 * KK + 63) / 64 : kFpMaxWLoads;
  static constexpr int NQ = T * S * S;  // accumulators per lane
  // floats of LDS a wave parks its chunk in
  __host__ __device__ static constexpr int priv(int rr, int kkp) { return OC * rr * PITCH + OC * 4 * kkp + 64; }
  __host__ __device__ static constexpr size_t ldsBytes(int rr, int kkp) {
    const size_t a = (size_t)kFpWaves * priv(rr, kkp), b = (size_t)kFpWaves * (NQ < kFpRedQ ? NQ : kFpRedQ) * 256;
    return (a > b ? a : b) * sizeof(float);
  }
};

template <int S, int T, int KC, int PADC>
__global__ void __launch_bounds__(64 * kFpWaves)
convFewPlanesGradInputKernel(FpArgs p, FpTaps tp) {
  using Sh = FpShape<S, T, KC, PADC>;
  constexpr bool CT = Sh::CT;
  constexpr int OC = Sh::OC, SUB = kFpGroup / OC, PITCH = Sh::PITCH, NLG = Sh::NLG, NLW = Sh::NLW, NQ = Sh::NQ;
  extern __shared__ float ldsAll[];

  const int lane = threadIdx.x & 63, lr = lane >> 4, lc = lane & 15, cA = lane & 3;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int kH = CT ? KC : p.kH, kW = CT ? KC : p.kW, KK = kH * kW, KKP = CT ? Sh::KKP : (KK + 3) / 4 * 4;
  const int RR = CT ? Sh::RR : p.RR, CC = CT ? Sh::CC : p.CC;
  const int loH = CT ? Sh::LO : p.dh.lo, loW = CT ? Sh::LO : p.dw.lo;
  const int plane = RR * PITCH;                 // floats per parked output plane
  const int wBase = OC * plane;                 // where the weights start
  float *lds = ldsAll + wave * Sh::priv(RR, KKP);  // patch[OC][RR][PITCH], weights[OC][4][KKP], 64 spare

  int item = dev::xcdRemap(blockIdx.x, gridDim.x);
  const int n = dev::fastDiv(item, p.magicTiles);
  item -= n * p.tilesR * p.tilesC;
  const int tr = dev::fastDiv(item, p.magicTilesC), tc = item - tr * p.tilesC;
  const int I0 = tr * 4 * T, J0 = tc * 16;

  const long gyImg = (long)p.Cout * p.oH * p.oW;
  const int gyPlaneBytes = p.oH * p.oW * 4;
  const __amdgpu_buffer_rsrc_t gyr = dev::makeRsrc(p.gy + n * gyImg, gyImg * 4);

  // where this lane's elements of a patch come from and go to (the same for every output plane)
  int gOff[NLG], lOff[NLG];
#pragma unroll
  for (int k = 0; k < NLG; ++k) {
    const int idx = lane + 64 * k;
    const int rr = CT ? idx / CC : dev::fastDiv(idx, p.magicCC), cc = idx - rr * CC;
    const int row = I0 + loH + rr, col = J0 + loW + cc;
    const bool inPatch = idx < RR * CC;
    const bool ok = inPatch && row >= 0 && row < p.oH && col >= 0 && col < p.oW;
    gOff[k] = ok ? (row * p.oW + col) * 4 : dev::kBufOob;
    lOff[k] = inPatch ? rr * PITCH + cc : -1;
  }
  const int nlg = CT ? NLG : (RR * CC + 63) / 64;
  // element e = lane + 64 k of a chunk's weights is (o, c, tap) = (e / (Cin KK), ...): it goes to weights[o][c][tap];
  // elements past the chunk (the loads cover OC * 4 * KK) go to the lane's spare slot
  const int nlw = CT ? NLW : (OC * p.Cin * KK + 63) / 64;
  int wOff[NLW];
#pragma unroll
  for (int k = 0; k < NLW; ++k) {
    const int e = lane + 64 * k;
    const int o_ = dev::fastDiv(e, p.magicCK), rem = e - o_ * p.Cin * KK;
    const int c = dev::fastDiv(rem, p.magicKK), tap = rem - c * KK;
    wOff[k] = o_ < OC ? wBase + (o_ * 4 + c) * KKP + tap : wBase + OC * 4 * KKP + lane;
  }

  // The output planes go to the waves in groups of 4 (group g to wave g mod 4), a group in chunks of OC:
  // chunk number ci of this wave starts at plane
  auto firstPlane = [&](int ci) { return kFpGroup * (wave + kFpWaves * (ci / SUB)) + OC * (ci % SUB); };

  unsigned gv[OC][NLG];
  float wv[NLW];
  auto fetch = [&](int o0) {  // a chunk on its way to registers
    const int oc = min(OC, p.Cout - o0);
#pragma unroll
    for (int o = 0; o < OC; ++o)
      if (o < oc) {
#pragma unroll
        for (int k = 0; k < NLG; ++k)
          if (CT || k < nlg) gv[o][k] = __builtin_amdgcn_raw_buffer_load_b32(gyr, gOff[k], (o0 + o) * gyPlaneBytes, 0);
      }
    // the weights of the chunk are contiguous; what lies past the end of the matrix reads as 0
    const __amdgpu_buffer_rsrc_t wr = dev::makeRsrc(p.w + (long)o0 * p.Cin * KK, (long)(p.Cout - o0) * p.Cin * KK * 4);
#pragma unroll
    for (int k = 0; k < NLW; ++k)
      if (CT || k < nlw) wv[k] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(wr, lane * 4 + 256 * k, 0, 0));
  };
  auto park = [&](int o0) {  // registers -> LDS
    const int oc = min(OC, p.Cout - o0);
#pragma unroll
    for (int o = 0; o < OC; ++o)
      if (o < oc) {
#pragma unroll
        for (int k = 0; k < NLG; ++k)
          if (CT ? (64 * (k + 1) <= Sh::RR * Sh::CC || lOff[k] >= 0) : (k < nlg && lOff[k] >= 0))
            lds[o * plane + lOff[k]] = __uint_as_float(gv[o][k]);
      }
#pragma unroll
    for (int k = 0; k < NLW; ++k)
      if (CT || k < nlw) lds[wOff[k]] = wv[k];
  };

  float4v acc[T][S][S];
#pragma unroll
  for (int t = 0; t < T; ++t)
#pragma unroll
    for (int a = 0; a < S; ++a)
#pragma unroll
      for (int b = 0; b < S; ++b) acc[t][a][b] = float4v{0.f, 0.f, 0.f, 0.f};

  const int laneB = lr * T * PITCH + lc;  // the lane's corner of the parked patch
  const int laneA = wBase + cA * KKP;     // the lane's plane of the weights

  float bias[4] = {0.f, 0.f, 0.f, 0.f};  // fetched now: a load next to the stores would make every store wait for the one before
  if (p.bias) {
#pragma unroll
    for (int c = 0; c < 4; ++c)
      if (c < p.Cin) bias[c] = p.bias[c];
  }
  __builtin_amdgcn_s_setprio(2);  // setting up and winding down go ahead of the other waves' multiplications
  if (firstPlane(0) < p.Cout) fetch(firstPlane(0));
  for (int ci = 0; firstPlane(ci) < p.Cout; ++ci) {
    const int o0 = firstPlane(ci);
    const int oc = min(OC, p.Cout - o0);
    __builtin_amdgcn_s_setprio(2);
    // the reads of the chunk before are done (their values went into MFMAs already issued); LDS runs a wave's
    // accesses in order, so the wave needs no barrier with itself - only the compiler must keep the order
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    park(o0);
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    if (firstPlane(ci + 1) < p.Cout) fetch(firstPlane(ci + 1));
    __builtin_amdgcn_s_setprio(0);

    for (int o = 0; o < oc; ++o) {
      const float *gp = lds + o * plane + laneB;
      const float *wp = lds + laneA + o * 4 * KKP;
      if constexpr (CT) {
        constexpr int NRB = T + Sh::SPAN, NCB = Sh::SPAN + 1;
        float bv[NRB][NCB];
#pragma unroll
        for (int x = 0; x < NRB; ++x)
#pragma unroll
          for (int y = 0; y < NCB; ++y) bv[x][y] = gp[x * PITCH + y];
        float av[Sh::KKP];
#pragma unroll
        for (int q = 0; q < Sh::KKP / 4; ++q) {
          const float4 f = reinterpret_cast<const float4 *>(wp)[q];
          av[4 * q] = f.x, av[4 * q + 1] = f.y, av[4 * q + 2] = f.z, av[4 * q + 3] = f.w;
        }
#pragma unroll
        for (int ph = 0; ph < S; ++ph)
#pragma unroll
          for (int pw = 0; pw < S; ++pw)
#pragma unroll
            for (int a = 0; a < fpTaps(ph, PADC, S, KC); ++a)
#pragma unroll
              for (int b = 0; b < fpTaps(pw, PADC, S, KC); ++b) {
                const int kh = fpRem(ph, PADC, S) + a * S, kw = fpRem(pw, PADC, S) + b * S;
                const int x0 = fpQ0(ph, PADC, S) - a - Sh::LO, y0 = fpQ0(pw, PADC, S) - b - Sh::LO;
#pragma unroll
                for (int t = 0; t < T; ++t)
                  acc[t][ph][pw] =
                      __builtin_amdgcn_mfma_f32_4x4x1f32(av[kh * KC + kw], bv[t + x0][y0], acc[t][ph][pw], 0, 0, 0);
              }
      } else {
        // one table entry ahead: the operands of tap j + 1 are on their way from LDS while tap j multiplies
        struct Ops {
          float a, b[T];
        };
        auto load = [&](unsigned e) {
          Ops r;
          r.a = wp[e & 0xffff];
          const float *gq = gp + (e >> 16);
#pragma unroll
          for (int t = 0; t < T; ++t) r.b[t] = gq[t * PITCH];
          return r;
        };
#pragma unroll
        for (int ph = 0; ph < S; ++ph)
#pragma unroll
          for (int pw = 0; pw < S; ++pw) {
            const int j0 = tp.first[ph * S + pw], j1 = tp.first[ph * S + pw + 1];
            if (j0 >= j1) continue;
            Ops x = load(tp.e[j0]), y;
            for (int j = j0; j < j1; j += 2) {
              if (j + 1 < j1) y = load(tp.e[j + 1]);
#pragma unroll
              for (int t = 0; t < T; ++t)
                acc[t][ph][pw] = __builtin_amdgcn_mfma_f32_4x4x1f32(x.a, x.b[t], acc[t][ph][pw], 0, 0, 0);
              if (j + 1 >= j1) break;
              if (j + 2 < j1) x = load(tp.e[j + 2]);
#pragma unroll
              for (int t = 0; t < T; ++t)
                acc[t][ph][pw] = __builtin_amdgcn_mfma_f32_4x4x1f32(y.a, y.b[t], acc[t][ph][pw], 0, 0, 0);
            }
          }
      }
    }
  }

  // The four partial sums of every accumulator meet in LDS and are added in wave order; each wave adds and stores
  // a quarter of them. A lane holds, per tile and phase, the planes 0..3 of one gradInput position.
  const long giImg = (long)p.Cin * p.H * p.W;
  const __amdgpu_buffer_rsrc_t gir = dev::makeRsrc(p.gi + n * giImg, giImg * 4);
  const int giPlaneBytes = p.H * p.W * 4;
  __builtin_amdgcn_s_setprio(2);
  constexpr int QB = NQ < kFpRedQ ? NQ : kFpRedQ;
  float4v *red = reinterpret_cast<float4v *>(ldsAll);  // [wave][QB][64 lanes]
#pragma unroll
  for (int q0 = 0; q0 < NQ; q0 += QB) {
    __syncthreads();  // the chunks (or the pass before) are out of LDS
#pragma unroll
    for (int q = q0; q < q0 + QB && q < NQ; ++q) red[(wave * QB + (q - q0)) * 64 + lane] = acc[q / (S * S)][(q / S) % S][q % S];
    __syncthreads();
#pragma unroll
    for (int q = q0; q < q0 + QB && q < NQ; ++q) {
      if ((q & 3) != wave) continue;
      float4v v = red[(q - q0) * 64 + lane];
#pragma unroll
      for (int wv_ = 1; wv_ < kFpWaves; ++wv_) v += red[(wv_ * QB + (q - q0)) * 64 + lane];
      const int t = q / (S * S), ph = (q / S) % S, pw = q % S;
      const int h = S * (I0 + lr * T + t) + ph, w = S * (J0 + lc) + pw;
      const int off = (h < p.H && w < p.W) ? (h * p.W + w) * 4 : dev::kBufOob;
#pragma unroll
      for (int c = 0; c < 4; ++c)  // a plane that does not exist is an offset out of range: no branch between the stores
        __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v[c] + bias[c]), gir, c < p.Cin ? off : dev::kBufOob,
                                              c < p.Cin ? c * giPlaneBytes : 0, 0);
    }
  }
}
