// 1x1 convolutions (stride 1, no padding) with a short reduction: out(n, o, l) = bias(o) + sum_c W(o, c) x(n, c, l),
// lib/THCUNN/generic/SpatialConvolutionMM.cu:129-194 with K = Cin of 32 ... 256 (the pointwise layers of
// MobileNet / the bottleneck layers of ResNet, forward and - with transposed weights - gradInput; the host
// side sends K = 32, 64 and 128 here).
//
// With so few k-steps a tile-per-workgroup GEMM is all prologue and epilogue, and at K = 128 the layer needs
// ~5 TB/s of HBM traffic at the full MFMA rate: reads, multiplications and writes have to overlap all the time,
// inside every wave, or their times add up. This kernel turns the loop around:
//  * the weights are stationary: a wave keeps its 32*MR rows of W as the MFMA operands of all K/2 k-pairs in
//    registers (K/2 * MR VGPRs) for the life of the kernel;
//  * the positions stream: a workgroup owns a run of column tiles (32 positions each, numbered over the
//    flattened (n, l) positions of the batch) and moves along it in chunks of CT tiles. Chunk c is multiplied
//    out of one LDS buffer while chunk c + 1 waits in registers and chunk c + 2 is in flight from memory; the
//    rows of x are contiguous along l, so a chunk arrives as 16-byte loads and is parked k-major, exactly the
//    layout v_mfma_f32_32x32x2_f32 reads its second operand in (no transpose), fetched a few k-pairs ahead;
//  * results leave a job late: the accumulators of a finished group of tiles stay in a second register set and
//    their stores are dealt one by one between the MFMAs of the next group, so the matrix pipe always has
//    queued work and the memory system sees a steady trickle of full 128-byte lines instead of a burst from
//    every CU at once. Rows and image jumps are scalar / per-lane offsets of one buffer resource; lanes and rows
//    without an output carry an out-of-range offset and the buffer unit drops their stores.
// Results are independent of the decomposition (every output element is one K-long sum in k order).
#pragma once

struct PwArgs {
  const float *w;     // (M x K) row-major, 16-byte aligned; TRANS kernels: (K x M) row-major, read as its transpose
  const float *x;     // (N, K, L), 16-byte aligned, L % 4 == 0
  float *out;         // (N, M, L), 16-byte aligned
  const float *bias;  // M or null
  int M, L, P;        // rows (M % 8 == 0); positions per image; positions of the batch, N * L
  int nTiles;         // column tiles of 32 positions: ceil(P / 32)
  int tilesPerWg;     // consecutive column tiles per workgroup
  unsigned magicL;    // dev::magicOf(L)
  int xBytes, outBytes;  // < 2^31
};

// LDS floats of a workgroup: the two chunk buffers, or the slab of weights that passes through them first
constexpr int pwLdsFloats(int K, int MR, int WR, int CT) {
  const int ksl = K < 128 ? K : 128, rows = 32 * MR * WR;
  const int chunks = 2 * K * 32 * CT, slab = rows * (ksl + 4), slabT = ksl * (rows + 4);
  return chunks > slab ? (chunks > slabT ? chunks : slabT) : (slab > slabT ? slab : slabT);
}

// What a job (the MFMAs of JP column tiles x MR row tiles) leaves behind: its accumulators and, per tile and
// group of 8 rows, the lane's byte offset into out (position part; the row part is a scalar offset), out of
// range where there is nothing to store.
template <int JP, int MR>
struct PwDone {
  float16v acc[JP][MR];
  int voff[JP][MR][4];
};

// K: reduction length. A wave multiplies 32*MR rows; of the NW waves of a workgroup WR sit side by side along the
// rows and NW / WR along the positions (they share the chunk in LDS). CT: column tiles per chunk.
// NW = 8 is one workgroup per CU, two waves per SIMD that take turns on the matrix pipe and meet at every chunk's
// barrier: they advance together. (Two independent workgroups of 4 waves per CU do not - the SIMD favours the
// older wave, one workgroup of each pair finishes at 60 % of the time and the other runs the rest alone.)
// RELU: the stored value is v > 0 ? v : 0. TRANS: the weights are given as (K x M) and used as their transpose -
// the gradInput pass of a 1x1 convolution (gradInput = W^T gradOutput) reads the layer's own weight tensor.
template <int K, int MR, int WR, int CT, int NW, bool RELU = false, bool TRANS = false>
__global__ void __launch_bounds__(64 * NW, 2)
convPointwiseKernel(PwArgs p) {
  constexpr int BLK = 64 * NW;
  constexpr int WC = NW / WR;
  constexpr int CP = 32 * CT;          // positions of a chunk = floats per k row in LDS
  constexpr int G = CP / 4;            // 16-byte groups per k row
  constexpr int KS = BLK / G;          // k rows one load instruction of the workgroup covers
  constexpr int NLD = K / KS;          // loads per lane and chunk
  constexpr int JOBS = CT / WC;        // column tiles of a chunk per wave
  constexpr bool SWZ = CP >= 64;       // odd k rows keep their 32-position halves swapped: both k rows of an MFMA
                                       // operand then sit in disjoint banks (CP = 32 does that by itself)
  constexpr int JP = (MR == 1 && JOBS % 2 == 0) ? 2 : 1;  // column tiles multiplied side by side: a job has JP * MR
  constexpr int NJ = JOBS / JP;                           // independent accumulation chains; jobs per chunk and wave
  constexpr int S = K / 2;                                // MFMAs per chain
  constexpr int NST = JP * MR * 16;                       // stores of a job
  constexpr int PF = S < 8 ? S : 8;                       // k-pairs the LDS operands are fetched ahead
  static_assert(CT % WC == 0 && K % KS == 0 && KS % 2 == 0 && NLD >= 1, "chunk shape");
  using Done = PwDone<JP, MR>;
  extern __shared__ float4 pwSmem[];  // two buffers of K x CP floats
  float *Bs = reinterpret_cast<float *>(pwSmem);
  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wr = wave % WR, wc = wave / WR;
  const int grp = lane >> 5, idx = lane & 31;
  const int m0 = (int)blockIdx.y * (32 * MR * WR) + wr * (32 * MR);  // first row of the wave

  const int tile0 = (int)blockIdx.x * p.tilesPerWg, tile1 = min(p.nTiles, tile0 + p.tilesPerWg);
  if (tile0 >= tile1) return;  // the whole workgroup: no barrier has been reached
  const int nChunks = (tile1 - tile0 + CT - 1) / CT;

  const __amdgpu_buffer_rsrc_t xr = dev::makeRsrc(p.x, p.xBytes), outr = dev::makeRsrc(p.out, p.outBytes);

  // ---- the lane's part of a chunk load: 16-byte group gl of the chunk's positions, k rows ks + KS * i ----
  const int gl = t % G, ks = t / G;
  const int ldsStore = ks * CP + ((gl * 4) ^ (SWZ ? (ks & 1) << 5 : 0));
  const int rowStep = __builtin_amdgcn_readfirstlane(KS * p.L * 4);  // bytes between the rows of consecutive loads
  u32x4 stage[NLD];
  auto issue = [&](int c) {
    int pos = (tile0 + c * CT) * 32 + gl * 4;
    pos = min(pos, p.P - 4);  // groups past the batch re-read its last one; their columns are never stored
    const int n = dev::fastDiv(pos, p.magicL), l = pos - n * p.L;
    const int off = ((n * K + ks) * p.L + l) * 4;
#pragma unroll
    for (int i = 0; i < NLD; ++i) stage[i] = __builtin_amdgcn_raw_buffer_load_b128(xr, off, i * rowStep, 0);
  };
  auto commit = [&](int buf) {
    u32x4 *dst = reinterpret_cast<u32x4 *>(Bs + buf * (K * CP) + ldsStore);
#pragma unroll
    for (int i = 0; i < NLD; ++i) dst[i * (KS * CP / 4)] = stage[i];
  };

  issue(0);  // in flight while the weights arrive

  // ---- stationary operands ----------------------------------------------------------------------------
  // first operand of MFMA s (k pair 2s, 2s + 1): lane (i = lane % 32, kk = lane / 32) holds W[row i][2s + kk].
  // The workgroup's rows of W come in through LDS (coalesced 16-byte loads, slabs of up to 128 columns, row pitch
  // + 4 floats against bank conflicts): a lane fetching its own rows from memory touches 32 cache lines per load.
  float a[MR][S];
  float16v biasv[MR];
  {
    constexpr int ROWS = 32 * MR * WR;       // rows of the workgroup
    constexpr int KSL = K < 128 ? K : 128;   // columns per slab
    constexpr int WP = KSL + 4;              // LDS row pitch in floats
    constexpr int C4 = KSL / 4;              // 16-byte groups per row of a slab
    constexpr int NW4 = ROWS * C4;           // 16-byte groups of a slab
    static_assert(ROWS * WP <= pwLdsFloats(K, MR, WR, CT), "the slab fits the LDS the host asks for");
    const int rowW0 = (int)blockIdx.y * ROWS;
#pragma unroll
    for (int slab = 0; slab < K / KSL; ++slab) {
      if (slab > 0) __syncthreads();  // the previous slab has been read
      if constexpr (!TRANS) {
#pragma unroll
        for (int u = 0; u < (NW4 + BLK - 1) / BLK; ++u) {
          const int i = u * BLK + t;
          if (i < NW4) {
            const int row = i / C4, c4 = i - row * C4;
            const int grow = min(rowW0 + row, p.M - 1);  // rows past M are computed from row M - 1 and never stored
            *reinterpret_cast<float4 *>(Bs + row * WP + c4 * 4) =
                *reinterpret_cast<const float4 *>(p.w + (long)grow * K + slab * KSL + c4 * 4);
          }
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < MR; ++r) {
          const float *wrow = Bs + (wr * (32 * MR) + 32 * r + idx) * WP;
#pragma unroll
          for (int j = 0; j < C4; ++j) {
            const float4 q = *reinterpret_cast<const float4 *>(wrow + 4 * j);
            a[r][slab * (KSL / 2) + 2 * j] = grp ? q.y : q.x;
            a[r][slab * (KSL / 2) + 2 * j + 1] = grp ? q.w : q.z;
          }
        }
      } else {
        // the slab as memory holds it: KSL rows (k) of the workgroup's ROWS consecutive columns (m), coalesced along
        // m; a lane then picks its operands column-wise (consecutive lanes read consecutive floats)
        constexpr int WPT = ROWS + 4, R4 = ROWS / 4, NT4 = KSL * R4;
        static_assert(KSL * WPT <= pwLdsFloats(K, MR, WR, CT), "the transposed slab fits the LDS the host asks for");
#pragma unroll
        for (int u = 0; u < (NT4 + BLK - 1) / BLK; ++u) {
          const int i = u * BLK + t;
          if (i < NT4) {
            const int k = i / R4, j4 = i - k * R4;
            const int m = min(rowW0 + 4 * j4, p.M - 4);  // M % 8 == 0; columns past M repeat the last ones, never stored
            *reinterpret_cast<float4 *>(Bs + k * WPT + 4 * j4) =
                *reinterpret_cast<const float4 *>(p.w + (long)(slab * KSL + k) * p.M + m);
          }
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < MR; ++r) {
          const float *wcol = Bs + grp * WPT + (wr * (32 * MR) + 32 * r + idx);
#pragma unroll
          for (int j = 0; j < KSL / 2; ++j) a[r][slab * (KSL / 2) + j] = wcol[2 * j * WPT];
        }
      }
    }
    // an accumulator register v holds row 8 * (v / 4) + 4 * (lane / 32) + v % 4 of the tile
#pragma unroll
    for (int r = 0; r < MR; ++r)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int brow = m0 + 32 * r + 8 * (v >> 2) + 4 * grp + (v & 3);
        biasv[r][v] = (p.bias && brow < p.M) ? p.bias[brow] : 0.f;
      }
    __syncthreads();  // the slab is read: the buffers are free for the chunks
  }

  Done X, Y;
#pragma unroll
  for (int q = 0; q < JP; ++q)
#pragma unroll
    for (int r = 0; r < MR; ++r)
#pragma unroll
      for (int q8 = 0; q8 < 4; ++q8) X.voff[q][r][q8] = Y.voff[q][r][q8] = dev::kBufOob;

  // store number i of a finished job (i is a constant once the loops around the call are unrolled)
  auto storeOne = [&](const Done &d, int i) {
    const int q = i / (MR * 16), r = (i / 16) % MR, v = i % 16;
    const int rowBase = m0 + 32 * r + 8 * (v >> 2) + (v & 3);  // wave-uniform: a scalar offset
    float o = d.acc[q][r][v];
    // one instruction between the MFMAs: max(v, 0) is v > 0 ? v : 0 for every input (a NaN gives 0, -0 gives +0)
    if (RELU) asm volatile("v_max_f32 %0, 0, %1" : "=v"(o) : "v"(o));
    // K >= 64: streaming stores (the nt policy bit). Measured at N = 64: 64 -> 128 at 56 x 56 54.2 -> 43.6 us, 64 -> 64
    // 33.7 -> 27.1 us, 128 -> 128 at 56 x 56 77.2 -> 73.5 us, at 28 x 28 24.2 -> 22.4 us; at K = 32 plain stores are level
    // or better (32 -> 64 at 112 x 112: 44.9 against 46.1 us).
    __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(o), outr, d.voff[q][r][v >> 2], rowBase * p.L * 4, K >= 64 ? 2 : 0);
  };
  // second operand of MFMA s of column tile ct: lane (j = lane % 32, kk = lane / 32) holds x[2s + kk][position j]
  auto bAddr = [&](int buf, int ct) {
    return Bs + buf * (K * CP) + grp * CP + (((ct ^ (SWZ ? grp : 0)) << 5) + idx);
  };
  // j: job of the chunk (compile-time); cur: where it accumulates; prev: the job before it, stored meanwhile;
  // mid(): the hand-over of the next chunks, run inside the chunk's first job
  auto job = [&](auto jc, int c, int buf, Done &cur, const Done &prev, auto mid) {
    constexpr int j = decltype(jc)::value;
    if (tile0 + c * CT + wc + WC * (j * JP) >= tile1) {  // wave-uniform: the run ends before the job's first tile
#pragma unroll
      for (int i = 0; i < NST; ++i) storeOne(prev, i);
      if (j == 0) mid();
#pragma unroll
      for (int q = 0; q < JP; ++q)
#pragma unroll
        for (int r = 0; r < MR; ++r)
#pragma unroll
          for (int q8 = 0; q8 < 4; ++q8) cur.voff[q][r][q8] = dev::kBufOob;
      return;
    }
    const float *bp[JP];
#pragma unroll
    for (int q = 0; q < JP; ++q) {
      const int ct = wc + WC * (j * JP + q);
      bp[q] = bAddr(buf, ct);
      const int tile = tile0 + c * CT + ct;
      const int pos = tile * 32 + idx;
      const int n = dev::fastDiv(min(pos, p.P - 1), p.magicL), l = pos - n * p.L;
      const int off = ((n * p.M + 4 * grp) * p.L + l) * 4;
      const bool ok = tile < tile1 && pos < p.P;
#pragma unroll
      for (int r = 0; r < MR; ++r)
#pragma unroll
        for (int q8 = 0; q8 < 4; ++q8)
          cur.voff[q][r][q8] = (ok && m0 + 32 * r + 8 * q8 < p.M) ? off : dev::kBufOob;  // M % 8 == 0: 8 rows are there or not
    }
    float bv[JP][PF];  // operands in flight from LDS
#pragma unroll
    for (int s = 0; s < PF; ++s)
#pragma unroll
      for (int q = 0; q < JP; ++q) bv[q][s] = bp[q][s * 2 * CP];
    // the k-pairs in blocks of 16 with compile-time bounds, so that every register of the stationary operands and
    // of the operand ring is named statically however long the reduction is
    auto block = [&](auto sbc) {
      constexpr int SB = decltype(sbc)::value;
#pragma unroll
      for (int s = SB; s < (SB + 16 < S ? SB + 16 : S); ++s) {
        // (the waves that share a SIMD hand over at different points of the chunk, so that one of them always
        // has MFMAs to issue: wc is the same for the four waves of a row of SIMDs)
        if (j == 0 && s == S / 4 && (wc & 1) == 0) mid();
        if (j == 0 && s == (3 * S) / 4 && (wc & 1) == 1) mid();
#pragma unroll
        for (int q = 0; q < JP; ++q) {
          const float b = bv[q][s % PF];
          if (s + PF < S) bv[q][s % PF] = bp[q][(s + PF) * 2 * CP];
#pragma unroll
          for (int r = 0; r < MR; ++r)
            cur.acc[q][r] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[r][s], b, s == 0 ? biasv[r] : cur.acc[q][r], 0, 0, 0);
        }
        // the previous job's stores, dealt evenly over the k-pairs
#pragma unroll
        for (int i = 0; i < NST; ++i)
          if (i * S / NST == s) storeOne(prev, i);
        // nothing moves across a k-pair: the operand fetches stay PF pairs ahead of their use and the stores stay
        // spread out (the instruction scheduler otherwise pulls the fetches next to the MFMAs and bunches the stores)
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    block(std::integral_constant<int, 0>{});
    if constexpr (S > 16) block(std::integral_constant<int, 16>{});
    if constexpr (S > 32) block(std::integral_constant<int, 32>{});
    if constexpr (S > 48) block(std::integral_constant<int, 48>{});
    if constexpr (S > 64) block(std::integral_constant<int, 64>{});
    if constexpr (S > 80) block(std::integral_constant<int, 80>{});
    if constexpr (S > 96) block(std::integral_constant<int, 96>{});
    if constexpr (S > 112) block(std::integral_constant<int, 112>{});
    static_assert(S <= 128, "reduction length");
  };
  // a chunk: its NJ jobs, alternating between the two register sets
  auto chunk = [&](int c, Done &first, Done &second) {
    const int buf = c & 1;
    auto mid = [&]() {
      __builtin_amdgcn_sched_barrier(0);
      if (c + 1 < nChunks) commit(buf ^ 1);
      if (c + 2 < nChunks) issue(c + 2);
      __builtin_amdgcn_sched_barrier(0);
    };
    job(std::integral_constant<int, 0>{}, c, buf, first, second, mid);
    if constexpr (NJ >= 2) job(std::integral_constant<int, 1>{}, c, buf, second, first, mid);
    if constexpr (NJ >= 3) job(std::integral_constant<int, 2>{}, c, buf, first, second, mid);
    if constexpr (NJ >= 4) job(std::integral_constant<int, 3>{}, c, buf, second, first, mid);
    if constexpr (NJ >= 5) job(std::integral_constant<int, 4>{}, c, buf, first, second, mid);
    if constexpr (NJ >= 6) job(std::integral_constant<int, 5>{}, c, buf, second, first, mid);
    if constexpr (NJ >= 7) job(std::integral_constant<int, 6>{}, c, buf, first, second, mid);
    if constexpr (NJ >= 8) job(std::integral_constant<int, 7>{}, c, buf, second, first, mid);
    static_assert(NJ <= 8, "jobs per chunk");
    __syncthreads();
  };

  // ---- pipeline ------------------------------------------------------------------------------------------
  commit(0);
  if (nChunks > 1) issue(1);
  __syncthreads();
  bool lastInX;
  if constexpr (NJ % 2 == 0) {
    for (int c = 0; c < nChunks; ++c) chunk(c, X, Y);  // every chunk ends in Y
    lastInX = false;
  } else {
    int c = 0;
    for (; c + 1 < nChunks; c += 2) {
      chunk(c, X, Y);
      chunk(c + 1, Y, X);
    }
    lastInX = false;  // an even number of chunks ends in Y (NJ odd: chunk c + 1 ends in its first set)
    if (c < nChunks) {
      chunk(c, X, Y);
      lastInX = true;
    }
  }
  // the last job's results
  if (lastInX) {
#pragma unroll
    for (int i = 0; i < NST; ++i) storeOne(X, i);
  } else {
#pragma unroll
    for (int i = 0; i < NST; ++i) storeOne(Y, i);
  }
}
