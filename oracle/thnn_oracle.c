/*
 * thnn_oracle.c - CPU restatement of the THCUNN spatial-conv hot path.
 *
 * TEST INFRASTRUCTURE ONLY. This file is the checker the HIP kernels are
 * compared against and the CPU baseline that bench.py times; nothing in the
 * shipped library links, loads or calls it.
 *
 * Each function restates, on packed (contiguous) fp32 NCHW arrays, the
 * algorithm of the reference file:line it cites: the same loop structure
 * (per-sample / per-plane im2col + GEMM for the convolutions, per-channel
 * two-pass statistics for batch normalisation, per-output window scans for
 * pooling), the same accumulate-into semantics and the same index rules.
 * Where CPU-THNN (torch/nn, not part of the reference tree) is known to use a
 * wider accumulator than the CUDA code (double sums in batch normalisation),
 * the wider one is used, since CPU-THNN is the stated ground truth.
 *
 * Pinning (see tests/test_oracle_*.py): every function here is checked against
 * the reference's own known answers (test.lua:2597-2616 average pooling 3 and
 * 3/4; test.lua:6602-6661 depthwise == per-channel SpatialConvolution), against
 * brute-force NumPy loops that restate the closed-form definitions, against
 * PyTorch-CPU library routines (conv2d/batch_norm/max_pool2d/avg_pool2d and
 * autograd) and against adjoint identities. No function is "parity unpinned".
 *
 * OpenMP is applied over the batch / plane loop, the way CPU-THNN does.
 */
#include <float.h>
#include <math.h>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_INDEX_BASE 1 /* TH_INDEX_BASE of Lua-torch builds */

int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ------------------------------------------------------------------ im2col --
 * lib/THCUNN/im2col.h:9-38 (kernel) and :40-61 (output extent with dilation).
 * col is (C*kH*kW, oH*oW); entry ((c*kH+i)*kW+j, oh*oW+ow) =
 * im[c][oh*dH-padH+i*dilH][ow*dW-padW+j*dilW] or 0 outside the image. */
static int conv_out(int in, int pad, int k, int stride, int dil) {
  return (in + 2 * pad - (dil * (k - 1) + 1)) / stride + 1;
}

void oracle_im2col(const float *im, int C, int H, int W, int kH, int kW, int padH, int padW, int dH,
                   int dW, int dilH, int dilW, float *col) {
  int oH = conv_out(H, padH, kH, dH, dilH), oW = conv_out(W, padW, kW, dW, dilW);
  for (int c = 0; c < C; ++c)
    for (int i = 0; i < kH; ++i)
      for (int j = 0; j < kW; ++j) {
        float *row = col + (((size_t)c * kH + i) * kW + j) * oH * oW;
        for (int oh = 0; oh < oH; ++oh) {
          int h = oh * dH - padH + i * dilH;
          for (int ow = 0; ow < oW; ++ow) {
            int w = ow * dW - padW + j * dilW;
            row[oh * oW + ow] =
                (h >= 0 && w >= 0 && h < H && w < W) ? im[((size_t)c * H + h) * W + w] : 0.f;
          }
        }
      }
}

/* ------------------------------------------------------------------ col2im --
 * lib/THCUNN/im2col.h:63-102: one gather per image pixel over every column
 * entry that maps onto it, accumulated in float (accreal of the Cuda type). */
void oracle_col2im(const float *col, int C, int H, int W, int oH, int oW, int kH, int kW, int padH,
                   int padW, int dH, int dW, int dilH, int dilW, float *im) {
  int extW = (kW - 1) * dilW + 1, extH = (kH - 1) * dilH + 1;
  for (int c = 0; c < C; ++c)
    for (int y = 0; y < H; ++y)
      for (int x = 0; x < W; ++x) {
        float val = 0.f;
        int w_im = x + padW, h_im = y + padH;
        int ws = (w_im < extW) ? 0 : (w_im - extW) / dW + 1;
        int we = w_im / dW + 1 < oW ? w_im / dW + 1 : oW;
        int hs = (h_im < extH) ? 0 : (h_im - extH) / dH + 1;
        int he = h_im / dH + 1 < oH ? h_im / dH + 1 : oH;
        for (int hc = hs; hc < he; ++hc)
          for (int wc = ws; wc < we; ++wc) {
            int hk = h_im - hc * dH, wk = w_im - wc * dW;
            if (hk % dilH == 0 && wk % dilW == 0) {
              hk /= dilH;
              wk /= dilW;
              val += col[((((size_t)c * kH + hk) * kW + wk) * oH + hc) * oW + wc];
            }
          }
        im[((size_t)c * H + y) * W + x] = val;
      }
}

/* ------------------------------------------------------------- small GEMMs --
 * Row-major helpers standing in for the column-major cuBLAS calls of the
 * wrappers. C(MxN) = beta*C + alpha * A(MxK) * B(KxN). */
static void gemm_nn(int M, int N, int K, float alpha, const float *A, const float *B, float beta,
                    float *C) {
#pragma omp parallel for schedule(static) if ((size_t)M * N * K > 200000)
  for (int i = 0; i < M; ++i) {
    float *c = C + (size_t)i * N;
    if (beta == 0.f)
      for (int j = 0; j < N; ++j) c[j] = 0.f;
    else if (beta != 1.f)
      for (int j = 0; j < N; ++j) c[j] *= beta;
    for (int k = 0; k < K; ++k) {
      float a = alpha * A[(size_t)i * K + k];
      const float *b = B + (size_t)k * N;
      for (int j = 0; j < N; ++j) c[j] += a * b[j];
    }
  }
}
/* C(KxN) = A(MxK)^T * B(MxN) */
static void gemm_tn(int M, int N, int K, const float *A, const float *B, float *C) {
#pragma omp parallel for schedule(static) if ((size_t)M * N * K > 200000)
  for (int k = 0; k < K; ++k) {
    float *c = C + (size_t)k * N;
    for (int j = 0; j < N; ++j) c[j] = 0.f;
    for (int i = 0; i < M; ++i) {
      float a = A[(size_t)i * K + k];
      const float *b = B + (size_t)i * N;
      for (int j = 0; j < N; ++j) c[j] += a * b[j];
    }
  }
}
/* C(MxK) += alpha * A(MxL) * B(KxL)^T ; the dot over L is taken in double so
 * the checker is closer to the exact sum than either fp32 implementation */
static void gemm_nt_acc(int M, int K, int L, float alpha, const float *A, const float *B, float *C) {
#pragma omp parallel for schedule(static) collapse(2) if ((size_t)M * K * L > 200000)
  for (int i = 0; i < M; ++i)
    for (int k = 0; k < K; ++k) {
      const float *a = A + (size_t)i * L, *b = B + (size_t)k * L;
      double s = 0.0;
      for (int l = 0; l < L; ++l) s += (double)a[l] * (double)b[l];
      C[(size_t)i * K + k] += alpha * (float)s;
    }
}

/* ---------------------------------------------- SpatialDepthWiseConvolution --
 * weight (M, C, kH, kW), bias (M, C) or NULL, input (N, C, H, W),
 * output (N, C*M, oH, oW) with out-channel c*M + j
 * (lib/THCUNN/generic/SpatialDepthWiseConvolution.cu:121,244). */

/* generic/SpatialDepthWiseConvolution.cu:150-226: for each (n, c): out = bias
 * broadcast (or zero), im2col of the single plane, out += W_c(M x kHkW) * col */
void oracle_dwconv_updateOutput(const float *in, const float *weight, const float *bias, float *out,
                                int N, int C, int M, int H, int W, int kW, int kH, int dW, int dH,
                                int padW, int padH) {
  int oH = conv_out(H, padH, kH, dH, 1), oW = conv_out(W, padW, kW, dW, 1);
  int K = kH * kW, L = oH * oW;
#pragma omp parallel
  {
    float *col = (float *)malloc(sizeof(float) * (size_t)K * L);
    float *wc = (float *)malloc(sizeof(float) * (size_t)M * K);
#pragma omp for collapse(2) schedule(static)
    for (int n = 0; n < N; ++n)
      for (int c = 0; c < C; ++c) {
        float *o = out + ((size_t)n * C + c) * M * L;
        /* transposed weight/bias views (:87-101): W_c[j][k] = weight[j][c][k] */
        for (int j = 0; j < M; ++j) {
          memcpy(wc + (size_t)j * K, weight + ((size_t)j * C + c) * K, sizeof(float) * K);
          float b = bias ? bias[(size_t)j * C + c] : 0.f;
          for (int l = 0; l < L; ++l) o[(size_t)j * L + l] = b;
        }
        oracle_im2col(in + ((size_t)n * C + c) * H * W, 1, H, W, kH, kW, padH, padW, dH, dW, 1, 1, col);
        for (int j = 0; j < M; ++j)
          for (int k = 0; k < K; ++k) {
            float a = wc[(size_t)j * K + k];
            const float *b = col + (size_t)k * L;
            float *oo = o + (size_t)j * L;
            for (int l = 0; l < L; ++l) oo[l] += a * b[l];
          }
      }
    free(col);
    free(wc);
  }
}

/* generic/SpatialDepthWiseConvolution.cu:350-395: for each (n, c):
 * gradCol(kHkW x L) = W_c^T * gradOut_{n,c}(M x L); gradIn plane = col2im */
void oracle_dwconv_updateGradInput(const float *gradOut, const float *weight, float *gradIn, int N,
                                   int C, int M, int H, int W, int kW, int kH, int dW, int dH,
                                   int padW, int padH) {
  int oH = conv_out(H, padH, kH, dH, 1), oW = conv_out(W, padW, kW, dW, 1);
  int K = kH * kW, L = oH * oW;
#pragma omp parallel
  {
    float *col = (float *)malloc(sizeof(float) * (size_t)K * L);
#pragma omp for collapse(2) schedule(static)
    for (int n = 0; n < N; ++n)
      for (int c = 0; c < C; ++c) {
        const float *g = gradOut + ((size_t)n * C + c) * M * L;
        for (int k = 0; k < K; ++k) {
          float *cc = col + (size_t)k * L;
          for (int l = 0; l < L; ++l) cc[l] = 0.f;
          for (int j = 0; j < M; ++j) {
            float a = weight[((size_t)j * C + c) * K + k];
            const float *gg = g + (size_t)j * L;
            for (int l = 0; l < L; ++l) cc[l] += a * gg[l];
          }
        }
        oracle_col2im(col, 1, H, W, oH, oW, kH, kW, padH, padW, dH, dW, 1, 1,
                      gradIn + ((size_t)n * C + c) * H * W);
      }
    free(col);
  }
}

/* generic/SpatialDepthWiseConvolution.cu:531-615: for each (n, c):
 * gradW_c(M x kHkW) += scale * gradOut_{n,c}(M x L) * col^T ;
 * gradBias_c(M) += scale * gradOut_{n,c} * ones. Accumulates into the values
 * gradWeight (M,C,kH,kW) / gradBias (M,C) already hold (:478, :573, :619-629). */
void oracle_dwconv_accGradParameters(const float *in, const float *gradOut, float *gradWeight,
                                     float *gradBias, int N, int C, int M, int H, int W, int kW,
                                     int kH, int dW, int dH, int padW, int padH, float scale) {
  int oH = conv_out(H, padH, kH, dH, 1), oW = conv_out(W, padW, kW, dW, 1);
  int K = kH * kW, L = oH * oW;
#pragma omp parallel
  {
    float *col = (float *)malloc(sizeof(float) * (size_t)K * L);
#pragma omp for schedule(static)
    for (int c = 0; c < C; ++c)
      for (int n = 0; n < N; ++n) {
        oracle_im2col(in + ((size_t)n * C + c) * H * W, 1, H, W, kH, kW, padH, padW, dH, dW, 1, 1, col);
        const float *g = gradOut + ((size_t)n * C + c) * M * L;
        for (int j = 0; j < M; ++j) {
          const float *gg = g + (size_t)j * L;
          for (int k = 0; k < K; ++k) {
            const float *cc = col + (size_t)k * L;
            double s = 0.0;
            for (int l = 0; l < L; ++l) s += (double)gg[l] * (double)cc[l];
            gradWeight[((size_t)j * C + c) * K + k] += scale * (float)s;
          }
          if (gradBias) {
            double s = 0.0;
            for (int l = 0; l < L; ++l) s += (double)gg[l];
            gradBias[(size_t)j * C + c] += scale * (float)s;
          }
        }
      }
    free(col);
  }
}

/* ------------------------------------------------------ SpatialConvolutionMM --
 * weight (Cout, Cin*kH*kW), bias (Cout) or NULL, input (N, Cin, H, W). */

/* generic/SpatialConvolutionMM.cu:129-194: per sample: out = bias broadcast
 * (or zero); im2col; out(Cout x L) += W(Cout x K) * col(K x L) */
static void conv_forward(const float *in, const float *weight, const float *bias, float *out,
                         int N, int Cin, int Cout, int H, int W, int kW, int kH, int dW,
                         int dH, int padW, int padH, int dilW, int dilH) {
  int oH = conv_out(H, padH, kH, dH, dilH), oW = conv_out(W, padW, kW, dW, dilW);
  int K = Cin * kH * kW, L = oH * oW;
  float *col = (float *)malloc(sizeof(float) * (size_t)K * L);
  for (int n = 0; n < N; ++n) {
    float *o = out + (size_t)n * Cout * L;
    for (int oc = 0; oc < Cout; ++oc) {
      float b = bias ? bias[oc] : 0.f;
      for (int l = 0; l < L; ++l) o[(size_t)oc * L + l] = b;
    }
    oracle_im2col(in + (size_t)n * Cin * H * W, Cin, H, W, kH, kW, padH, padW, dH, dW, dilH, dilW, col);
    gemm_nn(Cout, L, K, 1.f, weight, col, 1.f, o);
  }
  free(col);
}
void oracle_convmm_updateOutput(const float *in, const float *weight, const float *bias, float *out,
                                int N, int Cin, int Cout, int H, int W, int kW, int kH, int dW,
                                int dH, int padW, int padH) {
  conv_forward(in, weight, bias, out, N, Cin, Cout, H, W, kW, kH, dW, dH, padW, padH, 1, 1);
}
/* generic/SpatialDilatedConvolution.cu:69-190: the same per-sample bias fill, im2col (with
 * dilation, im2col.h:24-36) and GEMM */
void oracle_dilconv_updateOutput(const float *in, const float *weight, const float *bias, float *out,
                                 int N, int Cin, int Cout, int H, int W, int kW, int kH, int dW,
                                 int dH, int padW, int padH, int dilW, int dilH) {
  conv_forward(in, weight, bias, out, N, Cin, Cout, H, W, kW, kH, dW, dH, padW, padH, dilW, dilH);
}

/* generic/SpatialConvolutionMM.cu:272-308: per sample: gradCol(K x L) =
 * W^T * gradOut_n ; gradIn_n = col2im(gradCol) */
static void conv_grad_input(const float *gradOut, const float *weight, float *gradIn, int N,
                            int Cin, int Cout, int H, int W, int kW, int kH, int dW, int dH,
                            int padW, int padH, int dilW, int dilH) {
  int oH = conv_out(H, padH, kH, dH, dilH), oW = conv_out(W, padW, kW, dW, dilW);
  int K = Cin * kH * kW, L = oH * oW;
  float *col = (float *)malloc(sizeof(float) * (size_t)K * L);
  for (int n = 0; n < N; ++n) {
    gemm_tn(Cout, L, K, weight, gradOut + (size_t)n * Cout * L, col);
    oracle_col2im(col, Cin, H, W, oH, oW, kH, kW, padH, padW, dH, dW, dilH, dilW,
                  gradIn + (size_t)n * Cin * H * W);
  }
  free(col);
}
void oracle_convmm_updateGradInput(const float *gradOut, const float *weight, float *gradIn, int N,
                                   int Cin, int Cout, int H, int W, int kW, int kH, int dW, int dH,
                                   int padW, int padH) {
  conv_grad_input(gradOut, weight, gradIn, N, Cin, Cout, H, W, kW, kH, dW, dH, padW, padH, 1, 1);
}
/* generic/SpatialDilatedConvolution.cu:192-293 */
void oracle_dilconv_updateGradInput(const float *gradOut, const float *weight, float *gradIn, int N,
                                    int Cin, int Cout, int H, int W, int kW, int kH, int dW, int dH,
                                    int padW, int padH, int dilW, int dilH) {
  conv_grad_input(gradOut, weight, gradIn, N, Cin, Cout, H, W, kW, kH, dW, dH, padW, padH, dilW, dilH);
}

/* generic/SpatialConvolutionMM.cu:396-470: per sample: im2col;
 * gradW(Cout x K) += scale * gradOut_n(Cout x L) * col^T (beta = 1);
 * gradBias += scale * gradOut_n * ones */
static void conv_acc_grad(const float *in, const float *gradOut, float *gradWeight,
                          float *gradBias, int N, int Cin, int Cout, int H, int W, int kW,
                          int kH, int dW, int dH, int padW, int padH, int dilW, int dilH, float scale) {
  int oH = conv_out(H, padH, kH, dH, dilH), oW = conv_out(W, padW, kW, dW, dilW);
  int K = Cin * kH * kW, L = oH * oW;
  float *col = (float *)malloc(sizeof(float) * (size_t)K * L);
  for (int n = 0; n < N; ++n) {
    const float *g = gradOut + (size_t)n * Cout * L;
    oracle_im2col(in + (size_t)n * Cin * H * W, Cin, H, W, kH, kW, padH, padW, dH, dW, dilH, dilW, col);
    gemm_nt_acc(Cout, K, L, scale, g, col, gradWeight);
    if (gradBias)
      for (int oc = 0; oc < Cout; ++oc) {
        double s = 0.0;
        for (int l = 0; l < L; ++l) s += (double)g[(size_t)oc * L + l];
        gradBias[oc] += scale * (float)s;
      }
  }
  free(col);
}
void oracle_convmm_accGradParameters(const float *in, const float *gradOut, float *gradWeight,
                                     float *gradBias, int N, int Cin, int Cout, int H, int W, int kW,
                                     int kH, int dW, int dH, int padW, int padH, float scale) {
  conv_acc_grad(in, gradOut, gradWeight, gradBias, N, Cin, Cout, H, W, kW, kH, dW, dH, padW, padH, 1, 1, scale);
}
/* generic/SpatialDilatedConvolution.cu:295-432 */
void oracle_dilconv_accGradParameters(const float *in, const float *gradOut, float *gradWeight,
                                      float *gradBias, int N, int Cin, int Cout, int H, int W, int kW,
                                      int kH, int dW, int dH, int padW, int padH, int dilW, int dilH,
                                      float scale) {
  conv_acc_grad(in, gradOut, gradWeight, gradBias, N, Cin, Cout, H, W, kW, kH, dW, dH, padW, padH, dilW, dilH, scale);
}

/* ------------------------------------------ SpatialFull(Dilated)Convolution --
 * weight (Cin, Cout, kH, kW) = (Cin, Cout*kH*kW), bias (Cout) or NULL, input (N, Cin, H, W),
 * output (N, Cout, oH, oW) with oH = (H-1)*dH - 2*padH + dilH*(kH-1) + 1 + adjH
 * (lib/THCUNN/generic/SpatialFullDilatedConvolution.cu:104-105). */

/* generic/SpatialFullDilatedConvolution.cu:129-193: per sample:
 * columns(Cout*kH*kW x H*W) = W^T * input_n ; output_n = col2im(columns) ; output_n += bias */
void oracle_fullconv_updateOutput(const float *in, const float *weight, const float *bias, float *out,
                                  int N, int Cin, int Cout, int H, int W, int oH, int oW, int kW, int kH,
                                  int dW, int dH, int padW, int padH, int dilW, int dilH) {
  int Kf = Cout * kH * kW, HW = H * W;
  float *col = (float *)malloc(sizeof(float) * (size_t)Kf * HW);
  for (int n = 0; n < N; ++n) {
    float *o = out + (size_t)n * Cout * oH * oW;
    gemm_tn(Cin, HW, Kf, weight, in + (size_t)n * Cin * HW, col);
    oracle_col2im(col, Cout, oH, oW, H, W, kH, kW, padH, padW, dH, dW, dilH, dilW, o);
    if (bias)
      for (int oc = 0; oc < Cout; ++oc)
        for (int l = 0; l < oH * oW; ++l) o[(size_t)oc * oH * oW + l] += bias[oc];
  }
  free(col);
}

/* generic/SpatialFullDilatedConvolution.cu:262-298: per sample:
 * gradColumns = im2col(gradOutput_n) ; gradInput_n(Cin x H*W) = W * gradColumns */
void oracle_fullconv_updateGradInput(const float *gradOut, const float *weight, float *gradIn, int N,
                                     int Cin, int Cout, int H, int W, int oH, int oW, int kW, int kH,
                                     int dW, int dH, int padW, int padH, int dilW, int dilH) {
  int Kf = Cout * kH * kW, HW = H * W;
  float *col = (float *)malloc(sizeof(float) * (size_t)Kf * HW);
  for (int n = 0; n < N; ++n) {
    oracle_im2col(gradOut + (size_t)n * Cout * oH * oW, Cout, oH, oW, kH, kW, padH, padW, dH, dW, dilH, dilW, col);
    gemm_nn(Cin, HW, Kf, 1.f, weight, col, 0.f, gradIn + (size_t)n * Cin * HW);
  }
  free(col);
}

/* generic/SpatialFullDilatedConvolution.cu:379-453: per sample: columns = im2col(gradOutput_n);
 * gradWeight(Cin x Cout*kH*kW) += scale * input_n * columns^T ; gradBias += scale * gradOutput_n * ones */
void oracle_fullconv_accGradParameters(const float *in, const float *gradOut, float *gradWeight,
                                       float *gradBias, int N, int Cin, int Cout, int H, int W, int oH,
                                       int oW, int kW, int kH, int dW, int dH, int padW, int padH, int dilW,
                                       int dilH, float scale) {
  int Kf = Cout * kH * kW, HW = H * W;
  float *col = (float *)malloc(sizeof(float) * (size_t)Kf * HW);
  for (int n = 0; n < N; ++n) {
    const float *g = gradOut + (size_t)n * Cout * oH * oW;
    oracle_im2col(g, Cout, oH, oW, kH, kW, padH, padW, dH, dW, dilH, dilW, col);
    gemm_nt_acc(Cin, Kf, HW, scale, in + (size_t)n * Cin * HW, col, gradWeight);
    if (gradBias)
      for (int oc = 0; oc < Cout; ++oc) {
        double sum = 0.0;
        for (int l = 0; l < oH * oW; ++l) sum += (double)g[(size_t)oc * oH * oW + l];
        gradBias[oc] += scale * (float)sum;
      }
  }
  free(col);
}

/* -------------------------------------------------------- BatchNormalization --
 * input viewed as (N, C, L) (lib/THCUNN/generic/BatchNormalization.cu:8-32).
 * Sums are taken in double, as CPU-THNN does for float tensors. */

/* lib/THCUNN/BatchNormalization.cu:166-212 (training) and :140-164 (inference).
 * saveStd receives 1/sqrt(var_biased + eps) (:198); runningVar is updated with
 * the unbiased variance varN/(n-1) (:196-200); invStd = 0 when varN == 0 and
 * eps == 0 (:188-191). weight/bias may be NULL (gamma 1, beta 0). */
void oracle_bn_updateOutput(const float *in, float *out, const float *weight, const float *bias,
                            float *runningMean, float *runningVar, float *saveMean, float *saveStd,
                            int N, int C, int L, int train, double momentum, double eps) {
#pragma omp parallel for schedule(static)
  for (int c = 0; c < C; ++c) {
    double mean, invStd;
    long cnt = (long)N * L;
    if (train) {
      double sum = 0.0;
      for (int n = 0; n < N; ++n) {
        const float *p = in + ((size_t)n * C + c) * L;
        for (int l = 0; l < L; ++l) sum += p[l];
      }
      mean = sum / cnt;
      double varN = 0.0;
      for (int n = 0; n < N; ++n) {
        const float *p = in + ((size_t)n * C + c) * L;
        for (int l = 0; l < L; ++l) varN += (p[l] - mean) * (p[l] - mean);
      }
      invStd = 0.0;
      if (varN != 0.0 || eps != 0.0) invStd = 1.0 / sqrt(varN / cnt + eps);
      double unbiased = varN / (cnt - 1);
      saveMean[c] = (float)mean;
      saveStd[c] = (float)invStd;
      runningMean[c] = (float)((1 - momentum) * runningMean[c] + momentum * mean);
      runningVar[c] = (float)((1 - momentum) * runningVar[c] + momentum * unbiased);
    } else {
      mean = runningMean[c];
      invStd = 1.0 / sqrt(runningVar[c] + eps);
    }
    double gamma = weight ? weight[c] : 1.0, beta = bias ? bias[c] : 0.0;
    for (int n = 0; n < N; ++n) {
      const float *p = in + ((size_t)n * C + c) * L;
      float *o = out + ((size_t)n * C + c) * L;
      for (int l = 0; l < L; ++l) o[l] = (float)(gamma * (p[l] - mean) * invStd + beta);
    }
  }
}

/* lib/THCUNN/BatchNormalization.cu:214-283. gradIn / gradWeight / gradBias may
 * each be NULL; gradWeight and gradBias accumulate (:272-282). */
void oracle_bn_backward(const float *in, const float *gradOut, float *gradIn, float *gradWeight,
                        float *gradBias, const float *weight, const float *runningMean,
                        const float *runningVar, const float *saveMean, const float *saveStd, int N,
                        int C, int L, int train, double scale, double eps) {
#pragma omp parallel for schedule(static)
  for (int c = 0; c < C; ++c) {
    double mean, stdVal;
    long cnt = (long)N * L;
    if (train) {
      mean = saveMean[c];
      stdVal = saveStd[c];
    } else {
      mean = runningMean[c];
      stdVal = 1.0 / sqrt(runningVar[c] + eps);
    }
    double w = weight ? weight[c] : 1.0;
    double sum = 0.0, dotp = 0.0;
    for (int n = 0; n < N; ++n) {
      const float *p = in + ((size_t)n * C + c) * L;
      const float *g = gradOut + ((size_t)n * C + c) * L;
      for (int l = 0; l < L; ++l) {
        sum += g[l];
        dotp += (p[l] - mean) * g[l];
      }
    }
    double gradMean = sum / cnt;
    double projScale = dotp / cnt * stdVal * stdVal;
    double gradScale = stdVal * w;
    if (gradIn)
      for (int n = 0; n < N; ++n) {
        const float *p = in + ((size_t)n * C + c) * L;
        const float *g = gradOut + ((size_t)n * C + c) * L;
        float *gi = gradIn + ((size_t)n * C + c) * L;
        for (int l = 0; l < L; ++l)
          gi[l] = train ? (float)((g[l] - (p[l] - mean) * projScale - gradMean) * gradScale)
                        : (float)(g[l] * gradScale);
      }
    if (gradWeight) gradWeight[c] += (float)(scale * dotp * stdVal);
    if (gradBias) gradBias[c] += (float)(scale * sum);
  }
}

/* ------------------------------------------------------------------ pooling --
 * Output extent: lib/THCUNN/generic/SpatialDilatedMaxPooling.cu:47-64 and
 * generic/SpatialAveragePooling.cu:41-58: float division, floor or ceil, + 1,
 * then (only when padded) drop the last window if it starts past the input
 * plus its left padding. */
int oracle_pool_out_size(int in, int k, int d, int pad, int dil, int ceil_mode) {
  float q = (float)(in - (dil * (k - 1) + 1) + 2 * pad) / (float)d;
  long o = (long)(ceil_mode ? ceilf(q) : floorf(q)) + 1;
  return (int)o;
}
int oracle_pool_out_size_fixed(int in, int k, int d, int pad, int dil, int ceil_mode, int anyPad) {
  long o = oracle_pool_out_size(in, k, d, pad, dil, ceil_mode);
  if (anyPad && (o - 1) * d >= in + pad) --o;
  return (int)o;
}

/* lib/THCUNN/SpatialDilatedMaxPooling.cu:7-42: window clipped to the image
 * (start advanced by whole dilation steps), scan h outer / w inner, strict '>'
 * against -FLT_MAX so the first maximum in row-major order wins and NaN is never
 * picked; index = h*W + w (per plane) + TH_INDEX_BASE, -1 + base if none. */
void oracle_maxpool_updateOutput(const float *in, float *out, long *indices, int N, int C, int H,
                                 int W, int oH, int oW, int kW, int kH, int dW, int dH, int padW,
                                 int padH, int dilW, int dilH) {
#pragma omp parallel for schedule(static)
  for (long p = 0; p < (long)N * C; ++p) {
    const float *ip = in + (size_t)p * H * W;
    for (int ph = 0; ph < oH; ++ph)
      for (int pw = 0; pw < oW; ++pw) {
        int hs = ph * dH - padH, ws = pw * dW - padW;
        int he = hs + (kH - 1) * dilH + 1 < H ? hs + (kH - 1) * dilH + 1 : H;
        int we = ws + (kW - 1) * dilW + 1 < W ? ws + (kW - 1) * dilW + 1 : W;
        while (hs < 0) hs += dilH;
        while (ws < 0) ws += dilW;
        float maxval = -FLT_MAX;
        int maxidx = -1;
        for (int h = hs; h < he; h += dilH)
          for (int w = ws; w < we; w += dilW)
            if (ip[h * W + w] > maxval) {
              maxidx = h * W + w;
              maxval = ip[maxidx];
            }
        out[((size_t)p * oH + ph) * oW + pw] = maxval;
        indices[((size_t)p * oH + ph) * oW + pw] = (long)maxidx + ORACLE_INDEX_BASE;
      }
  }
}

/* lib/THCUNN/SpatialDilatedMaxPooling.cu:45-80: per input pixel, sum gradOut of
 * every window in the candidate range whose stored index names this pixel. */
void oracle_maxpool_updateGradInput(const float *gradOut, const long *indices, float *gradIn, int N,
                                    int C, int H, int W, int oH, int oW, int kW, int kH, int dW,
                                    int dH, int padW, int padH, int dilW, int dilH) {
  int extH = (kH - 1) * dilH + 1, extW = (kW - 1) * dilW + 1;
#pragma omp parallel for schedule(static)
  for (long p = 0; p < (long)N * C; ++p) {
    const float *g = gradOut + (size_t)p * oH * oW;
    const long *ix = indices + (size_t)p * oH * oW;
    for (int h = 0; h < H; ++h)
      for (int w = 0; w < W; ++w) {
        int phs = (h + padH < extH) ? 0 : (h + padH - extH) / dH + 1;
        int phe = (h + padH) / dH + 1 < oH ? (h + padH) / dH + 1 : oH;
        int pws = (w + padW < extW) ? 0 : (w + padW - extW) / dW + 1;
        int pwe = (w + padW) / dW + 1 < oW ? (w + padW) / dW + 1 : oW;
        float grad = 0.f;
        for (int ph = phs; ph < phe; ++ph)
          for (int pw = pws; pw < pwe; ++pw)
            if (ix[ph * oW + pw] - ORACLE_INDEX_BASE == h * W + w) grad += g[ph * oW + pw];
        gradIn[((size_t)p * H + h) * W + w] = grad;
      }
  }
}

/* lib/THCUNN/SpatialAveragePooling.cu:6-39: divisor is the window area after
 * clipping to H+pad but before clipping to the image (count_include_pad) or
 * the in-image count. */
void oracle_avgpool_updateOutput(const float *in, float *out, int N, int C, int H, int W, int oH,
                                 int oW, int kW, int kH, int dW, int dH, int padW, int padH,
                                 int count_include_pad) {
#pragma omp parallel for schedule(static)
  for (long p = 0; p < (long)N * C; ++p) {
    const float *ip = in + (size_t)p * H * W;
    for (int ph = 0; ph < oH; ++ph)
      for (int pw = 0; pw < oW; ++pw) {
        int hs = ph * dH - padH, ws = pw * dW - padW;
        int he = hs + kH < H + padH ? hs + kH : H + padH;
        int we = ws + kW < W + padW ? ws + kW : W + padW;
        int pool = (he - hs) * (we - ws);
        hs = hs > 0 ? hs : 0;
        ws = ws > 0 ? ws : 0;
        he = he < H ? he : H;
        we = we < W ? we : W;
        float s = 0.f;
        for (int h = hs; h < he; ++h)
          for (int w = ws; w < we; ++w) s += ip[h * W + w];
        out[((size_t)p * oH + ph) * oW + pw] =
            count_include_pad ? s / pool : s / ((he - hs) * (we - ws));
      }
  }
}

/* lib/THCUNN/SpatialAveragePooling.cu:41-82 */
void oracle_avgpool_updateGradInput(const float *gradOut, float *gradIn, int N, int C, int H, int W,
                                    int oH, int oW, int kW, int kH, int dW, int dH, int padW,
                                    int padH, int count_include_pad) {
#pragma omp parallel for schedule(static)
  for (long p = 0; p < (long)N * C; ++p) {
    const float *g = gradOut + (size_t)p * oH * oW;
    for (int y = 0; y < H; ++y)
      for (int x = 0; x < W; ++x) {
        int w = x + padW, h = y + padH;
        int phs = (h < kH) ? 0 : (h - kH) / dH + 1;
        int phe = h / dH + 1 < oH ? h / dH + 1 : oH;
        int pws = (w < kW) ? 0 : (w - kW) / dW + 1;
        int pwe = w / dW + 1 < oW ? w / dW + 1 : oW;
        float grad = 0.f;
        for (int ph = phs; ph < phe; ++ph)
          for (int pw = pws; pw < pwe; ++pw) {
            int hs = ph * dH - padH, ws = pw * dW - padW;
            int he = hs + kH < H + padH ? hs + kH : H + padH;
            int we = ws + kW < W + padW ? ws + kW : W + padW;
            int pool = (he - hs) * (we - ws);
            hs = hs > 0 ? hs : 0;
            ws = ws > 0 ? ws : 0;
            he = he < H ? he : H;
            we = we < W ? we : W;
            grad += count_include_pad ? g[ph * oW + pw] / pool
                                      : g[ph * oW + pw] / ((he - hs) * (we - ws));
          }
        gradIn[((size_t)p * H + y) * W + x] = grad;
      }
  }
}
