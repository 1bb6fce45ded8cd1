/*
 * THCUNN.h - C ABI of the gfx950 spatial-convolution hot path.
 *
 * These are the fp32 ("Cuda") instantiations of the prototypes that
 * lib/THCUNN/generic/THCUNN.h declares through THNN_(NAME) =
 * THNN_ ## Cuda ## NAME (lib/THCUNN/THCUNN.h:7) and that THCUNN.lua:22-78 turns
 * into ffi.cdef text (THCTensor -> THCudaTensor, THCIndexTensor ->
 * THCudaLongTensor, accreal -> float: THCUNN.lua:42-48). Argument order and
 * meaning are the reference's; integer geometry arguments come W before H.
 * `[OPTIONAL]` tensors may be NULL. Every entry point enqueues its work on
 * THCState_getCurrentStream(state) and returns without synchronising.
 */
#ifndef THCUNN_H
#define THCUNN_H

#include "THCShim.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- BatchNormalization (SpatialBatchNormalization shares it: the input is
 * viewed as N x C x (H*W)) ------------------------------------------------ */

/* replaces lib/THCUNN/generic/THCUNN.h:30-42, lib/THCUNN/generic/BatchNormalization.cu:34-66 */
void THNN_CudaBatchNormalization_updateOutput(
    THCState *state, THCudaTensor *input_, THCudaTensor *output_,
    THCudaTensor *weight_,      /* [OPTIONAL] */
    THCudaTensor *bias_,        /* [OPTIONAL] */
    THCudaTensor *runningMean_, THCudaTensor *runningVar_,
    THCudaTensor *saveMean_, THCudaTensor *saveStd_,
    bool train, double momentum, double eps);

/* replaces lib/THCUNN/generic/THCUNN.h:44-58, lib/THCUNN/generic/BatchNormalization.cu:68-94 */
void THNN_CudaBatchNormalization_backward(
    THCState *state, THCudaTensor *input_, THCudaTensor *gradOutput_,
    THCudaTensor *gradInput_,   /* [OPTIONAL] */
    THCudaTensor *gradWeight_,  /* [OPTIONAL] */
    THCudaTensor *gradBias_,    /* [OPTIONAL] */
    THCudaTensor *weight_,      /* [OPTIONAL] */
    THCudaTensor *runningMean_, THCudaTensor *runningVar_,
    THCudaTensor *saveMean_, THCudaTensor *saveStd_,
    bool train, double scale, double eps);

/* ---- SpatialAveragePooling ---------------------------------------------- */

/* replaces lib/THCUNN/generic/THCUNN.h:548-556, lib/THCUNN/generic/SpatialAveragePooling.cu:72-150 */
void THNN_CudaSpatialAveragePooling_updateOutput(
    THCState *state, THCudaTensor *input, THCudaTensor *output,
    int kW, int kH, int dW, int dH, int padW, int padH,
    bool ceil_mode, bool count_include_pad);

/* replaces lib/THCUNN/generic/THCUNN.h:558-567, lib/THCUNN/generic/SpatialAveragePooling.cu:152-235 */
void THNN_CudaSpatialAveragePooling_updateGradInput(
    THCState *state, THCudaTensor *input, THCudaTensor *gradOutput, THCudaTensor *gradInput,
    int kW, int kH, int dW, int dH, int padW, int padH,
    bool ceil_mode, bool count_include_pad);

/* ---- SpatialConvolutionMM ------------------------------------------------ */

/* replaces lib/THCUNN/generic/THCUNN.h:630-640, lib/THCUNN/generic/SpatialConvolutionMM.cu:58-209 */
void THNN_CudaSpatialConvolutionMM_updateOutput(
    THCState *state, THCudaTensor *input, THCudaTensor *output, THCudaTensor *weight,
    THCudaTensor *bias,         /* [OPTIONAL] */
    THCudaTensor *columns, THCudaTensor *ones,
    int kW, int kH, int dW, int dH, int padW, int padH);

/* replaces lib/THCUNN/generic/THCUNN.h:642-652, lib/THCUNN/generic/SpatialConvolutionMM.cu:211-325 */
void THNN_CudaSpatialConvolutionMM_updateGradInput(
    THCState *state, THCudaTensor *input, THCudaTensor *gradOutput, THCudaTensor *gradInput,
    THCudaTensor *weight, THCudaTensor *gradColumns, THCudaTensor *ones,
    int kW, int kH, int dW, int dH, int padW, int padH);

/* replaces lib/THCUNN/generic/THCUNN.h:654-665, lib/THCUNN/generic/SpatialConvolutionMM.cu:327-486 */
void THNN_CudaSpatialConvolutionMM_accGradParameters(
    THCState *state, THCudaTensor *input, THCudaTensor *gradOutput, THCudaTensor *gradWeight,
    THCudaTensor *gradBias,     /* [OPTIONAL] */
    THCudaTensor *columns, THCudaTensor *ones,
    int kW, int kH, int dW, int dH, int padW, int padH, float scale);

/* ---- SpatialDepthWiseConvolution ----------------------------------------- */

/* replaces lib/THCUNN/generic/THCUNN.h:667-677, lib/THCUNN/generic/SpatialDepthWiseConvolution.cu:58-261 */
void THNN_CudaSpatialDepthWiseConvolution_updateOutput(
    THCState *state, THCudaTensor *input, THCudaTensor *output, THCudaTensor *weight,
    THCudaTensor *bias,         /* [OPTIONAL] */
    THCudaTensor *columns, THCudaTensor *ones,
    int kW, int kH, int dW, int dH, int padW, int padH);

/* replaces lib/THCUNN/generic/THCUNN.h:679-689, lib/THCUNN/generic/SpatialDepthWiseConvolution.cu:263-416 */
void THNN_CudaSpatialDepthWiseConvolution_updateGradInput(
    THCState *state, THCudaTensor *input, THCudaTensor *gradOutput, THCudaTensor *gradInput,
    THCudaTensor *weight, THCudaTensor *gradColumns, THCudaTensor *ones,
    int kW, int kH, int dW, int dH, int padW, int padH);

/* replaces lib/THCUNN/generic/THCUNN.h:691-702, lib/THCUNN/generic/SpatialDepthWiseConvolution.cu:418-650 */
void THNN_CudaSpatialDepthWiseConvolution_accGradParameters(
    THCState *state, THCudaTensor *input, THCudaTensor *gradOutput, THCudaTensor *gradWeight,
    THCudaTensor *gradBias,     /* [OPTIONAL] */
    THCudaTensor *columns, THCudaTensor *ones,
    int kW, int kH, int dW, int dH, int padW, int padH, float scale);

/* No counterpart in the reference. SpatialDepthWiseConvolution_accGradParameters for callers that cannot
 * allocate device memory (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc): same kernels and results, but the per-workgroup partial sums go to a fixed 4 MiB device array
 * that the library holds on each GPU it runs on, and nothing is allocated, freed or resized. It therefore
 * takes no `columns` / `ones`, and refuses (TH error, nothing launched) what the regular entry point would
 * allocate for: non-contiguous input / gradOutput, a 2-D gradWeight, and shapes whose partial sums exceed
 * 2^20 floats (C * M * P * N * bands-per-plane, P = kH*kW + 1 rounded up to 16). The state must have been made on the current
 * device. All calls on one GPU share the array: calls that overlap in time on one GPU (two streams, two
 * threads) race. */
void THNN_CudaSpatialDepthWiseConvolution_accGradParameters_noAlloc(
    THCState *state, THCudaTensor *input, THCudaTensor *gradOutput, THCudaTensor *gradWeight,
    THCudaTensor *gradBias,     /* [OPTIONAL] */
    int kW, int kH, int dW, int dH, int padW, int padH, float scale);

/* ---- SpatialDilatedMaxPooling / SpatialMaxPooling ------------------------ */

/* replaces lib/THCUNN/generic/THCUNN.h:808-817, lib/THCUNN/generic/SpatialDilatedMaxPooling.cu:84-158 */
void THNN_CudaSpatialDilatedMaxPooling_updateOutput(
    THCState *state, THCudaTensor *input, THCudaTensor *output, THCudaLongTensor *indices,
    int kW, int kH, int dW, int dH, int padW, int padH,
    int dilationW, int dilationH, bool ceil_mode);

/* replaces lib/THCUNN/generic/THCUNN.h:819-829, lib/THCUNN/generic/SpatialDilatedMaxPooling.cu:160-235 */
void THNN_CudaSpatialDilatedMaxPooling_updateGradInput(
    THCState *state, THCudaTensor *input, THCudaTensor *gradOutput, THCudaTensor *gradInput,
    THCudaLongTensor *indices,
    int kW, int kH, int dW, int dH, int padW, int padH,
    int dilationW, int dilationH, bool ceil_mode);

/* replaces lib/THCUNN/generic/THCUNN.h:888-896, lib/THCUNN/generic/SpatialMaxPooling.cu:7-21 */
void THNN_CudaSpatialMaxPooling_updateOutput(
    THCState *state, THCudaTensor *input, THCudaTensor *output, THCudaLongTensor *indices,
    int kW, int kH, int dW, int dH, int padW, int padH, bool ceil_mode);

/* replaces lib/THCUNN/generic/THCUNN.h:898-907, lib/THCUNN/generic/SpatialMaxPooling.cu:23-38 */
void THNN_CudaSpatialMaxPooling_updateGradInput(
    THCState *state, THCudaTensor *input, THCudaTensor *gradOutput, THCudaTensor *gradInput,
    THCudaLongTensor *indices,
    int kW, int kH, int dW, int dH, int padW, int padH, bool ceil_mode);

/* ---- next after the hot path: dilated and transposed convolution -------------
 * Same im2col/col2im + fp32 MFMA GEMM passes as SpatialConvolutionMM. */

/* replaces lib/THCUNN/generic/THCUNN.h:727-738, lib/THCUNN/generic/SpatialDilatedConvolution.cu:69-190 */
void THNN_CudaSpatialDilatedConvolution_updateOutput(
    THCState *state, THCudaTensor *input, THCudaTensor *output, THCudaTensor *weight,
    THCudaTensor *bias,         /* [OPTIONAL] */
    THCudaTensor *columns, THCudaTensor *ones,
    int kW, int kH, int dW, int dH, int padW, int padH, int dilationW, int dilationH);

/* replaces lib/THCUNN/generic/THCUNN.h:740-750, lib/THCUNN/generic/SpatialDilatedConvolution.cu:192-293 */
void THNN_CudaSpatialDilatedConvolution_updateGradInput(
    THCState *state, THCudaTensor *input, THCudaTensor *gradOutput, THCudaTensor *gradInput,
    THCudaTensor *weight, THCudaTensor *gradColumns,
    int kW, int kH, int dW, int dH, int padW, int padH, int dilationW, int dilationH);

/* replaces lib/THCUNN/generic/THCUNN.h:752-764, lib/THCUNN/generic/SpatialDilatedConvolution.cu:295-432 */
void THNN_CudaSpatialDilatedConvolution_accGradParameters(
    THCState *state, THCudaTensor *input, THCudaTensor *gradOutput, THCudaTensor *gradWeight,
    THCudaTensor *gradBias,     /* [OPTIONAL] */
    THCudaTensor *columns, THCudaTensor *ones,
    int kW, int kH, int dW, int dH, int padW, int padH, int dilationW, int dilationH, float scale);

/* replaces lib/THCUNN/generic/THCUNN.h:766-778, lib/THCUNN/generic/SpatialFullDilatedConvolution.cu:68-204 */
void THNN_CudaSpatialFullDilatedConvolution_updateOutput(
    THCState *state, THCudaTensor *input, THCudaTensor *output, THCudaTensor *weight,
    THCudaTensor *bias,         /* [OPTIONAL] */
    THCudaTensor *columns, THCudaTensor *ones,
    int kW, int kH, int dW, int dH, int padW, int padH, int dilationW, int dilationH, int adjW, int adjH);

/* replaces lib/THCUNN/generic/THCUNN.h:780-791, lib/THCUNN/generic/SpatialFullDilatedConvolution.cu:206-312 */
void THNN_CudaSpatialFullDilatedConvolution_updateGradInput(
    THCState *state, THCudaTensor *input, THCudaTensor *gradOutput, THCudaTensor *gradInput,
    THCudaTensor *weight, THCudaTensor *gradColumns,
    int kW, int kH, int dW, int dH, int padW, int padH, int dilationW, int dilationH, int adjW, int adjH);

/* replaces lib/THCUNN/generic/THCUNN.h:793-806, lib/THCUNN/generic/SpatialFullDilatedConvolution.cu:314-465 */
void THNN_CudaSpatialFullDilatedConvolution_accGradParameters(
    THCState *state, THCudaTensor *input, THCudaTensor *gradOutput, THCudaTensor *gradWeight,
    THCudaTensor *gradBias,     /* [OPTIONAL] */
    THCudaTensor *columns, THCudaTensor *ones,
    int kW, int kH, int dW, int dH, int padW, int padH, int dilationW, int dilationH, int adjW, int adjH,
    float scale);

/* replaces lib/THCUNN/generic/THCUNN.h:849-860, lib/THCUNN/generic/SpatialFullConvolution.cu:5-22 */
void THNN_CudaSpatialFullConvolution_updateOutput(
    THCState *state, THCudaTensor *input, THCudaTensor *output, THCudaTensor *weight,
    THCudaTensor *bias,         /* [OPTIONAL] */
    THCudaTensor *columns, THCudaTensor *ones,
    int kW, int kH, int dW, int dH, int padW, int padH, int adjW, int adjH);

/* replaces lib/THCUNN/generic/THCUNN.h:862-872, lib/THCUNN/generic/SpatialFullConvolution.cu:24-39 */
void THNN_CudaSpatialFullConvolution_updateGradInput(
    THCState *state, THCudaTensor *input, THCudaTensor *gradOutput, THCudaTensor *gradInput,
    THCudaTensor *weight, THCudaTensor *gradColumns,
    int kW, int kH, int dW, int dH, int padW, int padH, int adjW, int adjH);

/* replaces lib/THCUNN/generic/THCUNN.h:874-886, lib/THCUNN/generic/SpatialFullConvolution.cu:41-59 */
void THNN_CudaSpatialFullConvolution_accGradParameters(
    THCState *state, THCudaTensor *input, THCudaTensor *gradOutput, THCudaTensor *gradWeight,
    THCudaTensor *gradBias,     /* [OPTIONAL] */
    THCudaTensor *columns, THCudaTensor *ones,
    int kW, int kH, int dW, int dH, int padW, int padH, int adjW, int adjH, float scale);

/* ---- Threshold (ReLU): the element-wise step next to the convolution path --- */

/* replaces lib/THCUNN/generic/THCUNN.h:1220-1226, lib/THCUNN/generic/Threshold.cu:7-35 */
void THNN_CudaThreshold_updateOutput(
    THCState *state, THCudaTensor *input, THCudaTensor *output,
    float threshold, float val, bool inplace);

/* replaces lib/THCUNN/generic/THCUNN.h:1228-1235, lib/THCUNN/generic/Threshold.cu:37-67 */
void THNN_CudaThreshold_updateGradInput(
    THCState *state, THCudaTensor *input, THCudaTensor *gradOutput, THCudaTensor *gradInput,
    float threshold, float val, bool inplace);

#ifdef __cplusplus
}
#endif
#endif /* THCUNN_H */
