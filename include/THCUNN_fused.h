/*
 * THCUNN_fused.h - entry points that fuse two neighbouring modules of the path into one pass
 * (BatchNormalization + ReLU forward and backward, SpatialConvolutionMM + ReLU forward).
 *
 * Nothing here has a prototype in the reference: lib/THCUNN/generic/THCUNN.h declares one function per module and
 * the nn modules call them one after the other, so `conv -> BatchNormalization -> Threshold(0, 0)` writes the
 * normalised tensor, reads it again and writes the activation (lib/THCUNN/generic/BatchNormalization.cu:34-66, then
 * lib/THCUNN/generic/Threshold.cu:7-35). A binder that wants the fused pass binds these names explicitly; the
 * conventions (THCState first, optional tensors NULL, work enqueued on the state's stream, TH error handler) are
 * those of THCUNN.h.
 */
#ifndef THCUNN_FUSED_H
#define THCUNN_FUSED_H

#include "THCShim.h"

#ifdef __cplusplus
extern "C" {
#endif

/* output = max(BatchNormalization(input), 0) element-wise, exactly Threshold_updateOutput(threshold 0, value 0)
 * applied to what THNN_CudaBatchNormalization_updateOutput stores: v > 0 ? v : 0. Statistics (saveMean, saveStd,
 * running mean / variance) are those of the plain call. */
void THNN_CudaBatchNormalizationReLU_updateOutput(
    THCState *state, THCudaTensor *input_, THCudaTensor *output_,
    THCudaTensor *weight_,      /* [OPTIONAL] */
    THCudaTensor *bias_,        /* [OPTIONAL] */
    THCudaTensor *runningMean_, THCudaTensor *runningVar_,
    THCudaTensor *saveMean_, THCudaTensor *saveStd_,
    bool train, double momentum, double eps);

/* The backward pass of that pair: THNN_CudaBatchNormalization_backward applied to
 * Threshold_updateGradInput(output, gradOutput_) = gradOutput_ where the fused forward output was positive, 0
 * elsewhere. The output itself is not an argument: its sign is re-derived from input_ with the forward pass's own
 * arithmetic, which is why bias_ (the forward call's) is taken here. gradWeight_ / gradBias_ accumulate with
 * `scale` as in the plain call. */
void THNN_CudaBatchNormalizationReLU_backward(
    THCState *state, THCudaTensor *input_, THCudaTensor *gradOutput_,
    THCudaTensor *gradInput_,   /* [OPTIONAL] */
    THCudaTensor *gradWeight_,  /* [OPTIONAL] */
    THCudaTensor *gradBias_,    /* [OPTIONAL] */
    THCudaTensor *weight_,      /* [OPTIONAL] */
    THCudaTensor *bias_,        /* [OPTIONAL] */
    THCudaTensor *runningMean_, THCudaTensor *runningVar_,
    THCudaTensor *saveMean_, THCudaTensor *saveStd_,
    bool train, double scale, double eps);

/* output = max(SpatialConvolutionMM(input), 0): THNN_CudaSpatialConvolutionMM_updateOutput
 * (lib/THCUNN/generic/SpatialConvolutionMM.cu:58-209) followed by Threshold_updateOutput(threshold 0, value 0)
 * (lib/THCUNN/generic/Threshold.cu:7-35) - v > 0 ? v : 0 applied as the convolution stores its values, so the
 * pre-activation never reaches memory. Arguments and side effects are those of the plain call. The backward pass
 * of the pair is the plain one: Threshold_updateGradInput(output, gradOutput) - the sign of the stored output is the
 * sign of the pre-activation wherever it matters - then SpatialConvolutionMM_updateGradInput / _accGradParameters. */
void THNN_CudaSpatialConvolutionMMReLU_updateOutput(
    THCState *state, THCudaTensor *input, THCudaTensor *output, THCudaTensor *weight,
    THCudaTensor *bias,         /* [OPTIONAL] */
    THCudaTensor *columns, THCudaTensor *ones,
    int kW, int kH, int dW, int dH, int padW, int padH);

#ifdef __cplusplus
}
#endif
#endif /* THCUNN_FUSED_H */
