/*
 * THCShim.h - the minimal slice of cutorch's THC object model that the
 * THNN_Cuda* spatial entry points dereference, re-stated for HIP.
 *
 * The reference wrappers read tensor metadata straight out of the structs
 * (`weight->size[0]`, `weight->nDimension`, `weight->storage`,
 * `weight->storageOffset`: lib/THCUNN/generic/SpatialDepthWiseConvolution.cu:14,36-39,76-77,100;
 * lib/THCUNN/generic/SpatialConvolutionMM.cu:80-86), so the field order below is
 * part of the binary contract with the LuaJIT-FFI caller (THCUNN.lua:71-78).
 * cutorch's own headers are not part of the reference tree (`#include <THC/THC.h>`,
 * lib/THCUNN/THCUNN.h:1); the order used here is cutorch 1.0's
 * (THCStorage: data,size,refcount,flag,allocator,allocatorContext,view,device;
 *  THCTensor: size,stride,nDimension,storage,storageOffset,refcount,flag).
 *
 * Everything is plain C: pointers, sizes, no C++ or torch types.
 */
#ifndef THC_SHIM_H
#define THC_SHIM_H

#include <stddef.h>
#include <stdbool.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TH_INDEX_BASE 1 /* Lua-torch builds index from 1 (used at lib/THCUNN/SpatialDilatedMaxPooling.cu:40,73) */

#define TH_STORAGE_REFCOUNTED 1
#define TH_STORAGE_RESIZABLE 2
#define TH_STORAGE_FREEMEM 4
#define TH_TENSOR_REFCOUNTED 1

typedef struct THCState THCState; /* opaque: device, current stream, error hooks */

typedef struct THCudaStorage {
  float *data; /* device pointer */
  ptrdiff_t size; /* elements */
  int refcount;
  char flag;
  void *allocator;
  void *allocatorContext;
  struct THCudaStorage *view;
  int device;
} THCudaStorage;

typedef struct THCudaTensor {
  long *size;
  long *stride;
  int nDimension;
  THCudaStorage *storage;
  ptrdiff_t storageOffset;
  int refcount;
  char flag;
} THCudaTensor;

typedef struct THCudaLongStorage {
  long *data; /* device pointer, 64-bit elements */
  ptrdiff_t size;
  int refcount;
  char flag;
  void *allocator;
  void *allocatorContext;
  struct THCudaLongStorage *view;
  int device;
} THCudaLongStorage;

typedef struct THCudaLongTensor {
  long *size;
  long *stride;
  int nDimension;
  THCudaLongStorage *storage;
  ptrdiff_t storageOffset;
  int refcount;
  char flag;
} THCudaLongTensor;

/* ---- state ------------------------------------------------------------- */
/* Replaces cutorch.getState() (THCUNN.lua:14-16). One state per host thread
 * that drives a GPU; all work of an entry point is enqueued on the state's
 * current stream (the reference does the same through
 * THCState_getCurrentStream, e.g. lib/THCUNN/generic/BatchNormalization.cu:50). */
THCState *THCState_alloc(void);
void THCState_free(THCState *state);
void THCState_setCurrentStream(THCState *state, void *hipStream);
void *THCState_getCurrentStream(THCState *state);
void THCState_synchronize(THCState *state); /* cutorch.synchronize() */

/* ---- error hooks ------------------------------------------------------- */
/* TH reports shape/argument errors through a process-wide handler
 * (THError / THArgCheck, lib/THCUNN/common.h:28-83). The default handler
 * prints the message and aborts, as TH's does; a binder installs its own
 * (Lua raises a Lua error). The entry point returns right after the handler
 * does, having launched nothing. */
typedef void (*THErrorHandlerFunction)(const char *msg, void *data);
typedef void (*THArgErrorHandlerFunction)(int argNumber, const char *msg, void *data);
void THSetErrorHandler(THErrorHandlerFunction handler, void *data);
void THSetArgErrorHandler(THArgErrorHandlerFunction handler, void *data);

/* ---- tensors (float) ---------------------------------------------------- */
THCudaTensor *THCudaTensor_new(THCState *state);
THCudaTensor *THCudaTensor_newWithSize(THCState *state, int nDimension, const long *size);
/* non-owning view of device memory the caller allocated (e.g. a torch tensor):
 * storage flag has neither RESIZABLE nor FREEMEM; `capacity` is in elements,
 * `stride` may be NULL for contiguous. */
THCudaTensor *THCudaTensor_newWithData(THCState *state, float *devPtr, ptrdiff_t capacity,
                                       ptrdiff_t storageOffset, int nDimension,
                                       const long *size, const long *stride);
/* strided view sharing `src`'s storage (narrow/transpose/select made by the caller) */
THCudaTensor *THCudaTensor_newView(THCState *state, THCudaTensor *src, ptrdiff_t storageOffset,
                                   int nDimension, const long *size, const long *stride);
void THCudaTensor_retain(THCState *state, THCudaTensor *self);
void THCudaTensor_free(THCState *state, THCudaTensor *self);
void THCudaTensor_resizeNd(THCState *state, THCudaTensor *self, int nDimension, const long *size);
float *THCudaTensor_data(THCState *state, const THCudaTensor *self);
int THCudaTensor_nDimension(THCState *state, const THCudaTensor *self);
long THCudaTensor_size(THCState *state, const THCudaTensor *self, int dim);
long THCudaTensor_stride(THCState *state, const THCudaTensor *self, int dim);
ptrdiff_t THCudaTensor_nElement(THCState *state, const THCudaTensor *self);
int THCudaTensor_isContiguous(THCState *state, const THCudaTensor *self);
void THCudaTensor_fill(THCState *state, THCudaTensor *self, float value);
void THCudaTensor_copy(THCState *state, THCudaTensor *self, THCudaTensor *src); /* device to device, same nElement */
/* host <-> device copies of the logical (size-ordered) contents; synchronous */
void THCudaTensor_copyFromHost(THCState *state, THCudaTensor *self, const float *src);
void THCudaTensor_copyToHost(THCState *state, THCudaTensor *self, float *dst);

/* ---- tensors (int64 indices) ------------------------------------------- */
THCudaLongTensor *THCudaLongTensor_new(THCState *state);
THCudaLongTensor *THCudaLongTensor_newWithSize(THCState *state, int nDimension, const long *size);
THCudaLongTensor *THCudaLongTensor_newWithData(THCState *state, long *devPtr, ptrdiff_t capacity,
                                               ptrdiff_t storageOffset, int nDimension,
                                               const long *size, const long *stride);
void THCudaLongTensor_free(THCState *state, THCudaLongTensor *self);
void THCudaLongTensor_resizeNd(THCState *state, THCudaLongTensor *self, int nDimension, const long *size);
long *THCudaLongTensor_data(THCState *state, const THCudaLongTensor *self);
int THCudaLongTensor_nDimension(THCState *state, const THCudaLongTensor *self);
long THCudaLongTensor_size(THCState *state, const THCudaLongTensor *self, int dim);
ptrdiff_t THCudaLongTensor_nElement(THCState *state, const THCudaLongTensor *self);
void THCudaLongTensor_copyFromHost(THCState *state, THCudaLongTensor *self, const long *src);
void THCudaLongTensor_copyToHost(THCState *state, THCudaLongTensor *self, long *dst);

/* ---- hooks for parity tests (no counterpart in the reference's C ABI) ---------- */
/* The column kernels of lib/THCUNN/im2col.h:9-61 and :63-121 (C++ templates inside the reference library),
 * on raw device pointers: `im` is nImages x channels x height x width, `col` is
 * nImages x (channels*kH*kW) x (oH*oW); col2im overwrites `im` with the gathered sums. */
void THNN_Cuda_im2col(THCState *state, const float *im, int nImages, int channels, int height, int width,
                      int kH, int kW, int padH, int padW, int dH, int dW, int dilH, int dilW, float *col);
void THNN_Cuda_col2im(THCState *state, const float *col, int nImages, int channels, int height, int width,
                      int kH, int kW, int padH, int padW, int dH, int dW, int dilH, int dilW, float *im);
/* Several kernel families compute the same results; this forces one. `name` is one of THCUNN_DW_FORCE_DIRECT,
 * THCUNN_DW_SMALL, THCUNN_POOL_FORCE_DIRECT, THCUNN_POOL_RUNS, THCUNN_BN_FORCE_CHUNKED, THCUNN_CONV_FORCE_GENERIC,
 * THCUNN_CONV_GRADINPUT, THCUNN_CONV_POINTWISE; `value` is what the environment variable of that name would hold (read once, when the
 * library is loaded), NULL restores the choice by shape. Returns 0 for an unknown name. Not thread-safe
 * against concurrent calls of the entry points. */
int THCUNN_setSwitch(const char *name, const char *value);

#ifdef __cplusplus
}
#endif
#endif /* THC_SHIM_H */
