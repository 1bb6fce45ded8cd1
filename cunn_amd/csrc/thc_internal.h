// Internal C++ side of the THC shim: error plumbing, tensor metadata helpers
// and stream-ordered temporaries used by the THNN_Cuda* wrappers.
#pragma once

#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <exception>
#include <string>
#include <vector>

#include "../../include/THCUNN.h"

// Per stream: a block of device memory that entry points without a buffer argument use for their partial results
// (cutorch keeps such a scratch space per device and stream as well). It grows on demand and lives as long as the state.
struct StreamScratch {
  hipStream_t stream;
  void *ptr;
  size_t bytes;
};

struct THCState {
  int device = 0;
  hipStream_t stream = nullptr;
  std::vector<StreamScratch> scratch;
};

namespace thc {

// ---- errors ---------------------------------------------------------------
// THError / THArgCheck unwind to the extern "C" boundary as a C++ exception;
// the boundary hands the text to the installed TH handler and returns.
struct Error {
  std::string msg;
  int arg;  // 0: THError, >0: THArgCheck argument number
};

[[noreturn]] void error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
[[noreturn]] void argError(int arg, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
void dispatchError(const Error &e);  // calls the installed handler

#define THC_ARG_CHECK(cond, arg, ...) \
  do {                                \
    if (!(cond)) ::thc::argError(arg, __VA_ARGS__); \
  } while (0)

#define THC_HIP_CHECK(expr)                                                         \
  do {                                                                              \
    hipError_t err__ = (expr);                                                      \
    if (err__ != hipSuccess)                                                        \
      ::thc::error("HIP runtime error: %s (%s) at %s:%d", hipGetErrorString(err__), \
                   #expr, __FILE__, __LINE__);                                      \
  } while (0)

// Wraps the body of every extern "C" entry point: nothing may unwind into the C caller (ctypes, LuaJIT), so
// whatever the standard library throws (bad_alloc of a host container ...) goes to the TH handler as well.
#define THNN_ENTER try {
#define THNN_LEAVE                                                             \
  }                                                                            \
  catch (const ::thc::Error &e__) {                                            \
    ::thc::Error copy__ = e__;                                                 \
    ::thc::dispatchError(copy__);                                              \
  }                                                                            \
  catch (const std::exception &e__) {                                          \
    ::thc::dispatchError(::thc::Error{std::string("C++ exception: ") + e__.what(), 0}); \
  }                                                                            \
  catch (...) {                                                                \
    ::thc::dispatchError(::thc::Error{"unknown C++ exception", 0});           \
  }

// ---- type-erased tensor view of THCudaTensor / THCudaLongTensor ------------
struct Storage {
  void *data;
  ptrdiff_t size;
  int refcount;
  char flag;
  void *allocator;
  void *allocatorContext;
  Storage *view;
  int device;
};
struct Tensor {
  long *size;
  long *stride;
  int nDimension;
  Storage *storage;
  ptrdiff_t storageOffset;
  int refcount;
  char flag;
};
static_assert(sizeof(Tensor) == sizeof(THCudaTensor), "layout");
static_assert(sizeof(Storage) == sizeof(THCudaStorage), "layout");

inline Tensor *erase(THCudaTensor *t) { return reinterpret_cast<Tensor *>(t); }
inline const Tensor *erase(const THCudaTensor *t) { return reinterpret_cast<const Tensor *>(t); }
inline Tensor *erase(THCudaLongTensor *t) { return reinterpret_cast<Tensor *>(t); }
inline const Tensor *erase(const THCudaLongTensor *t) { return reinterpret_cast<const Tensor *>(t); }

Tensor *tensorNew();
void tensorFree(Tensor *t);
void tensorRetain(Tensor *t);
// TH resizeNd semantics: a tensor that already has these sizes is left alone
// (strides included); otherwise sizes are set, strides made contiguous and the
// storage grown (never shrunk) to hold storageOffset + numel elements.
void tensorResize(THCState *state, Tensor *t, int nd, const long *size, size_t elemSize);
void tensorSetView(Tensor *t, Storage *s, ptrdiff_t offset, int nd, const long *size, const long *stride);
ptrdiff_t numel(const Tensor *t);
bool isContiguous(const Tensor *t);
bool sameSize(const Tensor *a, const Tensor *b);
std::string sizeDesc(const Tensor *t);  // "[64 x 128 x 56 x 56]" as THCTensor_(sizeDesc)

inline void resize(THCState *s, THCudaTensor *t, std::initializer_list<long> dims) {
  std::vector<long> v(dims);
  tensorResize(s, erase(t), (int)v.size(), v.data(), sizeof(float));
}
inline void resize(THCState *s, THCudaLongTensor *t, std::initializer_list<long> dims) {
  std::vector<long> v(dims);
  tensorResize(s, erase(t), (int)v.size(), v.data(), sizeof(long));
}
inline float *data(const THCudaTensor *t) {
  return t->storage ? t->storage->data + t->storageOffset : nullptr;
}
inline long *data(const THCudaLongTensor *t) {
  return t->storage ? t->storage->data + t->storageOffset : nullptr;
}

// strided gather src(size,stride) -> dst contiguous (or the reverse scatter)
void stridedCopy(hipStream_t stream, const Tensor *t, void *contig, size_t elemSize, bool toContig);

// At least `bytes` of device memory that belongs to (state, current stream) and is reused by every call on that
// stream: work that uses it is ordered by the stream. Allocates only when a call needs more than any earlier call
// on the stream did (then the stream is drained before the smaller block is freed).
void *streamScratch(THCState *state, size_t bytes);

// Stream-ordered temporary: memory is returned to the pool after the work
// queued so far on `stream` has drained, with no host synchronisation.
class Temp {
 public:
  Temp() = default;
  Temp(hipStream_t stream, size_t bytes);
  Temp(Temp &&o) noexcept : p_(o.p_), stream_(o.stream_) { o.p_ = nullptr; }
  Temp &operator=(Temp &&o) noexcept;
  Temp(const Temp &) = delete;
  Temp &operator=(const Temp &) = delete;
  ~Temp();
  void *get() const { return p_; }

 private:
  void *p_ = nullptr;
  hipStream_t stream_ = nullptr;
};

// THCTensor_(newContiguous): the tensor's own data when it is contiguous,
// otherwise a packed stream-ordered copy that lives as long as this object.
class Contiguous {
 public:
  Contiguous(THCState *state, const THCudaTensor *t);
  const float *ptr() const { return ptr_; }

 private:
  const float *ptr_;
  Temp tmp_;
};

// ---- kernel-family switches ---------------------------------------------------
// Several kernel families compute the same results; the parity tests force each of them. The switches take
// their initial values from the environment once, when the library is loaded (THCUNN_DW_FORCE_DIRECT,
// THCUNN_DW_SMALL, THCUNN_POOL_FORCE_DIRECT, THCUNN_POOL_RUNS, THCUNN_BN_FORCE_CHUNKED,
// THCUNN_CONV_FORCE_GENERIC, THCUNN_CONV_GRADINPUT, THCUNN_CONV_POINTWISE), and change afterwards only through THCUNN_setSwitch:
// an entry point reads a plain int, never the environment.
struct Switches {
  int dwForce = 0;        // 1: shape-agnostic direct kernels, 2: generic LDS-tiled kernels
  int dwSmall = -1;       // 0: never the run-of-memory kernels, 1: also where the strip kernels would be chosen
  int poolForce = 0;      // as dwForce
  int poolRuns = -1;      // as dwSmall
  int bnChunked = 0;      // 1: the chunked two-pass kernels also where a channel fits one workgroup
  int convGeneric = 0;    // 1: first-generation convolution kernels
  int convGradInput = 0;  // 1: phase route, 2: gradient-column route, 3: few-plane kernel with run-time tap loops, 0: by shape
  int convPointwise = 1;  // 0: never the weight-stationary 1x1 kernel; n > 1: at most n workgroups per row block
};
extern Switches g_switches;

// Looks up, for the current device `device`, the address of the fixed scratch array behind
// THNN_CudaSpatialDepthWiseConvolution_accGradParameters_noAlloc (dwconv.hip). Called when a state is
// made, so that the entry point itself finds the address in a table.
void dwNoAllocInit(int device);
// x[i] = x[i] > 0 ? x[i] : 0 over n contiguous floats (threshold.hip)
void reluInPlace(hipStream_t stream, float *x, long n);

// THCUNN_check_dim_size (lib/THCUNN/common.h:69-75)
void checkDimSize(const Tensor *t, const char *name, int dim, int dimSize, long size);

}  // namespace thc
