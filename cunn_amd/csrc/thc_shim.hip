// THC shim: state, storages/tensors on hipMalloc, error hooks, strided copies.
// This is the part of cutorch the THNN_Cuda* wrappers lean on
// (THCTensor_(resizeNd/newContiguous/free/data/fill), THCState_getCurrentStream,
// THError/THArgCheck); cutorch itself is not part of the reference tree.
#include "thc_internal.h"

#include <cstdlib>
#include <cstring>
#include <mutex>

namespace thc {

// ---------------------------------------------------------------- errors ----
static void defaultErrorHandler(const char *msg, void *) {
  fprintf(stderr, "$ Error: %s\n", msg);
  abort();
}
static void defaultArgErrorHandler(int arg, const char *msg, void *) {
  fprintf(stderr, "$ Invalid argument %d: %s\n", arg, msg ? msg : "");
  abort();
}
static THErrorHandlerFunction g_errHandler = defaultErrorHandler;
static void *g_errData = nullptr;
static THArgErrorHandlerFunction g_argHandler = defaultArgErrorHandler;
static void *g_argData = nullptr;

static std::string vformat(const char *fmt, va_list ap) {
  char buf[2048];
  vsnprintf(buf, sizeof(buf), fmt, ap);
  return std::string(buf);
}

void error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  Error e{vformat(fmt, ap), 0};
  va_end(ap);
  throw e;
}
void argError(int arg, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  Error e{vformat(fmt, ap), arg};
  va_end(ap);
  throw e;
}
void dispatchError(const Error &e) {
  if (e.arg > 0)
    g_argHandler(e.arg, e.msg.c_str(), g_argData);
  else
    g_errHandler(e.msg.c_str(), g_errData);
}

// -------------------------------------------------------------- switches ----
static int switchValue(const char *name, const char *v, bool *known) {
  *known = true;
  if (!strcmp(name, "THCUNN_CONV_GRADINPUT")) return !v ? 0 : !strcmp(v, "phases") ? 1 : !strcmp(v, "columns") ? 2 : !strcmp(v, "planes") ? 3 : 0;
  if (!strcmp(name, "THCUNN_DW_SMALL") || !strcmp(name, "THCUNN_POOL_RUNS")) return v ? atoi(v) : -1;
  if (!strcmp(name, "THCUNN_CONV_POINTWISE")) return v ? atoi(v) : 1;
  if (!strcmp(name, "THCUNN_DW_FORCE_DIRECT") || !strcmp(name, "THCUNN_POOL_FORCE_DIRECT") ||
      !strcmp(name, "THCUNN_BN_FORCE_CHUNKED") || !strcmp(name, "THCUNN_CONV_FORCE_GENERIC"))
    return v ? atoi(v) : 0;
  *known = false;
  return 0;
}
static int *switchSlot(Switches &s, const char *name) {
  if (!strcmp(name, "THCUNN_DW_FORCE_DIRECT")) return &s.dwForce;
  if (!strcmp(name, "THCUNN_DW_SMALL")) return &s.dwSmall;
  if (!strcmp(name, "THCUNN_POOL_FORCE_DIRECT")) return &s.poolForce;
  if (!strcmp(name, "THCUNN_POOL_RUNS")) return &s.poolRuns;
  if (!strcmp(name, "THCUNN_BN_FORCE_CHUNKED")) return &s.bnChunked;
  if (!strcmp(name, "THCUNN_CONV_FORCE_GENERIC")) return &s.convGeneric;
  if (!strcmp(name, "THCUNN_CONV_GRADINPUT")) return &s.convGradInput;
  if (!strcmp(name, "THCUNN_CONV_POINTWISE")) return &s.convPointwise;
  return nullptr;
}
static Switches switchesFromEnvironment() {
  Switches s;
  for (const char *name : {"THCUNN_DW_FORCE_DIRECT", "THCUNN_DW_SMALL", "THCUNN_POOL_FORCE_DIRECT", "THCUNN_POOL_RUNS",
                           "THCUNN_BN_FORCE_CHUNKED", "THCUNN_CONV_FORCE_GENERIC", "THCUNN_CONV_GRADINPUT",
                           "THCUNN_CONV_POINTWISE"}) {
    bool known;
    *switchSlot(s, name) = switchValue(name, getenv(name), &known);
  }
  return s;
}
Switches g_switches = switchesFromEnvironment();  // read once, when the library is loaded

// ------------------------------------------------------- per-stream scratch ----
void *streamScratch(THCState *state, size_t bytes) {
  StreamScratch *slot = nullptr;
  for (StreamScratch &sc : state->scratch)
    if (sc.stream == state->stream) slot = &sc;
  if (!slot) {
    state->scratch.push_back(StreamScratch{state->stream, nullptr, 0});
    slot = &state->scratch.back();
  }
  if (slot->bytes < bytes) {
    if (slot->ptr) {
      THC_HIP_CHECK(hipStreamSynchronize(state->stream));
      THC_HIP_CHECK(hipFree(slot->ptr));
      slot->ptr = nullptr, slot->bytes = 0;
    }
    const size_t want = (bytes + 65535) / 65536 * 65536;
    THC_HIP_CHECK(hipMalloc(&slot->ptr, want));
    slot->bytes = want;
  }
  return slot->ptr;
}

// --------------------------------------------------------------- storage ----
static Storage *storageNew(int device) {
  Storage *s = (Storage *)calloc(1, sizeof(Storage));
  s->refcount = 1;
  s->flag = TH_STORAGE_REFCOUNTED | TH_STORAGE_RESIZABLE | TH_STORAGE_FREEMEM;
  s->device = device;
  return s;
}
static void storageFree(Storage *s) {
  if (!s) return;
  if (--s->refcount > 0) return;
  if ((s->flag & TH_STORAGE_FREEMEM) && s->data) (void)hipFree(s->data);
  free(s);
}
// Growth allocates with hipMalloc (which may wait for the device) and, when the storage already holds
// data, copies it over and waits for the stream before the old block is freed: a first call at a new size
// is not asynchronous. Steady-state calls (sizes unchanged) never get here.
static void storageGrow(THCState *state, Storage *s, ptrdiff_t elems, size_t elemSize) {
  if (elems <= s->size) return;
  if (!(s->flag & TH_STORAGE_RESIZABLE)) error("Trying to resize storage that is not resizable");
  // a storage that names an allocator of its own was not made by this library: its memory is that
  // allocator's to move, so the caller has to size the tensor before the call
  if (s->allocator)
    error("Trying to resize a storage that carries its own allocator: give the tensor its final size before the call");
  void *p = nullptr;
  THC_HIP_CHECK(hipMalloc(&p, (size_t)elems * elemSize));
  if (s->data && s->size > 0) {
    // THCStorage_resize keeps the old contents
    THC_HIP_CHECK(hipMemcpyAsync(p, s->data, (size_t)s->size * elemSize, hipMemcpyDeviceToDevice,
                                 state->stream));
    THC_HIP_CHECK(hipStreamSynchronize(state->stream));
    if (s->flag & TH_STORAGE_FREEMEM) THC_HIP_CHECK(hipFree(s->data));
  }
  s->data = p;
  s->size = elems;
  s->flag |= TH_STORAGE_FREEMEM;
}

// ---------------------------------------------------------------- tensor ----
Tensor *tensorNew() {
  Tensor *t = (Tensor *)calloc(1, sizeof(Tensor));
  t->refcount = 1;
  t->flag = TH_TENSOR_REFCOUNTED;
  return t;
}
void tensorRetain(Tensor *t) {
  if (t) ++t->refcount;
}
void tensorFree(Tensor *t) {
  if (!t) return;
  if (--t->refcount > 0) return;
  free(t->size);
  free(t->stride);
  storageFree(t->storage);
  free(t);
}
ptrdiff_t numel(const Tensor *t) {
  if (!t || t->nDimension == 0) return 0;
  ptrdiff_t n = 1;
  for (int i = 0; i < t->nDimension; ++i) n *= t->size[i];
  return n;
}
bool isContiguous(const Tensor *t) {
  long z = 1;
  for (int d = t->nDimension - 1; d >= 0; --d) {
    if (t->size[d] != 1) {
      if (t->stride[d] != z) return false;
      z *= t->size[d];
    }
  }
  return true;
}
bool sameSize(const Tensor *a, const Tensor *b) {
  if (a->nDimension != b->nDimension) return false;
  for (int i = 0; i < a->nDimension; ++i)
    if (a->size[i] != b->size[i]) return false;
  return true;
}
std::string sizeDesc(const Tensor *t) {
  std::string s = "[";
  for (int i = 0; i < t->nDimension; ++i) {
    s += std::to_string(t->size[i]);
    if (i + 1 < t->nDimension) s += " x ";
  }
  return s + "]";
}
static void setDims(Tensor *t, int nd, const long *size, const long *stride) {
  if (nd != t->nDimension) {
    t->size = (long *)realloc(t->size, sizeof(long) * (nd > 0 ? nd : 1));
    t->stride = (long *)realloc(t->stride, sizeof(long) * (nd > 0 ? nd : 1));
    t->nDimension = nd;
  }
  long z = 1;
  for (int d = nd - 1; d >= 0; --d) {
    t->size[d] = size[d];
    if (stride && stride[d] >= 0) {
      t->stride[d] = stride[d];
    } else {
      t->stride[d] = z;
    }
    z *= size[d];
  }
}
void tensorResize(THCState *state, Tensor *t, int nd, const long *size, size_t elemSize) {
  bool same = (nd == t->nDimension);
  for (int d = 0; same && d < nd; ++d) same = (size[d] == t->size[d]);
  if (same) return;
  setDims(t, nd, size, nullptr);
  ptrdiff_t n = numel(t);
  if (n > 0) {
    if (!t->storage) t->storage = storageNew(state->device);
    storageGrow(state, t->storage, n + t->storageOffset, elemSize);
  }
}
void tensorSetView(Tensor *t, Storage *s, ptrdiff_t offset, int nd, const long *size, const long *stride) {
  if (t->storage != s) {
    storageFree(t->storage);
    t->storage = s;
    if (s) ++s->refcount;
  }
  t->storageOffset = offset;
  setDims(t, nd, size, stride);
}
void checkDimSize(const Tensor *t, const char *name, int dim, int dimSize, long size) {
  if (t->nDimension != dim || t->size[dimSize] != size) {
    error("Need %s of dimension %d and %s.size[%d] == %ld but got %s to be of shape: %s", name, dim,
          name, dimSize, size, name, sizeDesc(t).c_str());
  }
}

// ----------------------------------------------------------- strided copy ----
constexpr int kMaxDims = 8;
struct StridedDesc {
  long size[kMaxDims];
  long stride[kMaxDims];
  int nd;
  long total;
};

template <typename T, bool TO_CONTIG>
__global__ void __launch_bounds__(256) stridedCopyKernel(T *strided, T *contig, StridedDesc d) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < d.total;
       i += (long)gridDim.x * blockDim.x) {
    long rem = i, off = 0;
    for (int k = d.nd - 1; k >= 0; --k) {
      long q = rem / d.size[k];
      off += (rem - q * d.size[k]) * d.stride[k];
      rem = q;
    }
    if (TO_CONTIG)
      contig[i] = strided[off];
    else
      strided[off] = contig[i];
  }
}

void stridedCopy(hipStream_t stream, const Tensor *t, void *contig, size_t elemSize, bool toContig) {
  if (t->nDimension > kMaxDims) error("tensors of more than %d dimensions are not supported", kMaxDims);
  StridedDesc d;
  d.nd = t->nDimension;
  d.total = numel(t);
  for (int i = 0; i < d.nd; ++i) {
    d.size[i] = t->size[i];
    d.stride[i] = t->stride[i];
  }
  if (d.total == 0) return;
  long blocks = (d.total + 255) / 256;
  if (blocks > 65535 * 16) blocks = 65535 * 16;
  void *base = (char *)t->storage->data + (size_t)t->storageOffset * elemSize;
  if (elemSize == 4) {
    if (toContig)
      stridedCopyKernel<uint32_t, true><<<(unsigned)blocks, 256, 0, stream>>>((uint32_t *)base, (uint32_t *)contig, d);
    else
      stridedCopyKernel<uint32_t, false><<<(unsigned)blocks, 256, 0, stream>>>((uint32_t *)base, (uint32_t *)contig, d);
  } else {
    if (toContig)
      stridedCopyKernel<uint64_t, true><<<(unsigned)blocks, 256, 0, stream>>>((uint64_t *)base, (uint64_t *)contig, d);
    else
      stridedCopyKernel<uint64_t, false><<<(unsigned)blocks, 256, 0, stream>>>((uint64_t *)base, (uint64_t *)contig, d);
  }
  THC_HIP_CHECK(hipGetLastError());
}

// ------------------------------------------------------------ temporaries ----
Temp::Temp(hipStream_t stream, size_t bytes) : stream_(stream) {
  if (bytes == 0) return;
  THC_HIP_CHECK(hipMallocAsync(&p_, bytes, stream));
}
Temp &Temp::operator=(Temp &&o) noexcept {
  if (this != &o) {
    if (p_) (void)hipFreeAsync(p_, stream_);
    p_ = o.p_;
    stream_ = o.stream_;
    o.p_ = nullptr;
  }
  return *this;
}
Temp::~Temp() {
  if (p_) (void)hipFreeAsync(p_, stream_);
}

Contiguous::Contiguous(THCState *state, const THCudaTensor *t) {
  const Tensor *e = erase(t);
  if (isContiguous(e)) {
    ptr_ = data(t);
    return;
  }
  tmp_ = Temp(state->stream, (size_t)numel(e) * sizeof(float));
  stridedCopy(state->stream, e, tmp_.get(), sizeof(float), true);
  ptr_ = (const float *)tmp_.get();
}

// dst[i] = src[i] over n4 float4s (+ tail): the plain streaming copy that bandwidth
// figures of the other kernels are calibrated against
__global__ void __launch_bounds__(256) copyKernel(const float *__restrict__ src, float *__restrict__ dst, long n) {
  const long n4 = n >> 2;
  const long stride = (long)gridDim.x * blockDim.x;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride)
    reinterpret_cast<float4 *>(dst)[i] = reinterpret_cast<const float4 *>(src)[i];
  for (long i = (n4 << 2) + (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = src[i];
}

template <typename T>
__global__ void __launch_bounds__(256) fillKernel(T *p, long n, T v) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
    p[i] = v;
}

// ------------------------------------------------------ generic C helpers ----
static Tensor *newWithSize(THCState *state, int nd, const long *size, size_t elemSize) {
  Tensor *t = tensorNew();
  if (nd > 0) tensorResize(state, t, nd, size, elemSize);
  return t;
}
static Tensor *newWithData(THCState *state, void *devPtr, ptrdiff_t capacity, ptrdiff_t offset, int nd,
                           const long *size, const long *stride) {
  Storage *s = (Storage *)calloc(1, sizeof(Storage));
  s->refcount = 1;
  s->flag = TH_STORAGE_REFCOUNTED;  // neither resizable nor owned
  s->data = devPtr;
  s->size = capacity;
  s->device = state->device;
  Tensor *t = tensorNew();
  tensorSetView(t, s, offset, nd, size, stride);
  storageFree(s);  // the tensor holds the only reference now
  return t;
}
static void copyHost(THCState *state, Tensor *t, void *host, size_t elemSize, bool toHost) {
  ptrdiff_t n = numel(t);
  if (n == 0) return;
  size_t bytes = (size_t)n * elemSize;
  void *base = (char *)t->storage->data + (size_t)t->storageOffset * elemSize;
  if (isContiguous(t)) {
    if (toHost) {
      THC_HIP_CHECK(hipStreamSynchronize(state->stream));
      THC_HIP_CHECK(hipMemcpy(host, base, bytes, hipMemcpyDeviceToHost));
    } else {
      THC_HIP_CHECK(hipMemcpy(base, host, bytes, hipMemcpyHostToDevice));
    }
    return;
  }
  void *tmp = nullptr;
  THC_HIP_CHECK(hipMalloc(&tmp, bytes));
  if (toHost) {
    stridedCopy(state->stream, t, tmp, elemSize, true);
    THC_HIP_CHECK(hipStreamSynchronize(state->stream));
    THC_HIP_CHECK(hipMemcpy(host, tmp, bytes, hipMemcpyDeviceToHost));
  } else {
    THC_HIP_CHECK(hipMemcpy(tmp, host, bytes, hipMemcpyHostToDevice));
    stridedCopy(state->stream, t, tmp, elemSize, false);
    THC_HIP_CHECK(hipStreamSynchronize(state->stream));
  }
  THC_HIP_CHECK(hipFree(tmp));
}

}  // namespace thc

using namespace thc;

// =============================================================== C API =======
extern "C" {

THCState *THCState_alloc(void) {
  THCState *s = nullptr;
  THNN_ENTER
  s = new THCState();
  THC_HIP_CHECK(hipGetDevice(&s->device));
  s->stream = nullptr;  // the device's default stream
  dwNoAllocInit(s->device);
  THNN_LEAVE
  return s;
}
void THCState_free(THCState *state) {
  if (!state) return;
  for (StreamScratch &sc : state->scratch)
    if (sc.ptr) (void)hipFree(sc.ptr);  // waits for the device: nothing still reads the block
  delete state;
}
void THCState_setCurrentStream(THCState *state, void *hipStream) { state->stream = (hipStream_t)hipStream; }
void *THCState_getCurrentStream(THCState *state) { return (void *)state->stream; }
void THCState_synchronize(THCState *state) {
  THNN_ENTER
  THC_HIP_CHECK(hipStreamSynchronize(state->stream));
  THNN_LEAVE
}

int THCUNN_setSwitch(const char *name, const char *value) {
  bool known = false;
  if (!name) return 0;
  const int v = switchValue(name, value, &known);
  if (!known) return 0;
  *switchSlot(g_switches, name) = v;
  return 1;
}

void THSetErrorHandler(THErrorHandlerFunction handler, void *data) {
  g_errHandler = handler ? handler : defaultErrorHandler;
  g_errData = data;
}
void THSetArgErrorHandler(THArgErrorHandlerFunction handler, void *data) {
  g_argHandler = handler ? handler : defaultArgErrorHandler;
  g_argData = data;
}

// ---- float tensors
THCudaTensor *THCudaTensor_new(THCState *) { return (THCudaTensor *)tensorNew(); }
THCudaTensor *THCudaTensor_newWithSize(THCState *state, int nd, const long *size) {
  Tensor *t = nullptr;
  THNN_ENTER
  t = newWithSize(state, nd, size, sizeof(float));
  THNN_LEAVE
  return (THCudaTensor *)t;
}
THCudaTensor *THCudaTensor_newWithData(THCState *state, float *devPtr, ptrdiff_t capacity, ptrdiff_t offset,
                                       int nd, const long *size, const long *stride) {
  return (THCudaTensor *)newWithData(state, devPtr, capacity, offset, nd, size, stride);
}
THCudaTensor *THCudaTensor_newView(THCState *, THCudaTensor *src, ptrdiff_t offset, int nd, const long *size,
                                   const long *stride) {
  Tensor *t = tensorNew();
  tensorSetView(t, erase(src)->storage, offset, nd, size, stride);
  return (THCudaTensor *)t;
}
void THCudaTensor_retain(THCState *, THCudaTensor *self) { tensorRetain(erase(self)); }
void THCudaTensor_free(THCState *, THCudaTensor *self) { tensorFree(erase(self)); }
void THCudaTensor_resizeNd(THCState *state, THCudaTensor *self, int nd, const long *size) {
  THNN_ENTER
  tensorResize(state, erase(self), nd, size, sizeof(float));
  THNN_LEAVE
}
float *THCudaTensor_data(THCState *, const THCudaTensor *self) { return data(self); }
int THCudaTensor_nDimension(THCState *, const THCudaTensor *self) { return self->nDimension; }
long THCudaTensor_size(THCState *, const THCudaTensor *self, int dim) { return self->size[dim]; }
long THCudaTensor_stride(THCState *, const THCudaTensor *self, int dim) { return self->stride[dim]; }
ptrdiff_t THCudaTensor_nElement(THCState *, const THCudaTensor *self) { return numel(erase(self)); }
int THCudaTensor_isContiguous(THCState *, const THCudaTensor *self) { return isContiguous(erase(self)); }
void THCudaTensor_fill(THCState *state, THCudaTensor *self, float value) {
  THNN_ENTER
  Tensor *t = erase(self);
  ptrdiff_t n = numel(t);
  if (n == 0) return;
  if (!isContiguous(t)) error("fill: contiguous tensor expected");
  long blocks = (n + 255) / 256;
  if (blocks > 16384) blocks = 16384;
  fillKernel<float><<<(unsigned)blocks, 256, 0, state->stream>>>(data(self), n, value);
  THC_HIP_CHECK(hipGetLastError());
  THNN_LEAVE
}
void THCudaTensor_copy(THCState *state, THCudaTensor *self, THCudaTensor *src) {
  THNN_ENTER
  Tensor *d = erase(self), *f = erase(src);
  ptrdiff_t n = numel(d);
  if (n != numel(f)) error("copy: sizes do not match: %s vs %s", sizeDesc(d).c_str(), sizeDesc(f).c_str());
  if (n == 0) return;
  if (isContiguous(d) && isContiguous(f) && ((reinterpret_cast<uintptr_t>(data(self)) | reinterpret_cast<uintptr_t>(data(src))) & 15) == 0) {
    long blocks = ((n >> 2) + 255) / 256;
    blocks = blocks < 1 ? 1 : (blocks > 16384 ? 16384 : blocks);
    copyKernel<<<(unsigned)blocks, 256, 0, state->stream>>>(data(src), data(self), n);
    THC_HIP_CHECK(hipGetLastError());
  } else {
    // through a packed temporary: gather src, scatter into self
    Temp tmp(state->stream, (size_t)n * sizeof(float));
    stridedCopy(state->stream, f, tmp.get(), sizeof(float), true);
    stridedCopy(state->stream, d, tmp.get(), sizeof(float), false);
  }
  THNN_LEAVE
}
void THCudaTensor_copyFromHost(THCState *state, THCudaTensor *self, const float *src) {
  THNN_ENTER
  copyHost(state, erase(self), (void *)src, sizeof(float), false);
  THNN_LEAVE
}
void THCudaTensor_copyToHost(THCState *state, THCudaTensor *self, float *dst) {
  THNN_ENTER
  copyHost(state, erase(self), dst, sizeof(float), true);
  THNN_LEAVE
}

// ---- int64 tensors
THCudaLongTensor *THCudaLongTensor_new(THCState *) { return (THCudaLongTensor *)tensorNew(); }
THCudaLongTensor *THCudaLongTensor_newWithSize(THCState *state, int nd, const long *size) {
  Tensor *t = nullptr;
  THNN_ENTER
  t = newWithSize(state, nd, size, sizeof(long));
  THNN_LEAVE
  return (THCudaLongTensor *)t;
}
THCudaLongTensor *THCudaLongTensor_newWithData(THCState *state, long *devPtr, ptrdiff_t capacity,
                                               ptrdiff_t offset, int nd, const long *size,
                                               const long *stride) {
  return (THCudaLongTensor *)newWithData(state, devPtr, capacity, offset, nd, size, stride);
}
void THCudaLongTensor_free(THCState *, THCudaLongTensor *self) { tensorFree(erase(self)); }
void THCudaLongTensor_resizeNd(THCState *state, THCudaLongTensor *self, int nd, const long *size) {
  THNN_ENTER
  tensorResize(state, erase(self), nd, size, sizeof(long));
  THNN_LEAVE
}
long *THCudaLongTensor_data(THCState *, const THCudaLongTensor *self) { return data(self); }
int THCudaLongTensor_nDimension(THCState *, const THCudaLongTensor *self) { return self->nDimension; }
long THCudaLongTensor_size(THCState *, const THCudaLongTensor *self, int dim) { return self->size[dim]; }
ptrdiff_t THCudaLongTensor_nElement(THCState *, const THCudaLongTensor *self) { return numel(erase(self)); }
void THCudaLongTensor_copyFromHost(THCState *state, THCudaLongTensor *self, const long *src) {
  THNN_ENTER
  copyHost(state, erase(self), (void *)src, sizeof(long), false);
  THNN_LEAVE
}
void THCudaLongTensor_copyToHost(THCState *state, THCudaLongTensor *self, long *dst) {
  THNN_ENTER
  copyHost(state, erase(self), dst, sizeof(long), true);
  THNN_LEAVE
}

}  // extern "C"
