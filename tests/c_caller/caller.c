/*
 * A caller of libTHCUNN.so that is not the library's own harness: plain C, playing what LuaJIT + cutorch do
 * under THCUNN.lua:129-133. include/THCUNN.h and include/THCUNN_fused.h are included for the prototypes only:
 * the tensor and storage structs this program fills in are declared HERE, field by field as cutorch 1.0 lays
 * them out (the layout the reference wrappers dereference: lib/THCUNN/generic/SpatialDepthWiseConvolution.cu:14,
 * 36-39, 76-77, 100), and handed to the entry points through pointer casts. If the library's own declaration of
 * those structs drifts from this one, the compile-time checks below stop the build, and without them the library
 * would read this program's tensors wrongly and the comparisons with the golden vectors would fail.
 *
 * It builds every tensor / storage itself (own malloc'ed size / stride arrays, storage
 * flags as cutorch sets them for an owned storage, device memory from hipMalloc), hands the entry
 * points EMPTY result tensors that the library has to resize (lib/THCUNN/generic/SpatialDepthWiseConvolution.cu:121,
 * generic/SpatialDilatedMaxPooling.cu:141 ...), a 2-D depthwise weight that the library reshapes in place
 * (generic/SpatialDepthWiseConvolution.cu:76-80), a strided input, and compares what comes back with
 * vectors read from files (the committed golden vectors, dumped by the test that runs this program).
 *
 *   caller <dir>      <dir>/manifest.txt: one line per array "<name> <f|l> <ndim> <dims...>", data in <dir>/<name>.bin
 *
 * Exit status 0 when every check holds; each check prints one line.
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <stddef.h>

#include "THCUNN.h"
#include "THCUNN_fused.h"

/* ---- cutorch 1.0's object layout, written out by this caller (not taken from the library's header) ---- */
typedef struct CallerStorage {
  float *data;           /* device pointer */
  ptrdiff_t size;        /* elements */
  int refcount;
  char flag;
  void *allocator;
  void *allocatorContext;
  struct CallerStorage *view;
  int device;
} CallerStorage;

typedef struct CallerTensor {
  long *size;
  long *stride;
  int nDimension;
  CallerStorage *storage;
  ptrdiff_t storageOffset;
  int refcount;
  char flag;
} CallerTensor;

typedef struct CallerLongStorage {
  long *data;            /* device pointer, 64-bit elements */
  ptrdiff_t size;
  int refcount;
  char flag;
  void *allocator;
  void *allocatorContext;
  struct CallerLongStorage *view;
  int device;
} CallerLongStorage;

typedef struct CallerLongTensor {
  long *size;
  long *stride;
  int nDimension;
  CallerLongStorage *storage;
  ptrdiff_t storageOffset;
  int refcount;
  char flag;
} CallerLongTensor;

enum { CALLER_STORAGE_REFCOUNTED = 1, CALLER_STORAGE_RESIZABLE = 2, CALLER_STORAGE_FREEMEM = 4, CALLER_TENSOR_REFCOUNTED = 1 };

#define SAME_FIELD(mine, theirs, f) \
  _Static_assert(offsetof(mine, f) == offsetof(theirs, f) && sizeof(((mine *)0)->f) == sizeof(((theirs *)0)->f), \
                 "field " #f " of " #theirs " moved")
_Static_assert(sizeof(CallerTensor) == sizeof(THCudaTensor) && sizeof(CallerStorage) == sizeof(THCudaStorage), "struct size");
_Static_assert(sizeof(CallerLongTensor) == sizeof(THCudaLongTensor) && sizeof(CallerLongStorage) == sizeof(THCudaLongStorage), "struct size");
SAME_FIELD(CallerTensor, THCudaTensor, size);
SAME_FIELD(CallerTensor, THCudaTensor, stride);
SAME_FIELD(CallerTensor, THCudaTensor, nDimension);
SAME_FIELD(CallerTensor, THCudaTensor, storage);
SAME_FIELD(CallerTensor, THCudaTensor, storageOffset);
SAME_FIELD(CallerTensor, THCudaTensor, refcount);
SAME_FIELD(CallerTensor, THCudaTensor, flag);
SAME_FIELD(CallerStorage, THCudaStorage, data);
SAME_FIELD(CallerStorage, THCudaStorage, size);
SAME_FIELD(CallerStorage, THCudaStorage, refcount);
SAME_FIELD(CallerStorage, THCudaStorage, flag);
SAME_FIELD(CallerStorage, THCudaStorage, allocator);
SAME_FIELD(CallerStorage, THCudaStorage, allocatorContext);
SAME_FIELD(CallerStorage, THCudaStorage, view);
SAME_FIELD(CallerStorage, THCudaStorage, device);
SAME_FIELD(CallerLongTensor, THCudaLongTensor, storage);
SAME_FIELD(CallerLongTensor, THCudaLongTensor, storageOffset);
SAME_FIELD(CallerLongStorage, THCudaLongStorage, data);
SAME_FIELD(CallerLongStorage, THCudaLongStorage, device);
_Static_assert(CALLER_STORAGE_REFCOUNTED == TH_STORAGE_REFCOUNTED && CALLER_STORAGE_RESIZABLE == TH_STORAGE_RESIZABLE &&
               CALLER_STORAGE_FREEMEM == TH_STORAGE_FREEMEM && CALLER_TENSOR_REFCOUNTED == TH_TENSOR_REFCOUNTED, "flag values");

/* how a tensor of this program is handed to an entry point */
#define T(t) ((THCudaTensor *)(t))
#define LT(t) ((THCudaLongTensor *)(t))

/* the HIP runtime calls this caller needs, declared by hand: no HIP header is included */
extern int hipMalloc(void **ptr, size_t size);
extern int hipFree(void *ptr);
extern int hipMemcpy(void *dst, const void *src, size_t bytes, int kind); /* 1: host to device, 2: device to host */
extern int hipMemset(void *dst, int value, size_t bytes);
extern int hipDeviceSynchronize(void);

static int failures = 0;
static int errors_seen = 0;
static char last_error[1024];

#define HIP_OK(call)                                              \
  do {                                                            \
    int rc__ = (call);                                            \
    if (rc__ != 0) {                                              \
      fprintf(stderr, "%s failed with hipError %d\n", #call, rc__); \
      exit(3);                                                    \
    }                                                             \
  } while (0)

static void on_error(const char *msg, void *data) {
  (void)data;
  ++errors_seen;
  snprintf(last_error, sizeof(last_error), "%s", msg);
}
static void on_arg_error(int arg, const char *msg, void *data) {
  (void)data;
  ++errors_seen;
  snprintf(last_error, sizeof(last_error), "argument %d: %s", arg, msg ? msg : "");
}

/* ------------------------------------------------------------------ vectors from files ---- */
typedef struct {
  char name[64];
  char type; /* 'f' float32, 'l' int64 */
  int nd;
  long dims[8];
  long n;
  void *data;
} Arr;

static Arr arrs[256];
static int narrs = 0;

static void load_all(const char *dir) {
  char path[4096];
  snprintf(path, sizeof(path), "%s/manifest.txt", dir);
  FILE *m = fopen(path, "r");
  if (!m) {
    perror(path);
    exit(2);
  }
  while (narrs < 256) {
    Arr *a = &arrs[narrs];
    if (fscanf(m, "%63s %c %d", a->name, &a->type, &a->nd) != 3) break;
    a->n = 1;
    for (int i = 0; i < a->nd; ++i) {
      if (fscanf(m, "%ld", &a->dims[i]) != 1) exit(2);
      a->n *= a->dims[i];
    }
    size_t es = a->type == 'f' ? sizeof(float) : sizeof(long);
    a->data = malloc(a->n * es + 1);
    snprintf(path, sizeof(path), "%s/%s.bin", dir, a->name);
    FILE *f = fopen(path, "rb");
    if (!f || fread(a->data, es, a->n, f) != (size_t)a->n) {
      fprintf(stderr, "cannot read %s\n", path);
      exit(2);
    }
    fclose(f);
    ++narrs;
  }
  fclose(m);
}

static const Arr *arr(const char *name) {
  for (int i = 0; i < narrs; ++i)
    if (!strcmp(arrs[i].name, name)) return &arrs[i];
  fprintf(stderr, "no array %s in the manifest\n", name);
  exit(2);
}

/* ------------------------------------------------- tensors built by the caller itself ---- */
static CallerStorage *storage_new(long elems) {
  CallerStorage *s = (CallerStorage *)calloc(1, sizeof(CallerStorage));
  s->size = elems;
  s->refcount = 1;
  s->flag = CALLER_STORAGE_REFCOUNTED | CALLER_STORAGE_RESIZABLE | CALLER_STORAGE_FREEMEM; /* an owned cutorch storage */
  s->allocator = NULL;
  s->allocatorContext = NULL;
  s->view = NULL;
  s->device = 0;
  if (elems > 0) HIP_OK(hipMalloc((void **)&s->data, elems * sizeof(float)));
  return s;
}

/* CallerTensor_new(): no dimensions, no storage */
static CallerTensor *tensor_empty(void) {
  CallerTensor *t = (CallerTensor *)calloc(1, sizeof(CallerTensor));
  t->refcount = 1;
  t->flag = CALLER_TENSOR_REFCOUNTED;
  return t;
}

/* A tensor of the given sizes over its own storage; rows (the last dimension) lie `pitch` floats apart
 * (pitch == last size: contiguous) and the tensor starts `offset` floats into the storage. */
static CallerTensor *tensor_sized(int nd, const long *dims, long pitch, long offset) {
  CallerTensor *t = tensor_empty();
  t->nDimension = nd;
  t->size = (long *)malloc(sizeof(long) * nd);
  t->stride = (long *)malloc(sizeof(long) * nd);
  long z = 1;
  for (int d = nd - 1; d >= 0; --d) {
    t->size[d] = dims[d];
    t->stride[d] = z;
    z *= (d == nd - 1) ? pitch : dims[d];
  }
  t->storageOffset = offset;
  t->storage = storage_new(z + offset);
  return t;
}

static CallerTensor *tensor_from(const Arr *a, long extraPitch, long offset) {
  const long W = a->dims[a->nd - 1], pitch = W + extraPitch, rows = a->n / W;
  CallerTensor *t = tensor_sized(a->nd, a->dims, pitch, offset);
  float *host = (float *)malloc(sizeof(float) * (rows * pitch + offset));
  for (long i = 0; i < rows * pitch + offset; ++i) host[i] = NAN; /* whatever is read outside the view poisons the result */
  for (long r = 0; r < rows; ++r) memcpy(host + offset + r * pitch, (const float *)a->data + r * W, sizeof(float) * W);
  HIP_OK(hipMemcpy(t->storage->data, host, sizeof(float) * (rows * pitch + offset), 1));
  free(host);
  return t;
}

static CallerTensor *tensor_zeros(int nd, const long *dims) {
  CallerTensor *t = tensor_sized(nd, dims, dims[nd - 1], 0);
  HIP_OK(hipMemset(t->storage->data, 0, sizeof(float) * t->storage->size));
  return t;
}

static CallerLongTensor *long_tensor_empty(void) {
  CallerLongTensor *t = (CallerLongTensor *)calloc(1, sizeof(CallerLongTensor));
  t->refcount = 1;
  t->flag = CALLER_TENSOR_REFCOUNTED;
  return t;
}

static void tensor_free(CallerTensor *t) {
  if (!t) return;
  if (t->storage) {
    if (t->storage->data) HIP_OK(hipFree(t->storage->data));
    free(t->storage);
  }
  free(t->size);
  free(t->stride);
  free(t);
}

/* ---------------------------------------------------------------------------- checks ---- */
static void report(const char *what, int ok, const char *detail) {
  printf("%-70s %s %s\n", what, ok ? "ok" : "FAILED", detail ? detail : "");
  fflush(stdout);
  if (!ok) ++failures;
}

static int has_shape(int nd, const long *size, const long *stride, const Arr *want) {
  if (nd != want->nd) return 0;
  long z = 1;
  for (int d = nd - 1; d >= 0; --d) {
    if (size[d] != want->dims[d] || stride[d] != z) return 0;
    z *= size[d];
  }
  return 1;
}

/* the library sized `t` like `want` (contiguous), gave it a storage, and the values agree */
static void check_tensor(const char *what, const CallerTensor *t, const Arr *want, double rtol, double atol) {
  char detail[256] = "";
  int ok = t->storage && t->storage->data && has_shape(t->nDimension, t->size, t->stride, want) &&
           t->storage->size >= t->storageOffset + want->n;
  if (!ok) {
    snprintf(detail, sizeof(detail), "(shape / storage: nDimension %d)", t->nDimension);
    report(what, 0, detail);
    return;
  }
  float *got = (float *)malloc(sizeof(float) * want->n);
  HIP_OK(hipMemcpy(got, t->storage->data + t->storageOffset, sizeof(float) * want->n, 2));
  const float *ref = (const float *)want->data;
  double worst = 0;
  for (long i = 0; i < want->n; ++i) {
    double err = fabs((double)got[i] - ref[i]) - rtol * fabs((double)ref[i]);
    if (!(err <= atol)) ok = 0; /* also catches NaN */
    if (err > worst) worst = err;
  }
  snprintf(detail, sizeof(detail), "(%ld values, worst |a-b| - rtol|b| = %.2e, atol %.0e)", want->n, worst, atol);
  report(what, ok, detail);
  free(got);
}

static void check_longs(const char *what, const CallerLongTensor *t, const Arr *want) {
  int ok = t->storage && t->storage->data && has_shape(t->nDimension, t->size, t->stride, want);
  if (ok) {
    long *got = (long *)malloc(sizeof(long) * want->n);
    HIP_OK(hipMemcpy(got, t->storage->data + t->storageOffset, sizeof(long) * want->n, 2));
    ok = memcmp(got, want->data, sizeof(long) * want->n) == 0;
    free(got);
  }
  report(what, ok, "(bit-exact)");
}

static int geom(const char *name, int i) { return (int)((const long *)arr(name)->data)[i]; }


static void long_tensor_free(CallerLongTensor *t) {
  if (!t) return;
  if (t->storage) {
    if (t->storage->data) HIP_OK(hipFree(t->storage->data));
    free(t->storage);
  }
  free(t->size);
  free(t->stride);
  free(t);
}

/* a vector of n floats, every element `v` */
static CallerTensor *tensor_const(long n, float v) {
  const long dims[1] = {n};
  CallerTensor *t = tensor_sized(1, dims, n, 0);
  float *h = (float *)malloc(sizeof(float) * n);
  for (long i = 0; i < n; ++i) h[i] = v;
  HIP_OK(hipMemcpy(t->storage->data, h, sizeof(float) * n, 1));
  free(h);
  return t;
}

/* an array derived from a golden one inside this program (same shape, new values) */
static Arr derived(const Arr *like) {
  Arr a = *like;
  a.data = malloc(sizeof(float) * a.n);
  return a;
}

int main(int argc, char **argv) {
  if (argc != 2) {
    fprintf(stderr, "usage: %s <vector directory>\n", argv[0]);
    return 2;
  }
  load_all(argv[1]);
  THSetErrorHandler(on_error, NULL);
  THSetArgErrorHandler(on_arg_error, NULL);
  THCState *state = THCState_alloc();
  if (!state || errors_seen) {
    fprintf(stderr, "THCState_alloc failed: %s\n", last_error);
    return 3;
  }
  char nm[96];
  const char *c;
#define NM(suffix) (snprintf(nm, sizeof(nm), "%s.%s", c, suffix), nm)

  /* ---- SpatialDepthWiseConvolution: forward, gradInput, accGradParameters (golden case dw_s2) ---- */
  {
    const int kW = geom("dw_s2.geom", 0), kH = geom("dw_s2.geom", 1), dW = geom("dw_s2.geom", 2), dH = geom("dw_s2.geom", 3),
              pW = geom("dw_s2.geom", 4), pH = geom("dw_s2.geom", 5);
    const Arr *w4 = arr("dw_s2.w");
    const long M = w4->dims[0], C = w4->dims[1];
    CallerTensor *x = tensor_from(arr("dw_s2.x"), 0, 0), *gy = tensor_from(arr("dw_s2.gy"), 0, 0), *b = tensor_from(arr("dw_s2.b"), 0, 0);
    /* the nn module holds the weight 2-D, (nOutputPlane, nInputPlane*kH*kW): the library reshapes it in place */
    const long w2dims[2] = {M, C * kH * kW};
    Arr w2 = *w4;
    w2.nd = 2, w2.dims[0] = w2dims[0], w2.dims[1] = w2dims[1];
    CallerTensor *w = tensor_from(&w2, 0, 0);
    CallerTensor *y = tensor_empty(), *gx = tensor_empty(), *columns = tensor_empty(), *ones = tensor_empty();
    THNN_CudaSpatialDepthWiseConvolution_updateOutput(state, T(x), T(y), T(w), T(b), T(columns), T(ones), kW, kH, dW, dH, pW, pH);
    check_tensor("depthwise updateOutput into an empty output (resized by the callee)", y, arr("dw_s2.y"), 1e-5, 1e-4);
    report("depthwise 2-D weight reshaped to 4-D in place", w->nDimension == 4 && w->size[0] == M && w->size[1] == C &&
           w->size[2] == kH && w->size[3] == kW && w->stride[3] == 1, NULL);
    THNN_CudaSpatialDepthWiseConvolution_updateGradInput(state, T(x), T(gy), T(gx), T(w), T(columns), T(ones), kW, kH, dW, dH, pW, pH);
    check_tensor("depthwise updateGradInput into an empty gradInput", gx, arr("dw_s2.gx"), 1e-5, 1e-4);
    CallerTensor *gw = tensor_zeros(2, w2dims), *gb = tensor_zeros(2, arr("dw_s2.b")->dims);
    THNN_CudaSpatialDepthWiseConvolution_accGradParameters(state, T(x), T(gy), T(gw), T(gb), T(columns), T(ones), kW, kH, dW, dH, pW, pH, 1.0f);
    check_tensor("depthwise accGradParameters: gradWeight (2-D, reshaped in place)", gw, arr("dw_s2.gw"), 1e-3, 1e-3);
    check_tensor("depthwise accGradParameters: gradBias", gb, arr("dw_s2.gb"), 1e-3, 1e-3);
    /* the variant that allocates nothing: a 4-D gradWeight of the caller, no buffer tensors */
    CallerTensor *gw4 = tensor_zeros(4, w4->dims), *gb4 = tensor_zeros(2, arr("dw_s2.b")->dims);
    THNN_CudaSpatialDepthWiseConvolution_accGradParameters_noAlloc(state, T(x), T(gy), T(gw4), T(gb4), kW, kH, dW, dH, pW, pH, 1.0f);
    check_tensor("depthwise accGradParameters_noAlloc: gradWeight", gw4, arr("dw_s2.gw"), 1e-3, 1e-3);
    check_tensor("depthwise accGradParameters_noAlloc: gradBias", gb4, arr("dw_s2.gb"), 1e-3, 1e-3);
    /* the same forward on a strided input: rows 5 floats apart from dense, 3 floats into the storage */
    CallerTensor *xs = tensor_from(arr("dw_s2.x"), 5, 3), *y2 = tensor_empty();
    THNN_CudaSpatialDepthWiseConvolution_updateOutput(state, T(xs), T(y2), T(w), T(b), T(columns), T(ones), kW, kH, dW, dH, pW, pH);
    check_tensor("depthwise updateOutput from a strided input at a storage offset", y2, arr("dw_s2.y"), 1e-5, 1e-4);
    /* an output that already has the right size is used as it is: no new storage */
    float *before = y->storage->data;
    THNN_CudaSpatialDepthWiseConvolution_updateOutput(state, T(x), T(y), T(w), T(b), T(columns), T(ones), kW, kH, dW, dH, pW, pH);
    check_tensor("depthwise updateOutput into an output of the right size", y, arr("dw_s2.y"), 1e-5, 1e-4);
    report("... keeps the caller's storage", y->storage->data == before, NULL);
    /* a bias of the wrong shape: the TH handler is called, nothing is launched, the output is untouched */
    const long badDims[2] = {M, C + 1};
    CallerTensor *bad = tensor_zeros(2, badDims), *y3 = tensor_empty();
    const int seen = errors_seen;
    THNN_CudaSpatialDepthWiseConvolution_updateOutput(state, T(x), T(y3), T(w), T(bad), T(columns), T(ones), kW, kH, dW, dH, pW, pH);
    report("depthwise updateOutput with a mis-shaped bias reports through the TH handler", errors_seen == seen + 1 &&
           y3->nDimension == 0 && y3->storage == NULL, last_error);
    THCState_synchronize(state);
    tensor_free(x), tensor_free(gy), tensor_free(b), tensor_free(w), tensor_free(y), tensor_free(gx), tensor_free(columns);
    tensor_free(ones), tensor_free(gw), tensor_free(gb), tensor_free(xs), tensor_free(y2), tensor_free(bad), tensor_free(y3);
    tensor_free(gw4), tensor_free(gb4);
  }

  /* ---- SpatialConvolutionMM, all three passes (golden cases conv_3x3 and the strided conv_s2), and the fused
   *      SpatialConvolutionMM + ReLU forward against max(golden output, 0) ---- */
  for (int which = 0; which < 2; ++which) {
    c = which ? "conv_s2" : "conv_3x3";
    const int kW = geom(NM("geom"), 0), kH = geom(NM("geom"), 1), dW = geom(NM("geom"), 2), dH = geom(NM("geom"), 3),
              pW = geom(NM("geom"), 4), pH = geom(NM("geom"), 5);
    CallerTensor *x = tensor_from(arr(NM("x")), 0, 0), *w = tensor_from(arr(NM("w")), 0, 0), *b = tensor_from(arr(NM("b")), 0, 0);
    CallerTensor *gy = tensor_from(arr(NM("gy")), 0, 0);
    CallerTensor *y = tensor_empty(), *gx = tensor_empty(), *columns = tensor_empty(), *gradColumns = tensor_empty(), *ones = tensor_empty();
    THNN_CudaSpatialConvolutionMM_updateOutput(state, T(x), T(y), T(w), T(b), T(columns), T(ones), kW, kH, dW, dH, pW, pH);
    check_tensor(which ? "SpatialConvolutionMM updateOutput, stride 2" : "SpatialConvolutionMM updateOutput into an empty output", y, arr(NM("y")), 1e-5, 1e-4);
    THNN_CudaSpatialConvolutionMM_updateGradInput(state, T(x), T(gy), T(gx), T(w), T(gradColumns), T(ones), kW, kH, dW, dH, pW, pH);
    check_tensor(which ? "SpatialConvolutionMM updateGradInput, stride 2" : "SpatialConvolutionMM updateGradInput into an empty gradInput", gx, arr(NM("gx")), 1e-5, 1e-4);
    CallerTensor *gw = tensor_zeros(2, arr(NM("gw"))->dims), *gb = tensor_zeros(1, arr(NM("gb"))->dims);
    THNN_CudaSpatialConvolutionMM_accGradParameters(state, T(x), T(gy), T(gw), T(gb), T(columns), T(ones), kW, kH, dW, dH, pW, pH, 1.0f);
    check_tensor(which ? "SpatialConvolutionMM accGradParameters, stride 2: gradWeight" : "SpatialConvolutionMM accGradParameters: gradWeight", gw, arr(NM("gw")), 1e-3, 1e-3);
    check_tensor(which ? "SpatialConvolutionMM accGradParameters, stride 2: gradBias" : "SpatialConvolutionMM accGradParameters: gradBias", gb, arr(NM("gb")), 1e-3, 1e-3);
    CallerTensor *a = tensor_empty();
    Arr relu = derived(arr(NM("y")));
    for (long i = 0; i < relu.n; ++i) {
      const float v = ((const float *)arr(NM("y"))->data)[i];
      ((float *)relu.data)[i] = v > 0.f ? v : 0.f;
    }
    THNN_CudaSpatialConvolutionMMReLU_updateOutput(state, T(x), T(a), T(w), T(b), T(columns), T(ones), kW, kH, dW, dH, pW, pH);
    check_tensor(which ? "SpatialConvolutionMMReLU updateOutput (fused), stride 2" : "SpatialConvolutionMMReLU updateOutput (fused)", a, &relu, 1e-5, 1e-4);
    free(relu.data);
    THCState_synchronize(state);
    tensor_free(x), tensor_free(w), tensor_free(b), tensor_free(gy), tensor_free(y), tensor_free(gx), tensor_free(columns);
    tensor_free(gradColumns), tensor_free(ones), tensor_free(gw), tensor_free(gb), tensor_free(a);
  }

  /* ---- BatchNormalization: the one signature with `bool train, double, double` behind nine / eleven pointers
   *      (lib/THCUNN/generic/THCUNN.h:30-58). Train forward + backward, eval forward, NULL weight and bias ---- */
  {
    c = "bn_4d";
    const Arr *ax = arr(NM("x"));
    const long C = ax->dims[1], L = ax->dims[2] * ax->dims[3];
    CallerTensor *x = tensor_from(ax, 0, 0), *g = tensor_from(arr(NM("g")), 0, 0), *b = tensor_from(arr(NM("b")), 0, 0);
    CallerTensor *gy = tensor_from(arr(NM("gy")), 0, 0);
    CallerTensor *rm = tensor_const(C, 0.f), *rv = tensor_const(C, 1.f), *sm = tensor_const(C, 0.f), *ss = tensor_const(C, 0.f);
    CallerTensor *y = tensor_empty();
    THNN_CudaBatchNormalization_updateOutput(state, T(x), T(y), T(g), T(b), T(rm), T(rv), T(sm), T(ss), true, 0.1, 1e-5);
    check_tensor("BatchNormalization updateOutput (train) into an empty output", y, arr(NM("y")), 1e-5, 1e-4);
    check_tensor("BatchNormalization saveMean", sm, arr(NM("save_mean")), 1e-3, 1e-5);
    check_tensor("BatchNormalization saveStd (1 / sigma)", ss, arr(NM("save_std")), 1e-3, 1e-6);
    check_tensor("BatchNormalization runningMean after one step (momentum 0.1)", rm, arr(NM("run_mean")), 1e-3, 1e-5);
    check_tensor("BatchNormalization runningVar after one step (unbiased)", rv, arr(NM("run_var")), 1e-3, 1e-5);
    CallerTensor *gx = tensor_zeros(4, ax->dims), *gw = tensor_const(C, 0.f), *gb = tensor_const(C, 0.f);
    THNN_CudaBatchNormalization_backward(state, T(x), T(gy), T(gx), T(gw), T(gb), T(g), T(rm), T(rv), T(sm), T(ss), true, 1.0, 1e-5);
    check_tensor("BatchNormalization backward (train): gradInput", gx, arr(NM("gx")), 1e-5, 1e-4);
    check_tensor("BatchNormalization backward: gradWeight", gw, arr(NM("gw")), 1e-3, 1e-3);
    check_tensor("BatchNormalization backward: gradBias", gb, arr(NM("gb")), 1e-3, 1e-3);
    /* gradWeight / gradBias accumulate with `scale`: a second call with scale 0.5 leaves 1.5 x the gradients */
    THNN_CudaBatchNormalization_backward(state, T(x), T(gy), NULL, T(gw), T(gb), T(g), T(rm), T(rv), T(sm), T(ss), true, 0.5, 1e-5);
    Arr gw15 = derived(arr(NM("gw")));
    for (long i = 0; i < gw15.n; ++i) ((float *)gw15.data)[i] = 1.5f * ((const float *)arr(NM("gw"))->data)[i];
    check_tensor("BatchNormalization backward with NULL gradInput, scale 0.5: accumulated gradWeight", gw, &gw15, 1e-3, 1e-3);
    free(gw15.data);
    /* eval mode: normalises with the running statistics as the training step above left them */
    CallerTensor *ye = tensor_empty();
    THNN_CudaBatchNormalization_updateOutput(state, T(x), T(ye), T(g), T(b), T(rm), T(rv), T(sm), T(ss), false, 0.1, 1e-5);
    check_tensor("BatchNormalization updateOutput (eval, running statistics)", ye, arr(NM("y_eval")), 1e-5, 1e-4);
    /* no affine parameters: (x - mean) / sigma from the golden statistics */
    Arr plain = derived(ax);
    for (long i = 0; i < plain.n; ++i) {
      const long ch = (i / L) % C;
      ((float *)plain.data)[i] = (float)(((double)((const float *)ax->data)[i] - ((const float *)arr(NM("save_mean"))->data)[ch]) *
                                         ((const float *)arr(NM("save_std"))->data)[ch]);
    }
    CallerTensor *rm2 = tensor_const(C, 0.f), *rv2 = tensor_const(C, 1.f), *yp = tensor_empty();
    THNN_CudaBatchNormalization_updateOutput(state, T(x), T(yp), NULL, NULL, T(rm2), T(rv2), T(sm), T(ss), true, 0.1, 1e-5);
    check_tensor("BatchNormalization updateOutput with NULL weight and bias", yp, &plain, 1e-4, 1e-4);
    free(plain.data);
    THCState_synchronize(state);
    tensor_free(x), tensor_free(g), tensor_free(b), tensor_free(gy), tensor_free(rm), tensor_free(rv), tensor_free(sm), tensor_free(ss);
    tensor_free(y), tensor_free(gx), tensor_free(gw), tensor_free(gb), tensor_free(ye);
    tensor_free(rm2), tensor_free(rv2), tensor_free(yp);
  }

  /* ---- BatchNormalization + ReLU, the fused pair (include/THCUNN_fused.h; golden case bnrelu_4d) ---- */
  {
    c = "bnrelu_4d";
    const Arr *ax = arr(NM("x"));
    const long C = ax->dims[1];
    CallerTensor *x = tensor_from(ax, 0, 0), *g = tensor_from(arr(NM("g")), 0, 0), *b = tensor_from(arr(NM("b")), 0, 0);
    CallerTensor *ga = tensor_from(arr(NM("ga")), 0, 0);
    CallerTensor *rm = tensor_const(C, 0.f), *rv = tensor_const(C, 1.f), *sm = tensor_const(C, 0.f), *ss = tensor_const(C, 0.f);
    CallerTensor *a = tensor_empty(), *gx = tensor_zeros(4, ax->dims), *gw = tensor_const(C, 0.f), *gb = tensor_const(C, 0.f);
    THNN_CudaBatchNormalizationReLU_updateOutput(state, T(x), T(a), T(g), T(b), T(rm), T(rv), T(sm), T(ss), true, 0.1, 1e-5);
    check_tensor("BatchNormalizationReLU updateOutput (fused)", a, arr(NM("a")), 1e-5, 1e-4);
    THNN_CudaBatchNormalizationReLU_backward(state, T(x), T(ga), T(gx), T(gw), T(gb), T(g), T(b), T(rm), T(rv), T(sm), T(ss), true, 1.0, 1e-5);
    check_tensor("BatchNormalizationReLU backward (fused): gradInput", gx, arr(NM("gx")), 1e-5, 1e-4);
    check_tensor("BatchNormalizationReLU backward (fused): gradWeight", gw, arr(NM("gw")), 1e-3, 1e-3);
    check_tensor("BatchNormalizationReLU backward (fused): gradBias", gb, arr(NM("gb")), 1e-3, 1e-3);
    THCState_synchronize(state);
    tensor_free(x), tensor_free(g), tensor_free(b), tensor_free(ga), tensor_free(rm), tensor_free(rv), tensor_free(sm), tensor_free(ss);
    tensor_free(a), tensor_free(gx), tensor_free(gw), tensor_free(gb);
  }

  /* ---- SpatialMaxPooling / SpatialAveragePooling forward + backward (ceil mode: pool_3s2p1_ceil; floor: pool_2s2) ---- */
  for (int which = 0; which < 2; ++which) {
    c = which ? "pool_2s2" : "pool_3s2p1_ceil";
    const int kW = geom(NM("geom"), 0), kH = geom(NM("geom"), 1), dW = geom(NM("geom"), 2), dH = geom(NM("geom"), 3),
              pW = geom(NM("geom"), 4), pH = geom(NM("geom"), 5), ceil_mode = geom(NM("geom"), 6);
    CallerTensor *x = tensor_from(arr(NM("x")), 0, 0), *gy = tensor_from(arr(NM("gy")), 0, 0);
    CallerTensor *y = tensor_empty(), *gx = tensor_empty();
    CallerLongTensor *idx = long_tensor_empty();
    THNN_CudaSpatialMaxPooling_updateOutput(state, T(x), T(y), LT(idx), kW, kH, dW, dH, pW, pH, ceil_mode != 0);
    check_tensor(which ? "SpatialMaxPooling updateOutput 2x2 stride 2" : "SpatialMaxPooling updateOutput (ceil mode) into an empty output", y, arr(NM("max_y")), 0.0, 0.0);
    check_longs(which ? "SpatialMaxPooling indices 2x2 stride 2" : "SpatialMaxPooling indices (int64, 1-based) into an empty index tensor", idx, arr(NM("max_idx")));
    THNN_CudaSpatialMaxPooling_updateGradInput(state, T(x), T(gy), T(gx), LT(idx), kW, kH, dW, dH, pW, pH, ceil_mode != 0);
    check_tensor(which ? "SpatialMaxPooling updateGradInput 2x2 stride 2" : "SpatialMaxPooling updateGradInput into an empty gradInput", gx, arr(NM("max_gx")), 1e-5, 1e-4);
    for (int inc = 1; inc >= 0; --inc) {
      CallerTensor *ya = tensor_empty(), *gxa = tensor_empty();
      THNN_CudaSpatialAveragePooling_updateOutput(state, T(x), T(ya), kW, kH, dW, dH, pW, pH, ceil_mode != 0, inc != 0);
      check_tensor(inc ? "SpatialAveragePooling updateOutput (count_include_pad)" : "SpatialAveragePooling updateOutput (pad excluded)", ya,
                   arr(NM(inc ? "avg_y_1" : "avg_y_0")), 1e-5, 1e-4);
      THNN_CudaSpatialAveragePooling_updateGradInput(state, T(x), T(gy), T(gxa), kW, kH, dW, dH, pW, pH, ceil_mode != 0, inc != 0);
      check_tensor(inc ? "SpatialAveragePooling updateGradInput (count_include_pad)" : "SpatialAveragePooling updateGradInput (pad excluded)", gxa,
                   arr(NM(inc ? "avg_gx_1" : "avg_gx_0")), 1e-5, 1e-4);
      THCState_synchronize(state);
      tensor_free(ya), tensor_free(gxa);
    }
    THCState_synchronize(state);
    tensor_free(x), tensor_free(gy), tensor_free(y), tensor_free(gx), long_tensor_free(idx);
  }

  /* ---- SpatialDilatedMaxPooling with dilation 2 (golden case pool_dil2) ---- */
  {
    c = "pool_dil2";
    const int kW = geom(NM("geom"), 0), kH = geom(NM("geom"), 1), dW = geom(NM("geom"), 2), dH = geom(NM("geom"), 3),
              pW = geom(NM("geom"), 4), pH = geom(NM("geom"), 5), dilW = geom(NM("geom"), 6), dilH = geom(NM("geom"), 7),
              ceil_mode = geom(NM("geom"), 8);
    CallerTensor *x = tensor_from(arr(NM("x")), 0, 0), *gy = tensor_from(arr(NM("gy")), 0, 0), *y = tensor_empty(), *gx = tensor_empty();
    CallerLongTensor *idx = long_tensor_empty();
    THNN_CudaSpatialDilatedMaxPooling_updateOutput(state, T(x), T(y), LT(idx), kW, kH, dW, dH, pW, pH, dilW, dilH, ceil_mode != 0);
    check_tensor("SpatialDilatedMaxPooling updateOutput (dilation 2)", y, arr(NM("max_y")), 0.0, 0.0);
    check_longs("SpatialDilatedMaxPooling indices (dilation 2)", idx, arr(NM("max_idx")));
    THNN_CudaSpatialDilatedMaxPooling_updateGradInput(state, T(x), T(gy), T(gx), LT(idx), kW, kH, dW, dH, pW, pH, dilW, dilH, ceil_mode != 0);
    check_tensor("SpatialDilatedMaxPooling updateGradInput (dilation 2)", gx, arr(NM("max_gx")), 1e-5, 1e-4);
    THCState_synchronize(state);
    tensor_free(x), tensor_free(gy), tensor_free(y), tensor_free(gx), long_tensor_free(idx);
  }

  /* ---- SpatialDilatedConvolution, dilation 2 (golden case dilconv_d2; 4-D weight) ---- */
  {
    c = "dilconv_d2";
    const int kW = geom(NM("geom"), 0), kH = geom(NM("geom"), 1), dW = geom(NM("geom"), 2), dH = geom(NM("geom"), 3),
              pW = geom(NM("geom"), 4), pH = geom(NM("geom"), 5), dilW = geom(NM("geom"), 6), dilH = geom(NM("geom"), 7);
    CallerTensor *x = tensor_from(arr(NM("x")), 0, 0), *w = tensor_from(arr(NM("w")), 0, 0), *b = tensor_from(arr(NM("b")), 0, 0);
    CallerTensor *gy = tensor_from(arr(NM("gy")), 0, 0);
    CallerTensor *y = tensor_empty(), *gx = tensor_empty(), *columns = tensor_empty(), *gradColumns = tensor_empty(), *ones = tensor_empty();
    THNN_CudaSpatialDilatedConvolution_updateOutput(state, T(x), T(y), T(w), T(b), T(columns), T(ones), kW, kH, dW, dH, pW, pH, dilW, dilH);
    check_tensor("SpatialDilatedConvolution updateOutput (dilation 2)", y, arr(NM("y")), 1e-5, 1e-4);
    THNN_CudaSpatialDilatedConvolution_updateGradInput(state, T(x), T(gy), T(gx), T(w), T(gradColumns), kW, kH, dW, dH, pW, pH, dilW, dilH);
    check_tensor("SpatialDilatedConvolution updateGradInput (dilation 2)", gx, arr(NM("gx")), 1e-5, 1e-4);
    CallerTensor *gw = tensor_zeros(4, arr(NM("gw"))->dims), *gb = tensor_zeros(1, arr(NM("gb"))->dims);
    THNN_CudaSpatialDilatedConvolution_accGradParameters(state, T(x), T(gy), T(gw), T(gb), T(columns), T(ones), kW, kH, dW, dH, pW, pH, dilW, dilH, 1.0f);
    check_tensor("SpatialDilatedConvolution accGradParameters: gradWeight", gw, arr(NM("gw")), 1e-3, 1e-3);
    check_tensor("SpatialDilatedConvolution accGradParameters: gradBias", gb, arr(NM("gb")), 1e-3, 1e-3);
    THCState_synchronize(state);
    tensor_free(x), tensor_free(w), tensor_free(b), tensor_free(gy), tensor_free(y), tensor_free(gx), tensor_free(columns);
    tensor_free(gradColumns), tensor_free(ones), tensor_free(gw), tensor_free(gb);
  }

  /* ---- SpatialFullConvolution and SpatialFullDilatedConvolution (dilation 1): the transposed convolution
   *      4x4 stride 2 pad 1 (golden case fullconv_s2; weight Cin x Cout x kH x kW) ---- */
  for (int dilated = 0; dilated < 2; ++dilated) {
    c = "fullconv_s2";
    const int kW = geom(NM("geom"), 0), kH = geom(NM("geom"), 1), dW = geom(NM("geom"), 2), dH = geom(NM("geom"), 3),
              pW = geom(NM("geom"), 4), pH = geom(NM("geom"), 5), aW = geom(NM("geom"), 6), aH = geom(NM("geom"), 7);
    CallerTensor *x = tensor_from(arr(NM("x")), 0, 0), *w = tensor_from(arr(NM("w")), 0, 0), *b = tensor_from(arr(NM("b")), 0, 0);
    CallerTensor *gy = tensor_from(arr(NM("gy")), 0, 0);
    CallerTensor *y = tensor_empty(), *gx = tensor_empty(), *columns = tensor_empty(), *gradColumns = tensor_empty(), *ones = tensor_empty();
    CallerTensor *gw = tensor_zeros(4, arr(NM("gw"))->dims), *gb = tensor_zeros(1, arr(NM("gb"))->dims);
    if (dilated) {
      THNN_CudaSpatialFullDilatedConvolution_updateOutput(state, T(x), T(y), T(w), T(b), T(columns), T(ones), kW, kH, dW, dH, pW, pH, 1, 1, aW, aH);
      THNN_CudaSpatialFullDilatedConvolution_updateGradInput(state, T(x), T(gy), T(gx), T(w), T(gradColumns), kW, kH, dW, dH, pW, pH, 1, 1, aW, aH);
      THNN_CudaSpatialFullDilatedConvolution_accGradParameters(state, T(x), T(gy), T(gw), T(gb), T(columns), T(ones), kW, kH, dW, dH, pW, pH, 1, 1, aW, aH, 1.0f);
    } else {
      THNN_CudaSpatialFullConvolution_updateOutput(state, T(x), T(y), T(w), T(b), T(columns), T(ones), kW, kH, dW, dH, pW, pH, aW, aH);
      THNN_CudaSpatialFullConvolution_updateGradInput(state, T(x), T(gy), T(gx), T(w), T(gradColumns), kW, kH, dW, dH, pW, pH, aW, aH);
      THNN_CudaSpatialFullConvolution_accGradParameters(state, T(x), T(gy), T(gw), T(gb), T(columns), T(ones), kW, kH, dW, dH, pW, pH, aW, aH, 1.0f);
    }
    check_tensor(dilated ? "SpatialFullDilatedConvolution updateOutput" : "SpatialFullConvolution updateOutput", y, arr(NM("y")), 1e-5, 1e-4);
    check_tensor(dilated ? "SpatialFullDilatedConvolution updateGradInput" : "SpatialFullConvolution updateGradInput", gx, arr(NM("gx")), 1e-5, 1e-4);
    check_tensor(dilated ? "SpatialFullDilatedConvolution accGradParameters: gradWeight" : "SpatialFullConvolution accGradParameters: gradWeight", gw, arr(NM("gw")), 1e-3, 1e-3);
    check_tensor(dilated ? "SpatialFullDilatedConvolution accGradParameters: gradBias" : "SpatialFullConvolution accGradParameters: gradBias", gb, arr(NM("gb")), 1e-3, 1e-3);
    THCState_synchronize(state);
    tensor_free(x), tensor_free(w), tensor_free(b), tensor_free(gy), tensor_free(y), tensor_free(gx), tensor_free(columns);
    tensor_free(gradColumns), tensor_free(ones), tensor_free(gw), tensor_free(gb);
  }

  /* ---- Threshold: out of place, then in place (the input tensor is also the output) ---- */
  {
    c = "thr";
    const float th = ((const float *)arr(NM("param"))->data)[0], val = ((const float *)arr(NM("param"))->data)[1];
    CallerTensor *x = tensor_from(arr(NM("x")), 0, 0), *gy = tensor_from(arr(NM("gy")), 0, 0), *y = tensor_empty(), *gx = tensor_empty();
    THNN_CudaThreshold_updateOutput(state, T(x), T(y), th, val, false);
    check_tensor("Threshold updateOutput", y, arr(NM("y")), 0.0, 0.0);
    THNN_CudaThreshold_updateGradInput(state, T(x), T(gy), T(gx), th, val, false);
    check_tensor("Threshold updateGradInput", gx, arr(NM("gx")), 0.0, 0.0);
    /* in place, backward first (it needs the unmodified input): gradOutput becomes gradInput, then input becomes output */
    THNN_CudaThreshold_updateGradInput(state, T(x), T(gy), T(gy), th, val, true);
    check_tensor("Threshold updateGradInput in place (gradOutput overwritten)", gy, arr(NM("gx")), 0.0, 0.0);
    THNN_CudaThreshold_updateOutput(state, T(x), T(x), th, val, true);
    check_tensor("Threshold updateOutput in place (input overwritten)", x, arr(NM("y")), 0.0, 0.0);
    THCState_synchronize(state);
    tensor_free(x), tensor_free(gy), tensor_free(y), tensor_free(gx);
  }

  THCState_free(state);
  printf("%d failure(s)\n", failures);
  return failures ? 1 : 0;
}
