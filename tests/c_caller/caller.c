/*
 * A caller of libTHCUNN.so that is not the library's own harness: plain C, compiled against
 * include/THCUNN.h only, playing what LuaJIT + cutorch do under THCUNN.lua:129-133.
 *
 * It builds every THCudaTensor / THCudaStorage itself (own malloc'ed size / stride arrays, storage
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

#include "THCUNN.h"

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
static THCudaStorage *storage_new(long elems) {
  THCudaStorage *s = (THCudaStorage *)calloc(1, sizeof(THCudaStorage));
  s->size = elems;
  s->refcount = 1;
  s->flag = TH_STORAGE_REFCOUNTED | TH_STORAGE_RESIZABLE | TH_STORAGE_FREEMEM; /* an owned cutorch storage */
  s->allocator = NULL;
  s->allocatorContext = NULL;
  s->view = NULL;
  s->device = 0;
  if (elems > 0) HIP_OK(hipMalloc((void **)&s->data, elems * sizeof(float)));
  return s;
}

/* THCudaTensor_new(): no dimensions, no storage */
static THCudaTensor *tensor_empty(void) {
  THCudaTensor *t = (THCudaTensor *)calloc(1, sizeof(THCudaTensor));
  t->refcount = 1;
  t->flag = TH_TENSOR_REFCOUNTED;
  return t;
}

/* A tensor of the given sizes over its own storage; rows (the last dimension) lie `pitch` floats apart
 * (pitch == last size: contiguous) and the tensor starts `offset` floats into the storage. */
static THCudaTensor *tensor_sized(int nd, const long *dims, long pitch, long offset) {
  THCudaTensor *t = tensor_empty();
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

static THCudaTensor *tensor_from(const Arr *a, long extraPitch, long offset) {
  const long W = a->dims[a->nd - 1], pitch = W + extraPitch, rows = a->n / W;
  THCudaTensor *t = tensor_sized(a->nd, a->dims, pitch, offset);
  float *host = (float *)malloc(sizeof(float) * (rows * pitch + offset));
  for (long i = 0; i < rows * pitch + offset; ++i) host[i] = NAN; /* whatever is read outside the view poisons the result */
  for (long r = 0; r < rows; ++r) memcpy(host + offset + r * pitch, (const float *)a->data + r * W, sizeof(float) * W);
  HIP_OK(hipMemcpy(t->storage->data, host, sizeof(float) * (rows * pitch + offset), 1));
  free(host);
  return t;
}

static THCudaTensor *tensor_zeros(int nd, const long *dims) {
  THCudaTensor *t = tensor_sized(nd, dims, dims[nd - 1], 0);
  HIP_OK(hipMemset(t->storage->data, 0, sizeof(float) * t->storage->size));
  return t;
}

static THCudaLongTensor *long_tensor_empty(void) {
  THCudaLongTensor *t = (THCudaLongTensor *)calloc(1, sizeof(THCudaLongTensor));
  t->refcount = 1;
  t->flag = TH_TENSOR_REFCOUNTED;
  return t;
}

static void tensor_free(THCudaTensor *t) {
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
static void check_tensor(const char *what, const THCudaTensor *t, const Arr *want, double rtol, double atol) {
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

static void check_longs(const char *what, const THCudaLongTensor *t, const Arr *want) {
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

  /* ---- SpatialDepthWiseConvolution: forward, gradInput, accGradParameters (golden case dw_s2) ---- */
  {
    const int kW = geom("dw_s2.geom", 0), kH = geom("dw_s2.geom", 1), dW = geom("dw_s2.geom", 2), dH = geom("dw_s2.geom", 3),
              pW = geom("dw_s2.geom", 4), pH = geom("dw_s2.geom", 5);
    const Arr *w4 = arr("dw_s2.w");
    const long M = w4->dims[0], C = w4->dims[1];
    THCudaTensor *x = tensor_from(arr("dw_s2.x"), 0, 0), *gy = tensor_from(arr("dw_s2.gy"), 0, 0), *b = tensor_from(arr("dw_s2.b"), 0, 0);
    /* the nn module holds the weight 2-D, (nOutputPlane, nInputPlane*kH*kW): the library reshapes it in place */
    const long w2dims[2] = {M, C * kH * kW};
    Arr w2 = *w4;
    w2.nd = 2, w2.dims[0] = w2dims[0], w2.dims[1] = w2dims[1];
    THCudaTensor *w = tensor_from(&w2, 0, 0);
    THCudaTensor *y = tensor_empty(), *gx = tensor_empty(), *columns = tensor_empty(), *ones = tensor_empty();
    THNN_CudaSpatialDepthWiseConvolution_updateOutput(state, x, y, w, b, columns, ones, kW, kH, dW, dH, pW, pH);
    check_tensor("depthwise updateOutput into an empty output (resized by the callee)", y, arr("dw_s2.y"), 1e-5, 1e-4);
    report("depthwise 2-D weight reshaped to 4-D in place", w->nDimension == 4 && w->size[0] == M && w->size[1] == C &&
           w->size[2] == kH && w->size[3] == kW && w->stride[3] == 1, NULL);
    THNN_CudaSpatialDepthWiseConvolution_updateGradInput(state, x, gy, gx, w, columns, ones, kW, kH, dW, dH, pW, pH);
    check_tensor("depthwise updateGradInput into an empty gradInput", gx, arr("dw_s2.gx"), 1e-5, 1e-4);
    THCudaTensor *gw = tensor_zeros(2, w2dims), *gb = tensor_zeros(2, arr("dw_s2.b")->dims);
    THNN_CudaSpatialDepthWiseConvolution_accGradParameters(state, x, gy, gw, gb, columns, ones, kW, kH, dW, dH, pW, pH, 1.0f);
    check_tensor("depthwise accGradParameters: gradWeight (2-D, reshaped in place)", gw, arr("dw_s2.gw"), 1e-3, 1e-3);
    check_tensor("depthwise accGradParameters: gradBias", gb, arr("dw_s2.gb"), 1e-3, 1e-3);
    /* the same forward on a strided input: rows 5 floats apart from dense, 3 floats into the storage */
    THCudaTensor *xs = tensor_from(arr("dw_s2.x"), 5, 3), *y2 = tensor_empty();
    THNN_CudaSpatialDepthWiseConvolution_updateOutput(state, xs, y2, w, b, columns, ones, kW, kH, dW, dH, pW, pH);
    check_tensor("depthwise updateOutput from a strided input at a storage offset", y2, arr("dw_s2.y"), 1e-5, 1e-4);
    /* an output that already has the right size is used as it is: no new storage */
    float *before = y->storage->data;
    THNN_CudaSpatialDepthWiseConvolution_updateOutput(state, x, y, w, b, columns, ones, kW, kH, dW, dH, pW, pH);
    check_tensor("depthwise updateOutput into an output of the right size", y, arr("dw_s2.y"), 1e-5, 1e-4);
    report("... keeps the caller's storage", y->storage->data == before, NULL);
    /* a bias of the wrong shape: the TH handler is called, nothing is launched, the output is untouched */
    const long badDims[2] = {M, C + 1};
    THCudaTensor *bad = tensor_zeros(2, badDims), *y3 = tensor_empty();
    const int seen = errors_seen;
    THNN_CudaSpatialDepthWiseConvolution_updateOutput(state, x, y3, w, bad, columns, ones, kW, kH, dW, dH, pW, pH);
    report("depthwise updateOutput with a mis-shaped bias reports through the TH handler", errors_seen == seen + 1 &&
           y3->nDimension == 0 && y3->storage == NULL, last_error);
    THCState_synchronize(state);
    tensor_free(x), tensor_free(gy), tensor_free(b), tensor_free(w), tensor_free(y), tensor_free(gx), tensor_free(columns);
    tensor_free(ones), tensor_free(gw), tensor_free(gb), tensor_free(xs), tensor_free(y2), tensor_free(bad), tensor_free(y3);
  }

  /* ---- SpatialConvolutionMM forward (golden case conv_3x3) ---- */
  {
    const int kW = geom("conv_3x3.geom", 0), kH = geom("conv_3x3.geom", 1), dW = geom("conv_3x3.geom", 2),
              dH = geom("conv_3x3.geom", 3), pW = geom("conv_3x3.geom", 4), pH = geom("conv_3x3.geom", 5);
    THCudaTensor *x = tensor_from(arr("conv_3x3.x"), 0, 0), *w = tensor_from(arr("conv_3x3.w"), 0, 0), *b = tensor_from(arr("conv_3x3.b"), 0, 0);
    THCudaTensor *gy = tensor_from(arr("conv_3x3.gy"), 0, 0);
    THCudaTensor *y = tensor_empty(), *gx = tensor_empty(), *columns = tensor_empty(), *gradColumns = tensor_empty(), *ones = tensor_empty();
    THNN_CudaSpatialConvolutionMM_updateOutput(state, x, y, w, b, columns, ones, kW, kH, dW, dH, pW, pH);
    check_tensor("SpatialConvolutionMM updateOutput into an empty output", y, arr("conv_3x3.y"), 1e-5, 1e-4);
    THNN_CudaSpatialConvolutionMM_updateGradInput(state, x, gy, gx, w, gradColumns, ones, kW, kH, dW, dH, pW, pH);
    check_tensor("SpatialConvolutionMM updateGradInput into an empty gradInput", gx, arr("conv_3x3.gx"), 1e-5, 1e-4);
    THCudaTensor *gw = tensor_zeros(2, arr("conv_3x3.gw")->dims), *gb = tensor_zeros(1, arr("conv_3x3.gb")->dims);
    THNN_CudaSpatialConvolutionMM_accGradParameters(state, x, gy, gw, gb, columns, ones, kW, kH, dW, dH, pW, pH, 1.0f);
    check_tensor("SpatialConvolutionMM accGradParameters: gradWeight", gw, arr("conv_3x3.gw"), 1e-3, 1e-3);
    check_tensor("SpatialConvolutionMM accGradParameters: gradBias", gb, arr("conv_3x3.gb"), 1e-3, 1e-3);
    THCState_synchronize(state);
    tensor_free(x), tensor_free(w), tensor_free(b), tensor_free(gy), tensor_free(y), tensor_free(gx), tensor_free(columns);
    tensor_free(gradColumns), tensor_free(ones), tensor_free(gw), tensor_free(gb);
  }

  /* ---- SpatialMaxPooling forward + backward (golden case pool_3s2p1_ceil: ceil mode) ---- */
  {
    const char *c = "pool_3s2p1_ceil";
    char nm[96];
#define NM(suffix) (snprintf(nm, sizeof(nm), "%s.%s", c, suffix), nm)
    const int kW = geom(NM("geom"), 0), kH = geom(NM("geom"), 1), dW = geom(NM("geom"), 2), dH = geom(NM("geom"), 3),
              pW = geom(NM("geom"), 4), pH = geom(NM("geom"), 5), ceil_mode = geom(NM("geom"), 6);
    THCudaTensor *x = tensor_from(arr(NM("x")), 0, 0), *gy = tensor_from(arr(NM("gy")), 0, 0);
    THCudaTensor *y = tensor_empty(), *gx = tensor_empty();
    THCudaLongTensor *idx = long_tensor_empty();
    THNN_CudaSpatialMaxPooling_updateOutput(state, x, y, idx, kW, kH, dW, dH, pW, pH, ceil_mode != 0);
    check_tensor("SpatialMaxPooling updateOutput (ceil mode) into an empty output", y, arr(NM("max_y")), 0.0, 0.0);
    check_longs("SpatialMaxPooling indices (int64, 1-based) into an empty index tensor", idx, arr(NM("max_idx")));
    THNN_CudaSpatialMaxPooling_updateGradInput(state, x, gy, gx, idx, kW, kH, dW, dH, pW, pH, ceil_mode != 0);
    check_tensor("SpatialMaxPooling updateGradInput into an empty gradInput", gx, arr(NM("max_gx")), 1e-5, 1e-4);
    THCudaTensor *ya = tensor_empty();
    THNN_CudaSpatialAveragePooling_updateOutput(state, x, ya, kW, kH, dW, dH, pW, pH, ceil_mode != 0, true);
    check_tensor("SpatialAveragePooling updateOutput (ceil mode, count_include_pad)", ya, arr(NM("avg_y_1")), 1e-5, 1e-4);
    THCState_synchronize(state);
    tensor_free(x), tensor_free(gy), tensor_free(y), tensor_free(gx), tensor_free(ya);
    if (idx->storage) {
      HIP_OK(hipFree(idx->storage->data));
      free(idx->storage);
    }
    free(idx->size), free(idx->stride), free(idx);
  }

  THCState_free(state);
  printf("%d failure(s)\n", failures);
  return failures ? 1 : 0;
}
