// Threshold (ReLU and friends) for gfx950: the element-wise step either side of the convolution
// path (conv -> BN -> ReLU).
//   updateOutput     out = x > threshold ? x : val            (lib/THCUNN/Threshold.cu:6-40)
//   updateGradInput  gradIn = x > threshold ? gradOut : 0     (lib/THCUNN/Threshold.cu:42-74)
// with the in-place variants of lib/THCUNN/generic/Threshold.cu:18-25, 50-56 (the result tensor
// becomes a view of the tensor that was overwritten). Pure streaming: 16-byte loads, one
// 16-byte streaming store per lane, one-shot workgroups in memory order.
#include "device_utils.h"
#include "launch_utils.h"
#include "thc_internal.h"

using namespace thc;

namespace {

// GRAD: out = x > thr ? other : 0 (other = gradOutput); else out = x > thr ? x : val.
// The in-place entry points pass out == x (forward) or out == other (backward): no __restrict__ here.
template <bool GRAD>
__global__ void __launch_bounds__(dev::kBlock)
thresholdKernel4(const float *x, const float *other, float *out, long n4, float thr, float val) {
  const long i = (long)blockIdx.x * dev::kBlock + threadIdx.x;
  if (i >= n4) return;
  // the backward pass is the last reader of the layer's input and of gradOutput: non-temporal loads
  typedef float f32x4v __attribute__((ext_vector_type(4)));
  auto loadOnce = [](const float *p, long at) {
    const f32x4v v = __builtin_nontemporal_load(reinterpret_cast<const f32x4v *>(p) + at);
    return make_float4(v.x, v.y, v.z, v.w);
  };
  const float4 a = GRAD ? loadOnce(x, i) : reinterpret_cast<const float4 *>(x)[i];
  float4 r;
  if (GRAD) {
    const float4 g = loadOnce(other, i);
    r = make_float4(a.x > thr ? g.x : 0.f, a.y > thr ? g.y : 0.f, a.z > thr ? g.z : 0.f, a.w > thr ? g.w : 0.f);
  } else {
    r = make_float4(a.x > thr ? a.x : val, a.y > thr ? a.y : val, a.z > thr ? a.z : val, a.w > thr ? a.w : val);
  }
  dev::storeStream4(out + i * 4, r);
}

template <bool GRAD>
__global__ void __launch_bounds__(dev::kBlock)
thresholdKernel1(const float *x, const float *other, float *out, long begin, long n, float thr, float val) {
  const long i = begin + (long)blockIdx.x * dev::kBlock + threadIdx.x;
  if (i >= n) return;
  const float a = x[i];
  out[i] = GRAD ? (a > thr ? other[i] : 0.f) : (a > thr ? a : val);
}

// contiguous arrays of n floats; out may alias x or other
template <bool GRAD>
void launchThreshold(hipStream_t s, const float *x, const float *other, float *out, long n, float thr, float val) {
  if (n <= 0) return;
  const bool vec = launch::aligned16(x) && launch::aligned16(out) && (!GRAD || launch::aligned16(other));
  const long n4 = vec ? n / 4 : 0;
  if (n4 > 0) {
    if ((n4 + dev::kBlock - 1) / dev::kBlock >= 0x7fffffffL) error("Threshold: tensor too large");
    thresholdKernel4<GRAD><<<(unsigned)((n4 + dev::kBlock - 1) / dev::kBlock), dev::kBlock, 0, s>>>(x, other, out, n4, thr, val);
    THC_HIP_CHECK(hipGetLastError());
  }
  const long rest = n - n4 * 4;
  if (rest > 0) {
    if ((rest + dev::kBlock - 1) / dev::kBlock >= 0x7fffffffL) error("Threshold: tensor too large");
    thresholdKernel1<GRAD><<<(unsigned)((rest + dev::kBlock - 1) / dev::kBlock), dev::kBlock, 0, s>>>(x, other, out, n4 * 4, n, thr, val);
    THC_HIP_CHECK(hipGetLastError());
  }
}

}  // namespace

namespace thc {
void reluInPlace(hipStream_t s, float *x, long n) { launchThreshold<false>(s, x, nullptr, x, n, 0.f, 0.f); }
}  // namespace thc

namespace {

// A tensor's elements as a contiguous device array: the tensor's own memory when it is
// contiguous, else a packed temporary that `commit` scatters back through the strides.
class Packed {
 public:
  Packed(THCState *state, THCudaTensor *t, bool load) : state_(state), t_(t) {
    if (isContiguous(erase(t))) {
      ptr_ = data(t);
    } else {
      tmp_ = Temp(state->stream, (size_t)numel(erase(t)) * sizeof(float));
      ptr_ = (float *)tmp_.get();
      if (load) stridedCopy(state->stream, erase(t), ptr_, sizeof(float), true);
      packed_ = true;
    }
  }
  float *ptr() const { return ptr_; }
  void commit() {
    if (packed_) stridedCopy(state_->stream, erase(t_), ptr_, sizeof(float), false);
  }

 private:
  THCState *state_;
  THCudaTensor *t_;
  float *ptr_ = nullptr;
  Temp tmp_;
  bool packed_ = false;
};

// THCTensor_(resizeAs)
void resizeAs(THCState *state, THCudaTensor *t, const THCudaTensor *src) {
  tensorResize(state, erase(t), src->nDimension, src->size, sizeof(float));
}

// THCTensor_(set): t becomes a view of src's storage with src's sizes and strides
void setTo(THCudaTensor *t, THCudaTensor *src) {
  if (t == src) return;
  tensorSetView(erase(t), erase(src)->storage, src->storageOffset, src->nDimension, src->size, src->stride);
}

}  // namespace

extern "C" {

void THNN_CudaThreshold_updateOutput(THCState *state, THCudaTensor *input, THCudaTensor *output, float threshold,
                                     float val, bool inplace) {
  THNN_ENTER
  THC_ARG_CHECK(input != nullptr, 2, "input tensor expected");
  THC_ARG_CHECK(output != nullptr, 3, "output tensor expected");
  const long n = numel(erase(input));
  if (inplace) {
    Packed x(state, input, true);
    launchThreshold<false>(state->stream, x.ptr(), nullptr, x.ptr(), n, threshold, val);
    x.commit();
    setTo(output, input);
  } else {
    resizeAs(state, output, input);
    Contiguous x(state, input);
    Packed y(state, output, false);
    launchThreshold<false>(state->stream, x.ptr(), nullptr, y.ptr(), n, threshold, val);
    y.commit();
  }
  THNN_LEAVE
}

void THNN_CudaThreshold_updateGradInput(THCState *state, THCudaTensor *input, THCudaTensor *gradOutput,
                                        THCudaTensor *gradInput, float threshold, float val, bool inplace) {
  THNN_ENTER
  (void)val;
  THC_ARG_CHECK(input != nullptr, 2, "input tensor expected");
  THC_ARG_CHECK(gradOutput != nullptr, 3, "gradOutput tensor expected");
  THC_ARG_CHECK(gradInput != nullptr, 4, "gradInput tensor expected");
  const long n = numel(erase(input)), n2 = numel(erase(gradOutput));
  if (n != n2)  // THCUNN_check_nElement (lib/THCUNN/common.h:49-61)
    error("input and gradOutput have different number of elements: input%s has %ld elements, while gradOutput%s has %ld "
          "elements",
          sizeDesc(erase(input)).c_str(), n, sizeDesc(erase(gradOutput)).c_str(), n2);
  Contiguous x(state, input);
  if (inplace) {
    Packed g(state, gradOutput, true);
    launchThreshold<true>(state->stream, x.ptr(), g.ptr(), g.ptr(), n, threshold, 0.f);
    g.commit();
    setTo(gradInput, gradOutput);
  } else {
    resizeAs(state, gradInput, input);
    Contiguous g(state, gradOutput);
    Packed gi(state, gradInput, false);
    launchThreshold<true>(state->stream, x.ptr(), g.ptr(), gi.ptr(), n, threshold, 0.f);
    gi.commit();
  }
  THNN_LEAVE
}

}  // extern "C"
