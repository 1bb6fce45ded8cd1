// Streaming probes: what trivial kernels reach on this part with the traffic shapes and the grain of the
// bandwidth-bound kernels of this library (one 256-lane workgroup per 56 x 56 plane, at most four 16-byte
// loads per lane in flight, the same load and store helpers). The bandwidth figures of the depthwise,
// pooling and BatchNormalization kernels are read against these, not against the 8 TB/s peak alone.
//
//   read      x-like + gy-like band, nothing written          (accGradParameters stage 1: 128.45 MB read)
//   fwd 4:1   784 float4 read, 196 written per workgroup        (stride-2 forward pass)
//   bwd 1:4   196 float4 read, 784 written per workgroup        (stride-2 gradInput pass)
//   copy 1:1  784 float4 read, 784 written per workgroup        (stride-1 forward pass, BatchNormalization)
//
// Every probe runs with plain and with hinted accesses (loads: non-temporal; stores: nt and sc1 nt), over
// 4 and over 16 rotating buffer sets: with 4 sets the small tensors (4 x 25.7 MB) stay in the 256 MB Infinity
// Cache from one use to the next when they are read with plain loads, with 16 sets they do not; the large ones
// (102.8 MB each) never do. 240 launches per figure, timed by one pair of HIP events.
//
// Build: make -C cunn_amd/csrc probes   ->  cunn_amd/lib/stream_probe ; run without arguments.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../device_utils.h"

#define CK(x)                                                        \
  do {                                                               \
    hipError_t e_ = (x);                                             \
    if (e_ != hipSuccess) {                                          \
      fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));        \
      exit(1);                                                       \
    }                                                                \
  } while (0)

namespace {

constexpr int kPlanes = 64 * 128;  // workgroups per launch (N x C of the depthwise configuration)
constexpr int kBig = 784;          // float4 of a 56 x 56 plane
constexpr int kSmall = 196;        // float4 of a 28 x 28 plane

// LOADS: 0 plain, 1 non-temporal. STORES: 0 plain, 1 nt, 2 sc1 nt.
template <int LOADS>
__device__ __forceinline__ float4 load4(__amdgpu_buffer_rsrc_t r, int i) {
  return LOADS ? dev::bufLoadStream4(r, i * 16) : dev::bufLoad4(r, i * 16);
}
template <int STORES>
__device__ __forceinline__ void store4(__amdgpu_buffer_rsrc_t r, float *base, int i, float4 v) {
  if (STORES == 2)
    dev::bufStoreStream4(r, i * 16, v);
  else if (STORES == 1)
    dev::storeStream4(base + (long)i * 4, v);
  else
    reinterpret_cast<float4 *>(base)[i] = v;
}

// reads nIn float4 of `in` (+ nIn2 of `in2`), writes nOut float4 of `out` per workgroup; what is written is a
// sum of what was read, so that no load can be dropped
template <int LOADS, int STORES>
__global__ void __launch_bounds__(256)
streamKernel(const float *__restrict__ in, int nIn, const float *__restrict__ in2, int nIn2, float *__restrict__ out,
             int nOut, float *__restrict__ sink) {
  const int tid = threadIdx.x;
  const float *pin = in + (long)blockIdx.x * nIn * 4;
  const __amdgpu_buffer_rsrc_t rin = dev::makeRsrc(pin, (long)nIn * 16);
  float4 v[5];
#pragma unroll
  for (int u = 0; u < 4; ++u) v[u] = u * 256 + tid < nIn ? load4<LOADS>(rin, u * 256 + tid) : make_float4(0.f, 0.f, 0.f, 0.f);
  v[4] = make_float4(0.f, 0.f, 0.f, 0.f);
  if (nIn2 > 0) {
    const __amdgpu_buffer_rsrc_t rin2 = dev::makeRsrc(in2 + (long)blockIdx.x * nIn2 * 4, (long)nIn2 * 16);
    if (tid < nIn2) v[4] = load4<LOADS>(rin2, tid);
  }
  float4 s;
  s.x = (v[0].x + v[1].x) + (v[2].x + v[3].x) + v[4].x;
  s.y = (v[0].y + v[1].y) + (v[2].y + v[3].y) + v[4].y;
  s.z = (v[0].z + v[1].z) + (v[2].z + v[3].z) + v[4].z;
  s.w = (v[0].w + v[1].w) + (v[2].w + v[3].w) + v[4].w;
  if (nOut > 0) {
    float *pout = out + (long)blockIdx.x * nOut * 4;
    const __amdgpu_buffer_rsrc_t rout = dev::makeRsrc(pout, (long)nOut * 16);
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (u * 256 + tid < nOut) store4<STORES>(rout, pout, u * 256 + tid, nIn == nOut ? v[u] : s);
  } else if (s.x + s.y + s.z + s.w == 12345.678f) {
    sink[blockIdx.x] = s.x;  // never true for the fill pattern: keeps the loads alive
  }
}

struct Probe {
  const char *name;
  int nIn, nIn2, nOut;
};

template <int LOADS, int STORES>
double run(const Probe &p, int sets, const std::vector<float *> &big, const std::vector<float *> &big2,
           const std::vector<float *> &small, const std::vector<float *> &small2, float *sink) {
  const int launches = 240;
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  auto pick = [&](int n, int i, bool second) { return n == kBig ? (second ? big2 : big)[i] : (second ? small2 : small)[i]; };
  for (int pass = 0; pass < 2; ++pass) {
    if (pass == 1) CK(hipEventRecord(e0, 0));
    for (int it = 0; it < launches; ++it) {
      const int i = it % sets;
      const float *in = pick(p.nIn, i, false);
      const float *in2 = p.nIn2 ? small[i] : nullptr;
      float *out = p.nOut ? pick(p.nOut, i, true) : nullptr;
      streamKernel<LOADS, STORES><<<kPlanes, 256>>>(in, p.nIn, in2, p.nIn2, out, p.nOut, sink);
    }
  }
  CK(hipGetLastError());
  CK(hipEventRecord(e1, 0));
  CK(hipEventSynchronize(e1));
  float ms = 0.f;
  CK(hipEventElapsedTime(&ms, e0, e1));
  CK(hipEventDestroy(e0));
  CK(hipEventDestroy(e1));
  return 1e3 * ms / launches;  // microseconds per launch
}

}  // namespace

int main() {
  const int maxSets = 16;
  const size_t bigBytes = (size_t)kPlanes * kBig * 16, smallBytes = (size_t)kPlanes * kSmall * 16;
  std::vector<float *> big(maxSets), big2(maxSets), small(maxSets), small2(maxSets);
  for (int i = 0; i < maxSets; ++i) {
    CK(hipMalloc(&big[i], bigBytes));
    CK(hipMalloc(&big2[i], bigBytes));
    CK(hipMalloc(&small[i], smallBytes));
    CK(hipMalloc(&small2[i], smallBytes));
    CK(hipMemset(big[i], 1, bigBytes));
    CK(hipMemset(big2[i], 1, bigBytes));
    CK(hipMemset(small[i], 1, smallBytes));
    CK(hipMemset(small2[i], 1, smallBytes));
  }
  float *sink;
  CK(hipMalloc(&sink, kPlanes * sizeof(float)));
  const Probe probes[] = {{"read     (x + gy)", kBig, kSmall, 0},
                          {"fwd 4:1  (x -> y)", kBig, 0, kSmall},
                          {"bwd 1:4  (gy -> gx)", kSmall, 0, kBig},
                          {"copy 1:1 (x -> y)", kBig, 0, kBig}};
  printf("%-20s %-22s %5s %10s %9s %8s\n", "probe", "loads / stores", "sets", "MB/launch", "us", "TB/s");
  for (int rep = 0; rep < 2; ++rep)  // the second round runs at settled clocks; both are printed
    for (const Probe &p : probes)
      for (int sets : {4, 16}) {
        const double mb = (double)kPlanes * (p.nIn + p.nIn2 + p.nOut) * 16 / 1e6;
        auto line = [&](const char *pol, double us) {
          printf("%-20s %-22s %5d %10.2f %9.2f %8.2f\n", p.name, pol, sets, mb, us, mb / us);
        };
        line("plain / plain", run<0, 0>(p, sets, big, big2, small, small2, sink));
        line("nt / plain", run<1, 0>(p, sets, big, big2, small, small2, sink));
        if (p.nOut) {
          line("plain / nt", run<0, 1>(p, sets, big, big2, small, small2, sink));
          line("plain / sc1 nt", run<0, 2>(p, sets, big, big2, small, small2, sink));
          line("nt / nt", run<1, 1>(p, sets, big, big2, small, small2, sink));
          line("nt / sc1 nt", run<1, 2>(p, sets, big, big2, small, small2, sink));
        }
        fflush(stdout);
      }
  return 0;
}
