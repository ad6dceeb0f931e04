// The feature map of the callers, phi(x) = elu(x) + 1, as one launch for the queries and the
// keys of a block (the reference's layers run two elementwise torch kernels per tensor:
// layers/linfusion.py:88-89, layers/mlla.py:74-75, layers/rala.py:52-53), and its derivative.
// Elementwise and HBM-bound: 16-byte vectors, grid-stride.  The arithmetic follows torch's:
// elu in fp32 rounded to the tensor's type, then "+ 1" rounded again, so that a block gives
// the same result with either path (up to the last place of the two exp routines).
#include <hip/hip_runtime.h>

#include "fbla_kernels.h"

namespace fbla {
namespace feature {

namespace {

constexpr int kThreads = 256;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct Elems { static constexpr int kPerVec = 16 / sizeof(T); };

template <typename T> __device__ __forceinline__ T phi(T x) {
  const float xf = (float)x;
  const T e = (T)(xf > 0.f ? xf : expf(xf) - 1.f);  // torch's elu: exp(x) - 1, not expm1
  return (T)((float)e + 1.f);
}
template <typename T> __device__ __forceinline__ T dphi(T x, T g) {
  const float xf = (float)x;
  return (T)(xf > 0.f ? (float)g : (float)g * expf(xf));
}

template <typename T>
__device__ __forceinline__ void map_tensor(const T* __restrict__ x, T* __restrict__ y, int64_t n, int64_t first_vec,
                                           int64_t vec_step) {
  constexpr int E = Elems<T>::kPerVec;
  const int64_t nvec = n / E;
  // two vectors per trip, both requested before the first is mapped; the input is read once
  // (streaming hint), the output is left to the caches for the kernel that follows
  int64_t i = first_vec;
  for (; i + vec_step < nvec; i += 2 * vec_step) {
    union { u32x4 w; T e[E]; } in0, in1, out0, out1;
    in0.w = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(x + i * E));
    in1.w = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(x + (i + vec_step) * E));
#pragma unroll
    for (int j = 0; j < E; ++j) out0.e[j] = phi(in0.e[j]);
#pragma unroll
    for (int j = 0; j < E; ++j) out1.e[j] = phi(in1.e[j]);
    *reinterpret_cast<u32x4*>(y + i * E) = out0.w;
    *reinterpret_cast<u32x4*>(y + (i + vec_step) * E) = out1.w;
  }
  if (i < nvec) {
    union { u32x4 w; T e[E]; } in, out;
    in.w = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(x + i * E));
#pragma unroll
    for (int j = 0; j < E; ++j) out.e[j] = phi(in.e[j]);
    *reinterpret_cast<u32x4*>(y + i * E) = out.w;
  }
  // the last, partial vector
  const int64_t tail = nvec * E + first_vec;
  if (tail < n && first_vec < E) y[tail] = phi(x[tail]);
}

// workgroups [0, wgs0) take tensor 0, the rest tensor 1
template <typename T>
__global__ __launch_bounds__(kThreads) void elu1_fwd_kernel(const T* __restrict__ x0, T* __restrict__ y0, int64_t n0,
                                                            const T* __restrict__ x1, T* __restrict__ y1, int64_t n1,
                                                            int wgs0) {
  const bool second = (int)blockIdx.x >= wgs0;
  const int wg = second ? blockIdx.x - wgs0 : blockIdx.x;
  const int wgs = second ? gridDim.x - wgs0 : wgs0;
  const int64_t first = (int64_t)wg * kThreads + threadIdx.x, step = (int64_t)wgs * kThreads;
  if (second) map_tensor<T>(x1, y1, n1, first, step);
  else map_tensor<T>(x0, y0, n0, first, step);
}

template <typename T>
__global__ __launch_bounds__(kThreads) void elu1_bwd_kernel(const T* __restrict__ x, const T* __restrict__ g,
                                                            T* __restrict__ dx, int64_t n) {
  constexpr int E = Elems<T>::kPerVec;
  const int64_t nvec = n / E;
  const int64_t first = (int64_t)blockIdx.x * kThreads + threadIdx.x, step = (int64_t)gridDim.x * kThreads;
  for (int64_t i = first; i < nvec; i += step) {
    union { u32x4 w; T e[E]; } xin, gin, out;
    xin.w = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(x + i * E));
    gin.w = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(g + i * E));
#pragma unroll
    for (int j = 0; j < E; ++j) out.e[j] = dphi(xin.e[j], gin.e[j]);
    *reinterpret_cast<u32x4*>(dx + i * E) = out.w;
  }
  const int64_t tail = nvec * E + first;
  if (tail < n && first < E) dx[tail] = dphi(x[tail], g[tail]);
}

// enough workgroups to fill the GPU a few times over, no more than the tensor has vectors
int grid_for(int64_t n, int elems_per_vec) {
  const int64_t nvec = (n + elems_per_vec - 1) / elems_per_vec;
  const int64_t want = (nvec + kThreads - 1) / kThreads;
  const int64_t cap = 256 * 8;
  return (int)(want < 1 ? 1 : (want > cap ? cap : want));
}

template <typename T>
void launch_fwd(const void* x0, void* y0, int64_t n0, const void* x1, void* y1, int64_t n1, hipStream_t st) {
  const int wgs0 = n0 > 0 ? grid_for(n0, Elems<T>::kPerVec) : 0;
  const int wgs1 = n1 > 0 ? grid_for(n1, Elems<T>::kPerVec) : 0;
  if (wgs0 + wgs1 == 0) return;
  elu1_fwd_kernel<T><<<dim3((unsigned)(wgs0 + wgs1)), dim3(kThreads), 0, st>>>(
      (const T*)x0, (T*)y0, n0, (const T*)x1, (T*)y1, n1, wgs0);
}

template <typename T>
void launch_bwd(const void* x, const void* g, void* dx, int64_t n, hipStream_t st) {
  if (n <= 0) return;
  elu1_bwd_kernel<T><<<dim3((unsigned)grid_for(n, Elems<T>::kPerVec)), dim3(kThreads), 0, st>>>(
      (const T*)x, (const T*)g, (T*)dx, n);
}

}  // namespace

void elu1_fwd(const void* x0, void* y0, int64_t n0, const void* x1, void* y1, int64_t n1, int dtype,
              hipStream_t st) {
  if (dtype == kF16) launch_fwd<_Float16>(x0, y0, n0, x1, y1, n1, st);
  else if (dtype == kBF16) launch_fwd<__bf16>(x0, y0, n0, x1, y1, n1, st);
  else launch_fwd<float>(x0, y0, n0, x1, y1, n1, st);
}

void elu1_bwd(const void* x, const void* g, void* dx, int64_t n, int dtype, hipStream_t st) {
  if (dtype == kF16) launch_bwd<_Float16>(x, g, dx, n, st);
  else if (dtype == kBF16) launch_bwd<__bf16>(x, g, dx, n, st);
  else launch_bwd<float>(x, g, dx, n, st);
}

}  // namespace feature
}  // namespace fbla
