// Dynamic Tanh norm around an fp32 residual stream, and the squared ReLU.
//
//   dyt(x) = tanh(alpha x) * w + b   per element: no mean, no variance, nothing couples a row's entries.
// So the residual add, the norm of the new residual and the cast for the next GEMM are ONE elementwise
// pass: x is read and written once (fp32), the sublayer outputs are read once (fp32), the activations
// written once (TA: bf16 as uint16_t, or float).  Four consecutive columns per thread where the width
// allows 16-byte accesses.
#include "common.h"

namespace k8s {

template <typename T>
__device__ __forceinline__ float ldd(const T* p, size_t i);
template <>
__device__ __forceinline__ float ldd<float>(const float* p, size_t i) { return p[i]; }
template <>
__device__ __forceinline__ float ldd<uint16_t>(const uint16_t* p, size_t i) { return bf2f(p[i]); }
template <typename T>
__device__ __forceinline__ void std_(T* p, size_t i, float v);
template <>
__device__ __forceinline__ void std_<float>(float* p, size_t i, float v) { p[i] = v; }
template <>
__device__ __forceinline__ void std_<uint16_t>(uint16_t* p, size_t i, float v) { p[i] = f2bf(v); }

template <typename T>
__device__ __forceinline__ void st4(T* p, size_t i, const float (&v)[4]);
template <>
__device__ __forceinline__ void st4<float>(float* p, size_t i, const float (&v)[4]) {
  *reinterpret_cast<f32x4*>(p + i) = f32x4{v[0], v[1], v[2], v[3]};
}
template <>
__device__ __forceinline__ void st4<uint16_t>(uint16_t* p, size_t i, const float (&v)[4]) {
  *reinterpret_cast<u16x4*>(p + i) = u16x4{f2bf(v[0]), f2bf(v[1]), f2bf(v[2]), f2bf(v[3])};
}

// x += sy * y + sy2 * y2 (y, y2 optional);  out = tanh(alpha x) w + b (w optional).  n4 = T * W / 4.
template <typename TA>
__global__ void __launch_bounds__(256) add_dyt4_kernel(float* __restrict__ x, const float* __restrict__ y, float sy,
                                                       const float* __restrict__ y2, float sy2, float alpha,
                                                       const float* __restrict__ w, const float* __restrict__ b,
                                                       TA* __restrict__ out, size_t n4, int W) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (size_t)gridDim.x * 256) {
    const size_t e = i * 4;
    const int c = (int)(e % (size_t)W);
    f32x4 xv = *reinterpret_cast<const f32x4*>(x + e);
    if (y) {
      const f32x4 yv = *reinterpret_cast<const f32x4*>(y + e);
#pragma unroll
      for (int k = 0; k < 4; ++k) xv[k] = fmaf(sy, yv[k], xv[k]);
      if (y2) {
        const f32x4 zv = *reinterpret_cast<const f32x4*>(y2 + e);
#pragma unroll
        for (int k = 0; k < 4; ++k) xv[k] = fmaf(sy2, zv[k], xv[k]);
      }
      *reinterpret_cast<f32x4*>(x + e) = xv;
    }
    if (w) {
      const f32x4 wv = *reinterpret_cast<const f32x4*>(w + c), bv = *reinterpret_cast<const f32x4*>(b + c);
      float o[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) o[k] = fmaf(tanhf(alpha * xv[k]), wv[k], bv[k]);
      st4(out, e, o);
    }
  }
}

template <typename TA>
__global__ void __launch_bounds__(256) add_dyt1_kernel(float* __restrict__ x, const float* __restrict__ y, float sy,
                                                       const float* __restrict__ y2, float sy2, float alpha,
                                                       const float* __restrict__ w, const float* __restrict__ b,
                                                       TA* __restrict__ out, size_t n, int W) {
  for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < n; e += (size_t)gridDim.x * 256) {
    const int c = (int)(e % (size_t)W);
    float xv = x[e];
    if (y) {
      xv = fmaf(sy, y[e], xv);
      if (y2) xv = fmaf(sy2, y2[e], xv);
      x[e] = xv;
    }
    if (w) std_(out, e, fmaf(tanhf(alpha * xv), w[c], b[c]));
  }
}

// x = embed[id] * scale;  out = dyt(x) (w optional).  One workgroup per row.
template <typename TE, typename TA>
__global__ void __launch_bounds__(256) embed_scale_dyt_kernel(const int* __restrict__ ids, const TE* __restrict__ embed,
                                                              float scale, float* __restrict__ x, float alpha,
                                                              const float* __restrict__ w, const float* __restrict__ b,
                                                              TA* __restrict__ out, int W) {
  const size_t o = (size_t)blockIdx.x * W, src = (size_t)ids[blockIdx.x] * W;
  for (int c = threadIdx.x; c < W; c += 256) {
    const float xv = ldd(embed, src + c) * scale;
    x[o + c] = xv;
    if (w) std_(out, o + c, fmaf(tanhf(alpha * xv), w[c], b[c]));
  }
}

template <typename TA>
__global__ void __launch_bounds__(256) relu_sq_kernel(const TA* __restrict__ u, TA* __restrict__ out, size_t n) {
  for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < n; e += (size_t)gridDim.x * 256) {
    const float v = fmaxf(ldd(u, e), 0.f);
    std_(out, e, v * v);
  }
}

template <>
__global__ void __launch_bounds__(256) relu_sq_kernel<uint16_t>(const uint16_t* __restrict__ u,
                                                                uint16_t* __restrict__ out, size_t n) {
  const size_t n8 = n / 8;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += (size_t)gridDim.x * 256) {
    const u16x8 a = *reinterpret_cast<const u16x8*>(u + i * 8);
    u16x8 r;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float v = fmaxf(bf2f(a[k]), 0.f);
      r[k] = f2bf(v * v);
    }
    *reinterpret_cast<u16x8*>(out + i * 8) = r;
  }
  if (blockIdx.x == 0)
    for (size_t e = n8 * 8 + threadIdx.x; e < n; e += 256) {
      const float v = fmaxf(bf2f(u[e]), 0.f);
      out[e] = f2bf(v * v);
    }
}

static int grid_for(size_t items) {
  const size_t g = (items + 255) / 256;
  return (int)(g < 1 ? 1 : (g > 8192 ? 8192 : g));
}

}  // namespace k8s

using namespace k8s;

K8S_API int k8s_add_dyt(float* x, const float* y, float sy, const float* y2, float sy2, float alpha, const float* w,
                        const float* b, void* out, int odt, int T, int W, hipStream_t s) {
  if (T <= 0 || W <= 0) return 0;
  if ((w == nullptr) != (out == nullptr) || (w && !b) || (y2 && !y)) return (int)hipErrorInvalidValue;
  const size_t n = (size_t)T * W;
  if (W % 4 == 0) {
    if (odt == 0)
      hipLaunchKernelGGL((add_dyt4_kernel<uint16_t>), dim3(grid_for(n / 4)), dim3(256), 0, s, x, y, sy, y2, sy2, alpha, w,
                         b, (uint16_t*)out, n / 4, W);
    else
      hipLaunchKernelGGL((add_dyt4_kernel<float>), dim3(grid_for(n / 4)), dim3(256), 0, s, x, y, sy, y2, sy2, alpha, w, b,
                         (float*)out, n / 4, W);
  } else {
    if (odt == 0)
      hipLaunchKernelGGL((add_dyt1_kernel<uint16_t>), dim3(grid_for(n)), dim3(256), 0, s, x, y, sy, y2, sy2, alpha, w, b,
                         (uint16_t*)out, n, W);
    else
      hipLaunchKernelGGL((add_dyt1_kernel<float>), dim3(grid_for(n)), dim3(256), 0, s, x, y, sy, y2, sy2, alpha, w, b,
                         (float*)out, n, W);
  }
  return (int)hipGetLastError();
}

K8S_API int k8s_embed_scale_dyt(const int* ids, const void* embed, int edt, float scale, float* x, float alpha,
                                const float* w, const float* b, void* out, int odt, int T, int W, hipStream_t s) {
  if (T <= 0 || W <= 0) return 0;
  if ((w == nullptr) != (out == nullptr) || (w && !b)) return (int)hipErrorInvalidValue;
#define K8S_EMB(TE, TA)                                                                                         \
  hipLaunchKernelGGL((embed_scale_dyt_kernel<TE, TA>), dim3(T), dim3(256), 0, s, ids, (const TE*)embed, scale, x, \
                     alpha, w, b, (TA*)out, W)
  if (edt == 0 && odt == 0) {
    K8S_EMB(uint16_t, uint16_t);
  } else if (edt == 0) {
    K8S_EMB(uint16_t, float);
  } else if (odt == 0) {
    K8S_EMB(float, uint16_t);
  } else {
    K8S_EMB(float, float);
  }
#undef K8S_EMB
  return (int)hipGetLastError();
}

K8S_API int k8s_relu_sq(const void* u, void* out, long n, int dt, hipStream_t s) {
  if (n <= 0) return 0;
  if (dt == 0)
    hipLaunchKernelGGL((relu_sq_kernel<uint16_t>), dim3(grid_for((size_t)n / 8 + 1)), dim3(256), 0, s,
                       (const uint16_t*)u, (uint16_t*)out, (size_t)n);
  else
    hipLaunchKernelGGL((relu_sq_kernel<float>), dim3(grid_for((size_t)n)), dim3(256), 0, s, (const float*)u,
                       (float*)out, (size_t)n);
  return (int)hipGetLastError();
}
