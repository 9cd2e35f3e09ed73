// Layer norms around an fp32 residual stream, and the weighted sum over depth.
//
// One workgroup per row; the row is held in LDS (W floats) between the passes:
// mean, then the mean of the squared deviations (the variance exactly as it is
// defined, no E[x^2] - mean^2 cancellation), then the output.  Residual rows,
// sublayer outputs and all small parameters (weights, biases, coefficients) are
// fp32; TA is the activation type written for the next GEMM (bf16 as uint16_t,
// or float).
#include "common.h"

namespace k8s {

template <typename T>
__device__ __forceinline__ float ldn(const T* p, size_t i);
template <>
__device__ __forceinline__ float ldn<float>(const float* p, size_t i) { return p[i]; }
template <>
__device__ __forceinline__ float ldn<uint16_t>(const uint16_t* p, size_t i) { return bf2f(p[i]); }
template <typename T>
__device__ __forceinline__ void stn(T* p, size_t i, float v);
template <>
__device__ __forceinline__ void stn<float>(float* p, size_t i, float v) { p[i] = v; }
template <>
__device__ __forceinline__ void stn<uint16_t>(uint16_t* p, size_t i, float v) { p[i] = f2bf(v); }

// mean and 1 / sqrt(var + eps) of the LDS row (all threads get both)
__device__ __forceinline__ void row_stats(const float* row, int W, float eps, float* red, float& mean, float& rstd) {
  float s = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) s += row[c];
  mean = block_sum(s, red) / (float)W;
  float q = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float d = row[c] - mean;
    q = fmaf(d, d, q);
  }
  rstd = 1.f / sqrtf(block_sum(q, red) / (float)W + eps);
}

// 1 / sqrt(mean(v^2) + eps) of a global fp32 row
__device__ __forceinline__ float row_rrms(const float* v, int W, float eps, float* red) {
  float q = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) q = fmaf(v[c], v[c], q);
  return 1.f / sqrtf(block_sum(q, red) / (float)W + eps);
}

template <typename TA>
__global__ void __launch_bounds__(1024) layernorm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                        const float* __restrict__ b, TA* __restrict__ out, int W,
                                                        float eps) {
  extern __shared__ float row[];
  __shared__ float red[16];
  const size_t o = (size_t)blockIdx.x * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) row[c] = x[o + c];
  __syncthreads();
  float mean, rstd;
  row_stats(row, W, eps, red, mean, rstd);
  for (int c = threadIdx.x; c < W; c += blockDim.x) stn(out, o + c, (row[c] - mean) * rstd * w[c] + b[c]);
}

// x_out = LN(embed[id]; w, b); optionally h = LN(x_out; nw, nb).
template <typename TE, typename TA>
__global__ void __launch_bounds__(1024) embed_ln_kernel(const int* __restrict__ ids, const TE* __restrict__ embed,
                                                       const float* __restrict__ w, const float* __restrict__ b,
                                                       float* __restrict__ x_out, const float* __restrict__ nw,
                                                       const float* __restrict__ nb, TA* __restrict__ h, int W,
                                                       float eps) {
  extern __shared__ float row[];
  __shared__ float red[16];
  const size_t o = (size_t)blockIdx.x * W, e0 = (size_t)ids[blockIdx.x] * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) row[c] = ldn(embed, e0 + c);
  __syncthreads();
  float mean, rstd;
  row_stats(row, W, eps, red, mean, rstd);
  __syncthreads();
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float v = (row[c] - mean) * rstd * w[c] + b[c];
    row[c] = v;
    x_out[o + c] = v;
  }
  if (nw == nullptr) return;
  __syncthreads();
  row_stats(row, W, eps, red, mean, rstd);
  for (int c = threadIdx.x; c < W; c += blockDim.x) stn(h, o + c, (row[c] - mean) * rstd * nw[c] + nb[c]);
}

// dst = src + LN(u; w, b); u = y (mode 0), (unit_rms(y) wl + unit_rms(y2) wr) / 2 (mode 1), y + y2 (mode 2),
// y + sigmoid(rg[row]) y2 (mode 3: rg holds one gate logit per row, row stride rgs).
// kind 1: an RMS norm instead, u / sqrt(mean(u^2) + eps) * w (no mean, b may be null).
// Optionally h = LN(dst; nw, nb); with h but without nw, h = dst as activations (the next sublayer reads the
// residual itself).
template <typename TA>
__global__ void __launch_bounds__(1024) ln_residual_kernel(const float* src, const float* __restrict__ y,
                                                          const float* __restrict__ y2, int mode,
                                                          const float* __restrict__ wl, const float* __restrict__ wr,
                                                          const float* __restrict__ w, const float* __restrict__ b,
                                                          float* dst, const float* __restrict__ nw,
                                                          const float* __restrict__ nb, TA* __restrict__ h, int W,
                                                          float eps, int kind, const float* __restrict__ rg, int rgs) {
  extern __shared__ float row[];
  __shared__ float red[16];
  const size_t o = (size_t)blockIdx.x * W;
  if (mode == 3) {
    const float gt = 1.f / (1.f + expf(-rg[(size_t)blockIdx.x * rgs]));
    for (int c = threadIdx.x; c < W; c += blockDim.x) row[c] = fmaf(gt, y2[o + c], y[o + c]);
  } else
  if (mode == 1) {
    const float ra = row_rrms(y + o, W, eps, red), rb = row_rrms(y2 + o, W, eps, red);
    for (int c = threadIdx.x; c < W; c += blockDim.x) row[c] = 0.5f * (y[o + c] * ra * wl[c] + y2[o + c] * rb * wr[c]);
  } else if (mode == 2) {
    for (int c = threadIdx.x; c < W; c += blockDim.x) row[c] = y[o + c] + y2[o + c];
  } else {
    for (int c = threadIdx.x; c < W; c += blockDim.x) row[c] = y[o + c];
  }
  __syncthreads();
  float mean, rstd;
  if (kind == 1) {
    mean = 0.f;
    rstd = row_rrms(row, W, eps, red);
  } else {
    row_stats(row, W, eps, red, mean, rstd);
  }
  __syncthreads();
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float v = src[o + c] + ((row[c] - mean) * rstd * w[c] + (b ? b[c] : 0.f));
    row[c] = v;
    dst[o + c] = v;
    if (h != nullptr && nw == nullptr) stn(h, o + c, v);
  }
  if (nw == nullptr) return;
  __syncthreads();
  row_stats(row, W, eps, red, mean, rstd);
  for (int c = threadIdx.x; c < W; c += blockDim.x) stn(h, o + c, (row[c] - mean) * rstd * nw[c] + nb[c]);
}

// a = sum_{j < n} coef[j] * stack[j][row]; h = LN(a; w, b).  stack: [n][T][W]; rows: optional gather.
template <typename TA>
__global__ void __launch_bounds__(1024) depth_mix_ln_kernel(const float* __restrict__ stack, size_t plane, int n,
                                                           const float* __restrict__ coef,
                                                           const int* __restrict__ rows, float* __restrict__ a_out,
                                                           const float* __restrict__ w, const float* __restrict__ b,
                                                           TA* __restrict__ h, int W, float eps) {
  extern __shared__ float row[];
  __shared__ float red[16];
  const size_t r = rows ? (size_t)rows[blockIdx.x] : (size_t)blockIdx.x;
  const size_t o = (size_t)blockIdx.x * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float a = 0.f;
    for (int j = 0; j < n; ++j) a = fmaf(coef[j], stack[(size_t)j * plane + r * W + c], a);
    row[c] = a;
    a_out[o + c] = a;
  }
  __syncthreads();
  float mean, rstd;
  row_stats(row, W, eps, red, mean, rstd);
  for (int c = threadIdx.x; c < W; c += blockDim.x) stn(h, o + c, (row[c] - mean) * rstd * w[c] + b[c]);
}

// x_out[r] = embed[ids[r]] (fp32) and h[r] the same as activations (h optional): 256 threads walk the row.
template <typename TE, typename TA>
__global__ void __launch_bounds__(256) embed_rows_kernel(const int* __restrict__ ids, const TE* __restrict__ embed,
                                                        float* __restrict__ x_out, TA* __restrict__ h, int W) {
  const size_t o = (size_t)blockIdx.x * W, e0 = (size_t)ids[blockIdx.x] * W;
  for (int c = threadIdx.x; c < W; c += 256) {
    const float v = ldn(embed, e0 + c);
    x_out[o + c] = v;
    if (h) stn(h, o + c, v);
  }
}

// Per-token input of a layer: out[r][j] = gelu_tanh(a[r][j]) * table[ids[r]][col0 + j], j < n, where
// gelu_tanh(z) = z / 2 (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3))).  a [T][n] fp32; table rows have tw entries.
template <typename TE, typename TA>
__global__ void __launch_bounds__(256) token_gate_kernel(const float* __restrict__ a, const int* __restrict__ ids,
                                                        const TE* __restrict__ table, int tw, int col0,
                                                        TA* __restrict__ out, int T, int n) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (size_t)T * n) return;
  const int r = (int)(i / n), j = (int)(i - (size_t)r * n);
  const float zv = a[i];
  const float g = 0.5f * zv * (1.f + tanhf(0.7978845608028654f * (zv + 0.044715f * zv * zv * zv)));
  stn(out, i, g * ldn(table, (size_t)ids[r] * tw + col0 + j));
}

__global__ void __launch_bounds__(256) softcap_kernel(float* __restrict__ z, size_t n, float scale, float cap) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const float v = z[i] * scale;
  z[i] = cap > 0.f ? cap * tanhf(v / cap) : v;
}

}  // namespace k8s

using namespace k8s;

#define K8S_ODT(dt, ...)   \
  if ((dt) == 0) {          \
    using TA = uint16_t;    \
    __VA_ARGS__;            \
  } else {                  \
    using TA = float;       \
    __VA_ARGS__;            \
  }

static inline bool row_fits(int W) { return W > 0 && (size_t)W * sizeof(float) <= 64 * 1024; }
// threads per row: few rows (decoding) leave most of the chip idle, so each row gets a wider workgroup
static inline int row_threads(int rows, int W) { return rows <= 256 && W >= 1024 ? 1024 : 256; }

K8S_API int k8s_layernorm(const float* x, const float* w, const float* b, void* out, int T, int W, float eps, int dt,
                          hipStream_t s) {
  if (T <= 0) return 0;
  if (!row_fits(W)) return (int)hipErrorInvalidValue;
  K8S_ODT(dt, hipLaunchKernelGGL((layernorm_kernel<TA>), dim3(T), dim3(row_threads(T, W)), W * sizeof(float), s, x, w, b, (TA*)out,
                                 W, eps));
  return (int)hipGetLastError();
}

K8S_API int k8s_embed_ln(const int* ids, const void* embed, int edt, const float* w, const float* b, float* x_out,
                         const float* nw, const float* nb, void* h, int dt, int T, int W, float eps, hipStream_t s) {
  if (T <= 0) return 0;
  if (!row_fits(W)) return (int)hipErrorInvalidValue;
  if (edt == 0) {
    K8S_ODT(dt, hipLaunchKernelGGL((embed_ln_kernel<uint16_t, TA>), dim3(T), dim3(row_threads(T, W)), W * sizeof(float), s, ids,
                                   (const uint16_t*)embed, w, b, x_out, nw, nb, (TA*)h, W, eps));
  } else {
    K8S_ODT(dt, hipLaunchKernelGGL((embed_ln_kernel<float, TA>), dim3(T), dim3(row_threads(T, W)), W * sizeof(float), s, ids,
                                   (const float*)embed, w, b, x_out, nw, nb, (TA*)h, W, eps));
  }
  return (int)hipGetLastError();
}

K8S_API int k8s_ln_residual(const float* src, const float* y, const float* y2, int mode, const float* wl,
                            const float* wr, const float* w, const float* b, float* dst, const float* nw,
                            const float* nb, void* h, int dt, int T, int W, float eps, hipStream_t s, int kind,
                            const float* rg, int rgs) {
  if (T <= 0) return 0;
  if (!row_fits(W) || (mode != 0 && y2 == nullptr) || (mode == 1 && (!wl || !wr)) || (mode == 3 && !rg) ||
      (kind == 0 && !b))
    return (int)hipErrorInvalidValue;
  K8S_ODT(dt, hipLaunchKernelGGL((ln_residual_kernel<TA>), dim3(T), dim3(row_threads(T, W)), W * sizeof(float), s, src, y, y2, mode,
                                 wl, wr, w, b, dst, nw, nb, (TA*)h, W, eps, kind, rg, rgs));
  return (int)hipGetLastError();
}

K8S_API int k8s_embed_rows(const int* ids, const void* embed, int edt, float* x_out, void* h, int dt, int T, int W,
                           hipStream_t s) {
  if (T <= 0) return 0;
  if (edt == 0) {
    K8S_ODT(dt, hipLaunchKernelGGL((embed_rows_kernel<uint16_t, TA>), dim3(T), dim3(256), 0, s, ids,
                                   (const uint16_t*)embed, x_out, (TA*)h, W));
  } else {
    K8S_ODT(dt, hipLaunchKernelGGL((embed_rows_kernel<float, TA>), dim3(T), dim3(256), 0, s, ids, (const float*)embed,
                                   x_out, (TA*)h, W));
  }
  return (int)hipGetLastError();
}

K8S_API int k8s_token_gate(const float* a, const int* ids, const void* table, int edt, int tw, int col0, void* out,
                           int dt, int T, int n, hipStream_t s) {
  if (T <= 0 || n <= 0) return 0;
  if (col0 < 0 || col0 + n > tw) return (int)hipErrorInvalidValue;
  const unsigned blocks = (unsigned)(((size_t)T * n + 255) / 256);
  if (edt == 0) {
    K8S_ODT(dt, hipLaunchKernelGGL((token_gate_kernel<uint16_t, TA>), dim3(blocks), dim3(256), 0, s, a, ids,
                                   (const uint16_t*)table, tw, col0, (TA*)out, T, n));
  } else {
    K8S_ODT(dt, hipLaunchKernelGGL((token_gate_kernel<float, TA>), dim3(blocks), dim3(256), 0, s, a, ids,
                                   (const float*)table, tw, col0, (TA*)out, T, n));
  }
  return (int)hipGetLastError();
}

K8S_API int k8s_depth_mix_ln(const float* stack, int T, int n, const float* coef, const int* rows, int R,
                             float* a_out, const float* w, const float* b, void* h, int dt, int W, float eps,
                             hipStream_t s) {
  if (R <= 0) return 0;
  if (!row_fits(W) || n < 1) return (int)hipErrorInvalidValue;
  K8S_ODT(dt, hipLaunchKernelGGL((depth_mix_ln_kernel<TA>), dim3(R), dim3(row_threads(R, W)), W * sizeof(float), s, stack,
                                 (size_t)T * W, n, coef, rows, a_out, w, b, (TA*)h, W, eps));
  return (int)hipGetLastError();
}

K8S_API int k8s_softcap(float* z, long n, float scale, float cap, hipStream_t s) {
  if (n <= 0) return 0;
  hipLaunchKernelGGL(softcap_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, z, (size_t)n, scale, cap);
  return (int)hipGetLastError();
}
