// Feed-forward pieces beside the SwiGLU / softmax-router ones of norm_act.hip and
// moe.hip: the PolyNorm activation, a gated unit with clamps, a router that
// scores with a sigmoid (or a softmax) straight from the hidden row in fp32, the
// scaled gather into expert order, the combine into an fp32 row, and a grouped
// GEMM for any shape and for fp32.
// TA (activations) and TW (weights) are bf16 (uint16_t) or float.
#include "common.h"

namespace k8s {

template <typename T>
__device__ __forceinline__ float ldx(const T* p, size_t i);
template <>
__device__ __forceinline__ float ldx<float>(const float* p, size_t i) { return p[i]; }
template <>
__device__ __forceinline__ float ldx<uint16_t>(const uint16_t* p, size_t i) { return bf2f(p[i]); }
template <typename T>
__device__ __forceinline__ void stx(T* p, size_t i, float v);
template <>
__device__ __forceinline__ void stx<float>(float* p, size_t i, float v) { p[i] = v; }
template <>
__device__ __forceinline__ void stx<uint16_t>(uint16_t* p, size_t i, float v) { p[i] = f2bf(v); }

// eight consecutive elements (the index a multiple of 8): one 16-byte load for bf16, two for fp32
__device__ __forceinline__ void ld8(const uint16_t* p, size_t i, float (&v)[8]) {
  const u16x8 raw = *reinterpret_cast<const u16x8*>(p + i);
#pragma unroll
  for (int k = 0; k < 8; ++k) v[k] = bf2f(raw[k]);
}
__device__ __forceinline__ void ld8(const float* p, size_t i, float (&v)[8]) {
  const f32x4 a = *reinterpret_cast<const f32x4*>(p + i), b = *reinterpret_cast<const f32x4*>(p + i + 4);
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    v[k] = a[k];
    v[4 + k] = b[k];
  }
}

// PolyNorm: out = a N(z) + b N(z^2) + c N(z^3) + e, N(v) = v / sqrt(mean(v^2) + eps)
// over the row; z fp32 [T][F], coef = (a, b, c, e).
template <typename TW, typename TA>
__global__ void __launch_bounds__(256) polynorm_kernel(const float* __restrict__ z, const TW* __restrict__ coef,
                                                       TA* __restrict__ out, int F, float eps) {
  __shared__ float scratch[16];
  const size_t o = (size_t)blockIdx.x * F;
  float s1 = 0.f, s2 = 0.f, s3 = 0.f;
  for (int c = threadIdx.x; c < F; c += 256) {
    const float v = z[o + c], v2 = v * v;
    s1 += v2;
    s2 = fmaf(v2, v2, s2);
    s3 = fmaf(v2 * v2, v2, s3);
  }
  s1 = block_sum(s1, scratch);
  s2 = block_sum(s2, scratch);
  s3 = block_sum(s3, scratch);
  const float i1 = 1.f / sqrtf(s1 / (float)F + eps), i2 = 1.f / sqrtf(s2 / (float)F + eps),
              i3 = 1.f / sqrtf(s3 / (float)F + eps);
  const float a = ldx(coef, 0) * i1, b = ldx(coef, 1) * i2, cc = ldx(coef, 2) * i3, e = ldx(coef, 3);
  for (int c = threadIdx.x; c < F; c += 256) {
    const float v = z[o + c], v2 = v * v;
    stx(out, o + c, a * v + b * v2 + cc * v2 * v + e);
  }
}

// Gated unit with clamps: gu [rows][2F] = (gate | up); g = min(gate, limit),
// u = clamp(up, -limit, limit); out = g * sigmoid(alpha g) * (u + up_shift).
template <typename TA>
__global__ void __launch_bounds__(256) glu_clamp_kernel(const TA* __restrict__ gu, TA* __restrict__ out, size_t n,
                                                        int F, float alpha, float limit, float up_shift) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const size_t r = i / F, c = i - r * F;
  const float g = fminf(ldx(gu, r * 2 * F + c), limit);
  const float u = fminf(fmaxf(ldx(gu, r * 2 * F + F + c), -limit), limit);
  stx(out, i, g / (1.f + expf(-alpha * g)) * (u + up_shift));
}

__device__ __forceinline__ void st8(uint16_t* p, size_t i, const float (&v)[8]) {
  u16x8 raw;
#pragma unroll
  for (int k = 0; k < 8; ++k) raw[k] = f2bf(v[k]);
  *reinterpret_cast<u16x8*>(p + i) = raw;
}
__device__ __forceinline__ void st8(float* p, size_t i, const float (&v)[8]) {
  *reinterpret_cast<f32x4*>(p + i) = f32x4{v[0], v[1], v[2], v[3]};
  *reinterpret_cast<f32x4*>(p + i + 4) = f32x4{v[4], v[5], v[6], v[7]};
}

// The same for F a multiple of 8: eight neighbouring outputs per thread, 16-byte accesses.
template <typename TA>
__global__ void __launch_bounds__(256) glu_clamp8_kernel(const TA* __restrict__ gu, TA* __restrict__ out, size_t n8,
                                                         int F, float alpha, float limit, float up_shift) {
  const size_t i8 = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i8 >= n8) return;
  const size_t i = i8 * 8, r = i / F, c = i - r * F;
  float gv[8], uv[8], o[8];
  ld8(gu, r * 2 * F + c, gv);
  ld8(gu, r * 2 * F + F + c, uv);
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const float g = fminf(gv[k], limit), u = fminf(fmaxf(uv[k], -limit), limit);
    o[k] = g / (1.f + expf(-alpha * g)) * (u + up_shift);
  }
  st8(out, i, o);
}

// Router: one wave per token.  logits = Wr h in fp32; scores = sigmoid(logits)
// (mode 0) or softmax (mode 1); the K largest (ties: lowest index), optionally
// renormalised to sum 1 (divided by their sum + renorm_eps).  With `bias` [E] the
// choice is made on score + bias while the weights stay the plain scores.  The weights are multiplied by
// out_scale at the end.  wr may hold X more rows behind the E experts' (Et = E + X): their logits are not
// routed but written as they are to extra[t][X] (per-token gates that read the same hidden row).
template <typename TA, typename TW>
__global__ void __launch_bounds__(256) router_kernel(const TA* __restrict__ h, const TW* __restrict__ wr, int T, int W,
                                                     int Et, int K, int mode, int renorm, float* __restrict__ w_out,
                                                     int* __restrict__ id_out, const float* __restrict__ bias,
                                                     float renorm_eps, int X, float* __restrict__ extra,
                                                     float out_scale) {
  extern __shared__ float sm[];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int t = blockIdx.x * 4 + wv;
  if (t >= T) return;
  float* sc = sm + wv * 2 * Et;
  float* ch = sc + Et;   // choice scores
  const int E = Et;      // rows whose logits are formed below; the routed ones are E - X
  if ((W & 7) == 0) {
    // 8 columns per lane and step, 16 experts at a time: the hidden row is read once per group
    for (int e0 = 0; e0 < E; e0 += 16) {
      float acc[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) acc[j] = 0.f;
      for (int c = lane * 8; c < W; c += 512) {
        float hv[8];
        ld8(h, (size_t)t * W + c, hv);
#pragma unroll
        for (int j = 0; j < 16; ++j)
          if (e0 + j < E) {
            float wv8[8];
            ld8(wr, (size_t)(e0 + j) * W + c, wv8);
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[j] = fmaf(hv[i], wv8[i], acc[j]);
          }
      }
#pragma unroll
      for (int j = 0; j < 16; ++j)
        if (e0 + j < E) {
          const float a = wave_sum(acc[j]);
          if (lane == 0) sc[e0 + j] = a;
        }
    }
  } else {
    for (int e = 0; e < E; ++e) {
      float a = 0.f;
      for (int c = lane; c < W; c += 64) a = fmaf(ldx(h, (size_t)t * W + c), ldx(wr, (size_t)e * W + c), a);
      a = wave_sum(a);
      if (lane == 0) sc[e] = a;
    }
  }
  __builtin_amdgcn_wave_barrier();
  if (lane == 0) {
    const int E = Et - X;
    for (int x = 0; x < X; ++x) extra[(size_t)t * X + x] = sc[E + x];
    if (mode == 0) {
      for (int e = 0; e < E; ++e) sc[e] = 1.f / (1.f + expf(-sc[e]));
    } else {
      float m = -INFINITY, s = 0.f;
      for (int e = 0; e < E; ++e) m = fmaxf(m, sc[e]);
      for (int e = 0; e < E; ++e) s += (sc[e] = expf(sc[e] - m));
      for (int e = 0; e < E; ++e) sc[e] /= s;
    }
    for (int e = 0; e < E; ++e) ch[e] = bias ? sc[e] + bias[e] : sc[e];
    float tot = 0.f;
    for (int k = 0; k < K; ++k) {
      int bi = 0;
      float bv = -INFINITY;
      for (int e = 0; e < E; ++e)
        if (ch[e] > bv) {
          bv = ch[e];
          bi = e;
        }
      w_out[t * K + k] = sc[bi];
      id_out[t * K + k] = bi;
      tot += sc[bi];
      ch[bi] = -INFINITY;
    }
    if (renorm)
      for (int k = 0; k < K; ++k) w_out[t * K + k] /= (tot + renorm_eps);
    if (out_scale != 1.f)
      for (int k = 0; k < K; ++k) w_out[t * K + k] *= out_scale;
  }
}

// xp[i] = (w ? w[order[i]] : 1) * h[order[i] / K]: rows in expert order, scaled
// by their routing weight when the weight multiplies the expert's input.
template <typename TA>
__global__ void __launch_bounds__(256) moe_gather_kernel(const TA* __restrict__ h, const int* __restrict__ order,
                                                         const float* __restrict__ w, TA* __restrict__ xp, int W,
                                                         int K) {
  const int i = blockIdx.x, slot = order[i];
  const float s = w ? w[slot] : 1.f;
  const size_t src = (size_t)(slot / K) * W, dst = (size_t)i * W;
  for (int c = threadIdx.x; c < W; c += 256) stx(xp, dst + c, s * ldx(h, src + c));
}

// out[t] = sum_k (w ? w[t][k] : 1) * y[inv[t K + k]] as an fp32 row.
template <typename TA>
__global__ void __launch_bounds__(256) moe_combine_f32_kernel(const TA* __restrict__ y, const int* __restrict__ inv,
                                                              const float* __restrict__ w, float* __restrict__ out,
                                                              int W, int K) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < W; c += 256) {
    float a = 0.f;
    for (int k = 0; k < K; ++k) a = fmaf(w ? w[t * K + k] : 1.f, ldx(y, (size_t)inv[t * K + k] * W + c), a);
    out[(size_t)t * W + c] = a;
  }
}

// Grouped GEMM of any shape: rows offsets[e] .. offsets[e + 1] of a [rows][K]
// times w[e]^T ([E][N][K]) -> out [rows][N].  64 x 64 tiles, 256 threads of
// 4 x 4 outputs, fp32 accumulation on the vector pipes.  Tiles are numbered over
// the experts on the device (no host read of the offsets).
template <typename TA, typename TW>
__global__ void __launch_bounds__(256) grouped_any_kernel(const TA* __restrict__ a, const TW* __restrict__ w,
                                                          const int* __restrict__ offsets, TA* __restrict__ out,
                                                          int E, int N, int K) {
  __shared__ float As[16][65];
  __shared__ float Ws[16][65];
  int tile = blockIdx.x, e = 0, lo = 0, hi = 0;
  for (; e < E; ++e) {
    lo = offsets[e];
    hi = offsets[e + 1];
    const int nt = (hi - lo + 63) >> 6;
    if (tile < nt) break;
    tile -= nt;
  }
  if (e >= E) return;
  const int m0 = lo + tile * 64, n0 = blockIdx.y * 64;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const TW* we = w + (size_t)e * N * K;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += 16) {
    for (int i = threadIdx.x; i < 64 * 16; i += 256) {
      const int rr = i >> 4, kk = i & 15;
      const int m = m0 + rr, n = n0 + rr, k = k0 + kk;
      As[kk][rr] = (m < hi && k < K) ? ldx(a, (size_t)m * K + k) : 0.f;
      Ws[kk][rr] = (n < N && k < K) ? ldx(we, (size_t)n * K + k) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        av[i] = As[kk][ty * 4 + i];
        wv[i] = Ws[kk][tx * 4 + i];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= hi) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) stx(out, (size_t)m * N + n, acc[i][j]);
    }
  }
}

}  // namespace k8s

using namespace k8s;

#define K8S_DT(dt, ...)     \
  if ((dt) == 0) {           \
    using TW = uint16_t;     \
    using TA = uint16_t;     \
    __VA_ARGS__;                    \
  } else {                   \
    using TW = float;        \
    using TA = float;        \
    __VA_ARGS__;                    \
  }

K8S_API int k8s_polynorm(const float* z, const void* coef, void* out, int T, int F, float eps, int dt,
                         hipStream_t s) {
  if (T <= 0) return 0;
  K8S_DT(dt, hipLaunchKernelGGL((polynorm_kernel<TW, TA>), dim3(T), dim3(256), 0, s, z, (const TW*)coef, (TA*)out, F,
                                 eps));
  return (int)hipGetLastError();
}

K8S_API int k8s_glu_clamp(const void* gu, void* out, int rows, int F, float alpha, float limit, float up_shift,
                          int dt, hipStream_t s) {
  const size_t n = (size_t)rows * F;
  if (n == 0) return 0;
  if (F % 8 == 0 && ((uintptr_t)gu & 15) == 0 && ((uintptr_t)out & 15) == 0) {
    const size_t n8 = n / 8;
    K8S_DT(dt, hipLaunchKernelGGL((glu_clamp8_kernel<TA>), dim3((unsigned)((n8 + 255) / 256)), dim3(256), 0, s,
                                   (const TA*)gu, (TA*)out, n8, F, alpha, limit, up_shift));
    return (int)hipGetLastError();
  }
  K8S_DT(dt, hipLaunchKernelGGL((glu_clamp_kernel<TA>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s,
                                 (const TA*)gu, (TA*)out, n, F, alpha, limit, up_shift));
  return (int)hipGetLastError();
}

K8S_API int k8s_router(const void* h, const void* wr, int T, int W, int E, int K, int mode, int renorm, float* w_out,
                       int* id_out, int dt, hipStream_t s, const float* bias, float renorm_eps, int X, float* extra,
                       float out_scale) {
  if (T <= 0) return 0;
  if (K > E || E + X > 2048 || X < 0 || (X > 0 && !extra)) return (int)hipErrorInvalidValue;
  K8S_DT(dt, hipLaunchKernelGGL((router_kernel<TA, TW>), dim3((T + 3) / 4), dim3(256), 8 * (E + X) * sizeof(float), s,
                                 (const TA*)h, (const TW*)wr, T, W, E + X, K, mode, renorm, w_out, id_out, bias,
                                 renorm_eps, X, extra, out_scale));
  return (int)hipGetLastError();
}

K8S_API int k8s_moe_gather(const void* h, const int* order, const float* w, void* xp, int rows, int W, int K, int dt,
                           hipStream_t s) {
  if (rows <= 0) return 0;
  K8S_DT(dt, hipLaunchKernelGGL((moe_gather_kernel<TA>), dim3(rows), dim3(256), 0, s, (const TA*)h, order, w,
                                 (TA*)xp, W, K));
  return (int)hipGetLastError();
}

K8S_API int k8s_moe_combine_f32(const void* y, const int* inv, const float* w, float* out, int T, int W, int K,
                                int dt, hipStream_t s) {
  if (T <= 0) return 0;
  K8S_DT(dt, hipLaunchKernelGGL((moe_combine_f32_kernel<TA>), dim3(T), dim3(256), 0, s, (const TA*)y, inv, w, out,
                                 W, K));
  return (int)hipGetLastError();
}

K8S_API int k8s_grouped_any(const void* a, const void* w, const int* offsets, void* out, int rows, int E, int N,
                            int K, int dt, hipStream_t s) {
  if (rows <= 0) return 0;
  const int max_tiles = (rows + 63) / 64 + E;
  K8S_DT(dt, hipLaunchKernelGGL((grouped_any_kernel<TA, TW>), dim3(max_tiles, (N + 63) / 64), dim3(256), 0, s,
                                 (const TA*)a, (const TW*)w, offsets, (TA*)out, E, N, K));
  return (int)hipGetLastError();
}
