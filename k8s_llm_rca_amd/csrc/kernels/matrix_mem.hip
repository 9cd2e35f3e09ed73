// Recurrences whose per-head state is a D x V matrix, over segments (seg_row0 / seg_pos0 / seg_slot as in
// mixer_ops.hip; a slot's state is read only when the segment does not start at position 0):
//
//   gated delta rule   S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
//                      with one decay per head and key channel, g = exp(-rate_h softplus(a + dt_bias)),
//                      q and k made unit vectors (q also times D^(-1/2)), grouped q / k heads;
//   matrix memory      m' = max(f + m, i);  S <- e^(f + m - m') S + e^(i - m') k v^T;  n likewise with k alone;
//                      o = S^T q / (max(|n.q|, e^(-m')) + den_eps), with soft-capped log gates i, f.
//
// Everything is fp32.  One workgroup of 256 threads owns 64 value columns of one (segment, head): thread
// (dg = tid & 3, v = tid >> 2) holds S[d][v] for the DPT consecutive d from dg * DPT in registers, so the two
// sums over d per token (S^T k and S^T q) are DPT multiply-adds per thread and two cross-lane exchanges among
// four neighbouring lanes -- no barrier inside a token.  Tokens pass through LDS in batches of 16 (q, k,
// decays, values and the per-token scalars), one barrier pair per batch.
// The matrix memory's gates, maximum and normaliser do not depend on the value columns: a kernel of their
// own (one wave per segment and head) runs that scalar / vector recurrence first and leaves per token the
// two factors and the output multiplier, so the matrix kernel's workgroups share no state.
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

__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }
__device__ __forceinline__ float sigmoid_f(float x) { return 1.f / (1.f + expf(-x)); }
__device__ __forceinline__ float logsigmoid_f(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

constexpr int kMemTb = 16;     // tokens per batch
constexpr int kMemVb = 64;     // value columns per workgroup
constexpr int kGatePer = 8;    // key channels per lane of the gate kernel: D <= 512

// Rows of x (fp32, stride xs): q [H][D] | k [H][D] | v [H][V] | gate [H][V] | i [H] | f [H].
// ab [T][H][3] receives (forget factor, input factor, D^(-1/2) / denominator) of every token.
__global__ void __launch_bounds__(256) memory_gates_kernel(const float* __restrict__ x, int xs,
                                                           const float* __restrict__ gate_bias, float cap,
                                                           float* __restrict__ nstate, float* __restrict__ mstate,
                                                           const int* __restrict__ seg_row0,
                                                           const int* __restrict__ seg_pos0,
                                                           const int* __restrict__ seg_slot, float* __restrict__ ab,
                                                           int n_seg, int H, int D, int V, float den_eps) {
  const int unit = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (unit >= n_seg * H) return;
  const int sg = unit / H, hh = unit - sg * H;
  const int r0 = seg_row0[sg], r1 = seg_row0[sg + 1];
  const bool fresh = seg_pos0[sg] == 0;
  const size_t so = (size_t)seg_slot[sg] * H + hh;
  float n[kGatePer];
#pragma unroll
  for (int i = 0; i < kGatePer; ++i) {
    const int d = lane + 64 * i;
    n[i] = (!fresh && d < D) ? nstate[so * D + d] : 0.f;
  }
  float m = fresh ? 0.f : mstate[so];
  const int HD = H * D, go = 2 * HD + 2 * H * V;
  const float bi = gate_bias[hh], bf = gate_bias[H + hh], qs = 1.f / sqrtf((float)D);
  for (int r = r0; r < r1; ++r) {
    const float* row = x + (size_t)r * xs;
    const float gi = cap * tanhf((row[go + hh] + bi) / cap);
    const float gf = logsigmoid_f(cap * tanhf((row[go + H + hh] + bf) / cap));
    const float mn = fmaxf(gf + m, gi);
    const float fa = expf(gf + m - mn), ia = expf(gi - mn);
    float dot = 0.f;
#pragma unroll
    for (int i = 0; i < kGatePer; ++i) {
      const int d = lane + 64 * i;
      if (d < D) {
        n[i] = fmaf(fa, n[i], ia * row[HD + hh * D + d]);
        dot = fmaf(n[i], row[hh * D + d] * qs, dot);
      }
    }
    dot = wave_sum(dot);
    m = mn;
    if (lane == 0) {
      float* o = ab + ((size_t)r * H + hh) * 3;
      o[0] = fa;
      o[1] = ia;
      o[2] = qs / (fmaxf(fabsf(dot), expf(-mn)) + den_eps);
    }
  }
#pragma unroll
  for (int i = 0; i < kGatePer; ++i) {
    const int d = lane + 64 * i;
    if (d < D) nstate[so * D + d] = n[i];
  }
  if (lane == 0) mstate[so] = m;
}

// KIND 0: gated delta rule.  qkv rows (TA, contiguous, width 2 G D + H V): q [G][D] | k [G][D] | v [H][V];
//         a [T][H D] fp32 (before bias and softplus); beta [T] rows of stride bs, column hh (before the sigmoid).
// KIND 1: matrix memory.  x rows (fp32, stride xs) as in memory_gates_kernel; ab from that kernel.
struct MatArgs {
  const void* x;
  int xs;
  const float* a;
  const float* rate;
  const float* dt_bias;
  const float* beta;
  int bs;
  const float* ab;
  float* state;
  const int* seg_row0;
  const int* seg_pos0;
  const int* seg_slot;
  float* out;          // [T][H V] fp32
  int H, G, D, V;
  float unit_eps;
};

template <int DPT, int KIND, typename TA>
__global__ void __launch_bounds__(256) matrix_state_kernel(MatArgs p) {
  extern __shared__ float sm[];
  const int sg = blockIdx.x, hh = blockIdx.y, v0 = blockIdx.z * kMemVb, tid = threadIdx.x;
  const int H = p.H, D = p.D, V = p.V;
  float* sq = sm;                                  // [TB][D]
  float* sk = sq + kMemTb * D;                     // [TB][D]
  float* sgd = sk + kMemTb * D;                    // [TB][D] decays (KIND 0)
  float* sv = sgd + (KIND == 0 ? kMemTb * D : 0);  // [TB][64]
  float* sc = sv + kMemTb * kMemVb;                // [TB][4] per-token scalars
  const int dg = tid & 3, vl = tid >> 2, lane = tid & 63, wv = tid >> 6;
  const bool vown = v0 + vl < V;
  const int r0 = p.seg_row0[sg], r1 = p.seg_row0[sg + 1];
  const bool fresh = p.seg_pos0[sg] == 0;
  float* st = p.state + ((size_t)p.seg_slot[sg] * H + hh) * D * V + v0 + vl;
  float S[DPT];
#pragma unroll
  for (int i = 0; i < DPT; ++i) {
    const int d = dg * DPT + i;
    S[i] = (vown && d < D && !fresh) ? st[(size_t)d * V] : 0.f;
  }
  const int kvh = hh / (H / p.G);
  const float rate = KIND == 0 ? p.rate[hh] : 0.f;
  for (int t0 = r0; t0 < r1; t0 += kMemTb) {
    const int nb = min(kMemTb, r1 - t0);
    __syncthreads();
    if (KIND == 0) {
      const TA* xq = (const TA*)p.x;
      const int GD = p.G * D, width = 2 * GD + H * V;
      for (int e = tid; e < nb * D; e += 256) {
        const int tb = e / D, d = e - tb * D;
        const size_t row = (size_t)(t0 + tb) * width;
        sq[e] = ldx(xq, row + kvh * D + d);
        sk[e] = ldx(xq, row + GD + kvh * D + d);
        const float lo = p.a[(size_t)(t0 + tb) * H * D + hh * D + d] + p.dt_bias[hh * D + d];
        sgd[e] = expf(-rate * softplus_f(lo));
      }
      for (int e = tid; e < nb * kMemVb; e += 256) {
        const int tb = e / kMemVb, vv = e - tb * kMemVb;
        sv[e] = v0 + vv < V ? ldx(xq, (size_t)(t0 + tb) * width + 2 * GD + hh * V + v0 + vv) : 0.f;
      }
    } else {
      const float* xf = (const float*)p.x;
      const int HD = H * D;
      for (int e = tid; e < nb * D; e += 256) {
        const int tb = e / D, d = e - tb * D;
        const float* row = xf + (size_t)(t0 + tb) * p.xs;
        sq[e] = row[hh * D + d];
        sk[e] = row[HD + hh * D + d];
      }
      for (int e = tid; e < nb * kMemVb; e += 256) {
        const int tb = e / kMemVb, vv = e - tb * kMemVb;
        sv[e] = v0 + vv < V ? xf[(size_t)(t0 + tb) * p.xs + 2 * HD + hh * V + v0 + vv] : 0.f;
      }
      for (int e = tid; e < nb * 3; e += 256) {
        const int tb = e / 3, c = e - tb * 3;
        sc[tb * 4 + c] = p.ab[((size_t)(t0 + tb) * H + hh) * 3 + c];
      }
    }
    __syncthreads();
    if (KIND == 0) {
      // unit-length factors of q and k (a wave per (token, which) pair), and beta
      for (int pr = wv; pr < 2 * nb; pr += 4) {
        const int tb = pr >> 1, which = pr & 1;
        const float* src = (which ? sk : sq) + tb * D;
        float ss = 0.f;
        for (int d = lane; d < D; d += 64) ss = fmaf(src[d], src[d], ss);
        ss = wave_sum(ss);
        if (lane == 0) sc[tb * 4 + which] = (which ? 1.f : 1.f / sqrtf((float)D)) / sqrtf(ss + p.unit_eps);
      }
      if (tid < nb) sc[tid * 4 + 2] = sigmoid_f(p.beta[(size_t)(t0 + tid) * p.bs + hh]);
      __syncthreads();
    }
    for (int tb = 0; tb < nb; ++tb) {
      const float vv = sv[tb * kMemVb + vl];
      const float* kq = sk + tb * D;
      const float* qq = sq + tb * D;
      float acc = 0.f;
      if (KIND == 0) {
        const float* gd = sgd + tb * D;
        const float qf = sc[tb * 4], kf = sc[tb * 4 + 1], beta = sc[tb * 4 + 2];
        float ks = 0.f;
#pragma unroll
        for (int i = 0; i < DPT; ++i) {
          const int d = dg * DPT + i;
          if (d < D) {
            S[i] *= gd[d];
            ks = fmaf(S[i], kq[d], ks);
          }
        }
        ks += __shfl_xor(ks, 1, 64);
        ks += __shfl_xor(ks, 2, 64);
        const float u = beta * (vv - ks * kf) * kf;          // times k's unit factor once more for k u^T
#pragma unroll
        for (int i = 0; i < DPT; ++i) {
          const int d = dg * DPT + i;
          if (d < D) {
            S[i] = fmaf(kq[d], u, S[i]);
            acc = fmaf(S[i], qq[d], acc);
          }
        }
        acc *= qf;
      } else {
        const float fa = sc[tb * 4], iv = sc[tb * 4 + 1] * vv;
#pragma unroll
        for (int i = 0; i < DPT; ++i) {
          const int d = dg * DPT + i;
          if (d < D) {
            S[i] = fmaf(fa, S[i], kq[d] * iv);
            acc = fmaf(S[i], qq[d], acc);
          }
        }
        acc *= sc[tb * 4 + 2];
      }
      acc += __shfl_xor(acc, 1, 64);
      acc += __shfl_xor(acc, 2, 64);
      if (dg == 0 && vown) p.out[(size_t)(t0 + tb) * H * V + hh * V + v0 + vl] = acc;
    }
  }
#pragma unroll
  for (int i = 0; i < DPT; ++i) {
    const int d = dg * DPT + i;
    if (vown && d < D) st[(size_t)d * V] = S[i];
  }
}

// out[r][h] = o / sqrt(mean(o^2 over the head's V) + eps) * w * sigmoid(gate): one wave per (row, head).
// w is indexed h * wh + c: wh = V for a weight of all heads' size, 0 for one shared by the heads.
template <typename TA>
__global__ void __launch_bounds__(256) head_norm_sigmoid_kernel(const float* __restrict__ o, const float* __restrict__ gate,
                                                                int gs, const float* __restrict__ w, int wh,
                                                                TA* __restrict__ out, int n_rh, int H, int V, float eps) {
  const int rh = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (rh >= n_rh) return;
  const int r = rh / H, h = rh - r * H;
  const float* op = o + (size_t)rh * V;
  float ss = 0.f;
  for (int c = lane; c < V; c += 64) ss = fmaf(op[c], op[c], ss);
  const float rn = 1.f / sqrtf(wave_sum(ss) / (float)V + eps);
  const float* g = gate + (size_t)r * gs + (size_t)h * V;
  const float* wp = w + (size_t)h * wh;
  for (int c = lane; c < V; c += 64) stx(out, (size_t)rh * V + c, op[c] * rn * wp[c] * sigmoid_f(g[c]));
}

template <int KIND, typename TA>
static int launch_matrix_state(const MatArgs& p, int n_seg, hipStream_t s) {
  const int D = p.D;
  if (D < 1 || D > 256 || p.V < 1 || p.H < 1) return (int)hipErrorInvalidValue;
  const size_t lds = (size_t)(kMemTb * ((KIND == 0 ? 3 : 2) * D + kMemVb + 4)) * sizeof(float);
  const dim3 grid(n_seg, p.H, (p.V + kMemVb - 1) / kMemVb);
#define K8S_MAT(DP)                                                                                                \
  {                                                                                                                \
    auto k = matrix_state_kernel<DP, KIND, TA>;                                                                    \
    if (lds > 48 * 1024 && hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)) \
      return (int)hipGetLastError();                                                                               \
    hipLaunchKernelGGL(k, grid, dim3(256), lds, s, p);                                                             \
  }
  if (D <= 32) {
    K8S_MAT(8)
  } else if (D <= 64) {
    K8S_MAT(16)
  } else if (D <= 128) {
    K8S_MAT(32)
  } else {
    K8S_MAT(64)
  }
#undef K8S_MAT
  return (int)hipGetLastError();
}

}  // namespace k8s

using namespace k8s;

K8S_API int k8s_gated_delta(const void* qkv, int dt, const float* a, const float* rate, const float* dt_bias,
                            const float* beta, int bs, float* state, const int* seg_row0, const int* seg_pos0,
                            const int* seg_slot, float* out, int n_seg, int T, int H, int G, int D, int V,
                            float unit_eps, hipStream_t s) {
  if (n_seg <= 0 || T <= 0) return 0;
  if (G < 1 || H % G) return (int)hipErrorInvalidValue;
  MatArgs p{};
  p.x = qkv;
  p.a = a;
  p.rate = rate;
  p.dt_bias = dt_bias;
  p.beta = beta;
  p.bs = bs;
  p.state = state;
  p.seg_row0 = seg_row0;
  p.seg_pos0 = seg_pos0;
  p.seg_slot = seg_slot;
  p.out = out;
  p.H = H;
  p.G = G;
  p.D = D;
  p.V = V;
  p.unit_eps = unit_eps;
  return dt == 0 ? launch_matrix_state<0, uint16_t>(p, n_seg, s) : launch_matrix_state<0, float>(p, n_seg, s);
}

K8S_API int k8s_matrix_memory(const float* x, int xs, const float* gate_bias, float cap, float* state, float* nstate,
                              float* mstate, const int* seg_row0, const int* seg_pos0, const int* seg_slot, float* ab,
                              float* out, int n_seg, int T, int H, int D, int V, float den_eps, hipStream_t s) {
  if (n_seg <= 0 || T <= 0) return 0;
  if (D < 1 || D > 64 * kGatePer || D > 256 || cap <= 0.f) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(memory_gates_kernel, dim3((n_seg * H + 3) / 4), dim3(256), 0, s, x, xs, gate_bias, cap, nstate,
                     mstate, seg_row0, seg_pos0, seg_slot, ab, n_seg, H, D, V, den_eps);
  MatArgs p{};
  p.x = x;
  p.xs = xs;
  p.ab = ab;
  p.state = state;
  p.seg_row0 = seg_row0;
  p.seg_pos0 = seg_pos0;
  p.seg_slot = seg_slot;
  p.out = out;
  p.H = H;
  p.G = H;
  p.D = D;
  p.V = V;
  return launch_matrix_state<1, float>(p, n_seg, s);
}

K8S_API int k8s_head_norm_gate(const float* o, const float* gate, int gs, const float* w, int wh, void* out, int T,
                               int H, int V, float eps, int odt, hipStream_t s) {
  if (T <= 0) return 0;
  const int n_rh = T * H;
  if (odt == 0)
    hipLaunchKernelGGL((head_norm_sigmoid_kernel<uint16_t>), dim3((n_rh + 3) / 4), dim3(256), 0, s, o, gate, gs, w, wh,
                       (uint16_t*)out, n_rh, H, V, eps);
  else
    hipLaunchKernelGGL((head_norm_sigmoid_kernel<float>), dim3((n_rh + 3) / 4), dim3(256), 0, s, o, gate, gs, w, wh,
                       (float*)out, n_rh, H, V, eps);
  return (int)hipGetLastError();
}
