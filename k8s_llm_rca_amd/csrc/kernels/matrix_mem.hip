// Recurrences whose per-head state is a D x V matrix, over segments (seg_row0 / seg_pos0 / seg_slot as in
// mixer_ops.hip; a slot's state is read only when the segment does not start at position 0):
//
//   gated delta rule   S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
//                      with one decay per head and key channel, g = exp(-rate_h softplus(a + dt_bias)),
//                      q and k made unit vectors (q also times D^(-1/2)), grouped q / k heads;
//   matrix memory      m' = max(f + m, i);  S <- e^(f + m - m') S + e^(i - m') k v^T;  n likewise with k alone;
//                      o = S^T q / (max(|n.q|, e^(-m')) + den_eps), with soft-capped log gates i, f.
//
// Everything is fp32.  One workgroup of 256 threads owns 64 state columns of one (item, head): thread
// (dg = tid & 3, c = tid >> 2) holds S[d][c] for the DPT consecutive d from dg * DPT in registers, so the two
// sums over d per token (S^T k and S^T q) are DPT multiply-adds per thread and two cross-lane exchanges among
// four neighbouring lanes -- no barrier inside a token.  Tokens pass through LDS in batches of 16 (q, k,
// decays, values and the per-token scalars), one barrier pair per batch.
//
// The matrix memory's normaliser n is the state of one more column whose value is 1 for every token; its
// read-out is n.q.  The gates and the running maximum are a scalar recurrence per head: a kernel of their
// own runs it as a parallel scan over 64 tokens per wave (m_t = F_t + max(m_0, max_{s<=t}(i_s - F_s)) with F
// the running sum of f) and leaves per token the two factors and m.  m only keeps the exponentials in
// range -- the state is e^(-m) times the unstabilised one for ANY sequence m as long as both factors of a
// token use the same values -- so the scan's different rounding of m does not show in the output.
//
// MODE 0: an item is a whole segment, from the slot's state (or zero) to the slot's state.
// Long segments are cut into chunks ([n][4]: segment, first row, rows, -) that run in parallel:
// MODE 1: a chunk from a zero state: its end state goes to cs [chunks][H][D][V].  What carries a start state
//         through the chunk goes beside it: for the matrix memory the product of the forget factors (cdec)
//         and the normaliser column (cx [chunks][H][D]); for the delta rule, whose step is
//         S <- (I - beta k k^T) diag(g) S + beta k v^T, the product of the chunk's D x D step matrices: D more
//         columns that start as the identity and see the value 0 (cx [chunks][H][D][D]);
// (the carry kernels then turn cs / cx into every chunk's START state and advance the slot's state)
// MODE 2: the chunk again from its start state, writing the outputs.
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
constexpr int kMemVb = 64;     // state columns per workgroup

// Rows of x (fp32, stride xs): q [H][D] | k [H][D] | v [H][V] | gate [H][V] | i [H] | f [H].
// ab [T][H][3] receives (forget factor, input factor, m) of every token; one wave per (segment, head),
// 64 tokens at a time, one per lane.
__global__ void __launch_bounds__(256) memory_gates_kernel(const float* __restrict__ x, int xs,
                                                           const float* __restrict__ gate_bias, float cap,
                                                           float* __restrict__ mstate,
                                                           const int* __restrict__ seg_row0,
                                                           const int* __restrict__ seg_pos0,
                                                           const int* __restrict__ seg_slot, float* __restrict__ ab,
                                                           int n_seg, int H, int D, int V) {
  const int unit = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (unit >= n_seg * H) return;
  const int sg = unit / H, hh = unit - sg * H;
  const int r0 = seg_row0[sg], r1 = seg_row0[sg + 1];
  const size_t so = (size_t)seg_slot[sg] * H + hh;
  float m0 = seg_pos0[sg] == 0 ? 0.f : mstate[so];
  const int go = 2 * H * D + 2 * H * V;
  const float bi = gate_bias[hh], bf = gate_bias[H + hh];
  for (int t0 = r0; t0 < r1; t0 += 64) {
    const int r = t0 + lane;
    const bool on = r < r1;
    float gi = -INFINITY, gf = 0.f;
    if (on) {
      const float* row = x + (size_t)r * xs;
      gi = cap * tanhf((row[go + hh] + bi) / cap);
      gf = logsigmoid_f(cap * tanhf((row[go + H + hh] + bf) / cap));
    }
    float F = gf;                                  // running sum of f over the batch
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const float up = __shfl_up(F, o, 64);
      if (lane >= o) F += up;
    }
    float pa = gi - F;                             // running maximum of i_s - F_s
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const float up = __shfl_up(pa, o, 64);
      if (lane >= o) pa = fmaxf(pa, up);
    }
    const float m = F + fmaxf(m0, pa);
    const float mup = __shfl_up(m, 1, 64);
    const float mprev = lane == 0 ? m0 : mup;
    if (on) {
      float* o = ab + ((size_t)r * H + hh) * 3;
      o[0] = expf(gf + mprev - m);
      o[1] = expf(gi - m);
      o[2] = m;
    }
    m0 = __shfl(m, min(63, r1 - t0 - 1), 64);
  }
  if (lane == 0) mstate[so] = m0;
}

// mul[r][h] = D^(-1/2) / (max(|nq|, e^(-m)) + den_eps): what the raw read-out S^T q (q unscaled) is multiplied by
__global__ void __launch_bounds__(256) memory_den_kernel(const float* __restrict__ nq, const float* __restrict__ ab,
                                                         float* __restrict__ mul, int n, float qs, float den_eps) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) mul[i] = qs / (fmaxf(fabsf(nq[i] * qs), expf(-ab[(size_t)i * 3 + 2])) + den_eps);
}

// o[r][h][:] *= mul[r][h]
__global__ void __launch_bounds__(256) scale_heads_kernel(float* __restrict__ o, const float* __restrict__ mul, size_t n,
                                                          int V) {
  for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < n; e += (size_t)gridDim.x * 256) o[e] *= mul[e / V];
}

// KIND 0: gated delta rule.  qkv rows (TA, contiguous, width 2 G D + H V): q [G][D] | k [G][D] | v [H][V];
//         a [T][H D] fp32 (before bias and softplus); beta [T] rows of stride bs, column hh (before the sigmoid).
// KIND 1: matrix memory.  x rows (fp32, stride xs) as in memory_gates_kernel; ab from that kernel; column V is
//         the normaliser (state in nstate [slots][H][D]), its read-out goes to nq [T][H]; out is S^T q, raw.
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
  float* nstate;
  const int* seg_row0;
  const int* seg_pos0;
  const int* seg_slot;
  float* out;          // [T][H V] fp32
  float* nq;           // [T][H]
  int H, G, D, V;
  float unit_eps;
  const int* chunks;   // MODE 1 / 2
  float* cs;           // [chunks][H][D][V]
  float* cx;           // [chunks][H][D] (memory) or [chunks][H][D][D] (delta)
  float* cdec;         // [chunks][H] (memory)
};

// FULL: D == 4 * DPT, every thread's DPT rows exist (no guards in the token loop: its LDS reads become
// 16-byte ones)
template <int DPT, int KIND, int MODE, bool FULL, typename TA>
__global__ void __launch_bounds__(256) matrix_state_kernel(MatArgs p) {
  extern __shared__ float sm[];
  const int it = blockIdx.x, hh = blockIdx.y, c0 = blockIdx.z * kMemVb, tid = threadIdx.x;
  const int H = p.H, D = p.D, V = p.V;
  float* sq = sm;                                  // [TB][D]
  float* sk = sq + kMemTb * D;                     // [TB][D]
  float* sgd = sk + kMemTb * D;                    // [TB][D] decays (KIND 0)
  float* sv = sgd + (KIND == 0 ? kMemTb * D : 0);  // [TB][64]
  float* sc = sv + kMemTb * kMemVb;                // [TB][4] per-token scalars
  const int dg = tid & 3, vl = tid >> 2, lane = tid & 63, wv = tid >> 6;
  int sg, r0, r1;
  bool fresh;
  if (MODE == 0) {
    sg = it;
    r0 = p.seg_row0[sg];
    r1 = p.seg_row0[sg + 1];
    fresh = p.seg_pos0[sg] == 0;
  } else {
    sg = p.chunks[it * 4];
    r0 = p.chunks[it * 4 + 1];
    r1 = r0 + p.chunks[it * 4 + 2];
    fresh = MODE == 1;
  }
  // this thread's column: a value column, or an extra one (the normaliser; a column of the step-matrix product)
  const int X = KIND == 1 ? 1 : (MODE == 1 ? D : 0);
  const int c = c0 + vl;
  const bool cown = c < V + X, extra = c >= V;
  float* colp;
  int cstride;
  if (!extra) {
    colp = (MODE == 0 ? p.state + ((size_t)p.seg_slot[sg] * H + hh) * D * V : p.cs + ((size_t)it * H + hh) * D * V) + c;
    cstride = V;
  } else if (KIND == 1) {
    colp = MODE == 0 ? p.nstate + ((size_t)p.seg_slot[sg] * H + hh) * D : p.cx + ((size_t)it * H + hh) * D;
    cstride = 1;
  } else {
    colp = p.cx + ((size_t)it * H + hh) * D * D + (c - V);
    cstride = D;
  }
  float S[DPT];
#pragma unroll
  for (int i = 0; i < DPT; ++i) {
    const int d = dg * DPT + i;
    if (fresh)
      S[i] = (KIND == 0 && extra && d == c - V) ? 1.f : 0.f;
    else
      S[i] = (cown && d < D) ? colp[(size_t)d * cstride] : 0.f;
  }
  const int kvh = hh / (H / p.G);
  const float rate = KIND == 0 ? p.rate[hh] : 0.f;
  float pdec = 1.f;
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
        sv[e] = c0 + vv < V ? ldx(xq, (size_t)(t0 + tb) * width + 2 * GD + hh * V + c0 + vv) : 0.f;
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
        sv[e] = c0 + vv < V ? xf[(size_t)(t0 + tb) * p.xs + 2 * HD + hh * V + c0 + vv] : (c0 + vv == V ? 1.f : 0.f);
      }
      for (int e = tid; e < nb * 2; e += 256) {
        const int tb = e >> 1, w = e & 1;
        sc[tb * 4 + w] = p.ab[((size_t)(t0 + tb) * H + hh) * 3 + w];
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
          if (FULL || d < D) {
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
          if (FULL || d < D) {
            S[i] = fmaf(kq[d], u, S[i]);
            if (MODE != 1) acc = fmaf(S[i], qq[d], acc);
          }
        }
        acc *= qf;
      } else {
        const float fa = sc[tb * 4], iv = sc[tb * 4 + 1] * vv;
        pdec *= fa;
#pragma unroll
        for (int i = 0; i < DPT; ++i) {
          const int d = dg * DPT + i;
          if (FULL || d < D) {
            S[i] = fmaf(fa, S[i], kq[d] * iv);
            if (MODE != 1) acc = fmaf(S[i], qq[d], acc);
          }
        }
      }
      if (MODE != 1) {
        acc += __shfl_xor(acc, 1, 64);
        acc += __shfl_xor(acc, 2, 64);
        if (dg == 0 && cown) {
          if (!extra)
            p.out[(size_t)(t0 + tb) * H * V + hh * V + c] = acc;
          else if (KIND == 1)
            p.nq[(size_t)(t0 + tb) * H + hh] = acc;
        }
      }
    }
  }
  if (MODE != 2) {
#pragma unroll
    for (int i = 0; i < DPT; ++i) {
      const int d = dg * DPT + i;
      if (cown && d < D) colp[(size_t)d * cstride] = S[i];
    }
    if (KIND == 1 && MODE == 1 && tid == 0 && blockIdx.z == 0) p.cdec[(size_t)it * H + hh] = pdec;
  }
}

// Matrix memory, between the two chunk passes: one thread per state entry of a (segment, head) -- the D V
// entries of S, then the D of n.  Walks the segment's chunks (seg_chunk0[s] .. seg_chunk0[s + 1]), replaces
// every chunk's end-from-zero state by its START state and leaves the segment's final state in the slot.
__global__ void __launch_bounds__(256) memory_carry_kernel(MatArgs p, const int* __restrict__ seg_chunk0) {
  const int sg = blockIdx.x, hh = blockIdx.y, e = blockIdx.z * 256 + threadIdx.x;
  const int H = p.H, DV = p.D * p.V, D = p.D;
  if (e >= DV + D) return;
  const bool isn = e >= DV;
  float* st = isn ? p.nstate + ((size_t)p.seg_slot[sg] * H + hh) * D + (e - DV)
                  : p.state + ((size_t)p.seg_slot[sg] * H + hh) * DV + e;
  float S = p.seg_pos0[sg] == 0 ? 0.f : *st;
  for (int k = seg_chunk0[sg]; k < seg_chunk0[sg + 1]; ++k) {
    float* ck = isn ? p.cx + ((size_t)k * H + hh) * D + (e - DV) : p.cs + ((size_t)k * H + hh) * DV + e;
    const float loc = *ck;
    *ck = S;
    S = fmaf(p.cdec[(size_t)k * H + hh], S, loc);
  }
  *st = S;
}

// Delta rule, between the two chunk passes: a workgroup per (segment, head, 64 value columns) holds its
// columns of the state in LDS and walks the segment's chunks:  S_start(k + 1) = P_k S_start(k) + local_k  with
// P_k the chunk's D x D step-matrix product (also through LDS).  Thread (dg, c) forms the DPT rows from dg DPT.
template <int DPT>
__global__ void __launch_bounds__(256) delta_carry_kernel(MatArgs p, const int* __restrict__ seg_chunk0) {
  extern __shared__ float sm[];
  const int sg = blockIdx.x, hh = blockIdx.y, c0 = blockIdx.z * kMemVb, tid = threadIdx.x;
  const int H = p.H, D = p.D, V = p.V;
  constexpr int DP = 4 * DPT;     // row length of the transposed product in LDS (>= D)
  float* sS = sm;                 // [D][64]
  float* sP = sS + D * kMemVb;    // [D][DP]
  const int dg = tid & 3, vl = tid >> 2, c = c0 + vl;
  const bool cown = c < V;
  float* st = p.state + ((size_t)p.seg_slot[sg] * H + hh) * D * V + c;
  const bool fresh = p.seg_pos0[sg] == 0;
  float S[DPT];
#pragma unroll
  for (int i = 0; i < DPT; ++i) {
    const int d = dg * DPT + i;
    S[i] = (cown && d < D && !fresh) ? st[(size_t)d * V] : 0.f;
  }
  for (int k = seg_chunk0[sg]; k < seg_chunk0[sg + 1]; ++k) {
    float* ck = p.cs + ((size_t)k * H + hh) * D * V + c;
    const float* P = p.cx + ((size_t)k * H + hh) * D * D;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < DPT; ++i) {
      const int d = dg * DPT + i;
      if (d < D) sS[d * kMemVb + vl] = S[i];
    }
    for (int e = tid; e < D * D; e += 256) {            // transposed: sP[j][d], a thread's DPT rows side by side
      const int d = e / D, j = e - d * D;
      sP[j * DP + d] = P[e];
    }
    __syncthreads();
    float acc[DPT];
#pragma unroll
    for (int i = 0; i < DPT; ++i) {
      const int d = dg * DPT + i;
      acc[i] = (cown && d < D) ? ck[(size_t)d * V] : 0.f;   // the chunk's end state from zero
      if (cown && d < D) ck[(size_t)d * V] = S[i];          // becomes its start state
    }
    for (int j = 0; j < D; ++j) {
      const float sj = sS[j * kMemVb + vl];
      const float* pc = sP + j * DP + dg * DPT;
#pragma unroll
      for (int i = 0; i < DPT; ++i) acc[i] = fmaf(pc[i], sj, acc[i]);
    }
#pragma unroll
    for (int i = 0; i < DPT; ++i) S[i] = acc[i];
  }
#pragma unroll
  for (int i = 0; i < DPT; ++i) {
    const int d = dg * DPT + i;
    if (cown && d < D) st[(size_t)d * V] = S[i];
  }
}

// out[r][h] = u / sqrt(mean(u^2 over the head's V) + eps) * w * sigmoid(gate) * oscale, u = o * mul[r][h] (mul
// optional): one wave per (row, head).  w and gate are optional (absent: 1).
// w is indexed h * wh + c: wh = V for a weight of all heads' size, 0 for one shared by the heads.
// sub: o holds two results per head, [r][h][2][V], and u = o[.][0] - lam o[.][1] (two score maps joined).
template <typename TA>
__global__ void __launch_bounds__(256) head_norm_sigmoid_kernel(const float* __restrict__ o, const float* __restrict__ gate,
                                                                int gs, const float* __restrict__ w, int wh,
                                                                TA* __restrict__ out, int n_rh, int H, int V, float eps,
                                                                const float* __restrict__ mul, int sub, float lam,
                                                                float oscale) {
  const int rh = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (rh >= n_rh) return;
  const int r = rh / H, h = rh - r * H;
  const float* op = o + (size_t)rh * V * (sub ? 2 : 1);
  const float mu = mul ? mul[rh] : 1.f;
  float ss = 0.f;
  for (int c = lane; c < V; c += 64) {
    const float u = (sub ? op[c] - lam * op[V + c] : op[c]) * mu;
    ss = fmaf(u, u, ss);
  }
  const float rn = mu * oscale / sqrtf(wave_sum(ss) / (float)V + eps);
  const float* g = gate ? gate + (size_t)r * gs + (size_t)h * V : nullptr;
  const float* wp = w ? w + (size_t)h * wh : nullptr;
  for (int c = lane; c < V; c += 64) {
    const float u = sub ? op[c] - lam * op[V + c] : op[c];
    stx(out, (size_t)rh * V + c, u * rn * (wp ? wp[c] : 1.f) * (g ? sigmoid_f(g[c]) : 1.f));
  }
}

template <int DPT, int KIND, int MODE, bool FULL, typename TA>
static int launch_state_full(const MatArgs& p, int items, int cols, size_t lds, hipStream_t s) {
  auto k = matrix_state_kernel<DPT, KIND, MODE, FULL, TA>;
  if (lds > 48 * 1024 && hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds))
    return (int)hipGetLastError();
  hipLaunchKernelGGL(k, dim3(items, p.H, (cols + kMemVb - 1) / kMemVb), dim3(256), lds, s, p);
  return (int)hipGetLastError();
}

template <int DPT, int KIND, int MODE, typename TA>
static int launch_state_mode(const MatArgs& p, int items, int cols, size_t lds, hipStream_t s) {
  return p.D == 4 * DPT ? launch_state_full<DPT, KIND, MODE, true, TA>(p, items, cols, lds, s)
                        : launch_state_full<DPT, KIND, MODE, false, TA>(p, items, cols, lds, s);
}

// n_chunks == 0: every segment token by token; otherwise the two chunk passes around the carry
template <int DPT, int KIND, typename TA>
static int launch_state_dpt(const MatArgs& p, int n_seg, int n_chunks, const int* seg_chunk0, hipStream_t s) {
  const int D = p.D, V = p.V;
  const size_t lds = (size_t)(kMemTb * ((KIND == 0 ? 3 : 2) * D + kMemVb + 4)) * sizeof(float);
  // (the delta rule's carry holds a D x D product and D x 64 state entries in LDS: token by token where that does not fit)
  const size_t cl = (size_t)(D * kMemVb + D * 4 * DPT) * sizeof(float);
  if (n_chunks <= 0 || (KIND == 0 && cl > 160 * 1024))
    return launch_state_mode<DPT, KIND, 0, TA>(p, n_seg, V + (KIND == 1 ? 1 : 0), lds, s);
  int rc = launch_state_mode<DPT, KIND, 1, TA>(p, n_chunks, V + (KIND == 1 ? 1 : D), lds, s);
  if (rc) return rc;
  if (KIND == 1) {
    hipLaunchKernelGGL(memory_carry_kernel, dim3(n_seg, p.H, (D * V + D + 255) / 256), dim3(256), 0, s, p, seg_chunk0);
  } else {
    auto k = delta_carry_kernel<DPT>;
    if (cl > 48 * 1024 && hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)cl))
      return (int)hipGetLastError();
    hipLaunchKernelGGL(k, dim3(n_seg, p.H, (V + kMemVb - 1) / kMemVb), dim3(256), cl, s, p, seg_chunk0);
  }
  rc = (int)hipGetLastError();
  if (rc) return rc;
  return launch_state_mode<DPT, KIND, 2, TA>(p, n_chunks, V + (KIND == 1 ? 1 : 0), lds, s);
}

template <int KIND, typename TA>
static int launch_matrix_state(const MatArgs& p, int n_seg, int n_chunks, const int* seg_chunk0, hipStream_t s) {
  const int D = p.D;
  if (D < 1 || D > 256 || p.V < 1 || p.H < 1) return (int)hipErrorInvalidValue;
  if (n_chunks > 0 && (!p.chunks || !seg_chunk0 || !p.cs || !p.cx || (KIND == 1 && !p.cdec)))
    return (int)hipErrorInvalidValue;
  if (D <= 32) return launch_state_dpt<8, KIND, TA>(p, n_seg, n_chunks, seg_chunk0, s);
  if (D <= 64) return launch_state_dpt<16, KIND, TA>(p, n_seg, n_chunks, seg_chunk0, s);
  if (D <= 128) return launch_state_dpt<32, KIND, TA>(p, n_seg, n_chunks, seg_chunk0, s);
  return launch_state_dpt<64, KIND, TA>(p, n_seg, n_chunks, seg_chunk0, s);
}

}  // namespace k8s

using namespace k8s;

K8S_API int k8s_gated_delta(const void* qkv, int dt, const float* a, const float* rate, const float* dt_bias,
                            const float* beta, int bs, float* state, const int* seg_row0, const int* seg_pos0,
                            const int* seg_slot, float* out, int n_seg, int T, int H, int G, int D, int V,
                            float unit_eps, hipStream_t s, const int* chunks, int n_chunks, const int* seg_chunk0,
                            float* cs, float* cx) {
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
  p.chunks = chunks;
  p.cs = cs;
  p.cx = cx;
  return dt == 0 ? launch_matrix_state<0, uint16_t>(p, n_seg, n_chunks, seg_chunk0, s)
                 : launch_matrix_state<0, float>(p, n_seg, n_chunks, seg_chunk0, s);
}

// out = S^T q raw (q unscaled), mul [T][H] = what it is to be multiplied by; scale_out != 0: out *= mul here
K8S_API int k8s_matrix_memory(const float* x, int xs, const float* gate_bias, float cap, float* state, float* nstate,
                              float* mstate, const int* seg_row0, const int* seg_pos0, const int* seg_slot, float* ab,
                              float* nq, float* mul, float* out, int n_seg, int T, int H, int D, int V, float den_eps,
                              int scale_out, hipStream_t s, const int* chunks, int n_chunks, const int* seg_chunk0,
                              float* cs, float* cx, float* cdec) {
  if (n_seg <= 0 || T <= 0) return 0;
  if (D < 1 || D > 256 || cap <= 0.f) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(memory_gates_kernel, dim3((n_seg * H + 3) / 4), dim3(256), 0, s, x, xs, gate_bias, cap, mstate,
                     seg_row0, seg_pos0, seg_slot, ab, n_seg, H, D, V);
  MatArgs p{};
  p.x = x;
  p.xs = xs;
  p.ab = ab;
  p.state = state;
  p.nstate = nstate;
  p.seg_row0 = seg_row0;
  p.seg_pos0 = seg_pos0;
  p.seg_slot = seg_slot;
  p.out = out;
  p.nq = nq;
  p.H = H;
  p.G = H;
  p.D = D;
  p.V = V;
  p.chunks = chunks;
  p.cs = cs;
  p.cx = cx;
  p.cdec = cdec;
  const int rc = launch_matrix_state<1, float>(p, n_seg, n_chunks, seg_chunk0, s);
  if (rc) return rc;
  hipLaunchKernelGGL(memory_den_kernel, dim3((T * H + 255) / 256), dim3(256), 0, s, nq, ab, mul, T * H,
                     1.f / sqrtf((float)D), den_eps);
  if (scale_out) {
    const size_t n = (size_t)T * H * V;
    const size_t g = (n + 255) / 256;
    hipLaunchKernelGGL(scale_heads_kernel, dim3((int)(g > 8192 ? 8192 : g)), dim3(256), 0, s, out, mul, n, V);
  }
  return (int)hipGetLastError();
}

// mul (optional) [T][H]: o is multiplied by it before the norm
K8S_API int k8s_head_norm_gate(const float* o, const float* gate, int gs, const float* w, int wh, void* out, int T,
                               int H, int V, float eps, int odt, hipStream_t s, const float* mul, int sub, float lam,
                               float oscale) {
  if (T <= 0) return 0;
  const int n_rh = T * H;
  if (odt == 0)
    hipLaunchKernelGGL((head_norm_sigmoid_kernel<uint16_t>), dim3((n_rh + 3) / 4), dim3(256), 0, s, o, gate, gs, w, wh,
                       (uint16_t*)out, n_rh, H, V, eps, mul, sub, lam, oscale);
  else
    hipLaunchKernelGGL((head_norm_sigmoid_kernel<float>), dim3((n_rh + 3) / 4), dim3(256), 0, s, o, gate, gs, w, wh,
                       (float*)out, n_rh, H, V, eps, mul, sub, lam, oscale);
  return (int)hipGetLastError();
}
