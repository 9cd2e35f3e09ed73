// Recurrent mixers over segments: a short causal convolution with bias and
// activation (its last taps - 1 inputs are per-sequence state), the selective
// scan of a diagonal state-space layer, and retention (linear attention with a
// fixed decay per head, rotary positions, per-head unit norm and output gate).
//
// Segments as in seq_ops.hip: seg_row0[n_seg + 1] row offsets, seg_pos0[s] the
// position of the segment's first token, seg_slot[s] the sequence's state slot,
// row_seg[T] the segment of every row.  State of a slot is read only when
// seg_pos0 > 0.  All recurrences, their decays, step sizes and gates are fp32;
// TA is the activation type (bf16 as uint16_t, or float).
#include "common.h"

namespace k8s {

template <typename T>
__device__ __forceinline__ float ldm(const T* p, size_t i);
template <>
__device__ __forceinline__ float ldm<float>(const float* p, size_t i) { return p[i]; }
template <>
__device__ __forceinline__ float ldm<uint16_t>(const uint16_t* p, size_t i) { return bf2f(p[i]); }
template <typename T>
__device__ __forceinline__ void stm(T* p, size_t i, float v);
template <>
__device__ __forceinline__ void stm<float>(float* p, size_t i, float v) { p[i] = v; }
template <>
__device__ __forceinline__ void stm<uint16_t>(uint16_t* p, size_t i, float v) { p[i] = f2bf(v); }

__device__ __forceinline__ float silu_f(float v) { return v / (1.f + expf(-v)); }

// exp of the recurrence's decays (arguments <= 0): the full-precision routine where activations are
// fp32; where they are bf16 the hardware exponential 2^x (about 1e-6 relative, tiny results flush to 0)
// with log2(e) folded into A beforehand
template <typename TA>
struct DecayExp;
template <>
struct DecayExp<float> {
  static constexpr float kPre = 1.f;
  static __device__ __forceinline__ float f(float x) { return expf(x); }
  static __device__ __forceinline__ float softplus(float x) { return x > 20.f ? x : log1pf(expf(x)); }
  static __device__ __forceinline__ float silu(float x) { return silu_f(x); }
};
template <>
struct DecayExp<uint16_t> {
  static constexpr float kPre = 1.4426950408889634f;
  static __device__ __forceinline__ float f(float x) { return __builtin_amdgcn_exp2f(x); }
  // hardware exp / log (relative error about 1e-6, far below the bf16 activations around them);
  // for small u = e^x the series u - u^2 / 2 + u^3 / 3 keeps the relative accuracy of small step
  // sizes, which log(1 + u) would lose
  static __device__ __forceinline__ float softplus(float x) {
    if (x > 20.f) return x;
    const float u = __expf(x);
    return x < -4.f ? u * (1.f - u * (0.5f - u * (1.f / 3.f))) : __logf(1.f + u);
  }
  static __device__ __forceinline__ float silu(float x) { return __fdividef(x, 1.f + __expf(-x)); }
};

// out[r][c] = act(b[c] + sum_j w[c][j] * in(r - (taps - 1 - j))): the last column is the current
// token's tap.  Inputs before the segment come from the slot's tail (entry k = the input at
// position pos0 - (taps - 1) + k), zeros before the sequence.  x rows have stride xs.
template <typename TA>
__global__ void __launch_bounds__(256) short_conv_kernel(const TA* __restrict__ x, int xs, const float* __restrict__ w,
                                                         const float* __restrict__ b, const float* __restrict__ tail,
                                                         const int* __restrict__ row_seg,
                                                         const int* __restrict__ seg_row0,
                                                         const int* __restrict__ seg_pos0,
                                                         const int* __restrict__ seg_slot, TA* __restrict__ out, int C,
                                                         int taps, int act) {
  const int r = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int sg = row_seg[r], r0 = seg_row0[sg], p0 = seg_pos0[sg];
  const float* tl = tail + (size_t)seg_slot[sg] * (taps - 1) * C;
  float acc = b ? b[c] : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int rr = r - (taps - 1 - j);
    float v;
    if (rr >= r0) {
      v = ldm(x, (size_t)rr * xs + c);
    } else {
      const int back = r0 - rr;          // 1 .. taps - 1 inputs before the segment
      v = (p0 - back >= 0) ? tl[(size_t)(taps - 1 - back) * C + c] : 0.f;
    }
    acc = fmaf(w[(size_t)c * taps + j], v, acc);
  }
  stm(out, (size_t)r * C + c, act ? silu_f(acc) : acc);
}

// The same over TILES of consecutive rows of one segment ([n][4]: segment, first row, rows, position
// of the first row), one workgroup per (tile, 256 channels): the segment's metadata is read once per
// tile instead of once per row, and a thread slides a window of TAPS - 1 earlier inputs in registers,
// so every input is loaded once.
template <int TAPS, typename TA>
__global__ void __launch_bounds__(256) short_conv_tile_kernel(const TA* __restrict__ x, int xs,
                                                              const float* __restrict__ w, const float* __restrict__ b,
                                                              const float* __restrict__ tail,
                                                              const int* __restrict__ items,
                                                              const int* __restrict__ seg_row0,
                                                              const int* __restrict__ seg_pos0,
                                                              const int* __restrict__ seg_slot, TA* __restrict__ out,
                                                              int C, int act) {
  const int it = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int sg = items[it * 4], row0 = items[it * 4 + 1], ntok = items[it * 4 + 2];
  const int r0 = seg_row0[sg], p0 = seg_pos0[sg];
  const float* tl = tail + (size_t)seg_slot[sg] * (TAPS - 1) * C;
  float wt[TAPS], hist[TAPS];   // hist[k]: the input (TAPS - 1 - k) rows before the current one
#pragma unroll
  for (int j = 0; j < TAPS; ++j) wt[j] = w[(size_t)c * TAPS + j];
#pragma unroll
  for (int k = 0; k < TAPS - 1; ++k) {
    const int rr = row0 - (TAPS - 1) + k;
    if (rr >= r0) {
      hist[k] = ldm(x, (size_t)rr * xs + c);
    } else {
      const int back = r0 - rr;
      hist[k] = (p0 - back >= 0) ? tl[(size_t)(TAPS - 1 - back) * C + c] : 0.f;
    }
  }
  const float bias = b ? b[c] : 0.f;
  for (int q = 0; q < ntok; ++q) {
    hist[TAPS - 1] = ldm(x, (size_t)(row0 + q) * xs + c);
    float acc = bias;
#pragma unroll
    for (int j = 0; j < TAPS; ++j) acc = fmaf(wt[j], hist[j], acc);
    stm(out, (size_t)(row0 + q) * C + c, act ? silu_f(acc) : acc);
#pragma unroll
    for (int j = 0; j < TAPS - 1; ++j) hist[j] = hist[j + 1];
  }
}

// After the convolution of a step: the slot's tail becomes the last taps - 1 inputs up to the
// segment's end (old entries shift down when the segment is shorter than the tail).
template <typename TA>
__global__ void __launch_bounds__(256) short_conv_tail_kernel(const TA* __restrict__ x, int xs, float* __restrict__ tail,
                                                              const int* __restrict__ seg_row0,
                                                              const int* __restrict__ seg_pos0,
                                                              const int* __restrict__ seg_slot, int C, int taps) {
  constexpr int kMaxTail = 15;
  const int sg = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int r0 = seg_row0[sg], n = seg_row0[sg + 1] - r0, p0 = seg_pos0[sg], nt = taps - 1;
  float* tl = tail + (size_t)seg_slot[sg] * nt * C;
  float nv[kMaxTail];
#pragma unroll
  for (int k = 0; k < kMaxTail; ++k) {
    if (k < nt) {
      const int back = nt - k;           // new entry k = the input `back` tokens before the new end
      const int rr = r0 + n - back;
      if (rr >= r0) {
        nv[k] = ldm(x, (size_t)rr * xs + c);
      } else {
        const int b0 = r0 - rr;          // inputs before the segment
        nv[k] = (p0 - b0 >= 0) ? tl[(size_t)(nt - b0) * C + c] : 0.f;
      }
    }
  }
#pragma unroll
  for (int k = 0; k < kMaxTail; ++k)
    if (k < nt) tl[(size_t)k * C + c] = nv[k];
}

// Selective scan, one thread per channel, the channel's N states in registers:
//   dt = softplus(dtp[r][c] + dt_bias[c]);  S[n] <- exp(dt A[c][n]) S[n] + dt x B[r][n];
//   y = (sum_n S[n] C[r][n] + D[c] x) * silu(z[r][c]).
// dbc rows (stride ds) hold B at column R and C at column R + N, fp32.  state [slots][C][N].
// MODE 0: a whole segment per workgroup row (blockIdx.x = segment), state read and written.
// Long segments are cut into chunks ([n][4]: segment, first row, rows, -) that run in parallel:
// MODE 1: a chunk from a zero state: its end state and the sum of its step sizes go to
//         cs [chunks][C][N] / csd [chunks][C] (the chunk's decay is exp(A * sum dt));
// (scan_carry_kernel then turns cs into every chunk's START state and advances the slot's state)
// MODE 2: the chunk again from its start state, writing y.
template <int NMAX, int MODE, typename TA>
__global__ void __launch_bounds__(128) selective_scan_kernel(const TA* __restrict__ xc, const float* __restrict__ dtp,
                                                             const float* __restrict__ dt_bias,
                                                             const float* __restrict__ dbc, int ds, int R,
                                                             const float* __restrict__ A, const float* __restrict__ Dp,
                                                             const TA* __restrict__ z, int zs, float* __restrict__ state,
                                                             const int* __restrict__ seg_row0,
                                                             const int* __restrict__ seg_pos0,
                                                             const int* __restrict__ seg_slot, TA* __restrict__ y,
                                                             int C, int N, const int* __restrict__ chunks,
                                                             float* __restrict__ cs, float* __restrict__ csd) {
  const int it = blockIdx.x, c = blockIdx.y * 128 + threadIdx.x;
  if (c >= C) return;
  int r0, r1;
  bool fresh;
  float* st;
  if (MODE == 0) {
    r0 = seg_row0[it];
    r1 = seg_row0[it + 1];
    fresh = seg_pos0[it] == 0;
    st = state + ((size_t)seg_slot[it] * C + c) * N;
  } else {
    r0 = chunks[it * 4 + 1];
    r1 = r0 + chunks[it * 4 + 2];
    fresh = MODE == 1;
    st = cs + ((size_t)it * C + c) * N;
  }
  float S[NMAX], Ac[NMAX];
#pragma unroll
  for (int n = 0; n < NMAX; ++n) {
    Ac[n] = n < N ? A[(size_t)c * N + n] * DecayExp<TA>::kPre : 0.f;
    S[n] = (n < N && !fresh) ? st[n] : 0.f;
  }
  const float Dc = Dp[c], bias = dt_bias[c];
  float sd = 0.f;
  for (int r = r0; r < r1; ++r) {
    const float dv = dtp[(size_t)r * C + c] + bias;
    const float dt = DecayExp<TA>::softplus(dv);
    const float xv = ldm(xc, (size_t)r * C + c);
    const float dx = dt * xv;
    const float* Bp = dbc + (size_t)r * ds + R;
    const float* Cp = Bp + N;
    float acc = 0.f;
    sd += dt;
#pragma unroll
    for (int n = 0; n < NMAX; ++n)
      if (n < N) {
        S[n] = fmaf(DecayExp<TA>::f(dt * Ac[n]), S[n], dx * Bp[n]);
        if (MODE != 1) acc = fmaf(S[n], Cp[n], acc);
      }
    if (MODE != 1) {
      const float zv = ldm(z, (size_t)r * zs + c);
      stm(y, (size_t)r * C + c, (acc + Dc * xv) * DecayExp<TA>::silu(zv));
    }
  }
  if (MODE != 2) {
#pragma unroll
    for (int n = 0; n < NMAX; ++n)
      if (n < N) st[n] = S[n];
  }
  if (MODE == 1) csd[(size_t)it * C + c] = sd;
}

// Between the two chunk passes, one thread per (segment, channel): walk the segment's chunks
// (seg_chunk0[s] .. seg_chunk0[s + 1]), replace every chunk's end-from-zero state by its START state,
// and leave the segment's final state in the slot.
template <int NMAX>
__global__ void __launch_bounds__(128) scan_carry_kernel(const float* __restrict__ A, float* __restrict__ state,
                                                         const int* __restrict__ seg_pos0,
                                                         const int* __restrict__ seg_slot,
                                                         const int* __restrict__ seg_chunk0, float* __restrict__ cs,
                                                         const float* __restrict__ csd, int C, int N) {
  const int sg = blockIdx.x, c = blockIdx.y * 128 + threadIdx.x;
  if (c >= C) return;
  float* st = state + ((size_t)seg_slot[sg] * C + c) * N;
  const bool fresh = seg_pos0[sg] == 0;
  float S[NMAX], Ac[NMAX];
#pragma unroll
  for (int n = 0; n < NMAX; ++n) {
    Ac[n] = n < N ? A[(size_t)c * N + n] : 0.f;
    S[n] = (n < N && !fresh) ? st[n] : 0.f;
  }
  for (int k = seg_chunk0[sg]; k < seg_chunk0[sg + 1]; ++k) {
    float* ck = cs + ((size_t)k * C + c) * N;
    const float sd = csd[(size_t)k * C + c];
#pragma unroll
    for (int n = 0; n < NMAX; ++n)
      if (n < N) {
        const float loc = ck[n];
        ck[n] = S[n];
        S[n] = fmaf(expf(sd * Ac[n]), S[n], loc);
      }
  }
#pragma unroll
  for (int n = 0; n < NMAX; ++n)
    if (n < N) st[n] = S[n];
}

// State-space recurrence with ONE decay per head and token (the scalar-decay form of the selective scan), one
// thread per channel c = h P + p of head h, the channel's N states in registers:
//   dt = softplus(dtp[r][h] + dt_bias[h]);  a = exp(-rate[h] dt);  S[n] <- a S[n] + dt x[r][c] B[r][g][n];
//   y[r][c] = (sum_n S[n] C[r][g][n] + D[h] x[r][c]) * silu(z[r][c]),   g = h / hpg (heads per B / C group).
// x (row stride xs), bc rows (stride bs: B [G][N] | C [G][N]) and z (stride zs) have type TA; dtp (stride dts) is
// fp32; y [T][C] fp32.  state [slots][C][N].  EX picks the exponentials (DecayExp).  MODE 0 / 1 / 2 and the chunk
// arrays as in selective_scan_kernel; a chunk's decay is exp(-rate * sum dt), kept per (chunk, channel) in csd.
// VEC (fp32 inputs, N a multiple of 4, rows 16-byte aligned): B and C are read four states per load.
template <int NMAX, int MODE, typename TA, typename EX, bool VEC = false>
__global__ void __launch_bounds__(128) ssd_scan_kernel(const TA* __restrict__ x, int xs, const TA* __restrict__ bc, int bs,
                                                       const float* __restrict__ dtp, int dts,
                                                       const float* __restrict__ dt_bias, const float* __restrict__ rate,
                                                       const float* __restrict__ Dp, const TA* __restrict__ z, int zs,
                                                       float* __restrict__ state, const int* __restrict__ seg_row0,
                                                       const int* __restrict__ seg_pos0, const int* __restrict__ seg_slot,
                                                       float* __restrict__ y, int C, int N, int P, int hpg, int G,
                                                       const int* __restrict__ chunks, float* __restrict__ cs,
                                                       float* __restrict__ csd) {
  const int it = blockIdx.x, c = blockIdx.y * 128 + threadIdx.x;
  if (c >= C) return;
  int r0, r1;
  bool fresh;
  float* st;
  if (MODE == 0) {
    r0 = seg_row0[it];
    r1 = seg_row0[it + 1];
    fresh = seg_pos0[it] == 0;
    st = state + ((size_t)seg_slot[it] * C + c) * N;
  } else {
    r0 = chunks[it * 4 + 1];
    r1 = r0 + chunks[it * 4 + 2];
    fresh = MODE == 1;
    st = cs + ((size_t)it * C + c) * N;
  }
  const int h = c / P, g = h / hpg;
  float S[NMAX];
#pragma unroll
  for (int n = 0; n < NMAX; ++n) S[n] = (n < N && !fresh) ? st[n] : 0.f;
  const float Dc = Dp[h], bias = dt_bias[h], nrate = -rate[h] * EX::kPre;
  float sd = 0.f;
  for (int r = r0; r < r1; ++r) {
    const float dt = EX::softplus(dtp[(size_t)r * dts + h] + bias);
    const float a = EX::f(dt * nrate);
    const float xv = ldm(x, (size_t)r * xs + c);
    const float dx = dt * xv;
    const TA* Bp = bc + (size_t)r * bs + (size_t)g * N;
    const TA* Cp = Bp + (size_t)G * N;
    float acc = 0.f;
    sd += dt;
    if (VEC) {
      const f32x4* B4 = reinterpret_cast<const f32x4*>(Bp);
      const f32x4* C4 = reinterpret_cast<const f32x4*>(Cp);
#pragma unroll
      for (int n4 = 0; n4 < NMAX / 4; ++n4)
        if (4 * n4 < N) {
          const f32x4 b = B4[n4];
#pragma unroll
          for (int k = 0; k < 4; ++k) S[4 * n4 + k] = fmaf(a, S[4 * n4 + k], dx * b[k]);
          if (MODE != 1) {
            const f32x4 cv = C4[n4];
#pragma unroll
            for (int k = 0; k < 4; ++k) acc = fmaf(S[4 * n4 + k], cv[k], acc);
          }
        }
    } else {
#pragma unroll
      for (int n = 0; n < NMAX; ++n)
        if (n < N) {
          S[n] = fmaf(a, S[n], dx * ldm(Bp, n));
          if (MODE != 1) acc = fmaf(S[n], ldm(Cp, n), acc);
        }
    }
    if (MODE != 1) y[(size_t)r * C + c] = (acc + Dc * xv) * EX::silu(ldm(z, (size_t)r * zs + c));
  }
  if (MODE != 2) {
#pragma unroll
    for (int n = 0; n < NMAX; ++n)
      if (n < N) st[n] = S[n];
  }
  if (MODE == 1) csd[(size_t)it * C + c] = sd;
}

// Between the two chunk passes of ssd_scan_kernel: every chunk's end-from-zero state becomes its START state,
// the segment's final state goes to the slot (scan_carry_kernel with one decay per head).
template <int NMAX>
__global__ void __launch_bounds__(128) ssd_carry_kernel(const float* __restrict__ rate, float* __restrict__ state,
                                                        const int* __restrict__ seg_pos0, const int* __restrict__ seg_slot,
                                                        const int* __restrict__ seg_chunk0, float* __restrict__ cs,
                                                        const float* __restrict__ csd, int C, int N, int P) {
  const int sg = blockIdx.x, c = blockIdx.y * 128 + threadIdx.x;
  if (c >= C) return;
  float* st = state + ((size_t)seg_slot[sg] * C + c) * N;
  const bool fresh = seg_pos0[sg] == 0;
  const float nrate = -rate[c / P];
  float S[NMAX];
#pragma unroll
  for (int n = 0; n < NMAX; ++n) S[n] = (n < N && !fresh) ? st[n] : 0.f;
  for (int k = seg_chunk0[sg]; k < seg_chunk0[sg + 1]; ++k) {
    float* ck = cs + ((size_t)k * C + c) * N;
    const float a = expf(csd[(size_t)k * C + c] * nrate);
#pragma unroll
    for (int n = 0; n < NMAX; ++n)
      if (n < N) {
        const float loc = ck[n];
        ck[n] = S[n];
        S[n] = fmaf(a, S[n], loc);
      }
  }
#pragma unroll
  for (int n = 0; n < NMAX; ++n)
    if (n < N) st[n] = S[n];
}

// Retention in three kernels.  Rows of qkvg (fp32, stride qs): q [H][D] | k [H][D] | v [H][V] | g [H][V].
//   1. retention_rope_kernel (one workgroup per token, in place): q and k are rotated on their first
//      `rot` entries (entry i with i + rot / 2; angle = pos * base^(-2 i / rot), formed in double) and k is
//      scaled by D^(-1/2);
//   2. retention_scan_kernel, one workgroup per (segment, head, block of <= 32 value columns), tokens
//      in batches of 16 through LDS:  S <- decay S + k v^T;  o = S^T q  (fp32, written raw).
//      Thread (dg, v) of NDG x VBS owns S[d][v] for the DPT consecutive d from dg DPT (its q and k
//      entries are neighbours in LDS).  state [slots][H][D][V];
//   3. head_norm_gate_kernel: out = o / rms(o over the head's V) * silu(g).
__global__ void __launch_bounds__(256) retention_rope_kernel(float* __restrict__ qkvg, int qs,
                                                             const int* __restrict__ positions, int H, int D, int rot,
                                                             float base) {
  extern __shared__ float cs[];   // [half] cos | [half] sin
  const int r = blockIdx.x, tid = threadIdx.x, half = rot >> 1;
  float* row = qkvg + (size_t)r * qs;
  const double lb = log((double)base), p = (double)positions[r];
  for (int i = tid; i < half; i += 256) {
    const double ang = p * exp(-(double)(2 * i) / (double)rot * lb);
    cs[i] = (float)cos(ang);
    cs[half + i] = (float)sin(ang);
  }
  __syncthreads();
  const float ks = 1.f / sqrtf((float)D);
  for (int e = tid; e < 2 * H * half; e += 256) {        // the rotated pairs of q (first H heads) and k
    const int hd = e / half, i = e - hd * half;
    float* x = row + (size_t)hd * D;
    const float u = x[i], v = x[i + half], sc = hd >= H ? ks : 1.f;
    x[i] = (u * cs[i] - v * cs[half + i]) * sc;
    x[i + half] = (v * cs[i] + u * cs[half + i]) * sc;
  }
  const int rest = D - rot;
  for (int e = tid; e < H * rest; e += 256) {            // k's entries behind the rotated ones
    const int h = e / rest, i = e - h * rest;
    row[(size_t)(H + h) * D + rot + i] *= ks;
  }
}

constexpr int kRetTb = 16;    // tokens per batch
// MODE 0: blockIdx.x = segment, from the slot's state (or zero at position 0) to the slot's state.
// Long segments are cut into chunks ([n][4]: segment, first row, rows, -) that run in parallel:
// MODE 1: a chunk from a zero state, its end state goes to cs [chunks][H][D][V], no output;
// (retention_carry_kernel then turns cs into every chunk's START state and advances the slot's state)
// MODE 2: the chunk again from its start state, writing o.
template <int DPT, int MODE>
__global__ void __launch_bounds__(256) retention_scan_kernel(const float* __restrict__ qkvg, int qs,
                                                             const float* __restrict__ decay, float* __restrict__ state,
                                                             const int* __restrict__ seg_row0,
                                                             const int* __restrict__ seg_pos0,
                                                             const int* __restrict__ seg_slot, float* __restrict__ oraw,
                                                             int H, int D, int V, int VBS,
                                                             const int* __restrict__ chunks, float* __restrict__ cs) {
  extern __shared__ float sm[];
  const int it = blockIdx.x, hh = blockIdx.y, v0 = blockIdx.z * VBS, tid = threadIdx.x;
  const int NDG = 256 / VBS;
  float* sq = sm;                          // [TB][D]
  float* sk = sq + kRetTb * D;             // [TB][D]
  float* sv = sk + kRetTb * D;             // [TB][VBS]
  float* part = sv + kRetTb * VBS;         // [TB][NDG][VBS]
  const int v = tid % VBS, dg = tid / VBS;
  const bool own = dg < NDG && v0 + v < V;
  int r0, r1;
  bool fresh;
  float* st;
  if (MODE == 0) {
    r0 = seg_row0[it];
    r1 = seg_row0[it + 1];
    fresh = seg_pos0[it] == 0;
    st = state + ((size_t)seg_slot[it] * H + hh) * D * V + v0;
  } else {
    r0 = chunks[it * 4 + 1];
    r1 = r0 + chunks[it * 4 + 2];
    fresh = MODE == 1;
    st = cs + ((size_t)it * H + hh) * D * V + v0;
  }
  const float dec = decay[hh];
  float S[DPT];
#pragma unroll
  for (int i = 0; i < DPT; ++i) {
    const int d = dg * DPT + i;
    S[i] = (own && d < D && !fresh) ? st[(size_t)d * V + v] : 0.f;
  }
  for (int t0 = r0; t0 < r1; t0 += kRetTb) {
    const int nb = min(kRetTb, r1 - t0);
    __syncthreads();
    for (int e = tid; e < nb * D; e += 256) {
      const int tb = e / D, d = e - tb * D;
      const float* row = qkvg + (size_t)(t0 + tb) * qs;
      sq[e] = row[hh * D + d];
      sk[e] = row[(H + hh) * D + d];
    }
    for (int e = tid; e < nb * VBS; e += 256) {
      const int tb = e / VBS, vv = e - tb * VBS;
      sv[e] = v0 + vv < V ? qkvg[(size_t)(t0 + tb) * qs + 2 * H * D + hh * V + v0 + vv] : 0.f;
    }
    __syncthreads();
    if (dg < NDG) {
      for (int tb = 0; tb < nb; ++tb) {
        const float vv = sv[tb * VBS + v];
        const float* kq = sk + tb * D;
        const float* qq = sq + tb * D;
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < DPT; ++i) {
          const int d = dg * DPT + i;
          if (d < D) {
            S[i] = fmaf(dec, S[i], kq[d] * vv);
            if (MODE != 1) acc = fmaf(S[i], qq[d], acc);
          }
        }
        if (MODE != 1) part[(tb * NDG + dg) * VBS + v] = acc;
      }
    }
    if (MODE != 1) {
      __syncthreads();
      for (int e = tid; e < nb * VBS; e += 256) {
        const int tb = e / VBS, vv = e - tb * VBS;
        if (v0 + vv < V) {
          float o = 0.f;
          for (int g = 0; g < NDG; ++g) o += part[(tb * NDG + g) * VBS + vv];
          oraw[(size_t)(t0 + tb) * H * V + hh * V + v0 + vv] = o;
        }
      }
    }
  }
  if (MODE != 2) {
#pragma unroll
    for (int i = 0; i < DPT; ++i) {
      const int d = dg * DPT + i;
      if (own && d < D) st[(size_t)d * V + v] = S[i];
    }
  }
}

// Between the two chunk passes, one thread per state entry of a (segment, head): walk the segment's
// chunks, replace every chunk's end-from-zero state by its START state, leave the final state in the slot.
__global__ void __launch_bounds__(256) retention_carry_kernel(const float* __restrict__ decay, float* __restrict__ state,
                                                              const int* __restrict__ seg_pos0,
                                                              const int* __restrict__ seg_slot,
                                                              const int* __restrict__ seg_chunk0,
                                                              const int* __restrict__ chunks, float* __restrict__ cs,
                                                              int H, int DV) {
  const int sg = blockIdx.x, hh = blockIdx.y, e = blockIdx.z * 256 + threadIdx.x;
  if (e >= DV) return;
  float* st = state + ((size_t)seg_slot[sg] * H + hh) * DV + e;
  float S = seg_pos0[sg] == 0 ? 0.f : *st;
  const float dec = decay[hh];
  for (int k = seg_chunk0[sg]; k < seg_chunk0[sg + 1]; ++k) {
    float* ck = cs + ((size_t)k * H + hh) * DV + e;
    const int n = chunks[k * 4 + 2];
    float p = 1.f;
    for (int i = 0; i < n; ++i) p *= dec;
    const float loc = *ck;
    *ck = S;
    S = fmaf(p, S, loc);
  }
  *st = S;
}

// out[r][h] = o / sqrt(mean(o^2 over V) + eps) * silu(g): one wave per (row, head).
template <typename TA>
__global__ void __launch_bounds__(256) head_norm_gate_kernel(const float* __restrict__ oraw,
                                                             const float* __restrict__ gate, int gs,
                                                             TA* __restrict__ out, int n_rh, int H, int V, float eps) {
  const int rh = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (rh >= n_rh) return;
  const int r = rh / H, h = rh - r * H;
  const float* o = oraw + (size_t)rh * V;
  float ss = 0.f;
  for (int c = lane; c < V; c += 64) ss = fmaf(o[c], o[c], ss);
  const float rn = 1.f / sqrtf(wave_sum(ss) / (float)V + eps);
  const float* g = gate + (size_t)r * gs + (size_t)h * V;
  for (int c = lane; c < V; c += 64) stm(out, (size_t)rh * V + c, o[c] * rn * silu_f(g[c]));
}

}  // namespace k8s

using namespace k8s;

#define K8S_MDT(dt, ...)   \
  if ((dt) == 0) {          \
    using TA = uint16_t;    \
    __VA_ARGS__;            \
  } else {                  \
    using TA = float;       \
    __VA_ARGS__;            \
  }

K8S_API int k8s_short_conv(const void* x, int xs, int xdt, const float* w, const float* b, float* tail,
                           const int* row_seg, const int* seg_row0, const int* seg_pos0, const int* seg_slot,
                           void* out, int T, int n_seg, int C, int taps, int act, int odt, hipStream_t s,
                           const int* items, int n_items) {
  if (T <= 0) return 0;
  if (taps < 1 || taps > 16 || xdt != odt) return (int)hipErrorInvalidValue;
  const dim3 g1(T, (C + 255) / 256), g2(n_seg, (C + 255) / 256);
  const bool tiles = items != nullptr && n_items > 0 && taps >= 2 && taps <= 4;
  const dim3 gt(n_items > 0 ? n_items : 1, (C + 255) / 256);
#define K8S_CONV_T(TP)                                                                                          \
  hipLaunchKernelGGL((short_conv_tile_kernel<TP, TA>), gt, dim3(256), 0, s, (const TA*)x, xs, w, b, tail, items, \
                     seg_row0, seg_pos0, seg_slot, (TA*)out, C, act)
  K8S_MDT(odt, {
    if (tiles && taps == 2) {
      K8S_CONV_T(2);
    } else if (tiles && taps == 3) {
      K8S_CONV_T(3);
    } else if (tiles) {
      K8S_CONV_T(4);
    } else {
      hipLaunchKernelGGL((short_conv_kernel<TA>), g1, dim3(256), 0, s, (const TA*)x, xs, w, b, tail, row_seg, seg_row0,
                         seg_pos0, seg_slot, (TA*)out, C, taps, act);
    }
    if (taps > 1)
      hipLaunchKernelGGL((short_conv_tail_kernel<TA>), g2, dim3(256), 0, s, (const TA*)x, xs, tail, seg_row0,
                         seg_pos0, seg_slot, C, taps);
  });
#undef K8S_CONV_T
  return (int)hipGetLastError();
}

K8S_API int k8s_selective_scan(const void* xc, int dt, const float* dtp, const float* dt_bias, const float* dbc,
                               int ds, int R, const float* A, const float* D, const void* z, int zs, float* state,
                               const int* seg_row0, const int* seg_pos0, const int* seg_slot, void* y, int n_seg,
                               int C, int N, int T, hipStream_t s, const int* chunks, int n_chunks,
                               const int* seg_chunk0, float* cs, float* csd) {
  if (T <= 0 || n_seg <= 0) return 0;
  if (N < 1 || N > 128) return (int)hipErrorInvalidValue;
  const int cb = (C + 127) / 128;
#define K8S_SCAN_M(NM, MODE, items)                                                                               \
  K8S_MDT(dt, hipLaunchKernelGGL((selective_scan_kernel<NM, MODE, TA>), dim3(items, cb), dim3(128), 0, s,          \
                                 (const TA*)xc, dtp, dt_bias, dbc, ds, R, A, D, (const TA*)z, zs, state, seg_row0, \
                                 seg_pos0, seg_slot, (TA*)y, C, N, chunks, cs, csd))
#define K8S_SCAN(NM)                                                                                              \
  if (chunks == nullptr) {                                                                                        \
    K8S_SCAN_M(NM, 0, n_seg);                                                                                     \
  } else {                                                                                                        \
    K8S_SCAN_M(NM, 1, n_chunks);                                                                                  \
    hipLaunchKernelGGL((scan_carry_kernel<NM>), dim3(n_seg, cb), dim3(128), 0, s, A, state, seg_pos0, seg_slot,   \
                       seg_chunk0, cs, csd, C, N);                                                                \
    K8S_SCAN_M(NM, 2, n_chunks);                                                                                  \
  }
  if (N <= 16) {
    K8S_SCAN(16)
  } else if (N <= 32) {
    K8S_SCAN(32)
  } else if (N <= 64) {
    K8S_SCAN(64)
  } else {
    K8S_SCAN(128)
  }
#undef K8S_SCAN
#undef K8S_SCAN_M
  return (int)hipGetLastError();
}

// fast != 0: the hardware exponentials (DecayExp<uint16_t>), else expf / log1pf.  dt: the type of x, bc and z.
K8S_API int k8s_ssd_scan(const void* x, int xs, const void* bc, int bs, int dt, const float* dtp, int dts,
                         const float* dt_bias, const float* rate, const float* D, const void* z, int zs, float* state,
                         const int* seg_row0, const int* seg_pos0, const int* seg_slot, float* y, int n_seg, int H,
                         int P, int G, int N, int T, int fast, hipStream_t s, const int* chunks, int n_chunks,
                         const int* seg_chunk0, float* cs, float* csd) {
  if (T <= 0 || n_seg <= 0) return 0;
  if (N < 1 || N > 128 || H < 1 || P < 1 || G < 1 || H % G) return (int)hipErrorInvalidValue;
  const int C = H * P, cb = (C + 127) / 128, hpg = H / G;
  const bool vec = dt == 1 && N % 4 == 0 && bs % 4 == 0 && ((uintptr_t)bc & 15) == 0;
#define K8S_SSD_E(NM, MODE, items, EX)                                                                            \
  if (vec) {                                                                                                      \
    hipLaunchKernelGGL((ssd_scan_kernel<NM, MODE, float, EX, true>), dim3(items, cb), dim3(128), 0, s,            \
                       (const float*)x, xs, (const float*)bc, bs, dtp, dts, dt_bias, rate, D, (const float*)z, zs, \
                       state, seg_row0, seg_pos0, seg_slot, y, C, N, P, hpg, G, chunks, cs, csd);                 \
  } else {                                                                                                        \
    K8S_MDT(dt, hipLaunchKernelGGL((ssd_scan_kernel<NM, MODE, TA, EX>), dim3(items, cb), dim3(128), 0, s,         \
                                   (const TA*)x, xs, (const TA*)bc, bs, dtp, dts, dt_bias, rate, D, (const TA*)z, \
                                   zs, state, seg_row0, seg_pos0, seg_slot, y, C, N, P, hpg, G, chunks, cs, csd)) \
  }
#define K8S_SSD_M(NM, MODE, items)                \
  if (fast) {                                     \
    K8S_SSD_E(NM, MODE, items, DecayExp<uint16_t>) \
  } else {                                        \
    K8S_SSD_E(NM, MODE, items, DecayExp<float>)   \
  }
#define K8S_SSD(NM)                                                                                             \
  if (chunks == nullptr) {                                                                                      \
    K8S_SSD_M(NM, 0, n_seg)                                                                                     \
  } else {                                                                                                      \
    K8S_SSD_M(NM, 1, n_chunks)                                                                                  \
    hipLaunchKernelGGL((ssd_carry_kernel<NM>), dim3(n_seg, cb), dim3(128), 0, s, rate, state, seg_pos0, seg_slot, \
                       seg_chunk0, cs, csd, C, N, P);                                                           \
    K8S_SSD_M(NM, 2, n_chunks)                                                                                  \
  }
  if (N <= 16) {
    K8S_SSD(16)
  } else if (N <= 32) {
    K8S_SSD(32)
  } else if (N <= 64) {
    K8S_SSD(64)
  } else {
    K8S_SSD(128)
  }
#undef K8S_SSD
#undef K8S_SSD_M
#undef K8S_SSD_E
  return (int)hipGetLastError();
}

K8S_API int k8s_retention(float* qkvg, int qs, const int* positions, const float* decay, float* state,
                          const int* seg_row0, const int* seg_pos0, const int* seg_slot, void* out, int n_seg, int H,
                          int D, int V, int rot, float base, float eps, int odt, hipStream_t s, int T, float* oraw,
                          const int* chunks, int n_chunks, const int* seg_chunk0, float* cs) {
  if (n_seg <= 0 || T <= 0) return 0;
  if (V < 1 || rot < 0 || rot > D || (rot & 1)) return (int)hipErrorInvalidValue;
  const int VBS = V < 32 ? V : 32, NDG = 256 / VBS, dpt = (D + NDG - 1) / NDG;
  if (dpt > 64) return (int)hipErrorInvalidValue;
  const size_t lds = (size_t)kRetTb * (2 * D + VBS + NDG * VBS) * sizeof(float);
  if (lds > 160 * 1024 || (size_t)rot * sizeof(float) > 64 * 1024) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(retention_rope_kernel, dim3(T), dim3(256), rot * sizeof(float) + 8, s, qkvg, qs, positions, H, D,
                     rot, base);
  const int vb = (V + VBS - 1) / VBS;
#define K8S_RET_M(DP, MODE, items)                                                                              \
  {                                                                                                             \
    auto k = retention_scan_kernel<DP, MODE>;                                                                   \
    if (lds > 48 * 1024 && hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)) \
      return (int)hipGetLastError();                                                                            \
    hipLaunchKernelGGL(k, dim3(items, H, vb), dim3(256), lds, s, qkvg, qs, decay, state, seg_row0, seg_pos0,    \
                       seg_slot, oraw, H, D, V, VBS, chunks, cs);                                               \
  }
#define K8S_RET(DP)                                                                                             \
  if (chunks == nullptr) {                                                                                      \
    K8S_RET_M(DP, 0, n_seg)                                                                                     \
  } else {                                                                                                      \
    K8S_RET_M(DP, 1, n_chunks)                                                                                  \
    hipLaunchKernelGGL(retention_carry_kernel, dim3(n_seg, H, (D * V + 255) / 256), dim3(256), 0, s, decay, state, \
                       seg_pos0, seg_slot, seg_chunk0, chunks, cs, H, D * V);                                   \
    K8S_RET_M(DP, 2, n_chunks)                                                                                  \
  }
  if (dpt <= 4) {
    K8S_RET(4)
  } else if (dpt <= 8) {
    K8S_RET(8)
  } else if (dpt <= 16) {
    K8S_RET(16)
  } else if (dpt <= 32) {
    K8S_RET(32)
  } else {
    K8S_RET(64)
  }
#undef K8S_RET
#undef K8S_RET_M
  const int n_rh = T * H;
  K8S_MDT(odt, hipLaunchKernelGGL((head_norm_gate_kernel<TA>), dim3((n_rh + 3) / 4), dim3(256), 0, s, oraw,
                                  qkvg + 2 * H * D + H * V, qs, (TA*)out, n_rh, H, V, eps));
  return (int)hipGetLastError();
}
