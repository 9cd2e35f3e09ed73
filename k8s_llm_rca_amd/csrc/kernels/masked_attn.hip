// Softmax attention over a paged key / value cache under a position mask, behind a pass that prepares
// q and k.
//
// attn_prep:  rows of the joint projection (fp32: q [H][D] | k [G][D] | v [G][V], row stride qs)
//   + bias;  q, k rotated on their first `rot` entries per head (entry i with i + rot / 2, angle
//   pos * base^(-2 i / rot), formed in double);  q, k divided by the head's root mean square (eps inside the
//   root) and multiplied by a weight [D] where given;  v optionally kept as projected (v_keep) and mixed
//   with another layer's values of the same token, (1 - lam) v + lam v_other;  k and v written to their pages
//   (and v to the transposed twin), q written as activations.
//
// masked attention:  position i sees j <= i with  (chunk > 0:  i / chunk == j / chunk)  and
//   (window > 0:  i - j < window  or  j < keep_first).  s = scale q.k, then softcap tanh(s / softcap) for
//   softcap > 0.  A sink adds exp(sink_h) to head h's denominator.  Head h's output may be multiplied by
//   sigmoid(gate[t][h]).  Query head h reads key / value head h / (H / G).
//   The visible keys of a row are two runs, [a0, a1) (kept first tokens) and [lo, pos]; both kernels walk
//   them as one virtual range whose tile borders depend on the row's position only, so a row's result
//   does not depend on how the prompt was cut or on what else is in the step.
//
// Pages: kc [pages][BS][G D], vc [pages][BS][G V], vt [pages][G V][BS]; a token's slot = page * BS + offset.
// Scores, weights and accumulation are fp32; TA (bf16 as uint16_t, or float) is the type of q, the pages
// and the output.
#include "common.h"

namespace k8s {

template <typename T>
__device__ __forceinline__ float lda(const T* p, size_t i);
template <>
__device__ __forceinline__ float lda<float>(const float* p, size_t i) { return p[i]; }
template <>
__device__ __forceinline__ float lda<uint16_t>(const uint16_t* p, size_t i) { return bf2f(p[i]); }
template <typename T>
__device__ __forceinline__ void sta(T* p, size_t i, float v);
template <>
__device__ __forceinline__ void sta<float>(float* p, size_t i, float v) { p[i] = v; }
template <>
__device__ __forceinline__ void sta<uint16_t>(uint16_t* p, size_t i, float v) { p[i] = f2bf(v); }

constexpr int kPrepPer = 8;    // entries of a head per lane: D <= 512

template <typename TA>
__global__ void __launch_bounds__(256) attn_prep_kernel(const float* __restrict__ qkv, int qs,
                                                        const float* __restrict__ bias, int H, int G, int D, int V,
                                                        const int* __restrict__ positions,
                                                        const int* __restrict__ slots, TA* __restrict__ kc,
                                                        TA* __restrict__ vc, TA* __restrict__ vt, int BS,
                                                        TA* __restrict__ q_out, int norm, const float* __restrict__ q_w,
                                                        const float* __restrict__ k_w, float eps, int rot, float base,
                                                        float lam, const float* __restrict__ v_other,
                                                        float* __restrict__ v_keep) {
  extern __shared__ float sm[];   // [rot]: cos | sin;  [4][D]: one head per wave
  const int r = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int half = rot >> 1;
  float* cs = sm;
  float* buf = sm + rot + wv * D;
  if (rot) {
    const double lb = log((double)base), p = (double)positions[r];
    for (int i = tid; i < half; i += 256) {
      const double ang = p * exp(-(double)(2 * i) / (double)rot * lb);
      cs[i] = (float)cos(ang);
      cs[half + i] = (float)sin(ang);
    }
  }
  const int sl = slots[r];
  const int NQ = H * D, NK = G * D, NV = G * V, units = H + G;
  const float* row = qkv + (size_t)r * qs;
  for (int u0 = 0; u0 < units; u0 += 4) {      // every wave takes the same number of turns (barriers inside)
    const int u = u0 + wv;
    if (u < units)
      for (int d = lane; d < D; d += 64) buf[d] = row[u * D + d] + (bias ? bias[u * D + d] : 0.f);
    __syncthreads();
    if (u < units) {
      float val[kPrepPer];
      float ss = 0.f;
#pragma unroll
      for (int i = 0; i < kPrepPer; ++i) {
        const int d = lane + 64 * i;
        float xv = 0.f;
        if (d < D) {
          xv = buf[d];
          if (d < half) {
            xv = xv * cs[d] - buf[d + half] * cs[half + d];
          } else if (d < rot) {
            const int j = d - half;
            xv = xv * cs[j] + buf[j] * cs[half + j];
          }
        }
        val[i] = xv;
        ss = fmaf(xv, xv, ss);
      }
      float rn = 1.f;
      if (norm) rn = 1.f / sqrtf(wave_sum(ss) / (float)D + eps);
      const float* wgt = u < H ? q_w : k_w;
#pragma unroll
      for (int i = 0; i < kPrepPer; ++i) {
        const int d = lane + 64 * i;
        if (d < D) {
          const float o = val[i] * rn * (wgt ? wgt[d] : 1.f);
          if (u < H)
            sta(q_out, (size_t)r * NQ + u * D + d, o);
          else if (sl >= 0)
            sta(kc, (size_t)sl * NK + (u - H) * D + d, o);
        }
      }
    }
    __syncthreads();
  }
  const int page = sl >= 0 ? sl / BS : 0, off = sl >= 0 ? sl - page * BS : 0;
  for (int c = tid; c < NV; c += 256) {
    float v = row[NQ + NK + c] + (bias ? bias[NQ + NK + c] : 0.f);
    if (v_keep) v_keep[(size_t)r * NV + c] = v;
    if (v_other) v = (1.f - lam) * v + lam * v_other[(size_t)r * NV + c];
    if (sl >= 0) {
      sta(vc, (size_t)sl * NV + c, v);
      if (vt) sta(vt, ((size_t)page * NV + c) * BS + off, v);
    }
  }
}

// The visible keys of position `pos`: [a0, a1) and [lo, pos], walked as x in [0, nA + nB).
struct KeyRuns {
  int a0, nA, lo, total;
  __device__ __forceinline__ int key(int x) const { return x < nA ? a0 + x : lo + (x - nA); }
};

__device__ __forceinline__ KeyRuns key_runs(int pos, int chunk, int window, int keep_first) {
  KeyRuns k;
  k.a0 = chunk > 0 ? (pos / chunk) * chunk : 0;
  k.lo = k.a0;
  k.nA = 0;
  if (window > 0) {
    k.lo = max(k.a0, pos - window + 1);
    k.nA = max(0, min(keep_first, k.lo) - k.a0);
  }
  k.total = k.nA + pos - k.lo + 1;
  return k;
}

constexpr int kMaskTile = 64;   // keys per tile: one per lane
constexpr int kMaskOut = 16;    // outputs per thread: H * V <= 256 * kMaskOut

template <typename TA>
__device__ __forceinline__ float mask_score(const float* q, const TA* __restrict__ kc, const int* __restrict__ bt, int BS,
                                            int NK, int D, int g, int j, float scale, float softcap) {
  const TA* kr = kc + ((size_t)bt[j / BS] * BS + (j % BS)) * NK + (size_t)g * D;
  float a = 0.f;
  for (int d = 0; d < D; ++d) a = fmaf(q[d], lda(kr, d), a);
  a *= scale;
  return softcap > 0.f ? softcap * tanhf(a / softcap) : a;
}

// One workgroup per row, two passes over the row's visible keys in tiles of 64:
//   1. per head the maximum (the sink included) and the denominator, online (a wave per head);
//   2. scores again -> weights in LDS -> times the values (a thread per output column).
template <typename TA>
__global__ void __launch_bounds__(256) masked_attn_rows_kernel(const TA* __restrict__ q, const TA* __restrict__ kc,
                                                               const TA* __restrict__ vc,
                                                               const int* __restrict__ block_tables, int maxb,
                                                               const int* __restrict__ row_seg,
                                                               const int* __restrict__ seg_row0,
                                                               const int* __restrict__ seg_pos0,
                                                               const float* __restrict__ sink,
                                                               const float* __restrict__ gate, int gs,
                                                               TA* __restrict__ out, int H, int G, int D, int V, int BS,
                                                               int chunk, int window, int keep_first, float scale,
                                                               float softcap) {
  extern __shared__ float sm[];
  float* qf = sm;                      // [H][D]
  float* p = qf + H * D;               // [H][64]
  float* mh = p + H * kMaskTile;       // [H]
  float* lh = mh + H;                  // [H]
  const int r = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int sg = row_seg[r], pos = seg_pos0[sg] + r - seg_row0[sg];
  const KeyRuns kr = key_runs(pos, chunk, window, keep_first);
  const int* bt = block_tables + (size_t)sg * maxb;
  const int NK = G * D, NV = G * V, hpg = H / G;
  for (int i = tid; i < H * D; i += 256) qf[i] = lda(q, (size_t)r * H * D + i);
  __syncthreads();
  for (int h = wv; h < H; h += 4) {
    const int g = h / hpg;
    float m = sink ? sink[h] : -INFINITY, l = sink ? 1.f : 0.f;
    for (int x0 = 0; x0 < kr.total; x0 += kMaskTile) {
      const int x = x0 + lane;
      const bool ok = x < kr.total;
      const float s = ok ? mask_score(qf + h * D, kc, bt, BS, NK, D, g, kr.key(x), scale, softcap) : -INFINITY;
      const float mn = fmaxf(m, wave_max(s));     // finite: every tile holds a visible key
      l = l * expf(m - mn) + wave_sum(ok ? expf(s - mn) : 0.f);
      m = mn;
    }
    if (lane == 0) {
      mh[h] = m;
      lh[h] = l;
    }
  }
  __syncthreads();
  float acc[kMaskOut];
#pragma unroll
  for (int i = 0; i < kMaskOut; ++i) acc[i] = 0.f;
  for (int x0 = 0; x0 < kr.total; x0 += kMaskTile) {
    for (int h = wv; h < H; h += 4) {
      const int x = x0 + lane;
      const bool ok = x < kr.total;
      const float s = ok ? mask_score(qf + h * D, kc, bt, BS, NK, D, h / hpg, kr.key(x), scale, softcap) : 0.f;
      p[h * kMaskTile + lane] = ok ? expf(s - mh[h]) / lh[h] : 0.f;
    }
    __syncthreads();
    const int nk = min(kMaskTile, kr.total - x0);
#pragma unroll
    for (int i = 0; i < kMaskOut; ++i) {
      const int o = tid + i * 256;
      if (o < H * V) {
        const int h = o / V, v = o - h * V, g = h / hpg;
        float a = acc[i];
        for (int jj = 0; jj < nk; ++jj) {
          const int j = kr.key(x0 + jj);
          a = fmaf(p[h * kMaskTile + jj], lda(vc, ((size_t)bt[j / BS] * BS + (j % BS)) * NV + (size_t)g * V + v), a);
        }
        acc[i] = a;
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < kMaskOut; ++i) {
    const int o = tid + i * 256;
    if (o < H * V) {
      float a = acc[i];
      if (gate) a *= 1.f / (1.f + expf(-gate[(size_t)r * gs + o / V]));
      sta(out, (size_t)r * H * V + o, a);
    }
  }
}

}  // namespace k8s

using namespace k8s;

K8S_API int k8s_attn_prep(const float* qkv, int qs, const float* bias, int H, int G, int D, int V, const int* positions,
                          const int* slots, void* kc, void* vc, void* vt, int BS, void* q_out, int dt, int norm,
                          const float* q_w, const float* k_w, float eps, int rot, float base, float lam,
                          const float* v_other, float* v_keep, int T, hipStream_t s) {
  if (T <= 0) return 0;
  if (H < 1 || G < 1 || D < 1 || D > 64 * kPrepPer || V < 1 || rot < 0 || rot > D || (rot & 1) || BS < 1)
    return (int)hipErrorInvalidValue;
  const size_t lds = (size_t)(rot + 4 * D) * sizeof(float);
  if (dt == 0)
    hipLaunchKernelGGL((attn_prep_kernel<uint16_t>), dim3(T), dim3(256), lds, s, qkv, qs, bias, H, G, D, V, positions,
                       slots, (uint16_t*)kc, (uint16_t*)vc, (uint16_t*)vt, BS, (uint16_t*)q_out, norm, q_w, k_w, eps, rot,
                       base, lam, v_other, v_keep);
  else
    hipLaunchKernelGGL((attn_prep_kernel<float>), dim3(T), dim3(256), lds, s, qkv, qs, bias, H, G, D, V, positions, slots,
                       (float*)kc, (float*)vc, (float*)vt, BS, (float*)q_out, norm, q_w, k_w, eps, rot, base, lam,
                       v_other, v_keep);
  return (int)hipGetLastError();
}

K8S_API int k8s_masked_attn_rows(const void* q, const void* kc, const void* vc, const int* block_tables, int maxb,
                                 const int* row_seg, const int* seg_row0, const int* seg_pos0, const float* sink,
                                 const float* gate, int gs, void* out, int T, int H, int G, int D, int V, int BS,
                                 int chunk, int window, int keep_first, float scale, float softcap, int dt,
                                 hipStream_t s) {
  if (T <= 0) return 0;
  const size_t lds = (size_t)(H * D + H * kMaskTile + 2 * H) * sizeof(float);
  if (H < 1 || G < 1 || H % G || H * V > 256 * kMaskOut || chunk < 0 || window < 0 || keep_first < 0 ||
      lds > 64 * 1024)
    return (int)hipErrorInvalidValue;
  if (dt == 0)
    hipLaunchKernelGGL((masked_attn_rows_kernel<uint16_t>), dim3(T), dim3(256), lds, s, (const uint16_t*)q,
                       (const uint16_t*)kc, (const uint16_t*)vc, block_tables, maxb, row_seg, seg_row0, seg_pos0, sink,
                       gate, gs, (uint16_t*)out, H, G, D, V, BS, chunk, window, keep_first, scale, softcap);
  else
    hipLaunchKernelGGL((masked_attn_rows_kernel<float>), dim3(T), dim3(256), lds, s, (const float*)q, (const float*)kc,
                       (const float*)vc, block_tables, maxb, row_seg, seg_row0, seg_pos0, sink, gate, gs, (float*)out, H,
                       G, D, V, BS, chunk, window, keep_first, scale, softcap);
  return (int)hipGetLastError();
}
