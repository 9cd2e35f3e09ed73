// Softmax attention over a paged key / value cache under a position mask, behind a pass that prepares
// q and k.
//
// attn_prep:  rows of the joint projection (fp32: q [H][D] | k [G][D] | v [NV], row stride qs)
//   + bias;  q, k rotated on their first `rot` entries per head (entry i with i + rot / 2, angle
//   pos * base^(-2 i / rot), formed in double);  norm 1: q, k divided by the head's root mean square (eps inside
//   the root) behind the rotation and multiplied by a weight [D] where given;  norm 2: q and k each divided by
//   the root mean square of the WHOLE projection (all heads at once) and multiplied by a weight of that size,
//   in front of the rotation;  q multiplied by the position's temperature 1 + tq_coef ln(floor((pos + 1) /
//   tq_every) + 1) (tq_every > 0);  v optionally kept as projected (v_keep) and mixed with another layer's
//   values of the same token, (1 - lam) v + lam v_other;  k and v written to their pages (and v to the
//   transposed twin), q written as activations.  The values start at column v_col of the row: behind the
//   keys, or AT the keys (the values are the keys as projected).  G = 0: a layer that reads another layer's
//   pages prepares its queries only.  H and G count heads of D entries: a layer with several score maps per
//   head passes maps * heads.
//
// masked attention:  position i sees j <= i with  (chunk > 0:  i / chunk == j / chunk)  and
//   (window > 0:  i - j < window  or  j < keep_first).  s = scale q.k, then softcap tanh(s / softcap) for
//   softcap > 0.  A sink adds exp(sink_h) to head h's denominator.  Head h's output may be multiplied by
//   sigmoid(gate[t][h]).  Query head h reads key / value head h / (H / G).  With M > 1 score maps per head, q
//   holds H M heads laid out [h][m] and the key pages G M heads [g][m]: map m of head h scores against key
//   head (h / (H / G)) M + m and applies its weights to value head h / (H / G); the output is [T][H][M][V],
//   each map's result by itself (fp32 where the caller joins the maps).
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
                                                        const float* __restrict__ bias, int H, int G, int D, int NV,
                                                        const int* __restrict__ positions,
                                                        const int* __restrict__ slots, TA* __restrict__ kc,
                                                        TA* __restrict__ vc, TA* __restrict__ vt, int BS,
                                                        TA* __restrict__ q_out, int norm, const float* __restrict__ q_w,
                                                        const float* __restrict__ k_w, float eps, int rot, float base,
                                                        float lam, const float* __restrict__ v_other,
                                                        float* __restrict__ v_keep, int upr, int v_col, float tq_coef,
                                                        int tq_every) {
  extern __shared__ float sm[];   // [rot]: cos | sin;  [upr][D]: the heads of one round
  __shared__ float red[16];
  const int r = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int half = rot >> 1;
  float* cs = sm;
  if (rot) {
    const double lb = log((double)base), p = (double)positions[r];
    for (int i = tid; i < half; i += 256) {
      const double ang = p * exp(-(double)(2 * i) / (double)rot * lb);
      cs[i] = (float)cos(ang);
      cs[half + i] = (float)sin(ang);
    }
  }
  const int sl = slots[r];
  const int NQ = H * D, NK = G * D, units = H + G;
  const float* row = qkv + (size_t)r * qs;
  const float tq = tq_every > 0 ? 1.f + tq_coef * logf((float)((positions[r] + 1) / tq_every) + 1.f) : 1.f;
  // norm 2: 1 / rms of the whole q and of the whole k projection
  float rq = 1.f, rk = 1.f;
  if (norm == 2) {
    float sq = 0.f, sk = 0.f;
    for (int i = tid; i < NQ; i += 256) {
      const float v = row[i] + (bias ? bias[i] : 0.f);
      sq = fmaf(v, v, sq);
    }
    for (int i = tid; i < NK; i += 256) {
      const float v = row[NQ + i] + (bias ? bias[NQ + i] : 0.f);
      sk = fmaf(v, v, sk);
    }
    rq = 1.f / sqrtf(block_sum(sq, red) / (float)NQ + eps);
    if (NK) rk = 1.f / sqrtf(block_sum(sk, red) / (float)NK + eps);
  }
  // rounds of upr heads (all of the row's q and k heads where LDS holds them: one barrier pair per row):
  // the round's heads are loaded, then every wave works on its own
  for (int u0 = 0; u0 < units; u0 += upr) {
    const int u1 = min(units, u0 + upr);
    for (int u = u0 + wv; u < u1; u += 4) {
      float* buf = sm + rot + (u - u0) * D;
      for (int d = lane; d < D; d += 64) {
        float v = row[u * D + d] + (bias ? bias[u * D + d] : 0.f);
        if (norm == 2) v *= u < H ? rq * (q_w ? q_w[u * D + d] : 1.f) : rk * (k_w ? k_w[(u - H) * D + d] : 1.f);
        buf[d] = v;
      }
    }
    __syncthreads();
    for (int u = u0 + wv; u < u1; u += 4) {
      const float* buf = sm + rot + (u - u0) * D;
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
      if (norm == 1) rn = 1.f / sqrtf(wave_sum(ss) / (float)D + eps);
      const float* wgt = norm == 1 ? (u < H ? q_w : k_w) : nullptr;
      if (u < H) rn *= tq;
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
    if (u1 < units) __syncthreads();
  }
  const int page = sl >= 0 ? sl / BS : 0, off = sl >= 0 ? sl - page * BS : 0;
  for (int c = tid; c < NV; c += 256) {
    float v = row[v_col + c] + (bias ? bias[v_col + c] : 0.f);
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
constexpr int kMaskOut = 32;    // outputs per thread: H * V <= 256 * kMaskOut

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
template <typename TA, typename TO>
__global__ void __launch_bounds__(256) masked_attn_rows_kernel(const TA* __restrict__ q, const TA* __restrict__ kc,
                                                               const TA* __restrict__ vc,
                                                               const int* __restrict__ block_tables, int maxb,
                                                               const int* __restrict__ row_seg,
                                                               const int* __restrict__ seg_row0,
                                                               const int* __restrict__ seg_pos0,
                                                               const float* __restrict__ sink,
                                                               const float* __restrict__ gate, int gs,
                                                               TO* __restrict__ out, int H, int G, int D, int V, int BS,
                                                               int chunk, int window, int keep_first, float scale,
                                                               float softcap, int M) {
  // H counts the query heads of D entries (heads x maps); hpg of them share a key / value head group
  extern __shared__ float sm[];
  float* qf = sm;                      // [H][D]
  float* p = qf + H * D;               // [H][64]
  float* mh = p + H * kMaskTile;       // [H]
  float* lh = mh + H;                  // [H]
  const int r = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int sg = row_seg[r], pos = seg_pos0[sg] + r - seg_row0[sg];
  const KeyRuns kr = key_runs(pos, chunk, window, keep_first);
  const int* bt = block_tables + (size_t)sg * maxb;
  const int NK = G * M * D, NV = G * V, hpg = H / (G * M);
  for (int i = tid; i < H * D; i += 256) qf[i] = lda(q, (size_t)r * H * D + i);
  __syncthreads();
  for (int h = wv; h < H; h += 4) {
    const int g = (h / M / hpg) * M + h % M;
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
      const float s =
          ok ? mask_score(qf + h * D, kc, bt, BS, NK, D, (h / M / hpg) * M + h % M, kr.key(x), scale, softcap) : 0.f;
      p[h * kMaskTile + lane] = ok ? expf(s - mh[h]) / lh[h] : 0.f;
    }
    __syncthreads();
    const int nk = min(kMaskTile, kr.total - x0);
#pragma unroll
    for (int i = 0; i < kMaskOut; ++i) {
      const int o = tid + i * 256;
      if (o < H * V) {
        const int h = o / V, v = o - h * V, g = h / M / hpg;
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
      sta(out, (size_t)r * H * V + o, a);   // (gates count heads x maps like H)
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Matrix-core form (bf16, v_mfma_f32_16x16x32_bf16), one pass with an online softmax.  A work item is a
// tile of up to 16 consecutive tokens of one segment; wave w of workgroup (item, y) owns the heads
// (8 y + w) HW .. + HW - 1 and shares nothing with the other waves (no LDS, no barrier).  Keys go in
// blocks of 32 that never cross a page (BS % 32 == 0): first the blocks that hold kept first tokens, then
// the blocks from the first token's window / chunk start to the tile's last position; the exact mask is
// applied per (query, key).  Swapped QK^T as in the other attention kernels: a lane owns ONE query
// (lane & 15) and per block the scores of keys 8 q .. 8 q + 7 of its quarter q = lane >> 4, which is the
// layout of the PV product's first operand, so the weights go from accumulator to operand in place.
// The output accumulator's rows are the queries 4 q + i: their rescaling factors come from the lanes
// that own those queries by a cross-lane read.
struct MaskArgs {
  const uint16_t* q;      // [T][H * D]
  const uint16_t* kc;     // [pages][BS][G * D]
  const uint16_t* vt;     // [pages][G * V][BS]
  const int* bt;
  int maxb;
  const int* items;       // [n][4]: segment, first row, tokens (<= 16), position of the first token
  int n_items;
  const float* sink;      // [H] or null
  const float* gate;      // [T] rows of stride gs, column h, or null
  int gs;
  uint16_t* out;          // [T][H * V]
  float* out32;           // the same in fp32 instead, where the caller joins score maps
  int H, G, M, BS, chunk, window, keep_first;   // H: query heads of D entries (heads x M maps)
  float scale, softcap;
  // steps of few rows: a tile's key blocks are split over grid.z workgroups, part_blocks blocks each
  int part_blocks, n_parts;
  float* pml;             // [items][parts][H][16][2]: a part's maximum (log2 units) and denominator
  float* po;              // [items][parts][16][H * V]: a part's unnormalised output
};

__device__ __forceinline__ bf16x8 mld16(const uint16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }

// SPLIT: workgroup z walks the blocks [z part_blocks, (z + 1) part_blocks) of its tile and leaves its maximum,
// denominator and unnormalised output; masked_attn_merge_kernel joins the parts (and adds the sink).  Part
// borders count blocks of the tile's own block list, so they depend on positions only.
// KH = 2 (two score maps per head, HW = 2): the wave's two query heads are the two maps of ONE head; each has its
// own key head (its own key fragments) and both apply their weights to the same value fragments.
template <int NDC, int NV, int HW, bool CAP, bool SPLIT, int KH = 1>
__global__ void __launch_bounds__(512) masked_attn_mfma_kernel(MaskArgs a) {
  constexpr int D = NDC * 32, V = NV * 16;
  constexpr float kLog2e = 1.4426950408889634f;
  const int lane = threadIdx.x & 63, r = lane & 15, hq = lane >> 4;
  const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // tiles are listed by position within their segments and a later tile mostly has more keys: the
  // last ones start first, so the launch does not end on its longest items
  const int item = a.n_items - 1 - blockIdx.x;
  const int sg = a.items[item * 4], row0 = a.items[item * 4 + 1], ntok = a.items[item * 4 + 2],
            pos0 = a.items[item * 4 + 3];
  const int H = a.H, hpg = H / (a.G * a.M), NK = a.G * a.M * D, NVt = a.G * V;
  const int h0 = (blockIdx.y * 8 + wv) * HW, nh = min(HW, H - h0);
  if (nh <= 0) return;                                     // the whole wave; nothing below synchronises waves
  const int posq = pos0 + r, pos_last = pos0 + ntok - 1;
  const bool qvalid = r < ntok;
  // this query's own bounds
  const int cq_lo = a.chunk > 0 ? (posq / a.chunk) * a.chunk : 0;
  const int wq_lo = a.window > 0 ? posq - a.window + 1 : 0;
  const int keep = a.window > 0 ? a.keep_first : 0;
  // the tile's key blocks: [a_beg, a_end) (kept first tokens) and [lo_al, pos_last]
  const KeyRuns k0 = key_runs(pos0, a.chunk, a.window, a.keep_first);
  const int lo_al = k0.lo & ~31, a_beg = k0.a0 & ~31;
  const int a_end = a.window > 0 ? min(lo_al, (a.keep_first + 31) & ~31) : a_beg;
  const int nblkA = max(0, (a_end - a_beg) >> 5), nblk = nblkA + ((pos_last - lo_al) >> 5) + 1;
  const int* pages = a.bt + (size_t)sg * a.maxb;
  const int b_lo = SPLIT ? (int)blockIdx.z * a.part_blocks : 0;
  const int b_hi = (!SPLIT || (int)blockIdx.z == a.n_parts - 1) ? nblk : min(nblk, b_lo + a.part_blocks);
  if (SPLIT && b_lo >= b_hi) {                             // a part without blocks: nothing to join
    if (hq == 0)
      for (int hh = 0; hh < nh; ++hh) {
        float* ml = a.pml + ((((size_t)item * a.n_parts + blockIdx.z) * H + h0 + hh) * 16 + r) * 2;
        ml[0] = -INFINITY;
        ml[1] = 0.f;
      }
    return;
  }
  bf16x8 qf[HW][NDC];
  float m2[HW], l[HW];
  f32x4 o[HW][NV];
#pragma unroll
  for (int hh = 0; hh < HW; ++hh) {
    const bool on = hh < nh && qvalid;
    const uint16_t* qp = a.q + (size_t)(row0 + (on ? r : 0)) * H * D + (size_t)(on ? h0 + hh : 0) * D;
#pragma unroll
    for (int cc = 0; cc < NDC; ++cc) {
      qf[hh][cc] = mld16(qp + 32 * cc + 8 * hq);
      if (!on)
#pragma unroll
        for (int j = 0; j < 8; ++j) qf[hh][cc][j] = (__bf16)0.f;
    }
    m2[hh] = (!SPLIT && a.sink && hh < nh) ? a.sink[h0 + hh] * kLog2e : -INFINITY;
    l[hh] = 0.f;
#pragma unroll
    for (int dt = 0; dt < NV; ++dt) o[hh][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const float sc2 = a.scale * kLog2e, cap2 = a.softcap * kLog2e, icap = a.softcap > 0.f ? a.scale / a.softcap : 0.f;
  // a block whose 32 keys every query of a full tile sees needs no mask: all keys at or before the first
  // position, inside the last query's chunk, and inside the last query's window or among the kept tokens
  const int cl_lo = a.chunk > 0 ? (pos_last / a.chunk) * a.chunk : 0;
  const int wl_lo = a.window > 0 ? pos_last - a.window + 1 : 0;
  // The wave's heads share one key / value head (the launch picks HW so).  A block's page lookup, key
  // loads and value loads are dependent memory accesses, so they are issued a block ahead into the SAME
  // registers: the next keys as soon as this block's scores are formed, the next values as soon as this
  // block's value products are issued; the softmax and the products run meanwhile.
  // (with score maps: map m of a head reads key head m of its group and the group's one value head)
  const int gv = h0 / a.M / hpg, g = gv * a.M + h0 % a.M;
  bf16x8 kf[KH][2][NDC];
  bf16x8 vf[NV];
  auto block_at = [&](int bi) { return bi < nblkA ? a_beg + 32 * bi : lo_al + 32 * (bi - nblkA); };
  // lane i of (kbv, pgv, ofv) holds the first key, the page and the offset within the page of block
  // pg_base + i (64 blocks per fill): the divisions and the page lookup are done for 64 blocks at once,
  // off the chain of dependent loads
  int pg_base = 0, kbv = 0, pgv = 0, ofv = 0;
  auto fill_pages = [&](int base) {
    pg_base = base;
    const int bi = base + lane;
    kbv = block_at(bi);
    const int pi = kbv / a.BS;
    ofv = kbv - pi * a.BS;
    pgv = bi < nblk ? pages[pi] : 0;
  };
  fill_pages(b_lo);
  auto load_k = [&](int page, int off) {
    const uint16_t* kp = a.kc + ((size_t)page * a.BS + off) * NK + g * D + 8 * hq;
#pragma unroll
    for (int kh = 0; kh < KH; ++kh)
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int key = 8 * (r >> 2) + 4 * t + (r & 3);
#pragma unroll
        for (int cc = 0; cc < NDC; ++cc) kf[kh][t][cc] = mld16(kp + (size_t)key * NK + kh * D + 32 * cc);
      }
  };
  auto load_v = [&](int page, int off) {
    const uint16_t* vp = a.vt + ((size_t)page * NVt + (size_t)gv * V) * a.BS + off + 8 * hq;
#pragma unroll
    for (int dt = 0; dt < NV; ++dt) vf[dt] = mld16(vp + (size_t)(16 * dt + r) * a.BS);
  };
  int kb_next = __shfl(kbv, 0, 64), pg_next = __shfl(pgv, 0, 64), of_next = __shfl(ofv, 0, 64);
  load_k(pg_next, of_next);
  load_v(pg_next, of_next);
  for (int bi = b_lo; bi < b_hi; ++bi) {
    const int kb = kb_next;
    if (bi + 1 < b_hi) {
      if (bi + 1 - pg_base == 64) fill_pages(bi + 1);
      kb_next = __shfl(kbv, bi + 1 - pg_base, 64);
      pg_next = __shfl(pgv, bi + 1 - pg_base, 64);
      of_next = __shfl(ofv, bi + 1 - pg_base, 64);
    }
    const bool open_blk = ntok == 16 && kb + 31 <= pos0 && kb >= cl_lo && (kb >= wl_lo || kb + 32 <= keep);
    float p[HW][8];
#pragma unroll
    for (int hh = 0; hh < HW; ++hh) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        f32x4 sacc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int cc = 0; cc < NDC; ++cc)
          sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[KH == 1 ? 0 : hh][t][cc], qf[hh][cc], sacc, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) p[hh][4 * t + i] = sacc[i];
      }
    }
    if (bi + 1 < b_hi) load_k(pg_next, of_next);
    bf16x8 pf[HW];
#pragma unroll
    for (int hh = 0; hh < HW; ++hh) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if (CAP) {
          // cap tanh(x), tanh(x) = 1 - 2 / (1 + e^(2x)), in log2 units
          const float e = __builtin_amdgcn_exp2f(fminf(p[hh][j] * icap * (2.f * kLog2e), 60.f));
          p[hh][j] = cap2 * (1.f - 2.f * __builtin_amdgcn_rcpf(1.f + e));
        } else {
          p[hh][j] *= sc2;
        }
      }
      if (!open_blk) {                                     // (a wave-uniform branch)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int key = kb + 8 * hq + j;                 // j = 4 t + i
          const bool ok = qvalid && key <= posq && key >= cq_lo && (key >= wq_lo || key < keep);
          p[hh][j] = ok ? p[hh][j] : -INFINITY;
        }
      }
      float cmax = p[hh][0];
#pragma unroll
      for (int j = 1; j < 8; ++j) cmax = fmaxf(cmax, p[hh][j]);
      cmax = fmaxf(cmax, __shfl_xor(cmax, 16, 64));
      cmax = fmaxf(cmax, __shfl_xor(cmax, 32, 64));
      // the maximum moves only where a query meets a larger score; while no query of the wave does, the
      // accumulators need no rescaling (a wave-uniform branch)
      const bool grow = cmax > m2[hh];
      const float mn = grow ? cmax : m2[hh];
      const float ms = mn == -INFINITY ? 0.f : mn;         // a query that has seen no key yet
      float ps = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float e = __builtin_amdgcn_exp2f(p[hh][j] - ms);
        ps += e;
        pf[hh][j] = (__bf16)e;
      }
      if (__any(grow)) {
        const float alpha = __builtin_amdgcn_exp2f(m2[hh] - ms);
        l[hh] *= alpha;
        m2[hh] = mn;
        float ai[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) ai[i] = __shfl(alpha, 4 * hq + i, 64);
#pragma unroll
        for (int dt = 0; dt < NV; ++dt)
#pragma unroll
          for (int i = 0; i < 4; ++i) o[hh][dt][i] *= ai[i];
      }
      l[hh] += ps;
    }
#pragma unroll
    for (int hh = 0; hh < HW; ++hh)
#pragma unroll
      for (int dt = 0; dt < NV; ++dt) o[hh][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf[hh], vf[dt], o[hh][dt], 0, 0, 0);
    if (bi + 1 < b_hi) load_v(pg_next, of_next);
  }
#pragma unroll
  for (int hh = 0; hh < HW; ++hh) {
    if (hh < nh) {
      float lt = l[hh];
      lt += __shfl_xor(lt, 16, 64);
      lt += __shfl_xor(lt, 32, 64);
      if (SPLIT) {
        if (hq == 0) {
          float* ml = a.pml + ((((size_t)item * a.n_parts + blockIdx.z) * H + h0 + hh) * 16 + r) * 2;
          ml[0] = m2[hh];
          ml[1] = lt;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int qi = 4 * hq + i;
          if (qi < ntok) {
            float* op = a.po + (((size_t)item * a.n_parts + blockIdx.z) * 16 + qi) * H * V + (size_t)(h0 + hh) * V + r;
#pragma unroll
            for (int dt = 0; dt < NV; ++dt) op[16 * dt] = o[hh][dt][i];
          }
        }
        continue;
      }
      if (a.sink) lt += __builtin_amdgcn_exp2f(a.sink[h0 + hh] * kLog2e - m2[hh]);
      const float inv = 1.f / lt;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int qi = 4 * hq + i;
        float f = __shfl(inv, qi, 64);
        if (qi < ntok) {
          if (a.gate) f *= 1.f / (1.f + __expf(-a.gate[(size_t)(row0 + qi) * a.gs + h0 + hh]));
          const size_t oo = (size_t)(row0 + qi) * H * V + (size_t)(h0 + hh) * V + r;
          if (a.out32) {
#pragma unroll
            for (int dt = 0; dt < NV; ++dt) a.out32[oo + 16 * dt] = o[hh][dt][i] * f;
          } else {
#pragma unroll
            for (int dt = 0; dt < NV; ++dt) a.out[oo + 16 * dt] = f2bf(o[hh][dt][i] * f);
          }
        }
      }
    }
  }
}

// out[row][h][:] = sum_p o_p 2^(m_p - M) / (sum_p l_p 2^(m_p - M) + 2^(sink - M)) * sigmoid(gate), parts in order
__global__ void __launch_bounds__(256) masked_attn_merge_kernel(MaskArgs a, int V) {
  constexpr float kLog2e = 1.4426950408889634f;
  const int item = blockIdx.x;
  const int row0 = a.items[item * 4 + 1], ntok = a.items[item * 4 + 2];
  const int H = a.H, HV = H * V;
  for (int e = blockIdx.y * 256 + threadIdx.x; e < ntok * HV; e += gridDim.y * 256) {
    const int q = e / HV, c = e - q * HV, h = c / V;
    const float sk = a.sink ? a.sink[h] * kLog2e : -INFINITY;
    float M = sk;
    for (int p2 = 0; p2 < a.n_parts; ++p2)
      M = fmaxf(M, a.pml[((((size_t)item * a.n_parts + p2) * H + h) * 16 + q) * 2]);
    float L = a.sink ? __builtin_amdgcn_exp2f(sk - M) : 0.f, acc = 0.f;
    for (int p2 = 0; p2 < a.n_parts; ++p2) {
      const float* ml = a.pml + ((((size_t)item * a.n_parts + p2) * H + h) * 16 + q) * 2;
      if (ml[0] == -INFINITY) continue;                    // an empty part, or one whose keys this row does not see
      const float w = __builtin_amdgcn_exp2f(ml[0] - M);
      L = fmaf(ml[1], w, L);
      acc = fmaf(a.po[(((size_t)item * a.n_parts + p2) * 16 + q) * HV + c], w, acc);
    }
    float f = 1.f / L;
    if (a.gate) f *= 1.f / (1.f + __expf(-a.gate[(size_t)(row0 + q) * a.gs + h]));
    if (a.out32)
      a.out32[(size_t)(row0 + q) * HV + c] = acc * f;
    else
      a.out[(size_t)(row0 + q) * HV + c] = f2bf(acc * f);
  }
}

template <int NDC, int NV, int HW, bool CAP, int KH>
static int launch_mask_cap(const MaskArgs& a, int n_items, hipStream_t s) {
  const int waves_all = (a.H + HW - 1) / HW;               // HW heads per wave, up to eight waves per workgroup
  const int gy = (waves_all + 7) / 8, waves = gy > 1 ? 8 : waves_all;
  if (a.n_parts > 1) {
    hipLaunchKernelGGL((masked_attn_mfma_kernel<NDC, NV, HW, CAP, true, KH>), dim3(n_items, gy, a.n_parts),
                       dim3(64 * waves), 0, s, a);
    hipLaunchKernelGGL(masked_attn_merge_kernel, dim3(n_items, 8), dim3(256), 0, s, a, NV * 16);
  } else {
    hipLaunchKernelGGL((masked_attn_mfma_kernel<NDC, NV, HW, CAP, false, KH>), dim3(n_items, gy), dim3(64 * waves), 0, s,
                       a);
  }
  return (int)hipGetLastError();
}

template <int NDC, int NV, int HW, int KH = 1>
static int launch_mask_hw(const MaskArgs& a, int n_items, hipStream_t s) {
  if (KH == 1 && a.softcap > 0.f) return launch_mask_cap<NDC, NV, HW, true, 1>(a, n_items, s);
  return launch_mask_cap<NDC, NV, HW, false, KH>(a, n_items, s);
}

// two heads per wave where the heads of a key / value head come in pairs, or where a head has two score maps
// (uncapped: the pair is the head's two maps, which share their values); else one
template <int NDC, int NV>
static int launch_mask_mfma(const MaskArgs& a, int n_items, hipStream_t s) {
  if (a.M == 2 && !(a.softcap > 0.f)) return launch_mask_hw<NDC, NV, 2, 2>(a, n_items, s);
  return a.M == 1 && (a.H / a.G) % 2 == 0 ? launch_mask_hw<NDC, NV, 2>(a, n_items, s)
                                          : launch_mask_hw<NDC, NV, 1>(a, n_items, s);
}

}  // namespace k8s

using namespace k8s;

K8S_API int k8s_attn_prep(const float* qkv, int qs, const float* bias, int H, int G, int D, int NV, const int* positions,
                          const int* slots, void* kc, void* vc, void* vt, int BS, void* q_out, int dt, int norm,
                          const float* q_w, const float* k_w, float eps, int rot, float base, float lam,
                          const float* v_other, float* v_keep, int T, hipStream_t s, int v_col, float tq_coef,
                          int tq_every) {
  if (T <= 0) return 0;
  if (H < 1 || G < 0 || D < 1 || D > 64 * kPrepPer || NV < 0 || rot < 0 || rot > D || (rot & 1) || BS < 1 ||
      norm < 0 || norm > 2 || v_col < 0 || tq_every < 0 || ((G > 0 || NV > 0) && (!kc || !vc)))
    return (int)hipErrorInvalidValue;
  const int units = H + G;
  const int upr = (size_t)(rot + units * D) * sizeof(float) <= 64 * 1024 ? units : 4;    // heads per round
  const size_t lds = (size_t)(rot + upr * D) * sizeof(float);
  if (dt == 0)
    hipLaunchKernelGGL((attn_prep_kernel<uint16_t>), dim3(T), dim3(256), lds, s, qkv, qs, bias, H, G, D, NV, positions,
                       slots, (uint16_t*)kc, (uint16_t*)vc, (uint16_t*)vt, BS, (uint16_t*)q_out, norm, q_w, k_w, eps, rot,
                       base, lam, v_other, v_keep, upr, v_col, tq_coef, tq_every);
  else
    hipLaunchKernelGGL((attn_prep_kernel<float>), dim3(T), dim3(256), lds, s, qkv, qs, bias, H, G, D, NV, positions, slots,
                       (float*)kc, (float*)vc, (float*)vt, BS, (float*)q_out, norm, q_w, k_w, eps, rot, base, lam,
                       v_other, v_keep, upr, v_col, tq_coef, tq_every);
  return (int)hipGetLastError();
}

K8S_API int k8s_masked_attn_rows(const void* q, const void* kc, const void* vc, const int* block_tables, int maxb,
                                 const int* row_seg, const int* seg_row0, const int* seg_pos0, const float* sink,
                                 const float* gate, int gs, void* out, int T, int H, int G, int D, int V, int BS,
                                 int chunk, int window, int keep_first, float scale, float softcap, int dt,
                                 hipStream_t s, int maps, int out_f32) {
  if (T <= 0) return 0;
  if (maps < 1) return (int)hipErrorInvalidValue;
  const int HQ = H * maps;
  const size_t lds = (size_t)(HQ * D + HQ * kMaskTile + 2 * HQ) * sizeof(float);
  if (H < 1 || G < 1 || H % G || HQ * V > 256 * kMaskOut || chunk < 0 || window < 0 || keep_first < 0 ||
      lds > 64 * 1024)
    return (int)hipErrorInvalidValue;
#define K8S_ROWS(TA, TO)                                                                                             \
  hipLaunchKernelGGL((masked_attn_rows_kernel<TA, TO>), dim3(T), dim3(256), lds, s, (const TA*)q, (const TA*)kc,    \
                     (const TA*)vc, block_tables, maxb, row_seg, seg_row0, seg_pos0, sink, gate, gs, (TO*)out, HQ, G, \
                     D, V, BS, chunk, window, keep_first, scale, softcap, maps)
  if (dt == 0 && out_f32) {
    K8S_ROWS(uint16_t, float);
  } else if (dt == 0) {
    K8S_ROWS(uint16_t, uint16_t);
  } else {
    K8S_ROWS(float, float);
  }
#undef K8S_ROWS
  return (int)hipGetLastError();
}

// 1 when the matrix-core kernel takes these sizes (bf16 only)
K8S_API int k8s_masked_attn_mfma_ok(int H, int G, int D, int V) {
  return H >= 1 && G >= 1 && H % G == 0 && (D == 64 || D == 128) && (V == 64 || V == 128);
}

K8S_API int k8s_masked_attn_mfma(const void* q, const void* kc, const void* vt, const int* block_tables, int maxb,
                                 const int* items, int n_items, const float* sink, const float* gate, int gs, void* out,
                                 int H, int G, int D, int V, int BS, int chunk, int window, int keep_first, float scale,
                                 float softcap, hipStream_t s, int part_blocks, int n_parts, float* pml, float* po,
                                 int maps, int out_f32) {
  if (n_items <= 0) return 0;
  if (!k8s_masked_attn_mfma_ok(H, G, D, V) || BS % 32 || chunk < 0 || window < 0 || keep_first < 0 || maps < 1)
    return (int)hipErrorInvalidValue;
  if (n_parts > 1 && (part_blocks < 1 || !pml || !po)) return (int)hipErrorInvalidValue;
  MaskArgs a;
  a.q = (const uint16_t*)q;
  a.kc = (const uint16_t*)kc;
  a.vt = (const uint16_t*)vt;
  a.bt = block_tables;
  a.maxb = maxb;
  a.items = items;
  a.n_items = n_items;
  a.sink = sink;
  a.gate = gate;
  a.gs = gs;
  a.out = out_f32 ? nullptr : (uint16_t*)out;
  a.out32 = out_f32 ? (float*)out : nullptr;
  a.H = H * maps;
  a.G = G;
  a.M = maps;
  a.BS = BS;
  a.chunk = chunk;
  a.window = window;
  a.keep_first = keep_first;
  a.scale = scale;
  a.softcap = softcap;
  a.part_blocks = n_parts > 1 ? part_blocks : 1;
  a.n_parts = n_parts > 1 ? n_parts : 1;
  a.pml = pml;
  a.po = po;
  if (D == 64 && V == 64) return launch_mask_mfma<2, 4>(a, n_items, s);
  if (D == 64 && V == 128) return launch_mask_mfma<2, 8>(a, n_items, s);
  if (D == 128 && V == 64) return launch_mask_mfma<4, 4>(a, n_items, s);
  return launch_mask_mfma<4, 8>(a, n_items, s);
}
