// Mechanisms of hybrid decoders (layer-list models whose sublayers are normed on their output):
// softmax attention over a sliding window with kept first tokens, also over latent rows that
// serve as key and value at once; rotary turns of a sub-vector with a magnitude factor; a causal
// convolution with a carried tail; the step sizes of a state-space recurrence; routed experts
// grouped by expert on the device; the residual update with a norm on the sublayer's output.
//
// Arithmetic as in sd_seqmix.hip: activations are f32 buffers, scores, softmax weights, norms,
// router scores, step sizes and decays are f32 always; with bf16 weights the operands of matrix
// products are rounded to bf16 values where they are produced and the cache holds bf16.  Every
// output element is summed in an order fixed by the token's own position in its sequence.
#include <math.h>

#include "sd_common.h"

namespace {

template <typename T> __device__ __forceinline__ float ld_f(const T* p);
template <> __device__ __forceinline__ float ld_f<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ld_f<bf16_t>(const bf16_t* p) { return (float)*p; }
template <typename T> __device__ __forceinline__ void st_f(T* p, float v);
template <> __device__ __forceinline__ void st_f<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void st_f<bf16_t>(bf16_t* p, float v) { *p = (bf16_t)v; }

__device__ __forceinline__ float maybe_round(float v, int round) { return round ? round_bf16(v) : v; }
__device__ __forceinline__ float sigmoid_f(float z) { return 1.f / (1.f + expf(-z)); }
__device__ __forceinline__ float silu_f(float z) { return z * sigmoid_f(z); }

// Sum over a workgroup of up to 256 threads in a fixed order (waves' sums in wave order).
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6, n_waves = (blockDim.x + 63) >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[wave] = v;
  __syncthreads();
  float s = red[0];
  for (int w = 1; w < n_waves; ++w) s += red[w];
  return s;
}

// ------------------------------------------------------------------ embedding
template <typename T>
__global__ void embed_hashed_kernel(const int32_t* __restrict__ tokens, const int32_t* __restrict__ prev,
                                    const T* __restrict__ table, const T* __restrict__ bigram, float scale,
                                    int buckets, int mul_prev, int mul_cur, float* __restrict__ x,
                                    bf16_t* __restrict__ x_b, int W, int vocab) {
  const int r = blockIdx.x;
  int tok = tokens[r];
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  long long brow = -1;
  if (bigram) {
    const int p = prev ? prev[r] : -1;
    brow = p < 0 ? (long long)buckets
                 : (long long)(((long long)p * mul_prev + (long long)tokens[r] * mul_cur) % buckets);
    if (brow < 0) brow += buckets;
  }
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float v = ld_f(table + (size_t)tok * W + c) * scale;
    if (brow >= 0) v += ld_f(bigram + (size_t)brow * W + c);
    x[(size_t)r * W + c] = v;
    if (x_b) x_b[(size_t)r * W + c] = (bf16_t)v;
  }
}

// ------------------------------------------------------------------ norm over parts of a row
// One workgroup per (row, part).
template <typename T>
__global__ void rmsnorm_parts_kernel(const float* __restrict__ x, int64_t ldx, const float* __restrict__ gate,
                                     int64_t ldg, const T* __restrict__ w, float eps, float* __restrict__ out,
                                     int64_t ldo, bf16_t* __restrict__ out_b, int64_t ldob, int pw, int round) {
  __shared__ float red[4];
  const int r = blockIdx.x, c0 = blockIdx.y * pw;
  const float* xr = x + (size_t)r * ldx + c0;
  const float* gr = gate ? gate + (size_t)r * ldg + c0 : nullptr;
  float ss = 0.f;
  for (int c = threadIdx.x; c < pw; c += blockDim.x) {
    const float v = gr ? xr[c] * silu_f(gr[c]) : xr[c];
    ss = fmaf(v, v, ss);
  }
  ss = block_sum(ss, red);
  const float rstd = 1.f / sqrtf(ss / (float)pw + eps);
  for (int c = threadIdx.x; c < pw; c += blockDim.x) {
    float v = gr ? xr[c] * silu_f(gr[c]) : xr[c];
    v *= rstd;
    if (w) v *= ld_f(w + c0 + c);
    v = maybe_round(v, round);
    out[(size_t)r * ldo + c0 + c] = v;
    if (out_b) out_b[(size_t)r * ldob + c0 + c] = (bf16_t)v;
  }
}

// ------------------------------------------------------------------ rotary turn of a sub-vector
// One wave per (row, head): n channels from src to dst (the same place or another), the first
// `dims` of them turned; the angle is formed in f64 (position times frequency).
__global__ void rope_copy_kernel(const float* __restrict__ src, int64_t lds_, int src_hs, int src_off,
                                 float* __restrict__ dst, int64_t ldd, int dst_hs, int dst_off,
                                 const int32_t* __restrict__ row_pos, int n, int dims, int layout,
                                 const double* __restrict__ inv_freq, float mag) {
  const int r = blockIdx.x, h = blockIdx.y;
  const float* in = src + (size_t)r * lds_ + (size_t)h * src_hs + src_off;
  float* out = dst + (size_t)r * ldd + (size_t)h * dst_hs + dst_off;
  const int pos = row_pos[r];
  for (int i = threadIdx.x; i < dims / 2; i += blockDim.x) {
    const double a = (double)pos * inv_freq[i];
    const float cs = (float)cos(a) * mag, sn = (float)sin(a) * mag;
    const int iu = layout ? 2 * i : i, iv = layout ? 2 * i + 1 : i + dims / 2;
    const float u = in[iu], v = in[iv];
    out[iu] = u * cs - v * sn;
    out[iv] = v * cs + u * sn;
  }
  if (in != out)
    for (int c = dims + threadIdx.x; c < n; c += blockDim.x) out[c] = in[c];
}

// ------------------------------------------------------------------ cache append
template <typename T>
__global__ void cache_append_kernel(const float* __restrict__ k, int64_t ldk, const float* __restrict__ v,
                                    int64_t ldv, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                    const int32_t* __restrict__ row_pos, const int32_t* __restrict__ row_slot,
                                    const int32_t* __restrict__ block_tables, int max_blocks, int page, int G,
                                    int dk, int dv) {
  const int r = blockIdx.x, g = blockIdx.y;
  const int pos = row_pos[r];
  const int pg = block_tables[(size_t)row_slot[r] * max_blocks + pos / page];
  const size_t at = ((size_t)pg * G + g) * page + pos % page;
  for (int c = threadIdx.x; c < dk; c += blockDim.x) st_f(k_cache + at * dk + c, k[(size_t)r * ldk + (size_t)g * dk + c]);
  if (v)
    for (int c = threadIdx.x; c < dv; c += blockDim.x) st_f(v_cache + at * dv + c, v[(size_t)r * ldv + (size_t)g * dv + c]);
}

// ------------------------------------------------------------------ softmax window attention
constexpr int kLoads = 16;     // 16-byte pieces of a key row a thread has in flight

template <typename T> struct Piece;
template <> struct Piece<bf16_t> {
  static constexpr int E = 8;
  static __device__ __forceinline__ void unpack(const u32x4& raw, float* f) {
    const bf16x8 v = __builtin_bit_cast(bf16x8, raw);
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = (float)v[i];
  }
};
template <> struct Piece<float> {
  static constexpr int E = 4;
  static __device__ __forceinline__ void unpack(const u32x4& raw, float* f) {
    const f32x4 v = __builtin_bit_cast(f32x4, raw);
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = v[i];
  }
};

// A score capped smoothly at +-cap (cap <= 0: as it is).
__device__ __forceinline__ float cap_score(float s, float cap) { return cap > 0.f ? cap * tanhf(s / cap) : s; }

// s[hq] += q[hq] . k over n channels, ascending (kr and qs point at the first of them; a head's
// query is q_stride floats from the next).  vec: rows are 16-byte aligned and n a multiple of
// the piece size; then up to kLoads pieces are asked for before the first is used.
template <typename KT_, int NH>
__device__ __forceinline__ void score_key(const KT_* __restrict__ kr, const float* __restrict__ qs, int q_stride, int n,
                                          int nh, bool vec, float* s) {
  constexpr int E = Piece<KT_>::E;
  if (vec) {
    for (int c = 0; c < n; c += kLoads * E) {
      u32x4 raw[kLoads];
#pragma unroll
      for (int i = 0; i < kLoads; ++i) {   // unguarded, on an address clamped into the row
        const int ci = c + i * E < n ? c + i * E : n - E;
        raw[i] = *reinterpret_cast<const u32x4*>(kr + ci);
      }
#pragma unroll
      for (int i = 0; i < kLoads; ++i) {
        if (c + i * E < n) {
          float kf[E];
          Piece<KT_>::unpack(raw[i], kf);
#pragma unroll
          for (int hq = 0; hq < NH; ++hq)
            if (hq < nh) {
#pragma unroll
              for (int e = 0; e < E; ++e) s[hq] = fmaf(qs[hq * q_stride + c + i * E + e], kf[e], s[hq]);
            }
        }
      }
    }
    return;
  }
  for (int c = 0; c < n; ++c) {
    const float kf = ld_f(kr + c);
#pragma unroll
    for (int hq = 0; hq < NH; ++hq)
      if (hq < nh) s[hq] = fmaf(qs[hq * q_stride + c], kf, s[hq]);
  }
}

// One workgroup of 256 threads per (row, kv head, group of up to NH query heads of that kv head).
// Per tile of KT keys: the keys are scored against the query heads (q in LDS) by 256 / KT threads
// each, over consecutive parts of the channels whose sums are added in part order; the tile's
// maximum moves the running maximum and rescales what has been summed; then a wave per key, lanes
// over value columns, adds the weighted value rows.  NC: value columns per lane (dv <= 64 * NC).
// n_splits > 1 (few rows): workgroup (.., .., z) takes tile z / n_hgroups of the row's keys only
// and leaves its maximum, its sum of weights and its unnormalised weighted values in part_ml /
// part_acc; softmax_merge_kernel puts a row's tiles together in tile order.
// maps > 1: a head holds `maps` queries of dk channels (unit h * maps + m of a row of q), the key
// cache `maps` key rows per kv head (cache head g * maps + m), and every map reads the kv head's
// one value row; blockIdx.y counts key heads, and out / sinks count units.
template <typename T, int NH, int NC, int KT>
__global__ __launch_bounds__(256) void window_softmax_attn_kernel(
    const float* __restrict__ q, int64_t ldq, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    int v_row, const int32_t* __restrict__ row_pos, const int32_t* __restrict__ row_slot,
    const int32_t* __restrict__ block_tables, int max_blocks, int page, int H, int G, int dk, int dv, int window,
    int keep_first, float scale, float* __restrict__ out, bf16_t* __restrict__ out_b, int n_hgroups, int n_splits,
    float* __restrict__ part_acc, float* __restrict__ part_ml, int chunk, float softcap,
    const float* __restrict__ sinks, int maps) {
  extern __shared__ float lds[];
  constexpr int nthr = 256, nw = 4, PARTS = nthr / KT, KW = KT / 64;
  unsigned long long* vat = reinterpret_cast<unsigned long long*>(lds);  // [KT] cache row of the key
  float* wt = reinterpret_cast<float*>(vat + KT);                        // [NH][KT]
  float* qs = wt + NH * KT;                                              // [NH][dk]
  float* m_run = qs + NH * dk;                                           // [NH] running maximum
  float* l_run = m_run + NH;                                             // [NH] running sum
  float* corr = l_run + NH;                                              // [NH]
  float* red = corr + NH;                                                // [nw][dv]
  float* ps = red + nw * dv;                                             // [PARTS][NH][KT] (PARTS > 1)
  const int r = blockIdx.x, gk = blockIdx.y, g = gk / maps, mp = gk % maps, tid = threadIdx.x;
  const int hgroup = blockIdx.z % n_hgroups, split = blockIdx.z / n_hgroups;
  const int qh = H / G, HM = H * maps, GM = G * maps;
  const int hh0 = g * qh + hgroup * NH;            // the group's first query head
  const int h0 = hh0 * maps + mp;                  // ... and its unit; the next head's is `maps` further
  const int nh = qh - hgroup * NH < NH ? qh - hgroup * NH : NH;
  const int i = row_pos[r];
  const int32_t* tbl = block_tables + (size_t)row_slot[r] * max_blocks;
  for (int c = tid; c < nh * dk; c += nthr)
    qs[c] = q[(size_t)r * ldq + (size_t)(h0 + (c / dk) * maps) * dk + c % dk];
  if (tid < NH) {
    // (a sink is one more term exp(sink) of the denominator, with no key and no value: the first
    // tile's workgroup starts its running maximum and sum from it)
    const bool sunk = sinks && split == 0 && tid < nh;
    m_run[tid] = sunk ? sinks[h0 + tid * maps] : -INFINITY;
    l_run[tid] = sunk ? 1.f : 0.f;
  }
  int t_first = i - window + 1 > 0 ? i - window + 1 : 0;
  if (chunk > 0 && i - i % chunk > t_first) t_first = i - i % chunk;   // keys of the row's own chunk only
  const int n_kept = keep_first < t_first ? keep_first : t_first;   // kept tokens that left the window
  const int total = n_kept + (i - t_first + 1);
  const int key_lo = n_splits > 1 ? split * KT : 0;
  const int key_hi = n_splits > 1 ? (total < key_lo + KT ? total : key_lo + KT) : total;
  constexpr int E = Piece<T>::E;
  const bool vec = dk % E == 0 && (reinterpret_cast<uintptr_t>(k_cache) & 15) == 0;
  // the channels of this thread's part, in whole pieces
  const int key = tid % KT, part = tid / KT;
  const int unit = vec ? E : 1, units = dk / unit, per = (units + PARTS - 1) / PARTS;
  const int c_lo = (part * per < units ? part * per : units) * unit;
  const int c_hi = ((part + 1) * per < units ? (part + 1) * per : units) * unit;
  const int wave = tid >> 6, lane = tid & 63;
  float acc[NH][NC];
#pragma unroll
  for (int hq = 0; hq < NH; ++hq)
#pragma unroll
    for (int m = 0; m < NC; ++m) acc[hq][m] = 0.f;
  __syncthreads();
  for (int base = key_lo; base < key_hi; base += KT) {
    const int idx = base + key;
    {
      float s[NH];
#pragma unroll
      for (int hq = 0; hq < NH; ++hq) s[hq] = 0.f;
      if (idx < key_hi) {
        const int j = idx < n_kept ? idx : t_first + (idx - n_kept);
        const size_t at = ((size_t)tbl[j / page] * GM + gk) * page + j % page;
        if (c_hi > c_lo) score_key<T, NH>(k_cache + at * dk + c_lo, qs + c_lo, dk, c_hi - c_lo, nh, vec, s);
        if (part == 0) vat[key] = ((size_t)tbl[j / page] * G + g) * page + j % page;
      }
      if constexpr (PARTS == 1) {
#pragma unroll
        for (int hq = 0; hq < NH; ++hq)
          if (hq < nh) wt[hq * KT + key] = idx < key_hi ? cap_score(s[hq] * scale, softcap) : -INFINITY;
      } else {
#pragma unroll
        for (int hq = 0; hq < NH; ++hq)
          if (hq < nh) ps[(part * NH + hq) * KT + key] = s[hq];
        __syncthreads();
        if (part == 0) {
#pragma unroll
          for (int hq = 0; hq < NH; ++hq)
            if (hq < nh) {
              float sum = ps[hq * KT + key];
#pragma unroll
              for (int pp = 1; pp < PARTS; ++pp) sum += ps[(pp * NH + hq) * KT + key];
              wt[hq * KT + key] = idx < key_hi ? cap_score(sum * scale, softcap) : -INFINITY;
            }
        }
      }
    }
    __syncthreads();
    for (int hq = wave; hq < nh; hq += nw) {     // the tile's maximum per head, a wave per head
      float m = wt[hq * KT + lane];
#pragma unroll
      for (int u = 1; u < KW; ++u) m = fmaxf(m, wt[hq * KT + 64 * u + lane]);
      m = wave_max(m);
      if (lane == 0) {
        const float m_old = m_run[hq], m_new = fmaxf(m_old, m);
        corr[hq] = m_old == -INFINITY ? 0.f : expf(m_old - m_new);
        m_run[hq] = m_new;
      }
    }
    __syncthreads();
    if (tid < KT) {
#pragma unroll
      for (int hq = 0; hq < NH; ++hq)
        if (hq < nh) {
          const float sv = wt[hq * KT + tid];
          wt[hq * KT + tid] = base + tid < key_hi ? expf(sv - m_run[hq]) : 0.f;
        }
    }
    __syncthreads();
    for (int hq = wave; hq < nh; hq += nw) {     // running sum of the weights
      float sum = wt[hq * KT + lane];
#pragma unroll
      for (int u = 1; u < KW; ++u) sum += wt[hq * KT + 64 * u + lane];
      sum = wave_sum(sum);
      if (lane == 0) l_run[hq] = l_run[hq] * corr[hq] + sum;
    }
#pragma unroll
    for (int hq = 0; hq < NH; ++hq)
      if (hq < nh) {
        const float cf = corr[hq];
#pragma unroll
        for (int m = 0; m < NC; ++m) acc[hq][m] *= cf;
      }
    const int n_here = key_hi - base < KT ? key_hi - base : KT;
    constexpr int kBatch = NC <= 2 ? 16 : (NC <= 4 || NH <= 4 ? 8 : 4);   // value rows a wave has in flight
    for (int kk0 = wave; kk0 < n_here; kk0 += nw * kBatch) {
      float vf[kBatch][NC];
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const int kk = kk0 + nw * u < n_here ? kk0 + nw * u : n_here - 1;
        const size_t at = vat[kk];
#pragma unroll
        for (int m = 0; m < NC; ++m)
          vf[u][m] = ld_f(v_cache + at * v_row + (lane + 64 * m < dv ? lane + 64 * m : dv - 1));
      }
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const int kk = kk0 + nw * u;
        if (kk < n_here) {
#pragma unroll
          for (int hq = 0; hq < NH; ++hq)
            if (hq < nh) {
              const float w = wt[hq * KT + kk];
#pragma unroll
              for (int m = 0; m < NC; ++m) acc[hq][m] = fmaf(w, vf[u][m], acc[hq][m]);
            }
        }
      }
    }
    __syncthreads();
  }
  // the waves' sums in wave order, one head at a time
  const int R = gridDim.x;
#pragma unroll
  for (int hq = 0; hq < NH; ++hq) {
    if (hq < nh) {
#pragma unroll
      for (int m = 0; m < NC; ++m)
        if (lane + 64 * m < dv) red[wave * dv + lane + 64 * m] = acc[hq][m];
      __syncthreads();
      // (no key and no sink: a row past its own keys, which a cut launch's merge skips)
      const float inv = n_splits > 1 ? 1.f : 1.f / l_run[hq];
      for (int c = tid; c < dv; c += nthr) {
        float o = red[c];
#pragma unroll
        for (int u = 1; u < nw; ++u) o += red[u * dv + c];
        o *= inv;
        if (n_splits > 1) {
          part_acc[(((size_t)split * R + r) * HM + h0 + hq * maps) * dv + c] = o;
        } else {
          const size_t at = (size_t)r * HM * dv + (size_t)(h0 + hq * maps) * dv + c;
          out[at] = o;
          if (out_b) out_b[at] = (bf16_t)o;
        }
      }
      if (n_splits > 1 && tid == 0) {
        float* ml = part_ml + (((size_t)split * R + r) * HM + h0 + hq * maps) * 2;
        ml[0] = m_run[hq];
        ml[1] = l_run[hq];
      }
      __syncthreads();
    }
  }
}

// out[r, h] = sum_s acc_s exp(m_s - M) / sum_s l_s exp(m_s - M), M = max m_s.  The first wave takes
// the tiles' maxima and sums a lane per tile (butterfly sums: a fixed order) and leaves every
// tile's factor in LDS; then a thread per column adds the tiles' rows in tile order, eight loads
// in flight.
__global__ void softmax_merge_kernel(const float* __restrict__ part_acc, const float* __restrict__ part_ml,
                                     int n_splits, float* __restrict__ out, bf16_t* __restrict__ out_b, int H, int dv) {
  extern __shared__ float fac[];   // [n_splits]
  __shared__ float inv_l;
  const int r = blockIdx.x, h = blockIdx.y, R = gridDim.x, tid = threadIdx.x;
  const size_t stride = (size_t)R * H;             // (row, head) pairs of one tile
  const size_t at0 = (size_t)r * H + h;
  if (tid < 64) {
    float M = -INFINITY;
    for (int s = tid; s < n_splits; s += 64) M = fmaxf(M, part_ml[(s * stride + at0) * 2]);
    M = wave_max(M);
    float L = 0.f;
    for (int s = tid; s < n_splits; s += 64) {
      const float* ml = part_ml + (s * stride + at0) * 2;
      const float f = ml[0] == -INFINITY ? 0.f : expf(ml[0] - M);
      fac[s] = f;
      L += ml[1] * f;
    }
    L = wave_sum(L);
    if (tid == 0) inv_l = 1.f / L;
  }
  __syncthreads();
  constexpr int kU = 8;
  for (int c = tid; c < dv; c += blockDim.x) {
    float o = 0.f;
    for (int s0 = 0; s0 < n_splits; s0 += kU) {
      float v[kU];
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int s = s0 + u < n_splits ? s0 + u : n_splits - 1;
        v[u] = part_acc[(s * stride + at0) * dv + c];
      }
#pragma unroll
      for (int u = 0; u < kU; ++u)
        if (s0 + u < n_splits && fac[s0 + u] != 0.f) o = fmaf(v[u], fac[s0 + u], o);
    }
    o *= inv_l;
    const size_t at = at0 * dv + c;
    out[at] = o;
    if (out_b) out_b[at] = (bf16_t)o;
  }
}

constexpr int kSplitRows = 64;   // batches of at most this many rows cut their keys over workgroups
constexpr int kSplitKeys = 64;   // ... in tiles of this many keys (four threads score a key)

template <typename T, int NH>
void launch_softmax_nc(dim3 grid, int kt, size_t lds, hipStream_t st, int nc, const float* q, int64_t ldq,
                       const void* kc, const void* vc, int v_row, const int32_t* row_pos, const int32_t* row_slot,
                       const int32_t* bt, int max_blocks, int page, int H, int G, int dk, int dv, int window,
                       int keep_first, float scale, float* out, bf16_t* out_b, int n_hgroups, int n_splits,
                       float* part_acc, float* part_ml, int chunk, float softcap, const float* sinks, int maps) {
#define SD_GO2(NC, KT)                                                                                               \
  window_softmax_attn_kernel<T, NH, NC, KT><<<grid, 256, lds, st>>>(q, ldq, (const T*)kc, (const T*)vc, v_row, row_pos, \
                                                                    row_slot, bt, max_blocks, page, H, G, dk, dv,       \
                                                                    window, keep_first, scale, out, out_b, n_hgroups,   \
                                                                    n_splits, part_acc, part_ml, chunk, softcap, sinks, \
                                                                    maps)
#define SD_GO(NC)                                          \
  do {                                                     \
    if constexpr (NH <= 4) {                               \
      if (kt == kSplitKeys) { SD_GO2(NC, kSplitKeys); break; } \
    }                                                      \
    SD_GO2(NC, 256);                                       \
  } while (0)
  if (nc == 1) SD_GO(1);
  else if (nc == 2) SD_GO(2);
  else if (nc == 4) SD_GO(4);
  else SD_GO(8);
#undef SD_GO
#undef SD_GO2
}

// ------------------------------------------------------------------ fused preparation of attention inputs
// Row norm over n columns in place (times w, rounded to bf16 values when round), by a whole
// workgroup of 256 threads: the sums of rmsnorm_parts_kernel with one part, the same bits.
template <typename T>
__device__ __forceinline__ void norm_in_place(float* __restrict__ v, const T* __restrict__ w, int n, float eps,
                                              int round, bf16_t* __restrict__ copy, float* red) {
  float ss = 0.f;
  for (int c = threadIdx.x; c < n; c += blockDim.x) ss = fmaf(v[c], v[c], ss);
  ss = block_sum(ss, red);
  const float rstd = 1.f / sqrtf(ss / (float)n + eps);
  for (int c = threadIdx.x; c < n; c += blockDim.x) {
    const float o = maybe_round(v[c] * rstd * ld_f(w + c), round);
    v[c] = o;
    if (copy) copy[c] = (bf16_t)o;
  }
}

// Latent attention, per row.  Workgroup (r, 0): the query latent normed in place (+ bf16 copy).
// Workgroup (r, 1): the key/value latent normed in place, the shared rotated part turned in place,
// and the row [latent | rotated part] appended to the cache.
template <typename T>
__global__ __launch_bounds__(256) void latent_prep_kernel(
    float* __restrict__ q_lat, int q_rank, const T* __restrict__ q_w, bf16_t* __restrict__ q_copy, int64_t ld_copy,
    float* __restrict__ kv, int kv_rank, int rot_dim, const T* __restrict__ kv_w, int64_t ld, float eps, int round,
    int dims, int layout, const double* __restrict__ inv_freq, float mag, const int32_t* __restrict__ row_pos,
    const int32_t* __restrict__ row_slot, const int32_t* __restrict__ block_tables, int max_blocks, int page,
    T* __restrict__ k_cache) {
  __shared__ float red[4];
  const int r = blockIdx.x;
  if (blockIdx.y == 0 && q_lat) {
    norm_in_place<T>(q_lat + (size_t)r * ld, q_w, q_rank, eps, round, q_copy ? q_copy + (size_t)r * ld_copy : nullptr, red);
    return;
  }
  float* row = kv + (size_t)r * ld;
  norm_in_place<T>(row, kv_w, kv_rank, eps, round, nullptr, red);
  const int pos = row_pos[r];
  float* vec = row + kv_rank;
  for (int i = threadIdx.x; i < dims / 2; i += blockDim.x) {
    const double a = (double)pos * inv_freq[i];
    const float cs = (float)cos(a) * mag, sn = (float)sin(a) * mag;
    const int iu = layout ? 2 * i : i, iv = layout ? 2 * i + 1 : i + dims / 2;
    const float u = vec[iu], v = vec[iv];
    vec[iu] = u * cs - v * sn;
    vec[iv] = v * cs + u * sn;
  }
  __syncthreads();
  const int de = kv_rank + rot_dim;
  const int pg = block_tables[(size_t)row_slot[r] * max_blocks + pos / page];
  T* dst = k_cache + ((size_t)pg * page + pos % page) * de;
  for (int c = threadIdx.x; c < de; c += blockDim.x) st_f(dst + c, row[c]);
}

// Attention whose q and k are normed over the whole projection, per row.  Workgroup (r, 0): q
// normed in place.  Workgroup (r, 1): k normed in place, then the key and value rows appended.
template <typename T>
__global__ __launch_bounds__(256) void qk_norm_append_kernel(
    float* __restrict__ q, int nq, const T* __restrict__ q_w, float* __restrict__ k, int G, int dk,
    const T* __restrict__ k_w, const float* __restrict__ v, int dv, int64_t ld, float eps,
    const int32_t* __restrict__ row_pos, const int32_t* __restrict__ row_slot,
    const int32_t* __restrict__ block_tables, int max_blocks, int page, T* __restrict__ k_cache,
    T* __restrict__ v_cache) {
  __shared__ float red[4];
  const int r = blockIdx.x;
  if (blockIdx.y == 0) {
    norm_in_place<T>(q + (size_t)r * ld, q_w, nq, eps, 0, nullptr, red);
    return;
  }
  float* kr = k + (size_t)r * ld;
  norm_in_place<T>(kr, k_w, G * dk, eps, 0, nullptr, red);
  __syncthreads();
  const int pos = row_pos[r];
  const int pg = block_tables[(size_t)row_slot[r] * max_blocks + pos / page];
  for (int c = threadIdx.x; c < G * dk; c += blockDim.x) {
    const int g = c / dk;
    st_f(k_cache + (((size_t)pg * G + g) * page + pos % page) * dk + c % dk, kr[c]);
  }
  const float* vr = v + (size_t)r * ld;
  for (int c = threadIdx.x; c < G * dv; c += blockDim.x) {
    const int g = c / dv;
    st_f(v_cache + (((size_t)pg * G + g) * page + pos % page) * dv + c % dv, vr[c]);
  }
}

// Attention whose q and k are normed per head with one weight [dk] shared by the heads, per row.
// Workgroup (r, 0): the H query heads in place, a wave per head.  Workgroup (r, 1): the G key
// heads in place, then the key and value rows appended.
template <typename T>
__device__ __forceinline__ void norm_heads_in_place(float* __restrict__ v, int heads, int dk, const T* __restrict__ w,
                                                    float eps) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
  for (int h = wave; h < heads; h += nw) {
    float* x = v + (size_t)h * dk;
    float ss = 0.f;
    for (int c = lane; c < dk; c += 64) ss = fmaf(x[c], x[c], ss);
    ss = wave_sum(ss);
    const float rstd = 1.f / sqrtf(ss / (float)dk + eps);
    for (int c = lane; c < dk; c += 64) x[c] = x[c] * rstd * ld_f(w + c);
  }
}
template <typename T>
__global__ __launch_bounds__(256) void qk_head_norm_append_kernel(
    float* __restrict__ q, int H, const T* __restrict__ q_w, float* __restrict__ k, int G, int dk,
    const T* __restrict__ k_w, const float* __restrict__ v, int dv, int64_t ld, float eps,
    const int32_t* __restrict__ row_pos, const int32_t* __restrict__ row_slot,
    const int32_t* __restrict__ block_tables, int max_blocks, int page, T* __restrict__ k_cache,
    T* __restrict__ v_cache) {
  const int r = blockIdx.x;
  if (blockIdx.y == 0) {
    norm_heads_in_place<T>(q + (size_t)r * ld, H, dk, q_w, eps);
    return;
  }
  float* kr = k + (size_t)r * ld;
  norm_heads_in_place<T>(kr, G, dk, k_w, eps);
  __syncthreads();
  const int pos = row_pos[r];
  const int pg = block_tables[(size_t)row_slot[r] * max_blocks + pos / page];
  for (int c = threadIdx.x; c < G * dk; c += blockDim.x) {
    const int g = c / dk;
    st_f(k_cache + (((size_t)pg * G + g) * page + pos % page) * dk + c % dk, kr[c]);
  }
  const float* vr = v + (size_t)r * ld;
  for (int c = threadIdx.x; c < G * dv; c += blockDim.x) {
    const int g = c / dv;
    st_f(v_cache + (((size_t)pg * G + g) * page + pos % page) * dv + c % dv, vr[c]);
  }
}

// y[r, h, :] *= sigmoid(z[r, h]): one gate per (row, head).  y_b (or nullptr): the result as bf16.
// Grouped-query attention's preparation in general, per row.  Workgroup (r, 0): the query row of
// nq units of dk channels in place: + bias, norm (1: over the whole row, weight [nq*dk]; 2: per
// unit, one weight [dk]), rotary turn of every unit's first `dims` channels.  Workgroup (r, 1): the
// key row of nk units the same way, then appended (cache head = unit); the value row (G heads of
// dv channels) appended as it is, or, v_from_k, the key row as it stood after its bias and before
// norm and turn (then G * dv == nk * dk).  k == nullptr: the layer reads keys and values another
// layer appended, and only the query is prepared.
template <typename T>
__device__ __forceinline__ void prep_units(float* __restrict__ x, int n_units, int dk, const T* __restrict__ bias,
                                           int norm_kind, const T* __restrict__ w, float eps, int dims, int layout,
                                           const double* __restrict__ inv_freq, float mag, int pos, float* red,
                                           T* __restrict__ raw_dst_base, int raw_dv, size_t raw_head_stride,
                                           float* __restrict__ cs) {
  const int n = n_units * dk;
  // the row's cosines and sines once, for every unit (the angle is formed in f64)
  for (int i = threadIdx.x; i < dims / 2; i += blockDim.x) {
    const double a = (double)pos * inv_freq[i];
    cs[i] = (float)cos(a) * mag;
    cs[dims / 2 + i] = (float)sin(a) * mag;
  }
  float ss = 0.f;
  for (int c = threadIdx.x; c < n; c += blockDim.x) {
    float v = x[c];
    if (bias) {
      v += ld_f(bias + c);
      x[c] = v;
    }
    if (raw_dst_base) st_f(raw_dst_base + (size_t)(c / raw_dv) * raw_head_stride + c % raw_dv, v);
    ss = fmaf(v, v, ss);
  }
  if (norm_kind == 1) {
    ss = block_sum(ss, red);
    const float rstd = 1.f / sqrtf(ss / (float)n + eps);
    for (int c = threadIdx.x; c < n; c += blockDim.x) x[c] = x[c] * rstd * ld_f(w + c);
  }
  __syncthreads();
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
  if (norm_kind == 2) {
    for (int u = wave; u < n_units; u += nw) {   // a wave per unit
      float* xu = x + (size_t)u * dk;
      float s2 = 0.f;
      for (int c = lane; c < dk; c += 64) s2 = fmaf(xu[c], xu[c], s2);
      s2 = wave_sum(s2);
      const float rstd = 1.f / sqrtf(s2 / (float)dk + eps);
      for (int c = lane; c < dk; c += 64) xu[c] = xu[c] * rstd * ld_f(w + c);
    }
    __syncthreads();
  }
  for (int u = wave; u < n_units; u += nw) {     // a wave per unit
    float* xu = x + (size_t)u * dk;
    for (int i = lane; i < dims / 2; i += 64) {
      const float c = cs[i], sn = cs[dims / 2 + i];
      const int iu = layout ? 2 * i : i, iv = layout ? 2 * i + 1 : i + dims / 2;
      const float p = xu[iu], q = xu[iv];
      xu[iu] = p * c - q * sn;
      xu[iv] = q * c + p * sn;
    }
  }
}
template <typename T>
__global__ __launch_bounds__(256) void attn_prep_kernel(
    float* __restrict__ q, int nq, float* __restrict__ k, int nk, int dk, const float* __restrict__ v, int G, int dv,
    int v_from_k, int64_t ld, const T* __restrict__ q_bias, const T* __restrict__ k_bias, int norm_kind,
    const T* __restrict__ q_w, const T* __restrict__ k_w, float eps, int dims, int layout,
    const double* __restrict__ inv_freq, float mag, const int32_t* __restrict__ row_pos,
    const int32_t* __restrict__ row_slot, const int32_t* __restrict__ block_tables, int max_blocks, int page,
    T* __restrict__ k_cache, T* __restrict__ v_cache) {
  extern __shared__ float cs[];   // [dims]: cosines, then sines
  __shared__ float red[4];
  const int r = blockIdx.x;
  const int pos = row_pos[r];
  if (blockIdx.y == 0) {
    prep_units<T>(q + (size_t)r * ld, nq, dk, q_bias, norm_kind, q_w, eps, dims, layout, inv_freq, mag, pos, red,
                  nullptr, 1, 0, cs);
    return;
  }
  const int pg = block_tables[(size_t)row_slot[r] * max_blocks + pos / page];
  float* kr = k + (size_t)r * ld;
  // (cache rows of one token: head g at ((pg * heads + g) * page + pos % page) * channels)
  T* v_dst = v_cache + ((size_t)pg * G * page + pos % page) * dv;
  prep_units<T>(kr, nk, dk, k_bias, norm_kind, k_w, eps, dims, layout, inv_freq, mag, pos, red,
                v_from_k ? v_dst : nullptr, dv, (size_t)page * dv, cs);
  __syncthreads();
  for (int c = threadIdx.x; c < nk * dk; c += blockDim.x)
    st_f(k_cache + (((size_t)pg * nk + c / dk) * page + pos % page) * dk + c % dk, kr[c]);
  if (!v_from_k) {
    const float* vr = v + (size_t)r * ld;
    for (int c = threadIdx.x; c < G * dv; c += blockDim.x) st_f(v_dst + (size_t)(c / dv) * page * dv + c % dv, vr[c]);
  }
}

// Two score maps per head put together: t = a[r, h, 0] - lambda * a[r, h, 1], then t divided by its
// root mean square over the head's dv channels and multiplied by out_scale.  A wave per (row, head).
__global__ __launch_bounds__(256) void diff_combine_kernel(const float* __restrict__ a, float lambda, float eps,
                                                           float out_scale, float* __restrict__ y,
                                                           bf16_t* __restrict__ y_b, int n_pairs, int dv, int round) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int p = blockIdx.x * (blockDim.x >> 6) + wave;     // (row, head)
  if (p >= n_pairs) return;
  const float* a1 = a + (size_t)p * 2 * dv;
  const float* a2 = a1 + dv;
  float ss = 0.f;
  for (int c = lane; c < dv; c += 64) {
    const float t = a1[c] - lambda * a2[c];
    ss = fmaf(t, t, ss);
  }
  ss = wave_sum(ss);
  const float f = out_scale / sqrtf(ss / (float)dv + eps);
  for (int c = lane; c < dv; c += 64) {
    const float o = maybe_round((a1[c] - lambda * a2[c]) * f, round);
    y[(size_t)p * dv + c] = o;
    if (y_b) y_b[(size_t)p * dv + c] = (bf16_t)o;
  }
}

__global__ void head_gate_kernel(float* __restrict__ y, int64_t ldy, const float* __restrict__ z, int64_t ldz,
                                 bf16_t* __restrict__ y_b, int64_t ldyb, int H, int dv, int round) {
  const int r = blockIdx.x;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < H * dv; c += gridDim.y * blockDim.x) {
    const float o = maybe_round(y[(size_t)r * ldy + c] * sigmoid_f(z[(size_t)r * ldz + c / dv]), round);
    y[(size_t)r * ldy + c] = o;
    if (y_b) y_b[(size_t)r * ldyb + c] = (bf16_t)o;
  }
}

// A feed-forward's activation, a[r, c]: kind 0 relu(g) u, 1 silu(g) u, 2 relu(g)^2 (no u).
// out (may be g itself) and out_b (bf16, or nullptr) receive it.
__global__ void act_rows_kernel(const float* __restrict__ g, const float* __restrict__ u, int64_t ld,
                                float* __restrict__ out, int64_t ldo, bf16_t* __restrict__ out_b, int64_t ldob, int F,
                                int kind, int round) {
  const int r = blockIdx.x;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < F; c += gridDim.y * blockDim.x) {
    const float z = g[(size_t)r * ld + c];
    float a;
    if (kind == 2) {
      const float p = fmaxf(z, 0.f);
      a = p * p;
    } else {
      a = (kind == 1 ? silu_f(z) : fmaxf(z, 0.f)) * u[(size_t)r * ld + c];
    }
    a = maybe_round(a, round);
    if (out) out[(size_t)r * ldo + c] = a;
    if (out_b) out_b[(size_t)r * ldob + c] = (bf16_t)a;
  }
}

// ------------------------------------------------------------------ causal convolution
// out[r, c] = act(b[c] + sum_j w[c, taps-1-j] * in(r, j)).  One workgroup per (row, 256 channels).
template <typename T>
__global__ void causal_conv_rows_kernel(const float* __restrict__ x, int64_t ldx, const T* __restrict__ w,
                                        const T* __restrict__ b, const float* __restrict__ conv_state,
                                        const int32_t* __restrict__ row_pos, const int32_t* __restrict__ row_slot,
                                        float* __restrict__ out, int64_t ldo, int C, int taps, int act) {
  const int r = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int slot = row_slot[r], pos = row_pos[r];
  int t = 0;   // rows of this entry before r, as far as the taps reach
  while (t < taps - 1 && r - t - 1 >= 0 && row_slot[r - t - 1] == slot) ++t;
  float acc = b ? ld_f(b + c) : 0.f;
  // oldest input first, so that the sum's order is that of a plain convolution
  for (int j = taps - 1; j >= 0; --j) {
    float in = 0.f;
    if (j <= t) in = x[(size_t)(r - j) * ldx + c];
    else if (pos - j >= 0) in = conv_state[((size_t)slot * (taps - 1) + (taps - 1 - (j - t))) * C + c];
    acc = fmaf(ld_f(w + (size_t)c * taps + (taps - 1 - j)), in, acc);
  }
  out[(size_t)r * ldo + c] = act ? silu_f(acc) : acc;
}

// The entry's last taps-1 inputs become the slot's state (oldest first).  One thread per channel.
__global__ void conv_state_update_kernel(const float* __restrict__ x, int64_t ldx, float* __restrict__ conv_state,
                                         const int32_t* __restrict__ entries, int C, int taps) {
  const int e = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int slot = entries[4 * e], row0 = entries[4 * e + 1], len = entries[4 * e + 2], pos0 = entries[4 * e + 3];
  float* st = conv_state + (size_t)slot * (taps - 1) * C + c;
  for (int s = 0; s < taps - 1; ++s) {   // ascending: an old element is read before its place is written
    const int at = len + s - (taps - 1);  // index among the entry's inputs, negative: before the entry
    float v;
    if (at >= 0) v = x[(size_t)(row0 + at) * ldx + c];
    else v = pos0 + at >= 0 ? st[(size_t)(len + s) * C] : 0.f;
    st[(size_t)s * C] = v;
  }
}

template <typename T>
__global__ void ssd_steps_kernel(const float* __restrict__ dt, int64_t ld, const T* __restrict__ dt_bias,
                                 const T* __restrict__ a_log, float* __restrict__ step, float* __restrict__ decay,
                                 int n, int H) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int r = i / H, h = i % H;
  const float z = dt[(size_t)r * ld + h] + ld_f(dt_bias + h);
  const float sp = z > 20.f ? z : log1pf(expf(z));
  step[i] = sp;
  decay[i] = expf(-expf(ld_f(a_log + h)) * sp);
}

// ------------------------------------------------------------------ scan with a decay per (row, head)
constexpr int kStrip = 16;
constexpr int kScanLoads = 8;
constexpr int kScanLoadsV = 16;
constexpr int kScanChunk = 16;
// S <- d_t S + (a_t k_t) v_t^T, o_t = S^T q_t + skip v_t.  A thread owns 16 consecutive key channels
// of one value column; strips' partial dot products are added in strip order (the skip term rides
// on strip 0).  Chunks of tokens go global -> registers -> LDS with the next chunk's loads in flight.
template <typename T>
__global__ __launch_bounds__(256) void decay_scan_rows_kernel(
    const float* __restrict__ q, const float* __restrict__ k, int64_t ldqk, const float* __restrict__ v, int64_t ldv,
    const float* __restrict__ decay, const float* __restrict__ k_scale, const T* __restrict__ skip,
    float* __restrict__ state, const int32_t* __restrict__ entries,
    float* __restrict__ out, int H, int hpg, int dk, int dv, int CT, int NS, int CH) {
  extern __shared__ float lds[];
  const int dkp = NS * kStrip;
  float* qs = lds;                  // [CH][dkp]
  float* ks = qs + CH * dkp;        // [CH][dkp]
  float* vs = ks + CH * dkp;        // [CH][CT]
  float* dsc = vs + CH * CT;        // [CH] decay
  float* asc = dsc + CH;            // [CH] key scale
  float* part = asc + CH;           // [CH][NS][CT]
  const int tid = threadIdx.x, nthr = CT * NS;
  const int c = tid % CT, s = tid / CT;
  const int h = blockIdx.y, e = blockIdx.z;
  const int gq = h / hpg;
  const int col = blockIdx.x * CT + c;
  const int slot = entries[4 * e], row0 = entries[4 * e + 1], len = entries[4 * e + 2], pos0 = entries[4 * e + 3];
  float* st = state + ((size_t)slot * H + h) * dk * dv;
  const int r0 = s * kStrip;
  float S[kStrip];
#pragma unroll
  for (int r = 0; r < kStrip; ++r)
    S[r] = (pos0 > 0 && r0 + r < dk && col < dv) ? st[(size_t)(r0 + r) * dv + col] : 0.f;
  const float skip_h = skip ? ld_f(skip + h) : 0.f;
  float pq[kScanLoads], pk[kScanLoads], pv[kScanLoadsV], pd = 0.f, pa = 1.f;
  auto fetch = [&](int t0) {
    const int nt = len - t0 < CH ? len - t0 : CH;
#pragma unroll
    for (int i = 0; i < kScanLoads; ++i) {
      const int idx = tid + i * nthr;
      const int t = idx / dkp, ch = idx % dkp;
      const bool in = idx < nt * dkp && ch < dk;
      const int tc = t < nt ? t : nt - 1, cc = ch < dk ? ch : dk - 1;
      const size_t at = (size_t)(row0 + t0 + tc) * ldqk + (size_t)gq * dk + cc;
      const float lq = q[at], lk = k[at];
      pq[i] = in ? lq : 0.f;
      pk[i] = in ? lk : 0.f;
    }
#pragma unroll
    for (int i = 0; i < kScanLoadsV; ++i) {
      const int idx = tid + i * nthr;
      const int t = idx / CT, vcol = blockIdx.x * CT + idx % CT;
      const bool in = idx < nt * CT && vcol < dv;
      const int tc = t < nt ? t : nt - 1, vc2 = vcol < dv ? vcol : dv - 1;
      const float lv = v[(size_t)(row0 + t0 + tc) * ldv + (size_t)h * dv + vc2];
      pv[i] = in ? lv : 0.f;
    }
    {
      const int tc = tid < nt ? tid : nt - 1;
      pd = decay[(size_t)(row0 + t0 + tc) * H + h];
      pa = k_scale ? k_scale[(size_t)(row0 + t0 + tc) * H + h] : 1.f;
    }
  };
  fetch(0);
  for (int t0 = 0; t0 < len; t0 += CH) {
    const int nt = len - t0 < CH ? len - t0 : CH;
#pragma unroll
    for (int i = 0; i < kScanLoads; ++i) {
      const int idx = tid + i * nthr;
      if (idx < CH * dkp) {
        qs[idx] = pq[i];
        ks[idx] = pk[i];
      }
    }
#pragma unroll
    for (int i = 0; i < kScanLoadsV; ++i) {
      const int idx = tid + i * nthr;
      if (idx < CH * CT) vs[idx] = pv[i];
    }
    if (tid < CH) {
      dsc[tid] = pd;
      asc[tid] = pa;
    }
    __syncthreads();
    if (t0 + CH < len) fetch(t0 + CH);
    for (int t = 0; t < nt; ++t) {
      const float vv = vs[t * CT + c];
      const float d = dsc[t], av = asc[t] * vv;
      const float* qt = qs + t * dkp + r0;
      const float* kt = ks + t * dkp + r0;
      float acc = 0.f;
#pragma unroll
      for (int r = 0; r < kStrip; ++r) {
        S[r] = fmaf(d, S[r], kt[r] * av);
        acc = fmaf(S[r], qt[r], acc);
      }
      if (s == 0) acc = fmaf(skip_h, vv, acc);
      part[(t * NS + s) * CT + c] = acc;
    }
    __syncthreads();
    for (int idx = tid; idx < nt * CT; idx += nthr) {
      const int t = idx / CT, cc = idx % CT;
      const int ocol = blockIdx.x * CT + cc;
      if (ocol >= dv) continue;
      float o = part[(t * NS) * CT + cc];
      for (int ss = 1; ss < NS; ++ss) o += part[(t * NS + ss) * CT + cc];
      out[(size_t)(row0 + t0 + t) * ((size_t)H * dv) + (size_t)h * dv + ocol] = o;
    }
  }
  if (col < dv) {
#pragma unroll
    for (int r = 0; r < kStrip; ++r)
      if (r0 + r < dk) st[(size_t)(r0 + r) * dv + col] = S[r];
  }
}

// ------------------------------------------------------------------ routed experts
// One wave per row: scores, then `top` rounds of a wave-wide arg-max (lowest index among equals).
__global__ void moe_route_kernel(const float* __restrict__ logits, int64_t ld, int32_t* __restrict__ sel_e,
                                 float* __restrict__ sel_w, int E, int top, int score_kind, int renorm) {
  extern __shared__ float sc[];   // [E]
  const int r = blockIdx.x, lane = threadIdx.x;
  const float* z = logits + (size_t)r * ld;
  if (score_kind == 0) {
    for (int e = lane; e < E; e += 64) sc[e] = sigmoid_f(z[e]);
  } else {
    float m = -INFINITY;
    for (int e = lane; e < E; e += 64) m = fmaxf(m, z[e]);
    m = wave_max(m);
    float sum = 0.f;
    for (int e = lane; e < E; e += 64) {
      const float p = expf(z[e] - m);
      sc[e] = p;
      sum += p;
    }
    sum = wave_sum(sum);
    for (int e = lane; e < E; e += 64) sc[e] /= sum;
  }
  __syncthreads();
  float total = 0.f;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float v = sc[e];
      if (v > best) {   // (ascending e: the first of equals stays)
        best = v;
        bi = e;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ob > best || (ob == best && oi < bi)) {
        best = ob;
        bi = oi;
      }
    }
    if (lane == 0) {
      sel_e[(size_t)r * top + j] = bi;
      sel_w[(size_t)r * top + j] = best;
      sc[bi] = -INFINITY;
    }
    total += best;
    __syncthreads();
  }
  if (renorm && lane == 0)
    for (int j = 0; j < top; ++j) sel_w[(size_t)r * top + j] /= total;
}

// The router's product and the choice in one launch: a workgroup per row, a wave per expert
// (lanes stride over the row's channels, then a butterfly sum: an order that no other row
// changes), then the first wave chooses as moe_route_kernel does.
template <typename T>
__global__ __launch_bounds__(1024) void moe_route_rows_kernel(const float* __restrict__ x, int64_t ldx,
                                                             const T* __restrict__ w, float* __restrict__ logits,
                                                             int32_t* __restrict__ sel_e, float* __restrict__ sel_w,
                                                             int E, int K, int top, int score_kind, int renorm,
                                                             int round, float renorm_eps, float weight_scale,
                                                             const T* __restrict__ w_gate, int n_gate,
                                                             float* __restrict__ gate_out,
                                                             const float* __restrict__ bias) {
  extern __shared__ float sc[];   // [E]
  const int r = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
  const float* xr = x + (size_t)r * ldx;
  constexpr int kU = 8;   // loads of a lane in flight
  // (rows E .. E + n_gate - 1 are further products of the same input: gates computed as the router is)
  for (int e = wave; e < E + n_gate; e += nw) {
    const T* wr = e < E ? w + (size_t)e * K : w_gate + (size_t)(e - E) * K;
    float acc = 0.f;
    for (int k0 = 0; k0 < K; k0 += 64 * kU) {
      float xv[kU], wv[kU];
#pragma unroll
      for (int u = 0; u < kU; ++u) {   // unguarded, on an index clamped into the row
        const int k = k0 + 64 * u + lane < K ? k0 + 64 * u + lane : K - 1;
        xv[u] = xr[k];
        wv[u] = ld_f(wr + k);
      }
#pragma unroll
      for (int u = 0; u < kU; ++u)
        if (k0 + 64 * u + lane < K) acc = fmaf(maybe_round(xv[u], round), wv[u], acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) {
      if (e < E) {
        if (bias) acc += bias[e];
        sc[e] = acc;
        if (logits) logits[(size_t)r * E + e] = acc;
      } else {
        gate_out[(size_t)r * n_gate + e - E] = acc;
      }
    }
  }
  __syncthreads();
  if (wave != 0) return;
  if (score_kind == 0) {
    for (int e = lane; e < E; e += 64) sc[e] = sigmoid_f(sc[e]);
  } else {
    float m = -INFINITY;
    for (int e = lane; e < E; e += 64) m = fmaxf(m, sc[e]);
    m = wave_max(m);
    float sum = 0.f;
    for (int e = lane; e < E; e += 64) {
      const float p = expf(sc[e] - m);
      sc[e] = p;
      sum += p;
    }
    sum = wave_sum(sum);
    for (int e = lane; e < E; e += 64) sc[e] /= sum;
  }
  float total = 0.f;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float v = sc[e];
      if (v > best) {
        best = v;
        bi = e;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ob > best || (ob == best && oi < bi)) {
        best = ob;
        bi = oi;
      }
    }
    if (lane == 0) {
      sel_e[(size_t)r * top + j] = bi;
      sel_w[(size_t)r * top + j] = best;
      sc[bi] = -INFINITY;
    }
    total += best;
  }
  if (lane == 0 && (renorm || weight_scale != 1.f))
    for (int j = 0; j < top; ++j) {
      const float v = sel_w[(size_t)r * top + j];
      sel_w[(size_t)r * top + j] = (renorm ? v / (total + renorm_eps) : v) * weight_scale;
    }
}

// An expert's activation from its (scaled) first product a and, when gated, its second product u:
// kind 0 silu(a) u; kind 1 relu(a)^2, an expert of two matrices only.
__device__ __forceinline__ float expert_act(float a, float u, int kind) {
  if (kind == 1) {
    const float p = fmaxf(a, 0.f);
    return p * p;
  }
  return silu_f(a) * u;
}

constexpr int kMoeBM = 32;   // assignment rows per tile of the grouped products
constexpr int kMoeDirect = 16;  // at most this many assignments: each is its own tile, nothing is grouped
// cnt[e] = assignments of expert e.  One workgroup per expert.
__global__ void moe_count_kernel(const int32_t* __restrict__ sel_e, int n, int32_t* __restrict__ cnt) {
  __shared__ float red[4];
  const int e = blockIdx.x;
  float c = 0.f;
  for (int a = threadIdx.x; a < n; a += blockDim.x) c += sel_e[a] == e ? 1.f : 0.f;
  c = block_sum(c, red);
  if (threadIdx.x == 0) cnt[e] = (int)c;
}
// perm: assignments grouped by expert, ascending inside a group; tiles[t] = {expert, first index
// in perm, rows <= bm}; n_tiles[0] = number of tiles.  One workgroup of 256 per expert.
__global__ void moe_group_kernel(const int32_t* __restrict__ sel_e, int n, const int32_t* __restrict__ cnt, int E,
                                 int32_t* __restrict__ perm, int32_t* __restrict__ tiles, int32_t* __restrict__ n_tiles,
                                 int bm) {
  __shared__ int wsum[4];
  __shared__ int base_s;
  const int e = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  int off = 0, toff = 0;
  for (int i = 0; i < e; ++i) {
    off += cnt[i];
    toff += (cnt[i] + bm - 1) / bm;
  }
  const int mine = cnt[e];
  const int my_tiles = (mine + bm - 1) / bm;
  for (int t = tid; t < my_tiles; t += 256) {
    tiles[3 * (toff + t)] = e;
    tiles[3 * (toff + t) + 1] = off + t * bm;
    tiles[3 * (toff + t) + 2] = mine - t * bm < bm ? mine - t * bm : bm;
  }
  if (e == E - 1 && tid == 0) n_tiles[0] = toff + my_tiles;
  if (tid == 0) base_s = 0;
  __syncthreads();
  for (int a0 = 0; a0 < n; a0 += 256) {
    const int a = a0 + tid;
    const bool hit = a < n && sel_e[a] == e;
    const unsigned long long bal = __ballot(hit);
    const int before = __popcll(bal & ((1ull << lane) - 1ull));
    if (lane == 0) wsum[wave] = __popcll(bal);
    __syncthreads();
    int wbase = base_s;
    for (int w = 0; w < wave; ++w) wbase += wsum[w];
    if (hit) perm[off + wbase + before] = a;
    __syncthreads();
    if (tid == 0) base_s += wsum[0] + wsum[1] + wsum[2] + wsum[3];
    __syncthreads();
  }
}

// act[a, n] = silu(s * (gate_e x)) * (s * (up_e x)) for the assignments of one tile (s = weight of
// the assignment when scale_input, else 1).  Each output is summed over k ascending.
template <typename T>
__global__ __launch_bounds__(256) void moe_gate_up_kernel(
    const float* __restrict__ X, int64_t ldx, const int32_t* __restrict__ perm, const int32_t* __restrict__ tiles,
    const int32_t* __restrict__ n_tiles, const float* __restrict__ sel_w, const T* __restrict__ Wgu,
    float* __restrict__ act, int top, int F, int K, int scale_input, int round, int act_kind) {
  constexpr int BM = kMoeBM, BN = 64, BK = 16, TM = 2, TN = 4;
  const bool gated = act_kind == 0;   // (else Wgu holds one matrix [F, K] per expert)
  if (tiles && (int)blockIdx.y >= n_tiles[0]) return;
  __shared__ float xs[BK][BM + 1];
  __shared__ float wg[BK][BN + 1];
  __shared__ float wu[BK][BN + 1];
  __shared__ int arow[BM];
  // (tiles == nullptr: assignment blockIdx.y alone, perm is then the chosen experts themselves)
  const int e = tiles ? tiles[3 * blockIdx.y] : perm[blockIdx.y];
  const int p0 = tiles ? tiles[3 * blockIdx.y + 1] : blockIdx.y, rows = tiles ? tiles[3 * blockIdx.y + 2] : 1;
  const int tid = threadIdx.x, tx = tid % (BN / TN), ty = tid / (BN / TN);
  const int n0 = blockIdx.x * BN;
  const T* Wg = Wgu + (size_t)e * (gated ? 2 : 1) * F * K;
  const T* Wu = gated ? Wg + (size_t)F * K : Wg;
  if (tid < BM) arow[tid] = tid < rows ? (tiles ? perm[p0 + tid] : p0) : -1;
  __syncthreads();
  float ag[TM][TN], au[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) ag[i][j] = au[i][j] = 0.f;
  for (int k0 = 0; k0 < K; k0 += BK) {
    for (int idx = tid; idx < BM * BK; idx += 256) {
      const int m = idx / BK, kk = idx % BK;
      const int a = arow[m];
      xs[kk][m] = (a >= 0 && k0 + kk < K) ? maybe_round(X[(size_t)(a / top) * ldx + k0 + kk], round) : 0.f;
    }
    for (int idx = tid; idx < BN * BK; idx += 256) {
      const int n = idx / BK, kk = idx % BK;
      const bool in = n0 + n < F && k0 + kk < K;
      wg[kk][n] = in ? ld_f(Wg + (size_t)(n0 + n) * K + k0 + kk) : 0.f;
      wu[kk][n] = in && gated ? ld_f(Wu + (size_t)(n0 + n) * K + k0 + kk) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float a[TM], bg[TN], bu[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = xs[kk][ty * TM + i];
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        bg[j] = wg[kk][tx * TN + j];
        bu[j] = wu[kk][tx * TN + j];
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          ag[i][j] = fmaf(a[i], bg[j], ag[i][j]);
          au[i][j] = fmaf(a[i], bu[j], au[i][j]);
        }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int a = arow[ty * TM + i];
    if (a < 0) continue;
    const float s = scale_input ? sel_w[a] : 1.f;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + tx * TN + j;
      if (n < F) act[(size_t)a * F + n] = maybe_round(expert_act(s * ag[i][j], s * au[i][j], act_kind), round);
    }
  }
}

// out[a, n] = (down_e act[a])[n] (times the assignment's weight unless scale_input)
template <typename T>
__global__ __launch_bounds__(256) void moe_down_kernel(
    const float* __restrict__ act, const int32_t* __restrict__ perm, const int32_t* __restrict__ tiles,
    const int32_t* __restrict__ n_tiles, const float* __restrict__ sel_w, const T* __restrict__ Wd,
    float* __restrict__ out, int N, int K, int scale_input) {
  constexpr int BM = kMoeBM, BN = 64, BK = 16, TM = 2, TN = 4;
  if (tiles && (int)blockIdx.y >= n_tiles[0]) return;
  __shared__ float xs[BK][BM + 1];
  __shared__ float ws[BK][BN + 1];
  __shared__ int arow[BM];
  // (tiles == nullptr: assignment blockIdx.y alone, perm is then the chosen experts themselves)
  const int e = tiles ? tiles[3 * blockIdx.y] : perm[blockIdx.y];
  const int p0 = tiles ? tiles[3 * blockIdx.y + 1] : blockIdx.y, rows = tiles ? tiles[3 * blockIdx.y + 2] : 1;
  const int tid = threadIdx.x, tx = tid % (BN / TN), ty = tid / (BN / TN);
  const int n0 = blockIdx.x * BN;
  const T* W = Wd + (size_t)e * N * K;
  if (tid < BM) arow[tid] = tid < rows ? (tiles ? perm[p0 + tid] : p0) : -1;
  __syncthreads();
  float acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = 0.f;
  for (int k0 = 0; k0 < K; k0 += BK) {
    for (int idx = tid; idx < BM * BK; idx += 256) {
      const int m = idx / BK, kk = idx % BK;
      const int a = arow[m];
      xs[kk][m] = (a >= 0 && k0 + kk < K) ? act[(size_t)a * K + k0 + kk] : 0.f;
    }
    for (int idx = tid; idx < BN * BK; idx += 256) {
      const int n = idx / BK, kk = idx % BK;
      ws[kk][n] = (n0 + n < N && k0 + kk < K) ? ld_f(W + (size_t)(n0 + n) * K + k0 + kk) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = xs[kk][ty * TM + i];
#pragma unroll
      for (int j = 0; j < TN; ++j) b[j] = ws[kk][tx * TN + j];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int a = arow[ty * TM + i];
    if (a < 0) continue;
    const float s = scale_input ? 1.f : sel_w[a];
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + tx * TN + j;
      if (n < N) out[(size_t)a * N + n] = s * acc[i][j];
    }
  }
}

// ---- the same two products on the matrix cores (bf16 weights, K a multiple of 32).  A workgroup
// takes one tile of 16*MT assignment rows; its rows are staged in LDS as bf16 in chunks of KC
// columns, every wave reads its weight fragments straight from the row-major matrices (a lane's 8
// consecutive k of one weight row are 16 contiguous bytes).  16x16x32 tiles: operand lane l holds
// row l%16, k-block l/16; result lane l holds rows 4*(l/16)..+3 of column l%16.
__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// act[a, n] (bf16) = silu(s * gate) * (s * up); a wave owns 32 columns of gate and of up.  Xb (or
// nullptr): the rows of X as bf16 already.
template <int MT, int KC, bool GATED>
__global__ __launch_bounds__(256) void moe_gate_up_mfma_kernel(
    const float* __restrict__ X, const bf16_t* __restrict__ Xb, int64_t ldx, const int32_t* __restrict__ perm,
    const int32_t* __restrict__ tiles, const int32_t* __restrict__ n_tiles, const float* __restrict__ sel_w,
    const bf16_t* __restrict__ Wgu, bf16_t* __restrict__ act, int top, int F, int K, int scale_input) {
  if (tiles && (int)blockIdx.y >= n_tiles[0]) return;
  constexpr int BM = 16 * MT, LD = KC + 8;   // LDS row stride: 16 rows at one k fall into distinct banks
  __shared__ __attribute__((aligned(16))) bf16_t xs[BM * LD];
  __shared__ int arow[BM];
  // (tiles == nullptr: assignment blockIdx.y alone, perm is then the chosen experts themselves)
  const int e = tiles ? tiles[3 * blockIdx.y] : perm[blockIdx.y];
  const int p0 = tiles ? tiles[3 * blockIdx.y + 1] : blockIdx.y, rows = tiles ? tiles[3 * blockIdx.y + 2] : 1;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lr = lane & 15, kq = lane >> 4;
  const int n0 = blockIdx.x * 128 + wave * 32 + lr, n1 = n0 + 16;
  constexpr int NM = GATED ? 2 : 1;   // matrices of an expert in Wgu
  const bf16_t* wg0 = Wgu + ((size_t)e * NM * F + (n0 < F ? n0 : F - 1)) * K + 8 * kq;
  const bf16_t* wg1 = Wgu + ((size_t)e * NM * F + (n1 < F ? n1 : F - 1)) * K + 8 * kq;
  const bf16_t* wu0 = GATED ? wg0 + (size_t)F * K : wg0;
  const bf16_t* wu1 = GATED ? wg1 + (size_t)F * K : wg1;
  if (tid < BM) arow[tid] = tid < rows ? (tiles ? perm[p0 + tid] : p0) : -1;
  f32x4 ag[MT][2], au[MT][2];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) ag[mt][0] = ag[mt][1] = au[mt][0] = au[mt][1] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int m_tiles = (rows + 15) / 16;
  for (int kc0 = 0; kc0 < K; kc0 += KC) {
    const int kc = K - kc0 < KC ? K - kc0 : KC;
    __syncthreads();
    if (Xb) {
      for (int idx = tid; idx < 16 * m_tiles * (kc / 8); idx += 256) {
        const int m = idx / (kc / 8), k8 = (idx % (kc / 8)) * 8;
        const int a = arow[m];
        bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
        if (a >= 0) v = *reinterpret_cast<const bf16x8*>(Xb + (size_t)(a / top) * ldx + kc0 + k8);
        *reinterpret_cast<bf16x8*>(xs + m * LD + k8) = v;
      }
    } else {
      for (int idx = tid; idx < 16 * m_tiles * (kc / 4); idx += 256) {
        const int m = idx / (kc / 4), k4 = (idx % (kc / 4)) * 4;
        const int a = arow[m];
        bf16x4 v = {0, 0, 0, 0};
        if (a >= 0) {
          const f32x4 xv = *reinterpret_cast<const f32x4*>(X + (size_t)(a / top) * ldx + kc0 + k4);
          v = bf16x4{(bf16_t)xv[0], (bf16_t)xv[1], (bf16_t)xv[2], (bf16_t)xv[3]};
        }
        *reinterpret_cast<bf16x4*>(xs + m * LD + k4) = v;
      }
    }
    __syncthreads();
#pragma unroll(KC / 32 <= 4 ? KC / 32 : 4)
    for (int k0 = 0; k0 < kc; k0 += 32) {
      const bf16x8 fg0 = *reinterpret_cast<const bf16x8*>(wg0 + kc0 + k0);
      const bf16x8 fg1 = *reinterpret_cast<const bf16x8*>(wg1 + kc0 + k0);
      bf16x8 fu0 = fg0, fu1 = fg1;
      if constexpr (GATED) {
        fu0 = *reinterpret_cast<const bf16x8*>(wu0 + kc0 + k0);
        fu1 = *reinterpret_cast<const bf16x8*>(wu1 + kc0 + k0);
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if (mt < m_tiles) {
          const bf16x8 a = *reinterpret_cast<const bf16x8*>(xs + (16 * mt + lr) * LD + k0 + 8 * kq);
          ag[mt][0] = mfma16(a, fg0, ag[mt][0]);
          ag[mt][1] = mfma16(a, fg1, ag[mt][1]);
          if constexpr (GATED) {
            au[mt][0] = mfma16(a, fu0, au[mt][0]);
            au[mt][1] = mfma16(a, fu1, au[mt][1]);
          }
        }
      }
    }
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int a = arow[mt * 16 + 4 * kq + i];
      if (a < 0) continue;
      const float sc = scale_input ? sel_w[a] : 1.f;
      if (n0 < F) act[(size_t)a * F + n0] = (bf16_t)expert_act(sc * ag[mt][0][i], sc * au[mt][0][i], GATED ? 0 : 1);
      if (n1 < F) act[(size_t)a * F + n1] = (bf16_t)expert_act(sc * ag[mt][1][i], sc * au[mt][1][i], GATED ? 0 : 1);
    }
}

// out[a, n] = down_e act[a]; a wave owns 32 columns.
template <int MT, int KC>
__global__ __launch_bounds__(256) void moe_down_mfma_kernel(
    const bf16_t* __restrict__ act, const int32_t* __restrict__ perm, const int32_t* __restrict__ tiles,
    const int32_t* __restrict__ n_tiles, const float* __restrict__ sel_w, const bf16_t* __restrict__ Wd,
    float* __restrict__ out, int N, int K, int scale_input) {
  if (tiles && (int)blockIdx.y >= n_tiles[0]) return;
  constexpr int BM = 16 * MT, LD = KC + 8;
  __shared__ __attribute__((aligned(16))) bf16_t xs[BM * LD];
  __shared__ int arow[BM];
  const int e = tiles ? tiles[3 * blockIdx.y] : perm[blockIdx.y];
  const int p0 = tiles ? tiles[3 * blockIdx.y + 1] : blockIdx.y, rows = tiles ? tiles[3 * blockIdx.y + 2] : 1;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lr = lane & 15, kq = lane >> 4;
  const int n0 = blockIdx.x * 128 + wave * 32 + lr, n1 = n0 + 16;
  const bf16_t* w0 = Wd + ((size_t)e * N + (n0 < N ? n0 : N - 1)) * K + 8 * kq;
  const bf16_t* w1 = Wd + ((size_t)e * N + (n1 < N ? n1 : N - 1)) * K + 8 * kq;
  if (tid < BM) arow[tid] = tid < rows ? (tiles ? perm[p0 + tid] : p0) : -1;
  f32x4 acc[MT][2];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt][0] = acc[mt][1] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int m_tiles = (rows + 15) / 16;
  for (int kc0 = 0; kc0 < K; kc0 += KC) {
    const int kc = K - kc0 < KC ? K - kc0 : KC;
    __syncthreads();
    for (int idx = tid; idx < 16 * m_tiles * (kc / 8); idx += 256) {
      const int m = idx / (kc / 8), k8 = (idx % (kc / 8)) * 8;
      const int a = arow[m];
      bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
      if (a >= 0) v = *reinterpret_cast<const bf16x8*>(act + (size_t)a * K + kc0 + k8);
      *reinterpret_cast<bf16x8*>(xs + m * LD + k8) = v;
    }
    __syncthreads();
#pragma unroll(KC / 32 <= 8 ? KC / 32 : 8)
    for (int k0 = 0; k0 < kc; k0 += 32) {
      const bf16x8 f0 = *reinterpret_cast<const bf16x8*>(w0 + kc0 + k0);
      const bf16x8 f1 = *reinterpret_cast<const bf16x8*>(w1 + kc0 + k0);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if (mt < m_tiles) {
          const bf16x8 a = *reinterpret_cast<const bf16x8*>(xs + (16 * mt + lr) * LD + k0 + 8 * kq);
          acc[mt][0] = mfma16(a, f0, acc[mt][0]);
          acc[mt][1] = mfma16(a, f1, acc[mt][1]);
        }
      }
    }
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int a = arow[mt * 16 + 4 * kq + i];
      if (a < 0) continue;
      const float sc = scale_input ? 1.f : sel_w[a];
      if (n0 < N) out[(size_t)a * N + n0] = sc * acc[mt][0][i];
      if (n1 < N) out[(size_t)a * N + n1] = sc * acc[mt][1][i];
    }
}

// ---- a few assignments (decoding): each is a matrix-vector product.  A workgroup holds the
// assignment's input row in LDS; a wave owns a few output columns, its lanes stride over k in
// 16-byte pieces of the weight rows (a row is read in whole coalesced lines, all of a wave's
// loads asked for before the first is used), then a butterfly sum.
constexpr int kGemvMaxK = 8192;
// act[a, n] (bf16) = silu(s * gate_e[n] . x) * (s * up_e[n] . x); wave: two columns, gate and up.
// Not gated (an expert's first matrix alone, [F, K]): act[a, n] = relu(s * up_e[n] . x)^2; wave: four columns.
template <bool GATED>
__global__ __launch_bounds__(256) void moe_gemv_gate_up_kernel(
    const float* __restrict__ X, int64_t ldx, const int32_t* __restrict__ sel_e, const float* __restrict__ sel_w,
    const bf16_t* __restrict__ Wgu, bf16_t* __restrict__ act, int top, int F, int K, int scale_input) {
  extern __shared__ float xs[];   // [K]
  const int a = blockIdx.y, e = sel_e[a], tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const float* xr = X + (size_t)(a / top) * ldx;
  for (int k = tid; k < K; k += 256) xs[k] = round_bf16(xr[k]);
  __syncthreads();
  constexpr int COLS = GATED ? 2 : 4;   // output columns of a wave: its four weight rows are gate, up of two, or four rows
  const int n0 = (blockIdx.x * 4 + wave) * COLS;
  if (n0 >= F) return;
  const bf16_t* wg = Wgu + (size_t)e * (GATED ? 2 : 1) * F * K;
  const bf16_t* rows[4];
  if constexpr (GATED) {
    const int n1 = n0 + 1 < F ? n0 + 1 : n0;
    const bf16_t* wu = wg + (size_t)F * K;
    rows[0] = wg + (size_t)n0 * K;
    rows[1] = wu + (size_t)n0 * K;
    rows[2] = wg + (size_t)n1 * K;
    rows[3] = wu + (size_t)n1 * K;
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) rows[j] = wg + (size_t)(n0 + j < F ? n0 + j : n0) * K;
  }
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = lane * 8; k0 < K; k0 += 4 * 512) {
    bf16x8 f[4][4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int k = k0 + 512 * u < K ? k0 + 512 * u : k0;   // unguarded, on an address inside the row
#pragma unroll
      for (int j = 0; j < 4; ++j) f[u][j] = *reinterpret_cast<const bf16x8*>(rows[j] + k);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int k = k0 + 512 * u;
      if (k < K) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float xv = xs[k + i];
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[j] = fmaf(xv, (float)f[u][j][i], acc[j]);
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) acc[j] = wave_sum(acc[j]);
  if (lane == 0) {
    const float sc = scale_input ? sel_w[a] : 1.f;
    if constexpr (GATED) {
      act[(size_t)a * F + n0] = (bf16_t)expert_act(sc * acc[0], sc * acc[1], 0);
      if (n0 + 1 < F) act[(size_t)a * F + n0 + 1] = (bf16_t)expert_act(sc * acc[2], sc * acc[3], 0);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (n0 + j < F) act[(size_t)a * F + n0 + j] = (bf16_t)expert_act(sc * acc[j], 0.f, 1);
    }
  }
}

// out[a, n] = down_e[n] . act[a]; wave: four columns.
__global__ __launch_bounds__(256) void moe_gemv_down_kernel(
    const bf16_t* __restrict__ act, const int32_t* __restrict__ sel_e, const float* __restrict__ sel_w,
    const bf16_t* __restrict__ Wd, float* __restrict__ out, int N, int K, int scale_input) {
  extern __shared__ float xs[];   // [K]
  const int a = blockIdx.y, e = sel_e[a], tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  for (int k = tid; k < K; k += 256) xs[k] = (float)act[(size_t)a * K + k];
  __syncthreads();
  const int n0 = blockIdx.x * 16 + wave * 4;
  if (n0 >= N) return;
  const bf16_t* w = Wd + (size_t)e * N * K;
  const bf16_t* rows[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) rows[j] = w + (size_t)(n0 + j < N ? n0 + j : n0) * K;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = lane * 8; k0 < K; k0 += 4 * 512) {
    bf16x8 f[4][4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int k = k0 + 512 * u < K ? k0 + 512 * u : k0;
#pragma unroll
      for (int j = 0; j < 4; ++j) f[u][j] = *reinterpret_cast<const bf16x8*>(rows[j] + k);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int k = k0 + 512 * u;
      if (k < K) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float xv = xs[k + i];
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[j] = fmaf(xv, (float)f[u][j][i], acc[j]);
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) acc[j] = wave_sum(acc[j]);
  if (lane == 0) {
    const float sc = scale_input ? 1.f : sel_w[a];
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (n0 + j < N) out[(size_t)a * N + n0 + j] = sc * acc[j];
  }
}

struct MoeScratch {
  size_t cnt, n_tiles, perm, tiles, act, total;
};
inline size_t al256(size_t v) { return (v + 255) & ~(size_t)255; }
MoeScratch moe_plan(int n_rows, int top, int E, int F) {
  MoeScratch s;
  const size_t n = (size_t)n_rows * top;
  size_t off = 0;
  s.cnt = off;     off += al256(sizeof(int32_t) * E);
  s.n_tiles = off; off += al256(sizeof(int32_t));
  s.perm = off;    off += al256(sizeof(int32_t) * n);
  s.tiles = off;   off += al256(sizeof(int32_t) * 3 * (n / kMoeBM + E + 1));
  s.act = off;     off += al256(sizeof(float) * n * F);
  s.total = off;
  return s;
}

// ------------------------------------------------------------------ residual update, norm on the output
template <typename T>
__global__ void postnorm_residual_kernel(float* __restrict__ x, const float* __restrict__ a, int n_a, float sa,
                                         const float* __restrict__ b, float sb, const T* __restrict__ w, float eps,
                                         bf16_t* __restrict__ x_b, int W) {
  __shared__ float red[4];
  const int r = blockIdx.x;
  auto term = [&](int c) {
    float v = a[((size_t)r * n_a) * W + c];
    for (int j = 1; j < n_a; ++j) v += a[((size_t)r * n_a + j) * W + c];
    v *= sa;
    if (b) v += sb * b[(size_t)r * W + c];
    return v;
  };
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float v = term(c);
    ss = fmaf(v, v, ss);
  }
  ss = block_sum(ss, red);
  const float rstd = 1.f / sqrtf(ss / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float xn = x[(size_t)r * W + c] + term(c) * rstd * ld_f(w + c);
    x[(size_t)r * W + c] = xn;
    if (x_b) x_b[(size_t)r * W + c] = (bf16_t)xn;
  }
}

// A layer normed before and after its sublayers, per row, in one launch:
//   t = the sum of the row's n_a rows of a (+ sigmoid(b_gate[r]) * b[r]);  x += rms_norm(t) * w_post
// (a == nullptr: no update); x_copy (or nullptr) receives the row as it is then; x += add (a
// vector [W], or nullptr); unless w_next == nullptr, h = rms_norm(x) * w_next, the input of the
// sublayer that follows (h_b: the same as bf16).  The row is held in LDS between the steps.
template <typename T>
__global__ __launch_bounds__(256) void residual_norm_kernel(
    float* __restrict__ x, const float* __restrict__ a, int n_a, const float* __restrict__ b,
    const float* __restrict__ b_gate, int64_t ldg, const T* __restrict__ w_post, const T* __restrict__ add,
    const T* __restrict__ w_next, float eps, float* __restrict__ x_copy, float* __restrict__ h,
    bf16_t* __restrict__ h_b, int W, int round, const T* __restrict__ a_bias, float mult) {
  extern __shared__ float row[];   // [W]
  __shared__ float red[4];
  const int r = blockIdx.x;
  float rstd = 0.f;
  if (a) {
    const float gate = b ? (b_gate ? sigmoid_f(b_gate[(size_t)r * ldg]) : 1.f) : 0.f;
    float ss = 0.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
      float v = a[((size_t)r * n_a) * W + c];
      for (int j = 1; j < n_a; ++j) v += a[((size_t)r * n_a + j) * W + c];
      if (b) v += gate * b[(size_t)r * W + c];
      if (a_bias) v += ld_f(a_bias + c);
      row[c] = v;
      ss = fmaf(v, v, ss);
    }
    ss = block_sum(ss, red);
    rstd = 1.f / sqrtf(ss / (float)W + eps);
  }
  float ss2 = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float xn = x[(size_t)r * W + c];
    if (a) xn += mult * (row[c] * rstd * ld_f(w_post + c));
    if (x_copy) x_copy[(size_t)r * W + c] = xn;
    if (add) xn += ld_f(add + c);
    if (a || add) x[(size_t)r * W + c] = xn;
    row[c] = xn;
    ss2 = fmaf(xn, xn, ss2);
  }
  if (!w_next) return;
  ss2 = block_sum(ss2, red);
  const float rstd2 = 1.f / sqrtf(ss2 / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float v = maybe_round(row[c] * rstd2 * ld_f(w_next + c), round);
    if (h) h[(size_t)r * W + c] = v;
    if (h_b) h_b[(size_t)r * W + c] = (bf16_t)v;
  }
}

// The same update four columns per thread (W a multiple of 4, rows 16-byte aligned), for up to
// 1024 threads: a row of a few thousand columns is one or two pieces per thread, so every phase
// waits for memory once.  Sums go lane -> wave -> workgroup in a fixed order.
template <typename T> struct Quad;
template <> struct Quad<float> {
  static __device__ __forceinline__ f32x4 ld(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
};
template <> struct Quad<bf16_t> {
  static __device__ __forceinline__ f32x4 ld(const bf16_t* p) {
    const bf16x4 v = *reinterpret_cast<const bf16x4*>(p);
    return f32x4{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
  }
};
__device__ __forceinline__ float block_sum_wide(float v, float* red) {   // up to 16 waves
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6, n_waves = (blockDim.x + 63) >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[wave] = v;
  __syncthreads();
  float s = red[0];
  for (int w = 1; w < n_waves; ++w) s += red[w];
  return s;
}
template <typename T>
__global__ __launch_bounds__(1024) void residual_norm_quad_kernel(
    float* __restrict__ x, const float* __restrict__ a, int n_a, const float* __restrict__ b,
    const float* __restrict__ b_gate, int64_t ldg, const T* __restrict__ w_post, const T* __restrict__ add,
    const T* __restrict__ w_next, float eps, float* __restrict__ x_copy, float* __restrict__ h,
    bf16_t* __restrict__ h_b, int W, int round, const T* __restrict__ a_bias, float mult) {
  extern __shared__ float row[];   // [W]
  __shared__ float red[16];
  const int r = blockIdx.x, nq = W / 4;
  float rstd = 0.f;
  if (a) {
    const float gate = b ? (b_gate ? sigmoid_f(b_gate[(size_t)r * ldg]) : 1.f) : 0.f;
    float ss = 0.f;
    for (int c = threadIdx.x; c < nq; c += blockDim.x) {
      f32x4 v = Quad<float>::ld(a + ((size_t)r * n_a) * W + 4 * c);
      for (int j = 1; j < n_a; ++j) v += Quad<float>::ld(a + ((size_t)r * n_a + j) * W + 4 * c);
      if (b) v += gate * Quad<float>::ld(b + (size_t)r * W + 4 * c);
      if (a_bias) v += Quad<T>::ld(a_bias + 4 * c);
      *reinterpret_cast<f32x4*>(row + 4 * c) = v;
#pragma unroll
      for (int i = 0; i < 4; ++i) ss = fmaf(v[i], v[i], ss);
    }
    ss = block_sum_wide(ss, red);
    rstd = 1.f / sqrtf(ss / (float)W + eps);
  }
  float ss2 = 0.f;
  for (int c = threadIdx.x; c < nq; c += blockDim.x) {
    f32x4 xn = Quad<float>::ld(x + (size_t)r * W + 4 * c);
    if (a) {
      const f32x4 t = *reinterpret_cast<const f32x4*>(row + 4 * c), wp = Quad<T>::ld(w_post + 4 * c);
#pragma unroll
      for (int i = 0; i < 4; ++i) xn[i] += mult * (t[i] * rstd * wp[i]);
    }
    if (x_copy) *reinterpret_cast<f32x4*>(x_copy + (size_t)r * W + 4 * c) = xn;
    if (add) xn += Quad<T>::ld(add + 4 * c);
    if (a || add) *reinterpret_cast<f32x4*>(x + (size_t)r * W + 4 * c) = xn;
    *reinterpret_cast<f32x4*>(row + 4 * c) = xn;
#pragma unroll
    for (int i = 0; i < 4; ++i) ss2 = fmaf(xn[i], xn[i], ss2);
  }
  if (!w_next) return;
  ss2 = block_sum_wide(ss2, red);
  const float rstd2 = 1.f / sqrtf(ss2 / (float)W + eps);
  for (int c = threadIdx.x; c < nq; c += blockDim.x) {
    const f32x4 xn = *reinterpret_cast<const f32x4*>(row + 4 * c), wn = Quad<T>::ld(w_next + 4 * c);
    f32x4 v;
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = maybe_round(xn[i] * rstd2 * wn[i], round);
    if (h) *reinterpret_cast<f32x4*>(h + (size_t)r * W + 4 * c) = v;
    if (h_b) *reinterpret_cast<bf16x4*>(h_b + (size_t)r * W + 4 * c) = bf16x4{(bf16_t)v[0], (bf16_t)v[1], (bf16_t)v[2], (bf16_t)v[3]};
  }
}

__global__ void scale_rows_kernel(float* __restrict__ x, int64_t ld, float s, int n_cols) {
  const int r = blockIdx.x;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < n_cols; c += gridDim.y * blockDim.x)
    x[(size_t)r * ld + c] *= s;
}

}  // namespace

// ====================================================================== C entry points
extern "C" int sd_embed_hashed(const int32_t* tokens, const int32_t* prev_tokens, const void* table,
                               const void* bigram, int w_f32, float scale, int buckets, int mul_prev, int mul_cur,
                               float* x, void* x_bf16, int n_rows, int W, int vocab, sd_stream_t stream) {
  SD_REQUIRE(tokens && table && x && n_rows >= 1 && W >= 1 && vocab >= 1, SD_ERR_INVALID, "sd_embed_hashed: bad argument");
  SD_REQUIRE(!bigram || buckets >= 1, SD_ERR_INVALID, "sd_embed_hashed: a bigram table needs buckets >= 1");
  hipStream_t st = (hipStream_t)stream;
  if (w_f32)
    embed_hashed_kernel<float><<<n_rows, 256, 0, st>>>(tokens, prev_tokens, (const float*)table, (const float*)bigram,
                                                       scale, buckets, mul_prev, mul_cur, x, (bf16_t*)x_bf16, W, vocab);
  else
    embed_hashed_kernel<bf16_t><<<n_rows, 256, 0, st>>>(tokens, prev_tokens, (const bf16_t*)table, (const bf16_t*)bigram,
                                                        scale, buckets, mul_prev, mul_cur, x, (bf16_t*)x_bf16, W, vocab);
  SD_CHECK_LAUNCH("sd_embed_hashed");
  return SD_OK;
}

extern "C" int sd_rmsnorm_parts(const float* x, int64_t ldx, const float* gate, int64_t ldg, const void* w, int w_f32,
                                float eps, float* out, int64_t ldo, void* out_bf16, int64_t ldob, int n_rows,
                                int width, int parts, int round_bf16_out, sd_stream_t stream) {
  SD_REQUIRE(x && out && n_rows >= 1 && width >= 1 && parts >= 1 && width % parts == 0 && ldx >= width && ldo >= width,
             SD_ERR_INVALID, "sd_rmsnorm_parts: bad argument (width %d in %d parts)", width, parts);
  hipStream_t st = (hipStream_t)stream;
  dim3 grid(n_rows, parts);
  const int pw = width / parts;
  if (w_f32)
    rmsnorm_parts_kernel<float><<<grid, 256, 0, st>>>(x, ldx, gate, ldg, (const float*)w, eps, out, ldo,
                                                      (bf16_t*)out_bf16, ldob, pw, round_bf16_out);
  else
    rmsnorm_parts_kernel<bf16_t><<<grid, 256, 0, st>>>(x, ldx, gate, ldg, (const bf16_t*)w, eps, out, ldo,
                                                       (bf16_t*)out_bf16, ldob, pw, round_bf16_out);
  SD_CHECK_LAUNCH("sd_rmsnorm_parts");
  return SD_OK;
}

extern "C" int sd_rope_copy_rows(const float* src, int64_t ld_src, int src_head_stride, int src_offset, float* dst,
                                 int64_t ld_dst, int dst_head_stride, int dst_offset, const int32_t* row_pos,
                                 int n_rows, int heads, int n, int rot_dims, int rot_layout, const double* inv_freq,
                                 float mag, sd_stream_t stream) {
  SD_REQUIRE(src && dst && row_pos && n_rows >= 1 && heads >= 1 && src_offset >= 0 && dst_offset >= 0 && n >= 0,
             SD_ERR_INVALID, "sd_rope_copy_rows: bad argument");
  SD_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= n && (rot_dims == 0 || inv_freq), SD_ERR_INVALID,
             "sd_rope_copy_rows: rot_dims %d must be even, at most %d, with a frequency table", rot_dims, n);
  if (n == 0 || (rot_dims == 0 && src == dst)) return SD_OK;
  rope_copy_kernel<<<dim3(n_rows, heads), 64, 0, (hipStream_t)stream>>>(src, ld_src, src_head_stride, src_offset, dst,
                                                                        ld_dst, dst_head_stride, dst_offset, row_pos, n,
                                                                        rot_dims, rot_layout, inv_freq, mag);
  SD_CHECK_LAUNCH("sd_rope_copy_rows");
  return SD_OK;
}

extern "C" int sd_rope_rows(float* x, int64_t ld, const int32_t* row_pos, int n_rows, int heads, int head_stride,
                            int offset, int rot_dims, int rot_layout, const double* inv_freq, float mag,
                            sd_stream_t stream) {
  return sd_rope_copy_rows(x, ld, head_stride, offset, x, ld, head_stride, offset, row_pos, n_rows, heads, rot_dims,
                           rot_dims, rot_layout, inv_freq, mag, stream);
}

extern "C" int sd_latent_prep(float* q_latent, int q_rank, const void* q_norm_w, void* q_bf16, int64_t ld_q_bf16,
                              float* kv, int kv_rank, int rot_dim, const void* kv_norm_w, int64_t ld, int w_f32,
                              float eps, int rot_dims, int rot_layout, const double* inv_freq, float mag, void* k_cache,
                              const int32_t* row_pos, const int32_t* row_slot, const int32_t* block_tables,
                              int max_blocks, int page, int n_rows, sd_stream_t stream) {
  SD_REQUIRE((!q_latent || q_norm_w) && kv && kv_norm_w && k_cache && row_pos && row_slot && block_tables, SD_ERR_INVALID,
             "sd_latent_prep: null argument");
  SD_REQUIRE(n_rows >= 1 && (!q_latent || q_rank >= 1) && kv_rank >= 1 && rot_dim >= 0 && page >= 1 && max_blocks >= 1, SD_ERR_INVALID,
             "sd_latent_prep: bad shape");
  SD_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= rot_dim && (rot_dims == 0 || inv_freq), SD_ERR_INVALID,
             "sd_latent_prep: rot_dims %d must be even, at most rot_dim %d, with a frequency table", rot_dims, rot_dim);
  hipStream_t st = (hipStream_t)stream;
  dim3 grid(n_rows, q_latent ? 2 : 1);   // (queries that come straight from the input have no latent to norm)
  if (w_f32)
    latent_prep_kernel<float><<<grid, 256, 0, st>>>(q_latent, q_rank, (const float*)q_norm_w, (bf16_t*)q_bf16, ld_q_bf16,
                                                    kv, kv_rank, rot_dim, (const float*)kv_norm_w, ld, eps, 0, rot_dims,
                                                    rot_layout, inv_freq, mag, row_pos, row_slot, block_tables,
                                                    max_blocks, page, (float*)k_cache);
  else
    latent_prep_kernel<bf16_t><<<grid, 256, 0, st>>>(q_latent, q_rank, (const bf16_t*)q_norm_w, (bf16_t*)q_bf16,
                                                     ld_q_bf16, kv, kv_rank, rot_dim, (const bf16_t*)kv_norm_w, ld, eps, 1,
                                                     rot_dims, rot_layout, inv_freq, mag, row_pos, row_slot, block_tables,
                                                     max_blocks, page, (bf16_t*)k_cache);
  SD_CHECK_LAUNCH("sd_latent_prep");
  return SD_OK;
}

extern "C" int sd_qk_norm_append(float* q, int n_q, const void* q_norm_w, float* k, int G, int dk, const void* k_norm_w,
                                 const float* v, int dv, int64_t ld, int w_f32, float eps, void* k_cache, void* v_cache,
                                 const int32_t* row_pos, const int32_t* row_slot, const int32_t* block_tables,
                                 int max_blocks, int page, int n_rows, sd_stream_t stream) {
  SD_REQUIRE(q && q_norm_w && k && k_norm_w && v && k_cache && v_cache && row_pos && row_slot && block_tables,
             SD_ERR_INVALID, "sd_qk_norm_append: null argument");
  SD_REQUIRE(n_rows >= 1 && n_q >= 1 && G >= 1 && dk >= 1 && dv >= 1 && page >= 1 && max_blocks >= 1, SD_ERR_INVALID,
             "sd_qk_norm_append: bad shape");
  hipStream_t st = (hipStream_t)stream;
  dim3 grid(n_rows, 2);
  if (w_f32)
    qk_norm_append_kernel<float><<<grid, 256, 0, st>>>(q, n_q, (const float*)q_norm_w, k, G, dk, (const float*)k_norm_w, v,
                                                       dv, ld, eps, row_pos, row_slot, block_tables, max_blocks, page,
                                                       (float*)k_cache, (float*)v_cache);
  else
    qk_norm_append_kernel<bf16_t><<<grid, 256, 0, st>>>(q, n_q, (const bf16_t*)q_norm_w, k, G, dk, (const bf16_t*)k_norm_w,
                                                        v, dv, ld, eps, row_pos, row_slot, block_tables, max_blocks, page,
                                                        (bf16_t*)k_cache, (bf16_t*)v_cache);
  SD_CHECK_LAUNCH("sd_qk_norm_append");
  return SD_OK;
}

extern "C" int sd_qk_head_norm_append(float* q, int H, const void* q_norm_w, float* k, int G, int dk,
                                      const void* k_norm_w, const float* v, int dv, int64_t ld, int w_f32, float eps,
                                      void* k_cache, void* v_cache, const int32_t* row_pos, const int32_t* row_slot,
                                      const int32_t* block_tables, int max_blocks, int page, int n_rows,
                                      sd_stream_t stream) {
  SD_REQUIRE(q && q_norm_w && k && k_norm_w && v && k_cache && v_cache && row_pos && row_slot && block_tables,
             SD_ERR_INVALID, "sd_qk_head_norm_append: null argument");
  SD_REQUIRE(n_rows >= 1 && H >= 1 && G >= 1 && dk >= 1 && dv >= 1 && page >= 1 && max_blocks >= 1, SD_ERR_INVALID,
             "sd_qk_head_norm_append: bad shape");
  hipStream_t st = (hipStream_t)stream;
  dim3 grid(n_rows, 2);
  if (w_f32)
    qk_head_norm_append_kernel<float><<<grid, 256, 0, st>>>(q, H, (const float*)q_norm_w, k, G, dk,
                                                            (const float*)k_norm_w, v, dv, ld, eps, row_pos, row_slot,
                                                            block_tables, max_blocks, page, (float*)k_cache,
                                                            (float*)v_cache);
  else
    qk_head_norm_append_kernel<bf16_t><<<grid, 256, 0, st>>>(q, H, (const bf16_t*)q_norm_w, k, G, dk,
                                                             (const bf16_t*)k_norm_w, v, dv, ld, eps, row_pos, row_slot,
                                                             block_tables, max_blocks, page, (bf16_t*)k_cache,
                                                             (bf16_t*)v_cache);
  SD_CHECK_LAUNCH("sd_qk_head_norm_append");
  return SD_OK;
}

extern "C" int sd_attn_prep(float* q, int n_q_units, float* k, int n_k_units, int dk, const float* v, int G, int dv,
                            int value_from_key, int64_t ld, const void* q_bias, const void* k_bias, int norm_kind,
                            const void* q_norm_w, const void* k_norm_w, int w_f32, float eps, int rot_dims,
                            int rot_layout, const double* inv_freq, float mag, void* k_cache, void* v_cache,
                            const int32_t* row_pos, const int32_t* row_slot, const int32_t* block_tables,
                            int max_blocks, int page, int n_rows, sd_stream_t stream) {
  SD_REQUIRE(q && row_pos && n_rows >= 1 && n_q_units >= 1 && dk >= 1 && ld >= (int64_t)n_q_units * dk, SD_ERR_INVALID,
             "sd_attn_prep: bad argument");
  SD_REQUIRE(norm_kind >= 0 && norm_kind <= 2 && (norm_kind == 0 || (q_norm_w && (!k || k_norm_w))), SD_ERR_INVALID,
             "sd_attn_prep: norm kind %d unknown, or a norm without its weights", norm_kind);
  SD_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= dk && (rot_dims == 0 || inv_freq), SD_ERR_INVALID,
             "sd_attn_prep: rotary dims %d (dim %d)", rot_dims, dk);
  if (k) {
    SD_REQUIRE(n_k_units >= 1 && G >= 1 && dv >= 1 && k_cache && v_cache && row_slot && block_tables && page >= 1 &&
                   max_blocks >= 1 && ld >= (int64_t)n_k_units * dk,
               SD_ERR_INVALID, "sd_attn_prep: keys without their caches or page table");
    SD_REQUIRE(value_from_key ? (int64_t)G * dv == (int64_t)n_k_units * dk : (v != nullptr && ld >= (int64_t)G * dv),
               SD_ERR_INVALID, "sd_attn_prep: values missing, or values taken from keys of another size");
  }
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid(n_rows, k ? 2 : 1);
  if (w_f32)
    attn_prep_kernel<float><<<grid, 256, sizeof(float) * (rot_dims > 0 ? rot_dims : 1), st>>>(q, n_q_units, k, n_k_units, dk, v, G, dv, value_from_key, ld,
                                                  (const float*)q_bias, (const float*)k_bias, norm_kind,
                                                  (const float*)q_norm_w, (const float*)k_norm_w, eps, rot_dims,
                                                  rot_layout, inv_freq, mag, row_pos, row_slot, block_tables,
                                                  max_blocks, page, (float*)k_cache, (float*)v_cache);
  else
    attn_prep_kernel<bf16_t><<<grid, 256, sizeof(float) * (rot_dims > 0 ? rot_dims : 1), st>>>(q, n_q_units, k, n_k_units, dk, v, G, dv, value_from_key, ld,
                                                   (const bf16_t*)q_bias, (const bf16_t*)k_bias, norm_kind,
                                                   (const bf16_t*)q_norm_w, (const bf16_t*)k_norm_w, eps, rot_dims,
                                                   rot_layout, inv_freq, mag, row_pos, row_slot, block_tables,
                                                   max_blocks, page, (bf16_t*)k_cache, (bf16_t*)v_cache);
  SD_CHECK_LAUNCH("sd_attn_prep");
  return SD_OK;
}

extern "C" int sd_diff_combine_rows(const float* a, float lambda, float eps, float out_scale, float* y, void* y_bf16,
                                    int n_rows, int H, int dv, int round_bf16_out, sd_stream_t stream) {
  SD_REQUIRE(a && y && n_rows >= 1 && H >= 1 && dv >= 1, SD_ERR_INVALID, "sd_diff_combine_rows: bad argument");
  const long long pairs = (long long)n_rows * H;
  SD_REQUIRE(pairs <= 0x7fffffff, SD_ERR_UNSUPPORTED, "sd_diff_combine_rows: too many (row, head) pairs");
  diff_combine_kernel<<<(unsigned)((pairs + 3) / 4), 256, 0, (hipStream_t)stream>>>(a, lambda, eps, out_scale, y,
                                                                                   (bf16_t*)y_bf16, (int)pairs, dv,
                                                                                   round_bf16_out);
  SD_CHECK_LAUNCH("sd_diff_combine_rows");
  return SD_OK;
}

extern "C" int sd_head_gate_rows(float* y, int64_t ldy, const float* z, int64_t ldz, void* y_bf16, int64_t ldyb,
                                 int n_rows, int H, int dv, int round_bf16_out, sd_stream_t stream) {
  SD_REQUIRE(y && z && n_rows >= 1 && H >= 1 && dv >= 1 && ldy >= (int64_t)H * dv && ldz >= H, SD_ERR_INVALID,
             "sd_head_gate_rows: bad argument");
  int by = (H * dv + 255) / 256;
  if (by > 32) by = 32;
  head_gate_kernel<<<dim3(n_rows, by), 256, 0, (hipStream_t)stream>>>(y, ldy, z, ldz, (bf16_t*)y_bf16, ldyb, H, dv,
                                                                      round_bf16_out);
  SD_CHECK_LAUNCH("sd_head_gate_rows");
  return SD_OK;
}

extern "C" int sd_act_rows(const float* gate, const float* up, int64_t ld, float* out, int64_t ldo, void* out_bf16,
                           int64_t ldob, int n_rows, int F, int act_kind, int round_bf16_out, sd_stream_t stream) {
  SD_REQUIRE(gate && (out || out_bf16) && n_rows >= 1 && F >= 1 && ld >= F, SD_ERR_INVALID, "sd_act_rows: bad argument");
  SD_REQUIRE(act_kind >= 0 && act_kind <= 2 && (act_kind == 2 || up), SD_ERR_INVALID,
             "sd_act_rows: activation %d unknown, or a gated one without its second input", act_kind);
  int by = (F + 255) / 256;
  if (by > 64) by = 64;
  act_rows_kernel<<<dim3(n_rows, by), 256, 0, (hipStream_t)stream>>>(gate, up, ld, out, ldo, (bf16_t*)out_bf16, ldob, F,
                                                                     act_kind, round_bf16_out);
  SD_CHECK_LAUNCH("sd_act_rows");
  return SD_OK;
}

extern "C" int sd_cache_append(const float* k, int64_t ldk, const float* v, int64_t ldv, void* k_cache, void* v_cache,
                               int cache_f32, const int32_t* row_pos, const int32_t* row_slot,
                               const int32_t* block_tables, int max_blocks, int page, int n_rows, int G, int dk, int dv,
                               sd_stream_t stream) {
  SD_REQUIRE(k && k_cache && row_pos && row_slot && block_tables && n_rows >= 1 && G >= 1 && dk >= 1 && page >= 1 &&
                 max_blocks >= 1 && (!v || (v_cache && dv >= 1)),
             SD_ERR_INVALID, "sd_cache_append: bad argument");
  hipStream_t st = (hipStream_t)stream;
  dim3 grid(n_rows, G);
  if (cache_f32)
    cache_append_kernel<float><<<grid, 128, 0, st>>>(k, ldk, v, ldv, (float*)k_cache, (float*)v_cache, row_pos, row_slot,
                                                     block_tables, max_blocks, page, G, dk, dv);
  else
    cache_append_kernel<bf16_t><<<grid, 128, 0, st>>>(k, ldk, v, ldv, (bf16_t*)k_cache, (bf16_t*)v_cache, row_pos,
                                                      row_slot, block_tables, max_blocks, page, G, dk, dv);
  SD_CHECK_LAUNCH("sd_cache_append");
  return SD_OK;
}

extern "C" size_t sd_masked_softmax_attention_scratch_bytes(int n_rows, int H, int dv, int window, int keep_first,
                                                             int chunk, int max_ctx) {
  return sd_multimap_softmax_attention_scratch_bytes(n_rows, H, 1, dv, window, keep_first, chunk, max_ctx);
}

extern "C" size_t sd_multimap_softmax_attention_scratch_bytes(int n_rows, int H, int maps, int dv, int window,
                                                               int keep_first, int chunk, int max_ctx) {
  if (n_rows < 1 || n_rows > kSplitRows || H < 1 || maps < 1 || dv < 1 || window < 1) return 0;
  H *= maps;
  long long max_keys = (long long)(chunk > 0 && chunk < window ? chunk : window) + (keep_first > 0 ? keep_first : 0);
  if (max_keys > max_ctx) max_keys = max_ctx;
  const int splits = (int)((max_keys + kSplitKeys - 1) / kSplitKeys);
  return splits > 1 ? (size_t)splits * n_rows * H * (dv + 2) * sizeof(float) : 0;
}

extern "C" int sd_masked_softmax_attention(const float* q, int64_t ldq, const void* k_cache, const void* v_cache,
                                           int cache_f32, const int32_t* row_pos, const int32_t* row_slot,
                                           const int32_t* block_tables, int max_blocks, int page, int n_rows, int H,
                                           int G, int dk, int dv, int window, int keep_first, int chunk, float scale,
                                           float softcap, const float* sinks, float* out, void* out_bf16,
                                           void* scratch, size_t scratch_bytes, sd_stream_t stream) {
  return sd_multimap_softmax_attention(q, ldq, k_cache, v_cache, cache_f32, row_pos, row_slot, block_tables, max_blocks,
                                       page, n_rows, H, G, 1, dk, dv, window, keep_first, chunk, scale, softcap, sinks,
                                       out, out_bf16, scratch, scratch_bytes, stream);
}

extern "C" int sd_multimap_softmax_attention(const float* q, int64_t ldq, const void* k_cache, const void* v_cache,
                                             int cache_f32, const int32_t* row_pos, const int32_t* row_slot,
                                             const int32_t* block_tables, int max_blocks, int page, int n_rows, int H,
                                             int G, int maps, int dk, int dv, int window, int keep_first, int chunk,
                                             float scale, float softcap, const float* sinks, float* out,
                                             void* out_bf16, void* scratch, size_t scratch_bytes, sd_stream_t stream) {
  SD_REQUIRE(q && k_cache && row_pos && row_slot && block_tables && out, SD_ERR_INVALID,
             "sd_masked_softmax_attention: null argument");
  SD_REQUIRE(n_rows >= 1 && H >= 1 && G >= 1 && H % G == 0 && dk >= 1 && window >= 1 && keep_first >= 0 && page >= 1 &&
                 chunk >= 0 && softcap >= 0.f && maps >= 1 && (maps == 1 || v_cache) &&
                 ldq >= (int64_t)H * maps * dk,
             SD_ERR_INVALID, "sd_masked_softmax_attention: bad shape");
  SD_REQUIRE(dv >= 1 && dv <= 512 && (v_cache || dv <= dk), SD_ERR_UNSUPPORTED,
             "sd_masked_softmax_attention: value size %d outside 1..512 (or above the key row it is part of)", dv);
  hipStream_t st = (hipStream_t)stream;
  const int qh = H / G;
  const int HM = H * maps;
  const size_t need = sd_multimap_softmax_attention_scratch_bytes(n_rows, H, maps, dv, window, keep_first, chunk,
                                                                  max_blocks * page);
  const bool split = need > 0 && scratch && scratch_bytes >= need && sd_aligned16(scratch);
  const int n_splits = split ? (int)(need / ((size_t)n_rows * HM * (dv + 2) * sizeof(float))) : 1;
  const int kt = split ? kSplitKeys : 256;   // keys per tile
  // (a cut launch has many workgroups already: fewer heads each, so that a thread scores its key sooner)
  const int cap = split ? 4 : 8;
  const int NH = qh <= 1 ? 1 : (qh <= 2 ? 2 : (qh <= 4 || cap == 4 ? 4 : 8));
  const int n_hgroups = (qh + NH - 1) / NH;
  const int nc = dv <= 64 ? 1 : (dv <= 128 ? 2 : (dv <= 256 ? 4 : 8));
  const size_t lds = sizeof(unsigned long long) * kt +
                     sizeof(float) * ((size_t)NH * kt + (size_t)NH * dk + 3 * (size_t)NH + (size_t)4 * dv +
                                      (kt < 256 ? (size_t)(256 / kt) * NH * kt : 0));
  SD_REQUIRE(lds <= 64 * 1024, SD_ERR_UNSUPPORTED, "sd_masked_softmax_attention: dim %d / vdim %d need %zu bytes of LDS",
             dk, dv, lds);
  const void* vc = v_cache ? v_cache : k_cache;
  const int v_row = v_cache ? dv : dk;
  float* part_acc = split ? (float*)scratch : nullptr;
  float* part_ml = split ? part_acc + (size_t)n_splits * n_rows * HM * dv : nullptr;
  dim3 grid(n_rows, G * maps, n_hgroups * n_splits);
#define SD_NH(T, N)                                                                                                  \
  launch_softmax_nc<T, N>(grid, kt, lds, st, nc, q, ldq, k_cache, vc, v_row, row_pos, row_slot, block_tables,      \
                          max_blocks, page, H, G, dk, dv, window, keep_first, scale, out, (bf16_t*)out_bf16, n_hgroups, \
                          n_splits, part_acc, part_ml, chunk, softcap, sinks, maps)
#define SD_T(T)                      \
  do {                               \
    if (NH == 1) SD_NH(T, 1);        \
    else if (NH == 2) SD_NH(T, 2);   \
    else if (NH == 4) SD_NH(T, 4);   \
    else SD_NH(T, 8);                \
  } while (0)
  if (cache_f32) SD_T(float);
  else SD_T(bf16_t);
#undef SD_T
#undef SD_NH
  SD_CHECK_LAUNCH("sd_masked_softmax_attention");
  if (split) {
    softmax_merge_kernel<<<dim3(n_rows, HM), dv <= 64 ? 64 : (dv <= 128 ? 128 : 256), sizeof(float) * n_splits, st>>>(
        part_acc, part_ml, n_splits, out, (bf16_t*)out_bf16, HM, dv);
    SD_CHECK_LAUNCH("sd_masked_softmax_attention (merge)");
  }
  return SD_OK;
}

extern "C" size_t sd_window_softmax_attention_scratch_bytes(int n_rows, int H, int dv, int window, int keep_first,
                                                             int max_ctx) {
  return sd_masked_softmax_attention_scratch_bytes(n_rows, H, dv, window, keep_first, 0, max_ctx);
}

extern "C" int sd_window_softmax_attention(const float* q, int64_t ldq, const void* k_cache, const void* v_cache,
                                           int cache_f32, const int32_t* row_pos, const int32_t* row_slot,
                                           const int32_t* block_tables, int max_blocks, int page, int n_rows, int H,
                                           int G, int dk, int dv, int window, int keep_first, float scale, float* out,
                                           void* out_bf16, void* scratch, size_t scratch_bytes, sd_stream_t stream) {
  return sd_masked_softmax_attention(q, ldq, k_cache, v_cache, cache_f32, row_pos, row_slot, block_tables, max_blocks,
                                     page, n_rows, H, G, dk, dv, window, keep_first, 0, scale, 0.f, nullptr, out,
                                     out_bf16, scratch, scratch_bytes, stream);
}

extern "C" int sd_causal_conv_rows(const float* x, int64_t ldx, const void* w, const void* b, int w_f32,
                                   float* conv_state, const int32_t* row_pos, const int32_t* row_slot,
                                   const int32_t* entries, int n_entries, float* out, int64_t ldo, int n_rows, int C,
                                   int taps, int act, sd_stream_t stream) {
  SD_REQUIRE(x && w && conv_state && row_pos && row_slot && entries && out && n_entries >= 1 && n_rows >= 1 && C >= 1 &&
                 taps >= 1 && ldx >= C && ldo >= C,
             SD_ERR_INVALID, "sd_causal_conv_rows: bad argument");
  SD_REQUIRE(out != x, SD_ERR_INVALID, "sd_causal_conv_rows: not in place (rows read their predecessors)");
  hipStream_t st = (hipStream_t)stream;
  const int cb = (C + 255) / 256;
  if (w_f32)
    causal_conv_rows_kernel<float><<<dim3(n_rows, cb), 256, 0, st>>>(x, ldx, (const float*)w, (const float*)b, conv_state,
                                                                     row_pos, row_slot, out, ldo, C, taps, act);
  else
    causal_conv_rows_kernel<bf16_t><<<dim3(n_rows, cb), 256, 0, st>>>(x, ldx, (const bf16_t*)w, (const bf16_t*)b,
                                                                      conv_state, row_pos, row_slot, out, ldo, C, taps, act);
  SD_CHECK_LAUNCH("sd_causal_conv_rows");
  if (taps > 1) {
    conv_state_update_kernel<<<dim3(n_entries, cb), 256, 0, st>>>(x, ldx, conv_state, entries, C, taps);
    SD_CHECK_LAUNCH("sd_causal_conv_rows (state)");
  }
  return SD_OK;
}

extern "C" int sd_ssd_steps(const float* dt, int64_t ld, const void* dt_bias, const void* a_log, int w_f32, float* step,
                            float* decay, int n_rows, int H, sd_stream_t stream) {
  SD_REQUIRE(dt && dt_bias && a_log && step && decay && n_rows >= 1 && H >= 1 && ld >= H, SD_ERR_INVALID,
             "sd_ssd_steps: bad argument");
  hipStream_t st = (hipStream_t)stream;
  const int n = n_rows * H;
  if (w_f32)
    ssd_steps_kernel<float><<<(n + 255) / 256, 256, 0, st>>>(dt, ld, (const float*)dt_bias, (const float*)a_log, step, decay, n, H);
  else
    ssd_steps_kernel<bf16_t><<<(n + 255) / 256, 256, 0, st>>>(dt, ld, (const bf16_t*)dt_bias, (const bf16_t*)a_log, step, decay, n, H);
  SD_CHECK_LAUNCH("sd_ssd_steps");
  return SD_OK;
}

extern "C" int sd_decay_scan_rows(const float* q, const float* k, int64_t ldqk, const float* v, int64_t ldv,
                                  const float* decay, const float* k_scale, const void* skip, int w_f32, float* state,
                                  const int32_t* entries, int n_entries, float* out, int H, int Gq, int dk, int dv,
                                  sd_stream_t stream) {
  SD_REQUIRE(q && k && v && decay && state && entries && out && n_entries >= 1 && H >= 1 && Gq >= 1 && H % Gq == 0 &&
                 dv >= 1,
             SD_ERR_INVALID, "sd_decay_scan_rows: bad argument");
  SD_REQUIRE(dk >= 1 && dk <= 256, SD_ERR_UNSUPPORTED, "sd_decay_scan_rows: key size %d outside 1..256", dk);
  SD_REQUIRE(H <= 4096, SD_ERR_UNSUPPORTED, "sd_decay_scan_rows: more than 4096 heads");
  const int NS = (dk + kStrip - 1) / kStrip;
  hipStream_t st = (hipStream_t)stream;
  int CT = 256 / NS;
  if (CT > dv) CT = dv;
  if (CT > 64) CT = 64;
  const int tiles = (dv + CT - 1) / CT;
  const int dkp = NS * kStrip;
  int CH = kScanLoads * (CT * NS) / dkp;
  if (CH > kScanChunk) CH = kScanChunk;
  SD_REQUIRE(CH >= 1 && CH * CT <= kScanLoadsV * CT * NS, SD_ERR_UNSUPPORTED,
             "sd_decay_scan_rows: key size %d with value size %d leaves no chunk", dk, dv);
  const size_t lds = sizeof(float) * ((size_t)2 * CH * dkp + (size_t)CH * CT + 2 * (size_t)CH + (size_t)CH * NS * CT);
  dim3 grid(tiles, H, n_entries);
  const int hpg = H / Gq;
  if (w_f32)
    decay_scan_rows_kernel<float><<<grid, CT * NS, lds, st>>>(q, k, ldqk, v, ldv, decay, k_scale, (const float*)skip,
                                                              state, entries, out, H, hpg, dk, dv, CT, NS, CH);
  else
    decay_scan_rows_kernel<bf16_t><<<grid, CT * NS, lds, st>>>(q, k, ldqk, v, ldv, decay, k_scale, (const bf16_t*)skip,
                                                               state, entries, out, H, hpg, dk, dv, CT, NS, CH);
  SD_CHECK_LAUNCH("sd_decay_scan_rows");
  return SD_OK;
}

extern "C" int sd_moe_route(const float* logits, int64_t ld, int32_t* sel_expert, float* sel_weight, int n_rows, int E,
                            int top, int score_kind, int renorm, sd_stream_t stream) {
  SD_REQUIRE(logits && sel_expert && sel_weight && n_rows >= 1 && E >= 1 && top >= 1 && top <= E && ld >= E,
             SD_ERR_INVALID, "sd_moe_route: bad argument (E=%d top=%d)", E, top);
  SD_REQUIRE(E <= 8192, SD_ERR_UNSUPPORTED, "sd_moe_route: more than 8192 experts");
  moe_route_kernel<<<n_rows, 64, sizeof(float) * E, (hipStream_t)stream>>>(logits, ld, sel_expert, sel_weight, E, top,
                                                                           score_kind, renorm);
  SD_CHECK_LAUNCH("sd_moe_route");
  return SD_OK;
}

extern "C" int sd_moe_route_rows_gated(const float* x, int64_t ldx, const void* w_router, int w_f32, float* logits,
                                       int32_t* sel_expert, float* sel_weight, int n_rows, int E, int K, int top,
                                       int score_kind, int renorm, float renorm_eps, float weight_scale,
                                       const void* w_gate, int n_gate, float* gate_out, sd_stream_t stream) {
  return sd_moe_route_rows_biased(x, ldx, w_router, nullptr, w_f32, logits, sel_expert, sel_weight, n_rows, E, K, top,
                                  score_kind, renorm, renorm_eps, weight_scale, w_gate, n_gate, gate_out, stream);
}

extern "C" int sd_moe_route_rows_biased(const float* x, int64_t ldx, const void* w_router, const float* router_bias,
                                        int w_f32, float* logits, int32_t* sel_expert, float* sel_weight, int n_rows,
                                        int E, int K, int top, int score_kind, int renorm, float renorm_eps,
                                        float weight_scale, const void* w_gate, int n_gate, float* gate_out,
                                        sd_stream_t stream) {
  SD_REQUIRE(x && w_router && sel_expert && sel_weight && n_rows >= 1 && E >= 1 && K >= 1 && top >= 1 && top <= E &&
                 ldx >= K,
             SD_ERR_INVALID, "sd_moe_route_rows: bad argument (E=%d top=%d)", E, top);
  SD_REQUIRE(n_gate >= 0 && (n_gate == 0 || (w_gate && gate_out)), SD_ERR_INVALID,
             "sd_moe_route_rows: gate rows without their matrix or output");
  SD_REQUIRE(E <= 8192, SD_ERR_UNSUPPORTED, "sd_moe_route_rows: more than 8192 experts");
  hipStream_t st = (hipStream_t)stream;
  const int nthr = 64 * (E >= 16 ? 16 : (E >= 8 ? 8 : 4));   // a wave per expert, up to 16 at a time
  if (w_f32)
    moe_route_rows_kernel<float><<<n_rows, nthr, sizeof(float) * E, st>>>(
        x, ldx, (const float*)w_router, logits, sel_expert, sel_weight, E, K, top, score_kind, renorm, 0, renorm_eps,
        weight_scale, (const float*)w_gate, n_gate, gate_out, router_bias);
  else
    moe_route_rows_kernel<bf16_t><<<n_rows, nthr, sizeof(float) * E, st>>>(
        x, ldx, (const bf16_t*)w_router, logits, sel_expert, sel_weight, E, K, top, score_kind, renorm, 1, renorm_eps,
        weight_scale, (const bf16_t*)w_gate, n_gate, gate_out, router_bias);
  SD_CHECK_LAUNCH("sd_moe_route_rows");
  return SD_OK;
}

extern "C" int sd_moe_route_rows(const float* x, int64_t ldx, const void* w_router, int w_f32, float* logits,
                                 int32_t* sel_expert, float* sel_weight, int n_rows, int E, int K, int top,
                                 int score_kind, int renorm, sd_stream_t stream) {
  return sd_moe_route_rows_gated(x, ldx, w_router, w_f32, logits, sel_expert, sel_weight, n_rows, E, K, top, score_kind,
                                 renorm, 0.f, 1.f, nullptr, 0, nullptr, stream);
}

extern "C" size_t sd_moe_experts_scratch_bytes(int n_rows, int top, int E, int F, int W) {
  (void)W;
  if (n_rows < 1 || top < 1 || E < 1 || F < 1) return 0;
  return moe_plan(n_rows, top, E, F).total;
}

extern "C" int sd_moe_experts(const float* x, const void* x_bf16, int64_t ldx, const int32_t* sel_expert,
                              const float* sel_weight,
                              const void* w_gate_up, const void* w_down, int w_f32, float* out, int n_rows, int top,
                              int E, int F, int W, int scale_input, int act_kind, void* scratch, size_t scratch_bytes,
                              sd_stream_t stream) {
  SD_REQUIRE(x && sel_expert && sel_weight && w_gate_up && w_down && out && scratch, SD_ERR_INVALID,
             "sd_moe_experts: null argument");
  SD_REQUIRE(n_rows >= 1 && top >= 1 && E >= 1 && F >= 1 && W >= 1 && ldx >= W, SD_ERR_INVALID, "sd_moe_experts: bad shape");
  SD_REQUIRE(act_kind == 0 || act_kind == 1, SD_ERR_UNSUPPORTED, "sd_moe_experts: activation %d is not provided", act_kind);
  const MoeScratch p = moe_plan(n_rows, top, E, F);
  SD_REQUIRE(scratch_bytes >= p.total, SD_ERR_WORKSPACE, "sd_moe_experts: scratch %zu < %zu bytes", scratch_bytes, p.total);
  SD_REQUIRE(sd_aligned16(scratch), SD_ERR_INVALID, "sd_moe_experts: scratch unaligned");
  hipStream_t st = (hipStream_t)stream;
  char* base = (char*)scratch;
  int32_t* cnt = (int32_t*)(base + p.cnt);
  int32_t* n_tiles = (int32_t*)(base + p.n_tiles);
  int32_t* perm = (int32_t*)(base + p.perm);
  int32_t* tiles = (int32_t*)(base + p.tiles);
  float* act = (float*)(base + p.act);
  const int n = n_rows * top;
  const bool mfma = !w_f32 && W % 32 == 0 && F % 32 == 0 && sd_aligned16(w_gate_up) && sd_aligned16(w_down) &&
                    ldx % 8 == 0 && sd_aligned16(x) && (!x_bf16 || sd_aligned16(x_bf16));
  // (tiles of 128 rows for experts with many rows, the template's MT = 8 with chunks of 128 columns,
  // measured slower than tiles of 32: 95-156 against 153-183 TFLOP/s at 1024-2048 rows)
  const int bm = kMoeBM;
  int tiles_y = n;
  if (n <= kMoeDirect) {   // a few assignments: each runs as a tile of its own, straight from the router's choice
    perm = const_cast<int32_t*>(sel_expert);
    tiles = nullptr;
  } else {
    moe_count_kernel<<<E, 256, 0, st>>>(sel_expert, n, cnt);
    SD_CHECK_LAUNCH("sd_moe_experts (count)");
    moe_group_kernel<<<E, 256, 0, st>>>(sel_expert, n, cnt, E, perm, tiles, n_tiles, bm);
    SD_CHECK_LAUNCH("sd_moe_experts (group)");
    const int max_tiles = n / bm + E;
    tiles_y = max_tiles < n ? max_tiles : n;   // never more tiles than assignments
  }
  if (w_f32) {
    moe_gate_up_kernel<float><<<dim3((F + 63) / 64, tiles_y), 256, 0, st>>>(x, ldx, perm, tiles, n_tiles, sel_weight,
                                                                            (const float*)w_gate_up, act, top, F, W, scale_input, 0, act_kind);
    SD_CHECK_LAUNCH("sd_moe_experts (gate, up)");
    moe_down_kernel<float><<<dim3((W + 63) / 64, tiles_y), 256, 0, st>>>(act, perm, tiles, n_tiles, sel_weight,
                                                                         (const float*)w_down, out, W, F, scale_input);
  } else if (!tiles && W % 8 == 0 && F % 8 == 0 && W <= kGemvMaxK && F <= kGemvMaxK && sd_aligned16(w_gate_up) &&
             sd_aligned16(w_down)) {
    bf16_t* act_b = (bf16_t*)act;
    if (act_kind == 0)
      moe_gemv_gate_up_kernel<true><<<dim3((F + 7) / 8, n), 256, sizeof(float) * W, st>>>(
          x, ldx, sel_expert, sel_weight, (const bf16_t*)w_gate_up, act_b, top, F, W, scale_input);
    else
      moe_gemv_gate_up_kernel<false><<<dim3((F + 15) / 16, n), 256, sizeof(float) * W, st>>>(
          x, ldx, sel_expert, sel_weight, (const bf16_t*)w_gate_up, act_b, top, F, W, scale_input);
    SD_CHECK_LAUNCH("sd_moe_experts (gate, up)");
    moe_gemv_down_kernel<<<dim3((W + 15) / 16, n), 256, sizeof(float) * F, st>>>(
        act_b, sel_expert, sel_weight, (const bf16_t*)w_down, out, W, F, scale_input);
  } else if (mfma) {
    // (act holds n * F floats: its first half serves as the bf16 activations)
    bf16_t* act_b = (bf16_t*)act;
    const dim3 g1((F + 127) / 128, tiles_y), g2((W + 127) / 128, tiles_y);
    const bf16_t* xb = (const bf16_t*)x_bf16;
    if (act_kind == 0)
      moe_gate_up_mfma_kernel<2, 512, true><<<g1, 256, 0, st>>>(x, xb, ldx, perm, tiles, n_tiles, sel_weight,
                                                                (const bf16_t*)w_gate_up, act_b, top, F, W, scale_input);
    else
      moe_gate_up_mfma_kernel<2, 512, false><<<g1, 256, 0, st>>>(x, xb, ldx, perm, tiles, n_tiles, sel_weight,
                                                                 (const bf16_t*)w_gate_up, act_b, top, F, W, scale_input);
    SD_CHECK_LAUNCH("sd_moe_experts (gate, up)");
    moe_down_mfma_kernel<2, 512><<<g2, 256, 0, st>>>(act_b, perm, tiles, n_tiles, sel_weight, (const bf16_t*)w_down,
                                                     out, W, F, scale_input);
  } else {
    moe_gate_up_kernel<bf16_t><<<dim3((F + 63) / 64, tiles_y), 256, 0, st>>>(x, ldx, perm, tiles, n_tiles, sel_weight,
                                                                             (const bf16_t*)w_gate_up, act, top, F, W, scale_input, 1, act_kind);
    SD_CHECK_LAUNCH("sd_moe_experts (gate, up)");
    moe_down_kernel<bf16_t><<<dim3((W + 63) / 64, tiles_y), 256, 0, st>>>(act, perm, tiles, n_tiles, sel_weight,
                                                                          (const bf16_t*)w_down, out, W, F, scale_input);
  }
  SD_CHECK_LAUNCH("sd_moe_experts (down)");
  return SD_OK;
}

extern "C" int sd_postnorm_residual(float* x, const float* a, int n_a, float sa, const float* b, float sb, const void* w,
                                    int w_f32, float eps, void* x_bf16, int n_rows, int W, sd_stream_t stream) {
  SD_REQUIRE(x && a && w && n_a >= 1 && n_rows >= 1 && W >= 1, SD_ERR_INVALID, "sd_postnorm_residual: bad argument");
  hipStream_t st = (hipStream_t)stream;
  if (w_f32)
    postnorm_residual_kernel<float><<<n_rows, 256, 0, st>>>(x, a, n_a, sa, b, sb, (const float*)w, eps, (bf16_t*)x_bf16, W);
  else
    postnorm_residual_kernel<bf16_t><<<n_rows, 256, 0, st>>>(x, a, n_a, sa, b, sb, (const bf16_t*)w, eps, (bf16_t*)x_bf16, W);
  SD_CHECK_LAUNCH("sd_postnorm_residual");
  return SD_OK;
}

extern "C" int sd_residual_norm(float* x, const float* a, int n_a, const float* b, const float* b_gate, int64_t ldg,
                                const void* w_post, const void* add, const void* w_next, int w_f32, float eps,
                                float* x_copy, float* h, void* h_bf16, int n_rows, int W, sd_stream_t stream) {
  return sd_residual_norm_scaled(x, a, n_a, nullptr, b, b_gate, ldg, w_post, 1.f, add, w_next, w_f32, eps, x_copy, h,
                                 h_bf16, n_rows, W, stream);
}

extern "C" int sd_residual_norm_scaled(float* x, const float* a, int n_a, const void* a_bias, const float* b,
                                       const float* b_gate, int64_t ldg, const void* w_post, float mult,
                                       const void* add, const void* w_next, int w_f32, float eps, float* x_copy,
                                       float* h, void* h_bf16, int n_rows, int W, sd_stream_t stream) {
  SD_REQUIRE(!a_bias || a, SD_ERR_INVALID, "sd_residual_norm: a bias without the rows it is added to");
  SD_REQUIRE(x && n_rows >= 1 && W >= 1 && (!a || (w_post && n_a >= 1)) && (!b || a) && (!b_gate || (b && ldg >= 1)) &&
                 (!w_next || h || h_bf16),
             SD_ERR_INVALID, "sd_residual_norm: bad argument");
  SD_REQUIRE((size_t)W * sizeof(float) <= 60 * 1024, SD_ERR_UNSUPPORTED, "sd_residual_norm: width %d above 15360", W);
  hipStream_t st = (hipStream_t)stream;
  const size_t lds = (size_t)W * sizeof(float);
  auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  // (weights are 4 or 2 bytes an element: four of them are 16 or 8 bytes, and a vector [W] starts aligned to that
  // when its address is a multiple of 16; `add` may be a row of a table, whose rows are W elements apart)
  if (W % 4 == 0 && W >= 256 && al16(x) && al16(a) && al16(b) && al16(w_post) && al16(w_next) && al16(x_copy) &&
      al16(h) && al16(h_bf16) && (reinterpret_cast<uintptr_t>(add) & 7) == 0 && (!w_f32 || al16(add)) &&
      al16(a_bias)) {
    int nthr = ((W / 4 + 63) / 64) * 64;
    if (nthr > 1024) nthr = 1024;
    if (w_f32)
      residual_norm_quad_kernel<float><<<n_rows, nthr, lds, st>>>(x, a, n_a, b, b_gate, ldg, (const float*)w_post,
                                                                  (const float*)add, (const float*)w_next, eps, x_copy,
                                                                  h, (bf16_t*)h_bf16, W, 0, (const float*)a_bias, mult);
    else
      residual_norm_quad_kernel<bf16_t><<<n_rows, nthr, lds, st>>>(x, a, n_a, b, b_gate, ldg, (const bf16_t*)w_post,
                                                                   (const bf16_t*)add, (const bf16_t*)w_next, eps,
                                                                   x_copy, h, (bf16_t*)h_bf16, W, 1,
                                                                   (const bf16_t*)a_bias, mult);
    SD_CHECK_LAUNCH("sd_residual_norm");
    return SD_OK;
  }
  if (w_f32)
    residual_norm_kernel<float><<<n_rows, 256, lds, st>>>(x, a, n_a, b, b_gate, ldg, (const float*)w_post,
                                                          (const float*)add, (const float*)w_next, eps, x_copy, h,
                                                          (bf16_t*)h_bf16, W, 0, (const float*)a_bias, mult);
  else
    residual_norm_kernel<bf16_t><<<n_rows, 256, lds, st>>>(x, a, n_a, b, b_gate, ldg, (const bf16_t*)w_post,
                                                           (const bf16_t*)add, (const bf16_t*)w_next, eps, x_copy, h,
                                                           (bf16_t*)h_bf16, W, 1, (const bf16_t*)a_bias, mult);
  SD_CHECK_LAUNCH("sd_residual_norm");
  return SD_OK;
}

extern "C" int sd_scale_rows(float* x, int64_t ld, float s, int n_rows, int n_cols, sd_stream_t stream) {
  SD_REQUIRE(x && n_rows >= 1 && n_cols >= 1 && ld >= n_cols, SD_ERR_INVALID, "sd_scale_rows: bad argument");
  int by = (n_cols + 255) / 256;
  if (by > 64) by = 64;
  scale_rows_kernel<<<dim3(n_rows, by), 256, 0, (hipStream_t)stream>>>(x, ld, s, n_cols);
  SD_CHECK_LAUNCH("sd_scale_rows");
  return SD_OK;
}
