// Sequence mixers beyond softmax attention, for decoders whose layers are listed one by one
// (sd_seq_model): decayed linear-attention recurrences (a fixed decay per head, or a decay per
// key channel computed from the input), sliding-window attention with pooled blocks and sigmoid
// weights, offset RMS norms, partial rotary embeddings in both pair layouts, gated residuals.
//
// Arithmetic.  Activations travel as f32 buffers; with bf16 weights the operands of the
// matrix products (norm outputs, gated mixer outputs, feed-forward activations) are rounded to
// bf16 values when they are stored, and keys / values are stored in the cache as bf16.  Norms,
// angles, scores and weights, decays, the recurrent state and the residual sum are f32 always.
// With f32 weights nothing is rounded.  Every output element is summed in an order that depends
// only on its own position in its sequence (never on what else is in the batch or on how a prompt
// was cut), so a token's result is the same bits in any batch.
#include <math.h>

#include <vector>

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

// Sum over a workgroup of up to 256 threads in a fixed order: butterfly inside each wave, then
// the waves' sums in wave order.  `red` holds at least 4 floats.
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

// ------------------------------------------------------------------ rows in, rows out
template <typename T>
__global__ void embed_rows_kernel(const int32_t* __restrict__ tokens, const T* __restrict__ table,
                                  float* __restrict__ x, int W, int vocab) {
  const int r = blockIdx.x;
  int tok = tokens[r];
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  for (int c = threadIdx.x; c < W; c += blockDim.x) x[(size_t)r * W + c] = ld_f(table + (size_t)tok * W + c);
}

// out[i] = x[rows ? rows[i] : i] / sqrt(mean(x^2) + eps) * (offset + w); out_b: the same as bf16
template <typename T>
__global__ void rmsnorm_rows_kernel(const float* __restrict__ x, const int32_t* __restrict__ rows,
                                    const T* __restrict__ w, float offset, float eps,
                                    float* __restrict__ out, bf16_t* __restrict__ out_b, int W, int round) {
  __shared__ float red[4];
  const int i = blockIdx.x;
  const float* xr = x + (size_t)(rows ? rows[i] : i) * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) ss = fmaf(xr[c], xr[c], ss);
  ss = block_sum(ss, red);
  const float rstd = 1.f / sqrtf(ss / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float v = maybe_round(xr[c] * rstd * (offset + ld_f(w + c)), round);
    out[(size_t)i * W + c] = v;
    if (out_b) out_b[(size_t)i * W + c] = (bf16_t)v;
  }
}

// Y[M, N] = X[M, K] W[N, K]^T + bias.  X is f32 (rounded to bf16 values on load when `round`;
// with x2: the operand is relu(X) * X2, the gated feed-forward's activation).  Every output is
// summed over k in ascending order, whatever the tile shape, so a row's bits do not depend on M.
template <typename T, int BM, int BN, int TM, int TN>
__global__ __launch_bounds__(256) void matmul_rows_kernel(
    const float* __restrict__ X, const float* __restrict__ X2, int64_t ldx, const T* __restrict__ Wt,
    const float* __restrict__ bias, float* __restrict__ Y, int64_t ldy, int M, int N, int K, int round,
    int64_t bx = 0, int64_t bw = 0, int64_t by = 0, bf16_t* __restrict__ Yb = nullptr) {
  constexpr int BK = 16;
  X += (size_t)blockIdx.z * bx;    // blockIdx.z: one product of a batch (operands bx / bw / by apart)
  Wt += (size_t)blockIdx.z * bw;
  Y += (size_t)blockIdx.z * by;
  if (Yb) Yb += (size_t)blockIdx.z * by;
  static_assert((BM / TM) * (BN / TN) == 256, "256 threads");
  __shared__ float xs[BK][BM + 1];
  __shared__ float ws[BK][BN + 1];
  const int tid = threadIdx.x;
  const int tx = tid % (BN / TN), ty = tid / (BN / TN);
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  float acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = 0.f;
  for (int k0 = 0; k0 < K; k0 += BK) {
    for (int idx = tid; idx < BM * BK; idx += 256) {
      const int m = idx / BK, kk = idx % BK;
      float v = 0.f;
      if (m0 + m < M && k0 + kk < K) {
        v = X[(size_t)(m0 + m) * ldx + k0 + kk];
        if (X2) v = fmaxf(v, 0.f) * X2[(size_t)(m0 + m) * ldx + k0 + kk];
        v = maybe_round(v, round);
      }
      xs[kk][m] = v;
    }
    for (int idx = tid; idx < BN * BK; idx += 256) {
      const int n = idx / BK, kk = idx % BK;
      ws[kk][n] = (n0 + n < N && k0 + kk < K) ? ld_f(Wt + (size_t)(n0 + n) * K + k0 + kk) : 0.f;
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
    const int m = m0 + ty * TM + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + tx * TN + j;
      if (n < N) {
        const float o = acc[i][j] + (bias ? bias[n] : 0.f);
        Y[(size_t)m * ldy + n] = o;
        if (Yb) Yb[(size_t)m * ldy + n] = (bf16_t)o;
      }
    }
  }
}

// ------------------------------------------------------------------ rotary embedding
// One wave per (row, head).  Heads 0..Hq-1 are query heads at q, heads Hq..Hq+Hk-1 key heads at k.
// The first `dims` channels are rotated in place: pair i is (i, i + dims/2) (layout 0) or
// (2i, 2i + 1) (layout 1), by the angle pos * inv_freq[i], formed in f64 (the product of a position
// in the thousands and an f32 frequency loses the low bits of the angle otherwise).  Then the
// vector is divided by its root mean square (unit_norm) and multiplied by q_scale / k_scale.
// Key heads with a cache: the finished key and the value row go to the paged cache.  Every lane
// re-reads only what it wrote itself.
template <typename T>
__global__ void head_prep_kernel(float* __restrict__ q, float* __restrict__ k, const float* __restrict__ v,
                                 int64_t ld, const int32_t* __restrict__ row_pos,
                                 const int32_t* __restrict__ row_slot, int Hq, int Hk, int dk, int dv,
                                 int dims, int layout, const double* __restrict__ inv_freq, int unit_norm,
                                 float eps, float q_scale, float k_scale, T* __restrict__ k_cache,
                                 T* __restrict__ v_cache, const int32_t* __restrict__ block_tables,
                                 int max_blocks, int page) {
  const int r = blockIdx.x, hh = blockIdx.y, lane = threadIdx.x;
  const bool is_q = hh < Hq;
  const int head = is_q ? hh : hh - Hq;
  float* vec = (is_q ? q : k) + (size_t)r * ld + (size_t)head * dk;
  const int pos = row_pos[r];
  float ss = 0.f;
  for (int i = lane; i < dims / 2; i += 64) {
    const double a = (double)pos * inv_freq[i];
    const float cs = (float)cos(a), sn = (float)sin(a);
    const int iu = layout ? 2 * i : i, iv = layout ? 2 * i + 1 : i + dims / 2;
    const float u = vec[iu], w = vec[iv];
    const float ru = u * cs - w * sn, rw = w * cs + u * sn;
    vec[iu] = ru;
    vec[iv] = rw;
    ss = fmaf(ru, ru, ss);
    ss = fmaf(rw, rw, ss);
  }
  for (int c = dims + lane; c < dk; c += 64) ss = fmaf(vec[c], vec[c], ss);
  float scale = is_q ? q_scale : k_scale;
  if (unit_norm) {
    ss = wave_sum(ss);
    scale *= 1.f / sqrtf(ss / (float)dk + eps);
  }
  T* kc = nullptr;
  T* vc = nullptr;
  if (!is_q && k_cache) {
    const int pg = block_tables[(size_t)row_slot[r] * max_blocks + pos / page];
    const size_t at = ((size_t)pg * Hk + head) * page + pos % page;
    kc = k_cache + at * dk;
    vc = v_cache + at * dv;
  }
  for (int i = lane; i < dims / 2; i += 64) {
    const int iu = layout ? 2 * i : i, iv = layout ? 2 * i + 1 : i + dims / 2;
    const float ou = vec[iu] * scale, ov = vec[iv] * scale;
    vec[iu] = ou;
    vec[iv] = ov;
    if (kc) {
      st_f(kc + iu, ou);
      st_f(kc + iv, ov);
    }
  }
  for (int c = dims + lane; c < dk; c += 64) {
    const float o = vec[c] * scale;
    vec[c] = o;
    if (kc) st_f(kc + c, o);
  }
  if (vc) {
    const float* vr = v + (size_t)r * ld + (size_t)head * dv;
    for (int c = lane; c < dv; c += 64) st_f(vc + c, vr[c]);
  }
}

// Element-wise kernels take (row, block of kColsPerBlock columns) per workgroup: a few rows of a
// decode step still spread over many compute units.
constexpr int kColsPerBlock = 1024;
// decay[r, c] = sigmoid(z[r, c])^(1/tau) = exp(-softplus(-z) / tau)
__global__ void sigmoid_power_kernel(const float* __restrict__ z, int64_t ldz, float inv_tau,
                                     float* __restrict__ out, int n_cols) {
  const int r = blockIdx.x;
  const int c_end = (blockIdx.y + 1) * kColsPerBlock < n_cols ? (blockIdx.y + 1) * kColsPerBlock : n_cols;
  for (int c = blockIdx.y * kColsPerBlock + threadIdx.x; c < c_end; c += blockDim.x) {
    const float x = z[(size_t)r * ldz + c];
    const float log_sig = x >= 0.f ? -log1pf(expf(-x)) : x - log1pf(expf(x));
    out[(size_t)r * n_cols + c] = expf(log_sig * inv_tau);
  }
}

// ------------------------------------------------------------------ decayed outer-product scan
// S <- diag(d_t) S + k_t v_t^T,  o_t = S^T q_t, token by token, per (entry, head).  A thread owns
// 16 consecutive key channels of one value column; the strips' partial dot products are added in
// strip order.  d_t: a factor per key channel (PER_CHANNEL, [rows, H*dk]) or per head ([H]).
constexpr int kStrip = 16;
constexpr int kScanLoads = 8;    // q / k / decay elements a thread stages per chunk, at most
constexpr int kScanLoadsV = 16;  // value elements
constexpr int kScanChunk = 16;   // tokens per chunk, at most
template <bool PER_CHANNEL>
__global__ __launch_bounds__(256) void decay_scan_kernel(
    const float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ v, int64_t ld,
    const float* __restrict__ decay, float* __restrict__ state, const int32_t* __restrict__ entries,
    float* __restrict__ out, int H, int dk, int dv, int CT, int NS, int CH) {
  extern __shared__ float lds[];
  const int dkp = NS * kStrip;
  float* qs = lds;                  // [CH][dkp]
  float* ks = qs + CH * dkp;        // [CH][dkp]
  float* ds = ks + CH * dkp;        // [CH][dkp] (PER_CHANNEL only)
  float* vs = ds + (PER_CHANNEL ? CH * dkp : 0);  // [CH][CT]
  float* part = vs + CH * CT;       // [CH][NS][CT]
  const int tid = threadIdx.x, nthr = CT * NS;
  const int c = tid % CT, s = tid / CT;
  const int h = blockIdx.y, e = blockIdx.z;
  const int col = blockIdx.x * CT + c;
  const int slot = entries[4 * e], row0 = entries[4 * e + 1], len = entries[4 * e + 2],
            pos0 = entries[4 * e + 3];
  float* st = state + ((size_t)slot * H + h) * dk * dv;
  const int r0 = s * kStrip;
  float S[kStrip];
#pragma unroll
  for (int r = 0; r < kStrip; ++r)
    S[r] = (pos0 > 0 && r0 + r < dk && col < dv) ? st[(size_t)(r0 + r) * dv + col] : 0.f;
  const float dh = PER_CHANNEL ? 0.f : decay[h];
  // A chunk of CH tokens goes global -> registers -> LDS; the next chunk's loads are in flight
  // while this one is computed.
  float pq[kScanLoads], pk[kScanLoads], pd[kScanLoads], pv[kScanLoadsV];
  auto fetch = [&](int t0) {
    const int nt = len - t0 < CH ? len - t0 : CH;
#pragma unroll
    for (int i = 0; i < kScanLoads; ++i) {
      const int idx = tid + i * nthr;
      const int t = idx / dkp, ch = idx % dkp;
      const bool in = idx < nt * dkp && ch < dk;
      // (every load is issued, on an address clamped into the chunk: a guarded load would become
      // a branch whose join waits for the loads in flight)
      const int tc = t < nt ? t : nt - 1, cc = ch < dk ? ch : dk - 1;
      const size_t at = (size_t)(row0 + t0 + tc) * ld + (size_t)h * dk + cc;
      const float lq = q[at], lk = k[at];
      pq[i] = in ? lq : 0.f;
      pk[i] = in ? lk : 0.f;
      if (PER_CHANNEL) {
        const float ldc = decay[(size_t)(row0 + t0 + tc) * ((size_t)H * dk) + (size_t)h * dk + cc];
        pd[i] = in ? ldc : 0.f;
      }
    }
#pragma unroll
    for (int i = 0; i < kScanLoadsV; ++i) {
      const int idx = tid + i * nthr;
      const int t = idx / CT, vcol = blockIdx.x * CT + idx % CT;
      const bool in = idx < nt * CT && vcol < dv;
      const int tc = t < nt ? t : nt - 1, vc2 = vcol < dv ? vcol : dv - 1;
      const float lv = v[(size_t)(row0 + t0 + tc) * ld + (size_t)h * dv + vc2];
      pv[i] = in ? lv : 0.f;
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
        if (PER_CHANNEL) ds[idx] = pd[i];
      }
    }
#pragma unroll
    for (int i = 0; i < kScanLoadsV; ++i) {
      const int idx = tid + i * nthr;
      if (idx < CH * CT) vs[idx] = pv[i];
    }
    __syncthreads();
    if (t0 + CH < len) fetch(t0 + CH);
    for (int t = 0; t < nt; ++t) {
      const float vv = vs[t * CT + c];
      const float* qt = qs + t * dkp + r0;
      const float* kt = ks + t * dkp + r0;
      const float* dt = ds + t * dkp + r0;
      float acc = 0.f;
#pragma unroll
      for (int r = 0; r < kStrip; ++r) {
        const float d = PER_CHANNEL ? dt[r] : dh;
        S[r] = fmaf(d, S[r], kt[r] * vv);
        acc = fmaf(S[r], qt[r], acc);
      }
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
    // (the next chunk's LDS stores touch qs / ks / ds / vs only; `part` is rewritten after the
    // barrier that follows them)
  }
  if (col < dv) {
#pragma unroll
    for (int r = 0; r < kStrip; ++r)
      if (r0 + r < dk) st[(size_t)(r0 + r) * dv + col] = S[r];
  }
}

// y[r, h*dv + c] = o * (unit_norm ? rstd(o over the head) : 1) * (norm_w ? norm_w[c] : 1) * gate(g)
// gate: 0 = silu, 1 = sigmoid.  One wave per (row, head).
template <typename T>
__global__ void head_post_kernel(const float* __restrict__ o, const float* __restrict__ g, int64_t ldg,
                                 const T* __restrict__ norm_w, int unit_norm, float eps, int gate_kind,
                                 float* __restrict__ y, bf16_t* __restrict__ y_b, int H, int dv, int round) {
  const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float* orow = o + (size_t)r * H * dv + (size_t)h * dv;
  const float* grow = g + (size_t)r * ldg + (size_t)h * dv;
  float rstd = 1.f;
  if (unit_norm) {
    float ss = 0.f;
    for (int c = lane; c < dv; c += 64) ss = fmaf(orow[c], orow[c], ss);
    ss = wave_sum(ss);
    rstd = 1.f / sqrtf(ss / (float)dv + eps);
  }
  for (int c = lane; c < dv; c += 64) {
    const float gz = grow[c];
    const float gate = gate_kind ? sigmoid_f(gz) : gz * sigmoid_f(gz);
    float val = orow[c] * rstd;
    if (norm_w) val *= ld_f(norm_w + c);
    const float res = maybe_round(val * gate, round);
    y[(size_t)r * H * dv + (size_t)h * dv + c] = res;
    if (y_b) y_b[(size_t)r * H * dv + (size_t)h * dv + c] = (bf16_t)res;
  }
}

// ------------------------------------------------------------------ window + pooled blocks
// In-page slot of pooled block b, whose last token lies in logical page lp.
__device__ __forceinline__ int pooled_slot(int b, int lp, int page, int pool) { return b - (lp * page) / pool; }

// Mean key / value of every block of `pool` tokens that a new row completes, from the rows the
// cache holds.  One wave per (row, kv head).
template <typename T>
__global__ void pool_blocks_kernel(const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                                   float* __restrict__ pk_cache, float* __restrict__ pv_cache,
                                   const int32_t* __restrict__ row_pos, const int32_t* __restrict__ row_slot,
                                   const int32_t* __restrict__ block_tables, int max_blocks, int page,
                                   int pslots, int G, int dk, int dv, int pool) {
  const int r = blockIdx.x, g = blockIdx.y, lane = threadIdx.x;
  const int pos = row_pos[r];
  if (pos % pool != pool - 1) return;
  const int b = pos / pool;
  const int32_t* tbl = block_tables + (size_t)row_slot[r] * max_blocks;
  const int lp = pos / page;
  const size_t dst = ((size_t)tbl[lp] * G + g) * pslots + pooled_slot(b, lp, page, pool);
  for (int c = lane; c < dk + dv; c += 64) {
    const bool is_k = c < dk;
    const int cc = is_k ? c : c - dk;
    const int d = is_k ? dk : dv;
    const T* cache = is_k ? k_cache : v_cache;
    float sum = 0.f;
    for (int j = b * pool; j <= pos; ++j)
      sum += ld_f(cache + (((size_t)tbl[j / page] * G + g) * page + j % page) * d + cc);
    (is_k ? pk_cache : pv_cache)[dst * d + cc] = sum / (float)pool;
  }
}

// Position i sees the tokens j with 0 <= i - j < window and the pooled blocks b with
// b*pool + pool - 1 <= i - window.  Weight of a key: sigmoid(q.k * scale + head_bias[h]); the
// weighted values are summed, not normalised.  One workgroup per (row, kv head, group of up to
// kAttnHeads query heads of that kv head): a key or value row is read once for all of them.
// Phase 1, a thread per key of a 256-key tile: its scores against the query heads (q in LDS).
// Phase 2, a wave per key, lanes over value columns: the weighted sum.  Keys are taken in the
// order pooled blocks, then tokens, whatever the batch: a row's bits depend on its position only.
constexpr int kAttnTile = 256;
constexpr int kAttnBatch = 8;   // value rows a wave has in flight (twice as many when a lane holds <= 2 columns)
constexpr int kAttnLoads = 16;  // 16-byte pieces of a key row a thread has in flight
constexpr int kAttnSplitRows = 64;  // batches of at most this many rows may split their keys over workgroups

template <typename T> struct Piece;   // a 16-byte piece of a row as floats
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

// s[hq] += sum_c qs[hq][c] * k[c], channels in ascending order.  vec: the row is 16-byte aligned
// and dk a multiple of 8; then up to kAttnLoads pieces of the row are asked for before the first
// is used.
template <typename KT, int NH>
__device__ __forceinline__ void score_key(const KT* __restrict__ kr, const float* __restrict__ qs, int dk, int nh,
                                          bool vec, float* s) {
  constexpr int E = Piece<KT>::E;
  int c = 0;
  if (vec) {
    for (; c < dk; c += kAttnLoads * E) {
      u32x4 raw[kAttnLoads];
#pragma unroll
      for (int i = 0; i < kAttnLoads; ++i) {   // unguarded, on an address clamped into the row
        const int ci = c + i * E < dk ? c + i * E : dk - E;
        raw[i] = *reinterpret_cast<const u32x4*>(kr + ci);
      }
#pragma unroll
      for (int i = 0; i < kAttnLoads; ++i) {
        if (c + i * E < dk) {
          float kf[E];
          Piece<KT>::unpack(raw[i], kf);
#pragma unroll
          for (int hq = 0; hq < NH; ++hq) {
            if (hq < nh) {
#pragma unroll
              for (int e = 0; e < E; ++e) s[hq] = fmaf(qs[hq * dk + c + i * E + e], kf[e], s[hq]);
            }
          }
        }
      }
    }
    return;
  }
  for (; c < dk; ++c) {
    const float kf = ld_f(kr + c);
#pragma unroll
    for (int hq = 0; hq < NH; ++hq)
      if (hq < nh) s[hq] = fmaf(qs[hq * dk + c], kf, s[hq]);
  }
}

// NH: query heads per workgroup (of one kv head), NC: value columns per lane (vdim <= 64 * NC).
// n_splits > 1: workgroup (.., .., z) takes the keys of tile z / n_hgroups only and writes its sum
// to out + split * split_stride (sum_splits_kernel adds the splits in order).
template <typename T, int NH, int NC>
__global__ __launch_bounds__(256) void window_pool_attn_kernel(
    const float* __restrict__ q, int64_t ldq, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const float* __restrict__ pk_cache, const float* __restrict__ pv_cache,
    const int32_t* __restrict__ row_pos, const int32_t* __restrict__ row_slot,
    const int32_t* __restrict__ block_tables, int max_blocks, int page, int pslots, int H, int G, int dk,
    int dv, int window, int pool, float scale, const float* __restrict__ head_bias,
    float* __restrict__ out, int n_hgroups, int n_splits, size_t split_stride) {
  extern __shared__ float lds[];
  unsigned long long* vat = reinterpret_cast<unsigned long long*>(lds);  // [kAttnTile] cache row of the value
  float* wt = reinterpret_cast<float*>(vat + kAttnTile);                 // [NH][kAttnTile]
  float* qs = wt + NH * kAttnTile;                                       // [nh][dk]
  float* red = qs + NH * dk;                                             // [4][nh][dv]
  const int r = blockIdx.x, g = blockIdx.y, tid = threadIdx.x;
  const int hgroup = blockIdx.z % n_hgroups, split = blockIdx.z / n_hgroups;
  const int qh = H / G;
  const int h0 = g * qh + hgroup * NH;                                   // first query head here
  const int nh = qh - hgroup * NH < NH ? qh - hgroup * NH : NH;
  const int i = row_pos[r];
  const int32_t* tbl = block_tables + (size_t)row_slot[r] * max_blocks;
  for (int c = tid; c < nh * dk; c += 256) qs[c] = q[(size_t)r * ldq + (size_t)h0 * dk + c];
  const int t_first = i - window + 1 > 0 ? i - window + 1 : 0;
  const int n_blocks = i - window + 1 >= 0 ? (i - window + 1) / pool : 0;
  const int total = n_blocks + (i - t_first + 1);
  const int key_lo = n_splits > 1 ? split * kAttnTile : 0;
  const int key_hi = n_splits > 1 ? (total < key_lo + kAttnTile ? total : key_lo + kAttnTile) : total;
  const bool vec_t = dk % 8 == 0 && (reinterpret_cast<uintptr_t>(k_cache) & 15) == 0;
  const bool vec_p = dk % 8 == 0 && (reinterpret_cast<uintptr_t>(pk_cache) & 15) == 0;
  float bias[NH];
#pragma unroll
  for (int hq = 0; hq < NH; ++hq) bias[hq] = (head_bias && hq < nh) ? head_bias[h0 + hq] : 0.f;
  const int wave = tid >> 6, lane = tid & 63;
  float acc[NH][NC];
#pragma unroll
  for (int hq = 0; hq < NH; ++hq)
#pragma unroll
    for (int m = 0; m < NC; ++m) acc[hq][m] = 0.f;
  __syncthreads();
  for (int base = key_lo; base < key_hi; base += kAttnTile) {
    const int idx = base + tid;
    if (idx < key_hi) {
      float s[NH];
#pragma unroll
      for (int hq = 0; hq < NH; ++hq) s[hq] = 0.f;
      if (idx < n_blocks) {
        const int last = idx * pool + pool - 1, lp = last / page;
        const size_t at = ((size_t)tbl[lp] * G + g) * pslots + pooled_slot(idx, lp, page, pool);
        score_key<float, NH>(pk_cache + at * dk, qs, dk, nh, vec_p, s);
        vat[tid] = at;
      } else {
        const int j = t_first + (idx - n_blocks);
        const size_t at = ((size_t)tbl[j / page] * G + g) * page + j % page;
        score_key<T, NH>(k_cache + at * dk, qs, dk, nh, vec_t, s);
        vat[tid] = at;
      }
#pragma unroll
      for (int hq = 0; hq < NH; ++hq)
        if (hq < nh) wt[hq * kAttnTile + tid] = sigmoid_f(s[hq] * scale + bias[hq]);
    }
    __syncthreads();
    const int n_here = key_hi - base < kAttnTile ? key_hi - base : kAttnTile;
    // A wave takes every fourth key; kAttnBatch value rows are asked for before any is used.  The
    // tile's pooled keys come first, then its tokens: each loop reads one element type, with
    // unguarded loads on clamped addresses.
    const int nb_here = n_blocks - base < 0 ? 0 : (n_blocks - base < n_here ? n_blocks - base : n_here);
    constexpr int kBatch = NC <= 2 ? 2 * kAttnBatch : kAttnBatch;
    auto sweep = [&](int lo, int hi, auto load_row) {
      for (int kk0 = lo + wave; kk0 < hi; kk0 += 4 * kBatch) {
        float vf[kBatch][NC];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
          const int kk = kk0 + 4 * u < hi ? kk0 + 4 * u : hi - 1;
          const size_t at = vat[kk];
#pragma unroll
          for (int m = 0; m < NC; ++m) vf[u][m] = load_row(at, lane + 64 * m < dv ? lane + 64 * m : dv - 1);
        }
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
          const int kk = kk0 + 4 * u;
          if (kk < hi) {
#pragma unroll
            for (int hq = 0; hq < NH; ++hq) {
              if (hq < nh) {
                const float w = wt[hq * kAttnTile + kk];
#pragma unroll
                for (int m = 0; m < NC; ++m)
                  if (lane + 64 * m < dv) acc[hq][m] = fmaf(w, vf[u][m], acc[hq][m]);
              }
            }
          }
        }
      }
    };
    sweep(0, nb_here, [&](size_t at, int col) { return pv_cache[at * dv + col]; });
    sweep(nb_here, n_here, [&](size_t at, int col) { return ld_f(v_cache + at * dv + col); });
    __syncthreads();
  }
#pragma unroll
  for (int hq = 0; hq < NH; ++hq)
    if (hq < nh)
#pragma unroll
      for (int m = 0; m < NC; ++m)
        if (lane + 64 * m < dv) red[((size_t)wave * nh + hq) * dv + lane + 64 * m] = acc[hq][m];
  __syncthreads();
  float* dst = out + (n_splits > 1 ? (size_t)split * split_stride : 0);
  for (int c = tid; c < nh * dv; c += 256) {
    const size_t step = (size_t)nh * dv;
    dst[(size_t)r * H * dv + (size_t)h0 * dv + c] = ((red[c] + red[step + c]) + red[2 * step + c]) + red[3 * step + c];
  }
}

// out[i] = part[0][i] + part[1][i] + ... in split order
__global__ void sum_splits_kernel(const float* __restrict__ part, size_t split_stride, int n_splits,
                                  float* __restrict__ out, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float sum = part[i];
  for (int sp = 1; sp < n_splits; ++sp) sum += part[(size_t)sp * split_stride + i];
  out[i] = sum;
}

template <typename T, int NH>
void launch_attn_nc(dim3 grid, size_t lds, hipStream_t st, int nc, const float* q, int64_t ldq, const void* kc,
                    const void* vc, const float* pk, const float* pv, const int32_t* row_pos,
                    const int32_t* row_slot, const int32_t* bt, int max_blocks, int page, int pslots, int H, int G,
                    int dk, int dv, int window, int pool, float scale, const float* head_bias, float* out,
                    int n_hgroups, int n_splits, size_t split_stride) {
#define SD_ATTN_GO(NC)                                                                                           \
  window_pool_attn_kernel<T, NH, NC><<<grid, 256, lds, st>>>(q, ldq, (const T*)kc, (const T*)vc, pk, pv, row_pos, \
                                                             row_slot, bt, max_blocks, page, pslots, H, G, dk, dv, \
                                                             window, pool, scale, head_bias, out, n_hgroups,       \
                                                             n_splits, split_stride)
  if (nc == 1) SD_ATTN_GO(1);
  else if (nc == 2) SD_ATTN_GO(2);
  else SD_ATTN_GO(4);
#undef SD_ATTN_GO
}

// x += sigmoid(z1 + c1) * a + sigmoid(z2 + c2) * b   (b == nullptr: one sublayer; c1, c2 may be null)
__global__ void gated_residual_kernel(float* __restrict__ x, const float* __restrict__ z1,
                                      const float* __restrict__ z2, int64_t ldz, const float* __restrict__ c1,
                                      const float* __restrict__ c2, const float* __restrict__ a,
                                      const float* __restrict__ b, int W) {
  const int r = blockIdx.x;
  const int c_end = (blockIdx.y + 1) * kColsPerBlock < W ? (blockIdx.y + 1) * kColsPerBlock : W;
  for (int c = blockIdx.y * kColsPerBlock + threadIdx.x; c < c_end; c += blockDim.x) {
    float add = sigmoid_f(z1[(size_t)r * ldz + c] + (c1 ? c1[c] : 0.f)) * a[(size_t)r * W + c];
    if (b) add += sigmoid_f(z2[(size_t)r * ldz + c] + (c2 ? c2[c] : 0.f)) * b[(size_t)r * W + c];
    x[(size_t)r * W + c] += add;
  }
}

// The same update followed by the next layer's norm of the updated row (one workgroup per row):
// h = x / sqrt(mean(x^2) + eps) * (offset + w), also as bf16 when h_b is given.
template <typename T>
__global__ void gated_residual_norm_kernel(float* __restrict__ x, const float* __restrict__ z1,
                                           const float* __restrict__ z2, int64_t ldz, const float* __restrict__ c1,
                                           const float* __restrict__ c2, const float* __restrict__ a,
                                           const float* __restrict__ b, int W, const T* __restrict__ w, float offset,
                                           float eps, float* __restrict__ h, bf16_t* __restrict__ h_b, int round) {
  __shared__ float red[4];
  const int r = blockIdx.x;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float add = sigmoid_f(z1[(size_t)r * ldz + c] + (c1 ? c1[c] : 0.f)) * a[(size_t)r * W + c];
    if (b) add += sigmoid_f(z2[(size_t)r * ldz + c] + (c2 ? c2[c] : 0.f)) * b[(size_t)r * W + c];
    const float xn = x[(size_t)r * W + c] + add;
    x[(size_t)r * W + c] = xn;
    ss = fmaf(xn, xn, ss);
  }
  ss = block_sum(ss, red);
  const float rstd = 1.f / sqrtf(ss / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += blockDim.x) {   // each thread re-reads what it wrote itself
    const float v = maybe_round(x[(size_t)r * W + c] * rstd * (offset + ld_f(w + c)), round);
    h[(size_t)r * W + c] = v;
    if (h_b) h_b[(size_t)r * W + c] = (bf16_t)v;
  }
}

// out[r, c] = bf16(relu(gate[r, c]) * up[r, c]): the gated feed-forward's activation as the bf16
// operand of the tiled linear kernels
__global__ void relu_mul_rows_kernel(const float* __restrict__ gate, const float* __restrict__ up, int64_t ld,
                                     bf16_t* __restrict__ out, int F) {
  const int r = blockIdx.x;
  const int c_end = (blockIdx.y + 1) * kColsPerBlock < F ? (blockIdx.y + 1) * kColsPerBlock : F;
  for (int c = blockIdx.y * kColsPerBlock + threadIdx.x; c < c_end; c += blockDim.x)
    out[(size_t)r * F + c] = (bf16_t)(fmaxf(gate[(size_t)r * ld + c], 0.f) * up[(size_t)r * ld + c]);
}

// The same product for at most 16 rows: a workgroup takes one row (held in LDS) and a block of
// output columns, a thread owns one column and walks its weight row in 16-byte pieces, many in
// flight.  Every output is summed over k in ascending order with the same fused multiply-adds
// as matmul_rows_kernel: the same bits.
constexpr int kSkinnyRows = 16;
constexpr int kSkinnyLoads = 16;
template <typename T>
__global__ __launch_bounds__(256) void matmul_skinny_kernel(
    const float* __restrict__ X, int64_t ldx, const T* __restrict__ Wt, const float* __restrict__ bias,
    float* __restrict__ Y, int64_t ldy, int N, int K, int round, int64_t bx, int64_t bw, int64_t by,
    bf16_t* __restrict__ Yb, int vec) {
  extern __shared__ float xs[];   // [K]
  const int i = blockIdx.y;
  X += (size_t)blockIdx.z * bx + (size_t)i * ldx;
  Wt += (size_t)blockIdx.z * bw;
  Y += (size_t)blockIdx.z * by + (size_t)i * ldy;
  if (Yb) Yb += (size_t)blockIdx.z * by + (size_t)i * ldy;
  for (int k = threadIdx.x; k < K; k += blockDim.x) xs[k] = maybe_round(X[k], round);
  __syncthreads();
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  if (n >= N) return;
  const T* wr = Wt + (size_t)n * K;
  float acc = 0.f;
  constexpr int E = 16 / sizeof(T);
  int k = 0;
  if (vec) {
    for (; k < K; k += kSkinnyLoads * E) {
      u32x4 raw[kSkinnyLoads];
#pragma unroll
      for (int p = 0; p < kSkinnyLoads; ++p) {   // unguarded, on an address clamped into the row
        const int kp = k + p * E < K ? k + p * E : K - E;
        raw[p] = *reinterpret_cast<const u32x4*>(wr + kp);
      }
#pragma unroll
      for (int p = 0; p < kSkinnyLoads; ++p) {
        if (k + p * E < K) {
          float wf[E];
          if constexpr (sizeof(T) == 2) {
            const bf16x8 v = __builtin_bit_cast(bf16x8, raw[p]);
#pragma unroll
            for (int e = 0; e < E; ++e) wf[e] = (float)v[e];
          } else {
            const f32x4 v = __builtin_bit_cast(f32x4, raw[p]);
#pragma unroll
            for (int e = 0; e < E; ++e) wf[e] = v[e];
          }
#pragma unroll
          for (int e = 0; e < E; ++e) acc = fmaf(xs[k + p * E + e], wf[e], acc);
        }
      }
    }
  } else {
    for (; k < K; ++k) acc = fmaf(xs[k], ld_f(wr + k), acc);
  }
  const float o = acc + (bias ? bias[n] : 0.f);
  Y[n] = o;
  if (Yb) Yb[n] = (bf16_t)o;
}

template <typename T>
int launch_matmul(const float* X, const float* X2, int64_t ldx, const void* Wt, const float* bias, float* Y,
                  int64_t ldy, int M, int N, int K, int round, hipStream_t st, int batch = 1, int64_t bx = 0,
                  int64_t bw = 0, int64_t by = 0, bf16_t* Yb = nullptr) {
  if (M <= kSkinnyRows && !X2 && N >= 64 && (size_t)K * sizeof(float) <= 48 * 1024) {
    const int vec = (K * sizeof(T)) % 16 == 0 && (bw * sizeof(T)) % 16 == 0 && sd_aligned16(Wt);
    const int nthr = N >= 4096 ? 256 : (N >= 1024 ? 128 : 64);   // few columns: more, smaller workgroups
    dim3 grid((N + nthr - 1) / nthr, M, batch);
    matmul_skinny_kernel<T><<<grid, nthr, (size_t)K * sizeof(float), st>>>(X, ldx, (const T*)Wt, bias, Y, ldy, N, K,
                                                                           round, bx, bw, by, Yb, vec);
    SD_CHECK_LAUNCH("sd_matmul_rows");
    return SD_OK;
  }
  if (M <= 16) {
    dim3 grid((N + 127) / 128, (M + 15) / 16, batch);
    matmul_rows_kernel<T, 16, 128, 2, 4><<<grid, 256, 0, st>>>(X, X2, ldx, (const T*)Wt, bias, Y, ldy, M, N, K, round,
                                                               bx, bw, by, Yb);
  } else {
    dim3 grid((N + 63) / 64, (M + 63) / 64, batch);
    matmul_rows_kernel<T, 64, 64, 4, 4><<<grid, 256, 0, st>>>(X, X2, ldx, (const T*)Wt, bias, Y, ldy, M, N, K, round,
                                                              bx, bw, by, Yb);
  }
  SD_CHECK_LAUNCH("sd_matmul_rows");
  return SD_OK;
}

}  // namespace

// ====================================================================== C entry points
extern "C" int sd_matmul_rows(const float* x, const float* x2, int64_t ldx, const void* w, int w_f32,
                              const float* bias, float* y, int64_t ldy, int M, int N, int K,
                              sd_stream_t stream) {
  SD_REQUIRE(x && w && y && M >= 1 && N >= 1 && K >= 1 && ldx >= K && ldy >= N, SD_ERR_INVALID,
             "sd_matmul_rows: bad argument (M=%d N=%d K=%d)", M, N, K);
  hipStream_t st = (hipStream_t)stream;
  return w_f32 ? launch_matmul<float>(x, x2, ldx, w, bias, y, ldy, M, N, K, 0, st)
               : launch_matmul<bf16_t>(x, x2, ldx, w, bias, y, ldy, M, N, K, 1, st);
}

extern "C" int sd_matmul_rows_batched(const float* x, int64_t ldx, int64_t bx, const void* w, int w_f32, int64_t bw,
                                      float* y, int64_t ldy, int64_t by, void* y_bf16, int M, int N, int K, int batch,
                                      sd_stream_t stream) {
  SD_REQUIRE(x && w && y && M >= 1 && N >= 1 && K >= 1 && batch >= 1 && batch <= 65535 && ldx >= K && ldy >= N,
             SD_ERR_INVALID, "sd_matmul_rows_batched: bad argument (M=%d N=%d K=%d batch=%d)", M, N, K, batch);
  hipStream_t st = (hipStream_t)stream;
  return w_f32 ? launch_matmul<float>(x, nullptr, ldx, w, nullptr, y, ldy, M, N, K, 0, st, batch, bx, bw, by, (bf16_t*)y_bf16)
               : launch_matmul<bf16_t>(x, nullptr, ldx, w, nullptr, y, ldy, M, N, K, 1, st, batch, bx, bw, by, (bf16_t*)y_bf16);
}

extern "C" int sd_rmsnorm_rows(const float* x, const int32_t* rows, const void* w, int w_f32, float offset,
                               float eps, float* out, void* out_bf16, int n, int W, sd_stream_t stream) {
  SD_REQUIRE(x && w && out && n >= 1 && W >= 1, SD_ERR_INVALID, "sd_rmsnorm_rows: bad argument");
  hipStream_t st = (hipStream_t)stream;
  bf16_t* ob = (bf16_t*)out_bf16;
  if (w_f32) rmsnorm_rows_kernel<float><<<n, 256, 0, st>>>(x, rows, (const float*)w, offset, eps, out, ob, W, 0);
  else rmsnorm_rows_kernel<bf16_t><<<n, 256, 0, st>>>(x, rows, (const bf16_t*)w, offset, eps, out, ob, W, 1);
  SD_CHECK_LAUNCH("sd_rmsnorm_rows");
  return SD_OK;
}

extern "C" int sd_head_prep(float* q, float* k, const float* v, int64_t ld, const int32_t* row_pos,
                            const int32_t* row_slot, int n_rows, int Hq, int Hk, int dk, int dv,
                            int rot_dims, int rot_layout, const double* inv_freq, int unit_norm, float eps,
                            float q_scale, float k_scale, void* k_cache, void* v_cache, int cache_f32,
                            const int32_t* block_tables, int max_blocks, int page, sd_stream_t stream) {
  SD_REQUIRE(q && k && row_pos && n_rows >= 1 && Hq >= 1 && Hk >= 1 && dk >= 1, SD_ERR_INVALID,
             "sd_head_prep: bad argument");
  SD_REQUIRE(rot_dims >= 0 && rot_dims <= dk && rot_dims % 2 == 0 && (rot_dims == 0 || inv_freq),
             SD_ERR_INVALID, "sd_head_prep: rot_dims %d must be even, at most dim %d, with a frequency table",
             rot_dims, dk);
  SD_REQUIRE(!k_cache || (v_cache && v && row_slot && block_tables && page >= 1 && max_blocks >= 1),
             SD_ERR_INVALID, "sd_head_prep: a cache needs values, slots and block tables");
  hipStream_t st = (hipStream_t)stream;
  dim3 grid(n_rows, Hq + Hk);
  if (cache_f32)
    head_prep_kernel<float><<<grid, 64, 0, st>>>(q, k, v, ld, row_pos, row_slot, Hq, Hk, dk, dv, rot_dims,
                                                 rot_layout, inv_freq, unit_norm, eps, q_scale, k_scale,
                                                 (float*)k_cache, (float*)v_cache, block_tables, max_blocks, page);
  else
    head_prep_kernel<bf16_t><<<grid, 64, 0, st>>>(q, k, v, ld, row_pos, row_slot, Hq, Hk, dk, dv, rot_dims,
                                                  rot_layout, inv_freq, unit_norm, eps, q_scale, k_scale,
                                                  (bf16_t*)k_cache, (bf16_t*)v_cache, block_tables, max_blocks, page);
  SD_CHECK_LAUNCH("sd_head_prep");
  return SD_OK;
}

extern "C" int sd_sigmoid_power(const float* z, int64_t ldz, float tau, float* out, int n_rows, int n_cols,
                                sd_stream_t stream) {
  SD_REQUIRE(z && out && n_rows >= 1 && n_cols >= 1 && tau > 0.f, SD_ERR_INVALID, "sd_sigmoid_power: bad argument");
  sigmoid_power_kernel<<<dim3(n_rows, (n_cols + kColsPerBlock - 1) / kColsPerBlock), 256, 0, (hipStream_t)stream>>>(
      z, ldz, 1.f / tau, out, n_cols);
  SD_CHECK_LAUNCH("sd_sigmoid_power");
  return SD_OK;
}

extern "C" int sd_decay_scan(const float* q, const float* k, const float* v, int64_t ld, const float* decay,
                             int per_channel, float* state, const int32_t* entries, int n_entries,
                             float* out, int H, int dk, int dv, sd_stream_t stream) {
  SD_REQUIRE(q && k && v && decay && state && entries && out && n_entries >= 1 && H >= 1 && dv >= 1,
             SD_ERR_INVALID, "sd_decay_scan: bad argument");
  SD_REQUIRE(dk >= 1 && dk <= 256, SD_ERR_UNSUPPORTED, "sd_decay_scan: key size %d outside 1..256", dk);
  const int NS = (dk + kStrip - 1) / kStrip;
  hipStream_t st = (hipStream_t)stream;
  int CT = 256 / NS;
  if (CT > dv) CT = dv;
  if (CT > 64) CT = 64;
  const int tiles = (dv + CT - 1) / CT;
  const int dkp = NS * kStrip;
  int CH = kScanLoads * (CT * NS) / dkp;   // a chunk's q / k elements fit kScanLoads per thread
  if (CH > kScanChunk) CH = kScanChunk;
  SD_REQUIRE(CH >= 1 && CH * CT <= kScanLoadsV * CT * NS, SD_ERR_UNSUPPORTED,
             "sd_decay_scan: key size %d with value size %d leaves no chunk", dk, dv);
  const size_t lds = sizeof(float) * ((size_t)(per_channel ? 3 : 2) * CH * dkp + (size_t)CH * CT + (size_t)CH * NS * CT);
  dim3 grid(tiles, H, n_entries);
  if (per_channel)
    decay_scan_kernel<true><<<grid, CT * NS, lds, st>>>(q, k, v, ld, decay, state, entries, out, H, dk, dv, CT, NS, CH);
  else
    decay_scan_kernel<false><<<grid, CT * NS, lds, st>>>(q, k, v, ld, decay, state, entries, out, H, dk, dv, CT, NS, CH);
  SD_CHECK_LAUNCH("sd_decay_scan");
  return SD_OK;
}

extern "C" int sd_head_post(const float* o, const float* g, int64_t ldg, const void* norm_w, int w_f32,
                            int unit_norm, float eps, int gate_kind, float* y, void* y_bf16, int n_rows, int H,
                            int dv, int round_bf16_out, sd_stream_t stream) {
  SD_REQUIRE(o && g && y && n_rows >= 1 && H >= 1 && dv >= 1, SD_ERR_INVALID, "sd_head_post: bad argument");
  dim3 grid(n_rows, H);
  hipStream_t st = (hipStream_t)stream;
  if (w_f32)
    head_post_kernel<float><<<grid, 64, 0, st>>>(o, g, ldg, (const float*)norm_w, unit_norm, eps, gate_kind, y, (bf16_t*)y_bf16, H, dv, round_bf16_out);
  else
    head_post_kernel<bf16_t><<<grid, 64, 0, st>>>(o, g, ldg, (const bf16_t*)norm_w, unit_norm, eps, gate_kind, y, (bf16_t*)y_bf16, H, dv, round_bf16_out);
  SD_CHECK_LAUNCH("sd_head_post");
  return SD_OK;
}

extern "C" int sd_pooled_slots_per_page(int page, int pool) {
  if (page < 1 || pool < 1) return 0;
  return page / pool + 2;
}

extern "C" size_t sd_window_pool_attention_scratch_bytes(int n_rows, int H, int dv, int window, int pool,
                                                        int max_ctx) {
  if (n_rows < 1 || n_rows > kAttnSplitRows || pool < 1) return 0;
  const int max_keys = window + max_ctx / pool + 1;
  const int splits = (max_keys + kAttnTile - 1) / kAttnTile;
  return splits > 1 ? (size_t)splits * n_rows * H * dv * sizeof(float) : 0;
}

extern "C" int sd_window_pool_attention(const float* q, int64_t ldq, const void* k_cache, const void* v_cache,
                                        int cache_f32, float* pk_cache, float* pv_cache,
                                        const int32_t* row_pos, const int32_t* row_slot,
                                        const int32_t* block_tables, int max_blocks, int page, int n_rows,
                                        int H, int G, int dk, int dv, int window, int pool, float scale,
                                        const float* head_bias, float* out, void* scratch, size_t scratch_bytes,
                                        sd_stream_t stream) {
  SD_REQUIRE(q && k_cache && v_cache && pk_cache && pv_cache && row_pos && row_slot && block_tables && out,
             SD_ERR_INVALID, "sd_window_pool_attention: null argument");
  SD_REQUIRE(n_rows >= 1 && H >= 1 && G >= 1 && H % G == 0 && dk >= 1 && window >= 1 && pool >= 1 && page >= 1,
             SD_ERR_INVALID, "sd_window_pool_attention: bad shape");
  SD_REQUIRE(dv >= 1 && dv <= 256, SD_ERR_UNSUPPORTED, "sd_window_pool_attention: value size %d outside 1..256", dv);
  const int pslots = sd_pooled_slots_per_page(page, pool);
  hipStream_t st = (hipStream_t)stream;
  dim3 gp(n_rows, G);
  const int qh = H / G;
  const int NH = qh <= 1 ? 1 : (qh <= 2 ? 2 : (qh <= 4 ? 4 : 8));
  const int nh = qh < NH ? qh : NH;
  const int n_hgroups = (qh + NH - 1) / NH;
  const int nc = dv <= 64 ? 1 : (dv <= 128 ? 2 : 4);
  // Few rows: the keys of a row are cut into tiles that run as workgroups of their own.
  const size_t need = sd_window_pool_attention_scratch_bytes(n_rows, H, dv, window, pool, max_blocks * page);
  const bool split = need > 0 && scratch && scratch_bytes >= need;
  const int n_splits = split ? (int)(need / ((size_t)n_rows * H * dv * sizeof(float))) : 1;
  const size_t split_stride = (size_t)n_rows * H * dv;
  dim3 ga(n_rows, G, n_hgroups * n_splits);
  const size_t lds = sizeof(unsigned long long) * kAttnTile +
                     sizeof(float) * ((size_t)NH * kAttnTile + (size_t)NH * dk + (size_t)4 * nh * dv);
  SD_REQUIRE(lds <= 64 * 1024, SD_ERR_UNSUPPORTED, "sd_window_pool_attention: dim %d / vdim %d need %zu bytes of LDS",
             dk, dv, lds);
  float* dst = split ? (float*)scratch : out;
  if (cache_f32)
    pool_blocks_kernel<float><<<gp, 64, 0, st>>>((const float*)k_cache, (const float*)v_cache, pk_cache, pv_cache,
                                                 row_pos, row_slot, block_tables, max_blocks, page, pslots, G, dk, dv, pool);
  else
    pool_blocks_kernel<bf16_t><<<gp, 64, 0, st>>>((const bf16_t*)k_cache, (const bf16_t*)v_cache, pk_cache, pv_cache,
                                                  row_pos, row_slot, block_tables, max_blocks, page, pslots, G, dk, dv, pool);
  SD_CHECK_LAUNCH("sd_window_pool_attention (pool)");
#define SD_ATTN_NH(T, N)                                                                                          \
  launch_attn_nc<T, N>(ga, lds, st, nc, q, ldq, k_cache, v_cache, pk_cache, pv_cache, row_pos, row_slot, block_tables, \
                       max_blocks, page, pslots, H, G, dk, dv, window, pool, scale, head_bias, dst, n_hgroups,     \
                       n_splits, split_stride)
#define SD_ATTN_T(T)                  \
  do {                                \
    if (NH == 1) SD_ATTN_NH(T, 1);    \
    else if (NH == 2) SD_ATTN_NH(T, 2); \
    else if (NH == 4) SD_ATTN_NH(T, 4); \
    else SD_ATTN_NH(T, 8);            \
  } while (0)
  if (cache_f32) SD_ATTN_T(float);
  else SD_ATTN_T(bf16_t);
#undef SD_ATTN_T
#undef SD_ATTN_NH
  SD_CHECK_LAUNCH("sd_window_pool_attention");
  if (split) {
    const size_t n = split_stride;
    sum_splits_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>((const float*)scratch, split_stride, n_splits, out, n);
    SD_CHECK_LAUNCH("sd_window_pool_attention (sum)");
  }
  return SD_OK;
}

extern "C" int sd_gated_residual(float* x, const float* z1, const float* z2, int64_t ldz, const float* c1,
                                 const float* c2, const float* a, const float* b, int n_rows, int W,
                                 sd_stream_t stream) {
  SD_REQUIRE(x && z1 && a && (!b || z2) && n_rows >= 1 && W >= 1, SD_ERR_INVALID, "sd_gated_residual: bad argument");
  gated_residual_kernel<<<dim3(n_rows, (W + kColsPerBlock - 1) / kColsPerBlock), 256, 0, (hipStream_t)stream>>>(
      x, z1, z2, ldz, c1, c2, a, b, W);
  SD_CHECK_LAUNCH("sd_gated_residual");
  return SD_OK;
}

extern "C" int sd_gated_residual_norm(float* x, const float* z1, const float* z2, int64_t ldz, const float* c1,
                                      const float* c2, const float* a, const float* b, int n_rows, int W,
                                      const void* norm_w, int w_f32, float offset, float eps, float* h,
                                      void* h_bf16, sd_stream_t stream) {
  SD_REQUIRE(x && z1 && a && (!b || z2) && norm_w && h && n_rows >= 1 && W >= 1, SD_ERR_INVALID,
             "sd_gated_residual_norm: bad argument");
  hipStream_t st = (hipStream_t)stream;
  if (w_f32)
    gated_residual_norm_kernel<float><<<n_rows, 256, 0, st>>>(x, z1, z2, ldz, c1, c2, a, b, W, (const float*)norm_w,
                                                              offset, eps, h, (bf16_t*)h_bf16, 0);
  else
    gated_residual_norm_kernel<bf16_t><<<n_rows, 256, 0, st>>>(x, z1, z2, ldz, c1, c2, a, b, W, (const bf16_t*)norm_w,
                                                               offset, eps, h, (bf16_t*)h_bf16, 1);
  SD_CHECK_LAUNCH("sd_gated_residual_norm");
  return SD_OK;
}

extern "C" int sd_relu_mul_rows(const float* gate, const float* up, int64_t ld, void* out_bf16, int n_rows,
                                int F, sd_stream_t stream) {
  SD_REQUIRE(gate && up && out_bf16 && n_rows >= 1 && F >= 1 && ld >= F, SD_ERR_INVALID,
             "sd_relu_mul_rows: bad argument");
  relu_mul_rows_kernel<<<dim3(n_rows, (F + kColsPerBlock - 1) / kColsPerBlock), 256, 0, (hipStream_t)stream>>>(
      gate, up, ld, (bf16_t*)out_bf16, F);
  SD_CHECK_LAUNCH("sd_relu_mul_rows");
  return SD_OK;
}

// ====================================================================== the layer-list model
struct sd_seq_model {
  sd_seq_model_desc d;
  std::vector<sd_seq_layer> layers;
};

namespace {
struct InCols {  // column offsets inside a layer's fused input projection
  int q, k, v, g, r1, r2, gate, up, a1, total;
};
InCols in_cols(const sd_seq_layer& l, int W) {
  InCols c;
  int at = 0;
  c.q = at;    at += l.heads * l.dim;
  c.k = at;    at += l.kv_heads * l.dim;
  c.v = at;    at += l.kv_heads * l.vdim;
  c.g = at;    at += l.heads * l.vdim;
  c.r1 = at;   at += W;
  c.r2 = at;   at += l.ff > 0 ? W : 0;
  c.gate = at; at += l.ff;
  c.up = at;   at += l.ff;
  c.a1 = at;   at += l.kind == SD_MIX_CHANNEL_DECAY ? l.rank : 0;
  c.total = at;
  return c;
}
inline size_t al(size_t v) { return (v + 255) & ~(size_t)255; }
constexpr int kWideRows = 256;  // rows one call of the many-row linear family takes
struct SeqWs {
  size_t x, h, proj, dec, o, y, mix, ffo, hout, hb, yb, actb, houtb, wide, wide_bytes, attn, attn_bytes, total;
  size_t sg;   // a shared expert's gate per row
  // layers normed on their output
  size_t pq, qe, cqb, conv, step, decay, rlog, sel_e, sel_w, dn, moe, moe_bytes;
};
// column offsets inside the fused input projection of a layer normed on its output
struct PnCols {
  int dq, dkv, q, k, v, z, xbc, dt, total, inner, conv_ch;
};
// column offsets inside the fused input projection of a layer normed before and after its sublayers
struct SwCols {
  int q, dkv, g, k, v, total;
};
SwCols sw_cols(const sd_seq_layer& l) {
  SwCols c = {};
  int at = 0;
  if (l.kind == SD_MIX_LATENT) {
    c.q = at;   at += l.heads * (l.dim + l.rot_dim);
    c.dkv = at; at += l.kv_rank + l.rot_dim;
    c.g = at;   at += l.head_gate ? l.heads : 0;
  } else {
    const int maps = l.maps > 1 ? l.maps : 1;
    c.q = at; at += l.heads * maps * l.dim;
    c.k = at; at += l.kv_shared ? 0 : l.kv_heads * maps * l.dim;
    c.v = at; at += l.kv_shared || l.value_from_key ? 0 : l.kv_heads * l.vdim;
  }
  c.total = at;
  return c;
}
// whether a grouped-query softmax layer needs the general preparation (sd_attn_prep) rather than
// norms per head alone (sd_qk_head_norm_append)
inline bool general_prep(const sd_seq_layer& l) {
  return l.maps > 1 || l.rot_dims > 0 || l.w_in_bias || l.qk_full_norm || l.value_from_key || l.kv_shared ||
         !l.qk_head_norm;
}
inline int act_inputs(int act_kind) { return act_kind == 2 ? 1 : 2; }   // matrices an activation of sd_act_rows reads
PnCols pn_cols(const sd_seq_layer& l) {
  PnCols c = {};
  int at = 0;
  if (l.kind == SD_MIX_LATENT) {
    c.dq = at;  at += l.q_rank;
    c.dkv = at; at += l.kv_rank + l.rot_dim;
  } else {
    c.inner = l.s_heads * l.s_vdim;
    c.conv_ch = c.inner + 2 * l.s_groups * l.s_state;
    c.q = at;   at += l.heads * l.dim;
    c.k = at;   at += l.kv_heads * l.dim;
    c.v = at;   at += l.kv_heads * l.vdim;
    c.z = at;   at += c.inner;
    c.xbc = at; at += c.conv_ch;
    c.dt = at;  at += l.s_heads;
  }
  c.total = at;
  return c;
}
SeqWs plan_seq(const sd_seq_model& m, int rows, int n_out, int max_ctx) {
  const int W = m.d.width;
  size_t proj = 0, hk = 0, hv = 0, ff = 0, wide = 0, attn = 0;
  size_t pq = 0, qe = 0, cq = 0, conv = 0, sh = 0, ne = 0, top = 0, moe = 0;
  const int wr = rows < kWideRows ? rows : kWideRows;
  auto up = [](size_t& a, size_t b) { a = b > a ? b : a; };
  auto need = [&](const void* tiled, int M, int N, int K) {
    if (!tiled || M <= 16) return;
    const size_t n = sd_linear_wide_workspace_bytes(M, N, K, SD_EPI_F32);
    wide = n > wide ? n : wide;
  };
  for (const sd_seq_layer& l : m.layers) {
    if (l.block == SD_BLOCK_SANDWICH) {
      const SwCols c = sw_cols(l);
      up(proj, (size_t)c.total);
      need(l.w_in_tiled, wr, c.total, W);
      need(l.w_o_tiled, wr, W, l.heads * l.vdim);
      const int maps = l.kind == SD_MIX_SOFTMAX && l.maps > 1 ? l.maps : 1;
      up(hv, (size_t)l.heads * maps * l.vdim);
      up(attn, sd_multimap_softmax_attention_scratch_bytes(rows, l.heads, maps, l.kind == SD_MIX_LATENT ? l.kv_rank : l.vdim,
                                                           l.window, 0, l.chunk, max_ctx));
      if (l.kind == SD_MIX_LATENT) {
        up(qe, (size_t)l.heads * (l.kv_rank + l.rot_dim));
        up(hv, (size_t)l.heads * l.kv_rank);
      }
      if (l.ff > 0) {
        up(proj, (size_t)act_inputs(l.ff_act) * l.ff);
        up(ff, (size_t)l.ff);
        need(l.w_ff_in_tiled, wr, act_inputs(l.ff_act) * l.ff, W);
        need(l.w_down_tiled, wr, W, l.ff);
      }
      if (l.n_experts > 0) {
        up(ne, (size_t)l.n_experts);
        up(top, (size_t)l.top);
        up(moe, sd_moe_experts_scratch_bytes(rows, l.top, l.n_experts, l.expert_ff, W));
      }
      if (l.shared_ff > 0) {
        up(proj, (size_t)act_inputs(l.shared_act) * l.shared_ff);
        up(ff, (size_t)l.shared_ff);
        need(l.w_shared_in_tiled, wr, act_inputs(l.shared_act) * l.shared_ff, W);
        need(l.w_shared_down_tiled, wr, W, l.shared_ff);
      }
      continue;
    }
    if (l.block == SD_BLOCK_POSTNORM) {
      const PnCols c = pn_cols(l);
      up(proj, (size_t)c.total);
      need(l.w_in_tiled, wr, c.total, W);
      need(l.w_o_tiled, wr, W, l.heads * l.vdim);
      up(hv, (size_t)l.heads * l.vdim);
      up(attn, sd_window_softmax_attention_scratch_bytes(rows, l.heads, l.kind == SD_MIX_LATENT ? l.kv_rank : l.vdim,
                                                         l.window, l.keep_first, max_ctx));
      if (l.kind == SD_MIX_LATENT) {
        up(pq, (size_t)l.heads * (l.dim + l.rot_dim));
        up(qe, (size_t)l.heads * (l.kv_rank + l.rot_dim));
        up(cq, (size_t)l.q_rank);
        up(hv, (size_t)l.heads * l.kv_rank);
        need(l.w_uq_tiled, wr, l.heads * (l.dim + l.rot_dim), l.q_rank);
      } else {
        up(hv, (size_t)c.inner);
        up(conv, (size_t)c.conv_ch);
        up(sh, (size_t)l.s_heads);
        need(l.w_o2_tiled, wr, W, c.inner);
      }
      if (l.n_experts > 0) {
        up(ne, (size_t)l.n_experts);
        up(top, (size_t)l.top);
        up(moe, sd_moe_experts_scratch_bytes(rows, l.top, l.n_experts, l.expert_ff, W));
      }
      continue;
    }
    const size_t t = in_cols(l, W).total;
    proj = t > proj ? t : proj;
    const size_t a = (size_t)l.heads * l.dim, b = (size_t)l.heads * l.vdim;
    hk = a > hk ? a : hk;
    hv = b > hv ? b : hv;
    ff = (size_t)l.ff > ff ? (size_t)l.ff : ff;
    need(l.w_in_tiled, wr, (int)t, W);
    need(l.w_o_tiled, wr, W, l.heads * l.vdim);
    need(l.w_down_tiled, wr, W, l.ff);
    if (l.kind == SD_MIX_WINDOW_POOL) {
      const size_t n = sd_window_pool_attention_scratch_bytes(rows, l.heads, l.vdim, l.window, l.pool, max_ctx);
      attn = n > attn ? n : attn;
    }
  }
  const int no = n_out > 0 ? n_out : 1;
  need(m.d.head_tiled, no < kWideRows ? no : kWideRows, m.d.vocab, W);
  SeqWs w;
  size_t off = 0;
  const size_t R = (size_t)rows, f = sizeof(float);
  w.x = off;    off += al(R * W * f);
  w.h = off;    off += al(R * W * f);
  w.proj = off; off += al(R * proj * f);
  w.dec = off;  off += al(R * hk * f);   // low-rank decay logits, then decays
  w.o = off;    off += al(R * hv * f);
  w.y = off;    off += al(R * hv * f);
  w.mix = off;  off += al(R * W * f);
  w.ffo = off;  off += al(R * W * f);
  w.hout = off; off += al((size_t)no * W * f);
  // bf16 copies of the matrix products' operands, for the tiled linear kernels
  w.hb = off;    off += al(R * W * 2);
  w.yb = off;    off += al(R * hv * 2);
  w.actb = off;  off += al(R * (ff ? ff : 1) * 2);
  w.houtb = off; off += al((size_t)no * W * 2);
  w.wide_bytes = wide;
  w.wide = off; off += al(wide ? wide : 16);
  w.attn_bytes = attn;
  w.attn = off; off += al(attn ? attn : 16);
  w.pq = off;    off += al(R * pq * f);
  w.qe = off;    off += al(R * qe * f);
  w.cqb = off;   off += al(R * cq * 2);
  w.conv = off;  off += al(R * conv * f);
  w.step = off;  off += al(R * sh * f);
  w.decay = off; off += al(R * sh * f);
  w.rlog = off;  off += al(R * ne * f);
  w.sel_e = off; off += al(R * top * sizeof(int32_t));
  w.sel_w = off; off += al(R * top * f);
  w.dn = off;    off += al(R * top * W * f);
  w.moe_bytes = moe;
  w.moe = off;   off += al(moe ? moe : 16);
  w.sg = off;    off += al(R * f);
  w.total = off;
  return w;
}

// y[M, N] f32 = x w^T: through the tiled bf16 kernels of the other decoders when the matrix has a
// tiled copy (x_b: the operand as bf16), else the plain kernel over the row-major matrix.
int seq_linear(const void* w_rm, const void* w_tiled, int w_f32, const float* x, const float* x2, int64_t ldx,
               const void* x_b, int64_t ldxb, const float* bias, float* y, int64_t ldy, int M, int N, int K,
               void* wide_ws, size_t wide_bytes, sd_stream_t stream) {
  if (!w_tiled) return sd_matmul_rows(x, x2, ldx, w_rm, w_f32, bias, y, ldy, M, N, K, stream);
  SD_REQUIRE(!bias, SD_ERR_INVALID, "seq_linear: a tiled matrix takes no f32 bias");
  if (M <= 16) return sd_linear(w_tiled, nullptr, x_b, ldxb, nullptr, nullptr, y, ldy, M, N, K, SD_EPI_F32, stream);
  for (int r0 = 0; r0 < M; r0 += kWideRows) {
    const int mm = M - r0 < kWideRows ? M - r0 : kWideRows;
    const int rc = sd_linear_wide(w_tiled, nullptr, (const bf16_t*)x_b + (size_t)r0 * ldxb, ldxb, nullptr, nullptr,
                                  y + (size_t)r0 * ldy, ldy, mm, N, K, SD_EPI_F32, wide_ws, wide_bytes, stream);
    if (rc != SD_OK) return rc;
  }
  return SD_OK;
}
}  // namespace

extern "C" sd_seq_model* sd_seq_model_create(const sd_seq_model_desc* desc) {
  if (!desc || !desc->layers || desc->n_layers < 1 || desc->width < 1 || desc->vocab < 1 || !desc->embed ||
      !desc->final_norm_w) {
    sd_set_error("sd_seq_model_create: null descriptor, no layers or a missing table");
    return nullptr;
  }
  sd_seq_model* m = new sd_seq_model;
  m->d = *desc;
  m->layers.assign(desc->layers, desc->layers + desc->n_layers);
  m->d.layers = m->layers.data();
  for (int i = 0; i < desc->n_layers; ++i) {
    const sd_seq_layer& l = m->layers[i];
    const char* bad = nullptr;
    if (l.block == SD_BLOCK_SANDWICH) {
      if (l.kind != SD_MIX_LATENT && l.kind != SD_MIX_SOFTMAX) bad = "a layer normed before and after its sublayers takes latent or grouped-query softmax attention";
      else if (i > 0 && m->layers[i - 1].block != SD_BLOCK_SANDWICH) bad = "it follows a layer of another kind";
      else if (l.heads < 1 || l.dim < 1 || l.vdim < 1 || l.window < 1 || l.chunk < 0 || l.softcap < 0.f) bad = "head counts / sizes / window / chunk / cap";
      else if (!l.norm_w || !l.post_norm_w || !(l.w_in || l.w_in_tiled) || !(l.w_o || l.w_o_tiled) || !l.k_cache) bad = "a null weight or cache";
      else if ((l.w_in_tiled || l.w_o_tiled || l.w_ff_in_tiled || l.w_down_tiled || l.w_shared_in_tiled || l.w_shared_down_tiled) && desc->weights_f32) bad = "tiled matrices are bf16";
      else if (l.kind == SD_MIX_LATENT && (l.q_rank != 0 || l.kv_rank < 1 || l.kv_rank > 512 || l.rot_dim < 0 || l.rot_dims < 0 || l.rot_dims > l.rot_dim ||
               l.rot_dims % 2 || (l.rot_dims && !l.inv_freq) || !l.dkv_norm_w || !l.w_uk_t || !l.w_uv)) bad = "latent size / rotary dims / a null latent weight";
      else if (l.kind == SD_MIX_SOFTMAX && (l.kv_heads < 1 || l.heads % l.kv_heads || l.vdim > 512 || !l.v_cache)) bad = "attention needs kv heads that divide the heads, vdim <= 512 and a value cache";
      else if (l.kind == SD_MIX_SOFTMAX && ((l.qk_head_norm && l.qk_full_norm) || ((l.qk_head_norm || l.qk_full_norm) && (!l.q_norm_w || (!l.kv_shared && !l.k_norm_w))))) bad = "q and k are normed per head or over the whole projection, with weights for both";
      else if (l.kind == SD_MIX_SOFTMAX && (l.maps < 0 || l.maps > 2 || (l.value_from_key && (l.maps > 1 || l.vdim != l.dim || l.kv_shared)) || (l.kv_shared && i == 0))) bad = "one or two score maps; values taken from keys need one map and vdim == dim; shared keys need an earlier layer";
      else if (l.kind == SD_MIX_SOFTMAX && (l.rot_dims < 0 || l.rot_dims % 2 || l.rot_dims > l.dim || (l.rot_dims && !l.inv_freq))) bad = "rotary dims";
      else if (l.ff < 0 || (l.ff > 0 && (l.n_experts > 0 || l.ff_act < 0 || l.ff_act > 2 || !(l.w_ff_in || l.w_ff_in_tiled) || !(l.w_down || l.w_down_tiled)))) bad = "a dense feed-forward needs its two matrices and a known activation, and excludes experts";
      else if (l.n_experts > 0 && (l.top < 1 || l.top > l.n_experts || l.expert_ff < 1 || !l.w_router || !l.w_gate_up || !l.w_down_e || l.expert_act < 0 || l.expert_act > 1)) bad = "routed experts need top <= experts, their matrices and a known activation";
      else if (l.shared_ff < 0 || (l.shared_ff > 0 && (l.n_experts < 1 || l.shared_act < 0 || l.shared_act > 2 || !(l.w_shared_in || l.w_shared_in_tiled) || !(l.w_shared_down || l.w_shared_down_tiled)))) bad = "a shared expert stands beside routed experts and needs its matrices";
      else if ((l.ff > 0 || l.n_experts > 0) && (!l.norm2_w || !l.post_norm2_w)) bad = "a feed-forward needs its two norms";
    } else
    if (l.block == SD_BLOCK_POSTNORM) {
      if (l.kind != SD_MIX_LATENT && l.kind != SD_MIX_SOFTMAX_SSD) bad = "a layer normed on its output takes latent attention or attention beside a state-space recurrence";
      else if (i > 0 && m->layers[i - 1].block == SD_BLOCK_SANDWICH) bad = "it follows a layer normed before and after its sublayers";
      else if (l.heads < 1 || l.dim < 1 || l.vdim < 1 || l.window < 1 || l.keep_first < 0) bad = "head counts / sizes / window";
      else if (!l.norm_w || !(l.w_in || l.w_in_tiled) || !(l.w_o || l.w_o_tiled) || !l.k_cache) bad = "a null weight or cache";
      else if ((l.w_in_tiled || l.w_o_tiled || l.w_uq_tiled || l.w_o2_tiled) && desc->weights_f32) bad = "tiled matrices are bf16";
      else if (l.ff != 0) bad = "a dense feed-forward is not provided for layers normed on their output";
      else if (l.n_experts > 0 && (l.top < 1 || l.top > l.n_experts || l.expert_ff < 1 || !l.w_router || !l.w_gate_up || !l.w_down_e || !l.norm2_w)) bad = "routed experts need top <= experts, their matrices and norm2";
      else if (l.kind == SD_MIX_LATENT) {
        if (l.q_rank < 1 || l.kv_rank < 1 || l.rot_dim < 0 || l.rot_dims < 0 || l.rot_dims > l.rot_dim || l.rot_dims % 2 ||
            (l.rot_dims && !l.inv_freq)) bad = "latent ranks / rotary dims";
        else if (!l.dq_norm_w || !l.dkv_norm_w || !(l.w_uq || l.w_uq_tiled) || !l.w_uk_t || !l.w_uv) bad = "a null latent weight";
        else if (l.kv_rank > 512) bad = "latent size above 512";
      } else {
        if (l.kv_heads < 1 || l.heads % l.kv_heads || l.vdim > 512 || !l.v_cache || !l.q_norm_w || !l.k_norm_w) bad = "attention part";
        else if (l.s_heads < 1 || l.s_vdim < 1 || l.s_state < 1 || l.s_state > 256 || l.s_groups < 1 || l.s_heads % l.s_groups ||
                 l.s_taps < 1 || l.s_norm_groups < 1 || (l.s_heads * l.s_vdim) % l.s_norm_groups) bad = "state-space sizes";
        else if (!l.conv_w || !l.dt_bias || !l.a_log || !l.s_norm_w || !(l.w_o2 || l.w_o2_tiled) || !l.state ||
                 (l.s_taps > 1 && !l.conv_state)) bad = "a null state-space weight or state";
      }
    } else
    if (l.kind != SD_MIX_HEAD_DECAY && l.kind != SD_MIX_CHANNEL_DECAY && l.kind != SD_MIX_WINDOW_POOL) bad = "unknown mixer";
    else if (l.heads < 1 || l.kv_heads < 1 || l.heads % l.kv_heads || l.dim < 1 || l.vdim < 1) bad = "head counts / sizes";
    else if (!l.norm_w || !(l.w_in || l.w_in_tiled) || !(l.w_o || l.w_o_tiled) ||
             (l.ff > 0 && !(l.w_down || l.w_down_tiled)) || l.ff < 0) bad = "a null weight";
    else if ((l.w_in_tiled || l.w_o_tiled || l.w_down_tiled) && desc->weights_f32) bad = "tiled matrices are bf16";
    else if ((l.w_in_tiled && desc->width % 32) || (l.w_o_tiled && (l.heads * l.vdim) % 32) ||
             (l.w_down_tiled && l.ff % 32)) bad = "a tiled matrix needs an input width that is a multiple of 32";
    else if (l.rot_dims < 0 || l.rot_dims > l.dim || l.rot_dims % 2 || (l.rot_dims && !l.inv_freq)) bad = "rotary dims";
    else if (l.kind == SD_MIX_WINDOW_POOL) {
      if (!l.k_cache || !l.v_cache || !l.pk_cache || !l.pv_cache || l.window < 1 || l.pool < 1 || l.vdim > 256)
        bad = "window attention needs caches, window >= 1, pool >= 1, vdim <= 256";
    } else {
      if (l.heads != l.kv_heads || !l.state || l.dim > 256) bad = "a recurrent mixer needs a state, dim <= 256, no grouped heads";
      else if (l.kind == SD_MIX_HEAD_DECAY && !l.head_decay) bad = "decay per head missing";
      else if (l.kind == SD_MIX_CHANNEL_DECAY && (!l.w_a2 || !l.b_a2 || l.rank < 1 || !(l.tau > 0.f))) bad = "channel decay needs its low-rank pair and tau > 0";
    }
    if (bad) {
      sd_set_error("sd_seq_model_create: layer %d: %s", i, bad);
      delete m;
      return nullptr;
    }
  }
  return m;
}

extern "C" void sd_seq_model_destroy(sd_seq_model* m) { delete m; }

extern "C" size_t sd_seq_model_workspace_bytes(const sd_seq_model* m, int max_rows, int max_out, int max_ctx) {
  if (!m || max_rows < 1) return 0;
  // (the split scratch of the window layers exists for small batches only: take the larger plan)
  const size_t a = plan_seq(*m, max_rows, max_out, max_ctx).total;
  const size_t b = plan_seq(*m, max_rows < kAttnSplitRows ? max_rows : kAttnSplitRows, max_out, max_ctx).total;
  return a > b ? a : b;
}

#define SQ_TRY(expr)                \
  do {                              \
    int rc__ = (expr);              \
    if (rc__ != SD_OK) return rc__; \
  } while (0)

namespace {
// One layer normed on its sublayers' outputs: x += norm1(mixer(x)); x += norm2(experts(x)).
// x [R, W] f32 and its bf16 copy hb are current on entry and on return.
int postnorm_layer(const sd_seq_model& m, const sd_seq_layer& l, const sd_seq_batch& b, char* base, const SeqWs& w,
                   sd_stream_t stream) {
  const sd_seq_model_desc& d = m.d;
  const int W = d.width, R = b.n_rows, f32 = d.weights_f32, rnd = !f32;
  const float eps = d.norm_eps;
  float* x = (float*)(base + w.x);
  float* proj = (float*)(base + w.proj);
  float* o = (float*)(base + w.o);
  float* y = (float*)(base + w.y);
  float* mix = (float*)(base + w.mix);
  float* mix2 = (float*)(base + w.ffo);
  bf16_t* hb = (bf16_t*)(base + w.hb);
  bf16_t* yb = (bf16_t*)(base + w.yb);
  void* wide_ws = base + w.wide;
  const PnCols c = pn_cols(l);
  const int64_t ld = c.total;
  const int H = l.heads, dk = l.dim, dv = l.vdim;
  SQ_TRY(seq_linear(l.w_in, l.w_in_tiled, f32, x, nullptr, W, hb, W, nullptr, proj, ld, R, c.total, W, wide_ws,
                    w.wide_bytes, stream));
  if (l.kind == SD_MIX_LATENT) {
    const int qr = l.q_rank, rk = l.kv_rank, dr = l.rot_dim, dh = dk + dr, de = rk + dr;
    float* pq = (float*)(base + w.pq);
    float* qe = (float*)(base + w.qe);
    bf16_t* cqb = (bf16_t*)(base + w.cqb);
    // both latents normed, the shared rotated key part turned, the row [latent | rotated part] cached: one launch
    SQ_TRY(sd_latent_prep(proj + c.dq, qr, l.dq_norm_w, l.w_uq_tiled ? cqb : nullptr, qr, proj + c.dkv, rk, dr,
                          l.dkv_norm_w, ld, f32, eps, l.rot_dims, 1, l.inv_freq, l.rot_mag, l.k_cache, b.row_pos,
                          b.row_slot, b.block_tables, b.max_blocks, b.page, R, stream));
    SQ_TRY(seq_linear(l.w_uq, l.w_uq_tiled, f32, proj + c.dq, nullptr, ld, cqb, qr, nullptr, pq, (int64_t)H * dh, R,
                      H * dh, qr, wide_ws, w.wide_bytes, stream));
    // a head's query against the latent: its key expansion, transposed, applied to the unrotated
    // part; the rotated part is turned into place behind it
    SQ_TRY(sd_matmul_rows_batched(pq, (int64_t)H * dh, dh, l.w_uk_t, f32, (int64_t)rk * dk, qe, (int64_t)H * de, de,
                                  nullptr, R, rk, dk, H, stream));
    if (dr > 0)
      SQ_TRY(sd_rope_copy_rows(pq, (int64_t)H * dh, dh, dk, qe, (int64_t)H * de, de, rk, b.row_pos, R, H, dr,
                               l.rot_dims, 1, l.inv_freq, l.rot_mag, stream));
    SQ_TRY(sd_window_softmax_attention(qe, (int64_t)H * de, l.k_cache, nullptr, f32, b.row_pos, b.row_slot,
                                       b.block_tables, b.max_blocks, b.page, R, H, 1, de, rk, l.window, 0,
                                       l.score_scale, o, nullptr, base + w.attn, w.attn_bytes, stream));
    // a head's value expansion applied to its weighted latent
    SQ_TRY(sd_matmul_rows_batched(o, (int64_t)H * rk, rk, l.w_uv, f32, (int64_t)dv * rk, y, (int64_t)H * dv, dv,
                                  l.w_o_tiled ? yb : nullptr, R, dv, rk, H, stream));
    SQ_TRY(seq_linear(l.w_o, l.w_o_tiled, f32, y, nullptr, (int64_t)H * dv, yb, (int64_t)H * dv, nullptr, mix, W, R, W,
                      H * dv, wide_ws, w.wide_bytes, stream));
    SQ_TRY(sd_postnorm_residual(x, mix, 1, 1.f, nullptr, 0.f, l.norm_w, f32, eps, hb, R, W, stream));
  } else {
    const int G = l.kv_heads;
    // attention: q and k normed over the whole projection, no rotation
    SQ_TRY(sd_qk_norm_append(proj + c.q, H * dk, l.q_norm_w, proj + c.k, G, dk, l.k_norm_w, proj + c.v, dv, ld, f32, eps,
                             l.k_cache, l.v_cache, b.row_pos, b.row_slot, b.block_tables, b.max_blocks, b.page, R,
                             stream));
    SQ_TRY(sd_window_softmax_attention(proj + c.q, ld, l.k_cache, l.v_cache, f32, b.row_pos, b.row_slot,
                                       b.block_tables, b.max_blocks, b.page, R, H, G, dk, dv, l.window, l.keep_first,
                                       l.score_scale, o, l.w_o_tiled ? yb : nullptr, base + w.attn, w.attn_bytes,
                                       stream));
    SQ_TRY(seq_linear(l.w_o, l.w_o_tiled, f32, o, nullptr, (int64_t)H * dv, yb, (int64_t)H * dv, nullptr, mix, W, R, W,
                      H * dv, wide_ws, w.wide_bytes, stream));
    // state-space recurrence: convolution + silu over x, B, C; step sizes; scan; gate, group norm
    float* conv = (float*)(base + w.conv);
    float* step = (float*)(base + w.step);
    float* decay = (float*)(base + w.decay);
    const int Hs = l.s_heads, P = l.s_vdim, N = l.s_state, Gs = l.s_groups, inner = c.inner;
    SQ_TRY(sd_causal_conv_rows(proj + c.xbc, ld, l.conv_w, l.conv_b, f32, l.conv_state, b.row_pos, b.row_slot,
                               b.entries, b.n_entries, conv, c.conv_ch, R, c.conv_ch, l.s_taps, 1, stream));
    SQ_TRY(sd_ssd_steps(proj + c.dt, ld, l.dt_bias, l.a_log, f32, step, decay, R, Hs, stream));
    SQ_TRY(sd_decay_scan_rows(conv + inner + Gs * N, conv + inner, c.conv_ch, conv, c.conv_ch, decay, step, l.skip_d,
                              f32, l.state, b.entries, b.n_entries, o, Hs, Gs, N, P, stream));
    SQ_TRY(sd_rmsnorm_parts(o, inner, proj + c.z, ld, l.s_norm_w, f32, eps, y, inner, l.w_o2_tiled ? yb : nullptr,
                            inner, R, inner, l.s_norm_groups, rnd, stream));
    SQ_TRY(seq_linear(l.w_o2, l.w_o2_tiled, f32, y, nullptr, inner, yb, inner, nullptr, mix2, W, R, W, inner, wide_ws,
                      w.wide_bytes, stream));
    SQ_TRY(sd_postnorm_residual(x, mix, 1, l.left_scale, mix2, l.right_scale, l.norm_w, f32, eps, hb, R, W, stream));
  }
  if (l.n_experts > 0) {
    float* rlog = (float*)(base + w.rlog);
    int32_t* sel_e = (int32_t*)(base + w.sel_e);
    float* sel_w = (float*)(base + w.sel_w);
    float* dn = (float*)(base + w.dn);
    const int E = l.n_experts;
    SQ_TRY(sd_moe_route_rows(x, W, l.w_router, f32, rlog, sel_e, sel_w, R, E, W, l.top, 0, 0, stream));
    SQ_TRY(sd_moe_experts(x, hb, W, sel_e, sel_w, l.w_gate_up, l.w_down_e, f32, dn, R, l.top, E, l.expert_ff, W, 1, 0,
                          base + w.moe, w.moe_bytes, stream));
    SQ_TRY(sd_postnorm_residual(x, dn, l.top, 1.f, nullptr, 0.f, l.norm2_w, f32, eps, hb, R, W, stream));
  }
  return SD_OK;
}

// One layer normed before and after its sublayers: x += post_norm(mixer(norm(x))); x +=
// post_norm2(ff(norm2(x))).  On entry h / hb hold norm(x + pre_add) already (the layer before, or
// the caller, left them); on return they hold the next layer's, or nothing after the last.
int sandwich_layer(const sd_seq_model& m, const sd_seq_layer& l, const sd_seq_layer* next, const sd_seq_batch& b,
                   char* base, const SeqWs& w, float* x_copy, sd_stream_t stream) {
  const sd_seq_model_desc& d = m.d;
  const int W = d.width, R = b.n_rows, f32 = d.weights_f32, rnd = !f32;
  const float eps = d.norm_eps;
  float* x = (float*)(base + w.x);
  float* h = (float*)(base + w.h);
  float* proj = (float*)(base + w.proj);
  float* o = (float*)(base + w.o);
  float* y = (float*)(base + w.y);
  float* mix = (float*)(base + w.mix);
  float* ffo = (float*)(base + w.ffo);
  bf16_t* hb = (bf16_t*)(base + w.hb);
  bf16_t* yb = (bf16_t*)(base + w.yb);
  bf16_t* actb = (bf16_t*)(base + w.actb);
  void* wide_ws = base + w.wide;
  const SwCols c = sw_cols(l);
  const int64_t ld = c.total;
  const int H = l.heads, dk = l.dim, dv = l.vdim;
  const void* next_add = next ? next->pre_add : nullptr;
  const void* next_norm = next ? next->norm_w : nullptr;
  const bool has_ff = l.ff > 0 || l.n_experts > 0;
  SQ_TRY(seq_linear(l.w_in, l.w_in_tiled, f32, h, nullptr, W, hb, W, nullptr, proj, ld, R, c.total, W, wide_ws,
                    w.wide_bytes, stream));
  if (l.kind == SD_MIX_LATENT) {
    const int rk = l.kv_rank, dr = l.rot_dim, dh = dk + dr, de = rk + dr;
    float* qe = (float*)(base + w.qe);
    // the latent normed, the shared rotated key part turned, the row [latent | rotated part] cached
    SQ_TRY(sd_latent_prep(nullptr, 0, nullptr, nullptr, 0, proj + c.dkv, rk, dr, l.dkv_norm_w, ld, f32, eps, l.rot_dims,
                          l.rot_layout, l.inv_freq, l.rot_mag, l.k_cache, b.row_pos, b.row_slot, b.block_tables,
                          b.max_blocks, b.page, R, stream));
    // a head's query against the latent: its key expansion, transposed, applied to the unrotated
    // part; the rotated part is turned into place behind it
    SQ_TRY(sd_matmul_rows_batched(proj + c.q, ld, dh, l.w_uk_t, f32, (int64_t)rk * dk, qe, (int64_t)H * de, de, nullptr,
                                  R, rk, dk, H, stream));
    if (dr > 0)
      SQ_TRY(sd_rope_copy_rows(proj + c.q, ld, dh, dk, qe, (int64_t)H * de, de, rk, b.row_pos, R, H, dr, l.rot_dims,
                               l.rot_layout, l.inv_freq, l.rot_mag, stream));
    SQ_TRY(sd_masked_softmax_attention(qe, (int64_t)H * de, l.k_cache, nullptr, f32, b.row_pos, b.row_slot,
                                       b.block_tables, b.max_blocks, b.page, R, H, 1, de, rk, l.window, 0, l.chunk,
                                       l.score_scale, l.softcap, l.sinks, o, nullptr, base + w.attn, w.attn_bytes,
                                       stream));
    // a head's value expansion applied to its weighted latent, then the head's gate
    bf16_t* y_b = l.w_o_tiled ? yb : nullptr;
    SQ_TRY(sd_matmul_rows_batched(o, (int64_t)H * rk, rk, l.w_uv, f32, (int64_t)dv * rk, y, (int64_t)H * dv, dv,
                                  l.head_gate ? nullptr : y_b, R, dv, rk, H, stream));
    if (l.head_gate)
      SQ_TRY(sd_head_gate_rows(y, (int64_t)H * dv, proj + c.g, ld, y_b, (int64_t)H * dv, R, H, dv, rnd, stream));
    SQ_TRY(seq_linear(l.w_o, l.w_o_tiled, f32, y, nullptr, (int64_t)H * dv, yb, (int64_t)H * dv, nullptr, mix, W, R, W,
                      H * dv, wide_ws, w.wide_bytes, stream));
  } else {
    const int G = l.kv_heads, maps = l.maps > 1 ? l.maps : 1;
    if (general_prep(l)) {
      // biases, norms, rotary turn, and the append of keys and values (unless another layer's are read): one launch
      const char* bias = (const char*)l.w_in_bias;
      const size_t es = f32 ? sizeof(float) : sizeof(bf16_t);
      SQ_TRY(sd_attn_prep(proj + c.q, H * maps, l.kv_shared ? nullptr : proj + c.k, G * maps, dk,
                          l.kv_shared || l.value_from_key ? nullptr : proj + c.v, G, dv, l.value_from_key, ld,
                          bias ? bias + (size_t)c.q * es : nullptr, bias && !l.kv_shared ? bias + (size_t)c.k * es : nullptr,
                          l.qk_full_norm ? 1 : (l.qk_head_norm ? 2 : 0), l.q_norm_w, l.k_norm_w, f32, eps, l.rot_dims,
                          l.rot_layout, l.inv_freq, l.rot_mag != 0.f ? l.rot_mag : 1.f, l.k_cache, l.v_cache, b.row_pos,
                          b.row_slot, b.block_tables, b.max_blocks, b.page, R, stream));
    } else {
      SQ_TRY(sd_qk_head_norm_append(proj + c.q, H, l.q_norm_w, proj + c.k, G, dk, l.k_norm_w, proj + c.v, dv, ld, f32,
                                    eps, l.k_cache, l.v_cache, b.row_pos, b.row_slot, b.block_tables, b.max_blocks,
                                    b.page, R, stream));
    }
    bf16_t* y_b = l.w_o_tiled ? yb : nullptr;
    SQ_TRY(sd_multimap_softmax_attention(proj + c.q, ld, l.k_cache, l.v_cache, f32, b.row_pos, b.row_slot,
                                         b.block_tables, b.max_blocks, b.page, R, H, G, maps, dk, dv, l.window, 0,
                                         l.chunk, l.score_scale, l.softcap, l.sinks, o, maps > 1 ? nullptr : y_b,
                                         base + w.attn, w.attn_bytes, stream));
    const float* heads_out = o;
    if (maps > 1) {   // the two maps of a head put together, the head's difference normed
      SQ_TRY(sd_diff_combine_rows(o, l.diff_lambda, eps, l.diff_scale, y, y_b, R, H, dv, rnd, stream));
      heads_out = y;
    }
    SQ_TRY(seq_linear(l.w_o, l.w_o_tiled, f32, heads_out, nullptr, (int64_t)H * dv, yb, (int64_t)H * dv, nullptr, mix, W,
                      R, W, H * dv, wide_ws, w.wide_bytes, stream));
  }
  const float mult = l.residual_mult != 0.f ? l.residual_mult : 1.f;
  if (!has_ff)
    return sd_residual_norm_scaled(x, mix, 1, l.w_o_bias, nullptr, nullptr, 0, l.post_norm_w, mult, next_add, next_norm,
                                   f32, eps, x_copy, h, hb, R, W, stream);
  SQ_TRY(sd_residual_norm_scaled(x, mix, 1, l.w_o_bias, nullptr, nullptr, 0, l.post_norm_w, mult, nullptr, l.norm2_w,
                                 f32, eps, nullptr, h, hb, R, W, stream));
  if (l.ff > 0) {
    const int F = l.ff, n_in = act_inputs(l.ff_act);
    SQ_TRY(seq_linear(l.w_ff_in, l.w_ff_in_tiled, f32, h, nullptr, W, hb, W, nullptr, proj, (int64_t)n_in * F, R,
                      n_in * F, W, wide_ws, w.wide_bytes, stream));
    SQ_TRY(sd_act_rows(proj, n_in > 1 ? proj + F : nullptr, (int64_t)n_in * F, proj, (int64_t)n_in * F,
                       l.w_down_tiled ? actb : nullptr, F, R, F, l.ff_act, rnd, stream));
    SQ_TRY(seq_linear(l.w_down, l.w_down_tiled, f32, proj, nullptr, (int64_t)n_in * F, actb, F, nullptr, ffo, W, R, W,
                      F, wide_ws, w.wide_bytes, stream));
    return sd_residual_norm_scaled(x, ffo, 1, nullptr, nullptr, nullptr, 0, l.post_norm2_w, mult, next_add, next_norm,
                                   f32, eps, x_copy, h, hb, R, W, stream);
  }
  float* rlog = (float*)(base + w.rlog);
  int32_t* sel_e = (int32_t*)(base + w.sel_e);
  float* sel_w = (float*)(base + w.sel_w);
  float* dn = (float*)(base + w.dn);
  float* sg = (float*)(base + w.sg);
  const bool gated_shared = l.shared_ff > 0 && l.w_shared_gate;
  SQ_TRY(sd_moe_route_rows_biased(h, W, l.w_router, l.router_bias, f32, rlog, sel_e, sel_w, R, l.n_experts, W, l.top,
                                  l.route_score, l.route_renorm, l.route_renorm_eps,
                                  l.route_scale != 0.f ? l.route_scale : 1.f, gated_shared ? l.w_shared_gate : nullptr,
                                  gated_shared ? 1 : 0, sg, stream));
  SQ_TRY(sd_moe_experts(h, hb, W, sel_e, sel_w, l.w_gate_up, l.w_down_e, f32, dn, R, l.top, l.n_experts, l.expert_ff, W,
                        l.expert_scale_input, l.expert_act, base + w.moe, w.moe_bytes, stream));
  if (l.shared_ff > 0) {
    const int F = l.shared_ff, n_in = act_inputs(l.shared_act);
    SQ_TRY(seq_linear(l.w_shared_in, l.w_shared_in_tiled, f32, h, nullptr, W, hb, W, nullptr, proj, (int64_t)n_in * F,
                      R, n_in * F, W, wide_ws, w.wide_bytes, stream));
    SQ_TRY(sd_act_rows(proj, n_in > 1 ? proj + F : nullptr, (int64_t)n_in * F, proj, (int64_t)n_in * F,
                       l.w_shared_down_tiled ? actb : nullptr, F, R, F, l.shared_act, rnd, stream));
    SQ_TRY(seq_linear(l.w_shared_down, l.w_shared_down_tiled, f32, proj, nullptr, (int64_t)n_in * F, actb, F, nullptr,
                      ffo, W, R, W, F, wide_ws, w.wide_bytes, stream));
  }
  return sd_residual_norm_scaled(x, dn, l.top, nullptr, l.shared_ff > 0 ? ffo : nullptr, gated_shared ? sg : nullptr, 1,
                                 l.post_norm2_w, mult, next_add, next_norm, f32, eps, x_copy, h, hb, R, W, stream);
}
}  // namespace

extern "C" int sd_seq_model_forward(sd_seq_model* m, const sd_seq_batch* b, void* workspace,
                                    size_t workspace_bytes, sd_stream_t stream) {
  SD_REQUIRE(m && b && workspace, SD_ERR_INVALID, "sd_seq_model_forward: null argument");
  SD_REQUIRE(b->n_rows >= 1 && b->n_entries >= 1 && b->tokens && b->row_pos && b->row_slot && b->entries,
             SD_ERR_INVALID, "sd_seq_model_forward: empty batch or null array");
  SD_REQUIRE(b->n_out >= 0 && (b->n_out == 0 || (b->out_rows && b->logits)), SD_ERR_INVALID,
             "sd_seq_model_forward: wanted rows need out_rows and logits");
  const SeqWs w = plan_seq(*m, b->n_rows, b->n_out, b->max_blocks * b->page);
  SD_REQUIRE(workspace_bytes >= w.total, SD_ERR_WORKSPACE, "sd_seq_model_forward: workspace %zu < %zu bytes",
             workspace_bytes, w.total);
  SD_REQUIRE(sd_aligned16(workspace), SD_ERR_INVALID, "sd_seq_model_forward: workspace unaligned");
  const sd_seq_model_desc& d = m->d;
  const int W = d.width, R = b->n_rows, f32 = d.weights_f32, rnd = !f32;
  hipStream_t st = (hipStream_t)stream;
  char* base = (char*)workspace;
  float* x = (float*)(base + w.x);
  float* h = (float*)(base + w.h);
  float* proj = (float*)(base + w.proj);
  float* dec = (float*)(base + w.dec);
  float* o = (float*)(base + w.o);
  float* y = (float*)(base + w.y);
  float* mix = (float*)(base + w.mix);
  float* ffo = (float*)(base + w.ffo);
  float* hout = (float*)(base + w.hout);

  bf16_t* hb = (bf16_t*)(base + w.hb);
  bf16_t* yb = (bf16_t*)(base + w.yb);
  bf16_t* actb = (bf16_t*)(base + w.actb);
  bf16_t* houtb = (bf16_t*)(base + w.houtb);
  void* wide_ws = base + w.wide;

  const bool hashed = d.bigram || (d.embed_scale != 0.f && d.embed_scale != 1.f) || m->layers[0].block != SD_BLOCK_GATED;
  if (hashed) {
    SD_REQUIRE(!d.bigram || b->prev_tokens, SD_ERR_INVALID, "sd_seq_model_forward: a bigram table needs prev_tokens");
    SQ_TRY(sd_embed_hashed(b->tokens, b->prev_tokens, d.embed, d.bigram, f32, d.embed_scale != 0.f ? d.embed_scale : 1.f,
                           d.buckets, d.mul_prev, d.mul_cur, x, hb, R, W, d.vocab, stream));
  } else {
    if (f32) embed_rows_kernel<float><<<R, 256, 0, st>>>(b->tokens, (const float*)d.embed, x, W, d.vocab);
    else embed_rows_kernel<bf16_t><<<R, 256, 0, st>>>(b->tokens, (const bf16_t*)d.embed, x, W, d.vocab);
    SD_CHECK_LAUNCH("sd_seq_model_forward (embed)");
  }

  for (int li = 0; li < d.n_layers; ++li) {
    const sd_seq_layer& l = m->layers[li];
    if (l.block == SD_BLOCK_SANDWICH) {
      if (li == 0)   // the first layer's input: what is added before it, then its norm
        SQ_TRY(sd_residual_norm(x, nullptr, 0, nullptr, nullptr, 0, nullptr, l.pre_add, l.norm_w, f32, d.norm_eps,
                                nullptr, h, hb, R, W, stream));
      SQ_TRY(sandwich_layer(*m, l, li + 1 < d.n_layers ? &m->layers[li + 1] : nullptr, *b, base, w,
                            b->layer_out ? b->layer_out + (size_t)li * R * W : nullptr, stream));
      continue;
    }
    if (l.block == SD_BLOCK_POSTNORM) {
      SQ_TRY(postnorm_layer(*m, l, *b, base, w, stream));
      if (b->layer_out) {
        const hipError_t e = hipMemcpyAsync(b->layer_out + (size_t)li * R * W, x, (size_t)R * W * sizeof(float),
                                            hipMemcpyDeviceToDevice, st);
        SD_REQUIRE(e == hipSuccess, SD_ERR_HIP, "sd_seq_model_forward: copying a layer's output: %s",
                   hipGetErrorString(e));
      }
      continue;
    }
    SD_REQUIRE(li == 0 || m->layers[li - 1].block == SD_BLOCK_GATED, SD_ERR_UNSUPPORTED,
               "sd_seq_model_forward: a gated layer after a layer normed on its output is not provided");
    const InCols c = in_cols(l, W);
    const int64_t ld = c.total;
    const int H = l.heads, G = l.kv_heads, dk = l.dim, dv = l.vdim;
    // (layers after the first find their normed input ready: the residual update of the layer
    // before wrote it)
    if (li == 0)
      SQ_TRY(sd_rmsnorm_rows(x, nullptr, l.norm_w, f32, 1.f, d.norm_eps, h, l.w_in_tiled ? hb : nullptr, R, W, stream));
    // every matrix that reads h, in one product: q k v g | residual gates | ff gate, up | low-rank decay
    SQ_TRY(seq_linear(l.w_in, l.w_in_tiled, f32, h, nullptr, W, hb, W, nullptr, proj, ld, R, c.total, W, wide_ws,
                      w.wide_bytes, stream));
    bf16_t* y_b = l.w_o_tiled ? yb : nullptr;
    if (l.kind == SD_MIX_WINDOW_POOL) {
      SQ_TRY(sd_head_prep(proj + c.q, proj + c.k, proj + c.v, ld, b->row_pos, b->row_slot, R, H, G, dk, dv,
                          l.rot_dims, l.rot_layout, l.inv_freq, l.qk_unit_norm, d.norm_eps, l.q_scale, l.k_scale,
                          l.k_cache, l.v_cache, f32, b->block_tables, b->max_blocks, b->page, stream));
      SQ_TRY(sd_window_pool_attention(proj + c.q, ld, l.k_cache, l.v_cache, f32, l.pk_cache, l.pv_cache,
                                      b->row_pos, b->row_slot, b->block_tables, b->max_blocks, b->page, R, H, G,
                                      dk, dv, l.window, l.pool, l.score_scale, l.head_bias, o, base + w.attn,
                                      w.attn_bytes, stream));
      SQ_TRY(sd_head_post(o, proj + c.g, ld, nullptr, f32, 0, d.norm_eps, 1, y, y_b, R, H, dv, rnd, stream));
    } else {
      SQ_TRY(sd_head_prep(proj + c.q, proj + c.k, nullptr, ld, b->row_pos, b->row_slot, R, H, H, dk, dv,
                          l.rot_dims, l.rot_layout, l.inv_freq, l.qk_unit_norm, d.norm_eps, l.q_scale, l.k_scale,
                          nullptr, nullptr, f32, nullptr, 0, 0, stream));
      const bool pc = l.kind == SD_MIX_CHANNEL_DECAY;
      if (pc) {
        // decay logits through the low-rank pair (its first half came out of the fused product)
        float* z = o;  // free until the scan writes it; the scan reads `dec`
        SQ_TRY(sd_matmul_rows(proj + c.a1, nullptr, ld, l.w_a2, f32, l.b_a2, z, (int64_t)H * dk, R, H * dk, l.rank, stream));
        SQ_TRY(sd_sigmoid_power(z, (int64_t)H * dk, l.tau, dec, R, H * dk, stream));
      }
      SQ_TRY(sd_decay_scan(proj + c.q, proj + c.k, proj + c.v, ld, pc ? dec : l.head_decay, pc, l.state,
                           b->entries, b->n_entries, o, H, dk, dv, stream));
      SQ_TRY(sd_head_post(o, proj + c.g, ld, l.head_norm_w, f32, 1, d.norm_eps, 0, y, y_b, R, H, dv, rnd, stream));
    }
    SQ_TRY(seq_linear(l.w_o, l.w_o_tiled, f32, y, nullptr, (int64_t)H * dv, yb, (int64_t)H * dv, nullptr, mix, W, R,
                      W, H * dv, wide_ws, w.wide_bytes, stream));
    if (l.ff > 0) {
      if (l.w_down_tiled) SQ_TRY(sd_relu_mul_rows(proj + c.gate, proj + c.up, ld, actb, R, l.ff, stream));
      SQ_TRY(seq_linear(l.w_down, l.w_down_tiled, f32, proj + c.gate, proj + c.up, ld, actb, l.ff, nullptr, ffo, W,
                        R, W, l.ff, wide_ws, w.wide_bytes, stream));
    }
    if (li + 1 < d.n_layers) {
      const sd_seq_layer& nx = m->layers[li + 1];
      SQ_TRY(sd_gated_residual_norm(x, proj + c.r1, l.ff > 0 ? proj + c.r2 : nullptr, ld, l.r1_bias,
                                    l.ff > 0 ? l.r2_bias : nullptr, mix, l.ff > 0 ? ffo : nullptr, R, W, nx.norm_w,
                                    f32, 1.f, d.norm_eps, h, nx.w_in_tiled ? hb : nullptr, stream));
    } else {
      SQ_TRY(sd_gated_residual(x, proj + c.r1, l.ff > 0 ? proj + c.r2 : nullptr, ld, l.r1_bias,
                               l.ff > 0 ? l.r2_bias : nullptr, mix, l.ff > 0 ? ffo : nullptr, R, W, stream));
    }
    if (b->layer_out) {
      const hipError_t e = hipMemcpyAsync(b->layer_out + (size_t)li * R * W, x, (size_t)R * W * sizeof(float),
                                          hipMemcpyDeviceToDevice, st);
      SD_REQUIRE(e == hipSuccess, SD_ERR_HIP, "sd_seq_model_forward: copying a layer's output: %s",
                 hipGetErrorString(e));
    }
  }
  if (b->n_out > 0) {
    SQ_TRY(sd_rmsnorm_rows(x, b->out_rows, d.final_norm_w, f32, d.plain_norm ? 0.f : 1.f, d.norm_eps, hout,
                           d.head_tiled ? houtb : nullptr, b->n_out, W, stream));
    SQ_TRY(seq_linear(d.head ? d.head : d.embed, d.head_tiled, f32, hout, nullptr, W, houtb, W, nullptr, b->logits,
                      d.vocab, b->n_out, d.vocab, W, wide_ws, w.wide_bytes, stream));
    if (d.logit_scale != 0.f && d.logit_scale != 1.f)
      SQ_TRY(sd_scale_rows(b->logits, d.vocab, d.logit_scale, b->n_out, d.vocab, stream));
  }
  return SD_OK;
}
