// Attention over a window of a paged cache with what some designs add to it: queries and keys normed before they are turned,
// one mean key and value per block of tokens behind the window, a learned bias by distance, a sink in the denominator.
//
//   norm_turn_write   what a step's projections become before attention: every query and key head is divided by a root mean
//                     square (its own, or that of the whole projection of its row) and multiplied by a weight, then turned by
//                     its row's position (pairs (i, i + n/2), angles from a table); keys and values go to their rows' cache
//                     slots; a design whose values are its keys as projected gets them written before the norm.
//   pool_blocks       rows that complete a block of P tokens leave the mean of the block's keys and the mean of its values, as
//                     the pages hold them, in pages of their own (one place per P tokens of a page).
//   span_attention    the always-valid kernel, a wavefront per (row, head): softmax over the tokens of the window and the
//                     blocks wholly behind it, scores plus a bias by distance, exp(sink) in the denominator, a sigmoid gate
//                     per channel or per head.
//
// Cache layout (that of the other attention kernels): keys [page, kv_head, slot, d], values transposed [page, kv_head, dv, slot].
// Pooled: keys [page, kv_head, place, d], values [page, kv_head, dv, place], block b at page table[(b P) / S], place ((b P) % S) / P.
//
// Arithmetic: products and sums in Acc (float; double in the exact path), in ascending key order per output channel, so a
// row's result depends on the keys it sees and on nothing else: not on how rows were cut into steps, on the batch or on pages.
#include "common.h"

#include <float.h>

namespace alofa {

enum NormScope : int { kNormNone = 0, kNormHead = 1, kNormAll = 2 };

// 1 / sqrt(mean(x^2) + eps) over the whole query projection and over the whole key projection of every row: inv[t][0], inv[t][1].
// The mean is taken over q_count and k_count channels (heads that were widened with zeros hold fewer than their width).
template <typename T, typename Acc>
__global__ void __launch_bounds__(256) projection_inv_rms_kernel(double* __restrict__ inv, const T* __restrict__ qkv, int64_t stride, int tokens, int q_width, int k_width, int q_count, int k_count, float eps) {
  __shared__ Acc scratch[4];
  const int unit = blockIdx.x;      // (a block per row and projection)
  const int t = unit / 2, which = unit % 2;
  const T* x = qkv + static_cast<int64_t>(t) * stride + (which ? q_width : 0);
  const int n = which ? k_width : q_width;
  Acc ss = 0;
  for (int c = threadIdx.x; c < n; c += 256) {
    const Acc v = static_cast<Acc>(load_f32(x + c));
    ss += v * v;
  }
  ss = block_sum<Acc, 256>(ss, scratch);
  if (threadIdx.x == 0) inv[unit] = static_cast<double>(static_cast<Acc>(1) / sqrt(ss / static_cast<Acc>(which ? k_count : q_count) + static_cast<Acc>(eps)));
}

// One wavefront per (row, unit): query heads first, then key heads, then (unless the values are the keys) value heads.
template <typename T, typename Acc>
__global__ void __launch_bounds__(256) norm_turn_write_kernel(T* __restrict__ qkv, int64_t stride, const int32_t* __restrict__ positions,
                                                              const float* __restrict__ cos_t, const float* __restrict__ sin_t, int half,
                                                              int scope, const float* __restrict__ wq, const float* __restrict__ wk, float eps, const double* __restrict__ row_inv,
                                                              const int64_t* __restrict__ slots, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                                              int block_size, int tokens, int heads, int kv_heads, int d, int dv, int d_true, int values_are_keys) {
  const int per_row = heads + kv_heads + (values_are_keys ? 0 : kv_heads);
  const int64_t unit = static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / kWave;
  if (unit >= static_cast<int64_t>(tokens) * per_row) return;
  const int lane = threadIdx.x % kWave;
  const int t = static_cast<int>(unit / per_row), u = static_cast<int>(unit % per_row);
  T* row = qkv + static_cast<int64_t>(t) * stride;
  const int64_t slot = kv_heads ? slots[t] : 0;
  if (u >= heads + kv_heads) {      // a value head: copied to its page as projected
    const int g = u - heads - kv_heads;
    const T* src = row + static_cast<int64_t>(heads + kv_heads) * d + static_cast<int64_t>(g) * dv;
    T* dst = v_cache + ((slot / block_size) * kv_heads + g) * static_cast<int64_t>(dv) * block_size + slot % block_size;
    for (int c = lane; c < dv; c += kWave) dst[static_cast<int64_t>(c) * block_size] = src[c];
    return;
  }
  const bool is_k = u >= heads;
  const int local = is_k ? u - heads : u;
  T* src = row + static_cast<int64_t>(u) * d;
  const float* w = is_k ? wk : wq;
  constexpr int kOwn = 4;      // heads up to 256 channels
  float x[kOwn];
  Acc ss = 0;
#pragma unroll
  for (int n = 0; n < kOwn; ++n) {
    const int c = lane + n * kWave;
    x[n] = c < d ? load_f32(src + c) : 0.f;
    ss += static_cast<Acc>(x[n]) * static_cast<Acc>(x[n]);
  }
  if (is_k && values_are_keys) {
    T* dst = v_cache + ((slot / block_size) * kv_heads + local) * static_cast<int64_t>(d) * block_size + slot % block_size;
#pragma unroll
    for (int n = 0; n < kOwn; ++n) {
      const int c = lane + n * kWave;
      if (c < d) store_f32(dst + static_cast<int64_t>(c) * block_size, x[n]);
    }
  }
  if (scope != kNormNone) {
    Acc inv;
    if (scope == kNormAll) {      // the whole projection of the row: its factor was made beforehand (the heads are written back in place meanwhile)
      inv = static_cast<Acc>(row_inv[2 * static_cast<int64_t>(t) + (is_k ? 1 : 0)]);
      w = w ? w + static_cast<int64_t>(local) * d : nullptr;
    } else {
      ss = wave_sum(ss);
      inv = static_cast<Acc>(1) / sqrt(ss / static_cast<Acc>(d_true) + static_cast<Acc>(eps));
    }
#pragma unroll
    for (int n = 0; n < kOwn; ++n) {
      const int c = lane + n * kWave;
      if (c < d) x[n] = static_cast<float>(static_cast<Acc>(x[n]) * inv * static_cast<Acc>(w ? w[c] : 1.f));
    }
  }
  // the turn: pair (i, i + half); a lane finds its partner's value in a small staging area of its wavefront
  __shared__ float stage[4][256];
  float* mine = stage[threadIdx.x / kWave];
#pragma unroll
  for (int n = 0; n < kOwn; ++n) {
    const int c = lane + n * kWave;
    if (c < d) mine[c] = x[n];
  }
  wave_lds_sync();
  T* dst = src;
  if (is_k) dst = k_cache + (((slot / block_size) * kv_heads + local) * block_size + slot % block_size) * static_cast<int64_t>(d);
  const int p = positions[t];
#pragma unroll
  for (int n = 0; n < kOwn; ++n) {
    const int c = lane + n * kWave;
    if (c >= d) continue;
    float y = x[n];
    if (cos_t != nullptr && c < 2 * half) {
      const int i = c < half ? c : c - half;
      const float cs = cos_t[static_cast<int64_t>(p) * half + i], sn = sin_t[static_cast<int64_t>(p) * half + i];
      const float a = mine[i], b = mine[i + half];
      y = c < half ? a * cs - b * sn : b * cs + a * sn;
    }
    store_f32(dst + c, y);
  }
}

// A block per (row, kv head); rows that do not end a block of P tokens leave at once.
template <typename T, typename Acc>
__global__ void __launch_bounds__(128) pool_blocks_kernel(const T* __restrict__ k_cache, const T* __restrict__ v_cache, T* __restrict__ pk, T* __restrict__ pv,
                                                          const int32_t* __restrict__ table, int max_blocks, const int32_t* __restrict__ pool_table, int pool_max_blocks,
                                                          const int32_t* __restrict__ req_of_token, const int32_t* __restrict__ positions,
                                                          int kv_heads, int d, int dv, int block_size, int P, int places) {
  const int t = blockIdx.x, g = blockIdx.y;
  const int p = positions[t];
  if ((p + 1) % P != 0) return;
  const int r = req_of_token ? req_of_token[t] : t;
  const int32_t* tab = table + static_cast<int64_t>(r) * max_blocks;
  const int first = p + 1 - P;
  const int64_t page = pool_table[static_cast<int64_t>(r) * pool_max_blocks + first / block_size];
  const int place = (first % block_size) / P;
  for (int c = threadIdx.x; c < d + dv; c += 128) {
    Acc acc = 0;
    for (int j = first; j <= p; ++j) {
      const int64_t blk = tab[j / block_size];
      const int s = j % block_size;
      acc += c < d ? static_cast<Acc>(load_f32(k_cache + ((blk * kv_heads + g) * block_size + s) * static_cast<int64_t>(d) + c))
                   : static_cast<Acc>(load_f32(v_cache + ((blk * kv_heads + g) * static_cast<int64_t>(dv) + (c - d)) * block_size + s));
    }
    const float mean = static_cast<float>(acc / static_cast<Acc>(P));
    if (c < d) store_f32(pk + ((page * kv_heads + g) * places + place) * static_cast<int64_t>(d) + c, mean);
    else store_f32(pv + ((page * kv_heads + g) * static_cast<int64_t>(dv) + (c - d)) * places + place, mean);
  }
}

// ---- the always-valid attention kernel: a wavefront per (row, head) ------------------------------------------
struct SpanArgs {
  int64_t out_stride, q_stride, gate_stride;
  const int32_t* table;        // the pages of the window's tokens
  int max_blocks;
  const int32_t* pool_table;   // the pages of the pooled blocks (nullptr: none)
  int pool_max_blocks;
  const int32_t* req_of_token;
  const int32_t* positions;
  int tokens, heads, kv_heads, d, dv, block_size, window, P, places;
  float scale;
  const float* bias;           // [heads, bias_len] by distance, the last entry for every distance beyond (nullptr: none)
  int bias_len;
  const float* sink;           // [heads] (nullptr: none)
  int gate_kind;               // 0 none, 1 a gate per channel [T, heads * dv], 2 a gate per head [T, heads]
};

template <typename T, typename Acc>
__global__ void __launch_bounds__(256) span_attention_kernel(T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                                                             const T* __restrict__ pk, const T* __restrict__ pv, const T* __restrict__ gate, SpanArgs a) {
  __shared__ float qs[4][256];
  __shared__ float ws[4][kWave];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int64_t unit = static_cast<int64_t>(blockIdx.x) * 4 + wave;
  if (unit >= static_cast<int64_t>(a.tokens) * a.heads) return;
  const int t = static_cast<int>(unit / a.heads), h = static_cast<int>(unit % a.heads);
  const int g = h / (a.heads / a.kv_heads);
  const int d = a.d, dv = a.dv, S = a.block_size;
  const int p = a.positions[t];
  const int r = a.req_of_token ? a.req_of_token[t] : t;
  const int lo = (a.window > 0 && p - a.window + 1 > 0) ? p - a.window + 1 : 0;
  const int n_tok = p - lo + 1;
  const int n_blk = (a.pool_table != nullptr && a.window > 0 && p - a.window + 1 >= a.P) ? (p - a.window + 1) / a.P : 0;
  const int n_all = n_tok + n_blk;
  const int32_t* tab = a.table + static_cast<int64_t>(r) * a.max_blocks;
  const int32_t* ptab = a.pool_table ? a.pool_table + static_cast<int64_t>(r) * a.pool_max_blocks : nullptr;
  float* myq = qs[wave];
  for (int c = lane; c < d; c += kWave) myq[c] = load_f32(q + static_cast<int64_t>(t) * a.q_stride + static_cast<int64_t>(h) * d + c);
  wave_lds_sync();

  // entry e of the row's list: the window's tokens in ascending order, then the blocks behind it in ascending order
  auto score = [&](int e) -> Acc {
    const T* k;
    Acc b = 0;
    if (e < n_tok) {
      const int j = lo + e;
      k = k_cache + ((static_cast<int64_t>(tab[j / S]) * a.kv_heads + g) * S + j % S) * static_cast<int64_t>(d);
      if (a.bias) {
        const int dist = p - j;
        b = static_cast<Acc>(a.bias[static_cast<int64_t>(h) * a.bias_len + (dist < a.bias_len ? dist : a.bias_len - 1)]);
      }
    } else {
      const int first = (e - n_tok) * a.P;
      k = pk + ((static_cast<int64_t>(ptab[first / S]) * a.kv_heads + g) * a.places + (first % S) / a.P) * static_cast<int64_t>(d);
    }
    Acc acc = 0;
    for (int c = 0; c < d; ++c) acc += static_cast<Acc>(myq[c]) * static_cast<Acc>(load_f32(k + c));
    return acc * static_cast<Acc>(a.scale) + b;
  };

  Acc m = -DBL_MAX, l = 0;
  bool any = false;
  for (int e = lane; e < n_all; e += kWave) {
    const Acc s = score(e);
    if (!any || s > m) {
      l = any ? l * exp(m - s) : static_cast<Acc>(0);
      m = s;
      any = true;
    }
    l += exp(s - m);
  }
  float top = wave_max(any ? static_cast<float>(m) : -FLT_MAX);      // (any float at least as large as every score, up to rounding, serves)
  if (a.sink) top = fmaxf(top, a.sink[h]);
  const Acc top_acc = static_cast<Acc>(top);
  Acc total = wave_sum(any ? l * exp(m - top_acc) : static_cast<Acc>(0));
  if (a.sink) total += exp(static_cast<Acc>(a.sink[h]) - top_acc);

  constexpr int kOwn = 4;
  Acc acc[kOwn];
#pragma unroll
  for (int n = 0; n < kOwn; ++n) acc[n] = 0;
  for (int e0 = 0; e0 < n_all; e0 += kWave) {
    const int e = e0 + lane;
    ws[wave][lane] = e < n_all ? static_cast<float>(exp(score(e) - top_acc) / total) : 0.f;
    wave_lds_sync();
    const int n = n_all - e0 < kWave ? n_all - e0 : kWave;
    for (int i = 0; i < n; ++i) {
      const int ee = e0 + i;
      const T* v;
      int64_t step;
      if (ee < n_tok) {
        const int j = lo + ee;
        v = v_cache + (static_cast<int64_t>(tab[j / S]) * a.kv_heads + g) * static_cast<int64_t>(dv) * S + j % S;
        step = S;
      } else {
        const int first = (ee - n_tok) * a.P;
        v = pv + (static_cast<int64_t>(ptab[first / S]) * a.kv_heads + g) * static_cast<int64_t>(dv) * a.places + (first % S) / a.P;
        step = a.places;
      }
      const Acc w = static_cast<Acc>(ws[wave][i]);
#pragma unroll
      for (int n2 = 0; n2 < kOwn; ++n2) {
        const int c = lane + n2 * kWave;
        if (c < dv) acc[n2] += w * static_cast<Acc>(load_f32(v + c * step));
      }
    }
    wave_lds_sync();
  }
#pragma unroll
  for (int n = 0; n < kOwn; ++n) {
    const int c = lane + n * kWave;
    if (c >= dv) continue;
    Acc y = acc[n];
    if (a.gate_kind != 0) {
      const int64_t at = a.gate_kind == 1 ? static_cast<int64_t>(h) * dv + c : h;
      const Acc z = static_cast<Acc>(load_f32(gate + static_cast<int64_t>(t) * a.gate_stride + at));
      y = y / (static_cast<Acc>(1) + exp(-z));
    }
    store_f32(out + static_cast<int64_t>(t) * a.out_stride + static_cast<int64_t>(h) * dv + c, static_cast<float>(y));
  }
}

// ---- the matrix-core kernel: a wavefront, or a block of wavefronts, per (16 rows of one request, head), bfloat16
// Where a block's wavefronts share a head they take the tiles of keys in turn (a row's chain of dependent tiles is as many times shorter) and
// their running states meet in LDS at the end, combined in wavefront order.
// Both products are taken transposed (v_mfma_f32_16x16x32_bf16; lane l: A row and B column l % 16, reduction slots 8 (l / 16) .. + 7,
// D column l % 16 and rows 4 (l / 16) .. + 3), so a lane stays with one query row throughout:
//   S^T[key, q] = K[key, :] . Q[q, :]       A = keys straight from the pages (16 bytes a lane), B = queries (registers)
//   O^T[c, q] += V^T[c, key] * P^T[key, q]   A = transposed values straight from the pages (two runs of four keys a lane), B = weights
// Keys are walked in tiles of 32 that start at multiples of 32: after the first product lane l holds, for query l % 16, the scores of
// keys 4 g + r and 16 + 4 g + r (g = l / 16, r = 0..3), which are the eight reduction slots of the second product when the values are read
// in that order, so the weights never leave their registers. The four lanes of a query meet for the tile's maximum; the running
// maximum, the weights' sum and the scores are float. Then the blocks behind the window, 32 at a time, the same way (their places
// are looked up one by one). The sink joins the denominator at the end; the gate rides on the store. Every weight enters the second
// product as two bfloat16 numbers (sixteen bits of it count).
typedef __bf16 span_bf16x8 __attribute__((ext_vector_type(8)));
typedef float span_f32x4 __attribute__((ext_vector_type(4)));

struct SpanFastArgs {
  int64_t out_stride, q_stride, gate_stride;
  const int32_t* tiles;        // [n_tiles, 3]: request, first row, rows (<= 16); nullptr: tile t is row t alone, of request req_of_token[t] (or t)
  const int32_t* table;
  int max_blocks;
  const int32_t* pool_table;
  int pool_max_blocks;
  const int32_t* req_of_token;
  const int32_t* positions;
  int n_tiles, heads, kv_heads, bs_shift, window, P, places, dv_true;
  float scale;
  const float* bias;
  int bias_len;
  const float* sink;
  int gate_kind;
};

template <int DT, int NW, bool kDeal>
__global__ void __launch_bounds__(64 * NW) span_attention_mfma_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache,
                                                                  const bf16_t* __restrict__ v_cache, const bf16_t* __restrict__ pk, const bf16_t* __restrict__ pv,
                                                                  const bf16_t* __restrict__ gate, SpanFastArgs a) {
  constexpr int d = DT * 16, DS = (d + 31) / 32;
  constexpr float kLow = -1e30f;
  // kDeal: the block's wavefronts share one head and deal its tiles of keys out; else every wavefront has a head of its own (NW heads a block, neighbours of one
  // key head: they walk the same tiles at about the same time, and what one has fetched the others find in the caches)
  __shared__ float others_acc[kDeal ? NW - 1 : 1][kDeal ? DT : 1][kDeal ? kWave : 1][4];      // what the other wavefronts hand to the first: their sums, ...
  __shared__ float others_ml[kDeal ? NW - 1 : 1][2][kDeal ? kWave : 1];                       // ... maxima and weights' sums
  const int lane = threadIdx.x % kWave, col = lane % 16, grp = lane / 16, wave = kDeal ? threadIdx.x / kWave : 0;
  const int h = kDeal ? blockIdx.y : blockIdx.y * NW + threadIdx.x / kWave;
  constexpr int kStep = kDeal ? 32 * NW : 32;
  if (!kDeal && h >= a.heads) return;
  const int g = h / (a.heads / a.kv_heads), S = 1 << a.bs_shift;
  int r, row0, n;
  if (a.tiles) {
    r = a.tiles[3 * blockIdx.x], row0 = a.tiles[3 * blockIdx.x + 1], n = a.tiles[3 * blockIdx.x + 2];
  } else {
    row0 = blockIdx.x, n = 1, r = a.req_of_token ? a.req_of_token[row0] : row0;
  }
  const bool valid = col < n;
  const int row = row0 + (valid ? col : 0);
  const int p = a.positions[row];
  const int p_first = a.positions[row0], p_last = a.positions[row0 + n - 1];
  const int W = a.window;
  const int lo = (W > 0 && p_first - W + 1 > 0) ? p_first - W + 1 : 0;
  const int32_t* tab = a.table + static_cast<int64_t>(r) * a.max_blocks;

  span_bf16x8 qf[DS];
#pragma unroll
  for (int s = 0; s < DS; ++s) {
    const int c = s * 32 + grp * 8;
    qf[s] = span_bf16x8{};
    if (valid && c < d) qf[s] = *reinterpret_cast<const span_bf16x8*>(q + static_cast<int64_t>(row) * a.q_stride + static_cast<int64_t>(h) * d + c);
  }
  span_f32x4 acc[DT];
#pragma unroll
  for (int o = 0; o < DT; ++o) acc[o] = span_f32x4{0.f, 0.f, 0.f, 0.f};
  float m = kLow, l = 0.f;
  const float* bias = a.bias ? a.bias + static_cast<int64_t>(h) * a.bias_len : nullptr;

  // one tile of 32 entries: scores sc[u][r] for entries e(u, r) = t0 + 16 u + 4 grp + r of query col, their visibility, and the second product
  auto softmax_step = [&](span_f32x4 (&sc)[2], const bool (&seen)[2][4], auto&& values) {
    float top = kLow;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int x = 0; x < 4; ++x) top = fmaxf(top, seen[u][x] ? sc[u][x] : kLow);
    top = rows_max(top);
    const float m_new = fmaxf(m, top), alpha = __expf(m - m_new);
    // (the weights are 32-bit numbers: each meets the values as two bfloat16 numbers, its rounding and what the rounding took away)
    span_bf16x8 w, rest;
    float sum = 0.f;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const float e = seen[u][x] ? __expf(sc[u][x] - m_new) : 0.f;
        sum += e;
        w[4 * u + x] = static_cast<__bf16>(e);
        rest[4 * u + x] = static_cast<__bf16>(e - static_cast<float>(w[4 * u + x]));
      }
    l = l * alpha + sum;
    m = m_new;
#pragma unroll
    for (int o = 0; o < DT; ++o) {
      const span_bf16x8 vf = values(o);
      acc[o] *= alpha;
      acc[o] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, w, acc[o], 0, 0, 0);
      acc[o] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, rest, acc[o], 0, 0, 0);
    }
  };

  // ---- the window's tokens
  for (int t0 = (lo / 32) * 32 + 32 * wave; t0 <= p_last; t0 += kStep) {
    span_f32x4 sc[2];
    bool seen[2][4];
    // the tile's values are asked for first: they are on their way while the scores are formed (they do not depend on them)
    uint2 vraw[DT][2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      int j = t0 + 16 * u + 4 * grp;      // (four keys of one page; clamped to a run whose page is held)
      j = j < (lo & ~3) ? (lo & ~3) : (j > (p_last & ~3) ? (p_last & ~3) : j);
      const bf16_t* vrow = v_cache + ((static_cast<int64_t>(tab[j >> a.bs_shift]) * a.kv_heads + g) * d + col) * S + (j & (S - 1));
#pragma unroll
      for (int o = 0; o < DT; ++o) vraw[o][u] = *reinterpret_cast<const uint2*>(vrow + static_cast<int64_t>(o) * 16 * S);
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      int key = t0 + 16 * u + col;      // (the key this lane fetches for the first product: clamped to one whose page is held)
      key = key < lo ? lo : (key > p_last ? p_last : key);
      const bf16_t* krow = k_cache + ((static_cast<int64_t>(tab[key >> a.bs_shift]) * a.kv_heads + g) * S + (key & (S - 1))) * d;
      sc[u] = span_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < DS; ++s) {
        const int c = s * 32 + grp * 8;
        span_bf16x8 kf = span_bf16x8{};
        if (c < d) kf = *reinterpret_cast<const span_bf16x8*>(krow + c);
        sc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[s], sc[u], 0, 0, 0);
      }
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const int j = t0 + 16 * u + 4 * grp + x, dist = p - j;
        seen[u][x] = valid && dist >= 0 && (W <= 0 || dist < W);
        float b = 0.f;
        if (bias && seen[u][x]) b = bias[dist < a.bias_len ? dist : a.bias_len - 1];
        sc[u][x] = sc[u][x] * a.scale + b;
      }
    }
    softmax_step(sc, seen, [&](int o) {
      typedef uint32_t span_u32x4 __attribute__((ext_vector_type(4)));
      const span_u32x4 raw = {vraw[o][0].x, vraw[o][0].y, vraw[o][1].x, vraw[o][1].y};
      return __builtin_bit_cast(span_bf16x8, raw);
    });
  }

  // ---- the blocks wholly behind the window
  const int n_blk_tile = (a.pool_table && W > 0 && p_last - W + 1 >= a.P) ? (p_last - W + 1) / a.P : 0;
  if (n_blk_tile > 0) {
    const int32_t* ptab = a.pool_table + static_cast<int64_t>(r) * a.pool_max_blocks;
    const int mine = (p - W + 1 >= a.P) ? (p - W + 1) / a.P : 0;      // how many blocks this lane's query sees
    auto place_of = [&](int e, int64_t& page, int& place) {
      e = e < n_blk_tile ? e : n_blk_tile - 1;
      const int first = e * a.P;
      page = ptab[first >> a.bs_shift];
      place = (first & (S - 1)) / a.P;
    };
    for (int e0 = 32 * wave; e0 < n_blk_tile; e0 += kStep) {
      span_f32x4 sc[2];
      bool seen[2][4];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        int64_t page;
        int place;
        place_of(e0 + 16 * u + col, page, place);
        const bf16_t* krow = pk + ((page * a.kv_heads + g) * a.places + place) * d;
        sc[u] = span_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < DS; ++s) {
          const int c = s * 32 + grp * 8;
          span_bf16x8 kf = span_bf16x8{};
          if (c < d) kf = *reinterpret_cast<const span_bf16x8*>(krow + c);
          sc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[s], sc[u], 0, 0, 0);
        }
#pragma unroll
        for (int x = 0; x < 4; ++x) {
          seen[u][x] = valid && e0 + 16 * u + 4 * grp + x < mine;
          sc[u][x] *= a.scale;
        }
      }
      int64_t pages[8];
      int places[8];
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int x = 0; x < 4; ++x) place_of(e0 + 16 * u + 4 * grp + x, pages[4 * u + x], places[4 * u + x]);
      softmax_step(sc, seen, [&](int o) {
        span_bf16x8 vf;
#pragma unroll
        for (int i = 0; i < 8; ++i)
          vf[i] = __builtin_bit_cast(__bf16, pv[((pages[i] * a.kv_heads + g) * d + o * 16 + col) * a.places + places[i]]);
        return vf;
      });
    }
  }

  float total = rows_sum(l);
  if constexpr (kDeal) {
  if (wave > 0) {
    others_ml[wave - 1][0][lane] = m;
    others_ml[wave - 1][1][lane] = total;
#pragma unroll
    for (int o = 0; o < DT; ++o)
#pragma unroll
      for (int x = 0; x < 4; ++x) others_acc[wave - 1][o][lane][x] = acc[o][x];
  }
  __syncthreads();
  if (wave > 0) return;
#pragma unroll
  for (int w = 0; w < NW - 1; ++w) {
    const float m_w = others_ml[w][0][lane], m_new = fmaxf(m, m_w), mine = __expf(m - m_new), theirs = __expf(m_w - m_new);
    total = total * mine + others_ml[w][1][lane] * theirs;
    m = m_new;
#pragma unroll
    for (int o = 0; o < DT; ++o)
#pragma unroll
      for (int x = 0; x < 4; ++x) acc[o][x] = acc[o][x] * mine + others_acc[w][o][lane][x] * theirs;
  }
  }
  if (a.sink) {
    const float sk = a.sink[h], m_f = fmaxf(m, sk), alpha = __expf(m - m_f);
    total = total * alpha + __expf(sk - m_f);
#pragma unroll
    for (int o = 0; o < DT; ++o) acc[o] *= alpha;
  }
  if (!valid) return;
  const float inv = 1.f / total;
  bf16_t* orow = out + static_cast<int64_t>(row) * a.out_stride + static_cast<int64_t>(h) * d;
  const bf16_t* grow = a.gate_kind ? gate + static_cast<int64_t>(row) * a.gate_stride : nullptr;
  const float head_gate = a.gate_kind == 2 ? 1.f / (1.f + __expf(-bf16_to_f32(grow[h]))) : 1.f;
#pragma unroll
  for (int o = 0; o < DT; ++o) {
    float y[4];
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const int c = o * 16 + 4 * grp + x;
      y[x] = acc[o][x] * inv * head_gate;
      if (a.gate_kind == 1) y[x] = c < a.dv_true ? y[x] / (1.f + __expf(-bf16_to_f32(grow[static_cast<int64_t>(h) * a.dv_true + c]))) : 0.f;
    }
    *reinterpret_cast<uint2*>(orow + o * 16 + 4 * grp) = uint2{pack_bf16x2(y[0], y[1]), pack_bf16x2(y[2], y[3])};
  }
}

// out[t, h, :] *= sigmoid(gate[t, h]) (one gate per head) or sigmoid(gate[t, h, :]) (one per channel): what the matrix-core
// attention kernels leave, on its way to the output projection.
template <typename T>
__global__ void __launch_bounds__(256) head_gate_kernel(T* __restrict__ x, int64_t x_stride, const T* __restrict__ gate, int64_t gate_stride,
                                                        int64_t rows, int heads, int dv, int dv_stored, int per_head) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  const int width = heads * dv;
  if (idx >= rows * width) return;
  const int64_t t = idx / width;
  const int e = static_cast<int>(idx % width), h = e / dv, c = e % dv;
  const float z = load_f32(gate + t * gate_stride + (per_head ? h : e));
  T* at = x + t * x_stride + static_cast<int64_t>(h) * dv_stored + c;
  store_f32(at, load_f32(at) / (1.f + expf(-z)));
}

}  // namespace alofa

using namespace alofa;

extern "C" int alofa_norm_turn_write(void* qkv, int64_t stride, int dtype, const int32_t* positions, const float* cos_t, const float* sin_t, int half,
                                     int scope, const float* wq, const float* wk, float eps, double* row_inv, const int64_t* slots, void* k_cache, void* v_cache,
                                     int block_size, int tokens, int heads, int kv_heads, int d, int dv, int d_true, int values_are_keys, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(tokens >= 0 && heads > 0 && kv_heads >= 0 && d > 0 && d <= 256 && dv > 0 && dv <= 256, "norm_turn_write: bad sizes (heads=%d kv_heads=%d d=%d dv=%d; heads of up to 256 channels)", heads, kv_heads, d, dv);
  ALOFA_REQUIRE(half >= 0 && 2 * half <= d && (half == 0 || (cos_t && sin_t)), "norm_turn_write: %d pairs do not fit a head of %d channels, or their table is absent", half, d);
  ALOFA_REQUIRE(scope >= kNormNone && scope <= kNormAll && eps >= 0.f, "norm_turn_write: no such norm (%d)", scope);
  ALOFA_REQUIRE(kv_heads == 0 || (slots && k_cache && v_cache && block_size > 0), "norm_turn_write: keys and values need slots and caches");
  ALOFA_REQUIRE(!values_are_keys || d == dv, "norm_turn_write: values that are the keys have the keys' size");
  ALOFA_REQUIRE(d_true > 0 && d_true <= d, "norm_turn_write: a head holds %d channels of which %d count", d, d_true);
  ALOFA_REQUIRE(!exact || dtype == kF32, "norm_turn_write: the exact path is float32");
  if (tokens == 0) return 0;
  const int per_row = heads + kv_heads + (values_are_keys ? 0 : kv_heads);
  ALOFA_REQUIRE(scope != kNormAll || row_inv != nullptr, "norm_turn_write: a norm over the whole projection needs room for the rows' factors");
  if (scope == kNormAll) {
    const unsigned g2 = static_cast<unsigned>(2 * static_cast<int64_t>(tokens));
    if (exact) projection_inv_rms_kernel<float, double><<<g2, 256, 0, stream>>>(row_inv, static_cast<const float*>(qkv), stride, tokens, heads * d, kv_heads * d, heads * d_true, kv_heads * d_true, eps);
    else if (dtype == kF32) projection_inv_rms_kernel<float, float><<<g2, 256, 0, stream>>>(row_inv, static_cast<const float*>(qkv), stride, tokens, heads * d, kv_heads * d, heads * d_true, kv_heads * d_true, eps);
    else projection_inv_rms_kernel<bf16_t, float><<<g2, 256, 0, stream>>>(row_inv, static_cast<const bf16_t*>(qkv), stride, tokens, heads * d, kv_heads * d, heads * d_true, kv_heads * d_true, eps);
  }
  const unsigned grid = static_cast<unsigned>((static_cast<int64_t>(tokens) * per_row + 3) / 4);
#define ALOFA_NTW(T, ACC) norm_turn_write_kernel<T, ACC><<<grid, 256, 0, stream>>>(static_cast<T*>(qkv), stride, positions, half ? cos_t : nullptr, half ? sin_t : nullptr, half, scope, wq, wk, eps, row_inv, \
    slots, static_cast<T*>(k_cache), static_cast<T*>(v_cache), block_size, tokens, heads, kv_heads, d, dv, d_true, values_are_keys)
  if (exact) ALOFA_NTW(float, double);
  else if (dtype == kF32) ALOFA_NTW(float, float);
  else ALOFA_NTW(bf16_t, float);
#undef ALOFA_NTW
  return check_launch("norm_turn_write");
}

extern "C" int alofa_pool_blocks(const void* k_cache, const void* v_cache, void* pk, void* pv, int dtype, const int32_t* table, int max_blocks,
                                 const int32_t* pool_table, int pool_max_blocks, const int32_t* req_of_token, const int32_t* positions, int tokens,
                                 int kv_heads, int d, int dv, int block_size, int P, int places, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(tokens >= 0 && kv_heads > 0 && d > 0 && dv > 0 && block_size > 0 && P > 0 && places == (block_size - 1) / P + 1, "pool_blocks: bad sizes (kv_heads=%d d=%d dv=%d page=%d P=%d places=%d)", kv_heads, d, dv, block_size, P, places);
  ALOFA_REQUIRE(!exact || dtype == kF32, "pool_blocks: the exact path is float32");
  if (tokens == 0) return 0;
  const dim3 grid(tokens, kv_heads);
#define ALOFA_POOL(T, ACC) pool_blocks_kernel<T, ACC><<<grid, 128, 0, stream>>>(static_cast<const T*>(k_cache), static_cast<const T*>(v_cache), static_cast<T*>(pk), static_cast<T*>(pv), \
    table, max_blocks, pool_table, pool_max_blocks, req_of_token, positions, kv_heads, d, dv, block_size, P, places)
  if (exact) ALOFA_POOL(float, double);
  else if (dtype == kF32) ALOFA_POOL(float, float);
  else ALOFA_POOL(bf16_t, float);
#undef ALOFA_POOL
  return check_launch("pool_blocks");
}

extern "C" int alofa_span_attention(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k_cache, const void* v_cache, const void* pk, const void* pv,
                                    int dtype, const int32_t* table, int max_blocks, const int32_t* pool_table, int pool_max_blocks, const int32_t* req_of_token,
                                    const int32_t* positions, int tokens, int heads, int kv_heads, int d, int dv, int block_size, int window, int P, int places, float scale,
                                    const float* bias, int bias_len, const float* sink, const void* gate, int64_t gate_stride, int gate_kind, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(tokens >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "span_attention: tokens=%d heads=%d kv_heads=%d (kv_heads must divide heads)", tokens, heads, kv_heads);
  ALOFA_REQUIRE(d > 0 && d <= 256 && dv > 0 && dv <= 256, "span_attention: head sizes %d and %d (up to 256 channels)", d, dv);
  ALOFA_REQUIRE(block_size > 0 && max_blocks > 0 && window >= 0, "span_attention: block_size=%d max_blocks=%d window=%d", block_size, max_blocks, window);
  ALOFA_REQUIRE(pool_table == nullptr || (pk && pv && window > 0 && P > 0 && places == (block_size - 1) / P + 1 && pool_max_blocks > 0), "span_attention: pooled blocks need their pages, a window and P (P=%d places=%d)", P, places);
  ALOFA_REQUIRE(bias == nullptr || bias_len > 0, "span_attention: an empty bias table");
  ALOFA_REQUIRE(gate_kind >= 0 && gate_kind <= 2 && (gate_kind == 0 || gate != nullptr), "span_attention: no such gate (%d)", gate_kind);
  ALOFA_REQUIRE(!exact || dtype == kF32, "span_attention: the exact path is float32");
  if (tokens == 0) return 0;
  SpanArgs a{out_stride, q_stride, gate_stride, table, max_blocks, pool_table, pool_max_blocks, req_of_token, positions, tokens, heads, kv_heads, d, dv, block_size, window,
             P, places, scale, bias, bias_len, sink, gate_kind};
  const unsigned grid = static_cast<unsigned>((static_cast<int64_t>(tokens) * heads + 3) / 4);
#define ALOFA_SPAN(T, ACC) span_attention_kernel<T, ACC><<<grid, 256, 0, stream>>>(static_cast<T*>(out), static_cast<const T*>(q), static_cast<const T*>(k_cache), static_cast<const T*>(v_cache), \
    static_cast<const T*>(pk), static_cast<const T*>(pv), static_cast<const T*>(gate), a)
  if (exact) ALOFA_SPAN(float, double);
  else if (dtype == kF32) ALOFA_SPAN(float, float);
  else ALOFA_SPAN(bf16_t, float);
#undef ALOFA_SPAN
  return check_launch("span_attention");
}

template <int DT>
static void launch_span_mfma(dim3 grid, hipStream_t stream, void* out, const void* q, const void* k_cache, const void* v_cache, const void* pk, const void* pv, const void* gate,
                             const SpanFastArgs& a) {
  // Single rows, where blocks are few: a block per row and head, its eight wavefronts (four for heads wider than 128 channels: their states must fit the LDS a block
  // may name) deal the tiles of keys out. Runs of rows, where blocks are many: four heads a block, a wavefront each (a layer of a 2,048-token prompt at 16 heads of 128:
  // 78 us, against 79 with four and 91 with eight wavefronts dealing a head's tiles out, and no LDS).
#define ALOFA_SPAN_LAUNCH(NW, DEAL, GRID) span_attention_mfma_kernel<DT, NW, DEAL><<<GRID, 64 * NW, 0, stream>>>(static_cast<bf16_t*>(out), static_cast<const bf16_t*>(q), \
    static_cast<const bf16_t*>(k_cache), static_cast<const bf16_t*>(v_cache), static_cast<const bf16_t*>(pk), static_cast<const bf16_t*>(pv), static_cast<const bf16_t*>(gate), a)
  if (a.tiles != nullptr) ALOFA_SPAN_LAUNCH(4, false, dim3(grid.x, (a.heads + 3) / 4));
  else if (DT <= 8) ALOFA_SPAN_LAUNCH((DT <= 8 ? 8 : 4), true, grid);
  else ALOFA_SPAN_LAUNCH(4, true, grid);
#undef ALOFA_SPAN_LAUNCH
}

// bfloat16 on the matrix cores: heads of d = dv channels in steps of 16, pages of a power of two of at least 8 tokens, rows 16-byte aligned.
extern "C" int alofa_span_attention_mfma(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k_cache, const void* v_cache, const void* pk, const void* pv,
                                         const int32_t* tiles, int n_tiles, const int32_t* table, int max_blocks, const int32_t* pool_table, int pool_max_blocks,
                                         const int32_t* req_of_token, const int32_t* positions, int heads, int kv_heads, int d, int dv_true, int block_size, int window, int P,
                                         int places, float scale, const float* bias, int bias_len, const float* sink, const void* gate, int64_t gate_stride, int gate_kind,
                                         hipStream_t stream) {
  ALOFA_REQUIRE(n_tiles >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "span_attention_mfma: tiles=%d heads=%d kv_heads=%d (kv_heads must divide heads)", n_tiles, heads, kv_heads);
  ALOFA_REQUIRE(d >= 16 && d <= 256 && d % 16 == 0 && dv_true > 0 && dv_true <= d, "span_attention_mfma: head size %d (16 to 256 in steps of 16), of which %d value channels count", d, dv_true);
  ALOFA_REQUIRE(block_size >= 8 && (block_size & (block_size - 1)) == 0 && max_blocks > 0 && window >= 0, "span_attention_mfma: pages of a power of two of at least 8 tokens (block_size=%d), window=%d", block_size, window);
  ALOFA_REQUIRE(pool_table == nullptr || (pk && pv && window > 0 && P > 0 && places == (block_size - 1) / P + 1 && pool_max_blocks > 0), "span_attention_mfma: pooled blocks need their pages, a window and P (P=%d places=%d)", P, places);
  ALOFA_REQUIRE(bias == nullptr || bias_len > 0, "span_attention_mfma: an empty bias table");
  ALOFA_REQUIRE(gate_kind >= 0 && gate_kind <= 2 && (gate_kind == 0 || gate != nullptr), "span_attention_mfma: no such gate (%d)", gate_kind);
  ALOFA_REQUIRE(q_stride % 8 == 0 && out_stride % 4 == 0 && reinterpret_cast<uintptr_t>(q) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 8 == 0, "span_attention_mfma: rows must be 16-byte aligned");
  if (n_tiles == 0) return 0;
  int shift = 0;
  while ((1 << shift) < block_size) ++shift;
  SpanFastArgs a{out_stride, q_stride, gate_stride, tiles, table, max_blocks, pool_table, pool_max_blocks, req_of_token, positions, n_tiles, heads, kv_heads, shift, window,
                 P, places, dv_true, scale, bias, bias_len, sink, gate_kind};
  const dim3 grid(n_tiles, heads);
  switch (d / 16) {
#define ALOFA_SPAN_DT(N) case N: launch_span_mfma<N>(grid, stream, out, q, k_cache, v_cache, pk, pv, gate, a); break;
    ALOFA_SPAN_DT(1) ALOFA_SPAN_DT(2) ALOFA_SPAN_DT(3) ALOFA_SPAN_DT(4) ALOFA_SPAN_DT(5) ALOFA_SPAN_DT(6) ALOFA_SPAN_DT(7) ALOFA_SPAN_DT(8)
    ALOFA_SPAN_DT(9) ALOFA_SPAN_DT(10) ALOFA_SPAN_DT(11) ALOFA_SPAN_DT(12) ALOFA_SPAN_DT(13) ALOFA_SPAN_DT(14) ALOFA_SPAN_DT(15) ALOFA_SPAN_DT(16)
#undef ALOFA_SPAN_DT
    default: ALOFA_REQUIRE(false, "span_attention_mfma: head size %d", d);
  }
  return check_launch("span_attention_mfma");
}

extern "C" int alofa_head_gate(void* x, int64_t x_stride, const void* gate, int64_t gate_stride, int dtype, int64_t rows, int heads, int dv, int dv_stored, int per_head, hipStream_t stream) {
  ALOFA_REQUIRE(rows >= 0 && heads > 0 && dv > 0 && dv_stored >= dv, "head_gate: bad sizes (heads=%d dv=%d stored=%d)", heads, dv, dv_stored);
  if (rows == 0) return 0;
  const unsigned grid = static_cast<unsigned>((rows * heads * dv + 255) / 256);
  if (dtype == kF32) head_gate_kernel<float><<<grid, 256, 0, stream>>>(static_cast<float*>(x), x_stride, static_cast<const float*>(gate), gate_stride, rows, heads, dv, dv_stored, per_head);
  else head_gate_kernel<bf16_t><<<grid, 256, 0, stream>>>(static_cast<bf16_t*>(x), x_stride, static_cast<const bf16_t*>(gate), gate_stride, rows, heads, dv, dv_stored, per_head);
  return check_launch("head_gate");
}
