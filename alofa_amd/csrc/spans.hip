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
  const int64_t unit = static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / kWave;
  if (unit >= 2 * static_cast<int64_t>(tokens)) return;
  const int lane = threadIdx.x % kWave;
  const int t = static_cast<int>(unit / 2), which = static_cast<int>(unit % 2);
  const T* x = qkv + static_cast<int64_t>(t) * stride + (which ? q_width : 0);
  const int n = which ? k_width : q_width;
  Acc ss = 0;
  for (int c = lane; c < n; c += kWave) {
    const Acc v = static_cast<Acc>(load_f32(x + c));
    ss += v * v;
  }
  ss = wave_sum(ss);
  if (lane == 0) inv[unit] = static_cast<double>(static_cast<Acc>(1) / sqrt(ss / static_cast<Acc>(which ? k_count : q_count) + static_cast<Acc>(eps)));
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
    const unsigned g2 = static_cast<unsigned>((2 * static_cast<int64_t>(tokens) + 3) / 4);
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

extern "C" int alofa_head_gate(void* x, int64_t x_stride, const void* gate, int64_t gate_stride, int dtype, int64_t rows, int heads, int dv, int dv_stored, int per_head, hipStream_t stream) {
  ALOFA_REQUIRE(rows >= 0 && heads > 0 && dv > 0 && dv_stored >= dv, "head_gate: bad sizes (heads=%d dv=%d stored=%d)", heads, dv, dv_stored);
  if (rows == 0) return 0;
  const unsigned grid = static_cast<unsigned>((rows * heads * dv + 255) / 256);
  if (dtype == kF32) head_gate_kernel<float><<<grid, 256, 0, stream>>>(static_cast<float*>(x), x_stride, static_cast<const float*>(gate), gate_stride, rows, heads, dv, dv_stored, per_head);
  else head_gate_kernel<bf16_t><<<grid, 256, 0, stream>>>(static_cast<bf16_t*>(x), x_stride, static_cast<const bf16_t*>(gate), gate_stride, rows, heads, dv, dv_stored, per_head);
  return check_launch("head_gate");
}
