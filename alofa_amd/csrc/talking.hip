// Attention whose heads talk to one another after the softmax, over a paged cache, with unit-norm queries and keys and
// values that are turned by their positions:
//
//   turn_norm_write   what a step's projections become before attention: every query and key head is turned by its
//                     row's position on its first channels (pairs (i, i + n/2), angles from a table), then divided by its
//                     root mean square; every value head is turned on all its channels by a table of its own; keys and
//                     values go to their rows' cache slots.
//   talking_attention softmax over the keys a row may see (all before it, or the last `window`), per query head; then the
//                     heads' weights are mixed, w_h(j) = sum_g M[h, g] p_g(j), and head h applies its mixed weights to the
//                     values of its own key/value head; the result is turned back by the row's own position (values were
//                     turned by theirs), and optionally multiplied by the sigmoid of a gate.
//
// Cache layout (that of the other attention kernels): keys [block, kv_head, slot, d], values transposed [block, kv_head, dv, slot]; d and dv may differ.
//
// Arithmetic: products and sums in Acc (float; double in the exact path), in ascending key order per output channel, so a
// row's result depends on the keys it sees and on nothing else: not on how rows were cut into steps, on the batch or on pages.
#include "common.h"

#include <float.h>

namespace alofa {

// One wavefront per (row, head): query heads first, then key heads, then value heads.
template <typename T, typename Acc>
__global__ void __launch_bounds__(256) turn_norm_write_kernel(T* __restrict__ qkv, int64_t stride, const int32_t* __restrict__ positions,
                                                              const float* __restrict__ cos_qk, const float* __restrict__ sin_qk, int half_qk,
                                                              const float* __restrict__ cos_v, const float* __restrict__ sin_v,
                                                              const int64_t* __restrict__ slots, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                                              int block_size, int tokens, int heads, int kv_heads, int d, int dv, float eps, int unit_norm) {
  const int per_row = heads + 2 * kv_heads;
  const int64_t unit = static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / kWave;
  if (unit >= static_cast<int64_t>(tokens) * per_row) return;
  const int lane = threadIdx.x % kWave;
  const int t = static_cast<int>(unit / per_row), u = static_cast<int>(unit % per_row);
  const int p = positions[t];
  const bool is_v = u >= heads + kv_heads, is_k = !is_v && u >= heads;
  const int width = is_v ? dv : d, half = is_v ? dv / 2 : half_qk;
  T* src = qkv + static_cast<int64_t>(t) * stride + (is_v ? static_cast<int64_t>(heads + kv_heads) * d + static_cast<int64_t>(u - heads - kv_heads) * dv : static_cast<int64_t>(u) * d);
  T* dst = src;
  int64_t step = 1;      // between two channels at the destination (values lie transposed in their pages: a channel's slots side by side)
  if (is_k) {
    const int64_t slot = slots[t];
    dst = k_cache + (((slot / block_size) * kv_heads + (u - heads)) * block_size + slot % block_size) * static_cast<int64_t>(d);
  } else if (is_v) {
    const int64_t slot = slots[t];
    dst = v_cache + ((slot / block_size) * kv_heads + (u - heads - kv_heads)) * static_cast<int64_t>(dv) * block_size + slot % block_size;
    step = block_size;
  }
  const float* ct = (is_v ? cos_v : cos_qk) + static_cast<int64_t>(p) * half;
  const float* st = (is_v ? sin_v : sin_qk) + static_cast<int64_t>(p) * half;
  constexpr int kPairs = 2, kPass = 4;      // heads up to 256 channels
  float a[kPairs], b[kPairs], rest[kPass];
  Acc ss = 0;
#pragma unroll
  for (int n = 0; n < kPairs; ++n) {
    const int i = lane + n * kWave;
    a[n] = b[n] = 0.f;
    if (i < half) {
      const float x = load_f32(src + i), y = load_f32(src + i + half), c = ct[i], s = st[i];
      a[n] = x * c - y * s;
      b[n] = y * c + x * s;
    }
    ss += static_cast<Acc>(a[n]) * static_cast<Acc>(a[n]) + static_cast<Acc>(b[n]) * static_cast<Acc>(b[n]);
  }
#pragma unroll
  for (int n = 0; n < kPass; ++n) {
    const int c = 2 * half + lane + n * kWave;
    rest[n] = c < width ? load_f32(src + c) : 0.f;
    ss += static_cast<Acc>(rest[n]) * static_cast<Acc>(rest[n]);
  }
  Acc inv = 1;
  if (unit_norm && !is_v) {
    ss = wave_sum(ss);
    inv = static_cast<Acc>(1) / sqrt(ss / static_cast<Acc>(width) + static_cast<Acc>(eps));
  }
#pragma unroll
  for (int n = 0; n < kPairs; ++n) {
    const int i = lane + n * kWave;
    if (i < half) {
      store_f32(dst + i * step, static_cast<float>(static_cast<Acc>(a[n]) * inv));
      store_f32(dst + (i + half) * step, static_cast<float>(static_cast<Acc>(b[n]) * inv));
    }
  }
#pragma unroll
  for (int n = 0; n < kPass; ++n) {
    const int c = 2 * half + lane + n * kWave;
    if (c < width) store_f32(dst + c * step, static_cast<float>(static_cast<Acc>(rest[n]) * inv));
  }
}

// ---- the always-valid attention kernel: a block per row ---------------------------------------------------
// Four wavefronts share the heads out for the scores (a lane a key, the whole dot product in the lane); the mixing of the
// heads' weights and the sum over the values are shared out over all threads (a thread owns outputs (head, channel)).
constexpr int kTalkOwn = 32;      // outputs a thread may own: heads * dv <= 256 * kTalkOwn

template <typename T, typename Acc>
__device__ __forceinline__ Acc talk_score(const float* qs, const T* __restrict__ k_cache, const int32_t* __restrict__ table, int j, int c,
                                          int kv_heads, int d, int block_size, float scale) {
  const int64_t blk = table[j / block_size];
  const T* k = k_cache + ((blk * kv_heads + c) * block_size + (j % block_size)) * static_cast<int64_t>(d);
  Acc acc = 0;
  for (int e = 0; e < d; ++e) acc += static_cast<Acc>(qs[e]) * static_cast<Acc>(load_f32(k + e));
  return acc * static_cast<Acc>(scale);
}

template <typename T, typename Acc>
__global__ void __launch_bounds__(256) talking_attention_kernel(
    T* __restrict__ out, int64_t out_stride, const T* __restrict__ q, int64_t q_stride, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int32_t* __restrict__ block_table, int max_blocks, const int32_t* __restrict__ req_of_token, const int32_t* __restrict__ positions,
    int heads, int kv_heads, int d, int dv, int block_size, int window, float scale, const float* __restrict__ talk,
    const float* __restrict__ cos_v, const float* __restrict__ sin_v, const T* __restrict__ gate, int64_t gate_stride) {
  extern __shared__ float4 talk_lds4[];
  float* qs = reinterpret_cast<float*>(talk_lds4);      // [heads * d]
  float* mix = qs + heads * d;                          // [heads * heads]
  float* P = mix + heads * heads;                       // [heads][64]
  float* Wm = P + heads * kWave;                        // [heads][64]
  float* O = Wm + heads * kWave;                        // [heads * dv]
  Acc* ms = reinterpret_cast<Acc*>((reinterpret_cast<uintptr_t>(O + heads * dv) + 7) & ~static_cast<uintptr_t>(7));     // [heads] maxima, [heads] sums
  Acc* ls = ms + heads;
  const int t = blockIdx.x, tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  const int per = heads / kv_heads;
  const int p = positions[t];
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int32_t* table = block_table + static_cast<int64_t>(req_of_token ? req_of_token[t] : t) * max_blocks;
  const T* qrow = q + static_cast<int64_t>(t) * q_stride;
  for (int e = tid; e < heads * d; e += 256) qs[e] = load_f32(qrow + e);
  for (int e = tid; e < heads * heads; e += 256) mix[e] = talk ? talk[e] : (e / heads == e % heads ? 1.f : 0.f);
  __syncthreads();

  // every head's maximum and sum of exponentials (a lane keeps its own running pair; the lanes' pairs meet at the end)
  for (int g = wave; g < heads; g += 4) {
    Acc m = -DBL_MAX, l = 0;
    bool any = false;
    for (int j = lo + lane; j <= p; j += kWave) {
      const Acc s = talk_score<T, Acc>(qs + g * d, k_cache, table, j, g / per, kv_heads, d, block_size, scale);
      if (!any || s > m) {
        l = any ? l * exp(m - s) : static_cast<Acc>(0);
        m = s;
        any = true;
      }
      l += exp(s - m);
    }
    float mf = any ? static_cast<float>(m) : -FLT_MAX;
    const float top = wave_max(mf);      // (a float at least as large as every lane's maximum, up to rounding: any such value serves)
    Acc top_acc = static_cast<Acc>(top);
    const Acc mine = any ? l * exp(m - top_acc) : static_cast<Acc>(0);
    const Acc total = wave_sum(mine);
    if (lane == 0) {
      ms[g] = top_acc;
      ls[g] = total;
    }
  }
  __syncthreads();

  Acc acc[kTalkOwn];
#pragma unroll
  for (int n = 0; n < kTalkOwn; ++n) acc[n] = 0;
  const int outputs = heads * dv;
  for (int j0 = lo; j0 <= p; j0 += kWave) {
    for (int g = wave; g < heads; g += 4) {
      const int j = j0 + lane;
      float w = 0.f;
      if (j <= p) {
        const Acc s = talk_score<T, Acc>(qs + g * d, k_cache, table, j, g / per, kv_heads, d, block_size, scale);
        w = static_cast<float>(exp(s - ms[g]) / ls[g]);
      }
      P[g * kWave + lane] = w;
    }
    __syncthreads();
    for (int e = tid; e < heads * kWave; e += 256) {
      const int h = e / kWave, jj = e % kWave;
      Acc w = 0;
      for (int g = 0; g < heads; ++g) w += static_cast<Acc>(mix[h * heads + g]) * static_cast<Acc>(P[g * kWave + jj]);
      Wm[e] = static_cast<float>(w);
    }
    __syncthreads();
    const int n_keys = (p - j0 + 1 < kWave) ? p - j0 + 1 : kWave;
    for (int jj = 0; jj < n_keys; ++jj) {
      const int j = j0 + jj;
      const int64_t blk = table[j / block_size];
      const T* vrow = v_cache + blk * kv_heads * static_cast<int64_t>(dv) * block_size + (j % block_size);
#pragma unroll
      for (int n = 0; n < kTalkOwn; ++n) {
        const int e = tid + n * 256;
        if (e < outputs) {
          const int h = e / dv, c = e % dv;
          acc[n] += static_cast<Acc>(Wm[h * kWave + jj]) * static_cast<Acc>(load_f32(vrow + (static_cast<int64_t>(h / per) * dv + c) * block_size));
        }
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int n = 0; n < kTalkOwn; ++n) {
    const int e = tid + n * 256;
    if (e < outputs) O[e] = static_cast<float>(acc[n]);
  }
  __syncthreads();
  // turned back by the row's own position: pair (c, c + dv/2) by minus the angle
  const int half = dv / 2;
  for (int e = tid; e < outputs; e += 256) {
    const int h = e / dv, c = e % dv;
    float y = O[e];
    if (cos_v) {
      const int i = c < half ? c : c - half;
      const float cs = cos_v[static_cast<int64_t>(p) * half + i], sn = sin_v[static_cast<int64_t>(p) * half + i];
      const float x0 = O[h * dv + i], x1 = O[h * dv + i + half];
      y = c < half ? x0 * cs + x1 * sn : x1 * cs - x0 * sn;
    }
    if (gate) {
      const Acc z = static_cast<Acc>(load_f32(gate + static_cast<int64_t>(t) * gate_stride + e));
      y = static_cast<float>(static_cast<Acc>(y) / (static_cast<Acc>(1) + exp(-z)));
    }
    store_f32(out + static_cast<int64_t>(t) * out_stride + e, y);
  }
}

// ---- the heads' talk after the fact ---------------------------------------------------------------------
// Mixing the heads' weights is linear in what the weights are applied to: with A[c][g] = sum_j p_g(j) v_c(j), the
// unmixed weights of query head g applied to the values of value head c (float rows [kv_heads][T][heads * dv], from
// the matrix-core attention kernels run once per value head), head h's result is sum_g M[h, g] A[c(h)][g]. A thread owns
// a pair of channels (i, i + dv/2) of one head (a block per row and head): sums over g in ascending order, turns the pair back by the row's
// position and multiplies by the sigmoid of the gate.
template <typename T>
__global__ void __launch_bounds__(64) talk_mix_kernel(T* __restrict__ out, int64_t out_stride, const float* __restrict__ applied, int64_t plane,
                                                      const int32_t* __restrict__ positions, int heads, int kv_heads, int dv,
                                                      const float* __restrict__ talk, const float* __restrict__ cos_v, const float* __restrict__ sin_v,
                                                      const T* __restrict__ gate, int64_t gate_stride) {
  const int t = blockIdx.x, h = blockIdx.y, half = dv / 2, per = heads / kv_heads;
  const float* rows = applied + static_cast<int64_t>(h / per) * plane + static_cast<int64_t>(t) * heads * dv;
  const float* mix = talk ? talk + h * heads : nullptr;
  for (int i = threadIdx.x; i < half; i += 64) {
    const float* src = rows + i;
    float x0 = 0.f, x1 = 0.f;
    int g = 0;
    for (; g + 4 <= heads; g += 4) {      // (four heads' loads on their way together; the sums in ascending order of g)
      float a[4], b[4], w[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        a[u] = src[(g + u) * dv];
        b[u] = src[(g + u) * dv + half];
        w[u] = mix ? mix[g + u] : (g + u == h ? 1.f : 0.f);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        x0 += w[u] * a[u];
        x1 += w[u] * b[u];
      }
    }
    for (; g < heads; ++g) {
      const float w = mix ? mix[g] : (g == h ? 1.f : 0.f);
      x0 += w * src[g * dv];
      x1 += w * src[g * dv + half];
    }
    float y0 = x0, y1 = x1;
    if (cos_v) {
      const int p = positions[t];
      const float cs = cos_v[static_cast<int64_t>(p) * half + i], sn = sin_v[static_cast<int64_t>(p) * half + i];
      y0 = x0 * cs + x1 * sn;
      y1 = x1 * cs - x0 * sn;
    }
    const int64_t at = static_cast<int64_t>(h) * dv + i;
    if (gate) {
      y0 = y0 / (1.f + expf(-load_f32(gate + static_cast<int64_t>(t) * gate_stride + at)));
      y1 = y1 / (1.f + expf(-load_f32(gate + static_cast<int64_t>(t) * gate_stride + at + half)));
    }
    store_f32(out + static_cast<int64_t>(t) * out_stride + at, y0);
    store_f32(out + static_cast<int64_t>(t) * out_stride + at + half, y1);
  }
}

}  // namespace alofa

using namespace alofa;

extern "C" int alofa_talk_mix(void* out, int64_t out_stride, int dtype, const float* applied, const int32_t* positions, int tokens, int heads, int kv_heads, int dv,
                              const float* talk, const float* cos_v, const float* sin_v, const void* gate, int64_t gate_stride, hipStream_t stream) {
  ALOFA_REQUIRE(tokens >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dv > 0 && dv % 2 == 0, "talk_mix: tokens=%d heads=%d kv_heads=%d dv=%d (kv_heads divides heads; an even value size)", tokens, heads, kv_heads, dv);
  ALOFA_REQUIRE(!cos_v || (sin_v && positions), "talk_mix: turning back needs cos, sin and positions");
  if (tokens == 0) return 0;
  const int64_t plane = static_cast<int64_t>(tokens) * heads * dv;
  if (dtype == kF32) talk_mix_kernel<float><<<dim3(tokens, heads), 64, 0, stream>>>(static_cast<float*>(out), out_stride, applied, plane, positions, heads, kv_heads, dv, talk, cos_v, sin_v, static_cast<const float*>(gate), gate_stride);
  else talk_mix_kernel<bf16_t><<<dim3(tokens, heads), 64, 0, stream>>>(static_cast<bf16_t*>(out), out_stride, applied, plane, positions, heads, kv_heads, dv, talk, cos_v, sin_v, static_cast<const bf16_t*>(gate), gate_stride);
  return check_launch("talk_mix");
}

extern "C" int alofa_turn_norm_write(void* qkv, int64_t stride, int dtype, const int32_t* positions, const float* cos_qk, const float* sin_qk, int half_qk,
                                     const float* cos_v, const float* sin_v, const int64_t* slots, void* k_cache, void* v_cache, int block_size,
                                     int tokens, int heads, int kv_heads, int d, int dv, float eps, int unit_norm, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(tokens >= 0 && heads > 0 && kv_heads >= 0 && d > 0 && d <= 256 && dv > 0 && dv <= 256 && dv % 2 == 0, "turn_norm_write: bad sizes (heads=%d kv_heads=%d d=%d dv=%d; heads of up to 256 channels, an even value size)", heads, kv_heads, d, dv);
  ALOFA_REQUIRE(half_qk >= 0 && 2 * half_qk <= d && half_qk <= 128, "turn_norm_write: %d pairs do not fit a head of %d channels", half_qk, d);
  ALOFA_REQUIRE(kv_heads == 0 || (slots && k_cache && v_cache && block_size > 0 && cos_v && sin_v), "turn_norm_write: keys and values need slots, caches and the values' table");
  ALOFA_REQUIRE(!exact || dtype == kF32, "turn_norm_write: the exact path is float32");
  if (tokens == 0) return 0;
  const unsigned grid = static_cast<unsigned>((static_cast<int64_t>(tokens) * (heads + 2 * kv_heads) + 3) / 4);
#define ALOFA_TURN(T, ACC) turn_norm_write_kernel<T, ACC><<<grid, 256, 0, stream>>>(static_cast<T*>(qkv), stride, positions, cos_qk, sin_qk, half_qk, cos_v, sin_v, slots, \
    static_cast<T*>(k_cache), static_cast<T*>(v_cache), block_size, tokens, heads, kv_heads, d, dv, eps, unit_norm)
  if (exact) ALOFA_TURN(float, double);
  else if (dtype == kF32) ALOFA_TURN(float, float);
  else ALOFA_TURN(bf16_t, float);
#undef ALOFA_TURN
  return check_launch("turn_norm_write");
}

static inline size_t talking_lds(int heads, int d, int dv, size_t acc) {
  return (static_cast<size_t>(heads) * d + static_cast<size_t>(heads) * heads + 2 * static_cast<size_t>(heads) * kWave + static_cast<size_t>(heads) * dv) * sizeof(float) + 2 * heads * acc + 16;
}

extern "C" int alofa_talking_attention(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k_cache, const void* v_cache, int dtype,
                                       const int32_t* block_table, int max_blocks, const int32_t* req_of_token, const int32_t* positions, int tokens,
                                       int heads, int kv_heads, int d, int dv, int block_size, int window, float scale, const float* talk,
                                       const float* cos_v, const float* sin_v, const void* gate, int64_t gate_stride, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(tokens >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "talking_attention: tokens=%d heads=%d kv_heads=%d (kv_heads must divide heads)", tokens, heads, kv_heads);
  ALOFA_REQUIRE(d > 0 && dv > 0 && dv % 2 == 0 && heads * dv <= 256 * kTalkOwn, "talking_attention: head sizes %d and %d (an even value size; heads x value size at most %d)", d, dv, 256 * kTalkOwn);
  ALOFA_REQUIRE(block_size > 0 && max_blocks > 0 && window >= 0, "talking_attention: block_size=%d max_blocks=%d window=%d", block_size, max_blocks, window);
  ALOFA_REQUIRE(!exact || dtype == kF32, "talking_attention: the exact path is float32");
  if (tokens == 0) return 0;
  const size_t lds = talking_lds(heads, d, dv, exact ? sizeof(double) : sizeof(float));
  ALOFA_REQUIRE(lds <= 160 * 1024, "talking_attention: %d heads of %d and %d channels need %zu bytes of LDS a block (at most 163840)", heads, d, dv, lds);
  // (more than 64 KB of a compute unit's 160 KB: the kernel has to be told)
#define ALOFA_TALK(T, ACC) do { \
  if (lds > 64 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void*>(&talking_attention_kernel<T, ACC>), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)) != hipSuccess) { \
    (void)hipGetLastError(); \
    ALOFA_REQUIRE(false, "talking_attention: %zu bytes of LDS a block were refused", lds); \
  } \
  talking_attention_kernel<T, ACC><<<tokens, 256, lds, stream>>>(static_cast<T*>(out), out_stride, static_cast<const T*>(q), q_stride, static_cast<const T*>(k_cache), \
    static_cast<const T*>(v_cache), block_table, max_blocks, req_of_token, positions, heads, kv_heads, d, dv, block_size, window, scale, talk, cos_v, sin_v, static_cast<const T*>(gate), gate_stride); } while (0)
  if (exact) ALOFA_TALK(float, double);
  else if (dtype == kF32) ALOFA_TALK(float, float);
  else ALOFA_TALK(bf16_t, float);
#undef ALOFA_TALK
  return check_launch("talking_attention");
}
