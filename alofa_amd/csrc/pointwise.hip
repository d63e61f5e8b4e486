// Row-wise and element-wise kernels of layers that are not plain pre-norm attention blocks: layer norm
// with weight and bias, a per-head unit norm with gate, the xIELU and tanh activations, the weighted
// average over the outputs of all earlier layers, a scaled sum of two branches into the residual
// stream, and a scale.
//
// Acc = double is the exact path (float32 storage, float64 sums and one rounding at the end);
// otherwise sums are float. Norms, gates and averages are float arithmetic in both; only the
// results that feed a matrix product are rounded to the activation type.
#include "common.h"

namespace alofa {

// ---- layer norm ------------------------------------------------------------------------------
// y = (x - mean) / sqrt(var + eps) * w + b per row, var = mean of the squared deviations (taken in a
// second pass over the row, not from the mean of squares). Row r of the output is made from row
// rows[r] of x when `rows` is given. out may be x itself (float): every element is read by the
// thread that writes it, after the block has finished both sums.
template <typename TO, typename Acc>
__global__ void __launch_bounds__(256) layernorm_kernel(TO* __restrict__ out, const float* x, const float* __restrict__ w,
                                                        const float* __restrict__ b, const int32_t* __restrict__ rows,
                                                        int width, float eps, float out_scale) {
  __shared__ Acc scratch[4];
  const int r = blockIdx.x;
  const float* src = x + static_cast<int64_t>(rows ? rows[r] : r) * width;
  TO* dst = out + static_cast<int64_t>(r) * width;
  Acc s = 0;
  for (int c = threadIdx.x; c < width; c += 256) s += static_cast<Acc>(src[c]);
  const Acc mean = block_sum<Acc, 256>(s, scratch) / static_cast<Acc>(width);
  Acc ss = 0;
  for (int c = threadIdx.x; c < width; c += 256) {
    const Acc d = static_cast<Acc>(src[c]) - mean;
    ss += d * d;
  }
  const Acc var = block_sum<Acc, 256>(ss, scratch) / static_cast<Acc>(width);
  const Acc inv = static_cast<Acc>(1) / sqrt(var + static_cast<Acc>(eps));
  for (int c = threadIdx.x; c < width; c += 256) {
    const Acc y = (static_cast<Acc>(src[c]) - mean) * inv * static_cast<Acc>(w[c]) + static_cast<Acc>(b[c]);
    store_f32(dst + c, static_cast<float>(y * static_cast<Acc>(out_scale)));
  }
}

// residual[r] += layer norm of x[r] (weight, bias): the norm behind a sub-layer, on its way into the stream.
template <typename Acc>
__global__ void __launch_bounds__(256) layernorm_add_kernel(float* __restrict__ residual, const float* __restrict__ x, const float* __restrict__ w,
                                                            const float* __restrict__ b, int width, float eps) {
  __shared__ Acc scratch[4];
  const int r = blockIdx.x;
  const float* src = x + static_cast<int64_t>(r) * width;
  float* dst = residual + static_cast<int64_t>(r) * width;
  Acc s = 0;
  for (int c = threadIdx.x; c < width; c += 256) s += static_cast<Acc>(src[c]);
  const Acc mean = block_sum<Acc, 256>(s, scratch) / static_cast<Acc>(width);
  Acc ss = 0;
  for (int c = threadIdx.x; c < width; c += 256) {
    const Acc d = static_cast<Acc>(src[c]) - mean;
    ss += d * d;
  }
  const Acc var = block_sum<Acc, 256>(ss, scratch) / static_cast<Acc>(width);
  const Acc inv = static_cast<Acc>(1) / sqrt(var + static_cast<Acc>(eps));
  for (int c = threadIdx.x; c < width; c += 256) {
    const Acc y = (static_cast<Acc>(src[c]) - mean) * inv * static_cast<Acc>(w[c]) + static_cast<Acc>(b[c]);
    dst[c] = static_cast<float>(static_cast<Acc>(dst[c]) + y);
  }
}

// The same, and then the layer norm (w2, b2) of the row as it now stands, left in `out`: the norm behind one sub-layer and the one in front
// of the next in one launch. Every thread reads back what it wrote itself; the sums are those of the two kernels run one after the other.
template <typename TO, typename Acc>
__global__ void __launch_bounds__(256) layernorm_add_norm_kernel(float* __restrict__ residual, const float* __restrict__ x, const float* __restrict__ w,
                                                                 const float* __restrict__ b, float eps, TO* __restrict__ out, const float* __restrict__ w2,
                                                                 const float* __restrict__ b2, float eps2, int width) {
  __shared__ Acc scratch[4];
  const int r = blockIdx.x;
  const float* src = x + static_cast<int64_t>(r) * width;
  float* dst = residual + static_cast<int64_t>(r) * width;
  Acc s = 0;
  for (int c = threadIdx.x; c < width; c += 256) s += static_cast<Acc>(src[c]);
  const Acc mean = block_sum<Acc, 256>(s, scratch) / static_cast<Acc>(width);
  Acc ss = 0;
  for (int c = threadIdx.x; c < width; c += 256) {
    const Acc d = static_cast<Acc>(src[c]) - mean;
    ss += d * d;
  }
  const Acc var = block_sum<Acc, 256>(ss, scratch) / static_cast<Acc>(width);
  const Acc inv = static_cast<Acc>(1) / sqrt(var + static_cast<Acc>(eps));
  Acc s2 = 0;
  for (int c = threadIdx.x; c < width; c += 256) {
    const Acc y = (static_cast<Acc>(src[c]) - mean) * inv * static_cast<Acc>(w[c]) + static_cast<Acc>(b[c]);
    const float now = static_cast<float>(static_cast<Acc>(dst[c]) + y);
    dst[c] = now;
    s2 += static_cast<Acc>(now);
  }
  const Acc mean2 = block_sum<Acc, 256>(s2, scratch) / static_cast<Acc>(width);
  Acc ss2 = 0;
  for (int c = threadIdx.x; c < width; c += 256) {
    const Acc d = static_cast<Acc>(dst[c]) - mean2;
    ss2 += d * d;
  }
  const Acc var2 = block_sum<Acc, 256>(ss2, scratch) / static_cast<Acc>(width);
  const Acc inv2 = static_cast<Acc>(1) / sqrt(var2 + static_cast<Acc>(eps2));
  TO* normed = out + static_cast<int64_t>(r) * width;
  for (int c = threadIdx.x; c < width; c += 256)
    store_f32(normed + c, static_cast<float>((static_cast<Acc>(dst[c]) - mean2) * inv2 * static_cast<Acc>(w2[c]) + static_cast<Acc>(b2[c])));
}

// out[t, c] += w[t] * x[t, c]: a row handed on with a weight of its own (float rows out, rows of any type in).
template <typename T, typename Acc>
__global__ void __launch_bounds__(256) add_row_scaled_kernel(float* __restrict__ out, const T* __restrict__ x, int64_t x_stride, const float* __restrict__ w,
                                                             int64_t rows, int width) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= rows * width) return;
  const int64_t r = idx / width;
  const float wr = w[r];
  if (wr == 0.f) return;
  out[idx] = static_cast<float>(static_cast<Acc>(out[idx]) + static_cast<Acc>(wr) * static_cast<Acc>(load_f32(x + r * x_stride + idx % width)));
}

// ---- per-head unit norm, weight and gate -------------------------------------------------------
// out[t, h, :] = o[t, h, :] / sqrt(mean_j o[t, h, j]^2 + eps) * w[h, :] * silu(g[t, h, :]); w may be
// absent. One wavefront per (token, head). o is float (what a recurrence or attention left); g and
// out have the activation type. `sigmoid_gate`: the gate is sigmoid(g) instead of silu(g). `extra`: a head of o holds so
// many more channels behind its dv; with `floor` [tokens, heads] the first of them is a normaliser: the head's dv values
// are divided by max(|it|, floor[t, h]) + 1e-6 before the norm.
template <typename T, typename Acc>
__global__ void __launch_bounds__(256) headnorm_gate_kernel(T* __restrict__ out, int64_t out_stride, const float* __restrict__ o,
                                                            const T* __restrict__ g, int64_t g_stride, const float* __restrict__ w,
                                                            int tokens, int heads, int dv, float eps, float out_scale, int parts, int64_t part_stride,
                                                            int sigmoid_gate, int extra, const float* __restrict__ floor) {
  const int64_t unit = static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / kWave;
  if (unit >= static_cast<int64_t>(tokens) * heads) return;
  const int lane = threadIdx.x % kWave;
  const int t = static_cast<int>(unit / heads), h = static_cast<int>(unit % heads);
  const float* src = o + (static_cast<int64_t>(t) * heads + h) * (dv + extra);
  float under = 1.f;      // what the head's values are divided by first
  if (floor) {
    float n = 0.f;
    for (int p = 0; p < parts; ++p) n += src[p * part_stride + dv];
    under = fmaxf(fabsf(n), floor[static_cast<int64_t>(t) * heads + h]) + 1e-6f;
  }
  // (o may come in parts, left by blocks that each held a share of the key channels: they are added here, in their order)
  constexpr int kOwn = 4;      // values a lane keeps between the sum of squares and the scaling (heads up to 256 wide; wider ones are added again)
  float own[kOwn];
  Acc ss = 0;
#pragma unroll
  for (int c = 0; c < kOwn; ++c) {
    const int j = lane + c * kWave;
    float v = 0.f;
    if (j < dv)
      for (int p = 0; p < parts; ++p) v += src[p * part_stride + j];
    if (floor) v /= under;
    own[c] = v;
    ss += static_cast<Acc>(v) * static_cast<Acc>(v);
  }
  for (int j = lane + kOwn * kWave; j < dv; j += kWave) {
    float v = 0.f;
    for (int p = 0; p < parts; ++p) v += src[p * part_stride + j];
    if (floor) v /= under;
    ss += static_cast<Acc>(v) * static_cast<Acc>(v);
  }
  ss = wave_sum(ss);
  const Acc inv = static_cast<Acc>(1) / sqrt(ss / static_cast<Acc>(dv) + static_cast<Acc>(eps));
  const T* gate = g + static_cast<int64_t>(t) * g_stride + static_cast<int64_t>(h) * dv;
  T* dst = out + static_cast<int64_t>(t) * out_stride + static_cast<int64_t>(h) * dv;
  for (int j = lane; j < dv; j += kWave) {
    const Acc z = static_cast<Acc>(load_f32(gate + j));
    const Acc silu = (sigmoid_gate ? static_cast<Acc>(1) : z) / (static_cast<Acc>(1) + exp(-z));
    float v = 0.f;
    if (j < kOwn * kWave) {
#pragma unroll
      for (int c = 0; c < kOwn; ++c)
        if (j == lane + c * kWave) v = own[c];
    } else {
      for (int p = 0; p < parts; ++p) v += src[p * part_stride + j];
      if (floor) v /= under;
    }
    Acc y = static_cast<Acc>(v) * inv;
    if (w) y *= static_cast<Acc>(w[h * dv + j]);
    store_f32(dst + j, static_cast<float>(y * silu * static_cast<Acc>(out_scale)));
  }
}

// The same for wide heads (several heads normed together as one row, say): a block of 256 threads per (token, head), the sum of squares over
// the lanes of each wave and then over the four waves in their order.
template <typename T, typename Acc>
__global__ void __launch_bounds__(256) headnorm_gate_wide_kernel(T* __restrict__ out, int64_t out_stride, const float* __restrict__ o,
                                                                 const T* __restrict__ g, int64_t g_stride, const float* __restrict__ w,
                                                                 int tokens, int heads, int dv, float eps, float out_scale, int parts, int64_t part_stride,
                                                                 int sigmoid_gate, int extra, const float* __restrict__ floor) {
  __shared__ Acc wave_ss[4];
  const int64_t unit = blockIdx.x;
  const int t = static_cast<int>(unit / heads), h = static_cast<int>(unit % heads);
  const float* src = o + (static_cast<int64_t>(t) * heads + h) * (dv + extra);
  float under = 1.f;
  if (floor) {
    float n = 0.f;
    for (int p = 0; p < parts; ++p) n += src[p * part_stride + dv];
    under = fmaxf(fabsf(n), floor[static_cast<int64_t>(t) * heads + h]) + 1e-6f;
  }
  constexpr int kOwn = 8;      // values a thread keeps between the sum of squares and the scaling (rows up to 2,048 wide; wider ones are added again)
  float own[kOwn];
  Acc ss = 0;
  auto value = [&](int j) {
    float v = 0.f;
    for (int p = 0; p < parts; ++p) v += src[p * part_stride + j];
    return floor ? v / under : v;
  };
#pragma unroll
  for (int c = 0; c < kOwn; ++c) {
    const int j = threadIdx.x + c * 256;
    own[c] = j < dv ? value(j) : 0.f;
    ss += static_cast<Acc>(own[c]) * static_cast<Acc>(own[c]);
  }
  for (int j = threadIdx.x + kOwn * 256; j < dv; j += 256) {
    const float v = value(j);
    ss += static_cast<Acc>(v) * static_cast<Acc>(v);
  }
  ss = wave_sum(ss);
  if (threadIdx.x % kWave == 0) wave_ss[threadIdx.x / kWave] = ss;
  __syncthreads();
  ss = ((wave_ss[0] + wave_ss[1]) + wave_ss[2]) + wave_ss[3];
  const Acc inv = static_cast<Acc>(1) / sqrt(ss / static_cast<Acc>(dv) + static_cast<Acc>(eps));
  const T* gate = g + static_cast<int64_t>(t) * g_stride + static_cast<int64_t>(h) * dv;
  T* dst = out + static_cast<int64_t>(t) * out_stride + static_cast<int64_t>(h) * dv;
  auto leave = [&](int j, float v) {
    const Acc z = static_cast<Acc>(load_f32(gate + j));
    const Acc silu = (sigmoid_gate ? static_cast<Acc>(1) : z) / (static_cast<Acc>(1) + exp(-z));
    Acc y = static_cast<Acc>(v) * inv;
    if (w) y *= static_cast<Acc>(w[h * dv + j]);
    store_f32(dst + j, static_cast<float>(y * silu * static_cast<Acc>(out_scale)));
  };
#pragma unroll
  for (int c = 0; c < kOwn; ++c) {
    const int j = threadIdx.x + c * 256;
    if (j < dv) leave(j, own[c]);
  }
  for (int j = threadIdx.x + kOwn * 256; j < dv; j += 256) leave(j, value(j));
}

// ---- activations -------------------------------------------------------------------------------
// kind 0: xIELU with a = softplus(p) and b = 1/2 + softplus(q) given: z > 0: a z^2 + z/2; else b (exp(z) - 1 - z) + z/2.
// kind 1: tanh. kind 2: silu, z sigmoid(z). kind 3: the tanh form of gelu, z/2 (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))).
// In place or not; rows of `width` values with a row stride.
template <typename T, typename Acc>
__global__ void __launch_bounds__(256) activation_kernel(T* __restrict__ out, int64_t out_stride, const T* __restrict__ x, int64_t x_stride,
                                                         int64_t rows, int width, int kind, float a, float b) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= rows * width) return;
  const int64_t r = idx / width;
  const int c = static_cast<int>(idx % width);
  const Acc z = static_cast<Acc>(load_f32(x + r * x_stride + c));
  Acc y;
  if (kind == 0) {
    y = z > 0 ? static_cast<Acc>(a) * z * z + z / 2 : static_cast<Acc>(b) * (expm1(z) - z) + z / 2;
  } else if (kind == 1) {
    y = tanh(z);
  } else if (kind == 2) {
    y = z / (static_cast<Acc>(1) + exp(-z));
  } else {
    y = z / 2 * (static_cast<Acc>(1) + tanh(static_cast<Acc>(0.7978845608028654) * (z + static_cast<Acc>(0.044715) * z * z * z)));
  }
  store_f32(out + r * out_stride + c, static_cast<float>(y));
}

// ---- weighted average over depth -----------------------------------------------------------------
// stack[n - 1] = x; then x = sum_{j < n} w[j] * stack[j], j ascending. stack is [levels, elements].
// Without weights only the copy is made (the first level: what the layers start from).
template <typename Acc>
__global__ void __launch_bounds__(256) depth_average_kernel(float* __restrict__ x, float* __restrict__ stack, int64_t level_stride,
                                                            const float* __restrict__ w, int n, int64_t elements) {
  const int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (e >= elements) return;
  const float mine = x[e];
  stack[static_cast<int64_t>(n - 1) * level_stride + e] = mine;
  if (w == nullptr) return;
  Acc acc = 0;
  for (int j = 0; j < n - 1; ++j) acc += static_cast<Acc>(w[j]) * static_cast<Acc>(stack[static_cast<int64_t>(j) * level_stride + e]);
  acc += static_cast<Acc>(w[n - 1]) * static_cast<Acc>(mine);
  x[e] = static_cast<float>(acc);
}

// ---- residual += a * x + b * y; x *= s --------------------------------------------------------------
template <typename Acc>
__global__ void __launch_bounds__(256) add_scaled_kernel(float* __restrict__ residual, const float* __restrict__ x, float a,
                                                         const float* __restrict__ y, float b, int64_t elements) {
  const int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (e >= elements) return;
  Acc acc = static_cast<Acc>(a) * static_cast<Acc>(x[e]);
  if (y) acc += static_cast<Acc>(b) * static_cast<Acc>(y[e]);
  residual[e] = static_cast<float>(static_cast<Acc>(residual[e]) + acc);
}

__global__ void __launch_bounds__(256) scale_kernel(float* __restrict__ x, float s, int64_t elements) {
  const int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (e < elements) x[e] *= s;
}

}  // namespace alofa

using namespace alofa;

static inline unsigned blocks_of(int64_t n) { return static_cast<unsigned>((n + 255) / 256); }

extern "C" int alofa_layernorm(void* out, int out_dtype, const float* x, const float* w, const float* b, const int32_t* rows,
                               int n_rows, int width, float eps, float out_scale, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(n_rows >= 0 && width > 0 && eps > 0.f, "layernorm: bad sizes (rows=%d width=%d eps=%g)", n_rows, width, eps);
  ALOFA_REQUIRE(!exact || out_dtype == kF32, "layernorm: the exact path writes float32");
  if (n_rows == 0) return 0;
  if (exact) layernorm_kernel<float, double><<<n_rows, 256, 0, stream>>>(static_cast<float*>(out), x, w, b, rows, width, eps, out_scale);
  else if (out_dtype == kF32) layernorm_kernel<float, float><<<n_rows, 256, 0, stream>>>(static_cast<float*>(out), x, w, b, rows, width, eps, out_scale);
  else layernorm_kernel<bf16_t, float><<<n_rows, 256, 0, stream>>>(static_cast<bf16_t*>(out), x, w, b, rows, width, eps, out_scale);
  return check_launch("layernorm");
}

extern "C" int alofa_layernorm_add(float* residual, const float* x, const float* w, const float* b, int n_rows, int width, float eps, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(n_rows >= 0 && width > 0 && eps > 0.f, "layernorm_add: bad sizes (rows=%d width=%d)", n_rows, width);
  if (n_rows == 0) return 0;
  if (exact) layernorm_add_kernel<double><<<n_rows, 256, 0, stream>>>(residual, x, w, b, width, eps);
  else layernorm_add_kernel<float><<<n_rows, 256, 0, stream>>>(residual, x, w, b, width, eps);
  return check_launch("layernorm_add");
}

extern "C" int alofa_layernorm_add_norm(float* residual, const float* x, const float* w, const float* b, float eps, void* out, int out_dtype, const float* w2,
                                        const float* b2, float eps2, int n_rows, int width, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(n_rows >= 0 && width > 0 && eps > 0.f && eps2 > 0.f, "layernorm_add_norm: bad sizes (rows=%d width=%d)", n_rows, width);
  ALOFA_REQUIRE(!exact || out_dtype == kF32, "layernorm_add_norm: the exact path is float32");
  if (n_rows == 0) return 0;
  if (exact) layernorm_add_norm_kernel<float, double><<<n_rows, 256, 0, stream>>>(residual, x, w, b, eps, static_cast<float*>(out), w2, b2, eps2, width);
  else if (out_dtype == kF32) layernorm_add_norm_kernel<float, float><<<n_rows, 256, 0, stream>>>(residual, x, w, b, eps, static_cast<float*>(out), w2, b2, eps2, width);
  else layernorm_add_norm_kernel<bf16_t, float><<<n_rows, 256, 0, stream>>>(residual, x, w, b, eps, static_cast<bf16_t*>(out), w2, b2, eps2, width);
  return check_launch("layernorm_add_norm");
}

extern "C" int alofa_add_row_scaled(float* out, const void* x, int64_t x_stride, int dtype, const float* w, int64_t rows, int width, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(rows >= 0 && width > 0, "add_row_scaled: bad sizes");
  if (rows == 0) return 0;
  const unsigned grid = static_cast<unsigned>((rows * width + 255) / 256);
  if (exact && dtype == kF32) add_row_scaled_kernel<float, double><<<grid, 256, 0, stream>>>(out, static_cast<const float*>(x), x_stride, w, rows, width);
  else if (dtype == kF32) add_row_scaled_kernel<float, float><<<grid, 256, 0, stream>>>(out, static_cast<const float*>(x), x_stride, w, rows, width);
  else add_row_scaled_kernel<bf16_t, float><<<grid, 256, 0, stream>>>(out, static_cast<const bf16_t*>(x), x_stride, w, rows, width);
  return check_launch("add_row_scaled");
}

extern "C" int alofa_headnorm_gate(void* out, int64_t out_stride, const float* o, const void* g, int64_t g_stride, int dtype, const float* w,
                                   int tokens, int heads, int dv, float eps, float out_scale, int parts, int64_t part_stride, int exact,
                                   int sigmoid_gate, int extra, const float* floor, hipStream_t stream) {
  ALOFA_REQUIRE(extra >= 0 && (!floor || extra >= 1), "headnorm_gate: a normaliser needs a channel behind the head's own");
  ALOFA_REQUIRE(tokens >= 0 && heads > 0 && dv > 0 && eps > 0.f && parts >= 1, "headnorm_gate: bad sizes (tokens=%d heads=%d dv=%d)", tokens, heads, dv);
  ALOFA_REQUIRE(!exact || dtype == kF32, "headnorm_gate: the exact path is float32");
  if (tokens == 0) return 0;
  if (dv > 256) {      // wide rows: a block each
    const unsigned units = static_cast<unsigned>(static_cast<int64_t>(tokens) * heads);
    if (exact) headnorm_gate_wide_kernel<float, double><<<units, 256, 0, stream>>>(static_cast<float*>(out), out_stride, o, static_cast<const float*>(g), g_stride, w, tokens, heads, dv, eps, out_scale, parts, part_stride, sigmoid_gate, extra, floor);
    else if (dtype == kF32) headnorm_gate_wide_kernel<float, float><<<units, 256, 0, stream>>>(static_cast<float*>(out), out_stride, o, static_cast<const float*>(g), g_stride, w, tokens, heads, dv, eps, out_scale, parts, part_stride, sigmoid_gate, extra, floor);
    else headnorm_gate_wide_kernel<bf16_t, float><<<units, 256, 0, stream>>>(static_cast<bf16_t*>(out), out_stride, o, static_cast<const bf16_t*>(g), g_stride, w, tokens, heads, dv, eps, out_scale, parts, part_stride, sigmoid_gate, extra, floor);
    return check_launch("headnorm_gate");
  }
  const unsigned grid = static_cast<unsigned>((static_cast<int64_t>(tokens) * heads + 3) / 4);
  if (exact) headnorm_gate_kernel<float, double><<<grid, 256, 0, stream>>>(static_cast<float*>(out), out_stride, o, static_cast<const float*>(g), g_stride, w, tokens, heads, dv, eps, out_scale, parts, part_stride, sigmoid_gate, extra, floor);
  else if (dtype == kF32) headnorm_gate_kernel<float, float><<<grid, 256, 0, stream>>>(static_cast<float*>(out), out_stride, o, static_cast<const float*>(g), g_stride, w, tokens, heads, dv, eps, out_scale, parts, part_stride, sigmoid_gate, extra, floor);
  else headnorm_gate_kernel<bf16_t, float><<<grid, 256, 0, stream>>>(static_cast<bf16_t*>(out), out_stride, o, static_cast<const bf16_t*>(g), g_stride, w, tokens, heads, dv, eps, out_scale, parts, part_stride, sigmoid_gate, extra, floor);
  return check_launch("headnorm_gate");
}

extern "C" int alofa_activation(void* out, int64_t out_stride, const void* x, int64_t x_stride, int dtype, int64_t rows, int width,
                                int kind, float a, float b, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(rows >= 0 && width > 0 && kind >= 0 && kind <= 3, "activation: bad arguments (rows=%lld width=%d kind=%d)", (long long)rows, width, kind);
  ALOFA_REQUIRE(!exact || dtype == kF32, "activation: the exact path is float32");
  if (rows == 0) return 0;
  const unsigned grid = blocks_of(rows * width);
  if (exact) activation_kernel<float, double><<<grid, 256, 0, stream>>>(static_cast<float*>(out), out_stride, static_cast<const float*>(x), x_stride, rows, width, kind, a, b);
  else if (dtype == kF32) activation_kernel<float, float><<<grid, 256, 0, stream>>>(static_cast<float*>(out), out_stride, static_cast<const float*>(x), x_stride, rows, width, kind, a, b);
  else activation_kernel<bf16_t, float><<<grid, 256, 0, stream>>>(static_cast<bf16_t*>(out), out_stride, static_cast<const bf16_t*>(x), x_stride, rows, width, kind, a, b);
  return check_launch("activation");
}

extern "C" int alofa_depth_average(float* x, float* stack, int64_t level_stride, const float* w, int n, int64_t elements, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(n >= 1 && elements >= 0 && level_stride >= elements, "depth_average: bad sizes (n=%d elements=%lld stride=%lld)", n, (long long)elements, (long long)level_stride);
  if (elements == 0) return 0;
  if (exact) depth_average_kernel<double><<<blocks_of(elements), 256, 0, stream>>>(x, stack, level_stride, w, n, elements);
  else depth_average_kernel<float><<<blocks_of(elements), 256, 0, stream>>>(x, stack, level_stride, w, n, elements);
  return check_launch("depth_average");
}

extern "C" int alofa_add_scaled(float* residual, const float* x, float a, const float* y, float b, int64_t elements, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(elements >= 0 && x != nullptr, "add_scaled: bad arguments");
  if (elements == 0) return 0;
  if (exact) add_scaled_kernel<double><<<blocks_of(elements), 256, 0, stream>>>(residual, x, a, y, b, elements);
  else add_scaled_kernel<float><<<blocks_of(elements), 256, 0, stream>>>(residual, x, a, y, b, elements);
  return check_launch("add_scaled");
}

extern "C" int alofa_scale(float* x, float s, int64_t elements, hipStream_t stream) {
  ALOFA_REQUIRE(elements >= 0, "scale: bad size");
  if (elements == 0) return 0;
  scale_kernel<<<blocks_of(elements), 256, 0, stream>>>(x, s, elements);
  return check_launch("scale");
}

// =================================================================================================
// Kernels of designs whose sub-layers are scaled channel by channel on their way into the stream,
// whose embedding adds a row named by a hash of two tokens, and whose stream is joined with the
// embedding's output by a projection.
namespace alofa {

// ---- token row times a factor, plus the row of a second table named by (token before, token) ----------
// out[t] = table[id] * scale + pairs[(before * mul_prev + id * mul_cur) mod buckets]; for a request's first token
// (position 0) the row `buckets`. The token before row t is row t - 1's within a request's rows, and for the first
// row of a request in this step what `state` holds for its slot. The block of a request's first row then leaves the
// request's last token of this step there (it alone touches the slot: read, barrier, write). Negative ids name tokens
// in `store`, as in embed_gather.
__device__ __forceinline__ int token_at(const int32_t* ids, int t, const int32_t* store, int vocab) {
  int id = ids[t];
  if (id < 0) {
    id = store[-(id + 1)];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  }
  return id;
}

template <typename TW>
__global__ void pair_embed_kernel(float* __restrict__ out, const TW* __restrict__ table, const TW* __restrict__ pairs,
                                  const int32_t* __restrict__ ids, const int32_t* __restrict__ positions, int32_t* state,
                                  const int32_t* __restrict__ req_slot, const int32_t* __restrict__ row_off, const int32_t* __restrict__ req_of_row,
                                  int width, const int32_t* __restrict__ store, int vocab, float scale,
                                  int64_t buckets, int64_t mul_prev, int64_t mul_cur) {
  const int t = blockIdx.x;
  int first = t, last = t, slot = 0;
  if (pairs) {
    const int r = req_of_row ? req_of_row[t] : t;
    if (row_off) first = row_off[r], last = row_off[r + 1] - 1;
    slot = req_slot[r];
  }
  const int id = token_at(ids, t, store, vocab);
  int64_t row = buckets;
  if (pairs && positions[t] != 0) {
    const int64_t before = t == first ? state[slot] : token_at(ids, t - 1, store, vocab);
    row = (before * mul_prev + static_cast<int64_t>(id) * mul_cur) % buckets;
    if (row < 0) row += buckets;
  }
  const TW* a = table + static_cast<int64_t>(id) * width;
  float* dst = out + static_cast<int64_t>(t) * width;
  if (pairs) {
    const TW* b = pairs + row * width;
    for (int c = threadIdx.x; c < width; c += blockDim.x) dst[c] = load_f32(a + c) * scale + load_f32(b + c);
  } else {
    for (int c = threadIdx.x; c < width; c += blockDim.x) dst[c] = load_f32(a + c) * scale;
  }
  if (state && t == first) {
    const int keep = token_at(ids, last, store, vocab);
    __syncthreads();
    if (threadIdx.x == 0) state[slot] = keep;
  }
}

// ---- out[t] = [a[t] | b[t]] in the activation type (two float streams side by side, the operand of one product) ----
template <typename TO>
__global__ void __launch_bounds__(256) concat_rows_kernel(TO* __restrict__ out, const float* __restrict__ a, const float* __restrict__ b, int64_t rows, int width) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= rows * 2 * width) return;
  const int64_t r = idx / (2 * width);
  const int c = static_cast<int>(idx % (2 * width));
  store_f32(out + idx, c < width ? a[r * width + c] : b[r * width + c - width]);
}

// ---- RMSNorm of short rows, left several times side by side ------------------------------------------------
// y = x / sqrt(mean(x^2) + eps) * w of `width` values; out[t, k * pad + j] = y[j] for k < copies, zeros for
// width <= j < pad. One wavefront per row.
template <typename TO, typename Acc, typename TI = float>
__global__ void __launch_bounds__(256) rmsnorm_spread_kernel(TO* __restrict__ out, int64_t out_stride, const TI* __restrict__ x, int64_t x_stride,
                                                             const float* __restrict__ w, int rows, int width, int pad, int copies, float eps) {
  const int t = blockIdx.x * 4 + threadIdx.x / kWave;
  if (t >= rows) return;
  const int lane = threadIdx.x % kWave;
  const TI* src = x + static_cast<int64_t>(t) * x_stride;
  Acc ss = 0;
  for (int j = lane; j < width; j += kWave) ss += static_cast<Acc>(load_f32(src + j)) * static_cast<Acc>(load_f32(src + j));
  ss = wave_sum(ss);
  const Acc inv = static_cast<Acc>(1) / sqrt(ss / static_cast<Acc>(width) + static_cast<Acc>(eps));
  TO* dst = out + static_cast<int64_t>(t) * out_stride;
  for (int j = lane; j < pad; j += kWave) {
    const float y = j < width ? static_cast<float>(static_cast<Acc>(load_f32(src + j)) * inv * static_cast<Acc>(w[j])) : 0.f;
    for (int k = 0; k < copies; ++k) store_f32(dst + static_cast<int64_t>(k) * pad + j, y);
  }
}

// ---- x[t, c] *= sigmoid(g[t, c]) ------------------------------------------------------------------------------
template <typename T, typename Acc>
__global__ void __launch_bounds__(256) sigmoid_gate_kernel(T* __restrict__ x, int64_t x_stride, const T* __restrict__ g, int64_t g_stride, int64_t rows, int width) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= rows * width) return;
  const int64_t r = idx / width;
  const int c = static_cast<int>(idx % width);
  const Acc z = static_cast<Acc>(load_f32(g + r * g_stride + c));
  const Acc s = static_cast<Acc>(1) / (static_cast<Acc>(1) + exp(-z));
  store_f32(x + r * x_stride + c, static_cast<float>(static_cast<Acc>(load_f32(x + r * x_stride + c)) * s));
}

// ---- residual[t, c] += scale[c] * x[t, c] ------------------------------------------------------------------------
template <typename Acc>
__global__ void __launch_bounds__(256) add_channel_scaled_kernel(float* __restrict__ residual, const float* __restrict__ x, const float* __restrict__ scale,
                                                                 int64_t elements, int width) {
  const int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (e >= elements) return;
  residual[e] = static_cast<float>(static_cast<Acc>(residual[e]) + static_cast<Acc>(scale[e % width]) * static_cast<Acc>(x[e]));
}

// ---- residual[t, :] += scale * x[t, :], and normed[t, :] = rmsnorm(residual[t, :]) * w: the sum into the stream and the norm the
// next sub-layer starts with in one pass over the row (a block per row; the row's new values wait in registers) ----
template <typename TO, typename Acc>
__global__ void __launch_bounds__(256) add_channel_scaled_norm_kernel(float* __restrict__ residual, const float* __restrict__ x, const float* __restrict__ scale,
                                                                      TO* __restrict__ normed, const float* __restrict__ w, int width, float eps) {
  __shared__ Acc scratch[4];
  constexpr int kOwn = 8;      // values a thread keeps (rows up to 2,048 wide; wider ones are read again)
  const int64_t at = static_cast<int64_t>(blockIdx.x) * width;
  float own[kOwn];
  Acc ss = 0;
#pragma unroll
  for (int i = 0; i < kOwn; ++i) {
    const int c = threadIdx.x + i * 256;
    own[i] = 0.f;
    if (c < width) {
      own[i] = static_cast<float>(static_cast<Acc>(residual[at + c]) + static_cast<Acc>(scale[c]) * static_cast<Acc>(x[at + c]));
      residual[at + c] = own[i];
      ss += static_cast<Acc>(own[i]) * static_cast<Acc>(own[i]);
    }
  }
  for (int c = threadIdx.x + kOwn * 256; c < width; c += 256) {
    const float v = static_cast<float>(static_cast<Acc>(residual[at + c]) + static_cast<Acc>(scale[c]) * static_cast<Acc>(x[at + c]));
    residual[at + c] = v;
    ss += static_cast<Acc>(v) * static_cast<Acc>(v);
  }
  const Acc inv = static_cast<Acc>(1) / sqrt(block_sum<Acc, 256>(ss, scratch) / static_cast<Acc>(width) + static_cast<Acc>(eps));
#pragma unroll
  for (int i = 0; i < kOwn; ++i) {
    const int c = threadIdx.x + i * 256;
    if (c < width) store_f32(normed + at + c, static_cast<float>(static_cast<Acc>(own[i]) * inv * static_cast<Acc>(w[c])));
  }
  for (int c = threadIdx.x + kOwn * 256; c < width; c += 256)
    store_f32(normed + at + c, static_cast<float>(static_cast<Acc>(residual[at + c]) * inv * static_cast<Acc>(w[c])));
}

// ---- x = cap * tanh(x / cap) ---------------------------------------------------------------------------------------
template <typename Acc>
__global__ void __launch_bounds__(256) softcap_kernel(float* __restrict__ x, float cap, int64_t elements) {
  const int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (e < elements) x[e] = static_cast<float>(static_cast<Acc>(cap) * tanh(static_cast<Acc>(x[e]) / static_cast<Acc>(cap)));
}

// ---- the square of relu --------------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256) relu_squared_kernel(T* __restrict__ out, int64_t out_stride, const T* __restrict__ x, int64_t x_stride, int64_t rows, int width) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= rows * width) return;
  const int64_t r = idx / width;
  const int c = static_cast<int>(idx % width);
  const float z = fmaxf(load_f32(x + r * x_stride + c), 0.f);
  store_f32(out + r * out_stride + c, z * z);
}

}  // namespace alofa

extern "C" int alofa_pair_embed(float* out, const void* table, const void* pairs, int table_dtype, const int32_t* ids, const int32_t* positions, int32_t* state,
                                const int32_t* req_slot, const int32_t* row_off, const int32_t* req_of_row, int tokens, int width, const int32_t* store,
                                int vocab, float scale, int64_t buckets, int64_t mul_prev, int64_t mul_cur, hipStream_t stream) {
  ALOFA_REQUIRE(tokens > 0 && width > 0 && vocab > 0, "pair_embed: tokens=%d width=%d vocab=%d must be positive", tokens, width, vocab);
  ALOFA_REQUIRE(pairs == nullptr || (buckets > 0 && state && positions && req_slot), "pair_embed: a pair table comes with buckets, positions, slots and state");
  ALOFA_REQUIRE((row_off == nullptr) == (req_of_row == nullptr), "pair_embed: row offsets and request indices come together");
  const int threads = width >= 256 ? 256 : 64;
  if (table_dtype == kF32)
    pair_embed_kernel<float><<<tokens, threads, 0, stream>>>(out, static_cast<const float*>(table), static_cast<const float*>(pairs), ids, positions, pairs ? state : nullptr,
                                                             req_slot, row_off, req_of_row, width, store, vocab, scale, buckets, mul_prev, mul_cur);
  else if (table_dtype == kBF16)
    pair_embed_kernel<bf16_t><<<tokens, threads, 0, stream>>>(out, static_cast<const bf16_t*>(table), static_cast<const bf16_t*>(pairs), ids, positions, pairs ? state : nullptr,
                                                              req_slot, row_off, req_of_row, width, store, vocab, scale, buckets, mul_prev, mul_cur);
  else
    ALOFA_REQUIRE(false, "pair_embed: unknown table dtype %d", table_dtype);
  return check_launch("pair_embed");
}

extern "C" int alofa_concat_rows(void* out, int out_dtype, const float* a, const float* b, int64_t rows, int width, hipStream_t stream) {
  ALOFA_REQUIRE(rows >= 0 && width > 0, "concat_rows: bad sizes");
  if (rows == 0) return 0;
  if (out_dtype == kF32) concat_rows_kernel<float><<<blocks_of(rows * 2 * width), 256, 0, stream>>>(static_cast<float*>(out), a, b, rows, width);
  else concat_rows_kernel<bf16_t><<<blocks_of(rows * 2 * width), 256, 0, stream>>>(static_cast<bf16_t*>(out), a, b, rows, width);
  return check_launch("concat_rows");
}

extern "C" int alofa_rmsnorm_spread(void* out, int out_dtype, int64_t out_stride, const void* xv, int x_dtype, int64_t x_stride, const float* w, int rows, int width, int pad,
                                    int copies, float eps, int exact, hipStream_t stream) {
  const float* x = static_cast<const float*>(xv);
  ALOFA_REQUIRE(x_dtype == kF32 || (x_dtype == kBF16 && out_dtype == kBF16 && !exact), "rmsnorm_spread: rows are float32, or bfloat16 with a bfloat16 result");
  ALOFA_REQUIRE(rows >= 0 && width > 0 && pad >= width && copies >= 1 && eps > 0.f && out_stride >= static_cast<int64_t>(copies) * pad && x_stride >= width,
                "rmsnorm_spread: bad sizes (rows=%d width=%d pad=%d copies=%d)", rows, width, pad, copies);
  ALOFA_REQUIRE(!exact || out_dtype == kF32, "rmsnorm_spread: the exact path writes float32");
  if (rows == 0) return 0;
  const unsigned grid = static_cast<unsigned>((rows + 3) / 4);
  if (x_dtype == kBF16) rmsnorm_spread_kernel<bf16_t, float, bf16_t><<<grid, 256, 0, stream>>>(static_cast<bf16_t*>(out), out_stride, static_cast<const bf16_t*>(xv), x_stride, w, rows, width, pad, copies, eps);
  else if (exact) rmsnorm_spread_kernel<float, double><<<grid, 256, 0, stream>>>(static_cast<float*>(out), out_stride, x, x_stride, w, rows, width, pad, copies, eps);
  else if (out_dtype == kF32) rmsnorm_spread_kernel<float, float><<<grid, 256, 0, stream>>>(static_cast<float*>(out), out_stride, x, x_stride, w, rows, width, pad, copies, eps);
  else rmsnorm_spread_kernel<bf16_t, float><<<grid, 256, 0, stream>>>(static_cast<bf16_t*>(out), out_stride, x, x_stride, w, rows, width, pad, copies, eps);
  return check_launch("rmsnorm_spread");
}

extern "C" int alofa_sigmoid_gate(void* x, int64_t x_stride, const void* g, int64_t g_stride, int dtype, int64_t rows, int width, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(rows >= 0 && width > 0, "sigmoid_gate: bad sizes");
  ALOFA_REQUIRE(!exact || dtype == kF32, "sigmoid_gate: the exact path is float32");
  if (rows == 0) return 0;
  const unsigned grid = blocks_of(rows * width);
  if (exact) sigmoid_gate_kernel<float, double><<<grid, 256, 0, stream>>>(static_cast<float*>(x), x_stride, static_cast<const float*>(g), g_stride, rows, width);
  else if (dtype == kF32) sigmoid_gate_kernel<float, float><<<grid, 256, 0, stream>>>(static_cast<float*>(x), x_stride, static_cast<const float*>(g), g_stride, rows, width);
  else sigmoid_gate_kernel<bf16_t, float><<<grid, 256, 0, stream>>>(static_cast<bf16_t*>(x), x_stride, static_cast<const bf16_t*>(g), g_stride, rows, width);
  return check_launch("sigmoid_gate");
}

extern "C" int alofa_add_channel_scaled(float* residual, const float* x, const float* scale, int64_t rows, int width, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(rows >= 0 && width > 0 && scale != nullptr, "add_channel_scaled: bad arguments");
  if (rows == 0) return 0;
  if (exact) add_channel_scaled_kernel<double><<<blocks_of(rows * width), 256, 0, stream>>>(residual, x, scale, rows * width, width);
  else add_channel_scaled_kernel<float><<<blocks_of(rows * width), 256, 0, stream>>>(residual, x, scale, rows * width, width);
  return check_launch("add_channel_scaled");
}

extern "C" int alofa_add_channel_scaled_norm(float* residual, const float* x, const float* scale, void* normed, int normed_dtype, const float* w, int64_t rows,
                                             int width, float eps, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(rows >= 0 && width > 0 && scale && normed && w && eps > 0.f, "add_channel_scaled_norm: bad arguments");
  ALOFA_REQUIRE(!exact || normed_dtype == kF32, "add_channel_scaled_norm: the exact path writes float32");
  if (rows == 0) return 0;
  const unsigned grid = static_cast<unsigned>(rows);
  if (exact) add_channel_scaled_norm_kernel<float, double><<<grid, 256, 0, stream>>>(residual, x, scale, static_cast<float*>(normed), w, width, eps);
  else if (normed_dtype == kF32) add_channel_scaled_norm_kernel<float, float><<<grid, 256, 0, stream>>>(residual, x, scale, static_cast<float*>(normed), w, width, eps);
  else add_channel_scaled_norm_kernel<bf16_t, float><<<grid, 256, 0, stream>>>(residual, x, scale, static_cast<bf16_t*>(normed), w, width, eps);
  return check_launch("add_channel_scaled_norm");
}

extern "C" int alofa_softcap(float* x, float cap, int64_t elements, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(elements >= 0 && cap > 0.f, "softcap: bad arguments");
  if (elements == 0) return 0;
  if (exact) softcap_kernel<double><<<blocks_of(elements), 256, 0, stream>>>(x, cap, elements);
  else softcap_kernel<float><<<blocks_of(elements), 256, 0, stream>>>(x, cap, elements);
  return check_launch("softcap");
}

extern "C" int alofa_relu_squared(void* out, int64_t out_stride, const void* x, int64_t x_stride, int dtype, int64_t rows, int width, hipStream_t stream) {
  ALOFA_REQUIRE(rows >= 0 && width > 0, "relu_squared: bad sizes");
  if (rows == 0) return 0;
  if (dtype == kF32) relu_squared_kernel<float><<<blocks_of(rows * width), 256, 0, stream>>>(static_cast<float*>(out), out_stride, static_cast<const float*>(x), x_stride, rows, width);
  else relu_squared_kernel<bf16_t><<<blocks_of(rows * width), 256, 0, stream>>>(static_cast<bf16_t*>(out), out_stride, static_cast<const bf16_t*>(x), x_stride, rows, width);
  return check_launch("relu_squared");
}
