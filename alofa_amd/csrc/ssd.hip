// A state-space mixer with a scalar decay per head and step (the "state-space duality" form), around the recurrence kernel
// that the other mixers with state of fixed size use:
//
//   conv_bias_act     a short causal convolution per channel with a bias and silu behind it, within each request; the
//                     inputs before a request's first row of this step come from its state (the last taps - 1 inputs).
//   ssd_operands      the recurrence's operands as float32 rows: step size dt = softplus(z + bias) per head, decay
//                     exp(-exp(A_log) dt), keys dt * B and queries C of the head's group, values x.
//   ssd_finish        y = (read-out + D x) * silu(z), an RMS norm over each of several equal parts of the row, a weight.
//   ssd_step          for steps of single rows: conv_bias_act with the state's step in one launch, then ssd_operands.
//   rms_pair_add_norm the sum of two normed branches into the stream, times a factor per channel, and the next norm, one launch.
//   rms_pair_sum      out = sa * rms(a) * wa + sb * rms(b) * wb: two branches, each normed over the width, summed (out may be a or b:
//                     a thread reads what it owns of a row before it writes there).
//
// Softplus, exponentials, step sizes and decays are float32 (double in the exact path), whatever the activations' type.
#include "common.h"

namespace alofa {

static inline unsigned blocks_for(int64_t n) { return static_cast<unsigned>((n + 255) / 256); }

template <typename TO, typename TI, typename Acc>
__global__ void __launch_bounds__(256) conv_bias_act_kernel(TO* __restrict__ out, int64_t out_stride, const TI* __restrict__ x, int64_t x_stride,
                                                            const float* __restrict__ w, const float* __restrict__ bias, const TI* __restrict__ state,
                                                            const int32_t* __restrict__ req_slot, const int32_t* __restrict__ row_off,
                                                            const int32_t* __restrict__ req_of_row, int rows, int width, int taps, int act) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= static_cast<int64_t>(rows) * width) return;
  const int t = static_cast<int>(idx / width), c = static_cast<int>(idx % width);
  const int r = req_of_row ? req_of_row[t] : t;
  const int row0 = row_off ? row_off[r] : r;
  const TI* st = state + static_cast<int64_t>(req_slot[r]) * (taps - 1) * width;
  const float* wc = w + static_cast<int64_t>(c) * taps;
  Acc acc = bias ? static_cast<Acc>(bias[c]) : static_cast<Acc>(0);
  for (int j = 0; j < taps; ++j) {
    const int s = t - taps + 1 + j;
    const Acc v = s >= row0 ? static_cast<Acc>(load_f32(x + static_cast<int64_t>(s) * x_stride + c))
                            : static_cast<Acc>(load_f32(st + static_cast<int64_t>(taps - 1 + s - row0) * width + c));
    acc += static_cast<Acc>(wc[j]) * v;
  }
  if (act) acc = acc / (static_cast<Acc>(1) + exp(-acc));
  store_f32(out + static_cast<int64_t>(t) * out_stride + c, static_cast<float>(acc));
}

// The last `keep` inputs a request has seen once this step's rows are in (rows with a stride; older ones from the state itself).
constexpr int kConvMaxKeep = 15;
template <typename TI>
__global__ void __launch_bounds__(256) conv_keep_kernel(TI* __restrict__ state, const TI* __restrict__ x, int64_t x_stride, const int32_t* __restrict__ req_slot,
                                                        const int32_t* __restrict__ row_off, int requests, int width, int keep) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= static_cast<int64_t>(requests) * width) return;
  const int r = static_cast<int>(idx / width), c = static_cast<int>(idx % width);
  const int row0 = row_off ? row_off[r] : r, end = row_off ? row_off[r + 1] : r + 1;
  TI* st = state + static_cast<int64_t>(req_slot[r]) * keep * width;
  TI kept[kConvMaxKeep];
#pragma unroll
  for (int i = 0; i < kConvMaxKeep; ++i) {
    if (i < keep) {
      const int s = end - keep + i;
      kept[i] = s >= row0 ? x[static_cast<int64_t>(s) * x_stride + c] : st[static_cast<int64_t>(keep + s - row0) * width + c];
    }
  }
#pragma unroll
  for (int i = 0; i < kConvMaxKeep; ++i)
    if (i < keep) st[static_cast<int64_t>(i) * width + c] = kept[i];
}

// A block per (row, head). xbc: the row's x [heads * dv], B [groups * N], C [groups * N] side by side.
template <typename T, typename Acc>
__global__ void __launch_bounds__(128) ssd_operands_kernel(float* __restrict__ qf, float* __restrict__ kf, float* __restrict__ vf, float* __restrict__ decay,
                                                           const T* __restrict__ xbc, int64_t xbc_stride, const T* __restrict__ dt_raw, int64_t dt_stride,
                                                           const float* __restrict__ dt_bias, const float* __restrict__ a_log, int heads, int groups, int N, int dv) {
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, g = h / (heads / groups);
  const Acc z = static_cast<Acc>(load_f32(dt_raw + t * dt_stride + h)) + static_cast<Acc>(dt_bias[h]);
  const Acc dt = (z > 0 ? z : static_cast<Acc>(0)) + log1p(exp(-fabs(z)));      // softplus, no clamp
  const Acc keep = exp(-exp(static_cast<Acc>(a_log[h])) * dt);
  const T* row = xbc + t * xbc_stride;
  const T* B = row + static_cast<int64_t>(heads) * dv + static_cast<int64_t>(g) * N;
  const T* C = B + static_cast<int64_t>(groups) * N;
  const int64_t at_k = (t * heads + h) * N, at_v = (t * heads + h) * dv;
  for (int n = threadIdx.x; n < N; n += 128) {
    qf[at_k + n] = load_f32(C + n);
    kf[at_k + n] = static_cast<float>(dt * static_cast<Acc>(load_f32(B + n)));
    decay[at_k + n] = static_cast<float>(keep);
  }
  for (int c = threadIdx.x; c < dv; c += 128) vf[at_v + c] = load_f32(row + static_cast<int64_t>(h) * dv + c);
}

// A block per (row, part of the row that is normed by itself).
template <typename T, typename Acc>
__global__ void __launch_bounds__(256) ssd_finish_kernel(T* __restrict__ out, int64_t out_stride, const float* __restrict__ o, int parts, int64_t part_stride,
                                                         const T* __restrict__ x, int64_t x_stride, const T* __restrict__ z, int64_t z_stride,
                                                         const float* __restrict__ skip, const float* __restrict__ weight, int heads, int dv, int norm_parts, float eps) {
  __shared__ Acc scratch[4];
  const int64_t t = blockIdx.x;
  const int inner = heads * dv, span = inner / norm_parts, c0 = blockIdx.y * span;
  auto value = [&](int c) -> Acc {
    Acc y = 0;
    for (int p = 0; p < parts; ++p) y += static_cast<Acc>(o[p * part_stride + t * inner + c]);
    y += static_cast<Acc>(skip[c / dv]) * static_cast<Acc>(load_f32(x + t * x_stride + c));
    const Acc g = static_cast<Acc>(load_f32(z + t * z_stride + c));
    return y * (g / (static_cast<Acc>(1) + exp(-g)));
  };
  // (parts of up to 2,048 channels wait in registers between the sum of squares and the scaling; wider ones are formed twice)
  constexpr int kOwn = 8;
  Acc own[kOwn];
  Acc ss = 0;
#pragma unroll
  for (int n = 0; n < kOwn; ++n) {
    const int c = c0 + threadIdx.x + n * 256;
    own[n] = c < c0 + span ? value(c) : static_cast<Acc>(0);
    ss += own[n] * own[n];
  }
  for (int c = c0 + threadIdx.x + kOwn * 256; c < c0 + span; c += 256) {
    const Acc y = value(c);
    ss += y * y;
  }
  ss = block_sum<Acc, 256>(ss, scratch);
  const Acc inv = static_cast<Acc>(1) / sqrt(ss / static_cast<Acc>(span) + static_cast<Acc>(eps));
#pragma unroll
  for (int n = 0; n < kOwn; ++n) {
    const int c = c0 + threadIdx.x + n * 256;
    if (c < c0 + span) store_f32(out + t * out_stride + c, static_cast<float>(own[n] * inv * static_cast<Acc>(weight[c])));
  }
  for (int c = c0 + threadIdx.x + kOwn * 256; c < c0 + span; c += 256)
    store_f32(out + t * out_stride + c, static_cast<float>(value(c) * inv * static_cast<Acc>(weight[c])));
}

// A block per row.
template <typename Acc>
__global__ void __launch_bounds__(256) rms_pair_sum_kernel(float* out, const float* a, const float* __restrict__ wa, float sa,
                                                           const float* b, const float* __restrict__ wb, float sb, int width, float eps) {
  __shared__ Acc scratch[4];
  const int64_t t = blockIdx.x;
  const float* ra = a + t * width;
  const float* rb = b + t * width;
  Acc ssa = 0, ssb = 0;
  for (int c = threadIdx.x; c < width; c += 256) {
    const Acc u = static_cast<Acc>(ra[c]), v = static_cast<Acc>(rb[c]);
    ssa += u * u;
    ssb += v * v;
  }
  ssa = block_sum<Acc, 256>(ssa, scratch);
  ssb = block_sum<Acc, 256>(ssb, scratch);
  const Acc ia = static_cast<Acc>(sa) / sqrt(ssa / static_cast<Acc>(width) + static_cast<Acc>(eps));
  const Acc ib = static_cast<Acc>(sb) / sqrt(ssb / static_cast<Acc>(width) + static_cast<Acc>(eps));
  for (int c = threadIdx.x; c < width; c += 256)
    out[t * width + c] = static_cast<float>(static_cast<Acc>(ra[c]) * ia * static_cast<Acc>(wa[c]) + static_cast<Acc>(rb[c]) * ib * static_cast<Acc>(wb[c]));
}

// residual[t, c] += scale[c] * (sa * rms(a[t]) wa + sb * rms(b[t]) wb)[c], and, where asked, normed[t] = rms(residual[t]) * nw: the sum of two
// normed branches on its way into the stream with the norm that the next sub-layer starts with, one launch. A block per row; a thread
// reads back only what it wrote itself.
template <typename TO, typename Acc>
__global__ void __launch_bounds__(256) rms_pair_add_norm_kernel(float* __restrict__ residual, const float* __restrict__ a, const float* __restrict__ wa, float sa,
                                                                const float* __restrict__ b, const float* __restrict__ wb, float sb, const float* __restrict__ scale,
                                                                int width, float eps, TO* __restrict__ normed, const float* __restrict__ nw, float norm_eps) {
  __shared__ Acc scratch[4];
  const int64_t t = blockIdx.x;
  const float* ra = a + t * width;
  const float* rb = b + t * width;
  float* rr = residual + t * width;
  Acc ssa = 0, ssb = 0;
  for (int c = threadIdx.x; c < width; c += 256) {
    const Acc u = static_cast<Acc>(ra[c]), v = static_cast<Acc>(rb[c]);
    ssa += u * u;
    ssb += v * v;
  }
  ssa = block_sum<Acc, 256>(ssa, scratch);
  ssb = block_sum<Acc, 256>(ssb, scratch);
  const Acc ia = static_cast<Acc>(sa) / sqrt(ssa / static_cast<Acc>(width) + static_cast<Acc>(eps));
  const Acc ib = static_cast<Acc>(sb) / sqrt(ssb / static_cast<Acc>(width) + static_cast<Acc>(eps));
  Acc ss = 0;
  for (int c = threadIdx.x; c < width; c += 256) {
    const float sum = static_cast<float>(static_cast<Acc>(ra[c]) * ia * static_cast<Acc>(wa[c]) + static_cast<Acc>(rb[c]) * ib * static_cast<Acc>(wb[c]));
    const float y = static_cast<float>(static_cast<Acc>(rr[c]) + static_cast<Acc>(scale ? scale[c] : 1.f) * static_cast<Acc>(sum));
    rr[c] = y;
    ss += static_cast<Acc>(y) * static_cast<Acc>(y);
  }
  if (normed == nullptr) return;
  ss = block_sum<Acc, 256>(ss, scratch);
  const Acc inv = static_cast<Acc>(1) / sqrt(ss / static_cast<Acc>(width) + static_cast<Acc>(norm_eps));
  for (int c = threadIdx.x; c < width; c += 256) store_f32(normed + t * width + c, static_cast<float>(static_cast<Acc>(rr[c]) * inv * static_cast<Acc>(nw[c])));
}

// A step in which every request brings one row (row r is request r): the convolution with bias and silu and the state's step in one
// launch. A thread owns one channel of one row: it fetches what the state holds of its channel, then writes.
template <typename T, typename Acc>
__global__ void __launch_bounds__(256) conv_step_kernel(T* __restrict__ xbc, int64_t xbc_stride, const T* __restrict__ raw, int64_t raw_stride, const float* __restrict__ w,
                                                        const float* __restrict__ bias, T* __restrict__ state, const int32_t* __restrict__ req_slot, int width, int taps) {
  const int64_t t = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x, keep = taps - 1;
  if (c >= width) return;
  T* st = state + static_cast<int64_t>(req_slot[t]) * keep * width;
  const float* wc = w + static_cast<int64_t>(c) * taps;
  T kept[kConvMaxKeep];
  Acc acc = bias ? static_cast<Acc>(bias[c]) : static_cast<Acc>(0);
#pragma unroll
  for (int j = 0; j < kConvMaxKeep; ++j)
    if (j < keep) {
      kept[j] = st[static_cast<int64_t>(j) * width + c];
      acc += static_cast<Acc>(wc[j]) * static_cast<Acc>(load_f32(&kept[j]));
    }
  const T mine = raw[t * raw_stride + c];
  acc += static_cast<Acc>(wc[keep]) * static_cast<Acc>(load_f32(&mine));
#pragma unroll
  for (int j = 0; j < kConvMaxKeep; ++j)
    if (j < keep) st[static_cast<int64_t>(j) * width + c] = j + 1 < keep ? kept[j + 1] : mine;
  acc = acc / (static_cast<Acc>(1) + exp(-acc));
  store_f32(xbc + t * xbc_stride + c, static_cast<float>(acc));
}

}  // namespace alofa

using namespace alofa;

extern "C" int alofa_rms_pair_add_norm(float* residual, const float* a, const float* wa, float sa, const float* b, const float* wb, float sb, const float* scale, int64_t rows,
                                       int width, float eps, void* normed, int normed_dtype, const float* nw, float norm_eps, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(rows >= 0 && width > 0 && residual && a && b && wa && wb, "rms_pair_add_norm: bad arguments");
  ALOFA_REQUIRE(normed == nullptr || nw != nullptr, "rms_pair_add_norm: a norm needs its weight");
  ALOFA_REQUIRE(!exact || normed == nullptr || normed_dtype == kF32, "rms_pair_add_norm: the exact path is float32");
  if (rows == 0) return 0;
  const unsigned grid = static_cast<unsigned>(rows);
  if (exact) rms_pair_add_norm_kernel<float, double><<<grid, 256, 0, stream>>>(residual, a, wa, sa, b, wb, sb, scale, width, eps, static_cast<float*>(normed), nw, norm_eps);
  else if (normed == nullptr || normed_dtype == kF32) rms_pair_add_norm_kernel<float, float><<<grid, 256, 0, stream>>>(residual, a, wa, sa, b, wb, sb, scale, width, eps, static_cast<float*>(normed), nw, norm_eps);
  else rms_pair_add_norm_kernel<bf16_t, float><<<grid, 256, 0, stream>>>(residual, a, wa, sa, b, wb, sb, scale, width, eps, static_cast<bf16_t*>(normed), nw, norm_eps);
  return check_launch("rms_pair_add_norm");
}

extern "C" int alofa_conv_bias_act(void* out, int64_t out_stride, int out_dtype, const void* x, int64_t x_stride, int x_dtype, const float* w, const float* bias,
                                   const void* state, const int32_t* req_slot, const int32_t* row_off, const int32_t* req_of_row, int rows, int width, int taps,
                                   int act, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(rows >= 0 && width > 0 && taps >= 1 && taps - 1 <= kConvMaxKeep, "conv_bias_act: bad sizes (rows=%d width=%d taps=%d, at most %d taps)", rows, width, taps, kConvMaxKeep + 1);
  ALOFA_REQUIRE(!exact || (out_dtype == kF32 && x_dtype == kF32), "conv_bias_act: the exact path is float32");
  ALOFA_REQUIRE(out_dtype == x_dtype, "conv_bias_act: rows in and out have one type (out=%d in=%d)", out_dtype, x_dtype);
  if (rows == 0) return 0;
  const unsigned grid = blocks_for(static_cast<int64_t>(rows) * width);
#define ALOFA_CBA(T, ACC) conv_bias_act_kernel<T, T, ACC><<<grid, 256, 0, stream>>>(static_cast<T*>(out), out_stride, static_cast<const T*>(x), x_stride, w, bias, static_cast<const T*>(state), \
    req_slot, row_off, req_of_row, rows, width, taps, act)
  if (exact) ALOFA_CBA(float, double);
  else if (x_dtype == kF32) ALOFA_CBA(float, float);
  else ALOFA_CBA(bf16_t, float);
#undef ALOFA_CBA
  return check_launch("conv_bias_act");
}

extern "C" int alofa_conv_keep(void* state, const void* x, int64_t x_stride, int dtype, const int32_t* req_slot, const int32_t* row_off, int requests, int width, int keep,
                               hipStream_t stream) {
  ALOFA_REQUIRE(requests >= 0 && width > 0 && keep >= 0 && keep <= kConvMaxKeep, "conv_keep: bad sizes (requests=%d width=%d keep=%d)", requests, width, keep);
  if (requests == 0 || keep == 0) return 0;
  const unsigned grid = blocks_for(static_cast<int64_t>(requests) * width);
  if (dtype == kF32) conv_keep_kernel<float><<<grid, 256, 0, stream>>>(static_cast<float*>(state), static_cast<const float*>(x), x_stride, req_slot, row_off, requests, width, keep);
  else conv_keep_kernel<bf16_t><<<grid, 256, 0, stream>>>(static_cast<bf16_t*>(state), static_cast<const bf16_t*>(x), x_stride, req_slot, row_off, requests, width, keep);
  return check_launch("conv_keep");
}

extern "C" int alofa_ssd_operands(float* qf, float* kf, float* vf, float* decay, const void* xbc, int64_t xbc_stride, const void* dt_raw, int64_t dt_stride, int dtype,
                                  const float* dt_bias, const float* a_log, int64_t rows, int heads, int groups, int N, int dv, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(rows >= 0 && heads > 0 && groups > 0 && heads % groups == 0 && N > 0 && dv > 0, "ssd_operands: bad sizes (heads=%d groups=%d state=%d dv=%d)", heads, groups, N, dv);
  ALOFA_REQUIRE(!exact || dtype == kF32, "ssd_operands: the exact path is float32");
  if (rows == 0) return 0;
  const dim3 grid(static_cast<unsigned>(rows), heads);
#define ALOFA_SSDO(T, ACC) ssd_operands_kernel<T, ACC><<<grid, 128, 0, stream>>>(qf, kf, vf, decay, static_cast<const T*>(xbc), xbc_stride, static_cast<const T*>(dt_raw), dt_stride, dt_bias, a_log, heads, groups, N, dv)
  if (exact) ALOFA_SSDO(float, double);
  else if (dtype == kF32) ALOFA_SSDO(float, float);
  else ALOFA_SSDO(bf16_t, float);
#undef ALOFA_SSDO
  return check_launch("ssd_operands");
}

extern "C" int alofa_ssd_finish(void* out, int64_t out_stride, const float* o, int parts, int64_t part_stride, const void* x, int64_t x_stride, const void* z, int64_t z_stride,
                                int dtype, const float* skip, const float* weight, int64_t rows, int heads, int dv, int norm_parts, float eps, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(rows >= 0 && heads > 0 && dv > 0 && parts >= 1 && norm_parts > 0 && (heads * dv) % norm_parts == 0, "ssd_finish: bad sizes (heads=%d dv=%d parts=%d norm parts=%d)", heads, dv, parts, norm_parts);
  ALOFA_REQUIRE(!exact || dtype == kF32, "ssd_finish: the exact path is float32");
  if (rows == 0) return 0;
  const dim3 grid(static_cast<unsigned>(rows), norm_parts);
#define ALOFA_SSDF(T, ACC) ssd_finish_kernel<T, ACC><<<grid, 256, 0, stream>>>(static_cast<T*>(out), out_stride, o, parts, part_stride, static_cast<const T*>(x), x_stride, static_cast<const T*>(z), z_stride, \
    skip, weight, heads, dv, norm_parts, eps)
  if (exact) ALOFA_SSDF(float, double);
  else if (dtype == kF32) ALOFA_SSDF(float, float);
  else ALOFA_SSDF(bf16_t, float);
#undef ALOFA_SSDF
  return check_launch("ssd_finish");
}

extern "C" int alofa_rms_pair_sum(float* out, const float* a, const float* wa, float sa, const float* b, const float* wb, float sb, int64_t rows, int width, float eps,
                                  int exact, hipStream_t stream) {
  ALOFA_REQUIRE(rows >= 0 && width > 0 && a && b && wa && wb, "rms_pair_sum: bad arguments");
  if (rows == 0) return 0;
  if (exact) rms_pair_sum_kernel<double><<<static_cast<unsigned>(rows), 256, 0, stream>>>(out, a, wa, sa, b, wb, sb, width, eps);
  else rms_pair_sum_kernel<float><<<static_cast<unsigned>(rows), 256, 0, stream>>>(out, a, wa, sa, b, wb, sb, width, eps);
  return check_launch("rms_pair_sum");
}

// The convolution (bias, silu) with its state's step for single rows, then the operands: two launches where rows of any number take three.
// (All of it in one launch, a block per row that waits for its own row between the two halves, was measured and is slower: 18 us against the
// 14 us of the three launches at eight rows of 2,560 channels; the two launches take 10.)
extern "C" int alofa_ssd_step(void* xbc, int64_t xbc_stride, const void* raw, int64_t raw_stride, int dtype, const float* w, const float* bias, void* state,
                              const int32_t* req_slot, int taps, float* qf, float* kf, float* vf, float* decay, const void* dt_raw, int64_t dt_stride,
                              const float* dt_bias, const float* a_log, int64_t rows, int heads, int groups, int N, int dv, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(rows >= 0 && heads > 0 && groups > 0 && heads % groups == 0 && N > 0 && dv > 0, "ssd_step: bad sizes (heads=%d groups=%d state=%d dv=%d)", heads, groups, N, dv);
  ALOFA_REQUIRE(taps >= 1 && taps - 1 <= kConvMaxKeep && (taps == 1 || state != nullptr), "ssd_step: 1 to %d taps, and a state for more than one", kConvMaxKeep + 1);
  ALOFA_REQUIRE(!exact || dtype == kF32, "ssd_step: the exact path is float32");
  if (rows == 0) return 0;
  const int width = heads * dv + 2 * groups * N;
  const dim3 grid((width + 255) / 256, static_cast<unsigned>(rows));
#define ALOFA_SSDS(T, ACC) conv_step_kernel<T, ACC><<<grid, 256, 0, stream>>>(static_cast<T*>(xbc), xbc_stride, static_cast<const T*>(raw), raw_stride, w, bias, static_cast<T*>(state), \
    req_slot, width, taps)
  if (exact) ALOFA_SSDS(float, double);
  else if (dtype == kF32) ALOFA_SSDS(float, float);
  else ALOFA_SSDS(bf16_t, float);
#undef ALOFA_SSDS
  if (int e = check_launch("ssd_step")) return e;
  return alofa_ssd_operands(qf, kf, vf, decay, xbc, xbc_stride, dt_raw, dt_stride, dtype, dt_bias, a_log, rows, heads, groups, N, dv, exact, stream);
}
