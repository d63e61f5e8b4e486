// Kernels of layers that carry state of fixed size per request instead of (or beside) pages of keys:
// a short causal convolution over time, the mix of a token with the one before it, and the linear
// recurrence S_t = diag(w_t) S_(t-1) + k_t v_t^T with its read-out, which serves retention (one decay per
// head), gated linear attention (a decay per key channel and token) and RWKV-style time mixing (the same with
// the read-out taken before the update and a bonus for the current token).
//
// How a step's rows belong to requests: request r of the step owns the rows row_off[r] .. row_off[r+1]-1,
// in position order, and keeps its state in slot req_slot[r]. With row_off absent every request brings one
// row (row r). req_of_row[t] names the request of row t (absent: t itself). What came before a request's
// first row of this step is in its state, which is zero for a new request, so no kernel asks for positions.
//
// State and all arithmetic of the recurrences are float; q, k, v and gates come in the activation type.
#include "common.h"

#include <type_traits>

namespace alofa {

// ---- short causal convolution ------------------------------------------------------------------------
// out[t, c] = h[t, c] + sum_j w[c, j] * h[t - taps + 1 + j, c], rows before the request's first row of this step
// taken from state[slot, i, c], which holds the last taps - 1 inputs (i = taps - 2 is the newest). The state
// is not written here: rows of one request are spread over blocks that all read it.
template <typename TO, typename TI, typename Acc>
__global__ void __launch_bounds__(256) short_conv_kernel(TO* __restrict__ out, const TI* __restrict__ h, const float* __restrict__ w,
                                                         const TI* __restrict__ state, const int32_t* __restrict__ req_slot,
                                                         const int32_t* __restrict__ row_off, const int32_t* __restrict__ req_of_row,
                                                         int rows, int width, int taps) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= static_cast<int64_t>(rows) * width) return;
  const int t = static_cast<int>(idx / width), c = static_cast<int>(idx % width);
  const int r = req_of_row ? req_of_row[t] : t;
  const int row0 = row_off ? row_off[r] : r;
  const TI* st = state + static_cast<int64_t>(req_slot[r]) * (taps - 1) * width;
  const float* wc = w + static_cast<int64_t>(c) * taps;
  const Acc mine = static_cast<Acc>(load_f32(h + static_cast<int64_t>(t) * width + c));
  Acc acc = mine;
  for (int j = 0; j < taps; ++j) {
    const int s = t - taps + 1 + j;
    const Acc v = j == taps - 1 ? mine
                  : s >= row0  ? static_cast<Acc>(load_f32(h + static_cast<int64_t>(s) * width + c))
                               : static_cast<Acc>(load_f32(st + static_cast<int64_t>(taps - 1 + s - row0) * width + c));
    acc += static_cast<Acc>(wc[j]) * v;
  }
  store_f32(out + static_cast<int64_t>(t) * width + c, static_cast<float>(acc));
}

// The last `keep` rows a request has seen, after this step: state[slot, i, c] = the input at (end of the request's
// rows) - keep + i, from this step's rows or, where the step brought fewer, from the old state. A thread owns one
// channel of one request, reads what it needs and writes afterwards.
constexpr int kMaxKeep = 15;
template <typename TI>
__global__ void __launch_bounds__(256) keep_last_rows_kernel(TI* __restrict__ state, const TI* __restrict__ h, const int32_t* __restrict__ req_slot,
                                                             const int32_t* __restrict__ row_off, int requests, int width, int keep) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= static_cast<int64_t>(requests) * width) return;
  const int r = static_cast<int>(idx / width), c = static_cast<int>(idx % width);
  const int row0 = row_off ? row_off[r] : r, end = row_off ? row_off[r + 1] : r + 1;
  TI* st = state + static_cast<int64_t>(req_slot[r]) * keep * width;
  TI kept[kMaxKeep];
#pragma unroll
  for (int i = 0; i < kMaxKeep; ++i) {
    if (i < keep) {
      const int s = end - keep + i;
      kept[i] = s >= row0 ? h[static_cast<int64_t>(s) * width + c] : st[static_cast<int64_t>(keep + s - row0) * width + c];
    }
  }
#pragma unroll
  for (int i = 0; i < kMaxKeep; ++i)
    if (i < keep) st[static_cast<int64_t>(i) * width + c] = kept[i];
}

// Layer norm, convolution and the state's step in one launch, for steps in which every request brings one row (row r is
// request r): out[r] = n + conv(n) with n = layer norm of x[r] (weight and bias), the rows before it taken from the state,
// which then moves on by n. A block owns 256 channels of a row (every block of a row takes the row's two sums itself: the
// row is a few kilobytes), a thread one channel of the request's state: it fetches what the state holds at once, and
// writes afterwards.
template <typename TO, typename Acc>
__global__ void __launch_bounds__(256) norm_conv_step_kernel(TO* __restrict__ out, const float* __restrict__ x, const float* __restrict__ nw,
                                                             const float* __restrict__ nb, float eps, const float* __restrict__ w,
                                                             float* __restrict__ state, const int32_t* __restrict__ req_slot, int width, int taps) {
  __shared__ Acc scratch[4];
  const int r = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  const float* src = x + static_cast<int64_t>(r) * width;
  float* st = state + static_cast<int64_t>(req_slot[r]) * (taps - 1) * width;
  float kept[kMaxKeep], wc[kMaxKeep + 1];
#pragma unroll
  for (int jj = 0; jj < kMaxKeep; ++jj) kept[jj] = (c < width && jj < taps - 1) ? st[static_cast<int64_t>(jj) * width + c] : 0.f;
#pragma unroll
  for (int jj = 0; jj <= kMaxKeep; ++jj) wc[jj] = (c < width && jj < taps) ? w[static_cast<int64_t>(c) * taps + jj] : 0.f;
  Acc s = 0;
  for (int e = threadIdx.x; e < width; e += 256) s += static_cast<Acc>(src[e]);
  const Acc mean = block_sum<Acc, 256>(s, scratch) / static_cast<Acc>(width);
  Acc ss = 0;
  for (int e = threadIdx.x; e < width; e += 256) {
    const Acc d = static_cast<Acc>(src[e]) - mean;
    ss += d * d;
  }
  const Acc var = block_sum<Acc, 256>(ss, scratch) / static_cast<Acc>(width);
  if (c >= width) return;
  const Acc inv = static_cast<Acc>(1) / sqrt(var + static_cast<Acc>(eps));
  const float n = static_cast<float>((static_cast<Acc>(src[c]) - mean) * inv * static_cast<Acc>(nw[c]) + static_cast<Acc>(nb[c]));
  Acc acc = static_cast<Acc>(n);
  float last = n;      // the filter's own tap on the row itself comes last, as in the kernel for any rows
#pragma unroll
  for (int jj = 0; jj < kMaxKeep; ++jj) {
    if (jj < taps - 1) {
      acc += static_cast<Acc>(wc[jj]) * static_cast<Acc>(kept[jj]);
      if (jj > 0) st[static_cast<int64_t>(jj - 1) * width + c] = kept[jj];
    }
  }
#pragma unroll
  for (int jj = 0; jj <= kMaxKeep; ++jj)
    if (jj == taps - 1) acc += static_cast<Acc>(wc[jj]) * static_cast<Acc>(last);
  if (taps > 1) st[static_cast<int64_t>(taps - 2) * width + c] = n;
  store_f32(out + static_cast<int64_t>(r) * width + c, static_cast<float>(acc));
}

// ---- mix with the token before --------------------------------------------------------------------------
// out[s, t, c] = x[t, c] + (x[t-1, c] - x[t, c]) * mu[s, c] for s < n_mixes; the row before a request's first row
// of this step is state[slot, c] (zeros for a new request). The state is kept by keep_last_rows (keep = 1), or, in steps of
// single rows (row_off absent) with `keep` set, here: the thread that read a request's channel writes the row over it.
template <typename T>
__global__ void __launch_bounds__(256) shift_mix_kernel(T* __restrict__ out, const T* __restrict__ x, const float* __restrict__ mu,
                                                        T* __restrict__ state, const int32_t* __restrict__ req_slot,
                                                        const int32_t* __restrict__ row_off, const int32_t* __restrict__ req_of_row,
                                                        int rows, int width, int n_mixes, int keep) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= static_cast<int64_t>(rows) * width) return;
  const int t = static_cast<int>(idx / width), c = static_cast<int>(idx % width);
  const int r = req_of_row ? req_of_row[t] : t;
  const int row0 = row_off ? row_off[r] : r;
  const T mine = x[static_cast<int64_t>(t) * width + c];
  const float cur = load_f32(&mine);
  T* kept = state + static_cast<int64_t>(req_slot[r]) * width + c;
  const float prev = t > row0 ? load_f32(x + static_cast<int64_t>(t - 1) * width + c) : load_f32(kept);
  if (keep) *kept = mine;
  const float diff = prev - cur;
  for (int s = 0; s < n_mixes; ++s)
    store_f32(out + (static_cast<int64_t>(s) * rows + t) * width + c, cur + diff * mu[static_cast<int64_t>(s) * width + c]);
}

// ---- the linear recurrence ----------------------------------------------------------------------------------
// Per request and head, a state S [dk, dv] (float, in the request's slot) and for its rows in order:
//   after-update form:   S = diag(w_t) S + k_t v_t^T;  o_t = S^T q_t
//   before-update form:  o_t = (S + diag(u) k_t v_t^T)^T q_t;  S = diag(w_t) S + k_t v_t^T     (bonus u per head and key channel)
// with q scaled by q_scale and k by k_scale first. The decay w_t per key channel comes as
//   kDecayPerHead:     a constant per head (decay[head]),
//   kDecaySigmoidRoot: sigmoid(z)^(1/tau), z = decay_in[t, head * dk + i], formed as exp(log_sigmoid(z) / tau),
//   kDecayExpNegExp:   exp(-exp(z)).
//
// A block owns (request, head, a slice of CW value channels), CW = 16, 32 or 64: the fewer blocks a step has, the narrower
// the slices, so that a lone prompt still spreads over the chip. A wavefront is 64 / CW groups of CW lanes; lanes of a group
// are value channels, and group g of wave w owns the KL key channels from (w * groups + g) * KL on and keeps its share of S
// in registers (KL floats per lane). Rows go through LDS in chunks: all threads fetch the chunk's q, k, decays (made once
// per row and channel, not per lane) and v; then every wave runs the chunk's rows in order against LDS alone (16-byte
// reads that a group shares), leaving its groups' partial read-outs there; after a barrier they are added over waves and
// groups in a fixed order and written. A read-out depends on nothing but the rows before it: not on how rows were cut
// into steps or chunks.
enum DecayKind : int { kDecayPerHead = 0, kDecaySigmoidRoot = 1, kDecayExpNegExp = 2, kDecayGiven = 3 };

__device__ __forceinline__ float decay_of(float z, int kind, float inv_tau) {
  if (kind == kDecaySigmoidRoot) {
    // log sigmoid(z) = -(max(-z, 0) + log1p(exp(-|z|)))
    const float ls = -(fmaxf(-z, 0.f) + log1pf(expf(-fabsf(z))));
    return expf(ls * inv_tau);
  }
  return kind == kDecayExpNegExp ? expf(-expf(z)) : z;
}

// The decays of many rows, made in place before the recurrence runs (which then takes them as given): a prompt's rows
// are all there, and making their decays takes the whole chip a few microseconds, where the blocks of the recurrence,
// few and each bound to its rows' order, would spend more time on them than on the recurrence itself.
__global__ void __launch_bounds__(256) decay_kernel(float* __restrict__ z, int64_t stride, int64_t rows, int width, int kind, float inv_tau) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= rows * width) return;
  float* p = z + idx / width * stride + idx % width;
  *p = decay_of(*p, kind, inv_tau);
}

// v of lane kLane of the caller's row of 16 lanes, for every lane of the row (a data-parallel-primitive move, which the
// compiler folds into the multiply that uses it).
template <int kLane>
__device__ __forceinline__ float row_lane(float v) {
  return __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), 0x150 + kLane, 0xf, 0xf, true));      // row_newbcast:kLane
}

template <int kFrom, int kTo, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (kFrom < kTo) {
    f(std::integral_constant<int, kFrom>{});
    static_for<kFrom + 1, kTo>(f);
  }
}

// What a group needs of one row, q then k then (unless the decay is the head's) w of its KL key channels, lies in LDS as one
// run of floats; a lane reads the floats r, r + 16, ... (r its place in its row of 16 lanes) and the lanes of the row hand
// them to one another. Runs begin an odd multiple of 16 floats apart, so that the rows of a wave read different banks.
template <int KL, bool kPerHead>
struct RunOfOperands {
  static constexpr int kFloats = (kPerHead ? 2 : 3) * KL;
  static constexpr int kLoads = (kFloats + 15) / 16;
  static constexpr int kStride = 16 * (kLoads | 1);
};

template <typename T, int KL, bool kPerHead, bool kDirect>
__global__ void __launch_bounds__((KL <= 8 || KL == 64) ? 512 : 256) linear_recurrence_kernel(
    float* __restrict__ out, const T* __restrict__ q, int64_t q_stride, const T* __restrict__ k, int64_t k_stride,
    const T* __restrict__ v, int64_t v_stride, const float* __restrict__ decay_in, int64_t decay_stride, const float* __restrict__ decay_head,
    const float* __restrict__ bonus, float* __restrict__ state, const int32_t* __restrict__ req_slot, const int32_t* __restrict__ row_off,
    int heads, int dk, int dv, int decay_kind, float inv_tau, float q_scale, float k_scale, int before_update, int chunk, int cw_log2,
    int key_blocks, int64_t part_stride) {
  extern __shared__ float4 lds4[];
  float* lds = reinterpret_cast<float*>(lds4);
  const int cw = 1 << cw_log2, groups = kWave >> cw_log2;
  const int n_waves = blockDim.x / kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int col = lane & (cw - 1), group = lane >> cw_log2;
  // (with key_blocks > 1 the key channels of a head are dealt out over so many blocks, each with its share of the state's rows;
  // block kb leaves its part of every read-out in out + kb * part_stride, and whoever reads them adds the parts)
  const int r = blockIdx.z, head = blockIdx.y / key_blocks, kb = blockIdx.y % key_blocks, j0 = blockIdx.x * cw;
  const int row0 = row_off ? row_off[r] : r, end = row_off ? row_off[r + 1] : r + 1;
  const int j = j0 + col;
  const bool live = j < dv;
  // LDS: the groups' runs of operands as [chunk][waves * groups][kStride]; v as [chunk][cw]; partial read-outs as [chunk][waves * groups][cw]
  using Run = RunOfOperands<KL, kPerHead>;
  const int dk_pad = n_waves * groups * KL, parts = n_waves * groups, part = wave * groups + group;      // (dk_pad: the key channels of this block)
  const int key0 = kb * dk_pad, i0 = key0 + part * KL;      // the block's first key channel, and this lane's
  float* lx = lds;
  float* lv = lx + chunk * parts * Run::kStride;
  float* lp = lv + chunk * cw;

  float* S_g = state + ((static_cast<int64_t>(req_slot[r]) * heads + head) * dk) * dv;
  float S[KL], u[KL];
#pragma unroll
  for (int i = 0; i < KL; ++i) {
    S[i] = (live && i0 + i < dk) ? S_g[static_cast<int64_t>(i0 + i) * dv + j] : 0.f;
    u[i] = (bonus && i0 + i < dk) ? bonus[head * dk + i0 + i] : 0.f;
  }
  const float head_decay = kPerHead ? decay_head[head] : 1.f;

  // A chunk's q, k and decay operands are fetched into registers while the chunk before runs (kFetch values of each per
  // thread), and go to LDS, decays made, once that one's read-outs are written.
  constexpr int kFetch = 16, kFetchV = 8;      // chunk * dk_pad <= kFetch * threads, chunk * cw <= kFetchV * threads: the host sees to it
  T fq[kFetch], fk[kFetch];
  float fz[kFetch], fv[kFetchV];
  // (value f of a thread is element threadIdx.x + f * threads of the chunk's [rows][dk_pad]: its row and channel follow from
  // the one before by additions, the only divisions are these)
  const int threads = blockDim.x;
  const int first_row = threadIdx.x / dk_pad, first_i = threadIdx.x % dk_pad, step_row = threads / dk_pad, step_i = threads % dk_pad;
  const int passes = (chunk * dk_pad + threads - 1) / threads, v_passes = ((chunk << cw_log2) + threads - 1) / threads;
  auto fetch = [&](int c0) {
    const int n = min(chunk, end - c0);
    int tt = first_row, i = first_i;
#pragma unroll
    for (int f = 0; f < kFetch; ++f) {
      if (f < passes) {
        const bool in = tt < n && key0 + i < dk;      // (every lane loads: from the chunk's first row and channel where its own is not wanted)
        const int64_t t = c0 + (in ? tt : 0);
        const int ch = head * dk + (in ? key0 + i : 0);
        fq[f] = q[t * q_stride + ch];
        fk[f] = k[t * k_stride + ch];
        if constexpr (!kPerHead) fz[f] = decay_in[t * decay_stride + ch];
        i += step_i;
        tt += step_row;
        if (i >= dk_pad) i -= dk_pad, ++tt;
      }
    }
#pragma unroll
    for (int f = 0; f < kFetchV; ++f) {
      if (f < v_passes) {
        const int e = threadIdx.x + f * threads;
        const int tv = e >> cw_log2, jj = e & (cw - 1);
        const bool in = tv < n && j0 + jj < dv;
        fv[f] = load_f32(v + static_cast<int64_t>(c0 + (in ? tv : 0)) * v_stride + head * dv + (in ? j0 + jj : 0));
        if (!in) fv[f] = 0.f;
      }
    }
  };
  if (row0 < end) fetch(row0);
  for (int c0 = row0; c0 < end; c0 += chunk) {
    const int n = min(chunk, end - c0);
    __syncthreads();      // the chunk before is written out; LDS is free again
    {
      int tt = first_row, i = first_i;
#pragma unroll
      for (int f = 0; f < kFetch; ++f) {
        if (f < passes) {
          if (tt < n) {
            float qv = 0.f, kv = 0.f, wv = 1.f;
            if (key0 + i < dk) {
              qv = load_f32(&fq[f]) * q_scale;
              kv = load_f32(&fk[f]) * k_scale;
              if constexpr (!kPerHead) wv = decay_of(fz[f], decay_kind, inv_tau);
            }
            float* run = lx + (tt * parts + i / KL) * Run::kStride + i % KL;
            run[0] = qv;
            run[KL] = kv;
            if constexpr (!kPerHead) run[2 * KL] = wv;
          }
          i += step_i;
          tt += step_row;
          if (i >= dk_pad) i -= dk_pad, ++tt;
        }
      }
    }
#pragma unroll
    for (int f = 0; f < kFetchV; ++f) {
      const int e = threadIdx.x + f * threads;
      if (f < v_passes && e < n * cw) lv[e] = fv[f];
    }
    __syncthreads();
    if (c0 + chunk < end) fetch(c0 + chunk);
    auto run_rows = [&](auto before) {
      constexpr bool kBefore = decltype(before)::value;
      // kRows rows at a time: their operands are asked of LDS together, then the rows run in order (a wave is alone on
      // its SIMD, so what it waits for is not hidden by others)
      constexpr int kRows = kDirect ? (KL <= 4 ? 4 : KL <= 16 ? 2 : 1) : (KL <= 16 ? 4 : KL == 32 ? 2 : 1);
      // ... and, in the shape of long steps, the next rows' operands are asked for before these rows run: two sets of registers take turns.
      constexpr int kOperands = kDirect ? Run::kFloats : Run::kLoads;
      const float* my_v = lv + col;
      const float* my_run = lx + part * Run::kStride + (kDirect ? 0 : (lane & 15));
      float* my_part = lp + part * cw + col;
      const int run_step = parts * Run::kStride, part_step = parts * cw;
      auto ask = [&](int t0, float (&vj)[kRows], float (&x)[kRows][kOperands]) {
#pragma unroll
        for (int a = 0; a < kRows; ++a) {
          const int tt = min(t0 + a, n - 1);      // (rows past the chunk's end: read again, never used)
          vj[a] = my_v[tt * cw];
          if constexpr (kDirect) {      // the wave is one group: every lane reads the whole run (reads of one address, 16 bytes at a time)
            const float4* run = reinterpret_cast<const float4*>(my_run + tt * run_step);
#pragma unroll
            for (int m = 0; m < Run::kFloats / 4; ++m) {
              const float4 f4 = run[m];
              x[a][4 * m] = f4.x, x[a][4 * m + 1] = f4.y, x[a][4 * m + 2] = f4.z, x[a][4 * m + 3] = f4.w;
            }
          } else {
            const float* run = my_run + tt * run_step;
#pragma unroll
            for (int m = 0; m < Run::kLoads; ++m) x[a][m] = run[16 * m];
          }
        }
      };
      auto run = [&](int t0, const float (&vj)[kRows], const float (&x)[kRows][kOperands]) {
#pragma unroll
        for (int a = 0; a < kRows; ++a) {
          if (t0 + a < n) {
            float acc[4] = {0.f, 0.f, 0.f, 0.f};
            static_for<0, KL>([&](auto at) {
              constexpr int e = decltype(at)::value;
              float qe, ke, we = head_decay;
              if constexpr (kDirect) {
                qe = x[a][e], ke = x[a][KL + e];
                if constexpr (!kPerHead) we = x[a][2 * KL + e];
              } else {
                qe = row_lane<e % 16>(x[a][e / 16]), ke = row_lane<(KL + e) % 16>(x[a][(KL + e) / 16]);
                if constexpr (!kPerHead) we = row_lane<(2 * KL + e) % 16>(x[a][(2 * KL + e) / 16]);
              }
              const float kvv = ke * vj[a];
              if constexpr (kBefore) {
                acc[e % 4] += qe * (S[e] + u[e] * kvv);
                S[e] = we * S[e] + kvv;
              } else {
                S[e] = we * S[e] + kvv;
                acc[e % 4] += qe * S[e];
              }
            });
            my_part[(t0 + a) * part_step] = (acc[0] + acc[1]) + (acc[2] + acc[3]);
          }
        }
      };
      float vj_a[kRows], x_a[kRows][kOperands];
      if constexpr (kDirect && KL <= 8) {      // (the shape of long steps: few keys a lane)
        float vj_b[kRows], x_b[kRows][kOperands];
        ask(0, vj_a, x_a);
        for (int t0 = 0; t0 < n; t0 += 2 * kRows) {
          const bool more = t0 + kRows < n;
          if (more) ask(t0 + kRows, vj_b, x_b);
          run(t0, vj_a, x_a);
          if (more) {
            if (t0 + 2 * kRows < n) ask(t0 + 2 * kRows, vj_a, x_a);
            run(t0 + kRows, vj_b, x_b);
          }
        }
      } else {      // (steps of few rows: one set of registers, so that more blocks share a compute unit)
        for (int t0 = 0; t0 < n; t0 += kRows) {
          ask(t0, vj_a, x_a);
          run(t0, vj_a, x_a);
        }
      }
    };
    if (before_update) run_rows(std::true_type{});
    else run_rows(std::false_type{});
    __syncthreads();
    for (int e = threadIdx.x; e < n * cw; e += blockDim.x) {
      const int tt = e >> cw_log2, jj = e & (cw - 1);
      if (j0 + jj < dv) {
        float acc = 0.f;
        for (int g = 0; g < parts; ++g) acc += lp[(tt * parts + g) * cw + jj];
        out[kb * part_stride + (static_cast<int64_t>(c0 + tt) * heads + head) * dv + j0 + jj] = acc;
      }
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < KL; ++i)
      if (i0 + i < dk) S_g[static_cast<int64_t>(i0 + i) * dv + j] = S[i];
  }
}

// ---- exponential gates kept in range by a running maximum (the matrix memory of xLSTM) ---------------------------
// Per request and head, over the request's rows in order, with m the running maximum kept in the request's slot (0 for a new request):
//   i = cap tanh(zi / cap), f = log sigmoid(cap tanh(zf / cap));  m' = max(f + m, i);  keep = exp(f + m - m'), take = exp(i - m')
// gates[0 / 1 / 2][t, head] = keep / take / exp(-m') (three planes of [rows, heads]). One block of four wavefronts per (request, head), 256 rows at a
// time: every thread forms the two gates of its row (the next 256 rows' loads are on their way meanwhile); then the first wavefront walks the maximum
// through the rows in order, 64 at a time, every lane doing the same two operations a row on values read from the lanes in turn (the same sums in the
// same order whatever the rows' number and however they were cut into steps); then every thread leaves its row's three factors.
__global__ void __launch_bounds__(256) gate_scan_kernel(float* __restrict__ gates, const float* __restrict__ z, int64_t z_stride, float* __restrict__ state,
                                                        const int32_t* __restrict__ req_slot, const int32_t* __restrict__ row_off, int requests, int64_t rows, int heads, float cap) {
  __shared__ float s_f[256], s_i[256], s_before[256], s_after[256];
  const int idx = blockIdx.x, tid = threadIdx.x, lane = tid % kWave;
  const bool walker = tid < kWave;
  if (idx >= requests * heads) return;
  const int r = idx / heads, h = idx % heads;
  const int row0 = row_off ? row_off[r] : r, end = row_off ? row_off[r + 1] : r + 1;
  float* kept = state + static_cast<int64_t>(req_slot[r]) * heads + h;
  float m = *kept;      // (the first wavefront's copy is the one that walks)
  auto ask = [&](int t, float& zi, float& zf) {
    zi = zf = 0.f;
    if (t < end) {
      zi = z[t * z_stride + h];
      zf = z[t * z_stride + heads + h];
    }
  };
  float zi, zf;
  ask(row0 + tid, zi, zf);
  for (int t0 = row0; t0 < end; t0 += 256) {      // uniform over the block
    float zi_next, zf_next;
    ask(t0 + 256 + tid, zi_next, zf_next);
    const int t = t0 + tid, n = end - t0 < 256 ? end - t0 : 256;
    const float gi = cap * tanhf(zi / cap), x = cap * tanhf(zf / cap);
    const float gf = -(fmaxf(-x, 0.f) + log1pf(expf(-fabsf(x))));      // log sigmoid(x)
    s_f[tid] = gf;
    s_i[tid] = gi;
    __syncthreads();
    if (walker) {
      for (int c = 0; c * kWave < n; ++c) {
        const float f = s_f[c * kWave + lane], i = s_i[c * kWave + lane];
        const int nn = n - c * kWave < kWave ? n - c * kWave : kWave;
        float before = m, after = m;
        auto step = [&](int j) __attribute__((always_inline)) {
          const float fj = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(f), j)), ij = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(i), j));
          const float next = fmaxf(fj + m, ij);
          if (lane == j) {
            before = m;
            after = next;
          }
          m = next;
        };
        if (nn == kWave) {
#pragma unroll
          for (int j = 0; j < kWave; ++j) step(j);
        } else {
          for (int j = 0; j < nn; ++j) step(j);
        }
        s_before[c * kWave + lane] = before;
        s_after[c * kWave + lane] = after;
      }
    }
    __syncthreads();
    if (t < end) {
      const float before = s_before[tid], after = s_after[tid];
      float* g = gates + static_cast<int64_t>(t) * heads + h;
      g[0] = expf(gf + before - after);
      g[rows * heads] = expf(gi - after);
      g[2 * rows * heads] = expf(-after);
    }
    zi = zi_next;
    zf = zf_next;
  }
  if (tid == 0) *kept = m;
}

// The operands of the recurrence as float rows, gates applied: qf = q, kf = take * k, decay[t, head, :] = keep, vf = [v, 1] per head
// (the channel of ones carries the normaliser n_t = keep n + take k through the same recurrence: its read-out is n . q).
template <typename T>
__global__ void __launch_bounds__(256) gated_operands_kernel(float* __restrict__ qf, float* __restrict__ kf, float* __restrict__ vf, float* __restrict__ decay,
                                                             const T* __restrict__ q, int64_t q_stride, const T* __restrict__ k, int64_t k_stride,
                                                             const T* __restrict__ v, int64_t v_stride, const float* __restrict__ gates,
                                                             int64_t rows, int heads, int dk, int dv) {
  const int per_row = heads * (dk + dv + 1);
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= rows * per_row) return;
  const int64_t t = idx / per_row;
  const int e = static_cast<int>(idx % per_row);
  if (e < heads * dk) {
    const float* g = gates + t * heads + e / dk;
    qf[t * heads * dk + e] = load_f32(q + t * q_stride + e);
    kf[t * heads * dk + e] = g[rows * heads] * load_f32(k + t * k_stride + e);
    decay[t * heads * dk + e] = g[0];
  } else {
    const int c = e - heads * dk, h = c / (dv + 1), j = c % (dv + 1);
    vf[t * heads * (dv + 1) + c] = j < dv ? load_f32(v + t * v_stride + h * dv + j) : 1.f;
  }
}

}  // namespace alofa

using namespace alofa;

static inline unsigned blocks_of(int64_t n) { return static_cast<unsigned>((n + 255) / 256); }

extern "C" int alofa_gate_scan(float* gates, const float* z, int64_t z_stride, float* state, const int32_t* req_slot, const int32_t* row_off, int requests,
                               int64_t rows, int heads, float cap, hipStream_t stream) {
  ALOFA_REQUIRE(requests >= 0 && heads > 0 && cap > 0.f, "gate_scan: bad arguments (requests=%d heads=%d cap=%g)", requests, heads, cap);
  if (requests == 0) return 0;
  gate_scan_kernel<<<requests * heads, 256, 0, stream>>>(gates, z, z_stride, state, req_slot, row_off, requests, rows, heads, cap);
  return check_launch("gate_scan");
}

extern "C" int alofa_gated_operands(float* qf, float* kf, float* vf, float* decay, const void* q, int64_t q_stride, const void* k, int64_t k_stride,
                                    const void* v, int64_t v_stride, int dtype, const float* gates, int64_t rows, int heads, int dk, int dv, hipStream_t stream) {
  ALOFA_REQUIRE(rows >= 0 && heads > 0 && dk > 0 && dv > 0, "gated_operands: bad sizes");
  if (rows == 0) return 0;
  const unsigned grid = blocks_of(rows * heads * (dk + dv + 1));
  if (dtype == kF32) gated_operands_kernel<float><<<grid, 256, 0, stream>>>(qf, kf, vf, decay, static_cast<const float*>(q), q_stride, static_cast<const float*>(k), k_stride, static_cast<const float*>(v), v_stride, gates, rows, heads, dk, dv);
  else gated_operands_kernel<bf16_t><<<grid, 256, 0, stream>>>(qf, kf, vf, decay, static_cast<const bf16_t*>(q), q_stride, static_cast<const bf16_t*>(k), k_stride, static_cast<const bf16_t*>(v), v_stride, gates, rows, heads, dk, dv);
  return check_launch("gated_operands");
}

extern "C" int alofa_short_conv(void* out, int out_dtype, const void* h, int h_dtype, const float* w, const void* state, const int32_t* req_slot,
                                const int32_t* row_off, const int32_t* req_of_row, int rows, int width, int taps, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(rows >= 0 && width > 0 && taps >= 1 && taps - 1 <= kMaxKeep, "short_conv: bad sizes (rows=%d width=%d taps=%d, at most %d taps)", rows, width, taps, kMaxKeep + 1);
  ALOFA_REQUIRE(!exact || (out_dtype == kF32 && h_dtype == kF32), "short_conv: the exact path is float32");
  if (rows == 0) return 0;
  const unsigned grid = blocks_of(static_cast<int64_t>(rows) * width);
#define ALOFA_CONV(TO, TI, ACC) short_conv_kernel<TO, TI, ACC><<<grid, 256, 0, stream>>>(static_cast<TO*>(out), static_cast<const TI*>(h), w, static_cast<const TI*>(state), req_slot, row_off, req_of_row, rows, width, taps)
  if (exact) ALOFA_CONV(float, float, double);
  else if (out_dtype == kF32 && h_dtype == kF32) ALOFA_CONV(float, float, float);
  else if (out_dtype == kBF16 && h_dtype == kF32) ALOFA_CONV(bf16_t, float, float);
  else if (out_dtype == kBF16 && h_dtype == kBF16) ALOFA_CONV(bf16_t, bf16_t, float);
  else ALOFA_REQUIRE(false, "short_conv: no such pair of types (out=%d in=%d)", out_dtype, h_dtype);
#undef ALOFA_CONV
  return check_launch("short_conv");
}

extern "C" int alofa_norm_conv_step(void* out, int out_dtype, const float* x, const float* nw, const float* nb, float eps, const float* w, float* state,
                                    const int32_t* req_slot, int rows, int width, int taps, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(rows >= 0 && width > 0 && taps >= 1 && eps > 0.f, "norm_conv_step: bad sizes (rows=%d width=%d taps=%d)", rows, width, taps);
  ALOFA_REQUIRE(taps - 1 <= kMaxKeep, "norm_conv_step: at most %d taps", kMaxKeep + 1);
  ALOFA_REQUIRE(!exact || out_dtype == kF32, "norm_conv_step: the exact path writes float32");
  if (rows == 0) return 0;
  const dim3 grid((width + 255) / 256, rows);
  if (exact) norm_conv_step_kernel<float, double><<<grid, 256, 0, stream>>>(static_cast<float*>(out), x, nw, nb, eps, w, state, req_slot, width, taps);
  else if (out_dtype == kF32) norm_conv_step_kernel<float, float><<<grid, 256, 0, stream>>>(static_cast<float*>(out), x, nw, nb, eps, w, state, req_slot, width, taps);
  else norm_conv_step_kernel<bf16_t, float><<<grid, 256, 0, stream>>>(static_cast<bf16_t*>(out), x, nw, nb, eps, w, state, req_slot, width, taps);
  return check_launch("norm_conv_step");
}

extern "C" int alofa_keep_last_rows(void* state, const void* h, int dtype, const int32_t* req_slot, const int32_t* row_off, int requests, int width,
                                    int keep, hipStream_t stream) {
  ALOFA_REQUIRE(requests >= 0 && width > 0 && keep >= 0 && keep <= kMaxKeep, "keep_last_rows: bad sizes (requests=%d width=%d keep=%d)", requests, width, keep);
  if (requests == 0 || keep == 0) return 0;
  const unsigned grid = blocks_of(static_cast<int64_t>(requests) * width);
  if (dtype == kF32) keep_last_rows_kernel<float><<<grid, 256, 0, stream>>>(static_cast<float*>(state), static_cast<const float*>(h), req_slot, row_off, requests, width, keep);
  else keep_last_rows_kernel<bf16_t><<<grid, 256, 0, stream>>>(static_cast<bf16_t*>(state), static_cast<const bf16_t*>(h), req_slot, row_off, requests, width, keep);
  return check_launch("keep_last_rows");
}

extern "C" int alofa_shift_mix(void* out, const void* x, int dtype, const float* mu, void* state, const int32_t* req_slot, const int32_t* row_off,
                               const int32_t* req_of_row, int rows, int width, int n_mixes, int keep, hipStream_t stream) {
  ALOFA_REQUIRE(rows >= 0 && width > 0 && n_mixes >= 1, "shift_mix: bad sizes (rows=%d width=%d mixes=%d)", rows, width, n_mixes);
  ALOFA_REQUIRE(!keep || row_off == nullptr, "shift_mix: the state is kept here only in steps of single rows");
  if (rows == 0) return 0;
  const unsigned grid = blocks_of(static_cast<int64_t>(rows) * width);
  if (dtype == kF32) shift_mix_kernel<float><<<grid, 256, 0, stream>>>(static_cast<float*>(out), static_cast<const float*>(x), mu, static_cast<float*>(state), req_slot, row_off, req_of_row, rows, width, n_mixes, keep);
  else shift_mix_kernel<bf16_t><<<grid, 256, 0, stream>>>(static_cast<bf16_t*>(out), static_cast<const bf16_t*>(x), mu, static_cast<bf16_t*>(state), req_slot, row_off, req_of_row, rows, width, n_mixes, keep);
  return check_launch("shift_mix");
}

constexpr int kDecayApartFrom = 64;      // steps of more rows make their decays in a launch of their own

// How a launch is shaped. A step of few rows per request (decoding, short portions): a block owns all key channels of a head
// and a slice of value channels, halved while the step has too few blocks to fill the chip, down to 16; from the slice's width
// follow the keys a lane keeps and the waves of a block (four where the key size allows). A step of many rows (prompts), where
// the caller has room for parts of the read-outs: slices of 64 value channels (a wave is one group, its operands come by
// plain reads of one address), and the key channels of a head dealt out over blocks of 4 waves x 8 or 4 keys, so that a lone
// prompt fills the chip with blocks that each issue few instructions a row.
struct RecurrenceShape {
  int cw_log2, kl, waves, key_blocks;
};
static inline RecurrenceShape recurrence_shape(int requests, int rows, int heads, int dk, int dv, int max_parts) {
  int cw_log2 = dv <= 16 ? 4 : dv <= 32 ? 5 : 6;
  if (rows > kDecayApartFrom && max_parts > 1) {
    const int groups = 64 >> cw_log2, slices = (dv + (1 << cw_log2) - 1) >> cw_log2;
    for (int kl = 8; kl >= 4; kl /= 2) {
      const int per_block = 4 * groups * kl, kb = (dk + per_block - 1) / per_block;
      const bool fills = static_cast<int64_t>(requests) * heads * slices * kb >= compute_units();
      if (kb <= max_parts && (fills || kl == 4 || 2 * kb > max_parts)) return {cw_log2, kl, 4, kb};
    }
  }
  const int64_t want = 2 * static_cast<int64_t>(compute_units());
  while (cw_log2 > 4 && static_cast<int64_t>(requests) * heads * ((dv + (1 << cw_log2) - 1) >> cw_log2) < want) --cw_log2;
  const int groups = 64 >> cw_log2;
  const int share = (dk + 4 * groups - 1) / (4 * groups);
  const int kl = share <= 4 ? 4 : share <= 8 ? 8 : share <= 16 ? 16 : share <= 32 ? 32 : 64;
  return {cw_log2, kl, (dk + kl * groups - 1) / (kl * groups), 1};
}

static inline int recurrence_lds_bytes(const RecurrenceShape& s, int chunk, bool per_head) {
  const int groups = 64 >> s.cw_log2;
  const int loads = ((per_head ? 2 : 3) * s.kl + 15) / 16, stride = 16 * (loads | 1);      // (RunOfOperands)
  return chunk * (s.waves * groups * stride + (1 << s.cw_log2) + s.waves * kWave) * static_cast<int>(sizeof(float));
}

// The most parts a step's read-outs may come in (the caller gives room for so many, or for one).
extern "C" int alofa_linear_recurrence_max_parts(int dk) { return dk >= 32 ? min(8, (dk + 15) / 16) : 1; }

// parts_used: in how many parts the read-outs were left (out + p * part_stride, p < parts_used; to be added by the reader).
extern "C" int alofa_linear_recurrence(float* out, int max_parts, int64_t part_stride, int* parts_used, const void* q, int64_t q_stride, const void* k, int64_t k_stride,
                                       const void* v, int64_t v_stride, int dtype, float* decay_in, int64_t decay_stride, const float* decay_head, const float* bonus,
                                       float* state, const int32_t* req_slot, const int32_t* row_off, int requests, int rows, int heads, int dk, int dv,
                                       int decay_kind, float tau, float q_scale, float k_scale, int before_update, hipStream_t stream) {
  ALOFA_REQUIRE(requests >= 0 && heads > 0 && dk > 0 && dk <= 512 && dv > 0 && max_parts >= 1, "linear_recurrence: bad sizes (requests=%d heads=%d dk=%d dv=%d; dk at most 512)", requests, heads, dk, dv);
  ALOFA_REQUIRE(decay_kind >= kDecayPerHead && decay_kind <= kDecayGiven && rows >= requests, "linear_recurrence: no such kind of decay (%d), or fewer rows than requests", decay_kind);
  ALOFA_REQUIRE(decay_kind == kDecayPerHead ? decay_head != nullptr : decay_in != nullptr, "linear_recurrence: the decay's operand is absent");
  ALOFA_REQUIRE(decay_kind != kDecaySigmoidRoot || tau > 0.f, "linear_recurrence: tau must be positive");
  *parts_used = 1;
  if (requests == 0) return 0;
  if (decay_kind != kDecayPerHead && decay_kind != kDecayGiven && rows > kDecayApartFrom) {
    const float inv = decay_kind == kDecaySigmoidRoot ? 1.f / tau : 0.f;
    decay_kernel<<<blocks_of(static_cast<int64_t>(rows) * heads * dk), 256, 0, stream>>>(decay_in, decay_stride, rows, heads * dk, decay_kind, inv);
    if (check_launch("linear_recurrence (decays)")) return 1;
    decay_kind = kDecayGiven;
  }
  const RecurrenceShape shape = recurrence_shape(requests, rows, heads, dk, dv, max_parts);
  const bool per_head = decay_kind == kDecayPerHead;
  // rows staged in LDS at a time: sixteen (thirty-two where a block has a share of the keys only), or as many as 64 KB hold for long
  // keys; one where every request brings a single row (decoding: little LDS a block, so that many blocks share a compute unit
  // and hide each other's waits)
  int chunk = rows == requests ? 1 : shape.key_blocks > 1 ? 32 : 16;
  const int groups = 64 >> shape.cw_log2, threads = shape.waves * kWave;
  // (... and as a thread's registers fetch ahead: 16 values of q, k and the decay's operand each, 8 of v)
  while (chunk > 1 && (recurrence_lds_bytes(shape, chunk, per_head) > 64 * 1024 || chunk * shape.waves * groups * shape.kl > 16 * threads || (chunk << shape.cw_log2) > 8 * threads)) chunk /= 2;
  ALOFA_REQUIRE(shape.waves * groups * shape.kl <= 16 * threads, "linear_recurrence: %d keys do not fit a block's registers", dk);
  const int lds = recurrence_lds_bytes(shape, chunk, per_head);
  ALOFA_REQUIRE(lds <= 64 * 1024 && threads <= ((shape.kl <= 8 || shape.kl == 64) ? 512 : 256), "linear_recurrence: %d keys do not fit a block", dk);
  const int cw = 1 << shape.cw_log2;
  const dim3 grid((dv + cw - 1) / cw, heads * shape.key_blocks, requests), block(threads);
  const float inv_tau = decay_kind == kDecaySigmoidRoot ? 1.f / tau : 0.f;
  *parts_used = shape.key_blocks;
#define ALOFA_SCAN(T, KL, PH, DIRECT) linear_recurrence_kernel<T, KL, PH, DIRECT><<<grid, block, lds, stream>>>(out, static_cast<const T*>(q), q_stride, static_cast<const T*>(k), k_stride, \
    static_cast<const T*>(v), v_stride, decay_in, decay_stride, decay_head, bonus, state, req_slot, row_off, heads, dk, dv, decay_kind, inv_tau, q_scale, k_scale, before_update, chunk, \
    shape.cw_log2, shape.key_blocks, part_stride)
#define ALOFA_SCAN_K(T, PH)                                                          \
  if (groups == 1) {                                                                 \
    switch (shape.kl) {                                                              \
      case 4: ALOFA_SCAN(T, 4, PH, true); break;                                     \
      case 8: ALOFA_SCAN(T, 8, PH, true); break;                                     \
      case 16: ALOFA_SCAN(T, 16, PH, true); break;                                   \
      case 32: ALOFA_SCAN(T, 32, PH, true); break;                                   \
      default: ALOFA_SCAN(T, 64, PH, true); break;                                   \
    }                                                                                \
  } else {                                                                           \
    switch (shape.kl) {                                                              \
      case 4: ALOFA_SCAN(T, 4, PH, false); break;                                    \
      case 8: ALOFA_SCAN(T, 8, PH, false); break;                                    \
      case 16: ALOFA_SCAN(T, 16, PH, false); break;                                  \
      case 32: ALOFA_SCAN(T, 32, PH, false); break;                                  \
      default: ALOFA_SCAN(T, 64, PH, false); break;                                  \
    }                                                                                \
  }
  if (dtype == kF32) {
    if (per_head) { ALOFA_SCAN_K(float, true) } else { ALOFA_SCAN_K(float, false) }
  } else {
    if (per_head) { ALOFA_SCAN_K(bf16_t, true) } else { ALOFA_SCAN_K(bf16_t, false) }
  }
#undef ALOFA_SCAN_K
#undef ALOFA_SCAN
  return check_launch("linear_recurrence");
}
