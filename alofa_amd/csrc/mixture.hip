// Feed-forwards of which every token takes a few (a mixture of experts): the choice, and the gated
// activation of the experts.
//
// The choice is float arithmetic on float scores (double in the exact path); ties go to the lower index.
#include "common.h"

namespace alofa {

// ---- the choice -------------------------------------------------------------------------------
// z [T, E] router products. Per token the `top` experts with the largest z (the same as the largest
// sigmoid(z), without its saturation), the lower index first among equals. Outputs:
//   dense [T, E]: sigmoid(z) * scale at the chosen experts, 0 elsewhere (weights sum to one first when `renorm`);
//   chosen [T, top], weights [T, top]: the same as lists, in order of falling score.
// A wavefront per token: lane l holds the products l, l + 64, ... (E up to kMaxExperts); a pick is the best of the lanes'
// own bests, found by exchanges between lanes (value falling, index rising).
constexpr int kMaxExperts = 512;

template <typename Acc>
__global__ void __launch_bounds__(256) route_top_kernel(const float* __restrict__ z, float* __restrict__ dense, int32_t* __restrict__ chosen,
                                                        float* __restrict__ weights, int tokens, int experts, int top, float scale, int renorm) {
  constexpr int kOwn = kMaxExperts / kWave;
  const int t = blockIdx.x * 4 + threadIdx.x / kWave, lane = threadIdx.x % kWave;
  if (t >= tokens) return;
  const float* row = z + static_cast<int64_t>(t) * experts;
  float* d = dense + static_cast<int64_t>(t) * experts;
  float own[kOwn];
  bool taken[kOwn];
#pragma unroll
  for (int i = 0; i < kOwn; ++i) {
    const int e = lane + i * kWave;
    own[i] = e < experts ? row[e] : 0.f;
    taken[i] = e >= experts;
    if (e < experts) d[e] = 0.f;
  }
  Acc total = 0;
  for (int k = 0; k < top; ++k) {
    float best = 0.f;
    int best_e = 1 << 30;
#pragma unroll
    for (int i = 0; i < kOwn; ++i) {
      const int e = lane + i * kWave;
      if (!taken[i] && (best_e == 1 << 30 || own[i] > best)) {      // (rising e within the lane: the first of equals stays)
        best = own[i];
        best_e = e;
      }
    }
#pragma unroll
    for (int m = 1; m < kWave; m <<= 1) {
      const float other = __shfl_xor(best, m);
      const int other_e = __shfl_xor(best_e, m);
      if (other_e != 1 << 30 && (best_e == 1 << 30 || other > best || (other == best && other_e < best_e))) {
        best = other;
        best_e = other_e;
      }
    }
#pragma unroll
    for (int i = 0; i < kOwn; ++i)
      if (lane + i * kWave == best_e) taken[i] = true;
    const Acc s = static_cast<Acc>(1) / (static_cast<Acc>(1) + exp(-static_cast<Acc>(best)));
    total += s;
    if (lane == 0) {
      chosen[static_cast<int64_t>(t) * top + k] = best_e;
      weights[static_cast<int64_t>(t) * top + k] = static_cast<float>(s);      // (made final below)
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  if (lane == 0) {
    for (int k = 0; k < top; ++k) {
      Acc w = static_cast<Acc>(weights[static_cast<int64_t>(t) * top + k]);
      if (renorm) w /= total;
      const float f = static_cast<float>(w * static_cast<Acc>(scale));
      weights[static_cast<int64_t>(t) * top + k] = f;
      d[chosen[static_cast<int64_t>(t) * top + k]] = f;
    }
  }
}

// ---- the choice among experts in groups, by softmax scores with a correction -----------------------------------
// z [T, E] router products over all experts, the last `pass` of which hand their input on (they have no matrices).
// s = softmax(z); the choice goes by c = s + correction; the experts form `groups` equal groups of neighbours, a group's
// score is its largest c, and only experts of the `keep` best groups can be taken (the lower group among equals); of those
// the `top` with the largest c (the lower index among equals); their weights are their s (times `scale`; made to sum to one
// first when `renorm`). Outputs: chosen, weights [T, top] in order of falling c; dense [T, E - pass] the weights at the taken
// experts with matrices, 0 elsewhere; pass_weight [T] the sum of the weights of taken experts without.
// A wavefront per token; lane l holds the experts l, l + 64, ...
template <typename Acc>
__global__ void __launch_bounds__(256) route_groups_kernel(const float* __restrict__ z, const float* __restrict__ correction, float* __restrict__ dense,
                                                           int32_t* __restrict__ chosen, float* __restrict__ weights, float* __restrict__ pass_weight,
                                                           int tokens, int experts, int pass, int top, int groups, int keep, float scale, int renorm) {
  constexpr int kOwn = kMaxExperts / kWave;
  __shared__ float group_best[4][kMaxExperts], all_scores[4][kMaxExperts];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int t = blockIdx.x * 4 + wave;
  if (t >= tokens) return;      // (no block-wide barrier below: a wavefront is on its own)
  const float* row = z + static_cast<int64_t>(t) * experts;
  const int real = experts - pass, size = experts / groups;
  float* d = dense + static_cast<int64_t>(t) * real;
  float zs[kOwn];
  float top_z = -3.402823466e+38f;
#pragma unroll
  for (int i = 0; i < kOwn; ++i) {
    const int e = lane + i * kWave;
    zs[i] = e < experts ? row[e] : -3.402823466e+38f;
    top_z = fmaxf(top_z, zs[i]);
    if (e < real) d[e] = 0.f;
  }
  top_z = wave_max(top_z);
  Acc ex[kOwn], sum = 0;
#pragma unroll
  for (int i = 0; i < kOwn; ++i) {
    const int e = lane + i * kWave;
    ex[i] = e < experts ? exp(static_cast<Acc>(zs[i]) - static_cast<Acc>(top_z)) : static_cast<Acc>(0);
    sum += ex[i];
  }
  sum = wave_sum(sum);
  float s[kOwn], c[kOwn];
  bool taken[kOwn];
  float* best = group_best[wave];
  float* all = all_scores[wave];
#pragma unroll
  for (int i = 0; i < kOwn; ++i) {
    const int e = lane + i * kWave;
    s[i] = static_cast<float>(ex[i] / sum);
    c[i] = e < experts ? static_cast<float>(static_cast<Acc>(s[i]) + static_cast<Acc>(correction ? correction[e] : 0.f)) : 0.f;
    if (e < experts) all[e] = c[i];
  }
  wave_lds_sync();
  for (int g = lane; g < groups; g += kWave) {      // a group's score: the largest of its members' (a lane a group)
    float m = all[g * size];
    for (int o = 1; o < size; ++o) m = fmaxf(m, all[g * size + o]);
    best[g] = m;
  }
  wave_lds_sync();
#pragma unroll
  for (int i = 0; i < kOwn; ++i) {
    const int e = lane + i * kWave;
    taken[i] = true;
    if (e < experts) {
      const int g = e / size;
      const float mine = best[g];
      int ahead = 0;      // groups that come before this one: a larger best, or an equal one with a lower index
      for (int o = 0; o < groups; ++o) ahead += (best[o] > mine || (best[o] == mine && o < g)) ? 1 : 0;
      taken[i] = ahead >= keep;      // (out of the choice from the start)
    }
  }
  Acc total = 0, passed = 0;
  for (int k = 0; k < top; ++k) {
    float bc = 0.f, bs = 0.f;
    int be = 1 << 30;
#pragma unroll
    for (int i = 0; i < kOwn; ++i) {
      const int e = lane + i * kWave;
      if (!taken[i] && (be == 1 << 30 || c[i] > bc)) {
        bc = c[i];
        bs = s[i];
        be = e;
      }
    }
#pragma unroll
    for (int m = 1; m < kWave; m <<= 1) {
      const float oc = __shfl_xor(bc, m), os = __shfl_xor(bs, m);
      const int oe = __shfl_xor(be, m);
      if (oe != 1 << 30 && (be == 1 << 30 || oc > bc || (oc == bc && oe < be))) {
        bc = oc;
        bs = os;
        be = oe;
      }
    }
#pragma unroll
    for (int i = 0; i < kOwn; ++i)
      if (lane + i * kWave == be) taken[i] = true;
    total += static_cast<Acc>(bs);
    if (lane == 0) {
      chosen[static_cast<int64_t>(t) * top + k] = be == 1 << 30 ? -1 : be;
      weights[static_cast<int64_t>(t) * top + k] = be == 1 << 30 ? 0.f : bs;      // (made final below)
    }
  }
  wave_lds_sync();
  if (lane == 0) {
    for (int k = 0; k < top; ++k) {
      const int e = chosen[static_cast<int64_t>(t) * top + k];
      Acc w = static_cast<Acc>(weights[static_cast<int64_t>(t) * top + k]);
      if (renorm) w /= total;
      const float f = static_cast<float>(w * static_cast<Acc>(scale));
      weights[static_cast<int64_t>(t) * top + k] = f;
      if (e >= 0 && e < real) d[e] = f;
      else if (e >= real) passed += static_cast<Acc>(f);
    }
    if (pass_weight) pass_weight[t] = static_cast<float>(passed);
  }
}

// ---- gated activation of all experts side by side ------------------------------------------------
// g, u [T, F]: gate and up products of every expert (E experts of `ff` channels each, then `shared_ff` channels of an
// expert every token takes). act[t, c] = w * a * sigmoid(slope * a) * (b + 1) with a = min(g, limit),
// b = clamp(u, -limit, limit) (`offset` stands where the 1 does), and w = dense[t, expert of c] (0: the token does not take that expert) or 1 for the
// shared channels.
template <typename T, typename Acc>
__global__ void __launch_bounds__(256) clamped_glu_kernel(T* __restrict__ act, const T* __restrict__ g, const T* __restrict__ u, const float* __restrict__ dense,
                                                          int64_t rows, int experts, int ff, int shared_ff, float limit, float shared_limit, float slope, float offset) {
  const int F = experts * ff + shared_ff;
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= rows * F) return;
  const int64_t t = idx / F;
  const int c = static_cast<int>(idx % F);
  const bool own = c < experts * ff;
  const float w = own ? dense[t * experts + c / ff] : 1.f;
  float y = 0.f;
  if (w != 0.f) {
    const Acc lim = static_cast<Acc>(own ? limit : shared_limit);
    Acc a = static_cast<Acc>(load_f32(g + idx)), b = static_cast<Acc>(load_f32(u + idx));
    a = a < lim ? a : lim;
    b = b < -lim ? -lim : (b > lim ? lim : b);
    const Acc s = static_cast<Acc>(1) / (static_cast<Acc>(1) + exp(-static_cast<Acc>(slope) * a));
    y = static_cast<float>(static_cast<Acc>(w) * (a * s * (b + static_cast<Acc>(offset))));
  }
  store_f32(act + idx, y);
}

}  // namespace alofa

using namespace alofa;

extern "C" int alofa_route_top(const float* z, float* dense, int32_t* chosen, float* weights, int tokens, int experts, int top, float scale, int renorm,
                               int exact, hipStream_t stream) {
  ALOFA_REQUIRE(tokens >= 0 && experts > 0 && experts <= kMaxExperts && top > 0 && top <= experts, "route_top: bad sizes (tokens=%d experts=%d top=%d)", tokens, experts, top);
  if (tokens == 0) return 0;
  const unsigned grid = static_cast<unsigned>((tokens + 3) / 4);
  if (exact) route_top_kernel<double><<<grid, 256, 0, stream>>>(z, dense, chosen, weights, tokens, experts, top, scale, renorm);
  else route_top_kernel<float><<<grid, 256, 0, stream>>>(z, dense, chosen, weights, tokens, experts, top, scale, renorm);
  return check_launch("route_top");
}

extern "C" int alofa_clamped_glu(void* act, const void* g, const void* u, int dtype, const float* dense, int64_t rows, int experts, int ff, int shared_ff,
                                 float limit, float shared_limit, float slope, float offset, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(rows >= 0 && experts >= 0 && ff >= 0 && shared_ff >= 0 && experts * ff + shared_ff > 0 && (experts == 0 || dense), "clamped_glu: bad sizes");
  ALOFA_REQUIRE(!exact || dtype == kF32, "clamped_glu: the exact path is float32");
  if (rows == 0) return 0;
  const unsigned grid = static_cast<unsigned>((rows * (experts * ff + shared_ff) + 255) / 256);
  if (exact) clamped_glu_kernel<float, double><<<grid, 256, 0, stream>>>(static_cast<float*>(act), static_cast<const float*>(g), static_cast<const float*>(u), dense, rows, experts, ff, shared_ff, limit, shared_limit, slope, offset);
  else if (dtype == kF32) clamped_glu_kernel<float, float><<<grid, 256, 0, stream>>>(static_cast<float*>(act), static_cast<const float*>(g), static_cast<const float*>(u), dense, rows, experts, ff, shared_ff, limit, shared_limit, slope, offset);
  else clamped_glu_kernel<bf16_t, float><<<grid, 256, 0, stream>>>(static_cast<bf16_t*>(act), static_cast<const bf16_t*>(g), static_cast<const bf16_t*>(u), dense, rows, experts, ff, shared_ff, limit, shared_limit, slope, offset);
  return check_launch("clamped_glu");
}

extern "C" int alofa_route_groups(const float* z, const float* correction, float* dense, int32_t* chosen, float* weights, float* pass_weight, int tokens,
                                  int experts, int pass, int top, int groups, int keep, float scale, int renorm, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(tokens >= 0 && experts > 0 && experts <= kMaxExperts && pass >= 0 && pass < experts && top > 0 && top <= experts,
                "route_groups: bad sizes (tokens=%d experts=%d pass=%d top=%d)", tokens, experts, pass, top);
  ALOFA_REQUIRE(groups >= 1 && experts % groups == 0 && keep >= 1 && keep <= groups && top <= keep * (experts / groups),
                "route_groups: %d experts in %d groups of which %d are kept cannot give %d choices", experts, groups, keep, top);
  if (tokens == 0) return 0;
  const unsigned grid = static_cast<unsigned>((tokens + 3) / 4);
  if (exact) route_groups_kernel<double><<<grid, 256, 0, stream>>>(z, correction, dense, chosen, weights, pass_weight, tokens, experts, pass, top, groups, keep, scale, renorm);
  else route_groups_kernel<float><<<grid, 256, 0, stream>>>(z, correction, dense, chosen, weights, pass_weight, tokens, experts, pass, top, groups, keep, scale, renorm);
  return check_launch("route_groups");
}
