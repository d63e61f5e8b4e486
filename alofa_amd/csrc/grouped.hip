// Many small matrix products in one launch, each with a matrix of its own: the heads of a layer (head a's
// channels of every row against W[a]) and the experts of a mixture (the rows that take expert e against W[e]).
//
// A task is a tile of 16 rows that share a matrix, times a group of NC * 16 output columns; a wavefront owns a
// task, a block four of them. v_mfma_f32_16x16x32_bf16 with the matrix as the A operand and the rows as B
// (lane l: A holds matrix row l % 16, B holds input row l % 16, both the reduction indices 8 * (l / 16) .. + 7;
// D holds input row l % 16 and outputs 4 * (l / 16) .. + 3), so that a lane ends with four consecutive outputs
// of one row. Operands come straight from memory (the matrices are small or shared by many tiles and stay in
// the caches); one accumulator per output, ascending k, so a row's result depends on nothing but that row.
//
// Two ways of naming the tiles. Dense: tile = batch * tiles_per_batch + row tile, rows are the step's rows.
// Listed: tile_batch[tile] names the batch (-1: nothing), the tile's rows are the slots 16 * tile .. + 15, and
// row_in[slot] names the input row (-1: nothing); the output row is the slot.
#include "common.h"

#include <stdlib.h>

namespace alofa {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

enum GroupedEpilogue : int { kGrStore = 0, kGrSigmoidGate = 1, kGrClampedGlu = 2 };

struct GroupedShape {
  int64_t out_stride, out_batch_step;   // out[row, batch * out_batch_step + o]
  int64_t x_stride, x_batch_step;       // x[row, batch * x_batch_step + k]
  int64_t w_stride, w_batch_step;       // W[batch * w_batch_step + o * w_stride + k]
  int n_out, K;                         // outputs and reduction length of a batch ...
  int last_batch, n_out_last, K_last;   // ... and of the batch `last_batch`, which may differ (-1: none does)
  int rows;                             // dense: rows of the step; listed: slots
  int x_by_slot;                        // listed: the input row is the slot itself (row_in only says which slots are in use)
  int tiles, tiles_per_batch;           // tiles in all; dense: row tiles of a batch (0: listed)
  int64_t gate_stride;                  // kGrSigmoidGate: gate[row, batch * out_batch_step + o]
  float limit, limit_last, slope, offset;       // kGrClampedGlu: a sigmoid(slope a) (b + offset)
};

// Every lane issues every load (from the operand's first bytes where its own are not wanted) and what is not wanted is cleared
// afterwards: loads under a branch are waited for one by one, loads without one are in flight together.
__device__ __forceinline__ uint4 grouped_load(const bf16_t* __restrict__ base, int64_t offset, bool ok) {
  return *reinterpret_cast<const uint4*>(base + (ok ? offset : 0));
}
__device__ __forceinline__ bf16x8 grouped_frag(uint4 v, bool ok) {
  if (!ok) v = make_uint4(0, 0, 0, 0);
  return __builtin_bit_cast(bf16x8, v);
}

// RT: 16-row tiles a task takes together (a tile is then 16 * RT rows): a fragment of the matrix serves them all.
// KW: wavefronts that share a task's reduction (1: a block runs four tasks, a wavefront each; 4: a block runs one task, wavefront w
// takes the steps of 32 along K numbered w, w + 4, ..., and the four partial sums are added in LDS in the wavefronts' order: for
// steps of few rows, where the tasks are few and a lone wavefront's chain of loads is what the launch waits for).
// kAhead: steps of 32 along K whose loads are issued together.
template <int RT, int NC, int KW, int kEpilogue, typename TO>
__global__ void __launch_bounds__(256) grouped_product_kernel(TO* __restrict__ out, const bf16_t* __restrict__ x, const bf16_t* __restrict__ W,
                                                              const bf16_t* __restrict__ W2, const int32_t* __restrict__ tile_batch,
                                                              const int32_t* __restrict__ row_in, const bf16_t* __restrict__ gate,
                                                              const float* __restrict__ slot_weight, GroupedShape s, int col_groups) {
  constexpr bool kGlu = kEpilogue == kGrClampedGlu;
  constexpr int kAhead = RT == 1 ? 4 : 2;
  constexpr int kSums = kGlu ? 2 : 1;
  __shared__ f32x4 red[KW == 1 ? 1 : 3][KW == 1 ? 1 : RT * NC * kSums][KW == 1 ? 1 : 64];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int64_t task = KW == 1 ? static_cast<int64_t>(blockIdx.x) * 4 + wave : blockIdx.x;
  const int kw = KW == 1 ? 0 : wave;
  const int tile = static_cast<int>(task / col_groups), cg = static_cast<int>(task % col_groups);
  if (tile >= s.tiles) return;
  int batch, slot0;
  if (s.tiles_per_batch > 0) {
    batch = tile / s.tiles_per_batch;
    slot0 = (tile % s.tiles_per_batch) * 16 * RT;
  } else {
    batch = tile_batch[tile];
    slot0 = tile * 16 * RT;
  }
  if (batch < 0) return;
  const bool last = batch == s.last_batch;
  const int n_out = last ? s.n_out_last : s.n_out, K = last ? s.K_last : s.K;
  const int o0 = cg * NC * 16;
  if (o0 >= n_out) return;
  const int r = lane % 16, kq = (lane / 16) * 8;
  int row[RT];
  int64_t x_at[RT];
  bool any = false;
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    const int slot = slot0 + t * 16 + r;
    row[t] = -1;
    if (slot < s.rows) row[t] = row_in ? row_in[slot] : slot;
    x_at[t] = static_cast<int64_t>(row[t] < 0 ? 0 : (s.x_by_slot ? slot : row[t])) * s.x_stride + batch * s.x_batch_step;
    any = any || row[t] >= 0;
  }
  if (!__any(any)) return;      // (the whole block alike when it shares a task: no barrier is left waiting)
  const bf16_t* wb = W + batch * s.w_batch_step, *wb2 = kGlu ? W2 + batch * s.w_batch_step : nullptr;
  int64_t w_at[NC];
  bool o_ok[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int o = o0 + c * 16 + r;
    o_ok[c] = o < n_out;
    w_at[c] = static_cast<int64_t>(o_ok[c] ? o : 0) * s.w_stride;
  }
  f32x4 acc[RT][NC], acc2[RT][NC];
#pragma unroll
  for (int t = 0; t < RT; ++t)
#pragma unroll
    for (int c = 0; c < NC; ++c) acc[t][c] = acc2[t][c] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = kw * 32; k0 < K; k0 += 32 * KW * kAhead) {
    uint4 xv[kAhead][RT], wv[kAhead][NC], wv2[kAhead][kGlu ? NC : 1];
#pragma unroll
    for (int a = 0; a < kAhead; ++a) {
      const int k = k0 + a * 32 * KW + kq;
      const bool k_ok = k < K;
#pragma unroll
      for (int t = 0; t < RT; ++t) xv[a][t] = grouped_load(x, x_at[t] + k, k_ok);
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        wv[a][c] = grouped_load(wb, w_at[c] + k, k_ok);
        if constexpr (kGlu) wv2[a][c] = grouped_load(wb2, w_at[c] + k, k_ok);
      }
    }
#pragma unroll
    for (int a = 0; a < kAhead; ++a) {
      const bool k_ok = k0 + a * 32 * KW + kq < K;
      bf16x8 xf[RT];
#pragma unroll
      for (int t = 0; t < RT; ++t) xf[t] = grouped_frag(xv[a][t], k_ok && row[t] >= 0);
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const bf16x8 wf = grouped_frag(wv[a][c], k_ok && o_ok[c]);
#pragma unroll
        for (int t = 0; t < RT; ++t) acc[t][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, xf[t], acc[t][c], 0, 0, 0);
        if constexpr (kGlu) {
          const bf16x8 wf2 = grouped_frag(wv2[a][c], k_ok && o_ok[c]);
#pragma unroll
          for (int t = 0; t < RT; ++t) acc2[t][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf2, xf[t], acc2[t][c], 0, 0, 0);
        }
      }
    }
  }
  if constexpr (KW > 1) {      // the partial sums of wavefronts 1, 2, 3 join wavefront 0's, in that order
    if (wave > 0) {
#pragma unroll
      for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          red[wave - 1][(t * NC + c) * kSums][lane] = acc[t][c];
          if constexpr (kGlu) red[wave - 1][(t * NC + c) * kSums + 1][lane] = acc2[t][c];
        }
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int w = 0; w < 3; ++w)
#pragma unroll
      for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          acc[t][c] += red[w][(t * NC + c) * kSums][lane];
          if constexpr (kGlu) acc2[t][c] += red[w][(t * NC + c) * kSums + 1][lane];
        }
  }
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    if (row[t] < 0) continue;
    const int slot = slot0 + t * 16 + r;
    const int out_row = s.tiles_per_batch > 0 ? row[t] : slot;
    TO* dst = out + static_cast<int64_t>(out_row) * s.out_stride + batch * s.out_batch_step;
    float weight = 1.f, lim = 0.f;
    if constexpr (kGlu) {
      weight = slot_weight ? slot_weight[slot] : 1.f;
      lim = last ? s.limit_last : s.limit;
    }
#pragma unroll
    for (int c = 0; c < NC; ++c) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int o = o0 + c * 16 + (lane / 16) * 4 + i;
        if (o >= n_out) continue;
        float y = acc[t][c][i];
        if constexpr (kEpilogue == kGrSigmoidGate) {
          const float g = bf16_to_f32(gate[static_cast<int64_t>(out_row) * s.gate_stride + batch * s.out_batch_step + o]);
          y *= 1.f / (1.f + __expf(-g));
        } else if constexpr (kGlu) {
          const float a = fminf(y, lim);
          const float b = fminf(fmaxf(acc2[t][c][i], -lim), lim);
          y = weight * (a * (1.f / (1.f + __expf(-s.slope * a))) * (b + s.offset));
        }
        store_f32(dst + o, y);
      }
    }
  }
}

// ---- tiles of 64 rows through LDS ---------------------------------------------------------------------------
// The same products for steps of many rows: a block owns a tile of 64 rows and 256 rows of the matrix (256 output columns, or,
// for the GLU, 128 gate and 128 up rows of the same columns), a wavefront 64 x 64 of it. Slabs of 32 along K take turns in two
// LDS buffers: while the block multiplies one, every thread has the next one's five 16-byte pieces on their way in registers. A
// slab's row is 64 bytes, its four pieces permuted by (row >> 2) & 3, so that the sixteen rows a quarter of a wavefront reads
// together fall on distinct banks. Fragments and sums are those of the kernel above (one accumulator an output, ascending k).
template <int kEpilogue, typename TO>
__global__ void __launch_bounds__(256) grouped_tiled_kernel(TO* __restrict__ out, const bf16_t* __restrict__ x, const bf16_t* __restrict__ W,
                                                            const bf16_t* __restrict__ W2, const int32_t* __restrict__ tile_batch,
                                                            const int32_t* __restrict__ row_in, const bf16_t* __restrict__ gate,
                                                            const float* __restrict__ slot_weight, GroupedShape s, int col_blocks) {
  constexpr bool kGlu = kEpilogue == kGrClampedGlu;
  constexpr int kCols = kGlu ? 128 : 256;      // output columns of a block
  __shared__ __attribute__((aligned(16))) uint4 xs[2][64 * 4], ws[2][256 * 4];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int tile = blockIdx.x / col_blocks, cb = blockIdx.x % col_blocks;
  int batch, slot0;
  if (s.tiles_per_batch > 0) {
    batch = tile / s.tiles_per_batch;
    slot0 = (tile % s.tiles_per_batch) * 64;
  } else {
    batch = tile_batch[tile];
    slot0 = tile * 64;
  }
  if (batch < 0) return;
  const bool last = batch == s.last_batch;
  const int n_out = last ? s.n_out_last : s.n_out, K = last ? s.K_last : s.K;
  const int o0 = cb * kCols;
  if (o0 >= n_out) return;
  // what this thread brings in of every slab: piece `pc` of row `lr` of the rows, and of four rows of the matrix
  const int lr = threadIdx.x / 4, pc = threadIdx.x % 4;
  const int my_slot = slot0 + lr;
  int my_row = -1;
  if (my_slot < s.rows) my_row = row_in ? row_in[my_slot] : my_slot;
  const bf16_t* x_src = x + static_cast<int64_t>(my_row < 0 ? 0 : (s.x_by_slot ? my_slot : my_row)) * s.x_stride + batch * s.x_batch_step;
  const bf16_t* w_src[4];
  bool w_ok[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int wr = lr + 64 * j;      // row of the block's 256 staged matrix rows
    const int o = o0 + (kGlu ? wr % 128 : wr);
    w_ok[j] = o < n_out;
    w_src[j] = ((kGlu && wr >= 128) ? W2 : W) + batch * s.w_batch_step + static_cast<int64_t>(w_ok[j] ? o : 0) * s.w_stride;
  }
  const int x_dst = lr * 4 + (pc ^ ((lr >> 2) & 3));
  // this wavefront's four chunks of 16 staged matrix rows: its 64 columns, or its 32 gate columns and the same 32 up columns
  int chunk_row[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) chunk_row[c] = kGlu ? (c < 2 ? wave * 32 + c * 16 : 128 + wave * 32 + (c - 2) * 16) : wave * 64 + c * 16;
  const int r = lane % 16, q = lane / 16;
  f32x4 acc[4][4];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[t][c] = f32x4{0.f, 0.f, 0.f, 0.f};
  uint4 xv, wv[4];
  auto fetch = [&](int k0) {
    const bool k_ok = k0 + pc * 8 < K;
    const int64_t k = k_ok ? k0 + pc * 8 : 0;      // (a piece past the end of K reads the row's first bytes and is cleared)
    xv = *reinterpret_cast<const uint4*>(x_src + k);
#pragma unroll
    for (int j = 0; j < 4; ++j) wv[j] = *reinterpret_cast<const uint4*>(w_src[j] + k);
    if (!k_ok || my_row < 0) xv = make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (!k_ok || !w_ok[j]) wv[j] = make_uint4(0, 0, 0, 0);
  };
  auto stage = [&](int buf) {
    xs[buf][x_dst] = xv;
#pragma unroll
    for (int j = 0; j < 4; ++j) ws[buf][(lr + 64 * j) * 4 + (pc ^ ((lr >> 2) & 3))] = wv[j];      // ((lr + 64 j) >> 2) & 3 == (lr >> 2) & 3
  };
  fetch(0);
  stage(0);
  __syncthreads();
  const int slabs = (K + 31) / 32;
  for (int sl = 0; sl < slabs; ++sl) {
    const int buf = sl & 1;
    if (sl + 1 < slabs) fetch((sl + 1) * 32);
    bf16x8 xf[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int row = t * 16 + r;
      xf[t] = __builtin_bit_cast(bf16x8, xs[buf][row * 4 + (q ^ ((row >> 2) & 3))]);
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int row = chunk_row[c] + r;
      const bf16x8 wf = __builtin_bit_cast(bf16x8, ws[buf][row * 4 + (q ^ ((row >> 2) & 3))]);
#pragma unroll
      for (int t = 0; t < 4; ++t) acc[t][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, xf[t], acc[t][c], 0, 0, 0);
    }
    if (sl + 1 < slabs) stage(buf ^ 1);
    __syncthreads();
  }
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int slot = slot0 + t * 16 + r;
    int row = -1;
    if (slot < s.rows) row = row_in ? row_in[slot] : slot;
    if (row < 0) continue;
    const int out_row = s.tiles_per_batch > 0 ? row : slot;
    TO* dst = out + static_cast<int64_t>(out_row) * s.out_stride + batch * s.out_batch_step;
    float weight = 1.f, lim = 0.f;
    if constexpr (kGlu) {
      weight = slot_weight ? slot_weight[slot] : 1.f;
      lim = last ? s.limit_last : s.limit;
    }
#pragma unroll
    for (int c = 0; c < (kGlu ? 2 : 4); ++c) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int o = o0 + (kGlu ? wave * 32 : wave * 64) + c * 16 + q * 4 + i;
        if (o >= n_out) continue;
        float y = acc[t][c][i];
        if constexpr (kEpilogue == kGrSigmoidGate) {
          const float g = bf16_to_f32(gate[static_cast<int64_t>(out_row) * s.gate_stride + batch * s.out_batch_step + o]);
          y *= 1.f / (1.f + __expf(-g));
        } else if constexpr (kGlu) {
          const float a = fminf(y, lim);
          const float b = fminf(fmaxf(acc[t][c + 2][i], -lim), lim);
          y = weight * (a * (1.f / (1.f + __expf(-s.slope * a))) * (b + s.offset));
        }
        store_f32(dst + o, y);
      }
    }
  }
}

// ---- the rows of every expert, side by side ------------------------------------------------------------------
// chosen, weights [T, top]: the experts a row takes and its weights. Slots: every expert's rows together, an
// expert's share padded to a multiple of `pad` (a tile's rows: 16 or 64), in expert order; then (with `shared`) all T rows once more for the
// expert every row takes, as batch E. Outputs: row_in[slot] (the row, or -1), slot_weight[slot], slot_of[t * top + k]
// (where row t's k-th choice went) and slot_of[T * top + t] (its slot of the shared expert), tile_batch[tile] (the
// expert of a tile of `pad` slots, -1 beyond the last). Which slot of its expert's share a row gets depends on the
// order in which threads arrive, which changes no result: a slot's values depend on its row alone.
// One block; experts up to 512.
__global__ void __launch_bounds__(1024) expert_rows_kernel(const int32_t* __restrict__ chosen, const float* __restrict__ weights, int32_t* __restrict__ row_in,
                                                           float* __restrict__ slot_weight, int32_t* __restrict__ slot_of, int32_t* __restrict__ tile_batch,
                                                           int T, int top, int experts, int shared, int slots, int tiles, int pad) {
  __shared__ int count[512], first[513], cursor[512];
  for (int e = threadIdx.x; e < experts; e += 1024) count[e] = cursor[e] = 0;
  for (int i = threadIdx.x; i < slots; i += 1024) {
    row_in[i] = -1;
    slot_weight[i] = 0.f;
  }
  for (int i = threadIdx.x; i < tiles; i += 1024) tile_batch[i] = -1;
  __syncthreads();
  const int pairs = T * top;
  for (int i = threadIdx.x; i < pairs; i += 1024)
    if (chosen[i] >= 0 && chosen[i] < experts) atomicAdd(&count[chosen[i]], 1);      // (a choice beyond the experts with matrices takes no slot)
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0;
    for (int e = 0; e < experts; ++e) {
      first[e] = at;
      at += (count[e] + pad - 1) / pad * pad;
    }
    first[experts] = at;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < experts; e += 1024)
    for (int t = first[e] / pad; t < first[e + 1] / pad; ++t) tile_batch[t] = e;
  for (int i = threadIdx.x; i < pairs; i += 1024) {
    const int e = chosen[i];
    if (e < 0 || e >= experts) {
      slot_of[i] = -1;
      continue;
    }
    const int slot = first[e] + atomicAdd(&cursor[e], 1);
    row_in[slot] = i / top;
    slot_weight[slot] = weights[i];
    slot_of[i] = slot;
  }
  if (shared) {
    const int base = first[experts];
    for (int t = threadIdx.x; t < T; t += 1024) {
      row_in[base + t] = t;
      slot_weight[base + t] = 1.f;
      slot_of[pairs + t] = base + t;
    }
    for (int t = threadIdx.x; t < (T + pad - 1) / pad; t += 1024) tile_batch[base / pad + t] = experts;
  }
}

// ---- residual[t, c] += scale[c] * sum_k y[slot_of[t, k], c], k ascending (then the shared expert's) --------------
__global__ void __launch_bounds__(256) experts_sum_kernel(float* __restrict__ residual, const float* __restrict__ y, const int32_t* __restrict__ slot_of,
                                                          const float* __restrict__ scale, int T, int width, int top, int shared,
                                                          const float* __restrict__ pass_weight, const bf16_t* __restrict__ pass_x, int64_t pass_stride, int assign) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= static_cast<int64_t>(T) * width) return;
  const int t = static_cast<int>(idx / width), c = static_cast<int>(idx % width);
  float sum = 0.f;
  for (int k = 0; k < top; ++k) {
    const int slot = slot_of[t * top + k];
    if (slot >= 0) sum += y[static_cast<int64_t>(slot) * width + c];      // (-1: a choice without a slot)
  }
  if (shared) sum += y[static_cast<int64_t>(slot_of[T * top + t]) * width + c];
  if (pass_weight) sum += pass_weight[t] * bf16_to_f32(pass_x[static_cast<int64_t>(t) * pass_stride + c]);      // (the row itself, handed on with a weight)
  if (scale) sum *= scale[c];
  residual[idx] = assign ? sum : residual[idx] + sum;
}

}  // namespace alofa

using namespace alofa;

// ALOFA_GROUPED_LDS=0 (read once; for measurements): tiles of 64 rows run without the LDS stage
static const bool g_tiled = [] { const char* v = getenv("ALOFA_GROUPED_LDS"); return !(v && v[0] == '0'); }();

template <int kEpilogue, typename TO>
static int launch_grouped(void* out, const void* x, const void* W, const void* W2, const int32_t* tile_batch, const int32_t* row_in, const void* gate,
                          const float* slot_weight, const GroupedShape& s, int tile_rows, hipStream_t stream) {
  const int widest = s.n_out > s.n_out_last ? s.n_out : s.n_out_last;
  // Tiles of 64 rows: a wavefront a task of 64 columns. Tiles of 16 rows: while the tasks of 64 columns are too few to give every
  // SIMD of the chip two wavefronts, a block a task of 32 or 16 columns, its four wavefronts sharing the reduction.
  const int64_t wide_tasks = static_cast<int64_t>(s.tiles) * ((widest + 63) / 64);
  const int64_t fill = 2 * static_cast<int64_t>(compute_units()) * 4;
  const bool shared_k = tile_rows == 16 && wide_tasks < fill;
  const int nc = !shared_k ? 4 : (wide_tasks * 4 >= fill ? 2 : 1);
  const int col_groups = (widest + nc * 16 - 1) / (nc * 16);
  const int64_t tasks = static_cast<int64_t>(s.tiles) * col_groups;
  const unsigned grid = static_cast<unsigned>(shared_k ? tasks : (tasks + 3) / 4);
#define ALOFA_GROUPED(RT, NC, KW) grouped_product_kernel<RT, NC, KW, kEpilogue, TO><<<grid, 256, 0, stream>>>(static_cast<TO*>(out), static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(W), \
    static_cast<const bf16_t*>(W2), tile_batch, row_in, static_cast<const bf16_t*>(gate), slot_weight, s, col_groups)
  if (tile_rows == 64 && g_tiled) {
    const int col_blocks = (widest + (kEpilogue == kGrClampedGlu ? 128 : 256) - 1) / (kEpilogue == kGrClampedGlu ? 128 : 256);
    grouped_tiled_kernel<kEpilogue, TO><<<static_cast<unsigned>(s.tiles) * col_blocks, 256, 0, stream>>>(
        static_cast<TO*>(out), static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(W), static_cast<const bf16_t*>(W2), tile_batch, row_in,
        static_cast<const bf16_t*>(gate), slot_weight, s, col_blocks);
  } else if (tile_rows == 64) ALOFA_GROUPED(4, 4, 1);
  else if (!shared_k) ALOFA_GROUPED(1, 4, 1);
  else if (nc == 2) ALOFA_GROUPED(1, 2, 4);
  else ALOFA_GROUPED(1, 1, 4);
#undef ALOFA_GROUPED
  return check_launch("grouped_product");
}

// out dtype: kBF16 or kF32; x, W, W2, gate bfloat16. epilogue: 0 store, 1 times sigmoid(gate), 2 clamped GLU of (W, W2) times slot_weight.
extern "C" int alofa_grouped_product(void* out, int out_dtype, int64_t out_stride, int64_t out_batch_step, const void* x, int64_t x_stride, int64_t x_batch_step,
                                     const void* W, const void* W2, int64_t w_stride, int64_t w_batch_step, int n_out, int K, int last_batch, int n_out_last,
                                     int K_last, int rows, int x_by_slot, int tiles, int tiles_per_batch, int tile_rows, const int32_t* tile_batch, const int32_t* row_in, const void* gate,
                                     int64_t gate_stride, const float* slot_weight, float limit, float limit_last, float slope, float offset, int epilogue, hipStream_t stream) {
  ALOFA_REQUIRE(n_out > 0 && K > 0 && rows >= 0 && tiles >= 0, "grouped_product: bad sizes (n_out=%d K=%d rows=%d tiles=%d)", n_out, K, rows, tiles);
  ALOFA_REQUIRE(K % 8 == 0 && K_last % 8 == 0 && x_stride % 8 == 0 && x_batch_step % 8 == 0 && w_stride % 8 == 0 && w_batch_step % 8 == 0 &&
                    reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(W) % 16 == 0 && (W2 == nullptr || reinterpret_cast<uintptr_t>(W2) % 16 == 0),
                "grouped_product: operands must be 16-byte aligned along the reduction (K=%d x_stride=%lld w_stride=%lld)", K, (long long)x_stride, (long long)w_stride);
  ALOFA_REQUIRE((tiles_per_batch > 0) != (tile_batch != nullptr), "grouped_product: tiles are dense (tiles_per_batch) or listed (tile_batch)");
  ALOFA_REQUIRE(tile_rows == 16 || tile_rows == 64, "grouped_product: tiles of 16 or 64 rows (tile_rows=%d)", tile_rows);
  ALOFA_REQUIRE(epilogue != kGrSigmoidGate || gate, "grouped_product: the gate epilogue needs gates");
  ALOFA_REQUIRE(epilogue != kGrClampedGlu || (W2 && out_dtype == kBF16), "grouped_product: the GLU epilogue needs a second matrix and writes bfloat16");
  if (rows == 0 || tiles == 0) return 0;
  GroupedShape s{out_stride, out_batch_step, x_stride, x_batch_step, w_stride, w_batch_step, n_out, K, last_batch, n_out_last, K_last, rows, x_by_slot, tiles, tiles_per_batch,
                 gate_stride, limit, limit_last, slope, offset};
  if (epilogue == kGrStore && out_dtype == kBF16) return launch_grouped<kGrStore, bf16_t>(out, x, W, W2, tile_batch, row_in, gate, slot_weight, s, tile_rows, stream);
  if (epilogue == kGrStore && out_dtype == kF32) return launch_grouped<kGrStore, float>(out, x, W, W2, tile_batch, row_in, gate, slot_weight, s, tile_rows, stream);
  if (epilogue == kGrSigmoidGate && out_dtype == kBF16) return launch_grouped<kGrSigmoidGate, bf16_t>(out, x, W, W2, tile_batch, row_in, gate, slot_weight, s, tile_rows, stream);
  if (epilogue == kGrClampedGlu) return launch_grouped<kGrClampedGlu, bf16_t>(out, x, W, W2, tile_batch, row_in, gate, slot_weight, s, tile_rows, stream);
  ALOFA_REQUIRE(false, "grouped_product: no such epilogue and output type (epilogue=%d out=%d)", epilogue, out_dtype);
  return 1;
}

extern "C" int alofa_expert_rows(const int32_t* chosen, const float* weights, int32_t* row_in, float* slot_weight, int32_t* slot_of, int32_t* tile_batch,
                                 int T, int top, int experts, int shared, int slots, int tiles, int pad, hipStream_t stream) {
  ALOFA_REQUIRE(T > 0 && top > 0 && experts > 0 && experts <= 512 && top <= experts, "expert_rows: bad sizes (T=%d top=%d experts=%d)", T, top, experts);
  ALOFA_REQUIRE(pad == 16 || pad == 64, "expert_rows: tiles of 16 or 64 rows (pad=%d)", pad);
  const int64_t need = (static_cast<int64_t>(T) * top + pad - 1) / pad * pad + pad * static_cast<int64_t>(experts) + (shared ? (T + pad - 1) / pad * pad : 0);
  ALOFA_REQUIRE(slots >= need && static_cast<int64_t>(tiles) * pad >= slots, "expert_rows: room for %lld slots is needed (slots=%d tiles=%d)", (long long)need, slots, tiles);
  expert_rows_kernel<<<1, 1024, 0, stream>>>(chosen, weights, row_in, slot_weight, slot_of, tile_batch, T, top, experts, shared, slots, tiles, pad);
  return check_launch("expert_rows");
}

extern "C" int alofa_experts_sum(float* residual, const float* y, const int32_t* slot_of, const float* scale, int T, int width, int top, int shared,
                                 const float* pass_weight, const void* pass_x, int64_t pass_stride, int assign, hipStream_t stream) {
  ALOFA_REQUIRE(T >= 0 && width > 0 && top > 0, "experts_sum: bad sizes");
  if (T == 0) return 0;
  experts_sum_kernel<<<static_cast<unsigned>((static_cast<int64_t>(T) * width + 255) / 256), 256, 0, stream>>>(residual, y, slot_of, scale, T, width, top, shared, pass_weight, static_cast<const bf16_t*>(pass_x), pass_stride, assign);
  return check_launch("experts_sum");
}
