// Mixtures of small feed-forward layers.  The experts of a token are named by a table: looked up by token id (no
// router, equal weights), or a row per token of the step that a router has just filled (`moe_route_kernel`: softmax
// scores, groups of experts, the best of the best groups, weights from the scores).  The products here are rows
// against the weights of each row's own expert, for few rows one row at a time, for many rows sorted by expert;
// the activation between them is a kernel of its own or rides in the first product.
//
// A row's sums are formed in one fixed order (the lanes of a wave stride over the inner size, then a
// butterfly), whatever else the step holds.  Accumulation is float32 in both precisions.
#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / TL_WAVE;
// Output columns a workgroup of the per-row products owns (a quarter of them a wave): 64, or 16 in steps of few
// rows, whose waves then form one group of four sums each instead of four in a row (the grid is four times larger,
// and a decode step's handful of rows still fills the chip).
constexpr int kColsWide = 64, kColsFew = 16, kFewRows = 256;

__device__ __forceinline__ float dot_lanes(const float* __restrict__ a, const float* __restrict__ w, int K, int lane) {
  float acc = 0.f;
  if ((K & 3) == 0 && ((((uintptr_t)a) | ((uintptr_t)w)) & 15) == 0) {
    for (int k = lane * 4; k < K; k += TL_WAVE * 4) {
      const f32x4 x = *(const f32x4*)(a + k), y = *(const f32x4*)(w + k);
      acc = fmaf(x[0], y[0], acc);
      acc = fmaf(x[1], y[1], acc);
      acc = fmaf(x[2], y[2], acc);
      acc = fmaf(x[3], y[3], acc);
    }
  } else {
    for (int k = lane; k < K; k += TL_WAVE) acc = fmaf(a[k], w[k], acc);
  }
  return wave_sum(acc);
}

__device__ __forceinline__ float dot_lanes(const bf16_t* __restrict__ a, const bf16_t* __restrict__ w, int K, int lane) {
  float acc = 0.f;
  if ((K & 7) == 0 && ((((uintptr_t)a) | ((uintptr_t)w)) & 15) == 0) {
    for (int k = lane * 8; k < K; k += TL_WAVE * 8) {
      const bf16x8 x = *(const bf16x8*)(a + k), y = *(const bf16x8*)(w + k);
#pragma unroll
      for (int j = 0; j < 8; ++j) acc = fmaf((float)x[j], (float)y[j], acc);
    }
  } else {
    for (int k = lane; k < K; k += TL_WAVE) acc = fmaf((float)a[k], (float)w[k], acc);
  }
  return wave_sum(acc);
}

// Four dot products of one row at once (the loads of four weight rows in flight together); each sum is formed
// exactly as dot_lanes forms it.
__device__ __forceinline__ void dot_lanes4(const float* __restrict__ a, const float* const* w, int K, int lane, float* out) {
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  bool vec = (K & 3) == 0 && (((uintptr_t)a) & 15) == 0;
#pragma unroll
  for (int c = 0; c < 4; ++c) vec = vec && (((uintptr_t)w[c]) & 15) == 0;
  if (vec) {
    for (int k = lane * 4; k < K; k += TL_WAVE * 4) {
      const f32x4 x = *(const f32x4*)(a + k);
      f32x4 y[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) y[c] = *(const f32x4*)(w[c] + k);
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        acc[c] = fmaf(x[0], y[c][0], acc[c]);
        acc[c] = fmaf(x[1], y[c][1], acc[c]);
        acc[c] = fmaf(x[2], y[c][2], acc[c]);
        acc[c] = fmaf(x[3], y[c][3], acc[c]);
      }
    }
  } else {
    for (int k = lane; k < K; k += TL_WAVE) {
      const float x = a[k];
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[c] = fmaf(x, w[c][k], acc[c]);
    }
  }
#pragma unroll
  for (int c = 0; c < 4; ++c) out[c] = wave_sum(acc[c]);
}

__device__ __forceinline__ void dot_lanes4(const bf16_t* __restrict__ a, const bf16_t* const* w, int K, int lane, float* out) {
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  bool vec = (K & 7) == 0 && (((uintptr_t)a) & 15) == 0;
#pragma unroll
  for (int c = 0; c < 4; ++c) vec = vec && (((uintptr_t)w[c]) & 15) == 0;
  if (vec) {
    for (int k = lane * 8; k < K; k += TL_WAVE * 8) {
      const bf16x8 x = *(const bf16x8*)(a + k);
      bf16x8 y[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) y[c] = *(const bf16x8*)(w[c] + k);
#pragma unroll
      for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[c] = fmaf((float)x[j], (float)y[c][j], acc[c]);
    }
  } else {
    for (int k = lane; k < K; k += TL_WAVE) {
      const float x = (float)a[k];
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[c] = fmaf(x, (float)w[c][k], acc[c]);
    }
  }
#pragma unroll
  for (int c = 0; c < 4; ++c) out[c] = wave_sum(acc[c]);
}

__device__ __forceinline__ int expert_of(const int32_t* tokens, const int32_t* table, int t, int j, int top, int vocab,
                                         int experts) {
  int tok = tokens ? tokens[t] : t;          // no token ids: the table has a row per token of the step
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  int e = table[(int64_t)tok * top + j];
  return e < 0 ? 0 : (e >= experts ? experts - 1 : e);
}

// What follows an expert's first product: nothing, or the square of max(., 0).
constexpr int kActNone = 0, kActRelu2 = 1, kActSiluGate = 2;     // the last one in the per-row first product only
__device__ __forceinline__ float activate(float v, int act) {
  if (act == kActRelu2) {
    v = fmaxf(v, 0.f);
    return v * v;
  }
  return v;
}

// out[t * top + j, n] = act(sum_k a[t, k] * w[e(t, j)][n, k]); with the gated activation an expert's N rows are
// (gate_0, up_0, gate_1, up_1, ...) and out[t * top + j, n] = silu(gate_n) * up_n for n < N / 2, formed from the
// float32 sums (a wave's four dot products are then two gates and their two ups).
template <typename T>
__global__ __launch_bounds__(kThreads) void table_moe_up_kernel(const T* __restrict__ a, int64_t a_stride,
                                                                const T* __restrict__ w,
                                                                const int32_t* __restrict__ tokens,
                                                                const int32_t* __restrict__ table, T* __restrict__ out,
                                                                int top, int experts, int vocab, int N, int K, int act,
                                                                int kCols) {
  const int row = blockIdx.x, t = row / top, j = row - t * top;
  const int wave = threadIdx.x / TL_WAVE, lane = threadIdx.x % TL_WAVE;
  const int e = expert_of(tokens, table, t, j, top, vocab, experts);
  const T* arow = a + (int64_t)t * a_stride;
  const T* we = w + (int64_t)e * N * K;
  const int n0 = blockIdx.y * kCols + wave * (kCols / kWaves);
  if (act == kActSiluGate) {
    const int F = N / 2;
    for (int n = n0; n < min(F, n0 + kCols / kWaves); n += 2) {
      const T* wr[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) wr[c] = we + (int64_t)(2 * min(n + c / 2, F - 1) + (c & 1)) * K;
      float v[4];
      dot_lanes4(arow, wr, K, lane, v);
      if (lane < 2 && n + lane < F) {
        const float g = v[2 * lane], u = v[2 * lane + 1];
        out[(int64_t)row * F + n + lane] = from_f32<T>(g / (1.f + expf(-g)) * u);
      }
    }
    return;
  }
  for (int n = n0; n < min(N, n0 + kCols / kWaves); n += 4) {
    const T* wr[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) wr[c] = we + (int64_t)min(n + c, N - 1) * K;
    float v[4];
    dot_lanes4(arow, wr, K, lane, v);
    if (lane < 4 && n + lane < N) out[(int64_t)row * N + n + lane] = from_f32<T>(activate(v[lane], act));
  }
}

// out[t, c] = base[t, c] * base_scale[t] + coef * sum_j row_w[t * top + j] * sum_k z[t * top + j, k] * w[e(t, j)][c, k]
// (base, base_scale and row_w optional; the experts of a token are added in the table's order)
template <typename T>
__global__ __launch_bounds__(kThreads) void table_moe_down_kernel(const T* __restrict__ z, const T* __restrict__ w,
                                                                  const int32_t* __restrict__ tokens,
                                                                  const int32_t* __restrict__ table,
                                                                  const float* __restrict__ base,
                                                                  const float* __restrict__ base_scale,
                                                                  const float* __restrict__ row_w,
                                                                  float* __restrict__ out, int top, int experts,
                                                                  int vocab, int N, int K, float coef, int kCols) {
  const int t = blockIdx.x;
  const int wave = threadIdx.x / TL_WAVE, lane = threadIdx.x % TL_WAVE;
  const int n0 = blockIdx.y * kCols + wave * (kCols / kWaves);
  const float bsc = base_scale ? base_scale[t] : 1.f;
  for (int n = n0; n < min(N, n0 + kCols / kWaves); n += 4) {
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int j = 0; j < top; ++j) {
      const int e = expert_of(tokens, table, t, j, top, vocab, experts);
      const T* wr[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) wr[c] = w + ((int64_t)e * N + min(n + c, N - 1)) * K;
      float v[4];
      dot_lanes4(z + ((int64_t)t * top + j) * K, wr, K, lane, v);
      const float wj = row_w ? row_w[(int64_t)t * top + j] : 1.f;
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[c] = fmaf(wj, v[c], acc[c]);
    }
    if (lane < 4 && n + lane < N) {
      const float b = base ? base[(int64_t)t * N + n + lane] * bsc : 0.f;
      out[(int64_t)t * N + n + lane] = fmaf(coef, acc[lane], b);
    }
  }
}

// out[t] = sigmoid(a[t, :] . w): one wave a row.
template <typename T>
__global__ __launch_bounds__(TL_WAVE) void row_dot_sigmoid_kernel(const T* __restrict__ a, int64_t a_stride,
                                                                  const T* __restrict__ w, float* __restrict__ out,
                                                                  int K) {
  const float v = dot_lanes(a + (int64_t)blockIdx.x * a_stride, w, K, threadIdx.x);
  if (threadIdx.x == 0) out[blockIdx.x] = 1.f / (1.f + expf(-v));
}

// ------------------------------------------------------------------ many rows: grouped by expert
// Steps with many rows sort them by expert on the device and multiply tiles of 32 rows of ONE expert on
// the matrix cores, so that an expert's weights are read once per tile and not once per row.  The plan is
// a few arrays of int32: counts[E], cursor[E], offsets[E + 1], n_tiles, then per tile its expert, its first
// place in `sorted` and its number of rows, then sorted[rows] (the row indices t * top + j by expert; the
// order inside an expert is whatever the atomics give: a row's result does not depend on its place).
constexpr int kTileRows = 32;

// A workgroup counts its 256 rows in LDS first and adds one number per expert to the shared counters (a prompt's
// thousands of rows over a few experts would otherwise queue up at a handful of addresses).
__global__ __launch_bounds__(kThreads) void moe_count_kernel(const int32_t* __restrict__ tokens,
                                                             const int32_t* __restrict__ table,
                                                             int32_t* __restrict__ counts, int rows, int top,
                                                             int experts, int vocab) {
  __shared__ int32_t local[1024];
  for (int e = threadIdx.x; e < experts; e += kThreads) local[e] = 0;
  __syncthreads();
  const int i = blockIdx.x * kThreads + threadIdx.x;
  if (i < rows) atomicAdd(&local[expert_of(tokens, table, i / top, i % top, top, vocab, experts)], 1);
  __syncthreads();
  for (int e = threadIdx.x; e < experts; e += kThreads)
    if (local[e]) atomicAdd(&counts[e], local[e]);
}

// One workgroup: offsets of the experts' runs in `sorted`, and the list of tiles.
__global__ __launch_bounds__(kThreads) void moe_plan_kernel(const int32_t* __restrict__ counts,
                                                            int32_t* __restrict__ cursor, int32_t* __restrict__ offsets,
                                                            int32_t* __restrict__ n_tiles,
                                                            int32_t* __restrict__ tile_expert,
                                                            int32_t* __restrict__ tile_start,
                                                            int32_t* __restrict__ tile_rows, int experts, int max_tiles,
                                                            int rows_a_tile) {
  const int kTileRows = rows_a_tile;
  __shared__ int32_t first_tile[1025];
  if (threadIdx.x == 0) {
    int at = 0, nt = 0;
    for (int e = 0; e < experts; ++e) {
      offsets[e] = at;
      first_tile[e] = nt;
      at += counts[e];
      nt += (counts[e] + kTileRows - 1) / kTileRows;
    }
    offsets[experts] = at;
    first_tile[experts] = nt;
    n_tiles[0] = min(nt, max_tiles);
  }
  __syncthreads();
  for (int e = threadIdx.x; e < experts; e += kThreads) {
    cursor[e] = 0;
    const int c = counts[e];
    for (int i = 0, t = first_tile[e]; i * kTileRows < c && t < max_tiles; ++i, ++t) {
      tile_expert[t] = e;
      tile_start[t] = offsets[e] + i * kTileRows;
      tile_rows[t] = min(kTileRows, c - i * kTileRows);
    }
  }
  // tiles behind the last one hold no row
  for (int t = first_tile[experts] + threadIdx.x; t < max_tiles; t += kThreads) {
    tile_expert[t] = -1;
    tile_start[t] = 0;
    tile_rows[t] = 0;
  }
}

// The rows of every tile copied side by side: dst[tile * rows_a_tile + i] = a[sorted row / a_div], and where each
// row went (row_pos[row] = tile * rows_a_tile + i).  One workgroup a (tile, run of 8 rows).
__global__ __launch_bounds__(kThreads) void moe_gather_kernel(const bf16_t* __restrict__ a, int64_t a_stride, int a_div,
                                                              bf16_t* __restrict__ dst, int32_t* __restrict__ row_pos,
                                                              const int32_t* __restrict__ tile_start,
                                                              const int32_t* __restrict__ tile_rows,
                                                              const int32_t* __restrict__ sorted, int K,
                                                              int rows_a_tile) {
  const int tile = blockIdx.x, n = tile_rows[tile];
  for (int i = blockIdx.y * 8; i < min(n, blockIdx.y * 8 + 8); ++i) {
    const int src = sorted[tile_start[tile] + i];
    const int64_t at = (int64_t)tile * rows_a_tile + i;
    if (row_pos && threadIdx.x == 0) row_pos[src] = (int32_t)at;
    if (a) {
      const bf16_t* from = a + (int64_t)(src / a_div) * a_stride;
      for (int k = threadIdx.x * 8; k < K; k += kThreads * 8) *(bf16x8*)(dst + at * K + k) = *(const bf16x8*)(from + k);
    }
  }
}

// out[t, c] = base[t, c] * base_scale[t] + coef * sum_j row_w[t * top + j] * y[row_pos[t * top + j], c]
__global__ void moe_combine_at_kernel(const float* __restrict__ y, const int32_t* __restrict__ row_pos,
                                      const float* __restrict__ base, const float* __restrict__ base_scale,
                                      const float* __restrict__ row_w, float* __restrict__ out, int64_t total, int N,
                                      int top, float coef) {
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= total) return;
  const int64_t t = i / N;
  const int c = (int)(i - t * N);
  float acc = 0.f;
  for (int j = 0; j < top; ++j)
    acc = fmaf(row_w ? row_w[t * top + j] : 1.f, y[(int64_t)row_pos[t * top + j] * N + c], acc);
  const float b = base ? base[i] * (base_scale ? base_scale[t] : 1.f) : 0.f;
  out[i] = fmaf(coef, acc, b);
}

// A workgroup ranks its rows inside every expert in LDS, takes one range per expert from the shared cursors and
// writes its rows there.
__global__ __launch_bounds__(kThreads) void moe_scatter_kernel(const int32_t* __restrict__ tokens,
                                                               const int32_t* __restrict__ table,
                                                               const int32_t* __restrict__ offsets,
                                                               int32_t* __restrict__ cursor, int32_t* __restrict__ sorted,
                                                               int rows, int top, int experts, int vocab) {
  __shared__ int32_t local[1024];
  for (int e = threadIdx.x; e < experts; e += kThreads) local[e] = 0;
  __syncthreads();
  const int i = blockIdx.x * kThreads + threadIdx.x;
  int e = 0, rank = 0;
  if (i < rows) {
    e = expert_of(tokens, table, i / top, i % top, top, vocab, experts);
    rank = atomicAdd(&local[e], 1);
  }
  __syncthreads();
  for (int x = threadIdx.x; x < experts; x += kThreads)       // the count turns into the range's first place
    if (local[x]) local[x] = offsets[x] + atomicAdd(&cursor[x], local[x]);
  __syncthreads();
  if (i < rows) sorted[local[e] + rank] = i;
}

// out[row, n] = sum_k a[row / a_div, k] * w[expert of row][n, k] for the rows of one tile; bfloat16 operands
// straight from memory into v_mfma_f32_16x16x32_bf16 (weights as the first operand, so that a lane holds four
// neighbouring columns of one row), float32 sums.  A workgroup of four waves owns 32 rows x 256 columns, a wave
// 32 x 64: six operand loads per eight matrix instructions.
template <typename TO>
__global__ __launch_bounds__(kThreads) void grouped_rows_gemm_bf16_kernel(
    const bf16_t* __restrict__ a, int64_t a_stride, int a_div, const bf16_t* __restrict__ w, TO* __restrict__ out,
    const int32_t* __restrict__ n_tiles, const int32_t* __restrict__ tile_expert, const int32_t* __restrict__ tile_start,
    const int32_t* __restrict__ tile_rows, const int32_t* __restrict__ sorted, int N, int K) {
  const int tile = blockIdx.x;
  if (tile >= n_tiles[0]) return;
  const int e = tile_expert[tile], start = tile_start[tile], nrows = tile_rows[tile];
  const int wave = threadIdx.x / TL_WAVE, lane = threadIdx.x % TL_WAVE, r16 = lane % 16, kq = lane / 16;
  const int col0 = blockIdx.y * 256 + wave * 64;
  if (col0 >= N) return;
  int src[2];
  const bf16_t* ap[2];
#pragma unroll
  for (int rb = 0; rb < 2; ++rb) {
    src[rb] = sorted[start + min(rb * 16 + r16, nrows - 1)];
    ap[rb] = a + (int64_t)(src[rb] / a_div) * a_stride + kq * 8;
  }
  const bf16_t* wp[4];
#pragma unroll
  for (int cb = 0; cb < 4; ++cb) wp[cb] = w + ((int64_t)e * N + min(col0 + cb * 16 + r16, N - 1)) * K + kq * 8;
  f32x4 acc[2][4];
#pragma unroll
  for (int rb = 0; rb < 2; ++rb)
#pragma unroll
    for (int cb = 0; cb < 4; ++cb) acc[rb][cb] = f32x4{0.f, 0.f, 0.f, 0.f};
  const bool second = nrows > 16;
  for (int k0 = 0; k0 < K; k0 += 32) {
    const bool in = k0 + kq * 8 < K;                // K is a multiple of 8
    bf16x8 af[2], wf[4];
    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) af[rb] = in ? *(const bf16x8*)(ap[rb] + k0) : zero;
#pragma unroll
    for (int cb = 0; cb < 4; ++cb) wf[cb] = in ? *(const bf16x8*)(wp[cb] + k0) : zero;
#pragma unroll
    for (int cb = 0; cb < 4; ++cb) {
      acc[0][cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[cb], af[0], acc[0][cb], 0, 0, 0);
      if (second) acc[1][cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[cb], af[1], acc[1][cb], 0, 0, 0);
    }
  }
#pragma unroll
  for (int rb = 0; rb < 2; ++rb) {
    if (rb * 16 + r16 >= nrows) continue;
    TO* orow = out + (int64_t)src[rb] * N;
#pragma unroll
    for (int cb = 0; cb < 4; ++cb)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = col0 + cb * 16 + kq * 4 + i;
        if (c < N) orow[c] = from_f32<TO>(acc[rb][cb][i]);
      }
  }
}

// out[t, c] = base[t, c] * base_scale[t] + coef * sum_j row_w[t * top + j] * y[t * top + j, c]   (the experts in the
// table's order)
__global__ void moe_combine_kernel(const float* __restrict__ y, const float* __restrict__ base,
                                   const float* __restrict__ base_scale, const float* __restrict__ row_w,
                                   float* __restrict__ out, int64_t total, int N, int top, float coef) {
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= total) return;
  const int64_t t = i / N;
  const int c = (int)(i - t * N);
  float acc = 0.f;
  for (int j = 0; j < top; ++j) acc = fmaf(row_w ? row_w[t * top + j] : 1.f, y[(t * top + j) * N + c], acc);
  const float b = base ? base[i] * (base_scale ? base_scale[t] : 1.f) : 0.f;
  out[i] = fmaf(coef, acc, b);
}

// ------------------------------------------------------------------------------- a router
// One wave a token.  z [n_tokens, experts] are the router's logits (float32).  Scores s = softmax(z) over all
// experts.  The experts lie in `groups` equal runs of neighbours; a run's score is its largest score, and only
// experts of the `keep` best runs may be chosen (groups <= 1: all may).  The `top` largest scores among those
// are chosen, largest first (equal scores: the lower index first); ids[t, j] names them, and
// wts[t, j] = s_j / (sum of the chosen s + 1e-20) * scale.
constexpr int kMaxRouted = 1024;

struct Best {
  float v;
  int i;
};
__device__ __forceinline__ Best better(Best a, Best b) { return (b.v > a.v || (b.v == a.v && b.i < a.i)) ? b : a; }
__device__ __forceinline__ Best wave_best(Best x) {
#pragma unroll
  for (int d = TL_WAVE / 2; d >= 1; d >>= 1) {
    Best o;
    o.v = __shfl_xor(x.v, d, TL_WAVE);
    o.i = __shfl_xor(x.i, d, TL_WAVE);
    x = better(x, o);
  }
  return x;
}

__global__ __launch_bounds__(TL_WAVE) void moe_route_kernel(const float* __restrict__ z, int64_t z_stride,
                                                            const float* __restrict__ bias, int32_t* __restrict__ ids,
                                                            float* __restrict__ wts, int experts, int top, int groups,
                                                            int keep, float scale) {
  __shared__ float s[kMaxRouted];         // scores; -1 once an expert is chosen or its run is out
  __shared__ float gs[kMaxRouted];        // the runs' scores
  const int t = blockIdx.x, lane = threadIdx.x;
  const float* zr = z + (int64_t)t * z_stride;
  float m = -INFINITY;
  for (int e = lane; e < experts; e += TL_WAVE) {     // the logits (a bias per expert added), kept in s for the next pass
    const float l = bias ? zr[e] + bias[e] : zr[e];
    s[e] = l;
    m = fmaxf(m, l);
  }
  m = wave_max(m);
  float sum = 0.f;
  for (int e = lane; e < experts; e += TL_WAVE) {
    const float p = expf(s[e] - m);
    s[e] = p;
    sum += p;
  }
  sum = wave_sum(sum);
  const float inv = 1.f / sum;
  for (int e = lane; e < experts; e += TL_WAVE) s[e] *= inv;
  __syncthreads();
  if (groups > 1 && keep < groups) {
    const int per = experts / groups;
    for (int g = lane; g < groups; g += TL_WAVE) {
      float b = -1.f;
      for (int e = g * per; e < (g + 1) * per; ++e) b = fmaxf(b, s[e]);
      gs[g] = b;
    }
    __syncthreads();
    for (int k = 0; k < keep; ++k) {      // the best runs, one a pass; a kept run is marked with -2
      Best b = {-1.f, 0x7fffffff};
      for (int g = lane; g < groups; g += TL_WAVE) b = better(b, Best{gs[g], g});
      b = wave_best(b);
      __syncthreads();
      if (lane == 0) gs[b.i] = -2.f;
      __syncthreads();
    }
    for (int e = lane; e < experts; e += TL_WAVE)
      if (gs[e / per] != -2.f) s[e] = -1.f;
    __syncthreads();
  }
  float total = 0.f;
  for (int j = 0; j < top; ++j) {         // the best of what is left, one a pass; gs now keeps the chosen scores
    Best b = {-2.f, 0x7fffffff};
    for (int e = lane; e < experts; e += TL_WAVE) b = better(b, Best{s[e], e});
    b = wave_best(b);
    __syncthreads();
    if (lane == 0) {
      s[b.i] = -3.f;
      gs[j] = b.v;
      ids[(int64_t)t * top + j] = b.i;
    }
    total += b.v;
    __syncthreads();
  }
  const float f = scale / (total + 1e-20f);
  for (int j = lane; j < top; j += TL_WAVE) wts[(int64_t)t * top + j] = gs[j] * f;
}

// out[i] = act(in[i]) over rows of `cols` elements (the input's rows may be wider).
template <typename TI, typename TO>
__global__ void activate_rows_kernel(const TI* __restrict__ in, int64_t in_stride, TO* __restrict__ out, int64_t total,
                                     int cols, int act) {
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= total) return;
  const int64_t t = i / cols;
  out[i] = from_f32<TO>(activate(to_f32(in[t * in_stride + (i - t * cols)]), act));
}

}  // namespace

extern "C" {

int tl_moe_tile_rows(void) { return kTileRows; }

// plan: int32 [2 * experts + (experts + 1) + 1 + 3 * max_tiles + n_tokens * top], counts and cursor zeroed by the
// caller; max_tiles >= ceil(n_tokens * top / 32) + experts.
int tl_moe_plan(const int32_t* tokens, const int32_t* table, int32_t* plan, int n_tokens, int top, int experts, int vocab,
                int max_tiles, int rows_a_tile, hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  const int64_t rows = (int64_t)n_tokens * top;
  if (top <= 0 || experts <= 0 || experts > 1024 || vocab <= 0 || rows > 0x7fffffff || (!tokens && vocab < n_tokens) || !table || !plan ||
      rows_a_tile <= 0 || max_tiles < (rows + rows_a_tile - 1) / rows_a_tile + experts)
    return TL_ERR_ARG;
  int32_t* counts = plan;
  int32_t* cursor = counts + experts;
  int32_t* offsets = cursor + experts;
  int32_t* n_tiles = offsets + experts + 1;
  int32_t* tile_expert = n_tiles + 1;
  int32_t* tile_start = tile_expert + max_tiles;
  int32_t* tile_rows = tile_start + max_tiles;
  int32_t* sorted = tile_rows + max_tiles;
  const unsigned blocks = (unsigned)ceil_div64(rows, kThreads);
  hipLaunchKernelGGL(moe_count_kernel, dim3(blocks), dim3(kThreads), 0, stream, tokens, table, counts, (int)rows, top,
                     experts, vocab);
  hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(kThreads), 0, stream, counts, cursor, offsets, n_tiles, tile_expert,
                     tile_start, tile_rows, experts, max_tiles, rows_a_tile);
  hipLaunchKernelGGL(moe_scatter_kernel, dim3(blocks), dim3(kThreads), 0, stream, tokens, table, offsets, cursor, sorted,
                     (int)rows, top, experts, vocab);
  return tl_launch_status();
}

// a: bfloat16 rows (row r of the plan reads a[r / a_div]); w: bfloat16 [experts, N, K]; out: [rows, N] bfloat16
// (out_dtype 1) or float32 (0), written at the rows' own places.
int tl_grouped_rows_gemm(const void* a, int64_t a_stride, int a_div, const void* w, void* out, const int32_t* plan,
                         int n_rows, int experts, int max_tiles, int N, int K, int out_dtype, hipStream_t stream) {
  if (n_rows <= 0) return TL_OK;
  if (a_div <= 0 || experts <= 0 || N <= 0 || K <= 0 || K % 8 || a_stride % 8 || a_stride < K || !a || !w || !out || !plan ||
      max_tiles <= 0 || (N + 255) / 256 > 65535)
    return TL_ERR_ARG;
  const int32_t* n_tiles = plan + 3 * experts + 1;
  const int32_t* tile_expert = n_tiles + 1;
  const int32_t* tile_start = tile_expert + max_tiles;
  const int32_t* tile_rows = tile_start + max_tiles;
  const int32_t* sorted = tile_rows + max_tiles;
  dim3 g(max_tiles, (N + 255) / 256), b(kThreads);
  if (out_dtype == 1)
    hipLaunchKernelGGL(grouped_rows_gemm_bf16_kernel<bf16_t>, g, b, 0, stream, (const bf16_t*)a, a_stride, a_div,
                       (const bf16_t*)w, (bf16_t*)out, n_tiles, tile_expert, tile_start, tile_rows, sorted, N, K);
  else if (out_dtype == 0)
    hipLaunchKernelGGL(grouped_rows_gemm_bf16_kernel<float>, g, b, 0, stream, (const bf16_t*)a, a_stride, a_div,
                       (const bf16_t*)w, (float*)out, n_tiles, tile_expert, tile_start, tile_rows, sorted, N, K);
  else
    return TL_ERR_ARG;
  return tl_launch_status();
}

// The plan's rows (tiles of rows_a_tile rows) copied side by side into dst [max_tiles * rows_a_tile, K] (a null: no
// copy), and row_pos[row] = where it went (null: not wanted).
int tl_moe_gather(const void* a, int64_t a_stride, int a_div, void* dst, int32_t* row_pos, const int32_t* plan,
                  int experts, int max_tiles, int rows_a_tile, int K, hipStream_t stream) {
  if (max_tiles <= 0) return TL_OK;
  if (a_div <= 0 || experts <= 0 || rows_a_tile <= 0 || K <= 0 || K % 8 || (a && (a_stride % 8 || !dst)) || !plan ||
      max_tiles > 0x7fffff00 / rows_a_tile)
    return TL_ERR_ARG;
  const int32_t* tile_start = plan + 3 * experts + 2 + max_tiles;
  const int32_t* tile_rows = tile_start + max_tiles;
  const int32_t* sorted = tile_rows + max_tiles;
  hipLaunchKernelGGL(moe_gather_kernel, dim3(max_tiles, (rows_a_tile + 7) / 8), dim3(kThreads), 0, stream,
                     (const bf16_t*)a, a_stride, a_div, (bf16_t*)dst, row_pos, tile_start, tile_rows, sorted, K,
                     rows_a_tile);
  return tl_launch_status();
}

// As tl_moe_combine with the rows of y looked up in row_pos.
int tl_moe_combine_at(const float* y, const int32_t* row_pos, const float* base, const float* base_scale,
                      const float* row_w, float* out, int n_tokens, int N, int top, float coef, hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  if (N <= 0 || top <= 0 || !y || !out || !row_pos) return TL_ERR_ARG;
  const int64_t total = (int64_t)n_tokens * N;
  hipLaunchKernelGGL(moe_combine_at_kernel, dim3((unsigned)ceil_div64(total, kThreads)), dim3(kThreads), 0, stream, y,
                     row_pos, base, base_scale, row_w, out, total, N, top, coef);
  return tl_launch_status();
}

int tl_moe_combine(const float* y, const float* base, const float* base_scale, const float* row_w, float* out,
                   int n_tokens, int N, int top, float coef, hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  if (N <= 0 || top <= 0 || !y || !out) return TL_ERR_ARG;
  const int64_t total = (int64_t)n_tokens * N;
  hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)ceil_div64(total, kThreads)), dim3(kThreads), 0, stream, y, base,
                     base_scale, row_w, out, total, N, top, coef);
  return tl_launch_status();
}

// a: [n_tokens, K] (row stride a_stride); w: [experts, N, K]; table: int32 [vocab, top], looked up by tokens[t], or
// (tokens null) by t itself; out: [n_tokens * top, N], with the activation `act` (0 none, 1 squared relu) applied.
int tl_table_moe_up(const void* a, int64_t a_stride, const void* w, const int32_t* tokens, const int32_t* table, void* out,
                    int n_tokens, int top, int experts, int vocab, int N, int K, int act, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  if (top <= 0 || experts <= 0 || vocab <= 0 || N <= 0 || K <= 0 || a_stride < K || !a || !w || !table || !out ||
      (act != kActNone && act != kActRelu2 && act != kActSiluGate) || (act == kActSiluGate && (N & 1)) ||
      (!tokens && vocab < n_tokens) || (int64_t)n_tokens * top > 0x7fffffff || (N + kColsFew - 1) / kColsFew > 65535)
    return TL_ERR_ARG;
  const int kCols = (int64_t)n_tokens * top <= kFewRows ? kColsFew : kColsWide;
  const int n_out = act == kActSiluGate ? N / 2 : N;      // output columns
  dim3 g(n_tokens * top, (n_out + kCols - 1) / kCols), b(kThreads);
  if (dtype == 0)
    hipLaunchKernelGGL(table_moe_up_kernel<float>, g, b, 0, stream, (const float*)a, a_stride, (const float*)w, tokens,
                       table, (float*)out, top, experts, vocab, N, K, act, kCols);
  else if (dtype == 1)
    hipLaunchKernelGGL(table_moe_up_kernel<bf16_t>, g, b, 0, stream, (const bf16_t*)a, a_stride, (const bf16_t*)w, tokens,
                       table, (bf16_t*)out, top, experts, vocab, N, K, act, kCols);
  else
    return TL_ERR_ARG;
  return tl_launch_status();
}

// z: [n_tokens * top, K]; w: [experts, N, K]; base: float32 [n_tokens, N] or null; base_scale: float32 [n_tokens] or
// null; row_w: float32 [n_tokens * top] or null; out: float32 [n_tokens, N] (may be base).
int tl_table_moe_down(const void* z, const void* w, const int32_t* tokens, const int32_t* table, const float* base,
                      const float* base_scale, const float* row_w, float* out, int n_tokens, int top, int experts,
                      int vocab, int N, int K, float coef, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  if (top <= 0 || experts <= 0 || vocab <= 0 || N <= 0 || K <= 0 || !z || !w || !table || !out ||
      (!tokens && vocab < n_tokens) ||
      (N + kColsFew - 1) / kColsFew > 65535)
    return TL_ERR_ARG;
  const int kCols = (int64_t)n_tokens * top <= kFewRows ? kColsFew : kColsWide;
  dim3 g(n_tokens, (N + kCols - 1) / kCols), b(kThreads);
  if (dtype == 0)
    hipLaunchKernelGGL(table_moe_down_kernel<float>, g, b, 0, stream, (const float*)z, (const float*)w, tokens, table,
                       base, base_scale, row_w, out, top, experts, vocab, N, K, coef, kCols);
  else if (dtype == 1)
    hipLaunchKernelGGL(table_moe_down_kernel<bf16_t>, g, b, 0, stream, (const bf16_t*)z, (const bf16_t*)w, tokens, table,
                       base, base_scale, row_w, out, top, experts, vocab, N, K, coef, kCols);
  else
    return TL_ERR_ARG;
  return tl_launch_status();
}

int tl_row_dot_sigmoid(const void* a, int64_t a_stride, const void* w, float* out, int n_rows, int K, int dtype,
                       hipStream_t stream) {
  if (n_rows <= 0) return TL_OK;
  if (K <= 0 || a_stride < K || !a || !w || !out) return TL_ERR_ARG;
  dim3 g(n_rows), b(TL_WAVE);
  if (dtype == 0)
    hipLaunchKernelGGL(row_dot_sigmoid_kernel<float>, g, b, 0, stream, (const float*)a, a_stride, (const float*)w, out, K);
  else if (dtype == 1)
    hipLaunchKernelGGL(row_dot_sigmoid_kernel<bf16_t>, g, b, 0, stream, (const bf16_t*)a, a_stride, (const bf16_t*)w, out,
                       K);
  else
    return TL_ERR_ARG;
  return tl_launch_status();
}

// z: float32 [n_tokens, experts] (row stride z_stride); ids: int32 [n_tokens, top]; wts: float32 [n_tokens, top].
int tl_moe_route(const float* z, int64_t z_stride, const float* bias, int32_t* ids, float* wts, int n_tokens, int experts,
                 int top, int groups, int keep, float scale, hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  if (experts <= 0 || experts > kMaxRouted || top <= 0 || top > experts || z_stride < experts || !z || !ids || !wts ||
      groups < 0 || (groups > 1 && (experts % groups || keep <= 0 || keep > groups || top > keep * (experts / groups))))
    return TL_ERR_ARG;
  hipLaunchKernelGGL(moe_route_kernel, dim3(n_tokens), dim3(TL_WAVE), 0, stream, z, z_stride, bias, ids, wts, experts, top,
                     groups, keep, scale);
  return tl_launch_status();
}

// in: [n_rows, >= cols] float32 (dtype_in 0) or bfloat16 (1); out: contiguous [n_rows, cols] in dtype_out.
int tl_activate_rows(const void* in, int64_t in_stride, void* out, int n_rows, int cols, int act, int dtype_in,
                     int dtype_out, hipStream_t stream) {
  if (n_rows <= 0) return TL_OK;
  if (cols <= 0 || in_stride < cols || !in || !out || (act != kActNone && act != kActRelu2)) return TL_ERR_ARG;
  const int64_t total = (int64_t)n_rows * cols;
  dim3 g((unsigned)ceil_div64(total, kThreads)), b(kThreads);
#define TL_ACT(TI, TO) \
  hipLaunchKernelGGL((activate_rows_kernel<TI, TO>), g, b, 0, stream, (const TI*)in, in_stride, (TO*)out, total, cols, act)
  if (dtype_in == 0 && dtype_out == 0) TL_ACT(float, float);
  else if (dtype_in == 0 && dtype_out == 1) TL_ACT(float, bf16_t);
  else if (dtype_in == 1 && dtype_out == 1) TL_ACT(bf16_t, bf16_t);
  else return TL_ERR_ARG;
#undef TL_ACT
  return tl_launch_status();
}

}  // extern "C"
