// The gated delta rule with one decay per head and key channel (or one per head, laid out over the
// channels where the recurrence reads it), as a recurrence over a state
// S [dim, vdim] per request and head:
//     S <- diag(g_t) S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t
// and what surrounds it: short causal convolutions with SiLU on q, k and v (their last taps - 1
// inputs are state as well), unit vectors q and k, the decay g = exp(-exp(A_log) softplus(a + dt_bias)),
// and the per-head norm with its gate on the way out.  The state, and everything that enters the
// recurrence, is float32 in both precisions.
//
// Per request the state is ONE row of float32: [S of every head: heads x dim x vdim | the
// convolutions' last inputs: channels x (taps - 1), oldest first].
#include "common.h"

namespace {

constexpr int kPrepThreads = 128;
constexpr int kPrepWaves = kPrepThreads / TL_WAVE;
constexpr int kMaxDim = 256;      // key channels a head may have

__device__ __forceinline__ float silu(float x) { return x / (1.f + expf(-x)); }
__device__ __forceinline__ float softplus(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// Input m of channel c (column `col` of the projections) of the request whose tokens of this step
// start at row t0: m >= 0 is row t0 + m of this step, m < 0 reaches back into the saved inputs.
template <typename T>
__device__ __forceinline__ float conv_input(const T* __restrict__ p, int64_t p_stride, int t0, int m, int col,
                                            const float* __restrict__ saved, int taps) {
  return m >= 0 ? to_f32(p[(int64_t)(t0 + m) * p_stride + col]) : saved[(taps - 1) + m];
}

// Up to four taps (the usual sizes) are requested together; the sum runs from the oldest input to the
// current one either way.
template <typename T>
__device__ __forceinline__ float conv_silu(const T* __restrict__ p, int64_t p_stride, int t0, int n, int col,
                                           const float* __restrict__ saved, const float* __restrict__ w, int taps) {
  float acc = 0.f;
  if (taps <= 4) {
    float x[4], wt[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {       // tap j of the weights meets input n - (taps - 1) + j
      x[j] = j < taps ? conv_input(p, p_stride, t0, n - (taps - 1) + j, col, saved, taps) : 0.f;
      wt[j] = j < taps ? w[j] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) acc = fmaf(wt[j], x[j], acc);
    return silu(acc);
  }
  for (int j = 0; j < taps; ++j) acc = fmaf(w[j], conv_input(p, p_stride, t0, n - (taps - 1) + j, col, saved, taps), acc);
  return silu(acc);
}

// One workgroup per (token, head).  Row t of `p` holds [q (kv_heads x dim) | k (kv_heads x dim) |
// v (heads x vdim)] from column conv_off on, and beta's pre-activation at column b_off + head;
// row t of `a` holds the decay's pre-activation at column head * dim + i, or, with a_per_head, one per
// head at column head (dt_bias is indexed likewise).
template <typename T>
__global__ __launch_bounds__(kPrepThreads) void delta_prepare_kernel(
    const T* __restrict__ p, int64_t p_stride, int conv_off, int b_off, const float* __restrict__ a, int64_t a_stride,
    const float* __restrict__ conv_w, const float* __restrict__ a_log, const float* __restrict__ dt_bias,
    const float* __restrict__ state, int64_t state_stride, int64_t saved_off, const int32_t* __restrict__ req_of_token,
    const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ state_slots, float* __restrict__ qn,
    float* __restrict__ kn, float* __restrict__ vc, float* __restrict__ beta, float* __restrict__ decay, int heads,
    int kv_heads, int dim, int vdim, int taps, float q_scale, int a_per_head) {
  __shared__ float qs[kMaxDim], ks[kMaxDim], red[kPrepWaves];
  const int t = blockIdx.x, h = blockIdx.y;
  const int r = req_of_token[t];
  const int t0 = cu_seqlens[r], t1 = cu_seqlens[r + 1];
  const int64_t base = (int64_t)t * heads + h;
  if (t < t0 || t >= t1) {            // a padding row of a captured step: finite stand-ins, never read
    for (int i = threadIdx.x; i < dim; i += kPrepThreads) qn[base * dim + i] = kn[base * dim + i] = decay[base * dim + i] = 0.f;
    for (int j = threadIdx.x; j < vdim; j += kPrepThreads) vc[base * vdim + j] = 0.f;
    if (threadIdx.x == 0) beta[base] = 0.f;
    return;
  }
  const int n = t - t0;
  const int kh = h / (heads / kv_heads);
  const float* saved = state + (int64_t)state_slots[r] * state_stride + saved_off;
  const int q_ch = kh * dim, k_ch = kv_heads * dim + kh * dim, v_ch = 2 * kv_heads * dim + h * vdim;
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x; i < dim; i += kPrepThreads) {
    const float q = conv_silu(p, p_stride, t0, n, conv_off + q_ch + i, saved + (int64_t)(q_ch + i) * (taps - 1),
                              conv_w + (int64_t)(q_ch + i) * taps, taps);
    const float k = conv_silu(p, p_stride, t0, n, conv_off + k_ch + i, saved + (int64_t)(k_ch + i) * (taps - 1),
                              conv_w + (int64_t)(k_ch + i) * taps, taps);
    qs[i] = q;
    ks[i] = k;
    sq += q * q;
    sk += k * k;
  }
  sq = block_sum<kPrepWaves>(sq, red);
  sk = block_sum<kPrepWaves>(sk, red);
  const float rq = q_scale / sqrtf(sq + 1e-6f), rk = 1.f / sqrtf(sk + 1e-6f);
  const float rate = expf(a_log[h]);
  for (int i = threadIdx.x; i < dim; i += kPrepThreads) {
    qn[base * dim + i] = qs[i] * rq;
    kn[base * dim + i] = ks[i] * rk;
    const int ai = a_per_head ? h : h * dim + i;
    const float pre = a[(int64_t)t * a_stride + ai] + dt_bias[ai];
    decay[base * dim + i] = expf(-rate * softplus(pre));
  }
  for (int j = threadIdx.x; j < vdim; j += kPrepThreads)
    vc[base * vdim + j] = conv_silu(p, p_stride, t0, n, conv_off + v_ch + j, saved + (int64_t)(v_ch + j) * (taps - 1),
                                    conv_w + (int64_t)(v_ch + j) * taps, taps);
  if (threadIdx.x == 0) beta[base] = 1.f / (1.f + expf(-to_f32(p[(int64_t)t * p_stride + b_off + h])));
}

// The convolutions' saved inputs after a step: the last taps - 1 of (what was saved, this step's
// inputs).  One thread per (request, channel); it reads all it needs before it writes.
constexpr int kMaxTaps = 16;
template <typename T>
__global__ void conv_state_update_kernel(const T* __restrict__ p, int64_t p_stride, int conv_off, int channels,
                                         float* __restrict__ state, int64_t state_stride, int64_t saved_off,
                                         const int32_t* __restrict__ cu_seqlens,
                                         const int32_t* __restrict__ state_slots, int taps) {
  const int r = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int t0 = cu_seqlens[r], n = cu_seqlens[r + 1] - t0;
  if (c >= channels || n <= 0) return;
  float* saved = state + (int64_t)state_slots[r] * state_stride + saved_off + (int64_t)c * (taps - 1);
  float next[kMaxTaps];
#pragma unroll
  for (int i = 0; i < kMaxTaps; ++i)
    if (i < taps - 1) next[i] = conv_input(p, p_stride, t0, n - (taps - 1) + i, conv_off + c, saved, taps);
#pragma unroll
  for (int i = 0; i < kMaxTaps; ++i)
    if (i < taps - 1) saved[i] = next[i];
}

// The recurrence.  A wave owns 8 value columns of one (request, head): lane (s, c) keeps rows
// [s * DS, (s + 1) * DS) of column c of S in registers (eight slices of the key channels side by side,
// 8 lanes each), so a token costs DS steps and two sums over the eight slices instead of `dim` steps.
// The wave walks the request's tokens of this step in order, kCh at a time: q, k, decay, v and beta of a
// chunk go through LDS, and the next chunk's are requested before this one is worked on.  The four waves
// of a workgroup (32 columns) share the staged chunk: q, k and decay are the same for every column.
constexpr int kCh = 16;           // tokens per staged chunk
constexpr int kCols = 8;          // value columns per wave
constexpr int kRecWaves = 4, kRecThreads = kRecWaves * TL_WAVE, kRecCols = kRecWaves * kCols;
constexpr int kSlices = TL_WAVE / kCols;
// the sum over the lanes c, c + 8, ..., c + 56; every lane gets it
__device__ __forceinline__ float sum_over_slices(float v) { return sum_over_rows(v + dpp_f32<TL_DPP_ROR8>(v)); }
template <int DS>
__global__ __launch_bounds__(kRecThreads) void delta_recurrence_kernel(
    const float* __restrict__ qn, const float* __restrict__ kn, const float* __restrict__ vc,
    const float* __restrict__ beta, const float* __restrict__ decay, float* __restrict__ state, int64_t state_stride,
    const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ state_slots, float* __restrict__ out,
    int heads, int dim, int vdim) {
  constexpr int DP = kSlices * DS;                // key channels, padded
  constexpr int PER = (kCh * DP + kRecThreads - 1) / kRecThreads;    // floats of one staged array a thread moves per chunk
  constexpr int PERV = kCh * kRecCols / kRecThreads;
  __shared__ float ks[kCh][DP], qs[kCh][DP], gs[kCh][DP], vs[kCh][kRecCols], bs[kCh];
  const int r = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, wave = tid / TL_WAVE, lane = tid % TL_WAVE;
  const int s = lane / kCols, c = wave * kCols + lane % kCols;
  const int col = blockIdx.z * kRecCols + c;
  const int t0 = cu_seqlens[r], t1 = cu_seqlens[r + 1];
  if (t1 <= t0) return;                           // a padding request owns no state
  const bool live = col < vdim;
  float* S_mem = state + (int64_t)state_slots[r] * state_stride + (int64_t)h * dim * vdim + col;
  float S[DS];
#pragma unroll
  for (int i = 0; i < DS; ++i) S[i] = (live && s * DS + i < dim) ? S_mem[(int64_t)(s * DS + i) * vdim] : 0.f;

  float rk[PER], rq[PER], rg[PER], rv[PERV], rb = 0.f;
  // element e of a staged array: token e / DP of the chunk, channel e % DP (channels beyond dim: k = q = 0, g = 1)
  auto fetch = [&](int tc) {
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = j * kRecThreads + tid, tt = e / DP, i = e % DP;
      const bool ok = e < kCh * DP && tc + tt < t1 && i < dim;
      const int64_t at = ((int64_t)(tc + tt) * heads + h) * dim + i;
      rk[j] = ok ? kn[at] : 0.f;
      rq[j] = ok ? qn[at] : 0.f;
      rg[j] = ok ? decay[at] : 1.f;
    }
#pragma unroll
    for (int j = 0; j < PERV; ++j) {
      const int e = j * kRecThreads + tid, tt = e / kRecCols, cc = e % kRecCols;
      const int vcol = blockIdx.z * kRecCols + cc;
      rv[j] = (tc + tt < t1 && vcol < vdim) ? vc[((int64_t)(tc + tt) * heads + h) * vdim + vcol] : 0.f;
    }
    rb = (tid < kCh && tc + tid < t1) ? beta[(int64_t)(tc + tid) * heads + h] : 0.f;
  };
  fetch(t0);
  for (int tc = t0; tc < t1; tc += kCh) {
    __syncthreads();                              // the chunk before has been read
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = j * kRecThreads + tid;
      if (e < kCh * DP) {
        (&ks[0][0])[e] = rk[j];
        (&qs[0][0])[e] = rq[j];
        (&gs[0][0])[e] = rg[j];
      }
    }
#pragma unroll
    for (int j = 0; j < PERV; ++j) (&vs[0][0])[j * kRecThreads + tid] = rv[j];
    if (tid < kCh) bs[tid] = rb;
    __syncthreads();
    if (tc + kCh < t1) fetch(tc + kCh);           // on its way while this chunk is worked on
    const int n = min(kCh, t1 - tc);
    // With S' = diag(g) S:  o = (S' + k u^T)^T q = S'^T q + u (k . q).  Both sums over S' and k . q are
    // taken in ONE pass (in four independent parts) and meet in one round of exchanges between the
    // slices; the update of S hangs off it.  A token's operands are read from LDS while the token before
    // it is worked on (two register sets, the loop goes two tokens at a time).
    auto load = [&](int tt, float* k, float* q, float* g, float& v, float& bt) {
#pragma unroll
      for (int i = 0; i < DS; ++i) {
        k[i] = ks[tt][s * DS + i];
        q[i] = qs[tt][s * DS + i];
        g[i] = gs[tt][s * DS + i];
      }
      v = vs[tt][c];
      bt = bs[tt];
    };
    auto step = [&](int tt, const float* k, const float* q, const float* g, float v, float bt) {
      float sk[4] = {0.f, 0.f, 0.f, 0.f}, sq[4] = {0.f, 0.f, 0.f, 0.f}, kq[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < DS; ++i) {
        S[i] *= g[i];
        sk[i & 3] = fmaf(S[i], k[i], sk[i & 3]);
        sq[i & 3] = fmaf(S[i], q[i], sq[i & 3]);
        kq[i & 3] = fmaf(k[i], q[i], kq[i & 3]);
      }
      const float sk_all = sum_over_slices((sk[0] + sk[1]) + (sk[2] + sk[3]));
      const float sq_all = sum_over_slices((sq[0] + sq[1]) + (sq[2] + sq[3]));
      const float kq_all = sum_over_slices((kq[0] + kq[1]) + (kq[2] + kq[3]));
      const float u = bt * (v - sk_all);
#pragma unroll
      for (int i = 0; i < DS; ++i) S[i] = fmaf(k[i], u, S[i]);
      if (s == 0 && live) out[((int64_t)(tc + tt) * heads + h) * vdim + col] = fmaf(u, kq_all, sq_all);
    };
    float ka[DS], qa2[DS], ga[DS], kb[DS], qb[DS], gb[DS], va, ba, vb, bb;
    load(0, ka, qa2, ga, va, ba);
    for (int tt = 0; tt < n; tt += 2) {
      load(min(tt + 1, kCh - 1), kb, qb, gb, vb, bb);
      step(tt, ka, qa2, ga, va, ba);
      load(min(tt + 2, kCh - 1), ka, qa2, ga, va, ba);
      if (tt + 1 < n) step(tt + 1, kb, qb, gb, vb, bb);
    }
  }
#pragma unroll
  for (int i = 0; i < DS; ++i)
    if (live && s * DS + i < dim) S_mem[(int64_t)(s * DS + i) * vdim] = S[i];
}

// z[t, h, :] = scale * w * o[t, h, :] / sqrt(mean(o[t, h, :]^2) + eps) * act(gate[t, h, :]); one wave per (t, h).
// w is shared by the heads (w_head_stride 0) or each head's own (w_head_stride = vdim); act is the sigmoid
// (gate_kind 0) or g * sigmoid(g) (gate_kind 1).
template <typename T>
__global__ __launch_bounds__(TL_WAVE) void head_norm_gate_kernel(const float* __restrict__ o,
                                                                 const float* __restrict__ w, int w_head_stride,
                                                                 const float* __restrict__ gate, int64_t gate_stride,
                                                                 T* __restrict__ z, int heads, int vdim, float eps,
                                                                 int gate_kind, float scale) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float* src = o + ((int64_t)t * heads + h) * vdim;
  const float* wh = w + (int64_t)h * w_head_stride;
  float ss = 0.f;
  for (int j = lane; j < vdim; j += TL_WAVE) ss += src[j] * src[j];
  ss = wave_sum(ss);
  const float r = scale / sqrtf(ss / (float)vdim + eps);
  const float* gp = gate + (int64_t)t * gate_stride + (int64_t)h * vdim;
  T* dst = z + ((int64_t)t * heads + h) * vdim;
  for (int j = lane; j < vdim; j += TL_WAVE) {
    const float g = gp[j], sg = 1.f / (1.f + expf(-g));
    dst[j] = from_f32<T>(src[j] * r * wh[j] * (gate_kind ? g * sg : sg));
  }
}

// Sum over a workgroup of `nw` waves (nw <= 16); `red` is LDS of 16 floats.  Fixed order.
__device__ __forceinline__ float block_sum_dyn(float v, float* red, int nw) {
  v = wave_sum(v);
  __syncthreads();
  if (threadIdx.x % TL_WAVE == 0) red[threadIdx.x / TL_WAVE] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nw; ++i) t += red[i];
  return t;
}

// A decode step in one kernel: every request brings ONE token.  One workgroup per (request, head),
// a thread per value column: the convolutions, unit vectors, decay and beta of the token, the
// recurrence on the column in registers, and the head's norm and gate on the way out
// (z[t, h, :] = w * o / rms(o) * act(gate), act the sigmoid or, with gate_kind 1, g * sigmoid(g)).  The saved convolution inputs are brought up to date
// here when every head has q/k channels of its own (update_saved); else several workgroups read a
// channel's saved inputs and conv_state_update_kernel runs behind this kernel.
constexpr int kDecodeThreads = 256;     // value columns the one-kernel decode step takes (a thread each)
// The inputs and weights of one channel's convolution for the token at row t (n = 0 in its step),
// oldest first; taps <= 4.
template <typename T>
__device__ __forceinline__ void load_taps(const T* __restrict__ p, int64_t p_stride, int t, int col,
                                          const float* __restrict__ saved, const float* __restrict__ w, int taps,
                                          float* x, float* wt) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    x[j] = j < taps ? conv_input(p, p_stride, t, j - (taps - 1), col, saved, taps) : 0.f;
    wt[j] = j < taps ? w[j] : 0.f;
  }
}
__device__ __forceinline__ float conv_of(const float* x, const float* wt) {
  float acc = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j) acc = fmaf(wt[j], x[j], acc);
  return silu(acc);
}
// after the token the saved inputs are the last taps - 1 of x
__device__ __forceinline__ void store_saved(float* __restrict__ saved, const float* x, int taps) {
#pragma unroll
  for (int j = 1; j < 4; ++j)
    if (j < taps) saved[j - 1] = x[j];
}

// State phase of the kernel: thread (sl, cq) keeps rows [sl * DS, (sl + 1) * DS) of the FOUR value columns
// 4 cq .. 4 cq + 3 of S in registers (16-byte loads and stores: a lane that moves four bytes at a time gets a
// fraction of what a compute unit can fetch), the four slices' partial sums meet in LDS in a fixed order.
template <typename T, typename TZ, int DS>
__global__ __launch_bounds__(kDecodeThreads) void delta_decode_kernel(
    const T* __restrict__ p, int64_t p_stride, int conv_off, int b_off, const float* __restrict__ a, int64_t a_stride,
    int a_per_head, const float* __restrict__ gate, int64_t gate_stride, int gate_kind,
    const float* __restrict__ conv_w, const float* __restrict__ a_log, const float* __restrict__ dt_bias,
    const float* __restrict__ w_norm, float* __restrict__ state, int64_t state_stride, int64_t saved_off,
    const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ state_slots, TZ* __restrict__ z, int heads,
    int kv_heads, int dim, int vdim, int taps, float q_scale, float eps, int update_saved) {
  __shared__ float qs[kMaxDim], ks[kMaxDim], gs[kMaxDim], vs[kDecodeThreads], red[16];
  __shared__ f32x4 part[4][kDecodeThreads / 4];
  const int r = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int nw = blockDim.x / TL_WAVE;
  const int t = cu_seqlens[r];
  if (cu_seqlens[r + 1] - t != 1) return;         // a padding request owns no state
  const int kh = h / (heads / kv_heads);
  float* row = state + (int64_t)state_slots[r] * state_stride;
  float* saved = row + saved_off;
  const int q_ch = kh * dim, k_ch = kv_heads * dim + kh * dim, v_ch = 2 * kv_heads * dim + h * vdim;
  const int quads = vdim / 4;
  const int cq = tid % quads, sl = tid / quads;     // state phase: column quad and slice of the key channels
  const bool owner = sl < 4;
  // Everything the token needs is requested here, before the first value is used.
  float xq[4], wq[4], xk[4], wk[4], xv[4], wv[4];
  const int i0 = min(tid, dim - 1), c0 = min(tid, vdim - 1);        // threads beyond read what exists
  float* sv_q = saved + (int64_t)(q_ch + i0) * (taps - 1);
  float* sv_k = saved + (int64_t)(k_ch + i0) * (taps - 1);
  float* sv_v = saved + (int64_t)(v_ch + c0) * (taps - 1);
  load_taps(p, p_stride, t, conv_off + q_ch + i0, sv_q, conv_w + (int64_t)(q_ch + i0) * taps, taps, xq, wq);
  load_taps(p, p_stride, t, conv_off + k_ch + i0, sv_k, conv_w + (int64_t)(k_ch + i0) * taps, taps, xk, wk);
  load_taps(p, p_stride, t, conv_off + v_ch + c0, sv_v, conv_w + (int64_t)(v_ch + c0) * taps, taps, xv, wv);
  const int ai = a_per_head ? h : h * dim + i0;
  const float pre_a = a[(int64_t)t * a_stride + ai] + dt_bias[ai];
  const float pre_b = to_f32(p[(int64_t)t * p_stride + b_off + h]);
  const float rate = expf(a_log[h]);
  float pre_g[4], wn[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    pre_g[e] = gate[(int64_t)t * gate_stride + h * vdim + cq * 4 + e];
    wn[e] = w_norm[cq * 4 + e];
  }
  float* S_mem = row + (int64_t)h * dim * vdim + cq * 4;
  f32x4 S[DS];
#pragma unroll
  for (int j = 0; j < DS; ++j) {
    const int i = sl * DS + j;
    S[j] = (owner && i < dim) ? *(const f32x4*)(S_mem + (int64_t)i * vdim) : f32x4{0.f, 0.f, 0.f, 0.f};
  }

  float sq = 0.f, sk = 0.f;
  if (tid < dim) {
    const float q = conv_of(xq, wq), k = conv_of(xk, wk);
    qs[tid] = q;
    ks[tid] = k;
    sq = q * q;
    sk = k * k;
    gs[tid] = expf(-rate * softplus(pre_a));
    if (update_saved) {         // no other head reads these channels: this thread is their only reader
      store_saved(sv_q, xq, taps);
      store_saved(sv_k, xk, taps);
    }
  }
  if (tid < vdim) {
    vs[tid] = conv_of(xv, wv);
    if (update_saved) store_saved(sv_v, xv, taps);
  }
  sq = block_sum_dyn(sq, red, nw);
  sk = block_sum_dyn(sk, red, nw);      // its barriers also make qs, ks, gs and vs visible
  const float rq = q_scale / sqrtf(sq + 1e-6f), rk = 1.f / sqrtf(sk + 1e-6f);
  const float beta = 1.f / (1.f + expf(-pre_b));
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  if (owner) {
#pragma unroll
    for (int j = 0; j < DS; ++j) {
      const int i = sl * DS + j;
      if (i < dim) {
        const float g = gs[i], k = ks[i] * rk;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          S[j][e] *= g;
          acc[e] = fmaf(S[j][e], k, acc[e]);
        }
      }
    }
    part[sl][cq] = acc;
  }
  __syncthreads();
  f32x4 o = {0.f, 0.f, 0.f, 0.f};
  if (owner) {
    const f32x4 p0 = part[0][cq], p1 = part[1][cq], p2 = part[2][cq], p3 = part[3][cq];
    f32x4 u;
#pragma unroll
    for (int e = 0; e < 4; ++e) u[e] = beta * (vs[cq * 4 + e] - (((p0[e] + p1[e]) + p2[e]) + p3[e]));
#pragma unroll
    for (int j = 0; j < DS; ++j) {
      const int i = sl * DS + j;
      if (i < dim) {
        const float k = ks[i] * rk, q = qs[i] * rq;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          S[j][e] = fmaf(k, u[e], S[j][e]);
          o[e] = fmaf(S[j][e], q, o[e]);
        }
        *(f32x4*)(S_mem + (int64_t)i * vdim) = S[j];
      }
    }
  }
  __syncthreads();                      // the first round's sums have been read
  if (owner) part[sl][cq] = o;
  __syncthreads();
  float oo = 0.f;
  if (sl == 0) {
    const f32x4 p0 = part[0][cq], p1 = part[1][cq], p2 = part[2][cq], p3 = part[3][cq];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      o[e] = ((p0[e] + p1[e]) + p2[e]) + p3[e];
      oo += o[e] * o[e];
    }
  }
  const float ss = block_sum_dyn(oo, red, nw);
  if (sl == 0) {
    const float rn = 1.f / sqrtf(ss / (float)vdim + eps);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float sg = 1.f / (1.f + expf(-pre_g[e]));
      z[((int64_t)t * heads + h) * vdim + cq * 4 + e] = from_f32<TZ>(o[e] * rn * wn[e] * (gate_kind ? pre_g[e] * sg : sg));
    }
  }
}

}  // namespace

#define TL_DISPATCH_T(dtype, ...)                 \
  if ((dtype) == 0) { using T = float; __VA_ARGS__ } \
  else if ((dtype) == 1) { using T = bf16_t; __VA_ARGS__ } \
  else return TL_ERR_ARG;

extern "C" {

int tl_delta_prepare(const void* p, int64_t p_stride, int conv_off, int b_off, const float* a, int64_t a_stride,
                     const float* conv_w, const float* a_log, const float* dt_bias, const float* state,
                     int64_t state_stride, int64_t saved_off, const int32_t* req_of_token, const int32_t* cu_seqlens,
                     const int32_t* state_slots, float* qn, float* kn, float* vc, float* beta, float* decay,
                     int n_tokens, int heads, int kv_heads, int dim, int vdim, int taps, float q_scale, int a_per_head,
                     int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  if (heads <= 0 || heads > 65535 || kv_heads <= 0 || heads % kv_heads || dim <= 0 || dim > kMaxDim || vdim <= 0 ||
      taps < 1 || taps > kMaxTaps)
    return TL_ERR_ARG;
  dim3 g(n_tokens, heads), b(kPrepThreads);
  TL_DISPATCH_T(dtype, hipLaunchKernelGGL(delta_prepare_kernel<T>, g, b, 0, stream, (const T*)p, p_stride, conv_off,
                                          b_off, a, a_stride, conv_w, a_log, dt_bias, state, state_stride, saved_off,
                                          req_of_token, cu_seqlens, state_slots, qn, kn, vc, beta, decay, heads,
                                          kv_heads, dim, vdim, taps, q_scale, a_per_head);)
  return tl_launch_status();
}

int tl_conv_state_update(const void* p, int64_t p_stride, int conv_off, int channels, float* state,
                         int64_t state_stride, int64_t saved_off, const int32_t* cu_seqlens,
                         const int32_t* state_slots, int n_requests, int taps, int dtype, hipStream_t stream) {
  if (n_requests <= 0 || taps <= 1) return TL_OK;
  if (channels <= 0 || taps > kMaxTaps || n_requests > 65535) return TL_ERR_ARG;
  dim3 g((channels + 255) / 256, n_requests), b(256);
  TL_DISPATCH_T(dtype, hipLaunchKernelGGL(conv_state_update_kernel<T>, g, b, 0, stream, (const T*)p, p_stride,
                                          conv_off, channels, state, state_stride, saved_off, cu_seqlens, state_slots,
                                          taps);)
  return tl_launch_status();
}

int tl_delta_recurrence(const float* qn, const float* kn, const float* vc, const float* beta, const float* decay,
                        float* state, int64_t state_stride, const int32_t* cu_seqlens, const int32_t* state_slots,
                        float* out, int n_requests, int heads, int dim, int vdim, hipStream_t stream) {
  if (n_requests <= 0) return TL_OK;
  if (heads <= 0 || heads > 65535 || dim <= 0 || dim > kMaxDim || vdim <= 0 || (vdim + kRecCols - 1) / kRecCols > 65535)
    return TL_ERR_ARG;
  dim3 g(n_requests, heads, (vdim + kRecCols - 1) / kRecCols), b(kRecThreads);
#define TL_REC(DS)                                                                                                   \
  hipLaunchKernelGGL(delta_recurrence_kernel<DS>, g, b, 0, stream, qn, kn, vc, beta, decay, state, state_stride,     \
                     cu_seqlens, state_slots, out, heads, dim, vdim)
  if (dim <= 16) TL_REC(2);
  else if (dim <= 32) TL_REC(4);
  else if (dim <= 64) TL_REC(8);
  else if (dim <= 128) TL_REC(16);
  else TL_REC(32);
#undef TL_REC
  return tl_launch_status();
}

// Row t of `a`: the decay's pre-activations (heads x dim, or heads with a_per_head); of `gate`: the gate's (heads x
// vdim); both float32.
int tl_delta_decode(const void* p, int64_t p_stride, int conv_off, int b_off, const float* a, int64_t a_stride,
                    int a_per_head, const float* gate, int64_t gate_stride, int gate_kind, const float* conv_w, const float* a_log, const float* dt_bias, const float* w_norm, float* state,
                    int64_t state_stride, int64_t saved_off, const int32_t* cu_seqlens, const int32_t* state_slots,
                    void* z, int n_requests, int heads, int kv_heads, int dim, int vdim, int taps, float q_scale,
                    float eps, int update_saved, int dtype, int z_dtype, hipStream_t stream) {
  if (n_requests <= 0) return TL_OK;
  if (heads <= 0 || heads > 65535 || kv_heads <= 0 || heads % kv_heads || dim <= 0 || dim > kMaxDim || vdim <= 0 ||
      vdim > kDecodeThreads || vdim % 4 || state_stride % 4 || dim > kDecodeThreads || taps < 1 || taps > 4 ||
      (update_saved && heads != kv_heads) || gate_kind < 0 || gate_kind > 1 || !a || !gate)
    return TL_ERR_ARG;
  const int threads = vdim > dim ? vdim : dim;      // a thread per value column and per key channel
  dim3 g(n_requests, heads), b((threads + TL_WAVE - 1) / TL_WAVE * TL_WAVE);
#define TL_DEC(TT, TZ, D)                                                                                          \
  hipLaunchKernelGGL((delta_decode_kernel<TT, TZ, D>), g, b, 0, stream, (const TT*)p, p_stride, conv_off, b_off, a, \
                     a_stride, a_per_head, gate, gate_stride, gate_kind, conv_w, a_log, dt_bias, w_norm, state,     \
                     state_stride, saved_off, cu_seqlens, state_slots, (TZ*)z, heads, kv_heads, dim, vdim, taps,    \
                     q_scale, eps, update_saved)
#define TL_DEC_D(TT, TZ)                  \
  if (dim <= 16) TL_DEC(TT, TZ, 4);       \
  else if (dim <= 32) TL_DEC(TT, TZ, 8);  \
  else if (dim <= 64) TL_DEC(TT, TZ, 16); \
  else if (dim <= 128) TL_DEC(TT, TZ, 32); \
  else TL_DEC(TT, TZ, 64);
  // the projections' element type and the result's: float32 projections may feed a bfloat16 output product
  if (dtype == 0 && z_dtype == 0) { TL_DEC_D(float, float) }
  else if (dtype == 0 && z_dtype == 1) { TL_DEC_D(float, bf16_t) }
  else if (dtype == 1 && z_dtype == 1) { TL_DEC_D(bf16_t, bf16_t) }
  else return TL_ERR_ARG;
#undef TL_DEC_D
#undef TL_DEC
  return tl_launch_status();
}

int tl_head_norm_gate(const float* o, const float* w, int w_head_stride, const float* gate, int64_t gate_stride, void* z,
                      int n_tokens, int heads, int vdim, float eps, int gate_kind, float scale, int dtype,
                      hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  if (heads <= 0 || heads > 65535 || vdim <= 0 || (w_head_stride != 0 && w_head_stride != vdim) || gate_kind < 0 ||
      gate_kind > 1)
    return TL_ERR_ARG;
  dim3 g(n_tokens, heads), b(TL_WAVE);
  TL_DISPATCH_T(dtype, hipLaunchKernelGGL(head_norm_gate_kernel<T>, g, b, 0, stream, o, w, w_head_stride, gate,
                                          gate_stride, (T*)z, heads, vdim, eps, gate_kind, scale);)
  return tl_launch_status();
}

}  // extern "C"
