// Layer norm with weight and bias, (v - mean) / sqrt(var + eps) * w + b with var the mean squared
// deviation, in two forms: on the sum of a sublayer's result and the scaled residual stream, written
// back into the stream (a layer whose norm FOLLOWS the sum: x <- LN(alpha * x + y)), and on gathered
// rows of the stream for the output head; and on a sublayer's result by itself, added to the stream times a
// constant (a layer with a norm in front of AND behind every sublayer: x <- x + m * LN(y)), with the norm that
// reads the new stream next in the same pass over the row.
//
// Statistics, weight, bias and the stream are float32 in both precisions.  The mean is taken first and
// the variance from the deviations (two sums), not from the mean of squares.
#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / TL_WAVE;

// v[j] = alpha * x[row, j] + y[row, j] (y optional); x[row] <- LN(v) * w + b (when `inplace`), out[row] likewise
// in TO (optional).  `rows` (optional) gathers: output row i reads stream row rows[i].  One workgroup a row;
// rows of up to KEEP * kThreads elements stay in registers between the passes, longer ones are formed again.
template <typename TO, int KEEP>
__global__ __launch_bounds__(kThreads) void layer_norm_kernel(const float* __restrict__ y, const float* __restrict__ w,
                                                              const float* __restrict__ b, float* __restrict__ x,
                                                              const int32_t* __restrict__ rows, TO* __restrict__ out,
                                                              int hidden, float alpha, float eps, int inplace) {
  __shared__ float red[kWaves];
  const int64_t src_row = rows ? rows[blockIdx.x] : blockIdx.x;
  float* xr = x + src_row * hidden;
  const float* yr = y ? y + src_row * hidden : nullptr;
  TO* dst = out ? out + (int64_t)blockIdx.x * hidden : nullptr;
  const float inv_n = 1.f / (float)hidden;
  if (hidden <= KEEP * kThreads) {
    float v[KEEP];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < KEEP; ++i) {
      const int j = threadIdx.x + i * kThreads;
      v[i] = 0.f;
      if (j < hidden) v[i] = yr ? fmaf(alpha, xr[j], yr[j]) : alpha * xr[j];
      s += v[i];
    }
    const float mean = block_sum<kWaves>(s, red) * inv_n;
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < KEEP; ++i) {
      const int j = threadIdx.x + i * kThreads;
      const float d = j < hidden ? v[i] - mean : 0.f;
      q += d * d;
    }
    const float r = 1.f / sqrtf(block_sum<kWaves>(q, red) * inv_n + eps);
#pragma unroll
    for (int i = 0; i < KEEP; ++i) {
      const int j = threadIdx.x + i * kThreads;
      if (j < hidden) {
        const float o = (v[i] - mean) * r * w[j] + b[j];
        if (inplace) xr[j] = o;
        if (dst) dst[j] = from_f32<TO>(o);
      }
    }
    return;
  }
  float s = 0.f;
  for (int j = threadIdx.x; j < hidden; j += kThreads) s += yr ? fmaf(alpha, xr[j], yr[j]) : alpha * xr[j];
  const float mean = block_sum<kWaves>(s, red) * inv_n;
  float q = 0.f;
  for (int j = threadIdx.x; j < hidden; j += kThreads) {
    const float d = (yr ? fmaf(alpha, xr[j], yr[j]) : alpha * xr[j]) - mean;
    q += d * d;
  }
  const float r = 1.f / sqrtf(block_sum<kWaves>(q, red) * inv_n + eps);
  for (int j = threadIdx.x; j < hidden; j += kThreads) {
    const float o = ((yr ? fmaf(alpha, xr[j], yr[j]) : alpha * xr[j]) - mean) * r * w[j] + b[j];
    if (inplace) xr[j] = o;
    if (dst) dst[j] = from_f32<TO>(o);
  }
}

// x[row] <- x[row] + mult * (LN(y[row]) * w + b); then, if w2 is given, out[row] = LN(x[row]) * w2 + b2 in TO: the
// norm of whatever reads the stream next, formed while the row is in registers.  One workgroup a row.  Everything
// the row needs (y, x, both norms' weights and biases) is requested before the first sum is taken, so the four sums
// over the workgroup are all that stands between the loads and the stores.  VEC 4: rows of a multiple of four
// elements, KEEP vectors of four a thread; VEC 1: any row, KEEP elements a thread.
template <typename TO, int KEEP, int VEC>
__global__ __launch_bounds__(kThreads) void layer_norm_add_kernel(const float* __restrict__ y, const float* __restrict__ w,
                                                                  const float* __restrict__ b, float* __restrict__ x,
                                                                  const float* __restrict__ w2, const float* __restrict__ b2,
                                                                  TO* __restrict__ out, int hidden, float mult, float eps,
                                                                  float eps2) {
  __shared__ float red[kWaves];
  const int64_t row = blockIdx.x;
  float* xr = x + row * hidden;
  const float* yr = y + row * hidden;
  const float inv_n = 1.f / (float)hidden;
  constexpr int N = KEEP * VEC;
  float v[N], xv[N], wv[N], bv[N], w2v[N], b2v[N];
#pragma unroll
  for (int i = 0; i < KEEP; ++i) {
    const int j = (threadIdx.x + i * kThreads) * VEC;
    const bool in = j < hidden;
    if constexpr (VEC == 4) {
      const f32x4 z = {0.f, 0.f, 0.f, 0.f};
      const f32x4 a = in ? *(const f32x4*)(yr + j) : z, c = in ? *(const f32x4*)(xr + j) : z;
      const f32x4 d = in ? *(const f32x4*)(w + j) : z, e = in ? *(const f32x4*)(b + j) : z;
      const f32x4 f = (in && w2) ? *(const f32x4*)(w2 + j) : z, g = (in && w2) ? *(const f32x4*)(b2 + j) : z;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        v[i * 4 + u] = a[u];
        xv[i * 4 + u] = c[u];
        wv[i * 4 + u] = d[u];
        bv[i * 4 + u] = e[u];
        w2v[i * 4 + u] = f[u];
        b2v[i * 4 + u] = g[u];
      }
    } else {
      v[i] = in ? yr[j] : 0.f;
      xv[i] = in ? xr[j] : 0.f;
      wv[i] = in ? w[j] : 0.f;
      bv[i] = in ? b[j] : 0.f;
      w2v[i] = (in && w2) ? w2[j] : 0.f;
      b2v[i] = (in && w2) ? b2[j] : 0.f;
    }
  }
  auto inside = [&](int i) { return (threadIdx.x + (i / VEC) * kThreads) * VEC + i % VEC < hidden; };
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < N; ++i) s += v[i];
  float mean = block_sum<kWaves>(s, red) * inv_n;
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < N; ++i) {
    const float d = inside(i) ? v[i] - mean : 0.f;
    q += d * d;
  }
  float r = 1.f / sqrtf(block_sum<kWaves>(q, red) * inv_n + eps);
  s = 0.f;
#pragma unroll
  for (int i = 0; i < N; ++i) {
    v[i] = inside(i) ? fmaf(mult, (v[i] - mean) * r * wv[i] + bv[i], xv[i]) : 0.f;
    s += v[i];
  }
#pragma unroll
  for (int i = 0; i < KEEP; ++i) {
    const int j = (threadIdx.x + i * kThreads) * VEC;
    if (j < hidden) {
      if constexpr (VEC == 4) *(f32x4*)(xr + j) = f32x4{v[i * 4], v[i * 4 + 1], v[i * 4 + 2], v[i * 4 + 3]};
      else xr[j] = v[i];
    }
  }
  if (!w2) return;
  mean = block_sum<kWaves>(s, red) * inv_n;
  q = 0.f;
#pragma unroll
  for (int i = 0; i < N; ++i) {
    const float d = inside(i) ? v[i] - mean : 0.f;
    q += d * d;
  }
  r = 1.f / sqrtf(block_sum<kWaves>(q, red) * inv_n + eps2);
  TO* dst = out + row * hidden;
#pragma unroll
  for (int i = 0; i < KEEP; ++i) {
    const int j = (threadIdx.x + i * kThreads) * VEC;
    if (j < hidden) {
      if constexpr (VEC == 4) {
        typedef __attribute__((ext_vector_type(4))) decltype(from_f32<TO>(0.f)) out4;
        out4 o;
#pragma unroll
        for (int u = 0; u < 4; ++u) o[u] = from_f32<TO>((v[i * 4 + u] - mean) * r * w2v[i * 4 + u] + b2v[i * 4 + u]);
        *(out4*)(dst + j) = o;
      } else {
        dst[j] = from_f32<TO>((v[i] - mean) * r * w2v[i] + b2v[i]);
      }
    }
  }
}

template <typename TO>
int launch_add(const float* y, const float* w, const float* b, float* x, const float* w2, const float* b2, TO* out, int n,
               int hidden, float mult, float eps, float eps2, hipStream_t stream) {
  dim3 g(n), blk(kThreads);
#define TL_LNA(KEEP, VEC)                                                                                            \
  hipLaunchKernelGGL((layer_norm_add_kernel<TO, KEEP, VEC>), g, blk, 0, stream, y, w, b, x, w2, b2, out, hidden, mult, \
                     eps, eps2)
  const uintptr_t ptrs = (uintptr_t)y | (uintptr_t)w | (uintptr_t)b | (uintptr_t)x | (uintptr_t)w2 | (uintptr_t)b2 | (uintptr_t)out;
  if (hidden % 4 == 0 && (ptrs & 15) == 0) {      // vectors of four need 16-byte boundaries
    const int vecs = hidden / 4;
    if (vecs <= kThreads) TL_LNA(1, 4);
    else if (vecs <= 2 * kThreads) TL_LNA(2, 4);
    else if (vecs <= 4 * kThreads) TL_LNA(4, 4);
    else TL_LNA(8, 4);
  } else {
    if (hidden <= 4 * kThreads) TL_LNA(4, 1);
    else if (hidden <= 16 * kThreads) TL_LNA(16, 1);
    else TL_LNA(32, 1);
  }
#undef TL_LNA
  return tl_launch_status();
}

template <typename TO>
int launch(const float* y, const float* w, const float* b, float* x, const int32_t* rows, TO* out, int n, int hidden,
           float alpha, float eps, int inplace, hipStream_t stream) {
  dim3 g(n), blk(kThreads);
  if (hidden <= 8 * kThreads)
    hipLaunchKernelGGL((layer_norm_kernel<TO, 8>), g, blk, 0, stream, y, w, b, x, rows, out, hidden, alpha, eps, inplace);
  else
    hipLaunchKernelGGL((layer_norm_kernel<TO, 32>), g, blk, 0, stream, y, w, b, x, rows, out, hidden, alpha, eps, inplace);
  return tl_launch_status();
}

}  // namespace

extern "C" {

// x[t] <- LN(alpha * x[t] + y[t]) * w + b for n_rows rows (y may be null); copy (optional, copy_dtype 0
// float32 / 1 bfloat16) receives the new rows too.
int tl_layer_norm_sum(const float* y, const float* w, const float* b, float* x, void* copy, int n_rows, int hidden,
                      float alpha, float eps, int copy_dtype, hipStream_t stream) {
  if (n_rows <= 0) return TL_OK;
  if (hidden <= 0 || !w || !b || !x) return TL_ERR_ARG;
  if (copy_dtype == 1) return launch<bf16_t>(y, w, b, x, nullptr, (bf16_t*)copy, n_rows, hidden, alpha, eps, 1, stream);
  if (copy_dtype == 0) return launch<float>(y, w, b, x, nullptr, (float*)copy, n_rows, hidden, alpha, eps, 1, stream);
  return TL_ERR_ARG;
}

// x[t] <- x[t] + mult * (LN(y[t]) * w + b) for n_rows rows; with w2, b2 and out (out_dtype 0 float32 / 1 bfloat16)
// also out[t] = LN(x[t]) * w2 + b2 of the new rows.  Rows of at most 8,192 elements.
int tl_layer_norm_add(const float* y, const float* w, const float* b, float* x, const float* w2, const float* b2,
                      void* out, int n_rows, int hidden, float mult, float eps, float eps2, int out_dtype,
                      hipStream_t stream) {
  if (n_rows <= 0) return TL_OK;
  if (hidden <= 0 || hidden > 32 * kThreads || !y || !w || !b || !x || (w2 && (!b2 || !out))) return TL_ERR_ARG;
  if (out_dtype == 1) return launch_add<bf16_t>(y, w, b, x, w2, b2, (bf16_t*)out, n_rows, hidden, mult, eps, eps2, stream);
  if (out_dtype == 0) return launch_add<float>(y, w, b, x, w2, b2, (float*)out, n_rows, hidden, mult, eps, eps2, stream);
  return TL_ERR_ARG;
}

// out[i] = LN(x[rows[i] or i]) * w + b; x is not written.
int tl_layer_norm_rows(const float* x, const int32_t* rows, const float* w, const float* b, void* out, int n,
                       int hidden, float eps, int out_dtype, hipStream_t stream) {
  if (n <= 0) return TL_OK;
  if (hidden <= 0 || !w || !b || !x || !out) return TL_ERR_ARG;
  if (out_dtype == 1)
    return launch<bf16_t>(nullptr, w, b, const_cast<float*>(x), rows, (bf16_t*)out, n, hidden, 1.f, eps, 0, stream);
  if (out_dtype == 0)
    return launch<float>(nullptr, w, b, const_cast<float*>(x), rows, (float*)out, n, hidden, 1.f, eps, 0, stream);
  return TL_ERR_ARG;
}

}  // extern "C"
