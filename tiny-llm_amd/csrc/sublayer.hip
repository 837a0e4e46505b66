// Kernels around a sublayer whose norm sits on its OUTPUT: x += scale * w * y / rms(y), the copy
// of the residual stream in the engine's element type that the next sublayer's products read, a
// gated unit with clamped inputs, and the soft cap of the logits.
//
// The residual stream, the norm's statistics and its weight are float32 in both precisions.
#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / TL_WAVE;

// x[t] += scale * w * y[t] / sqrt(mean(y[t]^2) + eps); copy[t] = x[t] in TC (optional).
// One workgroup per row.  `w` is the norm's effective weight, `scale` (optional) a factor per channel.
// Rows of up to KEEP * kThreads elements stay in registers between the two passes, and what the second
// pass needs (x, w, scale) is requested before the sum of squares is known (KEEP 8 for rows of up to
// 2,048 elements, 32 up to 8,192; longer rows are read twice).
template <typename TC, int KEEP>
__global__ __launch_bounds__(kThreads) void norm_scale_add_kernel(const float* __restrict__ y,
                                                                  const float* __restrict__ w,
                                                                  const float* __restrict__ scale,
                                                                  float* __restrict__ x, TC* __restrict__ copy,
                                                                  int hidden, float eps) {
  __shared__ float red[kWaves];
  const float* src = y + (int64_t)blockIdx.x * hidden;
  float* dst = x + (int64_t)blockIdx.x * hidden;
  float ss = 0.f;
  if (hidden <= KEEP * kThreads) {
    float yv[KEEP], xv[KEEP], wv[KEEP];
#pragma unroll
    for (int i = 0; i < KEEP; ++i) {
      const int j = threadIdx.x + i * kThreads;
      const bool in = j < hidden;
      yv[i] = in ? src[j] : 0.f;
      xv[i] = in ? dst[j] : 0.f;
      wv[i] = in ? (scale ? w[j] * scale[j] : w[j]) : 0.f;
      ss += yv[i] * yv[i];
    }
    ss = block_sum<kWaves>(ss, red);
    const float r = 1.f / sqrtf(ss / (float)hidden + eps);
#pragma unroll
    for (int i = 0; i < KEEP; ++i) {
      const int j = threadIdx.x + i * kThreads;
      if (j < hidden) {
        const float s = xv[i] + yv[i] * r * wv[i];
        dst[j] = s;
        if (copy) copy[(int64_t)blockIdx.x * hidden + j] = from_f32<TC>(s);
      }
    }
    return;
  }
  for (int j = threadIdx.x; j < hidden; j += kThreads) {
    const float v = src[j];
    ss += v * v;
  }
  ss = block_sum<kWaves>(ss, red);
  const float r = 1.f / sqrtf(ss / (float)hidden + eps);
  for (int j = threadIdx.x; j < hidden; j += kThreads) {
    float v = src[j] * r * w[j];
    if (scale) v *= scale[j];
    const float s = dst[j] + v;
    dst[j] = s;
    if (copy) copy[(int64_t)blockIdx.x * hidden + j] = from_f32<TC>(s);
  }
}

template <typename TO>
__global__ void cast_rows_kernel(const float* __restrict__ x, TO* __restrict__ out, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i < total) out[i] = from_f32<TO>(x[i]);
}

// z[t, j] = g * sigmoid(alpha * g) * (u + shift), g = min(gate_up[t, j], limit),
// u = clamp(gate_up[t, inter + j], -limit, limit).
template <typename T>
__global__ void clamped_glu_kernel(const T* __restrict__ gate_up, T* __restrict__ z, int64_t total, int inter,
                                   int64_t in_stride, float limit, float alpha, float shift) {
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= total) return;
  const int64_t t = i / inter;
  const int j = (int)(i - t * inter);
  const float g = fminf(to_f32(gate_up[t * in_stride + j]), limit);
  const float u = fminf(fmaxf(to_f32(gate_up[t * in_stride + inter + j]), -limit), limit);
  z[i] = from_f32<T>(g / (1.f + expf(-alpha * g)) * (u + shift));
}

// z[t, j] = gelu(gate_up[t, j]) * gate_up[t, inter + j], gelu in its tanh form:
// 0.5 g (1 + tanh(sqrt(2 / pi) (g + 0.044715 g^3))).
template <typename T>
__global__ void gelu_glu_kernel(const T* __restrict__ gate_up, T* __restrict__ z, int64_t total, int inter,
                                int64_t in_stride) {
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= total) return;
  const int64_t t = i / inter;
  const int j = (int)(i - t * inter);
  const float g = to_f32(gate_up[t * in_stride + j]);
  const float u = to_f32(gate_up[t * in_stride + inter + j]);
  const float act = 0.5f * g * (1.f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
  z[i] = from_f32<T>(act * u);
}

__global__ void softcap_kernel(float* __restrict__ x, int64_t total, float cap) {
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i < total) x[i] = cap * tanhf(x[i] / cap);
}

// Two streams side by side as the operand of one product: operand[t] = [a[t] | b[t]] rounded to T, and
// init[t] = vec (a row that the product then adds its result to, so a vector joins every row without a kernel of
// its own).  One thread an element of the wider of the two outputs.
template <typename T>
__global__ void stream_join_kernel(const float* __restrict__ a, const float* __restrict__ b, const float* __restrict__ vec,
                                   T* __restrict__ operand, float* __restrict__ init, int64_t total, int width) {
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= total) return;
  const int64_t t = i / (2 * width);
  const int c = (int)(i - t * 2 * width);
  operand[i] = from_f32<T>(c < width ? a[t * width + c] : b[t * width + c - width]);
  if (c < width) init[t * width + c] = vec ? vec[c] : 0.f;
}

}  // namespace

extern "C" {

// copy_dtype: 0 float32, 1 bfloat16; copy and scale may be null.
int tl_norm_scale_add(const float* y, const float* w, const float* scale, float* x, void* copy, int n_rows,
                      int hidden, float eps, int copy_dtype, hipStream_t stream) {
  if (n_rows <= 0) return TL_OK;
  if (hidden <= 0) return TL_ERR_ARG;
  dim3 g(n_rows), b(kThreads);
  const bool few = hidden <= 8 * kThreads;
  if (copy_dtype == 1 && few)
    hipLaunchKernelGGL((norm_scale_add_kernel<bf16_t, 8>), g, b, 0, stream, y, w, scale, x, (bf16_t*)copy, hidden, eps);
  else if (copy_dtype == 1)
    hipLaunchKernelGGL((norm_scale_add_kernel<bf16_t, 32>), g, b, 0, stream, y, w, scale, x, (bf16_t*)copy, hidden, eps);
  else if (copy_dtype == 0 && few)
    hipLaunchKernelGGL((norm_scale_add_kernel<float, 8>), g, b, 0, stream, y, w, scale, x, (float*)copy, hidden, eps);
  else if (copy_dtype == 0)
    hipLaunchKernelGGL((norm_scale_add_kernel<float, 32>), g, b, 0, stream, y, w, scale, x, (float*)copy, hidden, eps);
  else
    return TL_ERR_ARG;
  return tl_launch_status();
}

int tl_cast_rows(const float* x, void* out, int64_t total, int out_dtype, hipStream_t stream) {
  if (total <= 0) return TL_OK;
  dim3 g((unsigned)ceil_div64(total, kThreads)), b(kThreads);
  if (out_dtype == 1)
    hipLaunchKernelGGL(cast_rows_kernel<bf16_t>, g, b, 0, stream, x, (bf16_t*)out, total);
  else if (out_dtype == 0)
    hipLaunchKernelGGL(cast_rows_kernel<float>, g, b, 0, stream, x, (float*)out, total);
  else
    return TL_ERR_ARG;
  return tl_launch_status();
}

int tl_clamped_glu(const void* gate_up, void* z, int n_rows, int inter, int64_t in_stride, float limit, float alpha,
                   float shift, int dtype, hipStream_t stream) {
  if (n_rows <= 0) return TL_OK;
  if (inter <= 0 || in_stride < 2 * (int64_t)inter) return TL_ERR_ARG;
  const int64_t total = (int64_t)n_rows * inter;
  dim3 g((unsigned)ceil_div64(total, kThreads)), b(kThreads);
  if (dtype == 0)
    hipLaunchKernelGGL(clamped_glu_kernel<float>, g, b, 0, stream, (const float*)gate_up, (float*)z, total, inter,
                       in_stride, limit, alpha, shift);
  else if (dtype == 1)
    hipLaunchKernelGGL(clamped_glu_kernel<bf16_t>, g, b, 0, stream, (const bf16_t*)gate_up, (bf16_t*)z, total, inter,
                       in_stride, limit, alpha, shift);
  else
    return TL_ERR_ARG;
  return tl_launch_status();
}

int tl_gelu_glu(const void* gate_up, void* z, int n_rows, int inter, int64_t in_stride, int dtype, hipStream_t stream) {
  if (n_rows <= 0) return TL_OK;
  if (inter <= 0 || in_stride < 2 * (int64_t)inter) return TL_ERR_ARG;
  const int64_t total = (int64_t)n_rows * inter;
  dim3 g((unsigned)ceil_div64(total, kThreads)), b(kThreads);
  if (dtype == 0)
    hipLaunchKernelGGL(gelu_glu_kernel<float>, g, b, 0, stream, (const float*)gate_up, (float*)z, total, inter, in_stride);
  else if (dtype == 1)
    hipLaunchKernelGGL(gelu_glu_kernel<bf16_t>, g, b, 0, stream, (const bf16_t*)gate_up, (bf16_t*)z, total, inter,
                       in_stride);
  else
    return TL_ERR_ARG;
  return tl_launch_status();
}

int tl_softcap(float* x, int64_t total, float cap, hipStream_t stream) {
  if (total <= 0) return TL_OK;
  if (!(cap > 0.f)) return TL_ERR_ARG;
  hipLaunchKernelGGL(softcap_kernel, dim3((unsigned)ceil_div64(total, kThreads)), dim3(kThreads), 0, stream, x, total,
                     cap);
  return tl_launch_status();
}

// a, b: float32 [n_rows, width]; operand: [n_rows, 2 * width] in dtype; init: float32 [n_rows, width] (every row
// becomes vec, or zeros without one).
int tl_stream_join(const float* a, const float* b, const float* vec, void* operand, float* init, int n_rows, int width,
                   int dtype, hipStream_t stream) {
  if (n_rows <= 0) return TL_OK;
  if (width <= 0 || !a || !b || !operand || !init) return TL_ERR_ARG;
  const int64_t total = (int64_t)n_rows * 2 * width;
  dim3 g((unsigned)ceil_div64(total, kThreads)), blk(kThreads);
  if (dtype == 0)
    hipLaunchKernelGGL(stream_join_kernel<float>, g, blk, 0, stream, a, b, vec, (float*)operand, init, total, width);
  else if (dtype == 1)
    hipLaunchKernelGGL(stream_join_kernel<bf16_t>, g, blk, 0, stream, a, b, vec, (bf16_t*)operand, init, total, width);
  else
    return TL_ERR_ARG;
  return tl_launch_status();
}

}  // extern "C"
