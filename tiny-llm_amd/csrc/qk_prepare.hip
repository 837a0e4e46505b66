// Between the query/key product and the attention kernel, for attention whose queries and keys carry a
// bias, are rotated on part of their dims and then scaled to unit root mean square, and whose values
// may be the keys themselves as projected; and behind the attention kernel, a sigmoid gate per head.
//
// Everything here is float32 arithmetic on the float32 result of the product; what leaves is rounded
// once to the engine's element type (queries, cached keys and values).
#include "common.h"

namespace {

// One wave per (token, head); heads 0 .. nq - 1 are queries, nq .. nq + nkv - 1 keys.
//   a = p[t, head, :] + bias[head, :]
//   keys with values_are_keys: v_cache[slot] = a           (before rotation and norm)
//   values otherwise (v_off >= 0): v_cache[slot] = p[t, v_off + kv head, :]
//   a <- rotate(a) on the first `rot` dims, pair i = (2i, 2i + 1) or (i, i + rot / 2), angle table row of the position
//   a <- a / sqrt(mean(a^2) + eps)   if unit_norm
//   queries -> q_out[t, head, :], keys -> k_cache[slot]    (a negative slot stores nothing)
template <typename T>
__global__ __launch_bounds__(TL_WAVE) void qk_prepare_kernel(
    const float* __restrict__ p, int64_t p_stride, const float* __restrict__ bias, const int32_t* __restrict__ positions,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, const int32_t* __restrict__ slot_mapping,
    T* __restrict__ q_out, int64_t q_stride, T* __restrict__ k_cache, T* __restrict__ v_cache, int nq, int nkv, int hd,
    int rot, int interleaved, int unit_norm, float eps, int values_are_keys, int v_off, int block_size) {
  const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const bool is_key = head >= nq;
  const int slot = slot_mapping ? slot_mapping[t] : -1;
  if (is_key && slot < 0) return;
  const float* src = p + (int64_t)t * p_stride + (int64_t)head * hd;
  const float* bs = bias ? bias + (int64_t)head * hd : nullptr;
  const int half = rot / 2, pairs = hd / 2;       // hd is even
  const int pos = positions[t];
  const float* cs = cos_t ? cos_t + (int64_t)pos * half : nullptr;
  const float* sn = sin_t ? sin_t + (int64_t)pos * half : nullptr;
  int64_t cache_row = 0;
  if (is_key) cache_row = (((int64_t)(slot / block_size) * nkv + (head - nq)) * block_size + slot % block_size) * hd;
  constexpr int kPairs = 2;                        // head sizes up to 256: at most 128 pairs, two a lane
  float ra[kPairs], rb[kPairs];
  int ia[kPairs], ib[kPairs];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kPairs; ++i) {
    const int j = lane + i * TL_WAVE;
    ra[i] = rb[i] = 0.f;
    ia[i] = ib[i] = 0;
    if (j < pairs) {
      if (j < half) {
        ia[i] = interleaved ? 2 * j : j;
        ib[i] = interleaved ? 2 * j + 1 : j + half;
      } else {
        ia[i] = rot + 2 * (j - half);
        ib[i] = ia[i] + 1;
      }
      float a = src[ia[i]], b = src[ib[i]];
      if (bs) {
        a += bs[ia[i]];
        b += bs[ib[i]];
      }
      if (is_key && values_are_keys) {
        v_cache[cache_row + ia[i]] = from_f32<T>(a);
        v_cache[cache_row + ib[i]] = from_f32<T>(b);
      }
      if (j < half) {
        const float c = cs[j], s = sn[j];
        ra[i] = c * a - s * b;
        rb[i] = s * a + c * b;
      } else {
        ra[i] = a;
        rb[i] = b;
      }
      ss += ra[i] * ra[i] + rb[i] * rb[i];
    }
  }
  float r = 1.f;
  if (unit_norm) r = 1.f / sqrtf(wave_sum(ss) / (float)hd + eps);
  T* dst = is_key ? k_cache + cache_row : q_out + (int64_t)t * q_stride + (int64_t)head * hd;
#pragma unroll
  for (int i = 0; i < kPairs; ++i) {
    const int j = lane + i * TL_WAVE;
    if (j < pairs) {
      dst[ia[i]] = from_f32<T>(ra[i] * r);
      dst[ib[i]] = from_f32<T>(rb[i] * r);
    }
  }
  if (is_key && !values_are_keys && v_off >= 0) {
    const float* vs = p + (int64_t)t * p_stride + v_off + (int64_t)(head - nq) * hd;
    for (int d = lane; d < hd; d += TL_WAVE) v_cache[cache_row + d] = from_f32<T>(vs[d]);
  }
}

// z[t, h, :] = a[t, h, :] * sigmoid(g[t, h]) * scale; one thread an element.
template <typename T>
__global__ void head_gate_kernel(const T* __restrict__ a, int64_t a_stride, const float* __restrict__ g, int64_t g_stride,
                                 T* __restrict__ z, int64_t z_stride, int64_t total, int heads, int hd, float scale) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int width = heads * hd;
  const int64_t t = i / width;
  const int c = (int)(i - t * width);
  const float gate = 1.f / (1.f + expf(-g[t * g_stride + c / hd]));
  z[t * z_stride + c] = from_f32<T>(to_f32(a[t * a_stride + c]) * gate * scale);
}

// The general form of the step between the product that reads the mixer's input and the attention kernel: the
// workgroups (t, 0 .. gridDim.y - 1) share a token's units and values out, a wave a unit at a time (steps of few
// tokens get many workgroups a token; each forms the sums of the whole-projection norm for itself).  Row t of p (float32) holds q as `q_units` units of `dim` numbers, then k as
// `k_units` units, then v as `nkv` heads of `vdim` numbers (from column v_off); a unit is one score map of one
// head, unit u = head * maps + map.  In this order, each step an option:
//   a = p + bias                                      (bias over [q | k | v], or null)
//   a <- a / sqrt(mean over ALL of the token's q (or k) numbers of a^2 + eps) * norm_w    (whole_norm; norm_w over [q | k])
//   a <- rotate(a) on the first `rot` dims of every unit, pair (i, i + rot/2) or (2i, 2i + 1)
//   a <- a / sqrt(mean over the unit of a^2 + eps)     (unit_norm)
//   q <- q * (1 + temp_coef * ln(floor((pos + 1) / temp_every) + 1))                       (temp_every > 0)
// Queries of map m leave as q_out[m][t][head][0 .. D), keys go to k_cache[m] and values to v_cache at the
// token's slot, pages [blocks, nkv, block_size, D]; D >= dim, vdim, and what lies beyond dim (vdim) is written as
// zeros, so that an attention kernel over heads of D computes the same scores and leaves the values' columns first.
// A negative slot (padding) stores nothing.
constexpr int kPrepThreads = 256, kPrepWaves = kPrepThreads / TL_WAVE, kPrepPerLane = 4;     // units of up to 256
template <typename T>
__global__ __launch_bounds__(kPrepThreads) void attn_prepare_kernel(
    const float* __restrict__ p, int64_t p_stride, const float* __restrict__ bias, const float* __restrict__ norm_w,
    const int32_t* __restrict__ positions, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int32_t* __restrict__ slot_mapping, T* __restrict__ q_out, int64_t q_stride, int64_t q_map_stride,
    T* __restrict__ k_cache0, T* __restrict__ k_cache1, T* __restrict__ v_cache, int heads, int nkv, int maps, int dim,
    int vdim, int D, int v_off, int rot, int interleaved, int whole_norm, int unit_norm, float eps, float temp_coef,
    int temp_every, int block_size) {
  __shared__ float red[kPrepWaves];
  const int t = blockIdx.x, tid = threadIdx.x, wave = tid / TL_WAVE, lane = tid % TL_WAVE;
  const float* row = p + (int64_t)t * p_stride;
  const int q_units = heads * maps, k_units = nkv * maps;
  const int q_size = q_units * dim, k_size = k_units * dim;
  const int pos = positions[t];
  const int slot = slot_mapping ? slot_mapping[t] : -1;
  float rq = 1.f, rk = 1.f;
  if (whole_norm) {
    float sq = 0.f, sk = 0.f;
    for (int c = tid; c < q_size; c += kPrepThreads) {
      const float a = row[c] + (bias ? bias[c] : 0.f);
      sq += a * a;
    }
    for (int c = q_size + tid; c < q_size + k_size; c += kPrepThreads) {
      const float a = row[c] + (bias ? bias[c] : 0.f);
      sk += a * a;
    }
    rq = 1.f / sqrtf(block_sum<kPrepWaves>(sq, red) / (float)q_size + eps);
    rk = 1.f / sqrtf(block_sum<kPrepWaves>(sk, red) / (float)k_size + eps);
  }
  float temp = 1.f;
  if (temp_every > 0) temp = 1.f + temp_coef * logf((float)((pos + 1) / temp_every) + 1.f);
  const int half = rot / 2;
  const float* cs = rot ? cos_t + (int64_t)pos * half : nullptr;
  const float* sn = rot ? sin_t + (int64_t)pos * half : nullptr;
  const int64_t page_row = slot >= 0 ? (int64_t)(slot / block_size) * nkv * block_size + slot % block_size : 0;
  for (int u = blockIdx.y * kPrepWaves + wave; u < q_units + k_units; u += gridDim.y * kPrepWaves) {
    const bool is_key = u >= q_units;
    if (is_key && slot < 0) continue;
    const int uu = is_key ? u - q_units : u;
    const int head = uu / maps, map = uu % maps;
    const int c0 = (is_key ? q_size : 0) + uu * dim;        // the unit's first column in p, bias and norm_w
    const float r = is_key ? rk : rq;
    auto value = [&](int d) {
      float a = row[c0 + d] + (bias ? bias[c0 + d] : 0.f);
      if (whole_norm) a = a * r * norm_w[c0 + d];
      return a;
    };
    float out[kPrepPerLane];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < kPrepPerLane; ++i) {
      const int d = lane + i * TL_WAVE;
      out[i] = 0.f;
      if (d < dim) {
        float a = value(d);
        if (d < rot) {
          int j, partner;
          bool first;
          if (interleaved) {
            j = d / 2;
            first = (d & 1) == 0;
            partner = first ? d + 1 : d - 1;
          } else {
            first = d < half;
            j = first ? d : d - half;
            partner = first ? d + half : d - half;
          }
          const float b = value(partner);
          a = first ? a * cs[j] - b * sn[j] : a * cs[j] + b * sn[j];
        }
        out[i] = a;
        ss += a * a;
      }
    }
    float f = is_key ? 1.f : temp;
    if (unit_norm) f *= 1.f / sqrtf(wave_sum(ss) / (float)dim + eps);
    T* dst;
    if (is_key)
      dst = (map == 0 ? k_cache0 : k_cache1) + (page_row + (int64_t)head * block_size) * D;
    else
      dst = q_out + (int64_t)map * q_map_stride + (int64_t)t * q_stride + (int64_t)head * D;
#pragma unroll
    for (int i = 0; i < kPrepPerLane; ++i) {
      const int d = lane + i * TL_WAVE;
      if (d < D) dst[d] = from_f32<T>(d < dim ? out[i] * f : 0.f);
    }
  }
  if (slot < 0) return;
  for (int c = blockIdx.y * kPrepThreads + tid; c < nkv * D; c += gridDim.y * kPrepThreads) {
    const int g = c / D, d = c - g * D;
    float a = 0.f;
    if (d < vdim) {
      const int col = v_off + g * vdim + d;
      a = row[col] + (bias ? bias[q_size + k_size + g * vdim + d] : 0.f);
    }
    v_cache[(page_row + (int64_t)g * block_size) * D + d] = from_f32<T>(a);
  }
}

// Behind the attention kernel, one wave per (token, head): the head's `vdim` values out of rows of D,
//   o = a0 - lambda * a1      (two maps; one map: o = a0)
//   o <- o / sqrt(mean(o^2) + eps)                (sub_norm)
//   o <- o * scale * gate,  gate = 1, sigmoid(g[t, head]) (gate_kind 1) or sigmoid(g[t, head * vdim + j]) (2)
// written side by side as z[t, head * vdim + j]; columns heads * vdim .. heads * vdim + tail - 1 of z become
// 1, 0, 0, ...: the one meets a bias stored as one more column of the output product's weight.
template <typename TA, typename T>
__global__ __launch_bounds__(TL_WAVE) void attn_finish_kernel(const TA* __restrict__ a0, const TA* __restrict__ a1,
                                                              int64_t a_stride, const float* __restrict__ g,
                                                              int64_t g_stride, T* __restrict__ z, int64_t z_stride,
                                                              int heads, int vdim, int D, float lambda, int sub_norm,
                                                              float eps, float scale, int gate_kind, int tail) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const TA* s0 = a0 + (int64_t)t * a_stride + (int64_t)h * D;
  const TA* s1 = a1 ? a1 + (int64_t)t * a_stride + (int64_t)h * D : nullptr;
  constexpr int kPer = 4;       // heads of up to 256 values
  float o[kPer];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    const int j = lane + i * TL_WAVE;
    o[i] = 0.f;
    if (j < vdim) {
      o[i] = to_f32(s0[j]);
      if (s1) o[i] -= lambda * to_f32(s1[j]);
      ss += o[i] * o[i];
    }
  }
  float f = scale;
  if (sub_norm) f *= 1.f / sqrtf(wave_sum(ss) / (float)vdim + eps);
  if (gate_kind == 1) f *= 1.f / (1.f + expf(-g[(int64_t)t * g_stride + h]));
  T* dst = z + (int64_t)t * z_stride + (int64_t)h * vdim;
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    const int j = lane + i * TL_WAVE;
    if (j < vdim) {
      float v = o[i] * f;
      if (gate_kind == 2) v *= 1.f / (1.f + expf(-g[(int64_t)t * g_stride + (int64_t)h * vdim + j]));
      dst[j] = from_f32<T>(v);
    }
  }
  if (h == 0 && lane < tail) z[(int64_t)t * z_stride + (int64_t)heads * vdim + lane] = from_f32<T>(lane == 0 ? 1.f : 0.f);
}

}  // namespace

extern "C" {

// p: float32 [n_tokens, >= (nq + nkv) * hd] (row stride p_stride): query heads, then key heads; with
// values_are_keys == 0 and v_off >= 0 the value heads start at column v_off.  bias: [(nq + nkv) * hd] or null.
// cos_t / sin_t: [positions, rot / 2] (null when rot == 0).  Caches: [blocks, nkv, block_size, hd].
int tl_qk_prepare(const float* p, int64_t p_stride, const float* bias, const int32_t* positions, const float* cos_t,
                  const float* sin_t, const int32_t* slot_mapping, void* q_out, int64_t q_stride, void* k_cache,
                  void* v_cache, int n_tokens, int nq, int nkv, int hd, int rot, int interleaved, int unit_norm, float eps,
                  int values_are_keys, int v_off, int block_size, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  if (nq <= 0 || nkv < 0 || nq + nkv > 65535 || hd <= 0 || hd > 256 || (hd & 1) || rot < 0 || rot > hd || (rot & 1) ||
      block_size <= 0 || !p || !positions || !q_out)
    return TL_ERR_ARG;
  if (rot > 0 && (!cos_t || !sin_t)) return TL_ERR_ARG;
  if (slot_mapping && (!k_cache || !v_cache)) return TL_ERR_ARG;
  if (interleaved != 0 && interleaved != 1) return TL_ERR_ARG;
  dim3 g(n_tokens, nq + nkv), b(TL_WAVE);
  if (dtype == 0)
    hipLaunchKernelGGL(qk_prepare_kernel<float>, g, b, 0, stream, p, p_stride, bias, positions, cos_t, sin_t, slot_mapping,
                       (float*)q_out, q_stride, (float*)k_cache, (float*)v_cache, nq, nkv, hd, rot, interleaved, unit_norm,
                       eps, values_are_keys, v_off, block_size);
  else if (dtype == 1)
    hipLaunchKernelGGL(qk_prepare_kernel<bf16_t>, g, b, 0, stream, p, p_stride, bias, positions, cos_t, sin_t,
                       slot_mapping, (bf16_t*)q_out, q_stride, (bf16_t*)k_cache, (bf16_t*)v_cache, nq, nkv, hd, rot,
                       interleaved, unit_norm, eps, values_are_keys, v_off, block_size);
  else
    return TL_ERR_ARG;
  return tl_launch_status();
}

// a, z: [n_tokens, heads * hd] of the engine's type (z may be a); g: float32, one number per token and head.
int tl_head_gate(const void* a, int64_t a_stride, const float* g, int64_t g_stride, void* z, int64_t z_stride,
                 int n_tokens, int heads, int hd, float scale, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  if (heads <= 0 || hd <= 0 || !a || !g || !z) return TL_ERR_ARG;
  const int64_t total = (int64_t)n_tokens * heads * hd;
  dim3 grid((unsigned)ceil_div64(total, 256)), b(256);
  if (dtype == 0)
    hipLaunchKernelGGL(head_gate_kernel<float>, grid, b, 0, stream, (const float*)a, a_stride, g, g_stride, (float*)z,
                       z_stride, total, heads, hd, scale);
  else if (dtype == 1)
    hipLaunchKernelGGL(head_gate_kernel<bf16_t>, grid, b, 0, stream, (const bf16_t*)a, a_stride, g, g_stride,
                       (bf16_t*)z, z_stride, total, heads, hd, scale);
  else
    return TL_ERR_ARG;
  return tl_launch_status();
}

// p: float32 [n_tokens, p_stride]; bias [q | k | v] and norm_w [q | k] float32 or null; cos_t / sin_t [positions,
// rot / 2] (null when rot == 0); q_out: `maps` arrays of [n_tokens, q_stride], q_map_stride elements apart; caches
// [blocks, nkv, block_size, D], k_cache1 for the second map.
int tl_attn_prepare(const float* p, int64_t p_stride, const float* bias, const float* norm_w, const int32_t* positions,
                    const float* cos_t, const float* sin_t, const int32_t* slot_mapping, void* q_out, int64_t q_stride,
                    int64_t q_map_stride, void* k_cache0, void* k_cache1, void* v_cache, int n_tokens, int heads, int nkv,
                    int maps, int dim, int vdim, int D, int v_off, int rot, int interleaved, int whole_norm, int unit_norm,
                    float eps, float temp_coef, int temp_every, int block_size, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  if (heads <= 0 || nkv <= 0 || maps < 1 || maps > 2 || dim <= 0 || vdim <= 0 || D < dim || D < vdim ||
      D > kPrepPerLane * TL_WAVE || rot < 0 || rot > dim || (rot & 1) || block_size <= 0 || !p || !positions || !q_out ||
      v_off < (heads + nkv) * maps * dim || temp_every < 0)
    return TL_ERR_ARG;
  if (rot > 0 && (!cos_t || !sin_t)) return TL_ERR_ARG;
  if (whole_norm && !norm_w) return TL_ERR_ARG;
  if (slot_mapping && (!k_cache0 || !v_cache || (maps == 2 && !k_cache1))) return TL_ERR_ARG;
  if (interleaved != 0 && interleaved != 1) return TL_ERR_ARG;
  // about 256 workgroups in all where the units allow it, a wave with at least one unit
  const int units = (heads + nkv) * maps, most = (units + kPrepWaves - 1) / kPrepWaves;
  const int share = n_tokens >= 256 ? 1 : (256 / n_tokens < most ? 256 / n_tokens : most);
  dim3 g(n_tokens, share), b(kPrepThreads);
  if (dtype == 0)
    hipLaunchKernelGGL(attn_prepare_kernel<float>, g, b, 0, stream, p, p_stride, bias, norm_w, positions, cos_t, sin_t,
                       slot_mapping, (float*)q_out, q_stride, q_map_stride, (float*)k_cache0, (float*)k_cache1,
                       (float*)v_cache, heads, nkv, maps, dim, vdim, D, v_off, rot, interleaved, whole_norm, unit_norm, eps,
                       temp_coef, temp_every, block_size);
  else if (dtype == 1)
    hipLaunchKernelGGL(attn_prepare_kernel<bf16_t>, g, b, 0, stream, p, p_stride, bias, norm_w, positions, cos_t, sin_t,
                       slot_mapping, (bf16_t*)q_out, q_stride, q_map_stride, (bf16_t*)k_cache0, (bf16_t*)k_cache1,
                       (bf16_t*)v_cache, heads, nkv, maps, dim, vdim, D, v_off, rot, interleaved, whole_norm, unit_norm,
                       eps, temp_coef, temp_every, block_size);
  else
    return TL_ERR_ARG;
  return tl_launch_status();
}

// a0, a1 (a1 null for one map): [n_tokens, heads * D] in a_dtype (float32, or z's type), rows a_stride apart; g:
// float32 gates or null; z: [n_tokens, >= heads * vdim + tail] in dtype, rows z_stride apart.
int tl_attn_finish(const void* a0, const void* a1, int64_t a_stride, const float* g, int64_t g_stride, void* z,
                   int64_t z_stride, int n_tokens, int heads, int vdim, int D, float lambda, int sub_norm, float eps,
                   float scale, int gate_kind, int tail, int a_dtype, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  if (heads <= 0 || heads > 65535 || vdim <= 0 || D < vdim || vdim > 4 * TL_WAVE || !a0 || !z || gate_kind < 0 ||
      gate_kind > 2 || (gate_kind && !g) || tail < 0 || tail > TL_WAVE)
    return TL_ERR_ARG;
  dim3 grid(n_tokens, heads), b(TL_WAVE);
#define TL_FINISH(TA, TZ)                                                                                             \
  hipLaunchKernelGGL((attn_finish_kernel<TA, TZ>), grid, b, 0, stream, (const TA*)a0, (const TA*)a1, a_stride, g,       \
                     g_stride, (TZ*)z, z_stride, heads, vdim, D, lambda, sub_norm, eps, scale, gate_kind, tail)
  if (a_dtype == 0 && dtype == 0) TL_FINISH(float, float);
  else if (a_dtype == 0 && dtype == 1) TL_FINISH(float, bf16_t);
  else if (a_dtype == 1 && dtype == 1) TL_FINISH(bf16_t, bf16_t);
  else return TL_ERR_ARG;
#undef TL_FINISH
  return tl_launch_status();
}

}  // extern "C"
