// Attention over a cache of latent vectors: per token the cache holds one normed latent c
// [kv_rank] and one rotated key part kr [rot] that all heads share.  A head's unrotated key is
// W_uk c and its value W_uv c; neither is ever formed.  With q' = W_uk^T q_unrotated the score is
// (q' . c + q_rot . kr) * scale, and the head's output is W_uv (sum_j p_j c_j): the kernel works on
// [q' | q_rot] against [c | kr] and returns sum_j p_j c_j; the two small products per head run
// outside.  Scores, softmax and the weighted sum are float32 whatever the cache's element type.
#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / TL_WAVE;
constexpr int kMaxRank = 512;                 // latent size the attention kernel takes
constexpr int kRPL = kMaxRank / TL_WAVE;      // latent dims per lane
constexpr int kMaxQ = 1024;                   // kv_rank + rot

// One workgroup per token.  Row t of `d` holds the down projections side by side:
// [q latent (q_rank) at q_off | kv latent (kv_rank) then the shared key part (rot) at kv_off].
// cq[t] = w_q * rms_unit(q latent); if the layer keeps a cache of its own (kv_rank > 0):
// latent[slot] = w_kv * rms_unit(kv latent), rope[slot] = the key part rotated by the angle
// table's row positions[t] (its first `rdims` dims; pair i is (i, i + rdims/2), or (2i, 2i + 1) when
// `interleaved`).  A negative slot stores nothing.  q_rank == 0: there is no query latent.
template <typename T>
__global__ void latent_prepare_kernel(const T* __restrict__ d, int64_t d_stride, int q_off, int q_rank, int kv_off,
                                      int kv_rank, int rot, int rdims, const float* __restrict__ w_q,
                                      const float* __restrict__ w_kv, float eps, const int32_t* __restrict__ positions,
                                      const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                      const int32_t* __restrict__ slot_mapping, T* __restrict__ cq,
                                      T* __restrict__ latent, T* __restrict__ rope, int interleaved) {
  __shared__ float red[kWaves];
  const int t = blockIdx.x;
  const T* row = d + (int64_t)t * d_stride;
  float ss = 0.f, r = 0.f;
  if (q_rank > 0) {
    for (int j = threadIdx.x; j < q_rank; j += kThreads) {
      const float v = to_f32(row[q_off + j]);
      ss += v * v;
    }
    ss = block_sum<kWaves>(ss, red);
    r = 1.f / sqrtf(ss / (float)q_rank + eps);
    for (int j = threadIdx.x; j < q_rank; j += kThreads)
      cq[(int64_t)t * q_rank + j] = from_f32<T>(to_f32(row[q_off + j]) * r * w_q[j]);
  }
  if (kv_rank <= 0) return;
  const int slot = slot_mapping[t];
  ss = 0.f;
  for (int j = threadIdx.x; j < kv_rank; j += kThreads) {
    const float v = to_f32(row[kv_off + j]);
    ss += v * v;
  }
  ss = block_sum<kWaves>(ss, red);
  if (slot < 0) return;
  r = 1.f / sqrtf(ss / (float)kv_rank + eps);
  for (int j = threadIdx.x; j < kv_rank; j += kThreads)
    latent[(int64_t)slot * kv_rank + j] = from_f32<T>(to_f32(row[kv_off + j]) * r * w_kv[j]);
  const int half = rdims / 2;
  const int pos = positions[t];
  for (int i = threadIdx.x; i < half; i += kThreads) {
    const float c = cos_t[(int64_t)pos * half + i], s = sin_t[(int64_t)pos * half + i];
    const int a = interleaved ? 2 * i : i, b = interleaved ? 2 * i + 1 : half + i;
    const float u = to_f32(row[kv_off + kv_rank + a]), v = to_f32(row[kv_off + kv_rank + b]);
    rope[(int64_t)slot * rot + a] = from_f32<T>(u * c - v * s);
    rope[(int64_t)slot * rot + b] = from_f32<T>(v * c + u * s);
  }
  for (int i = rdims + threadIdx.x; i < rot; i += kThreads)       // dims beyond the rotated ones pass unchanged
    rope[(int64_t)slot * rot + i] = row[kv_off + kv_rank + i];
}

// out[t, h, out_off + i] (float32) = the `rot` dims at in_off of head h of row t, the first `rdims`
// of them rotated by the angle table's row positions[t] (pair i is (i, i + rdims/2), or (2i, 2i + 1) when
// `interleaved`).
template <typename T>
__global__ void rotate_into_kernel(const T* __restrict__ q, int64_t q_stride, int head_width, int in_off, int rot,
                                   int rdims, int heads, const int32_t* __restrict__ positions, const float* __restrict__ cos_t,
                                   const float* __restrict__ sin_t, float* __restrict__ out, int out_width,
                                   int out_off, int interleaved) {
  const int t = blockIdx.x;
  const int half = rdims / 2, rest = rot - rdims, per_head = half + rest;
  const int pos = positions[t];
  for (int e = threadIdx.x; e < heads * per_head; e += kThreads) {
    const int h = e / per_head, i = e - h * per_head;
    const T* src = q + (int64_t)t * q_stride + (int64_t)h * head_width + in_off;
    float* dst = out + ((int64_t)t * heads + h) * out_width + out_off;
    if (i >= half) {
      dst[rdims + i - half] = to_f32(src[rdims + i - half]);
      continue;
    }
    const float c = cos_t[(int64_t)pos * half + i], s = sin_t[(int64_t)pos * half + i];
    const int a = interleaved ? 2 * i : i, b = interleaved ? 2 * i + 1 : half + i;
    const float u = to_f32(src[a]), v = to_f32(src[b]);
    dst[a] = u * c - v * s;
    dst[b] = v * c + u * s;
  }
}

// One wave64 per (token, head).  Lanes split the keys of a 64-key tile for the scores and the
// latent's dims for the weighted sum.  The result is multiplied by sigmoid(gate[t, h]) (optional).
// window > 0: position i sees j with 0 <= i - j < window.  sinks (optional): one number per head whose
// exponential joins the softmax's denominator (it has no key and no value and is not scaled).
template <typename T>
__global__ __launch_bounds__(TL_WAVE) void latent_attention_kernel(
    const float* __restrict__ qa, const T* __restrict__ latent, const T* __restrict__ rope,
    const int32_t* __restrict__ block_tables, int max_blocks, const int32_t* __restrict__ req_of_token,
    const int32_t* __restrict__ positions, const T* __restrict__ gate, int64_t gate_stride, T* __restrict__ out,
    int heads, int kv_rank, int rot, int block_size, float scale, int window, const float* __restrict__ sinks) {
  __shared__ float qs[kMaxQ];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int r = req_of_token[t];
  const int kv_end = positions[t] + 1;
  const int kv_begin = window > 0 ? max(0, kv_end - window) : 0;
  const int32_t* bt = block_tables + (int64_t)r * max_blocks;
  const int width = kv_rank + rot;
  const float* qrow = qa + ((int64_t)t * heads + h) * width;
  for (int dd = lane; dd < width; dd += TL_WAVE) qs[dd] = qrow[dd];
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float o[kRPL];
#pragma unroll
  for (int i = 0; i < kRPL; ++i) o[i] = 0.f;

  for (int base = kv_begin; base < kv_end; base += TL_WAVE) {
    const int j = base + lane;
    const bool valid = j < kv_end;
    float s = -INFINITY;
    int slot = 0;
    if (valid) {
      slot = bt[j / block_size] * block_size + (j % block_size);
      const T* cp = latent + (int64_t)slot * kv_rank;
      const T* kp = rope + (int64_t)slot * rot;
      float dot = 0.f;
      for (int dd = 0; dd < kv_rank; ++dd) dot = fmaf(qs[dd], to_f32(cp[dd]), dot);
      for (int dd = 0; dd < rot; ++dd) dot = fmaf(qs[kv_rank + dd], to_f32(kp[dd]), dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));      // lane 0 of every tile is valid: m_new is finite
    const float p = valid ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);
    l = l * alpha + wave_sum(p);
#pragma unroll
    for (int i = 0; i < kRPL; ++i) o[i] *= alpha;
    const int n_keys = min(TL_WAVE, kv_end - base);
    for (int jj = 0; jj < n_keys; ++jj) {
      const float pj = __shfl(p, jj, TL_WAVE);
      const T* cp = latent + (int64_t)__shfl(slot, jj, TL_WAVE) * kv_rank;
#pragma unroll
      for (int i = 0; i < kRPL; ++i) {
        const int dd = lane + i * TL_WAVE;
        if (dd < kv_rank) o[i] = fmaf(pj, to_f32(cp[dd]), o[i]);
      }
    }
    m = m_new;
  }
  float f = 1.f / l;
  if (sinks) {                                        // the sink may lie above every score
    const float sk = sinks[h], m_fin = fmaxf(m, sk), a = expf(m - m_fin);
    f = a / (l * a + expf(sk - m_fin));
  }
  if (gate) f /= 1.f + expf(-to_f32(gate[(int64_t)t * gate_stride + h]));
  T* orow = out + ((int64_t)t * heads + h) * kv_rank;
#pragma unroll
  for (int i = 0; i < kRPL; ++i) {
    const int dd = lane + i * TL_WAVE;
    if (dd < kv_rank) orow[dd] = from_f32<T>(o[i] * f);
  }
}

// ===================================================================== bfloat16 on MFMA
// latent_flash_bf16_kernel: the same function on the matrix cores.  A workgroup of four waves owns a
// tile of 16 query rows of ONE request: `tpt` consecutive tokens times up to 16 heads (row = token *
// hg + head, hg = min(heads, 16)); every head scores against the same cached rows [c | kr], so 16 heads
// of one token fill a matrix tile.  The waves deal the request's 16-key tiles out between them (and
// `n_splits` workgroups split them further: decoding with few requests), each with its own running
// (max, sum, output), merged at the end.  Scores are computed transposed, S^T = [C | Kr] Q^T with
// v_mfma_f32_16x16x32_bf16 (keys straight from memory into operands), so that a lane holds four scores
// of ONE query row and the softmax needs two exchanges; the probabilities are then already the operand
// of O^T = C^T P^T (v_mfma_f32_16x16x16_bf16), whose other operand comes from the wave's own LDS copy
// of the key tile's latents through the transposing read.  The queries [W_uk^T q | q_rot] enter the score
// product as a sum of two bfloat16 terms (staged once per tile), so nothing of their float32 value is
// lost against float32 scores over bfloat16 keys; scores, softmax and sums are float32.
constexpr int LF_WAVES = 4;
constexpr int LF_MAXKS = 18;        // (512 + 64) / 32 steps of the score product
constexpr int LF_MAXDT = 32;        // 512 / 16 tiles of the output
constexpr int LF_PAD = 8;           // elements added to an LDS row (rows 16 bytes apart in the banks)
constexpr float kNegBig = -1.0e30f; // "no key yet": finite, so exp2(m - m') never sees inf - inf
typedef short lf_i16x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ bf16x4 lf_read_transposed(const bf16_t* p) {
  return __builtin_bit_cast(bf16x4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) lf_i16x4*)p));
}
// The factor of an unnormalised output whose running maximum is m (in units of log2 e) and whose sum is l,
// when exp(sink) joins the denominator: 1 / (l + 2^(sink log2 e - m)), formed so that a sink far above every
// score overflows nothing.
__device__ __forceinline__ float with_sink(float m, float l, float sink) {
  const float sk = sink * 1.44269504088896f, m_fin = fmaxf(m, sk);
  const float a = __builtin_amdgcn_exp2f(m - m_fin);
  return a / (l * a + __builtin_amdgcn_exp2f(sk - m_fin));
}
__device__ __forceinline__ void lf_wave_sync() {      // a wave's LDS operations are carried out in order
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__global__ __launch_bounds__(LF_WAVES * TL_WAVE) void latent_flash_bf16_kernel(
    const float* __restrict__ qa, const bf16_t* __restrict__ latent, const bf16_t* __restrict__ rope,
    const int32_t* __restrict__ block_tables, int max_blocks, const int32_t* __restrict__ tile_req,
    const int32_t* __restrict__ tile_tok0, const int32_t* __restrict__ tile_ntok,
    const int32_t* __restrict__ positions, const bf16_t* __restrict__ gate, int64_t gate_stride,
    bf16_t* __restrict__ out, float* __restrict__ part, int n_tokens, int heads, int tpt, int kv_rank, int rot,
    int block_size, float scale, int n_splits, int window, const float* __restrict__ sinks) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lf_smem[];
  const int wave = threadIdx.x / TL_WAVE, lane = threadIdx.x % TL_WAVE, g = lane / 16, c = lane % 16;
  const int tile = blockIdx.x, head0 = blockIdx.y * 16, split = blockIdx.z;
  const int hg = min(heads, 16);
  const int r = tile_req ? tile_req[tile] : tile;
  const int tok0 = tile_tok0 ? tile_tok0[tile] : tile;
  const int ntok = tile_ntok ? tile_ntok[tile] : 1;
  if (ntok <= 0) return;                              // a padding tile
  const int W = kv_rank + rot, WP = (W + 31) / 32 * 32, KS = WP / 32, KDT = kv_rank / 16;
  const int QS = WP + LF_PAD, VS = kv_rank + LF_PAD;
  bf16_t* Ql = (bf16_t*)lf_smem;                     // the queries' upper terms, then their lower terms
  bf16_t* Qlo = Ql + 16 * QS;
  bf16_t* Vl = Qlo + 16 * QS + wave * 16 * VS;
  const int32_t* bt = block_tables + (int64_t)r * max_blocks;

  // the query tile as q = hi + lo in bfloat16; rows without a query and dims beyond W are zero.  Sixteen
  // threads a row, four consecutive floats at a time, everything requested before anything is used.
  {
    const int qrow = threadIdx.x / 16, seg = threadIdx.x % 16;
    const int tt = qrow / hg, hh = head0 + qrow % hg;
    const bool has = tt < ntok && tt < tpt && hh < heads;
    const float* qsrc = qa + ((int64_t)(tok0 + min(tt, ntok - 1)) * heads + min(hh, heads - 1)) * W;
    constexpr int NQ = LF_MAXKS / 2;                  // 64 floats a step of the sixteen threads
    f32x4 qv[NQ];
#pragma unroll
    for (int j = 0; j < NQ; ++j) {
      const int d = seg * 4 + 64 * j;
      qv[j] = (has && d < W) ? *(const f32x4*)(qsrc + d) : f32x4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int j = 0; j < NQ; ++j) {
      const int d = seg * 4 + 64 * j;
      if (d < WP) {
        bf16x4 hi, lo;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          hi[i] = (bf16_t)qv[j][i];
          lo[i] = (bf16_t)(qv[j][i] - (float)hi[i]);
        }
        *(bf16x4*)(Ql + qrow * QS + d) = hi;
        *(bf16x4*)(Qlo + qrow * QS + d) = lo;
      }
    }
  }
  const int my_tt = c / hg, my_h = head0 + c % hg;
  const bool row_valid = my_tt < ntok && my_tt < tpt && my_h < heads;
  const int my_tok = tok0 + min(my_tt, ntok - 1);
  const int pos = positions[my_tok];
  const int kv_end = positions[tok0 + ntok - 1] + 1;  // what the tile's last token sees
  const int n_kt = (kv_end + 15) / 16;
  // the first key tile that the tile's first token still sees through its window
  const int kv_first = window > 0 ? max(0, positions[tok0] - window + 1) : 0;
  const int kt0 = kv_first / 16;
  const int lowest = window > 0 ? pos - window : -1;  // keys at or before this position are hidden from this row
  const float c_log2 = scale * 1.44269504088896f;
  __syncthreads();

  bf16x8 kop[LF_MAXKS];
  auto fetch = [&](int kt) {
    // keys beyond the end, and keys that every window of the tile has left (their pages may have been given
    // back), read a row that exists: they are masked, but what they hold would still enter the products
    const int j = max(min(kt * 16 + c, kv_end - 1), kv_first);
    const int64_t slot = (int64_t)bt[j / block_size] * block_size + (j % block_size);
#pragma unroll
    for (int ks = 0; ks < LF_MAXKS; ++ks) {
      if (ks < KS) {
        const int d0 = ks * 32 + g * 8;
        if (d0 < kv_rank) kop[ks] = *(const bf16x8*)(latent + slot * kv_rank + d0);
        else if (d0 - kv_rank < rot) kop[ks] = *(const bf16x8*)(rope + slot * rot + (d0 - kv_rank));
        else kop[ks] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
      }
    }
  };
  float m_run = kNegBig, l_run = 0.f;
  f32x4 o[LF_MAXDT];
#pragma unroll
  for (int dt = 0; dt < LF_MAXDT; ++dt) o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int first = kt0 + split * LF_WAVES + wave, stride = n_splits * LF_WAVES;
  if (first < n_kt) fetch(first);
  for (int kt = first; kt < n_kt; kt += stride) {
    // the tile's latents into this wave's LDS area (row c, the chunk this lane holds), and the scores
    f32x4 sc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < LF_MAXKS; ++ks) {
      if (ks < KS) {
        const int d0 = ks * 32 + g * 8;
        if (d0 < kv_rank) *(bf16x8*)(Vl + c * VS + d0) = kop[ks];
        const bf16x8 qf = *(const bf16x8*)(Ql + c * QS + d0), ql = *(const bf16x8*)(Qlo + c * QS + d0);
        sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop[ks], qf, sc, 0, 0, 0);
        sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop[ks], ql, sc, 0, 0, 0);
      }
    }
    if (kt + stride < n_kt) fetch(kt + stride);       // on its way while this tile is worked on
    lf_wave_sync();
    // sc[i] = S^T[key kt*16 + g*4 + i][row c]
    float m_tile = kNegBig;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int j = kt * 16 + g * 4 + i;
      const bool ok = row_valid && j <= pos && j > lowest;
      sc[i] = ok ? sc[i] * c_log2 : -INFINITY;
      m_tile = fmaxf(m_tile, sc[i]);
    }
    m_tile = max_over_rows(m_tile);
    const float m_new = fmaxf(m_run, m_tile);
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    float psum = 0.f;
    bf16x4 pb;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float p = __builtin_amdgcn_exp2f(sc[i] - m_new);
      psum += p;
      pb[i] = (bf16_t)p;
    }
    psum = sum_over_rows(psum);
    l_run = l_run * alpha + psum;
    m_run = m_new;
    // lane s of a group names keys g*4 + s/4, dims dt*16 + 4*(s%4) ..; it receives keys g*4 .. g*4+3 of dim dt*16 + s
    const bf16_t* vsrc = Vl + (g * 4 + c / 4) * VS + 4 * (c % 4);
#pragma unroll
    for (int dt = 0; dt < LF_MAXDT; ++dt) {
      if (dt < KDT) {
        const bf16x4 vf = lf_read_transposed(vsrc + dt * 16);
#pragma unroll
        for (int i = 0; i < 4; ++i) o[dt][i] *= alpha;
        o[dt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(lf_i16x4, vf),
                                                          __builtin_bit_cast(lf_i16x4, pb), o[dt], 0, 0, 0);
      }
    }
    lf_wave_sync();                                   // the reads are done before the next tile is written
  }
  __syncthreads();                                    // the merge writes over the staging areas

  // merge: waves 1 to 3 leave (O, m, l) in turn, wave 0 adds them to its own; o[dt][i] = O[row c][dt*16 + g*4 + i]
  float* Mg = (float*)(Qlo + 16 * QS);
  const int MROW = kv_rank + 2;
  for (int src = 1; src < LF_WAVES; ++src) {
    if (wave == src) {
#pragma unroll
      for (int dt = 0; dt < LF_MAXDT; ++dt)
        if (dt < KDT) *(f32x4*)(Mg + c * MROW + dt * 16 + g * 4) = o[dt];
      if (g == 0) {
        Mg[c * MROW + kv_rank] = m_run;
        Mg[c * MROW + kv_rank + 1] = l_run;
      }
    }
    __syncthreads();
    if (wave == 0) {
      const float m_o = Mg[c * MROW + kv_rank], l_o = Mg[c * MROW + kv_rank + 1];
      const float m_new = fmaxf(m_run, m_o);
      const float a = __builtin_amdgcn_exp2f(m_run - m_new), b = __builtin_amdgcn_exp2f(m_o - m_new);
#pragma unroll
      for (int dt = 0; dt < LF_MAXDT; ++dt)
        if (dt < KDT) {
          const f32x4 other = *(const f32x4*)(Mg + c * MROW + dt * 16 + g * 4);
#pragma unroll
          for (int i = 0; i < 4; ++i) o[dt][i] = o[dt][i] * a + other[i] * b;
        }
      l_run = l_run * a + l_o * b;
      m_run = m_new;
    }
    __syncthreads();
  }
  if (wave != 0 || !row_valid) return;
  if (n_splits > 1) {                                 // unnormalised, for latent_combine_kernel (which adds the sink)
    float* prow = part + (((int64_t)split * n_tokens + my_tok) * heads + my_h) * MROW;
#pragma unroll
    for (int dt = 0; dt < LF_MAXDT; ++dt)
      if (dt < KDT) *(f32x4*)(prow + dt * 16 + g * 4) = o[dt];
    if (g == 0) {
      prow[kv_rank] = m_run;
      prow[kv_rank + 1] = l_run;
    }
    return;
  }
  float f = l_run > 0.f ? 1.f / l_run : 0.f;
  if (sinks) f = with_sink(m_run, l_run, sinks[my_h]);
  if (gate) f /= 1.f + expf(-(float)gate[(int64_t)my_tok * gate_stride + my_h]);
  bf16_t* orow = out + ((int64_t)my_tok * heads + my_h) * kv_rank + g * 4;
#pragma unroll
  for (int dt = 0; dt < LF_MAXDT; ++dt)
    if (dt < KDT) {
      bf16x4 v4;
#pragma unroll
      for (int i = 0; i < 4; ++i) v4[i] = (bf16_t)(o[dt][i] * f);
      *(bf16x4*)(orow + dt * 16) = v4;
    }
}

// latent_prefill_bf16_kernel: the same function for steps with many query rows.  A workgroup owns up to
// 4 * tpt consecutive tokens of one request, a wave the 16 rows of `tpt` of them (16 heads of one token, or
// 16 / heads tokens), and ALL its waves walk the same tiles of 32 keys: a tile [c | kr] is fetched once by the
// whole workgroup as whole rows, staged in LDS (two buffers, one barrier a tile) and serves four times the
// query rows; the score product reads its key operands from there, the value product reads the same rows
// through the transposing read.  The queries are two bfloat16 terms, the upper in registers, the lower in
// LDS.  A wave keeps its own (max, sum, output): nothing is merged.
constexpr int LP_KEYS = 32;         // keys a staged tile holds (two 16-key tiles of the products)
constexpr int LP_NPF = 9;           // 16-byte pieces of a staged tile a thread fetches: 32 * 72 / 256
__global__ __launch_bounds__(LF_WAVES * TL_WAVE) void latent_prefill_bf16_kernel(
    const float* __restrict__ qa, const bf16_t* __restrict__ latent, const bf16_t* __restrict__ rope,
    const int32_t* __restrict__ block_tables, int max_blocks, const int32_t* __restrict__ tile_req,
    const int32_t* __restrict__ tile_tok0, const int32_t* __restrict__ tile_ntok,
    const int32_t* __restrict__ positions, const bf16_t* __restrict__ gate, int64_t gate_stride,
    bf16_t* __restrict__ out, int heads, int tpt, int kv_rank, int rot, int block_size, float scale, int window,
    const float* __restrict__ sinks) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lf_smem[];
  const int tid = threadIdx.x, wave = tid / TL_WAVE, lane = tid % TL_WAVE, g = lane / 16, c = lane % 16;
  const int tile = blockIdx.x, head0 = blockIdx.y * 16;
  const int hg = min(heads, 16);
  const int r = tile_req[tile], tok0 = tile_tok0[tile], ntok = tile_ntok[tile];
  if (ntok <= 0) return;                              // a padding tile
  const int W = kv_rank + rot, WP = (W + 31) / 32 * 32, KS = WP / 32, KDT = kv_rank / 16;
  const int KSTR = WP + LF_PAD, CPR = WP / 8;
  bf16_t* Kl = (bf16_t*)lf_smem;                      // two buffers of LP_KEYS rows
  bf16_t* Qlo = Kl + 2 * LP_KEYS * KSTR + wave * 16 * KSTR;     // this wave's queries' lower terms
  const int32_t* bt = block_tables + (int64_t)r * max_blocks;
  const int my_tt = wave * tpt + c / hg, my_h = head0 + c % hg;
  const bool row_valid = c / hg < tpt && my_tt < ntok && my_h < heads;
  const int my_tok = tok0 + min(my_tt, ntok - 1);
  const int pos = positions[my_tok];
  const int kv_end = positions[tok0 + ntok - 1] + 1;  // what the workgroup's last token sees
  const int wave_end = wave * tpt < ntok ? positions[tok0 + min((wave + 1) * tpt, ntok) - 1] + 1 : 0;
  const int n_kt = (kv_end + LP_KEYS - 1) / LP_KEYS;
  // through a window the workgroup's first token sees no key before kv_first, this wave's first token none before
  // wave_first, and this row none at or before `lowest`
  const int kv_first = window > 0 ? max(0, positions[tok0] - window + 1) : 0;
  const int wave_first = window > 0 && wave * tpt < ntok ? max(0, positions[tok0 + wave * tpt] - window + 1) : 0;
  const int lowest = window > 0 ? pos - window : -1;
  const int kt0 = kv_first / LP_KEYS;
  const float c_log2 = scale * 1.44269504088896f;

  // this lane's pieces of its query row, q = hi + lo: the upper terms stay in registers, the lower ones
  // wait in the wave's LDS area (the registers hold the output and the tile on its way)
  bf16x8 qh[LF_MAXKS];
  {
    const float* qsrc = qa + ((int64_t)my_tok * heads + min(my_h, heads - 1)) * W;
#pragma unroll
    for (int ks = 0; ks < LF_MAXKS; ++ks) {
      if (ks < KS) {
        const int d0 = ks * 32 + g * 8;
        const bool has = row_valid && d0 < W;
        const f32x4 a = has ? *(const f32x4*)(qsrc + d0) : f32x4{0.f, 0.f, 0.f, 0.f};
        const f32x4 b = has ? *(const f32x4*)(qsrc + d0 + 4) : f32x4{0.f, 0.f, 0.f, 0.f};
        bf16x8 lo;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float v = e < 4 ? a[e] : b[e - 4];
          qh[ks][e] = (bf16_t)v;
          lo[e] = (bf16_t)(v - (float)qh[ks][e]);
        }
        *(bf16x8*)(Qlo + c * KSTR + d0) = lo;
      }
    }
  }
  // A staged tile is fetched in pieces: piece f is row f / CPR, dims 8 (f % CPR) ...  The pages of a
  // tile are looked up an iteration before its rows are requested, so that a request never begins
  // with a round trip of its own.
  bf16x8 pf[LP_NPF];
  int page[LP_NPF];
  auto lookup = [&](int kt) {
#pragma unroll
    for (int j = 0; j < LP_NPF; ++j) {
      const int f = tid + j * LF_WAVES * TL_WAVE;
      // keys beyond the end, and keys every window has left (their pages may be given back), read a row that exists
      const int key = max(min(kt * LP_KEYS + min(f / CPR, LP_KEYS - 1), kv_end - 1), kv_first);
      page[j] = bt[key / block_size];
    }
  };
  auto fetch = [&](int kt) {
#pragma unroll
    for (int j = 0; j < LP_NPF; ++j) {
      const int f = tid + j * LF_WAVES * TL_WAVE;
      if (f < LP_KEYS * CPR) {
        const int row = f / CPR, d0 = (f - row * CPR) * 8;
        const int key = max(min(kt * LP_KEYS + row, kv_end - 1), kv_first);
        const int64_t slot = (int64_t)page[j] * block_size + (key % block_size);
        if (d0 < kv_rank) pf[j] = *(const bf16x8*)(latent + slot * kv_rank + d0);
        else if (d0 - kv_rank < rot) pf[j] = *(const bf16x8*)(rope + slot * rot + (d0 - kv_rank));
        else pf[j] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
      }
    }
  };
  auto stage = [&](bf16_t* buf) {
#pragma unroll
    for (int j = 0; j < LP_NPF; ++j) {
      const int f = tid + j * LF_WAVES * TL_WAVE;
      if (f < LP_KEYS * CPR) {
        const int row = f / CPR, d0 = (f - row * CPR) * 8;
        *(bf16x8*)(buf + row * KSTR + d0) = pf[j];
      }
    }
  };
  float m_run = kNegBig, l_run = 0.f;
  f32x4 o[LF_MAXDT];
#pragma unroll
  for (int dt = 0; dt < LF_MAXDT; ++dt) o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

  lookup(kt0);
  fetch(kt0);
  if (n_kt > kt0 + 1) lookup(kt0 + 1);
  stage(Kl + (kt0 & 1) * LP_KEYS * KSTR);
  __syncthreads();
  for (int kt = kt0; kt < n_kt; ++kt) {
    const bf16_t* cur = Kl + (kt & 1) * LP_KEYS * KSTR;
    if (kt + 1 < n_kt) {
      fetch(kt + 1);                                  // on its way while this tile is worked on
      if (kt + 2 < n_kt) lookup(kt + 2);
    }
#pragma unroll
    for (int half = 0; half < LP_KEYS / 16; ++half) {
      const int j0 = kt * LP_KEYS + half * 16;
      if (j0 >= wave_end || j0 + 16 <= wave_first) continue;      // no key of these sixteen is seen by this wave's tokens
      const bf16_t* rows = cur + half * 16 * KSTR;
      f32x4 sc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < LF_MAXKS; ++ks) {
        if (ks < KS) {
          const bf16x8 kop = *(const bf16x8*)(rows + c * KSTR + ks * 32 + g * 8);
          const bf16x8 ql = *(const bf16x8*)(Qlo + c * KSTR + ks * 32 + g * 8);
          sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop, qh[ks], sc, 0, 0, 0);
          sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop, ql, sc, 0, 0, 0);
        }
      }
      float m_tile = kNegBig;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int j = j0 + g * 4 + i;
        const bool ok = row_valid && j <= pos && j > lowest;
        sc[i] = ok ? sc[i] * c_log2 : -INFINITY;
        m_tile = fmaxf(m_tile, sc[i]);
      }
      m_tile = max_over_rows(m_tile);
      const float m_new = fmaxf(m_run, m_tile);
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
      float psum = 0.f;
      bf16x4 pb;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = __builtin_amdgcn_exp2f(sc[i] - m_new);
        psum += p;
        pb[i] = (bf16_t)p;
      }
      psum = sum_over_rows(psum);
      l_run = l_run * alpha + psum;
      m_run = m_new;
      const bf16_t* vsrc = rows + (g * 4 + c / 4) * KSTR + 4 * (c % 4);
#pragma unroll
      for (int dt = 0; dt < LF_MAXDT; ++dt) {
        if (dt < KDT) {
          const bf16x4 vf = lf_read_transposed(vsrc + dt * 16);
#pragma unroll
          for (int i = 0; i < 4; ++i) o[dt][i] *= alpha;
          o[dt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(lf_i16x4, vf),
                                                            __builtin_bit_cast(lf_i16x4, pb), o[dt], 0, 0, 0);
        }
      }
    }
    // the other buffer was last read before the barrier of the tile before: it may be written now
    if (kt + 1 < n_kt) stage(Kl + ((kt + 1) & 1) * LP_KEYS * KSTR);
    __syncthreads();
  }
  if (!row_valid) return;
  float f = l_run > 0.f ? 1.f / l_run : 0.f;
  if (sinks) f = with_sink(m_run, l_run, sinks[my_h]);
  if (gate) f /= 1.f + expf(-(float)gate[(int64_t)my_tok * gate_stride + my_h]);
  bf16_t* orow = out + ((int64_t)my_tok * heads + my_h) * kv_rank + g * 4;
#pragma unroll
  for (int dt = 0; dt < LF_MAXDT; ++dt)
    if (dt < KDT) {
      bf16x4 v4;
#pragma unroll
      for (int i = 0; i < 4; ++i) v4[i] = (bf16_t)(o[dt][i] * f);
      *(bf16x4*)(orow + dt * 16) = v4;
    }
}

// Merges the partial results of `n_splits` (<= 64) workgroups: one wave per (token, head).  Lane s
// fetches split s's maximum and sum, the weights 2^(m_s - M) are formed once, and the output dims are
// then summed over the splits with every load independent of the others.  Maxima are in units of
// log2 e; a split without keys has l = 0.
__global__ __launch_bounds__(TL_WAVE) void latent_combine_kernel(const float* __restrict__ part,
                                                                 const bf16_t* __restrict__ gate, int64_t gate_stride,
                                                                 bf16_t* __restrict__ out, int n_tokens, int heads,
                                                                 int kv_rank, int n_splits,
                                                                 const float* __restrict__ sinks) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int MROW = kv_rank + 2;
  const int64_t row = (int64_t)t * heads + h, step = (int64_t)n_tokens * heads;
  const bool mine = lane < n_splits;
  const float m = mine ? part[(row + lane * step) * MROW + kv_rank] : kNegBig;
  const float l = mine ? part[(row + lane * step) * MROW + kv_rank + 1] : 0.f;
  const float M = wave_max(m);
  const float wgt = mine ? __builtin_amdgcn_exp2f(m - M) : 0.f;
  const float L = wave_sum(wgt * l);
  float f = L > 0.f ? 1.f / L : 0.f;
  if (sinks) f = with_sink(M, L, sinks[h]);
  if (gate) f /= 1.f + expf(-(float)gate[(int64_t)t * gate_stride + h]);
  float acc[kRPL];
#pragma unroll
  for (int i = 0; i < kRPL; ++i) acc[i] = 0.f;
  for (int s0 = 0; s0 < n_splits; s0 += 4) {         // four splits requested at a time
    float v[4][kRPL], ws[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int s = min(s0 + u, n_splits - 1);
      ws[u] = s0 + u < n_splits ? __shfl(wgt, s, TL_WAVE) : 0.f;
      const float* src = part + (row + s * step) * MROW;
#pragma unroll
      for (int i = 0; i < kRPL; ++i) {
        const int d = lane + i * TL_WAVE;
        v[u][i] = d < kv_rank ? src[d] : 0.f;
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int i = 0; i < kRPL; ++i) acc[i] = fmaf(ws[u], v[u][i], acc[i]);
  }
#pragma unroll
  for (int i = 0; i < kRPL; ++i) {
    const int d = lane + i * TL_WAVE;
    if (d < kv_rank) out[row * kv_rank + d] = (bf16_t)(acc[i] * f);
  }
}

// Small products per head for steps of few rows: out[t, h, n] = sum_k w[h, k, n] * in[t, h, k].
// The weights lie [heads, inner, cols_padded] (cols_padded a multiple of 8).  A workgroup owns 64 output
// columns of one head for up to kRows rows.  A lane is (k slice, column octet): it fetches eight columns
// of one weight row in one access and takes every 32nd k (eight slices a wave, four waves); the eight
// slices of a wave meet through lane exchanges, the four waves in LDS, both in a fixed order.
constexpr int kRows = 8;
constexpr int kMaxInner = 1024;
constexpr int kHpCols = 64, kHpSlices = 32;
template <typename TW>
__device__ __forceinline__ void load8(const TW* p, float* v) {
  if constexpr (sizeof(TW) == 2) {
    const bf16x8 x = *(const bf16x8*)p;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (float)x[e];
  } else {
    const f32x4 a = *(const f32x4*)p, b2 = *(const f32x4*)(p + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      v[e] = a[e];
      v[4 + e] = b2[e];
    }
  }
}
template <typename TI, typename TW, typename TO>
__global__ __launch_bounds__(kThreads) void head_products_kernel(const TI* __restrict__ in, int64_t in_stride,
                                                                 int in_head_width, const TW* __restrict__ w,
                                                                 TO* __restrict__ out, int64_t out_stride,
                                                                 int out_head_width, int n_rows, int inner, int cols,
                                                                 int cols_padded, const TI* __restrict__ gate,
                                                                 int64_t gate_stride) {
  __shared__ float xs[kRows][kMaxInner];
  __shared__ float part[kWaves][kRows][kHpCols];
  const int h = blockIdx.x, wave = threadIdx.x / TL_WAVE, lane = threadIdx.x % TL_WAVE;
  const int oc = lane % 8, slice = wave * 8 + lane / 8;
  const int col0 = blockIdx.y * kHpCols;
  const int t0 = blockIdx.z * kRows, rows = min(kRows, n_rows - t0);
  {                                   // the rows' inputs: everything requested before anything is stored
    constexpr int NX = kRows * kMaxInner / kThreads;
    float tmp[NX];
#pragma unroll
    for (int j = 0; j < NX; ++j) {
      const int e = threadIdx.x + j * kThreads, r = e / inner, k = e - r * inner;
      tmp[j] = (e < kRows * inner && r < rows) ? to_f32(in[(int64_t)(t0 + r) * in_stride + (int64_t)h * in_head_width + k]) : 0.f;
    }
#pragma unroll
    for (int j = 0; j < NX; ++j) {
      const int e = threadIdx.x + j * kThreads, r = e / inner, k = e - r * inner;
      if (e < kRows * inner) xs[r][k] = tmp[j];
    }
  }
  __syncthreads();
  float acc[kRows][8];
#pragma unroll
  for (int r = 0; r < kRows; ++r)
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[r][e] = 0.f;
  const bool has_cols = col0 + oc * 8 < cols_padded;
  const TW* wp = w + (int64_t)h * inner * cols_padded + min(col0 + oc * 8, cols_padded - 8);
  for (int k0 = slice; k0 < inner; k0 += kHpSlices * 4) {        // four weight rows requested at a time
    float wv[4][8];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int k = k0 + u * kHpSlices;
      load8(wp + (int64_t)min(k, inner - 1) * cols_padded, wv[u]);
      if (k >= inner || !has_cols) {
#pragma unroll
        for (int e = 0; e < 8; ++e) wv[u][e] = 0.f;
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int k = min(k0 + u * kHpSlices, inner - 1);
#pragma unroll
      for (int r = 0; r < kRows; ++r) {
        const float x = xs[r][k];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[r][e] = fmaf(wv[u][e], x, acc[r][e]);
      }
    }
  }
  // the eight slices of the wave: lanes oc, oc + 8, ..., oc + 56
#pragma unroll
  for (int r = 0; r < kRows; ++r)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float v = acc[r][e];
      acc[r][e] = sum_over_rows(v + dpp_f32<TL_DPP_ROR8>(v));
    }
  if (lane < 8) {
#pragma unroll
    for (int r = 0; r < kRows; ++r)
#pragma unroll
      for (int e = 0; e < 8; ++e) part[wave][r][oc * 8 + e] = acc[r][e];
  }
  __syncthreads();
  for (int e = threadIdx.x; e < rows * kHpCols; e += kThreads) {
    const int r = e / kHpCols, c2 = e % kHpCols, n2 = col0 + c2;
    float sum = 0.f;
#pragma unroll
    for (int q = 0; q < kWaves; ++q) sum += part[q][r][c2];
    if (n2 < cols) {
      // a gate per element (optional): its pre-activations lie as the heads' results do, cols a head
      if (gate) sum /= 1.f + expf(-to_f32(gate[(int64_t)(t0 + r) * gate_stride + (int64_t)h * cols + n2]));
      out[(int64_t)(t0 + r) * out_stride + (int64_t)h * out_head_width + n2] = from_f32<TO>(sum);
    }
  }
}

// The same products for steps of many rows, on the matrix cores (bfloat16): out[t, h, n] =
// sum_k w[h, n, k] * in[t, h, k] with the weights [heads, cols, inner] (k contiguous, as the checkpoint
// stores them).  A workgroup of four waves owns 64 columns x 64 rows of one head, a wave 32 x 32 as
// 2 x 2 tiles of v_mfma_f32_16x16x32_bf16; both operands go straight from memory into registers (a
// lane's eight consecutive k of one row).  The product is computed transposed (columns as the
// instruction's rows), so a lane ends with four consecutive output columns of one row.
template <typename TO>
__global__ __launch_bounds__(kThreads) void head_gemm_bf16_kernel(const bf16_t* __restrict__ in, int64_t in_stride,
                                                                  int in_head_width, const bf16_t* __restrict__ w,
                                                                  TO* __restrict__ out, int64_t out_stride,
                                                                  int out_head_width, int n_rows, int inner, int cols,
                                                                  const bf16_t* __restrict__ gate, int64_t gate_stride) {
  const int h = blockIdx.x, wave = threadIdx.x / TL_WAVE, lane = threadIdx.x % TL_WAVE, g = lane / 16, c = lane % 16;
  const int col0 = blockIdx.y * 64 + (wave & 1) * 32, row0 = blockIdx.z * 64 + (wave >> 1) * 32;
  if (col0 >= cols || row0 >= n_rows) return;
  const bf16_t* wp[2];
  const bf16_t* xp[2];
#pragma unroll
  for (int a = 0; a < 2; ++a) {
    wp[a] = w + ((int64_t)h * cols + min(col0 + a * 16 + c, cols - 1)) * inner;
    xp[a] = in + (int64_t)min(row0 + a * 16 + c, n_rows - 1) * in_stride + (int64_t)h * in_head_width;
  }
  f32x4 acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b) acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int k0 = 0; k0 < inner; k0 += 32) {
    const int d0 = k0 + g * 8;
    bf16x8 wa[2], xb[2];
#pragma unroll
    for (int a = 0; a < 2; ++a) {
      wa[a] = d0 < inner ? *(const bf16x8*)(wp[a] + d0) : zero;
      xb[a] = d0 < inner ? *(const bf16x8*)(xp[a] + d0) : zero;
    }
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int b = 0; b < 2; ++b) acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[a], xb[b], acc[a][b], 0, 0, 0);
  }
  // acc[a][b][i] = out[row0 + b*16 + c][col0 + a*16 + g*4 + i]
#pragma unroll
  for (int b = 0; b < 2; ++b) {
    const int row = row0 + b * 16 + c;
    if (row >= n_rows) continue;
#pragma unroll
    for (int a = 0; a < 2; ++a) {
      const int n = col0 + a * 16 + g * 4;
      TO* dst = out + (int64_t)row * out_stride + (int64_t)h * out_head_width + n;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (n + i < cols) {
          float v = acc[a][b][i];
          if (gate) v /= 1.f + expf(-(float)gate[(int64_t)row * gate_stride + (int64_t)h * cols + n + i]);
          dst[i] = from_f32<TO>(v);
        }
    }
  }
}

// z[t, c] = a[t, c] * sigmoid(g[t, c]): a gate per element, its pre-activation in the rows of another tensor.
template <typename T>
__global__ void gate_rows_kernel(const T* __restrict__ a, int64_t a_stride, const T* __restrict__ g, int64_t g_stride,
                                 T* __restrict__ z, int64_t z_stride, int64_t total, int cols) {
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= total) return;
  const int64_t t = i / cols;
  const int c = (int)(i - t * cols);
  const float gv = to_f32(g[t * g_stride + c]);
  z[t * z_stride + c] = from_f32<T>(to_f32(a[t * a_stride + c]) / (1.f + expf(-gv)));
}

}  // namespace

#define TL_DISPATCH_T(dtype, ...)                 \
  if ((dtype) == 0) { using T = float; __VA_ARGS__ } \
  else if ((dtype) == 1) { using T = bf16_t; __VA_ARGS__ } \
  else return TL_ERR_ARG;

extern "C" {

// kv_rank == 0: a layer that keeps no cache of its own (it only needs its query latent).
int tl_latent_prepare(const void* d, int64_t d_stride, int q_off, int q_rank, int kv_off, int kv_rank, int rot,
                      int rdims, const float* w_q, const float* w_kv, float eps, const int32_t* positions, const float* cos_t,
                      const float* sin_t, const int32_t* slot_mapping, void* cq, void* latent, void* rope,
                      int n_tokens, int interleaved, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  if (q_rank < 0 || kv_rank < 0 || q_rank + kv_rank == 0 || rot < 0 || rdims < 0 || rdims % 2 || rdims > rot ||
      (q_rank > 0 && (!w_q || !cq)) || (interleaved != 0 && interleaved != 1))
    return TL_ERR_ARG;
  if (kv_rank > 0 && (!slot_mapping || !latent || (rot > 0 && !rope) || (rdims > 0 && (!cos_t || !sin_t || !positions))))
    return TL_ERR_ARG;
  TL_DISPATCH_T(dtype, hipLaunchKernelGGL(latent_prepare_kernel<T>, dim3(n_tokens), dim3(kThreads), 0, stream,
                                          (const T*)d, d_stride, q_off, q_rank, kv_off, kv_rank, rot, rdims, w_q, w_kv, eps,
                                          positions, cos_t, sin_t, slot_mapping, (T*)cq, (T*)latent, (T*)rope,
                                          interleaved);)
  return tl_launch_status();
}

int tl_rotate_into(const void* q, int64_t q_stride, int head_width, int in_off, int rot, int rdims, int heads,
                   const int32_t* positions, const float* cos_t, const float* sin_t, float* out, int out_width,
                   int out_off, int n_tokens, int interleaved, int dtype, hipStream_t stream) {
  if (n_tokens <= 0 || rot == 0) return TL_OK;
  if (rot < 0 || rdims < 0 || rdims % 2 || rdims > rot || heads <= 0 || in_off + rot > head_width ||
      out_off + rot > out_width || (interleaved != 0 && interleaved != 1))
    return TL_ERR_ARG;
  TL_DISPATCH_T(dtype, hipLaunchKernelGGL(rotate_into_kernel<T>, dim3(n_tokens), dim3(kThreads), 0, stream,
                                          (const T*)q, q_stride, head_width, in_off, rot, rdims, heads, positions, cos_t,
                                          sin_t, out, out_width, out_off, interleaved);)
  return tl_launch_status();
}

int tl_latent_attention(const float* qa, const void* latent, const void* rope, const int32_t* block_tables,
                        int max_blocks, const int32_t* req_of_token, const int32_t* positions, const void* gate,
                        int64_t gate_stride, void* out, int n_tokens, int heads, int kv_rank, int rot,
                        int block_size, float scale, int window, const float* sinks, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  if (heads <= 0 || heads > 65535 || kv_rank <= 0 || kv_rank > kMaxRank || rot < 0 || kv_rank + rot > kMaxQ ||
      block_size <= 0 || max_blocks <= 0 || window < 0)
    return TL_ERR_ARG;
  dim3 g(n_tokens, heads), b(TL_WAVE);
  TL_DISPATCH_T(dtype, hipLaunchKernelGGL(latent_attention_kernel<T>, g, b, 0, stream, qa, (const T*)latent,
                                          (const T*)rope, block_tables, max_blocks, req_of_token, positions,
                                          (const T*)gate, gate_stride, (T*)out, heads, kv_rank, rot, block_size,
                                          scale, window, sinks);)
  return tl_launch_status();
}

// bfloat16 on the matrix cores.  Tiles: `tpt` = 16 / min(heads, 16) tokens of one request each (null
// arrays: tile i is token i of request i).  n_splits > 1: `part` is scratch of
// n_splits * n_tokens * heads * (kv_rank + 2) floats.  kv_rank a multiple of 16 up to 512, rot a multiple of 8 up to 64.
int tl_latent_flash(const float* qa, const void* latent, const void* rope, const int32_t* block_tables, int max_blocks,
                    const int32_t* tile_req, const int32_t* tile_tok0, const int32_t* tile_ntok,
                    const int32_t* positions, const void* gate, int64_t gate_stride, void* out, float* part,
                    int n_tiles, int n_tokens, int heads, int tpt, int kv_rank, int rot, int block_size, float scale,
                    int n_splits, int window, const float* sinks, hipStream_t stream) {
  if (n_tiles <= 0 || n_tokens <= 0) return TL_OK;
  if (window < 0 || heads <= 0 || kv_rank <= 0 || kv_rank % 16 || kv_rank > 16 * LF_MAXDT || rot < 0 || rot % 8 ||
      kv_rank + rot > 32 * LF_MAXKS || block_size <= 0 || max_blocks <= 0 || n_splits < 1 || n_splits > TL_WAVE ||
      tpt != 16 / (heads < 16 ? heads : 16) || (n_splits > 1 && !part) || (heads + 15) / 16 > 65535)
    return TL_ERR_ARG;
  const int WP = (kv_rank + rot + 31) / 32 * 32;
  const size_t lds = (size_t)2 * 16 * (WP + LF_PAD) * 2 + (size_t)LF_WAVES * 16 * (kv_rank + LF_PAD) * 2;
  static int granted = 0;                 // the most dynamic LDS asked for so far (the default limit is 64 KB)
  if ((int)lds > granted) {
    if (hipFuncSetAttribute((const void*)latent_flash_bf16_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds) != hipSuccess)
      return TL_ERR_LAUNCH;
    granted = (int)lds;
  }
  dim3 g(n_tiles, (heads + 15) / 16, n_splits), b(LF_WAVES * TL_WAVE);
  hipLaunchKernelGGL(latent_flash_bf16_kernel, g, b, lds, stream, qa, (const bf16_t*)latent, (const bf16_t*)rope,
                     block_tables, max_blocks, tile_req, tile_tok0, tile_ntok, positions, (const bf16_t*)gate,
                     gate_stride, (bf16_t*)out, part, n_tokens, heads, tpt, kv_rank, rot, block_size, scale, n_splits,
                     window, sinks);
  if (n_splits > 1)
    hipLaunchKernelGGL(latent_combine_kernel, dim3(n_tokens, heads), dim3(TL_WAVE), 0, stream, part,
                       (const bf16_t*)gate, gate_stride, (bf16_t*)out, n_tokens, heads, kv_rank, n_splits, sinks);
  return tl_launch_status();
}

// Steps with many query rows: tiles of up to 4 * tpt tokens of one request each (tile lists required).
int tl_latent_prefill(const float* qa, const void* latent, const void* rope, const int32_t* block_tables,
                      int max_blocks, const int32_t* tile_req, const int32_t* tile_tok0, const int32_t* tile_ntok,
                      const int32_t* positions, const void* gate, int64_t gate_stride, void* out, int n_tiles,
                      int heads, int tpt, int kv_rank, int rot, int block_size, float scale, int window,
                      const float* sinks, hipStream_t stream) {
  if (n_tiles <= 0) return TL_OK;
  if (window < 0 || heads <= 0 || kv_rank <= 0 || kv_rank % 16 || kv_rank > 16 * LF_MAXDT || rot < 0 || rot % 8 ||
      kv_rank + rot > 32 * LF_MAXKS || block_size <= 0 || max_blocks <= 0 || !tile_req || !tile_tok0 || !tile_ntok ||
      tpt != 16 / (heads < 16 ? heads : 16) || (heads + 15) / 16 > 65535)
    return TL_ERR_ARG;
  const int WP = (kv_rank + rot + 31) / 32 * 32;
  // two staged tiles and the four waves' lower query terms: at most 150 KB (the default limit is 64 KB)
  const size_t lds = (size_t)(2 * LP_KEYS + LF_WAVES * 16) * (WP + LF_PAD) * 2;
  static int granted_prefill = 0;
  if ((int)lds > granted_prefill) {
    if (hipFuncSetAttribute((const void*)latent_prefill_bf16_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds) != hipSuccess)
      return TL_ERR_LAUNCH;
    granted_prefill = (int)lds;
  }
  dim3 g(n_tiles, (heads + 15) / 16), b(LF_WAVES * TL_WAVE);
  hipLaunchKernelGGL(latent_prefill_bf16_kernel, g, b, lds, stream, qa, (const bf16_t*)latent, (const bf16_t*)rope,
                     block_tables, max_blocks, tile_req, tile_tok0, tile_ntok, positions, (const bf16_t*)gate,
                     gate_stride, (bf16_t*)out, heads, tpt, kv_rank, rot, block_size, scale, window, sinks);
  return tl_launch_status();
}

// in / out: rows with a stride, head h at column h * head_width.  w [heads, inner, cols_padded] of in's type;
// out float32 (out_dtype 0) or of in's type.  gate (optional, of in's type): rows of heads * cols pre-activations
// with a stride; the result is multiplied by their sigmoid, element by element.
int tl_head_products(const void* in, int64_t in_stride, int in_head_width, const void* w, void* out,
                     int64_t out_stride, int out_head_width, int n_rows, int heads, int inner, int cols,
                     int cols_padded, const void* gate, int64_t gate_stride, int dtype, int out_dtype,
                     hipStream_t stream) {
  if (n_rows <= 0) return TL_OK;
  if (heads <= 0 || inner <= 0 || inner > kMaxInner || cols <= 0 || inner > in_head_width || cols > out_head_width ||
      cols_padded < cols || cols_padded % 8 ||
      (n_rows + kRows - 1) / kRows > 65535 || (cols + kHpCols - 1) / kHpCols > 65535)
    return TL_ERR_ARG;
  dim3 g(heads, (cols + kHpCols - 1) / kHpCols, (n_rows + kRows - 1) / kRows), b(kThreads);
#define TL_HP(TI, TO)                                                                                              \
  hipLaunchKernelGGL((head_products_kernel<TI, TI, TO>), g, b, 0, stream, (const TI*)in, in_stride, in_head_width, \
                     (const TI*)w, (TO*)out, out_stride, out_head_width, n_rows, inner, cols, cols_padded,         \
                     (const TI*)gate, gate_stride)
  if (dtype == 0 && out_dtype == 0) TL_HP(float, float);
  else if (dtype == 1 && out_dtype == 0) TL_HP(bf16_t, float);
  else if (dtype == 1 && out_dtype == 1) TL_HP(bf16_t, bf16_t);
  else return TL_ERR_ARG;
#undef TL_HP
  return tl_launch_status();
}

// bfloat16, many rows: w [heads, cols, inner]; inner a multiple of 8, operands 16-byte aligned.
int tl_head_gemm(const void* in, int64_t in_stride, int in_head_width, const void* w, void* out, int64_t out_stride,
                 int out_head_width, int n_rows, int heads, int inner, int cols, const void* gate, int64_t gate_stride,
                 int out_dtype, hipStream_t stream) {
  if (n_rows <= 0) return TL_OK;
  if (heads <= 0 || inner <= 0 || inner % 8 || cols <= 0 || inner > in_head_width || cols > out_head_width ||
      in_stride % 8 || in_head_width % 8 || (n_rows + 63) / 64 > 65535 || (cols + 63) / 64 > 65535)
    return TL_ERR_ARG;
  dim3 g(heads, (cols + 63) / 64, (n_rows + 63) / 64), b(kThreads);
  if (out_dtype == 0)
    hipLaunchKernelGGL(head_gemm_bf16_kernel<float>, g, b, 0, stream, (const bf16_t*)in, in_stride, in_head_width,
                       (const bf16_t*)w, (float*)out, out_stride, out_head_width, n_rows, inner, cols,
                       (const bf16_t*)gate, gate_stride);
  else if (out_dtype == 1)
    hipLaunchKernelGGL(head_gemm_bf16_kernel<bf16_t>, g, b, 0, stream, (const bf16_t*)in, in_stride, in_head_width,
                       (const bf16_t*)w, (bf16_t*)out, out_stride, out_head_width, n_rows, inner, cols,
                       (const bf16_t*)gate, gate_stride);
  else
    return TL_ERR_ARG;
  return tl_launch_status();
}

// a, g, z: rows of `cols` elements of the engine's type, each with a row stride of its own (z may be a).
int tl_gate_rows(const void* a, int64_t a_stride, const void* g, int64_t g_stride, void* z, int64_t z_stride,
                 int n_rows, int cols, int dtype, hipStream_t stream) {
  if (n_rows <= 0) return TL_OK;
  if (cols <= 0 || a_stride < cols || g_stride < cols || z_stride < cols || !a || !g || !z) return TL_ERR_ARG;
  const int64_t total = (int64_t)n_rows * cols;
  dim3 grid((unsigned)ceil_div64(total, kThreads)), b(kThreads);
  TL_DISPATCH_T(dtype, hipLaunchKernelGGL(gate_rows_kernel<T>, grid, b, 0, stream, (const T*)a, a_stride, (const T*)g,
                                          g_stride, (T*)z, z_stride, total, cols);)
  return tl_launch_status();
}

}  // extern "C"
