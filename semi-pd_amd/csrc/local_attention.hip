// Block-local attention with a sink term, and the step in front of it (gfx950, wave64).
//
//  * unit_norm_kv_store_kernel: per head, q <- q / rms(q) in place, k <- k / rms(k) into the key pool,
//    v <- (1 - a) v + a v0 (optional) into the value pool.  Everything between the projection GEMM and the attention
//    in one launch; sums of squares, the division and the blend in fp32.
//  * local_attention_rows_kernel: one wave per (query row, head) for every element type, any head sizes up to 512 / 512.
//    Keys come from the paged pools through the request's row of req_to_token, so a prompt portion, a whole prompt and
//    a decode step are the same walk: query at position p sees keys lo(p) .. p, lo(p) = floor(p / chunk) * chunk
//    (chunk 0: lo = 0).  score = cap * tanh(scale * q.k / cap) (cap 0: none); the softmax denominator holds one more
//    term exp(sink[head]) that has no value row.  Optional epilogue: out *= sigmoid(gate).
//  * local_attention_mfma_kernel (bf16 / f16, head sizes in steps of 32 / 16): 64 query rows of one request and head
//    per workgroup, S^T = K Q^T and O^T += V^T P^T on v_mfma_f32_16x16x32, P^T taken from the accumulators in place, V^T
//    through transposing reads of a row-major LDS tile, the next step's loads in flight during the current one.
//  * local_attention_decode_kernel (bf16 / f16): one workgroup per (request, kv head); the waves split the visible keys,
//    the q heads of the group are the MFMA's columns, partials meet in LDS.
//
// The same walks serve a second family of masks and weights (semipd_window_attention):
//  * mask: the last `window` positions up to the query, plus the first `keep_first` positions of the sequence, which stay
//    visible at their true positions however far the window has moved on (window 0: the block mask above);
//  * weights: with `sigmoid` set every visible key weighs sigmoid(score + head_bias[head]) on its own -- no maximum, no
//    denominator, no sink -- and the result is the plain weighted sum of the value rows, times out_scale.
//  * bias_rope_vnorm_kv_store_kernel, the step in front of it: projection biases, rotation of neighbouring pairs of q and k
//    by angles position * inv_freq[pair] (fp32 product, sincosf), values scaled to unit RMS; k and v into the pools.
#include "common.h"
#include "mfma_frag.h"

namespace semipd {

// ------------------------------------------------------------------------------------------------ norm + store
template <typename T>
__global__ void __launch_bounds__(256) unit_norm_kv_store_kernel(
    T* __restrict__ qkv, int64_t ld, int64_t num_tokens, int H, int G, int D, int E, int64_t k_off, int64_t v_off, float eps,
    const T* __restrict__ v_first, int64_t v_first_ld, const T* __restrict__ mix, T* __restrict__ k_pool,
    T* __restrict__ v_pool, const int64_t* __restrict__ loc) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int items = H + 2 * G;
  const int64_t item = (int64_t)blockIdx.x * 4 + wave;
  if (item >= num_tokens * items) return;
  const int64_t t = item / items;
  const int h = (int)(item % items);
  T* row = qkv + t * ld;
  if (h < H + G) {
    const bool is_q = h < H;
    T* src = is_q ? row + (int64_t)h * D : row + k_off + (int64_t)(h - H) * D;
    float ss = 0.f;
    for (int d = lane; d < D; d += 64) {
      const float x = Elem<T>::to_f(src[d]);
      ss += x * x;
    }
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(ss / (float)D + eps);
    T* dst = is_q ? src : k_pool + (loc[t] * G + (h - H)) * D;
    for (int d = lane; d < D; d += 64) dst[d] = Elem<T>::from_f(Elem<T>::to_f(src[d]) * r);
  } else {
    const int g = h - H - G;
    const T* src = row + v_off + (int64_t)g * E;
    T* dst = v_pool + (loc[t] * G + g) * E;
    if (v_first != nullptr) {
      const float a = Elem<T>::to_f(mix[0]);
      const T* v0 = v_first + t * v_first_ld + (int64_t)g * E;
      for (int e = lane; e < E; e += 64)
        dst[e] = Elem<T>::from_f((1.0f - a) * Elem<T>::to_f(src[e]) + a * Elem<T>::to_f(v0[e]));
    } else {
      for (int e = lane; e < E; e += 64) dst[e] = src[e];
    }
  }
}

// The same for 16-bit types with 16-byte accesses: a head is taken by L = D / 8 lanes (a power of two), 64 / L heads per wave.
template <typename T, int L>
__global__ void __launch_bounds__(256) unit_norm_kv_store_vec_kernel(
    T* __restrict__ qkv, int64_t ld, int64_t num_tokens, int H, int G, int D, int E, int64_t k_off, int64_t v_off, float eps,
    const T* __restrict__ v_first, int64_t v_first_ld, const T* __restrict__ mix, T* __restrict__ k_pool,
    T* __restrict__ v_pool, const int64_t* __restrict__ loc) {
  constexpr int PER_WAVE = 64 / L;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, sl = lane % L;
  const int items = H + 2 * G;
  const int64_t item = ((int64_t)blockIdx.x * 4 + wave) * PER_WAVE + lane / L;
  const bool on = item < num_tokens * items;
  const int64_t t = on ? item / items : 0;
  const int h = on ? (int)(item % items) : 0;
  T* row = qkv + t * ld;
  if (h < H + G) {               // (lanes of finished items still take part in the shuffles)
    const bool is_q = h < H;
    T* src = (is_q ? row + (int64_t)h * D : row + k_off + (int64_t)(h - H) * D) + sl * 8;
    const Vec16<T> x = load16(src);
    float f[8], ss = 0.f;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      f[u] = Elem<T>::to_f(x.e[u]);
      ss += f[u] * f[u];
    }
#pragma unroll
    for (int o = L / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
    if (!on) return;
    const float r = 1.0f / sqrtf(ss / (float)D + eps);
    Vec16<T> y;
#pragma unroll
    for (int u = 0; u < 8; ++u) y.e[u] = Elem<T>::from_f(f[u] * r);
    store16(is_q ? src : k_pool + (loc[t] * G + (h - H)) * D + sl * 8, y);
  } else {
    if (!on) return;
    const int g = h - H - G;
    const T* src = row + v_off + (int64_t)g * E;
    T* dst = v_pool + (loc[t] * G + g) * E;
    const float a = v_first ? Elem<T>::to_f(mix[0]) : 0.f;
    const T* v0 = v_first ? v_first + t * v_first_ld + (int64_t)g * E : nullptr;
    for (int e = sl * 8; e < E; e += L * 8) {
      Vec16<T> x = load16(src + e);
      if (v0) {
        const Vec16<T> z = load16(v0 + e);
#pragma unroll
        for (int u = 0; u < 8; ++u) x.e[u] = Elem<T>::from_f((1.0f - a) * Elem<T>::to_f(x.e[u]) + a * Elem<T>::to_f(z.e[u]));
      }
      store16(dst + e, x);
    }
  }
}


// ------------------------------------------------------------------------------------------------ bias + rotation + value norm + store
// One wave per (token, head) of q | k | v.  q and k: x + bias, then the first `rot` elements of the head as rot / 2 neighbouring
// pairs (2i, 2i + 1), pair i turned by the angle pos * inv_freq[i] (fp32 product; sincosf reduces the argument itself); the
// rest of the head passes.  q in place, k into the key pool.  v: (x + bias) / sqrt(mean((x + bias)^2) + eps) into the value
// pool.  Everything in fp32, one rounding on the way out.
template <typename T>
__global__ void __launch_bounds__(256) bias_rope_vnorm_kv_store_kernel(
    T* __restrict__ qkv, int64_t ld, int64_t num_tokens, int H, int G, int D, int E, int64_t k_off, int64_t v_off,
    const T* __restrict__ bq, const T* __restrict__ bk, const T* __restrict__ bv, const int64_t* __restrict__ positions,
    const float* __restrict__ inv_freq, int rot, float eps, T* __restrict__ k_pool, T* __restrict__ v_pool,
    const int64_t* __restrict__ loc) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int items = H + 2 * G;
  const int64_t item = (int64_t)blockIdx.x * 4 + wave;
  if (item >= num_tokens * items) return;
  const int64_t t = item / items;
  const int h = (int)(item % items);
  T* row = qkv + t * ld;
  if (h < H + G) {
    const bool is_q = h < H;
    const int hh = is_q ? h : h - H;
    T* src = is_q ? row + (int64_t)hh * D : row + k_off + (int64_t)hh * D;
    const T* bias = is_q ? bq : bk;
    T* dst = is_q ? src : k_pool + (loc[t] * G + hh) * D;
    const float pos = (float)positions[t];
    for (int i = lane; i < rot / 2; i += 64) {
      float x0 = Elem<T>::to_f(src[2 * i]), x1 = Elem<T>::to_f(src[2 * i + 1]);
      if (bias) {
        x0 += Elem<T>::to_f(bias[hh * D + 2 * i]);
        x1 += Elem<T>::to_f(bias[hh * D + 2 * i + 1]);
      }
      float sn, cs;
      sincosf(pos * inv_freq[i], &sn, &cs);
      dst[2 * i] = Elem<T>::from_f(x0 * cs - x1 * sn);
      dst[2 * i + 1] = Elem<T>::from_f(x1 * cs + x0 * sn);
    }
    for (int d = rot + lane; d < D; d += 64) {
      float x = Elem<T>::to_f(src[d]);
      if (bias) x += Elem<T>::to_f(bias[hh * D + d]);
      dst[d] = Elem<T>::from_f(x);
    }
  } else {
    const int g = h - H - G;
    const T* src = row + v_off + (int64_t)g * E;
    T* dst = v_pool + (loc[t] * G + g) * E;
    float x[8], ss = 0.f;      // E <= 512
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int e = lane + 64 * u;
      x[u] = 0.f;
      if (e < E) {
        x[u] = Elem<T>::to_f(src[e]);
        if (bv) x[u] += Elem<T>::to_f(bv[g * E + e]);
        ss += x[u] * x[u];
      }
    }
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(ss / (float)E + eps);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int e = lane + 64 * u;
      if (e < E) dst[e] = Elem<T>::from_f(x[u] * r);
    }
  }
}

// The same for 16-bit types with 16-byte accesses, one wave per TOKEN: the cosines and sines of the token's angles are
// computed once (into LDS) and serve every q and k head; a head of q / k is D / 8 pieces of four pairs, taken by the lanes in
// turn; value heads go Lp lanes each (the power of two above E / 8) with the sum of squares reduced inside the group.
// D, E, rot multiples of 8 (a piece is rotated wholly or not at all), rot <= 512, E <= 512.
// gridDim.y waves share a token (few tokens: a decode batch would otherwise be a handful of waves walking all heads in turn);
// each computes the angles it needs itself.
template <typename T>
__global__ void __launch_bounds__(256) bias_rope_vnorm_kv_store_vec_kernel(
    T* __restrict__ qkv, int64_t ld, int64_t num_tokens, int H, int G, int D, int E, int64_t k_off, int64_t v_off,
    const T* __restrict__ bq, const T* __restrict__ bk, const T* __restrict__ bv, const int64_t* __restrict__ positions,
    const float* __restrict__ inv_freq, int rot, float eps, T* __restrict__ k_pool, T* __restrict__ v_pool,
    const int64_t* __restrict__ loc) {
  __shared__ float cs_lds[4][2][256];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t t = (int64_t)blockIdx.x * 4 + wave;
  if (t >= num_tokens) return;            // (whole waves leave: what follows synchronises inside a wave only)
  const float pos = (float)positions[t];
  for (int i = lane; i < rot / 2; i += 64) {
    float sn, cs;
    sincosf(pos * inv_freq[i], &sn, &cs);
    cs_lds[wave][0][i] = cs;
    cs_lds[wave][1][i] = sn;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  T* row = qkv + t * ld;
  const int64_t slot = loc[t];
  const int L = D >> 3, n_qk = (H + G) * L;
  const int part = blockIdx.y, parts = gridDim.y;
  for (int idx = lane + 64 * part; idx < n_qk; idx += 64 * parts) {
    const int h = idx / L, pc = idx - h * L;
    const bool is_q = h < H;
    const int hh = is_q ? h : h - H;
    T* src = (is_q ? row + (int64_t)h * D : row + k_off + (int64_t)hh * D) + pc * 8;
    const Vec16<T> x = load16(src);
    float f[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) f[u] = Elem<T>::to_f(x.e[u]);
    const T* bias = is_q ? bq : bk;
    if (bias) {
      const Vec16<T> bb = load16(bias + hh * D + pc * 8);
#pragma unroll
      for (int u = 0; u < 8; ++u) f[u] += Elem<T>::to_f(bb.e[u]);
    }
    if (pc * 8 < rot) {
      const float4 c4 = *reinterpret_cast<const float4*>(&cs_lds[wave][0][pc * 4]);
      const float4 s4 = *reinterpret_cast<const float4*>(&cs_lds[wave][1][pc * 4]);
      const float cs[4] = {c4.x, c4.y, c4.z, c4.w}, sn[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float x0 = f[2 * j], x1 = f[2 * j + 1];
        f[2 * j] = x0 * cs[j] - x1 * sn[j];
        f[2 * j + 1] = x1 * cs[j] + x0 * sn[j];
      }
    }
    Vec16<T> y;
#pragma unroll
    for (int u = 0; u < 8; ++u) y.e[u] = Elem<T>::from_f(f[u]);
    store16(is_q ? src : k_pool + (slot * G + hh) * D + pc * 8, y);
  }
  const int LV = E >> 3;
  int Lp = 1;
  while (Lp < LV) Lp <<= 1;
  const int per_iter = 64 / Lp, sl = lane & (Lp - 1);
  for (int g0 = per_iter * part; g0 < G; g0 += per_iter * parts) {
    const int g = g0 + lane / Lp;
    const bool on = g < G && sl < LV;
    float f[8], ss = 0.f;
#pragma unroll
    for (int u = 0; u < 8; ++u) f[u] = 0.f;
    if (on) {
      const Vec16<T> x = load16(row + v_off + (int64_t)g * E + sl * 8);
#pragma unroll
      for (int u = 0; u < 8; ++u) f[u] = Elem<T>::to_f(x.e[u]);
      if (bv) {
        const Vec16<T> bb = load16(bv + g * E + sl * 8);
#pragma unroll
        for (int u = 0; u < 8; ++u) f[u] += Elem<T>::to_f(bb.e[u]);
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) ss += f[u] * f[u];
    }
    for (int o = Lp >> 1; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
    if (on) {
      const float r = 1.0f / sqrtf(ss / (float)E + eps);
      Vec16<T> y;
#pragma unroll
      for (int u = 0; u < 8; ++u) y.e[u] = Elem<T>::from_f(f[u] * r);
      store16(v_pool + (slot * G + g) * E + sl * 8, y);
    }
  }
}

// ------------------------------------------------------------------------------------------------ latent attention: preparation
// Rows of `proj` hold, per head, [D unrotated | P rotated] query elements from column 0; rows of `latent` (the same rows at
// another column, or the rows of another projection) the latent [R] and one rotated key part [P] shared by all heads.
// `halves`: pair i of a rotation is elements (i, i + rot_dims / 2) instead of the neighbours (2i, 2i + 1).
// One workgroup per token:
//   latent / sqrt(mean(latent^2) + eps) * weight -> pool row [0, R); the key part, its first rot_dims elements turned
//   in neighbouring pairs by position * freq[i] (cos and sin times `mscale`) -> pool row [R, R + P);
//   the rotated part of every head's query, turned the same way -> q_out[t, h * q_head_stride + q_head_off ...): behind
//   the R elements that the query times the key up-projection fills, or in place.
// Angles, the norm and the products are fp32; one rounding on the way out.
template <typename T>
__global__ void __launch_bounds__(256) latent_prep_kernel(const T* __restrict__ proj, int64_t ld, int64_t num_tokens, int H, int D,
                                                          int P, int R, const T* __restrict__ latent, int64_t latent_ld,
                                                          int halves, const T* __restrict__ norm_w, float eps,
                                                          const int64_t* __restrict__ positions, const float* __restrict__ freq,
                                                          int rot_dims, float mscale, T* __restrict__ pool, int64_t pool_ld,
                                                          const int64_t* __restrict__ loc, T* __restrict__ q_out, int64_t q_ld,
                                                          int q_head_stride, int q_head_off) {
  // a workgroup per token: the token's cosines and sines once into LDS for the key part and every head, wave 0 norms the
  // latent meanwhile, then all threads walk the (unit, pair) items
  extern __shared__ float cs_l[];          // [rot_dims / 2][2]
  __shared__ float rs_l;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t t = blockIdx.x;
  const float pos = (float)positions[t];
  const int half = rot_dims >> 1;
  const T* c = latent + t * latent_ld;
  T* row = pool + loc[t] * pool_ld;
  if (wave == 0) {
    float sq = 0.f;
    for (int i = lane; i < R; i += 64) {
      const float v = Elem<T>::to_f(c[i]);
      sq += v * v;
    }
    sq = wave_sum(sq);
    if (lane == 0) rs_l = 1.0f / sqrtf(sq / (float)R + eps);
  } else {
    for (int i = tid - 64; i < half; i += 192) {
      float sn, cs;
      sincosf(pos * freq[i], &sn, &cs);
      cs_l[2 * i] = cs * mscale;
      cs_l[2 * i + 1] = sn * mscale;
    }
  }
  __syncthreads();
  const float rs = rs_l;
  for (int i = tid; i < R; i += 256) row[i] = Elem<T>::from_f(Elem<T>::to_f(c[i]) * rs * Elem<T>::to_f(norm_w[i]));
  // unit 0: the shared key part behind the latent in the pool row; unit 1 + h: head h's rotated query part
  const int per = half + (P - rot_dims);             // items of a unit: the pairs, then the elements that pass unchanged
  for (int item = tid; item < (H + 1) * per; item += 256) {
    const int u = item / per, i = item % per;
    const T* src = u == 0 ? c + R : proj + t * ld + (int64_t)(u - 1) * (D + P) + D;
    T* dst = u == 0 ? row + R : q_out + t * q_ld + (int64_t)(u - 1) * q_head_stride + q_head_off;
    if (i < half) {
      const float cs = cs_l[2 * i], sn = cs_l[2 * i + 1];
      const int i1 = halves ? i : 2 * i, i2 = halves ? i + half : 2 * i + 1;     // pair i: (i, i + dims / 2) or (2i, 2i + 1)
      const float x1 = Elem<T>::to_f(src[i1]), x2 = Elem<T>::to_f(src[i2]);
      dst[i1] = Elem<T>::from_f(x1 * cs - x2 * sn);
      dst[i2] = Elem<T>::from_f(x2 * cs + x1 * sn);
    } else {
      dst[rot_dims + (i - half)] = src[rot_dims + (i - half)];
    }
  }
}


// ------------------------------------------------------------------------------------------------ attention whose heads talk
// Preparation behind the q | k | v projection of a layer whose queries and keys are normed over the WHOLE projection (all
// heads at once): q / sqrt(mean(q^2) + eps) * q_weight over its H * D elements, the same for k over G * D, then the first
// rot_dims elements of every head turned by position * freq[i] (pair i = elements (2i, 2i + 1), or (i, i + rot_dims / 2)
// with `halves`; cos and sin times `mscale`), then every query head times head_scale[h] (a per-head temperature, folded into the query in fp32).
// q in place, k and v into the pools at loc.  A workgroup per token; norms, angles and products fp32, one rounding.
template <typename T>
__global__ void __launch_bounds__(256) qk_norm_rope_kv_store_kernel(T* __restrict__ qkv, int64_t ld, int H, int G, int D, int E,
                                                                    int64_t k_off, int64_t v_off, const T* __restrict__ q_w,
                                                                    const T* __restrict__ k_w, float eps,
                                                                    const int64_t* __restrict__ positions,
                                                                    const float* __restrict__ freq, int rot_dims, int halves,
                                                                    float mscale, const float* __restrict__ head_scale,
                                                                    T* __restrict__ k_pool,
                                                                    T* __restrict__ v_pool, const int64_t* __restrict__ loc) {
  extern __shared__ float cs_l[];          // [rot_dims / 2][2]
  __shared__ float red[16];
  const int tid = threadIdx.x;
  const int64_t t = blockIdx.x;
  T* row = qkv + t * ld;
  const int64_t slot = loc[t];
  const float pos = (float)positions[t];
  const int half = rot_dims >> 1;
  for (int i = tid; i < half; i += 256) {
    float sn, cs;
    sincosf(pos * freq[i], &sn, &cs);
    cs_l[2 * i] = cs * mscale;
    cs_l[2 * i + 1] = sn * mscale;
  }
  float sq = 0.f, sk = 0.f;
  if (q_w)
    for (int i = tid; i < H * D; i += 256) {
      const float v = Elem<T>::to_f(row[i]);
      sq += v * v;
    }
  if (k_w)
    for (int i = tid; i < G * D; i += 256) {
      const float v = Elem<T>::to_f(row[k_off + i]);
      sk += v * v;
    }
  sq = block_sum(sq, red);
  sk = block_sum(sk, red);                 // (block_sum's first barrier also orders the reads of red above and cs_l's writes)
  const float rq = q_w ? 1.0f / sqrtf(sq / (float)(H * D) + eps) : 1.0f;
  const float rk = k_w ? 1.0f / sqrtf(sk / (float)(G * D) + eps) : 1.0f;
  __syncthreads();
  const int per = half + (D - rot_dims);             // items of a head: the pairs, then the elements that pass unchanged
  for (int item = tid; item < (H + G) * per; item += 256) {
    const int u = item / per, i = item % per;
    const bool is_q = u < H;
    const int h = is_q ? u : u - H;
    const T* src = is_q ? row + (int64_t)h * D : row + k_off + (int64_t)h * D;
    const T* wv = is_q ? (q_w ? q_w + (int64_t)h * D : nullptr) : (k_w ? k_w + (int64_t)h * D : nullptr);
    T* dst = is_q ? row + (int64_t)h * D : k_pool + (slot * G + h) * D;
    const float r = is_q ? rq : rk;
    const float hs = (is_q && head_scale) ? head_scale[h] : 1.0f;
    if (i < half) {
      const int i1 = halves ? i : 2 * i, i2 = halves ? i + half : 2 * i + 1;
      const float cs = cs_l[2 * i], sn = cs_l[2 * i + 1];
      const float x1 = Elem<T>::to_f(src[i1]) * r * (wv ? Elem<T>::to_f(wv[i1]) : 1.0f);
      const float x2 = Elem<T>::to_f(src[i2]) * r * (wv ? Elem<T>::to_f(wv[i2]) : 1.0f);
      dst[i1] = Elem<T>::from_f((x1 * cs - x2 * sn) * hs);
      dst[i2] = Elem<T>::from_f((x2 * cs + x1 * sn) * hs);
    } else {
      const int e = rot_dims + (i - half);
      dst[e] = Elem<T>::from_f(Elem<T>::to_f(src[e]) * r * (wv ? Elem<T>::to_f(wv[e]) : 1.0f) * hs);
    }
  }
  for (int i = tid; i < G * E; i += 256) v_pool[slot * (int64_t)G * E + i] = row[v_off + i];
}

// The heads' attention weights mixed AFTER the softmax: w'_h(i, j) = sum_g talk[h, g] w_g(i, j), and head h applies w'_h to
// the values of its own key/value head c(h).  The sum over the keys is linear, so
//     out_h = sum_g talk[h, g] * (w_g applied to the values of head c(h)),
// and `parts` [T, H, G, E] holds w_g applied to the values of EVERY key/value head (attention whose value row is shared).
// A workgroup per token, a thread per element of out [T, H * E]; fp32 sums.  STAGED: the token's row of `parts` and the mix
// matrix go through LDS first (every element of the row is read by the H / G heads of its key/value head).
template <typename T, bool STAGED>
__global__ void __launch_bounds__(256) talk_mix_kernel(const T* __restrict__ parts, int64_t p_ld, const float* __restrict__ talk,
                                                       T* __restrict__ out, int64_t out_ld, int H, int G, int E) {
  extern __shared__ float mix_l[];         // STAGED: talk [H * H] | the row [H * G * E]
  const int64_t t = blockIdx.x;
  const T* p = parts + t * p_ld;
  const int per = H / G;
  if constexpr (STAGED) {
    float* tk = mix_l;
    float* pr = mix_l + H * H;
    for (int i = threadIdx.x; i < H * H; i += 256) tk[i] = talk[i];
    const int n = H * G * E;
    constexpr int V = Elem<T>::kVec;
    if (n % V == 0 && p_ld % V == 0 && (reinterpret_cast<uintptr_t>(parts) & 15u) == 0) {
      for (int i = threadIdx.x * V; i < n; i += 256 * V) {
        const Vec16<T> v = load16(p + i);
#pragma unroll
        for (int u = 0; u < V; ++u) pr[i + u] = Elem<T>::to_f(v.e[u]);
      }
    } else {
      for (int i = threadIdx.x; i < n; i += 256) pr[i] = Elem<T>::to_f(p[i]);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < H * E; i += 256) {
      const int h = i / E, e = i - h * E, c = h / per;
      float y = 0.f;
      for (int g = 0; g < H; ++g) y += tk[h * H + g] * pr[(g * G + c) * E + e];
      out[t * out_ld + i] = Elem<T>::from_f(y);
    }
  } else {
    for (int i = threadIdx.x; i < H * E; i += 256) {
      const int h = i / E, e = i - h * E, c = h / per;
      float y = 0.f;
      for (int g = 0; g < H; ++g) y += talk[h * H + g] * Elem<T>::to_f(p[((int64_t)g * G + c) * E + e]);
      out[t * out_ld + i] = Elem<T>::from_f(y);
    }
  }
}

// ------------------------------------------------------------------------------------------------ shared pieces
struct LocalAttnArgs {
  const void* q; int64_t q_ld;
  const void* gate; int64_t gate_ld;
  void* out; int64_t out_ld;
  const void* k_pool; const void* v_pool;
  const int32_t* req_to_token; int64_t r2t_stride;
  const int64_t* req_pool_indices; const int64_t* seq_lens;
  const int32_t* q_start; const int32_t* q_len;
  int64_t batch, num_tokens;
  int H, G, D, E;
  const float* sink;
  float scale, cap;
  int chunk;
  int64_t n_tiles;       // prompt form: 64-row tiles, an upper bound (tiles past the last request's do nothing)
  int window, keep_first;          // window > 0: keys pos - window + 1 .. pos and keys 0 .. keep_first - 1
  const float* head_bias;          // sigmoid weights: added to the score of every key of the head (may be NULL)
  int sigmoid;                     // 0: softmax over the visible keys (+ sink); 1: independent sigmoid weights
  float out_scale;
  int64_t k_ld, v_ld;              // elements between the rows of two slots (G * D and G * E for pools of their own)
  int n_splits;                    // decode form: workgroups that share the keys of one (request, kv head, 16 q heads) (0 / 1: one)
  float* partial;                  // [rows, H, n_splits, E + 2] fp32: unnormalised sums, running maximum, denominator
  int v_shared;                    // 1: the value row of a slot is ONE head of E elements that every key/value head's queries read
};

// first visible position of the contiguous range that ends at the query (the kept first positions come on top)
__device__ __forceinline__ int64_t range_lo(const LocalAttnArgs& a, int64_t pos) {
  if (a.window > 0) return pos - a.window + 1 > 0 ? pos - a.window + 1 : 0;
  return a.chunk > 0 ? (pos / a.chunk) * a.chunk : 0;
}
// how many of the kept first positions lie in front of that range
__device__ __forceinline__ int64_t kept_before(const LocalAttnArgs& a, int64_t lo) {
  if (a.window <= 0) return 0;
  return a.keep_first < lo ? a.keep_first : lo;
}

__device__ __forceinline__ float capped(float s, float scale, float cap) {
  s *= scale;
  return cap > 0.f ? cap * tanhf(s / cap) : s;
}

// the request that owns query row t, its position and its table row (q_start == NULL: row t is request t's newest token)
__device__ __forceinline__ bool locate_row(const LocalAttnArgs& a, int64_t t, int& b, int64_t& pos) {
  if (a.q_start == nullptr) {
    b = (int)t;
    pos = a.seq_lens[b] - 1;
    return pos >= 0;
  }
  for (int r = 0; r < (int)a.batch; ++r) {
    const int64_t s = a.q_start[r], n = a.q_len[r];
    if (t >= s && t < s + n) {
      b = r;
      pos = a.seq_lens[r] - n + (t - s);
      return true;
    }
  }
  return false;
}

// ------------------------------------------------------------------------------------------------ one wave per row
template <typename T, int NA>      // head sizes up to 64 * NA
__global__ void __launch_bounds__(256) local_attention_rows_kernel(LocalAttnArgs a) {
  __shared__ float q_lds[4][64 * NA];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t t = (int64_t)blockIdx.x * 4 + wave;
  const int h = blockIdx.y;
  if (t >= a.num_tokens) return;
  int b;
  int64_t pos;
  if (!locate_row(a, t, b, pos)) return;
  const int D = a.D, E = a.E, G = a.G;
  const int g = h / (a.H / G);
  const T* q = (const T*)a.q + t * a.q_ld + (int64_t)h * D;
  for (int d = lane; d < D; d += 64) q_lds[wave][d] = Elem<T>::to_f(q[d]);
  __builtin_amdgcn_wave_barrier();
  const int32_t* row = a.req_to_token + a.req_pool_indices[b] * a.r2t_stride;
  const int64_t lo = range_lo(a, pos), n_first = kept_before(a, lo);
  const T* kp = (const T*)a.k_pool;
  const T* vp = (const T*)a.v_pool;
  const bool sig = a.sigmoid != 0;
  const float hb = (sig && a.head_bias) ? a.head_bias[h] : 0.f;
  float m = sig ? 0.f : -INFINITY, l = 0.f, acc[NA];
#pragma unroll
  for (int u = 0; u < NA; ++u) acc[u] = 0.f;
  constexpr int V = Elem<T>::kVec;
  // the kept first positions (none without a window), then the range that ends at the query
  for (int seg = n_first > 0 ? 0 : 1; seg < 2; ++seg) {
    const int64_t j_begin = seg == 0 ? 0 : lo, j_last = seg == 0 ? n_first - 1 : pos;
    for (int64_t j0 = j_begin; j0 <= j_last; j0 += 64) {
      const int64_t j = j0 + lane;
      const bool valid = j <= j_last;
      const int slot = valid ? row[j] : 0;
      float s = -INFINITY;
      if (valid) {
        const T* k = kp + (int64_t)slot * a.k_ld + (int64_t)g * D;
        float dot = 0.f;
        if ((D % V) == 0) {
          for (int d = 0; d < D; d += V) {
            const Vec16<T> kv = load16(k + d);
#pragma unroll
            for (int u = 0; u < V; ++u) dot += q_lds[wave][d + u] * Elem<T>::to_f(kv.e[u]);
          }
        } else {
          for (int d = 0; d < D; ++d) dot += q_lds[wave][d] * Elem<T>::to_f(k[d]);
        }
        s = capped(dot, a.scale, a.cap);
      }
      float p;
      if (sig) {
        p = valid ? 1.0f / (1.0f + expf(-(s + hb))) : 0.f;
      } else {
        const float m_new = fmaxf(m, wave_max(s));
        const float alpha = expf(m - m_new);      // first tile: exp(-inf) = 0
        p = valid ? expf(s - m_new) : 0.f;
        l = l * alpha + wave_sum(p);
#pragma unroll
        for (int u = 0; u < NA; ++u) acc[u] *= alpha;
        m = m_new;
      }
      const int n = (int)((j_last - j0 + 1) < 64 ? (j_last - j0 + 1) : 64);
      for (int jj = 0; jj < n; ++jj) {
        const float pj = __shfl(p, jj, 64);
        const int sj = __shfl(slot, jj, 64);
        const T* v = vp + (int64_t)sj * a.v_ld + (a.v_shared ? 0 : (int64_t)g * E);
#pragma unroll
        for (int u = 0; u < NA; ++u) {
          const int e = lane + 64 * u;
          if (e < E) acc[u] += pj * Elem<T>::to_f(v[e]);
        }
      }
    }
  }
  if (!sig && a.sink != nullptr) l += expf(a.sink[h] - m);
  const float inv = sig ? a.out_scale : a.out_scale / l;
  T* o = (T*)a.out + t * a.out_ld + (int64_t)h * E;
  const T* gt = a.gate ? (const T*)a.gate + t * a.gate_ld + (int64_t)h * E : nullptr;
#pragma unroll
  for (int u = 0; u < NA; ++u) {
    const int e = lane + 64 * u;
    if (e < E) {
      float y = acc[u] * inv;
      if (gt) y *= 1.0f / (1.0f + expf(-Elem<T>::to_f(gt[e])));
      o[e] = Elem<T>::from_f(y);
    }
  }
}

// ------------------------------------------------------------------------------------------------ matrix-core forms
// v_mfma_f32_16x16x32 (lane l: r = l & 15, g = l >> 4): a = A[row r][k 8g .. 8g+7], b = B[k 8g .. 8g+7][col r],
// d[i] = D[row 4g + i][col r].  One step covers 32 keys: S^T = K Q^T in two 16-row groups (keys 0 .. 15 and 16 .. 31 of the
// step), so lane (r, g) ends with the scores of keys 4g .. 4g+3 and 16 + 4g .. + 3 of query r, which IS the b operand of
// O^T += V^T P^T once the a operand numbers its k slots the same way: V^T comes out of a row-major LDS tile [32][E] through
// the transposing read ds_read_b64_tr_b16, four keys x 16 value elements per 16-lane group.
// The loads of step i + 1 (K fragments, V rows) are in flight in registers while step i is multiplied.
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <typename T> __device__ __forceinline__ f32x4 mma16(const Frag16& a, const Frag16& b, f32x4 c);
template <> __device__ __forceinline__ f32x4 mma16<bf16_t>(const Frag16& a, const Frag16& b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.b, b.b, c, 0, 0, 0);
}
template <> __device__ __forceinline__ f32x4 mma16<f16_t>(const Frag16& a, const Frag16& b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(a.f, b.f, c, 0, 0, 0);
}

// Scores live in the base-2 domain (multiplied by log2 e) so that every exponential is one v_exp_f32, and the cap is
//   cap * tanh(x / cap) * log2e = A - 2 A / (exp2(c raw) + 1),  A = cap log2e,  c = 2 scale log2e / cap
// (one exp, one reciprocal: exp2 overflow gives A, underflow -A).  Without a cap: raw * scale * log2e.
constexpr float kLog2e = 1.4426950408889634f;
struct ScoreMap {
  float c, A;          // A == 0: no cap
  __device__ __forceinline__ ScoreMap(float scale, float cap)
      : c(cap > 0.f ? 2.0f * scale * kLog2e / cap : scale * kLog2e), A(cap > 0.f ? cap * kLog2e : 0.f) {}
  __device__ __forceinline__ float operator()(float raw) const {
    const float t = raw * c;
    if (A == 0.f) return t;
    return A - 2.0f * A * __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(t) + 1.0f);
  }
};

// bytes per row of the V tile: E halves + padding so that the stride is 16 or 48 dwords mod 64 (conflict-free transposing
// reads) and a multiple of 16 bytes
__host__ __device__ inline int v_tile_row_bytes(int E) { return (E / 2 + (((16 - E / 2) % 32) + 32) % 32) * 4; }

constexpr int kIdxLds = 2048;      // slots of the visible keys kept in LDS (8 KB): ranges up to this long

template <int NE> struct SoftState {
  float m, l;
  f32x4 acc[NE];
};
template <int ND> struct KFrags {
  Frag16 a[ND], b[ND];
};

// The walk over keys j_begin, j_begin + j_step, ... (steps of 32 keys, keys past j_end masked) for the 16 columns of this wave.
//   NT threads (a workgroup with BLOCK_SYNC, else one wave) stage the V tile of every step; `tid` is the thread's index among
//   them.  relevant(j0): whether this wave has anything to multiply in the step at j0 (it stages and syncs anyway).
//   ok(j): whether key j is visible to this lane's column.
//   BLOCK_SYNC (a workgroup walks together): the K rows of a step go through an LDS tile as well, loaded once for all waves
//   in whole rows; a wave on its own takes its K fragments straight from the pool into operand layout.
//   32 keys per step (64 between one pair of barriers measured slower: the staging registers of 64 rows push the 128 / 128
//   kernel into scratch).
template <typename T, int ND, int NE, int NT, bool BLOCK_SYNC, bool SIG, typename Ok, typename Relevant>
__device__ __forceinline__ void key_walk(SoftState<NE>& st, const Frag16 (&qf)[ND], int nd, int ne, int E, const T* kp,
                                         int64_t kstride, const T* vp, int64_t vstride, const int32_t* row, int64_t j_begin,
                                         int64_t j_end, int64_t j_step, uint8_t* v_lds, int tid, float scale, float cap, Ok ok,
                                         Relevant relevant, int r, int g, const int32_t* idx_lds, int64_t idx_base,
                                         float hb = 0.f) {
  constexpr int KS = 32;                          // keys per step
  constexpr int NV = (NE * 2 * KS) / NT;          // 16-byte pieces of V per thread and step, at most
  constexpr int NK = BLOCK_SYNC ? (ND * 4 * KS) / NT : 1;   // the same for K rows that go through LDS
  const int per_key = E >> 3, pieces = KS * per_key, rs = v_tile_row_bytes(E);
  const int per_key_k = nd * 4, pieces_k = KS * per_key_k, rsk = nd * 64 + 32;
  // a workgroup keeps TWO pairs of tiles: while step i is multiplied out of one, the rows of step i + 1 land in the other,
  // and one barrier per step separates them
  const int tile_pair = KS * (rs + rsk);
  uint8_t* k_lds = v_lds + KS * rs;
  uint4 vr[NV];
  uint4 kr[NK];
  const ScoreMap smap(scale, cap);
  // which row and which 16 bytes of it each of this thread's pieces is (the same in every step)
  int v_key[NV], v_ec[NV], k_key[NK], k_ec[NK];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = i * NT + tid;
    v_key[i] = c < pieces ? c / per_key : -1;
    v_ec[i] = c < pieces ? c - v_key[i] * per_key : 0;
  }
#pragma unroll
  for (int i = 0; i < NK; ++i) {
    const int c = i * NT + tid;
    k_key[i] = (BLOCK_SYNC && c < pieces_k) ? c / per_key_k : -1;
    k_ec[i] = (BLOCK_SYNC && c < pieces_k) ? c - k_key[i] * per_key_k : 0;
  }
  // pool slot of key j: from the copy of this part of the request's row in LDS when the caller made one (the load of a row
  // of the pool then waits for nothing but itself), else from the table
  auto slot_of = [&](int64_t j) -> int64_t { return idx_lds ? idx_lds[j - idx_base] : row[j]; };
  auto sync = [&]() {
    if constexpr (BLOCK_SYNC) {
      __syncthreads();
    } else {   // one wave: its LDS accesses execute in order; keep the compiler from reordering them
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
  };
  auto load_v = [&](int64_t j0) {
#pragma unroll
    for (int i = 0; i < NV; ++i)
      if (v_key[i] >= 0) {
        const int64_t j = j0 + v_key[i];
        vr[i] = j <= j_end ? *reinterpret_cast<const uint4*>(vp + slot_of(j) * vstride + v_ec[i] * 8) : uint4{0u, 0u, 0u, 0u};
      }
  };
  auto store_v = [&](int buf) {        // buf: which pair of tiles (a lone wave has one)
#pragma unroll
    for (int i = 0; i < NV; ++i)
      if (v_key[i] >= 0) *reinterpret_cast<uint4*>(v_lds + buf * tile_pair + v_key[i] * rs + v_ec[i] * 16) = vr[i];
    if constexpr (BLOCK_SYNC) {
#pragma unroll
      for (int i = 0; i < NK; ++i)
        if (k_key[i] >= 0) *reinterpret_cast<uint4*>(k_lds + buf * tile_pair + k_key[i] * rsk + k_ec[i] * 16) = kr[i];
    }
  };
  auto load_k_rows = [&](int64_t j0) {
#pragma unroll
    for (int i = 0; i < NK; ++i)
      if (k_key[i] >= 0) {
        const int64_t j = j0 + k_key[i];
        kr[i] = j <= j_end ? *reinterpret_cast<const uint4*>(kp + slot_of(j) * kstride + k_ec[i] * 8) : uint4{0u, 0u, 0u, 0u};
      }
  };
  auto load_k = [&](int64_t j0, auto& k) {
    const int64_t ja = j0 + r, jb = ja + 16;
    const T* pa = kp + (ja <= j_end ? slot_of(ja) : 0) * kstride + 8 * g;
    const T* pb = kp + (jb <= j_end ? slot_of(jb) : 0) * kstride + 8 * g;
#pragma unroll
    for (int kk = 0; kk < ND; ++kk)
      if (kk < nd) {
        k.a[kk].u = *reinterpret_cast<const uint4*>(pa + 32 * kk);
        k.b[kk].u = *reinterpret_cast<const uint4*>(pb + 32 * kk);
      }
  };
  auto compute = [&](int64_t j0, const auto& k, int half, auto after_scores) {   // keys j0 .. j0 + 31 out of tile pair `half`
    f32x4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
    if constexpr (BLOCK_SYNC) {
      const uint8_t* ra = k_lds + half * tile_pair + r * rsk + g * 16;
      const uint8_t* rb = ra + 16 * rsk;
#pragma unroll
      for (int kk = 0; kk < ND; ++kk)
        if (kk < nd) {
          Frag16 fa, fb;
          fa.u = *reinterpret_cast<const uint4*>(ra + kk * 64);
          fb.u = *reinterpret_cast<const uint4*>(rb + kk * 64);
          sa = mma16<T>(fa, qf[kk], sa);
          sb = mma16<T>(fb, qf[kk], sb);
        }
    } else {
#pragma unroll
      for (int kk = 0; kk < ND; ++kk)
        if (kk < nd) {
          sa = mma16<T>(k.a[kk], qf[kk], sa);
          sb = mma16<T>(k.b[kk], qf[kk], sb);
        }
    }
    after_scores();            // (a lone wave asks for the next step's K fragments here: the registers are free again)
    float sc[8];
    const int64_t ja = j0 + 4 * g, jb = ja + 16;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      sc[i] = ok(ja + i) ? smap(sa[i]) : -INFINITY;
      sc[4 + i] = ok(jb + i) ? smap(sb[i]) : -INFINITY;
    }
    float p[8];
    if constexpr (SIG) {
      // independent weights sigmoid(score + hb) in the base-2 domain (hb comes multiplied by log2 e): no maximum, no sum;
      // a masked key has score -inf: exp2(+inf) = inf, 1 / inf = 0
#pragma unroll
      for (int i = 0; i < 8; ++i) p[i] = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-(sc[i] + hb)));
    } else {
    float mt = sc[0];
#pragma unroll
    for (int i = 1; i < 8; ++i) mt = fmaxf(mt, sc[i]);
    mt = fmaxf(mt, __shfl_xor(mt, 16, 64));
    mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
    const float m_new = fmaxf(st.m, mt);
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    if (__any(m_new > st.m)) {
      const float alpha = __builtin_amdgcn_exp2f(st.m - m_safe);   // st.m = -inf: 0, and nothing has been accumulated yet
      st.l *= alpha;
#pragma unroll
      for (int eb = 0; eb < NE; ++eb)
        if (eb < ne)
#pragma unroll
          for (int i = 0; i < 4; ++i) st.acc[eb][i] *= alpha;
      st.m = m_new;
    }
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      p[i] = __builtin_amdgcn_exp2f(sc[i] - m_safe);
      sum += p[i];
    }
    st.l += sum;
    }
    Frag16 pb;
#pragma unroll
    for (int i = 0; i < 4; ++i) pb.w[i] = pack2<T>(p[2 * i], p[2 * i + 1]);
    // 16-lane group g reads the 4 x 16 blocks {keys 4g .. 4g+3, then 16 + 4g ..} x {e = 16 eb .. + 15}: lane r of the group
    // supplies row (r >> 2), columns 4 (r & 3) .. + 3 and receives column r
    const uint8_t* vrow = v_lds + half * tile_pair + (g * 4 + (r >> 2)) * rs + (r & 3) * 8;
#pragma unroll
    for (int eb = 0; eb < NE; ++eb)
      if (eb < ne) {
        Frag16 va;
        va.s[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(vrow + eb * 32));
        va.s[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(vrow + 16 * rs + eb * 32));
        st.acc[eb] = mma16<T>(va, pb, st.acc[eb]);
      }
  };
  if (j_begin > j_end) return;
  KFrags<BLOCK_SYNC ? 1 : ND> k0;      // one set: a lone wave refills it as soon as the scores of a step are taken
  load_v(j_begin);
  if constexpr (BLOCK_SYNC) load_k_rows(j_begin);
  else load_k(j_begin, k0);
  if constexpr (BLOCK_SYNC) {
    store_v(0);
    sync();
    int buf = 0;
    for (int64_t j0 = j_begin; j0 <= j_end; j0 += j_step, buf ^= 1) {
      const int64_t jn = j0 + j_step;
      if (jn <= j_end) {                                 // in flight while this step is multiplied
        load_v(jn);
        load_k_rows(jn);
      }
      if (relevant(j0)) compute(j0, k0, buf, [] {});
      if (jn <= j_end) store_v(buf ^ 1);
      sync();       // the next step's rows are in place, and everyone is done with this step's
    }
  } else {
    for (int64_t j0 = j_begin; j0 <= j_end; j0 += j_step) {
      const int64_t jn = j0 + j_step;
      sync();                                            // the previous step's reads of the tile are done
      store_v(0);
      sync();
      if (jn <= j_end) load_v(jn);                       // in flight while this step is multiplied
      compute(j0, k0, 0, [&] {
        if (jn <= j_end) load_k(jn, k0);
      });
    }
  }
}

// Prompt portions: 64 query rows of one request and one head per workgroup, 16 per wave.
template <typename T, int ND, int NE, bool SIG>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(ND <= 4 ? 4 : 1))) local_attention_mfma_kernel(LocalAttnArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t v_lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 15, g = lane >> 4;
  // Workgroup -> (kv head, 64-row tile, q head of the group), the last fastest.  Consecutive workgroup ids go round the
  // eight XCDs, each with an L2 of its own; id L is therefore given work item (L % 8) * (N / 8) + L / 8, so that an XCD walks
  // a CONTIGUOUS range of items: the q heads of a kv head and the neighbouring tiles of a block of positions -- which read the
  // same K / V rows -- run next to each other on one L2 (N = gridDim.x, a multiple of 8).  (One workgroup per kv head and
  // tile that takes the q heads in turn measured slower: a quarter of the workgroups, four times as long, fill the chip badly.)
  const int64_t n_items = gridDim.x, item = (int64_t)(blockIdx.x & 7) * (n_items >> 3) + (blockIdx.x >> 3);
  const int rep_h = a.H / a.G;
  const int64_t n_tiles = a.n_tiles;
  if (item >= n_tiles * a.H) return;
  const int h = (int)(item / (n_tiles * rep_h)) * rep_h + (int)(item % rep_h);
  // (tiles from the last to the first: the workgroups that start last are the first tiles of a block of positions, the ones
  //  with the fewest keys, so the launch ends without a long tail)
  const int64_t tile_id = n_tiles - 1 - (item / rep_h) % n_tiles;
  // which request and which 64-row tile of it
  int b = -1;
  int64_t q0 = 0;
  {
    int64_t left = tile_id;
    for (int rq0 = 0; rq0 < (int)a.batch && b < 0; rq0 += 8) {     // eight lengths per round trip
      int32_t n[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) n[u] = rq0 + u < (int)a.batch ? a.q_len[rq0 + u] : 0;
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int64_t tiles = ((int64_t)n[u] + 63) >> 6;
        if (b < 0 && left < tiles) {
          b = rq0 + u;
          q0 = left << 6;
        }
        if (b < 0) left -= tiles;
      }
    }
  }
  if (b < 0) return;
  const int D = a.D, E = a.E, G = a.G, nd = D >> 5, ne = E >> 4;
  const int gk = h / (a.H / G);
  const int64_t qn = a.q_len[b], base_pos = a.seq_lens[b] - qn, t0 = a.q_start[b];
  auto lo_of = [&](int64_t p) -> int64_t { return range_lo(a, p); };
  const int64_t keep = a.window > 0 ? a.keep_first : 0;      // first positions that stay visible in front of the window
  const int64_t blk_last = (q0 + 63 < qn - 1 ? q0 + 63 : qn - 1);
  const int64_t blk_lo = lo_of(base_pos + q0), blk_hi = base_pos + blk_last;
  // this wave's 16 rows
  const int64_t wq0 = q0 + 16 * wave;
  const bool wave_on = wq0 < qn;
  const int64_t wq_last = wq0 + 15 < qn - 1 ? wq0 + 15 : qn - 1;
  const int64_t w_lo = lo_of(base_pos + wq0), w_hi = base_pos + wq_last;
  const bool q_ok = wq0 + r < qn;
  const int64_t my_q = q_ok ? wq0 + r : (wave_on ? wq_last : 0);
  const int64_t my_pos = base_pos + my_q, my_lo = lo_of(my_pos);
  Frag16 qf[ND];
  {
    const T* q = (const T*)a.q + (t0 + my_q) * a.q_ld + (int64_t)h * D;
#pragma unroll
    for (int kk = 0; kk < ND; ++kk)
      if (kk < nd) qf[kk].u = *reinterpret_cast<const uint4*>(q + 32 * kk + 8 * g);
  }
  SoftState<NE> st;
  st.m = -INFINITY;
  st.l = 0.f;
#pragma unroll
  for (int eb = 0; eb < NE; ++eb) st.acc[eb] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int32_t* row = a.req_to_token + a.req_pool_indices[b] * a.r2t_stride;
  const float hb = (SIG && a.head_bias) ? a.head_bias[h] * kLog2e : 0.f;
  // the kept first positions that lie in front of the tile's window range: visible to every row of the tile
  const int64_t n_first = keep < blk_lo ? keep : blk_lo;
  if (n_first > 0)
    key_walk<T, ND, NE, 256, true, SIG>(
        st, qf, nd, ne, E, (const T*)a.k_pool + (int64_t)gk * D, a.k_ld, (const T*)a.v_pool + (a.v_shared ? 0 : (int64_t)gk * E),
        a.v_ld, row, 0, n_first - 1, 32, v_lds, tid, a.scale, a.cap, [&](int64_t j) { return q_ok && j < n_first; },
        [&](int64_t) { return wave_on; }, r, g, nullptr, 0, hb);
  key_walk<T, ND, NE, 256, true, SIG>(
      st, qf, nd, ne, E, (const T*)a.k_pool + (int64_t)gk * D, a.k_ld, (const T*)a.v_pool + (a.v_shared ? 0 : (int64_t)gk * E),
      a.v_ld, row, blk_lo, blk_hi, 32, v_lds, tid, a.scale, a.cap,
      [&](int64_t j) { return q_ok && j <= my_pos && (j >= my_lo || j < keep); },
      [&](int64_t j0) { return wave_on && j0 <= w_hi && (j0 + 31 >= w_lo || j0 < keep); }, r, g, nullptr, blk_lo, hb);
  float l = st.l;
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (!wave_on) return;
  if (!SIG && a.sink != nullptr) l += __builtin_amdgcn_exp2f(a.sink[h] * kLog2e - st.m);      // (the running maximum is in the base-2 domain)
  const float inv = q_ok ? (SIG ? a.out_scale : a.out_scale / l) : 0.f;
  // Epilogue through LDS (the tiles are free: the walk ends on a barrier): a lane holds 4 value elements of one row per
  // 16-element block -- written out like that, rows would go to memory in 8-byte pieces; the wave lays its 16 x E tile down in
  // LDS and takes it up again in whole 16-byte pieces of consecutive lanes, so the gate is read and the result written in
  // full rows.
  const int ors = E * 2 + 16;
  uint8_t* o_lds = v_lds + wave * 16 * ors;
#pragma unroll
  for (int eb = 0; eb < NE; ++eb)
    if (eb < ne) {
      uint2 w;
      w.x = pack2<T>(st.acc[eb][0] * inv, st.acc[eb][1] * inv);
      w.y = pack2<T>(st.acc[eb][2] * inv, st.acc[eb][3] * inv);
      *reinterpret_cast<uint2*>(o_lds + r * ors + (eb * 16 + 4 * g) * 2) = w;
    }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  const int per_row = E >> 3;
  for (int c = lane; c < 16 * per_row; c += 64) {
    const int rr = c / per_row, ec = c - rr * per_row;
    if (wq0 + rr >= qn) continue;
    Vec16<T> v = *reinterpret_cast<const Vec16<T>*>(o_lds + rr * ors + ec * 16);
    const int64_t t = t0 + wq0 + rr;
    if (a.gate) {
      const Vec16<T> gv = load16((const T*)a.gate + t * a.gate_ld + (int64_t)h * E + ec * 8);
#pragma unroll
      for (int u = 0; u < 8; ++u)
        v.e[u] = Elem<T>::from_f(Elem<T>::to_f(v.e[u]) *
                                 __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-kLog2e * Elem<T>::to_f(gv.e[u]))));
    }
    store16((T*)a.out + t * a.out_ld + (int64_t)h * E + ec * 8, v);
  }
}

// Decode steps: one workgroup per (request, kv head, group of 16 q heads); the q heads are the 16 columns, the waves
// take the 32-key steps in turn, each with a V tile of its own, and meet in LDS.
// (eight waves for head sizes up to 128, four above: the walk's registers at 256 / 256 do not fit eight waves per CU)
template <typename T, int ND, int NE, int NW, bool SIG>
__global__ void __launch_bounds__(64 * NW) local_attention_decode_kernel(LocalAttnArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t v_lds[];
  __shared__ float part_ml[NW][2][16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 15, g = lane >> 4;
  const int b = blockIdx.x, gk = blockIdx.y;
  const int D = a.D, E = a.E, G = a.G, nd = D >> 5, ne = E >> 4;
  const int rep = a.H / G;
  const int n_splits = a.n_splits > 1 ? a.n_splits : 1, head_groups = (rep + 15) / 16;
  const int split = blockIdx.z / head_groups;
  const int col0 = (blockIdx.z % head_groups) * 16;
  const bool col_ok = col0 + r < rep;
  const int h = gk * rep + (col_ok ? col0 + r : col0);
  const int64_t t = a.q_start ? (int64_t)a.q_start[b] + a.q_len[b] - 1 : b;     // the request's newest row
  const int64_t pos_q = a.seq_lens[b] - 1;
  if (pos_q < 0) return;
  const int64_t lo_q = range_lo(a, pos_q), n_first = split == 0 ? kept_before(a, lo_q) : 0;
  // with several workgroups per (request, kv head, 16 q heads) this one walks a slice of the range (whole 32-key steps; it
  // may be empty) and leaves unnormalised sums for the merge kernel
  int64_t lo = lo_q, pos = pos_q;
  if (n_splits > 1) {
    int64_t chunk = (pos_q - lo_q + n_splits) / n_splits;
    chunk = (chunk + 31) / 32 * 32;
    lo = lo_q + split * chunk;
    pos = lo + chunk - 1 < pos_q ? lo + chunk - 1 : pos_q;
  }
  const float hb = (SIG && a.head_bias) ? a.head_bias[h] * kLog2e : 0.f;
  Frag16 qf[ND];
  {
    const T* q = (const T*)a.q + t * a.q_ld + (int64_t)h * D;
#pragma unroll
    for (int kk = 0; kk < ND; ++kk)
      if (kk < nd) qf[kk].u = *reinterpret_cast<const uint4*>(q + 32 * kk + 8 * g);
  }
  SoftState<NE> st;
  st.m = SIG ? 0.f : -INFINITY;       // (sigmoid weights need no running maximum: the partial sums merge as they are)
  st.l = 0.f;
#pragma unroll
  for (int eb = 0; eb < NE; ++eb) st.acc[eb] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int32_t* row = a.req_to_token + a.req_pool_indices[b] * a.r2t_stride;
  // a wave's tile: 32 rows of the V tile, and room for its partial sums afterwards ([E][17] floats)
  const int tile_bytes = 32 * v_tile_row_bytes(E) > E * 17 * 4 ? 32 * v_tile_row_bytes(E) : E * 17 * 4;
  uint8_t* mine_b = v_lds + wave * tile_bytes;
  __shared__ int32_t idx_lds[kIdxLds];
  const bool idx_fits = pos - lo < kIdxLds;
  if (idx_fits) {
    for (int64_t j = lo + tid; j <= pos; j += 64 * NW) idx_lds[j - lo] = row[j];
    __syncthreads();
  }
  // (pos < lo: an empty slice; the walk below does nothing and the partial sums are those of no keys)
  // the kept first positions in front of the window (none without one), then the range that ends at the query
  if (n_first > 0)
    key_walk<T, ND, NE, 64, false, SIG>(
        st, qf, nd, ne, E, (const T*)a.k_pool + (int64_t)gk * D, a.k_ld, (const T*)a.v_pool + (a.v_shared ? 0 : (int64_t)gk * E),
        a.v_ld, row, (int64_t)32 * wave, n_first - 1, 32 * NW, mine_b, lane, a.scale, a.cap,
        [&](int64_t j) { return j < n_first; }, [&](int64_t) { return true; }, r, g, nullptr, 0, hb);
  key_walk<T, ND, NE, 64, false, SIG>(
      st, qf, nd, ne, E, (const T*)a.k_pool + (int64_t)gk * D, a.k_ld, (const T*)a.v_pool + (a.v_shared ? 0 : (int64_t)gk * E),
      a.v_ld, row, lo + 32 * wave, pos, 32 * NW, mine_b, lane, a.scale, a.cap, [&](int64_t j) { return j <= pos; },
      [&](int64_t) { return true; }, r, g, idx_fits ? idx_lds : nullptr, lo, hb);
  float l = st.l;
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (g == 0) {
    part_ml[wave][0][r] = st.m;
    part_ml[wave][1][r] = l;
  }
  // a wave's partial sums go where its V tile was; only the wave itself read it
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  float* mine = reinterpret_cast<float*>(mine_b);
#pragma unroll
  for (int eb = 0; eb < NE; ++eb)
    if (eb < ne)
#pragma unroll
      for (int i = 0; i < 4; ++i) mine[(eb * 16 + 4 * g + i) * 17 + r] = st.acc[eb][i];
  __syncthreads();
  // merge: thread (column c, slice) walks the value elements slice, slice + 16, ...
  const int c = tid & 15, slice = tid >> 4;
  if (col0 + c >= rep) return;
  float m = -INFINITY;
#pragma unroll
  for (int w = 0; w < NW; ++w) m = fmaxf(m, part_ml[w][0][c]);
  float f[NW], lt = 0.f;
#pragma unroll
  for (int w = 0; w < NW; ++w) {
    const float mw = part_ml[w][0][c];
    f[w] = mw == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mw - m);
    lt += f[w] * part_ml[w][1][c];
  }
  const int hh = gk * rep + col0 + c;
  if (n_splits > 1) {
    float* part = a.partial + ((t * a.H + hh) * n_splits + split) * (int64_t)(E + 2);
    for (int e = slice; e < E; e += 4 * NW) {
      float y = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) y += f[w] * reinterpret_cast<const float*>(v_lds + w * tile_bytes)[e * 17 + c];
      part[e] = y;
    }
    if (slice == 0) {
      part[E] = m;
      part[E + 1] = lt;
    }
    return;
  }
  if (!SIG && a.sink != nullptr) lt += __builtin_amdgcn_exp2f(a.sink[hh] * kLog2e - m);
  const float inv = SIG ? a.out_scale : a.out_scale / lt;
  T* o = (T*)a.out + t * a.out_ld + (int64_t)hh * E;
  const T* gt = a.gate ? (const T*)a.gate + t * a.gate_ld + (int64_t)hh * E : nullptr;
  for (int e = slice; e < E; e += 4 * NW) {
    float y = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) y += f[w] * reinterpret_cast<const float*>(v_lds + w * tile_bytes)[e * 17 + c];
    y *= inv;
    if (gt) y *= __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-kLog2e * Elem<T>::to_f(gt[e])));
    o[e] = Elem<T>::from_f(y);
  }
}

// The slices of a decode row's keys, each with its own running maximum (base-2 domain), denominator and unnormalised sums:
// out = sum_s 2^(m_s - m) y_s / (sum_s 2^(m_s - m) l_s + 2^(sink log2 e - m)), a workgroup per (row, head).
template <typename T, bool SIG>
__global__ void __launch_bounds__(64) local_attention_merge_kernel(LocalAttnArgs a) {
  const int64_t b = blockIdx.x;
  const int h = blockIdx.y, E = a.E, n = a.n_splits;
  const int64_t t = a.q_start ? (int64_t)a.q_start[b] + a.q_len[b] - 1 : b;
  if (a.seq_lens[b] - 1 < 0) return;
  const float* part = a.partial + (t * a.H + h) * n * (int64_t)(E + 2);
  float m = -INFINITY;
  for (int s = 0; s < n; ++s) m = fmaxf(m, part[s * (E + 2) + E]);
  float lt = 0.f;
  for (int s = 0; s < n; ++s) {
    const float ms = part[s * (E + 2) + E];
    lt += (ms == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ms - m)) * part[s * (E + 2) + E + 1];
  }
  if (!SIG && a.sink != nullptr) lt += __builtin_amdgcn_exp2f(a.sink[h] * kLog2e - m);
  const float inv = SIG ? a.out_scale : a.out_scale / lt;
  T* o = (T*)a.out + t * a.out_ld + (int64_t)h * E;
  const T* gt = a.gate ? (const T*)a.gate + t * a.gate_ld + (int64_t)h * E : nullptr;
  for (int e = threadIdx.x; e < E; e += 64) {
    float y = 0.f;
    for (int s = 0; s < n; ++s) {
      const float ms = part[s * (E + 2) + E];
      y += (ms == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ms - m)) * part[s * (E + 2) + e];
    }
    y *= inv;
    if (gt) y *= __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-kLog2e * Elem<T>::to_f(gt[e])));
    o[e] = Elem<T>::from_f(y);
  }
}

}  // namespace semipd

using namespace semipd;

static inline bool local_mfma_shape_ok(int qk_dim, int v_dim) {
  return qk_dim % 32 == 0 && qk_dim <= 256 && v_dim % 16 == 0 && v_dim <= 256;
}

extern "C" int semipd_unit_norm_kv_store(void* qkv, int64_t ld, int64_t num_tokens, int num_q_heads, int num_kv_heads,
                                         int qk_dim, int v_dim, int64_t k_off, int64_t v_off, float eps, const void* v_first,
                                         int64_t v_first_ld, const void* mix, void* k_pool, void* v_pool, const int64_t* loc,
                                         int dtype, void* stream) {
  SEMIPD_CHECK_ARG(num_tokens >= 0 && num_q_heads > 0 && num_kv_heads > 0 && qk_dim > 0 && v_dim > 0, SEMIPD_EINVAL,
                   "unit_norm_kv_store: bad sizes");
  if (num_tokens == 0) return 0;
  SEMIPD_CHECK_ARG(qkv && k_pool && v_pool && loc, SEMIPD_EINVAL, "unit_norm_kv_store: null pointer");
  SEMIPD_CHECK_ARG((v_first == nullptr) == (mix == nullptr), SEMIPD_EINVAL,
                   "unit_norm_kv_store: the first values and their weight come together");
  SEMIPD_CHECK_ARG(ld >= v_off + (int64_t)num_kv_heads * v_dim && k_off >= (int64_t)num_q_heads * qk_dim &&
                       v_off >= k_off + (int64_t)num_kv_heads * qk_dim,
                   SEMIPD_EINVAL, "unit_norm_kv_store: column ranges overlap or leave the row");
  const int64_t items = num_tokens * (num_q_heads + 2 * num_kv_heads);
  const int L = qk_dim / 8;
  if ((dtype == SEMIPD_BF16 || dtype == SEMIPD_F16) && qk_dim % 8 == 0 && (L & (L - 1)) == 0 && L <= 64 && v_dim % 8 == 0 &&
      ld % 8 == 0 && k_off % 8 == 0 && v_off % 8 == 0 && aligned16(qkv) && aligned16(k_pool) && aligned16(v_pool) &&
      (!v_first || (aligned16(v_first) && v_first_ld % 8 == 0))) {
    const int64_t per_block = 4 * (64 / L);
    const unsigned vb = (unsigned)((items + per_block - 1) / per_block);
#define SEMIPD_UNKS(LL)                                                                                                        \
  SEMIPD_DISPATCH_HALF(dtype, T,                                                                                               \
                       hipLaunchKernelGGL((unit_norm_kv_store_vec_kernel<T, LL>), dim3(vb), dim3(256), 0, as_stream(stream),     \
                                          (T*)qkv, ld, num_tokens, num_q_heads, num_kv_heads, qk_dim, v_dim, k_off, v_off, eps,  \
                                          (const T*)v_first, v_first_ld, (const T*)mix, (T*)k_pool, (T*)v_pool, loc))
    switch (L) {
      case 1: SEMIPD_UNKS(1); break;
      case 2: SEMIPD_UNKS(2); break;
      case 4: SEMIPD_UNKS(4); break;
      case 8: SEMIPD_UNKS(8); break;
      case 16: SEMIPD_UNKS(16); break;
      case 32: SEMIPD_UNKS(32); break;
      default: SEMIPD_UNKS(64); break;
    }
#undef SEMIPD_UNKS
    return launch_status("unit_norm_kv_store");
  }
  const unsigned blocks = (unsigned)((items + 3) / 4);
  SEMIPD_DISPATCH_DTYPE(dtype, T,
                        hipLaunchKernelGGL((unit_norm_kv_store_kernel<T>), dim3(blocks), dim3(256), 0, as_stream(stream),
                                           (T*)qkv, ld, num_tokens, num_q_heads, num_kv_heads, qk_dim, v_dim, k_off, v_off, eps,
                                           (const T*)v_first, v_first_ld, (const T*)mix, (T*)k_pool, (T*)v_pool, loc));
  return launch_status("unit_norm_kv_store");
}

static int launch_local_attention(LocalAttnArgs a, int64_t max_q_len, int form, int dtype, void* stream);

extern "C" int semipd_local_attention(const void* q, int64_t q_ld, const void* gate, int64_t gate_ld, void* out, int64_t out_ld,
                                      const void* k_pool, const void* v_pool, const int32_t* req_to_token,
                                      int64_t req_to_token_stride, const int64_t* req_pool_indices, const int64_t* seq_lens,
                                      const int32_t* q_start, const int32_t* q_len, int64_t batch, int64_t num_tokens,
                                      int64_t max_q_len, int num_q_heads, int num_kv_heads, int qk_dim, int v_dim,
                                      const float* sink, float scale, float logit_cap, int chunk, int form, int dtype,
                                      void* stream) {
  SEMIPD_CHECK_ARG(chunk >= 0, SEMIPD_EINVAL, "local_attention: bad chunk");
  LocalAttnArgs a{q, q_ld, gate, gate_ld, out, out_ld, k_pool, v_pool, req_to_token, req_to_token_stride, req_pool_indices,
                  seq_lens, q_start, q_len, batch, num_tokens, num_q_heads, num_kv_heads, qk_dim, v_dim, sink, scale, logit_cap,
                  chunk, 0, 0, 0, nullptr, 0, 1.0f};
  return launch_local_attention(a, max_q_len, form, dtype, stream);
}

extern "C" int semipd_window_attention(const void* q, int64_t q_ld, void* out, int64_t out_ld, const void* k_pool,
                                       const void* v_pool, const int32_t* req_to_token, int64_t req_to_token_stride,
                                       const int64_t* req_pool_indices, const int64_t* seq_lens, const int32_t* q_start,
                                       const int32_t* q_len, int64_t batch, int64_t num_tokens, int64_t max_q_len,
                                       int num_q_heads, int num_kv_heads, int qk_dim, int v_dim, float scale, int window,
                                       int keep_first, const float* head_bias, int sigmoid, const float* sink, float out_scale,
                                       int form, int dtype, void* stream) {
  SEMIPD_CHECK_ARG(window >= 0 && keep_first >= 0, SEMIPD_EINVAL, "window_attention: bad window or number of kept positions");
  SEMIPD_CHECK_ARG(window > 0 || keep_first == 0, SEMIPD_EINVAL, "window_attention: kept first positions need a window");
  SEMIPD_CHECK_ARG(!sigmoid || sink == nullptr, SEMIPD_EINVAL, "window_attention: sigmoid weights have no denominator for a sink");
  LocalAttnArgs a{q, q_ld, nullptr, 0, out, out_ld, k_pool, v_pool, req_to_token, req_to_token_stride, req_pool_indices,
                  seq_lens, q_start, q_len, batch, num_tokens, num_q_heads, num_kv_heads, qk_dim, v_dim, sink, scale, 0.f,
                  0, 0, window, keep_first, head_bias, sigmoid ? 1 : 0, out_scale};
  return launch_local_attention(a, max_q_len, form, dtype, stream);
}

static int launch_local_attention(LocalAttnArgs a, int64_t max_q_len, int form, int dtype, void* stream) {
  const void* q = a.q; const void* gate = a.gate; void* out = a.out; const void* k_pool = a.k_pool; const void* v_pool = a.v_pool;
  const int64_t q_ld = a.q_ld, gate_ld = a.gate_ld, out_ld = a.out_ld, batch = a.batch, num_tokens = a.num_tokens;
  const int32_t* q_start = a.q_start; const int32_t* q_len = a.q_len;
  const int num_q_heads = a.H, num_kv_heads = a.G, qk_dim = a.D, v_dim = a.E;
  SEMIPD_CHECK_ARG(batch >= 0 && num_tokens >= 0, SEMIPD_EINVAL, "local_attention: bad sizes");
  if (batch == 0 || num_tokens == 0) return 0;
  if (a.k_ld == 0) a.k_ld = (int64_t)num_kv_heads * qk_dim;
  if (a.v_ld == 0) a.v_ld = a.v_shared ? (int64_t)v_dim : (int64_t)num_kv_heads * v_dim;
  SEMIPD_CHECK_ARG(num_q_heads > 0 && num_kv_heads > 0 && num_q_heads % num_kv_heads == 0, SEMIPD_ESHAPE,
                   "local_attention: %d query heads over %d key/value heads", num_q_heads, num_kv_heads);
  SEMIPD_CHECK_ARG(qk_dim > 0 && qk_dim <= 1024 && v_dim > 0 && v_dim <= 1024, SEMIPD_ESHAPE,
                   "local_attention: head sizes %d / %d (at most 1024 / 1024)", qk_dim, v_dim);
  SEMIPD_CHECK_ARG(q && out && k_pool && v_pool && a.req_to_token && a.req_pool_indices && a.seq_lens, SEMIPD_EINVAL,
                   "local_attention: null pointer");
  SEMIPD_CHECK_ARG((q_start == nullptr) == (q_len == nullptr), SEMIPD_EINVAL, "local_attention: q_start and q_len come together");
  SEMIPD_CHECK_ARG(q_start != nullptr || num_tokens == batch, SEMIPD_EINVAL, "local_attention: one row per request without q_start");
  SEMIPD_CHECK_ARG(a.cap >= 0.f, SEMIPD_EINVAL, "local_attention: bad cap");
  const bool half = dtype == SEMIPD_BF16 || dtype == SEMIPD_F16;
  const bool mfma_ok = half && local_mfma_shape_ok(qk_dim, v_dim) && aligned16(q) && q_ld % 8 == 0 && aligned16(k_pool) &&
                       aligned16(v_pool) && a.k_ld % 8 == 0 && a.v_ld % 8 == 0 && aligned16(out) && out_ld % 8 == 0 &&
                       (gate == nullptr || (aligned16(gate) && gate_ld % 8 == 0));
  SEMIPD_CHECK_ARG(form != 2 || mfma_ok, SEMIPD_ESHAPE, "local_attention: the matrix-core forms do not take this shape or type");
  if (form != 1 && mfma_ok) {
    const bool small = qk_dim <= 128 && v_dim <= 128;
    const int tile = 32 * v_tile_row_bytes(v_dim);                       // at most 32 * 576 bytes: below the 64 KB default
    const bool sig = a.sigmoid != 0;
    if (q_start == nullptr || max_q_len <= 1) {
      const int n_splits = (a.n_splits > 1 && a.partial != nullptr) ? a.n_splits : 1;
      a.n_splits = n_splits;
      const dim3 grid((unsigned)batch, (unsigned)num_kv_heads, (unsigned)((num_q_heads / num_kv_heads + 15) / 16 * n_splits));
      const int merge = v_dim * 17 * 4;
      const int nw = small ? 8 : 4;
      const size_t lds = nw * (size_t)(tile > merge ? tile : merge);      // up to 80 KB: above the 64 KB default
      static std::atomic<uint64_t> done[8] = {};
      int rc = -1;
#define SEMIPD_LA_DEC(TT, NDD, NEE, NWW, SS, SLOT)                                                                              \
  do {                                                                                                                          \
    if (lds > 65536 && ensure_dynamic_lds((const void*)local_attention_decode_kernel<TT, NDD, NEE, NWW, SS>, lds, done[SLOT],  \
                                          "local_attention"))                                                                   \
      return SEMIPD_EINVAL;                                                                                                     \
    hipLaunchKernelGGL((local_attention_decode_kernel<TT, NDD, NEE, NWW, SS>), grid, dim3(64 * NWW), lds, as_stream(stream), a); \
    rc = 0;                                                                                                                     \
  } while (0)
      if (dtype == SEMIPD_BF16) {
        if (small && !sig) SEMIPD_LA_DEC(bf16_t, 4, 8, 8, false, 0);
        else if (small) SEMIPD_LA_DEC(bf16_t, 4, 8, 8, true, 1);
        else if (!sig) SEMIPD_LA_DEC(bf16_t, 8, 16, 4, false, 2);
        else SEMIPD_LA_DEC(bf16_t, 8, 16, 4, true, 3);
      } else {
        if (small && !sig) SEMIPD_LA_DEC(f16_t, 4, 8, 8, false, 4);
        else if (small) SEMIPD_LA_DEC(f16_t, 4, 8, 8, true, 5);
        else if (!sig) SEMIPD_LA_DEC(f16_t, 8, 16, 4, false, 6);
        else SEMIPD_LA_DEC(f16_t, 8, 16, 4, true, 7);
      }
#undef SEMIPD_LA_DEC
      (void)rc;
      if (n_splits > 1) {
        const dim3 mgrid((unsigned)batch, (unsigned)num_q_heads);
        if (dtype == SEMIPD_BF16) {
          if (sig) hipLaunchKernelGGL((local_attention_merge_kernel<bf16_t, true>), mgrid, dim3(64), 0, as_stream(stream), a);
          else hipLaunchKernelGGL((local_attention_merge_kernel<bf16_t, false>), mgrid, dim3(64), 0, as_stream(stream), a);
        } else {
          if (sig) hipLaunchKernelGGL((local_attention_merge_kernel<f16_t, true>), mgrid, dim3(64), 0, as_stream(stream), a);
          else hipLaunchKernelGGL((local_attention_merge_kernel<f16_t, false>), mgrid, dim3(64), 0, as_stream(stream), a);
        }
      }
      return launch_status("local_attention_decode");
    }
    a.n_tiles = (num_tokens + 63) / 64 + batch;
    const dim3 grid((unsigned)((a.n_tiles * num_q_heads + 7) / 8 * 8));
    const size_t tiles = 2 * ((size_t)tile + 32 * (size_t)(qk_dim * 2 + 32));   // two pairs of (32 V rows, 32 K rows): at most 71.7 KB
    static std::atomic<uint64_t> done_p[8] = {};
#define SEMIPD_LA_PRE(TT, NDD, NEE, SS, SLOT)                                                                                   \
  do {                                                                                                                          \
    if (tiles > 65536 && ensure_dynamic_lds((const void*)local_attention_mfma_kernel<TT, NDD, NEE, SS>, tiles, done_p[SLOT],    \
                                            "local_attention"))                                                                 \
      return SEMIPD_EINVAL;                                                                                                     \
    hipLaunchKernelGGL((local_attention_mfma_kernel<TT, NDD, NEE, SS>), grid, dim3(256), tiles, as_stream(stream), a);           \
  } while (0)
    if (dtype == SEMIPD_BF16) {
      if (small && !sig) SEMIPD_LA_PRE(bf16_t, 4, 8, false, 0);
      else if (small) SEMIPD_LA_PRE(bf16_t, 4, 8, true, 1);
      else if (!sig) SEMIPD_LA_PRE(bf16_t, 8, 16, false, 2);
      else SEMIPD_LA_PRE(bf16_t, 8, 16, true, 3);
    } else {
      if (small && !sig) SEMIPD_LA_PRE(f16_t, 4, 8, false, 4);
      else if (small) SEMIPD_LA_PRE(f16_t, 4, 8, true, 5);
      else if (!sig) SEMIPD_LA_PRE(f16_t, 8, 16, false, 6);
      else SEMIPD_LA_PRE(f16_t, 8, 16, true, 7);
    }
#undef SEMIPD_LA_PRE
    return launch_status("local_attention_mfma");
  }
  const dim3 grid((unsigned)((num_tokens + 3) / 4), (unsigned)num_q_heads);
  if (qk_dim <= 512 && v_dim <= 512) {
    SEMIPD_DISPATCH_DTYPE(dtype, T,
                          hipLaunchKernelGGL((local_attention_rows_kernel<T, 8>), grid, dim3(256), 0, as_stream(stream), a));
  } else {
    SEMIPD_DISPATCH_DTYPE(dtype, T,
                          hipLaunchKernelGGL((local_attention_rows_kernel<T, 16>), grid, dim3(256), 0, as_stream(stream), a));
  }
  return launch_status("local_attention");
}

extern "C" int semipd_latent_prep(const void* proj, int64_t ld, int64_t num_tokens, int num_heads, int dim, int rot_dim, int rank,
                                  const void* latent, int64_t latent_ld, int halves, const void* norm_weight, float eps,
                                  const int64_t* positions, const float* freq, int rot_dims, float mscale, void* pool,
                                  int64_t pool_ld, const int64_t* loc, void* q_out, int64_t q_ld, int q_head_stride, int q_head_off,
                                  int dtype, void* stream) {
  SEMIPD_CHECK_ARG(num_tokens >= 0 && num_heads > 0 && dim >= 0 && rot_dim >= 0 && rank > 0, SEMIPD_EINVAL, "latent_prep: bad sizes");
  if (num_tokens == 0) return 0;
  SEMIPD_CHECK_ARG(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= rot_dim, SEMIPD_ESHAPE,
                   "latent_prep: %d rotated elements of a part of %d", rot_dims, rot_dim);
  SEMIPD_CHECK_ARG(proj && latent && norm_weight && positions && pool && loc && q_out && (freq || rot_dims == 0), SEMIPD_EINVAL,
                   "latent_prep: null pointer");
  SEMIPD_CHECK_ARG(ld >= (int64_t)num_heads * (dim + rot_dim) && latent_ld >= rank + rot_dim && pool_ld >= rank + rot_dim &&
                       q_head_stride >= rot_dim && q_head_off >= 0 && q_head_off + rot_dim <= q_head_stride &&
                       q_ld >= (int64_t)num_heads * q_head_stride,
                   SEMIPD_EINVAL, "latent_prep: column ranges overlap or leave the row");
  SEMIPD_DISPATCH_DTYPE(dtype, T,
                        hipLaunchKernelGGL((latent_prep_kernel<T>), dim3((unsigned)num_tokens), dim3(256),
                                           (size_t)(rot_dims > 0 ? rot_dims : 2) * sizeof(float), as_stream(stream),
                                           (const T*)proj, ld, num_tokens, num_heads, dim, rot_dim, rank, (const T*)latent, latent_ld,
                                           halves, (const T*)norm_weight, eps, positions, freq, rot_dims, mscale, (T*)pool, pool_ld, loc, (T*)q_out, q_ld, q_head_stride,
                                           q_head_off));
  return launch_status("latent_prep");
}

// Attention of all heads over ONE row per token that holds the latent [R] and the shared rotated key part [P]: a head's query
// is [its unrotated part times its key up-projection | its rotated part] (R + P elements), the row is the key and its
// first R elements are the value -- the softmax-with-sink form of the kernels above with one key/value head whose values are
// a prefix of its keys.
extern "C" int semipd_latent_attention(const void* q, int64_t q_ld, void* out, int64_t out_ld, const void* pool, int64_t pool_ld,
                                       const int32_t* req_to_token, int64_t req_to_token_stride, const int64_t* req_pool_indices,
                                       const int64_t* seq_lens, const int32_t* q_start, const int32_t* q_len, int64_t batch,
                                       int64_t num_tokens, int64_t max_q_len, int num_heads, int rank, int rot_dim, float scale,
                                       const float* sink, int n_splits, float* partial, int form, int dtype, void* stream) {
  SEMIPD_CHECK_ARG(rank > 0 && rot_dim >= 0 && pool_ld >= rank + rot_dim, SEMIPD_EINVAL, "latent_attention: bad sizes");
  SEMIPD_CHECK_ARG(n_splits >= 0 && n_splits <= 64 && (n_splits <= 1 || partial != nullptr), SEMIPD_EINVAL,
                   "latent_attention: up to 64 slices of the keys, with room for their partial sums");
  LocalAttnArgs a{q, q_ld, nullptr, 0, out, out_ld, pool, pool, req_to_token, req_to_token_stride, req_pool_indices,
                  seq_lens, q_start, q_len, batch, num_tokens, num_heads, 1, rank + rot_dim, rank, sink, scale, 0.f,
                  0, 0, 0, 0, nullptr, 0, 1.0f, pool_ld, pool_ld, n_splits, partial};
  return launch_local_attention(a, max_q_len, form, dtype, stream);
}

extern "C" int semipd_local_attention_mfma_supported(int num_q_heads, int num_kv_heads, int qk_dim, int v_dim, int dtype) {
  return (dtype == SEMIPD_BF16 || dtype == SEMIPD_F16) && num_kv_heads > 0 && num_q_heads % num_kv_heads == 0 &&
         local_mfma_shape_ok(qk_dim, v_dim);
}

extern "C" int semipd_bias_rope_vnorm_kv_store(void* qkv, int64_t ld, int64_t num_tokens, int num_q_heads, int num_kv_heads,
                                               int qk_dim, int v_dim, int64_t k_off, int64_t v_off, const void* bias_q,
                                               const void* bias_k, const void* bias_v, const int64_t* positions,
                                               const float* inv_freq, int rot_dims, float eps, void* k_pool, void* v_pool,
                                               const int64_t* loc, int dtype, void* stream) {
  SEMIPD_CHECK_ARG(num_tokens >= 0 && num_q_heads > 0 && num_kv_heads > 0 && qk_dim > 0 && v_dim > 0 && v_dim <= 512, SEMIPD_EINVAL,
                   "bias_rope_vnorm_kv_store: bad sizes (value rows of at most 512 elements)");
  SEMIPD_CHECK_ARG(rot_dims >= 0 && rot_dims <= qk_dim && rot_dims % 2 == 0, SEMIPD_EINVAL,
                   "bias_rope_vnorm_kv_store: %d rotated elements of a head of %d", rot_dims, qk_dim);
  if (num_tokens == 0) return 0;
  SEMIPD_CHECK_ARG(qkv && k_pool && v_pool && loc && positions && (rot_dims == 0 || inv_freq), SEMIPD_EINVAL,
                   "bias_rope_vnorm_kv_store: null pointer");
  SEMIPD_CHECK_ARG(ld >= v_off + (int64_t)num_kv_heads * v_dim && k_off >= (int64_t)num_q_heads * qk_dim &&
                       v_off >= k_off + (int64_t)num_kv_heads * qk_dim,
                   SEMIPD_EINVAL, "bias_rope_vnorm_kv_store: column ranges overlap or leave the row");
  if ((dtype == SEMIPD_BF16 || dtype == SEMIPD_F16) && qk_dim % 8 == 0 && v_dim % 8 == 0 && rot_dims % 8 == 0 && rot_dims <= 512 &&
      ld % 8 == 0 && k_off % 8 == 0 && v_off % 8 == 0 && aligned16(qkv) && aligned16(k_pool) && aligned16(v_pool) &&
      (!bias_q || aligned16(bias_q)) && (!bias_k || aligned16(bias_k)) && (!bias_v || aligned16(bias_v))) {
    const unsigned vb = (unsigned)((num_tokens + 3) / 4);
    // about a thousand waves at least: the waves of a token split its heads' pieces
    const int64_t iters = ((int64_t)(num_q_heads + num_kv_heads) * (qk_dim / 8) + 63) / 64;
    int64_t parts = 1024 / (num_tokens < 1024 ? num_tokens : 1024);
    parts = parts < 1 ? 1 : (parts > iters ? iters : parts);
    SEMIPD_DISPATCH_HALF(dtype, T,
                         hipLaunchKernelGGL((bias_rope_vnorm_kv_store_vec_kernel<T>), dim3(vb, (unsigned)parts), dim3(256), 0, as_stream(stream),
                                            (T*)qkv, ld, num_tokens, num_q_heads, num_kv_heads, qk_dim, v_dim, k_off, v_off,
                                            (const T*)bias_q, (const T*)bias_k, (const T*)bias_v, positions, inv_freq, rot_dims,
                                            eps, (T*)k_pool, (T*)v_pool, loc));
    return launch_status("bias_rope_vnorm_kv_store");
  }
  const int64_t items = num_tokens * (num_q_heads + 2 * num_kv_heads);
  const unsigned blocks = (unsigned)((items + 3) / 4);
  SEMIPD_DISPATCH_DTYPE(dtype, T,
                        hipLaunchKernelGGL((bias_rope_vnorm_kv_store_kernel<T>), dim3(blocks), dim3(256), 0, as_stream(stream),
                                           (T*)qkv, ld, num_tokens, num_q_heads, num_kv_heads, qk_dim, v_dim, k_off, v_off,
                                           (const T*)bias_q, (const T*)bias_k, (const T*)bias_v, positions, inv_freq, rot_dims,
                                           eps, (T*)k_pool, (T*)v_pool, loc));
  return launch_status("bias_rope_vnorm_kv_store");
}


extern "C" int semipd_qk_norm_rope_kv_store(void* qkv, int64_t ld, int64_t num_tokens, int num_q_heads, int num_kv_heads, int qk_dim,
                                            int v_dim, int64_t k_off, int64_t v_off, const void* q_weight, const void* k_weight,
                                            float eps, const int64_t* positions, const float* freq, int rot_dims, int halves,
                                            float mscale, const float* head_scale, void* k_pool, void* v_pool,
                                            const int64_t* loc, int dtype, void* stream) {
  SEMIPD_CHECK_ARG(num_tokens >= 0 && num_q_heads > 0 && num_kv_heads > 0 && qk_dim > 0 && v_dim > 0, SEMIPD_EINVAL,
                   "qk_norm_rope_kv_store: bad sizes");
  if (num_tokens == 0) return 0;
  SEMIPD_CHECK_ARG(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= qk_dim, SEMIPD_ESHAPE,
                   "qk_norm_rope_kv_store: %d rotated elements of a head of %d", rot_dims, qk_dim);
  SEMIPD_CHECK_ARG(qkv && k_pool && v_pool && loc && positions && (rot_dims == 0 || freq), SEMIPD_EINVAL,
                   "qk_norm_rope_kv_store: null pointer");
  SEMIPD_CHECK_ARG(k_off >= (int64_t)num_q_heads * qk_dim && v_off >= k_off + (int64_t)num_kv_heads * qk_dim &&
                       ld >= v_off + (int64_t)num_kv_heads * v_dim,
                   SEMIPD_EINVAL, "qk_norm_rope_kv_store: column ranges overlap or leave the row");
  SEMIPD_DISPATCH_DTYPE(dtype, T,
                        hipLaunchKernelGGL((qk_norm_rope_kv_store_kernel<T>), dim3((unsigned)num_tokens), dim3(256),
                                           (size_t)(rot_dims > 0 ? rot_dims : 2) * sizeof(float), as_stream(stream), (T*)qkv, ld,
                                           num_q_heads, num_kv_heads, qk_dim, v_dim, k_off, v_off, (const T*)q_weight,
                                           (const T*)k_weight, eps, positions, freq, rot_dims, halves, mscale, head_scale, (T*)k_pool,
                                           (T*)v_pool, loc));
  return launch_status("qk_norm_rope_kv_store");
}

// Causal softmax attention in which every query head's weights are applied to the WHOLE value row of a slot (the values of
// all key/value heads side by side, v_row elements): out [T, heads * v_row].  Keys as in semipd_local_attention.
extern "C" int semipd_shared_value_attention(const void* q, int64_t q_ld, void* out, int64_t out_ld, const void* k_pool,
                                             const void* v_pool, const int32_t* req_to_token, int64_t req_to_token_stride,
                                             const int64_t* req_pool_indices, const int64_t* seq_lens, const int32_t* q_start,
                                             const int32_t* q_len, int64_t batch, int64_t num_tokens, int64_t max_q_len,
                                             int num_q_heads, int num_kv_heads, int qk_dim, int v_row, float scale, int n_splits,
                                             float* partial, int form, int dtype, void* stream) {
  SEMIPD_CHECK_ARG(n_splits >= 0 && n_splits <= 64 && (n_splits <= 1 || partial != nullptr), SEMIPD_EINVAL,
                   "shared_value_attention: up to 64 slices of the keys, with room for their partial sums");
  LocalAttnArgs a{q, q_ld, nullptr, 0, out, out_ld, k_pool, v_pool, req_to_token, req_to_token_stride, req_pool_indices,
                  seq_lens, q_start, q_len, batch, num_tokens, num_q_heads, num_kv_heads, qk_dim, v_row, nullptr, scale, 0.f,
                  0, 0, 0, 0, nullptr, 0, 1.0f, 0, 0, n_splits, partial, 1};
  return launch_local_attention(a, max_q_len, form, dtype, stream);
}

extern "C" int semipd_talk_mix(const void* parts, int64_t parts_ld, const float* talk, void* out, int64_t out_ld, int64_t num_tokens,
                               int num_q_heads, int num_kv_heads, int v_dim, int dtype, void* stream) {
  SEMIPD_CHECK_ARG(num_tokens >= 0 && num_q_heads > 0 && num_kv_heads > 0 && num_q_heads % num_kv_heads == 0 && v_dim > 0,
                   SEMIPD_EINVAL, "talk_mix: bad sizes");
  if (num_tokens == 0) return 0;
  SEMIPD_CHECK_ARG(parts && talk && out && parts_ld >= (int64_t)num_q_heads * num_kv_heads * v_dim &&
                       out_ld >= (int64_t)num_q_heads * v_dim,
                   SEMIPD_EINVAL, "talk_mix: null pointer or rows too short");
  const size_t staged = ((size_t)num_q_heads * num_q_heads + (size_t)num_q_heads * num_kv_heads * v_dim) * sizeof(float);
  SEMIPD_DISPATCH_DTYPE(dtype, T, {
    if (staged <= 65536)
      hipLaunchKernelGGL((talk_mix_kernel<T, true>), dim3((unsigned)num_tokens), dim3(256), staged, as_stream(stream),
                         (const T*)parts, parts_ld, talk, (T*)out, out_ld, num_q_heads, num_kv_heads, v_dim);
    else
      hipLaunchKernelGGL((talk_mix_kernel<T, false>), dim3((unsigned)num_tokens), dim3(256), 0, as_stream(stream),
                         (const T*)parts, parts_ld, talk, (T*)out, out_ld, num_q_heads, num_kv_heads, v_dim);
  });
  return launch_status("talk_mix");
}
