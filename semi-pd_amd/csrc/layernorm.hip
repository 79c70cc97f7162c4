// LayerNorm of post-norm residual blocks and the squared-ReLU activation (gfx950, wave64).
//
//  * layernorm_kernel: y = (x + in_bias - mean) / sqrt(var + eps) * w + b per row, var = mean of the squared deviations,
//    all in fp32.  With a residual stream (fp32, updated in place) the result is ADDED to it and the sum is what comes
//    out in the activation type: the block "x <- x + norm(sublayer(x))" between two GEMMs in one launch, the residual
//    never leaving fp32.  Input rows are of the activation type or fp32 (the final norm reads the stream itself).
//  * bias_relu_square_kernel: u <- max(u + b, 0)^2 in place.
//  * dyn_tanh_kernel: the element-wise squashing tanh(alpha x) * w + b that stands where a norm would (no row statistics),
//    fp32.  One launch is the seam between two sublayers of a block with a squashing before AND after each sublayer:
//    stream += dyn_tanh_a(sublayer output), then out = dyn_tanh_b(stream) for the next sublayer's GEMM; either half may
//    be left out (the first squashing of a model, the last one in front of the vocabulary head).
//  * routed_relu_square_kernel: experts evaluated side by side on every token (one GEMM over the stacked up-projections):
//    u[t, e * F + f] <- w(t, e) * max(u, 0)^2 with w the routing weight of expert e for token t, 0 when e is not one of the
//    token's experts, so that ONE GEMM over the stacked down-projections gives the weighted sum of the chosen experts.
#include "common.h"

namespace semipd {

template <typename T, typename TIn>
__global__ void __launch_bounds__(256) layernorm_kernel(const TIn* __restrict__ in, int64_t in_ld, const T* __restrict__ in_bias,
                                                        const T* __restrict__ w, const T* __restrict__ b, float eps,
                                                        float* __restrict__ residual, int64_t res_ld, T* __restrict__ out,
                                                        int64_t out_ld, int64_t width) {
  __shared__ float red[16];
  const int64_t r = blockIdx.x;
  const TIn* x = in + r * in_ld;
  auto at = [&](int64_t i) -> float {
    float v = Elem<TIn>::to_f(x[i]);
    if (in_bias) v += Elem<T>::to_f(in_bias[i]);
    return v;
  };
  float s = 0.f;
  for (int64_t i = threadIdx.x; i < width; i += 256) s += at(i);
  const float mean = block_sum(s, red) / (float)width;
  float q = 0.f;
  for (int64_t i = threadIdx.x; i < width; i += 256) {
    const float d = at(i) - mean;
    q += d * d;
  }
  __syncthreads();
  const float var = block_sum(q, red) / (float)width;
  const float rs = 1.0f / sqrtf(var + eps);
  for (int64_t i = threadIdx.x; i < width; i += 256) {
    float v = (at(i) - mean) * rs * Elem<T>::to_f(w[i]) + Elem<T>::to_f(b[i]);
    if (residual) {
      v += residual[r * res_ld + i];
      residual[r * res_ld + i] = v;
    }
    if (out) out[r * out_ld + i] = Elem<T>::from_f(v);
  }
}

// The same with the row held in registers: 16-byte loads, one pass over memory.  width % 8 == 0 (fp32 input: % 4 is
// implied), width <= 256 * 8 * NC; rows and pointers 16-byte aligned.
template <typename T, typename TIn, int NC>
__global__ void __launch_bounds__(256) layernorm_vec_kernel(const TIn* __restrict__ in, int64_t in_ld, const T* __restrict__ in_bias,
                                                            const T* __restrict__ w, const T* __restrict__ b, float eps,
                                                            float* __restrict__ residual, int64_t res_ld, T* __restrict__ out,
                                                            int64_t out_ld, int64_t width) {
  __shared__ float red[16];
  const int64_t r = blockIdx.x;
  const TIn* x = in + r * in_ld;
  float v[NC][8];
  float s = 0.f;
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int64_t i = ((int64_t)c * 256 + threadIdx.x) * 8;
    if (i < width) {
      if constexpr (sizeof(TIn) == 4) {
        const float4 a = *reinterpret_cast<const float4*>(x + i), d = *reinterpret_cast<const float4*>(x + i + 4);
        v[c][0] = a.x; v[c][1] = a.y; v[c][2] = a.z; v[c][3] = a.w; v[c][4] = d.x; v[c][5] = d.y; v[c][6] = d.z; v[c][7] = d.w;
      } else {
        const Vec16<TIn> a = load16(x + i);
#pragma unroll
        for (int u = 0; u < 8; ++u) v[c][u] = Elem<TIn>::to_f(a.e[u]);
      }
      if (in_bias) {
        if constexpr (sizeof(T) == 2) {
          const Vec16<T> a = load16(in_bias + i);
#pragma unroll
          for (int u = 0; u < 8; ++u) v[c][u] += Elem<T>::to_f(a.e[u]);
        } else {
#pragma unroll
          for (int u = 0; u < 8; ++u) v[c][u] += Elem<T>::to_f(in_bias[i + u]);
        }
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) s += v[c][u];
    }
  }
  const float mean = block_sum(s, red) / (float)width;
  float q = 0.f;
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int64_t i = ((int64_t)c * 256 + threadIdx.x) * 8;
    if (i < width) {
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const float d = v[c][u] - mean;
        q += d * d;
      }
    }
  }
  __syncthreads();
  const float var = block_sum(q, red) / (float)width;
  const float rs = 1.0f / sqrtf(var + eps);
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int64_t i = ((int64_t)c * 256 + threadIdx.x) * 8;
    if (i < width) {
      float y[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) y[u] = (v[c][u] - mean) * rs * Elem<T>::to_f(w[i + u]) + Elem<T>::to_f(b[i + u]);
      if (residual) {
        float* rp = residual + r * res_ld + i;
        float4 a = *reinterpret_cast<float4*>(rp), d = *reinterpret_cast<float4*>(rp + 4);
        y[0] += a.x; y[1] += a.y; y[2] += a.z; y[3] += a.w; y[4] += d.x; y[5] += d.y; y[6] += d.z; y[7] += d.w;
        a = float4{y[0], y[1], y[2], y[3]};
        d = float4{y[4], y[5], y[6], y[7]};
        *reinterpret_cast<float4*>(rp) = a;
        *reinterpret_cast<float4*>(rp + 4) = d;
      }
      if (out) {
        T* op = out + r * out_ld + i;
        if constexpr (sizeof(T) == 2) {
          Vec16<T> o;
#pragma unroll
          for (int u = 0; u < 8; ++u) o.e[u] = Elem<T>::from_f(y[u]);
          store16(op, o);
        } else {
#pragma unroll
          for (int u = 0; u < 8; ++u) op[u] = Elem<T>::from_f(y[u]);
        }
      }
    }
  }
}

// 8 elements per thread and step, 16-byte accesses (width % 8 == 0, rows 16-byte aligned); a workgroup walks whole rows
template <typename T>
__global__ void __launch_bounds__(256) bias_relu_square_vec_kernel(T* __restrict__ u, int64_t ld, const T* __restrict__ bias,
                                                                   int64_t rows, int64_t width) {
  for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
    for (int64_t c = (int64_t)threadIdx.x * 8; c < width; c += (int64_t)blockDim.x * 8) {
      T* p = u + r * ld + c;
      float v[8];
      if constexpr (sizeof(T) == 2) {
        const Vec16<T> a = load16(p);
#pragma unroll
        for (int k = 0; k < 8; ++k) v[k] = Elem<T>::to_f(a.e[k]);
      } else {
#pragma unroll
        for (int k = 0; k < 8; ++k) v[k] = Elem<T>::to_f(p[k]);
      }
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        if (bias) v[k] += Elem<T>::to_f(bias[c + k]);
        v[k] = v[k] > 0.f ? v[k] * v[k] : 0.f;
      }
      if constexpr (sizeof(T) == 2) {
        Vec16<T> o;
#pragma unroll
        for (int k = 0; k < 8; ++k) o.e[k] = Elem<T>::from_f(v[k]);
        store16(p, o);
      } else {
#pragma unroll
        for (int k = 0; k < 8; ++k) p[k] = Elem<T>::from_f(v[k]);
      }
    }
  }
}

template <typename T>
__global__ void __launch_bounds__(256) bias_relu_square_kernel(T* __restrict__ u, int64_t ld, const T* __restrict__ bias,
                                                               int64_t rows, int64_t width) {
  const int64_t n = rows * width;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / width, c = i - r * width;
    float v = Elem<T>::to_f(u[r * ld + c]);
    if (bias) v += Elem<T>::to_f(bias[c]);
    v = v > 0.f ? v * v : 0.f;
    u[r * ld + c] = Elem<T>::from_f(v);
  }
}


// ------------------------------------------------------------------------------------------------ dynamic tanh
// tanh in fp32 from one v_exp_f32 and one v_rcp_f32: 1 - 2 / (exp(2 |a|) + 1) with the sign put back (overflow of the
// exponential gives 1).  That difference cancels for small |a| (its absolute error stays near 1e-7), so below |a| = 0.1 the odd
// series a (1 - a^2 / 3 + 2 a^4 / 15 - 17 a^6 / 315) takes over (its next term is below 3e-10 relative there): the relative
// error is at most ~1e-6, at the switch.  A fraction of tanhf's instructions: the kernel has two of them per element and is
// otherwise bound by memory.
__device__ __forceinline__ float tanh_fast(float a) {
  const float x = fabsf(a);
  const float e = __builtin_amdgcn_exp2f(x * 2.8853900817779268f);          // exp(2 x)
  const float big = 1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f);
  const float a2 = a * a;
  const float small = x * (1.0f + a2 * (-0.33333333333f + a2 * (0.13333333333f - a2 * 0.05396825397f)));
  return copysignf(x < 0.1f ? small : big, a);
}

// A workgroup per row; V elements per thread and step (V = 8: 16-byte accesses on 16-bit rows; V = 1: any width and alignment)
template <typename T, typename TIn, int V>
__global__ void __launch_bounds__(256) dyn_tanh_kernel(const TIn* __restrict__ y, int64_t y_ld, const T* __restrict__ wa,
                                                       const T* __restrict__ ba, const T* __restrict__ alpha_a,
                                                       float* __restrict__ residual, int64_t res_ld, int accumulate,
                                                       const T* __restrict__ wb, const T* __restrict__ bb,
                                                       const T* __restrict__ alpha_b, T* __restrict__ out, int64_t out_ld,
                                                       int64_t rows, int64_t width) {
  const float aa = alpha_a ? Elem<T>::to_f(alpha_a[0]) : 0.f, ab = alpha_b ? Elem<T>::to_f(alpha_b[0]) : 0.f;
  for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
    for (int64_t c = (int64_t)threadIdx.x * V; c < width; c += (int64_t)blockDim.x * V) {
      float v[V];
#pragma unroll
      for (int k = 0; k < V; ++k) v[k] = 0.f;
      if (y) {
        float w[V], b[V];
        if constexpr (V == 8 && sizeof(TIn) == 2) {
          const Vec16<TIn> a = load16(y + r * y_ld + c);
#pragma unroll
          for (int k = 0; k < V; ++k) v[k] = Elem<TIn>::to_f(a.e[k]);
        } else {
#pragma unroll
          for (int k = 0; k < V; ++k) v[k] = Elem<TIn>::to_f(y[r * y_ld + c + k]);
        }
        if constexpr (V == 8 && sizeof(T) == 2) {
          const Vec16<T> w8 = load16(wa + c), b8 = load16(ba + c);
#pragma unroll
          for (int k = 0; k < V; ++k) {
            w[k] = Elem<T>::to_f(w8.e[k]);
            b[k] = Elem<T>::to_f(b8.e[k]);
          }
        } else {
#pragma unroll
          for (int k = 0; k < V; ++k) {
            w[k] = Elem<T>::to_f(wa[c + k]);
            b[k] = Elem<T>::to_f(ba[c + k]);
          }
        }
#pragma unroll
        for (int k = 0; k < V; ++k) v[k] = tanh_fast(aa * v[k]) * w[k] + b[k];
      }
      if (residual) {
        float* rp = residual + r * res_ld + c;
        if (accumulate || !y) {
          if constexpr (V == 8) {
            const float4 a = *reinterpret_cast<const float4*>(rp), d = *reinterpret_cast<const float4*>(rp + 4);
            v[0] += a.x; v[1] += a.y; v[2] += a.z; v[3] += a.w; v[4] += d.x; v[5] += d.y; v[6] += d.z; v[7] += d.w;
          } else {
#pragma unroll
            for (int k = 0; k < V; ++k) v[k] += rp[k];
          }
        }
        if (y) {
          if constexpr (V == 8) {
            *reinterpret_cast<float4*>(rp) = float4{v[0], v[1], v[2], v[3]};
            *reinterpret_cast<float4*>(rp + 4) = float4{v[4], v[5], v[6], v[7]};
          } else {
#pragma unroll
            for (int k = 0; k < V; ++k) rp[k] = v[k];
          }
        }
      }
      if (out) {
        if (wb) {
#pragma unroll
          for (int k = 0; k < V; ++k) v[k] = tanh_fast(ab * v[k]) * Elem<T>::to_f(wb[c + k]) + Elem<T>::to_f(bb[c + k]);
        }
        T* op = out + r * out_ld + c;
        if constexpr (V == 8 && sizeof(T) == 2) {
          Vec16<T> o;
#pragma unroll
          for (int k = 0; k < V; ++k) o.e[k] = Elem<T>::from_f(v[k]);
          store16(op, o);
        } else {
#pragma unroll
          for (int k = 0; k < V; ++k) op[k] = Elem<T>::from_f(v[k]);
        }
      }
    }
  }
}

// one thread per element of u [rows, experts * ff]
template <typename T>
__global__ void __launch_bounds__(256) routed_relu_square_kernel(T* __restrict__ u, int64_t ld, const float* __restrict__ topk_weights,
                                                                 const int32_t* __restrict__ topk_ids, int topk, int64_t rows,
                                                                 int64_t ff, int experts) {
  const int64_t width = ff * experts, n = rows * width;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / width, c = i - r * width;
    const int e = (int)(c / ff);
    float wgt = 0.f;
    for (int k = 0; k < topk; ++k)
      if (topk_ids[r * topk + k] == e) wgt = topk_weights[r * topk + k];
    float v = Elem<T>::to_f(u[r * ld + c]);
    v = v > 0.f ? v * v * wgt : 0.f;
    u[r * ld + c] = Elem<T>::from_f(v);
  }
}


// ---- RMS norm around an fp32 residual stream: stream (+)= y;  out = stream / sqrt(mean(stream^2) + eps) * (weight + shift)
// (shift 1: a weight stored around zero).  A workgroup per row; the row is summed while it is updated and read once more.
template <typename T, typename TIn>
__global__ void __launch_bounds__(256) rms_stream_kernel(const TIn* __restrict__ y, int64_t y_ld, float* __restrict__ stream,
                                                         int64_t s_ld, const T* __restrict__ w, float shift, float eps,
                                                         T* __restrict__ out, int64_t out_ld, int64_t width) {
  __shared__ float red[16];
  const int64_t r = blockIdx.x;
  float* x = stream + r * s_ld;
  float q = 0.f;
  for (int64_t i = threadIdx.x; i < width; i += 256) {
    float v = x[i];
    if (y) {
      v += Elem<TIn>::to_f(y[r * y_ld + i]);
      x[i] = v;
    }
    q += v * v;
  }
  if (!out) return;
  const float rs = 1.0f / sqrtf(block_sum(q, red) / (float)width + eps);
  for (int64_t i = threadIdx.x; i < width; i += 256)           // (every thread re-reads the elements it wrote itself)
    out[r * out_ld + i] = Elem<T>::from_f(x[i] * rs * (Elem<T>::to_f(w[i]) + shift));
}

// ---- token embedding times a scale plus a row of a hashed bigram table, into the fp32 stream.  The previous token of a
// row that starts its request's portion is the request's entry of `prev` (an int32 column of the state rows); the first
// token of a sequence takes the table's last row.  The block of a portion's first row also leaves the portion's last token there.
template <typename T>
__global__ void __launch_bounds__(256) embed_bigram_kernel(const int64_t* __restrict__ ids, const T* __restrict__ embed,
                                                           const T* __restrict__ bigram, float scale, int64_t mul_prev,
                                                           int64_t mul_cur, int64_t buckets, int32_t* prev, int64_t prev_ld,
                                                           const int64_t* __restrict__ state_indices,
                                                           const int64_t* __restrict__ seq_lens, const int32_t* __restrict__ q_start,
                                                           const int32_t* __restrict__ q_len, int64_t batch, float* __restrict__ out,
                                                           int64_t width) {
  __shared__ int64_t row_s;
  const int64_t t = blockIdx.x;
  if (threadIdx.x == 0) {
    int b = -1;
    int64_t li = 0, n = 1, first_pos = 0;
    if (q_start == nullptr) {
      b = (int)t;
      first_pos = seq_lens[b] - 1;
    } else {
      for (int r = 0; r < (int)batch; ++r)
        if (t >= q_start[r] && t < (int64_t)q_start[r] + q_len[r]) {
          b = r; li = t - q_start[r]; n = q_len[r]; first_pos = seq_lens[r] - n;
        }
    }
    const int64_t tok = ids[t];
    int64_t row = buckets;
    if (b >= 0) {
      int32_t* slot = prev + state_indices[b] * prev_ld;
      if (first_pos + li > 0) {
        const int64_t before = li > 0 ? ids[t - 1] : (int64_t)*slot;
        row = (before * mul_prev + tok * mul_cur) % buckets;
      }
      if (li == 0) *slot = (int32_t)ids[t + n - 1];
    }
    row_s = row;
  }
  __syncthreads();
  const T* e = embed + ids[t] * width;
  const T* g = bigram + row_s * width;
  for (int64_t i = threadIdx.x; i < width; i += 256) out[t * width + i] = Elem<T>::to_f(e[i]) * scale + Elem<T>::to_f(g[i]);
}

// ---- gated activation with clamps: rows of `groups` x [gate F | up F] -> rows of `groups` x F,
//     a = min(gate, limit), b = clamp(up, -limit, limit), y = a * sigmoid(alpha a) * (b + 1)
// times, when routing is given, the routing weight of the group's expert for the row's token (0 if not chosen).
template <typename T>
__global__ void __launch_bounds__(256) clamped_glu_kernel(const T* __restrict__ x, int64_t x_ld, T* __restrict__ out, int64_t out_ld,
                                                          int64_t rows, int64_t ff, int groups, const float* __restrict__ topk_weights,
                                                          const int32_t* __restrict__ topk_ids, int topk, float limit, float alpha) {
  const int64_t width = ff * groups, n = rows * width;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / width, c = i - r * width;
    const int e = (int)(c / ff);
    const int64_t f = c - (int64_t)e * ff;
    float wgt = 1.f;
    if (topk_ids) {
      wgt = 0.f;
      for (int k = 0; k < topk; ++k)
        if (topk_ids[r * topk + k] == e) wgt = topk_weights[r * topk + k];
    }
    const T* row = x + r * x_ld + (int64_t)e * 2 * ff;
    const float a = fminf(Elem<T>::to_f(row[f]), limit);
    const float b = fminf(fmaxf(Elem<T>::to_f(row[ff + f]), -limit), limit);
    out[r * out_ld + c] = Elem<T>::from_f(a / (1.0f + expf(-alpha * a)) * (b + 1.0f) * wgt);
  }
}


// ---- x <- x * sigmoid(gate), element by element in fp32 (rows of one type, any row strides)
template <typename T>
__global__ void __launch_bounds__(256) sigmoid_gate_kernel(T* __restrict__ x, int64_t x_ld, const T* __restrict__ gate, int64_t gate_ld,
                                                           int64_t rows, int64_t width) {
  const int64_t n = rows * width;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / width, c = i - r * width;
    const float g = Elem<T>::to_f(gate[r * gate_ld + c]);
    x[r * x_ld + c] = Elem<T>::from_f(Elem<T>::to_f(x[r * x_ld + c]) / (1.0f + expf(-g)));
  }
}

// ---- x <- x * sigmoid(gate[head]): one gate per (row, head) over the head's `head_width` elements, fp32 arithmetic
template <typename T>
__global__ void __launch_bounds__(256) sigmoid_gate_heads_kernel(T* __restrict__ x, int64_t x_ld, const T* __restrict__ gate,
                                                                 int64_t gate_ld, int64_t rows, int64_t heads, int64_t head_width) {
  const int64_t width = heads * head_width, n = rows * width;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / width, c = i - r * width;
    const float g = Elem<T>::to_f(gate[r * gate_ld + c / head_width]);
    x[r * x_ld + c] = Elem<T>::from_f(Elem<T>::to_f(x[r * x_ld + c]) / (1.0f + expf(-g)));
  }
}

// ---- token embedding times a scale as the start of an fp32 stream
template <typename T>
__global__ void __launch_bounds__(256) embed_stream_kernel(const int64_t* __restrict__ ids, const T* __restrict__ embed, float scale,
                                                           float* __restrict__ out, int64_t width) {
  const int64_t t = blockIdx.x;
  const T* e = embed + ids[t] * width;
  for (int64_t i = threadIdx.x; i < width; i += 256) out[t * width + i] = Elem<T>::to_f(e[i]) * scale;
}

// The request that owns row t of a batch, the row's index in the request's portion, the portion's length and the position
// of its first row (q_start == NULL: row t is request t's newest token).
__device__ __forceinline__ bool portion_of_row(int64_t t, int64_t batch, const int64_t* seq_lens, const int32_t* q_start,
                                               const int32_t* q_len, int& b, int64_t& li, int64_t& n, int64_t& first_pos) {
  if (q_start == nullptr) {
    b = (int)t; li = 0; n = 1; first_pos = seq_lens[b] - 1;
    return first_pos >= 0;
  }
  for (int r = 0; r < (int)batch; ++r) {
    const int64_t s = q_start[r], m = q_len[r];
    if (t >= s && t < s + m) {
      b = r; li = t - s; n = m; first_pos = seq_lens[r] - m;
      return true;
    }
  }
  return false;
}

// ---- norm AFTER the sum on an fp32 stream, with a per-channel scale on the sublayer's result:
//     stream <- (alpha stream + ls * y) / sqrt(mean((alpha stream + ls * y)^2) + eps) * weight          (fp32, in place)
// and, when `out` is given, what the next sublayer reads, in the activation type: the new stream itself, or -- with `mu` --
// the token-shifted stream  s + (s_prev - s) * mu,  s_prev the previous token's new stream.  The shifted form is for
// batches of ONE row per request (q_start == NULL): s_prev is the request's entry of `prev` (zeros at position 0), which
// the row then replaces by its own stream.  A workgroup per row.
template <typename T>
__global__ void __launch_bounds__(256) postnorm_stream_kernel(const T* __restrict__ y, int64_t y_ld, const T* __restrict__ ls,
                                                              float* __restrict__ stream, int64_t s_ld, float alpha,
                                                              const T* __restrict__ w, float eps, T* __restrict__ out, int64_t out_ld,
                                                              const T* __restrict__ mu, float* __restrict__ prev, int64_t prev_ld,
                                                              const int64_t* __restrict__ state_indices,
                                                              const int64_t* __restrict__ seq_lens, int64_t width) {
  __shared__ float red[16];
  const int64_t r = blockIdx.x;
  float* x = stream + r * s_ld;
  float q = 0.f;
  for (int64_t i = threadIdx.x; i < width; i += 256) {
    float v = alpha * x[i];
    if (y) v += Elem<T>::to_f(y[r * y_ld + i]) * (ls ? Elem<T>::to_f(ls[i]) : 1.0f);
    x[i] = v;
    q += v * v;
  }
  const float rs = 1.0f / sqrtf(block_sum(q, red) / (float)width + eps);
  float* pv = nullptr;
  bool first = true;
  if (mu) {
    pv = prev + state_indices[r] * prev_ld;
    first = seq_lens[r] <= 1;
  }
  for (int64_t i = threadIdx.x; i < width; i += 256) {          // (every thread re-reads the elements it wrote itself)
    const float v = x[i] * rs * Elem<T>::to_f(w[i]);
    x[i] = v;
    if (!out) continue;
    if (mu) {
      const float before = first ? 0.f : pv[i];
      pv[i] = v;
      out[r * out_ld + i] = Elem<T>::from_f(v + (before - v) * Elem<T>::to_f(mu[i]));
    } else {
      out[r * out_ld + i] = Elem<T>::from_f(v);
    }
  }
}

// ---- token shift on an fp32 stream: out[t] = s_t + (s_(t-1) - s_t) * mu in the activation type, s_(t-1) the previous row of
// the request's portion, for the portion's first row the request's entry of `prev` (zeros at position 0).  The workgroup of
// a portion's first row also leaves the portion's LAST row in `prev`, element by element behind its own read.
template <typename T>
__global__ void __launch_bounds__(256) token_shift_kernel(const float* __restrict__ stream, int64_t s_ld, const T* __restrict__ mu,
                                                          float* __restrict__ prev, int64_t prev_ld,
                                                          const int64_t* __restrict__ state_indices,
                                                          const int64_t* __restrict__ seq_lens, const int32_t* __restrict__ q_start,
                                                          const int32_t* __restrict__ q_len, int64_t batch, T* __restrict__ out,
                                                          int64_t out_ld, int64_t width) {
  const int64_t t = blockIdx.x;
  int b;
  int64_t li, n, first_pos;
  if (!portion_of_row(t, batch, seq_lens, q_start, q_len, b, li, n, first_pos)) return;
  const float* x = stream + t * s_ld;
  if (li > 0) {
    const float* xp = stream + (t - 1) * s_ld;
    for (int64_t i = threadIdx.x; i < width; i += 256)
      out[t * out_ld + i] = Elem<T>::from_f(x[i] + (xp[i] - x[i]) * Elem<T>::to_f(mu[i]));
    return;
  }
  float* pv = prev + state_indices[b] * prev_ld;
  const float* last = stream + (t + n - 1) * s_ld;
  for (int64_t i = threadIdx.x; i < width; i += 256) {
    const float before = first_pos == 0 ? 0.f : pv[i];
    pv[i] = last[i];
    out[t * out_ld + i] = Elem<T>::from_f(x[i] + (before - x[i]) * Elem<T>::to_f(mu[i]));
  }
}

}  // namespace semipd

using namespace semipd;

extern "C" int semipd_layernorm(const void* in, int64_t in_ld, int in_is_f32, const void* in_bias, const void* weight,
                                const void* bias, float eps, float* residual, int64_t residual_ld, void* out, int64_t out_ld,
                                int64_t rows, int64_t width, int dtype, void* stream) {
  SEMIPD_CHECK_ARG(rows >= 0 && width > 0, SEMIPD_EINVAL, "layernorm: bad sizes");
  if (rows == 0) return 0;
  SEMIPD_CHECK_ARG(in && weight && bias && (residual || out), SEMIPD_EINVAL, "layernorm: null pointer");
  const int64_t esz = dtype == SEMIPD_F32 ? 4 : 2, in_esz = in_is_f32 ? 4 : esz;
  const bool vec = width % 8 == 0 && width <= 256 * 8 * 4 && aligned16(in) && (in_ld * in_esz) % 16 == 0 &&
                   (!in_bias || aligned16(in_bias)) && (!residual || (aligned16(residual) && residual_ld % 4 == 0)) &&
                   (!out || (aligned16(out) && (out_ld * esz) % 16 == 0));
  if (vec) {
    const bool two = width <= 256 * 8 * 2;
    SEMIPD_DISPATCH_DTYPE(dtype, T, {
      if (in_is_f32 && two)
        hipLaunchKernelGGL((layernorm_vec_kernel<T, float, 2>), dim3((unsigned)rows), dim3(256), 0, as_stream(stream),
                           (const float*)in, in_ld, (const T*)in_bias, (const T*)weight, (const T*)bias, eps, residual, residual_ld,
                           (T*)out, out_ld, width);
      else if (in_is_f32)
        hipLaunchKernelGGL((layernorm_vec_kernel<T, float, 4>), dim3((unsigned)rows), dim3(256), 0, as_stream(stream),
                           (const float*)in, in_ld, (const T*)in_bias, (const T*)weight, (const T*)bias, eps, residual, residual_ld,
                           (T*)out, out_ld, width);
      else if (two)
        hipLaunchKernelGGL((layernorm_vec_kernel<T, T, 2>), dim3((unsigned)rows), dim3(256), 0, as_stream(stream), (const T*)in,
                           in_ld, (const T*)in_bias, (const T*)weight, (const T*)bias, eps, residual, residual_ld, (T*)out, out_ld,
                           width);
      else
        hipLaunchKernelGGL((layernorm_vec_kernel<T, T, 4>), dim3((unsigned)rows), dim3(256), 0, as_stream(stream), (const T*)in,
                           in_ld, (const T*)in_bias, (const T*)weight, (const T*)bias, eps, residual, residual_ld, (T*)out, out_ld,
                           width);
    });
    return launch_status("layernorm");
  }
  SEMIPD_DISPATCH_DTYPE(dtype, T, {
    if (in_is_f32)
      hipLaunchKernelGGL((layernorm_kernel<T, float>), dim3((unsigned)rows), dim3(256), 0, as_stream(stream), (const float*)in,
                         in_ld, (const T*)in_bias, (const T*)weight, (const T*)bias, eps, residual, residual_ld, (T*)out, out_ld,
                         width);
    else
      hipLaunchKernelGGL((layernorm_kernel<T, T>), dim3((unsigned)rows), dim3(256), 0, as_stream(stream), (const T*)in, in_ld,
                         (const T*)in_bias, (const T*)weight, (const T*)bias, eps, residual, residual_ld, (T*)out, out_ld, width);
  });
  return launch_status("layernorm");
}

extern "C" int semipd_bias_relu_square(void* u, int64_t ld, const void* bias, int64_t rows, int64_t width, int dtype,
                                       void* stream) {
  SEMIPD_CHECK_ARG(rows >= 0 && width > 0 && ld >= width, SEMIPD_EINVAL, "bias_relu_square: bad sizes");
  if (rows == 0) return 0;
  SEMIPD_CHECK_ARG(u, SEMIPD_EINVAL, "bias_relu_square: null pointer");
  const int64_t n = rows * width;
  const int64_t esz = dtype == SEMIPD_F32 ? 4 : 2;
  if (width % 8 == 0 && aligned16(u) && (ld * esz) % 16 == 0) {
    const unsigned vblocks = (unsigned)(rows < (1 << 20) ? rows : (1 << 20));
    const unsigned threads = (unsigned)(width / 8 >= 256 ? 256 : (width / 8 + 63) / 64 * 64);
    SEMIPD_DISPATCH_DTYPE(dtype, T,
                          hipLaunchKernelGGL((bias_relu_square_vec_kernel<T>), dim3(vblocks), dim3(threads), 0, as_stream(stream),
                                             (T*)u, ld, (const T*)bias, rows, width));
    return launch_status("bias_relu_square");
  }
  const unsigned blocks = (unsigned)((n + 255) / 256 < 8192 ? (n + 255) / 256 : 8192);
  SEMIPD_DISPATCH_DTYPE(dtype, T,
                        hipLaunchKernelGGL((bias_relu_square_kernel<T>), dim3(blocks), dim3(256), 0, as_stream(stream), (T*)u, ld,
                                           (const T*)bias, rows, width));
  return launch_status("bias_relu_square");
}

extern "C" int semipd_dyn_tanh(const void* in, int64_t in_ld, int in_is_f32, const void* weight_a, const void* bias_a,
                               const void* alpha_a, float* residual, int64_t residual_ld, int accumulate, const void* weight_b,
                               const void* bias_b, const void* alpha_b, void* out, int64_t out_ld, int64_t rows, int64_t width,
                               int dtype, void* stream) {
  SEMIPD_CHECK_ARG(rows >= 0 && width > 0, SEMIPD_EINVAL, "dyn_tanh: bad sizes");
  if (rows == 0) return 0;
  SEMIPD_CHECK_ARG((in || residual) && (residual || out), SEMIPD_EINVAL, "dyn_tanh: nothing to read or nothing to write");
  SEMIPD_CHECK_ARG(!in || (weight_a && bias_a && alpha_a), SEMIPD_EINVAL, "dyn_tanh: the input's weight, bias and alpha come together");
  SEMIPD_CHECK_ARG((weight_b == nullptr) == (bias_b == nullptr) && (weight_b == nullptr) == (alpha_b == nullptr), SEMIPD_EINVAL,
                   "dyn_tanh: the output's weight, bias and alpha come together");
  SEMIPD_CHECK_ARG(!weight_b || out, SEMIPD_EINVAL, "dyn_tanh: output parameters without an output");
  const int64_t esz = dtype == SEMIPD_F32 ? 4 : 2, in_esz = in_is_f32 ? 4 : esz;
  const bool vec = width % 8 == 0 && (!in || (aligned16(in) && (in_ld * in_esz) % 16 == 0 && aligned16(weight_a) && aligned16(bias_a))) &&
                   (!residual || (aligned16(residual) && residual_ld % 4 == 0)) && (!out || (aligned16(out) && (out_ld * esz) % 16 == 0));
  const unsigned blocks = (unsigned)(rows < (1 << 20) ? rows : (1 << 20));
  // (narrow rows: as many waves as the row has work for)
  const int64_t per_row = (width + (vec ? 8 : 1) - 1) / (vec ? 8 : 1);
  const unsigned threads = (unsigned)(per_row >= 256 ? 256 : (per_row + 63) / 64 * 64);
#define SEMIPD_DYT(TIN, VV)                                                                                                     \
  hipLaunchKernelGGL((dyn_tanh_kernel<T, TIN, VV>), dim3(blocks), dim3(threads), 0, as_stream(stream), (const TIN*)in, in_ld,          \
                     (const T*)weight_a, (const T*)bias_a, (const T*)alpha_a, residual, residual_ld, accumulate,                 \
                     (const T*)weight_b, (const T*)bias_b, (const T*)alpha_b, (T*)out, out_ld, rows, width)
  SEMIPD_DISPATCH_DTYPE(dtype, T, {
    if (in_is_f32 && vec) SEMIPD_DYT(float, 8);
    else if (in_is_f32) SEMIPD_DYT(float, 1);
    else if (vec) SEMIPD_DYT(T, 8);
    else SEMIPD_DYT(T, 1);
  });
#undef SEMIPD_DYT
  return launch_status("dyn_tanh");
}

extern "C" int semipd_routed_relu_square(void* u, int64_t ld, const float* topk_weights, const int32_t* topk_ids, int topk,
                                         int64_t rows, int64_t ff, int experts, int dtype, void* stream) {
  SEMIPD_CHECK_ARG(rows >= 0 && ff > 0 && experts > 0 && topk > 0 && topk <= experts && ld >= ff * experts, SEMIPD_EINVAL,
                   "routed_relu_square: bad sizes");
  if (rows == 0) return 0;
  SEMIPD_CHECK_ARG(u && topk_weights && topk_ids, SEMIPD_EINVAL, "routed_relu_square: null pointer");
  const int64_t n = rows * ff * experts;
  const unsigned blocks = (unsigned)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
  SEMIPD_DISPATCH_DTYPE(dtype, T,
                        hipLaunchKernelGGL((routed_relu_square_kernel<T>), dim3(blocks), dim3(256), 0, as_stream(stream), (T*)u,
                                           ld, topk_weights, topk_ids, topk, rows, ff, experts));
  return launch_status("routed_relu_square");
}


extern "C" int semipd_rms_stream(const void* y, int64_t y_ld, int y_is_f32, float* stream, int64_t stream_ld, const void* weight,
                                 float weight_shift, float eps, void* out, int64_t out_ld, int64_t rows, int64_t width, int dtype,
                                 void* stream_handle) {
  SEMIPD_CHECK_ARG(rows >= 0 && width > 0, SEMIPD_EINVAL, "rms_stream: bad sizes");
  if (rows == 0) return 0;
  SEMIPD_CHECK_ARG(stream && (y || out) && (!out || weight), SEMIPD_EINVAL, "rms_stream: null pointer");
  SEMIPD_DISPATCH_DTYPE(dtype, T, {
    if (y_is_f32)
      hipLaunchKernelGGL((rms_stream_kernel<T, float>), dim3((unsigned)rows), dim3(256), 0, as_stream(stream_handle),
                         (const float*)y, y_ld, stream, stream_ld, (const T*)weight, weight_shift, eps, (T*)out, out_ld, width);
    else
      hipLaunchKernelGGL((rms_stream_kernel<T, T>), dim3((unsigned)rows), dim3(256), 0, as_stream(stream_handle), (const T*)y, y_ld,
                         stream, stream_ld, (const T*)weight, weight_shift, eps, (T*)out, out_ld, width);
  });
  return launch_status("rms_stream");
}

extern "C" int semipd_embed_bigram(const int64_t* ids, const void* embed, const void* bigram, float scale, int64_t mul_prev,
                                   int64_t mul_cur, int64_t buckets, int32_t* prev, int64_t prev_ld, const int64_t* state_indices,
                                   const int64_t* seq_lens, const int32_t* q_start, const int32_t* q_len, int64_t batch,
                                   int64_t num_tokens, float* out, int64_t width, int dtype, void* stream) {
  SEMIPD_CHECK_ARG(num_tokens >= 0 && batch >= 0 && width > 0 && buckets > 0, SEMIPD_EINVAL, "embed_bigram: bad sizes");
  if (num_tokens == 0) return 0;
  SEMIPD_CHECK_ARG(ids && embed && bigram && prev && state_indices && seq_lens && out, SEMIPD_EINVAL, "embed_bigram: null pointer");
  SEMIPD_CHECK_ARG((q_start == nullptr) == (q_len == nullptr) && (q_start != nullptr || num_tokens == batch), SEMIPD_EINVAL,
                   "embed_bigram: q_start and q_len come together; without them one row per request");
  SEMIPD_DISPATCH_DTYPE(dtype, T,
                        hipLaunchKernelGGL((embed_bigram_kernel<T>), dim3((unsigned)num_tokens), dim3(256), 0, as_stream(stream), ids,
                                           (const T*)embed, (const T*)bigram, scale, mul_prev, mul_cur, buckets, prev, prev_ld,
                                           state_indices, seq_lens, q_start, q_len, batch, out, width));
  return launch_status("embed_bigram");
}

extern "C" int semipd_clamped_glu(const void* x, int64_t x_ld, void* out, int64_t out_ld, int64_t rows, int64_t ff, int groups,
                                  const float* topk_weights, const int32_t* topk_ids, int topk, float limit, float alpha, int dtype,
                                  void* stream) {
  SEMIPD_CHECK_ARG(rows >= 0 && ff > 0 && groups > 0 && x_ld >= 2 * ff * groups && out_ld >= ff * groups, SEMIPD_EINVAL,
                   "clamped_glu: bad sizes");
  if (rows == 0) return 0;
  SEMIPD_CHECK_ARG(x && out && ((topk_weights == nullptr) == (topk_ids == nullptr)) && (!topk_ids || topk > 0), SEMIPD_EINVAL,
                   "clamped_glu: null pointer, or routing weights without ids");
  const int64_t n = rows * ff * groups;
  const unsigned blocks = (unsigned)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
  SEMIPD_DISPATCH_DTYPE(dtype, T,
                        hipLaunchKernelGGL((clamped_glu_kernel<T>), dim3(blocks), dim3(256), 0, as_stream(stream), (const T*)x, x_ld,
                                           (T*)out, out_ld, rows, ff, groups, topk_weights, topk_ids, topk, limit, alpha));
  return launch_status("clamped_glu");
}

extern "C" int semipd_sigmoid_gate(void* x, int64_t x_ld, const void* gate, int64_t gate_ld, int64_t rows, int64_t width, int dtype,
                                   void* stream) {
  SEMIPD_CHECK_ARG(rows >= 0 && width > 0 && x_ld >= width && gate_ld >= width, SEMIPD_EINVAL, "sigmoid_gate: bad sizes");
  if (rows == 0) return 0;
  SEMIPD_CHECK_ARG(x && gate, SEMIPD_EINVAL, "sigmoid_gate: null pointer");
  const int64_t n = rows * width;
  const unsigned blocks = (unsigned)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
  SEMIPD_DISPATCH_DTYPE(dtype, T,
                        hipLaunchKernelGGL((sigmoid_gate_kernel<T>), dim3(blocks), dim3(256), 0, as_stream(stream), (T*)x, x_ld,
                                           (const T*)gate, gate_ld, rows, width));
  return launch_status("sigmoid_gate");
}


extern "C" int semipd_sigmoid_gate_heads(void* x, int64_t x_ld, const void* gate, int64_t gate_ld, int64_t rows, int64_t heads,
                                         int64_t head_width, int dtype, void* stream) {
  SEMIPD_CHECK_ARG(rows >= 0 && heads > 0 && head_width > 0 && x_ld >= heads * head_width && gate_ld >= heads, SEMIPD_EINVAL,
                   "sigmoid_gate_heads: bad sizes");
  if (rows == 0) return 0;
  SEMIPD_CHECK_ARG(x && gate, SEMIPD_EINVAL, "sigmoid_gate_heads: null pointer");
  const int64_t n = rows * heads * head_width;
  const unsigned blocks = (unsigned)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
  SEMIPD_DISPATCH_DTYPE(dtype, T,
                        hipLaunchKernelGGL((sigmoid_gate_heads_kernel<T>), dim3(blocks), dim3(256), 0, as_stream(stream), (T*)x, x_ld,
                                           (const T*)gate, gate_ld, rows, heads, head_width));
  return launch_status("sigmoid_gate_heads");
}

extern "C" int semipd_embed_stream(const int64_t* ids, const void* embed, float scale, int64_t num_tokens, float* out, int64_t width,
                                   int dtype, void* stream) {
  SEMIPD_CHECK_ARG(num_tokens >= 0 && width > 0, SEMIPD_EINVAL, "embed_stream: bad sizes");
  if (num_tokens == 0) return 0;
  SEMIPD_CHECK_ARG(ids && embed && out, SEMIPD_EINVAL, "embed_stream: null pointer");
  SEMIPD_DISPATCH_DTYPE(dtype, T,
                        hipLaunchKernelGGL((embed_stream_kernel<T>), dim3((unsigned)num_tokens), dim3(256), 0, as_stream(stream), ids,
                                           (const T*)embed, scale, out, width));
  return launch_status("embed_stream");
}

extern "C" int semipd_postnorm_stream(const void* y, int64_t y_ld, const void* layer_scale, float* stream, int64_t stream_ld,
                                      float alpha, const void* weight, float eps, void* out, int64_t out_ld, const void* shift_mu,
                                      float* prev, int64_t prev_ld, const int64_t* state_indices, const int64_t* seq_lens,
                                      int64_t rows, int64_t width, int dtype, void* stream_handle) {
  SEMIPD_CHECK_ARG(rows >= 0 && width > 0, SEMIPD_EINVAL, "postnorm_stream: bad sizes");
  if (rows == 0) return 0;
  SEMIPD_CHECK_ARG(stream && weight, SEMIPD_EINVAL, "postnorm_stream: null pointer");
  SEMIPD_CHECK_ARG(shift_mu == nullptr || (out && prev && state_indices && seq_lens && prev_ld >= width), SEMIPD_EINVAL,
                   "postnorm_stream: the shifted form needs out, the previous rows and the batch's state rows and lengths");
  SEMIPD_DISPATCH_DTYPE(dtype, T,
                        hipLaunchKernelGGL((postnorm_stream_kernel<T>), dim3((unsigned)rows), dim3(256), 0, as_stream(stream_handle),
                                           (const T*)y, y_ld, (const T*)layer_scale, stream, stream_ld, alpha, (const T*)weight, eps,
                                           (T*)out, out_ld, (const T*)shift_mu, prev, prev_ld, state_indices, seq_lens, width));
  return launch_status("postnorm_stream");
}

extern "C" int semipd_token_shift(const float* stream, int64_t stream_ld, const void* mu, float* prev, int64_t prev_ld,
                                  const int64_t* state_indices, const int64_t* seq_lens, const int32_t* q_start,
                                  const int32_t* q_len, int64_t batch, int64_t num_tokens, void* out, int64_t out_ld, int64_t width,
                                  int dtype, void* stream_handle) {
  SEMIPD_CHECK_ARG(num_tokens >= 0 && batch >= 0 && width > 0 && prev_ld >= width, SEMIPD_EINVAL, "token_shift: bad sizes");
  if (num_tokens == 0) return 0;
  SEMIPD_CHECK_ARG(stream && mu && prev && state_indices && seq_lens && out, SEMIPD_EINVAL, "token_shift: null pointer");
  SEMIPD_CHECK_ARG((q_start == nullptr) == (q_len == nullptr) && (q_start != nullptr || num_tokens == batch), SEMIPD_EINVAL,
                   "token_shift: q_start and q_len come together; without them one row per request");
  SEMIPD_DISPATCH_DTYPE(dtype, T,
                        hipLaunchKernelGGL((token_shift_kernel<T>), dim3((unsigned)num_tokens), dim3(256), 0,
                                           as_stream(stream_handle), stream, stream_ld, (const T*)mu, prev, prev_ld, state_indices,
                                           seq_lens, q_start, q_len, batch, (T*)out, out_ld, width));
  return launch_status("token_shift");
}
