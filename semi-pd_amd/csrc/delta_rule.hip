// Gated delta rule over a pool of per-request state rows (gfx950, wave64).
//
// Per head, a matrix S [D, E] in fp32 that starts at zero and is carried from token to token:
//     S <- g_t S;   u_t = beta_t (v_t - S^T k_t);   S <- S + k_t u_t^T;   o_t = S^T q_t
// with q, k unit vectors per head (q also times D^-1/2), g_t = exp(-exp(A_log) softplus(a_t + dt_bias)) and
// beta_t = sigmoid(b_t) one number per head and token.  q, k and v first pass a short causal convolution over time per
// channel and silu; the last taps - 1 inputs of every channel are part of the request's state.  Several heads may share a
// q / k head.  Everything behind the projection GEMM is fp32 whatever the activation type.
//
//  * delta_prep_kernel: a workgroup per token, its waves taking the token's q, k and v heads in turn: convolution (inputs in
//    front of the portion come from the state row), silu, unit norms, decay and beta -> an fp32 work row per token.
//  * delta_conv_state_kernel: the last taps - 1 inputs of the portion (shifted in behind what the row held) -> state row.
//  * delta_scan_kernel: ONE WAVE per (request, head, block of columns); column j of S lives in the registers of DS adjacent
//    lanes (D / DS rows each), so a step is two dot products over the lanes' rows, a 2-step lane reduction and one update
//    of the column: dk = S^T k, dq = S^T q from the old S, then u = beta (v - g dk), o = g dq + u (k . q), S <- g S + k u
//    (the same values as the sequence above: the read-out sees the current token's write).  k, q, v of kStage tokens come in
//    as 16-byte pieces that are in flight a stage ahead and sit in LDS (k . q, g, beta beside them); o leaves the same way.
//    The state is read when the rows of the launch do not start the sequence and written back after the last row, so a
//    prompt cut into portions, single decode tokens and a slot that another request held all take one path.
//  * delta_post_kernel: o / rms(o) * weight * silu(gate) -> the output projection's input, a workgroup per token.
//  * delta_decode_kernel: all of the above for batches of one token per request, a workgroup per (request, head).
#include "common.h"

namespace semipd {

struct DeltaArgs {
  const void* p; int64_t ld;                       // projection rows: q | k | v | gate | a | b at the offsets below
  int64_t q_off, k_off, v_off, gate_off, a_off, b_off;
  const void* conv_q; const void* conv_k; const void* conv_v;    // [channels, taps] of the activation type
  const float* a_log; const float* dt_bias;        // [H] fp32
  const void* norm_w;                              // [E] of the activation type
  float* work; int64_t wld;                        // fp32 [T, wld]: q [G D] | k [G D] | v, later o [H E] | g [H] | beta [H]
  float* state; int64_t state_ld;                  // fp32 [slots, >= H D E]: S[h][d][e]
  float* conv_state; int64_t conv_ld;              // fp32 [slots, >= (taps - 1) C]: [tap][channel], C = 2 G D + H E
  const int64_t* state_indices; const int64_t* seq_lens;
  const int32_t* q_start; const int32_t* q_len;    // [B] or NULL (one row per request)
  int64_t batch, num_tokens;
  int H, G, D, E, taps;
  float eps;
  void* out; int64_t out_ld;                       // [T, H E] of the activation type
};

__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + expf(-x)); }
__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// two adjacent elements in one access
template <typename T> __device__ __forceinline__ void load2(const T* p, float& x0, float& x1) {
  if constexpr (sizeof(T) == 2) {
    const uint32_t w = *reinterpret_cast<const uint32_t*>(p);
    T lo, hi;
    lo.v = (uint16_t)(w & 0xffffu);
    hi.v = (uint16_t)(w >> 16);
    x0 = Elem<T>::to_f(lo);
    x1 = Elem<T>::to_f(hi);
  } else {
    const float2 w = *reinterpret_cast<const float2*>(p);
    x0 = w.x;
    x1 = w.y;
  }
}

// the sum over groups of 2 / 4 adjacent lanes, in every lane of the group (data-parallel-primitive moves inside a quad)
template <int DS> __device__ __forceinline__ float quad_sum(float x) {
  if (DS >= 2) x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0xB1, 0xF, 0xF, true));   // lane ^ 1
  if (DS >= 4) x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x4E, 0xF, 0xF, true));   // lane ^ 2
  return x;
}

// the request that owns row t, the row's index inside the request's portion, the portion's length and its first position
__device__ __forceinline__ bool delta_locate(const DeltaArgs& a, int64_t t, int& b, int64_t& li, int64_t& n, int64_t& first_pos) {
  if (a.q_start == nullptr) {
    b = (int)t;
    li = 0;
    n = 1;
    first_pos = a.seq_lens[b] - 1;
    return first_pos >= 0;
  }
  for (int r = 0; r < (int)a.batch; ++r) {
    const int64_t s = a.q_start[r], m = a.q_len[r];
    if (t >= s && t < s + m) {
      b = r;
      li = t - s;
      n = m;
      first_pos = a.seq_lens[r] - m;
      return true;
    }
  }
  return false;
}

// ---------------------------------------------------------------------------------- convolution, silu, norms, gates
template <typename T>
__global__ void __launch_bounds__(256) delta_prep_kernel(DeltaArgs a) {
  // a workgroup per token; its waves take the token's units (q heads, k heads, v heads) in turn
  const int lane = threadIdx.x & 63;
  const int units = 2 * a.G + a.H;
  const int64_t t = blockIdx.x;
  int b;
  int64_t li, n, first_pos;
  if (!delta_locate(a, t, b, li, n, first_pos)) return;
  const int D = a.D, E = a.E, G = a.G, taps = a.taps;
  const int C = 2 * G * D + a.H * E;
  const T* p = (const T*)a.p;
  const float* cs = a.conv_state + a.state_indices[b] * a.conv_ld;
  const bool fresh = first_pos == 0;
  for (int u = threadIdx.x >> 6; u < units; u += 4) {
  // unit u: q head u, k head u - G, or v head u - 2 G
  const bool is_v = u >= 2 * G;
  const int size = is_v ? E : D;
  const int64_t col0 = is_v ? a.v_off + (int64_t)(u - 2 * G) * E : (u < G ? a.q_off + (int64_t)u * D : a.k_off + (int64_t)(u - G) * D);
  const int ch0 = is_v ? 2 * G * D + (u - 2 * G) * E : u * D;               // channel in the state's order (q | k | v)
  const T* cw = is_v ? (const T*)a.conv_v + (int64_t)(u - 2 * G) * E * taps
                     : (u < G ? (const T*)a.conv_q + (int64_t)u * D * taps : (const T*)a.conv_k + (int64_t)(u - G) * D * taps);
  float* w = a.work + t * a.wld + (is_v ? 2 * G * D + (u - 2 * G) * E : u * D);
  float sq = 0.f;
  // two adjacent channels per lane in one access each when everything is even (the work rows and the state rows are)
  const bool two = ((size | D | E) & 1) == 0 && ((col0 | a.ld | a.conv_ld) & 1) == 0;
  for (int c = 2 * lane; two && c < size; c += 128) {
    float y0 = 0.f, y1 = 0.f;
    for (int i = 0; i < taps; ++i) {
      const int64_t l = li - i;
      float x0 = 0.f, x1 = 0.f;
      if (l >= 0) load2(p + (t - i) * a.ld + col0 + c, x0, x1);
      else if (!fresh) {
        const float2 x = *reinterpret_cast<const float2*>(cs + (int64_t)(taps - 1 + l) * C + ch0 + c);
        x0 = x.x;
        x1 = x.y;
      }
      y0 += Elem<T>::to_f(cw[(int64_t)c * taps + (taps - 1 - i)]) * x0;
      y1 += Elem<T>::to_f(cw[(int64_t)(c + 1) * taps + (taps - 1 - i)]) * x1;
    }
    y0 = silu_f(y0);
    y1 = silu_f(y1);
    sq += y0 * y0 + y1 * y1;
    *reinterpret_cast<float2*>(w + c) = float2{y0, y1};
  }
  for (int c = lane; !two && c < size; c += 64) {
    float y = 0.f;
    for (int i = 0; i < taps; ++i) {
      const int64_t l = li - i;
      float x;
      if (l >= 0) x = Elem<T>::to_f(p[(t - i) * a.ld + col0 + c]);
      else if (fresh) x = 0.f;
      else x = cs[(int64_t)(taps - 1 + l) * C + ch0 + c];
      y += Elem<T>::to_f(cw[(int64_t)c * taps + (taps - 1 - i)]) * x;
    }
    y = silu_f(y);
    sq += y * y;
    w[c] = y;
  }
  if (!is_v) {
    sq = wave_sum(sq);
    const float inv = (u < G ? rsqrtf((float)D) : 1.0f) / sqrtf(sq + 1e-6f);
    for (int c = 2 * lane; two && c < size; c += 128) {      // (each lane rescales what it wrote itself)
      w[c] *= inv;
      w[c + 1] *= inv;
    }
    for (int c = lane; !two && c < size; c += 64) w[c] *= inv;
  } else if (lane == 0) {
    const int h = u - 2 * G;
    const float av = Elem<T>::to_f(p[t * a.ld + a.a_off + h]), bv = Elem<T>::to_f(p[t * a.ld + a.b_off + h]);
    float* gb = a.work + t * a.wld + C;
    gb[h] = expf(-expf(a.a_log[h]) * softplus_f(av + a.dt_bias[h]));
    gb[a.H + h] = sigmoid_f(bv);
  }
  }
}

// ---------------------------------------------------------------------------------- the inputs the next portion looks back at
template <typename T>
__global__ void __launch_bounds__(256) delta_conv_state_kernel(DeltaArgs a) {
  const int b = blockIdx.y;
  const int C = 2 * a.G * a.D + a.H * a.E;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  int64_t t0, n, first_pos;
  if (a.q_start == nullptr) {
    t0 = b; n = 1; first_pos = a.seq_lens[b] - 1;
  } else {
    t0 = a.q_start[b]; n = a.q_len[b]; first_pos = a.seq_lens[b] - n;
  }
  if (n <= 0 || first_pos < 0) return;
  const int GD = a.G * a.D;
  const int64_t col = c < GD ? a.q_off + c : (c < 2 * GD ? a.k_off + (c - GD) : a.v_off + (c - 2 * GD));
  float* cs = a.conv_state + a.state_indices[b] * a.conv_ld;
  const T* p = (const T*)a.p;
  const int keep = a.taps - 1;
  // entry s of the new state is the input at index n - keep + s of the portion; a negative index reaches into the old
  // state (entry s + n > s, read before entry s is written) or, at the start of a sequence, in front of it
  for (int s = 0; s < keep; ++s) {
    const int64_t l = n - keep + s;
    float x;
    if (l >= 0) x = Elem<T>::to_f(p[(t0 + l) * a.ld + col]);
    else if (first_pos == 0) x = 0.f;
    else x = cs[(int64_t)(keep + l) * C + c];
    cs[(int64_t)s * C + c] = x;
  }
}

// ---------------------------------------------------------------------------------- the recurrence
constexpr int kStage = 16;      // tokens whose k, q and scalars sit in LDS at a time

template <int DPT, int DS>
__global__ void __launch_bounds__(64) delta_scan_kernel(DeltaArgs a) {
  // per staged token: k and q, each as DS slices of DPT elements with 4 elements of padding behind every slice (the DS lanes
  // of a column read 16-byte pieces of different banks), then k . q, g, beta; then the block's columns of v, later o
  extern __shared__ __attribute__((aligned(16))) float lds[];
  constexpr int DP = DPT * DS, SL = DPT + 4, KQ = 2 * DS * SL;
  constexpr int COLS = 64 / DS;                                    // columns of S per workgroup (one wave)
  constexpr int NV = (kStage * 2 * DP / 4 + 63) / 64;              // 16-byte pieces of k | q per lane and stage
  constexpr int NO = (kStage * COLS / 4 + 63) / 64;                // ... of v / o
  const int b = blockIdx.x, h = blockIdx.y;
  const int D = a.D, E = a.E, G = a.G, H = a.H;
  const int gk = h / (H / G);
  int64_t t0, n, first_pos;
  if (a.q_start == nullptr) {
    t0 = b; n = 1; first_pos = a.seq_lens[b] - 1;
  } else {
    t0 = a.q_start[b]; n = a.q_len[b]; first_pos = a.seq_lens[b] - n;
  }
  if (n <= 0 || first_pos < 0) return;
  const int tid = threadIdx.x;
  const int s = tid % DS;
  const int C = 2 * G * D + H * E;
  float* kq_l = lds;
  float* sc_l = lds + kStage * KQ;
  float* vo_l = sc_l + kStage * 4;
  float* st = a.state + a.state_indices[b] * a.state_ld + (int64_t)h * D * E;
  const int jc = tid / DS;                                         // this lane's column inside the block
  const int j0 = blockIdx.z * COLS, j = j0 + jc;                   // ... and of S
  const bool on = j < E;
  // 16-byte accesses when every piece is whole and aligned (the work rows are: their width is a multiple of 4)
  const bool vec = (D & 3) == 0 && (E & 3) == 0 && COLS >= 4 && DP >= 4;
  float S[DPT];
#pragma unroll
  for (int r = 0; r < DPT; ++r) {
    const int d = s * DPT + r;
    S[r] = (on && d < D && first_pos > 0) ? st[(int64_t)d * E + j] : 0.f;
  }
  float4 pkq[NV], pvo[NO];
  // the pieces of stage c0 into registers: all loads of a stage are in flight together
  auto fetch = [&](int64_t c0) {
    const int m = (int)(n - c0 < kStage ? n - c0 : kStage);
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int f = tid + 64 * u, tok = f / (2 * DP / 4), within = f % (2 * DP / 4), which = within / (DP / 4), d = 4 * (within % (DP / 4));
      pkq[u] = (tok < m && d < D) ? *reinterpret_cast<const float4*>(a.work + (t0 + c0 + tok) * a.wld + (which ? 0 : G * D) + gk * D + d)
                                  : float4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int u = 0; u < NO; ++u) {
      const int f = tid + 64 * u, tok = f / (COLS / 4 > 0 ? COLS / 4 : 1), c = 4 * (f % (COLS / 4 > 0 ? COLS / 4 : 1));
      pvo[u] = (tok < m && j0 + c < E) ? *reinterpret_cast<const float4*>(a.work + (t0 + c0 + tok) * a.wld + 2 * G * D + h * E + j0 + c)
                                       : float4{0.f, 0.f, 0.f, 0.f};
    }
  };
  if (vec) fetch(0);
  for (int64_t c0 = 0; c0 < n; c0 += kStage) {
    const int m = (int)(n - c0 < kStage ? n - c0 : kStage);
    __syncthreads();
    if (vec) {
#pragma unroll
      for (int u = 0; u < NV; ++u) {
        const int f = tid + 64 * u, tok = f / (2 * DP / 4), within = f % (2 * DP / 4), which = within / (DP / 4), d = 4 * (within % (DP / 4));
        if (tok < kStage)
          *reinterpret_cast<float4*>(kq_l + tok * KQ + (which ? DS * SL : 0) + (d / DPT) * SL + d % DPT) = pkq[u];   // k first, then q
      }
#pragma unroll
      for (int u = 0; u < NO; ++u) {
        const int f = tid + 64 * u;
        if (f < kStage * COLS / 4) *reinterpret_cast<float4*>(vo_l + 4 * f) = pvo[u];
      }
    } else {
      for (int i = tid; i < m * 2 * DP; i += 64) {
        const int tok = i / (2 * DP), r = i % (2 * DP), d = r % DP;
        const float* wrow = a.work + (t0 + c0 + tok) * a.wld;
        const float x = d < D ? wrow[(r < DP ? G * D : 0) + gk * D + d] : 0.f;
        kq_l[tok * KQ + (r < DP ? 0 : DS * SL) + (d / DPT) * SL + d % DPT] = x;
      }
      for (int i = tid; i < m * COLS; i += 64) {
        const int tok = i / COLS, c = i % COLS;
        vo_l[i] = j0 + c < E ? a.work[(t0 + c0 + tok) * a.wld + 2 * G * D + h * E + j0 + c] : 0.f;
      }
    }
    __syncthreads();
    if (vec && c0 + kStage < n) fetch(c0 + kStage);                // the next stage's loads fly while this one is walked
    {                                                              // k . q, g, beta per token: four lanes a token
      static_assert(kStage * 4 == 64, "four lanes per staged token");
      const int tok = tid >> 2, part = tid & 3;
      float acc = 0.f;
      if (tok < m)
        for (int d = part; d < DP; d += 4) {
          const int o = (d / DPT) * SL + d % DPT;
          acc += kq_l[tok * KQ + o] * kq_l[tok * KQ + DS * SL + o];
        }
      acc = quad_sum<4>(acc);
      if (part == 0 && tok < m) {
        const float* gb = a.work + (t0 + c0 + tok) * a.wld + C;
        sc_l[tok * 4 + 0] = acc;
        sc_l[tok * 4 + 1] = gb[h];
        sc_l[tok * 4 + 2] = gb[H + h];
      }
    }
    __syncthreads();
#pragma unroll 2
    for (int tok = 0; tok < m; ++tok) {
      const float v = vo_l[tok * COLS + jc];
      const float4* kk4 = reinterpret_cast<const float4*>(kq_l + tok * KQ + s * SL);
      const float4* qq4 = reinterpret_cast<const float4*>(kq_l + tok * KQ + DS * SL + s * SL);
      float kk[DPT];
      float dk0 = 0.f, dq0 = 0.f, dk1 = 0.f, dq1 = 0.f;
#pragma unroll
      for (int r = 0; r < DPT; r += 4) {
        const float4 kv = kk4[r >> 2], qv = qq4[r >> 2];
        kk[r] = kv.x; kk[r + 1] = kv.y; kk[r + 2] = kv.z; kk[r + 3] = kv.w;
        dk0 += S[r] * kv.x;
        dq0 += S[r] * qv.x;
        dk1 += S[r + 1] * kv.y;
        dq1 += S[r + 1] * qv.y;
        dk0 += S[r + 2] * kv.z;
        dq0 += S[r + 2] * qv.z;
        dk1 += S[r + 3] * kv.w;
        dq1 += S[r + 3] * qv.w;
      }
      const float dk = quad_sum<DS>(dk0 + dk1), dq = quad_sum<DS>(dq0 + dq1);
      const float kq = sc_l[tok * 4 + 0], g = sc_l[tok * 4 + 1], beta = sc_l[tok * 4 + 2];
      const float u = beta * (v - g * dk);
#pragma unroll
      for (int r = 0; r < DPT; ++r) S[r] = g * S[r] + kk[r] * u;
      if (s == 0) vo_l[tok * COLS + jc] = g * dq + u * kq;         // (only this lane group reads or writes the element)
    }
    __syncthreads();
    if (vec) {
      for (int f = tid; f < m * COLS / 4; f += 64) {
        const int tok = f / (COLS / 4 > 0 ? COLS / 4 : 1), c = 4 * (f % (COLS / 4 > 0 ? COLS / 4 : 1));
        if (j0 + c < E)
          *reinterpret_cast<float4*>(a.work + (t0 + c0 + tok) * a.wld + 2 * G * D + h * E + j0 + c) = *reinterpret_cast<const float4*>(vo_l + 4 * f);
      }
    } else {
      for (int i = tid; i < m * COLS; i += 64) {
        const int tok = i / COLS, c = i % COLS;
        if (j0 + c < E) a.work[(t0 + c0 + tok) * a.wld + 2 * G * D + h * E + j0 + c] = vo_l[i];
      }
    }
  }
  if (on) {
#pragma unroll
    for (int r = 0; r < DPT; ++r) {
      const int d = s * DPT + r;
      if (d < D) st[(int64_t)d * E + j] = S[r];
    }
  }
}

// ---------------------------------------------------------------------------------- one token per request: everything at once
// A decode batch: a workgroup per (request, head) with all columns of S (DS lanes each) does the convolutions of its q / k head
// and of its value head, the unit norms, the gates, the step of the recurrence and the output norm and gate: one launch in
// place of three, and no work rows.  The same arithmetic as the kernels above (the unit norms multiply in at the use).
template <typename T, int DPT, int DS>
__global__ void __launch_bounds__(1024) delta_decode_kernel(DeltaArgs a) {
  extern __shared__ float lds[];          // k [DP] | q [DP] | scalars
  __shared__ float red[16];
  constexpr int DP = DPT * DS;
  const int b = blockIdx.x, h = blockIdx.y;
  const int D = a.D, E = a.E, G = a.G, H = a.H, taps = a.taps;
  const int gk = h / (H / G);
  const int64_t pos = a.seq_lens[b] - 1;
  if (pos < 0) return;
  const bool fresh = pos == 0;
  const int tid = threadIdx.x, s = tid % DS, j = tid / DS;
  const bool on = j < E;
  const int C = 2 * G * D + H * E;
  const int64_t slot = a.state_indices[b];
  const T* p = (const T*)a.p + (int64_t)b * a.ld;
  const float* cs = a.conv_state + slot * a.conv_ld;
  float* sc = lds + 2 * DP;
  auto conv = [&](const T* cw, int64_t col, int ch) -> float {      // cw: the channel's taps; ch: its place in the state
    float y = Elem<T>::to_f(cw[taps - 1]) * Elem<T>::to_f(p[col]);
    if (!fresh)
      for (int i = 1; i < taps; ++i) y += Elem<T>::to_f(cw[taps - 1 - i]) * cs[(int64_t)(taps - 1 - i) * C + ch];
    return silu_f(y);
  };
  for (int i = tid; i < 2 * DP; i += blockDim.x) {
    const bool is_q = i >= DP;
    const int d = is_q ? i - DP : i;
    float y = 0.f;
    if (d < D)
      y = is_q ? conv((const T*)a.conv_q + (int64_t)(gk * D + d) * taps, a.q_off + gk * D + d, gk * D + d)
               : conv((const T*)a.conv_k + (int64_t)(gk * D + d) * taps, a.k_off + gk * D + d, G * D + gk * D + d);
    lds[i] = y;
  }
  __syncthreads();
  if (tid < 64) {
    float sk = 0.f, sq = 0.f, kq = 0.f;
    for (int d = tid; d < DP; d += 64) {
      const float kv = lds[d], qv = lds[DP + d];
      sk += kv * kv;
      sq += qv * qv;
      kq += kv * qv;
    }
    sk = wave_sum(sk);
    sq = wave_sum(sq);
    kq = wave_sum(kq);
    if (tid == 0) {
      const float ik = 1.0f / sqrtf(sk + 1e-6f), iq = rsqrtf((float)D) / sqrtf(sq + 1e-6f);
      sc[0] = ik;
      sc[1] = iq;
      sc[2] = kq * ik * iq;
    }
  }
  __syncthreads();
  const float ik = sc[0], iq = sc[1], kq = sc[2];
  const float g = expf(-expf(a.a_log[h]) * softplus_f(Elem<T>::to_f(p[a.a_off + h]) + a.dt_bias[h]));
  const float beta = sigmoid_f(Elem<T>::to_f(p[a.b_off + h]));
  const float v = on ? conv((const T*)a.conv_v + (int64_t)(h * E + j) * taps, a.v_off + h * E + j, 2 * G * D + h * E + j) : 0.f;
  float* st = a.state + slot * a.state_ld + (int64_t)h * D * E;
  const float* kk = lds + s * DPT;
  const float* qq = kk + DP;
  float S[DPT];
  float dk = 0.f, dq = 0.f;
#pragma unroll
  for (int r = 0; r < DPT; ++r) {
    const int d = s * DPT + r;
    S[r] = (on && d < D && !fresh) ? st[(int64_t)d * E + j] : 0.f;
    dk += S[r] * (kk[r] * ik);
    dq += S[r] * (qq[r] * iq);
  }
  dk = quad_sum<DS>(dk);
  dq = quad_sum<DS>(dq);
  const float u = beta * (v - g * dk);
  const float o = g * dq + u * kq;
  if (on) {
#pragma unroll
    for (int r = 0; r < DPT; ++r) {
      const int d = s * DPT + r;
      if (d < D) st[(int64_t)d * E + j] = g * S[r] + (kk[r] * ik) * u;
    }
  }
  const float sq_o = block_sum((on && s == 0) ? o * o : 0.f, red);
  if (on && s == 0) {
    const float inv = 1.0f / sqrtf(sq_o / (float)E + a.eps);
    const float gate = Elem<T>::to_f(p[a.gate_off + h * E + j]);
    ((T*)a.out)[(int64_t)b * a.out_ld + h * E + j] = Elem<T>::from_f(o * inv * Elem<T>::to_f(((const T*)a.norm_w)[j]) * silu_f(gate));
  }
}

// ---------------------------------------------------------------------------------- unit RMS, weight, gate
template <typename T>
__global__ void __launch_bounds__(256) delta_post_kernel(DeltaArgs a) {
  // a workgroup per token; its waves take the token's heads in turn
  const int lane = threadIdx.x & 63;
  const int64_t t = blockIdx.x;
  const int E = a.E;
  for (int h = threadIdx.x >> 6; h < a.H; h += 4) {
  const float* o = a.work + t * a.wld + 2 * a.G * a.D + h * E;
  float sq = 0.f;
  for (int e = lane; e < E; e += 64) sq += o[e] * o[e];
  sq = wave_sum(sq);
  const float inv = 1.0f / sqrtf(sq / (float)E + a.eps);
  const T* gate = (const T*)a.p + t * a.ld + a.gate_off + (int64_t)h * E;
  const T* nw = (const T*)a.norm_w;
  T* out = (T*)a.out + t * a.out_ld + (int64_t)h * E;
  for (int e = lane; e < E; e += 64)
    out[e] = Elem<T>::from_f(o[e] * inv * Elem<T>::to_f(nw[e]) * silu_f(Elem<T>::to_f(gate[e])));
  }
}

}  // namespace semipd

using namespace semipd;

extern "C" int64_t semipd_delta_rule_work_width(int num_heads, int num_k_heads, int k_dim, int v_dim) {
  const int64_t w = 2 * (int64_t)num_k_heads * k_dim + (int64_t)num_heads * v_dim + 2 * (int64_t)num_heads;
  return (w + 3) / 4 * 4;
}

extern "C" int semipd_delta_rule(const void* proj, int64_t ld, int64_t q_off, int64_t k_off, int64_t v_off, int64_t gate_off,
                                 int64_t a_off, int64_t b_off, const void* conv_q, const void* conv_k, const void* conv_v,
                                 const float* a_log, const float* dt_bias, const void* norm_weight, float eps, float* work,
                                 int64_t work_ld, float* state, int64_t state_ld, float* conv_state, int64_t conv_ld,
                                 const int64_t* state_indices, const int64_t* seq_lens, const int32_t* q_start,
                                 const int32_t* q_len, int64_t batch, int64_t num_tokens, int num_heads, int num_k_heads,
                                 int k_dim, int v_dim, int taps, void* out, int64_t out_ld, int dtype, void* stream) {
  SEMIPD_CHECK_ARG(batch >= 0 && num_tokens >= 0, SEMIPD_EINVAL, "delta_rule: bad sizes");
  if (batch == 0 || num_tokens == 0) return 0;
  SEMIPD_CHECK_ARG(num_heads > 0 && num_k_heads > 0 && num_heads % num_k_heads == 0, SEMIPD_ESHAPE,
                   "delta_rule: %d heads over %d q / k heads", num_heads, num_k_heads);
  SEMIPD_CHECK_ARG(k_dim > 0 && k_dim <= 256 && v_dim > 0 && taps >= 1 && taps <= 64, SEMIPD_ESHAPE,
                   "delta_rule: key size %d (at most 256), value size %d, %d taps (1 .. 64)", k_dim, v_dim, taps);
  SEMIPD_CHECK_ARG(proj && conv_q && conv_k && conv_v && a_log && dt_bias && norm_weight && work && state && state_indices &&
                       seq_lens && out && (conv_state || taps == 1),
                   SEMIPD_EINVAL, "delta_rule: null pointer");
  SEMIPD_CHECK_ARG((q_start == nullptr) == (q_len == nullptr), SEMIPD_EINVAL, "delta_rule: q_start and q_len come together");
  SEMIPD_CHECK_ARG(q_start != nullptr || num_tokens == batch, SEMIPD_EINVAL, "delta_rule: one row per request without q_start");
  const int64_t C = 2 * (int64_t)num_k_heads * k_dim + (int64_t)num_heads * v_dim;
  SEMIPD_CHECK_ARG(work_ld >= C + 2 * num_heads && state_ld >= (int64_t)num_heads * k_dim * v_dim &&
                       (taps == 1 || conv_ld >= (taps - 1) * C) && out_ld >= (int64_t)num_heads * v_dim,
                   SEMIPD_EINVAL, "delta_rule: a row of the work buffer, the state or the output is too short");
  DeltaArgs a{proj, ld, q_off, k_off, v_off, gate_off, a_off, b_off, conv_q, conv_k, conv_v, a_log, dt_bias, norm_weight,
              work, work_ld, state, state_ld, conv_state, conv_ld, state_indices, seq_lens, q_start, q_len, batch, num_tokens,
              num_heads, num_k_heads, k_dim, v_dim, taps, eps, out, out_ld};
  hipStream_t st = as_stream(stream);
  // lanes per column and rows of S per lane: four lanes share a column from 32 rows up
  const int ds = k_dim >= 32 ? 4 : 1;
  const int per = (k_dim + ds - 1) / ds;
  const int dpt = per <= 4 ? 4 : (per <= 8 ? 8 : (per <= 16 ? 16 : (per <= 32 ? 32 : 64)));
  if (q_start == nullptr && (int64_t)ds * v_dim <= 1024) {
    // a decode batch: one launch, then the convolutions' inputs move on (the launch above has read the old ones)
    const int threads = (ds * v_dim + 63) / 64 * 64;
    const size_t lds = (size_t)(2 * dpt * ds + 4) * sizeof(float);
    const dim3 grid((unsigned)batch, (unsigned)num_heads);
#define SEMIPD_DELTA_DEC(DPT, DS) \
  SEMIPD_DISPATCH_DTYPE(dtype, T, hipLaunchKernelGGL((delta_decode_kernel<T, DPT, DS>), grid, dim3(threads), lds, st, a))
    if (ds == 1) {
      switch (dpt) {
        case 4: SEMIPD_DELTA_DEC(4, 1); break;
        case 8: SEMIPD_DELTA_DEC(8, 1); break;
        case 16: SEMIPD_DELTA_DEC(16, 1); break;
        default: SEMIPD_DELTA_DEC(32, 1); break;
      }
    } else {
      switch (dpt) {
        case 8: SEMIPD_DELTA_DEC(8, 4); break;
        case 16: SEMIPD_DELTA_DEC(16, 4); break;
        case 32: SEMIPD_DELTA_DEC(32, 4); break;
        default: SEMIPD_DELTA_DEC(64, 4); break;
      }
    }
#undef SEMIPD_DELTA_DEC
    if (taps > 1)
      SEMIPD_DISPATCH_DTYPE(dtype, T, hipLaunchKernelGGL((delta_conv_state_kernel<T>), dim3((unsigned)((C + 255) / 256), (unsigned)batch),
                                                         dim3(256), 0, st, a));
    return launch_status("delta_rule(decode)");
  }
  SEMIPD_DISPATCH_DTYPE(dtype, T, {
    hipLaunchKernelGGL((delta_prep_kernel<T>), dim3((unsigned)num_tokens), dim3(256), 0, st, a);
    if (taps > 1)
      hipLaunchKernelGGL((delta_conv_state_kernel<T>), dim3((unsigned)((C + 255) / 256), (unsigned)batch), dim3(256), 0, st, a);
  });
  // one wave per workgroup: the workgroups of a CU stage and walk their tokens independently, so the loads of one overlap
  // the arithmetic of the others
  const int threads = 64;
  const int cols = threads / ds;
  const size_t lds = (size_t)kStage * (2 * ds * (dpt + 4) + 4 + cols) * sizeof(float);
  const dim3 grid((unsigned)batch, (unsigned)num_heads, (unsigned)((v_dim + cols - 1) / cols));
#define SEMIPD_DELTA_SCAN(DPT, DS) hipLaunchKernelGGL((delta_scan_kernel<DPT, DS>), grid, dim3(threads), lds, st, a)
  if (ds == 1) {
    switch (dpt) {
      case 4: SEMIPD_DELTA_SCAN(4, 1); break;
      case 8: SEMIPD_DELTA_SCAN(8, 1); break;
      case 16: SEMIPD_DELTA_SCAN(16, 1); break;
      default: SEMIPD_DELTA_SCAN(32, 1); break;
    }
  } else {
    switch (dpt) {
      case 8: SEMIPD_DELTA_SCAN(8, 4); break;
      case 16: SEMIPD_DELTA_SCAN(16, 4); break;
      case 32: SEMIPD_DELTA_SCAN(32, 4); break;
      default: SEMIPD_DELTA_SCAN(64, 4); break;
    }
  }
#undef SEMIPD_DELTA_SCAN
  SEMIPD_DISPATCH_DTYPE(dtype, T,
                        hipLaunchKernelGGL((delta_post_kernel<T>), dim3((unsigned)num_tokens), dim3(256), 0, st, a));
  return launch_status("delta_rule");
}
