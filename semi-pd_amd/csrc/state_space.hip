// Selective state-space recurrence (the scalar-decay form with a matrix state per head) over a pool of per-request state
// rows (gfx950, wave64).
//
// Rows of the projection hold [z: H E | x: H E | B: G N | C: G N | dt: H].  x, B and C pass a causal convolution over time
// per channel (taps weights and a bias per channel, zeros in front of the sequence) and silu; the last taps - 1 inputs of
// every channel are part of the request's state.  Per head h (group g = h / (H / G)), with S [N, E] in fp32 from zero:
//     dt_t = softplus(dt_t + dt_bias_h);   S <- exp(-exp(A_log_h) dt_t) S + dt_t B_t x_t^T;   y_t = S^T C_t + D_h x_t
// then y * silu(z), an RMS norm over each of `norm_groups` equal parts of the row, times a weight.  Everything behind the
// projection GEMM is fp32 whatever the activation type.
//
//  * ssm_prep_kernel: a workgroup per (tile of 32 tokens -- one token in small batches --, 1024 channels), four channels per
//    thread with their taps in registers where alignment allows: convolution + bias + silu of the token's x | B | C channels (inputs in front
//    of the portion come from the state row), dt and the decay -> an fp32 work row per token.
//  * ssm_conv_state_kernel: the last taps - 1 inputs of the portion (shifted in behind what the row held) -> state row.
//  * ssm_scan_kernel: ONE WAVE per (request, head, block of 64 / NS columns of S); a column of S lives in the registers of NS
//    adjacent lanes, NPT rows each, so a step is one multiply-add per register for the update, one for the read-out, and a
//    log2(NS)-step lane reduction.  B, C, x, dt and the decay of kStage tokens sit in LDS; the next stage's 16-byte pieces are
//    fetched into registers while a stage is multiplied and go into the other half of the LDS buffer behind it.  The state is read when the rows
//    of the launch do not start the sequence and written back after the last row, so a prompt cut into portions, single
//    decode tokens and a slot that another request held all take one path.
//  * ssm_post_kernel: gate, grouped norm, weight -> the output projection's input, a workgroup per token.
//  * ssm_decode_kernel: all of the above for batches of one token per request whose state is small, a workgroup per request.
#include "common.h"

namespace semipd {

struct SsmArgs {
  const void* p; int64_t ld;                       // projection rows
  int64_t z_off, x_off, dt_off;                    // columns of z, of x | B | C (one range, the convolution's channels), of dt
  const void* conv_w; const void* conv_b;          // [C, taps], [C] of the activation type, C = H E + 2 G N
  const float* dt_bias; const float* a_log; const float* d_skip;      // [H] fp32
  const void* norm_w; int norm_groups; float eps;  // [H E] of the activation type
  float* work; int64_t wld;                        // fp32 [T, wld]: x (later y) [H E] | B [G N] | C [G N] | dt [H] | decay [H]
  float* state; int64_t state_ld;                  // fp32 [slots, >= H N E]: S[h][n][e]
  float* conv_state; int64_t conv_ld;              // fp32 [slots, >= (taps - 1) C]: [tap][channel]
  const int64_t* state_indices; const int64_t* seq_lens;
  const int32_t* q_start; const int32_t* q_len;    // [B] or NULL (one row per request)
  int64_t batch, num_tokens;
  int H, G, N, E, taps;
  void* out; int64_t out_ld;                       // [T, H E] of the activation type
};

__device__ __forceinline__ float ssm_silu(float x) { return x / (1.0f + expf(-x)); }
__device__ __forceinline__ float ssm_softplus(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// the request that owns row t, the row's index inside the request's portion, the portion's length and its first position
__device__ __forceinline__ bool ssm_locate(const SsmArgs& a, int64_t t, int& b, int64_t& li, int64_t& n, int64_t& first_pos) {
  if (a.q_start == nullptr) {
    b = (int)t; li = 0; n = 1; first_pos = a.seq_lens[b] - 1;
    return first_pos >= 0;
  }
  for (int r = 0; r < (int)a.batch; ++r) {
    const int64_t s = a.q_start[r], m = a.q_len[r];
    if (t >= s && t < s + m) {
      b = r; li = t - s; n = m; first_pos = a.seq_lens[r] - m;
      return true;
    }
  }
  return false;
}

// one channel of the convolution for row t (index li of its portion): bias + sum of taps, then silu
template <typename T>
__device__ __forceinline__ float ssm_conv_channel(const SsmArgs& a, const T* p, const float* cs, bool fresh, int64_t t, int64_t li,
                                                  int c, int C) {
  const T* cw = (const T*)a.conv_w + (int64_t)c * a.taps;
  float y = a.conv_b ? Elem<T>::to_f(((const T*)a.conv_b)[c]) : 0.f;
  for (int i = 0; i < a.taps; ++i) {
    const int64_t l = li - i;
    float x;
    if (l >= 0) x = Elem<T>::to_f(p[(t - i) * a.ld + a.x_off + c]);
    else if (fresh) x = 0.f;
    else x = cs[(int64_t)(a.taps - 1 + l) * C + c];
    y += Elem<T>::to_f(cw[a.taps - 1 - i]) * x;
  }
  return ssm_silu(y);
}

// ---------------------------------------------------------------------------------- convolution, silu, step sizes, decays
constexpr int kPrepChannels = 1024;      // channels per workgroup (blockIdx.y walks a token's channels)

// four adjacent elements of the activation type in one access
template <typename T> __device__ __forceinline__ void load4(const T* p, float (&x)[4]) {
  if constexpr (sizeof(T) == 2) {
    const uint2 w = *reinterpret_cast<const uint2*>(p);
    T e;
    e.v = (uint16_t)(w.x & 0xffffu); x[0] = Elem<T>::to_f(e);
    e.v = (uint16_t)(w.x >> 16);     x[1] = Elem<T>::to_f(e);
    e.v = (uint16_t)(w.y & 0xffffu); x[2] = Elem<T>::to_f(e);
    e.v = (uint16_t)(w.y >> 16);     x[3] = Elem<T>::to_f(e);
  } else {
    const float4 w = *reinterpret_cast<const float4*>(p);
    x[0] = w.x; x[1] = w.y; x[2] = w.z; x[3] = w.w;
  }
}

constexpr int kPrepMaxTaps = 8;          // taps whose weights the four-channel form keeps in registers
constexpr int kPrepTile = 32;            // tokens a workgroup of a prompt batch walks with them

template <typename T, bool VEC4>
__global__ void __launch_bounds__(256) ssm_prep_kernel(SsmArgs a, int tile) {
  const int C = a.H * a.E + 2 * a.G * a.N;
  const T* p = (const T*)a.p;
  const int c_lo = blockIdx.y * kPrepChannels;
  const int c_hi = c_lo + kPrepChannels < C ? c_lo + kPrepChannels : C;
  const int taps = a.taps;
  // four channels per thread (8- / 16-byte reads of the inputs and of the state's rows, one 16-byte write), their taps and
  // bias in registers for all tokens of the tile
  const int c4 = c_lo + 4 * threadIdx.x;
  const bool mine = VEC4 && c4 < c_hi;
  float wt[kPrepMaxTaps][4], bias[4] = {0.f, 0.f, 0.f, 0.f};
  if (mine) {
    const T* cw = (const T*)a.conv_w + (int64_t)c4 * taps;
#pragma unroll
    for (int i = 0; i < kPrepMaxTaps; ++i)
#pragma unroll
      for (int u = 0; u < 4; ++u) wt[i][u] = i < taps ? Elem<T>::to_f(cw[u * taps + taps - 1 - i]) : 0.f;      // i tokens back
    if (a.conv_b)
#pragma unroll
      for (int u = 0; u < 4; ++u) bias[u] = Elem<T>::to_f(((const T*)a.conv_b)[c4 + u]);
  }
  for (int tt = 0; tt < tile; ++tt) {
    const int64_t t = (int64_t)blockIdx.x * tile + tt;
    if (t >= a.num_tokens) break;
    int b;
    int64_t li, n, first_pos;
    if (!ssm_locate(a, t, b, li, n, first_pos)) continue;
    const float* cs = a.conv_state + a.state_indices[b] * a.conv_ld;
    float* w = a.work + t * a.wld;
    const bool fresh = first_pos == 0;
    if constexpr (VEC4) {
      if (mine) {
        float y[4] = {bias[0], bias[1], bias[2], bias[3]};
#pragma unroll
        for (int i = 0; i < kPrepMaxTaps; ++i) {
          if (i >= taps) break;
          const int64_t l = li - i;
          float x[4] = {0.f, 0.f, 0.f, 0.f};
          if (l >= 0) load4(p + (t - i) * a.ld + a.x_off + c4, x);
          else if (!fresh) {
            const float4 v = *reinterpret_cast<const float4*>(cs + (int64_t)(taps - 1 + l) * C + c4);
            x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
          }
#pragma unroll
          for (int u = 0; u < 4; ++u) y[u] += wt[i][u] * x[u];
        }
        *reinterpret_cast<float4*>(w + c4) = float4{ssm_silu(y[0]), ssm_silu(y[1]), ssm_silu(y[2]), ssm_silu(y[3])};
      }
    } else {
      for (int c = c_lo + threadIdx.x; c < c_hi; c += 256) w[c] = ssm_conv_channel<T>(a, p, cs, fresh, t, li, c, C);
    }
    if (blockIdx.y == 0)
      for (int h = threadIdx.x; h < a.H; h += 256) {
        const float dt = ssm_softplus(Elem<T>::to_f(p[t * a.ld + a.dt_off + h]) + a.dt_bias[h]);
        w[C + h] = dt;
        w[C + a.H + h] = expf(-expf(a.a_log[h]) * dt);
      }
  }
}

// ---------------------------------------------------------------------------------- the inputs the next portion looks back at
template <typename T>
__global__ void __launch_bounds__(256) ssm_conv_state_kernel(SsmArgs a) {
  const int b = blockIdx.y;
  const int C = a.H * a.E + 2 * a.G * a.N;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  int64_t t0, n, first_pos;
  if (a.q_start == nullptr) {
    t0 = b; n = 1; first_pos = a.seq_lens[b] - 1;
  } else {
    t0 = a.q_start[b]; n = a.q_len[b]; first_pos = a.seq_lens[b] - n;
  }
  if (n <= 0 || first_pos < 0) return;
  float* cs = a.conv_state + a.state_indices[b] * a.conv_ld;
  const T* p = (const T*)a.p;
  const int keep = a.taps - 1;
  // entry s of the new state is the input at index n - keep + s of the portion; a negative index reaches into the old
  // state (entry s + n > s, read before entry s is written) or, at the start of a sequence, in front of it
  for (int s = 0; s < keep; ++s) {
    const int64_t l = n - keep + s;
    float x;
    if (l >= 0) x = Elem<T>::to_f(p[(t0 + l) * a.ld + a.x_off + c]);
    else if (first_pos == 0) x = 0.f;
    else x = cs[(int64_t)(keep + l) * C + c];
    cs[(int64_t)s * C + c] = x;
  }
}

// ---------------------------------------------------------------------------------- the recurrence
constexpr int kSsmStage = 8;       // tokens of a stage: their B, C, x, dt and decay sit in LDS, the next stage's in registers

template <int NPT, int NS, bool VEC4>
__global__ void __launch_bounds__(64) ssm_scan_kernel(SsmArgs a) {
  // per staged token: B [NP] | C [NP] | x of the block's columns [COLS] | dt | decay | 2 unused.  B and C are cut into the NS
  // slices that the lanes of a column read, each slice followed by 4 unused floats: the 16-byte reads of the NS lanes then
  // fall into different banks (slices of 32 floats alone would put lanes 0 and 2 on the same ones)
  extern __shared__ __attribute__((aligned(16))) float lds[];
  constexpr int SEG = NS > 1 ? NPT + 4 : NPT, NP = SEG * NS, COLS = 64 / NS, TOK = 2 * NP + COLS + 4, TOKU = TOK / 4;
  constexpr int U = (kSsmStage * TOKU + 63) / 64;          // 16-byte pieces of a stage per lane
  const int lane = threadIdx.x;
  const int H = a.H, G = a.G, N = a.N, E = a.E;
  const int eblocks = (E + COLS - 1) / COLS;
  int64_t id = blockIdx.x;
  const int eb = (int)(id % eblocks); id /= eblocks;
  const int h = (int)(id % H);
  const int b = (int)(id / H);
  int64_t t0, n, first_pos;
  if (a.q_start == nullptr) {
    t0 = b; n = 1; first_pos = a.seq_lens[b] - 1;
  } else {
    t0 = a.q_start[b]; n = a.q_len[b]; first_pos = a.seq_lens[b] - n;
  }
  if (n <= 0 || first_pos < 0) return;
  const int g = h / (H / G);
  const int col = lane / NS, ns = lane % NS;
  const int e = eb * COLS + col;
  const bool e_ok = e < E;
  const int n0 = ns * NPT;
  const int C = H * E + 2 * G * N;
  float* st = a.state + a.state_indices[b] * a.state_ld + (int64_t)h * N * E;
  float S[NPT];
#pragma unroll
  for (int i = 0; i < NPT; ++i) S[i] = (first_pos > 0 && e_ok && n0 + i < N) ? st[(int64_t)(n0 + i) * E + e] : 0.f;
  const float dskip = a.d_skip ? a.d_skip[h] : 0.f;
  // piece u of a staged token: four of B, of C, of the block's x, or (dt, decay, -, -); rows shorter than NP are zero-filled
  auto piece = [&](const float* w, int u) -> float4 {
    const float* src;
    int have;                     // elements of the piece that exist
    if (u < NP / 2) {
      const int pos = 4 * (u < NP / 4 ? u : u - NP / 4), off = pos % SEG;
      if (off >= NPT) return float4{0.f, 0.f, 0.f, 0.f};                 // the gap behind a slice
      const int i = (pos / SEG) * NPT + off;                               // row of the state
      src = w + H * E + (u < NP / 4 ? 0 : G * N) + g * N + i;
      have = N - i;
    } else if (u < NP / 2 + COLS / 4) {
      src = w + h * E + eb * COLS + 4 * (u - NP / 2);
      have = E - eb * COLS - 4 * (u - NP / 2);
    } else {
      return float4{w[C + h], w[C + H + h], 0.f, 0.f};
    }
    if (have <= 0) return float4{0.f, 0.f, 0.f, 0.f};
    if (VEC4 && have >= 4) return *reinterpret_cast<const float4*>(src);
    return float4{src[0], have > 1 ? src[1] : 0.f, have > 2 ? src[2] : 0.f, have > 3 ? src[3] : 0.f};
  };
  // A stage's pieces are fetched into registers while the stage in front of it is multiplied, and put into the other half
  // of the LDS buffer behind it: the loads of HBM rows are in flight during the arithmetic.
  float4 v[U];
  auto fetch = [&](int64_t s0) {
    const int cnt = (int)((n - s0) < kSsmStage ? (n - s0) : kSsmStage);
    const int total = cnt * TOKU;
    const float* w0 = a.work + (t0 + s0) * a.wld;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int it = u * 64 + lane;
      v[u] = it < total ? piece(w0 + (int64_t)(it / TOKU) * a.wld, it % TOKU) : float4{0.f, 0.f, 0.f, 0.f};
    }
  };
  auto stash = [&](float* buf) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int it = u * 64 + lane;
      if (it < kSsmStage * TOKU) *reinterpret_cast<float4*>(buf + 4 * it) = v[u];
    }
  };
  fetch(0);
  stash(lds);
  __syncthreads();
  int half = 0;
  for (int64_t s0 = 0; s0 < n; s0 += kSsmStage) {
    const int cnt = (int)((n - s0) < kSsmStage ? (n - s0) : kSsmStage);
    const bool more = s0 + kSsmStage < n;
    if (more) fetch(s0 + kSsmStage);
    const float* stage = lds + half * (kSsmStage * TOK);
    for (int k = 0; k < cnt; ++k) {
      const float* l = stage + k * TOK;
      const float xv = l[2 * NP + col], dtv = l[2 * NP + COLS], dec = l[2 * NP + COLS + 1];
      const float dx = dtv * xv;
      float y = 0.f;
#pragma unroll
      for (int i = 0; i < NPT; i += 4) {
        const float4 bv = *reinterpret_cast<const float4*>(l + ns * SEG + i);
        const float4 cv = *reinterpret_cast<const float4*>(l + NP + ns * SEG + i);
        S[i] = dec * S[i] + bv.x * dx;         y += S[i] * cv.x;
        S[i + 1] = dec * S[i + 1] + bv.y * dx; y += S[i + 1] * cv.y;
        S[i + 2] = dec * S[i + 2] + bv.z * dx; y += S[i + 2] * cv.z;
        S[i + 3] = dec * S[i + 3] + bv.w * dx; y += S[i + 3] * cv.w;
      }
      if (NS >= 2) y += __shfl_xor(y, 1, 64);
      if (NS >= 4) y += __shfl_xor(y, 2, 64);
      if (NS >= 8) y += __shfl_xor(y, 4, 64);
      if (ns == 0 && e_ok) a.work[(t0 + s0 + k) * a.wld + h * E + e] = y + dskip * xv;
    }
    half ^= 1;
    if (more) stash(lds + half * (kSsmStage * TOK));
    __syncthreads();
  }
  if (e_ok) {
#pragma unroll
    for (int i = 0; i < NPT; ++i)
      if (n0 + i < N) st[(int64_t)(n0 + i) * E + e] = S[i];
  }
}

// ---------------------------------------------------------------------------------- gate, grouped norm, weight
template <typename T>
__device__ __forceinline__ void ssm_gate_norm_store(const SsmArgs& a, const float* y, const T* z, T* o, float* red) {
  const int inner = a.H * a.E, gs = inner / a.norm_groups;
  for (int grp = 0; grp < a.norm_groups; ++grp) {
    float sq = 0.f;
    for (int i = threadIdx.x; i < gs; i += blockDim.x) {
      const int c = grp * gs + i;
      const float v = y[c] * ssm_silu(Elem<T>::to_f(z[c]));
      sq += v * v;
    }
    const float rs = 1.0f / sqrtf(block_sum(sq, red) / (float)gs + a.eps);
    for (int i = threadIdx.x; i < gs; i += blockDim.x) {
      const int c = grp * gs + i;
      const float v = y[c] * ssm_silu(Elem<T>::to_f(z[c]));
      o[c] = Elem<T>::from_f(v * rs * Elem<T>::to_f(((const T*)a.norm_w)[c]));
    }
  }
}

template <typename T>
__global__ void __launch_bounds__(256) ssm_post_kernel(SsmArgs a) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  ssm_gate_norm_store<T>(a, a.work + t * a.wld, (const T*)a.p + t * a.ld + a.z_off, (T*)a.out + t * a.out_ld, red);
}

// ---------------------------------------------------------------------------------- one token per request: one launch
// A workgroup per request: convolution of the token's channels into LDS (and the shifted inputs back into the state row),
// step sizes and decays, then thread (h, e) walks column e of head h's S in the state row (N multiply-adds for the update,
// N for the read-out; lanes of a wave read adjacent e), then gate, grouped norm and weight.
template <typename T>
__global__ void __launch_bounds__(1024) ssm_decode_kernel(SsmArgs a) {
  extern __shared__ __attribute__((aligned(16))) float lds[];       // x | B | C [C], dt [H], decay [H], y [H E]
  __shared__ float red[16];
  const int b = blockIdx.x;
  const int H = a.H, G = a.G, N = a.N, E = a.E, taps = a.taps;
  const int inner = H * E, C = inner + 2 * G * N;
  const int64_t first_pos = a.seq_lens[b] - 1;
  if (first_pos < 0) return;
  const bool fresh = first_pos == 0;
  const T* p = (const T*)a.p;
  const int64_t slot = a.state_indices[b];
  float* cs = a.conv_state + slot * a.conv_ld;
  float* xbc = lds;
  float* dts = lds + C;
  float* ys = lds + C + 2 * H;
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    const T* cw = (const T*)a.conv_w + (int64_t)c * taps;
    const float cur = Elem<T>::to_f(p[(int64_t)b * a.ld + a.x_off + c]);
    float y = (a.conv_b ? Elem<T>::to_f(((const T*)a.conv_b)[c]) : 0.f) + Elem<T>::to_f(cw[taps - 1]) * cur;
    // state entry s is the input s - (taps - 1) tokens back; every entry moves one place down and the token comes in last
    for (int s = 0; s < taps - 1; ++s) {
      const float x = fresh ? 0.f : cs[(int64_t)s * C + c];
      y += Elem<T>::to_f(cw[s]) * x;
      if (s > 0) cs[(int64_t)(s - 1) * C + c] = x;
    }
    if (taps > 1) cs[(int64_t)(taps - 2) * C + c] = cur;
    xbc[c] = ssm_silu(y);
  }
  for (int h = threadIdx.x; h < H; h += blockDim.x) {
    const float dt = ssm_softplus(Elem<T>::to_f(p[(int64_t)b * a.ld + a.dt_off + h]) + a.dt_bias[h]);
    dts[h] = dt;
    dts[H + h] = expf(-expf(a.a_log[h]) * dt);
  }
  __syncthreads();
  float* st = a.state + slot * a.state_ld;
  for (int c = threadIdx.x; c < inner; c += blockDim.x) {
    const int h = c / E, e = c - h * E, g = h / (H / G);
    const float xv = xbc[c], dec = dts[H + h], dx = dts[h] * xv;
    const float* Bv = xbc + inner + g * N;
    const float* Cv = xbc + inner + G * N + g * N;
    float* col = st + (int64_t)h * N * E + e;
    float y = 0.f;
    for (int i = 0; i < N; ++i) {
      const float s = (fresh ? 0.f : dec * col[(int64_t)i * E]) + Bv[i] * dx;
      col[(int64_t)i * E] = s;
      y += s * Cv[i];
    }
    ys[c] = y + (a.d_skip ? a.d_skip[h] : 0.f) * xv;
  }
  __syncthreads();
  ssm_gate_norm_store<T>(a, ys, p + (int64_t)b * a.ld + a.z_off, (T*)a.out + (int64_t)b * a.out_ld, red);
}

}  // namespace semipd

using namespace semipd;

extern "C" int64_t semipd_state_space_work_width(int num_heads, int groups, int state, int v_dim) {
  const int64_t w = (int64_t)num_heads * v_dim + 2 * (int64_t)groups * state + 2 * num_heads;
  return (w + 3) / 4 * 4;
}

extern "C" int semipd_state_space(const void* proj, int64_t ld, int64_t z_off, int64_t x_off, int64_t dt_off, const void* conv_w,
                                  const void* conv_b, const float* dt_bias, const float* a_log, const float* d_skip,
                                  const void* norm_w, int norm_groups, float eps, float* work, int64_t work_ld, float* state,
                                  int64_t state_ld, float* conv_state, int64_t conv_ld, const int64_t* state_indices,
                                  const int64_t* seq_lens, const int32_t* q_start, const int32_t* q_len, int64_t batch,
                                  int64_t num_tokens, int num_heads, int groups, int state_size, int v_dim, int taps, void* out,
                                  int64_t out_ld, int fused_decode, int dtype, void* stream) {
  SEMIPD_CHECK_ARG(batch >= 0 && num_tokens >= 0, SEMIPD_EINVAL, "state_space: bad sizes");
  if (batch == 0 || num_tokens == 0) return 0;
  SEMIPD_CHECK_ARG(num_heads > 0 && groups > 0 && num_heads % groups == 0 && state_size > 0 && v_dim > 0 && taps >= 1 && taps <= 64,
                   SEMIPD_ESHAPE, "state_space: %d heads over %d groups, state %d, values %d, %d taps", num_heads, groups,
                   state_size, v_dim, taps);
  SEMIPD_CHECK_ARG(state_size <= 256, SEMIPD_ESHAPE, "state_space: a state of %d rows per head (at most 256)", state_size);
  const int64_t inner = (int64_t)num_heads * v_dim, C = inner + 2 * (int64_t)groups * state_size;
  SEMIPD_CHECK_ARG(norm_groups > 0 && inner % norm_groups == 0, SEMIPD_ESHAPE, "state_space: %d norm groups over %lld elements",
                   norm_groups, (long long)inner);
  SEMIPD_CHECK_ARG(proj && conv_w && dt_bias && a_log && norm_w && state && out && state_indices && seq_lens &&
                       (taps == 1 || conv_state),
                   SEMIPD_EINVAL, "state_space: null pointer");
  SEMIPD_CHECK_ARG((q_start == nullptr) == (q_len == nullptr), SEMIPD_EINVAL, "state_space: q_start and q_len come together");
  SEMIPD_CHECK_ARG(q_start != nullptr || num_tokens == batch, SEMIPD_EINVAL, "state_space: one row per request without q_start");
  SEMIPD_CHECK_ARG(state_ld >= inner * state_size && (taps == 1 || conv_ld >= (int64_t)(taps - 1) * C) && out_ld >= inner,
                   SEMIPD_EINVAL, "state_space: rows too short");
  SEMIPD_CHECK_ARG(z_off >= 0 && x_off >= 0 && dt_off >= 0 && ld >= z_off + inner && ld >= x_off + C && ld >= dt_off + num_heads,
                   SEMIPD_EINVAL, "state_space: a column range leaves the row");
  SsmArgs a{proj, ld, z_off, x_off, dt_off, conv_w, conv_b, dt_bias, a_log, d_skip, norm_w, norm_groups, eps, work, work_ld, state,
            state_ld, conv_state, conv_ld, state_indices, seq_lens, q_start, q_len, batch, num_tokens, num_heads, groups, state_size,
            v_dim, taps, out, out_ld};
  hipStream_t s = as_stream(stream);
  const size_t dec_lds = (size_t)(C + 2 * num_heads + inner) * sizeof(float);
  if (q_start == nullptr && fused_decode && dec_lds <= 160 * 1024 - 256) {
    const int threads = inner >= 1024 ? 1024 : (int)((inner + 63) / 64 * 64);
    static std::atomic<uint64_t> done[3] = {};
    int rc = 0;
    SEMIPD_DISPATCH_DTYPE(dtype, T, {
      const int slot = sizeof(T) == 4 ? 0 : (dtype == SEMIPD_BF16 ? 1 : 2);
      if (dec_lds > 65536 && ensure_dynamic_lds((const void*)ssm_decode_kernel<T>, dec_lds, done[slot], "state_space")) rc = 1;
      if (!rc) hipLaunchKernelGGL((ssm_decode_kernel<T>), dim3((unsigned)batch), dim3(threads), dec_lds, s, a);
    });
    if (rc) return SEMIPD_EINVAL;
    return launch_status("state_space_decode");
  }
  SEMIPD_CHECK_ARG(work && work_ld >= semipd_state_space_work_width(num_heads, groups, state_size, v_dim), SEMIPD_EINVAL,
                   "state_space: the work rows are missing or too short");
  const unsigned cblocks = (unsigned)((C + kPrepChannels - 1) / kPrepChannels);
  // four channels per thread: every row and column range starts on a multiple of four elements
  const bool prep4 = C % 4 == 0 && x_off % 4 == 0 && ld % 4 == 0 && work_ld % 4 == 0 && (taps == 1 || conv_ld % 4 == 0) &&
                     ((uintptr_t)proj % 16) == 0 && aligned16(work) && (taps == 1 || aligned16(conv_state)) &&
                     aligned16(conv_w) && taps <= kPrepMaxTaps;
  // a prompt batch: a workgroup walks a tile of tokens with its channels' taps in registers; one row per request: a token each
  const int tile = (q_start != nullptr && prep4 && num_tokens >= 8 * kPrepTile) ? kPrepTile : 1;
  const dim3 pgrid((unsigned)((num_tokens + tile - 1) / tile), cblocks);
  SEMIPD_DISPATCH_DTYPE(dtype, T, {
    if (prep4) hipLaunchKernelGGL((ssm_prep_kernel<T, true>), pgrid, dim3(256), 0, s, a, tile);
    else hipLaunchKernelGGL((ssm_prep_kernel<T, false>), pgrid, dim3(256), 0, s, a, tile);
  });
  if (taps > 1) {
    const dim3 grid((unsigned)((C + 255) / 256), (unsigned)batch);
    SEMIPD_DISPATCH_DTYPE(dtype, T, hipLaunchKernelGGL((ssm_conv_state_kernel<T>), grid, dim3(256), 0, s, a));
  }
  // 16-byte staging reads: B, C and x of a token start on multiples of four floats
  const bool scan4 = work_ld % 4 == 0 && aligned16(work) && inner % 4 == 0 && state_size % 4 == 0 && v_dim % 4 == 0;
#define SEMIPD_SSM_SCAN(NPT, NS)                                                                                              \
  do {                                                                                                                        \
    constexpr int cols = 64 / NS;                                                                                             \
    const unsigned blocks = (unsigned)(batch * num_heads * ((v_dim + cols - 1) / cols));                                      \
    const size_t bytes = 2 * (size_t)kSsmStage * (2 * (NS > 1 ? NPT + 4 : NPT) * NS + cols + 4) * sizeof(float);              \
    if (scan4) hipLaunchKernelGGL((ssm_scan_kernel<NPT, NS, true>), dim3(blocks), dim3(64), bytes, s, a);                     \
    else hipLaunchKernelGGL((ssm_scan_kernel<NPT, NS, false>), dim3(blocks), dim3(64), bytes, s, a);                          \
  } while (0)
  if (state_size <= 16) SEMIPD_SSM_SCAN(16, 1);
  else if (state_size <= 32) SEMIPD_SSM_SCAN(32, 1);
  else if (state_size <= 64) SEMIPD_SSM_SCAN(32, 2);
  else if (state_size <= 128) SEMIPD_SSM_SCAN(32, 4);
  else SEMIPD_SSM_SCAN(32, 8);
#undef SEMIPD_SSM_SCAN
  SEMIPD_DISPATCH_DTYPE(dtype, T, hipLaunchKernelGGL((ssm_post_kernel<T>), dim3((unsigned)num_tokens), dim3(256), 0, s, a));
  return launch_status("state_space");
}
