// Mixers that carry a matrix of fixed size from token to token instead of a growing cache.
//
// A head keeps S [D][V] in float32 for every request slot.  With a decay a_t [D] (one number a key
// channel, acting on the rows of S), a key k_t [D], a value v_t [V] and a query q_t [D]:
//
//   rule 0 (gated linear attention):  S <- diag(a_t) S + k_t v_t^T;                    o_t = S^T q_t
//   rule 1 (gated delta rule):        S <- diag(a_t) S;  u = b_t (v_t - S^T k_t);
//                                     S <- S + k_t u^T;                                o_t = S^T q_t
//   rule 2 (state-space duality):     S <- diag(a_t) S + k_t (b_t v_t)^T;              o_t = S^T q_t
//                                     (b_t the step size a head; with `decay_per_head` a_t is one number a head)
//
// `linear_scan` walks the tokens that a step brings for a request one after the other, from the
// state that the steps before left in the request's slot, and leaves the new state there: a
// portion of a prompt and a single token are the same kernel, and a token's result does not
// depend on where its prompt was cut.  A wave owns four columns of S, a lane a sixteenth of the rows of
// one of them; the sixteen lanes of a column add their parts up in a fixed order.  In memory the state of a
// head lies in blocks of four columns, each in the order in which a wave's lanes hold it.
//
// Around it, each in float32 whatever the engine's dtype:
//   short_conv          y_t = act(sum_j taps[K-1-j] (x_(t-j) + in_bias) + out_bias) per channel, act the SiLU or
//                       nothing, the K-1 inputs before the step's first token from the slot's state (zeros at a
//                       sequence's start, also where the inputs have a bias)
//   short_conv_keep     the slot's state <- the last K-1 inputs (with their bias)
//   unit_heads          x / sqrt(sum(x^2) + eps) * factor over each head
//   scan_gate           what a projection becomes before it enters the recurrence:
//                       0  exp(-exp(A[head]) softplus(z + bias))      (a decay from a step size)
//                       1  exp(logsigmoid(z + bias) / tau)            (a decay sigmoid(z)^(1/tau))
//                       2  sigmoid(z)                                 (a writing strength)
//                       3  z * factor for the first columns, z for the rest (a cast)
//                       4  softplus(z + bias)                         (a step size)
//   rglru_scan          the real-gated linear recurrent unit, a number a channel:
//                       a = exp(rate * sigmoid(r)), S <- a S + sqrt(1 - a^2) sigmoid(i) u, out = S * gelu(y + bias)
//   gate_group_norm     out = norm((o + D[head] x) * silu(z)) * weight, the norm over each of `groups` equal parts
//   head_norm_gate      out = o / sqrt(mean(o^2) + eps) * weight * act(gate) over each head,
//                       act the sigmoid or the SiLU, in the engine's dtype for the product behind it
#include "common.h"

using namespace hfee;

namespace {

__device__ __forceinline__ float softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// x: [n, C] rows of the step; state: [slots][K-1][C], index K-2 the newest; taps: float32 [C][K], the
// last column the current token's; y: float32 [n, C].
// An input's bias is added before the input is rounded to T, in the step's rows here as in the rows
// that short_conv_keep leaves in the state: a token's result does not depend on where its sequence was cut.
template <typename T>
__device__ __forceinline__ float conv_input(const T* p, const float* in_bias, int c) {
  const float v = to_float<T>(*p);
  return in_bias != nullptr ? to_float<T>(from_float<T>(v + in_bias[c])) : v;
}

template <typename T>
__global__ __launch_bounds__(256) void short_conv_silu_kernel(
    float* __restrict__ y, int64_t ldy, const T* __restrict__ x, int64_t ldx, const T* __restrict__ state,
    const float* __restrict__ taps, const int* __restrict__ token_segment, const int* __restrict__ segment_rows,
    const int* __restrict__ segment_slots, int C, int K, const float* __restrict__ in_bias,
    const float* __restrict__ out_bias, int act) {
  const int t = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int seg = token_segment[t];
  const int i = t - segment_rows[seg];                      // the token's place in its portion
  const T* st = state + (int64_t)segment_slots[seg] * (K - 1) * C;
  float sum = 0.f;
  for (int j = K - 1; j >= 0; --j) {                        // the oldest input first
    const int at = i - j;
    const float v = at >= 0 ? conv_input<T>(x + (int64_t)(t - j) * ldx + c, in_bias, c) : to_float<T>(st[(int64_t)(K - 1 + at) * C + c]);
    sum = fmaf(taps[(int64_t)c * K + (K - 1 - j)], v, sum);
  }
  if (out_bias != nullptr) sum += out_bias[c];
  y[(int64_t)t * ldy + c] = act == 1 ? sum / (1.0f + expf(-sum)) : sum;
}

template <typename T>
__global__ __launch_bounds__(256) void short_conv_keep_kernel(
    T* __restrict__ state, const T* __restrict__ x, int64_t ldx, const int* __restrict__ segment_rows,
    const int* __restrict__ segment_lengths, const int* __restrict__ segment_slots, int C, int K,
    const float* __restrict__ in_bias) {
  const int seg = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int len = segment_lengths[seg], row0 = segment_rows[seg];
  T* st = state + (int64_t)segment_slots[seg] * (K - 1) * C;
  for (int m = 0; m < K - 1; ++m) {                         // ascending: what is read lies behind what was written
    const int i = len - (K - 1) + m;
    st[(int64_t)m * C + c] = i >= 0 ? from_float<T>(conv_input<T>(x + (int64_t)(row0 + i) * ldx + c, in_bias, c))
                                    : st[(int64_t)(m + len) * C + c];
  }
}

// One wave a (token, head): x float32 [n, heads * D], in place.
__global__ __launch_bounds__(256) void unit_heads_kernel(float* __restrict__ x, int64_t ldx, int heads, int D, float eps,
                                                         float factor, int n) {
  const int64_t item = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (item >= (int64_t)n * heads) return;
  const int lane = threadIdx.x & 63;
  float* p = x + item / heads * ldx + item % heads * D;
  float ss = 0.f;
  for (int d = lane; d < D; d += 64) ss = fmaf(p[d], p[d], ss);
  const float inv = factor / sqrtf(wave_sum(ss) + eps);
  for (int d = lane; d < D; d += 64) p[d] *= inv;
}

template <typename T>
__global__ __launch_bounds__(256) void scan_gate_kernel(float* __restrict__ out, int64_t ldo, const T* __restrict__ z,
                                                        int64_t ldz, const float* __restrict__ bias,
                                                        const float* __restrict__ per_head, int head_width, int mode,
                                                        float number, int first_columns, int width) {
  const int64_t t = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= width) return;
  float v = to_float<T>(z[t * ldz + c]);
  if (bias != nullptr) v += bias[c];
  float r;
  if (mode == 0) r = expf(-expf(per_head[c / head_width]) * softplus(v));
  else if (mode == 1) r = expf(log_sigmoid(v) / number);
  else if (mode == 2) r = 1.0f / (1.0f + expf(-v));
  else if (mode == 4) r = softplus(v);
  else r = c < first_columns ? v * number : v;
  out[t * ldo + c] = r;
}

// grid (blocks of 16 columns, heads, segments), four waves; a wave owns four columns of S, lane =
// 16 * column + part, and a lane the rows d = DPT * part + i (i < DPT) of its column (DPT = D / 16 filled up
// to a power of two).  The state lies in memory as [slot][head][blocks of four columns][i][lane]: a wave's
// load or store is 256 neighbouring bytes; rows at and beyond D and columns at and beyond V are zeros
// that stay zeros.  The sixteen lanes of a column add their parts
// up in a fixed tree.  The keys, queries, decays, values and writing strengths of the next TB tokens are
// asked for by the whole workgroup while it works on the current TB, and wait in LDS: the walk over the
// tokens, which nothing can shorten, reads only LDS and registers.
constexpr int kScanParts = 16, kScanColumns = 4, kScanWaves = 4;

template <int DPT>
struct ScanShape {
  static constexpr int DP = kScanParts * DPT;                       // rows of S, filled up
  static constexpr int TB = DPT <= 8 ? 16 : DPT == 16 ? 8 : 4;      // tokens a block
  static constexpr int WIDE = 3 * TB * DP;                          // k, q, a of a block
  static constexpr int BUFFER = WIDE + TB * kScanWaves * kScanColumns + TB;
  static constexpr int PER_THREAD = WIDE / (kScanWaves * 64);
};

// What a lane needs of one token, read from a block in LDS (sixteen bytes a read where a lane has four
// rows or more).
template <int DPT>
struct ScanToken {
  float k[DPT], q[DPT], a[DPT], v, b;
  __device__ __forceinline__ void read(const float* buffer, int t, int d0, int column) {
    typedef ScanShape<DPT> Sh;
    typedef float f32x4_t __attribute__((ext_vector_type(4)));
    const float* kt = buffer + t * Sh::DP + d0;
    const float* qt = kt + Sh::TB * Sh::DP;
    const float* at = qt + Sh::TB * Sh::DP;
    if constexpr (DPT % 4 == 0) {
#pragma unroll
      for (int i = 0; i < DPT; i += 4) {
        const f32x4_t kv = *reinterpret_cast<const f32x4_t*>(kt + i), qv = *reinterpret_cast<const f32x4_t*>(qt + i),
                      av = *reinterpret_cast<const f32x4_t*>(at + i);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          k[i + j] = kv[j];
          q[i + j] = qv[j];
          a[i + j] = av[j];
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < DPT; ++i) {
        k[i] = kt[i];
        q[i] = qt[i];
        a[i] = at[i];
      }
    }
    v = buffer[Sh::WIDE + t * kScanWaves * kScanColumns + column];
    b = buffer[Sh::WIDE + Sh::TB * kScanWaves * kScanColumns + t];
  }
};

// Over the sixteen lanes of a column, which are one row of the data-parallel primitives: neighbours in a
// quad, the quads of a half, the halves.  Every step adds two numbers that both lanes of a pair hold the
// other way round, so all sixteen lanes end with the same bits.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float x) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, false));
}

__device__ __forceinline__ float column_sum(float x) {
  x += dpp_move<0xB1>(x);      // quad_perm [1, 0, 3, 2]
  x += dpp_move<0x4E>(x);      // quad_perm [2, 3, 0, 1]
  x += dpp_move<0x141>(x);     // row_half_mirror: lane i of eight reads lane 7 - i
  x += dpp_move<0x140>(x);     // row_mirror: lane i of sixteen reads lane 15 - i
  return x;
}

template <int DPT, int RULE>
__global__ __launch_bounds__(kScanWaves * 64) void linear_scan_kernel(
    float* __restrict__ out, int64_t ldo, float* __restrict__ state, const float* __restrict__ q, int64_t ldq,
    const float* __restrict__ k, int64_t ldk, const float* __restrict__ v, int64_t ldv, const float* __restrict__ decay,
    int64_t ldd, const float* __restrict__ beta, int64_t ldb, const int* __restrict__ segment_rows,
    const int* __restrict__ segment_lengths, const int* __restrict__ segment_slots, int heads, int qk_heads, int D, int V,
    int decay_per_head) {
  typedef ScanShape<DPT> Sh;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int seg = blockIdx.z, h = blockIdx.y, tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int part = lane & (kScanParts - 1), c = lane >> 4;
  const int block = blockIdx.x * kScanWaves + wave;                 // of four columns
  const int col = block * kScanColumns + c;
  const bool live = col < V;
  const int g = h / (heads / qk_heads);
  const int blocks = (V + kScanColumns - 1) / kScanColumns;
  const int d0 = part * DPT;
  // (a wave whose four columns all lie beyond V works on the last block's numbers and stores nothing)
  const bool mine = block < blocks;
  float* S = state + (((int64_t)segment_slots[seg] * heads + h) * blocks + (mine ? block : blocks - 1)) * (DPT * 64) + lane;
  float s[DPT];
#pragma unroll
  for (int i = 0; i < DPT; ++i) s[i] = S[i * 64];
  const int row0 = segment_rows[seg], len = segment_lengths[seg];

  if (len == 1) {      // a single token (every thread of the workgroup sees the same len): straight from memory
    const int64_t row = row0;
    float u = live ? v[row * ldv + (int64_t)h * V + col] : 0.f;
    float kk[DPT], qq[DPT], aa[DPT];
    const float* kp = k + row * ldk + (int64_t)g * D + d0;
    const float* qp = q + row * ldq + (int64_t)g * D + d0;
    const float* ap = decay + row * ldd + (decay_per_head ? (int64_t)h : (int64_t)h * D + d0);
    const int astep = decay_per_head ? 0 : 1;
    if (DPT % 4 == 0 && D == DPT * kScanParts &&
        (((uintptr_t)kp | (uintptr_t)qp | (decay_per_head ? (uintptr_t)0 : (uintptr_t)ap)) & 15) == 0) {
      typedef float f32x4_t __attribute__((ext_vector_type(4)));      // (sixteen bytes a load where the rows allow)
      const float one_decay = decay_per_head ? ap[0] : 0.f;
#pragma unroll
      for (int i = 0; i + 3 < DPT; i += 4) {
        const f32x4_t kv = *reinterpret_cast<const f32x4_t*>(kp + i), qv = *reinterpret_cast<const f32x4_t*>(qp + i);
        f32x4_t av = {one_decay, one_decay, one_decay, one_decay};
        if (!decay_per_head) av = *reinterpret_cast<const f32x4_t*>(ap + i);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          kk[i + j] = kv[j];
          qq[i + j] = qv[j];
          aa[i + j] = av[j];
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < DPT; ++i) {
        const bool in = d0 + i < D;
        kk[i] = in ? kp[i] : 0.f;
        qq[i] = in ? qp[i] : 0.f;
        aa[i] = in ? ap[i * astep] : 0.f;
      }
    }
    if constexpr (RULE == 1) {
      float p0 = 0.f, p1 = 0.f;
#pragma unroll
      for (int i = 0; i < DPT; ++i) {
        s[i] *= aa[i];
        if (i & 1) p1 = fmaf(s[i], kk[i], p1); else p0 = fmaf(s[i], kk[i], p0);
      }
      u = beta[row * ldb + h] * (u - column_sum(p0 + p1));
    }
    if constexpr (RULE == 2) u *= beta[row * ldb + h];
    float o0 = 0.f, o1 = 0.f;
#pragma unroll
    for (int i = 0; i < DPT; ++i) {
      if constexpr (RULE == 1) s[i] = fmaf(kk[i], u, s[i]);
      else s[i] = fmaf(s[i], aa[i], kk[i] * u);
      if (i & 1) o1 = fmaf(s[i], qq[i], o1); else o0 = fmaf(s[i], qq[i], o0);
        if (mine) S[i * 64] = s[i];
    }
    const float o = column_sum(o0 + o1);
    if (live && part == 0) out[row * ldo + (int64_t)h * V + col] = o;
    return;
  }

  float wide[Sh::PER_THREAD], narrow = 0.f, strength = 0.f;
  auto ask = [&](int first) {          // the block of tokens that begins at `first`, into registers
#pragma unroll
    for (int r = 0; r < Sh::PER_THREAD; ++r) {
      const int e = tid + r * kScanWaves * 64;
      const int which = e / (Sh::TB * Sh::DP), rest = e - which * (Sh::TB * Sh::DP);
      const int t = rest / Sh::DP, d = rest - t * Sh::DP;
      float x = 0.f;
      if (first + t < len && d < D) {
        const int64_t row = row0 + first + t;
        x = which == 0 ? k[row * ldk + (int64_t)g * D + d] : which == 1 ? q[row * ldq + (int64_t)g * D + d]
                                                                      : decay[row * ldd + (decay_per_head ? (int64_t)h : (int64_t)h * D + d)];
      }
      wide[r] = x;
    }
    {
      const int t = tid / (kScanWaves * kScanColumns), cc = tid - t * (kScanWaves * kScanColumns);
      const int column = blockIdx.x * kScanWaves * kScanColumns + cc;
      narrow = t < Sh::TB && first + t < len && column < V ? v[(int64_t)(row0 + first + t) * ldv + (int64_t)h * V + column] : 0.f;
    }
    if (RULE != 0 && tid < Sh::TB) strength = first + tid < len ? beta[(int64_t)(row0 + first + tid) * ldb + h] : 0.f;
  };
  auto put = [&](float* buffer) {
#pragma unroll
    for (int r = 0; r < Sh::PER_THREAD; ++r) buffer[tid + r * kScanWaves * 64] = wide[r];
    if (tid < Sh::TB * kScanWaves * kScanColumns) buffer[Sh::WIDE + tid] = narrow;
    if (RULE != 0 && tid < Sh::TB) buffer[Sh::WIDE + Sh::TB * kScanWaves * kScanColumns + tid] = strength;
  };

  ask(0);
  put(lds);
  __syncthreads();
  for (int first = 0, turn = 0; first < len; first += Sh::TB, turn ^= 1) {
    const float* buffer = lds + turn * Sh::BUFFER;
    const bool more = first + Sh::TB < len;
    if (more) ask(first + Sh::TB);
    const int count = min(Sh::TB, len - first);
    ScanToken<DPT> now, next;
    now.read(buffer, 0, d0, wave * kScanColumns + c);
    for (int t = 0; t < count; ++t) {
      if (t + 1 < count) next.read(buffer, t + 1, d0, wave * kScanColumns + c);      // (ahead of the sums that wait on one another)
      float u = now.v;
      if constexpr (RULE == 1) {
        float p0 = 0.f, p1 = 0.f;
#pragma unroll
        for (int i = 0; i < DPT; ++i) {
          s[i] *= now.a[i];
          if (i & 1) p1 = fmaf(s[i], now.k[i], p1); else p0 = fmaf(s[i], now.k[i], p0);
        }
        u = now.b * (now.v - column_sum(p0 + p1));
      }
      if constexpr (RULE == 2) u = now.b * now.v;
      float o0 = 0.f, o1 = 0.f;
#pragma unroll
      for (int i = 0; i < DPT; ++i) {
        if constexpr (RULE == 1) s[i] = fmaf(now.k[i], u, s[i]);
        else s[i] = fmaf(s[i], now.a[i], now.k[i] * u);
        if (i & 1) o1 = fmaf(s[i], now.q[i], o1); else o0 = fmaf(s[i], now.q[i], o0);
      }
      const float o = column_sum(o0 + o1);
      if (live && part == 0) out[(int64_t)(row0 + first + t) * ldo + (int64_t)h * V + col] = o;
      now = next;
    }
    if (more) put(lds + (turn ^ 1) * Sh::BUFFER);
    __syncthreads();
  }
  if (mine) {
#pragma unroll
    for (int i = 0; i < DPT; ++i) S[i * 64] = s[i];
  }
}

// One wave a (token, head).  o: float32 [n, heads * V]; gate: [n, heads * V] in T; weight: float32 [V].
template <typename T>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(T* __restrict__ out, int64_t ldo, const float* __restrict__ o,
                                                             int64_t ldi, const T* __restrict__ gate, int64_t ldg,
                                                             const float* __restrict__ weight, int heads, int V,
                                                             float eps, int act, int n) {
  const int64_t item = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (item >= (int64_t)n * heads) return;
  const int lane = threadIdx.x & 63;
  const int64_t t = item / heads, h = item % heads;
  const float* p = o + t * ldi + h * V;
  float ss = 0.f;
  for (int d = lane; d < V; d += 64) ss = fmaf(p[d], p[d], ss);
  const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)V + eps);
  for (int d = lane; d < V; d += 64) {
    const float z = to_float<T>(gate[t * ldg + h * V + d]);
    const float sig = 1.0f / (1.0f + expf(-z));
    out[t * ldo + h * V + d] = from_float<T>(p[d] * inv * weight[d] * (act == 0 ? sig : z * sig));
  }
}

// The real-gated linear recurrent unit: one number a channel and request.  A thread owns a channel and
// walks the tokens that the step brings for a request in order; what a token needs (its two gates, its
// input, the other branch) is asked for kRgTokens tokens at a time, all at once, and the chain from token
// to token is one multiply-add.  gates: float32 [n][blocks][2 * block] before their biases and sigmoids,
// a block's decay gates, then its input gates.  rate: float32 [W], what the decay gate is multiplied by
// to give the decay's logarithm (not positive).
constexpr int kRgTokens = 8;

__device__ __forceinline__ void rglru_token(float& decay, float& inject, float r, float g, float x, float bias_r,
                                            float bias_i, float rt) {
  const float log_a = rt / (1.0f + expf(-(r + bias_r)));
  decay = expf(log_a);
  inject = sqrtf(-expm1f(2.0f * log_a)) * x / (1.0f + expf(-(g + bias_i)));
}

template <typename T>
__global__ __launch_bounds__(256) void rglru_scan_kernel(
    T* __restrict__ out, int64_t ldo, float* __restrict__ state, const float* __restrict__ gates, int64_t ldg,
    const float* __restrict__ gate_bias, const float* __restrict__ u, int64_t ldu, const float* __restrict__ rate,
    const T* __restrict__ y, int64_t ldy, const float* __restrict__ y_bias, const int* __restrict__ segment_rows,
    const int* __restrict__ segment_lengths, const int* __restrict__ segment_slots, int W, int block) {
  const int seg = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= W) return;
  const int b = c / block, at_r = b * 2 * block + (c - b * block), at_i = at_r + block;
  const float bias_r = gate_bias[at_r], bias_i = gate_bias[at_i], rt = rate[c], yb = y_bias != nullptr ? y_bias[c] : 0.f;
  const int row0 = segment_rows[seg], len = segment_lengths[seg];
  float* sp = state + (int64_t)segment_slots[seg] * W + c;
  float S = *sp;
  for (int first = 0; first < len; first += kRgTokens) {
    float r[kRgTokens], g[kRgTokens], x[kRgTokens], z[kRgTokens];
#pragma unroll
    for (int j = 0; j < kRgTokens; ++j) {
      const bool in = first + j < len;
      const int64_t row = row0 + first + (in ? j : 0);
      r[j] = gates[row * ldg + at_r];
      g[j] = gates[row * ldg + at_i];
      x[j] = u[row * ldu + c];
      z[j] = to_float<T>(y[row * ldy + c]);
    }
#pragma unroll
    for (int j = 0; j < kRgTokens; ++j) {
      // 1 - a^2 = -(exp(2 log a) - 1): no cancellation where the decay is close to one
      rglru_token(r[j], g[j], r[j], g[j], x[j], bias_r, bias_i, rt);
      const float v = z[j] + yb;
      z[j] = 0.5f * v * (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
    }
#pragma unroll
    for (int j = 0; j < kRgTokens; ++j) {
      if (first + j < len) {
        S = fmaf(r[j], S, g[j]);
        out[(int64_t)(row0 + first + j) * ldo + c] = from_float<T>(S * z[j]);
      }
    }
  }
  *sp = S;
}

// The same unit for long portions, cut into chunks of kRgChunk tokens so that a portion of thousands of tokens
// is walked by as many threads as it has (channel, chunk) pairs instead of one a channel.  A chunk's tokens
// act on what comes into it as S -> P S + Q with P the product of its decays and Q its walk from zero:
//   chunk_ends   every chunk but a portion's last: P and Q, and the slot's state set aside (`starts`);
//   chunk_walk   a chunk's incoming S from `starts` through the chunks before it, one multiply-add a chunk in
//                their order (every thread of a channel does the same sums, so they agree on each chunk's
//                S to the bit); then the walk over its own tokens as in rglru_scan; the last chunk leaves
//                the state.
// ends: float32 [segments][chunks_most][2][W]; starts: float32 [segments][W].  Chunks count from the
// portion's first token, so how a prompt was cut moves the roundings of P S + Q and nothing else.
constexpr int kRgChunk = 32;

__global__ __launch_bounds__(256) void rglru_chunk_ends_kernel(
    float* __restrict__ ends, float* __restrict__ starts, int chunks_most, const float* __restrict__ state,
    const float* __restrict__ gates, int64_t ldg, const float* __restrict__ gate_bias, const float* __restrict__ u,
    int64_t ldu, const float* __restrict__ rate, const int* __restrict__ segment_rows,
    const int* __restrict__ segment_lengths, const int* __restrict__ segment_slots, int W, int block) {
  const int seg = blockIdx.z, chunk = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
  const int len = segment_lengths[seg], first = chunk * kRgChunk;
  if (c >= W || first >= len) return;
  if (chunk == 0) starts[(int64_t)seg * W + c] = state[(int64_t)segment_slots[seg] * W + c];
  if (first + kRgChunk >= len) return;          // (nothing comes behind a portion's last chunk)
  const int b = c / block, at_r = b * 2 * block + (c - b * block), at_i = at_r + block;
  const float bias_r = gate_bias[at_r], bias_i = gate_bias[at_i], rt = rate[c];
  const int64_t row0 = segment_rows[seg] + first;
  float P = 1.f, Q = 0.f;
  for (int t = 0; t < kRgChunk; t += kRgTokens) {
    float r[kRgTokens], g[kRgTokens], x[kRgTokens];
#pragma unroll
    for (int j = 0; j < kRgTokens; ++j) {
      const int64_t row = row0 + t + j;
      r[j] = gates[row * ldg + at_r];
      g[j] = gates[row * ldg + at_i];
      x[j] = u[row * ldu + c];
    }
#pragma unroll
    for (int j = 0; j < kRgTokens; ++j) rglru_token(r[j], g[j], r[j], g[j], x[j], bias_r, bias_i, rt);
#pragma unroll
    for (int j = 0; j < kRgTokens; ++j) {
      P *= r[j];
      Q = fmaf(r[j], Q, g[j]);
    }
  }
  float* e = ends + ((int64_t)seg * chunks_most + chunk) * 2 * W + c;
  e[0] = P;
  e[W] = Q;
}

template <typename T>
__global__ __launch_bounds__(256) void rglru_chunk_walk_kernel(
    T* __restrict__ out, int64_t ldo, float* __restrict__ state, const float* __restrict__ ends,
    const float* __restrict__ starts, int chunks_most, const float* __restrict__ gates, int64_t ldg,
    const float* __restrict__ gate_bias, const float* __restrict__ u, int64_t ldu, const float* __restrict__ rate,
    const T* __restrict__ y, int64_t ldy, const float* __restrict__ y_bias, const int* __restrict__ segment_rows,
    const int* __restrict__ segment_lengths, const int* __restrict__ segment_slots, int W, int block) {
  const int seg = blockIdx.z, chunk = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
  const int len = segment_lengths[seg], first = chunk * kRgChunk;
  if (c >= W || first >= len) return;
  const int b = c / block, at_r = b * 2 * block + (c - b * block), at_i = at_r + block;
  const float bias_r = gate_bias[at_r], bias_i = gate_bias[at_i], rt = rate[c], yb = y_bias != nullptr ? y_bias[c] : 0.f;
  float S = starts[(int64_t)seg * W + c];
  const float* e = ends + (int64_t)seg * chunks_most * 2 * W + c;
  for (int k = 0; k < chunk; k += 8) {
    float P[8], Q[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int kk = k + j < chunk ? k + j : k;
      P[j] = e[(int64_t)kk * 2 * W];
      Q[j] = e[(int64_t)kk * 2 * W + W];
    }
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (k + j < chunk) S = fmaf(P[j], S, Q[j]);
  }
  const int64_t row0 = segment_rows[seg] + first;
  const int count = len - first < kRgChunk ? len - first : kRgChunk;
  for (int t = 0; t < count; t += kRgTokens) {
    float r[kRgTokens], g[kRgTokens], x[kRgTokens], z[kRgTokens];
#pragma unroll
    for (int j = 0; j < kRgTokens; ++j) {
      const int64_t row = row0 + t + (t + j < count ? j : 0);
      r[j] = gates[row * ldg + at_r];
      g[j] = gates[row * ldg + at_i];
      x[j] = u[row * ldu + c];
      z[j] = to_float<T>(y[row * ldy + c]);
    }
#pragma unroll
    for (int j = 0; j < kRgTokens; ++j) {
      rglru_token(r[j], g[j], r[j], g[j], x[j], bias_r, bias_i, rt);
      const float v = z[j] + yb;
      z[j] = 0.5f * v * (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
    }
#pragma unroll
    for (int j = 0; j < kRgTokens; ++j) {
      if (t + j < count) {
        S = fmaf(r[j], S, g[j]);
        out[(row0 + t + j) * ldo + c] = from_float<T>(S * z[j]);
      }
    }
  }
  if (first + kRgChunk >= len) state[(int64_t)segment_slots[seg] * W + c] = S;
}

// One workgroup a (token, part).  o: float32 [n, inner], what the recurrence read; x: float32 [n, inner],
// the recurrence's input, of which skip[head] times is added; z: the gate's branch in T; weight: float32 [inner].
template <typename T>
__global__ __launch_bounds__(256) void gate_group_norm_kernel(
    T* __restrict__ out, int64_t ldo, const float* __restrict__ o, int64_t ldi, const float* __restrict__ x, int64_t ldx,
    const float* __restrict__ skip, int head_width, const T* __restrict__ z, int64_t ldz,
    const float* __restrict__ weight, int part_width, float eps) {
  __shared__ float scratch[16];
  const int64_t t = blockIdx.x;
  const int j0 = blockIdx.y * part_width;
  float ss = 0.f;
  for (int j = j0 + threadIdx.x; j < j0 + part_width; j += blockDim.x) {
    const float g = to_float<T>(z[t * ldz + j]);
    const float v = fmaf(skip[j / head_width], x[t * ldx + j], o[t * ldi + j]) * (g / (1.0f + expf(-g)));
    ss = fmaf(v, v, ss);
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)part_width + eps);
  for (int j = j0 + threadIdx.x; j < j0 + part_width; j += blockDim.x) {
    const float g = to_float<T>(z[t * ldz + j]);
    const float v = fmaf(skip[j / head_width], x[t * ldx + j], o[t * ldi + j]) * (g / (1.0f + expf(-g)));
    out[t * ldo + j] = from_float<T>(v * inv * weight[j]);
  }
}

}  // namespace

HFEE_API int hfee_short_conv_silu(float* y, int64_t ldy, const void* x, int64_t ldx, const void* state, int dtype,
                                  const float* taps, const int* token_segment, const int* segment_rows,
                                  const int* segment_slots, int channels, int taps_count, int n, const float* in_bias,
                                  const float* out_bias, int act, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && channels > 0 && taps_count >= 1 && taps_count <= 64, "short_conv_silu: bad sizes");
  HFEE_REQUIRE(act == 0 || act == 1, "short_conv: the activation is none (0) or the SiLU (1)");
  if (n == 0) return 0;
  HFEE_REQUIRE(ldx >= channels && ldy >= channels && (channels + 255) / 256 <= 65535, "short_conv_silu: rows too short or too wide");
  dim3 grid(n, (channels + 255) / 256);
  if (dtype == 0)
    short_conv_silu_kernel<float><<<grid, 256, 0, stream>>>(y, ldy, (const float*)x, ldx, (const float*)state, taps,
        token_segment, segment_rows, segment_slots, channels, taps_count, in_bias, out_bias, act);
  else if (dtype == 1)
    short_conv_silu_kernel<bf16_t><<<grid, 256, 0, stream>>>(y, ldy, (const bf16_t*)x, ldx, (const bf16_t*)state, taps,
        token_segment, segment_rows, segment_slots, channels, taps_count, in_bias, out_bias, act);
  else
    return fail("short_conv_silu: unknown dtype %d", dtype);
  HFEE_CHECK_LAUNCH("short_conv_silu");
  return 0;
}

HFEE_API int hfee_short_conv_keep(void* state, const void* x, int64_t ldx, int dtype, const int* segment_rows,
                                  const int* segment_lengths, const int* segment_slots, int channels, int taps_count,
                                  int segments, const float* in_bias, hipStream_t stream) {
  HFEE_REQUIRE(segments >= 0 && segments <= 65535 && channels > 0 && taps_count >= 1, "short_conv_keep: bad sizes");
  if (segments == 0 || taps_count == 1) return 0;
  dim3 grid((channels + 255) / 256, segments);
  if (dtype == 0)
    short_conv_keep_kernel<float><<<grid, 256, 0, stream>>>((float*)state, (const float*)x, ldx, segment_rows,
        segment_lengths, segment_slots, channels, taps_count, in_bias);
  else if (dtype == 1)
    short_conv_keep_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)state, (const bf16_t*)x, ldx, segment_rows,
        segment_lengths, segment_slots, channels, taps_count, in_bias);
  else
    return fail("short_conv_keep: unknown dtype %d", dtype);
  HFEE_CHECK_LAUNCH("short_conv_keep");
  return 0;
}

HFEE_API int hfee_unit_heads(float* x, int64_t ldx, int heads, int dim, float eps, float factor, int n, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && heads > 0 && dim > 0 && ldx >= (int64_t)heads * dim, "unit_heads: bad sizes");
  if (n == 0) return 0;
  const int64_t items = (int64_t)n * heads;
  unit_heads_kernel<<<(unsigned)((items + 3) / 4), 256, 0, stream>>>(x, ldx, heads, dim, eps, factor, n);
  HFEE_CHECK_LAUNCH("unit_heads");
  return 0;
}

namespace {

// Rotation of projections on their way into a recurrence, in float32: out[t][h][d] (float32) from x[t][h][d]
// (the engine's dtype), `heads` heads of `dim` side by side (queries and keys of a token as one row).  The
// first 2 * half dims of a head are turned by the token's position (pairs (i, i + half), tables
// [positions][half]); heads from `scaled_from` on are multiplied by `factor` behind the rotation.
template <typename T>
__global__ __launch_bounds__(256) void rotate_rows_kernel(
    float* __restrict__ out, int64_t ldo, const T* __restrict__ x, int64_t ldx, const int* __restrict__ positions,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, int half, int heads, int dim, int scaled_from,
    float factor) {
  const int t = blockIdx.x;
  const float* c = cos_t + (int64_t)positions[t] * half;
  const float* s = sin_t + (int64_t)positions[t] * half;
  const T* xr = x + (int64_t)t * ldx;
  float* orow = out + (int64_t)t * ldo;
  for (int e = blockIdx.y * blockDim.x + threadIdx.x; e < heads * dim; e += gridDim.y * blockDim.x) {
    const int h = e / dim, d = e - h * dim;
    float v = to_float<T>(xr[e]);
    if (d < half) v = v * c[d] - to_float<T>(xr[e + half]) * s[d];
    else if (d < 2 * half) v = v * c[d - half] + to_float<T>(xr[e - half]) * s[d - half];
    orow[e] = h >= scaled_from ? v * factor : v;
  }
}

}  // namespace

HFEE_API int hfee_rotate_rows(float* out, int64_t ldo, const void* x, int64_t ldx, int dtype, const int* positions,
                              const float* cos_t, const float* sin_t, int half, int table_positions, int max_position,
                              int heads, int dim, int scaled_from, float factor, int n, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && heads > 0 && dim > 0 && half >= 0 && 2 * half <= dim, "rotate_rows: bad sizes");
  HFEE_REQUIRE(ldo >= (int64_t)heads * dim && ldx >= (int64_t)heads * dim, "rotate_rows: rows too short");
  HFEE_REQUIRE(half == 0 || (cos_t != nullptr && sin_t != nullptr && max_position < table_positions),
               "rotate_rows: position %d is beyond the rotation tables of %d positions", max_position, table_positions);
  if (n == 0) return 0;
  int parts = (heads * dim + 255) / 256;
  if (parts > 16) parts = 16;
  dim3 grid(n, parts);
  if (dtype == 0)
    rotate_rows_kernel<float><<<grid, 256, 0, stream>>>(out, ldo, (const float*)x, ldx, positions, cos_t, sin_t, half, heads,
                                                        dim, scaled_from, factor);
  else if (dtype == 1)
    rotate_rows_kernel<bf16_t><<<grid, 256, 0, stream>>>(out, ldo, (const bf16_t*)x, ldx, positions, cos_t, sin_t, half,
                                                         heads, dim, scaled_from, factor);
  else
    return fail("rotate_rows: unknown dtype %d", dtype);
  HFEE_CHECK_LAUNCH("rotate_rows");
  return 0;
}

HFEE_API int hfee_scan_gate(float* out, int64_t ldo, const void* z, int64_t ldz, int dtype, const float* bias,
                            const float* per_head, int head_width, int mode, float number, int first_columns, int n,
                            int width, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && width > 0 && (width + 255) / 256 <= 65535 && ldo >= width && ldz >= width, "scan_gate: bad sizes");
  HFEE_REQUIRE(mode >= 0 && mode <= 4, "scan_gate: unknown mode %d", mode);
  HFEE_REQUIRE(mode != 0 || (per_head != nullptr && head_width > 0), "scan_gate: a decay from a step size needs a number a head");
  HFEE_REQUIRE(mode != 1 || number > 0.f, "scan_gate: tau must be positive");
  if (n == 0) return 0;
  dim3 grid(n, (width + 255) / 256);
  if (dtype == 0)
    scan_gate_kernel<float><<<grid, 256, 0, stream>>>(out, ldo, (const float*)z, ldz, bias, per_head, head_width, mode,
                                                      number, first_columns, width);
  else if (dtype == 1)
    scan_gate_kernel<bf16_t><<<grid, 256, 0, stream>>>(out, ldo, (const bf16_t*)z, ldz, bias, per_head, head_width, mode,
                                                       number, first_columns, width);
  else
    return fail("scan_gate: unknown dtype %d", dtype);
  HFEE_CHECK_LAUNCH("scan_gate");
  return 0;
}

HFEE_API int hfee_linear_scan(float* out, int64_t ldo, float* state, const float* q, int64_t ldq, const float* k,
                              int64_t ldk, const float* v, int64_t ldv, const float* decay, int64_t ldd,
                              const float* beta, int64_t ldb, const int* segment_rows, const int* segment_lengths,
                              const int* segment_slots, int segments, int heads, int qk_heads, int dim, int vdim,
                              int rule, int decay_per_head, hipStream_t stream) {
  HFEE_REQUIRE(segments >= 0 && segments <= 65535, "linear_scan: bad segment count");
  if (segments == 0) return 0;
  HFEE_REQUIRE(heads > 0 && qk_heads > 0 && heads % qk_heads == 0 && heads <= 65535,
               "linear_scan: %d heads are not a multiple of %d query/key heads", heads, qk_heads);
  HFEE_REQUIRE(dim >= 1 && dim <= 512 && vdim >= 1, "linear_scan: key sizes of 1 to 512");
  HFEE_REQUIRE(rule == 0 || ((rule == 1 || rule == 2) && beta != nullptr && ldb >= heads),
               "linear_scan: rule 0, or rule 1 or 2 with a number a head and token");
  HFEE_REQUIRE(ldq >= (int64_t)qk_heads * dim && ldk >= (int64_t)qk_heads * dim && ldv >= (int64_t)heads * vdim &&
               (ldd >= (decay_per_head ? (int64_t)heads : (int64_t)heads * dim) || (decay_per_head && ldd == 0)) && ldo >= (int64_t)heads * vdim, "linear_scan: rows too short");
  const int columns = kScanWaves * kScanColumns;
  dim3 grid((vdim + columns - 1) / columns, heads, segments);
  const int per = (dim + kScanParts - 1) / kScanParts;
#define LAUNCH(DPT, RULE)                                                                                             \
  linear_scan_kernel<DPT, RULE><<<grid, kScanWaves * 64, 2 * ScanShape<DPT>::BUFFER * sizeof(float), stream>>>(out, ldo, state, q, ldq, k, ldk, v, ldv, decay, ldd, beta, ldb, \
      segment_rows, segment_lengths, segment_slots, heads, qk_heads, dim, vdim, decay_per_head)
#define PICK(RULE)                                                                                                    \
  if (per <= 1) LAUNCH(1, RULE); else if (per <= 2) LAUNCH(2, RULE); else if (per <= 4) LAUNCH(4, RULE);              \
  else if (per <= 8) LAUNCH(8, RULE); else if (per <= 16) LAUNCH(16, RULE); else LAUNCH(32, RULE)
  if (rule == 0) { PICK(0); } else if (rule == 1) { PICK(1); } else { PICK(2); }
#undef PICK
#undef LAUNCH
  HFEE_CHECK_LAUNCH("linear_scan");
  return 0;
}

HFEE_API int hfee_head_norm_gate(void* out, int64_t ldo, const float* o, int64_t ldi, const void* gate, int64_t ldg,
                                 int dtype, const float* weight, int heads, int vdim, float eps, int act, int n,
                                 hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && heads > 0 && vdim > 0 && (act == 0 || act == 1), "head_norm_gate: bad sizes");
  HFEE_REQUIRE(ldo >= (int64_t)heads * vdim && ldi >= (int64_t)heads * vdim && ldg >= (int64_t)heads * vdim,
               "head_norm_gate: rows too short");
  if (n == 0) return 0;
  const int64_t items = (int64_t)n * heads;
  const unsigned blocks = (unsigned)((items + 3) / 4);
  if (dtype == 0)
    head_norm_gate_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, ldo, o, ldi, (const float*)gate, ldg, weight,
                                                            heads, vdim, eps, act, n);
  else if (dtype == 1)
    head_norm_gate_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)out, ldo, o, ldi, (const bf16_t*)gate, ldg, weight,
                                                             heads, vdim, eps, act, n);
  else
    return fail("head_norm_gate: unknown dtype %d", dtype);
  HFEE_CHECK_LAUNCH("head_norm_gate");
  return 0;
}

// longest: the step's longest portion (host).  Portions of more than 2 * kRgChunk tokens go through the kernels
// in chunks, which need (segments * ceil(longest / kRgChunk) * 2 + segments) * width floats of scratch.
HFEE_API int hfee_rglru_scan(void* out, int64_t ldo, int dtype, float* state, const float* gates, int64_t ldg,
                             const float* gate_bias, const float* u, int64_t ldu, const float* rate, const void* y,
                             int64_t ldy, const float* y_bias, const int* segment_rows, const int* segment_lengths,
                             const int* segment_slots, int segments, int width, int block, int longest, float* scratch,
                             int64_t scratch_floats, hipStream_t stream) {
  HFEE_REQUIRE(segments >= 0 && segments <= 65535 && width > 0 && block > 0 && width % block == 0,
               "rglru_scan: %d channels are not whole blocks of %d", width, block);
  HFEE_REQUIRE(ldo >= width && ldu >= width && ldy >= width && ldg >= 2 * (int64_t)width, "rglru_scan: rows too short");
  HFEE_REQUIRE(gate_bias != nullptr && rate != nullptr, "rglru_scan: the gates' biases and the decay's rates");
  HFEE_REQUIRE(dtype == 0 || dtype == 1, "rglru_scan: unknown dtype %d", dtype);
  if (segments == 0) return 0;
  if (longest > 2 * kRgChunk && scratch != nullptr) {
    const int chunks_most = (longest + kRgChunk - 1) / kRgChunk;
    HFEE_REQUIRE(chunks_most <= 65535 && ((int64_t)segments * chunks_most * 2 + segments) * width <= scratch_floats,
                 "rglru_scan: %lld floats of scratch do not hold %d portions of up to %d chunks", (long long)scratch_floats,
                 segments, chunks_most);
    float* starts = scratch + (int64_t)segments * chunks_most * 2 * width;
    dim3 grid((width + 255) / 256, chunks_most, segments);
    rglru_chunk_ends_kernel<<<grid, 256, 0, stream>>>(scratch, starts, chunks_most, state, gates, ldg, gate_bias, u, ldu,
                                                      rate, segment_rows, segment_lengths, segment_slots, width, block);
    HFEE_CHECK_LAUNCH("rglru_scan (chunk ends)");
    if (dtype == 0)
      rglru_chunk_walk_kernel<float><<<grid, 256, 0, stream>>>((float*)out, ldo, state, scratch, starts, chunks_most, gates,
          ldg, gate_bias, u, ldu, rate, (const float*)y, ldy, y_bias, segment_rows, segment_lengths, segment_slots, width, block);
    else
      rglru_chunk_walk_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)out, ldo, state, scratch, starts, chunks_most, gates,
          ldg, gate_bias, u, ldu, rate, (const bf16_t*)y, ldy, y_bias, segment_rows, segment_lengths, segment_slots, width, block);
    HFEE_CHECK_LAUNCH("rglru_scan (chunk walk)");
    return 0;
  }
  dim3 grid((width + 255) / 256, segments);
  if (dtype == 0)
    rglru_scan_kernel<float><<<grid, 256, 0, stream>>>((float*)out, ldo, state, gates, ldg, gate_bias, u, ldu, rate,
        (const float*)y, ldy, y_bias, segment_rows, segment_lengths, segment_slots, width, block);
  else
    rglru_scan_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)out, ldo, state, gates, ldg, gate_bias, u, ldu, rate,
        (const bf16_t*)y, ldy, y_bias, segment_rows, segment_lengths, segment_slots, width, block);
  HFEE_CHECK_LAUNCH("rglru_scan");
  return 0;
}

HFEE_API int hfee_gate_group_norm(void* out, int64_t ldo, int dtype, const float* o, int64_t ldi, const float* x,
                                  int64_t ldx, const float* skip, int head_width, const void* z, int64_t ldz,
                                  const float* weight, int parts, int inner, float eps, int n, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && inner > 0 && parts > 0 && parts <= 65535 && inner % parts == 0 && head_width > 0 && inner % head_width == 0,
               "gate_group_norm: %d values are not %d equal parts (or whole heads of %d)", inner, parts, head_width);
  HFEE_REQUIRE(ldo >= inner && ldi >= inner && ldx >= inner && ldz >= inner && eps >= 0.f, "gate_group_norm: rows too short");
  if (n == 0) return 0;
  dim3 grid(n, parts);
  if (dtype == 0)
    gate_group_norm_kernel<float><<<grid, 256, 0, stream>>>((float*)out, ldo, o, ldi, x, ldx, skip, head_width,
        (const float*)z, ldz, weight, inner / parts, eps);
  else if (dtype == 1)
    gate_group_norm_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)out, ldo, o, ldi, x, ldx, skip, head_width,
        (const bf16_t*)z, ldz, weight, inner / parts, eps);
  else
    return fail("gate_group_norm: unknown dtype %d", dtype);
  HFEE_CHECK_LAUNCH("gate_group_norm");
  return 0;
}
