// Attention whose keys and values have sizes of their own, with an optional sink: the cache
// write with rotation of a part of each head, the plain attention kernel (one wave per (token,
// head), both dtypes, any sizes), and a small per-head product.
//
// One kernel family serves two mixers.  Grouped attention with a key size Dk and a value size
// Dv; and latent attention in its absorbed form: the per-head up-projection of the keys is
// moved onto the query, so that every head scores against the one cached row [latent | rotated
// part] (Dk = rank + rotated dims, one key/value head) and mixes the latents themselves
// (Dv = rank); the per-head value up-projection follows the attention.
//
// The paged cache of a layer here is [pages][kv_heads][page_size * (Dk + Dv)]: the keys of a
// (page, head) as [slot][Dk], then its values transposed as [Dv][slot] (`KvLayout`).
//
// softmax with a sink: the denominator holds one more term exp(sink_h), which has no key and
// no value: p_j = exp(s_j - m) / (exp(sink_h - m) + sum_i exp(s_i - m)), m the maximum over
// the scores and the sink.
//
// Without a softmax (`weighting` 1): a visible key weighs sigmoid(s_j + b_h), b_h a number a head (where
// the softmax has its sinks); the weights are not normalized over the keys.
//
// qk_norm_write is the other way into the cache: no rotation; q and k are divided by their root mean
// square over each head and multiplied by a weight shared by the heads, q also by a temperature that
// grows with the logarithm of the position in steps of `every` tokens:
// 1 + coef * ln(floor((p + 1) / every) + 1).
#include "attention_kv.h"

using namespace hfee;

namespace {

// ---------------------------------------------------------------- rotation + cache write
// A token's elements (pairs of q, elements of k and of v) are spread over the threads of
// gridDim.y workgroups.  q is rotated in place; k (rotated) and v (blended, if asked) go
// into the token's slot.  The rotated dims of a head are [rot_off, rot_off + 2 * half), pairs
// (i, i + half); cos/sin tables [positions][half] carry the amplitude.
template <typename T>
__global__ __launch_bounds__(256) void kv_write_kernel(
    T* __restrict__ q, int64_t ldq, int num_heads, int q_dim, int q_rot_off,
    const T* __restrict__ k, int64_t ldk, int k_rot_off, const T* __restrict__ v, int64_t ldv,
    T* __restrict__ v_first, int v_first_mode, const T* __restrict__ v_mix,
    const int* __restrict__ positions, const int* __restrict__ token_segment,
    const int* __restrict__ block_tables, int bt_stride, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, int half, T* __restrict__ cache, KvLayout lay) {
  const int t = blockIdx.x;
  const int pos = positions[t];
  const float* c = cos_t + (int64_t)pos * half;
  const float* s = sin_t + (int64_t)pos * half;
  const int first = blockIdx.y * blockDim.x + threadIdx.x, stride = gridDim.y * blockDim.x;
  if (q != nullptr) {
    T* qr = q + (int64_t)t * ldq;
    for (int e = first; e < num_heads * half; e += stride) {
      const int h = e / half, i = e - h * half;
      T* p = qr + (int64_t)h * q_dim + q_rot_off + i;
      const float a = to_float<T>(p[0]), b = to_float<T>(p[half]);
      p[0] = from_float<T>(a * c[i] - b * s[i]);
      p[half] = from_float<T>(b * c[i] + a * s[i]);
    }
  }
  if (k == nullptr) return;
  const int page = block_tables[(int64_t)token_segment[t] * bt_stride + (pos >> lay.page_shift)];
  const int slot = pos & (lay.page_size - 1);
  const T* kr = k + (int64_t)t * ldk;
  for (int e = first; e < lay.kv_heads * lay.dk; e += stride) {
    const int g = e / lay.dk, d = e - g * lay.dk;
    const int i = d - k_rot_off;
    float val;
    if (i >= 0 && i < half) {
      val = to_float<T>(kr[e]) * c[i] - to_float<T>(kr[e + half]) * s[i];
    } else if (i >= half && i < 2 * half) {
      val = to_float<T>(kr[e]) * c[i - half] + to_float<T>(kr[e - half]) * s[i - half];
    } else {
      val = to_float<T>(kr[e]);
    }
    cache[lay.key_offset(page, g, slot, d)] = finite_for_cache<T>(from_float<T>(val));
  }
  const T* vr = v + (int64_t)t * ldv;
  const int vw = lay.kv_heads * lay.dv;
  const float lam = v_first_mode == 2 ? to_float<T>(v_mix[0]) : 0.f;
  for (int e = first; e < vw; e += stride) {
    const int g = e / lay.dv, d = e - g * lay.dv;
    T val = vr[e];
    if (v_first_mode == 1) {
      v_first[(int64_t)t * vw + e] = val;
    } else if (v_first_mode == 2) {
      val = from_float<T>((1.0f - lam) * to_float<T>(val) + lam * to_float<T>(v_first[(int64_t)t * vw + e]));
    }
    cache[lay.value_offset(page, g, slot, d)] = finite_for_cache<T>(val);
  }
}

// ---------------------------------------------------------------- norm of q and k + cache write
// One wave a (token, unit): the units of a token are its query heads (normed in place), its key heads
// (normed into the token's slot) and its value heads (copied into the slot).  qw, kw: float32 [dk].
template <typename T>
__global__ __launch_bounds__(256) void qk_norm_write_kernel(
    T* __restrict__ q, int64_t ldq, int num_heads, const T* __restrict__ k, int64_t ldk, const T* __restrict__ v,
    int64_t ldv, const float* __restrict__ qw, const float* __restrict__ kw, float eps, float temp_coef, int temp_every,
    const int* __restrict__ positions, const int* __restrict__ token_segment, const int* __restrict__ block_tables,
    int bt_stride, T* __restrict__ cache, KvLayout lay, int n) {
  const int units = num_heads + (k != nullptr ? 2 * lay.kv_heads : 0);
  const int64_t item = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (item >= (int64_t)n * units) return;
  const int t = (int)(item / units), unit = (int)(item % units), lane = threadIdx.x & 63;
  const int pos = positions[t];
  if (unit < num_heads) {
    T* p = q + (int64_t)t * ldq + (int64_t)unit * lay.dk;
    float ss = 0.f;
    for (int d = lane; d < lay.dk; d += 64) {
      const float x = to_float<T>(p[d]);
      ss = fmaf(x, x, ss);
    }
    float factor = 1.0f / sqrtf(wave_sum(ss) / (float)lay.dk + eps);
    if (temp_every > 0) factor *= 1.0f + temp_coef * logf((float)((pos + 1) / temp_every) + 1.0f);
    for (int d = lane; d < lay.dk; d += 64) p[d] = from_float<T>(to_float<T>(p[d]) * factor * qw[d]);
    return;
  }
  const int page = block_tables[(int64_t)token_segment[t] * bt_stride + (pos >> lay.page_shift)];
  const int slot = pos & (lay.page_size - 1);
  if (unit < num_heads + lay.kv_heads) {
    const int g = unit - num_heads;
    const T* p = k + (int64_t)t * ldk + (int64_t)g * lay.dk;
    float ss = 0.f;
    for (int d = lane; d < lay.dk; d += 64) {
      const float x = to_float<T>(p[d]);
      ss = fmaf(x, x, ss);
    }
    const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)lay.dk + eps);
    for (int d = lane; d < lay.dk; d += 64)
      cache[lay.key_offset(page, g, slot, d)] = finite_for_cache<T>(from_float<T>(to_float<T>(p[d]) * inv * kw[d]));
    return;
  }
  const int g = unit - num_heads - lay.kv_heads;
  const T* p = v + (int64_t)t * ldv + (int64_t)g * lay.dv;
  for (int d = lane; d < lay.dv; d += 64) cache[lay.value_offset(page, g, slot, d)] = finite_for_cache<T>(p[d]);
}

// ---------------------------------------------------------------- rotation + value norm + cache write, from float32
// One wave a (token, unit), for projections that arrive in float32 (behind a short convolution): the
// units of a token are its query heads (rotated, written to q_out in the cache's dtype), its key heads
// (rotated into the token's slot) and its value heads (divided by their root mean square over the head
// where value_eps >= 0, into the slot).  The first 2 * half dims of a q or k head are rotated, pairs
// (i, i + half); cos/sin tables [positions][half].
template <typename T>
__global__ __launch_bounds__(256) void rotate_norm_write_kernel(
    T* __restrict__ q_out, int64_t ldqo, const float* __restrict__ q, int64_t ldq, int num_heads,
    const float* __restrict__ k, int64_t ldk, const float* __restrict__ v, int64_t ldv, float value_eps,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, int half,
    const int* __restrict__ positions, const int* __restrict__ token_segment, const int* __restrict__ block_tables,
    int bt_stride, T* __restrict__ cache, KvLayout lay, int n) {
  const int units = num_heads + (k != nullptr ? 2 * lay.kv_heads : 0);
  const int64_t item = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (item >= (int64_t)n * units) return;
  const int t = (int)(item / units), unit = (int)(item % units), lane = threadIdx.x & 63;
  const int pos = positions[t];
  const float* c = cos_t + (int64_t)pos * half;
  const float* s = sin_t + (int64_t)pos * half;
  auto turned = [&](const float* p, int d) {
    if (d < half) return p[d] * c[d] - p[d + half] * s[d];
    if (d < 2 * half) return p[d] * c[d - half] + p[d - half] * s[d - half];
    return p[d];
  };
  if (unit < num_heads) {
    const float* p = q + (int64_t)t * ldq + (int64_t)unit * lay.dk;
    T* o = q_out + (int64_t)t * ldqo + (int64_t)unit * lay.dk;
    for (int d = lane; d < lay.dk; d += 64) o[d] = from_float<T>(turned(p, d));
    return;
  }
  const int page = block_tables[(int64_t)token_segment[t] * bt_stride + (pos >> lay.page_shift)];
  const int slot = pos & (lay.page_size - 1);
  if (unit < num_heads + lay.kv_heads) {
    const int g = unit - num_heads;
    const float* p = k + (int64_t)t * ldk + (int64_t)g * lay.dk;
    for (int d = lane; d < lay.dk; d += 64)
      cache[lay.key_offset(page, g, slot, d)] = finite_for_cache<T>(from_float<T>(turned(p, d)));
    return;
  }
  const int g = unit - num_heads - lay.kv_heads;
  const float* p = v + (int64_t)t * ldv + (int64_t)g * lay.dv;
  float inv = 1.0f;
  if (value_eps >= 0.f) {
    float ss = 0.f;
    for (int d = lane; d < lay.dv; d += 64) ss = fmaf(p[d], p[d], ss);
    inv = 1.0f / sqrtf(wave_sum(ss) / (float)lay.dv + value_eps);
  }
  for (int d = lane; d < lay.dv; d += 64)
    cache[lay.value_offset(page, g, slot, d)] = finite_for_cache<T>(from_float<T>(p[d] * inv));
}

// ---------------------------------------------------------------- pooled blocks
// One wave a (token, key/value head, 64 of the key's and value's dims): a token at the last position of a block of `pool` positions
// (position % pool == pool - 1) leaves the block's key and value in the pooled blocks' cache layer under
// the block's number: the means of the block's keys and values as the cache holds them, summed in the
// order of the positions in float32.  Every other token's wave has nothing to do.  Runs behind the
// launch that wrote the step's keys and values.
template <typename T>
__global__ __launch_bounds__(256) void kv_pool_write_kernel(
    const T* __restrict__ cache, T* __restrict__ pooled, KvLayout lay, int pool, const int* __restrict__ positions,
    const int* __restrict__ token_segment, const int* __restrict__ block_tables, int bt_stride,
    const int* __restrict__ pool_tables, int pool_bt_stride, int n) {
  const int parts = (lay.dk + lay.dv + 63) >> 6;
  const int64_t item = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (item >= (int64_t)n * lay.kv_heads * parts) return;
  const int part_of_row = (int)(item % parts), lane = threadIdx.x & 63;
  const int t = (int)(item / parts / lay.kv_heads), g = (int)(item / parts % lay.kv_heads);
  const int pos = positions[t];
  if (pos % pool != pool - 1) return;
  const int b = pos / pool;
  const int* bt = block_tables + (int64_t)token_segment[t] * bt_stride;
  const int* pbt = pool_tables + (int64_t)token_segment[t] * pool_bt_stride;
  const int to_page = pbt[b >> lay.page_shift], to_slot = b & (lay.page_size - 1);
  const float share = 1.0f / (float)pool;
  const int d = part_of_row * 64 + lane;
  if (d < lay.dk + lay.dv) {
    float sum = 0.f;
    for (int j0 = pos - pool + 1; j0 <= pos; j0 += 8) {       // eight loads on their way at a time, added in order
      T part[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int j = min(j0 + i, pos);
        const int page = bt[j >> lay.page_shift], slot = j & (lay.page_size - 1);
        part[i] = cache[d < lay.dk ? lay.key_offset(page, g, slot, d) : lay.value_offset(page, g, slot, d - lay.dk)];
      }
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (j0 + i <= pos) sum += to_float<T>(part[i]);
    }
    pooled[d < lay.dk ? lay.key_offset(to_page, g, to_slot, d) : lay.value_offset(to_page, g, to_slot, d - lay.dk)] =
        from_float<T>(sum * share);
  }
}

// ---------------------------------------------------------------- plain attention
// Lane (j mod 64) owns key j, so which lane adds which term depends only on the key's
// absolute position: a token's result does not change with the way the work was cut into
// steps, with the batch around it or with page numbers.
constexpr int kMaxDvPerLane = 16;     // value sizes up to 1,024

// What a query sees besides the keys up to its own position (`KeySight`): with a window it sees the last
// `window` positions, itself included; with pooled blocks it also sees, for every block of `pool`
// positions that lies wholly before the window, one key and one value (the block's means, kept in the
// pooled section of the cache under the block's number); a score may be capped as
// cap * tanh(score / cap) before it is weighed.  Tokens and blocks share one softmax.
template <typename T>
__global__ __launch_bounds__(64) void attention_kv_plain_kernel(
    T* __restrict__ out, int64_t ld_out, const T* __restrict__ q, int64_t ldq,
    const T* __restrict__ cache, KvLayout lay, const int* __restrict__ positions,
    const int* __restrict__ token_segment, const int* __restrict__ block_tables, int bt_stride,
    int num_heads, float scale, const float* __restrict__ sinks, int weighting, KeySight sight,
    const T* __restrict__ gate, int64_t ld_gate) {
  extern __shared__ float lds[];
  const int dk = lay.dk, dv = lay.dv;
  float* qs = lds;            // [dk]
  float* es = lds + dk;       // [64]
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int kvh = h / (num_heads / lay.kv_heads);
  const int pos = positions[t];
  const int* bt = block_tables + (int64_t)token_segment[t] * bt_stride;
  const int first = sight.first_key(pos), blocks = sight.pooled_blocks(pos);
  const T* pooled = static_cast<const T*>(sight.pooled);
  const int* pbt = sight.pool_tables + (int64_t)token_segment[t] * sight.pool_bt_stride;

  for (int d = lane; d < dk; d += 64) qs[d] = to_float<T>(q[(int64_t)t * ldq + (int64_t)h * dk + d]);
  __syncthreads();

  // the score of entry j of a layer (the tokens' or the pooled blocks'), as the softmax takes it
  auto score = [&](const T* section, const int* table, int j) {
    const T* kr = section + lay.key_offset(table[j >> lay.page_shift], kvh, j & (lay.page_size - 1), 0);
    float s = 0.f;
    for (int d = 0; d < dk; ++d) s = fmaf(qs[d], to_float<T>(kr[d]), s);
    return sight.capped(s * scale);
  };
  float m = -INFINITY;
  if (weighting == 0) {
    for (int base = 0; base < blocks; base += 64)
      if (base + lane < blocks) m = fmaxf(m, score(pooled, pbt, base + lane));
    for (int base = first & ~63; base <= pos; base += 64) {
      const int j = base + lane;
      if (j >= first && j <= pos) m = fmaxf(m, score(cache, bt, j));
    }
  }
  m = wave_max(m);
  const bool has_sink = sinks != nullptr && weighting == 0;
  const float sink = sinks != nullptr ? sinks[h] : 0.f;      // (without a softmax: the number that joins every score)
  if (has_sink) m = fmaxf(m, sink);

  float lsum = 0.f;
  float o[kMaxDvPerLane];
#pragma unroll
  for (int r = 0; r < kMaxDvPerLane; ++r) o[r] = 0.f;
  // entries [from, to] of a layer, 64 at a time from a multiple of 64: lane (j mod 64) owns entry j
  auto walk = [&](const T* section, const int* table, int from, int to) {
    for (int base = from & ~63; base <= to; base += 64) {
      const int j = base + lane;
      float e = 0.f;
      if (j >= from && j <= to) {
        const float s = score(section, table, j);
        e = weighting == 0 ? expf(s - m) : 1.0f / (1.0f + expf(-(s + sink)));
        lsum += e;
      }
      __syncthreads();
      es[lane] = e;
      __syncthreads();
      const int je = min(base + 63, to);
      for (int jj = max(base, from); jj <= je; ++jj) {
        const float w = es[jj - base];
        const int page = table[jj >> lay.page_shift], slot = jj & (lay.page_size - 1);
#pragma unroll
        for (int r = 0; r < kMaxDvPerLane; ++r) {
          const int d = lane + 64 * r;
          if (d < dv) o[r] = fmaf(w, to_float<T>(section[lay.value_offset(page, kvh, slot, d)]), o[r]);
        }
      }
    }
  };
  if (blocks > 0) walk(pooled, pbt, 0, blocks - 1);
  walk(cache, bt, first, pos);
  lsum = wave_sum(lsum);
  if (has_sink) lsum += expf(sink - m);
  if (weighting != 0) lsum = 1.0f;
  // a gate a head: the head's result times sigmoid(gate[t][h])
  const float g = gate != nullptr ? 1.0f / (1.0f + expf(-to_float<T>(gate[(int64_t)t * ld_gate + h]))) : 1.0f;
#pragma unroll
  for (int r = 0; r < kMaxDvPerLane; ++r) {
    const int d = lane + 64 * r;
    if (d < dv) out[(int64_t)t * ld_out + (int64_t)h * dv + d] = from_float<T>(o[r] / lsum * g);
  }
}

// ---------------------------------------------------------------- per-head product
// out[t, h, o] = sum_i w[h][i][o] * x[t, h, i] for o < n_out (w stored [heads][n_in][n_out], so
// that neighbouring threads read neighbouring weights); then `tail` elements x[t, h, n_in ..]
// are copied behind them.  A workgroup takes one head, kHeadLinearTokens tokens and 32 outputs;
// its 256 threads are 8 slices of the inputs x 32 outputs, each slice summed in ascending i and
// the slices added in their order: a token's result does not depend on the tokens beside it.
constexpr int kHeadLinearTokens = 8, kHeadLinearOutputs = 32, kHeadLinearSlices = 8;

template <typename T>
__global__ __launch_bounds__(256) void head_linear_kernel(
    T* __restrict__ out, int64_t ldo, int64_t out_head_stride, const T* __restrict__ x, int64_t ldx,
    int64_t x_head_stride, const T* __restrict__ w, int n_in, int n_out, int tail, int n) {
  extern __shared__ float xs[];      // [kTokens][n_in], then [slices][kTokens][32] partial sums
  float* part = xs + kHeadLinearTokens * n_in;
  const int h = blockIdx.y, t0 = blockIdx.x * kHeadLinearTokens, o0 = blockIdx.z * kHeadLinearOutputs;
  const int count = min(kHeadLinearTokens, n - t0);
  for (int e = threadIdx.x; e < kHeadLinearTokens * n_in; e += blockDim.x) {
    const int r = e / n_in, i = e - r * n_in;
    xs[e] = r < count ? to_float<T>(x[(int64_t)(t0 + r) * ldx + (int64_t)h * x_head_stride + i]) : 0.f;
  }
  __syncthreads();
  const int lane_o = threadIdx.x & (kHeadLinearOutputs - 1), slice = threadIdx.x / kHeadLinearOutputs;
  const int o = o0 + lane_o;
  const int per = (n_in + kHeadLinearSlices - 1) / kHeadLinearSlices;
  const int i0 = slice * per, i1 = min(n_in, i0 + per);
  const T* wh = w + (int64_t)h * n_in * n_out;
  float acc[kHeadLinearTokens];
#pragma unroll
  for (int r = 0; r < kHeadLinearTokens; ++r) acc[r] = 0.f;
  if (o < n_out) {
#pragma unroll 4
    for (int i = i0; i < i1; ++i) {
      const float wv = to_float<T>(wh[(int64_t)i * n_out + o]);
#pragma unroll
      for (int r = 0; r < kHeadLinearTokens; ++r) acc[r] = fmaf(wv, xs[r * n_in + i], acc[r]);
    }
  }
#pragma unroll
  for (int r = 0; r < kHeadLinearTokens; ++r) part[(slice * kHeadLinearTokens + r) * kHeadLinearOutputs + lane_o] = acc[r];
  __syncthreads();
  {
    const int r = threadIdx.x / kHeadLinearOutputs;       // 8 tokens x 32 outputs = the workgroup's 256 threads
    if (r < count && o < n_out) {
      float sum = 0.f;
#pragma unroll
      for (int sl = 0; sl < kHeadLinearSlices; ++sl) sum += part[(sl * kHeadLinearTokens + r) * kHeadLinearOutputs + lane_o];
      out[(int64_t)(t0 + r) * ldo + (int64_t)h * out_head_stride + o] = from_float<T>(sum);
    }
  }
  if (blockIdx.z == 0)
    for (int e = threadIdx.x; e < count * tail; e += blockDim.x) {
      const int r = e / tail, i = e - r * tail;
      out[(int64_t)(t0 + r) * ldo + (int64_t)h * out_head_stride + n_out + i] =
          x[(int64_t)(t0 + r) * ldx + (int64_t)h * x_head_stride + n_in + i];
    }
}

}  // namespace

HFEE_API int hfee_kv_write(void* q, int64_t ldq, int num_heads, int q_dim, int q_rot_off, const void* k, int64_t ldk,
                           int k_rot_off, const void* v, int64_t ldv, void* v_first, int v_first_mode,
                           const void* v_mix, int dtype, const int* positions, const int* token_segment,
                           const int* block_tables, int bt_stride, const float* cos_t, const float* sin_t, int half,
                           int table_positions, int max_position, void* cache, int kv_heads, int dk, int dv,
                           int page_size, int n, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0, "kv_write: bad token count");
  if (n == 0) return 0;
  HFEE_REQUIRE(q != nullptr || k != nullptr, "kv_write: nothing to do");
  HFEE_REQUIRE(half >= 0 && (half == 0 || (cos_t != nullptr && sin_t != nullptr)), "kv_write: rotation tables missing");
  HFEE_REQUIRE(half == 0 || max_position < table_positions,
               "kv_write: position %d is beyond the rotation tables of %d positions", max_position, table_positions);
  HFEE_REQUIRE(q == nullptr || (q_rot_off >= 0 && q_rot_off + 2 * half <= q_dim && ldq >= (int64_t)num_heads * q_dim),
               "kv_write: the rotated dims do not fit the query heads");
  HFEE_REQUIRE(v_first_mode >= 0 && v_first_mode <= 2 && (v_first_mode == 0 || v_first != nullptr) &&
               (v_first_mode != 2 || v_mix != nullptr), "kv_write: value blending needs its buffers");
  KvLayout lay;
  if (k != nullptr) {
    HFEE_REQUIRE(v != nullptr && cache != nullptr && token_segment != nullptr && block_tables != nullptr,
                 "kv_write: k, v, the cache and the block tables come together");
    if (make_kv_layout(&lay, kv_heads, dk, dv, page_size)) return 1;
    HFEE_REQUIRE(k_rot_off >= 0 && k_rot_off + 2 * half <= dk, "kv_write: the rotated dims do not fit the key heads");
    HFEE_REQUIRE(ldk >= (int64_t)kv_heads * dk && ldv >= (int64_t)kv_heads * dv, "kv_write: k/v rows too short");
  } else {
    lay = KvLayout{};
  }
  // few tokens: as many workgroups a token as its largest run of elements has blocks of 256 (at most 16)
  int most = num_heads * half;
  if (k != nullptr && kv_heads * dk > most) most = kv_heads * dk;
  if (k != nullptr && kv_heads * dv > most) most = kv_heads * dv;
  int parts = n >= 1024 ? 1 : (most + 255) / 256;
  if (parts > 16) parts = 16;
  if (parts < 1) parts = 1;
#define LAUNCH(T)                                                                                                    \
  kv_write_kernel<T><<<dim3(n, parts), 256, 0, stream>>>((T*)q, ldq, num_heads, q_dim, q_rot_off, (const T*)k, ldk, k_rot_off,    \
      (const T*)v, ldv, (T*)v_first, v_first_mode, (const T*)v_mix, positions, token_segment, block_tables,          \
      bt_stride, cos_t, sin_t, half, (T*)cache, lay)
  if (dtype == 0) LAUNCH(float);
  else if (dtype == 1) LAUNCH(bf16_t);
  else return fail("kv_write: unknown dtype %d", dtype);
#undef LAUNCH
  HFEE_CHECK_LAUNCH("kv_write");
  return 0;
}

HFEE_API int hfee_qk_norm_write(void* q, int64_t ldq, int num_heads, const void* k, int64_t ldk, const void* v, int64_t ldv,
                                int dtype, const float* q_weight, const float* k_weight, float eps, float temp_coef,
                                int temp_every, const int* positions, const int* token_segment, const int* block_tables,
                                int bt_stride, void* cache, int kv_heads, int dk, int dv, int page_size, int n,
                                hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && num_heads > 0 && q != nullptr && q_weight != nullptr && eps >= 0.f, "qk_norm_write: bad arguments");
  if (n == 0) return 0;
  KvLayout lay;
  if (make_kv_layout(&lay, kv_heads, dk, dv, page_size)) return 1;
  HFEE_REQUIRE(ldq >= (int64_t)num_heads * dk, "qk_norm_write: q rows too short");
  if (k != nullptr) {
    HFEE_REQUIRE(v != nullptr && cache != nullptr && k_weight != nullptr && token_segment != nullptr && block_tables != nullptr,
                 "qk_norm_write: k, v, the keys' weight, the cache and the block tables come together");
    HFEE_REQUIRE(ldk >= (int64_t)kv_heads * dk && ldv >= (int64_t)kv_heads * dv, "qk_norm_write: k/v rows too short");
  }
  const int64_t items = (int64_t)n * (num_heads + (k != nullptr ? 2 * kv_heads : 0));
  HFEE_REQUIRE((items + 3) / 4 <= 0x7fffffff, "qk_norm_write: too much work for one launch");
#define LAUNCH(T)                                                                                                    \
  qk_norm_write_kernel<T><<<(unsigned)((items + 3) / 4), 256, 0, stream>>>((T*)q, ldq, num_heads, (const T*)k, ldk,  \
      (const T*)v, ldv, q_weight, k_weight, eps, temp_coef, temp_every, positions, token_segment, block_tables,      \
      bt_stride, (T*)cache, lay, n)
  if (dtype == 0) LAUNCH(float);
  else if (dtype == 1) LAUNCH(bf16_t);
  else return fail("qk_norm_write: unknown dtype %d", dtype);
#undef LAUNCH
  HFEE_CHECK_LAUNCH("qk_norm_write");
  return 0;
}

HFEE_API int hfee_rotate_norm_write(void* q_out, int64_t ldqo, const float* q, int64_t ldq, int num_heads, const float* k,
                                    int64_t ldk, const float* v, int64_t ldv, float value_eps, int dtype, const float* cos_t,
                                    const float* sin_t, int half, int table_positions, int max_position,
                                    const int* positions, const int* token_segment, const int* block_tables, int bt_stride,
                                    void* cache, int kv_heads, int dk, int dv, int page_size, int n,
                                    hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && num_heads > 0 && q != nullptr && q_out != nullptr, "rotate_norm_write: bad arguments");
  if (n == 0) return 0;
  HFEE_REQUIRE(half >= 0 && 2 * half <= dk && (half == 0 || (cos_t != nullptr && sin_t != nullptr)),
               "rotate_norm_write: the rotated dims do not fit the heads, or their tables are missing");
  HFEE_REQUIRE(half == 0 || max_position < table_positions,
               "rotate_norm_write: position %d is beyond the rotation tables of %d positions", max_position, table_positions);
  KvLayout lay;
  if (make_kv_layout(&lay, kv_heads, dk, dv, page_size)) return 1;
  HFEE_REQUIRE(ldq >= (int64_t)num_heads * dk && ldqo >= (int64_t)num_heads * dk, "rotate_norm_write: q rows too short");
  if (k != nullptr) {
    HFEE_REQUIRE(v != nullptr && cache != nullptr && token_segment != nullptr && block_tables != nullptr,
                 "rotate_norm_write: k, v, the cache and the block tables come together");
    HFEE_REQUIRE(ldk >= (int64_t)kv_heads * dk && ldv >= (int64_t)kv_heads * dv, "rotate_norm_write: k/v rows too short");
  }
  const int64_t items = (int64_t)n * (num_heads + (k != nullptr ? 2 * kv_heads : 0));
  HFEE_REQUIRE((items + 3) / 4 <= 0x7fffffff, "rotate_norm_write: too much work for one launch");
#define LAUNCH(T)                                                                                                    \
  rotate_norm_write_kernel<T><<<(unsigned)((items + 3) / 4), 256, 0, stream>>>((T*)q_out, ldqo, q, ldq, num_heads, k, ldk, v, \
      ldv, value_eps, cos_t, sin_t, half, positions, token_segment, block_tables, bt_stride, (T*)cache, lay, n)
  if (dtype == 0) LAUNCH(float);
  else if (dtype == 1) LAUNCH(bf16_t);
  else return fail("rotate_norm_write: unknown dtype %d", dtype);
#undef LAUNCH
  HFEE_CHECK_LAUNCH("rotate_norm_write");
  return 0;
}

HFEE_API int hfee_kv_pool_write(const void* cache, void* pooled, int dtype, int pool, const int* positions,
                                const int* token_segment, const int* block_tables, int bt_stride, const int* pool_tables,
                                int pool_bt_stride, int kv_heads, int dk, int dv, int page_size, int n, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && pool >= 1 && cache != nullptr && pooled != nullptr && block_tables != nullptr && pool_tables != nullptr,
               "kv_pool_write: bad arguments");
  if (n == 0) return 0;
  KvLayout lay;
  if (make_kv_layout(&lay, kv_heads, dk, dv, page_size)) return 1;
  const int64_t items = (int64_t)n * kv_heads * ((dk + dv + 63) / 64);
  HFEE_REQUIRE((items + 3) / 4 <= 0x7fffffff, "kv_pool_write: too much work for one launch");
#define LAUNCH(T)                                                                                                    \
  kv_pool_write_kernel<T><<<(unsigned)((items + 3) / 4), 256, 0, stream>>>((const T*)cache, (T*)pooled, lay, pool, positions, \
      token_segment, block_tables, bt_stride, pool_tables, pool_bt_stride, n)
  if (dtype == 0) LAUNCH(float);
  else if (dtype == 1) LAUNCH(bf16_t);
  else return fail("kv_pool_write: unknown dtype %d", dtype);
#undef LAUNCH
  HFEE_CHECK_LAUNCH("kv_pool_write");
  return 0;
}

HFEE_API int hfee_attention_kv_plain(void* out, int64_t ld_out, const void* q, int64_t ldq, const void* cache,
                                     int dtype, const int* positions, const int* token_segment,
                                     const int* block_tables, int bt_stride, int num_heads, int kv_heads, int dk,
                                     int dv, int page_size, float scale, const float* sinks, int weighting, int window,
                                     int pool, float softcap, const void* pooled, const int* pool_tables, int pool_bt_stride,
                                     const void* gate, int64_t ld_gate, int n, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0, "attention_kv_plain: bad token count");
  KeySight sight;
  if (make_key_sight(&sight, window, pool, softcap, pooled, pool_tables, pool_bt_stride)) return 1;
  HFEE_REQUIRE(gate == nullptr || ld_gate >= num_heads, "attention_kv_plain: the gates' rows are too short");
  HFEE_REQUIRE(weighting == 0 || weighting == 1, "attention_kv_plain: the weights are a softmax's (0) or sigmoids (1)");
  if (n == 0) return 0;
  HFEE_REQUIRE(num_heads > 0 && kv_heads > 0 && num_heads % kv_heads == 0,
               "attention_kv_plain: %d heads are not a multiple of %d kv heads", num_heads, kv_heads);
  HFEE_REQUIRE(dk >= 1 && dk <= 4096 && dv >= 1 && dv <= 64 * kMaxDvPerLane,
               "attention_kv_plain: key size %d or value size %d is out of range", dk, dv);
  HFEE_REQUIRE(num_heads <= 65535, "attention_kv_plain: too many heads");
  HFEE_REQUIRE(ldq >= (int64_t)num_heads * dk && ld_out >= (int64_t)num_heads * dv, "attention_kv_plain: q/out row too short");
  KvLayout lay;
  if (make_kv_layout(&lay, kv_heads, dk, dv, page_size)) return 1;
  dim3 grid(n, num_heads);
  const size_t lds = (dk + 64) * sizeof(float);
  if (dtype == 0)
    attention_kv_plain_kernel<float><<<grid, 64, lds, stream>>>((float*)out, ld_out, (const float*)q, ldq,
        (const float*)cache, lay, positions, token_segment, block_tables, bt_stride, num_heads, scale, sinks, weighting,
        sight, (const float*)gate, ld_gate);
  else if (dtype == 1)
    attention_kv_plain_kernel<bf16_t><<<grid, 64, lds, stream>>>((bf16_t*)out, ld_out, (const bf16_t*)q, ldq,
        (const bf16_t*)cache, lay, positions, token_segment, block_tables, bt_stride, num_heads, scale, sinks, weighting,
        sight, (const bf16_t*)gate, ld_gate);
  else
    return fail("attention_kv_plain: unknown dtype %d", dtype);
  HFEE_CHECK_LAUNCH("attention_kv_plain");
  return 0;
}

namespace {

// The same products in float32 on the matrix cores, for steps of many tokens: a workgroup takes one head,
// 64 tokens and 128 outputs, a wave 64 x 32 of them as two tiles of `32x32x2` float32 products (full
// float32 operands and sums; nothing is rounded to fewer bits).  The tokens' inputs pass LDS in chunks of 64
// (rows one word longer than that, so that the 32 rows a wave reads lie in different banks), a wave reads its
// weights straight from memory, 32 neighbouring outputs a row.  An output's sum runs over the inputs in a
// fixed order whatever else the tile holds: a token's result does not depend on the tokens beside it.
typedef float f32x16_t __attribute__((ext_vector_type(16)));
constexpr int kHeadMatrixTokens = 64, kHeadMatrixOutputs = 128, kHeadMatrixInputs = 64;

__global__ __launch_bounds__(256) void head_linear_f32_matrix_kernel(
    float* __restrict__ out, int64_t ldo, int64_t out_head_stride, const float* __restrict__ x, int64_t ldx,
    int64_t x_head_stride, const float* __restrict__ w, int n_in, int n_out, int tail, int n) {
  __shared__ float xs[kHeadMatrixTokens][kHeadMatrixInputs + 1];
  const int h = blockIdx.y, t0 = blockIdx.x * kHeadMatrixTokens, o0 = blockIdx.z * kHeadMatrixOutputs;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 31, half = lane >> 5;
  const int o = o0 + wave * 32 + col;
  const float* wh = w + (int64_t)h * n_in * n_out;
  const float* xh = x + (int64_t)h * x_head_stride;
  f32x16_t acc0, acc1;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc0[v] = acc1[v] = 0.f;
  for (int k0 = 0; k0 < n_in; k0 += kHeadMatrixInputs) {
    const int count = min(kHeadMatrixInputs, n_in - k0);
    // a lane's weights of the chunk are asked for first, so that they travel while the inputs are put into LDS:
    // of each pair of inputs lanes 0..31 take the first, lanes 32..63 the second
    float b[kHeadMatrixInputs / 2];
#pragma unroll
    for (int p = 0; p < kHeadMatrixInputs / 2; ++p) {
      const int k = 2 * p + half;
      b[p] = k < count && o < n_out ? wh[(int64_t)(k0 + k) * n_out + o] : 0.f;
    }
    __syncthreads();                                   // (the chunk before has been read)
    for (int e = threadIdx.x; e < kHeadMatrixTokens * kHeadMatrixInputs; e += 256) {
      const int r = e / kHeadMatrixInputs, i = e - r * kHeadMatrixInputs;
      xs[r][i] = t0 + r < n && k0 + i < n_in ? xh[(int64_t)(t0 + r) * ldx + k0 + i] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int p = 0; p < kHeadMatrixInputs / 2; ++p) {    // (beyond `count` both operands are zero)
      const int k = 2 * p + half;
      acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(xs[col][k], b[p], acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(xs[32 + col][k], b[p], acc1, 0, 0, 0);
    }
  }
  if (o < n_out) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {                      // a lane's sixteen sums: rows 8 (v / 4) + 4 half + v % 4 of its column
      const int r = t0 + (v >> 2) * 8 + half * 4 + (v & 3);
      if (r < n) out[(int64_t)r * ldo + (int64_t)h * out_head_stride + o] = acc0[v];
      if (r + 32 < n) out[(int64_t)(r + 32) * ldo + (int64_t)h * out_head_stride + o] = acc1[v];
    }
  }
  if (blockIdx.z == 0) {
    const int count = min(kHeadMatrixTokens, n - t0);
    for (int e = threadIdx.x; e < count * tail; e += blockDim.x) {
      const int r = e / tail, i = e - r * tail;
      out[(int64_t)(t0 + r) * ldo + (int64_t)h * out_head_stride + n_out + i] =
          x[(int64_t)(t0 + r) * ldx + (int64_t)h * x_head_stride + n_in + i];
    }
  }
}

}  // namespace

HFEE_API int hfee_head_linear(void* out, int64_t ldo, int64_t out_head_stride, const void* x, int64_t ldx,
                              int64_t x_head_stride, const void* w, int dtype, int heads, int n_in, int n_out,
                              int tail, int n, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && heads > 0 && n_in > 0 && n_out > 0 && tail >= 0, "head_linear: bad sizes");
  if (n == 0) return 0;
  HFEE_REQUIRE(heads <= 65535 && n_in <= 1536, "head_linear: at most 65535 heads and 1536 inputs a head");
  HFEE_REQUIRE(x_head_stride >= n_in + tail && out_head_stride >= n_out + tail, "head_linear: heads overlap");
  HFEE_REQUIRE((n_out + kHeadLinearOutputs - 1) / kHeadLinearOutputs <= 65535, "head_linear: too many outputs a head");
  dim3 grid((n + kHeadLinearTokens - 1) / kHeadLinearTokens, heads, (n_out + kHeadLinearOutputs - 1) / kHeadLinearOutputs);
  const size_t lds = ((size_t)kHeadLinearTokens * n_in + kHeadLinearSlices * kHeadLinearTokens * kHeadLinearOutputs) * sizeof(float);
  if (dtype == 0 && n >= 32) {       // (out == x with a tail would be read and written by different workgroups: never so)
    dim3 tiles((n + kHeadMatrixTokens - 1) / kHeadMatrixTokens, heads, (n_out + kHeadMatrixOutputs - 1) / kHeadMatrixOutputs);
    head_linear_f32_matrix_kernel<<<tiles, 256, 0, stream>>>((float*)out, ldo, out_head_stride, (const float*)x, ldx,
        x_head_stride, (const float*)w, n_in, n_out, tail, n);
  } else if (dtype == 0)
    head_linear_kernel<float><<<grid, 256, lds, stream>>>((float*)out, ldo, out_head_stride, (const float*)x, ldx,
        x_head_stride, (const float*)w, n_in, n_out, tail, n);
  else if (dtype == 1)
    head_linear_kernel<bf16_t><<<grid, 256, lds, stream>>>((bf16_t*)out, ldo, out_head_stride, (const bf16_t*)x, ldx,
        x_head_stride, (const bf16_t*)w, n_in, n_out, tail, n);
  else
    return fail("head_linear: unknown dtype %d", dtype);
  HFEE_CHECK_LAUNCH("head_linear");
  return 0;
}
