// A feed-forward of many small gated experts, of which every token uses `top`.
//
// Which experts a token uses is given from outside as int32 [n, top] (`chosen`), or looked up here in
// a table [vocabulary, top] under the token's id; expert e of a token counts with pair_weights[t][j]
// or, without them, with the one number `weight`.
//
//   up:    act[t][j][f] = silu(W_gate[e][f] . h_t) * (W_up[e][f] . h_t),   e = the j-th expert of t
//   down:  x[t][c] (+)= sum_j weight_tj (W_down[e_j][c] . act[t][j])
//
// Experts without a gate (`form` 1, no W_gate): act[t][j][f] = relu(w_tj (W_up[e][f] . h_t))^2, where w_tj
// (in_weights, or one) multiplies the expert's input: a product is linear, so the number meets the sum in
// float32 before the activation instead of every element of h before it is rounded.
//
// router_topk: scores sigmoid(z) of router logits z (float32 [n, experts]); the `top` largest choose a
// token's experts (the lower number of two equal ones), its pair weights are the chosen scores as they are.
//
// The experts' matrices are stacked [experts][rows][columns].  Two forms:
//
// Token by token (moe_up, moe_down): a wave a dot product, lanes over the summed dimension, added up in a
// fixed order; every token reads the rows of its own experts.  For steps of few tokens, whose time is
// the experts' bytes, and for float32.
//
// Grouped (moe_group, moe_group_tiled, moe_combine; bfloat16): the (token, expert) pairs of a step are put
// in the order of their experts on the device, cut into tiles of 64 pairs of one expert, and a workgroup
// multiplies a tile by 256 rows of that expert's matrix on the matrix cores (both operands staged through
// LDS in steps of 32 columns, a wave 64 x 64 of v_mfma_f32_32x32x16_bf16): an expert's matrices are read
// once a 64 pairs and not once a pair.  A pair's numbers do not depend on which pairs share its tile.
#include "common.h"

using namespace hfee;

namespace {

__device__ __forceinline__ int expert_of(const int* chosen, const int* table, const int* token_ids, int t, int j, int top) {
  return chosen != nullptr ? chosen[(int64_t)t * top + j] : table[(int64_t)token_ids[t] * top + j];
}

constexpr int kRowsPerWave = 4;

// sum_c a[c] b[c] and sum_c a2[c] b[c] over `count` elements, a lane's share: lanes take turns of one
// element, or of eight bfloat16 (sixteen bytes) where count is a multiple of eight and the rows are aligned.
template <typename T>
__device__ __forceinline__ void two_dots(const T* a, const T* a2, const T* b, int count, int lane, bool wide, float& s, float& s2) {
  s = s2 = 0.f;
  if constexpr (sizeof(T) == 2) {
    if (wide) {
      typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
      for (int c = lane * 8; c < count; c += 64 * 8) {
        const u32x4_t va = load_streamed(reinterpret_cast<const u32x4_t*>(a + c));
        const u32x4_t vb = *reinterpret_cast<const u32x4_t*>(b + c);
        u32x4_t va2 = va;
        if (a2 != nullptr) va2 = load_streamed(reinterpret_cast<const u32x4_t*>(a2 + c));
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float b0 = __uint_as_float(vb[i] << 16), b1 = __uint_as_float(vb[i] & 0xffff0000u);
          s = fmaf(__uint_as_float(va[i] << 16), b0, s);
          s = fmaf(__uint_as_float(va[i] & 0xffff0000u), b1, s);
          if (a2 != nullptr) {
            s2 = fmaf(__uint_as_float(va2[i] << 16), b0, s2);
            s2 = fmaf(__uint_as_float(va2[i] & 0xffff0000u), b1, s2);
          }
        }
      }
      return;
    }
  }
  for (int c = lane; c < count; c += 64) {
    const float x = to_float<T>(b[c]);
    s = fmaf(to_float<T>(a[c]), x, s);
    if (a2 != nullptr) s2 = fmaf(to_float<T>(a2[c]), x, s2);
  }
}

template <typename T>
__device__ __forceinline__ bool rows_aligned(const T* a, const T* b, int count, int64_t row_stride_b) {
  return sizeof(T) == 2 && count % 8 == 0 && row_stride_b % 8 == 0 && ((uintptr_t)a | (uintptr_t)b) % 16 == 0;
}

template <typename T>
__global__ __launch_bounds__(256) void moe_up_kernel(T* __restrict__ act, const T* __restrict__ h, int64_t ldh,
                                                     const T* __restrict__ w_gate, const T* __restrict__ w_up,
                                                     const int* __restrict__ chosen, const int* __restrict__ table,
                                                     const int* __restrict__ token_ids, int top, int experts, int F,
                                                     int width, const float* __restrict__ in_weights) {
  const int pair = blockIdx.x, t = pair / top, j = pair - t * top;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int e = expert_of(chosen, table, token_ids, t, j, top);
  if (e < 0 || e >= experts) return;                       // (a table that names no such expert: nothing is read)
  const T* hr = h + (int64_t)t * ldh;
  const bool wide = rows_aligned<T>(w_up, h, width, ldh) && (uintptr_t)w_gate % 16 == 0;
  const int f0 = (blockIdx.y * 4 + wave) * kRowsPerWave;
  const float wt = in_weights != nullptr ? in_weights[pair] : 1.0f;
#pragma unroll
  for (int r = 0; r < kRowsPerWave; ++r) {
    const int f = f0 + r;
    if (f >= F) break;
    const T* u = w_up + ((int64_t)e * F + f) * width;
    float sg, su;
    if (w_gate == nullptr) {        // no gate: the square of relu
      two_dots<T>(u, nullptr, hr, width, lane, wide, su, sg);
      su = fmaxf(wave_sum(su) * wt, 0.f);
      if (lane == 0) act[(int64_t)pair * F + f] = from_float<T>(su * su);
      continue;
    }
    const T* g = w_gate + ((int64_t)e * F + f) * width;
    two_dots<T>(g, u, hr, width, lane, wide, sg, su);
    sg = wave_sum(sg);
    su = wave_sum(su);
    if (lane == 0) act[(int64_t)pair * F + f] = from_float<T>(sg / (1.0f + expf(-sg)) * su);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_down_kernel(float* __restrict__ x, int64_t ldx, const T* __restrict__ act,
                                                       const T* __restrict__ w_down, const int* __restrict__ chosen,
                                                       const int* __restrict__ table, const int* __restrict__ token_ids,
                                                       const float* __restrict__ pair_weights, float weight, int top,
                                                       int experts, int F, int width, int accumulate) {
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c0 = (blockIdx.y * 4 + wave) * kRowsPerWave;
  const bool wide = rows_aligned<T>(w_down, act, F, F);
#pragma unroll
  for (int r = 0; r < kRowsPerWave; ++r) {
    const int c = c0 + r;
    if (c >= width) break;
    float total = 0.f;
    for (int j = 0; j < top; ++j) {
      const int e = expert_of(chosen, table, token_ids, t, j, top);
      if (e < 0 || e >= experts) continue;
      const T* w = w_down + ((int64_t)e * width + c) * F;
      const T* a = act + ((int64_t)t * top + j) * F;
      float s, unused;
      two_dots<T>(w, nullptr, a, F, lane, wide, s, unused);
      total = fmaf(wave_sum(s), pair_weights != nullptr ? pair_weights[(int64_t)t * top + j] : weight, total);
    }
    if (lane == 0) {
      float* o = x + (int64_t)t * ldx + c;
      *o = accumulate ? *o + total : total;
    }
  }
}

// ---------------------------------------------------------------------------- grouped
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kTilePairs = 64, kTileRows = 256;

// One workgroup.  order: the pairs (t * top + j) by expert; tiles: (expert, first place in order, pairs)
// for every tile, tiles[3 * most_tiles] holds their number.  Which of an expert's pairs comes first is
// left to chance; nothing that is computed depends on it.
__global__ __launch_bounds__(1024) void moe_group_kernel(int* __restrict__ order, int* __restrict__ tiles, int most_tiles,
                                                         const int* __restrict__ chosen, const int* __restrict__ table,
                                                         const int* __restrict__ token_ids, int n, int top, int experts) {
  extern __shared__ int lds[];
  int* counts = lds;                  // [experts]
  int* starts = lds + experts;        // [experts]
  int* cursor = lds + 2 * experts;    // [experts]
  int* first_tile = lds + 3 * experts;
  const int pairs = n * top;
  for (int e = threadIdx.x; e < experts; e += blockDim.x) counts[e] = cursor[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
    const int e = expert_of(chosen, table, token_ids, p / top, p % top, top);
    if (e >= 0 && e < experts) atomicAdd(&counts[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, tile = 0;
    for (int e = 0; e < experts; ++e) {
      starts[e] = at;
      first_tile[e] = tile;
      at += counts[e];
      tile += (counts[e] + kTilePairs - 1) / kTilePairs;
    }
    tiles[3 * most_tiles] = tile;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
    const int e = expert_of(chosen, table, token_ids, p / top, p % top, top);
    if (e >= 0 && e < experts) order[starts[e] + atomicAdd(&cursor[e], 1)] = p;
  }
  for (int e = threadIdx.x; e < experts; e += blockDim.x)
    for (int i = 0; i * kTilePairs < counts[e]; ++i) {
      int* tl = tiles + 3 * (first_tile[e] + i);
      tl[0] = e;
      tl[1] = starts[e] + i * kTilePairs;
      tl[2] = min(kTilePairs, counts[e] - i * kTilePairs);
    }
}

// The grouped products through LDS.  A workgroup takes a tile of up to 64 pairs of one expert and 256 rows of
// weights (KIND 0: 128 rows of the gate's matrix and the same 128 of the up matrix); K in steps of 32: every
// thread asks for its 16-byte pieces of the next step (one of the pairs' rows, four of the weights') while the
// matrix cores work on the current one out of LDS, then lays them into the other buffer; rows of 40 elements
// so that the operand reads of 32 rows spread over the banks.  A wave owns 64 weight rows (KIND 0: 32 of each
// matrix) x 64 pairs as 2 x 2 tiles of `32x32x16`, the weights as the row operand, so that a lane ends with
// four neighbouring rows of the matrix for one pair and stores them at once.  A sum runs over K in the same
// order whichever pairs share the tile.
//   KIND 0: act = silu(gate) * up      KIND 1: act = relu(weight * up)^2      KIND 2: out (+)= scale * down
typedef float f32x16 __attribute__((ext_vector_type(16)));
constexpr int kStageK = 32, kStagePitch = 40;

template <int KIND>
__global__ __launch_bounds__(256) void moe_group_tiled_kernel(
    void* __restrict__ dst, int64_t ldo, const bf16_t* __restrict__ src, int64_t lds_rows, const bf16_t* __restrict__ w0,
    const bf16_t* __restrict__ w1, const int* __restrict__ order, const int* __restrict__ tiles, int most_tiles, int top,
    int n_rows, int K, int add, const float* __restrict__ pair_weights, float weight) {
  __shared__ __attribute__((aligned(16))) bf16_t As[2][kTilePairs * kStagePitch];
  __shared__ __attribute__((aligned(16))) bf16_t Ws[2][kTileRows * kStagePitch];
  if ((int)blockIdx.x >= tiles[3 * most_tiles]) return;
  const int* tl = tiles + 3 * blockIdx.x;
  const int e = tl[0], first = tl[1], count = tl[2];
  constexpr int kRowsOut = KIND == 0 ? kTileRows / 2 : kTileRows;      // rows of the result a workgroup makes
  const int row0 = blockIdx.y * kRowsOut;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  // what this thread brings of every step: piece (tid & 3) of pair row tid / 4, and of weight rows tid / 4 + 64 p
  const int piece = (tid & 3) * 8, srow = tid >> 2;
  const int my_pair = order[first + (srow < count ? srow : 0)];
  const bf16_t* a_src = src + (int64_t)(KIND == 2 ? my_pair : my_pair / top) * lds_rows + piece;
  const bf16_t* w_src[4];
  bool w_ok[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const int s = srow + 64 * p;                                        // the row's place in the staged tile
    const bf16_t* base = KIND == 0 && s >= kRowsOut ? w1 : w0;
    const int row = row0 + (KIND == 0 && s >= kRowsOut ? s - kRowsOut : s);
    w_ok[p] = row < n_rows;
    w_src[p] = base + ((int64_t)e * n_rows + (w_ok[p] ? row : 0)) * K + piece;
  }
  const u32x4 zero = {0u, 0u, 0u, 0u};
  u32x4 ra = *reinterpret_cast<const u32x4*>(a_src), rw[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) rw[p] = w_ok[p] ? *reinterpret_cast<const u32x4*>(w_src[p]) : zero;
  *reinterpret_cast<u32x4*>(&As[0][srow * kStagePitch + piece]) = ra;
#pragma unroll
  for (int p = 0; p < 4; ++p) *reinterpret_cast<u32x4*>(&Ws[0][(srow + 64 * p) * kStagePitch + piece]) = rw[p];
  __syncthreads();

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  const int lrow = lane & 31, lk = (lane >> 5) * 8;
  // the wave's two groups of 32 staged weight rows
  const int base_i[2] = {KIND == 0 ? wave * 32 : wave * 64, KIND == 0 ? kRowsOut + wave * 32 : wave * 64 + 32};
  const int steps = K / kStageK;
  int buf = 0;
  for (int kt = 0; kt < steps; ++kt) {
    if (kt + 1 < steps) {
      const int k = (kt + 1) * kStageK;
      ra = *reinterpret_cast<const u32x4*>(a_src + k);
#pragma unroll
      for (int p = 0; p < 4; ++p) rw[p] = w_ok[p] ? *reinterpret_cast<const u32x4*>(w_src[p] + k) : zero;
    }
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      bf16x8 a[2], b[2];
#pragma unroll
      for (int i = 0; i < 2; ++i)
        a[i] = *reinterpret_cast<const bf16x8*>(&Ws[buf][(base_i[i] + lrow) * kStagePitch + ks * 16 + lk]);
#pragma unroll
      for (int j = 0; j < 2; ++j)
        b[j] = *reinterpret_cast<const bf16x8*>(&As[buf][(j * 32 + lrow) * kStagePitch + ks * 16 + lk]);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < steps) {
      *reinterpret_cast<u32x4*>(&As[buf ^ 1][srow * kStagePitch + piece]) = ra;
#pragma unroll
      for (int p = 0; p < 4; ++p) *reinterpret_cast<u32x4*>(&Ws[buf ^ 1][(srow + 64 * p) * kStagePitch + piece]) = rw[p];
    }
    __syncthreads();
    buf ^= 1;
  }

  // register r of lane l in tile (i, j): row 8 (r / 4) + 4 (l / 32) + r % 4 of the wave's group i, pair 32 j + l % 32
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int at = j * 32 + lrow;
    if (at >= count) continue;
    const int pair = order[first + at];
    if constexpr (KIND == 0) {
      bf16_t* o = (bf16_t*)dst + (int64_t)pair * ldo;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int f = row0 + wave * 32 + 8 * q + 4 * (lane >> 5);
        if (f >= n_rows) continue;
        bf16_t four[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float g = acc[0][j][4 * q + r];
          four[r] = float_to_bf16(g / (1.0f + expf(-g)) * acc[1][j][4 * q + r]);
        }
        *reinterpret_cast<u32x2*>(o + f) = *reinterpret_cast<const u32x2*>(four);
      }
    } else {
      const float scale = KIND == 1 ? (pair_weights != nullptr ? pair_weights[pair] : 1.0f)
                                    : add ? (pair_weights != nullptr ? pair_weights[pair] : weight) : 1.0f;
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int f = row0 + wave * 64 + 32 * i + 8 * q + 4 * (lane >> 5);
          if (f >= n_rows) continue;
          if constexpr (KIND == 1) {
            bf16_t four[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const float u = fmaxf(acc[i][j][4 * q + r] * scale, 0.f);
              four[r] = float_to_bf16(u * u);
            }
            *reinterpret_cast<u32x2*>((bf16_t*)dst + (int64_t)pair * ldo + f) = *reinterpret_cast<const u32x2*>(four);
          } else {
            float* o = (float*)dst + (int64_t)pair * ldo + f;
#pragma unroll
            for (int r = 0; r < 4; ++r) o[r] = add ? fmaf(acc[i][j][4 * q + r], scale, o[r]) : acc[i][j][4 * q + r];
          }
        }
    }
  }
}

// x[t] += sum_j weight_tj y[t * top + j], j ascending.
__global__ __launch_bounds__(256) void moe_combine_kernel(float* __restrict__ x, int64_t ldx, const float* __restrict__ y,
                                                          const float* __restrict__ pair_weights, float weight, int top,
                                                          int width) {
  const int64_t t = blockIdx.x;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < width; c += gridDim.y * blockDim.x) {
    float total = 0.f;
    for (int j = 0; j < top; ++j)
      total = fmaf(y[(t * top + j) * width + c], pair_weights != nullptr ? pair_weights[t * top + j] : weight, total);
    x[t * ldx + c] += total;
  }
}

// One wave a token.  A lane looks through its share of the experts (lane, lane + 64, ...) for the largest
// logit that is not chosen yet (a bit a share in the lane's own registers says which are); the wave's lanes
// meet over (logit, number), the larger logit and of two equal ones the lower number, and every lane ends
// with the same answer.  The sigmoid grows with its argument, so the largest scores are the largest logits.
constexpr int kRouterMostExperts = 64 * 128;

// score_kind 0: a score is sigmoid(z); 1: the softmax of z over all experts.  correction (float32 [experts] or
// null) is added to a score where the experts are chosen and nowhere else: the weights are the scores.
__global__ __launch_bounds__(256) void router_topk_kernel(const float* __restrict__ logits, int64_t ld, int n, int experts,
                                                          int top, int* __restrict__ chosen, float* __restrict__ weights,
                                                          int score_kind, const float* __restrict__ correction) {
  const int t = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (t >= n) return;
  const float* z = logits + (int64_t)t * ld;
  float zmax = 0.f, inv_sum = 1.f;
  if (score_kind == 1) {
    zmax = -INFINITY;
    for (int e = lane; e < experts; e += 64) zmax = fmaxf(zmax, z[e]);
    zmax = wave_max(zmax);
    float sum = 0.f;
    for (int e = lane; e < experts; e += 64) sum += expf(z[e] - zmax);
    inv_sum = 1.0f / wave_sum(sum);
  }
  auto score = [&](int e) { return score_kind == 1 ? expf(z[e] - zmax) * inv_sum : 1.0f / (1.0f + expf(-z[e])); };
  // without a correction the order of the scores is the order of the logits (both scores grow with them)
  auto choice = [&](int e) { return correction != nullptr ? score(e) + correction[e] : z[e]; };
  unsigned long long taken[2] = {0ull, 0ull};
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane, i = 0; e < experts; e += 64, ++i) {
      const float v = choice(e);
      if (!((taken[i >> 6] >> (i & 63)) & 1ull) && (at == 0x7fffffff || v > best)) { best = v; at = e; }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
      const float ob = __shfl_xor(best, off, 64);
      const int oa = __shfl_xor(at, off, 64);
      if (oa != 0x7fffffff && (at == 0x7fffffff || ob > best || (ob == best && oa < at))) { best = ob; at = oa; }
    }
    if ((at & 63) == lane) taken[(at >> 6) >> 6] |= 1ull << ((at >> 6) & 63);
    if (lane == 0) {
      chosen[(int64_t)t * top + j] = at;
      weights[(int64_t)t * top + j] = score(at);
    }
  }
}

}  // namespace

HFEE_API int hfee_router_topk(const float* logits, int64_t ld, int n, int experts, int top, int* chosen, float* weights,
                              int score_kind, const float* correction, hipStream_t stream) {
  HFEE_REQUIRE(score_kind == 0 || score_kind == 1, "router_topk: the scores are sigmoids (0) or a softmax (1)");
  HFEE_REQUIRE(n >= 0 && experts >= 1 && experts <= kRouterMostExperts && top >= 1 && top <= experts && ld >= experts,
               "router_topk: a token uses 1 to %d experts (of at most %d), not %d", experts, kRouterMostExperts, top);
  if (n == 0) return 0;
  router_topk_kernel<<<(n + 3) / 4, 256, 0, stream>>>(logits, ld, n, experts, top, chosen, weights, score_kind, correction);
  HFEE_CHECK_LAUNCH("router_topk");
  return 0;
}

// The whole feed-forward in its grouped form, bfloat16: x (float32 [n, width]) += the experts' weighted
// outputs.  order: int32 [n * top]; tiles: int32 [3 * hfee_moe_group_tiles(n, top, experts) + 1]; act:
// bfloat16 [n * top, ff]; y: float32 [n * top, width], needed where top > 1.
HFEE_API int hfee_moe_group_tiles(int n, int top, int experts) {
  return (int)(((int64_t)n * top + kTilePairs - 1) / kTilePairs) + experts;
}

HFEE_API int hfee_moe_grouped(float* x, int64_t ldx, const void* h, int64_t ldh, const void* w_gate, const void* w_up,
                              const void* w_down, const int* chosen, const int* table, const int* token_ids,
                              const float* pair_weights, float weight, int top, int experts, int ff, int width, int n,
                              int* order, int* tiles, void* act, float* y, const float* in_weights, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && top >= 1 && experts >= 1 && experts <= 8192 && ff >= 1 && width >= 1, "moe_grouped: bad sizes");
  HFEE_REQUIRE(chosen != nullptr || (table != nullptr && token_ids != nullptr), "moe_grouped: the experts of a token, or a table and the ids");
  HFEE_REQUIRE(width % 32 == 0 && ff % 32 == 0 && ldh % 8 == 0 && ldx >= width && ldh >= width,
               "moe_grouped: the width and the experts' size must be multiples of 32");
  HFEE_REQUIRE(w_gate != nullptr || pair_weights == nullptr, "moe_grouped: experts without a gate take their weights on the input");
  HFEE_REQUIRE(((uintptr_t)h | (uintptr_t)w_gate | (uintptr_t)w_up | (uintptr_t)w_down | (uintptr_t)act) % 16 == 0,
               "moe_grouped: operands must be 16-byte aligned");
  HFEE_REQUIRE(order != nullptr && tiles != nullptr && act != nullptr && (top == 1 || y != nullptr), "moe_grouped: scratch missing");
  HFEE_REQUIRE((int64_t)n * top < (1 << 30), "moe_grouped: too many pairs");
  if (n == 0) return 0;
  const int most = hfee_moe_group_tiles(n, top, experts);
  moe_group_kernel<<<1, 1024, 4 * experts * sizeof(int), stream>>>(order, tiles, most, chosen, table, token_ids, n, top, experts);
  HFEE_CHECK_LAUNCH("moe_group");
  // (rows in whole groups of four: ff and width are multiples of 32)
  if (w_gate != nullptr)
    moe_group_tiled_kernel<0><<<dim3(most, (ff + kTileRows / 2 - 1) / (kTileRows / 2)), 256, 0, stream>>>(
        act, ff, (const bf16_t*)h, ldh, (const bf16_t*)w_gate, (const bf16_t*)w_up, order, tiles, most, top, ff, width, 0,
        nullptr, 1.0f);
  else
    moe_group_tiled_kernel<1><<<dim3(most, (ff + kTileRows - 1) / kTileRows), 256, 0, stream>>>(
        act, ff, (const bf16_t*)h, ldh, (const bf16_t*)w_up, nullptr, order, tiles, most, top, ff, width, 0, in_weights, 1.0f);
  HFEE_CHECK_LAUNCH("moe_group_up");
  moe_group_tiled_kernel<2><<<dim3(most, (width + kTileRows - 1) / kTileRows), 256, 0, stream>>>(
      top == 1 ? (void*)x : (void*)y, top == 1 ? ldx : (int64_t)width, (const bf16_t*)act, ff, (const bf16_t*)w_down, nullptr,
      order, tiles, most, top, width, ff, top == 1 ? 1 : 0, pair_weights, weight);
  HFEE_CHECK_LAUNCH("moe_group_down");
  if (top > 1) {
    int parts = (width + 255) / 256;
    if (parts > 64) parts = 64;
    moe_combine_kernel<<<dim3(n, parts), 256, 0, stream>>>(x, ldx, y, pair_weights, weight, top, width);
    HFEE_CHECK_LAUNCH("moe_combine");
  }
  return 0;
}

HFEE_API int hfee_moe_up(void* act, const void* h, int64_t ldh, const void* w_gate, const void* w_up, int dtype,
                         const int* chosen, const int* table, const int* token_ids, int top, int experts, int ff,
                         int width, int n, const float* in_weights, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && top >= 1 && experts >= 1 && ff >= 1 && width >= 1 && ldh >= width, "moe_up: bad sizes");
  HFEE_REQUIRE(chosen != nullptr || (table != nullptr && token_ids != nullptr), "moe_up: the experts of a token, or a table and the ids");
  if (n == 0) return 0;
  const int per_block = 4 * kRowsPerWave;
  HFEE_REQUIRE((ff + per_block - 1) / per_block <= 65535, "moe_up: experts too wide");
  dim3 grid((unsigned)((int64_t)n * top), (ff + per_block - 1) / per_block);
  if (dtype == 0)
    moe_up_kernel<float><<<grid, 256, 0, stream>>>((float*)act, (const float*)h, ldh, (const float*)w_gate, (const float*)w_up,
                                                   chosen, table, token_ids, top, experts, ff, width, in_weights);
  else if (dtype == 1)
    moe_up_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)act, (const bf16_t*)h, ldh, (const bf16_t*)w_gate,
                                                    (const bf16_t*)w_up, chosen, table, token_ids, top, experts, ff, width, in_weights);
  else
    return fail("moe_up: unknown dtype %d", dtype);
  HFEE_CHECK_LAUNCH("moe_up");
  return 0;
}

HFEE_API int hfee_moe_down(float* x, int64_t ldx, const void* act, const void* w_down, int dtype, const int* chosen,
                           const int* table, const int* token_ids, const float* pair_weights, float weight, int top,
                           int experts, int ff, int width, int accumulate, int n, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && top >= 1 && experts >= 1 && ff >= 1 && width >= 1 && ldx >= width, "moe_down: bad sizes");
  HFEE_REQUIRE(chosen != nullptr || (table != nullptr && token_ids != nullptr), "moe_down: the experts of a token, or a table and the ids");
  if (n == 0) return 0;
  const int per_block = 4 * kRowsPerWave;
  HFEE_REQUIRE((width + per_block - 1) / per_block <= 65535, "moe_down: rows too wide");
  dim3 grid(n, (width + per_block - 1) / per_block);
  if (dtype == 0)
    moe_down_kernel<float><<<grid, 256, 0, stream>>>(x, ldx, (const float*)act, (const float*)w_down, chosen, table,
                                                     token_ids, pair_weights, weight, top, experts, ff, width, accumulate);
  else if (dtype == 1)
    moe_down_kernel<bf16_t><<<grid, 256, 0, stream>>>(x, ldx, (const bf16_t*)act, (const bf16_t*)w_down, chosen, table,
                                                      token_ids, pair_weights, weight, top, experts, ff, width, accumulate);
  else
    return fail("moe_down: unknown dtype %d", dtype);
  HFEE_CHECK_LAUNCH("moe_down");
  return 0;
}
