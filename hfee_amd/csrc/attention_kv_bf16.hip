// Matrix-core attention over the paged cache for keys of HFEE_DK and values of HFEE_DV dims
// (multiples of 16, compiled per pair), with an optional sink; bfloat16 operands, float32
// scores, weights and sums.  The cache layout is `KvLayout` (attention_kv.h).
//
// A wave owns 16 query rows and walks tiles of 32 keys: S^T = K Q^T (the keys are the row
// operand: a lane loads eight dims of one key, 16 bytes), then O^T += V^T P^T with the
// weights as they stand in the score registers (the k index of a matrix instruction is only a
// label shared by both operands: label 8g + e of lane group g means key 4g + e of the tile's
// first 16 keys for e < 4 and key 4g + e - 4 of its second 16 otherwise, so a lane's eight
// values of a value column are two loads of 8 bytes from the transposed values).
//
// Two meanings of the 16 rows (`mode`):
//   0  a portion of a prompt: up to four blocks of 16 consecutive tokens of one sequence (as many as
//      the registers hold for the sizes), one head a wave;
//   1  a single token: up to 16 query heads that share a key/value head; the keys may be
//      split over several waves, whose partial results a second kernel joins.
// The sink joins the denominator once, at the very end.
//
// A query may see less than every earlier key (`KeySight`, attention_kv.h): the last `window` positions only,
// and beside them one pooled key and value for every block of `pool` positions that lies wholly before the
// window (a cache layer of their own with block tables of its own, under the block's number); a score may be capped as
// cap * tanh(score / cap); a head's result may be multiplied by sigmoid of a gate.  The kernel then walks
// the tiles of the pooled layer that any of its rows sees, and after them the token tiles from the one
// that holds the first key of its first row's window; a key weighs where it lies within its row's bounds.
//
// Compiled with -DHFEE_KV_WEIGHTS=1 there is no softmax: a visible key weighs sigmoid(score + b_h), b_h a
// number a head (given where the softmax has its sinks), nothing is normalized over the keys, and the
// splits of a single token's keys are plain sums.
#include "attention_kv.h"

#ifndef HFEE_DK
#error "compile with -DHFEE_DK=<key size> -DHFEE_DV=<value size>"
#endif

using namespace hfee;

namespace {

#ifndef HFEE_KV_WEIGHTS
#define HFEE_KV_WEIGHTS 0
#endif
constexpr int DK = HFEE_DK, DV = HFEE_DV;
constexpr bool SIGMOID = HFEE_KV_WEIGHTS == 1;
static_assert(DK % 16 == 0 && DV % 16 == 0 && DK >= 16 && DV >= 16, "key and value sizes are multiples of 16");
constexpr int KSTEPS = (DK + 31) / 32;     // steps of 32 dims (the last may be half empty)
constexpr int VBLOCKS = DV / 16;
constexpr float kLog2e = 1.4426950408889634f;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

union Operand {
  bf16x8 v;
  u32x4 u;
  u32x2 h[2];
};

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  return (uint32_t)float_to_bf16(a) | ((uint32_t)float_to_bf16(b) << 16);
}

// The weights of one row block against a tile's 32 keys, in place in the score registers, and as the
// column operand of the value product.  The exponentials are taken against a reference that lags
// the running maximum: the sums are rescaled only when a maximum has moved by more than 2^8 (the
// quotient at the end does not depend on the reference), so most tiles cost no pass over the
// output sums and no exchange between lanes.  Keys beyond the row's own position weigh nothing; `masked` says whether the tile
// has any (the same answer in every lane).
// A score as the weights take it, in base 2: s * scale, capped where a cap is given
// (cap * tanh(x / cap), with tanh(y) = 1 - 2 / (e^(2y) + 1)).
struct ScoreScale {
  float scale_log2;      // scale * log2(e)
  float twice_over_cap;  // 2 * scale * log2(e) / cap, or 0 without a cap
  float cap_log2;        // cap * log2(e)
  __device__ __forceinline__ float operator()(float s) const {
    if (twice_over_cap == 0.f) return s * scale_log2;
    const float e = __builtin_amdgcn_exp2f(s * twice_over_cap);
    return cap_log2 * (1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f));
  }
};

// `lo`, `hi`: the first and the last entry of the section that the lane's row sees.
__device__ __forceinline__ void weigh_tile(f32x4 (&s)[2], float& reference, float& lsum, f32x4 (&acc)[VBLOCKS],
                                           Operand& pop, int j0, int g, int lo, int hi, ScoreScale scaled, bool masked) {
  if constexpr (SIGMOID) {      // `reference` is the head's number (in base 2), and stays
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = 1.0f / (1.0f + __builtin_amdgcn_exp2f(-(scaled(s[kb][i]) + reference)));
        const int j = j0 + kb * 16 + g * 4 + i;
        s[kb][i] = masked && (j > hi || j < lo) ? 0.f : p;
      }
    pop.u = u32x4{pack_bf16(s[0][0], s[0][1]), pack_bf16(s[0][2], s[0][3]), pack_bf16(s[1][0], s[1][1]),
                  pack_bf16(s[1][2], s[1][3])};
    return;
  }
  float tmax = -INFINITY;
#pragma unroll
  for (int kb = 0; kb < 2; ++kb)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float v = scaled(s[kb][i]);
      const int j = j0 + kb * 16 + g * 4 + i;
      if (masked && (j > hi || j < lo)) v = -INFINITY;
      s[kb][i] = v;
      tmax = fmaxf(tmax, v);
    }
  // (a lane looks at its own eight keys first: the four lanes of a query meet over the maximum only
  // when one of them is beyond the reference by 2^8, which after the first tiles is rare)
  if (__builtin_amdgcn_ballot_w64(tmax > reference + 8.0f) != 0) {      // (-inf + 8 = -inf: the first tile always)
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float moved = fmaxf(reference, tmax);
    const float use = moved == -INFINITY ? 0.f : moved;
    const float alpha = __builtin_amdgcn_exp2f(reference - use);
    reference = moved;
    lsum *= alpha;
#pragma unroll
    for (int vb = 0; vb < VBLOCKS; ++vb) acc[vb] = acc[vb] * alpha;
  }
  const float use = reference == -INFINITY ? 0.f : reference;
  float psum = 0.f;
#pragma unroll
  for (int kb = 0; kb < 2; ++kb)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float p = __builtin_amdgcn_exp2f(s[kb][i] - use);
      s[kb][i] = p;
      psum += p;
    }
  lsum += psum;
  pop.u = u32x4{pack_bf16(s[0][0], s[0][1]), pack_bf16(s[0][2], s[0][3]), pack_bf16(s[1][0], s[1][1]),
                pack_bf16(s[1][2], s[1][3])};
}

// partial results of a split: [item][head][split][4 + DV] float32: maximum (base 2), sum, two unused, O
constexpr int kPartial = 4 + DV;

// Row blocks of 16 that a wave of a prompt portion owns: the key and value operands of a tile
// are loaded once and multiplied with every row block, so the more blocks the registers hold
// (queries and output sums of a block: 4 (KSTEPS + VBLOCKS) registers a lane), the fewer bytes a
// product costs.
constexpr int kRegistersABlock = 4 * (KSTEPS + VBLOCKS);
#ifdef HFEE_KV_BLOCKS
constexpr int PORTION_BLOCKS = HFEE_KV_BLOCKS;
#else
constexpr int PORTION_BLOCKS = kRegistersABlock <= 64 ? 2 : 1;
#endif
// The keys of the next tile are asked for while the weights of this one are made (a second set of
// key operands: 8 KSTEPS registers a lane), where the registers allow it.
#ifdef HFEE_KV_PIPE
constexpr bool PIPE = HFEE_KV_PIPE;
#else
constexpr bool PIPE = 8 * KSTEPS + 4 * VBLOCKS <= 160;
#endif

template <int MODE, int RB>
__global__ __launch_bounds__(256) void attention_kv_kernel(
    bf16_t* __restrict__ out, int64_t ld_out, const bf16_t* __restrict__ q, int64_t ldq,
    const bf16_t* __restrict__ cache, KvLayout lay, const int* __restrict__ items, int num_items,
    const int* __restrict__ block_tables, int bt_stride, int num_heads, ScoreScale scaled,
    const float* __restrict__ sinks, float* __restrict__ partial, int splits, KeySight sight,
    const bf16_t* __restrict__ gate, int64_t ld_gate) {
  const int lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
  const int hpg = num_heads / lay.kv_heads;
  const int groups16 = (hpg + 15) / 16;
  const int units = MODE == 0 ? num_heads : lay.kv_heads * groups16;
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (wave >= (int64_t)num_items * splits * units) return;
  const int unit = (int)(wave % units);
  const int split = (int)((wave / units) % splits);
  const int item = (int)(wave / ((int64_t)units * splits));
  const int row0 = items[item * 4 + 0], rows = items[item * 4 + 1], pos0 = items[item * 4 + 2];
  const int* bt = block_tables + (int64_t)items[item * 4 + 3] * bt_stride;

  // row r of block b: a token of the portion (mode 0), or a head of the key/value head's group (mode 1)
  int token[RB], head[RB], pos[RB], kvh;
  bool valid[RB];
  if (MODE == 0) {
    kvh = unit / hpg;
#pragma unroll
    for (int b = 0; b < RB; ++b) {
      const int rr = min(16 * b + r, rows - 1);
      token[b] = row0 + rr; pos[b] = pos0 + rr; head[b] = unit; valid[b] = 16 * b + r < rows;
    }
  } else {
    kvh = unit / groups16;
    const int in_group = (unit % groups16) * 16 + r;
    valid[0] = in_group < hpg;
    token[0] = row0; pos[0] = pos0; head[0] = kvh * hpg + min(in_group, hpg - 1);
  }
  const int max_pos = MODE == 0 ? pos0 + rows - 1 : pos0;
  const int blocks = MODE == 0 ? (rows + 15) >> 4 : 1;       // row blocks that hold rows at all

  // the queries as the column operand: lane (r, g) holds dims 8g .. 8g+7 of every step of row r
  Operand qop[RB][KSTEPS];
#pragma unroll
  for (int b = 0; b < RB; ++b) {
    const bf16_t* qr = q + (int64_t)token[b] * ldq + (int64_t)head[b] * DK + g * 8;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      if (s * 32 + g * 8 < DK) qop[b][s].u = *reinterpret_cast<const u32x4*>(qr + s * 32);
      else qop[b][s].u = u32x4{0, 0, 0, 0};
    }
  }

  f32x4 acc[RB][VBLOCKS];
  float m[RB], lsum[RB];
#pragma unroll
  for (int b = 0; b < RB; ++b) {
    m[b] = SIGMOID ? (sinks != nullptr ? sinks[head[b]] * kLog2e : 0.f) : -INFINITY; lsum[b] = 0.f;
#pragma unroll
    for (int vb = 0; vb < VBLOCKS; ++vb) acc[b][vb] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // the tiles to walk: those of the pooled layer that any row sees, then the token tiles from the first
  // key of the first row's window on (without a window or pooled blocks: the token tiles from the first)
  const int pool_tiles = (sight.pooled_blocks(max_pos) + 31) >> 5;
  const int tile_lo = sight.first_key(pos0) >> 5;
  const int ntiles = pool_tiles + (max_pos >> 5) + 1 - tile_lo;
  const int per_split = (ntiles + splits - 1) / splits;
  const int tile_begin = split * per_split, tile_end = min(ntiles, tile_begin + per_split);
  const int last_block = max_pos >> lay.page_shift;
  const int slot_mask = lay.page_size - 1;
  const bf16_t* const pooled = static_cast<const bf16_t*>(sight.pooled);
  const int* const pbt = sight.pool_tables + (int64_t)items[item * 4 + 3] * sight.pool_bt_stride;
  const int last_pool_block = max(sight.pooled_blocks(max_pos) - 1, 0) >> lay.page_shift;

  // the key operands of a tile: lane (r, g) holds dims 8g .. 8g+7 of every step of key r of each of the
  // tile's two blocks of 16 keys; `values` gets where the lane's value columns of the two blocks begin
  auto load_keys = [&](int walked, Operand (&kop)[2][PIPE ? KSTEPS : 1], const bf16_t* (&values)[2]) {
    const bf16_t* section = walked < pool_tiles ? pooled : cache;
    const int tile = walked < pool_tiles ? walked : tile_lo + walked - pool_tiles;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      const int jb = (tile << 5) + kb * 16;
      const int page = walked < pool_tiles ? pbt[min(jb >> lay.page_shift, last_pool_block)] : bt[min(jb >> lay.page_shift, last_block)];
      const int slot0 = jb & slot_mask;
      const bf16_t* kr = section + lay.key_offset(page, kvh, slot0 + r, g * 8);
      values[kb] = section + lay.values_of(page, kvh) + slot0 + g * 4;
#pragma unroll
      for (int st = 0; st < (PIPE ? KSTEPS : 1); ++st) {
        if (st * 32 + g * 8 < DK) kop[kb][st].u = *reinterpret_cast<const u32x4*>(kr + st * 32);
        else kop[kb][st].u = u32x4{0, 0, 0, 0};
      }
    }
  };
  // (without the second set, a key operand lives from its load to its products only)
  auto load_keys_of_block = [&](int walked, int kb, int st, const bf16_t*& values) {
    const bf16_t* section = walked < pool_tiles ? pooled : cache;
    const int tile = walked < pool_tiles ? walked : tile_lo + walked - pool_tiles;
    const int jb = (tile << 5) + kb * 16;
    const int page = walked < pool_tiles ? pbt[min(jb >> lay.page_shift, last_pool_block)] : bt[min(jb >> lay.page_shift, last_block)];
    const int slot0 = jb & slot_mask;
    values = section + lay.values_of(page, kvh) + slot0 + g * 4;
    Operand one;
    if (st * 32 + g * 8 < DK) one.u = *reinterpret_cast<const u32x4*>(section + lay.key_offset(page, kvh, slot0 + r, g * 8) + st * 32);
    else one.u = u32x4{0, 0, 0, 0};
    return one;
  };
  Operand kop[2][PIPE ? KSTEPS : 1];
  const bf16_t* vnext[2];
  if constexpr (PIPE) {
    if (tile_begin < tile_end) load_keys(tile_begin, kop, vnext);
  }

  for (int tile = tile_begin; tile < tile_end; ++tile) {
    const bool in_pool = tile < pool_tiles;
    const int j0 = (in_pool ? tile : tile_lo + tile - pool_tiles) << 5;
    // which row blocks see any key of this tile (the same answer in every lane), and whether all their rows
    // see all of it: the entries that a row at position p sees are lo(p) .. hi(p), both growing with p
    bool live[RB], masked_tile[RB];
#pragma unroll
    for (int b = 0; b < RB; ++b) {
      const int p_first = MODE == 0 ? pos0 + min(rows - 1, 16 * b) : pos0;
      const int p_last = MODE == 0 ? pos0 + min(rows - 1, 16 * b + 15) : pos0;
      const int hi_first = in_pool ? sight.pooled_blocks(p_first) - 1 : p_first;
      const int hi_last = in_pool ? sight.pooled_blocks(p_last) - 1 : p_last;
      const int lo_first = in_pool ? 0 : sight.first_key(p_first), lo_last = in_pool ? 0 : sight.first_key(p_last);
      live[b] = (MODE == 1 || b < blocks) && j0 <= hi_last && j0 + 31 >= lo_first;
      masked_tile[b] = j0 + 31 > hi_first || j0 < lo_last;
    }
    f32x4 s[RB][2];
    const bf16_t* vbase[2];
    if constexpr (PIPE) {
      vbase[0] = vnext[0];
      vbase[1] = vnext[1];
    }
    Operand vop[PIPE ? VBLOCKS : 1];
    if constexpr (PIPE) {
#pragma unroll
      for (int vb = 0; vb < VBLOCKS; ++vb) {
        const int64_t column = (int64_t)(vb * 16 + r) * lay.page_size;
        vop[vb].h[0] = *reinterpret_cast<const u32x2*>(vbase[0] + column);
        vop[vb].h[1] = *reinterpret_cast<const u32x2*>(vbase[1] + column);
      }
    }
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
      for (int b = 0; b < RB; ++b) s[b][kb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int st = 0; st < KSTEPS; ++st) {
        Operand now;
        if constexpr (PIPE) now = kop[kb][st];
        else now = load_keys_of_block(tile, kb, st, vbase[kb]);
#pragma unroll
        for (int b = 0; b < RB; ++b)
          if (live[b]) s[b][kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(now.v, qop[b][st].v, s[b][kb], 0, 0, 0);
      }
    }
    if constexpr (PIPE) {
      if (tile + 1 < tile_end) load_keys(tile + 1, kop, vnext);
    }
    // scores of query r (this lane's column) against keys j0 + 16 kb + 4 g + i
    Operand pop[RB];
#pragma unroll
    for (int b = 0; b < RB; ++b) {
      if (!live[b]) continue;
      const int lo = in_pool ? 0 : sight.first_key(pos[b]);
      const int hi = in_pool ? sight.pooled_blocks(pos[b]) - 1 : pos[b];
      weigh_tile(s[b], m[b], lsum[b], acc[b], pop[b], j0, g, lo, hi, scaled, masked_tile[b]);
    }
#pragma unroll
    for (int vb = 0; vb < VBLOCKS; ++vb) {
      Operand values;
      if constexpr (PIPE) {
        values = vop[vb];
      } else {
        const int64_t column = (int64_t)(vb * 16 + r) * lay.page_size;
        values.h[0] = *reinterpret_cast<const u32x2*>(vbase[0] + column);
        values.h[1] = *reinterpret_cast<const u32x2*>(vbase[1] + column);
      }
#pragma unroll
      for (int b = 0; b < RB; ++b) {
        if (!live[b]) continue;
        acc[b][vb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(values.v, pop[b].v, acc[b][vb], 0, 0, 0);
      }
    }
  }

#pragma unroll
  for (int b = 0; b < RB; ++b) {
    if (b >= blocks) continue;
    float l = lsum[b];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (splits == 1) {
      float a = 1.f;
      if constexpr (SIGMOID) l = 1.f;
      if (!SIGMOID && sinks != nullptr) {
        const float sk = sinks[head[b]] * kLog2e;
        const float m_all = fmaxf(m[b], sk);
        a = exp2f(m[b] - m_all);
        l = l * a + exp2f(sk - m_all);
      }
      if (!valid[b]) continue;
      float inv = a / l;
      if (gate != nullptr)
        inv *= 1.0f / (1.0f + __expf(-bf16_to_float(gate[(int64_t)token[b] * ld_gate + head[b]])));
      bf16_t* orow = out + (int64_t)token[b] * ld_out + (int64_t)head[b] * DV + g * 4;
#pragma unroll
      for (int vb = 0; vb < VBLOCKS; ++vb) {
        const u32x2 w = {pack_bf16(acc[b][vb][0] * inv, acc[b][vb][1] * inv),
                         pack_bf16(acc[b][vb][2] * inv, acc[b][vb][3] * inv)};
        *reinterpret_cast<u32x2*>(orow + vb * 16) = w;
      }
    } else {
      if (!valid[b]) continue;
      float* pr = partial + (((int64_t)item * num_heads + head[b]) * splits + split) * kPartial;
      if (g == 0) {
        pr[0] = m[b];
        pr[1] = l;
      }
#pragma unroll
      for (int vb = 0; vb < VBLOCKS; ++vb)
        *reinterpret_cast<f32x4*>(pr + 4 + vb * 16 + g * 4) = acc[b][vb];
    }
  }
}

// Prompt portions where four query heads (or a multiple) share a key/value head: the four waves of
// a workgroup are four heads of one group over the same rows, and every key tile comes from
// memory once for all of them, into LDS (two stages: the next tile is on its way while this one is
// multiplied; rows of keys padded by 16 bytes and value columns to 80 so that the operand reads of
// a wave fall into different banks).  Long row tiles run first.
constexpr int kKeyRow = DK + 8;            // elements of a key row in LDS
constexpr int kValueColumn = 40;           // elements of a value column in LDS (32 keys + padding)
constexpr int kStage = 32 * kKeyRow + DV * kValueColumn;
constexpr int kKeyChunks = 32 * (DK / 8), kValueChunks = DV * 4;        // 16-byte chunks of a tile
constexpr int kKeyLoads = (kKeyChunks + 255) / 256, kValueLoads = (kValueChunks + 255) / 256;
// (two stages have to fit the 160 KB of a CU; sizes beyond that take the kernel without LDS)
constexpr bool kSharedFits = 2 * (size_t)kStage * sizeof(bf16_t) <= 160 * 1024;
#ifdef HFEE_KV_SHARED_BLOCKS
constexpr int SHARED_BLOCKS = HFEE_KV_SHARED_BLOCKS;
#else
constexpr int SHARED_BLOCKS = 1;     // (two blocks a wave measured slower: fewer waves to hide the waits)
#endif

template <int RB>
__global__ __launch_bounds__(256) void attention_kv_shared_kernel(
    bf16_t* __restrict__ out, int64_t ld_out, const bf16_t* __restrict__ q, int64_t ldq,
    const bf16_t* __restrict__ cache, KvLayout lay, const int* __restrict__ items, int num_items,
    const int* __restrict__ block_tables, int bt_stride, int num_heads, ScoreScale scaled,
    const float* __restrict__ sinks, KeySight sight, const bf16_t* __restrict__ gate, int64_t ld_gate) {
  extern __shared__ __attribute__((aligned(16))) bf16_t stages[];
  const int lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4, w = threadIdx.x >> 6;
  const int hpg = num_heads / lay.kv_heads;
  const int quads = num_heads / 4;
  const int item = num_items - 1 - (int)(blockIdx.x / quads);
  const int head = (int)(blockIdx.x % quads) * 4 + w;
  const int kvh = head / hpg;
  const int row0 = items[item * 4 + 0], rows = items[item * 4 + 1], pos0 = items[item * 4 + 2];
  const int* bt = block_tables + (int64_t)items[item * 4 + 3] * bt_stride;
  const int blocks = (rows + 15) >> 4;

  int token[RB], pos[RB];
  bool valid[RB];
#pragma unroll
  for (int b = 0; b < RB; ++b) {
    const int rr = min(16 * b + r, rows - 1);
    token[b] = row0 + rr; pos[b] = pos0 + rr; valid[b] = 16 * b + r < rows;
  }
  Operand qop[RB][KSTEPS];
#pragma unroll
  for (int b = 0; b < RB; ++b) {
    const bf16_t* qr = q + (int64_t)token[b] * ldq + (int64_t)head * DK + g * 8;
#pragma unroll
    for (int st = 0; st < KSTEPS; ++st) {
      if (st * 32 + g * 8 < DK) qop[b][st].u = *reinterpret_cast<const u32x4*>(qr + st * 32);
      else qop[b][st].u = u32x4{0, 0, 0, 0};
    }
  }
  f32x4 acc[RB][VBLOCKS];
  float m[RB], lsum[RB];
#pragma unroll
  for (int b = 0; b < RB; ++b) {
    m[b] = SIGMOID ? (sinks != nullptr ? sinks[head] * kLog2e : 0.f) : -INFINITY; lsum[b] = 0.f;
#pragma unroll
    for (int vb = 0; vb < VBLOCKS; ++vb) acc[b][vb] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const int max_pos = pos0 + rows - 1;
  // the tiles to walk: those of the pooled layer that any row sees, then the token tiles from the first key
  // of the first row's window on
  const int pool_tiles = (sight.pooled_blocks(max_pos) + 31) >> 5;
  const int tile_lo = sight.first_key(pos0) >> 5;
  const int ntiles = pool_tiles + (max_pos >> 5) + 1 - tile_lo;
  const int last_block = max_pos >> lay.page_shift;
  const int slot_mask = lay.page_size - 1;
  const bf16_t* const pooled = static_cast<const bf16_t*>(sight.pooled);
  const int* const pbt = sight.pool_tables + (int64_t)items[item * 4 + 3] * sight.pool_bt_stride;
  const int last_pool_block = max(sight.pooled_blocks(max_pos) - 1, 0) >> lay.page_shift;

  // two sets of registers for the chunks on their way, where that is few registers: a tile is then
  // asked for two tiles before it is multiplied (memory takes longer than one tile's products)
  constexpr bool DEEP = 4 * (kKeyLoads + kValueLoads) <= 32;
  u32x4 kst_a[kKeyLoads], vst_a[kValueLoads], kst_b[DEEP ? kKeyLoads : 1], vst_b[DEEP ? kValueLoads : 1];
  auto fetch = [&](int walked, u32x4* kst, u32x4* vst) {          // this thread's chunks of the tile, into registers
    const bf16_t* section = walked < pool_tiles ? pooled : cache;
    const int tile = walked < pool_tiles ? walked : tile_lo + walked - pool_tiles;
    const bf16_t* keys[2];
    const bf16_t* values[2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      const int jb = (tile << 5) + kb * 16;
      const int page = walked < pool_tiles ? pbt[min(jb >> lay.page_shift, last_pool_block)] : bt[min(jb >> lay.page_shift, last_block)];
      keys[kb] = section + lay.key_offset(page, kvh, jb & slot_mask, 0);
      values[kb] = section + lay.values_of(page, kvh) + (jb & slot_mask);
    }
#pragma unroll
    for (int i = 0; i < kKeyLoads; ++i) {
      const int c = i * 256 + threadIdx.x;
      if (c < kKeyChunks) {
        const int row = c / (DK / 8), col = c % (DK / 8);
        kst[i] = *reinterpret_cast<const u32x4*>(keys[row >> 4] + (row & 15) * DK + col * 8);
      }
    }
#pragma unroll
    for (int i = 0; i < kValueLoads; ++i) {
      const int c = i * 256 + threadIdx.x;
      if (c < kValueChunks) {
        const int col = c >> 2, part = c & 3;
        vst[i] = *reinterpret_cast<const u32x4*>(values[part >> 1] + (int64_t)col * lay.page_size + (part & 1) * 8);
      }
    }
  };
  auto commit = [&](int buffer, const u32x4* kst, const u32x4* vst) {       // the registers into a stage
    bf16_t* st = stages + buffer * kStage;
#pragma unroll
    for (int i = 0; i < kKeyLoads; ++i) {
      const int c = i * 256 + threadIdx.x;
      if (c < kKeyChunks) *reinterpret_cast<u32x4*>(st + (c / (DK / 8)) * kKeyRow + (c % (DK / 8)) * 8) = kst[i];
    }
#pragma unroll
    for (int i = 0; i < kValueLoads; ++i) {
      const int c = i * 256 + threadIdx.x;
      if (c < kValueChunks) *reinterpret_cast<u32x4*>(st + 32 * kKeyRow + (c >> 2) * kValueColumn + (c & 3) * 8) = vst[i];
    }
  };
  auto multiply = [&](int walked, const bf16_t* st) {
    const bool in_pool = walked < pool_tiles;
    const int j0 = (in_pool ? walked : tile_lo + walked - pool_tiles) << 5;
    // (the entries that a row at position p sees are lo(p) .. hi(p), both growing with p)
    bool live[RB], masked_tile[RB];
#pragma unroll
    for (int b = 0; b < RB; ++b) {
      const int p_first = pos0 + min(rows - 1, 16 * b), p_last = pos0 + min(rows - 1, 16 * b + 15);
      const int hi_first = in_pool ? sight.pooled_blocks(p_first) - 1 : p_first;
      const int hi_last = in_pool ? sight.pooled_blocks(p_last) - 1 : p_last;
      const int lo_first = in_pool ? 0 : sight.first_key(p_first), lo_last = in_pool ? 0 : sight.first_key(p_last);
      live[b] = b < blocks && j0 <= hi_last && j0 + 31 >= lo_first;
      masked_tile[b] = j0 + 31 > hi_first || j0 < lo_last;
    }
    f32x4 s[RB][2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
      for (int b = 0; b < RB; ++b) s[b][kb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        Operand kop;
        if (ks * 32 + g * 8 < DK) kop.u = *reinterpret_cast<const u32x4*>(st + (kb * 16 + r) * kKeyRow + ks * 32 + g * 8);
        else kop.u = u32x4{0, 0, 0, 0};
#pragma unroll
        for (int b = 0; b < RB; ++b)
          if (live[b]) s[b][kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop.v, qop[b][ks].v, s[b][kb], 0, 0, 0);
      }
    }
    Operand pop[RB];
#pragma unroll
    for (int b = 0; b < RB; ++b) {
      if (!live[b]) continue;
      const int lo = in_pool ? 0 : sight.first_key(pos[b]);
      const int hi = in_pool ? sight.pooled_blocks(pos[b]) - 1 : pos[b];
      weigh_tile(s[b], m[b], lsum[b], acc[b], pop[b], j0, g, lo, hi, scaled, masked_tile[b]);
    }
#pragma unroll
    for (int vb = 0; vb < VBLOCKS; ++vb) {
      Operand vop;
      const bf16_t* column = st + 32 * kKeyRow + (vb * 16 + r) * kValueColumn + g * 4;
      vop.h[0] = *reinterpret_cast<const u32x2*>(column);
      vop.h[1] = *reinterpret_cast<const u32x2*>(column + 16);
#pragma unroll
      for (int b = 0; b < RB; ++b) {
        if (!live[b]) continue;
        acc[b][vb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vop.v, pop[b].v, acc[b][vb], 0, 0, 0);
      }
    }
  };
  fetch(0, kst_a, vst_a);
  if (DEEP && ntiles > 1) fetch(1, kst_b, vst_b);
  commit(0, kst_a, vst_a);
  __syncthreads();
  if constexpr (DEEP) {
    for (int tile = 0; tile < ntiles; tile += 2) {
      if (tile + 2 < ntiles) fetch(tile + 2, kst_a, vst_a);
      multiply(tile, stages + (tile & 1) * kStage);
      if (tile + 1 < ntiles) commit((tile + 1) & 1, kst_b, vst_b);
      __syncthreads();
      if (tile + 1 >= ntiles) break;
      if (tile + 3 < ntiles) fetch(tile + 3, kst_b, vst_b);
      multiply(tile + 1, stages + ((tile + 1) & 1) * kStage);
      if (tile + 2 < ntiles) commit((tile + 2) & 1, kst_a, vst_a);
      __syncthreads();
    }
  } else {
    for (int tile = 0; tile < ntiles; ++tile) {
      if (tile + 1 < ntiles) fetch(tile + 1, kst_a, vst_a);
      multiply(tile, stages + (tile & 1) * kStage);
      if (tile + 1 < ntiles) commit((tile + 1) & 1, kst_a, vst_a);
      __syncthreads();
    }
  }

#pragma unroll
  for (int b = 0; b < RB; ++b) {
    if (b >= blocks) continue;
    float l = lsum[b];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    float a = 1.f;
    if constexpr (SIGMOID) l = 1.f;
    if (!SIGMOID && sinks != nullptr) {
      const float sk = sinks[head] * kLog2e;
      const float m_all = fmaxf(m[b], sk);
      a = exp2f(m[b] - m_all);
      l = l * a + exp2f(sk - m_all);
    }
    if (!valid[b]) continue;
    float inv = a / l;
    if (gate != nullptr) inv *= 1.0f / (1.0f + __expf(-bf16_to_float(gate[(int64_t)token[b] * ld_gate + head])));
    bf16_t* orow = out + (int64_t)token[b] * ld_out + (int64_t)head * DV + g * 4;
#pragma unroll
    for (int vb = 0; vb < VBLOCKS; ++vb) {
      const u32x2 wv = {pack_bf16(acc[b][vb][0] * inv, acc[b][vb][1] * inv),
                        pack_bf16(acc[b][vb][2] * inv, acc[b][vb][3] * inv)};
      *reinterpret_cast<u32x2*>(orow + vb * 16) = wv;
    }
  }
}

// joins the splits of a single token's heads: one wave per (item, head, 64 value dims).  Lane sp holds split
// sp's maximum and sum (at most 64 splits), the weights of the splits come from one reduction over the
// wave, and the wave's value dims are then summed over the splits in their order, lanes over the dims.
__global__ __launch_bounds__(64) void attention_kv_join_kernel(
    bf16_t* __restrict__ out, int64_t ld_out, const int* __restrict__ items, const float* __restrict__ partial,
    int splits, int num_heads, const float* __restrict__ sinks, const bf16_t* __restrict__ gate, int64_t ld_gate) {
  const int item = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const float* pr = partial + ((int64_t)item * num_heads + head) * splits * kPartial;
  const int token = items[item * 4];
  const float sk = !SIGMOID && sinks != nullptr ? sinks[head] * kLog2e : -INFINITY;
  const float my_m = lane < splits ? pr[lane * kPartial] : -INFINITY;
  const float my_l = lane < splits ? pr[lane * kPartial + 1] : 0.f;
  const float m = fmaxf(wave_max(my_m), sk);
  // (0 for a split without keys and for lanes beyond the splits; without a softmax every split counts as it is)
  const float my_w = SIGMOID ? (lane < splits ? 1.f : 0.f) : exp2f(my_m - m);
  const float lsum = wave_sum(my_l * my_w) + (!SIGMOID && sinks != nullptr ? exp2f(sk - m) : 0.f);
  float inv = SIGMOID ? 1.0f : 1.0f / lsum;
  if (gate != nullptr) inv *= 1.0f / (1.0f + __expf(-bf16_to_float(gate[(int64_t)token * ld_gate + head])));
  const int d = blockIdx.z * 64 + lane;
  float o = 0.f;
#pragma unroll 8
  for (int sp = 0; sp < splits; ++sp) o = fmaf(d < DV ? pr[sp * kPartial + 4 + d] : 0.f, __shfl(my_w, sp, 64), o);
  if (d < DV) out[(int64_t)token * ld_out + (int64_t)head * DV + d] = float_to_bf16(o * inv);
}

}  // namespace

HFEE_DEFINE_LAST_ERROR

HFEE_API int hfee_attention_kv_bf16_dk() { return DK; }
HFEE_API int hfee_attention_kv_bf16_dv() { return DV; }
HFEE_API int hfee_attention_kv_bf16_weights() { return HFEE_KV_WEIGHTS; }
// the most rows of an item of mode 0, for this many query heads a key/value head (where they are a
// multiple of four, the kernel that shares the key tiles through LDS runs)
HFEE_API int hfee_attention_kv_bf16_rows(int heads_per_kv_head) {
  return 16 * (kSharedFits && heads_per_kv_head % 4 == 0 ? SHARED_BLOCKS : PORTION_BLOCKS);
}

// float32 words of `partial` that `splits` > 1 need for `num_items` single tokens
HFEE_API int64_t hfee_attention_kv_bf16_partial(int num_items, int num_heads, int splits) {
  return splits > 1 ? (int64_t)num_items * num_heads * splits * kPartial : 0;
}

// items: [num_items][4] int32 on the device: first row, rows (1..hfee_attention_kv_bf16_rows() in
// mode 0; 1 in mode 1), first position, block-table row.
HFEE_API int hfee_attention_kv_bf16(void* out, int64_t ld_out, const void* q, int64_t ldq, const void* cache,
                                    const int* items, int num_items, int mode, const int* block_tables,
                                    int bt_stride, int num_heads, int kv_heads, int page_size, float scale,
                                    const float* sinks, float* partial, int64_t partial_words, int splits,
                                    int window, int pool, float softcap, const void* pooled, const int* pool_tables,
                                    int pool_bt_stride, const void* gate,
                                    int64_t ld_gate, hipStream_t stream) {
  HFEE_REQUIRE(num_items >= 0, "attention_kv_bf16: bad item count");
  KeySight sight;
  if (make_key_sight(&sight, window, pool, softcap, pooled, pool_tables, pool_bt_stride)) return 1;
  HFEE_REQUIRE(pooled == nullptr || (uintptr_t)pooled % 16 == 0, "attention_kv_bf16: the pooled layer must be aligned for vector access");
  HFEE_REQUIRE(gate == nullptr || ld_gate >= num_heads, "attention_kv_bf16: the gates' rows are too short");
  if (num_items == 0) return 0;
  HFEE_REQUIRE(mode == 0 || mode == 1, "attention_kv_bf16: mode is 0 (portions) or 1 (single tokens)");
  HFEE_REQUIRE(num_heads > 0 && kv_heads > 0 && num_heads % kv_heads == 0,
               "attention_kv_bf16: %d heads are not a multiple of %d kv heads", num_heads, kv_heads);
  HFEE_REQUIRE(num_heads <= 65535, "attention_kv_bf16: too many heads");
  HFEE_REQUIRE(ldq >= (int64_t)num_heads * DK && ld_out >= (int64_t)num_heads * DV, "attention_kv_bf16: q/out row too short");
  HFEE_REQUIRE(ldq % 8 == 0 && ld_out % 4 == 0 && (uintptr_t)q % 16 == 0 && (uintptr_t)out % 8 == 0 &&
               (uintptr_t)cache % 16 == 0, "attention_kv_bf16: q, out and the cache must be aligned for vector access");
  HFEE_REQUIRE(splits >= 1 && splits <= 64 && (splits == 1 || mode == 1), "attention_kv_bf16: only single tokens split their keys, into at most 64");
  HFEE_REQUIRE(splits == 1 || (partial != nullptr &&
               partial_words >= hfee_attention_kv_bf16_partial(num_items, num_heads, splits)),
               "attention_kv_bf16: the partial results need more room");
  KvLayout lay;
  if (make_kv_layout(&lay, kv_heads, DK, DV, page_size)) return 1;
  const int hpg = num_heads / kv_heads;
  const int64_t units = mode == 0 ? num_heads : (int64_t)kv_heads * ((hpg + 15) / 16);
  const int64_t waves = (int64_t)num_items * splits * units;
  const int64_t blocks = (waves + 3) / 4;
  HFEE_REQUIRE(blocks <= 0x7fffffff, "attention_kv_bf16: too much work for one launch");
  ScoreScale scaled;
  scaled.scale_log2 = scale * kLog2e;
  scaled.twice_over_cap = softcap > 0.f ? 2.0f * scale * kLog2e / softcap : 0.f;
  scaled.cap_log2 = softcap * kLog2e;
  if (mode == 0 && kSharedFits && hpg % 4 == 0) {
    const size_t lds = 2 * (size_t)kStage * sizeof(bf16_t);
    static bool allowed = false;       // (more than 64 KB of LDS has to be asked for once)
    if (!allowed) {
      if (hipFuncSetAttribute((const void*)attention_kv_shared_kernel<SHARED_BLOCKS>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
        return fail("attention_kv_bf16: %zu bytes of LDS are not to be had", lds);
      allowed = true;
    }
    const int64_t groups = (int64_t)num_items * (num_heads / 4);
    HFEE_REQUIRE(groups <= 0x7fffffff, "attention_kv_bf16: too much work for one launch");
    attention_kv_shared_kernel<SHARED_BLOCKS><<<(unsigned)groups, 256, lds, stream>>>((bf16_t*)out, ld_out,
        (const bf16_t*)q, ldq, (const bf16_t*)cache, lay, items, num_items, block_tables, bt_stride, num_heads,
        scaled, sinks, sight, (const bf16_t*)gate, ld_gate);
  } else if (mode == 0)
    attention_kv_kernel<0, PORTION_BLOCKS><<<(unsigned)blocks, 256, 0, stream>>>((bf16_t*)out, ld_out, (const bf16_t*)q, ldq,
        (const bf16_t*)cache, lay, items, num_items, block_tables, bt_stride, num_heads, scaled, sinks, partial, 1, sight,
        (const bf16_t*)gate, ld_gate);
  else
    attention_kv_kernel<1, 1><<<(unsigned)blocks, 256, 0, stream>>>((bf16_t*)out, ld_out, (const bf16_t*)q, ldq,
        (const bf16_t*)cache, lay, items, num_items, block_tables, bt_stride, num_heads, scaled, sinks, partial, splits,
        sight, (const bf16_t*)gate, ld_gate);
  HFEE_CHECK_LAUNCH("attention_kv_bf16");
  if (splits > 1) {
    attention_kv_join_kernel<<<dim3(num_items, num_heads, (DV + 63) / 64), 64, 0, stream>>>((bf16_t*)out, ld_out, items, partial,
                                                                            splits, num_heads, sinks,
                                                                            (const bf16_t*)gate, ld_gate);
    HFEE_CHECK_LAUNCH("attention_kv_bf16 join");
  }
  return 0;
}
