// bfloat16 paged attention on the matrix cores for one head size (MLR_HEAD_DIM,
// a multiple of 16 up to 256); one shared library per head size.
//
// Both kernels compute scores transposed, S^T[key, row] = K[key, :] . Q[row, :],
// so that the accumulator layout of the first product (a lane holds 4 consecutive
// keys of one row) is exactly the operand layout of the second product
// O^T[dim, row] = V^T[dim, key] . P^T[key, row]: probabilities go from one MFMA
// to the next in registers.  Keys are read from pages [page, kv_head, offset, dim]
// (dim fastest: operand of the first product), values from pages
// [page, kv_head, dim, offset] (key position fastest: operand of the second).
// Softmax is the online form with float32 max, sum and accumulator
// (csrc/paged_attention_cuda.cu:87-105 of the reference); a lane's column is one
// row (a query head, or a query token), so max and sum are per lane.
//
//  * attn_decode: entries with ONE new token.  A workgroup takes one (entry,
//    KV head, partition of the keys); the g query heads that share the KV head
//    are the 16 columns of the MFMA tile, so keys and values are read once per
//    KV head (the reference's kernel reads them once per query head,
//    csrc/paged_attention_cuda.cu:44-46).  Four wavefronts take 32-key tiles in
//    turn, all of a wavefront's loads in flight before it computes, one softmax
//    update per tile, and merge through LDS; partitions merge in attn_decode_merge with the
//    reference's rule m = max m_j, O = sum w_j a_j / sum w_j l_j, w_j = exp(m_j - m)
//    (csrc/paged_attention_split_cuda.cu:66-88).
//  * attn_prefill: entries with several new tokens (prompt portions), in tiles of
//    64 queries of one head; key and value tiles of 64 positions are staged in LDS
//    and shared by the four wavefronts (16 queries each).  A query at position p
//    sees keys first..p of its request, read from the pages after the step's own
//    keys were written, so a portion behind a cached prefix needs nothing special.
#define MLR_ERROR_CHANNEL
#include "common.h"
#include "mfma.h"

#ifndef MLR_HEAD_DIM
#error "compile with -DMLR_HEAD_DIM=<multiple of 16>"
#endif

namespace mlr {

constexpr int D = MLR_HEAD_DIM;
static_assert(D % 16 == 0 && D >= 16 && D <= 256, "head size must be a multiple of 16 within 16..256");
// The score product runs over the head dims in 16x16x32 steps.  When D is an odd
// multiple of 16 the last step covers 16 dims only: lanes of quarters 2 and 3 (k 16..31
// of that step) feed zeros on both sides.
constexpr int kSteps = (D + 31) / 32;
constexpr bool kHalfLast = (D % 32) != 0;
constexpr int kDimTiles = D / 16;

// One row of D dims (a query, or a key) as the operand chunks of the score product.
struct RowOperand {
  bf16x8_t step[kSteps];
};

// `row` points at dim 0 of this lane's row, in global memory or LDS.
__device__ __forceinline__ RowOperand load_row(const bf16* row, bool valid, int quarter) {
  RowOperand r;
#pragma unroll
  for (int s = 0; s < kSteps; ++s) {
    const bool inside = valid && !(kHalfLast && s == kSteps - 1 && quarter >= 2);
    r.step[s] = inside ? load_bf16x8(row + s * 32 + quarter * 8) : zero_bf16x8();
  }
  return r;
}

// The same for rows that a step reads once (cached keys at decode): the non-temporal hint lets
// them pass the caches by.
__device__ __forceinline__ RowOperand load_row_once(const bf16* row, int quarter) {
  RowOperand r;
#pragma unroll
  for (int s = 0; s < kSteps; ++s) {
    const bool inside = !(kHalfLast && s == kSteps - 1 && quarter >= 2);
    r.step[s] = inside ? __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(row + s * 32 + quarter * 8))
                       : zero_bf16x8();
  }
  return r;
}

// S^T tile [16 keys x 16 rows].
__device__ __forceinline__ f32x4_t score_tile(const RowOperand& k, const RowOperand& q) {
  f32x4_t s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int st = 0; st < kSteps; ++st) s = mfma_16x16x32(k.step[st], q.step[st], s);
  return s;
}

// Running softmax state of one column (row of the attention problem) in a lane, in base 2:
// m is the running maximum of score * scale * log2(e).
struct Softmax {
  float m;
  float l;  // this lane's share of the sum (its own keys of every tile)
};

// ---- decode ---------------------------------------------------------------------------------
constexpr int kDecodeWaves = D > 128 ? 2 : 4;  // bounded by the LDS the merge needs
constexpr int kPartialStride = D + 2;  // numerator[D], max, denominator
constexpr int kMaxDecodeDepth = D > 128 ? 1 : (D > 64 ? 2 : 4);  // 32-key tiles of a wavefront in flight at once (registers)

typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4v_t __attribute__((ext_vector_type(4)));

// Operands of one 32-key tile (two 16-key halves), loaded ahead of their use.
struct DecodeTile {
  RowOperand k[2];
  u32x2_t v[kDimTiles][2];  // per 16 dims: this lane's 4 keys of each half
  bool bad;
};

// Where one 32-key tile's operands lie: the page of this lane's key row and of its 4 value
// keys, per half.  Looked up for ALL of a wavefront's tiles before any operand is loaded, and
// without branches: the wait for a later tile's table entry would otherwise also wait for
// every operand load issued before it, one trip to memory after the other.
struct DecodeTilePages {
  int key_page[2], value_page[2];
};

__device__ __forceinline__ DecodeTilePages find_decode_tile(const int* __restrict__ table, int ts, int ke,
                                                            int block_size, int col, int quarter) {
  DecodeTilePages p;
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    // positions past the end look at the last position's entry instead: always inside the table
    p.key_page[half] = table[min(ts + half * 16 + col, ke - 1) / block_size];
    p.value_page[half] = table[min(ts + half * 16 + quarter * 4, ke - 1) / block_size];
  }
  return p;
}

// Loads are unconditional (what is absent reads page 0 instead): a key outside first..ke-1 is
// masked by its position and its values are cleared there; a missing page inside that range
// poisons the output.
__device__ __forceinline__ DecodeTile load_decode_tile(const bf16* __restrict__ key_pages,
                                                       const bf16* __restrict__ value_pages,
                                                       const DecodeTilePages& pages, int ts, int ke, int first,
                                                       int kvh, int kv_heads, int block_size, int num_pages,
                                                       int col, int quarter) {
  DecodeTile t;
  t.bad = false;
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    // key operand: this lane's row is key ts + half * 16 + col
    const int key_a = ts + half * 16 + col;
    const bool here_a = static_cast<unsigned>(pages.key_page[half]) < static_cast<unsigned>(num_pages);
    t.bad = t.bad || (!here_a && key_a >= first && key_a < ke);
    const int page_a = here_a ? pages.key_page[half] : 0;
    const int off_a = min(key_a, ke - 1) % block_size;
    t.k[half] = load_row_once(key_pages + ((static_cast<int64_t>(page_a) * kv_heads + kvh) * block_size + off_a) * D,
                              quarter);
    // value operand: this lane's 4 keys are ts + half * 16 + quarter * 4 .. + 3, inside one page
    const int key_v = ts + half * 16 + quarter * 4;
    const bool here_v = static_cast<unsigned>(pages.value_page[half]) < static_cast<unsigned>(num_pages);
    const int page_v = here_v ? pages.value_page[half] : 0;
    const int off_v = key_v < ke ? key_v % block_size : 0;
    const bf16* vbase = value_pages + (static_cast<int64_t>(page_v) * kv_heads + kvh) * D * block_size + off_v;
#pragma unroll
    for (int dt = 0; dt < kDimTiles; ++dt)
      t.v[dt][half] = __builtin_nontemporal_load(
          reinterpret_cast<const u32x2_t*>(vbase + static_cast<int64_t>(dt * 16 + col) * block_size));
  }
  return t;
}

template <int kDecodeDepth>
__global__ __launch_bounds__(kDecodeWaves* kWave) void attn_decode_kernel(
    const bf16* __restrict__ q, int64_t q_stride, const bf16* __restrict__ key_pages,
    const bf16* __restrict__ value_pages, const int* __restrict__ block_table, int table_width,
    const int* __restrict__ cu_q, const int* __restrict__ context_lens, bf16* __restrict__ out,
    float* __restrict__ partial, int heads, int kv_heads, int head_tiles, int block_size, int num_pages,
    float scale, int window, int part, int splits) {
  __shared__ float sm_acc[kDecodeWaves][16][D];
  __shared__ float sm_m[kDecodeWaves][16];
  __shared__ float sm_l[kDecodeWaves][16];
  __shared__ int sm_bad;

  const int entry = blockIdx.x;
  const int kvh = blockIdx.y / head_tiles;
  const int htile = blockIdx.y % head_tiles;
  const int split = blockIdx.z;
  const int t = cu_q[entry];
  if (cu_q[entry + 1] - t != 1) return;  // not a single-token entry: the prefill kernel owns it

  const int tid = threadIdx.x;
  const int lane = tid % kWave;
  const int wave = tid / kWave;
  const int col = lane % 16;      // query head within the tile
  const int quarter = lane / 16;  // which 4 keys of a tile / which chunk of the dims
  const int group = heads / kv_heads;
  const int head_in_group = htile * 16 + col;
  const bool head_ok = head_in_group < group;
  const int head = kvh * group + head_in_group;

  const int ctx = context_lens[entry];
  const int p = ctx - 1;
  const int first = window > 0 ? max(0, p - window + 1) : 0;
  const int base = (first / 16) * 16;
  const int kb = base + split * part;
  const int ke = min(kb + part, ctx);
  if (kb >= ke) return;  // a partition past this entry's keys: the merge does not look at it
  const int* table = block_table + static_cast<int64_t>(entry) * table_width;
  if (tid == 0) sm_bad = 0;
  __syncthreads();

  const RowOperand qo =
      load_row(q + t * q_stride + static_cast<int64_t>(head_ok ? head : 0) * D, head_ok, quarter);

  Softmax sm{-INFINITY, 0.f};
  f32x4_t acc[kDimTiles];
#pragma unroll
  for (int dt = 0; dt < kDimTiles; ++dt) acc[dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  bool bad = false;

  // The wavefronts take the partition's 32-key tiles in turn.  A tile's work is far shorter
  // than a trip to memory, so a wavefront first issues the loads of up to kDecodeDepth of
  // its tiles (the host picks the depth so that this is all of them whenever registers allow;
  // tiles past the end would be loaded all the same) and only then starts on the first.
  // Per tile: scores of both halves, ONE softmax update, one 32-key value product per 16 dims.
  constexpr int kStride = kDecodeWaves * 32;
  const float scale2 = scale * 1.44269504088896340736f;
  for (int ts0 = kb + wave * 32; ts0 < ke; ts0 += kDecodeDepth * kStride) {
    DecodeTilePages pages[kDecodeDepth];
#pragma unroll
    for (int j = 0; j < kDecodeDepth; ++j)
      pages[j] = find_decode_tile(table, ts0 + j * kStride, ke, block_size, col, quarter);
    DecodeTile tile[kDecodeDepth];
#pragma unroll
    for (int j = 0; j < kDecodeDepth; ++j)
      tile[j] = load_decode_tile(key_pages, value_pages, pages[j], ts0 + j * kStride, ke, first, kvh, kv_heads,
                                 block_size, num_pages, col, quarter);
#pragma unroll
    for (int j = 0; j < kDecodeDepth; ++j) {
      const int ts = ts0 + j * kStride;
      if (ts >= ke) break;
      DecodeTile& cur = tile[j];
      bad = bad || cur.bad;
      f32x4_t sc[2];
      float tmax = -INFINITY;
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        sc[half] = score_tile(cur.k[half], qo);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = ts + half * 16 + quarter * 4 + i;
          if (!(key >= first && key < ke)) {
            sc[half][i] = -INFINITY;
            // unwritten slots may hold NaN, and 0 * NaN would reach the output
            const uint32_t keep = (i & 1) ? 0x0000ffffu : 0xffff0000u;
#pragma unroll
            for (int dt = 0; dt < kDimTiles; ++dt) cur.v[dt][half][i / 2] &= keep;
          }
          tmax = fmaxf(tmax, sc[half][i]);
        }
      }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, kWave));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
      const float m_new = fmaxf(sm.m, tmax * scale2);
      const float m_use = (m_new == -INFINITY) ? 0.f : m_new;  // a column that has seen no key yet
      const float alpha = fast_exp2(sm.m - m_use);
      float sum = 0.f;
      float pr[2][4];
#pragma unroll
      for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          pr[half][i] = fast_exp2(fmaf(sc[half][i], scale2, -m_use));
          sum += pr[half][i];
        }
      sm.l = sm.l * alpha + sum;
      sm.m = m_new;
      if (__any(alpha != 1.0f)) {
#pragma unroll
        for (int dt = 0; dt < kDimTiles; ++dt)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[dt][i] *= alpha;
      }
      // k-slots 0..3 of a lane are its 4 keys of the first half, slots 4..7 those of the second
      const u32x4v_t pb = {pack_bf16x2(pr[0][0], pr[0][1]), pack_bf16x2(pr[0][2], pr[0][3]),
                           pack_bf16x2(pr[1][0], pr[1][1]), pack_bf16x2(pr[1][2], pr[1][3])};
      const bf16x8_t pop = __builtin_bit_cast(bf16x8_t, pb);
#pragma unroll
      for (int dt = 0; dt < kDimTiles; ++dt) {
        const u32x4v_t va = {cur.v[dt][0][0], cur.v[dt][0][1], cur.v[dt][1][0], cur.v[dt][1][1]};
        acc[dt] = mfma_16x16x32(__builtin_bit_cast(bf16x8_t, va), pop, acc[dt]);
      }
    }
  }

  // the column's sum is spread over the four lanes that share it
  sm.l += __shfl_xor(sm.l, 16, kWave);
  sm.l += __shfl_xor(sm.l, 32, kWave);
  if (bad) atomicOr(&sm_bad, 1);
  if (quarter == 0) {
    sm_m[wave][col] = sm.m;
    sm_l[wave][col] = sm.l;
  }
#pragma unroll
  for (int dt = 0; dt < kDimTiles; ++dt)
#pragma unroll
    for (int i = 0; i < 4; ++i) sm_acc[wave][col][dt * 16 + quarter * 4 + i] = acc[dt][i];
  __syncthreads();

  // merge the wavefronts; with one partition this is the result
  const bool poisoned = sm_bad != 0;
  const int tile_heads = min(16, group - htile * 16);
  for (int idx = tid; idx < tile_heads * D; idx += kDecodeWaves * kWave) {
    const int c = idx / D;
    const int d = idx - c * D;
    float mstar = -INFINITY;
#pragma unroll
    for (int w = 0; w < kDecodeWaves; ++w) mstar = fmaxf(mstar, sm_m[w][c]);
    float num = 0.f, den = 0.f;
#pragma unroll
    for (int w = 0; w < kDecodeWaves; ++w) {
      const float wgt = (sm_m[w][c] == -INFINITY) ? 0.f : fast_exp2(sm_m[w][c] - mstar);
      num += wgt * sm_acc[w][c][d];
      den += wgt * sm_l[w][c];
    }
    const int h = kvh * group + htile * 16 + c;
    if (splits == 1) {
      const float v = poisoned ? __builtin_nanf("") : num / den;
      out[(static_cast<int64_t>(t) * heads + h) * D + d] = f32_to_bf16(v);
    } else {
      float* dst = partial + ((static_cast<int64_t>(entry) * heads + h) * splits + split) * kPartialStride;
      dst[d] = poisoned ? __builtin_nanf("") : num;
      if (d == 0) {
        dst[D] = mstar;
        dst[D + 1] = den;
      }
    }
  }
}

// Merge of the partitions of one (entry, query head): m = max m_j, w_j = exp(m_j - m),
// O = sum w_j a_j / sum w_j l_j (csrc/paged_attention_split_cuda.cu:66-88 of the
// reference).  Lane j holds partition j's max and sum, so the weights come from two
// wavefront reductions; every lane then sums its output dims over the partitions
// with independent loads.
__global__ __launch_bounds__(kWave) void attn_decode_merge_kernel(const float* __restrict__ partial,
                                                                  const int* __restrict__ cu_q,
                                                                  const int* __restrict__ context_lens,
                                                                  bf16* __restrict__ out, int heads, int window,
                                                                  int part, int all_splits) {
  const int entry = blockIdx.x;
  const int h = blockIdx.y;
  const int lane = threadIdx.x;
  const int t = cu_q[entry];
  if (cu_q[entry + 1] - t != 1) return;
  const float* src = partial + (static_cast<int64_t>(entry) * heads + h) * all_splits * kPartialStride;
  // the partitions that hold keys of this entry (the others wrote nothing), as attn_decode cuts them
  const int ctx = context_lens[entry];
  const int first = window > 0 ? max(0, ctx - window) : 0;
  const int splits = min(all_splits, (ctx - (first / 16) * 16 + part - 1) / part);
  // The numerators are read kMergeBatch partitions at a time, all loads of a batch issued
  // before the first is used, and the first batch before the reductions below: this kernel's
  // time is the latency of its loads, so they must not wait for one another.
  constexpr int kPerLane = (D + kWave - 1) / kWave;
  constexpr int kMergeBatch = D <= 128 ? 16 : 8;
  float ms[kMergeBatch], piece[kMergeBatch][kPerLane];
  auto load_batch = [&](int s0) {
#pragma unroll
    for (int u = 0; u < kMergeBatch; ++u) {
      const int sp = min(s0 + u, splits - 1);
      ms[u] = src[sp * kPartialStride + D];
#pragma unroll
      for (int j = 0; j < kPerLane; ++j) {
        const int d = lane + j * kWave;
        piece[u][j] = d < D ? src[sp * kPartialStride + d] : 0.f;
      }
    }
  };
  load_batch(0);

  float mstar = -INFINITY;
  float den = 0.f;
  // more than 64 partitions: several rounds of the same two reductions
  for (int s0 = 0; s0 < splits; s0 += kWave) {
    const int sp = s0 + lane;
    const float m_sp = sp < splits ? src[sp * kPartialStride + D] : -INFINITY;
    const float l_sp = sp < splits ? src[sp * kPartialStride + D + 1] : 0.f;
    const float round_max = wave_max(m_sp);
    const float m_new = fmaxf(mstar, round_max);
    const float w = (m_sp == -INFINITY) ? 0.f : fast_exp2(m_sp - m_new);
    const float rescale = (mstar == -INFINITY) ? 0.f : fast_exp2(mstar - m_new);
    den = den * rescale + wave_sum(w * l_sp);
    mstar = m_new;
  }
  float num[kPerLane];
#pragma unroll
  for (int j = 0; j < kPerLane; ++j) num[j] = 0.f;
  for (int s0 = 0;;) {
#pragma unroll
    for (int u = 0; u < kMergeBatch; ++u) {
      const float w = (s0 + u >= splits || ms[u] == -INFINITY) ? 0.f : fast_exp2(ms[u] - mstar);
#pragma unroll
      for (int j = 0; j < kPerLane; ++j) num[j] += w * piece[u][j];
    }
    s0 += kMergeBatch;
    if (s0 >= splits) break;
    load_batch(s0);
  }
#pragma unroll
  for (int j = 0; j < (D + kWave - 1) / kWave; ++j) {
    const int d = lane + j * kWave;
    if (d < D) out[(static_cast<int64_t>(t) * heads + h) * D + d] = f32_to_bf16(num[j] / den);
  }
}

// ---- prefill ----------------------------------------------------------------------------------
constexpr int kTileQ = 64;                 // queries per workgroup (16 per wavefront), times QB (see the kernel)
constexpr int kTileK = D > 192 ? 32 : 64;  // key positions per LDS tile (bounded by LDS)
// Wavefront groups of a workgroup that take the key tiles in turn and merge at the end: a
// query tile's keys are a chain of dependent steps, and a second group halves it.  Measured:
// two groups for the small head sizes (where registers allow two workgroups of them per
// compute unit); four groups, or two for the larger head sizes, leave one workgroup per
// compute unit and are slower.
constexpr int kKeyGroups = D <= 64 ? 2 : 1;
constexpr int kSubTiles = kTileK / 16;
constexpr int kPairs = kSubTiles / 2;      // the value product takes 32 key positions per MFMA
// LDS rows are read 16 bytes a lane, 16 rows x 4 consecutive pieces per wavefront instruction.
// Measured on gfx950: that pattern is free of bank conflicts when the row stride is 32 bytes
// modulo 64, two-way conflicted at 16 or 48 modulo 64 and worse at multiples of 64; an 8-byte
// read costs as much as a 16-byte one.  So rows are padded to 32 modulo 64 bytes and every
// operand is one 16-byte read.
constexpr int kKLd = (D % 32 == 0) ? D + 16 : D;  // key row in LDS (elements)
constexpr int kVLd = kTileK + 16;                  // value row (one head dim, the tile's key positions)
constexpr int kPieces = (kTileK * (D / 8) + 255) / 256;  // 16-byte pieces per thread, of the key and of the value tile
constexpr int kNoPiece = 0x3fffffff;                      // position of a piece that a thread does not have
// The workgroup's flag lives in the padding of a key row where rows are padded (two
// workgroups of the small head sizes then fill a compute unit's 160 KB exactly), else behind the buffers.
constexpr int kFlagInPadding = kKLd > D;
constexpr int kPrefillLds = 2 * kKeyGroups * (kTileK * kKLd + D * kVLd) * 2 + (kFlagInPadding ? 0 : 16);  // bytes: two buffers per group

// Where key `k` of a tile lies in LDS.  The 16 rows that a score product reads for sub-tile
// 2 * pair + half hold the keys pair * 32 + 8 * (m / 4) + 4 * half + m % 4 (m = 0..15), so that a
// lane's accumulator elements of the pair's two sub-tiles (4 keys each) are 8 consecutive keys:
// exactly one 16-byte piece of a value row for the second product.
__host__ __device__ constexpr int key_row_in_lds(int k) {
  const int pair = k / 32, w = k % 32;
  return (2 * pair + (w % 8) / 4) * 16 + (w / 8) * 4 + w % 4;
}

// One key/value tile on its way from the pages to LDS.
struct TileInFlight {
  bf16x8_t k[kPieces];
  bf16x8_t v[kPieces];
};

// QB: blocks of 16 queries per wavefront (1 or 2).  With 2 a workgroup takes 128 queries and every
// key and value operand read from LDS serves two matrix-core products, which halves the LDS
// traffic per flop (LDS bandwidth, not the matrix cores, bounds the kernel with 1); it needs
// twice the accumulators and is offered up to head size 128.
// UNIFORM: the head size is a power of two and head size x page size at least 512 elements, so
// that the 64 pieces a wavefront moves with one instruction lie in one page: the page ids are then looked up with scalar loads
// and the addresses of the pieces are a scalar base plus a lane offset, which takes the
// address arithmetic (a third of the vector instructions of a tile) off the vector unit.
template <int QB, bool UNIFORM>
__global__ __launch_bounds__(256 * kKeyGroups) void attn_prefill_kernel(
    const bf16* __restrict__ q, int64_t q_stride, const bf16* __restrict__ key_pages,
    const bf16* __restrict__ value_pages, const int* __restrict__ block_table, int table_width,
    const int* __restrict__ tiles, const int* __restrict__ cu_q, const int* __restrict__ context_lens,
    bf16* __restrict__ out, int num_tiles, int heads, int kv_heads, int bs_shift, int num_pages, float scale,
    int window, float* __restrict__ partial) {
  // gridDim.y > 1: the keys of every tile are cut into that many runs, one workgroup each, which
  // leave their unnormalised results in `partial` for attn_prefill_merge (few tiles behind a long
  // context would otherwise be as many long chains on a few compute units).
  // Two groups of four wavefronts work on the same 64 queries; group g takes the key tiles
  // g, g + 2, g + 4, ... and the groups' states are merged at the end.  The heaviest tiles (the
  // end of a long prompt) bound the kernel's time by their chain of key tiles, one after the
  // other; this halves the chain and doubles the wavefronts that hide each other's latencies.
  // LDS: per group two buffers of (key tile, value tile), then a flag; offsets from one array
  // keep LDS addressing.
  extern __shared__ __attribute__((aligned(16))) unsigned char prefill_lds[];
  bf16* const lds = reinterpret_cast<bf16*>(prefill_lds);
  constexpr int kBuffer = kTileK * kKLd + D * kVLd;  // elements
  // the flag: in the padding of the last buffer's last key row (the groups' handover at the end
  // overlays the front of the buffers), or behind the buffers
  constexpr int kFlagAt = kFlagInPadding ? ((2 * kKeyGroups - 1) * kBuffer + (kTileK - 1) * kKLd + D) * 2 : 2 * kKeyGroups * kBuffer * 2;
  int& sm_bad = *reinterpret_cast<int*>(prefill_lds + kFlagAt);

  const int block_size = 1 << bs_shift;
  // Workgroup -> (tile, head).  The tile list comes heaviest first (a tile late in a long
  // prompt has many key tiles before it, an early one few), and all heads of a tile weigh the
  // same.  Workgroups are handed out round-robin, 256 to a round of the compute units, and
  // usually all are resident at once: even rounds take work from the heavy end of the list,
  // odd rounds from the light end, so that a compute unit's workgroups add up alike.
  const int total = num_tiles * heads;
  const int round = blockIdx.x / 256, in_round = blockIdx.x % 256;
  const int work = (round & 1) == 0 ? (round / 2) * 256 + in_round : total - 1 - ((round / 2) * 256 + in_round);
  const int tile = work / heads;
  const int head = work - tile * heads;
  const int entry = tiles[2 * tile];
  const int q0 = tiles[2 * tile + 1];
  const int kvh = head / (heads / kv_heads);
  constexpr int kWaveQ = 16 * QB;  // queries of a wavefront
  constexpr int kWgQ = kTileQ * QB;  // queries of the workgroup
  // uniform in a wavefront, and said so: everything derived from them (tile positions, the
  // conditions on them) then lives in scalar registers and scalar branches
  const int group = __builtin_amdgcn_readfirstlane(threadIdx.x / 256);  // key group
  const int tid = threadIdx.x % 256;                                     // thread within the group
  const int lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);  // which 16 queries
  const int col = lane % 16;
  const int quarter = lane / 16;

  const int t_first = cu_q[entry];
  const int q_len = cu_q[entry + 1] - t_first;
  const int ctx = context_lens[entry];
  const int pos0 = ctx - q_len;  // position of the entry's first new token
  const int* table = block_table + static_cast<int64_t>(entry) * table_width;
  if (threadIdx.x == 0) sm_bad = 0;

  // this lane's queries (columns of S^T), one per block
  int qi[QB], pq[QB], pq_first[QB];
  bool q_ok[QB];
  RowOperand qo[QB];
#pragma unroll
  for (int b = 0; b < QB; ++b) {
    qi[b] = q0 + wave * kWaveQ + b * 16 + col;
    q_ok[b] = qi[b] < q_len;
    pq[b] = pos0 + qi[b];  // its absolute position
    pq_first[b] = window > 0 ? max(0, pq[b] - window + 1) : 0;
    qo[b] = load_row(q + static_cast<int64_t>(t_first + (q_ok[b] ? qi[b] : 0)) * q_stride + static_cast<int64_t>(head) * D,
                     q_ok[b], quarter);
  }

  // key range of the workgroup: from the first query's window start to the last query's position
  const int last_q = min(q0 + kWgQ, q_len) - 1;
  const int k_end = pos0 + last_q + 1;
  const int k_begin_raw = window > 0 ? max(0, pos0 + q0 - window + 1) : 0;
  const int k_begin_all = (k_begin_raw / kTileK) * kTileK;
  // this workgroup's run of the keys: whole turns of the loop below (all key groups together)
  constexpr int kTurn = kKeyGroups * kTileK;
  const int splits = gridDim.y;
  const int turns = (k_end - k_begin_all + kTurn - 1) / kTurn;
  const int turns_each = (turns + splits - 1) / splits;
  const int k_begin = k_begin_all + static_cast<int>(blockIdx.y) * turns_each * kTurn;
  const int k_stop = min(k_end, k_begin + turns_each * kTurn);  // keys from here on belong to the next run
  // the wavefront's own range (uniform within the wavefront)
  const int w_last = pos0 + min(q0 + wave * kWaveQ + kWaveQ - 1, q_len - 1);
  const int w_first = window > 0 ? max(0, pos0 + q0 + wave * kWaveQ - window + 1) : 0;
  const bool wave_has_queries = q0 + wave * kWaveQ < q_len;
  // a tile is fully visible to the wavefront when it ends at or before its first query's position
  // and starts at or after its last query's window start (queries beyond q_len are never stored)
  const int w_min_pos = pos0 + q0 + wave * kWaveQ;
  const int w_max_first = window > 0 ? max(0, pos0 + q0 + wave * kWaveQ + kWaveQ - 1 - window + 1) : 0;
  // softmax in base 2: exp(x) = exp2(x * log2(e))
  const float scale2 = scale * 1.44269504088896340736f;

  float m_run[QB], l_run[QB];  // l: this lane's share of the sum
  f32x4_t acc[QB][kDimTiles];
#pragma unroll
  for (int b = 0; b < QB; ++b) {
    m_run[b] = -INFINITY;
    l_run[b] = 0.f;
#pragma unroll
    for (int dt = 0; dt < kDimTiles; ++dt) acc[b][dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }
  bool bad = false;

  // Which pieces of a tile each thread moves does not change from tile to tile: work out once
  // the page of the tile a piece lies in, its place inside that page and its place in LDS.
  // A tile is kTileK / block_size pages; a key page holds [offset][dim], a value page [dim][offset].
  const int bs_mask = block_size - 1;
  int k_row[kPieces], k_page[kPieces], k_in_page[kPieces], k_lds[kPieces];
#pragma unroll
  for (int i = 0; i < kPieces; ++i) {
    const int c = tid + i * 256;
    const int row = c / (D / 8);
    const int ch = c - row * (D / 8);
    k_row[i] = c < kTileK * (D / 8) ? row : kNoPiece;
    k_page[i] = row >> bs_shift;
    k_in_page[i] = (kvh * block_size + (row & bs_mask)) * D + ch * 8;
    k_lds[i] = key_row_in_lds(row % kTileK) * kKLd + ch * 8;
  }
  int v_pos[kPieces], v_page[kPieces], v_in_page[kPieces], v_lds[kPieces];
  const int per_page = D * (block_size / 8);  // 16-byte pieces of a value page (one kv head)
#pragma unroll
  for (int i = 0; i < kPieces; ++i) {
    const int c = tid + i * 256;
    const int pg = c / per_page;
    const int within = c - pg * per_page;
    const int d = within >> (bs_shift - 3);
    const int part = within & ((block_size >> 3) - 1);
    v_pos[i] = c < kTileK * (D / 8) ? pg * block_size + part * 8 : kNoPiece;  // first position, relative to the tile
    v_page[i] = pg;
    v_in_page[i] = (kvh * D + d) * block_size + part * 8;
    v_lds[i] = kTileK * kKLd + d * kVLd + pg * block_size + part * 8;
  }
  const uint32_t page_elems = static_cast<uint32_t>(kv_heads) * block_size * D;  // one multiply-add per address
  const int last_page = (k_end - 1) >> bs_shift;  // the last table entry that any query here may use

  // Loads are unconditional (a page that is absent or past the end reads page 0 instead) so
  // that the tile loop stays free of branches.  Keys read that way need no clearing: their
  // scores are masked by position.  Values are cleared, since 0 * NaN would reach the output;
  // that can only happen in the last tile and under a window, whose early pages may be gone.
  // The page ids of a tile are looked up one tile ahead of its loads (two ahead of its use):
  // a lookup right before the loads that need it would put two trips to memory, one after the
  // other, into every turn of the loop.
  int k_ids[kPieces], v_ids[kPieces];
  auto lookup = [&](int kt0) {
    const int page0 = kt0 >> bs_shift;
#pragma unroll
    for (int i = 0; i < kPieces; ++i) {
      const int kp = UNIFORM ? __builtin_amdgcn_readfirstlane(k_page[i]) : k_page[i];
      const int vp = UNIFORM ? __builtin_amdgcn_readfirstlane(v_page[i]) : v_page[i];
      k_ids[i] = table[min(page0 + kp, last_page)];
      v_ids[i] = table[min(page0 + vp, last_page)];
    }
  };
  auto fetch = [&](int kt0, TileInFlight& t) {  // with the ids that lookup(kt0) left
    const int lim = k_end - kt0;  // positions of this tile that exist
#pragma unroll
    for (int i = 0; i < kPieces; ++i) {
      const int page = k_ids[i];
      const bool in = static_cast<unsigned>(page) < static_cast<unsigned>(num_pages);
      if (!in) bad = bad || (k_row[i] < lim && kt0 + k_row[i] >= k_begin_raw);
      t.k[i] = load_bf16x8(key_pages + (static_cast<uint64_t>(in ? static_cast<uint32_t>(page) : 0u) * page_elems + k_in_page[i]));
    }
    const bool guard = lim < kTileK || window > 0;  // uniform
#pragma unroll
    for (int i = 0; i < kPieces; ++i) {
      const int page = v_ids[i];
      const bool in = static_cast<unsigned>(page) < static_cast<unsigned>(num_pages);
      bf16x8_t val = load_bf16x8(value_pages + (static_cast<uint64_t>(in ? static_cast<uint32_t>(page) : 0u) * page_elems + v_in_page[i]));
      if (guard) {
        asm volatile("" ::: "memory");  // keeps this a branch that full tiles skip
        u16x8_t bits = __builtin_bit_cast(u16x8_t, val);
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (!in || v_pos[i] + e >= lim) bits[e] = 0;
        val = __builtin_bit_cast(bf16x8_t, bits);
      }
      t.v[i] = val;
    }
  };
  auto stash = [&](const TileInFlight& t, int buf) {
#pragma unroll
    for (int i = 0; i < kPieces; ++i)
      if (k_row[i] != kNoPiece) {
        *reinterpret_cast<bf16x8_t*>(lds + (buf * kKeyGroups + group) * kBuffer + k_lds[i]) = t.k[i];
        *reinterpret_cast<bf16x8_t*>(lds + (buf * kKeyGroups + group) * kBuffer + v_lds[i]) = t.v[i];
      }
  };

  // The query has to be there before the loop: a load still pending at the loop's head makes
  // the compiler wait, in every turn, for everything in flight, the next tile's loads included.
#pragma unroll
  for (int b = 0; b < QB; ++b)
#pragma unroll
    for (int st = 0; st < kSteps; ++st) asm volatile("" ::"v"(qo[b].step[st]));

  TileInFlight flight;
  constexpr int kStep = kKeyGroups * kTileK;  // keys per turn of the loop, all groups together
  const int k_mine = k_begin + group * kTileK;  // this group's first tile
  if (k_mine < k_stop) {
    lookup(k_mine);
    fetch(k_mine, flight);
    lookup(k_mine + kStep);
    stash(flight, 0);
  }
  __syncthreads();
  int buf = 0;
  for (int kt0 = k_mine; kt0 - group * kTileK < k_stop; kt0 += kStep, buf ^= 1) {  // as many turns for every group
    const bool mine = kt0 < k_stop;
    const bool more = kt0 + kStep < k_stop;
    if (more) {
      fetch(kt0 + kStep, flight);  // in flight while this tile is computed
      lookup(kt0 + 2 * kStep);
    }
    const bf16* ks = lds + (buf * kKeyGroups + group) * kBuffer;
    const bf16* vs = ks + kTileK * kKLd;

    if (mine && wave_has_queries && kt0 <= w_last && kt0 + kTileK - 1 >= w_first) {
      // Scores of the whole tile, then ONE softmax update for its kTileK positions.  The
      // vector ALU, not the matrix core, bounds this loop (a wavefront instruction takes four
      // cycles, an exponential sixteen), so every per-score operation counts: the scale is
      // folded into the exponent's multiply-add, hidden scores are -inf and become 0 in the
      // exponential by themselves, and only tiles that cross a query's limits build masks.
      f32x4_t s[QB][kSubTiles];
      const bool full = kt0 + kTileK - 1 <= w_min_pos && kt0 >= w_max_first;  // uniform in the wavefront
#pragma unroll
      for (int sub = 0; sub < kSubTiles; ++sub) {
        const RowOperand keys = load_row(ks + (sub * 16 + col) * kKLd, true, quarter);
#pragma unroll
        for (int b = 0; b < QB; ++b) s[b][sub] = score_tile(keys, qo[b]);
      }
      // The value operands of the tile's first 32 keys leave LDS now: the softmax below hides
      // their way, which would otherwise be waited for once per product.
      typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
      auto value_operand = [&](int dt, int pr) {  // dim dt * 16 + col, keys pr * 32 + quarter * 8 .. + 7
        return *reinterpret_cast<const u32x4_t*>(vs + (dt * 16 + col) * kVLd + pr * 32 + quarter * 8);
      };
      constexpr bool kValuesAhead = kDimTiles * QB <= 8;  // registers allow it
      u32x4_t ahead[kValuesAhead ? kDimTiles : 1];
      if constexpr (kValuesAhead) {
#pragma unroll
        for (int dt = 0; dt < kDimTiles; ++dt) ahead[dt] = value_operand(dt, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (!full) {
        // a branch of its own: folded into selects, these comparisons would run for every tile
        asm volatile("" ::: "memory");
#pragma unroll
        for (int b = 0; b < QB; ++b)
#pragma unroll
          for (int sub = 0; sub < kSubTiles; ++sub)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int key = kt0 + (sub / 2) * 32 + quarter * 8 + (sub % 2) * 4 + i;  // see key_row_in_lds
              if (!(q_ok[b] && key <= pq[b] && key >= pq_first[b])) s[b][sub][i] = -INFINITY;
            }
      }
      uint32_t pw[QB][kSubTiles][2];
#pragma unroll
      for (int b = 0; b < QB; ++b) {
        float tmax = -INFINITY;
#pragma unroll
        for (int sub = 0; sub < kSubTiles; ++sub)
#pragma unroll
          for (int i = 0; i < 4; ++i) tmax = fmaxf(tmax, s[b][sub][i]);
        tmax = fmaxf(tmax, __shfl_xor(tmax, 16, kWave));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
        const float m_new = fmaxf(m_run[b], tmax * scale2);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;  // a column that has seen no key yet
        const float alpha = fast_exp2(m_run[b] - m_use);          // 2^-inf = 0 for the first tile
        float sum = 0.f;
#pragma unroll
        for (int sub = 0; sub < kSubTiles; ++sub) {
          float p[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            p[i] = fast_exp2(fmaf(s[b][sub][i], scale2, -m_use));
            sum += p[i];
          }
          pw[b][sub][0] = pack_bf16x2(p[0], p[1]);
          pw[b][sub][1] = pack_bf16x2(p[2], p[3]);
        }
        l_run[b] = l_run[b] * alpha + sum;
        m_run[b] = m_new;
        if (__any(alpha != 1.0f)) {
#pragma unroll
          for (int dt = 0; dt < kDimTiles; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[b][dt][i] *= alpha;
        }
      }
      // O^T += V^T P^T, 32 key positions per MFMA: k-slots 0..3 of a lane are its 4 keys of the
      // pair's first sub-tile, slots 4..7 those of the second: 8 consecutive keys, by the order of the
      // key rows in LDS
#pragma unroll
      for (int pr = 0; pr < kPairs; ++pr) {
        bf16x8_t pop[QB];
#pragma unroll
        for (int b = 0; b < QB; ++b) {
          const u32x4_t pb = {pw[b][2 * pr][0], pw[b][2 * pr][1], pw[b][2 * pr + 1][0], pw[b][2 * pr + 1][1]};
          pop[b] = __builtin_bit_cast(bf16x8_t, pb);
        }
#pragma unroll
        for (int dt = 0; dt < kDimTiles; ++dt) {
          const u32x4_t va = (kValuesAhead && pr == 0) ? ahead[dt] : value_operand(dt, pr);
#pragma unroll
          for (int b = 0; b < QB; ++b) acc[b][dt] = mfma_16x16x32(__builtin_bit_cast(bf16x8_t, va), pop[b], acc[b][dt]);
        }
      }
    }

    // the other buffer was last read one iteration ago, before that iteration's barrier
    if (more) stash(flight, buf ^ 1);
    __syncthreads();
  }

  // merge the key groups: the second hands its state over through LDS (the tiles are done with)
  float* const handover = reinterpret_cast<float*>(prefill_lds);  // [group - 1][block][component][thread of the group]
  constexpr int kPerBlock = (2 + kDimTiles * 4) * 256;
  constexpr int kHandover = QB * kPerBlock;
  static_assert((kKeyGroups - 1) * kHandover * 4 <= kFlagAt, "the handover fits the tile buffers in front of the flag");
  if (kKeyGroups > 1 && group > 0) {
#pragma unroll
    for (int b = 0; b < QB; ++b) {
      float* mine = handover + (group - 1) * kHandover + b * kPerBlock;
      mine[tid] = m_run[b];
      mine[256 + tid] = l_run[b];
#pragma unroll
      for (int dt = 0; dt < kDimTiles; ++dt)
#pragma unroll
        for (int i = 0; i < 4; ++i) mine[(2 + dt * 4 + i) * 256 + tid] = acc[b][dt][i];
    }
  }
  if (bad) atomicOr(&sm_bad, 1);
  __syncthreads();
  if (group != 0) return;
  const bool poisoned = sm_bad != 0;
#pragma unroll
  for (int b = 0; b < QB; ++b) {
#pragma unroll
    for (int g = 1; g < kKeyGroups; ++g) {  // in the groups' order, whichever finished first
      const float* other = handover + (g - 1) * kHandover + b * kPerBlock;
      const float m_other = other[tid];
      const float m_new = fmaxf(m_run[b], m_other);
      const float w_mine = (m_run[b] == -INFINITY) ? 0.f : fast_exp2(m_run[b] - m_new);
      const float w_other = (m_other == -INFINITY) ? 0.f : fast_exp2(m_other - m_new);
      l_run[b] = l_run[b] * w_mine + other[256 + tid] * w_other;
#pragma unroll
      for (int dt = 0; dt < kDimTiles; ++dt)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          acc[b][dt][i] = acc[b][dt][i] * w_mine + other[(2 + dt * 4 + i) * 256 + tid] * w_other;
      m_run[b] = m_new;
    }
    float l = l_run[b];
    l += __shfl_xor(l, 16, kWave);
    l += __shfl_xor(l, 32, kWave);
    if (splits > 1) {
      // this run's share, unnormalised: [tile, head, run, query of the tile, head size + 2]
      float* dst = partial + (((static_cast<int64_t>(tile) * heads + head) * splits + blockIdx.y) * kWgQ +
                              (wave * kWaveQ + b * 16 + col)) * kPartialStride;
      typedef float f32x2_t __attribute__((ext_vector_type(2)));
#pragma unroll
      for (int dt = 0; dt < kDimTiles; ++dt) {
        const float nan = __builtin_nanf("");
        *reinterpret_cast<f32x2_t*>(dst + dt * 16 + quarter * 4) =
            f32x2_t{poisoned ? nan : acc[b][dt][0], poisoned ? nan : acc[b][dt][1]};
        *reinterpret_cast<f32x2_t*>(dst + dt * 16 + quarter * 4 + 2) =
            f32x2_t{poisoned ? nan : acc[b][dt][2], poisoned ? nan : acc[b][dt][3]};
      }
      if (quarter == 0) {
        dst[D] = m_run[b];
        dst[D + 1] = l;
      }
      continue;
    }
    if (q_ok[b]) {
      const float inv = 1.0f / l;
      bf16* orow = out + (static_cast<int64_t>(t_first + qi[b]) * heads + head) * D;
#pragma unroll
      for (int dt = 0; dt < kDimTiles; ++dt) {
        u16x4_t packed;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          packed[i] = f32_to_bf16(poisoned ? __builtin_nanf("") : acc[b][dt][i] * inv).bits;
        *reinterpret_cast<u16x4_t*>(orow + dt * 16 + quarter * 4) = packed;
      }
    }
  }
}

// Merge of the key runs of a prompt tile (see attn_prefill_kernel): for every query of the tile
// and every head, m = max m_j, w_j = 2^(m_j - m), O = sum w_j a_j / sum w_j l_j, in the runs'
// order.  One workgroup per (tile, head).
__global__ __launch_bounds__(256) void attn_prefill_merge_kernel(const float* __restrict__ partial,
                                                                 const int* __restrict__ tiles,
                                                                 const int* __restrict__ cu_q,
                                                                 bf16* __restrict__ out, int heads, int splits,
                                                                 int tile_q) {
  const int tile = blockIdx.x / heads;
  const int head = blockIdx.x - tile * heads;
  const int entry = tiles[2 * tile];
  const int q0 = tiles[2 * tile + 1];
  const int t_first = cu_q[entry];
  const int q_len = cu_q[entry + 1] - t_first;
  const float* base = partial + static_cast<int64_t>(blockIdx.x) * splits * tile_q * kPartialStride;
  for (int idx = threadIdx.x; idx < tile_q * (D / 2); idx += 256) {
    const int qq = idx / (D / 2);
    const int d = (idx - qq * (D / 2)) * 2;
    if (q0 + qq >= q_len) continue;
    float mstar = -INFINITY;
    for (int sp = 0; sp < splits; ++sp)
      mstar = fmaxf(mstar, base[(static_cast<int64_t>(sp) * tile_q + qq) * kPartialStride + D]);
    float num0 = 0.f, num1 = 0.f, den = 0.f;
    for (int sp = 0; sp < splits; ++sp) {
      const float* row = base + (static_cast<int64_t>(sp) * tile_q + qq) * kPartialStride;
      const float m = row[D];
      const float w = (m == -INFINITY) ? 0.f : fast_exp2(m - mstar);
      num0 += w * row[d];
      num1 += w * row[d + 1];
      den += w * row[D + 1];
    }
    bf16* orow = out + (static_cast<int64_t>(t_first + q0 + qq) * heads + head) * D;
    orow[d] = f32_to_bf16(num0 / den);
    orow[d + 1] = f32_to_bf16(num1 / den);
  }
}

}  // namespace mlr

using namespace mlr;

extern "C" {

int mlr_attention_head_dim() { return D; }

// Key positions per LDS tile of the prefill kernel; block_size must divide it.
int mlr_attention_key_tile() { return kTileK; }

// Floats of scratch the decode kernel needs for `splits` partitions.
int64_t mlr_attention_decode_scratch(int entries, int heads, int splits) {
  return splits <= 1 ? 0 : static_cast<int64_t>(entries) * heads * splits * kPartialStride;
}

// Attention of every single-token entry (entries with more tokens are skipped).
// Keys of an entry are cut into `splits` partitions of `part` positions (a
// multiple of 64); with more than one partition `partial` must hold
// mlr_attention_decode_scratch floats, laid out [entry, head, split, head size + 2]
// (numerator, maximum in base 2, denominator).  `merge` 0 leaves the partitions unmerged in
// `partial` for a consumer that merges them itself (or for mlr_attention_decode_merge).
int mlr_attention_decode(const void* q, int64_t q_stride, const void* key_pages, const void* value_pages,
                         const int* block_table, int table_width, const int* cu_q, const int* context_lens,
                         void* out, float* partial, int entries, int heads, int kv_heads, int block_size,
                         int num_pages, float scale, int window, int part, int splits, int merge,
                         hipStream_t stream) {
  MLR_REQUIRE(q && key_pages && value_pages && block_table && cu_q && context_lens && out, "null pointer");
  MLR_REQUIRE(entries > 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "bad head counts");
  MLR_REQUIRE(block_size > 0 && block_size % 4 == 0, "block_size must be a multiple of 4");
  MLR_REQUIRE(num_pages > 0 && table_width > 0, "page sizes must be > 0");
  MLR_REQUIRE(part > 0 && part % 64 == 0, "part must be a positive multiple of 64");
  MLR_REQUIRE(splits >= 1 && splits <= 65535, "splits out of range");
  MLR_REQUIRE(splits == 1 || partial != nullptr, "several partitions need scratch memory");
  MLR_REQUIRE(q_stride >= static_cast<int64_t>(heads) * D && q_stride % 8 == 0, "q_stride must cover a row and keep 16-byte alignment");
  MLR_REQUIRE(reinterpret_cast<uintptr_t>(q) % 16 == 0 && reinterpret_cast<uintptr_t>(key_pages) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(value_pages) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 8 == 0,
              "operands must be 16-byte aligned");
  MLR_REQUIRE(scale > 0.f && scale < INFINITY && window >= 0, "bad scale or window");
  const int group = heads / kv_heads;
  const int head_tiles = (group + 15) / 16;
  MLR_REQUIRE(kv_heads * head_tiles <= 65535, "too many heads for one launch");
  dim3 grid(entries, kv_heads * head_tiles, splits);
  const bf16* qp = static_cast<const bf16*>(q);
  const bf16* kp = static_cast<const bf16*>(key_pages);
  const bf16* vp = static_cast<const bf16*>(value_pages);
  bf16* op = static_cast<bf16*>(out);
  const int tiles_per_wave = (part + 32 * kDecodeWaves - 1) / (32 * kDecodeWaves);
#define MLR_DECODE(depth)                                                                                       \
  attn_decode_kernel<depth><<<grid, kDecodeWaves * kWave, 0, stream>>>(                                         \
      qp, q_stride, kp, vp, block_table, table_width, cu_q, context_lens, op, partial, heads, kv_heads,         \
      head_tiles, block_size, num_pages, scale, window, part, splits)
  bool launched = false;
  if constexpr (kMaxDecodeDepth >= 4) {
    if (tiles_per_wave >= 4) {
      MLR_DECODE(4);
      launched = true;
    }
  }
  if constexpr (kMaxDecodeDepth >= 2) {
    if (!launched && tiles_per_wave >= 2) {
      MLR_DECODE(2);
      launched = true;
    }
  }
  if (!launched) MLR_DECODE(1);
#undef MLR_DECODE
  MLR_LAUNCH_CHECK();
  if (splits > 1 && merge) {
    attn_decode_merge_kernel<<<dim3(entries, heads), kWave, 0, stream>>>(
        partial, cu_q, context_lens, static_cast<bf16*>(out), heads, window, part, splits);
    MLR_LAUNCH_CHECK();
  }
  return 0;
}

// The merge that mlr_attention_decode left out: out[t] of every single-token entry from its
// partitions in `partial`.
int mlr_attention_decode_merge(const float* partial, const int* cu_q, const int* context_lens, void* out, int entries,
                               int heads, int window, int part, int splits, hipStream_t stream) {
  MLR_REQUIRE(partial && cu_q && context_lens && out, "null pointer");
  MLR_REQUIRE(entries > 0 && heads > 0 && heads <= 65535, "bad sizes");
  MLR_REQUIRE(part > 0 && part % 64 == 0 && splits > 1 && window >= 0, "bad partitions");
  attn_decode_merge_kernel<<<dim3(entries, heads), kWave, 0, stream>>>(partial, cu_q, context_lens,
                                                                      static_cast<bf16*>(out), heads, window, part, splits);
  MLR_LAUNCH_CHECK();
  return 0;
}

// Queries per tile of the wide variant of mlr_attention_prefill (`wide` = 1); 0 if this head
// size has none.
int mlr_attention_wide_tile() { return D <= 128 ? 2 * kTileQ : 0; }

// Floats of scratch mlr_attention_prefill needs when the keys of every tile are cut into
// `splits` runs (0 for one run).
int64_t mlr_attention_prefill_scratch(int num_tiles, int heads, int splits, int wide) {
  if (splits <= 1) return 0;
  return static_cast<int64_t>(num_tiles) * heads * splits * (wide ? 2 * kTileQ : kTileQ) * kPartialStride;
}

// Attention of the query tiles listed in `tiles` ([num_tiles][2]: entry, first
// query of the tile within the entry's new tokens; 64 queries per tile, or
// mlr_attention_wide_tile() with `wide`).  splits > 1: the keys of every tile are cut into that
// many runs, each a workgroup of its own, and merged by a second kernel; `partial` then holds
// mlr_attention_prefill_scratch floats.  For few tiles behind long contexts.
int mlr_attention_prefill(const void* q, int64_t q_stride, const void* key_pages, const void* value_pages,
                          const int* block_table, int table_width, const int* tiles, int num_tiles, int wide,
                          const int* cu_q, const int* context_lens, void* out, int heads, int kv_heads,
                          int block_size, int num_pages, float scale, int window, int splits, float* partial,
                          hipStream_t stream) {
  MLR_REQUIRE(splits >= 1 && splits <= 64, "splits must lie within 1..64");
  MLR_REQUIRE(splits == 1 || partial != nullptr, "several key runs need scratch memory");
  MLR_REQUIRE(q && key_pages && value_pages && block_table && tiles && cu_q && context_lens && out, "null pointer");
  MLR_REQUIRE(num_tiles > 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "bad sizes");
  MLR_REQUIRE(kv_heads <= 65535, "too many key/value heads");  // a page's elements fit 32 bits
  MLR_REQUIRE(block_size >= 8 && (block_size & (block_size - 1)) == 0 && block_size <= kTileK,
              "block_size must be a power of two within 8 and the key tile");
  MLR_REQUIRE(!wide || mlr_attention_wide_tile() > 0, "this head size has no wide query tiles");
  int bs_shift = 0;
  while ((1 << bs_shift) < block_size) ++bs_shift;
  MLR_REQUIRE(num_pages > 0 && table_width > 0, "page sizes must be > 0");
  MLR_REQUIRE(q_stride >= static_cast<int64_t>(heads) * D && q_stride % 8 == 0, "q_stride must cover a row and keep 16-byte alignment");
  MLR_REQUIRE(reinterpret_cast<uintptr_t>(q) % 16 == 0 && reinterpret_cast<uintptr_t>(key_pages) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(value_pages) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 8 == 0,
              "operands must be 16-byte aligned");
  MLR_REQUIRE(scale > 0.f && scale < INFINITY && window >= 0, "bad scale or window");
  MLR_REQUIRE(static_cast<int64_t>(num_tiles) * heads < (1ll << 31), "too many tiles for one launch");
  static bool configured = false;
  if (!configured) {
    hipError_t e = hipSuccess;
    const void* kernels[] = {reinterpret_cast<const void*>(attn_prefill_kernel<1, false>),
                             reinterpret_cast<const void*>(attn_prefill_kernel<1, true>),
                             reinterpret_cast<const void*>(attn_prefill_kernel<D <= 128 ? 2 : 1, false>),
                             reinterpret_cast<const void*>(attn_prefill_kernel<D <= 128 ? 2 : 1, true>)};
    for (const void* kernel : kernels)
      if (e == hipSuccess) e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kPrefillLds);
    if (e != hipSuccess) {
      set_error(std::string("mlr_attention_prefill: cannot raise the LDS limit: ") + hipGetErrorString(e));
      return -1;
    }
    configured = true;
  }
  const dim3 grid(static_cast<unsigned>(num_tiles) * heads, splits);
  // a wavefront's 64 pieces of a tile lie in one page: whole key rows (D / 8 pieces each, a power
  // of two) that fit a page, and as many pieces of a value page
  const bool uniform = (D & (D - 1)) == 0 && D * block_size >= 512;
#define MLR_PREFILL(qb)                                                                                       \
  do {                                                                                                        \
    if (uniform)                                                                                              \
      attn_prefill_kernel<qb, true><<<grid, 256 * kKeyGroups, kPrefillLds, stream>>>(                         \
          static_cast<const bf16*>(q), q_stride, static_cast<const bf16*>(key_pages),                         \
          static_cast<const bf16*>(value_pages), block_table, table_width, tiles, cu_q, context_lens,         \
          static_cast<bf16*>(out), num_tiles, heads, kv_heads, bs_shift, num_pages, scale, window, partial);  \
    else                                                                                                      \
      attn_prefill_kernel<qb, false><<<grid, 256 * kKeyGroups, kPrefillLds, stream>>>(                        \
          static_cast<const bf16*>(q), q_stride, static_cast<const bf16*>(key_pages),                         \
          static_cast<const bf16*>(value_pages), block_table, table_width, tiles, cu_q, context_lens,         \
          static_cast<bf16*>(out), num_tiles, heads, kv_heads, bs_shift, num_pages, scale, window, partial);  \
  } while (0)
  if constexpr (D <= 128) {
    if (wide)
      MLR_PREFILL(2);
    else
      MLR_PREFILL(1);
  } else {
    MLR_PREFILL(1);
  }
#undef MLR_PREFILL
  MLR_LAUNCH_CHECK();
  if (splits > 1) {
    const int tile_q = (wide && D <= 128) ? 2 * kTileQ : kTileQ;
    attn_prefill_merge_kernel<<<dim3(static_cast<unsigned>(num_tiles) * heads), 256, 0, stream>>>(
        partial, tiles, cu_q, static_cast<bf16*>(out), heads, splits, tile_q);
    MLR_LAUNCH_CHECK();
  }
  return 0;
}

}  // extern "C"
