// bfloat16 matrix products on the matrix cores: y[M, N] = x[M, K] * w[N, K]^T (+ bias).
//
// Both operands have k as their fastest index, which is what MFMA wants of both
// inputs, so tiles go from memory to the operand registers without a transpose.
// The weight tile is the A operand and the activation tile the B operand: the
// accumulator then holds four consecutive output features of one token per lane,
// which gives 8-byte stores and lets an epilogue see neighbouring features.
//
// Kernels:
//  * gemm_skinny_split: up to 16 tokens (decode at small batch).  Bound by streaming
//    w once, and a single compute unit can only keep a few dozen cache lines in
//    flight, so the stream has to be spread over all of them: a workgroup owns 16
//    output features and one slice of K (grid.y slices); its wavefronts split the
//    slice between them (interleaved, so the workgroup reads contiguous spans of
//    every weight row), keep eight 16-byte loads in flight per lane, and add their
//    partial sums through LDS.  Activations come straight from L2.
//  * gemm_tiled: everything else.  An output tile per workgroup (256 x 256 with
//    sixteen wavefronts for large products, 128 x 128 or 64 x 64 with four, whichever
//    is the largest that still keeps the compute units busy), K in
//    slices of 64 staged through double-buffered LDS by range-checked
//    buffer loads (edge tiles and the tail of K read zeros, no branches),
//    32x32x16 MFMA.  Beyond 64 tokens the two larger tilings run gemm_direct: the same tiles
//    loaded straight into LDS (no registers, no LDS stores; rows swizzled instead of padded),
//    with a step's barrier ahead of its last quarter of products.  Workgroups are placed so that those resident on
//    one XCD share operands in its L2.  Up to 16 tokens take this kernel too once
//    its tiles fill the compute units (it streams a wide weight fastest).
//    With more than one K slice both kernels write float32 partial sums
//    [slice, M, N]; the consumer (the residual-adding norm kernel) sums them in a
//    fixed order, so results do not depend on which slice finishes first.
//  * Both also run the query/key/value product with bias, rotation and the cache write as
//    their epilogue (QkvTarget): the streaming kernel for up to 64 tokens (in slabs of 16),
//    the tiled one beyond.
// K must be a multiple of 8 (16-byte rows); other shapes take the FMA kernel.
//
// SwiGLU epilogue: with gate and up rows interleaved in pairs
// (g0 g1 u0 u1 g2 g3 u2 u3 ...) a lane holds two gate sums and their two up sums
// and stores silu(gate) * up (src/mini_llm_runtime/qwen_model_runner.py:215-216)
// directly, which saves a kernel and a round trip of the widest activation.
#include "api.h"
#include "common.h"
#include "mfma.h"
#include "gemm_epilogue.h"

namespace mlr {

// ---- skinny, up to 16 tokens: wavefronts split K ------------------------------------------
// MT: slabs of 16 tokens a workgroup multiplies its weight rows with (1 for the plain product).
template <int WAVES, bool QKV, int MT>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_split_kernel(const bf16* __restrict__ x,
                                                                       const bf16* __restrict__ w,
                                                                       GemmEpilogue ep, QkvTarget qkv, int M, int N,
                                                                       int K) {
  constexpr int U = MT > 2 ? 4 : 8;  // k-steps in flight per wavefront
  __shared__ float red[WAVES][MT][kWave][4];
  __shared__ float scales[MT * 16];
  RowScaleLoads<MT * 16 / WAVES, 4 / MT> owed;  // up to 256 partial sums a row for 16 tokens, 64 for 64 tokens
  const int token0 = blockIdx.z * (MT * 16);  // grid.z: further groups of MT slabs, a workgroup each
  if (ep.row_sumsq != nullptr) row_scales_issue(ep, owed, token0, min(M - token0, MT * 16), M);
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int r = lane % 16;
  const int q = lane / 16;
  const int n0 = blockIdx.x * 16;
  const int slices = gridDim.y;
  const int chunks = K / 8;             // 16-byte chunks per row
  const int ksteps = (chunks + 3) / 4;  // one MFMA consumes 4 chunks (32 elements of k)
  const int per = (ksteps + slices - 1) / slices;
  const int sb = blockIdx.y * per;
  const int se = min(ksteps, sb + per);
  // the weight row behind accumulator row `slot` of this workgroup
  int head = 0, block_in_head = 0;
  bool rotated = false;
  if constexpr (QKV) {
    const int per_head = qkv.head_dim / 16;
    head = blockIdx.x / per_head;
    block_in_head = blockIdx.x - head * per_head;
    rotated = qkv.cos != nullptr && head < qkv.heads + qkv.kv_heads;
  }
  auto row_of = [&](int slot) {
    if (!rotated) return n0 + slot;
    return head * qkv.head_dim + block_in_head * 8 + (slot < 8 ? slot : qkv.head_dim / 2 + slot - 8);
  };
  const bf16x8_t* wp = reinterpret_cast<const bf16x8_t*>(w + static_cast<int64_t>(min(row_of(r), N - 1)) * K);
  const bf16x8_t* xp[MT];
  bool xok[MT];
  f32x4_t acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    xp[mt] = reinterpret_cast<const bf16x8_t*>(x + static_cast<int64_t>(min(token0 + mt * 16 + r, M - 1)) * K);
    xok[mt] = token0 + mt * 16 + r < M;
    acc[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }

  for (int s0 = sb + wave; s0 < se; s0 += WAVES * U) {
    bf16x8_t a[U], b[U][MT];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int s = s0 + u * WAVES;
      const int c = s * 4 + q;
      a[u] = (s < se && c < chunks) ? __builtin_nontemporal_load(wp + c) : zero_bf16x8();
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int s = s0 + u * WAVES;
      const int c = s * 4 + q;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) b[u][mt] = (xok[mt] && s < se && c < chunks) ? xp[mt][c] : zero_bf16x8();
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[mt] = mfma_16x16x32(a[u], b[u][mt], acc[mt]);
  }

#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[wave][mt][lane][i] = acc[mt][i];
  if (ep.row_sumsq != nullptr) row_scales_finish(ep, owed, token0, min(M - token0, MT * 16), M, K, scales);
  __syncthreads();
  // Slab mt is finished by wavefront mt % WAVES: the epilogue of a slab waits for memory more than once
  // (rotation tables, cache slots, the stores), and one wavefront doing four slabs in turn was a third
  // of the kernel's time at 64 tokens.
  if (wave >= MT) return;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    if (mt % WAVES != wave) continue;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    for (int ww = 0; ww < WAVES; ++ww)
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] += red[ww][mt][lane][i];
    const int token = token0 + mt * 16 + r;
    if (ep.row_sumsq != nullptr && token < M) {
      const float scale = scales[mt * 16 + r];
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] *= scale;
    }
    if constexpr (!QKV) {
      finish4(ep, blockIdx.y, slices, token, n0 + q * 4, M, N, v);
    } else {
      // the lane holds accumulator rows 4q..4q+3 of its token: four consecutive dims of one head
      qkv_finish(ep, qkv, head, block_in_head, rotated, row_of(q * 4) - head * qkv.head_dim, q, min(token, M - 1),
                 token < M, v);
    }
  }
}

// ---- skinny fused query/key/value product, up to 8 tokens: 8 weight rows a workgroup ----------
// The 16 x 16 matrix-core block is filled with two halves of K instead of 16 weight rows: lane
// rows 0..7 multiply the 8 weight rows with the tokens over the first half of K, rows 8..15 the
// same weight rows over the second half; tokens 0..7 stand in columns 0..7 and again in 8..15.
// The two diagonal quadrants of the result are the two partial sums, the others are not used.
// Every lane still streams weights, and there are twice as many workgroups as with 16 rows each,
// which counts where those leave compute units without work or give a few of them two.
template <int WAVES>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_qkv8_kernel(const bf16* __restrict__ x,
                                                                      const bf16* __restrict__ w, GemmEpilogue ep,
                                                                      QkvTarget qkv, int M, int N, int K) {
  constexpr int U = 8;  // k-steps in flight per wavefront
  __shared__ float red[WAVES][kWave][4];
  __shared__ float scales[8];
  RowScaleLoads<8 / WAVES, 4> owed;
  if (ep.row_sumsq != nullptr) row_scales_issue(ep, owed, 0, min(M, 8), M);
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int r = lane % 16;
  const int q = lane / 16;
  const int r8 = r % 8;
  const int n0 = blockIdx.x * 8;
  const int chunks = K / 8;
  const int ksteps = (chunks + 3) / 4;
  const int half_steps = (ksteps + 1) / 2;
  const int shift = (r / 8) * half_steps;  // the k-step this lane's half of K starts at
  const int per_head = qkv.head_dim / 8;
  const int head = blockIdx.x / per_head;
  const int block_in_head = blockIdx.x - head * per_head;
  const bool rotated = qkv.cos != nullptr && head < qkv.heads + qkv.kv_heads;
  // the weight row behind slot 0..7: four low halves of rotation pairs, then their high halves
  auto row_of = [&](int slot) {
    if (!rotated) return n0 + slot;
    return head * qkv.head_dim + block_in_head * 4 + (slot < 4 ? slot : qkv.head_dim / 2 + slot - 4);
  };
  const bf16x8_t* wp = reinterpret_cast<const bf16x8_t*>(w + static_cast<int64_t>(min(row_of(r8), N - 1)) * K);
  const bf16x8_t* xp = reinterpret_cast<const bf16x8_t*>(x + static_cast<int64_t>(min(r8, M - 1)) * K);
  const bool xok = r8 < M;
  f32x4_t acc{0.f, 0.f, 0.f, 0.f};

  for (int s0 = wave; s0 < half_steps; s0 += WAVES * U) {
    bf16x8_t a[U], b[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int s = s0 + u * WAVES;
      const int c = (s + shift) * 4 + q;
      a[u] = (s < half_steps && s + shift < ksteps && c < chunks) ? __builtin_nontemporal_load(wp + c) : zero_bf16x8();
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int s = s0 + u * WAVES;
      const int c = (s + shift) * 4 + q;
      b[u] = (xok && s < half_steps && s + shift < ksteps && c < chunks) ? xp[c] : zero_bf16x8();
    }
#pragma unroll
    for (int u = 0; u < U; ++u) acc = mfma_16x16x32(a[u], b[u], acc);
  }

#pragma unroll
  for (int i = 0; i < 4; ++i) red[wave][lane][i] = acc[i];
  if (ep.row_sumsq != nullptr) row_scales_finish(ep, owed, 0, min(M, 8), M, K, scales);
  __syncthreads();
  if (wave != 0) return;
  // lane (r < 8, q < 2) owns weight slots 4q..4q+3 of token r: its own quadrant over the first
  // half of K plus the quadrant of lane (r + 8, q + 2) over the second half
  const bool owner = r < 8 && q < 2;
  const int other = owner ? lane + 8 + 32 : lane;
  float v[4] = {0.f, 0.f, 0.f, 0.f};
  for (int ww = 0; ww < WAVES; ++ww)
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] += red[ww][lane][i] + red[ww][other][i];
  if (ep.row_sumsq != nullptr && r8 < M) {
    const float scale = scales[r8];
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] *= scale;
  }
  const int qq = q & 1;
  qkv_finish_pairs(ep, qkv, head, rotated, row_of(qq * 4) - head * qkv.head_dim, block_in_head * 4, qq == 0, 16,
                   min(r8, M - 1), owner && r8 < M, v);
}

// ---- tiled: more than 16 tokens, and wide products of fewer ---------------------------------
// Four wavefronts in a 2 x 2 arrangement; each owns WM x WN blocks of 32 x 32 (tokens x
// features), so the workgroup tile is (64 WM) tokens x (64 WN) features.  K in slices of 64
// through double-buffered LDS (one barrier per slice).  grid.z cuts K into slices whose
// float32 partial sums go to [slice, M, N].
constexpr int kBK = 64;       // k per LDS slice
constexpr int kLd = kBK + 8;  // padded LDS row, in elements (144 bytes)

template <int WM, int WN, int GM = 2, int GN = 2>
struct TiledShape {
  static constexpr int kThreads = 64 * GM * GN;
  static constexpr int BM = 32 * WM * GM;
  static constexpr int BN = 32 * WN * GN;
  static constexpr int kPieces = (BM + BN) * (kBK / 8) / kThreads;  // 16-byte pieces per thread and slice
  static constexpr int kLds = 2 * (BM + BN) * kLd * 2;              // bytes, two buffers
  // slices of K in flight ahead of the one in LDS: one for the large tiles, two for the small ones
  // (a slice of their work is shorter than a trip to memory; four were no faster, also for the
  // tile of few tokens, which only streams weights)
  static constexpr int kDepth = WM * WN >= 4 || GM * GN > 4 ? 1 : 2;
};

// Workgroup -> (slice, token tile, feature tile).  Consecutive workgroups go to the eight
// XCDs in turn, each with an L2 of its own: the ones that land on one XCD take a contiguous
// run of the tile order, and that order walks groups of eight token tiles feature tile by
// feature tile, so that the workgroups resident on an XCD at one time form a compact block
// of the output and share their operands in its L2.
// `light`: the last token tile holds so few tokens that only the first row of wavefronts has any
// (a prompt portion of 2,048 tokens beside 32 decoding requests: the ninth tile of 256).  Such
// tiles cost a fraction of a full one, and at the end of the order they would all land on the last
// XCD, which would then idle while the others work: they are dealt out evenly instead, behind each
// XCD's share of the full tiles.
struct TileOrder {
  int m_tiles, n_tiles, slices, light;
};
__host__ __device__ inline TileOrder make_tile_order(int m, int n_tiles, int slices, int tile_tokens, int wave_rows) {
  const int m_tiles = (m + tile_tokens - 1) / tile_tokens;
  const int last = m - (m_tiles - 1) * tile_tokens;
  return TileOrder{m_tiles, n_tiles, slices, m_tiles > 1 && last * wave_rows <= tile_tokens ? 1 : 0};
}
__device__ __forceinline__ void place_workgroup(const TileOrder& order, int id, int& slice, int& mt, int& nt) {
  constexpr int kXcds = 8, kGroup = 8;
  const int full_rows = order.m_tiles - order.light;
  const int tiles = full_rows * order.n_tiles;  // full tiles of a slice
  const int full = tiles * order.slices;
  const int total = full + order.light * order.n_tiles * order.slices;
  const int q = total / kXcds, r = total % kXcds;
  const int qf = full / kXcds, rf = full % kXcds;
  const int xcd = id % kXcds, local = id / kXcds;
  const int full_here = qf + (xcd < rf ? 1 : 0);
  if (local >= full_here) {  // one of this XCD's light tiles
    const int before = (xcd * q + min(xcd, r)) - (xcd * qf + min(xcd, rf));
    const int pos = before + local - full_here;
    slice = pos / order.n_tiles;
    nt = pos - slice * order.n_tiles;
    mt = order.m_tiles - 1;
    return;
  }
  int pos = xcd * qf + min(xcd, rf) + local;
  slice = pos / tiles;
  pos -= slice * tiles;
  const int per_group = kGroup * order.n_tiles;
  const int group = pos / per_group;
  const int first = group * kGroup;
  const int size = min(full_rows - first, kGroup);
  const int in_group = pos - group * per_group;
  mt = first + in_group % size;
  nt = in_group / size;
}

// QKV: the fused query/key/value product (see QkvTarget).  The 32-feature blocks of a tile of
// the rotated part (query and key heads) come in pairs: an even block holds 32 dims j of the
// first half of their heads, the odd block after it their partners j + head_dim/2; tiles of the
// value heads (and all tiles, without rotation) hold consecutive rows.
template <int WM, int WN, int DEPTH, int GM = 2, int GN = 2, bool QKV = false, bool ONCE = false>
__global__ __launch_bounds__(64 * GM * GN) void gemm_tiled_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w,
                                                                  GemmEpilogue ep, QkvTarget qkv, TileOrder order, int M,
                                                                  int N, int K) {
  using Shape = TiledShape<WM, WN, GM, GN>;
  constexpr int BM = Shape::BM, BN = Shape::BN, PIECES = Shape::kPieces, THREADS = Shape::kThreads;
  // Two LDS buffers, each BN rows of w and then BM rows of x.  Addressed as offsets from
  // the one shared array so that every access stays an LDS instruction.
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  bf16* const lds = reinterpret_cast<bf16*>(smem);
  constexpr int kBuffer = (BM + BN) * kLd;
  __shared__ float scales[BM];  // of the tile's token rows, when their normalisation is still owed

  const int tid = threadIdx.x;
  const int lane = tid % kWave;
  const int wave = tid / kWave;
  const int wn = wave % GN;
  const int wm = wave / GN;
  const int r32 = lane % 32;
  const int h = lane / 32;
  int slice, mt, nt;
  place_workgroup(order, blockIdx.x, slice, mt, nt);
  const int n0 = nt * BN;
  const int m0 = mt * BM;
  // (tiles of up to 64 tokens hold their rows' partial sums in registers over the loop; larger
  // tiles never see such rows in practice and fetch them the slow way)
  RowScaleLoads<(BM <= 64 ? BM / (GM * GN) : 1), (BM <= 64 ? 2 : 1)> owed;
  if (ep.row_sumsq != nullptr) row_scales_issue(ep, owed, m0, BM, M);
  const int chunks = K / 8;
  const int slices = order.slices;
  const int k_slices = (K + kBK - 1) / kBK;
  const int per = (k_slices + slices - 1) / slices;
  const int s_begin = slice * per;
  const int s_end = min(k_slices, s_begin + per);

  // which weight row stands behind feature slot `slot` of this tile (-1: none)
  bool rotated = false;
  int pair_base = 0, row_base = n0, rot_pairs = 0;
  if constexpr (QKV) {
    rot_pairs = qkv.cos != nullptr ? (qkv.heads + qkv.kv_heads) * (qkv.head_dim / 2) : 0;
    const int rot_tiles = (rot_pairs + BN / 2 - 1) / (BN / 2);
    rotated = nt < rot_tiles;
    pair_base = nt * (BN / 2);
    row_base = 2 * rot_pairs + (nt - rot_tiles) * BN;
  }
  auto row_of = [&](int slot) {
    if constexpr (QKV) {
      if (rotated) {
        const int block = slot / 32;
        const int pair = pair_base + (block / 2) * 32 + slot % 32;
        if (pair >= rot_pairs) return -1;
        const int half = qkv.head_dim / 2;
        const int head = pair / half;
        return head * qkv.head_dim + (pair - head * half) + ((block & 1) ? half : 0);
      }
    }
    return row_base + slot < N ? row_base + slot : -1;
  };

  // global -> register staging through two buffer resources: rows past the end of the
  // matrix, and the tail of K, read as zeros.  The weight resource covers this tile's rows
  // (QKV: the whole matrix, since a tile's rows lie apart).
  const int w_rows = min(BN, N - n0), x_rows = min(BM, M - m0);
  const __amdgpu_buffer_rsrc_t w_buf =
      QKV ? make_buffer(w, static_cast<unsigned>(N) * K * 2u)
          : make_buffer(w + static_cast<int64_t>(n0) * K, static_cast<unsigned>(w_rows) * K * 2u);
  const __amdgpu_buffer_rsrc_t x_buf = make_buffer(x + static_cast<int64_t>(m0) * K, static_cast<unsigned>(x_rows) * K * 2u);
  unsigned piece_off[PIECES];  // byte offset of the piece in slice 0
  int lds_off[PIECES];
  int piece_chunk[PIECES];
#pragma unroll
  for (int it = 0; it < PIECES; ++it) {
    const int idx = tid + it * THREADS;
    const int row = idx / (kBK / 8);
    const int ch = idx % (kBK / 8);
    piece_off[it] = static_cast<unsigned>(row < BN ? row : row - BN) * K * 2u + ch * 16u;
    if constexpr (QKV) {
      if (row < BN) {
        const int weight_row = row_of(row);
        piece_off[it] = weight_row >= 0 ? static_cast<unsigned>(weight_row) * K * 2u + ch * 16u : kOutOfBuffer;
      }
    }
    lds_off[it] = row * kLd + ch * 8;
    piece_chunk[it] = ch;
  }

  f32x16_t acc[WN][WM];
#pragma unroll
  for (int i = 0; i < WN; ++i)
#pragma unroll
    for (int j = 0; j < WM; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // The LDS buffers run one slice ahead of the matrix cores, and DEPTH register sets hold the
  // slices behind it on their way from memory (with a small tile one slice of work is shorter
  // than a trip to memory).  A slice past the end reads zeros through the range check, so the
  // loop bodies need no conditions on it.
  bf16x8_t regs[DEPTH][PIECES];
  auto fetch = [&](int slice, auto& reg) {
    const int left = slice < s_end ? chunks - slice * (kBK / 8) : 0;  // chunks of K from this slice on
#pragma unroll
    for (int it = 0; it < PIECES; ++it) {
      const unsigned off = piece_chunk[it] < left ? piece_off[it] + slice * (kBK * 2u) : kOutOfBuffer;
      // ONCE: one tile of tokens, so every weight byte is read once and need not stay in a cache
      // (the tokens are read by every workgroup and do stay)
      if (ONCE && it * THREADS / (kBK / 8) < BN)
        reg[it] = buffer_load_bf16x8_once(w_buf, off);
      else
        reg[it] = buffer_load_bf16x8(it * THREADS / (kBK / 8) < BN ? w_buf : x_buf, off);
    }
    // the loads are issued here, ahead of the products: the instruction scheduler would
    // otherwise move them down next to the LDS stores that consume them
    __builtin_amdgcn_sched_barrier(0);
  };
  auto stash = [&](int buf, const auto& reg) {
#pragma unroll
    for (int it = 0; it < PIECES; ++it) *reinterpret_cast<bf16x8_t*>(lds + buf * kBuffer + lds_off[it]) = reg[it];
  };
  // A tile at the lower edge of the matrix may have tokens for its first rows of wavefronts only:
  // the others skip the products and only help to stage the operands.
  const bool idle = __builtin_amdgcn_readfirstlane(static_cast<int>(wm * 32 * WM >= x_rows)) != 0;
  auto multiply = [&](int buf) {
    if (idle) return;
    const bf16* wt = lds + buf * kBuffer + (wn * 32 * WN + r32) * kLd + h * 8;
    const bf16* xt = lds + buf * kBuffer + (BN + wm * 32 * WM + r32) * kLd + h * 8;
#pragma unroll
    for (int kk = 0; kk < kBK / 16; ++kk) {
      bf16x8_t a[WN], b[WM];
#pragma unroll
      for (int i = 0; i < WN; ++i) a[i] = load_bf16x8(wt + i * 32 * kLd + kk * 16);
#pragma unroll
      for (int j = 0; j < WM; ++j) b[j] = load_bf16x8(xt + j * 32 * kLd + kk * 16);
#pragma unroll
      for (int i = 0; i < WN; ++i)
#pragma unroll
        for (int j = 0; j < WM; ++j) acc[i][j] = mfma_32x32x16(a[i], b[j], acc[i][j]);
    }
  };

  // set j holds slice s + 1 + j while slice s is multiplied; the set that was stashed is loaded
  // again at once, DEPTH slices further on
#pragma unroll
  for (int j = 0; j < DEPTH; ++j) fetch(s_begin + j, regs[j]);
  stash(0, regs[0]);
  __syncthreads();
  for (int s = s_begin; s < s_end; s += DEPTH) {
#pragma unroll
    for (int j = 0; j < DEPTH; ++j) {
      if (s + j >= s_end) break;
      const int buf = (s + j - s_begin) & 1;
      fetch(s + j + DEPTH, regs[j]);
      multiply(buf);
      stash(buf ^ 1, regs[(j + 1) % DEPTH]);  // slice s + j + 1
      __syncthreads();
    }
  }

  if (ep.row_sumsq != nullptr) {
    row_scales_finish(ep, owed, m0, BM, M, K, scales);
    __syncthreads();
  }
  if constexpr (!QKV) {
#pragma unroll
    for (int i = 0; i < WN; ++i)
#pragma unroll
      for (int j = 0; j < WM; ++j) {
        const int m = m0 + (wm * WM + j) * 32 + r32;
        const float scale = ep.row_sumsq != nullptr ? scales[(wm * WM + j) * 32 + r32] : 1.f;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int n = n0 + (wn * WN + i) * 32 + g * 8 + h * 4;
          const float v[4] = {acc[i][j][g * 4 + 0] * scale, acc[i][j][g * 4 + 1] * scale, acc[i][j][g * 4 + 2] * scale,
                              acc[i][j][g * 4 + 3] * scale};
          finish4(ep, slice, slices, m, n, M, N, v);
        }
      }
  } else {
    // sums -> bias -> bfloat16 (as the unfused kernels hand the product on)
    int row0[WN][4];  // weight row of the lane's first feature in group g of block i
#pragma unroll
    for (int i = 0; i < WN; ++i)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        row0[i][g] = row_of((wn * WN + i) * 32 + g * 8 + h * 4);
#pragma unroll
        for (int j = 0; j < WM; ++j)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float v = acc[i][j][g * 4 + e];
            if (ep.row_sumsq != nullptr) v *= scales[(wm * WM + j) * 32 + r32];
            if (ep.bias != nullptr && row0[i][g] >= 0) v += load_as_f32(ep.bias, row0[i][g] + e, ep.bias_is_f32);
            acc[i][j][g * 4 + e] = to_f32(f32_to_bf16(v));
          }
      }
    // a rotated block needs its partner block: in the same wavefront when it holds two blocks
    // side by side, else in the neighbouring wavefront, through LDS (the tiles are done with)
    float* const exchange = reinterpret_cast<float*>(smem);
    if constexpr (WN == 1) {
      if (rotated) {
        __syncthreads();  // every wavefront has read its last tile
#pragma unroll
        for (int j = 0; j < WM; ++j)
#pragma unroll
          for (int e = 0; e < 16; ++e) exchange[((wave * WM + j) * 16 + e) * kWave + lane] = acc[0][j][e];
        __syncthreads();
      }
    }
#pragma unroll
    for (int i = 0; i < WN; ++i)
#pragma unroll
      for (int j = 0; j < WM; ++j) {
        const int m = m0 + (wm * WM + j) * 32 + r32;
        const int token = min(m, M - 1);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          if (row0[i][g] < 0) continue;
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = acc[i][j][g * 4 + e];
          if (rotated) {
            const int D = qkv.head_dim, half = D / 2;
            const int d = row0[i][g] % D;
            const bool low = d < half;
            const float* cs = qkv.cos + static_cast<int64_t>(token) * half + (low ? d : d - half);
            const float* sn = qkv.sin + static_cast<int64_t>(token) * half + (low ? d : d - half);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              float partner;
              if constexpr (WN == 1)
                partner = exchange[(((wave ^ 1) * WM + j) * 16 + g * 4 + e) * kWave + lane];
              else
                partner = acc[i ^ 1][j][g * 4 + e];
              v[e] = low ? v[e] * cs[e] - partner * sn[e] : v[e] * cs[e] + partner * sn[e];
            }
          }
          if (m >= M) continue;
          u16x4_t packed;
#pragma unroll
          for (int e = 0; e < 4; ++e) packed[e] = f32_to_bf16(v[e]).bits;
          qkv_store4(qkv, row0[i][g], m, packed);
        }
      }
  }
}

// ---- tiled, tiles loaded straight into LDS ---------------------------------------------------------
// The tiles of gemm_tiled_kernel (wavefronts of WM x WN blocks of 32 x 32 in a GM x GN arrangement; square
// ones and, for products whose square tiles would not go round the compute units, 256 tokens x 192 or
// x 160 features) with two changes to what a step of k costs beside its products.
//  * The tiles go from memory into LDS without passing registers.  A lane's 16 bytes land at wavefront
//    base + 16 * lane, so a row of a slice (BKT * 2 bytes) has no padding; instead its 16-byte pieces
//    are stored in the order piece ^ key.  LDS serves sixteen lanes' 16 bytes a cycle from 64 banks
//    (256 bytes: two rows of a 64-wide slice), so the key is (row / 2) % 8 there: the operand reads of
//    sixteen consecutive rows fall on sixteen different places.  (With row % 8 as the key the bank
//    conflict counter showed a third of the kernel's cycles.)
//  * The one barrier of a step stands before its last quarter of products: behind it every wavefront
//    first asks for the next slice's first operands and for the slice NBUF slices on, then multiplies
//    the quarter it kept, so the matrix cores have work while those arrive.
// Measured against the register-staged kernel on one matrix streamed again and again: 7B gate-up at
// 2,048 tokens 592 to 527 us (the vendor library: 584), 7B down in two slices 262 to 247, 32B down in
// three slices 541 to 493, 0.5B gate-up 57 to 51 (the library: 53); on a model's weights, which come
// from memory, 1 to 10 %.  Variants that lost: two quarters kept (KEEP 2: spills a register, no gain);
// slices of 32 in four buffers or of 64 in three (BKT, NBUF; NBUF - 1 slices on their way: 5 to 25 %
// slower from 512 tokens on, up to 16 % faster at 128 to 256, where other tilings are chosen); a 64 x 64
// tile (7 to 15 % slower than the staged kernel, which has two slices on their way, at up to 512 tokens
// of weights that come from memory; equal beyond); eight wavefronts of 128 x 64 or 64 x 128 on the
// 256 x 256 tile (like sixteen of 64 x 64), four of 128 x 128 (7B gate-up 791 us against 571: one wavefront
// per SIMD has nobody to fill its waits); sixteen of 32 x 32 on the 128 x 128 tile (slower than four).

// LDS of a tile of `tokens` x `features` under `waves` wavefronts: a buffer holds the tile's 1 KB runs
// and, where they do not go round the wavefronts, one more for the surplus loads (see kPieces).
constexpr int direct_lds_bytes(int tokens, int features, int waves, int bk, int buffers) {
  const int runs = (tokens + features) * bk * 2 / 1024;
  return buffers * (runs + (runs % waves != 0 ? 1 : 0)) * 1024;
}

template <int KEEP, int WM, int WN, int GM, int GN, int BKT = kBK, int NBUF = 2, bool ONCE = false>
__global__ __launch_bounds__(64 * GM * GN) void gemm_direct_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w,
                                                                  GemmEpilogue ep, TileOrder order, int M, int N, int K) {
  constexpr int BM = 32 * WM * GM, BN = 32 * WN * GN, WAVES = GM * GN;
  constexpr int kRowBytes = BKT * 2;            // 128 or 64
  constexpr int kRowPieces = BKT / 8;           // 16-byte pieces of a row
  constexpr int kRunRows = 1024 / kRowBytes;    // rows of a 1 KB run, the unit a wavefront loads
  constexpr int kBankRows = 256 / kRowBytes;    // rows that LDS serves side by side in one cycle
  constexpr int kRuns = (BM + BN) / kRunRows;   // dealt out to the wavefronts in turn
  constexpr int kWeightRuns = BN / kRunRows;    // the first of them are weight rows, the others token rows
  // Every wavefront issues kPieces loads per slice (the wait counters count instructions); where the
  // runs do not go round, the last wavefronts' surplus loads are out of range and bring zeros to one
  // spare run behind the tile, which nobody reads.
  constexpr int kPieces = (kRuns + WAVES - 1) / WAVES;
  // (loops over a wavefront's runs go to this fixed bound and break: with a bound that depends on the
  // template's parameters the host pass left the kernel uninstantiated, without a message)
  constexpr int kMostPieces = 16;               // at most this many per wavefront
  constexpr int kSteps = BKT / 16;              // products of k = 16 per slice
  static_assert(kPieces <= kMostPieces && BN % 32 == 0 && BM % 32 == 0, "whole runs of weight rows and of token rows");
  static_assert(WAVES % 2 == 0 && KEEP >= 1 && KEEP < kSteps + 1 && NBUF >= 2, "see the swizzle key and the loop");
  constexpr int kInFlight = (NBUF - 2) * kPieces;  // loads of this wavefront that may still be out when a slice is needed
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  constexpr int kBufferBytes = (kRuns + (kRuns % WAVES != 0 ? 1 : 0)) * 1024;
  __shared__ float scales[BM];

  const int tid = threadIdx.x;
  const int lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wn = wave % GN;
  const int wm = wave / GN;
  const int r32 = lane % 32;
  const int h = lane / 32;
  int slice, mt, nt;
  place_workgroup(order, blockIdx.x, slice, mt, nt);
  const int n0 = nt * BN;
  const int m0 = mt * BM;
  RowScaleLoads<1, 1> owed;
  if (ep.row_sumsq != nullptr) row_scales_issue(ep, owed, m0, BM, M);
  const int chunks = K / 8;
  const int slices = order.slices;
  const int k_slices = (K + BKT - 1) / BKT;
  const int per = (k_slices + slices - 1) / slices;
  const int s_begin = slice * per;
  const int s_end = min(k_slices, s_begin + per);

  const int w_rows = min(BN, N - n0), x_rows = min(BM, M - m0);
  const __amdgpu_buffer_rsrc_t w_buf = make_buffer(w + static_cast<int64_t>(n0) * K, static_cast<unsigned>(w_rows) * K * 2u);
  const __amdgpu_buffer_rsrc_t x_buf = make_buffer(x + static_cast<int64_t>(m0) * K, static_cast<unsigned>(x_rows) * K * 2u);
  // piece p of this wavefront fills the run of rows kRunRows * (WAVES p + wave) .. of a buffer (its first
  // half: weights, its second: tokens): lane l brings row + l / kRowPieces, piece (l % kRowPieces) ^ key to
  // slot l % kRowPieces, key = (row / kBankRows) % kRowPieces (the same for every p)
  const int lane_row = lane / kRowPieces;
  const int lane_chunk = (lane % kRowPieces) ^ (((kRunRows / kBankRows) * wave + lane_row / kBankRows) % kRowPieces);
  unsigned piece_off[kMostPieces];
#pragma unroll
  for (int p = 0; p < kMostPieces; ++p) {
    const int run = WAVES * p + wave;
    const int row = kRunRows * run + lane_row;  // rows of the buffer: BN weight rows, then BM token rows
    piece_off[p] = run >= kRuns ? kOutOfBuffer : static_cast<unsigned>(row < BN ? row : row - BN) * K * 2u + lane_chunk * 16u;
  }
  auto fetch = [&](int s, int buf) {
    const int left = s < s_end ? chunks - s * kRowPieces : 0;
    const unsigned off_ok = lane_chunk < left ? 0u : kOutOfBuffer;
#pragma unroll
    for (int p = 0; p < kMostPieces; ++p) {
      if (p >= kPieces) break;
      __attribute__((address_space(3))) void* dst =
          (__attribute__((address_space(3))) void*)(smem + buf * kBufferBytes + min(WAVES * p + wave, kRuns) * 1024);
      const bool weights = (p + 1) * WAVES <= kWeightRuns || (p * WAVES < kWeightRuns && WAVES * p + wave < kWeightRuns);
      const unsigned off = (piece_off[p] + s * (BKT * 2u)) | off_ok;
      if (ONCE && weights) __builtin_amdgcn_raw_ptr_buffer_load_lds(w_buf, dst, 16, off, 0, 0, 2);  // read once: non-temporal
      else __builtin_amdgcn_raw_ptr_buffer_load_lds(weights ? w_buf : x_buf, dst, 16, off, 0, 0, 0);
    }
  };

  f32x16_t acc[WN][WM];
#pragma unroll
  for (int i = 0; i < WN; ++i)
#pragma unroll
    for (int j = 0; j < WM; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  const bool idle = __builtin_amdgcn_readfirstlane(static_cast<int>(wm * 32 * WM >= x_rows)) != 0;
  // operand rows of this lane: weight rows (wn WN + i) * 32 + r32, token rows BN + (wm WM + j) * 32 + r32;
  // piece kk * 2 + h of a row sits in slot (kk * 2 + h) ^ key, and the key is (r32 / kBankRows) % kRowPieces for all of them
  const int swz = (r32 / kBankRows) % kRowPieces;
  const int a_base = (wn * 32 * WN + r32) * kRowBytes;
  const int b_base = (BN + wm * 32 * WM + r32) * kRowBytes;
  struct Fragments {
    bf16x8_t a[WN], b[WM];
  };
  auto read = [&](int buf, int kk) {
    Fragments f;
    const unsigned char* base = smem + buf * kBufferBytes + (((kk * 2 + h) ^ swz) * 16);
#pragma unroll
    for (int i = 0; i < WN; ++i) f.a[i] = load_bf16x8(base + a_base + i * 32 * kRowBytes);
#pragma unroll
    for (int j = 0; j < WM; ++j) f.b[j] = load_bf16x8(base + b_base + j * 32 * kRowBytes);
    return f;
  };
  auto multiply = [&](const Fragments& f) {
#pragma unroll
    for (int i = 0; i < WN; ++i)
#pragma unroll
      for (int j = 0; j < WM; ++j) acc[i][j] = mfma_32x32x16(f.a[i], f.b[j], acc[i][j]);
  };

  // NBUF - 1 slices are on their way or in LDS ahead of the one that is multiplied
#pragma unroll
  for (int b = 0; b < NBUF; ++b) fetch(s_begin + b, b);
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NBUF - 1) * kPieces) : "memory");
  __syncthreads();
  Fragments cur = read(0, 0);
  int buf = 0;
  for (int s = s_begin; s < s_end; ++s) {
    Fragments kept[KEEP];
    if (!idle) {
#pragma unroll
      for (int kk = 0; kk < kSteps - KEEP; ++kk) {
        const Fragments next = read(buf, kk + 1);
        multiply(cur);
        cur = next;
      }
      kept[0] = cur;
#pragma unroll
      for (int e = 1; e < KEEP; ++e) kept[e] = read(buf, kSteps - KEEP + e);
    }
    // the slice after this one has landed (this wavefront's share; the barrier answers for the others),
    // and nobody reads this slice's buffer any more
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(kInFlight) : "memory");
    __syncthreads();
    fetch(s + NBUF, buf);
    const int next_buf = buf + 1 == NBUF ? 0 : buf + 1;
    if (!idle) {
      cur = read(next_buf, 0);
#pragma unroll
      for (int e = 0; e < KEEP; ++e) multiply(kept[e]);  // the part kept for behind the barrier
    }
    buf = next_buf;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may still be on its way into LDS when the workgroup ends

  if (ep.row_sumsq != nullptr) {
    row_scales_finish(ep, owed, m0, BM, M, K, scales);
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < WN; ++i)
#pragma unroll
    for (int j = 0; j < WM; ++j) {
      const int m = m0 + (wm * WM + j) * 32 + r32;
      const float scale = ep.row_sumsq != nullptr ? scales[(wm * WM + j) * 32 + r32] : 1.f;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n = n0 + (wn * WN + i) * 32 + g * 8 + h * 4;
        const float v[4] = {acc[i][j][g * 4 + 0] * scale, acc[i][j][g * 4 + 1] * scale, acc[i][j][g * 4 + 2] * scale,
                            acc[i][j][g * 4 + 3] * scale};
        finish4(ep, slice, slices, m, n, M, N, v);
      }
    }
}

using DirectKernel = void (*)(const bf16*, const bf16*, GemmEpilogue, TileOrder, int, int, int);
// `wave_rows`: rows of wavefronts in the tile (a last token tile that fills only the first is light)
static int launch_direct(DirectKernel kernel, int tile_tokens, int tile_features, int threads, int wave_rows, int lds_bytes,
                         bool& configured, const bf16* xb, const bf16* wb, const GemmEpilogue& ep, int m, int n, int k,
                         int slices, hipStream_t stream) {
  const TileOrder order = make_tile_order(m, (n + tile_features - 1) / tile_features, slices, tile_tokens, wave_rows);
  const int64_t groups = static_cast<int64_t>(order.m_tiles) * order.n_tiles * slices;
  if (groups >= (1ll << 31)) {
    set_error("mlr_gemm_bf16: too many tiles for one launch");
    return -1;
  }
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e != hipSuccess) {
      set_error(std::string("mlr_gemm_bf16: cannot raise the LDS limit: ") + hipGetErrorString(e));
      return -1;
    }
    configured = true;
  }
  hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(groups)), dim3(threads), lds_bytes, stream, xb, wb, ep, order, m, n, k);
  return 0;
}

// ONCE: the tokens fit one tile, so every weight byte is read once; the kernel then loads the
// weights with the non-temporal hint (measured on matrices far larger than the caches, as a
// model's layers are to each other: 7B gate-up at 8 tokens 50.7 to 45.4 us, the output head 191
// to 168 us; a 7B decode step at batch 8 3.76 to 3.53 ms).
template <int WM, int WN, int GM, int GN, bool ONCE>
static int launch_tiled_as(const bf16* xb, const bf16* wb, const GemmEpilogue& ep, const TileOrder& order, int64_t groups,
                           int m, int n, int k, hipStream_t stream) {
  using Shape = TiledShape<WM, WN, GM, GN>;
  constexpr int kDepth = Shape::kDepth;
  static bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_tiled_kernel<WM, WN, kDepth, GM, GN, false, ONCE>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, Shape::kLds);
    if (e != hipSuccess) {
      set_error(std::string("mlr_gemm_bf16: cannot raise the LDS limit: ") + hipGetErrorString(e));
      return -1;
    }
    configured = true;
  }
  gemm_tiled_kernel<WM, WN, kDepth, GM, GN, false, ONCE>
      <<<dim3(static_cast<unsigned>(groups)), Shape::kThreads, Shape::kLds, stream>>>(xb, wb, ep, QkvTarget{}, order, m, n, k);
  return 0;
}

template <int WM, int WN, int GM = 2, int GN = 2>
static int launch_tiled(const bf16* xb, const bf16* wb, const GemmEpilogue& ep, int m, int n, int k, int slices,
                        hipStream_t stream) {
  using Shape = TiledShape<WM, WN, GM, GN>;
  const TileOrder order = make_tile_order(m, (n + Shape::BN - 1) / Shape::BN, slices, Shape::BM, GM);
  const int64_t groups = static_cast<int64_t>(order.m_tiles) * order.n_tiles * slices;
  if (groups >= (1ll << 31)) {
    set_error("mlr_gemm_bf16: too many tiles for one launch");
    return -1;
  }
  if (order.m_tiles == 1) return launch_tiled_as<WM, WN, GM, GN, true>(xb, wb, ep, order, groups, m, n, k, stream);
  return launch_tiled_as<WM, WN, GM, GN, false>(xb, wb, ep, order, groups, m, n, k, stream);
}

// The fused query/key/value product on the tiled kernel: tiles of the rotated part first
// (pairs of 32-dim blocks), then tiles of consecutive rows for the rest.
template <int WM, int WN, int GM = 2, int GN = 2>
static int launch_tiled_qkv(const bf16* xb, const bf16* wb, GemmEpilogue ep, const QkvTarget& qkv, int m, int n, int k,
                            hipStream_t stream) {
  using Shape = TiledShape<WM, WN, GM, GN>;
  constexpr int kDepth = Shape::kDepth;
  static_assert(WN == 1 || WN == 2, "a rotated block finds its partner beside it or in the next wavefront");
  const int rot_pairs = qkv.cos != nullptr ? (qkv.heads + qkv.kv_heads) * (qkv.head_dim / 2) : 0;
  const int rot_tiles = (rot_pairs + Shape::BN / 2 - 1) / (Shape::BN / 2);
  const int rest_tiles = (n - 2 * rot_pairs + Shape::BN - 1) / Shape::BN;
  const TileOrder order = make_tile_order(m, rot_tiles + rest_tiles, 1, Shape::BM, GM);
  const int64_t groups = static_cast<int64_t>(order.m_tiles) * order.n_tiles;
  MLR_REQUIRE(groups < (1ll << 31), "too many tiles for one launch");
  static bool prepared = false;
  if (!prepared) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_tiled_kernel<WM, WN, kDepth, GM, GN, true>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, Shape::kLds);
    if (e != hipSuccess) {
      set_error(std::string("mlr_qkv_rope_write_bf16: cannot raise the LDS limit: ") + hipGetErrorString(e));
      return -1;
    }
    prepared = true;
  }
  gemm_tiled_kernel<WM, WN, kDepth, GM, GN, true>
      <<<dim3(static_cast<unsigned>(groups)), Shape::kThreads, Shape::kLds, stream>>>(xb, wb, ep, qkv, order, m, n, k);
  MLR_LAUNCH_CHECK();
  return 0;
}

// K slices for a skinny product: enough workgroups to keep every compute unit
// streaming, as long as a slice keeps a few MFMA steps.  1 unless `allowed`.
static int choose_slices(int groups, int ksteps, int allowed, int enough = 256) {
  if (allowed <= 1) return 1;
  int slices = 1;
  while (slices < allowed && groups * slices < enough && ksteps / (slices * 2) >= 8) slices *= 2;
  return slices;
}

// Tiles of a shape under the 64 x 64 tiling.
static int tiles_64(int m, int n) { return ((n + 63) / 64) * ((m + 63) / 64); }

// Up to 16 tokens: the LDS-tiled kernel once its 64-feature tiles (times slices) fill seven
// eighths of the compute units, the 16-feature streaming kernel below that.
static bool few_tokens_tiled(int n, int slices) { return ((n + 63) / 64) * slices >= 224; }

// Up to 8 tokens of the fused query/key/value product: workgroups of 8 weight rows instead of
// 16 when that shortens the longest queue of workgroups on a compute unit (256 of them).
static bool half_rows_fill_better(int blocks16) {
  return (2 * blocks16 + 255) / 256 < 2 * ((blocks16 + 255) / 256);
}

// Kernel and number of K slices for more than 64 tokens, when the consumer takes up to
// `max_slices` partial sums: the pair with the smallest estimated time.  The estimate counts
// rounds of workgroups over the 256 compute units.  A workgroup of a tiling spends `fixed` us
// outside its K loop and, per 64-wide step of K, `alone` us when it has its compute unit to itself
// or `busy` us times the workgroups resident beside each other (operand fetch and matrix cores
// do not overlap within a compute unit, so co-resident workgroups queue); steps are faster, down
// to 72 % of that, while only a part of the compute units has work (less traffic into L2).
// Partial sums cost their consumer, a norm that streams at 5.7 TB/s, 4 bytes per slice and
// element instead of 2.  Constants fitted to the measured times of the four products of a layer
// at five model sizes (hidden 896 to 5120) and 96 to 2,048 tokens, with weights that rotate
// through more memory than the caches hold: rms error of the estimate 8 %, the chosen pair within
// 1 % of the best one on average, where rules on tile counts had been 8 % off and up to 76 %.
// (Fitted with the register-staged kernels.  The two larger tilings now run gemm_direct_kernel, whose
// steps measured 4 % shorter on such weights (128 to 2,048 tokens, 0.5B and 7B gate-up and down: 0 to
// 10 % with 128 x 128 tiles, 1 to 7 % with 256 x 256); the 64 x 64 tiling keeps the staged kernel, which
// has two slices of k on their way and streams weights faster at up to some 500 tokens.)
struct GemmPlan {
  int kernel, slices;
};
struct TilingCost {
  int kernel, tile_tokens, tile_features, resident;
  float alone, busy, fixed;
};
// The narrower tiles of 256 tokens (gemm_direct; a step of k costs 7.2 ns per feature of the tile at 256
// features, 7.6 at 192, 8.4 at 160) are there for products whose 256 x 256 tiles leave compute units
// without work or make a round for a few tiles.  Weights from memory, 2,048 tokens: 7B query/key/value
// (4,608 features: 144 tiles, or 232 of 160 features) 92 to 80 us, 32B output projection (160 or 256
// tiles) 130 to 112, 1.5B gate-up 139 to 132; 7B gate-up at 512 tokens 199 to 165.  Over the four
// products of four model sizes at 256 to 4,096 tokens the chosen pairs add up to 0.6 % more than the
// best pairs.  (256 x 224 by fourteen wavefronts was level with 256 x 256 and is not built.)
// 256 x 320 by eight wavefronts of 64 x 160 (ten wavefronts have too few registers each) needs 0.7
// operand reads per product where the square tile needs 1, and makes one round where the others make
// two: 0.5B gate-up (248 tiles) 53 to 49 us, 7B gate-up at 512 tokens 168 to 135, 7B query/key/value at
// 4,096 tokens 159 to 134, 32B down at 4,096 tokens 1,084 to 938; level or behind where the square
// tiles already go round (7B gate-up at 2,048 tokens 533 against 517 on weights from memory).
constexpr TilingCost kTilingCosts[] = {{11, 64, 64, 8, 0.401f, 0.251f, 6.4f},
                                       {23, 128, 128, 2, 0.927f, 0.579f, 6.5f},
                                       {45, 256, 256, 1, 1.09f, 1.84f, 10.5f},
                                       {46, 256, 192, 1, 0.86f, 1.45f, 10.5f},
                                       {47, 256, 160, 1, 0.79f, 1.34f, 10.5f},
                                       {48, 256, 320, 1, 1.39f, 2.35f, 12.f}};
constexpr int kComputeUnits = 256;
static float tiled_time_us(const TilingCost& c, int m, int n, int k, int slices) {
  const int64_t tiles = static_cast<int64_t>((m + c.tile_tokens - 1) / c.tile_tokens) * ((n + c.tile_features - 1) / c.tile_features);
  const int64_t groups = tiles * slices;
  const int ksteps = (k + kBK - 1) / kBK;
  const float per = static_cast<float>((ksteps + slices - 1) / slices);
  auto step = [&](int resident, float fill) {
    return fmaxf(c.alone, resident * c.busy * (0.724f + 0.276f * fill));
  };
  const int64_t capacity = static_cast<int64_t>(kComputeUnits) * c.resident;
  const int64_t full = groups / capacity, rest = groups % capacity;
  float t = full * (c.fixed + per * step(c.resident, 1.f));
  if (rest > 0) {
    const int resident = static_cast<int>((rest + kComputeUnits - 1) / kComputeUnits);
    t += c.fixed + per * step(resident, fminf(1.f, static_cast<float>(rest) / kComputeUnits));
  }
  return t;
}
static GemmPlan plan_many_tokens(int m, int n, int k, int max_slices) {
  GemmPlan best{11, 1};
  float best_time = 0.f;
  const int ksteps = (k + kBK - 1) / kBK;
  for (const TilingCost& c : kTilingCosts)
    for (int slices = 1; slices <= min(max_slices, 4); ++slices) {
      if (slices > 1 && ksteps / slices < 3) break;  // every slice keeps a few steps (0.5B output
                                                     // projection at 128 tokens, 14 steps: whole 8.0 us, in 4 slices 5.4)
      float t = tiled_time_us(c, m, n, k, slices);
      if (slices > 1) t += (4.f * slices - 2.f) * m * n / 5.7e6f;
      if (best_time == 0.f || t < best_time) best = {c.kernel, slices}, best_time = t;
    }
  return best;
}

// The kernel for a shape: 16 = gemm_skinny_split, 11 / 22 / 44 = gemm_tiled with 64 x 64,
// 128 x 128 (four wavefronts each) and 256 x 256 (sixteen wavefronts) tiles, 23 / 45 = gemm_direct
// with the two larger ones, 46 / 47 / 48 = gemm_direct with tiles of 256 tokens x 192 features (twelve
// wavefronts of 64 x 64), x 160 features (ten of 128 x 32) and x 320 features (eight of 64 x 160), 14 = gemm_tiled
// with tiles of 32 tokens x 64 features (two wavefronts): for up to 32 tokens it stages half the
// rows of the 64 x 64 tile and streams weights 5 to 15 % faster, 62 to 68 = gemm_direct with tiles of
// 64 tokens x 64, 96, ... 256 features for up to 64 tokens (see choose_few_token_tiles).
// A small matrix (an output projection of a narrow model) at 17 to 64 tokens: the tiled kernels have
// too few tiles of it to keep the compute units busy, the row-splitting kernel with its 16 features a
// workgroup has four times as many workgroups (0.5B output projection with the norm behind it, in a
// replayed graph: 32 tokens 9.0 us tiled in 2 slices, 6.4 row-splitting in 4; 64 tokens 9.4 and 7.3).
// Larger matrices read the tokens too often that way (0.5B gate-up at 64 tokens: 10 us tiled, 16).
static bool small_matrix(int n, int k) { return static_cast<int64_t>(n) * k * 2 <= (4ll << 20); }

// Up to 64 tokens through tiles: such a product streams its weights once and is done when the busiest
// compute unit has streamed its share, so what counts is how the tiles go round the 256 units and what
// a unit takes in.  Fitted to replayed graphs over weights that come from memory (the five products of
// seven model sizes at 8 to 64 tokens, 1,500 timings, rms error 9 %): a unit takes in 44 GB/s through the
// tiles of gemm_direct and 37 through the register-staged ones, tokens included (a tile of 64 tokens x
// 64 features reads as many token bytes as weight bytes, one of 256 features a fifth of that), all
// units together 6.1 TB/s of weights (23.8 GB/s each), a launch costs 3.7 us and a round of tiles that
// have their unit to themselves 2 us until their first bytes arrive (0.8 where two share a unit).
// The tiles of 64 tokens x 64 ... 256 features of gemm_direct (a wavefront per 32 x 32 block; as many
// slices of k in LDS as fit, 3 to 6, where the staged kernels have 2 on their way) are there so that some
// width makes one round that fills the units: 7B gate-up (37,888 rows) at 64 tokens 67 us in staged
// 64-feature tiles, 48.8 in 237 tiles of 160; 32B gate-up 130 to 92 (247 tiles of 224; at 8 tokens 101
// to 92, 6.2 TB/s); cut along k in 8: 7B down 31.8 to 28.4, 32B down 69.6 to 50.1; the 7B output head
// 244 to 212; 0.5B gate-up 10.3 to 8.9.  Over the sweep the chosen tilings add up to 1.4 % more than the
// best ones, and to 7 % less than the staged 64-feature tiles everywhere.
struct FewTokenTiling {
  int kernel, tokens, features;
  bool direct;
  float round_us;  // per round of tiles
};
constexpr FewTokenTiling kFewTokenTilings[] = {
    {62, 64, 64, true, 0.77f},  {63, 64, 96, true, 2.f},  {64, 64, 128, true, 2.f}, {65, 64, 160, true, 2.f}, {66, 64, 192, true, 2.f},
    {67, 64, 224, true, 2.f},   {68, 64, 256, true, 2.f}, {14, 32, 64, false, 0.f}, {11, 64, 64, false, 0.f}};
static float few_token_time_us(const FewTokenTiling& t, int m, int n, int k, int slices) {
  constexpr float kDirectIntake = 44.f, kStagedIntake = 37.f, kUnitShare = 23.8f, kLaunch = 3.7f;  // GB/s, GB/s, GB/s, us
  // more tokens than a tile: every tile of tokens streams the weights again, but only the first from memory
  const int token_tiles = (m + t.tokens - 1) / t.tokens;
  const int64_t groups = static_cast<int64_t>((n + t.features - 1) / t.features) * slices * token_tiles;
  const float tile_kb = static_cast<float>(t.features) * ((k + slices - 1) / slices) * 2.f / 1e3f;
  const float unit = (t.direct ? kDirectIntake : kStagedIntake) * t.features / (t.features + min(m, t.tokens));
  const float share = kUnitShare * token_tiles;
  const int64_t full = groups / kComputeUnits, rest = groups % kComputeUnits;
  float time = kLaunch + full * (tile_kb / fminf(unit, share) + t.round_us);
  if (rest > 0) time += tile_kb / fminf(unit, share * kComputeUnits / rest) + t.round_us;
  return time;
}
static int choose_few_token_tiles(int m, int n, int k, int slices) {
  int best = 0;
  float best_time = 0.f;
  // narrow tiles first (at a tie the one that fills more units), the staged ones last and only when
  // clearly ahead: where the estimate has them level the direct tile measured 10 to 20 % faster
  for (const FewTokenTiling& t : kFewTokenTilings) {
    if ((t.kernel == 14 && m > t.tokens) || (t.kernel == 11 && m <= 32)) continue;
    const float time = few_token_time_us(t, m, n, k, slices);
    if (best == 0 || time < (t.direct ? 0.99f : 0.97f) * best_time) best = t.kernel, best_time = time;
  }
  return best;
}

static int choose_kernel(int m, int n, int k, int slices) {
  if (m <= 16 && !few_tokens_tiled(n, slices)) return 16;
  if (m <= 64 && small_matrix(n, k)) return 16;
  if (m <= 64) return choose_few_token_tiles(m, n, k, slices);
  const GemmPlan plan = plan_many_tokens(m, n, k, slices);
  const int kernel = plan.slices == slices ? plan.kernel : 11;
  // up to 256 tokens in tiles of 64: the same choice of widths as for one tile of tokens (7B down at 128
  // tokens in 4 slices: 50.6 us staged, 41.8 in tiles of 128 features; 32B down at 192 tokens 131 and
  // 106).  Not for small matrices: the staged tiles, four workgroups to a compute unit, share the weights
  // of neighbouring token tiles (1.5B query/key/value, 6 MB, at 192 tokens: 7.4 us against 9.1).
  if (kernel == 11 && m <= 256 && static_cast<int64_t>(n) * k * 2 >= (16ll << 20)) return choose_few_token_tiles(m, n, k, slices);
  return kernel;
}

static int gemm_bf16(const bf16* xb, const bf16* wb, const GemmEpilogue& ep, int m, int n, int k, int slices,
                     int kernel, hipStream_t stream) {
  switch (kernel) {
    case 16: {
      if (m > 64) {
        set_error("mlr_gemm_bf16: the streaming kernel takes up to 64 tokens");
        return -1;
      }
      dim3 grid((n + 15) / 16, slices);
      if (m <= 16) gemm_skinny_split_kernel<4, false, 1><<<grid, 256, 0, stream>>>(xb, wb, ep, QkvTarget{}, m, n, k);
      else if (m <= 32) gemm_skinny_split_kernel<4, false, 2><<<grid, 256, 0, stream>>>(xb, wb, ep, QkvTarget{}, m, n, k);
      else gemm_skinny_split_kernel<4, false, 4><<<grid, 256, 0, stream>>>(xb, wb, ep, QkvTarget{}, m, n, k);
      return 0;
    }
    case 11: return launch_tiled<1, 1>(xb, wb, ep, m, n, k, slices, stream);
    case 14: return launch_tiled<1, 1, 1, 2>(xb, wb, ep, m, n, k, slices, stream);  // 32 tokens x 64 features, two wavefronts
    case 22: return launch_tiled<2, 2>(xb, wb, ep, m, n, k, slices, stream);
    case 44: return launch_tiled<2, 2, 4, 4>(xb, wb, ep, m, n, k, slices, stream);
    case 45: {
      static bool configured = false;
      return launch_direct(gemm_direct_kernel<1, 2, 2, 4, 4>, 256, 256, 1024, 4, direct_lds_bytes(256, 256, 16, 64, 2), configured,
                           xb, wb, ep, m, n, k, slices, stream);
    }
    // 64 tokens x 64 to 256 features, a wavefront per 32 x 32 block, as many slices of k in LDS as fit
    case 62: {
      static bool configured = false;
      return launch_direct(gemm_direct_kernel<1, 1, 1, 2, 2, 64, 4, true>, 64, 64, 256, 2, direct_lds_bytes(64, 64, 4, 64, 4),
                           configured, xb, wb, ep, m, n, k, slices, stream);
    }
    case 63: {
      static bool configured = false;
      return launch_direct(gemm_direct_kernel<1, 1, 1, 2, 3, 64, 6, true>, 64, 96, 384, 2, direct_lds_bytes(64, 96, 6, 64, 6),
                           configured, xb, wb, ep, m, n, k, slices, stream);
    }
    case 64: {
      static bool configured = false;
      return launch_direct(gemm_direct_kernel<1, 1, 1, 2, 4, 64, 6, true>, 64, 128, 512, 2, direct_lds_bytes(64, 128, 8, 64, 6),
                           configured, xb, wb, ep, m, n, k, slices, stream);
    }
    case 65: {
      static bool configured = false;
      return launch_direct(gemm_direct_kernel<1, 1, 1, 2, 5, 64, 5, true>, 64, 160, 640, 2, direct_lds_bytes(64, 160, 10, 64, 5),
                           configured, xb, wb, ep, m, n, k, slices, stream);
    }
    case 66: {
      static bool configured = false;
      return launch_direct(gemm_direct_kernel<1, 1, 1, 2, 6, 64, 4, true>, 64, 192, 768, 2, direct_lds_bytes(64, 192, 12, 64, 4),
                           configured, xb, wb, ep, m, n, k, slices, stream);
    }
    case 67: {
      static bool configured = false;
      return launch_direct(gemm_direct_kernel<1, 1, 1, 2, 7, 64, 3, true>, 64, 224, 896, 2, direct_lds_bytes(64, 224, 14, 64, 3),
                           configured, xb, wb, ep, m, n, k, slices, stream);
    }
    case 68: {
      static bool configured = false;
      return launch_direct(gemm_direct_kernel<1, 1, 1, 2, 8, 64, 3, true>, 64, 256, 1024, 2, direct_lds_bytes(64, 256, 16, 64, 3),
                           configured, xb, wb, ep, m, n, k, slices, stream);
    }
    case 48: {  // 256 tokens x 320 features, eight wavefronts of 64 x 160
      static bool configured = false;
      return launch_direct(gemm_direct_kernel<1, 2, 5, 4, 2>, 256, 320, 512, 4, direct_lds_bytes(256, 320, 8, 64, 2), configured,
                           xb, wb, ep, m, n, k, slices, stream);
    }
    case 46: {  // 256 tokens x 192 features, twelve wavefronts of 64 x 64
      static bool configured = false;
      return launch_direct(gemm_direct_kernel<1, 2, 2, 4, 3>, 256, 192, 768, 4, direct_lds_bytes(256, 192, 12, 64, 2), configured,
                           xb, wb, ep, m, n, k, slices, stream);
    }
    case 47: {  // 256 tokens x 160 features, ten wavefronts of 128 x 32
      static bool configured = false;
      return launch_direct(gemm_direct_kernel<1, 4, 1, 2, 5>, 256, 160, 640, 2, direct_lds_bytes(256, 160, 10, 64, 2), configured,
                           xb, wb, ep, m, n, k, slices, stream);
    }
    case 23: {
      static bool configured = false;
      return launch_direct(gemm_direct_kernel<1, 2, 2, 2, 2>, 128, 128, 256, 2, direct_lds_bytes(128, 128, 4, 64, 2), configured,
                           xb, wb, ep, m, n, k, slices, stream);
    }
    default: set_error("mlr_gemm_bf16: kernel must be 0 (chosen by shape), 16, 14, 11, 22, 23, 44 to 48 or 62 to 68"); return -1;
  }
}

}  // namespace mlr

using namespace mlr;

extern "C" {

// How many K slices mlr_gemm_bf16 would use for this shape when the caller can take
// partial sums (at most `max_slices`); 1 means it writes the finished product.
int mlr_gemm_bf16_slices(int m, int n, int k, int max_slices) {
  if (k % 8 != 0) return 1;
  if (m > 64) return plan_many_tokens(m, n, k, max_slices).slices;
  if (m <= 16) {
    // Measured with the norm kernel that adds the slices up (its cost grows with their number):
    // a weight of 64 MB or more streams fastest through the LDS-tiled kernel cut into 8 slices;
    // smaller ones through the 16-feature kernel, cut until the compute units are filled and at
    // least once per 2,560 of k (up to 4 times).
    const int64_t bytes = static_cast<int64_t>(n) * k * 2;
    if (bytes >= (64ll << 20) && max_slices >= 8 && k >= 8 * 256 && few_tokens_tiled(n, 8)) return 8;
    // from 20 MB on, the LDS-tiled kernel cut into 4 once that fills the compute units, into 8 where
    // 4 would not fill them twice (7B output projection at 8 tokens: 10.1 us in 4 slices, 8.4 in 8)
    if (bytes >= (20ll << 20) && max_slices >= 8 && k >= 8 * 256 && few_tokens_tiled(n, 4) && !few_tokens_tiled(n, 2))
      return 8;
    if (bytes >= (20ll << 20) && max_slices >= 4 && k >= 4 * 256 && few_tokens_tiled(n, 4)) return 4;
    // the 16-feature kernel: two workgroups per compute unit before the cutting stops (1.5B down at 8
    // tokens: 384 workgroups 11.8 us, 768 workgroups 9.8 us), at most 8 slices for the norm to add up
    const int by_fill = choose_slices((n + 15) / 16, (k / 8 + 3) / 4, min(max_slices, 8), 512);
    return max(by_fill, min(min(4, max_slices), k / 2560));
  }
  // 17 to 64 tokens of a small matrix: the row-splitting kernel (see choose_kernel) cut into 4 where
  // every slice keeps a few steps of k
  if (small_matrix(n, k)) return (k / 8 + 3) / 4 >= 16 ? min(4, max_slices) : 1;
  // 17 to 64 tokens: the small tiles keep few bytes in flight each, so two workgroups per compute
  // unit before the cutting stops (32B down at 32 tokens: 320 workgroups 65 us, 640 workgroups 56 us)
  return choose_slices(tiles_64(m, n), (k / 8 + 3) / 4, min(max_slices, 8), 512);
}

int mlr_gemm_bf16_kernel(int m, int n, int k, int slices) { return choose_kernel(m, n, k, slices); }

// y = x w^T (+ bias) in bfloat16 on the matrix cores; see mlr_gemm_simple for the
// argument meanings.  Requires k % 8 == 0 and 16-byte aligned x and w.  With
// `swiglu` the rows of w are (gate, gate, up, up) groups, there is no bias, n is
// a multiple of 4 and y is [m, n / 2].  With slices > 1 (the value of
// mlr_gemm_bf16_slices; not with swiglu) y is float32 [slices, m, n]: partial sums
// over slices of k, the bias in slice 0, for the consumer to add up.
int mlr_gemm_bf16(const void* x, const void* w, const void* bias, int bias_is_f32, void* y, int out_is_f32,
                  int swiglu, int slices, int kernel, int m, int n, int k, const float* row_sumsq, int sumsq_parts,
                  float norm_eps, hipStream_t stream) {
  MLR_REQUIRE(x && w && y, "null pointer");
  MLR_REQUIRE(m > 0 && n > 0 && k > 0, "sizes must be > 0");
  MLR_REQUIRE(k % 8 == 0, "k must be a multiple of 8");
  MLR_REQUIRE(k <= (1 << 20), "k must not exceed 2^20 (32-bit byte offsets inside a tile)");
  MLR_REQUIRE(!swiglu || (n % 4 == 0 && bias == nullptr), "swiglu needs n % 4 == 0 and no bias");
  MLR_REQUIRE(slices >= 1 && slices <= 64, "slices must be within 1..64");
  MLR_REQUIRE(slices == 1 || (!swiglu && out_is_f32), "partial sums are float32, without SwiGLU");
  MLR_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0,
              "x and w must be 16-byte aligned");
  MLR_REQUIRE(row_sumsq == nullptr || (sumsq_parts > 0 && sumsq_parts <= (1 << 16) && norm_eps >= 0.f),
              "sums of squares come with their number per row (1..65536) and an eps >= 0");
  GemmEpilogue ep{bias, bias_is_f32, y, out_is_f32, swiglu, row_sumsq, sumsq_parts, norm_eps};
  if (kernel == 0) kernel = choose_kernel(m, n, k, slices);
  if (gemm_bf16(static_cast<const bf16*>(x), static_cast<const bf16*>(w), ep, m, n, k, slices, kernel, stream) != 0)
    return -1;
  MLR_LAUNCH_CHECK();
  return 0;
}

// The query/key/value product with everything that follows it before attention: bias, rotation of the query and key heads (cos, sin: [m, head_dim / 2] float32,
// or null for none), queries to q_out [m, heads * head_dim], keys and values into the slots
// of their pages (`write` 0: another layer owns the pages).  w is [(heads + 2 kv_heads) *
// head_dim, k]; head_dim a multiple of 16, k of 8.  kernel: 0 chooses (the streaming kernel up
// to 64 tokens unless it would read x too often, else a tiled one), or 16, 11, 22, 44.
int mlr_qkv_rope_write_bf16(const void* x, const void* w, const void* bias, int bias_is_f32, const float* cos,
                            const float* sin, const int* slots, void* key_pages, void* value_pages, void* q_out,
                            int m, int k, int heads, int kv_heads, int head_dim, int block_size, int num_pages,
                            int write, int kernel, const float* row_sumsq, int sumsq_parts, float norm_eps,
                            hipStream_t stream) {
  MLR_REQUIRE(x && w && q_out, "null pointer");
  MLR_REQUIRE(row_sumsq == nullptr || (sumsq_parts > 0 && sumsq_parts <= (1 << 16) && norm_eps >= 0.f),
              "sums of squares come with their number per row (1..65536) and an eps >= 0");
  MLR_REQUIRE(m > 0, "no tokens");
  MLR_REQUIRE(k > 0 && k % 8 == 0 && k <= (1 << 20), "k must be a positive multiple of 8, at most 2^20");
  MLR_REQUIRE(heads > 0 && kv_heads > 0 && head_dim >= 16 && head_dim % 16 == 0, "head_dim must be a multiple of 16");
  MLR_REQUIRE((cos == nullptr) == (sin == nullptr), "cos and sin come together");
  MLR_REQUIRE(!write || (slots && key_pages && value_pages && block_size > 0 && num_pages > 0),
              "a cache write needs slots, pages and their sizes");
  MLR_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(q_out) % 8 == 0 && reinterpret_cast<uintptr_t>(key_pages) % 8 == 0 &&
                  reinterpret_cast<uintptr_t>(cos) % 16 == 0 && reinterpret_cast<uintptr_t>(sin) % 16 == 0,
              "operands must be 16-byte aligned");
  const int64_t n = static_cast<int64_t>(heads + 2 * kv_heads) * head_dim;
  MLR_REQUIRE(n / 16 < (1ll << 31), "too many rows for one launch");
  GemmEpilogue ep{bias, bias_is_f32, nullptr, 0, 0, row_sumsq, sumsq_parts, norm_eps};
  QkvTarget target{cos, sin, write ? slots : nullptr, static_cast<bf16*>(key_pages), static_cast<bf16*>(value_pages),
                   static_cast<bf16*>(q_out), heads, kv_heads, head_dim, block_size, num_pages};
  const bf16* xb = static_cast<const bf16*>(x);
  const bf16* wb = static_cast<const bf16*>(w);
  if (kernel == 0) {
    // Beyond 64 tokens the 64 x 64 tiles: with this epilogue (rotation, scattered cache stores) the
    // larger tiles are slower than they are for the plain product, and where those would pay the
    // caller does better with the plain product and the rotation kernel behind it.
    kernel = m <= 64 ? 16 : 11;
    if (kernel == 16 && m > 16 && (n / 16) * m * k * 2 > (32ll << 20)) kernel = 11;  // too many passes over x
  }
  if (kernel == 8) {
    MLR_REQUIRE(m <= 8, "the 8-row kernel takes 1..8 tokens");
    gemm_skinny_qkv8_kernel<4><<<dim3(static_cast<unsigned>(n / 8)), 256, 0, stream>>>(xb, wb, ep, target, m, static_cast<int>(n), k);
    MLR_LAUNCH_CHECK();
    return 0;
  }
  if (kernel == 16) {
    MLR_REQUIRE(m <= 64, "the row-splitting kernel takes 1..64 tokens");
    const dim3 grid(static_cast<unsigned>(n / 16));
    if (m <= 8 && half_rows_fill_better(static_cast<int>(n / 16)))
      gemm_skinny_qkv8_kernel<4><<<dim3(static_cast<unsigned>(n / 8)), 256, 0, stream>>>(xb, wb, ep, target, m, static_cast<int>(n), k);
    else if (m <= 16)
      gemm_skinny_split_kernel<4, true, 1><<<grid, 256, 0, stream>>>(xb, wb, ep, target, m, static_cast<int>(n), k);
    else if (n * k * 2 <= (8ll << 20))
      // a small matrix: a workgroup per slab of 16 tokens reads a quarter of the tokens and the weights
      // again from L2, where one workgroup for all slabs is held up by the tokens it takes in (0.5B at
      // 64 tokens 8.4 to 6.8 us, at 48 7.7 to 5.2; 1.5B at 64 12.0 to 10.1; a 10 MB matrix: 14.6 to 16.1).
      // The same sums in the same order either way.
      gemm_skinny_split_kernel<4, true, 1><<<dim3(grid.x, 1, (m + 15) / 16), 256, 0, stream>>>(xb, wb, ep, target, m, static_cast<int>(n), k);
    else if (m <= 32)
      gemm_skinny_split_kernel<4, true, 2><<<grid, 256, 0, stream>>>(xb, wb, ep, target, m, static_cast<int>(n), k);
    else
      gemm_skinny_split_kernel<4, true, 4><<<grid, 256, 0, stream>>>(xb, wb, ep, target, m, static_cast<int>(n), k);
    MLR_LAUNCH_CHECK();
    return 0;
  }
  // the tiled kernels address the whole weight matrix, and one token's rows of x, with 31-bit offsets
  MLR_REQUIRE(n * k * 2 < (1ll << 31), "the weight matrix is too large for the tiled fused product");
  switch (kernel) {
    case 11: return launch_tiled_qkv<1, 1>(xb, wb, ep, target, m, static_cast<int>(n), k, stream);
    case 22: return launch_tiled_qkv<2, 2>(xb, wb, ep, target, m, static_cast<int>(n), k, stream);
    case 44: return launch_tiled_qkv<2, 2, 4, 4>(xb, wb, ep, target, m, static_cast<int>(n), k, stream);
    default: MLR_REQUIRE(false, "unknown kernel");
  }
  return 0;
}

}  // extern "C"
