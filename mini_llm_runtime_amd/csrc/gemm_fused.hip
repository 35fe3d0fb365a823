// Matrix products of a few tokens (up to 16: decoding at small batch) whose activations
// are made by the kernel itself instead of being read from memory.
//
// A decode step of a small model is a chain of short dependent kernels, and each link
// costs a few microseconds whatever it computes.  Two links per layer go away when the
// product that follows a norm computes the norm itself, and one more when the output
// product of the attention merges the split-KV partitions itself:
//  * norm prologue: every workgroup adds the not-yet-added delta (a bfloat16 tensor, or
//    float32 partial sums of a K-sliced product, in slice order) to the float32 residual
//    stream, takes the RMSNorm of the sum (src/mini_llm_runtime/qwen_model_runner.py:22-26,
//    statistics in 32-bit) and keeps the normed rows as bfloat16 in LDS; the workgroups whose
//    index matches a row also write that row of the updated stream to `x_out` (a buffer of
//    its own: other workgroups still read `x_in`).  The few rows are re-read by every
//    workgroup, from L2.
//  * merge prologue: every workgroup merges the partitions of the attention of its slice
//    of K (m = max m_j, O = sum w_j a_j / sum w_j l_j, w_j = exp2(m_j - m),
//    csrc/paged_attention_split_cuda.cu:66-88 of the reference) into LDS.
// Then the weights stream exactly as in gemm_skinny_split: a workgroup owns 16 * NT output
// features (and one slice of K), its four wavefronts split K, range-checked buffer loads
// keep two batches of eight 16-byte loads per lane in flight, the first of them issued
// before the prologue, and the wavefronts' sums meet in LDS.  Epilogues are those of
// gemm_mfma.hip: bias, SwiGLU, partial sums, or the query/key/value product's rotation and
// cache write.
#include "api.h"
#include "common.h"
#include "gemm_epilogue.h"
#include "mfma.h"

namespace mlr {

typedef float f32x4 __attribute__((ext_vector_type(4)));

struct NormPrologue {
  const float* x_in;     // [M, K] residual stream
  float* x_out;          // [M, K] the stream with the delta added; null when there is no delta
  const bf16* delta;     // [M, K] or null
  const float* partial;  // [slices, M, K] or null
  int slices;
  const void* weight;  // [K]
  int weight_is_f32;
  float eps;
};

struct MergePrologue {
  const float* partial;     // [M, heads, all_splits, head_dim + 2]: numerator, max, denominator
  const int* context_lens;  // [M]
  int heads, head_dim, window, part, all_splits;
  unsigned bytes;  // of `partial`
};

constexpr int kFusedWaves = 4;
// k-steps per batch of loads and wavefront: eight 16-byte loads of a lane per batch and row block
constexpr int fused_depth(int row_blocks) { return row_blocks == 1 ? 8 : 4; }

// ---- norm prologue ------------------------------------------------------------------------
// A wavefront takes one row (so the kernels take up to four tokens).  Its work comes in two
// halves so that the caller can put other loads between them: `issue` sends every load of the
// row (the stream, the delta, up to a batch of partial sums, the norm's weights), `finish` adds
// up, takes the statistics and writes the normed row to LDS: one trip to L2.  Every load is a
// range-checked buffer load without a condition around it: what is absent (no delta, fewer
// partial sums than the batch holds) reads zeros from an empty or missed range.
//
// Every workgroup reads the same few rows; were they all to read them in the same order, the
// whole chip would ask the same few L2 channels for the same lines at the same moment.  So a
// workgroup starts at a column of its own and wraps around.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ f32x4 buffer_load_f32x4(__amdgpu_buffer_rsrc_t rsrc, unsigned byte_offset) {
  return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, byte_offset, 0, 0));
}
__device__ __forceinline__ u32x2 buffer_load_u32x2(__amdgpu_buffer_rsrc_t rsrc, unsigned byte_offset) {
  return __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(rsrc, byte_offset, 0, 0));
}
__device__ __forceinline__ float bf16_low(uint32_t pair) { return __builtin_bit_cast(float, pair << 16); }
__device__ __forceinline__ float bf16_high(uint32_t pair) { return __builtin_bit_cast(float, pair & 0xffff0000u); }

// SB: partial sums per trip.  Their registers decide how many workgroups share a compute unit:
// a product of few workgroups (query/key/value) takes many per trip, a wide one few.
template <int VPT, int SB>
struct NormRow {
  static constexpr int kSliceBatch = SB;
  unsigned at[VPT];  // byte offset of this lane's columns within a float32 row, out of range past the end
  f32x4 v[VPT];
  f32x4 p[VPT][kSliceBatch];
  u32x2 d[VPT];
  f32x4 wf[VPT];
  u32x2 wh[VPT];
};

template <int VPT, int SB>
__device__ __forceinline__ void norm_issue(const NormPrologue& np, NormRow<VPT, SB>& t, int row, int M, int K) {
  const int lane = threadIdx.x % kWave;
  const int quads = K / 4;
  const int rot = static_cast<int>((static_cast<unsigned>(blockIdx.x + blockIdx.y) * 40503u) % static_cast<unsigned>(quads));
  const unsigned row_bytes = static_cast<unsigned>(K) * 4u;
  const unsigned slab = static_cast<unsigned>(M) * row_bytes;
  const __amdgpu_buffer_rsrc_t x_buf = make_buffer(np.x_in + static_cast<int64_t>(row) * K, row_bytes);
  const __amdgpu_buffer_rsrc_t d_buf = make_buffer(np.delta + static_cast<int64_t>(row) * K, np.delta ? row_bytes / 2 : 0u);
  const __amdgpu_buffer_rsrc_t p_buf =
      make_buffer(np.partial + static_cast<int64_t>(row) * K, np.partial ? static_cast<unsigned>(np.slices - 1) * slab + row_bytes : 0u);
  const __amdgpu_buffer_rsrc_t wf_buf = make_buffer(np.weight, np.weight_is_f32 ? row_bytes : 0u);
  const __amdgpu_buffer_rsrc_t wh_buf = make_buffer(np.weight, np.weight_is_f32 ? 0u : row_bytes / 2);
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int idx = lane + kWave * j;
    const int i = idx + rot;
    t.at[j] = idx < quads ? static_cast<unsigned>(i >= quads ? i - quads : i) * 16u : kOutOfBuffer;
  }
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    t.v[j] = buffer_load_f32x4(x_buf, t.at[j]);
    t.d[j] = buffer_load_u32x2(d_buf, t.at[j] / 2);
#pragma unroll
    for (int u = 0; u < SB; ++u) t.p[j][u] = buffer_load_f32x4(p_buf, t.at[j] + static_cast<unsigned>(u) * slab);
    t.wf[j] = buffer_load_f32x4(wf_buf, t.at[j]);
    t.wh[j] = buffer_load_u32x2(wh_buf, t.at[j] / 2);
  }
  __builtin_amdgcn_sched_barrier(0);
}

template <int VPT, int SB>
__device__ __forceinline__ void norm_finish(const NormPrologue& np, NormRow<VPT, SB>& t, bf16* hb, int ldk, int row, int M,
                                            int K, int kcols) {
  const int lane = threadIdx.x % kWave;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    t.v[j][0] += bf16_low(t.d[j][0]);
    t.v[j][1] += bf16_high(t.d[j][0]);
    t.v[j][2] += bf16_low(t.d[j][1]);
    t.v[j][3] += bf16_high(t.d[j][1]);
#pragma unroll
    for (int u = 0; u < SB; ++u)
#pragma unroll
      for (int e = 0; e < 4; ++e) t.v[j][e] += t.p[j][u][e];  // in slice order; absent slices are zeros
  }
  if (np.slices > SB) {  // more partial sums than the first batch held
    const unsigned row_bytes = static_cast<unsigned>(K) * 4u;
    const unsigned slab = static_cast<unsigned>(M) * row_bytes;
    const __amdgpu_buffer_rsrc_t p_buf =
        make_buffer(np.partial + static_cast<int64_t>(row) * K, static_cast<unsigned>(np.slices - 1) * slab + row_bytes);
    for (int s0 = SB; s0 < np.slices; s0 += SB) {
#pragma unroll
      for (int j = 0; j < VPT; ++j)
#pragma unroll
        for (int u = 0; u < SB; ++u) t.p[j][u] = buffer_load_f32x4(p_buf, t.at[j] + static_cast<unsigned>(s0 + u) * slab);
#pragma unroll
      for (int j = 0; j < VPT; ++j)
#pragma unroll
        for (int u = 0; u < SB; ++u)
#pragma unroll
          for (int e = 0; e < 4; ++e) t.v[j][e] += t.p[j][u][e];
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < VPT; ++j)
#pragma unroll
    for (int e = 0; e < 4; ++e) ss += t.v[j][e] * t.v[j][e];  // columns past the end read zeros
  const float total = wave_sum(ss);
  const float inv = 1.0f / sqrtf(total / static_cast<float>(K) + np.eps);
  const bool writes_stream = np.x_out != nullptr && row % static_cast<int>(gridDim.x) == static_cast<int>(blockIdx.x) &&
                             blockIdx.y == 0;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    if (t.at[j] == kOutOfBuffer) continue;
    const unsigned col = t.at[j] / 4;
    if (writes_stream) *reinterpret_cast<f32x4*>(np.x_out + static_cast<int64_t>(row) * K + col) = t.v[j];
    // one of the two weight loads found an empty buffer and returned zeros
    const float w0 = t.wf[j][0] + bf16_low(t.wh[j][0]), w1 = t.wf[j][1] + bf16_high(t.wh[j][0]);
    const float w2 = t.wf[j][2] + bf16_low(t.wh[j][1]), w3 = t.wf[j][3] + bf16_high(t.wh[j][1]);
    const u32x2 packed = {pack_bf16x2(w0 * (t.v[j][0] * inv), w1 * (t.v[j][1] * inv)),
                          pack_bf16x2(w2 * (t.v[j][2] * inv), w3 * (t.v[j][3] * inv))};
    *reinterpret_cast<u32x2*>(hb + row * ldk + col) = packed;
  }
  // the tail of the last k-step: zeros (0 * whatever LDS held could be NaN)
  for (int c = K + lane; c < kcols; c += kWave) hb[row * ldk + c].bits = 0;
}

// ---- merge prologue -----------------------------------------------------------------------
// Merged attention of the tokens' heads that fall into columns [k_begin, k_end) into LDS.
// A thread makes 8 consecutive columns of one token (inside one head: the head size is a
// multiple of 8) from all partitions of that head, eight partitions per trip to L2, keeping a
// running maximum as the attention kernels do.  There is at most one such item per thread (the
// host sees to it).  `issue` sends the loads of the first eight partitions.
typedef float f32x2 __attribute__((ext_vector_type(2)));
constexpr int kMergeBatch = 8;

struct MergeItem {
  int m, c, splits;  // token, chunk of 8 columns within the slice, partitions of the token's entry
  unsigned at;       // byte offset of the chunk's first column within partition 0 of (token, head)
  unsigned tail;     // byte offset of (maximum, denominator) within partition 0
  f32x2 ml[kMergeBatch];
  f32x4 piece[kMergeBatch][2];
};

__device__ __forceinline__ void merge_load(const MergePrologue& mp, MergeItem& t, int s0) {
  const unsigned stride = static_cast<unsigned>(mp.head_dim + 2) * 4u;
  // one resource over all tokens' partitions (the same for every lane); partitions past an
  // entry's own read as zeros (out of range)
  const __amdgpu_buffer_rsrc_t buf = make_buffer(mp.partial, mp.bytes);
#pragma unroll
  for (int u = 0; u < kMergeBatch; ++u) {
    const unsigned off = s0 + u < t.splits ? static_cast<unsigned>(s0 + u) * stride : kOutOfBuffer;
    t.ml[u] = __builtin_bit_cast(f32x2, __builtin_amdgcn_raw_buffer_load_b64(buf, t.tail + off, 0, 0));
    // rows of head_dim + 2 floats are 8-byte aligned only
    const u32x2 a = buffer_load_u32x2(buf, t.at + off), b = buffer_load_u32x2(buf, t.at + off + 8u);
    const u32x2 c = buffer_load_u32x2(buf, t.at + off + 16u), d = buffer_load_u32x2(buf, t.at + off + 24u);
    t.piece[u][0] = __builtin_bit_cast(f32x4, u32x4{a[0], a[1], b[0], b[1]});
    t.piece[u][1] = __builtin_bit_cast(f32x4, u32x4{c[0], c[1], d[0], d[1]});
  }
}

__device__ __forceinline__ void merge_issue(const MergePrologue& mp, MergeItem& t, int item, int M, int k_begin,
                                            int k_end, int kcols) {
  const int per_row = kcols / 8;
  t.m = item / per_row;
  t.c = item - t.m * per_row;
  const int k = min(k_begin + t.c * 8, k_end - 8);  // chunks past the end of K become zeros; their loads stay inside
  const int D = mp.head_dim;
  const int h = k / D;
  // the partitions that hold keys of this entry, as attn_decode cuts them
  const int ctx = mp.context_lens[t.m];
  const int first = mp.window > 0 ? max(0, ctx - mp.window) : 0;
  t.splits = min(mp.all_splits, (ctx - (first / 16) * 16 + mp.part - 1) / mp.part);
  const unsigned head_at = (static_cast<unsigned>(t.m) * mp.heads + h) * mp.all_splits * (D + 2) * 4u;
  t.at = head_at + static_cast<unsigned>(k - h * D) * 4u;
  t.tail = head_at + static_cast<unsigned>(D) * 4u;
  merge_load(mp, t, 0);
  __builtin_amdgcn_sched_barrier(0);
}

__device__ __forceinline__ void merge_finish(const MergePrologue& mp, MergeItem& t, bf16* hb, int ldk, int k_begin,
                                             int k_end) {
  float mstar = -INFINITY, den = 0.f;
  float num[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (int s0 = 0; s0 < t.splits; s0 += kMergeBatch) {
    if (s0 > 0) merge_load(mp, t, s0);
    float batch_max = -INFINITY;
#pragma unroll
    for (int u = 0; u < kMergeBatch; ++u) batch_max = fmaxf(batch_max, s0 + u < t.splits ? t.ml[u][0] : -INFINITY);
    const float m_new = fmaxf(mstar, batch_max);
    const float rescale = (mstar == -INFINITY) ? 0.f : fast_exp2(mstar - m_new);
    den *= rescale;
#pragma unroll
    for (int e = 0; e < 8; ++e) num[e] *= rescale;
    mstar = m_new;
#pragma unroll
    for (int u = 0; u < kMergeBatch; ++u) {
      const float wgt = (s0 + u >= t.splits || t.ml[u][0] == -INFINITY) ? 0.f : fast_exp2(t.ml[u][0] - mstar);
      den += wgt * t.ml[u][1];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        num[e] += wgt * t.piece[u][0][e];
        num[4 + e] += wgt * t.piece[u][1][e];
      }
    }
  }
  u32x4 packed = {0u, 0u, 0u, 0u};
  if (k_begin + t.c * 8 < k_end && t.splits > 0) {
    const float inv = 1.0f / den;
#pragma unroll
    for (int e = 0; e < 4; ++e) packed[e] = pack_bf16x2(num[2 * e] * inv, num[2 * e + 1] * inv);
  }
  *reinterpret_cast<u32x4*>(hb + t.m * ldk + t.c * 8) = packed;
}

// PRO: 0 norm, 1 merge.  QKV: the fused query/key/value epilogue (NT = 1).
template <int NT, int VPT, int PRO, bool QKV>
__global__ __launch_bounds__(kFusedWaves* kWave) void gemm_few_fused_kernel(const bf16* __restrict__ w, GemmEpilogue ep,
                                                                            QkvTarget qkv, NormPrologue np,
                                                                            MergePrologue mp, int ldk, int M, int N,
                                                                            int K) {
  static_assert(!QKV || NT == 1, "the query/key/value epilogue owns one block of 16 rows");
  constexpr int U = fused_depth(NT);
  extern __shared__ __attribute__((aligned(16))) unsigned char fused_lds[];
  bf16* const hb = reinterpret_cast<bf16*>(fused_lds);
  __shared__ float red[kFusedWaves][NT][kWave][4];
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);  // uniform, and said so: it picks buffers
  const int r = lane % 16;
  const int q = lane / 16;
  const int n0 = blockIdx.x * 16 * NT;
  const int slices = gridDim.y;
  const int chunks = K / 8;
  const int ksteps = (chunks + 3) / 4;
  const int per = (ksteps + slices - 1) / slices;
  const int sb = blockIdx.y * per;
  const int se = max(sb, min(ksteps, sb + per));  // a slice past the end of K is empty: its partial sums are zeros
  const int kcols = (se - sb) * 32;

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

  // Weights through a buffer resource: rows past the end of the matrix, chunks past the end of
  // K and k-steps past this slice read as zeros, without a branch around any load.
  const unsigned row_bytes = static_cast<unsigned>(K) * 2u;
  const __amdgpu_buffer_rsrc_t w_buf =
      QKV ? make_buffer(w, static_cast<unsigned>(N) * row_bytes)
          : make_buffer(w + static_cast<int64_t>(n0) * K, static_cast<unsigned>(min(16 * NT, N - n0)) * row_bytes);
  unsigned row_off[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
    row_off[nt] = QKV ? static_cast<unsigned>(row_of(r)) * row_bytes : static_cast<unsigned>(nt * 16 + r) * row_bytes;
  auto load_weights = [&](int s0, bf16x8_t (&a)[U][NT]) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int s = s0 + u * kFusedWaves;
      const int c = s * 4 + q;
      const bool in = s < se && c < chunks;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        a[u][nt] = __builtin_bit_cast(
            bf16x8_t, __builtin_amdgcn_raw_buffer_load_b128(w_buf, in ? row_off[nt] + c * 16u : kOutOfBuffer, 0, 2));
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  // Order of the loads: the prologue's own first (they come from L2 and are waited for first;
  // loads return in the order they were sent), then the first batch of weights, which streams
  // from memory while the activations are made.
  bf16x8_t a0[U][NT], a1[U][NT];
  if constexpr (PRO == 0) {
    NormRow<VPT, (QKV ? 32 : 8) / VPT> row;
    if (wave < M) norm_issue(np, row, wave, M, K);
    load_weights(sb + wave, a0);
    if (wave < M) norm_finish(np, row, hb, ldk, wave, M, K, kcols);
  } else {
    MergeItem item;
    const int k_begin = sb * 32, k_end = min(K, se * 32);
    const int items = M * (kcols / 8);
    // a workgroup starts at an item of its own (see the norm prologue: everybody reads the same rows)
    const int turn = static_cast<int>((static_cast<unsigned>(blockIdx.x) * 40503u) % static_cast<unsigned>(max(items, 1)));
    const int mine = static_cast<int>(threadIdx.x) + turn >= items ? static_cast<int>(threadIdx.x) + turn - items
                                                                      : static_cast<int>(threadIdx.x) + turn;
    const bool has = static_cast<int>(threadIdx.x) < items;
    if (has) merge_issue(mp, item, mine, M, k_begin, k_end, kcols);
    load_weights(sb + wave, a0);
    if (has) merge_finish(mp, item, hb, ldk, k_begin, k_end);
  }
  __syncthreads();

  f32x4_t acc[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) acc[nt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const bf16* brow = hb + min(r, M - 1) * ldk + q * 8;  // columns past M repeat the last row; their sums are dropped
  auto multiply = [&](int s0, const bf16x8_t (&a)[U][NT]) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int s = min(s0 + u * kFusedWaves, se - 1);  // past the slice: the weights are zeros
      const bf16x8_t b = load_bf16x8(brow + (s - sb) * 32);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) acc[nt] = mfma_16x16x32(a[u][nt], b, acc[nt]);
    }
  };
  constexpr int kBatch = kFusedWaves * U;
  for (int s0 = sb + wave; s0 < se; s0 += 2 * kBatch) {
    load_weights(s0 + kBatch, a1);
    multiply(s0, a0);
    if (s0 + kBatch >= se) break;
    load_weights(s0 + 2 * kBatch, a0);
    multiply(s0 + kBatch, a1);
  }

#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[wave][nt][lane][i] = acc[nt][i];
  __syncthreads();
  if (wave != 0) return;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    float v[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ww = 0; ww < kFusedWaves; ++ww)
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] += red[ww][nt][lane][i];
    if constexpr (!QKV) {
      finish4(ep, blockIdx.y, slices, r, n0 + nt * 16 + q * 4, M, N, v);
    } else {
      qkv_finish(ep, qkv, head, block_in_head, rotated, row_of(q * 4) - head * qkv.head_dim, q, min(r, M - 1), r < M, v);
    }
  }
}

constexpr int kFusedMaxLds = 140 * 1024;  // the device's 160 KB less the wavefronts' meeting place (up to 16 KB) and slack

template <int NT, int VPT, int PRO, bool QKV>
static int launch_fused(const bf16* w, const GemmEpilogue& ep, const QkvTarget& qkv, const NormPrologue& np,
                        const MergePrologue& mp, int m, int n, int k, int slices, hipStream_t stream, const char* who) {
  const int ksteps = (k / 8 + 3) / 4;
  const int per = (ksteps + slices - 1) / slices;
  const int ldk = per * 32 + 8;  // padded so that the 16 rows of an operand load fall into different banks
  const int lds = m * ldk * 2;
  if (lds > kFusedMaxLds) {
    set_error(std::string(who) + ": the activations do not fit LDS (" + std::to_string(lds) + " bytes)");
    return -1;
  }
  static int configured = 0;
  if (lds > configured) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_few_fused_kernel<NT, VPT, PRO, QKV>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, kFusedMaxLds);
    if (e != hipSuccess) {
      set_error(std::string(who) + ": cannot raise the LDS limit: " + hipGetErrorString(e));
      return -1;
    }
    configured = kFusedMaxLds;
  }
  const dim3 grid(static_cast<unsigned>((n + 16 * NT - 1) / (16 * NT)), static_cast<unsigned>(slices));
  gemm_few_fused_kernel<NT, VPT, PRO, QKV><<<grid, kFusedWaves * kWave, lds, stream>>>(w, ep, qkv, np, mp, ldk, m, n, k);
  return 0;
}

// Row blocks per workgroup: as many as still leave a workgroup for every compute unit.
static int choose_row_blocks(int n, int slices) {
  return static_cast<int64_t>((n + 31) / 32) * slices >= 256 ? 2 : 1;
}

static bool norm_arguments_ok(const void* x_in, const void* x_out, const void* delta, const void* partial,
                              int slices_in, const void* norm_weight, int m, int k, std::string& why) {
  if (!x_in || !norm_weight) why = "null pointer";
  else if (m <= 0 || m > kFusedWaves) why = "takes 1..4 tokens (a wavefront per row)";
  else if (k <= 0 || k % 8 != 0 || k > 2048) why = "k must be a multiple of 8, at most 2048";
  else if (delta != nullptr && partial != nullptr) why = "one kind of delta at a time";
  else if ((partial != nullptr) != (slices_in > 0) || slices_in < 0 || slices_in > 64) why = "partial sums and their count come together (at most 64)";
  else if ((delta != nullptr || partial != nullptr) != (x_out != nullptr)) why = "x_out is needed exactly when something is added";
  else if (x_out == x_in) why = "x_out must not be x_in (other workgroups still read it)";
  else if (reinterpret_cast<uintptr_t>(x_in) % 16 || reinterpret_cast<uintptr_t>(x_out) % 16 ||
           reinterpret_cast<uintptr_t>(delta) % 8 || reinterpret_cast<uintptr_t>(partial) % 16)
    why = "operands must be 16-byte aligned";
  return why.empty();
}

}  // namespace mlr

using namespace mlr;

extern "C" {

int mlr_gemm_norm_fused_bf16(const float* x_in, float* x_out, const void* delta, const float* partial, int slices_in,
                             const void* norm_weight, int norm_weight_is_f32, float eps, const void* w,
                             const void* bias, int bias_is_f32, void* y, int out_is_f32, int swiglu, int row_blocks,
                             int m, int n, int k, hipStream_t stream) {
  std::string why;
  if (!norm_arguments_ok(x_in, x_out, delta, partial, slices_in, norm_weight, m, k, why)) {
    set_error("mlr_gemm_norm_fused_bf16: " + why);
    return -1;
  }
  MLR_REQUIRE(w && y && n > 0, "null pointer or empty product");
  MLR_REQUIRE(reinterpret_cast<uintptr_t>(w) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0, "w and y must be 16-byte aligned");
  MLR_REQUIRE(!swiglu || (n % 4 == 0 && bias == nullptr), "swiglu needs n % 4 == 0 and no bias");
  MLR_REQUIRE(row_blocks == 0 || row_blocks == 1 || row_blocks == 2, "row_blocks must be 0 (chosen), 1 or 2");
  const GemmEpilogue ep{bias, bias_is_f32, y, out_is_f32, swiglu};
  const NormPrologue np{x_in, x_out, static_cast<const bf16*>(delta), partial, slices_in, norm_weight, norm_weight_is_f32, eps};
  const bf16* wb = static_cast<const bf16*>(w);
  // one block of 16 features per workgroup: the prologue of a few rows is cheap to repeat, and
  // twice as many workgroups keep more loads in flight
  const int nt = row_blocks ? row_blocks : 1;
  const bool small = k <= 1024;
  int status;
#define MLR_FUSED(NT)                                                                                              \
  status = small ? launch_fused<NT, 4, 0, false>(wb, ep, QkvTarget{}, np, MergePrologue{}, m, n, k, 1, stream, __func__) \
                 : launch_fused<NT, 8, 0, false>(wb, ep, QkvTarget{}, np, MergePrologue{}, m, n, k, 1, stream, __func__)
  if (nt == 2) MLR_FUSED(2);
  else MLR_FUSED(1);
#undef MLR_FUSED
  if (status != 0) return -1;
  MLR_LAUNCH_CHECK();
  return 0;
}

int mlr_qkv_norm_fused_bf16(const float* x_in, float* x_out, const void* delta, const float* partial, int slices_in,
                            const void* norm_weight, int norm_weight_is_f32, float eps, const void* w,
                            const void* bias, int bias_is_f32, const float* cos, const float* sin, const int* slots,
                            void* key_pages, void* value_pages, void* q_out, int m, int k, int heads, int kv_heads,
                            int head_dim, int block_size, int num_pages, int write, hipStream_t stream) {
  std::string why;
  if (!norm_arguments_ok(x_in, x_out, delta, partial, slices_in, norm_weight, m, k, why)) {
    set_error("mlr_qkv_norm_fused_bf16: " + why);
    return -1;
  }
  MLR_REQUIRE(w && q_out, "null pointer");
  MLR_REQUIRE(heads > 0 && kv_heads > 0 && head_dim >= 16 && head_dim % 16 == 0, "head_dim must be a multiple of 16");
  MLR_REQUIRE((cos == nullptr) == (sin == nullptr), "cos and sin come together");
  MLR_REQUIRE(!write || (slots && key_pages && value_pages && block_size > 0 && num_pages > 0),
              "a cache write needs slots, pages and their sizes");
  MLR_REQUIRE(reinterpret_cast<uintptr_t>(w) % 16 == 0 && reinterpret_cast<uintptr_t>(q_out) % 8 == 0 &&
                  reinterpret_cast<uintptr_t>(key_pages) % 8 == 0 && reinterpret_cast<uintptr_t>(cos) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(sin) % 16 == 0,
              "operands must be 16-byte aligned");
  const int64_t n = static_cast<int64_t>(heads + 2 * kv_heads) * head_dim;
  MLR_REQUIRE(n * k * 2 < (1ll << 32) && n / 16 < (1ll << 31), "the weight matrix is too large");
  const GemmEpilogue ep{bias, bias_is_f32, nullptr, 0, 0};
  const QkvTarget target{cos, sin, write ? slots : nullptr, static_cast<bf16*>(key_pages), static_cast<bf16*>(value_pages),
                         static_cast<bf16*>(q_out), heads, kv_heads, head_dim, block_size, num_pages};
  const NormPrologue np{x_in, x_out, static_cast<const bf16*>(delta), partial, slices_in, norm_weight, norm_weight_is_f32, eps};
  const bf16* wb = static_cast<const bf16*>(w);
  const int status = k <= 1024 ? launch_fused<1, 4, 0, true>(wb, ep, target, np, MergePrologue{}, m, static_cast<int>(n), k, 1, stream, __func__)
                               : launch_fused<1, 8, 0, true>(wb, ep, target, np, MergePrologue{}, m, static_cast<int>(n), k, 1, stream, __func__);
  if (status != 0) return -1;
  MLR_LAUNCH_CHECK();
  return 0;
}

int mlr_gemm_merge_fused_bf16(const float* attn_partial, const int* context_lens, int heads, int head_dim, int window,
                              int part, int splits, const void* w, const void* bias, int bias_is_f32, void* y,
                              int out_is_f32, int slices, int m, int n, hipStream_t stream) {
  MLR_REQUIRE(attn_partial && context_lens && w && y, "null pointer");
  MLR_REQUIRE(m > 0 && m <= 16, "takes 1..16 tokens (one per entry)");
  MLR_REQUIRE(slices >= 1 && static_cast<int64_t>(m) * ((((heads * head_dim / 8 + 3) / 4 + slices - 1) / slices) * 4) <= kFusedWaves * kWave,
              "a workgroup merges at most 256 chunks of 8 columns: more K slices or fewer tokens");
  MLR_REQUIRE(heads > 0 && head_dim > 0 && head_dim % 8 == 0 && head_dim <= 256, "head_dim must be a multiple of 8, at most 256");
  MLR_REQUIRE(splits >= 1 && splits <= 64, "takes 1..64 partitions");
  MLR_REQUIRE(part > 0 && window >= 0, "bad partition size or window");
  MLR_REQUIRE(n > 0 && slices >= 1 && slices <= 64, "bad sizes");
  MLR_REQUIRE(slices == 1 || out_is_f32, "partial sums are float32");
  MLR_REQUIRE(reinterpret_cast<uintptr_t>(w) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0, "w and y must be 16-byte aligned");
  const int k = heads * head_dim;
  const GemmEpilogue ep{bias, bias_is_f32, y, out_is_f32, 0};
  const int64_t partial_bytes = static_cast<int64_t>(m) * heads * splits * (head_dim + 2) * 4;
  MLR_REQUIRE(partial_bytes < (1ll << 31), "the partitions are too large for 32-bit offsets");
  const MergePrologue mp{attn_partial, context_lens, heads, head_dim, window, part, splits, static_cast<unsigned>(partial_bytes)};
  const bf16* wb = static_cast<const bf16*>(w);
  const int nt = choose_row_blocks(n, slices);
  int status;
  if (nt == 2) status = launch_fused<2, 1, 1, false>(wb, ep, QkvTarget{}, NormPrologue{}, mp, m, n, k, slices, stream, __func__);
  else status = launch_fused<1, 1, 1, false>(wb, ep, QkvTarget{}, NormPrologue{}, mp, m, n, k, slices, stream, __func__);
  if (status != 0) return -1;
  MLR_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
