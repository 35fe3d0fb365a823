// What the bfloat16 matrix-product kernels do with their sums: bias, float32 or bfloat16
// stores, the SwiGLU pairing, partial sums of K slices, and the query/key/value product's
// rotation and cache write.  Shared by gemm_mfma.hip and gemm_fused.hip.
#pragma once

#include "common.h"
#include "mfma.h"

namespace mlr {

struct GemmEpilogue {
  const void* bias;
  int bias_is_f32;
  void* y;
  int out_is_f32;
  int swiglu;  // store silu(v0) * v2, silu(v1) * v3 into a row of N / 2
  // Rows whose normalisation is still owed (see gemm_stream.hip): x holds weight * stream, not yet
  // divided by the root mean square of the stream.  The sums of a row m are then scaled by
  // rsqrt(sum_p row_sumsq[m, p] / K + eps) before the bias: the factor is the same for the whole
  // row, so it commutes with the product.  Null: no scaling.
  const float* row_sumsq = nullptr;  // [M, sumsq_parts]: partial sums of squares of every stream row
  int sumsq_parts = 0;
  float norm_eps = 0.f;
};

// The scaling factors of rows m0 .. m0 + count - 1 into `scales` (LDS), by all wavefronts of the
// workgroup (a whole number of them): wavefront w takes the rows w, w + waves, ..., its lanes the
// partial sums lane, lane + 64, ... of a row, added in that fixed order.  The work comes in two
// halves so that the loads can be sent before the product's own loads and be added up after its
// loop, when they have long arrived: a wait for them in front of the loop would put a trip to L2
// before the first weight is asked for.  `issue` sends the loads of up to ROWS rows per wavefront
// and LOADS partial sums per lane and row; `finish` adds up, and fetches whatever `issue` could
// not hold the slow way (shapes beyond ROWS x waves rows or 64 x LOADS partial sums).  The
// caller's next __syncthreads() makes the factors visible.
template <int ROWS, int LOADS>
struct RowScaleLoads {
  float v[ROWS][LOADS];
  bool held;  // the registers hold everything
};

template <int ROWS, int LOADS>
__device__ __forceinline__ void row_scales_issue(const GemmEpilogue& ep, RowScaleLoads<ROWS, LOADS>& t, int m0, int count,
                                                 int M) {
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int waves = blockDim.x / kWave;
  t.held = count <= ROWS * waves && ep.sumsq_parts <= kWave * LOADS;
  if (!t.held) return;
  // range-checked buffer loads, no condition around any of them (a load inside a conditional block
  // makes the compiler wait for every outstanding load where the block ends): what is past a row's
  // partial sums or past the last row reads zero
  const __amdgpu_buffer_rsrc_t buf = make_buffer(ep.row_sumsq, static_cast<unsigned>(M) * ep.sumsq_parts * 4u);
#pragma unroll
  for (int i = 0; i < ROWS; ++i) {
    const int row = wave + i * waves;
    const int m = m0 + row;
#pragma unroll
    for (int j = 0; j < LOADS; ++j) {
      const int p = lane + j * kWave;
      const unsigned off = (row < count && m < M && p < ep.sumsq_parts)
                               ? (static_cast<unsigned>(m) * ep.sumsq_parts + p) * 4u
                               : kOutOfBuffer;
      t.v[i][j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(buf, off, 0, 0));
    }
  }
  __builtin_amdgcn_sched_barrier(0);  // sent here, ahead of the product's loads
}

template <int ROWS, int LOADS>
__device__ __forceinline__ void row_scales_finish(const GemmEpilogue& ep, const RowScaleLoads<ROWS, LOADS>& t, int m0,
                                                  int count, int M, int K, float* scales) {
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int waves = blockDim.x / kWave;
  if (t.held) {
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
      const int row = wave + i * waves;
      float s = 0.f;
#pragma unroll
      for (int j = 0; j < LOADS; ++j) s += t.v[i][j];
      s = wave_sum(s);
      if (lane == 0 && row < count) scales[row] = m0 + row < M ? 1.0f / sqrtf(s / static_cast<float>(K) + ep.norm_eps) : 0.f;
    }
    return;
  }
  // what the registers could not hold: a wavefront per row in turn, its lanes over the row's partial sums
  for (int row = wave; row < count; row += waves) {
    const int m = m0 + row;
    float s = 0.f;
    if (m < M)
      for (int p = lane; p < ep.sumsq_parts; p += kWave) s += ep.row_sumsq[static_cast<int64_t>(m) * ep.sumsq_parts + p];
    s = wave_sum(s);
    if (lane == 0) scales[row] = m < M ? 1.0f / sqrtf(s / static_cast<float>(K) + ep.norm_eps) : 0.f;
  }
}

__device__ __forceinline__ float silu(float g) { return g / (1.0f + __expf(-g)); }

// Store four consecutive output features n..n+3 of token m (n is a multiple of 4).
__device__ __forceinline__ void store4(const GemmEpilogue& ep, int64_t m, int n, int N, float v0, float v1,
                                       float v2, float v3) {
  float v[4] = {v0, v1, v2, v3};
  if (ep.swiglu) {
    // n..n+3 = gate 2j, gate 2j+1, up 2j, up 2j+1 with j = n / 4; N is a multiple of 4
    const int64_t at = m * (N / 2) + n / 2;
    const float a = silu(v[0]) * v[2];
    const float b = silu(v[1]) * v[3];
    if (ep.out_is_f32) {
      float* y = static_cast<float*>(ep.y) + at;
      y[0] = a;
      y[1] = b;
    } else {
      const uint32_t packed =
          static_cast<uint32_t>(f32_to_bf16(a).bits) | (static_cast<uint32_t>(f32_to_bf16(b).bits) << 16);
      *reinterpret_cast<uint32_t*>(static_cast<bf16*>(ep.y) + at) = packed;
    }
    return;
  }
  if (ep.bias != nullptr) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (n + i < N) v[i] += load_as_f32(ep.bias, n + i, ep.bias_is_f32);
  }
  const int64_t at = m * N + n;
  if (ep.out_is_f32) {
    float* y = static_cast<float*>(ep.y) + at;
    if (n + 3 < N && (at & 3) == 0) {
      *reinterpret_cast<f32x4_t*>(y) = f32x4_t{v[0], v[1], v[2], v[3]};
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (n + i < N) y[i] = v[i];
    }
  } else {
    bf16* y = static_cast<bf16*>(ep.y) + at;
    if (n + 3 < N && (at & 3) == 0) {
      u16x4_t packed = {f32_to_bf16(v[0]).bits, f32_to_bf16(v[1]).bits, f32_to_bf16(v[2]).bits,
                        f32_to_bf16(v[3]).bits};
      *reinterpret_cast<u16x4_t*>(y) = packed;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (n + i < N) y[i] = f32_to_bf16(v[i]);
    }
  }
}

// Store one accumulator tile (4 consecutive features of one token per lane): the
// final result, or this K slice's partial sums.
__device__ __forceinline__ void finish4(const GemmEpilogue& ep, int slice, int slices, int m, int n, int M, int N,
                                        const float (&v)[4]) {
  if (m >= M || n >= N) return;
  if (slices == 1) {
    store4(ep, m, n, N, v[0], v[1], v[2], v[3]);
    return;
  }
  const int64_t at = (static_cast<int64_t>(slice) * M + m) * N + n;
  float* dst = static_cast<float*>(ep.y) + at;
  float out[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    out[i] = v[i];
    if (slice == 0 && ep.bias != nullptr && n + i < N) out[i] += load_as_f32(ep.bias, n + i, ep.bias_is_f32);
  }
  if (n + 3 < N && (at & 3) == 0) {
    *reinterpret_cast<f32x4_t*>(dst) = f32x4_t{out[0], out[1], out[2], out[3]};
    return;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
    if (n + i < N) dst[i] = out[i];
}

// What the fused query/key/value product needs beside the product itself: the rotation
// tables, the cache pages and where each token goes in them.
struct QkvTarget {
  const float* cos;  // [M, head_dim / 2], or null: no rotation
  const float* sin;
  const int* slots;  // [M] cache slot of each token (negative: none), or null: no cache write
  bf16* key_pages;   // [page, kv_head, offset, head_dim]
  bf16* value_pages; // [page, kv_head, head_dim, offset]
  bf16* q_out;       // [M, heads * head_dim]
  int heads, kv_heads, head_dim, block_size, num_pages;
};

// QKV: w is [(heads + 2 kv_heads) * head_dim, K], the rows of the query heads, then the key
// heads, then the value heads.  A workgroup of the rotated part owns 8 dims j..j+7 of a head
// AND their partners j + head_dim/2 .. (src/mini_llm_runtime/qwen_model_runner.py:56-61 pairs
// dim j with j + head_dim/2), so the rotation happens on the sums before anything is stored:
// queries go to q_out, keys and values straight into their pages (:105-109).
// Four consecutive features row0..row0+3 of the fused product of `token` go where they belong:
// query heads to q_out, key and value heads into the token's cache slot (if it has one).
__device__ __forceinline__ void qkv_store4(const QkvTarget& qkv, int row0, int token, u16x4_t packed) {
  const int D = qkv.head_dim;
  const int head = row0 / D;
  const int d0 = row0 - head * D;
  if (head < qkv.heads) {
    *reinterpret_cast<u16x4_t*>(qkv.q_out + (static_cast<int64_t>(token) * qkv.heads + head) * D + d0) = packed;
    return;
  }
  if (qkv.slots == nullptr) return;
  const int slot = qkv.slots[token];
  if (slot < 0) return;
  const int page = slot / qkv.block_size;
  const int off = slot - page * qkv.block_size;
  if (page >= qkv.num_pages) return;
  if (head < qkv.heads + qkv.kv_heads) {
    const int kvh = head - qkv.heads;
    bf16* dst = qkv.key_pages + ((static_cast<int64_t>(page) * qkv.kv_heads + kvh) * qkv.block_size + off) * D + d0;
    *reinterpret_cast<u16x4_t*>(dst) = packed;
  } else {
    const int kvh = head - qkv.heads - qkv.kv_heads;
    bf16* dst = qkv.value_pages + ((static_cast<int64_t>(page) * qkv.kv_heads + kvh) * D + d0) * qkv.block_size + off;
#pragma unroll
    for (int i = 0; i < 4; ++i) dst[static_cast<int64_t>(i) * qkv.block_size].bits = packed[i];
  }
}

// Rotation and stores of the fused query/key/value product for one token: the lane holds the
// sums of four consecutive dims d0..d0+3 of `head`, which are the low halves (`low`) or the high
// halves of the rotation pairs j0..j0+3; the lane `partner_mask` away holds the other halves.
// Called by all lanes (it shuffles); `live` guards the stores.
__device__ __forceinline__ void qkv_finish_pairs(const GemmEpilogue& ep, const QkvTarget& qkv, int head, bool rotated,
                                                 int d0, int j0, bool low, int partner_mask, int token, bool live,
                                                 float (&v)[4]) {
  const int D = qkv.head_dim;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (ep.bias != nullptr) v[i] += load_as_f32(ep.bias, head * D + d0 + i, ep.bias_is_f32);
    v[i] = to_f32(f32_to_bf16(v[i]));  // the product as bfloat16, as the unfused kernels hand it on
  }
  if (rotated) {
    const int half = D / 2;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float partner = __shfl_xor(v[i], partner_mask, kWave);
      const float c = qkv.cos[static_cast<int64_t>(token) * half + j0 + i];
      const float sn = qkv.sin[static_cast<int64_t>(token) * half + j0 + i];
      v[i] = low ? v[i] * c - partner * sn : v[i] * c + partner * sn;
    }
  }
  if (!live) return;
  u16x4_t packed;
#pragma unroll
  for (int i = 0; i < 4; ++i) packed[i] = f32_to_bf16(v[i]).bits;
  qkv_store4(qkv, head * D + d0, token, packed);
}

// The same for a block of 16 weight rows (8 pairs) spread over the lane quads q = 0..3 of a
// token: quads q and q ^ 2 hold the two halves of the same pairs.
__device__ __forceinline__ void qkv_finish(const GemmEpilogue& ep, const QkvTarget& qkv, int head, int block_in_head,
                                           bool rotated, int d0, int q, int token, bool live, float (&v)[4]) {
  qkv_finish_pairs(ep, qkv, head, rotated, d0, block_in_head * 8 + (q & 1) * 4, q < 2, 32, token, live, v);
}

}  // namespace mlr
