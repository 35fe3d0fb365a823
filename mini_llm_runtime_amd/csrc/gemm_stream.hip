// Products that finish the residual stream themselves: y = a w^T (+ bias) for up to 64 tokens,
// then stream += y, and the next norm prepared, all in the product's own epilogue.
//
// The output and the down projection of a decoder layer end in "add to the residual, then
// RMSNorm" (src/mini_llm_runtime/qwen_model_runner.py:199-218).  Cut along k over many
// workgroups, such a product needs a second kernel that adds the slices up, adds the residual and
// takes the norm, and a decode step of a small model is bound by its number of dependent kernels.
// Here a workgroup owns whole rows of w instead (16 output features, or 8 or 4 for fewer tokens: more
// workgroups), so that its sums are final:
//   * it adds them to its own columns of the float32 stream, in place (no other workgroup reads or
//     writes those columns);
//   * it writes h = norm_weight * stream in bfloat16: the next norm's activations but for their
//     division by the root mean square, which is one factor per row and therefore commutes with
//     the product that consumes h (that product scales its sums, see GemmEpilogue::row_sumsq);
//   * it writes its share of every row's sum of squares, one float per (row, workgroup); the
//     consumer adds the shares of a row in a fixed order.
// Nothing is summed across workgroups, so there is no atomic, no fence, and the result does not
// depend on which workgroup finishes first.  The price: every workgroup reads all rows of a (from
// L2), which is why this pays for few tokens and products whose k is not too long.
//
// The streaming loop is that of gemm_skinny_split and gemm_skinny_qkv8 (gemm_mfma.hip): the
// wavefronts of a workgroup split k, keep eight 16-byte weight loads in flight per lane and add
// their partial sums through LDS.
#include "api.h"
#include "common.h"
#include "mfma.h"

namespace mlr {

struct StreamTarget {
  const void* bias;  // [N] or null
  int bias_is_f32;
  float* stream;  // [M, N] residual stream, updated in place
  const void* norm_weight;  // [N]: the weight of the norm that follows
  int norm_weight_is_f32;
  bf16* h;       // [M, N] norm_weight * stream
  float* sumsq;  // [M, parts]
  int parts;
};

typedef float f32x4s __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2s __attribute__((ext_vector_type(2)));

// What the epilogue of one lane needs of memory for four consecutive features n..n+3 of a token:
// asked for before the product's loop (range-checked buffer loads, no branches: a lane without such
// features reads zeros), used after it.  A wait for these at the end of the kernel would be a trip to
// memory that nothing overlaps with.
struct StreamOperands {
  f32x4s x, bias_f, weight_f;
  u32x2s bias_h, weight_h;
};

__device__ __forceinline__ float bf16_lo(uint32_t pair) { return __builtin_bit_cast(float, pair << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t pair) { return __builtin_bit_cast(float, pair & 0xffff0000u); }

__device__ __forceinline__ void stream_operands_issue(const StreamTarget& t, StreamOperands& o, bool live, int token, int n,
                                                      int M, int N) {
  const unsigned row_f = static_cast<unsigned>(N) * 4u;
  const __amdgpu_buffer_rsrc_t x_buf = make_buffer(t.stream, static_cast<unsigned>(M) * row_f);
  const __amdgpu_buffer_rsrc_t bf_buf = make_buffer(t.bias, t.bias != nullptr && t.bias_is_f32 ? row_f : 0u);
  const __amdgpu_buffer_rsrc_t bh_buf = make_buffer(t.bias, t.bias != nullptr && !t.bias_is_f32 ? row_f / 2 : 0u);
  const __amdgpu_buffer_rsrc_t wf_buf = make_buffer(t.norm_weight, t.norm_weight_is_f32 ? row_f : 0u);
  const __amdgpu_buffer_rsrc_t wh_buf = make_buffer(t.norm_weight, t.norm_weight_is_f32 ? 0u : row_f / 2);
  const unsigned col = live ? static_cast<unsigned>(n) * 4u : kOutOfBuffer;
  const unsigned at = live ? (static_cast<unsigned>(token) * N + n) * 4u : kOutOfBuffer;
  o.x = __builtin_bit_cast(f32x4s, __builtin_amdgcn_raw_buffer_load_b128(x_buf, at, 0, 0));
  o.bias_f = __builtin_bit_cast(f32x4s, __builtin_amdgcn_raw_buffer_load_b128(bf_buf, col, 0, 0));
  o.bias_h = __builtin_bit_cast(u32x2s, __builtin_amdgcn_raw_buffer_load_b64(bh_buf, live ? col / 2 : kOutOfBuffer, 0, 0));
  o.weight_f = __builtin_bit_cast(f32x4s, __builtin_amdgcn_raw_buffer_load_b128(wf_buf, col, 0, 0));
  o.weight_h = __builtin_bit_cast(u32x2s, __builtin_amdgcn_raw_buffer_load_b64(wh_buf, live ? col / 2 : kOutOfBuffer, 0, 0));
}

// Four consecutive features n..n+3 of `token` (n a multiple of 4, N too): stream, h, and the
// squares' sum of the four new stream values.
__device__ __forceinline__ float finish_stream4(const StreamTarget& t, const StreamOperands& o, int token, int n, int N,
                                                const float (&v)[4]) {
  // of the two loads of the bias (and of the weight) one found an empty buffer and returned zeros
  const float bias[4] = {o.bias_f[0] + bf16_lo(o.bias_h[0]), o.bias_f[1] + bf16_hi(o.bias_h[0]),
                         o.bias_f[2] + bf16_lo(o.bias_h[1]), o.bias_f[3] + bf16_hi(o.bias_h[1])};
  const float weight[4] = {o.weight_f[0] + bf16_lo(o.weight_h[0]), o.weight_f[1] + bf16_hi(o.weight_h[0]),
                           o.weight_f[2] + bf16_lo(o.weight_h[1]), o.weight_f[3] + bf16_hi(o.weight_h[1])};
  f32x4_t s;
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    s[i] = o.x[i] + (v[i] + bias[i]);
    ss += s[i] * s[i];
  }
  *reinterpret_cast<f32x4_t*>(t.stream + static_cast<int64_t>(token) * N + n) = s;
  u16x4_t packed;
#pragma unroll
  for (int i = 0; i < 4; ++i) packed[i] = f32_to_bf16(weight[i] * s[i]).bits;
  *reinterpret_cast<u16x4_t*>(t.h + static_cast<int64_t>(token) * N + n) = packed;
  return ss;
}

// R output features a workgroup (16, 8 or 4), NB blocks of R tokens.  The 16 x 16 matrix-core block
// holds the R weight rows over 16 / R segments of k in its rows (row i: weight row i % R over segment
// i / R) and the R tokens of a block over the same segments in its columns; the blocks on the
// diagonal (row segment == column segment) are the partial sums, one per segment, the others are not
// used.  Every lane streams weights whatever R is, and fewer rows a workgroup mean more workgroups:
// what a compute unit takes in from memory is bounded (some 20 GB/s), so a long k wants all of them.
template <int WAVES, int R, int NB>
__global__ __launch_bounds__(WAVES * 64) void gemm_residual_kernel(const bf16* __restrict__ a, const bf16* __restrict__ w,
                                                                   StreamTarget target, int M, int N, int K) {
  constexpr int SEG = 16 / R;           // segments of k side by side in the block
  constexpr int FQ = R / 4;             // lanes (groups of four features) that share a token's features
  constexpr int U = NB > 2 ? 4 : 8;     // k-steps in flight per wavefront
  __shared__ float red[WAVES][NB][kWave][4];
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int r = lane % 16;
  const int q = lane / 16;
  const int rr = r % R;   // weight row (as A operand) and token within a block (as B operand)
  const int seg = r / R;  // this lane's segment of k
  const int n0 = blockIdx.x * R;
  const int chunks = K / 8;             // 16-byte chunks per row
  const int ksteps = (chunks + 3) / 4;  // one MFMA consumes 4 chunks (32 elements of k)
  const int seg_steps = (ksteps + SEG - 1) / SEG;
  const int shift = seg * seg_steps;    // the k-step this lane's segment starts at

  // the lanes of wavefront 0 that finish (token rr of a block, features n0 + 4q .. + 3) ask for their
  // epilogue operands now
  const bool owner = wave == 0 && r < R && q < FQ;
  const int n_own = n0 + q * 4;
  StreamOperands pre[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
    stream_operands_issue(target, pre[nb], owner && nb * R + rr < M && n_own < N, nb * R + rr, n_own, M, N);

  const bf16x8_t* wp = reinterpret_cast<const bf16x8_t*>(w + static_cast<int64_t>(min(n0 + rr, N - 1)) * K);
  const bf16x8_t* ap[NB];
  bool aok[NB];
  f32x4_t acc[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    ap[nb] = reinterpret_cast<const bf16x8_t*>(a + static_cast<int64_t>(min(nb * R + rr, M - 1)) * K);
    aok[nb] = nb * R + rr < M;
    acc[nb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }

  for (int s0 = wave; s0 < seg_steps; s0 += WAVES * U) {
    bf16x8_t wa[U], b[U][NB];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int s = s0 + u * WAVES;
      const int c = (s + shift) * 4 + q;
      wa[u] = (s < seg_steps && s + shift < ksteps && c < chunks) ? __builtin_nontemporal_load(wp + c) : zero_bf16x8();
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int s = s0 + u * WAVES;
      const int c = (s + shift) * 4 + q;
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
        b[u][nb] = (aok[nb] && s < seg_steps && s + shift < ksteps && c < chunks) ? ap[nb][c] : zero_bf16x8();
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) acc[nb] = mfma_16x16x32(wa[u], b[u][nb], acc[nb]);
  }

#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[wave][nb][lane][i] = acc[nb][i];
  __syncthreads();
  if (wave != 0) return;
  // Lane (column j, row group q) of the accumulator holds rows 4q .. 4q + 3 of column j.  The partial
  // sum of segment g for (token t, features 4f .. 4f + 3) is in column t + g R, row group f + g FQ.
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    if (owner) {
      for (int ww = 0; ww < WAVES; ++ww)
#pragma unroll
        for (int g = 0; g < SEG; ++g)
#pragma unroll
          for (int i = 0; i < 4; ++i) v[i] += red[ww][nb][(r + g * R) + 16 * (q + g * FQ)][i];
    }
    const int token = nb * R + rr;
    float ss = 0.f;
    if (owner && token < M && n_own < N) ss = finish_stream4(target, pre[nb], token, n_own, N, v);
    // a token's R features sit in the FQ lanes r, r + 16, ... of the first FQ row groups
    if constexpr (FQ >= 2) ss += __shfl_xor(ss, 16, kWave);
    if constexpr (FQ >= 4) ss += __shfl_xor(ss, 32, kWave);
    if (owner && q == 0 && token < M) target.sumsq[static_cast<int64_t>(token) * target.parts + blockIdx.x] = ss;
  }
}

// Rows a workgroup owns: the fewest (most workgroups) whose token blocks (of as many tokens as rows)
// stay within four.
static int residual_rows(int m) { return m <= 16 ? 4 : (m <= 32 ? 8 : 16); }

}  // namespace mlr

using namespace mlr;

extern "C" {

int mlr_gemm_residual_parts(int m, int n) {
  const int rows = residual_rows(m);
  return (n + rows - 1) / rows;
}

int mlr_gemm_residual_bf16(const void* a, const void* w, const void* bias, int bias_is_f32, float* stream,
                           const void* norm_weight, int norm_weight_is_f32, void* h, float* sumsq, int m, int n,
                           int k, hipStream_t stream_handle) {
  MLR_REQUIRE(a && w && stream && norm_weight && h && sumsq, "null pointer");
  MLR_REQUIRE(m > 0 && m <= 64, "takes 1..64 tokens");
  MLR_REQUIRE(n > 0 && n % 4 == 0, "n must be a positive multiple of 4");
  MLR_REQUIRE(k > 0 && k % 8 == 0 && k <= (1 << 20), "k must be a positive multiple of 8, at most 2^20");
  MLR_REQUIRE(reinterpret_cast<uintptr_t>(a) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(stream) % 16 == 0 && reinterpret_cast<uintptr_t>(h) % 8 == 0 &&
                  reinterpret_cast<uintptr_t>(sumsq) % 4 == 0,
              "a, w and the stream must be 16-byte aligned, h 8-byte");
  const int parts = mlr_gemm_residual_parts(m, n);
  const StreamTarget target{bias, bias_is_f32, stream, norm_weight, norm_weight_is_f32, static_cast<bf16*>(h), sumsq, parts};
  const bf16* ab = static_cast<const bf16*>(a);
  const bf16* wb = static_cast<const bf16*>(w);
  const dim3 grid(static_cast<unsigned>(parts));
  const int rows = residual_rows(m);
  const int blocks = (m + rows - 1) / rows;
#define MLR_RESIDUAL(R, NB) gemm_residual_kernel<4, R, NB><<<grid, 256, 0, stream_handle>>>(ab, wb, target, m, n, k)
#define MLR_RESIDUAL_ROWS(R)                   \
  do {                                         \
    if (blocks == 1) MLR_RESIDUAL(R, 1);       \
    else if (blocks == 2) MLR_RESIDUAL(R, 2);  \
    else MLR_RESIDUAL(R, 4);                   \
  } while (0)
  if (rows == 4) MLR_RESIDUAL_ROWS(4);
  else if (rows == 8) MLR_RESIDUAL_ROWS(8);
  else MLR_RESIDUAL_ROWS(16);
#undef MLR_RESIDUAL_ROWS
#undef MLR_RESIDUAL
  MLR_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
