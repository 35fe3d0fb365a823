// bfloat16 matrix products on the matrix cores: y[M, N] = x[M, K] * w[N, K]^T (+ bias).
//
// Both operands have k as their fastest index, which is what MFMA wants of both
// inputs, so tiles go from memory to the operand registers without a transpose.
// The weight tile is the A operand and the activation tile the B operand: the
// accumulator then holds four consecutive output features of one token per lane,
// which gives 8-byte stores and lets an epilogue see neighbouring features.
//
// Two kernels:
//  * gemm_skinny: up to 64 tokens (decode).  Bound by streaming w once.  A
//    workgroup owns 16 output features; its wavefronts split K between them
//    (interleaved, so the workgroup reads contiguous spans of every weight row),
//    keep several 16-byte loads in flight per lane, and add their partial sums
//    through LDS.  Activations come straight from L2.
//  * gemm_tiled: many tokens (prompts).  128 x 128 output tile per workgroup,
//    K in slices of 64 staged through double-buffered LDS, four wavefronts of
//    64 x 64 each, 32x32x16 MFMA.
// K must be a multiple of 8 (16-byte rows); other shapes take the FMA kernel.
//
// Fusions (they save whole kernels in a decode step, which is a chain of very
// short ones):
//  * norm prologue (skinny only): the input is the float32 residual stream plus
//    a not-yet-added delta; the kernel adds them, writes the sum out once,
//    multiplies by the norm weight while building its operand, collects the sum
//    of squares on the way and scales the finished sums by rsqrt(mean + eps).
//    RMSNorm commutes with the product because its statistic is one scalar per
//    token (formula: src/mini_llm_runtime/qwen_model_runner.py:22-26).
//  * SwiGLU epilogue: with gate and up rows interleaved in pairs
//    (g0 g1 u0 u1 g2 g3 u2 u3 ...) a lane holds two gate sums and their two up
//    sums and stores silu(gate) * up (qwen_model_runner.py:215-216) directly.
#include "api.h"
#include "common.h"
#include "mfma.h"

namespace mlr {

struct GemmEpilogue {
  const void* bias;
  int bias_is_f32;
  void* y;
  int out_is_f32;
  int swiglu;  // store silu(v0) * v2, silu(v1) * v3 into a row of N / 2
};

struct NormPrologue {
  const float* x;      // residual stream [M, K]
  const bf16* delta;   // not-yet-added delta [M, K], may be null
  const void* weight;  // norm weight [K]
  int weight_is_f32;
  float* x_out;        // x + delta [M, K], may be null
  float eps;
};

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

// Eight consecutive elements of the normed-but-not-yet-scaled input of token row
// `m` at chunk c: (x + delta) * weight, rounded to bfloat16; adds their squares
// to `ssq` and, when asked, writes x + delta out.
__device__ __forceinline__ bf16x8_t norm_chunk(const NormPrologue& np, int64_t row_offset, int c, bool write_out,
                                               float& ssq) {
  const f32x4_t* xp = reinterpret_cast<const f32x4_t*>(np.x + row_offset) + 2 * c;
  f32x4_t lo = xp[0];
  f32x4_t hi = xp[1];
  float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  if (np.delta != nullptr) {
    const u16x8_t d = *(reinterpret_cast<const u16x8_t*>(np.delta + row_offset) + c);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] += to_f32(bf16{d[i]});
  }
  if (write_out) {
    f32x4_t* op = reinterpret_cast<f32x4_t*>(np.x_out + row_offset) + 2 * c;
    op[0] = f32x4_t{v[0], v[1], v[2], v[3]};
    op[1] = f32x4_t{v[4], v[5], v[6], v[7]};
  }
  float w[8];
  if (np.weight_is_f32) {
    const f32x4_t* wp = reinterpret_cast<const f32x4_t*>(np.weight) + 2 * c;
    const f32x4_t a = wp[0], b = wp[1];
    w[0] = a[0]; w[1] = a[1]; w[2] = a[2]; w[3] = a[3];
    w[4] = b[0]; w[5] = b[1]; w[6] = b[2]; w[7] = b[3];
  } else {
    const u16x8_t ww = *(reinterpret_cast<const u16x8_t*>(np.weight) + c);
#pragma unroll
    for (int i = 0; i < 8; ++i) w[i] = to_f32(bf16{ww[i]});
  }
  u16x8_t out;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    ssq += v[i] * v[i];
    out[i] = f32_to_bf16(v[i] * w[i]).bits;
  }
  return __builtin_bit_cast(bf16x8_t, out);
}

// ---- skinny: M <= 16 * MT ---------------------------------------------------------------
template <int MT, int WAVES, bool NORM>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(const bf16* __restrict__ x,
                                                                 const bf16* __restrict__ w, NormPrologue np,
                                                                 GemmEpilogue ep, int M, int N, int K) {
  constexpr int U = NORM ? 4 : 8;  // k-steps in flight per wavefront
  __shared__ float red[WAVES][MT][kWave][4];
  __shared__ float red_ssq[NORM ? WAVES : 1][MT][16];
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int r = lane % 16;
  const int q = lane / 16;
  const int n0 = blockIdx.x * 16;
  const int wrow = min(n0 + r, N - 1);
  const int chunks = K / 8;             // 16-byte chunks per row
  const int ksteps = (chunks + 3) / 4;  // one MFMA consumes 4 chunks (32 elements of k)
  const bf16x8_t* wp = reinterpret_cast<const bf16x8_t*>(w + static_cast<int64_t>(wrow) * K);
  const bf16x8_t* xp[MT];
  int64_t xoff[MT];
  bool xok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + r;
    xok[mt] = m < M;
    xoff[mt] = static_cast<int64_t>(min(m, M - 1)) * K;
    xp[mt] = NORM ? nullptr : reinterpret_cast<const bf16x8_t*>(x + xoff[mt]);
  }
  const bool write_out = NORM && np.x_out != nullptr && blockIdx.x == 0;
  f32x4_t acc[MT];
  float ssq[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    acc[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    ssq[mt] = 0.f;
  }

  for (int s0 = wave; s0 < ksteps; s0 += WAVES * U) {
    bf16x8_t a[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = (s0 + u * WAVES) * 4 + q;
      a[u] = c < chunks ? __builtin_nontemporal_load(wp + c) : zero_bf16x8();
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = (s0 + u * WAVES) * 4 + q;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        bf16x8_t b = zero_bf16x8();
        if (xok[mt] && c < chunks) {
          if (NORM)
            b = norm_chunk(np, xoff[mt], c, write_out, ssq[mt]);
          else
            b = xp[mt][c];
        }
        acc[mt] = mfma_16x16x32(a[u], b, acc[mt]);
      }
    }
  }

#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
    for (int i = 0; i < 4; ++i) red[wave][mt][lane][i] = acc[mt][i];
    if (NORM) {
      float s = ssq[mt];
      s += __shfl_xor(s, 16, kWave);
      s += __shfl_xor(s, 32, kWave);
      if (q == 0) red_ssq[wave][mt][r] = s;
    }
  }
  __syncthreads();
  // wavefront w < MT finishes token tile w (MT <= WAVES)
  if (wave < MT) {
    const int mt = wave;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    for (int ww = 0; ww < WAVES; ++ww)
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] += red[ww][mt][lane][i];
    if (NORM) {
      float total = 0.f;
      for (int ww = 0; ww < WAVES; ++ww) total += red_ssq[ww][mt][r];
      const float inv = 1.0f / sqrtf(total / static_cast<float>(K) + np.eps);
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] *= inv;
    }
    const int m = mt * 16 + r;
    const int n = n0 + q * 4;
    if (m < M && n < N) store4(ep, m, n, N, v[0], v[1], v[2], v[3]);
  }
}

// ---- tiled: many tokens -----------------------------------------------------------------
constexpr int kBM = 128;  // tokens per workgroup tile
constexpr int kBN = 128;  // output features per workgroup tile
constexpr int kBK = 64;   // k per LDS slice
constexpr int kLd = kBK + 8;  // padded LDS row, in elements (144 bytes)
constexpr int kTiledLds = 2 * (kBM + kBN) * kLd * 2;  // bytes, two buffers

__global__ __launch_bounds__(256) void gemm_tiled_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w,
                                                         GemmEpilogue ep, int M, int N, int K) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  bf16* ws[2];
  bf16* xs[2];
  ws[0] = reinterpret_cast<bf16*>(smem);
  xs[0] = ws[0] + kBN * kLd;
  ws[1] = xs[0] + kBM * kLd;
  xs[1] = ws[1] + kBN * kLd;

  const int tid = threadIdx.x;
  const int lane = tid % kWave;
  const int wave = tid / kWave;
  const int wn = wave % 2;
  const int wm = wave / 2;
  const int r32 = lane % 32;
  const int h = lane / 32;
  const int n0 = blockIdx.x * kBN;
  const int m0 = blockIdx.y * kBM;
  const int chunks = K / 8;

  // global -> register staging: 4 chunks of w and 4 of x per thread and slice
  const bf16x8_t* wsrc[4];
  const bf16x8_t* xsrc[4];
  int lds_off[4];
  int chunk_in_slice[4];
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int idx = tid + it * 256;
    const int row = idx / 8;
    const int ch = idx % 8;
    wsrc[it] = reinterpret_cast<const bf16x8_t*>(w + static_cast<int64_t>(min(n0 + row, N - 1)) * K);
    xsrc[it] = reinterpret_cast<const bf16x8_t*>(x + static_cast<int64_t>(min(m0 + row, M - 1)) * K);
    lds_off[it] = row * kLd + ch * 8;
    chunk_in_slice[it] = ch;
  }

  f32x16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  const int slices = (K + kBK - 1) / kBK;
  bf16x8_t wreg[4], xreg[4];
  auto fetch = [&](int slice) {
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int c = slice * (kBK / 8) + chunk_in_slice[it];
      wreg[it] = c < chunks ? wsrc[it][c] : zero_bf16x8();
      xreg[it] = c < chunks ? xsrc[it][c] : zero_bf16x8();
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      *reinterpret_cast<bf16x8_t*>(ws[buf] + lds_off[it]) = wreg[it];
      *reinterpret_cast<bf16x8_t*>(xs[buf] + lds_off[it]) = xreg[it];
    }
  };

  fetch(0);
  stash(0);
  __syncthreads();
  for (int s = 0; s < slices; ++s) {
    const int buf = s & 1;
    if (s + 1 < slices) fetch(s + 1);
    const bf16* wt = ws[buf] + (wn * 64 + r32) * kLd + h * 8;
    const bf16* xt = xs[buf] + (wm * 64 + r32) * kLd + h * 8;
#pragma unroll
    for (int kk = 0; kk < kBK / 16; ++kk) {
      bf16x8_t a[2], b[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) a[i] = load_bf16x8(wt + i * 32 * kLd + kk * 16);
#pragma unroll
      for (int j = 0; j < 2; ++j) b[j] = load_bf16x8(xt + j * 32 * kLd + kk * 16);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = mfma_32x32x16(a[i], b[j], acc[i][j]);
    }
    if (s + 1 < slices) stash(buf ^ 1);
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int64_t m = m0 + wm * 64 + j * 32 + r32;
      if (m >= M) continue;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n = n0 + wn * 64 + i * 32 + g * 8 + h * 4;
        if (n < N)
          store4(ep, m, n, N, acc[i][j][g * 4 + 0], acc[i][j][g * 4 + 1], acc[i][j][g * 4 + 2],
                 acc[i][j][g * 4 + 3]);
      }
    }
}

template <int MT, int WAVES>
static void launch_skinny(const bf16* x, const bf16* w, const NormPrologue* np, const GemmEpilogue& ep, int m,
                          int n, int k, hipStream_t stream) {
  const unsigned grid = (n + 15) / 16;
  if (np != nullptr)
    gemm_skinny_kernel<MT, WAVES, true><<<grid, WAVES * 64, 0, stream>>>(x, w, *np, ep, m, n, k);
  else
    gemm_skinny_kernel<MT, WAVES, false><<<grid, WAVES * 64, 0, stream>>>(x, w, NormPrologue{}, ep, m, n, k);
}

static int gemm_bf16(const bf16* xb, const bf16* wb, const NormPrologue* np, const GemmEpilogue& ep, int m, int n,
                     int k, hipStream_t stream) {
  if (m <= 64) {
    const bool deep = k >= 2048;
    if (m <= 16) {
      if (deep) launch_skinny<1, 16>(xb, wb, np, ep, m, n, k, stream);
      else launch_skinny<1, 4>(xb, wb, np, ep, m, n, k, stream);
    } else if (m <= 32) {
      if (deep) launch_skinny<2, 8>(xb, wb, np, ep, m, n, k, stream);
      else launch_skinny<2, 4>(xb, wb, np, ep, m, n, k, stream);
    } else {
      if (deep) launch_skinny<4, 8>(xb, wb, np, ep, m, n, k, stream);
      else launch_skinny<4, 4>(xb, wb, np, ep, m, n, k, stream);
    }
  } else {
    static bool configured = false;
    if (!configured) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_tiled_kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, kTiledLds);
      if (e != hipSuccess) {
        set_error(std::string("mlr_gemm_bf16: cannot raise the LDS limit: ") + hipGetErrorString(e));
        return -1;
      }
      configured = true;
    }
    dim3 grid((n + kBN - 1) / kBN, (m + kBM - 1) / kBM);
    if (grid.y >= 65536u) {
      set_error("mlr_gemm_bf16: too many rows for one launch");
      return -1;
    }
    gemm_tiled_kernel<<<grid, 256, kTiledLds, stream>>>(xb, wb, ep, m, n, k);
  }
  return 0;
}

}  // namespace mlr

using namespace mlr;

extern "C" {

// y = x w^T (+ bias) in bfloat16 on the matrix cores; see mlr_gemm_simple for the
// argument meanings.  Requires k % 8 == 0 and 16-byte aligned x and w.  With
// `swiglu` the rows of w are (gate, gate, up, up) groups, there is no bias, n is
// a multiple of 4 and y is [m, n / 2].
int mlr_gemm_bf16(const void* x, const void* w, const void* bias, int bias_is_f32, void* y, int out_is_f32,
                  int swiglu, int m, int n, int k, hipStream_t stream) {
  MLR_REQUIRE(x && w && y, "null pointer");
  MLR_REQUIRE(m > 0 && n > 0 && k > 0, "sizes must be > 0");
  MLR_REQUIRE(k % 8 == 0, "k must be a multiple of 8");
  MLR_REQUIRE(!swiglu || (n % 4 == 0 && bias == nullptr), "swiglu needs n % 4 == 0 and no bias");
  MLR_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0,
              "x and w must be 16-byte aligned");
  GemmEpilogue ep{bias, bias_is_f32, y, out_is_f32, swiglu};
  if (gemm_bf16(static_cast<const bf16*>(x), static_cast<const bf16*>(w), nullptr, ep, m, n, k, stream) != 0)
    return -1;
  MLR_LAUNCH_CHECK();
  return 0;
}

// The same product with the RMSNorm of its input fused in, for up to 64 tokens:
// input = norm(x + delta) with x float32 [m, k], delta bfloat16 (may be null),
// norm weight [k] (float32 when norm_weight_is_f32, else bfloat16); x + delta is
// written to x_out (float32 [m, k], may be null; must not alias x).
int mlr_gemm_bf16_norm(const float* x, const void* delta, const void* norm_weight, int norm_weight_is_f32,
                       float eps, float* x_out, const void* w, const void* bias, int bias_is_f32, void* y,
                       int out_is_f32, int swiglu, int m, int n, int k, hipStream_t stream) {
  MLR_REQUIRE(x && norm_weight && w && y, "null pointer");
  MLR_REQUIRE(m > 0 && m <= 64 && n > 0 && k > 0, "sizes must be > 0 and m <= 64");
  MLR_REQUIRE(k % 8 == 0, "k must be a multiple of 8");
  MLR_REQUIRE(eps >= 0.f, "eps must be >= 0");
  MLR_REQUIRE(x_out != x, "x_out must not alias x");
  MLR_REQUIRE(!swiglu || (n % 4 == 0 && bias == nullptr), "swiglu needs n % 4 == 0 and no bias");
  MLR_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(delta) % 16 == 0 && reinterpret_cast<uintptr_t>(norm_weight) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(x_out) % 16 == 0,
              "operands must be 16-byte aligned");
  NormPrologue np{x, static_cast<const bf16*>(delta), norm_weight, norm_weight_is_f32, x_out, eps};
  GemmEpilogue ep{bias, bias_is_f32, y, out_is_f32, swiglu};
  if (gemm_bf16(nullptr, static_cast<const bf16*>(w), &np, ep, m, n, k, stream) != 0) return -1;
  MLR_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
