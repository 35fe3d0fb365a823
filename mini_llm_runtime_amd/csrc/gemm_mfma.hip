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
#include "api.h"
#include "common.h"
#include "mfma.h"

namespace mlr {

struct GemmEpilogue {
  const void* bias;
  int bias_is_f32;
  void* y;
  int out_is_f32;
};

// Store four consecutive output features n..n+3 of token m.
__device__ __forceinline__ void store4(const GemmEpilogue& ep, int64_t m, int n, int N, float v0, float v1,
                                       float v2, float v3) {
  float v[4] = {v0, v1, v2, v3};
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

// ---- skinny: M <= 16 * MT ---------------------------------------------------------------
template <int MT, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(const bf16* __restrict__ x,
                                                                 const bf16* __restrict__ w, GemmEpilogue ep,
                                                                 int M, int N, int K) {
  constexpr int U = 4;  // k-steps in flight per wavefront
  __shared__ float red[WAVES][MT][kWave][4];
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
  bool xok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + r;
    xok[mt] = m < M;
    xp[mt] = reinterpret_cast<const bf16x8_t*>(x + static_cast<int64_t>(min(m, M - 1)) * K);
  }
  f32x4_t acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  for (int s0 = wave; s0 < ksteps; s0 += WAVES * U) {
    bf16x8_t a[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = (s0 + u * WAVES) * 4 + q;
      a[u] = c < chunks ? wp[c] : zero_bf16x8();
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = (s0 + u * WAVES) * 4 + q;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const bf16x8_t b = (xok[mt] && c < chunks) ? xp[mt][c] : zero_bf16x8();
        acc[mt] = mfma_16x16x32(a[u], b, acc[mt]);
      }
    }
  }

#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[wave][mt][lane][i] = acc[mt][i];
  __syncthreads();
  if (wave < MT) {
    const int mt = wave;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    for (int ww = 0; ww < WAVES; ++ww)
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] += red[ww][mt][lane][i];
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
static void launch_skinny(const bf16* x, const bf16* w, const GemmEpilogue& ep, int m, int n, int k,
                          hipStream_t stream) {
  gemm_skinny_kernel<MT, WAVES><<<(n + 15) / 16, WAVES * 64, 0, stream>>>(x, w, ep, m, n, k);
}

}  // namespace mlr

using namespace mlr;

// y = x w^T (+ bias) in bfloat16 on the matrix cores; see mlr_gemm_simple for the
// argument meanings.  Requires k % 8 == 0 and 16-byte aligned x and w.
extern "C" int mlr_gemm_bf16(const void* x, const void* w, const void* bias, int bias_is_f32, void* y,
                             int out_is_f32, int m, int n, int k, hipStream_t stream) {
  MLR_REQUIRE(x && w && y, "null pointer");
  MLR_REQUIRE(m > 0 && n > 0 && k > 0, "sizes must be > 0");
  MLR_REQUIRE(k % 8 == 0, "k must be a multiple of 8");
  MLR_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0,
              "x and w must be 16-byte aligned");
  const bf16* xb = static_cast<const bf16*>(x);
  const bf16* wb = static_cast<const bf16*>(w);
  GemmEpilogue ep{bias, bias_is_f32, y, out_is_f32};
  if (m <= 64) {
    const bool deep = k >= 2048;
    if (m <= 16) {
      if (deep) launch_skinny<1, 8>(xb, wb, ep, m, n, k, stream);
      else launch_skinny<1, 4>(xb, wb, ep, m, n, k, stream);
    } else if (m <= 32) {
      if (deep) launch_skinny<2, 8>(xb, wb, ep, m, n, k, stream);
      else launch_skinny<2, 4>(xb, wb, ep, m, n, k, stream);
    } else {
      if (deep) launch_skinny<4, 8>(xb, wb, ep, m, n, k, stream);
      else launch_skinny<4, 4>(xb, wb, ep, m, n, k, stream);
    }
  } else {
    static bool configured = false;
    if (!configured) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_tiled_kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, kTiledLds);
      MLR_REQUIRE(e == hipSuccess, std::string("cannot raise the LDS limit: ") + hipGetErrorString(e));
      configured = true;
    }
    dim3 grid((n + kBN - 1) / kBN, (m + kBM - 1) / kBM);
    MLR_REQUIRE(grid.y < 65536u, "too many rows for one launch");
    gemm_tiled_kernel<<<grid, 256, kTiledLds, stream>>>(xb, wb, ep, m, n, k);
  }
  MLR_LAUNCH_CHECK();
  return 0;
}
