// y[M, N] = x[M, K] * w[N, K]^T (+ bias), plain float32 FMA arithmetic.
//
// This is the matrix product of the true 32-bit path (no matrix-core input
// rounding of any kind) and accepts bfloat16 operands as well, which makes it
// the reference the MFMA kernels are checked against on the GPU.  64x64 output
// tile per workgroup, 16-wide K slices staged through LDS, 4x4 outputs per lane.
// Any M, N, K > 0.  F.linear semantics: weights are [out_features, in_features]
// (src/mini_llm_runtime/qwen_model_runner.py:88-102).
#include "api.h"
#include "common.h"

namespace mlr {

constexpr int kTM = 64;
constexpr int kTN = 64;
constexpr int kTK = 16;

template <typename T>
__global__ __launch_bounds__(256) void gemm_simple_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                          const void* __restrict__ bias, int bias_is_f32,
                                                          void* __restrict__ y, int out_is_f32, int swiglu,
                                                          int M, int N, int K) {
  __shared__ float xs[kTK][kTM + 4];
  __shared__ float ws[kTK][kTN + 4];
  const int tid = threadIdx.x;
  const int tm = tid / 16;  // 0..15 -> rows tm*4 .. tm*4+3
  const int tn = tid % 16;  // 0..15 -> cols tn*4 .. tn*4+3
  const int64_t m0 = static_cast<int64_t>(blockIdx.y) * kTM;
  const int64_t n0 = static_cast<int64_t>(blockIdx.x) * kTN;

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += kTK) {
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int idx = tid + it * 256;  // 0..1023
      const int row = idx / kTK;       // 0..63
      const int kk = idx % kTK;
      const int64_t gk = k0 + kk;
      const int64_t gm = m0 + row;
      const int64_t gn = n0 + row;
      xs[kk][row] = (gm < M && gk < K) ? to_f32(x[gm * K + gk]) : 0.f;
      ws[kk][row] = (gn < N && gk < K) ? to_f32(w[gn * K + gk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kTK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[kk][tm * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[kk][tn * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t gm = m0 + tm * 4 + i;
    if (gm >= M) continue;
    if (swiglu) {
      // columns n..n+3 = gate 2j, gate 2j+1, up 2j, up 2j+1 (rows of w interleaved in pairs);
      // qwen_model_runner.py:215-216: silu(gate) * up
      const int64_t gn = n0 + tn * 4;
      if (gn >= N) continue;
      const int64_t at = gm * (N / 2) + gn / 2;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const float g = acc[i][j];
        const float v = g / (1.0f + expf(-g)) * acc[i][j + 2];
        if (out_is_f32)
          static_cast<float*>(y)[at + j] = v;
        else
          static_cast<T*>(y)[at + j] = from_f32<T>(v);
      }
      continue;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t gn = n0 + tn * 4 + j;
      if (gn >= N) continue;
      float v = acc[i][j];
      if (bias != nullptr) v += load_as_f32(bias, gn, bias_is_f32);
      if (out_is_f32)
        static_cast<float*>(y)[gm * N + gn] = v;
      else
        static_cast<T*>(y)[gm * N + gn] = from_f32<T>(v);
    }
  }
}

}  // namespace mlr

using namespace mlr;

extern "C" int mlr_gemm_simple(const void* x, const void* w, const void* bias, int bias_is_f32, void* y,
                               int out_is_f32, int swiglu, int dtype, int m, int n, int k, hipStream_t stream) {
  MLR_REQUIRE(x && w && y, "null pointer");
  MLR_REQUIRE(m > 0 && n > 0 && k > 0, "sizes must be > 0");
  MLR_REQUIRE(dtype == kF32 || dtype == kBF16, "dtype must be 0 (float32) or 1 (bfloat16)");
  MLR_REQUIRE(dtype == kBF16 || (out_is_f32 && (bias == nullptr || bias_is_f32)),
              "a float32 product has float32 bias and output");
  MLR_REQUIRE(!swiglu || (n % 4 == 0 && bias == nullptr), "swiglu needs n % 4 == 0 and no bias");
  dim3 grid((n + kTN - 1) / kTN, (m + kTM - 1) / kTM);
  MLR_REQUIRE(grid.y < 65536u, "too many rows for one launch");
  if (dtype == kF32)
    gemm_simple_kernel<float><<<grid, 256, 0, stream>>>(static_cast<const float*>(x),
                                                        static_cast<const float*>(w), bias, bias_is_f32, y,
                                                        out_is_f32, swiglu, m, n, k);
  else
    gemm_simple_kernel<bf16><<<grid, 256, 0, stream>>>(static_cast<const bf16*>(x), static_cast<const bf16*>(w),
                                                       bias, bias_is_f32, y, out_is_f32, swiglu, m, n, k);
  MLR_LAUNCH_CHECK();
  return 0;
}
