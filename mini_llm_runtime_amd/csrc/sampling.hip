// Next-token choice over float32 logits: argmax (first maximum, as torch.argmax in
// src/mini_llm_runtime/engine.py:222) and temperature sampling by inverse CDF.
// The reference samples greedily only; temperature is this engine's addition.
//
// One workgroup per row.  Every lane owns one contiguous chunk of the vocabulary,
// so the cumulative sums are taken in index order and the result for a given
// uniform number does not depend on what else is in the batch.
#include "api.h"
#include "common.h"

namespace mlr {

constexpr int kSampleThreads = 256;

__global__ __launch_bounds__(kSampleThreads) void sample_kernel(const float* __restrict__ logits,
                                                                const float* __restrict__ temperature,
                                                                const float* __restrict__ uniform,
                                                                int* __restrict__ tokens, int vocab) {
  __shared__ float s_val[kSampleThreads];
  __shared__ int s_idx[kSampleThreads];
  __shared__ float s_part[kSampleThreads];
  __shared__ int s_pick;
  __shared__ float s_before;
  __shared__ float s_target;

  const int row = blockIdx.x;
  const int tid = threadIdx.x;
  const float* z = logits + static_cast<int64_t>(row) * vocab;
  const int chunk = (vocab + kSampleThreads - 1) / kSampleThreads;
  const int begin = min(vocab, tid * chunk);
  const int end = min(vocab, begin + chunk);

  float best = -INFINITY;
  int best_i = 0x7fffffff;
  for (int i = begin; i < end; ++i) {
    const float v = z[i];
    if (v > best || best_i == 0x7fffffff) {
      best = v;
      best_i = i;
    }
  }
  s_val[tid] = best;
  s_idx[tid] = best_i;
  __syncthreads();
  for (int step = kSampleThreads / 2; step > 0; step >>= 1) {
    if (tid < step) {
      const float ov = s_val[tid + step];
      const int oi = s_idx[tid + step];
      // chunks are in index order, so on a tie the lower thread already holds the lower index
      if (oi != 0x7fffffff && (s_idx[tid] == 0x7fffffff || ov > s_val[tid])) {
        s_val[tid] = ov;
        s_idx[tid] = oi;
      }
    }
    __syncthreads();
  }
  const float zmax = s_val[0];
  const int arg = s_idx[0];
  const float temp = temperature != nullptr ? temperature[row] : 0.f;
  if (!(temp > 0.f)) {
    if (tid == 0) tokens[row] = arg;
    return;
  }

  const float inv_t = 1.0f / temp;
  float part = 0.f;
  for (int i = begin; i < end; ++i) part += expf((z[i] - zmax) * inv_t);
  s_part[tid] = part;
  __syncthreads();
  if (tid == 0) {
    float total = 0.f;
    for (int i = 0; i < kSampleThreads; ++i) total += s_part[i];
    const float target = uniform[row] * total;
    float before = 0.f;
    int pick = -1;
    for (int i = 0; i < kSampleThreads; ++i) {
      const float after = before + s_part[i];
      if (after > target && s_part[i] > 0.f) {
        pick = i;
        break;
      }
      before = after;
    }
    s_pick = pick;
    s_before = before;
    s_target = target;
    if (pick < 0) tokens[row] = arg;  // uniform rounded up to the total: fall back to the mode
  }
  __syncthreads();
  if (s_pick == tid) {
    float cum = s_before;
    int chosen = -1;
    int last_positive = arg;
    for (int i = begin; i < end; ++i) {
      const float e = expf((z[i] - zmax) * inv_t);
      cum += e;
      if (e > 0.f) last_positive = i;
      if (cum > s_target) {
        chosen = i;
        break;
      }
    }
    // rounding may leave the chunk's own running sum a hair below the target
    tokens[row] = chosen >= 0 ? chosen : last_positive;
  }
}

}  // namespace mlr

using namespace mlr;

extern "C" int mlr_sample(const float* logits, const float* temperature, const float* uniform, int* tokens,
                          int rows, int vocab, hipStream_t stream) {
  MLR_REQUIRE(logits && tokens, "null pointer");
  MLR_REQUIRE(rows > 0 && vocab > 0, "sizes must be > 0");
  MLR_REQUIRE((temperature == nullptr) == (uniform == nullptr), "temperature and uniform come together");
  sample_kernel<<<rows, kSampleThreads, 0, stream>>>(logits, temperature, uniform, tokens, vocab);
  MLR_LAUNCH_CHECK();
  return 0;
}
