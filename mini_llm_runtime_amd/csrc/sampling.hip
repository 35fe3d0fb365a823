// Next-token choice over float32 logits: argmax (first maximum, as torch.argmax in
// src/mini_llm_runtime/engine.py:222) and temperature sampling by inverse CDF.
// The reference samples greedily only; temperature is this engine's addition.
//
// Two kernels.  sample_partial: one workgroup per (row, segment of 4,096 vocabulary
// entries) reads its segment once, coalesced, and leaves (max, first index of the
// max, sum of exp((x - max) / T)).  sample_final: one workgroup per row combines
// the segments; for a sampled row it finds the segment in which the cumulative
// sum passes uniform * total, then the 16-entry chunk, then the entry, always in
// index order.  The draw for a given uniform number therefore depends on the row's
// logits only, never on what else is in the batch.
#include "api.h"
#include "common.h"

#include <mutex>

namespace mlr {

// Scratch of mlr_sample_static: the (max, argmax, sum) triples that sample_partial leaves for
// sample_final, held by the library itself so that the entry point never allocates.  Every GPU
// the library runs on holds its own copy of this array, at its own address, until the process
// ends.  In host code the name is only a handle for hipGetSymbolAddress, never a device address.
constexpr int kStaticScratchFloats = 65536;  // 256 KiB
static __device__ __align__(256) float sample_scratch[kStaticScratchFloats];

constexpr int kSegment = 4096;
constexpr int kSampleThreads = 256;
constexpr int kChunk = kSegment / kSampleThreads;  // 16 consecutive entries per thread in the final scan

__global__ __launch_bounds__(kSampleThreads) void sample_partial_kernel(const float* __restrict__ logits,
                                                                        const float* __restrict__ temperature,
                                                                        float* __restrict__ partial, int vocab,
                                                                        int segments) {
  __shared__ float s_val[kSampleThreads];
  __shared__ int s_idx[kSampleThreads];
  __shared__ float scratch[16];
  const int row = blockIdx.x;
  const int seg = blockIdx.y;
  const int tid = threadIdx.x;
  const float* z = logits + static_cast<int64_t>(row) * vocab;
  const int begin = seg * kSegment;
  const int end = min(vocab, begin + kSegment);

  float best = -INFINITY;
  int best_i = 0x7fffffff;
  for (int i = begin + tid; i < end; i += kSampleThreads) {
    const float v = z[i];
    if (best_i == 0x7fffffff || v > best) {  // i grows, so '>' keeps the first maximum
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
      const float mv = s_val[tid];
      const int mi = s_idx[tid];
      if (oi != 0x7fffffff && (mi == 0x7fffffff || ov > mv || (ov == mv && oi < mi))) {
        s_val[tid] = ov;
        s_idx[tid] = oi;
      }
    }
    __syncthreads();
  }
  const float zmax = s_val[0];
  const int arg = s_idx[0];
  float total = 0.f;
  const float temp = temperature != nullptr ? temperature[row] : 0.f;
  if (temp > 0.f) {
    const float inv_t = 1.0f / temp;
    float part = 0.f;
    for (int i = begin + tid; i < end; i += kSampleThreads) part += expf((z[i] - zmax) * inv_t);
    total = block_sum(part, scratch);
  }
  if (tid == 0) {
    float* dst = partial + (static_cast<int64_t>(row) * segments + seg) * 3;
    dst[0] = zmax;
    dst[1] = __int_as_float(arg);
    dst[2] = total;
  }
}

__global__ __launch_bounds__(kSampleThreads) void sample_final_kernel(const float* __restrict__ logits,
                                                                      const float* __restrict__ temperature,
                                                                      const float* __restrict__ uniform,
                                                                      const float* __restrict__ partial,
                                                                      int* __restrict__ tokens, int vocab,
                                                                      int segments) {
  __shared__ float s_part[kSampleThreads];
  __shared__ int s_seg;
  __shared__ int s_pick;
  __shared__ float s_before;
  __shared__ float s_target;
  __shared__ float s_max;
  const int row = blockIdx.x;
  const int tid = threadIdx.x;
  const float* src = partial + static_cast<int64_t>(row) * segments * 3;
  const float temp = temperature != nullptr ? temperature[row] : 0.f;
  const float inv_t = temp > 0.f ? 1.0f / temp : 0.f;

  if (tid == 0) {
    float zmax = -INFINITY;
    int arg = 0;
    for (int s = 0; s < segments; ++s) {
      const float m = src[3 * s];
      if (s == 0 || m > zmax) {  // segments are in index order: '>' keeps the first maximum
        zmax = m;
        arg = __float_as_int(src[3 * s + 1]);
      }
    }
    s_max = zmax;
    s_seg = -1;
    if (!(temp > 0.f)) {
      tokens[row] = arg;
    } else {
      float total = 0.f;
      for (int s = 0; s < segments; ++s) total += src[3 * s + 2] * expf((src[3 * s] - zmax) * inv_t);
      const float target = uniform[row] * total;
      float before = 0.f;
      int pick = -1;
      for (int s = 0; s < segments; ++s) {
        const float w = src[3 * s + 2] * expf((src[3 * s] - zmax) * inv_t);
        if (before + w > target && w > 0.f) {
          pick = s;
          break;
        }
        before += w;
      }
      if (pick < 0) {
        tokens[row] = arg;  // uniform * total rounded up to the total: the mode stands in
      } else {
        s_seg = pick;
        s_before = before;
        s_target = target;
      }
    }
  }
  __syncthreads();
  const int seg = s_seg;
  if (seg < 0) return;
  const float zmax = s_max;
  const float* z = logits + static_cast<int64_t>(row) * vocab;
  const int begin = min(vocab, seg * kSegment + tid * kChunk);
  const int end = min(vocab, begin + kChunk);
  float part = 0.f;
  for (int i = begin; i < end; ++i) part += expf((z[i] - zmax) * inv_t);
  s_part[tid] = part;
  __syncthreads();
  if (tid == 0) {
    float before = s_before;
    int pick = -1;
    int last_positive = -1;
    for (int i = 0; i < kSampleThreads; ++i) {
      if (s_part[i] > 0.f) last_positive = i;
      if (before + s_part[i] > s_target && s_part[i] > 0.f) {
        pick = i;
        break;
      }
      before += s_part[i];
    }
    if (pick < 0) {  // rounding left the running sum a hair below the target
      pick = last_positive;
      before = INFINITY;
    }
    s_pick = pick;
    s_before = before;
  }
  __syncthreads();
  if (s_pick == tid) {
    float cum = s_before;
    int chosen = -1;
    int last_positive = begin;
    for (int i = begin; i < end; ++i) {
      const float e = expf((z[i] - zmax) * inv_t);
      if (e > 0.f) last_positive = i;
      if (cum != INFINITY) {
        cum += e;
        if (cum > s_target) {
          chosen = i;
          break;
        }
      }
    }
    tokens[row] = chosen >= 0 ? chosen : last_positive;
  }
}

}  // namespace mlr

using namespace mlr;

extern "C" {

// Floats of scratch mlr_sample needs.
int64_t mlr_sample_scratch(int rows, int vocab) {
  return static_cast<int64_t>(rows) * ((vocab + kSegment - 1) / kSegment) * 3;
}

int mlr_sample(const float* logits, const float* temperature, const float* uniform, int* tokens, float* scratch,
               int rows, int vocab, hipStream_t stream) {
  MLR_REQUIRE(logits && tokens && scratch, "null pointer");
  MLR_REQUIRE(rows > 0 && vocab > 0, "sizes must be > 0");
  MLR_REQUIRE((temperature == nullptr) == (uniform == nullptr), "temperature and uniform come together");
  const int segments = (vocab + kSegment - 1) / kSegment;
  MLR_REQUIRE(segments <= 65535, "vocabulary too large for one launch");
  sample_partial_kernel<<<dim3(rows, segments), kSampleThreads, 0, stream>>>(logits, temperature, scratch, vocab,
                                                                             segments);
  MLR_LAUNCH_CHECK();
  sample_final_kernel<<<rows, kSampleThreads, 0, stream>>>(logits, temperature, uniform, scratch, tokens, vocab,
                                                           segments);
  MLR_LAUNCH_CHECK();
  return 0;
}

int64_t mlr_sample_static_capacity() { return kStaticScratchFloats; }

int mlr_sample_static(const float* logits, const float* temperature, const float* uniform, int* tokens, int rows,
                      int vocab, hipStream_t stream) {
  MLR_REQUIRE(logits && tokens, "null pointer");
  MLR_REQUIRE(rows > 0 && vocab > 0, "sizes must be > 0");
  MLR_REQUIRE((temperature == nullptr) == (uniform == nullptr), "temperature and uniform come together");
  const int segments = (vocab + kSegment - 1) / kSegment;
  MLR_REQUIRE(segments <= 65535, "vocabulary too large for one launch");
  const int64_t needed = static_cast<int64_t>(rows) * segments * 3;
  if (needed > kStaticScratchFloats) {
    set_error("mlr_sample_static: " + std::to_string(rows) + " rows of " + std::to_string(vocab) + " logits need " +
              std::to_string(needed) + " floats of scratch, the library holds " + std::to_string(kStaticScratchFloats) +
              " (rows * ceil(vocab / 4096) * 3 must not exceed that); use mlr_sample with a buffer of the caller");
    return -1;
  }
  // The array's address on the current device, asked for once per device.
  constexpr int kMaxDevices = 64;
  static float* address[kMaxDevices] = {};
  static std::mutex guard;
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess || device < 0 || device >= kMaxDevices) {
    set_error(std::string("mlr_sample_static: no usable current device: ") + hipGetErrorString(e));
    return -1;
  }
  // The array whose address is used below is the current device's: a stream of another GPU would
  // run the kernels there with this GPU's address.
  hipDevice_t stream_device = -1;
  if (hipStreamGetDevice(stream, &stream_device) == hipSuccess && stream_device != device) {
    set_error("mlr_sample_static: the stream belongs to device " + std::to_string(stream_device) +
              ", the current device is " + std::to_string(device) + "; make the stream's device current first");
    return -1;
  }
  (void)hipGetLastError();  // a runtime without that query leaves an error behind: not this call's business
  float* scratch_ptr = nullptr;
  {
    std::lock_guard<std::mutex> lock(guard);
    if (address[device] == nullptr) {
      void* found = nullptr;
      e = hipGetSymbolAddress(&found, HIP_SYMBOL(sample_scratch));
      if (e != hipSuccess || found == nullptr) {
        set_error(std::string("mlr_sample_static: cannot find the scratch array on device ") + std::to_string(device) +
                  ": " + hipGetErrorString(e));
        return -1;
      }
      address[device] = static_cast<float*>(found);
    }
    scratch_ptr = address[device];
  }
  // Nothing in the array has to start at zero: sample_partial writes every triple that
  // sample_final reads, and what an earlier, larger call left behind them is never looked at.
  sample_partial_kernel<<<dim3(rows, segments), kSampleThreads, 0, stream>>>(logits, temperature, scratch_ptr, vocab,
                                                                             segments);
  MLR_LAUNCH_CHECK();
  sample_final_kernel<<<rows, kSampleThreads, 0, stream>>>(logits, temperature, uniform, scratch_ptr, tokens, vocab,
                                                           segments);
  MLR_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
