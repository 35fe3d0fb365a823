// Shared helpers of the gfx950 kernel library: element types, conversions,
// wavefront (64 lanes) and workgroup reductions, and the error channel of the
// extern "C" entry points.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>

namespace mlr {

// Element type codes of the C interface.
enum DType : int { kF32 = 0, kBF16 = 1 };

constexpr int kWave = 64;

// bfloat16 as raw bits; all arithmetic happens in float.
struct bf16 {
  uint16_t bits;
};

__host__ __device__ inline float to_f32(float v) { return v; }
__host__ __device__ inline float to_f32(bf16 v) {
  union {
    uint32_t u;
    float f;
  } c;
  c.u = static_cast<uint32_t>(v.bits) << 16;
  return c.f;
}

// Round to nearest even; NaN stays NaN.  On the device this is the hardware conversion.
__host__ __device__ inline bf16 f32_to_bf16(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
  bf16 hw;
  hw.bits = __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
  return hw;
#endif
  union {
    uint32_t u;
    float f;
  } c;
  c.f = f;
  uint32_t u = c.u;
  bf16 out;
  if ((u & 0x7fffffffu) > 0x7f800000u) {
    out.bits = static_cast<uint16_t>((u >> 16) | 0x0040u);
    return out;
  }
  u += 0x7fffu + ((u >> 16) & 1u);
  out.bits = static_cast<uint16_t>(u >> 16);
  return out;
}

template <typename T>
__host__ __device__ inline T from_f32(float v);
template <>
__host__ __device__ inline float from_f32<float>(float v) {
  return v;
}
template <>
__host__ __device__ inline bf16 from_f32<bf16>(float v) {
  return f32_to_bf16(v);
}

// Load an element whose type is only known at run time (0: float, else bf16).
__device__ inline float load_as_f32(const void* p, int64_t i, int is_f32) {
  return is_f32 ? static_cast<const float*>(p)[i] : to_f32(static_cast<const bf16*>(p)[i]);
}

// Reductions over a wavefront whose 64 lanes are all active; every lane gets the result.
// Inside a row of 16 lanes the values rotate through the vector ALU's own lane crossbar
// (DPP row_ror: every lane reads the lane 1, 2, 4, 8 places to its left, cyclically), then the
// four rows' results meet as scalars.  A shuffle would go through LDS six times instead.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float lane_value(float v, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

__device__ inline float wave_sum(float v) {
  v += dpp_move<0x121>(v);  // row_ror:1
  v += dpp_move<0x122>(v);  // row_ror:2
  v += dpp_move<0x124>(v);  // row_ror:4
  v += dpp_move<0x128>(v);  // row_ror:8
  return (lane_value(v, 0) + lane_value(v, 16)) + (lane_value(v, 32) + lane_value(v, 48));
}

__device__ inline float wave_max(float v) {
  v = fmaxf(v, dpp_move<0x121>(v));
  v = fmaxf(v, dpp_move<0x122>(v));
  v = fmaxf(v, dpp_move<0x124>(v));
  v = fmaxf(v, dpp_move<0x128>(v));
  return fmaxf(fmaxf(lane_value(v, 0), lane_value(v, 16)), fmaxf(lane_value(v, 32), lane_value(v, 48)));
}

// Sum over a workgroup of up to 1024 threads (a whole number of wavefronts);
// `scratch` holds at least 16 floats of LDS.  Every thread gets the result.
__device__ inline float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int waves = (blockDim.x + kWave - 1) / kWave;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < waves; ++w) total += scratch[w];
  return total;
}

__device__ inline float block_max(float v, float* scratch) {
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int waves = (blockDim.x + kWave - 1) / kWave;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = scratch[0];
  for (int w = 1; w < waves; ++w) total = fmaxf(total, scratch[w]);
  return total;
}

// ---- host side ---------------------------------------------------------------

void set_error(const std::string& message);

// Each shared library defines MLR_ERROR_CHANNEL in exactly one of its sources.
#ifdef MLR_ERROR_CHANNEL
static thread_local std::string g_error;
void set_error(const std::string& message) { g_error = message; }
#endif

}  // namespace mlr

#ifdef MLR_ERROR_CHANNEL
extern "C" const char* mlr_last_error() { return mlr::g_error.c_str(); }
#endif

// Entry points return 0 on success and -1 after storing a message for
// mlr_last_error().
#define MLR_REQUIRE(cond, msg)                                      \
  do {                                                              \
    if (!(cond)) {                                                  \
      mlr::set_error(std::string(__func__) + ": " + (msg));         \
      return -1;                                                    \
    }                                                               \
  } while (0)

#define MLR_LAUNCH_CHECK()                                                          \
  do {                                                                              \
    hipError_t e_ = hipGetLastError();                                              \
    if (e_ != hipSuccess) {                                                         \
      mlr::set_error(std::string(__func__) + ": launch failed: " +                  \
                     hipGetErrorString(e_));                                        \
      return -1;                                                                    \
    }                                                                               \
  } while (0)
