// Matrix-core (MFMA) vocabulary for gfx950 and the lane layouts the kernels rely on.
//
// v_mfma_f32_16x16x32_bf16: D[16x16] += A[16x32] * B[32x16].  Lane l holds
//   A[row l%16][k (l/16)*8 .. +8], B[k (l/16)*8 .. +8][col l%16],
//   D[row (l/16)*4 + i][col l%16] for i = 0..3.
// v_mfma_f32_32x32x16_bf16: D[32x32] += A[32x16] * B[16x32].  Lane l holds
//   A[row l%32][k (l/32)*8 .. +8], B[k (l/32)*8 .. +8][col l%32],
//   D[row (i/4)*8 + (l/32)*4 + i%4][col l%32] for i = 0..15.
// Both operands want 8 consecutive k per lane, i.e. 16 contiguous bytes of a
// matrix whose k index is the fastest.
#pragma once

#include <hip/hip_runtime.h>

namespace mlr {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef unsigned short u16x4_t __attribute__((ext_vector_type(4)));
typedef unsigned short u16x8_t __attribute__((ext_vector_type(8)));

__device__ __forceinline__ bf16x8_t load_bf16x8(const void* p) {
  return *reinterpret_cast<const bf16x8_t*>(p);
}

__device__ __forceinline__ bf16x8_t zero_bf16x8() {
  u16x8_t z = {0, 0, 0, 0, 0, 0, 0, 0};
  return __builtin_bit_cast(bf16x8_t, z);
}

// Buffer resource over `bytes` bytes at p: loads through it return zero beyond the end, so
// tiles at the edge of a matrix need no branches.  Offsets are unsigned 32-bit byte counts.
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
constexpr unsigned kOutOfBuffer = 0x80000000u;  // larger than any resource made here
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_buffer(const void* p, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, static_cast<int>(bytes), 0x00020000);
}
__device__ __forceinline__ bf16x8_t buffer_load_bf16x8(__amdgpu_buffer_rsrc_t rsrc, unsigned byte_offset) {
  return __builtin_bit_cast(bf16x8_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc, byte_offset, 0, 0));
}
// The same with the non-temporal hint, for bytes that are read once (weights of a few-token product).
__device__ __forceinline__ bf16x8_t buffer_load_bf16x8_once(__amdgpu_buffer_rsrc_t rsrc, unsigned byte_offset) {
  return __builtin_bit_cast(bf16x8_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc, byte_offset, 0, 2));
}

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

// Two floats to two bfloat16 in one 32-bit word (v_cvt_pk_bf16_f32, round to nearest even).
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// 2^x by the hardware instruction (no denormal fix-up: results below 2^-126 become 0,
// 2^-inf is 0), for softmax weights.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ f32x4_t mfma_16x16x32(bf16x8_t a, bf16x8_t b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ f32x16_t mfma_32x32x16(bf16x8_t a, bf16x8_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

}  // namespace mlr
