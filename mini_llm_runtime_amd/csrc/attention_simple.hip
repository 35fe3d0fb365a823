// Paged causal attention, one wavefront per (token, query head), plain float32
// arithmetic.  It serves the true 32-bit path for every head size up to 256 and
// every group size, for prompt portions and decoded tokens alike, and is the
// on-GPU reference the MFMA attention kernels are checked against.
//
// Per tile of 64 keys: each lane scores one key (dot product over the head),
// the tile joins a running (max, sum, accumulator) softmax state, then the
// lanes switch to owning output dims and add the tile's weighted values.
// Formulas: src/mini_llm_runtime/qwen_model_runner.py:157-177 and the online
// form of csrc/paged_attention_cuda.cu:87-105; GQA head mapping
// csrc/paged_attention_cuda.cu:44-46; page addressing :71-74.
#include "api.h"
#include "common.h"

namespace mlr {

constexpr int kMaxHeadDim = 256;

template <typename T>
__global__ __launch_bounds__(64) void paged_attention_simple_kernel(
    const T* __restrict__ q, int64_t q_stride, const T* __restrict__ key_pages,
    const T* __restrict__ value_pages, const int* __restrict__ block_table, int table_width,
    const int* __restrict__ token_entry, const int* __restrict__ positions, T* __restrict__ out, int entries,
    int heads, int kv_heads, int head_dim, int block_size, int num_pages, float scale, int window) {
  __shared__ float qs[kMaxHeadDim];
  __shared__ float ps[kWave];
  __shared__ int64_t offs[kWave];
  __shared__ int64_t voffs[kWave];

  const int t = blockIdx.x;
  const int h = blockIdx.y;
  const int lane = threadIdx.x;
  const int entry = token_entry[t];
  const int p = positions[t];
  const int kvh = h / (heads / kv_heads);
  T* orow = out + (static_cast<int64_t>(t) * heads + h) * head_dim;

  if (entry < 0 || entry >= entries || p < 0) {
    for (int i = lane; i < head_dim; i += kWave) orow[i] = from_f32<T>(__builtin_nanf(""));
    return;
  }
  const T* qrow = q + t * q_stride + static_cast<int64_t>(h) * head_dim;
  for (int i = lane; i < head_dim; i += kWave) qs[i] = to_f32(qrow[i]) * scale;
  __syncthreads();

  const int* table = block_table + static_cast<int64_t>(entry) * table_width;
  const int first = window > 0 ? max(0, p - window + 1) : 0;
  float m = -INFINITY;
  float l = 0.f;
  float acc[kMaxHeadDim / kWave] = {0.f, 0.f, 0.f, 0.f};
  bool bad = false;

  for (int k0 = first; k0 <= p; k0 += kWave) {
    const int kpos = k0 + lane;
    float s = -INFINITY;
    int64_t off = -1;
    int64_t voff = -1;
    if (kpos <= p) {
      const int logical = kpos / block_size;
      const int page = logical < table_width ? table[logical] : -1;
      if (page < 0 || page >= num_pages) {
        bad = true;
      } else {
        const int in_page = kpos - logical * block_size;
        const int64_t head_base = (static_cast<int64_t>(page) * kv_heads + kvh) * block_size * head_dim;
        off = head_base + static_cast<int64_t>(in_page) * head_dim;  // keys: [offset][dim]
        voff = head_base + in_page;                                   // values: [dim][offset]
        const T* kp = key_pages + off;
        float dot = 0.f;
        for (int i = 0; i < head_dim; ++i) dot = fmaf(qs[i], to_f32(kp[i]), dot);
        s = dot;
      }
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float pr = (off >= 0) ? expf(s - m_new) : 0.f;
    const float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);
    l = l * alpha + wave_sum(pr);
    m = m_new;
    ps[lane] = pr;
    offs[lane] = off;
    voffs[lane] = voff;
    __syncthreads();
    const int count = min(kWave, p - k0 + 1);
#pragma unroll
    for (int j = 0; j < kMaxHeadDim / kWave; ++j) acc[j] *= alpha;
    for (int i = 0; i < count; ++i) {
      if (offs[i] < 0) continue;
      const float pi = ps[i];
      const T* vp = value_pages + voffs[i];
#pragma unroll
      for (int j = 0; j < kMaxHeadDim / kWave; ++j) {
        const int dim = lane + j * kWave;
        if (dim < head_dim) acc[j] = fmaf(pi, to_f32(vp[static_cast<int64_t>(dim) * block_size]), acc[j]);
      }
    }
    __syncthreads();
  }

  const bool any_bad = __any(bad);
  const float inv = 1.0f / l;
#pragma unroll
  for (int j = 0; j < kMaxHeadDim / kWave; ++j) {
    const int dim = lane + j * kWave;
    if (dim < head_dim) orow[dim] = from_f32<T>(any_bad ? __builtin_nanf("") : acc[j] * inv);
  }
}

}  // namespace mlr

using namespace mlr;

extern "C" int mlr_paged_attention_simple(const void* q, int64_t q_stride, const void* key_pages,
                                          const void* value_pages, const int* block_table, int table_width,
                                          const int* token_entry, const int* positions, void* out, int dtype,
                                          int tokens, int entries, int heads, int kv_heads, int head_dim,
                                          int block_size, int num_pages, float scale, int window,
                                          hipStream_t stream) {
  MLR_REQUIRE(q && key_pages && value_pages && block_table && token_entry && positions && out, "null pointer");
  MLR_REQUIRE(tokens > 0 && entries > 0 && heads > 0 && kv_heads > 0, "sizes must be > 0");
  MLR_REQUIRE(heads % kv_heads == 0, "query heads must be a multiple of KV heads");
  MLR_REQUIRE(head_dim > 0 && head_dim <= kMaxHeadDim, "head_dim must be within 1..256");
  MLR_REQUIRE(block_size > 0 && num_pages > 0 && table_width > 0, "page sizes must be > 0");
  MLR_REQUIRE(q_stride >= static_cast<int64_t>(heads) * head_dim, "q_stride is smaller than a row of queries");
  MLR_REQUIRE(scale > 0.f && scale < INFINITY, "scale must be positive and finite");
  MLR_REQUIRE(window >= 0, "window must be >= 0");
  MLR_REQUIRE(heads < 65536, "too many heads for one launch");
  MLR_REQUIRE(dtype == kF32 || dtype == kBF16, "dtype must be 0 (float32) or 1 (bfloat16)");
  dim3 grid(tokens, heads);
  if (dtype == kF32)
    paged_attention_simple_kernel<float><<<grid, kWave, 0, stream>>>(
        static_cast<const float*>(q), q_stride, static_cast<const float*>(key_pages),
        static_cast<const float*>(value_pages), block_table, table_width, token_entry, positions,
        static_cast<float*>(out), entries, heads, kv_heads, head_dim, block_size, num_pages, scale, window);
  else
    paged_attention_simple_kernel<bf16><<<grid, kWave, 0, stream>>>(
        static_cast<const bf16*>(q), q_stride, static_cast<const bf16*>(key_pages),
        static_cast<const bf16*>(value_pages), block_table, table_width, token_entry, positions,
        static_cast<bf16*>(out), entries, heads, kv_heads, head_dim, block_size, num_pages, scale, window);
  MLR_LAUNCH_CHECK();
  return 0;
}
