// Row-wise and element-wise kernels: embedding gather, RMSNorm fused with the
// residual addition, SiLU-multiply, rotary tables, and the fused rotary encoding
// plus paged key/value store.  All arithmetic is float32; bfloat16 only exists
// in memory.
#define MLR_ERROR_CHANNEL
#include "api.h"
#include "common.h"
#include "mfma.h"

namespace mlr {

typedef float f32x4 __attribute__((ext_vector_type(4)));

// ---- embedding -------------------------------------------------------------------
// qwen_model_runner.py:263 (F.embedding): a row gather, no scaling.
template <typename T>
__global__ __launch_bounds__(256) void embedding_kernel(const T* __restrict__ table,
                                                        const int* __restrict__ ids,
                                                        float* __restrict__ out, int hidden, int vocab) {
  const int t = blockIdx.x;
  const int id = ids[t];
  float* dst = out + static_cast<int64_t>(t) * hidden;
  if (id < 0 || id >= vocab) {
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = __builtin_nanf("");
    return;
  }
  const T* src = table + static_cast<int64_t>(id) * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = to_f32(src[i]);
}

// ---- RMSNorm (+ residual addition) ---------------------------------------------------
// qwen_model_runner.py:22-26: weight * x * rsqrt(mean(x^2) + eps), statistics in float32.
// The not-yet-added delta is either one tensor in the engine's dtype or `slices`
// float32 partial sums [slice, rows, hidden] of a product that was cut along k;
// they are added in slice order, so the sum does not depend on timing.
// One workgroup per row; a row of up to THREADS * 4 * VPT elements stays in registers
// between the statistics and the scaling (hidden must be a multiple of 4).  Few wide rows
// (a decode step of a large model) take 1,024 threads each: a compute unit takes in what its
// wavefronts keep in flight, and a row with eight slices of partial sums is 100 KB and more.
template <typename T, typename TW, int VPT, int THREADS = 256>
__global__ __launch_bounds__(THREADS) void rmsnorm_kernel(float* __restrict__ x, const T* __restrict__ delta,
                                                      const float* __restrict__ partial, int slices, int rows,
                                                      const TW* __restrict__ weight, T* __restrict__ out,
                                                      int hidden, float eps) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  const int quads = hidden / 4;
  // Loads first, all of them unconditional (an index past the end is clamped and its value
  // dropped), so that they are in flight together: a wait per slice would cost more than the
  // whole kernel otherwise.
  constexpr int kSliceBatch = 8;
  f32x4 v[VPT];
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int i = min(threadIdx.x + j * THREADS, quads - 1);
    const int64_t at = row * hidden + 4 * i;
    v[j] = *reinterpret_cast<const f32x4*>(x + at);
    if (delta != nullptr) {
#pragma unroll
      for (int e = 0; e < 4; ++e) v[j][e] += to_f32(delta[at + e]);
    }
  }
  for (int s0 = 0; s0 < slices; s0 += kSliceBatch) {
    f32x4 p[VPT][kSliceBatch];
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
      const int i = min(threadIdx.x + j * THREADS, quads - 1);
#pragma unroll
      for (int u = 0; u < kSliceBatch; ++u) {
        const int sl = min(s0 + u, slices - 1);
        p[j][u] = *reinterpret_cast<const f32x4*>(partial + (static_cast<int64_t>(sl) * rows + row) * hidden + 4 * i);
      }
    }
#pragma unroll
    for (int u = 0; u < kSliceBatch; ++u) {
      const bool live = s0 + u < slices;
#pragma unroll
      for (int j = 0; j < VPT; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) v[j][e] = live ? v[j][e] + p[j][u][e] : v[j][e];
    }
  }
  float ss = 0.f;
  const bool changed = delta != nullptr || slices > 0;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int i = threadIdx.x + j * THREADS;
    if (i >= quads) {
      v[j] = f32x4{0.f, 0.f, 0.f, 0.f};
      continue;
    }
    if (changed) *reinterpret_cast<f32x4*>(x + row * hidden + 4 * i) = v[j];
#pragma unroll
    for (int e = 0; e < 4; ++e) ss += v[j][e] * v[j][e];
  }
  const float total = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(total / static_cast<float>(hidden) + eps);
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int i = threadIdx.x + j * THREADS;
    if (i >= quads) continue;
    const int64_t at = row * hidden + 4 * i;
#pragma unroll
    for (int e = 0; e < 4; ++e) out[at + e] = from_f32<T>(to_f32(weight[4 * i + e]) * (v[j][e] * inv));
  }
}

// Any width: the row is read again for the scaling.
template <typename T, typename TW>
__global__ __launch_bounds__(256) void rmsnorm_any_kernel(float* __restrict__ x, const T* __restrict__ delta,
                                                          const float* __restrict__ partial, int slices, int rows,
                                                          const TW* __restrict__ weight, T* __restrict__ out,
                                                          int hidden, float eps) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  float* xr = x + row * hidden;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float v = xr[i];
    if (delta != nullptr) v += to_f32(delta[row * hidden + i]);
    for (int s = 0; s < slices; ++s) v += partial[(static_cast<int64_t>(s) * rows + row) * hidden + i];
    if (delta != nullptr || slices > 0) xr[i] = v;
    ss += v * v;
  }
  const float total = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(total / static_cast<float>(hidden) + eps);
  T* orow = out + row * hidden;
  // each thread re-reads the elements it wrote itself
  for (int i = threadIdx.x; i < hidden; i += blockDim.x)
    orow[i] = from_f32<T>(to_f32(weight[i]) * (xr[i] * inv));
}

template <typename T, typename TW>
static void launch_rmsnorm(float* x, const void* delta, const float* partial, int slices, const void* weight,
                           void* out, int rows, int hidden, float eps, hipStream_t stream) {
  const T* d = static_cast<const T*>(delta);
  const TW* w = static_cast<const TW*>(weight);
  T* o = static_cast<T*>(out);
  const int quads = hidden / 4;
  if (hidden % 4 != 0 || quads > 256 * 8)
    rmsnorm_any_kernel<T, TW><<<rows, 256, 0, stream>>>(x, d, partial, slices, rows, w, o, hidden, eps);
  else if (rows <= 64 && quads > 512 && quads <= 1024)
    rmsnorm_kernel<T, TW, 1, 1024><<<rows, 1024, 0, stream>>>(x, d, partial, slices, rows, w, o, hidden, eps);
  else if (rows <= 64 && quads > 1024)
    rmsnorm_kernel<T, TW, 2, 1024><<<rows, 1024, 0, stream>>>(x, d, partial, slices, rows, w, o, hidden, eps);
  else if (quads <= 256)
    rmsnorm_kernel<T, TW, 1><<<rows, 256, 0, stream>>>(x, d, partial, slices, rows, w, o, hidden, eps);
  else if (quads <= 512)
    rmsnorm_kernel<T, TW, 2><<<rows, 256, 0, stream>>>(x, d, partial, slices, rows, w, o, hidden, eps);
  else if (quads <= 1024)
    rmsnorm_kernel<T, TW, 4><<<rows, 256, 0, stream>>>(x, d, partial, slices, rows, w, o, hidden, eps);
  else
    rmsnorm_kernel<T, TW, 8><<<rows, 256, 0, stream>>>(x, d, partial, slices, rows, w, o, hidden, eps);
}

template <typename T>
__global__ __launch_bounds__(256) void add_kernel(float* __restrict__ x, const T* __restrict__ delta,
                                                  int64_t count) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < count) x[i] += to_f32(delta[i]);
}

__global__ __launch_bounds__(256) void gather_rows_kernel(const uint32_t* __restrict__ src,
                                                          const int* __restrict__ rows,
                                                          uint32_t* __restrict__ out, int64_t row_words,
                                                          int src_rows) {
  const int k = blockIdx.x;
  const int r = rows[k];
  src += static_cast<int64_t>(blockIdx.y) * src_rows * row_words;  // plane of a [planes, rows, width] source
  uint32_t* dst = out + (static_cast<int64_t>(blockIdx.y) * gridDim.x + k) * row_words;
  if (r < 0 || r >= src_rows) {
    for (int64_t i = threadIdx.x; i < row_words; i += blockDim.x) dst[i] = 0xffffffffu;  // NaN in both types
    return;
  }
  const uint32_t* s = src + static_cast<int64_t>(r) * row_words;
  for (int64_t i = threadIdx.x; i < row_words; i += blockDim.x) dst[i] = s[i];
}

// qwen_model_runner.py:215-216: silu(gate) * up, silu(z) = z * sigmoid(z).
template <typename T>
__global__ __launch_bounds__(256) void silu_mul_kernel(const T* __restrict__ gate_up, T* __restrict__ out,
                                                       int rows, int inter) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t total = static_cast<int64_t>(rows) * inter;
  if (i >= total) return;
  const int64_t m = i / inter;
  const int64_t c = i - m * inter;
  const float g = to_f32(gate_up[m * 2 * inter + c]);
  const float u = to_f32(gate_up[m * 2 * inter + inter + c]);
  const float s = g / (1.0f + expf(-g));
  out[i] = from_f32<T>(s * u);
}

// ---- rotary tables -------------------------------------------------------------------
// qwen_model_runner.py:45-57: angle = position * inv_freq[j]; here the product and
// its cosine and sine are evaluated in float64 and rounded once to float32.
__global__ __launch_bounds__(256) void rope_table_kernel(const int* __restrict__ positions,
                                                         const double* __restrict__ inv_freq,
                                                         float* __restrict__ cos_out,
                                                         float* __restrict__ sin_out, int tokens, int half) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= static_cast<int64_t>(tokens) * half) return;
  const int t = static_cast<int>(i / half);
  const int j = static_cast<int>(i - static_cast<int64_t>(t) * half);
  const double angle = static_cast<double>(positions[t]) * inv_freq[j];
  cos_out[i] = static_cast<float>(cos(angle));
  sin_out[i] = static_cast<float>(sin(angle));
}

// ---- rotary encoding + paged key/value store ------------------------------------------
// qwen_model_runner.py:56-61 (x * cos + rotate_half(x) * sin: dims j and j + r/2 are
// a pair) and :105-109 (the cache keeps the rotated k and the raw v).  Key pages are
// [page, kv_head, offset, head_dim] as paged_kv_cache.py:287-291; value pages are
// transposed inside a page, [page, kv_head, head_dim, offset].
template <typename T>
__global__ __launch_bounds__(256) void rope_kv_write_kernel(
    T* __restrict__ qkv, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ slots, T* __restrict__ key_pages, T* __restrict__ value_pages, int heads,
    int kv_heads, int head_dim, int rotary_dim, int block_size, int num_pages, int write) {
  const int t = blockIdx.x;
  const int half = rotary_dim / 2;
  const int64_t width = static_cast<int64_t>(heads + 2 * kv_heads) * head_dim;
  T* q = qkv + t * width;
  T* k = q + static_cast<int64_t>(heads) * head_dim;
  T* v = k + static_cast<int64_t>(kv_heads) * head_dim;
  const float* cs = cos_t + static_cast<int64_t>(t) * half;
  const float* sn = sin_t + static_cast<int64_t>(t) * half;

  int64_t page_base = -1;   // element offset of key (page, kv_head 0, offset, 0)
  int64_t value_base = -1;  // element offset of value (page, kv_head 0, dim 0, offset)
  int64_t head_stride = static_cast<int64_t>(block_size) * head_dim;
  if (write) {
    const int slot = slots[t];
    if (slot >= 0) {
      const int page = slot / block_size;
      const int off = slot - page * block_size;
      if (page < num_pages) {
        page_base = (static_cast<int64_t>(page) * kv_heads * block_size + off) * head_dim;
        value_base = static_cast<int64_t>(page) * kv_heads * head_stride + off;
      }
    }
  }

  for (int i = threadIdx.x; i < heads * half; i += blockDim.x) {
    const int h = i / half;
    const int j = i - h * half;
    T* p = q + h * head_dim;
    const float a = to_f32(p[j]);
    const float b = to_f32(p[j + half]);
    p[j] = from_f32<T>(a * cs[j] - b * sn[j]);
    p[j + half] = from_f32<T>(b * cs[j] + a * sn[j]);
  }
  for (int i = threadIdx.x; i < kv_heads * half; i += blockDim.x) {
    const int h = i / half;
    const int j = i - h * half;
    T* p = k + h * head_dim;
    const float a = to_f32(p[j]);
    const float b = to_f32(p[j + half]);
    const T ra = from_f32<T>(a * cs[j] - b * sn[j]);
    const T rb = from_f32<T>(b * cs[j] + a * sn[j]);
    p[j] = ra;
    p[j + half] = rb;
    if (page_base >= 0) {
      T* dst = key_pages + page_base + h * head_stride;
      dst[j] = ra;
      dst[j + half] = rb;
    }
  }
  if (page_base >= 0) {
    const int tail = head_dim - rotary_dim;
    for (int i = threadIdx.x; i < kv_heads * tail; i += blockDim.x) {
      const int h = i / tail;
      const int j = rotary_dim + (i - h * tail);
      key_pages[page_base + h * head_stride + j] = k[h * head_dim + j];
    }
    for (int i = threadIdx.x; i < kv_heads * head_dim; i += blockDim.x) {
      const int h = i / head_dim;
      const int j = i - h * head_dim;
      value_pages[value_base + h * head_stride + static_cast<int64_t>(j) * block_size] = v[h * head_dim + j];
    }
  }
}

// The same for bfloat16 with the whole head rotated and a head size that is a multiple of 16: a thread
// takes 8 dims of the first half of a head and their 8 partners in 16-byte loads and stores (2,048 tokens
// of the 7B shape: 17.7 to 15.6 us; what is left is the values' scatter into their transposed pages,
// 2 bytes at a stride of a page row).
__global__ __launch_bounds__(256) void rope_kv_write_bf16x8_kernel(
    bf16* __restrict__ qkv, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ slots, bf16* __restrict__ key_pages, bf16* __restrict__ value_pages, int heads, int kv_heads,
    int head_dim, int block_size, int num_pages, int write) {
  const int t = blockIdx.x;
  const int half = head_dim / 2;
  const int per_head = half / 8;  // pairs of 16-byte pieces
  const int64_t width = static_cast<int64_t>(heads + 2 * kv_heads) * head_dim;
  bf16* q = qkv + t * width;
  bf16* v = q + static_cast<int64_t>(heads + kv_heads) * head_dim;
  const float* cs = cos_t + static_cast<int64_t>(t) * half;
  const float* sn = sin_t + static_cast<int64_t>(t) * half;

  int64_t page_base = -1, value_base = -1;  // as in rope_kv_write_kernel
  const int64_t head_stride = static_cast<int64_t>(block_size) * head_dim;
  if (write) {
    const int slot = slots[t];
    if (slot >= 0) {
      const int page = slot / block_size;
      const int off = slot - page * block_size;
      if (page < num_pages) {
        page_base = (static_cast<int64_t>(page) * kv_heads * block_size + off) * head_dim;
        value_base = static_cast<int64_t>(page) * kv_heads * head_stride + off;
      }
    }
  }
  for (int i = threadIdx.x; i < (heads + kv_heads) * per_head; i += blockDim.x) {
    const int h = i / per_head;  // query heads first, then key heads: they lie behind one another in the row
    const int j = (i - h * per_head) * 8;
    bf16* p = q + static_cast<int64_t>(h) * head_dim;
    const u16x8_t lo = *reinterpret_cast<const u16x8_t*>(p + j);
    const u16x8_t hi = *reinterpret_cast<const u16x8_t*>(p + j + half);
    const f32x4_t c0 = *reinterpret_cast<const f32x4_t*>(cs + j), c1 = *reinterpret_cast<const f32x4_t*>(cs + j + 4);
    const f32x4_t s0 = *reinterpret_cast<const f32x4_t*>(sn + j), s1 = *reinterpret_cast<const f32x4_t*>(sn + j + 4);
    u16x8_t out_lo, out_hi;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float a = to_f32(bf16{lo[e]}), b = to_f32(bf16{hi[e]});
      const float c = e < 4 ? c0[e] : c1[e - 4], sv = e < 4 ? s0[e] : s1[e - 4];
      out_lo[e] = f32_to_bf16(a * c - b * sv).bits;
      out_hi[e] = f32_to_bf16(b * c + a * sv).bits;
    }
    *reinterpret_cast<u16x8_t*>(p + j) = out_lo;
    *reinterpret_cast<u16x8_t*>(p + j + half) = out_hi;
    if (h >= heads && page_base >= 0) {
      bf16* dst = key_pages + page_base + (h - heads) * head_stride;
      *reinterpret_cast<u16x8_t*>(dst + j) = out_lo;
      *reinterpret_cast<u16x8_t*>(dst + j + half) = out_hi;
    }
  }
  if (page_base >= 0) {
    for (int i = threadIdx.x; i < kv_heads * head_dim; i += blockDim.x) {
      const int h = i / head_dim;
      const int j = i - h * head_dim;
      value_pages[value_base + h * head_stride + static_cast<int64_t>(j) * block_size] = v[h * head_dim + j];
    }
  }
}

// ---- the query/key/value product that came as K slices -----------------------------------------
// A wide product of few tokens streams its weights fastest through the LDS-tiled kernel cut
// along K, which leaves float32 partial sums [slice, token, width] (the bias in slice 0).  This
// kernel finishes them as the fused kernels would: the slices are added in their order, the sum
// is rounded to bfloat16 (what the unfused product hands on), query and key heads are rotated
// (qwen_model_runner.py:56-61: dim j with j + head_dim / 2), queries go to q_out
// [token, heads * head_dim], keys and values into the token's cache slot (:105-109).  One
// wavefront per (token, head).
__global__ __launch_bounds__(64) void qkv_finish_kernel(const float* __restrict__ partial, int slices,
                                                       const float* __restrict__ cos_t,
                                                       const float* __restrict__ sin_t,
                                                       const int* __restrict__ slots, bf16* __restrict__ key_pages,
                                                       bf16* __restrict__ value_pages, bf16* __restrict__ q_out,
                                                       int tokens, int heads, int kv_heads, int head_dim,
                                                       int block_size, int num_pages) {
  const int t = blockIdx.x;
  const int head = blockIdx.y;
  const int half = head_dim / 2;
  const int64_t width = static_cast<int64_t>(heads + 2 * kv_heads) * head_dim;
  const int64_t slice_stride = static_cast<int64_t>(tokens) * width;
  const float* row = partial + t * width + static_cast<int64_t>(head) * head_dim;
  const bool rotated = cos_t != nullptr && head < heads + kv_heads;
  // where this head's values go
  bf16* q_row = nullptr;
  bf16* key_row = nullptr;    // [head_dim] of the token's slot
  bf16* value_col = nullptr;  // dim d at value_col[d * block_size]
  if (head < heads) {
    q_row = q_out + (static_cast<int64_t>(t) * heads + head) * head_dim;
  } else if (slots != nullptr) {
    const int slot = slots[t];
    if (slot >= 0 && slot / block_size < num_pages) {
      const int page = slot / block_size, off = slot - page * block_size;
      if (head < heads + kv_heads)
        key_row = key_pages + ((static_cast<int64_t>(page) * kv_heads + (head - heads)) * block_size + off) * head_dim;
      else
        value_col = value_pages + (static_cast<int64_t>(page) * kv_heads + (head - heads - kv_heads)) * head_dim * block_size + off;
    }
  }
  for (int j = threadIdx.x; j < half; j += 64) {
    float a = 0.f, b = 0.f;
#pragma unroll 8
    for (int s = 0; s < slices; ++s) {
      a += row[s * slice_stride + j];
      b += row[s * slice_stride + j + half];
    }
    a = to_f32(f32_to_bf16(a));
    b = to_f32(f32_to_bf16(b));
    float ra = a, rb = b;
    if (rotated) {
      const float c = cos_t[static_cast<int64_t>(t) * half + j];
      const float sn = sin_t[static_cast<int64_t>(t) * half + j];
      ra = a * c - b * sn;
      rb = b * c + a * sn;
    }
    const bf16 lo = f32_to_bf16(ra), hi = f32_to_bf16(rb);
    if (q_row != nullptr) {
      q_row[j] = lo;
      q_row[j + half] = hi;
    } else if (key_row != nullptr) {
      key_row[j] = lo;
      key_row[j + half] = hi;
    } else if (value_col != nullptr) {
      value_col[static_cast<int64_t>(j) * block_size] = lo;
      value_col[static_cast<int64_t>(j + half) * block_size] = hi;
    }
  }
}

}  // namespace mlr

using namespace mlr;

extern "C" {

int mlr_version() { return 1; }

int mlr_embedding(const void* table, int dtype, const int* ids, float* out, int tokens, int hidden,
                  int vocab, hipStream_t stream) {
  MLR_REQUIRE(table && ids && out, "null pointer");
  MLR_REQUIRE(tokens > 0 && hidden > 0 && vocab > 0, "sizes must be > 0");
  MLR_REQUIRE(dtype == kF32 || dtype == kBF16, "dtype must be 0 (float32) or 1 (bfloat16)");
  if (dtype == kF32)
    embedding_kernel<float><<<tokens, 256, 0, stream>>>(static_cast<const float*>(table), ids, out, hidden, vocab);
  else
    embedding_kernel<bf16><<<tokens, 256, 0, stream>>>(static_cast<const bf16*>(table), ids, out, hidden, vocab);
  MLR_LAUNCH_CHECK();
  return 0;
}

int mlr_rmsnorm(float* x, const void* delta, const float* partial, int slices, const void* weight,
                int weight_is_f32, void* out, int dtype, int rows, int hidden, float eps, hipStream_t stream) {
  MLR_REQUIRE(x && weight && out, "null pointer");
  MLR_REQUIRE(rows > 0 && hidden > 0, "sizes must be > 0");
  MLR_REQUIRE(eps >= 0.f, "eps must be >= 0");
  MLR_REQUIRE(slices >= 0 && slices <= 64 && (slices == 0) == (partial == nullptr), "partial sums and their count come together");
  MLR_REQUIRE(delta == nullptr || partial == nullptr, "one kind of delta at a time");
  MLR_REQUIRE(dtype == kF32 || dtype == kBF16, "dtype must be 0 (float32) or 1 (bfloat16)");
  if (dtype == kF32) {
    MLR_REQUIRE(weight_is_f32, "a float32 engine needs float32 norm weights");
    launch_rmsnorm<float, float>(x, delta, partial, slices, weight, out, rows, hidden, eps, stream);
  } else if (weight_is_f32) {
    launch_rmsnorm<bf16, float>(x, delta, partial, slices, weight, out, rows, hidden, eps, stream);
  } else {
    launch_rmsnorm<bf16, bf16>(x, delta, partial, slices, weight, out, rows, hidden, eps, stream);
  }
  MLR_LAUNCH_CHECK();
  return 0;
}

// x = cap * tanh(x * scale / cap) when cap > 0, else x * scale (float32, in place).
__global__ __launch_bounds__(256) void scale_softcap_kernel(float* __restrict__ x, float scale, float cap, int64_t count) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= count) return;
  const float v = x[i] * scale;
  x[i] = cap > 0.f ? cap * tanhf(v / cap) : v;
}

int mlr_scale_softcap(float* x, float scale, float cap, int64_t count, hipStream_t stream) {
  MLR_REQUIRE(x != nullptr, "null pointer");
  MLR_REQUIRE(count > 0 && cap >= 0.f, "count must be > 0 and the cap >= 0");
  const int64_t blocks = (count + 255) / 256;
  MLR_REQUIRE(blocks < (1ll << 31), "too many elements");
  scale_softcap_kernel<<<static_cast<unsigned>(blocks), 256, 0, stream>>>(x, scale, cap, count);
  MLR_LAUNCH_CHECK();
  return 0;
}

int mlr_add(float* x, const void* delta, int dtype, int64_t count, hipStream_t stream) {
  MLR_REQUIRE(x && delta, "null pointer");
  MLR_REQUIRE(count > 0, "count must be > 0");
  MLR_REQUIRE(dtype == kF32 || dtype == kBF16, "dtype must be 0 (float32) or 1 (bfloat16)");
  const int64_t blocks = (count + 255) / 256;
  MLR_REQUIRE(blocks < (1ll << 31), "too many elements");
  if (dtype == kF32)
    add_kernel<float><<<static_cast<unsigned>(blocks), 256, 0, stream>>>(x, static_cast<const float*>(delta), count);
  else
    add_kernel<bf16><<<static_cast<unsigned>(blocks), 256, 0, stream>>>(x, static_cast<const bf16*>(delta), count);
  MLR_LAUNCH_CHECK();
  return 0;
}

int mlr_gather_rows(const void* src, const int* rows, void* out, int count, int64_t row_bytes, int src_rows,
                    int planes, hipStream_t stream) {
  MLR_REQUIRE(src && rows && out, "null pointer");
  MLR_REQUIRE(count > 0 && src_rows > 0 && planes > 0 && planes < 65536, "sizes must be > 0");
  MLR_REQUIRE(row_bytes > 0 && row_bytes % 4 == 0, "rows must be a multiple of 4 bytes wide");
  gather_rows_kernel<<<dim3(count, planes), 256, 0, stream>>>(static_cast<const uint32_t*>(src), rows,
                                                static_cast<uint32_t*>(out), row_bytes / 4, src_rows);
  MLR_LAUNCH_CHECK();
  return 0;
}

int mlr_silu_mul(const void* gate_up, void* out, int dtype, int rows, int inter, hipStream_t stream) {
  MLR_REQUIRE(gate_up && out, "null pointer");
  MLR_REQUIRE(rows > 0 && inter > 0, "sizes must be > 0");
  MLR_REQUIRE(dtype == kF32 || dtype == kBF16, "dtype must be 0 (float32) or 1 (bfloat16)");
  const int64_t total = static_cast<int64_t>(rows) * inter;
  const int64_t blocks = (total + 255) / 256;
  MLR_REQUIRE(blocks < (1ll << 31), "too many elements");
  if (dtype == kF32)
    silu_mul_kernel<float><<<static_cast<unsigned>(blocks), 256, 0, stream>>>(
        static_cast<const float*>(gate_up), static_cast<float*>(out), rows, inter);
  else
    silu_mul_kernel<bf16><<<static_cast<unsigned>(blocks), 256, 0, stream>>>(
        static_cast<const bf16*>(gate_up), static_cast<bf16*>(out), rows, inter);
  MLR_LAUNCH_CHECK();
  return 0;
}

int mlr_rope_table(const int* positions, const double* inv_freq, float* cos, float* sin, int tokens, int half,
                   hipStream_t stream) {
  MLR_REQUIRE(positions && inv_freq && cos && sin, "null pointer");
  MLR_REQUIRE(tokens > 0 && half > 0, "sizes must be > 0");
  const int64_t total = static_cast<int64_t>(tokens) * half;
  const int64_t blocks = (total + 255) / 256;
  MLR_REQUIRE(blocks < (1ll << 31), "too many elements");
  rope_table_kernel<<<static_cast<unsigned>(blocks), 256, 0, stream>>>(positions, inv_freq, cos, sin, tokens, half);
  MLR_LAUNCH_CHECK();
  return 0;
}

int mlr_rope_kv_write(void* qkv, int dtype, const float* cos, const float* sin, const int* slots,
                      void* key_pages, void* value_pages, int tokens, int heads, int kv_heads, int head_dim,
                      int rotary_dim, int block_size, int num_pages, int write, hipStream_t stream) {
  MLR_REQUIRE(qkv, "null pointer");
  MLR_REQUIRE(tokens > 0 && heads > 0 && kv_heads > 0 && head_dim > 0, "sizes must be > 0");
  MLR_REQUIRE(rotary_dim >= 0 && rotary_dim % 2 == 0 && rotary_dim <= head_dim,
              "rotary_dim must be even and within head_dim");
  MLR_REQUIRE(rotary_dim == 0 || (cos && sin), "rotation needs cos and sin tables");
  MLR_REQUIRE(!write || (slots && key_pages && value_pages && block_size > 0 && num_pages > 0),
              "a cache write needs slots, pages and their sizes");
  MLR_REQUIRE(dtype == kF32 || dtype == kBF16, "dtype must be 0 (float32) or 1 (bfloat16)");
  if (dtype == kF32)
    rope_kv_write_kernel<float><<<tokens, 256, 0, stream>>>(
        static_cast<float*>(qkv), cos, sin, slots, static_cast<float*>(key_pages),
        static_cast<float*>(value_pages), heads, kv_heads, head_dim, rotary_dim, block_size, num_pages, write);
  else if (rotary_dim == head_dim && head_dim % 16 == 0 && reinterpret_cast<uintptr_t>(qkv) % 16 == 0 &&
           reinterpret_cast<uintptr_t>(key_pages) % 16 == 0 && reinterpret_cast<uintptr_t>(cos) % 16 == 0 &&
           reinterpret_cast<uintptr_t>(sin) % 16 == 0)
    rope_kv_write_bf16x8_kernel<<<tokens, 256, 0, stream>>>(
        static_cast<bf16*>(qkv), cos, sin, slots, static_cast<bf16*>(key_pages), static_cast<bf16*>(value_pages), heads,
        kv_heads, head_dim, block_size, num_pages, write);
  else
    rope_kv_write_kernel<bf16><<<tokens, 256, 0, stream>>>(
        static_cast<bf16*>(qkv), cos, sin, slots, static_cast<bf16*>(key_pages),
        static_cast<bf16*>(value_pages), heads, kv_heads, head_dim, rotary_dim, block_size, num_pages, write);
  MLR_LAUNCH_CHECK();
  return 0;
}

int mlr_qkv_finish(const float* partial, int slices, const float* cos, const float* sin, const int* slots,
                   void* key_pages, void* value_pages, void* q_out, int tokens, int heads, int kv_heads, int head_dim,
                   int block_size, int num_pages, int write, hipStream_t stream) {
  MLR_REQUIRE(partial && q_out, "null pointer");
  MLR_REQUIRE(tokens > 0 && tokens <= 65535 && heads > 0 && kv_heads > 0 && heads + 2 * kv_heads <= 65535, "bad sizes");
  MLR_REQUIRE(head_dim > 0 && head_dim % 2 == 0, "head_dim must be even");
  MLR_REQUIRE(slices >= 1 && slices <= 64, "slices must lie within 1..64");
  MLR_REQUIRE((cos == nullptr) == (sin == nullptr), "cos and sin come together");
  MLR_REQUIRE(!write || (slots && key_pages && value_pages && block_size > 0 && num_pages > 0),
              "a cache write needs slots, pages and their sizes");
  qkv_finish_kernel<<<dim3(tokens, heads + 2 * kv_heads), 64, 0, stream>>>(
      partial, slices, cos, sin, write ? slots : nullptr, static_cast<bf16*>(key_pages), static_cast<bf16*>(value_pages),
      static_cast<bf16*>(q_out), tokens, heads, kv_heads, head_dim, block_size, num_pages);
  MLR_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
