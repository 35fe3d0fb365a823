// C interface of the gfx950 kernel library.  Every entry point takes device
// pointers, sizes, element type codes (0: float32, 1: bfloat16) and the HIP
// stream to launch on; it checks its arguments on the host, launches, and
// returns 0, or -1 with a message for mlr_last_error().  Nothing here
// allocates or synchronises.
//
// The reference has one native op, its decode attention
// (csrc/paged_attention_binding.cpp:16-35); everything else below stands where
// it calls PyTorch operators (src/mini_llm_runtime/qwen_model_runner.py).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

extern "C" {

const char* mlr_last_error();
int mlr_version();

// out[t, :] = float(table[ids[t], :]); an id outside [0, vocab) gives a NaN row.
int mlr_embedding(const void* table, int dtype, const int* ids, float* out, int tokens, int hidden,
                  int vocab, hipStream_t stream);

// x (float32 [rows, hidden]) += delta, then out = weight * x * rsqrt(mean(x^2) + eps)
// in `dtype`; weight is float32 when weight_is_f32, else `dtype`.  The delta is
// `delta` ([rows, hidden] in `dtype`), or `slices` float32 partial sums `partial`
// [slices, rows, hidden] added in slice order, or nothing (both null).
int mlr_rmsnorm(float* x, const void* delta, const float* partial, int slices, const void* weight,
                int weight_is_f32, void* out, int dtype, int rows, int hidden, float eps,
                hipStream_t stream);

// x (float32) += delta (dtype), count elements.
int mlr_add(float* x, const void* delta, int dtype, int64_t count, hipStream_t stream);

// x (float32, in place) = x * scale, and, when cap > 0, cap * tanh(that / cap).
int mlr_scale_softcap(float* x, float scale, float cap, int64_t count, hipStream_t stream);

// out[p, k, :] = src[p, rows[k], :] for every plane p of src [planes, src_rows, width];
// rows are `row_bytes` wide (a multiple of 4).
int mlr_gather_rows(const void* src, const int* rows, void* out, int count, int64_t row_bytes,
                    int src_rows, int planes, hipStream_t stream);

// out[m, i] = silu(gate_up[m, i]) * gate_up[m, inter + i].
int mlr_silu_mul(const void* gate_up, void* out, int dtype, int rows, int inter, hipStream_t stream);

// cos/sin [tokens, half] float32 of positions[t] * inv_freq[j], computed in float64.
int mlr_rope_table(const int* positions, const double* inv_freq, float* cos, float* sin, int tokens,
                   int half, hipStream_t stream);

// Rotate q and k of qkv [tokens, (heads + 2 kv_heads) * head_dim] in place (first
// rotary_dim dims of every head, half-split pairs; rotary_dim 0: no rotation) and,
// when `write`, store the rotated k and the raw v at slots[t] of the key pages
// [num_pages, kv_heads, block_size, head_dim] and the value pages
// [num_pages, kv_heads, head_dim, block_size]; a negative slot writes nothing.
int mlr_rope_kv_write(void* qkv, int dtype, const float* cos, const float* sin, const int* slots,
                      void* key_pages, void* value_pages, int tokens, int heads, int kv_heads,
                      int head_dim, int rotary_dim, int block_size, int num_pages, int write,
                      hipStream_t stream);

// The query/key/value product of few tokens that came as `slices` float32 partial sums
// [slice, tokens, (heads + 2 kv_heads) * head_dim] (mlr_gemm_bf16 with slices, the bias in slice
// 0): added up in order, rounded to bfloat16, query and key heads rotated over the whole head
// (cos, sin: [tokens, head_dim / 2], or null), queries to q_out [tokens, heads * head_dim], keys
// and values into their cache slots (`write` 0: none).  bfloat16 only.
int mlr_qkv_finish(const float* partial, int slices, const float* cos, const float* sin, const int* slots,
                   void* key_pages, void* value_pages, void* q_out, int tokens, int heads, int kv_heads, int head_dim,
                   int block_size, int num_pages, int write, hipStream_t stream);

// y[M, N] = x[M, K] * w[N, K]^T (+ bias[N]); x, w in `dtype`; bias float32 when
// bias_is_f32 else `dtype` (null: none); y float32 when out_is_f32 else `dtype`.
// Plain 32-bit FMA arithmetic on every path (no matrix-core rounding).
// With `swiglu` the rows of w come in groups (gate 2j, gate 2j+1, up 2j, up 2j+1),
// there is no bias, n is a multiple of 4 and y[M, N / 2] = silu(gate) * up.
int mlr_gemm_simple(const void* x, const void* w, const void* bias, int bias_is_f32, void* y,
                    int out_is_f32, int swiglu, int dtype, int m, int n, int k, hipStream_t stream);

// The same product in bfloat16 on the matrix cores (float32 accumulation).  Needs
// k % 8 == 0 and 16-byte aligned x and w; any m and n.  With slices > 1 (a value
// mlr_gemm_bf16_slices returned for this shape) y is float32 [slices, m, n]: partial
// sums over slices of k, the bias in slice 0, for the consumer to add up in order.
int mlr_gemm_bf16_slices(int m, int n, int k, int max_slices);
// The kernel mlr_gemm_bf16 chooses for a shape cut into `slices` (its `kernel` argument's numbers).
int mlr_gemm_bf16_kernel(int m, int n, int k, int slices);
// `kernel` 0 lets the shape choose; 16 (streaming, up to 64 tokens), 14 (LDS-tiled, tiles of 32
// tokens x 64 features), 11, 22, 44 (LDS-tiled with 64 x 64, 128 x 128, 256 x 256 tiles), 23, 45 (the
// two larger tiles loaded straight into LDS), 46, 47, 48 (the same with tiles of 256 tokens x 192,
// x 160 and x 320 features), 62 to 68 (64 tokens x 64, 96, ... 256 features straight into LDS, for up to 64
// tokens) force one, for tests and tuning.
// Any `slices` within
// 1..64 is accepted with a float32 [slices, m, n] output.
// row_sumsq (null: none): the rows of x still owe their normalisation (mlr_gemm_residual_bf16 made
// them): float32 [m, sumsq_parts] partial sums of squares of every row of the residual stream; the
// sums of row i are scaled by rsqrt(sum_p row_sumsq[i, p] / k + norm_eps) before the bias.
int mlr_gemm_bf16(const void* x, const void* w, const void* bias, int bias_is_f32, void* y,
                  int out_is_f32, int swiglu, int slices, int kernel, int m, int n, int k,
                  const float* row_sumsq, int sumsq_parts, float norm_eps, hipStream_t stream);

// A product that finishes the residual stream (gemm_stream.hip): y = a w^T (+ bias), a [m, k] and w
// [n, k] bfloat16; then, every workgroup for its own columns of all rows, stream[m, n] (float32, in
// place) += y, h[m, n] (bfloat16) = norm_weight * stream (the next norm's weight, float32 or
// bfloat16; its division by the root mean square is left to the consumer), and sumsq[m, parts] =
// this workgroup's share of every row's sum of squares of the new stream, parts =
// mlr_gemm_residual_parts(m, n).  One kernel where a product cut along k needs a second one to add
// the slices up, to add the residual and to norm; it pays while a workgroup can afford to read all
// m rows of a (up to 64 tokens, n a multiple of 4, k of 8).
int mlr_gemm_residual_parts(int m, int n);
int mlr_gemm_residual_bf16(const void* a, const void* w, const void* bias, int bias_is_f32, float* stream,
                           const void* norm_weight, int norm_weight_is_f32, void* h, float* sumsq, int m, int n,
                           int k, hipStream_t stream_handle);

// The query/key/value product fused with bias, rotation (cos, sin: [m, head_dim / 2] float32,
// or null), the queries' store to q_out [m, heads * head_dim] and the keys' and values' store
// into their cache slots (`write` 0: no cache write).  kernel: 0 chooses; 16 the row-splitting
// kernel (up to 64 tokens); 8 its variant with 8 weight rows a workgroup (up to 8 tokens); 11,
// 22, 44 the tiled kernels as in mlr_gemm_bf16.  row_sumsq, sumsq_parts, norm_eps as there.
int mlr_qkv_rope_write_bf16(const void* x, const void* w, const void* bias, int bias_is_f32, const float* cos,
                            const float* sin, const int* slots, void* key_pages, void* value_pages, void* q_out,
                            int m, int k, int heads, int kv_heads, int head_dim, int block_size, int num_pages,
                            int write, int kernel, const float* row_sumsq, int sumsq_parts, float norm_eps,
                            hipStream_t stream);

// Products of up to 16 tokens that make their own activations (gemm_fused.hip).
// Norm prologue: h = RMSNorm(x_in + delta) * norm_weight with the delta a bfloat16 [m, k]
// tensor, or `slices_in` float32 partial sums [slices_in, m, k] added in order, or nothing;
// x_out (another buffer than x_in; null when nothing is added) receives x_in + delta.  Then
// y = h w^T with the epilogues of mlr_gemm_bf16 (bias, float32 output, SwiGLU), or the
// query/key/value epilogue of mlr_qkv_rope_write_bf16.  k a multiple of 8, at most 2048.
// row_blocks: 0 chooses how many blocks of 16 features a workgroup owns, or 1, 2.
int mlr_gemm_norm_fused_bf16(const float* x_in, float* x_out, const void* delta, const float* partial, int slices_in,
                             const void* norm_weight, int norm_weight_is_f32, float eps, const void* w,
                             const void* bias, int bias_is_f32, void* y, int out_is_f32, int swiglu, int row_blocks,
                             int m, int n, int k, hipStream_t stream);
int mlr_qkv_norm_fused_bf16(const float* x_in, float* x_out, const void* delta, const float* partial, int slices_in,
                            const void* norm_weight, int norm_weight_is_f32, float eps, const void* w,
                            const void* bias, int bias_is_f32, const float* cos, const float* sin, const int* slots,
                            void* key_pages, void* value_pages, void* q_out, int m, int k, int heads, int kv_heads,
                            int head_dim, int block_size, int num_pages, int write, hipStream_t stream);
// Merge prologue: the activations are the decode attention's output of m single-token entries,
// merged here from its unmerged partitions (`attn_partial`, as mlr_attention_decode with
// merge 0 leaves them; part, splits, window as given there).  y = attended w^T (+ bias), k =
// heads * head_dim; with slices > 1 y is float32 [slices, m, n] partial sums.
int mlr_gemm_merge_fused_bf16(const float* attn_partial, const int* context_lens, int heads, int head_dim, int window,
                              int part, int splits, const void* w, const void* bias, int bias_is_f32, void* y,
                              int out_is_f32, int slices, int m, int n, hipStream_t stream);

// Attention of every token over its request's pages: token t (entry
// token_entry[t], absolute position positions[t]) sees the keys
// max(0, p - window + 1) .. p of its entry's block table row (window 0: all).
// q is read from q[t * q_stride + head * head_dim + i]; out is [tokens, heads * head_dim];
// pages are laid out as for mlr_rope_kv_write.
// A page id outside [0, num_pages) among the visible keys gives a NaN row.
int mlr_paged_attention_simple(const void* q, int64_t q_stride, const void* key_pages,
                               const void* value_pages, const int* block_table, int table_width,
                               const int* token_entry, const int* positions, void* out, int dtype,
                               int tokens, int entries, int heads, int kv_heads, int head_dim,
                               int block_size, int num_pages, float scale, int window,
                               hipStream_t stream);

// tokens[k] = argmax(logits[k, :]) (first maximum), or, where temperature[k] > 0,
// the first index whose cumulative exp((x - max) / temperature) exceeds
// uniform[k] * total.  temperature and uniform may be null (all greedy).  `scratch`
// holds mlr_sample_scratch(rows, vocab) floats.
int64_t mlr_sample_scratch(int rows, int vocab);
int mlr_sample(const float* logits, const float* temperature, const float* uniform, int* tokens,
               float* scratch, int rows, int vocab, hipStream_t stream);

// mlr_sample without a scratch argument and without any allocation: the segment results live
// in an array inside the library (256 KiB per GPU, held until the process ends).  It has no
// counterpart in the reference; it is for callers that cannot allocate device memory: code
// under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  Same
// kernels and same results as mlr_sample.  rows * ceil(vocab / 4096) * 3 must not exceed
// mlr_sample_static_capacity() floats, else -1 with a message.  The stream's device must be the
// current device.  All calls on one GPU share that GPU's array: calls that overlap there (two
// streams, two threads) race, so order them.  The first call on a device looks up the array's
// address (no allocation); make it outside a graph capture.
int64_t mlr_sample_static_capacity();
int mlr_sample_static(const float* logits, const float* temperature, const float* uniform, int* tokens,
                      int rows, int vocab, hipStream_t stream);

}  // extern "C"
