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

// out[t, :] = table[ids[t], :], as float32 (out_is_f32) or in the table's type; an id outside
// [0, vocab) gives a NaN row.
int mlr_embedding(const void* table, int dtype, const int* ids, void* out, int out_is_f32, int tokens, int hidden,
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
// x += delta[0] + delta[1] + ... for float32 partial sums delta [slices, count], added in order.
int mlr_add_slices(float* x, const float* delta, int slices, int64_t count, hipStream_t stream);

// x (float32, in place) = x * scale, and, when cap > 0, cap * tanh(that / cap).
int mlr_scale_softcap(float* x, float scale, float cap, int64_t count, hipStream_t stream);

// out[p, k, :] = src[p, rows[k], :] for every plane p of src [planes, src_rows, width];
// rows are `row_bytes` wide (a multiple of 4).
int mlr_gather_rows(const void* src, const int* rows, void* out, int count, int64_t row_bytes,
                    int src_rows, int planes, hipStream_t stream);

// out[m, i] = silu(gate_up[m, i]) * gate_up[m, inter + i].
int mlr_silu_mul(const void* gate_up, void* out, int dtype, int rows, int inter, hipStream_t stream);

// cos/sin [tokens, half] float32 of positions[t] * inv_freq[j], times `amplitude`, computed in float64.
int mlr_rope_table(const int* positions, const double* inv_freq, float* cos, float* sin, int tokens,
                   int half, float amplitude, hipStream_t stream);

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
// `swiglu` 2 and 3 are element-wise activations instead: the squared ReLU max(v, 0)^2 and the
// sigmoid, applied after the bias, any n.  `multiply` ([M, N] in `dtype`, or null; not with the
// pairing) is multiplied into the activated sums: y = act(x w^T + bias) * multiply.
int mlr_gemm_simple(const void* x, const void* w, const void* bias, int bias_is_f32, void* y,
                    int out_is_f32, int swiglu, int dtype, int m, int n, int k, const void* multiply,
                    const int* multiply_rows, float glu_limit, float glu_alpha, hipStream_t stream);

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
                  const float* row_sumsq, int sumsq_parts, float norm_eps, const void* multiply,
                  const int* multiply_rows, float glu_limit, float glu_alpha, hipStream_t stream);

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
// max(0, p - window + 1) .. p of its entry's block table row (window 0: all), or, with a
// chunked mask (chunk > 0, window 0), the keys p - p % chunk .. p.
// q is read from q[t * q_stride + head * head_dim + i]; out is [tokens, heads * head_dim];
// pages are laid out as for mlr_rope_kv_write.
// A page id outside [0, num_pages) among the visible keys gives a NaN row.
// sinks (float32 [heads], or null): the softmax's denominator also holds exp(sinks[head]).
// pool > 0 (with a window): beside its window a query also sees pooled entries, one key and value for every
// run of `pool` positions whose last position is <= p - window, read from pages of their own (same layout,
// `block_size` entries a page, entry b of a request at pooled_table[entry][b / block_size]) in the same softmax.
int mlr_paged_attention_simple(const void* q, int64_t q_stride, const void* key_pages,
                               const void* value_pages, const int* block_table, int table_width,
                               const int* token_entry, const int* positions, void* out, int dtype,
                               int tokens, int entries, int heads, int kv_heads, int head_dim,
                               int block_size, int num_pages, float scale, int window, int chunk,
                               const float* sinks, const void* pooled_keys, const void* pooled_values,
                               const int* pooled_table, int pooled_width, int pooled_pages, int pool,
                               const float* score_bias, hipStream_t stream);

// x (float32 [rows, hidden], in place) += weight * y * rsqrt(mean(y^2) + eps), y [rows, hidden] float32
// or `dtype`, or `slices` float32 partial sums [slices, rows, hidden].  Then mode 1: out = next_weight * x *
// rsqrt(mean(x^2) + next_eps), mode 2: out = x, both in `dtype`; mode 0: no output.
int mlr_add_normed(float* x, const void* y, int y_is_f32, int slices, const void* weight, int weight_is_f32, float eps,
                   const void* next_weight, int next_is_f32, float next_eps, int mode, void* out, int dtype, int rows,
                   int hidden, hipStream_t stream);

// out[m, i] = g * sigmoid(alpha * g) * (u + 1), g = min(sums[m, i], limit), u = clamp(sums[m, inter + i],
// -limit, limit).
int mlr_glu_clamped(const void* sums, int sums_is_f32, void* out, int dtype, int rows, int inter, float limit,
                    float alpha, hipStream_t stream);

// What a latent-attention layer does between its input product and the attention kernels (see mixers.hip).
int mlr_latent_prepare(const float* projected, int width, void* q_plain, void* q_latent, float* gate, const float* cos,
                       const float* sin, int rotary_dims, const void* norm_weight, int weight_is_f32, float eps,
                       const int* slots, void* key_pages, void* value_pages, int dtype, int tokens, int heads, int dim,
                       int rot, int rank, int kernel_dim, int block_size, int num_pages, int own_cache, int gated,
                       const float* queries, int q_width, hipStream_t stream);

// out[t * out_row + h * out_stride + j] = row_scale[t, h] * sum_i x[t * in_row + h * in_stride + i] * w[h, j, i].
int mlr_heads_linear(const void* x, int64_t in_row, int in_stride, const void* w, void* out, int64_t out_row,
                     int out_stride, const float* row_scale, int dtype, int tokens, int heads, int n, int k,
                     hipStream_t stream);

// Retention over every entry's tokens in order, from and to rows of the state banks (see mixers.hip).
// chunked: 64 tokens at a time on the matrix cores in true 32-bit (for entries of many tokens) instead of
// token by token; q and k of `projected` ([total_tokens, width]) are then rotated and scaled in place first,
// and `scratch` holds mlr_retention_scratch floats (what every chunk adds to the state).
int64_t mlr_retention_scratch(int total_tokens, int entries, int heads, int dim, int vdim);
int mlr_retention_scan(float* projected, int width, float* state, int state_rows, const int* read_rows,
                       const int* write_rows, const int* cu_q, const int* q_starts, const float* decay,
                       const float* cos, const float* sin, int rotary_dims, float key_scale, float* out, int entries,
                       int heads, int dim, int vdim, int chunked, int total_tokens, float* scratch, int64_t scratch_floats,
                       hipStream_t stream);

// out[t * out_row + h * vdim + :] = retained[t, h, :] / rms(retained[t, h, :]) * norm_weight * act(projected[t,
// gate_offset + h * vdim + :]) * out_scale; norm_weight [vdim] is shared by the heads, or with `weight_per_head`
// [heads * vdim] (null: none); act is silu (gate_kind 0) or the sigmoid (1).
int mlr_retention_gate(const float* retained, const float* projected, int width, int gate_offset, void* out, int dtype,
                       int tokens, int heads, int vdim, float eps, const void* norm_weight, int weight_is_f32,
                       float out_scale, int64_t out_row, int weight_per_head, int gate_kind, hipStream_t stream);

// out[t] = (add_input ? h[t] : 0) + a causal convolution over the entry's inputs of `taps` taps per channel (weight
// [width, taps], the last tap on the token itself); the taps - 1 inputs before a step are carried in `state`
// [state_rows, taps - 1, width] float32 (row read_rows[entry], zeros where q_starts[entry] == 0) and the newest are
// left in row write_rows[entry].
int mlr_short_conv(const void* h, const void* weight, int weight_is_f32, float* state, int state_rows,
                   const int* read_rows, const int* write_rows, const int* token_entry, const int* cu_q,
                   const int* q_starts, void* out, int dtype, int tokens, int width, int taps, int add_input,
                   hipStream_t stream);

// projected [tokens, width] float32: q (heads * dim), k (kv_heads * dim), v (kv_heads * vdim), (gated) heads gate
// logits.  q and k normed over their whole projection (weights q_norm, k_norm or null), rotated (two halves of the
// first rotary_dim dims of a head), q times head_scale[head] into q_out [tokens, heads * head_dim], k and v into the
// pages at slots[t] (heads padded with zeros to head_dim), gate = sigmoid(logits) float32 [tokens, heads].
int mlr_qk_norm_rope_write(const float* projected, int width, const void* q_norm, const void* k_norm, int weight_is_f32,
                           float eps, const float* head_scale, const float* cos_t, const float* sin_t, int rotary_dim,
                           const int* slots, void* key_pages, void* value_pages, void* q_out, float* gate, int dtype,
                           int tokens, int heads, int kv_heads, int dim, int vdim, int head_dim, int block_size,
                           int num_pages, int gated, hipStream_t stream);

// Tokens with pooled_slots[t] >= 0 complete a run of `pool` positions: the means of the run's keys and values, read
// from the token pages through the block table, go to that slot of the pooled pages.
int mlr_pool_kv_write(const void* key_pages, const void* value_pages, const int* block_table, int table_width,
                      int num_pages, const int* token_entry, const int* positions, const int* pooled_slots,
                      void* pooled_keys, void* pooled_values, int pooled_pages, int dtype, int tokens, int kv_heads,
                      int head_dim, int block_size, int pool, hipStream_t stream);

// The pooled entries' share of a softmax that the matrix-core attention kernels finish (their `extra`): for every
// token and head, over the entries j < (position - window + 1) / pool of the entry's pooled pages, share[t, h] =
// [numerator (head_dim floats), maximum of score * scale * log2(e), denominator]; bfloat16 queries and pages.
int mlr_pooled_share(const void* q, int64_t q_stride, const void* pooled_keys, const void* pooled_values,
                     const int* pooled_table, int table_width, int pooled_pages, const int* token_entry,
                     const int* positions, float* share, int tokens, int heads, int kv_heads, int head_dim,
                     int block_size, float scale, int window, int pool, hipStream_t stream);

// out[t * out_row + head * out_dim + j] = attended[t, head * head_dim + j] * gate[t, head] * scale, j < out_dim.
int mlr_scale_heads(const void* attended, const float* gate, void* out, int64_t out_row, int dtype, int tokens, int heads,
                    int head_dim, int out_dim, float scale, hipStream_t stream);

// Linear attention with a decay per key channel and token: decay = sigmoid(W2 low + bias)^(1 / tau) with `low` the
// `rank` columns of `projected` from low_offset on (with `runs`, left in `decay` [tokens, heads * dim]); S = diag(decay) S + k v^T,
// o = S^T (q * q_scale) per head; q, k, v are the leading columns of `projected` (float32).  State rows as for
// mlr_retention_scan.  `runs` (or null: every entry token by token in one wavefront per 16 value columns): scratch of
// mlr_gla_runs(tokens, entries) * heads * dim * vdim floats, `run_decay` of mlr_gla_runs(...) * heads * dim; entries are
// then cut into runs of 64 tokens that are walked in parallel (two walks and a carry between them).
int mlr_gla_runs(int tokens, int entries);
int mlr_gla_scan(const float* projected, int width, int low_offset, int rank, const void* decay_weight,
                 const void* decay_bias, int weight_is_f32, int bias_is_f32, float tau, float* decay, float* state,
                 int state_rows, const int* read_rows, const int* write_rows, const int* cu_q, const int* q_starts,
                 float q_scale, float* out, int entries, int heads, int dim, int vdim, int tokens, float* runs,
                 float* run_decay, hipStream_t stream);

// Several residual streams, per-head norms before the cache, a matrix memory with exponential gates
// (stream_mixers.hip; the kernels' comments say what each computes).
int mlr_streams_fill(const float* x, float* out, int tokens, int width, int streams, hipStream_t stream);
int mlr_streams_step(float* x, int streams, int tokens, int width, const int* rows, int out_rows, const void* y,
                     int y_is_f32, int slices, const float* mix, const float* out_w, const float* in_w,
                     const void* norm_w, int norm_is_f32, float eps, void* h_out, float* sum_out, int dtype,
                     hipStream_t stream);
int mlr_head_norm_rope_write(const float* projected, int width, void* q_out, float* gate, const float* cos,
                             const float* sin, int rotary_dims, float eps, const int* slots, void* key_pages,
                             void* value_pages, float* v_keep, const float* v_first, const float* lambda, int dtype,
                             int tokens, int heads, int kv_heads, int dim, int vdim, int kernel_dim, int block_size,
                             int num_pages, hipStream_t stream);
int mlr_matrix_memory_scan(const float* projected, int width, int q_off, int k_off, int v_off, int i_off, int f_off,
                           float* state, int state_rows, const int* read_rows, const int* write_rows, const int* cu_q,
                           const int* q_starts, float cap, float q_scale, float* out, int entries, int heads, int dim,
                           int vdim, int tokens, float* runs, float* run_gates, hipStream_t stream);
// runs (or null: every entry is walked whole): float32 [mlr_matrix_memory_runs(tokens, entries), heads, dim * vdim + dim
// + 1] and run_gates [that many, heads, 2] of scratch; entries are then walked in runs of 64 tokens, all at once.
int mlr_matrix_memory_runs(int tokens, int entries);

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

// Routed experts (moe.hip).  mlr_moe_route: per token, from the router's float32 logits [tokens,
// experts]: s = sigmoid(z) (score_kind 0) or softmax(z) over all experts (1), choice scores c = s + correction (float32 [experts], or null); the
// expert axis is cut into `groups` contiguous blocks of experts / groups; block score = top-2 sum of
// c; eligible are the experts of the `keep` highest blocks; ids [tokens, top] = arg-top-`top` of c over
// the eligible (ties to the lower index), weights [tokens, top] = s[id] * scale, with `normalise` divided by the
// sum of a token's chosen s (+ 1e-20) first.
int mlr_moe_route(const float* logits, const float* correction, int* ids, float* weights, int tokens, int experts,
                  int top, int groups, int keep, float scale, int score_kind, int normalise, hipStream_t stream);
// out[j, t, :] = weights[t, j] * h[t, :] where ids[t, j] >= first: experts without matrices that hand their input on.
int mlr_moe_identity(const void* h, const int* ids, const float* weights, float* out, int dtype, int tokens, int top,
                     int hidden, int first, hipStream_t stream);
// The (token, choice) pairs p = token * top + choice sorted by expert: sorted [pairs], offsets
// [experts + 1], tiles [max_tiles, 2] = (expert, first row of `sorted`) with up to
// mlr_moe_tile_rows(big) rows each (16, or 64 with `big`), unused tiles (-1, 0).  max_tiles >=
// mlr_moe_max_tiles(pairs, experts, big).
int mlr_moe_tile_rows(int big);
int mlr_moe_max_tiles(int pairs, int experts, int big);
int mlr_moe_align(const int* ids, int pairs, int experts, int big, int max_tiles, int* sorted, int* offsets,
                  int* tiles, hipStream_t stream);
// One grouped product over those tiles; w is [experts, n, k] in `dtype` (0 float32, 1 bfloat16).
// up 1: a = h [tokens, k]; out [pairs, n] in `dtype`, row r = act(h[sorted[r] / top] w[e]^T), act 0
// none, 2 squared ReLU, 3 sigmoid.  up 0: a = the rows of the first product [pairs, k]; out float32
// [top, tokens, n], out[choice, token] = pair_weights[p] * (a[r] w[e]^T).  mfma 1 and 2: on the matrix
// cores (bfloat16, k % 8 == 0; 1 streams tiles of 16 rows, 2 runs tiles of 64 rows through LDS and
// needs n % 8 == 0), 0: plain 32-bit FMA arithmetic (tiles of 16 rows).
int mlr_moe_gemm(const void* a, const void* w, const int* sorted, const int* offsets, const int* tiles,
                 const float* pair_weights, void* out, int up, int dtype, int mfma, int max_tiles, int tokens, int top,
                 int n, int k, int act, hipStream_t stream);

}  // extern "C"
