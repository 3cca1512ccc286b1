// Kernels of mixers that run side by side on one input: a short causal convolution with carried
// inputs, queries and keys normed over their whole projection, rotated and stored, pooled entries of
// the key/value cache, a gate per head, and linear attention with a decay per key channel and token.
#include "api.h"
#include "common.h"

namespace mlr {
namespace {

// out[t, c] = h[t, c] + sum_j w[c, j] * in(t - (taps - 1) + j), in() = the entry's inputs in order: those
// of this step, before them the `taps - 1` inputs that the state row read_rows[entry] carries
// ([rows, taps - 1, width] float32, the oldest first; zeros where the entry starts its request or the
// request is shorter).  The entry's last token leaves the newest taps - 1 inputs in row write_rows[entry].
// Sums in float32, one rounding.  A workgroup per token, threads over the channels.
template <typename T>
__global__ __launch_bounds__(256) void short_conv_kernel(const T* __restrict__ h, const void* __restrict__ weight,
                                                         int weight_is_f32, float* __restrict__ state,
                                                         const int* __restrict__ read_rows,
                                                         const int* __restrict__ write_rows,
                                                         const int* __restrict__ token_entry,
                                                         const int* __restrict__ cu_q, const int* __restrict__ q_starts,
                                                         T* __restrict__ out, int width, int taps, int add_input) {
  const int64_t t = blockIdx.x;
  const int entry = token_entry[t];
  const int first = cu_q[entry];
  const int end = cu_q[entry + 1];
  const int i = static_cast<int>(t) - first;  // place among the step's tokens of the entry
  const int carried = taps - 1;
  const bool fresh = q_starts[entry] == 0;
  const float* old = state + static_cast<int64_t>(read_rows[entry]) * carried * width;
  auto input = [&](int idx, int c) -> float {  // idx counts from the step's first token of the entry
    if (idx >= 0) return to_f32(h[(static_cast<int64_t>(first) + idx) * width + c]);
    if (fresh) return 0.f;
    return old[static_cast<int64_t>(carried + idx) * width + c];
  };
  for (int c = threadIdx.x; c < width; c += 256) {
    float acc = add_input ? to_f32(h[t * width + c]) : 0.f;
    for (int j = 0; j < taps; ++j)
      acc = fmaf(load_as_f32(weight, static_cast<int64_t>(c) * taps + j, weight_is_f32), input(i - carried + j, c), acc);
    out[t * width + c] = from_f32<T>(acc);
  }
  if (static_cast<int>(t) == end - 1 && carried > 0) {
    const int n = end - first;
    float* dst = state + static_cast<int64_t>(write_rows[entry]) * carried * width;
    for (int c = threadIdx.x; c < width; c += 256)
      for (int s = 0; s < carried; ++s) dst[static_cast<int64_t>(s) * width + c] = input(n - carried + s, c);
  }
}

// One token's projected row p[t] (float32): q (heads * dim), k (kv_heads * dim), v (kv_heads * vdim),
// then (gated) one gate logit per head.
//  * q and k are each divided by the root mean square over their WHOLE projection and multiplied by a
//    weight of that size (q_norm, k_norm; null: no norm),
//  * the first `rdims` dims of every head turn in two halves (pair j, j + rdims / 2) by cos/sin[t],
//  * q times head_scale[head] (null: 1) goes to q_out [tokens, heads * D], k and v to slot[t] of the key pages
//    [page, kv_head, offset, D] and the value pages [page, kv_head, D, offset]; dims beyond dim / vdim are
//    zeros; a negative slot stores nothing,
//  * gate[t, head] = sigmoid(logit), float32.
// Everything in float32, one rounding.
template <typename T>
__global__ __launch_bounds__(256) void qk_norm_rope_write_kernel(
    const float* __restrict__ p, int width, const void* __restrict__ q_norm, const void* __restrict__ k_norm,
    int weight_is_f32, float eps, const float* __restrict__ head_scale, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, int rdims, const int* __restrict__ slots, T* __restrict__ key_pages,
    T* __restrict__ value_pages, T* __restrict__ q_out, float* __restrict__ gate, int heads, int kv_heads, int dim,
    int vdim, int D, int block_size, int num_pages, int gated) {
  __shared__ float scratch[16];
  const int64_t t = blockIdx.x;
  const float* q = p + t * width;
  const float* k = q + heads * dim;
  const float* v = k + kv_heads * dim;
  const int half = rdims / 2;
  const float* cs = cos_t ? cos_t + t * half : nullptr;
  const float* sn = sin_t ? sin_t + t * half : nullptr;
  float q_inv = 1.f, k_inv = 1.f;
  if (q_norm != nullptr) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < heads * dim; i += 256) ss += q[i] * q[i];
    q_inv = 1.0f / sqrtf(block_sum(ss, scratch) / static_cast<float>(heads * dim) + eps);
  }
  if (k_norm != nullptr) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < kv_heads * dim; i += 256) ss += k[i] * k[i];
    k_inv = 1.0f / sqrtf(block_sum(ss, scratch) / static_cast<float>(kv_heads * dim) + eps);
  }
  // dim j of head `head` of a normed, rotated projection
  auto turned = [&](const float* part, const void* w, float inv, int head, int j) -> float {
    const int at = head * dim + j;
    auto normed = [&](int idx) { return w ? (part[idx] * inv) * load_as_f32(w, idx, weight_is_f32) : part[idx]; };
    if (j >= rdims || cs == nullptr) return normed(at);
    return j < half ? normed(at) * cs[j] - normed(at + half) * sn[j]
                    : normed(at) * cs[j - half] + normed(at - half) * sn[j - half];
  };
  for (int i = threadIdx.x; i < heads * D; i += 256) {
    const int hd = i / D;
    const int j = i - hd * D;
    float val = 0.f;
    if (j < dim) {
      val = turned(q, q_norm, q_inv, hd, j);
      if (head_scale != nullptr) val *= head_scale[hd];
    }
    q_out[t * heads * D + i] = from_f32<T>(val);
  }
  const int slot = slots[t];
  if (slot >= 0) {
    const int page = slot / block_size;
    const int off = slot - page * block_size;
    if (page < num_pages) {
      for (int i = threadIdx.x; i < kv_heads * D; i += 256) {
        const int g = i / D;
        const int j = i - g * D;
        const int64_t head_base = (static_cast<int64_t>(page) * kv_heads + g) * block_size * D;
        key_pages[head_base + static_cast<int64_t>(off) * D + j] = from_f32<T>(j < dim ? turned(k, k_norm, k_inv, g, j) : 0.f);
        value_pages[head_base + static_cast<int64_t>(j) * block_size + off] = from_f32<T>(j < vdim ? v[g * vdim + j] : 0.f);
      }
    }
  }
  if (gated) {
    const float* logits = v + kv_heads * vdim;
    for (int hd = threadIdx.x; hd < heads; hd += 256) gate[t * heads + hd] = 1.0f / (1.0f + expf(-logits[hd]));
  }
}

// A token that completes a run of `pool` positions (pooled_slots[t] >= 0; its position p is the run's
// last) stores the means of the run's keys and of its values, as the token pages hold them, at that
// slot of the pooled pages (same layouts).  Sums in float32: the run's positions in four quarters, each summed in
// the order of its positions by a wavefront of its own, then the quarters in order.  Grid (tokens, kv_heads).
template <typename T>
__global__ __launch_bounds__(256) void pool_kv_write_kernel(const T* __restrict__ key_pages,
                                                           const T* __restrict__ value_pages,
                                                           const int* __restrict__ block_table, int table_width,
                                                           int num_pages, const int* __restrict__ token_entry,
                                                           const int* __restrict__ positions,
                                                           const int* __restrict__ pooled_slots,
                                                           T* __restrict__ pooled_keys, T* __restrict__ pooled_values,
                                                           int pooled_pages, int kv_heads, int D, int block_size,
                                                           int pool) {
  const int t = blockIdx.x;
  const int slot = pooled_slots[t];
  if (slot < 0) return;
  const int g = blockIdx.y;
  const int p = positions[t];
  const int* table = block_table + static_cast<int64_t>(token_entry[t]) * table_width;
  const int dst_page = slot / block_size;
  const int dst_off = slot - dst_page * block_size;
  if (dst_page >= pooled_pages || p - pool + 1 < 0) return;
  const float inv = 1.0f / static_cast<float>(pool);
  const int64_t dst_base = (static_cast<int64_t>(dst_page) * kv_heads + g) * block_size * D;
  __shared__ float part_k[4][64], part_v[4][64];
  __shared__ int part_gone[4];
  const int lane = threadIdx.x % 64;
  const int quarter = threadIdx.x / 64;
  const int each = (pool + 3) / 4;
  const int j_first = p - pool + 1 + quarter * each;
  const int j_last = min(p, j_first + each - 1);
  for (int i0 = 0; i0 < D; i0 += 64) {
    const int i = min(i0 + lane, D - 1);
    float ks = 0.f, vs = 0.f;
    bool gone = false;
    // (no early exit: the loads of several positions are then on their way together)
#pragma unroll 8
    for (int j = j_first; j <= j_last; ++j) {
      const int logical = j / block_size;
      const int page = logical < table_width ? table[logical] : -1;
      const bool here = page >= 0 && page < num_pages;
      gone = gone || !here;
      const int off = j - logical * block_size;
      const int64_t head_base = (static_cast<int64_t>(here ? page : 0) * kv_heads + g) * block_size * D;
      ks += to_f32(key_pages[head_base + static_cast<int64_t>(off) * D + i]);
      vs += to_f32(value_pages[head_base + static_cast<int64_t>(i) * block_size + off]);
    }
    __syncthreads();  // the dims before are done with
    part_k[quarter][lane] = ks;
    part_v[quarter][lane] = vs;
    if (lane == 0) part_gone[quarter] = gone;
    __syncthreads();
    if (quarter == 0 && i0 + lane < D) {
      ks = ((part_k[0][lane] + part_k[1][lane]) + part_k[2][lane]) + part_k[3][lane];
      vs = ((part_v[0][lane] + part_v[1][lane]) + part_v[2][lane]) + part_v[3][lane];
      // a run whose tokens are gone cannot be pooled: show it
      if (part_gone[0] || part_gone[1] || part_gone[2] || part_gone[3]) ks = vs = NAN;
      pooled_keys[dst_base + static_cast<int64_t>(dst_off) * D + i] = from_f32<T>(ks * inv);
      pooled_values[dst_base + static_cast<int64_t>(i) * block_size + dst_off] = from_f32<T>(vs * inv);
    }
  }
}

// The pooled entries' share of a softmax that another kernel finishes: for token t (entry token_entry[t], position
// p) and head h, over the entries j < (p - window + 1) / pool of the entry's pooled pages (none if that is not
// positive): s_j = q . k_j * scale * log2(e), m = max s_j, l = sum 2^(s_j - m), a = sum 2^(s_j - m) v_j, left as
// share[t, h] = [a (D floats), m, l] (m = -infinity, l = 0, a = 0 without entries).  q is bfloat16 [tokens,
// q_stride], pages as everywhere ([page, kv head, offset, D] keys, [page, kv head, D, offset] values).  One
// wavefront per (token, head): a lane takes every 64th entry's score, then every 64th dim of the values; 64
// entries at a time with a running maximum.  A missing page among the entries poisons the share.
__global__ __launch_bounds__(64) void pooled_share_kernel(const bf16* __restrict__ q, int64_t q_stride,
                                                          const bf16* __restrict__ key_pages,
                                                          const bf16* __restrict__ value_pages,
                                                          const int* __restrict__ table, int table_width, int num_pages,
                                                          const int* __restrict__ token_entry,
                                                          const int* __restrict__ positions, float* __restrict__ share,
                                                          int heads, int kv_heads, int D, int block_size, float scale2,
                                                          int window, int pool) {
  extern __shared__ float pooled_lds[];
  float* qs = pooled_lds;      // D
  float* ws = pooled_lds + D;  // 64 weights, then 64 page offsets (as ints)
  int* where = reinterpret_cast<int*>(ws + 64);
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y;
  const int lane = threadIdx.x;
  const int kvh = h / (heads / kv_heads);
  const int p = positions[t];
  const int count = p - window + 1 > 0 ? (p - window + 1) / pool : 0;
  float* dst = share + (t * heads + h) * (D + 2);
  constexpr int kMaxPerLane = 4;  // head sizes up to 256
  float acc[kMaxPerLane] = {0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  bool bad = false;
  if (count > 0) {
    for (int d = lane; d < D; d += 64) qs[d] = to_f32(q[t * q_stride + static_cast<int64_t>(h) * D + d]);
    const int* row = table + static_cast<int64_t>(token_entry[t]) * table_width;
    for (int j0 = 0; j0 < count; j0 += 64) {
      __syncthreads();  // qs is written; the batch before is done with
      const int j = j0 + lane;
      float s = -INFINITY;
      int at = -1;
      if (j < count) {
        const int logical = j / block_size;
        const int page = logical < table_width ? row[logical] : -1;
        if (page < 0 || page >= num_pages) {
          bad = true;
        } else {
          at = (page * kv_heads + kvh) * block_size + (j - logical * block_size);
          const bf16* k = key_pages + static_cast<int64_t>(at) * D;
          float dot = 0.f;
          if (D % 8 == 0) {  // rows of whole 16-byte pieces (pages are 16-byte aligned)
            for (int d = 0; d < D; d += 8) {
              const uint4 piece = *reinterpret_cast<const uint4*>(k + d);
              const uint32_t words[4] = {piece.x, piece.y, piece.z, piece.w};
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                dot = fmaf(qs[d + 2 * j], __uint_as_float(words[j] << 16), dot);
                dot = fmaf(qs[d + 2 * j + 1], __uint_as_float(words[j] & 0xffff0000u), dot);
              }
            }
          } else {
            for (int d = 0; d < D; ++d) dot = fmaf(qs[d], to_f32(k[d]), dot);
          }
          s = dot * scale2;
        }
      }
      const float m_new = fmaxf(m, wave_max(s));
      const float keep = (m == -INFINITY) ? 0.f : exp2f(m - m_new);
      const float w = (s == -INFINITY) ? 0.f : exp2f(s - m_new);
      l = l * keep + wave_sum(w);
      m = m_new;
      ws[lane] = w;
      where[lane] = at;
      __syncthreads();
      const int n = min(64, count - j0);
#pragma unroll
      for (int i = 0; i < kMaxPerLane; ++i) {
        const int d = lane + 64 * i;
        if (d >= D) break;
        float sum = acc[i] * keep;
        for (int u = 0; u < n; ++u) {
          const int src = where[u];
          if (src < 0) continue;
          // value pages are [page, kv head, D, offset]: `src` counts (page, kv head, offset)
          const int head_base = src / block_size;
          const int off = src - head_base * block_size;
          sum = fmaf(ws[u], to_f32(value_pages[(static_cast<int64_t>(head_base) * D + d) * block_size + off]), sum);
        }
        acc[i] = sum;
      }
    }
  }
  const bool poisoned = wave_max(bad ? 1.f : 0.f) > 0.f;
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i) {
    const int d = lane + 64 * i;
    if (d < D) dst[d] = poisoned ? NAN : acc[i];
  }
  if (lane == 0) {
    dst[D] = poisoned ? NAN : m;
    dst[D + 1] = l;
  }
}

// out[t, column + head * out_dim + j] = attended[t, head * D + j] * gate[t, head] * scale for j < out_dim; gate
// float32 [tokens, heads] (null: 1); a row of `out` is out_row elements long.
template <typename T>
__global__ __launch_bounds__(256) void scale_heads_kernel(const T* __restrict__ attended, const float* __restrict__ gate,
                                                          T* __restrict__ out, int64_t out_row, int heads, int D,
                                                          int out_dim, float scale) {
  const int64_t t = blockIdx.x;
  for (int i = threadIdx.x; i < heads * out_dim; i += 256) {
    const int hd = i / out_dim;
    const int j = i - hd * out_dim;
    float val = to_f32(attended[(t * heads + hd) * D + j]) * scale;
    if (gate != nullptr) val *= gate[t * heads + hd];
    out[t * out_row + i] = from_f32<T>(val);
  }
}

// decay[t, c] = sigmoid(z)^(1 / tau), z = sum_r w2[c, r] * low[t, r] + bias[c]: `low` are `rank` columns of
// the projected rows p (float32) from column low_offset on, w2 [channels, rank], all sums in float32.
// log sigmoid(z) = -softplus(-z), taken on the side where the exponential is small.
constexpr int kDecayTokens = 8;

__global__ __launch_bounds__(256) void gla_decay_kernel(const float* __restrict__ p, int width, int low_offset, int rank,
                                                        const void* __restrict__ w2, const void* __restrict__ bias,
                                                        int weight_is_f32, int bias_is_f32, float inv_tau,
                                                        float* __restrict__ decay, int channels, int tokens) {
  // a workgroup takes kDecayTokens tokens, so that a row of w2 is read once for all of them
  extern __shared__ float low[];  // [kDecayTokens][rank]
  const int64_t t0 = static_cast<int64_t>(blockIdx.x) * kDecayTokens;
  const int count = static_cast<int>(min(static_cast<int64_t>(kDecayTokens), tokens - t0));
  for (int idx = threadIdx.x; idx < count * rank; idx += 256) {
    const int u = idx / rank;
    const int r = idx - u * rank;
    low[idx] = p[(t0 + u) * width + low_offset + r];
  }
  __syncthreads();
  for (int c = threadIdx.x; c < channels; c += 256) {
    float z[kDecayTokens];
    const float b = bias ? load_as_f32(bias, c, bias_is_f32) : 0.f;
#pragma unroll
    for (int u = 0; u < kDecayTokens; ++u) z[u] = b;
    for (int r = 0; r < rank; ++r) {
      const float w = load_as_f32(w2, static_cast<int64_t>(c) * rank + r, weight_is_f32);
#pragma unroll
      for (int u = 0; u < kDecayTokens; ++u) z[u] = fmaf(w, low[min(u, count - 1) * rank + r], z[u]);
    }
#pragma unroll
    for (int u = 0; u < kDecayTokens; ++u) {
      if (u >= count) break;
      const float log_sigmoid = z[u] >= 0.f ? -log1pf(expf(-z[u])) : z[u] - log1pf(expf(z[u]));
      decay[(t0 + u) * channels + c] = expf(log_sigmoid * inv_tau);
    }
  }
}

// S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T (q_t * q_scale) per (entry, head), the entry's tokens in
// order; a_t [dim] from `decay` [tokens, heads * dim].  `p` [tokens, width] float32 holds q (heads * dim), k
// (heads * dim), v (heads * vdim).  A wavefront owns 16 columns of one head's state: lane = (group of dims g =
// lane / 16, column c = lane % 16) keeps S[d][c] for d = 4 i + g in registers; tokens go through LDS kBatch at
// a time, shared by the kGlaWaves wavefronts of a workgroup (64 columns: q, k and the decays are read from memory
// once per 64 columns, not once per 16).  State rows as for the other recurrent kernels: read_rows[entry] (zeros when the entry starts its
// request) to write_rows[entry]; out [tokens, heads * vdim] float32.
//
// Long entries are cut into runs of kGlaRun tokens (`runs` != null: blockIdx.x counts the runs of all entries, see
// find_run), and the recurrence, which is linear in the state, is walked in three kernels:
//   kRunSums:  every run from a zero state, no outputs: leaves U = sum_j diag(prod_{s > j} a_s) k_j v_j^T in
//              runs[run, head] and the run's whole decay prod_s a_s in run_decay[run, head],
//   gla_carry_kernel: per entry, run after run, S' = diag(run_decay) S + U, leaving the state BEFORE every run where
//              its U was (the first run's: the carried state or zeros),
//   kRunScan:  every run from its own start state, with outputs; an entry's last run stores the state.
// Decays only ever multiply (no quotient of cumulated decays), so any decay in [0, 1] is safe.
constexpr int kGlaRun = 64;
constexpr int kGlaWaves = 4;
// tokens that go through LDS together: every batch costs a trip to memory, but a workgroup is one wavefront and
// a compute unit hides those trips behind its other workgroups: 12 KB each leaves room for a dozen (measured:
// 24 KB each, six to a compute unit, is slower than batches of half the size)
__host__ __device__ constexpr int gla_batch(int dpl) { return dpl <= 16 ? 16 : 8; }

// What makes the decay of a token inside the scan kernel (entries walked whole: steps of few tokens, where a kernel
// of its own for the decays would cost as much as the scan; inside the walks over runs it was measured slower than
// that kernel: it holds up a workgroup's four wavefronts and is made again for every 64 value columns): see
// gla_decay_kernel.
struct GlaDecayInputs {
  int low_offset;
  int rank;
  const void* w2;
  const void* bias;
  int weight_is_f32;
  int bias_is_f32;
  float inv_tau;
};
enum GlaMode { kWholeEntries = 0, kRunSums = 1, kRunScan = 2 };

// Run `b` of all entries' runs of kGlaRun tokens: its entry, its place among the entry's runs and their number.
__device__ inline bool find_run(int b, const int* __restrict__ cu_q, int entries, int& entry, int& index, int& count) {
  int before = 0;
  for (int e = 0; e < entries; ++e) {
    const int n = (cu_q[e + 1] - cu_q[e] + kGlaRun - 1) / kGlaRun;
    if (b < before + n) {
      entry = e;
      index = b - before;
      count = n;
      return true;
    }
    before += n;
  }
  return false;
}

template <int DPL, int MODE>
__global__ __launch_bounds__(64 * kGlaWaves) void gla_scan_kernel(const float* __restrict__ p, int width,
                                                      const float* __restrict__ decay, float* __restrict__ state,
                                                      const int* __restrict__ read_rows,
                                                      const int* __restrict__ write_rows, const int* __restrict__ cu_q,
                                                      const int* __restrict__ q_starts, float q_scale,
                                                      float* __restrict__ out, int heads, int dim, int vdim,
                                                      int entries, float* __restrict__ runs,
                                                      float* __restrict__ run_decay, GlaDecayInputs made_here) {
  constexpr int kGlaBatch = gla_batch(DPL);
  // dim d = 4 i + g lies at g * kGroup + i: a lane's DPL dims are consecutive (16-byte reads), and the four
  // groups of a wavefront start four floats further each, in banks of their own
  constexpr int kGroup = DPL + 4;
  __shared__ __attribute__((aligned(16))) float qs[kGlaBatch][4 * kGroup];
  __shared__ __attribute__((aligned(16))) float ks[kGlaBatch][4 * kGroup];
  __shared__ __attribute__((aligned(16))) float as[kGlaBatch][4 * kGroup];
  __shared__ float vs[kGlaBatch][16 * kGlaWaves];
  const int h = blockIdx.y;
  const int wave = threadIdx.x / 64;
  const int v0 = (blockIdx.z * kGlaWaves + wave) * 16;
  const int lane = threadIdx.x % 64;
  const int g = lane / 16;
  const int c = lane % 16;
  const bool column = v0 + c < vdim;
  const int64_t head_state = static_cast<int64_t>(dim) * vdim;
  int entry = blockIdx.x, index = 0, count = 1;
  if (MODE != kWholeEntries && !find_run(blockIdx.x, cu_q, entries, entry, index, count)) return;
  int t_first = cu_q[entry];
  int t_end = cu_q[entry + 1];
  if (MODE != kWholeEntries) {
    t_first += index * kGlaRun;
    t_end = min(t_end, t_first + kGlaRun);
  }
  float* mine = MODE == kWholeEntries ? nullptr : runs + (static_cast<int64_t>(blockIdx.x) * heads + h) * head_state;
  // dims beyond `dim` read zeros (a decay of 0 on a state of 0), so that the walk below needs no condition per dim:
  // a condition there makes every LDS read wait for the one before
  for (int idx = threadIdx.x; idx < kGlaBatch * 4 * kGroup; idx += 64 * kGlaWaves) {
    (&qs[0][0])[idx] = 0.f;
    (&ks[0][0])[idx] = 0.f;
    (&as[0][0])[idx] = 0.f;
  }

  float S[DPL];
  float whole[MODE == kRunSums ? DPL : 1];
  const bool carried = MODE == kRunScan || (MODE == kWholeEntries && q_starts[entry] > 0);
  const float* src = MODE == kRunScan ? mine : state + (static_cast<int64_t>(read_rows[entry]) * heads + h) * head_state;
#pragma unroll
  for (int i = 0; i < DPL; ++i) {
    const int d = 4 * i + g;
    S[i] = (MODE != kRunSums && carried && column && d < dim) ? src[static_cast<int64_t>(d) * vdim + v0 + c] : 0.f;
    if constexpr (MODE == kRunSums) whole[i] = 1.f;
  }
  for (int tb = t_first; tb < t_end; tb += kGlaBatch) {
    const int count_b = min(kGlaBatch, t_end - tb);
    __syncthreads();  // the batch before is done with
    for (int idx = threadIdx.x; idx < count_b * dim; idx += 64 * kGlaWaves) {
      const int u = idx / dim;
      const int d = idx - u * dim;
      const int64_t t = tb + u;
      const float* q = p + t * width + static_cast<int64_t>(h) * dim;
      const int at = (d & 3) * kGroup + (d >> 2);
      if (MODE != kRunSums) qs[u][at] = q[d] * q_scale;
      ks[u][at] = q[static_cast<int64_t>(heads) * dim + d];
      if (MODE == kWholeEntries) {
        const int ch = h * dim + d;
        const float* low = p + t * width + made_here.low_offset;
        float z = made_here.bias ? load_as_f32(made_here.bias, ch, made_here.bias_is_f32) : 0.f;
        for (int r = 0; r < made_here.rank; ++r)
          z = fmaf(load_as_f32(made_here.w2, static_cast<int64_t>(ch) * made_here.rank + r, made_here.weight_is_f32), low[r], z);
        const float log_sigmoid = z >= 0.f ? -log1pf(expf(-z)) : z - log1pf(expf(z));
        as[u][at] = expf(log_sigmoid * made_here.inv_tau);
      } else {
        as[u][at] = decay[(t * heads + h) * dim + d];
      }
    }
    for (int idx = threadIdx.x; idx < count_b * 16 * kGlaWaves; idx += 64 * kGlaWaves) {
      const int u = idx / (16 * kGlaWaves);
      const int cc = idx - u * (16 * kGlaWaves);
      const int v = blockIdx.z * 16 * kGlaWaves + cc;
      vs[u][cc] = v < vdim ? p[static_cast<int64_t>(tb + u) * width + 2ll * heads * dim + static_cast<int64_t>(h) * vdim + v] : 0.f;
    }
    __syncthreads();
    for (int u = 0; u < count_b; ++u) {
      const float vv = vs[u][wave * 16 + c];
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < DPL; ++i) {
        const float a = as[u][g * kGroup + i];
        S[i] = fmaf(a, S[i], ks[u][g * kGroup + i] * vv);
        if constexpr (MODE == kRunSums)
          whole[i] *= a;
        else
          o = fmaf(S[i], qs[u][g * kGroup + i], o);
      }
      if (MODE != kRunSums) {
        o += __shfl_xor(o, 16, kWave);
        o += __shfl_xor(o, 32, kWave);
        if (g == 0 && column) out[static_cast<int64_t>(tb + u) * heads * vdim + static_cast<int64_t>(h) * vdim + v0 + c] = o;
      }
    }
  }
  if constexpr (MODE == kRunSums) {
#pragma unroll
    for (int i = 0; i < DPL; ++i) {
      const int d = 4 * i + g;
      if (column && d < dim) mine[static_cast<int64_t>(d) * vdim + v0 + c] = S[i];
      if (blockIdx.z == 0 && wave == 0 && c == 0 && d < dim) run_decay[(static_cast<int64_t>(blockIdx.x) * heads + h) * dim + d] = whole[i];
    }
    return;
  }
  if (MODE == kRunScan && index != count - 1) return;  // only an entry's last run leaves the state
  float* dst = state + (static_cast<int64_t>(write_rows[entry]) * heads + h) * head_state;
#pragma unroll
  for (int i = 0; i < DPL; ++i) {
    const int d = 4 * i + g;
    if (column && d < dim) dst[static_cast<int64_t>(d) * vdim + v0 + c] = S[i];
  }
}

// Between the two walks over the runs (see gla_scan_kernel): a thread owns one element of one head's state and goes
// through its entry's runs in order.  Grid (entries, heads, ceil(dim * vdim / 256)).
__global__ __launch_bounds__(256) void gla_carry_kernel(float* __restrict__ runs, const float* __restrict__ run_decay,
                                                        const float* __restrict__ state,
                                                        const int* __restrict__ read_rows, const int* __restrict__ cu_q,
                                                        const int* __restrict__ q_starts, int heads, int dim, int vdim) {
  const int entry = blockIdx.x;
  const int h = blockIdx.y;
  const int e = blockIdx.z * 256 + threadIdx.x;
  const int head_state = dim * vdim;
  if (e >= head_state) return;
  const int d = e / vdim;
  int first = 0;  // the entry's first run among all runs
  for (int i = 0; i < entry; ++i) first += (cu_q[i + 1] - cu_q[i] + kGlaRun - 1) / kGlaRun;
  const int count = (cu_q[entry + 1] - cu_q[entry] + kGlaRun - 1) / kGlaRun;
  float S = q_starts[entry] > 0 ? state[(static_cast<int64_t>(read_rows[entry]) * heads + h) * head_state + e] : 0.f;
  for (int r = 0; r < count; ++r) {
    float* at = runs + (static_cast<int64_t>(first + r) * heads + h) * head_state + e;
    const float U = *at;
    *at = S;
    S = fmaf(run_decay[(static_cast<int64_t>(first + r) * heads + h) * dim + d], S, U);
  }
}

}  // namespace
}  // namespace mlr

using namespace mlr;

extern "C" {

int mlr_short_conv(const void* h, const void* weight, int weight_is_f32, float* state, int state_rows,
                   const int* read_rows, const int* write_rows, const int* token_entry, const int* cu_q,
                   const int* q_starts, void* out, int dtype, int tokens, int width, int taps, int add_input,
                   hipStream_t stream) {
  MLR_REQUIRE(h && weight && read_rows && write_rows && token_entry && cu_q && q_starts && out, "null pointer");
  MLR_REQUIRE(tokens > 0 && width > 0 && taps > 0, "sizes must be > 0");
  MLR_REQUIRE(taps == 1 || (state != nullptr && state_rows > 0), "carried inputs need a state");
  MLR_REQUIRE(dtype == kF32 || dtype == kBF16, "dtype must be 0 (float32) or 1 (bfloat16)");
  if (dtype == kF32)
    short_conv_kernel<float><<<tokens, 256, 0, stream>>>(static_cast<const float*>(h), weight, weight_is_f32, state,
                                                         read_rows, write_rows, token_entry, cu_q, q_starts,
                                                         static_cast<float*>(out), width, taps, add_input);
  else
    short_conv_kernel<bf16><<<tokens, 256, 0, stream>>>(static_cast<const bf16*>(h), weight, weight_is_f32, state,
                                                        read_rows, write_rows, token_entry, cu_q, q_starts,
                                                        static_cast<bf16*>(out), width, taps, add_input);
  MLR_LAUNCH_CHECK();
  return 0;
}

int mlr_qk_norm_rope_write(const float* projected, int width, const void* q_norm, const void* k_norm, int weight_is_f32,
                           float eps, const float* head_scale, const float* cos_t, const float* sin_t, int rotary_dim,
                           const int* slots, void* key_pages, void* value_pages, void* q_out, float* gate, int dtype,
                           int tokens, int heads, int kv_heads, int dim, int vdim, int head_dim, int block_size,
                           int num_pages, int gated, hipStream_t stream) {
  MLR_REQUIRE(projected && slots && key_pages && value_pages && q_out, "null pointer");
  MLR_REQUIRE(tokens > 0 && heads > 0 && kv_heads > 0 && dim > 0 && vdim > 0, "sizes must be > 0");
  MLR_REQUIRE(head_dim >= dim && head_dim >= vdim, "the pages' head size must hold keys and values");
  MLR_REQUIRE(rotary_dim >= 0 && rotary_dim % 2 == 0 && rotary_dim <= dim, "rotary_dim must be even and within dim");
  MLR_REQUIRE(rotary_dim == 0 || (cos_t && sin_t), "a rotation needs its tables");
  MLR_REQUIRE(!gated || gate, "gates need their output");
  MLR_REQUIRE(width >= heads * dim + kv_heads * (dim + vdim) + (gated ? heads : 0), "the projected rows are too narrow");
  MLR_REQUIRE(block_size > 0 && num_pages > 0, "pages must exist");
  MLR_REQUIRE(dtype == kF32 || dtype == kBF16, "dtype must be 0 (float32) or 1 (bfloat16)");
  if (dtype == kF32)
    qk_norm_rope_write_kernel<float><<<tokens, 256, 0, stream>>>(
        projected, width, q_norm, k_norm, weight_is_f32, eps, head_scale, rotary_dim ? cos_t : nullptr,
        rotary_dim ? sin_t : nullptr, rotary_dim, slots, static_cast<float*>(key_pages), static_cast<float*>(value_pages),
        static_cast<float*>(q_out), gate, heads, kv_heads, dim, vdim, head_dim, block_size, num_pages, gated);
  else
    qk_norm_rope_write_kernel<bf16><<<tokens, 256, 0, stream>>>(
        projected, width, q_norm, k_norm, weight_is_f32, eps, head_scale, rotary_dim ? cos_t : nullptr,
        rotary_dim ? sin_t : nullptr, rotary_dim, slots, static_cast<bf16*>(key_pages), static_cast<bf16*>(value_pages),
        static_cast<bf16*>(q_out), gate, heads, kv_heads, dim, vdim, head_dim, block_size, num_pages, gated);
  MLR_LAUNCH_CHECK();
  return 0;
}

int mlr_pool_kv_write(const void* key_pages, const void* value_pages, const int* block_table, int table_width,
                      int num_pages, const int* token_entry, const int* positions, const int* pooled_slots,
                      void* pooled_keys, void* pooled_values, int pooled_pages, int dtype, int tokens, int kv_heads,
                      int head_dim, int block_size, int pool, hipStream_t stream) {
  MLR_REQUIRE(key_pages && value_pages && block_table && token_entry && positions && pooled_slots && pooled_keys &&
                  pooled_values,
              "null pointer");
  MLR_REQUIRE(tokens > 0 && kv_heads > 0 && kv_heads < 65536 && head_dim > 0 && block_size > 0 && pool > 0,
              "sizes must be > 0");
  MLR_REQUIRE(table_width > 0 && num_pages > 0 && pooled_pages > 0, "pages must exist");
  MLR_REQUIRE(dtype == kF32 || dtype == kBF16, "dtype must be 0 (float32) or 1 (bfloat16)");
  dim3 grid(tokens, kv_heads);
  if (dtype == kF32)
    pool_kv_write_kernel<float><<<grid, 256, 0, stream>>>(
        static_cast<const float*>(key_pages), static_cast<const float*>(value_pages), block_table, table_width, num_pages,
        token_entry, positions, pooled_slots, static_cast<float*>(pooled_keys), static_cast<float*>(pooled_values),
        pooled_pages, kv_heads, head_dim, block_size, pool);
  else
    pool_kv_write_kernel<bf16><<<grid, 256, 0, stream>>>(
        static_cast<const bf16*>(key_pages), static_cast<const bf16*>(value_pages), block_table, table_width, num_pages,
        token_entry, positions, pooled_slots, static_cast<bf16*>(pooled_keys), static_cast<bf16*>(pooled_values),
        pooled_pages, kv_heads, head_dim, block_size, pool);
  MLR_LAUNCH_CHECK();
  return 0;
}

int mlr_pooled_share(const void* q, int64_t q_stride, const void* pooled_keys, const void* pooled_values,
                     const int* pooled_table, int table_width, int pooled_pages, const int* token_entry,
                     const int* positions, float* share, int tokens, int heads, int kv_heads, int head_dim,
                     int block_size, float scale, int window, int pool, hipStream_t stream) {
  MLR_REQUIRE(q && pooled_keys && pooled_values && pooled_table && token_entry && positions && share, "null pointer");
  MLR_REQUIRE(tokens > 0 && heads > 0 && heads < 65536 && kv_heads > 0 && heads % kv_heads == 0, "bad head counts");
  MLR_REQUIRE(head_dim > 0 && head_dim <= 256, "head sizes up to 256");
  MLR_REQUIRE(block_size > 0 && table_width > 0 && pooled_pages > 0, "pages must exist");
  MLR_REQUIRE(q_stride >= static_cast<int64_t>(heads) * head_dim, "q_stride must cover a row");
  MLR_REQUIRE(scale > 0.f && scale < INFINITY && window > 0 && pool > 0, "bad scale, window or run length");
  MLR_REQUIRE(static_cast<int64_t>(pooled_pages) * kv_heads * block_size < (1ll << 31), "too many pooled slots");
  pooled_share_kernel<<<dim3(tokens, heads), 64, (head_dim + 128) * sizeof(float), stream>>>(
      static_cast<const bf16*>(q), q_stride, static_cast<const bf16*>(pooled_keys),
      static_cast<const bf16*>(pooled_values), pooled_table, table_width, pooled_pages, token_entry, positions, share,
      heads, kv_heads, head_dim, block_size, scale * 1.44269504088896340736f, window, pool);
  MLR_LAUNCH_CHECK();
  return 0;
}

int mlr_scale_heads(const void* attended, const float* gate, void* out, int64_t out_row, int dtype, int tokens, int heads,
                    int head_dim, int out_dim, float scale, hipStream_t stream) {
  MLR_REQUIRE(attended && out, "null pointer");
  MLR_REQUIRE(tokens > 0 && heads > 0 && head_dim > 0 && out_dim > 0 && out_dim <= head_dim, "sizes must be > 0");
  MLR_REQUIRE(out_row >= static_cast<int64_t>(heads) * out_dim, "a row of the output is shorter than the heads");
  MLR_REQUIRE(dtype == kF32 || dtype == kBF16, "dtype must be 0 (float32) or 1 (bfloat16)");
  if (dtype == kF32)
    scale_heads_kernel<float><<<tokens, 256, 0, stream>>>(static_cast<const float*>(attended), gate,
                                                          static_cast<float*>(out), out_row, heads, head_dim, out_dim,
                                                          scale);
  else
    scale_heads_kernel<bf16><<<tokens, 256, 0, stream>>>(static_cast<const bf16*>(attended), gate,
                                                         static_cast<bf16*>(out), out_row, heads, head_dim, out_dim,
                                                         scale);
  MLR_LAUNCH_CHECK();
  return 0;
}

int mlr_gla_runs(int tokens, int entries) { return tokens / kGlaRun + entries; }

int mlr_gla_scan(const float* projected, int width, int low_offset, int rank, const void* decay_weight,
                 const void* decay_bias, int weight_is_f32, int bias_is_f32, float tau, float* decay, float* state,
                 int state_rows, const int* read_rows, const int* write_rows, const int* cu_q, const int* q_starts,
                 float q_scale, float* out, int entries, int heads, int dim, int vdim, int tokens, float* runs,
                 float* run_decay, hipStream_t stream) {
  MLR_REQUIRE(projected && decay_weight && state && read_rows && write_rows && cu_q && q_starts && out, "null pointer");
  MLR_REQUIRE(runs == nullptr || decay != nullptr, "runs need room for the tokens' decays");
  MLR_REQUIRE(tokens > 0 && entries > 0 && heads > 0 && heads < 65536 && dim > 0 && vdim > 0 && state_rows > 0,
              "sizes must be > 0");
  MLR_REQUIRE(rank > 0 && rank <= 2048 && low_offset >= 0 && width >= low_offset + rank, "the projected rows do not hold the decay's inputs");
  MLR_REQUIRE(width >= 2 * heads * dim + heads * vdim, "the projected rows do not hold q, k and v");
  MLR_REQUIRE(tau > 0.f, "tau must be > 0");
  MLR_REQUIRE(dim <= 256, "heads of up to 256 dims");
  const bool by_runs = runs != nullptr;
  const GlaDecayInputs made_here{low_offset, rank, decay_weight, decay_bias, weight_is_f32, bias_is_f32, 1.0f / tau};
  if (by_runs) {  // entries walked whole make their decays themselves
    gla_decay_kernel<<<(tokens + kDecayTokens - 1) / kDecayTokens, 256, kDecayTokens * rank * sizeof(float), stream>>>(
        projected, width, low_offset, rank, decay_weight, decay_bias, weight_is_f32, bias_is_f32, 1.0f / tau, decay,
        heads * dim, tokens);
    MLR_LAUNCH_CHECK();
  }
  const dim3 whole(entries, heads, (vdim + 16 * kGlaWaves - 1) / (16 * kGlaWaves));
  const int most_runs = tokens / kGlaRun + entries;  // no fewer than the sum of the entries' runs
  const dim3 cut(most_runs, heads, (vdim + 16 * kGlaWaves - 1) / (16 * kGlaWaves));
  MLR_REQUIRE(!by_runs || run_decay != nullptr, "runs need room for their decays");
#define MLR_GLA(DPL)                                                                                               \
  do {                                                                                                             \
    if (!by_runs) {                                                                                                \
      gla_scan_kernel<DPL, kWholeEntries><<<whole, 64 * kGlaWaves, 0, stream>>>(projected, width, decay, state, read_rows,     \
                                                                    write_rows, cu_q, q_starts, q_scale, out,      \
                                                                    heads, dim, vdim, entries, nullptr, nullptr,   \
                                                                    made_here);                                    \
    } else {                                                                                                       \
      gla_scan_kernel<DPL, kRunSums><<<cut, 64 * kGlaWaves, 0, stream>>>(projected, width, decay, state, read_rows,            \
                                                             write_rows, cu_q, q_starts, q_scale, out, heads, dim, \
                                                             vdim, entries, runs, run_decay, made_here);           \
      gla_carry_kernel<<<dim3(entries, heads, (dim * vdim + 255) / 256), 256, 0, stream>>>(                        \
          runs, run_decay, state, read_rows, cu_q, q_starts, heads, dim, vdim);                                    \
      gla_scan_kernel<DPL, kRunScan><<<cut, 64 * kGlaWaves, 0, stream>>>(projected, width, decay, state, read_rows,            \
                                                             write_rows, cu_q, q_starts, q_scale, out, heads, dim, \
                                                             vdim, entries, runs, run_decay, made_here);           \
    }                                                                                                              \
  } while (0)
  if (dim <= 32)
    MLR_GLA(8);
  else if (dim <= 64)
    MLR_GLA(16);
  else if (dim <= 128)
    MLR_GLA(32);
  else
    MLR_GLA(64);
#undef MLR_GLA
  MLR_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
