// Several residual streams side by side (hyper-connections), the preparation of an attention whose
// queries, keys and values are normed per head, and a matrix memory with exponential gates.
// Everything here is 32-bit inside; activations leave in the engine's dtype.
#include "api.h"
#include "common.h"

namespace mlr {

constexpr int kMaxStreams = 16;

// ---- residual streams -------------------------------------------------------------------------------
// x [streams, tokens, width] float32.  One workgroup per output row r (token rows[r], or r).  In order:
//  1. (y given) all streams at once from the old ones: x_t = sum_s mix[s, t] x_s + out_w[t] * y, y a row of
//     activations (engine dtype or float32) or the sum, in order, of `slices` float32 rows; written back
//     unless `rows` choose tokens (then the streams stay as they are and only the outputs below are made);
//  2. u = sum_s in_w[s] x_s (in_w null: the plain sum of the streams);
//  3. (sum_out) u as float32; (h_out) u * rsqrt(mean(u^2) + eps) * norm_w in the engine's dtype.
template <typename T>
__global__ __launch_bounds__(256) void streams_step_kernel(
    float* __restrict__ x, int streams, int tokens, int width, const int* __restrict__ rows, const void* __restrict__ y,
    int y_is_f32, int slices, const float* __restrict__ mix, const float* __restrict__ out_w,
    const float* __restrict__ in_w, const void* __restrict__ norm_w, int norm_is_f32, float eps, T* __restrict__ h_out,
    float* __restrict__ sum_out) {
  __shared__ float scratch[16];
  __shared__ float s_mix[kMaxStreams * kMaxStreams];
  __shared__ float s_out[kMaxStreams];
  __shared__ float s_in[kMaxStreams];
  const int r = blockIdx.x;
  const int64_t t = rows != nullptr ? rows[r] : r;
  const bool write_back = rows == nullptr;
  const int64_t plane = static_cast<int64_t>(tokens) * width;
  for (int i = threadIdx.x; i < streams * streams; i += 256) s_mix[i] = mix != nullptr ? mix[i] : 0.f;
  for (int i = threadIdx.x; i < streams; i += 256) {
    s_out[i] = out_w != nullptr ? out_w[i] : 0.f;
    s_in[i] = in_w != nullptr ? in_w[i] : 1.f;
  }
  __syncthreads();
  float ss = 0.f;
  for (int pass = 0; pass < 2; ++pass) {
    // the second pass makes the same numbers again (from the old streams when nothing was written back)
    if (pass == 1 && h_out == nullptr) break;
    float inv = 0.f;
    if (pass == 1) inv = 1.0f / sqrtf(block_sum(ss, scratch) / static_cast<float>(width) + eps);
    for (int c = threadIdx.x; c < width; c += 256) {
      float xs[kMaxStreams];
#pragma unroll
      for (int s = 0; s < kMaxStreams; ++s) xs[s] = s < streams ? x[s * plane + t * width + c] : 0.f;
      float u = 0.f;
      if (y != nullptr && !(pass == 1 && write_back)) {
        float yv = 0.f;
        if (slices > 0) {
          for (int k = 0; k < slices; ++k) yv += static_cast<const float*>(y)[k * plane + t * width + c];
        } else {
          yv = load_as_f32(y, t * width + c, y_is_f32);
        }
#pragma unroll
        for (int to = 0; to < kMaxStreams; ++to) {
          if (to < streams) {
            float v = 0.f;
#pragma unroll
            for (int s = 0; s < kMaxStreams; ++s)
              if (s < streams) v = fmaf(s_mix[s * streams + to], xs[s], v);
            v = fmaf(s_out[to], yv, v);
            if (write_back) x[to * plane + t * width + c] = v;
            u = fmaf(s_in[to], v, u);
          }
        }
      } else {
#pragma unroll
        for (int s = 0; s < kMaxStreams; ++s)
          if (s < streams) u = fmaf(s_in[s], xs[s], u);
      }
      if (pass == 0) {
        ss += u * u;
        if (sum_out != nullptr) sum_out[static_cast<int64_t>(r) * width + c] = u;
      } else {
        h_out[static_cast<int64_t>(r) * width + c] = from_f32<T>(u * inv * load_as_f32(norm_w, c, norm_is_f32));
      }
    }
  }
}

// The same for up to four streams and rows of up to 4,096 numbers that are a multiple of four: a thread owns groups
// of four neighbouring columns (16-byte loads and stores), all of its loads are asked for before the first is
// used, and its sums u stay in registers between the row's sum of squares and the normed result, so every
// number is read once.
typedef float f32x4 __attribute__((ext_vector_type(4)));
constexpr int kStreamGroups = 4;  // groups of four columns a thread owns: 256 * 4 * 4 columns a row at most

template <typename T, int S>
__global__ __launch_bounds__(256) void streams_step_rows_kernel(
    float* __restrict__ x, int tokens, int width, const int* __restrict__ rows, const void* __restrict__ y,
    int y_is_f32, int slices, const float* __restrict__ mix, const float* __restrict__ out_w,
    const float* __restrict__ in_w, const void* __restrict__ norm_w, int norm_is_f32, float eps, T* __restrict__ h_out,
    float* __restrict__ sum_out) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const int64_t t = rows != nullptr ? rows[r] : r;
  const bool write_back = rows == nullptr;
  const int64_t plane = static_cast<int64_t>(tokens) * width;
  float w_mix[S][S], w_out[S], w_in[S];  // uniform: scalar registers
#pragma unroll
  for (int a = 0; a < S; ++a) {
#pragma unroll
    for (int b = 0; b < S; ++b) w_mix[a][b] = mix != nullptr ? mix[a * S + b] : 0.f;
    w_out[a] = out_w != nullptr ? out_w[a] : 0.f;
    w_in[a] = in_w != nullptr ? in_w[a] : 1.f;
  }
  f32x4 xs[kStreamGroups][S], yv[kStreamGroups];
#pragma unroll
  for (int i = 0; i < kStreamGroups; ++i) {
    const int c = (threadIdx.x + i * 256) * 4;
    const bool in = c < width;
    const int64_t at = t * width + (in ? c : 0);
#pragma unroll
    for (int a = 0; a < S; ++a) xs[i][a] = in ? *reinterpret_cast<const f32x4*>(x + a * plane + at) : f32x4{0.f, 0.f, 0.f, 0.f};
    yv[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (y != nullptr && in) {
      if (slices > 0) {
        for (int k = 0; k < slices; ++k) yv[i] += *reinterpret_cast<const f32x4*>(static_cast<const float*>(y) + k * plane + at);
      } else if (y_is_f32) {
        yv[i] = *reinterpret_cast<const f32x4*>(static_cast<const float*>(y) + at);
      } else {
        typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
        const u16x4 raw = *reinterpret_cast<const u16x4*>(static_cast<const bf16*>(y) + at);
#pragma unroll
        for (int e = 0; e < 4; ++e) yv[i][e] = to_f32(bf16{raw[e]});
      }
    }
  }
  f32x4 us[kStreamGroups];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kStreamGroups; ++i) {
    const int c = (threadIdx.x + i * 256) * 4;
    const bool in = c < width;
    f32x4 u = {0.f, 0.f, 0.f, 0.f};
    if (y != nullptr) {
#pragma unroll
      for (int to = 0; to < S; ++to) {
        f32x4 v = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int a = 0; a < S; ++a)
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = fmaf(w_mix[a][to], xs[i][a][e], v[e]);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[e] = fmaf(w_out[to], yv[i][e], v[e]);
          u[e] = fmaf(w_in[to], v[e], u[e]);
        }
        if (write_back && in) *reinterpret_cast<f32x4*>(x + to * plane + t * width + c) = v;
      }
    } else {
#pragma unroll
      for (int a = 0; a < S; ++a)
#pragma unroll
        for (int e = 0; e < 4; ++e) u[e] = fmaf(w_in[a], xs[i][a][e], u[e]);
    }
    us[i] = u;
    ss += (u[0] * u[0] + u[1] * u[1]) + (u[2] * u[2] + u[3] * u[3]);
    if (sum_out != nullptr && in) *reinterpret_cast<f32x4*>(sum_out + static_cast<int64_t>(r) * width + c) = u;
  }
  if (h_out == nullptr) return;
  const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / static_cast<float>(width) + eps);
#pragma unroll
  for (int i = 0; i < kStreamGroups; ++i) {
    const int c = (threadIdx.x + i * 256) * 4;
    if (c >= width) continue;
    float o[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = us[i][e] * inv * load_as_f32(norm_w, c + e, norm_is_f32);
    T* dst = h_out + static_cast<int64_t>(r) * width + c;
    if constexpr (sizeof(T) == 4) {
      *reinterpret_cast<f32x4*>(dst) = f32x4{o[0], o[1], o[2], o[3]};
    } else {
      typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
      *reinterpret_cast<u16x4*>(dst) = u16x4{f32_to_bf16(o[0]).bits, f32_to_bf16(o[1]).bits, f32_to_bf16(o[2]).bits, f32_to_bf16(o[3]).bits};
    }
  }
}

__global__ __launch_bounds__(256) void streams_fill_kernel(const float* __restrict__ x, float* __restrict__ out,
                                                           int64_t plane, int streams) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= plane) return;
  const float v = x[i];
  for (int s = 0; s < streams; ++s) out[s * plane + i] = v;
}

// ---- queries, keys and values normed per head -----------------------------------------------------------
// p [tokens, width] float32 holds per token: heads * dim query sums, kv_heads * dim key sums, kv_heads * vdim value
// sums, then `heads` gate logits (if gate is given).  Per token:
//  * every query and key head: rotation of its first rdims dims in two halves (pair j, j + rdims / 2), then the
//    head divided by its root mean square over dim (eps inside the root); queries to q_out [tokens, heads * D]
//    (columns dim .. D - 1 zero), keys to the key pages [page, kv_head, offset, D] at slot[t];
//  * every value head divided by its root mean square over vdim; (v_keep) the normed values as float32 [tokens,
//    kv_heads * vdim]; (v_first) v = (1 - lambda) v + lambda v_first[t]; values to [page, kv_head, D, offset];
//  * gate[t, head] = sigmoid(logit).
// One wavefront per head; a negative slot stores nothing.
template <typename T>
__global__ __launch_bounds__(256) void head_norm_rope_write_kernel(
    const float* __restrict__ p, int width, T* __restrict__ q_out, float* __restrict__ gate,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rdims, float eps,
    const int* __restrict__ slots, T* __restrict__ key_pages, T* __restrict__ value_pages, float* __restrict__ v_keep,
    const float* __restrict__ v_first, const float* __restrict__ lambda_p, int heads, int kv_heads, int dim, int vdim,
    int D, int block_size, int num_pages) {
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const float* row = p + t * width;
  const int half = rdims / 2;
  const float* cs = cos_t != nullptr ? cos_t + t * half : nullptr;
  const float* sn = sin_t != nullptr ? sin_t + t * half : nullptr;
  const int slot = slots[t];
  const int page = slot >= 0 ? slot / block_size : -1;
  const int off = slot >= 0 ? slot - page * block_size : 0;
  const bool store = page >= 0 && page < num_pages;
  const float lambda = (v_first != nullptr && lambda_p != nullptr) ? lambda_p[0] : 0.f;
  const int jobs = heads + 2 * kv_heads;
  for (int job = wave; job < jobs; job += 4) {
    const bool is_q = job < heads;
    const bool is_k = !is_q && job < heads + kv_heads;
    const int h = is_q ? job : (is_k ? job - heads : job - heads - kv_heads);
    const int n = (is_q || is_k) ? dim : vdim;
    const float* src = row + (is_q ? h * dim : (is_k ? heads * dim + h * dim : (heads + kv_heads) * dim + h * vdim));
    auto value = [&](int j) {
      if (!(is_q || is_k) || j >= rdims || cs == nullptr) return src[j];
      return j < half ? src[j] * cs[j] - src[j + half] * sn[j] : src[j] * cs[j - half] + src[j - half] * sn[j - half];
    };
    float ss = 0.f;
    for (int j = lane; j < n; j += kWave) {
      const float v = value(j);
      ss += v * v;
    }
    const float inv = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(n) + eps);
    if (is_q) {
      T* dst = q_out + (t * heads + h) * D;
      for (int j = lane; j < D; j += kWave) dst[j] = from_f32<T>(j < n ? value(j) * inv : 0.f);
    } else if (is_k) {
      if (store) {
        T* dst = key_pages + ((static_cast<int64_t>(page) * kv_heads + h) * block_size + off) * D;
        for (int j = lane; j < D; j += kWave) dst[j] = from_f32<T>(j < n ? value(j) * inv : 0.f);
      }
    } else {
      T* dst = value_pages + (static_cast<int64_t>(page) * kv_heads + h) * D * block_size + off;
      for (int j = lane; j < D; j += kWave) {
        float v = 0.f;
        if (j < n) {
          v = src[j] * inv;
          if (v_keep != nullptr) v_keep[(t * kv_heads + h) * vdim + j] = v;
          if (v_first != nullptr) v = (1.0f - lambda) * v + lambda * v_first[(t * kv_heads + h) * vdim + j];
        }
        if (store) dst[static_cast<int64_t>(j) * block_size] = from_f32<T>(v);
      }
    }
  }
  if (gate != nullptr) {
    const float* z = row + (heads + kv_heads) * dim + kv_heads * vdim;
    for (int h = threadIdx.x; h < heads; h += 256) gate[t * heads + h] = 1.0f / (1.0f + expf(-z[h]));
  }
}

// ---- matrix memory with exponential gates ------------------------------------------------------------------
// Per head: a matrix C [dim, vdim], a vector n [dim] and a running maximum m, all float32, in `state` [state_rows,
// heads, dim * vdim + dim + 1] (C row-major, then n, then m).  Per token, with a = the input gate's sum and b = the
// forget gate's sum (both with their biases):
//   i = cap tanh(a / cap),  f = logsigmoid(cap tanh(b / cap)),  m' = max(f + m, i),
//   C' = exp(f + m - m') C + exp(i - m') k v^T,  n' likewise with k alone,
//   o = C'^T q / (max(|n' . q|, exp(-m')) + 1e-6),  q scaled by q_scale.
// An entry that starts its request starts from zeros (m = 0 too) whatever its row holds.  A workgroup of four
// wavefronts owns 64 value columns of one head of one entry: lane (g, c) of a wavefront holds a quarter of the rows
// of column c of C (consecutive ones: 16-byte LDS reads) and the same rows of n; eight tokens' q and k at a time go
// through LDS, rows beyond dim as zeros, so the inner loops have no conditions, and the eight after them are on
// their way from memory meanwhile.
constexpr int kMemTokens = 8;
constexpr int kMemRun = 64;  // tokens of a run when long entries are walked in runs

// Long entries are cut into runs of kMemRun tokens, all runs of all entries walked at once, twice.  With F the
// sum of a run's f and the run walked from nothing (C = n = 0, m = -inf), its own sums U (of C and n alike) and
// maximum m_u relate the states before and after it:  m' = max(F + m, m_u),  X' = exp(F + m - m') X + exp(m_u -
// m') U.  kRunSums makes U, m_u and F of every run; matrix_memory_carry_kernel walks an entry's runs element by
// element and leaves the state BEFORE every run where its U was (and the entry's last state in its row);
// kRunScan walks every run again from that state and writes the outputs.
enum MemoryMode : int { kWholeEntries = 0, kRunSums = 1, kRunScan = 2 };

// Which entry run number `run` (counted over all entries in order) belongs to, and its tokens.
__device__ inline bool find_memory_run(const int* __restrict__ cu_q, int entries, int run, int& entry, int& t_begin,
                                       int& t_end) {
  int at = 0;
  for (int e = 0; e < entries; ++e) {
    const int a = cu_q[e], b = cu_q[e + 1];
    const int runs = (b - a + kMemRun - 1) / kMemRun;
    if (run < at + runs) {
      entry = e;
      t_begin = a + (run - at) * kMemRun;
      t_end = min(t_begin + kMemRun, b);
      return true;
    }
    at += runs;
  }
  return false;
}

__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

template <int R, int MODE>  // R: rows of the state a lane holds, dim <= 4 * R
__global__ __launch_bounds__(256) void matrix_memory_scan_kernel(
    const float* __restrict__ p, int width, int q_off, int k_off, int v_off, int i_off, int f_off,
    float* __restrict__ state, const int* __restrict__ read_rows, const int* __restrict__ write_rows,
    const int* __restrict__ cu_q, const int* __restrict__ q_starts, float cap, float q_scale, float* __restrict__ out,
    int heads, int dim, int vdim, int entries, float* __restrict__ runs, float* __restrict__ run_gates) {
  constexpr int MAXD = 4 * R;
  constexpr int kGroup = R + 4;  // floats of a group of rows in LDS: the four groups' 16-byte reads fall into banks of their own
  __shared__ __attribute__((aligned(16))) float sq[kMemTokens][4][kGroup];
  __shared__ __attribute__((aligned(16))) float sk[kMemTokens][4][kGroup];
  __shared__ float sv[kMemTokens][64];
  __shared__ float sg[kMemTokens][2];
  const int h = blockIdx.y;
  const int tid = threadIdx.x;
  const int lane = tid % kWave;
  const int wave = tid / kWave;
  const int g = lane / 16;  // this lane's rows: g * R .. g * R + R - 1
  const int c_local = wave * 16 + lane % 16;
  const int col = blockIdx.z * 64 + c_local;
  const bool col_ok = col < vdim;
  const int64_t per_head = static_cast<int64_t>(dim) * vdim + dim + 1;
  int entry = blockIdx.x, t_begin, t_end;
  bool fresh;
  const float* src;
  float* dst;
  if constexpr (MODE == kWholeEntries) {
    t_begin = cu_q[entry];
    t_end = cu_q[entry + 1];
    fresh = q_starts[entry] == 0;
    src = state + (static_cast<int64_t>(read_rows[entry]) * heads + h) * per_head;
    dst = state + (static_cast<int64_t>(write_rows[entry]) * heads + h) * per_head;
  } else {
    if (!find_memory_run(cu_q, entries, blockIdx.x, entry, t_begin, t_end)) return;  // the grid is sized for the most runs
    fresh = MODE == kRunSums;
    src = dst = runs + (static_cast<int64_t>(blockIdx.x) * heads + h) * per_head;
  }

  // The next eight tokens' q, k, v and gate sums are asked for while the present eight are walked, and wait in
  // registers: a thread carries kPer numbers of q and of k, two of v and (the first eight threads) a token's gates.
  constexpr int kPer = kMemTokens * MAXD / 256;
  float rq[kPer], rk[kPer], rv[2], rgate[2];
  auto fetch = [&](int t0) {
    const int nb = min(kMemTokens, t_end - t0);
#pragma unroll
    for (int u = 0; u < kPer; ++u) {
      const int idx = tid + u * 256;
      const int tt = idx / MAXD;
      const int r = idx - tt * MAXD;
      const bool in = tt < nb && r < dim;
      const float* row = p + static_cast<int64_t>(t0 + (in ? tt : 0)) * width + h * dim + (in ? r : 0);
      rq[u] = in ? row[q_off] * q_scale : 0.f;
      rk[u] = in ? row[k_off] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int idx = tid + u * 256;
      const int tt = idx / 64;
      const int c = blockIdx.z * 64 + (idx - tt * 64);
      const bool in = tt < nb && c < vdim;
      rv[u] = in ? p[static_cast<int64_t>(t0 + tt) * width + v_off + h * vdim + c] : 0.f;
    }
    rgate[0] = rgate[1] = 0.f;
    if (tid < nb) {
      const float* row = p + static_cast<int64_t>(t0 + tid) * width;
      rgate[0] = row[i_off + h];
      rgate[1] = row[f_off + h];
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int u = 0; u < kPer; ++u) {
      const int idx = tid + u * 256;
      const int tt = idx / MAXD;
      const int r = idx - tt * MAXD;
      sq[tt][r / R][r % R] = rq[u];
      sk[tt][r / R][r % R] = rk[u];
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int idx = tid + u * 256;
      sv[idx / 64][idx % 64] = rv[u];
    }
    if (tid < kMemTokens) {
      sg[tid][0] = cap * tanhf(rgate[0] / cap);
      sg[tid][1] = log_sigmoid(cap * tanhf(rgate[1] / cap));
    }
  };
  fetch(t_begin);

  // n is the same for every column: a wavefront's 64 lanes share its rows among them (lane (g, c) holds rows
  // g * R + c * NR .. + NR - 1) and n . q is a sum over the wavefront
  constexpr int NR = R / 16;
  const int n_at = (lane % 16) * NR;  // within the lane's group of rows
  float C[R], n[NR];
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const int r = g * R + j;
    C[j] = (r < dim && !fresh && col_ok) ? src[static_cast<int64_t>(r) * vdim + col] : 0.f;
  }
#pragma unroll
  for (int u = 0; u < NR; ++u) {
    const int r = g * R + n_at + u;
    n[u] = (r < dim && !fresh) ? src[static_cast<int64_t>(dim) * vdim + r] : 0.f;
  }
  float m = fresh ? (MODE == kRunSums ? -INFINITY : 0.f) : src[static_cast<int64_t>(dim) * vdim + dim];
  float f_sum = 0.f;

  for (int t0 = t_begin; t0 < t_end; t0 += kMemTokens) {
    const int nb = min(kMemTokens, t_end - t0);
    __syncthreads();  // the tokens before are walked
    stash();
    __syncthreads();
    if (t0 + kMemTokens < t_end) fetch(t0 + kMemTokens);  // on their way during the walk
    for (int tt = 0; tt < nb; ++tt) {
      const float ig = sg[tt][0];
      const float fg = sg[tt][1];
      const float m_new = fmaxf(fg + m, ig);
      const float keep = expf(fg + m - m_new);  // exp(-inf) = 0 where a run starts from nothing
      const float take = expf(ig - m_new);
      m = m_new;
      f_sum += fg;
      const float v = sv[tt][c_local] * take;
      float num = 0.f, nq = 0.f;
#pragma unroll
      for (int u = 0; u < NR; ++u) {
        n[u] = fmaf(keep, n[u], sk[tt][g][n_at + u] * take);
        nq = fmaf(n[u], sq[tt][g][n_at + u], nq);
      }
#pragma unroll
      for (int j = 0; j < R; j += 4) {
        const f32x4 k4 = *reinterpret_cast<const f32x4*>(&sk[tt][g][j]);
        const f32x4 q4 = *reinterpret_cast<const f32x4*>(&sq[tt][g][j]);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          C[j + e] = fmaf(keep, C[j + e], k4[e] * v);
          if constexpr (MODE != kRunSums) num = fmaf(C[j + e], q4[e], num);
        }
      }
      if constexpr (MODE != kRunSums) {
        num += __shfl_xor(num, 16, kWave);
        num += __shfl_xor(num, 32, kWave);
        nq = wave_sum(nq);
        if (g == 0 && col_ok)
          out[(static_cast<int64_t>(t0 + tt) * heads + h) * vdim + col] = num / (fmaxf(fabsf(nq), expf(-m)) + 1e-6f);
      }
    }
  }
  if constexpr (MODE == kRunScan) return;  // the carry has left the entry's last state in its row
  if constexpr (MODE == kRunSums) {
    if (blockIdx.z == 0 && tid == 0) {
      run_gates[(static_cast<int64_t>(blockIdx.x) * heads + h) * 2] = f_sum;
      run_gates[(static_cast<int64_t>(blockIdx.x) * heads + h) * 2 + 1] = m;
    }
  }
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const int r = g * R + j;
    if (r < dim && col_ok) dst[static_cast<int64_t>(r) * vdim + col] = C[j];
  }
  if (blockIdx.z == 0 && wave == 0) {
#pragma unroll
    for (int u = 0; u < NR; ++u) {
      const int r = g * R + n_at + u;
      if (r < dim) dst[static_cast<int64_t>(dim) * vdim + r] = n[u];
    }
  }
  if (MODE == kWholeEntries && blockIdx.z == 0 && tid == 0) dst[static_cast<int64_t>(dim) * vdim + dim] = m;
}

// One thread per element of a head's C and n: walks its entry's runs in order (see kMemRun above).
__global__ __launch_bounds__(256) void matrix_memory_carry_kernel(
    float* __restrict__ runs, const float* __restrict__ run_gates, float* __restrict__ state,
    const int* __restrict__ read_rows, const int* __restrict__ write_rows, const int* __restrict__ cu_q,
    const int* __restrict__ q_starts, int heads, int dim, int vdim) {
  const int entry = blockIdx.x;
  const int h = blockIdx.y;
  const int elem = blockIdx.z * 256 + threadIdx.x;
  const int cells = dim * vdim + dim;  // C and n; m sits behind them
  if (elem >= cells) return;
  const int64_t per_head = cells + 1;
  int first_run = 0;
  for (int e = 0; e < entry; ++e) first_run += (cu_q[e + 1] - cu_q[e] + kMemRun - 1) / kMemRun;
  const int count = (cu_q[entry + 1] - cu_q[entry] + kMemRun - 1) / kMemRun;
  const bool fresh = q_starts[entry] == 0;
  const float* src = state + (static_cast<int64_t>(read_rows[entry]) * heads + h) * per_head;
  float x = fresh ? 0.f : src[elem];
  float m = fresh ? 0.f : src[cells];
  for (int r = 0; r < count; ++r) {
    const int64_t at = static_cast<int64_t>(first_run + r) * heads + h;
    float* slot = runs + at * per_head;
    const float u = slot[elem];
    const float f_sum = run_gates[at * 2];
    const float m_u = run_gates[at * 2 + 1];
    slot[elem] = x;
    if (elem == 0) slot[cells] = m;
    const float m_new = fmaxf(f_sum + m, m_u);
    x = expf(f_sum + m - m_new) * x + expf(m_u - m_new) * u;
    m = m_new;
  }
  float* dst = state + (static_cast<int64_t>(write_rows[entry]) * heads + h) * per_head;
  dst[elem] = x;
  if (elem == 0) dst[cells] = m;
}

}  // namespace mlr

using namespace mlr;

extern "C" {

int mlr_streams_fill(const float* x, float* out, int tokens, int width, int streams, hipStream_t stream) {
  MLR_REQUIRE(x && out, "null pointer");
  MLR_REQUIRE(tokens > 0 && width > 0 && streams > 0 && streams <= kMaxStreams, "sizes must be > 0, at most 16 streams");
  const int64_t plane = static_cast<int64_t>(tokens) * width;
  streams_fill_kernel<<<static_cast<unsigned>((plane + 255) / 256), 256, 0, stream>>>(x, out, plane, streams);
  MLR_LAUNCH_CHECK();
  return 0;
}

int mlr_streams_step(float* x, int streams, int tokens, int width, const int* rows, int out_rows, const void* y,
                     int y_is_f32, int slices, const float* mix, const float* out_w, const float* in_w,
                     const void* norm_w, int norm_is_f32, float eps, void* h_out, float* sum_out, int dtype,
                     hipStream_t stream) {
  MLR_REQUIRE(x, "null pointer");
  MLR_REQUIRE(tokens > 0 && width > 0 && streams > 0 && streams <= kMaxStreams, "sizes must be > 0, at most 16 streams");
  MLR_REQUIRE(out_rows > 0 && (rows != nullptr || out_rows == tokens), "without chosen rows every token is a row");
  MLR_REQUIRE(y == nullptr || (mix && out_w), "an update needs its mixing matrix and output weights");
  MLR_REQUIRE(slices >= 0 && (slices == 0 || (y && y_is_f32)), "partial sums are float32");
  MLR_REQUIRE(h_out == nullptr || norm_w, "normed activations need a norm weight");
  MLR_REQUIRE(dtype == kF32 || dtype == kBF16, "dtype must be 0 (float32) or 1 (bfloat16)");
  if (streams <= 4 && width % 4 == 0 && width <= 256 * 4 * kStreamGroups) {
#define MLR_STREAMS(T, S)                                                                                          \
  streams_step_rows_kernel<T, S><<<out_rows, 256, 0, stream>>>(x, tokens, width, rows, y, y_is_f32, slices, mix, out_w, \
                                                               in_w, norm_w, norm_is_f32, eps, static_cast<T*>(h_out), \
                                                               sum_out)
#define MLR_STREAMS_OF(T)   \
  do {                      \
    if (streams == 1)       \
      MLR_STREAMS(T, 1);    \
    else if (streams == 2)  \
      MLR_STREAMS(T, 2);    \
    else if (streams == 3)  \
      MLR_STREAMS(T, 3);    \
    else                    \
      MLR_STREAMS(T, 4);    \
  } while (0)
    if (dtype == kF32)
      MLR_STREAMS_OF(float);
    else
      MLR_STREAMS_OF(bf16);
#undef MLR_STREAMS_OF
#undef MLR_STREAMS
    MLR_LAUNCH_CHECK();
    return 0;
  }
  if (dtype == kF32)
    streams_step_kernel<float><<<out_rows, 256, 0, stream>>>(x, streams, tokens, width, rows, y, y_is_f32, slices, mix,
                                                             out_w, in_w, norm_w, norm_is_f32, eps,
                                                             static_cast<float*>(h_out), sum_out);
  else
    streams_step_kernel<bf16><<<out_rows, 256, 0, stream>>>(x, streams, tokens, width, rows, y, y_is_f32, slices, mix,
                                                            out_w, in_w, norm_w, norm_is_f32, eps,
                                                            static_cast<bf16*>(h_out), sum_out);
  MLR_LAUNCH_CHECK();
  return 0;
}

int mlr_head_norm_rope_write(const float* projected, int width, void* q_out, float* gate, const float* cos,
                             const float* sin, int rotary_dims, float eps, const int* slots, void* key_pages,
                             void* value_pages, float* v_keep, const float* v_first, const float* lambda, int dtype,
                             int tokens, int heads, int kv_heads, int dim, int vdim, int kernel_dim, int block_size,
                             int num_pages, hipStream_t stream) {
  MLR_REQUIRE(projected && q_out && slots && key_pages && value_pages, "null pointer");
  MLR_REQUIRE(tokens > 0 && heads > 0 && kv_heads > 0 && dim > 0 && vdim > 0, "sizes must be > 0");
  MLR_REQUIRE(kernel_dim >= dim && kernel_dim >= vdim, "the kernels' head size must hold keys and values");
  MLR_REQUIRE(rotary_dims >= 0 && rotary_dims % 2 == 0 && rotary_dims <= dim, "rotary_dims must be even and within dim");
  MLR_REQUIRE(rotary_dims == 0 || (cos && sin), "a rotation needs cos and sin tables");
  MLR_REQUIRE(width >= (heads + kv_heads) * dim + kv_heads * vdim + (gate ? heads : 0), "the projected rows are too narrow");
  MLR_REQUIRE(v_first == nullptr || lambda, "mixing values in needs its weight");
  MLR_REQUIRE(block_size > 0 && num_pages > 0, "page sizes must be > 0");
  MLR_REQUIRE(dtype == kF32 || dtype == kBF16, "dtype must be 0 (float32) or 1 (bfloat16)");
  if (dtype == kF32)
    head_norm_rope_write_kernel<float><<<tokens, 256, 0, stream>>>(
        projected, width, static_cast<float*>(q_out), gate, cos, sin, rotary_dims, eps, slots,
        static_cast<float*>(key_pages), static_cast<float*>(value_pages), v_keep, v_first, lambda, heads, kv_heads, dim,
        vdim, kernel_dim, block_size, num_pages);
  else
    head_norm_rope_write_kernel<bf16><<<tokens, 256, 0, stream>>>(
        projected, width, static_cast<bf16*>(q_out), gate, cos, sin, rotary_dims, eps, slots,
        static_cast<bf16*>(key_pages), static_cast<bf16*>(value_pages), v_keep, v_first, lambda, heads, kv_heads, dim,
        vdim, kernel_dim, block_size, num_pages);
  MLR_LAUNCH_CHECK();
  return 0;
}

// The most runs that `tokens` tokens in `entries` entries make (every entry may end in a run that is not full).
int mlr_matrix_memory_runs(int tokens, int entries) { return tokens / kMemRun + entries; }

int mlr_matrix_memory_scan(const float* projected, int width, int q_off, int k_off, int v_off, int i_off, int f_off,
                           float* state, int state_rows, const int* read_rows, const int* write_rows, const int* cu_q,
                           const int* q_starts, float cap, float q_scale, float* out, int entries, int heads, int dim,
                           int vdim, int tokens, float* runs, float* run_gates, hipStream_t stream) {
  MLR_REQUIRE(projected && state && read_rows && write_rows && cu_q && q_starts && out, "null pointer");
  MLR_REQUIRE((runs == nullptr) == (run_gates == nullptr) && (runs == nullptr || tokens > 0), "runs come with their gates' sums");
  MLR_REQUIRE(entries > 0 && heads > 0 && heads < 65536 && dim > 0 && vdim > 0 && state_rows > 0, "sizes must be > 0");
  MLR_REQUIRE(dim <= 256, "heads of up to 256 dims");
  MLR_REQUIRE(cap > 0.f, "the gates' cap must be > 0");
  MLR_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && i_off >= 0 && f_off >= 0 && q_off + heads * dim <= width &&
                  k_off + heads * dim <= width && v_off + heads * vdim <= width && i_off + heads <= width &&
                  f_off + heads <= width,
              "the projected rows do not hold what the offsets name");
#define MLR_MEMORY(R, MODE, FIRST)                                                                                \
  matrix_memory_scan_kernel<R, MODE><<<dim3(FIRST, heads, (vdim + 63) / 64), 256, 0, stream>>>(                    \
      projected, width, q_off, k_off, v_off, i_off, f_off, state, read_rows, write_rows, cu_q, q_starts, cap,     \
      q_scale, out, heads, dim, vdim, entries, runs, run_gates)
#define MLR_MEMORY_SIZED(MODE, FIRST) \
  do {                                \
    if (dim <= 64)                    \
      MLR_MEMORY(16, MODE, FIRST);    \
    else if (dim <= 128)              \
      MLR_MEMORY(32, MODE, FIRST);    \
    else                              \
      MLR_MEMORY(64, MODE, FIRST);    \
  } while (0)
  if (runs == nullptr) {
    MLR_MEMORY_SIZED(kWholeEntries, entries);
    MLR_LAUNCH_CHECK();
    return 0;
  }
  const int most = mlr_matrix_memory_runs(tokens, entries);
  MLR_MEMORY_SIZED(kRunSums, most);
  MLR_LAUNCH_CHECK();
  matrix_memory_carry_kernel<<<dim3(entries, heads, (dim * vdim + dim + 255) / 256), 256, 0, stream>>>(
      runs, run_gates, state, read_rows, write_rows, cu_q, q_starts, heads, dim, vdim);
  MLR_LAUNCH_CHECK();
  MLR_MEMORY_SIZED(kRunScan, most);
  MLR_LAUNCH_CHECK();
#undef MLR_MEMORY_SIZED
#undef MLR_MEMORY
  return 0;
}

}  // extern "C"
