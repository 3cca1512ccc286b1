// Kernels of mixers and arrangements beyond grouped-query attention: a sublayer's output added
// to the stream through a norm of its own, the gating of a clamped feed-forward, what a
// latent-attention layer does between its input product and the attention kernels, products with
// one small matrix per head, and retention (linear attention with a decaying matrix state).
// All arithmetic is float32; bfloat16 only exists in memory.
#include "api.h"
#include "common.h"
#include "mfma.h"

namespace mlr {

typedef float f32x4v __attribute__((ext_vector_type(4)));

// ---- x += weight * y * rsqrt(mean(y^2) + eps), then what reads the stream next -----------------
// y is one tensor (float32 or the engine's dtype) or `slices` float32 partial sums added in slice
// order.  mode 1: out = next_weight * x * rsqrt(mean(x^2) + next_eps); mode 2: out = x rounded to the
// engine's dtype; mode 0: nothing more.  One workgroup per row; the row stays in LDS between the
// passes, and a thread only ever reads the elements it wrote itself.
template <typename T>
__global__ __launch_bounds__(256) void add_normed_kernel(float* __restrict__ x, const void* __restrict__ y,
                                                         int y_is_f32, int slices, int rows,
                                                         const void* __restrict__ weight, int weight_is_f32, float eps,
                                                         const void* __restrict__ next_weight, int next_is_f32,
                                                         float next_eps, int mode, T* __restrict__ out, int hidden) {
  extern __shared__ float row_lds[];
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += 256) {
    float v;
    if (slices > 0) {
      v = 0.f;
      const float* p = static_cast<const float*>(y);
      for (int s = 0; s < slices; ++s) v += p[(static_cast<int64_t>(s) * rows + row) * hidden + i];
    } else {
      v = y_is_f32 ? static_cast<const float*>(y)[row * hidden + i] : to_f32(static_cast<const T*>(y)[row * hidden + i]);
    }
    row_lds[i] = v;
    ss += v * v;
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / static_cast<float>(hidden) + eps);
  float* xr = x + row * hidden;
  float ss2 = 0.f;
  for (int i = threadIdx.x; i < hidden; i += 256) {
    const float v = xr[i] + (row_lds[i] * inv) * load_as_f32(weight, i, weight_is_f32);
    xr[i] = v;
    row_lds[i] = v;
    ss2 += v * v;
  }
  if (mode == 0) return;
  T* orow = out + row * hidden;
  if (mode == 2) {
    for (int i = threadIdx.x; i < hidden; i += 256) orow[i] = from_f32<T>(row_lds[i]);
    return;
  }
  const float inv2 = 1.0f / sqrtf(block_sum(ss2, scratch) / static_cast<float>(hidden) + next_eps);
  for (int i = threadIdx.x; i < hidden; i += 256)
    orow[i] = from_f32<T>(load_as_f32(next_weight, i, next_is_f32) * (row_lds[i] * inv2));
}

// The same for rows whose width is a multiple of 4 and fits the registers of a workgroup: a thread keeps
// VPT groups of 4 elements between the passes, and all loads of a pass (every slice of partial sums
// included) are issued before the first is used: the kernel's time is the latency of its loads.
template <typename T, int VPT, int THREADS>
__global__ __launch_bounds__(THREADS) void add_normed_rows_kernel(
    float* __restrict__ x, const void* __restrict__ y, int y_is_f32, int slices, int rows,
    const void* __restrict__ weight, int weight_is_f32, float eps, const void* __restrict__ next_weight,
    int next_is_f32, float next_eps, int mode, T* __restrict__ out, int hidden) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  const int quads = hidden / 4;
  constexpr int kSliceBatch = 8;
  f32x4v v[VPT], xv[VPT], wv[VPT], nv[VPT];
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int i = min(static_cast<int>(threadIdx.x) + j * THREADS, quads - 1);
    const int64_t at = row * hidden + 4 * i;
    xv[j] = *reinterpret_cast<const f32x4v*>(x + at);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      wv[j][e] = load_as_f32(weight, 4 * i + e, weight_is_f32);
      nv[j][e] = mode == 1 ? load_as_f32(next_weight, 4 * i + e, next_is_f32) : 0.f;
    }
    if (slices > 0) {
      v[j] = f32x4v{0.f, 0.f, 0.f, 0.f};
    } else if (y_is_f32) {
      v[j] = *reinterpret_cast<const f32x4v*>(static_cast<const float*>(y) + at);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) v[j][e] = to_f32(static_cast<const T*>(y)[at + e]);
    }
  }
  for (int s0 = 0; s0 < slices; s0 += kSliceBatch) {
    f32x4v part[VPT][kSliceBatch];
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
      const int i = min(static_cast<int>(threadIdx.x) + j * THREADS, quads - 1);
#pragma unroll
      for (int u = 0; u < kSliceBatch; ++u) {
        const int sl = min(s0 + u, slices - 1);
        part[j][u] = *reinterpret_cast<const f32x4v*>(static_cast<const float*>(y) +
                                                      (static_cast<int64_t>(sl) * rows + row) * hidden + 4 * i);
      }
    }
#pragma unroll
    for (int u = 0; u < kSliceBatch; ++u) {
      const bool live = s0 + u < slices;
#pragma unroll
      for (int j = 0; j < VPT; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) v[j][e] = live ? v[j][e] + part[j][u][e] : v[j][e];
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    if (static_cast<int>(threadIdx.x) + j * THREADS >= quads) v[j] = f32x4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int e = 0; e < 4; ++e) ss += v[j][e] * v[j][e];
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / static_cast<float>(hidden) + eps);
  float ss2 = 0.f;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int i = threadIdx.x + j * THREADS;
    if (i >= quads) {
      xv[j] = f32x4v{0.f, 0.f, 0.f, 0.f};
      continue;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      xv[j][e] += (v[j][e] * inv) * wv[j][e];
      ss2 += xv[j][e] * xv[j][e];
    }
    *reinterpret_cast<f32x4v*>(x + row * hidden + 4 * i) = xv[j];
  }
  if (mode == 0) return;
  float inv2 = 1.0f;
  if (mode == 1) inv2 = 1.0f / sqrtf(block_sum(ss2, scratch) / static_cast<float>(hidden) + next_eps);
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int i = threadIdx.x + j * THREADS;
    if (i >= quads) continue;
    const int64_t at = row * hidden + 4 * i;
#pragma unroll
    for (int e = 0; e < 4; ++e) out[at + e] = from_f32<T>(mode == 1 ? nv[j][e] * (xv[j][e] * inv2) : xv[j][e]);
  }
}

template <typename T>
static void launch_add_normed(float* x, const void* y, int y_is_f32, int slices, const void* weight, int weight_is_f32,
                              float eps, const void* next_weight, int next_is_f32, float next_eps, int mode, void* out,
                              int rows, int hidden, hipStream_t stream) {
  T* o = static_cast<T*>(out);
  const int quads = hidden / 4;
#define MLR_ROWS(VPT, THREADS)                                                                                     \
  add_normed_rows_kernel<T, VPT, THREADS><<<rows, THREADS, 0, stream>>>(x, y, y_is_f32, slices, rows, weight,     \
                                                                        weight_is_f32, eps, next_weight, next_is_f32, \
                                                                        next_eps, mode, o, hidden)
  if (hidden % 4 != 0 || quads > 2048)
    add_normed_kernel<T><<<rows, 256, static_cast<size_t>(hidden) * sizeof(float), stream>>>(
        x, y, y_is_f32, slices, rows, weight, weight_is_f32, eps, next_weight, next_is_f32, next_eps, mode, o, hidden);
  else if (rows <= 64 && quads > 512)
    MLR_ROWS(2, 1024);
  else if (rows <= 64 && quads > 256)
    MLR_ROWS(1, 1024);
  else if (quads <= 256)
    MLR_ROWS(1, 256);
  else if (quads <= 512)
    MLR_ROWS(2, 256);
  else if (quads <= 1024)
    MLR_ROWS(4, 256);
  else
    MLR_ROWS(8, 256);
#undef MLR_ROWS
}

// ---- g = min(gate, limit), u = clamp(up, -limit, limit): g * sigmoid(alpha g) * (u + 1) ---------
// sums [rows, 2 * inter]: the gate sums, then the up sums.
template <typename TI, typename T>
__global__ __launch_bounds__(256) void glu_clamped_kernel(const TI* __restrict__ sums, T* __restrict__ out, int rows,
                                                          int inter, float limit, float alpha) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= static_cast<int64_t>(rows) * inter) return;
  const int64_t m = i / inter;
  const int64_t c = i - m * inter;
  const float g = fminf(to_f32(sums[m * 2 * inter + c]), limit);
  const float u = fminf(fmaxf(to_f32(sums[m * 2 * inter + inter + c]), -limit), limit);
  out[i] = from_f32<T>(g / (1.0f + expf(-alpha * g)) * (u + 1.0f));
}

// ---- latent attention: between the input product and the attention kernels ----------------------
// `p` [tokens, width] float32 holds, per token: the queries (per head `dim` unrotated then `rot`
// rotated dims), then (own_cache) the latent of `rank` dims and the shared key part of `rot` dims,
// then (gated) one gate logit per head.  Per token this
//  * rounds the unrotated query parts into q_plain [tokens, heads * dim],
//  * rotates the rotated query parts into columns rank .. rank + rot of every head's latent query
//    (q_latent [tokens, heads * D]; columns beyond rank + rot are cleared, the first `rank` belong
//    to the product that follows),
//  * (own_cache) norms the latent (weight, eps), rotates the key part, and stores the row
//    [latent ; key part ; 0] at slot[t] of the key pages [page, 1, offset, D] and [latent ; 0]
//    of the value pages [page, 1, D, offset]; a negative slot stores nothing,
//  * (gated) gate[t, head] = sigmoid(logit), float32.
// The rotation takes the first `rdims` of the `rot` dims in two halves (pair j, j + rdims / 2).
template <typename T>
__global__ __launch_bounds__(256) void latent_prepare_kernel(
    const float* __restrict__ p, int width, T* __restrict__ q_plain, T* __restrict__ q_latent,
    float* __restrict__ gate, const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rdims,
    const void* __restrict__ norm_weight, int weight_is_f32, float eps, const int* __restrict__ slots,
    T* __restrict__ key_pages, T* __restrict__ value_pages, int heads, int dim, int rot, int rank, int D,
    int block_size, int num_pages, int own_cache, int gated, const float* __restrict__ queries, int q_width) {
  __shared__ float scratch[16];
  const int64_t t = blockIdx.x;
  const float* row = p + t * width;
  // the query sums: the leading columns of the row, or (a mixer whose queries go through a product of their
  // own) a row of another tensor, the row then starts with what follows the queries
  const float* qrow = queries != nullptr ? queries + t * q_width : row;
  const int half = rdims / 2;
  const float* cs = cos_t ? cos_t + t * half : nullptr;
  const float* sn = sin_t ? sin_t + t * half : nullptr;
  auto rotated = [&](const float* part, int j) {  // dim j of a rotated part of `rot` dims
    if (j >= rdims || cs == nullptr) return part[j];
    return j < half ? part[j] * cs[j] - part[j + half] * sn[j] : part[j] * cs[j - half] + part[j - half] * sn[j - half];
  };
  const int qd = dim + rot;
  for (int i = threadIdx.x; i < heads * dim; i += 256) {
    const int h = i / dim;
    q_plain[t * heads * dim + i] = from_f32<T>(qrow[h * qd + (i - h * dim)]);
  }
  const int tail = D - rank;  // columns of a latent query that this kernel owns
  for (int i = threadIdx.x; i < heads * tail; i += 256) {
    const int h = i / tail;
    const int j = i - h * tail;
    q_latent[(t * heads + h) * D + rank + j] = from_f32<T>(j < rot ? rotated(qrow + h * qd + dim, j) : 0.f);
  }
  int at = queries != nullptr ? 0 : heads * qd;
  if (own_cache) {
    const float* c = row + at;
    float ss = 0.f;
    for (int i = threadIdx.x; i < rank; i += 256) ss += c[i] * c[i];
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / static_cast<float>(rank) + eps);
    const int slot = slots[t];
    if (slot >= 0) {
      const int page = slot / block_size;
      const int off = slot - page * block_size;
      if (page < num_pages) {
        T* krow = key_pages + (static_cast<int64_t>(page) * block_size + off) * D;
        T* vcol = value_pages + static_cast<int64_t>(page) * D * block_size + off;
        for (int i = threadIdx.x; i < D; i += 256) {
          float kv = 0.f, vv = 0.f;
          if (i < rank) {
            kv = vv = (c[i] * inv) * load_as_f32(norm_weight, i, weight_is_f32);
          } else if (i < rank + rot) {
            kv = rotated(c + rank, i - rank);
          }
          krow[i] = from_f32<T>(kv);
          vcol[static_cast<int64_t>(i) * block_size] = from_f32<T>(vv);
        }
      }
    }
    at += rank + rot;
  }
  if (gated)
    for (int h = threadIdx.x; h < heads; h += 256) gate[t * heads + h] = 1.0f / (1.0f + expf(-row[at + h]));
}

// ---- one small matrix per head --------------------------------------------------------------------
// y[t, h, n] = sum_k x[t, h * in_stride + k] * w[h, n, k]  (times row_scale[t, h], float32, if given),
// stored at out[t * out_row + h * out_stride + n].  Plain float32 arithmetic, 64 x 64 output tile per
// workgroup and head, 16-wide slices of k through LDS, 4 x 4 outputs a lane.
template <typename T>
__global__ __launch_bounds__(256) void heads_linear_kernel(const T* __restrict__ x, int64_t in_row, int in_stride,
                                                           const T* __restrict__ w, T* __restrict__ out,
                                                           int64_t out_row, int out_stride,
                                                           const float* __restrict__ row_scale, int heads, int M,
                                                           int N, int K) {
  __shared__ float xs[16][64 + 4];
  __shared__ float ws[16][64 + 4];
  const int tid = threadIdx.x;
  const int tm = tid / 16;
  const int tn = tid % 16;
  const int h = blockIdx.z;
  const int64_t m0 = static_cast<int64_t>(blockIdx.y) * 64;
  const int64_t n0 = static_cast<int64_t>(blockIdx.x) * 64;
  const T* xh = x + static_cast<int64_t>(h) * in_stride;
  const T* wh = w + static_cast<int64_t>(h) * N * K;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  for (int k0 = 0; k0 < K; k0 += 16) {
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int idx = tid + it * 256;
      const int r = idx / 16;
      const int kk = idx % 16;
      const int64_t gk = k0 + kk;
      xs[kk][r] = (m0 + r < M && gk < K) ? to_f32(xh[(m0 + r) * in_row + gk]) : 0.f;
      ws[kk][r] = (n0 + r < N && gk < K) ? to_f32(wh[(n0 + r) * K + gk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[kk][tm * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[kk][tn * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t gm = m0 + tm * 4 + i;
    if (gm >= M) continue;
    const float s = row_scale ? row_scale[gm * heads + h] : 1.0f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t gn = n0 + tn * 4 + j;
      if (gn < N) out[gm * out_row + static_cast<int64_t>(h) * out_stride + gn] = from_f32<T>(acc[i][j] * s);
    }
  }
}

// The same product in bfloat16 on the matrix cores: a wavefront owns 16 tokens x (16 NT) outputs of one
// head and reads both operands straight from memory, 8 consecutive k a lane (the matrices are small:
// what one wavefront reads again, another has left in L2).  The weights are the A operand, so a lane
// ends up with 4 consecutive outputs of one token.  k is a multiple of 8; rows and head strides keep
// every 8 k values 16-byte aligned.
template <int NT>
__global__ __launch_bounds__(64) void heads_linear_mfma_kernel(const bf16* __restrict__ x, int64_t in_row, int in_stride,
                                                               const bf16* __restrict__ w, bf16* __restrict__ out,
                                                               int64_t out_row, int out_stride,
                                                               const float* __restrict__ row_scale, int heads, int M,
                                                               int N, int K) {
  const int lane = threadIdx.x;
  const int r16 = lane % 16;
  const int quad = lane / 16;
  const int h = blockIdx.z;
  const int m0 = blockIdx.y * 16;
  const int n0 = blockIdx.x * 16 * NT;
  const int t = min(m0 + r16, M - 1);  // rows past the end read the last row; their results are dropped
  const bf16* xrow = x + static_cast<int64_t>(t) * in_row + static_cast<int64_t>(h) * in_stride;
  const bf16* wh = w + static_cast<int64_t>(h) * N * K;
  f32x4_t acc[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) acc[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += 32) {
    const int k = k0 + quad * 8;
    const bool inside = k < K;
    const bf16x8_t b = inside ? load_bf16x8(xrow + k) : zero_bf16x8();
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const int n = min(n0 + 16 * j + r16, N - 1);
      const bf16x8_t a = inside ? load_bf16x8(wh + static_cast<int64_t>(n) * K + k) : zero_bf16x8();
      acc[j] = mfma_16x16x32(a, b, acc[j]);
    }
  }
  if (m0 + r16 >= M) return;
  const float scale = row_scale ? row_scale[static_cast<int64_t>(m0 + r16) * heads + h] : 1.0f;
  bf16* orow = out + static_cast<int64_t>(m0 + r16) * out_row + static_cast<int64_t>(h) * out_stride;
#pragma unroll
  for (int j = 0; j < NT; ++j) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int n = n0 + 16 * j + 4 * quad + e;
      if (n < N) orow[n] = f32_to_bf16(acc[j][e] * scale);
    }
  }
}

// ---- retention ------------------------------------------------------------------------------------
// S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t per (entry, head), the entry's tokens in order.
// `p` [tokens, width] float32 holds q (heads * dim), k (heads * dim), v (heads * vdim) and more; q and
// k are rotated here (first rdims dims of a head in two halves) and k scaled by key_scale, all in
// float32.  A wavefront owns 16 columns of one head's state: lane = (group of dims g = lane / 16,
// column c = lane % 16) keeps S[d][c] for d = 4 i + g in registers.  Tokens are taken kBatch at a
// time: their rotated q and k and their v go to LDS first, so the trip to memory is paid once per
// batch and the chain from token to token is arithmetic only.  The state is read from row
// read_rows[entry] of `state` [rows, heads, dim, vdim] (zeros when the entry starts its request) and
// left in row write_rows[entry].  out [tokens, heads * vdim] float32.
constexpr int kRetBatch = 8;

template <int DPL>  // dims per lane: dim <= 4 * DPL
__global__ __launch_bounds__(64) void retention_scan_kernel(
    const float* __restrict__ p, int width, float* __restrict__ state, const int* __restrict__ read_rows,
    const int* __restrict__ write_rows, const int* __restrict__ cu_q, const int* __restrict__ q_starts,
    const float* __restrict__ decay, const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rdims,
    float key_scale, float* __restrict__ out, int heads, int dim, int vdim) {
  __shared__ float qs[kRetBatch][4 * DPL];
  __shared__ float ks[kRetBatch][4 * DPL];
  __shared__ float vs[kRetBatch][16];
  const int entry = blockIdx.x;
  const int h = blockIdx.y;
  const int v0 = blockIdx.z * 16;
  const int lane = threadIdx.x;
  const int g = lane / 16;
  const int c = lane % 16;
  const bool column = v0 + c < vdim;
  const int t_first = cu_q[entry];
  const int t_end = cu_q[entry + 1];
  const float gamma = decay[h];
  const int half = rdims / 2;
  const int64_t head_state = static_cast<int64_t>(dim) * vdim;

  float S[DPL];
  const bool carried = q_starts[entry] > 0;
  const float* src = state + (static_cast<int64_t>(read_rows[entry]) * heads + h) * head_state;
#pragma unroll
  for (int i = 0; i < DPL; ++i) {
    const int d = 4 * i + g;
    S[i] = (carried && column && d < dim) ? src[static_cast<int64_t>(d) * vdim + v0 + c] : 0.f;
  }

  for (int tb = t_first; tb < t_end; tb += kRetBatch) {
    const int count = min(kRetBatch, t_end - tb);
    __syncthreads();  // the batch before is done with
    for (int idx = lane; idx < count * dim; idx += 64) {
      const int u = idx / dim;
      const int d = idx - u * dim;
      const int64_t t = tb + u;
      const float* q = p + t * width + static_cast<int64_t>(h) * dim;
      const float* k = q + static_cast<int64_t>(heads) * dim;
      float qv = q[d], kv = k[d];
      if (d < rdims && cos_t != nullptr) {
        const int j = d < half ? d : d - half;
        const float cv = cos_t[t * half + j], sv = sin_t[t * half + j];
        const int partner = d < half ? d + half : d - half;
        const float sign = d < half ? -1.f : 1.f;
        qv = qv * cv + sign * q[partner] * sv;
        kv = kv * cv + sign * k[partner] * sv;
      }
      qs[u][d] = qv;
      ks[u][d] = kv * key_scale;
    }
    for (int idx = lane; idx < count * 16; idx += 64) {
      const int u = idx / 16;
      const int cc = idx - u * 16;
      vs[u][cc] = v0 + cc < vdim
                      ? p[static_cast<int64_t>(tb + u) * width + 2ll * heads * dim + static_cast<int64_t>(h) * vdim + v0 + cc]
                      : 0.f;
    }
    __syncthreads();
    for (int u = 0; u < count; ++u) {
      const float vv = vs[u][c];
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < DPL; ++i) {
        const int d = 4 * i + g;
        if (d < dim) {
          S[i] = fmaf(gamma, S[i], ks[u][d] * vv);
          o = fmaf(S[i], qs[u][d], o);
        }
      }
      o += __shfl_xor(o, 16, kWave);
      o += __shfl_xor(o, 32, kWave);
      if (g == 0 && column) out[static_cast<int64_t>(tb + u) * heads * vdim + static_cast<int64_t>(h) * vdim + v0 + c] = o;
    }
  }
  float* dst = state + (static_cast<int64_t>(write_rows[entry]) * heads + h) * head_state;
#pragma unroll
  for (int i = 0; i < DPL; ++i) {
    const int d = 4 * i + g;
    if (column && d < dim) dst[static_cast<int64_t>(d) * vdim + v0 + c] = S[i];
  }
}

// q and k of `p` ([tokens, width] float32: q, then k, heads * dim each) rotated in place and k
// scaled: what the chunked kernel below reads.  A thread owns a pair (d, d + rdims / 2) or an
// unrotated dim.
__global__ __launch_bounds__(256) void retention_rotate_kernel(float* __restrict__ p, int width,
                                                               const float* __restrict__ cos_t,
                                                               const float* __restrict__ sin_t, int rdims,
                                                               float key_scale, int heads, int dim) {
  const int64_t t = blockIdx.x;
  const int half = rdims / 2;
  float* q = p + t * width;
  float* k = q + static_cast<int64_t>(heads) * dim;
  for (int idx = threadIdx.x; idx < heads * dim; idx += 256) {
    const int h = idx / dim;
    const int d = idx - h * dim;
    if (d >= rdims || cos_t == nullptr) {
      k[idx] *= key_scale;
    } else if (d < half) {
      const float c = cos_t[t * half + d], sn = sin_t[t * half + d];
      const float q0 = q[idx], q1 = q[idx + half], k0 = k[idx], k1 = k[idx + half];
      q[idx] = q0 * c - q1 * sn;
      q[idx + half] = q1 * c + q0 * sn;
      k[idx] = (k0 * c - k1 * sn) * key_scale;
      k[idx + half] = (k1 * c + k0 * sn) * key_scale;
    }
  }
}

// The same recurrence for entries of many tokens, a chunk of 64 tokens at a time, on the matrix
// cores in true 32-bit (v_mfma_f32_16x16x4_f32: operands and sums are float32).  With S the state
// before a chunk of n tokens (local index i, j), g the decay and A_ij = (q_i . k_j) g^(i-j) for j <= i:
//     o_i = g^(i+1) S^T q_i + sum_j A_ij v_j,      S' = g^n S + U,   U = sum_j g^(n-1-j) k_j v_j^T.
// q and k come rotated and scaled (retention_rotate_kernel).  Only S links the chunks, so the work is
// cut in two.  retention_local_kernel: a workgroup per (chunk, head, 16 value columns), all chunks of
// all entries at once, makes the chunk's own part of o (the sum over j) and its U.
// retention_state_kernel walks every entry's chunks in order, element by element (S' = g^n S + U needs no
// product), and leaves the state before every chunk; retention_apply_kernel, all chunks at once again, adds
// g^(i+1) S^T q_i to o.  The chain from chunk to chunk is one multiply-add an element.
// Wavefront w of four owns the query rows 16 w .. 16 w + 15 of a chunk and, in the first kernel, every
// fourth 16-row tile of U.  LDS of the first kernel: the chunk's q and k [64][DP + 4] (DP: dim rounded up
// to 16, 32, 64 or 128, zero padded; rows 4 words apart modulo 32 keep the operand reads of 16 rows x 4
// columns off each other's banks), its values [64][16], the masked scores per wavefront [16][68], the
// powers g^0..g^64.
// Lane layouts of the product D[16x16] += A[16x4] B[4x16]: lane l holds A[l % 16][l / 16],
// B[l / 16][l % 16] and D[4 (l / 16) + e][l % 16], e = 0..3.
constexpr int kChunk = 64;
constexpr int kScoreLd = kChunk + 4;

__device__ __forceinline__ f32x4v mfma_f32(float a, float b, f32x4v c) {
  return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

// Chunks are numbered through the entries in order, an entry of n tokens having ceil(n / 64).
__device__ __forceinline__ int chunks_of(int tokens) { return (tokens + kChunk - 1) / kChunk; }

template <int DP>
__global__ __launch_bounds__(256) void retention_local_kernel(const float* __restrict__ p, int width,
                                                              const int* __restrict__ cu_q,
                                                              const float* __restrict__ decay, float* __restrict__ out,
                                                              float* __restrict__ local, int entries, int heads, int dim,
                                                              int vdim, int vpad) {
  extern __shared__ float chunk_lds[];
  constexpr int LD = DP + 4;
  float* const Qs = chunk_lds;                    // [64][LD]
  float* const Ks = Qs + kChunk * LD;             // [64][LD]
  float* const Vs = Ks + kChunk * LD;             // [64][16]
  float* const As = Vs + kChunk * 16;             // [4][16][kScoreLd]
  float* const pw = As + 4 * 16 * kScoreLd;       // [65]
  int entry = -1, left = blockIdx.x;
  for (int e = 0; e < entries; ++e) {
    const int have = chunks_of(cu_q[e + 1] - cu_q[e]);
    if (left < have) {
      entry = e;
      break;
    }
    left -= have;
  }
  if (entry < 0) return;  // the grid is sized for the most chunks that the step's tokens could make
  const int tb = cu_q[entry] + left * kChunk;
  const int n = min(kChunk, cu_q[entry + 1] - tb);
  const int h = blockIdx.y;
  const int tid = threadIdx.x;
  const int lane = tid % kWave;
  const int w = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int r16 = lane % 16;
  const int quad = lane / 16;
  const float gamma = decay[h];
  float* const As_w = As + w * 16 * kScoreLd;

  if (tid <= kChunk) pw[tid] = powf(gamma, static_cast<float>(tid));  // g^0 = 1 also when g = 0
  // loads are unconditional (a row past the end reads the chunk's last row, a dim past the head reads
  // the head's last dim); what does not exist is cleared on its way to LDS
  for (int idx = tid; idx < kChunk * (DP / 4); idx += 256) {
    const int i = idx / (DP / 4);
    const int d0 = 4 * (idx % (DP / 4));
    const float* q = p + static_cast<int64_t>(tb + min(i, n - 1)) * width + static_cast<int64_t>(h) * dim;
    const float* k = q + static_cast<int64_t>(heads) * dim;
    float qv[4], kv[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int d = min(d0 + e, dim - 1);
      qv[e] = q[d];
      kv[e] = k[d];
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const bool there = i < n && d0 + e < dim;
      Qs[i * LD + d0 + e] = there ? qv[e] : 0.f;
      Ks[i * LD + d0 + e] = there ? kv[e] : 0.f;
    }
  }
  __syncthreads();

  // scores of this wavefront's 16 queries against the key tiles up to the diagonal
  f32x4v sc[4];
#pragma unroll
  for (int jt = 0; jt < 4; ++jt) sc[jt] = f32x4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll 8
  for (int s = 0; s < DP / 4; ++s) {
    const int d = 4 * s + quad;
    const float a = Qs[(16 * w + r16) * LD + d];
#pragma unroll
    for (int jt = 0; jt < 4; ++jt)
      if (jt <= w) sc[jt] = mfma_f32(a, Ks[(16 * jt + r16) * LD + d], sc[jt]);
  }
#pragma unroll
  for (int jt = 0; jt < 4; ++jt) {
    if (jt > w) continue;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int i = 16 * w + 4 * quad + e;  // query, key: local indices of the chunk
      const int j = 16 * jt + r16;
      As_w[(4 * quad + e) * kScoreLd + j] = j <= i ? sc[jt][e] * pw[i - j] : 0.f;
    }
  }
  // the keys as the state takes them, k_j g^(n-1-j), in place (the scores are done with them)
  __syncthreads();
  for (int idx = tid; idx < kChunk * DP; idx += 256) {
    const int j = idx / DP;
    Ks[j * LD + idx % DP] *= j < n ? pw[n - 1 - j] : 0.f;
  }
  // the scores are made once; 16 value columns at a time go through them
  for (int v0 = 0; v0 < vdim; v0 += 16) {
    __syncthreads();  // the columns before are done with (and, the first time, the scores are whole)
    for (int idx = tid; idx < kChunk * 16; idx += 256) {
      const int i = idx / 16, c = idx % 16;
      const float v = p[static_cast<int64_t>(tb + min(i, n - 1)) * width + 2ll * heads * dim + static_cast<int64_t>(h) * vdim +
                        min(v0 + c, vdim - 1)];
      Vs[idx] = (i < n && v0 + c < vdim) ? v : 0.f;
    }
    __syncthreads();
    f32x4v o = {0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < 4 * (w + 1); ++s) {
      const int j = 4 * s + quad;
      o = mfma_f32(As_w[r16 * kScoreLd + j], Vs[j * 16 + r16], o);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int i = 16 * w + 4 * quad + e;
      if (i < n && v0 + r16 < vdim)
        out[static_cast<int64_t>(tb + i) * heads * vdim + static_cast<int64_t>(h) * vdim + v0 + r16] = o[e];
    }
    // what the chunk adds to the state: rows of tile dt, for every fourth tile
    float* dst = local + ((static_cast<int64_t>(blockIdx.x) * heads + h) * DP) * vpad + v0;
    for (int dt = w; dt < DP / 16; dt += 4) {
      f32x4v up[2] = {f32x4v{0.f, 0.f, 0.f, 0.f}, f32x4v{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
      for (int s = 0; s < kChunk / 4; ++s) {
        const int j = 4 * s + quad;
        up[s % 2] = mfma_f32(Ks[j * LD + 16 * dt + r16], Vs[j * 16 + r16], up[s % 2]);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) dst[static_cast<int64_t>(16 * dt + 4 * quad + e) * vpad + r16] = up[0][e] + up[1][e];
    }
  }
}

// The state from chunk to chunk: S' = g^n S + U, element by element.  A thread owns one element of a head's
// state and walks the entry's chunks; it leaves the state BEFORE every chunk where that chunk's U was
// (`local`), for retention_apply_kernel.  The U values do not depend on the chain, so four chunks' loads are
// on their way at a time.
__global__ __launch_bounds__(256) void retention_state_kernel(float* __restrict__ state, const int* __restrict__ read_rows,
                                                              const int* __restrict__ write_rows,
                                                              const int* __restrict__ cu_q, const int* __restrict__ q_starts,
                                                              const float* __restrict__ decay, float* __restrict__ local,
                                                              int heads, int dim, int vdim, int dp, int vpad) {
  const int entry = blockIdx.x;
  const int h = blockIdx.y;
  const int idx = blockIdx.z * 256 + threadIdx.x;
  if (idx >= dp * vpad) return;
  const int d = idx / vpad;
  const int v = idx - d * vpad;
  const bool real = d < dim && v < vdim;
  const int tokens = cu_q[entry + 1] - cu_q[entry];
  const int count = chunks_of(tokens);
  int first = 0;  // number of this entry's first chunk
  for (int e = 0; e < entry; ++e) first += chunks_of(cu_q[e + 1] - cu_q[e]);
  const float gamma = decay[h];
  const float whole = powf(gamma, static_cast<float>(kChunk));
  const float rest = powf(gamma, static_cast<float>(tokens - (count - 1) * kChunk));  // the last chunk's tokens
  const int64_t head_state = static_cast<int64_t>(dim) * vdim;
  float s = 0.f;
  if (real && q_starts[entry] > 0)
    s = state[(static_cast<int64_t>(read_rows[entry]) * heads + h) * head_state + static_cast<int64_t>(d) * vdim + v];
  float* u = local + ((static_cast<int64_t>(first) * heads + h) * dp) * vpad + idx;
  const int64_t step = static_cast<int64_t>(heads) * dp * vpad;
  for (int c0 = 0; c0 < count; c0 += 4) {
    float add[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) add[k] = u[static_cast<int64_t>(min(c0 + k, count - 1)) * step];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int c = c0 + k;
      if (c < count) {
        u[static_cast<int64_t>(c) * step] = s;
        s = (c == count - 1 ? rest : whole) * s + add[k];
      }
    }
  }
  if (real)
    state[(static_cast<int64_t>(write_rows[entry]) * heads + h) * head_state + static_cast<int64_t>(d) * vdim + v] = s;
}

// o_i += g^(i+1) S^T q_i for every chunk at once, S the state before the chunk as retention_state_kernel
// left it.  A workgroup per (chunk, head); wavefront w owns the query rows 16 w .. 16 w + 15, 16 value
// columns at a time; the chunk's q goes through LDS, the state comes straight from memory.
template <int DP>
__global__ __launch_bounds__(256) void retention_apply_kernel(const float* __restrict__ p, int width,
                                                              const int* __restrict__ cu_q,
                                                              const int* __restrict__ q_starts,
                                                              const float* __restrict__ decay, float* __restrict__ out,
                                                              const float* __restrict__ local, int entries, int heads,
                                                              int dim, int vdim, int vpad) {
  constexpr int LD = DP + 4;
  __shared__ float Qs[kChunk * LD];
  int entry = -1, left = blockIdx.x;
  for (int e = 0; e < entries; ++e) {
    const int have = chunks_of(cu_q[e + 1] - cu_q[e]);
    if (left < have) {
      entry = e;
      break;
    }
    left -= have;
  }
  if (entry < 0) return;  // the grid is sized for the most chunks that the step's tokens could make
  if (left == 0 && q_starts[entry] == 0) return;  // the first chunk of a request: the state before it is zero
  const int tb = cu_q[entry] + left * kChunk;
  const int n = min(kChunk, cu_q[entry + 1] - tb);
  const int h = blockIdx.y;
  const int tid = threadIdx.x;
  const int lane = tid % kWave;
  const int w = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int r16 = lane % 16;
  const int quad = lane / 16;
  const float gamma = decay[h];
  for (int idx = tid; idx < kChunk * (DP / 4); idx += 256) {
    const int i = idx / (DP / 4);
    const int d0 = 4 * (idx % (DP / 4));
    const float* q = p + static_cast<int64_t>(tb + min(i, n - 1)) * width + static_cast<int64_t>(h) * dim;
    float qv[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) qv[e] = q[min(d0 + e, dim - 1)];
#pragma unroll
    for (int e = 0; e < 4; ++e) Qs[i * LD + d0 + e] = (i < n && d0 + e < dim) ? qv[e] : 0.f;
  }
  __syncthreads();
  if (16 * w >= n) return;  // no query in this wavefront's rows
  float power[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) power[e] = powf(gamma, static_cast<float>(16 * w + 4 * quad + e + 1));
  const float* sb = local + ((static_cast<int64_t>(blockIdx.x) * heads + h) * DP) * vpad;
  for (int v0 = 0; v0 < vdim; v0 += 16) {
    f32x4v part[2] = {f32x4v{0.f, 0.f, 0.f, 0.f}, f32x4v{0.f, 0.f, 0.f, 0.f}};
#pragma unroll 8
    for (int s = 0; s < DP / 4; ++s)
      part[s % 2] = mfma_f32(Qs[(16 * w + r16) * LD + 4 * s + quad], sb[static_cast<int64_t>(4 * s + quad) * vpad + v0 + r16],
                             part[s % 2]);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int i = 16 * w + 4 * quad + e;
      if (i < n && v0 + r16 < vdim) {
        float* at = out + static_cast<int64_t>(tb + i) * heads * vdim + static_cast<int64_t>(h) * vdim + v0 + r16;
        *at += power[e] * (part[0][e] + part[1][e]);
      }
    }
  }
}

// out[t, h, :] = o / sqrt(mean(o^2) + eps) * w * act(z) * out_scale, o = retained[t, h, :] (float32), z = the gate
// sums at column gate_offset + h * vdim of p [tokens, width] (float32), w [vdim] a weight that all heads share, or
// with `weight_per_head` [heads * vdim] (null: none); act is silu (gate_kind 0) or the sigmoid (1).  A row of `out` is out_row elements long and the heads start at its column 0.  One wavefront
// per (token, head).
template <typename T>
__global__ __launch_bounds__(64) void retention_gate_kernel(const float* __restrict__ retained,
                                                            const float* __restrict__ p, int width, int gate_offset,
                                                            T* __restrict__ out, int64_t out_row, int heads, int vdim,
                                                            float eps, const void* __restrict__ norm_weight,
                                                            int weight_is_f32, float out_scale,
                                                            int weight_per_head, int gate_kind) {
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y;
  const int w0 = weight_per_head ? h * vdim : 0;
  const float* o = retained + (t * heads + h) * vdim;
  float ss = 0.f;
  for (int i = threadIdx.x; i < vdim; i += 64) ss += o[i] * o[i];
  const float inv = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(vdim) + eps);
  const float* z = p + t * width + gate_offset + static_cast<int64_t>(h) * vdim;
  T* dst = out + t * out_row + static_cast<int64_t>(h) * vdim;
  for (int i = threadIdx.x; i < vdim; i += 64) {
    const float zv = z[i];
    float normed = o[i] * inv;
    if (norm_weight != nullptr) normed *= load_as_f32(norm_weight, w0 + i, weight_is_f32);
    const float sg = 1.0f / (1.0f + expf(-zv));
    dst[i] = from_f32<T>(normed * (gate_kind ? sg : zv * sg) * out_scale);
  }
}

}  // namespace mlr

using namespace mlr;

extern "C" {

int mlr_add_normed(float* x, const void* y, int y_is_f32, int slices, const void* weight, int weight_is_f32, float eps,
                   const void* next_weight, int next_is_f32, float next_eps, int mode, void* out, int dtype, int rows,
                   int hidden, hipStream_t stream) {
  MLR_REQUIRE(x && y && weight, "null pointer");
  MLR_REQUIRE(rows > 0 && hidden > 0 && hidden <= 16384, "rows must be > 0 and hidden within 1..16384");
  MLR_REQUIRE(slices >= 0 && (slices == 0 || y_is_f32), "partial sums are float32");
  MLR_REQUIRE(mode >= 0 && mode <= 2 && (mode == 0 || out) && (mode != 1 || next_weight), "bad mode or missing output");
  MLR_REQUIRE(dtype == kF32 || dtype == kBF16, "dtype must be 0 (float32) or 1 (bfloat16)");
  MLR_REQUIRE(dtype == kBF16 || y_is_f32, "a float32 engine has float32 activations");
  if (dtype == kF32)
    launch_add_normed<float>(x, y, y_is_f32, slices, weight, weight_is_f32, eps, next_weight, next_is_f32, next_eps, mode,
                             out, rows, hidden, stream);
  else
    launch_add_normed<bf16>(x, y, y_is_f32, slices, weight, weight_is_f32, eps, next_weight, next_is_f32, next_eps, mode,
                            out, rows, hidden, stream);
  MLR_LAUNCH_CHECK();
  return 0;
}

int mlr_glu_clamped(const void* sums, int sums_is_f32, void* out, int dtype, int rows, int inter, float limit,
                    float alpha, hipStream_t stream) {
  MLR_REQUIRE(sums && out, "null pointer");
  MLR_REQUIRE(rows > 0 && inter > 0 && limit > 0.f, "sizes and limit must be > 0");
  MLR_REQUIRE(dtype == kF32 || dtype == kBF16, "dtype must be 0 (float32) or 1 (bfloat16)");
  MLR_REQUIRE(dtype == kBF16 || sums_is_f32, "a float32 engine has float32 sums");
  const int64_t total = static_cast<int64_t>(rows) * inter;
  const int64_t blocks = (total + 255) / 256;
  MLR_REQUIRE(blocks < (1ll << 31), "too many elements");
  const unsigned grid = static_cast<unsigned>(blocks);
  if (dtype == kF32)
    glu_clamped_kernel<float, float><<<grid, 256, 0, stream>>>(static_cast<const float*>(sums), static_cast<float*>(out),
                                                               rows, inter, limit, alpha);
  else if (sums_is_f32)
    glu_clamped_kernel<float, bf16><<<grid, 256, 0, stream>>>(static_cast<const float*>(sums), static_cast<bf16*>(out),
                                                              rows, inter, limit, alpha);
  else
    glu_clamped_kernel<bf16, bf16><<<grid, 256, 0, stream>>>(static_cast<const bf16*>(sums), static_cast<bf16*>(out),
                                                             rows, inter, limit, alpha);
  MLR_LAUNCH_CHECK();
  return 0;
}

int mlr_latent_prepare(const float* projected, int width, void* q_plain, void* q_latent, float* gate, const float* cos,
                       const float* sin, int rotary_dims, const void* norm_weight, int weight_is_f32, float eps,
                       const int* slots, void* key_pages, void* value_pages, int dtype, int tokens, int heads, int dim,
                       int rot, int rank, int kernel_dim, int block_size, int num_pages, int own_cache, int gated,
                       const float* queries, int q_width, hipStream_t stream) {
  MLR_REQUIRE(projected && q_plain && q_latent, "null pointer");
  MLR_REQUIRE(queries == nullptr || q_width >= heads * (dim + rot), "the query rows are too narrow");
  MLR_REQUIRE(tokens > 0 && heads > 0 && dim > 0 && rot > 0 && rank > 0, "sizes must be > 0");
  MLR_REQUIRE(kernel_dim >= rank + rot, "the kernels' head size must hold latent and rotated part");
  MLR_REQUIRE(rotary_dims >= 0 && rotary_dims % 2 == 0 && rotary_dims <= rot, "rotary_dims must be even and within rot");
  MLR_REQUIRE(rotary_dims == 0 || (cos && sin), "a rotation needs cos and sin tables");
  MLR_REQUIRE(width >= (queries ? 0 : heads * (dim + rot)) + (own_cache ? rank + rot : 0) + (gated ? heads : 0),
              "the projected rows are too narrow");
  MLR_REQUIRE(!own_cache || (norm_weight && slots && key_pages && value_pages && block_size > 0 && num_pages > 0),
              "a cache write needs the latent's norm weight, slots, pages and their sizes");
  MLR_REQUIRE(!gated || gate, "a gated mixer needs room for its gates");
  MLR_REQUIRE(dtype == kF32 || dtype == kBF16, "dtype must be 0 (float32) or 1 (bfloat16)");
  if (dtype == kF32)
    latent_prepare_kernel<float><<<tokens, 256, 0, stream>>>(
        projected, width, static_cast<float*>(q_plain), static_cast<float*>(q_latent), gate, cos, sin, rotary_dims,
        norm_weight, weight_is_f32, eps, slots, static_cast<float*>(key_pages), static_cast<float*>(value_pages), heads,
        dim, rot, rank, kernel_dim, block_size, num_pages, own_cache, gated, queries, q_width);
  else
    latent_prepare_kernel<bf16><<<tokens, 256, 0, stream>>>(
        projected, width, static_cast<bf16*>(q_plain), static_cast<bf16*>(q_latent), gate, cos, sin, rotary_dims,
        norm_weight, weight_is_f32, eps, slots, static_cast<bf16*>(key_pages), static_cast<bf16*>(value_pages), heads,
        dim, rot, rank, kernel_dim, block_size, num_pages, own_cache, gated, queries, q_width);
  MLR_LAUNCH_CHECK();
  return 0;
}

int mlr_heads_linear(const void* x, int64_t in_row, int in_stride, const void* w, void* out, int64_t out_row,
                     int out_stride, const float* row_scale, int dtype, int tokens, int heads, int n, int k,
                     hipStream_t stream) {
  MLR_REQUIRE(x && w && out, "null pointer");
  MLR_REQUIRE(tokens > 0 && heads > 0 && n > 0 && k > 0, "sizes must be > 0");
  MLR_REQUIRE(in_stride >= k && in_row >= static_cast<int64_t>(heads) * in_stride, "the input rows do not hold every head's k values");
  MLR_REQUIRE(out_stride >= n && out_row >= static_cast<int64_t>(heads) * out_stride, "the output rows do not hold every head's n values");
  MLR_REQUIRE(dtype == kF32 || dtype == kBF16, "dtype must be 0 (float32) or 1 (bfloat16)");
  MLR_REQUIRE(heads < 65536 && (tokens + 15) / 16 < 65536, "too many rows or heads for one launch");
  if (dtype == kBF16 && k % 8 == 0 && in_stride % 8 == 0 && in_row % 8 == 0 &&
      reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0) {
    // few tokens: a wavefront per 16 outputs, so that many compute units share the weights' bytes
    if (tokens <= 64)
      heads_linear_mfma_kernel<1><<<dim3((n + 15) / 16, (tokens + 15) / 16, heads), 64, 0, stream>>>(
          static_cast<const bf16*>(x), in_row, in_stride, static_cast<const bf16*>(w), static_cast<bf16*>(out), out_row,
          out_stride, row_scale, heads, tokens, n, k);
    else
      heads_linear_mfma_kernel<4><<<dim3((n + 63) / 64, (tokens + 15) / 16, heads), 64, 0, stream>>>(
          static_cast<const bf16*>(x), in_row, in_stride, static_cast<const bf16*>(w), static_cast<bf16*>(out), out_row,
          out_stride, row_scale, heads, tokens, n, k);
    MLR_LAUNCH_CHECK();
    return 0;
  }
  dim3 grid((n + 63) / 64, (tokens + 63) / 64, heads);
  MLR_REQUIRE(grid.y < 65536u && grid.z < 65536u, "too many rows or heads for one launch");
  if (dtype == kF32)
    heads_linear_kernel<float><<<grid, 256, 0, stream>>>(static_cast<const float*>(x), in_row, in_stride,
                                                         static_cast<const float*>(w), static_cast<float*>(out), out_row,
                                                         out_stride, row_scale, heads, tokens, n, k);
  else
    heads_linear_kernel<bf16><<<grid, 256, 0, stream>>>(static_cast<const bf16*>(x), in_row, in_stride,
                                                        static_cast<const bf16*>(w), static_cast<bf16*>(out), out_row,
                                                        out_stride, row_scale, heads, tokens, n, k);
  MLR_LAUNCH_CHECK();
  return 0;
}

// Floats of scratch memory that mlr_retention_scan needs for its chunked way (0: it will not go that way).
int64_t mlr_retention_scratch(int total_tokens, int entries, int heads, int dim, int vdim) {
  if (dim > 128 || total_tokens <= 0) return 0;
  const int dp = dim <= 16 ? 16 : (dim <= 32 ? 32 : (dim <= 64 ? 64 : 128));
  return static_cast<int64_t>(total_tokens / kChunk + entries) * heads * dp * ((vdim + 15) / 16 * 16);
}

int mlr_retention_scan(float* projected, int width, float* state, int state_rows, const int* read_rows,
                       const int* write_rows, const int* cu_q, const int* q_starts, const float* decay,
                       const float* cos, const float* sin, int rotary_dims, float key_scale, float* out, int entries,
                       int heads, int dim, int vdim, int chunked, int total_tokens, float* scratch, int64_t scratch_floats,
                       hipStream_t stream) {
  MLR_REQUIRE(projected && state && read_rows && write_rows && cu_q && q_starts && decay && out, "null pointer");
  MLR_REQUIRE(entries > 0 && heads > 0 && dim > 0 && vdim > 0 && state_rows > 0, "sizes must be > 0");
  MLR_REQUIRE(dim <= 256, "a head's state has up to 256 rows");
  MLR_REQUIRE(width >= 2 * heads * dim + heads * vdim, "the projected rows are too narrow");
  MLR_REQUIRE(rotary_dims >= 0 && rotary_dims % 2 == 0 && rotary_dims <= dim, "rotary_dims must be even and within dim");
  MLR_REQUIRE(rotary_dims == 0 || (cos && sin), "a rotation needs cos and sin tables");
  dim3 grid(entries, heads, (vdim + 15) / 16);
  MLR_REQUIRE(grid.y < 65536u && grid.z < 65536u, "too many heads or columns for one launch");
  if (chunked && dim <= 128) {  // wider heads keep the state of the token-by-token kernel
    const int dp = dim <= 16 ? 16 : (dim <= 32 ? 32 : (dim <= 64 ? 64 : 128));
    const int vpad = static_cast<int>(grid.z) * 16;
    const int max_chunks = total_tokens / kChunk + entries;  // sum over the entries of ceil(tokens / 64) is at most this
    MLR_REQUIRE(total_tokens > 0 && scratch != nullptr, "the chunked kernels need the number of tokens and scratch memory");
    MLR_REQUIRE(scratch_floats >= static_cast<int64_t>(max_chunks) * heads * dp * vpad, "the scratch memory is too small");
    const size_t lds = (2 * kChunk * (dp + 4) + kChunk * 16 + 4 * 16 * kScoreLd + kChunk + 1) * sizeof(float);
    static bool configured = false;
    if (!configured) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(retention_local_kernel<128>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);
      if (e != hipSuccess) {
        set_error(std::string("mlr_retention_scan: cannot raise the LDS limit: ") + hipGetErrorString(e));
        return -1;
      }
      configured = true;
    }
    retention_rotate_kernel<<<total_tokens, 256, 0, stream>>>(projected, width, cos, sin, rotary_dims, key_scale, heads, dim);
    MLR_LAUNCH_CHECK();
    const dim3 all(max_chunks, heads);
#define MLR_CHUNK(DP)                                                                                              \
  do {                                                                                                             \
    retention_local_kernel<DP><<<all, 256, lds, stream>>>(projected, width, cu_q, decay, out, scratch, entries, heads, dim, \
                                                          vdim, vpad);                                             \
    retention_state_kernel<<<dim3(entries, heads, (DP * vpad + 255) / 256), 256, 0, stream>>>(                    \
        state, read_rows, write_rows, cu_q, q_starts, decay, scratch, heads, dim, vdim, DP, vpad);                 \
    retention_apply_kernel<DP><<<all, 256, 0, stream>>>(projected, width, cu_q, q_starts, decay, out, scratch, entries, \
                                                        heads, dim, vdim, vpad);                                   \
  } while (0)
    if (dp == 16)
      MLR_CHUNK(16);
    else if (dp == 32)
      MLR_CHUNK(32);
    else if (dp == 64)
      MLR_CHUNK(64);
    else
      MLR_CHUNK(128);
#undef MLR_CHUNK
    MLR_LAUNCH_CHECK();
    return 0;
  }
#define MLR_SCAN(dpl)                                                                                              \
  retention_scan_kernel<dpl><<<grid, 64, 0, stream>>>(projected, width, state, read_rows, write_rows, cu_q, q_starts, \
                                                      decay, cos, sin, rotary_dims, key_scale, out, heads, dim, vdim)
  if (dim <= 16)
    MLR_SCAN(4);
  else if (dim <= 32)
    MLR_SCAN(8);
  else if (dim <= 64)
    MLR_SCAN(16);
  else if (dim <= 128)
    MLR_SCAN(32);
  else
    MLR_SCAN(64);
#undef MLR_SCAN
  MLR_LAUNCH_CHECK();
  return 0;
}

int mlr_retention_gate(const float* retained, const float* projected, int width, int gate_offset, void* out, int dtype,
                       int tokens, int heads, int vdim, float eps, const void* norm_weight, int weight_is_f32,
                       float out_scale, int64_t out_row, int weight_per_head, int gate_kind, hipStream_t stream) {
  MLR_REQUIRE(retained && projected && out, "null pointer");
  MLR_REQUIRE(gate_kind == 0 || gate_kind == 1, "the gate is silu (0) or the sigmoid (1)");
  MLR_REQUIRE(tokens > 0 && heads > 0 && heads < 65536 && vdim > 0, "sizes must be > 0");
  MLR_REQUIRE(gate_offset >= 0 && width >= gate_offset + heads * vdim, "the projected rows do not hold the gate");
  MLR_REQUIRE(out_row >= static_cast<int64_t>(heads) * vdim, "a row of the output is shorter than the heads");
  MLR_REQUIRE(dtype == kF32 || dtype == kBF16, "dtype must be 0 (float32) or 1 (bfloat16)");
  dim3 grid(tokens, heads);
  if (dtype == kF32)
    retention_gate_kernel<float><<<grid, 64, 0, stream>>>(retained, projected, width, gate_offset,
                                                          static_cast<float*>(out), out_row, heads, vdim, eps,
                                                          norm_weight, weight_is_f32, out_scale, weight_per_head, gate_kind);
  else
    retention_gate_kernel<bf16><<<grid, 64, 0, stream>>>(retained, projected, width, gate_offset,
                                                         static_cast<bf16*>(out), out_row, heads, vdim, eps,
                                                         norm_weight, weight_is_f32, out_scale, weight_per_head,
                                                         gate_kind);
  MLR_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
