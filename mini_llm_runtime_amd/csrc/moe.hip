// Routed experts: which experts a token uses and with what weight, the (token, choice) pairs
// sorted by expert into row tiles, and the two grouped products over those tiles.  Nothing here
// comes back to the host between the router's logits and the weighted expert outputs, so a step
// with routed experts can be recorded and replayed like any other.
//
// A pair is p = token * top + choice.  `sorted` lists the pairs expert by expert, `offsets[e]` is
// where expert e's run starts, and a tile is (expert, first row of `sorted`): up to `tile_rows`
// pairs of one expert, which share that expert's weights in a product.  The order of the pairs
// inside an expert's run is whatever the atomics made it; every output row is computed from its own
// input row alone, with the sums over k in a fixed order, so no value depends on that order or on
// what else is in the batch.
#include "api.h"
#include "common.h"
#include "mfma.h"

namespace mlr {

// ---- routing ---------------------------------------------------------------------------------

__device__ __forceinline__ void wave_argmax(float& v, int& i) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(v, off, kWave);
    const int oi = __shfl_xor(i, off, kWave);
    if (ov > v || (ov == v && oi < i)) {
      v = ov;
      i = oi;
    }
  }
}

// One wavefront per token.  s = sigmoid(z) (score_kind 0) or softmax(z) over all experts (1), c = s + correction;
// with `normalise` the chosen weights are divided by their sum (+ 1e-20) before the scale.  Block g of experts / groups
// consecutive experts scores top-2 sum of its c; c := -inf outside the `keep` highest blocks; then
// `top` rounds of arg-max over c (ties to the lower index), each winner e leaving ids = e and
// weights = s[e] * scale.
__global__ __launch_bounds__(kWave) void moe_route_kernel(const float* __restrict__ logits,
                                                          const float* __restrict__ correction,
                                                          int* __restrict__ ids, float* __restrict__ weights,
                                                          int experts, int top, int groups, int keep, float scale,
                                                          int score_kind, int normalise) {
  extern __shared__ float route_lds[];
  float* c = route_lds;            // [experts]
  float* s = route_lds + experts;  // [experts]
  float* gs = s + experts;         // [groups]
  const int t = blockIdx.x;
  const int lane = threadIdx.x;
  const int per = experts / groups;
  const float* z = logits + static_cast<int64_t>(t) * experts;
  float z_max = 0.f, z_inv = 1.f;
  if (score_kind == 1) {
    float mx = -INFINITY;
    for (int e = lane; e < experts; e += kWave) mx = fmaxf(mx, z[e]);
    z_max = wave_max(mx);
    float sum = 0.f;
    for (int e = lane; e < experts; e += kWave) sum += expf(z[e] - z_max);
    z_inv = 1.0f / wave_sum(sum);
  }
  for (int e = lane; e < experts; e += kWave) {
    const float sv = score_kind == 1 ? expf(z[e] - z_max) * z_inv : 1.0f / (1.0f + expf(-z[e]));
    s[e] = sv;
    c[e] = sv + (correction != nullptr ? correction[e] : 0.f);
  }
  __syncthreads();
  if (groups > 1 && keep < groups) {
    for (int g = lane; g < groups; g += kWave) {
      float a = -INFINITY, b = -INFINITY;  // running top-2 of the block
      for (int e = g * per; e < (g + 1) * per; ++e) {
        const float v = c[e];
        if (v > a) {
          b = a;
          a = v;
        } else if (v > b) {
          b = v;
        }
      }
      gs[g] = per > 1 ? a + b : a;
    }
    __syncthreads();
    // the kept groups get +inf as their mark, one after the other
    for (int k = 0; k < keep; ++k) {
      float v = -INFINITY;
      int i = 0x7fffffff;
      for (int g = lane; g < groups; g += kWave) {
        const float x = gs[g];
        if (x != INFINITY && (x > v || (x == v && g < i))) {
          v = x;
          i = g;
        }
      }
      wave_argmax(v, i);
      if (lane == 0 && i < groups) gs[i] = INFINITY;
      __syncthreads();
    }
    for (int e = lane; e < experts; e += kWave)
      if (gs[e / per] != INFINITY) c[e] = -INFINITY;
    __syncthreads();
  }
  float chosen_sum = 0.f;
  for (int k = 0; k < top; ++k) {
    float v = -INFINITY;
    int i = 0x7fffffff;
    for (int e = lane; e < experts; e += kWave) {
      const float x = c[e];
      if (x > v || (x == v && e < i)) {
        v = x;
        i = e;
      }
    }
    wave_argmax(v, i);
    if (i >= experts) i = 0;  // only if every score left is NaN or -inf: keep the id in range
    chosen_sum += s[i];
    if (lane == 0) {
      ids[static_cast<int64_t>(t) * top + k] = i;
      weights[static_cast<int64_t>(t) * top + k] = s[i] * scale;
      c[i] = -INFINITY;
    }
    __syncthreads();
  }
  if (normalise) {
    const float inv = 1.0f / (chosen_sum + 1e-20f);
    for (int k = lane; k < top; k += kWave) weights[static_cast<int64_t>(t) * top + k] *= inv;
  }
}

// Experts that hand their input on: where ids[t, j] >= first (such an expert has no matrices and the grouped
// products skip its pairs) out[j, t, :] = weights[t, j] * h[t, :].  One workgroup per pair.
template <typename T>
__global__ __launch_bounds__(256) void moe_identity_kernel(const T* __restrict__ h, const int* __restrict__ ids,
                                                           const float* __restrict__ weights, float* __restrict__ out,
                                                           int tokens, int top, int hidden, int first) {
  const int pair = blockIdx.x;
  if (ids[pair] < first) return;
  const int t = pair / top;
  const int j = pair - t * top;
  const float w = weights[pair];
  const T* src = h + static_cast<int64_t>(t) * hidden;
  float* dst = out + (static_cast<int64_t>(j) * tokens + t) * hidden;
  for (int i = threadIdx.x; i < hidden; i += 256) dst[i] = w * to_f32(src[i]);
}

// ---- pairs sorted by expert ------------------------------------------------------------------

// One workgroup.  counts -> offsets and tiles (thread 0) -> placement.
__global__ __launch_bounds__(1024) void moe_align_kernel(const int* __restrict__ ids, int pairs, int experts,
                                                         int tile_rows, int max_tiles, int* __restrict__ sorted,
                                                         int* __restrict__ offsets, int* __restrict__ tiles) {
  extern __shared__ int align_lds[];
  int* counts = align_lds;            // [experts]
  int* start = align_lds + experts;   // [experts]
  __shared__ int used_tiles;
  const int tid = threadIdx.x;
  for (int e = tid; e < experts; e += blockDim.x) counts[e] = 0;
  __syncthreads();
  for (int p = tid; p < pairs; p += blockDim.x) {
    const int e = ids[p];
    if (e >= 0 && e < experts) atomicAdd(&counts[e], 1);
  }
  __syncthreads();
  if (tid == 0) {
    int at = 0, nt = 0;
    for (int e = 0; e < experts; ++e) {
      const int n = counts[e];
      offsets[e] = at;
      start[e] = at;
      for (int r = 0; r < n && nt < max_tiles; r += tile_rows) {
        tiles[2 * nt] = e;
        tiles[2 * nt + 1] = at + r;
        ++nt;
      }
      at += n;
    }
    offsets[experts] = at;
    used_tiles = nt;
  }
  __syncthreads();
  for (int i = used_tiles + tid; i < max_tiles; i += blockDim.x) {
    tiles[2 * i] = -1;  // a workgroup that finds this has nothing to do
    tiles[2 * i + 1] = 0;
  }
  for (int e = tid; e < experts; e += blockDim.x) counts[e] = 0;
  __syncthreads();
  for (int p = tid; p < pairs; p += blockDim.x) {
    const int e = ids[p];
    if (e >= 0 && e < experts) sorted[start[e] + atomicAdd(&counts[e], 1)] = p;
  }
}

// ---- grouped products, plain 32-bit FMA arithmetic -----------------------------------------------
//
// UP:   act[row, n]  = f(sum_k h[token(row), k] * w[e, n, k])                  (rows in sorted order)
// DOWN: out[choice(row), token(row), n] = weight[pair(row)] * sum_k act[row, k] * w[e, n, k]
// A workgroup owns 16 rows of one tile and 64 features; K in slices of 16 through LDS.

constexpr int kMoeRows = 16;
constexpr int kMoeCols = 64;
constexpr int kMoeK = 16;

template <typename T, bool UP>
__global__ __launch_bounds__(256) void moe_gemm_simple_kernel(const T* __restrict__ a, const T* __restrict__ w,
                                                              const int* __restrict__ sorted,
                                                              const int* __restrict__ offsets,
                                                              const int* __restrict__ tiles,
                                                              const float* __restrict__ pair_weights,
                                                              void* __restrict__ out, int tokens, int top, int N,
                                                              int K, int act) {
  const int expert = tiles[2 * blockIdx.x];
  if (expert < 0) return;
  const int row0 = tiles[2 * blockIdx.x + 1];
  const int row_end = offsets[expert + 1];
  __shared__ float xs[kMoeK][kMoeRows + 1];
  __shared__ float ws[kMoeK][kMoeCols + 4];
  __shared__ int pair_of[kMoeRows];
  const int tid = threadIdx.x;
  if (tid < kMoeRows) pair_of[tid] = row0 + tid < row_end ? sorted[row0 + tid] : -1;
  __syncthreads();
  const int tm = tid / 16;  // row of the tile
  const int tn = tid % 16;  // features tn * 4 .. tn * 4 + 3
  const int n0 = blockIdx.y * kMoeCols;
  const T* wbase = w + static_cast<int64_t>(expert) * N * K;
  // the row of `a` this thread stages (one element per slice)
  const int lrow = tid / kMoeK;
  const int lk = tid % kMoeK;
  const int lpair = pair_of[lrow];
  const T* arow = nullptr;
  if (lpair >= 0) arow = UP ? a + static_cast<int64_t>(lpair / top) * K : a + static_cast<int64_t>(row0 + lrow) * K;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += kMoeK) {
    xs[lk][lrow] = (arow != nullptr && k0 + lk < K) ? to_f32(arow[k0 + lk]) : 0.f;
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int idx = tid + it * 256;
      const int col = idx / kMoeK;
      const int kk = idx % kMoeK;
      const int gn = n0 + col;
      ws[kk][col] = (gn < N && k0 + kk < K) ? to_f32(wbase[static_cast<int64_t>(gn) * K + k0 + kk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kMoeK; ++kk) {
      const float x = xs[kk][tm];
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] = fmaf(x, ws[kk][tn * 4 + j], acc[j]);
    }
    __syncthreads();
  }
  const int pair = pair_of[tm];
  if (pair < 0) return;
  const int token = pair / top;
  const int choice = pair - token * top;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int gn = n0 + tn * 4 + j;
    if (gn >= N) continue;
    float v = acc[j];
    if (UP) {
      if (act == 2) {
        v = fmaxf(v, 0.f);
        v *= v;
      } else if (act == 3) {
        v = 1.0f / (1.0f + expf(-v));
      }
      static_cast<T*>(out)[static_cast<int64_t>(row0 + tm) * N + gn] = from_f32<T>(v);
    } else {
      static_cast<float*>(out)[(static_cast<int64_t>(choice) * tokens + token) * N + gn] = pair_weights[pair] * v;
    }
  }
}

// ---- grouped products in bfloat16 on the matrix cores ---------------------------------------------
//
// The same two products, two kernels.
//
// Streaming (tiles of 16 rows; decoding, where an expert sees a few rows): a workgroup of four
// wavefronts owns 16 rows of a tile (the columns of the 16 x 16 x 32 block; weights are the row
// operand, as in the other product kernels) and 64 features, 16 per wavefront.  A lane reads 8
// consecutive k of one weight row and of one input row per block, both straight from memory through
// range-checked buffer loads (rows past the tile's end, features past N and k past K read zeros, no
// branch around a load), eight blocks in flight before the first product: the kernel's time is the
// expert weights it streams, read once (non-temporal).
constexpr int kMoeDepth = 8;

template <bool UP>
__global__ __launch_bounds__(256) void moe_gemm_mfma_kernel(const bf16* __restrict__ a, const bf16* __restrict__ w,
                                                            const int* __restrict__ sorted,
                                                            const int* __restrict__ offsets,
                                                            const int* __restrict__ tiles,
                                                            const float* __restrict__ pair_weights,
                                                            void* __restrict__ out, int tokens, int top, int N, int K,
                                                            int act, int a_rows) {
  const int expert = tiles[2 * blockIdx.x];
  if (expert < 0) return;
  const int row0 = tiles[2 * blockIdx.x + 1];
  const int row_end = offsets[expert + 1];
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int col = lane % 16;   // operand row: weight row / input row of the tile
  const int quad = lane / 16;  // which 8 of a block's 32 k
  const int n_base = (blockIdx.y * (blockDim.x / kWave) + wave) * 16;  // 16 features a wavefront
  if (n_base >= N) return;
  // the input row this lane loads (as the column operand), and the rows whose sums it ends up with
  const int in_row = row0 + col;
  const int in_pair = in_row < row_end ? sorted[in_row] : -1;
  const int a_row = in_pair < 0 ? -1 : (UP ? in_pair / top : in_row);
  const unsigned row_bytes = static_cast<unsigned>(K) * 2u;
  const __amdgpu_buffer_rsrc_t wbuf =
      make_buffer(w + static_cast<int64_t>(expert) * N * K, static_cast<unsigned>(N) * row_bytes);
  const __amdgpu_buffer_rsrc_t abuf = make_buffer(a, static_cast<unsigned>(a_rows) * row_bytes);
  const int wn = n_base + col;
  const unsigned w_off = wn < N ? static_cast<unsigned>(wn) * row_bytes : kOutOfBuffer;
  const unsigned a_off = a_row >= 0 ? static_cast<unsigned>(a_row) * row_bytes : kOutOfBuffer;
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
  for (int kb = 0; kb < K; kb += 32 * kMoeDepth) {
    bf16x8_t wv[kMoeDepth], xv[kMoeDepth];
#pragma unroll
    for (int u = 0; u < kMoeDepth; ++u) {
      const int k = kb + u * 32 + quad * 8;
      const unsigned koff = static_cast<unsigned>(k) * 2u;
      const bool in = k < K;
      wv[u] = buffer_load_bf16x8_once(wbuf, in && w_off != kOutOfBuffer ? w_off + koff : kOutOfBuffer);
      xv[u] = buffer_load_bf16x8(abuf, in && a_off != kOutOfBuffer ? a_off + koff : kOutOfBuffer);
    }
#pragma unroll
    for (int u = 0; u < kMoeDepth; ++u) acc = mfma_16x16x32(wv[u], xv[u], acc);
  }
  // acc[i]: feature n_base + quad * 4 + i of tile row `col`
  if (in_pair < 0) return;
  const int token = in_pair / top;
  const int choice = in_pair - token * top;
  const int n = n_base + quad * 4;
  if (UP) {
    bf16* dst = static_cast<bf16*>(out) + static_cast<int64_t>(in_row) * N + n;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float v = acc[i];
      if (act == 2) {
        v = fmaxf(v, 0.f);
        v *= v;
      } else if (act == 3) {
        v = 1.0f / (1.0f + __expf(-v));
      }
      if (n + i < N) dst[i] = f32_to_bf16(v);
    }
  } else {
    const float pw = pair_weights[in_pair];
    float* dst = static_cast<float*>(out) + (static_cast<int64_t>(choice) * tokens + token) * N + n;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (n + i < N) dst[i] = pw * acc[i];
  }
}

// Streaming through LDS (tiles of 16 rows, as above): the same work with loads that cover whole lines.
// A workgroup owns 16 rows of a tile and 64 features; k in slices of 128.  Sixteen neighbouring lanes
// fetch the 256 contiguous bytes that a slice holds of one weight row (the kernel above reads 64 bytes
// of 16 different rows per instruction, which streams a large matrix at little more than half the
// rate), two slices ahead in registers, and stage them through two LDS buffers whose rows of 288 bytes
// are free of bank conflicts for the operand pattern of the 16 x 16 x 32 block.  Wavefront w multiplies
// features w * 16 .. + 16.
constexpr int kStCols = 64;
constexpr int kStK = 128;
constexpr int kStLd = kStK + 16;  // bf16 elements per LDS row: 288 bytes

template <bool UP>
__global__ __launch_bounds__(256) void moe_gemm_stream_kernel(const bf16* __restrict__ a, const bf16* __restrict__ w,
                                                              const int* __restrict__ sorted,
                                                              const int* __restrict__ offsets,
                                                              const int* __restrict__ tiles,
                                                              const float* __restrict__ pair_weights,
                                                              void* __restrict__ out, int tokens, int top, int N, int K,
                                                              int act, int a_rows) {
  const int expert = tiles[2 * blockIdx.x];
  if (expert < 0) return;
  const int row0 = tiles[2 * blockIdx.x + 1];
  const int row_end = offsets[expert + 1];
  __shared__ __attribute__((aligned(16))) bf16 ws[2][kStCols * kStLd];
  __shared__ __attribute__((aligned(16))) bf16 xs[2][kMoeRows * kStLd];
  __shared__ int pair_of[kMoeRows];
  const int tid = threadIdx.x;
  const int lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int n0 = blockIdx.y * kStCols;
  if (tid < kMoeRows) pair_of[tid] = row0 + tid < row_end ? sorted[row0 + tid] : -1;
  __syncthreads();
  const unsigned row_bytes = static_cast<unsigned>(K) * 2u;
  const __amdgpu_buffer_rsrc_t wbuf =
      make_buffer(w + static_cast<int64_t>(expert) * N * K, static_cast<unsigned>(N) * row_bytes);
  const __amdgpu_buffer_rsrc_t abuf = make_buffer(a, static_cast<unsigned>(a_rows) * row_bytes);
  // per slice a thread moves four 16-byte pieces of the weight tile (rows prow, prow + 16, ...) and one
  // of the input tile (row prow), all at k piece `piece` of the slice
  const int piece = tid % 16;
  const int prow = tid / 16;
  unsigned w_off[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = n0 + prow + i * 16;
    w_off[i] = row < N ? static_cast<unsigned>(row) * row_bytes + piece * 16u : kOutOfBuffer;
  }
  const int my_pair = pair_of[prow];
  const int src = my_pair < 0 ? -1 : (UP ? my_pair / top : row0 + prow);
  const unsigned x_off = src >= 0 ? static_cast<unsigned>(src) * row_bytes + piece * 16u : kOutOfBuffer;
  const int lds_at = prow * kStLd + piece * 8;
  bf16x8_t w_a[4], w_b[4], x_a, x_b;  // two slices on their way
  auto fetch = [&](bf16x8_t(&wreg)[4], bf16x8_t& xreg, int k0) {
    const bool k_in = k0 + piece * 8 < K;
    const unsigned koff = static_cast<unsigned>(k0) * 2u;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      wreg[i] = buffer_load_bf16x8_once(wbuf, k_in && w_off[i] != kOutOfBuffer ? w_off[i] + koff : kOutOfBuffer);
    xreg = buffer_load_bf16x8(abuf, k_in && x_off != kOutOfBuffer ? x_off + koff : kOutOfBuffer);
  };
  auto stage = [&](const bf16x8_t(&wreg)[4], const bf16x8_t& xreg, int buf) {
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<bf16x8_t*>(&ws[buf][lds_at + i * 16 * kStLd]) = wreg[i];
    *reinterpret_cast<bf16x8_t*>(&xs[buf][lds_at]) = xreg;
  };
  const int col = lane % 16;
  const int quad = lane / 16;
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
  auto multiply = [&](int buf) {
    const bf16* wt = &ws[buf][(wave * 16 + col) * kStLd + quad * 8];
    const bf16* xt = &xs[buf][col * kStLd + quad * 8];
#pragma unroll
    for (int ks = 0; ks < kStK / 32; ++ks)
      acc = mfma_16x16x32(*reinterpret_cast<const bf16x8_t*>(wt + ks * 32),
                          *reinterpret_cast<const bf16x8_t*>(xt + ks * 32), acc);
  };
  const int slices = (K + kStK - 1) / kStK;
  fetch(w_a, x_a, 0);
  if (slices > 1) fetch(w_b, x_b, kStK);
  stage(w_a, x_a, 0);
  __syncthreads();
  // two slices a turn, so that the register sets and the LDS buffers keep their names; `slices` is the
  // same for every thread, so are the barriers
  for (int s = 0; s < slices; s += 2) {
    if (s + 2 < slices) fetch(w_a, x_a, (s + 2) * kStK);
    multiply(0);
    if (s + 1 < slices) stage(w_b, x_b, 1);
    __syncthreads();
    if (s + 1 >= slices) break;
    if (s + 3 < slices) fetch(w_b, x_b, (s + 3) * kStK);
    multiply(1);
    if (s + 2 < slices) stage(w_a, x_a, 0);
    __syncthreads();
  }
  // acc[i]: feature n0 + wave * 16 + quad * 4 + i of tile row `col`
  const int pair = pair_of[col];
  if (pair < 0) return;
  const int token = pair / top;
  const int choice = pair - token * top;
  const int n = n0 + wave * 16 + quad * 4;
  if (UP) {
    bf16* dst = static_cast<bf16*>(out) + static_cast<int64_t>(row0 + col) * N + n;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float v = acc[i];
      if (act == 2) {
        v = fmaxf(v, 0.f);
        v *= v;
      } else if (act == 3) {
        v = 1.0f / (1.0f + __expf(-v));
      }
      if (n + i < N) dst[i] = f32_to_bf16(v);
    }
  } else {
    const float pw = pair_weights[pair];
    float* dst = static_cast<float*>(out) + (static_cast<int64_t>(choice) * tokens + token) * N + n;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (n + i < N) dst[i] = pw * acc[i];
  }
}

// Tiled (prompts, where an expert sees hundreds of rows): a workgroup owns a tile of 64 x RB rows and
// 128 features; k in slices of 64 through two LDS buffers (rows padded to 144 bytes: free of bank
// conflicts for the operand pattern of the 32 x 32 x 16 block), the next slice on its way into
// registers while this one is multiplied.  Wavefront (wr, wc) of 2 x 2 owns rows wr * 32 RB .. + 32 RB
// and features wc * 64 .. + 64: 2 RB blocks of 32 x 32; with RB = 2 every operand read from LDS serves
// two products.
constexpr int kBigCols = 128;
constexpr int kBigK = 64;
constexpr int kBigLd = kBigK + 8;  // bf16 elements per LDS row
constexpr int big_rows(int rb) { return 64 * rb; }
constexpr int big_lds_bytes(int rb) { return 2 * (kBigCols + big_rows(rb)) * kBigLd * 2 + big_rows(rb) * 4; }

template <bool UP, int RB>
__global__ __launch_bounds__(256) void moe_gemm_tiled_kernel(const bf16* __restrict__ a, const bf16* __restrict__ w,
                                                             const int* __restrict__ sorted,
                                                             const int* __restrict__ offsets,
                                                             const int* __restrict__ tiles,
                                                             const float* __restrict__ pair_weights,
                                                             void* __restrict__ out, int tokens, int top, int N, int K,
                                                             int act, int a_rows) {
  constexpr int kRows = big_rows(RB);
  const int expert = tiles[2 * blockIdx.x];
  if (expert < 0) return;
  const int row0 = tiles[2 * blockIdx.x + 1];
  const int row_end = offsets[expert + 1];
  extern __shared__ __attribute__((aligned(16))) unsigned char moe_lds[];
  bf16* const ws = reinterpret_cast<bf16*>(moe_lds);   // [2][kBigCols][kBigLd]
  bf16* const xs = ws + 2 * kBigCols * kBigLd;         // [2][kRows][kBigLd]
  int* const pair_of = reinterpret_cast<int*>(xs + 2 * kRows * kBigLd);  // [kRows]
  const int tid = threadIdx.x;
  const int lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wr = wave / 2;
  const int wc = wave % 2;
  const int n0 = blockIdx.y * kBigCols;
  if (tid < kRows) pair_of[tid] = row0 + tid < row_end ? sorted[row0 + tid] : -1;
  __syncthreads();
  const unsigned row_bytes = static_cast<unsigned>(K) * 2u;
  const __amdgpu_buffer_rsrc_t wbuf =
      make_buffer(w + static_cast<int64_t>(expert) * N * K, static_cast<unsigned>(N) * row_bytes);
  const __amdgpu_buffer_rsrc_t abuf = make_buffer(a, static_cast<unsigned>(a_rows) * row_bytes);
  // what this thread moves per slice: 16-byte pieces of the weight tile and of the input tile
  // (piece c: row c / 8, k piece c % 8), the same rows for every slice
  constexpr int kWPieces = kBigCols * 8 / 256;
  constexpr int kXPieces = kRows * 8 / 256;
  unsigned w_off[kWPieces], x_off[kXPieces];
  const int piece = tid % 8;  // the same for all of a thread's pieces: 256 is a multiple of 8
#pragma unroll
  for (int i = 0; i < kWPieces; ++i) {
    const int row = (tid + i * 256) / 8;
    w_off[i] = n0 + row < N ? static_cast<unsigned>(n0 + row) * row_bytes + piece * 16u : kOutOfBuffer;
  }
#pragma unroll
  for (int i = 0; i < kXPieces; ++i) {
    const int row = (tid + i * 256) / 8;
    const int pair = pair_of[row];
    const int src = pair < 0 ? -1 : (UP ? pair / top : row0 + row);
    x_off[i] = src >= 0 ? static_cast<unsigned>(src) * row_bytes + piece * 16u : kOutOfBuffer;
  }
  const int lds_at = (tid / 8) * kBigLd + piece * 8;  // piece i of either tile: + i * 32 rows
  bf16x8_t wreg[kWPieces], xreg[kXPieces];
  auto fetch = [&](int k0) {
    const bool k_in = k0 + piece * 8 < K;
    const unsigned koff = static_cast<unsigned>(k0) * 2u;
#pragma unroll
    for (int i = 0; i < kWPieces; ++i)
      wreg[i] = buffer_load_bf16x8(wbuf, k_in && w_off[i] != kOutOfBuffer ? w_off[i] + koff : kOutOfBuffer);
#pragma unroll
    for (int i = 0; i < kXPieces; ++i)
      xreg[i] = buffer_load_bf16x8(abuf, k_in && x_off[i] != kOutOfBuffer ? x_off[i] + koff : kOutOfBuffer);
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int i = 0; i < kWPieces; ++i)
      *reinterpret_cast<bf16x8_t*>(ws + buf * kBigCols * kBigLd + lds_at + i * 32 * kBigLd) = wreg[i];
#pragma unroll
    for (int i = 0; i < kXPieces; ++i)
      *reinterpret_cast<bf16x8_t*>(xs + buf * kRows * kBigLd + lds_at + i * 32 * kBigLd) = xreg[i];
  };
  f32x16_t acc[RB][2];
#pragma unroll
  for (int r = 0; r < RB; ++r)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[r][b][i] = 0.f;
  const int r32 = lane % 32;
  const int khalf = lane / 32;  // which 8 of a block's 16 k
  fetch(0);
  stage(0);
  __syncthreads();
  int buf = 0;
  for (int k0 = 0; k0 < K; k0 += kBigK) {
    const bool more = k0 + kBigK < K;
    if (more) fetch(k0 + kBigK);
    const bf16* wt = ws + buf * kBigCols * kBigLd + (wc * 64 + r32) * kBigLd + khalf * 8;
    const bf16* xt = xs + buf * kRows * kBigLd + (wr * 32 * RB + r32) * kBigLd + khalf * 8;
#pragma unroll
    for (int ks = 0; ks < kBigK / 16; ++ks) {
      const bf16x8_t w0 = *reinterpret_cast<const bf16x8_t*>(wt + ks * 16);
      const bf16x8_t w1 = *reinterpret_cast<const bf16x8_t*>(wt + 32 * kBigLd + ks * 16);
#pragma unroll
      for (int r = 0; r < RB; ++r) {
        const bf16x8_t xb = *reinterpret_cast<const bf16x8_t*>(xt + r * 32 * kBigLd + ks * 16);
        acc[r][0] = mfma_32x32x16(w0, xb, acc[r][0]);
        acc[r][1] = mfma_32x32x16(w1, xb, acc[r][1]);
      }
    }
    if (more) stage(buf ^ 1);
    __syncthreads();
    buf ^= 1;
  }
  // acc[r][b][i]: feature n0 + wc * 64 + b * 32 + (i / 4) * 8 + khalf * 4 + i % 4 of tile row
  // wr * 32 RB + r * 32 + r32
#pragma unroll
  for (int r = 0; r < RB; ++r) {
    const int row = wr * 32 * RB + r * 32 + r32;
    const int pair = pair_of[row];
    if (pair < 0) continue;
    const int token = pair / top;
    const int choice = pair - token * top;
    const float pw = UP ? 1.f : pair_weights[pair];
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n = n0 + wc * 64 + b * 32 + g * 8 + khalf * 4;
        if (n >= N) continue;  // N is a multiple of 8 here: four features are all inside or all outside
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = acc[r][b][g * 4 + i];
        if (UP) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            if (act == 2) {
              v[i] = fmaxf(v[i], 0.f);
              v[i] *= v[i];
            } else if (act == 3) {
              v[i] = 1.0f / (1.0f + __expf(-v[i]));
            }
          }
          const u16x4_t packed = {f32_to_bf16(v[0]).bits, f32_to_bf16(v[1]).bits, f32_to_bf16(v[2]).bits,
                                  f32_to_bf16(v[3]).bits};
          *reinterpret_cast<u16x4_t*>(static_cast<bf16*>(out) + static_cast<int64_t>(row0 + row) * N + n) = packed;
        } else {
          float* dst = static_cast<float*>(out) + (static_cast<int64_t>(choice) * tokens + token) * N + n;
          *reinterpret_cast<f32x4_t*>(dst) = f32x4_t{pw * v[0], pw * v[1], pw * v[2], pw * v[3]};
        }
      }
  }
}

template <bool UP, int RB>
static int launch_moe_tiled(const bf16* a, const bf16* w, const int* sorted, const int* offsets, const int* tiles,
                            const float* pair_weights, void* out, int max_tiles, int tokens, int top, int n, int k,
                            int act, int a_rows, hipStream_t stream) {
  static bool configured = false;
  if (!configured) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(moe_gemm_tiled_kernel<UP, RB>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, big_lds_bytes(RB));
    if (e != hipSuccess) {
      set_error(std::string("mlr_moe_gemm: cannot raise the LDS limit: ") + hipGetErrorString(e));
      return -1;
    }
    configured = true;
  }
  const dim3 grid(max_tiles, (n + kBigCols - 1) / kBigCols);
  moe_gemm_tiled_kernel<UP, RB><<<grid, 256, big_lds_bytes(RB), stream>>>(a, w, sorted, offsets, tiles, pair_weights, out,
                                                                        tokens, top, n, k, act, a_rows);
  return 0;
}

}  // namespace mlr

using namespace mlr;

extern "C" {

int mlr_moe_route(const float* logits, const float* correction, int* ids, float* weights, int tokens, int experts,
                  int top, int groups, int keep, float scale, int score_kind, int normalise, hipStream_t stream) {
  MLR_REQUIRE(logits && ids && weights, "null pointer");
  MLR_REQUIRE(score_kind == 0 || score_kind == 1, "scores are sigmoids (0) or a softmax (1)");
  MLR_REQUIRE(tokens > 0 && experts > 0 && top > 0 && top <= experts, "sizes must be > 0 and top <= experts");
  MLR_REQUIRE(groups > 0 && experts % groups == 0 && keep > 0 && keep <= groups, "bad groups");
  MLR_REQUIRE(top <= keep * (experts / groups), "the kept groups hold fewer experts than a token uses");
  MLR_REQUIRE(experts <= 4096, "at most 4096 experts");
  const size_t lds = (2 * static_cast<size_t>(experts) + groups) * sizeof(float);
  moe_route_kernel<<<tokens, kWave, lds, stream>>>(logits, correction, ids, weights, experts, top, groups, keep, scale,
                                                   score_kind, normalise);
  MLR_LAUNCH_CHECK();
  return 0;
}

int mlr_moe_identity(const void* h, const int* ids, const float* weights, float* out, int dtype, int tokens, int top,
                     int hidden, int first, hipStream_t stream) {
  MLR_REQUIRE(h && ids && weights && out, "null pointer");
  MLR_REQUIRE(tokens > 0 && top > 0 && hidden > 0 && first >= 0, "sizes must be > 0");
  MLR_REQUIRE(dtype == kF32 || dtype == kBF16, "dtype must be 0 (float32) or 1 (bfloat16)");
  if (dtype == kF32)
    moe_identity_kernel<float><<<tokens * top, 256, 0, stream>>>(static_cast<const float*>(h), ids, weights, out, tokens,
                                                                 top, hidden, first);
  else
    moe_identity_kernel<bf16><<<tokens * top, 256, 0, stream>>>(static_cast<const bf16*>(h), ids, weights, out, tokens,
                                                                top, hidden, first);
  MLR_LAUNCH_CHECK();
  return 0;
}

// Rows of one tile of the grouped products: `big` 0 the kernels for few rows an expert (16), 1 and 2
// the tiled matrix-core kernel for many (64 and 128).
int mlr_moe_tile_rows(int big) { return big ? big_rows(big) : kMoeRows; }

// The most tiles `pairs` pairs over `experts` experts can make.
int mlr_moe_max_tiles(int pairs, int experts, int big) {
  const int most = pairs / mlr_moe_tile_rows(big) + experts;  // full tiles, and at most one that is not per expert
  return most < pairs ? most : pairs;
}

int mlr_moe_align(const int* ids, int pairs, int experts, int big, int max_tiles, int* sorted, int* offsets, int* tiles,
                  hipStream_t stream) {
  MLR_REQUIRE(ids && sorted && offsets && tiles, "null pointer");
  MLR_REQUIRE(pairs > 0 && experts > 0 && experts <= 4096 && max_tiles > 0 && big >= 0 && big <= 2, "bad sizes");
  MLR_REQUIRE(max_tiles >= mlr_moe_max_tiles(pairs, experts, big), "too few tiles for these pairs");
  moe_align_kernel<<<1, 1024, 2 * static_cast<size_t>(experts) * sizeof(int), stream>>>(
      ids, pairs, experts, mlr_moe_tile_rows(big), max_tiles, sorted, offsets, tiles);
  MLR_LAUNCH_CHECK();
  return 0;
}

// One of the two grouped products (`up` 1: act = f(h w_up^T) for the sorted rows, `act` 0 none, 2
// squared ReLU, 3 sigmoid; `up` 0: out[choice, token] = weight * (act w_down^T), float32).  a and w
// in `dtype`; w is [experts, n, k].  `mfma` 1: the streaming matrix-core kernel (bfloat16, k % 8 == 0;
// tiles of 16 rows), 2 and 3: the tiled one (tiles of 64 and of 128 rows, as mlr_moe_align made them
// with `big` 1 and 2; n % 8 == 0 too); 0: plain arithmetic (tiles of 16 rows).
int mlr_moe_gemm(const void* a, const void* w, const int* sorted, const int* offsets, const int* tiles,
                 const float* pair_weights, void* out, int up, int dtype, int mfma, int max_tiles, int tokens, int top,
                 int n, int k, int act, hipStream_t stream) {
  MLR_REQUIRE(a && w && sorted && offsets && tiles && out, "null pointer");
  MLR_REQUIRE(up || pair_weights, "the down product needs the pairs' weights");
  MLR_REQUIRE(max_tiles > 0 && tokens > 0 && top > 0 && n > 0 && k > 0, "sizes must be > 0");
  MLR_REQUIRE(dtype == kF32 || dtype == kBF16, "dtype must be 0 (float32) or 1 (bfloat16)");
  MLR_REQUIRE(act == 0 || act == 2 || act == 3, "unknown activation");
  MLR_REQUIRE((n + kMoeCols - 1) / kMoeCols <= 65535, "too many features for one launch");
  const dim3 grid(max_tiles, (n + kMoeCols - 1) / kMoeCols);
  if (mfma) {
    MLR_REQUIRE(mfma >= 1 && mfma <= 3, "mfma must be within 0..3");
    MLR_REQUIRE(dtype == kBF16 && k % 8 == 0, "the matrix-core kernels take bfloat16 and k % 8 == 0");
    MLR_REQUIRE(mfma == 1 || n % 8 == 0, "the tiled kernel needs n % 8 == 0");
    MLR_REQUIRE(reinterpret_cast<uintptr_t>(a) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(out) % 16 == 0,
                "a, w and out must be 16-byte aligned");
    // rows of `a`: the tokens for the first product, the pairs for the second; both fit 32-bit offsets
    const int64_t a_rows = up ? tokens : static_cast<int64_t>(tokens) * top;
    MLR_REQUIRE(a_rows * k * 2 < (1ll << 32) && static_cast<int64_t>(n) * k * 2 < (1ll << 31),
                "the inputs or one expert's matrix are too large for 32-bit offsets");
    const bf16* ab = static_cast<const bf16*>(a);
    const bf16* wb = static_cast<const bf16*>(w);
    const int rows = static_cast<int>(a_rows);
    if (mfma >= 2) {
      int status;
      if (mfma == 2)
        status = up ? launch_moe_tiled<true, 1>(ab, wb, sorted, offsets, tiles, pair_weights, out, max_tiles, tokens, top, n, k, act, rows, stream)
                    : launch_moe_tiled<false, 1>(ab, wb, sorted, offsets, tiles, pair_weights, out, max_tiles, tokens, top, n, k, act, rows, stream);
      else
        status = up ? launch_moe_tiled<true, 2>(ab, wb, sorted, offsets, tiles, pair_weights, out, max_tiles, tokens, top, n, k, act, rows, stream)
                    : launch_moe_tiled<false, 2>(ab, wb, sorted, offsets, tiles, pair_weights, out, max_tiles, tokens, top, n, k, act, rows, stream);
      if (status != 0) return -1;
    } else if (static_cast<int64_t>(n) * k * 2 >= (1ll << 20)) {
      // an expert's matrix of a megabyte or more: whole lines through LDS
      const dim3 stream_grid(max_tiles, (n + kStCols - 1) / kStCols);
      if (up)
        moe_gemm_stream_kernel<true><<<stream_grid, 256, 0, stream>>>(ab, wb, sorted, offsets, tiles, pair_weights, out, tokens, top, n, k, act, rows);
      else
        moe_gemm_stream_kernel<false><<<stream_grid, 256, 0, stream>>>(ab, wb, sorted, offsets, tiles, pair_weights, out, tokens, top, n, k, act, rows);
    } else {
      // four wavefronts (64 features) a workgroup, or two where that leaves the compute units with too
      // few workgroups to keep their loads in flight
      const int waves = static_cast<int64_t>(max_tiles) * ((n + 63) / 64) < 2048 ? 2 : 4;
      const dim3 small_grid(max_tiles, (n + waves * 16 - 1) / (waves * 16));
      if (up)
        moe_gemm_mfma_kernel<true><<<small_grid, waves * kWave, 0, stream>>>(ab, wb, sorted, offsets, tiles, pair_weights, out, tokens, top, n, k, act, rows);
      else
        moe_gemm_mfma_kernel<false><<<small_grid, waves * kWave, 0, stream>>>(ab, wb, sorted, offsets, tiles, pair_weights, out, tokens, top, n, k, act, rows);
    }
    MLR_LAUNCH_CHECK();
    return 0;
  }
#define MLR_MOE_SIMPLE(T, UP)                                                                                  \
  moe_gemm_simple_kernel<T, UP><<<grid, 256, 0, stream>>>(static_cast<const T*>(a), static_cast<const T*>(w), \
                                                          sorted, offsets, tiles, pair_weights, out, tokens, top, n, k, act)
  if (dtype == kF32) {
    if (up)
      MLR_MOE_SIMPLE(float, true);
    else
      MLR_MOE_SIMPLE(float, false);
  } else {
    if (up)
      MLR_MOE_SIMPLE(bf16, true);
    else
      MLR_MOE_SIMPLE(bf16, false);
  }
#undef MLR_MOE_SIMPLE
  MLR_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
