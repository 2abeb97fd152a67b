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

// One wavefront per token.  s = sigmoid(z); choice score c = s + correction; a group's score is the
// sum of its two largest c; experts outside the `keep` best groups get c = -inf; the `top` largest c
// win, and a winner's weight is its s times `scale`.  Ties go to the lower index.
__global__ __launch_bounds__(kWave) void moe_route_kernel(const float* __restrict__ logits,
                                                          const float* __restrict__ correction,
                                                          int* __restrict__ ids, float* __restrict__ weights,
                                                          int experts, int top, int groups, int keep, float scale) {
  extern __shared__ float route_lds[];
  float* c = route_lds;            // [experts]
  float* s = route_lds + experts;  // [experts]
  float* gs = s + experts;         // [groups]
  const int t = blockIdx.x;
  const int lane = threadIdx.x;
  const int per = experts / groups;
  const float* z = logits + static_cast<int64_t>(t) * experts;
  for (int e = lane; e < experts; e += kWave) {
    const float sv = 1.0f / (1.0f + expf(-z[e]));
    s[e] = sv;
    c[e] = sv + (correction != nullptr ? correction[e] : 0.f);
  }
  __syncthreads();
  if (groups > 1 && keep < groups) {
    for (int g = lane; g < groups; g += kWave) {
      float a = -INFINITY, b = -INFINITY;  // the two largest of the group
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
    if (lane == 0) {
      ids[static_cast<int64_t>(t) * top + k] = i;
      weights[static_cast<int64_t>(t) * top + k] = s[i] * scale;
      c[i] = -INFINITY;
    }
    __syncthreads();
  }
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
// The same two products.  A workgroup of four wavefronts owns 16 rows of a tile (the columns of the
// 16 x 16 x 32 block; weights are the row operand, as in the other product kernels) and 64 features,
// 16 per wavefront.  A lane reads 8 consecutive k of one weight row and of one input row per block:
// both operands straight from memory, no LDS; rows past the tile's end and features past N read
// nothing and multiply zeros.  Few rows a tile (decoding) make this a streaming kernel, whose time
// is the expert weights it reads; with many rows a tile the weights are re-read by every 16 rows
// from L2.
template <bool UP>
__global__ __launch_bounds__(256) void moe_gemm_mfma_kernel(const bf16* __restrict__ a, const bf16* __restrict__ w,
                                                            const int* __restrict__ sorted,
                                                            const int* __restrict__ offsets,
                                                            const int* __restrict__ tiles,
                                                            const float* __restrict__ pair_weights,
                                                            void* __restrict__ out, int tokens, int top, int N, int K,
                                                            int act) {
  const int expert = tiles[2 * blockIdx.x];
  if (expert < 0) return;
  const int row0 = tiles[2 * blockIdx.x + 1];
  const int row_end = offsets[expert + 1];
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int col = lane % 16;   // operand row: weight row / input row of the tile
  const int quad = lane / 16;  // which 8 of a block's 32 k
  const int n_base = blockIdx.y * 64 + wave * 16;
  if (n_base >= N) return;
  // the input row this lane loads (as the column operand), and the rows whose sums it ends up with
  const int in_row = row0 + col;
  const int in_pair = in_row < row_end ? sorted[in_row] : -1;
  const bf16* arow = nullptr;
  if (in_pair >= 0) arow = UP ? a + static_cast<int64_t>(in_pair / top) * K : a + static_cast<int64_t>(in_row) * K;
  const int wn = n_base + col;
  const bf16* wrow = wn < N ? w + (static_cast<int64_t>(expert) * N + wn) * K : nullptr;
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
  const bf16x8_t zero = zero_bf16x8();
  // two blocks of 32 k a turn; the loop's bounds are the same for every lane
  for (int kb = 0; kb < K; kb += 64) {
    const int k1 = kb + quad * 8;
    const int k2 = k1 + 32;
    bf16x8_t wa = zero, xa = zero, wb = zero, xb = zero;
    if (wrow != nullptr && k1 < K) wa = load_bf16x8(wrow + k1);
    if (arow != nullptr && k1 < K) xa = load_bf16x8(arow + k1);
    if (wrow != nullptr && k2 < K) wb = load_bf16x8(wrow + k2);
    if (arow != nullptr && k2 < K) xb = load_bf16x8(arow + k2);
    acc = mfma_16x16x32(wa, xa, acc);
    acc = mfma_16x16x32(wb, xb, acc);
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

}  // namespace mlr

using namespace mlr;

extern "C" {

int mlr_moe_route(const float* logits, const float* correction, int* ids, float* weights, int tokens, int experts,
                  int top, int groups, int keep, float scale, hipStream_t stream) {
  MLR_REQUIRE(logits && ids && weights, "null pointer");
  MLR_REQUIRE(tokens > 0 && experts > 0 && top > 0 && top <= experts, "sizes must be > 0 and top <= experts");
  MLR_REQUIRE(groups > 0 && experts % groups == 0 && keep > 0 && keep <= groups, "bad groups");
  MLR_REQUIRE(top <= keep * (experts / groups), "the kept groups hold fewer experts than a token uses");
  MLR_REQUIRE(experts <= 4096, "at most 4096 experts");
  const size_t lds = (2 * static_cast<size_t>(experts) + groups) * sizeof(float);
  moe_route_kernel<<<tokens, kWave, lds, stream>>>(logits, correction, ids, weights, experts, top, groups, keep, scale);
  MLR_LAUNCH_CHECK();
  return 0;
}

// Rows of one tile of the grouped products (fixed by their kernels).
int mlr_moe_tile_rows() { return kMoeRows; }

// The most tiles `pairs` pairs over `experts` experts can make.
int mlr_moe_max_tiles(int pairs, int experts) {
  const int most = pairs / kMoeRows + experts;  // full tiles, and at most one that is not per expert
  return most < pairs ? most : pairs;
}

int mlr_moe_align(const int* ids, int pairs, int experts, int max_tiles, int* sorted, int* offsets, int* tiles,
                  hipStream_t stream) {
  MLR_REQUIRE(ids && sorted && offsets && tiles, "null pointer");
  MLR_REQUIRE(pairs > 0 && experts > 0 && experts <= 4096 && max_tiles > 0, "bad sizes");
  MLR_REQUIRE(max_tiles >= mlr_moe_max_tiles(pairs, experts), "too few tiles for these pairs");
  moe_align_kernel<<<1, 1024, 2 * static_cast<size_t>(experts) * sizeof(int), stream>>>(ids, pairs, experts, kMoeRows,
                                                                                      max_tiles, sorted, offsets, tiles);
  MLR_LAUNCH_CHECK();
  return 0;
}

// One of the two grouped products (`up` 1: act = f(h w_up^T) for the sorted rows, `act` 0 none, 2
// squared ReLU, 3 sigmoid; `up` 0: out[choice, token] = weight * (act w_down^T), float32).  a and w
// in `dtype`; w is [experts, n, k].  `mfma` 1: the matrix-core kernel (bfloat16, k % 8 == 0).
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
    MLR_REQUIRE(dtype == kBF16 && k % 8 == 0, "the matrix-core kernel takes bfloat16 and k % 8 == 0");
    MLR_REQUIRE(reinterpret_cast<uintptr_t>(a) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0,
                "a and w must be 16-byte aligned");
    if (up)
      moe_gemm_mfma_kernel<true><<<grid, 256, 0, stream>>>(static_cast<const bf16*>(a), static_cast<const bf16*>(w),
                                                           sorted, offsets, tiles, pair_weights, out, tokens, top, n, k, act);
    else
      moe_gemm_mfma_kernel<false><<<grid, 256, 0, stream>>>(static_cast<const bf16*>(a), static_cast<const bf16*>(w),
                                                            sorted, offsets, tiles, pair_weights, out, tokens, top, n, k, act);
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
