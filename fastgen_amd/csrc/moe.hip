// A routed feed-forward (mixture of experts) on the device, without a look of the host at what went
// where, so that a step with it can be recorded:
//
//  route    per token: fp32 router logits (x W_r^T + b), the `top` largest, softmax over those
//  sort     the (token, choice) pairs ordered by expert, cut into tiles of at most TM rows of one expert
//  gate_up  per tile: act = silu(x W_gate^T) * (x W_up^T) with the expert's matrices, rows gathered by token
//  down     per tile: y[pair] = act W_down^T in fp32, one row per pair
//  combine  out[t] = plus[t] + sum_j weight[t][j] * y[t * top + j], in fp32, j ascending
//
// A tile's rows do not depend on one another: every output element is one dot product over k in an
// order fixed by k alone, so a token's result is the same whatever else the step holds and wherever
// the sort puts it.  The bf16 kernels run on the matrix cores (v_mfma_f32_16x16x32_bf16, the expert's
// matrix as the A operand: 16 of its rows x 32 k, a tile's rows of x as B), one wave per 16 output
// channels of a tile, its matrices streamed once for up to 16 * MB rows; the generic kernels (fp32 FMA,
// any dtype and size) are the true 32-bit path.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// ------------------------------------------------------------------- route
// One wave a token.  LDS per wave: n_experts logits, then `top` chosen values.
template <class T>
__global__ __launch_bounds__(256) void moe_route_kernel(
    const T* __restrict__ x, int ldx, const float* __restrict__ wr, const float* __restrict__ bias,
    int n_tokens, int dim, int n_experts, int top, int* __restrict__ choice, float* __restrict__ weight) {
  extern __shared__ float lds[];
  const int lane = threadIdx.x % FG_WAVE, wave = threadIdx.x / FG_WAVE;
  const int t_raw = blockIdx.x * 4 + wave;
  const int t = min(t_raw, n_tokens - 1);  // a wave beyond the tokens computes the last one again and stores nothing
  float* z = lds + (size_t)wave * (n_experts + top);
  float* chosen = z + n_experts;
  const T* xr = x + (size_t)t * ldx;
  for (int e = 0; e < n_experts; ++e) {
    const float* w = wr + (size_t)e * dim;
    float s = 0.f;
    for (int k = lane; k < dim; k += FG_WAVE) s = fmaf(to_f<T>(xr[k]), w[k], s);
    s = wave_sum(s);
    if (lane == 0) z[e] = s + (bias ? bias[e] : 0.f);
  }
  __syncthreads();
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < n_experts; e += FG_WAVE) {
      const float v = z[e];
      if (v > best || (v == best && e < at)) { best = v; at = e; }
    }
#pragma unroll
    for (int m = FG_WAVE / 2; m > 0; m >>= 1) {
      const float ov = __shfl_xor(best, m, FG_WAVE);
      const int oa = __shfl_xor(at, m, FG_WAVE);
      if (ov > best || (ov == best && oa < at)) { best = ov; at = oa; }
    }
    __syncthreads();
    if (lane == 0) {
      at = min(at, n_experts - 1);  // (only if every logit is NaN)
      z[at] = -INFINITY;
      chosen[j] = best;
      if (t_raw < n_tokens) choice[(size_t)t * top + j] = at;
    }
    __syncthreads();
  }
  if (lane == 0 && t_raw < n_tokens) {
    const float m = chosen[0];  // the largest
    float sum = 0.f;
    for (int j = 0; j < top; ++j) sum += expf(chosen[j] - m);
    for (int j = 0; j < top; ++j) weight[(size_t)t * top + j] = expf(chosen[j] - m) / sum;
  }
}

extern "C" int fg_moe_route(const void* x, int ldx, int dtype, const float* wr, const float* bias, int n_tokens, int dim,
                            int n_experts, int top, int* choice, float* weight, hipStream_t stream) {
  if (n_tokens <= 0) return FG_OK;
  if (dim <= 0 || ldx < dim || n_experts <= 0 || top < 1 || top > n_experts) return FG_ERR_ARG;
  const size_t lds = (size_t)4 * (n_experts + top) * sizeof(float);
  if (lds > 60000) return FG_ERR_ARG;
  const int blocks = (n_tokens + 3) / 4;
  if (dtype == FG_F32)
    moe_route_kernel<float><<<blocks, 256, lds, stream>>>((const float*)x, ldx, wr, bias, n_tokens, dim, n_experts, top,
                                                          choice, weight);
  else if (dtype == FG_BF16)
    moe_route_kernel<bf16_t><<<blocks, 256, lds, stream>>>((const bf16_t*)x, ldx, wr, bias, n_tokens, dim, n_experts,
                                                           top, choice, weight);
  else
    return FG_ERR_ARG;
  return fg_launch_status();
}

// -------------------------------------------------------------------- sort
// One workgroup.  sorted[pos] = pair (token * top + j) for the pairs in the order of their experts;
// tiles[i] = (expert, first pos, rows, 0) for i < max_tiles, rows = 0 for tiles that do not exist.
// LDS: 3 * n_experts ints (count, first pos, first tile).
#define SORT_THREADS 1024
__global__ __launch_bounds__(SORT_THREADS) void moe_sort_kernel(
    const int* __restrict__ choice, int n_pairs, int n_experts, int tile_rows, int max_tiles,
    int* __restrict__ sorted, int* __restrict__ tiles) {
  extern __shared__ int sm[];
  int* count = sm;
  int* first = sm + n_experts;
  int* first_tile = sm + 2 * n_experts;
  for (int e = threadIdx.x; e < n_experts; e += SORT_THREADS) count[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < n_pairs; p += SORT_THREADS) atomicAdd(&count[min(max(choice[p], 0), n_experts - 1)], 1);
  __syncthreads();
  if (threadIdx.x < FG_WAVE) {  // exclusive sums of rows and of tiles, 64 experts a round
    const int lane = threadIdx.x;
    int rows_before = 0, tiles_before = 0;
    for (int base = 0; base < n_experts; base += FG_WAVE) {
      const int e = base + lane;
      const int c = e < n_experts ? count[e] : 0;
      const int nt = (c + tile_rows - 1) / tile_rows;
      int sc = c, st = nt;
#pragma unroll
      for (int d = 1; d < FG_WAVE; d <<= 1) {
        const int uc = __shfl_up(sc, d, FG_WAVE), ut = __shfl_up(st, d, FG_WAVE);
        if (lane >= d) { sc += uc; st += ut; }
      }
      if (e < n_experts) {
        first[e] = rows_before + sc - c;
        first_tile[e] = tiles_before + st - nt;
      }
      rows_before += __shfl(sc, FG_WAVE - 1, FG_WAVE);
      tiles_before += __shfl(st, FG_WAVE - 1, FG_WAVE);
    }
    // tiles that do not exist
    for (int i = tiles_before + lane; i < max_tiles; i += FG_WAVE) *(int4*)(tiles + 4 * (size_t)i) = make_int4(0, 0, 0, 0);
  }
  __syncthreads();
  for (int e = threadIdx.x; e < n_experts; e += SORT_THREADS) {
    const int c = count[e], f = first[e];
    for (int i = 0, r = 0; r < c; ++i, r += tile_rows) {
      const int at = first_tile[e] + i;
      if (at < max_tiles) *(int4*)(tiles + 4 * (size_t)at) = make_int4(e, f + r, min(tile_rows, c - r), 0);
    }
    count[e] = 0;  // now the cursor of the second pass
  }
  __syncthreads();
  for (int p = threadIdx.x; p < n_pairs; p += SORT_THREADS) {
    const int e = min(max(choice[p], 0), n_experts - 1);
    sorted[first[e] + atomicAdd(&count[e], 1)] = p;
  }
}

extern "C" int fg_moe_sort(const int* choice, int n_pairs, int n_experts, int tile_rows, int max_tiles, int* sorted,
                           int* tiles, hipStream_t stream) {
  if (n_pairs <= 0) return FG_OK;
  if (n_experts <= 0 || tile_rows <= 0 || max_tiles <= 0 || (size_t)3 * n_experts * sizeof(int) > 60000) return FG_ERR_ARG;
  moe_sort_kernel<<<1, SORT_THREADS, (size_t)3 * n_experts * sizeof(int), stream>>>(choice, n_pairs, n_experts, tile_rows,
                                                                                    max_tiles, sorted, tiles);
  return fg_launch_status();
}

// ------------------------------------------------------------ generic tiles
// fp32 FMA; a thread owns one (row, channel) and sums k ascending in partial sums of 16.
// Tiles of 16 rows; 256 threads: row = tid / 16, channel = blockIdx.y * 16 + tid % 16.
template <class T>
__device__ __forceinline__ float dot_ordered(const T* __restrict__ a, const T* __restrict__ b, int K) {
  float total = 0.f;
  for (int k0 = 0; k0 < K; k0 += 16) {
    float part = 0.f;
    const int k1 = min(K, k0 + 16);
    for (int k = k0; k < k1; ++k) part = fmaf(to_f<T>(a[k]), to_f<T>(b[k]), part);
    total += part;
  }
  return total;
}

template <class T>
__global__ __launch_bounds__(256) void moe_gate_up_generic_kernel(
    const T* __restrict__ x, int ldx, const T* __restrict__ wg, const T* __restrict__ wu, int ldw /* row stride of wg, wu */,
    const int* __restrict__ sorted, const int* __restrict__ tiles, int top, int dim, int hidden, T* __restrict__ act,
    int lda) {
  const int4 tile = *(const int4*)(tiles + 4 * (size_t)blockIdx.x);
  const int r = threadIdx.x / 16, c = blockIdx.y * 16 + threadIdx.x % 16;
  if (r >= tile.z || c >= hidden) return;
  const int pos = tile.y + r;
  const T* xr = x + (size_t)(sorted[pos] / top) * ldx;
  const size_t wrow = ((size_t)tile.x * hidden + c) * ldw;
  const float g = dot_ordered<T>(xr, wg + wrow, dim), u = dot_ordered<T>(xr, wu + wrow, dim);
  act[(size_t)pos * lda + c] = from_f<T>(g / (1.f + expf(-g)) * u);
}

template <class T>
__global__ __launch_bounds__(256) void moe_down_generic_kernel(
    const T* __restrict__ act, int lda, const T* __restrict__ wd, int ldw, const int* __restrict__ sorted,
    const int* __restrict__ tiles, int dim, int hidden, float* __restrict__ y) {
  const int4 tile = *(const int4*)(tiles + 4 * (size_t)blockIdx.x);
  const int r = threadIdx.x / 16, c = blockIdx.y * 16 + threadIdx.x % 16;
  if (r >= tile.z || c >= dim) return;
  const int pos = tile.y + r;
  y[(size_t)sorted[pos] * dim + c] = dot_ordered<T>(act + (size_t)pos * lda, wd + ((size_t)tile.x * dim + c) * ldw, hidden);
}

// --------------------------------------------------------------- MFMA tiles
// One wave per (tile, 16 output channels); a tile has up to 16 * MB rows.  Lane 16 g + r holds, of the A
// operand, row r of the 16 matrix rows at k 8 g .. 8 g + 7, and of B the same k of the tile's row r.
__device__ __forceinline__ bf16x8 moe_zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}
// 16 bytes at row + k if k < K, else zeros; the load is always issued (from the row's start if not)
__device__ __forceinline__ bf16x8 load_k(const bf16_t* row, int k, int K) {
  const bf16x8 v = *(const bf16x8*)(row + (k < K ? k : 0));
  return k < K ? v : moe_zero8();
}

template <int MB>
__global__ __launch_bounds__(256) void moe_gate_up_mfma_kernel(
    const bf16_t* __restrict__ x, int ldx, const bf16_t* __restrict__ wg, const bf16_t* __restrict__ wu, int ldw,
    const int* __restrict__ sorted, const int* __restrict__ tiles, int max_tiles, int top, int dim, int hidden,
    bf16_t* __restrict__ act, int lda) {
  const int lane = threadIdx.x % FG_WAVE, wave = threadIdx.x / FG_WAVE;
  const int cblocks = (hidden + 15) / 16;
  const int item = blockIdx.x * 4 + wave;
  const int ti = item / cblocks, c0 = (item % cblocks) * 16;
  if (ti >= max_tiles) return;
  const int4 tile = *(const int4*)(tiles + 4 * (size_t)ti);
  if (tile.z <= 0) return;
  const int r16 = lane & 15, g = lane >> 4;
  const size_t wrow = ((size_t)tile.x * hidden + min(c0 + r16, hidden - 1)) * ldw;  // rows beyond the matrix: clamped, not stored
  const bf16_t* pg = wg + wrow;
  const bf16_t* pu = wu + wrow;
  const bf16_t* px[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int r = min(mb * 16 + r16, tile.z - 1);
    px[mb] = x + (size_t)(sorted[tile.y + r] / top) * ldx;
  }
  f32x4 ag[MB], au[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) ag[mb] = au[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 8 * g; k0 < dim + 8 * g; k0 += 64) {  // this lane's k: 8 g, 8 g + 32, ...
    bf16x8 a0 = load_k(pg, k0, dim), a1 = load_k(pg, k0 + 32, dim);
    bf16x8 u0 = load_k(pu, k0, dim), u1 = load_k(pu, k0 + 32, dim);
    bf16x8 b0[MB], b1[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      b0[mb] = load_k(px[mb], k0, dim);
      b1[mb] = load_k(px[mb], k0 + 32, dim);
    }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      ag[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, b0[mb], ag[mb], 0, 0, 0);
      au[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(u0, b0[mb], au[mb], 0, 0, 0);
      ag[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, b1[mb], ag[mb], 0, 0, 0);
      au[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(u1, b1[mb], au[mb], 0, 0, 0);
    }
  }
  // the lane holds, for the tile's row mb * 16 + r16, channels c0 + 4 g .. + 3
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int r = mb * 16 + r16, c = c0 + 4 * g;
    if (r >= tile.z || c >= hidden) continue;
    bf16x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float gv = ag[mb][i];
      o[i] = (__bf16)(gv * __frcp_rn(1.f + __expf(-gv)) * au[mb][i]);
    }
    bf16_t* dst = act + (size_t)(tile.y + r) * lda + c;
    if (c + 3 < hidden) {
      *(bf16x4*)dst = o;
    } else {
      for (int i = 0; c + i < hidden; ++i) dst[i] = o[i];
    }
  }
}

template <int MB>
__global__ __launch_bounds__(256) void moe_down_mfma_kernel(
    const bf16_t* __restrict__ act, int lda, const bf16_t* __restrict__ wd, int ldw, const int* __restrict__ sorted,
    const int* __restrict__ tiles, int max_tiles, int dim, int hidden, float* __restrict__ y) {
  const int lane = threadIdx.x % FG_WAVE, wave = threadIdx.x / FG_WAVE;
  const int cblocks = (dim + 15) / 16;
  const int item = blockIdx.x * 4 + wave;
  const int ti = item / cblocks, c0 = (item % cblocks) * 16;
  if (ti >= max_tiles) return;
  const int4 tile = *(const int4*)(tiles + 4 * (size_t)ti);
  if (tile.z <= 0) return;
  const int r16 = lane & 15, g = lane >> 4;
  const bf16_t* pw = wd + ((size_t)tile.x * dim + min(c0 + r16, dim - 1)) * ldw;
  const bf16_t* pa[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) pa[mb] = act + (size_t)(tile.y + min(mb * 16 + r16, tile.z - 1)) * lda;
  f32x4 acc[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) acc[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 8 * g; k0 < hidden + 8 * g; k0 += 64) {
    bf16x8 a0 = load_k(pw, k0, hidden), a1 = load_k(pw, k0 + 32, hidden);
    bf16x8 b0[MB], b1[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      b0[mb] = load_k(pa[mb], k0, hidden);
      b1[mb] = load_k(pa[mb], k0 + 32, hidden);
    }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, b0[mb], acc[mb], 0, 0, 0);
      acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, b1[mb], acc[mb], 0, 0, 0);
    }
  }
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int r = mb * 16 + r16, c = c0 + 4 * g;
    if (r >= tile.z || c >= dim) continue;
    float* dst = y + (size_t)sorted[tile.y + r] * dim + c;
    if (c + 3 < dim && dim % 4 == 0) {
      *(f32x4*)dst = acc[mb];
    } else {
      for (int i = 0; c + i < dim; ++i) dst[i] = acc[mb][i];
    }
  }
}

// x [T, dim] rows gathered by token; wg, wu [E, hidden, ldw], act [n_pairs, lda] in the sorted order.
// mfma: bf16 with dim % 8 == 0, ldx % 8 == 0, ldw % 8 == 0 (16-byte loads); tile_rows = 16 * MB, MB in 1, 2, 4.
extern "C" int fg_moe_gate_up(const void* x, int ldx, const void* wg, const void* wu, int ldw, const int* sorted,
                              const int* tiles, int max_tiles, int tile_rows, int top, int dim, int hidden, void* act,
                              int lda, int dtype, int mfma, hipStream_t stream) {
  if (max_tiles <= 0) return FG_OK;
  if (dim <= 0 || hidden <= 0 || top <= 0 || ldx < dim || ldw < dim || lda < hidden) return FG_ERR_ARG;
  if (mfma) {
    if (dtype != FG_BF16 || dim % 8 || ldx % 8 || ldw % 8 || lda % 4) return FG_ERR_ARG;
    const long long items = (long long)max_tiles * ((hidden + 15) / 16);
    const unsigned blocks = (unsigned)((items + 3) / 4);
#define GO(MB)                                                                                                   \
  moe_gate_up_mfma_kernel<MB><<<blocks, 256, 0, stream>>>((const bf16_t*)x, ldx, (const bf16_t*)wg, (const bf16_t*)wu, \
                                                          ldw, sorted, tiles, max_tiles, top, dim, hidden, (bf16_t*)act, lda)
    if (tile_rows == 16) GO(1);
    else if (tile_rows == 32) GO(2);
    else if (tile_rows == 64) GO(4);
    else return FG_ERR_ARG;
#undef GO
    return fg_launch_status();
  }
  if (tile_rows != 16 || max_tiles > 2147483647 / 4) return FG_ERR_ARG;
  dim3 grid(max_tiles, (hidden + 15) / 16);
  if (grid.y > 65535) return FG_ERR_ARG;
  if (dtype == FG_F32)
    moe_gate_up_generic_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, ldx, (const float*)wg, (const float*)wu,
                                                                ldw, sorted, tiles, top, dim, hidden, (float*)act, lda);
  else if (dtype == FG_BF16)
    moe_gate_up_generic_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, ldx, (const bf16_t*)wg,
                                                                 (const bf16_t*)wu, ldw, sorted, tiles, top, dim, hidden,
                                                                 (bf16_t*)act, lda);
  else
    return FG_ERR_ARG;
  return fg_launch_status();
}

// act [n_pairs, lda] in the sorted order; wd [E, dim, ldw]; y fp32 [n_pairs, dim], row = pair.
extern "C" int fg_moe_down(const void* act, int lda, const void* wd, int ldw, const int* sorted, const int* tiles,
                           int max_tiles, int tile_rows, int dim, int hidden, float* y, int dtype, int mfma,
                           hipStream_t stream) {
  if (max_tiles <= 0) return FG_OK;
  if (dim <= 0 || hidden <= 0 || lda < hidden || ldw < hidden) return FG_ERR_ARG;
  if (mfma) {
    if (dtype != FG_BF16 || hidden % 8 || lda % 8 || ldw % 8) return FG_ERR_ARG;
    const long long items = (long long)max_tiles * ((dim + 15) / 16);
    const unsigned blocks = (unsigned)((items + 3) / 4);
#define GO(MB)                                                                                                      \
  moe_down_mfma_kernel<MB><<<blocks, 256, 0, stream>>>((const bf16_t*)act, lda, (const bf16_t*)wd, ldw, sorted, tiles, \
                                                       max_tiles, dim, hidden, y)
    if (tile_rows == 16) GO(1);
    else if (tile_rows == 32) GO(2);
    else if (tile_rows == 64) GO(4);
    else return FG_ERR_ARG;
#undef GO
    return fg_launch_status();
  }
  if (tile_rows != 16) return FG_ERR_ARG;
  dim3 grid(max_tiles, (dim + 15) / 16);
  if (grid.y > 65535) return FG_ERR_ARG;
  if (dtype == FG_F32)
    moe_down_generic_kernel<float><<<grid, 256, 0, stream>>>((const float*)act, lda, (const float*)wd, ldw, sorted, tiles,
                                                             dim, hidden, y);
  else if (dtype == FG_BF16)
    moe_down_generic_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)act, lda, (const bf16_t*)wd, ldw, sorted,
                                                              tiles, dim, hidden, y);
  else
    return FG_ERR_ARG;
  return fg_launch_status();
}

// ----------------------------------------------------------------- combine
// out[t] = plus[t] + sum_j weight[t][j] * y[t * top + j]: the weighted sum first, j ascending, all fp32.
template <class TP>
__global__ __launch_bounds__(256) void moe_combine_kernel(
    const float* __restrict__ y, const float* __restrict__ weight, const TP* __restrict__ plus, int ldp, int top, int dim,
    float* __restrict__ out) {
  const int t = blockIdx.x;
  for (int d = threadIdx.x; d < dim; d += 256) {
    float s = 0.f;
    for (int j = 0; j < top; ++j) s = fmaf(weight[(size_t)t * top + j], y[((size_t)t * top + j) * dim + d], s);
    if (plus) s += to_f<TP>(plus[(size_t)t * ldp + d]);
    out[(size_t)t * dim + d] = s;
  }
}

extern "C" int fg_moe_combine(const float* y, const float* weight, const void* plus, int ldp, int plus_dtype,
                              int n_tokens, int top, int dim, float* out, hipStream_t stream) {
  if (n_tokens <= 0) return FG_OK;
  if (top <= 0 || dim <= 0 || (plus && ldp < dim)) return FG_ERR_ARG;
  if (plus_dtype == FG_F32)
    moe_combine_kernel<float><<<n_tokens, 256, 0, stream>>>(y, weight, (const float*)plus, ldp, top, dim, out);
  else if (plus_dtype == FG_BF16)
    moe_combine_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>(y, weight, (const bf16_t*)plus, ldp, top, dim, out);
  else
    return FG_ERR_ARG;
  return fg_launch_status();
}
