// A routed feed-forward (mixture of experts) on the device, without a look of the host at what went
// where, so that a step with it can be recorded:
//
//  route    per token (a workgroup): fp32 router logits (x W_r^T + b), the `top` largest, softmax over those
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
// A workgroup a token.  Logits: the WAVES waves take the experts in turns of EPW (a wave reads the row of
// x once for its EPW experts, eight elements a lane and round; the lanes' partial sums are added by the
// wave in a fixed order), into LDS.  Few tokens (decode) get 16 waves a token and 2 experts a turn, so that
// the router's rows are asked for by many waves at once; many tokens 4 waves and 4 experts a turn.  Then the `top` largest (ties: the lower expert) by a
// wave-wide argmax repeated `top` times, and the softmax over them; every wave does this on the same LDS
// values, the first one stores.  LDS: n_experts logits, then `top` chosen values, then n_experts scores.
//
// A second way of scoring (`sigmoid_scores`): an expert's score is sigmoid(logit); the choice goes by the
// score plus `correction` (per expert, or null), inside the `keep_groups` best of `n_groups` groups of
// neighbouring experts (a group's rank: the sum of its two largest choice scores; the experts of the other
// groups cannot be chosen); the weights are the chosen experts' scores without the correction, divided by
// their sum (+ 1e-20) and multiplied by `weight_scale`.  A third way (`sigmoid_scores` = 2): the scores are the
// softmax of the logits over all experts; choice, groups and weights as with sigmoid scores.
//
// `n_extra`: the router matrix has that many rows more than there are experts; their logits (no bias) take no
// part in the choice and are stored as they are in `extra [n_tokens, n_extra]` (a gate of a shared expert, say).
struct RouteMode {
  int sigmoid_scores;
  const float* correction;
  int n_groups, keep_groups;
  float weight_scale;
  int n_extra;
  float* extra;
};
template <class T, int WAVES, int EPW>
__global__ __launch_bounds__(64 * WAVES) void moe_route_kernel(
    const T* __restrict__ x, int ldx, const float* __restrict__ wr, const float* __restrict__ bias,
    int dim, int n_experts, int top, int* __restrict__ choice, float* __restrict__ weight, const RouteMode mode) {
  extern __shared__ float lds[];
  float* z = lds;
  float* chosen = lds + n_experts + mode.n_extra;
  const int n_rows = n_experts + mode.n_extra;  // rows of the router matrix
  float* score = chosen + top;
  const int lane = threadIdx.x % FG_WAVE, wave = threadIdx.x / FG_WAVE;
  const size_t t = blockIdx.x;
  const T* xr = x + t * ldx;
  for (int e0 = wave * EPW; e0 < n_rows; e0 += WAVES * EPW) {
    float s[EPW];
#pragma unroll
    for (int j = 0; j < EPW; ++j) s[j] = 0.f;
    if (dim % 8 == 0 && ldx % 8 == 0) {
      for (int k = lane * 8; k < dim; k += FG_WAVE * 8) {
        float xv[8];
        load8<T>(xr + k, xv);
#pragma unroll
        for (int j = 0; j < EPW; ++j) {
          float wv[8];
          load8<float>(wr + (size_t)min(e0 + j, n_rows - 1) * dim + k, wv);
#pragma unroll
          for (int i = 0; i < 8; ++i) s[j] = fmaf(xv[i], wv[i], s[j]);
        }
      }
    } else {
      for (int k = lane; k < dim; k += FG_WAVE) {
        const float xv = to_f<T>(xr[k]);
#pragma unroll
        for (int j = 0; j < EPW; ++j) s[j] = fmaf(xv, wr[(size_t)min(e0 + j, n_rows - 1) * dim + k], s[j]);
      }
    }
#pragma unroll
    for (int j = 0; j < EPW; ++j) {
      const float v = wave_sum(s[j]);
      if (lane == 0 && e0 + j < n_rows) z[e0 + j] = v + (bias && e0 + j < n_experts ? bias[e0 + j] : 0.f);
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < mode.n_extra; e += blockDim.x) mode.extra[t * mode.n_extra + e] = z[n_experts + e];
  if (mode.sigmoid_scores) {  // uniform
    float top_z = 0.f, all = 1.f;
    if (mode.sigmoid_scores == 2) {
      // every thread takes the maximum and the sum over all experts itself, in the experts' order
      top_z = -INFINITY;
      for (int e = 0; e < n_experts; ++e) top_z = fmaxf(top_z, z[e]);
      all = 0.f;
      for (int e = 0; e < n_experts; ++e) all += expf(z[e] - top_z);
      __syncthreads();  // every thread has read the logits before any of them is overwritten
    }
    for (int e = threadIdx.x; e < n_experts; e += blockDim.x) {
      const float sc = mode.sigmoid_scores == 2 ? expf(z[e] - top_z) / all : 1.f / (1.f + expf(-z[e]));
      score[e] = sc;
      z[e] = sc + (mode.correction ? mode.correction[e] : 0.f);
    }
    __syncthreads();
    if (mode.n_groups > 1 && mode.keep_groups < mode.n_groups) {  // uniform
      // one wave ranks the groups (a lane a group, in turns) and strikes the experts of those that lose
      float* rank = score + n_experts;  // n_groups values
      const int per = n_experts / mode.n_groups;
      if (wave == 0) {
        for (int g = lane; g < mode.n_groups; g += FG_WAVE) {
          float a = -INFINITY, b = -INFINITY;  // the two largest
          for (int i = 0; i < per; ++i) {
            const float v = z[g * per + i];
            if (v > a) { b = a; a = v; } else if (v > b) { b = v; }
          }
          rank[g] = per > 1 ? a + b : a;
        }
      }
      __syncthreads();
      if (wave == 0) {
        for (int g = lane; g < mode.n_groups; g += FG_WAVE) {
          // a group stays if fewer than keep_groups groups rank before it (ties: the lower group first)
          int before = 0;
          const float mine = rank[g];
          for (int o = 0; o < mode.n_groups; ++o) before += (rank[o] > mine || (rank[o] == mine && o < g)) ? 1 : 0;
          if (before >= mode.keep_groups)
            for (int i = 0; i < per; ++i) z[g * per + i] = -INFINITY;
        }
      }
      __syncthreads();
    }
  }
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
    __syncthreads();  // every wave has read the logits of this turn
    if (threadIdx.x == 0) {
      at = min(at, n_experts - 1);  // (only if every logit is NaN)
      z[at] = -INFINITY;
      chosen[j] = mode.sigmoid_scores ? score[at] : best;
      choice[t * top + j] = at;
    }
    __syncthreads();
  }
  if (threadIdx.x == 0 && mode.sigmoid_scores) {
    float sum = 0.f;
    for (int j = 0; j < top; ++j) sum += chosen[j];
    for (int j = 0; j < top; ++j) weight[t * top + j] = chosen[j] / (sum + 1e-20f) * mode.weight_scale;
  } else if (threadIdx.x == 0) {
    const float m = chosen[0];  // the largest
    float sum = 0.f;
    for (int j = 0; j < top; ++j) sum += expf(chosen[j] - m);
    for (int j = 0; j < top; ++j) weight[t * top + j] = expf(chosen[j] - m) / sum;
  }
}

extern "C" int fg_moe_route_mode(const void* x, int ldx, int dtype, const float* wr, const float* bias, int n_tokens,
                                 int dim, int n_experts, int top, int* choice, float* weight, int sigmoid_scores,
                                 const float* correction, int n_groups, int keep_groups, float weight_scale,
                                 int n_extra, float* extra, hipStream_t stream) {
  if (n_tokens <= 0) return FG_OK;
  if (sigmoid_scores < 0 || sigmoid_scores > 2 || n_extra < 0 || (n_extra > 0 && !extra)) return FG_ERR_ARG;
  if (dim <= 0 || ldx < dim || n_experts <= 0 || top < 1 || top > n_experts) return FG_ERR_ARG;
  if (n_groups < 1 || n_experts % n_groups || keep_groups < 1 || keep_groups > n_groups ||
      top > keep_groups * (n_experts / n_groups) || (!sigmoid_scores && (correction || n_groups > 1)))
    return FG_ERR_ARG;
  const RouteMode mode = {sigmoid_scores, correction, n_groups, keep_groups, weight_scale, n_extra, extra};
  const size_t lds = (size_t)(2 * n_experts + n_extra + top + n_groups) * sizeof(float);
  if (lds > 60000) return FG_ERR_ARG;
#define GO(T, WAVES, EPW)                                                                                        \
  moe_route_kernel<T, WAVES, EPW><<<n_tokens, 64 * WAVES, lds, stream>>>((const T*)x, ldx, wr, bias, dim, n_experts, \
                                                                         top, choice, weight, mode)
  const bool few = n_tokens <= 64;
  if (dtype == FG_F32) {
    if (few) GO(float, 16, 2); else GO(float, 4, 4);
  } else if (dtype == FG_BF16) {
    if (few) GO(bf16_t, 16, 2); else GO(bf16_t, 4, 4);
  } else {
    return FG_ERR_ARG;
  }
#undef GO
  return fg_launch_status();
}

extern "C" int fg_moe_route(const void* x, int ldx, int dtype, const float* wr, const float* bias, int n_tokens, int dim,
                            int n_experts, int top, int* choice, float* weight, hipStream_t stream) {
  return fg_moe_route_mode(x, ldx, dtype, wr, bias, n_tokens, dim, n_experts, top, choice, weight, 0, nullptr, 1, 1, 1.f,
                           0, nullptr, stream);
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
    int lda, const GatedAct fn) {
  const int4 tile = *(const int4*)(tiles + 4 * (size_t)blockIdx.x);
  const int r = threadIdx.x / 16, c = blockIdx.y * 16 + threadIdx.x % 16;
  if (r >= tile.z || c >= hidden) return;
  const int pos = tile.y + r;
  const T* xr = x + (size_t)(sorted[pos] / top) * ldx;
  const size_t wrow = ((size_t)tile.x * hidden + c) * ldw;
  const float g = dot_ordered<T>(xr, wg + wrow, dim), u = dot_ordered<T>(xr, wu + wrow, dim);
  act[(size_t)pos * lda + c] = from_f<T>(gated_act<false>(g, u, fn));
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
    bf16_t* __restrict__ act, int lda, const GatedAct fn) {
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
  // U steps of 32 k a round, all their loads issued before the first MFMA: with few rows a wave is a chain of
  // memory round trips, and the fewer of them the better (8 steps for one block of rows: 24 loads in flight)
  constexpr int U = MB == 1 ? 8 : (MB == 2 ? 4 : 2);
  for (int k0 = 8 * g; k0 < dim + 8 * g; k0 += 32 * U) {  // this lane's k: 8 g, 8 g + 32, ...
    bf16x8 a[U], u[U], b[U][MB];
#pragma unroll
    for (int i = 0; i < U; ++i) {
      a[i] = load_k(pg, k0 + 32 * i, dim);
      u[i] = load_k(pu, k0 + 32 * i, dim);
    }
#pragma unroll
    for (int i = 0; i < U; ++i)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) b[i][mb] = load_k(px[mb], k0 + 32 * i, dim);
#pragma unroll
    for (int i = 0; i < U; ++i)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        ag[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[i][mb], ag[mb], 0, 0, 0);
        au[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(u[i], b[i][mb], au[mb], 0, 0, 0);
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
      o[i] = (__bf16)gated_act<true>(ag[mb][i], au[mb][i], fn);
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
  constexpr int U = MB == 1 ? 8 : (MB == 2 ? 4 : 2);  // as in gate_up
  for (int k0 = 8 * g; k0 < hidden + 8 * g; k0 += 32 * U) {
    bf16x8 a[U], b[U][MB];
#pragma unroll
    for (int i = 0; i < U; ++i) a[i] = load_k(pw, k0 + 32 * i, hidden);
#pragma unroll
    for (int i = 0; i < U; ++i)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) b[i][mb] = load_k(pa[mb], k0 + 32 * i, hidden);
#pragma unroll
    for (int i = 0; i < U; ++i)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[i][mb], acc[mb], 0, 0, 0);
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

// ------------------------------------------------------- large tiles through LDS
// Many rows an expert (prompt steps): a workgroup owns a tile of up to 64 WM rows of one expert and 128
// output columns, its WM x 2 waves 64 x 64 each; both operands go from memory straight into LDS
// (global_load_lds) through a ring of NST stages of 32 k, as in gemm_tiled.hip, whose loop this is.  What
// differs is where the rows come from and go to: the tile's rows of x are gathered by token (gate_up) or
// are its sorted places (down), the matrix is the tile's expert's, and for gate_up its 16-row blocks are
// made of 8 gate rows and the 8 up rows of the same channels as they are loaded (nothing is stored
// interleaved), so that silu(gate) * up is applied to the accumulators.
#define MT_GATE_UP 0
#define MT_DOWN 1

template <int N>
__device__ __forceinline__ void moe_wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt has six bits");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

template <int WM, int NST, int EPI>
__global__ __launch_bounds__(128 * WM) void moe_tiled_kernel(
    const bf16_t* __restrict__ x, int ldx, const bf16_t* __restrict__ w0, const bf16_t* __restrict__ w1, int ldw,
    void* __restrict__ y, int ldy, const int* __restrict__ sorted, const int* __restrict__ tiles, int top,
    int N /* rows of the matrix as the tile sees it: 2 * hidden (gate_up), dim (down) */, int K, const GatedAct fn) {
  constexpr int WN = 2, NW = WM * WN, WB = 4 * WN, XB = 4 * WM, NB = WB + XB, LPW = NB / NW, BLOCK = 16 * 32;
  static_assert(NB % NW == 0 && NST >= 3 && LPW * (NST - 2) < 64, "blocks divide over the waves; loads fit the counter");
  extern __shared__ __attribute__((aligned(16))) bf16_t ring[];  // [NST][NB][BLOCK]
  const int4 tile = *(const int4*)(tiles + 4 * (size_t)blockIdx.y);
  if (tile.z <= 0) return;  // (the whole workgroup)
  const int lane = threadIdx.x % FG_WAVE, wave = threadIdx.x / FG_WAVE;
  const int r16 = lane & 15, g = lane >> 4;
  const int wm = wave / WN, wn = wave % WN;
  const int n_base = blockIdx.x * (64 * WN);
  const int n_stages = (K + 31) / 32;

  const bf16_t* src[LPW];
#pragma unroll
  for (int j = 0; j < LPW; ++j) {
    const int b = wave + NW * j;
    if (b >= WB) {
      const int pos = tile.y + min(16 * (b - WB) + r16, tile.z - 1);  // rows beyond the tile: its last row, not stored
      src[j] = x + (size_t)(EPI == MT_GATE_UP ? sorted[pos] / top : pos) * ldx + 8 * g;
    } else {
      const int vr = min(n_base + 16 * b + r16, N - 1);
      if (EPI == MT_GATE_UP)
        src[j] = ((vr & 8) ? w1 : w0) + ((size_t)tile.x * (N >> 1) + ((vr >> 4) << 3) + (vr & 7)) * ldw + 8 * g;
      else
        src[j] = w0 + ((size_t)tile.x * N + vr) * ldw + 8 * g;
    }
  }
  auto issue = [&](int s) {
    const int k = 32 * min(s, n_stages - 1);
    const int koff = k + 8 * g < K ? k : 0;  // a chunk beyond k: any readable one, zeroed at use
    bf16_t* slot = ring + (size_t)(s % NST) * NB * BLOCK;
#pragma unroll
    for (int j = 0; j < LPW; ++j)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src[j] + koff),
                                       (__attribute__((address_space(3))) void*)(slot + (wave + NW * j) * BLOCK), 16, 0, 0);
  };

  f32x4 acc[4][4];  // [row block mb][column block nb]
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) acc[mb][nb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int s = 0; s < NST - 1; ++s) issue(s);
  for (int i = 0; i < n_stages; ++i) {
    moe_wait_vmcnt<LPW*(NST - 2)>();  // this wave's loads of stage i have landed
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();  // everybody's have, and nobody reads stage i - 1 any more
    asm volatile("" ::: "memory");
    issue(i + NST - 1);
    const bf16_t* st = ring + (size_t)(i % NST) * NB * BLOCK;
    const bool in = 32 * i + 8 * g < K;
    bf16x8 a[4], b[4];
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
      a[nb] = *(const bf16x8*)(st + (wn * 4 + nb) * BLOCK + lane * 8);
      a[nb] = in ? a[nb] : moe_zero8();
    }
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) b[mb] = *(const bf16x8*)(st + (WB + wm * 4 + mb) * BLOCK + lane * 8);
#pragma unroll
    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
      for (int mb = 0; mb < 4; ++mb) acc[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[nb], b[mb], acc[mb][nb], 0, 0, 0);
  }
  moe_wait_vmcnt<0>();  // the loads issued past the end land before the workgroup's LDS is given up

  // acc[mb][nb][i]: the tile's row 64 wm + 16 mb + r16, matrix row n_base + 64 wn + 16 nb + 4 g + i
#pragma unroll
  for (int mb = 0; mb < 4; ++mb) {
    const int ml = 64 * wm + 16 * mb + r16;
    const bool valid = ml < tile.z;
    const int pos = tile.y + min(ml, tile.z - 1);
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
      const int n0 = n_base + 64 * wn + 16 * nb;
      if (EPI == MT_DOWN) {
        const int n = n0 + 4 * g;
        if (!valid) continue;
        float* dst = (float*)y + (size_t)sorted[pos] * ldy + n;
        if (n + 3 < N && (ldy & 3) == 0) {
          *(f32x4*)dst = acc[mb][nb];
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (n + i < N) dst[i] = acc[mb][nb][i];
        }
      } else {
        // lane groups 0, 1 hold the gate rows 4 g + i of 8 channels, groups 2, 3 the up rows of the same channels
        bf16x4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float up = __shfl_xor(acc[mb][nb][i], 32, FG_WAVE);
          const float gate = acc[mb][nb][i];
          v[i] = (__bf16)gated_act<true>(gate, up, fn);
        }
        if (g < 2 && valid && n0 + 15 < N) *(bf16x4*)((bf16_t*)y + (size_t)pos * ldy + n0 / 2 + 4 * g) = v;
      }
    }
  }
}

template <int WM, int EPI>
static int launch_moe_tiled(const void* x, int ldx, const void* w0, const void* w1, int ldw, void* y, int ldy,
                            const int* sorted, const int* tiles, int max_tiles, int top, int N, int K, const GatedAct fn,
                            hipStream_t stream) {
  constexpr int NST = 4, lds = NST * 4 * (WM + 2) * 1024;
  static bool raised = false;  // more than 64 KB of dynamic LDS has to be asked for once
  auto kernel = moe_tiled_kernel<WM, NST, EPI>;
  if (lds > 65536 && !raised) {
    if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
      return FG_ERR_LAUNCH;
    raised = true;
  }
  if (max_tiles > 65535) return FG_ERR_ARG;
  const dim3 grid((N + 127) / 128, max_tiles);
  kernel<<<grid, 128 * WM, lds, stream>>>((const bf16_t*)x, ldx, (const bf16_t*)w0, (const bf16_t*)w1, ldw, y, ldy, sorted,
                                          tiles, top, N, K, fn);
  return fg_launch_status();
}

// x [T, dim] rows gathered by token; wg, wu [E, hidden, ldw], act [n_pairs, lda] in the sorted order.
// mfma: bf16 with dim % 8 == 0, ldx % 8 == 0, ldw % 8 == 0 (16-byte loads); tile_rows = 16 * MB, MB in 1, 2, 4,
// or 128 / 256: the tiles that go through LDS.
// act_kind, limit, alpha: the gated activation (GatedAct in common.h).
extern "C" int fg_moe_gate_up_act(const void* x, int ldx, const void* wg, const void* wu, int ldw, const int* sorted,
                                  const int* tiles, int max_tiles, int tile_rows, int top, int dim, int hidden, void* act,
                                  int lda, int dtype, int mfma, int act_kind, float limit, float alpha,
                                  hipStream_t stream) {
  if (max_tiles <= 0) return FG_OK;
  if (act_kind != FG_ACT_SILU && !(act_kind == FG_ACT_LIMITED && limit > 0.f)) return FG_ERR_ARG;
  const GatedAct fn = {act_kind, limit, alpha};
  if (dim <= 0 || hidden <= 0 || top <= 0 || ldx < dim || ldw < dim || lda < hidden) return FG_ERR_ARG;
  if (mfma) {
    if (dtype != FG_BF16 || dim % 8 || ldx % 8 || ldw % 8 || lda % 4) return FG_ERR_ARG;
    if (tile_rows == 128 || tile_rows == 256) {
      if (hidden % 8 || dim < 32) return FG_ERR_ARG;  // (a lane's stand-in load reads the row's first 32 k)
      return tile_rows == 128
                 ? launch_moe_tiled<2, MT_GATE_UP>(x, ldx, wg, wu, ldw, act, lda, sorted, tiles, max_tiles, top, 2 * hidden, dim, fn, stream)
                 : launch_moe_tiled<4, MT_GATE_UP>(x, ldx, wg, wu, ldw, act, lda, sorted, tiles, max_tiles, top, 2 * hidden, dim, fn, stream);
    }
    const long long items = (long long)max_tiles * ((hidden + 15) / 16);
    const unsigned blocks = (unsigned)((items + 3) / 4);
#define GO(MB)                                                                                                   \
  moe_gate_up_mfma_kernel<MB><<<blocks, 256, 0, stream>>>((const bf16_t*)x, ldx, (const bf16_t*)wg, (const bf16_t*)wu, \
                                                          ldw, sorted, tiles, max_tiles, top, dim, hidden, (bf16_t*)act, lda, fn)
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
                                                                ldw, sorted, tiles, top, dim, hidden, (float*)act, lda, fn);
  else if (dtype == FG_BF16)
    moe_gate_up_generic_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, ldx, (const bf16_t*)wg,
                                                                 (const bf16_t*)wu, ldw, sorted, tiles, top, dim, hidden,
                                                                 (bf16_t*)act, lda, fn);
  else
    return FG_ERR_ARG;
  return fg_launch_status();
}

extern "C" int fg_moe_gate_up(const void* x, int ldx, const void* wg, const void* wu, int ldw, const int* sorted,
                              const int* tiles, int max_tiles, int tile_rows, int top, int dim, int hidden, void* act,
                              int lda, int dtype, int mfma, hipStream_t stream) {
  return fg_moe_gate_up_act(x, ldx, wg, wu, ldw, sorted, tiles, max_tiles, tile_rows, top, dim, hidden, act, lda, dtype,
                            mfma, FG_ACT_SILU, 0.f, 1.f, stream);
}

// act [n_pairs, lda] in the sorted order; wd [E, dim, ldw]; y fp32 [n_pairs, dim], row = pair.
extern "C" int fg_moe_down(const void* act, int lda, const void* wd, int ldw, const int* sorted, const int* tiles,
                           int max_tiles, int tile_rows, int dim, int hidden, float* y, int dtype, int mfma,
                           hipStream_t stream) {
  if (max_tiles <= 0) return FG_OK;
  if (dim <= 0 || hidden <= 0 || lda < hidden || ldw < hidden) return FG_ERR_ARG;
  if (mfma) {
    if (dtype != FG_BF16 || hidden % 8 || lda % 8 || ldw % 8) return FG_ERR_ARG;
    if ((tile_rows == 128 || tile_rows == 256) && hidden < 32) return FG_ERR_ARG;
    if (tile_rows == 128 || tile_rows == 256)
      return tile_rows == 128
                 ? launch_moe_tiled<2, MT_DOWN>(act, lda, wd, nullptr, ldw, y, dim, sorted, tiles, max_tiles, 1, dim, hidden, GatedAct{0, 0.f, 1.f}, stream)
                 : launch_moe_tiled<4, MT_DOWN>(act, lda, wd, nullptr, ldw, y, dim, sorted, tiles, max_tiles, 1, dim, hidden, GatedAct{0, 0.f, 1.f}, stream);
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
// plus: rows of the activation dtype, or (n_plus > 0) fp32 partial sums plus[p * plus_stride + t * ldp + d],
// whose sum, in order, is what is added.  plus_gate (fp32, one number a token at plus_gate[t * gate_stride]): the
// rows of plus are multiplied by its sigmoid before they are added.
template <class TP>
__global__ __launch_bounds__(256) void moe_combine_kernel(
    const float* __restrict__ y, const float* __restrict__ weight, const TP* __restrict__ plus, int ldp, int n_plus,
    size_t plus_stride, int top, int dim, float* __restrict__ out, const float* __restrict__ plus_gate, int gate_stride) {
  const int t = blockIdx.x;
  const float pg = plus_gate ? 1.f / (1.f + expf(-plus_gate[(size_t)t * gate_stride])) : 1.f;
  for (int d = threadIdx.x; d < dim; d += 256) {
    float s = 0.f;
    for (int j = 0; j < top; ++j) s = fmaf(weight[(size_t)t * top + j], y[((size_t)t * top + j) * dim + d], s);
    if (plus) {
      float m = to_f<TP>(plus[(size_t)t * ldp + d]);
      for (int p = 1; p < n_plus; ++p) m += to_f<TP>(plus[p * plus_stride + (size_t)t * ldp + d]);
      s = (plus_gate ? m * pg : m) + s;
    }
    out[(size_t)t * dim + d] = s;
  }
}

extern "C" int fg_moe_combine_gated(const float* y, const float* weight, const void* plus, int ldp, int plus_dtype,
                                    int n_plus, long long plus_stride, int n_tokens, int top, int dim, float* out,
                                    const float* plus_gate, int gate_stride, hipStream_t stream) {
  if (n_tokens <= 0) return FG_OK;
  if (plus_gate && (!plus || gate_stride < 1)) return FG_ERR_ARG;
  if (top <= 0 || dim <= 0 || (plus && (ldp < dim || n_plus < 1)) || (n_plus > 1 && plus_dtype != FG_F32)) return FG_ERR_ARG;
  if (plus_dtype == FG_F32)
    moe_combine_kernel<float><<<n_tokens, 256, 0, stream>>>(y, weight, (const float*)plus, ldp, n_plus, (size_t)plus_stride,
                                                            top, dim, out, plus_gate, gate_stride);
  else if (plus_dtype == FG_BF16)
    moe_combine_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>(y, weight, (const bf16_t*)plus, ldp, n_plus,
                                                             (size_t)plus_stride, top, dim, out, plus_gate, gate_stride);
  else
    return FG_ERR_ARG;
  return fg_launch_status();
}

extern "C" int fg_moe_combine(const float* y, const float* weight, const void* plus, int ldp, int plus_dtype, int n_plus,
                              long long plus_stride, int n_tokens, int top, int dim, float* out, hipStream_t stream) {
  return fg_moe_combine_gated(y, weight, plus, ldp, plus_dtype, n_plus, plus_stride, n_tokens, top, dim, out, nullptr, 0,
                              stream);
}
