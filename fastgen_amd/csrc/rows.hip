// Row-wise kernels: embedding gather, residual add fused with RMSNorm,
// SiLU(gate)*up.  The residual stream is fp32 in both precisions.
//
// Formulas: embedding fastgen/forward.py:406-409; RMSNorm
// fastgen/kernels/rmsnorm.py:33-60 (fp32 sum of squares, rsqrt(mean+eps),
// a*rstd*w left to right, one rounding at the store); SiLU*mul
// fastgen/forward.py:495 (here in fp32 with one rounding).
#include "common.h"

#define ROWS_THREADS 256

// ---------------------------------------------------------------- embedding
template <class TW>
__global__ __launch_bounds__(ROWS_THREADS) void embed_kernel(
    const TW* __restrict__ table, const int* __restrict__ tokens, float* __restrict__ out,
    int dim, int vocab, float scale) {
  const int t = blockIdx.x;
  int tok = tokens[t];
  // ids are validated on the host; the clamp only keeps a bad id from faulting
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  const TW* src = table + (size_t)tok * dim;
  float* dst = out + (size_t)t * dim;
  for (int i = threadIdx.x; i < dim; i += ROWS_THREADS) dst[i] = to_f<TW>(src[i]) * scale;
}

extern "C" int fg_embed(const void* table, int table_dtype, const int* tokens, float* out,
                        int n_tokens, int dim, int vocab, float scale, hipStream_t stream) {
  if (n_tokens <= 0) return FG_OK;
  if (dim <= 0 || vocab <= 0) return FG_ERR_ARG;
  if (table_dtype == FG_F32)
    embed_kernel<float><<<n_tokens, ROWS_THREADS, 0, stream>>>((const float*)table, tokens, out, dim, vocab, scale);
  else if (table_dtype == FG_BF16)
    embed_kernel<bf16_t><<<n_tokens, ROWS_THREADS, 0, stream>>>((const bf16_t*)table, tokens, out, dim, vocab, scale);
  else
    return FG_ERR_ARG;
  return fg_launch_status();
}

// -------------------------------------------------- additions to the stream
// h[t] = ((h[t] + delta[t]) + again[t]) + row, all fp32, in that order: what a layer left to be added
// (rows of the activation dtype, or fp32 partial sums in order), then rows that enter the stream once
// more (the embedding's output), then one vector for all tokens.  Each of the three may be absent.
template <class TA>
__global__ __launch_bounds__(ROWS_THREADS) void stream_add_kernel(
    float* __restrict__ h, const TA* __restrict__ delta, const float* __restrict__ parts, int n_parts,
    size_t part_stride, const float* __restrict__ again, const float* __restrict__ row, int dim) {
  const size_t t = blockIdx.x;
  for (int i = threadIdx.x; i < dim; i += ROWS_THREADS) {
    float v = h[t * dim + i];
    if (delta) v += to_f<TA>(delta[t * dim + i]);
    if (parts)
      for (int p = 0; p < n_parts; ++p) v += parts[p * part_stride + t * dim + i];
    if (again) v += again[t * dim + i];
    if (row) v += row[i];
    h[t * dim + i] = v;
  }
}

extern "C" int fg_stream_add(float* h, const void* delta, int delta_dtype, const float* parts, int n_parts,
                             long long part_stride, const float* again, const float* row, int n_rows, int dim,
                             hipStream_t stream) {
  if (n_rows <= 0) return FG_OK;
  if (dim <= 0 || (parts && n_parts < 1)) return FG_ERR_ARG;
  if (delta_dtype == FG_F32)
    stream_add_kernel<float><<<n_rows, ROWS_THREADS, 0, stream>>>(h, (const float*)delta, parts, n_parts,
                                                                  (size_t)part_stride, again, row, dim);
  else if (delta_dtype == FG_BF16)
    stream_add_kernel<bf16_t><<<n_rows, ROWS_THREADS, 0, stream>>>(h, (const bf16_t*)delta, parts, n_parts,
                                                                   (size_t)part_stride, again, row, dim);
  else
    return FG_ERR_ARG;
  return fg_launch_status();
}

// out[t] = a[t] + b[t] in fp32 (two sublayers' outputs that go to the stream as one sum)
template <class TA>
__global__ __launch_bounds__(ROWS_THREADS) void add_rows_kernel(const TA* __restrict__ a, const TA* __restrict__ b,
                                                                float* __restrict__ out, size_t n) {
  const size_t i = (size_t)blockIdx.x * ROWS_THREADS + threadIdx.x;
  if (i < n) out[i] = to_f<TA>(a[i]) + to_f<TA>(b[i]);
}

extern "C" int fg_add_rows(const void* a, const void* b, float* out, long long n, int dtype, hipStream_t stream) {
  if (n <= 0) return FG_OK;
  const unsigned blocks = (unsigned)((n + ROWS_THREADS - 1) / ROWS_THREADS);
  if (dtype == FG_F32)
    add_rows_kernel<float><<<blocks, ROWS_THREADS, 0, stream>>>((const float*)a, (const float*)b, out, (size_t)n);
  else if (dtype == FG_BF16)
    add_rows_kernel<bf16_t><<<blocks, ROWS_THREADS, 0, stream>>>((const bf16_t*)a, (const bf16_t*)b, out, (size_t)n);
  else
    return FG_ERR_ARG;
  return fg_launch_status();
}

// x[t][i] *= sigmoid(g[t][i]) (or g[t][i] itself when the sigmoid was taken where g was made), fp32
// inside, one rounding.  Rows of x and g have strides of their own (g may be columns of a wider product).
template <class TA>
__global__ __launch_bounds__(ROWS_THREADS) void gate_mul_kernel(TA* __restrict__ x, int ldx, const TA* __restrict__ g,
                                                                int ldg, int width, int sigmoid) {
  const size_t t = blockIdx.y;
  const int i = blockIdx.x * ROWS_THREADS + threadIdx.x;
  if (i >= width) return;
  float gv = to_f<TA>(g[t * ldg + i]);
  if (sigmoid) gv = 1.f / (1.f + expf(-gv));
  x[t * ldx + i] = from_f<TA>(to_f<TA>(x[t * ldx + i]) * gv);
}

extern "C" int fg_gate_mul(void* x, int ldx, const void* g, int ldg, int n_rows, int width, int sigmoid, int dtype,
                           hipStream_t stream) {
  if (n_rows <= 0) return FG_OK;
  if (width <= 0 || ldx < width || ldg < width) return FG_ERR_ARG;
  for (int r0 = 0; r0 < n_rows; r0 += 65535) {
    const int nr = n_rows - r0 < 65535 ? n_rows - r0 : 65535;
    dim3 grid((width + ROWS_THREADS - 1) / ROWS_THREADS, nr);
    if (dtype == FG_F32)
      gate_mul_kernel<float><<<grid, ROWS_THREADS, 0, stream>>>((float*)x + (size_t)r0 * ldx, ldx,
                                                                (const float*)g + (size_t)r0 * ldg, ldg, width, sigmoid);
    else if (dtype == FG_BF16)
      gate_mul_kernel<bf16_t><<<grid, ROWS_THREADS, 0, stream>>>((bf16_t*)x + (size_t)r0 * ldx, ldx,
                                                                 (const bf16_t*)g + (size_t)r0 * ldg, ldg, width, sigmoid);
    else
      return FG_ERR_ARG;
  }
  return fg_launch_status();
}

// ------------------------------------------------------ residual add + norm
// Row r of the output is norm(h[src] (+ delta[src])) * w with src = rows ?
// rows[r] : r.  When delta is given and all rows are normed (rows == null)
// the sum is written back to h, so the residual stream is updated in the pass
// that reads it for the norm; a gathered call leaves h as it is (rows may
// name a row twice).
// What is added to h is either `delta` (rows of the activation dtype) or the sum, in order, of
// `n_parts` fp32 partial results `parts[p]` (a matrix product whose k range was cut).
template <class TA, class TW>
__global__ __launch_bounds__(ROWS_THREADS) void add_rmsnorm_kernel(
    float* __restrict__ h, const TA* __restrict__ delta, const float* __restrict__ parts, int n_parts,
    size_t part_stride, const TW* __restrict__ w, TA* __restrict__ out, const int* __restrict__ rows, int dim,
    float eps) {
  __shared__ float red[16];
  const int r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : (size_t)r;
  float* hrow = h + src * dim;
  const TA* drow = delta ? delta + src * dim : nullptr;
  const bool adds = drow || parts;
  float ss = 0.f;
  for (int i = threadIdx.x; i < dim; i += ROWS_THREADS) {
    float v = hrow[i];
    if (drow) v += to_f<TA>(drow[i]);
    if (parts)
      for (int p = 0; p < n_parts; ++p) v += parts[p * part_stride + src * dim + i];
    if (adds && !rows) hrow[i] = v;
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float rstd = rsqrtf(ss / (float)dim + eps);
  TA* orow = out + (size_t)r * dim;
  for (int i = threadIdx.x; i < dim; i += ROWS_THREADS) {
    // each thread re-reads only what it wrote itself above
    float v = hrow[i];
    if (rows) {
      if (drow) v += to_f<TA>(drow[i]);
      if (parts)
        for (int p = 0; p < n_parts; ++p) v += parts[p * part_stride + src * dim + i];
    }
    orow[i] = from_f<TA>(v * rstd * to_f<TW>(w[i]));
  }
}

// The same with each thread holding its share of the row in registers: 8
// consecutive elements per 256-thread round, all loads of a round issued at
// once.  For dim % 8 == 0 and dim <= 2048 * NIT.
template <class TA, class TW, int NIT>
__global__ __launch_bounds__(ROWS_THREADS) void add_rmsnorm_vec_kernel(
    float* __restrict__ h, const TA* __restrict__ delta, const float* __restrict__ parts, int n_parts,
    size_t part_stride, const TW* __restrict__ w, TA* __restrict__ out, const int* __restrict__ rows, int dim,
    float eps) {
  __shared__ float red[16];
  const int r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : (size_t)r;
  float* hrow = h + src * dim;
  const TA* drow = delta ? delta + src * dim : nullptr;
  // Every load of the row is issued before anything is added (the kernel is a chain of memory
  // round trips: as few of them as possible).  Loads are never conditional: a thread whose share
  // lies beyond the row reads the row's last 8 elements and stores nothing.
  int e[NIT], ec[NIT];
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    e[it] = (threadIdx.x + it * ROWS_THREADS) * 8;
    ec[it] = min(e[it], dim - 8);
  }
  float v[NIT][8], wv[NIT][8];
#pragma unroll
  for (int it = 0; it < NIT; ++it) load8<float>(hrow + ec[it], v[it]);
#pragma unroll
  for (int it = 0; it < NIT; ++it) load8<TW>(w + ec[it], wv[it]);
  if (drow) {
    float d[NIT][8];
#pragma unroll
    for (int it = 0; it < NIT; ++it) load8<TA>(drow + ec[it], d[it]);
#pragma unroll
    for (int it = 0; it < NIT; ++it)
#pragma unroll
      for (int i = 0; i < 8; ++i) v[it][i] += d[it][i];
  }
  if (parts) {
    constexpr int PB = NIT <= 2 ? 8 : 4;  // partial results whose loads are in flight together
    for (int p0 = 0; p0 < n_parts; p0 += PB) {
      float dp[NIT][PB][8];
#pragma unroll
      for (int it = 0; it < NIT; ++it)
#pragma unroll
        for (int p = 0; p < PB; ++p)
          load8<float>(parts + (size_t)min(p0 + p, n_parts - 1) * part_stride + src * dim + ec[it], dp[it][p]);
#pragma unroll
      for (int it = 0; it < NIT; ++it)
#pragma unroll
        for (int p = 0; p < PB; ++p)  // in order of the partial results
#pragma unroll
          for (int i = 0; i < 8; ++i) v[it][i] += p0 + p < n_parts ? dp[it][p][i] : 0.f;
    }
  }
  if ((drow || parts) && !rows) {
#pragma unroll
    for (int it = 0; it < NIT; ++it)
      if (e[it] < dim) store8<float>(hrow + e[it], v[it]);
  }
  float ss = 0.f;
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    if (e[it] < dim) {
#pragma unroll
      for (int i = 0; i < 8; ++i) ss += v[it][i] * v[it][i];
    }
  }
  ss = block_sum(ss, red);
  const float rstd = rsqrtf(ss / (float)dim + eps);
  TA* orow = out + (size_t)r * dim;
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    if (e[it] < dim) {
      float o[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) o[i] = v[it][i] * rstd * wv[it][i];
      store8<TA>(orow + e[it], o);
    }
  }
}

template <class TA, class TW>
static void launch_add_rmsnorm(float* h, const void* delta, const float* parts, int n_parts, size_t part_stride,
                               const void* w, void* out, const int* rows, int n_rows, int dim, float eps,
                               hipStream_t stream) {
#define VEC(NIT)                                                                              \
  add_rmsnorm_vec_kernel<TA, TW, NIT><<<n_rows, ROWS_THREADS, 0, stream>>>(                   \
      h, (const TA*)delta, parts, n_parts, part_stride, (const TW*)w, (TA*)out, rows, dim, eps)
  if (dim % 8 == 0 && dim <= 2048) VEC(1);
  else if (dim % 8 == 0 && dim <= 4096) VEC(2);
  else if (dim % 8 == 0 && dim <= 8192) VEC(4);
  else
    add_rmsnorm_kernel<TA, TW><<<n_rows, ROWS_THREADS, 0, stream>>>(
        h, (const TA*)delta, parts, n_parts, part_stride, (const TW*)w, (TA*)out, rows, dim, eps);
#undef VEC
}

extern "C" int fg_add_rmsnorm(float* h, const void* delta, const float* parts, int n_parts,
                              long long part_stride, const void* w, void* out, const int* rows, int n_rows,
                              int dim, float eps, int act_dtype, int w_dtype, hipStream_t stream) {
  if (n_rows <= 0) return FG_OK;
  if (dim <= 0 || (parts && n_parts < 1)) return FG_ERR_ARG;
#define LAUNCH(TA, TW) \
  launch_add_rmsnorm<TA, TW>(h, delta, parts, n_parts, (size_t)part_stride, w, out, rows, n_rows, dim, eps, stream)
  if (act_dtype == FG_F32 && w_dtype == FG_F32) LAUNCH(float, float);
  else if (act_dtype == FG_BF16 && w_dtype == FG_BF16) LAUNCH(bf16_t, bf16_t);
  else if (act_dtype == FG_BF16 && w_dtype == FG_F32) LAUNCH(bf16_t, float);
  else if (act_dtype == FG_F32 && w_dtype == FG_BF16) LAUNCH(float, bf16_t);
  else return FG_ERR_ARG;
#undef LAUNCH
  return fg_launch_status();
}

// Plain RMSNorm over rows of act dtype (no residual), for norms that sit
// elsewhere than on the residual stream (per head, after a block).
template <class TA, class TW>
__global__ __launch_bounds__(ROWS_THREADS) void rmsnorm_kernel(
    const TA* __restrict__ x, const TW* __restrict__ w, TA* __restrict__ out, int dim,
    float eps) {
  __shared__ float red[16];
  const TA* xrow = x + (size_t)blockIdx.x * dim;
  float ss = 0.f;
  for (int i = threadIdx.x; i < dim; i += ROWS_THREADS) {
    float v = to_f<TA>(xrow[i]);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float rstd = rsqrtf(ss / (float)dim + eps);
  TA* orow = out + (size_t)blockIdx.x * dim;
  for (int i = threadIdx.x; i < dim; i += ROWS_THREADS)
    orow[i] = from_f<TA>(to_f<TA>(xrow[i]) * rstd * to_f<TW>(w[i]));
}

extern "C" int fg_rmsnorm(const void* x, const void* w, void* out, int n_rows, int dim,
                          float eps, int act_dtype, int w_dtype, hipStream_t stream) {
  if (n_rows <= 0) return FG_OK;
  if (dim <= 0) return FG_ERR_ARG;
#define LAUNCH(TA, TW)                                                                       \
  rmsnorm_kernel<TA, TW><<<n_rows, ROWS_THREADS, 0, stream>>>((const TA*)x, (const TW*)w,    \
                                                              (TA*)out, dim, eps)
  if (act_dtype == FG_F32 && w_dtype == FG_F32) LAUNCH(float, float);
  else if (act_dtype == FG_BF16 && w_dtype == FG_BF16) LAUNCH(bf16_t, bf16_t);
  else if (act_dtype == FG_BF16 && w_dtype == FG_F32) LAUNCH(bf16_t, float);
  else if (act_dtype == FG_F32 && w_dtype == FG_BF16) LAUNCH(float, bf16_t);
  else return FG_ERR_ARG;
#undef LAUNCH
  return fg_launch_status();
}

// Rows times rsqrt(sum of the row's partial sums of squares / dim + eps): the second half of a norm
// whose first half (the weight, the sums of squares) was done where the rows were made.
template <class TA>
__global__ __launch_bounds__(ROWS_THREADS) void scale_rows_kernel(
    const TA* __restrict__ x, const float* __restrict__ ssq, TA* __restrict__ out, int width, int n_parts,
    float inv_dim, float eps) {
  __shared__ float red[16];
  const int r = blockIdx.x;
  float ss = 0.f;
  for (int p = threadIdx.x; p < n_parts; p += ROWS_THREADS) ss += ssq[(size_t)r * n_parts + p];
  ss = block_sum(ss, red);
  const float rstd = rsqrtf(ss * inv_dim + eps);
  for (int i = threadIdx.x; i < width; i += ROWS_THREADS)
    out[(size_t)r * width + i] = from_f<TA>(to_f<TA>(x[(size_t)r * width + i]) * rstd);
}

extern "C" int fg_scale_rows(const void* x, const float* ssq, void* out, int n_rows, int width, int n_parts,
                             int dim, float eps, int act_dtype, hipStream_t stream) {
  if (n_rows <= 0) return FG_OK;
  if (width <= 0 || n_parts <= 0 || dim <= 0 || !(eps >= 0.f)) return FG_ERR_ARG;
  if (act_dtype == FG_F32)
    scale_rows_kernel<float><<<n_rows, ROWS_THREADS, 0, stream>>>((const float*)x, ssq, (float*)out, width, n_parts,
                                                                  1.f / (float)dim, eps);
  else if (act_dtype == FG_BF16)
    scale_rows_kernel<bf16_t><<<n_rows, ROWS_THREADS, 0, stream>>>((const bf16_t*)x, ssq, (bf16_t*)out, width,
                                                                   n_parts, 1.f / (float)dim, eps);
  else
    return FG_ERR_ARG;
  return fg_launch_status();
}

// ------------------------------------------------------------- SiLU(g) * u
// gu is [n_rows, 2*hidden] with gate and up columns interleaved in groups of
// 8: columns 16k .. 16k+7 are gate 8k .. 8k+7, columns 16k+8 .. 16k+15 their up
// values (the row order in which the gate/up matrix is kept, so that one tile
// of a matrix product holds both).  hidden % 8 == 0.
// eight elements a thread, for hidden % 8 == 0
template <class TA>
__global__ __launch_bounds__(ROWS_THREADS) void silu_mul_vec_kernel(
    const TA* __restrict__ gu, TA* __restrict__ out, int hidden) {
  const TA* row = gu + (size_t)blockIdx.y * 2 * hidden;
  TA* o = out + (size_t)blockIdx.y * hidden;
  const int e = (blockIdx.x * ROWS_THREADS + threadIdx.x) * 8;
  if (e < hidden) {
    float gv[8], uv[8], r[8];
    load8<TA>(row + 2 * e, gv);
    load8<TA>(row + 2 * e + 8, uv);
    // bfloat16 results take the hardware's exponential and reciprocal (a few ulp of 32-bit, far below the
    // rounding of the result; the precise ones are most of this kernel's instructions); float32 stays exact
#pragma unroll
    for (int i = 0; i < 8; ++i)
      r[i] = sizeof(TA) == 2 ? gv[i] * __frcp_rn(1.f + __expf(-gv[i])) * uv[i] : gv[i] / (1.f + expf(-gv[i])) * uv[i];
    store8<TA>(o + e, r);
  }
}

extern "C" int fg_silu_mul(const void* gu, void* out, int n_rows, int hidden, int act_dtype,
                           hipStream_t stream) {
  if (n_rows <= 0) return FG_OK;
  if (hidden <= 0 || hidden % 8 || n_rows > 65535 * 32) return FG_ERR_ARG;
  // blockIdx.y is limited to 65535: rows beyond that go to further launches
  for (int r0 = 0; r0 < n_rows; r0 += 65535) {
    const int nr = n_rows - r0 < 65535 ? n_rows - r0 : 65535;
    const int per_block = ROWS_THREADS * 8;  // (hidden % 8 == 0 is what the interleaved layout asks for anyway)
    dim3 grid((hidden + per_block - 1) / per_block, nr);
    if (act_dtype == FG_F32) {
      const float* g = (const float*)gu + (size_t)r0 * 2 * hidden;
      float* o = (float*)out + (size_t)r0 * hidden;
      silu_mul_vec_kernel<float><<<grid, ROWS_THREADS, 0, stream>>>(g, o, hidden);
    } else if (act_dtype == FG_BF16) {
      const bf16_t* g = (const bf16_t*)gu + (size_t)r0 * 2 * hidden;
      bf16_t* o = (bf16_t*)out + (size_t)r0 * hidden;
      silu_mul_vec_kernel<bf16_t><<<grid, ROWS_THREADS, 0, stream>>>(g, o, hidden);
    } else {
      return FG_ERR_ARG;
    }
  }
  return fg_launch_status();
}

// ------------------------------------------- a sublayer's output, normed, then added
// The sublayer's output d (rows of the activation dtype, or fp32 partial sums added in order) is
// RMS-normed with the weight wp, the result is added to the fp32 stream, and, if `w` is given, the
// stream's row is normed with `w` into `out`:
//   h += d * rsqrt(mean(d^2) + eps_p) * wp ;  out = h * rsqrt(mean(h^2) + eps) * w
// all in fp32 with one rounding at the store of `out`.  With `rows` only the gathered rows are
// computed and h is left as it was.  A thread keeps its elements i = tid, tid + 256, .. in registers.
// `dbias` (fp32 per column, or null) is added to d before its norm (a projection's bias).  Without `w` but
// with `out` the stream's row itself is stored, rounded to the activation dtype: what a sublayer reads
// that takes the stream un-normed.  Without delta and parts nothing is added.
#define POST_MAX_PER_THREAD 64  // rows of up to 16,384 elements
template <class TA, class TW, int NIT>
__global__ __launch_bounds__(ROWS_THREADS) void post_add_rmsnorm_kernel(
    float* __restrict__ h, const TA* __restrict__ delta, const float* __restrict__ parts, int n_parts,
    size_t part_stride, const TW* __restrict__ wp, float eps_p, const TW* __restrict__ w, TA* __restrict__ out,
    const int* __restrict__ rows, int dim, float eps, const float* __restrict__ dbias) {
  __shared__ float red[16];
  const int r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : (size_t)r;
  float* hrow = h + src * dim;
  float d[NIT];
  float ss = 0.f;
  const bool adds = delta || parts;  // uniform
#pragma unroll
  for (int j = 0; j < NIT; ++j) {
    const int i = threadIdx.x + j * ROWS_THREADS;
    if (i >= dim) continue;
    float v = 0.f;
    if (delta) v = to_f<TA>(delta[src * dim + i]);
    if (parts)
      for (int p = 0; p < n_parts; ++p) v += parts[p * part_stride + src * dim + i];
    if (dbias && adds) v += dbias[i];
    d[j] = v;
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float rstd_p = rsqrtf(ss / (float)dim + eps_p);
  float s2 = 0.f;
#pragma unroll
  for (int j = 0; j < NIT; ++j) {
    const int i = threadIdx.x + j * ROWS_THREADS;
    if (i >= dim) continue;
    const float v = adds ? hrow[i] + d[j] * rstd_p * to_f<TW>(wp[i]) : hrow[i];
    if (!rows && adds) hrow[i] = v;
    d[j] = v;
    s2 += v * v;
  }
  if (!out) return;  // uniform
  float rstd = 1.f;
  if (w) {  // uniform
    s2 = block_sum(s2, red);
    rstd = rsqrtf(s2 / (float)dim + eps);
  }
  TA* orow = out + (size_t)r * dim;
#pragma unroll
  for (int j = 0; j < NIT; ++j) {
    const int i = threadIdx.x + j * ROWS_THREADS;
    if (i >= dim) continue;
    orow[i] = from_f<TA>(w ? d[j] * rstd * to_f<TW>(w[i]) : d[j]);
  }
}

extern "C" int fg_post_add_rmsnorm(float* h, const void* delta, const float* parts, int n_parts,
                                   long long part_stride, const void* wp, float eps_p, const void* w, void* out,
                                   const int* rows, int n_rows, int dim, float eps, int act_dtype, int w_dtype,
                                   const float* dbias, hipStream_t stream) {
  if (n_rows <= 0) return FG_OK;
  if (dim <= 0 || dim > POST_MAX_PER_THREAD * ROWS_THREADS || (parts && n_parts < 1) || (w && !out) ||
      ((delta || parts) && !wp) || (!delta && !parts && !out))
    return FG_ERR_ARG;
#define GO(TA, TW, NIT)                                                                                       \
  post_add_rmsnorm_kernel<TA, TW, NIT><<<n_rows, ROWS_THREADS, 0, stream>>>(                                  \
      h, (const TA*)delta, parts, n_parts, (size_t)part_stride, (const TW*)wp, eps_p, (const TW*)w, (TA*)out, \
      rows, dim, eps, dbias)
#define LAUNCH(TA, TW)                                 \
  do {                                                 \
    if (dim <= 4 * ROWS_THREADS) GO(TA, TW, 4);        \
    else if (dim <= 16 * ROWS_THREADS) GO(TA, TW, 16); \
    else GO(TA, TW, POST_MAX_PER_THREAD);              \
  } while (0)
  if (act_dtype == FG_F32 && w_dtype == FG_F32) LAUNCH(float, float);
  else if (act_dtype == FG_BF16 && w_dtype == FG_BF16) LAUNCH(bf16_t, bf16_t);
  else if (act_dtype == FG_BF16 && w_dtype == FG_F32) LAUNCH(bf16_t, float);
  else if (act_dtype == FG_F32 && w_dtype == FG_BF16) LAUNCH(float, bf16_t);
  else return FG_ERR_ARG;
#undef LAUNCH
#undef GO
  return fg_launch_status();
}

// ------------------------------------------------------ gelu_tanh(g) * u
// As silu_mul_vec_kernel, with the tanh form of GELU: 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3))).
template <class TA>
__global__ __launch_bounds__(ROWS_THREADS) void gelu_mul_vec_kernel(
    const TA* __restrict__ gu, TA* __restrict__ out, int hidden) {
  const TA* row = gu + (size_t)blockIdx.y * 2 * hidden;
  TA* o = out + (size_t)blockIdx.y * hidden;
  const int e = (blockIdx.x * ROWS_THREADS + threadIdx.x) * 8;
  if (e < hidden) {
    float gv[8], uv[8], r[8];
    load8<TA>(row + 2 * e, gv);
    load8<TA>(row + 2 * e + 8, uv);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float g = gv[i];
      r[i] = 0.5f * g * (1.f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g))) * uv[i];
    }
    store8<TA>(o + e, r);
  }
}

extern "C" int fg_gelu_mul(const void* gu, void* out, int n_rows, int hidden, int act_dtype,
                           hipStream_t stream) {
  if (n_rows <= 0) return FG_OK;
  if (hidden <= 0 || hidden % 8 || n_rows > 65535 * 32) return FG_ERR_ARG;
  for (int r0 = 0; r0 < n_rows; r0 += 65535) {
    const int nr = n_rows - r0 < 65535 ? n_rows - r0 : 65535;
    const int per_block = ROWS_THREADS * 8;
    dim3 grid((hidden + per_block - 1) / per_block, nr);
    if (act_dtype == FG_F32)
      gelu_mul_vec_kernel<float><<<grid, ROWS_THREADS, 0, stream>>>((const float*)gu + (size_t)r0 * 2 * hidden,
                                                                    (float*)out + (size_t)r0 * hidden, hidden);
    else if (act_dtype == FG_BF16)
      gelu_mul_vec_kernel<bf16_t><<<grid, ROWS_THREADS, 0, stream>>>((const bf16_t*)gu + (size_t)r0 * 2 * hidden,
                                                                     (bf16_t*)out + (size_t)r0 * hidden, hidden);
    else
      return FG_ERR_ARG;
  }
  return fg_launch_status();
}

// ------------------------------------------- act(g + b) * (u + b), any source dtype
// The general form of the two kernels above: the rows may be fp32 (a product's un-rounded result) while
// the result has the activation dtype, a bias per column of gu (fp32, in gu's interleaved order) is added
// first, and the activation is SiLU (0), the tanh form of GELU (1) or ReLU (2), or (3) both halves are limited
// first and the result is g * sigmoid(alpha g) * (u + 1) (GatedAct in common.h).  All of it in fp32.
template <class TS, class TA>
__global__ __launch_bounds__(ROWS_THREADS) void gated_mul_kernel(
    const TS* __restrict__ gu, const float* __restrict__ bias, TA* __restrict__ out, int hidden, int act,
    const GatedAct fn) {
  const TS* row = gu + (size_t)blockIdx.y * 2 * hidden;
  TA* o = out + (size_t)blockIdx.y * hidden;
  const int e = (blockIdx.x * ROWS_THREADS + threadIdx.x) * 8;
  if (e < hidden) {
    float gv[8], uv[8], r[8];
    load8<TS>(row + 2 * e, gv);
    load8<TS>(row + 2 * e + 8, uv);
    if (bias) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        gv[i] += bias[2 * e + i];
        uv[i] += bias[2 * e + 8 + i];
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float g = gv[i];
      if (act == FG_ACT_LIMITED) {
        r[i] = gated_act<false>(g, uv[i], fn);
        continue;
      }
      float a;
      if (act == 0) a = g / (1.f + expf(-g));
      else if (act == 1) a = 0.5f * g * (1.f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
      else a = fmaxf(g, 0.f);
      r[i] = a * uv[i];
    }
    store8<TA>(o + e, r);
  }
}

extern "C" int fg_gated_mul_act(const void* gu, const float* bias, void* out, int n_rows, int hidden, int act,
                                float limit, float alpha, int src_dtype, int act_dtype, hipStream_t stream) {
  if (n_rows <= 0) return FG_OK;
  if (hidden <= 0 || hidden % 8 || n_rows > 65535 * 32 || act < 0 || act > 3 || (act == 3 && !(limit > 0.f)))
    return FG_ERR_ARG;
  const GatedAct fn = {act, limit, alpha};
  for (int r0 = 0; r0 < n_rows; r0 += 65535) {
    const int nr = n_rows - r0 < 65535 ? n_rows - r0 : 65535;
    const int per_block = ROWS_THREADS * 8;
    dim3 grid((hidden + per_block - 1) / per_block, nr);
    const size_t so = (size_t)r0 * 2 * hidden, oo = (size_t)r0 * hidden;
    if (src_dtype == FG_F32 && act_dtype == FG_F32)
      gated_mul_kernel<float, float><<<grid, ROWS_THREADS, 0, stream>>>((const float*)gu + so, bias, (float*)out + oo, hidden, act, fn);
    else if (src_dtype == FG_F32 && act_dtype == FG_BF16)
      gated_mul_kernel<float, bf16_t><<<grid, ROWS_THREADS, 0, stream>>>((const float*)gu + so, bias, (bf16_t*)out + oo, hidden, act, fn);
    else if (src_dtype == FG_BF16 && act_dtype == FG_BF16)
      gated_mul_kernel<bf16_t, bf16_t><<<grid, ROWS_THREADS, 0, stream>>>((const bf16_t*)gu + so, bias, (bf16_t*)out + oo, hidden, act, fn);
    else
      return FG_ERR_ARG;
  }
  return fg_launch_status();
}

extern "C" int fg_gated_mul(const void* gu, const float* bias, void* out, int n_rows, int hidden, int act,
                            int src_dtype, int act_dtype, hipStream_t stream) {
  if (act < 0 || act > 2) return FG_ERR_ARG;
  return fg_gated_mul_act(gu, bias, out, n_rows, hidden, act, 0.f, 1.f, src_dtype, act_dtype, stream);
}

// ------------------------------------------------------------- soft cap
// x = cap * tanh(x / cap) in place on fp32 (logits).
__global__ __launch_bounds__(ROWS_THREADS) void softcap_kernel(float* __restrict__ x, size_t n, float cap) {
  const size_t i = (size_t)blockIdx.x * ROWS_THREADS + threadIdx.x;
  if (i < n) x[i] = cap * tanhf(x[i] / cap);
}

extern "C" int fg_softcap(float* x, long long n, float cap, hipStream_t stream) {
  if (n <= 0) return FG_OK;
  if (!(cap > 0.f) || (n + ROWS_THREADS - 1) / ROWS_THREADS > 2147483647LL) return FG_ERR_ARG;
  softcap_kernel<<<(unsigned)((n + ROWS_THREADS - 1) / ROWS_THREADS), ROWS_THREADS, 0, stream>>>(x, (size_t)n, cap);
  return fg_launch_status();
}

// x *= factor in place on fp32 (logits that a model multiplies by a constant).
__global__ __launch_bounds__(ROWS_THREADS) void scale_kernel(float* __restrict__ x, size_t n, float factor) {
  const size_t i = (size_t)blockIdx.x * ROWS_THREADS + threadIdx.x;
  if (i < n) x[i] *= factor;
}

extern "C" int fg_scale(float* x, long long n, float factor, hipStream_t stream) {
  if (n <= 0) return FG_OK;
  if ((n + ROWS_THREADS - 1) / ROWS_THREADS > 2147483647LL) return FG_ERR_ARG;
  scale_kernel<<<(unsigned)((n + ROWS_THREADS - 1) / ROWS_THREADS), ROWS_THREADS, 0, stream>>>(x, (size_t)n, factor);
  return fg_launch_status();
}
