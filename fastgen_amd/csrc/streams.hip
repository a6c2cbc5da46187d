// Several residual streams side by side (hyper-connections).
//
// The model keeps S copies X[0..S-1] of the residual stream, fp32 [S, T, dim].  A sublayer reads one
// weighted sum of them, u = sum_s a[s] X[s], normed, and its output y goes back into all of them at
// once, together with a mixing of the streams among themselves:
//
//   X'[t] = sum_s M[s][t] X[s] + b[t] y        (M is indexed [from][to])
//
// As the single-stream engine leaves the addition of a sublayer's output to the norm that follows, so
// here one kernel applies the update of the sublayer before (M, b, y: "pending"), stores the new
// streams, forms the next sublayer's u from them and norms it; nothing is rounded in between.  The
// last norm of the model is the same kernel with a = 1 (the sum of the streams).  A workgroup a
// token; a thread takes the elements tid, tid + 256, ... of the row and keeps its u values in
// registers between the two passes.
#include "common.h"

#define ST_THREADS 256
#define ST_MAX_STREAMS 8
#define ST_MAX_PER_THREAD 32  // rows of up to 8,192 elements

struct StreamArgs {
  float* x;               // [S, T, dim], updated in place (unless rows are gathered)
  const void* delta;      // the pending sublayer output: rows of the activation dtype, or null
  const float* parts;     // or fp32 partial sums [n_parts][T, dim], added in order
  int n_parts;
  long long part_stride;
  const float* mix;       // pending: [S, S] from-by-to; null: no update is pending
  const float* out_w;     // pending: [S]
  const float* in_w;      // [S] the weights of the sum that is read; null: all one
  const void* norm_w;     // [dim]; null: u is not normed
  void* out;              // [n_rows, dim] of the activation dtype: norm(u) * norm_w; or null
  float* u_out;           // [n_rows, dim] fp32: u itself; or null
  const int* rows;        // gather: only these tokens, X is left as it is; or null
  int n_streams, n_tokens, dim;
  float eps;
};

template <class TA, class TW, int NPT /* elements of the row a thread holds */>
__global__ __launch_bounds__(ST_THREADS) void streams_step_kernel(const StreamArgs a) {
  __shared__ float red[16];
  __shared__ float mix_s[ST_MAX_STREAMS * ST_MAX_STREAMS], out_s[ST_MAX_STREAMS], in_s[ST_MAX_STREAMS];
  const int S = a.n_streams, dim = a.dim;
  const size_t tok = a.rows ? (size_t)a.rows[blockIdx.x] : (size_t)blockIdx.x;
  const size_t stream_stride = (size_t)a.n_tokens * dim;
  if (threadIdx.x < S * S) mix_s[threadIdx.x] = a.mix ? a.mix[threadIdx.x] : 0.f;
  if (threadIdx.x < S) {
    out_s[threadIdx.x] = a.mix ? a.out_w[threadIdx.x] : 0.f;
    in_s[threadIdx.x] = a.in_w ? a.in_w[threadIdx.x] : 1.f;
  }
  __syncthreads();
  const bool pending = a.mix != nullptr;
  const TA* drow = a.delta ? (const TA*)a.delta + tok * dim : nullptr;
  float u[NPT];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < NPT; ++k) {
    const int i = threadIdx.x + k * ST_THREADS;
    u[k] = 0.f;
    if (i < dim) {
      float xs[ST_MAX_STREAMS];
#pragma unroll
      for (int s = 0; s < ST_MAX_STREAMS; ++s) xs[s] = s < S ? a.x[s * stream_stride + tok * dim + i] : 0.f;
      float acc = 0.f;
      if (pending) {
        float y = drow ? to_f<TA>(drow[i]) : 0.f;
        if (a.parts) {
          y = a.parts[tok * dim + i];
          for (int p = 1; p < a.n_parts; ++p) y += a.parts[p * a.part_stride + tok * dim + i];
        }
#pragma unroll
        for (int t = 0; t < ST_MAX_STREAMS; ++t) {
          if (t < S) {
            float v = 0.f;
#pragma unroll
            for (int s = 0; s < ST_MAX_STREAMS; ++s)
              if (s < S) v = fmaf(mix_s[s * S + t], xs[s], v);
            v = fmaf(out_s[t], y, v);
            if (!a.rows) a.x[t * stream_stride + tok * dim + i] = v;
            acc = fmaf(in_s[t], v, acc);
          }
        }
      } else {
#pragma unroll
        for (int s = 0; s < ST_MAX_STREAMS; ++s)
          if (s < S) acc = fmaf(in_s[s], xs[s], acc);
      }
      u[k] = acc;
      ss += acc * acc;
    }
  }
  float rstd = 1.f;
  if (a.norm_w) {
    ss = block_sum(ss, red);
    rstd = rsqrtf(ss / (float)dim + a.eps);
  }
  const size_t orow = (size_t)blockIdx.x * dim;
#pragma unroll
  for (int k = 0; k < NPT; ++k) {
    const int i = threadIdx.x + k * ST_THREADS;
    if (i < dim) {
      if (a.u_out) a.u_out[orow + i] = u[k];
      if (a.out) ((TA*)a.out)[orow + i] = from_f<TA>(a.norm_w ? u[k] * rstd * to_f<TW>(((const TW*)a.norm_w)[i]) : u[k]);
    }
  }
}

// n_rows: the rows of out / u_out: the tokens named by `rows`, or all n_tokens.
extern "C" int fg_streams_step_rows(const StreamArgs* args, int n_rows, int act_dtype, int w_dtype, hipStream_t stream) {
  const StreamArgs a = *args;
  if (a.n_tokens <= 0 || n_rows <= 0) return FG_OK;
  if (!a.x || a.n_streams < 1 || a.n_streams > ST_MAX_STREAMS || a.dim <= 0 || a.dim > ST_THREADS * ST_MAX_PER_THREAD)
    return FG_ERR_ARG;
  if (a.mix && (!a.out_w || (!a.delta && !a.parts) || (a.parts && a.n_parts < 1))) return FG_ERR_ARG;
  if (!a.mix && (a.delta || a.parts)) return FG_ERR_ARG;
  if (!a.out && !a.u_out && !a.mix) return FG_ERR_ARG;
  if (!a.rows && n_rows != a.n_tokens) return FG_ERR_ARG;
#define GO(TA, TW)                                                                               \
  do {                                                                                           \
    if (a.dim <= 2 * ST_THREADS) streams_step_kernel<TA, TW, 2><<<n_rows, ST_THREADS, 0, stream>>>(a);       \
    else if (a.dim <= 8 * ST_THREADS) streams_step_kernel<TA, TW, 8><<<n_rows, ST_THREADS, 0, stream>>>(a);  \
    else streams_step_kernel<TA, TW, ST_MAX_PER_THREAD><<<n_rows, ST_THREADS, 0, stream>>>(a);   \
  } while (0)
  if (act_dtype == FG_F32 && w_dtype == FG_F32) GO(float, float);
  else if (act_dtype == FG_BF16 && w_dtype == FG_BF16) GO(bf16_t, bf16_t);
  else if (act_dtype == FG_BF16 && w_dtype == FG_F32) GO(bf16_t, float);
  else if (act_dtype == FG_F32 && w_dtype == FG_BF16) GO(float, bf16_t);
  else return FG_ERR_ARG;
#undef GO
  return fg_launch_status();
}

// x[s][t] = h[t] for every stream s: the embedding's output copied into the S streams.
__global__ __launch_bounds__(ST_THREADS) void streams_spread_kernel(const float* __restrict__ h, float* __restrict__ x,
                                                                    size_t n, int n_streams) {
  const size_t i = (size_t)blockIdx.x * ST_THREADS + threadIdx.x;
  if (i >= n) return;
  const float v = h[i];
  for (int s = 0; s < n_streams; ++s) x[s * n + i] = v;
}

extern "C" int fg_streams_spread(const float* h, float* x, long long n, int n_streams, hipStream_t stream) {
  if (n <= 0) return FG_OK;
  if (n_streams < 1 || (n + ST_THREADS - 1) / ST_THREADS > 2147483647LL) return FG_ERR_ARG;
  streams_spread_kernel<<<(unsigned)((n + ST_THREADS - 1) / ST_THREADS), ST_THREADS, 0, stream>>>(h, x, (size_t)n, n_streams);
  return fg_launch_status();
}
