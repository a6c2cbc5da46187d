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
#define ST_MAX_STREAMS 16
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

// The same with a thread holding NV runs of four consecutive elements, for dim % 4 == 0, dim <= 1024 NV and at most
// SM streams: every load of the row (the streams, the update's rows, the norm's weight) is issued before anything
// is computed or stored (the streams are read and written through one pointer, so the compiler would otherwise
// keep a store of one run ahead of the next run's loads: a chain of memory round trips); the small weights are
// read at uniform addresses.  Loads are never conditional: a thread whose run lies beyond the row reads the
// row's last four elements and stores nothing.
template <class T> __device__ __forceinline__ float4 load4(const T* p);
template <> __device__ __forceinline__ float4 load4<float>(const float* p) { return *(const float4*)p; }
template <> __device__ __forceinline__ float4 load4<bf16_t>(const bf16_t* p) {
  const uint2 raw = *(const uint2*)p;
  return make_float4(__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u), __uint_as_float(raw.y << 16),
                     __uint_as_float(raw.y & 0xffff0000u));
}
template <class T> __device__ __forceinline__ void store4(T* p, float4 v);
template <> __device__ __forceinline__ void store4<float>(float* p, float4 v) { *(float4*)p = v; }
template <> __device__ __forceinline__ void store4<bf16_t>(bf16_t* p, float4 v) {
  typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
  bf16x4_t o;
  o[0] = (__bf16)v.x; o[1] = (__bf16)v.y; o[2] = (__bf16)v.z; o[3] = (__bf16)v.w;
  *(bf16x4_t*)p = o;
}
__device__ __forceinline__ float4 fma4(float w, float4 x, float4 acc) {
  return make_float4(fmaf(w, x.x, acc.x), fmaf(w, x.y, acc.y), fmaf(w, x.z, acc.z), fmaf(w, x.w, acc.w));
}

template <class TA, class TW, int NV, int SM>
__global__ __launch_bounds__(ST_THREADS) void streams_step_vec_kernel(const StreamArgs a) {
  __shared__ float red[16];
  const int S = a.n_streams, dim = a.dim;
  const size_t tok = a.rows ? (size_t)a.rows[blockIdx.x] : (size_t)blockIdx.x;
  const size_t stream_stride = (size_t)a.n_tokens * dim;
  const bool pending = a.mix != nullptr;
  int e[NV], ec[NV];
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    e[v] = (threadIdx.x + v * ST_THREADS) * 4;
    ec[v] = min(e[v], dim - 4);
  }
  // the small weights first, at uniform addresses (held in scalar registers); what lies beyond S is never used
  float mixr[SM][SM], outr[SM], inr[SM];
#pragma unroll
  for (int s = 0; s < SM; ++s) {
    outr[s] = pending && s < S ? a.out_w[s] : 0.f;
    inr[s] = a.in_w && s < S ? a.in_w[s] : 1.f;
#pragma unroll
    for (int t = 0; t < SM; ++t) mixr[s][t] = pending && s < S && t < S ? a.mix[s * S + t] : 0.f;
  }
  float4 xs[NV][SM], y[NV], w[NV];
#pragma unroll
  for (int v = 0; v < NV; ++v)
#pragma unroll
    for (int s = 0; s < SM; ++s) xs[v][s] = load4<float>(a.x + min(s, S - 1) * stream_stride + tok * dim + ec[v]);
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    y[v] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (a.delta) y[v] = load4<TA>((const TA*)a.delta + tok * dim + ec[v]);
    if (a.norm_w) w[v] = load4<TW>((const TW*)a.norm_w + ec[v]);
  }
  if (a.parts) {
    for (int p = 0; p < a.n_parts; ++p) {
#pragma unroll
      for (int v = 0; v < NV; ++v) {
        const float4 d = load4<float>(a.parts + p * a.part_stride + tok * dim + ec[v]);
        y[v] = p == 0 ? d : make_float4(y[v].x + d.x, y[v].y + d.y, y[v].z + d.z, y[v].w + d.w);
      }
    }
  }
  float4 u[NV];
  float ss = 0.f;
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    if (pending) {
#pragma unroll
      for (int t = 0; t < SM; ++t) {
        if (t < S) {
          float4 nv = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
          for (int s = 0; s < SM; ++s)
            if (s < S) nv = fma4(mixr[s][t], xs[v][s], nv);
          nv = fma4(outr[t], y[v], nv);
          if (!a.rows && e[v] < dim) store4<float>(a.x + t * stream_stride + tok * dim + e[v], nv);
          acc = fma4(inr[t], nv, acc);
        }
      }
    } else {
#pragma unroll
      for (int s = 0; s < SM; ++s)
        if (s < S) acc = fma4(inr[s], xs[v][s], acc);
    }
    u[v] = acc;
    if (e[v] < dim) ss += acc.x * acc.x + acc.y * acc.y + acc.z * acc.z + acc.w * acc.w;
  }
  float rstd = 1.f;
  if (a.norm_w) {
    ss = block_sum(ss, red);
    rstd = rsqrtf(ss / (float)dim + a.eps);
  }
  const size_t orow = (size_t)blockIdx.x * dim;
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    if (e[v] >= dim) continue;
    if (a.u_out) store4<float>(a.u_out + orow + e[v], u[v]);
    if (a.out) {
      const float4 n = a.norm_w ? make_float4(u[v].x * rstd * w[v].x, u[v].y * rstd * w[v].y, u[v].z * rstd * w[v].z,
                                              u[v].w * rstd * w[v].w)
                                : u[v];
      store4<TA>((TA*)a.out + orow + e[v], n);
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
  const int S = a.n_streams;
#define VEC(TA, TW, NV, SM) streams_step_vec_kernel<TA, TW, NV, SM><<<n_rows, ST_THREADS, 0, stream>>>(a)
#define GO(TA, TW)                                                                               \
  do {                                                                                           \
    if (a.dim % 4 == 0 && a.dim <= 1024 && S <= 4) VEC(TA, TW, 1, 4);                            \
    else if (a.dim % 4 == 0 && a.dim <= 1024 && S <= 8) VEC(TA, TW, 1, 8);                            \
    else if (a.dim % 4 == 0 && a.dim <= 2048 && S <= 4) VEC(TA, TW, 2, 4);                       \
    else if (a.dim % 4 == 0 && a.dim <= 2048 && S <= 8) VEC(TA, TW, 2, 8);                            \
    else if (a.dim % 4 == 0 && a.dim <= 4096 && S <= 4) VEC(TA, TW, 4, 4);                       \
    else if (a.dim <= 2 * ST_THREADS) streams_step_kernel<TA, TW, 2><<<n_rows, ST_THREADS, 0, stream>>>(a);  \
    else if (a.dim <= 8 * ST_THREADS) streams_step_kernel<TA, TW, 8><<<n_rows, ST_THREADS, 0, stream>>>(a);  \
    else streams_step_kernel<TA, TW, ST_MAX_PER_THREAD><<<n_rows, ST_THREADS, 0, stream>>>(a);   \
  } while (0)
  if (act_dtype == FG_F32 && w_dtype == FG_F32) GO(float, float);
  else if (act_dtype == FG_BF16 && w_dtype == FG_BF16) GO(bf16_t, bf16_t);
  else if (act_dtype == FG_BF16 && w_dtype == FG_F32) GO(bf16_t, float);
  else if (act_dtype == FG_F32 && w_dtype == FG_BF16) GO(float, bf16_t);
  else return FG_ERR_ARG;
#undef GO
#undef VEC
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
