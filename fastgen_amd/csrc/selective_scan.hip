// A selective state-space recurrence (the mixer of Mamba) and the short causal convolution before it.
//
// Per request and channel c the state is one fp32 row of a state tensor [slots, C, row_len]: the N values of
// the recurrence S[c, 0..N), then (from column `tail_off` = N) the last K - 1 inputs of the convolution.
//
//  causal_conv     y[t, c] = act(b[c] + sum_j taps[c, j] x[t - (K - 1) + j, c]): the last tap meets the token
//                  itself; tokens before this step's first come from the row's tail (zeros for a new request).
//                  A thread a (token, channel).  Reads the tail, does not write it.
//  selective_scan  per token, in order:  d = softplus(dt[t, c] + dt_bias[c]);
//                    S[c, n] <- exp(d A[c, n]) S[c, n] + d u[t, c] B[t, n];   y = sum_n S[c, n] C[t, n] + D[c] u[t, c];
//                    out[t, c] = y * silu(z[t, c]).
//                  A channel is LP lanes (a power of two), a lane holds SPL consecutive states; the sum over
//                  n is an exchange between those lanes.  A workgroup walks one sequence's tokens of this step
//                  (grid.y: the sequence), with the next token's operands in flight while one is computed.
//                  When it is done it stores the state and moves the convolution's tail on by this step's
//                  tokens (`x_raw`: the convolution's input rows), so the next step finds both.
//  Long prompts are scanned in chunks of tokens side by side, in three passes: every chunk from a zero state
//  (no outputs; what it adds to the state and the sum of its step sizes are kept), then the state that every
//  chunk starts from (scan_chunk_states), then every chunk from that state with its outputs.
//
// All arithmetic is fp32; the state never leaves fp32.  What a token gets depends on its sequence's earlier
// tokens alone, in their order: not on the batch and not on how the tokens were cut into steps.
#include "common.h"

#define SS_THREADS 256
#define SS_MAX_TAPS 16

template <class TS, class TA>
__global__ __launch_bounds__(SS_THREADS) void causal_conv_kernel(
    const TS* __restrict__ x, int ldx, const float* __restrict__ taps, const float* __restrict__ bias,
    const float* __restrict__ state, int row_len, int tail_off, const int* __restrict__ slot_ids,
    const int* __restrict__ seq_of_token, const int* __restrict__ q_start, TA* __restrict__ out, int ldo, int C,
    int K, int act) {
  const int c = blockIdx.y * SS_THREADS + threadIdx.x;
  const int t = blockIdx.x;
  if (c >= C) return;
  const int b = seq_of_token[t];
  const int t0 = q_start[b];
  const int i = t - t0;
  const float* tail = state + ((size_t)slot_ids[b] * C + c) * row_len + tail_off;
  float acc = bias ? bias[c] : 0.f;
  for (int j = 0; j < K; ++j) {
    const int idx = i - (K - 1) + j;
    const float v = idx >= 0 ? to_f<TS>(x[(size_t)(t0 + idx) * ldx + c]) : tail[K - 1 + idx];
    acc = fmaf(v, taps[(size_t)c * K + j], acc);
  }
  if (act == 1) acc = acc / (1.f + expf(-acc));
  out[(size_t)t * ldo + c] = from_f<TA>(acc);
}

extern "C" int fg_causal_conv(const void* x, int ldx, const float* taps, const float* bias, const float* state,
                              int row_len, int tail_off, const int* slot_ids, const int* seq_of_token,
                              const int* q_start, void* out, int ldo, int n_tokens, int C, int K, int act,
                              int src_dtype, int act_dtype, hipStream_t stream) {
  if (n_tokens <= 0) return FG_OK;
  if (C <= 0 || K < 1 || K > SS_MAX_TAPS || ldx < C || ldo < C || tail_off < 0 || tail_off + K - 1 > row_len ||
      (C + SS_THREADS - 1) / SS_THREADS > 65535 || act < 0 || act > 1)
    return FG_ERR_ARG;
  dim3 grid(n_tokens, (C + SS_THREADS - 1) / SS_THREADS);
#define GO(TS, TA)                                                                                             \
  causal_conv_kernel<TS, TA><<<grid, SS_THREADS, 0, stream>>>((const TS*)x, ldx, taps, bias, state, row_len,  \
                                                              tail_off, slot_ids, seq_of_token, q_start,       \
                                                              (TA*)out, ldo, C, K, act)
  if (src_dtype == FG_F32 && act_dtype == FG_F32) GO(float, float);
  else if (src_dtype == FG_BF16 && act_dtype == FG_BF16) GO(bf16_t, bf16_t);
  else if (src_dtype == FG_F32 && act_dtype == FG_BF16) GO(float, bf16_t);
  else return FG_ERR_ARG;
#undef GO
#undef GO_OUT
  return fg_launch_status();
}

struct ScanArgs {
  const void* u; int ldu;          // [T, >= C] the convolution's output (activation dtype)
  const void* dt; int lddt;        // [T, >= C] step sizes before bias and softplus (fp32 or activation dtype)
  const float* dt_bias;            // [C] or null
  const float* A;                  // [C, N], negative
  const void* bc; int ldbc, b_col, c_col;  // B[t, n] = bc[t * ldbc + b_col + n], C likewise (activation dtype)
  const float* D;                  // [C] or null
  const void* z; int ldz;          // [T, >= C] gate (activation dtype) or null
  const void* x_raw; int ldx;      // [T, >= C] the convolution's input (activation dtype); null with K == 1
  float* state; int row_len;       // [slots, C, row_len]
  const int* slot_ids; const int* q_start;
  void* out; int ldo;              // [T, >= C] activation dtype
  int C, N, K, LP;
  int write_out, write_state, write_tail;  // what a pass leaves behind (all three: the whole step in one pass)
  float* dsum;                     // [n_seqs, C] or null: the sum of a sequence's step sizes, per channel
};

template <class TA> __device__ __forceinline__ float fast_exp(float x);
template <> __device__ __forceinline__ float fast_exp<float>(float x) { return expf(x); }
// bfloat16 operands: the hardware's exponential (a few ulp of 32-bit)
template <> __device__ __forceinline__ float fast_exp<bf16_t>(float x) { return __expf(x); }
// softplus and the sigmoid of the gate: exact functions for 32-bit operands, the hardware's for bfloat16
template <class TA> __device__ __forceinline__ float softplus_of(float d);
template <> __device__ __forceinline__ float softplus_of<float>(float d) { return d > 20.f ? d : log1pf(expf(d)); }
template <> __device__ __forceinline__ float softplus_of<bf16_t>(float d) { return d > 20.f ? d : __logf(1.f + __expf(d)); }
template <class TA> __device__ __forceinline__ float silu_of(float z);
template <> __device__ __forceinline__ float silu_of<float>(float z) { return z / (1.f + expf(-z)); }
template <> __device__ __forceinline__ float silu_of<bf16_t>(float z) { return z * __builtin_amdgcn_rcpf(1.f + __expf(-z)); }

template <class TA, class TD, int SPL, bool OUT>
__global__ __launch_bounds__(SS_THREADS) void selective_scan_kernel(const ScanArgs a) {
  const int tid = blockIdx.x * SS_THREADS + threadIdx.x;
  const int c = tid / a.LP, g = tid % a.LP;
  const int b = blockIdx.y;
  const bool live = c < a.C;  // lanes of a channel are all live or all not; the exchanges below stay inside a channel
  const int cc = live ? c : a.C - 1;
  const int t0 = a.q_start[b], t1 = a.q_start[b + 1];
  float* row = a.state + ((size_t)a.slot_ids[b] * a.C + cc) * a.row_len;
  const int n0 = g * SPL;
  float S[SPL], An[SPL];
#pragma unroll
  for (int i = 0; i < SPL; ++i) {
    const bool in = n0 + i < a.N;
    S[i] = in ? row[n0 + i] : 0.f;
    An[i] = in ? a.A[(size_t)cc * a.N + n0 + i] : 0.f;
  }
  const float bias = a.dt_bias ? a.dt_bias[cc] : 0.f;
  const float skip = a.D ? a.D[cc] : 0.f;
  const TA* u = (const TA*)a.u + cc;
  const TD* dt = (const TD*)a.dt + cc;
  const TA* z = a.z ? (const TA*)a.z + cc : nullptr;
  const TA* Bp = (const TA*)a.bc + a.b_col + n0;
  const TA* Cp = (const TA*)a.bc + a.c_col + n0;
  TA* out = (TA*)a.out + cc;

  // the operands of token t, loaded one token ahead
  float n_u, n_dt, n_z = 0.f, n_B[SPL], n_C[SPL];
  auto fetch = [&](int t) {
    n_u = to_f<TA>(u[(size_t)t * a.ldu]);
    n_dt = to_f<TD>(dt[(size_t)t * a.lddt]);
    if (z) n_z = to_f<TA>(z[(size_t)t * a.ldz]);
#pragma unroll
    for (int i = 0; i < SPL; ++i) {
      const bool in = n0 + i < a.N;
      n_B[i] = in ? to_f<TA>(Bp[(size_t)t * a.ldbc + i]) : 0.f;
      n_C[i] = in ? to_f<TA>(Cp[(size_t)t * a.ldbc + i]) : 0.f;
    }
  };
  float d_total = 0.f;
  if (t0 < t1) fetch(t0);
  for (int t = t0; t < t1; ++t) {
    const float uv = n_u, zv = n_z;
    float d = n_dt + bias;
    float Bv[SPL], Cv[SPL];
#pragma unroll
    for (int i = 0; i < SPL; ++i) { Bv[i] = n_B[i]; Cv[i] = n_C[i]; }
    if (t + 1 < t1) fetch(t + 1);
    d = softplus_of<TA>(d);
    d_total += d;
    const float du = d * uv;
    float y = 0.f;
#pragma unroll
    for (int i = 0; i < SPL; ++i) {
      S[i] = fast_exp<TA>(d * An[i]) * S[i] + du * Bv[i];
      if (OUT) y = fmaf(S[i], Cv[i], y);
    }
    if (OUT) {
      for (int m = 1; m < a.LP; m <<= 1) y += __shfl_xor(y, m, FG_WAVE);
      if (g == 0 && live) {
        y = fmaf(skip, uv, y);
        if (z) y *= silu_of<TA>(zv);
        out[(size_t)t * a.ldo] = from_f<TA>(y);
      }
    }
  }
  if (!live) return;
  if (a.write_state) {
#pragma unroll
    for (int i = 0; i < SPL; ++i)
      if (n0 + i < a.N) row[n0 + i] = S[i];
  }
  if (a.dsum && g == 0) a.dsum[(size_t)b * a.C + cc] = d_total;
  if (g == 0 && a.K > 1 && a.write_tail) {
    // the convolution's tail: the last K - 1 inputs of the sequence, old ones where this step brought fewer
    float* tail = row + a.N;
    const int L = t1 - t0, keep = a.K - 1;
    float nt[SS_MAX_TAPS - 1];
    const TA* xr = (const TA*)a.x_raw + cc;
#pragma unroll
    for (int j = 0; j < SS_MAX_TAPS - 1; ++j) {
      if (j < keep) {
        const int src = L - keep + j;
        nt[j] = src >= 0 ? to_f<TA>(xr[(size_t)(t0 + src) * a.ldx]) : tail[j + L];
      }
    }
#pragma unroll
    for (int j = 0; j < SS_MAX_TAPS - 1; ++j)
      if (j < keep) tail[j] = nt[j];
  }
}

extern "C" int fg_selective_scan(const ScanArgs* args, int n_seqs, int dt_dtype, int act_dtype, hipStream_t stream) {
  if (n_seqs <= 0) return FG_OK;
  const ScanArgs& a = *args;
  if (a.C <= 0 || a.N <= 0 || a.N > 1024 || a.K < 1 || a.K > SS_MAX_TAPS || a.row_len < a.N + a.K - 1 || !a.u || !a.dt ||
      !a.A || !a.bc || !a.state || !a.out || (a.K > 1 && !a.x_raw) || n_seqs > 65535)
    return FG_ERR_ARG;
  const int spl = a.N <= 256 ? 4 : a.N <= 512 ? 8 : 16;
  if (a.LP < 1 || a.LP > 64 || (a.LP & (a.LP - 1)) || a.LP * spl < a.N) return FG_ERR_ARG;
  const long long threads = (long long)a.C * a.LP;
  dim3 grid((unsigned)((threads + SS_THREADS - 1) / SS_THREADS), n_seqs);
#define GO_OUT(TA, TD, OUT)                                                                          \
  do {                                                                                               \
    if (spl == 4) selective_scan_kernel<TA, TD, 4, OUT><<<grid, SS_THREADS, 0, stream>>>(a);        \
    else if (spl == 8) selective_scan_kernel<TA, TD, 8, OUT><<<grid, SS_THREADS, 0, stream>>>(a);   \
    else selective_scan_kernel<TA, TD, 16, OUT><<<grid, SS_THREADS, 0, stream>>>(a);                \
  } while (0)
#define GO(TA, TD)                                      \
  do {                                                  \
    if (a.write_out) GO_OUT(TA, TD, true);              \
    else GO_OUT(TA, TD, false);                         \
  } while (0)
  if (act_dtype == FG_F32 && dt_dtype == FG_F32) GO(float, float);
  else if (act_dtype == FG_BF16 && dt_dtype == FG_F32) GO(bf16_t, float);
  else if (act_dtype == FG_BF16 && dt_dtype == FG_BF16) GO(bf16_t, bf16_t);
  else return FG_ERR_ARG;
#undef GO
#undef GO_OUT
  return fg_launch_status();
}

// Long runs of tokens, scanned chunk by chunk: after every chunk was scanned from a zero state (its rows of
// `chunks` hold what it adds, `dsum` the sums of its step sizes), the state that each chunk starts from.  Over
// a chunk the decay of S[c, n] is exp(A[c, n] * dsum[c]).  Per sequence b with the chunks seq_chunk[b] ..
// seq_chunk[b+1]-1, in their order:  start_0 = state[slot];  start_{k+1} = exp(A dsum_k) start_k + chunks_k.
// chunks_k becomes start_k, and the state's row what the last chunk leaves.  A thread a (channel, state value).
// The convolution's tail moves on by the sequence's tokens (as the scan does it in one pass).
template <class TA>
__global__ __launch_bounds__(SS_THREADS) void scan_chunk_states_kernel(
    float* __restrict__ chunks, const float* __restrict__ dsum, const float* __restrict__ A, float* __restrict__ state,
    int row_len, const int* __restrict__ slot_ids, const int* __restrict__ seq_chunk, const int* __restrict__ q_start,
    const TA* __restrict__ x_raw, int ldx, int C, int N, int K) {
  const int i = blockIdx.x * SS_THREADS + threadIdx.x;
  if (i >= C * N) return;
  const int c = i / N, n = i % N;
  const int b = blockIdx.y;
  const float An = A[(size_t)c * N + n];
  float* row = state + ((size_t)slot_ids[b] * C + c) * row_len;
  float S = row[n];
  for (int k = seq_chunk[b]; k < seq_chunk[b + 1]; ++k) {
    float* at = chunks + ((size_t)k * C + c) * row_len + n;
    const float add = *at;
    *at = S;
    S = expf(An * dsum[(size_t)k * C + c]) * S + add;
  }
  row[n] = S;
  if (n == 0 && K > 1) {
    float* tail = row + N;
    const int t0 = q_start[b], L = q_start[b + 1] - t0, keep = K - 1;
    float nt[SS_MAX_TAPS - 1];
#pragma unroll
    for (int j = 0; j < SS_MAX_TAPS - 1; ++j) {
      if (j < keep) {
        const int src = L - keep + j;
        nt[j] = src >= 0 ? to_f<TA>(x_raw[(size_t)(t0 + src) * ldx + c]) : tail[j + L];
      }
    }
#pragma unroll
    for (int j = 0; j < SS_MAX_TAPS - 1; ++j)
      if (j < keep) tail[j] = nt[j];
  }
}

extern "C" int fg_scan_chunk_states(float* chunks, const float* dsum, const float* A, float* state, int row_len,
                                    const int* slot_ids, const int* seq_chunk, const int* q_start, const void* x_raw,
                                    int ldx, int n_seqs, int C, int N, int K, int act_dtype, hipStream_t stream) {
  if (n_seqs <= 0) return FG_OK;
  if (C <= 0 || N <= 0 || K < 1 || K > SS_MAX_TAPS || row_len < N + K - 1 || n_seqs > 65535 || (K > 1 && !x_raw) || !chunks ||
      !dsum || !A || !state)
    return FG_ERR_ARG;
  dim3 grid((unsigned)(((long long)C * N + SS_THREADS - 1) / SS_THREADS), n_seqs);
  if (act_dtype == FG_F32)
    scan_chunk_states_kernel<float><<<grid, SS_THREADS, 0, stream>>>(chunks, dsum, A, state, row_len, slot_ids, seq_chunk,
                                                                     q_start, (const float*)x_raw, ldx, C, N, K);
  else if (act_dtype == FG_BF16)
    scan_chunk_states_kernel<bf16_t><<<grid, SS_THREADS, 0, stream>>>(chunks, dsum, A, state, row_len, slot_ids, seq_chunk,
                                                                      q_start, (const bf16_t*)x_raw, ldx, C, N, K);
  else
    return FG_ERR_ARG;
  return fg_launch_status();
}
