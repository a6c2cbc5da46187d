// Per-head work around an attention or a recurrence that is no plain matrix product:
//
//  heads_prepare   what lies between the product that makes queries, keys and values and the
//                  attention: a bias, an RMS norm per head (over the head's first dimensions),
//                  the rotation of a run of dimensions, the queries to a buffer of their own (heads
//                  padded with zeros to the cache's head size) and keys and values into their cache
//                  pages.  A value is either columns of its own or the first dimensions of its
//                  processed key (a latent that serves as key and as value).
//  head_linear     y[t, h, :] = W_h x[t, h, :] with a matrix per head, an optional sigmoid gate per
//                  (token, head), and a run of x's columns behind the product's copied through.
//  head_norm_gate  RMS norm per head of fp32 rows times silu(gate).
//  head_diff_norm  the difference of two attention maps' outputs per head, divided by its root mean square.
//
// All arithmetic between a load and a store is fp32; a result is rounded once, at the store.
#include "common.h"
#include "kv_layout.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define HP_WAVES 4
#define HP_MAX_PAIRS 8  // pairs a lane holds: heads of up to 1,024 elements

struct PrepareArgs {
  const void* src; int src_stride;   // rows [T, src_stride]
  const float* bias;                 // per source column, or null
  int n_q, q_col, q_w, q_norm_dims; const float* q_norm_w;
  void* q_out; int q_out_stride, q_out_hw;  // queries: [T, q_out_stride], head h at h * q_out_hw, zeros behind q_w
  int n_kv, k_col, k_w, k_norm_dims; const float* k_norm_w;
  int v_col, v_w;                    // v_col < 0: a value is the first v_w elements of its processed key
  const float* table;                // [T, rotary_dim / 2, 2] cos, sin; null: nothing is rotated
  int rot_start, rotary_dim;         // pairs (rot_start + 2i, rot_start + 2i + 1) turn
  int rot_q, rot_k;                  // whether the query heads turn, and the key heads
  float eps;
  const int* slots; void* k_pages; void* v_pages; int page_size, hd_c;  // hd_c: the cache's head size
  int norm_plain;                    // a head with norm dims and no norm weight is divided by its root mean square
  const int* positions; float q_temp_coef; int q_temp_every;  // queries times 1 + coef * ln(floor((p + 1) / every) + 1)
  const void* v_first; int v_first_stride; float v_blend;     // values become (1 - v_blend) v + v_blend v_first[t, head, :]
};

// grid (T, ceil((n_q + n_kv) / HP_WAVES)); a wave a (token, head).  Lane l holds the pairs l, l + 64, ..
template <class TS, class TA>
__global__ __launch_bounds__(HP_WAVES* FG_WAVE) void heads_prepare_kernel(const PrepareArgs a) {
  const int lane = threadIdx.x % FG_WAVE, wave = threadIdx.x / FG_WAVE;
  const int t = blockIdx.x, job = blockIdx.y * HP_WAVES + wave;
  if (job >= a.n_q + a.n_kv) return;  // whole waves; no block barrier below
  const bool is_q = job < a.n_q;
  const int head = is_q ? job : job - a.n_q;
  int slot = -1;
  if (!is_q) {
    slot = a.slots[t];
    if (slot < 0) return;  // a token that writes nothing
  }
  const int w = is_q ? a.q_w : a.k_w;
  const int col = is_q ? a.q_col + head * a.q_w : a.k_col + head * a.k_w;
  const int norm_dims = is_q ? a.q_norm_dims : a.k_norm_dims;
  const float* norm_w = is_q ? a.q_norm_w : a.k_norm_w;
  const TS* row = (const TS*)a.src + (size_t)t * a.src_stride;
  float x[HP_MAX_PAIRS][2];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < HP_MAX_PAIRS; ++j) {
    const int d = 2 * (lane + FG_WAVE * j);
    x[j][0] = x[j][1] = 0.f;
    if (d < w) {
      x[j][0] = to_f<TS>(row[col + d]);
      x[j][1] = to_f<TS>(row[col + d + 1]);
      if (a.bias) {
        x[j][0] += a.bias[col + d];
        x[j][1] += a.bias[col + d + 1];
      }
      if (d < norm_dims) ss += x[j][0] * x[j][0] + x[j][1] * x[j][1];
    }
  }
  // a query's temperature grows with the logarithm of its position, in steps of `every` positions
  const bool tempered = is_q && a.positions && a.q_temp_every > 0;  // uniform
  const float temp = tempered ? 1.f + a.q_temp_coef * logf((float)((a.positions[t] + 1) / a.q_temp_every) + 1.f) : 1.f;
  if (norm_w || (a.norm_plain && norm_dims > 0)) {  // uniform
    ss = wave_sum(ss);
    const float rstd = rsqrtf(ss / (float)norm_dims + a.eps);
#pragma unroll
    for (int j = 0; j < HP_MAX_PAIRS; ++j) {
      const int d = 2 * (lane + FG_WAVE * j);
      if (d < norm_dims) {
        x[j][0] = x[j][0] * rstd * (norm_w ? norm_w[d] : 1.f);
        x[j][1] = x[j][1] * rstd * (norm_w ? norm_w[d + 1] : 1.f);
      }
    }
  }
  if (tempered) {
#pragma unroll
    for (int j = 0; j < HP_MAX_PAIRS; ++j) {
      x[j][0] *= temp;
      x[j][1] *= temp;
    }
  }
  if (a.table && (is_q ? a.rot_q : a.rot_k)) {  // uniform
#pragma unroll
    for (int j = 0; j < HP_MAX_PAIRS; ++j) {
      const int d = 2 * (lane + FG_WAVE * j);
      if (d >= a.rot_start && d < a.rot_start + a.rotary_dim && d < w) {
        const float2 cs = *(const float2*)(a.table + ((size_t)t * (a.rotary_dim / 2) + (d - a.rot_start) / 2) * 2);
        const float u = x[j][0], v = x[j][1];
        x[j][0] = u * cs.x - v * cs.y;
        x[j][1] = v * cs.x + u * cs.y;
      }
    }
  }
  if (is_q) {
    TA* o = (TA*)a.q_out + (size_t)t * a.q_out_stride + (size_t)head * a.q_out_hw;
#pragma unroll
    for (int j = 0; j < HP_MAX_PAIRS; ++j) {
      const int d = 2 * (lane + FG_WAVE * j);
      if (d < a.q_out_hw) {  // (x is zero from w on)
        o[d] = from_f<TA>(x[j][0]);
        o[d + 1] = from_f<TA>(x[j][1]);
      }
    }
    return;
  }
  const int page = slot / a.page_size, off = slot % a.page_size;
  const KvLayout lay(a.page_size, a.hd_c);
  const size_t head_elems = (size_t)a.page_size * a.hd_c;
  TA* kp = (TA*)a.k_pages + ((size_t)page * a.n_kv + head) * head_elems;
  TA* vp = (TA*)a.v_pages + ((size_t)page * a.n_kv + head) * head_elems;
#pragma unroll
  for (int j = 0; j < HP_MAX_PAIRS; ++j) {
    const int d = 2 * (lane + FG_WAVE * j);
    if (d < a.hd_c) {
      TA* dst = kp + lay.k_off(off, d);  // d is even: d + 1 lies in the same chunk of 8
      dst[0] = from_f<TA>(x[j][0]);
      dst[1] = from_f<TA>(x[j][1]);
      float v0 = 0.f, v1 = 0.f;
      if (d < a.v_w) {
        if (a.v_col < 0) {
          v0 = x[j][0];
          v1 = x[j][1];
        } else {
          const int c = a.v_col + head * a.v_w + d;
          v0 = to_f<TS>(row[c]) + (a.bias ? a.bias[c] : 0.f);
          v1 = to_f<TS>(row[c + 1]) + (a.bias ? a.bias[c + 1] : 0.f);
          if (a.v_first) {  // blended with the values that an earlier layer computed for this token
            const TS* f = (const TS*)a.v_first + (size_t)t * a.v_first_stride + head * a.v_w + d;
            v0 = (1.f - a.v_blend) * v0 + a.v_blend * to_f<TS>(f[0]);
            v1 = (1.f - a.v_blend) * v1 + a.v_blend * to_f<TS>(f[1]);
          }
        }
      }
      vp[lay.v_off(off, d)] = from_f<TA>(v0);
      vp[lay.v_off(off, d + 1)] = from_f<TA>(v1);
    }
  }
}

extern "C" int fg_heads_prepare(const PrepareArgs* args, int n_tokens, int src_dtype, int act_dtype,
                                hipStream_t stream) {
  if (n_tokens <= 0) return FG_OK;
  const PrepareArgs& a = *args;
  const int lim = 2 * FG_WAVE * HP_MAX_PAIRS;
  if (a.n_q < 0 || a.n_kv < 0 || a.n_q + a.n_kv <= 0 || !a.src) return FG_ERR_ARG;
  if (a.n_q && (a.q_w <= 0 || a.q_w % 2 || a.q_w > lim || a.q_out_hw < a.q_w || a.q_out_hw % 2 || a.q_out_hw > lim ||
                !a.q_out || a.q_norm_dims > a.q_w || a.q_norm_dims % 2))
    return FG_ERR_ARG;
  if (a.n_kv && (a.k_w <= 0 || a.k_w % 2 || a.hd_c < a.k_w || a.hd_c % 8 || a.hd_c > lim || a.v_w <= 0 || a.v_w % 2 ||
                 a.v_w > a.hd_c || (a.v_col < 0 && a.v_w > a.k_w) || a.page_size <= 0 || a.page_size % 8 ||
                 !a.slots || !a.k_pages || !a.v_pages || a.k_norm_dims > a.k_w || a.k_norm_dims % 2))
    return FG_ERR_ARG;
  if (a.table && (a.rot_start < 0 || a.rot_start % 2 || a.rotary_dim <= 0 || a.rotary_dim % 2)) return FG_ERR_ARG;
  const int jobs = a.n_q + a.n_kv;
  dim3 grid(n_tokens, (jobs + HP_WAVES - 1) / HP_WAVES);
  if (grid.y > 65535) return FG_ERR_ARG;
  if (src_dtype == FG_F32 && act_dtype == FG_F32)
    heads_prepare_kernel<float, float><<<grid, HP_WAVES * FG_WAVE, 0, stream>>>(a);
  else if (src_dtype == FG_F32 && act_dtype == FG_BF16)
    heads_prepare_kernel<float, bf16_t><<<grid, HP_WAVES * FG_WAVE, 0, stream>>>(a);
  else if (src_dtype == FG_BF16 && act_dtype == FG_BF16)
    heads_prepare_kernel<bf16_t, bf16_t><<<grid, HP_WAVES * FG_WAVE, 0, stream>>>(a);
  else
    return FG_ERR_ARG;
  return fg_launch_status();
}

// ------------------------------------------------------------------ head_linear
struct HeadLinearArgs {
  const void* x; int x_stride, x_hs;   // x[t, h, k] at t * x_stride + h * x_hs + k
  const void* w;                       // [H, N, K]
  void* y; int y_stride, y_hs;         // y[t, h, n] at t * y_stride + h * y_hs + n
  const float* gate; int gate_stride;  // gate[t * gate_stride + h] or null: y *= sigmoid(gate)
  int T, H, N, K;
  int tail, y_hw;  // y[t, h, N + j] = x[t, h, K + j] for j < tail; zeros from N + tail to y_hw
};

// Any dtype: grid (T, H), 256 threads; x's head goes through LDS, a thread an output element.
#define HL_MAX_K 1024
template <class T>
__global__ __launch_bounds__(256) void head_linear_kernel(const HeadLinearArgs a) {
  __shared__ float x_s[HL_MAX_K];
  const int t = blockIdx.x, h = blockIdx.y;
  const T* x = (const T*)a.x + (size_t)t * a.x_stride + (size_t)h * a.x_hs;
  for (int k = threadIdx.x; k < a.K; k += 256) x_s[k] = to_f<T>(x[k]);
  __syncthreads();
  float gv = 1.f;
  if (a.gate) gv = 1.f / (1.f + expf(-a.gate[(size_t)t * a.gate_stride + h]));
  T* y = (T*)a.y + (size_t)t * a.y_stride + (size_t)h * a.y_hs;
  const T* w = (const T*)a.w + (size_t)h * a.N * a.K;
  for (int n = threadIdx.x; n < a.y_hw; n += 256) {
    float acc = 0.f;
    if (n < a.N) {
      const T* wr = w + (size_t)n * a.K;
      for (int k = 0; k < a.K; ++k) acc += to_f<T>(wr[k]) * x_s[k];  // k ascending
      acc *= gv;
    } else if (n < a.N + a.tail) {
      acc = to_f<T>(x[a.K + n - a.N]);
    }
    y[n] = from_f<T>(acc);
  }
}

// bfloat16 on the matrix cores: grid (ceil(T / 64), ceil(N / 64), H), 4 waves; a wave takes 16
// output channels and 64 tokens (four blocks of 16), operands straight from memory.  K % 8 == 0 and
// rows of x 16-byte aligned.  acc[mb][i] = y[token 16 mb + (lane & 15)][channel 4 (lane >> 4) + i].
__global__ __launch_bounds__(256) void head_linear_mfma_kernel(const HeadLinearArgs a) {
  const int lane = threadIdx.x % FG_WAVE, wave = threadIdx.x / FG_WAVE;
  const int r16 = lane & 15, g = lane >> 4;
  const int m0 = blockIdx.x * 64, n0 = (blockIdx.y * 4 + wave) * 16, h = blockIdx.z;
  const bf16_t* xh = (const bf16_t*)a.x + (size_t)h * a.x_hs;
  if (n0 < a.N) {  // whole waves
    const bf16_t* wrow = (const bf16_t*)a.w + ((size_t)h * a.N + min(n0 + r16, a.N - 1)) * a.K;
    const bf16_t* xrow[4];
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) xrow[mb] = xh + (size_t)min(m0 + 16 * mb + r16, a.T - 1) * a.x_stride;
    f32x4 acc[4];
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) acc[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < a.K; k0 += 32) {
      const int kk = k0 + 8 * g;
      bf16x8 wa, xb[4];
      if (kk < a.K) {
        wa = *(const bf16x8*)(wrow + kk);
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) xb[mb] = *(const bf16x8*)(xrow[mb] + kk);
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) wa[i] = (__bf16)0.f;
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) xb[mb] = wa;
      }
#pragma unroll
      for (int mb = 0; mb < 4; ++mb) acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa, xb[mb], acc[mb], 0, 0, 0);
    }
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) {
      const int t = m0 + 16 * mb + r16;
      if (t >= a.T) continue;
      float gv = 1.f;
      if (a.gate) gv = 1.f / (1.f + __expf(-a.gate[(size_t)t * a.gate_stride + h]));
      bf16_t* y = (bf16_t*)a.y + (size_t)t * a.y_stride + (size_t)h * a.y_hs;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = n0 + 4 * g + i;
        if (n < a.N) y[n] = (bf16_t)(acc[mb][i] * gv);
      }
    }
  }
  if (blockIdx.y == 0) {  // what lies behind the product: copied columns, then zeros
    const int extra = a.y_hw - a.N;
    for (int e = threadIdx.x; e < 64 * extra; e += 256) {
      const int t = m0 + e / extra, j = e % extra;
      if (t >= a.T) break;
      const bf16_t v = j < a.tail ? xh[(size_t)t * a.x_stride + a.K + j] : (bf16_t)0.f;
      ((bf16_t*)a.y)[(size_t)t * a.y_stride + (size_t)h * a.y_hs + a.N + j] = v;
    }
  }
}

extern "C" int fg_head_linear(const HeadLinearArgs* args, int dtype, int use_mfma, hipStream_t stream) {
  const HeadLinearArgs& a = *args;
  if (a.T <= 0) return FG_OK;
  if (a.H <= 0 || a.N <= 0 || a.K <= 0 || a.tail < 0 || a.y_hw < a.N + a.tail || a.x_hs < a.K + a.tail ||
      a.y_hs < a.y_hw || !a.x || !a.w || !a.y)
    return FG_ERR_ARG;
  if (use_mfma) {
    if (dtype != FG_BF16 || a.K % 8 || a.x_stride % 8 || a.x_hs % 8 || a.H > 65535 || (a.N + 63) / 64 > 65535)
      return FG_ERR_ARG;
    head_linear_mfma_kernel<<<dim3((a.T + 63) / 64, (a.N + 63) / 64, a.H), 256, 0, stream>>>(a);
    return fg_launch_status();
  }
  if (a.K > HL_MAX_K || a.H > 65535) return FG_ERR_ARG;
  if (dtype == FG_F32) head_linear_kernel<float><<<dim3(a.T, a.H), 256, 0, stream>>>(a);
  else if (dtype == FG_BF16) head_linear_kernel<bf16_t><<<dim3(a.T, a.H), 256, 0, stream>>>(a);
  else return FG_ERR_ARG;
  return fg_launch_status();
}

// ---------------------------------------------------------------- head_norm_gate
// out[t, h, :] = x[t, h, :] * rsqrt(mean(x[t, h, :]^2) + eps) * w * silu(g[t, h, :]); x fp32 [T, H * e],
// g (act dtype) columns of a wider row.  grid (T, ceil(H / 4)); a wave a (token, head).
#define HN_MAX 16  // elements a lane holds: heads of up to 1,024
template <class TA>
__global__ __launch_bounds__(HP_WAVES* FG_WAVE) void head_norm_gate_kernel(
    const float* __restrict__ x, const float* __restrict__ w, const TA* __restrict__ gate, int gate_stride,
    TA* __restrict__ out, int H, int e, float eps) {
  const int lane = threadIdx.x % FG_WAVE, wave = threadIdx.x / FG_WAVE;
  const int t = blockIdx.x, h = blockIdx.y * HP_WAVES + wave;
  if (h >= H) return;
  const float* xr = x + ((size_t)t * H + h) * e;
  float v[HN_MAX];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < HN_MAX; ++j) {
    const int d = lane + FG_WAVE * j;
    v[j] = d < e ? xr[d] : 0.f;
    ss += v[j] * v[j];
  }
  ss = wave_sum(ss);
  const float rstd = rsqrtf(ss / (float)e + eps);
  const TA* gr = gate + (size_t)t * gate_stride + (size_t)h * e;
  TA* o = out + ((size_t)t * H + h) * e;
#pragma unroll
  for (int j = 0; j < HN_MAX; ++j) {
    const int d = lane + FG_WAVE * j;
    if (d < e) {
      const float gv = to_f<TA>(gr[d]);
      o[d] = from_f<TA>(v[j] * rstd * w[d] * (gv / (1.f + expf(-gv))));
    }
  }
}

extern "C" int fg_head_norm_gate(const float* x, const float* w, const void* gate, int gate_stride, void* out,
                                 int n_tokens, int H, int e, float eps, int act_dtype, hipStream_t stream) {
  if (n_tokens <= 0) return FG_OK;
  if (H <= 0 || e <= 0 || e > HN_MAX * FG_WAVE || gate_stride < H * e || (H + HP_WAVES - 1) / HP_WAVES > 65535)
    return FG_ERR_ARG;
  dim3 grid(n_tokens, (H + HP_WAVES - 1) / HP_WAVES);
  if (act_dtype == FG_F32)
    head_norm_gate_kernel<float><<<grid, HP_WAVES * FG_WAVE, 0, stream>>>(x, w, (const float*)gate, gate_stride,
                                                                         (float*)out, H, e, eps);
  else if (act_dtype == FG_BF16)
    head_norm_gate_kernel<bf16_t><<<grid, HP_WAVES * FG_WAVE, 0, stream>>>(x, w, (const bf16_t*)gate, gate_stride,
                                                                          (bf16_t*)out, H, e, eps);
  else
    return FG_ERR_ARG;
  return fg_launch_status();
}

// ---------------------------------------------------------------- head_diff_norm
// Two attention maps a head, one value: out[t, h, :] = n(a1 - lam * a2) * out_scale with
// n(o) = o * rsqrt(mean(o^2) + eps) over the head's e values (no weight).  `att` holds 2 H heads of `hw`
// columns (the first e are the head's output): the heads of a key/value group of `group` query heads lie
// as [map 1 of the group's heads | map 2 of the group's heads], so a1 of head h is head
// (h / group) * 2 * group + h % group of `att` and a2 lies `group` heads behind it.  All in fp32, one
// rounding at the store.  grid (T, ceil(H / 4)); a wave a (token, head).
template <class TA>
__global__ __launch_bounds__(HP_WAVES* FG_WAVE) void head_diff_norm_kernel(
    const TA* __restrict__ att, int att_stride, int hw, TA* __restrict__ out, int out_stride, int H, int group, int e,
    float lam, float eps, float out_scale) {
  const int lane = threadIdx.x % FG_WAVE, wave = threadIdx.x / FG_WAVE;
  const int t = blockIdx.x, h = blockIdx.y * HP_WAVES + wave;
  if (h >= H) return;
  const TA* a1 = att + (size_t)t * att_stride + (size_t)((h / group) * 2 * group + h % group) * hw;
  const TA* a2 = a1 + (size_t)group * hw;
  float v[HN_MAX];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < HN_MAX; ++j) {
    const int d = lane + FG_WAVE * j;
    v[j] = d < e ? to_f<TA>(a1[d]) - lam * to_f<TA>(a2[d]) : 0.f;
    ss += v[j] * v[j];
  }
  ss = wave_sum(ss);
  const float mul = rsqrtf(ss / (float)e + eps) * out_scale;
  TA* o = out + (size_t)t * out_stride + (size_t)h * e;
#pragma unroll
  for (int j = 0; j < HN_MAX; ++j) {
    const int d = lane + FG_WAVE * j;
    if (d < e) o[d] = from_f<TA>(v[j] * mul);
  }
}

extern "C" int fg_head_diff_norm(const void* att, int att_stride, int hw, void* out, int out_stride, int n_tokens, int H,
                                 int group, int e, float lam, float eps, float out_scale, int act_dtype,
                                 hipStream_t stream) {
  if (n_tokens <= 0) return FG_OK;
  if (H <= 0 || group <= 0 || H % group || e <= 0 || e > HN_MAX * FG_WAVE || hw < e || att_stride < 2 * H * hw ||
      out_stride < H * e || (H + HP_WAVES - 1) / HP_WAVES > 65535)
    return FG_ERR_ARG;
  dim3 grid(n_tokens, (H + HP_WAVES - 1) / HP_WAVES);
  if (act_dtype == FG_F32)
    head_diff_norm_kernel<float><<<grid, HP_WAVES * FG_WAVE, 0, stream>>>((const float*)att, att_stride, hw, (float*)out,
                                                                         out_stride, H, group, e, lam, eps, out_scale);
  else if (act_dtype == FG_BF16)
    head_diff_norm_kernel<bf16_t><<<grid, HP_WAVES * FG_WAVE, 0, stream>>>((const bf16_t*)att, att_stride, hw, (bf16_t*)out,
                                                                          out_stride, H, group, e, lam, eps, out_scale);
  else
    return FG_ERR_ARG;
  return fg_launch_status();
}
