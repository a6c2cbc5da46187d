// Causal attention over the paged cache whose weights are sigmoids, not a softmax, general form: any element
// type, every head of a token in one workgroup.
//
// For query token i (position p) and key j <= p of the same sequence, per query head h (kv head h / (H / G)):
//   s_h  = (q_h . k_j) * scale + dist_bias[min(p - j, n_dist - 1)][h]          (the bias is optional)
//   m_h  = sum_g talk[h][g] s_g                                                  (optional: the heads' scores mixed)
//   w_h  = sigmoid(m_h + head_bias[h])                                           (not normalised over the keys)
//   o_h  = sum_j w_h(j) v_j ;   out[i, h, :] = o_h * sigmoid(gate[i, h])         (the gate is optional)
// Because the mixing needs every head's score of a (query, key) pair, a workgroup owns a token and all its
// heads and walks the keys in tiles of 64 that start at multiples of 64: scores into LDS (a wave a head, a
// lane a key), mixing and sigmoid (a thread a (head, key)), then the product with the values (a thread a
// (head, value dim), keys of a tile in the order in which the page stores them).  The sums over keys are
// kept per chunk of SA_CHUNK_TILES tiles and the chunks added in order, so that cutting the keys over
// several workgroups (`partial`: a workgroup a (token, chunk), fp32 sums per chunk, added in the same order by
// the combine kernel) gives the same bits as one workgroup walking them all.  What a token gets depends on
// its own keys alone: not on the batch, the cut of the prompt, or the pages.
//
// Keys and values lie in pages of head size hd_c (kv_layout.h); a key's first d and a value's first e
// dimensions are read.  All arithmetic is fp32.
#include "common.h"
#include "kv_layout.h"

#define SA_THREADS 256
#define SA_WAVES 4
#define SA_TILE 64
#define SA_CHUNK_TILES 1
#define SA_MAX_ITEMS 16  // (head, value dim) pairs a thread owns: heads * e <= 4096

struct SigmoidAttentionArgs {
  const void* q; int q_stride, q_hs;  // q[t, h, :] at t * q_stride + h * q_hs
  const void* k_pages; const void* v_pages;
  const int* block_table; int bt_stride;
  const int* seq_of_token; const int* positions;
  int n_tokens, n_heads, n_kv, d, e, hd_c, page_size;
  float scale;
  const float* dist_bias; int n_dist;  // [n_dist, n_heads] or null
  const float* talk;                   // [n_heads, n_heads] or null
  const float* head_bias;              // [n_heads] or null
  const float* gate; int gate_stride;  // gate[t * gate_stride + h] or null
  void* out; int out_stride;           // out[t, h * e + x]
  float* partial; int n_chunks;        // [n_chunks, n_tokens, n_heads * e] or null
};

template <class T> struct SaVec8;
template <> struct SaVec8<float> {
  float v[8];
  __device__ __forceinline__ void load(const float* p) { load8<float>(p, v); }
};
template <> struct SaVec8<bf16_t> {
  float v[8];
  __device__ __forceinline__ void load(const bf16_t* p) { load8<bf16_t>(p, v); }
};

template <class T>
__global__ __launch_bounds__(SA_THREADS) void sigmoid_attention_kernel(const SigmoidAttentionArgs a) {
  extern __shared__ float lds[];
  const int H = a.n_heads, d8 = (a.d + 7) & ~7;
  float* q_s = lds;                     // [H][d8]
  float* raw = q_s + H * d8;            // [H][64]
  float* p_s = raw + H * SA_TILE;       // [H][64]
  float* talk_s = p_s + H * SA_TILE;    // [H][H]
  const int tid = threadIdx.x, lane = tid % FG_WAVE, wave = tid / FG_WAVE;
  const int t = blockIdx.x;
  const int seq = a.seq_of_token[t], pos = a.positions[t];
  const int rep = H / a.n_kv;
  const int n_items = H * a.e;
  const int chunk_keys = SA_CHUNK_TILES * SA_TILE;
  const int last_chunk = pos / chunk_keys;
  int c_lo = 0, c_hi = last_chunk;
  if (a.partial) {
    c_lo = c_hi = blockIdx.y;
    if (c_lo > last_chunk) return;  // uniform
  }
  const int* table = a.block_table + (size_t)seq * a.bt_stride;
  const KvLayout lay(a.page_size, a.hd_c);
  const size_t head_elems = (size_t)a.page_size * a.hd_c;
  const T* qrow = (const T*)a.q + (size_t)t * a.q_stride;
  for (int i = tid; i < H * d8; i += SA_THREADS) {
    const int h = i / d8, x = i % d8;
    q_s[i] = x < a.d ? to_f<T>(qrow[(size_t)h * a.q_hs + x]) : 0.f;
  }
  if (a.talk)
    for (int i = tid; i < H * H; i += SA_THREADS) talk_s[i] = a.talk[i];

  float total[SA_MAX_ITEMS], o[SA_MAX_ITEMS];
#pragma unroll
  for (int n = 0; n < SA_MAX_ITEMS; ++n) total[n] = 0.f;

  for (int c = c_lo; c <= c_hi; ++c) {
#pragma unroll
    for (int n = 0; n < SA_MAX_ITEMS; ++n) o[n] = 0.f;
    for (int kb = c * chunk_keys; kb < (c + 1) * chunk_keys && kb <= pos; kb += SA_TILE) {
      __syncthreads();  // q_s and talk_s are there; the tile before is done with raw and p_s
      // ---- scores: a wave a head in turns, a lane a key
      const int key = kb + lane;
      const bool valid = key <= pos;
      const T* kpage = nullptr;
      int kappa = 0, dist = 0;
      if (valid) {
        kpage = (const T*)a.k_pages + (size_t)table[key / a.page_size] * a.n_kv * head_elems;
        kappa = key % a.page_size;
        dist = pos - key < a.n_dist - 1 ? pos - key : a.n_dist - 1;
      }
      for (int h = wave; h < H; h += SA_WAVES) {
        float s = 0.f;
        if (valid) {
          const T* khead = kpage + (size_t)(h / rep) * head_elems;
          const float* qh = q_s + h * d8;
          float acc = 0.f;
          for (int x = 0; x < d8; x += 8) {
            SaVec8<T> kv;
            kv.load(khead + lay.k_off(kappa, x));
#pragma unroll
            for (int i = 0; i < 8; ++i) acc = fmaf(qh[x + i], kv.v[i], acc);
          }
          s = acc * a.scale;
          if (a.dist_bias) s += a.dist_bias[(size_t)dist * H + h];
        }
        raw[h * SA_TILE + lane] = s;
      }
      __syncthreads();
      // ---- mixing and sigmoid: a thread a (head, key)
      for (int i = tid; i < H * SA_TILE; i += SA_THREADS) {
        const int h = i / SA_TILE, j = i % SA_TILE;
        float m;
        if (a.talk) {
          m = 0.f;
          for (int g = 0; g < H; ++g) m = fmaf(talk_s[h * H + g], raw[g * SA_TILE + j], m);
        } else {
          m = raw[i];
        }
        if (a.head_bias) m += a.head_bias[h];
        p_s[i] = kb + j <= pos ? 1.f / (1.f + expf(-m)) : 0.f;
      }
      __syncthreads();
      // ---- o += w . v: a thread a (head, value dim); one stored chunk of eight key slots at a time
#pragma unroll
      for (int n = 0; n < SA_MAX_ITEMS; ++n) {
        const int item = tid + n * SA_THREADS;
        if (item >= n_items) break;
        const int h = item / a.e, x = item % a.e;
        const float* ph = p_s + h * SA_TILE;
        float acc = o[n];
        for (int qd = 0; qd < SA_TILE / 8; ++qd) {
          const int base = lay.permuted ? kb + 32 * (qd / 4) + 4 * (qd % 4) : kb + 8 * qd;  // lowest key of the chunk
          const int stride_hi = lay.permuted ? 12 : 0;  // slots 4..7 are 16 keys on
          if (base > pos) { if (lay.permuted) continue; else break; }
          const T* vhead = (const T*)a.v_pages + ((size_t)table[base / a.page_size] * a.n_kv + h / rep) * head_elems;
          SaVec8<T> vv;
          vv.load(vhead + lay.v_chunk_off(lay.v_slot(base % a.page_size) / 8, x));
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const int kk = base + i + (i >= 4 ? stride_hi : 0);
            if (kk <= pos) acc = fmaf(ph[kk - kb], vv.v[i], acc);  // select: a slot never written may hold NaN
          }
        }
        o[n] = acc;
      }
    }
    if (a.partial) {
      float* dst = a.partial + ((size_t)c * a.n_tokens + t) * n_items;
#pragma unroll
      for (int n = 0; n < SA_MAX_ITEMS; ++n) {
        const int item = tid + n * SA_THREADS;
        if (item < n_items) dst[item] = o[n];
      }
      return;
    }
#pragma unroll
    for (int n = 0; n < SA_MAX_ITEMS; ++n) total[n] += o[n];
  }
  T* orow = (T*)a.out + (size_t)t * a.out_stride;
#pragma unroll
  for (int n = 0; n < SA_MAX_ITEMS; ++n) {
    const int item = tid + n * SA_THREADS;
    if (item < n_items) {
      float y = total[n];
      if (a.gate) y *= 1.f / (1.f + expf(-a.gate[(size_t)t * a.gate_stride + item / a.e]));
      orow[item] = from_f<T>(y);
    }
  }
}

// out[t, item] = (sum over the token's chunks, in order) * sigmoid(gate[t, head]); a thread an element
template <class T>
__global__ __launch_bounds__(SA_THREADS) void sigmoid_attention_combine_kernel(const SigmoidAttentionArgs a) {
  const int t = blockIdx.x;
  const int n_items = a.n_heads * a.e;
  const int item = blockIdx.y * SA_THREADS + threadIdx.x;
  if (item >= n_items) return;
  const int last_chunk = a.positions[t] / (SA_CHUNK_TILES * SA_TILE);
  const size_t step = (size_t)a.n_tokens * n_items;
  const float* p = a.partial + (size_t)t * n_items + item;
  float y = 0.f;
  int c = 0;
  for (; c + 4 <= last_chunk + 1; c += 4) {  // four loads in flight, added in order
    const float p0 = p[c * step], p1 = p[(c + 1) * step], p2 = p[(c + 2) * step], p3 = p[(c + 3) * step];
    y += p0; y += p1; y += p2; y += p3;
  }
  for (; c <= last_chunk; ++c) y += p[c * step];
  if (a.gate) y *= 1.f / (1.f + expf(-a.gate[(size_t)t * a.gate_stride + item / a.e]));
  ((T*)a.out)[(size_t)t * a.out_stride + item] = from_f<T>(y);
}

extern "C" int fg_sigmoid_attention_chunk_keys() { return SA_CHUNK_TILES * SA_TILE; }

extern "C" int fg_sigmoid_attention(const SigmoidAttentionArgs* args, int dtype, hipStream_t stream) {
  const SigmoidAttentionArgs& a = *args;
  if (a.n_tokens <= 0) return FG_OK;
  if (a.n_heads <= 0 || a.n_kv <= 0 || a.n_heads % a.n_kv || a.d <= 0 || a.e <= 0 || a.hd_c % 8 || a.d > a.hd_c ||
      a.e > a.hd_c || a.page_size <= 0 || a.page_size % 8 || a.n_heads * a.e > SA_MAX_ITEMS * SA_THREADS ||
      (a.dist_bias && a.n_dist < 1) || (a.partial && a.n_chunks < 1) || !a.q || !a.out || !a.k_pages || !a.v_pages)
    return FG_ERR_ARG;
  const int d8 = (a.d + 7) & ~7;
  const size_t lds = ((size_t)a.n_heads * d8 + 2 * (size_t)a.n_heads * SA_TILE + (size_t)a.n_heads * a.n_heads) * sizeof(float);
  if (lds > 65536) return FG_ERR_ARG;
  dim3 grid(a.n_tokens, a.partial ? a.n_chunks : 1);
  if (grid.y > 65535) return FG_ERR_ARG;
  const dim3 combine_grid(a.n_tokens, (a.n_heads * a.e + SA_THREADS - 1) / SA_THREADS);
  if (dtype == FG_F32) {
    sigmoid_attention_kernel<float><<<grid, SA_THREADS, lds, stream>>>(a);
    if (a.partial) sigmoid_attention_combine_kernel<float><<<combine_grid, SA_THREADS, 0, stream>>>(a);
  } else if (dtype == FG_BF16) {
    sigmoid_attention_kernel<bf16_t><<<grid, SA_THREADS, lds, stream>>>(a);
    if (a.partial) sigmoid_attention_combine_kernel<bf16_t><<<combine_grid, SA_THREADS, 0, stream>>>(a);
  } else {
    return FG_ERR_ARG;
  }
  return fg_launch_status();
}
