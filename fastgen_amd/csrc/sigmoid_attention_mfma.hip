// Causal attention with sigmoid weights and mixed heads on the matrix cores, for prompt portions in bfloat16
// (gfx950).  Compiled once per width of a head in the cache: -DFG_HD=<multiple of 16, at most 256>.
//
// The general kernel (sigmoid_attention.hip) gives a token a workgroup; here a workgroup owns an *item*, up to
// 16 consecutive query tokens of one sequence with all their heads (at most 16), and a chunk of the keys.  Per
// tile of 32 keys, in three phases with LDS between them:
//   1. scores  S_g^T = K Q_g^T  per head g (v_mfma_f32_16x16x32_bf16; a wave owns a few heads): fp32 into
//      raw[g][key][token];
//   2. mixing  M = T' raw  over the heads, per key (v_mfma_f32_16x16x4_f32: a true fp32 product; T' = the
//      mixing matrix times the scale, zero padded to 16 x 16), plus mixed[dist][h] (the distance bias mixed the
//      same way plus the head's bias, made once by the host: mixing is linear), sigmoid, causal mask; the
//      weights go to LDS as two bfloat16 terms in one word (the weight and what its rounding dropped: 16
//      significant bits);
//   3. values  O_h^T += V^T W_h^T  (both terms), V read from the transposed pages (kv_layout.h: with pages of
//      a multiple of 32 keys a lane group's 8 keys are one 16-byte chunk).
// The sums over keys are fp32 and plain (no maximum, no normalisation), so chunks of keys add up: with more
// than one chunk an item's partial sums go to scratch and a second kernel adds them in order and applies the
// heads' gates.  What a token gets does not depend on the batch or on the cut of the prompt beyond the rounding
// of these sums.
#include "common.h"
#include "kv_layout.h"

#ifndef FG_HD
#error "compile with -DFG_HD=<head size>"
#endif
static_assert(FG_HD % 16 == 0 && FG_HD >= 16 && FG_HD <= 256, "head size: multiple of 16 up to 256");

constexpr int HD = FG_HD;
constexpr int NKS = (HD + 31) / 32;  // 32-wide steps over the head dimension (the last may be half)
constexpr int NDB = HD / 16;         // 16-wide blocks of the head dimension
constexpr int KT = 32;               // keys of a tile
constexpr int TQ = 16;               // query tokens of an item
constexpr int HP = 16;               // heads, padded
constexpr int ST_THREADS = 256;
constexpr int RAW_LD = TQ + 1;       // raw[g][key][token], padded against bank conflicts
constexpr int W_LD = KT + 4;         // weights[h][token][key] in words, rows 16-byte aligned

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

struct SigmoidTileArgs {
  const bf16_t* q; int q_stride, q_hs;  // q[t, h, :] at t * q_stride + h * q_hs
  const bf16_t* k_pages; const bf16_t* v_pages;
  const int* block_table; int bt_stride;
  const int* items; int n_items;        // [n_items, 4]: sequence, first flat token, tokens (<= 16), first position
  const int* positions;                 // [n_tokens]
  int n_tokens, n_heads, n_kv, d, e, page_size;
  const float* talk;                    // [16, 16]: (mixing matrix or identity) * scale, zero padded
  const float* mixed; int n_dist;       // [n_dist, 16]: mixed distance bias + head bias
  const float* gate; int gate_stride;   // gate[t * gate_stride + h] or null
  bf16_t* out; int out_stride;          // out[t, h * e + x]
  float* partial; int n_chunks, chunk_keys;  // [n_chunks, n_tokens, n_heads * e] or null (one chunk)
};

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

// zeroes the value slots of keys beyond `hi`; slot s of a chunk is key ka + (s & 3) + 16 * (s >> 2)
__device__ __forceinline__ bf16x8 mask_slots(bf16x8 v, int ka, int hi) {
  u32x4 m;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const int k_even = ka + ((2 * w) & 3) + 16 * ((2 * w) >> 2), k_odd = k_even + 1;
    m[w] = (k_even <= hi ? 0x0000ffffu : 0u) | (k_odd <= hi ? 0xffff0000u : 0u);
  }
  return __builtin_bit_cast(bf16x8, __builtin_bit_cast(u32x4, v) & m);
}

// KV1: the heads of a wave all belong to one kv head (the heads of a group are a multiple of a wave's heads).  Then
// a wave keeps one set of key operands and one of value operands, and they are asked for ahead of their use: the
// next tile's keys before the mixing of this one, this tile's values before its scores.
template <int HPW, bool KV1>
__global__ __launch_bounds__(ST_THREADS) void sigmoid_tile_kernel(const SigmoidTileArgs a) {
  extern __shared__ float lds[];
  float* raw = lds;                                          // [HP][KT][RAW_LD]
  uint32_t* wts = (uint32_t*)(lds + HP * KT * RAW_LD);       // [HP][TQ][W_LD]
  const int tid = threadIdx.x, lane = tid % FG_WAVE, wave = tid / FG_WAVE;
  const int g = lane >> 4, row = lane & 15;
  const int4 it = *(const int4*)(a.items + 4 * blockIdx.x);
  const int seq = it.x, tok0 = it.y, n_tok = it.z, pos0 = it.w;
  const int pos_last = pos0 + n_tok - 1;
  const int chunk = blockIdx.y;
  const int k_begin = chunk * a.chunk_keys;
  if (k_begin > pos_last) return;  // uniform
  const int k_last = min(pos_last, k_begin + a.chunk_keys - 1);
  const int H = a.n_heads, rep = H / a.n_kv;
  const bool row_valid = row < n_tok;
  const int pos_row = pos0 + row;
  const int* table = a.block_table + (size_t)seq * a.bt_stride;
  const KvLayout lay(a.page_size, HD);
  const size_t head_elems = (size_t)a.page_size * HD;

  for (int i = tid; i < HP * KT * RAW_LD; i += ST_THREADS) raw[i] = 0.f;  // the rows of heads that do not exist stay zero

  // this wave's heads: their queries as operands, their sums
  bf16x8 qop[HPW][NKS];
  f32x4 o[HPW][NDB];
#pragma unroll
  for (int j = 0; j < HPW; ++j) {
    const int h = wave * HPW + j;
    const bf16_t* qrow = a.q + (size_t)(tok0 + (row_valid ? row : 0)) * a.q_stride + (size_t)(h < H ? h : 0) * a.q_hs;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      bf16x8 v = zero8();
#pragma unroll
      for (int x = 0; x < 8; ++x) {
        const int dim = 32 * ks + 8 * g + x;
        if (row_valid && h < H && dim < a.d) v[x] = __builtin_bit_cast(__bf16, qrow[dim]);
      }
      qop[j][ks] = v;
    }
#pragma unroll
    for (int db = 0; db < NDB; ++db) o[j][db] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  // the mixing matrix as the fp32 products' first operand: A[m = lane % 16][k = 4 s + lane / 16]
  float talk_op[HP / 4];
#pragma unroll
  for (int s = 0; s < HP / 4; ++s) talk_op[s] = a.talk[row * HP + 4 * s + g];

  // A tile of 32 keys lies in one page (pages hold a multiple of 32 keys); keys of the tile beyond the item's last
  // position may never have been written: whatever they hold, their weights are masked by a select.
  const int my_kv = min(wave * HPW, H - 1) / rep;
  bf16x8 kpre[KT / 16][NKS], vpre[NDB];
  auto ask_keys = [&](int k0) {
    const bf16_t* kp = a.k_pages + ((size_t)table[k0 / a.page_size] * a.n_kv + my_kv) * head_elems;
#pragma unroll
    for (int kb = 0; kb < KT / 16; ++kb)
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        const int dim = 32 * ks + 8 * g;
        kpre[kb][ks] = dim < HD ? *(const bf16x8*)(kp + lay.k_off(k0 % a.page_size + 16 * kb + row, dim < HD ? dim : 0)) : zero8();
      }
  };
  auto ask_values = [&](int k0) {
    const bf16_t* vhead = a.v_pages + ((size_t)table[k0 / a.page_size] * a.n_kv + my_kv) * head_elems;
    const int kc = (k0 % a.page_size) / 8 + g;
#pragma unroll
    for (int db = 0; db < NDB; ++db) vpre[db] = *(const bf16x8*)(vhead + lay.v_chunk_off(kc, 16 * db + row));
  };
  if (KV1) ask_keys(k_begin);

  for (int k0 = k_begin; k0 <= k_last; k0 += KT) {
    __syncthreads();  // raw is zeroed; the tile before is done with raw (and its weights are read below, after a barrier)
    if (KV1) {
      ask_values(k0);
      // ---- 1. scores
#pragma unroll
      for (int kb = 0; kb < KT / 16; ++kb)
#pragma unroll
        for (int j = 0; j < HPW; ++j) {
          const int h = wave * HPW + j;
          if (h < H) {  // uniform in the wave
            f32x4 s = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kpre[kb][ks], qop[j][ks], s, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 4; ++i) raw[(h * KT + 16 * kb + 4 * g + i) * RAW_LD + row] = s[i];
          }
        }
      if (k0 + KT <= k_last) ask_keys(k0 + KT);
    }
    // ---- 1. scores (heads of one kv head that follow each other in a wave share its keys' operands)
#pragma unroll
    for (int kb = 0; kb < (KV1 ? 0 : KT / 16); ++kb) {
      const int key = min(k0 + 16 * kb + row, pos_last);  // a key that exists; those beyond a row's position are masked below
      const bf16_t* kpage = a.k_pages + (size_t)table[key / a.page_size] * a.n_kv * head_elems;
      const int kappa = key % a.page_size;
      bf16x8 kop[NKS];
      int loaded = -1;
#pragma unroll
      for (int j = 0; j < HPW; ++j) {
        const int h = wave * HPW + j;
        if (h < H) {  // uniform in the wave
          const int kvh = h / rep;
          if (kvh != loaded) {  // uniform in the wave
            loaded = kvh;
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) {
              const int dim = 32 * ks + 8 * g;
              kop[ks] = dim < HD ? *(const bf16x8*)(kpage + (size_t)kvh * head_elems + lay.k_off(kappa, dim < HD ? dim : 0)) : zero8();
            }
          }
          f32x4 s = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int ks = 0; ks < NKS; ++ks) s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop[ks], qop[j][ks], s, 0, 0, 0);
#pragma unroll
          for (int i = 0; i < 4; ++i) raw[(h * KT + 16 * kb + 4 * g + i) * RAW_LD + row] = s[i];
        }
      }
    }
    __syncthreads();
    // ---- 2. mixing, bias, sigmoid, mask: a wave a key in turns; a lane ends with 4 heads of a (token, key)
#pragma unroll  // (eight keys a wave: their chains of reads, products and exponentials run side by side)
    for (int kq = 0; kq < KT / (ST_THREADS / FG_WAVE); ++kq) {
      const int kk = wave + kq * (ST_THREADS / FG_WAVE);
      f32x4 m = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < HP / 4; ++s)
        m = __builtin_amdgcn_mfma_f32_16x16x4f32(talk_op[s], raw[((4 * s + g) * KT + kk) * RAW_LD + row], m, 0, 0, 0);
      const int dist = pos_row - (k0 + kk);
      const bool visible = row_valid && dist >= 0;
      const int dist_c = dist < 0 ? 0 : (dist < a.n_dist - 1 ? dist : a.n_dist - 1);
      const f32x4 mb = *(const f32x4*)(a.mixed + (size_t)dist_c * HP + 4 * g);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float w = visible ? __builtin_amdgcn_rcpf(1.f + __expf(-(m[i] + mb[i]))) : 0.f;  // (the reciprocal: one ulp)
        const __bf16 hi = (__bf16)w;
        const __bf16 lo = (__bf16)(w - (float)hi);
        wts[((4 * g + i) * TQ + row) * W_LD + kk] =
            ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16) | (uint32_t)__builtin_bit_cast(uint16_t, lo);
      }
    }
    __syncthreads();
    // ---- 3. values (a kv head's operands are read once for the heads of its group that follow each other)
    const int page = table[k0 / a.page_size];
    const int kc = (k0 % a.page_size) / 8 + g;
    bf16x8 vop[NDB];
    int loaded = -1;
    if (KV1) {
      loaded = my_kv;
#pragma unroll
      for (int db = 0; db < NDB; ++db) vop[db] = mask_slots(vpre[db], k0 + 4 * g, pos_last);
    }
#pragma unroll
    for (int j = 0; j < HPW; ++j) {
      const int h = wave * HPW + j;
      if (h < H) {
        const int kvh = h / rep;
        if (kvh != loaded) {
          loaded = kvh;
          const bf16_t* vhead = a.v_pages + ((size_t)page * a.n_kv + kvh) * head_elems;
#pragma unroll
          for (int db = 0; db < NDB; ++db)  // a slot never written may hold anything: masked
            vop[db] = mask_slots(*(const bf16x8*)(vhead + lay.v_chunk_off(kc, 16 * db + row)), k0 + 4 * g, pos_last);
        }
        const uint32_t* wr = wts + (h * TQ + row) * W_LD;
        const u32x4 w0 = *(const u32x4*)(wr + 4 * g), w1 = *(const u32x4*)(wr + 16 + 4 * g);
        u32x4 hi, lo;  // eight bfloat16 each: keys 4g..4g+3 and 16+4g..16+4g+3
        hi[0] = (w0[0] >> 16) | (w0[1] & 0xffff0000u);
        hi[1] = (w0[2] >> 16) | (w0[3] & 0xffff0000u);
        hi[2] = (w1[0] >> 16) | (w1[1] & 0xffff0000u);
        hi[3] = (w1[2] >> 16) | (w1[3] & 0xffff0000u);
        lo[0] = (w0[0] & 0xffffu) | (w0[1] << 16);
        lo[1] = (w0[2] & 0xffffu) | (w0[3] << 16);
        lo[2] = (w1[0] & 0xffffu) | (w1[1] << 16);
        lo[3] = (w1[2] & 0xffffu) | (w1[3] << 16);
        const bf16x8 p_hi = __builtin_bit_cast(bf16x8, hi), p_lo = __builtin_bit_cast(bf16x8, lo);
#pragma unroll
        for (int db = 0; db < NDB; ++db) {
          o[j][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vop[db], p_hi, o[j][db], 0, 0, 0);
          o[j][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vop[db], p_lo, o[j][db], 0, 0, 0);
        }
      }
    }
  }
  // ---- this lane's sums: token `row`, dimensions 16 db + 4 g + i of its wave's heads
  if (!row_valid) return;
  const int t = tok0 + row;
  const int n_items = H * a.e;
#pragma unroll
  for (int j = 0; j < HPW; ++j) {
    const int h = wave * HPW + j;
    if (h >= H) continue;
    float gate = 1.f;
    if (!a.partial && a.gate) gate = 1.f / (1.f + expf(-a.gate[(size_t)t * a.gate_stride + h]));
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int dim = 16 * db + 4 * g + i;
        if (dim < a.e) {
          if (a.partial) a.partial[((size_t)chunk * a.n_tokens + t) * n_items + h * a.e + dim] = o[j][db][i];
          else a.out[(size_t)t * a.out_stride + h * a.e + dim] = from_f<bf16_t>(o[j][db][i] * gate);
        }
      }
  }
}

// out[t, x] = (sum over the token's chunks, in order) * sigmoid(gate[t, head]); a thread an element
__global__ __launch_bounds__(ST_THREADS) void sigmoid_tile_combine_kernel(const SigmoidTileArgs a) {
  const int t = blockIdx.x;
  const int n_items = a.n_heads * a.e;
  const int x = blockIdx.y * ST_THREADS + threadIdx.x;
  if (x >= n_items) return;
  const int last_chunk = a.positions[t] / a.chunk_keys;
  const size_t step = (size_t)a.n_tokens * n_items;
  const float* p = a.partial + (size_t)t * n_items + x;
  float y = 0.f;
  int c = 0;
  for (; c + 4 <= last_chunk + 1; c += 4) {  // four loads in flight, added in order
    const float p0 = p[c * step], p1 = p[(c + 1) * step], p2 = p[(c + 2) * step], p3 = p[(c + 3) * step];
    y += p0; y += p1; y += p2; y += p3;
  }
  for (; c <= last_chunk; ++c) y += p[c * step];
  if (a.gate) y *= 1.f / (1.f + expf(-a.gate[(size_t)t * a.gate_stride + x / a.e]));
  a.out[(size_t)t * a.out_stride + x] = from_f<bf16_t>(y);
}

extern "C" int fg_sigmoid_tile_head_dim() { return HD; }

extern "C" int fg_sigmoid_attention_tiles(const SigmoidTileArgs* args, hipStream_t stream) {
  const SigmoidTileArgs& a = *args;
  if (a.n_items <= 0 || a.n_tokens <= 0) return FG_OK;
  if (a.n_heads <= 0 || a.n_heads > HP || a.n_kv <= 0 || a.n_heads % a.n_kv || a.d <= 0 || a.d > HD || a.e <= 0 ||
      a.e > HD || a.page_size <= 0 || a.page_size % 32 || a.n_dist < 1 || a.chunk_keys < KT || a.chunk_keys % KT ||
      a.n_chunks < 1 || a.n_chunks > 65535 || (a.n_chunks > 1 && !a.partial) || !a.q || !a.out || !a.k_pages || !a.v_pages ||
      !a.items || !a.positions || !a.talk || !a.mixed || ((uintptr_t)a.items & 15) || ((uintptr_t)a.mixed & 15))
    return FG_ERR_ARG;
  const size_t lds = (size_t)HP * KT * RAW_LD * sizeof(float) + (size_t)HP * TQ * W_LD * sizeof(uint32_t);
  dim3 grid(a.n_items, a.n_chunks);
  const int hpw = (a.n_heads + 3) / 4;
#define GO1(HPW, KV1)                                                                                                 \
  do {                                                                                                                \
    if (hipFuncSetAttribute((const void*)sigmoid_tile_kernel<HPW, KV1>, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) \
      return FG_ERR_LAUNCH;                                                                                           \
    sigmoid_tile_kernel<HPW, KV1><<<grid, ST_THREADS, lds, stream>>>(a);                                             \
  } while (0)
#define GO(HPW)                                       \
  do {                                                \
    if ((a.n_heads / a.n_kv) % HPW == 0) GO1(HPW, true); \
    else GO1(HPW, false);                             \
  } while (0)
  if (hpw == 1) GO(1);
  else if (hpw == 2) GO(2);
  else GO(4);
#undef GO
#undef GO1
  if (a.partial)
    sigmoid_tile_combine_kernel<<<dim3(a.n_tokens, (a.n_heads * a.e + ST_THREADS - 1) / ST_THREADS), ST_THREADS, 0, stream>>>(a);
  return fg_launch_status();
}
