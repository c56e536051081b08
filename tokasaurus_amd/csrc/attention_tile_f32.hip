// Paged attention in 32-bit arithmetic on the matrix cores (v_mfma_f32_16x16x4_f32): scores,
// softmax weights and the weighted values are 32-bit products of 32-bit operands, whatever the
// storage type of queries, keys and values.  For mixers that ask for exactly that: a sliding
// window, key and value heads of different sizes, a scale of the model's choosing and a
// learned sink per query head in the softmax's denominator; or, with `score_bias` (one number a
// query head), no softmax at all: a visible key's weight is sigmoid(score + score_bias[head]), not
// normalised over the keys (the sums of wavefronts and chunks are then added as they are).
//
// A wavefront owns a tile of 16 "columns": tt = 16 / gg neighbouring tokens of one request
// times gg neighbouring query heads of one kv head (gg = 1 for prompt portions; up to 16 for
// single decoded tokens, so that the heads that share keys share their loads).  It walks the
// keys in steps of 16, at absolute multiples of 16, from the first step that its earliest
// column sees to the last that its latest column sees:
//   S^T = K Q^T       keys as the first operand: a lane then holds, for its column (lane % 16),
//                     the scores of keys 4 * (lane / 16) + i, i < 4
//   O^T += V^T P^T    which is exactly its second operand here (the order of the sum over the
//                     16 keys is a free choice: slot lane / 16 of product i is key 4 * (lane / 16) + i)
// The sum over a head's elements is permuted the same way: a lane loads whole 8-element pieces
// of its key (the page layout's unit) and of its query, piece lane / 16 + 4 m.
//   K pages: [page][kv head][dk / 8][P][8]    V pages: [page][kv head][P / 4][dv][4]
// Needs dk % 8 == 0, dv % 16 == 0, P % 16 == 0 (a step of 16 keys lies inside one page).
#include "common.h"

typedef float v4f __attribute__((ext_vector_type(4)));
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;

// Scores from bfloat16 storage: the product of two bfloat16 numbers is exact in 32-bit, so the matrix cores'
// bfloat16 product with 32-bit sums (v_mfma_f32_16x16x32_bf16) gives 32-bit scores of the stored queries and keys
// like the 32-bit product of the converted operands, at an eighth of the instructions and without the conversions.
// Its operands are what a lane holds anyway: 8 neighbouring elements of key lane % 16 (of the column's query) from
// element 8 * (lane / 16) of every 32 on.  The weighted values stay 32-bit products: the weights are 32-bit numbers.
template <typename T>
struct ScoresFromStorage { static constexpr bool value = false; };
template <>
struct ScoresFromStorage<bf16_t> { static constexpr bool value = true; };
template <typename R>
__device__ __forceinline__ bf16x8_t as_bf16x8(const R& raw) {
  bf16x8_t v;
  __builtin_memcpy(&v, &raw, sizeof(v));
  return v;
}

#define AT_WAVES 4
#define AT_MAX_KM 8   // dk <= 256
#define AT_MAX_VT 16  // dv <= 256

// 8 (4) neighbouring elements of the storage type, moved as one: what a lane loads of a key (of the values)
template <typename T>
struct __align__(16) Raw8 { T v[8]; };
template <typename T>
struct __align__(sizeof(T) * 4) Raw4 { T v[4]; };

// What may follow the weighted sum of the values before it is stored, for mixers whose values were turned by their own
// positions and whose heads have a gate: pair m of a head's result is turned back by -position * vfreq[m] (pairs
// (m, m + dv/2) with `pair_half`, which the launch takes only where dv is 16 times the kernel's VT, and (2m, 2m + 1)
// without), then the head is multiplied by sigmoid(gate[token][head]).  Null pointers: nothing of the kind.
template <typename T>
struct AfterSum {
  const float* vfreq;
  int pair_half;
  const T* gate;
  int gate_stride;
};
__device__ __forceinline__ void turn_back(float& u, float& v, float pos, float freq) {
  float sn, cs;
  sincosf(__fmul_rn(pos, freq), &sn, &cs);
  rotate_pair(u, v, cs, -sn, u, v);
}
template <typename T>
__device__ __forceinline__ float gate_of(const AfterSum<T>& after, int tok, int head) {
  return after.gate ? 1.0f / (1.0f + expf(-to_f32<T>(after.gate[(size_t)tok * after.gate_stride + head]))) : 1.f;
}

// What may happen to a score between the scaling and the softmax, for mixers that ask for it: a soft cap
// (score <- cap * tanh(score / cap), cap > 0) and then a learned bias by distance, rel[bucket][head] with
// bucket = bucket_of[min(query position - key position, far)] (a table that the host made).
struct ScoreShape {
  float softcap;
  const int* bucket_of;
  int far;
  const float* rel;
};
__device__ __forceinline__ float shaped_score(const ScoreShape& sh, float s, int dist, int head, int nq) {
  if (sh.softcap > 0.f) s = sh.softcap * tanhf(s / sh.softcap);
  if (sh.rel) s += sh.rel[(size_t)sh.bucket_of[min(max(dist, 0), sh.far)] * nq + head];
  return s;
}

// SPLIT: the NW wavefronts of a workgroup share one tile and take its key steps in turn
// (wavefront w the steps w, w + NW, ..); they add up through LDS, always in wavefront order.
// For steps of few tiles (single decoded tokens), whose walks would else be one long chain each.
//
// PART (with SPLIT): the keys are also cut into chunks of `chunk` keys at absolute multiples of it, a workgroup a
// (tile, head block, chunk): blockIdx.z names the chunk.  A workgroup leaves its maxima, sums and weighted values
// unnormalised in `part`; attention_tile_merge_kernel adds the chunks in ascending order.  For single decoded
// tokens after long contexts, where a tile's walk would else keep one workgroup busy and the chip idle.
template <typename T, int KM, int VT, bool SPLIT, int NW, bool PART = false>
__global__ __launch_bounds__(NW * TK_WAVE) void attention_tile_f32_kernel(
    const T* __restrict__ q, int q_stride, T* __restrict__ out, int out_stride, const T* __restrict__ kcache,
    const T* __restrict__ vcache, const int* __restrict__ block_table, int table_stride,
    const int* __restrict__ q_start, const int* __restrict__ kv_len, const int* __restrict__ tile_req,
    const int* __restrict__ tile_row0, int nq, int nkv, int dk, int dv, int P, int window, float scale,
    const float* __restrict__ sink, const float* __restrict__ score_bias, int gg, AfterSum<T> after, ScoreShape shape,
    int chunk = 0, float* __restrict__ part = nullptr) {
  extern __shared__ float merge[];  // SPLIT: [waves][16] maxima, [waves][16] sums, [waves - 1][VT][4][64] weighted values
  const int lane = threadIdx.x & (TK_WAVE - 1), wave = threadIdx.x / TK_WAVE;
  const int group = nq / nkv;
  const int blocks_per_kv = group / gg;  // head blocks of gg heads
  const int hb = SPLIT ? blockIdx.y : blockIdx.y * NW + wave;
  if (hb >= nkv * blocks_per_kv) return;
  const int kvh = hb / blocks_per_kv;
  const int head0 = kvh * group + (hb % blocks_per_kv) * gg;
  const int tile = blockIdx.x;
  const int r = tile_req[tile];
  const int row0 = tile_row0[tile];
  const int tt = 16 / gg;
  const int col = lane & 15, c = lane >> 4;
  // this lane's column: a token and a query head
  const int tok = row0 + col / gg;
  const int head = head0 + col % gg;
  const int q_end = q_start[r + 1];
  const int kv = kv_len[r];
  const bool live = tok < q_end;
  const int n_tok = min(tt, q_end - row0);
  const int pos0 = kv - (q_end - row0);         // position of the tile's first token
  const int pos = pos0 + col / gg;              // of this column's token
  const int last_all = pos0 + n_tok - 1;  // the last key any column of the tile sees
  // (PART) this workgroup's chunk: with a window the launch holds only as many chunks as a window touches, and
  // blockIdx.z counts from the chunk of the first key that the tile sees (absolute multiples of `chunk` all the same)
  const int first_seen = window > 0 ? max(0, pos0 - window + 1) : 0;
  const int zc = PART ? first_seen / chunk + (int)blockIdx.z : 0;
  const int last = PART ? min(last_all, (zc + 1) * chunk - 1) : last_all;  // the last this workgroup walks
  const int lo_tile = max(first_seen, PART ? zc * chunk : 0);
  const int* table = block_table + (size_t)r * table_stride;
  const int pieces = dk / 8;
  const size_t key_page = key_page_elems(P, dk);

  // the column's query, piece c + 4 m (as stored, for scores from storage; else as 32-bit numbers)
  constexpr bool STORED = ScoresFromStorage<T>::value;
  float qv[STORED ? 1 : KM][8];
  Raw8<T> qraw[STORED ? KM : 1];
#pragma unroll
  for (int m = 0; m < KM; ++m) {
    const int piece = c + 4 * m;
    const bool in = live && piece < pieces;
    const T* src = q + (size_t)(in ? tok : 0) * q_stride + (size_t)head * dk + (in ? piece : 0) * 8;
    if constexpr (STORED) {
#pragma unroll
      for (int e = 0; e < 8; ++e) qraw[m].v[e] = in ? src[e] : from_f32<T>(0.f);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) qv[m][e] = in ? to_f32<T>(src[e]) : 0.f;
    }
  }

  v4f o[VT];
#pragma unroll
  for (int t = 0; t < VT; ++t) o[t] = (v4f){0.f, 0.f, 0.f, 0.f};
  const bool sig = score_bias != nullptr;
  const bool shaped = shape.softcap > 0.f || shape.rel != nullptr;
  const float pb = sig && live ? score_bias[head] : 0.f;
  // (sigmoid weights have no maximum to follow: it stays 0, so every merge below multiplies by exp(0))
  float m_run = sig ? 0.f : -INFINITY, l_run = 0.f;  // l_run: this lane's share of the column's sum

  // where this lane's pieces of a key and its values lie inside a page, for the page's first key: both offsets
  // grow linearly with the key's place in the page (8 elements a key, dv a key)
  int koff[KM], voff[VT];
#pragma unroll
  for (int m = 0; m < KM; ++m) koff[m] = (int)key_offset(P, col, (c + 4 * m < pieces ? c + 4 * m : 0) * 8);
#pragma unroll
  for (int t = 0; t < VT; ++t) voff[t] = (int)value_offset(dv, 4 * c, 16 * t < dv ? 16 * t + col : 0);
  const int step = SPLIT ? 16 * NW : 16;
  int k0 = (lo_tile / 16) * 16 + (SPLIT ? 16 * wave : 0);
  // The pages of this wavefront's steps, 64 steps at a time: lane j asks for the page of step `base + j`, and a
  // step reads its page's number from that lane.  So no load of keys or values waits for a load of a page number.
  const int k_first = k0;
  int pv = 0;
#define AT_PAGES(BASE)                                                  \
  do {                                                                  \
    const int kj = k_first + ((BASE) + lane) * step;                    \
    pv = kj <= last ? max(table[kj / P], 0) : 0;                        \
  } while (0)
  AT_PAGES(0);
  // this lane's pieces of key k0 + col and its values (element 16 t + col of keys k0 + 4 c + i); the keys are
  // asked for a step ahead, and (SPLIT, where nothing else hides the wait) the values too
  Raw8<T> kr[KM];
  Raw4<T> vr[VT];
  if (k0 <= last) {
    const int page = __builtin_amdgcn_readlane(pv, 0);
    const T* kbase = kcache + ((size_t)page * nkv + kvh) * key_page + (k0 % P) * 8;
#pragma unroll
    for (int m = 0; m < KM; ++m) kr[m] = *(const Raw8<T>*)(kbase + koff[m]);
    if constexpr (SPLIT) {
      const T* vbase = vcache + ((size_t)page * nkv + kvh) * P * dv + (k0 % P) * dv;
#pragma unroll
      for (int t = 0; t < VT; ++t)
        if (16 * t < dv) vr[t] = *(const Raw4<T>*)(vbase + voff[t]);
    }
  }
  int j = 0;
#pragma unroll 1
  for (; k0 <= last; k0 += step, ++j) {
    if constexpr (!SPLIT) {
      const int page = __builtin_amdgcn_readlane(pv, j & 63);
      const T* vbase = vcache + ((size_t)page * nkv + kvh) * P * dv + (k0 % P) * dv;
#pragma unroll
      for (int t = 0; t < VT; ++t)
        if (16 * t < dv) vr[t] = *(const Raw4<T>*)(vbase + voff[t]);
    }
    Raw8<T> kn[KM];
    Raw4<T> vn[VT];
    const int k1 = k0 + step;
    if (k1 <= last) {
      if (((j + 1) & 63) == 0) AT_PAGES(j + 1);
      const int page1 = __builtin_amdgcn_readlane(pv, (j + 1) & 63);
      const T* kbase = kcache + ((size_t)page1 * nkv + kvh) * key_page + (k1 % P) * 8;
#pragma unroll
      for (int m = 0; m < KM; ++m) kn[m] = *(const Raw8<T>*)(kbase + koff[m]);
      if constexpr (SPLIT) {
        const T* vbase = vcache + ((size_t)page1 * nkv + kvh) * P * dv + (k1 % P) * dv;
#pragma unroll
        for (int t = 0; t < VT; ++t)
          if (16 * t < dv) vn[t] = *(const Raw4<T>*)(vbase + voff[t]);
      }
    }
    // S^T = K Q^T (a piece beyond the head's size meets zeros of the query)
    v4f s = (v4f){0.f, 0.f, 0.f, 0.f};
    if constexpr (STORED) {
#pragma unroll
      for (int m = 0; m < KM; ++m)
        s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kr[m]), as_bf16x8(qraw[m]), s, 0, 0, 0);
    } else {
#pragma unroll
      for (int m = 0; m < KM; ++m)
#pragma unroll
        for (int e = 0; e < 8; ++e)
          s = __builtin_amdgcn_mfma_f32_16x16x4f32(to_f32<T>(kr[m].v[e]), qv[m][e], s, 0, 0, 0);
    }
    // this lane now holds, for its column, keys k0 + 4 c + i
    float sc[4];
    float tmax = -INFINITY;
    // a step that every column of the tile sees whole needs no masks (the same for all lanes)
    const bool whole = k0 + 15 <= pos0 && (window <= 0 || last_all - k0 < window) && n_tok * gg == 16;
    if (whole) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        sc[i] = s[i] * scale;
        if (shaped) sc[i] = shaped_score(shape, sc[i], pos - (k0 + 4 * c + i), head, nq);
        tmax = fmaxf(tmax, sc[i]);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int kp = k0 + 4 * c + i;
        const bool seen = live && kp <= pos && (window <= 0 || pos - kp < window);
        sc[i] = seen ? (shaped ? shaped_score(shape, s[i] * scale, pos - kp, head, nq) : s[i] * scale) : -INFINITY;
        tmax = fmaxf(tmax, sc[i]);
      }
    }
    float p[4];
    float alpha = 1.f;
    if (sig) {
      // 1 / (1 + exp(-(score + bias))); a masked score gives 1 / (1 + inf) = 0
#pragma unroll
      for (int i = 0; i < 4; ++i) p[i] = 1.0f / (1.0f + exp2f(-(sc[i] + pb) * 1.44269504088896341f));
    } else {
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, TK_WAVE));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, TK_WAVE));
      const float m_new = fmaxf(m_run, tmax);
      if (m_new == -INFINITY) {
#pragma unroll
        for (int i = 0; i < 4; ++i) p[i] = 0.f;
      } else {
        // exp2 of the difference times log2(e): the hardware's own exponential (a masked score gives exp2(-inf) = 0)
        alpha = exp2f((m_run - m_new) * 1.44269504088896341f);
#pragma unroll
        for (int i = 0; i < 4; ++i) p[i] = exp2f((sc[i] - m_new) * 1.44269504088896341f);
      }
      m_run = m_new;
      l_run = l_run * alpha + ((p[0] + p[1]) + (p[2] + p[3]));
    }
    // O^T += V^T P^T
#pragma unroll
    for (int t = 0; t < VT; ++t) {
      if (16 * t < dv) {
        v4f acc = o[t] * alpha;
#pragma unroll
        for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(to_f32<T>(vr[t].v[i]), p[i], acc, 0, 0, 0);
        o[t] = acc;
      }
    }
#pragma unroll
    for (int m = 0; m < KM; ++m) kr[m] = kn[m];
    if constexpr (SPLIT) {
#pragma unroll
      for (int t = 0; t < VT; ++t) vr[t] = vn[t];
    }
  }
#undef AT_PAGES
  // the column's sum, from the four lanes that share it (always in this order)
  float l = l_run;
  l += __shfl_xor(l, 16, TK_WAVE);
  l += __shfl_xor(l, 32, TK_WAVE);
  if constexpr (SPLIT) {
    float* sm = merge;
    float* sl = merge + NW * 16;
    float* so = merge + 2 * NW * 16;
    if (c == 0) {
      sm[wave * 16 + col] = m_run;
      sl[wave * 16 + col] = l;
    }
    // (the first wavefront adds the others' sums to its own, which never leave its registers)
    if (wave > 0) {
#pragma unroll
      for (int t = 0; t < VT; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) so[(((wave - 1) * VT + t) * 4 + i) * TK_WAVE + lane] = o[t][i];
    }
    __syncthreads();
    if (wave != 0) return;
    float m_all = -INFINITY;
#pragma unroll
    for (int w = 0; w < NW; ++w) m_all = fmaxf(m_all, sm[w * 16 + col]);
    l = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float mw = sm[w * 16 + col];
      const float f = (mw == -INFINITY) ? 0.f : expf(mw - m_all);
      l = fmaf(sl[w * 16 + col], f, l);
      if (w == 0) {
#pragma unroll
        for (int t = 0; t < VT; ++t) o[t] = o[t] * f;
      } else {
#pragma unroll
        for (int t = 0; t < VT; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) o[t][i] = fmaf(so[(((w - 1) * VT + t) * 4 + i) * TK_WAVE + lane], f, o[t][i]);
      }
    }
    m_run = m_all;
  }
  if constexpr (PART) {
    // [tile][head block][chunk]: 16 maxima, 16 sums, [VT][4][64] weighted values as the lanes hold them
    const size_t unit = 32 + (size_t)VT * 4 * TK_WAVE;
    float* dst = part + (((size_t)tile * gridDim.y + blockIdx.y) * gridDim.z + blockIdx.z) * unit;
    if (c == 0) {
      dst[col] = m_run;
      dst[16 + col] = l;
    }
#pragma unroll
    for (int t = 0; t < VT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) dst[32 + (t * 4 + i) * TK_WAVE + lane] = o[t][i];
    return;
  }
  float keep = 1.f;
  if (sink && live && !sig) {
    // the sink joins the softmax like one more score: the maximum may rise to it
    const float sk = sink[head], m_all = fmaxf(m_run, sk);
    keep = (m_run == -INFINITY) ? 0.f : expf(m_run - m_all);
    l = l * keep + expf(sk - m_all);
  }
  if (!live) return;
  const float inv = sig ? 1.f : keep / l;
#pragma unroll
  for (int t = 0; t < VT; ++t) o[t] = o[t] * inv;
  if (after.vfreq) {
    const float fp = (float)pos;
    if (after.pair_half) {  // dv == 16 VT: element 16 t + 4 c + i meets the one of block t + VT / 2
#pragma unroll
      for (int t = 0; t < VT / 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float u = o[t][i], v = o[t + VT / 2][i];
          turn_back(u, v, fp, after.vfreq[16 * t + 4 * c + i]);
          o[t][i] = u;
          o[t + VT / 2][i] = v;
        }
    } else {
#pragma unroll
      for (int t = 0; t < VT; ++t)
        if (16 * t < dv) {
#pragma unroll
          for (int i = 0; i < 4; i += 2) {
            float u = o[t][i], v = o[t][i + 1];
            turn_back(u, v, fp, after.vfreq[(16 * t + 4 * c + i) / 2]);
            o[t][i] = u;
            o[t][i + 1] = v;
          }
        }
    }
  }
  const float g = gate_of(after, tok, head);
  T* dst = out + (size_t)tok * out_stride + (size_t)head * dv;
#pragma unroll
  for (int t = 0; t < VT; ++t) {
    if (16 * t < dv) {
#pragma unroll
      for (int i = 0; i < 4; ++i) dst[16 * t + 4 * c + i] = from_f32<T>(o[t][i] * g);
    }
  }
}

// A workgroup a (tile, head block), a wavefront a block of 16 value elements: the chunks' partial results added in
// ascending order, then the sink and the division, with the lanes' places as in the kernel above.
template <typename T, int VT>
__global__ __launch_bounds__(VT * TK_WAVE) void attention_tile_merge_kernel(
    const float* __restrict__ part, int chunks, T* __restrict__ out, int out_stride, const int* __restrict__ q_start,
    const int* __restrict__ tile_req, const int* __restrict__ tile_row0, int nq, int nkv, int dv,
    const float* __restrict__ sink, int gg, int plain_sums, const int* __restrict__ kv_len, AfterSum<T> after) {
  __shared__ float ex[VT * TK_WAVE * 4];  // the wavefronts' results, where the halves of a head are turned back
  const int lane = threadIdx.x & (TK_WAVE - 1), t = threadIdx.x / TK_WAVE;
  if (16 * t >= dv) return;  // (never with halves to turn back: dv is 16 VT then, and every wavefront reaches the barrier)
  const int group = nq / nkv, blocks_per_kv = group / gg;
  const int hb = blockIdx.y, tile = blockIdx.x;
  const int head0 = (hb / blocks_per_kv) * group + (hb % blocks_per_kv) * gg;
  const int col = lane & 15, c = lane >> 4;
  const int tok = tile_row0[tile] + col / gg, head = head0 + col % gg;
  const bool live = tok < q_start[tile_req[tile] + 1];
  const size_t unit = 32 + (size_t)VT * 4 * TK_WAVE;
  const float* src = part + ((size_t)tile * gridDim.y + hb) * chunks * unit;
  float m_all = -INFINITY;
#pragma unroll 8
  for (int z = 0; z < chunks; ++z) m_all = fmaxf(m_all, src[z * unit + col]);
  float l = 0.f;
  v4f o = (v4f){0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
  for (int z = 0; z < chunks; ++z) {
    const float mz = src[z * unit + col];
    const float lz = src[z * unit + 16 + col];
    v4f oz;
#pragma unroll
    for (int i = 0; i < 4; ++i) oz[i] = src[z * unit + 32 + (t * 4 + i) * TK_WAVE + lane];
    // a chunk none of whose keys this column sees (maximum -inf, sums zero) adds nothing
    const float f = (mz == -INFINITY) ? 0.f : expf(mz - m_all);
    l = fmaf(lz, f, l);
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = fmaf(oz[i], f, o[i]);
  }
  float keep = 1.f;
  if (sink && live && !plain_sums) {
    const float sk = sink[head], m2 = fmaxf(m_all, sk);
    keep = (m_all == -INFINITY) ? 0.f : expf(m_all - m2);
    l = l * keep + expf(sk - m2);
  }
  const float inv = !live ? 0.f : (plain_sums ? 1.f : keep / l);  // (sigmoid weights: every chunk's maximum is 0 and its sums count as they are)
  float r[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) r[i] = live ? o[i] * inv : 0.f;
  if (after.vfreq) {
    const int req = tile_req[tile];
    const float fp = live ? (float)(kv_len[req] - (q_start[req + 1] - tok)) : 0.f;
    if (after.pair_half) {
#pragma unroll
      for (int i = 0; i < 4; ++i) ex[(t * TK_WAVE + lane) * 4 + i] = r[i];
      __syncthreads();
      const bool low = t < VT / 2;
      const int other = low ? t + VT / 2 : t - VT / 2;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float u = low ? r[i] : ex[(other * TK_WAVE + lane) * 4 + i];
        float v = low ? ex[(other * TK_WAVE + lane) * 4 + i] : r[i];
        turn_back(u, v, fp, after.vfreq[16 * (low ? t : other) + 4 * c + i]);
        r[i] = low ? u : v;
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; i += 2) turn_back(r[i], r[i + 1], fp, after.vfreq[(16 * t + 4 * c + i) / 2]);
    }
  }
  if (!live) return;
  const float g = gate_of(after, tok, head);
  T* dst = out + (size_t)tok * out_stride + (size_t)head * dv;
#pragma unroll
  for (int i = 0; i < 4; ++i) dst[16 * t + 4 * c + i] = from_f32<T>(r[i] * g);
}

// Whether this kernel takes the shape (else the caller uses the plain 32-bit kernel).
TK_API int tk_attention_tile_f32_fits(int nq, int nkv, int dk, int dv, int P) {
  return (nq > 0 && nkv > 0 && nq % nkv == 0 && dk > 0 && dk % 8 == 0 && dk <= 32 * AT_MAX_KM && dv > 0 && dv % 16 == 0 &&
          dv <= 16 * AT_MAX_VT && P > 0 && P % 16 == 0) ? 1 : 0;
}

// Whether the kernel can turn back the halves of a value head of dv elements itself: the two elements of a pair lie in
// one lane where the head fills the kernel's blocks of 16 (dv is 16 times 2, 4, 8 or 16).
TK_API int tk_attention_tile_turns_halves(int dv) { return (dv == 32 || dv == 64 || dv == 128 || dv == 256) ? 1 : 0; }

// 32-bit words of `part` that a (tile, head block, chunk) takes for a value head of dv elements
TK_API int tk_attention_tile_part_words(int dv) {
  const int vt = dv / 16;
  const int VT = vt <= 2 ? 2 : (vt <= 4 ? 4 : (vt <= 8 ? 8 : 16));
  return 32 + VT * 4 * TK_WAVE;
}

template <typename T, int KM, int VT>
static void at_launch(dim3 grid, bool split, hipStream_t stream, const void* q, int q_stride, void* out, int out_stride,
                      const void* kcache, const void* vcache, const int* block_table, int table_stride,
                      const int* q_start, const int* kv_len, const int* tile_req, const int* tile_row0, int nq,
                      int nkv, int dk, int dv, int P, int window, float scale, const float* sink, const float* score_bias,
                      int gg, int chunk, float* part, const float* vfreq, int v_pair_half, const void* gate, int gate_stride,
                      ScoreShape shape) {
  // halves of a head meet inside a lane only where the head fills the kernel's blocks of 16 (the entry point has checked)
  const AfterSum<T> after = {vfreq, v_pair_half, (const T*)gate, gate_stride};
  const AfterSum<T> none = {nullptr, 0, nullptr, 0};
  if (split && chunk > 0) {
    constexpr int NW = VT <= 4 ? 8 : 4;
    const size_t smem = sizeof(float) * (NW * 32 + (size_t)(NW - 1) * VT * 4 * TK_WAVE);
    hipLaunchKernelGGL((attention_tile_f32_kernel<T, KM, VT, true, NW, true>), grid, dim3(NW * TK_WAVE), smem, stream,
                       (const T*)q, q_stride, (T*)out, out_stride, (const T*)kcache, (const T*)vcache, block_table,
                       table_stride, q_start, kv_len, tile_req, tile_row0, nq, nkv, dk, dv, P, window, scale, sink, score_bias, gg,
                       none, shape, chunk, part);
    hipLaunchKernelGGL((attention_tile_merge_kernel<T, VT>), dim3(grid.x, grid.y), dim3(VT * TK_WAVE), 0, stream, part, (int)grid.z,
                       (T*)out, out_stride, q_start, tile_req, tile_row0, nq, nkv, dv, sink, gg, score_bias ? 1 : 0, kv_len, after);
  } else if (split) {
    // eight wavefronts a tile where their sums fit the local memory, else four
    constexpr int NW = VT <= 4 ? 8 : 4;
    const size_t smem = sizeof(float) * (NW * 32 + (size_t)(NW - 1) * VT * 4 * TK_WAVE);
    hipLaunchKernelGGL((attention_tile_f32_kernel<T, KM, VT, true, NW>), grid, dim3(NW * TK_WAVE), smem, stream,
                       (const T*)q, q_stride, (T*)out, out_stride, (const T*)kcache, (const T*)vcache, block_table,
                       table_stride, q_start, kv_len, tile_req, tile_row0, nq, nkv, dk, dv, P, window, scale, sink, score_bias, gg, after, shape);
  } else {
    hipLaunchKernelGGL((attention_tile_f32_kernel<T, KM, VT, false, AT_WAVES>), grid, dim3(AT_WAVES * TK_WAVE), 0, stream,
                       (const T*)q, q_stride, (T*)out, out_stride, (const T*)kcache, (const T*)vcache, block_table,
                       table_stride, q_start, kv_len, tile_req, tile_row0, nq, nkv, dk, dv, P, window, scale, sink, score_bias, gg, after, shape);
  }
}

// split: the wavefronts of a workgroup share a tile's keys (see the kernel); the caller chooses it for steps of few
// tiles.  It changes the order in which a token's keys are added up, nothing else.
TK_API int tk_attention_tile_f32(int dt, const void* q, int q_stride, void* out, int out_stride, const void* kcache,
                                 const void* vcache, const int* block_table, int table_stride, const int* q_start,
                                 const int* kv_len, const int* tile_req, const int* tile_row0, int n_tiles, int nq,
                                 int nkv, int dk, int dv, int P, int window, float scale, const float* sink,
                                 const float* score_bias, int gg, int split, int chunk, int chunks, float* part,
                                 const float* vfreq, int v_pair_half, const void* gate, int gate_stride, float softcap,
                                 const int* bucket_of, int far, const float* rel, hipStream_t stream) {
  TK_REQUIRE(!rel || (bucket_of && far >= 0), "attention_tile_f32: a bias by distance needs its table of buckets");
  TK_REQUIRE(!(score_bias && (rel || softcap > 0.f)), "attention_tile_f32: sigmoid weights take neither a soft cap nor a bias by distance");
  const ScoreShape shape = {softcap, bucket_of, far, rel};
  TK_REQUIRE(tk_attention_tile_f32_fits(nq, nkv, dk, dv, P), "attention_tile_f32: shape nq=%d nkv=%d dk=%d dv=%d P=%d not taken",
             nq, nkv, dk, dv, P);
  const int group = nq / nkv;
  TK_REQUIRE(gg >= 1 && gg <= 16 && (gg & (gg - 1)) == 0 && group % gg == 0, "attention_tile_f32: %d heads a tile of a group of %d", gg, group);
  TK_REQUIRE(q_stride >= nq * dk && out_stride >= nq * dv, "attention_tile_f32: row strides too short");
  if (n_tiles <= 0) return 0;
  const int head_blocks = nkv * (group / gg);
  const int km = (dk + 31) / 32, vt = dv / 16;
  TK_REQUIRE(!vfreq || (dv % 2 == 0 && (!v_pair_half || tk_attention_tile_turns_halves(dv))),
             "attention_tile_f32: the halves of a value head of %d do not meet inside a lane", dv);
  TK_REQUIRE(!gate || gate_stride >= nq, "attention_tile_f32: gate rows of %d hold no %d heads", gate_stride, nq);
  const bool sp = split != 0;
  const bool parts = sp && chunk > 0;
  TK_REQUIRE(!parts || (chunk % 128 == 0 && chunks > 0 && chunks < 65536 && part), "attention_tile_f32: chunks of a multiple of 128 keys, "
             "their number and a place for their results");
  const dim3 grid(n_tiles, sp ? head_blocks : (head_blocks + AT_WAVES - 1) / AT_WAVES, parts ? chunks : 1);
  TK_REQUIRE(grid.y < 65536, "attention_tile_f32: too many heads");
#define AT_ARGS grid, sp, stream, q, q_stride, out, out_stride, kcache, vcache, block_table, table_stride, q_start, kv_len, \
                tile_req, tile_row0, nq, nkv, dk, dv, P, window, scale, sink, score_bias, gg, parts ? chunk : 0, part, vfreq, v_pair_half, \
                gate, gate_stride, shape
#define AT_VT(T, KMV)                                      \
  do {                                                     \
    if (vt <= 2) at_launch<T, KMV, 2>(AT_ARGS);            \
    else if (vt <= 4) at_launch<T, KMV, 4>(AT_ARGS);       \
    else if (vt <= 8) at_launch<T, KMV, 8>(AT_ARGS);       \
    else at_launch<T, KMV, 16>(AT_ARGS);                   \
  } while (0)
#define AT_KM(T)                       \
  do {                                 \
    if (km <= 1) AT_VT(T, 1);          \
    else if (km <= 2) AT_VT(T, 2);     \
    else if (km <= 4) AT_VT(T, 4);     \
    else AT_VT(T, 8);                  \
  } while (0)
  if (dt == TK_F32) AT_KM(float);
  else AT_KM(bf16_t);
#undef AT_KM
#undef AT_VT
#undef AT_ARGS
  TK_CHECK_LAUNCH("attention_tile_f32");
  return 0;
}
