// Between the q|k|v product and the attention, for mixers that norm queries and keys over
// the whole projection and rotate neighbouring elements: one kernel a step that
//   * divides a token's whole query row (all heads at once) by its root mean square and
//     multiplies by a weight of that size, and the same for its whole key row,
//   * rotates the leading `rot` elements of every head, element 2i with element 2i + 1, by the
//     angle position * freq[i] (32-bit product, 32-bit sine and cosine computed here: no table,
//     so positions have no upper end),
//   * writes the queries back in place, the keys and the values into the token's page.
// Options: query heads of a size `dq` of their own (a query latent normed as one row beside a
// key latent of another size); `pair_half`: the rotation pairs element i with element
// i + rot/2 instead of neighbours; `v_from_k`: the row holds no values, a token's values are
// its keys as they are before the rotation (normed and weighted when the keys are).
// `per_head`: the norms' statistics are taken head by head and the weights have a head's size (one
// weight vector for all query heads, one for all key heads).  `k_skip`: the leading k_skip elements of
// a key head are neither normed nor weighted, and with `v_from_k` the values are the dk - k_skip
// elements behind them (a latent beside a rotated key part that is no part of it).  `vfreq`: the values
// are turned too, every element of a head, pair m by position * vfreq[m], pairs (m, m + dv/2) with
// `v_pair_half` and (2m, 2m + 1) without.  `rot_scale`: cosine and sine of the queries' and keys'
// rotation are both multiplied by it (1: a plain rotation).
// The arithmetic is 32-bit from the product's rounded output to the one rounding at the store.
//   row: [nq*dq | nkv*dk | nkv*dv]  (only the first part when !write_cache; no third part with v_from_k)
//   K pages: [page][kv head][dk / 8][P][8]    V pages: [page][kv head][P / 4][dv][4]
#include "common.h"

// The work items of a head of size d of which the leading `rot` elements are rotated: item j names
// one or two elements (e0, and e1 when `two`) and, when `turned`, the angle they are rotated by.
struct PairItem {
  int e0, e1, angle;
  bool two, turned;
};
__device__ __forceinline__ int pair_items(int d, int rot, int pair_half) {
  return pair_half ? rot / 2 + (d - rot + 1) / 2 : (d + 1) / 2;
}
__device__ __forceinline__ PairItem pair_item(int j, int d, int rot, int pair_half) {
  PairItem it;
  if (pair_half && j < rot / 2) {
    it.e0 = j; it.e1 = j + rot / 2; it.angle = j; it.two = true; it.turned = true;
  } else {
    const int e = pair_half ? rot + 2 * (j - rot / 2) : 2 * j;
    it.e0 = e; it.e1 = e + 1; it.angle = e / 2; it.two = e + 1 < d; it.turned = !pair_half && e < rot;
  }
  return it;
}

template <typename T>
__global__ __launch_bounds__(256) void qk_prepare_kernel(
    T* __restrict__ qkv, int row_stride, const int* __restrict__ positions,
    const int* __restrict__ token_req, const int* __restrict__ block_table, int table_stride,
    const float* __restrict__ q_weight, const float* __restrict__ k_weight, float eps,
    const float* __restrict__ freq, T* __restrict__ kcache, T* __restrict__ vcache, int nq, int nkv,
    int dq, int dk, int dv, int rot, int P, int write_cache, int pair_half, int v_from_k, int per_head, int k_skip,
    const float* __restrict__ vfreq, int v_pair_half, float rot_scale) {
  extern __shared__ float cs[];  // [rot / 2] cosines, [rot / 2] sines, then (vfreq) [dv / 2] cosines, [dv / 2] sines, then (per_head) [nq + nkv] factors
  __shared__ float red[16];
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int half = rot / 2;
  T* row = qkv + (size_t)t * row_stride;
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    const float angle = __fmul_rn((float)pos, freq[i]);
    float s, c;
    sincosf(angle, &s, &c);
    cs[i] = c * rot_scale;  // (a rotation may come with a factor on cosine and sine alike)
    cs[half + i] = s * rot_scale;
  }
  float* vcs = cs + (rot > 0 ? rot : 2);
  float* head_r = vcs + (vfreq ? dv : 0);
  if (vfreq)
    for (int i = threadIdx.x; i < dv / 2; i += blockDim.x) {
      const float angle = __fmul_rn((float)pos, vfreq[i]);
      float s, c;
      sincosf(angle, &s, &c);
      vcs[i] = c;
      vcs[dv / 2 + i] = s;
    }
  const int nqe = nq * dq, nke = nkv * dk;
  float rq = 1.f, rk = 1.f;
  if (per_head) {
    // sixteen lanes a head: 1 / rms of the head's own elements (the key's behind k_skip)
    const int sub = threadIdx.x & 15, team = threadIdx.x >> 4, teams = blockDim.x >> 4;
    const int heads = nq + (write_cache ? nkv : 0);
    for (int h = team; h < heads; h += teams) {
      const bool is_q = h < nq;
      const T* src = is_q ? row + (size_t)h * dq : row + nqe + (size_t)(h - nq) * dk + k_skip;
      const int n = is_q ? dq : dk - k_skip;
      const bool normed = is_q ? q_weight != nullptr : k_weight != nullptr;
      float ss = 0.f;
      if (normed)
        for (int i = sub; i < n; i += 16) {
          const float v = to_f32<T>(src[i]);
          ss = fmaf(v, v, ss);
        }
#pragma unroll
      for (int o = 8; o > 0; o >>= 1) ss += __shfl_xor(ss, o, TK_WAVE);  // (stays inside the sixteen lanes)
      if (sub == 0) head_r[h] = normed ? 1.0f / sqrtf(ss / (float)n + eps) : 1.f;
    }
  } else if (q_weight) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < nqe; i += blockDim.x) {
      const float v = to_f32<T>(row[i]);
      ss = fmaf(v, v, ss);
    }
    rq = 1.0f / sqrtf(block_sum(ss, red) / (float)nqe + eps);
  }
  if (!per_head && write_cache && k_weight) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < nke; i += blockDim.x) {
      const float v = (i % dk) >= k_skip ? to_f32<T>(row[nqe + i]) : 0.f;
      ss = fmaf(v, v, ss);
    }
    rk = 1.0f / sqrtf(block_sum(ss, red) / (float)(nkv * (dk - k_skip)) + eps);
  }
  __syncthreads();  // the table of this token's angles is written

  // queries, in place, a pair a thread (a head of odd size ends in a single element)
  const int hq = pair_items(dq, rot, pair_half);
  for (int i = threadIdx.x; i < nq * hq; i += blockDim.x) {
    const PairItem it = pair_item(i % hq, dq, rot, pair_half);
    const int x0 = (i / hq) * dq + it.e0, x1 = (i / hq) * dq + it.e1;
    if (per_head) rq = head_r[i / hq];
    float u = to_f32<T>(row[x0]) * rq, v = it.two ? to_f32<T>(row[x1]) * rq : 0.f;
    if (q_weight) {
      u *= q_weight[per_head ? it.e0 : x0];
      if (it.two) v *= q_weight[per_head ? it.e1 : x1];
    }
    if (it.turned) rotate_pair(u, v, cs[it.angle], cs[half + it.angle], u, v);
    row[x0] = from_f32<T>(u);
    if (it.two) row[x1] = from_f32<T>(v);
  }
  if (!write_cache) return;

  const int page = block_table[(size_t)token_req[t] * table_stride + pos / P];
  const int p = pos % P;
  const T* krow = row + nqe;
  const T* vrow = krow + nke;
  const int hk = pair_items(dk, rot, pair_half);
  for (int i = threadIdx.x; i < nkv * hk; i += blockDim.x) {
    const int h = i / hk;
    const PairItem it = pair_item(i % hk, dk, rot, pair_half);
    const int x0 = h * dk + it.e0, x1 = h * dk + it.e1;
    if (per_head) rk = head_r[nq + h];
    // (pairs never straddle k_skip: it is even, and with halves it is either none or the rotated part)
    const bool normed = it.e0 >= k_skip;
    float u = to_f32<T>(krow[x0]), v = it.two ? to_f32<T>(krow[x1]) : 0.f;
    if (normed) {
      u *= rk;
      v *= rk;
      if (k_weight) {
        const int dn = dk - k_skip;
        u *= k_weight[per_head ? it.e0 - k_skip : h * dn + it.e0 - k_skip];
        if (it.two) v *= k_weight[per_head ? it.e1 - k_skip : h * dn + it.e1 - k_skip];
      }
    }
    if (v_from_k && normed) {  // the values are the keys as they are here, before the rotation
      T* vdst = vcache + ((size_t)page * nkv + h) * P * dv;
      vdst[value_offset(dv, p, it.e0 - k_skip)] = from_f32<T>(u);
      if (it.two) vdst[value_offset(dv, p, it.e1 - k_skip)] = from_f32<T>(v);
    }
    if (it.turned) rotate_pair(u, v, cs[it.angle], cs[half + it.angle], u, v);
    T* dst = kcache + ((size_t)page * nkv + h) * key_page_elems(P, dk);
    dst[key_offset(P, p, it.e0)] = from_f32<T>(u);
    if (it.two) dst[key_offset(P, p, it.e1)] = from_f32<T>(v);
  }
  if (v_from_k) return;
  if (vfreq) {  // every element of a value head is turned by the token's own position
    const int hv = dv / 2;
    for (int i = threadIdx.x; i < nkv * hv; i += blockDim.x) {
      const int h = i / hv, m = i % hv;
      const int e0 = v_pair_half ? m : 2 * m, e1 = v_pair_half ? m + hv : 2 * m + 1;
      float u = to_f32<T>(vrow[h * dv + e0]), v = to_f32<T>(vrow[h * dv + e1]);
      rotate_pair(u, v, vcs[m], vcs[hv + m], u, v);
      T* vdst = vcache + ((size_t)page * nkv + h) * P * dv;
      vdst[value_offset(dv, p, e0)] = from_f32<T>(u);
      vdst[value_offset(dv, p, e1)] = from_f32<T>(v);
    }
    return;
  }
  for (int i = threadIdx.x; i < nkv * dv; i += blockDim.x) {
    const int h = i / dv, e = i % dv;
    vcache[((size_t)page * nkv + h) * P * dv + value_offset(dv, p, e)] = vrow[i];
  }
}

TK_API int tk_qk_prepare(int dt, void* qkv, int row_stride, const int* positions, const int* token_req,
                         const int* block_table, int table_stride, const float* q_weight,
                         const float* k_weight, float eps, const float* freq, void* kcache, void* vcache,
                         int n_tokens, int nq, int nkv, int dq, int dk, int dv, int rot, int P, int write_cache,
                         int pair_half, int v_from_k, int per_head, int k_skip, const float* vfreq, int v_pair_half,
                         float rot_scale, hipStream_t stream) {
  TK_REQUIRE(n_tokens >= 0 && nq >= 0 && nkv >= 0 && nq + nkv > 0 && dq > 0 && dk > 0 && dv > 0 && P > 0,
             "qk_prepare: bad sizes tokens=%d nq=%d nkv=%d dq=%d dk=%d dv=%d P=%d", n_tokens, nq, nkv, dq, dk, dv, P);
  TK_REQUIRE(rot >= 0 && rot <= dk && rot <= dq && rot % 2 == 0, "qk_prepare: %d rotated elements of heads of %d and %d", rot, dq, dk);
  TK_REQUIRE(rot == 0 || freq, "qk_prepare: a rotation needs its frequencies");
  TK_REQUIRE(k_skip >= 0 && k_skip % 2 == 0 && k_skip < dk && (k_skip == 0 || !pair_half || k_skip == rot),
             "qk_prepare: %d leading elements of a key of %d left out of its norm", k_skip, dk);
  TK_REQUIRE(!v_from_k || dv == dk - k_skip, "qk_prepare: values that are the keys have the keys' size, not %d for %d", dv, dk - k_skip);
  TK_REQUIRE(!vfreq || (dv % 2 == 0 && !v_from_k), "qk_prepare: turned values have an even size and a projection of their own");
  TK_REQUIRE(row_stride >= (write_cache ? nq * dq + nkv * (dk + (v_from_k ? 0 : dv)) : nq * dq),
             "qk_prepare: row stride %d is shorter than the heads it holds", row_stride);
  TK_REQUIRE(!write_cache || (kcache && vcache && block_table && nkv > 0), "qk_prepare: cache pointers missing");
  if (n_tokens == 0) return 0;
  const size_t smem = sizeof(float) * (size_t)((rot > 0 ? rot : 2) + (vfreq ? dv : 0) + (per_head ? nq + nkv : 0));
  TK_REQUIRE(smem <= 48 * 1024, "qk_prepare: too many heads for one workgroup's local memory");
  if (dt == TK_F32)
    hipLaunchKernelGGL(qk_prepare_kernel<float>, dim3(n_tokens), dim3(256), smem, stream, (float*)qkv,
                       row_stride, positions, token_req, block_table, table_stride, q_weight, k_weight, eps,
                       freq, (float*)kcache, (float*)vcache, nq, nkv, dq, dk, dv, rot, P, write_cache, pair_half, v_from_k,
                       per_head, k_skip, vfreq, v_pair_half, rot_scale);
  else
    hipLaunchKernelGGL(qk_prepare_kernel<bf16_t>, dim3(n_tokens), dim3(256), smem, stream, (bf16_t*)qkv,
                       row_stride, positions, token_req, block_table, table_stride, q_weight, k_weight, eps,
                       freq, (bf16_t*)kcache, (bf16_t*)vcache, nq, nkv, dq, dk, dv, rot, P, write_cache, pair_half, v_from_k,
                       per_head, k_skip, vfreq, v_pair_half, rot_scale);
  TK_CHECK_LAUNCH("qk_prepare");
  return 0;
}

// --------------------------------------------------------------------------
// out[i, :] = the key of kv head `head` that request req[i] holds at position pos[i], read back from the pages:
// for mixers that compute on cached keys outside the attention (a latent that is expanded for a prompt's portion).
// --------------------------------------------------------------------------
template <typename T>
__global__ void gather_keys_kernel(const T* __restrict__ kcache, const int* __restrict__ block_table, int table_stride,
                                   const int* __restrict__ req, const int* __restrict__ pos, T* __restrict__ out, int nkv,
                                   int head, int dk, int P) {
  const int i = blockIdx.x;
  const int p = pos[i];
  const int page = block_table[(size_t)req[i] * table_stride + p / P];
  const T* src = kcache + ((size_t)page * nkv + head) * key_page_elems(P, dk);
  for (int e = threadIdx.x; e < dk; e += blockDim.x) out[(size_t)i * dk + e] = src[key_offset(P, p % P, e)];
}

TK_API int tk_gather_keys(int dt, const void* kcache, const int* block_table, int table_stride, const int* req, const int* pos,
                          void* out, int n, int nkv, int head, int dk, int P, hipStream_t stream) {
  TK_REQUIRE(kcache && block_table && req && pos && out && n >= 0 && nkv > 0 && head >= 0 && head < nkv && dk > 0 && P > 0,
             "gather_keys: bad arguments");
  if (n == 0) return 0;
  const int threads = dk >= 256 ? 256 : (dk >= 128 ? 128 : 64);
  if (dt == TK_F32)
    hipLaunchKernelGGL(gather_keys_kernel<float>, dim3(n), dim3(threads), 0, stream, (const float*)kcache, block_table, table_stride,
                       req, pos, (float*)out, nkv, head, dk, P);
  else
    hipLaunchKernelGGL(gather_keys_kernel<bf16_t>, dim3(n), dim3(threads), 0, stream, (const bf16_t*)kcache, block_table,
                       table_stride, req, pos, (bf16_t*)out, nkv, head, dk, P);
  TK_CHECK_LAUNCH("gather_keys");
  return 0;
}

// --------------------------------------------------------------------------
// Behind the attention, for mixers whose values were turned by their own positions and whose heads
// have a gate: in place on the heads' results [nq][dv] of a token,
//   * pair m of every head is turned back by the token's position: by -position * vfreq[m], pairs
//     (m, m + dv/2) with `pair_half` and (2m, 2m + 1) without (vfreq null: no turn),
//   * head h is multiplied by sigmoid(gate[h]), `gate` being nq numbers of the token's row of
//     another matrix (null: no gate).
// One workgroup a token, 32-bit arithmetic, one rounding at the store.
// --------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void unrotate_gate_kernel(T* __restrict__ o, int o_stride, const int* __restrict__ positions,
                                                            const float* __restrict__ vfreq, int pair_half,
                                                            const T* __restrict__ gate, int gate_stride, int nq, int dv) {
  extern __shared__ float cs[];  // [dv / 2] cosines, [dv / 2] sines, [nq] gates
  const int t = blockIdx.x;
  const int hv = dv / 2;
  float* gs = cs + 2 * hv;
  if (vfreq) {
    const int pos = positions[t];
    for (int i = threadIdx.x; i < hv; i += blockDim.x) {
      const float angle = __fmul_rn((float)pos, vfreq[i]);
      float s, c;
      sincosf(angle, &s, &c);
      cs[i] = c;
      cs[hv + i] = -s;  // the turn back
    }
  }
  for (int h = threadIdx.x; h < nq; h += blockDim.x)
    gs[h] = gate ? 1.0f / (1.0f + expf(-to_f32<T>(gate[(size_t)t * gate_stride + h]))) : 1.f;
  __syncthreads();
  T* row = o + (size_t)t * o_stride;
  if (vfreq) {
    for (int i = threadIdx.x; i < nq * hv; i += blockDim.x) {
      const int h = i / hv, m = i % hv;
      const int e0 = h * dv + (pair_half ? m : 2 * m), e1 = h * dv + (pair_half ? m + hv : 2 * m + 1);
      float u = to_f32<T>(row[e0]), v = to_f32<T>(row[e1]);
      rotate_pair(u, v, cs[m], cs[hv + m], u, v);
      row[e0] = from_f32<T>(u * gs[h]);
      row[e1] = from_f32<T>(v * gs[h]);
    }
  } else {
    for (int i = threadIdx.x; i < nq * dv; i += blockDim.x) row[i] = from_f32<T>(to_f32<T>(row[i]) * gs[i / dv]);
  }
}

TK_API int tk_unrotate_gate(int dt, void* o, int o_stride, const int* positions, const float* vfreq, int pair_half,
                            const void* gate, int gate_stride, int n_tokens, int nq, int dv, hipStream_t stream) {
  TK_REQUIRE(o && n_tokens >= 0 && nq > 0 && dv > 0 && o_stride >= nq * dv, "unrotate_gate: bad sizes tokens=%d nq=%d dv=%d", n_tokens, nq, dv);
  TK_REQUIRE(!vfreq || (positions && dv % 2 == 0), "unrotate_gate: a turn needs positions and an even value size");
  TK_REQUIRE(!gate || gate_stride >= nq, "unrotate_gate: gate rows of %d hold no %d heads", gate_stride, nq);
  if (n_tokens == 0 || (!vfreq && !gate)) return 0;
  const size_t smem = sizeof(float) * (size_t)(dv + nq);
  TK_REQUIRE(smem <= 48 * 1024, "unrotate_gate: too many heads for one workgroup's local memory");
  if (dt == TK_F32)
    hipLaunchKernelGGL(unrotate_gate_kernel<float>, dim3(n_tokens), dim3(256), smem, stream, (float*)o, o_stride, positions, vfreq,
                       pair_half, (const float*)gate, gate_stride, nq, dv);
  else
    hipLaunchKernelGGL(unrotate_gate_kernel<bf16_t>, dim3(n_tokens), dim3(256), smem, stream, (bf16_t*)o, o_stride, positions, vfreq,
                       pair_half, (const bf16_t*)gate, gate_stride, nq, dv);
  TK_CHECK_LAUNCH("unrotate_gate");
  return 0;
}
