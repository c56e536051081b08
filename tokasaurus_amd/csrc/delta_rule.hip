// The gated delta rule with one decay per head and key channel, as a recurrence over the
// tokens of each request, and what stands around it: the short causal convolutions of q, k
// and v with their activation, the unit norms, the write strength and the decays (before), the
// per-head norm with its gate (after).  Everything that enters the recurrence is 32-bit.
//
// Per request a state row of 32-bit floats lives in the request's slot:
//   [ S: heads x dv x dk ][ tail: (taps - 1) x channels ]
// S is kept transposed (a value column's dk numbers lie together); the tail holds the last
// taps - 1 inputs of the convolutions, oldest first, channels = 2 * kv_heads * dk + heads * dv
// in the order q | k | v.  A slot's row is all zeros when a request takes it.
//
// Per token and head, with decay g (dk), write strength beta, unit k, scaled unit q, value v:
//   S <- diag(g) S;  u = beta * (v - S^T k);  S <- S + k u^T;  o = S^T q.
// The columns of S (one a value channel) do not meet: a column is owned by DR_LANES lanes that
// cut dk between them and add up through the wavefront, always in the same order, so a token's
// result does not depend on how its request's tokens were cut into steps or what shares the batch.
#include "common.h"

#define DR_LANES 16    // lanes that share a column of the state (a row of the wavefront's data paths)
#define DR_TOKENS 16   // most tokens staged in LDS at a time
#define DR_MAX_TAPS 16

__device__ __forceinline__ float silu_f32(float x) { return x / (1.0f + expf(-x)); }
__device__ __forceinline__ float sigmoid_f32(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float softplus_f32(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// --------------------------------------------------------------------------
// Before the recurrence.  A token's work is cut into units, one a wavefront: a q head or a k head
// (convolution, silu, unit norm), a v head (convolution, silu), a head's decays, and the write
// strengths of all heads.
//   proj row (T): [q | k | v] (channels) ... and the write strength's `heads` numbers at col_b
//   a_pre (32-bit) [tokens, heads * dk]: the decay's projection before bias and softplus
//   rec row (32-bit): [q: G*dk | k: G*dk | v: H*dv | decay: H*dk | beta: H]
// FUSE_TAIL (every request of the step brings one token): the lane that convolves a channel also
// moves the channel's tail on, which it alone reads; else the kernel below does it afterwards.
// --------------------------------------------------------------------------
#define DP_MAX_PER_LANE 8  // dk, dv <= 512

template <typename T, bool FUSE_TAIL>
__global__ __launch_bounds__(256) void delta_prepare_kernel(
    const T* __restrict__ proj, int ld, int col_b, const float* __restrict__ a_pre, int ld_a,
    const float* __restrict__ conv_w, int taps, const float* __restrict__ a_log,
    const float* __restrict__ dt_bias, float* __restrict__ state, size_t state_stride,
    size_t tail_off, const int* __restrict__ q_start, const int* __restrict__ token_req,
    const int* __restrict__ slots, float* __restrict__ rec, int ld_rec, int H, int G, int dk, int dv) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & (TK_WAVE - 1);
  const int unit = blockIdx.y * (blockDim.x / TK_WAVE) + threadIdx.x / TK_WAVE;
  const int n_units = 2 * G + 2 * H + 1;
  if (unit >= n_units) return;
  const int C = 2 * G * dk + H * dv;
  float* out = rec + (size_t)t * ld_rec;
  const int v_off = 2 * G * dk, decay_off = v_off + H * dv, beta_off = decay_off + H * dk;
  if (unit < 2 * G + H) {
    // a head's channels through the convolution: q head, k head or v head
    const bool is_v = unit >= 2 * G;
    const int width = is_v ? dv : dk;
    const int c0 = is_v ? v_off + (unit - 2 * G) * dv : unit * dk;
    const int r = token_req[t];
    const int first = q_start[r];
    const int local = t - first;
    float* tail = state + (size_t)slots[r] * state_stride + tail_off;
    float y[DP_MAX_PER_LANE];
    float ss = 0.f;
#pragma unroll
    for (int n = 0; n < DP_MAX_PER_LANE; ++n) {
      const int i = lane + n * TK_WAVE;
      y[n] = 0.f;
      if (i < width) {
        const int c = c0 + i;
        float acc = 0.f;
        for (int j = 0; j < taps; ++j) {
          const int src = local - (taps - 1) + j;
          const float x = src >= 0 ? to_f32<T>(proj[(size_t)(first + src) * ld + c])
                                   : tail[(size_t)(src + taps - 1) * C + c];
          acc = fmaf(conv_w[(size_t)c * taps + j], x, acc);
          if (FUSE_TAIL && j >= 1) tail[(size_t)(j - 1) * C + c] = x;  // (local is 0: entry j - 1 was read a tap ago)
        }
        y[n] = silu_f32(acc);
        ss = fmaf(y[n], y[n], ss);
      }
    }
    float mul = 1.f;
    if (!is_v) {  // unit vectors; the queries also times dk^-1/2
      mul = 1.0f / sqrtf(wave_sum(ss) + 1e-6f);
      if (unit < G) mul *= 1.0f / sqrtf((float)dk);
    }
#pragma unroll
    for (int n = 0; n < DP_MAX_PER_LANE; ++n) {
      const int i = lane + n * TK_WAVE;
      if (i < width) out[c0 + i] = y[n] * mul;
    }
  } else if (unit < 2 * G + 2 * H) {
    const int h = unit - 2 * G - H;
    const float rate = expf(a_log[h]);
    for (int i = lane; i < dk; i += TK_WAVE) {
      const int x = h * dk + i;
      out[decay_off + x] = expf(-rate * softplus_f32(a_pre[(size_t)t * ld_a + x] + dt_bias[x]));
    }
  } else {
    for (int i = lane; i < H; i += TK_WAVE)
      out[beta_off + i] = sigmoid_f32(to_f32<T>(proj[(size_t)t * ld + col_b + i]));
  }
}

// The convolutions' tails after the step: the last taps - 1 inputs of every request, taken
// from this step's rows and, where the step brought fewer, from the old tail.  A thread a
// (request, channel); it reads all it needs before it writes.
template <typename T>
__global__ void delta_tail_kernel(const T* __restrict__ proj, int ld, int taps, float* __restrict__ state,
                                  size_t state_stride, size_t tail_off, const int* __restrict__ q_start,
                                  const int* __restrict__ slots, int C) {
  const int r = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int first = q_start[r], n = q_start[r + 1] - first;
  float* tail = state + (size_t)slots[r] * state_stride + tail_off;
  float keep[DR_MAX_TAPS];
#pragma unroll
  for (int s = 0; s < DR_MAX_TAPS - 1; ++s) {
    if (s < taps - 1) {
      const int src = n - (taps - 1) + s;
      keep[s] = src >= 0 ? to_f32<T>(proj[(size_t)(first + src) * ld + c]) : tail[(size_t)(src + taps - 1) * C + c];
    }
  }
#pragma unroll
  for (int s = 0; s < DR_MAX_TAPS - 1; ++s)
    if (s < taps - 1) tail[(size_t)s * C + c] = keep[s];
}

// --------------------------------------------------------------------------
// The recurrence.  Workgroup (head, request, block of value columns); a column of the state is
// owned by DR_LANES neighbouring lanes: lane holds rows 4 * (lane + DR_LANES * n) + e, n < NQ,
// e < 4.  Per token, with the decayed column sd = g * s:
//     dot = k . sd,  qs = q . sd   (one round of sums through the lanes for both)
//     u = beta * (v - dot);  s = sd + k * u;  o = qs + u * (q . k)
// (o = q . s written out: the read-out sees the token's own write).  q . k does not depend on
// the column but costs little beside the other two sums.  The tokens' rows come through LDS
// in chunks: DR_LOADERS threads of the workgroup do nothing but move the next chunk in while
// the others compute this one, and meet them at a barrier a chunk.
// The sums through the lanes use the lanes' own data paths (no LDS): partners exchange and
// add, so every lane ends with the same bits, in an order that depends on nothing.
// --------------------------------------------------------------------------
// Rows of tokens t0 .. t0 + nt - 1 into a buffer [nt][q | k | decay (dkp each) | v (cols) | beta | padding], by
// `nmove` threads of which this is `me`.  Several loads are in flight a thread before the first is stored.
// VEC: the three long pieces move 16 bytes at a time (the caller found sizes and offsets to be multiples of 4).
template <bool VEC>
__device__ __forceinline__ void delta_move_rows(float* buf, const float* __restrict__ rec, int ld_rec, int t0, int nt,
                                                int me, int nmove, int row_floats, int dkp, int dk, int dv, int cols,
                                                int col0, int q_off, int k_off, int g_off, int v_off, int b_off) {
  constexpr int B = 8;
  if constexpr (VEC) {
    const int per_row = 3 * dkp / 4;
    for (int x0 = me; x0 < nt * per_row; x0 += B * nmove) {
      float4 v[B];
#pragma unroll
      for (int j = 0; j < B; ++j) {
        const int x = x0 + j * nmove;
        v[j] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (x < nt * per_row) {
          const int tt = x / per_row, rem = x % per_row, which = rem / (dkp / 4), i = 4 * (rem % (dkp / 4));
          if (i < dk)
            v[j] = *(const float4*)(rec + (size_t)(t0 + tt) * ld_rec + (which == 0 ? q_off : (which == 1 ? k_off : g_off)) + i);
        }
      }
#pragma unroll
      for (int j = 0; j < B; ++j) {
        const int x = x0 + j * nmove;
        if (x < nt * per_row) *(float4*)(buf + (x / per_row) * row_floats + 4 * (x % per_row)) = v[j];
      }
    }
  }
  const int first = VEC ? 3 * dkp : 0;  // what is left to move one by one
  const int per_row = row_floats - first;
  for (int x0 = me; x0 < nt * per_row; x0 += B * nmove) {
    float v[B];
#pragma unroll
    for (int j = 0; j < B; ++j) {
      const int x = x0 + j * nmove;
      v[j] = 0.f;
      if (x < nt * per_row) {
        const int tt = x / per_row, rem = first + x % per_row;
        const float* row = rec + (size_t)(t0 + tt) * ld_rec;
        if (rem < 3 * dkp) {
          const int which = rem / dkp, i = rem % dkp;
          if (i < dk) v[j] = row[(which == 0 ? q_off : (which == 1 ? k_off : g_off)) + i];
        } else if (rem < 3 * dkp + cols) {
          const int c = rem - 3 * dkp;
          if (col0 + c < dv) v[j] = row[v_off + col0 + c];
        } else if (rem == 3 * dkp + cols) {
          v[j] = row[b_off];
        }
      }
    }
#pragma unroll
    for (int j = 0; j < B; ++j) {
      const int x = x0 + j * nmove;
      if (x < nt * per_row) buf[(x / per_row) * row_floats + first + x % per_row] = v[j];
    }
  }
}

#define DR_LOADERS 128  // threads of a workgroup that only move the next chunk's rows into LDS

template <int NQ, bool VEC>
__global__ __launch_bounds__(NQ > 2 ? 384 : 1024) void delta_rule_kernel(
    const float* __restrict__ rec, int ld_rec, float* __restrict__ state, size_t state_stride,
    const int* __restrict__ q_start, const int* __restrict__ slots, float* __restrict__ o, int H, int G,
    int dk, int dv, int cols, int tok) {
  // two buffers of [tok][3][dkp] q, k, decay; [tok][cols] v; [tok] beta
  extern __shared__ __align__(16) float stage[];
  const int h = blockIdx.x, r = blockIdx.y;
  const int col0 = blockIdx.z * cols;
  const int ncompute = cols * DR_LANES;
  const bool loader = (int)threadIdx.x >= ncompute;
  const int lane = threadIdx.x % DR_LANES, grp = threadIdx.x / DR_LANES;
  const int col = col0 + grp;
  const bool live = !loader && col < dv;
  constexpr int dkp = NQ * DR_LANES * 4;  // dk rounded up to what the lanes of a column hold
  const int gk = h / (H / G);
  const int first = q_start[r], last = q_start[r + 1];
  float* s_col = state + (size_t)slots[r] * state_stride + ((size_t)h * dv + (live ? col : 0)) * dk;

  float s[NQ][4];
#pragma unroll
  for (int n = 0; n < NQ; ++n)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int i = 4 * (lane + DR_LANES * n) + e;
      s[n][e] = (live && i < dk) ? s_col[i] : 0.f;
    }

  const int row_floats = 3 * dkp + (cols + 1 + 3) / 4 * 4;
  const int buf_floats = tok * row_floats;
  const int q_off = gk * dk, k_off = G * dk + gk * dk, v_off = 2 * G * dk + h * dv;
  const int g_off = 2 * G * dk + H * dv + h * dk, b_off = 2 * G * dk + H * dv + H * dk + h;

#define move(BUF, T0, NT, ME, NMOVE) \
  delta_move_rows<VEC>(BUF, rec, ld_rec, T0, NT, ME, NMOVE, row_floats, dkp, dk, dv, cols, col0, q_off, k_off, g_off, v_off, b_off)
  if (first < last) move(stage, first, min(tok, last - first), threadIdx.x, blockDim.x);
  __syncthreads();
  int chunk = 0;
#pragma unroll 1
  for (int t0 = first; t0 < last; t0 += tok, ++chunk) {
    const int nt = min(tok, last - t0);
    const float* buf = stage + (chunk & 1) * buf_floats;
    if (loader) {
      const int next = t0 + tok;
      if (next < last) move(stage + ((chunk + 1) & 1) * buf_floats, next, min(tok, last - next), threadIdx.x - ncompute, DR_LOADERS);
    } else {
#pragma unroll 1
      for (int tt = 0; tt < nt; ++tt) {
        const float* row = buf + tt * row_floats;
        const float4* q4 = (const float4*)row;
        const float4* k4 = (const float4*)(row + dkp);
        const float4* g4 = (const float4*)(row + 2 * dkp);
        float kk[NQ][4];
        float dot[2] = {0.f, 0.f}, qs[2] = {0.f, 0.f}, kq[2] = {0.f, 0.f};
#pragma unroll
        for (int n = 0; n < NQ; ++n) {
          const float4 g = g4[lane + DR_LANES * n], k = k4[lane + DR_LANES * n], q = q4[lane + DR_LANES * n];
          kk[n][0] = k.x; kk[n][1] = k.y; kk[n][2] = k.z; kk[n][3] = k.w;
          s[n][0] *= g.x; s[n][1] *= g.y; s[n][2] *= g.z; s[n][3] *= g.w;
          dot[0] = fmaf(k.x, s[n][0], dot[0]); dot[1] = fmaf(k.y, s[n][1], dot[1]);
          dot[0] = fmaf(k.z, s[n][2], dot[0]); dot[1] = fmaf(k.w, s[n][3], dot[1]);
          qs[0] = fmaf(q.x, s[n][0], qs[0]); qs[1] = fmaf(q.y, s[n][1], qs[1]);
          qs[0] = fmaf(q.z, s[n][2], qs[0]); qs[1] = fmaf(q.w, s[n][3], qs[1]);
          kq[0] = fmaf(q.x, k.x, kq[0]); kq[1] = fmaf(q.y, k.y, kq[1]);
          kq[0] = fmaf(q.z, k.z, kq[0]); kq[1] = fmaf(q.w, k.w, kq[1]);
        }
        const float d = row_sum16(dot[0] + dot[1]);
        const float qsum = row_sum16(qs[0] + qs[1]);
        const float kqsum = row_sum16(kq[0] + kq[1]);
        const float u = row[3 * dkp + cols] * (row[3 * dkp + grp] - d);
#pragma unroll
        for (int n = 0; n < NQ; ++n)
#pragma unroll
          for (int e = 0; e < 4; ++e) s[n][e] = fmaf(kk[n][e], u, s[n][e]);
        if (live && lane == 0) o[(size_t)(t0 + tt) * H * dv + (size_t)h * dv + col] = fmaf(u, kqsum, qsum);
      }
    }
    __syncthreads();
  }
#undef move
  if (live) {
#pragma unroll
    for (int n = 0; n < NQ; ++n)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int i = 4 * (lane + DR_LANES * n) + e;
        if (i < dk) s_col[i] = s[n][e];
      }
  }
}

// --------------------------------------------------------------------------
// After the recurrence: every head's dv outputs divided by their root mean square, times a
// weight [dv] shared by the heads, times sigmoid(gate); rounded once to T.  A wavefront a
// (token, head).
// --------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void gated_head_norm_kernel(const float* __restrict__ o, const float* __restrict__ gate,
                                                              int ld_gate, int H, const float* __restrict__ w, float eps,
                                                              T* __restrict__ out, long units, int dv) {
  const int lane = threadIdx.x & (TK_WAVE - 1);
  const long unit = (long)blockIdx.x * (blockDim.x / TK_WAVE) + threadIdx.x / TK_WAVE;
  if (unit >= units) return;
  const float* x = o + (size_t)unit * dv;
  const float* g = gate + (size_t)(unit / H) * ld_gate + (size_t)(unit % H) * dv;
  float ss = 0.f;
  for (int i = lane; i < dv; i += TK_WAVE) ss = fmaf(x[i], x[i], ss);
  ss = wave_sum(ss);
  const float rstd = 1.0f / sqrtf(ss / (float)dv + eps);
  for (int i = lane; i < dv; i += TK_WAVE)
    out[(size_t)unit * dv + i] = from_f32<T>(x[i] * rstd * w[i] * sigmoid_f32(g[i]));
}

TK_API int tk_delta_prepare(int dt, const void* proj, int ld, int col_b, const float* a_pre, int ld_a,
                            const float* conv_w, int taps, const float* a_log, const float* dt_bias,
                            float* state, size_t state_stride, size_t tail_off, const int* q_start,
                            const int* token_req, const int* slots, float* rec, int ld_rec, int n_tokens,
                            int n_requests, int H, int G, int dk, int dv, hipStream_t stream) {
  TK_REQUIRE(n_tokens >= 0 && n_requests >= 0 && H > 0 && G > 0 && H % G == 0 && dk > 0 && dv > 0,
             "delta_prepare: bad sizes tokens=%d heads=%d kv heads=%d dk=%d dv=%d", n_tokens, H, G, dk, dv);
  TK_REQUIRE(taps >= 1 && taps <= DR_MAX_TAPS, "delta_prepare: %d taps (1..%d)", taps, DR_MAX_TAPS);
  const int C = 2 * G * dk + H * dv;
  TK_REQUIRE(ld >= C && col_b >= 0 && col_b + H <= ld, "delta_prepare: row stride %d too short", ld);
  TK_REQUIRE(ld_a >= H * dk, "delta_prepare: the decay projection's stride %d is too short", ld_a);
  TK_REQUIRE(ld_rec >= C + H * dk + H, "delta_prepare: output stride %d too short", ld_rec);
  TK_REQUIRE(tail_off + (size_t)(taps - 1) * C <= state_stride, "delta_prepare: the state row is too short");
  TK_REQUIRE(dk <= DP_MAX_PER_LANE * TK_WAVE && dv <= DP_MAX_PER_LANE * TK_WAVE, "delta_prepare: head sizes %d, %d (at most %d)",
             dk, dv, DP_MAX_PER_LANE * TK_WAVE);
  if (n_tokens == 0) return 0;
  const int units = 2 * G + 2 * H + 1;
  const dim3 grid(n_tokens, (units + 3) / 4);
  TK_REQUIRE(grid.y < 65536, "delta_prepare: too many heads");
  // every request brings one token: the convolving lane moves its channel's tail on itself
  const bool fuse_tail = n_tokens == n_requests && taps > 1;
#define DP_LAUNCH(T, FUSE)                                                                                         \
  hipLaunchKernelGGL((delta_prepare_kernel<T, FUSE>), grid, dim3(256), 0, stream, (const T*)proj, ld, col_b, a_pre, ld_a, \
                     conv_w, taps, a_log, dt_bias, state, state_stride, tail_off, q_start, token_req, slots, rec,  \
                     ld_rec, H, G, dk, dv)
  if (dt == TK_F32) {
    if (fuse_tail) DP_LAUNCH(float, true); else DP_LAUNCH(float, false);
  } else {
    if (fuse_tail) DP_LAUNCH(bf16_t, true); else DP_LAUNCH(bf16_t, false);
  }
#undef DP_LAUNCH
  TK_CHECK_LAUNCH("delta_prepare");
  if (taps > 1 && n_requests > 0 && !fuse_tail) {
    TK_REQUIRE(n_requests < 65536, "delta_prepare: too many requests");
    const dim3 tgrid((C + 255) / 256, n_requests);
    if (dt == TK_F32)
      hipLaunchKernelGGL(delta_tail_kernel<float>, tgrid, dim3(256), 0, stream, (const float*)proj, ld, taps, state,
                         state_stride, tail_off, q_start, slots, C);
    else
      hipLaunchKernelGGL(delta_tail_kernel<bf16_t>, tgrid, dim3(256), 0, stream, (const bf16_t*)proj, ld, taps, state,
                         state_stride, tail_off, q_start, slots, C);
    TK_CHECK_LAUNCH("delta_tail");
  }
  return 0;
}

TK_API int tk_delta_rule(const float* rec, int ld_rec, float* state, size_t state_stride, const int* q_start,
                         const int* slots, float* o, int n_requests, int H, int G, int dk, int dv, int cols,
                         hipStream_t stream) {
  TK_REQUIRE(n_requests >= 0 && H > 0 && G > 0 && H % G == 0 && dk > 0 && dv > 0,
             "delta_rule: bad sizes heads=%d kv heads=%d dk=%d dv=%d", H, G, dk, dv);
  TK_REQUIRE(dk <= 512, "delta_rule: key size %d (at most 512)", dk);
  TK_REQUIRE(cols > 0 && cols % (TK_WAVE / DR_LANES) == 0 && cols * DR_LANES <= 1024,
             "delta_rule: %d columns a workgroup", cols);
  TK_REQUIRE(ld_rec >= 2 * G * dk + H * dv + H * dk + H, "delta_rule: input stride %d too short", ld_rec);
  TK_REQUIRE((size_t)H * dv * dk <= state_stride, "delta_rule: the state row is too short");
  TK_REQUIRE(n_requests < 65536, "delta_rule: too many requests");
  if (n_requests == 0) return 0;
  int nq = (dk + DR_LANES * 4 - 1) / (DR_LANES * 4);
  nq = nq <= 2 ? nq : (nq <= 4 ? 4 : 8);  // the kernel's instances
  const int dkp = nq * DR_LANES * 4;
  const int threads = cols * DR_LANES + DR_LOADERS;
  TK_REQUIRE(threads <= (nq > 2 ? 384 : 1024), "delta_rule: %d columns a workgroup are too many for key size %d", cols, dk);
  const int row_floats = 3 * dkp + (cols + 1 + 3) / 4 * 4;
  int tok = 8192 / row_floats;  // two buffers of 32 KB at most
  tok = tok > DR_TOKENS ? DR_TOKENS : tok;
  TK_REQUIRE(tok >= 1, "delta_rule: key size %d with %d columns a workgroup", dk, cols);
  const size_t smem = sizeof(float) * 2 * (size_t)tok * row_floats;
  const dim3 grid(H, n_requests, (dv + cols - 1) / cols), block(threads);
  const bool vec = dk % 4 == 0 && (H * dv) % 4 == 0 && ld_rec % 4 == 0 && ((uintptr_t)rec & 15) == 0;
#define DR_CASE(NQ)                                                                                              \
  do {                                                                                                           \
    if (vec)                                                                                                     \
      hipLaunchKernelGGL((delta_rule_kernel<NQ, true>), grid, block, smem, stream, rec, ld_rec, state,           \
                         state_stride, q_start, slots, o, H, G, dk, dv, cols, tok);                              \
    else                                                                                                         \
      hipLaunchKernelGGL((delta_rule_kernel<NQ, false>), grid, block, smem, stream, rec, ld_rec, state,          \
                         state_stride, q_start, slots, o, H, G, dk, dv, cols, tok);                              \
  } while (0)
  if (nq == 1) DR_CASE(1);
  else if (nq == 2) DR_CASE(2);
  else if (nq == 4) DR_CASE(4);
  else DR_CASE(8);
#undef DR_CASE
  TK_CHECK_LAUNCH("delta_rule");
  return 0;
}

TK_API int tk_gated_head_norm(int dt, const float* o, const float* gate, int ld_gate, const float* w, float eps, void* out,
                              int n_tokens, int H, int dv, hipStream_t stream) {
  TK_REQUIRE(ld_gate >= H * dv, "gated_head_norm: the gate's stride %d is too short", ld_gate);
  TK_REQUIRE(n_tokens >= 0 && H > 0 && dv > 0, "gated_head_norm: bad sizes %d %d %d", n_tokens, H, dv);
  if (n_tokens == 0) return 0;
  const long units = (long)n_tokens * H;
  const long blocks = (units + 3) / 4;
  TK_REQUIRE(blocks < (1l << 31), "gated_head_norm: too many rows");
  if (dt == TK_F32)
    hipLaunchKernelGGL(gated_head_norm_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, stream, o, gate, ld_gate, H, w, eps,
                       (float*)out, units, dv);
  else
    hipLaunchKernelGGL(gated_head_norm_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, stream, o, gate, ld_gate, H, w, eps,
                       (bf16_t*)out, units, dv);
  TK_CHECK_LAUNCH("gated_head_norm");
  return 0;
}
