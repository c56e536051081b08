// Linear attention with a decay, as a recurrence over the tokens of each request, and what stands
// around it in the mixers that use it: the short causal convolution that is added to a mixer's input,
// the norm of the recurrence's result (head by head or over all heads) with an optional sigmoid gate,
// and a sigmoid gate on the rows of another mixer.
//
// Per head, with a matrix S [dk][dv] kept per request in 32-bit:
//     S_t = diag(a_t) S_(t-1) + k_t v_t^T        o_t = S_t^T q_t
// in two forms, both read from the 32-bit sums `proj` of one stacked product:
//   LA_CONSTANT  q = silu(.), k = silu(.), v = silu(.), a_t = decay[head] for every row and token
//   LA_FORGET    q = silu(.), f = low + (1 - low) * sigmoid(. + bias) per head and row of S; a_t = f, k_t = 1 - f; v as it is
// Everything from the sums on (activations, gates, the state, the read-out) is 32-bit arithmetic.
//
// The state row of a slot is [H][dv][dk]: a value column's dk numbers lie together.  The columns of S
// do not meet: a column is owned by LA_LANES neighbouring lanes that cut dk between them and add up through the
// wavefront's own data paths, always in the same order, so a token's result does not depend on how its request's
// tokens were cut into steps or on what shares the batch.
#include "common.h"

#define LA_LANES 16
#define LA_COLS 4      // value columns a wavefront owns
#define LA_WAVES 8     // most wavefronts of a workgroup (they share nothing: a workgroup is only a unit of dispatch)
enum { LA_CONSTANT = 0, LA_FORGET = 1 };

__device__ __forceinline__ float la_silu(float x) { return x / (1.0f + expf(-x)); }
__device__ __forceinline__ float la_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
// the forget gate, written out in one multiply-add so that every kernel that computes it gets the same bits
__device__ __forceinline__ float la_forget(float x, float bias, float lo) { return fmaf(1.0f - lo, la_sigmoid(x + bias), lo); }

// --------------------------------------------------------------------------
// Before the recurrence, once a token: the activations, into rows that the recurrence's lanes read 16 bytes at a
// time.  rec row: [q: H x dkp | k or f: H x dkp | v: H x dv (padded to a multiple of 4)], dkp = dk rounded up to 64
// times the pieces a lane holds, zeros in the padding (a padded row of S meets a zero of q).
//   LA_CONSTANT  q = silu(.), k = silu(.), v = silu(.)
//   LA_FORGET    q = silu(.), f = low + (1 - low) * sigmoid(. + bias), v as it is
// --------------------------------------------------------------------------
template <int MODE>
__global__ __launch_bounds__(256) void linear_attention_prepare_kernel(
    const float* __restrict__ proj, int ld, int q_off, int k_off, int v_off, const float* __restrict__ f_bias,
    const float* __restrict__ f_low, float* __restrict__ rec, int ld_rec, int H, int dk, int dv, int dkp) {
  const size_t t = blockIdx.y;
  const int x = blockIdx.x * blockDim.x + threadIdx.x;
  if (x >= ld_rec) return;
  const float* row = proj + t * ld;
  float val = 0.f;
  if (x < 2 * H * dkp) {
    const int which = x / (H * dkp), rem = x % (H * dkp), h = rem / dkp, i = rem % dkp;
    if (i < dk) {
      const int c = h * dk + i;
      if (which == 0) {
        val = la_silu(row[q_off + c]);
      } else if (MODE == LA_CONSTANT) {
        val = la_silu(row[k_off + c]);
      } else {
        val = la_forget(row[k_off + c], f_bias[c], f_low[c]);
      }
    }
  } else {
    const int c = x - 2 * H * dkp;
    if (c < H * dv) val = MODE == LA_CONSTANT ? la_silu(row[v_off + c]) : row[v_off + c];
  }
  rec[t * ld_rec + x] = val;
}

// --------------------------------------------------------------------------
// The recurrence.  A wavefront owns LA_COLS value columns of one (head, request); the wavefronts of a workgroup take
// neighbouring blocks of columns and share nothing (a step of single tokens is a launch of thousands of short
// wavefronts, which are dispatched faster in workgroups of several).  A column of S is
// owned by LA_LANES neighbouring lanes; lane l holds rows 4 * (l + LA_LANES * n) + e, n < NQ, e < 4, so that it reads
// its pieces of q and of k (or f) as whole 16-byte loads.  Nothing is staged in LDS and there is no barrier: the
// wavefronts of a head read the same rows of `rec` (served by the caches), PF tokens ahead of the arithmetic.
//   LA_CONSTANT  s = a s + k v        LA_FORGET  s = f s + (1 - f) v = v + f (s - v)        o = sum over rows of q s
// --------------------------------------------------------------------------
template <int NQ, int MODE, int PF>
__global__ __launch_bounds__(LA_WAVES * TK_WAVE) void linear_attention_kernel(
    const float* __restrict__ rec, int ld_rec, const float* __restrict__ decay, float* __restrict__ state,
    size_t state_stride, const int* __restrict__ q_start, const int* __restrict__ slots, float* __restrict__ o, int H,
    int dk, int dv, int dkp) {
  const int h = blockIdx.x, r = blockIdx.y;
  const int lane = threadIdx.x % LA_LANES, grp = threadIdx.x / LA_LANES;  // grp: a column of the workgroup's block
  const int col = blockIdx.z * (blockDim.x / LA_LANES) + grp;
  if ((col / LA_COLS) * LA_COLS >= dv) return;  // a wavefront none of whose columns exists
  const bool live = col < dv;
  const int first = q_start[r], last = q_start[r + 1];
  if (first >= last) return;
  float* s_col = state + (size_t)slots[r] * state_stride + ((size_t)h * dv + (live ? col : 0)) * dk;
  const bool vec = (dk % 4 == 0) && (state_stride % 4 == 0);
  float s[NQ][4];
#pragma unroll
  for (int n = 0; n < NQ; ++n) {
    const int i = 4 * (lane + LA_LANES * n);
    if (vec && live && i < dk) {
      const float4 v = *(const float4*)(s_col + i);
      s[n][0] = v.x; s[n][1] = v.y; s[n][2] = v.z; s[n][3] = v.w;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) s[n][e] = (live && i + e < dk) ? s_col[i + e] : 0.f;
    }
  }
  const float a_head = MODE == LA_CONSTANT ? decay[h] : 0.f;
  const int q_at = h * dkp + 4 * lane, k_at = H * dkp + q_at, v_at = 2 * H * dkp + h * dv + (live ? col : 0);

  float4 q[2][PF][NQ], k[2][PF][NQ];
  float v[2][PF];
  // rows of tokens t0 .. t0 + PF - 1 (those beyond the request's end repeat its last token and are not used)
#define LA_LOAD(B, T0)                                                               \
  _Pragma("unroll") for (int j = 0; j < PF; ++j) {                                   \
    const float* row = rec + (size_t)min((T0) + j, last - 1) * ld_rec;               \
    _Pragma("unroll") for (int n = 0; n < NQ; ++n) {                                 \
      q[B][j][n] = *(const float4*)(row + q_at + 4 * LA_LANES * n);                  \
      k[B][j][n] = *(const float4*)(row + k_at + 4 * LA_LANES * n);                  \
    }                                                                                \
    v[B][j] = row[v_at];                                                             \
  }
#define LA_STEP(B, T0)                                                               \
  _Pragma("unroll") for (int j = 0; j < PF; ++j) {                                   \
    if ((T0) + j < last) {                                                           \
      const float vv = v[B][j];                                                      \
      float acc0 = 0.f, acc1 = 0.f;                                                  \
      _Pragma("unroll") for (int n = 0; n < NQ; ++n) {                               \
        const float qq[4] = {q[B][j][n].x, q[B][j][n].y, q[B][j][n].z, q[B][j][n].w}; \
        const float kk[4] = {k[B][j][n].x, k[B][j][n].y, k[B][j][n].z, k[B][j][n].w}; \
        _Pragma("unroll") for (int e = 0; e < 4; ++e) {                              \
          if (MODE == LA_CONSTANT) s[n][e] = fmaf(a_head, s[n][e], kk[e] * vv);      \
          else s[n][e] = fmaf(kk[e], s[n][e] - vv, vv);                              \
        }                                                                            \
        acc0 = fmaf(qq[0], s[n][0], acc0); acc1 = fmaf(qq[1], s[n][1], acc1);        \
        acc0 = fmaf(qq[2], s[n][2], acc0); acc1 = fmaf(qq[3], s[n][3], acc1);        \
      }                                                                              \
      const float sum = row_sum16(acc0 + acc1);                                      \
      if (live && lane == 0) o[(size_t)((T0) + j) * H * dv + (size_t)h * dv + col] = sum; \
    }                                                                                \
  }
  LA_LOAD(0, first);
#pragma unroll 1
  for (int t0 = first; t0 < last; t0 += 2 * PF) {
    LA_LOAD(1, t0 + PF);
    LA_STEP(0, t0);
    LA_LOAD(0, t0 + 2 * PF);
    LA_STEP(1, t0 + PF);
  }
#undef LA_LOAD
#undef LA_STEP
#pragma unroll
  for (int n = 0; n < NQ; ++n) {
    const int i = 4 * (lane + LA_LANES * n);
    if (!live) continue;
    if (vec && i < dk) {
      *(float4*)(s_col + i) = make_float4(s[n][0], s[n][1], s[n][2], s[n][3]);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (i + e < dk) s_col[i + e] = s[n][e];
    }
  }
}

// 16-byte pieces of a head's keys that a lane holds: one of the kernel's instances (1, 2, 3, 4, 6, 8); a head's keys
// are padded to 64 times that in `rec`.
static int la_pieces(int dk) {
  const int nq = (dk + 63) / 64;
  return nq <= 4 ? nq : (nq <= 6 ? 6 : 8);
}

// --------------------------------------------------------------------------
// The same for steps in which every request brings one token: the activations are computed by the lanes that need
// them (there is no pass in front and no `rec`), with the functions of the pass above, so the sums are the same bits.
// --------------------------------------------------------------------------
template <int NQ, int MODE>
__global__ __launch_bounds__(LA_WAVES * TK_WAVE) void linear_attention_single_kernel(
    const float* __restrict__ proj, int ld, int q_off, int k_off, int v_off, const float* __restrict__ decay,
    const float* __restrict__ f_bias, const float* __restrict__ f_low, float* __restrict__ state, size_t state_stride,
    const int* __restrict__ q_start, const int* __restrict__ slots, float* __restrict__ o, int H, int dk, int dv) {
  const int h = blockIdx.x, r = blockIdx.y;
  const int lane = threadIdx.x % LA_LANES, grp = threadIdx.x / LA_LANES;
  const int col = blockIdx.z * (blockDim.x / LA_LANES) + grp;
  if ((col / LA_COLS) * LA_COLS >= dv) return;
  const bool live = col < dv;
  const int t = q_start[r];
  if (q_start[r + 1] <= t) return;
  float* s_col = state + (size_t)slots[r] * state_stride + ((size_t)h * dv + (live ? col : 0)) * dk;
  const bool vec = (dk % 4 == 0) && (state_stride % 4 == 0);
  const float* row = proj + (size_t)t * ld;
  const float a_head = MODE == LA_CONSTANT ? decay[h] : 0.f;
  const float raw_v = row[v_off + h * dv + (live ? col : 0)];
  const float vv = MODE == LA_CONSTANT ? la_silu(raw_v) : raw_v;
  float acc0 = 0.f, acc1 = 0.f;
  float s[NQ][4];
#pragma unroll
  for (int n = 0; n < NQ; ++n) {
    const int i = 4 * (lane + LA_LANES * n);
    if (vec && live && i < dk) {
      const float4 v = *(const float4*)(s_col + i);
      s[n][0] = v.x; s[n][1] = v.y; s[n][2] = v.z; s[n][3] = v.w;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) s[n][e] = (live && i + e < dk) ? s_col[i + e] : 0.f;
    }
    float qq[4], kk[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const bool in = i + e < dk;
      const int c = h * dk + (in ? i + e : 0);
      qq[e] = in ? la_silu(row[q_off + c]) : 0.f;
      if (MODE == LA_CONSTANT) kk[e] = in ? la_silu(row[k_off + c]) : 0.f;
      else kk[e] = in ? la_forget(row[k_off + c], f_bias[c], f_low[c]) : 0.f;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (MODE == LA_CONSTANT) s[n][e] = fmaf(a_head, s[n][e], kk[e] * vv);
      else s[n][e] = fmaf(kk[e], s[n][e] - vv, vv);
    }
    acc0 = fmaf(qq[0], s[n][0], acc0); acc1 = fmaf(qq[1], s[n][1], acc1);
    acc0 = fmaf(qq[2], s[n][2], acc0); acc1 = fmaf(qq[3], s[n][3], acc1);
  }
  const float sum = row_sum16(acc0 + acc1);
  if (!live) return;
  if (lane == 0) o[(size_t)t * H * dv + (size_t)h * dv + col] = sum;
#pragma unroll
  for (int n = 0; n < NQ; ++n) {
    const int i = 4 * (lane + LA_LANES * n);
    if (vec && i < dk) {
      *(float4*)(s_col + i) = make_float4(s[n][0], s[n][1], s[n][2], s[n][3]);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (i + e < dk) s_col[i + e] = s[n][e];
    }
  }
}

// Floats of a row of `rec` for these sizes.
TK_API int tk_linear_attention_rec_width(int H, int dk, int dv) {
  return 2 * H * la_pieces(dk) * 64 + (H * dv + 3) / 4 * 4;
}

TK_API int tk_linear_attention(int mode, const float* proj, int ld, int q_off, int k_off, int v_off, const float* decay,
                               const float* f_bias, const float* f_low, float* state, size_t state_stride,
                               const int* q_start, const int* slots, float* rec, float* o, int n_tokens, int n_requests, int H,
                               int dk, int dv, int longest, hipStream_t stream) {
  TK_REQUIRE(n_tokens >= 0 && n_requests >= 0 && H > 0 && dk > 0 && dv > 0 && dk <= 512,
             "linear_attention: bad sizes tokens=%d requests=%d heads=%d dk=%d dv=%d (dk up to 512)", n_tokens, n_requests, H, dk, dv);
  TK_REQUIRE(mode == LA_CONSTANT ? decay != nullptr : (mode == LA_FORGET && f_bias && f_low),
             "linear_attention: the constant form needs a decay a head, the forget-gate form a bias and a lower bound");
  const bool single = longest <= 1;
  TK_REQUIRE(proj && state && q_start && slots && o && (rec || single) && state_stride >= (size_t)H * dk * dv && n_requests < 65536 && n_tokens < 65536,
             "linear_attention: a pointer is missing, the state's rows are too short or the step too large");
  TK_REQUIRE((((uintptr_t)rec | (uintptr_t)state) & 15) == 0, "linear_attention: rec and state must start at multiples of 16 bytes");
  TK_REQUIRE(longest >= 1, "linear_attention: the longest portion of a step with tokens is at least one token");
  if (n_requests == 0 || n_tokens == 0) return 0;
  const int nq = la_pieces(dk), dkp = 64 * nq;
  if (single) {
    const int waves = min(LA_WAVES, (dv + LA_COLS - 1) / LA_COLS);
    const dim3 grid(H, n_requests, (dv + LA_COLS * waves - 1) / (LA_COLS * waves)), block(waves * TK_WAVE);
#define LA_SINGLE(NQ)                                                                                                           \
  do {                                                                                                                          \
    if (mode == LA_CONSTANT)                                                                                                    \
      hipLaunchKernelGGL((linear_attention_single_kernel<NQ, LA_CONSTANT>), grid, block, 0, stream, proj, ld, q_off, k_off,     \
                         v_off, decay, f_bias, f_low, state, state_stride, q_start, slots, o, H, dk, dv);                       \
    else                                                                                                                        \
      hipLaunchKernelGGL((linear_attention_single_kernel<NQ, LA_FORGET>), grid, block, 0, stream, proj, ld, q_off, k_off, v_off, \
                         decay, f_bias, f_low, state, state_stride, q_start, slots, o, H, dk, dv);                              \
  } while (0)
    if (nq <= 1) LA_SINGLE(1);
    else if (nq <= 2) LA_SINGLE(2);
    else if (nq <= 3) LA_SINGLE(3);
    else if (nq <= 4) LA_SINGLE(4);
    else if (nq <= 6) LA_SINGLE(6);
    else LA_SINGLE(8);
#undef LA_SINGLE
    TK_CHECK_LAUNCH("linear_attention");
    return 0;
  }
  const int ld_rec = tk_linear_attention_rec_width(H, dk, dv);
  const dim3 pgrid((ld_rec + 255) / 256, n_tokens);
  if (mode == LA_CONSTANT)
    hipLaunchKernelGGL(linear_attention_prepare_kernel<LA_CONSTANT>, pgrid, dim3(256), 0, stream, proj, ld, q_off, k_off, v_off,
                       f_bias, f_low, rec, ld_rec, H, dk, dv, dkp);
  else
    hipLaunchKernelGGL(linear_attention_prepare_kernel<LA_FORGET>, pgrid, dim3(256), 0, stream, proj, ld, q_off, k_off, v_off,
                       f_bias, f_low, rec, ld_rec, H, dk, dv, dkp);
  // A long walk is a chain of arithmetic in every wavefront: one wavefront a workgroup then spreads a prompt's few
  // wavefronts over all compute units (measured: 2 048 tokens of 8 heads of 128 x 128 in 180 us, against 360 us with
  // eight wavefronts a workgroup).  Steps of few tokens a request launch thousands of short wavefronts, in workgroups of eight.
  const int waves = longest > 16 ? 1 : min(LA_WAVES, (dv + LA_COLS - 1) / LA_COLS);
  const dim3 grid(H, n_requests, (dv + LA_COLS * waves - 1) / (LA_COLS * waves)), block(waves * TK_WAVE);
#define LA_CASE(NQ, PF)                                                                                                      \
  do {                                                                                                                       \
    if (mode == LA_CONSTANT)                                                                                                 \
      hipLaunchKernelGGL((linear_attention_kernel<NQ, LA_CONSTANT, PF>), grid, block, 0, stream, rec, ld_rec, decay, state,  \
                         state_stride, q_start, slots, o, H, dk, dv, dkp);                                                   \
    else                                                                                                                     \
      hipLaunchKernelGGL((linear_attention_kernel<NQ, LA_FORGET, PF>), grid, block, 0, stream, rec, ld_rec, decay, state,    \
                         state_stride, q_start, slots, o, H, dk, dv, dkp);                                                   \
  } while (0)
  if (nq <= 1) LA_CASE(1, 4);
  else if (nq <= 2) LA_CASE(2, 4);
  else if (nq <= 3) LA_CASE(3, 2);
  else if (nq <= 4) LA_CASE(4, 2);
  else if (nq <= 6) LA_CASE(6, 1);
  else LA_CASE(8, 1);
#undef LA_CASE
  TK_CHECK_LAUNCH("linear_attention");
  return 0;
}

// --------------------------------------------------------------------------
// Behind the recurrence: every group's `size` numbers of a token divided by their root mean square, times a
// weight [size] that the groups share, times sigmoid(gate) where there is a gate, times `scale`; rounded once
// to T.  A group is a head (a norm head by head) or the whole row (groups = 1).  A wavefront a (token, group).
// --------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void group_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ gate, int ld_gate,
                                                              int groups, const float* __restrict__ w, float eps, float scale,
                                                              T* __restrict__ out, int ld_out, long units, int size) {
  const int lane = threadIdx.x & (TK_WAVE - 1);
  const long unit = (long)blockIdx.x * (blockDim.x / TK_WAVE) + threadIdx.x / TK_WAVE;
  if (unit >= units) return;
  const long t = unit / groups;
  const int g = (int)(unit % groups);
  const float* x = o + (size_t)unit * size;
  float ss = 0.f;
  for (int i = lane; i < size; i += TK_WAVE) ss = fmaf(x[i], x[i], ss);
  ss = wave_sum(ss);
  const float rstd = 1.0f / sqrtf(ss / (float)size + eps);
  for (int i = lane; i < size; i += TK_WAVE) {
    float y = x[i] * rstd * w[i];
    if (gate) y *= la_sigmoid(gate[(size_t)t * ld_gate + (size_t)g * size + i]);
    out[(size_t)t * ld_out + (size_t)g * size + i] = from_f32<T>(y * scale);
  }
}

// The same with a workgroup a (token, group), for groups of many numbers (one norm over all heads): a wavefront alone
// would walk such a row as a chain of loads.
template <typename T>
__global__ __launch_bounds__(256) void group_norm_gate_wide_kernel(const float* __restrict__ o, const float* __restrict__ gate,
                                                                   int ld_gate, int groups, const float* __restrict__ w, float eps,
                                                                   float scale, T* __restrict__ out, int ld_out, int size) {
  __shared__ float red[16];
  const long unit = blockIdx.x;
  const long t = unit / groups;
  const int g = (int)(unit % groups);
  const float* x = o + (size_t)unit * size;
  float ss = 0.f;
  if (size % 4 == 0 && size <= 4 * 256 * 4 && ((uintptr_t)x & 15) == 0) {
    // the row in registers: up to four 16-byte pieces a thread, asked for together
    float4 v[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int i = threadIdx.x + q * 256;
      v[q] = i < size / 4 ? ((const float4*)x)[i] : make_float4(0.f, 0.f, 0.f, 0.f);
      ss = fmaf(v[q].x, v[q].x, ss); ss = fmaf(v[q].y, v[q].y, ss); ss = fmaf(v[q].z, v[q].z, ss); ss = fmaf(v[q].w, v[q].w, ss);
    }
    ss = block_sum(ss, red);
    const float rstd = 1.0f / sqrtf(ss / (float)size + eps);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int i = threadIdx.x + q * 256;
      if (i < size / 4) {
        const float xs[4] = {v[q].x, v[q].y, v[q].z, v[q].w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int c = 4 * i + e;
          float y = xs[e] * rstd * w[c];
          if (gate) y *= la_sigmoid(gate[(size_t)t * ld_gate + (size_t)g * size + c]);
          out[(size_t)t * ld_out + (size_t)g * size + c] = from_f32<T>(y * scale);
        }
      }
    }
    return;
  }
  for (int i = threadIdx.x; i < size; i += blockDim.x) ss = fmaf(x[i], x[i], ss);
  ss = block_sum(ss, red);
  const float rstd = 1.0f / sqrtf(ss / (float)size + eps);
  for (int i = threadIdx.x; i < size; i += blockDim.x) {
    float y = x[i] * rstd * w[i];
    if (gate) y *= la_sigmoid(gate[(size_t)t * ld_gate + (size_t)g * size + i]);
    out[(size_t)t * ld_out + (size_t)g * size + i] = from_f32<T>(y * scale);
  }
}

TK_API int tk_group_norm_gate(int dt, const float* o, const float* gate, int ld_gate, const float* w, float eps, float scale,
                              void* out, int ld_out, int n_tokens, int groups, int size, hipStream_t stream) {
  TK_REQUIRE(n_tokens >= 0 && groups > 0 && size > 0 && o && w && out, "group_norm_gate: bad sizes %d %d %d or a pointer is missing",
             n_tokens, groups, size);
  TK_REQUIRE(ld_out >= groups * size && (!gate || ld_gate >= groups * size), "group_norm_gate: a row stride is too short");
  if (n_tokens == 0) return 0;
  const long units = (long)n_tokens * groups;
  const long blocks = (units + 3) / 4;
  TK_REQUIRE(units < (1l << 31), "group_norm_gate: too many rows");
  if (size > 256) {
    if (dt == TK_F32)
      hipLaunchKernelGGL(group_norm_gate_wide_kernel<float>, dim3((unsigned)units), dim3(256), 0, stream, o, gate, ld_gate, groups, w,
                         eps, scale, (float*)out, ld_out, size);
    else
      hipLaunchKernelGGL(group_norm_gate_wide_kernel<bf16_t>, dim3((unsigned)units), dim3(256), 0, stream, o, gate, ld_gate, groups, w,
                         eps, scale, (bf16_t*)out, ld_out, size);
    TK_CHECK_LAUNCH("group_norm_gate");
    return 0;
  }
  if (dt == TK_F32)
    hipLaunchKernelGGL(group_norm_gate_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, stream, o, gate, ld_gate, groups, w, eps,
                       scale, (float*)out, ld_out, units, size);
  else
    hipLaunchKernelGGL(group_norm_gate_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, stream, o, gate, ld_gate, groups, w, eps,
                       scale, (bf16_t*)out, ld_out, units, size);
  TK_CHECK_LAUNCH("group_norm_gate");
  return 0;
}

// --------------------------------------------------------------------------
// out[t, i] = x[t, i] * sigmoid(gate[t, i]) * scale, element by element (rows a stride apart), 32-bit arithmetic,
// one rounding.
// --------------------------------------------------------------------------
template <typename T>
__global__ void sigmoid_gate_kernel(const T* __restrict__ x, int ld_x, const T* __restrict__ gate, int ld_gate, float scale,
                                    T* __restrict__ out, int ld_out, int width) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  const size_t t = blockIdx.y;
  if (i < width)
    out[t * ld_out + i] = from_f32<T>(to_f32<T>(x[t * ld_x + i]) * la_sigmoid(to_f32<T>(gate[t * ld_gate + i])) * scale);
}

// (16 bytes a load where widths, strides and addresses allow)
template <typename T>
__global__ void sigmoid_gate_vec_kernel(const T* __restrict__ x, int ld_x, const T* __restrict__ gate, int ld_gate, float scale,
                                        T* __restrict__ out, int ld_out, int width) {
  constexpr int N = 16 / sizeof(T);
  union Piece { uint4 raw; T v[N]; };
  const int i = (blockIdx.x * blockDim.x + threadIdx.x) * N;
  const size_t t = blockIdx.y;
  if (i >= width) return;
  Piece a, g, o;
  a.raw = *(const uint4*)(x + t * ld_x + i);
  g.raw = *(const uint4*)(gate + t * ld_gate + i);
#pragma unroll
  for (int e = 0; e < N; ++e) o.v[e] = from_f32<T>(to_f32<T>(a.v[e]) * la_sigmoid(to_f32<T>(g.v[e])) * scale);
  *(uint4*)(out + t * ld_out + i) = o.raw;
}

TK_API int tk_sigmoid_gate(int dt, const void* x, int ld_x, const void* gate, int ld_gate, float scale, void* out, int ld_out,
                           int rows, int width, hipStream_t stream) {
  TK_REQUIRE(rows >= 0 && rows < 65536 && width > 0 && x && gate && out && ld_x >= width && ld_gate >= width && ld_out >= width,
             "sigmoid_gate: bad sizes %d %d, a pointer is missing or a stride is too short", rows, width);
  if (rows == 0) return 0;
  const dim3 grid((width + 255) / 256, rows);
  const int per = dt == TK_F32 ? 4 : 8;
  if (width % per == 0 && ld_x % per == 0 && ld_gate % per == 0 && ld_out % per == 0 &&
      (((uintptr_t)x | (uintptr_t)gate | (uintptr_t)out) & 15) == 0) {
    const dim3 vgrid((width / per + 127) / 128, rows);
    if (dt == TK_F32)
      hipLaunchKernelGGL(sigmoid_gate_vec_kernel<float>, vgrid, dim3(128), 0, stream, (const float*)x, ld_x, (const float*)gate,
                         ld_gate, scale, (float*)out, ld_out, width);
    else
      hipLaunchKernelGGL(sigmoid_gate_vec_kernel<bf16_t>, vgrid, dim3(128), 0, stream, (const bf16_t*)x, ld_x, (const bf16_t*)gate,
                         ld_gate, scale, (bf16_t*)out, ld_out, width);
    TK_CHECK_LAUNCH("sigmoid_gate");
    return 0;
  }
  if (dt == TK_F32)
    hipLaunchKernelGGL(sigmoid_gate_kernel<float>, grid, dim3(256), 0, stream, (const float*)x, ld_x, (const float*)gate, ld_gate,
                       scale, (float*)out, ld_out, width);
  else
    hipLaunchKernelGGL(sigmoid_gate_kernel<bf16_t>, grid, dim3(256), 0, stream, (const bf16_t*)x, ld_x, (const bf16_t*)gate, ld_gate,
                       scale, (bf16_t*)out, ld_out, width);
  TK_CHECK_LAUNCH("sigmoid_gate");
  return 0;
}

// --------------------------------------------------------------------------
// A short causal convolution over time on every channel, added to its input:
//     out_t = h_t + sum_j w[j][c] * h_(t - taps + 1 + j)      (zeros before a request's first token)
// The taps are kept tap by tap, w [taps][width], so that neighbouring channels' weights of one tap lie together.
// The last taps - 1 inputs of a request live in its slot's `tail` [taps - 1][width] (32-bit, oldest first,
// zeros when the request takes the slot).  A thread a (token, channel).  FUSE_TAIL (every request of the step
// brings one token): the thread also moves its channel's tail on, which it alone reads; else the tail kernel
// below runs afterwards.
// --------------------------------------------------------------------------
#define SC_MAX_TAPS 16
template <typename T, bool FUSE_TAIL>
__global__ void short_conv_kernel(const T* __restrict__ h, int ld, const float* __restrict__ w, int taps, float* __restrict__ tails,
                                  size_t tail_stride, const int* __restrict__ q_start, const int* __restrict__ token_req,
                                  const int* __restrict__ slots, T* __restrict__ out, int width) {
  const int t = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= width) return;
  const int r = token_req[t];
  const int first = q_start[r];
  const int local = t - first;
  float* tail = tails + (size_t)slots[r] * tail_stride;
  float acc = 0.f, cur = 0.f;
  for (int j = 0; j < taps; ++j) {
    const int src = local - (taps - 1) + j;
    const float x = src >= 0 ? to_f32<T>(h[(size_t)(first + src) * ld + c]) : tail[(size_t)(src + taps - 1) * width + c];
    acc = fmaf(w[(size_t)j * width + c], x, acc);
    cur = x;
    if (FUSE_TAIL && j >= 1) tail[(size_t)(j - 1) * width + c] = x;  // (local is 0: entry j - 1 was read a tap ago)
  }
  out[(size_t)t * width + c] = from_f32<T>(cur + acc);
}

// The same with 16 bytes a load: a thread 16 / sizeof(T) neighbouring channels (widths and strides that are multiples
// of that, rows that start at multiples of 16 bytes).
template <typename T, bool FUSE_TAIL>
__global__ void short_conv_vec_kernel(const T* __restrict__ h, int ld, const float* __restrict__ w, int taps, float* __restrict__ tails,
                                      size_t tail_stride, const int* __restrict__ q_start, const int* __restrict__ token_req,
                                      const int* __restrict__ slots, T* __restrict__ out, int width) {
  constexpr int N = 16 / sizeof(T);
  union Piece { uint4 raw; T v[N]; };
  const int t = blockIdx.y;
  const int c0 = (blockIdx.x * blockDim.x + threadIdx.x) * N;
  if (c0 >= width) return;
  const int r = token_req[t];
  const int first = q_start[r];
  const int local = t - first;
  float* tail = tails + (size_t)slots[r] * tail_stride;
  float acc[N], cur[N];
#pragma unroll
  for (int e = 0; e < N; ++e) acc[e] = cur[e] = 0.f;
#pragma unroll 4
  for (int j = 0; j < taps; ++j) {
    const int src = local - (taps - 1) + j;
    float x[N];
    if (src >= 0) {
      Piece p;
      p.raw = *(const uint4*)(h + (size_t)(first + src) * ld + c0);
#pragma unroll
      for (int e = 0; e < N; ++e) x[e] = to_f32<T>(p.v[e]);
    } else {
      const float4* from = (const float4*)(tail + (size_t)(src + taps - 1) * width + c0);
#pragma unroll
      for (int e = 0; e < N; e += 4) {
        const float4 v = from[e / 4];
        x[e] = v.x; x[e + 1] = v.y; x[e + 2] = v.z; x[e + 3] = v.w;
      }
    }
    const float4* wj = (const float4*)(w + (size_t)j * width + c0);
#pragma unroll
    for (int e = 0; e < N; e += 4) {
      const float4 g = wj[e / 4];
      acc[e] = fmaf(g.x, x[e], acc[e]); acc[e + 1] = fmaf(g.y, x[e + 1], acc[e + 1]);
      acc[e + 2] = fmaf(g.z, x[e + 2], acc[e + 2]); acc[e + 3] = fmaf(g.w, x[e + 3], acc[e + 3]);
    }
#pragma unroll
    for (int e = 0; e < N; ++e) cur[e] = x[e];
    if (FUSE_TAIL && j >= 1) {  // (local is 0: entry j - 1 was read a tap ago)
      float4* to = (float4*)(tail + (size_t)(j - 1) * width + c0);
#pragma unroll
      for (int e = 0; e < N; e += 4) to[e / 4] = make_float4(x[e], x[e + 1], x[e + 2], x[e + 3]);
    }
  }
  Piece o;
#pragma unroll
  for (int e = 0; e < N; ++e) o.v[e] = from_f32<T>(cur[e] + acc[e]);
  *(uint4*)(out + (size_t)t * width + c0) = o.raw;
}

// The tails after the step: the last taps - 1 inputs of every request, from this step's rows and, where the
// step brought fewer, from the old tail.  A thread a (request, channel); it reads all it needs before it writes.
template <typename T>
__global__ void short_conv_tail_kernel(const T* __restrict__ h, int ld, int taps, float* __restrict__ tails, size_t tail_stride,
                                       const int* __restrict__ q_start, const int* __restrict__ slots, int width) {
  const int r = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= width) return;
  const int first = q_start[r], n = q_start[r + 1] - first;
  float* tail = tails + (size_t)slots[r] * tail_stride;
  float keep[SC_MAX_TAPS];
#pragma unroll
  for (int s = 0; s < SC_MAX_TAPS - 1; ++s) {
    if (s < taps - 1) {
      const int src = n - (taps - 1) + s;
      keep[s] = src >= 0 ? to_f32<T>(h[(size_t)(first + src) * ld + c]) : tail[(size_t)(src + taps - 1) * width + c];
    }
  }
#pragma unroll
  for (int s = 0; s < SC_MAX_TAPS - 1; ++s)
    if (s < taps - 1) tail[(size_t)s * width + c] = keep[s];
}

TK_API int tk_short_conv(int dt, const void* h, int ld, const float* w, int taps, float* tails, size_t tail_stride,
                         const int* q_start, const int* token_req, const int* slots, void* out, int n_tokens, int n_requests,
                         int width, int single_tokens, hipStream_t stream) {
  TK_REQUIRE(n_tokens >= 0 && n_requests >= 0 && width > 0 && taps >= 1 && taps <= SC_MAX_TAPS && ld >= width,
             "short_conv: bad sizes tokens=%d requests=%d width=%d taps=%d", n_tokens, n_requests, width, taps);
  TK_REQUIRE(h && w && out && q_start && token_req && slots && (taps == 1 || (tails && tail_stride >= (size_t)(taps - 1) * width)),
             "short_conv: a pointer is missing or the tails' rows are too short");
  TK_REQUIRE(n_tokens < 65536 * 32 && n_requests < 65536, "short_conv: too many rows for one call");
  if (n_tokens == 0) return 0;
  TK_REQUIRE(n_tokens < 65536, "short_conv: %d tokens are too many for one call", n_tokens);
  const dim3 grid((width + 255) / 256, n_tokens), tail_grid((width + 255) / 256, n_requests);
  const int per = dt == TK_F32 ? 4 : 8;  // channels of 16 bytes
  const bool vec = width % per == 0 && ld % per == 0 && (((uintptr_t)h | (uintptr_t)out | (uintptr_t)w) & 15) == 0 &&
                   (taps == 1 || ((((uintptr_t)tails) & 15) == 0 && tail_stride % 4 == 0));
  const dim3 vgrid((width / per + 127) / 128, n_tokens);
#define SC_VEC(T)                                                                                                                    \
  do {                                                                                                                               \
    if (single_tokens)                                                                                                               \
      hipLaunchKernelGGL((short_conv_vec_kernel<T, true>), vgrid, dim3(128), 0, stream, (const T*)h, ld, w, taps, tails, tail_stride, \
                         q_start, token_req, slots, (T*)out, width);                                                                 \
    else {                                                                                                                           \
      hipLaunchKernelGGL((short_conv_vec_kernel<T, false>), vgrid, dim3(128), 0, stream, (const T*)h, ld, w, taps, tails,            \
                         tail_stride, q_start, token_req, slots, (T*)out, width);                                                    \
      if (taps > 1)                                                                                                                  \
        hipLaunchKernelGGL(short_conv_tail_kernel<T>, tail_grid, dim3(256), 0, stream, (const T*)h, ld, taps, tails, tail_stride,    \
                           q_start, slots, width);                                                                                   \
    }                                                                                                                                \
  } while (0)
  if (vec) {
    if (dt == TK_F32) SC_VEC(float);
    else SC_VEC(bf16_t);
    TK_CHECK_LAUNCH("short_conv");
    return 0;
  }
#undef SC_VEC
#define SC_CASE(T)                                                                                                                   \
  do {                                                                                                                               \
    if (single_tokens)                                                                                                               \
      hipLaunchKernelGGL((short_conv_kernel<T, true>), grid, dim3(256), 0, stream, (const T*)h, ld, w, taps, tails, tail_stride,     \
                         q_start, token_req, slots, (T*)out, width);                                                                 \
    else {                                                                                                                           \
      hipLaunchKernelGGL((short_conv_kernel<T, false>), grid, dim3(256), 0, stream, (const T*)h, ld, w, taps, tails, tail_stride,    \
                         q_start, token_req, slots, (T*)out, width);                                                                 \
      if (taps > 1)                                                                                                                  \
        hipLaunchKernelGGL(short_conv_tail_kernel<T>, tail_grid, dim3(256), 0, stream, (const T*)h, ld, taps, tails, tail_stride,    \
                           q_start, slots, width);                                                                                   \
    }                                                                                                                                \
  } while (0)
  if (dt == TK_F32) SC_CASE(float);
  else SC_CASE(bf16_t);
#undef SC_CASE
  TK_CHECK_LAUNCH("short_conv");
  return 0;
}
