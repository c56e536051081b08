// A feed-forward made of many small gated experts of which a token uses a few, and the
// per-head products of a mixer whose heads share a latent.  T is the storage type of weights
// and activations; sums are 32-bit, and the router is 32-bit arithmetic throughout.
//
//   tk_expert_route      per token: logits over all experts, softmax, choice by score + correction
//                        inside the best groups of neighbouring experts, the chosen experts'
//                        scores as weights; optionally the sigmoid gate of a shared expert
//   tk_expert_gate_up    per (token, chosen expert): act(W_gate h) * (W_up h)
//   tk_expert_combine    per token: sum of weight * W_down(...) over its experts, weight * h for an
//                        identity expert, plus gate * (a shared expert's output)
//   tk_head_linear       y[t, h, :] = W[h] x[t, h, :]: one matrix a head
//   tk_squared_relu      x <- max(x, 0)^2, in place
//
// These kernels compute a row (a token, a pair) independently of every other row, with sums
// in an order that the sizes alone fix: a token's result does not depend on its batch.
#include <math.h>

#include "common.h"

// Sum over i < n of w[i] * x[i], the lanes of a wavefront taking pieces of 16 bytes in turn when
// both rows allow, single elements otherwise; every lane returns the sum.
template <typename T>
__device__ __forceinline__ float wave_dot(const T* __restrict__ w, const T* __restrict__ x, int n) {
  constexpr int V = 16 / sizeof(T);
  const int lane = threadIdx.x & (TK_WAVE - 1);
  float acc = 0.f;
  if (n % V == 0 && (((uintptr_t)w | (uintptr_t)x) & 15) == 0) {
    for (int i = lane * V; i < n; i += TK_WAVE * V) {
      const uint4 wa = *(const uint4*)(w + i), xa = *(const uint4*)(x + i);
      const T* wp = (const T*)&wa;
      const T* xp = (const T*)&xa;
#pragma unroll
      for (int e = 0; e < V; ++e) acc = fmaf(to_f32<T>(wp[e]), to_f32<T>(xp[e]), acc);
    }
  } else {
    for (int i = lane; i < n; i += TK_WAVE) acc = fmaf(to_f32<T>(w[i]), to_f32<T>(x[i]), acc);
  }
  return wave_sum(acc);
}

// The same for two rows of weights against one x, in one pass (each sum in the order wave_dot has).
template <typename T>
__device__ __forceinline__ void wave_dot2(const T* __restrict__ w0, const T* __restrict__ w1, const T* __restrict__ x, int n,
                                          float& d0, float& d1) {
  constexpr int V = 16 / sizeof(T);
  const int lane = threadIdx.x & (TK_WAVE - 1);
  float a0 = 0.f, a1 = 0.f;
  if (n % V == 0 && (((uintptr_t)w0 | (uintptr_t)w1 | (uintptr_t)x) & 15) == 0) {
    for (int i = lane * V; i < n; i += TK_WAVE * V) {
      const uint4 wa = *(const uint4*)(w0 + i), wb = *(const uint4*)(w1 + i), xa = *(const uint4*)(x + i);
      const T* wp = (const T*)&wa;
      const T* wq = (const T*)&wb;
      const T* xp = (const T*)&xa;
#pragma unroll
      for (int e = 0; e < V; ++e) {
        a0 = fmaf(to_f32<T>(wp[e]), to_f32<T>(xp[e]), a0);
        a1 = fmaf(to_f32<T>(wq[e]), to_f32<T>(xp[e]), a1);
      }
    }
  } else {
    for (int i = lane; i < n; i += TK_WAVE) {
      a0 = fmaf(to_f32<T>(w0[i]), to_f32<T>(x[i]), a0);
      a1 = fmaf(to_f32<T>(w1[i]), to_f32<T>(x[i]), a1);
    }
  }
  d0 = wave_sum(a0);
  d1 = wave_sum(a1);
}

// --------------------------------------------------------------------------
// The router.  One workgroup a token.  n_all = routed + identity experts.  ids [tokens, top] names
// the chosen experts in the order of their choice scores, weights [tokens, top] their softmax
// scores (the correction moves the choice, not the weight); with `norm_scale` != 0 the chosen scores divided by
// their sum (+ 1e-20) and multiplied by norm_scale.  Without `w_gate` a given `shared_gate` is filled with ones.
// --------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(1024) void expert_route_kernel(
    const T* __restrict__ h, int h_stride, const T* __restrict__ w_router, const float* __restrict__ correction,
    const T* __restrict__ w_gate, int width, int n_all, int groups, int keep, int top, int* __restrict__ ids,
    float* __restrict__ weights, float* __restrict__ shared_gate, float norm_scale) {
  extern __shared__ float sm[];
  float* score = sm;                 // [n_all] logits, then softmax scores
  float* choice = sm + n_all;        // [n_all] score + correction, -inf outside the kept groups and once taken
  float* mark = sm + 2 * n_all;      // [groups]
  const int t = blockIdx.x;
  const int lane = threadIdx.x & (TK_WAVE - 1), wave = threadIdx.x / TK_WAVE, nwaves = blockDim.x / TK_WAVE;
  const T* row = h + (size_t)t * h_stride;
  if (!w_gate && shared_gate && threadIdx.x == 0) shared_gate[t] = 1.f;
  for (int e = wave; e < n_all + (w_gate ? 1 : 0); e += nwaves) {
    const float d = wave_dot<T>(e < n_all ? w_router + (size_t)e * width : w_gate, row, width);
    if (lane == 0) {
      if (e < n_all) score[e] = d;
      else shared_gate[t] = 1.0f / (1.0f + expf(-d));
    }
  }
  __syncthreads();
  // the rest is the work of one wavefront; the others only keep the barriers
  const bool on = wave == 0;
  if (on) {
    float m = -INFINITY;
    for (int e = lane; e < n_all; e += TK_WAVE) m = fmaxf(m, score[e]);
    m = wave_max(m);
    float sum = 0.f;
    for (int e = lane; e < n_all; e += TK_WAVE) {
      const float x = expf(score[e] - m);
      score[e] = x;
      sum += x;
    }
    sum = wave_sum(sum);
    for (int e = lane; e < n_all; e += TK_WAVE) {
      const float s = score[e] / sum;
      score[e] = s;
      choice[e] = s + correction[e];
    }
  }
  __syncthreads();
  const int per = n_all / groups;
  if (on)
    for (int g = lane; g < groups; g += TK_WAVE) {
      float best = -INFINITY;
      for (int e = g * per; e < (g + 1) * per; ++e) best = fmaxf(best, choice[e]);
      mark[g] = best;
    }
  __syncthreads();
  if (on && keep < groups)
    for (int g = lane; g < groups; g += TK_WAVE) {
      int ahead = 0;  // groups that come before this one: a larger mark, or an equal one further left
      const float mine = mark[g];
      for (int o = 0; o < groups; ++o) ahead += (mark[o] > mine || (mark[o] == mine && o < g)) ? 1 : 0;
      if (ahead >= keep)
        for (int e = g * per; e < (g + 1) * per; ++e) choice[e] = -INFINITY;
    }
  __syncthreads();
  for (int r = 0; r < top; ++r) {
    if (on) {
      float best = -INFINITY;
      int at = 0x7fffffff;
      for (int e = lane; e < n_all; e += TK_WAVE) {
        const float c = choice[e];
        if (c > best) { best = c; at = e; }
      }
#pragma unroll
      for (int o = TK_WAVE / 2; o > 0; o >>= 1) {
        const float ob = __shfl_xor(best, o, TK_WAVE);
        const int oa = __shfl_xor(at, o, TK_WAVE);
        if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
      }
      if (at == 0x7fffffff) at = -1;  // fewer open experts than places: the place stays empty
      if (lane == 0) {
        ids[(size_t)t * top + r] = at;
        weights[(size_t)t * top + r] = at >= 0 ? score[at] : 0.f;
        if (at >= 0) choice[at] = -INFINITY;
      }
    }
    __syncthreads();
  }
  if (norm_scale != 0.f && threadIdx.x == 0) {
    float sum = 0.f;
    for (int r = 0; r < top; ++r) sum += weights[(size_t)t * top + r];
    for (int r = 0; r < top; ++r) weights[(size_t)t * top + r] = weights[(size_t)t * top + r] / (sum + 1e-20f) * norm_scale;
  }
}

TK_API int tk_expert_route(int dt, const void* h, int h_stride, const void* w_router, const float* correction,
                           const void* w_gate, int tokens, int width, int n_all, int groups, int keep, int top,
                           int* ids, float* weights, float* shared_gate, float norm_scale, hipStream_t stream) {
  TK_REQUIRE(tokens >= 0 && width > 0 && n_all > 0 && groups > 0 && n_all % groups == 0 && keep > 0 && keep <= groups &&
                 top > 0 && top <= n_all,
             "expert_route: bad sizes tokens=%d width=%d experts=%d groups=%d keep=%d top=%d", tokens, width, n_all,
             groups, keep, top);
  TK_REQUIRE(h && w_router && correction && ids && weights && (!w_gate || shared_gate) && h_stride >= width,
             "expert_route: a pointer is missing or the row stride is too short");
  const size_t smem = sizeof(float) * (size_t)(2 * n_all + groups);
  TK_REQUIRE(smem <= 48 * 1024, "expert_route: %d experts do not fit the local memory", n_all);
  if (tokens == 0) return 0;
  // a wavefront a logit where the step has few tokens (each dot product is a chain of loads), four wavefronts for many
  const int threads = tokens <= 64 ? 1024 : 256;
  if (dt == TK_F32)
    hipLaunchKernelGGL(expert_route_kernel<float>, dim3(tokens), dim3(threads), smem, stream, (const float*)h, h_stride,
                       (const float*)w_router, correction, (const float*)w_gate, width, n_all, groups, keep, top, ids,
                       weights, shared_gate, norm_scale);
  else
    hipLaunchKernelGGL(expert_route_kernel<bf16_t>, dim3(tokens), dim3(threads), smem, stream, (const bf16_t*)h, h_stride,
                       (const bf16_t*)w_router, correction, (const bf16_t*)w_gate, width, n_all, groups, keep, top, ids,
                       weights, shared_gate, norm_scale);
  TK_CHECK_LAUNCH("expert_route");
  return 0;
}

// --------------------------------------------------------------------------
// inter[pair, j] = silu(W_gate[e] h)_j * (W_up[e] h)_j for pair = (token, place), e = ids[pair] a routed
// expert (others are skipped).  w_gate_up: [experts][2 * ff][width], gate rows first.
// Workgroup (pair, block of EX_ROWS outputs), a wavefront an output at a time.
// --------------------------------------------------------------------------
#define EX_ROWS 4  // one output a wavefront: a step of few tokens is a chain of loads, so many short workgroups
template <typename T>
__global__ __launch_bounds__(256) void expert_gate_up_kernel(
    const T* __restrict__ h, int h_stride, const T* __restrict__ w_gate_up, const int* __restrict__ ids,
    T* __restrict__ inter, int width, int ff, int experts, int top) {
  const int pair = blockIdx.x;
  const int e = ids[pair];
  if (e < 0 || e >= experts) return;
  const int lane = threadIdx.x & (TK_WAVE - 1), wave = threadIdx.x / TK_WAVE, nwaves = blockDim.x / TK_WAVE;
  const T* row = h + (size_t)(pair / top) * h_stride;
  const T* wg = w_gate_up + (size_t)e * 2 * ff * width;
  const T* wu = wg + (size_t)ff * width;
  const int j0 = blockIdx.y * EX_ROWS;
  for (int j = j0 + wave; j < min(j0 + EX_ROWS, ff); j += nwaves) {
    float g, u;
    wave_dot2<T>(wg + (size_t)j * width, wu + (size_t)j * width, row, width, g, u);
    if (lane == 0) {
      // gate, up and the activation as the storage type sees them, as the dense feed-forward's epilogue
      const float gr = round_to<T>(g), ur = round_to<T>(u);
      const float a = round_to<T>(gr / (1.0f + expf(-gr)));
      inter[(size_t)pair * ff + j] = from_f32<T>(a * ur);
    }
  }
}

TK_API int tk_expert_gate_up(int dt, const void* h, int h_stride, const void* w_gate_up, const int* ids, void* inter,
                             int tokens, int width, int ff, int experts, int top, hipStream_t stream) {
  TK_REQUIRE(tokens >= 0 && width > 0 && ff > 0 && experts > 0 && top > 0 && h_stride >= width,
             "expert_gate_up: bad sizes tokens=%d width=%d ff=%d experts=%d top=%d", tokens, width, ff, experts, top);
  TK_REQUIRE(h && w_gate_up && ids && inter, "expert_gate_up: a pointer is missing");
  if (tokens == 0) return 0;
  const dim3 grid(tokens * top, (ff + EX_ROWS - 1) / EX_ROWS);
  TK_REQUIRE(grid.y < 65536, "expert_gate_up: an expert of %d rows is too large", ff);
  if (dt == TK_F32)
    hipLaunchKernelGGL(expert_gate_up_kernel<float>, grid, dim3(256), 0, stream, (const float*)h, h_stride,
                       (const float*)w_gate_up, ids, (float*)inter, width, ff, experts, top);
  else
    hipLaunchKernelGGL(expert_gate_up_kernel<bf16_t>, grid, dim3(256), 0, stream, (const bf16_t*)h, h_stride,
                       (const bf16_t*)w_gate_up, ids, (bf16_t*)inter, width, ff, experts, top);
  TK_CHECK_LAUNCH("expert_gate_up");
  return 0;
}

// --------------------------------------------------------------------------
// out[t, c] = sum over the places k of token t, in order, of
//     weights[t, k] * (W_down[e] inter[t, k])_c       e = ids[t, k] a routed expert
//     weights[t, k] * h[t, c]                         e an identity expert (e >= experts)
// plus shared_gate[t] * shared[t, c] when a shared expert's output is given.  out is 32-bit.
// w_down: [experts][width][ff].  Workgroup (token, block of EX_ROWS columns).
// --------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void expert_combine_kernel(
    const T* __restrict__ h, int h_stride, const T* __restrict__ inter, const T* __restrict__ w_down,
    const int* __restrict__ ids, const float* __restrict__ weights, const float* __restrict__ shared,
    const float* __restrict__ shared_gate, float* __restrict__ out, int width, int ff, int experts, int top) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & (TK_WAVE - 1), wave = threadIdx.x / TK_WAVE, nwaves = blockDim.x / TK_WAVE;
  const int c0 = blockIdx.y * EX_ROWS;
  for (int c = c0 + wave; c < min(c0 + EX_ROWS, width); c += nwaves) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k) {
      const int e = ids[(size_t)t * top + k];
      if (e < 0) continue;
      const float g = weights[(size_t)t * top + k];
      float y;
      if (e < experts)
        y = round_to<T>(wave_dot<T>(w_down + ((size_t)e * width + c) * ff, inter + ((size_t)t * top + k) * ff, ff));
      else
        y = to_f32<T>(h[(size_t)t * h_stride + c]);
      acc = fmaf(g, y, acc);
    }
    if (shared) acc = fmaf(shared_gate[t], shared[(size_t)t * width + c], acc);
    if (lane == 0) out[(size_t)t * width + c] = acc;
  }
}

TK_API int tk_expert_combine(int dt, const void* h, int h_stride, const void* inter, const void* w_down, const int* ids,
                             const float* weights, const float* shared, const float* shared_gate, float* out, int tokens,
                             int width, int ff, int experts, int top, hipStream_t stream) {
  TK_REQUIRE(tokens >= 0 && width > 0 && ff > 0 && experts > 0 && top > 0 && h_stride >= width,
             "expert_combine: bad sizes tokens=%d width=%d ff=%d experts=%d top=%d", tokens, width, ff, experts, top);
  TK_REQUIRE(h && inter && w_down && ids && weights && out && (!shared || shared_gate), "expert_combine: a pointer is missing");
  if (tokens == 0) return 0;
  const dim3 grid(tokens, (width + EX_ROWS - 1) / EX_ROWS);
  TK_REQUIRE(grid.y < 65536, "expert_combine: a width of %d is too large", width);
  if (dt == TK_F32)
    hipLaunchKernelGGL(expert_combine_kernel<float>, grid, dim3(256), 0, stream, (const float*)h, h_stride,
                       (const float*)inter, (const float*)w_down, ids, weights, shared, shared_gate, out, width, ff,
                       experts, top);
  else
    hipLaunchKernelGGL(expert_combine_kernel<bf16_t>, grid, dim3(256), 0, stream, (const bf16_t*)h, h_stride,
                       (const bf16_t*)inter, (const bf16_t*)w_down, ids, weights, shared, shared_gate, out, width, ff,
                       experts, top);
  TK_CHECK_LAUNCH("expert_combine");
  return 0;
}

// --------------------------------------------------------------------------
// y[t, hd * n_out + o] = sum_i W[hd][o][i] * x[t, hd * n_in + i]: a matrix a head.  y is T or 32-bit.
// Workgroup (token, head, block of HL_ROWS outputs).
// --------------------------------------------------------------------------
#define HL_ROWS 32
template <typename T, typename O>
__global__ __launch_bounds__(256) void head_linear_kernel(const T* __restrict__ x, int x_stride, const T* __restrict__ w,
                                                          O* __restrict__ y, int y_stride, int n_in, int n_out) {
  const int t = blockIdx.x, hd = blockIdx.y;
  const int lane = threadIdx.x & (TK_WAVE - 1), wave = threadIdx.x / TK_WAVE, nwaves = blockDim.x / TK_WAVE;
  const T* row = x + (size_t)t * x_stride + (size_t)hd * n_in;
  const T* wh = w + (size_t)hd * n_out * n_in;
  const int o0 = blockIdx.z * HL_ROWS;
  for (int o = o0 + wave; o < min(o0 + HL_ROWS, n_out); o += nwaves) {
    const float d = wave_dot<T>(wh + (size_t)o * n_in, row, n_in);
    if (lane == 0) y[(size_t)t * y_stride + (size_t)hd * n_out + o] = from_f32<O>(d);
  }
}

TK_API int tk_head_linear(int dt, const void* x, int x_stride, const void* w, void* y, int y_stride, int out_f32,
                          int tokens, int heads, int n_in, int n_out, hipStream_t stream) {
  TK_REQUIRE(tokens >= 0 && heads > 0 && n_in > 0 && n_out > 0 && x_stride >= heads * n_in && y_stride >= heads * n_out,
             "head_linear: bad sizes tokens=%d heads=%d in=%d out=%d strides %d %d", tokens, heads, n_in, n_out, x_stride,
             y_stride);
  TK_REQUIRE(x && w && y, "head_linear: a pointer is missing");
  if (tokens == 0) return 0;
  const dim3 grid(tokens, heads, (n_out + HL_ROWS - 1) / HL_ROWS);
  TK_REQUIRE(grid.y < 65536 && grid.z < 65536, "head_linear: too many heads or outputs");
  if (dt == TK_F32)
    hipLaunchKernelGGL((head_linear_kernel<float, float>), grid, dim3(256), 0, stream, (const float*)x, x_stride,
                       (const float*)w, (float*)y, y_stride, n_in, n_out);
  else if (out_f32)
    hipLaunchKernelGGL((head_linear_kernel<bf16_t, float>), grid, dim3(256), 0, stream, (const bf16_t*)x, x_stride,
                       (const bf16_t*)w, (float*)y, y_stride, n_in, n_out);
  else
    hipLaunchKernelGGL((head_linear_kernel<bf16_t, bf16_t>), grid, dim3(256), 0, stream, (const bf16_t*)x, x_stride,
                       (const bf16_t*)w, (bf16_t*)y, y_stride, n_in, n_out);
  TK_CHECK_LAUNCH("head_linear");
  return 0;
}

// --------------------------------------------------------------------------
// x <- max(x, 0)^2 in place.
// --------------------------------------------------------------------------
template <typename T>
__global__ void squared_relu_kernel(T* __restrict__ x, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) {
    const float v = fmaxf(to_f32<T>(x[i]), 0.f);
    x[i] = from_f32<T>(v * v);
  }
}

TK_API int tk_squared_relu(int dt, void* x, size_t n, hipStream_t stream) {
  if (n == 0) return 0;
  const size_t blocks = (n + 255) / 256;
  TK_REQUIRE(x && blocks < (1u << 31), "squared_relu: bad arguments");
  if (dt == TK_F32)
    hipLaunchKernelGGL(squared_relu_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, stream, (float*)x, n);
  else
    hipLaunchKernelGGL(squared_relu_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, stream, (bf16_t*)x, n);
  TK_CHECK_LAUNCH("squared_relu");
  return 0;
}
