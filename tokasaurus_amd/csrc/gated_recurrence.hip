// A gated recurrence whose gates read the current token only (minGRU): per channel
//     z = sigmoid(a + b_z),   u' = u + b_x,   cand = u' + 1/2 where u' >= 0, sigmoid(u') where u' < 0,
//     S_t = (1 - z) S_(t-1) + z cand,     out_t = S_t * silu(g)
// on the 32-bit sums of one stacked product whose rows are interleaved channel by channel, (a, u, g) of channel 0,
// then of channel 1, ..: a lane reads its channel's three sums as 12 neighbouring bytes and a wavefront 768 of a
// token's row (with [a | u | g] it read three pieces of 256 bytes thousands of bytes apart).  The two biases
// (32-bit, [b_z | b_x], or null) are added here, which saves the product a pass over its result.  The state S is one 32-bit number a
// channel in the request's slot; a step of any cut continues from it.  Everything is 32-bit
// arithmetic; `out` is rounded once to the storage type.
//
// A workgroup owns 64 neighbouring channels of one request (a lane a channel, so a wavefront's
// loads are whole lines).  The chain S_t is the only thing that is sequential: the W wavefronts of a
// workgroup each take L neighbouring tokens of a round of W * L, load them (a round ahead) and compute gates and
// candidates side by side, and then the state passes through the wavefronts in order, L
// multiply-adds each and nothing else (the products with the gates and the stores follow when the
// state has moved on).  The sums are those of the plain recurrence token by token, whatever the cut
// of the prompt and whatever W: the same bits.
#include "common.h"

// 1 / (1 + exp(-x)) on the hardware's own exponential and reciprocal (an instruction each, an ulp each): three of
// these a token and channel are most of this kernel's arithmetic, and with the library's exponential and an exact
// division they, not the chain or the bytes, set its time (exp2(inf) = inf gives 1 / inf = 0, exp2(-inf) = 0 gives 1).
__device__ __forceinline__ float sigmoid_hw(float x) {
  return __builtin_amdgcn_rcpf(1.0f + exp2f(x * -1.44269504088896341f));
}

template <typename T, int W, int L>
__global__ __launch_bounds__(W * TK_WAVE) void min_gru_kernel(const float* __restrict__ proj, int stride, const float* __restrict__ bias,
                                                              float* __restrict__ state, size_t state_stride,
                                                              const int* __restrict__ q_start, const int* __restrict__ slots,
                                                              T* __restrict__ out, int width) {
  __shared__ float carry[TK_WAVE];
  const int lane = threadIdx.x & (TK_WAVE - 1), wave = threadIdx.x / TK_WAVE;
  const int r = blockIdx.y;
  const int ch = blockIdx.x * TK_WAVE + lane;
  const bool live = ch < width;
  const int first = q_start[r], end = q_start[r + 1];
  float* sp = state + (size_t)slots[r] * state_stride + ch;
  const float bz = bias && live ? bias[ch] : 0.f, bx = bias && live ? bias[width + ch] : 0.f;
  if (wave == 0) carry[lane] = live ? *sp : 0.f;
  if (W > 1) __syncthreads();
  // a round's sums are asked for while the round before still hands the state on
  float ra[L], ru[L], rg[L];
  auto ask = [&](int base) {
    const int t0 = base + wave * L;
#pragma unroll
    for (int i = 0; i < L; ++i) {
      const bool in = live && t0 + i < end;
      const float* src = proj + (size_t)(in ? t0 + i : first) * stride + 3 * (live ? ch : 0);
      ra[i] = src[0];
      ru[i] = src[1];
      rg[i] = src[2];
    }
  };
  ask(first);
  for (int base = first; base < end; base += W * L) {
    const int t0 = base + wave * L;
    float keep[L], add[L], gate[L];
#pragma unroll
    for (int i = 0; i < L; ++i) {
      const float a = ra[i] + bz, u = ru[i] + bx, g = rg[i];
      const float z = sigmoid_hw(a);
      const float cand = u >= 0.f ? u + 0.5f : sigmoid_hw(u);
      keep[i] = 1.0f - z;
      add[i] = z * cand;
      gate[i] = g * sigmoid_hw(g);
    }
    if (base + W * L < end) ask(base + W * L);
#pragma unroll 1
    for (int phase = 0; phase < W; ++phase) {
      if (wave == phase && t0 < end) {
        float S = carry[lane];
#pragma unroll
        for (int i = 0; i < L; ++i) {
          if (t0 + i < end) S = fmaf(keep[i], S, add[i]);
          add[i] = S;  // the state behind token i
        }
        carry[lane] = S;
      }
      if (W > 1) __syncthreads();
    }
    if (live) {
#pragma unroll
      for (int i = 0; i < L; ++i)
        if (t0 + i < end) out[(size_t)(t0 + i) * width + ch] = from_f32<T>(add[i] * gate[i]);
    }
  }
  if (wave == 0 && live) *sp = carry[lane];
}

TK_API int tk_min_gru(int dt, const float* proj, int stride, const float* bias, float* state, size_t state_stride,
                      const int* q_start, const int* slots, void* out, int n_requests, int width, int longest, hipStream_t stream) {
  TK_REQUIRE(proj && state && q_start && slots && out && n_requests >= 0 && width > 0 && stride >= 3 * width && state_stride >= (size_t)width,
             "min_gru: bad arguments (requests %d, width %d, row stride %d)", n_requests, width, stride);
  if (n_requests == 0) return 0;
  TK_REQUIRE(n_requests < 65536, "min_gru: too many requests");
  const dim3 grid((width + TK_WAVE - 1) / TK_WAVE, n_requests);
#define MG_LAUNCH(T, W, L) hipLaunchKernelGGL((min_gru_kernel<T, W, L>), grid, dim3(W * TK_WAVE), 0, stream, proj, stride, bias, state, \
                                              state_stride, q_start, slots, (T*)out, width)
  if (longest <= 4) {
    if (dt == TK_F32) MG_LAUNCH(float, 1, 4); else MG_LAUNCH(bf16_t, 1, 4);
  } else if (longest <= 64) {
    if (dt == TK_F32) MG_LAUNCH(float, 4, 16); else MG_LAUNCH(bf16_t, 4, 16);
  } else {
    if (dt == TK_F32) MG_LAUNCH(float, 8, 16); else MG_LAUNCH(bf16_t, 8, 16);
  }
#undef MG_LAUNCH
  TK_CHECK_LAUNCH("min_gru");
  return 0;
}
