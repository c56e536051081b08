// Kernels for models whose residual stream is kept in 32-bit whatever the storage type of
// the weights: a scaled embedding that writes 32-bit rows, the residual update
//     x <- x + mult * (a + b)
// of a block whose branches run side by side, fused with the RMS norms that read the new
// stream (one statistic, up to two weight vectors), and the soft cap of the logits.
// T is the storage type of the normed rows that the next products read.
#include "common.h"

// --------------------------------------------------------------------------
// out[t, :] = float(table[id_t, :]) * scale; id_t < 0 names slot -id_t-1 of `last_token`.
// `pos_table` (null or [n_pos, hidden]): the learned row of the token's position is added, as it is.
// --------------------------------------------------------------------------
template <typename T>
__global__ void embed_scaled_kernel(const int* __restrict__ ids, const int* __restrict__ last_token,
                                    const T* __restrict__ table, float* __restrict__ out, int hidden,
                                    int vocab, float scale, const T* __restrict__ pos_table,
                                    const int* __restrict__ positions, int n_pos) {
  const int t = blockIdx.x;
  int id = ids[t];
  if (id < 0) id = last_token[-id - 1];
  id = min(max(id, 0), vocab - 1);
  const T* src = table + (size_t)id * hidden;
  float* dst = out + (size_t)t * hidden;
  if (pos_table) {
    const T* add = pos_table + (size_t)min(max(positions[t], 0), n_pos - 1) * hidden;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = fmaf(to_f32<T>(src[i]), scale, to_f32<T>(add[i]));
  } else {
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = to_f32<T>(src[i]) * scale;
  }
}

TK_API int tk_embed_scaled(int dt, const int* ids, const int* last_token, const void* table,
                           float* out, int n_tokens, int hidden, int vocab, float scale,
                           const void* pos_table, const int* positions, int n_pos, hipStream_t stream) {
  TK_REQUIRE(n_tokens >= 0 && hidden > 0 && vocab > 0, "embed_scaled: bad sizes %d %d %d", n_tokens,
             hidden, vocab);
  TK_REQUIRE(!pos_table || (positions && n_pos > 0), "embed_scaled: a table of positions needs the tokens' positions");
  if (n_tokens == 0) return 0;
  if (dt == TK_F32)
    hipLaunchKernelGGL(embed_scaled_kernel<float>, dim3(n_tokens), dim3(256), 0, stream, ids,
                       last_token, (const float*)table, out, hidden, vocab, scale, (const float*)pos_table, positions, n_pos);
  else
    hipLaunchKernelGGL(embed_scaled_kernel<bf16_t>, dim3(n_tokens), dim3(256), 0, stream, ids,
                       last_token, (const bf16_t*)table, out, hidden, vocab, scale, (const bf16_t*)pos_table, positions, n_pos);
  TK_CHECK_LAUNCH("embed_scaled");
  return 0;
}

// --------------------------------------------------------------------------
// A weighted sum over the streams a model has had so far, row by row:
//     out[r, :] = sum_{j < count} w[j] * hist[j][row(r), :]  (+ w[count] * last[r, :])
// `hist` holds `count` streams of equal shape `stride` floats apart; row(r) = rows[r] where `rows` is given
// (the streams then have more rows than the result: only some are wanted), else r.  `last` (or null) is one
// more stream that already has the result's rows.  For a norm that reads the result (`nw`, or null) the row
//     out / sqrt(mean(out^2) + eps) * (offset + nw)
// is written too, rounded once to T.  One row a workgroup; the sum runs over j in ascending order.
// `a`, `b` (either may be null): the branches of the block that has just run, with the result's rows; the newest
// stream (`last`, or the last of `hist` without one) first becomes itself + mult * (a + b), in place: the block's
// residual sum and this average are one pass.
// --------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void depth_average_kernel(float* __restrict__ hist, size_t stride, int count,
                                                            float* __restrict__ last, const int* __restrict__ rows,
                                                            const float* __restrict__ w, float* __restrict__ out,
                                                            const float* __restrict__ nw, float offset, float eps,
                                                            T* __restrict__ normed, int hidden, const float* __restrict__ a,
                                                            const float* __restrict__ b, float mult) {
  __shared__ float red[16];
  const size_t r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : r;
  const bool pending = a || b;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float branch = 0.f;
    if (pending) {
      branch = a ? a[r * hidden + i] : 0.f;
      if (b) branch += b[r * hidden + i];
    }
    float acc = 0.f;
    for (int j = 0; j < count; ++j) {
      float v = hist[(size_t)j * stride + src * hidden + i];
      if (pending && !last && j == count - 1) {
        v = fmaf(mult, branch, v);
        hist[(size_t)j * stride + src * hidden + i] = v;
      }
      acc = fmaf(w[j], v, acc);
    }
    if (last) {
      float v = last[r * hidden + i];
      if (pending) {
        v = fmaf(mult, branch, v);
        last[r * hidden + i] = v;
      }
      acc = fmaf(w[count], v, acc);
    }
    out[r * hidden + i] = acc;
    ss = fmaf(acc, acc, ss);
  }
  if (!nw) return;
  ss = block_sum(ss, red);
  const float rstd = 1.0f / sqrtf(ss / (float)hidden + eps);
  for (int i = threadIdx.x; i < hidden; i += blockDim.x)  // a thread reads back what it wrote
    normed[r * hidden + i] = from_f32<T>(out[r * hidden + i] * rstd * (offset + nw[i]));
}

// The same with 16 bytes a load and the row's sums held in registers: for widths that are multiples of 4 up to
// 4 * 256 * DA_QUADS.  A thread's loads of one stream are all asked for before the first is used, so a row of a step
// of few tokens is no chain of waits.
#define DA_QUADS 8
template <typename T>
__global__ __launch_bounds__(256) void depth_average_vec_kernel(float* __restrict__ hist, size_t stride, int count,
                                                                float* __restrict__ last, const int* __restrict__ rows,
                                                                const float* __restrict__ w, float* __restrict__ out,
                                                                const float* __restrict__ nw, float offset, float eps,
                                                                T* __restrict__ normed, int hidden, const float* __restrict__ a,
                                                                const float* __restrict__ b, float mult) {
  __shared__ float red[16];
  const size_t r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : r;
  const int quads = hidden / 4;
  const bool pending = a || b;
  float4 acc[DA_QUADS], branch[DA_QUADS];
#pragma unroll
  for (int q = 0; q < DA_QUADS; ++q) {
    const int i = threadIdx.x + q * 256;
    acc[q] = make_float4(0.f, 0.f, 0.f, 0.f);
    branch[q] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (pending && i < quads) {
      if (a) branch[q] = ((const float4*)(a + r * hidden))[i];
      if (b) {
        const float4 z = ((const float4*)(b + r * hidden))[i];
        branch[q].x += z.x; branch[q].y += z.y; branch[q].z += z.z; branch[q].w += z.w;
      }
    }
  }
  const int streams = count + (last ? 1 : 0);
#pragma unroll 1
  for (int j = 0; j < streams; ++j) {
    const bool is_last = last && j == count;
    float* row = is_last ? last + r * hidden : hist + (size_t)j * stride + src * hidden;
    const bool newest = pending && j == streams - 1;
    const float wj = w[j];
    float4 v[DA_QUADS];
#pragma unroll
    for (int q = 0; q < DA_QUADS; ++q) {
      const int i = threadIdx.x + q * 256;
      if (i < quads) v[q] = ((const float4*)row)[i];
    }
#pragma unroll
    for (int q = 0; q < DA_QUADS; ++q) {
      const int i = threadIdx.x + q * 256;
      if (i < quads) {
        if (newest) {
          v[q].x = fmaf(mult, branch[q].x, v[q].x); v[q].y = fmaf(mult, branch[q].y, v[q].y);
          v[q].z = fmaf(mult, branch[q].z, v[q].z); v[q].w = fmaf(mult, branch[q].w, v[q].w);
          ((float4*)row)[i] = v[q];
        }
        acc[q].x = fmaf(wj, v[q].x, acc[q].x); acc[q].y = fmaf(wj, v[q].y, acc[q].y);
        acc[q].z = fmaf(wj, v[q].z, acc[q].z); acc[q].w = fmaf(wj, v[q].w, acc[q].w);
      }
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int q = 0; q < DA_QUADS; ++q) {
    const int i = threadIdx.x + q * 256;
    if (i < quads) {
      ((float4*)(out + r * hidden))[i] = acc[q];
      ss = fmaf(acc[q].x, acc[q].x, ss); ss = fmaf(acc[q].y, acc[q].y, ss);
      ss = fmaf(acc[q].z, acc[q].z, ss); ss = fmaf(acc[q].w, acc[q].w, ss);
    }
  }
  if (!nw) return;
  ss = block_sum(ss, red);
  const float rstd = 1.0f / sqrtf(ss / (float)hidden + eps);
#pragma unroll
  for (int q = 0; q < DA_QUADS; ++q) {
    const int i = threadIdx.x + q * 256;
    if (i < quads) {
      const float4 g = ((const float4*)nw)[i];
      const float n4[4] = {acc[q].x * rstd * (offset + g.x), acc[q].y * rstd * (offset + g.y), acc[q].z * rstd * (offset + g.z),
                           acc[q].w * rstd * (offset + g.w)};
#pragma unroll
      for (int e = 0; e < 4; ++e) normed[r * hidden + 4 * i + e] = from_f32<T>(n4[e]);
    }
  }
}

TK_API int tk_depth_average(int dt, float* hist, size_t stride, int count, float* last, const int* rows,
                            const float* w, float* out, const float* nw, float offset, float eps, void* normed,
                            int n_rows, int hidden, const float* a, const float* b, float mult, hipStream_t stream) {
  TK_REQUIRE(!(a || b) || last || !rows, "depth_average: branches are added to a stream that has the result's rows");
  TK_REQUIRE(n_rows >= 0 && hidden > 0 && count >= 0 && (count > 0 || last) && w && out && (count == 0 || hist),
             "depth_average: bad sizes rows=%d hidden=%d streams=%d or a pointer is missing", n_rows, hidden, count);
  TK_REQUIRE(!nw || normed, "depth_average: a norm's weight needs a place for its rows");
  if (n_rows == 0) return 0;
  auto aligned = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
  if (hidden % 4 == 0 && hidden <= 4 * 256 * DA_QUADS && stride % 4 == 0 && aligned(hist) && aligned(last) && aligned(out) &&
      aligned(nw) && aligned(a) && aligned(b)) {
    if (dt == TK_F32)
      hipLaunchKernelGGL(depth_average_vec_kernel<float>, dim3(n_rows), dim3(256), 0, stream, hist, stride, count, last, rows, w,
                         out, nw, offset, eps, (float*)normed, hidden, a, b, mult);
    else
      hipLaunchKernelGGL(depth_average_vec_kernel<bf16_t>, dim3(n_rows), dim3(256), 0, stream, hist, stride, count, last, rows, w,
                         out, nw, offset, eps, (bf16_t*)normed, hidden, a, b, mult);
    TK_CHECK_LAUNCH("depth_average");
    return 0;
  }
  if (dt == TK_F32)
    hipLaunchKernelGGL(depth_average_kernel<float>, dim3(n_rows), dim3(256), 0, stream, hist, stride, count, last, rows, w, out,
                       nw, offset, eps, (float*)normed, hidden, a, b, mult);
  else
    hipLaunchKernelGGL(depth_average_kernel<bf16_t>, dim3(n_rows), dim3(256), 0, stream, hist, stride, count, last, rows, w, out,
                       nw, offset, eps, (bf16_t*)normed, hidden, a, b, mult);
  TK_CHECK_LAUNCH("depth_average");
  return 0;
}

// --------------------------------------------------------------------------
// out[t, :] = float(table[id_t, :]) * scale + float(pairs[row_t, :]) where row_t is a hash of the
// token before and the token itself, (prev * mul_prev + id * mul_cur) mod buckets, and row `buckets`
// (the table's last) for a request's first token.  The token before is the one in front of it in this
// step, or, for the first token that a request brings in a step, the one kept in the request's slot
// (`prev_token`), where the workgroup of that first token then leaves the last token that the request
// brings in this step (it alone reads and writes the slot's entry).  `cast` (null or T rows): the
// same rows rounded once to the storage type.
// --------------------------------------------------------------------------
template <typename T>
__global__ void embed_bigram_kernel(const int* __restrict__ ids, const int* __restrict__ last_token, const int* __restrict__ positions,
                                    const int* __restrict__ token_req, const int* __restrict__ q_start, const int* __restrict__ slots,
                                    int* __restrict__ prev_token, const T* __restrict__ table, const T* __restrict__ pairs,
                                    float* __restrict__ out, T* __restrict__ cast, int hidden, int vocab, float scale,
                                    int buckets, int mul_prev, int mul_cur) {
  const int t = blockIdx.x;
  const int r = token_req[t];
  const int first = q_start[r], last = q_start[r + 1] - 1;
  auto token_at = [&](int i) {
    int id = ids[i];
    if (id < 0) id = last_token[-id - 1];
    return min(max(id, 0), vocab - 1);
  };
  const int id = token_at(t);
  int row = buckets;
  if (positions[t] > 0) {
    const int prev = t > first ? token_at(t - 1) : prev_token[slots[r]];
    row = (int)(((long long)prev * mul_prev + (long long)id * mul_cur) % buckets);
  }
  if (t == first && threadIdx.x == 0) prev_token[slots[r]] = token_at(last);
  const T* src = table + (size_t)id * hidden;
  const T* add = pairs + (size_t)row * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float v = fmaf(to_f32<T>(src[i]), scale, to_f32<T>(add[i]));
    out[(size_t)t * hidden + i] = v;
    if (cast) cast[(size_t)t * hidden + i] = from_f32<T>(v);
  }
}

TK_API int tk_embed_bigram(int dt, const int* ids, const int* last_token, const int* positions, const int* token_req,
                           const int* q_start, const int* slots, int* prev_token, const void* table, const void* pairs,
                           float* out, void* cast, int n_tokens, int hidden, int vocab, float scale, int buckets,
                           int mul_prev, int mul_cur, hipStream_t stream) {
  TK_REQUIRE(n_tokens >= 0 && hidden > 0 && vocab > 0 && buckets > 0, "embed_bigram: bad sizes %d %d %d %d", n_tokens, hidden, vocab, buckets);
  TK_REQUIRE(ids && positions && token_req && q_start && slots && prev_token && table && pairs && out, "embed_bigram: a pointer is missing");
  if (n_tokens == 0) return 0;
  if (dt == TK_F32)
    hipLaunchKernelGGL(embed_bigram_kernel<float>, dim3(n_tokens), dim3(256), 0, stream, ids, last_token, positions, token_req, q_start,
                       slots, prev_token, (const float*)table, (const float*)pairs, out, (float*)nullptr, hidden, vocab, scale, buckets,
                       mul_prev, mul_cur);
  else
    hipLaunchKernelGGL(embed_bigram_kernel<bf16_t>, dim3(n_tokens), dim3(256), 0, stream, ids, last_token, positions, token_req, q_start,
                       slots, prev_token, (const bf16_t*)table, (const bf16_t*)pairs, out, (bf16_t*)cast, hidden, vocab, scale, buckets,
                       mul_prev, mul_cur);
  TK_CHECK_LAUNCH("embed_bigram");
  return 0;
}

// --------------------------------------------------------------------------
// out = T(x): a 32-bit stream rounded once to the storage type that a product reads.
// --------------------------------------------------------------------------
template <typename T>
__global__ void cast_rows_kernel(const float* __restrict__ x, T* __restrict__ out, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = from_f32<T>(x[i]);
}

TK_API int tk_cast_rows(int dt, const float* x, void* out, size_t n, hipStream_t stream) {
  TK_REQUIRE(dt == TK_BF16 && x && out, "cast_rows: 32-bit rows to bfloat16 rows");
  if (n == 0) return 0;
  const size_t blocks = (n + 255) / 256;
  TK_REQUIRE(blocks < (1u << 31), "cast_rows: too many values");
  hipLaunchKernelGGL(cast_rows_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, stream, x, (bf16_t*)out, n);
  TK_CHECK_LAUNCH("cast_rows");
  return 0;
}

// --------------------------------------------------------------------------
// One row a workgroup.  Reads x (32-bit) and the branches a, b (32-bit, either may be null),
// writes x_out = x + mult * (a + b) (32-bit; may be x itself; null when there is no branch and
// the stream stays as it is) and, for each of up to two norms, the row
//     x_out / sqrt(mean(x_out^2) + eps) * (offset + w)
// rounded once to T.  `offset` is 1 for weights stored around zero, 0 for plain ones.
// Norm weights are 32-bit.
// --------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void residual_norm_kernel(
    const float* __restrict__ x, const float* __restrict__ a, const float* __restrict__ b, float mult,
    float* x_out, const float* __restrict__ w1, const float* __restrict__ w2, float offset, float eps,
    T* __restrict__ h1, T* __restrict__ h2, int hidden) {
  __shared__ float red[16];
  const size_t row = (size_t)blockIdx.x * hidden;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float v = x[row + i];
    if (a || b) {
      float y = a ? a[row + i] : 0.f;
      if (b) y += b[row + i];
      v = fmaf(mult, y, v);
      x_out[row + i] = v;
    }
    ss = fmaf(v, v, ss);
  }
  if (!w1 && !w2) return;
  ss = block_sum(ss, red);
  const float rstd = 1.0f / sqrtf(ss / (float)hidden + eps);
  const float* src = (a || b) ? x_out : x;  // a thread reads back what it wrote
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float n = src[row + i] * rstd;
    if (w1) h1[row + i] = from_f32<T>(n * (offset + w1[i]));
    if (w2) h2[row + i] = from_f32<T>(n * (offset + w2[i]));
  }
}

// The same with 16 bytes a load and the new row held in registers between the two passes: for
// widths that are multiples of 4 up to 4 * 256 * RN_QUADS (one workgroup of 256 threads a row).
#define RN_QUADS 8
template <typename T>
__global__ __launch_bounds__(256) void residual_norm_vec_kernel(
    const float* __restrict__ x, const float* __restrict__ a, const float* __restrict__ b, float mult,
    float* x_out, const float* __restrict__ w1, const float* __restrict__ w2, float offset, float eps,
    T* __restrict__ h1, T* __restrict__ h2, int hidden) {
  __shared__ float red[16];
  const size_t row = (size_t)blockIdx.x * hidden;
  const int quads = hidden / 4;
  float4 v[RN_QUADS];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < RN_QUADS; ++j) {
    const int i = threadIdx.x + j * 256;
    if (i < quads) {
      v[j] = ((const float4*)(x + row))[i];
      if (a || b) {
        float4 y = a ? ((const float4*)(a + row))[i] : make_float4(0.f, 0.f, 0.f, 0.f);
        if (b) {
          const float4 z = ((const float4*)(b + row))[i];
          y.x += z.x; y.y += z.y; y.z += z.z; y.w += z.w;
        }
        v[j].x = fmaf(mult, y.x, v[j].x); v[j].y = fmaf(mult, y.y, v[j].y);
        v[j].z = fmaf(mult, y.z, v[j].z); v[j].w = fmaf(mult, y.w, v[j].w);
        ((float4*)(x_out + row))[i] = v[j];
      }
      ss = fmaf(v[j].x, v[j].x, ss); ss = fmaf(v[j].y, v[j].y, ss);
      ss = fmaf(v[j].z, v[j].z, ss); ss = fmaf(v[j].w, v[j].w, ss);
    }
  }
  if (!w1 && !w2) return;
  ss = block_sum(ss, red);
  const float rstd = 1.0f / sqrtf(ss / (float)hidden + eps);
#pragma unroll
  for (int j = 0; j < RN_QUADS; ++j) {
    const int i = threadIdx.x + j * 256;
    if (i < quads) {
      const float n[4] = {v[j].x * rstd, v[j].y * rstd, v[j].z * rstd, v[j].w * rstd};
      if (w1) {
        const float4 w = ((const float4*)w1)[i];
        const float ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) h1[row + 4 * i + e] = from_f32<T>(n[e] * (offset + ww[e]));
      }
      if (w2) {
        const float4 w = ((const float4*)w2)[i];
        const float ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) h2[row + 4 * i + e] = from_f32<T>(n[e] * (offset + ww[e]));
      }
    }
  }
}

TK_API int tk_residual_norm(int dt, const float* x, const float* a, const float* b, float mult,
                            float* x_out, const float* w1, const float* w2, float offset, float eps,
                            void* h1, void* h2, int rows, int hidden, hipStream_t stream) {
  TK_REQUIRE(rows >= 0 && hidden > 0, "residual_norm: bad sizes %d %d", rows, hidden);
  TK_REQUIRE(!(a || b) || x_out, "residual_norm: a branch needs a place for the new stream");
  TK_REQUIRE((!w1 || h1) && (!w2 || h2), "residual_norm: a norm needs a place for its rows");
  if (rows == 0) return 0;
  const uintptr_t all = (uintptr_t)x | (uintptr_t)a | (uintptr_t)b | (uintptr_t)x_out | (uintptr_t)w1 | (uintptr_t)w2;
  if (hidden % 4 == 0 && hidden <= 4 * 256 * RN_QUADS && (all & 15) == 0) {
    if (dt == TK_F32)
      hipLaunchKernelGGL(residual_norm_vec_kernel<float>, dim3(rows), dim3(256), 0, stream, x, a, b, mult, x_out, w1, w2,
                         offset, eps, (float*)h1, (float*)h2, hidden);
    else
      hipLaunchKernelGGL(residual_norm_vec_kernel<bf16_t>, dim3(rows), dim3(256), 0, stream, x, a, b, mult, x_out, w1, w2,
                         offset, eps, (bf16_t*)h1, (bf16_t*)h2, hidden);
    TK_CHECK_LAUNCH("residual_norm");
    return 0;
  }
  if (dt == TK_F32)
    hipLaunchKernelGGL(residual_norm_kernel<float>, dim3(rows), dim3(256), 0, stream, x, a, b, mult,
                       x_out, w1, w2, offset, eps, (float*)h1, (float*)h2, hidden);
  else
    hipLaunchKernelGGL(residual_norm_kernel<bf16_t>, dim3(rows), dim3(256), 0, stream, x, a, b, mult,
                       x_out, w1, w2, offset, eps, (bf16_t*)h1, (bf16_t*)h2, hidden);
  TK_CHECK_LAUNCH("residual_norm");
  return 0;
}

// --------------------------------------------------------------------------
// The update of a stream whose branches are normed before they are added (a norm in front of and
// behind every sublayer), one row a workgroup:
//     x_out = x + a / sqrt(mean(a^2) + eps_b) * wb
// and, when w is given, the row of the norm that reads the new stream,
//     h = x_out / sqrt(mean(x_out^2) + eps) * w     rounded once to T;
// with h and no w, h is x_out itself rounded once to T (for sublayers that read the stream unnormed).
// x, a, wb, w are 32-bit.  x_out may be x itself.  The row is held in registers between the
// passes when the width allows (multiples of 4 up to 4 * 256 * RN_QUADS), else read back.
// --------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void post_norm_residual_kernel(
    const float* x, const float* __restrict__ a, const float* __restrict__ wb, float eps_b,
    float* x_out, const float* __restrict__ w, float eps, T* __restrict__ h, int hidden) {
  __shared__ float red[16];
  const size_t row = (size_t)blockIdx.x * hidden;
  float sa = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float y = a[row + i];
    sa = fmaf(y, y, sa);
  }
  const float rb = 1.0f / sqrtf(block_sum(sa, red) / (float)hidden + eps_b);
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float v = x[row + i] + a[row + i] * rb * wb[i];
    x_out[row + i] = v;
    ss = fmaf(v, v, ss);
  }
  if (!h) return;
  if (!w) {  // the new stream itself, rounded once
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) h[row + i] = from_f32<T>(x_out[row + i]);
    return;
  }
  const float rstd = 1.0f / sqrtf(block_sum(ss, red) / (float)hidden + eps);
  for (int i = threadIdx.x; i < hidden; i += blockDim.x)  // a thread reads back what it wrote
    h[row + i] = from_f32<T>(x_out[row + i] * rstd * w[i]);
}

template <typename T>
__global__ __launch_bounds__(256) void post_norm_residual_vec_kernel(
    const float* x, const float* __restrict__ a, const float* __restrict__ wb, float eps_b,
    float* x_out, const float* __restrict__ w, float eps, T* __restrict__ h, int hidden) {
  __shared__ float red[16];
  const size_t row = (size_t)blockIdx.x * hidden;
  const int quads = hidden / 4;
  float4 v[RN_QUADS];
  float sa = 0.f;
#pragma unroll
  for (int j = 0; j < RN_QUADS; ++j) {
    const int i = threadIdx.x + j * 256;
    if (i < quads) {
      v[j] = ((const float4*)(a + row))[i];
      sa = fmaf(v[j].x, v[j].x, sa); sa = fmaf(v[j].y, v[j].y, sa);
      sa = fmaf(v[j].z, v[j].z, sa); sa = fmaf(v[j].w, v[j].w, sa);
    }
  }
  const float rb = 1.0f / sqrtf(block_sum(sa, red) / (float)hidden + eps_b);
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < RN_QUADS; ++j) {
    const int i = threadIdx.x + j * 256;
    if (i < quads) {
      const float4 xv = ((const float4*)(x + row))[i];
      const float4 g = ((const float4*)wb)[i];
      v[j].x = xv.x + v[j].x * rb * g.x; v[j].y = xv.y + v[j].y * rb * g.y;
      v[j].z = xv.z + v[j].z * rb * g.z; v[j].w = xv.w + v[j].w * rb * g.w;
      ((float4*)(x_out + row))[i] = v[j];
      ss = fmaf(v[j].x, v[j].x, ss); ss = fmaf(v[j].y, v[j].y, ss);
      ss = fmaf(v[j].z, v[j].z, ss); ss = fmaf(v[j].w, v[j].w, ss);
    }
  }
  if (!h) return;
  const float rstd = w ? 1.0f / sqrtf(block_sum(ss, red) / (float)hidden + eps) : 1.f;
#pragma unroll
  for (int j = 0; j < RN_QUADS; ++j) {
    const int i = threadIdx.x + j * 256;
    if (i < quads) {
      const float4 g = w ? ((const float4*)w)[i] : make_float4(1.f, 1.f, 1.f, 1.f);
      const float n[4] = {v[j].x * rstd * g.x, v[j].y * rstd * g.y, v[j].z * rstd * g.z, v[j].w * rstd * g.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) h[row + 4 * i + e] = from_f32<T>(n[e]);
    }
  }
}

TK_API int tk_post_norm_residual(int dt, const float* x, const float* a, const float* wb, float eps_b, float* x_out,
                                 const float* w, float eps, void* h, int rows, int hidden, hipStream_t stream) {
  TK_REQUIRE(rows >= 0 && hidden > 0, "post_norm_residual: bad sizes %d %d", rows, hidden);
  TK_REQUIRE(x && a && wb && x_out && (!w || h), "post_norm_residual: a pointer is missing");
  TK_REQUIRE(w || !h || dt != TK_F32, "post_norm_residual: 32-bit rows of the stream itself are the stream");
  if (rows == 0) return 0;
  const uintptr_t all = (uintptr_t)x | (uintptr_t)a | (uintptr_t)wb | (uintptr_t)x_out | (uintptr_t)w;
  const bool vec = hidden % 4 == 0 && hidden <= 4 * 256 * RN_QUADS && (all & 15) == 0;
#define PNR_LAUNCH(K, T) hipLaunchKernelGGL(K<T>, dim3(rows), dim3(256), 0, stream, x, a, wb, eps_b, x_out, w, eps, (T*)h, hidden)
  if (vec) {
    if (dt == TK_F32) PNR_LAUNCH(post_norm_residual_vec_kernel, float); else PNR_LAUNCH(post_norm_residual_vec_kernel, bf16_t);
  } else {
    if (dt == TK_F32) PNR_LAUNCH(post_norm_residual_kernel, float); else PNR_LAUNCH(post_norm_residual_kernel, bf16_t);
  }
#undef PNR_LAUNCH
  TK_CHECK_LAUNCH("post_norm_residual");
  return 0;
}

// --------------------------------------------------------------------------
// out[t, :] = T([x[t, :] | y[t, :]]): two 32-bit streams side by side, rounded once to the storage
// type that a product reads.
// --------------------------------------------------------------------------
template <typename T>
__global__ void concat_cast_kernel(const float* __restrict__ x, const float* __restrict__ y, T* __restrict__ out, int hidden) {
  const size_t row = blockIdx.x;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    out[row * 2 * hidden + i] = from_f32<T>(x[row * hidden + i]);
    out[row * 2 * hidden + hidden + i] = from_f32<T>(y[row * hidden + i]);
  }
}

TK_API int tk_concat_cast(int dt, const float* x, const float* y, void* out, int rows, int hidden, hipStream_t stream) {
  TK_REQUIRE(rows >= 0 && hidden > 0 && x && y && out, "concat_cast: bad arguments");
  if (rows == 0) return 0;
  if (dt == TK_F32)
    hipLaunchKernelGGL(concat_cast_kernel<float>, dim3(rows), dim3(256), 0, stream, x, y, (float*)out, hidden);
  else
    hipLaunchKernelGGL(concat_cast_kernel<bf16_t>, dim3(rows), dim3(256), 0, stream, x, y, (bf16_t*)out, hidden);
  TK_CHECK_LAUNCH("concat_cast");
  return 0;
}

// --------------------------------------------------------------------------
// logits <- cap * tanh(logits / cap), in place, 32-bit.
// --------------------------------------------------------------------------
__global__ void softcap_kernel(float* __restrict__ v, size_t n, float cap) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) v[i] = cap * tanhf(v[i] / cap);
}

// logits <- logits * scale, in place, 32-bit.
__global__ void scale_values_kernel(float* __restrict__ v, size_t n, float scale) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) v[i] = v[i] * scale;
}

TK_API int tk_scale_values(float* v, size_t n, float scale, hipStream_t stream) {
  if (n == 0) return 0;
  const size_t blocks = (n + 255) / 256;
  TK_REQUIRE(v && blocks < (1u << 31), "scale_values: bad arguments");
  hipLaunchKernelGGL(scale_values_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, v, n, scale);
  TK_CHECK_LAUNCH("scale_values");
  return 0;
}

TK_API int tk_softcap(float* v, size_t n, float cap, hipStream_t stream) {
  TK_REQUIRE(cap > 0.f, "softcap: the cap must be positive");
  if (n == 0) return 0;
  const size_t blocks = (n + 255) / 256;
  TK_REQUIRE(blocks < (1u << 31), "softcap: too many values");
  hipLaunchKernelGGL(softcap_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, v, n, cap);
  TK_CHECK_LAUNCH("softcap");
  return 0;
}
