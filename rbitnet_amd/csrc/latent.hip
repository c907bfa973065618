// Attention through a latent: every token leaves one vector c of kv_rank numbers in the cache, and each head's
// keys and values are products of c with matrices of that head.  The products are moved to the query's side, so that
// attention runs over the cached latents themselves, as one key/value head of size kv_rank that all query heads share:
//   score = q . (Wk c) = (Wk^T q) . c,      out = Wv (sum_j p_j c_j)
// Here: the RMS norms of the two down-projections with the cache write, and the per-head products on either side
// of attention.  float32 arithmetic; storage float32 or bfloat16.
#include <math.h>

#include "api.h"
#include "common.h"

// proj [T, stride] float32 holds, per token, q_rank numbers at column 0 and kv_rank numbers at column kv_col.
// cq[t] = rmsnorm(proj[t, 0:q_rank]) * q_gain; c = rmsnorm(proj[t, kv_col:kv_col + kv_rank]) * kv_gain goes into the
// token's place of the cache pages [pages, 1, 64, kv_rank].  Either half may be absent (rank 0).
template <typename TC>
__global__ void latent_norm_store_kernel(const float* __restrict__ proj, size_t stride, int q_rank,
                                         const float* __restrict__ q_gain, TC* __restrict__ cq, int kv_col, int kv_rank,
                                         const float* __restrict__ kv_gain, TC* __restrict__ pages,
                                         const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ tok_seq,
                                         const int32_t* __restrict__ block_table, int bt_stride, float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const float* row = proj + (size_t)t * stride;
  if (q_rank > 0) {
    float ss = 0.f;
    for (int j = threadIdx.x; j < q_rank; j += blockDim.x) ss = fmaf(row[j], row[j], ss);
    const float f = 1.0f / sqrtf(block_sum(ss, scratch) / (float)q_rank + eps);
    for (int j = threadIdx.x; j < q_rank; j += blockDim.x) Num<TC>::store(cq + (size_t)t * q_rank + j, row[j] * f * q_gain[j]);
  }
  if (kv_rank > 0) {
    const int pos = tok_pos[t];
    const int page = block_table[(size_t)tok_seq[t] * bt_stride + pos / RB_PAGE];
    TC* dst = pages + ((size_t)page * RB_PAGE + (size_t)(pos % RB_PAGE)) * kv_rank;
    const float* src = row + kv_col;
    float ss = 0.f;
    for (int j = threadIdx.x; j < kv_rank; j += blockDim.x) ss = fmaf(src[j], src[j], ss);
    const float f = 1.0f / sqrtf(block_sum(ss, scratch) / (float)kv_rank + eps);
    for (int j = threadIdx.x; j < kv_rank; j += blockDim.x) Num<TC>::store(dst + j, src[j] * f * kv_gain[j]);
  }
}

extern "C" int rb_latent_norm_store(const float* proj, long long stride, int q_rank, const float* q_gain, void* cq,
                                    int kv_col, int kv_rank, const float* kv_gain, void* pages, int dtype,
                                    const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* block_table,
                                    int bt_stride, float eps, int n_tokens, void* stream) {
  RB_RECORDED(rb_latent_norm_store(proj, stride, q_rank, q_gain, cq, kv_col, kv_rank, kv_gain, pages, dtype, tok_pos, tok_seq,
                                   block_table, bt_stride, eps, n_tokens, stream));
  RB_REQUIRE(n_tokens >= 0 && q_rank >= 0 && kv_rank >= 0 && kv_col >= 0, "rb_latent_norm_store: bad sizes");
  RB_REQUIRE(stride >= q_rank && stride >= (long long)kv_col + kv_rank, "rb_latent_norm_store: the row stride is too short");
  RB_REQUIRE(kv_rank == 0 || (pages && block_table), "rb_latent_norm_store: a latent needs cache pages");
  if (n_tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == RB_F32)
    latent_norm_store_kernel<float><<<n_tokens, 256, 0, s>>>(proj, (size_t)stride, q_rank, q_gain, (float*)cq, kv_col, kv_rank,
                                                             kv_gain, (float*)pages, tok_pos, tok_seq, block_table, bt_stride, eps);
  else if (dtype == RB_BF16)
    latent_norm_store_kernel<bf16_t><<<n_tokens, 256, 0, s>>>(proj, (size_t)stride, q_rank, q_gain, (bf16_t*)cq, kv_col, kv_rank,
                                                              kv_gain, (bf16_t*)pages, tok_pos, tok_seq, block_table, bt_stride, eps);
  else
    RB_REQUIRE(false, "rb_latent_norm_store: unknown dtype %d", dtype);
  RB_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- a product per head
// y[t, h, n] = sum_k w[h, k, n] * x[t, h, k]: H small matrices, stored [H, K, N] (the output index runs fastest, so
// that neighbouring lanes read neighbouring weights).  A workgroup of four waves takes HL_TOKENS tokens and 64 output
// columns of one head: the tokens' inputs in LDS, a lane per column with one sum per token; the waves share the inner
// index (wave w takes k = w, w + 4, ...), sixteen weights in flight per lane (the scheduler is told not to move a load
// down to its use: it would trade the registers for a trip to memory per weight), and add up through LDS in a fixed order.
#define HL_TOKENS 16
#define HL_WAVES 4
template <typename TX, typename TW, typename TY>
__global__ __launch_bounds__(RB_WAVE * HL_WAVES) void heads_linear_kernel(const TX* __restrict__ x, const TW* __restrict__ w,
                                                                          TY* __restrict__ y, int n_tokens, int n_heads, int n, int k) {
  extern __shared__ float xs[];                  // [HL_TOKENS][k], then [HL_WAVES - 1][HL_TOKENS][64] partial sums
  float* part = xs + HL_TOKENS * k;
  const int t0 = blockIdx.x * HL_TOKENS, h = blockIdx.y;
  const int lane = threadIdx.x & (RB_WAVE - 1), wave = threadIdx.x / RB_WAVE;
  const int nt = n_tokens - t0 < HL_TOKENS ? n_tokens - t0 : HL_TOKENS;
  // the tokens' inputs, eight loads in flight per lane (a step of few tokens is a chain of trips to memory otherwise)
  for (int base = 0; base < HL_TOKENS * k; base += 8 * RB_WAVE * HL_WAVES) {
    float v[8];
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const int idx = base + it * RB_WAVE * HL_WAVES + threadIdx.x;
      const int tt = idx / k, kk = idx - tt * k;
      v[it] = (idx < HL_TOKENS * k && tt < nt) ? Num<TX>::load(x + ((size_t)(t0 + tt) * n_heads + h) * k + kk) : 0.f;
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const int idx = base + it * RB_WAVE * HL_WAVES + threadIdx.x;
      if (idx < HL_TOKENS * k) xs[idx] = v[it];
    }
  }
  __syncthreads();
  const int col = blockIdx.z * RB_WAVE + lane;
  const bool on = col < n;
  const TW* wh = w + (size_t)h * k * n + (on ? col : 0);
  float acc[HL_TOKENS];
#pragma unroll
  for (int tt = 0; tt < HL_TOKENS; ++tt) acc[tt] = 0.f;
  int kk = wave;
  for (; kk + 15 * HL_WAVES < k; kk += 16 * HL_WAVES) {
    float wv[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) wv[j] = Num<TW>::load(wh + (size_t)(kk + j * HL_WAVES) * n);
    __builtin_amdgcn_sched_barrier(0);          // all sixteen loads are issued before the first is waited for
#pragma unroll
    for (int j = 0; j < 16; ++j)
#pragma unroll
      for (int tt = 0; tt < HL_TOKENS; ++tt) acc[tt] = fmaf(wv[j], xs[tt * k + kk + j * HL_WAVES], acc[tt]);
  }
  for (; kk < k; kk += HL_WAVES) {
    const float wv = Num<TW>::load(wh + (size_t)kk * n);
#pragma unroll
    for (int tt = 0; tt < HL_TOKENS; ++tt) acc[tt] = fmaf(wv, xs[tt * k + kk], acc[tt]);
  }
  if (wave > 0) {
#pragma unroll
    for (int tt = 0; tt < HL_TOKENS; ++tt) part[((wave - 1) * HL_TOKENS + tt) * RB_WAVE + lane] = acc[tt];
  }
  __syncthreads();
  if (wave > 0 || !on) return;
#pragma unroll
  for (int tt = 0; tt < HL_TOKENS; ++tt) {
    float v = acc[tt];
#pragma unroll
    for (int ww = 0; ww < HL_WAVES - 1; ++ww) v += part[(ww * HL_TOKENS + tt) * RB_WAVE + lane];
    if (tt < nt) Num<TY>::store(y + ((size_t)(t0 + tt) * n_heads + h) * n + col, v);
  }
}

template <typename TX, typename TW, typename TY>
static void launch_heads_linear(const void* x, const void* w, void* y, int n_tokens, int n_heads, int n, int k, hipStream_t s) {
  dim3 grid((n_tokens + HL_TOKENS - 1) / HL_TOKENS, n_heads, (n + RB_WAVE - 1) / RB_WAVE);
  const size_t lds = ((size_t)HL_TOKENS * k + (size_t)(HL_WAVES - 1) * HL_TOKENS * RB_WAVE) * sizeof(float);
  heads_linear_kernel<TX, TW, TY><<<grid, RB_WAVE * HL_WAVES, lds, s>>>((const TX*)x, (const TW*)w, (TY*)y, n_tokens, n_heads, n, k);
}

extern "C" int rb_heads_linear(const void* x, int x_dtype, const void* w, int w_dtype, void* y, int y_dtype, int n_tokens,
                               int n_heads, int n, int k, void* stream) {
  RB_RECORDED(rb_heads_linear(x, x_dtype, w, w_dtype, y, y_dtype, n_tokens, n_heads, n, k, stream));
  RB_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_heads <= 65535 && n > 0 && n <= 65535 * 64 && k > 0, "rb_heads_linear: bad sizes");
  RB_REQUIRE(k <= 768, "rb_heads_linear: inner size %d not supported (at most 768)", k);
  if (n_tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int key = x_dtype * 4 + w_dtype * 2 + y_dtype;
  switch (key) {
    case 0: launch_heads_linear<float, float, float>(x, w, y, n_tokens, n_heads, n, k, s); break;
    case 3: launch_heads_linear<float, bf16_t, bf16_t>(x, w, y, n_tokens, n_heads, n, k, s); break;
    case 6: launch_heads_linear<bf16_t, bf16_t, float>(x, w, y, n_tokens, n_heads, n, k, s); break;
    case 7: launch_heads_linear<bf16_t, bf16_t, bf16_t>(x, w, y, n_tokens, n_heads, n, k, s); break;
    case 2: launch_heads_linear<float, bf16_t, float>(x, w, y, n_tokens, n_heads, n, k, s); break;
    default: RB_REQUIRE(false, "rb_heads_linear: this combination of types is not built (x %d, w %d, y %d)", x_dtype, w_dtype, y_dtype);
  }
  RB_LAUNCH_CHECK();
  return 0;
}
