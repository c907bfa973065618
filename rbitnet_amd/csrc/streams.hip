// A residual stream kept as several copies (hyper-connections), layer norm with weight and bias, and two small
// element-wise functions: the xIELU activation and the tanh cap of logits.  float32 arithmetic throughout.
//
// The streams are x [S, T, E], stream_stride floats from one copy to the next.  A sublayer reads the mixture
// u = sum_s coef[s] x[s], and afterwards every copy is rebuilt from all the old ones:
//   x'[j] = sum_s mix[s, j] x[s] + out[j] * (scale * y)
// One stream with coef = mix = out = 1 is the plain residual sum.
#include <math.h>

#include "api.h"
#include "common.h"

#define ST_MAX_STREAMS 16

// out[r] = (u - mean(u)) / sqrt(mean((u - mean)^2) + eps) * weight + bias, u = sum_s coef[s] x[s][src] (+ delta[src]),
// src = rows ? rows[r] : r.  With one stream, a delta and no rows the sum is written back to x (the residual sum of
// a plain pre-norm layer).  coef null: every coefficient is 1.  bias null: none.  The row is held in LDS between
// the passes: mean first, then the squared deviations.
template <typename TO>
__global__ void streams_layernorm_kernel(float* __restrict__ x, int n_streams, size_t stream_stride,
                                         const float* __restrict__ coef, const float* __restrict__ delta,
                                         const float* __restrict__ weight, const float* __restrict__ bias, float eps,
                                         const int32_t* __restrict__ rows, int width, TO* __restrict__ out) {
  extern __shared__ float u[];
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : (size_t)r;
  const bool write_back = delta != nullptr && rows == nullptr && n_streams == 1;
  float sum = 0.f;
  for (int j = threadIdx.x; j < width; j += blockDim.x) {
    float v = 0.f;
    for (int s = 0; s < n_streams; ++s) {
      const float xv = x[(size_t)s * stream_stride + src * width + j];
      v = coef ? fmaf(coef[s], xv, v) : v + xv;
    }
    if (delta) v += delta[src * width + j];
    if (write_back) x[src * width + j] = v;
    u[j] = v;
    sum += v;
  }
  const float mean = block_sum(sum, scratch) / (float)width;
  float ss = 0.f;
  for (int j = threadIdx.x; j < width; j += blockDim.x) {
    const float d = u[j] - mean;
    ss = fmaf(d, d, ss);
  }
  const float f = 1.0f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
  TO* orow = out + (size_t)r * width;
  for (int j = threadIdx.x; j < width; j += blockDim.x) {
    const float v = (u[j] - mean) * f * weight[j];
    Num<TO>::store(orow + j, bias ? v + bias[j] : v);
  }
}

extern "C" int rb_streams_layernorm(float* x, int n_streams, long long stream_stride, const float* coef,
                                    const float* delta, const float* weight, const float* bias, float eps,
                                    const int32_t* rows, int n_rows, int width, void* out, int out_dtype, void* stream) {
  RB_RECORDED(rb_streams_layernorm(x, n_streams, stream_stride, coef, delta, weight, bias, eps, rows, n_rows, width, out,
                                   out_dtype, stream));
  RB_REQUIRE(n_rows >= 0 && width > 0 && width <= 16384, "rb_streams_layernorm: bad sizes %d x %d (width at most 16384)", n_rows, width);
  RB_REQUIRE(n_streams >= 1 && n_streams <= ST_MAX_STREAMS && stream_stride >= 0, "rb_streams_layernorm: %d streams (1 to %d)",
             n_streams, ST_MAX_STREAMS);
  if (n_rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const size_t lds = (size_t)width * sizeof(float);
  if (out_dtype == RB_F32)
    streams_layernorm_kernel<float><<<n_rows, 256, lds, s>>>(x, n_streams, (size_t)stream_stride, coef, delta, weight, bias, eps,
                                                             rows, width, (float*)out);
  else if (out_dtype == RB_BF16)
    streams_layernorm_kernel<bf16_t><<<n_rows, 256, lds, s>>>(x, n_streams, (size_t)stream_stride, coef, delta, weight, bias, eps,
                                                              rows, width, (bf16_t*)out);
  else
    RB_REQUIRE(false, "rb_streams_layernorm: unknown dtype %d", out_dtype);
  RB_LAUNCH_CHECK();
  return 0;
}

// x'[j] = sum_s mix[s, j] x[s] + out_coef[j] * scale * y for all copies j at once; a thread owns an element of
// all copies, reads them, then writes them.
__global__ void streams_update_kernel(float* __restrict__ x, int n_streams, size_t stream_stride,
                                      const float* __restrict__ mix, const float* __restrict__ out_coef,
                                      const float* __restrict__ y, const float* __restrict__ scale, int width,
                                      size_t n_elems) {
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n_elems; e += (size_t)gridDim.x * blockDim.x) {
    float old[ST_MAX_STREAMS];
#pragma unroll
    for (int s = 0; s < ST_MAX_STREAMS; ++s)
      if (s < n_streams) old[s] = x[(size_t)s * stream_stride + e];
    float yv = y[e];
    if (scale) yv *= scale[e % width];
#pragma unroll
    for (int j = 0; j < ST_MAX_STREAMS; ++j) {
      if (j < n_streams) {
        float v = out_coef[j] * yv;
#pragma unroll
        for (int s = 0; s < ST_MAX_STREAMS; ++s)
          if (s < n_streams) v = fmaf(mix[s * n_streams + j], old[s], v);
        x[(size_t)j * stream_stride + e] = v;
      }
    }
  }
}

extern "C" int rb_streams_update(float* x, int n_streams, long long stream_stride, const float* mix, const float* out_coef,
                                 const float* y, const float* scale, int n_tokens, int width, void* stream) {
  RB_RECORDED(rb_streams_update(x, n_streams, stream_stride, mix, out_coef, y, scale, n_tokens, width, stream));
  RB_REQUIRE(n_tokens >= 0 && width > 0, "rb_streams_update: bad sizes %d x %d", n_tokens, width);
  RB_REQUIRE(n_streams >= 1 && n_streams <= ST_MAX_STREAMS && stream_stride >= 0, "rb_streams_update: %d streams (1 to %d)",
             n_streams, ST_MAX_STREAMS);
  if (n_tokens == 0) return 0;
  const size_t n = (size_t)n_tokens * width;
  const size_t blocks = (n + 255) / 256;
  streams_update_kernel<<<(int)(blocks < 65535 ? blocks : 65535), 256, 0, (hipStream_t)stream>>>(
      x, n_streams, (size_t)stream_stride, mix, out_coef, y, scale, width, n);
  RB_LAUNCH_CHECK();
  return 0;
}

// x[s][t, :] = table[ids[t], :] for every copy s.
template <typename T>
__global__ void embed_streams_kernel(const T* __restrict__ table, const int32_t* __restrict__ ids, float* __restrict__ x,
                                     int n_streams, size_t stream_stride, int width) {
  const int t = blockIdx.x;
  const T* row = table + (size_t)ids[t] * width;
  for (int j = threadIdx.x; j < width; j += blockDim.x) {
    const float v = Num<T>::load(row + j);
    for (int s = 0; s < n_streams; ++s) x[(size_t)s * stream_stride + (size_t)t * width + j] = v;
  }
}

extern "C" int rb_embed_streams(const void* table, int table_dtype, const int32_t* ids, float* x, int n_streams,
                                long long stream_stride, int n_tokens, int width, void* stream) {
  RB_RECORDED(rb_embed_streams(table, table_dtype, ids, x, n_streams, stream_stride, n_tokens, width, stream));
  RB_REQUIRE(n_tokens >= 0 && width > 0 && n_streams >= 1, "rb_embed_streams: bad sizes");
  if (n_tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (table_dtype == RB_F32)
    embed_streams_kernel<float><<<n_tokens, 256, 0, s>>>((const float*)table, ids, x, n_streams, (size_t)stream_stride, width);
  else if (table_dtype == RB_BF16)
    embed_streams_kernel<bf16_t><<<n_tokens, 256, 0, s>>>((const bf16_t*)table, ids, x, n_streams, (size_t)stream_stride, width);
  else
    RB_REQUIRE(false, "rb_embed_streams: unknown dtype %d", table_dtype);
  RB_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- xIELU
// z > 0: softplus(p) z^2 + z / 2;  z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2, with (p, q) = act[0..1].
template <typename TO>
__global__ void xielu_kernel(const float* __restrict__ z, const float* __restrict__ act, TO* __restrict__ out, size_t n) {
  const float p = act[0], q = act[1];
  const float ap = p > 20.0f ? p : log1pf(expf(p));
  const float an = 0.5f + (q > 20.0f ? q : log1pf(expf(q)));
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (size_t)gridDim.x * blockDim.x) {
    const float v = z[e];
    const float r = v > 0.f ? fmaf(ap * v, v, 0.5f * v) : fmaf(an, expm1f(v) - v, 0.5f * v);
    Num<TO>::store(out + e, r);
  }
}

extern "C" int rb_xielu(const float* z, const float* act, void* out, int out_dtype, long long n, void* stream) {
  RB_RECORDED(rb_xielu(z, act, out, out_dtype, n, stream));
  RB_REQUIRE(n >= 0, "rb_xielu: bad size");
  if (n == 0) return 0;
  const size_t blocks = ((size_t)n + 255) / 256;
  const int grid = (int)(blocks < 65535 ? blocks : 65535);
  hipStream_t s = (hipStream_t)stream;
  if (out_dtype == RB_F32)
    xielu_kernel<float><<<grid, 256, 0, s>>>(z, act, (float*)out, (size_t)n);
  else if (out_dtype == RB_BF16)
    xielu_kernel<bf16_t><<<grid, 256, 0, s>>>(z, act, (bf16_t*)out, (size_t)n);
  else
    RB_REQUIRE(false, "rb_xielu: unknown dtype %d", out_dtype);
  RB_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- cap of the logits
// x <- cap * tanh(x / cap), in place.
__global__ void tanh_cap_kernel(float* __restrict__ x, float cap, size_t n) {
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (size_t)gridDim.x * blockDim.x)
    x[e] = cap * tanhf(x[e] / cap);
}

extern "C" int rb_tanh_cap(float* x, float cap, long long n, void* stream) {
  RB_RECORDED(rb_tanh_cap(x, cap, n, stream));
  RB_REQUIRE(n >= 0 && cap > 0.f, "rb_tanh_cap: bad size or cap");
  if (n == 0) return 0;
  const size_t blocks = ((size_t)n + 255) / 256;
  tanh_cap_kernel<<<(int)(blocks < 65535 ? blocks : 65535), 256, 0, (hipStream_t)stream>>>(x, cap, (size_t)n);
  RB_LAUNCH_CHECK();
  return 0;
}
