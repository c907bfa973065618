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
                                         const int32_t* __restrict__ rows, int width, TO* __restrict__ out,
                                         const float* __restrict__ mix, const float* __restrict__ out_coef,
                                         const float* __restrict__ y, const float* __restrict__ scale,
                                         const float* __restrict__ delta2, float dscale) {
  extern __shared__ float u[];
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : (size_t)r;
  const bool write_back = delta != nullptr && rows == nullptr && n_streams == 1;
  float sum = 0.f;
  for (int j = threadIdx.x; j < width; j += blockDim.x) {
    float v = 0.f;
    if (mix) {
      // the update that was still to be done: every copy from all the old ones, then the mixture of the new ones
      float old[ST_MAX_STREAMS];
#pragma unroll
      for (int s = 0; s < ST_MAX_STREAMS; ++s)
        if (s < n_streams) old[s] = x[(size_t)s * stream_stride + src * width + j];
      float yv = y[src * width + j];
      if (scale) yv *= scale[j];
#pragma unroll
      for (int k = 0; k < ST_MAX_STREAMS; ++k) {
        if (k < n_streams) {
          float nv = out_coef[k] * yv;
#pragma unroll
          for (int s = 0; s < ST_MAX_STREAMS; ++s)
            if (s < n_streams) nv = fmaf(mix[s * n_streams + k], old[s], nv);
          x[(size_t)k * stream_stride + src * width + j] = nv;
          v = coef ? fmaf(coef[k], nv, v) : v + nv;
        }
      }
    } else {
      for (int s = 0; s < n_streams; ++s) {
        const float xv = x[(size_t)s * stream_stride + src * width + j];
        v = coef ? fmaf(coef[s], xv, v) : v + xv;
      }
    }
    if (delta) v = fmaf(dscale, delta2 ? delta[src * width + j] + delta2[src * width + j] : delta[src * width + j], v);
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

// The same for widths that are multiples of 4, four values a thread with 16-byte loads and up to 1024 threads a row,
// so that a row's loads are all in flight together (a step of few tokens has few rows, and their time is the
// chain of trips to memory).
__device__ __forceinline__ float4 ld4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 fma4(float a, const float4& b, const float4& c) {
  return make_float4(fmaf(a, b.x, c.x), fmaf(a, b.y, c.y), fmaf(a, b.z, c.z), fmaf(a, b.w, c.w));
}
__device__ __forceinline__ void st4(float* p, float a, float b, float c, float d) { *reinterpret_cast<float4*>(p) = make_float4(a, b, c, d); }
__device__ __forceinline__ void st4(bf16_t* p, float a, float b, float c, float d) {
  *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16x2(a, b), pack_bf16x2(c, d));
}

template <typename TO>
__global__ __launch_bounds__(1024) void streams_layernorm_vec_kernel(
    float* __restrict__ x, int n_streams, size_t stream_stride, const float* __restrict__ coef, const float* __restrict__ delta,
    const float* __restrict__ weight, const float* __restrict__ bias, float eps, const int32_t* __restrict__ rows, int width,
    TO* __restrict__ out, const float* __restrict__ mix, const float* __restrict__ out_coef, const float* __restrict__ y,
    const float* __restrict__ scale, const float* __restrict__ delta2, float dscale) {
  extern __shared__ float u[];
  __shared__ float scratch[16];
  __shared__ float c_mix[ST_MAX_STREAMS * ST_MAX_STREAMS], c_out[ST_MAX_STREAMS], c_in[ST_MAX_STREAMS];
  const int r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : (size_t)r;
  const bool write_back = delta != nullptr && rows == nullptr && n_streams == 1;
  if ((int)threadIdx.x < n_streams) {
    c_in[threadIdx.x] = coef ? coef[threadIdx.x] : 1.0f;
    if (mix) c_out[threadIdx.x] = out_coef[threadIdx.x];
  }
  if (mix && (int)threadIdx.x < n_streams * n_streams) c_mix[threadIdx.x] = mix[threadIdx.x];
  __syncthreads();
  float sum = 0.f;
  for (int j = 4 * threadIdx.x; j < width; j += 4 * blockDim.x) {
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (mix) {
      float4 old[ST_MAX_STREAMS];
#pragma unroll
      for (int s = 0; s < ST_MAX_STREAMS; ++s)
        if (s < n_streams) old[s] = ld4(x + (size_t)s * stream_stride + src * width + j);
      float4 yv = ld4(y + src * width + j);
      if (scale) {
        const float4 sc = ld4(scale + j);
        yv = make_float4(yv.x * sc.x, yv.y * sc.y, yv.z * sc.z, yv.w * sc.w);
      }
#pragma unroll
      for (int k = 0; k < ST_MAX_STREAMS; ++k) {
        if (k < n_streams) {
          const float oc = c_out[k];
          float4 nv = make_float4(oc * yv.x, oc * yv.y, oc * yv.z, oc * yv.w);
#pragma unroll
          for (int s = 0; s < ST_MAX_STREAMS; ++s)
            if (s < n_streams) nv = fma4(c_mix[s * n_streams + k], old[s], nv);
          *reinterpret_cast<float4*>(x + (size_t)k * stream_stride + src * width + j) = nv;
          v = fma4(c_in[k], nv, v);
        }
      }
    } else {
#pragma unroll
      for (int s = 0; s < ST_MAX_STREAMS; ++s)
        if (s < n_streams) v = fma4(c_in[s], ld4(x + (size_t)s * stream_stride + src * width + j), v);
    }
    if (delta) {
      float4 d = ld4(delta + src * width + j);
      if (delta2) {
        const float4 e = ld4(delta2 + src * width + j);
        d = make_float4(d.x + e.x, d.y + e.y, d.z + e.z, d.w + e.w);
      }
      v = fma4(dscale, d, v);
    }
    if (write_back) *reinterpret_cast<float4*>(x + src * width + j) = v;
    *reinterpret_cast<float4*>(u + j) = v;
    sum += (v.x + v.y) + (v.z + v.w);
  }
  // weight and bias of this thread's first values are asked for now, so that they arrive under the two reductions
  const int j0 = 4 * threadIdx.x;
  float4 w0 = make_float4(0.f, 0.f, 0.f, 0.f), b0 = w0;
  if (j0 < width) {
    w0 = ld4(weight + j0);
    if (bias) b0 = ld4(bias + j0);
  }
  __builtin_amdgcn_sched_barrier(0);
  const float mean = block_sum(sum, scratch) / (float)width;
  float ss = 0.f;
  for (int j = 4 * threadIdx.x; j < width; j += 4 * blockDim.x) {
    const float4 v = *reinterpret_cast<const float4*>(u + j);
    const float a = v.x - mean, b = v.y - mean, c = v.z - mean, d = v.w - mean;
    ss += (a * a + b * b) + (c * c + d * d);
  }
  const float f = 1.0f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
  TO* orow = out + (size_t)r * width;
  for (int j = 4 * threadIdx.x; j < width; j += 4 * blockDim.x) {
    const float4 v = *reinterpret_cast<const float4*>(u + j);
    const float4 wv = j == j0 ? w0 : ld4(weight + j);
    float4 o = make_float4((v.x - mean) * f * wv.x, (v.y - mean) * f * wv.y, (v.z - mean) * f * wv.z, (v.w - mean) * f * wv.w);
    if (bias) {
      const float4 bv = j == j0 ? b0 : ld4(bias + j);
      o = make_float4(o.x + bv.x, o.y + bv.y, o.z + bv.z, o.w + bv.w);
    }
    st4(orow + j, o.x, o.y, o.z, o.w);
  }
}

extern "C" int rb_streams_layernorm(float* x, int n_streams, long long stream_stride, const float* coef,
                                    const float* delta, const float* weight, const float* bias, float eps,
                                    const int32_t* rows, int n_rows, int width, void* out, int out_dtype, void* stream) {
  return rb_streams_update_layernorm(x, n_streams, stream_stride, nullptr, nullptr, nullptr, nullptr, coef, delta, weight, bias,
                                     eps, rows, n_rows, width, out, out_dtype, stream);
}

// The same after an update of the copies that was still to be done (rb_streams_update's mix, out_coef, y, scale; mix
// null: none), in one pass over the rows: the copies are rewritten and the norm reads the new ones.  With an update
// every row is taken (rows must be null).
static int layernorm_launch(float* x, int n_streams, long long stream_stride, const float* mix, const float* out_coef, const float* y,
                            const float* scale, const float* coef, const float* delta, const float* delta2, float dscale,
                            const float* weight, const float* bias, float eps, const int32_t* rows, int n_rows, int width, void* out,
                            int out_dtype, void* stream);

extern "C" int rb_streams_update_layernorm(float* x, int n_streams, long long stream_stride, const float* mix,
                                           const float* out_coef, const float* y, const float* scale, const float* coef,
                                           const float* delta, const float* weight, const float* bias, float eps,
                                           const int32_t* rows, int n_rows, int width, void* out, int out_dtype,
                                           void* stream) {
  RB_RECORDED(rb_streams_update_layernorm(x, n_streams, stream_stride, mix, out_coef, y, scale, coef, delta, weight, bias, eps,
                                          rows, n_rows, width, out, out_dtype, stream));
  return layernorm_launch(x, n_streams, stream_stride, mix, out_coef, y, scale, coef, delta, nullptr, 1.0f, weight, bias, eps, rows,
                          n_rows, width, out, out_dtype, stream);
}

// Layer norm of a plain stream x [T, E] with the residual sum that was still to be done, in one pass:
//   v = x[src] + dscale * (delta[src] + (delta2 ? delta2[src] : 0)),  src = rows ? rows[r] : r;  without rows x[src] = v as well;
//   out[r] = (v - mean) / sqrt(var + eps) * weight + bias.   delta null: the norm alone.
extern "C" int rb_layernorm_residual(float* x, const float* delta, const float* delta2, float dscale, const float* weight,
                                     const float* bias, float eps, const int32_t* rows, int n_rows, int width, void* out,
                                     int out_dtype, void* stream) {
  RB_RECORDED(rb_layernorm_residual(x, delta, delta2, dscale, weight, bias, eps, rows, n_rows, width, out, out_dtype, stream));
  RB_REQUIRE(delta != nullptr || delta2 == nullptr, "rb_layernorm_residual: a second term without a first");
  return layernorm_launch(x, 1, 0, nullptr, nullptr, nullptr, nullptr, nullptr, delta, delta2, dscale, weight, bias, eps, rows, n_rows,
                          width, out, out_dtype, stream);
}

static int layernorm_launch(float* x, int n_streams, long long stream_stride, const float* mix, const float* out_coef, const float* y,
                            const float* scale, const float* coef, const float* delta, const float* delta2, float dscale,
                            const float* weight, const float* bias, float eps, const int32_t* rows, int n_rows, int width, void* out,
                            int out_dtype, void* stream) {
  RB_REQUIRE(mix == nullptr || (rows == nullptr && out_coef != nullptr && y != nullptr),
             "rb_streams_update_layernorm: an update takes every row and needs out_coef and y");
  RB_REQUIRE(n_rows >= 0 && width > 0 && width <= 16384, "rb_streams_layernorm: bad sizes %d x %d (width at most 16384)", n_rows, width);
  RB_REQUIRE(n_streams >= 1 && n_streams <= ST_MAX_STREAMS && stream_stride >= 0, "rb_streams_layernorm: %d streams (1 to %d)",
             n_streams, ST_MAX_STREAMS);
  if (n_rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const size_t lds = (size_t)width * sizeof(float);
  auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  if (width % 4 == 0 && stream_stride % 4 == 0 && aligned(x) && aligned(delta) && aligned(delta2) && aligned(weight) && aligned(bias) && aligned(out) &&
      aligned(y) && aligned(scale) && (out_dtype == RB_F32 || out_dtype == RB_BF16)) {
    int threads = ((width / 4 + RB_WAVE - 1) / RB_WAVE) * RB_WAVE;
    if (threads > 1024) threads = 1024;
    if (out_dtype == RB_F32)
      streams_layernorm_vec_kernel<float><<<n_rows, threads, lds, s>>>(x, n_streams, (size_t)stream_stride, coef, delta, weight, bias,
                                                                       eps, rows, width, (float*)out, mix, out_coef, y, scale, delta2, dscale);
    else
      streams_layernorm_vec_kernel<bf16_t><<<n_rows, threads, lds, s>>>(x, n_streams, (size_t)stream_stride, coef, delta, weight,
                                                                        bias, eps, rows, width, (bf16_t*)out, mix, out_coef, y, scale, delta2, dscale);
    RB_LAUNCH_CHECK();
    return 0;
  }
  if (out_dtype == RB_F32)
    streams_layernorm_kernel<float><<<n_rows, 256, lds, s>>>(x, n_streams, (size_t)stream_stride, coef, delta, weight, bias, eps,
                                                             rows, width, (float*)out, mix, out_coef, y, scale, delta2, dscale);
  else if (out_dtype == RB_BF16)
    streams_layernorm_kernel<bf16_t><<<n_rows, 256, lds, s>>>(x, n_streams, (size_t)stream_stride, coef, delta, weight, bias, eps,
                                                              rows, width, (bf16_t*)out, mix, out_coef, y, scale, delta2, dscale);
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
__device__ __forceinline__ void xielu_store4(float* p, float a, float b, float c, float d) {
  *reinterpret_cast<float4*>(p) = make_float4(a, b, c, d);
}
__device__ __forceinline__ void xielu_store4(bf16_t* p, float a, float b, float c, float d) {
  *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16x2(a, b), pack_bf16x2(c, d));
}

// four values a thread with 16-byte loads (n4 quads), then the rest one by one
template <typename TO>
__global__ void xielu_kernel(const float* __restrict__ z, const float* __restrict__ act, TO* __restrict__ out, size_t n) {
  const XieluPair pair = xielu_pair(act);
  const float ap = pair.ap, an = pair.an;
  const size_t n4 = n / 4;
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n4; e += (size_t)gridDim.x * blockDim.x) {
    const float4 v = *reinterpret_cast<const float4*>(z + 4 * e);
    xielu_store4(out + 4 * e, xielu_value(v.x, ap, an), xielu_value(v.y, ap, an), xielu_value(v.z, ap, an),
                 xielu_value(v.w, ap, an));
  }
  for (size_t e = 4 * n4 + (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (size_t)gridDim.x * blockDim.x)
    Num<TO>::store(out + e, xielu_value(z[e], ap, an));
}

extern "C" int rb_xielu(const float* z, const float* act, void* out, int out_dtype, long long n, void* stream) {
  RB_RECORDED(rb_xielu(z, act, out, out_dtype, n, stream));
  RB_REQUIRE(n >= 0, "rb_xielu: bad size");
  if (n == 0) return 0;
  const size_t blocks = ((size_t)n / 4 + 255) / 256 + 1;
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
