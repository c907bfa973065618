// What stands around attention when a head's keys and values differ in size or only a part of a head is rotated, a
// gate per head on attention's output, and the mean of two mixers' outputs after a norm of each.  float32 arithmetic.
#include <math.h>

#include "api.h"
#include "common.h"

// ---------------------------------------------------------------- rotation of a part of a head, heads padded for the cache
// A row of qkv holds Hq query heads and Hk key heads of `dim` numbers and Hk value heads of `vdim`.  Of every query and
// key head the first `rot` numbers are rotated, i paired with i + rot / 2, by the angles of the token's position
// (cos, sin [positions, rot / 2]); the rest pass.  Queries go to q_out [T, Hq, pad], keys and values to the token's
// place in pages [*, Hk, 64, pad]; what lies beyond a head's own size is zero, so that a kernel made for one head size
// `pad` computes the same scores and the same sums.
template <typename TC>
__global__ void rope_store_kernel(const float* __restrict__ qkv, size_t row_width, const float* __restrict__ cos_t,
                                  const float* __restrict__ sin_t, int rot, TC* __restrict__ q_out, TC* __restrict__ k_pages,
                                  TC* __restrict__ v_pages, const int32_t* __restrict__ tok_pos,
                                  const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ block_table, int bt_stride,
                                  int n_heads, int n_kv, int dim, int vdim, int pad) {
  const int t = blockIdx.x;
  const int pos = tok_pos[t];
  const int half = rot / 2;
  const float* src = qkv + (size_t)t * row_width;
  const float* cr = cos_t + (size_t)pos * half;
  const float* sr = sin_t + (size_t)pos * half;
  size_t page_base = 0;
  if (k_pages) {
    const int page = block_table[(size_t)tok_seq[t] * bt_stride + pos / RB_PAGE];
    page_base = ((size_t)page * n_kv) * RB_PAGE * pad + (size_t)(pos % RB_PAGE) * pad;
  }
  const int n_rot_heads = n_heads + (k_pages ? n_kv : 0);
  for (int idx = threadIdx.x; idx < n_rot_heads * pad; idx += blockDim.x) {
    const int h = idx / pad, d = idx - h * pad;
    const float* hp = src + (size_t)h * dim;
    float y = 0.f;
    if (d < half) {
      float y1;
      rotate_pair(hp[d], hp[d + half], cr[d], sr[d], y, y1);
    } else if (d < rot) {
      float y0;
      rotate_pair(hp[d - half], hp[d], cr[d - half], sr[d - half], y0, y);
    } else if (d < dim) {
      y = hp[d];
    }
    TC* dst = h < n_heads ? q_out + ((size_t)t * n_heads + h) * pad
                          : k_pages + page_base + (size_t)(h - n_heads) * RB_PAGE * pad;
    Num<TC>::store(dst + d, y);
  }
  if (v_pages) {
    const float* vsrc = src + (size_t)(n_heads + n_kv) * dim;
    for (int idx = threadIdx.x; idx < n_kv * pad; idx += blockDim.x) {
      const int h = idx / pad, d = idx - h * pad;
      Num<TC>::store(v_pages + page_base + (size_t)h * RB_PAGE * pad + d, d < vdim ? vsrc[(size_t)h * vdim + d] : 0.f);
    }
  }
}

extern "C" int rb_rope_store(const float* qkv, long long row_width, const float* cos, const float* sin, int rot, void* q_out,
                             void* k_pages, void* v_pages, int cache_dtype, const int32_t* tok_pos, const int32_t* tok_seq,
                             const int32_t* block_table, int bt_stride, int n_tokens, int n_heads, int n_kv_heads, int dim,
                             int vdim, int pad, void* stream) {
  RB_RECORDED(rb_rope_store(qkv, row_width, cos, sin, rot, q_out, k_pages, v_pages, cache_dtype, tok_pos, tok_seq, block_table,
                            bt_stride, n_tokens, n_heads, n_kv_heads, dim, vdim, pad, stream));
  RB_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv_heads >= 0 && dim > 0 && vdim > 0 && pad >= dim && pad >= vdim,
             "rb_rope_store: bad sizes T=%d Hq=%d Hk=%d dim=%d vdim=%d pad=%d", n_tokens, n_heads, n_kv_heads, dim, vdim, pad);
  RB_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= dim, "rb_rope_store: %d rotated numbers in a head of %d", rot, dim);
  RB_REQUIRE(rot == 0 || (cos != nullptr && sin != nullptr), "rb_rope_store: a rotation needs its tables");
  RB_REQUIRE((k_pages == nullptr) == (v_pages == nullptr), "rb_rope_store: k and v pages go together");
  const long long need = (long long)n_heads * dim + (k_pages ? (long long)n_kv_heads * (dim + vdim) : 0);
  RB_REQUIRE(row_width >= need, "rb_rope_store: rows of %lld numbers, %lld needed", row_width, need);
  if (n_tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (cache_dtype == RB_F32)
    rope_store_kernel<float><<<n_tokens, 256, 0, s>>>(qkv, (size_t)row_width, cos, sin, rot, (float*)q_out, (float*)k_pages,
                                                      (float*)v_pages, tok_pos, tok_seq, block_table, bt_stride, n_heads,
                                                      n_kv_heads, dim, vdim, pad);
  else if (cache_dtype == RB_BF16)
    rope_store_kernel<bf16_t><<<n_tokens, 256, 0, s>>>(qkv, (size_t)row_width, cos, sin, rot, (bf16_t*)q_out, (bf16_t*)k_pages,
                                                       (bf16_t*)v_pages, tok_pos, tok_seq, block_table, bt_stride, n_heads,
                                                       n_kv_heads, dim, vdim, pad);
  else
    RB_REQUIRE(false, "rb_rope_store: unknown dtype %d", cache_dtype);
  RB_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- a gate per head
// x[t, h, :] *= sigmoid(gate[t * gate_stride + h]), in place; x [T, H, D] of dtype.
template <typename TC>
__global__ void head_gate_kernel(TC* __restrict__ x, const float* __restrict__ gate, size_t gate_stride, int n_heads, int d,
                                 size_t n) {
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (size_t)gridDim.x * blockDim.x) {
    const size_t th = e / d;
    const size_t t = th / n_heads;
    const int h = (int)(th - t * n_heads);
    const float g = 1.0f / (1.0f + expf(-gate[t * gate_stride + h]));
    Num<TC>::store(x + e, Num<TC>::load(x + e) * g);
  }
}

extern "C" int rb_head_gate(void* x, int dtype, const float* gate, long long gate_stride, int n_tokens, int n_heads, int head_dim,
                            void* stream) {
  RB_RECORDED(rb_head_gate(x, dtype, gate, gate_stride, n_tokens, n_heads, head_dim, stream));
  RB_REQUIRE(n_tokens >= 0 && n_heads > 0 && head_dim > 0 && gate_stride >= n_heads, "rb_head_gate: bad sizes");
  if (n_tokens == 0) return 0;
  const size_t n = (size_t)n_tokens * n_heads * head_dim;
  const size_t blocks = (n + 255) / 256;
  const int grid = (int)(blocks < 65535 ? blocks : 65535);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == RB_F32)
    head_gate_kernel<float><<<grid, 256, 0, s>>>((float*)x, gate, (size_t)gate_stride, n_heads, head_dim, n);
  else if (dtype == RB_BF16)
    head_gate_kernel<bf16_t><<<grid, 256, 0, s>>>((bf16_t*)x, gate, (size_t)gate_stride, n_heads, head_dim, n);
  else
    RB_REQUIRE(false, "rb_head_gate: unknown dtype %d", dtype);
  RB_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- the mean of two normed outputs
// out[t, :] = (a / sqrt(mean a^2 + eps) * wa + b / sqrt(mean b^2 + eps) * wb) / 2; one workgroup a row.
__global__ void pair_norm_mean_kernel(const float* __restrict__ a, const float* __restrict__ wa, const float* __restrict__ b,
                                      const float* __restrict__ wb, float eps, float* __restrict__ out, int width) {
  __shared__ float scratch[16];
  const size_t r = blockIdx.x;
  const float* ar = a + r * width;
  const float* br = b + r * width;
  float sa = 0.f, sb = 0.f;
  for (int j = threadIdx.x; j < width; j += blockDim.x) {
    sa = fmaf(ar[j], ar[j], sa);
    sb = fmaf(br[j], br[j], sb);
  }
  const float fa = 1.0f / sqrtf(block_sum(sa, scratch) / (float)width + eps);
  const float fb = 1.0f / sqrtf(block_sum(sb, scratch) / (float)width + eps);
  for (int j = threadIdx.x; j < width; j += blockDim.x)
    out[r * width + j] = 0.5f * (ar[j] * fa * wa[j] + br[j] * fb * wb[j]);
}

extern "C" int rb_pair_norm_mean(const float* a, const float* wa, const float* b, const float* wb, float eps, float* out,
                                 int n_tokens, int width, void* stream) {
  RB_RECORDED(rb_pair_norm_mean(a, wa, b, wb, eps, out, n_tokens, width, stream));
  RB_REQUIRE(n_tokens >= 0 && width > 0, "rb_pair_norm_mean: bad sizes %d x %d", n_tokens, width);
  if (n_tokens == 0) return 0;
  const int threads = width >= 1024 ? 1024 : (width >= 256 ? 256 : 64);
  pair_norm_mean_kernel<<<n_tokens, threads, 0, (hipStream_t)stream>>>(a, wa, b, wb, eps, out, width);
  RB_LAUNCH_CHECK();
  return 0;
}
