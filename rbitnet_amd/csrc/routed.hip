// A feed-forward of many small experts of which every token uses a few.
//
//   route:  scores s = sigmoid(z) of a token's router logits z [n_experts]; the `top` largest are chosen (among equals
//           the lowest index); pair p = t * top + k holds the k-th choice of token t: sel[p] its expert, weight[p] its score.
//   sort:   the pairs in the order of their experts, every expert's run padded to a multiple of 16 rows, so that a
//           tile of 16 rows belongs to one expert: row_pair[row] (-1: padding), tile_expert[row / 16] (-1: past the end).
//   up:     for every row, x = weight * h[token] (the weight multiplies the expert's INPUT), g = min(Wg x, limit),
//           u = clamp(Wu x, -limit, limit), y[row] = g * sigmoid(alpha * g) * (u + 1)
//   down:   out[pair] = Wd y[row]; a token's result is the sum of its pairs, in the order of k.
//
// Nothing goes through the host: the grid is made for the most rows there can be (pairs rounded up to 16, plus 16 for
// every expert), and tiles past the end leave at once.  A row's sums do not depend on which rows share its tile, so
// the result of a token is the same bits whatever else the step holds.
// bfloat16 with sizes that are multiples of 32 runs on the matrix cores (the experts' rows as the row operand, 16
// rows of the step as the columns, gate and up of the same 16 channels in one wave so that a lane holds both);
// float32, and other sizes, on the vector units with a wave per output.
#include <math.h>

#include "api.h"
#include "common.h"
#include "mfma.h"

#define RT_TILE 16
#define RT_MAX_EXPERTS 1024

// ---------------------------------------------------------------- route
__global__ void route_kernel(const float* __restrict__ z, size_t z_stride, int n_experts, int top, int32_t* __restrict__ sel,
                             float* __restrict__ weight, int n_tokens) {
  const int t = blockIdx.x * (blockDim.x / RB_WAVE) + threadIdx.x / RB_WAVE;
  if (t >= n_tokens) return;
  const int lane = threadIdx.x & (RB_WAVE - 1);
  constexpr int PER = RT_MAX_EXPERTS / RB_WAVE;
  float v[PER];
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int e = lane + RB_WAVE * j;
    v[j] = e < n_experts ? z[(size_t)t * z_stride + e] : -INFINITY;
    if (v[j] != v[j]) v[j] = -INFINITY;
  }
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = lane + RB_WAVE * j;
      if (e < n_experts && (v[j] > best || (v[j] == best && e < at))) {
        best = v[j];
        at = e;
      }
    }
#pragma unroll
    for (int o = RB_WAVE / 2; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, RB_WAVE);
      const int oa = __shfl_xor(at, o, RB_WAVE);
      if (ob > best || (ob == best && oa < at)) {
        best = ob;
        at = oa;
      }
    }
    if (at == 0x7fffffff) at = k < n_experts ? k : 0;        // every logit was NaN or -inf: any expert, never out of range
    if (lane == 0) {
      sel[(size_t)t * top + k] = at;
      weight[(size_t)t * top + k] = 1.0f / (1.0f + expf(-best));
    }
#pragma unroll
    for (int j = 0; j < PER; ++j)
      if (lane + RB_WAVE * j == at) v[j] = -INFINITY;
  }
}

// ---------------------------------------------------------------- sort (one workgroup)
__global__ __launch_bounds__(1024) void route_sort_kernel(const int32_t* __restrict__ sel, int n_pairs, int n_experts,
                                                          int32_t* __restrict__ row_pair, int32_t* __restrict__ tile_expert,
                                                          int max_rows) {
  __shared__ int counts[RT_MAX_EXPERTS], offs[RT_MAX_EXPERTS], cursor[RT_MAX_EXPERTS];
  for (int e = threadIdx.x; e < n_experts; e += blockDim.x) counts[e] = cursor[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) atomicAdd(&counts[sel[p]], 1);
  for (int r = threadIdx.x; r < max_rows; r += blockDim.x) row_pair[r] = -1;
  for (int i = threadIdx.x; i < max_rows / RT_TILE; i += blockDim.x) tile_expert[i] = -1;
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0;
    for (int e = 0; e < n_experts; ++e) {
      offs[e] = at;
      at += (counts[e] + RT_TILE - 1) / RT_TILE * RT_TILE;
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < n_experts; e += blockDim.x)
    for (int i = 0; i < (counts[e] + RT_TILE - 1) / RT_TILE; ++i) tile_expert[offs[e] / RT_TILE + i] = e;
  for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) {
    const int e = sel[p];
    row_pair[offs[e] + atomicAdd(&cursor[e], 1)] = p;
  }
}

extern "C" int rb_route_top(const float* z, long long z_stride, int n_experts, int top, int32_t* sel, float* weight,
                            int32_t* row_pair, int32_t* tile_expert, int max_rows, int n_tokens, void* stream) {
  RB_RECORDED(rb_route_top(z, z_stride, n_experts, top, sel, weight, row_pair, tile_expert, max_rows, n_tokens, stream));
  RB_REQUIRE(n_tokens >= 0 && n_experts > 0 && n_experts <= RT_MAX_EXPERTS && top > 0 && top <= n_experts && z_stride >= n_experts,
             "rb_route_top: bad sizes T=%d experts=%d (at most %d) top=%d", n_tokens, n_experts, RT_MAX_EXPERTS, top);
  const long long pairs = (long long)n_tokens * top;
  RB_REQUIRE(max_rows % RT_TILE == 0 && max_rows >= (pairs + RT_TILE - 1) / RT_TILE * RT_TILE + (long long)RT_TILE * n_experts,
             "rb_route_top: room for %d rows, %lld pairs of %d experts may need more", max_rows, pairs, n_experts);
  if (n_tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  route_kernel<<<(n_tokens + 3) / 4, 256, 0, s>>>(z, (size_t)z_stride, n_experts, top, sel, weight, n_tokens);
  route_sort_kernel<<<1, 1024, 0, s>>>(sel, (int)pairs, n_experts, row_pair, tile_expert, max_rows);
  RB_LAUNCH_CHECK();
  return 0;
}

__device__ __forceinline__ float gated_unit(float g, float u, float limit, float alpha) {
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.0f + expf(-alpha * g)) * (u + 1.0f);
}

// ---------------------------------------------------------------- vector units: a wave per output
template <typename T>
__global__ void routed_up_generic_kernel(const T* __restrict__ h, const float* __restrict__ weight, int top,
                                         const int32_t* __restrict__ row_pair, const int32_t* __restrict__ tile_expert,
                                         const T* __restrict__ w_gate, const T* __restrict__ w_up, T* __restrict__ y, int width,
                                         int ff, float limit, float alpha) {
  const int e = tile_expert[blockIdx.x];
  if (e < 0) return;
  const int lane = threadIdx.x & (RB_WAVE - 1), wave = threadIdx.x / RB_WAVE, n_waves = blockDim.x / RB_WAVE;
  for (int i = 0; i < RT_TILE; ++i) {
    const int row = blockIdx.x * RT_TILE + i;
    const int p = row_pair[row];
    if (p < 0) continue;
    const T* x = h + (size_t)(p / top) * width;
    const float wt = weight[p];
    for (int j = blockIdx.y * n_waves + wave; j < ff; j += gridDim.y * n_waves) {
      const T* gr = w_gate + ((size_t)e * ff + j) * width;
      const T* ur = w_up + ((size_t)e * ff + j) * width;
      float g = 0.f, u = 0.f;
      for (int k = lane; k < width; k += RB_WAVE) {
        const float xv = Num<T>::load(x + k) * wt;
        g = fmaf(Num<T>::load(gr + k), xv, g);
        u = fmaf(Num<T>::load(ur + k), xv, u);
      }
      g = wave_sum(g);
      u = wave_sum(u);
      if (lane == 0) Num<T>::store(y + (size_t)row * ff + j, gated_unit(g, u, limit, alpha));
    }
  }
}

template <typename T>
__global__ void routed_down_generic_kernel(const T* __restrict__ y, const int32_t* __restrict__ row_pair,
                                           const int32_t* __restrict__ tile_expert, const T* __restrict__ w_down,
                                           float* __restrict__ out, int width, int ff) {
  const int e = tile_expert[blockIdx.x];
  if (e < 0) return;
  const int lane = threadIdx.x & (RB_WAVE - 1), wave = threadIdx.x / RB_WAVE, n_waves = blockDim.x / RB_WAVE;
  for (int i = 0; i < RT_TILE; ++i) {
    const int row = blockIdx.x * RT_TILE + i;
    const int p = row_pair[row];
    if (p < 0) continue;
    const T* yr = y + (size_t)row * ff;
    for (int j = blockIdx.y * n_waves + wave; j < width; j += gridDim.y * n_waves) {
      const T* dr = w_down + ((size_t)e * width + j) * ff;
      float acc = 0.f;
      for (int k = lane; k < ff; k += RB_WAVE) acc = fmaf(Num<T>::load(dr + k), Num<T>::load(yr + k), acc);
      acc = wave_sum(acc);
      if (lane == 0) out[(size_t)p * width + j] = acc;
    }
  }
}

// ---------------------------------------------------------------- matrix cores (bfloat16, sizes that are multiples of 32)
// A workgroup of 4 waves takes a tile of 16 rows and 64 channels; a wave 16 channels: the gate rows and the up rows of
// these channels are its two row operands, the 16 rows of the step (scaled by their weights, rounded to bfloat16) the
// column operand of both, so that lane l holds gate and up of channels 4 (l / 16) + i of row l % 16.
__global__ __launch_bounds__(256) void routed_up_mfma_kernel(const bf16_t* __restrict__ h, const float* __restrict__ weight, int top,
                                                             const int32_t* __restrict__ row_pair,
                                                             const int32_t* __restrict__ tile_expert,
                                                             const bf16_t* __restrict__ w_gate, const bf16_t* __restrict__ w_up,
                                                             bf16_t* __restrict__ y, int width, int ff, float limit, float alpha) {
  const int e = tile_expert[blockIdx.x];
  if (e < 0) return;
  const int lane = threadIdx.x & (RB_WAVE - 1), wave = threadIdx.x / RB_WAVE;
  const int c0 = (blockIdx.y * 4 + wave) * 16;
  if (c0 >= ff) return;
  const int r = lane & 15, grp = lane >> 4;
  const int row = blockIdx.x * RT_TILE + r;
  const int p = row_pair[row];
  const float wt = p >= 0 ? weight[p] : 0.f;
  const bf16_t* x = h + (size_t)(p >= 0 ? p / top : 0) * width + 8 * grp;
  const bf16_t* gr = w_gate + ((size_t)e * ff + c0 + r) * width + 8 * grp;
  const bf16_t* ur = w_up + ((size_t)e * ff + c0 + r) * width + 8 * grp;
  f32x4_t ag = {0.f, 0.f, 0.f, 0.f}, au = {0.f, 0.f, 0.f, 0.f};
  for (int k = 0; k < width; k += 32) {
    Frag8 fg, fu, fx;
    fg.u = load16(gr + k);
    fu.u = load16(ur + k);
    const uint4 raw = p >= 0 ? load16(x + k) : zero16();
    fx.u = make_uint4(pack_bf16x2(bf16_bits_to_f32(raw.x & 0xffffu) * wt, bf16_bits_to_f32(raw.x >> 16) * wt),
                      pack_bf16x2(bf16_bits_to_f32(raw.y & 0xffffu) * wt, bf16_bits_to_f32(raw.y >> 16) * wt),
                      pack_bf16x2(bf16_bits_to_f32(raw.z & 0xffffu) * wt, bf16_bits_to_f32(raw.z >> 16) * wt),
                      pack_bf16x2(bf16_bits_to_f32(raw.w & 0xffffu) * wt, bf16_bits_to_f32(raw.w >> 16) * wt));
    ag = mfma16(fg, fx, ag);
    au = mfma16(fu, fx, au);
  }
  // lane l: row l % 16 of the tile, channels c0 + 4 (l / 16) + i
  if (p >= 0) {
    bf16_t* dst = y + (size_t)row * ff + c0 + 4 * grp;
    *reinterpret_cast<uint2*>(dst) = make_uint2(pack_bf16x2(gated_unit(ag[0], au[0], limit, alpha), gated_unit(ag[1], au[1], limit, alpha)),
                                                pack_bf16x2(gated_unit(ag[2], au[2], limit, alpha), gated_unit(ag[3], au[3], limit, alpha)));
  }
}

__global__ __launch_bounds__(256) void routed_down_mfma_kernel(const bf16_t* __restrict__ y, const int32_t* __restrict__ row_pair,
                                                               const int32_t* __restrict__ tile_expert,
                                                               const bf16_t* __restrict__ w_down, float* __restrict__ out, int width,
                                                               int ff) {
  const int e = tile_expert[blockIdx.x];
  if (e < 0) return;
  const int lane = threadIdx.x & (RB_WAVE - 1), wave = threadIdx.x / RB_WAVE;
  const int c0 = (blockIdx.y * 4 + wave) * 16;
  if (c0 >= width) return;
  const int r = lane & 15, grp = lane >> 4;
  const int row = blockIdx.x * RT_TILE + r;
  const int p = row_pair[row];
  const bf16_t* yr = y + (size_t)row * ff + 8 * grp;
  const bf16_t* dr = w_down + ((size_t)e * width + c0 + r) * ff + 8 * grp;
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
  for (int k = 0; k < ff; k += 32) {
    Frag8 fd, fy;
    fd.u = load16(dr + k);
    fy.u = p >= 0 ? load16(yr + k) : zero16();
    acc = mfma16(fd, fy, acc);
  }
  if (p >= 0) *reinterpret_cast<float4*>(out + (size_t)p * width + c0 + 4 * grp) = make_float4(acc[0], acc[1], acc[2], acc[3]);
}

// h [T, width], weight [T * top], w_gate and w_up [experts, ff, width], w_down [experts, width, ff], all of dtype;
// y [max_rows, ff] of dtype is scratch; out [T * top, width] float32: the pairs' results.
extern "C" int rb_routed_experts(const void* h, int dtype, const float* weight, int top, const int32_t* row_pair,
                                 const int32_t* tile_expert, int max_rows, const void* w_gate, const void* w_up, const void* w_down,
                                 void* y, float* out, int n_experts, int width, int ff, float limit, float alpha, void* stream) {
  RB_RECORDED(rb_routed_experts(h, dtype, weight, top, row_pair, tile_expert, max_rows, w_gate, w_up, w_down, y, out, n_experts, width,
                                ff, limit, alpha, stream));
  RB_REQUIRE(max_rows >= 0 && max_rows % RT_TILE == 0 && n_experts > 0 && width > 0 && ff > 0 && top > 0,
             "rb_routed_experts: bad sizes rows=%d experts=%d width=%d ff=%d", max_rows, n_experts, width, ff);
  RB_REQUIRE(dtype == RB_F32 || dtype == RB_BF16, "rb_routed_experts: unknown dtype %d", dtype);
  if (max_rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int tiles = max_rows / RT_TILE;
  auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  if (dtype == RB_BF16 && width % 32 == 0 && ff % 32 == 0 && aligned(h) && aligned(w_gate) && aligned(w_up) && aligned(w_down) &&
      aligned(y) && aligned(out)) {
    routed_up_mfma_kernel<<<dim3(tiles, (ff + 63) / 64), 256, 0, s>>>((const bf16_t*)h, weight, top, row_pair, tile_expert,
                                                                      (const bf16_t*)w_gate, (const bf16_t*)w_up, (bf16_t*)y, width,
                                                                      ff, limit, alpha);
    routed_down_mfma_kernel<<<dim3(tiles, (width + 63) / 64), 256, 0, s>>>((const bf16_t*)y, row_pair, tile_expert,
                                                                           (const bf16_t*)w_down, out, width, ff);
  } else if (dtype == RB_BF16) {
    routed_up_generic_kernel<bf16_t><<<dim3(tiles, (ff + 3) / 4 < 64 ? (ff + 3) / 4 : 64), 256, 0, s>>>(
        (const bf16_t*)h, weight, top, row_pair, tile_expert, (const bf16_t*)w_gate, (const bf16_t*)w_up, (bf16_t*)y, width, ff, limit,
        alpha);
    routed_down_generic_kernel<bf16_t><<<dim3(tiles, (width + 3) / 4 < 64 ? (width + 3) / 4 : 64), 256, 0, s>>>(
        (const bf16_t*)y, row_pair, tile_expert, (const bf16_t*)w_down, out, width, ff);
  } else {
    routed_up_generic_kernel<float><<<dim3(tiles, (ff + 3) / 4 < 64 ? (ff + 3) / 4 : 64), 256, 0, s>>>(
        (const float*)h, weight, top, row_pair, tile_expert, (const float*)w_gate, (const float*)w_up, (float*)y, width, ff, limit, alpha);
    routed_down_generic_kernel<float><<<dim3(tiles, (width + 3) / 4 < 64 ? (width + 3) / 4 : 64), 256, 0, s>>>(
        (const float*)y, row_pair, tile_expert, (const float*)w_down, out, width, ff);
  }
  RB_LAUNCH_CHECK();
  return 0;
}

// out[t, :] = sum_k pairs[t * top + k, :], in the order of k.
__global__ void pairs_sum_kernel(const float* __restrict__ pairs, int top, float* __restrict__ out, int width, size_t n) {
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (size_t)gridDim.x * blockDim.x) {
    const size_t t = e / width, j = e - t * width;
    float v = pairs[(t * top) * width + j];
    for (int k = 1; k < top; ++k) v += pairs[(t * top + k) * width + j];
    out[e] = v;
  }
}

extern "C" int rb_pairs_sum(const float* pairs, int top, float* out, int n_tokens, int width, void* stream) {
  RB_RECORDED(rb_pairs_sum(pairs, top, out, n_tokens, width, stream));
  RB_REQUIRE(n_tokens >= 0 && width > 0 && top > 0, "rb_pairs_sum: bad sizes");
  if (n_tokens == 0) return 0;
  const size_t n = (size_t)n_tokens * width;
  const size_t blocks = (n + 255) / 256;
  pairs_sum_kernel<<<(int)(blocks < 65535 ? blocks : 65535), 256, 0, (hipStream_t)stream>>>(pairs, top, out, width, n);
  RB_LAUNCH_CHECK();
  return 0;
}
