// Small kernels around a latent attention and a mixture of experts.  All arithmetic is
// float32; T is the element type of activations (float or bf16).
//
//   * RMSNorm of the float32 stream with one or two weights at once (the two norms of a
//     block whose mixer and feed-forward read the same rows), x * rstd * w in float32 and
//     one rounding at the end;
//   * the step between the down projections of a latent attention and its cache: norms of
//     the query latent and of the key/value latent, and the key and value rows that the
//     paged attention kernels take;
//   * column ranges copied head by head;
//   * the router of a mixture of experts: sigmoid scores, the largest `top`, their weights;
//   * a counting sort of the (token, choice) pairs by expert, on the device;
//   * the weighted sum of the chosen experts' results, added into the stream.
#include "hal_common.h"
#include "hal_api.h"

// ---------------------------------------------------------------------------------
// out1[r] = T(x * rstd * w1), out2[r] = T(x * rstd * w2) with x = h[rows ? rows[r] : r]
// ---------------------------------------------------------------------------------
template <typename T>
__global__ void norm_pair_kernel(const float* __restrict__ h, const int* __restrict__ rows,
                                 const void* __restrict__ w1, const void* __restrict__ w2, int w_dtype,
                                 float eps, T* __restrict__ out1, T* __restrict__ out2, int d) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const float* hr = h + (size_t)(rows ? rows[r] : r) * d;
  float ss = 0.f;
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    const float x = hr[i];
    ss += x * x;
  }
  const float total = block_sum(ss, scratch);
  const float rstd = 1.0f / sqrtf(total / (float)d + eps);
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    const float x = hr[i] * rstd;
    out1[(size_t)r * d + i] = from_f32<T>(x * load_as_f32(w1, w_dtype, i));
    if (w2) out2[(size_t)r * d + i] = from_f32<T>(x * load_as_f32(w2, w_dtype, i));
  }
}

extern "C" int hal_norm_pair(const float* h, const int* rows, const void* w1, const void* w2,
                             int w_dtype, float eps, void* out1, void* out2, int dtype, int n_rows,
                             int d, hipStream_t stream) {
  HAL_REQUIRE(n_rows >= 0 && d > 0, "hal_norm_pair: bad sizes rows=%d d=%d", n_rows, d);
  HAL_REQUIRE(dtype == HAL_F32 || dtype == HAL_BF16, "hal_norm_pair: dtype %d", dtype);
  HAL_REQUIRE((w2 == nullptr) == (out2 == nullptr), "hal_norm_pair: a second weight and a second result come together");
  if (n_rows == 0) return 0;
  int threads = ((d + 3) / 4 + 63) / 64 * 64;
  if (threads > 1024) threads = 1024;
  if (dtype == HAL_F32)
    hipLaunchKernelGGL(norm_pair_kernel<float>, dim3(n_rows), dim3(threads), 0, stream, h, rows, w1, w2,
                       w_dtype, eps, (float*)out1, (float*)out2, d);
  else
    hipLaunchKernelGGL(norm_pair_kernel<bf16_t>, dim3(n_rows), dim3(threads), 0, stream, h, rows, w1,
                       w2, w_dtype, eps, (bf16_t*)out1, (bf16_t*)out2, d);
  HAL_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------
// a [T, lda] float32 holds, per token, the query latent (q_rank, from column q_col0; none
// if q_rank == 0), then at kv_col0 the key/value latent (kv_rank) and the shared rotated key
// part (rot, not normed).
//   cq[t]         = T(rmsnorm(query latent) * wq)
//   k row of t    = [rotated part (not yet rotated) | T(rmsnorm(latent) * wkv) | 0 ...]   (D)
//   v row of t    = [0 ...                          | the same                 | 0 ...]   (D)
// in the packed rows `qkv` at columns k_col0 and k_col0 + D.
// ---------------------------------------------------------------------------------
template <typename T>
__global__ void latent_prep_kernel(const float* __restrict__ a, int lda, int q_col0, int q_rank,
                                   int kv_col0, int kv_rank, int rot, int D, const void* wq,
                                   const void* wkv, int w_dtype, float eps, T* __restrict__ cq,
                                   T* __restrict__ qkv, int row_stride, int k_col0) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const float* ar = a + (size_t)t * lda;
  if (q_rank > 0) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < q_rank; i += blockDim.x) ss += ar[q_col0 + i] * ar[q_col0 + i];
    const float rstd = 1.0f / sqrtf(block_sum(ss, scratch) / (float)q_rank + eps);
    for (int i = threadIdx.x; i < q_rank; i += blockDim.x)
      cq[(size_t)t * q_rank + i] = from_f32<T>(ar[q_col0 + i] * rstd * load_as_f32(wq, w_dtype, i));
  }
  float ss = 0.f;
  for (int i = threadIdx.x; i < kv_rank; i += blockDim.x) ss += ar[kv_col0 + i] * ar[kv_col0 + i];
  const float rstd = 1.0f / sqrtf(block_sum(ss, scratch) / (float)kv_rank + eps);
  T* k = qkv + (size_t)t * row_stride + k_col0;
  T* v = k + D;
  for (int i = threadIdx.x; i < D; i += blockDim.x) {
    float kx = 0.f, vx = 0.f;
    if (i < rot) {
      kx = ar[kv_col0 + kv_rank + i];
    } else if (i < rot + kv_rank) {
      const int c = i - rot;
      // rounded once, so that keys and values hold the same number
      kx = vx = to_f32(from_f32<T>(ar[kv_col0 + c] * rstd * load_as_f32(wkv, w_dtype, c)));
    }
    k[i] = from_f32<T>(kx);
    v[i] = from_f32<T>(vx);
  }
}

extern "C" int hal_latent_prep(const float* a, int lda, int q_col0, int q_rank, int kv_col0,
                               int kv_rank, int rot, int D, const void* wq, const void* wkv,
                               int w_dtype, float eps, void* cq, void* qkv, int row_stride,
                               int k_col0, int dtype, int n_tokens, hipStream_t stream) {
  HAL_REQUIRE(n_tokens >= 0 && kv_rank > 0 && rot >= 0 && q_rank >= 0 && D >= rot + kv_rank,
              "hal_latent_prep: bad sizes T=%d q_rank=%d kv_rank=%d rot=%d D=%d", n_tokens, q_rank, kv_rank,
              rot, D);
  HAL_REQUIRE(q_col0 >= 0 && kv_col0 >= 0 && q_col0 + q_rank <= lda && kv_col0 + kv_rank + rot <= lda &&
                  k_col0 >= 0 && k_col0 + 2 * D <= row_stride,
              "hal_latent_prep: columns outside the rows");
  HAL_REQUIRE(dtype == HAL_F32 || dtype == HAL_BF16, "hal_latent_prep: dtype %d", dtype);
  if (n_tokens == 0) return 0;
  if (dtype == HAL_F32)
    hipLaunchKernelGGL(latent_prep_kernel<float>, dim3(n_tokens), dim3(256), 0, stream, a, lda, q_col0,
                       q_rank, kv_col0, kv_rank, rot, D, wq, wkv, w_dtype, eps, (float*)cq, (float*)qkv,
                       row_stride, k_col0);
  else
    hipLaunchKernelGGL(latent_prep_kernel<bf16_t>, dim3(n_tokens), dim3(256), 0, stream, a, lda, q_col0,
                       q_rank, kv_col0, kv_rank, rot, D, wq, wkv, w_dtype, eps, (bf16_t*)cq,
                       (bf16_t*)qkv, row_stride, k_col0);
  HAL_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------
// y[t, h * ys + y0 + j] = x[t, h * xs + x0 + j] for j < n, and zero for the `n_zero` columns
// from h * ys + z0 on
// ---------------------------------------------------------------------------------
template <typename T>
__global__ void head_cols_kernel(const T* __restrict__ x, int ldx, int xs, int x0, T* __restrict__ y,
                                 int ldy, int ys, int y0, int n, int z0, int n_zero, int H) {
  const int t = blockIdx.x;
  const int per = n + n_zero;
  for (int e = threadIdx.x; e < H * per; e += blockDim.x) {
    const int h = e / per, j = e % per;
    if (j < n) y[(size_t)t * ldy + h * ys + y0 + j] = x[(size_t)t * ldx + h * xs + x0 + j];
    else y[(size_t)t * ldy + h * ys + z0 + (j - n)] = from_f32<T>(0.f);
  }
}

extern "C" int hal_head_cols(const void* x, int ldx, int xs, int x0, void* y, int ldy, int ys, int y0,
                             int n, int z0, int n_zero, int H, int dtype, int n_tokens,
                             hipStream_t stream) {
  HAL_REQUIRE(n_tokens >= 0 && H > 0 && n >= 0 && n_zero >= 0, "hal_head_cols: bad sizes");
  HAL_REQUIRE(x0 >= 0 && x0 + n <= xs && H * xs <= ldx && y0 >= 0 && y0 + n <= ys && z0 >= 0 &&
                  z0 + n_zero <= ys && H * ys <= ldy,
              "hal_head_cols: columns outside the rows");
  HAL_REQUIRE(dtype == HAL_F32 || dtype == HAL_BF16, "hal_head_cols: dtype %d", dtype);
  if (n_tokens == 0 || n + n_zero == 0) return 0;
  if (dtype == HAL_F32)
    hipLaunchKernelGGL(head_cols_kernel<float>, dim3(n_tokens), dim3(256), 0, stream, (const float*)x, ldx,
                       xs, x0, (float*)y, ldy, ys, y0, n, z0, n_zero, H);
  else
    hipLaunchKernelGGL(head_cols_kernel<bf16_t>, dim3(n_tokens), dim3(256), 0, stream, (const bf16_t*)x,
                       ldx, xs, x0, (bf16_t*)y, ldy, ys, y0, n, z0, n_zero, H);
  HAL_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------
// x[i] *= s
// ---------------------------------------------------------------------------------
__global__ void scale_f32_kernel(float* __restrict__ x, size_t n, float s) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] *= s;
}

extern "C" int hal_scale_f32(float* x, long long n, float s, hipStream_t stream) {
  HAL_REQUIRE(n >= 0, "hal_scale_f32: n=%lld", n);
  if (n == 0) return 0;
  hipLaunchKernelGGL(scale_f32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, x, (size_t)n, s);
  HAL_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------
#define MOE_MAX_EXPERTS 1024
// Router: z [T, E] float32 logits.  score = sigmoid(z) (or, softmax == 1, the softmax over
// the experts); the `top` largest scores (the lower index wins a tie); weights = the chosen
// scores, divided by their sum + norm_eps if `normalize`.
// ---------------------------------------------------------------------------------
// One wave a token: lane l holds the scores of the experts l, l + 64, ...; each of the `top`
// rounds finds the largest score that is left (the lower index on a tie) across the wave.
#define MOE_ROUTE_PER_LANE (MOE_MAX_EXPERTS / HAL_WAVE)
__device__ __forceinline__ void moe_route_token(const float* __restrict__ z, int ldz, int E, int top, int softmax,
                                                int normalize, float norm_eps, int* __restrict__ idx,
                                                float* __restrict__ wgt, int t, int lane) {
  const float* zr = z + (size_t)t * ldz;
  float s[MOE_ROUTE_PER_LANE];
  float zmax = -INFINITY;
#pragma unroll
  for (int u = 0; u < MOE_ROUTE_PER_LANE; ++u) {
    const int e = lane + u * HAL_WAVE;
    s[u] = e < E ? zr[e] : -INFINITY;
    zmax = fmaxf(zmax, s[u]);
  }
  if (softmax) {
    zmax = wave_max(zmax);
    float part = 0.f;
#pragma unroll
    for (int u = 0; u < MOE_ROUTE_PER_LANE; ++u) {
      s[u] = lane + u * HAL_WAVE < E ? expf(s[u] - zmax) : -INFINITY;
      part += lane + u * HAL_WAVE < E ? s[u] : 0.f;
    }
    const float denom = wave_sum(part);
#pragma unroll
    for (int u = 0; u < MOE_ROUTE_PER_LANE; ++u) s[u] = s[u] / denom;
  } else {
#pragma unroll
    for (int u = 0; u < MOE_ROUTE_PER_LANE; ++u)
      if (lane + u * HAL_WAVE < E) s[u] = 1.0f / (1.0f + expf(-s[u]));
  }
  float sum = 0.f;
  float kept[MOE_ROUTE_PER_LANE];  // lane j % 64 keeps the j-th choice's score in kept[j / 64]
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int best_e = MOE_MAX_EXPERTS;
#pragma unroll
    for (int u = 0; u < MOE_ROUTE_PER_LANE; ++u)
      if (s[u] > best) best = s[u], best_e = lane + u * HAL_WAVE;  // rising index: the lower one stays on a tie
#pragma unroll
    for (int off = HAL_WAVE / 2; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, HAL_WAVE);
      const int oe = __shfl_xor(best_e, off, HAL_WAVE);
      if (ob > best || (ob == best && oe < best_e)) best = ob, best_e = oe;
    }
#pragma unroll
    for (int u = 0; u < MOE_ROUTE_PER_LANE; ++u)
      if (lane + u * HAL_WAVE == best_e) s[u] = -INFINITY;  // taken
    sum += best;
    if (lane == 0) idx[(size_t)t * top + j] = best_e;
#pragma unroll
    for (int u = 0; u < MOE_ROUTE_PER_LANE; ++u)
      if (u == j / HAL_WAVE && lane == j % HAL_WAVE) kept[u] = best;
  }
#pragma unroll
  for (int u = 0; u < MOE_ROUTE_PER_LANE; ++u) {
    const int j = lane + u * HAL_WAVE;
    if (j < top) wgt[(size_t)t * top + j] = normalize ? kept[u] / (sum + norm_eps) : kept[u];
  }
}

__global__ void __launch_bounds__(HAL_WAVE) moe_route_kernel(const float* __restrict__ z, int ldz, int E, int top, int softmax,
                                                             int normalize, float norm_eps, int* __restrict__ idx,
                                                             float* __restrict__ wgt, int n_tokens) {
  moe_route_token(z, ldz, E, top, softmax, normalize, norm_eps, idx, wgt, blockIdx.x, threadIdx.x);
}

extern "C" int hal_moe_route(const float* z, int ldz, int E, int top, int softmax, int normalize,
                             float norm_eps, int* idx, float* wgt, int n_tokens,
                             hipStream_t stream) {
  HAL_REQUIRE(n_tokens >= 0 && E > 0 && E <= MOE_MAX_EXPERTS && top > 0 && top <= E && ldz >= E,
              "hal_moe_route: bad sizes T=%d E=%d top=%d", n_tokens, E, top);
  if (n_tokens == 0) return 0;
  hipLaunchKernelGGL(moe_route_kernel, dim3(n_tokens), dim3(HAL_WAVE), 0, stream, z, ldz, E, top, softmax,
                     normalize, norm_eps, idx, wgt, n_tokens);
  HAL_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------
// Counting sort of the n = T * top pairs by expert, one workgroup.  offsets [E + 1]: where
// each expert's pairs begin in `sorted`; tile_offsets [E + 1]: the same counted in tiles of
// `tile` rows, each expert's count rounded up; sorted [n]: pair numbers (token * top +
// choice), expert by expert.  The order inside an expert is not fixed; nothing that is
// computed from it depends on it.
// ---------------------------------------------------------------------------------
// (idx without __restrict__: the kernel that routes and sorts in one has just written it)
__device__ __forceinline__ void moe_sort_pairs(const int* idx, int n, int E, int tile,
                                               int* __restrict__ offsets, int* __restrict__ tile_offsets,
                                               int* __restrict__ sorted, int* count, int* cursor) {
  for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int e = idx[i];
    if (e >= 0 && e < E) atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, tiles = 0;
    for (int e = 0; e < E; ++e) {
      offsets[e] = at;
      tile_offsets[e] = tiles;
      cursor[e] = at;
      at += count[e];
      tiles += (count[e] + tile - 1) / tile;
    }
    offsets[E] = at;
    tile_offsets[E] = tiles;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int e = idx[i];
    if (e >= 0 && e < E) sorted[atomicAdd(&cursor[e], 1)] = i;
  }
}

__global__ void __launch_bounds__(1024) moe_sort_kernel(const int* __restrict__ idx, int n, int E, int tile,
                                                        int* __restrict__ offsets,
                                                        int* __restrict__ tile_offsets,
                                                        int* __restrict__ sorted) {
  __shared__ int count[MOE_MAX_EXPERTS];
  __shared__ int cursor[MOE_MAX_EXPERTS];
  moe_sort_pairs(idx, n, E, tile, offsets, tile_offsets, sorted, count, cursor);
}

// Both in one workgroup, for steps of few tokens: its sixteen waves take the tokens in turn,
// then all of it sorts the pairs.
__global__ void __launch_bounds__(1024) moe_route_sort_kernel(const float* __restrict__ z, int ldz, int E, int top,
                                                              int softmax, int normalize, float norm_eps,
                                                              int* __restrict__ idx, float* __restrict__ wgt,
                                                              int n_tokens, int tile, int* __restrict__ offsets,
                                                              int* __restrict__ tile_offsets, int* __restrict__ sorted) {
  __shared__ int count[MOE_MAX_EXPERTS];
  __shared__ int cursor[MOE_MAX_EXPERTS];
  const int wave = threadIdx.x / HAL_WAVE, lane = threadIdx.x % HAL_WAVE;
  for (int t = wave; t < n_tokens; t += 1024 / HAL_WAVE)
    moe_route_token(z, ldz, E, top, softmax, normalize, norm_eps, idx, wgt, t, lane);
  __threadfence_block();
  __syncthreads();
  moe_sort_pairs(idx, n_tokens * top, E, tile, offsets, tile_offsets, sorted, count, cursor);
}

extern "C" int hal_moe_route_sort(const float* z, int ldz, int E, int top, int softmax, int normalize, float norm_eps,
                                  int* idx, float* wgt, int n_tokens, int tile, int* offsets, int* tile_offsets,
                                  int* sorted, hipStream_t stream) {
  HAL_REQUIRE(n_tokens >= 0 && E > 0 && E <= MOE_MAX_EXPERTS && top > 0 && top <= E && ldz >= E && tile > 0,
              "hal_moe_route_sort: bad sizes T=%d E=%d top=%d", n_tokens, E, top);
  hipLaunchKernelGGL(moe_route_sort_kernel, dim3(1), dim3(1024), 0, stream, z, ldz, E, top, softmax, normalize, norm_eps,
                     idx, wgt, n_tokens, tile, offsets, tile_offsets, sorted);
  HAL_LAUNCH_CHECK();
  return 0;
}

extern "C" int hal_moe_sort(const int* idx, int n, int E, int tile, int* offsets, int* tile_offsets,
                            int* sorted, hipStream_t stream) {
  HAL_REQUIRE(n >= 0 && E > 0 && E <= MOE_MAX_EXPERTS && tile > 0, "hal_moe_sort: bad sizes n=%d E=%d", n, E);
  hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 0, stream, idx, n, E, tile, offsets,
                     tile_offsets, sorted);
  HAL_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------
// h[t, :] += sum_j wgt[t, j] * y[t * top + j, :] (+ extra[t, :])   (y float32 [T * top, d])
// ---------------------------------------------------------------------------------
__global__ void moe_combine_kernel(float* __restrict__ h, const float* __restrict__ y,
                                   const float* __restrict__ wgt, const float* __restrict__ extra,
                                   const float* __restrict__ extra_gate, int ld_gate, int top, int d, bool overwrite) {
  const int t = blockIdx.x;
  const float eg = extra_gate ? 1.0f / (1.0f + expf(-extra_gate[(size_t)t * ld_gate])) : 1.0f;
  // (a step of few tokens spreads a row over several workgroups: blockIdx.y takes every gridDim.y-th run of columns)
  for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < d; i += blockDim.x * gridDim.y) {
    float s = extra ? eg * extra[(size_t)t * d + i] : 0.f;
    for (int j = 0; j < top; ++j) s += wgt[(size_t)t * top + j] * y[((size_t)t * top + j) * d + i];
    h[(size_t)t * d + i] = overwrite ? s : h[(size_t)t * d + i] + s;
  }
}

extern "C" int hal_moe_combine(float* h, const float* y, const float* wgt, const float* extra,
                               const float* extra_gate, int ld_gate, int top, int d, int n_tokens,
                               int overwrite, hipStream_t stream) {
  HAL_REQUIRE(n_tokens >= 0 && top > 0 && d > 0, "hal_moe_combine: bad sizes");
  if (n_tokens == 0) return 0;
  int threads = (d + 63) / 64 * 64;
  if (threads > 256) threads = 256;
  int parts = 1;  // workgroups a row, so that a decode step has a few hundred of them
  while (parts < 16 && n_tokens * parts < 256 && d / (threads * parts * 2) >= 1) parts *= 2;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(n_tokens, parts), dim3(threads), 0, stream, h, y, wgt, extra, extra_gate, ld_gate, top, d, overwrite != 0);
  HAL_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------
// out[t, f] = g * sigmoid(alpha * g) * (u + 1) with g = min(gu[t, f], limit) and
// u = clamp(gu[t, F + f], -limit, limit): the activation of a clamped gated feed-forward
// whose gate and up projections are the two halves of one product's rows.
// ---------------------------------------------------------------------------------
template <typename T>
__global__ void clamped_gate_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int F, float limit,
                                        float alpha, float up_shift) {
  const int t = blockIdx.x;
  const int f = blockIdx.y * blockDim.x + threadIdx.x;
  if (f >= F) return;
  const float g = fminf(to_f32(gu[(size_t)t * 2 * F + f]), limit);
  const float u = fminf(fmaxf(to_f32(gu[(size_t)t * 2 * F + F + f]), -limit), limit);
  out[(size_t)t * F + f] = from_f32<T>(g / (1.0f + __expf(-alpha * g)) * (u + up_shift));
}

extern "C" int hal_clamped_gate_mul(const void* gu, void* out, int dtype, int n_tokens, int F,
                                    float limit, float alpha, float up_shift, hipStream_t stream) {
  HAL_REQUIRE(n_tokens >= 0 && F > 0, "hal_clamped_gate_mul: bad sizes T=%d F=%d", n_tokens, F);
  HAL_REQUIRE(dtype == HAL_F32 || dtype == HAL_BF16, "hal_clamped_gate_mul: dtype %d", dtype);
  HAL_REQUIRE((F + 255) / 256 <= 65535, "hal_clamped_gate_mul: %d columns", F);
  if (n_tokens == 0) return 0;
  dim3 grid(n_tokens, (F + 255) / 256);
  if (dtype == HAL_F32)
    hipLaunchKernelGGL(clamped_gate_mul_kernel<float>, grid, dim3(256), 0, stream, (const float*)gu,
                       (float*)out, F, limit, alpha, up_shift);
  else
    hipLaunchKernelGGL(clamped_gate_mul_kernel<bf16_t>, grid, dim3(256), 0, stream, (const bf16_t*)gu,
                       (bf16_t*)out, F, limit, alpha, up_shift);
  HAL_LAUNCH_CHECK();
  return 0;
}
