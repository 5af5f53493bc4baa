// Small kernels on rows of the residual stream and of projections.  All arithmetic is
// float32; T is the element type of activations (float or bf16).
//
//   * the stream's rows rounded to the activation type (for a part that reads the stream
//     itself, without a norm before it);
//   * a norm on a part's *result*: h += a * rstd(a) * w, in one pass;
//   * the square of relu;
//   * y = alpha * y + beta * x on float32 rows (the sum of mixers that run side by side);
//   * queries and keys normed over the whole projection (all heads at once), the queries
//     multiplied by a temperature that grows with the logarithm of the position, and
//     queries, keys and values laid into the packed rows that the kernels which rotate,
//     append and attend take; the values may be the keys as they were projected.
#include "hal_common.h"
#include "hal_api.h"

template <typename T>
__global__ void cast_rows_kernel(const float* __restrict__ h, T* __restrict__ out, long long n4) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n4) return;
  float v[4];
  load4(h + i * 4, v);
  store4(out + i * 4, v);
}
template <typename T>
__global__ void cast_each_kernel(const float* __restrict__ h, T* __restrict__ out, long long n) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = from_f32<T>(h[i]);
}

extern "C" int hal_cast_rows(const float* h, void* out, int dtype, long long n, hipStream_t stream) {
  HAL_REQUIRE(n >= 0, "hal_cast_rows: %lld elements", n);
  HAL_REQUIRE(dtype == HAL_F32 || dtype == HAL_BF16, "hal_cast_rows: dtype %d", dtype);
  if (n == 0) return 0;
  if (n % 4 != 0 || ((uintptr_t)h % 16) != 0 || ((uintptr_t)out % 8) != 0) {  // no vectors of four
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (dtype == HAL_F32)
      hipLaunchKernelGGL(cast_each_kernel<float>, dim3(blocks), dim3(256), 0, stream, h, (float*)out, n);
    else
      hipLaunchKernelGGL(cast_each_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream, h, (bf16_t*)out, n);
    HAL_LAUNCH_CHECK();
    return 0;
  }
  const long long n4 = n / 4;
  const unsigned blocks = (unsigned)((n4 + 255) / 256);
  if (dtype == HAL_F32)
    hipLaunchKernelGGL(cast_rows_kernel<float>, dim3(blocks), dim3(256), 0, stream, h, (float*)out, n4);
  else
    hipLaunchKernelGGL(cast_rows_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream, h, (bf16_t*)out, n4);
  HAL_LAUNCH_CHECK();
  return 0;
}

// h[r] += x * rsqrt(mean(x^2) + eps) * w with x = s1 * a[r] (+ s2 * a2[r] if a2); cast (or
// null) receives the new row rounded to T
template <typename T>
__global__ void post_norm_add_kernel(float* __restrict__ h, const float* __restrict__ a,
                                     const float* __restrict__ a2, float s1, float s2,
                                     const void* __restrict__ w, int w_dtype, float eps,
                                     T* __restrict__ cast, int d) {
  __shared__ float scratch[16];
  const size_t r = blockIdx.x;
  const float* ar = a + r * d;
  const float* br = a2 ? a2 + r * d : nullptr;
  auto term = [&](int i) { return br ? __fadd_rn(__fmul_rn(s1, ar[i]), __fmul_rn(s2, br[i])) : __fmul_rn(s1, ar[i]); };
  float ss = 0.f;
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    const float x = term(i);
    ss += x * x;
  }
  const float total = block_sum(ss, scratch);
  const float rstd = 1.0f / sqrtf(total / (float)d + eps);
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    const float y = h[r * d + i] + term(i) * rstd * load_as_f32(w, w_dtype, i);
    h[r * d + i] = y;
    if (cast) cast[r * d + i] = from_f32<T>(y);
  }
}

// The same for rows of a multiple of four elements, up to 4 * VMAX * threads: a thread keeps
// its part of the row in registers between the sum of squares and the update, and every
// access is 16 bytes (a few rows of a decode step are a few workgroups whose time is the
// chain of their trips to memory).
template <typename T, int VMAX>
__global__ void post_norm_add_vec_kernel(float* __restrict__ h, const float* __restrict__ a,
                                         const float* __restrict__ a2, float s1, float s2,
                                         const void* __restrict__ w, int w_dtype, float eps,
                                         T* __restrict__ cast, int d) {
  __shared__ float scratch[16];
  const size_t r = blockIdx.x;
  const int nv = d / 4;
  float x[VMAX][4], hv[VMAX][4], wv[VMAX][4];
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < VMAX; ++u) {
    const int v = threadIdx.x + u * blockDim.x;
    if (v < nv) {
      load4(a + r * d + v * 4, x[u]);
      load4(h + r * d + v * 4, hv[u]);
      load4_any(w, w_dtype, (size_t)v * 4, wv[u]);
      if (a2) {
        float y[4];
        load4(a2 + r * d + v * 4, y);
#pragma unroll
        for (int i = 0; i < 4; ++i) x[u][i] = __fadd_rn(__fmul_rn(s1, x[u][i]), __fmul_rn(s2, y[i]));
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) x[u][i] = __fmul_rn(s1, x[u][i]);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) ss += x[u][i] * x[u][i];
    }
  }
  const float total = block_sum(ss, scratch);
  const float rstd = 1.0f / sqrtf(total / (float)d + eps);
#pragma unroll
  for (int u = 0; u < VMAX; ++u) {
    const int v = threadIdx.x + u * blockDim.x;
    if (v < nv) {
#pragma unroll
      for (int i = 0; i < 4; ++i) hv[u][i] = hv[u][i] + x[u][i] * rstd * wv[u][i];
      store4(h + r * d + v * 4, hv[u]);
      if (cast) store4(cast + r * d + v * 4, hv[u]);
    }
  }
}

extern "C" int hal_post_norm_add(float* h, const float* a, const float* a2, float s1, float s2, const void* w,
                                 int w_dtype, float eps, void* cast, int dtype, int n_rows, int d,
                                 hipStream_t stream) {
  HAL_REQUIRE(n_rows >= 0 && d > 0, "hal_post_norm_add: bad sizes rows=%d d=%d", n_rows, d);
  HAL_REQUIRE(dtype == HAL_F32 || dtype == HAL_BF16, "hal_post_norm_add: dtype %d", dtype);
  if (n_rows == 0) return 0;
  constexpr int VMAX = 8;
  const bool aligned = d % 4 == 0 && ((uintptr_t)h % 16) == 0 && ((uintptr_t)a % 16) == 0 && ((uintptr_t)a2 % 16) == 0 &&
                       ((uintptr_t)w % 16) == 0 && ((uintptr_t)cast % 16) == 0;
  if (aligned && d <= 4 * VMAX * 256) {
    const int nv = d / 4;
    const int threads = nv >= 1024 ? 256 : (nv >= 256 ? 128 : 64);  // (at most VMAX vectors a thread)
    if (dtype == HAL_F32)
      hipLaunchKernelGGL((post_norm_add_vec_kernel<float, VMAX>), dim3(n_rows), dim3(threads), 0, stream, h, a, a2, s1,
                         s2, w, w_dtype, eps, (float*)cast, d);
    else
      hipLaunchKernelGGL((post_norm_add_vec_kernel<bf16_t, VMAX>), dim3(n_rows), dim3(threads), 0, stream, h, a, a2, s1,
                         s2, w, w_dtype, eps, (bf16_t*)cast, d);
    HAL_LAUNCH_CHECK();
    return 0;
  }
  const int threads = d >= 1024 ? 256 : (d >= 256 ? 128 : 64);
  if (dtype == HAL_F32)
    hipLaunchKernelGGL(post_norm_add_kernel<float>, dim3(n_rows), dim3(threads), 0, stream, h, a, a2, s1, s2, w,
                       w_dtype, eps, (float*)cast, d);
  else
    hipLaunchKernelGGL(post_norm_add_kernel<bf16_t>, dim3(n_rows), dim3(threads), 0, stream, h, a, a2, s1, s2, w,
                       w_dtype, eps, (bf16_t*)cast, d);
  HAL_LAUNCH_CHECK();
  return 0;
}

template <typename T>
__global__ void relu_squared_kernel(const T* __restrict__ x, T* __restrict__ out, long long n) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float v = fmaxf(to_f32(x[i]), 0.f);
  out[i] = from_f32<T>(v * v);
}

template <typename T>
__global__ void relu_squared_vec_kernel(const T* __restrict__ x, T* __restrict__ out, long long n4) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n4) return;
  float v[4];
  load4(x + i * 4, v);
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const float r = fmaxf(v[u], 0.f);
    v[u] = r * r;
  }
  store4(out + i * 4, v);
}

extern "C" int hal_relu_squared(const void* x, void* out, int dtype, long long n, hipStream_t stream) {
  HAL_REQUIRE(n >= 0, "hal_relu_squared: %lld elements", n);
  HAL_REQUIRE(dtype == HAL_F32 || dtype == HAL_BF16, "hal_relu_squared: dtype %d", dtype);
  if (n == 0) return 0;
  if (n % 4 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)out % 16) == 0) {
    const unsigned blocks = (unsigned)((n / 4 + 255) / 256);
    if (dtype == HAL_F32)
      hipLaunchKernelGGL(relu_squared_vec_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)x, (float*)out, n / 4);
    else
      hipLaunchKernelGGL(relu_squared_vec_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream, (const bf16_t*)x, (bf16_t*)out, n / 4);
    HAL_LAUNCH_CHECK();
    return 0;
  }
  const unsigned blocks = (unsigned)((n + 255) / 256);
  if (dtype == HAL_F32)
    hipLaunchKernelGGL(relu_squared_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)x, (float*)out, n);
  else
    hipLaunchKernelGGL(relu_squared_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream, (const bf16_t*)x, (bf16_t*)out, n);
  HAL_LAUNCH_CHECK();
  return 0;
}

__global__ void scaled_sum_kernel(float* __restrict__ y, float alpha, const float* __restrict__ x, float beta,
                                  long long n) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) y[i] = __fadd_rn(__fmul_rn(alpha, y[i]), __fmul_rn(beta, x[i]));
}

extern "C" int hal_scaled_sum_f32(float* y, float alpha, const float* x, float beta, long long n,
                                  hipStream_t stream) {
  HAL_REQUIRE(n >= 0, "hal_scaled_sum_f32: %lld elements", n);
  if (n == 0) return 0;
  hipLaunchKernelGGL(scaled_sum_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, y, alpha, x, beta, n);
  HAL_LAUNCH_CHECK();
  return 0;
}

// One workgroup a token.  out row: [H heads of D | K heads of D | K heads of D], a head's
// first dq (values: dv) entries filled, the rest zero.
template <typename T>
__global__ void qk_norm_pack_kernel(const float* __restrict__ q, int ldq, const float* __restrict__ k, int ldk,
                                    const float* __restrict__ v, int ldv, const void* __restrict__ wq,
                                    const void* __restrict__ wk, int w_dtype, float eps,
                                    const int* __restrict__ positions, float temp_coef, int temp_every,
                                    T* __restrict__ out, int row_stride, int H, int K, int dq, int dv, int D,
                                    const int* __restrict__ token_seg, const int* __restrict__ block_table,
                                    int bt_stride, T* __restrict__ k_pages, T* __restrict__ v_pages,
                                    int page_size, int n_pages, bool tiled) {
  __shared__ float scratch[16];
  const size_t t = blockIdx.x;
  // with pages: keys and values go to the request's page of this position as well
  long long page = -1;
  int off = 0;
  if (k_pages) {
    const int pos = positions[t];
    page = block_table[(size_t)token_seg[t] * bt_stride + pos / page_size];
    off = pos % page_size;
    if (page < 0 || page >= n_pages) page = -1;  // checked on the host
  }
  const float* qr = q + t * ldq;
  const float* kr = k + t * ldk;
  const float* vr = v ? v + t * ldv : nullptr;
  const int nq = H * dq, nk = K * dq;
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x; i < nq; i += blockDim.x) sq += qr[i] * qr[i];
  for (int i = threadIdx.x; i < nk; i += blockDim.x) sk += kr[i] * kr[i];
  const float tq = block_sum(sq, scratch);
  const float tk = block_sum(sk, scratch);
  float rq = 1.0f / sqrtf(tq / (float)nq + eps);
  const float rk = 1.0f / sqrtf(tk / (float)nk + eps);
  if (temp_every > 0) {
    const int p = positions[t];
    rq *= 1.0f + temp_coef * logf((float)((p + 1) / temp_every + 1));
  }
  T* o = out + t * row_stride;
  for (int e = threadIdx.x; e < H * D; e += blockDim.x) {
    const int hd = e / D, d = e % D;
    float x = 0.f;
    if (d < dq) x = qr[hd * dq + d] * rq * load_as_f32(wq, w_dtype, hd * dq + d);
    o[e] = from_f32<T>(x);
  }
  for (int e = threadIdx.x; e < K * D; e += blockDim.x) {
    const int hd = e / D, d = e % D;
    float x = 0.f, y = 0.f;
    if (d < dq) x = kr[hd * dq + d] * rk * load_as_f32(wk, w_dtype, hd * dq + d);
    if (d < dv) y = vr ? vr[hd * dv + d] : kr[hd * dq + d];
    o[H * D + e] = from_f32<T>(x);
    o[(H + K) * D + e] = from_f32<T>(y);
    if (page >= 0) {
      k_pages[((size_t)page * K + hd) * page_size * D + kv_key_offset(tiled, page_size, D, off, d)] = from_f32<T>(x);
      v_pages[((size_t)page * K + hd) * D * page_size + kv_value_offset(tiled, page_size, D, off, d)] = from_f32<T>(y);
    }
  }
}

// The same with 16-byte accesses, for head sizes, row lengths and addresses in steps of four.
template <typename T>
__global__ void qk_norm_pack_vec_kernel(const float* __restrict__ q, int ldq, const float* __restrict__ k, int ldk,
                                        const float* __restrict__ v, int ldv, const void* __restrict__ wq,
                                        const void* __restrict__ wk, int w_dtype, float eps,
                                        const int* __restrict__ positions, float temp_coef, int temp_every,
                                        T* __restrict__ out, int row_stride, int H, int K, int dq, int dv, int D,
                                        const int* __restrict__ token_seg, const int* __restrict__ block_table,
                                        int bt_stride, T* __restrict__ k_pages, T* __restrict__ v_pages,
                                        int page_size, int n_pages, bool tiled) {
  __shared__ float scratch[16];
  const size_t t = blockIdx.x;
  long long page = -1;
  int off = 0;
  if (k_pages) {
    const int pos = positions[t];
    page = block_table[(size_t)token_seg[t] * bt_stride + pos / page_size];
    off = pos % page_size;
    if (page < 0 || page >= n_pages) page = -1;  // checked on the host
  }
  const float* qr = q + t * ldq;
  const float* kr = k + t * ldk;
  const float* vr = v ? v + t * ldv : nullptr;
  const int nq = H * dq, nk = K * dq;
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x * 4; i < nq; i += blockDim.x * 4) {
    float x[4];
    load4(qr + i, x);
    sq += (x[0] * x[0] + x[1] * x[1]) + (x[2] * x[2] + x[3] * x[3]);
  }
  for (int i = threadIdx.x * 4; i < nk; i += blockDim.x * 4) {
    float x[4];
    load4(kr + i, x);
    sk += (x[0] * x[0] + x[1] * x[1]) + (x[2] * x[2] + x[3] * x[3]);
  }
  const float tq = block_sum(sq, scratch);
  const float tk = block_sum(sk, scratch);
  float rq = 1.0f / sqrtf(tq / (float)nq + eps);
  const float rk = 1.0f / sqrtf(tk / (float)nk + eps);
  if (temp_every > 0) {
    const int p = positions[t];
    rq *= 1.0f + temp_coef * logf((float)((p + 1) / temp_every + 1));
  }
  T* o = out + t * row_stride;
  const int D4 = D / 4;
  for (int e = threadIdx.x; e < H * D4; e += blockDim.x) {
    const int hd = e / D4, d = (e % D4) * 4;
    float x[4] = {0.f, 0.f, 0.f, 0.f};
    if (d < dq) {
      float wv[4];
      load4(qr + hd * dq + d, x);
      load4_any(wq, w_dtype, (size_t)hd * dq + d, wv);
#pragma unroll
      for (int i = 0; i < 4; ++i) x[i] = x[i] * rq * wv[i];
    }
    store4(o + (size_t)hd * D + d, x);
  }
  for (int e = threadIdx.x; e < K * D4; e += blockDim.x) {
    const int hd = e / D4, d = (e % D4) * 4;
    float x[4] = {0.f, 0.f, 0.f, 0.f}, y[4] = {0.f, 0.f, 0.f, 0.f}, raw[4] = {0.f, 0.f, 0.f, 0.f};
    if (d < dq) {
      float wv[4];
      load4(kr + hd * dq + d, raw);
      load4_any(wk, w_dtype, (size_t)hd * dq + d, wv);
#pragma unroll
      for (int i = 0; i < 4; ++i) x[i] = raw[i] * rk * wv[i];
    }
    if (d < dv) {
      if (vr) load4(vr + hd * dv + d, y);
      else {
#pragma unroll
        for (int i = 0; i < 4; ++i) y[i] = raw[i];
      }
    }
    store4(o + (size_t)(H + hd) * D + d, x);
    store4(o + (size_t)(H + K + hd) * D + d, y);
    if (page >= 0) {
      store4(k_pages + ((size_t)page * K + hd) * page_size * D + kv_key_offset(tiled, page_size, D, off, d), x);
      T* vp = v_pages + ((size_t)page * K + hd) * D * page_size;
#pragma unroll
      for (int i = 0; i < 4; ++i) vp[kv_value_offset(tiled, page_size, D, off, d + i)] = from_f32<T>(y[i]);
    }
  }
}

extern "C" int hal_qk_norm_pack(const float* q, int ldq, const float* k, int ldk, const float* v, int ldv,
                                const void* wq, const void* wk, int w_dtype, float eps, const int* positions,
                                float temp_coef, int temp_every, void* out, int row_stride, int dtype,
                                int n_tokens, int H, int K, int dq, int dv, int D, const int* token_seg,
                                const int* block_table, int bt_stride, void* k_pages, void* v_pages,
                                int page_size, int n_pages, int tiled, hipStream_t stream) {
  HAL_REQUIRE(k_pages == nullptr || (v_pages && token_seg && block_table && positions && page_size > 0 && n_pages > 0),
              "hal_qk_norm_pack: pages without the arrays that say where a token's key goes");
  HAL_REQUIRE(n_tokens >= 0 && H > 0 && K > 0 && dq > 0 && dv > 0 && D >= dq && D >= dv,
              "hal_qk_norm_pack: bad sizes T=%d H=%d K=%d dq=%d dv=%d D=%d", n_tokens, H, K, dq, dv, D);
  HAL_REQUIRE(v != nullptr || dv == dq, "hal_qk_norm_pack: values that are the keys have the keys' size");
  HAL_REQUIRE(row_stride >= (H + 2 * K) * D, "hal_qk_norm_pack: rows of %d elements are too short", row_stride);
  HAL_REQUIRE(temp_every == 0 || positions != nullptr, "hal_qk_norm_pack: a temperature needs positions");
  HAL_REQUIRE(dtype == HAL_F32 || dtype == HAL_BF16, "hal_qk_norm_pack: dtype %d", dtype);
  if (n_tokens == 0) return 0;
  const bool by_four = dq % 4 == 0 && dv % 4 == 0 && D % 4 == 0 && ldq % 4 == 0 && ldk % 4 == 0 && ldv % 4 == 0 &&
                       row_stride % 4 == 0 && ((uintptr_t)q % 16) == 0 && ((uintptr_t)k % 16) == 0 &&
                       ((uintptr_t)v % 16) == 0 && ((uintptr_t)wq % 16) == 0 && ((uintptr_t)wk % 16) == 0 &&
                       ((uintptr_t)out % 16) == 0 && ((uintptr_t)k_pages % 16) == 0;
  if (by_four) {
    if (dtype == HAL_F32)
      hipLaunchKernelGGL(qk_norm_pack_vec_kernel<float>, dim3(n_tokens), dim3(256), 0, stream, q, ldq, k, ldk, v, ldv,
                         wq, wk, w_dtype, eps, positions, temp_coef, temp_every, (float*)out, row_stride, H, K, dq, dv,
                         D, token_seg, block_table, bt_stride, (float*)k_pages, (float*)v_pages, page_size, n_pages,
                         tiled != 0);
    else
      hipLaunchKernelGGL(qk_norm_pack_vec_kernel<bf16_t>, dim3(n_tokens), dim3(256), 0, stream, q, ldq, k, ldk, v, ldv,
                         wq, wk, w_dtype, eps, positions, temp_coef, temp_every, (bf16_t*)out, row_stride, H, K, dq, dv,
                         D, token_seg, block_table, bt_stride, (bf16_t*)k_pages, (bf16_t*)v_pages, page_size, n_pages,
                         tiled != 0);
    HAL_LAUNCH_CHECK();
    return 0;
  }
  if (dtype == HAL_F32)
    hipLaunchKernelGGL(qk_norm_pack_kernel<float>, dim3(n_tokens), dim3(256), 0, stream, q, ldq, k, ldk, v, ldv, wq,
                       wk, w_dtype, eps, positions, temp_coef, temp_every, (float*)out, row_stride, H, K, dq, dv, D,
                       token_seg, block_table, bt_stride, (float*)k_pages, (float*)v_pages, page_size, n_pages,
                       tiled != 0);
  else
    hipLaunchKernelGGL(qk_norm_pack_kernel<bf16_t>, dim3(n_tokens), dim3(256), 0, stream, q, ldq, k, ldk, v, ldv, wq,
                       wk, w_dtype, eps, positions, temp_coef, temp_every, (bf16_t*)out, row_stride, H, K, dq, dv, D,
                       token_seg, block_table, bt_stride, (bf16_t*)k_pages, (bf16_t*)v_pages, page_size, n_pages,
                       tiled != 0);
  HAL_LAUNCH_CHECK();
  return 0;
}

// ---- several copies of the residual stream.  x [S][T][W] float32; a workgroup a row.
// With y (a part's result, float32 [T][W]) every copy is made anew from the old ones,
//   x_t <- sum_s mix[s][t] x_s + m * out[t] * y,
// and, if `read`, the row that the next part reads is made of the new copies,
//   u = sum_s in[s] x_s   (in null: every copy counts once),
// and either written as it is (norm_w null) or normed: u / sqrt(mean(u^2) + eps) * (offset + w).
// `rows` (or null): which rows of x the workgroups take; the results are written in that order.
template <typename TO, int MAXS>
__global__ void streams_step_kernel(float* __restrict__ x, size_t copy_stride, int S, const float* __restrict__ y,
                                    const void* __restrict__ mix, const void* __restrict__ outw, float m,
                                    const void* __restrict__ inw, int c_dtype, int read,
                                    const void* __restrict__ norm_w, int norm_dtype, float offset, float eps,
                                    TO* __restrict__ result, const int* __restrict__ rows, int W) {
  extern __shared__ float u_row[];
  __shared__ float scratch[16];
  const size_t t = rows ? (size_t)rows[blockIdx.x] : (size_t)blockIdx.x;
  float cm[MAXS][MAXS], co[MAXS], ci[MAXS];
#pragma unroll
  for (int s = 0; s < MAXS; ++s) {
    co[s] = (y && s < S) ? m * load_as_f32(outw, c_dtype, s) : 0.f;
    ci[s] = s < S ? (inw ? load_as_f32(inw, c_dtype, s) : 1.0f) : 0.f;
#pragma unroll
    for (int d = 0; d < MAXS; ++d) cm[s][d] = (y && s < S && d < S) ? load_as_f32(mix, c_dtype, s * S + d) : 0.f;
  }
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float xs[MAXS];
#pragma unroll
    for (int s = 0; s < MAXS; ++s) xs[s] = s < S ? x[s * copy_stride + t * W + i] : 0.f;
    if (y) {
      const float yv = y[t * W + i];
      float nx[MAXS];
#pragma unroll
      for (int d = 0; d < MAXS; ++d) {
        float acc = co[d] * yv;
#pragma unroll
        for (int s = 0; s < MAXS; ++s) acc = fmaf(cm[s][d], xs[s], acc);
        nx[d] = acc;
      }
#pragma unroll
      for (int s = 0; s < MAXS; ++s) {
        xs[s] = nx[s];
        if (s < S) x[s * copy_stride + t * W + i] = nx[s];
      }
    }
    if (read) {
      float u = 0.f;
#pragma unroll
      for (int s = 0; s < MAXS; ++s) u = fmaf(ci[s], xs[s], u);
      if (norm_w) {
        u_row[i] = u;
        ss += u * u;
      } else {
        result[(size_t)blockIdx.x * W + i] = from_f32<TO>(u);
      }
    }
  }
  if (!read || !norm_w) return;
  const float total = block_sum(ss, scratch);
  const float rstd = 1.0f / sqrtf(total / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x)  // (a thread reads back what it wrote itself)
    result[(size_t)blockIdx.x * W + i] = from_f32<TO>(u_row[i] * rstd * (offset + load_as_f32(norm_w, norm_dtype, i)));
}

extern "C" int hal_streams_step(float* x, long long copy_stride, int S, const float* y, const void* mix,
                                const void* outw, float m, const void* inw, int c_dtype, int read,
                                const void* norm_w, int norm_dtype, float offset, float eps, void* result,
                                int result_dtype, const int* rows, int n_rows, int W, hipStream_t stream) {
  HAL_REQUIRE(S >= 1 && S <= 8, "hal_streams_step: %d copies of the stream (1 to 8)", S);
  HAL_REQUIRE(n_rows >= 0 && W > 0 && W <= 16384, "hal_streams_step: bad sizes rows=%d width=%d", n_rows, W);
  HAL_REQUIRE(y == nullptr || (mix && outw && rows == nullptr), "hal_streams_step: an update needs its weights and all rows");
  HAL_REQUIRE(!read || result, "hal_streams_step: nowhere to write the row that was read");
  HAL_REQUIRE(y || read, "hal_streams_step: nothing to do");
  HAL_REQUIRE(result_dtype == HAL_F32 || result_dtype == HAL_BF16, "hal_streams_step: dtype %d", result_dtype);
  if (n_rows == 0) return 0;
  const size_t lds = (read && norm_w) ? (size_t)W * sizeof(float) : 0;
#define STREAMS_LAUNCH(T_, M_)                                                                                      \
  hipLaunchKernelGGL((streams_step_kernel<T_, M_>), dim3(n_rows), dim3(256), lds, stream, x, (size_t)copy_stride, S, y, \
                     mix, outw, m, inw, c_dtype, read, norm_w, norm_dtype, offset, eps, (T_*)result, rows, W)
#define STREAMS_BY_COUNT(T_)                \
  do {                                      \
    if (S <= 2) STREAMS_LAUNCH(T_, 2);      \
    else if (S <= 4) STREAMS_LAUNCH(T_, 4); \
    else STREAMS_LAUNCH(T_, 8);             \
  } while (0)
  if (result_dtype == HAL_F32) STREAMS_BY_COUNT(float);
  else STREAMS_BY_COUNT(bf16_t);
#undef STREAMS_BY_COUNT
#undef STREAMS_LAUNCH
  HAL_LAUNCH_CHECK();
  return 0;
}

// ---- every head of q, k and v divided by its own root mean square (no weight), packed as
// [H heads of D | K heads of D | K heads of D] with zeros beyond a head's entries, keys and
// values appended to the pages as well (k_pages null: not).  A wave a (token, head). ---------
template <typename T>
__global__ void head_norm_pack_kernel(const float* __restrict__ q, int ldq, const float* __restrict__ k, int ldk,
                                      const float* __restrict__ v, int ldv, float eps,
                                      const void* __restrict__ w_q, const void* __restrict__ w_k, int w_dtype,
                                      bool norm_v, const float* __restrict__ v_other, int ldvo, float v_mix,
                                      const int* __restrict__ positions, T* __restrict__ out, int row_stride,
                                      int n_tokens, int H, int K, int dq, int dv, int D,
                                      const int* __restrict__ token_seg, const int* __restrict__ block_table,
                                      int bt_stride, T* __restrict__ k_pages, T* __restrict__ v_pages, int page_size,
                                      int n_pages, bool tiled) {
  const int lane = threadIdx.x % HAL_WAVE, slots = H + 2 * K;
  const size_t unit = (size_t)blockIdx.x * (blockDim.x / HAL_WAVE) + threadIdx.x / HAL_WAVE;
  if (unit >= (size_t)n_tokens * slots) return;
  const size_t t = unit / slots;
  const int hs = (int)(unit % slots);
  const int kind = hs < H ? 0 : (hs < H + K ? 1 : 2);
  const int head = kind == 0 ? hs : (kind == 1 ? hs - H : hs - H - K);
  const int n = kind == 2 ? dv : dq;
  const float* src = kind == 0 ? q + t * ldq + (size_t)head * dq
                               : (kind == 1 ? k + t * ldk + (size_t)head * dq : v + t * ldv + (size_t)head * dv);
  float rstd = 1.0f;
  if (kind != 2 || norm_v) {
    float ss = 0.f;
    for (int i = lane; i < n; i += HAL_WAVE) ss += src[i] * src[i];
    rstd = 1.0f / sqrtf(wave_sum(ss) / (float)n + eps);
  }
  // (a weight of the head's size, shared by the heads; values: a blend with another layer's)
  const void* w = kind == 0 ? w_q : (kind == 1 ? w_k : nullptr);
  const float* other = (kind == 2 && v_other) ? v_other + t * ldvo + (size_t)head * dv : nullptr;
  long long page = -1;
  int off = 0;
  if (k_pages && kind != 0) {
    const int pos = positions[t];
    page = block_table[(size_t)token_seg[t] * bt_stride + pos / page_size];
    off = pos % page_size;
    if (page < 0 || page >= n_pages) page = -1;  // checked on the host
  }
  T* o = out + t * row_stride + (size_t)hs * D;
  for (int d = lane; d < D; d += HAL_WAVE) {
    float f = d < n ? src[d] * rstd : 0.f;
    if (w && d < n) f *= load_as_f32(w, w_dtype, d);
    if (other && d < n) f = (1.0f - v_mix) * f + v_mix * other[d];
    const T x = from_f32<T>(f);
    o[d] = x;
    if (page >= 0) {
      if (kind == 1) k_pages[((size_t)page * K + head) * page_size * D + kv_key_offset(tiled, page_size, D, off, d)] = x;
      else v_pages[((size_t)page * K + head) * D * page_size + kv_value_offset(tiled, page_size, D, off, d)] = x;
    }
  }
}

extern "C" int hal_head_norm_pack(const float* q, int ldq, const float* k, int ldk, const float* v, int ldv, float eps,
                                  const void* w_q, const void* w_k, int w_dtype, int norm_v, const float* v_other,
                                  int ldvo, float v_mix, const int* positions, void* out, int row_stride, int dtype, int n_tokens, int H,
                                  int K, int dq, int dv, int D, const int* token_seg, const int* block_table,
                                  int bt_stride, void* k_pages, void* v_pages, int page_size, int n_pages, int tiled,
                                  hipStream_t stream) {
  HAL_REQUIRE(k_pages == nullptr || (v_pages && token_seg && block_table && positions && page_size > 0 && n_pages > 0),
              "hal_head_norm_pack: pages without the arrays that say where a token's key goes");
  HAL_REQUIRE(n_tokens >= 0 && H > 0 && K > 0 && dq > 0 && dv > 0 && D >= dq && D >= dv,
              "hal_head_norm_pack: bad sizes T=%d H=%d K=%d dq=%d dv=%d D=%d", n_tokens, H, K, dq, dv, D);
  HAL_REQUIRE(row_stride >= (H + 2 * K) * D && ldq >= H * dq && ldk >= K * dq && ldv >= K * dv,
              "hal_head_norm_pack: rows too short");
  HAL_REQUIRE(dtype == HAL_F32 || dtype == HAL_BF16, "hal_head_norm_pack: dtype %d", dtype);
  HAL_REQUIRE((w_q == nullptr) == (w_k == nullptr) && (w_q == nullptr || w_dtype == HAL_F32 || w_dtype == HAL_BF16),
              "hal_head_norm_pack: weights for both q and k or for neither, float32 or bf16");
  HAL_REQUIRE(v_other == nullptr || ldvo >= K * dv, "hal_head_norm_pack: rows of the other values too short");
  if (n_tokens == 0) return 0;
  const long long units = (long long)n_tokens * (H + 2 * K);
  const dim3 grid((unsigned)((units + 3) / 4));
  if (dtype == HAL_F32)
    hipLaunchKernelGGL(head_norm_pack_kernel<float>, grid, dim3(256), 0, stream, q, ldq, k, ldk, v, ldv, eps, w_q, w_k,
                       w_dtype, norm_v != 0, v_other, ldvo, v_mix, positions,
                       (float*)out, row_stride, n_tokens, H, K, dq, dv, D, token_seg, block_table, bt_stride,
                       (float*)k_pages, (float*)v_pages, page_size, n_pages, tiled != 0);
  else
    hipLaunchKernelGGL(head_norm_pack_kernel<bf16_t>, grid, dim3(256), 0, stream, q, ldq, k, ldk, v, ldv, eps, w_q, w_k,
                       w_dtype, norm_v != 0, v_other, ldvo, v_mix, positions,
                       (bf16_t*)out, row_stride, n_tokens, H, K, dq, dv, D, token_seg, block_table, bt_stride,
                       (bf16_t*)k_pages, (bf16_t*)v_pages, page_size, n_pages, tiled != 0);
  HAL_LAUNCH_CHECK();
  return 0;
}

// ---- y[t, h * n + j] = x[t, h * x_head + j] * sigmoid(g[t, h]) for j < n: every head's result
// times one number of its own, the heads' padding dropped on the way -------------------------
template <typename T>
__global__ void head_gate_cols_kernel(const T* __restrict__ x, int ldx, int x_head, const float* __restrict__ g, int ldg,
                                      T* __restrict__ y, int n, int H) {
  const size_t t = blockIdx.x;
  for (int e = threadIdx.x; e < H * n; e += blockDim.x) {
    const int h = e / n, j = e % n;
    const float gate = 1.0f / (1.0f + expf(-g[t * ldg + h]));
    y[t * H * n + e] = from_f32<T>(to_f32(x[t * ldx + (size_t)h * x_head + j]) * gate);
  }
}

extern "C" int hal_head_gate_cols(const void* x, int ldx, int x_head, const float* g, int ldg, void* y, int n, int H,
                                  int dtype, int n_tokens, hipStream_t stream) {
  HAL_REQUIRE(n_tokens >= 0 && H > 0 && n > 0 && x_head >= n && ldx >= H * x_head && ldg >= H,
              "hal_head_gate_cols: bad sizes T=%d heads=%d n=%d of %d", n_tokens, H, n, x_head);
  HAL_REQUIRE(dtype == HAL_F32 || dtype == HAL_BF16, "hal_head_gate_cols: dtype %d", dtype);
  if (n_tokens == 0) return 0;
  if (dtype == HAL_F32)
    hipLaunchKernelGGL(head_gate_cols_kernel<float>, dim3(n_tokens), dim3(256), 0, stream, (const float*)x, ldx, x_head,
                       g, ldg, (float*)y, n, H);
  else
    hipLaunchKernelGGL(head_gate_cols_kernel<bf16_t>, dim3(n_tokens), dim3(256), 0, stream, (const bf16_t*)x, ldx, x_head,
                       g, ldg, (bf16_t*)y, n, H);
  HAL_LAUNCH_CHECK();
  return 0;
}

// ---- a[t, c] += bias[c]: the bias of a projection whose float32 result something reads before
// anything else could add it (a convolution over time, whose inputs before the first token are
// zeros and not the bias) ------------------------------------------------------------------
__global__ void bias_rows_kernel(float* __restrict__ a, int lda, const void* __restrict__ bias, int b_dtype, int n_cols) {
  const size_t t = blockIdx.x;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < n_cols; c += gridDim.y * blockDim.x)
    a[t * lda + c] += load_as_f32(bias, b_dtype, c);
}

extern "C" int hal_bias_rows(float* a, int lda, const void* bias, int b_dtype, int n_rows, int n_cols, hipStream_t stream) {
  HAL_REQUIRE(n_rows >= 0 && n_cols > 0 && lda >= n_cols, "hal_bias_rows: bad sizes rows=%d cols=%d", n_rows, n_cols);
  HAL_REQUIRE(b_dtype == HAL_F32 || b_dtype == HAL_BF16, "hal_bias_rows: dtype %d", b_dtype);
  if (n_rows == 0) return 0;
  const int by = n_cols >= 4096 ? 4 : 1;
  hipLaunchKernelGGL(bias_rows_kernel, dim3(n_rows, by), dim3(256), 0, stream, a, lda, bias, b_dtype, n_cols);
  HAL_LAUNCH_CHECK();
  return 0;
}

// ---- out[t, c] = silu(a[t, c]) for the first n_cols columns of float32 rows --------------------
template <typename T>
__global__ void silu_rows_kernel(const float* __restrict__ a, int lda, T* __restrict__ out, int n_cols) {
  const size_t t = blockIdx.x;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < n_cols; c += gridDim.y * blockDim.x) {
    const float z = a[t * lda + c];
    out[t * n_cols + c] = from_f32<T>(z / (1.0f + expf(-z)));
  }
}

extern "C" int hal_silu_rows(const float* a, int lda, void* out, int dtype, int n_rows, int n_cols, hipStream_t stream) {
  HAL_REQUIRE(n_rows >= 0 && n_cols > 0 && lda >= n_cols, "hal_silu_rows: bad sizes rows=%d cols=%d", n_rows, n_cols);
  HAL_REQUIRE(dtype == HAL_F32 || dtype == HAL_BF16, "hal_silu_rows: dtype %d", dtype);
  if (n_rows == 0) return 0;
  const dim3 grid(n_rows, n_cols >= 4096 ? 4 : 1);
  if (dtype == HAL_F32)
    hipLaunchKernelGGL(silu_rows_kernel<float>, grid, dim3(256), 0, stream, a, lda, (float*)out, n_cols);
  else
    hipLaunchKernelGGL(silu_rows_kernel<bf16_t>, grid, dim3(256), 0, stream, a, lda, (bf16_t*)out, n_cols);
  HAL_LAUNCH_CHECK();
  return 0;
}

// ---- out[t, j] = gelu_tanh(g[t, j]) * table[tokens[t]][col0 + j]: a small projection of the
// stream gates the token's own row of a table (a column range of it) ----------------------------
template <typename T>
__global__ void token_gate_kernel(const float* __restrict__ g, int ldg, const void* __restrict__ table, int t_dtype,
                                  int ld_table, int col0, const int* __restrict__ tokens, int vocab,
                                  T* __restrict__ out, int dim) {
  const size_t t = blockIdx.x;
  const int tok = tokens[t];
  const bool ok = tok >= 0 && tok < vocab;
  for (int j = threadIdx.x; j < dim; j += blockDim.x) {
    const float z = g[t * ldg + j];
    const float act = 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    const float e = ok ? load_as_f32(table, t_dtype, (size_t)tok * ld_table + col0 + j) : NAN;
    out[t * dim + j] = from_f32<T>(act * e);
  }
}

extern "C" int hal_token_gate(const float* g, int ldg, const void* table, int t_dtype, int ld_table, int col0,
                              const int* tokens, int vocab, void* out, int dtype, int n_rows, int dim,
                              hipStream_t stream) {
  HAL_REQUIRE(n_rows >= 0 && dim > 0 && ldg >= dim && col0 >= 0 && col0 + dim <= ld_table && vocab > 0,
              "hal_token_gate: bad sizes rows=%d dim=%d col0=%d table row=%d", n_rows, dim, col0, ld_table);
  HAL_REQUIRE((dtype == HAL_F32 || dtype == HAL_BF16) && (t_dtype == HAL_F32 || t_dtype == HAL_BF16),
              "hal_token_gate: dtypes %d, %d", dtype, t_dtype);
  if (n_rows == 0) return 0;
  const int threads = dim >= 256 ? 256 : (dim > 64 ? 128 : 64);
  if (dtype == HAL_F32)
    hipLaunchKernelGGL(token_gate_kernel<float>, dim3(n_rows), dim3(threads), 0, stream, g, ldg, table, t_dtype,
                       ld_table, col0, tokens, vocab, (float*)out, dim);
  else
    hipLaunchKernelGGL(token_gate_kernel<bf16_t>, dim3(n_rows), dim3(threads), 0, stream, g, ldg, table, t_dtype,
                       ld_table, col0, tokens, vocab, (bf16_t*)out, dim);
  HAL_LAUNCH_CHECK();
  return 0;
}
