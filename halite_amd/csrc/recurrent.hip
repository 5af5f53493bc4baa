// Kernels of mixers that carry a state of fixed size from token to token: a short causal
// convolution over time on every channel, and a selective state-space recurrence with a
// scalar decay per head.  The state lives in float32 rows, one per request slot; a step's
// tokens come as a flat batch of segments (each the next tokens of one request, in order),
// described by the step's arrays: for every token its segment and its slot, for every
// segment where its tokens start and how many there are.
//
//   y[t, c] = act(bias[c] + sum_j w[c, j] * u[t - taps + 1 + j, c])   (u = 0 before a request's start)
//   (with `in_bias`, u[t, c] stands for u[t, c] + in_bias[c] wherever a token's input is read: the
//   bias of the projection that made u, which the zeros before a request's start do not get)
//   S_t = exp(-exp(A_log) * dt_t) S_(t-1) + dt_t * B_t x_t^T,  y_t = S_t^T C_t + D x_t,
//   dt_t = softplus(dt_raw_t + dt_bias)
//
// Decays, step sizes, the state and the sums over it are float32 whatever the activations'
// type is.
#include "hal_common.h"
#include "hal_api.h"

#define CONV_MAX_TAPS 16

__device__ __forceinline__ float silu_f32(float x) { return x / (1.0f + expf(-x)); }

// ---- the convolution: a thread a (token, channel) ------------------------------------------
// state [slots][taps - 1][C]: the last taps - 1 inputs of the request before this step
template <typename TY>
__global__ void short_conv_kernel(const float* __restrict__ u, int ldu, const void* __restrict__ w,
                                  const void* __restrict__ bias, int w_dtype, const void* __restrict__ in_bias,
                                  int ib_dtype, int taps,
                                  const float* __restrict__ state, const int* __restrict__ token_seg,
                                  const int* __restrict__ seg_q_start, const int* __restrict__ token_slot,
                                  TY* __restrict__ y, int ldy, int act, int n_tokens, int C) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int t = blockIdx.x;
  if (c >= C) return;
  const int i = t - seg_q_start[token_seg[t]];  // the token's place in its segment
  const float* st = state + (size_t)token_slot[t] * (taps - 1) * C;
  float acc = bias ? load_as_f32(bias, w_dtype, c) : 0.f;
  const float ib = in_bias ? load_as_f32(in_bias, ib_dtype, c) : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int back = taps - 1 - j;  // how many tokens before t
    const float x = back <= i ? u[(size_t)(t - back) * ldu + c] + ib : st[(size_t)(taps - 1 - (back - i)) * C + c];
    acc = fmaf(load_as_f32(w, w_dtype, (size_t)c * taps + j), x, acc);
  }
  if (act == 1) acc = silu_f32(acc);
  y[(size_t)t * ldy + c] = from_f32<TY>(acc);
}

// A step in which every segment is one token (decoding): the convolution and the carry in
// one kernel; a thread owns its (request, channel) and moves the carried inputs one on.
template <typename TY>
__global__ void short_conv_step_kernel(const float* __restrict__ u, int ldu, const void* __restrict__ w,
                                       const void* __restrict__ bias, int w_dtype, const void* __restrict__ in_bias,
                                       int ib_dtype, int taps,
                                       float* __restrict__ state, const int* __restrict__ token_slot,
                                       TY* __restrict__ y, int ldy, int act, int C) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int t = blockIdx.x;
  if (c >= C) return;
  float* st = state + (size_t)token_slot[t] * (taps - 1) * C + c;
  const float x = u[(size_t)t * ldu + c] + (in_bias ? load_as_f32(in_bias, ib_dtype, c) : 0.f);
  float acc = bias ? load_as_f32(bias, w_dtype, c) : 0.f;
  float old[CONV_MAX_TAPS];
#pragma unroll
  for (int j = 0; j < CONV_MAX_TAPS - 1; ++j)
    if (j < taps - 1) old[j] = st[(size_t)j * C];
#pragma unroll
  for (int j = 0; j < CONV_MAX_TAPS - 1; ++j) {
    if (j < taps - 1) {
      acc = fmaf(load_as_f32(w, w_dtype, (size_t)c * taps + j), old[j], acc);
      st[(size_t)j * C] = j + 1 < taps - 1 ? old[j + 1] : x;
    }
  }
  acc = fmaf(load_as_f32(w, w_dtype, (size_t)c * taps + taps - 1), x, acc);
  if (act == 1) acc = silu_f32(acc);
  y[(size_t)t * ldy + c] = from_f32<TY>(acc);
}

extern "C" int hal_short_conv_step(const float* u, int ldu, const void* w, const void* bias, int w_dtype,
                                   const void* in_bias, int ib_dtype, int taps,
                                   float* state, const int* token_slot, void* y, int ldy, int y_dtype, int act,
                                   int n_tokens, int C, hipStream_t stream) {
  HAL_REQUIRE(n_tokens >= 0 && C > 0 && taps >= 1 && taps <= CONV_MAX_TAPS && ldu >= C && ldy >= C,
              "hal_short_conv_step: bad sizes T=%d C=%d taps=%d", n_tokens, C, taps);
  HAL_REQUIRE(y_dtype == HAL_F32 || y_dtype == HAL_BF16, "hal_short_conv_step: dtype %d", y_dtype);
  HAL_REQUIRE(act == 0 || act == 1, "hal_short_conv_step: activation %d", act);
  HAL_REQUIRE((C + 255) / 256 <= 65535, "hal_short_conv_step: %d channels exceed the grid limit", C);
  if (n_tokens == 0) return 0;
  dim3 grid(n_tokens, (C + 255) / 256);
  if (y_dtype == HAL_F32)
    hipLaunchKernelGGL(short_conv_step_kernel<float>, grid, dim3(256), 0, stream, u, ldu, w, bias, w_dtype, in_bias, ib_dtype,
                       taps, state, token_slot, (float*)y, ldy, act, C);
  else
    hipLaunchKernelGGL(short_conv_step_kernel<bf16_t>, grid, dim3(256), 0, stream, u, ldu, w, bias, w_dtype, in_bias, ib_dtype,
                       taps, state, token_slot, (bf16_t*)y, ldy, act, C);
  HAL_LAUNCH_CHECK();
  return 0;
}

extern "C" int hal_short_conv(const float* u, int ldu, const void* w, const void* bias, int w_dtype,
                              const void* in_bias, int ib_dtype, int taps,
                              const float* state, const int* token_seg, const int* seg_q_start,
                              const int* token_slot, void* y, int ldy, int y_dtype, int act, int n_tokens, int C,
                              hipStream_t stream) {
  HAL_REQUIRE(n_tokens >= 0 && C > 0 && taps >= 1 && taps <= CONV_MAX_TAPS && ldu >= C && ldy >= C,
              "hal_short_conv: bad sizes T=%d C=%d taps=%d", n_tokens, C, taps);
  HAL_REQUIRE(y_dtype == HAL_F32 || y_dtype == HAL_BF16, "hal_short_conv: dtype %d", y_dtype);
  HAL_REQUIRE(act == 0 || act == 1, "hal_short_conv: activation %d", act);
  HAL_REQUIRE((C + 255) / 256 <= 65535, "hal_short_conv: %d channels exceed the grid limit", C);
  if (n_tokens == 0) return 0;
  dim3 grid(n_tokens, (C + 255) / 256);
  if (y_dtype == HAL_F32)
    hipLaunchKernelGGL(short_conv_kernel<float>, grid, dim3(256), 0, stream, u, ldu, w, bias, w_dtype, in_bias, ib_dtype, taps,
                       state, token_seg, seg_q_start, token_slot, (float*)y, ldy, act, n_tokens, C);
  else
    hipLaunchKernelGGL(short_conv_kernel<bf16_t>, grid, dim3(256), 0, stream, u, ldu, w, bias, w_dtype, in_bias, ib_dtype, taps,
                       state, token_seg, seg_q_start, token_slot, (bf16_t*)y, ldy, act, n_tokens, C);
  HAL_LAUNCH_CHECK();
  return 0;
}

// ---- what the convolution carries to the next step: a thread a (segment, channel) ---------
__global__ void short_conv_carry_kernel(const float* __restrict__ u, int ldu, const void* __restrict__ in_bias,
                                        int ib_dtype, float* __restrict__ state, int taps,
                                        const int* __restrict__ seg_q_start, const int* __restrict__ seg_q_len,
                                        const int* __restrict__ token_slot, int C) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int s = blockIdx.y;
  if (c >= C) return;
  const int t0 = seg_q_start[s], n = seg_q_len[s];
  if (n <= 0) return;
  float* st = state + (size_t)token_slot[t0] * (taps - 1) * C;
  const float ib = in_bias ? load_as_f32(in_bias, ib_dtype, c) : 0.f;
  float keep[CONV_MAX_TAPS];
  // the last taps - 1 of (what was carried, then the step's inputs)
#pragma unroll
  for (int i = 0; i < CONV_MAX_TAPS - 1; ++i) {
    if (i < taps - 1) {
      const int at = n + i;  // place in the joined row, whose first taps - 1 are the old ones
      keep[i] = at < taps - 1 ? st[(size_t)at * C + c] : u[(size_t)(t0 + at - (taps - 1)) * ldu + c] + ib;
    }
  }
#pragma unroll
  for (int i = 0; i < CONV_MAX_TAPS - 1; ++i)
    if (i < taps - 1) st[(size_t)i * C + c] = keep[i];
}

extern "C" int hal_short_conv_carry(const float* u, int ldu, const void* in_bias, int ib_dtype, float* state, int taps,
                                    const int* seg_q_start,
                                    const int* seg_q_len, const int* token_slot, int n_segs, int C,
                                    hipStream_t stream) {
  HAL_REQUIRE(n_segs >= 0 && n_segs <= 65535 && C > 0 && taps >= 1 && taps <= CONV_MAX_TAPS && ldu >= C,
              "hal_short_conv_carry: bad sizes segments=%d C=%d taps=%d", n_segs, C, taps);
  if (n_segs == 0 || taps == 1) return 0;
  hipLaunchKernelGGL(short_conv_carry_kernel, dim3((C + 255) / 256, n_segs), dim3(256), 0, stream, u, ldu, in_bias,
                     ib_dtype, state, taps, seg_q_start, seg_q_len, token_slot, C);
  HAL_LAUNCH_CHECK();
  return 0;
}

// ---- the recurrence: a wave takes 64 value channels of one head of one run of tokens and
// walks them; a lane holds its channel's column of the state (N numbers) in registers, so the
// sums over the state need no exchange between lanes.  A token's B and C (shared by the
// lanes) go through LDS, the next token's on their way meanwhile.
//
// MODE 0: a run is a segment; the state comes from the request's row and goes back there.
// Long segments are cut into chunks (`chunks` [n][4]: first token, tokens, segment, unused),
// so that the chip has a wave for every chunk and not for every request:
// MODE 1: a run is a chunk, walked from a zero state; what it leaves (sums [chunk][head][N][P])
//   and the product of its decays ([chunk][head]) are written, no output;
// then a wave per (segment, head, 64 channels) takes the request's state through the
//   segment's chunks in order, S <- decay_c S + sums_c, leaving in sums_c the state that
//   chunk c starts from, and writes the last state to the request's row;
// MODE 2: a run is a chunk again, walked from the state it starts from, for the outputs.
// The result is the recurrence's own, token by token; only the order of additions differs.
//
// `fixed_decay` (or null): float32 [heads], one constant decay a head; then every step size is 1,
// nothing is added for the token itself, and dt_raw, dt_bias, a_log and d_skip are not read:
// S <- decay_h S + B x^T, y = S^T C (a linear attention with keys B, queries C, values x).
// `in_silu`: x, B and C are what SiLU makes of the numbers in `xbc` (the activation of the
// projections that made them, applied as they are read). ----
template <typename T, int NREG, int MODE>
__global__ void __launch_bounds__(HAL_WAVE)
ssd_scan_kernel(const T* __restrict__ xbc, int ldx, const float* __restrict__ dt_raw, int ld_dt,
                const void* __restrict__ dt_bias, const void* __restrict__ a_log, const void* __restrict__ d_skip,
                int w_dtype, float* __restrict__ state, const int* __restrict__ seg_q_start,
                const int* __restrict__ seg_q_len, const int* __restrict__ token_slot, float* __restrict__ y,
                const int* __restrict__ chunks, float* __restrict__ sums, float* __restrict__ decays,
                int heads, int P, int N, int groups, const float* __restrict__ fixed_decay, bool in_silu) {
  __shared__ __align__(16) float bc[2][2 * NREG];
  const int s = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int p = blockIdx.z * HAL_WAVE + lane;
  const int t0 = MODE == 0 ? seg_q_start[s] : chunks[s * 4], n = MODE == 0 ? seg_q_len[s] : chunks[s * 4 + 1];
  if (n <= 0) return;
  const int inner = heads * P;
  const int g = h / (heads / groups);
  const bool live = p < P;
  float* st = MODE == 0 ? state + (((size_t)token_slot[t0] * heads + h) * N) * P + (live ? p : 0)
                        : sums + (((size_t)s * heads + h) * N) * P + (live ? p : 0);
  float S[NREG];
#pragma unroll
  for (int i = 0; i < NREG; ++i) S[i] = (MODE != 1 && live && i < N) ? st[(size_t)i * P] : 0.f;
  const bool fixed = fixed_decay != nullptr;
  const float rate = fixed ? 0.f : expf(load_as_f32(a_log, w_dtype, h));
  const float bias = fixed ? 0.f : load_as_f32(dt_bias, w_dtype, h);
  const float skip = fixed ? 0.f : load_as_f32(d_skip, w_dtype, h);
  const float decay_h = fixed ? fixed_decay[h] : 0.f;
  const size_t b_col = (size_t)inner + (size_t)g * N, c_col = (size_t)inner + (size_t)groups * N + (size_t)g * N;

  // a lane brings B[lane], B[lane + 64], .. and the same of C
  constexpr int PER = (NREG + HAL_WAVE - 1) / HAL_WAVE;
  float nb[PER], nc[PER];
  auto in = [&](size_t at) {
    const float v = to_f32(xbc[at]);
    return in_silu ? silu_f32(v) : v;
  };
  auto ask = [&](int t) {
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int i = lane + u * HAL_WAVE;
      nb[u] = i < N ? in((size_t)t * ldx + b_col + i) : 0.f;
      if (MODE != 1) nc[u] = i < N ? in((size_t)t * ldx + c_col + i) : 0.f;
    }
  };
  auto put = [&](int buf) {
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int i = lane + u * HAL_WAVE;
      if (i < NREG) {
        bc[buf][i] = nb[u];
        if (MODE != 1) bc[buf][NREG + i] = nc[u];
      }
    }
  };
  ask(t0);
  float x_next = live ? in((size_t)t0 * ldx + (size_t)h * P + p) : 0.f;
  float dt_next = fixed ? 0.f : dt_raw[(size_t)t0 * ld_dt + h];
  float decay_all = 1.f;
  for (int i = 0; i < n; ++i) {
    const int t = t0 + i, buf = i & 1;
    put(buf);
    const float x = x_next, raw = dt_next + bias;
    if (i + 1 < n) {
      ask(t + 1);
      x_next = live ? in((size_t)(t + 1) * ldx + (size_t)h * P + p) : 0.f;
      if (!fixed) dt_next = dt_raw[(size_t)(t + 1) * ld_dt + h];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const float dt = fixed ? 1.0f : (raw > 20.f ? raw : log1pf(expf(raw)));
    const float decay = fixed ? decay_h : expf(-rate * dt);
    const float dtx = dt * x;
    if (MODE == 1) {
      decay_all *= decay;
#pragma unroll
      for (int k = 0; k < NREG; k += 4) {
        const float4 b4 = *(const float4*)&bc[buf][k];
        S[k] = fmaf(decay, S[k], dtx * b4.x);
        S[k + 1] = fmaf(decay, S[k + 1], dtx * b4.y);
        S[k + 2] = fmaf(decay, S[k + 2], dtx * b4.z);
        S[k + 3] = fmaf(decay, S[k + 3], dtx * b4.w);
      }
    } else {
      float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
      for (int k = 0; k < NREG; k += 4) {
        const float4 b4 = *(const float4*)&bc[buf][k];
        const float4 c4 = *(const float4*)&bc[buf][NREG + k];
        S[k] = fmaf(decay, S[k], dtx * b4.x);
        acc0 = fmaf(S[k], c4.x, acc0);
        S[k + 1] = fmaf(decay, S[k + 1], dtx * b4.y);
        acc1 = fmaf(S[k + 1], c4.y, acc1);
        S[k + 2] = fmaf(decay, S[k + 2], dtx * b4.z);
        acc0 = fmaf(S[k + 2], c4.z, acc0);
        S[k + 3] = fmaf(decay, S[k + 3], dtx * b4.w);
        acc1 = fmaf(S[k + 3], c4.w, acc1);
      }
      if (live) y[(size_t)t * inner + (size_t)h * P + p] = (acc0 + acc1) + skip * x;
    }
  }
  if (MODE != 2 && live) {
#pragma unroll
    for (int i = 0; i < NREG; ++i)
      if (i < N) st[(size_t)i * P] = S[i];
  }
  if (MODE == 1 && blockIdx.z == 0 && lane == 0) decays[(size_t)s * heads + h] = decay_all;
}

// seg_chunks [segments][2]: a segment's first chunk and number of chunks.  A thread takes one
// number of the state of one head of one segment through the segment's chunks; the chunks'
// sums are asked for four at a time (the sums wait for each other, the loads need not).
__global__ void __launch_bounds__(256)
ssd_carry_kernel(float* __restrict__ state, float* __restrict__ sums, const float* __restrict__ decays,
                 const int* __restrict__ seg_chunks, const int* __restrict__ seg_q_start,
                 const int* __restrict__ seg_q_len, const int* __restrict__ token_slot, int heads, int NP) {
  const int s = blockIdx.x, h = blockIdx.y, e = blockIdx.z * blockDim.x + threadIdx.x;
  if (seg_q_len[s] <= 0 || e >= NP) return;
  const int c0 = seg_chunks[s * 2], nc = seg_chunks[s * 2 + 1];
  float* st = state + ((size_t)token_slot[seg_q_start[s]] * heads + h) * NP + e;
  float S = *st;
  constexpr int AHEAD = 4;
  for (int c = c0; c < c0 + nc; c += AHEAD) {
    float left[AHEAD], decay[AHEAD];
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) {
      const int cu = c + u < c0 + nc ? c + u : c0 + nc - 1;
      left[u] = sums[((size_t)cu * heads + h) * NP + e];
      decay[u] = decays[(size_t)cu * heads + h];
    }
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) {
      if (c + u < c0 + nc) {
        sums[((size_t)(c + u) * heads + h) * NP + e] = S;
        S = fmaf(decay[u], S, left[u]);
      }
    }
  }
  *st = S;
}

// chunks, seg_chunks, sums, decays: all null (a wave walks a whole segment), or the cut of the
// segments into n_chunks chunks and room for n_chunks * heads * N * P and n_chunks * heads floats.
extern "C" int hal_ssd_scan(const void* xbc, int ldx, int dtype, const float* dt_raw, int ld_dt,
                            const void* dt_bias, const void* a_log, const void* d_skip, int w_dtype, float* state,
                            const int* seg_q_start, const int* seg_q_len, const int* token_slot, float* y,
                            int n_segs, int heads, int P, int N, int groups, const int* chunks,
                            const int* seg_chunks, int n_chunks, float* sums, float* decays,
                            const float* fixed_decay, int in_silu, hipStream_t stream) {
  HAL_REQUIRE(n_segs >= 0 && heads > 0 && P > 0 && N > 0 && groups > 0 && heads % groups == 0,
              "hal_ssd_scan: bad sizes segments=%d heads=%d P=%d N=%d groups=%d", n_segs, heads, P, N, groups);
  HAL_REQUIRE(N <= 256, "hal_ssd_scan: a state of %d numbers a channel exceeds 256", N);
  HAL_REQUIRE(ldx >= heads * P + 2 * groups * N && (fixed_decay || ld_dt >= heads), "hal_ssd_scan: rows too short");
  HAL_REQUIRE(fixed_decay || (dt_raw && dt_bias && a_log && d_skip), "hal_ssd_scan: neither step sizes nor fixed decays");
  HAL_REQUIRE(heads <= 65535 && (P + HAL_WAVE - 1) / HAL_WAVE <= 65535, "hal_ssd_scan: grid limit");
  HAL_REQUIRE(dtype == HAL_F32 || dtype == HAL_BF16, "hal_ssd_scan: dtype %d", dtype);
  const bool cut = chunks != nullptr;
  HAL_REQUIRE(!cut || (seg_chunks && sums && decays && n_chunks >= 0), "hal_ssd_scan: chunks without their buffers");
  if (n_segs == 0) return 0;
  const dim3 block(HAL_WAVE);
  HAL_REQUIRE(((long long)N * P + 255) / 256 <= 65535, "hal_ssd_scan: a state of %d x %d exceeds the grid limit", N, P);
  const dim3 carry_grid(n_segs, heads, (N * P + 255) / 256);
  const dim3 seg_grid(n_segs, heads, (P + HAL_WAVE - 1) / HAL_WAVE), chunk_grid(cut ? n_chunks : 1, heads, (P + HAL_WAVE - 1) / HAL_WAVE);
#define SCAN_LAUNCH(T_, N_, MODE_, GRID_)                                                                      \
  hipLaunchKernelGGL((ssd_scan_kernel<T_, N_, MODE_>), GRID_, block, 0, stream, (const T_*)xbc, ldx, dt_raw,    \
                     ld_dt, dt_bias, a_log, d_skip, w_dtype, state, seg_q_start, seg_q_len, token_slot, y,     \
                     chunks, sums, decays, heads, P, N, groups, fixed_decay, in_silu != 0)
#define SCAN_STEPS(T_, N_)                                                                                    \
  do {                                                                                                        \
    if (!cut) {                                                                                               \
      SCAN_LAUNCH(T_, N_, 0, seg_grid);                                                                       \
    } else if (n_chunks > 0) {                                                                                \
      SCAN_LAUNCH(T_, N_, 1, chunk_grid);                                                                     \
      hipLaunchKernelGGL(ssd_carry_kernel, carry_grid, dim3(256), 0, stream, state, sums, decays, seg_chunks, \
                         seg_q_start, seg_q_len, token_slot, heads, N * P);                                   \
      SCAN_LAUNCH(T_, N_, 2, chunk_grid);                                                                     \
    }                                                                                                         \
  } while (0)
#define SCAN_BY_STATE(T_)                  \
  do {                                     \
    if (N <= 16) SCAN_STEPS(T_, 16);       \
    else if (N <= 32) SCAN_STEPS(T_, 32);  \
    else if (N <= 64) SCAN_STEPS(T_, 64);  \
    else if (N <= 128) SCAN_STEPS(T_, 128); \
    else SCAN_STEPS(T_, 256);              \
  } while (0)
  if (dtype == HAL_F32)
    SCAN_BY_STATE(float);
  else
    SCAN_BY_STATE(bf16_t);
#undef SCAN_BY_STATE
#undef SCAN_STEPS
#undef SCAN_LAUNCH
  HAL_LAUNCH_CHECK();
  return 0;
}

// ---- out = norm_g(y * silu(z)) * w: the gate first, then every one of `parts` equal parts of
// the row divided by its own root mean square; a workgroup a (token, part) -----------------
template <typename T>
__global__ void gated_part_norm_kernel(const float* __restrict__ y, const float* __restrict__ z, int ldz,
                                       const void* __restrict__ w, int w_dtype, float eps, T* __restrict__ out,
                                       int inner, int parts) {
  __shared__ float scratch[16];
  const size_t t = blockIdx.x;
  const int part = blockIdx.y, n = inner / parts, c0 = part * n;
  const float* yr = y + t * inner + c0;
  const float* zr = z + t * ldz + c0;
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float v = yr[i] * silu_f32(zr[i]);
    ss += v * v;
  }
  const float total = block_sum(ss, scratch);
  const float rstd = 1.0f / sqrtf(total / (float)n + eps);
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float v = yr[i] * silu_f32(zr[i]);
    out[t * inner + c0 + i] = from_f32<T>(v * rstd * load_as_f32(w, w_dtype, c0 + i));
  }
}

extern "C" int hal_gated_part_norm(const float* y, const float* z, int ldz, const void* w, int w_dtype, float eps,
                                   void* out, int dtype, int n_tokens, int inner, int parts, hipStream_t stream) {
  HAL_REQUIRE(n_tokens >= 0 && inner > 0 && parts > 0 && inner % parts == 0 && parts <= 65535 && ldz >= inner,
              "hal_gated_part_norm: bad sizes T=%d inner=%d parts=%d", n_tokens, inner, parts);
  HAL_REQUIRE(dtype == HAL_F32 || dtype == HAL_BF16, "hal_gated_part_norm: dtype %d", dtype);
  if (n_tokens == 0) return 0;
  const int n = inner / parts;
  const int threads = n >= 1024 ? 256 : (n >= 256 ? 128 : 64);
  if (dtype == HAL_F32)
    hipLaunchKernelGGL(gated_part_norm_kernel<float>, dim3(n_tokens, parts), dim3(threads), 0, stream, y, z, ldz, w,
                       w_dtype, eps, (float*)out, inner, parts);
  else
    hipLaunchKernelGGL(gated_part_norm_kernel<bf16_t>, dim3(n_tokens, parts), dim3(threads), 0, stream, y, z, ldz, w,
                       w_dtype, eps, (bf16_t*)out, inner, parts);
  HAL_LAUNCH_CHECK();
  return 0;
}
