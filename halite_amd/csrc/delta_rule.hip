// The generalized delta rule: per head a float32 state S [key channel][value channel] that
// every token decays per key channel, erases along its unit key and writes to,
//
//   S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T,   o_t = S_t^T r_t,
//   w = exp(-e^(-1/2) sigmoid(w0 + W2 tanh(x1))),  a = sigmoid(a_raw + a_bias),
//   u = k / sqrt(sum(k^2) + 1e-6)   (per head),
//
// where both middle terms read the old state.  The state lives in float32 rows, one per
// request slot, and a step's tokens come as a flat batch of segments, as for the other
// recurrences.  Three kernels: what a token contributes (decay, erase vector, unit key; all
// tokens side by side), the walk over the tokens of every segment (or, where every segment
// is one token, a kernel that reads and writes each state once in whole rows), and the norm
// and gate of the walk's result.  Everything here is float32 whatever the activations' type is.
#include "hal_common.h"
#include "hal_api.h"

#define DELTA_MAX_LORA 1024
#define DELTA_WAVES_FOR_WIDE 4096  // four waves a SIMD of 256 compute units
#define DELTA_VECTORS 5  // per token and head: decay, a * u, u, k, r

__device__ __forceinline__ float delta_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }

// sum_j row[j] * x[j] for j < n; `vec`: the row begins at a multiple of four elements
template <typename W>
__device__ __forceinline__ float delta_row_dot(const W* __restrict__ row, const float* x, int n, bool vec) {
  float z0 = 0.f, z1 = 0.f;
  int j = 0;
  if (vec) {
#pragma unroll 4
    for (; j + 4 <= n; j += 4) {
      float w[4];
      load4(row + j, w);
      z0 = fmaf(w[0], x[j], z0);
      z1 = fmaf(w[1], x[j + 1], z1);
      z0 = fmaf(w[2], x[j + 2], z0);
      z1 = fmaf(w[3], x[j + 3], z1);
    }
  }
  for (; j < n; ++j) z0 = fmaf(to_f32(row[j]), x[j], z0);
  return z0 + z1;
}

// ---- a workgroup takes DELTA_PREP_TOKENS tokens of one head; thread c a key channel, whose
// row of W2 it holds in registers (DELTA_PREP_RANK entries at a time) for all the tokens.
// pre [T][H][5][DP], zero beyond D.
#define DELTA_PREP_RANK 32
template <int DELTA_PREP_TOKENS, typename W>
__global__ void delta_prep_kernel(const float* __restrict__ r, int ldr, const float* __restrict__ k, int ldk,
                                  const float* __restrict__ a_raw, int lda, const float* __restrict__ x1, int ldx1,
                                  const W* __restrict__ w2, const W* __restrict__ w0,
                                  const W* __restrict__ a_bias, int lora, float decay_rate,
                                  float unit_eps, float* __restrict__ pre, int n_tokens, int H, int D, int DP) {
  __shared__ float scratch[16];
  __shared__ float tl[DELTA_PREP_TOKENS][DELTA_PREP_RANK];
  const int t0 = blockIdx.x * DELTA_PREP_TOKENS;
  const int nt = n_tokens - t0 < DELTA_PREP_TOKENS ? n_tokens - t0 : DELTA_PREP_TOKENS;
  const int h = blockIdx.y, c = threadIdx.x;
  const bool live = c < D;
  const size_t ch = (size_t)h * D + (live ? c : 0);
  float z[DELTA_PREP_TOKENS];
  const float z0 = to_f32(w0[ch]);
  const bool vec = lora % 4 == 0;
#pragma unroll
  for (int i = 0; i < DELTA_PREP_TOKENS; ++i) z[i] = z0;
  for (int j0 = 0; j0 < lora; j0 += DELTA_PREP_RANK) {
    const int nj = lora - j0 < DELTA_PREP_RANK ? lora - j0 : DELTA_PREP_RANK;
    __syncthreads();
    for (int i = threadIdx.x; i < DELTA_PREP_TOKENS * DELTA_PREP_RANK; i += blockDim.x) {
      const int tok = i / DELTA_PREP_RANK, j = i % DELTA_PREP_RANK;
      tl[tok][j] = (tok < nt && j < nj) ? tanhf(x1[(size_t)(t0 + tok) * ldx1 + j0 + j]) : 0.f;
    }
    float w[DELTA_PREP_RANK];
    const W* row = w2 + ch * lora + j0;
    if (vec && nj == DELTA_PREP_RANK) {
#pragma unroll
      for (int j = 0; j < DELTA_PREP_RANK; j += 4) {
        float q[4];
        load4(row + j, q);
        w[j] = q[0], w[j + 1] = q[1], w[j + 2] = q[2], w[j + 3] = q[3];
      }
    } else {
#pragma unroll
      for (int j = 0; j < DELTA_PREP_RANK; ++j) w[j] = j < nj ? to_f32(row[j]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < DELTA_PREP_TOKENS; ++i) {
#pragma unroll
      for (int j = 0; j < DELTA_PREP_RANK; j += 4) {
        const float4 x4 = *(const float4*)&tl[i][j];
        z[i] = fmaf(w[j], x4.x, z[i]);
        z[i] = fmaf(w[j + 1], x4.y, z[i]);
        z[i] = fmaf(w[j + 2], x4.z, z[i]);
        z[i] = fmaf(w[j + 3], x4.w, z[i]);
      }
    }
  }
  const float ab = to_f32(a_bias[ch]);
  float kc_[DELTA_PREP_TOKENS], ar_[DELTA_PREP_TOKENS], rc_[DELTA_PREP_TOKENS];
#pragma unroll
  for (int i = 0; i < DELTA_PREP_TOKENS; ++i) {  // all of a thread's loads on their way at once
    const bool have = live && i < nt;
    const size_t t = t0 + i;
    kc_[i] = have ? k[t * ldk + ch] : 0.f;
    ar_[i] = have ? a_raw[t * lda + ch] : 0.f;
    rc_[i] = have ? r[t * ldr + ch] : 0.f;
  }
#pragma unroll
  for (int i = 0; i < DELTA_PREP_TOKENS; ++i) {
    if (i >= nt) break;  // (the same for every thread of the workgroup)
    const size_t t = t0 + i;
    const float kc = kc_[i];
    const float kk = block_sum(kc * kc, scratch);
    if (c >= DP) continue;
    float* dst = pre + ((t * H + h) * DELTA_VECTORS) * DP + c;
    float decay = 0.f, au = 0.f, u = 0.f, rc = 0.f;
    if (live) {
      decay = expf(-decay_rate * delta_sigmoid(z[i]));
      u = kc / sqrtf(kk + unit_eps);
      au = delta_sigmoid(ar_[i] + ab) * u;
      rc = rc_[i];
    }
    dst[0] = decay;
    dst[DP] = au;
    dst[2 * DP] = u;
    dst[3 * DP] = kc;
    dst[4 * DP] = rc;
  }
}

// The sum of a value over the wave's four quarters of 16 lanes, in every lane: two swaps of
// lane halves inside the vector unit (rows 1 and 3 against rows 0 and 2, then the upper 32
// lanes against the lower), each followed by an addition.
__device__ __forceinline__ float quarters_sum(float x) {
  const unsigned b = __float_as_uint(x);
  const auto p = __builtin_amdgcn_permlane16_swap(b, b, false, false);
  const unsigned s = __float_as_uint(__uint_as_float(p[0]) + __uint_as_float(p[1]));
  const auto q = __builtin_amdgcn_permlane32_swap(s, s, false, false);
  return __uint_as_float(q[0]) + __uint_as_float(q[1]);
}

// ---- the walk: a wave takes COLS (16 or 8) value channels of one head of one segment; the
// key channels are split over the wave's 64 / COLS groups of lanes, so a lane holds NREG
// numbers of its channel's column of the state, and the two sums over the key channels
// (u^T S and S^T r) cross the groups inside the vector unit.  The tokens' five vectors
// (shared by the lanes) go through LDS in blocks of TB tokens, the next block's on their way
// from memory while one is walked, so that the memory's latency is paid once a block and not
// once a token; a whole block is walked without a branch between its tokens, each token's
// rows read from LDS while the token before is worked on.
template <int COLS>
__device__ __forceinline__ float groups_sum(float x) {
  if (COLS == 8)  // lanes i and i ^ 8: a rotation by 8 inside every row of 16 lanes
    x += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(x), 0x128, 0xf, 0xf, false));
  return quarters_sum(x);
}

template <int NREG, int COLS>
__global__ void __launch_bounds__(HAL_WAVE)
delta_scan_kernel(const float* __restrict__ pre, const float* __restrict__ v, int ldv, float* __restrict__ state,
                  const int* __restrict__ seg_q_start, const int* __restrict__ seg_q_len,
                  const int* __restrict__ token_slot, float* __restrict__ o, int H, int D) {
  constexpr int DP = NREG * (HAL_WAVE / COLS), TOTAL = DELTA_VECTORS * DP;
  constexpr int TB = DP <= 64 ? 8 : DP == 128 ? 4 : 2;
  constexpr int PER = TB * TOTAL / HAL_WAVE;
  static_assert(TB * TOTAL % HAL_WAVE == 0 && NREG % 4 == 0, "a block of tokens is whole loads of the wave");
  __shared__ __align__(16) float vec[2 * TB * TOTAL];
  const int s = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int col = blockIdx.z * COLS + lane % COLS, row0 = (lane / COLS) * NREG;
  const int t0 = seg_q_start[s], n = seg_q_len[s];
  if (n <= 0) return;
  const bool live = col < D;
  float* st = state + ((size_t)token_slot[t0] * H + h) * D * D + (live ? col : 0);
  float S[NREG];
#pragma unroll
  for (int i = 0; i < NREG; ++i) S[i] = (live && row0 + i < D) ? st[(size_t)(row0 + i) * D] : 0.f;

  float next[PER], v_next[TB];
  // where this lane's loads of a block lie from the block's first token on (in floats)
  int at_pre[PER], tok_pre[PER];
#pragma unroll
  for (int u = 0; u < PER; ++u) {
    const int i = lane + u * HAL_WAVE;
    tok_pre[u] = i / TOTAL;
    at_pre[u] = tok_pre[u] * (H * TOTAL - TOTAL) + i;  // token tok_pre[u], entry i - tok_pre[u] * TOTAL
  }
  const float* vp = v + (size_t)h * D + (live ? col : 0);
  auto ask = [&](int t, int cnt) {  // tokens t .. t + cnt - 1
    const float* src = pre + ((size_t)t * H + h) * TOTAL;
    const float* vs = vp + (size_t)t * ldv;
    if (cnt == TB) {
#pragma unroll
      for (int u = 0; u < PER; ++u) next[u] = src[at_pre[u]];
#pragma unroll
      for (int j = 0; j < TB; ++j) v_next[j] = live ? vs[(size_t)j * ldv] : 0.f;
    } else {
#pragma unroll
      for (int u = 0; u < PER; ++u) next[u] = tok_pre[u] < cnt ? src[at_pre[u]] : 0.f;
#pragma unroll
      for (int j = 0; j < TB; ++j) v_next[j] = (live && j < cnt) ? vs[(size_t)j * ldv] : 0.f;
    }
  };
  // a token's vectors for this lane's rows, read from LDS a token ahead of their use
  struct Rows { float4 w[NREG / 4], e[NREG / 4], u[NREG / 4], k[NREG / 4], r[NREG / 4]; };
  auto fetch = [&](Rows& x, int at) {  // at: where the token's vectors begin in vec
#pragma unroll
    for (int j = 0; j < NREG / 4; ++j) {
      x.u[j] = *(const float4*)(vec + at + 2 * DP + 4 * j);
      x.w[j] = *(const float4*)(vec + at + 4 * j);
      x.e[j] = *(const float4*)(vec + at + DP + 4 * j);
      x.k[j] = *(const float4*)(vec + at + 3 * DP + 4 * j);
      x.r[j] = *(const float4*)(vec + at + 4 * DP + 4 * j);
    }
  };
  const bool writer = live && lane < COLS;
  const size_t o_step = (size_t)H * D;
  float* op = o + (size_t)t0 * o_step + (size_t)h * D + (live ? col : 0);
  auto token = [&](const Rows& x, float val) {
    float d0 = 0.f, d1 = 0.f;
#pragma unroll
    for (int j = 0; j < NREG / 4; ++j) {
      d0 = fmaf(S[4 * j], x.u[j].x, d0);
      d1 = fmaf(S[4 * j + 1], x.u[j].y, d1);
      d0 = fmaf(S[4 * j + 2], x.u[j].z, d0);
      d1 = fmaf(S[4 * j + 3], x.u[j].w, d1);
    }
    const float dot = groups_sum<COLS>(d0 + d1);  // u^T S_(t-1) of this column
    float a0 = 0.f, a1 = 0.f;
#pragma unroll
    for (int j = 0; j < NREG / 4; ++j) {
      S[4 * j] = fmaf(x.w[j].x, S[4 * j], fmaf(-x.e[j].x, dot, x.k[j].x * val));
      a0 = fmaf(S[4 * j], x.r[j].x, a0);
      S[4 * j + 1] = fmaf(x.w[j].y, S[4 * j + 1], fmaf(-x.e[j].y, dot, x.k[j].y * val));
      a1 = fmaf(S[4 * j + 1], x.r[j].y, a1);
      S[4 * j + 2] = fmaf(x.w[j].z, S[4 * j + 2], fmaf(-x.e[j].z, dot, x.k[j].z * val));
      a0 = fmaf(S[4 * j + 2], x.r[j].z, a0);
      S[4 * j + 3] = fmaf(x.w[j].w, S[4 * j + 3], fmaf(-x.e[j].w, dot, x.k[j].w * val));
      a1 = fmaf(S[4 * j + 3], x.r[j].w, a1);
    }
    const float acc = groups_sum<COLS>(a0 + a1);
    if (writer) *op = acc;
    op += o_step;
  };
  ask(t0, n < TB ? n : TB);
  for (int b = 0; b * TB < n; ++b) {
    const int base = t0 + b * TB, left = n - b * TB;
    const int blk = (b & 1) * TB * TOTAL;
#pragma unroll
    for (int u = 0; u < PER; ++u) vec[blk + lane + u * HAL_WAVE] = next[u];
    float vv[TB];
#pragma unroll
    for (int j = 0; j < TB; ++j) vv[j] = v_next[j];
    if (left > TB) ask(base + TB, left - TB < TB ? left - TB : TB);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (left >= TB) {
      Rows even, odd;  // (TB is even)
      fetch(even, blk + row0);
#pragma unroll
      for (int jt = 0; jt < TB; jt += 2) {
        fetch(odd, blk + (jt + 1) * TOTAL + row0);
        token(even, vv[jt]);
        if (jt + 2 < TB) fetch(even, blk + (jt + 2) * TOTAL + row0);
        token(odd, vv[jt + 1]);
      }
    } else {
#pragma unroll
      for (int jt = 0; jt < TB; ++jt)
        if (jt < left) {
          Rows cur;
          fetch(cur, blk + jt * TOTAL + row0);
          token(cur, vv[jt]);
        }
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < NREG; ++i)
      if (row0 + i < D) st[(size_t)(row0 + i) * D] = S[i];
  }
}

// ---- a step in which every request brings one token: a workgroup of 256 threads takes one
// head of one request.  It reads the state once in rows of 16 bytes a thread (a wave covers
// whole rows), makes the token's five vectors itself while those loads are on their way
// (thread c < D a key channel), and the two sums over the key channels cross the waves
// through LDS.  D is 32, 64 or 128; a thread holds R rows of four neighbouring value channels.
template <int D, typename W>
__global__ void __launch_bounds__(256)
delta_step_kernel(const float* __restrict__ r, int ldr, const float* __restrict__ k, int ldk,
                  const float* __restrict__ v, int ldv, const float* __restrict__ a_raw, int lda,
                  const float* __restrict__ x1, int ldx1, const W* __restrict__ w2, const W* __restrict__ w0,
                  const W* __restrict__ a_bias, int lora, float decay_rate, float unit_eps,
                  float* __restrict__ state, const int* __restrict__ token_slot, float* __restrict__ o, int H) {
  constexpr int CG = D / 4, RG = 256 / CG, R = D / RG, WAVES = 256 / HAL_WAVE, PARTS = 256 / D;
  static_assert(CG <= HAL_WAVE && 256 % CG == 0 && D % RG == 0, "a head of 32, 64 or 128 channels");
  __shared__ __align__(16) float vec[DELTA_VECTORS * D];
  __shared__ float tl[DELTA_MAX_LORA];
  __shared__ float zpart[PARTS][D];
  __shared__ float ksum[WAVES];
  __shared__ float4 red[2][WAVES][CG];
  const size_t t = blockIdx.x;
  const int h = blockIdx.y, tid = threadIdx.x;
  const int cg = tid % CG, rg = tid / CG, col = cg * 4, wave = tid / HAL_WAVE;
  float* st = state + ((size_t)token_slot[t] * H + h) * D * D + col;
  float4 S[R];
#pragma unroll
  for (int j = 0; j < R; ++j) S[j] = *(const float4*)(st + (size_t)(rg + j * RG) * D);
  const float* vr = v + t * ldv + (size_t)h * D + col;
  const float4 vv = make_float4(vr[0], vr[1], vr[2], vr[3]);
  // the token's vectors
  const bool channel = tid < D;
  const size_t ch = (size_t)h * D + (channel ? tid : 0);
  const float kc = channel ? k[t * ldk + ch] : 0.f;
  const float ar = channel ? a_raw[t * lda + ch] : 0.f;
  const float rc = channel ? r[t * ldr + ch] : 0.f;
  for (int j = tid; j < lora; j += 256) tl[j] = tanhf(x1[t * ldx1 + j]);
  const float part = wave_sum(kc * kc);
  if (tid % HAL_WAVE == 0) ksum[wave] = part;
  __syncthreads();
  {  // the decay's sum over the rank, a part of it a thread: thread = (part, channel)
    const int c = tid % D, part = tid / D;
    const int per = ((lora + PARTS - 1) / PARTS + 3) & ~3, j0 = part * per;
    const int n = lora - j0 < per ? lora - j0 : per;
    zpart[part][c] = n > 0 ? delta_row_dot(w2 + ((size_t)h * D + c) * lora + j0, tl + j0, n, lora % 4 == 0) : 0.f;
  }
  __syncthreads();
  if (channel) {
    float kk = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) kk += ksum[w];
    float z = to_f32(w0[ch]);
#pragma unroll
    for (int q = 0; q < PARTS; ++q) z += zpart[q][tid];
    const float u = kc / sqrtf(kk + unit_eps);
    vec[tid] = expf(-decay_rate * delta_sigmoid(z));
    vec[D + tid] = delta_sigmoid(ar + to_f32(a_bias[ch])) * u;
    vec[2 * D + tid] = u;
    vec[3 * D + tid] = kc;
    vec[4 * D + tid] = rc;
  }
  __syncthreads();
  auto across = [&](float4 x, int which) {  // the sum over all row groups, in every thread
#pragma unroll
    for (int m = CG; m < HAL_WAVE; m <<= 1) {
      x.x += __shfl_xor(x.x, m, HAL_WAVE);
      x.y += __shfl_xor(x.y, m, HAL_WAVE);
      x.z += __shfl_xor(x.z, m, HAL_WAVE);
      x.w += __shfl_xor(x.w, m, HAL_WAVE);
    }
    if (tid % HAL_WAVE < CG) red[which][wave][cg] = x;
    __syncthreads();
    float4 sum = red[which][0][cg];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) {
      const float4 y = red[which][w][cg];
      sum.x += y.x, sum.y += y.y, sum.z += y.z, sum.w += y.w;
    }
    return sum;
  };
  float4 d = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const float u = vec[2 * D + rg + j * RG];
    d.x = fmaf(S[j].x, u, d.x), d.y = fmaf(S[j].y, u, d.y), d.z = fmaf(S[j].z, u, d.z), d.w = fmaf(S[j].w, u, d.w);
  }
  const float4 dot = across(d, 0);
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const int row = rg + j * RG;
    const float w = vec[row], e = vec[D + row], kr = vec[3 * D + row], rr = vec[4 * D + row];
    S[j].x = fmaf(w, S[j].x, fmaf(-e, dot.x, kr * vv.x));
    S[j].y = fmaf(w, S[j].y, fmaf(-e, dot.y, kr * vv.y));
    S[j].z = fmaf(w, S[j].z, fmaf(-e, dot.z, kr * vv.z));
    S[j].w = fmaf(w, S[j].w, fmaf(-e, dot.w, kr * vv.w));
    acc.x = fmaf(S[j].x, rr, acc.x), acc.y = fmaf(S[j].y, rr, acc.y), acc.z = fmaf(S[j].z, rr, acc.z), acc.w = fmaf(S[j].w, rr, acc.w);
    *(float4*)(st + (size_t)row * D) = S[j];
  }
  const float4 out = across(acc, 1);
  if (tid < CG) *(float4*)(o + t * H * D + (size_t)h * D + col) = out;
}

// r, k, v, a_raw: float32 [T, H * D] (row-strided views allowed), x1 float32 [T, lora];
// w2 [H * D, lora], w0 and a_bias [H * D] of one element type; state float32
// [slots][H][D][D], read and left as the step's last state; pre: room for T * H * 5 * DP
// floats with DP = D rounded up to 16, 32, 64, 128 or 256; o float32 [T, H * D].  No segment
// is empty: a step with as many tokens as segments brings one token a segment.
extern "C" int hal_delta_rule(const float* r, int ldr, const float* k, int ldk, const float* v, int ldv,
                              const float* a_raw, int lda, const float* x1, int ldx1, const void* w2,
                              const void* w0, const void* a_bias, int w_dtype, int lora, float decay_rate,
                              float unit_eps, float* pre, float* state, const int* seg_q_start,
                              const int* seg_q_len, const int* token_slot, float* o, int n_tokens, int n_segs,
                              int H, int D, hipStream_t stream) {
  HAL_REQUIRE(n_tokens >= 0 && n_segs >= 0 && H > 0 && D > 0 && lora > 0,
              "hal_delta_rule: bad sizes T=%d segments=%d heads=%d dim=%d lora=%d", n_tokens, n_segs, H, D, lora);
  HAL_REQUIRE(D <= 256, "hal_delta_rule: a head of %d channels exceeds 256", D);
  HAL_REQUIRE(lora <= DELTA_MAX_LORA, "hal_delta_rule: a decay projection of rank %d exceeds %d", lora, DELTA_MAX_LORA);
  HAL_REQUIRE(H <= 65535, "hal_delta_rule: %d heads exceed the grid limit", H);
  HAL_REQUIRE(ldr >= H * D && ldk >= H * D && ldv >= H * D && lda >= H * D && ldx1 >= lora,
              "hal_delta_rule: rows too short");
  HAL_REQUIRE(w_dtype == HAL_F32 || w_dtype == HAL_BF16, "hal_delta_rule: dtype %d", w_dtype);
  if (n_tokens == 0 || n_segs == 0) return 0;
  const int DP = D <= 16 ? 16 : D <= 32 ? 32 : D <= 64 ? 64 : D <= 128 ? 128 : 256;
  if (n_tokens == n_segs && (D == 32 || D == 64 || D == 128)) {
    const dim3 heads(n_tokens, H);
#define DELTA_STEP(D_, W_)                                                                                          \
  hipLaunchKernelGGL((delta_step_kernel<D_, W_>), heads, dim3(256), 0, stream, r, ldr, k, ldk, v, ldv, a_raw, lda, x1, \
                     ldx1, (const W_*)w2, (const W_*)w0, (const W_*)a_bias, lora, decay_rate, unit_eps, state,          \
                     token_slot, o, H)
#define DELTA_STEP_OF(W_)         \
  if (D == 32) DELTA_STEP(32, W_); \
  else if (D == 64) DELTA_STEP(64, W_); \
  else DELTA_STEP(128, W_)
    if (w_dtype == HAL_F32) { DELTA_STEP_OF(float); }
    else { DELTA_STEP_OF(bf16_t); }
#undef DELTA_STEP_OF
#undef DELTA_STEP
    HAL_LAUNCH_CHECK();
    return 0;
  }
  // few tokens: a workgroup a token, so that they are made side by side; many: sixteen a
  // workgroup, which reads its rows of W2 once for all of them
#define DELTA_PREP(TT_, W_)                                                                                            \
  hipLaunchKernelGGL((delta_prep_kernel<TT_, W_>), dim3((n_tokens + TT_ - 1) / TT_, H), dim3(DP < 64 ? 64 : DP), 0, stream, \
                     r, ldr, k, ldk, a_raw, lda, x1, ldx1, (const W_*)w2, (const W_*)w0, (const W_*)a_bias, lora,       \
                     decay_rate, unit_eps, pre, n_tokens, H, D, DP)
  if (n_tokens < 256) {
    if (w_dtype == HAL_F32) DELTA_PREP(1, float);
    else DELTA_PREP(1, bf16_t);
  } else {
    if (w_dtype == HAL_F32) DELTA_PREP(16, float);
    else DELTA_PREP(16, bf16_t);
  }
#undef DELTA_PREP
#define DELTA_SCAN(N_, COLS_)                                                                             \
  hipLaunchKernelGGL((delta_scan_kernel<N_, COLS_>), dim3(n_segs, H, (D + COLS_ - 1) / COLS_), dim3(HAL_WAVE), 0, \
                     stream, pre, v, ldv, state, seg_q_start, seg_q_len, token_slot, o, H, D)
  if (DP == 16) DELTA_SCAN(4, 16);
  else if (DP == 32) DELTA_SCAN(8, 16);
  // (eight columns a wave make a token's step short, which is what a lone prompt waits for;
  // with many waves a SIMD the walk is bound by its LDS reads, and sixteen columns a wave
  // read half as much for the same part of the state)
  else if (DP == 64 && (long long)n_segs * H * ((D + 7) / 8) > DELTA_WAVES_FOR_WIDE) DELTA_SCAN(16, 16);
  else if (DP == 64) DELTA_SCAN(8, 8);
  else if (DP == 128) DELTA_SCAN(16, 8);
  else DELTA_SCAN(32, 8);
#undef DELTA_SCAN
  HAL_LAUNCH_CHECK();
  return 0;
}

// ---- out = y / rms(y over each head) * w * sigmoid(z): a wave a (token, head) -------------
template <typename T>
__global__ void head_norm_gate_kernel(const float* __restrict__ y, const float* __restrict__ z, int ldz,
                                      const void* __restrict__ w, int w_dtype, float eps, T* __restrict__ out,
                                      int n_tokens, int H, int D) {
  const int lane = threadIdx.x % HAL_WAVE;
  const size_t unit = (size_t)blockIdx.x * (blockDim.x / HAL_WAVE) + threadIdx.x / HAL_WAVE;
  if (unit >= (size_t)n_tokens * H) return;
  const size_t t = unit / H;
  const int h = (int)(unit % H);
  const float* yr = y + (t * H + h) * D;
  float ss = 0.f;
  for (int i = lane; i < D; i += HAL_WAVE) ss += yr[i] * yr[i];
  const float rstd = 1.0f / sqrtf(wave_sum(ss) / (float)D + eps);
  for (int i = lane; i < D; i += HAL_WAVE) {
    const size_t c = (size_t)h * D + i;
    const float g = z ? delta_sigmoid(z[t * ldz + c]) : 1.0f;
    const float wt = w ? load_as_f32(w, w_dtype, c) : 1.0f;
    out[t * H * D + c] = from_f32<T>(yr[i] * rstd * wt * g);
  }
}

// The same for heads of many channels: a workgroup a (token, head).
template <typename T>
__global__ void __launch_bounds__(256)
head_norm_gate_wide_kernel(const float* __restrict__ y, const float* __restrict__ z, int ldz,
                           const void* __restrict__ w, int w_dtype, float eps, T* __restrict__ out, int H, int D) {
  __shared__ float scratch[16];
  const size_t t = blockIdx.x;
  const int h = blockIdx.y;
  const float* yr = y + (t * H + h) * D;
  float ss = 0.f;
  for (int i = threadIdx.x; i < D; i += blockDim.x) ss += yr[i] * yr[i];
  const float rstd = 1.0f / sqrtf(block_sum(ss, scratch) / (float)D + eps);
  for (int i = threadIdx.x; i < D; i += blockDim.x) {
    const size_t c = (size_t)h * D + i;
    const float g = z ? delta_sigmoid(z[t * ldz + c]) : 1.0f;
    const float wt = w ? load_as_f32(w, w_dtype, c) : 1.0f;
    out[t * H * D + c] = from_f32<T>(yr[i] * rstd * wt * g);
  }
}

extern "C" int hal_head_norm_gate(const float* y, const float* z, int ldz, const void* w, int w_dtype, float eps,
                                  void* out, int dtype, int n_tokens, int H, int D, hipStream_t stream) {
  HAL_REQUIRE(n_tokens >= 0 && H > 0 && D > 0 && (z == nullptr || ldz >= H * D),
              "hal_head_norm_gate: bad sizes T=%d heads=%d dim=%d", n_tokens, H, D);
  HAL_REQUIRE(dtype == HAL_F32 || dtype == HAL_BF16, "hal_head_norm_gate: dtype %d", dtype);
  if (n_tokens == 0) return 0;
  if (D >= 512 && H <= 65535) {
    const dim3 wide(n_tokens, H);
    if (dtype == HAL_F32)
      hipLaunchKernelGGL(head_norm_gate_wide_kernel<float>, wide, dim3(256), 0, stream, y, z, ldz, w, w_dtype, eps,
                         (float*)out, H, D);
    else
      hipLaunchKernelGGL(head_norm_gate_wide_kernel<bf16_t>, wide, dim3(256), 0, stream, y, z, ldz, w, w_dtype, eps,
                         (bf16_t*)out, H, D);
    HAL_LAUNCH_CHECK();
    return 0;
  }
  const long long units = (long long)n_tokens * H;
  const dim3 grid((unsigned)((units + 3) / 4));
  if (dtype == HAL_F32)
    hipLaunchKernelGGL(head_norm_gate_kernel<float>, grid, dim3(256), 0, stream, y, z, ldz, w, w_dtype, eps,
                       (float*)out, n_tokens, H, D);
  else
    hipLaunchKernelGGL(head_norm_gate_kernel<bf16_t>, grid, dim3(256), 0, stream, y, z, ldz, w, w_dtype, eps,
                       (bf16_t*)out, n_tokens, H, D);
  HAL_LAUNCH_CHECK();
  return 0;
}
