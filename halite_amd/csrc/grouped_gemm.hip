// Products in groups: Y_g = X_g * W_g^T for g = 0 .. G-1, one launch for all groups.
//
// A group is a head (every group has the same rows, its operands are column ranges of
// wider rows: the per-head projections of a latent attention) or an expert of a mixture
// (the groups' rows are slices of one sorted list of (token, choice) pairs whose bounds
// are on the device; rows of X are gathered and rows of Y scattered through index
// arrays).  W is [G, N, K] with row length ldw.  The epilogue can multiply by the sigmoid
// of a float32 gate (heads), or compute the clamped gated activation of two products
// (experts: W the gate's weight, W2 the up projection's), write float32 or bf16, or add
// into a float32 destination.  Accumulation is float32 throughout; a row's result depends
// on that row alone.
//
// Two kernels: tiles of 64 x 64 on the vector units for any element type and any sizes,
// and for bf16 operands whose addresses allow 16-byte loads tiles of 128 x 128 on the matrix
// cores (v_mfma_f32_16x16x32_bf16), K staged through LDS in the instruction's operand order.
#include "hal_common.h"
#include "hal_api.h"

struct GroupedArgs {
  const void* X;
  int ldx, x_group_cols, x_col0;
  const void* W;
  const void* W2;
  long long w_group_stride;
  int ldw;
  void* Y;
  int ldy, y_group_cols, y_col0, y_dtype, y_add;
  int M, N, K, G;
  const int* group_offsets;  // [G + 1] or null
  const int* tile_offsets;   // [G + 1] with group_offsets
  const int* row_src;        // or null
  int src_div;
  const int* row_dst;  // or null
  const float* gate;   // or null
  int ldg;
  int gate_group_cols, gate_cols;  // the gate of group g, column n: gate[row][g * gate_group_cols + (gate_cols ? n : 0)]
  float limit, alpha, up_shift;
  int act;  // without W2: 0 the product as it is, 1 the square of its positive part
};

#define GG_ROWS 128  // rows of a workgroup's tile (what the tile offsets count in)
#define GG_TM 64     // the vector-unit kernel takes them in two halves of 64 rows, 64 columns at a time
#define GG_TN 64
#define GG_TK 16

// which group and which rows a workgroup serves; false: nothing
__device__ __forceinline__ bool gg_locate(const GroupedArgs& a, int& g, int& row0, int& row_end) {
  if (a.group_offsets == nullptr) {
    g = blockIdx.z;
    row0 = blockIdx.y * GG_ROWS;
    row_end = a.M;
    return row0 < row_end;
  }
  const int tile = blockIdx.y;
  if (tile >= a.tile_offsets[a.G]) return false;
  int lo = 0, hi = a.G;  // the last group whose first tile is <= tile
  while (hi - lo > 1) {
    const int mid = (lo + hi) / 2;
    if (a.tile_offsets[mid] <= tile) lo = mid; else hi = mid;
  }
  g = lo;
  row0 = a.group_offsets[g] + (tile - a.tile_offsets[g]) * GG_ROWS;
  row_end = a.group_offsets[g + 1];
  return row0 < row_end;
}

__device__ __forceinline__ float gg_sigmoid(float z) { return 1.0f / (1.0f + __expf(-z)); }

__device__ __forceinline__ void gg_store(const GroupedArgs& a, int g, int i, int n, float v, float v2,
                                         bool gated) {
  if (gated) {
    const float gg = fminf(v, a.limit);
    const float uu = fminf(fmaxf(v2, -a.limit), a.limit);
    v = gg * gg_sigmoid(a.alpha * gg) * (uu + a.up_shift);
  }
  if (!gated && a.act == 1) {
    v = fmaxf(v, 0.f);
    v = v * v;
  }
  const int dst = a.row_dst ? a.row_dst[i] : i;
  const size_t col = (size_t)g * a.y_group_cols + a.y_col0 + n;
  if (a.gate) v *= gg_sigmoid(a.gate[(size_t)dst * a.ldg + (size_t)g * a.gate_group_cols + (a.gate_cols ? n : 0)]);
  const size_t at = (size_t)dst * a.ldy + col;
  if (a.y_dtype == HAL_F32) {
    float* y = (float*)a.Y;
    y[at] = a.y_add ? y[at] + v : v;
  } else {
    ((bf16_t*)a.Y)[at] = f32_to_bf16(v);
  }
}

template <typename T, bool GATED>
__global__ void __launch_bounds__(256) grouped_fma_kernel(GroupedArgs a) {
  int g, row0, row_end;
  if (!gg_locate(a, g, row0, row_end)) return;
  row0 += (blockIdx.x % (GG_ROWS / GG_TM)) * GG_TM;  // which half of the tile's rows
  if (row0 >= row_end) return;
  const int n0 = (blockIdx.x / (GG_ROWS / GG_TM)) * GG_TN;
  __shared__ float As[GG_TK][GG_TM + 4];
  __shared__ float Bs[GG_TK][GG_TN + 4];
  __shared__ float B2s[GATED ? GG_TK : 1][GG_TN + 4];
  __shared__ int src_rows[GG_TM];
  const int tid = threadIdx.x;
  if (tid < GG_TM) {
    const int i = row0 + tid;
    int s = -1;
    if (i < row_end) s = a.row_src ? a.row_src[i] / a.src_div : i;
    src_rows[tid] = s;
  }
  __syncthreads();
  const T* X = (const T*)a.X + (size_t)g * a.x_group_cols + a.x_col0;
  const T* W = (const T*)a.W + (size_t)g * a.w_group_stride;
  const T* W2 = GATED ? (const T*)a.W2 + (size_t)g * a.w_group_stride : nullptr;
  const int tm = (tid / 16) * 4, tn = (tid % 16) * 4;
  float acc[4][4] = {}, acc2[4][4] = {};
  // a thread brings element (r, kk) of each tile, r = tid / 4 (+ 0), kk = (tid % 4) * 4 .. + 3
  const int lr = tid / 4, lk = (tid % 4) * 4;
  for (int k0 = 0; k0 < a.K; k0 += GG_TK) {
    const int s = src_rows[lr];
    const int n = n0 + lr;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = k0 + lk + j;
      const bool kin = k < a.K;
      As[lk + j][lr] = (s >= 0 && kin) ? to_f32(X[(size_t)s * a.ldx + k]) : 0.f;
      Bs[lk + j][lr] = (n < a.N && kin) ? to_f32(W[(size_t)n * a.ldw + k]) : 0.f;
      if (GATED) B2s[lk + j][lr] = (n < a.N && kin) ? to_f32(W2[(size_t)n * a.ldw + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GG_TK; ++kk) {
      float av[4], bv[4], b2v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        av[i] = As[kk][tm + i];
        bv[i] = Bs[kk][tn + i];
        if (GATED) b2v[i] = B2s[kk][tn + i];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
          if (GATED) acc2[i][j] = fmaf(av[i], b2v[j], acc2[i][j]);
        }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = row0 + tm + i;
    if (r >= row_end) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tn + j;
      if (n < a.N) gg_store(a, g, r, n, acc[i][j], acc2[i][j], GATED);
    }
  }
}

typedef __attribute__((ext_vector_type(8))) __bf16 gg_bf16x8;
typedef __attribute__((ext_vector_type(4))) float gg_f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t gg_u32x4;

__device__ __forceinline__ gg_bf16x8 gg_frag(const bf16_t* p, bool valid) {
  gg_u32x4 raw = {0u, 0u, 0u, 0u};
  if (valid) raw = *(const gg_u32x4*)p;
  return __builtin_bit_cast(gg_bf16x8, raw);
}

// bf16 on the matrix cores: a workgroup of four waves takes 128 rows x 128 columns, a wave
// 64 x 64 (sixteen 16 x 16 results).  K goes through LDS 64 at a time: every thread brings
// 16-byte pieces (eight k of one row) of the X rows and of the W rows, the next stage's while
// this one is multiplied, and puts them down in the instruction's operand order, so that a
// wave reads an operand (16 rows x 32 k) as one contiguous KiB: lane l holds row l % 16 and
// the eight k from (l / 16) * 8 on.  Lane l of a result holds W row (column) l % 16 and the
// X rows 4 * (l / 16) .. + 3, so a store instruction writes runs of 16 neighbouring columns.
// K, ldx, ldw and the column offsets are multiples of 8 and the bases 16-byte aligned.
#define GM_TK 64
// Where the piece of eight k (q of four in step ks of 32 k) of row r of a 16-row tile lies in
// the tile-step's KiB: at lane q * 16 + r of the operand, with r's bits turned by q and ks, so
// that the sixteen lanes of a store (two rows, eight pieces) meet sixteen different banks, and
// the sixteen lanes of a load (one q, sixteen rows) still read one contiguous quarter KiB.
__device__ __forceinline__ int gm_slot(int q, int r, int ks) { return q * 16 + (r ^ (q << 2) ^ (ks << 1)); }
__device__ __forceinline__ int gm_lds_offset(int row, int kc) {  // kc: which piece of eight k
  return (((row / 16) * (GM_TK / 32) + kc / 4) * 64 + gm_slot(kc % 4, row % 16, kc / 4)) * 8;
}

// GATED: the tile's 128 W rows are, for each of the two column halves of the waves, 32 rows of
// the gate's weight and the same 32 rows of the up projection's, so a wave holds both products
// of its 32 result columns at the same lanes and the workgroup writes 64 columns.
template <bool GATED>
__global__ void __launch_bounds__(256, 2) grouped_mfma_kernel(GroupedArgs a) {
  int g, row0, row_end;
  if (!gg_locate(a, g, row0, row_end)) return;
  constexpr int COLS = GATED ? GG_ROWS / 2 : GG_ROWS;  // result columns of a workgroup
  constexpr int WCOLS = COLS / 2;                      // of a wave
  const int n0 = blockIdx.x * COLS;
  __shared__ __attribute__((aligned(16))) bf16_t As[GG_ROWS * GM_TK];
  __shared__ __attribute__((aligned(16))) bf16_t Bs[GG_ROWS * GM_TK];
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int wm = wave / 2, wn = wave % 2;
  const bf16_t* X = (const bf16_t*)a.X + (size_t)g * a.x_group_cols + a.x_col0;
  const bf16_t* W = (const bf16_t*)a.W + (size_t)g * a.w_group_stride;
  const bf16_t* W2 = GATED ? (const bf16_t*)a.W2 + (size_t)g * a.w_group_stride : nullptr;
  // the four pieces a thread brings of each operand: rows tid / 8 + 32 i, piece tid % 8
  const int kc = tid % 8;
  const bf16_t* xp[4];
  const bf16_t* wp[4];
  int at[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = tid / 8 + 32 * i;
    at[i] = gm_lds_offset(row, kc);
    const int r = row0 + row;
    xp[i] = nullptr;
    if (r < row_end) xp[i] = X + (size_t)(a.row_src ? a.row_src[r] / a.src_div : r) * a.ldx + kc * 8;
    int n = n0 + row;
    const bf16_t* from = W;
    if (GATED) {
      n = n0 + (row / 64) * WCOLS + row % WCOLS;
      if (row % 64 >= WCOLS) from = W2;
    }
    wp[i] = n < a.N ? from + (size_t)n * a.ldw + kc * 8 : nullptr;
  }
  gg_u32x4 rx[4], rw[4];
  auto bring = [&](int k0) {
    const bool kin = k0 + kc * 8 < a.K;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      rx[i] = gg_u32x4{0u, 0u, 0u, 0u};
      rw[i] = gg_u32x4{0u, 0u, 0u, 0u};
      if (xp[i] && kin) rx[i] = *(const gg_u32x4*)(xp[i] + k0);
      if (wp[i] && kin) rw[i] = *(const gg_u32x4*)(wp[i] + k0);
    }
  };
  gg_f32x4 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = gg_f32x4{0.f, 0.f, 0.f, 0.f};
  const bool active = row0 + wm * 64 < row_end && n0 + wn * WCOLS < a.N;  // a wave without rows or columns only carries
  bring(0);
  for (int k0 = 0; k0 < a.K; k0 += GM_TK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      *(gg_u32x4*)&As[at[i]] = rx[i];
      *(gg_u32x4*)&Bs[at[i]] = rw[i];
    }
    __syncthreads();
    if (k0 + GM_TK < a.K) bring(k0 + GM_TK);
    if (active) {
#pragma unroll
      for (int ks = 0; ks < GM_TK / 32; ++ks) {
        gg_bf16x8 xa[4], wa[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int slot = gm_slot(lane / 16, lane % 16, ks);
          xa[i] = *(const gg_bf16x8*)&As[(((wm * 4 + i) * (GM_TK / 32) + ks) * 64 + slot) * 8];
          wa[i] = *(const gg_bf16x8*)&Bs[(((wn * 4 + i) * (GM_TK / 32) + ks) * 64 + slot) * 8];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[i], wa[j], acc[i][j], 0, 0, 0);
      }
    }
    __syncthreads();
  }
  if (!active) return;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      const int r = row0 + wm * 64 + i * 16 + (lane / 16) * 4 + jj;
      if (r >= row_end) continue;
#pragma unroll
      for (int j = 0; j < (GATED ? 2 : 4); ++j) {
        const int n = n0 + wn * WCOLS + j * 16 + lane % 16;
        if (n < a.N) gg_store(a, g, r, n, acc[i][j][jj], GATED ? acc[i][j + 2][jj] : 0.f, GATED);
      }
    }
}

// bf16, few rows a group (decode steps): a workgroup takes 64 rows of W (GATED: 32 of the
// gate's weight and the same 32 of the up projection's) and the tile's rows 16 at a time.  Its
// four waves split K between them and read both operands straight from memory in the
// instruction's operand order, four steps of 32 k in flight at a time and no barrier on the
// way; their sums meet in LDS and are added in rising wave number.
#define GS_U 4
template <bool GATED>
__global__ void __launch_bounds__(256) grouped_skinny_kernel(GroupedArgs a) {
  int g, row0, row_end;
  if (!gg_locate(a, g, row0, row_end)) return;
  constexpr int COLS = GATED ? 32 : 64;
  const int n0 = blockIdx.x * COLS;
  __shared__ __attribute__((aligned(16))) float red[4][4][256];
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int r = lane % 16, q = lane / 16;
  const bf16_t* X = (const bf16_t*)a.X + (size_t)g * a.x_group_cols + a.x_col0;
  const bf16_t* W = (const bf16_t*)a.W + (size_t)g * a.w_group_stride;
  const bf16_t* W2 = GATED ? (const bf16_t*)a.W2 + (size_t)g * a.w_group_stride : nullptr;
  const bf16_t* wrow[4];
#pragma unroll
  for (int f = 0; f < 4; ++f) {
    const int n = n0 + (GATED ? f % 2 : f) * 16 + r;
    const bf16_t* from = (GATED && f >= 2) ? W2 : W;
    wrow[f] = n < a.N ? from + (size_t)n * a.ldw + q * 8 : nullptr;
  }
  const int steps = (a.K + 31) / 32;
  const int s_begin = (int)((long long)steps * wave / 4), s_end = (int)((long long)steps * (wave + 1) / 4);
  for (int r0 = row0; r0 < row_end; r0 += 16) {
    const int i = r0 + r;
    const bf16_t* xrow = nullptr;
    if (i < row_end) xrow = X + (size_t)(a.row_src ? a.row_src[i] / a.src_div : i) * a.ldx + q * 8;
    gg_f32x4 acc[4];
#pragma unroll
    for (int f = 0; f < 4; ++f) acc[f] = gg_f32x4{0.f, 0.f, 0.f, 0.f};
    for (int step = s_begin; step < s_end; step += GS_U) {
      gg_bf16x8 xa[GS_U], wa[GS_U][4];
#pragma unroll
      for (int u = 0; u < GS_U; ++u) {
        const int k = (step + u) * 32;
        const bool kin = step + u < s_end && k + q * 8 < a.K;
        xa[u] = gg_frag(xrow + k, kin && xrow != nullptr);
#pragma unroll
        for (int f = 0; f < 4; ++f) wa[u][f] = gg_frag(wrow[f] + k, kin && wrow[f] != nullptr);
      }
#pragma unroll
      for (int u = 0; u < GS_U; ++u)
#pragma unroll
        for (int f = 0; f < 4; ++f)
          acc[f] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[u], wa[u][f], acc[f], 0, 0, 0);
    }
#pragma unroll
    for (int f = 0; f < 4; ++f) *(gg_f32x4*)&red[wave][f][lane * 4] = acc[f];
    __syncthreads();
    // wave w adds up result w of all waves (GATED: waves 0 and 1, each the gate's and the up's)
    if (wave < (GATED ? 2 : 4)) {
      gg_f32x4 sum = gg_f32x4{0.f, 0.f, 0.f, 0.f}, sum2 = gg_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        sum += *(const gg_f32x4*)&red[w][wave][lane * 4];
        if (GATED) sum2 += *(const gg_f32x4*)&red[w][wave + 2][lane * 4];
      }
      const int n = n0 + wave * 16 + r;
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) {
        const int row = r0 + q * 4 + jj;
        if (row < row_end && n < a.N) gg_store(a, g, row, n, sum[jj], sum2[jj], GATED);
      }
    }
    __syncthreads();
  }
}

extern "C" int hal_grouped_gemm(const void* X, int ldx, int x_group_cols, int x_col0, const void* W,
                                const void* W2, long long w_group_stride, int ldw, int dtype,
                                void* Y, int ldy, int y_group_cols, int y_col0, int y_dtype,
                                int y_add, int M, int N, int K, int G, const int* group_offsets,
                                const int* tile_offsets, const int* row_src, int src_div,
                                const int* row_dst, const float* gate, int ldg, int gate_per_group,
                                float limit, float up_shift,
                                float alpha, int act, int allow_mfma, hipStream_t stream) {
  HAL_REQUIRE(act == 0 || (act == 1 && W2 == nullptr), "hal_grouped_gemm: activation %d", act);
  HAL_REQUIRE(M >= 0 && N > 0 && K > 0 && G > 0, "hal_grouped_gemm: bad sizes M=%d N=%d K=%d G=%d", M, N,
              K, G);
  HAL_REQUIRE(dtype == HAL_F32 || dtype == HAL_BF16, "hal_grouped_gemm: operand dtype %d", dtype);
  HAL_REQUIRE(y_dtype == HAL_F32 || y_dtype == HAL_BF16, "hal_grouped_gemm: result dtype %d", y_dtype);
  HAL_REQUIRE(!y_add || y_dtype == HAL_F32, "hal_grouped_gemm: only a float32 result is added into");
  HAL_REQUIRE((group_offsets == nullptr) == (tile_offsets == nullptr),
              "hal_grouped_gemm: group and tile offsets come together");
  HAL_REQUIRE(src_div > 0, "hal_grouped_gemm: src_div %d", src_div);
  HAL_REQUIRE(G <= 65535, "hal_grouped_gemm: %d groups", G);
  if (M == 0) return 0;
  GroupedArgs a;
  a.X = X; a.ldx = ldx; a.x_group_cols = x_group_cols; a.x_col0 = x_col0;
  a.W = W; a.W2 = W2; a.w_group_stride = w_group_stride; a.ldw = ldw;
  a.Y = Y; a.ldy = ldy; a.y_group_cols = y_group_cols; a.y_col0 = y_col0; a.y_dtype = y_dtype;
  a.y_add = y_add;
  a.M = M; a.N = N; a.K = K; a.G = G;
  a.group_offsets = group_offsets; a.tile_offsets = tile_offsets;
  a.row_src = row_src; a.src_div = src_div; a.row_dst = row_dst;
  a.gate = gate; a.ldg = ldg; a.limit = limit; a.alpha = alpha; a.act = act; a.up_shift = up_shift;
  a.gate_group_cols = gate_per_group ? 1 : y_group_cols;
  a.gate_cols = gate_per_group ? 0 : 1;
  const int row_tiles = (M + GG_ROWS - 1) / GG_ROWS;
  // (a list of M rows cut into G groups has at most M / tile + G tiles, each group's last one partly filled)
  dim3 grid((N + GG_TN - 1) / GG_TN * (GG_ROWS / GG_TM), group_offsets ? row_tiles + G : row_tiles,
            group_offsets ? 1 : G);
  HAL_REQUIRE(grid.y <= 65535, "hal_grouped_gemm: %u row tiles", grid.y);
  const bool aligned = K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0 && x_group_cols % 8 == 0 &&
                       x_col0 % 8 == 0 && w_group_stride % 8 == 0 && ((uintptr_t)X % 16 == 0) &&
                       ((uintptr_t)W % 16 == 0) && (W2 == nullptr || (uintptr_t)W2 % 16 == 0);
  // few rows a group: the kernel that keeps many loads in flight instead of staging tiles
  const long long rows_per_group = group_offsets ? M / G : M;
  if (dtype == HAL_BF16 && allow_mfma && aligned && rows_per_group <= 16) {
    grid.x = W2 ? (N + 31) / 32 : (N + 63) / 64;
    if (W2) hipLaunchKernelGGL(grouped_skinny_kernel<true>, grid, dim3(256), 0, stream, a);
    else hipLaunchKernelGGL(grouped_skinny_kernel<false>, grid, dim3(256), 0, stream, a);
  } else if (dtype == HAL_BF16 && allow_mfma && aligned) {
    grid.x = W2 ? (N + GG_ROWS / 2 - 1) / (GG_ROWS / 2) : (N + GG_ROWS - 1) / GG_ROWS;
    if (W2) hipLaunchKernelGGL(grouped_mfma_kernel<true>, grid, dim3(256), 0, stream, a);
    else hipLaunchKernelGGL(grouped_mfma_kernel<false>, grid, dim3(256), 0, stream, a);
  } else if (dtype == HAL_BF16) {
    if (W2) hipLaunchKernelGGL((grouped_fma_kernel<bf16_t, true>), grid, dim3(256), 0, stream, a);
    else hipLaunchKernelGGL((grouped_fma_kernel<bf16_t, false>), grid, dim3(256), 0, stream, a);
  } else {
    if (W2) hipLaunchKernelGGL((grouped_fma_kernel<float, true>), grid, dim3(256), 0, stream, a);
    else hipLaunchKernelGGL((grouped_fma_kernel<float, false>), grid, dim3(256), 0, stream, a);
  }
  HAL_LAUNCH_CHECK();
  return 0;
}
