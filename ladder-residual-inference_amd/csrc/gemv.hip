// Weight-streaming bf16 GEMV for decode: y[m, n] = bf16( sum_k x[m, k] * w[n, k] ), M <= 8.
//
// HBM-bound: every weight is read exactly once with 128-bit loads, lanes of a wave walking K in
// 1 KiB strides so that each load instruction covers a contiguous kilobyte of one weight row.
// A wave owns R rows; KSPLIT waves of the workgroup share a row group and split K between them.
// Partial sums are combined by a wave64 butterfly and then, across the KSPLIT waves, through LDS
// in a fixed order -- no atomics, so results are bit-reproducible run to run.
// x (a few KiB) is re-read by every wave and lives in L1/L2.
#include "lr_common.h"

constexpr int GEMV_WPB = 4;  // waves per workgroup

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
// c + a.lo * b.lo + a.hi * b.hi on packed bf16 pairs, fp32 accumulation (v_dot2_f32_bf16)
__device__ __forceinline__ float dot2(u32 a, u32 b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), c, false);
}

// 8 inputs of every row as packed bf16 pairs (the SwiGLU values are bf16 by definition)
template <int M, bool SWIGLU>
__device__ __forceinline__ void load_x(const u16* __restrict__ x, int64_t ldx, int K, int k, int m_real,
                                       uint4 (&xp)[M]) {
#pragma unroll
  for (int m = 0; m < M; ++m) {
    const int mm = m < m_real ? m : m_real - 1;
    if (SWIGLU) {
      float u[8], g[8], o[8];
      unpack8(ld16(x + mm * ldx + k), u);
      unpack8(ld16(x + mm * ldx + K + k), g);
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = swiglu_bf(u[j], g[j]);
      xp[m] = pack8(o);
    } else {
      xp[m] = ld16(x + mm * ldx + k);
    }
  }
}
// acc[r][m] += w[r] . x[m] over 8 elements: weights and inputs stay packed, 4 dot2 per pair of rows
template <int M, int R>
__device__ __forceinline__ void mac8(const uint4 (&wv)[R], const uint4 (&xp)[M], float (&acc)[R][M]) {
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < M; ++m) {
      float a = acc[r][m];
      a = dot2(wv[r].x, xp[m].x, a);
      a = dot2(wv[r].y, xp[m].y, a);
      a = dot2(wv[r].z, xp[m].z, a);
      a = dot2(wv[r].w, xp[m].w, a);
      acc[r][m] = a;
    }
}

template <int M, int R, int KSPLIT, int U, bool SWIGLU>
__global__ __launch_bounds__(GEMV_WPB * 64) void k_gemv(const u16* __restrict__ x, int64_t ldx,
                                                        const u16* __restrict__ w, u16* __restrict__ y, int64_t ldy,
                                                        int m_real, int N, int K) {
  constexpr int GR = GEMV_WPB / KSPLIT;  // row groups per workgroup
  __shared__ float part[GEMV_WPB][R * M];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int grp = wave / KSPLIT, ks = wave % KSPLIT;
  const int n0 = (blockIdx.x * GR + grp) * R;

  const u16* wrow[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int n = n0 + r < N ? n0 + r : N - 1;  // clamp: out-of-range rows compute garbage that is never stored
    wrow[r] = w + (int64_t)n * K;
  }

  float acc[R][M];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < M; ++m) acc[r][m] = 0.0f;

  constexpr int KSTEP = KSPLIT * 512;
  int k = (ks * 64 + lane) * 8;
  // main loop: U steps at a time, all weight loads issued before any use
  for (; k + (U - 1) * KSTEP < K; k += U * KSTEP) {
    uint4 wv[U][R];
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int r = 0; r < R; ++r) wv[u][r] = ld16(wrow[r] + k + u * KSTEP);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      uint4 xp[M];
      load_x<M, SWIGLU>(x, ldx, K, k + u * KSTEP, m_real, xp);
      mac8<M, R>(wv[u], xp, acc);
    }
  }
  // remainder steps
  for (; k < K; k += KSTEP) {
    uint4 wv[R];
#pragma unroll
    for (int r = 0; r < R; ++r) wv[r] = ld16(wrow[r] + k);
    uint4 xp[M];
    load_x<M, SWIGLU>(x, ldx, K, k, m_real, xp);
    mac8<M, R>(wv, xp, acc);
  }

#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < M; ++m) acc[r][m] = wave_sum(acc[r][m]);

  if (KSPLIT > 1) {
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < M; ++m)
        if (lane == r * M + m) part[wave][r * M + m] = acc[r][m];
    __syncthreads();
    if (ks == 0 && lane < R * M) {
      float s = part[wave][lane];
#pragma unroll
      for (int j = 1; j < KSPLIT; ++j) s += part[wave + j][lane];
      const int r = lane / M, m = lane % M;
      if (n0 + r < N && m < m_real) y[m * ldy + n0 + r] = f_to_bf(s);
    }
  } else {
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < M; ++m)
        if (lane == r * M + m && n0 + r < N && m < m_real) y[m * ldy + n0 + r] = f_to_bf(acc[r][m]);
  }
}

template <int M, int R, int KSPLIT, int U, bool SWIGLU>
static void launch_gemv(const u16* x, int64_t ldx, const u16* w, u16* y, int64_t ldy, int m_real, int N, int K,
                        hipStream_t s) {
  constexpr int rows_per_wg = (GEMV_WPB / KSPLIT) * R;
  const int grid = (N + rows_per_wg - 1) / rows_per_wg;
  k_gemv<M, R, KSPLIT, U, SWIGLU><<<dim3(grid), dim3(GEMV_WPB * 64), 0, s>>>(x, ldx, w, y, ldy, m_real, N, K);
}

template <int M, bool SWIGLU>
static void dispatch_cfg(int cfg, const u16* x, int64_t ldx, const u16* w, u16* y, int64_t ldy, int m_real, int N,
                         int K, hipStream_t s) {
  // cfg = R * 100 + KSPLIT * 10 + U
  switch (cfg) {
#define LR_GEMV_CASE(R, KS, UU) \
  case R * 100 + KS * 10 + UU: launch_gemv<M, R, KS, UU, SWIGLU>(x, ldx, w, y, ldy, m_real, N, K, s); break;
    LR_GEMV_CASE(1, 4, 4)
    LR_GEMV_CASE(2, 1, 2)
    LR_GEMV_CASE(2, 2, 2)
    LR_GEMV_CASE(2, 4, 2)
    LR_GEMV_CASE(2, 4, 4)
    LR_GEMV_CASE(4, 1, 2)
    LR_GEMV_CASE(4, 2, 2)
    LR_GEMV_CASE(4, 4, 2)
#undef LR_GEMV_CASE
    default: launch_gemv<M, 2, 4, 2, SWIGLU>(x, ldx, w, y, ldy, m_real, N, K, s); break;
  }
}

// Shape heuristic: enough waves to cover 256 CUs several times over, enough K per wave to keep
// 8+ KiB of loads in flight, fewer rows per wave when M is large (register pressure).
static int pick_cfg(int M, int N, int K) {
  const int r_max = M > 4 ? 2 : 4;
  int ksplit = K >= 4096 ? 4 : (K >= 2048 ? 2 : 1);
  int R = r_max;
  // waves = N / R * ksplit; want >= 4096 when the matrix is big enough
  while (R > 1 && (int64_t)N / R * ksplit < 4096) R >>= 1;
  if (R == 1 && ksplit != 4) R = 2;
  if (R == 1) return 144;
  const int steps = K / (ksplit * 512);
  const int U = (R == 2 && ksplit == 4 && steps >= 4) ? 4 : 2;
  return R * 100 + ksplit * 10 + U;
}

// gemv_cfg: rows-per-wave * 100 + K-split * 10 + unroll, or 0 for the shape heuristic
int lr_gemv_dispatch(const void* x, int64_t ldx, const void* w, void* y, int64_t ldy, int M, int N, int K,
                     int act_swiglu, int gemv_cfg, hipStream_t s) {
  const int cfg = gemv_cfg ? gemv_cfg : pick_cfg(M, N, K);
  const u16* xp = (const u16*)x;
  const u16* wp = (const u16*)w;
  u16* yp = (u16*)y;
#define LR_GEMV_M(MT)                                                              \
  if (act_swiglu) dispatch_cfg<MT, true>(cfg, xp, ldx, wp, yp, ldy, M, N, K, s);   \
  else dispatch_cfg<MT, false>(cfg, xp, ldx, wp, yp, ldy, M, N, K, s);
  if (M == 1) { LR_GEMV_M(1) }
  else if (M == 2) { LR_GEMV_M(2) }
  else if (M <= 4) { LR_GEMV_M(4) }
  else { LR_GEMV_M(8) }
#undef LR_GEMV_M
  return lr_launch_status();
}
