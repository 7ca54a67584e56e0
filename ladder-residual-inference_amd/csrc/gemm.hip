// LDS-tiled MFMA bf16 GEMM for prefill (and for decode batches above 8 rows):
//   y[m, n] = bf16( sum_k x[m, k] * w[n, k] ),  fp32 accumulation in v_mfma_f32_32x32x16_bf16.
//
// Workgroup tile 128 x 128 x 64, four waves in a 2 x 2 arrangement, each wave owning a 64 x 64
// block = 2 x 2 MFMA tiles (64 accumulator VGPRs).  Both operands are K-contiguous in memory, so
// the same staging path serves them: 128-bit global loads -> registers -> LDS rows padded by 16
// bytes (stride 144 B keeps ds_read_b128 of 16 consecutive rows on distinct banks) -> 128-bit LDS
// reads that deliver exactly the 8 consecutive k an MFMA lane feeds.  LDS is double-buffered and
// the global loads of tile t+1 are in flight while tile t is multiplied.
#include "lr_common.h"

int lr_gemv_dispatch(const void* x, int64_t ldx, const void* w, void* y, int64_t ldy, int M, int N, int K,
                     int act_swiglu, hipStream_t s);

constexpr int BM = 128, BN = 128, BK = 64, LDT = BK + 8;  // LDT: padded LDS row length in elements

template <bool SWIGLU>
__device__ __forceinline__ uint4 load_x_chunk(const u16* __restrict__ x, int64_t ldx, int M, int K, int m, int k) {
  if (m >= M || k >= K) return make_uint4(0, 0, 0, 0);
  if (SWIGLU) {
    float u[8], g[8], o[8];
    unpack8(ld16(x + (int64_t)m * ldx + k), u);
    unpack8(ld16(x + (int64_t)m * ldx + K + k), g);
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = swiglu_bf(u[j], g[j]);
    return pack8(o);
  }
  return ld16(x + (int64_t)m * ldx + k);
}

__device__ __forceinline__ uint4 load_w_chunk(const u16* __restrict__ w, int N, int K, int n, int k) {
  if (n >= N || k >= K) return make_uint4(0, 0, 0, 0);
  return ld16(w + (int64_t)n * K + k);
}

template <bool SWIGLU>
__global__ __launch_bounds__(256) void k_gemm(const u16* __restrict__ x, int64_t ldx, const u16* __restrict__ w,
                                              u16* __restrict__ y, int64_t ldy, int M, int N, int K) {
  __shared__ __attribute__((aligned(16))) u16 xs[2][BM * LDT];
  __shared__ __attribute__((aligned(16))) u16 ws[2][BN * LDT];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;

  // staging assignment: 1024 16-byte chunks per operand tile, 4 per thread
  int srow[4], scol[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int id = tid + i * 256;
    srow[i] = id >> 3;
    scol[i] = (id & 7) * 8;
  }

  f32x16_t acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.0f;

  uint4 xr[4], wr[4];
  const int nk = (K + BK - 1) / BK;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    xr[i] = load_x_chunk<SWIGLU>(x, ldx, M, K, m0 + srow[i], scol[i]);
    wr[i] = load_w_chunk(w, N, K, n0 + srow[i], scol[i]);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    st16(&xs[0][srow[i] * LDT + scol[i]], xr[i]);
    st16(&ws[0][srow[i] * LDT + scol[i]], wr[i]);
  }
  __syncthreads();

  const int arow = lane & 31, akq = (lane >> 5) * 8;
  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < nk) {
      const int k0 = (kt + 1) * BK;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        xr[i] = load_x_chunk<SWIGLU>(x, ldx, M, K, m0 + srow[i], k0 + scol[i]);
        wr[i] = load_w_chunk(w, N, K, n0 + srow[i], k0 + scol[i]);
      }
    }
#pragma unroll
    for (int kk = 0; kk < BK; kk += 16) {
      bf16x8_t af[2], bfr[2];
#pragma unroll
      for (int a = 0; a < 2; ++a)
        af[a] = *reinterpret_cast<const bf16x8_t*>(&xs[cur][(wm * 64 + a * 32 + arow) * LDT + kk + akq]);
#pragma unroll
      for (int b = 0; b < 2; ++b)
        bfr[b] = *reinterpret_cast<const bf16x8_t*>(&ws[cur][(wn * 64 + b * 32 + arow) * LDT + kk + akq]);
#pragma unroll
      for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[a], bfr[b], acc[a][b], 0, 0, 0);
    }
    if (kt + 1 < nk) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        st16(&xs[cur ^ 1][srow[i] * LDT + scol[i]], xr[i]);
        st16(&ws[cur ^ 1][srow[i] * LDT + scol[i]], wr[i]);
      }
    }
    __syncthreads();
  }

  // accumulator element v of a 32x32 tile: row = (v / 4) * 8 + (lane / 32) * 4 + v % 4, col = lane % 32
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int n = n0 + wn * 64 + b * 32 + (lane & 31);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + wm * 64 + a * 32 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
        if (m < M && n < N) y[(int64_t)m * ldy + n] = f_to_bf(acc[a][b][v]);
      }
    }
}

extern "C" int lr_linear(const void* x, int64_t ldx, const void* w, void* y, int64_t ldy, int M, int N, int K,
                         int act_swiglu, lr_stream_t stream) {
  LR_REQUIRE_PTR(x);
  LR_REQUIRE_PTR(w);
  LR_REQUIRE_PTR(y);
  if (M <= 0 || N <= 0 || K <= 0) return LR_E_SHAPE;
  if (ldx < (act_swiglu ? 2 : 1) * (int64_t)K || ldy < N) return LR_E_SHAPE;
  if (K % 8 || ldx % 8) return LR_E_ALIGN;
  hipStream_t s = (hipStream_t)stream;
  if (M <= 8) return lr_gemv_dispatch(x, ldx, w, y, ldy, M, N, K, act_swiglu, s);
  const dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  if (grid.y > 65535) return LR_E_UNSUPPORTED;
  if (act_swiglu)
    k_gemm<true><<<grid, dim3(256), 0, s>>>((const u16*)x, ldx, (const u16*)w, (u16*)y, ldy, M, N, K);
  else
    k_gemm<false><<<grid, dim3(256), 0, s>>>((const u16*)x, ldx, (const u16*)w, (u16*)y, ldy, M, N, K);
  return lr_launch_status();
}
