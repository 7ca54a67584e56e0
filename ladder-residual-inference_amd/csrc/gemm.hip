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

// ---------------------------------------------------------------------------------------------
// Skinny GEMM for decode batches (4 < M <= 64): the weights are streamed once, the few input rows
// ride along.  A workgroup owns 32 weight rows (N / 32 workgroups: every CU has work even for the
// 1280-row wqkv), stages [32 x 128] weight and [MT x 128] input tiles through LDS (coalesced
// 16-byte loads, double buffered) and its 4 waves split the tile's 8 k-steps; their partial
// accumulators meet in LDS at the end.  y^T = W x^T on the matrix cores: A = weight rows,
// B = input rows (MT / 32 column tiles), so a lane ends up with 4 consecutive n of one m.
// ---------------------------------------------------------------------------------------------
constexpr int SN = 32, SK = 128, SLD = SK + 8;

template <int MT>
__global__ __launch_bounds__(256) void k_gemm_skinny(const u16* __restrict__ x, int64_t ldx, const u16* __restrict__ w,
                                                     u16* __restrict__ y, int64_t ldy, int M, int N, int K) {
  constexpr int CT = MT / 32;                       // column tiles (input rows / 32)
  constexpr int XCH = MT * SK / 8 / 256;            // 16-byte chunks of the input tile per thread
  constexpr int WCH = SN * SK / 8 / 256;            // ... of the weight tile
  constexpr int STAGE = (SN + MT) * SLD;            // elements per LDS stage
  constexpr int LDS_ELEMS = 2 * STAGE > 4 * CT * 16 * 64 * 2 ? 2 * STAGE : 4 * CT * 16 * 64 * 2;
  __shared__ __attribute__((aligned(16))) u16 lds[LDS_ELEMS];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = blockIdx.x * SN;
  const int arow = lane & 31, akq = (lane >> 5) * 8;

  f32x16_t acc[CT];
#pragma unroll
  for (int c = 0; c < CT; ++c)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[c][v] = 0.0f;

  uint4 xr[XCH], wr[WCH];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < WCH; ++i) {
      const int id = tid + i * 256, r = id >> 4, c = (id & 15) * 8;
      wr[i] = load_w_chunk(w, N, K, n0 + r, k0 + c);
    }
#pragma unroll
    for (int i = 0; i < XCH; ++i) {
      const int id = tid + i * 256, r = id >> 4, c = (id & 15) * 8;
      xr[i] = load_x_chunk<false>(x, ldx, M, K, r, k0 + c);
    }
  };
  auto stage = [&](int buf) {
    u16* ws_ = lds + buf * STAGE;
    u16* xs_ = ws_ + SN * SLD;
#pragma unroll
    for (int i = 0; i < WCH; ++i) {
      const int id = tid + i * 256, r = id >> 4, c = (id & 15) * 8;
      st16(&ws_[r * SLD + c], wr[i]);
    }
#pragma unroll
    for (int i = 0; i < XCH; ++i) {
      const int id = tid + i * 256, r = id >> 4, c = (id & 15) * 8;
      st16(&xs_[r * SLD + c], xr[i]);
    }
  };
  const int nk = (K + SK - 1) / SK;
  fetch(0);
  stage(0);
  __syncthreads();
  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < nk) fetch((kt + 1) * SK);
    const u16* ws_ = lds + cur * STAGE;
    const u16* xs_ = ws_ + SN * SLD;
#pragma unroll
    for (int q = 0; q < 2; ++q) {  // this wave's two k-steps of the tile
      const int kk = (wave * 2 + q) * 16;
      const bf16x8_t af = *reinterpret_cast<const bf16x8_t*>(&ws_[arow * SLD + kk + akq]);
#pragma unroll
      for (int c = 0; c < CT; ++c) {
        const bf16x8_t bfr = *reinterpret_cast<const bf16x8_t*>(&xs_[(c * 32 + arow) * SLD + kk + akq]);
        acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, bfr, acc[c], 0, 0, 0);
      }
    }
    if (kt + 1 < nk) stage(cur ^ 1);
    __syncthreads();
  }
  // ---- sum the four waves' partial accumulators in a fixed order
  float* red = reinterpret_cast<float*>(lds);  // [wave][c][v][lane]
#pragma unroll
  for (int c = 0; c < CT; ++c)
#pragma unroll
    for (int v = 0; v < 16; ++v) red[((wave * CT + c) * 16 + v) * 64 + lane] = acc[c][v];
  __syncthreads();
  // wave w finishes accumulator elements v = 4 w .. 4 w + 3: four consecutive n of one m per lane
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    float o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int v = wave * 4 + j;
      o[j] = (red[((0 * CT + c) * 16 + v) * 64 + lane] + red[((1 * CT + c) * 16 + v) * 64 + lane]) +
             (red[((2 * CT + c) * 16 + v) * 64 + lane] + red[((3 * CT + c) * 16 + v) * 64 + lane]);
    }
    // element v: n = n0 + (v / 4) * 8 + (lane / 32) * 4 + v % 4,  m = c * 32 + lane % 32
    const int m = c * 32 + (lane & 31), n = n0 + wave * 8 + (lane >> 5) * 4;
    if (m < M) {
      if (n + 3 < N) {
        uint2 pk;
        pk.x = pack_bf2(o[0], o[1]);
        pk.y = pack_bf2(o[2], o[3]);
        *reinterpret_cast<uint2*>(y + (int64_t)m * ldy + n) = pk;
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (n + j < N) y[(int64_t)m * ldy + n + j] = f_to_bf(o[j]);
      }
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
  if (M <= 4 || (act_swiglu && M <= 8)) return lr_gemv_dispatch(x, ldx, w, y, ldy, M, N, K, act_swiglu, s);
  if (!act_swiglu && M <= 64 && ldy % 4 == 0) {
    const dim3 sgrid((N + SN - 1) / SN);
    if (M <= 32)
      k_gemm_skinny<32><<<sgrid, dim3(256), 0, s>>>((const u16*)x, ldx, (const u16*)w, (u16*)y, ldy, M, N, K);
    else
      k_gemm_skinny<64><<<sgrid, dim3(256), 0, s>>>((const u16*)x, ldx, (const u16*)w, (u16*)y, ldy, M, N, K);
    return lr_launch_status();
  }
  const dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  if (grid.y > 65535) return LR_E_UNSUPPORTED;
  if (act_swiglu)
    k_gemm<true><<<grid, dim3(256), 0, s>>>((const u16*)x, ldx, (const u16*)w, (u16*)y, ldy, M, N, K);
  else
    k_gemm<false><<<grid, dim3(256), 0, s>>>((const u16*)x, ldx, (const u16*)w, (u16*)y, ldy, M, N, K);
  return lr_launch_status();
}
