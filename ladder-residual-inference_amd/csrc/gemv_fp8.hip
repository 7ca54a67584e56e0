// Weight-only fp8 (e4m3) linears for decode:  y[m, n] = bf16( bf16( sum_k x[m, k] * w8[n, k] ) * scales[n] ).
//
// Same shape as the bf16 GEMV (gemv.hip) with half the HBM bytes: every weight byte is read once,
// lanes of a wave walking K in 1 KiB strides (16 weights per lane and load).  A dword of four e4m3
// values becomes two packed bf16 pairs with v_cvt_scalef32_pk_bf16_fp8 (exact: e4m3 is a subset of
// bf16) and goes through v_dot2_f32_bf16 against the packed inputs, fp32 accumulation.  The sum is
// rounded to bf16, multiplied by the row's scale and rounded again -- the two roundings of
// F.linear(x, w.to(bf16)) * scales.  Partial sums meet in a fixed order: bit-reproducible.
//
// For more than 8 input rows (prefill) the weights are expanded to bf16 in a caller-provided scratch
// buffer and the bf16 matrix-core GEMM runs on that, followed by the per-column scaling.
#include "lr_common.h"

namespace {

constexpr int WPB = 4;  // waves per workgroup

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float dot2(u32 a, bf16x2_t b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), b, c, false);
}
// the low (hi == false) or high two e4m3 values of a dword as a packed bf16 pair
template <bool HI>
__device__ __forceinline__ bf16x2_t fp8_pair(u32 v) {
  return __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(v, 1.0f, HI);
}

// acc[m] += sum over the 16 weights of `wv` times x[m][k .. k + 16)
template <int M>
__device__ __forceinline__ void mac16(const uint4& wv, const uint4 (&xa)[M], const uint4 (&xb)[M], float (&acc)[M]) {
  const bf16x2_t w0 = fp8_pair<false>(wv.x), w1 = fp8_pair<true>(wv.x), w2 = fp8_pair<false>(wv.y),
                 w3 = fp8_pair<true>(wv.y), w4 = fp8_pair<false>(wv.z), w5 = fp8_pair<true>(wv.z),
                 w6 = fp8_pair<false>(wv.w), w7 = fp8_pair<true>(wv.w);
#pragma unroll
  for (int m = 0; m < M; ++m) {
    float a = acc[m];
    a = dot2(xa[m].x, w0, a); a = dot2(xa[m].y, w1, a); a = dot2(xa[m].z, w2, a); a = dot2(xa[m].w, w3, a);
    a = dot2(xb[m].x, w4, a); a = dot2(xb[m].y, w5, a); a = dot2(xb[m].z, w6, a); a = dot2(xb[m].w, w7, a);
    acc[m] = a;
  }
}

// A wave owns R rows; KSPLIT waves of the workgroup split K.  K % 16 == 0.
template <int M, int R, int KSPLIT>
__global__ __launch_bounds__(WPB * 64) void k_gemv_fp8(const u16* __restrict__ x, int64_t ldx,
                                                       const unsigned char* __restrict__ w,
                                                       const u16* __restrict__ scales, u16* __restrict__ y, int64_t ldy,
                                                       int m_real, int N, int K) {
  constexpr int GR = WPB / KSPLIT;
  __shared__ float part[WPB][R * M];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int grp = wave / KSPLIT, ks = wave % KSPLIT;
  const int n0 = (blockIdx.x * GR + grp) * R;
  const unsigned char* wrow[R];
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

  constexpr int KSTEP = KSPLIT * 1024;
  int k = (ks * 64 + lane) * 16;
  // two steps at a time: all weight loads issued before any use
  for (; k + KSTEP < K; k += 2 * KSTEP) {
    uint4 wv[2][R];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int r = 0; r < R; ++r) wv[u][r] = ld16(wrow[r] + k + u * KSTEP);
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      uint4 xa[M], xb[M];
#pragma unroll
      for (int m = 0; m < M; ++m) {
        const int mm = m < m_real ? m : m_real - 1;
        xa[m] = ld16(x + mm * ldx + k + u * KSTEP);
        xb[m] = ld16(x + mm * ldx + k + u * KSTEP + 8);
      }
#pragma unroll
      for (int r = 0; r < R; ++r) mac16<M>(wv[u][r], xa, xb, acc[r]);
    }
  }
  for (; k < K; k += KSTEP) {
    uint4 wv[R];
#pragma unroll
    for (int r = 0; r < R; ++r) wv[r] = ld16(wrow[r] + k);
    uint4 xa[M], xb[M];
#pragma unroll
    for (int m = 0; m < M; ++m) {
      const int mm = m < m_real ? m : m_real - 1;
      xa[m] = ld16(x + mm * ldx + k);
      xb[m] = ld16(x + mm * ldx + k + 8);
    }
#pragma unroll
    for (int r = 0; r < R; ++r) mac16<M>(wv[r], xa, xb, acc[r]);
  }
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < M; ++m) acc[r][m] = wave_sum(acc[r][m]);
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
    if (n0 + r < N && m < m_real) y[m * ldy + n0 + r] = f_to_bf(round_bf(s) * bf_to_f(scales[n0 + r]));
  }
}

template <int M>
static void launch(const u16* x, int64_t ldx, const unsigned char* w, const u16* sc, u16* y, int64_t ldy, int m_real, int N,
                   int K, hipStream_t s) {
  // enough waves to cover the chip several times over; K split over the waves of a workgroup when rows are long
  if (K >= 4096) {
    constexpr int R = M > 4 ? 1 : 2;
    k_gemv_fp8<M, R, 4><<<dim3((N + R - 1) / R), dim3(WPB * 64), 0, s>>>(x, ldx, w, sc, y, ldy, m_real, N, K);
  } else if (K >= 2048) {
    constexpr int R = M > 4 ? 1 : 2;
    k_gemv_fp8<M, R, 2><<<dim3((N + 2 * R - 1) / (2 * R)), dim3(WPB * 64), 0, s>>>(x, ldx, w, sc, y, ldy, m_real, N, K);
  } else {
    constexpr int R = M > 4 ? 1 : 2;
    k_gemv_fp8<M, R, 1><<<dim3((N + 4 * R - 1) / (4 * R)), dim3(WPB * 64), 0, s>>>(x, ldx, w, sc, y, ldy, m_real, N, K);
  }
}

// ---- prefill path: expand to bf16, scale the GEMM's columns afterwards
__global__ __launch_bounds__(256) void k_fp8_to_bf16(const unsigned char* __restrict__ w, u16* __restrict__ out, int64_t n16) {
  for (int64_t i = blockIdx.x * 256 + threadIdx.x; i < n16; i += (int64_t)gridDim.x * 256) {
    const uint4 v = ld16(w + i * 16);
    uint4 lo, hi;
    lo.x = __builtin_bit_cast(u32, fp8_pair<false>(v.x)); lo.y = __builtin_bit_cast(u32, fp8_pair<true>(v.x));
    lo.z = __builtin_bit_cast(u32, fp8_pair<false>(v.y)); lo.w = __builtin_bit_cast(u32, fp8_pair<true>(v.y));
    hi.x = __builtin_bit_cast(u32, fp8_pair<false>(v.z)); hi.y = __builtin_bit_cast(u32, fp8_pair<true>(v.z));
    hi.z = __builtin_bit_cast(u32, fp8_pair<false>(v.w)); hi.w = __builtin_bit_cast(u32, fp8_pair<true>(v.w));
    st16(out + i * 16, lo);
    st16(out + i * 16 + 8, hi);
  }
}
__global__ __launch_bounds__(256) void k_scale_cols(u16* __restrict__ y, int64_t ldy, const u16* __restrict__ scales, int N) {
  u16* row = y + (int64_t)blockIdx.y * ldy;
  for (int n = blockIdx.x * 256 + threadIdx.x; n < N; n += gridDim.x * 256)
    row[n] = f_to_bf(bf_to_f(row[n]) * bf_to_f(scales[n]));
}

}  // namespace

extern "C" size_t lr_linear_fp8_scratch_bytes(int M, int N, int K) {
  if (M <= 8 || N <= 0 || K <= 0) return 0;
  return (size_t)N * K * 2;
}

extern "C" int lr_linear_fp8(const void* x, int64_t ldx, const void* w8, const void* scales, void* y, int64_t ldy, int M,
                             int N, int K, void* scratch, size_t scratch_bytes, lr_stream_t stream) {
  LR_REQUIRE_PTR(x);
  LR_REQUIRE_PTR(w8);
  LR_REQUIRE_PTR(y);
  if (scales == nullptr) return LR_E_NULL;
  if (M <= 0 || N <= 0 || K <= 0 || ldx < K || ldy < N) return LR_E_SHAPE;
  if (K % 16 || ldx % 8) return LR_E_ALIGN;
  hipStream_t s = (hipStream_t)stream;
  const u16* xp = (const u16*)x;
  const unsigned char* wp = (const unsigned char*)w8;
  const u16* sp = (const u16*)scales;
  u16* yp = (u16*)y;
  if (M <= 8) {
    if (M == 1) launch<1>(xp, ldx, wp, sp, yp, ldy, M, N, K, s);
    else if (M == 2) launch<2>(xp, ldx, wp, sp, yp, ldy, M, N, K, s);
    else if (M <= 4) launch<4>(xp, ldx, wp, sp, yp, ldy, M, N, K, s);
    else launch<8>(xp, ldx, wp, sp, yp, ldy, M, N, K, s);
    return lr_launch_status();
  }
  LR_REQUIRE_PTR(scratch);
  if (scratch_bytes < lr_linear_fp8_scratch_bytes(M, N, K)) return LR_E_SHAPE;
  const int64_t n16 = (int64_t)N * K / 16;
  const int grid = (int)((n16 + 255) / 256 < 65535 ? (n16 + 255) / 256 : 65535);
  k_fp8_to_bf16<<<dim3(grid), dim3(256), 0, s>>>(wp, (u16*)scratch, n16);
  const int rc = lr_linear(x, ldx, scratch, y, ldy, M, N, K, 0, stream);
  if (rc != LR_OK) return rc;
  if (M > 65535) return LR_E_UNSUPPORTED;
  k_scale_cols<<<dim3((N + 255) / 256 < 64 ? (N + 255) / 256 : 64, M), dim3(256), 0, s>>>(yp, ldy, sp, N);
  return lr_launch_status();
}
