// Weight-only fp8 (e4m3) linears for decode:  y[m, n] = bf16( bf16( sum_k x[m, k] * w8[n, k] ) * scales[n] ).
//
// Same shape as the bf16 GEMV (gemv.hip) with half the HBM bytes: every weight byte is read once,
// lanes of a wave walking K in 1 KiB strides (16 weights per lane and load).  A dword of four e4m3
// values becomes two packed bf16 pairs with v_cvt_scalef32_pk_bf16_fp8 (exact: e4m3 is a subset of
// bf16) and goes through v_dot2_f32_bf16 against the packed inputs, fp32 accumulation.  The sum is
// rounded to bf16, multiplied by the row's scale and rounded again -- the two roundings of
// F.linear(x, w.to(bf16)) * scales.  Partial sums meet in a fixed order: bit-reproducible.
//
// From 2 to 16 input rows (decode batches) the projections run as matrix-core bands that expand the
// weights on their way through LDS (stream_band.h, W8).  For more than 16 input rows (prefill) the
// weights are expanded to bf16 in a caller-provided scratch buffer and the bf16 matrix-core GEMM runs
// on that, followed by the per-column scaling.
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

// ---- one or two projections per launch, pairs of rows per wave, epilogues on the pair
// What the per-op decode path of a quantised ladder model needs per block in two launches instead of six:
// {q/k/v (rotated, k and v into the cache) next to up/gate (stored as silu(gate) * up)} and {wo next to w2}.
// A wave group owns two weight rows -- (2p, 2p + 1), or (p, p + I) for [up; gate] rows -- so that both halves of
// a rotation or an activation pair end up in one lane.  Per row the loads, the products and the order of the
// partial sums are those of k_gemv_fp8: the projected values are lr_linear_fp8's, bit for bit.
struct P8 {
  const u16* x;
  const unsigned char* w;
  const u16* scales;
  u16* y;
  int64_t ldx, ldy;
  int N, K;
  int pair_off;  // 0: rows (2p, 2p + 1); else rows (p, p + pair_off) and the output column is p
  int ksplit;    // waves that split K: 1, 2 or 4
  int npairs, nwg;
  const u16* rope_table;  // RoPE + KV-cache epilogue of a fused q/k/v projection (nullptr: none)
  const int32_t* pos;
  u16 *k_cache, *v_cache;
  int32_t* err;
  int Hq, Hkv, hd, Smax, block_size;
};

template <int M>
__global__ __launch_bounds__(WPB * 64) void k_gemv_fp8_multi(const P8 p0, const P8 p1, int m_real) {
  __shared__ float part[WPB][2 * M];
  const bool second = (int)blockIdx.x >= p0.nwg;
  const P8 p = second ? p1 : p0;
  const int wg = second ? (int)blockIdx.x - p0.nwg : (int)blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int ksplit = p.ksplit, grp = wave / ksplit, ks = wave % ksplit;
  const int pi = wg * (WPB / ksplit) + grp;
  const int N = p.N, K = p.K;
  const int r0 = p.pair_off ? pi : 2 * pi, r1 = p.pair_off ? pi + p.pair_off : 2 * pi + 1;
  // clamp: out-of-range rows compute garbage that is never stored
  const unsigned char* wrow[2] = {p.w + (int64_t)(r0 < N ? r0 : N - 1) * K, p.w + (int64_t)(r1 < N ? r1 : N - 1) * K};
  const u16* const x = p.x;
  const int64_t ldx = p.ldx;
  float acc[2][M];
#pragma unroll
  for (int r = 0; r < 2; ++r)
#pragma unroll
    for (int m = 0; m < M; ++m) acc[r][m] = 0.0f;
  const int kstep = ksplit * 1024;
  int k = (ks * 64 + lane) * 16;
  for (; k + kstep < K; k += 2 * kstep) {
    uint4 wv[2][2];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int r = 0; r < 2; ++r) wv[u][r] = ld16(wrow[r] + k + u * kstep);
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      uint4 xa[M], xb[M];
#pragma unroll
      for (int m = 0; m < M; ++m) {
        const int mm = m < m_real ? m : m_real - 1;
        xa[m] = ld16(x + mm * ldx + k + u * kstep);
        xb[m] = ld16(x + mm * ldx + k + u * kstep + 8);
      }
#pragma unroll
      for (int r = 0; r < 2; ++r) mac16<M>(wv[u][r], xa, xb, acc[r]);
    }
  }
  for (; k < K; k += kstep) {
    uint4 wv[2];
#pragma unroll
    for (int r = 0; r < 2; ++r) wv[r] = ld16(wrow[r] + k);
    uint4 xa[M], xb[M];
#pragma unroll
    for (int m = 0; m < M; ++m) {
      const int mm = m < m_real ? m : m_real - 1;
      xa[m] = ld16(x + mm * ldx + k);
      xb[m] = ld16(x + mm * ldx + k + 8);
    }
#pragma unroll
    for (int r = 0; r < 2; ++r) mac16<M>(wv[r], xa, xb, acc[r]);
  }
#pragma unroll
  for (int r = 0; r < 2; ++r)
#pragma unroll
    for (int m = 0; m < M; ++m) acc[r][m] = wave_sum(acc[r][m]);
#pragma unroll
  for (int r = 0; r < 2; ++r)
#pragma unroll
    for (int m = 0; m < M; ++m)
      if (lane == r * M + m) part[wave][r * M + m] = acc[r][m];
  __syncthreads();
  if (ks != 0 || lane >= M || lane >= m_real || pi >= p.npairs) return;
  const int m = lane;
  float s0 = part[wave][m], s1 = part[wave][M + m];
  for (int j = 1; j < ksplit; ++j) {
    s0 += part[wave + j][m];
    s1 += part[wave + j][M + m];
  }
  const bool has1 = r1 < N;
  const float x0 = round_bf(round_bf(s0) * bf_to_f(p.scales[r0]));
  const float x1 = has1 ? round_bf(round_bf(s1) * bf_to_f(p.scales[r1])) : 0.0f;
  u16* const yrow = p.y + (int64_t)m * p.ldy;
  if (p.pair_off) {  // rows (up, gate) of output column pi
    yrow[pi] = f_to_bf(swiglu_bf(x0, x1));
    return;
  }
  if (p.rope_table == nullptr) {
    yrow[r0] = f_to_bf(x0);
    if (has1) yrow[r1] = f_to_bf(x1);
    return;
  }
  // the fused q/k/v projection of a decode step (input row m is sequence m): what lr_rope_kv_write does to the
  // stored row, on the (even, odd) pair.  A position outside the cache or the table: the plain projection is
  // stored and the error word is set.
  const int hd = p.hd, nq = p.Hq * hd, nkv = p.Hkv * hd;
  const int ps = p.pos[0];
  const bool in_range = ps >= 0 && ps < p.Smax && ps < p.block_size;
  if (!in_range && p.err && pi == 0 && m == 0) *p.err = LR_DEV_POS_RANGE;
  u32 plain = pack_bf2(x0, x1), out = plain;
  if (in_range) {
    const int n = r0;
    const int sect = n < nq ? 0 : (n < nq + nkv ? 1 : 2);
    const int cc = n - (sect == 0 ? 0 : (sect == 1 ? nq : nq + nkv));
    const int h = cc / hd, d = cc - h * hd;
    if (sect < 2) {
#pragma clang fp contract(off)
      const u32 cs = *reinterpret_cast<const u32*>(p.rope_table + (int64_t)ps * hd + d);
      const float c = bf_lo(cs), sn = bf_hi(cs);
      const float a = x0 * c, b = x1 * sn, dd = x1 * c, ee = x0 * sn;
      out = pack_bf2(a - b, dd + ee);
    }
    if (sect == 0) plain = out;  // q is rotated in place; k and v stay as projected, the cache gets them
    if (sect == 1) *reinterpret_cast<u32*>(p.k_cache + (((int64_t)m * p.Hkv + h) * p.Smax + ps) * hd + d) = out;
    if (sect == 2) *reinterpret_cast<u32*>(p.v_cache + (((int64_t)m * p.Hkv + h) * p.Smax + ps) * hd + d) = plain;
  }
  *reinterpret_cast<u32*>(yrow + r0) = plain;
}

static int fill_p8(const lr_projection_fp8_t& q, P8& p) {
  LR_REQUIRE_PTR(q.x);
  LR_REQUIRE_PTR(q.w8);
  LR_REQUIRE_PTR(q.y);
  if (q.scales == nullptr) return LR_E_NULL;
  if (q.N <= 0 || q.K <= 0 || q.ldx < q.K) return LR_E_SHAPE;
  if (q.epilogue != LR_EPI_NONE && q.epilogue != LR_EPI_SWIGLU && q.epilogue != LR_EPI_ROPE_KV) return LR_E_SHAPE;
  const bool pair = q.epilogue == LR_EPI_SWIGLU;
  if (pair && q.N % 2) return LR_E_SHAPE;
  if (q.ldy < (pair ? q.N / 2 : q.N)) return LR_E_SHAPE;
  if (q.K % 16 || q.ldx % 8) return LR_E_ALIGN;
  p = P8{};
  p.x = (const u16*)q.x; p.w = (const unsigned char*)q.w8; p.scales = (const u16*)q.scales; p.y = (u16*)q.y;
  p.ldx = q.ldx; p.ldy = q.ldy; p.N = q.N; p.K = q.K;
  p.pair_off = pair ? q.N / 2 : 0;
  p.ksplit = q.K >= 4096 ? 4 : (q.K >= 2048 ? 2 : 1);  // as lr_linear_fp8 splits K
  p.npairs = pair ? q.N / 2 : (q.N + 1) / 2;
  const int per_wg = WPB / p.ksplit;
  p.nwg = (p.npairs + per_wg - 1) / per_wg;
  if (q.epilogue == LR_EPI_ROPE_KV) {
    const lr_rope_kv_t* r = q.rope;
    if (r == nullptr || r->pos == nullptr) return LR_E_NULL;
    LR_REQUIRE_PTR(r->table);
    LR_REQUIRE_PTR(r->k_cache);
    LR_REQUIRE_PTR(r->v_cache);
    if (r->n_head <= 0 || r->n_kv_head <= 0 || r->head_dim <= 0 || r->smax <= 0 || r->block_size <= 0 ||
        (int64_t)(r->n_head + 2 * r->n_kv_head) * r->head_dim != q.N || q.ldy % 2)
      return LR_E_SHAPE;
    if (r->head_dim % 8) return LR_E_ALIGN;
    p.rope_table = (const u16*)r->table; p.pos = r->pos; p.k_cache = (u16*)r->k_cache; p.v_cache = (u16*)r->v_cache;
    p.err = r->err; p.Hq = r->n_head; p.Hkv = r->n_kv_head; p.hd = r->head_dim; p.Smax = r->smax;
    p.block_size = r->block_size;
  }
  return LR_OK;
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

namespace lr_detail {
int stream_fp8_multi(const lr_projection_fp8_t* proj, int n_proj, int M, lr_stream_t stream);  // stream_gemm.hip
}

extern "C" size_t lr_linear_fp8_scratch_bytes(int M, int N, int K) {
  if (M <= 16 || N <= 0 || K <= 0) return 0;
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
  if (M > LR_FP8_GEMV_MAX_M && M <= 16 && !lr_misaligned(scales)) {
    // decode batches: the matrix-core bands of lr_linear_fp8_multi (one projection, no epilogue)
    const lr_projection_fp8_t one = {x, ldx, w8, scales, y, ldy, N, K, LR_EPI_NONE, nullptr};
    const int rc = lr_detail::stream_fp8_multi(&one, 1, M, stream);
    if (rc != LR_E_UNSUPPORTED || M > 8) return rc;
  }
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

extern "C" int lr_linear_fp8_multi(const lr_projection_fp8_t* proj, int n_proj, int M, lr_stream_t stream) {
  if (proj == nullptr) return LR_E_NULL;
  if (n_proj < 1 || n_proj > 2 || M < 1) return LR_E_SHAPE;
  if (M > 16) return LR_E_UNSUPPORTED;
  // from 2 rows on the matrix cores: the dot products of the matrix-vector kernel grow with every row
  if (M > LR_FP8_GEMV_MAX_M) return lr_detail::stream_fp8_multi(proj, n_proj, M, stream);
  P8 pr[2] = {};
  for (int i = 0; i < n_proj; ++i) {
    const int rc = fill_p8(proj[i], pr[i]);
    if (rc != LR_OK) return rc;
  }
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)(pr[0].nwg + pr[1].nwg)), block(WPB * 64);
  if (M == 1) k_gemv_fp8_multi<1><<<grid, block, 0, s>>>(pr[0], pr[1], M);
  else if (M == 2) k_gemv_fp8_multi<2><<<grid, block, 0, s>>>(pr[0], pr[1], M);
  else if (M <= 4) k_gemv_fp8_multi<4><<<grid, block, 0, s>>>(pr[0], pr[1], M);
  else k_gemv_fp8_multi<8><<<grid, block, 0, s>>>(pr[0], pr[1], M);
  return lr_launch_status();
}
