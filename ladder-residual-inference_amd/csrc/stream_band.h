// The band of the weight-streaming matrix-core kernel as a device function, and what its callers share on the host
// (stream_gemm.hip launches bands only; decode_pair.hip runs decode-attention items beside them).
#pragma once
#include "lr_common.h"

namespace {


constexpr int KC = 128;        // k elements per chunk
constexpr int NWV = 4;         // waves per workgroup
constexpr int SETS = 4;        // weight chunks in flight per wave
constexpr int LROW = KC + 8;   // LDS row length in elements (272 bytes)
constexpr int OOB = (int)0x80000000;  // a buffer offset beyond every resource: the load returns zero, untouched memory
// Input rows from which a band reads the inputs in whole cache lines (through LDS) rather than in fragment layout:
// always with the 32- and 64-row bands; the 16-row band has both forms and the launcher picks by the row count
// (70B rank shard, ms per step, fragment layout / whole lines: 4 rows 4.99 / 5.12, 8 rows 5.14 / 5.19, 16 rows
// 6.26 / 6.00; 8B, 16 rows: 4.00 / 3.78)
constexpr int XLDS_MIN_MT = 32;       // band heights that always read their inputs in whole lines
constexpr int XLDS_M16_FROM = 9;      // input rows from which the 16-row band does too
constexpr int AUX_WEIGHTS = 2;        // weights: non-temporal (every line is used exactly once)

#ifdef LR_BAND_PROFILE
// Profile builds only: when set (lr_band_profile, stream_gemm.hip), every wave of every band records 100 MHz
// wall-clock stamps at six points -- 0 entry, 1 first requests made, 2 first chunk in LDS, 3 end of the K loop,
// 4 partial sums exchanged (second barrier), 5 end -- at [(workgroup * NWV + wave) * 8 + point].
static __device__ unsigned long long* g_band_prof;
static __device__ unsigned g_band_prof_wgs;  // workgroups the buffer has room for; the others record nothing
#define LR_BAND_STAMP(k)                                                                              \
  if (g_band_prof && blockIdx.x < g_band_prof_wgs && lane == 0)                                       \
    g_band_prof[((size_t)blockIdx.x * NWV + wave) * 8 + (k)] = wall_clock64();
#else
#define LR_BAND_STAMP(k)
#endif

struct Proj {
  const u16* x;
  const u16* w;
  u16* y;
  int64_t ldx, ldy;
  int N, K;      // weight rows, row length
  int rpw;       // rows (row pairs if pair_off) per workgroup
  int pair_off;  // 0, or the distance from an up row to its gate row (= outputs)
  int nwg;       // workgroups of this projection
  const u16* scales;  // weight-only e4m3 weights (the W8 kernels): one bf16 scale per weight row; else nullptr
  // RoPE + KV-cache epilogue of a fused q/k/v projection (rope_table == nullptr: none)
  const u16* rope_table;
  const int32_t* pos;
  u16 *k_cache, *v_cache;
  int32_t* err;
  int Hq, Hkv, hd, Smax, block_size;
};

// the low (HI == false) or high two e4m3 values of a dword as a packed bf16 pair (exact)
template <bool HI>
__device__ __forceinline__ u32 sb_fp8_pair(u32 v) {
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  return __builtin_bit_cast(u32, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(v, 1.0f, HI));
}

template <int MT, int UNITS, bool W8 = false, bool XL = (MT >= XLDS_MIN_MT)>
constexpr size_t stream_band_lds_bytes() {
  constexpr int LRW = (W8 ? 2 * KC : KC) + 8;
  return (size_t)NWV * (UNITS * 16 * LRW + (XL ? MT * LRW : 0)) * sizeof(u16);
}

// One band of one projection, by the 256 lanes of a workgroup.  `sg_smem`: stream_band_lds_bytes<MT, UNITS>() bytes of LDS.
// W8: the weights are e4m3 bytes with one bf16 scale per row (p.scales): a load instruction still covers 4 rows x
// 256 bytes, now 256 elements of K, which are expanded to bf16 (exactly: e4m3 is a subset of bf16) on their way
// into the LDS piece; the sum is rounded to bf16, multiplied by the row's scale and rounded again, as
// F.linear(x, w.to(bf16)) * scales does, before the epilogue sees it.
template <int MT, int UNITS, bool W8 = false, bool XL = (MT >= XLDS_MIN_MT)>
__device__ __forceinline__ void stream_band(const Proj& p, const int M, const int band, u16* sg_smem) {
  static_assert(!W8 || MT == 16, "the e4m3 path is built for up to 16 input rows");
  constexpr int KCW = W8 ? 256 : 128;  // k elements per chunk
  constexpr int LRW = KCW + 8;         // LDS row length in elements
  constexpr int WB = W8 ? 1 : 2;       // bytes per weight
  // weight chunks in flight per wave: the e4m3 variant has twice the A fragments and input registers per chunk
  // and gives up two of its four sets for a second workgroup per CU
  constexpr int NS = W8 ? 2 : SETS;
  constexpr int MTILES = MT / 16, KS = KCW / 32, NLD = UNITS * 4;
  constexpr int NV = UNITS * MTILES * 4;  // accumulator registers per lane
  // XL: the inputs too are loaded in whole lines (4 rows x 256 bytes per instruction) and take the trip through
  // LDS into B-fragment layout: L2 serves whole-line reads 1.5 times as fast as the 16 rows x 64 bytes a
  // fragment-layout load touches, and at 64 rows the input bytes are twice the weight bytes.
  constexpr bool XLDS = XL;
  static_assert(!(XL && W8), "the e4m3 band reads its inputs in fragment layout");
  constexpr int WPIECE = UNITS * 16 * LRW, XPIECE = XLDS ? MT * LRW : 0;  // elements per wave
  // sg_smem: [NWV][WPIECE + XPIECE]
  static_assert(sizeof(float) * NV * 64 <= sizeof(u16) * WPIECE, "the partial sums reuse the wave's weight piece");

  const u16* const xg = p.x;
  const u16* const wg_ = p.w;
  u16* const yg = p.y;
  const int64_t ldx = p.ldx, ldy = p.ldy;
  const int N = p.N, K = p.K, rpw = p.rpw;
  const int pair_off = p.pair_off;
  const u16* const rope_table = p.rope_table;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15, l4 = lane >> 4;
  LR_BAND_STAMP(0)
  const int n_out = pair_off ? pair_off : N;         // output columns
  const int n0 = band * rpw;                          // first row (pair) of the band
  const int nrows = n_out - n0 < rpw ? n_out - n0 : rpw;

  // ---- lane constants of the weight loads: instruction i covers band rows 4 i .. 4 i + 3 (in pair mode
  //      unit 0 holds the up rows, unit 1 the gate rows of the same pairs)
  const __amdgpu_buffer_rsrc_t wres =
      __builtin_amdgcn_make_buffer_rsrc(
          const_cast<unsigned char*>(reinterpret_cast<const unsigned char*>(wg_) + (int64_t)n0 * K * WB), 0, 0x7fffffff,
          0x00020000);
  const __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc(const_cast<u16*>(xg), 0, 0x7fffffff, 0x00020000);
  int woff[NLD];
#pragma unroll
  for (int i = 0; i < NLD; ++i) {
    const int r = 4 * i + l4;  // row inside the LDS piece
    int rr = r, extra = 0;
    if (pair_off && r >= 16) { rr = r - 16; extra = pair_off; }
    woff[i] = rr < nrows ? (int)((int64_t)(extra + rr) * K * WB + l16 * 16) : OOB;
  }
  // fragment layout: tile mt, k-step ks <- input row 16 mt + lane % 16, elements 32 ks + 8 (lane / 16) ..;
  // whole-line layout: instruction i <- input rows 4 i + lane / 16, elements 8 (lane % 16) ..
  int xoff[XLDS ? MT / 4 : MTILES];
  if (XLDS) {
#pragma unroll
    for (int i = 0; i < MT / 4; ++i) {
      const int m = 4 * i + l4;
      xoff[i] = m < M ? (int)((m * ldx + l16 * 8) * 2) : OOB;
    }
  } else {
#pragma unroll
    for (int mt = 0; mt < MTILES; ++mt) {
      const int m = mt * 16 + l16;
      xoff[mt] = m < M ? (int)((m * ldx + l4 * 8) * 2) : OOB;
    }
  }
  u16* const my = sg_smem + wave * (WPIECE + XPIECE);
  u16* const myx = my + WPIECE;

  u32x4_t wr[NS][NLD];
  u32x4_t xr[2][MTILES][KS];
  f32x4_t acc[UNITS][MTILES];
#pragma unroll
  for (int u = 0; u < UNITS; ++u)
#pragma unroll
    for (int mt = 0; mt < MTILES; ++mt) acc[u][mt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};

  // chunk ci of this wave starts at k0 = (ci * NWV + wave) * KCW; what lies beyond K reads as zero (no
  // branch around a load: the number of loads in flight is fixed, so the waits between chunks are exact).
  // (Every band walks K from 0, so the whole grid asks for the same 4 KiB window of its rows at the same time.
  // Starting band b `b % chunks` chunks in, wrapping around, spreads that over the DRAM channels: 16-row bands
  // 1.5 % faster per step, 64-row bands 8 % slower -- their inputs come from L2, which likes the common window.
  // Not kept: the order of a sum would then depend on how the rows are cut into bands.)
  auto issue_w = [&](int ci, u32x4_t (&dst)[NLD]) {
    const int k0 = (ci * NWV + wave) * KCW;
    const bool kok = k0 + l16 * (16 / WB) < K;
#pragma unroll
    for (int i = 0; i < NLD; ++i)
      dst[i] = __builtin_amdgcn_raw_buffer_load_b128(wres, (kok && woff[i] != OOB) ? woff[i] : OOB, k0 * WB, AUX_WEIGHTS);
  };
  auto issue_x = [&](int ci, u32x4_t (&dst)[MTILES][KS]) {
    const int k0 = (ci * NWV + wave) * KCW;
    if (XLDS) {
      const bool kok = k0 + l16 * 8 < K;
#pragma unroll
      for (int i = 0; i < MT / 4; ++i)
        dst[i / KS][i % KS] =
            __builtin_amdgcn_raw_buffer_load_b128(xres, (kok && xoff[i] != OOB) ? xoff[i] : OOB, k0 * 2, 0);
      return;
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const bool kok = k0 + ks * 32 + l4 * 8 < K;
#pragma unroll
      for (int mt = 0; mt < MTILES; ++mt)
        dst[mt][ks] = __builtin_amdgcn_raw_buffer_load_b128(xres, (kok && xoff[mt] != OOB) ? xoff[mt] : OOB,
                                                           (k0 + ks * 32) * 2, 0);
    }
  };

  const int nck = (K + KCW - 1) / KCW;
  const int nch = wave < nck ? (nck - wave + NWV - 1) / NWV : 0;  // chunks of this wave
  // (the fences keep the requests in this order: the wait for chunk 0 counts the requests made after it, and the
  // scheduler, left alone, asks for chunk 0 last -- the loop then waited for all but the last 8 requests at the top
  // of every round of NS chunks)
  issue_x(0, xr[0]);
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    asm volatile("" ::: "memory");
    issue_w(s, wr[s]);
  }
  asm volatile("" ::: "memory");
  LR_BAND_STAMP(1)
  for (int c0 = 0; c0 < nch; c0 += NS) {
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      const int ci = c0 + s;
      issue_x(ci + 1, xr[(s + 1) & 1]);
      // ---- this chunk's weights: registers -> LDS (row-major) -> A fragments
      asm volatile("" ::: "memory");
#pragma unroll
      for (int i = 0; i < NLD; ++i) {
        if constexpr (W8) {
          u32x4_t lo, hi;
          lo[0] = sb_fp8_pair<false>(wr[s][i][0]); lo[1] = sb_fp8_pair<true>(wr[s][i][0]);
          lo[2] = sb_fp8_pair<false>(wr[s][i][1]); lo[3] = sb_fp8_pair<true>(wr[s][i][1]);
          hi[0] = sb_fp8_pair<false>(wr[s][i][2]); hi[1] = sb_fp8_pair<true>(wr[s][i][2]);
          hi[2] = sb_fp8_pair<false>(wr[s][i][3]); hi[3] = sb_fp8_pair<true>(wr[s][i][3]);
          *reinterpret_cast<u32x4_t*>(my + (4 * i + l4) * LRW + l16 * 16) = lo;
          *reinterpret_cast<u32x4_t*>(my + (4 * i + l4) * LRW + l16 * 16 + 8) = hi;
        } else {
          *reinterpret_cast<u32x4_t*>(my + (4 * i + l4) * LRW + l16 * 8) = wr[s][i];
        }
      }
      asm volatile("" ::: "memory");
#ifdef LR_BAND_PROFILE
      if (ci == 0) { LR_BAND_STAMP(2) }
#endif
      if constexpr (W8) {
        // 256 elements of K per chunk: the A fragments are taken in two halves to keep them at 32 registers
        issue_w(ci + NS, wr[s]);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          bf16x8_t ah[UNITS][KS / 2];
#pragma unroll
          for (int u = 0; u < UNITS; ++u)
#pragma unroll
            for (int k2 = 0; k2 < KS / 2; ++k2)
              ah[u][k2] =
                  *reinterpret_cast<const bf16x8_t*>(my + (16 * u + l16) * LRW + (h * (KS / 2) + k2) * 32 + l4 * 8);
#pragma unroll
          for (int k2 = 0; k2 < KS / 2; ++k2)
#pragma unroll
            for (int mt = 0; mt < MTILES; ++mt) {
              const bf16x8_t bx = __builtin_bit_cast(bf16x8_t, xr[s & 1][mt][h * (KS / 2) + k2]);
#pragma unroll
              for (int u = 0; u < UNITS; ++u)
                acc[u][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah[u][k2], bx, acc[u][mt], 0, 0, 0);
            }
        }
        asm volatile("" ::: "memory");
        continue;
      }
      bf16x8_t af[UNITS][KS];
#pragma unroll
      for (int u = 0; u < UNITS; ++u)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
          af[u][ks] = *reinterpret_cast<const bf16x8_t*>(my + (16 * u + l16) * LRW + ks * 32 + l4 * 8);
      asm volatile("" ::: "memory");
      issue_w(ci + NS, wr[s]);
      if (XLDS) {
#pragma unroll
        for (int i = 0; i < MT / 4; ++i)
          *reinterpret_cast<u32x4_t*>(myx + (4 * i + l4) * LRW + l16 * 8) = xr[s & 1][i / KS][i % KS];
        asm volatile("" ::: "memory");
      }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int mt = 0; mt < MTILES; ++mt) {
          bf16x8_t bx;
          if (XLDS) bx = *reinterpret_cast<const bf16x8_t*>(myx + (16 * mt + l16) * LRW + ks * 32 + l4 * 8);
          else bx = __builtin_bit_cast(bf16x8_t, xr[s & 1][mt][ks]);
#pragma unroll
          for (int u = 0; u < UNITS; ++u)
            acc[u][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[u][ks], bx, acc[u][mt], 0, 0, 0);
        }
      if (XLDS) asm volatile("" ::: "memory");
    }
  }

  LR_BAND_STAMP(3)
  // ---- the waves' partial sums meet in LDS (accumulator element e of tile (u, mt): band row
  //      16 u + 4 (lane / 16) + e, input row 16 mt + lane % 16) and are added in wave order
  __syncthreads();
  float* const red = reinterpret_cast<float*>(sg_smem);
  constexpr int WSTRIDE = (WPIECE + XPIECE) / 2;  // floats per wave piece
#pragma unroll
  for (int u = 0; u < UNITS; ++u)
#pragma unroll
    for (int mt = 0; mt < MTILES; ++mt)
#pragma unroll
      for (int e = 0; e < 4; ++e) red[wave * WSTRIDE + ((u * MTILES + mt) * 4 + e) * 64 + lane] = acc[u][mt][e];
  __syncthreads();
  LR_BAND_STAMP(4)
  const int rows_out = pair_off ? 16 : 16 * UNITS;
  if (rope_table != nullptr) {
    // The fused q/k/v projection of a decode step (one token per sequence: input row m is sequence m):
    // what lr_rope_kv_write would do to the stored row, done here on the (even, odd) output pairs.  A
    // position outside the cache or the table: the plain projection is stored, the error word is set.
    const Proj& pp = p;
    const int hd = pp.hd, nq = pp.Hq * hd, nkv = pp.Hkv * hd;
    const int ps = pp.pos[0];
    const bool in_range = ps >= 0 && ps < pp.Smax && ps < pp.block_size;
    if (!in_range && pp.err && band == 0 && tid == 0) *pp.err = LR_DEV_POS_RANGE;
    for (int o = tid; o < (rows_out / 2) * MT; o += NWV * 64) {
      const int r = 2 * (o % (rows_out / 2)), m = o / (rows_out / 2);
      if (r >= nrows || m >= M) continue;
      const int mt = m >> 4, ln = ((r & 15) >> 2) * 16 + (m & 15), e = r & 3, u = r >> 4;
      float s0 = 0.0f, s1 = 0.0f;
#pragma unroll
      for (int wv = 0; wv < NWV; ++wv) {
        s0 += red[wv * WSTRIDE + ((u * MTILES + mt) * 4 + e) * 64 + ln];
        s1 += red[wv * WSTRIDE + ((u * MTILES + mt) * 4 + e + 1) * 64 + ln];
      }
      const int n = n0 + r;
      float x0 = round_bf(s0), x1 = round_bf(s1);
      if constexpr (W8) {
        x0 = round_bf(x0 * bf_to_f(pp.scales[n]));
        x1 = round_bf(x1 * bf_to_f(pp.scales[n + 1]));
      }
      u32 plain = pack_bf2(x0, x1), out = plain;
      if (in_range) {
        const int sect = n < nq ? 0 : (n < nq + nkv ? 1 : 2);
        const int cc = n - (sect == 0 ? 0 : (sect == 1 ? nq : nq + nkv));
        const int h = cc / hd, d = cc - h * hd;
        if (sect < 2) {
#pragma clang fp contract(off)
          const u32 cs = *reinterpret_cast<const u32*>(rope_table + (int64_t)ps * hd + d);
          const float c = bf_lo(cs), sn = bf_hi(cs);
          const float a = x0 * c, b = x1 * sn, dd = x1 * c, ee = x0 * sn;
          out = pack_bf2(a - b, dd + ee);
        }
        if (sect == 0) plain = out;  // q is rotated in place; k and v stay as projected, the cache gets them
        if (sect == 1) *reinterpret_cast<u32*>(pp.k_cache + (((int64_t)m * pp.Hkv + h) * pp.Smax + ps) * hd + d) = out;
        if (sect == 2) *reinterpret_cast<u32*>(pp.v_cache + (((int64_t)m * pp.Hkv + h) * pp.Smax + ps) * hd + d) = plain;
      }
      *reinterpret_cast<u32*>(yg + (int64_t)m * ldy + n) = plain;
    }
    LR_BAND_STAMP(5)
    return;
  }
  for (int o = tid; o < rows_out * MT; o += NWV * 64) {
    const int r = o % rows_out, m = o / rows_out;
    if (r >= nrows || m >= M) continue;
    const int mt = m >> 4, ln = ((r & 15) >> 2) * 16 + (m & 15), e = r & 3, u = r >> 4;
    float s0 = 0.0f, s1 = 0.0f;
#pragma unroll
    for (int wv = 0; wv < NWV; ++wv) s0 += red[wv * WSTRIDE + ((u * MTILES + mt) * 4 + e) * 64 + ln];
    if (pair_off) {
      if (UNITS == 2) {
#pragma unroll
        for (int wv = 0; wv < NWV; ++wv) s1 += red[wv * WSTRIDE + ((MTILES + mt) * 4 + e) * 64 + ln];
      }
      float u_ = round_bf(s0), g_ = round_bf(s1);
      if constexpr (W8) {
        u_ = round_bf(u_ * bf_to_f(p.scales[n0 + r]));
        g_ = round_bf(g_ * bf_to_f(p.scales[pair_off + n0 + r]));
      }
      yg[(int64_t)m * ldy + n0 + r] = f_to_bf(swiglu_bf(u_, g_));
    } else if constexpr (W8) {
      yg[(int64_t)m * ldy + n0 + r] = f_to_bf(round_bf(s0) * bf_to_f(p.scales[n0 + r]));
    } else {
      yg[(int64_t)m * ldy + n0 + r] = f_to_bf(s0);
    }
  }
  LR_BAND_STAMP(5)
}

// Rows per workgroup: the rows are spread evenly over whole rounds of the CUs, at most `cap` per
// workgroup; with few weight rows and many input rows a band is not made thinner than `floor_rows`
// (every band re-reads all input rows from L2).
static void plan(Proj& p, int M, int cap, int ncu) {
  // (the RoPE epilogue works on output pairs: bands of an even number of rows)
  const int items = p.pair_off ? p.pair_off : p.N;
  const int rounds = (items + ncu * cap - 1) / (ncu * cap);
  int rpw = (items + ncu * rounds - 1) / (ncu * rounds);
  const int floor_rows = M > 32 ? 16 : (M > 16 ? 8 : 4);
  if (rpw < floor_rows) rpw = floor_rows;
  if (p.rope_table) rpw = (rpw + 1) & ~1;
  if (rpw > cap) rpw = cap;
  p.rpw = rpw;
  p.nwg = (items + rpw - 1) / rpw;
}

// lr_projection_t -> Proj (validated; rpw / nwg are set by plan())
static int sb_fill_projection(const lr_projection_t& q, Proj& p) {
  LR_REQUIRE_PTR(q.x);
  LR_REQUIRE_PTR(q.w);
  LR_REQUIRE_PTR(q.y);
  if (q.N <= 0 || q.K <= 0 || q.ldx < q.K) return LR_E_SHAPE;
  if (q.epilogue != LR_EPI_NONE && q.epilogue != LR_EPI_SWIGLU && q.epilogue != LR_EPI_ROPE_KV) return LR_E_SHAPE;
  const bool pair = q.epilogue == LR_EPI_SWIGLU;
  if (pair && q.N % 2) return LR_E_SHAPE;
  if (q.ldy < (pair ? q.N / 2 : q.N)) return LR_E_SHAPE;
  if (q.K % 8 || q.ldx % 8) return LR_E_ALIGN;
  // offsets inside a band and inside the input rows are 32-bit
  if ((int64_t)64 * q.ldx * 2 >= 0x7fffffff || ((int64_t)(pair ? q.N / 2 : 0) + 64) * q.K * 2 >= 0x7fffffff)
    return LR_E_UNSUPPORTED;
  p = Proj{};
  p.x = (const u16*)q.x; p.w = (const u16*)q.w; p.y = (u16*)q.y;
  p.ldx = q.ldx; p.ldy = q.ldy; p.N = q.N; p.K = q.K;
  p.pair_off = pair ? q.N / 2 : 0;
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

// lr_projection_fp8_t -> Proj for the e4m3 bands (W8 = true)
static int sb_fill_projection_fp8(const lr_projection_fp8_t& q, Proj& p) {
  if (q.scales == nullptr) return LR_E_NULL;
  if (lr_misaligned(q.w8)) return LR_E_ALIGN;
  if (q.K % 16) return LR_E_ALIGN;
  // the bf16 projection's checks, with the weight pointer standing in (its rows are half as long: every
  // 32-bit offset limit holds a fortiori)
  const lr_projection_t as_bf16 = {q.x, q.ldx, q.w8, q.y, q.ldy, q.N, q.K, q.epilogue, q.rope};
  const int rc = sb_fill_projection(as_bf16, p);
  if (rc != LR_OK) return rc;
  p.scales = (const u16*)q.scales;
  return LR_OK;
}

}  // namespace
