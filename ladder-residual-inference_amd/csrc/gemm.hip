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
#include <type_traits>

int lr_gemv_dispatch(const void* x, int64_t ldx, const void* w, void* y, int64_t ldy, int M, int N, int K,
                     int act_swiglu, int gemv_cfg, hipStream_t s);

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
// Large-tile variant for prefill-sized problems (M >= 512): workgroup tile 256 x 256 x 64, four
// waves in a 2 x 2 arrangement, each owning 128 x 128 = 4 x 4 MFMA tiles (256 accumulator
// registers; one workgroup per CU, so a wave has the whole 512-register budget).  The point is LDS
// traffic: a 64 x 64 wave tile reads 1 KiB of LDS per MFMA, which at 128 B/clk per CU takes as long
// as the MFMAs themselves; a 128 x 128 wave tile reads half of that.  Staging is the same as in
// k_gemm (128-bit global loads -> registers -> padded LDS rows, double-buffered, next tile's
// loads in flight during the multiply).  Tiles are dealt so that the 32 workgroups an XCD runs
// together cover 4 row tiles x 8 column tiles: they share operand rows in that XCD's L2
// (blockIdx % 8 is the XCD), which keeps the HBM demand ~5x below the L2 demand.
// ---------------------------------------------------------------------------------------------
constexpr int GM = 256, GN = 256;

// KTAIL: K is not a multiple of the 64-element k-tile, so the last tile needs a per-lane range check.  Without it the
// k position of a load is a scalar added by the load instruction itself and the row part of the address never
// changes: no vector instruction per load (with the check: add, select and a 16-register offset update per tile,
// ~60 vector instructions that the matrix instructions wait behind).
// ROPE: the projection is the fused q/k/v projection of a prefill (row b * S + s sits at position rpos[s]) and its
// output pass does what k_rope_kv_write would do to the stored rows: q rotated in y, rotated k and plain v into the
// caches, k and v left as projected in y; a position outside the cache or the table sets the error word and leaves
// the plain row.
struct GemmRope {
  int S, Hq, Hkv, hd, Smax, block_size;
};
template <bool KTAIL, bool ROPE>
__global__ __launch_bounds__(256) void k_gemm_big(const u16* __restrict__ x, int64_t ldx, const u16* __restrict__ w,
                                                  u16* __restrict__ y, int64_t ldy, int M, int N, int K, int tm,
                                                  int tn, int pair_off, const u16* __restrict__ rtable,
                                                  const int32_t* __restrict__ rpos, u16* __restrict__ rk,
                                                  u16* __restrict__ rv, int32_t* rerr, const GemmRope rp) {
  extern __shared__ __attribute__((aligned(16))) u16 gsm[];
  u16* xs = gsm;                      // [2][GM * LDT]
  u16* ws = gsm + 2 * GM * LDT;       // [2][GN * LDT]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  // ---- tile of this workgroup
  int mt, nt;
  {
    const int id = blockIdx.x;
    if (tm % 32 == 0) {  // XCD-aware: XCD x owns a band of tm / 8 row tiles, walked 4 row tiles x all column tiles at a time
      const int xcd = id & 7, j = id >> 3;
      const int per_group = 4 * tn;
      const int grp = j / per_group, r = j - grp * per_group;
      mt = xcd * (tm / 8) + grp * 4 + (r & 3);
      nt = r >> 2;
    } else {
      mt = id / tn;
      nt = id - mt * tn;
    }
  }
  // pair_off != 0: w holds [up; gate] rows (pair_off = number of pairs) and the tile covers 128 PAIRS: each wave's
  // 128 weight rows are 64 up rows followed by the 64 gate rows of the same pairs, so that a lane ends up with
  // both halves of a pair and stores bf16(bf16(silu(g)) * u) -- N is then the number of pairs
  const int m0 = mt * GM, n0 = nt * (pair_off ? GN / 2 : GN);

  // staging assignment: 2048 16-byte chunks per operand tile, 8 per thread
  f32x16_t acc[4][4];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.0f;

  const int srow0 = tid >> 3, scol = (tid & 7) * 8;  // chunk i sits 32 rows below chunk i - 1
  // Operand rows are read through buffer resources based at the tile's first row; a chunk beyond M,
  // N or K gets an offset outside the resource and reads as zero: no branches around the loads.
  const __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc(const_cast<u16*>(x + (int64_t)m0 * ldx), 0, 0x7fffffff, 0x00020000);
  const __amdgpu_buffer_rsrc_t wres = __builtin_amdgcn_make_buffer_rsrc(const_cast<u16*>(w + (int64_t)n0 * K), 0, 0x7fffffff, 0x00020000);
  int xoff[8], woff[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int r = srow0 + i * 32;
    xoff[i] = m0 + r < M ? (int)((int64_t)r * ldx * 2) : (int)0x80000000;
    if (pair_off) {
      const int wv = i >> 2, b = i & 3;                      // r = wv * 128 + b * 32 + srow0
      const int pr = wv * 64 + (b & 1) * 32 + srow0;          // pair inside the tile
      woff[i] = n0 + pr < N ? (int)((int64_t)((b >> 1) * pair_off + pr) * K * 2) : (int)0x80000000;
    } else {
      woff[i] = n0 + r < N ? r * K * 2 : (int)0x80000000;
    }
  }
  // k = first element of the k-tile (the same for all lanes); a tile beyond K is only ever requested, never used
  // (the two tiles asked for past the end): without the per-lane check it is replaced by the last real tile
  const int klast = ((K + BK - 1) / BK - 1) * BK;
  if (!KTAIL) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (xoff[i] >= 0) xoff[i] += scol * 2;
      if (woff[i] >= 0) woff[i] += scol * 2;
    }
  }
  auto fetch = [&](const __amdgpu_buffer_rsrc_t& res, int rowoff, int k) -> uint4 {
    u32x4_t v;
    if (KTAIL) {
      const int off = (k + scol < K && rowoff >= 0) ? rowoff + (k + scol) * 2 : (int)0x80000000;
      v = __builtin_amdgcn_raw_buffer_load_b128(res, off, 0, 0);
    } else {
      v = __builtin_amdgcn_raw_buffer_load_b128(res, rowoff, (k < klast ? k : klast) * 2, 0);
    }
    return make_uint4(v.x, v.y, v.z, v.w);
  };
  // Global -> LDS staging one tile ahead through ONE register set, in quarters: while tile kt is
  // multiplied, quarter q of tile kt + 1 (requested a whole iteration earlier, so it has landed) is
  // written to the other LDS buffer behind the MFMA group of k-step q, and the same registers are
  // at once refilled with quarter q of tile kt + 2.
  uint4 xr[8], wr[8];
  const int nk = (K + BK - 1) / BK;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    xr[i] = fetch(xres, xoff[i], 0);
    wr[i] = fetch(wres, woff[i], 0);
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    st16(&xs[(srow0 + i * 32) * LDT + scol], xr[i]);
    st16(&ws[(srow0 + i * 32) * LDT + scol], wr[i]);
  }
  // (requests beyond K read as zero: every load and LDS write below is unconditional, so the number of
  // loads in flight never depends on a branch and the waits can be exact)
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    xr[i] = fetch(xres, xoff[i], BK);
    wr[i] = fetch(wres, woff[i], BK);
  }
  __syncthreads();

  const int arow = lane & 31, akq = (lane >> 5) * 8;
  // Fragments of k-step ks + 1 are read from LDS while the matrix instructions of k-step ks run; those of the next
  // tile's k-step 0 during this tile's last k-step, behind the one workgroup barrier of the iteration.
  bf16x8_t af[2][4], bfr[2][4];
#pragma unroll
  for (int a = 0; a < 4; ++a) af[0][a] = *reinterpret_cast<const bf16x8_t*>(&xs[(wm * 128 + a * 32 + arow) * LDT + akq]);
#pragma unroll
  for (int b = 0; b < 4; ++b) bfr[0][b] = *reinterpret_cast<const bf16x8_t*>(&ws[(wn * 128 + b * 32 + arow) * LDT + akq]);
  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    const u16* xc = xs + cur * GM * LDT;
    const u16* wc = ws + cur * GN * LDT;
    u16* xn = xs + (cur ^ 1) * GM * LDT;
    u16* wn_ = ws + (cur ^ 1) * GN * LDT;
    const int k2 = (kt + 2) * BK;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      const int c = ks & 1, nx = c ^ 1;
      const bool last = ks + 1 == BK / 16;
      // One non-matrix instruction in the shadow of every matrix instruction (a wave issues in order: grouped, the
      // sixteen matrix instructions of a k-step would be followed by ~16 LDS / global instructions with the matrix
      // pipe idle).  K-steps 0..2: the eight fragment reads of the next k-step, the four LDS writes of the staged
      // quarter, the four global loads of the quarter after it.  Last k-step: the writes first, then the barrier
      // (every wave has written the next tile and has read all it needs of this one), the loads, and the fragment
      // reads of the NEXT tile's k-step 0 -- so that an iteration does not open with the matrix pipe waiting for LDS.
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int a4 = j >> 2, b4 = j & 3;
        acc[a4][b4] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[c][b4], af[c][a4], acc[a4][b4], 0, 0, 0);
        const int rd = last ? j - 8 : j;       // slot of the eight fragment reads
        const int wr_ = last ? j : j - 8;      // slot of the four LDS writes
        const int ft = last ? j - 4 : j - 12;  // slot of the four global loads
        if (rd >= 0 && rd < 8) {
          const u16* xf = last ? xn : xc;
          const u16* wf = last ? wn_ : wc;
          const int kk = last ? 0 : (ks + 1) * 16;
          if (rd < 4) af[nx][rd] = *reinterpret_cast<const bf16x8_t*>(&xf[(wm * 128 + rd * 32 + arow) * LDT + kk + akq]);
          else bfr[nx][rd - 4] = *reinterpret_cast<const bf16x8_t*>(&wf[(wn * 128 + (rd - 4) * 32 + arow) * LDT + kk + akq]);
        } else if (wr_ >= 0 && wr_ < 4) {
          const int i = 2 * ks + (wr_ >> 1);
          if ((wr_ & 1) == 0) st16(&xn[(srow0 + i * 32) * LDT + scol], xr[i]);
          else st16(&wn_[(srow0 + i * 32) * LDT + scol], wr[i]);
        } else if (ft >= 0 && ft < 4) {
          const int i = 2 * ks + (ft >> 1);
          if ((ft & 1) == 0) xr[i] = fetch(xres, xoff[i], k2);
          else wr[i] = fetch(wres, woff[i], k2);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (last && j == 3) {
          asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // LDS only: the global loads stay in flight
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  }

  // The products were formed as W-tile x X-tile^T, so accumulator element v of a 32 x 32 tile is
  // output column n = (v / 4) * 8 + (lane / 32) * 4 + v % 4 of output row m = lane % 32: a lane holds
  // four consecutive n of one row per group of four registers.  Stored from there, an instruction would
  // touch 16 bytes in each of 32 rows (32 partial cache lines, every line eight times per tile): the
  // tile's outputs take one trip through LDS instead (the operand tiles are dead; every wave has a piece
  // of its own) and leave as whole rows, an instruction covering 256 contiguous bytes of each of 4 rows
  // (128 bytes of 8 rows in pair mode).
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // nobody still reads the operand tiles
  u16* const eb = gsm + wave * (128 * (128 + 8));
  auto emit = [&](auto PAIR) {
    int lane = threadIdx.x & 63;  // (laundered: the addresses below are not formed before the k loop and kept through it)
    asm volatile("" : "+v"(lane));
    constexpr bool P = decltype(PAIR)::value;
    constexpr int WN = P ? 64 : 128;   // output columns of a wave
    constexpr int EP = WN + 8;         // row pitch of the wave's piece, in elements
    constexpr int LPR = WN / 8;        // lanes per row in the read-back
    constexpr int RPI = 64 / LPR;      // rows per instruction
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const int ml = a * 32 + (lane & 31);
#pragma unroll
      for (int b = 0; b < (P ? 2 : 4); ++b)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int nl = b * 32 + g * 8 + (lane >> 5) * 4;
          uint2 pk;
          if constexpr (P) {
            float o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = swiglu_bf(round_bf(acc[a][b][4 * g + e]), round_bf(acc[a][b + 2][4 * g + e]));
            pk.x = pack_bf2(o[0], o[1]);
            pk.y = pack_bf2(o[2], o[3]);
          } else {
            pk.x = pack_bf2(acc[a][b][4 * g], acc[a][b][4 * g + 1]);
            pk.y = pack_bf2(acc[a][b][4 * g + 2], acc[a][b][4 * g + 3]);
          }
          *reinterpret_cast<uint2*>(&eb[ml * EP + nl]) = pk;
        }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // a wave reads back only what it wrote itself
    const bool vec_ok = (ldy & 7) == 0;
    const int cl = (lane % LPR) * 8;
    const int ncol0 = n0 + wn * WN + cl;
    // ROPE: the lane's eight columns lie in one head of one section (head_dim % 8 == 0); its rows are RPI apart
    int rb = 0, rs = 0, sect = 0, hh = 0, dd = 0;
    if constexpr (ROPE && !P) {
      const int mfirst = m0 + wm * 128 + lane / LPR;
      rb = mfirst / rp.S;
      rs = mfirst - rb * rp.S;
      const int nq = rp.Hq * rp.hd, nkv = rp.Hkv * rp.hd;
      sect = ncol0 < nq ? 0 : (ncol0 < nq + nkv ? 1 : 2);
      const int cc = ncol0 - (sect == 0 ? 0 : (sect == 1 ? nq : nq + nkv));
      hh = cc / rp.hd;
      dd = cc - hh * rp.hd;
    }
    auto store_row = [&](int m, const uint4& v) {
      if (m < M) {
        if (vec_ok && ncol0 + 7 < N) {
          *reinterpret_cast<uint4*>(y + (int64_t)m * ldy + ncol0) = v;
        } else {
          const u32 q[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (ncol0 + e < N) y[(int64_t)m * ldy + ncol0 + e] = (u16)(q[e >> 1] >> ((e & 1) * 16));
        }
      }
    };
    if constexpr (ROPE && !P) {
      // Sixteen rows at a time: all their positions first, then all their table entries, then the arithmetic -- two
      // memory round trips per sixteen rows (row by row the position and the table entry it selects are a chain of
      // two dependent loads per row, and the output pass of a tile took three times as long).
      constexpr int RB = 16;
      for (int h0 = 0; h0 < 128 / RPI; h0 += RB) {
        int ps[RB], bb[RB];
#pragma unroll
        for (int i = 0; i < RB; ++i) {
          bb[i] = rb;
          const int m = m0 + wm * 128 + (h0 + i) * RPI + lane / LPR;
          ps[i] = (m < M && ncol0 < N) ? rpos[rs] : -1;  // (N % 8 == 0 and ldy % 8 == 0 here: the column group is whole)
          rs += RPI;
          while (rs >= rp.S) { rs -= rp.S; ++rb; }
        }
        uint4 tv[RB];
        bool ok[RB];
#pragma unroll
        for (int i = 0; i < RB; ++i) {
          ok[i] = ps[i] >= 0 && ps[i] < rp.Smax && ps[i] < rp.block_size;
          tv[i] = (ok[i] && sect < 2) ? ld16(rtable + (int64_t)ps[i] * rp.hd + dd) : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < RB; ++i) {
          const int ml = (h0 + i) * RPI + lane / LPR;
          const int m = m0 + wm * 128 + ml;
          uint4 v = *reinterpret_cast<const uint4*>(&eb[ml * EP + cl]);
          if (ok[i]) {
            const uint4 r = sect < 2 ? rope8(v, tv[i]) : v;
            if (sect == 0) v = r;
            else st16((sect == 1 ? rk : rv) + (((int64_t)bb[i] * rp.Hkv + hh) * rp.Smax + ps[i]) * rp.hd + dd, r);
          } else if (m < M && ncol0 < N && rerr && cl == 0 && wn == 0) {
            *rerr = LR_DEV_POS_RANGE;
          }
          store_row(m, v);
        }
      }
      return;
    }
#pragma unroll 4
    for (int r0 = 0; r0 < 128; r0 += RPI) {
      const int ml = r0 + lane / LPR;
      store_row(m0 + wm * 128 + ml, *reinterpret_cast<const uint4*>(&eb[ml * EP + cl]));
    }
  };
  if (pair_off) emit(std::true_type{});
  else emit(std::false_type{});
}

// pair_off != 0: N counts [up; gate] row pairs (see the kernel); rope != nullptr: the q/k/v projection of a prefill
// of S tokens per sequence (pair_off == 0, ldy % 8 == 0)
template <bool KTAIL, bool ROPE>
static int launch_gemm_big_as(const void* x, int64_t ldx, const void* w, void* y, int64_t ldy, int M, int N, int K,
                              int pair_off, const lr_rope_kv_t* rope, int S, hipStream_t s) {
  constexpr size_t lds = (size_t)2 * (GM + GN) * LDT * sizeof(u16);
  static std::atomic<unsigned long long> lds_raised{0};
  if (!lr_raise_lds_limit(reinterpret_cast<const void*>(&k_gemm_big<KTAIL, ROPE>), lds, lds_raised)) return LR_E_LAUNCH;
  const int gn = pair_off ? GN / 2 : GN;
  const int tm = (M + GM - 1) / GM, tn = (N + gn - 1) / gn;
  GemmRope rp = {};
  if (ROPE) rp = GemmRope{S, rope->n_head, rope->n_kv_head, rope->head_dim, rope->smax, rope->block_size};
  k_gemm_big<KTAIL, ROPE><<<dim3((unsigned)(tm * tn)), dim3(256), lds, s>>>(
      (const u16*)x, ldx, (const u16*)w, (u16*)y, ldy, M, N, K, tm, tn, pair_off, ROPE ? (const u16*)rope->table : nullptr,
      ROPE ? rope->pos : nullptr, ROPE ? (u16*)rope->k_cache : nullptr, ROPE ? (u16*)rope->v_cache : nullptr,
      ROPE ? rope->err : nullptr, rp);
  return lr_launch_status();
}

static int launch_gemm_big(const void* x, int64_t ldx, const void* w, void* y, int64_t ldy, int M, int N, int K,
                           int pair_off, hipStream_t s, const lr_rope_kv_t* rope = nullptr, int S = 0) {
  const bool ktail = K % BK != 0;
  if (rope)
    return ktail ? launch_gemm_big_as<true, true>(x, ldx, w, y, ldy, M, N, K, pair_off, rope, S, s)
                 : launch_gemm_big_as<false, true>(x, ldx, w, y, ldy, M, N, K, pair_off, rope, S, s);
  return ktail ? launch_gemm_big_as<true, false>(x, ldx, w, y, ldy, M, N, K, pair_off, nullptr, 0, s)
               : launch_gemm_big_as<false, false>(x, ldx, w, y, ldy, M, N, K, pair_off, nullptr, 0, s);
}

extern "C" int lr_linear_tuned(const void* x, int64_t ldx, const void* w, void* y, int64_t ldy, int M, int N, int K,
                               int act_swiglu, int gemv_cfg, lr_stream_t stream) {
  LR_REQUIRE_PTR(x);
  LR_REQUIRE_PTR(w);
  LR_REQUIRE_PTR(y);
  if (M <= 0 || N <= 0 || K <= 0) return LR_E_SHAPE;
  if (ldx < (act_swiglu ? 2 : 1) * (int64_t)K || ldy < N) return LR_E_SHAPE;
  if (K % 8 || ldx % 8) return LR_E_ALIGN;
  hipStream_t s = (hipStream_t)stream;
  if (M <= 4 || ((act_swiglu || gemv_cfg) && M <= 8))
    return lr_gemv_dispatch(x, ldx, w, y, ldy, M, N, K, act_swiglu, gemv_cfg, s);
  if (!act_swiglu && M <= 64) {
    // decode batches: the weight-streaming matrix-core kernel (stream_gemm.hip); shapes it declines fall through
    lr_projection_t pr;
    pr.x = x; pr.ldx = ldx; pr.w = w; pr.y = y; pr.ldy = ldy; pr.N = N; pr.K = K; pr.epilogue = LR_EPI_NONE; pr.rope = nullptr;
    const int rc = lr_linear_multi(&pr, 1, M, stream);
    if (rc != LR_E_UNSUPPORTED) return rc;
  }
  if (!act_swiglu && M >= 512 && N >= 256 && ((M + GM - 1) / GM) * ((N + GN - 1) / GN) >= 192 &&
      (int64_t)GM * ldx * 2 < 0x7fffffff && (int64_t)GN * K * 2 < 0x7fffffff)
    return launch_gemm_big(x, ldx, w, y, ldy, M, N, K, 0, s);
  const dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  if (grid.y > 65535) return LR_E_UNSUPPORTED;
  if (act_swiglu)
    k_gemm<true><<<grid, dim3(256), 0, s>>>((const u16*)x, ldx, (const u16*)w, (u16*)y, ldy, M, N, K);
  else
    k_gemm<false><<<grid, dim3(256), 0, s>>>((const u16*)x, ldx, (const u16*)w, (u16*)y, ldy, M, N, K);
  return lr_launch_status();
}

extern "C" int lr_linear(const void* x, int64_t ldx, const void* w, void* y, int64_t ldy, int M, int N, int K,
                         int act_swiglu, lr_stream_t stream) {
  return lr_linear_tuned(x, ldx, w, y, ldy, M, N, K, act_swiglu, 0, stream);
}

// The fused q/k/v projection of M = B * S rows (S tokens per sequence, row b * S + s at position pos[s]) finished as
// lr_rope_kv_write would finish it.  One launch where the 256 x 256-tile GEMM applies; otherwise the two calls.
extern "C" int lr_linear_rope_kv(const void* x, int64_t ldx, const void* w, void* y, int64_t ldy, int M, int K, int S,
                                 const lr_rope_kv_t* rope, lr_stream_t stream) {
  LR_REQUIRE_PTR(x);
  LR_REQUIRE_PTR(w);
  LR_REQUIRE_PTR(y);
  if (rope == nullptr || rope->pos == nullptr) return LR_E_NULL;
  LR_REQUIRE_PTR(rope->table);
  LR_REQUIRE_PTR(rope->k_cache);
  LR_REQUIRE_PTR(rope->v_cache);
  if (M <= 0 || K <= 0 || S <= 0 || M % S) return LR_E_SHAPE;
  if (rope->n_head <= 0 || rope->n_kv_head <= 0 || rope->head_dim <= 0 || rope->smax <= 0 || rope->block_size <= 0)
    return LR_E_SHAPE;
  const int64_t n64 = (int64_t)(rope->n_head + 2 * rope->n_kv_head) * rope->head_dim;
  if (n64 > 0x7fffffff || ldx < K || ldy < n64) return LR_E_SHAPE;
  if (K % 8 || ldx % 8 || ldy % 8 || rope->head_dim % 8) return LR_E_ALIGN;
  const int N = (int)n64;
  hipStream_t s = (hipStream_t)stream;
  if (M >= 512 && N >= 256 && ((M + GM - 1) / GM) * ((N + GN - 1) / GN) >= 192 && (int64_t)GM * ldx * 2 < 0x7fffffff &&
      (int64_t)GN * K * 2 < 0x7fffffff)
    return launch_gemm_big(x, ldx, w, y, ldy, M, N, K, 0, s, rope, S);
  const int rc = lr_linear(x, ldx, w, y, ldy, M, N, K, 0, stream);
  if (rc != LR_OK) return rc;
  return lr_rope_kv_write(y, ldy, rope->table, 0, rope->pos, rope->k_cache, rope->v_cache, M / S, S, rope->n_head,
                          rope->n_kv_head, rope->head_dim, rope->smax, rope->block_size, rope->err, stream);
}

// y[M, I] = bf16( bf16(silu(g)) * u ) for [u | g] = x w^T with w = [up; gate] rows (N = 2 I): the MLP's first
// projection with the activation applied on the way out (utils.py:145-148 without the [M, 2 I] tensor).
extern "C" int lr_linear_swiglu_out(const void* x, int64_t ldx, const void* w, void* y, int64_t ldy, int M, int N, int K,
                                    void* scratch, size_t scratch_bytes, lr_stream_t stream) {
  LR_REQUIRE_PTR(x);
  LR_REQUIRE_PTR(w);
  LR_REQUIRE_PTR(y);
  if (M <= 0 || N <= 0 || K <= 0 || N % 2 || ldx < K || ldy < N / 2) return LR_E_SHAPE;
  if (K % 8 || ldx % 8) return LR_E_ALIGN;
  const int I = N / 2;
  if (M <= 64) {
    lr_projection_t pr;
    pr.x = x; pr.ldx = ldx; pr.w = w; pr.y = y; pr.ldy = ldy; pr.N = N; pr.K = K; pr.epilogue = LR_EPI_SWIGLU; pr.rope = nullptr;
    const int rc = lr_linear_multi(&pr, 1, M, stream);
    if (rc != LR_E_UNSUPPORTED) return rc;
  }
  if (M >= 512 && I >= 128 && ((M + GM - 1) / GM) * ((I + GN / 2 - 1) / (GN / 2)) >= 192 &&
      (int64_t)GM * ldx * 2 < 0x7fffffff && ((int64_t)I + GN) * K * 2 < 0x7fffffff)
    return launch_gemm_big(x, ldx, w, y, ldy, M, I, K, I, (hipStream_t)stream);
  // other sizes: the projection into `scratch` [M, N], then the activation
  LR_REQUIRE_PTR(scratch);
  if (scratch_bytes < (size_t)M * N * sizeof(u16)) return LR_E_SHAPE;
  if (ldy != I) return LR_E_UNSUPPORTED;  // lr_swiglu writes dense rows
  const int rc = lr_linear(x, ldx, w, scratch, N, M, N, K, 0, stream);
  if (rc != LR_OK) return rc;
  return lr_swiglu(scratch, N, y, M, I, stream);
}
