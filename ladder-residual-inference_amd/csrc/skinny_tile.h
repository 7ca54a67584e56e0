// The 32-row tile of the skinny matrix-core GEMM as a device function (k_gemm_skinny in gemm.hip is a thin
// wrapper around it).
#pragma once
#include "lr_common.h"

// ---------------------------------------------------------------------------------------------
// Skinny GEMM for decode batches (4 < M <= 64): the weights are streamed once, the few input rows
// ride along from L2.  y^T = W x^T on the matrix cores: A = 32 weight rows, B = input rows (MT / 32
// column tiles), so a lane ends up with 4 consecutive n of one m.  A workgroup owns 32 weight rows
// (N / 32 workgroups: every CU has work even for the 1280-row wqkv) and its 8 waves split K in
// 64-element chunks (wave w takes chunks w, w + 8, ...: together they read 1 KiB contiguous per
// row and round).  Both operands are loaded straight into the MFMA register layout (a lane's 8
// consecutive k of its row: 16 bytes), no LDS staging; each wave keeps PF chunks (PF x 4 KiB of
// weights) in flight, so a CU has 64+ KiB of weight loads outstanding -- what a latency-bound
// stream needs.  The waves' partial accumulators meet in LDS at the end, summed in a fixed order.
// ---------------------------------------------------------------------------------------------
constexpr int SN = 32;       // weight rows per workgroup
constexpr int SW = 8;        // waves per workgroup
constexpr int SCH = 64;      // k elements per chunk (4 MFMA k-steps)
constexpr int SPF = 2;       // chunks in flight per wave beyond the one being multiplied

// One 32-row tile [n0, n0 + 32) of y = x w^T, by a workgroup of SW waves.  `red`: SW * (MT / 32) * 16 * 64
// floats of LDS.
template <int MT>
__device__ __forceinline__ void skinny_tile(const u16* __restrict__ x, int64_t ldx, const u16* __restrict__ w,
                                            u16* __restrict__ y, int64_t ldy, int M, int N, int K, int n0,
                                            float* __restrict__ red) {
  constexpr int CT = MT / 32;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, half = lane >> 5;
  const int n = n0 + r;
  const bool nok = n < N;
  const u16* wrow = w + (int64_t)(nok ? n : 0) * K;
  const u16* xrow[CT];
  bool mok[CT];
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    mok[c] = c * 32 + r < M;
    xrow[c] = x + (int64_t)(mok[c] ? c * 32 + r : 0) * ldx;
  }
  f32x16_t acc[CT];
#pragma unroll
  for (int c = 0; c < CT; ++c)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[c][v] = 0.0f;

  struct Chunk {
    uint4 a[4];
    uint4 b[CT][4];
  };
  // buffer resources: weights based at this workgroup's first row, inputs at row 0
  const __amdgpu_buffer_rsrc_t wres =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<u16*>(w + (int64_t)n0 * K), 0, 0x7fffffff, 0x00020000);
  const __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc(const_cast<u16*>(x), 0, 0x7fffffff, 0x00020000);
  const int woff = r * K * 2;
  int xoff[CT];
#pragma unroll
  for (int c = 0; c < CT; ++c) xoff[c] = (int)((c * 32 + r) * ldx * 2);
  auto fetch = [&](int ci, Chunk& ch) {  // chunk index ci of this wave -> elements [k0, k0 + 64)
    const int k0 = (ci * SW + wave) * SCH;
#pragma unroll
    for (int s4 = 0; s4 < 4; ++s4) {
      const int k = k0 + s4 * 16 + half * 8;
      // no branch around a load: what lies beyond N, M or K gets an offset outside the buffer and reads
      // as zero, so the number of loads in flight is fixed and the waits between chunks are exact
      const bool kok = k < K;
      const u32x4_t av = __builtin_amdgcn_raw_buffer_load_b128(wres, (kok && nok) ? woff + k * 2 : (int)0x80000000, 0, 0);
      ch.a[s4] = make_uint4(av.x, av.y, av.z, av.w);
#pragma unroll
      for (int c = 0; c < CT; ++c) {
        const u32x4_t bv =
            __builtin_amdgcn_raw_buffer_load_b128(xres, (kok && mok[c]) ? xoff[c] + k * 2 : (int)0x80000000, 0, 0);
        ch.b[c][s4] = make_uint4(bv.x, bv.y, bv.z, bv.w);
      }
    }
  };
  auto mul = [&](const Chunk& ch) {
#pragma unroll
    for (int s4 = 0; s4 < 4; ++s4) {
      const u32x4_t av = {ch.a[s4].x, ch.a[s4].y, ch.a[s4].z, ch.a[s4].w};
#pragma unroll
      for (int c = 0; c < CT; ++c) {
        const u32x4_t bv = {ch.b[c][s4].x, ch.b[c][s4].y, ch.b[c][s4].z, ch.b[c][s4].w};
        acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, av), __builtin_bit_cast(bf16x8_t, bv),
                                                        acc[c], 0, 0, 0);
      }
    }
  };
  const int nch = (K + SW * SCH - 1) / (SW * SCH);  // chunks per wave (the tail is zero-filled)
  Chunk c0, c1, c2;
  fetch(0, c0);
  fetch(1, c1);
  int ci = 0;
  for (; ci + 3 <= nch; ci += 3) {  // three register sets rotate without copies
    fetch(ci + 2, c2);
    mul(c0);
    fetch(ci + 3, c0);
    mul(c1);
    fetch(ci + 4, c1);
    mul(c2);
  }
  if (ci < nch) mul(c0);
  if (ci + 1 < nch) mul(c1);
  static_assert(SPF == 2, "the loop above keeps two chunks in flight");

  // ---- sum the waves' partial accumulators in a fixed order
#pragma unroll
  for (int c = 0; c < CT; ++c)
#pragma unroll
    for (int v = 0; v < 16; ++v) red[((wave * CT + c) * 16 + v) * 64 + lane] = acc[c][v];
  __syncthreads();
  // wave w finishes accumulator elements v = 2 w, 2 w + 1: two consecutive n of one m per lane
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    float o[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int v = wave * 2 + j;
      float t = 0.0f;
#pragma unroll
      for (int ww = 0; ww < SW; ++ww) t += red[((ww * CT + c) * 16 + v) * 64 + lane];
      o[j] = t;
    }
    // element v: n = n0 + (v / 4) * 8 + (lane / 32) * 4 + v % 4,  m = c * 32 + lane % 32
    const int v0 = wave * 2;
    const int m = c * 32 + r, nn = n0 + (v0 / 4) * 8 + half * 4 + (v0 % 4);
    if (m < M) {
      if (nn + 1 < N) *reinterpret_cast<u32*>(y + (int64_t)m * ldy + nn) = pack_bf2(o[0], o[1]);
      else if (nn < N) y[(int64_t)m * ldy + nn] = f_to_bf(o[0]);
    }
  }
}
