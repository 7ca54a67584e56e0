// Attention over the contiguous [B, Hkv, Smax, hd] KV cache.
//
// Decode (one query per sequence): the valid keys 0..pos are cut into `nsplit` contiguous chunks;
// one workgroup per (chunk, kv head, sequence) serves ALL q heads of that kv head, so K and V are
// read from HBM once per GQA group.  Scores, softmax and P.V stay in fp32 (P is never rounded),
// chunk results carry their own (max, sum) and a second tiny kernel merges them in chunk order.
// Only slots <= pos are touched: with the reference's boolean mask the other slots get weight
// exp(-inf) = 0, so this is the same function of the cache.
//
// Prefill (S >= 16 queries per sequence): flash-style causal attention on the matrix cores in the
// transposed form (k_attn_prefill_mfma below: a query is a lane, four waves share K / V^T tiles in
// LDS, P enters the second product as bf16 hi + lo so the fp32 softmax weights survive).  Shorter
// inputs (1 < S < 16) use the older lane-per-query kernel (k_attn_prefill: running max / sum /
// output in registers, K/V tiles of 32 keys broadcast from LDS as fp32).  Both: exact fp32
// softmax semantics, one rounding of the output.
#include "lr_common.h"
#include "attn_decode_item.h"
#include <atomic>

// ------------------------------------------------------------------------------------ decode
extern "C" size_t lr_attn_decode_scratch_bytes(int B, int Hq, int hd, int Smax) {
  if (B <= 0 || Hq <= 0 || hd <= 0 || Smax <= 0) return 0;
  return (size_t)B * Hq * attn_nsplit_cap(Smax) * (hd + 2) * sizeof(float);
}

template <int HD, int G>
__global__ __launch_bounds__(256) void k_attn_decode_partial(const u16* __restrict__ q, int64_t ldq,
                                                             const u16* __restrict__ kc, const u16* __restrict__ vc,
                                                             const int32_t* __restrict__ pos_ptr,
                                                             float* __restrict__ o_part, float* __restrict__ ml_part,
                                                             int Hkv, int Smax, int nsplit, int chunk_max) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  attn_partial_item<HD, G, true>(q, ldq, kc, vc, pos_ptr, o_part, ml_part, Hkv, Smax, nsplit, chunk_max, blockIdx.x,
                           blockIdx.y, blockIdx.z, smem);
}

template <int HD, int G>
static int launch_decode(const u16* q, int64_t ldq, const u16* kc, const u16* vc, const int32_t* pos, u16* y,
                         int64_t ldy, int B, int Hkv, int Smax, float* scratch, hipStream_t s) {
  const int Hq = Hkv * G;
  const int nsplit = attn_pick_nsplit(B, Hkv, Smax);
  const int chunk_max = ((Smax + nsplit - 1) / nsplit + 3) & ~3;
  float* o_part = scratch;
  float* ml_part = scratch + (size_t)B * Hq * nsplit * HD;
  const size_t lds = (size_t)attn_item_lds_floats<HD, G>(chunk_max) * sizeof(float);
  static std::atomic<unsigned long long> lds_raised{0};
  if (!lr_raise_lds_limit(reinterpret_cast<const void*>(&k_attn_decode_partial<HD, G>), lds, lds_raised)) return LR_E_LAUNCH;
  k_attn_decode_partial<HD, G><<<dim3(nsplit, Hkv, B), dim3(256), lds, s>>>(q, ldq, kc, vc, pos, o_part, ml_part, Hkv,
                                                                            Smax, nsplit, chunk_max);
  launch_attn_combine<HD>(o_part, ml_part, y, ldy, Hq, B, nsplit, s);
  return lr_launch_status();
}

extern "C" int lr_attn_decode(const void* q, int64_t ldq, const void* k_cache, const void* v_cache,
                              const int32_t* pos, void* y, int64_t ldy, int B, int Hq, int Hkv, int hd, int Smax,
                              void* scratch, size_t scratch_bytes, lr_stream_t stream) {
  LR_REQUIRE_PTR(q);
  LR_REQUIRE_PTR(k_cache);
  LR_REQUIRE_PTR(v_cache);
  LR_REQUIRE_PTR(y);
  LR_REQUIRE_PTR(scratch);
  if (pos == nullptr) return LR_E_NULL;
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || hd <= 0 || Smax <= 0 || Hq % Hkv) return LR_E_SHAPE;
  if ((int64_t)Smax * hd * 2 >= 0x7fffffff) return LR_E_UNSUPPORTED;  // the rows of one (sequence, head) are addressed with 32-bit offsets
  if (ldq < (int64_t)Hq * hd || ldy < (int64_t)Hq * hd || B > 65535) return LR_E_SHAPE;
  if (ldq % 8 || ldy % 8) return LR_E_ALIGN;
  if (scratch_bytes < lr_attn_decode_scratch_bytes(B, Hq, hd, Smax)) return LR_E_SHAPE;
  const int G = Hq / Hkv;
  hipStream_t s = (hipStream_t)stream;
#define LR_DEC(HDV, GV)                                                                                           \
  if (hd == HDV && G == GV)                                                                                       \
    return launch_decode<HDV, GV>((const u16*)q, ldq, (const u16*)k_cache, (const u16*)v_cache, pos, (u16*)y, ldy, \
                                  B, Hkv, Smax, (float*)scratch, s);
  LR_DEC(128, 1) LR_DEC(128, 2) LR_DEC(128, 4) LR_DEC(128, 8) LR_DEC(128, 16)
  LR_DEC(64, 1) LR_DEC(64, 2) LR_DEC(64, 4) LR_DEC(64, 8)
#undef LR_DEC
  return LR_E_UNSUPPORTED;
}

// ------------------------------------------------------------------------------------ decode, allocation-free
// lr_attn_decode for callers that cannot allocate or carry a workspace: the split-KV partial
// results live in a fixed device array of this library instead of caller memory.  `scratch` below
// is, in host code, only a stand-in for the device symbol: the address kernels may use is looked
// up once per device with hipGetSymbolAddress (every device holds its own copy of the array at
// its own address) and kept in g_static_scratch; host code never passes `scratch` itself.
constexpr size_t LR_STATIC_SCRATCH_BYTES = LR_ATTN_DECODE_STATIC_MAX_BYTES;
static __device__ __align__(256) unsigned char scratch[LR_STATIC_SCRATCH_BYTES];
static std::atomic<float*> g_static_scratch[LR_MAX_DEVICES];

// device address of `scratch` on the current device (looked up on the first call per device)
static int static_scratch(float** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= LR_MAX_DEVICES) return LR_E_LAUNCH;
  float* p = g_static_scratch[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    void* sym = nullptr;
    if (hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch)) != hipSuccess || sym == nullptr) {
      (void)hipGetLastError();
      return LR_E_LAUNCH;
    }
    p = reinterpret_cast<float*>(sym);
    g_static_scratch[dev].store(p, std::memory_order_release);  // concurrent first calls store the same address
  }
  *out = p;
  return LR_OK;
}

extern "C" int lr_attn_decode_static(const void* q, int64_t ldq, const void* k_cache, const void* v_cache,
                                     const int32_t* pos, void* y, int64_t ldy, int B, int Hq, int Hkv, int hd,
                                     int Smax, lr_stream_t stream) {
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || hd <= 0 || Smax <= 0) return LR_E_SHAPE;
  const size_t need = lr_attn_decode_scratch_bytes(B, Hq, hd, Smax);
  if (need > LR_STATIC_SCRATCH_BYTES) return LR_E_TOO_LARGE;
  float* ws = nullptr;
  const int rc = static_scratch(&ws);
  if (rc != LR_OK) return rc;
  return lr_attn_decode(q, ldq, k_cache, v_cache, pos, y, ldy, B, Hq, Hkv, hd, Smax, ws, need, stream);
}

// ------------------------------------------------------------------------------------ prefill
template <int HD>
__global__ __launch_bounds__(64) void k_attn_prefill(const u16* __restrict__ q, int64_t ldq,
                                                     const u16* __restrict__ kc, const u16* __restrict__ vc,
                                                     const int32_t* __restrict__ pos, u16* __restrict__ y, int64_t ldy,
                                                     int S, int Hq, int Hkv, int Smax) {
  constexpr int TK = 32;
  __shared__ __attribute__((aligned(16))) float ks[TK * HD];
  __shared__ __attribute__((aligned(16))) float vs[TK * HD];
  const int lane = threadIdx.x;
  const int h = blockIdx.y, b = blockIdx.z;
  const int kvh = h / (Hq / Hkv);
  const int s = blockIdx.x * 64 + lane;
  const bool valid = s < S;
  int p = valid ? pos[s] : -1;
  p = p >= Smax ? Smax - 1 : p;
  int kmax = p;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const int t = __shfl_xor(kmax, o, LR_WAVE);
    kmax = t > kmax ? t : kmax;
  }
  const int nkeys = kmax + 1;

  float qf[HD];
  {
    const u16* qrow = q + ((int64_t)b * S + (valid ? s : 0)) * ldq + h * HD;
#pragma unroll
    for (int c = 0; c < HD; c += 8) unpack8(ld16(qrow + c), &qf[c]);
  }
  float o[HD];
#pragma unroll
  for (int d = 0; d < HD; ++d) o[d] = 0.0f;
  float m = -INFINITY, l = 0.0f;
  const float scale = rsqrtf((float)HD);
  const u16* kbase = kc + ((int64_t)b * Hkv + kvh) * Smax * HD;
  const u16* vbase = vc + ((int64_t)b * Hkv + kvh) * Smax * HD;

  for (int t0 = 0; t0 < nkeys; t0 += TK) {
    // stage TK keys and values as fp32: TK * HD / 8 chunks of 8 elements over 64 lanes
    __syncthreads();
#pragma unroll
    for (int i = 0; i < TK * HD / 8 / 64; ++i) {
      const int c = lane + i * 64;
      const int key = t0 + c / (HD / 8), d = (c % (HD / 8)) * 8;
      float kf[8], vf[8];
      if (key < nkeys) {
        unpack8(ld16(kbase + (int64_t)key * HD + d), kf);
        unpack8(ld16(vbase + (int64_t)key * HD + d), vf);
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) kf[j] = vf[j] = 0.0f;
      }
      float4* kd = reinterpret_cast<float4*>(&ks[(c / (HD / 8)) * HD + d]);
      float4* vd = reinterpret_cast<float4*>(&vs[(c / (HD / 8)) * HD + d]);
      kd[0] = make_float4(kf[0], kf[1], kf[2], kf[3]);
      kd[1] = make_float4(kf[4], kf[5], kf[6], kf[7]);
      vd[0] = make_float4(vf[0], vf[1], vf[2], vf[3]);
      vd[1] = make_float4(vf[4], vf[5], vf[6], vf[7]);
    }
    __syncthreads();

    float sc[TK];
    float tmax = -INFINITY;
#pragma unroll
    for (int j = 0; j < TK; ++j) {
      float a = 0.0f;
#pragma unroll
      for (int d = 0; d < HD; d += 4) {
        const float4 kk = *reinterpret_cast<const float4*>(&ks[j * HD + d]);
        a = fmaf(qf[d], kk.x, a);
        a = fmaf(qf[d + 1], kk.y, a);
        a = fmaf(qf[d + 2], kk.z, a);
        a = fmaf(qf[d + 3], kk.w, a);
      }
      sc[j] = (t0 + j <= p) ? a * scale : -INFINITY;
      tmax = fmaxf(tmax, sc[j]);
    }
    const float mn = fmaxf(m, tmax);
    if (mn != -INFINITY) {  // this lane sees at least one key so far
      const float corr = expf(m - mn);  // m == -inf -> 0
      l *= corr;
#pragma unroll
      for (int d = 0; d < HD; ++d) o[d] *= corr;
#pragma unroll
      for (int j = 0; j < TK; ++j) {
        const float pj = expf(sc[j] - mn);  // masked -> 0
        l += pj;
#pragma unroll
        for (int d = 0; d < HD; d += 4) {
          const float4 vv = *reinterpret_cast<const float4*>(&vs[j * HD + d]);
          o[d] = fmaf(pj, vv.x, o[d]);
          o[d + 1] = fmaf(pj, vv.y, o[d + 1]);
          o[d + 2] = fmaf(pj, vv.z, o[d + 2]);
          o[d + 3] = fmaf(pj, vv.w, o[d + 3]);
        }
      }
      m = mn;
    }
  }
  if (valid) {
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
    u16* yrow = y + ((int64_t)b * S + s) * ldy + h * HD;
#pragma unroll
    for (int c = 0; c < HD; c += 8) {
      float t[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) t[j] = o[c + j] * inv;
      st16(yrow + c, pack8(t));
    }
  }
}

// ----------------------------------------------------------------------- prefill on the matrix cores
// Flash-style causal attention in the TRANSPOSED form, so that everything per query sits in one lane:
//   S^T[key][q]  = sum_d K[key][d] Q[q][d]          (A = K tile from LDS, B = Q from registers)
//   O^T[d][q]   += sum_key V^T[d][key] P^T[key][q]  (A = V^T tile from LDS, B = P^T from the S^T registers)
// with v_mfma_f32_32x32x16_bf16.  An accumulator column is a query (lane % 32), so row maxima, sums and
// the rescaling factor are per-lane scalars; the 16 S^T values a lane holds for its query are exactly,
// in order, the B operand of the two PV k-steps (the key order of a k-step is free as long as the V^T
// operand uses the same one), so P never moves between lanes.  P enters the bf16 MFMA as hi + lo
// (p = bf16(p) + bf16(p - bf16(p))), which keeps the fp32 softmax weights to ~2^-17: the result matches
// the fp32 "math" attention of the eager reference (utils.py:247-258) to rounding of the final bf16.
// A workgroup is 4 waves = NWH heads of one kv head x NWQ tiles of 32 queries sharing the K / V tiles.
// e^x through the hardware exp2 (1 ulp in fp32: far below the bf16 rounding of the output), with the score scale
// folded into its argument; the library expf costs ~15 VALU instructions, and this kernel is VALU-bound next to
// its MFMAs
// max(a, b) as the median of {a, b, +inf}: one instruction (fmaxf makes the compiler canonicalise both operands
// first, an instruction each, when they come out of a matrix-core product).  Not for NaN operands.
// (No inline assembler here: the compiler does not count the wait states between a matrix-core instruction and
// an assembler statement that reads its result, and the statement then reads the registers too early.)
__device__ __forceinline__ float max_med3(float a, float b) { return __builtin_amdgcn_fmed3f(a, b, INFINITY); }
__device__ __forceinline__ float exp2_hw(float x) { return __builtin_amdgcn_exp2f(x); }
// two fp32 -> one dword of two bf16 (round to nearest even): a single v_cvt_pk_bf16_f32
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ u32 cvt_pk_bf2(float lo, float hi) {
  return __builtin_bit_cast(u32, __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t));
}
constexpr float PREFILL_TAU2 = 8.0f;  // log2 of the largest softmax weight before the reference point moves

template <int HD, int NWH>
__global__ __launch_bounds__(256) void k_attn_prefill_mfma(const u16* __restrict__ q, int64_t ldq,
                                                           const u16* __restrict__ kc, const u16* __restrict__ vc,
                                                           const int32_t* __restrict__ pos, u16* __restrict__ y,
                                                           int64_t ldy, int S, int Hq, int Hkv, int Smax) {
  constexpr int NWQ = 4 / NWH;            // query tiles per workgroup
  constexpr int KS = HD / 16;             // k-steps of the score product
  constexpr int DT = HD / 32;             // 32-row tiles of O^T
  constexpr int KROW = HD + 8;            // K tile row length in elements (16 B pad: conflict-free 128-bit reads)
  constexpr int VROW = 32 + 4;            // V^T tile row length in elements (8 B pad)
  __shared__ __attribute__((aligned(16))) u16 ks[32 * KROW];
  __shared__ __attribute__((aligned(16))) u16 vt[HD * VROW];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int col = lane & 31, half = lane >> 5;
  const int G = Hq / Hkv;
  const int hgroups = G / NWH;                       // workgroups per kv head along heads
  // Which (query block, head group, sequence) this workgroup takes.  The grid is one-dimensional and workgroup i
  // runs on XCD i % 8, each with an L2 of its own: XCD k takes the k-th eighth of the work in its logical order, so
  // that the workgroups that share the K / V rows of one (sequence, kv head) -- the query blocks, neighbours in that
  // order -- meet in one L2.  Inside, the query blocks go from the last (the longest history) to the first.
  const int gx = (S + 32 * NWQ - 1) / (32 * NWQ), gy = Hq / NWH;
  int wg;
  {
    const int n = gridDim.x, xcd = blockIdx.x % 8, idx = blockIdx.x / 8;
    const int base = n / 8, rem = n % 8;
    wg = xcd * base + (xcd < rem ? xcd : rem) + idx;
  }
  const int bx = gx - 1 - wg % gx, by = (wg / gx) % gy;
  const int b = wg / (gx * gy);
  const int kvh = by / hgroups;
  const int head = kvh * G + (by % hgroups) * NWH + (wave % NWH);
  const int s = (bx * NWQ + wave / NWH) * 32 + col;  // this lane's query
  const bool valid = s < S;
  int p = valid ? pos[s] : -1;
  p = p >= Smax ? Smax - 1 : p;
  // keys needed by anybody in the workgroup
  int kmax = p;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const int t = __shfl_xor(kmax, o, LR_WAVE);
    kmax = t > kmax ? t : kmax;
  }
  __shared__ int s_kmax[4];
  if (lane == 0) s_kmax[wave] = kmax;
  __syncthreads();
  kmax = max(max(s_kmax[0], s_kmax[1]), max(s_kmax[2], s_kmax[3]));
  const int nkeys = kmax + 1;

  // Q as B operands: k-step ks_ holds elements 16 ks_ + 8 half .. + 8 of this lane's query
  u32x4_t qb[KS];
  {
    const u16* qrow = q + ((int64_t)b * S + (valid ? s : 0)) * ldq + head * HD;
#pragma unroll
    for (int i = 0; i < KS; ++i) {
      const uint4 t = valid ? ld16(qrow + 16 * i + 8 * half) : make_uint4(0, 0, 0, 0);
      qb[i] = u32x4_t{t.x, t.y, t.z, t.w};
    }
  }
  f32x16_t o[DT];
#pragma unroll
  for (int d = 0; d < DT; ++d)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[d][v] = 0.0f;
  float m = -INFINITY, l = 0.0f;  // m: reference point in raw score units; l: this lane's half of the row sum
  const float c2 = rsqrtf((float)HD) * 1.4426950408889634f;  // e^(x / sqrt(HD)) = 2^(x c2)
  const float tau_raw = PREFILL_TAU2 / c2;
  // the smallest position among the wave's queries (lanes without a query do not count)
  int pmin = valid ? p : 0x7fffffff;
#pragma unroll
  for (int o_ = 32; o_ > 0; o_ >>= 1) {
    const int t = __shfl_xor(pmin, o_, LR_WAVE);
    pmin = t < pmin ? t : pmin;
  }
  pmin = __builtin_amdgcn_readfirstlane(pmin);
  const u16* kbase = kc + ((int64_t)b * Hkv + kvh) * Smax * HD;
  const u16* vbase = vc + ((int64_t)b * Hkv + kvh) * Smax * HD;

  // Staging: a thread owns one 8-element slice of TWO neighbouring keys (key pair kp, slice dch), so
  // that V^T can be written as whole dwords (two keys of one dimension).  The pair index is XOR-ed
  // with 4 * (dch / 4): slices 32 dimensions apart would otherwise fall on the same LDS banks (row
  // stride 18 dwords, 8 rows per slice).  The next tile's loads are in flight during the products.
  const int dch = tid % (HD / 8), kp = tid / (HD / 8);
  const bool stager = kp < 16;
  const int kps = kp ^ ((dch >> 2) * 4);
  // (buffer loads: a key beyond the needed range, or a thread without a staging slot, asks with an offset outside
  // the resource and gets zeros -- no branch around a load)
  u32x4_t gk[2], gv[2];
  const __amdgpu_buffer_rsrc_t kres = __builtin_amdgcn_make_buffer_rsrc(const_cast<u16*>(kbase), 0, 0x7fffffff, 0x00020000);
  const __amdgpu_buffer_rsrc_t vres = __builtin_amdgcn_make_buffer_rsrc(const_cast<u16*>(vbase), 0, 0x7fffffff, 0x00020000);
  const int stage_off = stager ? (2 * kp * HD + dch * 8) * 2 : (int)0x80000000;  // bytes, first key of the pair
  auto stage_load = [&](int t0) {
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int off = (stager && t0 + 2 * kp + e < nkeys) ? stage_off + (t0 + e) * HD * 2 : (int)0x80000000;
      gk[e] = __builtin_amdgcn_raw_buffer_load_b128(kres, off, 0, 0);
      gv[e] = __builtin_amdgcn_raw_buffer_load_b128(vres, off, 0, 0);
    }
  };
  stage_load(0);
  u32* vt32 = reinterpret_cast<u32*>(vt);
  for (int t0 = 0; t0 < nkeys; t0 += 32) {
    __syncthreads();
    // ---- 32 keys into LDS: K row-major, V transposed ([d][key], two keys per dword)
    if (stager) {
#pragma unroll
      for (int e = 0; e < 2; ++e) *reinterpret_cast<u32x4_t*>(&ks[(2 * kp + e) * KROW + dch * 8]) = gk[e];
      const u32 a4[4] = {gv[0][0], gv[0][1], gv[0][2], gv[0][3]}, b4[4] = {gv[1][0], gv[1][1], gv[1][2], gv[1][3]};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        vt32[(dch * 8 + 2 * j) * (VROW / 2) + kps] = (a4[j] & 0xffffu) | (b4[j] << 16);
        vt32[(dch * 8 + 2 * j + 1) * (VROW / 2) + kps] = (a4[j] >> 16) | (b4[j] & 0xffff0000u);
      }
    }
    __syncthreads();
    stage_load(t0 + 32);
    // ---- S^T tile: rows = keys, columns = queries
    f32x16_t sacc;
#pragma unroll
    for (int v = 0; v < 16; ++v) sacc[v] = 0.0f;
#pragma unroll
    for (int i = 0; i < KS; ++i) {
      const uint4 t = *reinterpret_cast<const uint4*>(&ks[col * KROW + 16 * i + 8 * half]);
      const u32x4_t ka = {t.x, t.y, t.z, t.w};
      sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, ka), __builtin_bit_cast(bf16x8_t, qb[i]),
                                                     sacc, 0, 0, 0);
    }
    // element v is key t0 + (v / 4) * 8 + half * 4 + v % 4 for query `col`; only a tile that reaches past the
    // smallest position of the wave's queries has anything to mask
    if (t0 + 31 > pmin) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int key = t0 + (v / 4) * 8 + half * 4 + (v % 4);
        sacc[v] = key <= p ? sacc[v] : -INFINITY;
      }
    }
    float tmax = max_med3(sacc[0], sacc[1]);
#pragma unroll
    for (int v = 2; v < 16; ++v) tmax = max_med3(tmax, sacc[v]);
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, LR_WAVE));
    // The reference point m of the exponentials follows the running maximum lazily: it moves only when a tile's
    // maximum exceeds it by more than PREFILL_TAU2 / c2, so the weights stay below 2^PREFILL_TAU2 (harmless in fp32,
    // and hi + lo keeps their relative precision) and the accumulators are rescaled on few tiles instead of on
    // most (with 32 queries per wave, some running maximum moves in the majority of tiles).
    const bool grow = tmax > m + tau_raw;  // m = -inf: any finite maximum
    const float mn = grow ? tmax : m;
    const float corr = grow ? exp2_hw((m - mn) * c2) : 1.0f;  // m = -inf -> 0
    const float nmc = mn == -INFINITY ? 0.0f : -mn * c2;     // nothing seen yet: every score is -inf, weight 0
    m = mn;
    l *= corr;
    u32x4_t phi[2], plo[2];
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float a0 = exp2_hw(fmaf(sacc[8 * h2 + 2 * j], c2, nmc));  // masked -> 0
        const float a1 = exp2_hw(fmaf(sacc[8 * h2 + 2 * j + 1], c2, nmc));
        l += a0 + a1;
        const u32 hi = cvt_pk_bf2(a0, a1);
        phi[h2][j] = hi;
        plo[h2][j] = cvt_pk_bf2(a0 - __uint_as_float(hi << 16), a1 - __uint_as_float(hi & 0xffff0000u));
      }
    // ---- O^T += V^T P^T ; k-step h2 covers keys 16 h2 + {0..3, 8..11} + 4 half, in the order of sacc
    const bool rescale = __any(grow);
    if (rescale) {
#pragma unroll
      for (int d = 0; d < DT; ++d)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[d][v] *= corr;
    }
    // (consecutive matrix instructions go to different accumulators: one that adds to the result of the instruction
    // right before it has to wait for that result)
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2) {
      // keys 16 h2 + 4 half + {0..3} and + 8 + {0..3}; rows of tile d were stored with pairs XOR 4 d
      u32x4_t va[DT];
#pragma unroll
      for (int d = 0; d < DT; ++d) {
        const u16* vr = &vt[(d * 32 + col) * VROW];
        const uint2 v0 = *reinterpret_cast<const uint2*>(vr + ((16 * h2 + 4 * half) ^ (8 * d)));
        const uint2 v1 = *reinterpret_cast<const uint2*>(vr + ((16 * h2 + 8 + 4 * half) ^ (8 * d)));
        va[d] = u32x4_t{v0.x, v0.y, v1.x, v1.y};
      }
#pragma unroll
      for (int d = 0; d < DT; ++d)
        o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, va[d]),
                                                       __builtin_bit_cast(bf16x8_t, phi[h2]), o[d], 0, 0, 0);
#pragma unroll
      for (int d = 0; d < DT; ++d)
        o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, va[d]),
                                                       __builtin_bit_cast(bf16x8_t, plo[h2]), o[d], 0, 0, 0);
    }
  }
  l += __shfl_xor(l, 32, LR_WAVE);
  if (valid) {
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
    u16* yrow = y + ((int64_t)b * S + s) * ldy + head * HD;
    // element v of tile d: dimension d * 32 + (v / 4) * 8 + half * 4 + v % 4
#pragma unroll
    for (int d = 0; d < DT; ++d)
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        uint2 w2;
        w2.x = pack_bf2(o[d][4 * g4] * inv, o[d][4 * g4 + 1] * inv);
        w2.y = pack_bf2(o[d][4 * g4 + 2] * inv, o[d][4 * g4 + 3] * inv);
        *reinterpret_cast<uint2*>(yrow + d * 32 + g4 * 8 + half * 4) = w2;
      }
  }
}

template <int HD>
static int launch_prefill_mfma(const u16* q, int64_t ldq, const u16* kc, const u16* vc, const int32_t* pos, u16* y,
                               int64_t ldy, int B, int S, int Hq, int Hkv, int Smax, hipStream_t s) {
  const int G = Hq / Hkv;
  if (G % 4 == 0) {
    k_attn_prefill_mfma<HD, 4><<<dim3((unsigned)((int64_t)((S + 31) / 32) * (Hq / 4) * B)), dim3(256), 0, s>>>(
        q, ldq, kc, vc, pos, y, ldy, S, Hq, Hkv, Smax);
  } else if (G % 2 == 0) {
    k_attn_prefill_mfma<HD, 2><<<dim3((unsigned)((int64_t)((S + 63) / 64) * (Hq / 2) * B)), dim3(256), 0, s>>>(
        q, ldq, kc, vc, pos, y, ldy, S, Hq, Hkv, Smax);
  } else {
    k_attn_prefill_mfma<HD, 1><<<dim3((unsigned)((int64_t)((S + 127) / 128) * Hq * B)), dim3(256), 0, s>>>(
        q, ldq, kc, vc, pos, y, ldy, S, Hq, Hkv, Smax);
  }
  return lr_launch_status();
}

extern "C" int lr_attn_prefill(const void* q, int64_t ldq, const void* k_cache, const void* v_cache,
                               const int32_t* pos, void* y, int64_t ldy, int B, int S, int Hq, int Hkv, int hd,
                               int Smax, lr_stream_t stream) {
  LR_REQUIRE_PTR(q);
  LR_REQUIRE_PTR(k_cache);
  LR_REQUIRE_PTR(v_cache);
  LR_REQUIRE_PTR(y);
  if (pos == nullptr) return LR_E_NULL;
  if (B <= 0 || S <= 0 || Hq <= 0 || Hkv <= 0 || hd <= 0 || Smax <= 0 || Hq % Hkv) return LR_E_SHAPE;
  if (ldq < (int64_t)Hq * hd || ldy < (int64_t)Hq * hd || B > 65535 || Hq > 65535) return LR_E_SHAPE;
  if (ldq % 8 || ldy % 8) return LR_E_ALIGN;
  const dim3 grid((S + 63) / 64, Hq, B);
  hipStream_t s = (hipStream_t)stream;
  if (S >= 16 && Hq <= 65535 * 4) {  // matrix-core kernel; the lane-per-query kernel below serves short inputs
    // (its staging addresses the rows of one (sequence, kv head) with 32-bit byte offsets)
    if ((hd == 128 || hd == 64) && (int64_t)Smax * hd * 2 >= 0x7fffffff) return LR_E_UNSUPPORTED;
    // (and its grid is one-dimensional, at most (S / 32) * Hq * B workgroups of 256 lanes: 2^32 lanes is the limit)
    if ((hd == 128 || hd == 64) && (int64_t)((S + 31) / 32) * Hq * B >= (1 << 24)) return LR_E_UNSUPPORTED;
    if (hd == 128)
      return launch_prefill_mfma<128>((const u16*)q, ldq, (const u16*)k_cache, (const u16*)v_cache, pos, (u16*)y, ldy,
                                      B, S, Hq, Hkv, Smax, s);
    if (hd == 64)
      return launch_prefill_mfma<64>((const u16*)q, ldq, (const u16*)k_cache, (const u16*)v_cache, pos, (u16*)y, ldy, B,
                                     S, Hq, Hkv, Smax, s);
  }
  if (hd == 128)
    k_attn_prefill<128><<<grid, dim3(64), 0, s>>>((const u16*)q, ldq, (const u16*)k_cache, (const u16*)v_cache, pos,
                                                  (u16*)y, ldy, S, Hq, Hkv, Smax);
  else if (hd == 64)
    k_attn_prefill<64><<<grid, dim3(64), 0, s>>>((const u16*)q, ldq, (const u16*)k_cache, (const u16*)v_cache, pos,
                                                 (u16*)y, ldy, S, Hq, Hkv, Smax);
  else
    return LR_E_UNSUPPORTED;
  return lr_launch_status();
}
