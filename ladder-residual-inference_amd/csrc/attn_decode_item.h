#pragma once
#include "lr_common.h"

// ---- how the valid keys are cut into chunks (one workgroup item per chunk, kv head and sequence).
//      A chunk never exceeds ATT_CHUNK keys: the item then requests all of its K and V rows at once.
constexpr int ATT_CHUNK = 256;
constexpr int ATT_NCU = 256;  // CUs of the MI355X

static inline int attn_nsplit_cap(int Smax) {
  const int by_len = (Smax + ATT_CHUNK - 1) / ATT_CHUNK;
  return by_len > 64 ? by_len : 64;
}

static inline int attn_pick_nsplit(int B, int Hkv, int Smax) {
  const int cap = attn_nsplit_cap(Smax);
  int n = (512 + B * Hkv - 1) / (B * Hkv);   // aim at >= 512 workgroups
  const int by_work = (Smax + 63) / 64;      // but at least ~64 keys per chunk at full length
  if (n > by_work) n = by_work;
  const int by_len = (Smax + ATT_CHUNK - 1) / ATT_CHUNK;
  if (n < by_len) n = by_len;
  if (n < 1) n = 1;
  if (n > cap) n = cap;
  // With more items than CUs the slowest CU sets the time: among the neighbouring chunk counts take the one
  // whose items fill whole rounds of the 256 CUs best (64 sequences: 12 chunks = 768 items instead of 9 = 576).
  // (beyond four rounds the gain is smaller than the cost of more chunks to merge)
  if ((int64_t)n * B * Hkv >= ATT_NCU && (int64_t)n * B * Hkv < 4 * ATT_NCU) {
    int best = n;
    int64_t best_num = 0, best_den = 1;  // padded / real items of the best candidate
    const int lo = n - 3 > by_len ? n - 3 : by_len, hi = n + 3 < cap ? n + 3 : cap;
    for (int c = lo < 1 ? 1 : lo; c <= hi; ++c) {
      const int64_t items = (int64_t)c * B * Hkv, padded = (items + ATT_NCU - 1) / ATT_NCU * ATT_NCU;
      if (best_num == 0 || padded * best_den < best_num * items) { best = c; best_num = padded; best_den = items; }
    }
    n = best;
  }
  return n;
}

// LDS row length of the score buffer: whole 16-key tiles, plus 4 so that the 16 heads a tile's scores are
// written for do not share a bank
__host__ __device__ constexpr int attn_sc_ld(int chunk_max) { return ((chunk_max + 15) & ~15) + 4; }

// One (split, kv head, sequence) item of the split-KV decode attention, by 256 lanes (4 waves): scores,
// softmax statistics and the un-normalised P.V of keys [k0, k1) (at most ATT_CHUNK) for all G q heads of
// the kv head.  `smem`: attn_item_lds_floats<HD, G>(chunk_max) floats of LDS.  (A kv head with more q heads than
// an instantiation takes can be served as kv_share groups of G: every head's result is the same either way.)
//
// Every K and V row of the chunk is requested before anything else -- whole rows, 1 KiB contiguous per
// wave instruction, up to 32 KiB per wave in flight -- so the item costs one memory round trip.  Scores
// run on the matrix cores: a 16-key tile of K takes a trip through a wave-private piece of LDS (written
// row-major as loaded, read back as v_mfma_f32_16x16x32_bf16 A fragments, rows padded by 16 bytes), the
// q heads are the B operand (loaded straight into fragment layout, heads beyond G are zero columns).
// Softmax statistics and P.V stay in fp32 on the vector units: a lane owns 8 output elements of one key
// group, so the inner loop has no cross-lane traffic.
template <int HD, int G>
__host__ __device__ constexpr int attn_item_lds_floats(int chunk_max) {
  return (4 * G * HD > 32 * (HD + 8) ? 4 * G * HD : 32 * (HD + 8)) + G * attn_sc_ld(chunk_max) + 2 * G + 4;
}

// EAGER: every request is a buffer load whose offset lies outside the buffer for what is not wanted (it reads as
// zero), q first.  Written as `wanted ? load : 0` each load sits in a branch of its own, and the copy that merges
// one of them with its zero makes the compiler wait for everything in flight in the middle of the sequence: two
// memory round trips per item instead of one (70B shard, 64 sequences: 9.83 -> 9.43 ms per step; 8B, 16 sequences:
// 3.63 -> 3.57).  With short chunks beside a weight stream (8 sequences of the 70B shard: one tile of four per wave
// holds keys) the branches are the better neighbour (5.05 against 5.11 ms): the caller chooses.
template <int HD, int G, bool EAGER = false>
__device__ __forceinline__ void attn_partial_item(const u16* __restrict__ q, int64_t ldq, const u16* __restrict__ kc,
                                                  const u16* __restrict__ vc, const int32_t* __restrict__ pos_ptr,
                                                  float* __restrict__ o_part, float* __restrict__ ml_part, int Hkv,
                                                  int Smax, int nsplit, int chunk_max, int split, int kvh, int b,
                                                  float* __restrict__ smem, int kv_share = 1) {
  static_assert(G <= 16, "the q heads of a kv head are the 16 columns of one matrix-core tile");
  constexpr int LPK = HD / 8;    // lanes that share one key row (8 elements each)
  constexpr int KPW = 64 / LPK;  // keys per wave instruction
  constexpr int NI = 16 / KPW;   // instructions per 16-key tile
  constexpr int KS = HD / 32;    // matrix-core k-steps per row
  constexpr int TPW = ATT_CHUNK / 64;  // tiles per wave
  constexpr int LROW = HD + 8;   // LDS row length of the K piece, in elements
  constexpr int REGION = 4 * G * HD > 32 * LROW ? 4 * G * HD : 32 * LROW;
  float* ored = smem;                         // [4][G][HD]   (after the scores)
  u16* kpiece = reinterpret_cast<u16*>(smem);  // [4 waves][16][LROW] bf16 (during the scores)
  float* sc = smem + REGION;                  // [G][ldsc]
  const int ldsc = attn_sc_ld(chunk_max);
  float* s_m = sc + G * ldsc;                 // [G]
  float* s_l = s_m + G;                       // [G]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int Hq = Hkv * G;
  int nkeys = pos_ptr[0] + 1;
  nkeys = nkeys < 0 ? 0 : (nkeys > Smax ? Smax : nkeys);
  const int chunk = (nkeys + nsplit - 1) / nsplit;
  const int k0 = split * chunk;
  const int k1 = k0 + chunk < nkeys ? k0 + chunk : nkeys;
  const int n = k1 - k0;  // <= chunk_max <= ATT_CHUNK by construction

  float* o_out = o_part + (((int64_t)b * Hq + kvh * G) * nsplit + split) * HD;  // + g * nsplit * HD
  float* ml_out = ml_part + (((int64_t)b * Hq + kvh * G) * nsplit + split) * 2;  // + g * nsplit * 2
  if (n <= 0) {
    for (int i = tid; i < G * HD; i += 256) o_out[(int64_t)(i / HD) * nsplit * HD + (i % HD)] = 0.0f;
    if (tid < G) {
      ml_out[(int64_t)tid * nsplit * 2] = -INFINITY;
      ml_out[(int64_t)tid * nsplit * 2 + 1] = 0.0f;
    }
    return;
  }

  const int kl = lane / LPK, dl = (lane % LPK) * 8;
  // kv_share > 1: `Hkv` and `kvh` count groups of G q heads, kv_share of them on one head of the cache
  const u16* kbase = kc + ((int64_t)b * (Hkv / kv_share) + kvh / kv_share) * Smax * HD;
  const u16* vbase = vc + ((int64_t)b * (Hkv / kv_share) + kvh / kv_share) * Smax * HD;
  const float scale = rsqrtf((float)HD);
  // wave w owns the 16-key tiles w, w + 4, ...; instruction i of a tile covers keys i * KPW .. + KPW
  // q as B fragments: column = head lane % 16, k-step ks holds elements ks * 32 + (lane / 16) * 8 .. + 8
  const int l16 = lane & 15, l4 = lane >> 4;
  uint4 kr[TPW][NI], vr[TPW][NI];
  bf16x8_t qf[KS];
  if constexpr (EAGER) {
    constexpr int OOB_ = (int)0x80000000;
    const __amdgpu_buffer_rsrc_t kres = __builtin_amdgcn_make_buffer_rsrc(const_cast<u16*>(kbase), 0, 0x7fffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t vres = __builtin_amdgcn_make_buffer_rsrc(const_cast<u16*>(vbase), 0, 0x7fffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t qres = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<u16*>(q + (int64_t)b * ldq + (int64_t)kvh * G * HD), 0, 0x7fffffff, 0x00020000);
    auto bld = [](const __amdgpu_buffer_rsrc_t& r, int off) {
      const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0);
      return make_uint4(v.x, v.y, v.z, v.w);
    };
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const uint4 v = bld(qres, l16 < G ? (l16 * HD + ks * 32 + l4 * 8) * 2 : OOB_);
      const u32x4_t vv = {v.x, v.y, v.z, v.w};
      qf[ks] = __builtin_bit_cast(bf16x8_t, vv);
    }
#pragma unroll
    for (int j = 0; j < TPW; ++j)
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int key = k0 + (j * 4 + wave) * 16 + i * KPW + kl;
        kr[j][i] = bld(kres, key < k1 ? (key * HD + dl) * 2 : OOB_);
      }
#pragma unroll
    for (int j = 0; j < TPW; ++j)
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int key = k0 + (j * 4 + wave) * 16 + i * KPW + kl;
        vr[j][i] = bld(vres, key < k1 ? (key * HD + dl) * 2 : OOB_);
      }
  } else {
#pragma unroll
    for (int j = 0; j < TPW; ++j)
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int key = k0 + (j * 4 + wave) * 16 + i * KPW + kl;
        kr[j][i] = key < k1 ? ld16(kbase + (int64_t)key * HD + dl) : make_uint4(0, 0, 0, 0);
      }
#pragma unroll
    for (int j = 0; j < TPW; ++j)
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int key = k0 + (j * 4 + wave) * 16 + i * KPW + kl;
        vr[j][i] = key < k1 ? ld16(vbase + (int64_t)key * HD + dl) : make_uint4(0, 0, 0, 0);
      }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const uint4 v = l16 < G ? ld16(q + (int64_t)b * ldq + (kvh * G + l16) * HD + ks * 32 + l4 * 8) : make_uint4(0, 0, 0, 0);
      const u32x4_t vv = {v.x, v.y, v.z, v.w};
      qf[ks] = __builtin_bit_cast(bf16x8_t, vv);
    }
  }

  // ---- scores: S[key][head] = sum_d K[key][d] q[head][d] on the matrix cores
  {
    u16* my = kpiece + wave * 16 * LROW;
#pragma unroll
    for (int j = 0; j < TPW; ++j) {
      const int t16 = (j * 4 + wave) * 16;  // first key of the tile, relative to k0
      if (t16 < n) {  // uniform
        asm volatile("" ::: "memory");
#pragma unroll
        for (int i = 0; i < NI; ++i) st16(my + (i * KPW + kl) * LROW + dl, kr[j][i]);
        asm volatile("" ::: "memory");
        f32x4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const bf16x8_t af = *reinterpret_cast<const bf16x8_t*>(my + l16 * LROW + ks * 32 + l4 * 8);
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, qf[ks], acc, 0, 0, 0);
        }
        asm volatile("" ::: "memory");
        // accumulator element e: key t16 + 4 (lane / 16) + e, head lane % 16 (keys beyond n: never read)
        if (l16 < G)
          *reinterpret_cast<float4*>(sc + l16 * ldsc + t16 + 4 * l4) =
              make_float4(acc[0] * scale, acc[1] * scale, acc[2] * scale, acc[3] * scale);
      }
    }
  }
  __syncthreads();

  // ---- softmax statistics per head; sc becomes exp(s - max)
  for (int g = wave; g < G; g += 4) {
    float m = -INFINITY;
    for (int i = lane; i < n; i += 64) m = fmaxf(m, sc[g * ldsc + i]);
    m = wave_max(m);
    float l = 0.0f;
    for (int i = lane; i < n; i += 64) {
      const float p = expf(sc[g * ldsc + i] - m);
      sc[g * ldsc + i] = p;
      l += p;
    }
    l = wave_sum(l);
    if (lane == 0) { s_m[g] = m; s_l[g] = l; }
  }
  __syncthreads();

  // ---- P.V
  {
    float acc[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[g][j] = 0.0f;
#pragma unroll
    for (int j = 0; j < TPW; ++j) {
      const int t16 = (j * 4 + wave) * 16;
      if (t16 < n) {  // uniform
#pragma unroll
        for (int i = 0; i < NI; ++i) {
          const int kk = t16 + i * KPW + kl;  // relative to k0
          if (kk < n) {
            float vf[8];
            unpack8(vr[j][i], vf);
#pragma unroll
            for (int g = 0; g < G; ++g) {
              const float p = sc[g * ldsc + kk];
#pragma unroll
              for (int e = 0; e < 8; ++e) acc[g][e] = fmaf(p, vf[e], acc[g][e]);
            }
          }
        }
      }
    }
    // fold the KPW key groups of the wave, then the four waves through LDS (fixed order)
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float v = acc[g][j];
#pragma unroll
        for (int o = LPK; o < 64; o <<= 1) v += __shfl_xor(v, o, LR_WAVE);
        acc[g][j] = v;
      }
    if (kl == 0) {
#pragma unroll
      for (int g = 0; g < G; ++g)
#pragma unroll
        for (int j = 0; j < 8; ++j) ored[(wave * G + g) * HD + dl + j] = acc[g][j];
    }
  }
  __syncthreads();
  for (int i = tid; i < G * HD; i += 256) {
    const float v = (ored[i] + ored[G * HD + i]) + (ored[2 * G * HD + i] + ored[3 * G * HD + i]);
    o_out[(int64_t)(i / HD) * nsplit * HD + (i % HD)] = v;
  }
  if (tid < G) {
    ml_out[(int64_t)tid * nsplit * 2] = s_m[tid];
    ml_out[(int64_t)tid * nsplit * 2 + 1] = s_l[tid];
  }
}

// ---- merge of the chunk results: y = sum_s w_s o_s with w_s = exp(m_s - max) / sum_s' exp(m_s' - max) l_s'
template <int HD>
__global__ __launch_bounds__(HD) void k_attn_decode_combine(const float* __restrict__ o_part,
                                                            const float* __restrict__ ml_part, u16* __restrict__ y,
                                                            int64_t ldy, int Hq, int nsplit) {
  const int h = blockIdx.x, b = blockIdx.y, d = threadIdx.x;
  const float* ml = ml_part + ((int64_t)b * Hq + h) * nsplit * 2;
  const float* op = o_part + ((int64_t)b * Hq + h) * nsplit * HD;
  // branch-free loops, unrolled: the loads of eight splits are in flight together instead of one
  // dependent round trip per split
  float M = -INFINITY;
#pragma unroll 8
  for (int s = 0; s < nsplit; ++s) M = fmaxf(M, ml[2 * s]);
  float L = 0.0f, o = 0.0f;
#pragma unroll 8
  for (int s = 0; s < nsplit; ++s) {
    const float m = ml[2 * s];
    const float wgt = m == -INFINITY ? 0.0f : expf(m - M);  // an empty split carries (-inf, 0, 0)
    L = fmaf(wgt, ml[2 * s + 1], L);
    o = fmaf(wgt, op[(int64_t)s * HD + d], o);
  }
  y[(int64_t)b * ldy + h * HD + d] = f_to_bf(L > 0.0f ? o / L : 0.0f);
}

// The same for up to 32 * NB <= 64 splits.  The merge is a chain of memory round trips and little else, so here all of
// it is requested before anything is waited for: lane s of a wave asks for (max, sum) of split s, every lane for
// its element of every partial result (no branch around a load: a split beyond the last reads the last one again
// and gets weight zero).  The weights exp(m_s - max) are formed by the 64 lanes at once and handed round through
// v_readlane: one round trip, where the loop above makes two per eight splits and a scalar load per split.  The
// sums run over the splits in ascending order with the same operations: the results are the same bits.
template <int HD, int NB>
__global__ __launch_bounds__(HD) void k_attn_decode_combine_once(const float* __restrict__ o_part,
                                                                 const float* __restrict__ ml_part,
                                                                 u16* __restrict__ y, int64_t ldy, int Hq, int nsplit) {
  constexpr int NS = 32 * NB;
  const int h = blockIdx.x, b = blockIdx.y, d = threadIdx.x, lane = d & 63;
  const float* ml = ml_part + ((int64_t)b * Hq + h) * nsplit * 2;
  const float* op = o_part + ((int64_t)b * Hq + h) * nsplit * HD;
  const int sl = lane < nsplit ? lane : nsplit - 1;
  const float2 mlv = *reinterpret_cast<const float2*>(ml + 2 * sl);
  float ov[NS];
#pragma unroll
  for (int j = 0; j < NS; ++j) ov[j] = op[(int64_t)(j < nsplit ? j : nsplit - 1) * HD + d];
  const float M = wave_max(mlv.x);  // (lanes beyond the last split repeat it: the maximum is the same)
  const float w_lane = (lane >= nsplit || mlv.x == -INFINITY) ? 0.0f : expf(mlv.x - M);  // an empty split: (-inf, 0, 0)
  float L = 0.0f, o = 0.0f;
#pragma unroll
  for (int j = 0; j < NS; ++j) {
    const float wgt = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(w_lane), j));
    const float lj = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(mlv.y), j));
    if (j < nsplit) {  // uniform (a sum must not see the -0.0 + 0.0 of a padded split)
      L = fmaf(wgt, lj, L);
      o = fmaf(wgt, ov[j], o);
    }
  }
  y[(int64_t)b * ldy + h * HD + d] = f_to_bf(L > 0.0f ? o / L : 0.0f);
}

template <int HD>
static inline void launch_attn_combine(const float* o_part, const float* ml_part, u16* y, int64_t ldy, int Hq, int B,
                                       int nsplit, hipStream_t s) {
  if (nsplit <= 32) k_attn_decode_combine_once<HD, 1><<<dim3(Hq, B), dim3(HD), 0, s>>>(o_part, ml_part, y, ldy, Hq, nsplit);
  else if (nsplit <= 64) k_attn_decode_combine_once<HD, 2><<<dim3(Hq, B), dim3(HD), 0, s>>>(o_part, ml_part, y, ldy, Hq, nsplit);
  else k_attn_decode_combine<HD><<<dim3(Hq, B), dim3(HD), 0, s>>>(o_part, ml_part, y, ldy, Hq, nsplit);
}
