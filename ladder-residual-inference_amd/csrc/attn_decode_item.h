#pragma once
#include "lr_common.h"

// ---- how the valid keys are cut into chunks (one workgroup item per chunk, kv head and sequence)
static inline int attn_nsplit_cap(int Smax) {
  const int by_len = (Smax + 511) / 512;  // a chunk never exceeds 512 keys (LDS score buffer)
  return by_len > 64 ? by_len : 64;
}

static inline int attn_pick_nsplit(int B, int Hkv, int Smax) {
  const int cap = attn_nsplit_cap(Smax);
  int n = (512 + B * Hkv - 1) / (B * Hkv);   // aim at >= 512 workgroups
  const int by_work = (Smax + 63) / 64;      // but at least ~64 keys per chunk at full length
  if (n > by_work) n = by_work;
  const int by_len = (Smax + 511) / 512;
  if (n < by_len) n = by_len;
  if (n < 1) n = 1;
  return n > cap ? cap : n;
}


// One (split, kv head, sequence) item of the split-KV decode attention, by 256 lanes (4 waves): scores,
// softmax statistics and the un-normalised P.V of keys [k0, k1) for all G q heads of the kv head.
// `smem`: attn_item_lds_floats<HD, G>(chunk_max) floats of LDS.  A device function so that the plain
// kernel stays a thin wrapper.
template <int HD, int G>
__host__ __device__ constexpr int attn_item_lds_floats(int chunk_max) { return G * HD * 5 + G * chunk_max + 2 * G; }

template <int HD, int G>
__device__ __forceinline__ void attn_partial_item(const u16* __restrict__ q, int64_t ldq, const u16* __restrict__ kc,
                                                  const u16* __restrict__ vc, const int32_t* __restrict__ pos_ptr,
                                                  float* __restrict__ o_part, float* __restrict__ ml_part, int Hkv,
                                                  int Smax, int nsplit, int chunk_max, int split, int kvh, int b,
                                                  float* __restrict__ smem) {
  constexpr int LPK = HD / 8;    // lanes that share one key row (8 elements each)
  constexpr int KPW = 64 / LPK;  // keys per wave per iteration
  float* qs = smem;                       // [G][HD]
  float* ored = qs + G * HD;              // [4][G][HD]
  float* sc = ored + 4 * G * HD;          // [G][chunk_max]
  float* s_m = sc + G * chunk_max;        // [G]
  float* s_l = s_m + G;                   // [G]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int Hq = Hkv * G;
  int nkeys = pos_ptr[0] + 1;
  nkeys = nkeys < 0 ? 0 : (nkeys > Smax ? Smax : nkeys);
  const int chunk = (nkeys + nsplit - 1) / nsplit;
  const int k0 = split * chunk;
  const int k1 = k0 + chunk < nkeys ? k0 + chunk : nkeys;
  const int n = k1 - k0;  // <= chunk_max by construction

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
  const u16* kbase = kc + ((int64_t)b * Hkv + kvh) * Smax * HD;
  const u16* vbase = vc + ((int64_t)b * Hkv + kvh) * Smax * HD;
  const float scale = rsqrtf((float)HD);
  // Keys are walked PFB iterations at a time with all loads of a batch requested together, and the
  // first batch of K and of V is requested before anything else: a 64-key chunk (the usual size)
  // then costs one memory round trip instead of one per iteration and per operand.
  constexpr int PFB = 4;
  const int key00 = k0 + wave * KPW + kl;
  uint4 kfirst[PFB], vfirst[PFB];
#pragma unroll
  for (int u = 0; u < PFB; ++u) {
    const int key = key00 + u * 4 * KPW;
    kfirst[u] = key < k1 ? ld16(kbase + (int64_t)key * HD + dl) : make_uint4(0, 0, 0, 0);
    vfirst[u] = key < k1 ? ld16(vbase + (int64_t)key * HD + dl) : make_uint4(0, 0, 0, 0);
  }
  for (int i = tid; i < G * HD; i += 256)
    qs[i] = bf_to_f(q[(int64_t)b * ldq + (kvh * G + i / HD) * HD + (i % HD)]);
  __syncthreads();

  // ---- scores
  {
    float qf[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int j = 0; j < 8; ++j) qf[g][j] = qs[g * HD + dl + j];
    for (int kb = key00; kb < k1 + kl; kb += PFB * 4 * KPW) {  // "+ kl": keep the wave converged
      uint4 kr[PFB];
#pragma unroll
      for (int u = 0; u < PFB; ++u) {
        const int key = kb + u * 4 * KPW;
        kr[u] = kb == key00 ? kfirst[u] : (key < k1 ? ld16(kbase + (int64_t)key * HD + dl) : make_uint4(0, 0, 0, 0));
      }
#pragma unroll
      for (int u = 0; u < PFB; ++u) {
        const int key = kb + u * 4 * KPW;
        const bool live = key < k1;
        float kf[8];
        unpack8(kr[u], kf);
#pragma unroll
        for (int g = 0; g < G; ++g) {
          float s = 0.0f;
#pragma unroll
          for (int j = 0; j < 8; ++j) s = fmaf(kf[j], qf[g][j], s);
#pragma unroll
          for (int o = 1; o < LPK; o <<= 1) s += __shfl_xor(s, o, LR_WAVE);
          if (live && (lane % LPK) == 0) sc[g * chunk_max + key - k0] = s * scale;
        }
      }
    }
  }
  __syncthreads();

  // ---- softmax statistics per head; sc becomes exp(s - max)
  for (int g = wave; g < G; g += 4) {
    float m = -INFINITY;
    for (int i = lane; i < n; i += 64) m = fmaxf(m, sc[g * chunk_max + i]);
    m = wave_max(m);
    float l = 0.0f;
    for (int i = lane; i < n; i += 64) {
      const float p = expf(sc[g * chunk_max + i] - m);
      sc[g * chunk_max + i] = p;
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
    for (int kb = key00; kb < k1; kb += PFB * 4 * KPW) {
      uint4 vr[PFB];
#pragma unroll
      for (int u = 0; u < PFB; ++u) {
        const int key = kb + u * 4 * KPW;
        vr[u] = kb == key00 ? vfirst[u] : (key < k1 ? ld16(vbase + (int64_t)key * HD + dl) : make_uint4(0, 0, 0, 0));
      }
#pragma unroll
      for (int u = 0; u < PFB; ++u) {
        const int key = kb + u * 4 * KPW;
        if (key < k1) {
          float vf[8];
          unpack8(vr[u], vf);
#pragma unroll
          for (int g = 0; g < G; ++g) {
            const float p = sc[g * chunk_max + key - k0];
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[g][j] = fmaf(p, vf[j], acc[g][j]);
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
