// Attention over the contiguous [B, Hkv, Smax, hd] KV cache.
//
// Decode (one query per sequence): the valid keys 0..pos are cut into `nsplit` contiguous chunks;
// one workgroup per (chunk, kv head, sequence) serves ALL q heads of that kv head, so K and V are
// read from HBM once per GQA group.  Scores, softmax and P.V stay in fp32 (P is never rounded),
// chunk results carry their own (max, sum) and a second tiny kernel merges them in chunk order.
// Only slots <= pos are touched: with the reference's boolean mask the other slots get weight
// exp(-inf) = 0, so this is the same function of the cache.
//
// Prefill (S queries per sequence): one lane per query row with the running (max, sum, output)
// in registers, K/V tiles of 32 keys broadcast from LDS as fp32.  Exact fp32 softmax, one rounding
// at the end.
#include "lr_common.h"

// ------------------------------------------------------------------------------------ decode
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
  constexpr int LPK = HD / 8;    // lanes that share one key row (8 elements each)
  constexpr int KPW = 64 / LPK;  // keys per wave per iteration
  extern __shared__ __attribute__((aligned(16))) float smem[];
  float* qs = smem;                       // [G][HD]
  float* ored = qs + G * HD;              // [4][G][HD]
  float* sc = ored + 4 * G * HD;          // [G][chunk_max]
  __shared__ float s_m[G], s_l[G];

  const int split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
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

  for (int i = tid; i < G * HD; i += 256)
    qs[i] = bf_to_f(q[(int64_t)b * ldq + (kvh * G + i / HD) * HD + (i % HD)]);
  __syncthreads();

  const int kl = lane / LPK, dl = (lane % LPK) * 8;
  const u16* kbase = kc + ((int64_t)b * Hkv + kvh) * Smax * HD;
  const u16* vbase = vc + ((int64_t)b * Hkv + kvh) * Smax * HD;
  const float scale = rsqrtf((float)HD);

  // ---- scores
  {
    float qf[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int j = 0; j < 8; ++j) qf[g][j] = qs[g * HD + dl + j];
    for (int key = k0 + wave * KPW + kl; key < k1 + kl; key += 4 * KPW) {  // "+ kl": keep the wave converged
      const bool live = key < k1;
      float kf[8];
      unpack8(live ? ld16(kbase + (int64_t)key * HD + dl) : make_uint4(0, 0, 0, 0), kf);
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
    for (int key = k0 + wave * KPW + kl; key < k1; key += 4 * KPW) {
      float vf[8];
      unpack8(ld16(vbase + (int64_t)key * HD + dl), vf);
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const float p = sc[g * chunk_max + key - k0];
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[g][j] = fmaf(p, vf[j], acc[g][j]);
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

template <int HD>
__global__ __launch_bounds__(HD) void k_attn_decode_combine(const float* __restrict__ o_part,
                                                            const float* __restrict__ ml_part, u16* __restrict__ y,
                                                            int64_t ldy, int Hq, int nsplit) {
  const int h = blockIdx.x, b = blockIdx.y, d = threadIdx.x;
  const float* ml = ml_part + ((int64_t)b * Hq + h) * nsplit * 2;
  const float* op = o_part + ((int64_t)b * Hq + h) * nsplit * HD;
  float M = -INFINITY;
  for (int s = 0; s < nsplit; ++s) M = fmaxf(M, ml[2 * s]);
  float L = 0.0f, o = 0.0f;
  for (int s = 0; s < nsplit; ++s) {
    const float m = ml[2 * s];
    if (m == -INFINITY) continue;
    const float wgt = expf(m - M);
    L = fmaf(wgt, ml[2 * s + 1], L);
    o = fmaf(wgt, op[(int64_t)s * HD + d], o);
  }
  y[(int64_t)b * ldy + h * HD + d] = f_to_bf(L > 0.0f ? o / L : 0.0f);
}

template <int HD, int G>
static int launch_decode(const u16* q, int64_t ldq, const u16* kc, const u16* vc, const int32_t* pos, u16* y,
                         int64_t ldy, int B, int Hkv, int Smax, float* scratch, hipStream_t s) {
  const int Hq = Hkv * G;
  const int nsplit = attn_pick_nsplit(B, Hkv, Smax);
  const int chunk_max = ((Smax + nsplit - 1) / nsplit + 3) & ~3;
  float* o_part = scratch;
  float* ml_part = scratch + (size_t)B * Hq * nsplit * HD;
  const size_t lds = (size_t)(G * HD * 5 + G * chunk_max) * sizeof(float);
  if (lds > 64 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&k_attn_decode_partial<HD, G>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return LR_E_LAUNCH;
  }
  k_attn_decode_partial<HD, G><<<dim3(nsplit, Hkv, B), dim3(256), lds, s>>>(q, ldq, kc, vc, pos, o_part, ml_part, Hkv,
                                                                            Smax, nsplit, chunk_max);
  k_attn_decode_combine<HD><<<dim3(Hq, B), dim3(HD), 0, s>>>(o_part, ml_part, y, ldy, Hq, nsplit);
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
