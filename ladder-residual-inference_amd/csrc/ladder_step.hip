// One decode step of the Ladder model as ONE persistent kernel (batch 1 or 2).
//
// Why: at batch 1 a step streams 17 GB of weights through ~720 small dependent ops.  Launched
// one by one (even from a hipGraph) the ops pay a launch boundary each and the latency-bound
// ones (norms, RoPE, attention, combine) cost as much as the weight streaming.  Here one
// workgroup per CU (1024 lanes) stays resident for the whole step and walks the layers; the
// workgroups meet at device-wide barriers built from relaxed agent-scope atomics (a 16-group
// arrival tree: ~1.5 us on 256 CUs; acquire/release fences are avoided because they write back
// and invalidate the whole L2).
//
// The ladder schedule is what makes the phases wide: attention block t reads the residual
// stream WITHOUT the MLP output of layer t-1 (in the reference that output is still inside an
// all-reduce), so attention(t) and mlp(t-1) are independent and run side by side.  A "slot" t is
//     phase 1:  [residual adds + both RMSNorms]  wqkv(t) GEMV        ||  first part of w1(t-1) GEMV + SwiGLU
//     phase 2:  RoPE + KV write + attention(t) (+ split-KV combine)  ||  rest of w1(t-1) GEMV + SwiGLU
//     phase 3:  wo(t) GEMV                                           ||  w2(t-1) GEMV
// with one barrier after each phase: 3 per layer instead of 9 kernel launches, and every phase
// streams 60-75 MB of weights at the 70B shard shape.
//
// Data that crosses workgroups inside the step (residual, partial sums, qkv, attention output,
// activations) lives in a small fp32 workspace and is only touched with agent-scope relaxed
// atomic loads/stores (global_load/store ... sc1), which bypass the non-coherent per-XCD L2 lines;
// the values stored are bf16-representable, i.e. rounded exactly where the eager reference
// rounds.  Weights, KV cache and logits use ordinary accesses (read-only, or produced for the
// next launch).  GEMV rows are dealt to workgroups round-robin so that the CUs working at the
// same time read neighbouring rows (HBM-channel friendly); inside a workgroup the 16 waves split
// K, partial sums meet in LDS in a fixed order -- no float atomics, bit-reproducible.
//
// Every spin is bounded: on time-out a workgroup raises ctrl->fail and leaves; the others see the
// flag (or time out themselves), so the grid always drains.
#include "lr_common.h"

namespace {

constexpr int NT = 1024;          // lanes per workgroup
constexpr int NW = NT / 64;       // waves per workgroup
constexpr int BAR_GROUPS = 16;    // arrival-tree fan-in
constexpr int NJMAX = 64;         // GEMV rows a workgroup reduces per LDS round
constexpr int RB = 8;             // rows a wave keeps in flight
constexpr unsigned SPIN_LIMIT = 1u << 21;
constexpr int CHUNK_MAX = 128;    // keys per attention workgroup (LDS score buffer)

struct Ctrl {  // every hot word on its own 128-byte line
  unsigned root, _p0[31];
  unsigned gcount[BAR_GROUPS][32];
  unsigned gflag[BAR_GROUPS][32];
  unsigned epoch_base, _p1[31];
  unsigned att_count, _p2[31];
  unsigned att_base, _p3[31];
  unsigned fail, _p4[31];
  unsigned nwg, _p5[31];
};

struct LayerPtrs {
  const u16 *wqkv, *wo, *w1, *w2, *attn_norm, *ffn_norm;
  u16 *k_cache, *v_cache;
};

struct StepParams {
  int D, L, Hkv, I, V, vocab, Smax, block_size, B, NA, P1, nqkv;
  float eps;
  const u16 *tok_emb, *final_norm, *out_w, *rope;
  const LayerPtrs* layers;
  const int32_t* tokens;
  int32_t* pos;
  u16* logits;
  int64_t ldl;
  int32_t *next_token, *cur_token, *history;
  int64_t ld_hist;
  int hist_len, pos0, advance;
  Ctrl* ctrl;
  float *Rbuf, *abuf, *mbuf, *qkv, *y, *act, *opart, *mlpart, *cand;
};

// ---- coherent (cross-workgroup) accesses
__device__ __forceinline__ float cld(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void cst(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned cldu(const unsigned* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void cstu(unsigned* p, unsigned v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned cadd(unsigned* p) {
  return __hip_atomic_fetch_add(p, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void cld8(const float* p, float* f) {  // 8 floats, 32-byte aligned
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const unsigned long long u = __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p) + i,
                                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    f[2 * i] = __uint_as_float((unsigned)u);
    f[2 * i + 1] = __uint_as_float((unsigned)(u >> 32));
  }
}
__device__ __forceinline__ void cst8(float* p, const float* f) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const unsigned long long u = (unsigned long long)__float_as_uint(f[2 * i]) |
                                 ((unsigned long long)__float_as_uint(f[2 * i + 1]) << 32);
    __hip_atomic_store(reinterpret_cast<unsigned long long*>(p) + i, u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// All lanes: wait for this lane's outstanding memory operations, then meet.  After it, every
// coherent store issued by the workgroup has been acknowledged.
__device__ __forceinline__ void drain_and_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
}

// Device-wide barrier.  `epoch` counts barriers since the workspace was initialised (all
// workgroups advance it identically).  Returns false if the step must be abandoned.
__device__ __forceinline__ bool grid_barrier(Ctrl* c, unsigned& epoch, int* s_flag) {
  drain_and_sync();
  ++epoch;
  if (threadIdx.x == 0) {
    const unsigned nwg = gridDim.x;
    const unsigned ngr = nwg < BAR_GROUPS ? nwg : BAR_GROUPS;
    const unsigned g = blockIdx.x % ngr;
    const unsigned gn = nwg / ngr + (g < nwg % ngr ? 1u : 0u);
    int ok = 1;
    bool released = false;
    if (cadd(&c->gcount[g][0]) + 1u == epoch * gn) {
      if (cadd(&c->root) + 1u == epoch * ngr) {
        for (unsigned i = 0; i < ngr; ++i) cstu(&c->gflag[i][0], epoch);
        released = true;
      }
    }
    if (!released) {
      unsigned spins = 0;
      while ((int)(cldu(&c->gflag[g][0]) - epoch) < 0) {
        if ((++spins & 1023u) == 0 && (spins > SPIN_LIMIT || cldu(&c->fail))) {
          cstu(&c->fail, 1u);
          ok = 0;
          break;
        }
        __builtin_amdgcn_s_sleep(1);
      }
    }
    *s_flag = ok;
  }
  __syncthreads();
  return *s_flag != 0;
}

// ------------------------------------------------------------------------------------------------
// Residual bookkeeping + RMSNorm for the coming phase, done redundantly by every workgroup:
//   v1 = src (+ d1);  v2 = v1 (+ d2);  each add rounded to bf16.
//   x1 = norm(v1) * g1 -> LDS (if g1);  x2 = norm(v2) * g2 -> LDS (if g2);  workgroup 0 stores v2.
// src is either the coherent fp32 residual or rows of the bf16 embedding table.
// ------------------------------------------------------------------------------------------------
template <int M>
__device__ __forceinline__ void prologue(const StepParams& p, const float* src, const int* emb_rows,
                                         const float* d1, const float* d2, const u16* g1, const u16* g2,
                                         float* r_out, u16* x1, u16* x2, float* red) {
  constexpr int NIT = 2;  // D <= 16384
  const int tid = threadIdx.x, D = p.D;
  float v1[M][NIT][8], v2[M][NIT][8];
  float ss1[M], ss2[M];
#pragma unroll
  for (int m = 0; m < M; ++m) {
    ss1[m] = ss2[m] = 0.0f;
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int c = (tid + it * NT) * 8;
      if (c < D && m < p.B) {
        if (emb_rows) {
          const int id = emb_rows[m];
          const bool ok = id >= 0 && id < p.vocab;
          unpack8(ok ? ld16(p.tok_emb + (int64_t)id * D + c) : make_uint4(0, 0, 0, 0), v1[m][it]);
        } else {
          cld8(src + (int64_t)m * D + c, v1[m][it]);
        }
        if (d1) {
          float t[8];
          cld8(d1 + (int64_t)m * D + c, t);
#pragma unroll
          for (int j = 0; j < 8; ++j) v1[m][it][j] = round_bf(v1[m][it][j] + t[j]);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) v2[m][it][j] = v1[m][it][j];
        if (d2) {
          float t[8];
          cld8(d2 + (int64_t)m * D + c, t);
#pragma unroll
          for (int j = 0; j < 8; ++j) v2[m][it][j] = round_bf(v2[m][it][j] + t[j]);
        }
        if (r_out && blockIdx.x == 0) cst8(r_out + (int64_t)m * D + c, v2[m][it]);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          ss1[m] += v1[m][it][j] * v1[m][it][j];
          ss2[m] += v2[m][it][j] * v2[m][it][j];
        }
      }
    }
  }
#pragma unroll
  for (int m = 0; m < M; ++m) {
    ss1[m] = wave_sum(ss1[m]);
    ss2[m] = wave_sum(ss2[m]);
  }
  if ((tid & 63) == 0) {
#pragma unroll
    for (int m = 0; m < M; ++m) {
      red[((tid >> 6) * M + m) * 2] = ss1[m];
      red[((tid >> 6) * M + m) * 2 + 1] = ss2[m];
    }
  }
  __syncthreads();
#pragma unroll
  for (int m = 0; m < M; ++m) {
    float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
    for (int wv = 0; wv < NW; ++wv) {
      s1 += red[(wv * M + m) * 2];
      s2 += red[(wv * M + m) * 2 + 1];
    }
    const float inv1 = rsqrtf(s1 / (float)D + p.eps), inv2 = rsqrtf(s2 / (float)D + p.eps);
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int c = (tid + it * NT) * 8;
      if (c < D) {
        float g[8], o[8];
        if (g1) {
          unpack8(ld16(g1 + c), g);
#pragma unroll
          for (int j = 0; j < 8; ++j) o[j] = round_bf(v1[m][it][j] * inv1) * g[j];
          st16(x1 + m * D + c, pack8(o));
        }
        if (g2) {
          unpack8(ld16(g2 + c), g);
#pragma unroll
          for (int j = 0; j < 8; ++j) o[j] = round_bf(v2[m][it][j] * inv2) * g[j];
          st16(x2 + m * D + c, pack8(o));
        }
      }
    }
  }
  __syncthreads();
}

// Bring a coherent fp32 activation [M][K] (bf16-representable values) into LDS as bf16.
template <int M>
__device__ __forceinline__ void load_x(const StepParams& p, const float* src, int K, u16* x) {
  for (int c = threadIdx.x * 8; c < M * K; c += NT * 8) {
    const int m = c / K;
    float f[8];
    if (m < p.B) cld8(src + c, f);
    else {
#pragma unroll
      for (int j = 0; j < 8; ++j) f[j] = 0.0f;
    }
    st16(x + c, pack8(f));
  }
  __syncthreads();
}

// ------------------------------------------------------------------------------------------------
// GEMV over the rows this workgroup owns: item it = w + nwg * jj (jj = 0, 1, ...) of n_items.
//   EPI_STORE : item = row;   out[m][it]  = bf16(sum)                       (coherent fp32)
//   EPI_SWIGLU: item = pair;  rows it (up) and it + pair_off (gate);  out[m][it] = silu(g) * u
//   EPI_LOGITS: item = row;   logits[m][it] = bf16(sum) (plain store) + running argmax
// x: LDS bf16 [M][K].  part: LDS float [NW][NJMAX * M].
// ------------------------------------------------------------------------------------------------
enum { EPI_STORE = 0, EPI_SWIGLU = 1, EPI_LOGITS = 2 };

template <int M, int EPI>
__device__ __forceinline__ void gemv_phase(const StepParams& p, const u16* __restrict__ W, int K, int row_base,
                                           int n_items, int pair_off, const u16* x, float* part, float* out, int ldo,
                                           float* cand_v, int* cand_i, float* best_v, int* best_i) {
  constexpr int RPI = EPI == EPI_SWIGLU ? 2 : 1;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int w = blockIdx.x, nwg = gridDim.x;
  const int nit = n_items > w ? (n_items - w + nwg - 1) / nwg : 0;
  const int nj = nit * RPI;
  const int ksteps = (K + 511) >> 9;
  const int nkg = ksteps < NW ? ksteps : NW;
  const int nrg = NW / nkg;
  const bool active = wave < nrg * nkg;
  const int rg = wave / nkg, kg = wave - rg * nkg;

  for (int j0 = 0; j0 < nj; j0 += NJMAX) {
    const int njb = nj - j0 < NJMAX ? nj - j0 : NJMAX;
    if (active) {
      for (int jb = rg; jb < njb; jb += nrg * RB) {
        float acc[RB][M];
        const u16* wp[RB];
        bool rv[RB];
#pragma unroll
        for (int i = 0; i < RB; ++i) {
          const int j = jb + i * nrg;
          rv[i] = j < njb;
          const int jj = j0 + (rv[i] ? j : 0);
          const int row = row_base + w + nwg * (jj / RPI) + (jj % RPI) * pair_off;
          wp[i] = W + (int64_t)row * K;
#pragma unroll
          for (int m = 0; m < M; ++m) acc[i][m] = 0.0f;
        }
        for (int kk = kg; kk < ksteps; kk += nkg) {
          const int k = kk * 512 + lane * 8;
          const bool kv = k < K;
          uint4 wv[RB];
#pragma unroll
          for (int i = 0; i < RB; ++i) wv[i] = (kv && rv[i]) ? ld16(wp[i] + k) : make_uint4(0, 0, 0, 0);
          float xf[M][8];
#pragma unroll
          for (int m = 0; m < M; ++m)
            unpack8(kv ? *reinterpret_cast<const uint4*>(x + m * K + k) : make_uint4(0, 0, 0, 0), xf[m]);
#pragma unroll
          for (int i = 0; i < RB; ++i) {
            float wf[8];
            unpack8(wv[i], wf);
#pragma unroll
            for (int m = 0; m < M; ++m)
#pragma unroll
              for (int e = 0; e < 8; ++e) acc[i][m] = fmaf(wf[e], xf[m][e], acc[i][m]);
          }
        }
#pragma unroll
        for (int i = 0; i < RB; ++i)
#pragma unroll
          for (int m = 0; m < M; ++m) {
            const float s = wave_sum(acc[i][m]);
            if (lane == 0 && rv[i]) part[(kg * NJMAX + jb + i * nrg) * M + m] = s;
          }
      }
    }
    __syncthreads();
    // ---- cross-wave sum in fixed order + epilogue
    const int nout = (njb / RPI) * M;
    if (tid < nout) {
      const int jl = tid / M, m = tid - jl * M;
      float s[RPI];
#pragma unroll
      for (int r = 0; r < RPI; ++r) {
        float t = 0.0f;
        for (int g = 0; g < nkg; ++g) t += part[(g * NJMAX + jl * RPI + r) * M + m];
        s[r] = round_bf(t);
      }
      const int it = w + nwg * ((j0 / RPI) + jl);
      if (m < p.B) {
        if (EPI == EPI_STORE) cst(out + (int64_t)m * ldo + it, s[0]);
        if (EPI == EPI_SWIGLU) cst(out + (int64_t)m * ldo + it, swiglu_bf(s[0], s[RPI - 1]));
        if (EPI == EPI_LOGITS) p.logits[(int64_t)m * p.ldl + it] = f_to_bf(s[0]);
      }
      if (EPI == EPI_LOGITS) {
        cand_v[tid] = s[0];
        cand_i[tid] = it;
      }
    }
    if (EPI == EPI_LOGITS) {
      __syncthreads();
      if (tid < M) {  // items ascend with jl: strict '>' keeps the lowest index among equals
        for (int jl = 0; jl < njb; ++jl) {
          const float v = cand_v[jl * M + tid];
          if (v > *best_v) { *best_v = v; *best_i = cand_i[jl * M + tid]; }
        }
      }
    }
    __syncthreads();
  }
}

// ------------------------------------------------------------------------------------------------
// Attention of slot t for attention workgroup `aw` of NA: keys [k0, k1) of every (sequence, kv head).
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ void rope_pair(float x0, float x1, float c, float s, float& o0, float& o1) {
#pragma clang fp contract(off)
  const float a = x0 * c, b = x1 * s, d = x1 * c, e = x0 * s;
  o0 = round_bf(a - b);
  o1 = round_bf(d + e);
}

template <int M, int HD, int G>
__device__ __forceinline__ void attention_phase(const StepParams& p, const LayerPtrs& lp, int pos, unsigned att_epoch,
                                                float* qs, float* sc, float* ored, float* knew, float* vnew,
                                                float* s_m, float* s_l, int* s_flag) {
  constexpr int LPK = HD / 8, KPW = 64 / LPK;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int aw = blockIdx.x, NA = p.NA, Hkv = p.Hkv, Hq = Hkv * G;
  const int nkeys = pos + 1;
  const int chunk = (nkeys + NA - 1) / NA;
  const int k0 = aw * chunk;
  const int k1 = k0 + chunk < nkeys ? k0 + chunk : nkeys;
  const int n = k1 - k0;
  const bool owner = pos >= k0 && pos < k1;
  const float scale = rsqrtf((float)HD);
  const u16* trow = p.rope + (int64_t)pos * HD;  // (cos, sin) pairs of this position
  const int kl = lane / LPK, dl = (lane % LPK) * 8;

  for (int b = 0; b < p.B; ++b) {
    const float* qkv = p.qkv + (int64_t)b * p.nqkv;
    for (int kvh = 0; kvh < Hkv; ++kvh) {
      float* o_out = p.opart + (((int64_t)b * Hq + kvh * G) * NA + aw) * HD;
      float* ml_out = p.mlpart + (((int64_t)b * Hq + kvh * G) * NA + aw) * 2;
      // ---- rotate q (all G heads) into LDS; the owner also rotates k, keeps k/v in LDS and
      //      writes them to the cache for the following steps
      for (int i = tid; i < G * HD / 2; i += NT) {
        const int g = i / (HD / 2), j = i - g * (HD / 2);
        const float x0 = cld(qkv + (kvh * G + g) * HD + 2 * j), x1 = cld(qkv + (kvh * G + g) * HD + 2 * j + 1);
        rope_pair(x0, x1, bf_to_f(trow[2 * j]), bf_to_f(trow[2 * j + 1]), qs[g * HD + 2 * j], qs[g * HD + 2 * j + 1]);
      }
      if (owner && tid < HD / 2) {
        const int j = tid;
        const float* ksrc = qkv + Hq * HD + kvh * HD;
        const float* vsrc = qkv + (Hq + Hkv) * HD + kvh * HD;
        float r0, r1;
        rope_pair(cld(ksrc + 2 * j), cld(ksrc + 2 * j + 1), bf_to_f(trow[2 * j]), bf_to_f(trow[2 * j + 1]), r0, r1);
        const float v0 = cld(vsrc + 2 * j), v1 = cld(vsrc + 2 * j + 1);
        knew[2 * j] = r0; knew[2 * j + 1] = r1;
        vnew[2 * j] = v0; vnew[2 * j + 1] = v1;
        const int64_t slot = (((int64_t)b * Hkv + kvh) * p.Smax + pos) * HD + 2 * j;
        *reinterpret_cast<u32*>(lp.k_cache + slot) = pack_bf2(r0, r1);
        *reinterpret_cast<u32*>(lp.v_cache + slot) = pack_bf2(v0, v1);
      }
      __syncthreads();
      if (n > 0) {
        const u16* kbase = lp.k_cache + ((int64_t)b * Hkv + kvh) * p.Smax * HD;
        const u16* vbase = lp.v_cache + ((int64_t)b * Hkv + kvh) * p.Smax * HD;
        // ---- scores
        {
          float qf[G][8];
#pragma unroll
          for (int g = 0; g < G; ++g)
#pragma unroll
            for (int j = 0; j < 8; ++j) qf[g][j] = qs[g * HD + dl + j];
          for (int key = k0 + wave * KPW + kl; key < k1 + kl; key += NW * KPW) {
            const bool live = key < k1;
            float kf[8];
            if (live && key == pos) {
#pragma unroll
              for (int j = 0; j < 8; ++j) kf[j] = knew[dl + j];
            } else {
              unpack8(live ? ld16(kbase + (int64_t)key * HD + dl) : make_uint4(0, 0, 0, 0), kf);
            }
#pragma unroll
            for (int g = 0; g < G; ++g) {
              float s = 0.0f;
#pragma unroll
              for (int j = 0; j < 8; ++j) s = fmaf(kf[j], qf[g][j], s);
#pragma unroll
              for (int o = 1; o < LPK; o <<= 1) s += __shfl_xor(s, o, LR_WAVE);
              if (live && (lane % LPK) == 0) sc[g * CHUNK_MAX + key - k0] = s * scale;
            }
          }
        }
        __syncthreads();
        // ---- softmax statistics: one wave per head
        if (wave < G) {
          const int g = wave;
          float m = -INFINITY;
          for (int i = lane; i < n; i += 64) m = fmaxf(m, sc[g * CHUNK_MAX + i]);
          m = wave_max(m);
          float l = 0.0f;
          for (int i = lane; i < n; i += 64) {
            const float e = expf(sc[g * CHUNK_MAX + i] - m);
            sc[g * CHUNK_MAX + i] = e;
            l += e;
          }
          l = wave_sum(l);
          if (lane == 0) { s_m[g] = m; s_l[g] = l; }
        }
        __syncthreads();
        // ---- P.V, folded over the key groups of a wave, then over the 16 waves in two LDS rounds
        float acc[G][8];
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
          for (int j = 0; j < 8; ++j) acc[g][j] = 0.0f;
        for (int key = k0 + wave * KPW + kl; key < k1; key += NW * KPW) {
          float vf[8];
          if (key == pos) {
#pragma unroll
            for (int j = 0; j < 8; ++j) vf[j] = vnew[dl + j];
          } else {
            unpack8(ld16(vbase + (int64_t)key * HD + dl), vf);
          }
#pragma unroll
          for (int g = 0; g < G; ++g) {
            const float pr = sc[g * CHUNK_MAX + key - k0];
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[g][j] = fmaf(pr, vf[j], acc[g][j]);
          }
        }
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            float v = acc[g][j];
#pragma unroll
            for (int o = LPK; o < 64; o <<= 1) v += __shfl_xor(v, o, LR_WAVE);
            acc[g][j] = v;
          }
        if (wave >= NW / 2 && kl == 0) {
#pragma unroll
          for (int g = 0; g < G; ++g)
#pragma unroll
            for (int j = 0; j < 8; ++j) ored[((wave - NW / 2) * G + g) * HD + dl + j] = acc[g][j];
        }
        __syncthreads();
        if (wave < NW / 2 && kl == 0) {
#pragma unroll
          for (int g = 0; g < G; ++g)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              float* slot = &ored[(wave * G + g) * HD + dl + j];
              *slot = acc[g][j] + *slot;
            }
        }
        __syncthreads();
        for (int i = tid; i < G * HD; i += NT) {
          float v = 0.0f;
#pragma unroll
          for (int wv = 0; wv < NW / 2; ++wv) v += ored[wv * G * HD + i];
          cst(o_out + (int64_t)(i / HD) * NA * HD + (i % HD), v);
        }
        if (tid < G) {
          cst(ml_out + (int64_t)tid * NA * 2, s_m[tid]);
          cst(ml_out + (int64_t)tid * NA * 2 + 1, s_l[tid]);
        }
      } else {
        for (int i = tid; i < G * HD; i += NT) cst(o_out + (int64_t)(i / HD) * NA * HD + (i % HD), 0.0f);
        if (tid < G) {
          cst(ml_out + (int64_t)tid * NA * 2, -INFINITY);
          cst(ml_out + (int64_t)tid * NA * 2 + 1, 0.0f);
        }
      }
      __syncthreads();
    }
  }
  // ---- the last attention workgroup to get here merges the NA chunk results
  drain_and_sync();
  if (tid == 0) *s_flag = (cadd(&p.ctrl->att_count) + 1u == att_epoch * (unsigned)NA) ? 1 : 0;
  __syncthreads();
  if (*s_flag) {
    for (int i = tid; i < p.B * Hq * HD; i += NT) {
      const int d = i % HD, bh = i / HD;
      const float* ml = p.mlpart + (int64_t)bh * NA * 2;
      const float* op = p.opart + (int64_t)bh * NA * HD;
      float mx = -INFINITY;
      for (int s = 0; s < NA; ++s) mx = fmaxf(mx, cld(ml + 2 * s));
      float L = 0.0f, o = 0.0f;
      for (int s = 0; s < NA; ++s) {
        const float m = cld(ml + 2 * s);
        if (m == -INFINITY) continue;
        const float wgt = expf(m - mx);
        L = fmaf(wgt, cld(ml + 2 * s + 1), L);
        o = fmaf(wgt, cld(op + (int64_t)s * HD + d), o);
      }
      cst(p.y + i, round_bf(L > 0.0f ? o / L : 0.0f));
    }
  }
  __syncthreads();
}

// ------------------------------------------------------------------------------------------------
template <int M, int HD, int G>
__global__ __launch_bounds__(NT) void k_ladder_step(const StepParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int D = p.D, L = p.L, Hq = p.Hkv * G;
  // ---- LDS carve-up
  const int xlen = M * (D > p.I ? D : p.I);
  u16* xa = reinterpret_cast<u16*>(smem);              // attention-chain input  [M][<= D]
  u16* xb = xa + xlen;                                  // MLP-chain input        [M][<= D]
  float* part = reinterpret_cast<float*>(xb + xlen);    // [NW][NJMAX * M]
  float* red = part + NW * NJMAX * M;                   // [NW][M][2]
  float* qs = red + NW * M * 2;                         // [G][HD]
  float* sc = qs + G * HD;                              // [G][CHUNK_MAX]
  float* ored = sc + G * CHUNK_MAX;                     // [NW/2][G][HD]
  float* knew = ored + (NW / 2) * G * HD;               // [HD]
  float* vnew = knew + HD;                              // [HD]
  float* s_m = vnew + HD;                               // [G]
  float* s_l = s_m + G;                                 // [G]
  float* cand_v = s_l + G;                              // [NJMAX * M]
  int* cand_i = reinterpret_cast<int*>(cand_v + NJMAX * M);
  int* s_flag = cand_i + NJMAX * M;                     // [4]

  const int tid = threadIdx.x;
  if (tid == 0) {
    s_flag[1] = (int)cldu(&p.ctrl->epoch_base);
    s_flag[2] = (int)cldu(&p.ctrl->att_base);
  }
  __syncthreads();
  unsigned epoch = (unsigned)s_flag[1];
  const unsigned att_base = (unsigned)s_flag[2];
  int pos = p.pos[0];
  pos = pos < 0 ? 0 : (pos >= p.Smax ? p.Smax - 1 : pos);
  const bool att_wg = (int)blockIdx.x < p.NA;
  const int I = p.I;

  for (int t = 0; t <= L; ++t) {
    const bool has_a = t < L, has_b = t >= 1;
    const LayerPtrs la = p.layers[has_a ? t : L - 1];
    const LayerPtrs lb = p.layers[has_b ? t - 1 : 0];
    // ---------------- phase 1
    prologue<M>(p, p.Rbuf + (int64_t)((t + 1) & 1) * M * D, t == 0 ? p.tokens : nullptr,
                t >= 2 ? p.mbuf : nullptr, (t >= 1 && has_a) ? p.abuf : nullptr, has_b ? lb.ffn_norm : nullptr,
                has_a ? la.attn_norm : nullptr, p.Rbuf + (int64_t)(t & 1) * M * D, xb, xa, red);
    if (has_a)
      gemv_phase<M, EPI_STORE>(p, la.wqkv, D, 0, p.nqkv, 0, xa, part, p.qkv, p.nqkv, nullptr, nullptr, nullptr,
                               nullptr);
    if (has_b)
      gemv_phase<M, EPI_SWIGLU>(p, lb.w1, D, 0, p.P1, I, xb, part, p.act, I, nullptr, nullptr, nullptr, nullptr);
    if (!grid_barrier(p.ctrl, epoch, s_flag)) return;
    // ---------------- phase 2
    if (has_a && att_wg)
      attention_phase<M, HD, G>(p, la, pos, att_base + (unsigned)t + 1u, qs, sc, ored, knew, vnew, s_m, s_l, s_flag);
    if (has_b)
      gemv_phase<M, EPI_SWIGLU>(p, lb.w1, D, p.P1, I - p.P1, I, xb, part, p.act + p.P1, I, nullptr, nullptr, nullptr,
                                nullptr);
    if (!grid_barrier(p.ctrl, epoch, s_flag)) return;
    // ---------------- phase 3
    if (has_a) {
      load_x<M>(p, p.y, Hq * HD, xa);
      gemv_phase<M, EPI_STORE>(p, la.wo, Hq * HD, 0, D, 0, xa, part, p.abuf, D, nullptr, nullptr, nullptr, nullptr);
    }
    if (has_b) {
      load_x<M>(p, p.act, I, xb);
      gemv_phase<M, EPI_STORE>(p, lb.w2, I, 0, D, 0, xb, part, p.mbuf, D, nullptr, nullptr, nullptr, nullptr);
    }
    if (!grid_barrier(p.ctrl, epoch, s_flag)) return;
  }
  // ---------------- head: x = (R + a) + m, final norm, vocab-shard lm_head, argmax
  prologue<M>(p, p.Rbuf + (int64_t)(L & 1) * M * D, nullptr, p.abuf, p.mbuf, nullptr, p.final_norm, nullptr, xb, xa,
              red);
  float best_v = -INFINITY;
  int best_i = 0x7fffffff;
  gemv_phase<M, EPI_LOGITS>(p, p.out_w, D, 0, p.V, 0, xa, part, nullptr, 0, cand_v, cand_i, &best_v, &best_i);
  if (tid < M) {
    cst(p.cand + ((int64_t)blockIdx.x * M + tid) * 2, best_v);
    cst(p.cand + ((int64_t)blockIdx.x * M + tid) * 2 + 1, __int_as_float(best_i));
  }
  if (!grid_barrier(p.ctrl, epoch, s_flag)) return;
  if (blockIdx.x == 0) {
    if (tid < p.B) {
      float bv = -INFINITY;
      int bi = 0x7fffffff;
      for (int wg = 0; wg < (int)gridDim.x; ++wg) {
        const float v = cld(p.cand + ((int64_t)wg * M + tid) * 2);
        const int i = __float_as_int(cld(p.cand + ((int64_t)wg * M + tid) * 2 + 1));
        if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
      }
      if (bi == 0x7fffffff) bi = 0;
      if (p.next_token) p.next_token[tid] = bi;
      if (p.advance && p.cur_token) p.cur_token[tid] = bi;
      const int slot = p.pos[0] - p.pos0;
      if (p.advance && p.history && slot >= 0 && slot < p.hist_len) p.history[(int64_t)tid * p.ld_hist + slot] = bi;
    }
    __syncthreads();
    if (tid == 0) {
      if (p.advance) p.pos[0] = p.pos[0] + 1;
      cstu(&p.ctrl->epoch_base, epoch);
      cstu(&p.ctrl->att_base, att_base + (unsigned)L);
    }
  }
}

__global__ void k_step_init(Ctrl* c, unsigned nwg) {
  unsigned* w = reinterpret_cast<unsigned*>(c);
  for (int i = threadIdx.x; i < (int)(sizeof(Ctrl) / 4); i += blockDim.x) w[i] = 0u;
  __syncthreads();
  if (threadIdx.x == 0) c->nwg = nwg;
}

struct Layout {
  size_t ctrl, Rbuf, abuf, mbuf, qkv, y, act, opart, mlpart, cand, total;
};

static int num_cus() {
  static int n = 0;
  if (n == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 0;
    n = prop.multiProcessorCount;
  }
  return n;
}

static int pick_na(int Smax, int nwg) {
  int na = (Smax + 63) / 64;
  if (na > nwg) na = nwg;
  if (na < 1) na = 1;
  return na;
}

static Layout make_layout(const lr_ladder_model_t* md, int B, int nwg) {
  const int D = md->dim, Hq = md->n_head, hd = md->head_dim;
  const int nqkv = (Hq + 2 * md->n_kv_head) * hd;
  const int na = pick_na(md->smax, nwg);
  auto up = [](size_t x) { return (x + 255) & ~(size_t)255; };
  Layout l;
  size_t o = 0;
  l.ctrl = o; o = up(o + sizeof(Ctrl));
  l.Rbuf = o; o = up(o + sizeof(float) * 2 * B * D);
  l.abuf = o; o = up(o + sizeof(float) * B * D);
  l.mbuf = o; o = up(o + sizeof(float) * B * D);
  l.qkv = o; o = up(o + sizeof(float) * B * nqkv);
  l.y = o; o = up(o + sizeof(float) * B * Hq * hd);
  l.act = o; o = up(o + sizeof(float) * B * md->ffn);
  l.opart = o; o = up(o + sizeof(float) * B * Hq * na * hd);
  l.mlpart = o; o = up(o + sizeof(float) * B * Hq * na * 2);
  l.cand = o; o = up(o + sizeof(float) * nwg * B * 2);
  l.total = o;
  return l;
}

// (batch, head_dim, q heads per kv head) combinations the step kernel is instantiated for
#define LR_STEP_INSTANCES(X) \
  X(1, 128, 8) X(2, 128, 8) X(1, 128, 4) X(2, 128, 4) X(1, 64, 4) X(2, 64, 4) X(1, 128, 16) \
  X(1, 64, 2) X(2, 64, 2) X(1, 128, 2) X(1, 128, 1) X(1, 64, 1) X(1, 64, 8)

static bool has_instance(int B, int hd, int G) {
#define LR_HAS(MV, HDV, GV) if (B == MV && hd == HDV && G == GV) return true;
  LR_STEP_INSTANCES(LR_HAS)
#undef LR_HAS
  return false;
}

static int validate(const lr_ladder_model_t* md, int B) {
  if (md == nullptr) return LR_E_NULL;
  if (B < 1 || md->dim <= 0 || md->n_layer <= 0 || md->n_head <= 0 || md->n_kv_head <= 0 || md->ffn <= 0 ||
      md->out_rows <= 0 || md->vocab <= 0 || md->smax <= 0 || md->block_size <= 0 || md->n_head % md->n_kv_head)
    return LR_E_SHAPE;
  if (B > 2 || md->dim > 16384 || md->dim % 8 || md->ffn % 8 || (md->head_dim != 64 && md->head_dim != 128))
    return LR_E_UNSUPPORTED;
  if (!has_instance(B, md->head_dim, md->n_head / md->n_kv_head)) return LR_E_UNSUPPORTED;
  if (md->n_head * md->head_dim > 16384 || md->ffn > 16384) return LR_E_UNSUPPORTED;
  const int nwg = num_cus();
  if (nwg <= 0) return LR_E_LAUNCH;
  if ((md->smax + pick_na(md->smax, nwg) - 1) / pick_na(md->smax, nwg) > CHUNK_MAX) return LR_E_UNSUPPORTED;
  if (!md->tok_embeddings || !md->norm || !md->output || !md->freqs_cis || !md->layers_dev) return LR_E_NULL;
  return LR_OK;
}

template <int M, int HD, int G>
static size_t lds_bytes(int D, int I) {
  const int xlen = M * (D > I ? D : I);
  size_t fl = (size_t)NW * NJMAX * M + NW * M * 2 + G * HD + G * CHUNK_MAX + (NW / 2) * G * HD + 2 * HD + 2 * G +
              NJMAX * M /*cand_v*/ + NJMAX * M /*cand_i*/ + 4;
  return (size_t)xlen * 2 * sizeof(u16) + fl * sizeof(float);
}

template <int M, int HD, int G>
static int launch_step(const StepParams& sp, hipStream_t s) {
  const size_t lds = lds_bytes<M, HD, G>(sp.D, sp.I);
  if (lds > 160 * 1024) return LR_E_UNSUPPORTED;
  static bool attr_set = false;
  if (!attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&k_ladder_step<M, HD, G>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess)
      return LR_E_LAUNCH;
    attr_set = true;
  }
  k_ladder_step<M, HD, G><<<dim3(num_cus()), dim3(NT), lds, s>>>(sp);
  return lr_launch_status();
}

int g_p1_pairs_per_wg = -1;  // tuning hook: pairs of w1 rows per workgroup handled in phase 1

}  // namespace

extern "C" void lr_ladder_step_tune(int p1_pairs_per_wg) { g_p1_pairs_per_wg = p1_pairs_per_wg; }

extern "C" size_t lr_ladder_step_workspace_bytes(const lr_ladder_model_t* md, int batch) {
  if (validate(md, batch) != LR_OK) return 0;
  return make_layout(md, batch, num_cus()).total;
}

extern "C" size_t lr_ladder_step_fail_offset(void) { return offsetof(Ctrl, fail); }

extern "C" int lr_ladder_step_init(const lr_ladder_model_t* md, int batch, void* workspace, size_t bytes,
                                   lr_stream_t stream) {
  const int rc = validate(md, batch);
  if (rc != LR_OK) return rc;
  LR_REQUIRE_PTR(workspace);
  if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0) return LR_E_ALIGN;
  if (bytes < make_layout(md, batch, num_cus()).total) return LR_E_SHAPE;
  k_step_init<<<dim3(1), dim3(256), 0, (hipStream_t)stream>>>(reinterpret_cast<Ctrl*>(workspace),
                                                             (unsigned)num_cus());
  return lr_launch_status();
}

extern "C" int lr_ladder_decode_step(const lr_ladder_model_t* md, int batch, const int32_t* tokens, int32_t* pos,
                                     void* logits, int64_t ldl, int32_t* next_token, int advance,
                                     int32_t* cur_token, int32_t* history, int64_t ld_hist, int hist_len, int pos0,
                                     void* workspace, size_t bytes, lr_stream_t stream) {
  const int rc = validate(md, batch);
  if (rc != LR_OK) return rc;
  LR_REQUIRE_PTR(workspace);
  LR_REQUIRE_PTR(logits);
  if (tokens == nullptr || pos == nullptr) return LR_E_NULL;
  if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0) return LR_E_ALIGN;
  const int nwg = num_cus();
  const Layout l = make_layout(md, batch, nwg);
  if (bytes < l.total || ldl < md->out_rows) return LR_E_SHAPE;
  if (history && (ld_hist < hist_len || hist_len <= 0)) return LR_E_SHAPE;
  unsigned char* ws = reinterpret_cast<unsigned char*>(workspace);
  StepParams sp;
  sp.D = md->dim; sp.L = md->n_layer; sp.Hkv = md->n_kv_head; sp.I = md->ffn; sp.V = md->out_rows;
  sp.vocab = md->vocab; sp.Smax = md->smax; sp.block_size = md->block_size; sp.B = batch;
  sp.NA = pick_na(md->smax, nwg);
  sp.nqkv = (md->n_head + 2 * md->n_kv_head) * md->head_dim;
  // balance phase 1 (wqkv + first P1 pairs of w1) against phase 2 (attention + the other pairs)
  int per_wg = g_p1_pairs_per_wg >= 0 ? g_p1_pairs_per_wg : ((md->ffn - sp.nqkv / 2) / 2 + nwg / 2) / nwg + 1;
  long long p1 = (long long)per_wg * nwg;
  if (p1 > md->ffn) p1 = md->ffn;
  if (p1 < 0) p1 = 0;
  sp.P1 = (int)p1;
  sp.eps = md->eps;
  sp.tok_emb = (const u16*)md->tok_embeddings; sp.final_norm = (const u16*)md->norm;
  sp.out_w = (const u16*)md->output; sp.rope = (const u16*)md->freqs_cis;
  sp.layers = reinterpret_cast<const LayerPtrs*>(md->layers_dev);
  sp.tokens = tokens; sp.pos = pos; sp.logits = (u16*)logits; sp.ldl = ldl;
  sp.next_token = next_token; sp.cur_token = cur_token; sp.history = history; sp.ld_hist = ld_hist;
  sp.hist_len = hist_len; sp.pos0 = pos0; sp.advance = advance;
  sp.ctrl = reinterpret_cast<Ctrl*>(ws + l.ctrl);
  sp.Rbuf = reinterpret_cast<float*>(ws + l.Rbuf); sp.abuf = reinterpret_cast<float*>(ws + l.abuf);
  sp.mbuf = reinterpret_cast<float*>(ws + l.mbuf); sp.qkv = reinterpret_cast<float*>(ws + l.qkv);
  sp.y = reinterpret_cast<float*>(ws + l.y); sp.act = reinterpret_cast<float*>(ws + l.act);
  sp.opart = reinterpret_cast<float*>(ws + l.opart); sp.mlpart = reinterpret_cast<float*>(ws + l.mlpart);
  sp.cand = reinterpret_cast<float*>(ws + l.cand);
  hipStream_t s = (hipStream_t)stream;
  const int G = md->n_head / md->n_kv_head, hd = md->head_dim;
#define LR_STEP(MV, HDV, GV) \
  if (batch == MV && hd == HDV && G == GV) return launch_step<MV, HDV, GV>(sp, s);
  LR_STEP_INSTANCES(LR_STEP)
#undef LR_STEP
  return LR_E_UNSUPPORTED;
}
