// One decode step of the Ladder model as ONE persistent kernel (batch 1 or 2).
//
// Why: at batch 1 a step streams 17 GB of weights through ~720 small dependent ops.  Launched
// one by one (even from a hipGraph) the ops pay a launch boundary each and the latency-bound
// ones (norms, RoPE, attention, combine) cost as much as the weight streaming.  Here one
// workgroup per CU (512 lanes = 8 waves) stays resident for the whole step and walks the layers;
// the workgroups synchronise through event counters built from relaxed agent-scope atomics (a
// 16-group arrival tree where latency matters: ~1.5 us on 256 CUs; acquire/release fences are
// avoided because they write back and invalidate the whole L2).
//
// The ladder schedule is what makes this wide: attention block t reads the residual stream
// WITHOUT the MLP output of layer t-1 (in the reference that output is still inside an
// all-reduce), so attention(t) and mlp(t-1) are independent and run side by side.  A "slot" t is,
// per workgroup,
//     join:  wait until a(t-1) and m(t-2) are complete                      [tree event, exposed]
//     residual adds + both RMSNorms (redundantly in every workgroup)
//     wqkv(t) rows                                  -> signal E_qkv
//     attention workgroups (a handful): wait E_qkv, attention(t) over their key range with K/V
//         held in registers, partial results       -> signal E_att
//     all other workgroups: w1(t-1) rows + SwiGLU   -> signal E_act    (18 us of streaming that
//         hides the attention latency chain)
//     wait E_att (long since signalled), merge the partial results, wo(t) rows
//     wait E_act (signalled a few us earlier), w2(t-1) rows               -> signal "slot done"
// so one exposed device-wide wait per layer instead of 9 kernel launches.
//
// Weight streaming does not stop at these edges: every wave walks its GEMV work as a sequence of
// "units" (16 rows x 1 KiB of one K-slice) and always has the NEXT unit's loads in flight while it
// multiplies the current one -- also when the next unit belongs to the next GEMV or sits behind a
// wait (the loads are issued before the wait), so HBM stays busy through reductions, epilogues,
// norms and synchronisation latency.
//
// Data that crosses workgroups inside the step (residual, partial sums, qkv, attention output,
// activations) lives in a small fp32 workspace and is only touched with buffer loads/stores
// carrying the sc1 (agent-coherent) policy bit, which bypass the non-coherent per-XCD L2 lines;
// the values stored are bf16-representable, i.e. rounded exactly where the eager reference
// rounds.  Weights, KV cache and logits use ordinary accesses (read-only, or produced for the
// next launch).  GEMV rows are dealt to workgroups round-robin so that the CUs working at the
// same time read neighbouring rows (HBM-channel friendly); inside a workgroup the waves split K,
// partial sums meet in LDS in a fixed order -- no float atomics, bit-reproducible.
//
// Every spin is bounded: on time-out a workgroup raises ctrl->fail and leaves; the others see the
// flag (or time out themselves), so the grid always drains.
#include "lr_common.h"

namespace {

constexpr int NT = 512;           // lanes per workgroup
constexpr int NW = NT / 64;       // waves per workgroup
constexpr int EV_GROUPS = 16;     // arrival-tree fan-in
constexpr int NJMAX = 64;         // GEMV rows a workgroup reduces per LDS round
constexpr int RB = 8;             // rows per unit (loads a wave issues together)
constexpr unsigned SPIN_LIMIT = 1u << 21;
constexpr int ATT_NI = 9;         // key iterations an attention wave keeps in registers
constexpr int NA_MAX = 16;        // attention workgroups (partial results merged by everyone)
constexpr int PROF_SLOTS = 4, PROF_POINTS = 12;
constexpr int AUX_SC1 = 16;       // buffer cache policy: agent scope

// A tree event: every participant arrives once per epoch; the last one raises the group flags.
struct TreeEv {
  unsigned root, _p0[31];
  unsigned gcount[EV_GROUPS][32];
  unsigned gflag[EV_GROUPS][32];
};

struct Ctrl {  // every hot word on its own 128-byte line
  TreeEv qkv;   // wqkv(t) rows of all workgroups are stored
  TreeEv slot;  // slot finished (a(t) and m(t-1) stored); also the closing barrier of the head
  unsigned att_count, _p2[31];  // flat arrival counters (waited on late, latency not critical)
  unsigned act_count, _p3[31];
  unsigned base_qkv, base_slot, base_att, base_act, _p4[28];  // epochs / arrivals consumed by earlier steps
  unsigned fail, _p5[31];
  unsigned nwg, _p6[31];
};

struct LayerPtrs {
  const u16 *wqkv, *wo, *w1, *w2, *attn_norm, *ffn_norm;
  u16 *k_cache, *v_cache;
};

struct StepParams {
  int D, L, Hkv, I, V, vocab, Smax, block_size, B, NA, nqkv;
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
  unsigned char* ws;  // workspace base (Ctrl at offset 0)
  unsigned ws_bytes;
  unsigned oR, oa, om, oqkv, oact, oopart, omlpart, ocand;  // exchange buffers, offsets in floats
  unsigned long long* prof;  // optional [nwg][PROF_SLOTS][PROF_POINTS] wall-clock stamps (100 MHz)
  int prof_t0;
};

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));

// ---- coherent (cross-workgroup) accesses: one buffer resource over the workspace, sc1 policy.
//      Ordinary (non-atomic) instructions, so a lane can have several in flight.
struct Coh {
  __amdgpu_buffer_rsrc_t r;
  __device__ __forceinline__ float ld(unsigned fo) const {
    return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, fo * 4, 0, AUX_SC1));
  }
  __device__ __forceinline__ void ld2(unsigned fo, float& a, float& b) const {  // fo % 2 == 0
    const u32x2_t v = __builtin_amdgcn_raw_buffer_load_b64(r, fo * 4, 0, AUX_SC1);
    a = __uint_as_float(v.x);
    b = __uint_as_float(v.y);
  }
  __device__ __forceinline__ void st(unsigned fo, float v) const {
    __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), r, fo * 4, 0, AUX_SC1);
  }
  __device__ __forceinline__ void ld8(unsigned fo, float* f) const {  // fo % 4 == 0
    const u32x4_t a = __builtin_amdgcn_raw_buffer_load_b128(r, fo * 4, 0, AUX_SC1);
    const u32x4_t b = __builtin_amdgcn_raw_buffer_load_b128(r, fo * 4 + 16, 0, AUX_SC1);
    f[0] = __uint_as_float(a.x); f[1] = __uint_as_float(a.y); f[2] = __uint_as_float(a.z); f[3] = __uint_as_float(a.w);
    f[4] = __uint_as_float(b.x); f[5] = __uint_as_float(b.y); f[6] = __uint_as_float(b.z); f[7] = __uint_as_float(b.w);
  }
  __device__ __forceinline__ void st8(unsigned fo, const float* f) const {
    u32x4_t a, b;
    a.x = __float_as_uint(f[0]); a.y = __float_as_uint(f[1]); a.z = __float_as_uint(f[2]); a.w = __float_as_uint(f[3]);
    b.x = __float_as_uint(f[4]); b.y = __float_as_uint(f[5]); b.z = __float_as_uint(f[6]); b.w = __float_as_uint(f[7]);
    __builtin_amdgcn_raw_buffer_store_b128(a, r, fo * 4, 0, AUX_SC1);
    __builtin_amdgcn_raw_buffer_store_b128(b, r, fo * 4 + 16, 0, AUX_SC1);
  }
};

__device__ __forceinline__ unsigned cldu(const unsigned* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void cstu(unsigned* p, unsigned v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned cadd(unsigned* p) {
  return __hip_atomic_fetch_add(p, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// All lanes: wait for this lane's outstanding memory operations, then meet.  After it, every
// coherent store issued by the workgroup has been acknowledged.
__device__ __forceinline__ void drain_and_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
}

// ---- tree event: signal (all workgroups, once per epoch) / wait.  Loads may be put in flight
//      between the two.  `epoch` values are consumed in order and never reused.
__device__ __forceinline__ void tree_signal(TreeEv* e, unsigned epoch) {
  drain_and_sync();
  if (threadIdx.x == 0) {
    const unsigned nwg = gridDim.x;
    const unsigned ngr = nwg < EV_GROUPS ? nwg : EV_GROUPS;
    const unsigned g = blockIdx.x % ngr;
    const unsigned gn = nwg / ngr + (g < nwg % ngr ? 1u : 0u);
    if (cadd(&e->gcount[g][0]) + 1u == epoch * gn) {
      if (cadd(&e->root) + 1u == epoch * ngr) {
        for (unsigned i = 0; i < ngr; ++i) cstu(&e->gflag[i][0], epoch);
      }
    }
  }
}

// Bounded spin of lane 0 until *word has reached `target` (wrap-safe); the whole workgroup learns
// the outcome.  Returns false if the step must be abandoned.
__device__ __forceinline__ bool spin_until(const unsigned* word, unsigned target, unsigned* fail, int* s_flag) {
  if (threadIdx.x == 0) {
    int ok = 1;
    unsigned spins = 0;
    while ((int)(cldu(word) - target) < 0) {
      if ((++spins & 1023u) == 0 && (spins > SPIN_LIMIT || cldu(fail))) {
        cstu(fail, 1u);
        ok = 0;
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    s_flag[0] = ok;
  }
  __syncthreads();
  return s_flag[0] != 0;
}

__device__ __forceinline__ bool tree_wait(TreeEv* e, unsigned epoch, unsigned* fail, int* s_flag) {
  const unsigned nwg = gridDim.x;
  const unsigned ngr = nwg < EV_GROUPS ? nwg : EV_GROUPS;
  return spin_until(&e->gflag[blockIdx.x % ngr][0], epoch, fail, s_flag);
}

// flat event: arrivals only add (no return value needed, nobody stalls on it)
__device__ __forceinline__ void flat_signal(unsigned* counter) {
  drain_and_sync();
  if (threadIdx.x == 0) (void)cadd(counter);
}

// ---- per-lane accumulators -> wave totals.  reduce8: afterwards lane 16*r holds sum(v[2r]) in z0
//      and sum(v[2r+1]) in z1.  (permlane swaps fold halves / odd-even rows, DPP folds a row.)
__device__ __forceinline__ void swap32(float& a, float& b) {
  const u32x2_t r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
  a = __uint_as_float(r.x);
  b = __uint_as_float(r.y);
}
__device__ __forceinline__ void swap16(float& a, float& b) {
  const u32x2_t r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
  a = __uint_as_float(r.x);
  b = __uint_as_float(r.y);
}
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
  return __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float row_sum16(float r) {  // every lane of a 16-lane row gets the row total
  r += dpp_mov<0x128>(r);  // row_ror:8
  r += dpp_mov<0x124>(r);  // row_ror:4
  r += dpp_mov<0x4e>(r);   // quad_perm [2,3,0,1]
  r += dpp_mov<0xb1>(r);   // quad_perm [1,0,3,2]
  return r;
}
__device__ __forceinline__ float half_row_sum8(float r) {  // every lane of an 8-lane group gets the group total
  r += dpp_mov<0x4e>(r);
  r += dpp_mov<0xb1>(r);
  r += dpp_mov<0x141>(r);  // row_half_mirror
  return r;
}
__device__ __forceinline__ void reduce8(float* v, float& z0, float& z1) {
  float w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    swap32(v[i], v[i + 4]);
    w[i] = v[i] + v[i + 4];
  }
  swap16(w[0], w[2]);
  swap16(w[1], w[3]);
  z0 = row_sum16(w[0] + w[2]);
  z1 = row_sum16(w[1] + w[3]);
}

// ------------------------------------------------------------------------------------------------
// GEMV work of one workgroup in one matrix ("job").  Items (rows, or up/gate row pairs) are dealt
// round-robin over the `nwg` participating workgroups: participant w owns items w, w + nwg, ...
// Its rows are reduced in rounds of NJMAX; inside a round wave (rg, kg) owns rows j = rg (mod nrg)
// and K-slices kk = kg (mod nkg), RB rows x one 512-element slice per unit.
// ------------------------------------------------------------------------------------------------
struct Job {
  const u16* W;
  int K, row_base, n_items, pair_off, rpi;  // rpi: rows per item (1, or 2 for up/gate pairs)
  int w, nwg;                               // this workgroup's rank among the participants
  int nj, ksteps, nkg, nrg, rg, kg;         // derived for this workgroup / wave
  bool active;
};

__device__ __forceinline__ Job make_job(const u16* W, int K, int row_base, int n_items, int pair_off, int rpi,
                                        int w, int nwg, int wave) {
  Job j;
  j.W = W; j.K = K; j.row_base = row_base; j.n_items = n_items; j.pair_off = pair_off; j.rpi = rpi;
  j.w = w; j.nwg = nwg;
  const int nit = (W != nullptr && w >= 0 && n_items > w) ? (n_items - w + nwg - 1) / nwg : 0;
  j.nj = nit * rpi;
  j.ksteps = (K + 511) >> 9;
  j.nkg = j.ksteps < NW ? j.ksteps : NW;
  j.nrg = NW / j.nkg;
  j.rg = wave / j.nkg;
  j.kg = wave - j.rg * j.nkg;
  j.active = wave < j.nrg * j.nkg && j.rg < (j.nj < NJMAX ? j.nj : NJMAX);
  return j;
}

struct Unit {
  uint4 r[RB];
};

// Issue the loads of unit (j0, jb, kk) of `job`.  Rows beyond the round and columns beyond K are
// clamped to valid addresses: their products are discarded / multiplied by a zero x.
__device__ __forceinline__ void load_unit(const Job& job, int j0, int jb, int kk, int lane, Unit& u) {
  const int njb = job.nj - j0 < NJMAX ? job.nj - j0 : NJMAX;
  int k = kk * 512 + lane * 8;
  k = k < job.K ? k : 0;
#pragma unroll
  for (int i = 0; i < RB; ++i) {
    int j = jb + i * job.nrg;
    j = j < njb ? j : njb - 1;
    const int jj = j0 + j;
    const int row = job.row_base + job.w + job.nwg * (jj / job.rpi) + (jj % job.rpi) * job.pair_off;
    u.r[i] = ld16(job.W + (int64_t)row * job.K + k);
  }
}

__device__ __forceinline__ void first_unit(const Job& job, int lane, Unit& u) {
  if (job.active) {
    load_unit(job, 0, job.rg, job.kg, lane, u);
  } else {  // a defined value everywhere: ends the live range of whatever `u` held before
#pragma unroll
    for (int i = 0; i < RB; ++i) u.r[i] = make_uint4(0, 0, 0, 0);
  }
}

enum { EPI_STORE = 0, EPI_SWIGLU = 1, EPI_LOGITS = 2 };

// Run one job.  On entry `cur` holds this wave's first unit of the job (if it has one); on exit it
// holds the first unit of `next` (if the wave has one there) -- issued before this job's last
// reduction and epilogue.
template <int M, int EPI>
__device__ __forceinline__ void run_job(const StepParams& p, const Coh& coh, const Job& job, const Job& next,
                                        Unit& cur, const u16* x, float* part, unsigned out_fo, int ldo, float* cand_v,
                                        int* cand_i, float* best_v, int* best_i) {
  const int tid = threadIdx.x, lane = tid & 63;
  const int RPI = job.rpi;
  if (!job.active) first_unit(next, lane, cur);
  for (int j0 = 0; j0 < job.nj; j0 += NJMAX) {
    const int njb = job.nj - j0 < NJMAX ? job.nj - j0 : NJMAX;
    if (job.active && job.rg < njb) {
      for (int jb = job.rg; jb < njb; jb += job.nrg * RB) {
        float acc[M][RB];
#pragma unroll
        for (int m = 0; m < M; ++m)
#pragma unroll
          for (int i = 0; i < RB; ++i) acc[m][i] = 0.0f;
        for (int kk = job.kg; kk < job.ksteps; kk += job.nkg) {
          // ---- put the following unit in flight
          Unit nxt;
          if (kk + job.nkg < job.ksteps) load_unit(job, j0, jb, kk + job.nkg, lane, nxt);
          else if (jb + job.nrg * RB < njb) load_unit(job, j0, jb + job.nrg * RB, job.kg, lane, nxt);
          else if (j0 + NJMAX < job.nj && job.rg < job.nj - j0 - NJMAX)
            load_unit(job, j0 + NJMAX, job.rg, job.kg, lane, nxt);
          else first_unit(next, lane, nxt);
          // ---- multiply the current one
          const int k = kk * 512 + lane * 8;
          const bool kv = k < job.K;
          float xf[M][8];
#pragma unroll
          for (int m = 0; m < M; ++m)
            unpack8(kv ? *reinterpret_cast<const uint4*>(x + m * job.K + k) : make_uint4(0, 0, 0, 0), xf[m]);
#pragma unroll
          for (int i = 0; i < RB; ++i) {
            float wf[8];
            unpack8(cur.r[i], wf);
#pragma unroll
            for (int m = 0; m < M; ++m)
#pragma unroll
              for (int e = 0; e < 8; ++e) acc[m][i] = fmaf(wf[e], xf[m][e], acc[m][i]);
            __builtin_amdgcn_sched_barrier(0);  // keep the unpacked row short-lived (register pressure)
          }
#pragma unroll
          for (int i = 0; i < RB; ++i) cur.r[i] = nxt.r[i];
        }
#pragma unroll
        for (int m = 0; m < M; ++m)
#pragma unroll
          for (int h = 0; h < RB / 8; ++h) {
            float z0, z1;
            reduce8(&acc[m][8 * h], z0, z1);
            if ((lane & 15) == 0) {
              const int r = lane >> 4;
              const int ja = jb + (8 * h + 2 * r) * job.nrg, jc = jb + (8 * h + 2 * r + 1) * job.nrg;
              if (ja < njb) part[(job.kg * NJMAX + ja) * M + m] = z0;
              if (jc < njb) part[(job.kg * NJMAX + jc) * M + m] = z1;
            }
          }
      }
    }
    __syncthreads();
    // ---- cross-wave sum in fixed order + epilogue
    const int nout = (njb / RPI) * M;
    if (tid < nout) {
      const int jl = tid / M, m = tid - jl * M;
      float s0, s1 = 0.0f;
      {
        float t = 0.0f;
        for (int g = 0; g < job.nkg; ++g) t += part[(g * NJMAX + jl * RPI) * M + m];
        s0 = round_bf(t);
      }
      if (EPI == EPI_SWIGLU) {
        float t = 0.0f;
        for (int g = 0; g < job.nkg; ++g) t += part[(g * NJMAX + jl * RPI + 1) * M + m];
        s1 = round_bf(t);
      }
      const int it = job.w + job.nwg * ((j0 / RPI) + jl);
      if (m < p.B) {
        if (EPI == EPI_STORE) coh.st(out_fo + (unsigned)(m * ldo + it), s0);
        if (EPI == EPI_SWIGLU) coh.st(out_fo + (unsigned)(m * ldo + it), swiglu_bf(s0, s1));
        if (EPI == EPI_LOGITS) p.logits[(int64_t)m * p.ldl + it] = f_to_bf(s0);
      }
      if (EPI == EPI_LOGITS) {
        cand_v[tid] = s0;
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
// Residual bookkeeping + RMSNorm for the coming jobs, done redundantly by every workgroup:
//   v1 = src (+ d1);  v2 = v1 (+ d2);  each add rounded to bf16.
//   x1 = norm(v1) * g1 -> LDS (if g1);  x2 = norm(v2) * g2 -> LDS (if g2);  workgroup 0 stores v2.
// src is either the coherent fp32 residual or rows of the bf16 embedding table.
// ------------------------------------------------------------------------------------------------
template <int M>
__device__ __forceinline__ void prologue(const StepParams& p, const Coh& coh, unsigned src_fo, const int* emb_rows,
                                         bool has_d1, unsigned d1_fo, bool has_d2, unsigned d2_fo, const u16* g1,
                                         const u16* g2, bool write_r, unsigned rout_fo, u16* x1, u16* x2, float* red) {
  const int tid = threadIdx.x, D = p.D;
  float ss1[M], ss2[M];
  // pass 1: the (bf16-exact) sums go to LDS unscaled; sums of squares per lane
#pragma unroll
  for (int m = 0; m < M; ++m) {
    ss1[m] = ss2[m] = 0.0f;
    for (int c = tid * 8; c < D; c += NT * 8) {
      float v[8], t1[8], t2[8];
      if (emb_rows) {
        const int id = emb_rows[m];
        const bool ok = id >= 0 && id < p.vocab;
        unpack8(ok ? ld16(p.tok_emb + (int64_t)id * D + c) : make_uint4(0, 0, 0, 0), v);
      } else {
        coh.ld8(src_fo + m * D + c, v);
      }
      if (has_d1) coh.ld8(d1_fo + m * D + c, t1);
      if (has_d2) coh.ld8(d2_fo + m * D + c, t2);
      if (has_d1) {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = round_bf(v[j] + t1[j]);
      }
      if (g1) st16(x1 + m * D + c, pack8(v));
#pragma unroll
      for (int j = 0; j < 8; ++j) ss1[m] += v[j] * v[j];
      if (has_d2) {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = round_bf(v[j] + t2[j]);
      }
      if (g2) st16(x2 + m * D + c, pack8(v));
#pragma unroll
      for (int j = 0; j < 8; ++j) ss2[m] += v[j] * v[j];
      if (write_r && blockIdx.x == 0) coh.st8(rout_fo + m * D + c, v);
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
  // pass 2: scale in place (each lane revisits the elements it wrote)
#pragma unroll
  for (int m = 0; m < M; ++m) {
    float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
    for (int wv = 0; wv < NW; ++wv) {
      s1 += red[(wv * M + m) * 2];
      s2 += red[(wv * M + m) * 2 + 1];
    }
    const float inv1 = rsqrtf(s1 / (float)D + p.eps), inv2 = rsqrtf(s2 / (float)D + p.eps);
    for (int c = tid * 8; c < D; c += NT * 8) {
      float v[8], g[8], o[8];
      if (g1) {
        unpack8(*reinterpret_cast<const uint4*>(x1 + m * D + c), v);
        unpack8(ld16(g1 + c), g);
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = round_bf(v[j] * inv1) * g[j];
        st16(x1 + m * D + c, pack8(o));
      }
      if (g2) {
        unpack8(*reinterpret_cast<const uint4*>(x2 + m * D + c), v);
        unpack8(ld16(g2 + c), g);
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = round_bf(v[j] * inv2) * g[j];
        st16(x2 + m * D + c, pack8(o));
      }
    }
  }
  __syncthreads();
}

// Bring a coherent fp32 activation [M][K] (bf16-representable values) into LDS as bf16.
template <int M>
__device__ __forceinline__ void load_x(const Coh& coh, unsigned src_fo, int K, u16* x) {
  for (int c = threadIdx.x * 8; c < M * K; c += NT * 8) {
    float f[8];
    coh.ld8(src_fo + c, f);
    st16(x + c, pack8(f));
  }
  __syncthreads();
}

// ------------------------------------------------------------------------------------------------
// Attention of slot t in attention workgroup `aw` of NA: keys [k0, k1) of every (sequence, kv
// head), all G q heads of the kv head at once so K and V are read once per GQA group.  The K and V
// rows of the key range are loaded into registers in one go (before the wait for qkv), scores,
// softmax and P.V stay in fp32; each workgroup publishes an un-normalised partial result with its
// own (max, sum).
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ void rope_pair(float x0, float x1, float c, float s, float& o0, float& o1) {
#pragma clang fp contract(off)
  const float a = x0 * c, b = x1 * s, d = x1 * c, e = x0 * s;
  o0 = round_bf(a - b);
  o1 = round_bf(d + e);
}

template <int HD>
struct KV {
  uint4 k[ATT_NI], v[ATT_NI];
};

template <int HD>
__device__ __forceinline__ void attention_load(const StepParams& p, const LayerPtrs& lp, int b, int kvh, int k0,
                                               int k1, int pos, KV<HD>& kv) {
  constexpr int LPK = HD / 8, KPW = 64 / LPK;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int kl = lane / LPK, dl = (lane % LPK) * 8;
  const u16* kbase = lp.k_cache + ((int64_t)b * p.Hkv + kvh) * p.Smax * HD;
  const u16* vbase = lp.v_cache + ((int64_t)b * p.Hkv + kvh) * p.Smax * HD;
#pragma unroll
  for (int i = 0; i < ATT_NI; ++i) {
    const int key = k0 + (i * NW + wave) * KPW + kl;
    const bool live = key < k1 && key != pos;  // the slot of `pos` is filled from this step's qkv
    kv.k[i] = live ? ld16(kbase + (int64_t)key * HD + dl) : make_uint4(0, 0, 0, 0);
  }
#pragma unroll
  for (int i = 0; i < ATT_NI; ++i) {
    const int key = k0 + (i * NW + wave) * KPW + kl;
    const bool live = key < k1 && key != pos;
    kv.v[i] = live ? ld16(vbase + (int64_t)key * HD + dl) : make_uint4(0, 0, 0, 0);
  }
}

template <int M, int HD, int G>
__device__ __forceinline__ void attention_compute(const StepParams& p, const Coh& coh, const LayerPtrs& lp, int b,
                                                  int kvh, int k0, int k1, int pos, KV<HD>& kv, float* qs, float* sc,
                                                  int sc_ld, float* ored, float* knew, float* vnew, float* s_m,
                                                  float* s_l) {
  constexpr int LPK = HD / 8, KPW = 64 / LPK;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int aw = blockIdx.x, NA = p.NA, Hkv = p.Hkv, Hq = Hkv * G;
  const int n = k1 - k0;
  const bool owner = pos >= k0 && pos < k1;
  const float scale = rsqrtf((float)HD);
  const u16* trow = p.rope + (int64_t)pos * HD;  // (cos, sin) pairs of this position
  const int kl = lane / LPK, dl = (lane % LPK) * 8;
  const unsigned qkv = p.oqkv + (unsigned)(b * p.nqkv);
  const unsigned o_out = p.oopart + (unsigned)((((b * Hq + kvh * G) * NA) + aw) * HD);
  const unsigned ml_out = p.omlpart + (unsigned)((((b * Hq + kvh * G) * NA) + aw) * 2);

  // ---- rotate q (all G heads) into LDS; the owner of `pos` also rotates k, keeps k/v in LDS and
  //      writes them to the cache for the following steps
  for (int i = tid; i < G * HD / 2; i += NT) {
    const int g = i / (HD / 2), j = i - g * (HD / 2);
    float x0, x1;
    coh.ld2(qkv + (unsigned)((kvh * G + g) * HD + 2 * j), x0, x1);
    const u32 cs = *reinterpret_cast<const u32*>(trow + 2 * j);
    rope_pair(x0, x1, bf_lo(cs), bf_hi(cs), qs[g * HD + 2 * j], qs[g * HD + 2 * j + 1]);
  }
  if (owner && tid < HD / 2) {
    const int j = tid;
    float kx0, kx1, v0, v1, r0, r1;
    coh.ld2(qkv + (unsigned)(Hq * HD + kvh * HD + 2 * j), kx0, kx1);
    coh.ld2(qkv + (unsigned)((Hq + Hkv) * HD + kvh * HD + 2 * j), v0, v1);
    const u32 cs = *reinterpret_cast<const u32*>(trow + 2 * j);
    rope_pair(kx0, kx1, bf_lo(cs), bf_hi(cs), r0, r1);
    knew[2 * j] = r0; knew[2 * j + 1] = r1;
    vnew[2 * j] = v0; vnew[2 * j + 1] = v1;
    const int64_t slot = (((int64_t)b * Hkv + kvh) * p.Smax + pos) * HD + 2 * j;
    *reinterpret_cast<u32*>(lp.k_cache + slot) = pack_bf2(r0, r1);
    *reinterpret_cast<u32*>(lp.v_cache + slot) = pack_bf2(v0, v1);
  }
  __syncthreads();
  if (n <= 0) {
    for (int i = tid; i < G * HD; i += NT) coh.st(o_out + (unsigned)((i / HD) * NA * HD + (i % HD)), 0.0f);
    if (tid < G) {
      coh.st(ml_out + (unsigned)(tid * NA * 2), -INFINITY);
      coh.st(ml_out + (unsigned)(tid * NA * 2 + 1), 0.0f);
    }
    __syncthreads();
    return;
  }
  // ---- scores
  {
    float qf[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int j = 0; j < 8; ++j) qf[g][j] = qs[g * HD + dl + j];
#pragma unroll
    for (int i = 0; i < ATT_NI; ++i) {
      const int key = k0 + (i * NW + wave) * KPW + kl;
      float kf[8];
      unpack8(kv.k[i], kf);
      if (key == pos) {
#pragma unroll
        for (int j = 0; j < 8; ++j) kf[j] = knew[dl + j];
      }
#pragma unroll
      for (int g = 0; g < G; ++g) {
        float s = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) s = fmaf(kf[j], qf[g][j], s);
        s = LPK == 16 ? row_sum16(s) : half_row_sum8(s);
        if (key < k1 && (lane % LPK) == 0) sc[g * sc_ld + key - k0] = s * scale;
      }
    }
  }
  __syncthreads();
  // ---- softmax statistics: a wave per head; sc becomes exp(s - max)
  for (int g = wave; g < G; g += NW) {
    float m = -INFINITY;
    for (int i = lane; i < n; i += 64) m = fmaxf(m, sc[g * sc_ld + i]);
    m = wave_max(m);
    float l = 0.0f;
    for (int i = lane; i < n; i += 64) {
      const float e = expf(sc[g * sc_ld + i] - m);
      sc[g * sc_ld + i] = e;
      l += e;
    }
    l = wave_sum(l);
    if (lane == 0) { s_m[g] = m; s_l[g] = l; }
  }
  __syncthreads();
  // ---- P.V, folded over the key groups of a wave, then over the waves in two LDS rounds
  float acc[G][8];
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[g][j] = 0.0f;
#pragma unroll
  for (int i = 0; i < ATT_NI; ++i) {
    const int key = k0 + (i * NW + wave) * KPW + kl;
    if (key < k1) {
      float vf[8];
      unpack8(kv.v[i], vf);
      if (key == pos) {
#pragma unroll
        for (int j = 0; j < 8; ++j) vf[j] = vnew[dl + j];
      }
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const float pr = sc[g * sc_ld + key - k0];
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[g][j] = fmaf(pr, vf[j], acc[g][j]);
      }
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
    coh.st(o_out + (unsigned)((i / HD) * NA * HD + (i % HD)), v);
  }
  if (tid < G) {
    coh.st(ml_out + (unsigned)(tid * NA * 2), s_m[tid]);
    coh.st(ml_out + (unsigned)(tid * NA * 2 + 1), s_l[tid]);
  }
  __syncthreads();
}

// Every workgroup: merge the NA partial attention results into y [M][Hq * HD] (bf16, LDS).
//   y = sum_s w_s o_s,  w_s = exp(m_s - max) / sum_s' exp(m_s' - max) l_s'
template <int M, int HD>
__device__ __forceinline__ void attention_merge(const StepParams& p, const Coh& coh, int Hq, u16* y, float* wbuf) {
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int NA = p.NA, nbh = p.B * Hq;
  const int npairs = nbh * HD / 2;
  float o0[NA_MAX], o1[NA_MAX];
  // the first batch of partial outputs goes in flight together with the (max, sum) pairs
  int pp = tid;
  if (pp < npairs) {
    const int bh = (2 * pp) / HD, d = (2 * pp) % HD;
#pragma unroll
    for (int s = 0; s < NA_MAX; ++s) {
      o0[s] = o1[s] = 0.0f;
      if (s < NA) coh.ld2(p.oopart + (unsigned)((bh * NA + s) * HD + d), o0[s], o1[s]);
    }
  }
  // weights: a wave per (sequence, head); lanes < NA hold one chunk each
  for (int bh = wave; bh < nbh; bh += NW) {
    float m = -INFINITY, l = 0.0f;
    if (lane < NA) coh.ld2(p.omlpart + (unsigned)((bh * NA + lane) * 2), m, l);
    const float mx = wave_max(m);
    const float w = m == -INFINITY ? 0.0f : expf(m - mx);
    const float L = wave_sum(w * l);
    if (lane < NA) wbuf[bh * NA_MAX + lane] = L > 0.0f ? w / L : 0.0f;
  }
  __syncthreads();
  while (pp < npairs) {
    const int bh = (2 * pp) / HD;
    float y0 = 0.0f, y1 = 0.0f;
#pragma unroll
    for (int s = 0; s < NA_MAX; ++s) {
      if (s < NA) {
        const float w = wbuf[bh * NA_MAX + s];
        y0 = fmaf(w, o0[s], y0);
        y1 = fmaf(w, o1[s], y1);
      }
    }
    *reinterpret_cast<u32*>(y + 2 * pp) = pack_bf2(y0, y1);
    pp += NT;
    if (pp < npairs) {
      const int bh2 = (2 * pp) / HD, d2 = (2 * pp) % HD;
#pragma unroll
      for (int s = 0; s < NA_MAX; ++s)
        if (s < NA) coh.ld2(p.oopart + (unsigned)((bh2 * NA + s) * HD + d2), o0[s], o1[s]);
    }
  }
  __syncthreads();
}

// ------------------------------------------------------------------------------------------------
template <int M, int HD, int G>
__global__ __launch_bounds__(NT) void k_ladder_step(const StepParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int D = p.D, L = p.L, Hq = p.Hkv * G, I = p.I;
  // ---- LDS carve-up
  const int xlen = M * (D > I ? D : I);
  const int sc_ld = ATT_NI * NW * (64 / (HD / 8));      // keys an attention workgroup can hold
  u16* xa = reinterpret_cast<u16*>(smem);              // attention-chain input  [M][<= D]
  u16* xb = xa + xlen;                                  // MLP-chain input        [M][<= D]
  float* part = reinterpret_cast<float*>(xb + xlen);    // [NW][NJMAX * M]
  float* red = part + NW * NJMAX * M;                   // [NW][M][2]
  float* qs = red + NW * M * 2;                         // [G][HD]
  float* sc = qs + G * HD;                              // [G][sc_ld]
  float* ored = sc + G * sc_ld;                         // [NW/2][G][HD]
  float* knew = ored + (NW / 2) * G * HD;               // [HD]
  float* vnew = knew + HD;                              // [HD]
  float* s_m = vnew + HD;                               // [G]
  float* s_l = s_m + G;                                 // [G]
  float* wbuf = s_l + G;                                // [M * Hq][NA_MAX]
  float* cand_v = wbuf + M * Hq * NA_MAX;               // [NJMAX * M]
  int* cand_i = reinterpret_cast<int*>(cand_v + NJMAX * M);
  int* s_flag = cand_i + NJMAX * M;                     // [8]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int w = blockIdx.x, nwg = gridDim.x, NA = p.NA;
  Ctrl* ctrl = reinterpret_cast<Ctrl*>(p.ws);
  Coh coh;
  coh.r = __builtin_amdgcn_make_buffer_rsrc(p.ws, 0, (int)p.ws_bytes, 0x00020000);
  if (tid == 0) {
    s_flag[1] = (int)cldu(&ctrl->base_qkv);
    s_flag[2] = (int)cldu(&ctrl->base_slot);
    s_flag[3] = (int)cldu(&ctrl->base_att);
    s_flag[4] = (int)cldu(&ctrl->base_act);
  }
  __syncthreads();
  const unsigned base_qkv = (unsigned)s_flag[1], base_slot = (unsigned)s_flag[2];
  const unsigned base_att = (unsigned)s_flag[3], base_act = (unsigned)s_flag[4];
  __syncthreads();
  int pos = p.pos[0];
  pos = pos < 0 ? 0 : (pos >= p.Smax ? p.Smax - 1 : pos);
  const bool att_wg = w < NA;
  // attention key range of this workgroup
  const int nkeys = pos + 1;
  const int chunk = (nkeys + NA - 1) / NA;
  const int k0 = w * chunk;
  const int k1 = k0 + chunk < nkeys ? k0 + chunk : nkeys;

  const Job none = make_job(nullptr, 512, 0, 0, 0, 1, 0, 1, wave);
  Unit cur;
  first_unit(make_job(p.layers[0].wqkv, D, 0, p.nqkv, 0, 1, w, nwg, wave), lane, cur);

#define LR_STAMP(k)                                                                                  \
  if (p.prof && t >= p.prof_t0 && t < p.prof_t0 + PROF_SLOTS && tid == 0)                            \
    p.prof[((size_t)blockIdx.x * PROF_SLOTS + (t - p.prof_t0)) * PROF_POINTS + (k)] = wall_clock64();
  for (int t = 0; t <= L; ++t) {
    const bool has_a = t < L, has_b = t >= 1;
    const LayerPtrs la = p.layers[has_a ? t : L - 1];
    const LayerPtrs lb = p.layers[has_b ? t - 1 : 0];
    // jobs of this slot in execution order (absent ones own no rows).  w1 is dealt to the
    // workgroups that do not run attention in this slot.
    const Job j_qkv = has_a ? make_job(la.wqkv, D, 0, p.nqkv, 0, 1, w, nwg, wave) : none;
    const Job j_w1 = !has_b ? none
                            : (has_a ? make_job(lb.w1, D, 0, I, I, 2, w - NA, nwg - NA, wave)
                                     : make_job(lb.w1, D, 0, I, I, 2, w, nwg, wave));
    const Job j_wo = has_a ? make_job(la.wo, Hq * HD, 0, D, 0, 1, w, nwg, wave) : none;
    const Job j_w2 = has_b ? make_job(lb.w2, I, 0, D, 0, 1, w, nwg, wave) : none;
    const Job j_nxt = t + 1 < L ? make_job(p.layers[t + 1].wqkv, D, 0, p.nqkv, 0, 1, w, nwg, wave)
                                : (t + 1 == L ? make_job(p.layers[L - 1].w1, D, 0, I, I, 2, w, nwg, wave)
                                              : make_job(p.out_w, D, 0, p.V, 0, 1, w, nwg, wave));
    LR_STAMP(0)
    // ---------------- v1 = R + m(t-2) feeds mlp(t-1); v2 = v1 + a(t-1) feeds attention(t)
    prologue<M>(p, coh, p.oR + (unsigned)(((t + 1) & 1) * M * D), t == 0 ? p.tokens : nullptr, t >= 2, p.om,
                t >= 1 && has_a, p.oa, has_b ? lb.ffn_norm : nullptr, has_a ? la.attn_norm : nullptr, true,
                p.oR + (unsigned)((t & 1) * M * D), xb, xa, red);
    LR_STAMP(1)
    run_job<M, EPI_STORE>(p, coh, j_qkv, j_w1, cur, xa, part, p.oqkv, p.nqkv, nullptr, nullptr, nullptr, nullptr);
    LR_STAMP(2)
    if (has_a) tree_signal(&ctrl->qkv, base_qkv + (unsigned)t + 1u);
    if (has_a && att_wg) {
      // ---------------- attention workgroup: K/V of (sequence 0, head 0) go in flight, then wait for qkv
      KV<HD> kv;
      attention_load<HD>(p, la, 0, 0, k0, k1, pos, kv);
      if (!tree_wait(&ctrl->qkv, base_qkv + (unsigned)t + 1u, &ctrl->fail, s_flag)) return;
      LR_STAMP(3)
      for (int b = 0; b < p.B; ++b)
        for (int kvh = 0; kvh < p.Hkv; ++kvh) {
          if (b + kvh > 0) attention_load<HD>(p, la, b, kvh, k0, k1, pos, kv);
          attention_compute<M, HD, G>(p, coh, la, b, kvh, k0, k1, pos, kv, qs, sc, sc_ld, ored, knew, vnew, s_m, s_l);
        }
      flat_signal(&ctrl->att_count);
      first_unit(j_wo, lane, cur);
      LR_STAMP(4)
    } else {
      // ---------------- everyone else: the up/gate projection of the previous layer + SwiGLU
      LR_STAMP(3)
      run_job<M, EPI_SWIGLU>(p, coh, j_w1, has_a ? j_wo : j_w2, cur, xb, part, p.oact, I, nullptr, nullptr, nullptr,
                             nullptr);
      LR_STAMP(4)
    }
    if (has_b) flat_signal(&ctrl->act_count);
    LR_STAMP(5)
    // ---------------- merge attention partials, output projection
    if (has_a) {
      if (!spin_until(&ctrl->att_count, base_att + (unsigned)(t + 1) * (unsigned)NA, &ctrl->fail, s_flag)) return;
      LR_STAMP(6)
      attention_merge<M, HD>(p, coh, Hq, xa, wbuf);
      LR_STAMP(7)
      run_job<M, EPI_STORE>(p, coh, j_wo, j_w2, cur, xa, part, p.oa, D, nullptr, nullptr, nullptr, nullptr);
    }
    LR_STAMP(8)
    // ---------------- down projection of the previous layer
    if (has_b) {
      if (!spin_until(&ctrl->act_count, base_act + (unsigned)t * (unsigned)nwg, &ctrl->fail, s_flag)) return;
      load_x<M>(coh, p.oact, I, xb);
      run_job<M, EPI_STORE>(p, coh, j_w2, none, cur, xb, part, p.om, D, nullptr, nullptr, nullptr, nullptr);
    }
    LR_STAMP(9)
    tree_signal(&ctrl->slot, base_slot + (unsigned)t + 1u);
    first_unit(j_nxt, lane, cur);  // next slot's first weights, in flight across the join
    if (!tree_wait(&ctrl->slot, base_slot + (unsigned)t + 1u, &ctrl->fail, s_flag)) return;
    LR_STAMP(10)
  }
#undef LR_STAMP
  // ---------------- head: x = (R + a) + m, final norm, vocab-shard lm_head, argmax
  prologue<M>(p, coh, p.oR + (unsigned)((L & 1) * M * D), nullptr, true, p.oa, true, p.om, nullptr, p.final_norm,
              false, 0u, xb, xa, red);
  float best_v = -INFINITY;
  int best_i = 0x7fffffff;
  run_job<M, EPI_LOGITS>(p, coh, make_job(p.out_w, D, 0, p.V, 0, 1, w, nwg, wave), none, cur, xa, part, 0u, 0, cand_v,
                         cand_i, &best_v, &best_i);
  if (tid < M) {
    coh.st(p.ocand + (unsigned)((w * M + tid) * 2), best_v);
    coh.st(p.ocand + (unsigned)((w * M + tid) * 2 + 1), __int_as_float(best_i));
  }
  tree_signal(&ctrl->slot, base_slot + (unsigned)L + 2u);
  if (!tree_wait(&ctrl->slot, base_slot + (unsigned)L + 2u, &ctrl->fail, s_flag)) return;
  if (w == 0) {
    if (tid < p.B) {
      float bv = -INFINITY;
      int bi = 0x7fffffff;
      for (int wg = 0; wg < nwg; ++wg) {
        float v, fi;
        coh.ld2(p.ocand + (unsigned)((wg * M + tid) * 2), v, fi);
        const int i = __float_as_int(fi);
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
      cstu(&ctrl->base_qkv, base_qkv + (unsigned)L);
      cstu(&ctrl->base_slot, base_slot + (unsigned)L + 2u);
      cstu(&ctrl->base_att, base_att + (unsigned)L * (unsigned)NA);
      cstu(&ctrl->base_act, base_act + (unsigned)L * (unsigned)nwg);
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
  size_t ctrl, Rbuf, abuf, mbuf, qkv, act, opart, mlpart, cand, total;
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

// keys one attention workgroup can hold in registers
static int att_capacity(int hd) { return ATT_NI * NW * (64 / (hd / 8)); }

int g_na_override = -1;  // tuning hook: number of attention workgroups (must still cover Smax)

static int pick_na(int Smax, int hd, int nwg) {
  const int cap = att_capacity(hd);
  int na = (Smax + cap - 1) / cap;
  if (g_na_override > na) na = g_na_override;
  if (na < 1) na = 1;
  if (na >= nwg) na = nwg - 1;
  return na;
}

static Layout make_layout(const lr_ladder_model_t* md, int B, int nwg) {
  const int D = md->dim, Hq = md->n_head, hd = md->head_dim;
  const int nqkv = (Hq + 2 * md->n_kv_head) * hd;
  const int na = pick_na(md->smax, hd, nwg);
  auto up = [](size_t x) { return (x + 255) & ~(size_t)255; };
  Layout l;
  size_t o = 0;
  l.ctrl = o; o = up(o + sizeof(Ctrl));
  l.Rbuf = o; o = up(o + sizeof(float) * 2 * B * D);
  l.abuf = o; o = up(o + sizeof(float) * B * D);
  l.mbuf = o; o = up(o + sizeof(float) * B * D);
  l.qkv = o; o = up(o + sizeof(float) * B * nqkv);
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

template <int M, int HD, int G>
static size_t lds_bytes(int D, int I, int Hq) {
  const int xlen = M * (D > I ? D : I);
  const size_t fl = (size_t)NW * NJMAX * M + NW * M * 2 + G * HD + (size_t)G * att_capacity(HD) + (NW / 2) * G * HD +
                    2 * HD + 2 * G + (size_t)M * Hq * NA_MAX + 2 * NJMAX * M + 8;
  return (size_t)xlen * 2 * sizeof(u16) + fl * sizeof(float);
}

static size_t lds_need(int B, int hd, int G, int D, int I, int Hq) {
#define LR_LDS(MV, HDV, GV) if (B == MV && hd == HDV && G == GV) return lds_bytes<MV, HDV, GV>(D, I, Hq);
  LR_STEP_INSTANCES(LR_LDS)
#undef LR_LDS
  return ~(size_t)0;
}

static int validate(const lr_ladder_model_t* md, int B) {
  if (md == nullptr) return LR_E_NULL;
  if (B < 1 || md->dim <= 0 || md->n_layer <= 0 || md->n_head <= 0 || md->n_kv_head <= 0 || md->ffn <= 0 ||
      md->out_rows <= 0 || md->vocab <= 0 || md->smax <= 0 || md->block_size <= 0 || md->n_head % md->n_kv_head)
    return LR_E_SHAPE;
  if (B > 2 || md->dim > 16384 || md->dim % 8 || md->ffn % 8 || (md->head_dim != 64 && md->head_dim != 128))
    return LR_E_UNSUPPORTED;
  const int G = md->n_head / md->n_kv_head;
  if (!has_instance(B, md->head_dim, G)) return LR_E_UNSUPPORTED;
  if (md->n_head * md->head_dim > 16384 || md->ffn > 16384) return LR_E_UNSUPPORTED;
  if (lds_need(B, md->head_dim, G, md->dim, md->ffn, md->n_head) > 160 * 1024) return LR_E_UNSUPPORTED;
  const int nwg = num_cus();
  if (nwg < 2) return LR_E_LAUNCH;
  const int na = pick_na(md->smax, md->head_dim, nwg);
  if (na > NA_MAX || (md->smax + na - 1) / na > att_capacity(md->head_dim)) return LR_E_UNSUPPORTED;
  if (!md->tok_embeddings || !md->norm || !md->output || !md->freqs_cis || !md->layers_dev) return LR_E_NULL;
  return LR_OK;
}

template <int M, int HD, int G>
static int launch_step(const StepParams& sp, int Hq, hipStream_t s) {
  const size_t lds = lds_bytes<M, HD, G>(sp.D, sp.I, Hq);
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

unsigned long long* g_prof = nullptr;  // debug hook: device buffer for phase timestamps
int g_prof_t0 = 0;

}  // namespace

extern "C" void lr_ladder_step_tune(int attention_workgroups) { g_na_override = attention_workgroups; }

extern "C" size_t lr_ladder_step_profile(void* device_buffer, int first_slot) {
  g_prof = reinterpret_cast<unsigned long long*>(device_buffer);
  g_prof_t0 = first_slot;
  return (size_t)num_cus() * PROF_SLOTS * PROF_POINTS * sizeof(unsigned long long);
}

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
  if (bytes < l.total || ldl < md->out_rows || l.total > 0x7fffffffu) return LR_E_SHAPE;
  if (history && (ld_hist < hist_len || hist_len <= 0)) return LR_E_SHAPE;
  StepParams sp;
  sp.D = md->dim; sp.L = md->n_layer; sp.Hkv = md->n_kv_head; sp.I = md->ffn; sp.V = md->out_rows;
  sp.vocab = md->vocab; sp.Smax = md->smax; sp.block_size = md->block_size; sp.B = batch;
  sp.NA = pick_na(md->smax, md->head_dim, nwg);
  sp.nqkv = (md->n_head + 2 * md->n_kv_head) * md->head_dim;
  sp.eps = md->eps;
  sp.tok_emb = (const u16*)md->tok_embeddings; sp.final_norm = (const u16*)md->norm;
  sp.out_w = (const u16*)md->output; sp.rope = (const u16*)md->freqs_cis;
  sp.layers = reinterpret_cast<const LayerPtrs*>(md->layers_dev);
  sp.tokens = tokens; sp.pos = pos; sp.logits = (u16*)logits; sp.ldl = ldl;
  sp.next_token = next_token; sp.cur_token = cur_token; sp.history = history; sp.ld_hist = ld_hist;
  sp.hist_len = hist_len; sp.pos0 = pos0; sp.advance = advance;
  sp.ws = reinterpret_cast<unsigned char*>(workspace);
  sp.ws_bytes = (unsigned)l.total;
  sp.oR = (unsigned)(l.Rbuf / 4); sp.oa = (unsigned)(l.abuf / 4); sp.om = (unsigned)(l.mbuf / 4);
  sp.oqkv = (unsigned)(l.qkv / 4); sp.oact = (unsigned)(l.act / 4);
  sp.oopart = (unsigned)(l.opart / 4); sp.omlpart = (unsigned)(l.mlpart / 4); sp.ocand = (unsigned)(l.cand / 4);
  sp.prof = g_prof;
  sp.prof_t0 = g_prof_t0;
  hipStream_t s = (hipStream_t)stream;
  const int G = md->n_head / md->n_kv_head, hd = md->head_dim;
#define LR_STEP(MV, HDV, GV) \
  if (batch == MV && hd == HDV && G == GV) return launch_step<MV, HDV, GV>(sp, md->n_head, s);
  LR_STEP_INSTANCES(LR_STEP)
#undef LR_STEP
  return LR_E_UNSUPPORTED;
}
