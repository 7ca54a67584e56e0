// One decode step of the Ladder model as ONE persistent kernel (batch 1 or 2).
//
// Why: at batch 1 a step streams 17 GB of weights through ~720 small dependent ops.  Launched
// one by one (even from a hipGraph) the ops pay a launch boundary each and the latency-bound
// ones (norms, RoPE, attention, combine) cost as much as the weight streaming.  Here one
// workgroup per CU (512 lanes = 8 waves) stays resident for the whole step and walks the layers.
//
// The ladder schedule is what makes this wide: attention(t) and mlp(t) both read the residual
// stream BEFORE the other's output has been added (in the reference both outputs are still inside
// an all-reduce at that point), so the two modules of a layer are independent and run side by
// side.  A "slot" t = layer t is, per workgroup,
//     R += a(t-1), attention norm (redundantly in every workgroup; the residual stream itself
//         never leaves the workgroup's LDS); wqkv(t) rows
//     attention workgroups (about one per 128 keys, and per kv head where a rank has several): R += m(t-1), then attention(t) over their key
//         range with K/V held in registers -- scores on the matrix cores (v_mfma_f32_32x32x16_bf16,
//         one tile per 32 keys), fp32 softmax and P.V -- un-normalised partial results; then each of
//         them merges all partial results for its share of the output elements and publishes bf16
//         words (every workgroup merging every partial itself costs 32 times the coherent reads,
//         and those are what makes stragglers)
//     all other workgroups: R += m(t-1), ffn norm, w1(t) rows + SwiGLU  (15 us of streaming that
//         hides the attention latency chain)
//     read the merged attention output, wo(t) rows -> a(t)
//     read the activations, w2(t) rows -> m(t)
// Every hand-over between workgroups has independent streaming between its producer and its
// consumer: a(t-1) is written by wo(t-1) and read after w2(t-1); m(t-1) is written by w2(t-1) and
// read after the attention norm and wqkv(t); qkv(t) and the attention output are covered by w1(t);
// the activations of w1(t) by wo(t).
//
// No barriers, flags or fences: everything that crosses workgroups (module outputs a / m, qkv,
// activations, attention partials, argmax candidates) is exchanged as self-validating 32-bit
// words -- 16 payload bits plus the 16-bit tag of the slot that produced them -- written and read
// with buffer instructions carrying the sc1 policy (loads: sc0 sc1), which bypass the
// non-coherent per-XCD L2 lines.  A consumer optimistically loads what it needs and retries the
// words whose tag is not yet the expected one, so a value is consumed the moment it lands and a
// producer never waits.  Overwriting a word is safe once every workgroup has finished reading its
// previous value; that is implied by data flow alone (the chain is spelled out at the layer loop:
// e.g. a(t) is written in wo(t), which needs the merged attention output, which needs all of
// qkv(t), which every workgroup produces after it has read a(t-1)).
// The values stored are bf16-representable, i.e. rounded exactly where the eager reference
// rounds (fp32 attention partials take two words).  Weights, KV cache and logits use ordinary
// accesses (read-only, or produced for the next launch).
//
// Weight streaming does not stop at these edges: every wave walks its GEMV work as a sequence of
// "units" (8 rows x 1 KiB of one K-slice) held in two register sets; the set just multiplied is
// refilled at once with the unit two positions ahead -- also across the end of a job into the
// next one, through reductions, epilogues, norms and waits -- so a wave has 16 KiB of loads in
// flight.  (One exception: the first units of a slot's first job are requested inside the residual
// bookkeeping, right after the exchanged words have arrived, not at the end of the previous slot:
// loads return in order, and those words are what every workgroup is waiting for at that point.)
// The unit sequence of a job is padded to an even length (pad loads go out of the
// buffer's range and cost nothing) so that the two sets alternate in a fixed pattern, there is
// exactly ONE load sequence in the loop, and rows are addressed through a scalar offset from a
// small per-launch table: that is what lets the compiler place exact wait counts (vmcnt(8))
// instead of draining the pipeline.  Weight loads carry the non-temporal hint: each byte is used
// once per step and must not push the exchanged words out of the caches.  The multiply is
// v_dot2_f32_bf16 on packed bf16 pairs.  Every workgroup owns a run of CONSECUTIVE rows of a matrix,
// so the eight rows a wave requests together lie one row length (16 KiB in the 70B rank shard) apart.
// Dealt round-robin (row = workgroup + 256 j) they lie 4 MiB apart, which puts all of a workgroup's
// requests in flight on the same few DRAM banks: a CU then streams at most about 36 GB/s whatever it
// has queued, and the workgroup that is served slowest ends every phase 3 to 4 us after the others
// (measured: 3.13 ms per token round-robin, 3.00 ms consecutive).  Inside a workgroup the waves split K,
// partial sums meet in LDS in a fixed order -- no float atomics, bit-reproducible.  Workgroup barriers wait for
// LDS only (wg_sync): __syncthreads() would also wait for the prefetched units.
//
// A wave issues at most one instruction every four cycles, so bookkeeping is kept off the layer
// loop: everything about a job except its matrix pointer is tabulated once per launch in LDS
// (per job kind and wave), row offsets included, and the pointer records of the neighbouring
// layers sit in a small LDS ring filled one layer ahead.
//
// Every retry loop is bounded: on time-out a workgroup raises ctrl->fail and goes on with
// whatever it has; everybody leaves at the end of the slot in which they see the flag, so the
// grid always drains.
// LR_STEP_W8 (ladder_step_fp8.hip compiles this file with it set): the same kernel for weight-only e4m3
// projections.  A matrix [N, K] is N * K bytes followed by its N bf16 scales (one per output row); a unit is 8 rows x
// 1 KiB = 1024 elements of K, expanded to packed bf16 pairs (exactly: e4m3 is a subset of bf16) in front of the same
// v_dot2_f32_bf16; a sum is rounded to bf16, multiplied by its row's scale and rounded again -- what lr_linear_fp8
// computes.  Only lr_ladder_decode_step_fp8 is exported by that translation unit.
#include "lr_common.h"

#include <algorithm>

#ifndef LR_STEP_W8
#define LR_STEP_W8 0
#endif

namespace {

constexpr bool W8 = LR_STEP_W8 != 0;
constexpr int KSTEP = W8 ? 1024 : 512;  // elements of K a wave covers per unit (16 bytes per lane and row)
constexpr int KPL = KSTEP / 64;         // ... per lane
constexpr int WBYTES = W8 ? 1 : 2;      // bytes per weight

constexpr int NT = 512;           // lanes per workgroup
constexpr int NW = NT / 64;       // waves per workgroup
constexpr int NJMAX = 64;         // GEMV rows a workgroup reduces per LDS round
constexpr int RB = 8;  // rows per unit (loads a wave issues together)
constexpr unsigned SPIN_LIMIT = 1u << 18;
constexpr int ATT_NI = 9;         // key iterations an attention wave keeps in registers
constexpr int NA_MAX = 16;        // attention workgroups (each merges a share of the outputs)
constexpr int PROF_SLOTS = 4, PROF_POINTS = 32;
// Buffer cache policies (the `aux` operand of the raw buffer builtins: bit 0 sc0, bit 1 nt, bit 4 sc1).
// (exchange stores carry sc1 -- written through, visible to every XCD -- in their assembler text, see Coh)
constexpr int AUX_LD = 17;   // exchange loads: sc0 sc1, never served from a per-XCD L2 line
constexpr int AUX_W = 2;     // weight loads: non-temporal (measured: nt on the exchange words' loads or stores is far slower)
constexpr int POLL_SLEEP = 2;

struct Ctrl {
  unsigned epoch_base, _p0[31];  // slots consumed by earlier steps (tags continue from here)
  unsigned fail, _p1[31];  // 0 = healthy; FAIL_WAIT: a bounded wait expired; FAIL_POS: position outside the cache / RoPE table
  unsigned nwg, _p2[31];
};
constexpr unsigned FAIL_WAIT = 1u, FAIL_POS = 2u;

struct LayerPtrs {
  const u16 *wqkv, *wo, *w1, *w2, *attn_norm, *ffn_norm;
  u16 *k_cache, *v_cache;
};

struct StepParams {
  int D, L, Hkv, I, V, vocab, Smax, block_size, B, NA, nqkv;
  int NAK, NAH;  // NA = NAK key ranges x NAH groups of (sequence, kv head) pairs: attention workgroup w takes range w % NAK of group w / NAK
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
  unsigned oa, om, oqkv, oact, oopart, omlpart, ocand, oy;  // exchange buffers, offsets in 32-bit words
  unsigned long long* prof;  // optional [nwg][PROF_SLOTS][PROF_POINTS] wall-clock stamps (100 MHz)
  int prof_t0;
};


// The lane index as a value the optimiser cannot see through: index arithmetic derived from it
// stays inside the phase that uses it instead of being hoisted out of the layer loop (where it
// would be kept alive, and spilled, for the whole kernel).
__device__ __forceinline__ int opaque_tid() {
  int t = threadIdx.x;
  asm volatile("" : "+v"(t));
  return t;
}

// Workgroup barrier for data exchanged through LDS.  __syncthreads() also waits for every global
// load of the wave (vmcnt(0)), i.e. for the weight units just requested for later -- a full memory
// round trip at every reduction.  Waves of a workgroup only ever talk through LDS here, so waiting
// for the LDS operations is enough.
__device__ __forceinline__ void wg_sync() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

__device__ __forceinline__ unsigned cldu(const unsigned* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void cstu(unsigned* p, unsigned v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ------------------------------------------------------------------------------------------------
// Self-validating exchange words.  Every 32-bit word a workgroup hands to the others carries 16
// payload bits (high half) and the 16-bit tag of the slot that produced it (low half, never 0).
// A bf16-representable value is one word; an fp32 value is two.  Readers load with the sc1 policy
// (bypassing the non-coherent L2) and simply retry until the tag is the one they expect: no flag,
// no fence, no wait on the producer side.  A dword store is indivisible, so a word is either the
// old slot's or the new one's.  Retries are bounded.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ unsigned tag_of(unsigned epoch) { return epoch % 65535u + 1u; }

struct Coh {
  __amdgpu_buffer_rsrc_t r;
  unsigned* fail;
#ifdef LR_STEP_PROFILE
  // profile builds count, per exchange point, the words that had not arrived at the first look
  mutable unsigned long long* cnt = nullptr;
  mutable int where = 24;
  __device__ __forceinline__ void stale() const {
    if (cnt) atomicAdd(cnt + where, 1ull);
  }
  __device__ __forceinline__ void at(unsigned long long* c, int w) const { cnt = c; where = w; }
#else
  __device__ __forceinline__ void stale() const {}
  __device__ __forceinline__ void at(unsigned long long*, int) const {}
#endif

  // Exchange stores are written as inline assembly: the compiler's wait-count insertion does not see them.
  // With a store of its own pending, it must assume that loads and stores complete in any order and waits
  // for EVERYTHING in flight (vmcnt(0)) wherever a loaded value is used -- also for the weight units requested
  // for later.  Unseen stores only ever make a counted wait longer than needed, never shorter: if at most N
  // operations may be outstanding and the N younger loads the compiler counted are joined by a store, one
  // more operation has to finish, and loads finish in order.
  // (The scalar words of the resource may have been restored from a lane of a vector register one instruction
  // earlier; the assembler text is opaque to the hazard recogniser, hence the s_nop in front of every store.)
  u32x4_t rs;  // the same buffer resource as `r`, as four scalar words
  __device__ __forceinline__ void st_raw(unsigned word, unsigned byte_off) const {
    asm volatile("s_nop 4\n\tbuffer_store_dword %0, %1, %2, 0 offen sc1" ::"v"(word), "v"(byte_off), "s"(rs) : "memory");
  }
  __device__ __forceinline__ void st_raw2(u32x2_t w, unsigned byte_off) const {
    asm volatile("s_nop 4\n\tbuffer_store_dwordx2 %0, %1, %2, 0 offen sc1\n\ts_nop 1" ::"v"(w), "v"(byte_off), "s"(rs) : "memory");
  }
  __device__ __forceinline__ void st_raw4(u32x4_t w, unsigned byte_off) const {
    asm volatile("s_nop 4\n\tbuffer_store_dwordx4 %0, %1, %2, 0 offen sc1\n\ts_nop 1" ::"v"(w), "v"(byte_off), "s"(rs) : "memory");
  }
  __device__ __forceinline__ void st(unsigned wo, float v, unsigned tag) const {  // v is bf16-representable
    st_raw((__float_as_uint(v) & 0xffff0000u) | tag, wo * 4);
  }
  __device__ __forceinline__ void st8(unsigned wo, const float* f, unsigned tag) const {  // wo % 4 == 0
    u32x4_t a, b;
    a.x = (__float_as_uint(f[0]) & 0xffff0000u) | tag; a.y = (__float_as_uint(f[1]) & 0xffff0000u) | tag;
    a.z = (__float_as_uint(f[2]) & 0xffff0000u) | tag; a.w = (__float_as_uint(f[3]) & 0xffff0000u) | tag;
    b.x = (__float_as_uint(f[4]) & 0xffff0000u) | tag; b.y = (__float_as_uint(f[5]) & 0xffff0000u) | tag;
    b.z = (__float_as_uint(f[6]) & 0xffff0000u) | tag; b.w = (__float_as_uint(f[7]) & 0xffff0000u) | tag;
    st_raw4(a, wo * 4);
    st_raw4(b, wo * 4 + 16);
  }
  // two bf16-representable values as two words at wo, wo + 1 (wo % 2 == 0)
  __device__ __forceinline__ void st2(unsigned wo, float v0, float v1, unsigned tag) const {
    u32x2_t w;
    w.x = (__float_as_uint(v0) & 0xffff0000u) | tag;
    w.y = (__float_as_uint(v1) & 0xffff0000u) | tag;
    st_raw2(w, wo * 4);
  }
  // fp32 value as two words at wo, wo + 1 (wo % 2 == 0)
  __device__ __forceinline__ void st_f32(unsigned wo, float v, unsigned tag) const {
    const unsigned bits = __float_as_uint(v);
    u32x2_t w;
    w.x = (bits & 0xffff0000u) | tag;
    w.y = (bits << 16) | tag;
    st_raw2(w, wo * 4);
  }
  __device__ __forceinline__ bool give_up(unsigned& spins) const {
    if ((++spins & 255u) == 0) {
      const unsigned f = cldu(fail);
      if (spins > SPIN_LIMIT || f) {
        if (f == 0) cstu(fail, FAIL_WAIT);
        return true;
      }
    }
    return false;
  }
  // 4 tagged words -> raw words (tags still inside); spins until all four carry `tag`
  __device__ __forceinline__ u32x4_t poll4(unsigned wo, unsigned tag) const {
    unsigned spins = 0;
    for (;;) {
      const u32x4_t a = __builtin_amdgcn_raw_buffer_load_b128(r, wo * 4, 0, AUX_LD);
      if ((((a.x ^ tag) | (a.y ^ tag) | (a.z ^ tag) | (a.w ^ tag)) & 0xffffu) == 0) return a;
      if (give_up(spins)) return a;
      __builtin_amdgcn_s_sleep(POLL_SLEEP);
    }
  }
  __device__ __forceinline__ u32x2_t poll2(unsigned wo, unsigned tag) const {
    unsigned spins = 0;
    for (;;) {
      const u32x2_t a = __builtin_amdgcn_raw_buffer_load_b64(r, wo * 4, 0, AUX_LD);
      if ((((a.x ^ tag) | (a.y ^ tag)) & 0xffffu) == 0) return a;
      if (give_up(spins)) return a;
      __builtin_amdgcn_s_sleep(POLL_SLEEP);
    }
  }
  __device__ __forceinline__ unsigned poll1(unsigned wo, unsigned tag) const {
    unsigned spins = 0;
    for (;;) {
      const unsigned a = __builtin_amdgcn_raw_buffer_load_b32(r, wo * 4, 0, AUX_LD);
      if (((a ^ tag) & 0xffffu) == 0) return a;
      if (give_up(spins)) return a;
      __builtin_amdgcn_s_sleep(POLL_SLEEP);
    }
  }
  // Optimistic form: raw4/raw2 issue the load (many can be in flight), settle4/settle2 accept the
  // words if their tags match and fall back to polling otherwise.
  __device__ __forceinline__ u32x4_t raw4(unsigned wo) const {
    return __builtin_amdgcn_raw_buffer_load_b128(r, wo * 4, 0, AUX_LD);
  }
  __device__ __forceinline__ unsigned raw1(unsigned wo) const {
    return __builtin_amdgcn_raw_buffer_load_b32(r, wo * 4, 0, AUX_LD);
  }
  __device__ __forceinline__ u32x2_t raw2(unsigned wo) const {
    return __builtin_amdgcn_raw_buffer_load_b64(r, wo * 4, 0, AUX_LD);
  }
  __device__ __forceinline__ bool stale4(const u32x4_t& a, unsigned tag) const {
    return (((a.x ^ tag) | (a.y ^ tag) | (a.z ^ tag) | (a.w ^ tag)) & 0xffffu) != 0;
  }
  __device__ __forceinline__ u32x4_t settle4(unsigned wo, unsigned tag, const u32x4_t& a) const {
    if ((((a.x ^ tag) | (a.y ^ tag) | (a.z ^ tag) | (a.w ^ tag)) & 0xffffu) == 0) return a;
    stale();
    return poll4(wo, tag);
  }
  __device__ __forceinline__ u32x2_t settle2(unsigned wo, unsigned tag, const u32x2_t& a) const {
    if ((((a.x ^ tag) | (a.y ^ tag)) & 0xffffu) == 0) return a;
    stale();
    return poll2(wo, tag);
  }
  // 8 bf16-valued words -> 8 floats
  __device__ __forceinline__ void ld8(unsigned wo, unsigned tag, float* f) const {
    unsigned spins = 0;
    for (;;) {
      const u32x4_t a = __builtin_amdgcn_raw_buffer_load_b128(r, wo * 4, 0, AUX_LD);
      const u32x4_t b = __builtin_amdgcn_raw_buffer_load_b128(r, wo * 4 + 16, 0, AUX_LD);
      const unsigned bad = ((a.x ^ tag) | (a.y ^ tag) | (a.z ^ tag) | (a.w ^ tag) | (b.x ^ tag) | (b.y ^ tag) |
                            (b.z ^ tag) | (b.w ^ tag)) & 0xffffu;
      if (bad == 0 || give_up(spins)) {
        f[0] = __uint_as_float(a.x & 0xffff0000u); f[1] = __uint_as_float(a.y & 0xffff0000u);
        f[2] = __uint_as_float(a.z & 0xffff0000u); f[3] = __uint_as_float(a.w & 0xffff0000u);
        f[4] = __uint_as_float(b.x & 0xffff0000u); f[5] = __uint_as_float(b.y & 0xffff0000u);
        f[6] = __uint_as_float(b.z & 0xffff0000u); f[7] = __uint_as_float(b.w & 0xffff0000u);
        return;
      }
      if (spins == 0) stale();
      __builtin_amdgcn_s_sleep(POLL_SLEEP);
    }
  }
  __device__ __forceinline__ void ld2(unsigned wo, unsigned tag, float& x0, float& x1) const {
    const u32x2_t a = poll2(wo, tag);
    x0 = __uint_as_float(a.x & 0xffff0000u);
    x1 = __uint_as_float(a.y & 0xffff0000u);
  }
};
__device__ __forceinline__ void bf4_from(const u32x4_t& a, float* f) {
  f[0] = __uint_as_float(a.x & 0xffff0000u); f[1] = __uint_as_float(a.y & 0xffff0000u);
  f[2] = __uint_as_float(a.z & 0xffff0000u); f[3] = __uint_as_float(a.w & 0xffff0000u);
}
// two fp32 values from 4 words (hi, lo, hi, lo)
__device__ __forceinline__ void f32x2_from(const u32x4_t& a, float& v0, float& v1) {
  v0 = __uint_as_float((a.x & 0xffff0000u) | (a.y >> 16));
  v1 = __uint_as_float((a.z & 0xffff0000u) | (a.w >> 16));
}

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
// c + a.lo * b.lo + a.hi * b.hi on packed bf16 pairs, fp32 accumulation
__device__ __forceinline__ float dot2(u32 a, u32 b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), c, false);
}
// the low (HI == false) or high two e4m3 values of a dword as a packed bf16 pair (exact)
template <bool HI>
__device__ __forceinline__ u32 fp8_pair(u32 v) {
  return __builtin_bit_cast(u32, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(v, 1.0f, HI));
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
__device__ __forceinline__ float wave_sum_xbar(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, LR_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max_xbar(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, LR_WAVE));
  return v;
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
// GEMV work of one workgroup in one matrix ("job").  Items (rows, or up/gate row pairs) are dealt in
// runs over the participating workgroups: participant w owns items first .. first + n - 1.
// Its rows are reduced in rounds of NJMAX; inside a round wave (rg, kg) owns rows j = rg (mod nrg)
// and K-slices kk = kg (mod nkg), RB rows x one 512-element slice per unit.
// ------------------------------------------------------------------------------------------------
#define LR_UNI(x) __builtin_amdgcn_readfirstlane(x)

// The pointer records of the layers around the current one are kept in a small LDS ring (filled
// one layer ahead of use), so that a job never waits for a scalar load from global memory.
enum { LP_WQKV = 0, LP_WO, LP_W1, LP_W2, LP_ATTN_NORM, LP_FFN_NORM, LP_K_CACHE, LP_V_CACHE };
__device__ __forceinline__ const u16* ring_ptr(const u32* lring, int layer, int field) {
  const u32* e = lring + (layer & 3) * 16 + field * 2;
  const u32 lo = LR_UNI(e[0]), hi = LR_UNI(e[1]);
  return reinterpret_cast<const u16*>(((unsigned long long)hi << 32) | lo);
}

// Everything about a job that does not change from layer to layer (all but the matrix pointer) is
// worked out once per launch, per job kind and wave, and kept in LDS: the per-layer code then has
// no divisions and little scalar state (a wave issues at most one instruction every four cycles,
// so bookkeeping instructions are what small jobs are made of).
enum { JK_QKV = 0, JK_W1_SPLIT, JK_WO, JK_W2, JK_HEAD, JK_W1_ALL, JK_NONE, JK_COUNT };

struct Job {  // wave-uniform
  int K2;                  // bytes per row
  int pair_off, rsh;       // item -> rows: row = first + (jj >> rsh) + (jj & rsh) * pair_off   (rsh 0 or 1)
  int rank, first;         // this workgroup's rank among the participants; its first item
  int nj;                  // rows this workgroup owns
  int ksteps, nkg, nrg;    // 512-element K slices; waves along K; waves along rows
  int rg, kg;              // this wave's place
  int nk;                  // k-steps per row batch for this wave
  int bsh;                 // log2(nrg * RB): row stride between a wave's batches
  int active;              // this wave has work in the job
  int K;
  int kind;                // JK_*: selects the row-offset table
  const u16* W;            // not in LDS: set per layer
  const int* rowtab;       // not in LDS: row offsets of the first round (see build_row_table)
#if LR_STEP_W8
  const u16* S;            // the rows' scales: behind the matrix (table word 15 holds the distance in bytes)
#endif
};
static_assert(sizeof(Job) == 16 * 4 + 16 + (W8 ? 8 : 0), "16 table words + two pointers");

__device__ __forceinline__ void build_job(int* rec, int kind, int K, int n_items, int pair_off, int rsh, int w, int nwg,
                                          int wave) {
  Job j;
  j.K = K; j.K2 = K * WBYTES; j.pair_off = pair_off; j.rsh = rsh; j.rank = w;
  // participant w owns a run of consecutive items (the first n_items % nwg participants one more than the others)
  const int base = n_items / nwg, rem = n_items % nwg;
  const int nit = (w >= 0 && w < nwg) ? base + (w < rem ? 1 : 0) : 0;
  j.first = w >= 0 ? w * base + (w < rem ? w : rem) : 0;
  j.nj = nit << rsh;
  j.ksteps = (K + KSTEP - 1) / KSTEP;
  j.nkg = j.ksteps < NW ? j.ksteps : NW;
  j.nrg = NW / j.nkg;
  j.rg = wave / j.nkg;
  j.kg = wave - j.rg * j.nkg;
  j.active = (wave < j.nrg * j.nkg && j.rg < (j.nj < NJMAX ? j.nj : NJMAX)) ? 1 : 0;
  j.nk = j.kg < j.ksteps ? (j.ksteps - j.kg + j.nkg - 1) / j.nkg : 0;
  j.bsh = 31 - __builtin_clz(j.nrg * RB);
  j.kind = kind;
  const int* src = reinterpret_cast<const int*>(&j);
  for (int i = 0; i < 16; ++i) rec[i] = src[i];
  if (W8) rec[15] = (n_items << rsh) * K;  // all rows of the matrix, one byte per weight: where its scales start
}

// table: [JK_COUNT][NW][16] ints in LDS, filled once per launch
__device__ __forceinline__ void build_job_table(const StepParams& p, int* table, int qdim, int w, int nwg) {
  const int i = threadIdx.x;
  if (i < JK_COUNT * NW) {
    const int kind = i / NW, wave = i - kind * NW;
    int* rec = table + i * 16;
    if (kind == JK_QKV) build_job(rec, kind, p.D, p.nqkv, 0, 0, w, nwg, wave);
    else if (kind == JK_W1_SPLIT) build_job(rec, kind, p.D, p.I, p.I, 1, w - p.NA, nwg - p.NA, wave);
    else if (kind == JK_WO) build_job(rec, kind, qdim, p.D, 0, 0, w, nwg, wave);
    else if (kind == JK_W2) build_job(rec, kind, p.I, p.D, 0, 0, w, nwg, wave);
    else if (kind == JK_HEAD) build_job(rec, kind, p.D, p.V, 0, 0, w, nwg, wave);
    else if (kind == JK_W1_ALL) build_job(rec, kind, p.D, p.I, p.I, 1, w, nwg, wave);
    else build_job(rec, kind, 512, 0, 0, 0, 0, 1, wave);
  }
}

// Byte offsets of the rows of a job's FIRST round, per kind, ordered so that the RB rows of one
// unit are consecutive: entry ((rg * (64 >> bsh)) + batch) * RB + i is row j = rg + (batch << bsh) +
// i * nrg of the round, clamped to the last row the workgroup owns.  Later rounds (long lm_heads
// only) compute their offsets.  Filled once per launch, after the job table.
__device__ __forceinline__ void build_row_table(const int* table, int* rowtab) {
  const int i = threadIdx.x;
  if (i < JK_COUNT * NJMAX) {
    const int kind = i / NJMAX, e = i - kind * NJMAX;
    const Job* j = reinterpret_cast<const Job*>(table + kind * NW * 16);  // wave 0's record: these fields are common
    const int lg = j->bsh - 3;                                            // log2(nrg)
    const int nbmax = NJMAX >> j->bsh;
    const int rg = e / (nbmax * RB), b = (e / RB) % nbmax, ii = e % RB;
    const int njb = j->nj < NJMAX ? j->nj : NJMAX;
    int row_j = rg + (b << j->bsh) + (ii << lg);
    row_j = row_j < njb ? row_j : njb - 1;
    row_j = row_j < 0 ? 0 : row_j;
    const int row = j->first + (row_j >> j->rsh) + (row_j & ((1 << j->rsh) - 1)) * j->pair_off;
    rowtab[i] = (int)((unsigned)row * (unsigned)j->K2);
  }
}

__device__ __forceinline__ Job load_job(const int* table, int kind, int wave, const u16* W) {
  const int4* r = reinterpret_cast<const int4*>(table + (kind * NW + wave) * 16);
  const int4 a = r[0], b = r[1], c = r[2], d = r[3];
  Job j;
  j.K2 = LR_UNI(a.x); j.pair_off = LR_UNI(a.y); j.rsh = LR_UNI(a.z); j.rank = LR_UNI(a.w);
  j.first = LR_UNI(b.x); j.nj = LR_UNI(b.y); j.ksteps = LR_UNI(b.z); j.nkg = LR_UNI(b.w);
  j.nrg = LR_UNI(c.x); j.rg = LR_UNI(c.y); j.kg = LR_UNI(c.z); j.nk = LR_UNI(c.w);
  j.bsh = LR_UNI(d.x); j.active = LR_UNI(d.y); j.K = LR_UNI(d.z); j.kind = kind;
  j.W = W;
  j.rowtab = table + JK_COUNT * NW * 16 + kind * NJMAX;
#if LR_STEP_W8
  j.S = reinterpret_cast<const u16*>(reinterpret_cast<const unsigned char*>(W) + LR_UNI(d.w));
#endif
  return j;
}

struct Unit {
  u32x4_t r[RB];
};

// Issue the loads of unit (j0, jb, kk) of `job`: one buffer load per row, the row's offset in a
// scalar register, the lane's column offset shared by all rows.  Rows beyond the round and columns
// beyond K are clamped to valid addresses: their products are discarded / multiplied by a zero x.
// With real == false the same number of loads is issued out of the buffer's range (they return
// zero without touching memory): the number of loads in flight then never depends on a branch.
// That, and there being ONE load sequence in the loop (prod_issue selects the job by value), is
// what lets the compiler's wait-count insertion wait for exactly the older unit (vmcnt(RB))
// instead of for everything in flight.
__device__ __forceinline__ void load_unit(const Job& job, int j0, int jb, int kk, int lane, Unit& u, bool real) {
  int k = kk * KSTEP + lane * KPL;
  k = k < job.K ? k : 0;
  const int voff = real ? k * WBYTES : (int)0x80000000;
  __amdgpu_buffer_rsrc_t br = __builtin_amdgcn_make_buffer_rsrc(const_cast<u16*>(job.W), 0, job.W ? 0x7fffffff : 0, 0x00020000);
  int so[RB];
  if (j0 == 0) {  // first round: the offsets are tabulated (two LDS reads instead of ~10 scalar operations per row)
    const int e = ((job.rg * (NJMAX >> job.bsh)) + ((jb - job.rg) >> job.bsh)) * RB;
    const int4 t0 = *reinterpret_cast<const int4*>(job.rowtab + e);
    const int4 t1 = *reinterpret_cast<const int4*>(job.rowtab + e + 4);
    so[0] = t0.x; so[1] = t0.y; so[2] = t0.z; so[3] = t0.w;
    so[4] = t1.x; so[5] = t1.y; so[6] = t1.z; so[7] = t1.w;
  } else {
    const int njb = job.nj - j0 < NJMAX ? job.nj - j0 : NJMAX;
    const int rmask = (1 << job.rsh) - 1;
#pragma unroll
    for (int i = 0; i < RB; ++i) {
      int j = jb + i * job.nrg;
      j = j < njb ? j : njb - 1;
      const int jj = j0 + j;
      const int row = job.first + (jj >> job.rsh) + (jj & rmask) * job.pair_off;
      so[i] = (int)((unsigned)row * (unsigned)job.K2);
    }
  }
#pragma unroll
  for (int i = 0; i < RB; ++i)
    u.r[i] = __builtin_amdgcn_raw_buffer_load_b128(br, voff, LR_UNI(real ? so[i] : 0), AUX_W);
}
// ---- a wave's position in the unit sequence of a job.  The sequence is: for every round, the
//      wave's units (k-steps fastest, then row batches), padded to an even count, so that the two
//      register sets of the pipeline alternate in a fixed way.  All of it is wave-uniform.
struct Pos {
  int j0, u, ur, up, jb, kk;  // round, index in the round, real / padded units of the round, coordinates
  bool done;
};
__device__ __forceinline__ void pos_round(const Job& j, Pos& p) {
  // (written without branches: every field is assigned exactly once on every path, which keeps
  // the structure in registers)
  const int njb = j.nj - p.j0 < NJMAX ? j.nj - p.j0 : NJMAX;
  const bool ok = j.active && p.j0 < j.nj && j.rg < njb;
  const int nb = (njb - j.rg + (1 << j.bsh) - 1) >> j.bsh;
  const int ur = ok ? nb * j.nk : 0;
  p.done = !ok;
  p.ur = ur;
  p.up = (ur + 1) & ~1;
  p.u = 0;
  p.jb = j.rg;
  p.kk = j.kg;
}
__device__ __forceinline__ void pos_first(const Job& j, Pos& p) {
  p.j0 = 0;
  p.u = 0;
  p.done = false;
  pos_round(j, p);
}
__device__ __forceinline__ bool pos_real(const Pos& p) { return !p.done && p.u < p.ur; }
__device__ __forceinline__ void pos_next(const Job& j, Pos& p) {
  if (p.done) return;
  const int u = p.u + 1;
  if (u < p.up) {
    int kk = p.kk, jb = p.jb;
    if (u < p.ur) {
      kk += j.nkg;
      if (kk >= j.ksteps) {
        kk = j.kg;
        jb += 1 << j.bsh;
      }
    }
    p.u = u;
    p.kk = kk;
    p.jb = jb;
  } else {
    p.j0 += NJMAX;
    pos_round(j, p);
  }
}

// The weight pipeline of a wave: two register sets.  While one is multiplied the other is in
// flight, and the set just multiplied is refilled at once with the unit two positions ahead --
// also across the end of a job, into the next one.  On entry to run_job, `a` and `b` hold the
// wave's first two positions of that job (issued by the previous job, or by prime()).
struct Pipe {
  Unit a, b;
};
struct Prod {  // where the prefetch is: two positions ahead of the multiplier
  Pos p;
  Job job;  // the job it is walking (this one, later the next)
  bool in_next;
};
__device__ __forceinline__ void prod_issue(const Job& next, Prod& pr, int lane, Unit& u) {
  load_unit(pr.job, pr.p.j0, pr.p.jb, pr.p.kk, lane, u, pos_real(pr.p));  // the ONE load sequence of the loop
  pos_next(pr.job, pr.p);
  if (pr.p.done && !pr.in_next) {
    pr.in_next = true;
    pr.job = next;
    pos_first(next, pr.p);
  }
}
__device__ __forceinline__ void prime(const Job& job, int lane, Pipe& pipe) {
  Pos p;
  pos_first(job, p);
  load_unit(job, p.j0, p.jb, p.kk, lane, pipe.a, pos_real(p));
  pos_next(job, p);
  load_unit(job, p.j0, p.jb, p.kk, lane, pipe.b, pos_real(p));
}

enum { EPI_STORE = 0, EPI_SWIGLU = 1, EPI_LOGITS = 2 };

// multiply one unit into the accumulators of its row batch; at the batch's last k-step fold the
// lanes and leave the partial sums in LDS
template <int M>
__device__ __forceinline__ void consume_unit(const Job& job, const Pos& c, const Unit& u, const u16* x, float* part,
                                             float (&acc)[M][RB], int lane) {
  const int njb = job.nj - c.j0 < NJMAX ? job.nj - c.j0 : NJMAX;
  if (c.kk == job.kg) {
#pragma unroll
    for (int m = 0; m < M; ++m)
#pragma unroll
      for (int i = 0; i < RB; ++i) acc[m][i] = 0.0f;
  }
  const int k = c.kk * KSTEP + lane * KPL;
  const bool kv = k < job.K;
  // weights and inputs stay packed bf16 pairs: one v_dot2_f32_bf16 per pair of products (fp32 sums)
#if LR_STEP_W8
  uint4 xp[M][2];
#pragma unroll
  for (int m = 0; m < M; ++m) {
    xp[m][0] = kv ? *reinterpret_cast<const uint4*>(x + m * job.K + k) : make_uint4(0, 0, 0, 0);
    xp[m][1] = kv ? *reinterpret_cast<const uint4*>(x + m * job.K + k + 8) : make_uint4(0, 0, 0, 0);
  }
#pragma unroll
  for (int i = 0; i < RB; ++i) {
    // dword d of the lane's 16 bytes holds elements 4 d .. 4 d + 3
    u32 wp[8];
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      wp[2 * d] = fp8_pair<false>(u.r[i][d]);
      wp[2 * d + 1] = fp8_pair<true>(u.r[i][d]);
    }
#pragma unroll
    for (int m = 0; m < M; ++m) {
      float a = acc[m][i];
      a = dot2(wp[0], xp[m][0].x, a);
      a = dot2(wp[1], xp[m][0].y, a);
      a = dot2(wp[2], xp[m][0].z, a);
      a = dot2(wp[3], xp[m][0].w, a);
      a = dot2(wp[4], xp[m][1].x, a);
      a = dot2(wp[5], xp[m][1].y, a);
      a = dot2(wp[6], xp[m][1].z, a);
      a = dot2(wp[7], xp[m][1].w, a);
      acc[m][i] = a;
    }
  }
#else
  uint4 xp[M];
#pragma unroll
  for (int m = 0; m < M; ++m)
    xp[m] = kv ? *reinterpret_cast<const uint4*>(x + m * job.K + k) : make_uint4(0, 0, 0, 0);
#pragma unroll
  for (int i = 0; i < RB; ++i) {
#pragma unroll
    for (int m = 0; m < M; ++m) {
      float a = acc[m][i];
      a = dot2(u.r[i].x, xp[m].x, a);
      a = dot2(u.r[i].y, xp[m].y, a);
      a = dot2(u.r[i].z, xp[m].z, a);
      a = dot2(u.r[i].w, xp[m].w, a);
      acc[m][i] = a;
    }
  }
#endif
  if (c.kk + job.nkg >= job.ksteps) {
#pragma unroll
    for (int m = 0; m < M; ++m)
#pragma unroll
      for (int h = 0; h < RB / 8; ++h) {
        float z0, z1;
        reduce8(&acc[m][8 * h], z0, z1);
        if ((lane & 15) == 0) {
          const int r = lane >> 4;
          const int ja = c.jb + (8 * h + 2 * r) * job.nrg, jc = c.jb + (8 * h + 2 * r + 1) * job.nrg;
          if (ja < njb) part[(job.kg * NJMAX + ja) * M + m] = z0;
          if (jc < njb) part[(job.kg * NJMAX + jc) * M + m] = z1;
        }
      }
  }
}

// Run one job; see Pipe for what `pipe` holds on entry and on exit (`next` must be the job the
// following run_job call is made with).
template <int M, int EPI>
__device__ __forceinline__ void run_job(const StepParams& p, const Coh& coh, const Job& job, const Job& next,
                                        Pipe& pipe, const u16* x, float* part, unsigned out_wo, int ldo, unsigned tag,
                                        float* cand_v, int* cand_i, float* best_v, int* best_i,
                                        unsigned long long* stamp = nullptr, int sb = 0) {
  const int tid = opaque_tid(), lane = tid & 63;
  const int RPI = 1 << job.rsh;
  if (!job.active) prime(next, lane, pipe);
  Pos c;
  Prod pr;
  pos_first(job, c);
  pr.p = c;
  pr.job = job;
  pr.in_next = false;
  pos_next(job, pr.p);
  pos_next(job, pr.p);
  if (pr.p.done) {
    pr.in_next = true;
    pr.job = next;
    pos_first(next, pr.p);
  }
  float acc[M][RB];
  for (int j0 = 0; j0 < job.nj; j0 += NJMAX) {
    const int njb = job.nj - j0 < NJMAX ? job.nj - j0 : NJMAX;
#if LR_STEP_W8
    // The scales of the outputs this lane will finish are requested now: their round trip is over when the
    // round's units have been multiplied.  They stay raw bits until then: converted here, the conversion (and with
    // it a wait for the load, the youngest in flight, i.e. for everything) would sit at the top of every job.
    u32 sraw0 = 0x3f80, sraw1 = 0x3f80;  // 1.0
    if (tid < (njb >> job.rsh) * M) {
      const int it_s = job.first + (j0 >> job.rsh) + tid / M;
      sraw0 = gld2(job.S + it_s);
      if (EPI == EPI_SWIGLU) sraw1 = gld2(job.S + it_s + job.pair_off);
    }
#endif
    if (stamp && tid == 0 && (sb == 16 || sb == 20)) stamp[sb == 16 ? 30 : 31] = wall_clock64();
    if (job.active && job.rg < njb) {
      const int up = c.up;
      for (int u = 0; u < up; u += 2) {
        if (pos_real(c)) consume_unit<M>(job, c, pipe.a, x, part, acc, lane);
        prod_issue(next, pr, lane, pipe.a);
        pos_next(job, c);
        if (pos_real(c)) consume_unit<M>(job, c, pipe.b, x, part, acc, lane);
        prod_issue(next, pr, lane, pipe.b);
        pos_next(job, c);
      }
    }
    wg_sync();
    if (stamp && tid == 0) stamp[sb] = wall_clock64();
    // ---- cross-wave sum in fixed order + epilogue
    const int nout = (njb >> job.rsh) * M;
    if (tid < nout) {
      const int jl = tid / M, m = tid - jl * M;
      float s0, s1 = 0.0f;
      {  // all partial sums are requested at once; they are added in the same fixed order
        float v0[NW], v1[NW];
#pragma unroll
        for (int g = 0; g < NW; ++g) {
          v0[g] = part[(g * NJMAX + jl * RPI) * M + m];
          if (EPI == EPI_SWIGLU) v1[g] = part[(g * NJMAX + jl * RPI + 1) * M + m];
        }
        float t = 0.0f, t1 = 0.0f;
#pragma unroll
        for (int g = 0; g < NW; ++g) {
          t = g < job.nkg ? t + v0[g] : t;
          if (EPI == EPI_SWIGLU) t1 = g < job.nkg ? t1 + v1[g] : t1;
        }
        s0 = round_bf(t);
        if (EPI == EPI_SWIGLU) s1 = round_bf(t1);
      }
#if LR_STEP_W8
      asm volatile("" : "+v"(sraw0), "+v"(sraw1));  // (the conversion stays down here)
      s0 = round_bf(s0 * __uint_as_float(sraw0 << 16));
      s1 = round_bf(s1 * __uint_as_float(sraw1 << 16));
#endif
      const int it = job.first + (j0 >> job.rsh) + jl;
      if (m < p.B) {
        if (EPI == EPI_STORE) coh.st(out_wo + (unsigned)(m * ldo + it), s0, tag);
        if (EPI == EPI_SWIGLU) coh.st(out_wo + (unsigned)(m * ldo + it), swiglu_bf(s0, s1), tag);
        if (EPI == EPI_LOGITS) p.logits[(int64_t)m * p.ldl + it] = f_to_bf(s0);
      }
      if (EPI == EPI_LOGITS) {
        cand_v[tid] = s0;
        cand_i[tid] = it;
      }
    }
    if (EPI == EPI_LOGITS) {
      wg_sync();
      if (tid < M) {  // items ascend with jl: strict '>' keeps the lowest index among equals
        for (int jl = 0; jl < njb; ++jl) {
          const float v = cand_v[jl * M + tid];
          if (v > *best_v) { *best_v = v; *best_i = cand_i[jl * M + tid]; }
        }
      }
    }
    wg_sync();
    if (stamp && tid == 0) stamp[sb + 1] = wall_clock64();
  }
}

// ------------------------------------------------------------------------------------------------
// Residual bookkeeping + RMSNorm for the coming job, done redundantly by every workgroup (each keeps
// its own copy of the residual stream in LDS, so only module outputs are ever exchanged):
//   R <- bf16(R + d1) (if has_d1);  R <- bf16(R + d2) (if has_d2);  x = norm(R) * gain -> LDS (if gain).
// At the first slot R comes from rows of the bf16 embedding table.  d1 / d2 are tagged exchange
// arrays; all their loads are issued before the first one is checked.
// ------------------------------------------------------------------------------------------------
constexpr int PRO_NIT = 4;  // 8-element chunks per lane and row: dim <= PRO_NIT * NT * 8
constexpr int EARLY_NIT = 2;  // chunks whose exchange words can be requested ahead of time (dim <= 8192 entirely)

// The exchange words a coming residual_step will add (its d1), requested early -- before the job
// that runs in between, or while that job's epilogue runs -- so that their round trip is over when
// the step starts.  Words that were not there yet are polled by the step as usual.
// (Batch 1 only: at batch 2 the 32 registers the words would occupy across a job are not there.)
template <int M>
struct EarlyWords {
  static constexpr bool USED = M == 1;
  u32x4_t r[1][EARLY_NIT][2];
};
// (every field is assigned on every path, `real` or not, so that the structure stays in registers; a
// request that is not wanted goes out of the buffer's range and returns zero without touching memory)
template <int M>
__device__ __forceinline__ void issue_words(const Coh& coh, bool real, unsigned wo, int D, EarlyWords<M>& e) {
  if (!EarlyWords<M>::USED) return;
  const int tid = opaque_tid();
#pragma unroll
  for (int it = 0; it < EARLY_NIT; ++it) {
    const int c = (it * NT + tid) * 8;
    const unsigned o = (real && c < D) ? wo + (unsigned)c : 0x20000000u;
    e.r[0][it][0] = coh.raw4(o);
    e.r[0][it][1] = coh.raw4(o + 4u);
  }
}

template <int M>
__device__ __forceinline__ void residual_step(const StepParams& p, const Coh& coh, u16* xr, const int* emb_rows,
                                              bool has_d1, unsigned d1_wo, unsigned d1_tag, bool early1,
                                              const EarlyWords<M>& e1, bool has_d2, unsigned d2_wo, unsigned d2_tag,
                                              const u16* gain, u16* x, float* red, bool do_prime, const Job& first,
                                              Pipe& pipe, unsigned long long* stamp = nullptr) {
  const int tid = opaque_tid(), D = p.D;
  float ss[M];
  // the gain is needed only in pass 2 but is requested now: its latency hides behind pass 1
  uint4 gq[PRO_NIT];
#pragma unroll
  for (int it = 0; it < PRO_NIT; ++it) {
    const int c = (it * NT + tid) * 8;
    gq[it] = (gain && c < D) ? gld16(gain + c) : make_uint4(0, 0, 0, 0);
  }
  // pass 1: the (bf16-exact) sums go to LDS unscaled; sums of squares per lane
#pragma unroll
  for (int m = 0; m < M; ++m) {
    ss[m] = 0.0f;
    u32x4_t r1[PRO_NIT][2], r2[PRO_NIT][2];
#pragma unroll
    for (int it = 0; it < PRO_NIT; ++it) {
      const int c = (it * NT + tid) * 8;
      if (c < D && has_d1) {
        if (EarlyWords<M>::USED && early1 && it < EARLY_NIT) {
          r1[it][0] = e1.r[0][it < EARLY_NIT ? it : 0][0];
          r1[it][1] = e1.r[0][it < EARLY_NIT ? it : 0][1];
        } else {
          r1[it][0] = coh.raw4(d1_wo + m * D + c);
          r1[it][1] = coh.raw4(d1_wo + m * D + c + 4);
        }
      }
      if (c < D && has_d2) {
        r2[it][0] = coh.raw4(d2_wo + m * D + c);
        r2[it][1] = coh.raw4(d2_wo + m * D + c + 4);
      }
    }
#pragma unroll
    for (int it = 0; it < PRO_NIT; ++it) {
      const int c = (it * NT + tid) * 8;
      if (c < D) {
        float v[8], t[8];
        if (emb_rows) {
          const int id = emb_rows[m];
          const bool ok = id >= 0 && id < p.vocab;
          unpack8(ok ? gld16(p.tok_emb + (int64_t)id * D + c) : make_uint4(0, 0, 0, 0), v);
        } else {
          unpack8(*reinterpret_cast<const uint4*>(xr + m * D + c), v);
        }
        if (has_d1) {
          bf4_from(coh.settle4(d1_wo + m * D + c, d1_tag, r1[it][0]), t);
          bf4_from(coh.settle4(d1_wo + m * D + c + 4, d1_tag, r1[it][1]), t + 4);
#pragma unroll
          for (int j = 0; j < 8; ++j) v[j] = round_bf(v[j] + t[j]);
        }
        if (has_d2) {
          bf4_from(coh.settle4(d2_wo + m * D + c, d2_tag, r2[it][0]), t);
          bf4_from(coh.settle4(d2_wo + m * D + c + 4, d2_tag, r2[it][1]), t + 4);
#pragma unroll
          for (int j = 0; j < 8; ++j) v[j] = round_bf(v[j] + t[j]);
        }
        if (gain) st16(x + m * D + c, pack8(v));
#pragma unroll
        for (int j = 0; j < 8; ++j) ss[m] += v[j] * v[j];
        if (has_d1 || has_d2 || emb_rows) st16(xr + m * D + c, pack8(v));
      }
    }
  }
  // The first weight units of the coming job are requested only now, when the exchange words have arrived.
  // Requested earlier -- right behind the word requests, with the bookkeeping done while the words travel -- the
  // words come back later and the step is slower (measured, with exact wait counts): every workgroup then sends
  // its 128 KiB of requests at the moment all of them wait for the words.
  if (stamp && tid == 0) stamp[13] = wall_clock64();
  if (do_prime) prime(first, tid & 63, pipe);
  if (stamp && tid == 0) stamp[15] = wall_clock64();
  if (gain == nullptr) return;  // uniform: only the residual was wanted (each lane revisits its own elements later)
#pragma unroll
  for (int m = 0; m < M; ++m) ss[m] = wave_sum(ss[m]);
  if ((tid & 63) == 0) {
#pragma unroll
    for (int m = 0; m < M; ++m) red[(tid >> 6) * M + m] = ss[m];
  }
  wg_sync();
  if (stamp && tid == 0) stamp[14] = wall_clock64();
  // pass 2: scale in place (each lane revisits the elements it wrote)
#pragma unroll
  for (int m = 0; m < M; ++m) {
    float s1 = 0.0f;
#pragma unroll
    for (int wv = 0; wv < NW; ++wv) s1 += red[wv * M + m];
    const float inv = rsqrtf(s1 / (float)D + p.eps);
#pragma unroll
    for (int it = 0; it < PRO_NIT; ++it) {
      const int c = (it * NT + tid) * 8;
      if (c >= D) break;
      float v[8], g[8], o[8];
      unpack8(*reinterpret_cast<const uint4*>(x + m * D + c), v);
      unpack8(gq[it], g);
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = round_bf(v[j] * inv) * g[j];
      st16(x + m * D + c, pack8(o));
    }
  }
  wg_sync();
}

// Bring a tagged activation [M][K] into LDS as bf16 (waits for every word).
template <int M>
__device__ __forceinline__ void load_x(const Coh& coh, unsigned src_wo, unsigned tag, int K, u16* x) {
  const int tid_ = opaque_tid();
  for (int c = tid_ * 8; c < M * K; c += NT * 8) {
    float f[8];
    coh.ld8(src_wo + c, tag, f);
    st16(x + c, pack8(f));
  }
  wg_sync();
}

// ------------------------------------------------------------------------------------------------
// Attention of slot t in attention workgroup `aw` of NA: keys [k0, k1) of every (sequence, kv
// head), all G q heads of the kv head at once so K and V are read once per GQA group.  The K and V
// rows of the key range are loaded into registers in one go (before q is waited for), scores,
// softmax and P.V stay in fp32; each workgroup publishes an un-normalised partial result with its
// own (max, sum) as tagged fp32 word pairs.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ void rope_pair(float x0, float x1, float c, float s, float& o0, float& o1) {
#pragma clang fp contract(off)
  const float a = x0 * c, b = x1 * s, d = x1 * c, e = x0 * s;
  o0 = round_bf(a - b);
  o1 = round_bf(d + e);
}

constexpr int ATT_KT = 2;  // 32-key tiles of K an attention wave keeps in registers (MFMA operand layout)
template <int HD>
struct KV {
  uint4 k[ATT_KT][HD / 16];  // tile t, k-step s: key = lane % 32 of the tile, elements s * 16 + (lane / 32) * 8 .. + 8
  uint4 v[ATT_NI];           // key group layout (see attention_load)
};

template <int HD>
__device__ __forceinline__ void attention_load(const StepParams& p, const LayerPtrs& lp, int b, int kvh, int k0,
                                               int k1, int pos, KV<HD>& kv) {
  constexpr int LPK = HD / 8, KPW = 64 / LPK;
  const int tid_ = opaque_tid();
  const int wave = tid_ >> 6, lane = tid_ & 63;
  const int kl = lane / LPK, dl = (lane % LPK) * 8;
  const u16* kbase = lp.k_cache + ((int64_t)b * p.Hkv + kvh) * p.Smax * HD;
  const u16* vbase = lp.v_cache + ((int64_t)b * p.Hkv + kvh) * p.Smax * HD;
  // K: tile (wave + NW * t) of 32 keys; a lane holds, per k-step, the 8 elements the MFMA wants from it
#pragma unroll
  for (int t = 0; t < ATT_KT; ++t) {
    const int key = k0 + (t * NW + wave) * 32 + (lane & 31);
    const bool live = key < k1 && key != pos;  // the slot of `pos` is filled from this step's qkv
#pragma unroll
    for (int s = 0; s < HD / 16; ++s)
      kv.k[t][s] = live ? gld16(kbase + (int64_t)key * HD + s * 16 + (lane >> 5) * 8) : make_uint4(0, 0, 0, 0);
  }
#pragma unroll
  for (int i = 0; i < ATT_NI; ++i) {
    const int key = k0 + (i * NW + wave) * KPW + kl;
    const bool live = key < k1 && key != pos;
    kv.v[i] = live ? gld16(vbase + (int64_t)key * HD + dl) : make_uint4(0, 0, 0, 0);
  }
}

template <int M, int HD, int G>
__device__ __forceinline__ void attention_compute(const StepParams& p, const Coh& coh, const LayerPtrs& lp, int b,
                                                  int kvh, int k0, int k1, int pos, unsigned tag,
                                                  unsigned long long* stamp,
                                                  KV<HD>& kv, u32* qp,
                                                  float* sc, int sc_ld, float* ored, u32* kp, float* vnew,
                                                  float* s_m, float* s_l) {
  constexpr int LPK = HD / 8, KPW = 64 / LPK;
  const int tid = opaque_tid(), wave = tid >> 6, lane = tid & 63;
  const int aw = (int)blockIdx.x % p.NAK, NA = p.NAK, Hkv = p.Hkv, Hq = Hkv * G;  // key range, ranges per head
  const int n = k1 - k0;
  const bool owner = pos >= k0 && pos < k1;
  const float scale = rsqrtf((float)HD);
  const u16* trow = p.rope + (int64_t)pos * HD;  // (cos, sin) pairs of this position
  const int kl = lane / LPK, dl = (lane % LPK) * 8;
  const unsigned qkv = p.oqkv + (unsigned)(b * p.nqkv);
  // partial outputs: [b * Hq + h][NA][HD] fp32 as word pairs; (max, sum): [b * Hq + h][NA] as 4 words
  const unsigned o_out = p.oopart + (unsigned)((((b * Hq + kvh * G) * NA) + aw) * HD * 2);
  const unsigned ml_out = p.omlpart + (unsigned)((((b * Hq + kvh * G) * NA) + aw) * 4);

  // Everything this phase waits for is requested at once; what has not landed yet is polled.
  const bool own = owner && tid < HD / 2;
  const unsigned ko = qkv + (unsigned)(Hq * HD + kvh * HD + 2 * tid), vo = ko + (unsigned)(Hkv * HD);
  const unsigned q0 = qkv + (unsigned)(kvh * G * HD + 2 * tid);  // pair `tid` of the G * HD / 2 pairs of this group
  u32x2_t qr = {0u, 0u}, rk = {0u, 0u}, rv = {0u, 0u};
  if (tid < G * HD / 2) qr = coh.raw2(q0);
  if (own) {
    rk = coh.raw2(ko);
    rv = coh.raw2(vo);
  }
  // ---- rotate q (all G heads) into LDS; the owner of `pos` also rotates k, keeps k/v in LDS and
  //      writes them to the cache for the following steps
  for (int i = tid; i < G * HD / 2; i += NT) {
    const int g = i / (HD / 2), j = i - g * (HD / 2);
    const unsigned qo = qkv + (unsigned)((kvh * G + g) * HD + 2 * j);
    const u32x2_t sq = i == tid ? coh.settle2(qo, tag, qr) : coh.poll2(qo, tag);
    const u32 cs = *reinterpret_cast<const u32*>(trow + 2 * j);
    float r0, r1;
    rope_pair(__uint_as_float(sq.x & 0xffff0000u), __uint_as_float(sq.y & 0xffff0000u), bf_lo(cs), bf_hi(cs), r0, r1);
    qp[g * (HD / 2) + j] = pack_bf2(r0, r1);  // exact: both were just rounded to bf16
  }
  if (own) {
    const int j = tid;
    const u32x2_t sk = coh.settle2(ko, tag, rk), sv = coh.settle2(vo, tag, rv);
    const float kx0 = __uint_as_float(sk.x & 0xffff0000u), kx1 = __uint_as_float(sk.y & 0xffff0000u);
    const float v0 = __uint_as_float(sv.x & 0xffff0000u), v1 = __uint_as_float(sv.y & 0xffff0000u);
    float r0, r1;
    const u32 cs = *reinterpret_cast<const u32*>(trow + 2 * j);
    rope_pair(kx0, kx1, bf_lo(cs), bf_hi(cs), r0, r1);
    kp[j] = pack_bf2(r0, r1);
    vnew[2 * j] = v0; vnew[2 * j + 1] = v1;
    const int64_t slot = (((int64_t)b * Hkv + kvh) * p.Smax + pos) * HD + 2 * j;
    gst4(lp.k_cache + slot, pack_bf2(r0, r1));
    gst4(lp.v_cache + slot, pack_bf2(v0, v1));
  }
  wg_sync();
  if (stamp && tid == 0) stamp[10] = wall_clock64();
  if (n <= 0) {
    for (int i = tid; i < G * HD; i += NT)
      coh.st_f32(o_out + (unsigned)(((i / HD) * NA * HD + (i % HD)) * 2), 0.0f, tag);
    if (tid < G) {
      coh.st_f32(ml_out + (unsigned)(tid * NA * 4), -INFINITY, tag);
      coh.st_f32(ml_out + (unsigned)(tid * NA * 4 + 2), 0.0f, tag);
    }
    wg_sync();
    return;
  }
  // ---- scores on the matrix cores: S[key][head] = sum_d K[key][d] q[head][d], one 32 x 32 tile per
  //      32 keys (columns beyond the G heads multiply zeros), HD / 16 v_mfma_f32_32x32x16_bf16 each
#pragma unroll
  for (int t = 0; t < ATT_KT; ++t) {
    const int tile0 = (t * NW + wave) * 32;
    if (tile0 < n) {  // uniform
      const int key = k0 + tile0 + (lane & 31);
      const int g = lane & 31;
      f32x16_t acc;
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
#pragma unroll
      for (int s = 0; s < HD / 16; ++s) {
        const int e0 = s * 16 + (lane >> 5) * 8;
        uint4 ka = kv.k[t][s];
        if (key == pos) ka = *reinterpret_cast<const uint4*>(kp + e0 / 2);
        const uint4 qb = g < G ? *reinterpret_cast<const uint4*>(qp + g * (HD / 2) + e0 / 2) : make_uint4(0, 0, 0, 0);
        const u32x4_t kav = {ka.x, ka.y, ka.z, ka.w}, qbv = {qb.x, qb.y, qb.z, qb.w};
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, kav), __builtin_bit_cast(bf16x8_t, qbv),
                                                      acc, 0, 0, 0);
      }
      // accumulator element v: key row (v / 4) * 8 + (lane / 32) * 4 + v % 4, head column lane % 32
      if (g < G) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int kr = tile0 + (v / 4) * 8 + (lane >> 5) * 4 + (v % 4);
          if (kr < n) sc[g * sc_ld + kr] = acc[v] * scale;
        }
      }
    }
  }
  wg_sync();
  if (stamp && tid == 0) stamp[11] = wall_clock64();
  // ---- softmax statistics: a wave per head; sc becomes exp(s - max)
  for (int g = wave; g < G; g += NW) {
    float m = -INFINITY;
    for (int i = lane; i < n; i += 64) m = fmaxf(m, sc[g * sc_ld + i]);
    m = wave_max_xbar(m);
    float l = 0.0f;
    for (int i = lane; i < n; i += 64) {
      const float e = expf(sc[g * sc_ld + i] - m);
      sc[g * sc_ld + i] = e;
      l += e;
    }
    l = wave_sum_xbar(l);
    if (lane == 0) { s_m[g] = m; s_l[g] = l; }
  }
  wg_sync();
  if (stamp && tid == 0) stamp[12] = wall_clock64();
  // ---- P.V: GB heads at a time share the unpacked V rows; the key groups of a wave are folded with
  //      lane-half / lane-row swaps (one swap + one add folds two accumulators), the waves in LDS
  constexpr int GB = G < 8 ? G : 8;
#pragma unroll 1
  for (int g0 = 0; g0 < G; g0 += GB) {
    float acc[GB][8];
#pragma unroll
    for (int g = 0; g < GB; ++g)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[g][j] = 0.0f;
#pragma unroll
    for (int i = 0; i < ATT_NI; ++i) {
      if (i * NW * KPW < n) {
        const int key = k0 + (i * NW + wave) * KPW + kl;
        float vf[8];
        unpack8(kv.v[i], vf);
        if (key == pos) {
#pragma unroll
          for (int j = 0; j < 8; ++j) vf[j] = vnew[dl + j];
        }
#pragma unroll
        for (int g = 0; g < GB; ++g) {
          const float pr = key < k1 ? sc[(g0 + g) * sc_ld + key - k0] : 0.0f;
#pragma unroll
          for (int j = 0; j < 8; ++j) acc[g][j] = fmaf(pr, vf[j], acc[g][j]);
        }
      }
    }
#pragma unroll
    for (int g = 0; g < GB; ++g) {
      if (LPK == 8) {  // 8 key groups: fold lane bit 3 first
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[g][j] += dpp_mov<0x128>(acc[g][j]);  // row_ror:8
      }
      float w[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        swap32(acc[g][j], acc[g][j + 4]);
        w[j] = acc[g][j] + acc[g][j + 4];
      }
      swap16(w[0], w[2]);
      swap16(w[1], w[3]);
      // lane row r = lane / 16 now holds the wave totals of elements 2r (z0) and 2r + 1 (z1) of the
      // lane's 8-element slice
      const float z0 = w[0] + w[2], z1 = w[1] + w[3];
      if (LPK == 16 || (lane & 8) == 0)
        *reinterpret_cast<float2*>(ored + (wave * G + g0 + g) * HD + dl + 2 * (lane >> 4)) = make_float2(z0, z1);
    }
  }
  wg_sync();
  for (int i = tid; i < G * HD; i += NT) {
    float v = 0.0f;
#pragma unroll
    for (int wv = 0; wv < NW; ++wv) v += ored[wv * G * HD + i];
    coh.st_f32(o_out + (unsigned)(((i / HD) * NA * HD + (i % HD)) * 2), v, tag);
  }
  if (tid < G) {
    coh.st_f32(ml_out + (unsigned)(tid * NA * 4), s_m[tid], tag);
    coh.st_f32(ml_out + (unsigned)(tid * NA * 4 + 2), s_l[tid], tag);
  }
  wg_sync();
}

// Attention workgroup `aw`: merge the NA partial results for its share of the output pairs,
//   y = sum_s w_s o_s,  w_s = exp(m_s - max) / sum_s' exp(m_s' - max) l_s',
// and publish them as tagged bf16 words at p.oy ([M][Hq * HD]); everyone else then reads 2 bytes of
// payload per output element instead of NA fp32 partials.
template <int M, int HD>
__device__ __forceinline__ void attention_merge_slice(const StepParams& p, const Coh& coh, int Hq, unsigned tag,
                                                      float* wbuf, int aw) {
  const int tid = opaque_tid(), wave = tid >> 6, lane = tid & 63;
  const int NA = p.NAK, nbh = p.B * Hq;  // partial results per head
  const int npairs = nbh * HD / 2;
  const int per = (npairs + p.NA - 1) / p.NA;  // every attention workgroup merges a share of the outputs
  const int p0 = aw * per, p1 = p0 + per < npairs ? p0 + per : npairs;
  if (p0 >= p1) return;
  u32x4_t raw[NA_MAX];
  {
    const int pp = p0 + tid;
    const int bh = (2 * pp) / HD, d = (2 * pp) % HD;
#pragma unroll
    for (int s = 0; s < NA_MAX; ++s)
      raw[s] = (s < NA && pp < p1) ? coh.raw4(p.oopart + (unsigned)(((bh * NA + s) * HD + d) * 2))
                                   : u32x4_t{0u, 0u, 0u, 0u};
  }
  const int bh0 = (2 * p0) / HD, bh1 = (2 * (p1 - 1)) / HD;
  for (int bh = bh0 + wave; bh <= bh1; bh += NW) {
    float m = -INFINITY, l = 0.0f;
    if (lane < NA) f32x2_from(coh.poll4(p.omlpart + (unsigned)((bh * NA + lane) * 4), tag), m, l);
    const float mx = wave_max_xbar(m);
    const float w = m == -INFINITY ? 0.0f : expf(m - mx);
    const float L = wave_sum_xbar(w * l);
    if (lane < NA) wbuf[bh * NA_MAX + lane] = L > 0.0f ? w / L : 0.0f;
  }
  wg_sync();
  for (int pp = p0 + tid; pp < p1; pp += NT) {
    const int bh = (2 * pp) / HD, d = (2 * pp) % HD;
    float y0 = 0.0f, y1 = 0.0f;
    if (pp != p0 + tid) {
#pragma unroll
      for (int s = 0; s < NA_MAX; ++s)
        if (s < NA) raw[s] = coh.raw4(p.oopart + (unsigned)(((bh * NA + s) * HD + d) * 2));
    }
#pragma unroll
    for (int s = 0; s < NA_MAX; ++s) {
      if (s < NA) {
        float o0, o1;
        f32x2_from(coh.settle4(p.oopart + (unsigned)(((bh * NA + s) * HD + d) * 2), tag, raw[s]), o0, o1);
        const float w = wbuf[bh * NA_MAX + s];
        y0 = fmaf(w, o0, y0);
        y1 = fmaf(w, o1, y1);
      }
    }
    coh.st2(p.oy + (unsigned)(2 * pp), round_bf(y0), round_bf(y1), tag);
  }
  wg_sync();
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
  u16* xb = xa + xlen;                                  // MLP-chain input        [M][<= max(D, I)]
  u16* xr = xb + xlen;                                  // residual stream        [M][D]
  float* part = reinterpret_cast<float*>(xr + M * D);   // [NW][NJMAX * M]
  float* red = part + NW * NJMAX * M;                   // [NW][M] (space for [NW][M][2])
  float* qs = red + NW * M * 2;                         // [G][HD / 2] packed bf16 pairs (space for [G][HD])
  float* sc = qs + G * HD;                              // [G][sc_ld]
  float* ored = sc + G * sc_ld;                         // [NW][G][HD]
  float* knew = ored + NW * G * HD;                     // [HD / 2] packed bf16 pairs (space for [HD])
  float* vnew = knew + HD;                              // [HD]
  float* s_m = vnew + HD;                               // [G]
  float* s_l = s_m + G;                                 // [G]
  float* wbuf = s_m + ((2 * G + 3) & ~3);               // [M * Hq][NA_MAX]   (what follows stays 16-byte aligned for odd G)
  float* cand_v = wbuf + M * Hq * NA_MAX;               // [NJMAX * M]
  int* cand_i = reinterpret_cast<int*>(cand_v + NJMAX * M);
  int* s_flag = cand_i + NJMAX * M;                     // [8]
  u32* lring = reinterpret_cast<u32*>(s_flag + 8);      // [4][16] layer pointer records
  int* jtab = s_flag + 8 + 64;                               // [JK_COUNT][NW][16] job table, then [JK_COUNT][NJMAX] row offsets

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int w = blockIdx.x, nwg = gridDim.x, NA = p.NA;
  Ctrl* ctrl = reinterpret_cast<Ctrl*>(p.ws);
  Coh coh;
  coh.r = __builtin_amdgcn_make_buffer_rsrc(p.ws, 0, (int)p.ws_bytes, 0x00020000);
  {
    const unsigned long long base = reinterpret_cast<unsigned long long>(p.ws);
    coh.rs.x = LR_UNI((unsigned)base);
    coh.rs.y = LR_UNI((unsigned)(base >> 32) & 0xffffu);
    coh.rs.z = LR_UNI(p.ws_bytes);
    coh.rs.w = 0x00020000u;
  }
  coh.fail = &ctrl->fail;
  if (tid == 0) {
    s_flag[1] = (int)cldu(&ctrl->epoch_base);
    s_flag[0] = (int)cldu(&ctrl->fail);
  }
  build_job_table(p, jtab, Hq * HD, w, nwg);
  if (tid < 32 && (tid >> 4) < L) lring[tid] = reinterpret_cast<const u32*>(p.layers)[tid];  // layers 0 and 1
  wg_sync();
  build_row_table(jtab, jtab + JK_COUNT * NW * 16);
  wg_sync();
  const unsigned epoch_base = (unsigned)s_flag[1];
  const int pos = p.pos[0];
  // A position outside the cache or the RoPE table: nothing is computed or written (every workgroup
  // takes the same decision from the same word), the failure word says why.  A workspace whose
  // failure word is already set stays out of service until it is initialised again.
  if (pos < 0 || pos >= p.Smax || pos >= p.block_size) {
    if (w == 0 && tid == 0 && s_flag[0] == 0) cstu(&ctrl->fail, FAIL_POS);
    return;
  }
  if (s_flag[0]) return;
  const bool att_wg = w < NA;
  // attention key range of this workgroup
  const int nkeys = pos + 1;
  const int chunk = (nkeys + p.NAK - 1) / p.NAK;
  const int k0 = (w % p.NAK) * chunk;
  const int k1 = k0 + chunk < nkeys ? k0 + chunk : nkeys;

  const int qdim = Hq * HD;
  Pipe pipe;

#ifdef LR_STEP_PROFILE
#define LR_STAMP(k)                                                                                  \
  if (p.prof && t >= p.prof_t0 && t < p.prof_t0 + PROF_SLOTS && tid == 0)                            \
    p.prof[((size_t)blockIdx.x * PROF_SLOTS + (t - p.prof_t0)) * PROF_POINTS + (k)] = wall_clock64();
#define LR_STAMP_PTR                                                                                 \
  ((p.prof && t >= p.prof_t0 && t < p.prof_t0 + PROF_SLOTS)                                          \
       ? p.prof + ((size_t)blockIdx.x * PROF_SLOTS + (t - p.prof_t0)) * PROF_POINTS : nullptr)
#else
#define LR_STAMP(k)
#define LR_STAMP_PTR nullptr
#endif
#define LR_JOB(jk, field) load_job(jtab, jk, wave, ring_ptr(lring, t, field))
  const Job no_job = load_job(jtab, JK_NONE, wave, nullptr);
  const Job j_head = load_job(jtab, JK_HEAD, wave, p.out_w);
  // Slot t = layer t: attention(t) and mlp(t) both read the residual stream before the other's
  // output is added (the ladder schedule: in the reference both outputs are in flight in an
  // all-reduce at that point), so they run side by side.  Order of the hand-overs in a slot, each
  // with independent streaming between producer and consumer:
  //   a(t-1) [written by wo(t-1), then w2(t-1) streamed]      -> residual + attention norm -> wqkv(t)
  //   m(t-1) [written by w2(t-1), then the norm and wqkv(t)]  -> residual + ffn norm       -> w1(t)
  //   qkv(t) -> attention(t) on NA workgroups while the others stream w1(t) -> merged y(t) -> wo(t)
  //   act(t) [written by w1(t), then wo(t) streamed]          -> w2(t)
  // The m words are requested a phase ahead, before wqkv's rows, and w1's first weight units go out at
  // the end of wqkv: the ffn norm then finds its words there and w1 its first units.  (The same for the
  // a words -- requested while w2's epilogue runs -- is slower: they are often not all written yet, and a
  // word found stale costs a second dependent round trip.)
  // Overwriting an exchange array is safe by data flow alone: e.g. a(t) is written in wo(t), which
  // needs all of y(t), which needs every attention workgroup's merge, which needs all of qkv(t),
  // which every workgroup produces after it has read a(t-1); likewise for m (through act(t) and,
  // for the attention workgroups, y(t)), qkv, the partial results, y and act.
  // (The loop is rotated: the residual step that opens slot t + 1 sits at the END of iteration t, so
  // that it and the closing step after the last layer are one piece of code.)
  EarlyWords<M> ew;
  issue_words<M>(coh, false, 0u, D, ew);
  // ---------------- slot 0 opens with R = embedding rows; attention norm; the first weight units of wqkv(0)
  residual_step<M>(p, coh, xr, p.tokens, false, 0u, 0u, false, ew, false, 0u, 0u, ring_ptr(lring, 0, LP_ATTN_NORM), xa, red,
                   true, load_job(jtab, JK_QKV, wave, ring_ptr(lring, 0, LP_WQKV)), pipe);
  for (int t = 0; t < L; ++t) {
    // request the pointer record of layer t + 2 now; it goes into the ring at the end of the slot
    u32 ring_next = 0;
    if (tid < 16 && t + 2 < L) ring_next = reinterpret_cast<const u32*>(p.layers + t + 2)[tid];
    const unsigned tag = tag_of(epoch_base + (unsigned)t + 1u), tag_prev = tag_of(epoch_base + (unsigned)t);
    const unsigned act_wo = p.oact + (unsigned)((t & 1) * M * I);  // activations alternate between two buffers
    LR_STAMP(1)
#ifdef LR_STEP_PROFILE
    // where this workgroup runs: XCC_ID (hardware register 20) above the low 16 bits of HW_ID (register 4: wave,
    // SIMD, pipe, CU, shader array, shader engine), in stamp 9
    if (p.prof && t >= p.prof_t0 && t < p.prof_t0 + PROF_SLOTS && tid == 0)
      p.prof[((size_t)blockIdx.x * PROF_SLOTS + (t - p.prof_t0)) * PROF_POINTS + 9] =
          ((unsigned long long)__builtin_amdgcn_s_getreg((31 << 11) | 20) << 16) |
          (__builtin_amdgcn_s_getreg((15 << 11) | 4) & 0xffffu);
#endif
    const Job j_qkv = LR_JOB(JK_QKV, LP_WQKV);
    // m(t-1) for the coming residual step: on its way while the query/key/value rows are done
    issue_words<M>(coh, t >= 1, p.om, D, ew);
    if (att_wg) {
      // (no weight units are requested across the attention phase: it is where registers are scarcest, and
      // the attention workgroups are done well before the others have streamed w1)
      run_job<M, EPI_STORE>(p, coh, j_qkv, no_job, pipe, xa, part, p.oqkv, p.nqkv, tag, nullptr, nullptr, nullptr,
                            nullptr, LR_STAMP_PTR, 16);
      LR_STAMP(2)
      coh.at(LR_STAMP_PTR, 25);
      // ---------------- attention workgroup (it owns no rows of w1): R += m(t-1) while q is on its way
      if (t >= 1)
        residual_step<M>(p, coh, xr, nullptr, true, p.om, tag_prev, true, ew, false, 0u, 0u, nullptr, xb, red, false,
                         no_job, pipe);
      LR_STAMP(3)
      coh.at(LR_STAMP_PTR, 28);
      KV<HD> kv;
      LayerPtrs lcache;  // only the cache pointers are used
      lcache.k_cache = const_cast<u16*>(ring_ptr(lring, t, LP_K_CACHE));
      lcache.v_cache = const_cast<u16*>(ring_ptr(lring, t, LP_V_CACHE));
      // this workgroup's (sequence, kv head) pairs: pair b * Hkv + kvh, NAH groups of them
      const int ppg = p.B * p.Hkv / p.NAH, pair0 = (w / p.NAK) * ppg;
      for (int pr = pair0; pr < pair0 + ppg; ++pr) {
        const int b = pr / p.Hkv, kvh = pr - b * p.Hkv;
        attention_load<HD>(p, lcache, b, kvh, k0, k1, pos, kv);
        attention_compute<M, HD, G>(p, coh, lcache, b, kvh, k0, k1, pos, tag, LR_STAMP_PTR, kv,
                                    reinterpret_cast<u32*>(qs), sc, sc_ld, ored, reinterpret_cast<u32*>(knew), vnew,
                                    s_m, s_l);
      }
      coh.at(LR_STAMP_PTR, 29);
      attention_merge_slice<M, HD>(p, coh, Hq, tag, wbuf, w);
      prime(LR_JOB(JK_WO, LP_WO), opaque_tid() & 63, pipe);
    } else {
      const Job j_w1 = LR_JOB(JK_W1_SPLIT, LP_W1);
      run_job<M, EPI_STORE>(p, coh, j_qkv, j_w1, pipe, xa, part, p.oqkv, p.nqkv, tag, nullptr, nullptr, nullptr,
                            nullptr, LR_STAMP_PTR, 16);
      LR_STAMP(2)
      coh.at(LR_STAMP_PTR, 25);
      // ---------------- everyone else: R += m(t-1); ffn norm; the up/gate projection + SwiGLU
      residual_step<M>(p, coh, xr, nullptr, t >= 1, p.om, tag_prev, t >= 1, ew, false, 0u, 0u,
                       ring_ptr(lring, t, LP_FFN_NORM), xb, red, false, no_job, pipe);
      LR_STAMP(3)
      run_job<M, EPI_SWIGLU>(p, coh, j_w1, LR_JOB(JK_WO, LP_WO), pipe, xb, part, act_wo, I, tag, nullptr, nullptr, nullptr,
                             nullptr, LR_STAMP_PTR, 18);
    }
    LR_STAMP(4)
    // ---------------- merged attention output (published by the attention workgroups), output projection
    coh.at(LR_STAMP_PTR, 26);
    load_x<M>(coh, p.oy, tag, qdim, xa);
    LR_STAMP(5)
    run_job<M, EPI_STORE>(p, coh, LR_JOB(JK_WO, LP_WO), LR_JOB(JK_W2, LP_W2), pipe, xa, part, p.oa, D, tag, nullptr,
                          nullptr, nullptr, nullptr, LR_STAMP_PTR, 20);
    LR_STAMP(6)
    // ---------------- down projection
    coh.at(LR_STAMP_PTR, 27);
    load_x<M>(coh, act_wo, tag, I, xb);
    LR_STAMP(7)
    run_job<M, EPI_STORE>(p, coh, LR_JOB(JK_W2, LP_W2), no_job, pipe, xb, part, p.om, D, tag, nullptr, nullptr, nullptr,
                          nullptr, LR_STAMP_PTR, 22);
    LR_STAMP(8)
    coh.at(LR_STAMP_PTR, 24);
    // ---------------- slot t + 1 opens: R += a(t); attention norm; the first weight units of wqkv(t + 1) go out
    //                  behind the a words.  After the last layer: x = (R + a(L-1)) + m(L-1), the final norm and
    //                  the first units of the lm_head instead.
    {
      const bool last = t + 1 == L;
      Job j_first = j_head;
      if (!last) j_first = load_job(jtab, JK_QKV, wave, ring_ptr(lring, t + 1, LP_WQKV));
      residual_step<M>(p, coh, xr, nullptr, true, p.oa, tag, false, ew, last, p.om, tag,
                       last ? p.final_norm : ring_ptr(lring, t + 1, LP_ATTN_NORM), xa, red, true, j_first, pipe,
                       LR_STAMP_PTR);
    }
    LR_STAMP(0)
    {
      const int rt = opaque_tid();  // (not hoisted out of the loop and spilled: a scratch reload waits for every load in flight)
      if (rt < 16 && t + 2 < L) lring[((t + 2) & 3) * 16 + rt] = ring_next;
    }
    // one workgroup-wide look at the failure flag per slot keeps a broken step from running on
    if (tid == 0) s_flag[0] = (int)cldu(&ctrl->fail);
    wg_sync();
    if (s_flag[0]) return;
  }
#undef LR_JOB
#undef LR_STAMP
#undef LR_STAMP_PTR
  // ---------------- head: vocab-shard lm_head on the normed x, argmax
  const unsigned tag = tag_of(epoch_base + (unsigned)L + 1u);
  float best_v = -INFINITY;
  int best_i = 0x7fffffff;
  run_job<M, EPI_LOGITS>(p, coh, j_head, no_job, pipe, xa, part, 0u, 0, tag, cand_v, cand_i, &best_v, &best_i);
  if (tid < M) {  // candidate: value (bf16-exact), a filler word, index as two 16-bit halves
    const unsigned wo = p.ocand + (unsigned)((w * M + tid) * 4);
    coh.st(wo, best_v, tag);
    coh.st(wo + 1, 0.0f, tag);
    coh.st_f32(wo + 2, __int_as_float(best_i), tag);
  }
  if (w == 0) {
    for (int m = 0; m < p.B; ++m) {
      float bv = -INFINITY;
      int bi = 0x7fffffff;
      for (int wg = tid; wg < nwg; wg += NT) {
        const u32x4_t c = coh.poll4(p.ocand + (unsigned)((wg * M + m) * 4), tag);
        const float v = __uint_as_float(c.x & 0xffff0000u);
        const int i = (int)((c.z & 0xffff0000u) | (c.w >> 16));
        if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
      }
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(bv, o, LR_WAVE);
        const int oi = __shfl_xor(bi, o, LR_WAVE);
        if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
      }
      wg_sync();
      if (lane == 0) { cand_v[wave] = bv; cand_i[wave] = bi; }
      wg_sync();
      if (tid == 0) {
        for (int wv = 1; wv < NW; ++wv)
          if (cand_v[wv] > bv || (cand_v[wv] == bv && cand_i[wv] < bi)) { bv = cand_v[wv]; bi = cand_i[wv]; }
        if (bi == 0x7fffffff) bi = 0;
        if (p.next_token) p.next_token[m] = bi;
        if (p.advance && p.cur_token) p.cur_token[m] = bi;
        const int slot = p.pos[0] - p.pos0;
        if (p.advance && p.history && slot >= 0 && slot < p.hist_len) p.history[(int64_t)m * p.ld_hist + slot] = bi;
      }
    }
    wg_sync();
    if (tid == 0) {
      if (p.advance) p.pos[0] = p.pos[0] + 1;
      cstu(&ctrl->epoch_base, (epoch_base + (unsigned)L + 2u) % 65535u);
    }
  }
}

__global__ void k_step_init(Ctrl* c, unsigned nwg, unsigned* words, unsigned n_words) {
  // control block and every exchange word start at zero: tag 0 is never a valid tag
  unsigned* cw = reinterpret_cast<unsigned*>(c);
  for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < n_words; i += gridDim.x * blockDim.x) words[i] = 0u;
  if (blockIdx.x == 0) {
    for (int i = threadIdx.x; i < (int)(sizeof(Ctrl) / 4); i += blockDim.x) cw[i] = 0u;
    __syncthreads();
    if (threadIdx.x == 0) c->nwg = nwg;
  }
}

struct Layout {
  size_t ctrl, abuf, mbuf, qkv, act, opart, mlpart, cand, y, total;
};

// keys one attention workgroup can hold in registers: the V groups (ATT_NI * NW * keys per wave)
// and the K tiles of the score pass (ATT_KT * NW * 32) both have to cover its key range
static int att_capacity(int hd) {
  const int v_keys = ATT_NI * NW * (64 / (hd / 8)), k_keys = ATT_KT * NW * 32;
  return v_keys < k_keys ? v_keys : k_keys;
}
// LDS row length of the score buffer (the larger of the two, so either bound may be the binding one)
static int att_sc_ld(int hd) { return ATT_NI * NW * (64 / (hd / 8)); }

// `want_na` > 0: the caller's lower bound for the number of attention workgroups (lr_ladder_model_t)
static int pick_na(int Smax, int hd, int nwg, int want_na) {
  const int cap = att_capacity(hd);
  int na = (Smax + cap - 1) / cap;
  // more attention workgroups than capacity requires pay off up to about 128 keys each: attention is
  // instruction bound and sits on the critical path next to the w1 stream
  int want = (Smax + 127) / 128;
  if (want > NA_MAX) want = NA_MAX;
  if (want > nwg / 8) want = nwg / 8;
  if (want > na) na = want;
  if (want_na > NA_MAX) want_na = NA_MAX;
  if (want_na > na) na = want_na;
  if (na < 1) na = 1;
  if (na >= nwg) na = nwg - 1;
  return na;
}

// How the attention workgroups are laid out: `nak` key ranges times `nah` groups of (sequence, kv head) pairs.  With one kv
// head per rank (a TP shard) that is pick_na key ranges.  With several kv heads a workgroup that walked all of
// them one after the other would keep the weight-streaming workgroups waiting (8B model: 62 us of attention
// against 34 us of w1 per layer), so every kv head gets workgroups of its own and the key ranges become as long
// as the registers allow (at most 256 keys), within a quarter of the grid.
struct AttSplit {
  int nak, nah;
};
static AttSplit pick_split(const lr_ladder_model_t* md, int nwg, int B = 1) {
  const int hd = md->head_dim, hkv = md->n_kv_head;
  AttSplit a;
  if (hkv == 1) {
    a.nak = pick_na(md->smax, hd, nwg, md->attention_workgroups);
    // two sequences: each gets key-range workgroups of its own (walked one after the other by the same workgroups,
    // the attention takes 22.5 us per layer against 16.3 us of up/gate on the 70B shard)
    a.nah = (B == 2 && 2 * a.nak <= nwg / 4) ? 2 : 1;
    return a;
  }
  const int cap = att_capacity(hd) < 256 ? att_capacity(hd) : 256;
  a.nak = (md->smax + cap - 1) / cap;
  if (md->attention_workgroups > a.nak) a.nak = md->attention_workgroups;
  if (a.nak > NA_MAX) a.nak = NA_MAX;
  if (a.nak < 1) a.nak = 1;
  // kv heads per workgroup: whichever division makes the slower of the two sides fastest.  The model (times in
  // microseconds, measured on the MI355X): the other workgroups stream w1 at about 30 GB/s each; an attention
  // workgroup needs 4 to get q, 2.5 + 0.04 per key for each of its kv heads, 3 for its share of the merge.
  const float keys = (float)((md->smax + a.nak - 1) / a.nak);
  float best = 3.0e38f;
  a.nah = 1;
  const int pairs = B * hkv;  // (sequence, kv head) pairs to go round
  for (int nah = 1; nah <= pairs; ++nah) {
    if (pairs % nah || a.nak * nah > nwg / 2) continue;
    const float t_att = 7.0f + (float)(pairs / nah) * (2.5f + 0.04f * keys);
    const float t_w1 = 4.0f * (float)md->ffn * (float)md->dim / (float)(nwg - a.nak * nah) / 30.0e3f;
    const float t = t_att > t_w1 ? t_att : t_w1;
    if (t < best) { best = t; a.nah = nah; }
  }
  if (a.nak < 1) a.nak = 1;
  if (a.nak * a.nah >= nwg) a.nak = (nwg - 1) / a.nah > 0 ? (nwg - 1) / a.nah : 1;
  return a;
}

static Layout make_layout(const lr_ladder_model_t* md, int B, int nwg) {
  const int D = md->dim, Hq = md->n_head, hd = md->head_dim;
  const int nqkv = (Hq + 2 * md->n_kv_head) * hd;
  const int na = pick_split(md, nwg).nak;  // partial results per head
  auto up = [](size_t x) { return (x + 255) & ~(size_t)255; };
  Layout l;
  size_t o = 0;
  l.ctrl = o; o = up(o + sizeof(Ctrl));
  l.abuf = o; o = up(o + 4 * (size_t)B * D);
  l.mbuf = o; o = up(o + 4 * (size_t)B * D);
  l.qkv = o; o = up(o + 4 * (size_t)B * nqkv);
  l.act = o; o = up(o + 4 * (size_t)2 * B * md->ffn);
  l.opart = o; o = up(o + 4 * (size_t)B * Hq * na * hd * 2);
  l.mlpart = o; o = up(o + 4 * (size_t)B * Hq * na * 4);
  l.cand = o; o = up(o + 4 * (size_t)nwg * B * 4);
  l.y = o; o = up(o + 4 * (size_t)B * Hq * hd);
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
  const size_t fl = (size_t)NW * NJMAX * M + NW * M * 2 + G * HD + (size_t)G * att_sc_ld(HD) + NW * G * HD +
                    2 * HD + ((2 * G + 3) & ~3) + (size_t)M * Hq * NA_MAX + 2 * NJMAX * M + 8 + 64 + JK_COUNT * NW * 16 + JK_COUNT * NJMAX;
  return ((size_t)xlen * 2 + (size_t)M * D) * sizeof(u16) + fl * sizeof(float) + 16;
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
  // every cache slot needs a row of the RoPE table (block_size rows); the cache length itself is rounded up to 8
  if (md->smax > ((md->block_size + 7) & ~7)) return LR_E_SHAPE;
  if (B > 2 || md->dim > PRO_NIT * NT * 8 || md->dim % 8 || md->ffn % 8 || (md->head_dim != 64 && md->head_dim != 128))
    return LR_E_UNSUPPORTED;
  const int G = md->n_head / md->n_kv_head;
  if (!has_instance(B, md->head_dim, G)) return LR_E_UNSUPPORTED;
  if (md->n_head * md->head_dim > 16384 || md->ffn > 16384) return LR_E_UNSUPPORTED;
  if (W8) {
    // 16 weights per lane and row; a matrix and its scales are addressed with 32-bit byte offsets
    if (md->dim % 16 || md->ffn % 16 || (md->n_head * md->head_dim) % 16) return LR_E_UNSUPPORTED;
    const int64_t qkv_rows = (int64_t)(md->n_head + 2 * md->n_kv_head) * md->head_dim;
    const int64_t most = std::max<int64_t>(std::max<int64_t>(qkv_rows, 2 * (int64_t)md->ffn), md->out_rows) * md->dim;
    if (most >= 0x7fffffff || (int64_t)md->dim * md->ffn >= 0x7fffffff) return LR_E_UNSUPPORTED;
  }
  if (lds_need(B, md->head_dim, G, md->dim, md->ffn, md->n_head) > 160 * 1024) return LR_E_UNSUPPORTED;
  const int nwg = lr_num_cus();
  if (nwg < 2) return LR_E_LAUNCH;
  if (md->dim > NJMAX * nwg) return LR_E_UNSUPPORTED;  // a workgroup's rows of wo / w2 fit one reduction round
  // Overwriting an exchange array is ordered by data flow through the rows every workgroup produces (see the layer
  // loop): a workgroup without a row of wqkv, or a weight-streaming workgroup without a row pair of w1, would not
  // be part of that chain.  Such shapes (fewer q/k/v rows than CUs) are left to the per-op kernels.
  if ((md->n_head + 2 * md->n_kv_head) * md->head_dim < nwg) return LR_E_UNSUPPORTED;
  const AttSplit as = pick_split(md, nwg, B);
  if (as.nak > NA_MAX || (md->smax + as.nak - 1) / as.nak > att_capacity(md->head_dim) || as.nak * as.nah >= nwg ||
      (B * md->n_kv_head) % as.nah)
    return LR_E_UNSUPPORTED;
  if (md->ffn < nwg - as.nak * as.nah) return LR_E_UNSUPPORTED;
  if (!md->tok_embeddings || !md->norm || !md->output || !md->freqs_cis || !md->layers_dev) return LR_E_NULL;
  return LR_OK;
}

// Workgroups of one instance that can be resident on the current device at once, for `lds` bytes of dynamic LDS
// (occupancy per CU x CUs; 0 if the runtime cannot tell).  The answer for the largest size asked so far is kept per
// device: occupancy does not grow with the LDS size, so a smaller request is covered by it.
template <int M, int HD, int G>
static int resident_workgroups(size_t lds) {
  static std::atomic<unsigned long long> lds_raised{0};
  static std::atomic<size_t> asked[LR_MAX_DEVICES];
  static std::atomic<int> fits[LR_MAX_DEVICES];
  const void* fn = reinterpret_cast<const void*>(&k_ladder_step<M, HD, G>);
  const int dev = lr_current_device();
  if (dev < 0 || !lr_raise_lds_limit(fn, lds, lds_raised)) return 0;
  if (lds <= asked[dev].load(std::memory_order_acquire)) return fits[dev].load(std::memory_order_relaxed);
  int per_cu = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, fn, NT, lds) != hipSuccess || per_cu < 0) return 0;
  const int n = per_cu * lr_num_cus();
  if (n > 0) {  // (a size that does not fit is asked about again next time: nothing to remember)
    fits[dev].store(n, std::memory_order_relaxed);
    asked[dev].store(lds, std::memory_order_release);
  }
  return n;
}

template <int M, int HD, int G>
static int launch_step(const StepParams& sp, int Hq, hipStream_t s) {
  const size_t lds = lds_bytes<M, HD, G>(sp.D, sp.I, Hq);
  // Every workgroup polls words that the others write, so all of them have to be resident at the same time: a
  // launch that the device cannot hold whole is refused here instead of running into its bounded waits.  (What
  // else occupies the device at that moment is not known here; that case ends in LR_DEV_WAIT_EXPIRED.)
  const int grid = lr_num_cus();
  if (resident_workgroups<M, HD, G>(lds) < grid) return LR_E_LAUNCH;
  k_ladder_step<M, HD, G><<<dim3(grid), dim3(NT), lds, s>>>(sp);
  return lr_launch_status();
}

#ifdef LR_STEP_PROFILE
unsigned long long* g_prof = nullptr;  // device buffer for phase timestamps
int g_prof_t0 = 0;
#endif

}  // namespace

#ifdef LR_STEP_PROFILE
// Profile builds only (not declared in the public header): following steps record, per workgroup,
// wall-clock stamps (100 MHz) for PROF_SLOTS consecutive slots starting at `first_slot` into
// `device_buffer` (NULL switches it off).  Returns the bytes the buffer must hold.  The e4m3 instance has a
// hook of its own (lr_ladder_step_profile_fp8).
#if LR_STEP_W8
#define LR_PROFILE_ENTRY lr_ladder_step_profile_fp8
#else
#define LR_PROFILE_ENTRY lr_ladder_step_profile
#endif
extern "C" size_t LR_PROFILE_ENTRY(void* device_buffer, int first_slot) {
  g_prof = reinterpret_cast<unsigned long long*>(device_buffer);
  g_prof_t0 = first_slot;
  return (size_t)lr_num_cus() * PROF_SLOTS * PROF_POINTS * sizeof(unsigned long long);
}
#endif

#if !LR_STEP_W8
extern "C" size_t lr_ladder_step_workspace_bytes(const lr_ladder_model_t* md, int batch) {
  if (validate(md, batch) != LR_OK) return 0;
  return make_layout(md, batch, lr_num_cus()).total;
}

extern "C" size_t lr_ladder_step_fail_offset(void) { return offsetof(Ctrl, fail); }

extern "C" int lr_ladder_step_resident_workgroups(const lr_ladder_model_t* md, int batch) {
  if (validate(md, batch) != LR_OK) return 0;
  const int G = md->n_head / md->n_kv_head, hd = md->head_dim;
#define LR_RES(MV, HDV, GV) \
  if (batch == MV && hd == HDV && G == GV) \
    return resident_workgroups<MV, HDV, GV>(lds_bytes<MV, HDV, GV>(md->dim, md->ffn, md->n_head));
  LR_STEP_INSTANCES(LR_RES)
#undef LR_RES
  return 0;
}

extern "C" int lr_ladder_step_init(const lr_ladder_model_t* md, int batch, void* workspace, size_t bytes,
                                   lr_stream_t stream) {
  const int rc = validate(md, batch);
  if (rc != LR_OK) return rc;
  LR_REQUIRE_PTR(workspace);
  if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0) return LR_E_ALIGN;
  const Layout l = make_layout(md, batch, lr_num_cus());
  if (bytes < l.total) return LR_E_SHAPE;
  k_step_init<<<dim3(64), dim3(256), 0, (hipStream_t)stream>>>(reinterpret_cast<Ctrl*>(workspace), (unsigned)lr_num_cus(),
                                                              reinterpret_cast<unsigned*>(workspace),
                                                              (unsigned)(l.total / 4));
  return lr_launch_status();
}
#endif

#if LR_STEP_W8
#define LR_STEP_ENTRY lr_ladder_decode_step_fp8
#else
#define LR_STEP_ENTRY lr_ladder_decode_step
#endif
extern "C" int LR_STEP_ENTRY(const lr_ladder_model_t* md, int batch, const int32_t* tokens, int32_t* pos,
                             void* logits, int64_t ldl, int32_t* next_token, int advance,
                             int32_t* cur_token, int32_t* history, int64_t ld_hist, int hist_len, int pos0,
                             void* workspace, size_t bytes, lr_stream_t stream) {
  const int rc = validate(md, batch);
  if (rc != LR_OK) return rc;
  LR_REQUIRE_PTR(workspace);
  LR_REQUIRE_PTR(logits);
  if (tokens == nullptr || pos == nullptr) return LR_E_NULL;
  if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0) return LR_E_ALIGN;
  const int nwg = lr_num_cus();
  const Layout l = make_layout(md, batch, nwg);
  if (bytes < l.total || ldl < md->out_rows || l.total > 0x7fffffffu) return LR_E_SHAPE;
  if (history && (ld_hist < hist_len || hist_len <= 0)) return LR_E_SHAPE;
  StepParams sp;
  sp.D = md->dim; sp.L = md->n_layer; sp.Hkv = md->n_kv_head; sp.I = md->ffn; sp.V = md->out_rows;
  sp.vocab = md->vocab; sp.Smax = md->smax; sp.block_size = md->block_size; sp.B = batch;
  const AttSplit as = pick_split(md, nwg, batch);
  sp.NAK = as.nak; sp.NAH = as.nah; sp.NA = as.nak * as.nah;
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
  sp.oa = (unsigned)(l.abuf / 4); sp.om = (unsigned)(l.mbuf / 4);
  sp.oqkv = (unsigned)(l.qkv / 4); sp.oact = (unsigned)(l.act / 4);
  sp.oopart = (unsigned)(l.opart / 4); sp.omlpart = (unsigned)(l.mlpart / 4); sp.ocand = (unsigned)(l.cand / 4);
  sp.oy = (unsigned)(l.y / 4);
#ifdef LR_STEP_PROFILE
  sp.prof = g_prof;
  sp.prof_t0 = g_prof_t0;
#else
  sp.prof = nullptr;
  sp.prof_t0 = 0;
#endif
  hipStream_t s = (hipStream_t)stream;
  const int G = md->n_head / md->n_kv_head, hd = md->head_dim;
#define LR_STEP(MV, HDV, GV) \
  if (batch == MV && hd == HDV && G == GV) return launch_step<MV, HDV, GV>(sp, md->n_head, s);
  LR_STEP_INSTANCES(LR_STEP)
#undef LR_STEP
  return LR_E_UNSUPPORTED;
}
