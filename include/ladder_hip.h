/*
 * ladder_hip.h -- C ABI of libladder_hip.so: the gfx950 (MI355X) kernels behind the per-rank
 * forward pass of the Ladder-Residual transformer.
 *
 * The reference (mayank31398/ladder-residual-inference) has no FFI: its boundary is the Python
 * module API of gpt_fast/.  Every entry point below therefore replaces a call site of a
 * PyTorch / Triton / third-party kernel in the reference, cited per function as file:line under
 * the reference root.  The host side (the gpt_fast package shipped beside the HIP sources) binds
 * them with ctypes and keeps the reference's module names and signatures.
 *
 * Conventions, all entry points:
 *   - every tensor argument is a DEVICE pointer to bf16 (uint16 storage) unless stated otherwise,
 *     dense row-major, 16-byte aligned; row strides ("ld*") are in elements and multiples of 8;
 *   - `stream` is a hipStream_t; work is only enqueued on it.  No entry point allocates,
 *     synchronises, or touches host memory after it returns, so every call can be recorded into
 *     a hipGraph by stream capture;
 *   - positions are read on the DEVICE from `pos` (int32), never from the host, so a captured
 *     decode step can be replayed after the position buffer has been advanced on the device;
 *   - what the library remembers between calls are facts about a device (the number of its compute
 *     units, which kernels have had their dynamic-LDS limit raised, how many workgroups of a kernel
 *     it can hold, the address of the built-in scratch array of lr_attn_decode_static), looked up once
 *     per device and kept in atomics: calls from several host threads and for several devices may
 *     overlap; everything else lives in the caller's buffers;
 *   - the return value is LR_OK or a negative LR_E_* code; on error nothing was launched;
 *   - arithmetic: bf16 storage, fp32 accumulation, one round-to-nearest-even at each point where
 *     the eager reference materialises a bf16 tensor.
 */
#ifndef LADDER_HIP_H
#define LADDER_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* lr_stream_t; /* hipStream_t */

enum {
  LR_OK = 0,
  LR_E_NULL = -1,        /* a required pointer is NULL                                   */
  LR_E_ALIGN = -2,       /* a pointer is not 16-byte aligned or a stride is not % 8      */
  LR_E_SHAPE = -3,       /* a size is non-positive or inconsistent                        */
  LR_E_UNSUPPORTED = -4, /* a size the kernels are not built for (e.g. head_dim)          */
  LR_E_LAUNCH = -5,      /* the HIP runtime refused the launch                            */
  LR_E_TOO_LARGE = -6    /* more scratch needed than the library's built-in buffer holds  */
};

/* Values of device-side error words (lr_rope_kv_write's `err`, the workspace word at
 * lr_ladder_step_fail_offset()): conditions only the device can see, reported without a host
 * synchronisation.  0 = none. */
enum {
  LR_DEV_WAIT_EXPIRED = 1, /* a bounded cross-workgroup wait of the step kernel ran out          */
  LR_DEV_POS_RANGE = 2     /* a position outside the KV cache or the RoPE table                  */
};

/* Library version (major*10000 + minor*100 + patch) and text for an LR_E_* code. */
int lr_version(void);
const char* lr_error_string(int code);

/* out[t, :] = table[idx[t], :]   -- tok_embeddings(idx), gpt_ladder_TP.py:256.
 * idx: int64 (idx_is_i64 != 0) or int32, n_tokens entries; ids outside [0, vocab) give a zero row. */
int lr_embed(const void* table, const void* idx, int idx_is_i64, void* out, int64_t n_tokens, int dim, int vocab,
             lr_stream_t stream);

/* out = bf16(a + bf16(b / b_div))  over n elements.  b_div == 1 is the plain add of
 * add_tensor_forward_triton_kernel (gpt_ladder_TP.py:364-377, call sites :326-332, :346-349) and
 * of the dense / parallel residual adds (gpt_dense_TP.py:281-282, gpt_parallel_TP.py:224);
 * b_div == tp is desync's pre-scaled residual (gpt_desync_TP.py:369-382). `out` may alias a or b. */
int lr_add(const void* a, const void* b, float b_div, void* out, int64_t n, lr_stream_t stream);

/* Fused residual update + RMSNorm over `rows` rows of `dim`:
 *     r = resid_in;  if (d1) r = bf16(r + d1);  if (d2) r = bf16(r + d2);
 *     if (resid_out) resid_out = r;
 *     normed_out = bf16( bf16( r * rsqrt(mean(r^2) + eps) ) * gain )
 * Replaces the ladder add followed by attention_norm / ffn_norm (gpt_ladder_TP.py:326-337,
 * :346-354), the closing x + prev_attn + prev_mlp and final norm (:280-282), and RMSNorm itself
 * (utils.py:68-74).  d1, d2, resid_out may be NULL; resid_out may alias resid_in.  dim <= 16384. */
int lr_add_rmsnorm(const void* resid_in, const void* d1, const void* d2, const void* gain, void* resid_out,
                   void* normed_out, int rows, int dim, float eps, lr_stream_t stream);

/* Both residual updates and both RMSNorms of one ladder block in one launch:
 *     r1 = bf16(resid_in + d1),  normed1 = norm(r1) * gain1      (gpt_ladder_TP.py:326-337)
 *     r2 = bf16(r1 + d2),        normed2 = norm(r2) * gain2      (gpt_ladder_TP.py:346-354)
 *     resid_out = r2
 * with norm() as in lr_add_rmsnorm.  Legal because the block's MLP input does not contain the block's own
 * attention output (that is the ladder schedule): attention(normed1) and mlp(normed2) can then run
 * side by side, e.g. on two streams.  d1 / d2 may be NULL (the first block); resid_out may alias resid_in. */
int lr_ladder_norms(const void* resid_in, const void* d1, const void* d2, const void* gain1, const void* gain2,
                    void* resid_out, void* normed1, void* normed2, int rows, int dim, float eps, lr_stream_t stream);

/* y[m, n] = bf16( sum_k x[m, k] * w[n, k] )   x [M, K] (row stride ldx), w [N, K] dense,
 * y [M, N] (row stride ldy).  nn.Linear without bias: wqkv / wo (utils.py:191, 258), w1 / w2
 * (utils.py:146, 148), wqkv1 (utils.py:311), output (gpt_ladder_TP.py:283).
 * K % 8 == 0.  The kernel is chosen from the shape: M <= 4 (and M <= 8 with act_swiglu) the
 * weight-streaming GEMV (v_dot2 on packed pairs, every weight read once); 4 < M <= 64 the
 * weight-streaming matrix-core kernel of lr_linear_multi; M >= 512 on a large enough grid the
 * 256 x 256 tile matrix-core GEMM; everything else the 128 x 128 tile matrix-core GEMM.  All of
 * them accumulate in fp32 and round once; the summation order, hence the last bit, depends on the
 * kernel.
 * act_swiglu != 0: x is taken to be [M, 2K] = [u | g] (row stride ldx) and the kernel consumes
 * bf16( bf16(silu(g)) * u ) in its place -- w2(silu(g) * u), utils.py:147-148. */
int lr_linear(const void* x, int64_t ldx, const void* w, void* y, int64_t ldy, int M, int N, int K, int act_swiglu,
              lr_stream_t stream);

/* lr_linear with the launch configuration of the GEMV given by the caller instead of chosen from
 * the shape: gemv_cfg = rows per wave * 100 + K-split * 10 + unroll, one of 144, 212, 222, 242, 244,
 * 412, 422, 442 (anything else: 242; 0: the shape heuristic, i.e. lr_linear).  A non-zero gemv_cfg
 * also selects the GEMV for M of 5 to 8, where lr_linear would take the matrix-core streaming
 * kernel; beyond M = 8 it is ignored.  No counterpart in the reference: for callers that tune per shape.
 * Results do not depend on it beyond the fp32 summation order. */
int lr_linear_tuned(const void* x, int64_t ldx, const void* w, void* y, int64_t ldy, int M, int N, int K,
                    int act_swiglu, int gemv_cfg, lr_stream_t stream);

/* Up to two projections of the same M input rows (M <= 64) in ONE launch of the weight-streaming
 * kernel, e.g. the fused q/k/v projection (utils.py:188) next to the MLP's up/gate projection
 * (utils.py:142-148) in a ladder block, whose inputs are both ready before either runs
 * (gpt_ladder_TP.py:323-349).  Per projection: y[M, N] = x[M, K] w[N, K]^T as in lr_linear
 * (epilogue LR_EPI_NONE), or, for a weight holding [up; gate] rows (N = 2 I, the layout of
 * feed_forward.w1), y[M, I] = bf16( bf16(silu(g)) * u ) with u, g the bf16-rounded projections
 * (LR_EPI_SWIGLU: utils.py:145-148 without the [M, 2 I] round trip).  Sums are fp32, added in a
 * fixed order.  The reference has no such call; it is what its compiled decode graph amounts to. */
enum { LR_EPI_NONE = 0, LR_EPI_SWIGLU = 1, LR_EPI_ROPE_KV = 2 };
/* LR_EPI_ROPE_KV: the projection is the fused q/k/v projection of a DECODE step (one token per
 * sequence, input row m = sequence m, N = (n_head + 2 n_kv_head) * head_dim) and finishes with what
 * lr_rope_kv_write does to its output: q rotated in y, rotated k and v stored at slot pos[0] of the
 * caches (utils.py:193-198, :50-59), bit for bit.  A position outside the cache or the table sets
 * *err = LR_DEV_POS_RANGE and leaves the plain projection in y. */
typedef struct lr_rope_kv {
  const void* table;  /* freqs_cis [block_size, head_dim / 2, 2] */
  const int32_t* pos; /* device: the position of this step */
  void* k_cache;      /* [B, n_kv_head, smax, head_dim] */
  void* v_cache;
  int32_t* err;       /* device error word, may be NULL */
  int32_t n_head, n_kv_head, head_dim, smax, block_size;
} lr_rope_kv_t;
typedef struct lr_projection {
  const void* x; /* [M, K] bf16, row stride ldx */
  int64_t ldx;
  const void* w; /* [N, K] bf16, dense */
  void* y;       /* [M, N] (or [M, N / 2]) bf16, row stride ldy */
  int64_t ldy;
  int32_t N, K;
  int32_t epilogue;
  const lr_rope_kv_t* rope; /* LR_EPI_ROPE_KV only, else ignored; read during the call */
} lr_projection_t;
int lr_linear_multi(const lr_projection_t* projections, int n_projections, int M, lr_stream_t stream);

/* The fused q/k/v projection of a PREFILL, finished as lr_rope_kv_write would finish it: M = B * S input rows (S
 * tokens per sequence, row b * S + s sits at position rope->pos[s], pos int32 [S] on the device),
 * y[M, N] = x[M, K] w[N, K]^T with N = (n_head + 2 n_kv_head) * head_dim, then q rotated in y, rotated k and
 * v stored at slot pos[s] of the caches, k and v left as projected in y (Attention.forward, utils.py:188-198, and
 * KVCache.update, :50-59) -- bit for bit what lr_linear followed by lr_rope_kv_write (table_is_gathered = 0)
 * leaves, in one launch of the prefill GEMM where that kernel applies (M >= 512 and enough tiles), in those two
 * calls otherwise.  A position outside the cache or the table sets *rope->err = LR_DEV_POS_RANGE and leaves that
 * row as projected.  ldy % 8 == 0. */
int lr_linear_rope_kv(const void* x, int64_t ldx, const void* w, void* y, int64_t ldy, int M, int K, int S,
                      const lr_rope_kv_t* rope, lr_stream_t stream);

/* The MLP's first projection with the activation applied on the way out (utils.py:145-148):
 *     y[M, I] = bf16( bf16(silu(g)) * u ),  [u | g] = bf16(x w^T),  w [2 I, K] = [up; gate] rows, N = 2 I.
 * M <= 64: lr_linear_multi's LR_EPI_SWIGLU; M >= 512 on a large enough grid: the 256 x 256 tile
 * matrix-core GEMM on tiles of 128 row PAIRS (a lane holds both halves of a pair); otherwise the
 * projection goes to `scratch` ([M, N] bf16, scratch_bytes >= 2 M N, then ldy must equal I) and
 * lr_swiglu follows.  scratch may be NULL when one of the first two cases applies.  Same bits as
 * lr_linear followed by lr_swiglu. */
int lr_linear_swiglu_out(const void* x, int64_t ldx, const void* w, void* y, int64_t ldy, int M, int N, int K,
                         void* scratch, size_t scratch_bytes, lr_stream_t stream);

/* lr_attn_decode and one projection of lr_linear_multi in ONE launch: the first workgroups of the grid are the
 * attention's (split, kv head, sequence) items, the rest the bands of the projection, so the projection's weight
 * stream fills the chip while the attention waits for the KV cache.  For a ladder block, whose up/gate
 * projection does not depend on the block's own attention (gpt_ladder_TP.py:339-349: the reference overlaps
 * the attention's all-reduce with the MLP for the same reason); the two halves must be independent of each
 * other.  Same bits as lr_attn_decode(q, ..., y) followed by lr_linear_multi(projection, 1, M).
 * Arguments as there.  LR_E_UNSUPPORTED (nothing launched): M > 16, an LR_EPI_ROPE_KV projection (it would write
 * the cache the attention reads), q heads per kv head other than 1, 2, 4, 8, 16 -- the caller then makes the two
 * calls. */
int lr_attn_decode_beside(const void* q, int64_t ldq, const void* k_cache, const void* v_cache, const int32_t* pos,
                          void* y, int64_t ldy, int B, int Hq, int Hkv, int hd, int Smax, void* scratch,
                          size_t scratch_bytes, const lr_projection_t* projection, int M, lr_stream_t stream);

/* Weight-only fp8 linear:  y[m, n] = bf16( bf16( sum_k x[m, k] * w8[n, k] ) * scales[n] ).
 * w8 [N, K] dense float8 e4m3 (OCP "e4m3fn": bias 7, no infinities, max 448), one byte per weight;
 * scales [N] bf16, one per output row; x, y bf16 as in lr_linear.  K % 16 == 0.
 * The reference leaves the hook of gpt-fast's weight-only quantised layers -- a Linear replacement
 * holding `weight` in the narrow type and `scales` in the model dtype (gpt_ladder_TP.py:233-237) --
 * whose forward is F.linear(x, weight.to(x.dtype)) * scales; this is that forward with e4m3 weights
 * (the reference ships no quantiser and no quantised layer, so parity at this boundary is pinned by
 * the formula only).  M <= 16 (decode) streams the fp8 weights once: half the HBM bytes of lr_linear
 * (one row: matrix-vector kernel; 2 to 16 rows: the matrix-core bands of lr_linear_fp8_multi).
 * M > 16 (prefill) expands the weights to bf16 into `scratch` (lr_linear_fp8_scratch_bytes(M, N, K)
 * bytes, 16-byte aligned), runs lr_linear on them and scales the columns; scratch may be NULL for
 * M <= 16. */
size_t lr_linear_fp8_scratch_bytes(int M, int N, int K);
int lr_linear_fp8(const void* x, int64_t ldx, const void* w8, const void* scales, void* y, int64_t ldy, int M, int N,
                  int K, void* scratch, size_t scratch_bytes, lr_stream_t stream);

/* lr_linear_multi for weight-only e4m3 projections, M <= 16 input rows (LR_E_UNSUPPORTED beyond): one or two
 * projections per launch, per projection y = F.linear(x, w8.to(bf16)) * scales with lr_linear_fp8's two roundings
 * (M == 1: the matrix-vector kernel, lr_linear_fp8's bits; from 2 rows on the matrix-core bands of lr_linear_multi
 * with the weights expanded on their way through LDS), then the epilogue on those values -- LR_EPI_SWIGLU: w8 holds [up; gate] rows, y[M, N / 2] =
 * bf16( bf16(silu(g)) * u ) (utils.py:145-148); LR_EPI_ROPE_KV: the q/k/v projection of a decode step, finished
 * as lr_rope_kv_write would (utils.py:193-198, :50-59).  What the per-op decode step of a quantised ladder block
 * needs in two launches: {q/k/v next to up/gate} and {wo next to w2} (gpt_ladder_TP.py:323-349).  K % 16 == 0. */
typedef struct lr_projection_fp8 {
  const void* x; /* [M, K] bf16, row stride ldx */
  int64_t ldx;
  const void* w8;     /* [N, K] float8_e4m3fn, dense */
  const void* scales; /* [N] bf16 */
  void* y;            /* [M, N] (or [M, N / 2]) bf16, row stride ldy */
  int64_t ldy;
  int32_t N, K;
  int32_t epilogue;
  const lr_rope_kv_t* rope; /* LR_EPI_ROPE_KV only, else ignored; read during the call */
} lr_projection_fp8_t;
int lr_linear_fp8_multi(const lr_projection_fp8_t* projections, int n_projections, int M, lr_stream_t stream);

/* lr_attn_decode_beside with a weight-only e4m3 projection (one lr_projection_fp8_t of lr_linear_fp8_multi) in
 * place of the bf16 one: the quantised ladder block's up/gate projection next to its attention.  Same bits as
 * lr_attn_decode followed by lr_linear_fp8_multi(projection, 1, M).  LR_E_UNSUPPORTED (nothing launched): M == 1
 * (lr_linear_fp8_multi uses the matrix-vector kernel there) or M > 16, an LR_EPI_ROPE_KV projection, q heads per
 * kv head other than 1, 2, 4, 8, 16. */
int lr_attn_decode_beside_fp8(const void* q, int64_t ldq, const void* k_cache, const void* v_cache,
                              const int32_t* pos, void* y, int64_t ldy, int B, int Hq, int Hkv, int hd, int Smax,
                              void* scratch, size_t scratch_bytes, const lr_projection_fp8_t* projection, int M,
                              lr_stream_t stream);

/* out[r, i] = bf16( bf16(silu(h[r, I + i])) * h[r, i] ),  h [rows, 2I] = [u | g] (row stride ldh).
 * F.silu(g) * u after chunk(2), utils.py:147-148 and :386. */
int lr_swiglu(const void* h, int64_t ldh, void* out, int rows, int I, lr_stream_t stream);

/* RoPE on q and k plus the KV-cache write, for B*S rows of a fused projection output.
 *   qkv [B*S, ldqkv]: columns [0, Hq*hd) = q, then Hkv*hd of k, then Hkv*hd of v (utils.py:191).
 *   table [block_size, hd/2, 2] bf16 (cos, sin) (utils.py:103-117); pos int32 [S] on the device.
 *   table_is_gathered == 0: the row used for token s is table[pos[s]] (the whole freqs_cis table);
 *   table_is_gathered != 0: the caller already gathered freqs_cis[input_pos] (gpt_ladder_TP.py:255),
 *   `table` has S rows (block_size = S) and token s uses row s.
 * q is rotated IN PLACE; rotated k and raw v go to k_cache / v_cache [Bmax, Hkv, Smax, hd] at
 * slot pos[s] (apply_rotary_emb utils.py:120-132, 197-198; KVCache.update utils.py:50-59,
 * 248-250).  Rotation is done in fp32 on interleaved pairs with separately rounded products.
 * Rows whose position is outside [0, Smax) (or outside the table) are left untouched -- nothing is
 * rotated, nothing is written to the cache -- and, if `err` is not NULL, the device word *err
 * (int32) is set to LR_DEV_POS_RANGE.  The reference fails with an index error there
 * (utils.py:55, gpt_ladder_TP.py:255); a device-side check cannot raise, so the caller reads the
 * word when it next synchronises.  The word is only ever set, never cleared, by the library. */
int lr_rope_kv_write(void* qkv, int64_t ldqkv, const void* table, int table_is_gathered, const int32_t* pos,
                     void* k_cache, void* v_cache, int B, int S, int Hq, int Hkv, int hd, int Smax, int block_size,
                     int32_t* err, lr_stream_t stream);

/* KVCache.update (utils.py:50-59):  k_cache[b, h, pos[s], :] = k_val[b, h, s, :], likewise v, for b < B, h < H,
 * s < S.  k_val / v_val are [B, H, S, hd] views with element strides (stride_b, stride_h, stride_s) and a dense
 * head dimension; the caches are dense [*, H, Smax, hd].  Positions are read on the device; one outside
 * [0, Smax) writes nothing for that position and sets *err = LR_DEV_POS_RANGE (err may be NULL), where the
 * reference's indexed assignment would raise. */
int lr_kv_update(const void* k_val, const void* v_val, int64_t stride_b, int64_t stride_h, int64_t stride_s,
                 const int32_t* pos, void* k_cache, void* v_cache, int B, int H, int S, int hd, int Smax, int32_t* err,
                 lr_stream_t stream);

/* Bytes of fp32 scratch lr_attn_decode needs for (B, Hq, hd, Smax). */
size_t lr_attn_decode_scratch_bytes(int B, int Hq, int hd, int Smax);

/* One-query attention over the contiguous KV cache (decode, S == 1):
 *   y[b, h*hd : (h+1)*hd] = softmax_j<=pos( q[b,h] . K[b, h/G, j] / sqrt(hd) ) V[b, h/G, j]
 * q [B, Hq*hd] (row stride ldq, already rotated), caches [Bmax, Hkv, Smax, hd], pos int32 [1] on
 * the device, y [B, Hq*hd] (row stride ldy).  Only slots 0..pos are read; the reference reads
 * the whole cache under a mask (repeat_interleave + F.scaled_dot_product_attention,
 * utils.py:252-255, mask gpt_ladder_TP.py:254), which is the same function.  fp32 throughout,
 * one rounding of y.  scratch: lr_attn_decode_scratch_bytes().  The rows of one (sequence, kv
 * head) are addressed with 32-bit byte offsets: Smax * hd * 2 >= 2^31 - 1 is LR_E_UNSUPPORTED. */
int lr_attn_decode(const void* q, int64_t ldq, const void* k_cache, const void* v_cache, const int32_t* pos, void* y,
                   int64_t ldy, int B, int Hq, int Hkv, int hd, int Smax, void* scratch, size_t scratch_bytes,
                   lr_stream_t stream);

/* lr_attn_decode without a scratch argument, for callers that cannot allocate: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.
 * The split-KV partial results go to a fixed device array inside the library
 * (LR_ATTN_DECODE_STATIC_MAX_BYTES = 32 MiB, held by every GPU the library runs on until the
 * process ends); the call allocates nothing and frees nothing.  Same kernels, same results as
 * lr_attn_decode, bit for bit.  Limits: shapes whose lr_attn_decode_scratch_bytes() exceeds the
 * array are refused with LR_E_TOO_LARGE (the 70B rank shard at batch 64 needs 17 MB); all calls on
 * one GPU share the array, so calls that overlap on one GPU (two streams, two threads) race -- run
 * them in stream order.  Nothing in the array has to start at a particular value: every word a
 * call reads it has written itself.  The first call on a device looks up the array's address;
 * make that call outside stream capture (a warm-up step does it). */
#define LR_ATTN_DECODE_STATIC_MAX_BYTES ((size_t)32 << 20)
int lr_attn_decode_static(const void* q, int64_t ldq, const void* k_cache, const void* v_cache, const int32_t* pos,
                          void* y, int64_t ldy, int B, int Hq, int Hkv, int hd, int Smax, lr_stream_t stream);

/* Causal attention of S query tokens per sequence against the cache (prefill, S > 1):
 * query s of row b sits at position pos[s] and sees cache slots j <= pos[s].
 * q [B*S, Hq*hd] (row stride ldq), y [B*S, Hq*hd] (row stride ldy); the caches must already hold
 * this call's keys (lr_rope_kv_write).  Same maths and call sites as lr_attn_decode.  From 16
 * queries per sequence on (hd 64 or 128) the matrix-core kernel runs: Smax * hd * 2 >= 2^31 - 1 or
 * more than 2^24 query blocks ((S / 32) * Hq * B) are LR_E_UNSUPPORTED.  Equal sequences give equal
 * rows, bit for bit. */
int lr_attn_prefill(const void* q, int64_t ldq, const void* k_cache, const void* v_cache, const int32_t* pos, void* y,
                    int64_t ldy, int B, int S, int Hq, int Hkv, int hd, int Smax, lr_stream_t stream);

/* out[b] = argmax_v logits[b, v], lowest index on ties; logits [B, V] bf16 (row stride ldl),
 * out int32 [B].  Greedy stand-in for sample() (benchmark.py:73-77): torch.argmax(logits[:, -1]). */
int lr_argmax(const void* logits, int64_t ldl, int32_t* out, int B, int V, lr_stream_t stream);

/* Measurement aid, no counterpart in the reference: reads `bytes` of device memory at `src` once
 * with every CU streaming (16-byte non-temporal loads, nothing written unless the xor of the data
 * has one particular value, then one word at `sink`).  bench.py times it to report the read rate
 * this machine reaches beside the nominal HBM peak.  bytes >= 32 KiB; the tail beyond a multiple
 * of 32 KiB per workgroup round may be left unread. */
int lr_stream_read(const void* src, size_t bytes, uint32_t* sink, lr_stream_t stream);

/* Device-side bookkeeping between two decode steps, what generate_using_cuda_graphs does on the
 * host between replays (benchmark.py:208-217):
 *     if (history) history[b, pos[0] - pos0] = next_token[b]     (slots outside [0, hist_len) skipped)
 *     cur_token[b] = next_token[b]  for b < B;   pos[0] += 1
 * cur_token / next_token / pos / history may be NULL to skip their part.  history int32
 * [B, ld_hist].  Recorded after a decode step, it makes a captured step self-advancing. */
int lr_advance(int32_t* cur_token, const int32_t* next_token, int32_t* pos, int B, int32_t* history, int64_t ld_hist,
               int hist_len, int pos0, lr_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * One whole decode step of the Ladder model as a single persistent kernel (batch 1 or 2).
 * Replaces, for S == 1, the body of GPTLadder.forward (gpt_ladder_TP.py:252-284: embedding, the
 * n_layer LadderTransformerBlock.forward calls :312-358 with every op inside them, the closing
 * x + prev_attn + prev_mlp, final norm, lm_head) plus the greedy token choice and the
 * between-steps bookkeeping of generate_using_cuda_graphs (benchmark.py:208-217).
 * All sizes in lr_ladder_model_t are THIS RANK's (already divided by the tensor-parallel size). */
typedef struct {
  const void *wqkv, *wo, *w1, *w2, *attention_norm, *ffn_norm; /* bf16 weights of one layer        */
  void *k_cache, *v_cache;                                     /* [Bmax, n_kv_head, smax, head_dim] */
} lr_layer_t;

typedef struct {
  int32_t dim, n_layer, n_head, n_kv_head, head_dim, ffn, out_rows, vocab, smax, block_size;
  float eps;
  int32_t attention_workgroups; /* 0: chosen by the library; > 0: cut the keys into at least this many ranges
                                   (at most 16), one attention workgroup per range and group of kv heads --
                                   part of the workspace layout */
  const void *tok_embeddings, *norm, *output, *freqs_cis; /* [vocab, dim], [dim], [out_rows, dim], table */
  const lr_layer_t* layers_dev;                           /* DEVICE array of n_layer entries            */
} lr_ladder_model_t;

/* Bytes of device workspace the step needs (0: shape not supported by the fused step; callers
 * then use the per-op entry points).  The workspace must be 256-byte aligned, must be
 * initialised once with lr_ladder_step_init before the first step and belongs to one model. */
size_t lr_ladder_step_workspace_bytes(const lr_ladder_model_t* model, int batch);
int lr_ladder_step_init(const lr_ladder_model_t* model, int batch, void* workspace, size_t bytes, lr_stream_t stream);

/* logits[b, :] (bf16, row stride ldl) = model(tokens[b], position pos[0]) and
 * next_token[b] = argmax (lowest index on ties; may be NULL).  K/V of the new position are written
 * to the caches.  If advance != 0 the step also performs, on the device,
 *     history[b, pos[0] - pos0] = next_token[b] (if history),  cur_token[b] = next_token[b] (if
 *     cur_token),  pos[0] += 1,
 * so that replaying the captured step is a complete decode loop.  tokens and cur_token may alias.
 * The kernel occupies every CU (one resident workgroup each) and the workgroups wait for each
 * other's results: nothing else may run on the device concurrently, and two steps must not
 * overlap.  The workspace layout depends on the descriptor (smax, attention_workgroups, ...):
 * size, initialise and step with the same descriptor values.
 * Device-side failures: every wait is bounded, and if one ever expires the int32 workspace word at
 * lr_ladder_step_fail_offset() becomes LR_DEV_WAIT_EXPIRED; a position pos[0] outside
 * [0, min(smax, block_size)) makes it LR_DEV_POS_RANGE and the step computes and writes nothing
 * (the per-op path treats such a position the same way, see lr_rope_kv_write).  Once the word is
 * non-zero the outputs are undefined, later steps on that workspace return at once without
 * computing, and the workspace must be initialised again: callers read the word whenever they
 * synchronise anyway (after a generation, after a timed loop) and raise. */
int lr_ladder_decode_step(const lr_ladder_model_t* model, int batch, const int32_t* tokens, int32_t* pos, void* logits,
                          int64_t ldl, int32_t* next_token, int advance, int32_t* cur_token, int32_t* history,
                          int64_t ld_hist, int hist_len, int pos0, void* workspace, size_t bytes, lr_stream_t stream);
size_t lr_ladder_step_fail_offset(void);

/* How many workgroups of the step kernel the current device can hold at the same time for this descriptor
 * and batch (0: shape not supported, or the runtime cannot tell).  The step launches one workgroup per
 * compute unit and they wait for each other, so lr_ladder_decode_step returns LR_E_LAUNCH unless this is
 * at least the number of compute units.  No counterpart in the reference (its kernels come from a tracing
 * compiler and never wait across workgroups); for callers that want to know before they capture a graph. */
int lr_ladder_step_resident_workgroups(const lr_ladder_model_t* model, int batch);

/* The same step for a weight-only quantised model (every projection of the blocks and the lm_head; the size
 * accounting of gpt_ladder_TP.py:232-237 is the reference's hook for such layers, it ships no quantised layer):
 * wqkv / wo / w1 / w2 of lr_layer_t and `output` each point to a matrix of N * K float8_e4m3fn bytes FOLLOWED
 * IMMEDIATELY by its N bf16 scales (one per output row), and a projection is
 * bf16(bf16(x . w8^T, fp32 sums) * scales) -- what lr_linear_fp8 computes.  Norm gains, embedding table, RoPE
 * table and KV caches stay bf16.  Descriptor, workspace (lr_ladder_step_workspace_bytes / lr_ladder_step_init /
 * lr_ladder_step_fail_offset), arguments and failure reporting are those of lr_ladder_decode_step; in addition
 * dim, ffn and n_head * head_dim must be multiples of 16 and no matrix may reach 2 GiB (LR_E_UNSUPPORTED). */
int lr_ladder_decode_step_fp8(const lr_ladder_model_t* model, int batch, const int32_t* tokens, int32_t* pos,
                              void* logits, int64_t ldl, int32_t* next_token, int advance, int32_t* cur_token,
                              int32_t* history, int64_t ld_hist, int hist_len, int pos0, void* workspace, size_t bytes,
                              lr_stream_t stream);

/* benchmark.py:58-77 (sample, logits_to_probs, multinomial_sample_one_no_sync) on the bf16 logits of
 * the last position, one row per sequence: s = bf16(logits * (1 / max(temperature, 1e-5))); values
 * below the top_k-th largest become -inf (top_k <= 0: no cut; top_k > V: V); probs = bf16 softmax
 * of s (fp32 inside); next_token[b] = argmax_i bf16(probs[i] / noise[i]) (lowest index among equals).
 * `noise` holds the caller's Exp(1) draws (bf16 [B][ldn]; the reference draws them with
 * torch.empty_like(probs).exponential_(1), benchmark.py:59), `probs` is optional (bf16 [B][ldp]). */
int lr_sample_topk(const void* logits, int64_t ldl, const void* noise, int64_t ldn, int B, int V, float temperature,
                   int top_k, void* probs, int64_t ldp, int32_t* next_token, lr_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* LADDER_HIP_H */
