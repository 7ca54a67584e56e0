// Small HBM/latency-bound ops of the per-rank forward pass: embedding gather, residual add,
// fused residual-add + RMSNorm, SwiGLU, RoPE + KV-cache write, greedy argmax, device-side
// position advance.  All of them move 128 bits per lane and round to bf16 exactly where the eager
// reference materialises a tensor.
#include "lr_common.h"

// ------------------------------------------------------------------------------------ embed
__global__ __launch_bounds__(256) void k_embed(const u16* __restrict__ table, const void* __restrict__ idx,
                                               int idx_is_i64, u16* __restrict__ out, int dim, int vocab) {
  const int64_t t = blockIdx.x;
  const int64_t id = idx_is_i64 ? reinterpret_cast<const int64_t*>(idx)[t]
                                : (int64_t) reinterpret_cast<const int32_t*>(idx)[t];
  const bool ok = id >= 0 && id < vocab;
  const u16* src = table + (ok ? id : 0) * (int64_t)dim;
  u16* dst = out + t * (int64_t)dim;
  for (int c = threadIdx.x * 8; c < dim; c += 256 * 8) {
    uint4 v = ok ? ld16(src + c) : make_uint4(0, 0, 0, 0);
    st16(dst + c, v);
  }
}

extern "C" int lr_embed(const void* table, const void* idx, int idx_is_i64, void* out, int64_t n_tokens, int dim,
                        int vocab, lr_stream_t stream) {
  LR_REQUIRE_PTR(table);
  LR_REQUIRE_PTR(out);
  if (idx == nullptr) return LR_E_NULL;
  if (n_tokens <= 0 || dim <= 0 || vocab <= 0 || n_tokens > 0x7fffffff) return LR_E_SHAPE;
  if (dim % 8) return LR_E_ALIGN;
  k_embed<<<dim3((unsigned)n_tokens), dim3(256), 0, (hipStream_t)stream>>>(
      (const u16*)table, idx, idx_is_i64, (u16*)out, dim, vocab);
  return lr_launch_status();
}

// ------------------------------------------------------------------------------------ add
__global__ __launch_bounds__(256) void k_add(const u16* a, const u16* b, float b_div, u16* out, int64_t n) {
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
  if (i + 8 <= n) {
    float fa[8], fb[8], fo[8];
    unpack8(ld16(a + i), fa);
    unpack8(ld16(b + i), fb);
#pragma unroll
    for (int j = 0; j < 8; ++j) fo[j] = fa[j] + (b_div == 1.0f ? fb[j] : round_bf(fb[j] / b_div));
    st16(out + i, pack8(fo));
  } else {
    for (int64_t j = i; j < n; ++j) {
      float fb = bf_to_f(b[j]);
      out[j] = f_to_bf(bf_to_f(a[j]) + (b_div == 1.0f ? fb : round_bf(fb / b_div)));
    }
  }
}

extern "C" int lr_add(const void* a, const void* b, float b_div, void* out, int64_t n, lr_stream_t stream) {
  LR_REQUIRE_PTR(a);
  LR_REQUIRE_PTR(b);
  LR_REQUIRE_PTR(out);
  if (n <= 0 || !(b_div > 0.0f)) return LR_E_SHAPE;
  const int64_t blocks = (n + 2047) / 2048;
  if (blocks > 0x7fffffff) return LR_E_SHAPE;
  k_add<<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream>>>((const u16*)a, (const u16*)b, b_div, (u16*)out,
                                                                       n);
  return lr_launch_status();
}

// ------------------------------------------------------------------------------------ add + RMSNorm
// One workgroup per row; the updated residual row stays in registers between the two passes.
constexpr int NORM_MAXIT = 8;  // 256 threads x 8 elements x 8 iterations = 16384 columns

__global__ __launch_bounds__(256) void k_add_rmsnorm(const u16* __restrict__ rin, const u16* __restrict__ d1,
                                                     const u16* __restrict__ d2, const u16* __restrict__ gain,
                                                     u16* rout, u16* __restrict__ nout, int dim, float eps) {
  __shared__ float red[4];
  const int tid = threadIdx.x;
  const int64_t base = (int64_t)blockIdx.x * dim;
  // Every load of the row (residual, both addends, gain) is requested before the first one is
  // used: columns past `dim` are clamped to column 0 and ignored, so no branch separates the loads
  // and the kernel costs one memory round trip instead of one per iteration.
  uint4 qr[NORM_MAXIT], q1[NORM_MAXIT], q2[NORM_MAXIT], qg[NORM_MAXIT];
#pragma unroll
  for (int it = 0; it < NORM_MAXIT; ++it) {
    const int c0 = (tid + it * 256) * 8;
    if (it * 256 * 8 >= dim) break;  // uniform
    const int c = c0 < dim ? c0 : 0;
    qr[it] = ld16(rin + base + c);
    q1[it] = d1 ? ld16(d1 + base + c) : make_uint4(0, 0, 0, 0);
    q2[it] = d2 ? ld16(d2 + base + c) : make_uint4(0, 0, 0, 0);
    qg[it] = ld16(gain + c);
  }
  float r[NORM_MAXIT][8];
  float ss = 0.0f;
#pragma unroll
  for (int it = 0; it < NORM_MAXIT; ++it) {
    const int c = (tid + it * 256) * 8;
    if (it * 256 * 8 >= dim) break;
    unpack8(qr[it], r[it]);
    if (d1) {
      float t[8];
      unpack8(q1[it], t);
#pragma unroll
      for (int j = 0; j < 8; ++j) r[it][j] = round_bf(r[it][j] + t[j]);
    }
    if (d2) {
      float t[8];
      unpack8(q2[it], t);
#pragma unroll
      for (int j = 0; j < 8; ++j) r[it][j] = round_bf(r[it][j] + t[j]);
    }
    if (c < dim) {
      if (rout) st16(rout + base + c, pack8(r[it]));
#pragma unroll
      for (int j = 0; j < 8; ++j) ss += r[it][j] * r[it][j];
    }
  }
  ss = wave_sum(ss);
  if ((tid & 63) == 0) red[tid >> 6] = ss;
  __syncthreads();
  ss = (red[0] + red[1]) + (red[2] + red[3]);
  const float inv = rsqrtf(ss / (float)dim + eps);
  // (all results first, in registers of their own, then all stores: a store's data registers cannot be reused
  // before the store has completed, and with one set of them the compiler waits for the previous store in front of
  // every conversion)
  uint4 on[NORM_MAXIT];
#pragma unroll
  for (int it = 0; it < NORM_MAXIT; ++it) {
    if (it * 256 * 8 >= dim) break;
    float g[8], o[8];
    unpack8(qg[it], g);
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = round_bf(r[it][j] * inv) * g[j];
    on[it] = pack8(o);
  }
#pragma unroll
  for (int it = 0; it < NORM_MAXIT; ++it) {
    const int c = (tid + it * 256) * 8;
    if (it * 256 * 8 >= dim) break;
    if (c < dim) st16(nout + base + c, on[it]);
  }
}

extern "C" int lr_add_rmsnorm(const void* resid_in, const void* d1, const void* d2, const void* gain, void* resid_out,
                              void* normed_out, int rows, int dim, float eps, lr_stream_t stream) {
  LR_REQUIRE_PTR(resid_in);
  LR_REQUIRE_PTR(gain);
  LR_REQUIRE_PTR(normed_out);
  LR_OPTIONAL_PTR(d1);
  LR_OPTIONAL_PTR(d2);
  LR_OPTIONAL_PTR(resid_out);
  if (rows <= 0 || dim <= 0) return LR_E_SHAPE;
  if (dim % 8) return LR_E_ALIGN;
  if (dim > 256 * 8 * NORM_MAXIT) return LR_E_UNSUPPORTED;
  k_add_rmsnorm<<<dim3(rows), dim3(256), 0, (hipStream_t)stream>>>((const u16*)resid_in, (const u16*)d1,
                                                                   (const u16*)d2, (const u16*)gain, (u16*)resid_out,
                                                                   (u16*)normed_out, dim, eps);
  return lr_launch_status();
}

// ------------------------------------------------------------------------------------ both norms of a ladder block
// r1 = bf16(r + d1), n1 = norm(r1) * g1;  r2 = bf16(r1 + d2), n2 = norm(r2) * g2;  r <- r2.
// In the ladder schedule the MLP's input does not contain the attention output of the same block, so
// both residual updates and both norms of a block can be done before either module runs.
__global__ __launch_bounds__(256) void k_ladder_norms(const u16* __restrict__ rin, const u16* __restrict__ d1,
                                                      const u16* __restrict__ d2, const u16* __restrict__ g1,
                                                      const u16* __restrict__ g2, u16* rout, u16* __restrict__ n1,
                                                      u16* __restrict__ n2, int dim, float eps) {
  __shared__ float red[8];
  const int tid = threadIdx.x;
  const int64_t base = (int64_t)blockIdx.x * dim;
  uint4 qr[NORM_MAXIT], q1[NORM_MAXIT], q2[NORM_MAXIT], qg1[NORM_MAXIT], qg2[NORM_MAXIT];
#pragma unroll
  for (int it = 0; it < NORM_MAXIT; ++it) {
    const int c0 = (tid + it * 256) * 8;
    if (it * 256 * 8 >= dim) break;  // uniform
    const int c = c0 < dim ? c0 : 0;
    qr[it] = ld16(rin + base + c);
    q1[it] = d1 ? ld16(d1 + base + c) : make_uint4(0, 0, 0, 0);
    q2[it] = d2 ? ld16(d2 + base + c) : make_uint4(0, 0, 0, 0);
    qg1[it] = ld16(g1 + c);
    qg2[it] = ld16(g2 + c);
  }
  float ss1 = 0.0f, ss2 = 0.0f;
#pragma unroll
  for (int it = 0; it < NORM_MAXIT; ++it) {
    const int c = (tid + it * 256) * 8;
    if (it * 256 * 8 >= dim) break;
    float r[8], t[8];
    unpack8(qr[it], r);
    if (d1) {
      unpack8(q1[it], t);
#pragma unroll
      for (int j = 0; j < 8; ++j) r[j] = round_bf(r[j] + t[j]);
    }
    qr[it] = pack8(r);  // r1, exact in bf16
    if (c < dim) {
#pragma unroll
      for (int j = 0; j < 8; ++j) ss1 += r[j] * r[j];
    }
    if (d2) {
      unpack8(q2[it], t);
#pragma unroll
      for (int j = 0; j < 8; ++j) r[j] = round_bf(r[j] + t[j]);
    }
    q2[it] = pack8(r);  // r2
    if (c < dim) {
      st16(rout + base + c, q2[it]);
#pragma unroll
      for (int j = 0; j < 8; ++j) ss2 += r[j] * r[j];
    }
  }
  ss1 = wave_sum(ss1);
  ss2 = wave_sum(ss2);
  if ((tid & 63) == 0) {
    red[tid >> 6] = ss1;
    red[4 + (tid >> 6)] = ss2;
  }
  __syncthreads();
  const float inv1 = rsqrtf(((red[0] + red[1]) + (red[2] + red[3])) / (float)dim + eps);
  const float inv2 = rsqrtf(((red[4] + red[5]) + (red[6] + red[7])) / (float)dim + eps);
  // (all results first, in registers of their own, then all stores: a store's data registers cannot be reused
  // before the store has completed, and with one set of them the compiler waits for the previous stores in front of
  // every conversion)
  uint4 o1[NORM_MAXIT], o2[NORM_MAXIT];
#pragma unroll
  for (int it = 0; it < NORM_MAXIT; ++it) {
    if (it * 256 * 8 >= dim) break;
    float r[8], g[8], o[8];
    unpack8(qr[it], r);
    unpack8(qg1[it], g);
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = round_bf(r[j] * inv1) * g[j];
    o1[it] = pack8(o);
    unpack8(q2[it], r);
    unpack8(qg2[it], g);
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = round_bf(r[j] * inv2) * g[j];
    o2[it] = pack8(o);
  }
#pragma unroll
  for (int it = 0; it < NORM_MAXIT; ++it) {
    const int c = (tid + it * 256) * 8;
    if (it * 256 * 8 >= dim) break;
    if (c < dim) {
      st16(n1 + base + c, o1[it]);
      st16(n2 + base + c, o2[it]);
    }
  }
}

extern "C" int lr_ladder_norms(const void* resid_in, const void* d1, const void* d2, const void* gain1, const void* gain2,
                               void* resid_out, void* normed1, void* normed2, int rows, int dim, float eps,
                               lr_stream_t stream) {
  LR_REQUIRE_PTR(resid_in);
  LR_REQUIRE_PTR(gain1);
  LR_REQUIRE_PTR(gain2);
  LR_REQUIRE_PTR(resid_out);
  LR_REQUIRE_PTR(normed1);
  LR_REQUIRE_PTR(normed2);
  LR_OPTIONAL_PTR(d1);
  LR_OPTIONAL_PTR(d2);
  if (rows <= 0 || dim <= 0) return LR_E_SHAPE;
  if (dim % 8) return LR_E_ALIGN;
  if (dim > 256 * 8 * NORM_MAXIT) return LR_E_UNSUPPORTED;
  k_ladder_norms<<<dim3(rows), dim3(256), 0, (hipStream_t)stream>>>(
      (const u16*)resid_in, (const u16*)d1, (const u16*)d2, (const u16*)gain1, (const u16*)gain2, (u16*)resid_out,
      (u16*)normed1, (u16*)normed2, dim, eps);
  return lr_launch_status();
}

// ------------------------------------------------------------------------------------ SwiGLU
__global__ __launch_bounds__(256) void k_swiglu(const u16* __restrict__ h, int64_t ldh, u16* __restrict__ out, int I) {
  const int row = blockIdx.y;
  const int c = (blockIdx.x * 256 + threadIdx.x) * 8;
  if (c >= I) return;
  float u[8], g[8], o[8];
  unpack8(ld16(h + row * ldh + c), u);
  unpack8(ld16(h + row * ldh + I + c), g);
#pragma unroll
  for (int j = 0; j < 8; ++j) o[j] = swiglu_bf(u[j], g[j]);
  st16(out + (int64_t)row * I + c, pack8(o));
}

extern "C" int lr_swiglu(const void* h, int64_t ldh, void* out, int rows, int I, lr_stream_t stream) {
  LR_REQUIRE_PTR(h);
  LR_REQUIRE_PTR(out);
  if (rows <= 0 || I <= 0 || ldh < 2 * (int64_t)I || rows > 65535 * 64) return LR_E_SHAPE;
  if (I % 8 || ldh % 8) return LR_E_ALIGN;
  // rows ride on grid.y, which is limited to 65535: fold larger row counts into several launches
  const int per = 65535;
  for (int r0 = 0; r0 < rows; r0 += per) {
    const int nr = rows - r0 < per ? rows - r0 : per;
    k_swiglu<<<dim3((I / 8 + 255) / 256, nr), dim3(256), 0, (hipStream_t)stream>>>(
        (const u16*)h + (int64_t)r0 * ldh, ldh, (u16*)out + (int64_t)r0 * I, I);
  }
  return lr_launch_status();
}

// ------------------------------------------------------------------------------------ RoPE + KV write
__global__ __launch_bounds__(256) void k_rope_kv_write(u16* qkv, int64_t ldqkv, const u16* __restrict__ table,
                                                       int table_is_gathered, const int32_t* __restrict__ pos,
                                                       u16* __restrict__ k_cache,
                                                       u16* __restrict__ v_cache, int S, int Hq, int Hkv, int hd,
                                                       int Smax, int block_size, int32_t* err) {
  const int row = blockIdx.x;  // b * S + s
  const int b = row / S, s = row - b * S;
  const int p = pos[s];
  const int trow_idx = table_is_gathered ? s : p;
  if (p < 0 || p >= Smax || trow_idx >= block_size) {
    if (err && threadIdx.x == 0) *err = LR_DEV_POS_RANGE;
    return;
  }
  const int nq = Hq * hd, nkv = Hkv * hd;
  u16* x = qkv + (int64_t)row * ldqkv;
  const u16* trow = table + (int64_t)trow_idx * hd;
  for (int c = threadIdx.x * 8; c < nq + 2 * nkv; c += 256 * 8) {
    uint4 v = ld16(x + c);
    if (c < nq) {
      st16(x + c, rope8(v, ld16(trow + (c % hd))));
    } else if (c < nq + nkv) {
      const int cc = c - nq, h = cc / hd, d = cc - h * hd;
      st16(k_cache + (((int64_t)b * Hkv + h) * Smax + p) * hd + d, rope8(v, ld16(trow + d)));
    } else {
      const int cc = c - nq - nkv, h = cc / hd, d = cc - h * hd;
      st16(v_cache + (((int64_t)b * Hkv + h) * Smax + p) * hd + d, v);
    }
  }
}

extern "C" int lr_rope_kv_write(void* qkv, int64_t ldqkv, const void* table, int table_is_gathered,
                                const int32_t* pos, void* k_cache, void* v_cache, int B, int S, int Hq, int Hkv,
                                int hd, int Smax, int block_size, int32_t* err, lr_stream_t stream) {
  LR_REQUIRE_PTR(qkv);
  LR_REQUIRE_PTR(table);
  LR_REQUIRE_PTR(k_cache);
  LR_REQUIRE_PTR(v_cache);
  if (pos == nullptr) return LR_E_NULL;
  if (B <= 0 || S <= 0 || Hq <= 0 || Hkv <= 0 || hd <= 0 || Smax <= 0 || block_size <= 0) return LR_E_SHAPE;
  if ((int64_t)B * S > 0x7fffffff || ldqkv < (int64_t)(Hq + 2 * Hkv) * hd) return LR_E_SHAPE;
  if (hd % 8 || ldqkv % 8) return LR_E_ALIGN;
  k_rope_kv_write<<<dim3(B * S), dim3(256), 0, (hipStream_t)stream>>>((u16*)qkv, ldqkv, (const u16*)table,
                                                                      table_is_gathered, pos, (u16*)k_cache,
                                                                      (u16*)v_cache, S, Hq, Hkv, hd, Smax, block_size, err);
  return lr_launch_status();
}

// ------------------------------------------------------------------------------------ KVCache.update
// k_cache[b, h, pos[s], :] = k_val[b, h, s, :] (and v), one workgroup per (b, h, s); the values may be a strided view
// (element strides for b, h, s; the head dimension is dense).  Positions come from the device, as everywhere.
__global__ __launch_bounds__(64) void k_kv_update(const u16* __restrict__ kval, const u16* __restrict__ vval,
                                                  int64_t sb, int64_t sh, int64_t ss, const int32_t* __restrict__ pos,
                                                  u16* __restrict__ kc, u16* __restrict__ vc, int H, int S, int hd,
                                                  int Smax, int32_t* err) {
  const int s_ = blockIdx.x % S, h = (blockIdx.x / S) % H, b = blockIdx.x / (S * H);
  const int at = pos[s_];
  if (at < 0 || at >= Smax) {
    if (err && threadIdx.x == 0) *err = LR_DEV_POS_RANGE;
    return;
  }
  const int64_t src = (int64_t)b * sb + (int64_t)h * sh + (int64_t)s_ * ss;
  const int64_t dst = (((int64_t)b * H + h) * Smax + at) * hd;
  for (int c = threadIdx.x * 8; c < hd; c += 64 * 8) {
    st16(kc + dst + c, ld16(kval + src + c));
    st16(vc + dst + c, ld16(vval + src + c));
  }
}

extern "C" int lr_kv_update(const void* k_val, const void* v_val, int64_t stride_b, int64_t stride_h, int64_t stride_s,
                            const int32_t* pos, void* k_cache, void* v_cache, int B, int H, int S, int hd, int Smax,
                            int32_t* err, lr_stream_t stream) {
  LR_REQUIRE_PTR(k_val);
  LR_REQUIRE_PTR(v_val);
  LR_REQUIRE_PTR(k_cache);
  LR_REQUIRE_PTR(v_cache);
  if (pos == nullptr) return LR_E_NULL;
  if (B <= 0 || H <= 0 || S <= 0 || hd <= 0 || Smax <= 0 || (int64_t)B * H * S > 0x7fffffff) return LR_E_SHAPE;
  if (hd % 8 || stride_b % 8 || stride_h % 8 || stride_s % 8) return LR_E_ALIGN;
  k_kv_update<<<dim3((unsigned)(B * H * S)), dim3(64), 0, (hipStream_t)stream>>>(
      (const u16*)k_val, (const u16*)v_val, stride_b, stride_h, stride_s, pos, (u16*)k_cache, (u16*)v_cache, H, S, hd,
      Smax, err);
  return lr_launch_status();
}

// ------------------------------------------------------------------------------------ argmax
// One workgroup of 1024 lanes per row.  (value, index) pairs are merged with "greater value, or
// equal value and lower index", which makes the result independent of the merge order.
__device__ __forceinline__ void amax_merge(float& bv, int& bi, float v, int i) {
  if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
}

__global__ __launch_bounds__(1024) void k_argmax(const u16* __restrict__ logits, int64_t ldl,
                                                 int32_t* __restrict__ out, int V) {
  __shared__ float sv[16];
  __shared__ int si[16];
  const u16* row = logits + (int64_t)blockIdx.x * ldl;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  const int V8 = V & ~7;
  for (int c = threadIdx.x * 8; c < V8; c += 1024 * 8) {
    float f[8];
    unpack8(ld16(row + c), f);
#pragma unroll
    for (int j = 0; j < 8; ++j) amax_merge(bv, bi, f[j], c + j);
  }
  for (int c = V8 + threadIdx.x; c < V; c += 1024) amax_merge(bv, bi, bf_to_f(row[c]), c);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, LR_WAVE);
    const int oi = __shfl_xor(bi, o, LR_WAVE);
    amax_merge(bv, bi, ov, oi);
  }
  if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = bv; si[threadIdx.x >> 6] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 16; ++w) amax_merge(bv, bi, sv[w], si[w]);
    out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
  }
}

extern "C" int lr_argmax(const void* logits, int64_t ldl, int32_t* out, int B, int V, lr_stream_t stream) {
  LR_REQUIRE_PTR(logits);
  if (out == nullptr) return LR_E_NULL;
  if (B <= 0 || V <= 0 || ldl < V) return LR_E_SHAPE;
  if (ldl % 8) return LR_E_ALIGN;
  k_argmax<<<dim3(B), dim3(1024), 0, (hipStream_t)stream>>>((const u16*)logits, ldl, out, V);
  return lr_launch_status();
}

// ------------------------------------------------------------------------------------ advance
__global__ void k_advance(int32_t* cur, const int32_t* next, int32_t* pos, int B, int32_t* history, int64_t ld_hist,
                          int hist_len, int pos0) {
  // single workgroup: every lane reads the position before lane 0 bumps it
  const int i = threadIdx.x;
  const int p = pos ? pos[0] : 0;
  __syncthreads();
  for (int b = i; b < B; b += blockDim.x) {
    if (next && cur) cur[b] = next[b];
    const int slot = p - pos0;
    if (next && history && slot >= 0 && slot < hist_len) history[b * ld_hist + slot] = next[b];
  }
  if (pos && i == 0) pos[0] = p + 1;
}

extern "C" int lr_advance(int32_t* cur_token, const int32_t* next_token, int32_t* pos, int B, int32_t* history,
                          int64_t ld_hist, int hist_len, int pos0, lr_stream_t stream) {
  if (B <= 0 || (history && (ld_hist < hist_len || hist_len <= 0 || pos == nullptr))) return LR_E_SHAPE;
  k_advance<<<dim3(1), dim3(256), 0, (hipStream_t)stream>>>(cur_token, next_token, pos, B, history, ld_hist, hist_len,
                                                            pos0);
  return lr_launch_status();
}

// ------------------------------------------------------------------------------------ misc
extern "C" int lr_version(void) { return 100; }

extern "C" const char* lr_error_string(int code) {
  switch (code) {
    case LR_OK: return "ok";
    case LR_E_NULL: return "a required pointer is NULL";
    case LR_E_ALIGN: return "pointer not 16-byte aligned or stride not a multiple of 8 elements";
    case LR_E_SHAPE: return "non-positive or inconsistent size";
    case LR_E_UNSUPPORTED: return "size not supported by the gfx950 kernels";
    case LR_E_LAUNCH: return "HIP launch failed";
    case LR_E_TOO_LARGE: return "the problem needs more scratch memory than the library's built-in buffer holds";
    default: return "unknown error code";
  }
}

// ------------------------------------------------------------------------------------ stream read
// Plain streaming read of a buffer by the whole chip: 8 workgroups per CU, 8 x 16 bytes in flight
// per lane, consecutive workgroups on consecutive 32 KiB blocks, non-temporal loads.  The rate it
// reaches is the read ceiling of the machine the benchmark runs on, reported beside the nominal
// HBM peak.  The xor of everything read goes to `sink` only if it has one impossible value, so the
// loads cannot be dropped.
__global__ __launch_bounds__(256) void k_stream_read(const u32x4_t* __restrict__ p, size_t n16, unsigned* sink) {
  constexpr int U = 8;
  unsigned acc = 0;
  const size_t stride = (size_t)gridDim.x * 256 * U;
  for (size_t i = (size_t)blockIdx.x * 256 * U + threadIdx.x; i + (U - 1) * 256 < n16; i += stride) {
    u32x4_t v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(p + i + u * 256);
#pragma unroll
    for (int u = 0; u < U; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  if (acc == 0x9e3779b9u) sink[0] = acc;
}

extern "C" int lr_stream_read(const void* src, size_t bytes, uint32_t* sink, lr_stream_t stream) {
  LR_REQUIRE_PTR(src);
  if (sink == nullptr) return LR_E_NULL;
  if (bytes < (size_t)256 * 8 * 16) return LR_E_SHAPE;
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  k_stream_read<<<dim3(cus * 8), dim3(256), 0, (hipStream_t)stream>>>((const u32x4_t*)src, bytes / 16, sink);
  return lr_launch_status();
}
