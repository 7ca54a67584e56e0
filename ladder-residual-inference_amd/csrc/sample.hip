// Sampling of the next token from the last position's logits, one workgroup per sequence:
// temperature, top-k cut, softmax, exponential-race draw -- the arithmetic of the reference's
// sample / logits_to_probs / multinomial_sample_one_no_sync (benchmark.py:58-77) on bf16 logits,
// with every intermediate rounded to bf16 where the eager bf16 tensors of the reference round:
//     s_i = bf16(x_i * (1 / max(T, 1e-5)))            (a tensor divided by a host scalar is a
//                                                       multiply by the fp32 reciprocal on the GPU)
//     kth = k-th largest s_i;  s_i < kth  ->  -inf    (torch.topk pivot, benchmark.py:67-70)
//     p_i = bf16(exp(s_i - max s) / sum_j exp(s_j - max s))   (fp32 inside, as softmax on bf16 does)
//     token = argmax_i bf16(p_i / q_i),  q ~ Exp(1)   (lowest index among equals, NaN wins)
// The noise q is an INPUT (bf16, drawn by the caller with the same generator call as the
// reference's torch.empty_like(probs).exponential_(1)), so a run is reproducible against it.
//
// The k-th largest value is found exactly with a two-level radix select on the 16 bits of the
// rounded values (256-bin histograms in LDS): no sort, no tolerance.  The row (<= 256 KiB) is
// walked five times and stays in L2; the kernel is latency-, not bandwidth-bound.
#include "lr_common.h"

namespace {

constexpr int ST = 1024;  // lanes per workgroup

// bf16 bits -> 16-bit key whose unsigned order is the order of the values (-inf lowest)
__device__ __forceinline__ unsigned key_of(u16 b) { return (b & 0x8000u) ? (unsigned)(u16)~b : (unsigned)(b | 0x8000u); }
__device__ __forceinline__ u16 bits_of(unsigned key) { return (key & 0x8000u) ? (u16)(key & 0x7fffu) : (u16)~key; }

__device__ __forceinline__ u16 scaled_bits(const u16* row, int i, float inv_t) { return f_to_bf(bf_to_f(row[i]) * inv_t); }

// From a 256-bin histogram (bin = larger value for larger index): the bin holding the r-th largest
// element (r >= 1) and the rank left inside that bin.  One wave scans; everybody reads the result.
__device__ __forceinline__ void pick_bin(const unsigned* hist, unsigned r, unsigned* out_bin, unsigned* out_rank) {
  if (threadIdx.x == 0) {
    unsigned acc = 0, bin = 0, rank = 1;
    bool found = false;
    for (int b = 255; b >= 0; --b) {
      const unsigned c = hist[b];
      if (!found && acc + c >= r) { bin = (unsigned)b; rank = r - acc; found = true; }
      acc += c;
    }
    *out_bin = bin;
    *out_rank = rank;
  }
}

__global__ __launch_bounds__(ST) void k_sample_topk(const u16* __restrict__ logits, int64_t ldl,
                                                    const u16* __restrict__ noise, int64_t ldn, int V, float inv_t,
                                                    int top_k, u16* __restrict__ probs, int64_t ldp,
                                                    int32_t* __restrict__ out) {
  __shared__ unsigned hist[256];
  __shared__ unsigned s_bin, s_rank;
  __shared__ float s_f[ST / 64];
  __shared__ int s_i[ST / 64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const u16* row = logits + (int64_t)blockIdx.x * ldl;
  const u16* q = noise + (int64_t)blockIdx.x * ldn;

  // ---- pass 1: maximum of the scaled values, histogram of the high byte of their keys
  for (int b = tid; b < 256; b += ST) hist[b] = 0u;
  __syncthreads();
  unsigned kmax = 0u;
  for (int i = tid; i < V; i += ST) {
    const unsigned k = key_of(scaled_bits(row, i, inv_t));
    kmax = k > kmax ? k : kmax;
    atomicAdd(&hist[k >> 8], 1u);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const unsigned ok = (unsigned)__shfl_xor((int)kmax, o, LR_WAVE);
    kmax = ok > kmax ? ok : kmax;
  }
  if (lane == 0) s_i[wave] = (int)kmax;
  __syncthreads();
  kmax = 0u;
  for (int wv = 0; wv < ST / 64; ++wv) kmax = (unsigned)s_i[wv] > kmax ? (unsigned)s_i[wv] : kmax;
  const float vmax = bf_to_f(bits_of(kmax));

  // ---- k-th largest value (exact): high byte, then low byte among the elements of that bin
  unsigned kth_key = 0u;  // keep everything
  if (top_k > 0) {
    const unsigned r = (unsigned)(top_k < V ? top_k : V);
    pick_bin(hist, r, &s_bin, &s_rank);
    __syncthreads();
    const unsigned hi = s_bin, r2 = s_rank;
    __syncthreads();
    for (int b = tid; b < 256; b += ST) hist[b] = 0u;
    __syncthreads();
    for (int i = tid; i < V; i += ST) {
      const unsigned k = key_of(scaled_bits(row, i, inv_t));
      if ((k >> 8) == hi) atomicAdd(&hist[k & 255u], 1u);
    }
    __syncthreads();
    pick_bin(hist, r2, &s_bin, &s_rank);
    __syncthreads();
    kth_key = (hi << 8) | s_bin;
  }
  __syncthreads();

  // ---- pass 3: sum of exp(s - max) over the kept values (fp32)
  float sum = 0.0f;
  for (int i = tid; i < V; i += ST) {
    const u16 sb = scaled_bits(row, i, inv_t);
    if (key_of(sb) >= kth_key) sum += expf(bf_to_f(sb) - vmax);
  }
  sum = wave_sum(sum);
  if (lane == 0) s_f[wave] = sum;
  __syncthreads();
  sum = 0.0f;
  for (int wv = 0; wv < ST / 64; ++wv) sum += s_f[wv];
  __syncthreads();

  // ---- pass 4: probabilities (bf16), race p / q (bf16), argmax
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  bool bnan = false;
  for (int i = tid; i < V; i += ST) {
    const u16 sb = scaled_bits(row, i, inv_t);
    const float pr = key_of(sb) >= kth_key ? round_bf(expf(bf_to_f(sb) - vmax) / sum) : 0.0f;
    if (probs) probs[(int64_t)blockIdx.x * ldp + i] = f_to_bf(pr);
    const float sc = round_bf(pr / bf_to_f(q[i]));
    const bool isn = sc != sc;
    // a NaN beats every number (as in torch's argmax); among equals the lowest index
    if (!bnan && (isn || sc > bv || (sc == bv && i < bi))) { bv = sc; bi = i; bnan = isn; }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, LR_WAVE);
    const int oi = __shfl_xor(bi, o, LR_WAVE);
    const bool on = ov != ov;
    const bool take = bnan ? (on && oi < bi) : (on || ov > bv || (ov == bv && oi < bi));
    if (take) { bv = ov; bi = oi; bnan = on; }
  }
  if (lane == 0) { s_f[wave] = bv; s_i[wave] = bi; }
  __syncthreads();
  if (tid == 0) {
    for (int wv = 1; wv < ST / 64; ++wv) {
      const float ov = s_f[wv];
      const int oi = s_i[wv];
      const bool on = ov != ov;
      const bool take = bnan ? (on && oi < bi) : (on || ov > bv || (ov == bv && oi < bi));
      if (take) { bv = ov; bi = oi; bnan = on; }
    }
    out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
  }
}

}  // namespace

extern "C" int lr_sample_topk(const void* logits, int64_t ldl, const void* noise, int64_t ldn, int B, int V,
                              float temperature, int top_k, void* probs, int64_t ldp, int32_t* next_token,
                              lr_stream_t stream) {
  if (logits == nullptr || noise == nullptr || next_token == nullptr) return LR_E_NULL;
  if (B <= 0 || V <= 0 || ldl < V || ldn < V || (probs != nullptr && ldp < V)) return LR_E_SHAPE;
  const float t = temperature > 1e-5f ? temperature : 1e-5f;
  const float inv_t = 1.0f / t;
  k_sample_topk<<<dim3(B), dim3(ST), 0, (hipStream_t)stream>>>((const u16*)logits, ldl, (const u16*)noise, ldn, V, inv_t,
                                                              top_k, (u16*)probs, ldp, next_token);
  return lr_launch_status();
}
