// Decode attention and one weight-streaming projection in ONE launch.
//
// In a ladder block the MLP's input does not contain the block's own attention output, so the
// attention over the KV cache and the up/gate projection of the same block are independent.  The
// attention of a decode step is a latency chain (a few hundred workgroups that each wait for one
// memory round trip and then do a little arithmetic); the projection is pure streaming.  Launched
// one after the other, the chip idles through the first and the second cannot start; launched as
// one grid -- the first workgroups are attention items, the rest are bands of the projection --
// two workgroups share a CU and the attention disappears behind the weight stream.
//
// Both halves are the device functions their own kernels use (attn_partial_item, stream_band), so
// the results are bit-identical to lr_attn_decode followed by lr_linear_multi.  The merge of the
// attention's chunks stays a launch of its own: done inside this one by whoever stores the last
// chunk of a kv head (chunk results written through to the memory side, one ticket per kv head),
// it became the tail of the grid instead of hiding in it (0.4 ms per step slower at batch 8 and 16).
//
// lr_attn_decode_beside_fp8: the same grid with the e4m3 variant of the band (weight-only quantised models,
// 2 to 16 rows).
#include "attn_decode_item.h"
#include "stream_band.h"

namespace {

struct AttnItems {
  const u16* q;
  int64_t ldq;
  const u16* kc;
  const u16* vc;
  const int32_t* pos;
  float* o_part;
  float* ml_part;
  int Hkv, Smax, nsplit, chunk_max;  // Hkv: groups of G q heads (kv_share of them per head of the cache)
  int kv_share;
  int n_items;  // nsplit * Hkv * B: the first workgroups of the grid
};

constexpr int PAIR_MT = 16, PAIR_UNITS = 2;

// EAGER: how an attention item requests its rows (see attn_partial_item): all at once for long chunks
template <int HD, int G, bool W8, bool XL, bool EAGER>
__global__ __launch_bounds__(256) void k_attn_beside_band(const AttnItems a, const Proj p, const int M) {
  extern __shared__ __attribute__((aligned(16))) unsigned char pair_smem[];
  const int wg = blockIdx.x;
  if (wg < a.n_items) {
    const int split = wg % a.nsplit, rest = wg / a.nsplit;
    attn_partial_item<HD, G, EAGER>(a.q, a.ldq, a.kc, a.vc, a.pos, a.o_part, a.ml_part, a.Hkv, a.Smax, a.nsplit,
                             a.chunk_max, split, rest % a.Hkv, rest / a.Hkv, reinterpret_cast<float*>(pair_smem),
                             a.kv_share);
  } else {
    stream_band<PAIR_MT, PAIR_UNITS, W8, XL>(p, M, wg - a.n_items, reinterpret_cast<u16*>(pair_smem));
  }
}

template <int HD, int G, bool W8, bool XL, bool EAGER>
static int launch_pair_as(const AttnItems& a, const Proj& p, int M, u16* y, int64_t ldy, int B, hipStream_t s) {
  const int Hq = a.Hkv * G;
  const size_t lds_att = (size_t)attn_item_lds_floats<HD, G>(a.chunk_max) * sizeof(float);
  const size_t lds_band = stream_band_lds_bytes<PAIR_MT, PAIR_UNITS, W8, XL>();
  const size_t lds = lds_att > lds_band ? lds_att : lds_band;
  static std::atomic<unsigned long long> lds_raised{0};
  if (!lr_raise_lds_limit(reinterpret_cast<const void*>(&k_attn_beside_band<HD, G, W8, XL, EAGER>), lds, lds_raised)) return LR_E_LAUNCH;
  k_attn_beside_band<HD, G, W8, XL, EAGER><<<dim3((unsigned)(a.n_items + p.nwg)), dim3(256), lds, s>>>(a, p, M);
  launch_attn_combine<HD>(a.o_part, a.ml_part, y, ldy, Hq, B, a.nsplit, s);
  return lr_launch_status();
}

// (the band's inputs in whole lines or in fragment layout: the choice lr_linear_multi makes for the same rows)
template <int HD, int G, bool W8>
static int launch_pair(const AttnItems& a, const Proj& p, int M, u16* y, int64_t ldy, int B, hipStream_t s) {
  const bool eager = a.chunk_max > 128;  // more than half of a wave's four key tiles in use
  if (!W8 && M >= XLDS_M16_FROM)
    return eager ? launch_pair_as<HD, G, false, true, true>(a, p, M, y, ldy, B, s)
                 : launch_pair_as<HD, G, false, true, false>(a, p, M, y, ldy, B, s);
  return eager ? launch_pair_as<HD, G, W8, false, true>(a, p, M, y, ldy, B, s)
               : launch_pair_as<HD, G, W8, false, false>(a, p, M, y, ldy, B, s);
}

// shared body of the two entry points; `fill` turns the caller's projection into a Proj
template <bool W8, class Projection, class Fill>
static int beside(const void* q, int64_t ldq, const void* k_cache, const void* v_cache, const int32_t* pos, void* y,
                  int64_t ldy, int B, int Hq, int Hkv, int hd, int Smax, void* scratch, size_t scratch_bytes,
                  const Projection* proj, int M, int m_min, lr_stream_t stream, Fill fill) {
  LR_REQUIRE_PTR(q);
  LR_REQUIRE_PTR(k_cache);
  LR_REQUIRE_PTR(v_cache);
  LR_REQUIRE_PTR(y);
  LR_REQUIRE_PTR(scratch);
  if (pos == nullptr || proj == nullptr) return LR_E_NULL;
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || hd <= 0 || Smax <= 0 || Hq % Hkv || M < 1) return LR_E_SHAPE;
  if ((int64_t)Smax * hd * 2 >= 0x7fffffff) return LR_E_UNSUPPORTED;  // the rows of one (sequence, head) are addressed with 32-bit offsets
  if (ldq < (int64_t)Hq * hd || ldy < (int64_t)Hq * hd || B > 65535) return LR_E_SHAPE;
  if (ldq % 8 || ldy % 8) return LR_E_ALIGN;
  if (scratch_bytes < lr_attn_decode_scratch_bytes(B, Hq, hd, Smax)) return LR_E_SHAPE;
  // the projection must not touch the cache the attention reads, and only the 16-row band shares a CU
  if (proj->epilogue == LR_EPI_ROPE_KV || M > PAIR_MT || M < m_min) return LR_E_UNSUPPORTED;
  Proj p;
  const int rc = fill(*proj, p);
  if (rc != LR_OK) return rc;
  int G = Hq / Hkv;
  AttnItems a;
  a.kv_share = 1;
  a.q = (const u16*)q; a.ldq = ldq; a.kc = (const u16*)k_cache; a.vc = (const u16*)v_cache; a.pos = pos;
  a.Smax = Smax;
  a.nsplit = attn_pick_nsplit(B, Hkv, Smax);  // the chunks of lr_attn_decode
  if (G == 16) {
    // 16 q heads per kv head need the whole register file (one workgroup per CU): two groups of 8 instead
    G = 8;
    a.kv_share = 2;
  }
  a.Hkv = Hkv * a.kv_share;
  a.chunk_max = ((Smax + a.nsplit - 1) / a.nsplit + 3) & ~3;
  a.o_part = (float*)scratch;
  a.ml_part = a.o_part + (size_t)B * Hq * a.nsplit * hd;
  if ((int64_t)a.nsplit * a.Hkv * B > 0x3fffffff) return LR_E_UNSUPPORTED;
  a.n_items = a.nsplit * a.Hkv * B;
  if (!((hd == 128 || hd == 64) && (G == 1 || G == 2 || G == 4 || G == 8))) return LR_E_UNSUPPORTED;
  const int ncu = lr_num_cus();
  if (ncu < 1) return LR_E_LAUNCH;
  plan(p, M, p.pair_off ? 16 : 16 * PAIR_UNITS, ncu);
  hipStream_t s = (hipStream_t)stream;
#define LR_PAIR(HDV, GV) \
  if (hd == HDV && G == GV) return launch_pair<HDV, GV, W8>(a, p, M, (u16*)y, ldy, B, s);
  LR_PAIR(128, 1) LR_PAIR(128, 2) LR_PAIR(128, 4) LR_PAIR(128, 8)
  LR_PAIR(64, 1) LR_PAIR(64, 2) LR_PAIR(64, 4) LR_PAIR(64, 8)
#undef LR_PAIR
  return LR_E_UNSUPPORTED;
}

}  // namespace

extern "C" int lr_attn_decode_beside(const void* q, int64_t ldq, const void* k_cache, const void* v_cache,
                                     const int32_t* pos, void* y, int64_t ldy, int B, int Hq, int Hkv, int hd,
                                     int Smax, void* scratch, size_t scratch_bytes, const lr_projection_t* proj,
                                     int M, lr_stream_t stream) {
  return beside<false>(q, ldq, k_cache, v_cache, pos, y, ldy, B, Hq, Hkv, hd, Smax, scratch, scratch_bytes, proj, M, 1,
                       stream, sb_fill_projection);
}

// (for one row lr_linear_fp8_multi uses the matrix-vector kernel, which has no band to put beside the attention)
extern "C" int lr_attn_decode_beside_fp8(const void* q, int64_t ldq, const void* k_cache, const void* v_cache,
                                         const int32_t* pos, void* y, int64_t ldy, int B, int Hq, int Hkv, int hd,
                                         int Smax, void* scratch, size_t scratch_bytes,
                                         const lr_projection_fp8_t* proj, int M, lr_stream_t stream) {
  return beside<true>(q, ldq, k_cache, v_cache, pos, y, ldy, B, Hq, Hkv, hd, Smax, scratch, scratch_bytes, proj, M,
                      LR_FP8_GEMV_MAX_M + 1, stream, sb_fill_projection_fp8);
}
