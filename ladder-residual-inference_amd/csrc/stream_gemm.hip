// Weight-streaming GEMM for decode batches (up to 64 input rows):  y[m, n] = bf16( sum_k x[m, k] * w[n, k] ).
//
// The weights are read once, in whole cache lines: a load instruction covers 4 weight rows x 256
// contiguous bytes (16 lanes x 16 bytes per row), never a fraction of a line that another
// instruction would have to find in a cache again.  That is the layout a matrix-vector kernel
// streams in, not the one the matrix cores want (there a lane feeds 8 consecutive k of ITS OWN row,
// 16 different rows per instruction), so every chunk takes one trip through a wave-private piece of
// LDS: written row-major as it arrives, read back as v_mfma_f32_16x16x32_bf16 A fragments.  Rows
// are padded by 16 bytes, which puts the 16 rows of a fragment read on 16 different bank groups.
// No workgroup barrier is involved: the LDS unit executes a wave's instructions in order.
//
// A workgroup (4 waves, one per SIMD, so each has the whole register budget) owns a band of up to
// 32 weight rows -- the number of rows is chosen so that every CU gets the same share -- and its
// waves split K in 128-element chunks (wave w takes chunks w, w + 4, ...: together they read 1 KiB
// contiguous per row and round).  Each wave keeps 4 chunks of weights (32 KiB) in flight in
// registers, 128 KiB per CU.  The input rows come from L2 straight into B-fragment layout, one
// chunk ahead.  The waves' partial sums meet in LDS and are added in a fixed order.
//
// Two projections that read the same layer input can share one launch (the band index selects the
// projection), and a projection whose weight holds [up; gate] rows can take the band as row PAIRS
// and store bf16(bf16(silu(g)) * u) instead of u and g.  The fused q/k/v projection of a decode step
// can rotate q and k and put k and v into the cache on its way out (what lr_rope_kv_write does).
#include "stream_band.h"

namespace {

template <int MT, int UNITS, bool W8, bool XL>
__global__ __launch_bounds__(NWV * 64) void k_stream_gemm(const Proj p0, const Proj p1, const int M) {
  extern __shared__ __attribute__((aligned(16))) u16 sg_smem[];
  const bool second = (int)blockIdx.x >= p0.nwg;
  const Proj p = second ? p1 : p0;
  stream_band<MT, UNITS, W8, XL>(p, M, second ? (int)blockIdx.x - p0.nwg : (int)blockIdx.x, sg_smem);
}

template <int MT, int UNITS, bool W8 = false, bool XL = (MT >= XLDS_MIN_MT)>
static int launch_units(Proj& a, Proj& b, int M, hipStream_t s) {
  constexpr size_t lds = stream_band_lds_bytes<MT, UNITS, W8, XL>();
  static std::atomic<unsigned long long> lds_raised{0};
  if (!lr_raise_lds_limit(reinterpret_cast<const void*>(&k_stream_gemm<MT, UNITS, W8, XL>), lds, lds_raised)) return LR_E_LAUNCH;
  k_stream_gemm<MT, UNITS, W8, XL><<<dim3((unsigned)(a.nwg + b.nwg)), dim3(NWV * 64), lds, s>>>(a, b, M);
  return LR_OK;
}

template <int MT>
static int launch(Proj& a, Proj& b, int M, int units, hipStream_t s) {
  if (MT == 16 && M >= XLDS_M16_FROM)  // the 16-row band with its inputs read in whole lines
    return units == 2 ? launch_units<MT, 2, false, true>(a, b, M, s) : launch_units<MT, 1, false, true>(a, b, M, s);
  return units == 2 ? launch_units<MT, 2>(a, b, M, s) : launch_units<MT, 1>(a, b, M, s);
}

// one 16-row unit per workgroup when every CU still gets a band that way; row pairs always take two units
static int pick_units_and_plan(Proj* pr, int n_proj, int M, int ncu) {
  bool any_pair = false, all_thin = true;
  for (int i = 0; i < n_proj; ++i) {
    any_pair = any_pair || pr[i].pair_off != 0;
    if (pr[i].N > 16 * ncu) all_thin = false;
  }
  const int units = (any_pair || !all_thin) ? 2 : 1;
  for (int i = 0; i < n_proj; ++i) plan(pr[i], M, pr[i].pair_off ? 16 : 16 * units, ncu);
  return units;
}

}  // namespace

extern "C" int lr_linear_multi(const lr_projection_t* proj, int n_proj, int M, lr_stream_t stream) {
  if (proj == nullptr) return LR_E_NULL;
  if (n_proj < 1 || n_proj > 2 || M < 1) return LR_E_SHAPE;
  if (M > 64) return LR_E_UNSUPPORTED;
  Proj pr[2] = {};
  for (int i = 0; i < n_proj; ++i) {
    const int rc = sb_fill_projection(proj[i], pr[i]);
    if (rc != LR_OK) return rc;
  }
  const int ncu = lr_num_cus();
  if (ncu < 1) return LR_E_LAUNCH;
  const int units = pick_units_and_plan(pr, n_proj, M, ncu);
  hipStream_t s = (hipStream_t)stream;
  const int rc = M <= 16 ? launch<16>(pr[0], pr[1], M, units, s)
                 : (M <= 32 ? launch<32>(pr[0], pr[1], M, units, s) : launch<64>(pr[0], pr[1], M, units, s));
  return rc != LR_OK ? rc : lr_launch_status();
}

#ifdef LR_BAND_PROFILE
// Profile builds only (not declared in the public header): following launches of this file's kernels record, per
// wave, the six wall-clock stamps of stream_band.h into `device_buffer` (NULL switches it off).  Returns the
// bytes the buffer must hold for the first `workgroups` workgroups of a launch (the others record nothing), or a
// negative error code.
extern "C" long long lr_band_profile(void* device_buffer, int workgroups) {
  if (workgroups < 0) return LR_E_SHAPE;
  unsigned long long* ptr = (unsigned long long*)device_buffer;
  const unsigned wgs = (unsigned)workgroups;
  if (hipMemcpyToSymbol(HIP_SYMBOL(g_band_prof), &ptr, sizeof(ptr)) != hipSuccess ||
      hipMemcpyToSymbol(HIP_SYMBOL(g_band_prof_wgs), &wgs, sizeof(wgs)) != hipSuccess)
    return LR_E_LAUNCH;
  return (long long)workgroups * NWV * 8 * (long long)sizeof(unsigned long long);
}
#endif

// lr_linear_fp8_multi (gemv_fp8.hip) for 3 to 16 input rows: the same bands with e4m3 weights.
namespace lr_detail {
int stream_fp8_multi(const lr_projection_fp8_t* proj, int n_proj, int M, lr_stream_t stream) {
  if (M < 1 || M > 16) return LR_E_UNSUPPORTED;
  Proj pr[2] = {};
  for (int i = 0; i < n_proj; ++i) {
    const int rc = sb_fill_projection_fp8(proj[i], pr[i]);
    if (rc != LR_OK) return rc;
  }
  const int ncu = lr_num_cus();
  if (ncu < 1) return LR_E_LAUNCH;
  const int units = pick_units_and_plan(pr, n_proj, M, ncu);
  hipStream_t s = (hipStream_t)stream;
  const int rc = units == 2 ? launch_units<16, 2, true>(pr[0], pr[1], M, s) : launch_units<16, 1, true>(pr[0], pr[1], M, s);
  return rc != LR_OK ? rc : lr_launch_status();
}
}  // namespace lr_detail
