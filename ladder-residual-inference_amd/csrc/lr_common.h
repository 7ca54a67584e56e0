// Shared device helpers for the gfx950 kernels: bf16 <-> fp32, 128-bit loads, wave64 reductions,
// argument checks.  bf16 is carried as raw 16-bit words; conversions to bf16 round to nearest even
// (v_cvt_pk_bf16_f32 on gfx950).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/ladder_hip.h"

#define LR_WAVE 64

// Weight-only e4m3 projections of a decode step (lr_linear_fp8_multi, lr_attn_decode_beside_fp8): up to this many
// input rows the matrix-vector kernel, above it the matrix-core bands.  Measured on the 70B rank shard, ms per
// step, kernel / bands: 1 row 3.66 / 3.77, 2 rows 4.40 / 3.77, 4 rows 5.22 / 3.96, 8 rows 8.13 / 4.19.
constexpr int LR_FP8_GEMV_MAX_M = 1;

typedef uint16_t u16;
typedef uint32_t u32;
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float bf_lo(u32 p) { return __uint_as_float(p << 16); }
__device__ __forceinline__ float bf_hi(u32 p) { return __uint_as_float(p & 0xffff0000u); }
__device__ __forceinline__ float bf_to_f(u16 v) { return __uint_as_float(((u32)v) << 16); }
__device__ __forceinline__ u16 f_to_bf(float f) {
  __bf16 b = (__bf16)f;
  return __builtin_bit_cast(u16, b);
}
__device__ __forceinline__ u32 pack_bf2(float lo, float hi) { return (u32)f_to_bf(lo) | ((u32)f_to_bf(hi) << 16); }
// round an fp32 value to bf16 and back: the value a bf16 tensor would hold
__device__ __forceinline__ float round_bf(float f) { return bf_to_f(f_to_bf(f)); }

__device__ __forceinline__ uint4 ld16(const void* p) { return *reinterpret_cast<const uint4*>(p); }
// The same through pointers the compiler cannot trace back to a kernel argument (read from a table, chosen between
// two sources): stated to be global memory.  A generic ("flat") access could also target LDS, so it counts as an
// LDS operation as well, may complete out of order, and while one is pending every wait the compiler inserts
// becomes a wait for everything in flight.
// (The cast goes through an integer: a direct generic-to-global pointer cast is a no-op for the optimiser, which
// folds it away and leaves the generic access.)
__device__ __forceinline__ uint4 gld16(const void* p) {
  const u32x4_t v = *(const __attribute__((address_space(1))) u32x4_t*)((unsigned long long)p);
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ u16 gld2(const void* p) {
  return *(const __attribute__((address_space(1))) u16*)((unsigned long long)p);
}
__device__ __forceinline__ void gst4(void* p, u32 v) {
  *(__attribute__((address_space(1))) u32*)((unsigned long long)p) = v;
}
__device__ __forceinline__ void st16(void* p, uint4 v) { *reinterpret_cast<uint4*>(p) = v; }

// 8 bf16 packed in a uint4 -> 8 floats
__device__ __forceinline__ void unpack8(const uint4& v, float* f) {
  f[0] = bf_lo(v.x); f[1] = bf_hi(v.x); f[2] = bf_lo(v.y); f[3] = bf_hi(v.y);
  f[4] = bf_lo(v.z); f[5] = bf_hi(v.z); f[6] = bf_lo(v.w); f[7] = bf_hi(v.w);
}
__device__ __forceinline__ uint4 pack8(const float* f) {
  uint4 v;
  v.x = pack_bf2(f[0], f[1]); v.y = pack_bf2(f[2], f[3]); v.z = pack_bf2(f[4], f[5]); v.w = pack_bf2(f[6], f[7]);
  return v;
}

// RoPE on 8 consecutive elements = 4 interleaved (even, odd) pairs; their (cos, sin) entries are the 8
// consecutive bf16 at table[pos, d/2 .. d/2+3, :].  Products are rounded separately (no FMA
// contraction) to reproduce the element-wise eager evaluation bit for bit.
__device__ __forceinline__ uint4 rope8(const uint4& xv, const uint4& tv) {
#pragma clang fp contract(off)
  float x[8], t[8], o[8];
  unpack8(xv, x);
  unpack8(tv, t);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float c = t[2 * i], s = t[2 * i + 1];
    const float a = x[2 * i] * c;
    const float b = x[2 * i + 1] * s;
    const float d = x[2 * i + 1] * c;
    const float e = x[2 * i] * s;
    o[2 * i] = a - b;
    o[2 * i + 1] = d + e;
  }
  return pack8(o);
}

// Reductions over the 64 lanes of a wave, every lane getting the result.  Call them with all lanes active.
// The 16-lane rows are folded with DPP rotations (vector ALU, no LDS crossbar: a __shfl_xor is a ds_bpermute with
// the latency of an LDS access, six of them in a row for one sum), the four row results meet through scalar registers.
template <int CTRL>
__device__ __forceinline__ float lr_dpp(float v) {
  return __uint_as_float(__builtin_amdgcn_update_dpp(__float_as_uint(v), __float_as_uint(v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float lr_lane(float v, int lane) {
  return __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(v), lane));
}
__device__ __forceinline__ float wave_sum(float v) {
  v += lr_dpp<0x128>(v);  // row_ror:8
  v += lr_dpp<0x124>(v);  // row_ror:4
  v += lr_dpp<0x4e>(v);   // quad_perm [2,3,0,1]
  v += lr_dpp<0xb1>(v);   // quad_perm [1,0,3,2]
  return (lr_lane(v, 0) + lr_lane(v, 16)) + (lr_lane(v, 32) + lr_lane(v, 48));
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, lr_dpp<0x128>(v));
  v = fmaxf(v, lr_dpp<0x124>(v));
  v = fmaxf(v, lr_dpp<0x4e>(v));
  v = fmaxf(v, lr_dpp<0xb1>(v));
  return fmaxf(fmaxf(lr_lane(v, 0), lr_lane(v, 16)), fmaxf(lr_lane(v, 32), lr_lane(v, 48)));
}

// silu in fp32 the way the eager reference evaluates it: x / (1 + exp(-x)), rounded to bf16, then
// multiplied by u and rounded again.
__device__ __forceinline__ float swiglu_bf(float u, float g) {
  float s = round_bf(g / (1.0f + expf(-g)));
  return round_bf(s * u);
}

static inline bool lr_misaligned(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) != 0; }

#define LR_REQUIRE_PTR(p) \
  do {                    \
    if ((p) == nullptr) return LR_E_NULL; \
    if (lr_misaligned(p)) return LR_E_ALIGN; \
  } while (0)
#define LR_OPTIONAL_PTR(p) \
  do {                     \
    if ((p) != nullptr && lr_misaligned(p)) return LR_E_ALIGN; \
  } while (0)

static inline int lr_launch_status() { return hipGetLastError() == hipSuccess ? LR_OK : LR_E_LAUNCH; }

// ---- what the library remembers between calls: facts about a device, looked up once per DEVICE, in atomics (calls
//      from several host threads and on several devices may overlap; two first calls store the same value).
constexpr int LR_MAX_DEVICES = 64;

static inline int lr_current_device() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= LR_MAX_DEVICES) return -1;
  return dev;
}

// compute units of the current device (0: no device)
static inline int lr_num_cus() {
  static std::atomic<int> n[LR_MAX_DEVICES];
  const int dev = lr_current_device();
  if (dev < 0) return 0;
  int v = n[dev].load(std::memory_order_relaxed);
  if (v == 0) {
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) return 0;
    n[dev].store(v, std::memory_order_relaxed);
  }
  return v;
}

// A kernel that needs more than 64 KiB of dynamic LDS has its limit raised once per device.  `done` is a per-kernel
// word (one bit per device) owned by the caller; returns false if the runtime refuses.
static inline bool lr_raise_lds_limit(const void* kernel, size_t bytes, std::atomic<unsigned long long>& done) {
  if (bytes <= 64 * 1024) return true;
  const int dev = lr_current_device();
  if (dev < 0) return false;
  const unsigned long long bit = 1ull << dev;
  if (done.load(std::memory_order_acquire) & bit) return true;
  // the limit is set to all of the CU's LDS: a later call of the same kernel with another size needs no second visit
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess) return false;
  done.fetch_or(bit, std::memory_order_release);
  return true;
}
