// Shared device helpers for the gfx950 kernels: wave64 reductions, bf16 unpacking and the
// (max, sum[, weighted sum]) algebra of the online logsumexp.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

namespace tome {

// Host-side "done once per GPU" flag for settings that the runtime keeps per device (hipFuncSetAttribute): a bit per
// device ordinal.  Losing a race repeats the setting, which is harmless.
constexpr int kMaxDeviceOrdinals = 64;
struct DeviceOnce {
  std::atomic<uint64_t> done{0};
  bool first_on_current_device() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDeviceOrdinals) return true;  // cannot tell: set again
    const uint64_t bit = 1ull << dev;
    return (done.fetch_or(bit, std::memory_order_relaxed) & bit) == 0;
  }
};

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
// Floor of the running maximum, as in the reference kernel (mlx-impl/model.py:28).  Keeps
// (m - m_new) finite when a lane has seen nothing yet or only -inf.
constexpr float kMaxFloor = -1e30f;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// Raw v_exp_f32 / v_log_f32: 2^x and log2(x) without the denormal fix-up sequence.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// Plain v_max_f32 / v_max3_f32.  fmaxf() first canonicalises every operand the compiler cannot prove
// quiet (one extra v_max per MFMA result or loaded value); the instructions themselves already return
// the non-NaN operand, which is all the max tracking needs.
__device__ __forceinline__ float raw_max(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
// max(x, kMaxFloor) as one v_med3_f32 (no canonicalisation, and visible to the scheduler).
__device__ __forceinline__ float clamp_below(float x) { return __builtin_amdgcn_fmed3f(x, kMaxFloor, INFINITY); }
__device__ __forceinline__ float raw_max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

__device__ __forceinline__ float bf16_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }

// Round-to-nearest-even float -> bf16 bits (NaN kept quiet).
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

// Two floats -> packed bf16 (lo in bits 0..15), round-to-nearest-even: one v_cvt_pk_bf16_f32 on gfx950.
typedef __bf16 bf16x2_hw __attribute__((ext_vector_type(2)));
typedef float f32x2_hw __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_hw{lo, hi}, bf16x2_hw));
}

// ---- wave64 lane exchange --------------------------------------------------------------
// Steps inside a 16-lane row use DPP (no LDS traffic); the two steps that cross rows go
// through the LDS crossbar (ds_bpermute via __shfl_xor).  After steps 0..3 every lane of a
// row holds that row's reduction, so the mirror patterns pair the right halves.
template <int STEP>
__device__ __forceinline__ float wave_exchange(float v) {
  if constexpr (STEP == 0) {  // quad_perm [1,0,3,2]
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));
  } else if constexpr (STEP == 1) {  // quad_perm [2,3,0,1]
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));
  } else if constexpr (STEP == 2) {  // row_half_mirror
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));
  } else if constexpr (STEP == 3) {  // row_mirror
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true));
  } else if constexpr (STEP == 4) {
    return __shfl_xor(v, 16, 64);
  } else {
    return __shfl_xor(v, 32, 64);
  }
}
template <int STEP>
__device__ __forceinline__ int wave_exchange(int v) {
  return __float_as_int(wave_exchange<STEP>(__int_as_float(v)));
}

// ---- online logsumexp state ------------------------------------------------------------
// All quantities are in log2 units of the scaled logit y = x * (log2(e) / temperature):
//   mx  running maximum of the RAW x seen so far (exact compare for argmax), or kMaxFloor
//   s   sum of 2^(y - m), m = mx * scale
//   w   sum of y * 2^(y - m)          (entropy only)
//   bi  index of the first load unit that attained mx (argmax only)
struct RowStat {
  float mx;
  float s;
  float w;
  int bi;
};

__device__ __forceinline__ RowStat stat_identity() { return RowStat{kMaxFloor, 0.f, 0.f, 0x7fffffff}; }

// Merge b into a.  Ties on mx keep the lower unit index, so the first maximum wins.
// w = sum (y - m) 2^(y - m) is taken RELATIVE to the state's own maximum (y = x * scale, m = mx * scale; every term <= 0):
// moving a state to a larger maximum m' turns it into 2^(m - m') * (w + (m - m') * s).  The entropy then needs no m at
// all - ln 2 * (log2 s - w / s) - where sum y 2^(y - m) would have it cancel against m + log2 s at the logits' magnitude.
__device__ __forceinline__ void stat_merge(RowStat& a, const RowStat& b, float scale) {
  const float mx = fmaxf(a.mx, b.mx);
  const float da = (a.mx - mx) * scale, db = (b.mx - mx) * scale;  // finite: the maxima start at kMaxFloor, not at -inf
  const float fa = fast_exp2(da);
  const float fb = fast_exp2(db);
  const int bi = (b.mx > a.mx || (b.mx == a.mx && b.bi < a.bi)) ? b.bi : a.bi;
  a.w = fmaf(da, a.s, a.w) * fa + fmaf(db, b.s, b.w) * fb;
  a.s = a.s * fa + b.s * fb;
  a.mx = mx;
  a.bi = bi;
}

template <int STEP>
__device__ __forceinline__ void stat_wave_step(RowStat& a, float scale) {
  RowStat b;
  b.mx = wave_exchange<STEP>(a.mx);
  b.s = wave_exchange<STEP>(a.s);
  b.w = wave_exchange<STEP>(a.w);
  b.bi = wave_exchange<STEP>(a.bi);
  stat_merge(a, b, scale);
}

// Full wave64 all-reduce of a RowStat.
__device__ __forceinline__ void stat_wave_reduce(RowStat& a, float scale) {
  stat_wave_step<0>(a, scale);
  stat_wave_step<1>(a, scale);
  stat_wave_step<2>(a, scale);
  stat_wave_step<3>(a, scale);
  stat_wave_step<4>(a, scale);
  stat_wave_step<5>(a, scale);
}

}  // namespace tome
