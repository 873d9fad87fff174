// Pieces shared by the row kernels (log-prob and sampler): element types, the online
// (max, sum 2^(y-m)) update of one 16-byte load unit, and the workgroup reduction.
#pragma once
#include "common.hpp"

namespace tome {

// 256 lanes per workgroup, four 16-byte loads in flight per lane (8 workgroups = 128 KB in
// flight per CU).  Measured on MI355X at [4096, 151936] bf16: 512/1024-lane workgroups and
// deeper unrolling (fewer, fatter waves) are equal or slower.
constexpr int kRowWG = 256;
constexpr int kRowWaves = kRowWG / 64;
constexpr int kRowUnroll = 4;

template <typename T>
struct Elem;
template <>
struct Elem<float> {
  static constexpr int kVec = 4;
  __device__ static __forceinline__ float load1(const float* p) { return *p; }
  __device__ static __forceinline__ void unpack(const u32x4& v, float (&x)[kVec]) {
    x[0] = __uint_as_float(v.x);
    x[1] = __uint_as_float(v.y);
    x[2] = __uint_as_float(v.z);
    x[3] = __uint_as_float(v.w);
  }
};
template <>
struct Elem<uint16_t> {  // bf16 bit patterns
  static constexpr int kVec = 8;
  __device__ static __forceinline__ float load1(const uint16_t* p) { return bf16_bits_to_f32(*p); }
  __device__ static __forceinline__ void unpack(const u32x4& v, float (&x)[kVec]) {
    x[0] = bf16_lo(v.x);
    x[1] = bf16_hi(v.x);
    x[2] = bf16_lo(v.y);
    x[3] = bf16_hi(v.y);
    x[4] = bf16_lo(v.z);
    x[5] = bf16_hi(v.z);
    x[6] = bf16_lo(v.w);
    x[7] = bf16_hi(v.w);
  }
};

template <int N>
__device__ __forceinline__ float max_of(const float (&x)[N]) {
  float m = x[0];
#pragma unroll
  for (int i = 1; i + 1 < N; i += 2) m = fmaxf(m, fmaxf(x[i], x[i + 1]));  // v_max3_f32
  if constexpr (N % 2 == 0) m = fmaxf(m, x[N - 1]);
  return m;
}
// The same on the plain instructions (no canonicalising v_max per loaded value): for the sampler's scans, which are
// short of instruction issue.  The row kernel keeps max_of: with the entropy and the argmax its fp32 form measured
// 13-23 % slower on this one (64 rows 12.4 -> 14.0 us, 512 rows 47.9 -> 58.9), the statements being opaque to the scheduler.
template <int N>
__device__ __forceinline__ float max_of_raw(const float (&x)[N]) {
  float m = x[0];
#pragma unroll
  for (int i = 1; i + 1 < N; i += 2) m = raw_max3(m, x[i], x[i + 1]);
  if constexpr (N % 2 == 0) m = raw_max(m, x[N - 1]);
  return m;
}

// Fold N values of load unit `unit` into a lane's state; returns the unit's maximum.
template <int N, bool ENT, bool AMAX>
__device__ __forceinline__ float absorb(RowStat& st, const float (&x)[N], int unit, float scale) {
  const float cm = max_of<N>(x);
  const float mx_new = fmaxf(st.mx, cm);
  if constexpr (AMAX) st.bi = (cm > st.mx) ? unit : st.bi;
  const float d = (st.mx - mx_new) * scale;
  const float resc = fast_exp2(d);
  const float m = mx_new * scale;
  float w = ENT ? fmaf(d, st.s, st.w) * resc : 0.f;  // relative to the new maximum (see stat_merge)
  float s = st.s * resc;
#pragma unroll
  for (int i = 0; i < N; ++i) {
    const float t = fmaf(x[i], scale, -m);
    const float e = fast_exp2(t);
    s += e;
    if constexpr (ENT) w = fmaf(clamp_below(t), e, w);  // a -inf logit: floor * 0, not -inf * 0
  }
  st.mx = mx_new;
  st.s = s;
  if constexpr (ENT) st.w = w;
  return cm;
}

// What a workgroup leaves in the workspace when a row is split over several of them: one per (row, split).
struct RowPartial {
  float mx, s, w;
  int bi;
};

// Workgroup reduction of the per-lane states; the result is valid in every lane of wave 0.
// Fields go through LDS one by one: a whole-struct copy to LDS leaves a private stack slot behind.
template <int WAVES>
struct RowLdsT {
  float mx[WAVES], s[WAVES], w[WAVES];
  int bi[WAVES];
};
typedef RowLdsT<kRowWaves> RowLds;

// Workgroup reduction (WAVES waves, at most 64); the result is valid in wave 0 (every lane).
template <int WAVES>
__device__ __forceinline__ RowStat block_reduce(RowStat st, float scale, RowLdsT<WAVES>& lds) {
  stat_wave_reduce(st, scale);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) {
    lds.mx[wave] = st.mx;
    lds.s[wave] = st.s;
    lds.w[wave] = st.w;
    lds.bi[wave] = st.bi;
  }
  __syncthreads();
  RowStat r = stat_identity();
  if (wave == 0) {
    if (lane < WAVES) r = RowStat{lds.mx[lane], lds.s[lane], lds.w[lane], lds.bi[lane]};
    stat_wave_reduce(r, scale);
  }
  return r;
}

}  // namespace tome
