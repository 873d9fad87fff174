// Second pass of the full log-softmax matrix: out[r, j] = T(x[r, j] * inv_temp) - T(lse_r).
//
// The reference kernel (mlx-impl/model.py:57-65) computes the difference in the I/O dtype T:
// both operands are first cast to T, and for bf16 the result is rounded once more.  The row
// logsumexp comes from row_logprob_kernel, so the matrix is read twice and written once
// where the reference reads it three times.
#include "common.hpp"

namespace tome {

constexpr int kFullWG = 256;
constexpr int kFullUnroll = 4;

struct FullArgs {
  const void* in;
  void* out;
  const float* row_lse;
  int64_t V;
  int64_t in_stride;
  int64_t out_stride;
  int chunks;  // workgroups per row
  float inv_temp;
};

__device__ __forceinline__ float bf16_rt(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }

// Two elements: round the scaled logits to bf16, subtract, round again (v_cvt_pk_bf16_f32 twice; the
// software rounding this replaces cost more VALU time than the memory stream left room for).
__device__ __forceinline__ uint32_t sub_pack_bf16(uint32_t u, float inv_temp, float lse_t) {
  const uint32_t z = pack_bf16(__fmul_rn(bf16_lo(u), inv_temp), __fmul_rn(bf16_hi(u), inv_temp));
  return pack_bf16(__fsub_rn(bf16_lo(z), lse_t), __fsub_rn(bf16_hi(z), lse_t));
}

template <bool BF16, bool VECTOR>
__global__ __launch_bounds__(kFullWG) void full_log_softmax_kernel(FullArgs a) {
  const int64_t r = blockIdx.x / a.chunks;
  const int chunk = blockIdx.x % a.chunks;
  const float lse = a.row_lse[r];
  constexpr int kElem = BF16 ? 2 : 4;
  constexpr int kVec = VECTOR ? 16 / kElem : 1;
  const char* in_row = static_cast<const char*>(a.in) + r * a.in_stride * kElem;
  char* out_row = static_cast<char*>(a.out) + r * a.out_stride * kElem;
  const int64_t n_units = a.V / kVec;
  const int64_t per = (n_units + a.chunks - 1) / a.chunks;
  const int64_t u0 = per * chunk;
  const int64_t u1 = (u0 + per < n_units) ? u0 + per : n_units;
  const float lse_t = BF16 ? bf16_rt(lse) : lse;

  auto scalar_elem = [&](int64_t e) {
    if constexpr (BF16) {
      const uint16_t b = reinterpret_cast<const uint16_t*>(in_row)[e];
      reinterpret_cast<uint16_t*>(out_row)[e] =
          f32_to_bf16_bits(__fsub_rn(bf16_rt(__fmul_rn(bf16_bits_to_f32(b), a.inv_temp)), lse_t));
    } else {
      reinterpret_cast<float*>(out_row)[e] =
          __fsub_rn(__fmul_rn(reinterpret_cast<const float*>(in_row)[e], a.inv_temp), lse_t);
    }
  };

  if constexpr (VECTOR) {
    const u32x4* src = reinterpret_cast<const u32x4*>(in_row);
    u32x4* dst = reinterpret_cast<u32x4*>(out_row);
    auto convert = [&](const u32x4& v) {
      u32x4 o;
      if constexpr (BF16) {
        o.x = sub_pack_bf16(v.x, a.inv_temp, lse_t);
        o.y = sub_pack_bf16(v.y, a.inv_temp, lse_t);
        o.z = sub_pack_bf16(v.z, a.inv_temp, lse_t);
        o.w = sub_pack_bf16(v.w, a.inv_temp, lse_t);
      } else {
        o.x = __float_as_uint(__fsub_rn(__fmul_rn(__uint_as_float(v.x), a.inv_temp), lse_t));
        o.y = __float_as_uint(__fsub_rn(__fmul_rn(__uint_as_float(v.y), a.inv_temp), lse_t));
        o.z = __float_as_uint(__fsub_rn(__fmul_rn(__uint_as_float(v.z), a.inv_temp), lse_t));
        o.w = __float_as_uint(__fsub_rn(__fmul_rn(__uint_as_float(v.w), a.inv_temp), lse_t));
      }
      return o;
    };
    int64_t u = u0 + threadIdx.x;
    for (; u + (kFullUnroll - 1) * kFullWG < u1; u += kFullUnroll * kFullWG) {  // several 16-byte loads in flight per lane
      u32x4 v[kFullUnroll];
#pragma unroll
      for (int q = 0; q < kFullUnroll; ++q) v[q] = __builtin_nontemporal_load(src + u + q * kFullWG);
#pragma unroll
      for (int q = 0; q < kFullUnroll; ++q) __builtin_nontemporal_store(convert(v[q]), dst + u + q * kFullWG);
    }
    for (; u < u1; u += kFullWG) __builtin_nontemporal_store(convert(src[u]), dst + u);
    if (chunk == a.chunks - 1 && threadIdx.x == 0)
      for (int64_t e = n_units * kVec; e < a.V; ++e) scalar_elem(e);
  } else {
    for (int64_t u = u0 + threadIdx.x; u < u1; u += kFullWG) scalar_elem(u);
  }
}

hipError_t full_log_softmax_launch(const void* in, void* out, int dtype, int64_t rows, int64_t V,
                                   int64_t in_stride, int64_t out_stride, float temperature,
                                   const float* row_lse, hipStream_t stream) {
  const int esize = dtype == 0 ? 4 : 2;
  const int vec = 16 / esize;
  const bool vector_ok = reinterpret_cast<uintptr_t>(in) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 &&
                         in_stride % vec == 0 && out_stride % vec == 0;
  FullArgs a;
  a.in = in;
  a.out = out;
  a.row_lse = row_lse;
  a.V = V;
  a.in_stride = in_stride;
  a.out_stride = out_stride;
  a.inv_temp = 1.0f / temperature;  // the reference multiplies by 1/temp (model.py:27)
  const int64_t units = V / (vector_ok ? vec : 1);
  // Many short workgroups stream a read + write mix best (measured: aiming at 65536 workgroups instead of 4096
  // takes 512 x 151936 fp32 from 165 to 150 us and 4096 x 151936 bf16 from 655 to 633 us, both passes included),
  // as long as each still issues its four loads per lane.
  int64_t chunks = (65536 + rows - 1) / rows;
  const int64_t by_work = units / (kFullUnroll * kFullWG);
  if (chunks > by_work) chunks = by_work;
  if (chunks < 1) chunks = 1;
  a.chunks = (int)chunks;
  const dim3 grid((unsigned)(rows * chunks)), block(kFullWG);
  if (dtype == 0) {
    if (vector_ok) hipLaunchKernelGGL((full_log_softmax_kernel<false, true>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((full_log_softmax_kernel<false, false>), grid, block, 0, stream, a);
  } else {
    if (vector_ok) hipLaunchKernelGGL((full_log_softmax_kernel<true, true>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((full_log_softmax_kernel<true, false>), grid, block, 0, stream, a);
  }
  return hipGetLastError();
}

}  // namespace tome
