// Second pass of the full log-softmax matrix: out[r, j] = T(x[r, j] * inv_temp) - T(lse_r).
//
// The reference kernel (mlx-impl/model.py:57-65) computes the difference in the I/O dtype T:
// both operands are first cast to T, and for bf16 the result is rounded once more.  The row
// logsumexp comes from row_logprob_kernel, so the matrix is read twice and written once
// where the reference reads it three times.  Rows that row_logprob_kernel split over several
// workgroups are merged here, by every workgroup of the row for itself (a few partials), which
// saves the launch of a merge kernel between the two passes.
//
// bf16 rows of up to 155648 elements do not need the second read either: a 1024-lane workgroup
// holds such a row in its registers (full_log_softmax_onepass_kernel, below).
#include "row_common.hpp"

namespace tome {

constexpr int kFullWG = 256;
constexpr int kFullUnroll = 4;

struct FullArgs {
  const void* in;
  void* out;
  float* row_lse;              // read when splits == 1; written (by the row's first workgroup) otherwise
  const RowPartial* partials;  // [rows, splits] when splits > 1
  int splits;
  float scale;                 // log2(e) / temperature, as the pass that made the partials used it
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

template <bool BF16, bool VECTOR, int UNROLL = kFullUnroll>
__global__ __launch_bounds__(kFullWG) void full_log_softmax_kernel(FullArgs a) {
  const int64_t r = blockIdx.x / a.chunks;
  const int chunk = blockIdx.x % a.chunks;
  float lse;
  if (a.splits > 1) {  // merge the row's partials (at most 64: one per lane of wave 0)
    __shared__ float lse_sh;
    if (threadIdx.x < 64) {
      RowStat st = stat_identity();
      if ((int)threadIdx.x < a.splits) {
        const RowPartial p = a.partials[r * a.splits + threadIdx.x];
        st = RowStat{p.mx, p.s, p.w, p.bi};
      }
      stat_wave_reduce(st, a.scale);
      if (threadIdx.x == 0) {
        lse_sh = (st.mx * a.scale + fast_log2(st.s)) * kLn2;  // as finish_row forms it
        if (chunk == 0) a.row_lse[r] = lse_sh;
      }
    }
    __syncthreads();
    lse = lse_sh;
  } else {
    lse = a.row_lse[r];
  }
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
    for (; u + (UNROLL - 1) * kFullWG < u1; u += UNROLL * kFullWG) {  // several 16-byte loads in flight per lane
      u32x4 v[UNROLL];
#pragma unroll
      for (int q = 0; q < UNROLL; ++q) v[q] = __builtin_nontemporal_load(src + u + q * kFullWG);
#pragma unroll
      for (int q = 0; q < UNROLL; ++q) __builtin_nontemporal_store(convert(v[q]), dst + u + q * kFullWG);
    }
    for (; u < u1; u += kFullWG) __builtin_nontemporal_store(convert(__builtin_nontemporal_load(src + u)), dst + u);
    if (chunk == a.chunks - 1 && threadIdx.x == 0)
      for (int64_t e = n_units * kVec; e < a.V; ++e) scalar_elem(e);
  } else {
    for (int64_t u = u0 + threadIdx.x; u < u1; u += kFullWG) scalar_elem(u);
  }
}

// ---- one pass for bf16 rows that fit a workgroup's registers ----------------------------------------
// A 1024-lane workgroup (one per CU) holds a whole row in registers - up to CH 16-byte units per lane, all requested
// together - and writes T(x * inv_temp) - T(lse) from the same registers: the matrix is read ONCE and written once.
// With a single workgroup on the CU nothing else covers its arithmetic, so every lane keeps a running (maximum, sum) of
// its own and takes in each unit as it arrives (the row kernel's online update) instead of a sweep for the maximum, a
// barrier and a sweep for the sum after the last byte has landed; the lanes' states are merged through one barrier.
template <int CH>
__global__ __launch_bounds__(1024) void full_log_softmax_onepass_kernel(FullArgs a) {
  constexpr int kWaves = 16;
  __shared__ float red_m[kWaves], red_s[kWaves];
  const int64_t r = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint16_t* in_row = static_cast<const uint16_t*>(a.in) + r * a.in_stride;
  uint16_t* out_row = static_cast<uint16_t*>(a.out) + r * a.out_stride;
  const u32x4* src = reinterpret_cast<const u32x4*>(in_row);
  u32x4* dst = reinterpret_cast<u32x4*>(out_row);
  const int n_units = (int)(a.V / 8);
  const int n_tail = (int)(a.V - (int64_t)n_units * 8);  // single elements after the last whole unit: lane 0
  const float scale = a.scale;
  u32x4 v[CH];
#pragma unroll
  for (int q = 0; q < CH; ++q) {  // unconditional (clamped) loads; unit 0 exists (checked on the host)
    const int u = tid + q * 1024;
    v[q] = __builtin_nontemporal_load(src + (u < n_units ? u : 0));
  }
  // the lane's running maximum (floored like every kernel of this path) and sum of 2^((x - maximum) * scale)
  float lm = kMaxFloor, ls = 0.f;
#pragma unroll
  for (int q = 0; q < CH; ++q)
    if (tid + q * 1024 < n_units) {
      float x[8];
      Elem<uint16_t>::unpack(v[q], x);
      const float nm = raw_max3(raw_max3(x[0], x[1], x[2]), raw_max3(x[3], x[4], x[5]), raw_max3(lm, x[6], x[7]));
      const float m = nm * scale;
      float s0 = ls * fast_exp2((lm - nm) * scale), s1 = 0.f;
#pragma unroll
      for (int i = 0; i < 8; i += 2) {
        s0 += fast_exp2(fmaf(x[i], scale, -m));
        s1 += fast_exp2(fmaf(x[i + 1], scale, -m));
      }
      ls = s0 + s1;
      lm = nm;
    }
  if (n_tail != 0 && tid == 0) {  // rare (V not a multiple of 8): fetched here, so that no wait stands in front of the sweep
    for (int e = 0; e < n_tail; ++e) {
      const float x = bf16_bits_to_f32(in_row[(int64_t)n_units * 8 + e]);
      const float nm = fmaxf(lm, x);
      ls = ls * fast_exp2((lm - nm) * scale) + fast_exp2(fmaf(x, scale, -nm * scale));
      lm = nm;
    }
  }
  auto merge = [&](float om, float os) {
    const float nm = fmaxf(lm, om);
    ls = ls * fast_exp2((lm - nm) * scale) + os * fast_exp2((om - nm) * scale);
    lm = nm;
  };
  merge(wave_exchange<0>(lm), wave_exchange<0>(ls));
  merge(wave_exchange<1>(lm), wave_exchange<1>(ls));
  merge(wave_exchange<2>(lm), wave_exchange<2>(ls));
  merge(wave_exchange<3>(lm), wave_exchange<3>(ls));
  merge(wave_exchange<4>(lm), wave_exchange<4>(ls));
  merge(wave_exchange<5>(lm), wave_exchange<5>(ls));
  if (lane == 0) {
    red_m[wave] = lm;
    red_s[wave] = ls;
  }
  __syncthreads();
  float mx = red_m[0];
#pragma unroll
  for (int w = 1; w < kWaves; ++w) mx = fmaxf(mx, red_m[w]);
  float sum = 0.f;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) sum += red_s[w] * fast_exp2((red_m[w] - mx) * scale);
  const float lse = (mx * scale + fast_log2(sum)) * kLn2;
  if (tid == 0) a.row_lse[r] = lse;
  const float lse_t = bf16_rt(lse);
  if (a.inv_temp == 1.0f) {  // the usual call: T(x * 1) is x itself, one rounding and two operations per pair fewer
#pragma unroll
    for (int q = 0; q < CH; ++q) {
      const int u = tid + q * 1024;
      if (u < n_units) {
        u32x4 o;
        o.x = pack_bf16(__fsub_rn(bf16_lo(v[q].x), lse_t), __fsub_rn(bf16_hi(v[q].x), lse_t));
        o.y = pack_bf16(__fsub_rn(bf16_lo(v[q].y), lse_t), __fsub_rn(bf16_hi(v[q].y), lse_t));
        o.z = pack_bf16(__fsub_rn(bf16_lo(v[q].z), lse_t), __fsub_rn(bf16_hi(v[q].z), lse_t));
        o.w = pack_bf16(__fsub_rn(bf16_lo(v[q].w), lse_t), __fsub_rn(bf16_hi(v[q].w), lse_t));
        __builtin_nontemporal_store(o, dst + u);
      }
    }
  } else {
#pragma unroll
    for (int q = 0; q < CH; ++q) {
      const int u = tid + q * 1024;
      if (u < n_units) {
        u32x4 o;
        o.x = sub_pack_bf16(v[q].x, a.inv_temp, lse_t);
        o.y = sub_pack_bf16(v[q].y, a.inv_temp, lse_t);
        o.z = sub_pack_bf16(v[q].z, a.inv_temp, lse_t);
        o.w = sub_pack_bf16(v[q].w, a.inv_temp, lse_t);
        __builtin_nontemporal_store(o, dst + u);
      }
    }
  }
  if (n_tail != 0 && tid == 0)
    for (int e = 0; e < n_tail; ++e) {
      const float x = bf16_bits_to_f32(in_row[(int64_t)n_units * 8 + e]);
      out_row[(int64_t)n_units * 8 + e] = f32_to_bf16_bits(__fsub_rn(bf16_rt(__fmul_rn(x, a.inv_temp)), lse_t));
    }
}

constexpr int kOnePassUnits = 19;  // 16-byte units per lane: 1024 lanes hold 155648 bf16 elements

// Whether the one-pass kernel takes this call: bf16, 16-byte aligned rows, a row that fits the registers of one
// workgroup and is long enough to keep most of its 1024 lanes busy.
// One workgroup per row leaves most of the chip idle on a decode-sized batch, but it is ONE launch where the two-pass form
// is two: rows of up to 40960 elements always come here (16 rows of 16384 / 32000: 4.3 / 5.4 us against 6.8 / 7.9), longer
// ones from V / 3000 rows on.  Measured crossovers: 65536 elements ~24 rows (16 rows 7.5 against 7.0 us, 32 rows 7.5
// against 8.0), 131072 ~60 rows (32 rows 12.1 against 8.7, 64 rows 12.4 against 12.8), 151936 ~44 rows (32 / 48 / 64 rows:
// 13.2 / 13.3 / 13.4 against 11.6 / 14.3 / 16.5); larger batches of 151936: 128 / 512 / 2048 rows 16.9 / 58.4 / 227 against
// 25.4 / 77.5 / 291.
bool full_log_softmax_one_pass(const void* in, const void* out, int dtype, int64_t rows, int64_t V, int64_t in_stride, int64_t out_stride) {
  const bool aligned = reinterpret_cast<uintptr_t>(in) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 &&
                       in_stride % 8 == 0 && out_stride % 8 == 0;
  const bool enough_rows = V <= 40960 || rows * 3000 >= V;
  return dtype == 1 && aligned && enough_rows && V >= 16384 && V / 8 <= (int64_t)kOnePassUnits * 1024;
}

hipError_t full_log_softmax_onepass_launch(const void* in, void* out, int64_t rows, int64_t V, int64_t in_stride,
                                           int64_t out_stride, float temperature, float* row_lse, hipStream_t stream) {
  FullArgs a{};
  a.in = in;
  a.out = out;
  a.row_lse = row_lse;
  a.splits = 1;
  a.scale = kLog2e / temperature;
  a.V = V;
  a.in_stride = in_stride;
  a.out_stride = out_stride;
  a.chunks = 1;
  a.inv_temp = 1.0f / temperature;
  const dim3 grid((unsigned)rows), block(1024);
  if (V / 8 <= 8 * 1024) hipLaunchKernelGGL((full_log_softmax_onepass_kernel<8>), grid, block, 0, stream, a);
  else hipLaunchKernelGGL((full_log_softmax_onepass_kernel<kOnePassUnits>), grid, block, 0, stream, a);
  return hipGetLastError();
}

// Second pass.  `splits` > 1: the rows' partials (RowPartial [rows, splits]) are merged here and the merged lse is
// also written to row_lse; splits == 1: row_lse already holds it.
hipError_t full_log_softmax_launch(const void* in, void* out, int dtype, int64_t rows, int64_t V,
                                   int64_t in_stride, int64_t out_stride, float temperature,
                                   float* row_lse, const void* partials, int splits, hipStream_t stream) {
  const int esize = dtype == 0 ? 4 : 2;
  const int vec = 16 / esize;
  const bool vector_ok = reinterpret_cast<uintptr_t>(in) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 &&
                         in_stride % vec == 0 && out_stride % vec == 0;
  FullArgs a;
  a.in = in;
  a.out = out;
  a.row_lse = row_lse;
  a.partials = static_cast<const RowPartial*>(partials);
  a.splits = splits;
  a.scale = kLog2e / temperature;
  a.V = V;
  a.in_stride = in_stride;
  a.out_stride = out_stride;
  a.inv_temp = 1.0f / temperature;  // the reference multiplies by 1/temp (model.py:27)
  const int64_t units = V / (vector_ok ? vec : 1);
  // Many short workgroups stream a read + write mix best, as long as each still issues a few loads per lane.  bf16
  // rows (a batch too small or rows too long for the one-pass kernel): four loads per lane and pass, aiming at 65536
  // workgroups (against 4096: 4096 x 151936 bf16 655 -> 633 us, both passes included).  fp32 rows: workgroups of ONE pass
  // of two loads per lane - of one load per lane for matrices above 3/4 GB, the size up to which the first pass leaves the
  // rows in the caches (both passes, rows of 151936 fp32, four / two / one load: 64 rows 24.4 / 24.2 / 26.6 us, 1024 rows
  // 296 / 288 / 295, 2048 rows 629 / 618 / 588, 4096 rows 1370 / 1227 / 1168; rows of 32000: 4096 rows - / 248 / 253,
  // 8192 rows - / 503 / 491; rows of 65536: 2048 rows - / 254 / 256, 4096 rows - / 501 / 496).
  int64_t chunks = (65536 + rows - 1) / rows;
  int64_t by_work = units / (kFullUnroll * kFullWG);
  const int f32_unroll = (double)rows * (double)V * 4.0 > 768.0 * 1024 * 1024 ? 1 : 2;
  if (dtype == 0 && vector_ok) {
    chunks = by_work = units / (f32_unroll * kFullWG);
  }
  if (chunks > by_work) chunks = by_work;
  if (chunks < 1) chunks = 1;
  a.chunks = (int)chunks;
  const dim3 grid((unsigned)(rows * chunks)), block(kFullWG);
  if (dtype == 0) {
    if (!vector_ok) hipLaunchKernelGGL((full_log_softmax_kernel<false, false>), grid, block, 0, stream, a);
    else if (f32_unroll == 1) hipLaunchKernelGGL((full_log_softmax_kernel<false, true, 1>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((full_log_softmax_kernel<false, true, 2>), grid, block, 0, stream, a);
  } else {
    if (vector_ok) hipLaunchKernelGGL((full_log_softmax_kernel<true, true>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((full_log_softmax_kernel<true, false>), grid, block, 0, stream, a);
  }
  return hipGetLastError();
}

}  // namespace tome
