// Row kernel: logits[rows, V] -> log-prob of one target id per row (+ lse, entropy, argmax).
//
// Replaces local_compute_logprobs (mlx-impl/node.py:400-404) and the
// fused_log_softmax + host gather pair (mlx-impl/model.py:16-89, node.py:571,605).  The
// reference reads each row three times and writes a full [rows, V] matrix; here each
// element is read from HBM once with 16-byte loads and only per-row scalars are written.
//
// Grid: rows * splits workgroups of 256 lanes (4 wave64).  A workgroup owns a contiguous
// range of 16-byte load units of one row, every lane keeps an online (max, sum 2^(y-m))
// pair over the units it reads, lanes are merged by DPP / LDS-crossbar exchanges, the four
// waves through LDS.  splits == 1 finishes in the same launch; otherwise per-split
// partials go to the workspace and row_combine_kernel merges them (no float atomics, so
// results do not depend on scheduling).
#include "row_common.hpp"

#include <atomic>
#include <mutex>

namespace tome {

// A launch scores `problems`: problem i reads row i of the logits - or, with a row list, row row_index[i] - and
// owns entry i of targets, row_valid, the outputs and the partials.
struct RowArgs {
  const void* logits;
  const int32_t* row_index;  // nullable: problem -> row of `logits` (a row outside [0, n_rows) scores NaN, argmax -1)
  int64_t n_rows;            // rows the logits matrix holds (only read with a row list)
  const int32_t* targets;
  const int32_t* row_valid;
  float* out_lp;
  float* out_lse;
  float* out_entropy;
  int32_t* out_argmax;
  RowPartial* partials;
  int64_t V;
  int64_t row_stride;
  int splits;
  float scale;  // log2(e) / temperature
};

// Unit index -> first element and element count.  Units below n_units are full vectors;
// units at or above it are the single trailing elements of a row whose V % kVec != 0.
template <typename T, bool VECTOR>
__device__ __forceinline__ int argmax_in_unit(const T* row, int64_t V, int unit, float mx) {
  constexpr int kVec = VECTOR ? Elem<T>::kVec : 1;
  const int64_t n_units = V / kVec;
  // No element above the floor was seen (all -inf / NaN row): report index 0, as a first-max scan would.
  if (unit < 0 || unit >= n_units + (V - n_units * kVec)) return 0;
  int64_t first = (unit < n_units) ? (int64_t)unit * kVec : n_units * kVec + (unit - n_units);
  const int count = (unit < n_units) ? kVec : 1;
  for (int i = 0; i < count; ++i)
    if (Elem<T>::load1(row + first + i) == mx) return (int)(first + i);
  return (int)first;
}

// The target's logit, or NaN when no log-prob is asked for or the id is outside [0, V).  Lane 0 issues
// this at the start of its workgroup, so the dependent load pair (id, then logit) is long finished
// when the row has been streamed.
template <typename T>
__device__ __forceinline__ float load_target_logit(const RowArgs& a, const T* row, int64_t r) {
  if (!a.out_lp || !a.targets) return __builtin_nanf("");
  const int32_t t = a.targets[r];
  return (t >= 0 && t < a.V) ? Elem<T>::load1(row + t) : __builtin_nanf("");
}

template <typename T, bool ENT, bool AMAX>
__device__ __forceinline__ void finish_row(const RowArgs& a, const T* row, int64_t r, const RowStat& st, float x_t) {
  // Called by one lane.  lp = (y_t - m - log2 s) ln2 with the same fma that fed the sum, so
  // the target's own term is part of s and lp <= 0 up to the rounding of the merges.
  const float m = st.mx * a.scale;
  const float log2s = fast_log2(st.s);
  if (a.out_lp) a.out_lp[r] = (fmaf(x_t, a.scale, -m) - log2s) * kLn2;  // NaN in, NaN out
  if (a.out_lse) a.out_lse[r] = (m + log2s) * kLn2;
  if constexpr (ENT) a.out_entropy[r] = (log2s - st.w / st.s) * kLn2;  // w is relative to the maximum: no m here
  if constexpr (AMAX) a.out_argmax[r] = argmax_in_unit<T, true>(row, a.V, st.bi, st.mx);
}

// KEEP: the caller reads the rows again right away (the second pass of the full log-softmax matrix), so they are
// loaded with ordinary loads and stay in the caches; everyone else streams them past the caches.
template <typename T, bool VECTOR, bool ENT, bool AMAX, bool KEEP = false>
__global__ __launch_bounds__(kRowWG) void row_logprob_kernel(RowArgs a) {
  constexpr int kVec = VECTOR ? Elem<T>::kVec : 1;
  __shared__ RowLds lds;
  const int64_t r = blockIdx.x / a.splits;  // problem index
  const int split = blockIdx.x % a.splits;
  const int tid = threadIdx.x;

  if (a.row_valid && a.row_valid[r] == 0) {  // masked row: not read, outputs zeroed
    if (split == 0 && tid == 0) {
      if (a.out_lp) a.out_lp[r] = 0.f;
      if (a.out_lse) a.out_lse[r] = 0.f;
      if (ENT) a.out_entropy[r] = 0.f;
      if (AMAX) a.out_argmax[r] = -1;
    }
    return;
  }
  const int64_t src = a.row_index ? (int64_t)a.row_index[r] : r;  // row of the logits matrix
  if (a.row_index && (uint64_t)src >= (uint64_t)a.n_rows) {        // a list entry that names no row: not read
    if (split == 0 && tid == 0) {
      if (a.out_lp) a.out_lp[r] = __builtin_nanf("");
      if (a.out_lse) a.out_lse[r] = __builtin_nanf("");
      if (ENT) a.out_entropy[r] = __builtin_nanf("");
      if (AMAX) a.out_argmax[r] = -1;
    }
    return;
  }

  const T* row = static_cast<const T*>(a.logits) + src * a.row_stride;
  const int64_t n_units = a.V / kVec;
  const int64_t per_split = (n_units + a.splits - 1) / a.splits;
  const int64_t u0 = per_split * split;
  const int64_t u1 = (u0 + per_split < n_units) ? u0 + per_split : n_units;

  float x_t = 0.f;
  if (tid == 0 && a.splits == 1) x_t = load_target_logit<T>(a, row, r);
  RowStat st = stat_identity();
  if constexpr (VECTOR) {
    const u32x4* p = reinterpret_cast<const u32x4*>(row);
    int64_t u = u0 + tid;
    for (; u + (kRowUnroll - 1) * kRowWG < u1; u += kRowUnroll * kRowWG) {  // several 16-byte loads in flight per lane
      u32x4 v[kRowUnroll];
#pragma unroll
      for (int k = 0; k < kRowUnroll; ++k) v[k] = KEEP ? p[u + k * kRowWG] : __builtin_nontemporal_load(p + u + k * kRowWG);
#pragma unroll
      for (int k = 0; k < kRowUnroll; ++k) {
        float x[kVec];
        Elem<T>::unpack(v[k], x);
        absorb<kVec, ENT, AMAX>(st, x, (int)(u + k * kRowWG), a.scale);
      }
    }
    {  // leftover units of this lane, issued together so their latencies overlap
      u32x4 v[kRowUnroll - 1];
#pragma unroll
      for (int k = 0; k < kRowUnroll - 1; ++k)
        if (u + k * kRowWG < u1) v[k] = KEEP ? p[u + k * kRowWG] : __builtin_nontemporal_load(p + u + k * kRowWG);
#pragma unroll
      for (int k = 0; k < kRowUnroll - 1; ++k)
        if (u + k * kRowWG < u1) {
          float x[kVec];
          Elem<T>::unpack(v[k], x);
          absorb<kVec, ENT, AMAX>(st, x, (int)(u + k * kRowWG), a.scale);
        }
    }
    // Trailing V % kVec elements: one unit each, taken by lane 0 of the last split.
    if (split == a.splits - 1 && tid == 0) {
      for (int64_t e = n_units * kVec; e < a.V; ++e) {
        float x[1] = {Elem<T>::load1(row + e)};
        absorb<1, ENT, AMAX>(st, x, (int)(n_units + (e - n_units * kVec)), a.scale);
      }
    }
  } else {
    for (int64_t u = u0 + tid; u < u1; u += kRowWG) {
      float x[1] = {Elem<T>::load1(row + u)};
      absorb<1, ENT, AMAX>(st, x, (int)u, a.scale);
    }
  }

  const RowStat tot = block_reduce(st, a.scale, lds);
  if (tid != 0) return;
  if (a.splits == 1) {
    if constexpr (VECTOR) {
      finish_row<T, ENT, AMAX>(a, row, r, tot, x_t);
    } else {
      // Scalar path: unit index == element index.
      RowArgs b = a;
      b.out_argmax = nullptr;
      finish_row<T, ENT, false>(b, row, r, tot, x_t);
      if constexpr (AMAX) a.out_argmax[r] = tot.bi < a.V ? tot.bi : 0;
    }
  } else {
    a.partials[r * a.splits + split] = RowPartial{tot.mx, tot.s, tot.w, tot.bi};
  }
}

// One wave per row merges the per-split partials (splits <= 64).
template <typename T, bool VECTOR, bool ENT, bool AMAX>
__global__ __launch_bounds__(64) void row_combine_kernel(RowArgs a) {
  const int64_t r = blockIdx.x;
  if (a.row_valid && a.row_valid[r] == 0) return;  // outputs already zeroed by the main kernel
  const int64_t src = a.row_index ? (int64_t)a.row_index[r] : r;
  if (a.row_index && (uint64_t)src >= (uint64_t)a.n_rows) return;  // outputs already written by the main kernel
  const int lane = threadIdx.x;
  const T* row = static_cast<const T*>(a.logits) + src * a.row_stride;
  float x_t = 0.f;
  if (lane == 0) x_t = load_target_logit<T>(a, row, r);
  RowStat st = stat_identity();
  if (lane < a.splits) {
    const RowPartial p = a.partials[r * a.splits + lane];
    st = RowStat{p.mx, p.s, p.w, p.bi};
  }
  stat_wave_reduce(st, a.scale);
  if (lane != 0) return;
  if constexpr (VECTOR) {
    finish_row<T, ENT, AMAX>(a, row, r, st, x_t);
  } else {
    RowArgs b = a;
    b.out_argmax = nullptr;
    finish_row<T, ENT, false>(b, row, r, st, x_t);
    if constexpr (AMAX) a.out_argmax[r] = st.bi < a.V ? st.bi : 0;
  }
}

template <typename T, bool VECTOR, bool ENT, bool AMAX, bool KEEP = false>
static hipError_t launch_row(const RowArgs& a, int64_t rows, hipStream_t stream, bool skip_combine = false) {
  hipLaunchKernelGGL((row_logprob_kernel<T, VECTOR, ENT, AMAX, KEEP>), dim3((unsigned)(rows * a.splits)),
                     dim3(kRowWG), 0, stream, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || a.splits == 1 || skip_combine) return e;
  hipLaunchKernelGGL((row_combine_kernel<T, VECTOR, ENT, AMAX>), dim3((unsigned)rows), dim3(64), 0,
                     stream, a);
  return hipGetLastError();
}

template <typename T, bool VECTOR>
static hipError_t dispatch_flags(const RowArgs& a, int64_t rows, hipStream_t stream) {
  const bool ent = a.out_entropy != nullptr, amax = a.out_argmax != nullptr;
  if (ent && amax) return launch_row<T, VECTOR, true, true>(a, rows, stream);
  if (ent) return launch_row<T, VECTOR, true, false>(a, rows, stream);
  if (amax) return launch_row<T, VECTOR, false, true>(a, rows, stream);
  return launch_row<T, VECTOR, false, false>(a, rows, stream);
}

// How many workgroups share a row.  From 512 rows on one workgroup per row; smaller batches (decode steps,
// the 64-row CPU-comparison case) are split so that ~2 workgroups per CU are in flight, as long as every
// split keeps a few loads per lane.  Measured: aiming at 512 to 2048 workgroups is equal within 0.5 us for
// 32-256 rows, and 512 spares the 512- and 1024-row batches the combine launch (27.0 against 30.6 us,
// 50.3 against 52.7 us); 3072 and more are slower everywhere.
int row_splits_for(int64_t rows, int64_t V, int vec) {
  const int64_t units = V / vec;
  // Short rows (up to 128 KB) in batches of 256 and more: one workgroup per CU is there already, and the combine launch
  // costs more than the second half of the chip brings (256 rows of 32000: fp32 10.6 against 12.0 us, bf16 7.8 against 9.9).
  if (rows >= 256 && vec > 1 && units <= 8192) return 1;
  const int64_t want_wgs = 512;
  int64_t s = (want_wgs + rows - 1) / rows;
  const int64_t max_by_work = units / (2 * kRowWG);  // >= 2 loads per lane per split
  if (s > max_by_work) s = max_by_work;
  if (s > 64) s = 64;
  if (s < 1) s = 1;
  return (int)s;
}

// `rows` problems.  With `row_index` (device, one entry per problem) problem i reads row row_index[i] of a matrix
// of `n_rows` rows; without it, row i.
hipError_t row_logprob_launch_rows(const void* logits, int dtype, int64_t n_rows, const int32_t* row_index, int64_t rows,
                                   int64_t V, int64_t row_stride, const int32_t* targets, const int32_t* row_valid,
                                   float temperature, float* out_lp, float* out_lse, float* out_entropy,
                                   int32_t* out_argmax, void* workspace, hipStream_t stream) {
  const int esize = dtype == 0 ? 4 : 2;
  const int vec = 16 / esize;
  const bool vector_ok = (reinterpret_cast<uintptr_t>(logits) % 16 == 0) && (row_stride % vec == 0);
  RowArgs a;
  a.logits = logits;
  a.row_index = row_index;
  a.n_rows = n_rows;
  a.targets = targets;
  a.row_valid = row_valid;
  a.out_lp = out_lp;
  a.out_lse = out_lse;
  a.out_entropy = out_entropy;
  a.out_argmax = out_argmax;
  a.partials = static_cast<RowPartial*>(workspace);
  a.V = V;
  a.row_stride = row_stride;
  a.splits = row_splits_for(rows, V, vector_ok ? vec : 1);
  a.scale = kLog2e / temperature;
  if (dtype == 0) {
    return vector_ok ? dispatch_flags<float, true>(a, rows, stream) : dispatch_flags<float, false>(a, rows, stream);
  }
  return vector_ok ? dispatch_flags<uint16_t, true>(a, rows, stream)
                   : dispatch_flags<uint16_t, false>(a, rows, stream);
}

// The rows' logsumexp for a caller that merges split rows itself: only the main kernel is launched.  With
// *splits == 1 out_lse holds the result; otherwise the workspace holds *splits partials per row (RowPartial) and
// out_lse is untouched.
hipError_t row_lse_partials_launch(const void* logits, int dtype, int64_t rows, int64_t V, int64_t row_stride,
                                   float temperature, float* out_lse, void* workspace, int* splits, hipStream_t stream) {
  const int esize = dtype == 0 ? 4 : 2;
  const int vec = 16 / esize;
  const bool vector_ok = (reinterpret_cast<uintptr_t>(logits) % 16 == 0) && (row_stride % vec == 0);
  RowArgs a{};
  a.logits = logits;
  a.n_rows = rows;
  a.out_lse = out_lse;
  a.partials = static_cast<RowPartial*>(workspace);
  a.V = V;
  a.row_stride = row_stride;
  a.splits = row_splits_for(rows, V, vector_ok ? vec : 1);
  a.scale = kLog2e / temperature;
  *splits = a.splits;
  // The caller's second pass reads the matrix again: up to ~3/4 GB it pays to leave the rows in the caches (measured, both
  // passes, fp32 rows of 151936: 64 rows 25.9 -> 24.4 us, 512 rows 155 -> 145, 1024 rows 312 -> 294; 2048 rows 628 -> 648).
  const bool keep = vector_ok && (double)rows * (double)V * esize <= 768.0 * 1024 * 1024;
  if (dtype == 0) {
    if (keep) return launch_row<float, true, false, false, true>(a, rows, stream, true);
    return vector_ok ? launch_row<float, true, false, false>(a, rows, stream, true)
                     : launch_row<float, false, false, false>(a, rows, stream, true);
  }
  if (keep) return launch_row<uint16_t, true, false, false, true>(a, rows, stream, true);
  return vector_ok ? launch_row<uint16_t, true, false, false>(a, rows, stream, true)
                   : launch_row<uint16_t, false, false, false>(a, rows, stream, true);
}

hipError_t row_logprob_launch(const void* logits, int dtype, int64_t rows, int64_t V, int64_t row_stride,
                              const int32_t* targets, const int32_t* row_valid, float temperature,
                              float* out_lp, float* out_lse, float* out_entropy, int32_t* out_argmax,
                              void* workspace, hipStream_t stream) {
  return row_logprob_launch_rows(logits, dtype, rows, nullptr, rows, V, row_stride, targets, row_valid, temperature,
                                 out_lp, out_lse, out_entropy, out_argmax, workspace, stream);
}

// ---- allocation-free variant ---------------------------------------------------------------------
// The per-(row, split) partials of a split launch normally live in a caller-provided workspace.  For
// callers that cannot allocate one (code under graph capture, serving loops with a fixed memory plan)
// the same launches can use this array, which is part of the code object: every GPU the library runs on
// holds its own copy from the first launch until the process ends.  In host code the array's name is
// only a handle for hipGetSymbolAddress; kernels are given the address it returns for the current
// device.  Nothing in it has to start at zero: the combine kernel reads exactly the partials that the
// main kernel of the same call wrote.  All calls on one GPU share the array, so two calls that overlap
// in time on one GPU (different streams) race on it.
constexpr size_t kRowScratchBytes = 64 * 1024;
static __device__ __align__(256) unsigned char scratch[kRowScratchBytes];

constexpr int kMaxDevices = 64;
static std::atomic<void*> g_scratch_ptr[kMaxDevices];  // device address of `scratch`, per device ordinal
static std::mutex g_scratch_mutex;
// Bytes of the array a call may use: the whole array, unless a test lowered it to reach the error path.
static std::atomic<size_t> g_scratch_limit{kRowScratchBytes};

size_t row_scratch_capacity() { return kRowScratchBytes; }
size_t row_scratch_set_limit(size_t bytes) {
  const size_t lim = (bytes == 0 || bytes > kRowScratchBytes) ? kRowScratchBytes : bytes;
  g_scratch_limit.store(lim, std::memory_order_relaxed);
  return lim;
}

// Address of this device's copy of the scratch array; resolved once per device, with that device current.
// After that first call the address is read without taking the lock.
static hipError_t row_scratch_for_current_device(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    p = g_scratch_ptr[dev].load(std::memory_order_relaxed);
    if (!p) {
      e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
      if (e != hipSuccess) return e;
      if (!p) return hipErrorInvalidSymbol;
      g_scratch_ptr[dev].store(p, std::memory_order_release);
    }
  }
  *out = p;
  return hipSuccess;
}

// Bytes of partials a call with these shapes writes (0 when every row is one workgroup).
size_t row_partials_bytes(const void* logits, int dtype, int64_t rows, int64_t V, int64_t row_stride) {
  const int vec = 16 / (dtype == 0 ? 4 : 2);
  const bool vector_ok = (reinterpret_cast<uintptr_t>(logits) % 16 == 0) && (row_stride % vec == 0);
  const int splits = row_splits_for(rows, V, vector_ok ? vec : 1);
  return splits <= 1 ? 0 : (size_t)rows * (size_t)splits * sizeof(RowPartial);
}

// row_logprob_launch with the partials in the library's own scratch array.  `too_big` is set (and nothing
// launched) when the call would need more than the array holds.
hipError_t row_logprob_noalloc_launch(const void* logits, int dtype, int64_t rows, int64_t V, int64_t row_stride,
                                      const int32_t* targets, const int32_t* row_valid, float temperature,
                                      float* out_lp, float* out_lse, float* out_entropy, int32_t* out_argmax,
                                      bool* too_big, hipStream_t stream) {
  *too_big = row_partials_bytes(logits, dtype, rows, V, row_stride) > g_scratch_limit.load(std::memory_order_relaxed);
  if (*too_big) return hipSuccess;
  void* ptr = nullptr;
  const hipError_t e = row_scratch_for_current_device(&ptr);
  if (e != hipSuccess) return e;
  return row_logprob_launch(logits, dtype, rows, V, row_stride, targets, row_valid, temperature, out_lp, out_lse,
                            out_entropy, out_argmax, ptr, stream);
}

}  // namespace tome
