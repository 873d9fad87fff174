// Decode-step sampler fused onto the logits pass: per row, the top-k logits, one categorical draw
// among them, the log-prob of the drawn token under the FULL softmax, and the greedy token.
//
// Replaces, per decode step, _sample_token (mlx-impl/node.py:894-907: argpartition top-k of
// logits / temperature, mx.random.categorical over them) together with
// fused_log_softmax(...)[b, token] (node.py:590,605 / 356,373) and int(mx.argmax(logits))
// (node.py:602,897) - B host round trips per step in the reference, one launch and one small
// copy here.
//
// The draw is specified without an RNG: the caller passes one uniform u in [0, 1) per row and the
// kernel takes the inverse CDF of softmax(top-k logits / T), the k candidates ordered by logit
// (descending; equal logits by ascending token id).  MLX's own random stream cannot be matched.
//
// One workgroup per row, two passes over the row (the second comes from L2 / MALL for decode-sized
// batches):
//   1. online (max, sum 2^(y-m)) for the full-vocabulary lse, and every lane's own largest element;
//      the k-th largest of the 256 lane maxima is a lower bound `theta` of the k-th largest logit;
//   2. every element >= theta goes to a candidate buffer in LDS (typically k + a few entries).
// Candidates are 64-bit keys (order-preserving image of the float, then ~index), so there are no
// ties and "the top k" is unique.  A buffer overflow (adversarial orderings only) raises theta to
// the k-th largest of what was kept - still a lower bound - and repeats pass 2.  The final k are
// rank-sorted by one wave.
#include "row_common.hpp"

namespace tome {

constexpr int kSampCap = 2048;  // candidate keys per buffer (2 x 16 KB of LDS)
constexpr int kSampMaxK = 32;  // one tightening round is then sure to drop >= 32 of the 64 sampled keys

struct SampleArgs {
  const void* logits;
  const float* uniforms;      // one per row, or nullptr = greedy (candidate 0)
  const int32_t* row_valid;   // nullable
  int32_t* out_token;
  float* out_lp;              // nullable
  float* out_lse;             // nullable
  int32_t* out_argmax;        // nullable
  int32_t* out_topk_idx;      // nullable, [rows, top_k], -1 past the end of a short row
  float* out_topk_logit;      // nullable, [rows, top_k] raw logits
  int64_t V;
  int64_t row_stride;
  int top_k;
  float scale;                // log2(e) / temperature
};

// Order-preserving map float -> uint32 (NaN never gets here: candidates pass a float compare first).
__device__ __forceinline__ uint32_t float_key(float x) {
  const uint32_t u = __float_as_uint(x + 0.0f);  // -0.0 -> +0.0
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_float(uint32_t k) {
  return __uint_as_float((k & 0x80000000u) ? (k ^ 0x80000000u) : ~k);
}
__device__ __forceinline__ uint64_t make_key(float x, uint32_t idx) {
  return ((uint64_t)float_key(x) << 32) | (uint64_t)(0xFFFFFFFFu - idx);  // equal logits: lower id first
}
__device__ __forceinline__ uint32_t key_index(uint64_t k) { return 0xFFFFFFFFu - (uint32_t)k; }

struct SampleLds {
  uint64_t a[kSampCap];
  uint64_t b[kSampCap];
  uint64_t top[kSampMaxK];
  uint64_t thr;
  int cnt;
  RowLds red;
};

// Number of lanes of this wave whose key is larger than this lane's (keys of lanes >= m are ignored).
__device__ __forceinline__ int wave_rank(uint64_t key, int m) {
  int rank = 0;
  for (int j = 0; j < m; ++j) {
    const uint64_t o = __shfl(key, j, 64);
    rank += o > key ? 1 : 0;
  }
  return rank;
}

// Sorted top-k of the m keys in `cur` (m <= kSampCap; 0 = empty slot) into sh.top[0..k), the rest of
// sh.top zeroed; returns the k-th largest key (0 if there are fewer than k).  `cur` / `other` are
// the two LDS buffers; both are clobbered.  All lanes of the workgroup must call it.
__device__ uint64_t select_top_k(SampleLds& sh, uint64_t* cur, uint64_t* other, int m, int k) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  while (m > 64) {
    // Tighten: the k-th largest of 64 entries spread over the buffer is a lower bound of the k-th
    // largest overall, and at least 64 - k entries fall below it.
    if (wave == 0) {
      const uint64_t key = cur[(int)(((int64_t)lane * m) >> 6)];
      const int rank = wave_rank(key, 64);
      if (rank == k - 1) sh.thr = key;  // equal keys (empty slots only) write the same value
      if (lane == 0) sh.cnt = 0;
    }
    __syncthreads();
    const uint64_t thr = sh.thr;
    for (int i = tid; i < m; i += kRowWG) {
      const uint64_t key = cur[i];
      if (key >= thr && key != 0) other[atomicAdd(&sh.cnt, 1)] = key;
    }
    __syncthreads();
    const int kept = sh.cnt;
    __syncthreads();
    if (kept == m) break;  // cannot happen for k <= 32 (see kSampMaxK); guards against an endless loop
    m = kept;
    uint64_t* t = cur;
    cur = other;
    other = t;
  }
  if (m > 64) m = 64;  // unreachable, see above
  if (wave == 0) {
    const uint64_t key = lane < m ? cur[lane] : 0;
    const int rank = wave_rank(key, 64);
    sh.top[lane] = 0;
    __builtin_amdgcn_wave_barrier();
    if (key != 0 && rank < k) sh.top[rank] = key;
  }
  __syncthreads();
  return sh.top[k - 1];
}

template <typename T, bool VECTOR>
__global__ __launch_bounds__(kRowWG) void row_sample_kernel(SampleArgs a) {
  constexpr int kVec = VECTOR ? Elem<T>::kVec : 1;
  __shared__ SampleLds sh;
  const int64_t r = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int k = a.top_k;

  if (a.row_valid && a.row_valid[r] == 0) {  // masked row: not read
    if (tid == 0) {
      a.out_token[r] = -1;
      if (a.out_lp) a.out_lp[r] = 0.f;
      if (a.out_lse) a.out_lse[r] = 0.f;
      if (a.out_argmax) a.out_argmax[r] = -1;
    }
    if (tid < k) {
      if (a.out_topk_idx) a.out_topk_idx[r * k + tid] = -1;
      if (a.out_topk_logit) a.out_topk_logit[r * k + tid] = 0.f;
    }
    return;
  }

  const T* row = static_cast<const T*>(a.logits) + r * a.row_stride;
  const int64_t n_units = a.V / kVec;
  const int n_tail = (int)(a.V - n_units * kVec);  // single elements after the last whole unit (lane 0)

  // ---- pass 1: full-vocabulary statistics and this lane's own maximum --------------------------
  RowStat st = stat_identity();
  if constexpr (VECTOR) {
    const u32x4* p = reinterpret_cast<const u32x4*>(row);
    int64_t u = tid;
    for (; u + (kRowUnroll - 1) * kRowWG < n_units; u += kRowUnroll * kRowWG) {
      u32x4 v[kRowUnroll];
#pragma unroll
      for (int q = 0; q < kRowUnroll; ++q) v[q] = p[u + q * kRowWG];
#pragma unroll
      for (int q = 0; q < kRowUnroll; ++q) {
        float x[kVec];
        Elem<T>::unpack(v[q], x);
        absorb<kVec, false, true>(st, x, (int)(u + q * kRowWG), a.scale);
      }
    }
    for (; u < n_units; u += kRowWG) {
      float x[kVec];
      Elem<T>::unpack(p[u], x);
      absorb<kVec, false, true>(st, x, (int)u, a.scale);
    }
    if (tid == 0) {
      for (int e = 0; e < n_tail; ++e) {
        float x[1] = {Elem<T>::load1(row + n_units * kVec + e)};
        absorb<1, false, true>(st, x, (int)(n_units + e), a.scale);
      }
    }
  } else {
    for (int64_t u = tid; u < n_units; u += kRowWG) {
      float x[1] = {Elem<T>::load1(row + u)};
      absorb<1, false, true>(st, x, (int)u, a.scale);
    }
  }
  // This lane's maximum as a key: the first element of unit st.bi that equals st.mx.
  uint64_t lane_key = 0;
  if (st.bi != 0x7fffffff) {
    const int64_t first = st.bi < n_units ? (int64_t)st.bi * kVec : n_units * kVec + (st.bi - n_units);
    const int count = st.bi < n_units ? kVec : 1;
    int64_t idx = first;
    for (int i = count - 1; i >= 0; --i)
      if (Elem<T>::load1(row + first + i) == st.mx) idx = first + i;
    lane_key = make_key(st.mx, (uint32_t)idx);
  }
  const RowStat tot = block_reduce(st, a.scale, sh.red);  // valid in wave 0

  // ---- theta: k-th largest lane maximum (rows that fit the buffer skip the bound) ----------------
  uint64_t theta = 0;
  if (a.V > kSampCap) {
    sh.a[tid] = lane_key;
    __syncthreads();
    theta = select_top_k(sh, sh.a, sh.b, kRowWG, k);
    __syncthreads();
  }

  // ---- pass 2: collect every element >= theta ---------------------------------------------------
  int m = 0;
  for (;;) {
    if (tid == 0) sh.cnt = 0;
    __syncthreads();
    const float theta_val = theta == 0 ? -INFINITY : key_float((uint32_t)(theta >> 32));
    auto offer = [&](float x, int64_t idx) {
      if (x >= theta_val) {
        const uint64_t key = make_key(x, (uint32_t)idx);
        if (key >= theta) {
          const int pos = atomicAdd(&sh.cnt, 1);
          if (pos < kSampCap) sh.a[pos] = key;
        }
      }
    };
    if constexpr (VECTOR) {
      const u32x4* p = reinterpret_cast<const u32x4*>(row);
      int64_t u = tid;
      for (; u + (kRowUnroll - 1) * kRowWG < n_units; u += kRowUnroll * kRowWG) {
        u32x4 v[kRowUnroll];
#pragma unroll
        for (int q = 0; q < kRowUnroll; ++q) v[q] = p[u + q * kRowWG];
#pragma unroll
        for (int q = 0; q < kRowUnroll; ++q) {
          float x[kVec];
          Elem<T>::unpack(v[q], x);
          if (max_of<kVec>(x) >= theta_val) {
#pragma unroll
            for (int i = 0; i < kVec; ++i) offer(x[i], (u + q * kRowWG) * kVec + i);
          }
        }
      }
      for (; u < n_units; u += kRowWG) {
        float x[kVec];
        Elem<T>::unpack(p[u], x);
        if (max_of<kVec>(x) >= theta_val) {
#pragma unroll
          for (int i = 0; i < kVec; ++i) offer(x[i], u * kVec + i);
        }
      }
      if (tid == 0)
        for (int e = 0; e < n_tail; ++e) offer(Elem<T>::load1(row + n_units * kVec + e), n_units * kVec + e);
    } else {
      for (int64_t u = tid; u < n_units; u += kRowWG) offer(Elem<T>::load1(row + u), u);
    }
    __syncthreads();
    const int offered = sh.cnt;
    __syncthreads();
    if (offered <= kSampCap) {
      m = offered;
      break;
    }
    // Overflow: the k-th largest of the kSampCap keys that were kept is a strictly higher lower bound.
    theta = select_top_k(sh, sh.a, sh.b, kSampCap, k);
    __syncthreads();
  }

  // ---- final selection, draw and outputs (wave 0) -----------------------------------------------
  select_top_k(sh, sh.a, sh.b, m, k);
  if (wave != 0) return;
  const uint64_t key = lane < k ? sh.top[lane] : 0;
  const bool have = key != 0;
  const float x = have ? key_float((uint32_t)(key >> 32)) : -INFINITY;
  const int n_have = __builtin_popcountll(__ballot(have));
  const float x0 = __shfl(x, 0, 64);
  float cdf = have ? fast_exp2((x - x0) * a.scale) : 0.f;  // inclusive scan below
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const float up = __shfl_up(cdf, off, 64);
    if (lane >= off) cdf += up;
  }
  int chosen = 0;
  if (a.uniforms && n_have > 0) {
    const float total = __shfl(cdf, n_have - 1, 64);
    const float target = a.uniforms[r] * total;
    chosen = __builtin_popcountll(__ballot(have && cdf <= target));
    chosen = chosen < n_have ? chosen : n_have - 1;
  }
  const uint64_t ckey = __shfl(key, chosen, 64);
  if (a.out_topk_idx && lane < k) a.out_topk_idx[r * k + lane] = have ? (int32_t)key_index(key) : -1;
  if (a.out_topk_logit && lane < k) a.out_topk_logit[r * k + lane] = have ? x : 0.f;
  if (lane != 0) return;
  const float m2 = tot.mx * a.scale;
  const float log2s = fast_log2(tot.s);
  if (n_have == 0) {  // nothing above -inf in the row
    a.out_token[r] = -1;
    if (a.out_lp) a.out_lp[r] = __builtin_nanf("");
    if (a.out_argmax) a.out_argmax[r] = 0;
  } else {
    a.out_token[r] = (int32_t)key_index(ckey);
    if (a.out_lp) a.out_lp[r] = (fmaf(key_float((uint32_t)(ckey >> 32)), a.scale, -m2) - log2s) * kLn2;
    if (a.out_argmax) a.out_argmax[r] = (int32_t)key_index(key);
  }
  if (a.out_lse) a.out_lse[r] = (m2 + log2s) * kLn2;
}

hipError_t row_sample_launch(const void* logits, int dtype, int64_t rows, int64_t V, int64_t row_stride,
                             const float* uniforms, const int32_t* row_valid, float temperature, int top_k,
                             int32_t* out_token, float* out_lp, float* out_lse, int32_t* out_argmax,
                             int32_t* out_topk_idx, float* out_topk_logit, hipStream_t stream) {
  const int esize = dtype == 0 ? 4 : 2;
  const int vec = 16 / esize;
  const bool vector_ok = (reinterpret_cast<uintptr_t>(logits) % 16 == 0) && (row_stride % vec == 0);
  SampleArgs a{logits, uniforms, row_valid, out_token, out_lp, out_lse, out_argmax, out_topk_idx, out_topk_logit,
               V, row_stride, top_k, kLog2e / temperature};
  const dim3 grid((unsigned)rows), block(kRowWG);
  if (dtype == 0) {
    if (vector_ok) hipLaunchKernelGGL((row_sample_kernel<float, true>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((row_sample_kernel<float, false>), grid, block, 0, stream, a);
  } else {
    if (vector_ok) hipLaunchKernelGGL((row_sample_kernel<uint16_t, true>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((row_sample_kernel<uint16_t, false>), grid, block, 0, stream, a);
  }
  return hipGetLastError();
}

}  // namespace tome
