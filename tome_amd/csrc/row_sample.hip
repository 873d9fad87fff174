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
// A row is shared by `splits` workgroups (decode batches are a few dozen rows: one workgroup per row
// would leave most of the chip idle).  Each computes, over its range of the row,
//   * the online (max, sum 2^(y-m)) for the full-vocabulary lse and every lane's own largest element;
//   * a lower bound `theta` of the k-th largest logit: the k-th largest of the lane maxima (four waves,
//     each extracting its ceil(k/4) largest);
//   * every element >= theta, as a candidate in an LDS buffer (typically k + a few entries).
// Short ranges (a lane owns <= 8 load units) are loaded once and kept in registers for the candidate
// scan.  Long ranges are streamed once: theta comes from the lanes' first units, is renewed after a
// quarter of the range, and candidates are collected as the row goes by; only when the buffer overflows
// is the range scanned a second time with the bound from all of it.
// Candidates are 64-bit keys (order-preserving image of the float, then ~index), so there are no
// ties and "the top k" is unique.  A buffer overflow (adversarial orderings only) raises theta to
// the k-th largest of what was kept - still a lower bound - and rescans.  The final k are ranked by
// counting.  With splits > 1 every workgroup leaves its k keys and its (max, sum) in the workspace
// and row_sample_combine_kernel selects among the splits * k keys and draws.
#include "row_common.hpp"

namespace tome {

constexpr int kSampCap = 1024;      // candidate keys per buffer in the main kernel (2 x 8 KB of LDS: 8 workgroups per CU)
constexpr int kSampMergeCap = 2048; // in the combine kernel: up to 64 splits x 32 keys
constexpr int kSampCached = 8;      // a lane keeps up to this many load units in registers between the passes
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
  uint64_t* part_keys;        // workspace: [rows, splits, top_k] (splits > 1)
  float2* part_stat;          // workspace: [rows, splits] (max, sum)
  int64_t V;
  int64_t row_stride;
  int top_k;
  int splits;
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

template <int CAP>
struct SampleLds {
  uint64_t a[CAP];
  uint64_t b[CAP];
  uint64_t top[kSampMaxK];
  uint64_t thr4[kRowWaves];
  int cnt;
  int wave_cnt[kRowWaves];
  RowLds red;
};

// Wave-cooperative collection without atomics: every wave owns a quarter of a key buffer and a running count that is
// the same in all its lanes; the lanes that pass take consecutive slots by their position among the passing lanes.
// An LDS atomic that returns the slot costs a round trip per candidate, and those trips queue up behind each other.
constexpr int kSampWaveCap = kSampCap / kRowWaves;
struct WaveCollector {
  uint64_t* region;
  int cap;
  int count;  // wave-uniform; keeps counting past `cap` (overflow is detected from it), nothing is stored there
  // Must be reached by all lanes of the wave together.
  __device__ __forceinline__ void offer(bool pass, uint64_t key) {
    const uint64_t b = __ballot(pass);
    if (b == 0) return;
    const int pos = count + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(b >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)b, 0u));
    if (pass && pos < cap) region[pos] = key;
    count += __builtin_popcountll(b);
  }
};

// Keys of four wave regions (counts c[w], region w starting at base + w * stride) as one list: entry i.
__device__ __forceinline__ uint64_t region_entry(const uint64_t* base, int stride, const int* c, int i) {
  int w = 0;
#pragma unroll
  for (int q = 0; q < kRowWaves - 1; ++q)
    if (w == q && i >= c[q]) {
      i -= c[q];
      w = q + 1;
    }
  return base[w * stride + i];
}

// One wave sorts up to 64 keys held one per lane (0 = none; m = number of lanes that may hold one): returns in lane i
// the (i+1)-th largest key for i < k, 0 elsewhere.  Register traffic only (v_readlane broadcasts, one ds_permute pair).
__device__ __forceinline__ uint64_t wave_sorted_top_k(uint64_t key, int m, int k) {
  const uint32_t lo = (uint32_t)key, hi = (uint32_t)(key >> 32);
  int rank = 0;
  for (int j = 0; j < m; ++j) {
    const uint64_t o = ((uint64_t)__builtin_amdgcn_readlane(hi, j) << 32) | (uint32_t)__builtin_amdgcn_readlane(lo, j);
    rank += o > key ? 1 : 0;
  }
  const bool keep = key != 0 && rank < k;           // k <= kSampMaxK = 32: lane 63 is never a destination
  const int dst = (keep ? rank : 63) * 4;
  const uint32_t slo = (uint32_t)__builtin_amdgcn_ds_permute(dst, (int)(keep ? lo : 0u));
  const uint32_t shi = (uint32_t)__builtin_amdgcn_ds_permute(dst, (int)(keep ? hi : 0u));
  return ((uint64_t)shi << 32) | slo;               // lanes nobody sends to read 0
}

// Number of lanes of this wave whose key is larger than this lane's.  v_readlane broadcasts (the lane
// index is uniform), not LDS-crossbar shuffles: 64 dependent ds_bpermute round trips cost microseconds.
__device__ __forceinline__ int wave_rank(uint64_t key, int m) {
  const uint32_t lo = (uint32_t)key, hi = (uint32_t)(key >> 32);
  int rank = 0;
#pragma unroll 8
  for (int j = 0; j < m; ++j) {
    const uint64_t o = ((uint64_t)__builtin_amdgcn_readlane(hi, j) << 32) | (uint32_t)__builtin_amdgcn_readlane(lo, j);
    rank += o > key ? 1 : 0;
  }
  return rank;
}

// Sorted top-k of the m keys in `cur` (m <= the buffer size; 0 = empty slot) into sh.top[0..k), the rest of
// sh.top zeroed; returns the k-th largest key (0 if there are fewer than k).  `cur` / `other` are
// the two LDS buffers; both are clobbered.  All lanes of the workgroup must call it.
//
// Up to 256 keys are ranked directly: lane i counts the keys larger than key i (uniform LDS
// addresses: broadcast reads; a wave none of whose lanes holds a key skips the count - the chain of a
// decode-sized launch is bound by the instructions its waves issue, not by their latencies).  More than that are first thinned by a lower bound of the k-th
// largest from a sample: every wave ranks 64 keys of its own (256 distinct positions spread over the
// buffer), and the smallest of the four ceil(k/4)-th largest has >= k sampled keys at or above it;
// at least 32 sampled keys fall below it, so every round makes progress.
template <class Lds>
__device__ uint64_t select_top_k(Lds& sh, uint64_t* cur, uint64_t* other, int m, int k) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  while (m > kRowWG) {
    const uint64_t key = cur[(int)(((int64_t)tid * m) >> 8)];
    const int rank = wave_rank(key, 64);
    const int want = (k + kRowWaves - 1) / kRowWaves;
    if (lane == 0) sh.thr4[wave] = 0;  // stays 0 (no bound) when fewer than `want` sampled keys are real
    __builtin_amdgcn_wave_barrier();
    if (key != 0 && rank == want - 1) sh.thr4[wave] = key;
    if (tid == 0) sh.cnt = 0;
    __syncthreads();
    uint64_t thr = sh.thr4[0];
#pragma unroll
    for (int w = 1; w < kRowWaves; ++w) thr = sh.thr4[w] < thr ? sh.thr4[w] : thr;
    for (int i = tid; i < m; i += kRowWG) {
      const uint64_t key2 = cur[i];
      if (key2 >= thr && key2 != 0) other[atomicAdd(&sh.cnt, 1)] = key2;
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
  if (m > kRowWG) m = kRowWG;  // unreachable, see above
  const uint64_t key = tid < m ? cur[tid] : 0;
  int rank = 0;
  if (wave * 64 < m)  // wave-uniform: a wave whose lanes hold no key has nothing to rank
    for (int j = 0; j < m; ++j) rank += cur[j] > key ? 1 : 0;
  if (tid < kSampMaxK) sh.top[tid] = 0;
  __syncthreads();
  if (key != 0 && rank < k) sh.top[rank] = key;
  __syncthreads();
  return sh.top[k - 1];
}

// Lower bound of the k-th largest element of this workgroup's range from the lanes' own maxima (-inf
// for a lane that saw nothing): each wave extracts its ceil(k/4) largest lane maxima one by one (a
// wave-wide max, then the first lane that holds it steps aside), and the smallest of the four results
// has at least k lane maxima at or above it.  Values only - any element with that value passes.
template <class Lds>
__device__ uint64_t bound_from_lane_maxima(Lds& sh, float lane_max, int k) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int want = (k + kRowWaves - 1) / kRowWaves;
  float v = lane_max, kth = -INFINITY;
  for (int t = 0; t < want; ++t) {
    float m = v;  // wave-wide maximum: four DPP steps inside the rows, two exchanges across them
    m = fmaxf(m, wave_exchange<0>(m));
    m = fmaxf(m, wave_exchange<1>(m));
    m = fmaxf(m, wave_exchange<2>(m));
    m = fmaxf(m, wave_exchange<3>(m));
    m = fmaxf(m, wave_exchange<4>(m));
    m = fmaxf(m, wave_exchange<5>(m));
    kth = m;
    const uint64_t holders = __ballot(v == m);
    if (holders == 0) break;  // cannot happen (lane maxima are never NaN); guards the ctz below
    if (lane == __builtin_ctzll(holders)) v = -INFINITY;
  }
  if (lane == 0) sh.thr4[wave] = (uint64_t)float_key(kth) << 32;
  __syncthreads();
  uint64_t thr = sh.thr4[0];
#pragma unroll
  for (int w = 1; w < kRowWaves; ++w) thr = sh.thr4[w] < thr ? sh.thr4[w] : thr;
  __syncthreads();
  return thr;
}

// Wave 0: draw among the sorted candidates (lane i < k holds the (i+1)-th largest key, 0 = none) and write the
// row's outputs.  `tot` holds the full-vocabulary (max, sum) in every lane.
__device__ __forceinline__ void finish_sample(const SampleArgs& a, uint64_t key, int64_t r, const RowStat& tot, int lane) {
  const int k = a.top_k;
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

// CACHED: the host promises that a lane owns at most kSampCached load units (short ranges: decode
// batches split over many workgroups); they are loaded once and both passes run from registers.
template <typename T, bool VECTOR, bool CACHED>
__global__ __launch_bounds__(kRowWG) __attribute__((amdgpu_waves_per_eu(6, 8))) void row_sample_kernel(SampleArgs a) {
  static_assert(VECTOR || !CACHED, "the cached variant is for 16-byte units");
  constexpr int kVec = VECTOR ? Elem<T>::kVec : 1;
  __shared__ SampleLds<kSampCap> sh;
  const int64_t r = blockIdx.x / a.splits;
  const int split = blockIdx.x % a.splits;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int k = a.top_k;

  if (a.row_valid && a.row_valid[r] == 0) {  // masked row: not read
    if (split != 0) return;
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
  const int64_t per_split = (n_units + a.splits - 1) / a.splits;
  const int64_t u0 = per_split * split;
  const int64_t u1 = (u0 + per_split < n_units) ? u0 + per_split : n_units;
  // single elements after the last whole unit: lane 0 of the last split
  const int n_tail = split == a.splits - 1 ? (int)(a.V - n_units * kVec) : 0;

  const bool big_range = (u1 - u0) * kVec + n_tail > kSampCap;
  if (tid == 0) sh.cnt = 0;  // published by the first barrier below, before any candidate is offered
  // A candidate: a logit above -inf (a -inf logit has probability zero and is never drawn; NaN fails every
  // compare) at or above the bound (value first, then the whole key).
  auto offer = [&](float x, int64_t idx, uint64_t thr, float thr_val) {
    if (x >= thr_val && x > -INFINITY) {
      const uint64_t key = make_key(x, (uint32_t)idx);
      if (key >= thr) {
        const int pos = atomicAdd(&sh.cnt, 1);
        if (pos < kSampCap) sh.a[pos] = key;
      }
    }
  };
  bool collected = false;  // the streaming variant gathers its candidates during pass 1

  // ---- pass 1: full-vocabulary statistics and this lane's own maximum --------------------------
  RowStat st = stat_identity();
  u32x4 cached[CACHED ? kSampCached : 1];
  float lane_max = -INFINITY;  // this lane's largest element, or -inf when it saw nothing above -inf
  RowStat tot = stat_identity();
  uint64_t theta = 0;
  float tail[Elem<T>::kVec - 1];  // cached variant: the single elements after the last whole unit (lane 0 of the last split)
  if constexpr (CACHED) {
    // Everything a lane owns is in registers, so the statistics take two sweeps over them instead of an online
    // update: the maxima first, then the sum of 2^(y - m) against one reference per wave (no rescaling chain).
    const u32x4* p = reinterpret_cast<const u32x4*>(row);
#pragma unroll
    for (int q = 0; q < kSampCached; ++q) {  // unconditional (clamped) loads: all eight in flight together
      const int64_t u = u0 + tid + q * kRowWG;
      cached[q] = __builtin_nontemporal_load(p + (u < u1 ? u : 0));  // unit 0 exists (checked on the host)
    }
#pragma unroll
    for (int e = 0; e < kVec - 1; ++e) tail[e] = (tid == 0 && e < n_tail) ? Elem<T>::load1(row + n_units * kVec + e) : -INFINITY;
#pragma unroll
    for (int q = 0; q < kSampCached; ++q)
      if (u0 + tid + q * kRowWG < u1) {
        float x[kVec];
        Elem<T>::unpack(cached[q], x);
        lane_max = fmaxf(lane_max, max_of_raw<kVec>(x));
      }
#pragma unroll
    for (int e = 0; e < kVec - 1; ++e) lane_max = fmaxf(lane_max, tail[e]);
    float wmax = lane_max;  // maximum of the wave
    wmax = fmaxf(wmax, wave_exchange<0>(wmax));
    wmax = fmaxf(wmax, wave_exchange<1>(wmax));
    wmax = fmaxf(wmax, wave_exchange<2>(wmax));
    wmax = fmaxf(wmax, wave_exchange<3>(wmax));
    wmax = fmaxf(wmax, wave_exchange<4>(wmax));
    wmax = fmaxf(wmax, wave_exchange<5>(wmax));
    const float mref = fmaxf(wmax, kMaxFloor);
    const float mm = mref * a.scale;
    float s0 = 0.f, s1 = 0.f;
#pragma unroll
    for (int q = 0; q < kSampCached; ++q)
      if (u0 + tid + q * kRowWG < u1) {
        float x[kVec];
        Elem<T>::unpack(cached[q], x);
#pragma unroll
        for (int i = 0; i < kVec; i += 2) {
          s0 += fast_exp2(fmaf(x[i], a.scale, -mm));
          s1 += fast_exp2(fmaf(x[i + 1], a.scale, -mm));
        }
      }
#pragma unroll
    for (int e = 0; e < kVec - 1; ++e) s0 += fast_exp2(fmaf(tail[e], a.scale, -mm));  // -inf adds nothing
    float ws = s0 + s1;
    ws += wave_exchange<0>(ws);
    ws += wave_exchange<1>(ws);
    ws += wave_exchange<2>(ws);
    ws += wave_exchange<3>(ws);
    ws += wave_exchange<4>(ws);
    ws += wave_exchange<5>(ws);
    if (lane == 0) {
      sh.red.mx[wave] = mref;
      sh.red.s[wave] = ws;
    }
    __syncthreads();  // also publishes sh.cnt == 0
#pragma unroll
    for (int w = 0; w < kRowWaves; ++w) stat_merge(tot, RowStat{sh.red.mx[w], sh.red.s[w], 0.f, 0x7fffffff}, a.scale);
    // theta: k-th largest lane maximum (ranges that fit the buffer skip the bound)
    if (big_range) theta = bound_from_lane_maxima(sh, lane_max, k);
  } else if constexpr (VECTOR) {
    // Streaming variant: candidates are collected during this one pass.  The k-th largest of the
    // lanes' maxima over their FIRST units is already a lower bound of the row's k-th largest, so
    // everything at or above it goes to the buffer as it streams by; after a quarter of the range
    // the bound is renewed from the maxima so far, which lets far less through (a few hundred
    // candidates per row in all).
    const u32x4* p = reinterpret_cast<const u32x4*>(row);
    constexpr int kGroup = kRowUnroll * kRowWG;                    // units per workgroup and iteration
    const int64_t n_groups = (u1 > u0 ? u1 - u0 : 0) / kGroup;     // iterations in which every lane has all its units
    uint64_t early = 0;  // ranges that fit the buffer are collected whole
    float early_val = -INFINITY;
    auto consume = [&](const u32x4& v, int64_t unit) {
      float x[kVec];
      Elem<T>::unpack(v, x);
      if (absorb<kVec, false, true>(st, x, (int)unit, a.scale) >= early_val) {
#pragma unroll
        for (int i = 0; i < kVec; ++i) offer(x[i], unit * kVec + i, early, early_val);
      }
    };
    auto renew_bound = [&]() {
      early = bound_from_lane_maxima(sh, st.bi != 0x7fffffff ? st.mx : -INFINITY, k);
      early_val = early == 0 ? -INFINITY : key_float((uint32_t)(early >> 32));
    };
    int64_t g0 = 0;
    if (n_groups > 0 && big_range) {  // first iteration: statistics, then the bound, then its candidates
      u32x4 first[kRowUnroll];
#pragma unroll
      for (int q = 0; q < kRowUnroll; ++q) first[q] = __builtin_nontemporal_load(p + u0 + tid + q * kRowWG);
#pragma unroll
      for (int q = 0; q < kRowUnroll; ++q) {
        float x[kVec];
        Elem<T>::unpack(first[q], x);
        absorb<kVec, false, true>(st, x, (int)(u0 + tid + q * kRowWG), a.scale);
      }
      renew_bound();  // its barriers also publish sh.cnt == 0
#pragma unroll
      for (int q = 0; q < kRowUnroll; ++q) {
        float x[kVec];
        Elem<T>::unpack(first[q], x);
        if (max_of_raw<kVec>(x) >= early_val) {
#pragma unroll
          for (int i = 0; i < kVec; ++i) offer(x[i], (u0 + tid + q * kRowWG) * kVec + i, early, early_val);
        }
      }
      g0 = 1;
    } else {
      __syncthreads();  // sh.cnt == 0 is visible
    }
    const int64_t g_renew = n_groups >= 8 && big_range ? 1 + (n_groups - 1) / 4 : n_groups;
    for (int64_t gi = g0; gi < n_groups; ++gi) {
      if (gi == g_renew) renew_bound();  // uniform: every lane runs the same iterations
      u32x4 v[kRowUnroll];
#pragma unroll
      for (int q = 0; q < kRowUnroll; ++q) v[q] = __builtin_nontemporal_load(p + u0 + gi * kGroup + tid + q * kRowWG);
#pragma unroll
      for (int q = 0; q < kRowUnroll; ++q) consume(v[q], u0 + gi * kGroup + tid + q * kRowWG);
    }
    for (int64_t u = u0 + n_groups * kGroup + tid; u < u1; u += kRowWG) consume(__builtin_nontemporal_load(p + u), u);
    if (tid == 0) {
      for (int e = 0; e < n_tail; ++e) {
        float x[1] = {Elem<T>::load1(row + n_units * kVec + e)};
        absorb<1, false, true>(st, x, (int)(n_units + e), a.scale);
        offer(x[0], n_units * kVec + e, early, early_val);
      }
    }
    collected = true;
  } else {
    for (int64_t u = u0 + tid; u < u1; u += kRowWG) {
      float x[1] = {Elem<T>::load1(row + u)};
      absorb<1, false, true>(st, x, (int)u, a.scale);
    }
  }
  int m = 0;
  bool scan = true;
  if constexpr (!CACHED) {
    lane_max = st.bi != 0x7fffffff ? st.mx : -INFINITY;  // nothing above the floor seen: -inf
    tot = block_reduce(st, a.scale, sh.red);  // valid in wave 0; its barrier also ends the offers of pass 1
    if (collected) {
      const int offered = sh.cnt;
      if (offered <= kSampCap) {
        m = offered;
        scan = false;
      } else {  // the early bound let too much through: fall back to the bound from the whole range and rescan
        __syncthreads();
        if (tid == 0) sh.cnt = 0;
      }
    }
    // ---- theta: k-th largest lane maximum (ranges that fit the buffer skip the bound) --------------
    if (scan && big_range) theta = bound_from_lane_maxima(sh, lane_max, k);
    else if (scan && collected) __syncthreads();
  }

  // ---- pass 2: collect every element >= theta ---------------------------------------------------
  uint64_t sorted = 0;  // wave 0, lane i < k: the (i+1)-th largest key of this range
  if constexpr (CACHED) {
    // sh.cnt is zero here: cleared before the first barrier, and again after an overflow.
    for (;;) {
      const float theta_val = theta == 0 ? -INFINITY : key_float((uint32_t)(theta >> 32));
      // Opaque to the optimiser, so that the keys and element indices below are formed where they are
      // used (rarely) instead of being hoisted out of the retry loop into a hundred live registers.
      uint32_t first_elem = (uint32_t)((u0 + tid) * kVec);
      asm volatile("" : "+v"(first_elem));
#pragma unroll
      for (int q = 0; q < kSampCached; ++q)
        asm volatile("" : "+v"(cached[q].x), "+v"(cached[q].y), "+v"(cached[q].z), "+v"(cached[q].w));
#pragma unroll
      for (int q = 0; q < kSampCached; ++q)
        if (u0 + tid + q * kRowWG < u1) {
          float x[kVec];
          Elem<T>::unpack(cached[q], x);
          if (max_of_raw<kVec>(x) >= theta_val) {
#pragma unroll
            for (int i = 0; i < kVec; ++i) offer(x[i], first_elem + (uint32_t)(q * kRowWG * kVec + i), theta, theta_val);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      if (tid == 0)
#pragma unroll
        for (int e = 0; e < kVec - 1; ++e) offer(tail[e], n_units * kVec + e, theta, theta_val);  // -inf where there is none
      __syncthreads();
      const int offered = sh.cnt;
      if (offered <= kSampCap) {
        m = offered;
        break;
      }
      // Overflow: the k-th largest of the kSampCap keys that were kept is a strictly higher lower bound.
      __syncthreads();
      theta = select_top_k(sh, sh.a, sh.b, kSampCap, k);
      if (tid == 0) sh.cnt = 0;
      __syncthreads();
    }
    if (m <= 64) {  // the usual case: wave 0 ranks them in registers, the other waves are done
      if (wave != 0) return;
      sorted = wave_sorted_top_k(lane < m ? sh.a[lane] : 0, m, k);
    } else {
      select_top_k(sh, sh.a, sh.b, m, k);
      if (wave != 0) return;
      sorted = lane < k ? sh.top[lane] : 0;
    }
  } else {
    // sh.cnt is zero here: cleared before the first barrier, and again after an overflow.
    while (scan) {
      const float theta_val = theta == 0 ? -INFINITY : key_float((uint32_t)(theta >> 32));
      auto offer2 = [&](float x, int64_t idx) { offer(x, idx, theta, theta_val); };
      if constexpr (VECTOR) {
        const u32x4* p = reinterpret_cast<const u32x4*>(row);
        int64_t u = u0 + tid;
        for (; u + (kRowUnroll - 1) * kRowWG < u1; u += kRowUnroll * kRowWG) {
          u32x4 v[kRowUnroll];
#pragma unroll
          for (int q = 0; q < kRowUnroll; ++q) v[q] = p[u + q * kRowWG];
#pragma unroll
          for (int q = 0; q < kRowUnroll; ++q) {
            float x[kVec];
            Elem<T>::unpack(v[q], x);
            if (max_of_raw<kVec>(x) >= theta_val) {
#pragma unroll
              for (int i = 0; i < kVec; ++i) offer2(x[i], (u + q * kRowWG) * kVec + i);
            }
          }
        }
        for (; u < u1; u += kRowWG) {
          float x[kVec];
          Elem<T>::unpack(p[u], x);
          if (max_of_raw<kVec>(x) >= theta_val) {
#pragma unroll
            for (int i = 0; i < kVec; ++i) offer2(x[i], u * kVec + i);
          }
        }
        if (tid == 0)
          for (int e = 0; e < n_tail; ++e) offer2(Elem<T>::load1(row + n_units * kVec + e), n_units * kVec + e);
      } else {
        for (int64_t u = u0 + tid; u < u1; u += kRowWG) offer2(Elem<T>::load1(row + u), u);
      }
      __syncthreads();
      const int offered = sh.cnt;
      if (offered <= kSampCap) {
        m = offered;
        break;
      }
      // Overflow: the k-th largest of the kSampCap keys that were kept is a strictly higher lower bound.
      __syncthreads();
      theta = select_top_k(sh, sh.a, sh.b, kSampCap, k);
      if (tid == 0) sh.cnt = 0;
      __syncthreads();
    }
    select_top_k(sh, sh.a, sh.b, m, k);
    if (wave != 0) return;
    sorted = lane < k ? sh.top[lane] : 0;
  }

  // ---- wave 0: the row's outputs, or this range's record for the combine kernel -----------------------
  if (a.splits == 1) {
    finish_sample(a, sorted, r, tot, lane);
  } else {
    const int64_t slot = r * a.splits + split;
    if (lane < k) a.part_keys[slot * k + lane] = sorted;
    if (lane == 0) a.part_stat[slot] = float2{tot.mx, tot.s};
  }
}

// splits > 1: one workgroup per row merges the splits' candidates and statistics and draws.
__global__ __launch_bounds__(kRowWG) void row_sample_combine_kernel(SampleArgs a) {
  __shared__ SampleLds<kSampMergeCap> sh;
  const int64_t r = blockIdx.x;
  if (a.row_valid && a.row_valid[r] == 0) return;  // outputs already written by the main kernel
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int k = a.top_k, m = a.splits * k;         // <= 64 * 32 = kSampMergeCap
  const uint64_t* keys = a.part_keys + r * m;      // per split: its k keys in descending order, 0 past the end
  // Every key is fetched once, up front and together with the statistics and the heads for the bound: the kernel then
  // waits for global memory one time (the previous launch wrote these bytes on other dies, so each wait is a trip
  // beyond the L2).
  constexpr int kPer = kSampMergeCap / kRowWG;
  constexpr int kWaveCap = kSampMergeCap / kRowWaves;
  uint64_t mine[kPer];
#pragma unroll
  for (int q = 0; q < kPer; ++q) {
    const int i = tid + q * kRowWG;
    mine[q] = i < m ? keys[i] : 0;
  }
  RowStat st = stat_identity();
  uint64_t head = 0;
  if (wave == 0) {
    if (lane < a.splits) {
      const float2 p = a.part_stat[r * a.splits + lane];
      st.mx = p.x;
      st.s = p.y;
    }
    // A lower bound of the k-th largest from the heads of the lists: the largest 64 / splits keys of every
    // split; where those are k keys or more, their k-th largest keeps a few dozen of the splits * k keys.
    if (m > 64) {
      const int per = 64 / a.splits;               // >= 1: splits <= 64
      const int sp = lane / per, j = lane % per;
      if (sp < a.splits && j < k) head = keys[sp * k + j];
    }
    uint64_t thr = 0;
    if (m > 64) {
      const int rank = wave_rank(head, 64);
      const uint64_t at = __ballot(head != 0 && rank == k - 1);  // at most one lane: keys are distinct
      if (at != 0) {
        const int src = __builtin_ctzll(at);
        thr = ((uint64_t)__builtin_amdgcn_readlane((uint32_t)(head >> 32), src) << 32) |
              (uint32_t)__builtin_amdgcn_readlane((uint32_t)head, src);
      }
    }
    if (lane == 0) sh.thr4[0] = thr;
  }
  __syncthreads();
  const uint64_t thr = sh.thr4[0];
  WaveCollector col{sh.a + wave * kWaveCap, kWaveCap, 0};  // a wave offers at most kPer * 64 = kWaveCap keys: no overflow
#pragma unroll
  for (int q = 0; q < kPer; ++q)
    if (q * kRowWG + wave * 64 < m)  // wave-uniform
      col.offer(mine[q] != 0 && mine[q] >= thr, mine[q]);
  if (lane == 0) sh.wave_cnt[wave] = col.count;
  __syncthreads();
  int c[kRowWaves];
#pragma unroll
  for (int w = 0; w < kRowWaves; ++w) c[w] = sh.wave_cnt[w];
  const int kept = c[0] + c[1] + c[2] + c[3];
  uint64_t sorted;
  if (kept <= 64) {  // the usual case: wave 0 ranks them in registers
    if (wave != 0) return;
    sorted = wave_sorted_top_k(lane < kept ? region_entry(sh.a, kWaveCap, c, lane) : 0, kept, k);
  } else {
    for (int i = tid; i < kept; i += kRowWG) sh.b[i] = region_entry(sh.a, kWaveCap, c, i);
    __syncthreads();
    select_top_k(sh, sh.b, sh.a, kept, k);
    if (wave != 0) return;
    sorted = lane < k ? sh.top[lane] : 0;
  }
  stat_wave_reduce(st, a.scale);
  finish_sample(a, sorted, r, st, lane);
}

int row_splits_for(int64_t rows, int64_t V, int vec);

// Workgroups per row.  Decode-sized batches are cut into ranges of ~8192 elements whatever the batch size: the selection
// bookkeeping of a workgroup grows with its elements, 8192 fp32 elements are the most a workgroup keeps in
// registers between its passes, and fewer, fatter workgroups beat filling the chip (64 rows fp32: 19-20
// splits 23 us, 32 splits 27 us, 12 splits 37 us; 256 rows: 20 splits 47 us, the row kernel's 8 splits
// 68 us).  Very small batches still get enough workgroups to pull a row from many CUs.  Larger batches follow the
// row kernel (one workgroup per row from 512 rows on, which streams the row once); where that takes over was measured
// at V = 151936, ranges against the row kernel's policy: fp32 512 / 768 / 900 / 1024 / 1152 rows 62.5 / 85.4 / 97.4 / 110.5 /
// 125.2 us against 83.0 / 92.6 / 100.5 / 107.9 / 121.4; bf16 256 / 300 / 340 / 400 rows 41.3 / 46.6 / 50.5 / 56.8 against 47.7 /
// 50.4 / 50.9 / 53.6 (a bf16 range holds twice the elements per byte, and it is the per-element work that costs).
static int sample_splits_for(int64_t rows, int64_t V, int vec) {
  const int base = row_splits_for(rows, V, vec);
  int64_t s = (V + 8191) / 8192;
  const int64_t most_ranges = vec == 4 ? 18000 : 6500;   // rows * ranges: ~950 fp32 rows, ~340 bf16 rows at V = 151936
  if (rows * s > most_ranges) return base;
  const int64_t fill = (512 + rows - 1) / rows;
  if (s < fill) s = fill;
  const int64_t max_by_work = (V / vec) / (2 * kRowWG);  // >= 2 load units per lane and split
  if (s > max_by_work) s = max_by_work;
  if (s > 64) s = 64;
  if (s < 1) s = 1;
  return (int)s;
}

static size_t align256s(size_t b) { return (b + 255) & ~(size_t)255; }
size_t row_sample_workspace_bytes(int64_t rows, int64_t V, int dtype_vec, int top_k) {
  const int splits = sample_splits_for(rows, V, dtype_vec);
  if (splits == 1) return 0;
  return align256s((size_t)rows * splits * top_k * sizeof(uint64_t)) + align256s((size_t)rows * splits * sizeof(float2));
}

hipError_t row_sample_launch(const void* logits, int dtype, int64_t rows, int64_t V, int64_t row_stride,
                             const float* uniforms, const int32_t* row_valid, float temperature, int top_k,
                             int32_t* out_token, float* out_lp, float* out_lse, int32_t* out_argmax,
                             int32_t* out_topk_idx, float* out_topk_logit, void* workspace, hipStream_t stream) {
  const int esize = dtype == 0 ? 4 : 2;
  const int vec = 16 / esize;
  const bool vector_ok = (reinterpret_cast<uintptr_t>(logits) % 16 == 0) && (row_stride % vec == 0);
  // The workspace is sized for the vector layout; the element-wise instantiation uses the same split count.
  const int splits = sample_splits_for(rows, V, vec);
  char* ws = static_cast<char*>(workspace);
  SampleArgs a{logits, uniforms, row_valid, out_token, out_lp, out_lse, out_argmax, out_topk_idx, out_topk_logit,
               reinterpret_cast<uint64_t*>(ws),
               reinterpret_cast<float2*>(ws + align256s((size_t)rows * splits * top_k * sizeof(uint64_t))),
               V, row_stride, top_k, splits, kLog2e / temperature};
  const dim3 grid((unsigned)(rows * splits)), block(kRowWG);
  const int64_t units_per_split = (V / vec + splits - 1) / splits;
  const bool cached = vector_ok && V >= vec && units_per_split <= (int64_t)kSampCached * kRowWG;
  if (dtype == 0) {
    if (cached) hipLaunchKernelGGL((row_sample_kernel<float, true, true>), grid, block, 0, stream, a);
    else if (vector_ok) hipLaunchKernelGGL((row_sample_kernel<float, true, false>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((row_sample_kernel<float, false, false>), grid, block, 0, stream, a);
  } else {
    if (cached) hipLaunchKernelGGL((row_sample_kernel<uint16_t, true, true>), grid, block, 0, stream, a);
    else if (vector_ok) hipLaunchKernelGGL((row_sample_kernel<uint16_t, true, false>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((row_sample_kernel<uint16_t, false, false>), grid, block, 0, stream, a);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || splits == 1) return e;
  hipLaunchKernelGGL(row_sample_combine_kernel, dim3((unsigned)rows), block, 0, stream, a);
  return hipGetLastError();
}

}  // namespace tome
