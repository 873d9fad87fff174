// Fused lm_head + log-softmax: hidden[n, H] x weight[V, H]^T -> per-token log-prob of the
// target id (+ lse, entropy), with the [n, V] logits living only in MFMA accumulators.
//
// Replaces `logits = x @ embed_tokens.weight.T` (mlx-impl/model.py:538) followed by
// local_compute_logprobs (mlx-impl/node.py:400-404); the reference materialises the logits in
// bf16 and upcasts them again, here bf16 x bf16 products are accumulated in fp32 and consumed
// in place.
//
// Decomposition
//   * The GEMM is computed transposed: MFMA "A" rows are vocab entries (W is [V, H], K
//     contiguous), MFMA "B" columns are tokens (hidden is [n, H], K contiguous).  In the
//     accumulator layouts a lane then owns ONE token per block column (lane % 32 with the 32x32
//     MFMA, lane % 16 with the 16x16 one) and a few vocab rows per block, so the softmax row
//     statistics are per-lane registers that persist across the whole vocab sweep; the lanes
//     that share a token are merged once at the end.
//   * A workgroup owns one token tile and a contiguous range of 256-row vocab tiles.  Per vocab
//     tile it runs the K loop, then folds the accumulator tile into the running
//     (max, sum 2^(y-m), sum y 2^(y-m)) states.  Two kernels share this shape; a third,
//     fused_lmhead_small_kernel (<= 64 tokens, W streamed once, K split across waves), is
//     described where it is defined:
//       fused_lmhead_dma_kernel  (H % 64 == 0) 512 lanes, 256 vocab rows x 256 / 128 / 64 tokens,
//                                16x16x32 MFMA, K slabs DMA'd into LDS - described at the kernel;
//       fused_lmhead_kernel      (any H % 8) 256 lanes, 256 x 128 tile, 32x32x16 MFMA, 64-wide
//                                slabs staged through registers into padded LDS.
//   * The vocab axis is split over workgroups (fused_schedule); each writes one partial per
//     (token, split, vocab-wave) and fused_combine_kernel merges them deterministically.
//   * Masked tokens are compacted first (compact_rows_kernel); token tiles are built from
//     the compacted index list, so masked rows cost no FLOPs and no HBM traffic.
#include "common.hpp"
#include <atomic>
#include <type_traits>

namespace tome {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kBV = 256;                 // vocab rows per tile
constexpr int kBT = 128;                 // tokens per tile
constexpr int kBK = 64;                  // K slab
constexpr int kPitch = kBK * 2 + 16;     // LDS row pitch in bytes: 16 B pad -> conflict-free b128 reads
constexpr int kFusedWG = 256;
constexpr int kWaveV = 128, kWaveT = 64; // per-wave tile
constexpr int kNBV = kWaveV / 32, kNBT = kWaveT / 32;
constexpr int kALoads = kBV * 8 / kFusedWG;  // 16-byte chunks per lane per slab (W)
constexpr int kBLoads = kBT * 8 / kFusedWG;  // (hidden)
constexpr int kPartsPerSplit = kBV / kWaveV;

struct FusedPartial {  // 32 bytes per (token, part)
  float mx, s, w, tx;
  int bi;
  int pad[3];
};

// Work decomposition: token tiles x vocab splits.  It depends on the number of valid tokens, which is
// known on the host without a mask and only on the device with one, so it is computed by the host (and
// passed by value) or by compact_rows_kernel (and read from the workspace header); both run the
// same code.  Every kernel of a launch uses the same numbers.
//
// A workgroup owns one token tile and one contiguous range of vocab tiles.
//   * Few token tiles (n_ttiles * 8 <= slots): as many splits as fill the chip in ONE round, rounded
//     down - one workgroup too many would cost a whole extra round.
//   * Many token tiles: several rounds.  The candidates 1..32 are priced as
//         rounds * (longest vocab range + half a tile of prologue) * L2 penalty
//     where the penalty prefers >= 8 splits: the workgroups resident on an XCD are then a block of
//     ~4 token tiles x ~8 splits, which read 12 distinct slab streams through its L2 instead of 33
//     (measured on MI355X: 65536 tokens, H = 4096: 1 split 1.09 PFLOP/s, 8-9 splits 1.4).
struct FusedSchedule {
  int n_ttiles, n_splits, n_wg, pad;
};
// The vocab axis is dealt to the splits in UNITS: whole 256-row tiles for the generic kernel (one unit per tile), 32-row
// units for the DMA kernel (eight per tile), whose last tile of a range may be shorter than 256 rows.  `upt` = units per tile.
__host__ __device__ inline int64_t fused_split_cost(int n_ttiles, int n_splits, int slots, int n_vunits, int upt) {
  const int rounds = (n_ttiles * n_splits + slots - 1) / slots;
  const int longest = (n_vunits + n_splits - 1) / n_splits;  // in units
  const int pen64 = 60 + 32 / (n_splits < 8 ? n_splits : 8);
  return ((int64_t)rounds * (2 * longest + upt) * pen64) * 64 + n_splits;  // ties go to fewer splits
}
__host__ __device__ inline int fused_ttiles(int n_valid, int bt) {
  const int t = (n_valid + bt - 1) / bt;
  return t < 1 ? 1 : t;
}
__host__ __device__ inline int fused_one_round_splits(int n_ttiles, int slots, int n_vtiles) {
  int sp = slots / n_ttiles;
  if (sp > n_vtiles) sp = n_vtiles;  // every split keeps at least one tile's worth of rows
  return sp < 1 ? 1 : sp;
}
constexpr int kSplitCandidates = 32;
inline FusedSchedule fused_schedule(int n_valid, int bt, int slots, int n_vunits, int upt) {  // host
  FusedSchedule s;
  const int n_vtiles = (n_vunits + upt - 1) / upt;
  s.n_ttiles = fused_ttiles(n_valid, bt);
  s.pad = 0;
  if (s.n_ttiles * 8 <= slots) {
    s.n_splits = fused_one_round_splits(s.n_ttiles, slots, n_vtiles);
  } else {
    int64_t best = INT64_MAX;
    for (int c = 1; c <= kSplitCandidates && c <= n_vtiles; ++c) {
      const int64_t cost = fused_split_cost(s.n_ttiles, c, slots, n_vunits, upt);
      if (cost < best) best = cost;
    }
    s.n_splits = (int)(best & 63);
  }
  s.n_wg = s.n_ttiles * s.n_splits;
  return s;
}
// The same on the device, by one whole wave: lane c prices c + 1 splits.
__device__ inline FusedSchedule fused_schedule_wave(int n_valid, int bt, int slots, int n_vunits, int upt, int lane) {
  FusedSchedule s;
  const int n_vtiles = (n_vunits + upt - 1) / upt;
  s.n_ttiles = fused_ttiles(n_valid, bt);
  s.pad = 0;
  if (s.n_ttiles * 8 <= slots) {
    s.n_splits = fused_one_round_splits(s.n_ttiles, slots, n_vtiles);
  } else {
    const int c = lane + 1;
    int64_t cost = (c <= kSplitCandidates && c <= n_vtiles) ? fused_split_cost(s.n_ttiles, c, slots, n_vunits, upt) : INT64_MAX;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const int64_t o = __shfl_xor(cost, off, 64);
      cost = o < cost ? o : cost;
    }
    s.n_splits = (int)(cost & 63);
  }
  s.n_wg = s.n_ttiles * s.n_splits;
  return s;
}

// Workgroup id -> (token tile, vocab split).  The hardware deals consecutive workgroup ids round-robin
// over the 8 XCDs, each with its own L2; XCD x is given the contiguous logical ids
// [x * per, (x + 1) * per), and logical ids run over blocks of <= 8 splits, token tile by token tile,
// so that the workgroups resident on an XCD at any time share token tiles AND vocab ranges.
__device__ __forceinline__ bool fused_locate(const FusedSchedule& s, int bid, int& ttile, int& split) {
  const int per = (s.n_wg + 7) >> 3;
  const int li = bid >> 3;
  int g = (bid & 7) * per + li;
  if (li >= per || g >= s.n_wg) return false;  // the grid is sized for the worst case over n_valid
  const int nb = (s.n_splits + 7) >> 3, base = s.n_splits / nb, rem = s.n_splits % nb;
  int s0 = 0, w = base;
  for (int sb = 0; sb < nb; ++sb) {
    w = base + (sb < rem ? 1 : 0);
    const int cnt = s.n_ttiles * w;
    if (g < cnt) break;
    g -= cnt;
    s0 += w;
  }
  ttile = g / w;
  split = s0 + g % w;
  return true;
}

struct FusedArgs {
  const char* hidden;
  const char* weight;
  const int32_t* targets;
  const int32_t* row_index;  // compacted valid rows (position -> row of targets / outputs), or nullptr = identity
  const int32_t* hidden_index;  // position -> row of `hidden`: row_index, or nullptr when hidden is already compact
  const int32_t* n_valid;    // device scalar, or nullptr = n_tokens
  const FusedSchedule* sched_dev;  // written by compact_rows_kernel next to n_valid, or nullptr = `sched`
  FusedPartial* partials;
  uint32_t hidden_stride_b;  // bytes
  uint32_t weight_stride_b;
  uint32_t hidden_bytes;     // extent of the hidden matrix (< 4 GiB, checked on the host)
  int unit32;                // DMA kernel: 32-row blocks per vocab unit (1, or 7 / 8 when ranges are whole tiles of 224 / 256 rows)
  int n_tokens;
  int H;
  int V;
  int n_vunits;              // vocab units the splits share out: 256-row tiles (generic kernel) or 32-row units (DMA kernel)
  int slots;                 // workgroups that fit the chip at once (the schedule aims at one round)
  float scale;               // log2(e) / temperature
  FusedSchedule sched;       // host-computed schedule (no mask)
};

// Raw buffer descriptors: 16-byte loads addressed by a 32-bit per-lane byte offset plus a
// uniform (scalar) offset.  A per-lane offset at or past num_bytes reads as zero, which is how
// vocab rows past V are handled; the scalar offset is not range-checked.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const char* base, uint32_t num_bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(base), 0, num_bytes, 0x00020000);
}
__device__ __forceinline__ u32x4 ld16(__amdgpu_buffer_rsrc_t r, uint32_t lane_off, uint32_t uniform_off) {
  return __builtin_amdgcn_raw_buffer_load_b128(r, lane_off, uniform_off, 0);
}


// Fold one wave tile of logits (NBV x NBT blocks of 32x32 accumulators) into the per-token
// running states.  Accumulator element e of block i holds vocab row
//   vw0 + i*32 + 8*(e/4) + 4*lh + e%4        (vw0 = first vocab row of this wave's tile)
// for the token this lane owns in block column j.
template <bool ENT, bool AMAX, int NBV, int NBT>
__device__ __forceinline__ void fold_tile(f32x16 (&acc)[NBV][NBT], RowStat (&st)[NBT], float (&tx)[NBT],
                                          const int (&tgt)[NBT], int vw0, int lh, bool partial_tile, int V,
                                          float scale) {
  if (partial_tile) {  // last vocab tile: rows past V do not exist
#pragma unroll
    for (int i = 0; i < NBV; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const bool dead = vw0 + 4 * lh + i * 32 + 8 * (e / 4) + (e % 4) >= V;
#pragma unroll
        for (int j = 0; j < NBT; ++j) acc[i][j][e] = dead ? -INFINITY : acc[i][j][e];
      }
  }
  const int vlane = vw0 + 4 * lh;  // first vocab row this lane holds in block 0
#pragma unroll
  for (int j = 0; j < NBT; ++j) {
    // One scheduling region per token block: otherwise all accumulator reads of all blocks are
    // hoisted to the top and the register file overflows.
    __builtin_amdgcn_sched_barrier(0);
    // Target capture: rare (one tile in V/256 per token), so behind a wave-uniform test.
    const int rel = tgt[j] - vw0;
    const bool mine = tgt[j] >= 0 && rel >= 0 && rel < NBV * 32 && ((rel >> 2) & 1) == lh;
    if (__any(mine)) {
      const int want = mine ? ((rel >> 5) * 16 + ((rel & 31) >> 3) * 4 + (rel & 3)) : -1;
#pragma unroll
      for (int i = 0; i < NBV; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) tx[j] = (want == i * 16 + e) ? acc[i][j][e] : tx[j];
    }
    float cm = st[j].mx;
    int bi = st[j].bi;
#pragma unroll
    for (int i = 0; i < NBV; ++i) {
      if constexpr (AMAX) {
        // The running maximum carries the vocab row of the element that set it.  A lane meets its rows in
        // ascending order and only a strictly larger value replaces the holder, so the first maximum stays.
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const float x = acc[i][j][e];
          bi = x > cm ? vlane + i * 32 + 8 * (e / 4) + (e % 4) : bi;
          cm = raw_max(cm, x);
        }
      } else {
        float m = acc[i][j][0];
#pragma unroll
        for (int e = 1; e < 16; e += 2) m = raw_max3(m, acc[i][j][e], e + 1 < 16 ? acc[i][j][e + 1] : acc[i][j][e]);
        cm = raw_max(cm, m);
      }
    }
    const float dm = (st[j].mx - cm) * scale;
    const float resc = fast_exp2(dm);
    const float m = cm * scale;
    // w: sum (y - m) 2^(y - m), relative to the running maximum (stat_merge has the rule for moving it)
    float s0 = st[j].s * resc, s1 = 0.f, w0 = ENT ? fmaf(dm, st[j].s, st[j].w) * resc : 0.f, w1 = 0.f;
#pragma unroll
    for (int i = 0; i < NBV; ++i)
#pragma unroll
      for (int e = 0; e < 16; e += 2) {
        const float x0 = acc[i][j][e], x1 = acc[i][j][e + 1];
        const float t0 = fmaf(x0, scale, -m), t1 = fmaf(x1, scale, -m);
        const float e0 = fast_exp2(t0);
        const float e1 = fast_exp2(t1);
        s0 += e0;
        s1 += e1;
        if constexpr (ENT) {  // a masked row (-inf): floor * 0, not -inf * 0
          w0 = fmaf(clamp_below(t0), e0, w0);
          w1 = fmaf(clamp_below(t1), e1, w1);
        }
      }
    st[j].mx = cm;
    st[j].bi = bi;
    st[j].s = s0 + s1;
    if constexpr (ENT) st[j].w = w0 + w1;
  }
}

// Merge the two lane halves that share a token and write one partial per (token, part).
template <int NBT>
__device__ __forceinline__ void write_partials(RowStat (&st)[NBT], float (&tx)[NBT], FusedPartial* partials,
                                               int p0, int n_valid, int part, int n_parts, int l32, int lh,
                                               float scale) {
#pragma unroll
  for (int j = 0; j < NBT; ++j) {
    stat_wave_step<5>(st[j], scale);
    const float txo = wave_exchange<5>(tx[j]);
    tx[j] = fmaxf(tx[j], txo);
    const int p = p0 + j * 32 + l32;
    if (lh == 0 && p < n_valid) {
      FusedPartial out;
      out.mx = st[j].mx;
      out.s = st[j].s;
      out.w = st[j].w;
      out.tx = tx[j];
      out.bi = st[j].bi;
      out.pad[0] = out.pad[1] = out.pad[2] = 0;
      partials[(int64_t)p * n_parts + part] = out;
    }
  }
}

template <bool ENT, bool AMAX>
__global__ __launch_bounds__(kFusedWG, 2) void fused_lmhead_kernel(FusedArgs a) {
  __shared__ __attribute__((aligned(16))) char lds[(kBV + kBT) * kPitch];
  char* ldsA = lds;
  char* ldsB = lds + kBV * kPitch;

  const int n_valid = a.n_valid ? *a.n_valid : a.n_tokens;
  const FusedSchedule sch = a.sched_dev ? *a.sched_dev : a.sched;
  int ttile, split;
  if (n_valid <= 0 || !fused_locate(sch, blockIdx.x, ttile, split)) return;
  const int t0 = ttile * kBT;
  const int vt0 = (int)((int64_t)split * a.n_vunits / sch.n_splits);  // one unit = one 256-row tile here
  const int vt1 = (int)((int64_t)(split + 1) * a.n_vunits / sch.n_splits);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wave_v = wave & 1, wave_t = wave >> 1;
  const int l32 = lane & 31, lh = lane >> 5;

  // ---- global -> LDS staging assignment: 8 lanes cover one 128-byte row segment ----------
  const int ld_row = tid >> 3, ld_c = tid & 7;
  const __amdgpu_buffer_rsrc_t rsrcB = make_rsrc(a.hidden, a.hidden_bytes);
  uint32_t boff[kBLoads];
#pragma unroll
  for (int j = 0; j < kBLoads; ++j) {
    int p = t0 + ld_row + 32 * j;
    p = p < n_valid ? p : n_valid - 1;
    const int tok = a.hidden_index ? a.hidden_index[p] : p;
    boff[j] = (uint32_t)tok * a.hidden_stride_b + ld_c * 16;
  }
  uint32_t aoff[kALoads];
#pragma unroll
  for (int j = 0; j < kALoads; ++j) aoff[j] = (uint32_t)(ld_row + 32 * j) * a.weight_stride_b + ld_c * 16;
  const int st_off = ld_row * kPitch + ld_c * 16;

  // ---- per-lane token state ---------------------------------------------------------------
  RowStat st[kNBT];
  float tx[kNBT];
  int tgt[kNBT];
#pragma unroll
  for (int bt = 0; bt < kNBT; ++bt) {
    st[bt] = stat_identity();
    tx[bt] = -INFINITY;
    int p = t0 + wave_t * kWaveT + bt * 32 + l32;
    int t = -1;
    if (p < n_valid) t = a.targets[a.row_index ? a.row_index[p] : p];
    tgt[bt] = (t >= 0 && t < a.V) ? t : -1;
  }

  const int nk = (a.H + kBK - 1) / kBK;
  const char* rdA = ldsA + (wave_v * kWaveV + l32) * kPitch + lh * 16;
  const char* rdB = ldsB + (wave_t * kWaveT + l32) * kPitch + lh * 16;

  for (int vt = vt0; vt < vt1; ++vt) {
    const int v0 = vt * kBV;
    // Descriptor rebased to this tile: per-lane offsets stay constant and rows past V fall
    // outside num_bytes (read as zero, then masked to -inf in the epilogue).
    const __amdgpu_buffer_rsrc_t rsrcA =
        make_rsrc(a.weight + (int64_t)v0 * a.weight_stride_b, (uint32_t)(a.V - v0) * a.weight_stride_b);

    f32x16 acc[kNBV][kNBT];
#pragma unroll
    for (int i = 0; i < kNBV; ++i)
#pragma unroll
      for (int j = 0; j < kNBT; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    u32x4 ra[kALoads], rb[kBLoads];
    const bool in0 = ld_c * 8 < a.H;
#pragma unroll
    for (int j = 0; j < kALoads; ++j) ra[j] = in0 ? ld16(rsrcA, aoff[j], 0) : u32x4{0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < kBLoads; ++j) rb[j] = in0 ? ld16(rsrcB, boff[j], 0) : u32x4{0, 0, 0, 0};

    for (int kt = 0; kt < nk; ++kt) {
      __syncthreads();  // every wave has finished reading the previous slab
#pragma unroll
      for (int j = 0; j < kALoads; ++j) *reinterpret_cast<u32x4*>(ldsA + st_off + j * 32 * kPitch) = ra[j];
#pragma unroll
      for (int j = 0; j < kBLoads; ++j) *reinterpret_cast<u32x4*>(ldsB + st_off + j * 32 * kPitch) = rb[j];
      __syncthreads();
      if (kt + 1 < nk) {  // prefetch the next slab while this one is multiplied
        const int koff = (kt + 1) * kBK * 2;
        const bool in = (kt + 1) * kBK + ld_c * 8 < a.H;
#pragma unroll
        for (int j = 0; j < kALoads; ++j) ra[j] = in ? ld16(rsrcA, aoff[j], koff) : u32x4{0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < kBLoads; ++j) rb[j] = in ? ld16(rsrcB, boff[j], koff) : u32x4{0, 0, 0, 0};
      }
#pragma unroll
      for (int ks = 0; ks < kBK / 16; ++ks) {
        bf16x8 fa[kNBV], fb[kNBT];
#pragma unroll
        for (int i = 0; i < kNBV; ++i)
          fa[i] = *reinterpret_cast<const bf16x8*>(rdA + i * 32 * kPitch + ks * 32);
#pragma unroll
        for (int j = 0; j < kNBT; ++j)
          fb[j] = *reinterpret_cast<const bf16x8*>(rdB + j * 32 * kPitch + ks * 32);
#pragma unroll
        for (int i = 0; i < kNBV; ++i)
#pragma unroll
          for (int j = 0; j < kNBT; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
      }
    }

    fold_tile<ENT, AMAX>(acc, st, tx, tgt, v0 + wave_v * kWaveV, lh, v0 + kBV > a.V, a.V, a.scale);
  }

  write_partials(st, tx, a.partials, t0 + wave_t * kWaveT, n_valid, split * kPartsPerSplit + wave_v,
                 sch.n_splits * kPartsPerSplit, l32, lh, a.scale);
}



// ---- 16x16x32 MFMA accumulator layout --------------------------------------------------------------
// A 16x16 block lives in four registers: lane l holds token column l % 16 and vocab rows
// 4*(l/16) + e, e = 0..3.  A lane therefore owns one token per 16-token block, and the four lane
// groups l/16 share that token: they are merged once, at the end, over lane ^ 16 and lane ^ 32.
typedef float f32x4v __attribute__((ext_vector_type(4)));

// Fold one wave tile (NBV x NBT blocks of 16x16) into the per-token running states.  Element e of
// block i holds vocab row  vw0 + i*16 + 4*g + e  (g = lane / 16) for the token of block column j.
// NBV of the NBV_ALLOC block rows the array holds are folded (a short tile uses the first few).
template <bool ENT, bool AMAX, int NBV, int NBT, int NBV_ALLOC>
__device__ __forceinline__ void fold_tile16(f32x4v (&acc)[NBV_ALLOC][NBT], RowStat (&st)[NBT], float (&tx)[NBT],
                                            const int (&tgt)[NBT], int vw0, int g, bool partial_tile, int V,
                                            float scale) {
  if (partial_tile) {  // last vocab tile: rows past V do not exist
#pragma unroll
    for (int i = 0; i < NBV; ++i)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const bool dead = vw0 + i * 16 + 4 * g + e >= V;
#pragma unroll
        for (int j = 0; j < NBT; ++j) acc[i][j][e] = dead ? -INFINITY : acc[i][j][e];
      }
  }
  const int vlane = vw0 + 4 * g;  // first vocab row this lane holds in block 0
#pragma unroll
  for (int j = 0; j < NBT; ++j) {
    __builtin_amdgcn_sched_barrier(0);  // one scheduling region per token block (register pressure)
    // Target capture: rare (one tile in V/256 per token), so behind a wave-uniform test.
    const int rel = tgt[j] - vw0;
    const bool mine = tgt[j] >= 0 && rel >= 0 && rel < NBV * 16 && ((rel >> 2) & 3) == g;
    if (__any(mine)) {
      const int want = mine ? ((rel >> 4) * 4 + (rel & 3)) : -1;
#pragma unroll
      for (int i = 0; i < NBV; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) tx[j] = (want == i * 4 + e) ? acc[i][j][e] : tx[j];
    }
    float cm = st[j].mx;
    int bi = st[j].bi;
#pragma unroll
    for (int i = 0; i < NBV; ++i) {
      if constexpr (AMAX) {
        // Seven more VALU operations per block, only when the argmax is asked for: the block maximum comes
        // with the position of its first holder, and the running maximum carries the vocab row of the
        // element that set it.  Only a strictly larger value replaces the holder and a lane meets its rows in
        // ascending order, so the sweep itself names the first maximum of the fp32 logits it computed.
        const float x0 = acc[i][j][0], x1 = acc[i][j][1], x2 = acc[i][j][2], x3 = acc[i][j][3];
        const float m01 = raw_max(x0, x1), m23 = raw_max(x2, x3);
        const int e01 = x1 > x0 ? 1 : 0, e23 = x3 > x2 ? 3 : 2;
        const int e = m23 > m01 ? e23 : e01;
        const float bm = raw_max(m01, m23);
        bi = bm > cm ? vlane + i * 16 + e : bi;
        cm = raw_max(cm, bm);
      } else {
        const float bm = raw_max3(acc[i][j][0], acc[i][j][1], raw_max(acc[i][j][2], acc[i][j][3]));
        cm = raw_max(cm, bm);
      }
    }
    const float dm = (st[j].mx - cm) * scale;
    const float resc = fast_exp2(dm);
    const float m = cm * scale;
    // w: sum (y - m) 2^(y - m), relative to the running maximum (stat_merge has the rule for moving it)
    float s0 = st[j].s * resc, s1 = 0.f, w0 = ENT ? fmaf(dm, st[j].s, st[j].w) * resc : 0.f, w1 = 0.f;
#pragma unroll
    for (int i = 0; i < NBV; ++i)
#pragma unroll
      for (int e = 0; e < 4; e += 2) {
        const float x0 = acc[i][j][e], x1 = acc[i][j][e + 1];
        const float t0 = fmaf(x0, scale, -m), t1 = fmaf(x1, scale, -m);
        const float e0 = fast_exp2(t0);
        const float e1 = fast_exp2(t1);
        s0 += e0;
        s1 += e1;
        if constexpr (ENT) {  // a masked row (-inf): floor * 0, not -inf * 0
          w0 = fmaf(clamp_below(t0), e0, w0);
          w1 = fmaf(clamp_below(t1), e1, w1);
        }
      }
    st[j].mx = cm;
    st[j].bi = bi;
    st[j].s = s0 + s1;
    if constexpr (ENT) st[j].w = w0 + w1;
  }
}

// Merge the four lane groups that share a token and write one partial per (token, part).
template <int NBT>
__device__ __forceinline__ void write_partials16(RowStat (&st)[NBT], float (&tx)[NBT], FusedPartial* partials,
                                                 int p0, int n_valid, int part, int n_parts, int l16, int g,
                                                 float scale) {
#pragma unroll
  for (int j = 0; j < NBT; ++j) {
    stat_wave_step<4>(st[j], scale);
    stat_wave_step<5>(st[j], scale);
    tx[j] = fmaxf(tx[j], wave_exchange<4>(tx[j]));
    tx[j] = fmaxf(tx[j], wave_exchange<5>(tx[j]));
    const int p = p0 + j * 16 + l16;
    if (g == 0 && p < n_valid) {
      FusedPartial out;
      out.mx = st[j].mx;
      out.s = st[j].s;
      out.w = st[j].w;
      out.tx = tx[j];
      out.bi = st[j].bi;
      out.pad[0] = out.pad[1] = out.pad[2] = 0;
      partials[(int64_t)p * n_parts + part] = out;
    }
  }
}

// ===============================================================================================
// Fast path (H % 64 == 0): 512 lanes, 256 x 256 tile, v_mfma_f32_16x16x32_bf16, K slabs DMA'd straight
// into LDS, double-buffered (a third W buffer in the DEEP form, below).
//
//   * 8 waves as 2 (vocab) x 4 (token), 128 vocab x 64 tokens per wave as 8 x 4 blocks of 16x16.  The
//     16x16x32 MFMA moves half the accumulator bytes per FLOP of the 32x32x16 one; on this
//     power-limited part that alone is worth 12-16 % (measured with the instruction swapped in place).
//     The partial layout is shared with the other kernels.
//   * global_load_lds_dwordx4: every lane fetches 16 bytes and the wave's 1 KB lands contiguously
//     in LDS, bypassing registers.  No staging registers are needed, which leaves room to
//     double-buffer the MFMA fragments.
//   * What this kernel pays for beside its MFMAs is the L2 -> LDS fill (64 KB per 256x256x64 MACs and CU: the
//     requests cost in proportion to their number, wherever the data lands and whether or not it hits in L2 -
//     mostly as engine clock, which this power-limited part lowers under the added load, not as issue slots),
//     and the L2 serves it by the request, not by the byte: a slab row is therefore one whole 128-byte
//     cache line (K = 64), which streams 1.5x faster than 64-byte rows.  Two 64 KB slabs (W 256 rows +
//     hidden 256 rows each) fill the LDS; one is computed on while the other is in flight.  Step s (one
//     slab = two K = 32 MFMA sub-steps of 32 MFMAs per wave, each in two halves by vocab block) runs
//         MFMA(s, k0, blocks 0-3) | reads (s, k0, blocks 4-7), requests 5-6 of slab s+1
//         MFMA(s, k0, blocks 4-7) | reads (s, k1, blocks 0-3 and hidden), requests 7-8 of slab s+1
//         MFMA(s, k1, blocks 0-3) | reads (s, k1, blocks 4-7)
//         own reads and own share of slab s+1 complete; barrier
//         MFMA(s, k1, blocks 4-7) | reads (s+1, k0, blocks 0-3 and hidden), requests 1-4 of slab s+2
//     After the barrier everybody has read all of slab s, so it can be refilled, and slab s+1 is
//     visible before its first fragments are read, which happens under the last quarter of the
//     MFMAs - the MFMA stream has no bubble at step or vocab-tile boundaries.
//   * Bank conflicts are avoided by an XOR swizzle instead of padding (DMA writes are dense).
//     The LDS has 64 four-byte banks, so a 16-lane phase of a 128-bit read is conflict-free when
//     its 16 rows hit 16 different 16-byte bank groups.  A 128-byte row r covers groups
//     8*(r&1) .. +7, so chunk c of row r is stored at chunk position c ^ ((r >> 1) & 7); the
//     lane that DMA-writes position p of row r fetches global chunk p ^ ((r >> 1) & 7).
// ===============================================================================================
//
// The token tile is a template parameter: NBT = 4 token blocks per wave (256 tokens per workgroup) is the
// shape described above and the one the MFMA/DMA interleave is tuned for; NBT = 2 and 1 (128 and 64
// tokens) serve batches of up to one such tile, where W is streamed once and the kernel is bound by
// that stream: they do the MFMA work of 128 or 64 tokens instead of 256 per slab of W.
constexpr int k2BV = 256, k2WG = 512;
constexpr int k2BK = 64;
constexpr int k2RowBytes = k2BK * 2;                     // 128: one cache line
// Slab buffers, as many as fit the 160 KB of LDS: two for the 256-token tile (64 KB per slab), three otherwise.
// The W halves and the hidden halves form two rings of that depth.
constexpr int dma_bufs(int nbt) { return nbt == 4 ? 2 : 3; }
// With two buffers a slab's request is issued in three portions - in the last quarter of the step that frees
// its buffer, and in the first two quarters of the next step - instead of all at once: right after a barrier
// all eight waves are at the same point, and 64 requests issued together queue up in the memory pipeline
// while the waves that issued them cannot issue their MFMAs.
constexpr int kIssueQ4 = 4, kIssueQ1 = 2;   // instructions of the eight in the last / first quarter; the rest in the second
constexpr int k2Loads = k2BV * (k2RowBytes / 16) / k2WG; // DMA instructions per lane and slab for W (4)
constexpr int k2NBV = kWaveV / 16;                       // 16x16 vocab blocks per wave tile: 8
static_assert(k2Loads == 4 && k2NBV == 8, "the MFMA/DMA interleave is written for this shape");
constexpr int dma_tile_tokens(int nbt) { return nbt * 64; }                                   // 4 token waves x nbt x 16
constexpr int dma_w_bytes() { return k2BV * k2RowBytes; }                                      // 32768
constexpr int dma_h_bytes(int nbt) { return dma_tile_tokens(nbt) * k2RowBytes; }               // 32768 at nbt = 4
// DEEP (256-token tile only): a third W buffer, which is all of the CU's LDS; see the kernel.
constexpr int dma_w_bufs(int nbt, bool deep) { return deep ? 3 : dma_bufs(nbt); }
constexpr int dma_lds_bytes(int nbt, bool deep = false) {  // 131072 at nbt = 4, 163840 with the third W buffer
  return dma_w_bufs(nbt, deep) * dma_w_bytes() + dma_bufs(nbt) * dma_h_bytes(nbt);
}

// AUX: the request's cache policy bits (0 = default, 2 = non-temporal).  Hidden rows always go with the default; W rows
// do wherever several token tiles read them (there non-temporal requests for either operand measured 1.5-5 % slower),
// see WNT at the kernel.
template <int AUX = 0>
__device__ __forceinline__ void dma16(const char* gptr, char* lds_wave_base) {
  __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint32_t*>(gptr),
                                   (__attribute__((address_space(3))) uint32_t*)lds_wave_base, 16, 0, AUX);
}

// Scheduling pattern: N_READS times (N_MFMA MFMAs, then one LDS read).
template <int N_MFMA, int N_READS>
__device__ __forceinline__ void pair_reads() {
#pragma unroll
  for (int q = 0; q < N_READS; ++q) {
    __builtin_amdgcn_sched_group_barrier(0x008, N_MFMA, 0);  // MFMA
    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);       // DS read
  }
}

// Vocab ranges are dealt in units of 32 rows and a workgroup cuts its range into the fewest tiles of at most 256 rows,
// all of the same height or one unit apart (the taller ones first): V = 151936 over 16 splits is 297 units per
// workgroup = 31 tiles of 256 rows + 7 of 224, where whole 256-row tiles would give some workgroups 38 tiles and others
// 37 - and a tile costs its full MFMA work however few of its rows count.  A tile of nb blocks of 16 rows per wave
// (nb = 1 .. 8) runs the same pipeline with 8 * nb MFMAs per wave and step.  Its slab keeps the LDS layout of a whole
// tile (rows 0..127 for the waves of vocab half 0, 128..255 for half 1, so fragment addresses do not change); each
// half holds 16 * nb rows of W and the rest of its LDS rows are requested as copies of its last row and never multiplied.
//
// DEEP: the 256-token tile with THREE W buffers and two hidden buffers (160 KB, the whole LDS of a CU).  The W half of
// a slab is requested two steps ahead - in the first two quarters of a step, its buffer free since the previous step's
// barrier - and the hidden half, which comes from L2, one step ahead, after the step's own barrier; before a barrier
// the four W instructions of the newest request stay in flight.  Faster wherever a step waits for its fill: 10-15 %
// where every workgroup streams W rows of its own (one token tile), 2-3 % at 4096 x 1024 tokens x hidden, nothing from
// 8192 x 4096 on; with the entropy or the argmax its fold spills and it only pays at one or two token tiles
// (fused_plan holds the rule and the figures).
//
// WNT: W is requested non-temporally.  Where W streams through once or a few times (up to four token tiles) its rows have
// no business in the caches that the hidden rows and the partials live in: 64 x 4096 tokens x hidden 221 -> 205 us,
// 256 x 1024 88 -> 84, 128 x 4096 234 -> 230, 512 x 1024 138 -> 135.5, 1024 x 4096 924 -> 917; from 2048 tokens on the
// workgroups of an XCD that share a W tile want it kept (4096 x 1024: 936 -> 951), and so do three 128-token tiles
// (384 x 1024: 130 -> 138).
template <bool ENT, bool AMAX, int NBT, int HI, bool DEEP = false, bool WNT = false>
__global__ __launch_bounds__(k2WG) void fused_lmhead_dma_kernel(FusedArgs a) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  static_assert((NBT == 4 && (HI == 4 || HI == 3)) || (NBT != 4 && HI == 0), "256-token tile: every vocab tile 256 (HI = 4) or 224 rows; others: mixed heights");
  static_assert(!DEEP || NBT == 4, "the third W buffer is for the 256-token tile");
  // The 256-token tile runs at the limit of the register file: it keeps ONE tile height per launch (4 + HI blocks per wave,
  // the host picks 256 or 224 rows), because the code for two or more heights in one kernel costs it 60 and more spilled
  // registers whose reloads, at every tile change, wait for memory behind the W stream (measured with heights of 224 and
  // 256 rows mixed: +8 % at 4096 x 1024 instead of the 1.7 % that the even shares would save).  The smaller token tiles
  // have registers to spare and mix heights as described above.
  constexpr bool kMixed = HI == 0;
  constexpr int kMaxBlocks = kMixed ? 8 : 4 + HI;   // 16-row vocab blocks per wave in the tallest tile
  constexpr int kNBVw = 8;                          // accumulator block rows per wave
  constexpr int k2NBT = NBT;                        // 16-token blocks per wave
  constexpr int k2BT = dma_tile_tokens(NBT);        // tokens per workgroup
  constexpr int kWaveTok = NBT * 16;                // tokens per wave
  constexpr int kBufs = dma_bufs(NBT);              // hidden buffers
  constexpr int kBufsW = dma_w_bufs(NBT, DEEP);     // W buffers
  constexpr int kWBytes = dma_w_bytes(), kHBytes = dma_h_bytes(NBT);
  constexpr int kHBase = kBufsW * kWBytes;          // the hidden ring starts behind the W ring
  constexpr int kBLoads = NBT;                      // DMA instructions per lane and slab for the hidden rows
  constexpr int k2DmaPerSlab = k2Loads + kBLoads;   // 8 at NBT = 4
  // Portions of a request (see kIssueQ4): with three buffers everything goes out in the last quarter.
  constexpr int kP4 = NBT == 4 ? kIssueQ4 : k2DmaPerSlab;
  constexpr int kP1 = NBT == 4 ? kIssueQ1 : 0;
  constexpr int kP2 = k2DmaPerSlab - kP4 - kP1;
  static_assert(kP4 >= 1 && kP1 >= 0 && kP2 >= 0 && kP1 <= 8 && kP2 <= 8, "portions of the eight instructions");
  static_assert(kBufs == 2 || kP4 == k2DmaPerSlab, "split requests are written for two buffers");
  // Which of the eight instructions (0-3: W, 4-7: hidden) go out in the first, second and last quarter of a step.
  // Two buffers: a request starts in the last quarter of the step that frees its buffers (W first: it has furthest to
  // come) and ends in the second quarter of the next.  DEEP: request step + 2 as a whole inside one step, W in the first
  // two quarters (its buffer was freed by the previous step's barrier), hidden after this step's barrier.
  constexpr int kQ1Lo = DEEP ? 0 : kP4, kQ1Hi = DEEP ? 2 : kP4 + kP1;
  constexpr int kQ2Lo = kQ1Hi, kQ2Hi = DEEP ? 4 : k2DmaPerSlab;
  constexpr int kQ4Lo = DEEP ? 4 : 0, kQ4Hi = DEEP ? k2DmaPerSlab : kP4;
  constexpr bool kDoneAfterQ4 = DEEP || kP4 == k2DmaPerSlab;
  // Requests complete in the order they were issued, so "slab s has landed" is a count of newer instructions that
  // may still be in flight.  Before a step's barrier (slab step + 1 must be there) those are the whole requests
  // of the slabs after it (DEEP: the W instructions of request step + 2); before the loop (slab 0) also the first
  // portion of the newest request (DEEP: the whole request for slab 1).
  constexpr int kInFlightAtStep = DEEP ? k2Loads : (kBufs - 2) * k2DmaPerSlab;
  constexpr int kInFlightAtStart = DEEP ? k2DmaPerSlab : (kBufs - 2) * k2DmaPerSlab + kP4;

  const int n_valid = a.n_valid ? *a.n_valid : a.n_tokens;
  const FusedSchedule sch = a.sched_dev ? *a.sched_dev : a.sched;
  int ttile, split;
  if (n_valid <= 0 || !fused_locate(sch, blockIdx.x, ttile, split)) return;
  const int t0 = ttile * k2BT;
  // This workgroup's vocab range in 32-row blocks (a.unit32 = blocks per unit: 1, or 7 / 8 when ranges are whole tiles).
  const int u0 = (int)((int64_t)split * a.n_vunits / sch.n_splits) * a.unit32;
  const int u1 = (int)((int64_t)(split + 1) * a.n_vunits / sch.n_splits) * a.unit32;
  const int n_units = u1 - u0;                      // >= 1: every split holds at least one unit
  // With mixed heights every workgroup of a launch cuts its range into the SAME number of tiles (the longest range's), so
  // that all of them step through tiles of (nearly) the same heights at the same time: the workgroups that share a
  // hidden-state or W stream in an XCD's L2 only hit there while they stay in step.
  const int n_tiles = kMixed ? ((a.n_vunits + sch.n_splits - 1) / sch.n_splits * a.unit32 + 7) >> 3 : n_units / kMaxBlocks;
  const int nb_short = kMixed ? n_units / n_tiles : kMaxBlocks;  // 16-row blocks per wave of the shorter tiles (1 .. 8)
  const int n_tall = kMixed ? n_units - nb_short * n_tiles : 0;  // tiles with one block more: they come first
  const int row0 = u0 * 32;
  auto tile_blocks = [&](int tile) { return nb_short + (tile < n_tall ? 1 : 0); };
  auto tile_row0 = [&](int tile) {
    if constexpr (!kMixed) return row0 + tile * (32 * kMaxBlocks);
    else return row0 + 32 * (tile * nb_short + (tile < n_tall ? tile : n_tall));
  };

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keeps LDS bases scalar
  const int wave_v = wave & 1, wave_t = wave >> 1;
  const int l16 = lane & 15, g = lane >> 4;  // 16x16 MFMA: token column, lane group

  // ---- DMA assignment: instruction j of wave w fills LDS rows (j*8 + w)*8 .. +7 of an operand ----
  // All address arithmetic is incremental: per-lane pointers advance by one slab (128 bytes) per
  // request and are rebased at vocab-tile changes, so a step carries no multiplies or divides.
  const int dr = lane >> 3;                                   // row inside the 8-row group
  const int dc = (lane & 7) ^ (4 * (wave & 1) + (dr >> 1));   // global chunk: position ^ ((row >> 1) & 7)
  const char* pa[k2Loads];  // next W slab to request, per DMA instruction
  const char* pb[kBLoads];  // next hidden slab
  // Mixed heights: LDS row r of a W slab holds vocab row  base + (r / 128) * wr + min(r % 128, wr - 1)  of tile `tile`,
  // wr = rows per wave of that tile.  One height: LDS row r is tile row r; the 32 LDS rows past a 224-row tile are requested
  // as copies of rows that waves 0-3 fetch with the same instruction.  Rows past V (last tile only) read the last row
  // and are masked in the epilogue.
  auto point_a = [&](int tile) {
    const int64_t base = tile_row0(tile);
    const int wr = kMixed ? tile_blocks(tile) * 16 : kMaxBlocks * 16;
    // The lane's row and chunk are derived afresh here (the empty asm hides that they are loop invariants): hoisted
    // out of the sweep, the 64-bit per-lane address terms built from them would stay live across every step, and this
    // kernel has no register left for them.
    int ln = lane;
    asm volatile("" : "+v"(ln));
    const int dr = ln >> 3;
    const int dc = (ln & 7) ^ (4 * (wave & 1) + (dr >> 1));
#pragma unroll
    for (int j = 0; j < k2Loads; ++j) {
      const int r = (j * 8 + wave) * 8 + dr;
      int64_t v;
      if constexpr (kMixed) {
        const int in_half = (r & 127) < wr ? (r & 127) : wr - 1;
        v = base + (r >> 7) * wr + in_half;
      } else {
        v = base + ((HI == 4 || r < 2 * wr) ? r : r - 32);
      }
      v = v < a.V ? v : a.V - 1;
      pa[j] = a.weight + v * a.weight_stride_b + dc * 16;
    }
  };
  point_a(0);
#pragma unroll
  for (int j = 0; j < kBLoads; ++j) {
    int p = t0 + (j * 8 + wave) * 8 + dr;
    p = p < n_valid ? p : n_valid - 1;
    const int tok = a.hidden_index ? a.hidden_index[p] : p;
    pb[j] = a.hidden + (int64_t)tok * a.hidden_stride_b + dc * 16;
  }

  // ---- per-lane token state: one token per 16-token block, shared by the four lane groups ---------
  RowStat st[k2NBT];
  float tx[k2NBT];
  int tgt[k2NBT];
#pragma unroll
  for (int bt = 0; bt < k2NBT; ++bt) {
    st[bt] = stat_identity();
    tx[bt] = -INFINITY;
    const int p = t0 + wave_t * kWaveTok + bt * 16 + l16;
    int t = -1;
    if (p < n_valid) t = a.targets[a.row_index ? a.row_index[p] : p];
    tgt[bt] = (t >= 0 && t < a.V) ? t : -1;
  }

  // ---- fragment read offsets inside a slab (swizzled): lane group g reads chunk 4*ks + g ----------
  const int swz = (g ^ ((l16 >> 1) & 7)) * 16;  // sub-step k0; k1 is this ^ 64
  // the wave's first LDS row (128 with mixed heights) is a multiple of 16: the swizzle term stays l16's
  const int rdA = (wave_v * (kMixed ? 128 : kMaxBlocks * 16) + l16) * k2RowBytes + swz;
  const int rdB = (wave_t * kWaveTok + l16) * k2RowBytes + swz;

  const int nk = a.H / k2BK;
  const int n_steps = n_tiles * nk;
  const int64_t slab_rewind = (int64_t)(nk - 1) * k2RowBytes;
  int i_kt = 0, i_tile = 0;  // slab the next request fetches
  int issued = 0;            // slabs requested so far; request q lands in buffers q % kBufs

  // One of the DMA instructions of the next request (0-3: W rows; the others: hidden rows).  Past the last slab
  // the request is repeated (same addresses, same buffer, identical bytes): it is issued on every step so that
  // the code has no branch and the wait counts stay static.
  auto issue_piece = [&](int piece) {
    const unsigned slab = (unsigned)(issued < n_steps ? issued : n_steps - 1);
    if (piece < k2Loads) dma16<WNT ? 2 : 0>(pa[piece], smem + (slab % kBufsW) * kWBytes + wave * 1024 + piece * 8192);
    else dma16(pb[piece - k2Loads], smem + kHBase + (slab % kBufs) * kHBytes + wave * 1024 + (piece - k2Loads) * 8192);
  };
  auto issue_done = [&]() {
    ++issued;
    if (issued >= n_steps) return;  // the stream stays on the last slab
    if (++i_kt < nk) {
#pragma unroll
      for (int j = 0; j < k2Loads; ++j) pa[j] += k2RowBytes;
#pragma unroll
      for (int j = 0; j < kBLoads; ++j) pb[j] += k2RowBytes;
    } else {
      i_kt = 0;
      ++i_tile;
#pragma unroll
      for (int j = 0; j < kBLoads; ++j) pb[j] -= slab_rewind;
      if (i_tile < n_tiles) point_a(i_tile);
    }
  };
  // Fragments of one K = 32 sub-step of a slab: W blocks [i0, i0 + n) or the hidden blocks.
  // DEEP: the offsets of the second sub-step (rdA ^ 64, rdB ^ 64) are formed where they are used (the empty asm hides
  // that they are loop invariants).  Kept in registers across the sweep they are spilled, and a reload inside a step
  // makes the compiler wait for EVERY outstanding memory operation - the requests two slabs ahead included.
  auto read_a = [&](int slot, int ks, int i0, bf16x8 (&fa)[4], auto n) {
    const char* slab = smem + ((unsigned)slot % kBufsW) * kWBytes;
    int rd = rdA;
    if constexpr (DEEP) asm volatile("" : "+v"(rd));
#pragma unroll
    for (int i = 0; i < decltype(n)::value; ++i)
      fa[i] = *reinterpret_cast<const bf16x8*>(slab + (rd ^ (ks * 64)) + (i0 + i) * 16 * k2RowBytes);
  };
  auto read_b = [&](int slot, int ks, bf16x8 (&fb)[k2NBT]) {
    const char* slab = smem + kHBase + ((unsigned)slot % kBufs) * kHBytes;
    int rd = rdB;
    if constexpr (DEEP) asm volatile("" : "+v"(rd));
#pragma unroll
    for (int j = 0; j < k2NBT; ++j)
      fb[j] = *reinterpret_cast<const bf16x8*>(slab + (rd ^ (ks * 64)) + j * 16 * k2RowBytes);
  };

  // Prologue: whole requests for all buffers but the last, and the first portion of the last one's (DEEP: slabs 0 and 1).
#pragma unroll
  for (int q = 0; q < (DEEP ? 2 : kBufs - 1); ++q) {
#pragma unroll
    for (int piece = 0; piece < k2DmaPerSlab; ++piece) issue_piece(piece);
    issue_done();
  }
  if constexpr (!DEEP) {
#pragma unroll
    for (int piece = 0; piece < kP4; ++piece) issue_piece(piece);
    if constexpr (kP4 == k2DmaPerSlab) issue_done();
  }
  // Slab 0 has landed (this wave's share): only the requests of the later slabs may still be in flight.
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kInFlightAtStart) : "memory");
  __builtin_amdgcn_s_barrier();

  constexpr std::integral_constant<int, 4> kFour{};
  bf16x8 fa_lo[4], fa_hi[4], fb0[k2NBT], fb1[k2NBT];
  read_a(0, 0, 0, fa_lo, kFour);
  read_b(0, 0, fb0);

  f32x4v acc[kNBVw][k2NBT];
#pragma unroll
  for (int i = 0; i < kNBVw; ++i)
#pragma unroll
    for (int j = 0; j < k2NBT; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[i][j][e] = 0.f;

  // 4 * n MFMAs on n vocab blocks; in a whole tile the group barriers then put one LDS read or DMA request behind
  // every MFMA (or every second one), so that its issue hides under the MFMA's execution.
  // `fresh`: the first K sub-step of a vocab tile starts from a zero C operand, which saves clearing
  // the 128 accumulator registers after every fold.
  auto mfma_half = [&](int i0, bf16x8 (&fa)[4], bf16x8 (&fb)[k2NBT], auto fresh, auto n) {
    const f32x4v zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < decltype(n)::value; ++i)
#pragma unroll
      for (int j = 0; j < k2NBT; ++j)
        acc[i0 + i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[i], fb[j], decltype(fresh)::value ? zero : acc[i0 + i][j],
                                                                   0, 0, 0);
  };
  int step = 0;
  // N times (one MFMA, then one DMA request).
  auto pair_dma = [](auto n) {
#pragma unroll
    for (int q = 0; q < decltype(n)::value; ++q) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // VMEM (DMA request)
    }
  };
  // One K slab on a tile of `lo` + `hi` vocab blocks per wave: lo = min(nb, 4), hi = nb - lo.  The fragments of the
  // NEXT step's first quarter are always read for four blocks (the next step may belong to a taller tile).
  auto do_step = [&](auto fresh, auto lo, auto hi) {
    constexpr int LO = decltype(lo)::value, HIB = decltype(hi)::value;
    constexpr bool kTuned = NBT == 4 && LO == 4 && HIB >= 3;  // the interleave below is written for tiles of 224 and 256 rows
    __builtin_amdgcn_sched_barrier(0);
    read_a(step, 0, 4, fa_hi, hi);
#pragma unroll
    for (int piece = kQ1Lo; piece < kQ1Hi; ++piece) issue_piece(piece);  // two buffers: second portion of the request for slab step + 1
    mfma_half(0, fa_lo, fb0, fresh, lo);
    if constexpr (kTuned) {
      pair_reads<2, HIB>();
      pair_dma(std::integral_constant<int, kQ1Hi - kQ1Lo>{});
    }
    __builtin_amdgcn_sched_barrier(0);
    read_a(step, 1, 0, fa_lo, lo);
    read_b(step, 1, fb1);
#pragma unroll
    for (int piece = kQ2Lo; piece < kQ2Hi; ++piece) issue_piece(piece);  // third portion
    mfma_half(4, fa_hi, fb0, fresh, hi);
    if constexpr (kTuned) {
      if constexpr (kQ2Hi == kQ2Lo) {
        pair_reads<2, 8>();
      } else {
        pair_reads<1, 8>();
        pair_dma(std::integral_constant<int, kQ2Hi - kQ2Lo>{});
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (!kDoneAfterQ4) issue_done();
    read_a(step, 1, 4, fa_hi, hi);
    mfma_half(0, fa_lo, fb1, std::false_type{}, lo);
    if constexpr (kTuned) pair_reads<2, HIB>();
    __builtin_amdgcn_sched_barrier(0);
    // This wave has read all it needs of slab `step` and its share of slab step+1 has landed; after
    // the (fence-less) barrier both hold for everyone.  (With three buffers the request of slab step+2
    // stays in flight across the barrier.)
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(kInFlightAtStep) : "memory");
    __builtin_amdgcn_s_barrier();
    // Last quarter: first fragments of slab step+1 (after the last step a stale buffer, unused) and the
    // first portion of the next request, which refills the buffers of slab `step`.  The DMA requests write
    // LDS, so they keep their program order after the fragment reads.
    __builtin_amdgcn_sched_barrier(0);
    read_a(step + 1, 0, 0, fa_lo, kFour);
    read_b(step + 1, 0, fb0);
#pragma unroll
    for (int piece = kQ4Lo; piece < kQ4Hi; ++piece) issue_piece(piece);
    mfma_half(4, fa_hi, fb1, std::false_type{}, hi);
    if constexpr (kTuned) {
      pair_reads<1, 8>();
      pair_dma(std::integral_constant<int, kQ4Hi - kQ4Lo>{});
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (kDoneAfterQ4) issue_done();
    ++step;
  };

  // Two runs of tiles: n_tall tiles of nb_short + 1 blocks, then the others of nb_short blocks.
  auto run_tiles = [&](int first, int last, auto lo, auto hi) {
    constexpr int NB = decltype(lo)::value + decltype(hi)::value;
    for (int tile = first; tile < last; ++tile) {
      do_step(std::true_type{}, lo, hi);
      for (int kt = 1; kt < nk; ++kt) do_step(std::false_type{}, lo, hi);
      const int v0 = tile_row0(tile);
      fold_tile16<ENT, AMAX, NB>(acc, st, tx, tgt, v0 + wave_v * NB * 16, g, v0 + 2 * NB * 16 > a.V, a.V, a.scale);
    }
  };
  using std::integral_constant;
  if constexpr (!kMixed) {
    constexpr integral_constant<int, HI == 0 ? 4 : HI> kHi{};
    for (int tile = 0; tile < n_tiles; ++tile) {
      do_step(std::true_type{}, kFour, kHi);
      for (int kt = 1; kt < nk; ++kt) do_step(std::false_type{}, kFour, kHi);
      const int v0 = row0 + tile * (32 * kMaxBlocks);
      fold_tile16<ENT, AMAX, kMaxBlocks>(acc, st, tx, tgt, v0 + wave_v * kMaxBlocks * 16, g, v0 + 32 * kMaxBlocks > a.V, a.V, a.scale);
    }
  } else {
    for (int run = 0; run < 2; ++run) {
      const int first = run == 0 ? 0 : n_tall, last = run == 0 ? n_tall : n_tiles;
      if (first >= last) continue;
      const int nb = nb_short + (run == 0 ? 1 : 0);
      switch (nb) {
        case 1: run_tiles(first, last, integral_constant<int, 1>{}, integral_constant<int, 0>{}); break;
        case 2: run_tiles(first, last, integral_constant<int, 2>{}, integral_constant<int, 0>{}); break;
        case 3: run_tiles(first, last, integral_constant<int, 3>{}, integral_constant<int, 0>{}); break;
        case 4: run_tiles(first, last, integral_constant<int, 4>{}, integral_constant<int, 0>{}); break;
        case 5: run_tiles(first, last, integral_constant<int, 4>{}, integral_constant<int, 1>{}); break;
        case 6: run_tiles(first, last, integral_constant<int, 4>{}, integral_constant<int, 2>{}); break;
        case 7: run_tiles(first, last, integral_constant<int, 4>{}, integral_constant<int, 3>{}); break;
        default: run_tiles(first, last, kFour, kFour); break;
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no request may outlive the workgroup's LDS

  write_partials16(st, tx, a.partials, t0 + wave_t * kWaveTok, n_valid, split * kPartsPerSplit + wave_v,
                   sch.n_splits * kPartsPerSplit, l16, g, a.scale);
}

// ===============================================================================================
// Small batches (<= 64 tokens, the decode-step regime): W streams from HBM exactly once and nothing is
// reused, so the kernel is built like a streaming reduction, not like a GEMM.
//
//   * K is split across the waves of a workgroup (256 or 512 columns each).  A wave's slice of the
//     hidden states - all tokens - then fits its registers as MFMA B fragments for the whole launch,
//     and W goes from global memory into registers and through a wave-private LDS tile into A
//     fragments: no barrier on the load path.
//   * Each wave keeps 16 sixteen-byte loads in flight (two 16-row tiles of its K slice, refilled in
//     place right after the MFMA that consumed them); one workgroup per CU owns one contiguous range of
//     16-row vocab tiles.
//   * Per tile the waves' partial sums (16 rows x 16*NBT tokens, MFMA layout) meet in LDS; wave j sums
//     them in wave order and folds token block j into its online-softmax state.  One barrier per tile:
//     the buffer of tile t is rewritten at tile t + 2, after the barrier of tile t + 1, which the
//     folding waves only reach once tile t is folded.
//   * One partial per (token, workgroup); the combine kernel is shared with the other paths.
// ===============================================================================================
template <bool ENT, bool AMAX, int NBT, int KSTEPS>
__global__ __launch_bounds__(512) void fused_lmhead_small_kernel(FusedArgs a) {
  extern __shared__ __attribute__((aligned(16))) char small_mem[];  // [2][waves][NBT][64 lanes] f32x4, then [waves] 4 KB tiles
  constexpr int kBuf = 16 / KSTEPS;                                 // tile buffers in flight (registers): 16 loads per lane
  constexpr int kRed = 2;                                           // reduction buffers (LDS)
  const int n_valid = a.n_valid ? *a.n_valid : a.n_tokens;
  if (n_valid <= 0) return;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n_waves = blockDim.x >> 6;
  const int l16 = lane & 15, g = lane >> 4;
  const int n_tiles = (a.V + 15) >> 4;
  const int t0 = (int)((int64_t)blockIdx.x * n_tiles / gridDim.x);
  const int t1 = (int)((int64_t)(blockIdx.x + 1) * n_tiles / gridDim.x);
  const int kb0 = (wave * KSTEPS * 32 + 8 * g) * 2;  // byte offset of this lane's first K chunk in a row

  // Hidden-state fragments of this wave's K slice: lane (token l16, group g) holds K = 32 ks + 8 g .. + 7.
  bf16x8 fb[KSTEPS][NBT];
#pragma unroll
  for (int j = 0; j < NBT; ++j) {
    int p = j * 16 + l16;
    p = p < n_valid ? p : n_valid - 1;
    const int tok = a.hidden_index ? a.hidden_index[p] : p;
    const char* hp = a.hidden + (int64_t)tok * a.hidden_stride_b + kb0;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) fb[ks][j] = *reinterpret_cast<const bf16x8*>(hp + ks * 64);
  }
  // Token state of the block this wave folds (waves >= NBT fold nothing).
  RowStat st[1] = {stat_identity()};
  float tx[1] = {-INFINITY};
  int tgt[1] = {-1};
  if (wave < NBT) {
    const int p = wave * 16 + l16;
    int t = -1;
    if (p < n_valid) t = a.targets[a.row_index ? a.row_index[p] : p];
    tgt[0] = (t >= 0 && t < a.V) ? t : -1;
  }

  // W loads are shaped for HBM, not for the MFMA: one instruction fetches 4 rows x 256 bytes (lane = row
  // lane/16 of the group, 16-byte chunk lane%16), which streams 17 % faster than the operand shape of 16
  // rows x 64 bytes (6.85 against 5.84 TB/s in a copy kernel with this kernel's structure).  A unit of
  // 16 rows x 256 bytes (four K steps) then changes layout through a wave-private 4 KB LDS tile: chunk c
  // of row r is stored at position c ^ r, so the contiguous writes and the fragment reads (16 rows, one
  // chunk) are both free of bank conflicts.
  constexpr int kUnits = KSTEPS / 4;  // units per tile and wave
  const int lr = lane >> 4, lc = lane & 15;
  auto w_ptr = [&](int t, int q) {  // rows past V (last tile only) read the last row; masked in the fold
    int row = t * 16 + 4 * q + lr;
    row = row < a.V ? row : a.V - 1;
    return a.weight + (int64_t)row * a.weight_stride_b + wave * (KSTEPS * 64) + lc * 16;
  };
  char* stage = small_mem + (size_t)kRed * n_waves * NBT * 1024 + wave * 4096;
  u32x4 wb[kBuf][kUnits][4];
#pragma unroll
  for (int b = 0; b < kBuf && t0 < t1; ++b) {
    const int t = t0 + b < t1 ? t0 + b : t1 - 1;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const char* wp = w_ptr(t, q);
#pragma unroll
      for (int u = 0; u < kUnits; ++u) wb[b][u][q] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wp + u * 256));
    }
  }

  for (int tb = t0; tb < t1; tb += kBuf) {
#pragma unroll
    for (int b = 0; b < kBuf; ++b) {
      const int t = tb + b;
      if (t >= t1) break;  // uniform
      // The refill is unconditional (past the range it re-reads the tile just consumed, an L2 hit that is
      // never used): with a load behind a branch the compiler cannot count the loads in flight and waits
      // for far more of them than the one it needs.
      const int tn = t + kBuf < t1 ? t + kBuf : t;
      f32x4v acc[NBT];
#pragma unroll
      for (int j = 0; j < NBT; ++j) acc[j] = f32x4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int u = 0; u < kUnits; ++u) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
          *reinterpret_cast<u32x4*>(stage + (4 * q + lr) * 256 + ((lc ^ (4 * q + lr)) << 4)) = wb[b][u][q];
#pragma unroll
        for (int q = 0; q < 4; ++q)
          wb[b][u][q] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(w_ptr(tn, q) + u * 256));
        // The tile is private to this wave and LDS serves a wave's requests in order.
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        bf16x8 fa[4];
#pragma unroll
        for (int k4 = 0; k4 < 4; ++k4)
          fa[k4] = *reinterpret_cast<const bf16x8*>(stage + l16 * 256 + (((4 * k4 + g) ^ l16) << 4));
#pragma unroll
        for (int k4 = 0; k4 < 4; ++k4)
#pragma unroll
          for (int j = 0; j < NBT; ++j)
            acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[k4], fb[4 * u + k4][j], acc[j], 0, 0, 0);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  // the next unit overwrites what was just read
        __builtin_amdgcn_wave_barrier();
      }
      char* red = small_mem + (size_t)(((t & (kRed - 1)) * n_waves + wave) * NBT) * 1024 + lane * 16;
#pragma unroll
      for (int j = 0; j < NBT; ++j) *reinterpret_cast<f32x4v*>(red + j * 1024) = acc[j];
      __syncthreads();
      if (wave < NBT) {
        f32x4v sum[1][1] = {{f32x4v{0.f, 0.f, 0.f, 0.f}}};
        const char* src = small_mem + (size_t)((t & (kRed - 1)) * n_waves * NBT + wave) * 1024 + lane * 16;
        for (int w = 0; w < n_waves; ++w) sum[0][0] += *reinterpret_cast<const f32x4v*>(src + (size_t)w * NBT * 1024);
        fold_tile16<ENT, AMAX, 1>(sum, st, tx, tgt, t * 16, g, t * 16 + 16 > a.V, a.V, a.scale);
      }
    }
  }
  // One partial per (token, workgroup): part index = workgroup id.
  if (wave < NBT) write_partials16<1>(st, tx, a.partials, wave * 16, n_valid, (int)blockIdx.x, (int)gridDim.x, l16, g, a.scale);
}

// ---- compaction of valid rows ----------------------------------------------------------------
// One workgroup: row_index[0 .. n_valid) = ascending indices of rows with row_valid != 0.
// Outputs of masked rows are zeroed here.
struct CompactArgs {
  const int32_t* row_valid;
  int32_t* row_index;
  int32_t* n_valid;
  float* out0;
  float* out1;
  float* out2;
  float* out3;
  float* out4;
  int32_t* out_argmax;
  int n;
  int bt, slots, n_vunits, upt;  // inputs of the schedule, which this kernel derives from n_valid
};

// Rows are taken in batches of up to 16384: each of the 16 waves owns a run of consecutive rows of a batch (a
// sixteenth of the rows, at most 1024) and reads their mask values with 16 independent coalesced loads (lane
// l of chunk c reads row first + 64 c + l), which stay in registers for the second sweep; counts come from ballots,
// the waves' offsets from a scan through LDS.
__global__ __launch_bounds__(1024) void compact_rows_kernel(CompactArgs a) {
  constexpr int kChunks = 16;                       // 64-row chunks per wave and batch, at most
  __shared__ int wave_tot[16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint64_t below = (1ull << lane) - 1;        // lanes in front of this one
  int n_chunks = (int)((((int64_t)a.n + 15) / 16 + 63) / 64);  // per wave, so that small batches use all 16 waves
  n_chunks = n_chunks > kChunks ? kChunks : n_chunks;
  const int wave_rows = n_chunks * 64;
  const int64_t batch_rows = 16 * (int64_t)wave_rows;
  float* outs[5] = {a.out0, a.out1, a.out2, a.out3, a.out4};  // the float outputs that exist, packed to the front
  int n_outs = 0;
#pragma unroll
  for (int o = 0; o < 5; ++o)
    if (outs[o]) outs[n_outs++] = outs[o];
  int done = 0;                                     // valid rows of earlier batches
  for (int64_t b0 = 0; b0 < a.n; b0 += batch_rows) {
    const int64_t first = b0 + (int64_t)wave * wave_rows;
    int v[kChunks];
#pragma unroll
    for (int c = 0; c < kChunks; ++c) {  // unconditional (clamped) loads: all of them in flight together
      const int64_t r = first + c * 64 + lane;
      v[c] = a.row_valid[r < a.n ? r : a.n - 1];
    }
#pragma unroll
    for (int c = 0; c < kChunks; ++c) v[c] = (c < n_chunks && first + c * 64 + lane < a.n) ? v[c] : 0;
    int cnt = 0;
#pragma unroll
    for (int c = 0; c < kChunks; ++c) cnt += __builtin_popcountll(__ballot(v[c] != 0));
    if (lane == 0) wave_tot[wave] = cnt;
    __syncthreads();
    int pos = done, total = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      pos += w < wave ? wave_tot[w] : 0;
      total += wave_tot[w];
    }
    __syncthreads();                                // wave_tot is rewritten by the next batch
#pragma unroll
    for (int c = 0; c < kChunks; ++c) {
      const int64_t r = first + c * 64 + lane;
      const uint64_t mask = __ballot(v[c] != 0);    // zero for chunks past the end
      if (c < n_chunks && r < a.n) {
        if (v[c] != 0) {
          a.row_index[pos + __builtin_popcountll(mask & below)] = (int32_t)r;
        } else {
          for (int o = 0; o < n_outs; ++o) outs[o][r] = 0.f;
          if (a.out_argmax) a.out_argmax[r] = -1;
        }
      }
      pos += __builtin_popcountll(mask);
    }
    done += total;
  }
  if (tid == 0) *a.n_valid = done;
  if (wave == 15) {  // one wave also fixes the work decomposition, which depends on the total
    const FusedSchedule sch = fused_schedule_wave(done, a.bt, a.slots, a.n_vunits, a.upt, lane);
    if (lane == 0) *reinterpret_cast<FusedSchedule*>(a.n_valid + 4) = sch;
  }
}

// ---- final RMSNorm of the rows that will be multiplied ------------------------------------------
// y = w * T(x * rsqrt(mean(x^2) + eps)) in bf16 with fp32 statistics: mx.fast.rms_norm as
// mlx-impl/model.py:343 calls it on the last hidden states (model.py:536).  Only valid rows are
// normalised, and they are written compactly: position p of the output is row row_index[p] of x.
struct NormArgs {
  const char* x;             // bf16 [n, H]
  const uint16_t* w;         // bf16 [H]
  char* y;                   // bf16 [n_valid, H], dense
  const int32_t* row_index;  // or nullptr = identity
  const int32_t* n_valid;    // or nullptr = n
  uint32_t x_stride_b;
  int n, H;
  float eps;
};

__global__ __launch_bounds__(256) void rmsnorm_rows_kernel(NormArgs a) {
  const int lane = threadIdx.x & 63;
  const int p = blockIdx.x * 4 + (threadIdx.x >> 6);  // one wave per row
  const int n_valid = a.n_valid ? *a.n_valid : a.n;
  if (p >= n_valid) return;
  const int row = a.row_index ? a.row_index[p] : p;
  const u32x4* x = reinterpret_cast<const u32x4*>(a.x + (int64_t)row * a.x_stride_b);
  const u32x4* w = reinterpret_cast<const u32x4*>(a.w);
  u32x4* y = reinterpret_cast<u32x4*>(a.y + (int64_t)p * a.H * 2);
  const int n_chunks = a.H / 8;
  float ss = 0.f;
  for (int c = lane; c < n_chunks; c += 64) {
    const u32x4 v = x[c];
    const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float lo = bf16_lo(u[k]), hi = bf16_hi(u[k]);
      ss = fmaf(lo, lo, ss);
      ss = fmaf(hi, hi, ss);
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
  const float inv = 1.0f / sqrtf(ss / (float)a.H + a.eps);
  for (int c = lane; c < n_chunks; c += 64) {  // second read of the row comes from cache
    const u32x4 v = x[c], g = w[c];
    const uint32_t u[4] = {v.x, v.y, v.z, v.w}, gw[4] = {g.x, g.y, g.z, g.w};
    uint32_t o[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float lo = bf16_bits_to_f32(f32_to_bf16_bits(bf16_lo(u[k]) * inv));
      const float hi = bf16_bits_to_f32(f32_to_bf16_bits(bf16_hi(u[k]) * inv));
      o[k] = (uint32_t)f32_to_bf16_bits(bf16_lo(gw[k]) * lo) | ((uint32_t)f32_to_bf16_bits(bf16_hi(gw[k]) * hi) << 16);
    }
    y[c] = u32x4{o[0], o[1], o[2], o[3]};
  }
}

// ---- combine -----------------------------------------------------------------------------------
struct CombineArgs {
  const FusedPartial* partials;      // policy (or the only) weight set
  const FusedPartial* partials_ref;  // second weight set, or nullptr
  const int32_t* row_index;
  const int32_t* n_valid;
  float* out_lp;
  float* out_lse;
  float* out_entropy;
  float* out_ref_lp;
  float* out_k3;
  int32_t* out_argmax;
  int n_tokens;
  const FusedSchedule* sched_dev;  // as in FusedArgs
  FusedSchedule sched;
  float scale;
};

__device__ __forceinline__ void combine_one(const FusedPartial* parts, int n_parts, int lane, float scale,
                                            RowStat& st, float& tx) {
  st = stat_identity();
  tx = -INFINITY;
  // A lane's partials are fetched eight at a time before the first is merged (clamped, unconditional loads: all in
  // flight together): the merges form a chain, and a load inside it costs a trip to memory per partial - the previous
  // launch wrote these records on other dies.  Same merge order as a plain loop.
  constexpr int kBatch = 8;
  for (int base = 0; base < n_parts; base += 64 * kBatch) {
    f32x4 head[kBatch];
    int bi[kBatch];
#pragma unroll
    for (int q = 0; q < kBatch; ++q) {
      const int i = base + lane + 64 * q;
      const FusedPartial* src = parts + (i < n_parts ? i : n_parts - 1);
      head[q] = *reinterpret_cast<const f32x4*>(src);  // mx, s, w, tx
      bi[q] = src->bi;
    }
#pragma unroll
    for (int q = 0; q < kBatch; ++q) {
      if (base + lane + 64 * q < n_parts) {
        RowStat o{head[q][0], head[q][1], head[q][2], bi[q]};
        stat_merge(st, o, scale);
        tx = fmaxf(tx, head[q][3]);
      }
    }
  }
  stat_wave_reduce(st, scale);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) tx = fmaxf(tx, __shfl_xor(tx, off, 64));
}

__global__ __launch_bounds__(256) void fused_combine_kernel(CombineArgs a) {
  const int lane = threadIdx.x & 63;
  const int p = blockIdx.x * 4 + (threadIdx.x >> 6);  // compacted position, one wave each
  const int n_valid = a.n_valid ? *a.n_valid : a.n_tokens;
  if (p >= n_valid) return;
  const int tok = a.row_index ? a.row_index[p] : p;
  const int n_parts = (a.sched_dev ? a.sched_dev->n_splits : a.sched.n_splits) * kPartsPerSplit;
  RowStat st;
  float tx;
  combine_one(a.partials + (int64_t)p * n_parts, n_parts, lane, a.scale, st, tx);
  const float m = st.mx * a.scale;
  const float log2s = fast_log2(st.s);
  // tx stays -inf only when the target id was outside [0, V).
  const float lp = tx == -INFINITY ? __builtin_nanf("") : (fmaf(tx, a.scale, -m) - log2s) * kLn2;
  float ref_lp = 0.f;
  if (a.partials_ref) {
    RowStat sr;
    float txr;
    combine_one(a.partials_ref + (int64_t)p * n_parts, n_parts, lane, a.scale, sr, txr);
    const float mr = sr.mx * a.scale;
    ref_lp = txr == -INFINITY ? __builtin_nanf("") : (fmaf(txr, a.scale, -mr) - fast_log2(sr.s)) * kLn2;
  }
  if (lane != 0) return;
  // The sweep kernels name the element themselves: bi is the vocab row of the first maximum among the fp32
  // logits they accumulated (0 when nothing above the floor was seen, as a first-maximum scan would say).
  if (a.out_argmax) a.out_argmax[tok] = st.bi == 0x7fffffff ? 0 : st.bi;
  if (a.out_lp) a.out_lp[tok] = lp;
  if (a.out_lse) a.out_lse[tok] = (m + log2s) * kLn2;
  if (a.out_entropy) a.out_entropy[tok] = (log2s - st.w / st.s) * kLn2;
  if (a.out_ref_lp) a.out_ref_lp[tok] = ref_lp;
  if (a.out_k3) {
    const float d = ref_lp - lp;
    a.out_k3[tok] = expm1f(d) - d;
  }
}

// ---- host side -----------------------------------------------------------------------------------
// The DMA kernel needs whole 64-wide K slabs (ragged H goes to the generic kernel); its token tile shrinks
// with the batch.  Decode-sized batches whose hidden states fit the waves' registers take the streaming kernel.

enum FusedKind { kGeneric = 0, kDma = 1, kSmall = 2 };
constexpr int kForceDmaWholeTiles = 3;  // selector value: the DMA kernel with vocab ranges cut at whole 256-row tiles
constexpr int kForceDmaTwoWBuffers = 4, kForceDmaThreeWBuffers = 5;  // the DMA kernel, its 256-token tile with two / three W buffers

// Kernel selector for tests and tuning runs: -1 (the default) picks by shape, kGeneric / kDma force that
// sweep kernel wherever its shape rules allow.  Process-wide; set it while no call is in flight.
static std::atomic<int> g_forced_kind{-1};
void fused_force_kernel(int kind) { g_forced_kind.store(kind, std::memory_order_relaxed); }

struct FusedPlan {
  FusedKind kind;
  int dma_nbt;                               // kDma only: token blocks per wave (4, 2 or 1: 256, 128 or 64 tokens per tile)
  int unit32;                                // kDma only: 32-row blocks per vocab unit (1 = mixed tile heights; 7 / 8 = whole tiles of 224 / 256 rows)
  int dma_deep;                              // kDma, 256-token tile only: three W buffers - 0 never, 1 for sweeps without the entropy, 2 always
  bool w_nt;                                 // kDma only: W requested non-temporally (few token tiles: see the kernel's WNT)
  int small_nbt, small_ksteps, small_waves;  // kSmall only
  int bt, slots;
  int n_vunits, upt;   // vocab units the splits share out, and units per 256-row tile (what a unit costs, for the schedule)
  int grid;            // workgroups to launch: the most any number of valid tokens can ask for
  size_t max_records;  // partial records any number of valid tokens can produce
};

template <typename K>
static bool allow_big_lds(K kernel, int bytes) {
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes) == hipSuccess)
    return true;
  (void)hipGetLastError();  // the launch that follows reports its own error
  return false;
}
// Devices (bit per ordinal) that did not grant the 160 KB of dynamic LDS the three-buffer form asks for - all of a CU's
// LDS, which a driver may not hand out whole: the two-buffer form serves there.
static std::atomic<uint64_t> g_no_deep_lds{0};
static bool deep_lds_refused() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDeviceOrdinals) return false;
  return (g_no_deep_lds.load(std::memory_order_relaxed) >> dev) & 1;
}

// Workgroups of the small-batch kernel: one per CU.  Measured at 16 and 64 tokens, H = 1024: 256 workgroups
// 59 us, 512 66 us, 1024 (all that fit) 71 us, 2048 (queued) 95 us; a deeper load ring changes nothing.
// The stream is bound by the 16-rows-by-64-bytes shape of an MFMA operand load, which a plain copy
// kernel of the same shape and lifetime moves at 5.6 TB/s, and more concurrent streams lower that.
static int small_wg_count() {
  static std::atomic<int> cached[kMaxDeviceOrdinals];  // per device ordinal: GPUs of one process may differ
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDeviceOrdinals) return 0;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 2) return 0;
    if (cus > 512) cus = 512;  // the workspace holds 512 parts per token
    n = cus & ~1;              // even: the combine kernel counts parts in pairs
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

// Shape rules of the small-batch kernel: <= 64 tokens, K split over 2..8 waves in slices of 256 or 512
// (slices of 128 on twice the waves measured 2 us slower at H = 1024).  At H = 1024 it keeps up to 16 tokens only: since
// the tiled kernel requests W non-temporally where it streams through once, its 64- and 128-token tiles are faster there
// from 17 tokens on (17..64 tokens: 53.3-54.8 against 54.7-59 us; 65..128, which this kernel served with eight token blocks
// on K slices of 128: 61-64 against 67-72 us); at 1280, 1536 and 1792 the two are within 3 % of each other either way, at
// 2048 and above this kernel wins (64 x 2048: 108 against 125 us).
static bool small_shape(int64_t n_tokens, int64_t H, int64_t V, int& nbt, int& ksteps, int& waves) {
  if (n_tokens > 64 || V < 64) return false;
  if (H == 1024 && n_tokens > 16) return false;
  nbt = n_tokens <= 16 ? 1 : (n_tokens <= 32 ? 2 : 4);
  if (H % 256 == 0 && H / 256 <= 8 && H / 256 >= 2) {
    ksteps = 8;
    waves = (int)(H / 256);
  } else if (H % 512 == 0 && H / 512 <= 8 && H / 512 >= 2 && nbt <= 2) {
    ksteps = 16;
    waves = (int)(H / 512);
  } else {
    return false;
  }
  if (ksteps == 8 && nbt == 2) nbt = 4;  // instantiated token-block counts: 1 and 4 (K 256), 1 and 2 (K 512)
  return waves >= nbt;
}

static FusedPlan fused_plan(int64_t n_tokens, int64_t H, int64_t V) {
  FusedPlan p;
  p.kind = kGeneric;
  p.small_nbt = p.small_ksteps = p.small_waves = 0;
  p.dma_nbt = n_tokens > 128 ? 4 : (n_tokens > 64 ? 2 : 1);
  // 257 .. 384 tokens: three 128-token tiles do the MFMA work of 384 tokens where two 256-token tiles do that of 512
  // (measured at 384 x 1024: 125 against 139 us; at 512 tokens the 256-token tile wins again, 145 against 166 us).
  if (n_tokens > 256 && n_tokens <= 384) p.dma_nbt = 2;
  // The third W buffer (see the kernel), measured against the two-buffer form in the same runs.  One or two token tiles:
  // 6-13 % faster with any outputs (256 x 1024: 96 -> 87 us, 256 x 4096: 338 -> 297, 512 x 4096: 534 -> 503).  More token
  // tiles, log-probs only: 4096 x 1024 -2.3 %, 8192 x 1024 -1.5 %, 1024 x 4096 -5 %, 4096 x 4096 -1.7 %, 16384 x 2560 -2.6 %,
  // 8192 x 4096 -1.6..+0.2 % over boxes, but 32768 x 4096 +0.7 %, 65536 x 4096 +0.5..2 %.  With the argmax alone it follows
  // (1024 x 4096 -4 %, 4096 x 1024 equal, 8192 x 4096 -1 %); with the entropy the fold of the deeper form spills 29-37
  // registers around every tile change: 1024 x 4096 -3 %, but 4096 x 1024 +2.6 % and 8192 x 4096 +2.3 %.
  p.dma_deep = 0;
  if (p.dma_nbt == 4) p.dma_deep = n_tokens <= 1024 ? 2 : ((H < 4096 || n_tokens <= 8192) ? 1 : 0);
  // Non-temporal W (the kernel's WNT): few token tiles, and a W larger than the 256 MB memory-side cache - a smaller one is
  // found there again by the next call as long as it is requested normally (repeated calls, 64 tokens: V = 32000, H = 4096,
  // 262 MB: 48 us against 71 non-temporally; V = 50257, H = 768, 77 MB: 21.0 against 23.3).
  p.w_nt = (p.dma_nbt == 4 ? n_tokens <= 1024 : n_tokens <= dma_tile_tokens(p.dma_nbt)) && V * H * 2 >= (int64_t)288 << 20;
  p.unit32 = 8;   // 32-row blocks per vocab unit: whole 256-row tiles unless the DMA kernel is given something finer below
  if (H % k2BK == 0) p.kind = kDma;
  // The streaming kernel runs one workgroup per CU: without a CU count (no device) the tiled kernels serve.
  if (small_shape(n_tokens, H, V, p.small_nbt, p.small_ksteps, p.small_waves) && small_wg_count() >= 2) p.kind = kSmall;
  const int forced = g_forced_kind.load(std::memory_order_relaxed);
  if (forced == kGeneric) p.kind = kGeneric;
  if ((forced == kDma || (forced >= kForceDmaWholeTiles && forced <= kForceDmaThreeWBuffers)) && H % k2BK == 0) p.kind = kDma;
  if (forced == kForceDmaTwoWBuffers) p.dma_deep = 0;
  if (forced == kForceDmaThreeWBuffers && p.dma_nbt == 4) p.dma_deep = 2;
  if (p.kind == kSmall) {
    // One partial per (token, workgroup); one workgroup per CU, at most 512.
    p.bt = 64;
    p.slots = 1;     // only feed the schedule that the compaction kernel writes and this path ignores
    p.n_vunits = 1;
    p.upt = 1;
    p.grid = 0;
    p.max_records = (size_t)64 * 512;
    return p;
  }
  p.bt = p.kind == kGeneric ? kBT : dma_tile_tokens(p.dma_nbt);   // the DMA path: 256 vocab rows x 256, 128 or 64 tokens
  // resident workgroups on 256 CUs: 2 per CU, or 1 for the DMA path (80-128 KB of LDS; two 64-token workgroups of 80 KB
  // per CU measured slower than one: 288 against 277 us at 64 x 4096)
  p.slots = p.kind == kGeneric ? 512 : 256;
  // Vocab units.  Generic kernel: whole 256-row tiles.  DMA kernel with token tiles of 64 / 128: 32-row units (tile heights
  // are mixed inside the kernel).  DMA kernel with the 256-token tile: one tile height per launch - 256 rows, or 224 where
  // one round of workgroups streams W once and what counts is the longest vocab range in ROWS: whole 256-row tiles deal
  // V = 151936 as three tiles to 82 workgroups and two to the others, 224-row tiles as three to 167 and two to 89, an
  // eighth less for the longest.  The shorter tile moves 1/7 more hidden-state bytes per MAC, so it has to win by more
  // than that is worth (8 %), and it is only considered in the one-round regime.
  p.n_vunits = (int)((V + kBV - 1) / kBV);
  p.upt = 1;
  if (p.kind == kDma && forced != kForceDmaWholeTiles) {
    if (p.dma_nbt != 4) {
      p.unit32 = 1;
      p.n_vunits = (int)((V + 31) / 32);
      p.upt = 8;
    } else {
      const int tt = fused_ttiles((int)n_tokens, p.bt);
      if (tt * 8 <= 256) {
        const int sp = fused_one_round_splits(tt, 256, 1 << 30);
        auto longest_rows = [&](int rows) {
          const int64_t nvt = (V + rows - 1) / rows;
          const int64_t sv = sp < nvt ? sp : nvt;
          return ((nvt + sv - 1) / sv) * rows;
        };
        if (longest_rows(224) * 108 < longest_rows(256) * 100) {
          p.unit32 = 7;
          p.n_vunits = (int)((V + 223) / 224);
        }
      }
    }
  }
  p.grid = 0;
  p.max_records = 0;
  const int tt_max = (int)((n_tokens + p.bt - 1) / p.bt);
  for (int tt = 1; tt <= tt_max; ++tt) {  // the schedule depends on n_valid only through its tile count
    const FusedSchedule s = fused_schedule(tt * p.bt, p.bt, p.slots, p.n_vunits, p.upt);
    const int padded = 8 * ((s.n_wg + 7) / 8);  // fused_locate deals whole rows of 8 workgroup ids
    if (padded > p.grid) p.grid = padded;
    const size_t rec = (size_t)tt * p.bt * s.n_splits * kPartsPerSplit;
    if (rec > p.max_records) p.max_records = rec;
  }
  return p;
}

// Layout: [n_valid + schedule: 256 B][row_index: n_tokens int32, 256-aligned][partials per weight set]
// [normalised hidden rows, only with a norm weight].
static size_t off_index() { return 256; }
static size_t off_partials(int64_t n_tokens) { return 256 + (((size_t)n_tokens * 4 + 255) & ~(size_t)255); }
static size_t normed_bytes(int64_t n_tokens, int64_t H, bool with_norm) {
  return with_norm ? (((size_t)n_tokens * H * 2 + 255) & ~(size_t)255) : 0;
}
static size_t partial_bytes(int64_t n_tokens, int64_t H, int64_t V) {
  return fused_plan(n_tokens, H, V).max_records * sizeof(FusedPartial);
}

// The generic kernel addresses both matrices through buffer descriptors with 32-bit byte offsets.
bool fused_needs_32bit_extents(int64_t n_tokens, int64_t H, int64_t V) { return fused_plan(n_tokens, H, V).kind == kGeneric; }

size_t fused_workspace_bytes(int64_t n_tokens, int64_t H, int64_t V, int n_weights, bool with_norm) {
  return off_partials(n_tokens) + (size_t)n_weights * partial_bytes(n_tokens, H, V) + normed_bytes(n_tokens, H, with_norm);
}

template <bool ENT, bool AMAX, int NBT, int HI, bool DEEP = false, bool WNT = false>
static void launch_dma_nbt(const FusedArgs& a, int grid, hipStream_t stream) {
  static DeviceOnce attr_set;  // opt in to > 64 KB of dynamic LDS once per instantiation and device
  if (attr_set.first_on_current_device() &&
      !allow_big_lds(&fused_lmhead_dma_kernel<ENT, AMAX, NBT, HI, DEEP, WNT>, dma_lds_bytes(NBT, DEEP)) && DEEP) {
    int dev = 0;
    if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < kMaxDeviceOrdinals)
      g_no_deep_lds.fetch_or(1ull << dev, std::memory_order_relaxed);
  }
  if constexpr (DEEP) {
    if (deep_lds_refused()) return launch_dma_nbt<ENT, AMAX, NBT, HI, false>(a, grid, stream);
  }
  hipLaunchKernelGGL((fused_lmhead_dma_kernel<ENT, AMAX, NBT, HI, DEEP, WNT>), dim3((unsigned)grid), dim3(k2WG),
                     dma_lds_bytes(NBT, DEEP), stream, a);
}
// w_nt: non-temporal W requests (the kernel's WNT).
template <bool ENT, bool AMAX>
static void launch_dma(const FusedArgs& a, int nbt, int unit32, bool deep, bool w_nt, int grid, hipStream_t stream) {
  if (nbt == 4 && deep && w_nt) {
    if (unit32 == 7) launch_dma_nbt<ENT, AMAX, 4, 3, true, true>(a, grid, stream);
    else launch_dma_nbt<ENT, AMAX, 4, 4, true, true>(a, grid, stream);
  } else if (nbt == 4 && unit32 == 7 && deep) launch_dma_nbt<ENT, AMAX, 4, 3, true>(a, grid, stream);
  else if (nbt == 4 && deep) launch_dma_nbt<ENT, AMAX, 4, 4, true>(a, grid, stream);
  else if (nbt == 4 && unit32 == 7) launch_dma_nbt<ENT, AMAX, 4, 3>(a, grid, stream);   // 224-row tiles
  else if (nbt == 4) launch_dma_nbt<ENT, AMAX, 4, 4>(a, grid, stream);
  else if (nbt == 2 && w_nt) launch_dma_nbt<ENT, AMAX, 2, 0, false, true>(a, grid, stream);
  else if (nbt == 2) launch_dma_nbt<ENT, AMAX, 2, 0>(a, grid, stream);
  else if (w_nt) launch_dma_nbt<ENT, AMAX, 1, 0, false, true>(a, grid, stream);
  else launch_dma_nbt<ENT, AMAX, 1, 0>(a, grid, stream);
}

template <bool ENT, bool AMAX, int NBT, int KSTEPS>
static int launch_small(const FusedArgs& a, int waves, hipStream_t stream) {
  int n_wg = small_wg_count();
  const int n_tiles = (a.V + 15) / 16;
  if (n_wg > n_tiles) n_wg = n_tiles & ~1;  // no empty vocab ranges
  if (n_wg < 2) return 0;
  const size_t lds = (size_t)2 * waves * NBT * 1024 + (size_t)waves * 4096;
  static DeviceOnce attr_set;  // opt in to > 64 KB of dynamic LDS once per instantiation and device
  if (lds > 65536 && attr_set.first_on_current_device())
    allow_big_lds(&fused_lmhead_small_kernel<ENT, AMAX, NBT, KSTEPS>, 2 * 8 * 4 * 1024 + 8 * 4096);
  hipLaunchKernelGGL((fused_lmhead_small_kernel<ENT, AMAX, NBT, KSTEPS>), dim3((unsigned)n_wg), dim3((unsigned)waves * 64),
                     lds, stream, a);
  return n_wg;
}

// Launches the sweep kernel of `plan`.  Returns the number of partials per token it leaves (0 = the
// schedule's own count).
template <bool ENT>
static int launch_main(const FusedArgs& a, const FusedPlan& plan, bool want_argmax, hipStream_t stream) {
  if (plan.kind == kSmall) {
    int n = 0;
    const int w = plan.small_waves;
#define TOME_SMALL(NBT, KS)                                                 \
  n = want_argmax ? launch_small<ENT, true, NBT, KS>(a, w, stream) : launch_small<ENT, false, NBT, KS>(a, w, stream)
    if (plan.small_ksteps == 8 && plan.small_nbt == 1) TOME_SMALL(1, 8);
    else if (plan.small_ksteps == 8) TOME_SMALL(4, 8);
    else if (plan.small_nbt == 1) TOME_SMALL(1, 16);
    else TOME_SMALL(2, 16);
#undef TOME_SMALL
    return n;  // >= 2: fused_plan only picks this kernel when it can be placed
  }
  if (plan.kind == kDma) {
    if (want_argmax) launch_dma<ENT, true>(a, plan.dma_nbt, plan.unit32, plan.dma_deep >= (ENT ? 2 : 1), plan.w_nt, plan.grid, stream);
    else launch_dma<ENT, false>(a, plan.dma_nbt, plan.unit32, plan.dma_deep >= (ENT ? 2 : 1), plan.w_nt, plan.grid, stream);
  } else {
    if (want_argmax) hipLaunchKernelGGL((fused_lmhead_kernel<ENT, true>), dim3((unsigned)plan.grid), dim3(kFusedWG), 0, stream, a);
    else hipLaunchKernelGGL((fused_lmhead_kernel<ENT, false>), dim3((unsigned)plan.grid), dim3(kFusedWG), 0, stream, a);
  }
  return 0;
}

// One sweep per (hidden, weight) pair: the policy pair always, and a reference pair when a second weight
// set (`w1`) or a second hidden-state matrix (`hidden_ref`) is given; either may repeat the policy's.
static hipError_t fused_launch_impl(const void* hidden, const void* hidden_ref, const void* norm_weight,
                                    float norm_eps, const void* w0, const void* w1, int64_t n_tokens, int64_t H,
                                    int64_t V, int64_t hidden_stride, int64_t weight_stride, const int32_t* targets,
                                    const int32_t* row_valid, float temperature, float* out_lp, float* out_lse,
                                    float* out_entropy, int32_t* out_argmax, float* out_ref_lp, float* out_k3,
                                    void* workspace, hipStream_t stream) {
  const bool second = w1 != nullptr || hidden_ref != nullptr;
  if (!w1) w1 = w0;
  if (!hidden_ref) hidden_ref = hidden;
  char* ws = static_cast<char*>(workspace);
  const FusedPlan plan = fused_plan(n_tokens, H, V);
  int32_t* n_valid = nullptr;
  int32_t* row_index = nullptr;
  if (row_valid) {
    n_valid = reinterpret_cast<int32_t*>(ws);
    row_index = reinterpret_cast<int32_t*>(ws + off_index());
    CompactArgs c{row_valid, row_index, n_valid, out_lp, out_lse, out_entropy, out_ref_lp, out_k3, out_argmax,
                  (int)n_tokens, plan.bt, plan.slots, plan.n_vunits, plan.upt};
    hipLaunchKernelGGL(compact_rows_kernel, dim3(1), dim3(1024), 0, stream, c);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  FusedArgs a;
  a.hidden = static_cast<const char*>(hidden);
  a.targets = targets;
  a.row_index = row_index;
  a.hidden_index = row_index;
  a.n_valid = n_valid;
  a.hidden_stride_b = (uint32_t)(hidden_stride * 2);
  a.weight_stride_b = (uint32_t)(weight_stride * 2);
  a.hidden_bytes = (uint32_t)(((n_tokens - 1) * hidden_stride + H) * 2);  // read by the generic kernel only (< 4 GiB there)
  const char* second_hidden = static_cast<const char*>(hidden_ref);
  if (norm_weight) {  // normalise the valid rows into a dense buffer and multiply that
    char* normed = ws + off_partials(n_tokens) + (second ? 2 : 1) * partial_bytes(n_tokens, H, V);
    NormArgs na{a.hidden, static_cast<const uint16_t*>(norm_weight), normed, row_index, n_valid,
                a.hidden_stride_b, (int)n_tokens, (int)H, norm_eps};
    hipLaunchKernelGGL(rmsnorm_rows_kernel, dim3((unsigned)((n_tokens + 3) / 4)), dim3(256), 0, stream, na);
    if (hidden_ref != hidden) {
      na.x = static_cast<const char*>(hidden_ref);
      na.y = normed + normed_bytes(n_tokens, H, true);
      hipLaunchKernelGGL(rmsnorm_rows_kernel, dim3((unsigned)((n_tokens + 3) / 4)), dim3(256), 0, stream, na);
      second_hidden = na.y;
    } else {
      second_hidden = normed;
    }
    a.hidden = normed;
    a.hidden_index = nullptr;
    a.hidden_stride_b = (uint32_t)(H * 2);
    a.hidden_bytes = (uint32_t)(n_tokens * H * 2);
  }
  a.n_tokens = (int)n_tokens;
  a.H = (int)H;
  a.V = (int)V;
  a.n_vunits = plan.n_vunits;
  a.unit32 = plan.unit32;
  a.slots = plan.slots;
  // Workspace header: [0] n_valid, [16..32) the schedule derived from it on the device.
  a.sched_dev = row_valid ? reinterpret_cast<const FusedSchedule*>(n_valid + 4) : nullptr;
  a.sched = fused_schedule((int)n_tokens, plan.bt, plan.slots, plan.n_vunits, plan.upt);
  a.scale = kLog2e / temperature;
  FusedPartial* p0 = reinterpret_cast<FusedPartial*>(ws + off_partials(n_tokens));
  FusedPartial* p1 = reinterpret_cast<FusedPartial*>(ws + off_partials(n_tokens) + partial_bytes(n_tokens, H, V));

  a.weight = static_cast<const char*>(w0);
  a.partials = p0;
  int n_parts = out_entropy ? launch_main<true>(a, plan, out_argmax != nullptr, stream)
                            : launch_main<false>(a, plan, out_argmax != nullptr, stream);
  if (n_parts > 0) {  // small-batch kernel: one part per workgroup, whatever the mask
    a.sched = FusedSchedule{1, n_parts / kPartsPerSplit, n_parts, 0};
    a.sched_dev = nullptr;
  }
  const char* first_hidden = a.hidden;
  if (second) {
    a.weight = static_cast<const char*>(w1);
    a.hidden = second_hidden;
    a.partials = p1;
    launch_main<false>(a, plan, false, stream);
    a.hidden = first_hidden;
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;

  CombineArgs c;
  c.partials = p0;
  c.partials_ref = second ? p1 : nullptr;
  c.row_index = row_index;
  c.n_valid = n_valid;
  c.out_lp = out_lp;
  c.out_lse = out_lse;
  c.out_entropy = out_entropy;
  c.out_ref_lp = out_ref_lp;
  c.out_k3 = out_k3;
  c.out_argmax = out_argmax;
  c.n_tokens = (int)n_tokens;
  c.sched_dev = a.sched_dev;
  c.sched = a.sched;
  c.scale = a.scale;
  hipLaunchKernelGGL(fused_combine_kernel, dim3((unsigned)((n_tokens + 3) / 4)), dim3(256), 0, stream, c);
  return hipGetLastError();
}

hipError_t fused_lmhead_launch(const void* hidden, const void* norm_weight, float norm_eps, const void* w0,
                               const void* w1, int64_t n_tokens, int64_t H, int64_t V, int64_t hidden_stride,
                               int64_t weight_stride, const int32_t* targets,
                               const int32_t* row_valid, float temperature, float* out_lp, float* out_lse,
                               float* out_entropy, int32_t* out_argmax, float* out_ref_lp, float* out_k3,
                               void* workspace, hipStream_t stream) {
  return fused_launch_impl(hidden, nullptr, norm_weight, norm_eps, w0, w1, n_tokens, H, V, hidden_stride, weight_stride,
                           targets, row_valid, temperature, out_lp, out_lse, out_entropy, out_argmax, out_ref_lp, out_k3,
                           workspace, stream);
}

hipError_t fused_pair_launch(const void* hidden, const void* hidden_ref, const void* norm_weight, float norm_eps,
                             const void* w0, const void* w1, int64_t n_tokens, int64_t H, int64_t V,
                             int64_t hidden_stride, int64_t weight_stride, const int32_t* targets,
                             const int32_t* row_valid, float temperature, float* out_lp, float* out_entropy,
                             float* out_ref_lp, float* out_k3, void* workspace, hipStream_t stream) {
  return fused_launch_impl(hidden, hidden_ref, norm_weight, norm_eps, w0, w1, n_tokens, H, V, hidden_stride,
                           weight_stride, targets, row_valid, temperature, out_lp, nullptr, out_entropy, nullptr,
                           out_ref_lp, out_k3, workspace, stream);
}

}  // namespace tome
