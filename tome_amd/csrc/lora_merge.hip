// policy_W = base_W + scale * (lora_B @ lora_A) for a batch of weight matrices in ONE launch
// (mlx-impl/node.py:102-164, UpdateWeights).  Every tensor is bf16 and every intermediate is rounded
// to bf16 where the reference's array expressions round it:
//     d  = bf16(lora_B @ lora_A)        matmul, fp32 accumulate              (node.py:128)
//     d2 = bf16(bf16(scale) * d)        Python scalar times a bf16 array     (node.py:128)
//     W  = bf16(base + d2)              (node.py:137,146,149,151)
// The op reads base and writes W once each (4 bytes per element) against rank/2 flops per byte, so it
// is HBM-bound for every rank LoRA uses; the rank-r product rides on v_mfma_f32_16x16x32_bf16 so the
// vector ALU only does the three roundings.
//
// Work split.  A workgroup (4 waves) owns a 512-column chunk and a span of 16-row tiles; wave w owns
// columns [128w, 128w+128) of the chunk as 8 MFMA tiles of 16 columns x 16 rows.  MFMA's M index
// carries COLUMNS (operand A = lora_A^T) and its N index ROWS (operand B = lora_B); the M index of tile
// (p, h) is mapped to column 32p + 8(m/4) + 4h + (m%4), so that lane (n, g) ends up with the 8
// contiguous columns 32p + 8g .. +7 of row n across the tile pair (p, 0), (p, 1).
//
// HBM access shape.  In that layout one wave instruction would touch 16 rows x 64 bytes; measured on
// this part a copy kernel with that shape moves 4.1-4.9 TB/s (read + write) against 5.6-6.4 TB/s for
// 4 rows x 256 bytes.  So base is loaded and W stored as 4 rows x 256 B per instruction, and the
// rounded deltas (packed bf16, 16 bytes per lane and pair) change layout through a wave-private 16 x 128
// LDS tile.  lora_A is transposed once by a prologue kernel into the workspace ([cols, 32 * K steps],
// zero padded), which turns the strided operand gather into one 16-byte load per fragment.
#include "common.hpp"

namespace tome {

constexpr int kLoraWG = 256;
constexpr int kLoraChunk = 512;   // columns per workgroup
constexpr int kLoraMaxJobs = 56;  // jobs per upload launch (kernel-argument space)

typedef short bf16x8 __attribute__((ext_vector_type(8)));

struct LoraJob {
  const char* base;
  char* out;
  const uint16_t* a;  // [rank, cols], or nullptr: W = bf16(base + 0)
  const uint16_t* b;  // [rows, rank]
  uint16_t* a_t;      // workspace: lora_A transposed, [cols, rank rounded up to 32]
  int rows, cols, rank;
  uint32_t base_stride_b, out_stride_b;
  float scale;       // already rounded to bf16
  int wg0;           // first workgroup of this job
  int tiles_per_wg;  // 16-row tiles each workgroup walks
};

// The job table lives in the workspace so that one launch serves any number of jobs; it gets there
// through kernel arguments (kLoraMaxJobs jobs per upload launch), which keeps the call asynchronous
// and free of host-to-device copies.
struct LoraUpload {
  LoraJob job[kLoraMaxJobs];
  LoraJob* table;
  int n_jobs;  // in this upload
  int first;   // table index of job[0]
};

static_assert(sizeof(LoraUpload) <= 4096, "kernel arguments are limited to 4 KB");

__global__ __launch_bounds__(256) void lora_upload_kernel(LoraUpload u) {
  constexpr int kWords = sizeof(LoraJob) / 4;
  const uint32_t* src = reinterpret_cast<const uint32_t*>(u.job);
  uint32_t* dst = reinterpret_cast<uint32_t*>(u.table + u.first);
  for (int i = threadIdx.x; i < u.n_jobs * kWords; i += 256) dst[i] = src[i];
}

struct LoraTable {
  const LoraJob* job;
  int n_jobs;
};

// Job owning workgroup `wg`: the last one whose wg0 is <= wg (uniform binary search, scalar loads).
__device__ __forceinline__ int lora_find_job(const LoraTable& tab, int wg) {
  int lo = 0, hi = tab.n_jobs - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (tab.job[mid].wg0 <= wg) lo = mid;
    else hi = mid - 1;
  }
  return lo;
}

constexpr int kLoraTileStride = 272;  // bytes per row of the LDS tile: 256 + 16 keeps the 16 rows on distinct banks

// a [rank, cols] -> a_t [cols, kp] (kp = rank rounded up to 32, zero filled): one lane per column, so that
// adjacent lanes read adjacent elements of a lora_A row and each lane writes one whole row of a_t.
__global__ __launch_bounds__(256) void lora_transpose_kernel(LoraTable tab) {
  const LoraJob job = tab.job[blockIdx.y];
  if (!job.a) return;
  const int kp = (job.rank + 31) & ~31;
  const int col = blockIdx.x * 256 + threadIdx.x;
  if (col >= job.cols) return;
  for (int c = 0; c < kp / 8; ++c) {
    uint32_t w[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int k = 8 * c + 2 * e;
      const uint32_t lo = k < job.rank ? job.a[(int64_t)k * job.cols + col] : 0u;
      const uint32_t hi = k + 1 < job.rank ? job.a[(int64_t)(k + 1) * job.cols + col] : 0u;
      w[e] = lo | (hi << 16);
    }
    *reinterpret_cast<u32x4*>(job.a_t + ((int64_t)col * kp + 8 * c)) = u32x4{w[0], w[1], w[2], w[3]};
  }
}

// bf16(scale * bf16(acc)) for two accumulators, packed.
__device__ __forceinline__ uint32_t delta_pair(float acc_lo, float acc_hi, float scale) {
  const uint32_t d = pack_bf16(acc_lo, acc_hi);
  return pack_bf16(scale * bf16_lo(d), scale * bf16_hi(d));
}
// bf16(base + delta) for two packed pairs.
__device__ __forceinline__ uint32_t add_pair(uint32_t base2, uint32_t delta2) {
  return pack_bf16(bf16_lo(base2) + bf16_lo(delta2), bf16_hi(base2) + bf16_hi(delta2));
}

template <int KSTEPS>
struct LoraTileLoads {
  bf16x8 fb[KSTEPS];  // lora_B fragments, MFMA layout
  u32x4 base[4];      // base, 4 rows x 256 B per instruction
};

template <int KSTEPS>
__device__ __forceinline__ void lora_issue_loads(const LoraJob& job, int rank, int t, int c0, int lane,
                                                 LoraTileLoads<KSTEPS>& L) {
  const int l16 = lane & 15, g = lane >> 4;
  const int row = t * 16 + l16;
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) {
    const int k = 32 * s + 8 * g;  // rank % 8 == 0: a lane's 8 K values are all inside or all outside
    u32x4 raw = {0u, 0u, 0u, 0u};
    if (row < job.rows && k < rank) raw = *reinterpret_cast<const u32x4*>(job.b + (int64_t)row * rank + k);
    L.fb[s] = __builtin_bit_cast(bf16x8, raw);
  }
  const int col = c0 + 8 * l16;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int r = t * 16 + 4 * q + g;
    L.base[q] = u32x4{0u, 0u, 0u, 0u};
    if (r < job.rows && col < job.cols)
      L.base[q] = __builtin_nontemporal_load(
          reinterpret_cast<const u32x4*>(job.base + (int64_t)r * job.base_stride_b + (int64_t)col * 2));
  }
}

template <int KSTEPS>
__global__ __launch_bounds__(kLoraWG) void lora_merge_kernel(LoraTable tab) {
  __shared__ __attribute__((aligned(16))) char tile_mem[4][16 * kLoraTileStride];
  const LoraJob job = tab.job[lora_find_job(tab, (int)blockIdx.x)];
  const int rank = job.a ? job.rank : 0;
  if (rank > 32 * KSTEPS) return;  // launched per K-step class; other classes handle this job
  if (KSTEPS > 1 && rank <= 16 * KSTEPS) return;

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int l16 = lane & 15, g = lane >> 4;
  const int n_chunks = (job.cols + kLoraChunk - 1) / kLoraChunk;
  const int local = (int)blockIdx.x - job.wg0;
  const int chunk = local % n_chunks, span = local / n_chunks;
  const int c0 = chunk * kLoraChunk + wave * 128;
  const int n_row_tiles = (job.rows + 15) / 16;
  const int t_begin = span * job.tiles_per_wg;
  const int t_end = min(t_begin + job.tiles_per_wg, n_row_tiles);
  if (t_begin >= t_end) return;

  LoraTileLoads<KSTEPS> cur, nxt;
  lora_issue_loads<KSTEPS>(job, rank, t_begin, c0, lane, cur);

  // lora_A^T fragments: tile (p, h), K step s, lane (m = l16, g) holds a_t[col(p, h, m)][32s + 8g .. +7].
  // Columns past the matrix are clamped: their results are never stored.
  bf16x8 fa[8][KSTEPS];
  const int kp = 32 * ((rank + 31) / 32);
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    const int col = min(c0 + 32 * (t >> 1) + 8 * (l16 >> 2) + 4 * (t & 1) + (l16 & 3), job.cols - 1);
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      u32x4 raw = {0u, 0u, 0u, 0u};
      if (32 * s < kp) raw = *reinterpret_cast<const u32x4*>(job.a_t + ((int64_t)col * kp + 32 * s + 8 * g));
      fa[t][s] = __builtin_bit_cast(bf16x8, raw);
    }
  }

  char* tile = tile_mem[wave];
  for (int t = t_begin; t < t_end; ++t) {
    if (t + 1 < t_end) lora_issue_loads<KSTEPS>(job, rank, t + 1, c0, lane, nxt);
    // deltas in MFMA layout -> LDS tile [16 rows][128 columns]
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) {
        acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[2 * p][s], cur.fb[s], acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[2 * p + 1][s], cur.fb[s], acc1, 0, 0, 0);
      }
      u32x4 d;
      d.x = delta_pair(acc0[0], acc0[1], job.scale);
      d.y = delta_pair(acc0[2], acc0[3], job.scale);
      d.z = delta_pair(acc1[0], acc1[1], job.scale);
      d.w = delta_pair(acc1[2], acc1[3], job.scale);
      *reinterpret_cast<u32x4*>(tile + l16 * kLoraTileStride + 64 * p + 16 * g) = d;
    }
    // The tile is private to this wave and LDS serves a wave's requests in order: a wave-level fence is enough.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int col = c0 + 8 * l16;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int r = t * 16 + 4 * q + g;
      const u32x4 d = *reinterpret_cast<const u32x4*>(tile + (4 * q + g) * kLoraTileStride + 16 * l16);
      u32x4 o;
      o.x = add_pair(cur.base[q].x, d.x);
      o.y = add_pair(cur.base[q].y, d.y);
      o.z = add_pair(cur.base[q].z, d.z);
      o.w = add_pair(cur.base[q].w, d.w);
      if (r < job.rows && col < job.cols)
        __builtin_nontemporal_store(
            o, reinterpret_cast<u32x4*>(job.out + (int64_t)r * job.out_stride_b + (int64_t)col * 2));
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  // the next tile's deltas overwrite what was just read
    __builtin_amdgcn_wave_barrier();
    cur = nxt;
  }
}

struct LoraJobHost {  // mirror of TomeLoraJob in include/tome_logprob.h
  const void* base;
  void* out;
  const void* lora_a;
  const void* lora_b;
  int64_t rows, cols, rank, base_stride, out_stride;
  float scale;
  int32_t reserved;
};

static float to_bf16_value(float f) {
  uint32_t u;
  __builtin_memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) <= 0x7f800000u) u += 0x7fffu + ((u >> 16) & 1u);
  u &= 0xffff0000u;
  __builtin_memcpy(&f, &u, 4);
  return f;
}

static size_t lora_a_t_bytes(const LoraJobHost& h) {
  if (!h.lora_a) return 0;
  const size_t kp = (size_t)((h.rank + 31) / 32) * 32;
  return ((size_t)h.cols * kp * 2 + 255) & ~(size_t)255;
}
static size_t lora_table_bytes(int n_jobs) { return ((size_t)n_jobs * sizeof(LoraJob) + 255) & ~(size_t)255; }

// Workspace: [job table][lora_A^T of every job that has one].
size_t lora_workspace_bytes(const LoraJobHost* jobs, int n_jobs) {
  size_t total = lora_table_bytes(n_jobs);
  for (int i = 0; i < n_jobs; ++i) total += lora_a_t_bytes(jobs[i]);
  return total;
}

hipError_t lora_merge_launch(const LoraJobHost* jobs, int n_jobs, void* workspace, hipStream_t stream) {
  // A workgroup walks a few row tiles so that the lora_A^T fragments (as many bytes per workgroup as a
  // row tile of base at rank <= 32, more above) are reused, but stays short: many small workgroups keep
  // more loads in flight.  Measured on Qwen3-0.6B's 84 matrices at rank 8: 1 tile 301 us, 2 tiles 276 us,
  // 4 tiles 290 us, 8 tiles 319 us; at rank 64 four tiles beat two (141 against 147 us for 151936 x 1024).
  int64_t units = 0;
  int64_t max_rank = 0;
  for (int i = 0; i < n_jobs; ++i) {
    units += ((jobs[i].rows + 15) / 16) * ((jobs[i].cols + kLoraChunk - 1) / kLoraChunk);
    if (jobs[i].lora_a && jobs[i].rank > max_rank) max_rank = jobs[i].rank;
  }
  const int tiles_per_wg = units < 2048 ? 1 : ((max_rank > 32 && units >= 8192) ? 4 : 2);
  LoraJob* table = static_cast<LoraJob*>(workspace);
  char* ws = static_cast<char*>(workspace) + lora_table_bytes(n_jobs);

  int wg = 0;
  int64_t transpose_lanes = 0;
  bool classes[3] = {false, false, false};  // K steps 1, 2, 4
  for (int first = 0; first < n_jobs; first += kLoraMaxJobs) {
    LoraUpload up;
    up.table = table;
    up.first = first;
    up.n_jobs = n_jobs - first < kLoraMaxJobs ? n_jobs - first : kLoraMaxJobs;
    for (int i = 0; i < up.n_jobs; ++i) {
      const LoraJobHost& h = jobs[first + i];
      LoraJob& d = up.job[i];
      d.base = static_cast<const char*>(h.base);
      d.out = static_cast<char*>(h.out);
      d.a = static_cast<const uint16_t*>(h.lora_a);
      d.b = static_cast<const uint16_t*>(h.lora_b);
      d.a_t = d.a ? reinterpret_cast<uint16_t*>(ws) : nullptr;
      ws += lora_a_t_bytes(h);
      d.rows = (int)h.rows;
      d.cols = (int)h.cols;
      d.rank = (int)h.rank;
      d.base_stride_b = (uint32_t)(h.base_stride * 2);
      d.out_stride_b = (uint32_t)(h.out_stride * 2);
      d.scale = to_bf16_value(h.scale);
      d.wg0 = wg;
      d.tiles_per_wg = tiles_per_wg;
      const int n_chunks = (d.cols + kLoraChunk - 1) / kLoraChunk;
      const int n_spans = ((d.rows + 15) / 16 + tiles_per_wg - 1) / tiles_per_wg;
      wg += n_chunks * n_spans;
      const int r = d.a ? d.rank : 0;
      classes[r <= 32 ? 0 : (r <= 64 ? 1 : 2)] = true;
      if (d.a && d.cols > transpose_lanes) transpose_lanes = d.cols;
    }
    hipLaunchKernelGGL(lora_upload_kernel, dim3(1), dim3(256), 0, stream, up);
  }
  if (wg == 0) return hipGetLastError();
  const LoraTable tab{table, n_jobs};
  if (transpose_lanes > 0)
    hipLaunchKernelGGL(lora_transpose_kernel, dim3((unsigned)((transpose_lanes + 255) / 256), (unsigned)n_jobs), dim3(256),
                       0, stream, tab);
  if (classes[0]) hipLaunchKernelGGL(lora_merge_kernel<1>, dim3((unsigned)wg), dim3(kLoraWG), 0, stream, tab);
  if (classes[1]) hipLaunchKernelGGL(lora_merge_kernel<2>, dim3((unsigned)wg), dim3(kLoraWG), 0, stream, tab);
  if (classes[2]) hipLaunchKernelGGL(lora_merge_kernel<4>, dim3((unsigned)wg), dim3(kLoraWG), 0, stream, tab);
  return hipGetLastError();
}

}  // namespace tome
