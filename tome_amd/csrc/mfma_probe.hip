// Measurement probe: what the matrix cores of this part sustain on the fused kernel's inner loop when
// nothing else is in the way.  One workgroup per CU runs the LDS -> MFMA loop of fused_lmhead_dma_kernel
// (8 waves as 2 x 4, 128 x 64 wave tiles of v_mfma_f32_16x16x32_bf16, twelve 16-byte fragment reads per 32
// MFMAs, the same XOR-swizzled slab layout) on operands that are loaded into LDS once: no global loads in the
// loop, no barrier, no epilogue.  With random bf16 operands the result is the ceiling that the power limit of
// the part puts on any bf16 GEMM of this tiling; with constant operands the same loop runs near the
// published peak, which shows that the loop itself is not what holds the random case back.
//
// Flag 1 (requests): every wave also issues the fused kernel's eight global -> LDS requests per K slab (1 KB each,
// re-reading the 64 KB operand buffer, which stays in the caches; the data lands in a second LDS region that is never
// read): what the fill costs by being issued and returned at all, apart from what the L2 side adds in the real kernel.
// Flag 2 (fold): after every 16 slabs (one vocab tile at K = 1024) the accumulators are folded into per-token online
// softmax statistics with the arithmetic of the fused kernel's epilogue (block maxima, one rescale, exp2 and add per
// element) and the next slab starts from a zero C operand.
// Flag 4 (barrier): the fused kernel's wait for its own LDS reads and the workgroup barrier in every step.
// All three together are the fused kernel at config 3 on a memory system that always answers from cache, without its
// address bookkeeping and its uneven last round of vocab tiles: the rate this design could reach at most.
//
// No counterpart in the reference (it has no matrix-core code); bench.py reports the figure next to the
// published peak as `sustained_peak`.
#include "common.hpp"

namespace tome {

typedef __bf16 probe_bf16x8 __attribute__((ext_vector_type(8)));
typedef float probe_f32x4 __attribute__((ext_vector_type(4)));

constexpr int kProbeWG = 512;
constexpr int kProbeSlabBytes = 512 * 128;  // 256 weight rows + 256 token rows, 64 bf16 each
constexpr int kProbeFoldEvery = 16;         // slabs per vocab tile at K = 1024

template <int N_MFMA, int N_READS>
__device__ __forceinline__ void probe_pair_reads() {
#pragma unroll
  for (int q = 0; q < N_READS; ++q) {
    __builtin_amdgcn_sched_group_barrier(0x008, N_MFMA, 0);  // MFMA
    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);       // DS read
  }
}

template <int N>
__device__ __forceinline__ void probe_pair_dma() {
#pragma unroll
  for (int q = 0; q < N; ++q) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
    __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // VMEM (DMA request)
  }
}

__device__ __forceinline__ float probe_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

template <bool REQ, bool FOLD, bool BAR>
__global__ __launch_bounds__(kProbeWG) void mfma_ceiling_kernel(const u32x4* operands, int steps, float* sink) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
#pragma unroll
  for (int i = 0; i < kProbeSlabBytes / 16 / kProbeWG; ++i)
    reinterpret_cast<u32x4*>(smem)[tid + i * kProbeWG] = operands[tid + i * kProbeWG];
  __syncthreads();

  const int wave_v = wave & 1, wave_t = wave >> 1;
  const int l16 = lane & 15, g = lane >> 4;
  const int swz = (g ^ ((l16 >> 1) & 7)) * 16;
  const int rdA = (wave_v * 128 + l16) * 128 + swz;
  const int rdB = 256 * 128 + (wave_t * 64 + l16) * 128 + swz;
  auto read_a = [&](int ks, int i0, probe_bf16x8 (&fa)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) fa[i] = *reinterpret_cast<const probe_bf16x8*>(smem + (rdA ^ (ks * 64)) + (i0 + i) * 16 * 128);
  };
  auto read_b = [&](int ks, probe_bf16x8 (&fb)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) fb[j] = *reinterpret_cast<const probe_bf16x8*>(smem + (rdB ^ (ks * 64)) + j * 16 * 128);
  };

  probe_f32x4 acc[8][4];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = probe_f32x4{0.f, 0.f, 0.f, 0.f};
  probe_bf16x8 fa_lo[4], fa_hi[4], fb0[4], fb1[4];
  read_a(0, 0, fa_lo);
  read_b(0, fb0);
  auto mfma_half = [&](int i0, probe_bf16x8 (&fa)[4], probe_bf16x8 (&fb)[4], auto fresh) {
    const probe_f32x4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[i0 + i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[i], fb[j], decltype(fresh)::value ? zero : acc[i0 + i][j], 0, 0, 0);
  };
  float run_mx[4], run_s[4];  // FOLD: per-lane online softmax state, one token per block column
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    run_mx[j] = -1.0e30f;
    run_s[j] = 0.f;
  }
  const float scale = 1.44269504f;
  auto fold = [&]() {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      __builtin_amdgcn_sched_barrier(0);
      float cm = run_mx[j];
#pragma unroll
      for (int i = 0; i < 8; ++i)
        cm = fmaxf(cm, fmaxf(fmaxf(acc[i][j][0], acc[i][j][1]), fmaxf(acc[i][j][2], acc[i][j][3])));
      const float resc = probe_exp2((run_mx[j] - cm) * scale);
      const float m = cm * scale;
      float s0 = run_s[j] * resc, s1 = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int e = 0; e < 4; e += 2) {
          s0 += probe_exp2(fmaf(acc[i][j][e], scale, -m));
          s1 += probe_exp2(fmaf(acc[i][j][e + 1], scale, -m));
        }
      run_mx[j] = cm;
      run_s[j] = s0 + s1;
    }
  };
  // Requests (REQ): piece p of a wave fetches 1 KB of the operand buffer into the second 64 KB of LDS, 4 + 2 + 2 per
  // step in the quarters where the fused kernel issues them, at most one slab's worth in flight.
  const char* req_src = reinterpret_cast<const char*>(operands) + wave * 8192 + lane * 16;
  char* req_dst = smem + kProbeSlabBytes + wave * 1024;
  auto request = [&](int piece) {
    __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint32_t*>(req_src + piece * 1024),
                                     (__attribute__((address_space(3))) uint32_t*)(req_dst + piece * 8192), 16, 0, 0);
  };
  auto do_step = [&](auto fresh) {  // one step = one 64-wide K slab = 64 MFMAs per wave
    __builtin_amdgcn_sched_barrier(0);
    read_a(0, 4, fa_hi);
    if constexpr (REQ) {
      request(4);
      request(5);
    }
    mfma_half(0, fa_lo, fb0, fresh);
    probe_pair_reads<2, 4>();
    if constexpr (REQ) probe_pair_dma<2>();
    __builtin_amdgcn_sched_barrier(0);
    read_a(1, 0, fa_lo);
    read_b(1, fb1);
    if constexpr (REQ) {
      request(6);
      request(7);
    }
    mfma_half(4, fa_hi, fb0, fresh);
    if constexpr (REQ) {
      probe_pair_reads<1, 8>();
      probe_pair_dma<2>();
    } else {
      probe_pair_reads<2, 8>();
    }
    __builtin_amdgcn_sched_barrier(0);
    read_a(1, 4, fa_hi);
    mfma_half(0, fa_lo, fb1, std::false_type{});
    probe_pair_reads<2, 4>();
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (REQ) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the fused kernel's wait before its barrier
    if constexpr (BAR) {
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
    }
    read_a(0, 0, fa_lo);
    read_b(0, fb0);
    if constexpr (REQ) {
      request(0);
      request(1);
      request(2);
      request(3);
    }
    mfma_half(4, fa_hi, fb1, std::false_type{});
    if constexpr (REQ) {
      probe_pair_reads<1, 8>();
      probe_pair_dma<4>();
    } else {
      probe_pair_reads<2, 8>();
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  if constexpr (FOLD) {
    for (int t = 0; t < steps / kProbeFoldEvery; ++t) {
      do_step(std::true_type{});
      for (int k = 1; k < kProbeFoldEvery; ++k) do_step(std::false_type{});
      fold();
    }
  } else {
    for (int s = 0; s < steps; ++s) do_step(std::false_type{});
  }
  if constexpr (REQ) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no request may outlive the workgroup's LDS
  float total = 0.f;
  if constexpr (FOLD) {
#pragma unroll
    for (int j = 0; j < 4; ++j) total += run_mx[j] + run_s[j];
  }
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) total += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3];
  sink[(size_t)blockIdx.x * kProbeWG + tid] = total;
}

// `operands`: 64 KB of bf16 (device), `sink`: n_workgroups * 512 floats (device).  FLOP of one launch:
// n_workgroups * steps * 2 * 256 * 256 * 64.
template <bool REQ, bool FOLD, bool BAR>
static void mfma_probe_launch_one(const void* operands, int n_workgroups, int steps, float* sink, hipStream_t stream) {
  constexpr int lds = (REQ ? 2 : 1) * kProbeSlabBytes;
  static DeviceOnce attr_set;  // opt in to the large dynamic LDS once per instantiation and device
  if (attr_set.first_on_current_device())
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&mfma_ceiling_kernel<REQ, FOLD, BAR>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, lds);
  hipLaunchKernelGGL((mfma_ceiling_kernel<REQ, FOLD, BAR>), dim3((unsigned)n_workgroups), dim3(kProbeWG), lds, stream,
                     static_cast<const u32x4*>(operands), steps, sink);
}

// flags: 1 = with the fill requests, 2 = with the softmax fold every 16 slabs (steps is then rounded down to whole tiles),
// 4 = with the fused kernel's workgroup barrier in every step.
hipError_t mfma_probe_launch(const void* operands, int n_workgroups, int steps, int flags, float* sink, hipStream_t stream) {
  switch (flags & 7) {
    case 0: mfma_probe_launch_one<false, false, false>(operands, n_workgroups, steps, sink, stream); break;
    case 1: mfma_probe_launch_one<true, false, false>(operands, n_workgroups, steps, sink, stream); break;
    case 2: mfma_probe_launch_one<false, true, false>(operands, n_workgroups, steps, sink, stream); break;
    case 3: mfma_probe_launch_one<true, true, false>(operands, n_workgroups, steps, sink, stream); break;
    case 4: mfma_probe_launch_one<false, false, true>(operands, n_workgroups, steps, sink, stream); break;
    case 5: mfma_probe_launch_one<true, false, true>(operands, n_workgroups, steps, sink, stream); break;
    case 6: mfma_probe_launch_one<false, true, true>(operands, n_workgroups, steps, sink, stream); break;
    default: mfma_probe_launch_one<true, true, true>(operands, n_workgroups, steps, sink, stream); break;
  }
  return hipGetLastError();
}

}  // namespace tome
