// Measurement probe: what the matrix cores of this part sustain on the fused kernel's inner loop when
// nothing else is in the way.  One workgroup per CU runs the LDS -> MFMA loop of fused_lmhead_dma_kernel
// (8 waves as 2 x 4, 128 x 64 wave tiles of v_mfma_f32_16x16x32_bf16, twelve 16-byte fragment reads per 32
// MFMAs, the same XOR-swizzled slab layout) on operands that are loaded into LDS once: no global loads in the
// loop, no barrier, no epilogue.  With random bf16 operands the result is the ceiling that the power limit of
// the part puts on any bf16 GEMM of this tiling; with constant operands the same loop runs near the
// published peak, which shows that the loop itself is not what holds the random case back.
//
// With `with_requests` every wave also issues the fused kernel's eight global -> LDS requests per K slab (1 KB each,
// re-reading the 64 KB operand buffer, which stays in the caches; the data lands in a second LDS region that is never
// read): what the fill costs by being issued and returned at all, apart from what the L2 side adds in the real kernel.
//
// No counterpart in the reference (it has no matrix-core code); bench.py reports the figure next to the
// published peak as `sustained_peak`.
#include "common.hpp"

namespace tome {

typedef __bf16 probe_bf16x8 __attribute__((ext_vector_type(8)));
typedef float probe_f32x4 __attribute__((ext_vector_type(4)));

constexpr int kProbeWG = 512;
constexpr int kProbeSlabBytes = 512 * 128;  // 256 weight rows + 256 token rows, 64 bf16 each

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

template <bool REQ>
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
  auto mfma_half = [&](int i0, probe_bf16x8 (&fa)[4], probe_bf16x8 (&fb)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i0 + i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[i], fb[j], acc[i0 + i][j], 0, 0, 0);
  };
  // Requests (REQ): piece p of a wave fetches 1 KB of the operand buffer into the second 64 KB of LDS, 4 + 2 + 2 per
  // step in the quarters where the fused kernel issues them, at most one slab's worth in flight.
  const char* req_src = reinterpret_cast<const char*>(operands) + wave * 8192 + lane * 16;
  char* req_dst = smem + kProbeSlabBytes + wave * 1024;
  auto request = [&](int piece) {
    __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint32_t*>(req_src + piece * 1024),
                                     (__attribute__((address_space(3))) uint32_t*)(req_dst + piece * 8192), 16, 0, 0);
  };
  for (int s = 0; s < steps; ++s) {  // one step = one 64-wide K slab = 64 MFMAs per wave
    __builtin_amdgcn_sched_barrier(0);
    read_a(0, 4, fa_hi);
    if constexpr (REQ) {
      request(4);
      request(5);
    }
    mfma_half(0, fa_lo, fb0);
    probe_pair_reads<2, 4>();
    if constexpr (REQ) probe_pair_dma<2>();
    __builtin_amdgcn_sched_barrier(0);
    read_a(1, 0, fa_lo);
    read_b(1, fb1);
    if constexpr (REQ) {
      request(6);
      request(7);
    }
    mfma_half(4, fa_hi, fb0);
    if constexpr (REQ) {
      probe_pair_reads<1, 8>();
      probe_pair_dma<2>();
    } else {
      probe_pair_reads<2, 8>();
    }
    __builtin_amdgcn_sched_barrier(0);
    read_a(1, 4, fa_hi);
    mfma_half(0, fa_lo, fb1);
    probe_pair_reads<2, 4>();
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (REQ) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the fused kernel's wait before its barrier
    read_a(0, 0, fa_lo);
    read_b(0, fb0);
    if constexpr (REQ) {
      request(0);
      request(1);
      request(2);
      request(3);
    }
    mfma_half(4, fa_hi, fb1);
    if constexpr (REQ) {
      probe_pair_reads<1, 8>();
      probe_pair_dma<4>();
    } else {
      probe_pair_reads<2, 8>();
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  if constexpr (REQ) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no request may outlive the workgroup's LDS
  float total = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) total += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3];
  sink[(size_t)blockIdx.x * kProbeWG + tid] = total;
}

// `operands`: 64 KB of bf16 (device), `sink`: n_workgroups * 512 floats (device).  FLOP of one launch:
// n_workgroups * steps * 2 * 256 * 256 * 64.
hipError_t mfma_probe_launch(const void* operands, int n_workgroups, int steps, int with_requests, float* sink,
                             hipStream_t stream) {
  static bool attr_set = false;  // opt in to the large dynamic LDS once
  if (!attr_set) {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&mfma_ceiling_kernel<false>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, kProbeSlabBytes);
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&mfma_ceiling_kernel<true>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, 2 * kProbeSlabBytes);
    attr_set = true;
  }
  if (with_requests)
    hipLaunchKernelGGL(mfma_ceiling_kernel<true>, dim3((unsigned)n_workgroups), dim3(kProbeWG), 2 * kProbeSlabBytes, stream,
                       static_cast<const u32x4*>(operands), steps, sink);
  else
    hipLaunchKernelGGL(mfma_ceiling_kernel<false>, dim3((unsigned)n_workgroups), dim3(kProbeWG), kProbeSlabBytes, stream,
                       static_cast<const u32x4*>(operands), steps, sink);
  return hipGetLastError();
}

}  // namespace tome
