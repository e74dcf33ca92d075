// Matrix-pipe probe: a loop of nothing but MFMAs (optionally fed by LDS fragment reads at the
// GEMM kernels' ratio), used by the benchmark to measure what the chip sustains on a given kind
// of operand data -- the clock it holds under full matrix load depends on how many bits toggle.
// Not part of the forward path; it writes nothing.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "common.h"
#include "launch.h"

namespace gptmi {
namespace {

// One workgroup of 8 wavefronts per CU, 2 per SIMD, each with the register footprint of a GEMM
// wavefront: 128 accumulator registers (a 64 x 128 sub-tile) and the 12 operand fragments of two
// 32-wide k-steps.  SHAPE 32: v_mfma_f32_32x32x16_f16 (8 blocks of 32 x 32, two k16 slices per
// k-step), SHAPE 16: v_mfma_f32_16x16x32_f16 (32 blocks of 16 x 16).  Both do 2^18 MACs per k-step
// and wavefront.  LDS: the fragments of the next k-step are read from the wavefront's own 12 KB of
// LDS (the operand values, stored once in front of the loop), one 16-byte read per lane behind
// every second (SHAPE 16) MFMA, as the streaming GEMM kernels do.
template <int SHAPE, bool LDS>
__global__ __launch_bounds__(512, 2) void mfma_probe_kernel(const h8* __restrict__ src,
                                                            float* __restrict__ sink, int ksteps) {
  __shared__ h8 frag_lds[LDS ? 8 * 12 * 64 : 1];
  const int tid = blockIdx.x * 512 + threadIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  h8 f[2][12];
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int i = 0; i < 12; ++i) f[s][i] = src[(size_t)(tid * 24 + s * 12 + i) & ((1u << 20) - 1)];
  unsigned lds_addr = 0;
  if constexpr (LDS) {
    h8* mine = frag_lds + wave * (12 * 64);
#pragma unroll
    for (int i = 0; i < 12; ++i) mine[i * 64 + lane] = f[0][i];
    lds_addr = (unsigned)(uintptr_t)(mine + lane);
    __syncthreads();
  }
  // the next k-step's fragment rd into the other register set (same values every time)
  auto refill = [&](int s, int rd) __attribute__((always_inline)) {
    if constexpr (LDS) {
      __builtin_amdgcn_sched_barrier(0);
      asm volatile("ds_read_b128 %0, %1" : "=v"(f[s ^ 1][rd]) : "v"(lds_addr + rd * 1024));
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto landed = [&](int s) __attribute__((always_inline)) {
    if constexpr (LDS)
      asm volatile("s_waitcnt lgkmcnt(0)"
                   : "+v"(f[s ^ 1][0]), "+v"(f[s ^ 1][1]), "+v"(f[s ^ 1][2]), "+v"(f[s ^ 1][3]),
                     "+v"(f[s ^ 1][4]), "+v"(f[s ^ 1][5]), "+v"(f[s ^ 1][6]), "+v"(f[s ^ 1][7]),
                     "+v"(f[s ^ 1][8]), "+v"(f[s ^ 1][9]), "+v"(f[s ^ 1][10]), "+v"(f[s ^ 1][11]));
  };
  float total = 0.f;
  if constexpr (SHAPE == 32) {
    f16v acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    for (int it = 0; it < ksteps; it += 2) {
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        int rd = 0;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)  // a = f[s][6 ks + 0..1], b = f[s][6 ks + 2..5]
#pragma unroll
          for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
              const int j = (i & 1) ? 1 - jj : jj;  // one operand changes per MFMA
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f[s][6 * ks + 2 + i],
                                                                 f[s][6 * ks + j], acc[i][j], 0, 0, 0);
              if (rd < 12) refill(s, rd++);
            }
        landed(s);
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) total += acc[i][j][r];
  } else {
    f4 acc[8][4];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;
    for (int it = 0; it < ksteps; it += 2) {
#pragma unroll
      for (int s = 0; s < 2; ++s) {  // a = f[s][0..3], b = f[s][4..11]
        int rd = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
          for (int jj = 0; jj < 4; ++jj) {
            const int j = (i & 1) ? 3 - jj : jj;
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(f[s][4 + i], f[s][j], acc[i][j], 0, 0, 0);
            if ((jj & 1) && rd < 12) refill(s, rd++);
          }
        landed(s);
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) total += acc[i][j][r];
  }
  // keeps the loop alive; never true for finite operands of the sizes the benchmark uses
  if (total == 12345.678f) sink[tid & 1023] = total;
}

}  // namespace

// `operands`: 16 MiB of fp16 values on the device; `sink`: 4 KiB.  2 * 2^18 * ksteps FLOP per
// wavefront, 8 wavefronts per workgroup, `workgroups` workgroups.
int launch_mfma_probe(int shape, bool lds_reads, const void* operands, void* sink, int ksteps,
                      int workgroups, hipStream_t st) {
  const h8* src = (const h8*)operands;
  float* out = (float*)sink;
  dim3 grid((unsigned)workgroups), block(512);
  if (shape == 32) {
    if (lds_reads) hipLaunchKernelGGL((mfma_probe_kernel<32, true>), grid, block, 0, st, src, out, ksteps);
    else hipLaunchKernelGGL((mfma_probe_kernel<32, false>), grid, block, 0, st, src, out, ksteps);
  } else if (shape == 16) {
    if (lds_reads) hipLaunchKernelGGL((mfma_probe_kernel<16, true>), grid, block, 0, st, src, out, ksteps);
    else hipLaunchKernelGGL((mfma_probe_kernel<16, false>), grid, block, 0, st, src, out, ksteps);
  } else {
    return -2;
  }
  return 0;
}

}  // namespace gptmi
