// The arithmetic of one LayerNorm row (reference: fused_layer_norm_kernel, kernels.py:104-145),
// in one place so that every kernel that normalises a row gives the same bits: the LayerNorm
// kernel, the embedding kernel that emits the first LayerNorm, and the GEMM whose operand
// prologue normalises its rows.
#pragma once
#include "common.h"

namespace gptmi {

// A row is spread over LPR lanes: lane l holds the 16-byte chunks l, l + LPR, ... (VN elements
// each, converted to fp32 in v, their sum in s, accumulated in that order).  fp32 mean, then the
// centred biased variance, then (x - mean) * rstd * w + b.  Contraction is spelled out (fmaf where a multiply-add is fused,
// none elsewhere): left to the compiler, two kernels were fused differently.
#pragma clang fp contract(off)
template <int CH, int VN, int LPR>
__device__ __forceinline__ void layernorm_stats(const float (&v)[CH][VN], float s, int lane,
                                                int nchunks, int H, float eps, float& mean,
                                                float& rstd) {
  mean = group_sum<LPR>(s) / (float)H;
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    if (lane + i * LPR < nchunks) {
#pragma unroll
      for (int j = 0; j < VN; ++j) {
        const float d = v[i][j] - mean;
        q = __builtin_fmaf(d, d, q);
      }
    }
  }
  const float var = group_sum<LPR>(q) / (float)H;
  rstd = 1.0f / sqrtf(var + eps);
}
__device__ __forceinline__ float layernorm_apply(float x, float mean, float rstd, float w, float b) {
  const float z = (x - mean) * rstd;
  float r = __builtin_fmaf(z, w, b);
  // The result is an fp32 number that the caller rounds to the storage type (the reference's
  // fp32 arithmetic followed by a cast).  Without this fence the compiler may merge the
  // multiply-add and the conversion into one mixed-precision instruction that rounds the exact
  // result once, straight to fp16 -- in some kernels and not in others.
  asm("" : "+v"(r));
  return r;
}
#pragma clang fp contract(fast)

// Lanes per row for rows of `nchunks` 16-byte chunks: 32 if that leaves fewer idle lane slots
// than 64 (96 chunks: 3 passes of 32 against 2 passes of 64 with a quarter empty).
inline int lanes_per_row(int nchunks) {
  const int slots32 = (nchunks + 31) / 32 * 32, slots64 = (nchunks + 63) / 64 * 64;
  return slots32 < slots64 ? 32 : 64;
}

}  // namespace gptmi
