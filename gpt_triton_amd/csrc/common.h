// Shared device/host helpers for the gfx950 kernels of libgptmi.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

namespace gptmi {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
typedef uint32_t u2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

// Sum / max over the 64 lanes of a wavefront; every lane gets the result.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}

// tanh-form GELU of the reference (kernels.py:15-26): 0.5 x (1 + tanh(u)) with
// tanh(u) = 2 sigmoid(2u) - 1, u = sqrt(2/pi) (x + 0.044715 x^3).  Algebraically
// that is x * sigmoid(2u) = x / (1 + exp(-2u)); evaluated here as one exp2 and
// one hardware reciprocal (1 ulp), ~1e-7 relative from the reference's form.
__device__ __forceinline__ float gelu_new(float x) {
  // -2 * sqrt(2/pi) * log2(e)
  const float k = -2.0f * 0.7978845608028654f * 1.4426950408889634f;
  const float inner = x * fmaf(0.044715f, x * x, 1.0f);
  const float e = __builtin_amdgcn_exp2f(k * inner);
  return x * __builtin_amdgcn_rcpf(1.0f + e);
}

void set_error(const char* fmt, ...);

}  // namespace gptmi
