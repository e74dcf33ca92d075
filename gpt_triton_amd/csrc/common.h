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

// tanh-form GELU exactly as the reference spells it (kernels.py:15-26):
// tanh(u) = 2*sigmoid(2u) - 1, a = sqrt(2/pi), b = x + 0.044715 x^3.
__device__ __forceinline__ float gelu_new(float x) {
  const float a = 0.7978845608028654f;
  const float b = x + 0.044715f * x * x * x;
  const float u = a * b;
  const float sig = 1.0f / (1.0f + __expf(-2.0f * u));
  const float t = 2.0f * sig - 1.0f;
  return 0.5f * x * (1.0f + t);
}

void set_error(const char* fmt, ...);

}  // namespace gptmi
