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
// The same over aligned groups of G lanes (G = 64: the wavefront; G = 32: each half on its own).
template <int G>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
  for (int o = G / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}
template <int G>
__device__ __forceinline__ float group_max(float v) {
#pragma unroll
  for (int o = G / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}

// tanh-form GELU of the reference (kernels.py:15-26): 0.5 x (1 + tanh(u)) with
// tanh(u) = 2 sigmoid(2u) - 1, u = sqrt(2/pi) (x + 0.044715 x^3).  Algebraically
// that is x * sigmoid(2u) = x / (1 + exp(-2u)); evaluated here as one exp2 and
// one hardware reciprocal (1 ulp), ~1e-7 relative from the reference's form.
__device__ __forceinline__ float gelu_new(float x) {
  // k = -2 * sqrt(2/pi) * log2(e), folded into the cubic's coefficients: exp(-2u) = exp2(x (k +
  // 0.044715 k x^2)) -- one multiplication fewer per element of a GELU epilogue
  constexpr float k = -2.0f * 0.7978845608028654f * 1.4426950408889634f;
  const float e = __builtin_amdgcn_exp2f(x * fmaf(0.044715f * k, x * x, k));
  return x * __builtin_amdgcn_rcpf(1.0f + e);
}

// ---------------------------------------------------------------------------
// Dropout of the reference (kernels.py:31-34): keep where tl.rand(seed, offset) > p, scaled
// by a true division by (1 - p).  tl.rand is Philox-4x32-10 with counter (offset, 0, 0, 0) and
// the 64-bit seed as key; the first output word, read as int32 with negatives folded by
// -x-1, times 4.6566127342e-10 gives the uniform in [0, 1).  NCH independent offsets share
// one rolled round loop so that a call site stays a few dozen instructions.
// ---------------------------------------------------------------------------
struct DropoutArgs {
  float p;
  unsigned seed_lo, seed_hi;
};

template <int NCH>
__device__ __forceinline__ void philox_uniform(const DropoutArgs& d, const unsigned (&offset)[NCH],
                                               float (&u)[NCH]) {
  unsigned c0[NCH], c1[NCH], c2[NCH], c3[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    c0[i] = offset[i];
    c1[i] = c2[i] = c3[i] = 0u;
  }
  unsigned k0 = d.seed_lo, k1 = d.seed_hi;
#pragma unroll 1
  for (int r = 0; r < 10; ++r) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const unsigned hb = __umulhi(0xCD9E8D57u, c2[i]), lb = 0xCD9E8D57u * c2[i];
      const unsigned ha = __umulhi(0xD2511F53u, c0[i]), la = 0xD2511F53u * c0[i];
      c0[i] = hb ^ c1[i] ^ k0;
      c2[i] = ha ^ c3[i] ^ k1;
      c1[i] = lb;
      c3[i] = la;
    }
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    int x = (int)c0[i];
    x = x < 0 ? -x - 1 : x;
    u[i] = (float)x * 4.6566127342e-10f;
  }
}

template <int NCH>
__device__ __forceinline__ void dropout_apply(const DropoutArgs& d, const unsigned (&offset)[NCH],
                                              float (&x)[NCH]) {
  float u[NCH];
  philox_uniform<NCH>(d, offset, u);
  const float keep_scale = 1.0f - d.p;
#pragma unroll
  for (int i = 0; i < NCH; ++i) x[i] = u[i] > d.p ? x[i] / keep_scale : 0.0f;
}

void set_error(const char* fmt, ...);

}  // namespace gptmi
