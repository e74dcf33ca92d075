// Host-side launchers implemented by the kernel translation units and called
// by the C ABI in capi.cpp.  All of them only enqueue work on `st`.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace gptmi {

// Dropout of one launch: probability p (0 = none) and the 64-bit seed of the generator.
struct Dropout {
  float p;
  uint64_t seed;
};

int launch_embed(const int64_t* ids, const void* wte, const void* wpe, void* out,
                 int64_t rows, int64_t L, int64_t V, int H, Dropout drop, bool f16, hipStream_t st);
bool launch_embed_layernorm(const int64_t* ids, const void* wte, const void* wpe, const void* w,
                            const void* b, void* emb, void* out, int64_t rows, int64_t L,
                            int64_t V, int H, float eps, bool f16, hipStream_t st);
int launch_layernorm(const void* x, const void* w, const void* b, void* out,
                     int64_t M, int H, float eps, bool f16, hipStream_t st);
int launch_softmax(const void* x, void* out, int64_t M, int H, bool f16,
                   hipStream_t st);
void launch_pack_rows(const void* src, void* dst, int64_t R, int K, int Kp, bool f16,
                      hipStream_t st);
void launch_pack_transpose(const void* src, void* dst, int K, int N, int Kp, bool f16,
                           hipStream_t st);

// Epilogue description of one GEMM launch: out = gelu?(acc + bias) + residual,
// stored either as a plain [M][N] matrix or scattered into q/k/v [B][heads][L][d].
struct GemmEpilogue {
  const void* bias;      // [N] in the storage dtype, or nullptr
  const void* residual;  // [M][N] in the storage dtype, or nullptr
  void* out;             // [M][N] (plain mode)
  void* q;               // qkv mode: three [B][heads][L][d] tensors
  void* k;
  void* v;
  int64_t L;      // qkv mode: rows per sequence
  int heads;      // qkv mode
  int d;          // qkv mode: head size
  int gelu;       // apply tanh-GELU after the bias
  Dropout drop;   // after the GELU, before the residual (plain mode only)
  bool qkv;       // scatter mode
  bool f16;       // storage dtype of bias / residual / outputs
};

// C[M][N] = A[M][Kp] . Bt[N][Kp]^T with fp16 operands (Kp % 64 == 0), fp32
// accumulation and the fused epilogue above.
int launch_gemm(const void* A, const void* Bt, int64_t M, int N, int Kp,
                const GemmEpilogue& ep, hipStream_t st);

// The same product with A = LayerNorm(x; ln_w, ln_b, eps), x [M][H] fp16 with H = K a multiple
// of 64: every workgroup normalises the rows of its tile in its operand prologue (the bits of
// launch_layernorm's output) and the normalised matrix never goes to memory.  fp16, no residual,
// no dropout; meant for few rows, where a LayerNorm launch costs more than normalising the rows
// once per column tile.  gemm_layernorm_supported says whether (M, H) is taken.
bool gemm_layernorm_supported(int64_t M, int H);
int launch_gemm_layernorm(const void* x, const void* ln_w, const void* ln_b, float eps,
                          const void* Bt, int64_t M, int N, int H, const GemmEpilogue& ep,
                          hipStream_t st);

// q, out: L rows per (batch, head); k, v: Lk rows.
int launch_flash_attn(const void* q, const void* k, const void* v, void* out,
                      int64_t B, int64_t N, int64_t L, int64_t Lk, int d, float scale,
                      Dropout drop, bool out_blnd, bool f16, hipStream_t st);

}  // namespace gptmi
