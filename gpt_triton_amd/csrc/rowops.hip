// Bandwidth-bound row kernels: embedding gather, LayerNorm, row softmax and the
// operand packers of the GEMM.  One wavefront owns one row; a row is held in
// registers between its passes so HBM sees one read and one write per element.
#include "common.h"
#include "layernorm.h"
#include "launch.h"

namespace gptmi {

template <typename T> struct Vec;
template <> struct Vec<_Float16> {
  static constexpr int N = 8;
  typedef h8 type;
};
template <> struct Vec<float> {
  static constexpr int N = 4;
  typedef f4 type;
};

// ---------------------------------------------------------------------------
// Embedding gather: out[row,:] = wte[ids[row],:] + wpe[row % L,:]
// (reference: fused_embeddings_kernel, kernels.py:37-72).  The add is done in
// fp32 and rounded once, which equals one add in the storage dtype.  A token id
// outside [0, V) reads nothing: its wte row counts as zeros (the reference reads
// out of bounds there).
// ---------------------------------------------------------------------------
template <typename T, int LPR>
__global__ __launch_bounds__(256) void embed_vec_kernel(
    const int64_t* __restrict__ ids, const T* __restrict__ wte,
    const T* __restrict__ wpe, T* __restrict__ out, int64_t rows, int64_t L, int64_t V_, int H) {
  typedef typename Vec<T>::type V;
  constexpr int VN = Vec<T>::N;
  const int lane = threadIdx.x & (LPR - 1);  // LPR lanes per token, as in the LayerNorm kernel
  const int64_t row = (int64_t)blockIdx.x * (256 / LPR) + threadIdx.x / LPR;
  if (row >= rows) return;
  const int64_t tok = ids[row];
  const bool known = (uint64_t)tok < (uint64_t)V_;
  const int64_t pos = row % L;
  const V* a = reinterpret_cast<const V*>(wte + (known ? tok : 0) * H);
  const V* b = reinterpret_cast<const V*>(wpe + pos * H);
  V* o = reinterpret_cast<V*>(out + row * H);
  const int nchunks = H / VN;
  for (int c = lane; c < nchunks; c += LPR) {
    V va = a[c], vb = b[c], vo;
#pragma unroll
    for (int j = 0; j < VN; ++j) vo[j] = (T)((known ? (float)va[j] : 0.f) + (float)vb[j]);
    __builtin_nontemporal_store(vo, o + c);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void embed_scalar_kernel(
    const int64_t* __restrict__ ids, const T* __restrict__ wte,
    const T* __restrict__ wpe, T* __restrict__ out, int64_t rows, int64_t L, int64_t V_, int H) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int64_t tok = ids[row];
  const bool known = (uint64_t)tok < (uint64_t)V_;
  const int64_t pos = row % L;
  for (int c = lane; c < H; c += 64)
    out[row * H + c] = (T)((known ? (float)wte[tok * H + c] : 0.f) + (float)wpe[pos * H + c]);
}

// Embedding with dropout (kernels.py:65-70): the sum is rounded to the storage dtype first,
// the dropout works on that value in fp32 with the COLUMN as the generator's offset, so every
// token sees the same mask.  Training-mode path: one Philox evaluation per element.
template <typename T>
__global__ __launch_bounds__(256) void embed_dropout_kernel(
    const int64_t* __restrict__ ids, const T* __restrict__ wte,
    const T* __restrict__ wpe, T* __restrict__ out, int64_t rows, int64_t L, int64_t V_, int H,
    DropoutArgs drop) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int64_t tok = ids[row];
  const bool known = (uint64_t)tok < (uint64_t)V_;
  const int64_t pos = row % L;
  for (int c = lane; c < H; c += 64) {
    const T sum = (T)((known ? (float)wte[tok * H + c] : 0.f) + (float)wpe[pos * H + c]);
    unsigned off[1] = {(unsigned)c};
    float z[1] = {(float)sum};
    dropout_apply<1>(drop, off, z);
    out[row * H + c] = (T)z[0];
  }
}


// ---------------------------------------------------------------------------
// LayerNorm (reference: fused_layer_norm_kernel, kernels.py:104-145): fp32
// mean, then fp32 centred biased variance, rstd = 1/sqrt(var + eps),
// z = (x - mean) * rstd * w + b.  CH = 16-byte chunks per lane.
//
// LPR = lanes per row, 64 or 32.  With 32 a wavefront works on two rows at once: for rows of
// 96 chunks (H = 768 in fp16) every lane then has work in every pass -- with 64 lanes a
// quarter of them idle in the second pass -- and twice the rows are in flight per wavefront
// (LayerNorm at the headline: 89 -> 74 us).  The launchers pick 32 when that wastes fewer lanes.
// ---------------------------------------------------------------------------
template <typename T, int CH, int LPR>
__global__ __launch_bounds__(256) void layernorm_vec_kernel(
    const T* __restrict__ x, const T* __restrict__ w, const T* __restrict__ b,
    T* __restrict__ out, int64_t M, int H, float eps) {
  typedef typename Vec<T>::type V;
  constexpr int VN = Vec<T>::N;
  const int lane = threadIdx.x & (LPR - 1);
  const int64_t row = (int64_t)blockIdx.x * (256 / LPR) + threadIdx.x / LPR;
  if (row >= M) return;
  const int nchunks = H / VN;
  const V* xr = reinterpret_cast<const V*>(x + row * H);
  const V* wv = reinterpret_cast<const V*>(w);
  const V* bv = reinterpret_cast<const V*>(b);
  float v[CH][VN];
  V tw[CH], tb[CH];  // weight and bias chunks, requested with the row: off the tail of the row
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    const int c = lane + i * LPR;
    if (c < nchunks) {
      V t = __builtin_nontemporal_load(xr + c);
      if (CH <= 4) {
        tw[i] = wv[c];
        tb[i] = bv[c];
      }
#pragma unroll
      for (int j = 0; j < VN; ++j) {
        v[i][j] = (float)t[j];
        s += v[i][j];
      }
    } else {
#pragma unroll
      for (int j = 0; j < VN; ++j) v[i][j] = 0.f;
    }
  }
  float mean, rstd;
  layernorm_stats<CH, VN, LPR>(v, s, lane, nchunks, H, eps, mean, rstd);
  V* o = reinterpret_cast<V*>(out + row * H);
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    const int c = lane + i * LPR;
    if (c < nchunks) {
      if (CH > 4) {  // long rows: too many registers to hold them from the start
        tw[i] = wv[c];
        tb[i] = bv[c];
      }
      V to;
#pragma unroll
      for (int j = 0; j < VN; ++j)
        to[j] = (T)layernorm_apply(v[i][j], mean, rstd, (float)tw[i][j], (float)tb[i][j]);
      // cached (not streaming) store: the [T, H] output is what the following GEMM reads, two
      // or three times over; it fits the 256 MB memory-side cache, and a GEMM fed from there
      // instead of HBM ran 12 % faster (its operand loads are only one k-tile ahead)
      o[c] = to;
    }
  }
}

// Embedding gather and the first LayerNorm in one pass: emb[row,:] = wte[id,:] + wpe[pos,:]
// (rounded to the storage dtype, as embed_vec_kernel stores it) and ln[row,:] = LayerNorm of
// that ROUNDED row, so both outputs are bit-identical to embed_vec_kernel followed by
// layernorm_vec_kernel; the row never leaves the registers in between (fused_embeddings ->
// fused_layer_norm in the reference, gpt.py:166-170 and 40).
template <typename T, int CH, int LPR>
__global__ __launch_bounds__(256) void embed_layernorm_kernel(
    const int64_t* __restrict__ ids, const T* __restrict__ wte, const T* __restrict__ wpe,
    const T* __restrict__ w, const T* __restrict__ b, T* __restrict__ emb, T* __restrict__ out,
    int64_t rows, int64_t L, int64_t V_, int H, float eps) {
  typedef typename Vec<T>::type V;
  constexpr int VN = Vec<T>::N;
  const int lane = threadIdx.x & (LPR - 1);
  const int64_t row = (int64_t)blockIdx.x * (256 / LPR) + threadIdx.x / LPR;
  if (row >= rows) return;
  const int64_t tok = ids[row];
  const bool known = (uint64_t)tok < (uint64_t)V_;
  const int nchunks = H / VN;
  const V* ar = reinterpret_cast<const V*>(wte + (known ? tok : 0) * H);
  const V* pr = reinterpret_cast<const V*>(wpe + (row % L) * H);
  const V* wv = reinterpret_cast<const V*>(w);
  const V* bv = reinterpret_cast<const V*>(b);
  V* eo = reinterpret_cast<V*>(emb + row * H);
  float v[CH][VN];
  V tw[CH], tb[CH];
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    const int c = lane + i * LPR;
    if (c < nchunks) {
      const V va = ar[c], vb = pr[c];
      tw[i] = wv[c];
      tb[i] = bv[c];
      V e;
#pragma unroll
      for (int j = 0; j < VN; ++j) {
        e[j] = (T)((known ? (float)va[j] : 0.f) + (float)vb[j]);
        v[i][j] = (float)e[j];
        s += v[i][j];
      }
      __builtin_nontemporal_store(e, eo + c);  // the residual stream; next read by a GEMM epilogue
    } else {
#pragma unroll
      for (int j = 0; j < VN; ++j) v[i][j] = 0.f;
    }
  }
  float mean, rstd;
  layernorm_stats<CH, VN, LPR>(v, s, lane, nchunks, H, eps, mean, rstd);
  V* o = reinterpret_cast<V*>(out + row * H);
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    const int c = lane + i * LPR;
    if (c < nchunks) {
      V to;
#pragma unroll
      for (int j = 0; j < VN; ++j)
        to[j] = (T)layernorm_apply(v[i][j], mean, rstd, (float)tw[i][j], (float)tb[i][j]);
      o[c] = to;  // cached store, as in layernorm_vec_kernel: the following GEMM reads it
    }
  }
}

// Any H (no alignment requirement): the row is re-read from cache per pass.
template <typename T>
__global__ __launch_bounds__(256) void layernorm_scalar_kernel(
    const T* __restrict__ x, const T* __restrict__ w, const T* __restrict__ b,
    T* __restrict__ out, int64_t M, int H, float eps) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= M) return;
  const T* xr = x + row * H;
  float s = 0.f;
  for (int c = lane; c < H; c += 64) s += (float)xr[c];
  const float mean = wave_sum(s) / (float)H;
  float q = 0.f;
  for (int c = lane; c < H; c += 64) {
    const float d = (float)xr[c] - mean;
    q += d * d;
  }
  const float var = wave_sum(q) / (float)H;
  const float rstd = 1.0f / sqrtf(var + eps);
  for (int c = lane; c < H; c += 64) {
    const float z = ((float)xr[c] - mean) * rstd;
    out[row * H + c] = (T)(z * (float)w[c] + (float)b[c]);
  }
}

// ---------------------------------------------------------------------------
// Row softmax: fp32 max, exp(x - max), fp32 sum, divide.
// ---------------------------------------------------------------------------
template <typename T, int CH, int LPR>
__global__ __launch_bounds__(256) void softmax_vec_kernel(const T* __restrict__ x,
                                                          T* __restrict__ out,
                                                          int64_t M, int H) {
  typedef typename Vec<T>::type V;
  constexpr int VN = Vec<T>::N;
  const int lane = threadIdx.x & (LPR - 1);
  const int64_t row = (int64_t)blockIdx.x * (256 / LPR) + threadIdx.x / LPR;
  if (row >= M) return;
  const int nchunks = H / VN;
  const V* xr = reinterpret_cast<const V*>(x + row * H);
  float v[CH][VN];
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    const int c = lane + i * LPR;
    if (c < nchunks) {
      V t = __builtin_nontemporal_load(xr + c);
#pragma unroll
      for (int j = 0; j < VN; ++j) {
        v[i][j] = (float)t[j];
        mx = fmaxf(mx, v[i][j]);
      }
    } else {
#pragma unroll
      for (int j = 0; j < VN; ++j) v[i][j] = -INFINITY;
    }
  }
  mx = group_max<LPR>(mx);
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < CH; ++i) {
#pragma unroll
    for (int j = 0; j < VN; ++j) {
      v[i][j] = __expf(v[i][j] - mx);  // exp(-inf) = 0 for the padding lanes
      s += v[i][j];
    }
  }
  const float inv = 1.0f / group_sum<LPR>(s);
  V* o = reinterpret_cast<V*>(out + row * H);
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    const int c = lane + i * LPR;
    if (c < nchunks) {
      V to;
#pragma unroll
      for (int j = 0; j < VN; ++j) to[j] = (T)(v[i][j] * inv);
      __builtin_nontemporal_store(to, o + c);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void softmax_scalar_kernel(const T* __restrict__ x,
                                                             T* __restrict__ out,
                                                             int64_t M, int H) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= M) return;
  const T* xr = x + row * H;
  float mx = -INFINITY;
  for (int c = lane; c < H; c += 64) mx = fmaxf(mx, (float)xr[c]);
  mx = wave_max(mx);
  float s = 0.f;
  for (int c = lane; c < H; c += 64) s += __expf((float)xr[c] - mx);
  const float inv = 1.0f / wave_sum(s);
  for (int c = lane; c < H; c += 64)
    out[row * H + c] = (T)(__expf((float)xr[c] - mx) * inv);
}

// ---------------------------------------------------------------------------
// GEMM operand packers.  Both produce fp16 rows of Kp (a multiple of 64)
// elements, zero filled beyond K, which is the only operand form the MFMA
// kernel reads.
//   pack_rows:      src[R][K]  -> dst[R][Kp]   (x, or a weight given as [N][K])
//   pack_transpose: src[K][N]  -> dst[N][Kp]   (weight given as [K][N])
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void pack_rows_kernel(const T* __restrict__ src,
                                                        _Float16* __restrict__ dst,
                                                        int64_t R, int K, int Kp) {
  const int64_t total = R * (int64_t)Kp;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / Kp;
    const int k = (int)(i - r * Kp);
    dst[i] = k < K ? (_Float16)(float)src[r * K + k] : (_Float16)0.f;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void pack_transpose_kernel(const T* __restrict__ src,
                                                             _Float16* __restrict__ dst,
                                                             int K, int N, int Kp) {
  __shared__ _Float16 tile[64][65];
  const int k0 = blockIdx.x * 64, n0 = blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int i = ty; i < 64; i += 4) {
    const int k = k0 + i, n = n0 + tx;
    tile[i][tx] = (k < K && n < N) ? (_Float16)(float)src[(int64_t)k * N + n]
                                   : (_Float16)0.f;
  }
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    const int n = n0 + i, k = k0 + tx;
    if (n < N) dst[(int64_t)n * Kp + k] = tile[tx][i];
  }
}

// ---------------------------------------------------------------------------
// Host launchers
// ---------------------------------------------------------------------------
template <typename T>
static int launch_embed_t(const int64_t* ids, const void* wte, const void* wpe,
                          void* out, int64_t rows, int64_t L, int64_t V, int H, Dropout drop,
                          hipStream_t st) {
  const unsigned grid = (unsigned)((rows + 3) / 4);
  // The reference runs the dropout even at p = 0 (kernels.py:70), where it is the identity
  // unless a column's uniform is exactly 0; for the default seed no column below 2^20 has
  // that, so only other seeds or wider rows need the generator at p = 0.
  if (drop.p != 0.0f || drop.seed != 1337 || H > (1 << 20)) {
    const DropoutArgs d = {drop.p, (unsigned)drop.seed, (unsigned)(drop.seed >> 32)};
    hipLaunchKernelGGL(embed_dropout_kernel<T>, dim3(grid), dim3(256), 0, st, ids,
                       (const T*)wte, (const T*)wpe, (T*)out, rows, L, V, H, d);
    return 0;
  }
  const bool aligned = (H % Vec<T>::N) == 0 && ((uintptr_t)wte % 16) == 0 &&
                       ((uintptr_t)wpe % 16) == 0 && ((uintptr_t)out % 16) == 0;
  if (aligned)
    if (lanes_per_row(H / Vec<T>::N) == 32)
      hipLaunchKernelGGL((embed_vec_kernel<T, 32>), dim3((unsigned)((rows + 7) / 8)), dim3(256), 0,
                         st, ids, (const T*)wte, (const T*)wpe, (T*)out, rows, L, V, H);
    else
      hipLaunchKernelGGL((embed_vec_kernel<T, 64>), dim3(grid), dim3(256), 0, st, ids,
                         (const T*)wte, (const T*)wpe, (T*)out, rows, L, V, H);
  else
    hipLaunchKernelGGL(embed_scalar_kernel<T>, dim3(grid), dim3(256), 0, st, ids,
                       (const T*)wte, (const T*)wpe, (T*)out, rows, L, V, H);
  return 0;
}

int launch_embed(const int64_t* ids, const void* wte, const void* wpe, void* out,
                 int64_t rows, int64_t L, int64_t V, int H, Dropout drop, bool f16,
                 hipStream_t st) {
  return f16 ? launch_embed_t<_Float16>(ids, wte, wpe, out, rows, L, V, H, drop, st)
             : launch_embed_t<float>(ids, wte, wpe, out, rows, L, V, H, drop, st);
}

template <typename T, int CH>
static void ln_go(const void* x, const void* w, const void* b, void* out, int64_t M,
                  int H, float eps, int lpr, hipStream_t st) {
  if (lpr == 32)
    hipLaunchKernelGGL((layernorm_vec_kernel<T, CH, 32>), dim3((unsigned)((M + 7) / 8)),
                       dim3(256), 0, st, (const T*)x, (const T*)w, (const T*)b,
                       (T*)out, M, H, eps);
  else
    hipLaunchKernelGGL((layernorm_vec_kernel<T, CH, 64>), dim3((unsigned)((M + 3) / 4)),
                       dim3(256), 0, st, (const T*)x, (const T*)w, (const T*)b,
                       (T*)out, M, H, eps);
}

template <typename T>
static int launch_layernorm_t(const void* x, const void* w, const void* b, void* out,
                              int64_t M, int H, float eps, hipStream_t st) {
  constexpr int VN = Vec<T>::N;
  const bool aligned = (H % VN) == 0 && ((uintptr_t)x % 16) == 0 &&
                       ((uintptr_t)w % 16) == 0 && ((uintptr_t)b % 16) == 0 &&
                       ((uintptr_t)out % 16) == 0;
  const int lpr = lanes_per_row(H / VN);
  const int need = aligned ? (H / VN + lpr - 1) / lpr : 1 << 30;
  if (need <= 1) ln_go<T, 1>(x, w, b, out, M, H, eps, lpr, st);
  else if (need <= 2) ln_go<T, 2>(x, w, b, out, M, H, eps, lpr, st);
  else if (need <= 3) ln_go<T, 3>(x, w, b, out, M, H, eps, lpr, st);
  else if (need <= 4) ln_go<T, 4>(x, w, b, out, M, H, eps, lpr, st);
  else if (need <= 8) ln_go<T, 8>(x, w, b, out, M, H, eps, lpr, st);
  else if (need <= 16) ln_go<T, 16>(x, w, b, out, M, H, eps, lpr, st);
  else if (need <= 32) ln_go<T, 32>(x, w, b, out, M, H, eps, lpr, st);
  else
    hipLaunchKernelGGL(layernorm_scalar_kernel<T>, dim3((unsigned)((M + 3) / 4)),
                       dim3(256), 0, st, (const T*)x, (const T*)w, (const T*)b,
                       (T*)out, M, H, eps);
  return 0;
}

int launch_layernorm(const void* x, const void* w, const void* b, void* out,
                     int64_t M, int H, float eps, bool f16, hipStream_t st) {
  return f16 ? launch_layernorm_t<_Float16>(x, w, b, out, M, H, eps, st)
             : launch_layernorm_t<float>(x, w, b, out, M, H, eps, st);
}

template <typename T, int CH>
static void sm_go(const void* x, void* out, int64_t M, int H, int lpr, hipStream_t st) {
  if (lpr == 32)
    hipLaunchKernelGGL((softmax_vec_kernel<T, CH, 32>), dim3((unsigned)((M + 7) / 8)),
                       dim3(256), 0, st, (const T*)x, (T*)out, M, H);
  else
    hipLaunchKernelGGL((softmax_vec_kernel<T, CH, 64>), dim3((unsigned)((M + 3) / 4)),
                       dim3(256), 0, st, (const T*)x, (T*)out, M, H);
}

template <typename T>
static int launch_softmax_t(const void* x, void* out, int64_t M, int H,
                            hipStream_t st) {
  constexpr int VN = Vec<T>::N;
  const bool aligned =
      (H % VN) == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)out % 16) == 0;
  const int lpr = lanes_per_row(H / VN);
  const int need = aligned ? (H / VN + lpr - 1) / lpr : 1 << 30;
  if (need <= 1) sm_go<T, 1>(x, out, M, H, lpr, st);
  else if (need <= 2) sm_go<T, 2>(x, out, M, H, lpr, st);
  else if (need <= 3) sm_go<T, 3>(x, out, M, H, lpr, st);
  else if (need <= 4) sm_go<T, 4>(x, out, M, H, lpr, st);
  else if (need <= 8) sm_go<T, 8>(x, out, M, H, lpr, st);
  else if (need <= 16) sm_go<T, 16>(x, out, M, H, lpr, st);
  else if (need <= 32) sm_go<T, 32>(x, out, M, H, lpr, st);
  else
    hipLaunchKernelGGL(softmax_scalar_kernel<T>, dim3((unsigned)((M + 3) / 4)),
                       dim3(256), 0, st, (const T*)x, (T*)out, M, H);
  return 0;
}

int launch_softmax(const void* x, void* out, int64_t M, int H, bool f16,
                   hipStream_t st) {
  return f16 ? launch_softmax_t<_Float16>(x, out, M, H, st)
             : launch_softmax_t<float>(x, out, M, H, st);
}

template <typename T, int CH>
static void eln_go(const int64_t* ids, const void* wte, const void* wpe, const void* w,
                   const void* b, void* emb, void* out, int64_t rows, int64_t L, int64_t V, int H,
                   float eps, int lpr, hipStream_t st) {
  if (lpr == 32)
    hipLaunchKernelGGL((embed_layernorm_kernel<T, CH, 32>), dim3((unsigned)((rows + 7) / 8)),
                       dim3(256), 0, st, ids, (const T*)wte, (const T*)wpe, (const T*)w,
                       (const T*)b, (T*)emb, (T*)out, rows, L, V, H, eps);
  else
    hipLaunchKernelGGL((embed_layernorm_kernel<T, CH, 64>), dim3((unsigned)((rows + 3) / 4)),
                       dim3(256), 0, st, ids, (const T*)wte, (const T*)wpe, (const T*)w,
                       (const T*)b, (T*)emb, (T*)out, rows, L, V, H, eps);
}

template <typename T>
static bool launch_embed_layernorm_t(const int64_t* ids, const void* wte, const void* wpe,
                                     const void* w, const void* b, void* emb, void* out,
                                     int64_t rows, int64_t L, int64_t V, int H, float eps,
                                     hipStream_t st) {
  constexpr int VN = Vec<T>::N;
  auto al = [](const void* p) { return ((uintptr_t)p % 16) == 0; };
  if ((H % VN) != 0 || !al(wte) || !al(wpe) || !al(w) || !al(b) || !al(emb) || !al(out))
    return false;
  const int lpr = lanes_per_row(H / VN);
  const int need = (H / VN + lpr - 1) / lpr;
  if (need <= 1) eln_go<T, 1>(ids, wte, wpe, w, b, emb, out, rows, L, V, H, eps, lpr, st);
  else if (need <= 2) eln_go<T, 2>(ids, wte, wpe, w, b, emb, out, rows, L, V, H, eps, lpr, st);
  else if (need <= 3) eln_go<T, 3>(ids, wte, wpe, w, b, emb, out, rows, L, V, H, eps, lpr, st);
  else if (need <= 4) eln_go<T, 4>(ids, wte, wpe, w, b, emb, out, rows, L, V, H, eps, lpr, st);
  else return false;
  return true;
}

// The fused embedding + LayerNorm launch for rows that fit the register-resident form (16-byte
// aligned, at most 4 chunks per lane: H <= 2048 halves / 1024 floats); otherwise false, and
// the caller launches the two kernels one after the other.
bool launch_embed_layernorm(const int64_t* ids, const void* wte, const void* wpe, const void* w,
                            const void* b, void* emb, void* out, int64_t rows, int64_t L,
                            int64_t V, int H, float eps, bool f16, hipStream_t st) {
  return f16 ? launch_embed_layernorm_t<_Float16>(ids, wte, wpe, w, b, emb, out, rows, L, V, H,
                                                  eps, st)
             : launch_embed_layernorm_t<float>(ids, wte, wpe, w, b, emb, out, rows, L, V, H, eps,
                                               st);
}

void launch_pack_rows(const void* src, void* dst, int64_t R, int K, int Kp, bool f16,
                      hipStream_t st) {
  const int64_t total = R * (int64_t)Kp;
  int64_t blocks = (total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  if (f16)
    hipLaunchKernelGGL(pack_rows_kernel<_Float16>, dim3((unsigned)blocks), dim3(256),
                       0, st, (const _Float16*)src, (_Float16*)dst, R, K, Kp);
  else
    hipLaunchKernelGGL(pack_rows_kernel<float>, dim3((unsigned)blocks), dim3(256), 0,
                       st, (const float*)src, (_Float16*)dst, R, K, Kp);
}

void launch_pack_transpose(const void* src, void* dst, int K, int N, int Kp, bool f16,
                           hipStream_t st) {
  dim3 grid((unsigned)(Kp / 64), (unsigned)((N + 63) / 64));
  if (f16)
    hipLaunchKernelGGL(pack_transpose_kernel<_Float16>, grid, dim3(256), 0, st,
                       (const _Float16*)src, (_Float16*)dst, K, N, Kp);
  else
    hipLaunchKernelGGL(pack_transpose_kernel<float>, grid, dim3(256), 0, st,
                       (const float*)src, (_Float16*)dst, K, N, Kp);
}

}  // namespace gptmi
