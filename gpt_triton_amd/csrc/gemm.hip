// fp16 MFMA GEMM with a fused epilogue for gfx950.
//
//   C[M][N] = A[M][Kp] . Bt[N][Kp]^T      (both operands K-contiguous fp16)
//   out     = gelu?(C + bias) + residual  (fp32 math, one rounding at the store)
//
// Reference semantics: fused_ffn_kernel, kernels.py:169-257 (operands rounded to
// fp16, fp32 accumulation, epilogue order bias -> GELU -> residual -> cast) and
// the q/k/v relayout of matmul_and_split_qkv, kernels.py:347-367, which is done
// here by the store instead of by three copies.
//
// Structure of one workgroup (WM x WN wavefronts):
//   * a BM x BN output tile, K walked in steps of BK = 64 through a ring of
//     STAGES LDS buffers filled by direct global->LDS loads (16 B per lane,
//     no VGPR staging);
//   * LDS rows are 128 B (64 halves) = 8 chunks of 16 B; chunk c of row r is
//     kept at position c ^ (r & 7) so that the 16-byte fragment reads of 8
//     consecutive rows hit 8 different bank groups;
//   * each wavefront owns a (BM/WM) x (BN/WN) sub-tile as 32x32 MFMA blocks.
//     The MFMA is issued as D[n][m] (weight rows as the first operand) so a
//     lane ends up with 4 consecutive n for one m: an 8-byte packed store.
//   * workgroup ids are remapped so each XCD (ids are dealt round-robin over
//     the 8 XCDs) gets a contiguous range of tiles, N fastest: the tiles that
//     share a row block of A run on the same L2 at the same time.
#include "common.h"
#include "launch.h"

namespace gptmi {

namespace {

constexpr int BK = 64;
constexpr int ROW_BYTES = BK * 2;  // 128

struct EpiDev {
  const void* bias;
  const void* residual;
  void* out;
  void* q;
  void* k;
  void* v;
  int64_t L;
  int heads;
  int d;
  int gelu;
  int vec_ok;  // pointers and N allow 4-element vector accesses
};

__device__ __forceinline__ void lds_dma16(const void* gsrc, void* ldst) {
  __builtin_amdgcn_global_load_lds(
      (const __attribute__((address_space(1))) void*)gsrc,
      (__attribute__((address_space(3))) void*)ldst, 16, 0, 0);
}

// Workgroup barrier that does not drain the vector-memory counter: the
// compiler's own barrier waits for vmcnt(0), which would serialise the
// global->LDS prefetch of the younger pipeline stages behind it.
__device__ __forceinline__ void block_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  if constexpr (N == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  else if constexpr (N == 1) asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
  else if constexpr (N == 2) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
  else if constexpr (N == 3) asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
  else if constexpr (N == 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
  else if constexpr (N == 6) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
  else if constexpr (N == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
  else if constexpr (N == 12) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
  else if constexpr (N == 16) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
  else if constexpr (N == 24) asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
  else static_assert(N < 0, "add this vmcnt value");
}

template <typename T> struct Pack4;
template <> struct Pack4<_Float16> { typedef h4 type; };
template <> struct Pack4<float> { typedef f4 type; };

// Applies bias/GELU/residual to 4 consecutive columns [n0, n0+4) of row m and
// stores them.
template <typename T, bool QKV>
__device__ __forceinline__ void epilogue4(const EpiDev& ep, int64_t m, int n0, f4 acc,
                                          int N) {
  typedef typename Pack4<T>::type P;
  const bool full = (n0 + 3 < N) && ep.vec_ok;
  float z[4] = {acc[0], acc[1], acc[2], acc[3]};
  if (ep.bias) {
    const T* bp = (const T*)ep.bias + n0;
    if (full) {
      P b = *reinterpret_cast<const P*>(bp);
#pragma unroll
      for (int j = 0; j < 4; ++j) z[j] += (float)b[j];
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (n0 + j < N) z[j] += (float)bp[j];
    }
  }
  if (ep.gelu) {
#pragma unroll
    for (int j = 0; j < 4; ++j) z[j] = gelu_new(z[j]);
  }
  if constexpr (!QKV) {
    const int64_t off = m * (int64_t)N + n0;
    if (ep.residual) {
      const T* rp = (const T*)ep.residual + off;
      if (full) {
        P r = __builtin_nontemporal_load(reinterpret_cast<const P*>(rp));
#pragma unroll
        for (int j = 0; j < 4; ++j) z[j] += (float)r[j];
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (n0 + j < N) z[j] += (float)rp[j];
      }
    }
    T* op = (T*)ep.out + off;
    if (full) {
      P o;
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = (T)z[j];
      *reinterpret_cast<P*>(op) = o;
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (n0 + j < N) op[j] = (T)z[j];
    }
  } else {
    // column n of the [q | k | v] matrix -> (which, head, dd); row m -> (b, l)
    const int hd = ep.heads * ep.d;
    const int which = n0 / hd;
    const int within = n0 - which * hd;
    const int head = within / ep.d;
    const int dd = within - head * ep.d;
    const int64_t b = m / ep.L;
    const int64_t l = m - b * ep.L;
    T* base = (T*)(which == 0 ? ep.q : (which == 1 ? ep.k : ep.v));
    T* op = base + (((b * ep.heads + head) * ep.L + l) * ep.d + dd);
    if (full) {
      P o;
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = (T)z[j];
      *reinterpret_cast<P*>(op) = o;
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (n0 + j < N) op[j] = (T)z[j];
    }
  }
}

template <int BM, int BN, int WM, int WN, int STAGES, typename T, bool QKV>
__global__ __launch_bounds__(WM * WN * 64) void gemm_kernel(
    const _Float16* __restrict__ A, const _Float16* __restrict__ Bt, int M, int N,
    int Kp, int tiles_m, int tiles_n, EpiDev ep) {
  constexpr int T_ = WM * WN * 64;
  constexpr int TM = BM / WM, TN = BN / WN;
  constexpr int MB = TM / 32, NB = TN / 32;
  constexpr int A_IT = BM * 8 / T_, B_IT = BN * 8 / T_;
  constexpr int LPT = A_IT + B_IT;  // direct loads per thread per k-tile
  constexpr int STAGE_BYTES = (BM + BN) * ROW_BYTES;
  static_assert(BM * 8 % T_ == 0 && BN * 8 % T_ == 0, "tile/threads mismatch");
  static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tile must be 32-aligned");

  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave % WM, wn = wave / WM;

  // ---- XCD-aware tile id ------------------------------------------------
  const int num_tiles = tiles_m * tiles_n;
  int tile;
  {
    const int pid = blockIdx.x;
    const int per = (num_tiles + 7) >> 3;
    int tall = num_tiles & 7;
    if (tall == 0) tall = 8;
    const int xcd = pid & 7, loc = pid >> 3;
    tile = xcd < tall ? xcd * per + loc
                      : tall * per + (xcd - tall) * (per - 1) + loc;
  }
  const int tn = tile % tiles_n, tm = tile / tiles_n;
  const int m0 = tm * BM, n0 = tn * BN;

  // ---- per-thread sources of the direct global->LDS loads -----------------
  // Linear 16-byte slot s of a tile: row s>>3, stored chunk position s&7,
  // which holds source chunk (s&7) ^ (row&7).
  const _Float16* a_src[A_IT];
  const _Float16* b_src[B_IT];
#pragma unroll
  for (int it = 0; it < A_IT; ++it) {
    const int s = it * T_ + tid, r = s >> 3, c = (s & 7) ^ (r & 7);
    int row = m0 + r;
    row = row < M ? row : M - 1;
    a_src[it] = A + (size_t)row * Kp + c * 8;
  }
#pragma unroll
  for (int it = 0; it < B_IT; ++it) {
    const int s = it * T_ + tid, r = s >> 3, c = (s & 7) ^ (r & 7);
    int row = n0 + r;
    row = row < N ? row : N - 1;
    b_src[it] = Bt + (size_t)row * Kp + c * 8;
  }

  auto issue = [&](int stage, int kt) {
    char* as = smem + stage * STAGE_BYTES;
    char* bs = as + BM * ROW_BYTES;
#pragma unroll
    for (int it = 0; it < A_IT; ++it)
      lds_dma16(a_src[it] + (size_t)kt * BK, as + (it * T_ + wave * 64) * 16);
#pragma unroll
    for (int it = 0; it < B_IT; ++it)
      lds_dma16(b_src[it] + (size_t)kt * BK, bs + (it * T_ + wave * 64) * 16);
  };

  f16v acc[NB][MB];
#pragma unroll
  for (int i = 0; i < NB; ++i)
#pragma unroll
    for (int j = 0; j < MB; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int KT = Kp / BK;
#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s)
    if (s < KT) issue(s, s);

  // fragment read offsets (bytes) inside a stage: row-major 128-byte rows
  const int frow = lane & 31, fhalf = lane >> 5, fsw = lane & 7;
  const int a_row_off = (wm * TM + frow) * ROW_BYTES;
  const int b_row_off = BM * ROW_BYTES + (wn * TN + frow) * ROW_BYTES;

  for (int kt = 0; kt < KT; ++kt) {
    // tile kt must have landed; up to STAGES-2 younger tiles may be in flight
    if (kt + STAGES - 2 < KT) wait_vmcnt<(STAGES - 2) * LPT>();
    else wait_vmcnt<0>();
    block_barrier();
    if (kt + STAGES - 1 < KT) issue((kt + STAGES - 1) % STAGES, kt + STAGES - 1);

    const char* st = smem + (kt % STAGES) * STAGE_BYTES;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      const int choff = ((ks * 2 + fhalf) ^ fsw) << 4;
      h8 af[MB], bf[NB];
#pragma unroll
      for (int j = 0; j < MB; ++j)
        af[j] = *reinterpret_cast<const h8*>(st + a_row_off + j * 32 * ROW_BYTES + choff);
#pragma unroll
      for (int i = 0; i < NB; ++i)
        bf[i] = *reinterpret_cast<const h8*>(st + b_row_off + i * 32 * ROW_BYTES + choff);
#pragma unroll
      for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int j = 0; j < MB; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[i], af[j], acc[i][j], 0, 0, 0);
    }
  }

  // ---- epilogue: lane holds, per block, m = lane%32 and for g = 0..3 the 4
  // columns 8g + 4*(lane/32) + 0..3 -----------------------------------------
#pragma unroll
  for (int j = 0; j < MB; ++j) {
    const int64_t m = (int64_t)m0 + wm * TM + j * 32 + frow;
    if (m >= M) continue;
#pragma unroll
    for (int i = 0; i < NB; ++i) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n = n0 + wn * TN + i * 32 + g * 8 + fhalf * 4;
        if (n >= N) continue;
        f4 v4 = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2],
                 acc[i][j][4 * g + 3]};
        epilogue4<T, QKV>(ep, m, n, v4, N);
      }
    }
  }
}

template <int BM, int BN, int WM, int WN, int STAGES, typename T, bool QKV>
int launch_cfg(const void* A, const void* Bt, int64_t M, int N, int Kp,
               const EpiDev& ep, hipStream_t st) {
  auto kern = gemm_kernel<BM, BN, WM, WN, STAGES, T, QKV>;
  constexpr int smem = STAGES * (BM + BN) * ROW_BYTES;
  static bool attr_done = false;  // idempotent; a race only repeats the call
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) {
      set_error("hipFuncSetAttribute(%d bytes LDS): %s", smem, hipGetErrorString(e));
      return -4;
    }
    attr_done = true;
  }
  const int tiles_m = (int)((M + BM - 1) / BM), tiles_n = (N + BN - 1) / BN;
  hipLaunchKernelGGL(kern, dim3((unsigned)(tiles_m * tiles_n)), dim3(WM * WN * 64), smem,
                     st, (const _Float16*)A, (const _Float16*)Bt, (int)M, N, Kp, tiles_m,
                     tiles_n, ep);
  return 0;
}

template <typename T, bool QKV>
int launch_shape(const void* A, const void* Bt, int64_t M, int N, int Kp,
                 const EpiDev& ep, hipStream_t st) {
  // Big problems: 256x256 tiles, 8 waves.  Small ones: 128x128, 4 waves, so
  // that tests with a few hundred rows still spread over several CUs.
  if (M >= 2048 && N >= 256)
    return launch_cfg<256, 256, 2, 4, 2, T, QKV>(A, Bt, M, N, Kp, ep, st);
  return launch_cfg<128, 128, 2, 2, 3, T, QKV>(A, Bt, M, N, Kp, ep, st);
}

}  // namespace

int launch_gemm(const void* A, const void* Bt, int64_t M, int N, int Kp,
                const GemmEpilogue& e, hipStream_t st) {
  if (M >= (1ll << 31) - 512) {
    set_error("gemm: M=%lld does not fit the kernel's 32-bit row index", (long long)M);
    return -2;
  }
  EpiDev ep;
  ep.bias = e.bias;
  ep.residual = e.residual;
  ep.out = e.out;
  ep.q = e.q;
  ep.k = e.k;
  ep.v = e.v;
  ep.L = e.L;
  ep.heads = e.heads;
  ep.d = e.d;
  ep.gelu = e.gelu;
  const uintptr_t amask = e.f16 ? 7 : 15;
  bool vec = (N % 4) == 0;
  auto aligned = [&](const void* p) { return p == nullptr || ((uintptr_t)p & amask) == 0; };
  vec = vec && aligned(e.bias) && aligned(e.residual) && aligned(e.out) && aligned(e.q) &&
        aligned(e.k) && aligned(e.v);
  if (e.qkv) vec = vec && (e.d % 4) == 0;
  ep.vec_ok = vec ? 1 : 0;
  if (e.qkv && (e.d % 4) != 0) {
    set_error("gemm qkv epilogue: head size %d must be a multiple of 4", e.d);
    return -2;
  }
  if (e.f16)
    return e.qkv ? launch_shape<_Float16, true>(A, Bt, M, N, Kp, ep, st)
                 : launch_shape<_Float16, false>(A, Bt, M, N, Kp, ep, st);
  return e.qkv ? launch_shape<float, true>(A, Bt, M, N, Kp, ep, st)
               : launch_shape<float, false>(A, Bt, M, N, Kp, ep, st);
}

}  // namespace gptmi
