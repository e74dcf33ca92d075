// Causal flash attention for gfx950.
//
// Reference semantics: flash_attention_v1_kernel, kernels.py:375-474 -- q, k, v
// rounded to fp16; S = q.k^T in fp32, times scale; mask key <= query; keys
// visited in tiles of 64 in ascending order with the running max updated per
// tile; P = exp(S - max) summed unrounded into the denominator but rounded to
// fp16 for P.V; fp32 output accumulator; out = acc / denominator.
// Tiles that are entirely above the diagonal are skipped: for them the
// reference computes exp(-inf) = 0 and a multiplier of exactly 1, a no-op.
//
// One workgroup = 4 wavefronts = one (batch, head) x 128 queries; wavefront w
// owns queries [32w, 32w+32) of the block.  Everything is computed transposed
// so that one lane owns one query:
//   S^T[key][q] = K . Q^T   (MFMA 32x32x16: first operand K rows, second Q rows)
//   O^T[d][q]  += V^T . P^T (first operand V^T rows, second operand P^T)
// With the 32x32 accumulator layout a lane (q = lane%32, g = lane/32) holds,
// for the 32-key block kb, register r: key 32kb + 8(r/4) + 4g + r%4.  Row max
// and row sum are therefore in-lane reductions plus one exchange with lane^32,
// and registers [8t, 8t+8) of a block are, as they stand, the second MFMA
// operand for the 16-key step t -- P never moves between lanes.  The matching
// first operand needs V^T[d][those 8 keys]: V is transposed on its way into
// LDS (4 keys x 8 d per thread, register transpose, 8-byte stores).
// Wavefronts 0-1 stage the K tile, wavefronts 2-3 stage V^T; the next tile's
// global loads are in flight while the current one is consumed.
#include "common.h"
#include "launch.h"

namespace gptmi {

namespace {

constexpr int BQ = 128;  // queries per workgroup
constexpr int BKEY = 64; // keys per tile (fixed by the reference's numerics)

template <typename T> struct Ld8;  // 8 consecutive elements -> h8
template <> struct Ld8<_Float16> {
  static __device__ __forceinline__ h8 load(const _Float16* p) {
    return *reinterpret_cast<const h8*>(p);
  }
};
template <> struct Ld8<float> {
  static __device__ __forceinline__ h8 load(const float* p) {
    f4 a = *reinterpret_cast<const f4*>(p), b = *reinterpret_cast<const f4*>(p + 4);
    h8 r;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      r[j] = (_Float16)a[j];
      r[4 + j] = (_Float16)b[j];
    }
    return r;
  }
};

// exp for the softmax: the fp32-storage build keeps the accurate library
// routine (fewer fp16 rounding flips of P against the reference's np.exp);
// the fp16-storage build uses the hardware exp2 path.
template <typename T> __device__ __forceinline__ float softmax_exp(float x);
template <> __device__ __forceinline__ float softmax_exp<float>(float x) { return expf(x); }
template <> __device__ __forceinline__ float softmax_exp<_Float16>(float x) { return __expf(x); }

__device__ __forceinline__ h8 zero_h8() {
  h8 z;
#pragma unroll
  for (int j = 0; j < 8; ++j) z[j] = (_Float16)0.f;
  return z;
}

// D = head size.  LDS per stage: K tile [64][D] (16-byte chunk c of row r at
// position c ^ (r&7)) and V^T tile [D][64] (8-byte unit u of row d at position
// u ^ ((d>>1)&15)).
template <int D, typename T, bool BLND>
__global__ __launch_bounds__(256) void flash_attn_kernel(
    const T* __restrict__ Q, const T* __restrict__ K, const T* __restrict__ V,
    T* __restrict__ O, int heads, int L, float scale) {
  constexpr int CH = D / 8;             // 16-byte chunks per row
  constexpr int KS = D / 16;            // MFMA k-steps over the head dim
  constexpr int DB = D / 32;            // 32-row blocks of O^T
  constexpr int K_BYTES = BKEY * D * 2;
  constexpr int STAGE = 2 * K_BYTES;
  constexpr int K_LD = BKEY * CH / 128; // K chunks per staging thread
  constexpr int V_UNITS = 16 * CH / 128; // (4 keys x 8 d) units per staging thread
  __shared__ __attribute__((aligned(16))) char smem[2 * STAGE];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int bh = blockIdx.x;
  const int q_blocks = (L + BQ - 1) / BQ;
  // heavy (late) query blocks first so the tail of the grid is light
  const int qb = q_blocks - 1 - (int)blockIdx.y;
  const int q0 = qb * BQ;
  const int64_t base = (int64_t)bh * L * D;
  const T* Qp = Q + base;
  const T* Kp = K + base;
  const T* Vp = V + base;

  const int ql = lane & 31, g = lane >> 5;
  const int qw0 = q0 + wave * 32;    // first query of this wavefront
  const int q = qw0 + ql;            // this lane's query
  const bool wave_active = qw0 < L;

  // ---- Q fragments: lane (q, g) holds d = 16ks + 8g + 0..7 -----------------
  h8 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    qf[ks] = q < L ? Ld8<T>::load(Qp + (int64_t)q * D + ks * 16 + g * 8) : zero_h8();

  int last_q = q0 + BQ - 1;
  if (last_q > L - 1) last_q = L - 1;
  const int nt = last_q / BKEY + 1;  // key tiles 0..nt-1 touch this query block

  // ---- staging: each thread moves NLD 16-byte chunks per tile --------------
  // waves 0-1 (role K): chunk s = i*128 + st -> key s / CH, chunk s % CH
  // waves 2-3 (role V): unit  s = (i/4)*128 + st -> key group s & 15 (4 keys),
  //                     chunk s >> 4; register i holds key 4*group + i%4.
  // Rows past the end of the sequence are clamped to the last row: their keys
  // are masked (P = 0 exactly) and the values stay finite.
  constexpr int NLD = K_LD;
  static_assert(K_LD == 4 * V_UNITS, "K and V staging must move the same chunk count");
  const int st = tid & 127;
  const bool role_k = wave < 2;
  const T* sp = role_k ? Kp : Vp;
  int srow[NLD], scol[NLD];
#pragma unroll
  for (int i = 0; i < NLD; ++i) {
    if (role_k) {
      const int s = i * 128 + st;
      srow[i] = s / CH;
      scol[i] = (s % CH) * 8;
    } else {
      const int s = (i >> 2) * 128 + st;
      srow[i] = (s & 15) * 4 + (i & 3);
      scol[i] = (s >> 4) * 8;
    }
  }
  h8 stg[NLD];

  auto load_tile = [&](int t) {
    const int k0 = t * BKEY;
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      int row = k0 + srow[i];
      row = row < L ? row : L - 1;
      stg[i] = Ld8<T>::load(sp + (int64_t)row * D + scol[i]);
    }
  };

  auto store_tile = [&](int stage) {
    char* ks_ = smem + stage * STAGE;
    char* vs_ = ks_ + K_BYTES;
    if (role_k) {
#pragma unroll
      for (int i = 0; i < NLD; ++i) {
        const int key = srow[i], c = scol[i] >> 3;
        *reinterpret_cast<h8*>(ks_ + key * (D * 2) + ((c ^ (key & 7)) << 4)) = stg[i];
      }
    } else {
#pragma unroll
      for (int u = 0; u < V_UNITS; ++u) {
        const int kg = srow[4 * u] >> 2, d0 = scol[4 * u];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int d = d0 + j;
          h4 col = {stg[4 * u][j], stg[4 * u + 1][j], stg[4 * u + 2][j], stg[4 * u + 3][j]};
          *reinterpret_cast<h4*>(vs_ + d * 128 + ((kg ^ ((d >> 1) & 15)) << 3)) = col;
        }
      }
    }
  };

  f16v oacc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;
  float mrun = -INFINITY, den = 0.f;

  load_tile(0);
  store_tile(0);
  __syncthreads();

  for (int t = 0; t < nt; ++t) {
    if (t + 1 < nt) load_tile(t + 1);
    const int k0 = t * BKEY;
    if (wave_active && k0 <= qw0 + 31) {
      const char* ks_ = smem + (t & 1) * STAGE;
      const char* vs_ = ks_ + K_BYTES;
      // ---- S^T = K . Q^T ---------------------------------------------------
      f16v s[2];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
        for (int r = 0; r < 16; ++r) s[kb][r] = 0.f;
        const int key = kb * 32 + ql;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const h8 kf = *reinterpret_cast<const h8*>(
              ks_ + key * (D * 2) + (((ks * 2 + g) ^ (key & 7)) << 4));
          s[kb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[ks], s[kb], 0, 0, 0);
        }
      }
      // ---- scale, causal mask, running max -----------------------------------
      const bool need_mask = k0 + BKEY - 1 > qw0;
      float bmax = -INFINITY;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          float x = s[kb][r] * scale;
          if (need_mask) {
            const int key = k0 + kb * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
            x = key <= q ? x : -INFINITY;
          }
          s[kb][r] = x;
          bmax = fmaxf(bmax, x);
        }
      bmax = fmaxf(bmax, __shfl_xor(bmax, 32, kWave));
      const float mnew = bmax > mrun ? bmax : mrun;
      const float mult = softmax_exp<T>(mrun - mnew);
      float psum = 0.f;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float p = softmax_exp<T>(s[kb][r] - mnew);
          s[kb][r] = p;
          psum += p;
        }
      psum += __shfl_xor(psum, 32, kWave);
      den = den * mult + psum;
      mrun = mnew;
#pragma unroll
      for (int i = 0; i < DB; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[i][r] *= mult;
      // ---- O^T += V^T . P^T --------------------------------------------------
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
          h8 pf;
#pragma unroll
          for (int j = 0; j < 8; ++j) pf[j] = (_Float16)s[kb][8 * tt + j];
          // keys of this step held by lane group g: base+4g+0..3, base+8+4g+0..3
          const int u0 = (kb * 32 + tt * 16) / 4 + g;  // 8-byte unit of the first four
#pragma unroll
          for (int i = 0; i < DB; ++i) {
            const int d = i * 32 + ql;
            const int sw = (d >> 1) & 15;
            const h4 lo = *reinterpret_cast<const h4*>(vs_ + d * 128 + ((u0 ^ sw) << 3));
            const h4 hi =
                *reinterpret_cast<const h4*>(vs_ + d * 128 + (((u0 + 2) ^ sw) << 3));
            h8 vf = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            oacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf, oacc[i], 0, 0, 0);
          }
        }
    }
    if (t + 1 < nt) store_tile((t + 1) & 1);
    __syncthreads();
  }

  // ---- out[q][d] = O^T[d][q] / den ------------------------------------------
  if (q < L) {
    int64_t row_off;
    if (BLND) {
      const int b = bh / heads, n = bh - b * heads;
      row_off = (((int64_t)b * L + q) * heads + n) * D;
    } else {
      row_off = base + (int64_t)q * D;
    }
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        const int d = i * 32 + 8 * rg + 4 * g;
        if constexpr (sizeof(T) == 2) {
          h4 o;
#pragma unroll
          for (int j = 0; j < 4; ++j) o[j] = (_Float16)(oacc[i][4 * rg + j] / den);
          *reinterpret_cast<h4*>(O + row_off + d) = o;
        } else {
          f4 o;
#pragma unroll
          for (int j = 0; j < 4; ++j) o[j] = oacc[i][4 * rg + j] / den;
          *reinterpret_cast<f4*>(O + row_off + d) = o;
        }
      }
  }
}

template <int D, typename T>
int launch_d(const void* q, const void* k, const void* v, void* out, int64_t BN,
             int heads, int L, float scale, bool blnd, hipStream_t st) {
  dim3 grid((unsigned)BN, (unsigned)((L + BQ - 1) / BQ));
  if (blnd)
    hipLaunchKernelGGL((flash_attn_kernel<D, T, true>), grid, dim3(256), 0, st,
                       (const T*)q, (const T*)k, (const T*)v, (T*)out, heads, L, scale);
  else
    hipLaunchKernelGGL((flash_attn_kernel<D, T, false>), grid, dim3(256), 0, st,
                       (const T*)q, (const T*)k, (const T*)v, (T*)out, heads, L, scale);
  return 0;
}

template <typename T>
int launch_t(const void* q, const void* k, const void* v, void* out, int64_t BN,
             int heads, int L, int d, float scale, bool blnd, hipStream_t st) {
  switch (d) {
    case 64: return launch_d<64, T>(q, k, v, out, BN, heads, L, scale, blnd, st);
    case 128: return launch_d<128, T>(q, k, v, out, BN, heads, L, scale, blnd, st);
    default:
      set_error("flash_attn: head size %d not built (64 and 128 are)", d);
      return -2;
  }
}

}  // namespace

int launch_flash_attn(const void* q, const void* k, const void* v, void* out, int64_t B,
                      int64_t N, int64_t L, int d, float scale, bool out_blnd, bool f16,
                      hipStream_t st) {
  const int64_t BN = B * N;
  if (BN > 0x7fffffffll || L > (1 << 24)) {
    set_error("flash_attn: B*N=%lld or L=%lld beyond the grid limits", (long long)BN,
              (long long)L);
    return -2;
  }
  return f16 ? launch_t<_Float16>(q, k, v, out, BN, (int)N, (int)L, d, scale, out_blnd, st)
             : launch_t<float>(q, k, v, out, BN, (int)N, (int)L, d, scale, out_blnd, st);
}

}  // namespace gptmi
