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
template <int D, typename T, bool BLND, bool DROP>
__global__ __launch_bounds__(256, (D == 64 && !DROP) ? 2 : 1) void flash_attn_kernel(
    const T* __restrict__ Q, const T* __restrict__ K, const T* __restrict__ V,
    T* __restrict__ O, int heads, int L, float scale, DropoutArgs drop) {
  constexpr int CH = D / 8;             // 16-byte chunks per row
  constexpr int KS = D / 16;            // MFMA k-steps over the head dim
  constexpr int DB = D / 32;            // 32-row blocks of O^T
  constexpr int K_BYTES = BKEY * D * 2;
  constexpr int STAGE = 2 * K_BYTES;
  constexpr int K_LD = BKEY * CH / 128; // K chunks per staging thread
  constexpr int V_UNITS = 16 * CH / 128; // (4 keys x 8 d) units per staging thread
  extern __shared__ __attribute__((aligned(16))) char smem[];  // 2 * STAGE bytes

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
  // Two register sets: tile u travels in set u % 2.  It is requested two steps before it is
  // multiplied (during step u - 2) and written to LDS at the end of step u - 1, so a global load
  // has a whole step of arithmetic plus a barrier to arrive, not a fraction of one.
  h8 stg[2][NLD];

  auto load_tile = [&](int t, h8 (&dst)[NLD]) {
    const int k0 = t * BKEY;
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      int row = k0 + srow[i];
      row = row < L ? row : L - 1;
      dst[i] = Ld8<T>::load(sp + (int64_t)row * D + scol[i]);
    }
  };

  auto store_tile = [&](int stage, const h8 (&src)[NLD]) {
    char* ks_ = smem + stage * STAGE;
    char* vs_ = ks_ + K_BYTES;
    if (role_k) {
#pragma unroll
      for (int i = 0; i < NLD; ++i) {
        const int key = srow[i], c = scol[i] >> 3;
        *reinterpret_cast<h8*>(ks_ + key * (D * 2) + ((c ^ (key & 7)) << 4)) = src[i];
      }
    } else {
#pragma unroll
      for (int u = 0; u < V_UNITS; ++u) {
        const int kg = srow[4 * u] >> 2, d0 = scol[4 * u];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int d = d0 + j;
          h4 col = {src[4 * u][j], src[4 * u + 1][j], src[4 * u + 2][j], src[4 * u + 3][j]};
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

  load_tile(0, stg[0]);
  if (nt > 1) load_tile(1, stg[1]);
  store_tile(0, stg[0]);
  __syncthreads();

  // one step = one key tile; `step` is instantiated for even and odd t so that the register
  // set of tile t + 1 (written to LDS at the end) and of tile t + 2 (requested at the start,
  // into the set tile t just left) are compile-time choices
  auto step = [&](int t, h8 (&set_same)[NLD], h8 (&set_next)[NLD]) {
    if (t + 2 < nt) load_tile(t + 2, set_same);
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
      if (need_mask) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = k0 + kb * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
            s[kb][r] = key <= q ? s[kb][r] : -INFINITY;
          }
      }
      float mult, psum = 0.f;
      if constexpr (sizeof(T) == 2 && !DROP) {
        // fp16 storage: running max on the raw scores, scale * log2(e) folded into one fused
        // multiply-add in front of exp2 (as in the resident kernel below)
        const float c = scale * 1.4426950408889634f;
        float bmax = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) bmax = fmaxf(bmax, s[kb][r]);
        bmax = fmaxf(bmax, __shfl_xor(bmax, 32, kWave));
        const float mnew = bmax > mrun ? bmax : mrun;
        mult = __builtin_amdgcn_exp2f((mrun - mnew) * c);
        const float m2 = mnew * c;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float p = __builtin_amdgcn_exp2f(fmaf(s[kb][r], c, -m2));
            s[kb][r] = p;
            psum += p;
          }
        mrun = mnew;
      } else {
        float bmax = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            s[kb][r] *= scale;
            bmax = fmaxf(bmax, s[kb][r]);
          }
        bmax = fmaxf(bmax, __shfl_xor(bmax, 32, kWave));
        const float mnew = bmax > mrun ? bmax : mrun;
        mult = softmax_exp<T>(mrun - mnew);
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float p = softmax_exp<T>(s[kb][r] - mnew);
            s[kb][r] = p;
            psum += p;
          }
        mrun = mnew;
      }
      psum += __shfl_xor(psum, 32, kWave);
      den = den * mult + psum;
      if constexpr (DROP) {
        // dropout of P after the denominator has summed it, before the fp16 rounding;
        // offset = query * L + key, the same for every batch and head (kernels.py:457-460)
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int rg = 0; rg < 4; ++rg) {
            const unsigned key0 = (unsigned)(k0 + kb * 32 + 8 * rg + 4 * g);
            const unsigned base_off = (unsigned)q * (unsigned)L + key0;
            unsigned off[4] = {base_off, base_off + 1u, base_off + 2u, base_off + 3u};
            float pv[4] = {s[kb][4 * rg], s[kb][4 * rg + 1], s[kb][4 * rg + 2], s[kb][4 * rg + 3]};
            dropout_apply<4>(drop, off, pv);
#pragma unroll
            for (int e = 0; e < 4; ++e) s[kb][4 * rg + e] = pv[e];
          }
      }
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
    if (t + 1 < nt) store_tile((t + 1) & 1, set_next);
    __syncthreads();
  };
  for (int t = 0; t < nt; t += 2) {
    step(t, stg[0], stg[1]);
    if (t + 1 < nt) step(t + 1, stg[1], stg[0]);
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

// ---------------------------------------------------------------------------
// Resident-K/V variant for short sequences (L*D small enough that K and V^T of
// one (batch, head) fit in half a CU's LDS, e.g. L <= 320 at D = 64).
//
// One workgroup = 8 wavefronts (4 for head sizes above 64, which need more than 128
// registers) = one (batch, head).  K ([L][D], 16-byte chunks
// swizzled with (row >> 1) & 7) and V^T ([D][Lp + 4], Lp = L rounded up to 64;
// the 8 pad bytes per row spread the 32 rows a fragment read touches over all
// banks) are staged once, behind ONE barrier; after it the wavefronts never
// synchronise again.  Queries are cut into chunks of 32; chunk c costs
// c/2 + 1 key tiles (causal), and the chunks are dealt to the wavefronts in snake
// order from the most expensive one, which balances the triangle over the SIMDs
// (L = 300: 8, 8, 7, 7 tiles).  The arithmetic per tile is that of the tiled kernel.
// ---------------------------------------------------------------------------
template <int D, typename T, bool BLND, int NW>
__global__ __launch_bounds__(NW * 64, NW / 2) void flash_attn_resident_kernel(
    const T* __restrict__ Q, const T* __restrict__ K, const T* __restrict__ V,
    T* __restrict__ O, int heads, int L, float scale) {
  constexpr int CH = D / 8, KS = D / 16, DB = D / 32;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int Lp = (L + BKEY - 1) / BKEY * BKEY;
  const int vstride = 2 * Lp + 8;            // bytes per V^T row
  char* ks_ = smem;                          // K: L rows of D halves
  char* vs_ = smem + (size_t)L * D * 2;      // V^T: D rows of Lp (+4) halves

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int bh = blockIdx.x;
  const int64_t base = (int64_t)bh * L * D;
  const T* Qp = Q + base;
  const T* Kp = K + base;
  const T* Vp = V + base;

  // ---- stage K and V^T: every global load is requested before the first LDS store, so the
  // workgroup pays one memory round trip, not one per batch.  The 80 KB limit bounds the
  // work: at most 2560 16-byte chunks of K and 640 (4 keys x 8 d) units of V.
  //   K chunk s -> row s / CH, chunk s % CH
  //   V unit  u -> d-chunk u % CH, key group u / CH (4 keys); keys past the end repeat the
  //   last row: their weights are exactly 0
  constexpr int NT = NW * 64;
  constexpr int KI = (2560 + NT - 1) / NT, VI = (640 + NT - 1) / NT;
  const int kchunks = L * CH, units = (Lp / 4) * CH;
  h8 kr[KI], vr[VI][4];
#pragma unroll
  for (int i = 0; i < KI; ++i) {
    const int s = i * NT + tid;
    if (s < kchunks) kr[i] = Ld8<T>::load(Kp + (int64_t)(s / CH) * D + (s % CH) * 8);
  }
#pragma unroll
  for (int i = 0; i < VI; ++i) {
    const int u = i * NT + tid;
    const int c = u % CH, kg = u / CH;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      int key = kg * 4 + kk;
      key = key < L ? key : L - 1;
      if (u < units) vr[i][kk] = Ld8<T>::load(Vp + (int64_t)key * D + c * 8);
    }
  }
#pragma unroll
  for (int i = 0; i < KI; ++i) {
    const int s = i * NT + tid;
    if (s < kchunks) {
      const int row = s / CH, c = s % CH;
      *reinterpret_cast<h8*>(ks_ + row * (D * 2) + ((c ^ ((row >> 1) & 7)) << 4)) = kr[i];
    }
  }
#pragma unroll
  for (int i = 0; i < VI; ++i) {
    const int u = i * NT + tid;
    if (u < units) {
      const int c = u % CH, kg = u / CH;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        h4 col = {vr[i][0][j], vr[i][1][j], vr[i][2][j], vr[i][3][j]};
        *reinterpret_cast<h4*>(vs_ + (c * 8 + j) * vstride + kg * 8) = col;
      }
    }
  }
  __syncthreads();

  const int ql = lane & 31, g = lane >> 5;
  const int nc = (L + 31) / 32;
  // snake deal over NW wavefronts: of every 2*NW positions (position i = chunk nc-1-i,
  // most expensive first) wavefront w takes w and 2*NW-1-w
  for (int i0 = 0; i0 < nc; i0 += 2 * NW) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int i = i0 + (half == 0 ? wave : 2 * NW - 1 - wave);
      if (i >= nc) continue;
      const int qw0 = (nc - 1 - i) * 32;  // first query of the chunk
      const int q = qw0 + ql;
      h8 qf[KS];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        qf[ks] = q < L ? Ld8<T>::load(Qp + (int64_t)q * D + ks * 16 + g * 8) : zero_h8();
      f16v oacc[DB];
#pragma unroll
      for (int b = 0; b < DB; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[b][r] = 0.f;
      float mrun = -INFINITY, den = 0.f;
      int last_q = qw0 + 31;
      if (last_q > L - 1) last_q = L - 1;
      const int nt = last_q / BKEY + 1;
      for (int t = 0; t < nt; ++t) {
        const int k0 = t * BKEY;
        // ---- S^T = K . Q^T -----------------------------------------------------
        f16v s[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
          for (int r = 0; r < 16; ++r) s[kb][r] = 0.f;
          int key = k0 + kb * 32 + ql;
          key = key < L ? key : L - 1;  // masked anyway; keeps the read inside K
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            const h8 kf = *reinterpret_cast<const h8*>(
                ks_ + key * (D * 2) + (((ks * 2 + g) ^ ((key >> 1) & 7)) << 4));
            s[kb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[ks], s[kb], 0, 0, 0);
          }
        }
        // ---- causal mask, running max, exponentials -----------------------------
        const bool need_mask = k0 + BKEY - 1 > qw0;
        if (need_mask) {
#pragma unroll
          for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const int key = k0 + kb * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
              s[kb][r] = key <= q ? s[kb][r] : -INFINITY;
            }
        }
        float mult, psum = 0.f;
        if constexpr (sizeof(T) == 2) {
          // fp16 storage: the running max is kept on the raw scores and scale * log2(e) is
          // folded into one fused multiply-add in front of exp2 -- the same real-number
          // formula as the reference, two VALU operations per score fewer
          const float c = scale * 1.4426950408889634f;
          float bmax = -INFINITY;
#pragma unroll
          for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) bmax = fmaxf(bmax, s[kb][r]);
          bmax = fmaxf(bmax, __shfl_xor(bmax, 32, kWave));
          const float mnew = bmax > mrun ? bmax : mrun;
          mult = __builtin_amdgcn_exp2f((mrun - mnew) * c);
          const float m2 = mnew * c;
#pragma unroll
          for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const float p = __builtin_amdgcn_exp2f(fmaf(s[kb][r], c, -m2));
              s[kb][r] = p;
              psum += p;
            }
          mrun = mnew;
        } else {
          // fp32 storage: the reference's operation order, library exp
          float bmax = -INFINITY;
#pragma unroll
          for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              s[kb][r] *= scale;
              bmax = fmaxf(bmax, s[kb][r]);
            }
          bmax = fmaxf(bmax, __shfl_xor(bmax, 32, kWave));
          const float mnew = bmax > mrun ? bmax : mrun;
          mult = softmax_exp<T>(mrun - mnew);
#pragma unroll
          for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const float p = softmax_exp<T>(s[kb][r] - mnew);
              s[kb][r] = p;
              psum += p;
            }
          mrun = mnew;
        }
        psum += __shfl_xor(psum, 32, kWave);
        den = den * mult + psum;
#pragma unroll
        for (int b = 0; b < DB; ++b)
#pragma unroll
          for (int r = 0; r < 16; ++r) oacc[b][r] *= mult;
        // ---- O^T += V^T . P^T --------------------------------------------------
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int tt = 0; tt < 2; ++tt) {
            h8 pf;
#pragma unroll
            for (int j = 0; j < 8; ++j) pf[j] = (_Float16)s[kb][8 * tt + j];
            const int kbase = k0 + kb * 32 + tt * 16 + 4 * g;  // first of this lane's keys
#pragma unroll
            for (int b = 0; b < DB; ++b) {
              const char* row = vs_ + (b * 32 + ql) * vstride + kbase * 2;
              const h4 lo = *reinterpret_cast<const h4*>(row);
              const h4 hi = *reinterpret_cast<const h4*>(row + 16);
              h8 vf = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
              oacc[b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf, oacc[b], 0, 0, 0);
            }
          }
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
        const float inv = __builtin_amdgcn_rcpf(den);  // fp16 storage only (1 ulp of fp32)
#pragma unroll
        for (int b = 0; b < DB; ++b)
#pragma unroll
          for (int rg = 0; rg < 4; ++rg) {
            const int d = b * 32 + 8 * rg + 4 * g;
            if constexpr (sizeof(T) == 2) {
              h4 o;
#pragma unroll
              for (int j = 0; j < 4; ++j) o[j] = (_Float16)(oacc[b][4 * rg + j] * inv);
              *reinterpret_cast<h4*>(O + row_off + d) = o;
            } else {
              f4 o;
#pragma unroll
              for (int j = 0; j < 4; ++j) o[j] = oacc[b][4 * rg + j] / den;
              *reinterpret_cast<f4*>(O + row_off + d) = o;
            }
          }
      }
    }
  }
}

constexpr int RESIDENT_WAVES = 8;

// LDS bytes of the resident variant, or 0 if this (L, D) does not fit two workgroups per CU.
inline size_t resident_lds_bytes(int L, int D) {
  const int Lp = (L + BKEY - 1) / BKEY * BKEY;
  const size_t bytes = (size_t)L * D * 2 + (size_t)D * (2 * Lp + 8);
  return bytes <= 80 * 1024 ? bytes : 0;
}

template <int D, typename T, bool BLND>
int launch_resident(const void* q, const void* k, const void* v, void* out, int64_t BN, int heads,
                    int L, float scale, size_t lds, hipStream_t st) {
  constexpr int NW = D == 64 ? RESIDENT_WAVES : 4;  // larger heads need > 128 registers
  auto kern = flash_attn_resident_kernel<D, T, BLND, NW>;
  static bool attr_done = false;  // idempotent; a race only repeats the call
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 80 * 1024);
    if (e != hipSuccess) {
      set_error("hipFuncSetAttribute(80 KB LDS): %s", hipGetErrorString(e));
      return -4;
    }
    attr_done = true;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)BN), dim3(NW * 64), lds, st, (const T*)q, (const T*)k,
                     (const T*)v, (T*)out, heads, L, scale);
  return 0;
}

template <int D, typename T, bool BLND, bool DROP>
int launch_tiled(const void* q, const void* k, const void* v, void* out, int64_t BN, int heads,
                 int L, float scale, DropoutArgs drop, hipStream_t st) {
  dim3 grid((unsigned)BN, (unsigned)((L + BQ - 1) / BQ));
  constexpr int lds = 2 * 2 * BKEY * D * 2;  // two stages of a K tile and a V^T tile
  auto kern = flash_attn_kernel<D, T, BLND, DROP>;
  static bool attr_done = false;  // idempotent; a race only repeats the call
  if (!attr_done && lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) {
      set_error("hipFuncSetAttribute(%d bytes LDS): %s", lds, hipGetErrorString(e));
      return -4;
    }
  }
  attr_done = true;
  hipLaunchKernelGGL(kern, grid, dim3(256), lds, st, (const T*)q, (const T*)k, (const T*)v,
                     (T*)out, heads, L, scale, drop);
  return 0;
}

template <int D, typename T>
int launch_d(const void* q, const void* k, const void* v, void* out, int64_t BN,
             int heads, int L, float scale, Dropout drop, bool blnd, hipStream_t st) {
  const DropoutArgs da = {drop.p, (unsigned)drop.seed, (unsigned)(drop.seed >> 32)};
  if (drop.p > 0.f) {  // training-mode path: the tiled kernel carries the generator
    return blnd ? launch_tiled<D, T, true, true>(q, k, v, out, BN, heads, L, scale, da, st)
                : launch_tiled<D, T, false, true>(q, k, v, out, BN, heads, L, scale, da, st);
  }
  if (const size_t lds = resident_lds_bytes(L, D)) {
    return blnd ? launch_resident<D, T, true>(q, k, v, out, BN, heads, L, scale, lds, st)
                : launch_resident<D, T, false>(q, k, v, out, BN, heads, L, scale, lds, st);
  }
  return blnd ? launch_tiled<D, T, true, false>(q, k, v, out, BN, heads, L, scale, da, st)
              : launch_tiled<D, T, false, false>(q, k, v, out, BN, heads, L, scale, da, st);
}

template <typename T>
int launch_t(const void* q, const void* k, const void* v, void* out, int64_t BN,
             int heads, int L, int d, float scale, Dropout drop, bool blnd, hipStream_t st) {
  switch (d) {
    case 64: return launch_d<64, T>(q, k, v, out, BN, heads, L, scale, drop, blnd, st);
    case 128: return launch_d<128, T>(q, k, v, out, BN, heads, L, scale, drop, blnd, st);
    case 256: return launch_d<256, T>(q, k, v, out, BN, heads, L, scale, drop, blnd, st);
    default:
      set_error("flash_attn: head size %d not built (64, 128 and 256 are)", d);
      return -2;
  }
}

}  // namespace

int launch_flash_attn(const void* q, const void* k, const void* v, void* out, int64_t B,
                      int64_t N, int64_t L, int d, float scale, Dropout drop, bool out_blnd,
                      bool f16, hipStream_t st) {
  const int64_t BN = B * N;
  if (BN > 0x7fffffffll || L > (1 << 24)) {
    set_error("flash_attn: B*N=%lld or L=%lld beyond the grid limits", (long long)BN,
              (long long)L);
    return -2;
  }
  return f16 ? launch_t<_Float16>(q, k, v, out, BN, (int)N, (int)L, d, scale, drop, out_blnd, st)
             : launch_t<float>(q, k, v, out, BN, (int)N, (int)L, d, scale, drop, out_blnd, st);
}

}  // namespace gptmi
