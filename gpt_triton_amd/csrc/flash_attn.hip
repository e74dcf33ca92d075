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
#include <type_traits>

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

// D = head size of the LDS tiles.  LDS per stage: K tile [64][D] (16-byte chunk c of row r at
// position c ^ (r&7)) and V^T tile [D][64] (8-byte unit u of row d at position
// u ^ ((d>>1)&15)).  DG = head size of the tensors in memory: 16 and 32 run on the D = 64
// staging layout (columns at or past DG are written as zeros, never read from memory) with
// only DG / 16 k-steps of q . k and one 32-row block of O^T.
template <int D, typename T, bool BLND, bool DROP, bool UNEQ, int DG = D>
__global__ __launch_bounds__(256, (D == 64 && !DROP) ? 2 : 1) void flash_attn_kernel(
    const T* __restrict__ Q, const T* __restrict__ K, const T* __restrict__ V,
    T* __restrict__ O, int heads, int L, int Lk_arg, float scale, DropoutArgs drop) {
  // L = query rows, Lk = key rows of every (batch, head); UNEQ = they may differ.  The mask is
  // "key <= query" alone and key rows at or past Lk count as zero rows, as in the reference
  // (kernels.py:421-436): with L > Lk the queries at or past Lk also see the zero rows that fill
  // up the last key tile.  With L == Lk no valid query sees such a row, and the staging loads
  // read the last row again instead (no select per load).
  const int Lk = UNEQ ? Lk_arg : L;
  constexpr int CH = D / 8;             // 16-byte chunks per row
  static_assert(DG == D || (D == 64 && (DG == 16 || DG == 32) && UNEQ), "small heads: D = 64");
  constexpr int KS = DG / 16;           // MFMA k-steps over the head dim
  constexpr int DB = (DG + 31) / 32;    // 32-row blocks of O^T
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
  const int64_t base = (int64_t)bh * L * DG, kv_base = (int64_t)bh * Lk * DG;
  const T* Qp = Q + base;
  const T* Kp = K + kv_base;
  const T* Vp = V + kv_base;

  const int ql = lane & 31, g = lane >> 5;
  const int qw0 = q0 + wave * 32;    // first query of this wavefront
  const int q = qw0 + ql;            // this lane's query
  const bool wave_active = qw0 < L;

  // ---- Q fragments: lane (q, g) holds d = 16ks + 8g + 0..7 -----------------
  h8 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    qf[ks] = q < L ? Ld8<T>::load(Qp + (int64_t)q * DG + ks * 16 + g * 8) : zero_h8();

  int last_q = q0 + BQ - 1;
  if (last_q > L - 1) last_q = L - 1;
  // key tiles 0..nt-1 touch this query block: up to the diagonal, and no further than the keys go
  const int nt = UNEQ ? min(last_q / BKEY + 1, (Lk + BKEY - 1) / BKEY) : last_q / BKEY + 1;

  // ---- staging: each thread moves NLD 16-byte chunks per tile --------------
  // waves 0-1 (role K): chunk s = i*128 + st -> key s / CH, chunk s % CH
  // waves 2-3 (role V): unit  s = (i/4)*128 + st -> key group s & 15 (4 keys),
  //                     chunk s >> 4; register i holds key 4*group + i%4.
  // Rows at or past Lk: zero rows if the lengths may differ (visible padding when L > Lk);
  // otherwise the last row again -- the keys are masked (P = 0 exactly), the values finite.
  constexpr int NLD = K_LD;
  static_assert(K_LD == 4 * V_UNITS, "K and V staging must move the same chunk count");
  const int st = tid & 127;
  const bool role_k = wave < 2;
  const T* sp = role_k ? Kp : Vp;
  // Both are a lane part plus a part that depends on i alone (128 is a multiple of CH and of 16),
  // so two registers and compile-time increments stand for the 2 * NLD values.
  static_assert(128 % CH == 0, "a row is at most 128 chunks");
  const int srow0 = role_k ? st / CH : (st & 15) * 4;
  const int scol0 = role_k ? (st % CH) * 8 : (st >> 4) * 8;
  auto srow_of = [&](int i) { return srow0 + (role_k ? i * (128 / CH) : (i & 3)); };
  auto scol_of = [&](int i) { return scol0 + (role_k ? 0 : (i >> 2) * 64); };
  // Two register sets: tile u travels in set u % 2.  It is requested two steps before it is
  // multiplied (during step u - 2) and written to LDS at the end of step u - 1, so a global load
  // has a whole step of arithmetic plus a barrier to arrive, not a fraction of one.  Head size
  // 256 has room for one set only (a set is 64 registers there, beside 128 of O^T and 64 of Q):
  // its tile u is requested at the start of step u - 1 and written at that step's end.
  constexpr bool ONESET = D >= 256;
  h8 stg[ONESET ? 1 : 2][NLD];

  auto load_tile = [&](int t, h8 (&dst)[NLD]) {
    const int k0 = t * BKEY;
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      int row = k0 + srow_of(i);
      if constexpr (UNEQ) {
        const bool there = DG < D ? (row < Lk && scol_of(i) < DG) : row < Lk;
        dst[i] = there ? Ld8<T>::load(sp + (int64_t)row * DG + scol_of(i)) : zero_h8();
      } else {
        row = row < L ? row : L - 1;
        dst[i] = Ld8<T>::load(sp + (int64_t)row * D + scol_of(i));
      }
    }
  };

  auto store_tile = [&](int stage, const h8 (&src)[NLD]) {
    char* ks_ = smem + stage * STAGE;
    char* vs_ = ks_ + K_BYTES;
    if (role_k) {
#pragma unroll
      for (int i = 0; i < NLD; ++i) {
        const int key = srow_of(i), c = scol_of(i) >> 3;
        *reinterpret_cast<h8*>(ks_ + key * (D * 2) + ((c ^ (key & 7)) << 4)) = src[i];
      }
    } else {
#pragma unroll
      for (int u = 0; u < V_UNITS; ++u) {
        const int kg = srow_of(4 * u) >> 2, d0 = scol_of(4 * u);
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
  if constexpr (!ONESET) {
    if (nt > 1) load_tile(1, stg[1]);
  }
  store_tile(0, stg[0]);
  __syncthreads();

  // one step = one key tile; `step` is instantiated for even and odd t so that the register
  // set of tile t + 1 (written to LDS at the end) and of tile t + 2 (requested at the start,
  // into the set tile t just left) are compile-time choices
  auto step = [&](int t, h8 (&set_same)[NLD], h8 (&set_next)[NLD]) {
    if constexpr (ONESET) {
      if (t + 1 < nt) load_tile(t + 1, set_next);
    } else {
      if (t + 2 < nt) load_tile(t + 2, set_same);
    }
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
        // offset = query * Lk + key, the same for every batch and head (kernels.py:457-460)
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int rg = 0; rg < 4; ++rg) {
            const unsigned key0 = (unsigned)(k0 + kb * 32 + 8 * rg + 4 * g);
            const unsigned base_off = (unsigned)q * (unsigned)Lk + key0;
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
    step(t, stg[0], stg[ONESET ? 0 : 1]);
    if (t + 1 < nt) step(t + 1, stg[ONESET ? 0 : 1], stg[0]);
  }

  // ---- out[q][d] = O^T[d][q] / den ------------------------------------------
  if (q < L) {
    int64_t row_off;
    if (BLND) {
      const int b = bh / heads, n = bh - b * heads;
      row_off = (((int64_t)b * L + q) * heads + n) * DG;
    } else {
      row_off = base + (int64_t)q * DG;
    }
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        const int d = i * 32 + 8 * rg + 4 * g;
        if (DG < 32 && d >= DG) continue;
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
__global__ __launch_bounds__(NW * 64, D == 256 ? 1 : NW / 2) void flash_attn_resident_kernel(
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

// ---------------------------------------------------------------------------
// Streaming variant of the resident kernel: fp16 storage, head size 64, K and V of one (batch,
// head) no larger than 320 rows (two of them fill the CU's 160 KB of LDS).
//
// One persistent workgroup of 8 wavefronts per CU walks (batch, head) pairs bh = blockIdx.x,
// blockIdx.x + gridDim.x, ...  K and V of pair i+1 are brought into the second half of LDS by
// direct global->LDS loads (16 bytes per lane, no staging registers, no LDS store instructions)
// while pair i is multiplied, so HBM is kept busy through the arithmetic; the one barrier per
// pair publishes the buffer that has landed and frees the other.  The queries of pair i+1 are
// requested early in the iteration as well (see the pipeline at the end of the kernel).
//
// LDS, per buffer: K [Lp][64] then V [Lp][64] halves, Lp = L rounded up to 64, rows of 128 bytes
// in 16-byte units.  The loads write LDS in lane order, so the swizzle is applied on the source
// side: unit u of K row r holds source unit u ^ ((r >> 1) & 7) (conflict-free ds_read_b128 of one
// unit of 32 consecutive rows), unit u of V row r holds source unit u ^ (2 (r & 3)).  V stays
// row-major: the first operand of O^T += V^T . P^T is read with the transposing LDS load
// (ds_read_b64_tr_b16: within a block of 16 lanes, lane i receives element i % 4 of the 8 bytes
// addressed by lanes i / 4, i / 4 + 4, + 8, + 12), lane s of a block pointing at V[key0 + s / 4]
// [d0 + 4 (s % 4) ..]; the V swizzle spreads the four rows of such a block over all banks.
// Rows L .. Lp-1 are filled with copies of row L-1: their keys are masked (P = 0 exactly) and
// the values are finite.
//
// The causal diagonal is handled per 32 x 32 block instead of per 64-key tile.  The first query
// of a 32-query chunk is a multiple of 32, so in the chunk's last key tile one 32-key block is
// cut by the diagonal -- the same lanes and registers are masked in every chunk, by a compare
// against a constant and a select per score -- and the other block is either
// entirely visible (no mask) or entirely hidden (skipped: its weights are exactly 0 and add
// exactly 0 to the sums, so leaving it out changes no bit of the result).
//
// Chunk c costs c + 1 such blocks; the host deals the chunks to the 8 wavefronts (at most two
// each) so that the four SIMDs -- wavefronts w and w + 4 share one -- carry equal block counts.
// ---------------------------------------------------------------------------
struct StreamPlan {
  signed char chunk[8][2];  // query chunks (of 32) of wavefront w, -1 = none
};

typedef short s4v __attribute__((__vector_size__(4 * sizeof(short))));

// four keys x one d (transposed) from a row-major V tile; see the layout note above
__device__ __forceinline__ h4 lds_read_tr16(const char* p) {
  const s4v r = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (__attribute__((address_space(3))) s4v*)(uintptr_t)p);
  return __builtin_bit_cast(h4, r);
}

// 16 bytes per lane from (wavefront-uniform base) + lane_off straight into LDS at lds_off +
// 16 * lane.  Assembly, so that the compiler's wait-count model never sees an LDS-writing memory
// operation in flight (it would make every LDS read of the arithmetic wait for the prefetch);
// completion is awaited by hand (vmcnt(0)) in front of the barrier that publishes the buffer.
__device__ __forceinline__ void attn_dma16(const void* base, unsigned lane_off, unsigned lds_off) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_off), "v"(lane_off), "s"(base)
               : "memory", "m0");
}

template <bool BLND>
__global__ __launch_bounds__(512, 2) void flash_attn_stream_kernel(
    const _Float16* __restrict__ Q, const _Float16* __restrict__ K,
    const _Float16* __restrict__ V, _Float16* __restrict__ O, int heads, int L, int num_bh,
    float scale, StreamPlan plan) {
  constexpr int D = 64, KS = 4, DB = 2;
  constexpr int MAX_DMA = 10;  // 16-byte loads per lane per pair: Lp / 32, Lp <= 320
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int Lp = (L + BKEY - 1) / BKEY * BKEY;
  const int buf_bytes = Lp * 256;  // K then V, 128 bytes per row
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ql = lane & 31, g = lane >> 5;
  const unsigned smem_base = (unsigned)(uintptr_t)smem;

  // ---- what this wavefront loads: units [(wave * ndma + j) * 64 + lane] of the Lp * 16 units of
  // K followed by V (ndma = Lp / 32 loads per wavefront and pair, the same for all wavefronts)
  const int ndma = Lp >> 5;
  const int k_loads = Lp >> 3;  // the first Lp / 8 of the workgroup's 8 * ndma loads fill K
  // load `inst` covers rows 8 * inst' .. + 7 (inst' counted from the start of K or of V); lane l
  // fills position l % 8 of row 8 * inst' + l / 8 with source unit (l % 8) ^ key(row):
  // K key = (row >> 1) & 7 = (4 * (inst' & 1) + l / 16) & 7, V key = 2 * (row & 3) = 2 * ((l / 8) & 3)
  const int lrow = lane >> 3;
  const unsigned k_unit16 = (unsigned)(((lane & 7) ^ (lane >> 4)) << 4);
  const unsigned v_unit16 = (unsigned)(((lane & 7) ^ (2 * (lrow & 3))) << 4);
  auto issue_pair = [&](int bh, int buf) {
    const char* kb_ = (const char*)(K + (int64_t)bh * L * D);
    const char* vb_ = (const char*)(V + (int64_t)bh * L * D);
    const unsigned dst = smem_base + (unsigned)(buf * buf_bytes) + (unsigned)(wave * ndma) * 1024u;
#pragma unroll
    for (int j = 0; j < MAX_DMA; ++j)
      if (j < ndma) {
        const int inst = wave * ndma + j;
        const bool is_v = inst >= k_loads;
        const int rel = inst - (is_v ? k_loads : 0);
        int row = rel * 8 + lrow;
        row = row < L ? row : L - 1;  // rows L .. Lp-1 repeat the last row
        const unsigned unit16 = is_v ? v_unit16 : (k_unit16 ^ ((unsigned)(rel & 1) << 6));
        attn_dma16(is_v ? vb_ : kb_, (unsigned)row * 128u + unit16, dst + j * 1024);
      }
  };

  // ---- this wavefront's query chunks and their fragments: lane (ql, g) holds d = 16 ks + 8 g + 0..7
  const int c0 = plan.chunk[wave][0], c1 = plan.chunk[wave][1];
  auto load_q = [&](int bh, int c, h8 (&qf)[KS]) {
    int q = c * 32 + ql;
    q = q < L ? q : L - 1;  // rows past the end are computed and never stored
    const _Float16* qp = Q + ((int64_t)bh * L + q) * D + g * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *reinterpret_cast<const h8*>(qp + ks * 16);
  };

  // ---- the block cut by the diagonal: register r of a 32 x 32 score block is key offset
  // 8 (r / 4) + 4 g + r % 4, visible to query offset ql iff that is <= ql -- the same lanes and
  // registers in every chunk
  const int tri_q = ql - 4 * g;

  // ---- LDS read offsets (bytes inside a buffer) of this lane
  // K fragment of 32-key block at row k: row k + ql, unit (2 ks + g) ^ ((ql >> 1) & 7)
  int k_off[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) k_off[ks] = ql * 128 + (((ks * 2 + g) ^ ((ql >> 1) & 7)) << 4);
  // V^T fragment of d block i, keys key0 + 4 g + 0..3: lane s = lane % 16 of its block of 16 points
  // at V[key0 + 4 g + s / 4][32 i + 16 (block % 2) + 4 (s % 4)]
  const int sl = lane & 15, vrow = 4 * g + (sl >> 2);
  int v_off[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i) {
    const int unit = 4 * i + 2 * ((lane >> 4) & 1) + ((sl & 3) >> 1);
    v_off[i] = Lp * 128 + vrow * 128 + ((unit ^ (2 * (vrow & 3))) << 4) + (sl & 1) * 8;
  }
  const float cexp = scale * 1.4426950408889634f;

  // K fragments of the 64-key tile at row k0: [kb][ks]
  auto read_k = [&](const char* buf, int k0, h8 (&kf)[2][KS]) {
    const char* kt = buf + k0 * 128;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        kf[kb][ks] = *reinterpret_cast<const h8*>(kt + kb * 4096 + k_off[ks]);
  };

  // One 64-key tile of one chunk.  MODE 0: both 32-key blocks entirely visible; 1: block 0 cut
  // by the diagonal, block 1 hidden (skipped); 2: block 0 visible, block 1 cut by the diagonal.
  // The K fragments arrive in registers (read one step ahead); the V^T fragments and, if
  // `more`, the next tile's K fragments are requested right behind the score products, so that
  // the LDS round trips run under the softmax arithmetic and no product waits for one.  The
  // scheduling fences keep the compiler from sinking the reads back down to their uses.
  auto step = [&](auto mode_tag, const char* buf, int k0, bool more, h8 (&kf)[2][KS],
                  const h8 (&qf)[KS], f16v (&oacc)[DB], float& mrun, float& den) {
    constexpr int MODE = decltype(mode_tag)::value;
    constexpr int NKB = MODE == 1 ? 1 : 2;
    f16v s[NKB];
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) s[kb][r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int kb = 0; kb < NKB; ++kb)
        s[kb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[kb][ks], qf[ks], s[kb], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    // this lane group's keys of a 16-key step: base + 4 g + 0..3 (lo) and base + 8 + 4 g + 0..3 (hi);
    // block 0's fragments are requested here, block 1's when block 0's products start
    h4 vlo[2][DB], vhi[2][DB];
    auto read_v = [&](int kb) {
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        const char* vt = buf + (k0 + kb * 32 + tt * 16) * 128;
#pragma unroll
        for (int i = 0; i < DB; ++i) {
          vlo[tt][i] = lds_read_tr16(vt + v_off[i]);
          vhi[tt][i] = lds_read_tr16(vt + v_off[i] + 8 * 128);
        }
      }
    };
    read_v(0);
    if (more) read_k(buf, k0 + BKEY, kf);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (MODE != 0) {
#pragma unroll
      for (int r = 0; r < 16; ++r)
        s[NKB - 1][r] = 8 * (r >> 2) + (r & 3) <= tri_q ? s[NKB - 1][r] : -INFINITY;
    }
    float bmax = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) bmax = fmaxf(bmax, s[kb][r]);
    bmax = fmaxf(bmax, __shfl_xor(bmax, 32, kWave));
    const float mnew = bmax > mrun ? bmax : mrun;
    const float mult = __builtin_amdgcn_exp2f((mrun - mnew) * cexp);
    const float m2 = mnew * cexp;
    float psum = 0.f;
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float p = __builtin_amdgcn_exp2f(fmaf(s[kb][r], cexp, -m2));
        s[kb][r] = p;
        psum += p;
      }
    mrun = mnew;
    psum += __shfl_xor(psum, 32, kWave);
    den = den * mult + psum;
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[i][r] *= mult;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb) {
      h8 vf[2][DB];
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int i = 0; i < DB; ++i) {
          const h4 lo = vlo[tt][i], hi = vhi[tt][i];
          vf[tt][i] = h8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
      if (kb + 1 < NKB) {  // the registers are free again: request the next block's fragments
        __builtin_amdgcn_sched_barrier(0);
        read_v(kb + 1);
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        h8 pf;
#pragma unroll
        for (int j = 0; j < 8; ++j) pf[j] = (_Float16)s[kb][8 * tt + j];
#pragma unroll
        for (int i = 0; i < DB; ++i)
          oacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[tt][i], pf, oacc[i], 0, 0, 0);
      }
    }
  };

  auto run_chunk = [&](int bh, int c, const char* buf, const h8 (&qf)[KS]) {
    const int qw0 = c * 32, q = qw0 + ql;
    f16v oacc[DB];
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;
    float mrun = -INFINITY, den = 0.f;
    const int nfull = qw0 >> 6;  // key tiles entirely below the diagonal
    h8 kf[2][KS];
    read_k(buf, 0, kf);
    for (int t = 0; t < nfull; ++t)
      step(std::integral_constant<int, 0>{}, buf, t * BKEY, true, kf, qf, oacc, mrun, den);
    if ((qw0 & 32) == 0)
      step(std::integral_constant<int, 1>{}, buf, nfull * BKEY, false, kf, qf, oacc, mrun, den);
    else
      step(std::integral_constant<int, 2>{}, buf, nfull * BKEY, false, kf, qf, oacc, mrun, den);
    // Output.  A lane holds, per 8 consecutive d, the first (g = 0) or the second (g = 1) four of
    // its query's row; the two lanes of a query trade halves through the 32-lane swap (the upper
    // half of the first operand against the lower half of the second), after which each owns 8
    // consecutive d of every other group: 4 stores of 16 bytes per lane instead of 8 of 8, and
    // 32 contiguous bytes per row and instruction.
    const float inv = __builtin_amdgcn_rcpf(den);
    u4 out[DB][2];
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
      for (int pr = 0; pr < 2; ++pr) {
        h4 x, y;  // d = 32 i + 16 pr + 4 g + 0..3 and the same + 8
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          x[j] = (_Float16)(oacc[i][8 * pr + j] * inv);
          y[j] = (_Float16)(oacc[i][8 * pr + 4 + j] * inv);
        }
        const u2 xd = __builtin_bit_cast(u2, x), yd = __builtin_bit_cast(u2, y);
        const auto r0 = __builtin_amdgcn_permlane32_swap(xd[0], yd[0], false, false);
        const auto r1 = __builtin_amdgcn_permlane32_swap(xd[1], yd[1], false, false);
        // g = 0: own x, then the partner's x (d + 4..7); g = 1: the partner's y, then own y
        out[i][pr] = u4{r0[0], r1[0], r0[1], r1[1]};
      }
    if (q < L) {
      int64_t row_off;
      if (BLND) {
        const int b = bh / heads, n = bh - b * heads;
        row_off = (((int64_t)b * L + q) * heads + n) * D;
      } else {
        row_off = ((int64_t)bh * L + q) * D;
      }
#pragma unroll
      for (int i = 0; i < DB; ++i)
#pragma unroll
        for (int pr = 0; pr < 2; ++pr)
          *reinterpret_cast<u4*>(O + row_off + i * 32 + 16 * pr + 8 * g) = out[i][pr];
    }
  };

  // ---- the pipeline over this workgroup's pairs.  A wavefront's first chunk is its heavy one;
  // the light one (if any) runs first, so that both sets of queries for the next pair are
  // requested early in the iteration: the heavy chunk's into a second register set right behind
  // the K / V loads, the light chunk's into its own registers when it is done with them.
  h8 q_heavy[KS], q_heavy_next[KS], q_light[KS];
  int bh = blockIdx.x;
  if (bh >= num_bh) return;
  issue_pair(bh, 0);
  if (c0 >= 0) load_q(bh, c0, q_heavy_next);
  if (c1 >= 0) load_q(bh, c1, q_light);
  int buf = 0;
  bool stored = false;  // this wavefront's heavy chunk stored its 4 x 16 bytes right before
  while (true) {
    const int bh_next = bh + (int)gridDim.x;
    const bool has_next = bh_next < num_bh;
    // Everything this wavefront LOADED has landed (the pair's K / V units and queries); behind the
    // barrier that holds for every wavefront, and nobody reads the other buffer any more.  Loads
    // and stores retire in issue order, and the only operations younger than the last load are the
    // four output stores of the heavy chunk: waiting until four are outstanding leaves exactly
    // those in flight instead of waiting ~2 us for their acknowledgements once per pair.
    if (stored) asm volatile("s_waitcnt vmcnt(4)\n\ts_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)\n\ts_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    // The compiler cannot see the wait above.  Touching this pair's query registers here makes
    // it place its own wait for them at this point, where it costs nothing; otherwise it would
    // wait at their first use, inside the tile loop, with a count that knows nothing of the
    // prefetch loads issued below, i.e. until those have landed too.
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      asm volatile("" : "+v"(q_heavy_next[ks]));
      asm volatile("" : "+v"(q_light[ks]));
      q_heavy[ks] = q_heavy_next[ks];
    }
    if (has_next) {
      issue_pair(bh_next, buf ^ 1);
      if (c0 >= 0) load_q(bh_next, c0, q_heavy_next);
    }
    const char* b_ = smem + buf * buf_bytes;
    if (c1 >= 0) {
      run_chunk(bh, c1, b_, q_light);
      if (has_next) load_q(bh_next, c1, q_light);
    }
    if (c0 >= 0) run_chunk(bh, c0, b_, q_heavy);
    stored = c0 >= 0;
    if (!has_next) break;
    bh = bh_next;
    buf ^= 1;
  }
}

// ---------------------------------------------------------------------------
// Ring variant for sequences too long for the streaming kernel: fp16 storage, head size 64,
// equal query and key lengths, no dropout.  One workgroup = 4 wavefronts = one (batch, head) x
// 128 queries, as in the tiled kernel, but the 64-key tiles of K and V travel the way the
// streaming kernel moves them: by direct global->LDS loads (no staging registers, no LDS store
// instructions) into a ring of four 16 KB stages -- K tile [64][64] then V tile [64][64] halves,
// rows of 128 bytes, the swizzles applied on the source side -- and V stays row-major and is read
// with the transposing LDS load.  A tile is requested three steps before its P.V products.  Two
// workgroups per CU (198 registers; squeezed into the 168 of three wavefronts per SIMD the kernel
// spills and is slower).  GPT-2 XL's shape (64 x 25 heads, L = 1024): 0.544 -> 0.489 ms.
//
// Loads retire in issue order, so "tiles t and t + 1 have landed" is vmcnt(4): the four loads of
// tile t + 2 are the only younger ones (tile t + 3 is requested behind the barrier that follows
// the wait).  That barrier also says that every wavefront is done with tile t - 1, whose stage
// tile t + 3 then takes.  Causal structure per wavefront (first query qw0 a multiple of 32): tiles below
// qw0 / 64 are entirely visible, tile qw0 / 64 holds the block cut by the diagonal (and, for an
// odd 32-query chunk, one entirely visible block in front of it), later tiles are skipped -- as
// in the streaming kernel, whose arithmetic per tile this is.
// ---------------------------------------------------------------------------
template <bool BLND>
__global__ __launch_bounds__(256, 2) void flash_attn_ring_kernel(
    const _Float16* __restrict__ Q, const _Float16* __restrict__ K,
    const _Float16* __restrict__ V, _Float16* __restrict__ O, int heads, int L, float scale) {
  constexpr int D = 64, KS = 4, DB = 2, NS = 4;
  constexpr int STAGE = 2 * BKEY * D * 2;  // 16 KB: K tile, then V tile
  constexpr int V_AT = BKEY * D * 2;       // byte offset of the V tile inside a stage
  __shared__ __attribute__((aligned(1024))) char smem[NS * STAGE];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ql = lane & 31, g = lane >> 5;
  const unsigned smem_base = (unsigned)(uintptr_t)smem;

  const int bh = blockIdx.x;
  const int q_blocks = (L + BQ - 1) / BQ;
  const int qb = q_blocks - 1 - (int)blockIdx.y;  // heavy (late) query blocks first
  const int q0 = qb * BQ;
  const int qw0 = q0 + wave * 32, q = qw0 + ql;
  const bool wave_active = qw0 < L;
  int last_q = q0 + BQ - 1;
  if (last_q > L - 1) last_q = L - 1;
  const int nt = last_q / BKEY + 1;  // key tiles 0..nt-1 touch this query block

  // ---- queries first (the oldest loads in flight): lane (ql, g) holds d = 16 ks + 8 g + 0..7
  h8 qf[KS];
  {
    const int qr = q < L ? q : L - 1;  // rows past the end are computed and never stored
    const _Float16* qp = Q + ((int64_t)bh * L + qr) * D + g * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *reinterpret_cast<const h8*>(qp + ks * 16);
  }

  // ---- tile loads: a tile is 16 loads of 1 KB (8 rows each), K rows then V rows; wavefront w
  // issues loads 4 w .. 4 w + 3, so wavefronts 0-1 bring K and 2-3 bring V.  Lane l fills
  // position l % 8 of row 8 j + l / 8 with source unit (l % 8) ^ key(row): K key = (row >> 1) & 7
  // = (4 (j & 1) + l / 16) & 7, V key = 2 (row & 3) = 2 ((l / 8) & 3).  Rows past the end of the
  // sequence repeat the last row (their keys are masked, the values finite).
  const bool brings_v = wave >= 2;
  const char* src = (const char*)((brings_v ? V : K) + (int64_t)bh * L * D);
  const int lrow = lane >> 3;
  const unsigned unit16 =
      brings_v ? (unsigned)(((lane & 7) ^ (2 * (lrow & 3))) << 4)
               : (unsigned)(((lane & 7) ^ (lane >> 4)) << 4);
  auto issue_tile = [&](int t) {
    const unsigned dst = smem_base + (unsigned)((t % NS) * STAGE) + (unsigned)(wave * 4) * 1024u;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int rel = (wave & 1) * 4 + j;  // 8-row group inside the K (or V) tile
      int row = t * BKEY + rel * 8 + lrow;
      row = row < L ? row : L - 1;
      const unsigned u = brings_v ? unit16 : (unit16 ^ ((unsigned)(rel & 1) << 6));
      attn_dma16(src, (unsigned)row * 128u + u, dst + j * 1024);
    }
  };

  // ---- LDS read offsets (bytes inside a stage) of this lane, as in the streaming kernel
  const int tri_q = ql - 4 * g;
  int k_off[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) k_off[ks] = ql * 128 + (((ks * 2 + g) ^ ((ql >> 1) & 7)) << 4);
  const int sl = lane & 15, vrow = 4 * g + (sl >> 2);
  int v_off[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i) {
    const int unit = 4 * i + 2 * ((lane >> 4) & 1) + ((sl & 3) >> 1);
    v_off[i] = V_AT + vrow * 128 + ((unit ^ (2 * (vrow & 3))) << 4) + (sl & 1) * 8;
  }
  const float cexp = scale * 1.4426950408889634f;

  f16v oacc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;
  float mrun = -INFINITY, den = 0.f;

  // A 64-key tile is worked on in three parts.  MODE 0: both 32-key blocks entirely visible; 1:
  // block 0 cut by the diagonal, block 1 hidden (skipped: its weights are exactly 0); 2: block 0
  // visible, block 1 cut by the diagonal.
  f16v s[2];  // S^T of the tile whose softmax comes next
  // scores(MODE, stage): S^T = K . Q^T, one block's K fragments at a time (16 registers, not 32)
  auto scores = [&](auto mode_tag, const char* buf) {
    constexpr int NKB = decltype(mode_tag)::value == 1 ? 1 : 2;
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb) {
      h8 kf[KS];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        kf[ks] = *reinterpret_cast<const h8*>(buf + kb * 4096 + k_off[ks]);
#pragma unroll
      for (int r = 0; r < 16; ++r) s[kb][r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        s[kb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[ks], qf[ks], s[kb], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // V^T fragments of one 32-key block of the tile in `buf`
  h4 vlo[2][DB], vhi[2][DB];
  auto read_v = [&](const char* buf, int kb) {
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
      const char* vt = buf + (kb * 32 + tt * 16) * 128;
#pragma unroll
      for (int i = 0; i < DB; ++i) {
        vlo[tt][i] = lds_read_tr16(vt + v_off[i]);
        vhi[tt][i] = lds_read_tr16(vt + v_off[i] + 8 * 128);
      }
    }
  };
  // softmax(MODE): mask, running max, P = exp(S - max) summed into the denominator and rounded to
  // fp16 (pf: the second operand of the P.V products, [block][16-key step]), accumulator rescaled
  h8 pf[2][2];
  auto softmax = [&](auto mode_tag) {
    constexpr int MODE = decltype(mode_tag)::value;
    constexpr int NKB = MODE == 1 ? 1 : 2;
    if constexpr (MODE != 0) {
#pragma unroll
      for (int r = 0; r < 16; ++r)
        s[NKB - 1][r] = 8 * (r >> 2) + (r & 3) <= tri_q ? s[NKB - 1][r] : -INFINITY;
    }
    float bmax = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) bmax = fmaxf(bmax, s[kb][r]);
    bmax = fmaxf(bmax, __shfl_xor(bmax, 32, kWave));
    const float mnew = bmax > mrun ? bmax : mrun;
    const float mult = __builtin_amdgcn_exp2f((mrun - mnew) * cexp);
    const float m2 = mnew * cexp;
    float psum = 0.f;
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float p = __builtin_amdgcn_exp2f(fmaf(s[kb][8 * tt + j], cexp, -m2));
          psum += p;
          pf[kb][tt][j] = (_Float16)p;
        }
    mrun = mnew;
    psum += __shfl_xor(psum, 32, kWave);
    den = den * mult + psum;
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[i][r] *= mult;
  };
  // weighted(MODE, stage): O^T += V^T . P^T; block 0's V^T fragments are in registers already,
  // block 1's are requested when block 0's products start
  auto weighted = [&](auto mode_tag, const char* buf) {
    constexpr int NKB = decltype(mode_tag)::value == 1 ? 1 : 2;
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb) {
      h8 vf[2][DB];
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int i = 0; i < DB; ++i) {
          const h4 lo = vlo[tt][i], hi = vhi[tt][i];
          vf[tt][i] = h8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
      if (kb + 1 < NKB) {
        __builtin_amdgcn_sched_barrier(0);
        read_v(buf, kb + 1);
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int i = 0; i < DB; ++i)
          oacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[tt][i], pf[kb][tt], oacc[i], 0, 0, 0);
    }
  };

  // The order inside a wavefront: softmax of tile t, THEN the score products of tile t + 1, then
  // the P.V products of tile t.  The matrix pipe works through them in that order, so the scores
  // of tile t + 1 are ready when the softmax of tile t + 1 starts (they only queue behind nothing,
  // and the P.V products of tile t run under that softmax) instead of queueing behind the P.V
  // products.  Needs tile t + 1 published one step earlier: four stages, tile t + 3 requested at
  // step t.
  const int nfull = qw0 >> 6;  // key tiles entirely below this wavefront's diagonal
  const int diag_mode = (qw0 & 32) == 0 ? 1 : 2;
  auto stage_of = [&](int t) { return (const char*)smem + (t % NS) * STAGE; };
  auto scores_of = [&](int t) {  // t <= nfull
    if (t < nfull) scores(std::integral_constant<int, 0>{}, stage_of(t));
    else if (diag_mode == 1) scores(std::integral_constant<int, 1>{}, stage_of(t));
    else scores(std::integral_constant<int, 2>{}, stage_of(t));
  };
  issue_tile(0);
  if (nt > 1) issue_tile(1);
  if (nt > 2) issue_tile(2);
  for (int t = 0; t < nt; ++t) {
    // tiles t and t + 1 have landed in this wavefront's part (the queries too: they are older;
    // the four loads of tile t + 2 are the only younger ones); behind the barrier that holds for
    // every part, and nobody reads tile t - 1 any more
    if (t + 2 < nt) asm volatile("s_waitcnt vmcnt(4)\n\ts_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)\n\ts_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if (t == 0) {
      // the compiler cannot see the wait above; touching the query registers here makes it
      // place its own wait for them now instead of inside the first tile
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(qf[ks]));
    }
    if (t + 3 < nt) issue_tile(t + 3);
    if (wave_active && t <= nfull) {
      const char* buf = stage_of(t);
      if (t == 0) scores_of(0);
      read_v(buf, 0);
      __builtin_amdgcn_sched_barrier(0);
      if (t < nfull) {
        softmax(std::integral_constant<int, 0>{});
        __builtin_amdgcn_sched_barrier(0);
        scores_of(t + 1);
        weighted(std::integral_constant<int, 0>{}, buf);
      } else if (diag_mode == 1) {
        softmax(std::integral_constant<int, 1>{});
        __builtin_amdgcn_sched_barrier(0);
        weighted(std::integral_constant<int, 1>{}, buf);
      } else {
        softmax(std::integral_constant<int, 2>{});
        __builtin_amdgcn_sched_barrier(0);
        weighted(std::integral_constant<int, 2>{}, buf);
      }
    }
  }

  // ---- output, as in the streaming kernel: the two lanes of a query trade halves through the
  // 32-lane swap and store 16 bytes each
  const float inv = __builtin_amdgcn_rcpf(den);
  u4 out[DB][2];
#pragma unroll
  for (int i = 0; i < DB; ++i)
#pragma unroll
    for (int pr = 0; pr < 2; ++pr) {
      h4 x, y;  // d = 32 i + 16 pr + 4 g + 0..3 and the same + 8
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        x[j] = (_Float16)(oacc[i][8 * pr + j] * inv);
        y[j] = (_Float16)(oacc[i][8 * pr + 4 + j] * inv);
      }
      const u2 xd = __builtin_bit_cast(u2, x), yd = __builtin_bit_cast(u2, y);
      const auto r0 = __builtin_amdgcn_permlane32_swap(xd[0], yd[0], false, false);
      const auto r1 = __builtin_amdgcn_permlane32_swap(xd[1], yd[1], false, false);
      // g = 0: own x, then the partner's x (d + 4..7); g = 1: the partner's y, then own y
      out[i][pr] = u4{r0[0], r1[0], r0[1], r1[1]};
    }
  if (q < L) {
    int64_t row_off;
    if (BLND) {
      const int b = bh / heads, n = bh - b * heads;
      row_off = (((int64_t)b * L + q) * heads + n) * D;
    } else {
      row_off = ((int64_t)bh * L + q) * D;
    }
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
      for (int pr = 0; pr < 2; ++pr)
        *reinterpret_cast<u4*>(O + row_off + i * 32 + 16 * pr + 8 * g) = out[i][pr];
  }
}

// ---------------------------------------------------------------------------
// Head sizes 128 and 256 in fp16 storage, equal query and key lengths, no dropout.  One
// workgroup = 4 wavefronts = one (batch, head) x 128 queries, as in the tiled kernel, but the
// 64-key tiles of K and V travel by direct global->LDS loads into two stages (K tile [64][D],
// then V tile [64][D], both row-major, the swizzles applied on the source side), V is read with
// the transposing LDS load, and no register holds a tile on its way: what the tiled kernel
// spends on staging and on the index arrays of its staging (96 registers at head size 256,
// which it spills) is free for O^T (D / 2 registers), Q (D / 4) and the fragments.  Head size 128
// runs two workgroups per CU (64 KB of LDS each), head size 256 one (128 KB; a wavefront may
// then use all 512 registers of its SIMD lane).
//
// LDS layout of a stage.  K row r, 16-byte unit u sits at position u ^ (r & 15): the 16 lanes
// that read one unit of 16 consecutive rows (rows alias bank-wise, a row is 256 or 512 bytes)
// touch 16 different bank groups.  V row r, unit u sits at position u ^ (4 (r & 3)): a
// transposing read takes 64 contiguous bytes from each of rows r0 .. r0 + 3 (lanes 0-31) and
// r0 + 4 .. r0 + 7 (lanes 32-63), and the swizzle puts the four rows of a half in four different
// quarters of the banks.  Tile t + 1 is requested when the arithmetic of tile t starts (the
// barrier in front says everyone is done with tile t - 1, whose stage it takes) and awaited
// with vmcnt(0) in front of the next barrier.  Causal structure per wavefront as in the ring
// kernel: tiles below qw0 / 64 entirely visible, tile qw0 / 64 with the block cut by the diagonal.
// ---------------------------------------------------------------------------
template <int D, bool BLND>
__global__ __launch_bounds__(256, D == 128 ? 2 : 1) void flash_attn_wide_kernel(
    const _Float16* __restrict__ Q, const _Float16* __restrict__ K,
    const _Float16* __restrict__ V, _Float16* __restrict__ O, int heads, int L, float scale) {
  static_assert(D == 128 || D == 256, "head sizes 128 and 256");
  constexpr int KS = D / 16, DB = D / 32;
  constexpr int ROWB = D * 2;             // bytes of a row
  constexpr int CH = D / 8;               // 16-byte units of a row
  constexpr int RPI = 1024 / ROWB;        // rows one load instruction of 1 KB covers
  constexpr int TILE = BKEY * ROWB;       // bytes of a K (or V) tile
  constexpr int STAGE = 2 * TILE;
  constexpr int NDMA = D / 16;            // load instructions per wavefront and tile
  extern __shared__ __attribute__((aligned(1024))) char smem[];  // 2 * STAGE bytes
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ql = lane & 31, g = lane >> 5;
  const unsigned smem_base = (unsigned)(uintptr_t)smem;

  const int bh = blockIdx.y;
  const int q_blocks = (L + BQ - 1) / BQ;
  const int qb = q_blocks - 1 - (int)blockIdx.x;  // heavy (late) query blocks first
  const int q0 = qb * BQ;
  const int qw0 = q0 + wave * 32, q = qw0 + ql;
  const bool wave_active = qw0 < L;
  int last_q = q0 + BQ - 1;
  if (last_q > L - 1) last_q = L - 1;
  const int nt = last_q / BKEY + 1;  // key tiles 0..nt-1 touch this query block

  // ---- queries (the oldest loads in flight): lane (ql, g) holds d = 16 ks + 8 g + 0..7
  h8 qf[KS];
  {
    const int qr = q < L ? q : L - 1;  // rows past the end are computed and never stored
    const _Float16* qp = Q + ((int64_t)bh * L + qr) * D + g * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *reinterpret_cast<const h8*>(qp + ks * 16);
  }

  // ---- tile loads: wavefronts 0-1 bring the K tile, 2-3 the V tile, 32 rows each; load j of a
  // wavefront covers rows 32 (wave % 2) + RPI j + lane / CH, lane l filling position l % CH with
  // source unit (l % CH) ^ key(row): K key = row & 15, V key = 4 (row & 3).  RPI j contributes
  // compile-time bits to the key, lane / CH the lane's.  Rows past the end of the sequence
  // repeat the last row (their keys are masked, the values finite).
  const bool brings_v = wave >= 2;
  const char* src = (const char*)((brings_v ? V : K) + (int64_t)bh * L * D);
  const int lrow = lane / CH;
  const unsigned unit16 = brings_v ? (unsigned)(((lane % CH) ^ (4 * (lrow & 3))) << 4)
                                   : (unsigned)(((lane % CH) ^ lrow) << 4);
  auto issue_tile = [&](int t) {
    const unsigned dst = smem_base + (unsigned)((t & 1) * STAGE) + (brings_v ? (unsigned)TILE : 0u) +
                         (unsigned)((wave & 1) * NDMA) * 1024u;
#pragma unroll
    for (int j = 0; j < NDMA; ++j) {
      int row = t * BKEY + (wave & 1) * 32 + j * RPI + lrow;
      row = row < L ? row : L - 1;
      const unsigned key_j = brings_v ? (unsigned)(4 * ((j * RPI) & 3)) : (unsigned)((j * RPI) & 15);
      attn_dma16(src, (unsigned)row * (unsigned)ROWB + (unit16 ^ (key_j << 4)), dst + j * 1024);
    }
  };

  // ---- LDS read offsets (bytes inside a tile) of this lane
  // K fragment, k-step ks, of the 32-key block at row k: row k + ql, unit (2 ks + g) ^ (ql & 15);
  // bits 1-3 of the unit come from ks % 8, bit 4 (head size 256) from ks / 8
  const int tri_q = ql - 4 * g;
  int k_off[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) k_off[ks] = ql * ROWB + (((ks * 2 + g) ^ (ql & 15)) << 4);
  // V^T fragment of d block i, keys key0 + 4 g + 0..3: lane s = lane % 16 of its block of 16
  // points at V[key0 + 4 g + s / 4][32 i + 16 (block % 2) + 4 (s % 4)]: unit 4 i + 2 (block % 2)
  // + (s % 4) / 2, swizzled to 4 (i ^ (row & 3)) + ...; i % 4 varies the lane's offset, i / 4 adds
  // 256 bytes
  const int sl = lane & 15, vrow = 4 * g + (sl >> 2);
  int v_off[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int unit = 4 * (i ^ (vrow & 3)) + 2 * ((lane >> 4) & 1) + ((sl & 3) >> 1);
    v_off[i] = TILE + vrow * ROWB + (unit << 4) + (sl & 1) * 8;
  }
  const float cexp = scale * 1.4426950408889634f;

  f16v oacc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;
  float mrun = -INFINITY, den = 0.f;

  // One 64-key tile.  MODE 0: both 32-key blocks entirely visible; 1: block 0 cut by the
  // diagonal, block 1 hidden (skipped: its weights are exactly 0); 2: block 0 visible, block 1
  // cut by the diagonal.
  auto step = [&](auto mode_tag, const char* buf) {
    constexpr int MODE = decltype(mode_tag)::value;
    constexpr int NKB = MODE == 1 ? 1 : 2;
    f16v s[NKB];
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb) {
#pragma unroll
      for (int r = 0; r < 16; ++r) s[kb][r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const h8 kf = *reinterpret_cast<const h8*>(buf + kb * 32 * ROWB + k_off[ks & 7] +
                                                   (ks >> 3) * 256);
        s[kb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[ks], s[kb], 0, 0, 0);
      }
    }
    if constexpr (MODE != 0) {
#pragma unroll
      for (int r = 0; r < 16; ++r)
        s[NKB - 1][r] = 8 * (r >> 2) + (r & 3) <= tri_q ? s[NKB - 1][r] : -INFINITY;
    }
    float bmax = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) bmax = fmaxf(bmax, s[kb][r]);
    bmax = fmaxf(bmax, __shfl_xor(bmax, 32, kWave));
    const float mnew = bmax > mrun ? bmax : mrun;
    const float mult = __builtin_amdgcn_exp2f((mrun - mnew) * cexp);
    const float m2 = mnew * cexp;
    float psum = 0.f;
    h8 pf[NKB][2];
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float p = __builtin_amdgcn_exp2f(fmaf(s[kb][8 * tt + j], cexp, -m2));
          psum += p;
          pf[kb][tt][j] = (_Float16)p;
        }
    mrun = mnew;
    psum += __shfl_xor(psum, 32, kWave);
    den = den * mult + psum;
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[i][r] *= mult;
    // O^T += V^T . P^T: this lane group's keys of a 16-key step are base + 4 g + 0..3 (lo) and
    // base + 8 + 4 g + 0..3 (hi)
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        const char* vt = buf + (kb * 32 + tt * 16) * ROWB;
#pragma unroll
        for (int i = 0; i < DB; ++i) {
          const h4 lo = lds_read_tr16(vt + v_off[i & 3] + (i >> 2) * 256);
          const h4 hi = lds_read_tr16(vt + v_off[i & 3] + (i >> 2) * 256 + 8 * ROWB);
          const h8 vf = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
          oacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf[kb][tt], oacc[i], 0, 0, 0);
        }
      }
  };

  const int nfull = qw0 >> 6;  // key tiles entirely below this wavefront's diagonal
  issue_tile(0);
  for (int t = 0; t < nt; ++t) {
    // tile t has landed in this wavefront's part (the queries too: they are older); behind the
    // barrier that holds for every part, and nobody reads tile t - 1 any more
    asm volatile("s_waitcnt vmcnt(0)\n\ts_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if (t == 0) {
      // the compiler cannot see the wait above; touching the query registers here makes it
      // place its own wait for them now instead of inside the first tile
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(qf[ks]));
    }
    if (t + 1 < nt) issue_tile(t + 1);
    if (wave_active && t <= nfull) {
      const char* buf = smem + (t & 1) * STAGE;
      if (t < nfull) step(std::integral_constant<int, 0>{}, buf);
      else if ((qw0 & 32) == 0) step(std::integral_constant<int, 1>{}, buf);
      else step(std::integral_constant<int, 2>{}, buf);
    }
  }

  // ---- output, as in the streaming kernel: the two lanes of a query trade halves through the
  // 32-lane swap and store 16 bytes each
  const float inv = __builtin_amdgcn_rcpf(den);
  if (q < L) {
    int64_t row_off;
    if (BLND) {
      const int b = bh / heads, n = bh - b * heads;
      row_off = (((int64_t)b * L + q) * heads + n) * D;
    } else {
      row_off = ((int64_t)bh * L + q) * D;
    }
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
      for (int pr = 0; pr < 2; ++pr) {
        h4 x, y;  // d = 32 i + 16 pr + 4 g + 0..3 and the same + 8
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          x[j] = (_Float16)(oacc[i][8 * pr + j] * inv);
          y[j] = (_Float16)(oacc[i][8 * pr + 4 + j] * inv);
        }
        const u2 xd = __builtin_bit_cast(u2, x), yd = __builtin_bit_cast(u2, y);
        const auto r0 = __builtin_amdgcn_permlane32_swap(xd[0], yd[0], false, false);
        const auto r1 = __builtin_amdgcn_permlane32_swap(xd[1], yd[1], false, false);
        // g = 0: own x, then the partner's x (d + 4..7); g = 1: the partner's y, then own y
        *reinterpret_cast<u4*>(O + row_off + i * 32 + 16 * pr + 8 * g) =
            u4{r0[0], r1[0], r0[1], r1[1]};
      }
  }
}

// Deals the query chunks of a sequence of L <= 320 rows to the 8 wavefronts: chunk c costs
// c + 1 blocks; heaviest first, each to the SIMD (wavefronts w and w + 4) with the smallest
// load so far that still has a free slot, inside the SIMD to the lighter wavefront.
inline StreamPlan make_stream_plan(int L) {
  StreamPlan p;
  int wave_load[8] = {0, 0, 0, 0, 0, 0, 0, 0}, wave_n[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int w = 0; w < 8; ++w) p.chunk[w][0] = p.chunk[w][1] = -1;
  for (int c = (L + 31) / 32 - 1; c >= 0; --c) {
    int best = -1;
    for (int sd = 0; sd < 4; ++sd) {
      if (wave_n[sd] >= 2 && wave_n[sd + 4] >= 2) continue;
      if (best < 0 || wave_load[sd] + wave_load[sd + 4] < wave_load[best] + wave_load[best + 4])
        best = sd;
    }
    int w = best;
    if (wave_n[w] >= 2 || (wave_n[w + 4] < 2 && wave_load[w + 4] < wave_load[w])) w = best + 4;
    p.chunk[w][wave_n[w]++] = (signed char)c;
    wave_load[w] += c + 1;
  }
  return p;
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

template <int D, typename T, bool BLND, bool DROP, bool UNEQ, int DG = D>
int launch_tiled_as(const void* q, const void* k, const void* v, void* out, int64_t BN, int heads,
                    int L, int Lk, float scale, DropoutArgs drop, hipStream_t st) {
  dim3 grid((unsigned)BN, (unsigned)((L + BQ - 1) / BQ));
  constexpr int lds = 2 * 2 * BKEY * D * 2;  // two stages of a K tile and a V^T tile
  auto kern = flash_attn_kernel<D, T, BLND, DROP, UNEQ, DG>;
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
                     (T*)out, heads, L, Lk, scale, drop);
  return 0;
}

// L query rows, Lk key rows per (batch, head); equal lengths take the variant without the
// zero-row selects.
template <int D, typename T, bool BLND, bool DROP>
int launch_tiled(const void* q, const void* k, const void* v, void* out, int64_t BN, int heads,
                 int L, int Lk, float scale, DropoutArgs drop, hipStream_t st) {
  if (L != Lk)
    return launch_tiled_as<D, T, BLND, DROP, true>(q, k, v, out, BN, heads, L, Lk, scale, drop, st);
  return launch_tiled_as<D, T, BLND, DROP, false>(q, k, v, out, BN, heads, L, Lk, scale, drop, st);
}

// CUs of the current device, or a negative error code.
inline int attn_cu_count() {
  static int num_cus = 0;  // idempotent one-time setup; a race only repeats it
  if (num_cus == 0) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        cus < 1) {
      set_error("flash_attn: cannot query the CU count");
      return -4;
    }
    num_cus = cus;
  }
  return num_cus;
}

template <bool BLND>
int launch_stream_attn(const void* q, const void* k, const void* v, void* out, int64_t BN,
                       int heads, int L, float scale, hipStream_t st) {
  auto kern = flash_attn_stream_kernel<BLND>;
  static bool attr_done = false;  // idempotent; a race only repeats the call
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) {
      set_error("hipFuncSetAttribute(160 KB LDS): %s", hipGetErrorString(e));
      return -4;
    }
    attr_done = true;
  }
  const int cus = attn_cu_count();
  if (cus < 0) return cus;
  const int Lp = (L + BKEY - 1) / BKEY * BKEY;
  const int grid = BN < cus ? (int)BN : cus;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(512), (size_t)Lp * 512, st,
                     (const _Float16*)q, (const _Float16*)k, (const _Float16*)v, (_Float16*)out,
                     heads, L, (int)BN, scale, make_stream_plan(L));
  return 0;
}

template <bool BLND>
int launch_ring_attn(const void* q, const void* k, const void* v, void* out, int64_t BN, int heads,
                     int L, float scale, hipStream_t st) {
  dim3 grid((unsigned)BN, (unsigned)((L + BQ - 1) / BQ));
  hipLaunchKernelGGL(flash_attn_ring_kernel<BLND>, grid, dim3(256), 0, st, (const _Float16*)q,
                     (const _Float16*)k, (const _Float16*)v, (_Float16*)out, heads, L, scale);
  return 0;
}

template <int D, bool BLND>
int launch_wide_attn(const void* q, const void* k, const void* v, void* out, int64_t BN, int heads,
                     int L, float scale, hipStream_t st) {
  auto kern = flash_attn_wide_kernel<D, BLND>;
  constexpr int lds = 2 * 2 * BKEY * D * 2;  // two stages of a K tile and a V tile
  static bool attr_done = false;  // idempotent; a race only repeats the call
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) {
      set_error("hipFuncSetAttribute(%d bytes LDS): %s", lds, hipGetErrorString(e));
      return -4;
    }
    attr_done = true;
  }
  if (BN > 65535) {  // the (batch, head) pairs go to the grid's second dimension
    set_error("flash_attn: %lld (batch, head) pairs at head size %d: at most 65535",
              (long long)BN, D);
    return -2;
  }
  dim3 grid((unsigned)((L + BQ - 1) / BQ), (unsigned)BN);
  hipLaunchKernelGGL(kern, grid, dim3(256), lds, st, (const _Float16*)q, (const _Float16*)k,
                     (const _Float16*)v, (_Float16*)out, heads, L, scale);
  return 0;
}

template <int D, typename T>
int launch_d(const void* q, const void* k, const void* v, void* out, int64_t BN,
             int heads, int L, int Lk, float scale, Dropout drop, bool blnd, hipStream_t st) {
  const DropoutArgs da = {drop.p, (unsigned)drop.seed, (unsigned)(drop.seed >> 32)};
  if (drop.p > 0.f) {  // training-mode path: the tiled kernel carries the generator
    return blnd ? launch_tiled<D, T, true, true>(q, k, v, out, BN, heads, L, Lk, scale, da, st)
                : launch_tiled<D, T, false, true>(q, k, v, out, BN, heads, L, Lk, scale, da, st);
  }
  if (L != Lk)  // query and key sequences of different lengths: the tiled kernel knows both
    return blnd ? launch_tiled<D, T, true, false>(q, k, v, out, BN, heads, L, Lk, scale, da, st)
                : launch_tiled<D, T, false, false>(q, k, v, out, BN, heads, L, Lk, scale, da, st);
  if constexpr (D == 64 && sizeof(T) == 2) {
    // fp16, head size 64, two (batch, head) pairs fit the LDS, enough pairs to keep every
    // persistent workgroup busy for a while: the streaming kernel
    if (L <= 320 && BN >= 64)
      return blnd ? launch_stream_attn<true>(q, k, v, out, BN, heads, L, scale, st)
                  : launch_stream_attn<false>(q, k, v, out, BN, heads, L, scale, st);
    // sequences that do not fit the resident variant either: key tiles through the ring
    if (resident_lds_bytes(L, D) == 0)
      return blnd ? launch_ring_attn<true>(q, k, v, out, BN, heads, L, scale, st)
                  : launch_ring_attn<false>(q, k, v, out, BN, heads, L, scale, st);
  }
  if (const size_t lds = resident_lds_bytes(L, D)) {
    return blnd ? launch_resident<D, T, true>(q, k, v, out, BN, heads, L, scale, lds, st)
                : launch_resident<D, T, false>(q, k, v, out, BN, heads, L, scale, lds, st);
  }
  if constexpr (D >= 128 && sizeof(T) == 2) {
    // fp16, head sizes 128 and 256, longer sequences: tiles by direct loads, no staging registers
    // (pairs in the grid's second dimension; 32-bit byte offsets inside a pair)
    if (BN <= 65535 && (int64_t)L * D * 2 < (1ll << 31))
      return blnd ? launch_wide_attn<D, true>(q, k, v, out, BN, heads, L, scale, st)
                  : launch_wide_attn<D, false>(q, k, v, out, BN, heads, L, scale, st);
  }
  return blnd ? launch_tiled<D, T, true, false>(q, k, v, out, BN, heads, L, Lk, scale, da, st)
              : launch_tiled<D, T, false, false>(q, k, v, out, BN, heads, L, Lk, scale, da, st);
}

// Head sizes 16 and 32: the tiled kernel on its 64-wide staging layout, reading the tensors at
// their own row pitch (the variant that knows both sequence lengths serves equal ones too).
template <int DG, typename T>
int launch_small_head(const void* q, const void* k, const void* v, void* out, int64_t BN, int heads,
                      int L, int Lk, float scale, Dropout drop, bool blnd, hipStream_t st) {
  const DropoutArgs da = {drop.p, (unsigned)drop.seed, (unsigned)(drop.seed >> 32)};
  if (drop.p > 0.f)
    return blnd ? launch_tiled_as<64, T, true, true, true, DG>(q, k, v, out, BN, heads, L, Lk,
                                                               scale, da, st)
                : launch_tiled_as<64, T, false, true, true, DG>(q, k, v, out, BN, heads, L, Lk,
                                                                scale, da, st);
  return blnd ? launch_tiled_as<64, T, true, false, true, DG>(q, k, v, out, BN, heads, L, Lk,
                                                              scale, da, st)
              : launch_tiled_as<64, T, false, false, true, DG>(q, k, v, out, BN, heads, L, Lk,
                                                               scale, da, st);
}

template <typename T>
int launch_t(const void* q, const void* k, const void* v, void* out, int64_t BN,
             int heads, int L, int Lk, int d, float scale, Dropout drop, bool blnd, hipStream_t st) {
  switch (d) {
    case 16: return launch_small_head<16, T>(q, k, v, out, BN, heads, L, Lk, scale, drop, blnd, st);
    case 32: return launch_small_head<32, T>(q, k, v, out, BN, heads, L, Lk, scale, drop, blnd, st);
    case 64: return launch_d<64, T>(q, k, v, out, BN, heads, L, Lk, scale, drop, blnd, st);
    case 128: return launch_d<128, T>(q, k, v, out, BN, heads, L, Lk, scale, drop, blnd, st);
    case 256: return launch_d<256, T>(q, k, v, out, BN, heads, L, Lk, scale, drop, blnd, st);
    default:
      set_error("flash_attn: head size %d not built (16, 32, 64, 128 and 256 are)", d);
      return -2;
  }
}

}  // namespace

int launch_flash_attn(const void* q, const void* k, const void* v, void* out, int64_t B,
                      int64_t N, int64_t L, int64_t Lk, int d, float scale, Dropout drop,
                      bool out_blnd, bool f16, hipStream_t st) {
  const int64_t BN = B * N;
  if (BN > 0x7fffffffll || L > (1 << 24) || Lk > (1 << 24)) {
    set_error("flash_attn: B*N=%lld, Lq=%lld or Lk=%lld beyond the grid limits", (long long)BN,
              (long long)L, (long long)Lk);
    return -2;
  }
  return f16 ? launch_t<_Float16>(q, k, v, out, BN, (int)N, (int)L, (int)Lk, d, scale, drop,
                                  out_blnd, st)
             : launch_t<float>(q, k, v, out, BN, (int)N, (int)L, (int)Lk, d, scale, drop, out_blnd,
                               st);
}

}  // namespace gptmi
