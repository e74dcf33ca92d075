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
// Structure of one workgroup of gemm_kernel (WM x WN wavefronts):
//   * a BM x BN output tile; K is walked in steps of BKS (32 or 64) through NST LDS stages
//     filled by direct global->LDS loads (16 B per lane, no VGPR staging).  The barrier that
//     publishes k-tile kt+1 sits in front of the LAST k-slice of k-tile kt, whose fragments are
//     in registers by then; the first fragments of kt+1 are read right behind it and the stage
//     of kt is refilled with kt+NST while that last slice is multiplied, its load instructions
//     dealt between the MFMAs.  No MFMA waits for a barrier plus an LDS round trip;
//   * LDS rows are BKS halves wide; the 16-byte chunks of a row are XOR-swizzled
//     with a key taken from the row number so that the 16 lanes the LDS serves
//     per clock (64 banks x 4 B) never share a bank:
//         128-byte rows: chunk c of row r at c ^ ((r >> 1) & 7)
//          64-byte rows: chunk c of row r at c ^ ((r >> 2) & 3)
//   * each wavefront owns a (BM/WM) x (BN/WN) sub-tile as 32x32 MFMA blocks.
//     The MFMA is issued as D[n][m] (weight rows as the first operand) so a
//     lane ends up with 4 consecutive n for one m;
//   * the epilogue applies bias/GELU in that layout, transposes through a wavefront-private
//     LDS slab and stores row-major runs.  Four forms (dispatch in store_wave_tile and at the
//     end of the kernels): fp16 output, whole tile, no residual -> rounded first, slab of halves,
//     16-byte stores (store_wave_tile_h); the same with a residual -> the residual tile is
//     brought into the operand stages by direct loads as these fall free and added in the
//     accumulator layout before the one rounding (store_wave_tile_rl); everything else that is a
//     whole tile with aligned pointers -> fp32 slab, 8- or 16-byte accesses (store_wave_tile_v
//     FAST); tiles on the matrix edge, odd N, unaligned pointers, dropout -> the same slab with
//     element-wise predicated accesses;
//   * workgroup ids are remapped so each XCD (ids are dealt round-robin over
//     the 8 XCDs) gets a contiguous range of tiles; inside a group of column tiles whose
//     weight panels fit the XCD's L2 the column runs fastest, so the tiles that share a row
//     block of A run on the same L2 at the same time.
// gemm_stream_kernel and gemm_stream_res_kernel (further down) are the persistent forms of the
// 256 x 256 x 64 configuration for whole row tiles, without and with a residual: one workgroup
// per CU walks tiles and the pipeline runs across tile boundaries.  They multiply with
// v_mfma_f32_16x16x32_f16 (a sub-tile is 16 x 16 blocks there; same LDS layout, same products,
// less power per product on operands that toggle bits, so a higher clock).  launch_shape (at the
// end) picks kernel and configuration.
#include <stdlib.h>

#include <type_traits>

#include "common.h"
#include "launch.h"
#include "layernorm.h"

namespace gptmi {

namespace {

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
  int vec8_ok; // fp16 output: N, head size and the output pointers also allow 16-byte stores
  int m_off;   // head-major scatter: row 0 of this launch is row m_off of the [B*L] token rows
  DropoutArgs drop;  // p > 0: dropout between GELU and residual (predicated epilogue only)
};

// LayerNorm in the operand prologue (gemm_kernel<..., LNA = true>): weight, bias, epsilon and
// the lanes per row the LayerNorm kernel would use for rows of this width (the sums are then
// formed in the same order and the normalised operand has the same bits as that kernel's output).
struct LnArgs {
  const void* w;
  const void* b;
  float eps;
  int lpr;
};

// Direct global->LDS load of 16 bytes per lane: lane l's bytes land at LDS
// byte offset lds_off + 16*l (lds_off is wavefront-uniform and travels in M0).
// Issued as inline assembly so that the compiler's wait-count tracking does not
// see an LDS-writing memory instruction in flight: with the builtin, every LDS
// wait inside the pipelined loop degrades to "wait for everything".  Completion
// is tracked by hand with vmcnt (wait_vmcnt) ahead of the workgroup barrier.
__device__ __forceinline__ void lds_dma16(const void* gsrc, unsigned lds_off) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
               :
               : "s"(lds_off), "v"(gsrc)
               : "memory", "m0");
}

// The same with a wavefront-uniform 64-bit base in scalar registers and a 32-bit per-lane
// byte offset: one VGPR per load instead of an address pair, and the k-step is a scalar add.
__device__ __forceinline__ void lds_dma16_base(const void* base, unsigned lane_off,
                                               unsigned lds_off) {
  // s_mov + s_nop 3 = 5 wait states between a VALU write of `base` (v_readfirstlane, should
  // the compiler ever have to move it out of a vector register) and the load that reads it
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_off), "v"(lane_off), "s"(base)
               : "memory", "m0");
}

// Streaming store of 4 or 8 output elements at (wavefront-uniform 64-bit base) + (32-bit lane
// offset).  Written as assembly because the compiler otherwise materialises one 64-bit address
// pair per store of an unrolled epilogue and spills.  Two hazards the compiler handles for its
// own instructions and cannot see inside assembly:
//   * a scalar register written by a VALU instruction (v_readfirstlane) must not be read by a
//     memory instruction within the next 5 wait states -- the leading s_nop 4 covers a base
//     that the compiler had to move out of a vector register;
//   * a store of more than 64 bits reads its data registers a little after issue -- the
//     trailing s_nop 1 keeps the next VALU instruction from overwriting them.
__device__ __forceinline__ void store_nt_base(void* base, unsigned lane_off, h4 v) {
  asm volatile("s_nop 4\n\tglobal_store_dwordx2 %0, %1, %2 nt"
               :
               : "v"(lane_off), "v"(v), "s"(base)
               : "memory");
}
__device__ __forceinline__ void store_nt_base(void* base, unsigned lane_off, f4 v) {
  asm volatile("s_nop 4\n\tglobal_store_dwordx4 %0, %1, %2 nt\n\ts_nop 1"
               :
               : "v"(lane_off), "v"(v), "s"(base)
               : "memory");
}
__device__ __forceinline__ void store_nt_base(void* base, unsigned lane_off, h8 v) {
  asm volatile("s_nop 4\n\tglobal_store_dwordx4 %0, %1, %2 nt\n\ts_nop 1"
               :
               : "v"(lane_off), "v"(v), "s"(base)
               : "memory");
}

// Workgroup barrier that does not drain the vector-memory counter: the
// compiler's own barrier waits for vmcnt(0), which would serialise the
// global->LDS prefetch of the younger pipeline stages behind it.
__device__ __forceinline__ void block_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N <= 63, "vmcnt is a 6-bit counter");
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

template <typename T> struct Pack4;
template <> struct Pack4<_Float16> { typedef h4 type; };
template <> struct Pack4<float> { typedef f4 type; };

// Address of out[m][n] (plain) or of the q/k/v element that column n of row m
// scatters to (qkv mode; n is a multiple of 4 and head sizes are too, so 4
// consecutive columns stay inside one head).
template <typename T, bool QKV>
__device__ __forceinline__ T* out_ptr(const EpiDev& ep, int64_t m, int n, int N) {
  if constexpr (!QKV) {
    return (T*)ep.out + (m * (int64_t)N + n);
  } else {
    // m < 2^31 (checked by the launcher) and L <= m's range: 32-bit divisions
    const unsigned hd = (unsigned)(ep.heads * ep.d);
    const unsigned which = (unsigned)n / hd;
    const unsigned within = (unsigned)n - which * hd;
    const unsigned head = within / (unsigned)ep.d;
    const unsigned dd = within - head * (unsigned)ep.d;
    const unsigned L = (unsigned)ep.L;
    const unsigned b = (unsigned)m / L;
    const unsigned l = (unsigned)m - b * L;
    T* base = (T*)(which == 0 ? ep.q : (which == 1 ? ep.k : ep.v));
    return base + ((((int64_t)b * ep.heads + head) * ep.L + l) * ep.d + dd);
  }
}

// Head-major destination of column n, row 0 of batch 0: q/k/v base + (head * L + 0) * d + dd.
template <typename T>
__device__ __forceinline__ T* qkv_column_base(const EpiDev& ep, int n) {
  const unsigned hd = (unsigned)(ep.heads * ep.d);
  const unsigned which = (unsigned)n / hd;
  const unsigned within = (unsigned)n - which * hd;
  const unsigned head = within / (unsigned)ep.d;
  const unsigned dd = within - head * (unsigned)ep.d;
  T* base = (T*)(which == 0 ? ep.q : (which == 1 ? ep.k : ep.v));
  return base + ((int64_t)head * ep.L * ep.d + dd);
}

// Bias of a wavefront's columns in the accumulator layout: [i][g] -> the 4 consecutive columns
// nw0 + 32 i + 8 g + 4 fhalf + 0..3, as stored (load_bias) and as fp32 (bias_to_f32).  ONE branch
// stands around all the loads: with a test of ep.bias per load, every load got a basic block of
// its own and, behind it, a wait for everything in flight -- 8 memory round trips per tile, one
// after the other.  Needs 4-element vector access (N % 4 == 0, aligned bias: EpiDev::vec_ok).
template <typename T, int NB>
__device__ __forceinline__ void load_bias(const EpiDev& ep, int nw0, int fhalf,
                                          typename Pack4<T>::type (&raw)[NB][4]) {
  typedef typename Pack4<T>::type P4;
  if (ep.bias) {
    const T* bp = (const T*)ep.bias + (nw0 + fhalf * 4);
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int g = 0; g < 4; ++g) raw[i][g] = *reinterpret_cast<const P4*>(bp + i * 32 + g * 8);
  } else {
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int e = 0; e < 4; ++e) raw[i][g][e] = 0;
  }
}
template <typename P4, int NB>
__device__ __forceinline__ void bias_to_f32(const P4 (&raw)[NB][4], f4 (&bias_r)[NB][4]) {
#pragma unroll
  for (int i = 0; i < NB; ++i)
#pragma unroll
    for (int g = 0; g < 4; ++g)
#pragma unroll
      for (int e = 0; e < 4; ++e) bias_r[i][g][e] = (float)raw[i][g][e];
}

// The same for the accumulators of v_mfma_f32_16x16x32 (the streaming kernels): of a 32 x 32
// block a lane holds four quads, (mh, nh) -> row 16 mh + lane % 16, columns 16 nh + 4 (lane / 16)
// + 0..3, so two bias quads per block: [i][nh] -> columns nw0 + 32 i + 16 nh + 4 (lane / 16) + 0..3.
template <typename T, int NB>
__device__ __forceinline__ void load_bias16(const EpiDev& ep, int nw0, int lq,
                                            typename Pack4<T>::type (&raw)[NB][2]) {
  typedef typename Pack4<T>::type P4;
  if (ep.bias) {
    const T* bp = (const T*)ep.bias + (nw0 + lq * 4);
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int nh = 0; nh < 2; ++nh) raw[i][nh] = *reinterpret_cast<const P4*>(bp + i * 32 + nh * 16);
  } else {
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int nh = 0; nh < 2; ++nh)
#pragma unroll
        for (int e = 0; e < 4; ++e) raw[i][nh][e] = 0;
  }
}
template <typename P4, int NB>
__device__ __forceinline__ void bias_to_f32_16(const P4 (&raw)[NB][2], f4 (&bias_r)[NB][2]) {
#pragma unroll
  for (int i = 0; i < NB; ++i)
#pragma unroll
    for (int nh = 0; nh < 2; ++nh)
#pragma unroll
      for (int e = 0; e < 4; ++e) bias_r[i][nh][e] = (float)raw[i][nh][e];
}

constexpr int EP_STRIDE = 64 * 4 + 16;  // bytes of one staged epilogue row (64 fp32 + pad)
constexpr int EP_SLAB = 32 * EP_STRIDE; // one wavefront's staging slab

// Epilogue of one wavefront's (32*MB) x (32*NB) sub-tile whose first element is
// (mw0, nw0).  A lane holds, per 32x32 block, m = lane%32 and for g = 0..3 the 4
// columns 8g + 4*(lane/32) + 0..3.  Bias and GELU are applied in that layout,
// the fp32 values are staged through the wavefront's private LDS slab (32 rows
// x 64 columns, rows padded by 16 B) and read back row-major: 16 lanes cover one
// row's 64 columns, so residual loads and output stores are contiguous 128-byte
// (fp16) or 256-byte (fp32) runs per row.
//   FAST: the workgroup tile lies entirely inside M x N and every pointer
//   allows 4-element vector accesses -- straight-line code, no predicates.
template <int MB, int NB, typename T, bool QKV, bool FAST, bool GELU, bool RES, bool DROP = false>
__device__ __forceinline__ void store_wave_tile_v(f16v (&acc)[NB][MB], const EpiDev& ep,
                                                  int64_t mw0, int nw0, int M, int N, char* slab,
                                                  int lane) {
  typedef typename Pack4<T>::type P4;
  static_assert(NB % 2 == 0, "wave tile must be a multiple of 64 columns");
  const int frow = lane & 31, fhalf = lane >> 5;
  const int rrow = lane >> 4, rcol = (lane & 15) * 4;

  // bias of this lane's columns, fetched once: [i][g] -> 4 consecutive columns
  f4 bias_r[NB][4];
  if constexpr (FAST) {
    P4 raw[NB][4];
    load_bias<T, NB>(ep, nw0, fhalf, raw);
    bias_to_f32(raw, bias_r);
  } else {
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n = nw0 + i * 32 + g * 8 + fhalf * 4;
        f4 b = {0.f, 0.f, 0.f, 0.f};
        if (ep.bias) {
          const T* bp = (const T*)ep.bias + n;
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < N) b[e] = (float)bp[e];
        }
        bias_r[i][g] = b;
      }
  }

  // head-major scatter: the column part of the address once per 64-column slab, the row part
  // (b, l) = divmod(m, L) once for the lane's first row and then by stepping -- the sub-tile
  // spans fewer than 256 rows, so it crosses at most one batch boundary when L >= 256
  T* qkv_col[NB / 2];
  unsigned b0 = 0, l0 = 0;
  const unsigned Lu = (unsigned)ep.L;
  const bool step_rows = Lu >= 32u * MB;
  if (QKV && FAST) {
#pragma unroll
    for (int i2 = 0; i2 < NB / 2; ++i2) qkv_col[i2] = qkv_column_base<T>(ep, nw0 + i2 * 64 + rcol);
    const unsigned m_first = (unsigned)mw0 + (unsigned)rrow;
    b0 = m_first / Lu;
    l0 = m_first - b0 * Lu;
  }
  const int64_t batch_stride = (int64_t)ep.heads * ep.L * ep.d;

#pragma unroll
  for (int j = 0; j < MB; ++j) {
    const int64_t mbase = mw0 + j * 32;
#pragma unroll
    for (int i2 = 0; i2 < NB / 2; ++i2) {
      const int n = nw0 + i2 * 64 + rcol;
      // residual of the 8 row groups this lane stores, requested up front
      P4 res[8];
      if (RES && FAST) {
#pragma unroll
        for (int rr = 0; rr < 8; ++rr)
          res[rr] = __builtin_nontemporal_load(reinterpret_cast<const P4*>(
              (const T*)ep.residual + ((mbase + rr * 4 + rrow) * (int64_t)N + n)));
      }
#pragma unroll
      for (int ii = 0; ii < 2; ++ii) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int i = i2 * 2 + ii;
          f4 z;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            z[e] = acc[i][j][4 * g + e] + bias_r[i][g][e];
            if (GELU) z[e] = gelu_new(z[e]);
          }
          *reinterpret_cast<f4*>(slab + frow * EP_STRIDE + (ii * 32 + g * 8 + fhalf * 4) * 4) = z;
        }
      }
#pragma unroll(DROP ? 1 : 8)
      for (int rr = 0; rr < 8; ++rr) {
        const int row = rr * 4 + rrow;
        const int64_t m = mbase + row;
        f4 z = *reinterpret_cast<const f4*>(slab + row * EP_STRIDE + rcol * 4);
        if (FAST) {
          if (RES) {
#pragma unroll
            for (int e = 0; e < 4; ++e) z[e] += (float)res[rr][e];
          }
          P4 o;
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = (T)z[e];
          // streaming store: the output is not read again by this kernel and
          // must not push the operand panels out of L2
          T* dst;
          if constexpr (QKV) {
            unsigned b, l;
            if (step_rows) {
              b = b0;
              l = l0 + (unsigned)(j * 32 + rr * 4);
              if (l >= Lu) { l -= Lu; ++b; }
            } else {
              b = (unsigned)m / Lu;
              l = (unsigned)m - b * Lu;
            }
            dst = qkv_col[i2] + ((int64_t)b * batch_stride + (int64_t)l * ep.d);
          } else {
            dst = out_ptr<T, QKV>(ep, m, n, N);
          }
          __builtin_nontemporal_store(o, reinterpret_cast<P4*>(dst));
        } else {
          if (m >= M || n >= N) continue;
          T* op = out_ptr<T, QKV>(ep, m, n, N);
          const T* rp = RES ? (const T*)ep.residual + (m * (int64_t)N + n) : nullptr;
          if constexpr (DROP) {
            // the generator's offset is the flat index m*N + n in 32 bits (kernels.py:245)
            const unsigned flat = (unsigned)((uint64_t)m * (uint64_t)N + (uint64_t)n);
            unsigned off[4] = {flat, flat + 1u, flat + 2u, flat + 3u};
            float zz[4] = {z[0], z[1], z[2], z[3]};
            dropout_apply<4>(ep.drop, off, zz);
#pragma unroll
            for (int e = 0; e < 4; ++e) z[e] = zz[e];
          }
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < N) op[e] = (T)(z[e] + (RES ? (float)rp[e] : 0.f));
        }
      }
    }
  }
}

// fp16 output without residual, whole tile, vector accesses allowed (and head size % 8 == 0 for
// the head-major scatter): bias (+GELU) and the rounding to fp16 happen in the accumulator
// layout, the transposition through the wavefront's slab moves halves (32 rows x 64 columns x
// 2 bytes per pass, 16-byte units XOR-swizzled with row & 7), and a lane gets 8 neighbouring
// columns back: 16-byte stores, 8 lanes per 128-byte line -- half the LDS traffic and half the
// store instructions of the fp32 staging above.  With a residual the sum must stay in fp32 until
// the one rounding, so those epilogues keep the fp32 slabs.
// bias_r[i][g] = bias of the lane's 4 columns nw0 + 32 i + 8 g + 4 (lane / 32) + 0..3.
// (NB / 2) * MB * 4 stores per lane.
// L16: the accumulators are those of v_mfma_f32_16x16x32 -- acc[2 NB][2 MB] of 4 floats, and of
// the 32 x 32 block (i, j) a lane holds the quads (mh, nh) = acc[2 i + nh][2 j + mh]: row
// 16 mh + lane % 16, columns 16 nh + 4 (lane / 16) + 0..3, bias_r[i][nh] (see load_bias16).  Only
// where a quad comes from and where it lands in the slab differs; the slab and what leaves it do not.
template <int MB, int NB, bool QKV, bool GELU, bool L16 = false, typename Acc, typename Bias>
__device__ __forceinline__ void store_wave_tile_h(Acc& acc, const Bias& bias_r,
                                                  const EpiDev& ep, int64_t mw0, int nw0, int N,
                                                  char* slab, int lane) {
  static_assert(NB % 2 == 0, "wave tile must be a multiple of 64 columns");
  // key (row >> 1) & 7: the 32 rows x 2 lanes of one 8-byte write then cover 16 distinct
  // 16-byte slots of the 256-byte bank window twice -- the minimum for 512 bytes
  const int lq = lane >> 4;
  const int frow = L16 ? (lane & 15) : (lane & 31), fhalf = L16 ? (lq & 1) : (lane >> 5);
  const int fkey = (frow >> 1) & 7;  // rows 16 apart share a key
  const int rrow = lane >> 3, runit = lane & 7;
  const int rkey = rrow >> 1;  // key of row 8 rr + rrow = rkey ^ 4 (rr & 1)
  _Float16* qkv_col[NB / 2];
  unsigned b0 = 0, l0 = 0;
  const unsigned Lu = (unsigned)ep.L;
  const bool step_rows = Lu >= 32u * MB;
  if (QKV) {
#pragma unroll
    for (int i2 = 0; i2 < NB / 2; ++i2)
      qkv_col[i2] = qkv_column_base<_Float16>(ep, nw0 + i2 * 64 + runit * 8);
    const unsigned m_first = (unsigned)mw0 + (unsigned)rrow;
    b0 = m_first / Lu;
    l0 = m_first - b0 * Lu;
  }
  const int64_t batch_stride = (int64_t)ep.heads * ep.L * ep.d;
  const unsigned lane_byte_off = ((unsigned)rrow * (unsigned)N + runit * 8) * 2u;
#pragma unroll
  for (int j = 0; j < MB; ++j) {
#pragma unroll
    for (int i2 = 0; i2 < NB / 2; ++i2) {
#pragma unroll
      for (int ii = 0; ii < 2; ++ii)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int i = i2 * 2 + ii;
          const int mh = g >> 1, nh = g & 1;  // L16: quad g = (mh, nh)
          h4 o;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float z;
            if constexpr (L16) z = acc[2 * i + nh][2 * j + mh][e] + bias_r[i][nh][e];
            else z = acc[i][j][4 * g + e] + bias_r[i][g][e];
            if (GELU) z = gelu_new(z);
            o[e] = (_Float16)z;
          }
          const int row = L16 ? 16 * mh + frow : frow;
          const int grp = L16 ? 2 * nh + (lq >> 1) : g;  // 8-column group of the quad
          *reinterpret_cast<h4*>(slab + row * 128 + (((ii * 4 + grp) ^ fkey) << 4) + fhalf * 8) = o;
        }
      // all four reads first: the stores are assembly with a memory clobber, which no LDS
      // read may cross, so reading inside the store loop would expose one LDS latency per store
      h8 vv[4];
#pragma unroll
      for (int rr = 0; rr < 4; ++rr)
        vv[rr] = *reinterpret_cast<const h8*>(slab + (rr * 8 + rrow) * 128 +
                                              ((runit ^ rkey ^ ((rr & 1) * 4)) << 4));
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        const h8 v = vv[rr];
        if constexpr (QKV) {
          unsigned b, l;
          if (step_rows) {
            b = b0;
            l = l0 + (unsigned)(j * 32 + rr * 8);
            if (l >= Lu) { l -= Lu; ++b; }
          } else {
            const unsigned m = (unsigned)mw0 + (unsigned)(j * 32 + rr * 8 + rrow);
            b = m / Lu;
            l = m - b * Lu;
          }
          _Float16* dst = qkv_col[i2] + ((int64_t)b * batch_stride + (int64_t)l * ep.d);
          __builtin_nontemporal_store(v, reinterpret_cast<h8*>(dst));
        } else {
          // wavefront-uniform 64-bit part in scalar registers + one 32-bit lane offset.  mw0 and
          // nw0 derive from a wavefront index the kernel made provably uniform, so this is
          // scalar arithmetic: a base produced by v_readfirstlane right in front of the store
          // would need five wait states the compiler does not insert for assembly, and the
          // store would now and then go out with the previous base.
          store_nt_base(reinterpret_cast<char*>(ep.out) +
                            ((mw0 + j * 32 + rr * 8) * (int64_t)N + nw0 + i2 * 64) * 2,
                        lane_byte_off, v);
        }
      }
    }
  }
}

// fp16 output WITH residual, whole tile, 16-byte accesses allowed: the wavefront's 128 x 64
// residual sub-tile was brought into LDS by direct loads (rows 0..63 at res_lo while the last
// k-tile was multiplied, rows 64..127 at res_hi right after the loop; 128 bytes per row, 16-byte
// units XOR-swizzled with (row >> 1) & 7), so the epilogue reads it in the accumulator layout, adds it
// in fp32 behind bias (+GELU) -- the reference's order -- rounds once, and finishes like
// store_wave_tile_h.  No global load is waited for between the stores: the two waits below count
// exactly what is younger than the residual loads (the second half's 8 loads; then the 8
// stores of row bands 0 and 1).
template <int MB, int NB, bool GELU>
__device__ __forceinline__ void store_wave_tile_rl(f16v (&acc)[NB][MB], const f4 (&bias_r)[NB][4],
                                                   const EpiDev& ep, int64_t mw0, int nw0, int N,
                                                   const char* res_lo, const char* res_hi,
                                                   char* slab, int lane) {
  static_assert(MB == 4 && NB == 2, "128 x 64 sub-tile");
  const int frow = lane & 31, fhalf = lane >> 5, fkey = (frow >> 1) & 7;
  const int rrow = lane >> 3, runit = lane & 7, rkey = rrow >> 1;
  const unsigned lane_byte_off = ((unsigned)rrow * (unsigned)N + runit * 8) * 2u;
#pragma unroll
  for (int j = 0; j < MB; ++j) {
    if (j == 0 || j == 2) wait_vmcnt<8>();
    const char* rb = (j < 2 ? res_lo : res_hi) + ((j & 1) * 32 + frow) * 128 + fhalf * 8;
    h4 r[NB][4];
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int g = 0; g < 4; ++g)
        r[i][g] = *reinterpret_cast<const h4*>(rb + (((i * 4 + g) ^ fkey) << 4));
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        h4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float z = acc[i][j][4 * g + e] + bias_r[i][g][e];
          if (GELU) z = gelu_new(z);
          o[e] = (_Float16)(z + (float)r[i][g][e]);
        }
        *reinterpret_cast<h4*>(slab + frow * 128 + (((i * 4 + g) ^ fkey) << 4) + fhalf * 8) = o;
      }
    h8 vv[4];
#pragma unroll
    for (int rr = 0; rr < 4; ++rr)
      vv[rr] = *reinterpret_cast<const h8*>(slab + (rr * 8 + rrow) * 128 +
                                            ((runit ^ rkey ^ ((rr & 1) * 4)) << 4));
#pragma unroll
    for (int rr = 0; rr < 4; ++rr)
      store_nt_base(reinterpret_cast<char*>(ep.out) +
                        ((mw0 + j * 32 + rr * 8) * (int64_t)N + nw0) * 2,
                    lane_byte_off, vv[rr]);
  }
}

// store_wave_tile_rl for the streaming residual kernel.  The residual halves lie in the two
// operand stages; `mid` runs between row bands 1 and 2, when the stage that held the first half
// is free again (the kernel refills it there).  Younger than the first half's loads when band 0
// starts: the second half's 8 loads.  Younger than the second half's loads when band 2 starts: the
// 8 stores of bands 0 and 1 and, if `refilled`, the 8 operand loads `mid` issued.
template <int MB, int NB, bool GELU, typename Mid>
__device__ __forceinline__ void store_wave_tile_rs(f4 (&acc)[2 * NB][2 * MB], const f4 (&bias_r)[NB][2],
                                                   const EpiDev& ep, int64_t mw0, int nw0, int N,
                                                   const char* res_lo, const char* res_hi,
                                                   char* slab, int lane, bool refilled, Mid&& mid) {
  static_assert(MB == 4 && NB == 2, "128 x 64 sub-tile");
  // accumulators of v_mfma_f32_16x16x32: quad (mh, nh) of the 32 x 32 block (i, j), see
  // store_wave_tile_h<L16>
  const int frow = lane & 15, lq = lane >> 4, fhalf = lq & 1, fkey = (frow >> 1) & 7;
  const int rrow = lane >> 3, runit = lane & 7, rkey = rrow >> 1;
  const unsigned lane_byte_off = ((unsigned)rrow * (unsigned)N + runit * 8) * 2u;
#pragma unroll
  for (int j = 0; j < MB; ++j) {
    if (j == 0) wait_vmcnt<8>();
    if (j == 2) {
      mid();
      if (refilled) wait_vmcnt<16>();
      else wait_vmcnt<8>();
    }
    const char* rb = (j < 2 ? res_lo : res_hi) + ((j & 1) * 32 + frow) * 128 + fhalf * 8;
    h4 r[NB][4];
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int mh = g >> 1, nh = g & 1;
        r[i][g] = *reinterpret_cast<const h4*>(rb + mh * 16 * 128 +
                                               (((i * 4 + 2 * nh + (lq >> 1)) ^ fkey) << 4));
      }
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int mh = g >> 1, nh = g & 1;
        h4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float z = acc[2 * i + nh][2 * j + mh][e] + bias_r[i][nh][e];
          if (GELU) z = gelu_new(z);
          o[e] = (_Float16)(z + (float)r[i][g][e]);
        }
        *reinterpret_cast<h4*>(slab + (16 * mh + frow) * 128 +
                               (((i * 4 + 2 * nh + (lq >> 1)) ^ fkey) << 4) + fhalf * 8) = o;
      }
    h8 vv[4];
#pragma unroll
    for (int rr = 0; rr < 4; ++rr)
      vv[rr] = *reinterpret_cast<const h8*>(slab + (rr * 8 + rrow) * 128 +
                                            ((runit ^ rkey ^ ((rr & 1) * 4)) << 4));
#pragma unroll
    for (int rr = 0; rr < 4; ++rr)
      store_nt_base(reinterpret_cast<char*>(ep.out) +
                        ((mw0 + j * 32 + rr * 8) * (int64_t)N + nw0) * 2,
                    lane_byte_off, vv[rr]);
  }
}

template <int MB, int NB, typename T, bool QKV>
__device__ __forceinline__ void store_wave_tile(f16v (&acc)[NB][MB], const EpiDev& ep,
                                                int64_t mw0, int nw0, int M, int N, bool fast,
                                                char* slab, int lane) {
  const bool res = !QKV && ep.residual != nullptr;
  if constexpr (!QKV) {
    if (ep.drop.p > 0.f) {  // training-mode path: always the predicated variant
#define GPTMI_EPI_DROP(G, R) \
  store_wave_tile_v<MB, NB, T, QKV, false, G, R, true>(acc, ep, mw0, nw0, M, N, slab, lane)
      if (ep.gelu) { if (res) GPTMI_EPI_DROP(true, true); else GPTMI_EPI_DROP(true, false); }
      else { if (res) GPTMI_EPI_DROP(false, true); else GPTMI_EPI_DROP(false, false); }
#undef GPTMI_EPI_DROP
      return;
    }
  }
  if constexpr (sizeof(T) == 2) {
    if (fast && !res && ep.vec8_ok) {
      const int fhalf = lane >> 5;
      h4 raw[NB][4];
      f4 bias_r[NB][4];
      load_bias<_Float16, NB>(ep, nw0, fhalf, raw);
      bias_to_f32(raw, bias_r);
      if (ep.gelu) store_wave_tile_h<MB, NB, QKV, true>(acc, bias_r, ep, mw0, nw0, N, slab, lane);
      else store_wave_tile_h<MB, NB, QKV, false>(acc, bias_r, ep, mw0, nw0, N, slab, lane);
      return;
    }
  }
#define GPTMI_EPI(F, G, R) \
  store_wave_tile_v<MB, NB, T, QKV, F, G, R>(acc, ep, mw0, nw0, M, N, slab, lane)
  if (fast) {
    if (ep.gelu) { if (res) GPTMI_EPI(true, true, true); else GPTMI_EPI(true, true, false); }
    else { if (res) GPTMI_EPI(true, false, true); else GPTMI_EPI(true, false, false); }
  } else {
    if (ep.gelu) { if (res) GPTMI_EPI(false, true, true); else GPTMI_EPI(false, true, false); }
    else { if (res) GPTMI_EPI(false, false, true); else GPTMI_EPI(false, false, false); }
  }
#undef GPTMI_EPI
}

// XCD-aware tile id: workgroup ids are dealt round-robin over the 8 XCDs, so id
// p runs on XCD p % 8.  The remap hands every XCD a contiguous range of tiles.
__device__ __forceinline__ int xcd_tile(int pid, int num_tiles) {
  const int per = (num_tiles + 7) >> 3;
  int tall = num_tiles & 7;
  if (tall == 0) tall = 8;
  const int xcd = pid & 7, loc = pid >> 3;
  return xcd < tall ? xcd * per + loc : tall * per + (xcd - tall) * (per - 1) + loc;
}

// WPE = wavefronts per SIMD the register allocation must leave room for (two
// 4-wavefront workgroups per CU need 2).
// LNA: the A operand is LayerNorm(x).  The workgroup normalises its BM rows of x [M][Kp] once
// (fp32 statistics, the arithmetic and summation order of layernorm_vec_kernel, rounded to fp16)
// into an LDS panel that holds all k-tiles of those rows, and only the weights travel through
// the stages.  For few rows (the launcher's choice): the normalised matrix never goes to memory
// and its kernel launch is gone; every column tile of a row block normalises the rows again.
template <int BM, int BN, int WM, int WN, int BKS, int NST, int WPE, typename T, bool QKV,
          bool RESLDS = false, bool LNA = false>
__global__ __launch_bounds__(WM * WN * 64, WPE) void gemm_kernel(
    const _Float16* __restrict__ A, const _Float16* __restrict__ Bt, int M, int N, int Kp,
    int tiles_m, int tiles_n, int group_w, EpiDev ep, LnArgs ln) {
  static_assert(BKS == 32 || BKS == 64, "k-step of 32 or 64");
  static_assert(NST >= 2, "at least double buffering");
  static_assert(!LNA || (BKS == 64 && !RESLDS && sizeof(T) == 2), "LayerNorm prologue: fp16, k-step 64");
  constexpr int T_ = WM * WN * 64;
  constexpr int TM = BM / WM, TN = BN / WN;
  constexpr int MB = TM / 32, NB = TN / 32;
  constexpr int ROWB = BKS * 2;            // bytes per LDS row
  constexpr int CPR = ROWB / 16;           // 16-byte chunks per row (4 or 8)
  constexpr int CSH = CPR == 8 ? 3 : 2;    // log2(CPR)
  constexpr int KSH = CPR == 8 ? 1 : 2;    // swizzle key = (row >> KSH) & (CPR-1)
  // LNA: no A loads, the stages hold weight rows only, the panel lies behind the stages
  constexpr int A_IT = LNA ? 0 : BM * CPR / T_, B_IT = BN * CPR / T_;
  constexpr int A_N = A_IT ? A_IT : 1;     // array extent
  constexpr int LPT = A_IT + B_IT;         // direct loads per thread per k-tile
  constexpr int B_AT = LNA ? 0 : BM * ROWB;  // byte offset of the weight rows inside a stage
  constexpr int STAGE = B_AT + BN * ROWB;
  constexpr int KS = BKS / 16;             // MFMA k-steps per tile
  static_assert(BM * CPR % T_ == 0 && BN * CPR % T_ == 0, "tile/threads mismatch");
  static_assert(TM % 32 == 0 && TN % 64 == 0, "wave tile must be 32 x 64 aligned");
  static_assert(NST * STAGE >= WM * WN * EP_SLAB, "epilogue staging does not fit");
  static_assert((NST - 2) * LPT <= 63, "vmcnt range");
  // RESLDS (launched with a residual; 32 KB of LDS behind the stages for the epilogue slabs):
  // workgroups whose tile is whole bring the residual tile into the operand stages as these fall
  // free and run store_wave_tile_rl; tiles on the matrix edge take the predicated epilogue.
  static_assert(!RESLDS || (sizeof(T) == 2 && !QKV && NST == 2 && BM == 256 && BN == 256 &&
                            WM == 2 && WN == 4 && BKS == 64),
                "residual through LDS: the 256 x 256 x 64 configuration, fp16 row-major output");

  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  // provably wavefront-uniform, so that everything derived from the wavefront's sub-tile origin
  // (the base addresses of the epilogue's stores) is scalar arithmetic in scalar registers
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % WM, wn = wave / WM;
  // Tile order: the column tiles are cut into groups of group_w; inside a group the column
  // runs fastest, then the row block, and the groups follow each other.  Workgroups that run
  // at the same time then share few weight panels, which stay in the XCD's L2.
  const int tile = xcd_tile(blockIdx.x, tiles_m * tiles_n);
  const int grp = tile / (tiles_m * group_w);
  const int in_grp = tile - grp * tiles_m * group_w;
  const int grp_w = min(group_w, tiles_n - grp * group_w);
  const int tm = in_grp / grp_w, tn = grp * group_w + in_grp % grp_w;
  const int m0 = tm * BM, n0 = tn * BN;

  // ---- per-thread sources of the direct global->LDS loads -----------------
  // 16-byte slot s of an operand tile: row s / CPR, position s % CPR, which
  // holds source chunk (s % CPR) ^ key(row).  Rows past the matrix edge re-read
  // the last row (their products are never stored).
  const char* a_src[A_N];
  const char* b_src[B_IT];
#pragma unroll
  for (int it = 0; it < A_IT; ++it) {
    const int s = it * T_ + tid, r = s >> CSH, c = (s & (CPR - 1)) ^ ((r >> KSH) & (CPR - 1));
    int row = m0 + r;
    row = row < M ? row : M - 1;
    a_src[it] = (const char*)(A + (size_t)row * Kp) + c * 16;
  }
#pragma unroll
  for (int it = 0; it < B_IT; ++it) {
    const int s = it * T_ + tid, r = s >> CSH, c = (s & (CPR - 1)) ^ ((r >> KSH) & (CPR - 1));
    int row = n0 + r;
    row = row < N ? row : N - 1;
    b_src[it] = (const char*)(Bt + (size_t)row * Kp) + c * 16;
  }
  const unsigned wave_off =
      __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)smem + (unsigned)wave * 1024u);
  auto issue = [&](int kt) {
    const unsigned as = wave_off + (kt % NST) * STAGE;
    const unsigned bs = as + B_AT;
#pragma unroll
    for (int it = 0; it < A_IT; ++it)
      lds_dma16(a_src[it] + (size_t)kt * ROWB, as + it * T_ * 16);
#pragma unroll
    for (int it = 0; it < B_IT; ++it)
      lds_dma16(b_src[it] + (size_t)kt * ROWB, bs + it * T_ * 16);
  };

  // one of the A_IT + B_IT loads of k-tile kt (the A loads come first)
  auto issue_one = [&](int kt, int n) {
    const unsigned as = wave_off + (kt % NST) * STAGE;
    if (n < A_IT) lds_dma16(a_src[n < A_IT ? n : 0] + (size_t)kt * ROWB, as + n * T_ * 16);
    else lds_dma16(b_src[n - A_IT] + (size_t)kt * ROWB, as + B_AT + (n - A_IT) * T_ * 16);
  };

  f16v acc[NB][MB];
#pragma unroll
  for (int i = 0; i < NB; ++i)
#pragma unroll
    for (int j = 0; j < MB; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // fragment read offsets (bytes) inside a stage
  const int frow = lane & 31, fhalf = lane >> 5, fkey = (frow >> KSH) & (CPR - 1);
  const int a_row_off = (wm * TM + frow) * ROWB;
  const int b_row_off = B_AT + (wn * TN + frow) * ROWB;
  // LNA: k-tile kt of the normalised rows, laid out like the A part of a stage
  const char* panel = smem + NST * STAGE;
  h8 af[2][MB], bf[2][NB];
  auto read_frags = [&](int kt, int ks, int slot) {
    const char* st = smem + (kt % NST) * STAGE;
    const char* sa = LNA ? panel + kt * (BM * ROWB) : st;
    const int choff = ((ks * 2 + fhalf) ^ fkey) << 4;
#pragma unroll
    for (int j = 0; j < MB; ++j)
      af[slot][j] = *reinterpret_cast<const h8*>(sa + a_row_off + j * 32 * ROWB + choff);
#pragma unroll
    for (int i = 0; i < NB; ++i)
      bf[slot][i] = *reinterpret_cast<const h8*>(st + b_row_off + i * 32 * ROWB + choff);
  };
  auto mma = [&](int slot) {
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int j = 0; j < MB; ++j)
        acc[i][j] =
            __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[slot][i], af[slot][j], acc[i][j], 0, 0, 0);
  };

  // The MFMAs of one k-slice with the loads of k-tile kt_load dealt between them: a load
  // instruction (address add, M0, issue) then costs no MFMA time -- issued as one block right
  // behind the barrier, the loads of all wavefronts kept the matrix pipe idle for ~500 cycles
  // per k-tile.
  auto mma_and_issue = [&](int slot, int kt_load, bool go) {
    constexpr int PER = (A_IT + B_IT + MB * NB - 1) / (MB * NB);
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int j = 0; j < MB; ++j) {
        acc[i][j] =
            __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[slot][i], af[slot][j], acc[i][j], 0, 0, 0);
#pragma unroll
        for (int l = 0; l < PER; ++l) {
          const int n = (i * MB + j) * PER + l;  // a constant after unrolling
          if (n < A_IT + B_IT && go) issue_one(kt_load, n);
        }
      }
  };

  const int KT = Kp / BKS;
  // Residual through LDS.  Half h = rows 64 h .. 64 h + 63 of the wavefront's sub-tile goes
  // to this wavefront's own 8 KB of operand stage `stg`: 8 direct loads of 8 rows, lane l of
  // load q fetching 16-byte unit (l % 8) ^ key of row r = 8 q + l / 8, key = (r >> 1) & 7 =
  // (l / 16) ^ 4 (q & 1), so that unit u of row r lies at position u ^ key of the row's 128 bytes.
  const bool res_lds =
      RESLDS && ep.residual != nullptr && ep.vec_ok && n0 + BN <= N && m0 + BM <= M;
  unsigned res_lane_off[2];
#pragma unroll
  for (int odd = 0; odd < 2; ++odd)
    res_lane_off[odd] = ((unsigned)(lane >> 3) * (unsigned)N +
                         (unsigned)(((lane & 7) ^ (lane >> 4) ^ (odd * 4)) * 8)) * 2u;
  auto issue_res_half = [&](int h, int stg) {
    const char* base = (const char*)ep.residual +
                       (((int64_t)m0 + wm * TM + h * 64) * N + (n0 + wn * TN)) * 2;
    const unsigned lds = (unsigned)(uintptr_t)smem + (unsigned)stg * STAGE + (unsigned)wave * 8192u;
#pragma unroll
    for (int q = 0; q < 8; ++q)
      lds_dma16_base(base + (int64_t)q * 8 * N * 2, res_lane_off[q & 1], lds + q * 1024);
  };

  // Pipeline.  NST k-tiles are in LDS or on their way at any time.  Fragments of the next
  // k-slice are requested before the MFMAs of the current one issue (the scheduling fences keep
  // the compiler from sinking the reads behind the MFMAs again).  In front of the LAST k-slice of
  // tile kt -- whose fragments are in registers by then -- tile kt+1 is published (own loads
  // landed, own LDS reads retired, barrier), its first fragments are requested, and the stage of
  // tile kt, which nobody reads any more, is refilled with tile kt+NST while that last slice is
  // multiplied.  No MFMA ever waits for a barrier plus an LDS round trip.
#pragma unroll
  for (int s = 0; s < NST; ++s)
    if (s < KT) issue(s);
  if constexpr (LNA) {
    // The rows of this tile, normalised, into the panel: chunk c of row r goes to k-tile c / 8,
    // position (c % 8) ^ key(r) of the row's 128 bytes.  A row is spread over LPR lanes as in
    // layernorm_vec_kernel (T_ / LPR rows per pass); rows past the end repeat the last row.
    const int H = Kp, nchunks = H >> 3;
    auto ln_rows = [&](auto lpr_tag, auto ch_tag) {
      constexpr int LPR = decltype(lpr_tag)::value, CH = decltype(ch_tag)::value;
      constexpr int RPP = T_ / LPR;
      const int ll = tid & (LPR - 1), rsub = tid / LPR;
      const h8* wv = reinterpret_cast<const h8*>(ln.w);
      const h8* bv = reinterpret_cast<const h8*>(ln.b);
      // the parameters of the lane's chunks: held across the rows, unless the rows are so long
      // that they and a row do not fit the registers together (then fetched per row, from L1)
      constexpr bool HOLD = CH <= 4;
      h8 tw[CH], tb[CH];
      if constexpr (HOLD) {
#pragma unroll
        for (int i = 0; i < CH; ++i) {
          const int c = ll + i * LPR;
          if (c < nchunks) {
            tw[i] = wv[c];
            tb[i] = bv[c];
          }
        }
      }
      // G rows per thread group are requested together, so that a workgroup waits for memory
      // BM / (RPP * G) times and not once per row (G * CH 16-byte registers hold them)
      constexpr int PASSES = BM / RPP;
      constexpr int G0 = CH <= 3 ? 8 : CH <= 4 ? 4 : 2, G = G0 < PASSES ? G0 : PASSES;
      static_assert(PASSES % G == 0, "row groups");
      for (int p0 = 0; p0 < PASSES; p0 += G) {
        h8 t[G][CH];
#pragma unroll
        for (int g = 0; g < G; ++g) {
          int row = m0 + (p0 + g) * RPP + rsub;
          row = row < M ? row : M - 1;
          const h8* xr = reinterpret_cast<const h8*>(A + (size_t)row * Kp);
#pragma unroll
          for (int i = 0; i < CH; ++i) {
            const int c = ll + i * LPR;
            if (c < nchunks) t[g][i] = xr[c];
          }
        }
#pragma unroll
        for (int g = 0; g < G; ++g) {
          const int r = (p0 + g) * RPP + rsub;
          float v[CH][8];
          float sum = 0.f;
#pragma unroll
          for (int i = 0; i < CH; ++i) {
            const int c = ll + i * LPR;
            if (c < nchunks) {
#pragma unroll
              for (int j = 0; j < 8; ++j) {
                v[i][j] = (float)t[g][i][j];
                sum += v[i][j];
              }
            } else {
#pragma unroll
              for (int j = 0; j < 8; ++j) v[i][j] = 0.f;
            }
          }
          float mean, rstd;
          layernorm_stats<CH, 8, LPR>(v, sum, ll, nchunks, H, ln.eps, mean, rstd);
#pragma unroll
          for (int i = 0; i < CH; ++i) {
            const int c = ll + i * LPR;
            if (c < nchunks) {
              if constexpr (!HOLD) {
                tw[i] = wv[c];
                tb[i] = bv[c];
              }
              h8 to;
#pragma unroll
              for (int j = 0; j < 8; ++j)
                to[j] = (_Float16)layernorm_apply(v[i][j], mean, rstd, (float)tw[i][j],
                                                  (float)tb[i][j]);
              *reinterpret_cast<h8*>(const_cast<char*>(panel) + (c >> 3) * (BM * ROWB) + r * ROWB +
                                     (((c & 7) ^ ((r >> KSH) & 7)) << 4)) = to;
            }
          }
        }
      }
    };
    const int need = (nchunks + ln.lpr - 1) / ln.lpr;  // chunks per lane; the launcher checked <= 8
#define GPTMI_LN_ROWS(L)                                                            \
  do {                                                                              \
    using LT = std::integral_constant<int, L>;                                      \
    if (need <= 1) ln_rows(LT{}, std::integral_constant<int, 1>{});                 \
    else if (need <= 2) ln_rows(LT{}, std::integral_constant<int, 2>{});            \
    else if (need <= 3) ln_rows(LT{}, std::integral_constant<int, 3>{});            \
    else if (need <= 4) ln_rows(LT{}, std::integral_constant<int, 4>{});            \
    else ln_rows(LT{}, std::integral_constant<int, 8>{});                           \
  } while (0)
    if (ln.lpr == 32) GPTMI_LN_ROWS(32);
    else GPTMI_LN_ROWS(64);
#undef GPTMI_LN_ROWS
    // the first weight k-tiles have landed (their loads are older than the rows' loads, which
    // the arithmetic above waited for; said explicitly all the same), the panel is written
    wait_vmcnt<0>();
    __syncthreads();
  } else {
    // tile 0 must have landed; up to NST-1 younger tiles stay in flight
    if (KT >= NST) wait_vmcnt<(NST - 1) * LPT>();
    else wait_vmcnt<0>();
    asm volatile("s_barrier" ::: "memory");
  }
  read_frags(0, 0, 0);

  for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int cur = ks & 1;
      const bool last = ks + 1 == KS;
      if (!last) {
        read_frags(kt, ks + 1, cur ^ 1);
      } else if (kt + 1 < KT) {
        // tile kt+1 complete; tiles kt+2 .. kt+NST-1 may still be in flight
        if (kt + NST - 1 < KT) wait_vmcnt<(NST - 2) * LPT>();
        else wait_vmcnt<0>();
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        read_frags(kt + 1, 0, cur ^ 1);
      }
      __builtin_amdgcn_sched_barrier(0);
      if (last) mma_and_issue(cur, kt + NST, kt + NST < KT);
      else mma(cur);
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (RESLDS) {
      // the stage of k-tile KT-2 fell free at the barrier in front of its last slice
      if (res_lds && kt == KT - 2) {
        issue_res_half(0, kt % NST);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }

  // ---- epilogue -----------------------------------------------------------
  block_barrier();  // every wavefront is done reading the operand stages
  const bool fast = ep.vec_ok && n0 + BN <= N && m0 + BM <= M;
  bool stored = false;
  if constexpr (RESLDS) {
    if (res_lds) {
      const int nw0 = n0 + wn * TN, fhalf = lane >> 5;
      // the bias first, and waited for, so that no compiler-placed wait inside the epilogue
      // falls behind the second half's loads
      h4 raw[NB][4];
      f4 bias_r[NB][4];
      load_bias<_Float16, NB>(ep, nw0, fhalf, raw);
      bias_to_f32(raw, bias_r);
#pragma unroll
      for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int g = 0; g < 4; ++g) asm volatile("" : "+v"(bias_r[i][g]));
      const int s_lo = (KT - 2) % NST, s_hi = (KT - 1) % NST;
      issue_res_half(1, s_hi);
      const char* res_lo = smem + s_lo * STAGE + wave * 8192;
      const char* res_hi = smem + s_hi * STAGE + wave * 8192;
      char* slab = smem + NST * STAGE + wave * 4096;
      if (ep.gelu)
        store_wave_tile_rl<MB, NB, true>(acc, bias_r, ep, (int64_t)m0 + wm * TM, nw0, N, res_lo,
                                         res_hi, slab, lane);
      else
        store_wave_tile_rl<MB, NB, false>(acc, bias_r, ep, (int64_t)m0 + wm * TM, nw0, N, res_lo,
                                          res_hi, slab, lane);
      stored = true;
    }
  }
  if (!stored) {
    // the scatter finds (batch, position) from the token row: launch-relative row + m_off
    const int moff = QKV ? ep.m_off : 0;
    store_wave_tile<MB, NB, T, QKV>(acc, ep, (int64_t)m0 + wm * TM + moff, n0 + wn * TN, M + moff,
                                    N, fast, smem + wave * EP_SLAB, lane);
  }
}

// Width, in column tiles, of the groups the tile order walks through.  The weight panels of
// one group (group_w * BN rows of Kp halves) should stay in a 4 MB L2 beside the activation
// panels in flight, so they get about 2.4 MB; every group re-reads the activations once, so
// the groups are as few and as even as that allows.  Panels too long for two of them to fit
// (large K) keep the plain column-fastest order.
inline int column_group(int tiles_n, int bn, int Kp) {
  const int64_t panel = (int64_t)bn * Kp * 2;
  const int fit = (int)((2400 << 10) / panel);
  if (fit < 2 || tiles_n <= fit) return tiles_n;
  const int groups = (tiles_n + fit - 1) / fit;
  return (tiles_n + groups - 1) / groups;
}

template <int BM, int BN, int WM, int WN, int BKS, int NST, int WPE, typename T, bool QKV,
          bool RESLDS = false>
int launch_cfg(const void* A, const void* Bt, int64_t M, int N, int Kp, const EpiDev& ep,
               hipStream_t st) {
  auto kern = gemm_kernel<BM, BN, WM, WN, BKS, NST, WPE, T, QKV, RESLDS>;
  constexpr int smem = NST * (BM + BN) * BKS * 2 + (RESLDS ? WM * WN * 4096 : 0);
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
  const int group_w = column_group(tiles_n, BN, Kp);
  hipLaunchKernelGGL(kern, dim3((unsigned)(tiles_m * tiles_n)), dim3(WM * WN * 64), smem, st,
                     (const _Float16*)A, (const _Float16*)Bt, (int)M, N, Kp, tiles_m, tiles_n,
                     group_w, ep, LnArgs{});
  return 0;
}

// The LayerNorm-prologue form: 32 x 128 tiles, 2 wavefronts, three stages of weight rows
// (48 KB) and the panel of the tile's 32 normalised rows (64 * Kp bytes) behind them.
constexpr int LNA_BM = 32, LNA_BN = 128, LNA_NST = 3;
inline size_t lna_lds_bytes(int Kp) { return (size_t)LNA_NST * LNA_BN * 128 + (size_t)LNA_BM * Kp * 2; }

template <bool QKV>
int launch_lna(const void* x, const void* Bt, int64_t M, int N, int Kp, const EpiDev& ep,
               const LnArgs& ln, hipStream_t st) {
  auto kern = gemm_kernel<LNA_BM, LNA_BN, 1, 2, 64, LNA_NST, 2, _Float16, QKV, false, true>;
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
  const int tiles_m = (int)((M + LNA_BM - 1) / LNA_BM), tiles_n = (N + LNA_BN - 1) / LNA_BN;
  const int group_w = column_group(tiles_n, LNA_BN, Kp);
  hipLaunchKernelGGL(kern, dim3((unsigned)(tiles_m * tiles_n)), dim3(128), lna_lds_bytes(Kp), st,
                     (const _Float16*)x, (const _Float16*)Bt, (int)M, N, Kp, tiles_m, tiles_n,
                     group_w, ep, ln);
  return 0;
}

// ---------------------------------------------------------------------------
// Streaming variant of the 256x256x64 kernel: one workgroup per CU walks tiles
// blockIdx.x, blockIdx.x + gridDim.x, ...  The two operand stages keep alternating across tile
// boundaries, so the first two k-tiles of the NEXT output tile are requested while the current
// one finishes, and the epilogue runs with those loads in flight.  What this removes, per tile
// of ~28 us: the pipeline fill (3.5 k cycles) and the ~2.8 us a CU otherwise sits idle between
// two workgroups while the stores of the one that ended drain (measured: 231 of 256 CUs busy
// on average with one workgroup per tile, 251 when the kernel stores nothing).
//
// LDS: stages at [0, 128 KB), epilogue slabs behind them (8 wavefronts x 4 KB: 32 rows x 64
// halves for fp16 output, store_wave_tile_h; one 32 x 32 fp32 block for fp32 output, 16-byte
// units XOR-swizzled with (row >> 1) & 7), so the epilogue never touches a stage.
//
// Load/store counter.  Loads and stores of a wavefront retire in issue order on this ISA.  The
// loads of the next tile's k-tile 1 are issued BEFORE the epilogue's stores, so waiting for them
// with vmcnt(EPI_STORES) -- the epilogue issues exactly 16 (fp16) or 32 (fp32) stores per lane --
// does not wait for the stores' acknowledgements.  The bias is fetched, and waited for, before those loads are issued, so
// that no compiler-placed wait inside the epilogue falls behind them.  Only whole tiles, no
// residual, no dropout: the launcher sends everything else to gemm_kernel.
// ---------------------------------------------------------------------------
template <int MB, int NB, typename T, bool QKV, bool GELU>
__device__ __forceinline__ void store_wave_tile32(f4 (&acc)[2 * NB][2 * MB], const f4 (&bias_r)[NB][2],
                                                  const EpiDev& ep, int64_t mw0, int nw0, int N,
                                                  char* slab, int lane) {
  typedef typename Pack4<T>::type P4;
  // accumulators of v_mfma_f32_16x16x32: quad (mh, nh) of the 32 x 32 block (i, j) = row
  // 16 mh + lane % 16, columns 16 nh + 4 (lane / 16) + 0..3
  const int frow = lane & 15, lq = lane >> 4, fkey = (frow >> 1) & 7;
  const int rrow = lane >> 3, runit = lane & 7;
  T* qkv_col[NB];
  unsigned b0 = 0, l0 = 0;
  const unsigned Lu = (unsigned)ep.L;
  const bool step_rows = Lu >= 32u * MB;
  if (QKV) {
#pragma unroll
    for (int i = 0; i < NB; ++i) qkv_col[i] = qkv_column_base<T>(ep, nw0 + i * 32 + runit * 4);
    const unsigned m_first = (unsigned)mw0 + (unsigned)rrow;
    b0 = m_first / Lu;
    l0 = m_first - b0 * Lu;
  }
  const int64_t batch_stride = (int64_t)ep.heads * ep.L * ep.d;
  // byte offset of this lane's (row, 4 columns) inside a 32 x 32 pass of a row-major [.][N] matrix
  const unsigned lane_byte_off = ((unsigned)rrow * (unsigned)N + runit * 4) * (unsigned)sizeof(T);
#pragma unroll
  for (int j = 0; j < MB; ++j) {
#pragma unroll
    for (int i = 0; i < NB; ++i) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int mh = g >> 1, nh = g & 1;
        f4 z;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          z[e] = acc[2 * i + nh][2 * j + mh][e] + bias_r[i][nh][e];
          if (GELU) z[e] = gelu_new(z[e]);
        }
        *reinterpret_cast<f4*>(slab + (16 * mh + frow) * 128 + (((4 * nh + lq) ^ fkey) << 4)) = z;
      }
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        const int row = rr * 8 + rrow;
        const f4 z =
            *reinterpret_cast<const f4*>(slab + row * 128 + ((runit ^ ((row >> 1) & 7)) << 4));
        P4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = (T)z[e];
        if constexpr (QKV) {
          unsigned b, l;
          if (step_rows) {
            b = b0;
            l = l0 + (unsigned)(j * 32 + rr * 8);
            if (l >= Lu) { l -= Lu; ++b; }
          } else {
            const unsigned m = (unsigned)mw0 + (unsigned)(j * 32 + row);
            b = m / Lu;
            l = m - b * Lu;
          }
          T* dst = qkv_col[i] + ((int64_t)b * batch_stride + (int64_t)l * ep.d);
          __builtin_nontemporal_store(o, reinterpret_cast<P4*>(dst));
        } else {
          // wavefront-uniform 64-bit part in scalar registers + one 32-bit lane offset
          store_nt_base(reinterpret_cast<char*>(ep.out) +
                            ((mw0 + j * 32 + rr * 8) * (int64_t)N + (nw0 + i * 32)) *
                                (int64_t)sizeof(T),
                        lane_byte_off, o);
        }
      }
    }
  }
}

template <int WM, int WN, typename T, bool QKV>
__global__ __launch_bounds__(512, 2) void gemm_stream_kernel(
    const _Float16* __restrict__ A, const _Float16* __restrict__ Bt, int M, int N, int Kp,
    int tiles_m, int tiles_n, int group_w, EpiDev ep) {
  constexpr int BM = 256, BN = 256, ROWB = 128, T_ = 512, KS = 4;
  static_assert(WM * WN == 8, "8 wavefronts");
  constexpr int TM = BM / WM, TN = BN / WN;
  constexpr int MB = TM / 32, NB = TN / 32;
  constexpr int A_IT = 4, B_IT = 4, LPT = A_IT + B_IT;  // 16-byte loads per thread per k-tile
  constexpr int STAGE = (BM + BN) * ROWB;               // 64 KB
  constexpr int SLABS = 2 * STAGE;                      // epilogue slabs start behind the stages
  constexpr bool HALF_SLABS = sizeof(T) == 2;           // fp16 output: store_wave_tile_h
  constexpr int EPI_STORES = HALF_SLABS ? MB * NB * 2 : MB * NB * 4;  // stores per lane per epilogue

  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  // provably wavefront-uniform, so that everything derived from the wavefront's sub-tile origin
  // (output and residual bases) lives in scalar registers
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % WM, wn = wave / WM;
  const int num_tiles = tiles_m * tiles_n;
  const int KT = Kp / 64;  // >= 2 (checked by the launcher)

  // Operand-tile slot s = it * 512 + tid: row it * 64 + tid / 8, 16-byte position tid % 8,
  // which holds source chunk (tid % 8) ^ ((row >> 1) & 7) -- the key does not depend on `it`.
  // M and N are multiples of 256 here (the launcher sends other shapes to gemm_kernel), so no
  // row is clamped: a load address is a per-tile scalar base (first row of the tile, k-tile
  // offset) plus one of four per-thread 32-bit offsets shared by A and B.
  const int r0 = tid >> 3;
  unsigned lane_off[A_IT];
#pragma unroll
  for (int it = 0; it < A_IT; ++it)
    lane_off[it] = (unsigned)(r0 + it * 64) * (unsigned)Kp * 2u +
                   (unsigned)(((tid & 7) ^ ((r0 >> 1) & 7)) * 16);
  const unsigned wave_off =
      __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)smem + (unsigned)wave * 1024u);
  auto tile_origin = [&](int vp, int& m0, int& n0) __attribute__((always_inline)) {
    const int tile = xcd_tile(vp, num_tiles);
    const int grp = tile / (tiles_m * group_w);
    const int in_grp = tile - grp * tiles_m * group_w;
    const int grp_w = min(group_w, tiles_n - grp * group_w);
    m0 = (in_grp / grp_w) * BM;
    n0 = (grp * group_w + in_grp % grp_w) * BN;
  };
  // A k-tile is eight 16-byte loads per lane: four for the A rows, four for the B rows.  The
  // source of a half is a scalar (first row of the tile, first byte of the k-tile), computed once
  // and not per load: the scalar work of a load that goes between two MFMAs must fit under one.
  auto a_src = [&](int m0, int k) __attribute__((always_inline)) {
    return (const char*)A + ((size_t)m0 * Kp * 2 + (size_t)k * ROWB);
  };
  // Source of load n (64-row block n) of the B tile at n0.  N is a multiple of 64, not
  // necessarily of 256: in the last column tile a block that starts at or past row N loads
  // block 0 again (the shift goes into the scalar source, the lane offsets stay); its products
  // are never stored.
  const size_t blk_bytes = (size_t)64 * Kp * 2;
  auto b_src = [&](int n0, int k, int n) __attribute__((always_inline)) {
    const int vb = (N - n0) >> 6;  // valid blocks of this tile (4 or more: all)
    const char* p = (const char*)Bt + ((size_t)n0 * Kp * 2 + (size_t)k * ROWB);
    return n < vb ? p : p - n * blk_bytes;
  };
  auto issue_a = [&](int stage, const char* src, int n) __attribute__((always_inline)) {
    lds_dma16_base(src, lane_off[n], wave_off + stage * STAGE + n * T_ * 16);
  };
  auto issue_b = [&](int stage, const char* src, int n) __attribute__((always_inline)) {
    lds_dma16_base(src, lane_off[n], wave_off + stage * STAGE + BM * ROWB + n * T_ * 16);
  };
  auto issue = [&](int stage, int m0, int n0, int k) __attribute__((always_inline)) {
    const char* a = a_src(m0, k);
#pragma unroll
    for (int n = 0; n < A_IT; ++n) issue_a(stage, a, n);
#pragma unroll
    for (int n = 0; n < B_IT; ++n) issue_b(stage, b_src(n0, k, n), n);
  };

  // Fragments of v_mfma_f32_16x16x32_f16: a lane supplies row lane % 16 of a block of 16 rows and
  // the 8 halves of 16-byte unit lane / 16 of a 32-wide k-step.  (Which k goes to which lane group
  // is free as long as both operands agree: k is summed over.)  16 consecutive lanes read 16
  // consecutive rows at one unit, as with the 32-row fragments of the small-tile kernel: no bank
  // conflicts.
  const int lrow = lane & 15, lq = lane >> 4, fkey = (lrow >> 1) & 7;
  const int a_row_off = (wm * TM + lrow) * ROWB;
  const int b_row_off = BM * ROWB + (wn * TN + lrow) * ROWB;
  // A slice = one 32-wide k-step s times one half h of the sub-tile's rows: 4 A blocks (af; a
  // block's register takes the next slice's block as soon as its four MFMAs are issued) times 4 B
  // blocks (bf[s], good for both halves of step s).
  static_assert(TM == 128 && TN == 64, "128 x 64 sub-tiles");
  h8 af[4], bf[2][4];
  auto frag_a = [&](const char* st, int h, int jl, int s) __attribute__((always_inline)) {
    return *reinterpret_cast<const h8*>(st + a_row_off + (h * 64 + jl * 16) * ROWB +
                                        (((s * 4 + lq) ^ fkey) << 4));
  };
  auto frag_b = [&](const char* st, int i, int s) __attribute__((always_inline)) {
    return *reinterpret_cast<const h8*>(st + b_row_off + i * 16 * ROWB +
                                        (((s * 4 + lq) ^ fkey) << 4));
  };
  // the fragments of a k-tile's first slice
  auto read_first = [&](int stage) __attribute__((always_inline)) {
    const char* st = smem + stage * STAGE;
#pragma unroll
    for (int jl = 0; jl < 4; ++jl) af[jl] = frag_a(st, 0, jl, 0);
#pragma unroll
    for (int i = 0; i < 4; ++i) bf[0][i] = frag_b(st, i, 0);
  };

  int vp = blockIdx.x;
  int m0, n0;
  tile_origin(vp, m0, n0);
  issue(0, m0, n0, 0);
  issue(1, m0, n0, 1);
  wait_vmcnt<LPT>();
  asm volatile("s_barrier" ::: "memory");
  read_first(0);
  int stage = 0;           // stage of the k-tile being multiplied
  bool prev_stored = false;  // this wavefront stored a tile right before the current one

  while (true) {
    const int vp_next = vp + (int)gridDim.x;
    const bool has_next = vp_next < num_tiles;
    int m0_n = 0, n0_n = 0;
    if (has_next) tile_origin(vp_next, m0_n, n0_n);
    const int64_t mw0 = (int64_t)m0 + wm * TM;
    const int nw0 = n0 + wn * TN;
    const bool wave_stores = nw0 < N;  // else this wavefront's 64 columns lie past the edge

    // acc[i][j] = the 16 x 16 block of columns 16 i.., rows 16 j.. of the sub-tile: a lane holds
    // row lane % 16 and the 4 columns 4 (lane / 16) + 0..3
    f4 acc[2 * NB][2 * MB];
#pragma unroll
    for (int i = 0; i < 2 * NB; ++i)
#pragma unroll
      for (int j = 0; j < 2 * MB; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;

    // One slice, a quarter of a k-tile: 16 MFMAs of 16 x 16 x 32 in eight pairs (a pair takes the
    // matrix pipe as long as one 32 x 32 x 16, and this shape draws less power for the same
    // products: on random operands the chip holds a higher clock).  Behind the pairs, one each, go
    // the fragment reads for slice `rks` of `rstage`: a read issued in the shadow of an MFMA costs
    // no issue time, a burst of them in front of the MFMAs idles the pipe whenever both wavefronts
    // of a SIMD read at once (behind every barrier).  `extra(q)` runs behind pair q.
    auto slice = [&](int, bool fetch, int rstage, int rks, auto&& extra) __attribute__((always_inline)) {
      // this slice is t = rks - 1 (mod 4): k-step s = t / 2, row half h = t % 2
      const int t = (rks + 3) & 3, s = t >> 1, h = t & 1;
      const char* st = smem + rstage * STAGE;
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const int jl = q >> 1;
#pragma unroll
        for (int p = 0; p < 2; ++p) {
          const int ii = (q & 1) * 2 + p;
          const int i = (jl & 1) ? 3 - ii : ii;  // one operand changes per MFMA
          acc[i][4 * h + jl] = __builtin_amdgcn_mfma_f32_16x16x32_f16(bf[s][i], af[jl],
                                                                      acc[i][4 * h + jl], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (fetch) {
          // behind an A block's second pair: the same block of the next slice.  Behind the first
          // pairs: the B blocks of k-step 1 (during slice 1) or of the published k-tile's k-step 0
          // (during slice 3); each B set is idle while it is written.
          if (q & 1) af[jl] = frag_a(st, rks & 1, jl, rks >> 1);
          else if (t == 1) bf[1][jl] = frag_b(st, jl, 1);
          else if (t == 3) bf[0][jl] = frag_b(st, jl, 0);
        }
        extra(q);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    auto nothing = [](int) __attribute__((always_inline)) {};
    // A refill dealt one load behind every MFMA of one slice arrives at the texture unit faster
    // than it takes them (64 loads per CU in the time of 16 MFMAs): the wavefronts stall on
    // issue, the MFMAs behind the loads too.  So the A half goes behind every second MFMA of the
    // slice that frees the stage and the B half behind every second MFMA of the next slice.
    const char* b_half[B_IT] = {};  // B half still to be issued into the other stage
    auto with_b_half = [&](int q) __attribute__((always_inline)) {
      if (q & 1) issue_b(stage ^ 1, b_half[q / 2], q / 2);
    };
    // k-slices 0..2 of the k-tile in `stage`; `extra0` goes with the first
    auto first_slices = [&](auto&& extra0) __attribute__((always_inline)) {
      slice(0, true, stage, 1, extra0);
      slice(1, true, stage, 2, nothing);
      slice(0, true, stage, 3, nothing);
    };
    // publish the k-tile in the other stage
    auto publish_next = [&](bool behind_epilogue) __attribute__((always_inline)) {
      // behind an epilogue exactly EPI_STORES stores are younger than the loads waited for
      if (behind_epilogue) wait_vmcnt<EPI_STORES>();
      else wait_vmcnt<0>();
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    };
    // The final slice of k-tile kt (not the last): it takes the first fragments of the published
    // k-tile and starts the refill of this stage with the k-tile two ahead -- of this tile, or
    // the first of the next one; behind the last tile it loads this tile's first k-tile again,
    // which nobody reads (no branch around the loads).
    auto final_slice = [&](int kt) __attribute__((always_inline)) {
      const bool own = kt + 2 < KT;
      // (values, not a choice between two captured variables: that would index the closure)
      const bool stay = own || !has_next;
      const int ra = stay ? +m0 : +m0_n, rb = stay ? +n0 : +n0_n;
      const int kk = own ? kt + 2 : 0;
      const char* src = a_src(ra, kk);
      __builtin_amdgcn_sched_barrier(0);
      slice(1, true, stage ^ 1, 0, [&](int q) __attribute__((always_inline)) {
        if (q & 1) issue_a(stage, src, q / 2);
      });
#pragma unroll
      for (int n = 0; n < B_IT; ++n) b_half[n] = b_src(rb, kk, n);
      stage ^= 1;
    };

    // all k-tiles but the last; the first has no half refill to carry
    first_slices(nothing);
    publish_next(prev_stored);
    final_slice(0);
    for (int kt = 1; kt + 1 < KT; ++kt) {
      first_slices(with_b_half);
      publish_next(false);
      final_slice(kt);
    }

    // last k-tile: before its final slice the next tile's first k-tile is published (this
    // stage is free for a refill then); the bias is requested in front of the k-tile and waited
    // for BEFORE the next tile's second k-tile is requested, so that no wait inside the epilogue
    // falls behind those loads.  The next tile's first fragments are read after the epilogue.
    // fp16: requested a whole k-tile before it is needed; fp32 (twice the registers): in front
    // of the last slice
    typename Pack4<T>::type bias_raw[NB][2];
    if constexpr (sizeof(T) == 2) {
      if (wave_stores) load_bias16<T, NB>(ep, nw0, lq, bias_raw);
    }
    __builtin_amdgcn_sched_barrier(0);
    first_slices(with_b_half);
    if (has_next) publish_next(false);
    if constexpr (sizeof(T) == 4) {
      if (wave_stores) load_bias16<T, NB>(ep, nw0, lq, bias_raw);
    }
    __builtin_amdgcn_sched_barrier(0);
    slice(1, false, 0, 0, nothing);
    f4 bias_r[NB][2];
    bias_to_f32_16(bias_raw, bias_r);
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int g = 0; g < 2; ++g) asm volatile("" : "+v"(bias_r[i][g]));
    if (has_next) issue(stage, m0_n, n0_n, 1);
    stage ^= 1;

    // ---- epilogue: the next tile's first two k-tiles are landing meanwhile ----
    if (wave_stores) {
      char* slab = smem + SLABS + wave * 4096;
      // The lane id the epilogue derives its addresses from is re-made here from a value the
      // compiler cannot see through: otherwise it computes those addresses once, in front of the
      // tile loop, and they occupy registers through all the k-tiles.
      int lane_e = lane;
      asm volatile("" : "+v"(lane_e));
      if constexpr (HALF_SLABS) {
        if (ep.gelu) store_wave_tile_h<MB, NB, QKV, true, true>(acc, bias_r, ep, mw0, nw0, N, slab, lane_e);
        else store_wave_tile_h<MB, NB, QKV, false, true>(acc, bias_r, ep, mw0, nw0, N, slab, lane_e);
      } else {
        if (ep.gelu) store_wave_tile32<MB, NB, T, QKV, true>(acc, bias_r, ep, mw0, nw0, N, slab, lane_e);
        else store_wave_tile32<MB, NB, T, QKV, false>(acc, bias_r, ep, mw0, nw0, N, slab, lane_e);
      }
    }
    if (!has_next) break;
    read_first(stage);
    prev_stored = wave_stores;
    vp = vp_next;
    m0 = m0_n;
    n0 = n0_n;
  }
  wait_vmcnt<0>();  // the last tile's unread refill
}

// ---------------------------------------------------------------------------
// Streaming kernel WITH a residual (fp16 row-major output, whole 256 x 256 tiles): the
// persistent pipeline of gemm_stream_kernel, and the residual brought through LDS as in
// gemm_kernel<RESLDS>.  The residual of a tile (128 KB) has no place of its own in LDS, so it
// takes the operand stages as they fall free at the end of the tile, and the next tile's first two
// k-tiles take them back as the epilogue lets go of them:
//
//   final slice of k-tile KT-2   its stage is refilled with residual rows 0..63 of every
//                                wavefront's 128 x 64 sub-tile (8 loads, dealt between the MFMAs)
//   behind k-tile KT-1           barrier, then residual rows 64..127 into that stage (8 loads)
//   epilogue, row bands 0, 1     read the first half, 8 stores
//   between bands 1 and 2        barrier, then the NEXT tile's k-tile 0 into the first stage
//   epilogue, row bands 2, 3     read the second half, 8 stores
//   behind the epilogue          barrier, then the next tile's k-tile 1 into the second stage
//   start of the next tile       k-tile 0 has landed when at most 16 operations are outstanding
//                                (8 stores and 8 loads are younger), barrier, first fragments
//
// A barrier stands in front of every refill because a wavefront's loads write stripes of every
// wavefront's part of a stage.  What this buys over one workgroup per tile: no pipeline fill per
// tile beyond what the epilogue's second half hides, and no idle CU between two workgroups while
// the stores of the one that ended drain.  Whole tiles only; the launcher sends row tiles that
// do not fill a round of the persistent workgroups to the small-tile kernel.
// ---------------------------------------------------------------------------
template <int WM, int WN>
__global__ __launch_bounds__(512, 2) void gemm_stream_res_kernel(
    const _Float16* __restrict__ A, const _Float16* __restrict__ Bt, int M, int N, int Kp,
    int tiles_m, int tiles_n, int group_w, EpiDev ep) {
  constexpr int BM = 256, BN = 256, ROWB = 128, T_ = 512, KS = 4;
  static_assert(WM == 2 && WN == 4, "8 wavefronts, 128 x 64 sub-tiles");
  constexpr int TM = BM / WM, TN = BN / WN;
  constexpr int MB = TM / 32, NB = TN / 32;
  constexpr int A_IT = 4, B_IT = 4, LPT = A_IT + B_IT;
  constexpr int STAGE = (BM + BN) * ROWB;  // 64 KB
  constexpr int SLABS = 2 * STAGE;
  static_assert(MB * NB == LPT, "one load per MFMA of a k-slice");

  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % WM, wn = wave / WM;
  const int num_tiles = tiles_m * tiles_n;
  const int KT = Kp / 64;  // >= 3 (checked by the launcher)

  const int r0 = tid >> 3;
  unsigned lane_off[A_IT];
#pragma unroll
  for (int it = 0; it < A_IT; ++it)
    lane_off[it] = (unsigned)(r0 + it * 64) * (unsigned)Kp * 2u +
                   (unsigned)(((tid & 7) ^ ((r0 >> 1) & 7)) * 16);
  const unsigned smem_base = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)smem);
  const unsigned wave_off = smem_base + (unsigned)wave * 1024u;
  auto tile_origin = [&](int vp, int& m0, int& n0) __attribute__((always_inline)) {
    const int tile = xcd_tile(vp, num_tiles);
    const int grp = tile / (tiles_m * group_w);
    const int in_grp = tile - grp * tiles_m * group_w;
    const int grp_w = min(group_w, tiles_n - grp * group_w);
    m0 = (in_grp / grp_w) * BM;
    n0 = (grp * group_w + in_grp % grp_w) * BN;
  };
  // the halves of a k-tile (four loads per lane each) and their scalar sources, as in
  // gemm_stream_kernel
  auto a_src = [&](int m0, int k) __attribute__((always_inline)) {
    return (const char*)A + ((size_t)m0 * Kp * 2 + (size_t)k * ROWB);
  };
  // Source of load n (64-row block n) of the B tile at n0.  N is a multiple of 64, not
  // necessarily of 256: in the last column tile a block that starts at or past row N loads
  // block 0 again (the shift goes into the scalar source, the lane offsets stay); its products
  // are never stored.
  const size_t blk_bytes = (size_t)64 * Kp * 2;
  auto b_src = [&](int n0, int k, int n) __attribute__((always_inline)) {
    const int vb = (N - n0) >> 6;  // valid blocks of this tile (4 or more: all)
    const char* p = (const char*)Bt + ((size_t)n0 * Kp * 2 + (size_t)k * ROWB);
    return n < vb ? p : p - n * blk_bytes;
  };
  auto issue_a = [&](int stage, const char* src, int n) __attribute__((always_inline)) {
    lds_dma16_base(src, lane_off[n], wave_off + stage * STAGE + n * T_ * 16);
  };
  auto issue_b = [&](int stage, const char* src, int n) __attribute__((always_inline)) {
    lds_dma16_base(src, lane_off[n], wave_off + stage * STAGE + BM * ROWB + n * T_ * 16);
  };
  auto issue = [&](int stage, int m0, int n0, int k) __attribute__((always_inline)) {
    const char* a = a_src(m0, k);
#pragma unroll
    for (int n = 0; n < A_IT; ++n) issue_a(stage, a, n);
#pragma unroll
    for (int n = 0; n < B_IT; ++n) issue_b(stage, b_src(n0, k, n), n);
  };
  // Residual half h (rows 64 h .. 64 h + 63 of this wavefront's sub-tile) goes to the
  // wavefront's own 8 KB of `stage`: load q fetches 8 rows, lane l the 16-byte unit
  // (l % 8) ^ key of row 8 q + l / 8, key = (row >> 1) & 7 = (l / 16) ^ 4 (q & 1).
  unsigned res_lane_off[2];
#pragma unroll
  for (int odd = 0; odd < 2; ++odd)
    res_lane_off[odd] = ((unsigned)(lane >> 3) * (unsigned)N +
                         (unsigned)(((lane & 7) ^ (lane >> 4) ^ (odd * 4)) * 8)) * 2u;
  auto res_src = [&](int m0, int n0, int h) __attribute__((always_inline)) {
    return (const char*)ep.residual +
           (((int64_t)m0 + wm * TM + h * 64) * N + (n0 + wn * TN)) * 2;
  };
  const int64_t res_step = (int64_t)N * 16;  // 8 rows
  auto issue_res_one = [&](int stage, const char* src, int q) __attribute__((always_inline)) {
    lds_dma16_base(src + q * res_step, res_lane_off[q & 1],
                   smem_base + (unsigned)stage * STAGE + (unsigned)wave * 8192u + q * 1024);
  };

  // Fragments of v_mfma_f32_16x16x32_f16: a lane supplies row lane % 16 of a block of 16 rows and
  // the 8 halves of 16-byte unit lane / 16 of a 32-wide k-step.  (Which k goes to which lane group
  // is free as long as both operands agree: k is summed over.)  16 consecutive lanes read 16
  // consecutive rows at one unit, as with the 32-row fragments of the small-tile kernel: no bank
  // conflicts.
  const int lrow = lane & 15, lq = lane >> 4, fkey = (lrow >> 1) & 7;
  const int a_row_off = (wm * TM + lrow) * ROWB;
  const int b_row_off = BM * ROWB + (wn * TN + lrow) * ROWB;
  // A slice = one 32-wide k-step s times one half h of the sub-tile's rows: 4 A blocks (af; a
  // block's register takes the next slice's block as soon as its four MFMAs are issued) times 4 B
  // blocks (bf[s], good for both halves of step s).
  static_assert(TM == 128 && TN == 64, "128 x 64 sub-tiles");
  h8 af[4], bf[2][4];
  auto frag_a = [&](const char* st, int h, int jl, int s) __attribute__((always_inline)) {
    return *reinterpret_cast<const h8*>(st + a_row_off + (h * 64 + jl * 16) * ROWB +
                                        (((s * 4 + lq) ^ fkey) << 4));
  };
  auto frag_b = [&](const char* st, int i, int s) __attribute__((always_inline)) {
    return *reinterpret_cast<const h8*>(st + b_row_off + i * 16 * ROWB +
                                        (((s * 4 + lq) ^ fkey) << 4));
  };
  // the fragments of a k-tile's first slice
  auto read_first = [&](int stage) __attribute__((always_inline)) {
    const char* st = smem + stage * STAGE;
#pragma unroll
    for (int jl = 0; jl < 4; ++jl) af[jl] = frag_a(st, 0, jl, 0);
#pragma unroll
    for (int i = 0; i < 4; ++i) bf[0][i] = frag_b(st, i, 0);
  };
  auto barrier_lds = [&]() __attribute__((always_inline)) { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

  int vp = blockIdx.x;
  int m0, n0;
  tile_origin(vp, m0, n0);
  issue(0, m0, n0, 0);
  issue(1, m0, n0, 1);
  wait_vmcnt<LPT>();
  asm volatile("s_barrier" ::: "memory");
  read_first(0);
  int stage = 0;  // stage of the k-tile being multiplied

  while (true) {
    const int vp_next = vp + (int)gridDim.x;
    const bool has_next = vp_next < num_tiles;
    int m0_n = 0, n0_n = 0;
    if (has_next) tile_origin(vp_next, m0_n, n0_n);
    const int64_t mw0 = (int64_t)m0 + wm * TM;
    const int nw0 = n0 + wn * TN;
    // false: this wavefront's 64 columns lie past the edge -- it loads operands and keeps the
    // barriers, and has no residual, bias or output of its own
    const bool wave_stores = nw0 < N;

    // acc[i][j] = the 16 x 16 block of columns 16 i.., rows 16 j.. of the sub-tile: a lane holds
    // row lane % 16 and the 4 columns 4 (lane / 16) + 0..3
    f4 acc[2 * NB][2 * MB];
#pragma unroll
    for (int i = 0; i < 2 * NB; ++i)
#pragma unroll
      for (int j = 0; j < 2 * MB; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;

    // One slice, as in gemm_stream_kernel: eight pairs of MFMAs, the fragment reads for slice
    // `rks` of `rstage` behind them, `extra(q)` behind pair q.
    auto slice = [&](int, bool fetch, int rstage, int rks, auto&& extra) __attribute__((always_inline)) {
      // this slice is t = rks - 1 (mod 4): k-step s = t / 2, row half h = t % 2
      const int t = (rks + 3) & 3, s = t >> 1, h = t & 1;
      const char* st = smem + rstage * STAGE;
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const int jl = q >> 1;
#pragma unroll
        for (int p = 0; p < 2; ++p) {
          const int ii = (q & 1) * 2 + p;
          const int i = (jl & 1) ? 3 - ii : ii;  // one operand changes per MFMA
          acc[i][4 * h + jl] = __builtin_amdgcn_mfma_f32_16x16x32_f16(bf[s][i], af[jl],
                                                                      acc[i][4 * h + jl], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (fetch) {
          // behind an A block's second pair: the same block of the next slice.  Behind the first
          // pairs: the B blocks of k-step 1 (during slice 1) or of the published k-tile's k-step 0
          // (during slice 3); each B set is idle while it is written.
          if (q & 1) af[jl] = frag_a(st, rks & 1, jl, rks >> 1);
          else if (t == 1) bf[1][jl] = frag_b(st, jl, 1);
          else if (t == 3) bf[0][jl] = frag_b(st, jl, 0);
        }
        extra(q);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    auto nothing = [](int) __attribute__((always_inline)) {};
    // The three slices in front of a k-tile's last.  `extra0` deals the second half of the
    // refill that the slice before started: four loads there, four here, because eight behind
    // the MFMAs of one slice arrive faster than the texture unit takes them.
    auto first_slices = [&](auto&& extra0) __attribute__((always_inline)) {
      slice(0, true, stage, 1, extra0);
      slice(1, true, stage, 2, nothing);
      slice(0, true, stage, 3, nothing);
    };
    auto publish_next = [&]() __attribute__((always_inline)) {
      wait_vmcnt<0>();
      barrier_lds();
    };
    const char* b_half[B_IT] = {};  // B half still to be issued into the other stage
    auto with_b_half = [&](int q) __attribute__((always_inline)) {
      if (q & 1) issue_b(stage ^ 1, b_half[q / 2], q / 2);
    };
    // the final slice of a k-tile in front of the last but one: it takes the first fragments of
    // the published k-tile and starts the refill of this stage with the k-tile two ahead
    auto final_slice = [&](int kt) __attribute__((always_inline)) {
      const char* src = a_src(m0, kt + 2);
      __builtin_amdgcn_sched_barrier(0);
      slice(1, true, stage ^ 1, 0, [&](int q) __attribute__((always_inline)) {
        if (q & 1) issue_a(stage, src, q / 2);
      });
#pragma unroll
      for (int n = 0; n < B_IT; ++n) b_half[n] = b_src(n0, kt + 2, n);
      stage ^= 1;
    };

    // All k-tiles but the last two (KT >= 3, checked by the launcher): publish the next one (its
    // loads are the only ones in flight), refill this stage.  The first has no half refill to
    // carry.
    first_slices(nothing);
    publish_next();
    final_slice(0);
    for (int kt = 1; kt + 2 < KT; ++kt) {
      first_slices(with_b_half);
      publish_next();
      final_slice(kt);
    }
    // k-tile KT-2: its stage takes the first half of the residual
    const char* res0 = res_src(m0, n0, 0);
    first_slices(with_b_half);
    publish_next();
    slice(1, true, stage ^ 1, 0, [&](int q) __attribute__((always_inline)) {
      if ((q & 1) && wave_stores) issue_res_one(stage, res0, q / 2);
    });
    stage ^= 1;

    // last k-tile; its first slice carries the rest of the residual's first half, and behind its
    // fragment reads the stage is free for the second half.  The bias is requested in front of
    // the last slice and waited for behind it, before those loads are issued, so that no wait
    // the compiler places falls behind them.
    first_slices([&](int q) __attribute__((always_inline)) {
      if ((q & 1) && wave_stores) issue_res_one(stage ^ 1, res0, 4 + q / 2);
    });
    h4 bias_raw[NB][2];
    // all 4 loads in flight under the last slice
    if (wave_stores) load_bias16<_Float16, NB>(ep, nw0, lq, bias_raw);
    __builtin_amdgcn_sched_barrier(0);
    slice(1, false, 0, 0, nothing);
    f4 bias_r[NB][2];
    bias_to_f32_16(bias_raw, bias_r);
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int g = 0; g < 2; ++g) asm volatile("" : "+v"(bias_r[i][g]));
    barrier_lds();  // every wavefront has read the last k-tile's fragments
    if (wave_stores) {
      const char* res1 = res_src(m0, n0, 1);
#pragma unroll
      for (int q = 0; q < 8; ++q) issue_res_one(stage, res1, q);
    }
    stage ^= 1;  // now the stage of k-tile KT-2: the residual's first half, then the next tile's k-tile 0

    // ---- epilogue ----
    if (wave_stores) {
      const char* res_lo = smem + stage * STAGE + wave * 8192;
      const char* res_hi = smem + (stage ^ 1) * STAGE + wave * 8192;
      char* slab = smem + SLABS + wave * 4096;
      auto mid = [&]() __attribute__((always_inline)) {
        if (has_next) {
          barrier_lds();  // nobody reads the first half any more
          issue(stage, m0_n, n0_n, 0);
        }
      };
      if (ep.gelu)
        store_wave_tile_rs<MB, NB, true>(acc, bias_r, ep, mw0, nw0, N, res_lo, res_hi, slab, lane,
                                         has_next, mid);
      else
        store_wave_tile_rs<MB, NB, false>(acc, bias_r, ep, mw0, nw0, N, res_lo, res_hi, slab, lane,
                                          has_next, mid);
    } else if (has_next) {
      barrier_lds();  // the barrier and the refill of `mid`
      issue(stage, m0_n, n0_n, 0);
    }
    if (!has_next) break;
    barrier_lds();  // nobody reads the second half any more
    issue(stage ^ 1, m0_n, n0_n, 1);
    // the next tile's k-tile 0: younger are the 8 stores of row bands 2 and 3 (of a wavefront
    // that stores) and the 8 loads above
    if (wave_stores) wait_vmcnt<16>();
    else wait_vmcnt<8>();
    asm volatile("s_barrier" ::: "memory");
    read_first(stage);
    vp = vp_next;
    m0 = m0_n;
    n0 = n0_n;
  }
}

// CUs of the current device rounded down to a multiple of 8 (workgroup id % 8 = XCD for every
// tile of a persistent launch), or a negative error code.  The environment variable
// GPTMI_MAX_WORKGROUPS (read once) caps the number: a measurement knob -- with fewer persistent
// workgroups than CUs the chip's power management holds a higher clock, which is how one tells a
// kernel that is bound by the power budget from one that is bound by its own schedule.
inline int cu_count() {
  static int num_cus = 0;  // idempotent one-time setup; a race only repeats it
  if (num_cus == 0) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        cus < 8) {
      set_error("gemm: cannot query the CU count");
      return -4;
    }
    if (const char* cap = getenv("GPTMI_MAX_WORKGROUPS")) {
      const int c = atoi(cap);
      if (c >= 8 && c < cus) cus = c;
    }
    num_cus = cus - cus % 8;
  }
  return num_cus;
}

template <int WM, int WN, typename T, bool QKV>
int launch_stream(const void* A, const void* Bt, int64_t M, int N, int Kp, const EpiDev& ep,
                  hipStream_t st) {
  auto kern = gemm_stream_kernel<WM, WN, T, QKV>;
  constexpr int smem = 2 * 512 * 128 + 8 * 4096;  // 160 KB: two stages + the epilogue slabs
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
  const int num_cus = cu_count();
  if (num_cus < 0) return num_cus;
  const int tiles_m = (int)((M + 255) / 256), tiles_n = (N + 255) / 256;
  const int num_tiles = tiles_m * tiles_n;
  const int group_w = column_group(tiles_n, 256, Kp);
  const int grid = num_tiles < num_cus ? num_tiles : num_cus;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(512), smem, st, (const _Float16*)A,
                     (const _Float16*)Bt, (int)M, N, Kp, tiles_m, tiles_n, group_w, ep);
  return 0;
}

int launch_stream_res(const void* A, const void* Bt, int64_t M, int N, int Kp, const EpiDev& ep,
                      hipStream_t st) {
  auto kern = gemm_stream_res_kernel<2, 4>;
  constexpr int smem = 2 * 512 * 128 + 8 * 4096;  // 160 KB: two stages + the epilogue slabs
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
  const int num_cus = cu_count();
  if (num_cus < 0) return num_cus;
  const int tiles_m = (int)(M / 256), tiles_n = (N + 255) / 256;
  const int num_tiles = tiles_m * tiles_n;
  const int group_w = column_group(tiles_n, 256, Kp);
  const int grid = num_tiles < num_cus ? num_tiles : num_cus;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(512), smem, st, (const _Float16*)A,
                     (const _Float16*)Bt, (int)M, N, Kp, tiles_m, tiles_n, group_w, ep);
  return 0;
}

// Problems too small for the 256 x 256 tiles (and the last rows of the persistent launches): 4
// wavefronts on 128 x 128 tiles, K step 32, 4-stage ring -- unless that leaves most CUs without
// a workgroup; then smaller tiles with a K step of 64, so that the few k-tiles a workgroup walks
// (each a barrier and an LDS round trip) are as few as possible.  Last 768 rows of the headline
// GEMMs, one box: N = 768, K = 3072: 40 -> 19 us; N = K = 768: 15 -> 8; N = 2304: 15 -> 10;
// N = 3072: 14.6 -> 12.5.
template <typename T, bool QKV>
int launch_small(const void* A, const void* Bt, int64_t M, int N, int Kp, const EpiDev& ep,
                 hipStream_t st) {
  const int cus = cu_count();
  if (cus < 0) return cus;
  const int64_t tiles128 = ((M + 127) / 128) * ((N + 127) / 128);
  if (tiles128 * 4 <= cus) return launch_cfg<64, 64, 2, 1, 64, 4, 2, T, QKV>(A, Bt, M, N, Kp, ep, st);
  if (tiles128 <= cus) return launch_cfg<64, 128, 2, 2, 64, 3, 2, T, QKV>(A, Bt, M, N, Kp, ep, st);
  return launch_cfg<128, 128, 2, 2, 32, 4, 2, T, QKV>(A, Bt, M, N, Kp, ep, st);
}

template <typename T, bool QKV>
int launch_shape(const void* A, const void* Bt, int64_t M, int N, int Kp, const EpiDev& ep,
                 hipStream_t st) {
  // Big problems: 256x256 tiles, 8 wavefronts (2x4, wave tile 128x64), K step 64 -- full
  // 128-byte rows per direct load move ~1.5x the bytes per clock of 64-byte rows -- double
  // buffered (2 x 64 KB of LDS).  Small ones: 128x128 tiles, 4 wavefronts, K step 32, 4-stage
  // ring, so that a few hundred rows still spread over several CUs.
  if (M >= 2048 && N >= 256) {
    // N a multiple of 64 (the wavefronts of the last column tile whose 64 columns lie past the
    // edge store nothing), at least two k-tiles, vector epilogue (16-byte stores for fp16), no
    // dropout, no residual: the streaming kernel on the whole row tiles.  It has neither row edge
    // handling nor the generator; rows past the last whole tile go to the small tiles below.
    const int64_t m_full = M / 256 * 256;
    if (N % 64 == 0 && Kp >= 128 && Kp <= (1 << 21) && ep.vec_ok &&
        (sizeof(T) == 4 || ep.vec8_ok) && !(ep.drop.p > 0.f) && ep.residual == nullptr) {
      // Every persistent workgroup walks ceil(tiles / CUs) tiles, so a few tiles beyond a whole
      // number of rounds cost a full round.  Then the last rows leave the persistent launch --
      // as many row tiles stay as fill whole rounds -- and go to the small-tile kernel, whose
      // many short workgroups spread over all CUs (headline ffn1: 7200 tiles = 28 rounds + 32
      // tiles; 597 of the 600 row tiles stay, 768 rows follow as 288 tiles of 64 x 128).
      const int cus = cu_count();
      if (cus < 0) return cus;
      const int64_t tiles_m = m_full / 256, tiles_n = (N + 255) / 256, tiles = tiles_m * tiles_n;
      const int64_t rounds = tiles / cus, rem = tiles % cus;
      int64_t m_head = m_full;
      if (rounds >= 4 && rem != 0 && rem * 4 <= cus) m_head = rounds * cus / tiles_n * 256;
      int rc = launch_stream<2, 4, T, QKV>(A, Bt, m_head, N, Kp, ep, st);
      if (rc != 0 || m_head == M) return rc;
      EpiDev tail = ep;
      if (QKV) tail.m_off = ep.m_off + (int)m_head;
      else tail.out = (T*)ep.out + m_head * N;
      return launch_small<T, QKV>((const _Float16*)A + m_head * Kp, Bt,
                                                          M - m_head, N, Kp, tail, st);
    }
    // fp16 with a residual, no dropout: whole tiles fetch the residual through LDS
    if constexpr (sizeof(T) == 2 && !QKV) {
      if (ep.residual != nullptr && !(ep.drop.p > 0.f) && ep.vec8_ok && Kp >= 128 &&
          (((uintptr_t)ep.residual) & 15) == 0) {
        if (N % 64 == 0 && Kp >= 192 && Kp <= (1 << 21)) {
          // N a multiple of 64 and at least three k-tiles: the streaming kernel on the whole row
          // tiles, with the same cut as above -- the row tiles that fill whole rounds of the
          // persistent workgroups stay, the rest (headline N = 768: 1800 tiles = 7 rounds + 8;
          // 597 of 600 row tiles stay) go to the small tiles
          const int cus = cu_count();
          if (cus < 0) return cus;
          const int64_t tiles_m = m_full / 256, tiles_n = (N + 255) / 256, tiles = tiles_m * tiles_n;
          const int64_t rounds = tiles / cus, rem = tiles % cus;
          int64_t m_head = m_full;
          if (rounds >= 4 && rem != 0 && rem * 4 <= cus) m_head = rounds * cus / tiles_n * 256;
          int rc = launch_stream_res(A, Bt, m_head, N, Kp, ep, st);
          if (rc != 0 || m_head == M) return rc;
          EpiDev tail = ep;
          tail.out = (T*)ep.out + m_head * N;
          tail.residual = (const T*)ep.residual + m_head * N;
          return launch_small<T, QKV>((const _Float16*)A + m_head * Kp, Bt,
                                                              M - m_head, N, Kp, tail, st);
        }
        return launch_cfg<256, 256, 2, 4, 64, 2, 2, T, QKV, true>(A, Bt, M, N, Kp, ep, st);
      }
    }
    return launch_cfg<256, 256, 2, 4, 64, 2, 2, T, QKV>(A, Bt, M, N, Kp, ep, st);
  }
  return launch_small<T, QKV>(A, Bt, M, N, Kp, ep, st);
}

}  // namespace

// The device-side epilogue description of a launch, or a negative error code.
static int make_epi(const GemmEpilogue& e, int64_t M, int N, EpiDev& ep) {
  if (M >= (1ll << 31) - 512) {
    set_error("gemm: M=%lld does not fit the kernel's 32-bit row index", (long long)M);
    return -2;
  }
  if (e.qkv && (e.d % 4) != 0) {
    set_error("gemm qkv epilogue: head size %d must be a multiple of 4", e.d);
    return -2;
  }
  ep = EpiDev{};
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
  ep.drop = DropoutArgs{e.qkv ? 0.f : e.drop.p, (unsigned)e.drop.seed,
                        (unsigned)(e.drop.seed >> 32)};
  const uintptr_t amask = e.f16 ? 7 : 15;
  auto aligned = [&](const void* p) { return p == nullptr || ((uintptr_t)p & amask) == 0; };
  const bool vec = (N % 4) == 0 && aligned(e.bias) && aligned(e.residual) && aligned(e.out) &&
                   aligned(e.q) && aligned(e.k) && aligned(e.v);
  ep.vec_ok = vec ? 1 : 0;
  auto aligned16 = [&](const void* p) { return ((uintptr_t)p & 15) == 0; };
  ep.vec8_ok = vec && e.f16 && (N % 8) == 0 && aligned16(e.out) && aligned16(e.q) &&
               aligned16(e.k) && aligned16(e.v) && (!e.qkv || (e.d % 8) == 0);
  return 0;
}

int launch_gemm(const void* A, const void* Bt, int64_t M, int N, int Kp, const GemmEpilogue& e,
                hipStream_t st) {
  EpiDev ep;
  if (const int rc = make_epi(e, M, N, ep)) return rc;
  if (e.f16)
    return e.qkv ? launch_shape<_Float16, true>(A, Bt, M, N, Kp, ep, st)
                 : launch_shape<_Float16, false>(A, Bt, M, N, Kp, ep, st);
  return e.qkv ? launch_shape<float, true>(A, Bt, M, N, Kp, ep, st)
               : launch_shape<float, false>(A, Bt, M, N, Kp, ep, st);
}

bool gemm_layernorm_supported(int64_t M, int H) {
  if (H <= 0 || H % 64 != 0 || M <= 0) return false;
  const int nchunks = H / 8, lpr = lanes_per_row(nchunks);
  return (nchunks + lpr - 1) / lpr <= 8 && lna_lds_bytes(H) <= 160 * 1024;
}

int launch_gemm_layernorm(const void* x, const void* ln_w, const void* ln_b, float eps,
                          const void* Bt, int64_t M, int N, int H, const GemmEpilogue& e,
                          hipStream_t st) {
  if (!e.f16 || e.residual != nullptr || e.drop.p > 0.f || !gemm_layernorm_supported(M, H)) {
    set_error("gemm with LayerNorm prologue: fp16, no residual, no dropout, H=%d a multiple of "
              "64 whose 32-row panel fits the LDS", H);
    return -2;
  }
  if ((((uintptr_t)x | (uintptr_t)ln_w | (uintptr_t)ln_b | (uintptr_t)Bt) & 15) != 0) {
    set_error("gemm with LayerNorm prologue: x, the LayerNorm parameters and W must be 16-byte aligned");
    return -2;
  }
  EpiDev ep;
  if (const int rc = make_epi(e, M, N, ep)) return rc;
  const LnArgs ln = {ln_w, ln_b, eps, lanes_per_row(H / 8)};
  return e.qkv ? launch_lna<true>(x, Bt, M, N, H, ep, ln, st)
               : launch_lna<false>(x, Bt, M, N, H, ep, ln, st);
}

}  // namespace gptmi
