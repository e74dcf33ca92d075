/*
 * gptmi.h -- C ABI of libgptmi.so: the GPT-2 forward hot path as hand-written
 * HIP kernels for gfx950 (MI355X).
 *
 * Conventions shared by every entry point
 *   - all data pointers are DEVICE pointers into memory owned by the caller;
 *     nothing is allocated, freed or retained by the library;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *     every call only enqueues work on it and never synchronises;
 *   - `dtype` is a gptmi_dtype and names the storage type of the floating
 *     point tensors of that call (activations, weights and outputs alike);
 *   - the return value is 0 on success or a negative gptmi_status; the text of
 *     the most recent failure on the calling thread is gptmi_last_error();
 *   - besides that thread-local message the library keeps, per process, only
 *     facts it looks up once and never changes: the compute-unit count of the
 *     device that made the first GEMM / attention call (all devices of a
 *     process are assumed to be the same model), "kernel attribute set" flags,
 *     and the per-device address of gptmi_linear_static's scratch array.  A
 *     race on any of them only repeats the lookup, so calls from several host
 *     threads / streams are independent (gptmi_linear_static excepted: see
 *     its comment);
 *   - one environment variable is read, once: GPTMI_MAX_WORKGROUPS=<n> caps
 *     the persistent GEMM launches at n workgroups instead of one per compute
 *     unit (a measurement knob; unset in normal use).
 *
 * Each declaration cites the reference interface it stands in for
 * (thevasudevgupta/gpt-triton, file:line).  The reference has no FFI of its
 * own: its operators are Python functions that launch Triton kernels, and the
 * entry points below are what those Python functions bind to instead.
 */
#ifndef GPTMI_H
#define GPTMI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GPTMI_VERSION 102 /* major*10000 + minor*100 + patch */

/* Size of the scratch array built into the library for gptmi_linear_static (8 MiB). */
#define GPTMI_STATIC_SCRATCH_BYTES (8u << 20)

typedef enum gptmi_dtype {
  GPTMI_F32 = 0, /* IEEE binary32 storage */
  GPTMI_F16 = 1  /* IEEE binary16 storage, fp32 arithmetic inside kernels */
} gptmi_dtype;

typedef enum gptmi_status {
  GPTMI_OK = 0,
  GPTMI_ERR_INVALID = -1,     /* NULL pointer, non-positive size, bad enum, p outside [0,1) */
  GPTMI_ERR_UNSUPPORTED = -2, /* valid request the kernels do not implement */
  GPTMI_ERR_WORKSPACE = -3,   /* workspace missing or too small */
  GPTMI_ERR_LAUNCH = -4       /* hipGetLastError() after the launch != success */
} gptmi_status;

/* Layout of the weight operand of gptmi_linear. */
typedef enum gptmi_wlayout {
  GPTMI_W_KN = 0, /* W[K][N] row-major: the reference's (and HF Conv1D's) in x out layout */
  GPTMI_W_NK = 1, /* W[N][K] row-major: out x in, e.g. the tied LM head over wte[V][H] */
  GPTMI_W_PACKED = 2 /* the fp16 [N][round_up(K,64)] image written by gptmi_pack_weight */
} gptmi_wlayout;

/* Layout of the output of gptmi_flash_attn. */
typedef enum gptmi_olayout {
  GPTMI_O_BNLD = 0, /* out[B][N][Lq][d]: what the reference returns */
  GPTMI_O_BLND = 1  /* out[B][Lq][N][d]: heads already merged, i.e. the result of
                       out.transpose(1, 2).contiguous() without the copy */
} gptmi_olayout;

/* Library version (GPTMI_VERSION of the build). */
int gptmi_version(void);

/* Message of the last failing call on this thread ("" if none). */
const char* gptmi_last_error(void);

/*
 * out[b,l,:] = wte[ids[b,l],:] + wpe[l,:]            (one add in the storage dtype)
 *
 * Replaces fused_embeddings(x, wte, wpe, dropout_prob) -> kernels.py:75-101 and
 * fused_embeddings_kernel -> kernels.py:37-72.
 *   ids  int64 [B*L]          wte [V][H]     wpe [P][H]     out [B*L][H]
 * Requires L <= P.  A token id outside [0, V) reads no memory: its wte row counts as zeros, so
 * the output row is wpe[l,:] (the reference does not check and reads out of bounds).
 * Dropout (0 <= p < 1, dropout() -> kernels.py:31-34): the sum, rounded to the storage
 * dtype, is kept where rand(seed, column) > p and divided by (1 - p), else zeroed; rand is
 * Triton's tl.rand, i.e. Philox-4x32-10 with counter (column, 0, 0, 0), the 64-bit seed as
 * key and the first output word mapped to [0, 1).  The column is the only offset
 * (kernels.py:65-70), so every token gets the same mask; the reference's seed is 1337
 * (kernels.py:49).
 */
int gptmi_embed(const int64_t* ids, const void* wte, const void* wpe, void* out,
                int64_t B, int64_t L, int64_t V, int64_t P, int64_t H,
                float p, uint64_t seed, int dtype, void* stream);

/*
 * gptmi_embed (without dropout) and gptmi_layernorm of its result in one pass over the rows:
 *   emb[b,l,:] = wte[ids[b,l],:] + wpe[l,:]          out[b,l,:] = LayerNorm(emb[b,l,:]; ln_w, ln_b)
 * Both outputs are bit-identical to the two calls made one after the other (the LayerNorm works
 * on the sum as rounded to the storage dtype); the row stays in registers in between.
 *
 * Replaces the pair fused_embeddings(x, wte, wpe) -> gpt.py:166-170 / kernels.py:75-101 and the
 * first block's fused_layer_norm(x, weight, bias) -> gpt.py:40 / kernels.py:148-164, which the
 * reference's author marks as a fusion to do (kernels.py:132-133).
 *   ids int64 [B*L]   wte [V][H]   wpe [P][H]   ln_w, ln_b [H]   emb, out [B*L][H]   H <= 8192
 */
int gptmi_embed_layernorm(const int64_t* ids, const void* wte, const void* wpe,
                          const void* ln_w, const void* ln_b, void* emb, void* out,
                          int64_t B, int64_t L, int64_t V, int64_t P, int64_t H, float eps,
                          int dtype, void* stream);

/*
 * out[m,:] = (x[m,:] - mean_m) * rstd_m * w + b, rstd = 1/sqrt(var + eps),
 * mean and the centred, biased variance in fp32; x is read from HBM once.
 *
 * Replaces fused_layer_norm(x, weight, bias) -> kernels.py:148-164 and
 * fused_layer_norm_kernel -> kernels.py:104-145 (eps = 1e-5 there).
 *   x, out [M][H]     w, b [H]      1 <= H <= 8192
 */
int gptmi_layernorm(const void* x, const void* w, const void* b, void* out,
                    int64_t M, int64_t H, float eps, int dtype, void* stream);

/*
 * out[m,:] = softmax(x[m,:]) with fp32 max / sum; x is read from HBM once.
 *
 * The reference only sketches this op in a commented-out kernel
 * (kernels.py:318-342); the contract here is torch.softmax(x.float(), -1).
 *   x, out [M][H]     1 <= H <= 8192
 */
int gptmi_softmax(const void* x, void* out, int64_t M, int64_t H, int dtype,
                  void* stream);

/*
 * Bytes of workspace gptmi_linear / gptmi_linear_qkv need for these sizes
 * (0 if none).  The workspace holds the fp16, K-contiguous, zero-padded copy of
 * the weight (and of x when x is fp32 or K is not a multiple of 64).
 */
size_t gptmi_linear_workspace_bytes(int64_t M, int64_t N, int64_t K, int dtype,
                                    int wlayout);

/*
 * Bytes of the packed image of a [K][N] weight: fp16 [N][round_up(K, 64)].
 */
size_t gptmi_packed_weight_bytes(int64_t N, int64_t K);

/*
 * Writes the packed image of W (layout GPTMI_W_KN or GPTMI_W_NK, storage `dtype`)
 * into `packed` (gptmi_packed_weight_bytes(N, K) bytes, 256-byte aligned): the
 * weight rounded to fp16, K-contiguous, zero padded to a multiple of 64.  It is
 * what gptmi_linear builds in its workspace on every call; packing once and
 * passing GPTMI_W_PACKED skips that step for weights that do not change.
 * No counterpart in the reference (its Triton kernel reads W[K][N] in place,
 * kernels.py:231-234).
 */
int gptmi_pack_weight(const void* W, void* packed, int64_t N, int64_t K, int wlayout,
                      int dtype, void* stream);

/*
 * out = gelu?(x @ W + bias) + residual
 * Operands of the product are rounded to fp16, products and sums are fp32
 * (MFMA), then in fp32: + bias, tanh-GELU if `gelu`, + residual; one rounding
 * to the storage dtype at the store.
 *
 * Replaces fused_ffn(x, weight, bias, residual, add_gelu, dropout_prob) ->
 * kernels.py:260-315 and fused_ffn_kernel -> kernels.py:169-257.
 *   x [M][K]   W [K][N] (GPTMI_W_KN), [N][K] (GPTMI_W_NK) or packed (GPTMI_W_PACKED)
 *   bias [N] or NULL
 *   residual [M][N] or NULL     out [M][N] (may be the residual's own memory: every
 *                               element is read before it is written)
 * workspace: at least gptmi_linear_workspace_bytes(...) bytes, 256-byte aligned
 * (may be NULL when that is 0).
 * Any M >= 1 (below 2^31 - 512), 1 <= N <= 2^26, 1 <= K <= 2^30 (GPTMI_ERR_UNSUPPORTED beyond)
 * and any pointer alignment the element type allows are accepted; the fast
 * epilogues need N a multiple of 8 (fp16) or 4 (fp32) and 16-byte aligned bias, residual and
 * out, everything else takes element-wise code with the same results.
 * Dropout (0 < p < 1; 0 = none) sits between the GELU and the residual
 * (kernels.py:245-255): keep where rand(seed, (uint32)(m*N + n)) > p, divide by (1 - p);
 * same generator as gptmi_embed, reference seed 1337 (kernels.py:181).
 */
int gptmi_linear(const void* x, const void* W, const void* bias,
                 const void* residual, void* out, int64_t M, int64_t N, int64_t K,
                 int gelu, float p, uint64_t seed, int wlayout, void* workspace,
                 size_t workspace_bytes, int dtype, void* stream);

/*
 * gptmi_linear without the workspace arguments, for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No
 * counterpart in the reference.  Same arguments, arithmetic, kernels and results as gptmi_linear;
 * the packed operand images that gptmi_linear writes into the caller's workspace go into a
 * GPTMI_STATIC_SCRATCH_BYTES array of device memory that is part of the library image (each GPU
 * the library runs on holds it until the process ends).  The call allocates and frees nothing.
 *   - Sizes whose gptmi_linear_workspace_bytes(M, N, K, dtype, wlayout) exceeds
 *     gptmi_linear_static_capacity() are refused with GPTMI_ERR_WORKSPACE (fp16, K % 64 == 0,
 *     W[K][N]: N*K*2 <= 8 MiB, e.g. every GEMM of GPT-2 124M; GPTMI_W_PACKED needs no scratch).
 *   - Every call on a GPU shares that GPU's array and keeps nothing in it between calls (the
 *     images are rewritten in full by each call).  Calls that overlap on one GPU -- two streams,
 *     two host threads -- race on it; calls on one stream are ordered and safe.
 *   - The first call on a device resolves the array's address there (hipGetSymbolAddress); make
 *     that call outside a graph capture.
 */
size_t gptmi_linear_static_capacity(void);
int gptmi_linear_static(const void* x, const void* W, const void* bias,
                        const void* residual, void* out, int64_t M, int64_t N, int64_t K,
                        int gelu, float p, uint64_t seed, int wlayout, int dtype,
                        void* stream);

/*
 * y = x @ W + bias with y's 3*heads*d columns split as [q | k | v] and each
 * third scattered head-major by the GEMM epilogue:
 *   q[b][n][l][:] = y[b*L + l][n*d : (n+1)*d], k at column offset heads*d,
 *   v at 2*heads*d.
 *
 * Replaces matmul_and_split_qkv(x, weight, bias, num_heads) -> kernels.py:347-367
 * (fused_ffn followed by split + 3 x view/transpose/contiguous copies).
 *   x [B*L][K]   W [K][3*heads*d] (GPTMI_W_KN) or packed   bias [3*heads*d] or NULL
 *   q, k, v [B][heads][L][d]       d a multiple of 8 (GPTMI_ERR_UNSUPPORTED otherwise; the
 *                                  16-byte scatter stores also need 16-byte aligned q, k, v)
 */
int gptmi_linear_qkv(const void* x, const void* W, const void* bias, void* q,
                     void* k, void* v, int64_t B, int64_t L, int64_t heads,
                     int64_t d, int64_t K, int wlayout, void* workspace,
                     size_t workspace_bytes, int dtype, void* stream);

/*
 * out = gelu?(LayerNorm(x; ln_w, ln_b, eps) @ W + bias), and the same with the head-major
 * scatter of gptmi_linear_qkv: the LayerNorm runs in the GEMM's operand prologue.  Every
 * workgroup normalises the 32 rows of its tile (fp32 statistics, the arithmetic of
 * gptmi_layernorm: the operand has the bits of that call's output) into LDS; the normalised
 * matrix never goes to memory and its kernel launch is gone.  Each column tile of a row block
 * normalises the rows again, so this pays for FEW rows, where a forward is bound by its launches
 * (the callers in gpt.py use it below a row count and gptmi_layernorm + gptmi_linear above).
 *
 * Replaces the pairs fused_layer_norm -> matmul_and_split_qkv (gpt.py:40-41) and
 * fused_layer_norm -> fused_ffn (gpt.py:92-93) of the reference's blocks: the fusion its
 * author marks as to do at kernels.py:132-133.
 *   x [M][K] fp16 (M = B*L)   ln_w, ln_b [K]   W_packed: the image gptmi_pack_weight writes
 *   bias [N] or NULL          K a multiple of 64; fp16 storage only; no residual, no dropout
 * gptmi_layernorm_linear_supported(M, K, dtype) = 1 where the calls take these sizes; they
 * return GPTMI_ERR_UNSUPPORTED elsewhere (K not a multiple of 64 or beyond what the 32-row
 * panel of 64*K bytes leaves of the LDS beside 48 KB of weight stages; fp32 storage).
 */
int gptmi_layernorm_linear_supported(int64_t M, int64_t K, int dtype);
int gptmi_layernorm_linear(const void* x, const void* ln_w, const void* ln_b, float eps,
                           const void* W_packed, const void* bias, void* out, int64_t M,
                           int64_t N, int64_t K, int gelu, int dtype, void* stream);
int gptmi_layernorm_linear_qkv(const void* x, const void* ln_w, const void* ln_b, float eps,
                               const void* W_packed, const void* bias, void* q, void* k,
                               void* v, int64_t B, int64_t L, int64_t heads, int64_t d,
                               int64_t K, int dtype, void* stream);

/*
 * out = softmax(causal(q k^T * scale)) v, mask "key index <= query index".
 * q, k, v are rounded to fp16; scores, running max, exponentials and the
 * denominator are fp32; keys are visited in tiles of 64 in ascending order with
 * the running max updated per tile; P is rounded to fp16 for the P.V product
 * while the denominator sums the unrounded fp32 P; the final divide is fp32.
 *
 * Replaces flash_attention_v1(q, k, v, dropout_prob) -> kernels.py:477-525 and
 * flash_attention_v1_kernel -> kernels.py:375-474.
 *   q [B][N][Lq][d]    k, v [B][N][Lk][d]    d = 16, 32, 64, 128 or 256 (the reference's
 *   set, kernels.py:490; 16 and 32 are read at their own row pitch and multiplied on the
 *   64-wide tiles of the d = 64 kernel, the missing columns being zeros in LDS only)
 * Lq != Lk behaves as in the reference (kernels.py:421-436): the mask is "key <= query" from the
 * top left, nothing else, and the last 64-key tile is filled up with zero rows.  So with Lq < Lk
 * the keys past the last query play no part, and with Lq > Lk a query at or past Lk attends to all
 * Lk keys AND to the zero rows Lk .. min(query, round_up(Lk, 64) - 1) (score 0, value 0), which
 * only add to its denominator.
 *   out: [B][N][Lq][d] (GPTMI_O_BNLD) or [B][Lq][N][d] (GPTMI_O_BLND)
 * Dropout (0 < p < 1; 0 = none) hits P after the denominator has summed it and before its
 * fp16 rounding (kernels.py:457-466): keep where rand(seed, (uint32)(lq*Lk + lk)) > p,
 * divide by (1 - p); the offset ignores batch and head, reference seed 1337 (kernels.py:387).
 */
int gptmi_flash_attn(const void* q, const void* k, const void* v, void* out,
                     int64_t B, int64_t N, int64_t Lq, int64_t Lk, int64_t d,
                     float scale, float p, uint64_t seed, int olayout, int dtype,
                     void* stream);

#ifdef __cplusplus
}
#endif
#endif /* GPTMI_H */
