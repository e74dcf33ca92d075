// The C ABI of libgptmi (declared in include/gptmi.h): argument validation,
// operand packing for the GEMM, and dispatch to the kernel launchers.
#include "../../include/gptmi.h"

#include <stdarg.h>
#include <stdio.h>

#include <mutex>

#include "common.h"
#include "launch.h"

namespace gptmi {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

static int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return GPTMI_ERR_LAUNCH;
  }
  return GPTMI_OK;
}

static bool dtype_ok(int dtype) { return dtype == GPTMI_F32 || dtype == GPTMI_F16; }
static bool dropout_ok(float p) { return p >= 0.0f && p < 1.0f; }  // false for NaN too

static inline int64_t round_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

// Widest output row the GEMM epilogues address: their per-lane offsets cover up to 8 rows of N
// elements of 4 bytes in an unsigned 32-bit register (8 * 2^26 * 4 = 2^31).
constexpr int kMaxN = 1 << 26;

// Workspace plan of one GEMM: where the packed weight and (if needed) the
// packed activations live.
struct LinearPlan {
  int Kp;
  bool pack_x;     // x must be converted / zero padded into the workspace
  size_t w_off, w_bytes, x_off, x_bytes, total;
};

static LinearPlan plan_linear(int64_t M, int64_t N, int64_t K, int dtype, int wlayout) {
  LinearPlan p;
  p.Kp = (int)round_up(K, 64);
  p.pack_x = !(dtype == GPTMI_F16 && p.Kp == K);
  const bool pack_w = !(wlayout == GPTMI_W_PACKED ||
                        (wlayout == GPTMI_W_NK && dtype == GPTMI_F16 && p.Kp == K));
  p.w_off = 0;
  p.w_bytes = pack_w ? (size_t)round_up(N * (int64_t)p.Kp * 2, 256) : 0;
  p.x_off = p.w_bytes;
  p.x_bytes = p.pack_x ? (size_t)round_up(M * (int64_t)p.Kp * 2, 256) : 0;
  p.total = p.w_bytes + p.x_bytes;
  return p;
}

// Packs operands as the plan says; returns the A and Bt pointers the GEMM reads.
static int prepare_operands(const void* x, const void* W, int64_t M, int64_t N, int64_t K,
                            int dtype, int wlayout, void* workspace, size_t workspace_bytes,
                            hipStream_t st, const void** A, const void** Bt, int* Kp) {
  const LinearPlan p = plan_linear(M, N, K, dtype, wlayout);
  if (p.total > 0) {
    if (workspace == nullptr || workspace_bytes < p.total) {
      set_error("linear: workspace of %zu bytes needed, %zu given", p.total,
                workspace ? workspace_bytes : (size_t)0);
      return GPTMI_ERR_WORKSPACE;
    }
    if (((uintptr_t)workspace & 255) != 0) {
      set_error("linear: workspace must be 256-byte aligned");
      return GPTMI_ERR_WORKSPACE;
    }
  }
  const bool f16 = dtype == GPTMI_F16;
  char* ws = (char*)workspace;
  if (p.w_bytes) {
    if (wlayout == GPTMI_W_KN)
      launch_pack_transpose(W, ws + p.w_off, (int)K, (int)N, p.Kp, f16, st);
    else
      launch_pack_rows(W, ws + p.w_off, N, (int)K, p.Kp, f16, st);
    *Bt = ws + p.w_off;
  } else {
    *Bt = W;
  }
  if (p.pack_x) {
    launch_pack_rows(x, ws + p.x_off, M, (int)K, p.Kp, f16, st);
    *A = ws + p.x_off;
  } else {
    *A = x;
  }
  *Kp = p.Kp;
  return GPTMI_OK;
}

// Scratch of gptmi_linear_static: the packed operand images that gptmi_linear puts into the
// caller's workspace.  Every GPU the library runs on holds its own copy of the array (at its own
// address) until the process ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress -- never a device address -- so all uses go through static_scratch().
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[GPTMI_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;

// Device address of `scratch` on the current device, resolved once per device; nullptr (and
// the error text set) on failure.
static void* static_scratch() {
  static std::mutex mu;
  static void* ptrs[kMaxDevices] = {};
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    set_error("linear_static: cannot identify the current device (%s, device %d)",
              hipGetErrorString(e), dev);
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(mu);
  if (ptrs[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) {
      set_error("linear_static: hipGetSymbolAddress(scratch) on device %d: %s", dev,
                hipGetErrorString(e));
      return nullptr;
    }
    ptrs[dev] = p;
  }
  return ptrs[dev];
}

// gptmi_linear and gptmi_linear_static behind their argument checks: pack the operands into
// `workspace` as the plan says, then the GEMM.
static int linear_impl(const void* x, const void* W, const void* bias, const void* residual,
                       void* out, int64_t M, int64_t N, int64_t K, int gelu, float p,
                       uint64_t seed, int wlayout, void* workspace, size_t workspace_bytes,
                       int dtype, hipStream_t st) {
  const void *A, *Bt;
  int Kp;
  int rc = prepare_operands(x, W, M, N, K, dtype, wlayout, workspace, workspace_bytes, st,
                            &A, &Bt, &Kp);
  if (rc) return rc;
  if (((uintptr_t)A & 15) || ((uintptr_t)Bt & 15)) {
    set_error("linear: x and W must be 16-byte aligned");
    return GPTMI_ERR_INVALID;
  }
  GemmEpilogue ep = {};
  ep.bias = bias;
  ep.residual = residual;
  ep.out = out;
  ep.gelu = gelu ? 1 : 0;
  ep.drop = Dropout{p, seed};
  ep.qkv = false;
  ep.f16 = dtype == GPTMI_F16;
  rc = launch_gemm(A, Bt, M, (int)N, Kp, ep, st);
  if (rc) return rc;
  return check_launch("linear");
}

static int check_linear_args(const void* x, const void* W, const void* out, int64_t M, int64_t N,
                             int64_t K, float p, int wlayout, int dtype) {
  if (!x || !W || !out || M <= 0 || N <= 0 || K <= 0 || !dtype_ok(dtype) ||
      (wlayout != GPTMI_W_KN && wlayout != GPTMI_W_NK && wlayout != GPTMI_W_PACKED)) {
    set_error("linear: invalid argument");
    return GPTMI_ERR_INVALID;
  }
  // the epilogues form per-lane byte offsets of up to 8 rows (8 * N * 4 bytes in fp32) in 32 bits
  if (N > kMaxN || K > (1 << 30)) {
    set_error("linear: N=%lld beyond %d or K=%lld beyond 2^30", (long long)N, kMaxN, (long long)K);
    return GPTMI_ERR_UNSUPPORTED;
  }
  if (!dropout_ok(p)) {
    set_error("linear: dropout probability %g outside [0, 1)", (double)p);
    return GPTMI_ERR_INVALID;
  }
  return GPTMI_OK;
}

}  // namespace gptmi

using namespace gptmi;

extern "C" {

int gptmi_version(void) { return GPTMI_VERSION; }

const char* gptmi_last_error(void) { return g_err; }

int gptmi_embed(const int64_t* ids, const void* wte, const void* wpe, void* out, int64_t B,
                int64_t L, int64_t V, int64_t P, int64_t H, float p, uint64_t seed,
                int dtype, void* stream) {
  if (!ids || !wte || !wpe || !out || B <= 0 || L <= 0 || V <= 0 || P <= 0 || H <= 0 ||
      !dtype_ok(dtype)) {
    set_error("embed: invalid argument");
    return GPTMI_ERR_INVALID;
  }
  if (L > P) {
    set_error("embed: sequence length %lld exceeds the %lld position rows", (long long)L,
              (long long)P);
    return GPTMI_ERR_INVALID;
  }
  if (H > (1 << 24)) {
    set_error("embed: H=%lld too large", (long long)H);
    return GPTMI_ERR_UNSUPPORTED;
  }
  if (!dropout_ok(p)) {
    set_error("embed: dropout probability %g outside [0, 1)", (double)p);
    return GPTMI_ERR_INVALID;
  }
  launch_embed(ids, wte, wpe, out, B * L, L, V, (int)H, Dropout{p, seed}, dtype == GPTMI_F16,
               (hipStream_t)stream);
  return check_launch("embed");
}

int gptmi_embed_layernorm(const int64_t* ids, const void* wte, const void* wpe,
                          const void* ln_w, const void* ln_b, void* emb, void* out, int64_t B,
                          int64_t L, int64_t V, int64_t P, int64_t H, float eps, int dtype,
                          void* stream) {
  if (!ids || !wte || !wpe || !ln_w || !ln_b || !emb || !out || B <= 0 || L <= 0 || V <= 0 ||
      P <= 0 || H <= 0 || !dtype_ok(dtype)) {
    set_error("embed_layernorm: invalid argument");
    return GPTMI_ERR_INVALID;
  }
  if (L > P) {
    set_error("embed_layernorm: sequence length %lld exceeds the %lld position rows",
              (long long)L, (long long)P);
    return GPTMI_ERR_INVALID;
  }
  if (H > 8192) {
    set_error("embed_layernorm: H=%lld beyond the supported 8192", (long long)H);
    return GPTMI_ERR_UNSUPPORTED;
  }
  const bool f16 = dtype == GPTMI_F16;
  hipStream_t st = (hipStream_t)stream;
  if (!launch_embed_layernorm(ids, wte, wpe, ln_w, ln_b, emb, out, B * L, L, V, (int)H, eps, f16,
                              st)) {
    // rows the fused kernel does not hold in registers: the two kernels, same results
    launch_embed(ids, wte, wpe, emb, B * L, L, V, (int)H, Dropout{0.0f, 1337}, f16, st);
    launch_layernorm(emb, ln_w, ln_b, out, B * L, (int)H, eps, f16, st);
  }
  return check_launch("embed_layernorm");
}

int gptmi_layernorm(const void* x, const void* w, const void* b, void* out, int64_t M,
                    int64_t H, float eps, int dtype, void* stream) {
  if (!x || !w || !b || !out || M <= 0 || H <= 0 || !dtype_ok(dtype)) {
    set_error("layernorm: invalid argument");
    return GPTMI_ERR_INVALID;
  }
  if (H > 8192) {
    set_error("layernorm: H=%lld beyond the supported 8192", (long long)H);
    return GPTMI_ERR_UNSUPPORTED;
  }
  launch_layernorm(x, w, b, out, M, (int)H, eps, dtype == GPTMI_F16, (hipStream_t)stream);
  return check_launch("layernorm");
}

int gptmi_softmax(const void* x, void* out, int64_t M, int64_t H, int dtype, void* stream) {
  if (!x || !out || M <= 0 || H <= 0 || !dtype_ok(dtype)) {
    set_error("softmax: invalid argument");
    return GPTMI_ERR_INVALID;
  }
  if (H > 8192) {
    set_error("softmax: H=%lld beyond the supported 8192", (long long)H);
    return GPTMI_ERR_UNSUPPORTED;
  }
  launch_softmax(x, out, M, (int)H, dtype == GPTMI_F16, (hipStream_t)stream);
  return check_launch("softmax");
}

size_t gptmi_linear_workspace_bytes(int64_t M, int64_t N, int64_t K, int dtype, int wlayout) {
  if (M <= 0 || N <= 0 || K <= 0 || !dtype_ok(dtype)) return 0;
  return plan_linear(M, N, K, dtype, wlayout).total;
}

size_t gptmi_packed_weight_bytes(int64_t N, int64_t K) {
  if (N <= 0 || K <= 0) return 0;
  return (size_t)round_up(N * round_up(K, 64) * 2, 256);
}

int gptmi_pack_weight(const void* W, void* packed, int64_t N, int64_t K, int wlayout, int dtype,
                      void* stream) {
  if (!W || !packed || N <= 0 || K <= 0 || !dtype_ok(dtype) ||
      (wlayout != GPTMI_W_KN && wlayout != GPTMI_W_NK) || N > (1 << 30) || K > (1 << 30)) {
    set_error("pack_weight: invalid argument");
    return GPTMI_ERR_INVALID;
  }
  if (((uintptr_t)packed & 255) != 0) {
    set_error("pack_weight: destination must be 256-byte aligned");
    return GPTMI_ERR_INVALID;
  }
  const int Kp = (int)round_up(K, 64);
  if (wlayout == GPTMI_W_KN)
    launch_pack_transpose(W, packed, (int)K, (int)N, Kp, dtype == GPTMI_F16, (hipStream_t)stream);
  else
    launch_pack_rows(W, packed, N, (int)K, Kp, dtype == GPTMI_F16, (hipStream_t)stream);
  return check_launch("pack_weight");
}

int gptmi_linear(const void* x, const void* W, const void* bias, const void* residual,
                 void* out, int64_t M, int64_t N, int64_t K, int gelu, float p,
                 uint64_t seed, int wlayout, void* workspace, size_t workspace_bytes,
                 int dtype, void* stream) {
  const int rc = check_linear_args(x, W, out, M, N, K, p, wlayout, dtype);
  if (rc) return rc;
  return linear_impl(x, W, bias, residual, out, M, N, K, gelu, p, seed, wlayout, workspace,
                     workspace_bytes, dtype, (hipStream_t)stream);
}

size_t gptmi_linear_static_capacity(void) { return GPTMI_STATIC_SCRATCH_BYTES; }

int gptmi_linear_static(const void* x, const void* W, const void* bias, const void* residual,
                        void* out, int64_t M, int64_t N, int64_t K, int gelu, float p,
                        uint64_t seed, int wlayout, int dtype, void* stream) {
  const int rc = check_linear_args(x, W, out, M, N, K, p, wlayout, dtype);
  if (rc) return rc;
  // the size check comes before anything touches the device
  const size_t need = plan_linear(M, N, K, dtype, wlayout).total;
  if (need > (size_t)GPTMI_STATIC_SCRATCH_BYTES) {
    set_error("linear_static: these sizes need %zu bytes of packed operands, the built-in "
              "scratch holds %zu; use gptmi_linear with a workspace, or pack the weight once "
              "(GPTMI_W_PACKED)",
              need, (size_t)GPTMI_STATIC_SCRATCH_BYTES);
    return GPTMI_ERR_WORKSPACE;
  }
  void* ws = nullptr;
  if (need > 0) {
    ws = static_scratch();
    if (ws == nullptr) return GPTMI_ERR_LAUNCH;
  }
  return linear_impl(x, W, bias, residual, out, M, N, K, gelu, p, seed, wlayout, ws,
                     (size_t)GPTMI_STATIC_SCRATCH_BYTES, dtype, (hipStream_t)stream);
}

int gptmi_linear_qkv(const void* x, const void* W, const void* bias, void* q, void* k,
                     void* v, int64_t B, int64_t L, int64_t heads, int64_t d, int64_t K,
                     int wlayout, void* workspace, size_t workspace_bytes, int dtype,
                     void* stream) {
  if (!x || !W || !q || !k || !v || B <= 0 || L <= 0 || heads <= 0 || d <= 0 || K <= 0 ||
      !dtype_ok(dtype) || (wlayout != GPTMI_W_KN && wlayout != GPTMI_W_PACKED)) {
    set_error("linear_qkv: invalid argument");
    return GPTMI_ERR_INVALID;
  }
  if (d % 8 != 0) {
    set_error("linear_qkv: head size %lld must be a multiple of 8", (long long)d);
    return GPTMI_ERR_UNSUPPORTED;
  }
  const int64_t M = B * L, N = 3 * heads * d;
  if (N > kMaxN || K > (1 << 30)) {
    set_error("linear_qkv: N=%lld beyond %d or K=%lld beyond 2^30", (long long)N, kMaxN,
              (long long)K);
    return GPTMI_ERR_UNSUPPORTED;
  }
  hipStream_t st = (hipStream_t)stream;
  const void *A, *Bt;
  int Kp;
  int rc = prepare_operands(x, W, M, N, K, dtype, wlayout, workspace, workspace_bytes, st, &A,
                            &Bt, &Kp);
  if (rc) return rc;
  if (((uintptr_t)A & 15) || ((uintptr_t)Bt & 15)) {
    set_error("linear_qkv: x and W must be 16-byte aligned");
    return GPTMI_ERR_INVALID;
  }
  GemmEpilogue ep = {};
  ep.bias = bias;
  ep.q = q;
  ep.k = k;
  ep.v = v;
  ep.L = L;
  ep.heads = (int)heads;
  ep.d = (int)d;
  ep.qkv = true;
  ep.f16 = dtype == GPTMI_F16;
  rc = launch_gemm(A, Bt, M, (int)N, Kp, ep, st);
  if (rc) return rc;
  return check_launch("linear_qkv");
}

// Shared argument checks of the two LayerNorm-prologue entry points; K = H.
static int check_layernorm_linear(const char* what, const void* x, const void* ln_w,
                                  const void* ln_b, const void* W, int64_t M, int64_t N,
                                  int64_t K, int dtype) {
  if (!x || !ln_w || !ln_b || !W || M <= 0 || N <= 0 || K <= 0 || !dtype_ok(dtype)) {
    set_error("%s: invalid argument", what);
    return GPTMI_ERR_INVALID;
  }
  if (N > kMaxN) {
    set_error("%s: N=%lld beyond %d", what, (long long)N, kMaxN);
    return GPTMI_ERR_UNSUPPORTED;
  }
  if (dtype != GPTMI_F16 || K > (1 << 20) || !gemm_layernorm_supported(M, (int)K)) {
    set_error("%s: fp16 storage and a row width that is a multiple of 64 and fits the LDS panel "
              "(gptmi_layernorm_linear_supported); use gptmi_layernorm + gptmi_linear", what);
    return GPTMI_ERR_UNSUPPORTED;
  }
  return GPTMI_OK;
}

int gptmi_layernorm_linear_supported(int64_t M, int64_t K, int dtype) {
  return dtype == GPTMI_F16 && K > 0 && K <= (1 << 20) && gemm_layernorm_supported(M, (int)K) ? 1 : 0;
}

int gptmi_layernorm_linear(const void* x, const void* ln_w, const void* ln_b, float eps,
                           const void* W_packed, const void* bias, void* out, int64_t M,
                           int64_t N, int64_t K, int gelu, int dtype, void* stream) {
  int rc = check_layernorm_linear("layernorm_linear", x, ln_w, ln_b, W_packed, M, N, K, dtype);
  if (rc) return rc;
  if (!out) {
    set_error("layernorm_linear: invalid argument");
    return GPTMI_ERR_INVALID;
  }
  GemmEpilogue ep = {};
  ep.bias = bias;
  ep.out = out;
  ep.gelu = gelu ? 1 : 0;
  ep.drop = Dropout{0.0f, 1337};
  ep.qkv = false;
  ep.f16 = true;
  rc = launch_gemm_layernorm(x, ln_w, ln_b, eps, W_packed, M, (int)N, (int)K, ep,
                             (hipStream_t)stream);
  if (rc) return rc == -2 ? GPTMI_ERR_INVALID : rc;
  return check_launch("layernorm_linear");
}

int gptmi_layernorm_linear_qkv(const void* x, const void* ln_w, const void* ln_b, float eps,
                               const void* W_packed, const void* bias, void* q, void* k, void* v,
                               int64_t B, int64_t L, int64_t heads, int64_t d, int64_t K,
                               int dtype, void* stream) {
  if (B <= 0 || L <= 0 || heads <= 0 || d <= 0 || !q || !k || !v) {
    set_error("layernorm_linear_qkv: invalid argument");
    return GPTMI_ERR_INVALID;
  }
  if (d % 8 != 0) {
    set_error("layernorm_linear_qkv: head size %lld must be a multiple of 8", (long long)d);
    return GPTMI_ERR_UNSUPPORTED;
  }
  const int64_t M = B * L, N = 3 * heads * d;
  int rc = check_layernorm_linear("layernorm_linear_qkv", x, ln_w, ln_b, W_packed, M, N, K, dtype);
  if (rc) return rc;
  GemmEpilogue ep = {};
  ep.bias = bias;
  ep.q = q;
  ep.k = k;
  ep.v = v;
  ep.L = L;
  ep.heads = (int)heads;
  ep.d = (int)d;
  ep.drop = Dropout{0.0f, 1337};
  ep.qkv = true;
  ep.f16 = true;
  rc = launch_gemm_layernorm(x, ln_w, ln_b, eps, W_packed, M, (int)N, (int)K, ep,
                             (hipStream_t)stream);
  if (rc) return rc == -2 ? GPTMI_ERR_INVALID : rc;
  return check_launch("layernorm_linear_qkv");
}

int gptmi_flash_attn(const void* q, const void* k, const void* v, void* out, int64_t B,
                     int64_t N, int64_t Lq, int64_t Lk, int64_t d, float scale, float p,
                     uint64_t seed, int olayout, int dtype, void* stream) {
  if (!q || !k || !v || !out || B <= 0 || N <= 0 || Lq <= 0 || Lk <= 0 || d <= 0 ||
      !dtype_ok(dtype) || (olayout != GPTMI_O_BNLD && olayout != GPTMI_O_BLND)) {
    set_error("flash_attn: invalid argument");
    return GPTMI_ERR_INVALID;
  }
  if (!dropout_ok(p)) {
    set_error("flash_attn: dropout probability %g outside [0, 1)", (double)p);
    return GPTMI_ERR_INVALID;
  }
  if (((uintptr_t)q & 15) || ((uintptr_t)k & 15) || ((uintptr_t)v & 15) ||
      ((uintptr_t)out & 15)) {
    set_error("flash_attn: q, k, v and out must be 16-byte aligned");
    return GPTMI_ERR_INVALID;
  }
  int rc = launch_flash_attn(q, k, v, out, B, N, Lq, Lk, (int)d, scale, Dropout{p, seed},
                             olayout == GPTMI_O_BLND,
                             dtype == GPTMI_F16, (hipStream_t)stream);
  if (rc) return rc;
  return check_launch("flash_attn");
}

}  // extern "C"
