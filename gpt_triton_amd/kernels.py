"""Operator layer: the five public functions of the reference's kernels.py, with the same
names, argument order, defaults, assertions and return shapes, each handing raw device
pointers to one entry point of libgptmi.so (include/gptmi.h).

    fused_embeddings(x, wte, wpe, dropout_prob=0.0)              kernels.py:75-101
    fused_layer_norm(x, weight, bias)                            kernels.py:148-164
    fused_ffn(x, weight, bias=None, residual=None,
              add_gelu=False, dropout_prob=0.0)                  kernels.py:260-315
    matmul_and_split_qkv(x, weight, bias, num_heads)             kernels.py:347-367
    flash_attention_v1(q, k, v, dropout_prob=0.0)                kernels.py:477-525

plus `fused_embeddings_layer_norm` (the embedding gather and the first block's LayerNorm in one
kernel, the fusion the reference's author notes as a TODO, kernels.py:132-133), `fused_softmax(x)` (the reference only sketches a row softmax, kernels.py:318-342),
`lm_head(x, wte)` (the transposed-weight product the reference leaves as a TODO,
gpt.py:159-161) and `pack_weight(weight)`: the GEMM reads its weight as an fp16,
K-contiguous image which `fused_ffn` / `matmul_and_split_qkv` otherwise rebuild on every
call; a `PackedWeight` may be passed wherever they take `weight`.  Tensors must live on the
GPU: there is no CPU path.  dropout_prob > 0 reproduces the reference's masks: Philox-4x32-10
(Triton's tl.rand) with the kernels' default seed 1337 and the reference's offsets -- the column
for the embedding, the flat index m*N + n for fused_ffn, query*Lk + key for the attention
weights (kernels.py:31-34, 65-70, 245-251, 457-460).
"""
import math
import os

import torch

from . import _lib

_DTYPES = {torch.float32: _lib.GPTMI_F32, torch.float16: _lib.GPTMI_F16}


def _dtype_code(t, what):
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise TypeError(f"{what}: dtype {t.dtype} is not supported (float32 and float16 are)")


def _on_gpu(*tensors):
    dev = tensors[0].device
    if dev.type != "cuda":
        raise RuntimeError("gpt_triton_amd operators run on the GPU only; got a tensor on "
                           f"{dev} (there is no CPU fallback)")
    for t in tensors[1:]:
        if t is not None and t.device != dev:
            raise RuntimeError(f"tensors on different devices: {dev} and {t.device}")
    return dev


def _stream():
    # torch's current stream on the current device as the raw hipStream_t; the direct binding
    # costs a fraction of building a torch.cuda.Stream object per operator call
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def _device(dev):
    """Context in which `dev` is the current device: nothing to do (and nothing to pay per call)
    when it already is, torch's guard otherwise."""
    if dev.index is None or dev.index == torch._C._cuda_getDevice():
        return _NO_GUARD
    return torch.cuda.device(dev)


def _ptr(t):
    return None if t is None else t.data_ptr()


def _workspace(nbytes, device):
    if nbytes == 0:
        return None
    return torch.empty(nbytes, dtype=torch.uint8, device=device)


class PackedWeight:
    """The fp16 [N][round_up(K, 64)] image of a [K, N] weight (see gptmi_pack_weight).  `shape`
    and `dtype` are those of the weight it was made from, so it can stand in for it."""

    __slots__ = ("data", "shape", "dtype", "device", "vocab")

    def __init__(self, data, shape, dtype, vocab=None):
        self.data, self.shape, self.dtype, self.device = data, tuple(shape), dtype, data.device
        self.vocab = vocab  # pack_lm_head: rows of wte before the zero padding

    def is_contiguous(self):
        return True

    def data_ptr(self):
        return self.data.data_ptr()


@torch.no_grad()
def pack_weight(weight):
    """Packs a contiguous [K, N] weight once; the result replaces `weight` in `fused_ffn` and
    `matmul_and_split_qkv` and must be rebuilt when the weight changes."""
    assert weight.dim() == 2 and weight.is_contiguous()
    dev = _on_gpu(weight)
    K_, N = weight.shape
    lib = _lib.load()
    buf = torch.empty(lib.gptmi_packed_weight_bytes(N, K_), dtype=torch.uint8, device=dev)
    with _device(dev):
        rc = lib.gptmi_pack_weight(weight.data_ptr(), buf.data_ptr(), N, K_, _lib.GPTMI_W_KN,
                                   _dtype_code(weight, "pack_weight"), _stream())
    _lib.check(rc, "pack_weight")
    return PackedWeight(buf, weight.shape, weight.dtype)


@torch.no_grad()
def pack_lm_head(wte):
    """Packs wte [V, H] once for `lm_head`, with the vocabulary padded to a multiple of 64 by zero
    rows.  GPT-2's V = 50257 is odd: rows of a dense [T, V] fp16 matrix then start on 2-byte
    boundaries and every logit is stored on its own.  With the padded image the GEMM writes
    [T, Vp] rows of whole 128-byte lines -- the shape the persistent GEMM kernel takes -- and
    `lm_head` returns the [.., :V] view of it."""
    assert wte.dim() == 2 and wte.is_contiguous()
    dev = _on_gpu(wte)
    V, H = wte.shape
    Vp = -(-V // 64) * 64
    lib = _lib.load()
    buf = torch.zeros(lib.gptmi_packed_weight_bytes(Vp, H), dtype=torch.uint8, device=dev)
    with _device(dev):
        rc = lib.gptmi_pack_weight(wte.data_ptr(), buf.data_ptr(), V, H, _lib.GPTMI_W_NK,
                                   _dtype_code(wte, "pack_lm_head"), _stream())
    _lib.check(rc, "pack_lm_head")
    return PackedWeight(buf, (H, Vp), wte.dtype, vocab=V)


def check_token_ids(x, vocab_size):
    """Raises IndexError if a token id lies outside [0, vocab_size).  The embedding kernels
    themselves read no memory for such an id and use a zero wte row (the reference reads out of
    bounds); this check costs a device synchronisation, so the operators run it only when the
    environment variable GPTMI_CHECK_IDS is set to 1."""
    lo, hi = int(x.min()), int(x.max())
    if lo < 0 or hi >= vocab_size:
        raise IndexError(f"token ids span [{lo}, {hi}] but the vocabulary has {vocab_size} rows")


def _maybe_check_ids(x, vocab_size):
    if os.environ.get("GPTMI_CHECK_IDS") == "1" and x.numel() > 0:
        check_token_ids(x, vocab_size)


def _wlayout(weight, default):
    return _lib.GPTMI_W_PACKED if isinstance(weight, PackedWeight) else default


@torch.no_grad()
def fused_embeddings(x, wte, wpe, dropout_prob=0.0):
    """dropout(wte[x] + wpe[position]) for token ids x [B, L] -> [B, L, H] in wte's dtype."""
    assert wte.shape[1] == wpe.shape[1]
    assert x.is_contiguous()
    assert wte.is_contiguous()
    assert wpe.is_contiguous()
    B, L = x.shape
    V, H = wte.shape
    P = wpe.shape[0]
    if x.dtype != torch.int64:
        raise TypeError(f"fused_embeddings: token ids must be int64, got {x.dtype}")
    if wte.dtype != wpe.dtype:
        raise TypeError("fused_embeddings: wte and wpe must share a dtype")
    dev = _on_gpu(x, wte, wpe)
    _maybe_check_ids(x, V)
    z = torch.empty((B * L, H), device=dev, dtype=wte.dtype)
    lib = _lib.load()
    with _device(dev):
        rc = lib.gptmi_embed(x.data_ptr(), wte.data_ptr(), wpe.data_ptr(), z.data_ptr(), B, L, V,
                             P, H, float(dropout_prob), 1337, _dtype_code(wte, "fused_embeddings"),
                             _stream())
    _lib.check(rc, "fused_embeddings")
    return z.view((B, L, H))


@torch.no_grad()
def fused_embeddings_layer_norm(x, wte, wpe, weight, bias):
    """(fused_embeddings(x, wte, wpe), fused_layer_norm(of that, weight, bias)) from one kernel:
    the embedding row is normalised while it is still in registers.  Both results are
    bit-identical to the two separate calls.  No dropout (eval-mode forward)."""
    assert wte.shape[1] == wpe.shape[1]
    assert x.is_contiguous()
    assert wte.is_contiguous()
    assert wpe.is_contiguous()
    assert weight.is_contiguous()
    assert bias.is_contiguous()
    assert weight.shape == bias.shape
    assert wte.shape[1] == weight.shape[0]
    B, L = x.shape
    V, H = wte.shape
    P = wpe.shape[0]
    if x.dtype != torch.int64:
        raise TypeError(f"fused_embeddings_layer_norm: token ids must be int64, got {x.dtype}")
    if not (wte.dtype == wpe.dtype == weight.dtype == bias.dtype):
        raise TypeError("fused_embeddings_layer_norm: wte, wpe, weight and bias must share a dtype")
    dev = _on_gpu(x, wte, wpe, weight, bias)
    _maybe_check_ids(x, V)
    emb = torch.empty((B * L, H), device=dev, dtype=wte.dtype)
    out = torch.empty((B * L, H), device=dev, dtype=wte.dtype)
    lib = _lib.load()
    with _device(dev):
        rc = lib.gptmi_embed_layernorm(x.data_ptr(), wte.data_ptr(), wpe.data_ptr(),
                                       weight.data_ptr(), bias.data_ptr(), emb.data_ptr(),
                                       out.data_ptr(), B, L, V, P, H, 1e-5,
                                       _dtype_code(wte, "fused_embeddings_layer_norm"), _stream())
    _lib.check(rc, "fused_embeddings_layer_norm")
    return emb.view((B, L, H)), out.view((B, L, H))


@torch.no_grad()
def fused_layer_norm(x, weight, bias):
    """LayerNorm over the last dim (eps = 1e-5, biased variance), same shape and dtype as x."""
    assert x.is_contiguous()
    assert weight.is_contiguous()
    assert bias.is_contiguous()
    assert weight.shape == bias.shape
    assert x.shape[-1] == weight.shape[0]
    if not (x.dtype == weight.dtype == bias.dtype):
        raise TypeError("fused_layer_norm: x, weight and bias must share a dtype")
    dev = _on_gpu(x, weight, bias)
    H = x.shape[-1]
    M = x.numel() // H
    z = torch.empty(x.shape, device=dev, dtype=x.dtype)
    lib = _lib.load()
    with _device(dev):
        rc = lib.gptmi_layernorm(x.data_ptr(), weight.data_ptr(), bias.data_ptr(), z.data_ptr(), M,
                                 H, 1e-5, _dtype_code(x, "fused_layer_norm"), _stream())
    _lib.check(rc, "fused_layer_norm")
    return z


@torch.no_grad()
def fused_softmax(x):
    """softmax over the last dim with fp32 statistics, same shape and dtype as x."""
    assert x.is_contiguous()
    dev = _on_gpu(x)
    H = x.shape[-1]
    M = x.numel() // H
    z = torch.empty(x.shape, device=dev, dtype=x.dtype)
    lib = _lib.load()
    with _device(dev):
        rc = lib.gptmi_softmax(x.data_ptr(), z.data_ptr(), M, H, _dtype_code(x, "fused_softmax"),
                               _stream())
    _lib.check(rc, "fused_softmax")
    return z


def _linear(x2d, weight, bias, residual, z, gelu, dropout_prob, wlayout, what):
    M, K = x2d.shape
    N = z.shape[1]
    dev = x2d.device
    code = _dtype_code(x2d, what)
    for name, t in (("weight", weight), ("bias", bias), ("residual", residual)):
        if t is not None and t.dtype != x2d.dtype:
            raise TypeError(f"{what}: {name} is {t.dtype} but x is {x2d.dtype}")
    lib = _lib.load()
    ws_bytes = lib.gptmi_linear_workspace_bytes(M, N, K, code, wlayout)
    ws = _workspace(ws_bytes, dev)
    with _device(dev):
        rc = lib.gptmi_linear(x2d.data_ptr(), weight.data_ptr(), _ptr(bias), _ptr(residual),
                              z.data_ptr(), M, N, K, int(bool(gelu)), float(dropout_prob), 1337,
                              wlayout, _ptr(ws), ws_bytes, code, _stream())
    _lib.check(rc, what)
    return z


@torch.no_grad()
def fused_ffn(x, weight, bias=None, residual=None, add_gelu=False, dropout_prob=0.0):
    """dropout(gelu?(x @ weight + bias)) + residual; weight is [K, N] (in x out)."""
    out_shape_0 = x.shape[:-1]
    x = x.view((-1, x.shape[-1]))
    M, K = x.shape
    N = weight.shape[1]
    dev = _on_gpu(x, weight, bias, residual)
    z = torch.empty((M, N), device=dev, dtype=x.dtype)

    assert x.is_contiguous()
    assert weight.is_contiguous()
    assert x.shape[1] == weight.shape[0]
    if bias is not None:
        assert bias.is_contiguous()
        assert weight.shape[1] == bias.shape[0]
    if residual is not None:
        residual = residual.view(z.shape)
        assert residual.is_contiguous()

    _linear(x, weight, bias, residual, z, add_gelu, dropout_prob,
            _wlayout(weight, _lib.GPTMI_W_KN), "fused_ffn")
    return z.view((*out_shape_0, N))


@torch.no_grad()
def lm_head(x, wte):
    """x @ wte^T: logits [*, V].  `wte` is the [V, H] embedding matrix itself (read in place, no
    transposed copy; the result is contiguous) or its `pack_lm_head` image (the result is then
    the [*, :V] view of a buffer whose rows are padded to a multiple of 64 logits)."""
    out_shape_0 = x.shape[:-1]
    x = x.view((-1, x.shape[-1]))
    assert x.is_contiguous()
    assert wte.is_contiguous()
    if isinstance(wte, PackedWeight):
        assert wte.vocab is not None and x.shape[1] == wte.shape[0]
        dev = _on_gpu(x, wte)
        z = torch.empty((x.shape[0], wte.shape[1]), device=dev, dtype=x.dtype)
        _linear(x, wte, None, None, z, False, 0.0, _lib.GPTMI_W_PACKED, "lm_head")
        return z.view((*out_shape_0, wte.shape[1]))[..., :wte.vocab]
    assert x.shape[1] == wte.shape[1]
    dev = _on_gpu(x, wte)
    z = torch.empty((x.shape[0], wte.shape[0]), device=dev, dtype=x.dtype)
    _linear(x, wte, None, None, z, False, 0.0, _lib.GPTMI_W_NK, "lm_head")
    return z.view((*out_shape_0, wte.shape[0]))


@torch.no_grad()
def matmul_and_split_qkv(x, weight, bias, num_heads):
    """x [B, L, h] @ weight [h, 3h] + bias, returned as q, k, v [B, num_heads, L, h/num_heads],
    each contiguous; the GEMM's store does the head split."""
    batch_size, seqlen, _ = x.shape
    assert x.is_contiguous()
    assert weight.is_contiguous()
    assert x.shape[2] == weight.shape[0]
    hidden_size = weight.shape[1]
    assert hidden_size % 3 == 0, hidden_size
    hidden_size = hidden_size // 3
    assert hidden_size % num_heads == 0, (hidden_size, num_heads)
    head_size = hidden_size // num_heads
    if bias is not None:
        assert bias.is_contiguous()
        assert weight.shape[1] == bias.shape[0]
    dev = _on_gpu(x, weight, bias)
    code = _dtype_code(x, "matmul_and_split_qkv")
    if weight.dtype != x.dtype or (bias is not None and bias.dtype != x.dtype):
        raise TypeError("matmul_and_split_qkv: x, weight and bias must share a dtype")
    if head_size % 8 != 0 and isinstance(weight, PackedWeight):
        raise NotImplementedError("matmul_and_split_qkv: packed weights need head_size % 8 == 0")
    if head_size % 8 != 0:
        # the scatter epilogue stores 8-element groups; other head sizes take the plain GEMM
        y = fused_ffn(x, weight, bias=bias)
        q, k, v = y.split(hidden_size, dim=2)
        return tuple(t.view(batch_size, seqlen, num_heads, head_size).transpose(1, 2).contiguous()
                     for t in (q, k, v))
    shape = (batch_size, num_heads, seqlen, head_size)
    q = torch.empty(shape, device=dev, dtype=x.dtype)
    k = torch.empty(shape, device=dev, dtype=x.dtype)
    v = torch.empty(shape, device=dev, dtype=x.dtype)
    lib = _lib.load()
    M, K, N = batch_size * seqlen, x.shape[2], 3 * hidden_size
    wl = _wlayout(weight, _lib.GPTMI_W_KN)
    ws_bytes = lib.gptmi_linear_workspace_bytes(M, N, K, code, wl)
    ws = _workspace(ws_bytes, dev)
    with _device(dev):
        rc = lib.gptmi_linear_qkv(x.data_ptr(), weight.data_ptr(), _ptr(bias), q.data_ptr(),
                                  k.data_ptr(), v.data_ptr(), batch_size, seqlen, num_heads,
                                  head_size, K, wl, _ptr(ws), ws_bytes, code, _stream())
    _lib.check(rc, "matmul_and_split_qkv")
    return q, k, v


def layer_norm_linear_supported(x, weight):
    """True where `layer_norm_ffn` / `layer_norm_matmul_and_split_qkv` take these operands: fp16,
    a packed weight image, a row width the kernel's LDS panel holds."""
    if not isinstance(weight, PackedWeight) or x.dtype != torch.float16:
        return False
    H = x.shape[-1]
    return bool(_lib.load().gptmi_layernorm_linear_supported(x.numel() // H, H, _lib.GPTMI_F16))


def _check_layer_norm_linear(x, ln_weight, ln_bias, weight, bias, what):
    assert x.is_contiguous() and ln_weight.is_contiguous() and ln_bias.is_contiguous()
    assert ln_weight.shape == ln_bias.shape == (x.shape[-1],)
    assert x.shape[-1] == weight.shape[0]
    if not isinstance(weight, PackedWeight):
        raise NotImplementedError(f"{what}: takes the packed image of the weight (pack_weight)")
    if not (x.dtype == ln_weight.dtype == ln_bias.dtype == weight.dtype == torch.float16):
        raise NotImplementedError(f"{what}: fp16 operands only")
    if bias is not None:
        assert bias.is_contiguous() and bias.shape == (weight.shape[1],)
        if bias.dtype != x.dtype:
            raise TypeError(f"{what}: bias is {bias.dtype} but x is {x.dtype}")
    return _on_gpu(x, ln_weight, ln_bias, weight, bias)


@torch.no_grad()
def layer_norm_ffn(x, ln_weight, ln_bias, weight, bias=None, add_gelu=False):
    """gelu?(fused_layer_norm(x, ln_weight, ln_bias) @ weight + bias) in one launch: the
    LayerNorm runs in the GEMM's operand prologue (the fusion marked as to do in the reference,
    kernels.py:132-133) and gives the bits of fused_layer_norm followed by fused_ffn.  Meant for
    few rows; `weight` is a `pack_weight` image, fp16 only (NotImplementedError otherwise, and
    for row widths `layer_norm_linear_supported` turns down)."""
    dev = _check_layer_norm_linear(x, ln_weight, ln_bias, weight, bias, "layer_norm_ffn")
    K, N = weight.shape
    M = x.numel() // K
    z = torch.empty((*x.shape[:-1], N), device=dev, dtype=x.dtype)
    lib = _lib.load()
    with _device(dev):
        rc = lib.gptmi_layernorm_linear(x.data_ptr(), ln_weight.data_ptr(), ln_bias.data_ptr(),
                                        1e-5, weight.data_ptr(), _ptr(bias), z.data_ptr(), M, N, K,
                                        int(bool(add_gelu)), _lib.GPTMI_F16, _stream())
    _lib.check(rc, "layer_norm_ffn")
    return z


@torch.no_grad()
def layer_norm_matmul_and_split_qkv(x, ln_weight, ln_bias, weight, bias, num_heads):
    """matmul_and_split_qkv(fused_layer_norm(x, ln_weight, ln_bias), weight, bias, num_heads) in
    one launch, same bits; see `layer_norm_ffn`.  x [B, L, h]; head size a multiple of 8."""
    dev = _check_layer_norm_linear(x, ln_weight, ln_bias, weight, bias,
                                   "layer_norm_matmul_and_split_qkv")
    batch_size, seqlen, K = x.shape
    hidden_size = weight.shape[1] // 3
    assert weight.shape[1] == 3 * hidden_size and hidden_size % num_heads == 0
    head_size = hidden_size // num_heads
    shape = (batch_size, num_heads, seqlen, head_size)
    q = torch.empty(shape, device=dev, dtype=x.dtype)
    k = torch.empty(shape, device=dev, dtype=x.dtype)
    v = torch.empty(shape, device=dev, dtype=x.dtype)
    lib = _lib.load()
    with _device(dev):
        rc = lib.gptmi_layernorm_linear_qkv(x.data_ptr(), ln_weight.data_ptr(), ln_bias.data_ptr(),
                                            1e-5, weight.data_ptr(), _ptr(bias), q.data_ptr(),
                                            k.data_ptr(), v.data_ptr(), batch_size, seqlen,
                                            num_heads, head_size, K, _lib.GPTMI_F16, _stream())
    _lib.check(rc, "layer_norm_matmul_and_split_qkv")
    return q, k, v


@torch.no_grad()
def flash_attention_v1(q, k, v, dropout_prob=0.0, *, merged_heads_layout=False):
    """Causal softmax(q k^T / sqrt(d)) v for q, k, v [B, N, L, d] -> [B, N, L, d].

    merged_heads_layout=True (an extension; the default is the reference's behaviour)
    returns the same values as a [B, N, L, d]-shaped view of a [B, L, N, d] buffer, so the
    caller's `.transpose(1, 2).contiguous()` head merge costs no copy.
    """
    assert q.shape[:2] == k.shape[:2]
    assert q.shape[-1] == k.shape[-1]
    assert k.shape == v.shape
    B, N, Lq, H = q.shape
    Lk = k.shape[2]
    assert H in {16, 32, 64, 128, 256}
    assert q.is_contiguous()
    assert k.is_contiguous()
    assert v.is_contiguous()
    if not (q.dtype == k.dtype == v.dtype):
        raise TypeError("flash_attention_v1: q, k and v must share a dtype")
    dev = _on_gpu(q, k, v)
    code = _dtype_code(q, "flash_attention_v1")
    scale = 1 / math.sqrt(H)
    return _flash(q, k, v, scale, dropout_prob, merged_heads_layout, dev, code)


def _flash(q, k, v, scale, dropout_prob, merged_heads_layout, dev, code):
    B, N, Lq, H = q.shape
    Lk = k.shape[2]
    if merged_heads_layout:
        buf = torch.empty((B, Lq, N, H), device=dev, dtype=q.dtype)
        layout = _lib.GPTMI_O_BLND
    else:
        buf = torch.empty((B, N, Lq, H), device=dev, dtype=q.dtype)
        layout = _lib.GPTMI_O_BNLD
    lib = _lib.load()
    with _device(dev):
        rc = lib.gptmi_flash_attn(q.data_ptr(), k.data_ptr(), v.data_ptr(), buf.data_ptr(), B, N,
                                  Lq, Lk, H, scale, float(dropout_prob), 1337, layout, code,
                                  _stream())
    _lib.check(rc, "flash_attention_v1")
    return buf.transpose(1, 2) if merged_heads_layout else buf
