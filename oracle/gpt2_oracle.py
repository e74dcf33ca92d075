"""CPU restatement of the reference's GPT-2 forward hot path (numpy).

THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests/, the smoke check
and the cpu_baseline leg of bench.py may import it; nothing under
gpt_triton_amd/ does, and the GPU path never falls back to it.

Every function restates one operator of thevasudevgupta/gpt-triton with the
rounding points of its Triton kernels (which, under the reference's CPU
interpreter, are numpy operations: tl.dot(a, b, acc) = matmul of the fp16
operands in fp32 plus acc, casts = ndarray.astype, exp = np.exp):

  fused_embeddings      kernels.py:37-101
  fused_layer_norm      kernels.py:104-164
  gelu_new / tanh       kernels.py:15-26
  fused_ffn             kernels.py:169-315
  matmul_and_split_qkv  kernels.py:347-367
  flash_attention_v1    kernels.py:375-525
  softmax_rows          (dead sketch kernels.py:318-342; contract = softmax(x.float(), -1))
  dropout / tl_rand     kernels.py:31-34 over Triton's tl.rand (triton/language/random.py:
                        Philox-4x32-10, counter (offset,0,0,0), key = 64-bit seed, first word)
  gpt2_forward          gpt.py:38-60, 90-111, 163-180 (+ optional tied LM head,
                        the intent commented at gpt.py:159-161, 172-179)

What pins each function (tests/test_oracle.py):
  embeddings   closed form wte[x] + wpe[arange(L)] (test.py:41), bit exact
  layer norm   torch.nn.functional.layer_norm in fp64 (test.py:55-57)
  gelu         torch gelu(approximate="tanh") in fp64
  ffn          fp64 product of the fp16-rounded operands, no-bias / no-GELU /
               residual special cases (test.py:62-69)
  split        index identity q[b,n,l,:] == y[b,l,n*d:(n+1)*d] (kernels.py:355-365)
  attention    textbook causal softmax attention in fp64 on fp16-rounded q,k,v
               (test.py:98-106), row 0 == v[0], convex-combination bounds,
               single-tile case L <= 64, tile-size independence up to P rounding, and
               tests/golden/flash_attention_v1.npz: outputs of the reference's own
               flash_attention_v1 under Triton's CPU interpreter (bit-identical on
               > 95 % of the elements, <= 2e-7 relative on the rest)
  softmax      torch.softmax in fp64
  dropout      Philox-4x32-10 against the three known-answer vectors of the Random123
               distribution (counter/key all zero, all ones, digits of pi), the uniform map
               against its closed form on the int32 edge values, the keep rate against p, and
               tests/golden/dropout.npz: outputs of the reference's fused_embeddings, fused_ffn
               and flash_attention_v1 with dropout_prob > 0 under Triton's CPU interpreter
  fp32 chain   accumulation_dtype(np.float64) re-evaluates the same formulas with fp64 sums at
               the same rounding points; tests/test_oracle.py measures how far that moves the
               fp32-storage model output (the bound the GPU tests derive their tolerance from)
  model        an independently written fp64 torch GPT-2 (HF block order), and the
               transformers library's GPT2Model (random weights, built locally from a
               config) through the package's key conversion (test.py:120-133)
No function of this file is left unpinned.
"""
import contextlib
import math

import numpy as np

F32 = np.float32  # the arithmetic type between rounding points; see accumulation_dtype
F16 = np.float16
BLOCK_L = 64  # K/V tile of the reference's attention kernel (kernels.py:509)


@contextlib.contextmanager
def accumulation_dtype(dtype):
    """Inside the block every function of this file does its sums, products, exponentials and
    normalisations in `dtype` (np.float64) instead of fp32, while every rounding point of the
    reference stays where it is: operands still go through fp16, results are still stored in
    the tensors' own dtype.  The distance between the two evaluations is the part of a result
    that depends on nothing but the order and precision of fp32 accumulation -- the floor below
    which two correct implementations of the reference's formulas cannot be told apart."""
    global F32
    saved, F32 = F32, dtype
    try:
        yield
    finally:
        F32 = saved


def _as_f32(a):
    return np.asarray(a).astype(F32, copy=False)


def round_to_f16(a):
    """fp32 -> fp16 (round to nearest even) -> fp32, the `.to(tl.float16)` of the kernels."""
    return np.asarray(a).astype(F16).astype(F32)


U32 = np.uint32
SEED = 1337  # the default of every kernel's `seed` argument (kernels.py:49,181,387)


def philox4x32_10(c0, c1, c2, c3, k0, k1):
    """Ten rounds of Philox-4x32 (triton/language/random.py:13-43); uint32 arrays in and out."""
    c0, c1, c2, c3 = (np.asarray(c, dtype=U32).copy() for c in (c0, c1, c2, c3))
    k0, k1 = int(k0) & 0xFFFFFFFF, int(k1) & 0xFFFFFFFF
    A, B = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
    for _ in range(10):
        pa = A * c0.astype(np.uint64)  # 64-bit products: hi word = umulhi, lo word = mul
        pb = B * c2.astype(np.uint64)
        n0 = (pb >> np.uint64(32)).astype(U32) ^ c1 ^ U32(k0)
        n2 = (pa >> np.uint64(32)).astype(U32) ^ c3 ^ U32(k1)
        c1 = (pb & np.uint64(0xFFFFFFFF)).astype(U32)
        c3 = (pa & np.uint64(0xFFFFFFFF)).astype(U32)
        c0, c2 = n0, n2
        k0 = (k0 + 0x9E3779B9) & 0xFFFFFFFF
        k1 = (k1 + 0xBB67AE85) & 0xFFFFFFFF
    return c0, c1, c2, c3


def uint_to_uniform_float(x):
    """triton/language/random.py:88-105: the word as int32, negatives folded by -x-1, times
    4.6566127342e-10 in fp32 -> [0, 1)."""
    xi = np.asarray(x, dtype=U32).view(np.int32)
    xi = np.where(xi < 0, -xi - 1, xi)
    return xi.astype(F32) * F32(4.6566127342e-10)


def tl_rand(seed, offset):
    """tl.rand(seed, offset) for 32-bit offsets (random.py:46-69,108-117)."""
    off = np.asarray(offset).astype(np.int64).astype(U32)  # int32 offsets reinterpreted
    zero = np.zeros_like(off)
    c0, _, _, _ = philox4x32_10(off, zero, zero, zero, seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF)
    return uint_to_uniform_float(c0)


def dropout(x, p, seed, offset):
    """kernels.py:31-34: keep where rand > p, scaled by a true division by (1 - p); the
    arithmetic is fp32 (p is an fp32 scalar on the device)."""
    keep = tl_rand(seed, offset) > F32(p)
    return np.where(keep, _as_f32(x) / (F32(1.0) - F32(p)), F32(0.0)).astype(F32)


def fused_embeddings(ids, wte, wpe, dropout_prob=0.0, seed=SEED):
    """kernels.py:58-70: one add in the storage dtype, then dropout -- applied even at p = 0
    (kernels.py:70), with the COLUMN index as the only offset (kernels.py:65), so the mask is
    the same for every token.  At p = 0 a column would be zeroed only if its rand were exactly
    0; the tests check that no column below 2^20 has that for the default seed."""
    ids = np.asarray(ids)
    B, L = ids.shape
    assert wte.shape[1] == wpe.shape[1] and wte.dtype == wpe.dtype
    pos = np.arange(B * L) % L  # kernels.py:61 -- position = pid % L
    rows = wte[ids.reshape(-1)] + wpe[pos]  # numpy adds fp16 + fp16 with one rounding
    rows = rows.astype(wte.dtype, copy=False)
    if dropout_prob != 0.0:
        rows = dropout(rows, dropout_prob, seed, np.arange(wte.shape[1])[None, :])
    return rows.reshape(B, L, wte.shape[1]).astype(wte.dtype, copy=False)


def fused_layer_norm(x, weight, bias, eps=1e-5):
    """kernels.py:115-145: fp32 mean, fp32 centred biased variance, 1/sqrt(var+eps)."""
    out_dtype = x.dtype
    H = x.shape[-1]
    xf = _as_f32(x).reshape(-1, H)
    mean = xf.sum(axis=1, dtype=F32, keepdims=True) / F32(H)
    cen = xf - mean
    var = (cen * cen).sum(axis=1, dtype=F32, keepdims=True) / F32(H)
    rstd = F32(1.0) / np.sqrt(var + F32(eps))
    z = cen * rstd
    z = z * _as_f32(weight) + _as_f32(bias)
    return z.astype(out_dtype).reshape(x.shape)


def gelu_new(x):
    """kernels.py:15-26 in fp32: tanh(u) = 2*sigmoid(2u) - 1."""
    x = _as_f32(x)
    a = F32(math.sqrt(2.0 / math.pi))
    b = x + F32(0.044715) * x * x * x
    u = a * b
    with np.errstate(over="ignore"):
        sig = F32(1.0) / (F32(1.0) + np.exp(-(F32(2.0) * u)))
    t = F32(2.0) * sig - F32(1.0)
    return F32(0.5) * x * (F32(1.0) + t)


def fused_ffn(x, weight, bias=None, residual=None, add_gelu=False, dropout_prob=0.0, seed=SEED):
    """kernels.py:224-257: fp16 operands, fp32 accumulate, bias -> GELU -> dropout (only if
    p > 0, offset = flat index m*N + n in int32, kernels.py:245-251) -> residual -> cast."""
    out_dtype = x.dtype
    K = x.shape[-1]
    N = weight.shape[1]
    assert weight.shape[0] == K
    xa = round_to_f16(x).reshape(-1, K)
    wa = round_to_f16(weight)
    z = np.matmul(xa, wa, dtype=F32)
    if bias is not None:
        z = z + _as_f32(bias)
    if add_gelu:
        z = gelu_new(z)
    if dropout_prob > 0.0:
        M = z.shape[0]
        flat = (np.arange(M, dtype=np.int64)[:, None] * N + np.arange(N, dtype=np.int64)[None, :])
        z = dropout(z, dropout_prob, seed, flat & 0xFFFFFFFF)
    if residual is not None:
        z = z + _as_f32(residual).reshape(z.shape)
    return z.astype(out_dtype).reshape(*x.shape[:-1], N)


def matmul_and_split_qkv(x, weight, bias, num_heads):
    """kernels.py:350-367: GEMM, split the last dim in three, [B,L,N,d] -> [B,N,L,d]."""
    y = fused_ffn(x, weight, bias=bias)
    B, L, H3 = y.shape
    assert H3 % 3 == 0
    h = H3 // 3
    assert h % num_heads == 0
    d = h // num_heads
    parts = []
    for i in range(3):
        t = y[:, :, i * h:(i + 1) * h].reshape(B, L, num_heads, d)
        parts.append(np.ascontiguousarray(t.transpose(0, 2, 1, 3)))
    return tuple(parts)


def flash_attention_v1(q, k, v, block=BLOCK_L, dropout_prob=0.0, seed=SEED):
    """kernels.py:408-474.  Dropout (p > 0 only) hits P after the denominator has
    summed it and before the fp16 rounding, offset = lq * Lk + lk for every batch and head
    (kernels.py:457-460).

    Per query row: key tiles of `block` in ascending order; S = (q16 . k16^T) * scale in
    fp32; causal mask; running max m; P = exp(S - m_new); den = den * exp(m - m_new) +
    sum(P) with P unrounded; acc = acc * exp(m - m_new) + fp16(P) . v16 in fp32;
    out = acc / den.

    Lq != Lk (q [B, N, Lq, D]; k, v [B, N, Lk, D]) as the reference has it: the mask is
    `query >= key` alone (kernels.py:436) and the last key tile is filled up with zero rows
    (kernels.py:421-424, 462), so a query at or past Lk also attends to that padding (score 0,
    value 0); keys past the last query are never visible.  With Lq == Lk no valid query sees a
    padding row, and the tile may end at Lk.
    """
    out_dtype = q.dtype
    B, N, Lq, D = q.shape
    Lk = k.shape[2]
    assert k.shape == (B, N, Lk, D) and v.shape == k.shape
    scale = F32(1.0 / math.sqrt(D))  # a Python float in the reference, fp32 on the device
    Lkp = Lk if Lq <= Lk else -(-Lk // block) * block  # zero rows that a query can see
    q16 = round_to_f16(q).reshape(B * N, Lq, D)
    k16 = np.zeros((B * N, Lkp, D), dtype=F32)
    v16 = np.zeros((B * N, Lkp, D), dtype=F32)
    k16[:, :Lk] = round_to_f16(k).reshape(B * N, Lk, D)
    v16[:, :Lk] = round_to_f16(v).reshape(B * N, Lk, D)
    acc = np.zeros((B * N, Lq, D), dtype=F32)
    mrun = np.full((B * N, Lq, 1), -np.inf, dtype=F32)
    den = np.zeros((B * N, Lq, 1), dtype=F32)
    rows = np.arange(Lq)[:, None]
    for k0 in range(0, Lkp, block):
        k1 = min(k0 + block, Lkp)
        cols = np.arange(k0, k1)[None, :]
        s = np.matmul(q16, k16[:, k0:k1].transpose(0, 2, 1), dtype=F32) * scale
        s = np.where(rows >= cols, s, F32(-np.inf))
        bmax = s.max(axis=2, keepdims=True)
        mnew = np.where(bmax > mrun, bmax, mrun)
        with np.errstate(invalid="ignore"):
            p = np.exp(s - mnew)
            mult = np.exp(mrun - mnew)
        den = den * mult + p.sum(axis=2, dtype=F32, keepdims=True)
        if dropout_prob > 0.0:
            p = dropout(p, dropout_prob, seed, (rows * Lk + cols)[None])
        acc = acc * mult + np.matmul(round_to_f16(p), v16[:, k0:k1], dtype=F32)
        mrun = mnew
    out = acc / den
    return out.astype(out_dtype).reshape(B, N, Lq, D)


def softmax_rows(x):
    """softmax over the last dim with fp32 max / sum."""
    xf = _as_f32(x)
    m = xf.max(axis=-1, keepdims=True)
    e = np.exp(xf - m)
    return (e / e.sum(axis=-1, dtype=F32, keepdims=True)).astype(x.dtype)


# ---------------------------------------------------------------------------
# Model: parameters are a dict keyed like FusedGPT's state_dict (gpt.py:137-157)
# ---------------------------------------------------------------------------
def synthetic_params(n_layer, n_head, n_embd, vocab_size, block_size, seed=1337,
                     dtype=np.float32, std=0.02):
    """Weights N(0, std), biases 0, LayerNorm gamma 1 / beta 0, from numpy's PCG64
    (bit-stable for a given numpy version, so both sides of a parity test can
    regenerate them from the seed)."""
    rng = np.random.default_rng(seed)
    h = n_embd

    def normal(*shape):
        return (rng.standard_normal(shape, dtype=np.float32) * np.float32(std)).astype(dtype)

    p = {"wte_weight": normal(vocab_size, h), "wpe_weight": normal(block_size, h)}
    for i in range(n_layer):
        a, m = f"blocks.{i}.0.", f"blocks.{i}.1."
        p[a + "layer_norm_weight"] = np.ones(h, dtype)
        p[a + "layer_norm_bias"] = np.zeros(h, dtype)
        p[a + "c_attn_weight"] = normal(h, 3 * h)
        p[a + "c_attn_bias"] = np.zeros(3 * h, dtype)
        p[a + "c_proj_weight"] = normal(h, h)
        p[a + "c_proj_bias"] = np.zeros(h, dtype)
        p[m + "layer_norm_weight"] = np.ones(h, dtype)
        p[m + "layer_norm_bias"] = np.zeros(h, dtype)
        p[m + "ffn1_weight"] = normal(h, 4 * h)
        p[m + "ffn1_bias"] = np.zeros(4 * h, dtype)
        p[m + "ffn2_weight"] = normal(4 * h, h)
        p[m + "ffn2_bias"] = np.zeros(h, dtype)
    p["layer_norm_weight"] = np.ones(h, dtype)
    p["layer_norm_bias"] = np.zeros(h, dtype)
    return p


def synthetic_ids(batch, seqlen, vocab_size, seed=1337):
    rng = np.random.default_rng(seed + 1)
    return rng.integers(0, vocab_size, size=(batch, seqlen), dtype=np.int64)


def n_layers_of(params):
    return 1 + max(int(k.split(".")[1]) for k in params if k.startswith("blocks."))


def gpt2_forward(params, ids, n_head, lm_head=False, dropout_prob=0.0):
    """FusedGPT.forward (gpt.py:163-180); every operator output is stored in the parameter
    dtype, as it is between the reference's kernels.  dropout_prob = 0 is eval mode; in
    training mode the reference hands its dropout to the embedding, the attention weights,
    the attention projection and BOTH ffn products (gpt.py:44-58, 92-109, 165-167)."""
    p = dropout_prob
    x = fused_embeddings(ids, params["wte_weight"], params["wpe_weight"], dropout_prob=p)
    for i in range(n_layers_of(params)):
        a, m = f"blocks.{i}.0.", f"blocks.{i}.1."
        res = x
        y = fused_layer_norm(x, params[a + "layer_norm_weight"], params[a + "layer_norm_bias"])
        q, k, v = matmul_and_split_qkv(y, params[a + "c_attn_weight"], params[a + "c_attn_bias"],
                                       n_head)
        o = flash_attention_v1(q, k, v, dropout_prob=p)
        o = np.ascontiguousarray(o.transpose(0, 2, 1, 3)).reshape(res.shape)  # gpt.py:51
        x = fused_ffn(o, params[a + "c_proj_weight"], bias=params[a + "c_proj_bias"], residual=res,
                      dropout_prob=p)
        res = x
        y = fused_layer_norm(x, params[m + "layer_norm_weight"], params[m + "layer_norm_bias"])
        y = fused_ffn(y, params[m + "ffn1_weight"], bias=params[m + "ffn1_bias"], add_gelu=True,
                      dropout_prob=p)
        x = fused_ffn(y, params[m + "ffn2_weight"], bias=params[m + "ffn2_bias"], residual=res,
                      dropout_prob=p)
    x = fused_layer_norm(x, params["layer_norm_weight"], params["layer_norm_bias"])
    if not lm_head:
        return x
    # tied LM head: hidden @ wte^T through the same fp16-operand GEMM
    return x, fused_ffn(x, np.ascontiguousarray(params["wte_weight"].T))
