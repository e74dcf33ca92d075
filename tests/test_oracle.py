"""Pins the CPU oracle (oracle/gpt2_oracle.py) against things it did not come from: library
routines, fp64 closed forms, invariants and special cases chosen so that a dropped term, a
wrong sign/index or a transposed operand fails.  No GPU involved."""
import math
import os

import numpy as np
import pytest
import torch

from oracle import gpt2_oracle as O


def rng(seed=1337):
    return np.random.default_rng(seed)


def h16(a):
    return a.astype(np.float16).astype(np.float64)


# ----------------------------------------------------------------------------- embeddings
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("V,H,L,P", [(2, 32, 10, 20), (32, 128, 20, 20), (32, 256, 10, 20)])
def test_embeddings_closed_form(dtype, V, H, L, P):
    # the reference's own oracle, test.py:41
    r = rng()
    ids = r.integers(0, V, size=(8, L))
    wte = r.random((V, H)).astype(dtype)
    wpe = r.random((P, H)).astype(dtype)
    want = torch.from_numpy(wte)[torch.from_numpy(ids)] + torch.from_numpy(wpe)[torch.arange(L)][None]
    got = O.fused_embeddings(ids, wte, wpe)
    assert got.dtype == dtype
    assert np.array_equal(got, want.numpy())


def test_embeddings_position_is_row_mod_L():
    # wte = 0 isolates the position term: out[b, l] must be wpe[l] for every b
    ids = np.zeros((3, 5), dtype=np.int64)
    wte = np.zeros((1, 4), np.float32)
    wpe = np.arange(28, dtype=np.float32).reshape(7, 4)
    got = O.fused_embeddings(ids, wte, wpe)
    for b in range(3):
        assert np.array_equal(got[b], wpe[:5])


# ----------------------------------------------------------------------------- layer norm
@pytest.mark.parametrize("M,K", [(249, 123), (32, 128), (249, 64), (7, 768)])
def test_layer_norm_vs_torch_fp64(M, K):
    r = rng()
    x = r.random((M, K)).astype(np.float32)  # U[0,1) like test.py:17-25
    w = (1 + 0.1 * r.standard_normal(K)).astype(np.float32)
    b = (0.1 * r.standard_normal(K)).astype(np.float32)
    want = torch.nn.functional.layer_norm(torch.from_numpy(x).double(), (K,),
                                          torch.from_numpy(w).double(),
                                          torch.from_numpy(b).double(), 1e-5).numpy()
    got = O.fused_layer_norm(x, w, b)
    assert np.abs(got - want).max() < 2e-6


def test_layer_norm_invariants():
    r = rng(3)
    x = (5 + 3 * r.standard_normal((16, 96))).astype(np.float32)
    one, zero = np.ones(96, np.float32), np.zeros(96, np.float32)
    y = O.fused_layer_norm(x, one, zero)
    assert np.abs(y.mean(axis=1)).max() < 1e-6
    assert np.abs(y.var(axis=1) - 1).max() < 1e-4  # biased variance; eps makes it < 1
    # shift invariance and the eps term: a constant row normalises to exactly beta
    c = np.full((2, 96), 7.25, np.float32)
    assert np.array_equal(O.fused_layer_norm(c, one, zero + 0.5), np.full((2, 96), 0.5, np.float32))
    # eps = 1e-5 matters for tiny-variance rows: var = 1e-6 -> scale 1/sqrt(1.1e-5)
    t = np.tile(np.array([1e-3, -1e-3], np.float32), 48)[None]
    got = O.fused_layer_norm(t, one, zero)[0, 0]
    assert abs(got - 1e-3 / math.sqrt(1e-6 + 1e-5)) < 1e-6


def test_layer_norm_fp16_storage():
    r = rng(5)
    x = r.standard_normal((9, 768)).astype(np.float16)
    w = (1 + 0.02 * r.standard_normal(768)).astype(np.float16)
    b = (0.02 * r.standard_normal(768)).astype(np.float16)
    want = torch.nn.functional.layer_norm(torch.from_numpy(x).double(), (768,),
                                          torch.from_numpy(w).double(),
                                          torch.from_numpy(b).double(), 1e-5)
    got = O.fused_layer_norm(x, w, b)
    assert got.dtype == np.float16
    # one fp16 rounding of the fp64 answer
    assert np.abs(got.astype(np.float64) - want.numpy()).max() <= 2.0**-11 * 8


# ----------------------------------------------------------------------------- GELU
def test_gelu_vs_torch_tanh_form():
    x = np.linspace(-12, 12, 4801).astype(np.float32)
    want = torch.nn.functional.gelu(torch.from_numpy(x).double(), approximate="tanh").numpy()
    got = O.gelu_new(x)
    assert np.abs(got - want).max() < 2e-6
    big = O.gelu_new(np.array([-1e4, -100.0, 100.0, 1e4], np.float32))
    assert np.array_equal(big, np.array([0.0, 0.0, 100.0, 1e4], np.float32)) or \
        np.allclose(big, [0.0, 0.0, 100.0, 1e4])
    assert np.all(np.isfinite(big))


# ----------------------------------------------------------------------------- fused_ffn
def ffn_fp64(x, w, b=None, r=None, gelu=False):
    z = h16(x) @ h16(w)
    if b is not None:
        z = z + b.astype(np.float64)
    if gelu:
        z = torch.nn.functional.gelu(torch.from_numpy(z), approximate="tanh").numpy()
    if r is not None:
        z = z + r.astype(np.float64)
    return z


@pytest.mark.parametrize("M,N,K", [(128, 128, 256), (199, 129, 129), (61, 31, 23)])
@pytest.mark.parametrize("gelu", [True, False])
@pytest.mark.parametrize("bias", [True, False])
def test_ffn_vs_fp64(M, N, K, gelu, bias):
    # shapes and U[0,1) inputs of test.py:62-87; residual only when K == N (test.py:23-24)
    r = rng()
    x = r.random((M, K)).astype(np.float32)
    w = r.random((K, N)).astype(np.float32)
    b = r.random(N).astype(np.float32) if bias else None
    res = r.random((M, N)).astype(np.float32) if K == N else None
    want = ffn_fp64(x, w, b, res, gelu)
    got = O.fused_ffn(x, w, bias=b, residual=res, add_gelu=gelu)
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()


def test_ffn_rounds_operands_to_fp16_not_fp32():
    # a true-fp32 product differs from the fp16-operand product by ~4e-4 relative
    r = rng(11)
    x = r.standard_normal((64, 512)).astype(np.float32)
    w = (0.02 * r.standard_normal((512, 64))).astype(np.float32)
    got = O.fused_ffn(x, w).astype(np.float64)
    rounded = h16(x) @ h16(w)
    exact = x.astype(np.float64) @ w.astype(np.float64)
    assert np.abs(got - rounded).max() < 1e-5
    assert np.abs(got - exact).max() > 1e-4


def test_ffn_is_not_transposed_and_epilogue_order():
    # asymmetric one-hot operands: z[m, n] = x[m, :] . w[:, n]
    x = np.zeros((2, 3), np.float32)
    w = np.zeros((3, 4), np.float32)
    x[1, 2] = 2.0
    w[2, 3] = 3.0
    z = O.fused_ffn(x, w)
    want = np.zeros((2, 4), np.float32)
    want[1, 3] = 6.0
    assert np.array_equal(z, want)
    # order bias -> gelu -> residual: gelu(0 + b) + r, not gelu(0 + b + r)
    b = np.full(4, -3.0, np.float32)
    r = np.full((2, 4), 10.0, np.float32)
    z = O.fused_ffn(np.zeros((2, 3), np.float32), w, bias=b, residual=r, add_gelu=True)
    g = float(torch.nn.functional.gelu(torch.tensor(-3.0, dtype=torch.float64), approximate="tanh"))
    assert np.allclose(z, 10.0 + g, atol=1e-6)


def test_ffn_fp16_storage_rounds_once():
    r = rng(13)
    x = r.standard_normal((32, 768)).astype(np.float16)
    w = (0.02 * r.standard_normal((768, 96))).astype(np.float16)
    b = (0.02 * r.standard_normal(96)).astype(np.float16)
    want = ffn_fp64(x, w, b, None, True)
    got = O.fused_ffn(x, w, bias=b, add_gelu=True)
    assert got.dtype == np.float16
    assert np.abs(got.astype(np.float64) - want).max() <= 2.0**-11 * np.abs(want).max() + 1e-6


# ----------------------------------------------------------------------------- qkv split
def test_split_qkv_is_the_index_identity():
    r = rng(17)
    B, L, heads, d = 2, 5, 3, 8
    h = heads * d
    x = r.standard_normal((B, L, h)).astype(np.float32)
    w = (0.1 * r.standard_normal((h, 3 * h))).astype(np.float32)
    b = r.standard_normal(3 * h).astype(np.float32)
    y = O.fused_ffn(x, w, bias=b)
    q, k, v = O.matmul_and_split_qkv(x, w, b, heads)
    assert q.shape == (B, heads, L, d)
    for bb in range(B):
        for n in range(heads):
            for l in range(L):
                assert np.array_equal(q[bb, n, l], y[bb, l, n * d:(n + 1) * d])
                assert np.array_equal(k[bb, n, l], y[bb, l, h + n * d:h + (n + 1) * d])
                assert np.array_equal(v[bb, n, l], y[bb, l, 2 * h + n * d:2 * h + (n + 1) * d])


# ----------------------------------------------------------------------------- attention
def attention_fp64(q, k, v):
    # test.py:98-106 on the fp16-rounded operands
    B, N, L, D = q.shape
    q, k, v = (torch.from_numpy(h16(t)).view(B * N, L, D) for t in (q, k, v))
    s = (q @ k.transpose(1, 2)) / math.sqrt(D)
    mask = torch.tril(torch.ones((L, L), dtype=torch.bool))
    s = torch.where(mask, s, float("-inf"))
    return (s.softmax(-1) @ v).view(B, N, L, D).numpy()


@pytest.mark.parametrize("B,N", [(3, 9), (2, 7)])
@pytest.mark.parametrize("L", [199, 128, 63])
@pytest.mark.parametrize("D", [64, 128])
def test_attention_vs_textbook(B, N, L, D):
    r = rng()
    q, k, v = (r.random((B, N, L, D)).astype(np.float32) for _ in range(3))
    want = attention_fp64(q, k, v)
    got = O.flash_attention_v1(q, k, v)
    # the only modelled difference is the fp16 rounding of P (<= 2^-11 relative per weight)
    assert np.abs(got - want).max() <= 2.0**-11 * np.abs(want).max()


def test_attention_gaussian_inputs_and_invariants():
    r = rng(23)
    B, N, L, D = 2, 3, 150, 64
    q, k, v = (r.standard_normal((B, N, L, D)).astype(np.float32) for _ in range(3))
    got = O.flash_attention_v1(q, k, v)
    want = attention_fp64(q, k, v)
    assert np.abs(got - want).max() <= 2.0**-10 * np.abs(v).max()
    # row 0 attends to key 0 only -> exactly v16[0]
    assert np.array_equal(got[:, :, 0], v.astype(np.float16).astype(np.float32)[:, :, 0])
    # every output is a convex combination of the visible value rows
    v16 = v.astype(np.float16).astype(np.float32)
    for l in (1, 7, 64, 149):
        lo, hi = v16[:, :, :l + 1].min(axis=2), v16[:, :, :l + 1].max(axis=2)
        assert np.all(got[:, :, l] >= lo - 1e-3) and np.all(got[:, :, l] <= hi + 1e-3)
    # causality: changing a future key/value must not change earlier rows
    k2, v2 = k.copy(), v.copy()
    k2[:, :, 100:] += 1.0
    v2[:, :, 100:] -= 2.0
    got2 = O.flash_attention_v1(q, k2, v2)
    assert np.array_equal(got[:, :, :100], got2[:, :, :100])
    assert not np.array_equal(got[:, :, 100:], got2[:, :, 100:])


def test_attention_single_tile_equals_plain_softmax():
    # L <= 64: one key tile, no rescaling; P = exp(S - rowmax) rounded to fp16, denominator
    # from the unrounded P.  Restated here with plain loops, not with the oracle's code path.
    r = rng(29)
    L, D = 40, 64
    q, k, v = (r.standard_normal((1, 1, L, D)).astype(np.float32) for _ in range(3))
    got = O.flash_attention_v1(q, k, v)[0, 0]
    q16, k16, v16 = (t.astype(np.float16).astype(np.float32)[0, 0] for t in (q, k, v))
    for i in (0, 1, 17, 39):
        s = np.array([np.float32(np.dot(q16[i].astype(np.float64), k16[j].astype(np.float64)))
                      * np.float32(0.125) for j in range(i + 1)], dtype=np.float32)
        p = np.exp(s - s.max()).astype(np.float32)
        p16 = p.astype(np.float16).astype(np.float64)
        out = (p16[:, None] * v16[:i + 1].astype(np.float64)).sum(0) / p.astype(np.float64).sum()
        assert np.abs(got[i] - out).max() < 2e-6


def test_attention_tile_size_only_moves_the_p_rounding():
    r = rng(31)
    q, k, v = (r.standard_normal((1, 2, 200, 64)).astype(np.float32) for _ in range(3))
    a = O.flash_attention_v1(q, k, v, block=64)
    b = O.flash_attention_v1(q, k, v, block=32)
    assert 0 < np.abs(a - b).max() <= 2.0**-10 * np.abs(v).max()


def test_attention_vs_reference_golden_vectors():
    """tests/golden/flash_attention_v1.npz holds outputs of the reference's own
    flash_attention_v1 (Triton CPU interpreter, tests/golden/make_flash_vectors.py).  They pin
    what no closed form does: the fp16 rounding of P relative to the per-tile running max.  The
    oracle reproduces them to the last bit except for fp32 summation order inside matmul."""
    import os

    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "flash_attention_v1.npz"))
    for n in "abc":
        q, k, v = (z[f"{n}_{t}"].astype(np.float32) for t in "qkv")
        want = z[f"{n}_out"]
        got = O.flash_attention_v1(q, k, v)
        diff = np.abs(got.astype(np.float64) - want)
        assert diff.max() <= 2e-7 * np.abs(want).max()
        assert (diff == 0).mean() > 0.95
        # and the vectors themselves are sane: within the P-rounding distance of the textbook
        assert np.abs(want - attention_fp64(q, k, v)).max() <= 2.0**-11 * np.abs(v).max()
        # a tile of 32 instead of 64 moves the rounding and is told apart by the vectors
        other = O.flash_attention_v1(q, k, v, block=32)
        assert np.abs(other.astype(np.float64) - want).max() > 20 * diff.max()


def test_attention_unequal_lengths_vs_reference_golden_vectors():
    """tests/golden/flash_attention_v1_lq_lk.npz: the reference's flash_attention_v1 with
    Lq != Lk (Triton CPU interpreter, tests/golden/make_flash_lqlk_vectors.py).  The vectors pin
    the two things only the reference's code decides: keys past the last query are invisible
    (Lq < Lk), and the zero rows that fill up the last key tile are visible to the queries at or
    past Lk (Lq > Lk)."""
    import os

    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "flash_attention_v1_lq_lk.npz"))
    for n in ("short_q", "long_q", "long_q_whole_tile", "long_q_d128"):
        q, k, v = (z[f"{n}_{t}"].astype(np.float32) for t in "qkv")
        want = z[f"{n}_out"]
        got = O.flash_attention_v1(q, k, v)
        diff = np.abs(got.astype(np.float64) - want)
        assert diff.max() <= 2e-7 * np.abs(want).max(), n
        assert (diff == 0).mean() > 0.95, n
    # the vectors against the textbook, written out independently of the oracle: softmax over the
    # visible keys, where a padding row counts as a key with score 0 and value 0
    for n, pad_to in (("short_q", None), ("long_q", 128), ("long_q_whole_tile", 64),
                      ("long_q_d128", 64)):
        q, k, v = (z[f"{n}_{t}"].astype(np.float64) for t in "qkv")
        want = z[f"{n}_out"]
        Lq, Lk, D = q.shape[2], k.shape[2], q.shape[3]
        for bn in range(q.shape[1]):
            for i in (0, Lq // 3, Lq - 1):
                vis = min(i + 1, Lk)
                s = (k[0, bn, :vis] @ q[0, bn, i]) / np.sqrt(D)
                zeros = 0 if pad_to is None else max(0, min(i + 1, pad_to) - Lk)
                s_all = np.concatenate([s, np.zeros(zeros)])
                w = np.exp(s_all - s_all.max())
                out = (w[:vis, None] * v[0, bn, :vis]).sum(0) / w.sum()
                assert np.abs(out - want[0, bn, i]).max() <= 2.0**-10 * np.abs(v).max(), (n, i)
    # a plausible mistake -- masking the padding rows by Lk -- is told apart by the vectors
    q, k, v = (z[f"long_q_{t}"].astype(np.float64) for t in "qkv")
    i = 149
    s = (k[0, 0] @ q[0, 0, i]) / 8.0
    w = np.exp(s - s.max())
    no_pad = (w[:, None] * v[0, 0]).sum(0) / w.sum()
    assert np.abs(no_pad - z["long_q_out"][0, 0, i]).max() > 1e-2


def test_attention_shorter_queries_equal_truncated_keys():
    # Lq < Lk: exactly the attention over the first Lq keys (later tiles add exact zeros)
    r = rng(41)
    q = r.standard_normal((1, 2, 90, 64)).astype(np.float32)
    k, v = (r.standard_normal((1, 2, 200, 64)).astype(np.float32) for _ in range(2))
    a = O.flash_attention_v1(q, k, v)
    b = O.flash_attention_v1(q, k[:, :, :90], v[:, :, :90])
    assert np.array_equal(a, b)


# ----------------------------------------------------------------------------- softmax
def test_softmax_vs_torch():
    r = rng(37)
    x = (4 * r.standard_normal((33, 768))).astype(np.float32)
    want = torch.softmax(torch.from_numpy(x).double(), -1).numpy()
    got = O.softmax_rows(x)
    assert np.abs(got - want).max() < 5e-7  # a few fp32 ulps of values <= 1
    assert np.abs(got.sum(-1) - 1).max() < 1e-5
    x16 = x.astype(np.float16)
    got16 = O.softmax_rows(x16)
    want16 = torch.softmax(torch.from_numpy(x16).double(), -1).numpy()
    assert got16.dtype == np.float16
    assert np.abs(got16.astype(np.float64) - want16).max() <= 2.0**-11


# ----------------------------------------------------------------------------- whole model
def gpt2_fp64(params, ids, n_head):
    """An independently written GPT-2 (HF block order: ln_1 -> attn -> +res -> ln_2 -> mlp ->
    +res -> ln_f) in fp64 torch, true-precision matmuls, library softmax/gelu/layer_norm."""
    P = {k: torch.from_numpy(np.asarray(v)).double() for k, v in params.items()}
    ids_t = torch.from_numpy(ids)
    B, L = ids.shape
    h = P["wte_weight"].shape[1]
    d = h // n_head
    F = torch.nn.functional
    x = P["wte_weight"][ids_t] + P["wpe_weight"][:L]
    mask = torch.tril(torch.ones(L, L, dtype=torch.bool))
    for i in range(O.n_layers_of(params)):
        a, m = f"blocks.{i}.0.", f"blocks.{i}.1."
        y = F.layer_norm(x, (h,), P[a + "layer_norm_weight"], P[a + "layer_norm_bias"], 1e-5)
        qkv = y @ P[a + "c_attn_weight"] + P[a + "c_attn_bias"]
        q, k, v = (t.view(B, L, n_head, d).permute(0, 2, 1, 3) for t in qkv.split(h, dim=-1))
        s = (q @ k.transpose(-1, -2)) / math.sqrt(d)
        s = s.masked_fill(~mask, float("-inf"))
        o = (s.softmax(-1) @ v).permute(0, 2, 1, 3).reshape(B, L, h)
        x = x + o @ P[a + "c_proj_weight"] + P[a + "c_proj_bias"]
        y = F.layer_norm(x, (h,), P[m + "layer_norm_weight"], P[m + "layer_norm_bias"], 1e-5)
        y = F.gelu(y @ P[m + "ffn1_weight"] + P[m + "ffn1_bias"], approximate="tanh")
        x = x + y @ P[m + "ffn2_weight"] + P[m + "ffn2_bias"]
    x = F.layer_norm(x, (h,), P["layer_norm_weight"], P["layer_norm_bias"], 1e-5)
    return x.numpy(), (x @ P["wte_weight"].T).numpy()


def test_model_composition_vs_independent_fp64_gpt2():
    cfg = dict(n_layer=3, n_head=4, n_embd=128, vocab_size=211, block_size=96)
    params = O.synthetic_params(**cfg, seed=7, std=0.08)
    r = rng(41)
    for k in params:  # non-trivial biases and LayerNorm affine so a dropped term shows
        if k.endswith("_bias"):
            params[k] = (0.05 * r.standard_normal(params[k].shape)).astype(np.float32)
        elif "layer_norm_weight" in k:
            params[k] = (1 + 0.1 * r.standard_normal(params[k].shape)).astype(np.float32)
    ids = O.synthetic_ids(2, 80, cfg["vocab_size"], seed=7)
    want_h, want_logits = gpt2_fp64(params, ids, cfg["n_head"])
    got_h, got_logits = O.gpt2_forward(params, ids, cfg["n_head"], lm_head=True)
    # fp16 operand rounding inside every product: ~1e-3 relative overall
    assert np.abs(got_h - want_h).max() <= 5e-3 * np.abs(want_h).max()
    assert np.abs(got_logits - want_logits).max() <= 5e-3 * np.abs(want_logits).max()
    # and the bound discriminates: flipping the sign of one small (0.05 sigma) bias vector in
    # the middle of the network already lands far outside it
    bad = dict(params)
    bad["blocks.1.1.ffn2_bias"] = -params["blocks.1.1.ffn2_bias"]
    bad_h = O.gpt2_forward(bad, ids, cfg["n_head"])
    assert np.abs(bad_h - want_h).max() > 2e-2 * np.abs(want_h).max()


def hf_gpt2(seed=1337, **kw):
    """A randomly initialised HuggingFace GPT2Model (the reference's end-to-end oracle,
    test.py:120-133), built locally from a config: nothing is downloaded.  Biases and the
    LayerNorm affine get non-trivial values so that a dropped term shows."""
    from transformers import GPT2Config, GPT2Model

    torch.manual_seed(seed)
    cfg = GPT2Config(bos_token_id=None, eos_token_id=None, **kw)
    hf = GPT2Model(cfg).eval()
    with torch.no_grad():
        for name, p in hf.named_parameters():
            if name.endswith("bias"):
                p.normal_(0, 0.1)
            elif "ln_" in name:
                p.normal_(1, 0.1)
            else:
                p.normal_(0, 0.08)
    return hf

def test_fp32_chain_drift_is_accumulation_noise():
    """What "fp32 outputs within 1e-4 relative" can mean for the whole model.  Benchmark
    configuration 0 (124M, fp32 storage, batch 2 x seqlen 64) evaluated twice with the same
    formulas and the same rounding points (fp16 operands, fp32 storage between operators),
    once with fp32 and once with fp64 sums.  Every operator alone agrees to ~1e-6, but a last
    bit of difference in an activation now and then flips the fp16 rounding of a GEMM operand
    (a 2^-11 relative step) and the following layers carry it along: the two evaluations end
    up a few 1e-4 of max|b| apart.  Two correct implementations that order their fp32 sums
    differently (numpy's pairwise sums, the MFMA's k-blocked sums) are in the same position,
    so the GPU tests bound |gpu - oracle| by a multiple of this distance, measured on the
    spot, rather than by a hand-picked number."""
    cfg = dict(n_layer=12, n_head=12, n_embd=768, vocab_size=50257, block_size=1024)
    P = O.synthetic_params(**cfg, seed=1337, dtype=np.float32)
    ids = O.synthetic_ids(2, 64, cfg["vocab_size"], seed=1337)
    h32 = O.gpt2_forward(P, ids, cfg["n_head"])
    with O.accumulation_dtype(np.float64):
        h64 = O.gpt2_forward(P, ids, cfg["n_head"])
        # inside the block one operator differs from its fp32 evaluation by rounding noise only
        y64 = O.fused_ffn(P["wpe_weight"][:64], P["blocks.0.1.ffn1_weight"], add_gelu=True)
    assert O.F32 is np.float32 and h64.dtype == np.float32
    y32 = O.fused_ffn(P["wpe_weight"][:64], P["blocks.0.1.ffn1_weight"], add_gelu=True)
    assert np.abs(y64 - y32).max() <= 2e-6 * np.abs(y32).max()
    d = np.abs(h64.astype(np.float64) - h32.astype(np.float64))
    scale = np.abs(h32).max()
    rel_max, rel_med = d.max() / scale, np.median(d) / scale
    print(f"fp64- vs fp32-accumulate oracle, 124M hidden: max {rel_max:.3e}, median {rel_med:.3e} "
          f"of max|b| {scale:.3f}")
    # measured 5.6e-4 and 8.7e-5: well above the 1e-4 a per-operator comparison meets, and far
    # below anything a wrong formula, index or rounding point would produce
    assert 1e-4 < rel_max < 3e-3
    assert 1e-5 < rel_med < 4e-4



def test_model_vs_huggingface_gpt2():
    """The oracle's forward, fed HF weights through the package's key conversion, against the
    transformers library's own GPT2Model in fp32 on the CPU.  Tolerance: 1e-2 absolute on
    hidden states of magnitude ~5 (the oracle rounds every GEMM operand to fp16; the
    reference's own comparison allows 1e-1, test.py:133)."""
    from gpt_triton_amd.gpt import convert_huggingface_to_triton

    hf = hf_gpt2(vocab_size=97, n_positions=48, n_embd=128, n_layer=2, n_head=2)
    ids = torch.randint(0, 97, (3, 40))
    with torch.no_grad():
        want = hf(ids).last_hidden_state.numpy()
    sd, config = convert_huggingface_to_triton(hf.state_dict(), hf.config)
    assert config.block_size == 48  # n_positions: this transformers has no n_ctx (gpt.py:202)
    params = {k: v.numpy() for k, v in sd.items()}
    got = O.gpt2_forward(params, ids.numpy(), config.n_head)
    assert np.abs(want).max() > 2.0
    assert np.abs(got - want).max() <= 1e-2


# ---------------------------------------------------------------------------
# dropout: Philox-4x32-10 -> tl.rand -> keep mask (kernels.py:31-34)
# ---------------------------------------------------------------------------
PHILOX_KAT = [  # counter, key, output: the philox4x32 10-round vectors of the Random123 distribution
    ((0, 0, 0, 0), (0, 0), (0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8)),
    ((0xFFFFFFFF,) * 4, (0xFFFFFFFF,) * 2, (0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD)),
    ((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0),
     (0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1)),
]


@pytest.mark.parametrize("ctr,key,want", PHILOX_KAT)
def test_philox_known_answers(ctr, key, want):
    got = O.philox4x32_10(*[np.array([c], dtype=np.uint32) for c in ctr], *key)
    assert tuple(int(g[0]) for g in got) == want


def test_philox_is_elementwise():
    offs = np.array([0, 1, 2, 0xFFFFFFFF, 12345], dtype=np.uint32)
    z = np.zeros_like(offs)
    whole = O.philox4x32_10(offs, z, z, z, 1337, 0)[0]
    single = [O.philox4x32_10(offs[i:i + 1], z[:1], z[:1], z[:1], 1337, 0)[0][0] for i in range(5)]
    assert whole.tolist() == single
    assert len(set(whole.tolist())) == 5


def test_uniform_map_closed_form():
    # int32 view, negatives folded by -x-1, times 4.6566127342e-10 in fp32
    words = np.array([0, 1, 0x7FFFFFFF, 0x80000000, 0xFFFFFFFF, 0x40000000], dtype=np.uint32)
    want = np.array([0, 1, 2**31 - 1, 2**31 - 1, 0, 2**30], dtype=np.float64)
    got = O.uint_to_uniform_float(words)
    assert got.dtype == np.float32
    assert np.array_equal(got, (want.astype(np.float32) * np.float32(4.6566127342e-10)))
    assert got.max() < 1.0 and got.min() == 0.0


def test_rand_default_seed_statistics_and_no_exact_zero():
    r = O.tl_rand(1337, np.arange(1 << 20))
    # the embedding applies dropout even at p = 0 (kernels.py:70): identity iff rand > 0
    assert (r > 0).all() and (r < 1).all()
    assert abs(r.mean() - 0.5) < 2e-3
    for p in (0.1, 0.25, 0.5):
        assert abs((r > np.float32(p)).mean() - (1 - p)) < 2e-3
    # seeds and offsets are distinct streams
    assert not np.array_equal(r[:64], O.tl_rand(1338, np.arange(64)))
    # int32 offsets wrap like the device's: -1 is counter 0xFFFFFFFF
    assert O.tl_rand(1337, np.array([-1]))[0] == O.tl_rand(1337, np.array([0xFFFFFFFF]))[0]


def test_dropout_scales_by_true_division():
    x = rng(5).standard_normal((4, 50)).astype(np.float32)
    off = np.arange(200).reshape(4, 50)
    y = O.dropout(x, 0.3, 1337, off)
    keep = O.tl_rand(1337, off) > np.float32(0.3)
    assert np.array_equal(y[keep], x[keep] / (np.float32(1) - np.float32(0.3)))
    assert (y[~keep] == 0).all() and 0.55 < keep.mean() < 0.85


def _golden_dropout():
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "dropout.npz"))
    return g, (lambda k: g[k].astype(np.float32))


def test_dropout_embeddings_vs_reference_golden_vectors():
    """tests/golden/dropout.npz: outputs of the reference's own operators with dropout under
    Triton's CPU interpreter (tests/golden/make_dropout_vectors.py)."""
    g, f = _golden_dropout()
    got = O.fused_embeddings(g["emb_ids"], f("emb_wte"), f("emb_wpe"), dropout_prob=float(g["emb_p"]))
    assert np.array_equal(got, g["emb_out"])
    # one mask for all tokens: the zero pattern is a function of the column alone
    dropped = ~(O.tl_rand(1337, np.arange(200)) > g["emb_p"])
    assert 0 < dropped.mean() < 0.5
    assert (g["emb_out"][..., dropped] == 0).all()
    assert (g["emb_out"][..., ~dropped] != 0).mean() > 0.99  # a few sums cancel exactly
    assert np.array_equal(O.fused_embeddings(g["emb_ids"], f("emb_wte"), f("emb_wpe")), g["emb_out_p0"])


def test_dropout_ffn_vs_reference_golden_vectors():
    g, f = _golden_dropout()
    got = O.fused_ffn(f("ffn_x"), f("ffn_w"), bias=f("ffn_b"), residual=f("ffn_r"), add_gelu=True,
                      dropout_prob=float(g["ffn_p"]))
    assert np.abs(got - g["ffn_out"]).max() <= 4e-6  # summation order of the fp32 products
    # where the value was dropped the output is the residual itself: pins dropout-before-residual
    dropped = g["ffn_out"] == f("ffn_r")
    assert 0.05 < dropped.mean() < 0.16 and np.array_equal(dropped, got == f("ffn_r"))
    plain = O.fused_ffn(f("ffn_x"), f("ffn_w"), dropout_prob=0.5)
    assert np.array_equal(plain == 0, g["ffn_out_plain"] == 0)
    assert np.abs(plain - g["ffn_out_plain"]).max() <= 4e-6


def test_dropout_attention_vs_reference_golden_vectors():
    g, f = _golden_dropout()
    got = O.flash_attention_v1(f("att_q"), f("att_k"), f("att_v"), dropout_prob=float(g["att_p"]))
    d = np.abs(got - g["att_out"])
    assert d.max() <= 2e-6 * np.abs(g["att_out"]).max() and (d == 0).mean() > 0.95
    # and it is not the p = 0 result
    assert np.abs(O.flash_attention_v1(f("att_q"), f("att_k"), f("att_v")) - g["att_out"]).max() > 0.05
