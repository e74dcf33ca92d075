"""GPU parity of the GEMMs that run their LayerNorm in the operand prologue
(gptmi_layernorm_linear, gptmi_layernorm_linear_qkv): the fusion the reference's author marks as
to do (kernels.py:132-133) for the pairs fused_layer_norm -> matmul_and_split_qkv (gpt.py:40-41)
and fused_layer_norm -> fused_ffn (gpt.py:92-93).

Two bars, both through ctypes -> libgptmi.so:
  * against the oracle's fused_layer_norm followed by fused_ffn / matmul_and_split_qkv, fp16
    storage tolerance as everywhere (2 fp16 ulps of max|b|);
  * bit for bit against this library's own two launches (gptmi_layernorm, then gptmi_linear /
    gptmi_linear_qkv): the prologue forms its sums in the LayerNorm kernel's order, so the
    operand has the same bits and the model may switch between the two forms by row count.
Rows carry their own mean and scale so that the statistics matter."""
import numpy as np
import pytest
import torch

from oracle import gpt2_oracle as O

pytestmark = pytest.mark.gpu

ULP2 = 2 * 2.0**-10


@pytest.fixture(scope="module")
def K(gpu_device):
    from gpt_triton_amd import kernels

    return kernels


def dev(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def host(t):
    return t.detach().cpu().numpy()


def check_f16(got, want, what):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    assert np.all(np.isfinite(got)), f"{what}: non-finite output"
    scale = np.abs(want).max()
    diff = np.abs(got - want)
    assert diff.max() <= ULP2 * scale, (f"{what}: max|diff| {diff.max():.3e}, "
                                        f"tolerance {ULP2 * scale:.3e}")


def operands(M, H, N, seed):
    r = np.random.default_rng(seed)
    x = r.standard_normal((M, H)) * r.uniform(0.2, 5.0, (M, 1)) + r.uniform(-3.0, 3.0, (M, 1))
    ln_w = 1.0 + 0.2 * r.standard_normal(H)
    ln_b = 0.1 * r.standard_normal(H)
    w = r.standard_normal((H, N)) / np.sqrt(H)
    b = 0.1 * r.standard_normal(N)
    return tuple(a.astype(np.float16) for a in (x, ln_w, ln_b, w, b))


@pytest.mark.parametrize("M,H,N,gelu,bias", [
    (128, 768, 3072, True, True),    # GPT-2's ffn1 at benchmark configuration 0 (2 x 64 tokens)
    (128, 768, 768, False, True),
    (1, 768, 2304, False, True),     # one row: 31 rows of the tile repeat it
    (33, 768, 100, True, False),     # a second row tile with one row, a column tile cut at 100
    (70, 128, 256, False, True),     # one chunk per lane, 32 lanes per row
    (300, 256, 520, True, True),
    (64, 1024, 4096, True, True),    # GPT-2 medium's width: 64 lanes per row, two chunks each
    (40, 1280, 1280, False, True),   # large: five chunks per lane (the eight-chunk variant)
    (32, 1600, 6400, True, True),    # XL: seven chunks per lane, the widest panel that fits
    (5, 64, 64, False, False),
    (5000, 768, 768, False, True),   # 157 row tiles, the last with 8 rows (far beyond where the model uses it)
])
def test_layer_norm_ffn(K, gpu_device, M, H, N, gelu, bias):
    x, ln_w, ln_b, w, b = operands(M, H, N, seed=M + H + N)
    if not bias:
        b = None
    print(f"layer_norm_ffn: M={M} H={H} N={N} gelu={gelu} bias={bias}", flush=True)
    xd, lwd, lbd, wd = (dev(a, gpu_device) for a in (x, ln_w, ln_b, w))
    bd = dev(b, gpu_device) if bias else None
    wp = K.pack_weight(wd)
    assert K.layer_norm_linear_supported(xd, wp)
    z = K.layer_norm_ffn(xd, lwd, lbd, wp, bias=bd, add_gelu=gelu)
    assert z.shape == (M, N) and z.dtype == torch.float16 and z.is_contiguous()
    two = K.fused_ffn(K.fused_layer_norm(xd, lwd, lbd), wp, bias=bd, add_gelu=gelu)
    assert torch.equal(z, two), "differs from fused_layer_norm followed by fused_ffn"
    want = O.fused_ffn(O.fused_layer_norm(x, ln_w, ln_b), w, bias=b, add_gelu=gelu)
    check_f16(host(z), want, "layer_norm_ffn against the oracle")


@pytest.mark.parametrize("B,L,h,heads", [(2, 64, 768, 12), (1, 1, 768, 12), (3, 50, 256, 4),
                                         (2, 70, 128, 2), (1, 40, 1600, 25)])
def test_layer_norm_matmul_and_split_qkv(K, gpu_device, B, L, h, heads):
    x, ln_w, ln_b, w, b = operands(B * L, h, 3 * h, seed=B * L + h)
    x = x.reshape(B, L, h)
    print(f"layer_norm_matmul_and_split_qkv: B={B} L={L} h={h} heads={heads}", flush=True)
    xd, lwd, lbd, wd, bd = (dev(a, gpu_device) for a in (x, ln_w, ln_b, w, b))
    wp = K.pack_weight(wd)
    got = K.layer_norm_matmul_and_split_qkv(xd, lwd, lbd, wp, bd, heads)
    two = K.matmul_and_split_qkv(K.fused_layer_norm(xd, lwd, lbd), wp, bd, heads)
    want = O.matmul_and_split_qkv(O.fused_layer_norm(x, ln_w, ln_b), w, b, heads)
    for name, g, t, o in zip("qkv", got, two, want):
        assert g.shape == (B, heads, L, h // heads) and g.is_contiguous()
        assert torch.equal(g, t), f"{name} differs from the two launches"
        check_f16(host(g), o, f"{name} against the oracle")


def test_layer_norm_ffn_writes_its_rows_only(K, gpu_device):
    """Output pre-filled with NaN and followed by a guard row, through the C entry point."""
    M, H, N = 45, 768, 200
    x, ln_w, ln_b, w, b = operands(M, H, N, seed=5)
    xd, lwd, lbd, wd, bd = (dev(a, gpu_device) for a in (x, ln_w, ln_b, w, b))
    wp = K.pack_weight(wd)
    buf = torch.full((M + 1, N), float("nan"), device=gpu_device, dtype=torch.float16)
    lib = K._lib.load()
    rc = lib.gptmi_layernorm_linear(xd.data_ptr(), lwd.data_ptr(), lbd.data_ptr(), 1e-5,
                                    wp.data_ptr(), bd.data_ptr(), buf.data_ptr(), M, N, H, 0,
                                    K._lib.GPTMI_F16, torch.cuda.current_stream().cuda_stream)
    K._lib.check(rc, "layernorm_linear")
    assert torch.isnan(buf[M]).all(), "wrote past the last row"
    assert not torch.isnan(buf[:M]).any()
    check_f16(host(buf[:M]), O.fused_ffn(O.fused_layer_norm(x, ln_w, ln_b), w, bias=b),
              "against the oracle")


def test_layer_norm_linear_turns_down_what_it_does_not_hold(K, gpu_device):
    """fp32 storage, an unpacked weight, and rows too wide for the LDS panel: refused, not
    computed some other way."""
    x, ln_w, ln_b, w, b = (dev(a, gpu_device) for a in operands(8, 2048, 64, seed=1))
    wp = K.pack_weight(w)
    assert not K.layer_norm_linear_supported(x, wp)  # 48 KB of stages + 128 KB of panel
    with pytest.raises(NotImplementedError):
        K.layer_norm_ffn(x, ln_w, ln_b, wp, bias=b)
    x, ln_w, ln_b, w, b = (dev(a, gpu_device) for a in operands(8, 128, 64, seed=2))
    assert not K.layer_norm_linear_supported(x, w)
    with pytest.raises(NotImplementedError):
        K.layer_norm_ffn(x, ln_w, ln_b, w, bias=b)
    xf, lwf, lbf, wf, bf = (t.float() for t in (x, ln_w, ln_b, w, b))
    assert not K.layer_norm_linear_supported(xf, K.pack_weight(wf))
    with pytest.raises(NotImplementedError):
        K.layer_norm_ffn(xf, lwf, lbf, K.pack_weight(wf), bias=bf)
    lib = K._lib.load()
    assert lib.gptmi_layernorm_linear_supported(8, 100, K._lib.GPTMI_F16) == 0  # not a multiple of 64
    assert lib.gptmi_layernorm_linear_supported(8, 768, K._lib.GPTMI_F32) == 0
    assert lib.gptmi_layernorm_linear_supported(8, 768, K._lib.GPTMI_F16) == 1


def test_model_same_bits_with_and_without_the_prologue(gpu_device, monkeypatch):
    """FusedGPT at benchmark configuration 0 (2 x 64 tokens, the 124M architecture, fp16):
    hidden state and logits with the LayerNorms inside the GEMMs and with them as launches of
    their own are the same bits, and both stay within the model tolerance of the oracle."""
    from gpt_triton_amd import gpt as G

    cfg = dict(n_layer=12, n_head=12, n_embd=768, vocab_size=50257, block_size=1024)
    params = O.synthetic_params(**cfg, seed=1337, dtype=np.float16)
    model = G.FusedGPT(G.GPTConfig(dropout=0.1, **cfg))
    model.load_state_dict({k: torch.from_numpy(np.asarray(v)) for k, v in params.items()})
    model = model.to(device=gpu_device, dtype=torch.float16).eval()
    ids_np = O.synthetic_ids(2, 64, cfg["vocab_size"], seed=1337)
    ids = torch.from_numpy(ids_np).to(gpu_device)
    calls = {"n": 0}
    real = G.layer_norm_ffn

    def counting(*a, **kw):
        calls["n"] += 1
        return real(*a, **kw)

    monkeypatch.setattr(G, "layer_norm_ffn", counting)
    with torch.no_grad():
        hid_a, log_a = model(ids, return_logits=True)
        assert calls["n"] == cfg["n_layer"], "the fused form did not run"
        monkeypatch.setattr(G, "LN_PROLOGUE_MAX_ROWS", 0)
        hid_b, log_b = model(ids, return_logits=True)
        assert calls["n"] == cfg["n_layer"]
    assert torch.equal(hid_a, hid_b) and torch.equal(log_a, log_b)
    want = O.gpt2_forward(params, ids_np, cfg["n_head"])
    diff = np.abs(host(hid_a).astype(np.float64) - want.astype(np.float64)).max()
    print(f"2 x 64 forward, fp16: max|diff| to the oracle {diff:.3e}", flush=True)
    assert diff <= 2e-2
