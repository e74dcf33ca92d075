"""GPU parity at the benchmark configurations that the per-operator tests do not reach:

  * every element of the four GEMMs of the headline forward (M = 512 * 300 = 153600 rows) against
    the same arithmetic done by torch on the GPU, the outputs poisoned with NaN beforehand so that
    a tile which is not written, or written to the wrong place, cannot pass;
  * the max-batch memory point 2048 x 300 of the 124M model (the only size whose activations go
    beyond 2^31 bytes), sampled sequences against the oracle;
  * the GPT-2 XL shape (48 layers, d_model 1600, 25 heads x 64, FFN 6400) at batch 64 x seqlen
    1024: the 25-head q/k/v scatter with N = 4800 and the whole 48-layer forward on sampled
    sequences against the oracle.

Everything goes through ctypes -> libgptmi.so.  Tolerances: fp16 storage, elementwise
|a - b| <= 2^-10 |b| + 2^-12 max|b| for single GEMMs against the fp32 torch product (half an
fp16 ulp of rounding plus accumulation-order noise); model outputs <= 2e-2 absolute (124M) as
in tests/test_gpu_parity.py."""
import numpy as np
import pytest
import torch

from oracle import gpt2_oracle as O

pytestmark = pytest.mark.gpu

M_HEAD = 512 * 300


@pytest.fixture(scope="module")
def K(gpu_device):
    from gpt_triton_amd import kernels

    return kernels


def gelu_tanh(t):
    return torch.nn.functional.gelu(t, approximate="tanh")


def assert_all_close_f16(got, want, what):
    """Every element, on the GPU: got is fp16 storage, want the fp32 result of the same formula."""
    assert got.shape == want.shape, (got.shape, want.shape)
    g = got.float()
    bad_nan = int(torch.isnan(g).sum())
    assert bad_nan == 0, f"{what}: {bad_nan} elements were never written (NaN poison left)"
    scale = float(want.abs().max())
    tol = want.abs() * 2.0**-10 + 2.0**-12 * scale
    excess = (g - want).abs() - tol
    worst = int(torch.argmax(excess))
    n_bad = int((excess > 0).sum())
    assert n_bad == 0, (f"{what}: {n_bad} of {g.numel()} elements out of tolerance; worst at flat "
                        f"index {worst} (row {worst // g.shape[-1]}, col {worst % g.shape[-1]}): "
                        f"got {float(g.flatten()[worst]):.6f} want {float(want.flatten()[worst]):.6f}")


def headline_operands(gpu_device, Kd, N, seed):
    g = torch.Generator(device=gpu_device).manual_seed(seed)
    x = torch.randn((M_HEAD, Kd), generator=g, device=gpu_device).half()
    w = (0.02 * torch.randn((Kd, N), generator=g, device=gpu_device)).half()
    b = (0.02 * torch.randn(N, generator=g, device=gpu_device)).half()
    return x, w, b


@pytest.mark.parametrize("name,Kd,N,gelu,use_res", [
    ("ffn1 768->3072 +bias+GELU", 768, 3072, True, False),
    ("ffn2 3072->768 +bias+residual", 3072, 768, False, True),
    ("attention projection 768->768 +bias+residual", 768, 768, False, True),
])
@pytest.mark.parametrize("packed", [True, False])
def test_headline_gemm_every_element(K, gpu_device, name, Kd, N, gelu, use_res, packed):
    """Benchmark configuration 1 (and the projection): all 153600 x N outputs."""
    x, w, b = headline_operands(gpu_device, Kd, N, seed=N + Kd)
    res = None
    if use_res:
        g = torch.Generator(device=gpu_device).manual_seed(99)
        res = torch.randn((M_HEAD, N), generator=g, device=gpu_device).half()
    z = torch.full((M_HEAD, N), float("nan"), device=gpu_device, dtype=torch.float16)
    print(f"every element: {name} packed={packed}", flush=True)
    if packed:
        K._linear(x, K.pack_weight(w), b, res, z, gelu, 0.0, K._lib.GPTMI_W_PACKED, name)
    else:
        K._linear(x, w, b, res, z, gelu, 0.0, K._lib.GPTMI_W_KN, name)
    want = x.float() @ w.float() + b.float()
    if gelu:
        want = gelu_tanh(want)
    if use_res:
        want = want + res.float()
    assert_all_close_f16(z, want, name)


@pytest.mark.parametrize("M,N,Kd,gelu,bias,in_place", [
    (25600, 768, 128, False, True, False),    # 300 tiles: some workgroups walk two; 2 k-tiles
    (25600, 768, 192, True, False, False),    # 3 k-tiles, GELU in front of the residual, no bias
    (66560, 1024, 256, False, True, True),    # 1040 tiles = 4 rounds + 16: head + small-tile tail,
                                              # output written over the residual
    (4096, 768, 3072, False, True, False),    # 48 tiles: one each, nothing to refill
    (16384, 1600, 320, False, True, False),   # N = 6 x 256 + 64: three of four wavefront columns
                                              # of the last column tile lie past the edge
    (8192, 320, 256, True, True, True),       # two column tiles, the second 64 wide; in place
    (2048, 448, 192, False, True, False),     # 8 + 8 tiles, three k-tiles, last tile 192 wide
])
def test_residual_gemm_streaming_every_element(K, gpu_device, M, N, Kd, gelu, bias, in_place):
    """fp16 GEMM + residual on whole 256 x 256 tiles (the persistent kernel that carries the
    residual through the operand stages and refills them mid-epilogue): every element against the
    fp32 torch product, NaN-poisoned output, k-tile counts 2, 3, 4 and 48, one or several tiles
    per workgroup, with and without the small-tile tail, and in place."""
    g = torch.Generator(device=gpu_device).manual_seed(M + Kd)
    x = torch.randn((M, Kd), generator=g, device=gpu_device).half()
    w = (torch.randn((Kd, N), generator=g, device=gpu_device) / Kd ** 0.5).half()
    b = (0.1 * torch.randn(N, generator=g, device=gpu_device)).half() if bias else None
    res = torch.randn((M, N), generator=g, device=gpu_device).half()
    want = x.float() @ w.float()
    if bias:
        want = want + b.float()
    if gelu:
        want = gelu_tanh(want)
    want = want + res.float()
    print(f"residual streaming: M={M} N={N} K={Kd} gelu={gelu} bias={bias} in_place={in_place}",
          flush=True)
    if in_place:
        z = res.clone()
        K._linear(x, K.pack_weight(w), b, z, z, gelu, 0.0, K._lib.GPTMI_W_PACKED, "in place")
    else:
        z = torch.full((M, N), float("nan"), device=gpu_device, dtype=torch.float16)
        K._linear(x, K.pack_weight(w), b, res, z, gelu, 0.0, K._lib.GPTMI_W_PACKED, "residual")
    assert_all_close_f16(z, want, "residual streaming")


@pytest.mark.parametrize("M,N,Kd,gelu,dtype", [
    (8192, 1600, 256, True, torch.float16),   # 6 whole column tiles + 64 columns
    (4096, 4800, 128, False, torch.float16),  # 18 whole column tiles + 192 columns
    (2048, 448, 192, True, torch.float32),    # fp32 output: the other epilogue of the kernel
    (2048, 320, 128, False, torch.float16),   # two k-tiles, second column tile 64 wide
])
def test_gemm_streaming_ragged_columns_every_element(K, gpu_device, M, N, Kd, gelu, dtype):
    """GEMM + bias (+ GELU) without residual where N is a multiple of 64 and not of 256: the
    persistent kernel's last column tile has wavefronts whose columns lie past the edge (they
    load operands, keep the barriers and store nothing).  Every element against the fp32 torch
    product of the fp16-rounded operands; the output buffer is NaN-poisoned and followed by a
    guard row that must stay untouched."""
    g = torch.Generator(device=gpu_device).manual_seed(N + Kd)
    x = torch.randn((M, Kd), generator=g, device=gpu_device).to(dtype)
    w = (torch.randn((Kd, N), generator=g, device=gpu_device) / Kd ** 0.5).to(dtype)
    b = (0.1 * torch.randn(N, generator=g, device=gpu_device)).to(dtype)
    want = x.half().float() @ w.half().float() + b.float()
    if gelu:
        want = gelu_tanh(want)
    buf = torch.full((M + 1, N), float("nan"), device=gpu_device, dtype=dtype)
    z = buf[:M]
    print(f"ragged columns: M={M} N={N} K={Kd} gelu={gelu} {dtype}", flush=True)
    K._linear(x, K.pack_weight(w), b, None, z, gelu, 0.0, K._lib.GPTMI_W_PACKED, "ragged")
    assert torch.isnan(buf[M]).all(), "wrote past the last row"
    if dtype == torch.float16:
        assert_all_close_f16(z, want, "ragged columns")
    else:
        assert torch.isfinite(z).all()
        torch.testing.assert_close(z, want, rtol=2e-4, atol=2e-4)


def test_headline_qkv_every_element(K, gpu_device):
    """The headline q/k/v product [153600, 768] @ [768, 2304] + b scattered head-major, every
    element of q, k and v, through gptmi_linear_qkv with NaN-poisoned outputs."""
    B, L, heads, d = 512, 300, 12, 64
    h = heads * d
    x, w, b = headline_operands(gpu_device, h, 3 * h, seed=5)
    q, k, v = (torch.full((B, heads, L, d), float("nan"), device=gpu_device, dtype=torch.float16)
               for _ in range(3))
    lib = K._lib.load()
    pw = K.pack_weight(w)
    print("every element: qkv 768->2304 head-major", flush=True)
    rc = lib.gptmi_linear_qkv(x.data_ptr(), pw.data_ptr(), b.data_ptr(), q.data_ptr(), k.data_ptr(),
                              v.data_ptr(), B, L, heads, d, h, K._lib.GPTMI_W_PACKED, None, 0,
                              K._lib.GPTMI_F16, torch.cuda.current_stream().cuda_stream)
    K._lib.check(rc, "linear_qkv")
    want = (x.float() @ w.float() + b.float()).view(B, L, 3, heads, d)
    for i, (got, nm) in enumerate(((q, "q"), (k, "k"), (v, "v"))):
        assert_all_close_f16(got, want[:, :, i].permute(0, 2, 1, 3).contiguous(), f"qkv {nm}")


def test_batch2048_forward_sampled_sequences(gpu_device):
    """Benchmark configuration 3, max-batch memory point: the 124M forward in fp16 at batch 2048 x
    seqlen 300.  The ffn1 output is 3.8 GB, so row offsets in bytes pass 2^31 (sequence 1165) and
    approach 2^32.  Sequences do not interact: the first, the last, those around the 2^30 and 2^31
    byte marks of the widest activation, and a few spread over the batch are compared with the
    oracle run on those sequences alone."""
    from gpt_triton_amd.gpt import FusedGPT, GPTConfig

    cfg = dict(n_layer=12, n_head=12, n_embd=768, vocab_size=50257, block_size=1024)
    B, L = 2048, 300
    params = O.synthetic_params(**cfg, seed=1337, dtype=np.float16)
    ids = O.synthetic_ids(B, L, cfg["vocab_size"], seed=77)
    model = FusedGPT(GPTConfig(dropout=0.1, **cfg))
    model.load_state_dict({k: torch.from_numpy(v) for k, v in params.items()})
    model = model.to(device=gpu_device, dtype=torch.float16).eval()
    print("forward 2048 x 300", flush=True)
    hidden = model(torch.from_numpy(ids).to(gpu_device))
    assert hidden.shape == (B, L, 768) and bool(torch.isfinite(hidden).all())
    row_2_30 = (1 << 30) // (3072 * 2) // L   # sequence holding byte 2^30 of the ffn1 output
    row_2_31 = (1 << 31) // (3072 * 2) // L
    seqs = sorted({0, 1, row_2_30, row_2_30 + 1, row_2_31 - 1, row_2_31, row_2_31 + 1, 1023, 1024,
                   2046, 2047})
    want = O.gpt2_forward(params, ids[seqs], cfg["n_head"])
    got = hidden[torch.tensor(seqs, device=gpu_device)].cpu().numpy().astype(np.float64)
    err = np.abs(got - want).max(axis=(1, 2))
    print("max|diff| per sampled sequence:", dict(zip(seqs, np.round(err, 5))), flush=True)
    assert err.max() <= 2e-2


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_xl_qkv_split(K, gpu_device, dtype):
    """Benchmark configuration 4's q/k/v product: x [3, 1024, 1600] @ [1600, 4800] + b with 25 heads of
    64 -- N = 4800 is 18 whole 256-column tiles and a 192-column remainder, and a head-major
    scatter whose thirds (1600 columns) do not start on tile boundaries."""
    r = np.random.default_rng(41)
    B, L, heads, d = 3, 1024, 25, 64
    h = heads * d
    npdt = np.float16 if dtype == torch.float16 else np.float32
    x = r.standard_normal((B, L, h)).astype(npdt)
    w = (0.02 * r.standard_normal((h, 3 * h))).astype(npdt)
    b = (0.1 * r.standard_normal(3 * h)).astype(npdt)
    D = lambda a: torch.from_numpy(a).to(gpu_device)
    q, k, v = K.matmul_and_split_qkv(D(x), D(w), D(b), heads)
    wq, wk, wv = O.matmul_and_split_qkv(x, w, b, heads)
    for got, want, nm in ((q, wq, "q"), (k, wk, "k"), (v, wv, "v")):
        assert got.shape == (B, heads, L, d) and got.is_contiguous()
        gotf, wantf = got.cpu().numpy().astype(np.float64), want.astype(np.float64)
        scale = np.abs(wantf).max()
        tol = (2 * 2.0**-10 * scale) if dtype == torch.float16 else (1e-4 * np.abs(wantf) + 1e-4 * scale)
        assert np.all(np.abs(gotf - wantf) <= tol), f"xl qkv {nm} {dtype}"


def test_xl_forward_sampled_sequences(gpu_device):
    """Benchmark configuration 4: the GPT-2 XL-shape forward (48 layers, d_model 1600, 25 heads x 64, FFN
    6400, N(0, 0.02) fp16 weights) at batch 64 x seqlen 1024 -- the tiled attention kernel and the
    GEMM widths that are not multiples of the 256-wide tile -- two sampled sequences against the
    oracle.  The 124M bound of 2e-2 absolute on the final hidden state is kept: the final
    LayerNorm brings the 48-layer residual stream back to unit scale."""
    from gpt_triton_amd.gpt import FusedGPT, GPTConfig

    cfg = dict(n_layer=48, n_head=25, n_embd=1600, vocab_size=50257, block_size=1024)
    B, L = 64, 1024
    params = O.synthetic_params(**cfg, seed=4, dtype=np.float16)
    ids = O.synthetic_ids(B, L, cfg["vocab_size"], seed=4)
    model = FusedGPT(GPTConfig(dropout=0.1, **cfg))
    model.load_state_dict({k: torch.from_numpy(v) for k, v in params.items()})
    model = model.to(device=gpu_device, dtype=torch.float16).eval()
    print("forward xl 64 x 1024", flush=True)
    hidden = model(torch.from_numpy(ids).to(gpu_device))
    assert hidden.shape == (B, L, 1600) and bool(torch.isfinite(hidden).all())
    seqs = [0, 63]
    got = hidden[torch.tensor(seqs, device=gpu_device)].cpu().numpy().astype(np.float64)
    del model, hidden
    torch.cuda.empty_cache()
    want = O.gpt2_forward(params, ids[seqs], cfg["n_head"])
    diff = np.abs(got - want)
    print(f"xl forward: max|diff| {diff.max():.4e}, median {np.median(diff):.3e}, "
          f"max|ref| {np.abs(want).max():.3f}", flush=True)
    assert diff.max() <= 2e-2


@pytest.mark.parametrize("name,cfg,B,L", [
    ("gpt2-medium", dict(n_layer=24, n_head=16, n_embd=1024, vocab_size=50257, block_size=1024), 24, 300),
    ("gpt2-large", dict(n_layer=36, n_head=20, n_embd=1280, vocab_size=50257, block_size=1024), 16, 512),
])
def test_other_gpt2_sizes_forward_sampled_sequences(gpu_device, name, cfg, B, L):
    """The GPT-2 sizes between 124M and XL that the reference's converter loads just the same
    (gpt.py:199-247): 355M (24 x 1024, 16 heads) and 774M (36 x 1280, 20 heads), fp16, enough rows
    for the persistent GEMM kernels with their small-tile tails (7200 / 8192 rows; 1280 and 3840
    are 5 and 15 column tiles, 5120 is 20) and, at L = 512, the long-sequence attention kernel.
    Hidden state and logits of two sampled sequences against the oracle, 2e-2 absolute."""
    from gpt_triton_amd.gpt import FusedGPT, GPTConfig

    params = O.synthetic_params(**cfg, seed=6, dtype=np.float16)
    ids = O.synthetic_ids(B, L, cfg["vocab_size"], seed=6)
    model = FusedGPT(GPTConfig(dropout=0.1, **cfg))
    model.load_state_dict({k: torch.from_numpy(v) for k, v in params.items()})
    model = model.to(device=gpu_device, dtype=torch.float16).eval()
    print(f"forward {name} {B} x {L}", flush=True)
    hidden, logits = model(torch.from_numpy(ids).to(gpu_device), return_logits=True)
    assert hidden.shape == (B, L, cfg["n_embd"]) and bool(torch.isfinite(hidden).all())
    assert logits.shape == (B, L, cfg["vocab_size"]) and bool(torch.isfinite(logits).all())
    seqs = [0, B - 1]
    idx = torch.tensor(seqs, device=gpu_device)
    got_h = hidden[idx].cpu().numpy().astype(np.float64)
    got_l = logits[idx].cpu().numpy().astype(np.float64)
    del model, hidden, logits
    torch.cuda.empty_cache()
    want_h, want_l = O.gpt2_forward(params, ids[seqs], cfg["n_head"], lm_head=True)
    dh, dl = np.abs(got_h - want_h).max(), np.abs(got_l - want_l).max()
    print(f"{name}: hidden max|diff| {dh:.3e}, logits max|diff| {dl:.3e}", flush=True)
    assert dh <= 2e-2 and dl <= 2e-2


def test_headline_logits_every_element(K, gpu_device):
    """Benchmark configurations 0 / 3 ask for logits: the tied LM head at the headline's M = 153600
    rows, hidden states [153600, 768] against wte [50257, 768] through the padded image
    (kernels.pack_lm_head, gpt.py:159-161, 172-179 in the reference).  The padded output is
    153600 x 50304 fp16 = 15.45 GB: element and byte offsets pass 2^31 and 2^32.  The buffer is
    pre-filled with NaN; every logit is compared with the fp32 torch product computed in row
    chunks, the 47 padding columns of every row must be zero, and the rows that hold byte 2^31,
    byte 2^32, element 2^31 and element 2^32 of the padded buffer (with their neighbours), the
    first rows, both sides of the seam between the persistent launch and the small-tile launch
    (152831 | 152832) and the last row are compared with the oracle."""
    V, H, Vp = 50257, 768, 50304
    g = torch.Generator(device=gpu_device).manual_seed(41)
    x = torch.randn((M_HEAD, H), generator=g, device=gpu_device).half()
    wte = (0.02 * torch.randn((V, H), generator=g, device=gpu_device)).half()
    image = K.pack_lm_head(wte)
    buf = torch.full((M_HEAD, Vp), float("nan"), device=gpu_device, dtype=torch.float16)
    print("every element: logits [153600, 50257] through the padded image", flush=True)
    K._linear(x, image, None, None, buf, False, 0.0, K._lib.GPTMI_W_PACKED, "lm_head")
    torch.cuda.synchronize()
    wt = wte.float().t().contiguous()
    n_nan = n_bad = n_pad = 0
    scale = 0.0
    for r0 in range(0, M_HEAD, 4096):
        got = buf[r0:r0 + 4096]
        want = x[r0:r0 + 4096].float() @ wt
        gl = got[:, :V].float()
        n_nan += int(torch.isnan(got).sum())
        n_pad += int((got[:, V:] != 0).sum())
        scale = max(scale, float(want.abs().max()))
        # |b| * 2^-10 (fp16 rounding, with slack for the ordering of the fp32 sums) + a floor
        n_bad += int(((gl - want).abs() > want.abs() * 2.0**-10 + 2.0**-12 * 4.0).sum())
        del got, want, gl
    assert n_nan == 0, f"{n_nan} elements were never written (NaN poison left)"
    assert n_pad == 0, f"{n_pad} padding columns are not zero"
    assert n_bad == 0, f"{n_bad} logits out of tolerance (max|logit| {scale:.3f})"
    row_of = lambda off: off // Vp
    marks = [row_of(2**31 // 2), row_of(2**32 // 2), row_of(2**31), row_of(2**32)]
    rows = sorted({0, 1, 152831, 152832, M_HEAD - 1, *[m + d for m in marks for d in (-1, 0, 1)]})
    assert rows[-1] == M_HEAD - 1 and 85380 in rows and 21345 in rows
    idx = torch.tensor(rows, device=gpu_device)
    want = O.fused_ffn(x[idx].cpu().numpy(), np.ascontiguousarray(wte.cpu().numpy().T))
    got = buf[idx][:, :V].cpu().numpy().astype(np.float64)
    assert np.abs(got - want).max() <= 2 * 2.0**-10 * np.abs(want).max()
