"""GPU parity of the attention kernel the headline forward runs on: fp16, head size 64, equal
query and key lengths <= 320 and at least 64 (batch, head) pairs -- with fewer pairs, other head
sizes or fp32 storage `flash_attention_v1` picks other kernels, which tests/test_gpu_parity.py
covers.  Here every call has B * N >= 64:

  * every length either side of the 32-query chunk and 64-key tile boundaries, from 1 to the
    longest the kernel takes, both output layouts, against the oracle;
  * pair counts below, between multiples of and above the number of persistent workgroups;
  * the reference's own outputs (tests/golden/flash_attention_v1.npz, written by the reference's
    kernel under Triton's CPU interpreter) placed among random pairs, so that the reference's
    vectors are compared on this kernel and not only on the few-pair ones;
  * the benchmark shape [512, 12, 300, 64]: every element of every pair against the textbook
    attention evaluated by torch in fp32 on the GPU, the output pre-filled with NaN; the same
    check at the same bytes for head sizes 128 and 256 ([512, 6, 300, 128], [512, 3, 300, 256]),
    which run on the wide-head kernel.

Follows the reference's kernel and test: kernels.py:375-474, test.py:90-117.  Everything goes
through ctypes -> libgptmi.so.  Tolerances: against the oracle, fp16 storage as everywhere
(2 fp16 ulps of max|b|); against the fp32 torch attention, the bound that the reference's two
roundings allow, stated in `attention_bound`."""
import math
import os

import numpy as np
import pytest
import torch

from oracle import gpt2_oracle as O

pytestmark = pytest.mark.gpu

D = 64
ULP2 = 2 * 2.0**-10


@pytest.fixture(scope="module")
def K(gpu_device):
    from gpt_triton_amd import kernels

    return kernels


def dev(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def host(t):
    return t.detach().cpu().numpy()


def gaussian_qkv(B, N, L, seed):
    r = np.random.default_rng(seed)
    return tuple(r.standard_normal((B, N, L, D)).astype(np.float16) for _ in range(3))


def check_f16(got, want, what):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    assert np.all(np.isfinite(got)), f"{what}: non-finite output"
    scale = np.abs(want).max()
    diff = np.abs(got - want)
    assert diff.max() <= ULP2 * scale, (f"{what}: max|diff| {diff.max():.3e} at "
                                        f"{np.unravel_index(np.argmax(diff), diff.shape)}, "
                                        f"tolerance {ULP2 * scale:.3e}")


def both_layouts(K, q, k, v, device):
    args = [dev(t, device) for t in (q, k, v)]
    z = K.flash_attention_v1(*args)
    assert z.shape == q.shape and z.dtype == torch.float16 and z.is_contiguous()
    zm = K.flash_attention_v1(*args, merged_heads_layout=True)
    assert zm.shape == q.shape and zm.transpose(1, 2).is_contiguous()
    return host(z), host(zm)


LENGTHS = [1, 2, 31, 32, 33, 63, 64, 65, 95, 96, 97, 127, 128, 129, 191, 192, 193, 255, 256, 257,
           299, 300, 319, 320]


@pytest.mark.parametrize("L", LENGTHS)
def test_stream_attention_lengths(K, gpu_device, L):
    """72 pairs (fewer than persistent workgroups: one pair each), every boundary length."""
    B, N = 6, 12
    q, k, v = gaussian_qkv(B, N, L, seed=1000 + L)
    print(f"stream attention: B={B} N={N} L={L}", flush=True)
    z, zm = both_layouts(K, q, k, v, gpu_device)
    want = O.flash_attention_v1(q, k, v)
    check_f16(z, want, f"L={L} [B,N,L,d]")
    check_f16(zm, want, f"L={L} [B,L,N,d]")
    assert np.array_equal(z, zm)
    # query 0 sees key 0 only: its output is v[0] exactly
    assert np.array_equal(z[:, :, 0], v[:, :, 0])


@pytest.mark.parametrize("B,N", [(8, 8), (25, 12), (27, 19), (64, 12)])
@pytest.mark.parametrize("L", [77, 300])
def test_stream_attention_pair_counts(K, gpu_device, B, N, L):
    """64 pairs (the fewest the kernel is picked for), 300 (some workgroups walk two pairs, most
    one), 513 (two rounds and one pair of a third) and 768 (three whole rounds on 256 CUs):
    every pair against the oracle."""
    q, k, v = gaussian_qkv(B, N, L, seed=B * N + L)
    print(f"stream attention: B={B} N={N} ({B * N} pairs) L={L}", flush=True)
    z, zm = both_layouts(K, q, k, v, gpu_device)
    want = O.flash_attention_v1(q, k, v)
    check_f16(z, want, f"{B * N} pairs [B,N,L,d]")
    check_f16(zm, want, f"{B * N} pairs [B,L,N,d]")
    assert np.array_equal(z[:, :, 0], v[:, :, 0])


@pytest.mark.parametrize("case,heads", [("a", 3), ("c", 1)])
def test_stream_attention_reference_golden_vectors(K, gpu_device, case, heads):
    """The reference's own outputs for cases `a` ([1, 3, 150, 64]) and `c` ([1, 1, 300, 64]) of
    tests/golden/flash_attention_v1.npz: its (batch, head) pairs are placed at the first, a
    middle and the last positions of a [7, 11] grid of otherwise random pairs (77 pairs), so the
    call runs on the many-pair kernel; pairs are independent, so those positions must reproduce
    the reference's vectors."""
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "flash_attention_v1.npz"))
    gq, gk, gv, gout = (g[f"{case}_{t}"] for t in ("q", "k", "v", "out"))
    L = gq.shape[2]
    B, N = 7, 11
    q, k, v = gaussian_qkv(B, N, L, seed=77)
    spots = [(0, 0), (3, 5), (6, 10)]
    for i, (b, n) in enumerate(spots):
        h = i % heads
        q[b, n], k[b, n], v[b, n] = gq[0, h], gk[0, h], gv[0, h]
    print(f"stream attention: golden case {case} among {B * N} pairs, L={L}", flush=True)
    z, zm = both_layouts(K, q, k, v, gpu_device)
    for i, (b, n) in enumerate(spots):
        h = i % heads
        check_f16(z[b, n], gout[0, h], f"golden {case} head {h} at ({b},{n}) [B,N,L,d]")
        check_f16(zm[b, n], gout[0, h], f"golden {case} head {h} at ({b},{n}) [B,L,N,d]")
    check_f16(z, O.flash_attention_v1(q, k, v), f"golden {case}: the random pairs around it")


def attention_bound(q, k, v, scale):
    """Textbook causal attention of fp16 q, k, v in fp32 (torch, on the GPU) and the elementwise
    bound on |kernel - textbook| that the reference's arithmetic allows: the weights P are
    rounded to fp16 before P.V (kernels.py:466: each weight moves by at most 2^-11 of itself,
    so the output by at most 2^-11 * sum_j P_j |v_j| / sum_j P_j) and the output is rounded to
    fp16 (2^-11 |b|); fp32 summation order and the exp2-based exponential add ~1e-6 relative,
    covered by the slack term."""
    L = q.shape[2]
    s = torch.matmul(q.float(), k.float().transpose(-1, -2)) * scale
    mask = torch.ones((L, L), dtype=torch.bool, device=q.device).tril()
    s = s.masked_fill(~mask, float("-inf"))
    p = torch.softmax(s, dim=-1)
    want = torch.matmul(p, v.float())
    spread = torch.matmul(p, v.float().abs())
    tol = 2.0**-11 * want.abs() + 2.0**-11 * spread + 2e-5 * spread + 1e-6
    return want, tol


@pytest.mark.parametrize("layout", ["BNLD", "BLND"])
def test_headline_attention_every_element(K, gpu_device, layout):
    """Benchmark configuration 2, q, k, v [512, 12, 300, 64] fp16: all 6144 pairs, every element,
    through gptmi_flash_attn with a NaN-filled output, in the reference's layout and in the
    merged-heads layout the model uses."""
    B, N, L = 512, 12, 300
    g = torch.Generator(device=gpu_device).manual_seed(2)
    q, k, v = (torch.randn((B, N, L, D), generator=g, device=gpu_device).half() for _ in range(3))
    shape = (B, N, L, D) if layout == "BNLD" else (B, L, N, D)
    out = torch.full(shape, float("nan"), device=gpu_device, dtype=torch.float16)
    lib = K._lib.load()
    print(f"every element: attention [512, 12, 300, 64] output {layout}", flush=True)
    code = K._lib.GPTMI_O_BNLD if layout == "BNLD" else K._lib.GPTMI_O_BLND
    rc = lib.gptmi_flash_attn(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), B, N, L, L,
                              D, 1 / math.sqrt(D), 0.0, 1337, code, K._lib.GPTMI_F16,
                              torch.cuda.current_stream().cuda_stream)
    K._lib.check(rc, "flash_attn")
    z = out if layout == "BNLD" else out.transpose(1, 2)
    assert int(torch.isnan(z).sum()) == 0, "elements never written (NaN poison left)"
    n_bad, worst = 0, 0.0
    for b0 in range(0, B, 32):
        sl = slice(b0, b0 + 32)
        want, tol = attention_bound(q[sl], k[sl], v[sl], 1 / math.sqrt(D))
        excess = (z[sl].float() - want).abs() - tol
        n_bad += int((excess > 0).sum())
        worst = max(worst, float(excess.max()))
    assert n_bad == 0, f"{n_bad} elements beyond the rounding bound (worst excess {worst:.3e})"
    assert torch.equal(z[:, :, 0], v[:, :, 0])


@pytest.mark.parametrize("N,d", [(6, 128), (3, 256)])
def test_wide_head_attention_every_element(K, gpu_device, N, d):
    """The headline's bytes at head sizes 128 and 256 (the shapes `bench.py --workload ops`
    times): every element against the textbook attention in fp32, NaN-filled output, merged-heads
    layout (the one with the strided rows)."""
    B, L = 512, 300
    g = torch.Generator(device=gpu_device).manual_seed(d)
    q, k, v = (torch.randn((B, N, L, d), generator=g, device=gpu_device).half() for _ in range(3))
    out = torch.full((B, L, N, d), float("nan"), device=gpu_device, dtype=torch.float16)
    lib = K._lib.load()
    print(f"every element: attention [512, {N}, 300, {d}]", flush=True)
    rc = lib.gptmi_flash_attn(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), B, N, L, L,
                              d, 1 / math.sqrt(d), 0.0, 1337, K._lib.GPTMI_O_BLND, K._lib.GPTMI_F16,
                              torch.cuda.current_stream().cuda_stream)
    K._lib.check(rc, "flash_attn")
    z = out.transpose(1, 2)
    assert int(torch.isnan(z).sum()) == 0, "elements never written (NaN poison left)"
    n_bad, worst = 0, 0.0
    for b0 in range(0, B, 32):
        sl = slice(b0, b0 + 32)
        want, tol = attention_bound(q[sl], k[sl], v[sl], 1 / math.sqrt(d))
        excess = (z[sl].float() - want).abs() - tol
        n_bad += int((excess > 0).sum())
        worst = max(worst, float(excess.max()))
    assert n_bad == 0, f"{n_bad} elements beyond the rounding bound (worst excess {worst:.3e})"
    assert torch.equal(z[:, :, 0], v[:, :, 0])
