"""gptmi_linear_static -- the entry point that allocates nothing (its packed operand images live
in a device array built into the library) -- against gptmi_linear with a caller workspace.  Both
run the same kernels on the same packed images, so the bar is bit equality.  Each case makes two
calls in a row through the C ABI, the second with a smaller problem, because the array keeps the
first call's bytes.  Collected last (the file name sorts behind the other test files)."""
import ctypes

import pytest
import torch

from gpt_triton_amd import _lib

pytestmark = pytest.mark.gpu

CODE = {torch.float16: _lib.GPTMI_F16, torch.float32: _lib.GPTMI_F32}


def _problem(M, N, K, dtype, device, seed, bias, residual):
    g = torch.Generator(device="cpu").manual_seed(seed)
    rn = lambda *s, std=1.0: (std * torch.randn(*s, generator=g)).to(dtype).to(device)
    return dict(x=rn(M, K), w=rn(K, N, std=0.05), bias=rn(N, std=0.1) if bias else None,
                res=rn(M, N) if residual else None, M=M, N=N, K=K)


def _run(lib, pr, dtype, gelu, static):
    ptr = lambda t: None if t is None else t.data_ptr()
    out = torch.full((pr["M"], pr["N"]), float("nan"), dtype=dtype, device=pr["x"].device)
    stream = torch.cuda.current_stream().cuda_stream
    if static:
        rc = lib.gptmi_linear_static(pr["x"].data_ptr(), pr["w"].data_ptr(), ptr(pr["bias"]),
                                     ptr(pr["res"]), out.data_ptr(), pr["M"], pr["N"], pr["K"],
                                     int(gelu), 0.0, 1337, _lib.GPTMI_W_KN, CODE[dtype], stream)
    else:
        nbytes = lib.gptmi_linear_workspace_bytes(pr["M"], pr["N"], pr["K"], CODE[dtype],
                                                  _lib.GPTMI_W_KN)
        ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=out.device)
        rc = lib.gptmi_linear(pr["x"].data_ptr(), pr["w"].data_ptr(), ptr(pr["bias"]),
                              ptr(pr["res"]), out.data_ptr(), pr["M"], pr["N"], pr["K"], int(gelu),
                              0.0, 1337, _lib.GPTMI_W_KN, ws.data_ptr(), nbytes, CODE[dtype], stream)
    _lib.check(rc, "linear_static" if static else "linear")
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("dtype,first,second", [
    # fp16, K % 64 == 0: the packed weight alone is in the scratch (4.5 MiB, then 1.1 MiB)
    (torch.float16, (2304, 3072, 768), (600, 768, 768)),
    # fp16, K % 64 != 0 and fp32: x is packed into the scratch too, behind the weight
    (torch.float16, (500, 520, 200), (77, 136, 72)),
    (torch.float32, (1200, 768, 768), (130, 257, 65)),
])
def test_linear_static_matches_linear_twice_in_a_row(gpu_device, dtype, first, second):
    lib = _lib.load()
    assert lib.gptmi_linear_static_capacity() == 8 << 20
    for i, (M, N, K) in enumerate((first, second)):
        pr = _problem(M, N, K, dtype, gpu_device, seed=11 + i, bias=True, residual=(i == 1))
        need = lib.gptmi_linear_workspace_bytes(M, N, K, CODE[dtype], _lib.GPTMI_W_KN)
        assert 0 < need <= lib.gptmi_linear_static_capacity()
        print(f"linear_static {dtype} M={M} N={N} K={K} call {i}", flush=True)
        want = _run(lib, pr, dtype, gelu=(i == 0), static=False)
        got = _run(lib, pr, dtype, gelu=(i == 0), static=True)
        assert bool(torch.isfinite(got).all())
        assert torch.equal(got, want), f"call {i}: max|diff| {(got - want).abs().max().item():.3e}"


def test_linear_static_refuses_what_does_not_fit(gpu_device):
    lib = _lib.load()
    fake = ctypes.c_void_p(256)  # never dereferenced: the size check answers first
    # packed [6400][1600] fp16 = 19.5 MiB > 8 MiB
    rc = lib.gptmi_linear_static(fake, fake, None, None, fake, 1024, 6400, 1600, 0, 0.0, 1337,
                                 _lib.GPTMI_W_KN, _lib.GPTMI_F16, None)
    assert rc == -3 and b"scratch" in lib.gptmi_last_error()


def test_linear_static_under_graph_capture(gpu_device):
    """What the entry point is for: after one eager call (which resolves the scratch array's
    address on this device) it runs inside a stream capture, where an allocation or a
    synchronisation would fail the capture; three replays with eager work between them each
    reproduce gptmi_linear bit for bit, and the device's free memory is the same before and after
    an eager call."""
    lib = _lib.load()
    dtype = torch.float16
    pr = _problem(700, 768, 200, dtype, gpu_device, seed=21, bias=True, residual=True)
    want = _run(lib, pr, dtype, gelu=True, static=False)
    assert torch.equal(_run(lib, pr, dtype, gelu=True, static=True), want)
    free0 = torch.cuda.mem_get_info(gpu_device)[0]
    out = torch.full((pr["M"], pr["N"]), float("nan"), dtype=dtype, device=gpu_device)

    def call():
        rc = lib.gptmi_linear_static(pr["x"].data_ptr(), pr["w"].data_ptr(),
                                     pr["bias"].data_ptr(), pr["res"].data_ptr(), out.data_ptr(),
                                     pr["M"], pr["N"], pr["K"], 1, 0.0, 1337, _lib.GPTMI_W_KN,
                                     CODE[dtype], torch.cuda.current_stream().cuda_stream)
        _lib.check(rc, "linear_static")

    call()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(gpu_device)[0] == free0
    side = torch.cuda.Stream(device=gpu_device)
    side.wait_stream(torch.cuda.current_stream(gpu_device))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            call()
    torch.cuda.current_stream(gpu_device).wait_stream(side)
    for i in range(3):
        out.fill_(float("nan"))
        other = pr["x"].float().sum()  # eager work and a synchronisation between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.isfinite(other)
        assert torch.equal(out, want), f"replay {i}"
