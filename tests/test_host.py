"""Host-side checks that need no GPU: the C-ABI library loads and exports exactly what
include/gptmi.h declares, argument validation answers before any launch, the model helpers
reproduce the reference's known answers (test.py:136-152), and CPU tensors are refused."""
import ctypes
import os
import re

import pytest
import torch

from gpt_triton_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_lib.LIB_PATH):
        from gpt_triton_amd import build

        build.build()
    return _lib.load()


def declared_functions():
    text = open(os.path.join(ROOT, "include", "gptmi.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gptmi_[a-z_0-9]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound(lib):
    names = declared_functions()
    assert len(names) >= 11
    for name in names:
        assert hasattr(lib, name), f"{name} declared in gptmi.h but not exported"
    assert sorted(_lib.SIGNATURES) == names, "ctypes prototypes and gptmi.h disagree"


def test_version_and_error_string(lib):
    assert lib.gptmi_version() == 102
    assert isinstance(lib.gptmi_last_error(), bytes)


def test_invalid_arguments_are_rejected_before_any_launch(lib):
    # NULL pointers / bad sizes -> GPTMI_ERR_INVALID (-1); none of these touches the GPU
    assert lib.gptmi_embed(None, None, None, None, 1, 1, 1, 1, 1, 0.0, 0, 1, None) == -1
    assert lib.gptmi_layernorm(None, None, None, None, 4, 4, 1e-5, 1, None) == -1
    assert lib.gptmi_softmax(None, None, 4, 4, 0, None) == -1
    assert lib.gptmi_linear(None, None, None, None, None, 1, 1, 1, 0, 0.0, 0, 0, None, 0, 1, None) == -1
    assert lib.gptmi_flash_attn(None, None, None, None, 1, 1, 1, 1, 64, 0.125, 0.0, 0, 0, 1, None) == -1
    fake = ctypes.c_void_p(256)  # never dereferenced: validation fails first
    assert lib.gptmi_layernorm(fake, fake, fake, fake, 4, 4, 1e-5, 7, None) == -1       # bad dtype
    assert lib.gptmi_layernorm(fake, fake, fake, fake, 4, 10000, 1e-5, 1, None) == -2   # H too large
    assert b"8192" in lib.gptmi_last_error()
    assert lib.gptmi_embed(fake, fake, fake, fake, 1, 8, 4, 4, 8, 0.0, 0, 1, None) == -1  # L > P
    assert lib.gptmi_embed(fake, fake, fake, fake, 1, 4, 4, 4, 8, 1.0, 0, 1, None) == -1  # p >= 1
    assert lib.gptmi_flash_attn(fake, fake, fake, fake, 1, 1, 8, 8, 64, 0.125, -0.1, 0, 0, 1,
                                None) == -1                                             # p < 0
    assert lib.gptmi_flash_attn(fake, fake, fake, fake, 1, 1, 8, 9, 48, 0.125, 0.0, 0, 0, 1,
                                None) == -2                                             # head size
    # output rows wider than the epilogues' 32-bit lane offsets can address: refused, not wrapped
    wide = (1 << 26) + 8
    assert lib.gptmi_linear(fake, fake, None, None, fake, 4, wide, 64, 0, 0.0, 0, 2, None, 0, 1,
                            None) == -2
    assert b"N=" in lib.gptmi_last_error()
    assert lib.gptmi_linear_static(fake, fake, None, None, fake, 4, wide, 64, 0, 0.0, 0, 2, 1,
                                   None) == -2
    assert lib.gptmi_linear_qkv(fake, fake, None, fake, fake, fake, 1, 4, 1 << 20, 64, 64, 2,
                                None, 0, 1, None) == -2                    # N = 3 * 2^26
    assert lib.gptmi_linear(fake, fake, None, None, fake, 4, 4, 4, 0, 0.0, 0, 0, None, 0, 1,
                            None) == -3                                                 # workspace


def test_workspace_sizes(lib):
    # fp16, K multiple of 64, [K][N] weight: only the packed weight (N * K * 2 bytes)
    assert lib.gptmi_linear_workspace_bytes(153600, 3072, 768, 1, 0) == 3072 * 768 * 2
    # already [N][K] fp16: nothing to pack
    assert lib.gptmi_linear_workspace_bytes(153600, 50257, 768, 1, 1) == 0
    assert lib.gptmi_linear_workspace_bytes(153600, 3072, 768, 1, 2) == 0
    # fp32 storage: weight and activations are both repacked to fp16
    assert lib.gptmi_linear_workspace_bytes(128, 64, 64, 0, 0) == 64 * 64 * 2 + 128 * 64 * 2
    # K = 23 pads to 64
    assert lib.gptmi_packed_weight_bytes(31, 23) == 31 * 64 * 2 + (256 - 31 * 64 * 2 % 256) % 256


def test_flops_known_answers():
    # test.py:136-144
    from gpt_triton_amd.gpt import FusedGPT, GPTConfig, get_num_parameters

    model = FusedGPT(GPTConfig()).eval()
    fwd = model.get_fwd_flops(1024)
    n = get_num_parameters(model)
    assert fwd == 253997088768 and n == 124082688
    assert (fwd * 3) / (6 * n * 1024) >= 0.9995


def test_estimate_days_known_answer():
    # test.py:147-152
    from gpt_triton_amd.gpt import compute_mfu, estimate_days

    flops = 6 * (405 * 10**9) * (15 * 10**12)
    assert estimate_days(flops, mfu=0.45, gpu="h100", num_gpus=16_000) == 59.24544994944388
    assert compute_mfu(2 * 124 * 10**6 * 512 * 512 / 0.273, gpu="h100") == pytest.approx(0.2407, abs=2e-4)
    assert compute_mfu(1.0e15, gpu="mi355x") == pytest.approx(0.4)


def test_state_dict_keys_match_the_reference_layout():
    from gpt_triton_amd.gpt import FusedGPT, GPTConfig

    keys = set(FusedGPT(GPTConfig(n_layer=2)).state_dict())
    want = {"wte_weight", "wpe_weight", "layer_norm_weight", "layer_norm_bias"}
    for i in range(2):
        for k in ("layer_norm_weight", "layer_norm_bias", "c_attn_weight", "c_attn_bias",
                  "c_proj_weight", "c_proj_bias"):
            want.add(f"blocks.{i}.0.{k}")
        for k in ("layer_norm_weight", "layer_norm_bias", "ffn1_weight", "ffn1_bias", "ffn2_weight",
                  "ffn2_bias"):
            want.add(f"blocks.{i}.1.{k}")
    assert keys == want


def test_hf_key_conversion():
    from types import SimpleNamespace

    from gpt_triton_amd.gpt import FusedGPT, convert_huggingface_to_triton

    cfg = SimpleNamespace(vocab_size=11, n_positions=8, n_layer=1, n_head=2, n_embd=4)
    h = 4
    hf = {"wte.weight": torch.zeros(11, h), "wpe.weight": torch.zeros(8, h),
          "ln_f.weight": torch.ones(h), "ln_f.bias": torch.zeros(h),
          "h.0.ln_1.weight": torch.ones(h), "h.0.ln_1.bias": torch.zeros(h),
          "h.0.attn.bias": torch.ones(1, 1, 8, 8),
          "h.0.attn.c_attn.weight": torch.zeros(h, 3 * h), "h.0.attn.c_attn.bias": torch.zeros(3 * h),
          "h.0.attn.c_proj.weight": torch.zeros(h, h), "h.0.attn.c_proj.bias": torch.zeros(h),
          "h.0.ln_2.weight": torch.ones(h), "h.0.ln_2.bias": torch.zeros(h),
          "h.0.mlp.c_fc.weight": torch.zeros(h, 4 * h), "h.0.mlp.c_fc.bias": torch.zeros(4 * h),
          "h.0.mlp.c_proj.weight": torch.zeros(4 * h, h), "h.0.mlp.c_proj.bias": torch.zeros(h)}
    sd, config = convert_huggingface_to_triton(hf, cfg)
    assert config.block_size == 8 and config.n_head == 2
    FusedGPT(config).load_state_dict(sd)  # every key present, none extra


def test_cpu_tensors_are_refused_not_emulated(lib):
    from gpt_triton_amd import kernels as K

    x = torch.zeros(4, 64)
    w = torch.zeros(64, 64)
    with pytest.raises(RuntimeError, match="GPU only"):
        K.fused_ffn(x, w)
    with pytest.raises(RuntimeError, match="GPU only"):
        K.fused_layer_norm(x, torch.ones(64), torch.zeros(64))
    with pytest.raises(RuntimeError, match="GPU only"):
        K.fused_embeddings(torch.zeros(2, 3, dtype=torch.long), w, w)
    q = torch.zeros(1, 1, 8, 64)
    with pytest.raises(RuntimeError, match="GPU only"):
        K.flash_attention_v1(q, q, q)


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys

    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True)
    assert r.returncode != 0 and "--gpus must be 1" in r.stderr
