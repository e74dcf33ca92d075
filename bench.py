#!/usr/bin/env python3
"""Headline benchmark: GPT-2 124M forward, fp16 storage / fp32 accumulate, batch 512 x seqlen 300,
synthetic N(0, 0.02) weights and uniform token ids, one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one forward pass (hidden state [512, 300, 768], like the reference's forward, which
stops at the final LayerNorm) with the token ids already resident in HBM.  Prints ONE JSON
line.  Beside the whole-forward numbers it carries
  * "roofline": the dominant kernel (the ffn1 GEMM, M=153600 N=3072 K=768, GELU epilogue) timed
    live with events around each of its launches inside the timed region; achieved = 2*M*N*K /
    mean duration against the 2.5 PFLOP/s dense fp16 MFMA peak;
  * "cpu_baseline": the plain PyTorch fp32 forward of the same architecture (the stand-in for the
    reference's CPU-side comparator, HF GPT2Model in fp32) on this box's host cores, on a
    bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

BATCH, SEQLEN = 512, 300
ARCH = dict(vocab_size=50257, block_size=1024, n_layer=12, n_head=12, n_embd=768)
PEAK_FP16 = 2.5e15       # MI355X dense fp16 MFMA, FLOP/s
FFN1 = dict(M=BATCH * SEQLEN, N=3072, K=768)
# HBM-side bytes of one ffn1 launch from rocprofv3 --pmc FETCH_SIZE (890.7 MB after scaling by
# the copy kernel of --traffic-calibration) + WRITE_SIZE (943.7 MB); the counters cannot be read
# from inside this process, so the figure is the one of profiles/gemm_ffn1_hbm_traffic_pmc.md
FFN1_TRAFFIC_BYTES = 1.834e9


def forward_flops(tokens, seqlen):
    """Executed FLOPs of one forward without LM head: the four GEMMs per layer plus the causal
    half of the attention products."""
    h, L = ARCH["n_embd"], ARCH["n_layer"]
    gemm = 2 * tokens * h * (3 * h + h + 4 * h + 4 * h)
    attn = 4 * (tokens // seqlen) * ARCH["n_head"] * (h // ARCH["n_head"]) * seqlen * (seqlen + 1) // 2
    return L * (gemm + attn)


def cpu_baseline(sample_batch=16, reps=2):
    import numpy as np
    import torch

    from oracle import gpt2_oracle as O
    from oracle.torch_fp32 import gpt2_forward_fp32

    cores = os.cpu_count() or 1
    threads = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(threads)
    params = {k: torch.from_numpy(v) for k, v in O.synthetic_params(
        ARCH["n_layer"], ARCH["n_head"], ARCH["n_embd"], ARCH["vocab_size"], ARCH["block_size"],
        seed=1337).items()}
    ids = torch.from_numpy(O.synthetic_ids(sample_batch, SEQLEN, ARCH["vocab_size"], seed=1337))
    gpt2_forward_fp32(params, ids, ARCH["n_head"])  # warm-up
    t0 = time.perf_counter()
    for _ in range(reps):
        gpt2_forward_fp32(params, ids, ARCH["n_head"])
    dt = (time.perf_counter() - t0) / reps
    return {"value": round(sample_batch * SEQLEN / dt, 1), "unit": "tokens/s", "cores": threads,
            "kind": "port",
            "sample": f"PyTorch fp32 eager forward of the same 124M model on the host CPU, batch "
                      f"{sample_batch} x seqlen {SEQLEN} ({sample_batch * SEQLEN} tokens), "
                      f"mean of {reps} after 1 warm-up, {dt * 1e3:.0f} ms per forward"}


def copy_calibration(dev, rows=262144, cols=2048, reps=3):
    """pack_rows_kernel on an fp16 [rows][cols] matrix whose width is already a multiple of 64
    is an element-for-element copy: rows*cols*2 bytes read, the same written."""
    import torch

    from gpt_triton_amd import _lib

    lib = _lib.load()
    src = torch.randn(rows, cols, device=dev, dtype=torch.float16)
    dst = torch.empty(lib.gptmi_packed_weight_bytes(rows, cols), dtype=torch.uint8, device=dev)
    assert dst.numel() == src.numel() * 2
    for _ in range(reps):
        _lib.check(lib.gptmi_pack_weight(src.data_ptr(), dst.data_ptr(), rows, cols,
                                         _lib.GPTMI_W_NK, _lib.GPTMI_F16,
                                         torch.cuda.current_stream().cuda_stream), "copy calibration")
    torch.cuda.synchronize()
    assert torch.equal(dst.view(torch.float16).view(rows, cols), src)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true",
                    help="skip the host-CPU leg (used under rocprofv3)")
    ap.add_argument("--traffic-calibration", action="store_true",
                    help="also launch a plain copy kernel of known size (1 GiB read, 1 GiB "
                         "written) so that FETCH_SIZE / WRITE_SIZE counters of the same "
                         "rocprofv3 --pmc run can be scaled to bytes")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU's full share of the forward; "
                 "--gpus must be 1 (the path shards over the batch with no exchange, see DESIGN.md)")

    import torch

    from gpt_triton_amd import gpt as G
    from gpt_triton_amd import kernels as K

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    cfg = G.GPTConfig(dropout=0.1, **ARCH)
    model = G.FusedGPT(cfg).init_synthetic_(seed=1337).to(device=dev, dtype=torch.float16).eval()
    gen = torch.Generator(device="cpu").manual_seed(1338)
    ids = torch.randint(0, ARCH["vocab_size"], (BATCH, SEQLEN), generator=gen).to(dev)

    # events around every ffn1 launch (the GELU GEMM) on the stream it is launched on
    ffn1_events = []
    inner = K.fused_ffn

    def timed_ffn(x, weight, bias=None, residual=None, add_gelu=False, dropout_prob=0.0):
        if not (add_gelu and recording[0]):
            return inner(x, weight, bias, residual, add_gelu, dropout_prob)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        out = inner(x, weight, bias, residual, add_gelu, dropout_prob)
        e1.record()
        ffn1_events.append((e0, e1))
        return out

    recording = [False]
    G.fused_ffn = timed_ffn

    with torch.no_grad():
        for _ in range(args.warmup):
            model(ids)
        torch.cuda.synchronize()
        recording[0] = True
        t0 = time.perf_counter()
        for _ in range(args.steps):
            out = model(ids)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
    recording[0] = False
    assert out.shape == (BATCH, SEQLEN, ARCH["n_embd"]) and bool(torch.isfinite(out).all())

    ms = dt / args.steps * 1e3
    tokens = BATCH * SEQLEN
    flops = forward_flops(tokens, SEQLEN)
    ffn1_ms = sum(a.elapsed_time(b) for a, b in ffn1_events) / max(1, len(ffn1_events))
    ffn1_flops = 2 * FFN1["M"] * FFN1["N"] * FFN1["K"]
    achieved = ffn1_flops / (ffn1_ms * 1e-3) / 1e12

    line = {
        "metric": "gpt2_124m_forward_tokens_per_s",
        "baseline_metric": "GPT-2 124M fwd ms @512x300 fp16; tokens/s; MFU vs MI355X peak",
        "value": round(tokens / (ms * 1e-3), 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms, 3),
        "higher_is_better": True,
        "scaling": "weak",
        # the reference's published number for this forward is 273 ms on one A100-40GB
        # (README.md:17, bench.py:87-89); other hardware, so reported as a ratio of step times
        "vs_baseline": round(273.0 / ms, 3),
        "vs_baseline_ref": "273 ms, gpt-triton mixed fp16, 1x A100 40GB (README.md:17)",
        "dtype": "f16",
        "data": "synthetic",
        "mfu": round(flops / (ms * 1e-3) / PEAK_FP16, 4),
        "mfu_flops": flops,
        "mfu_note": "executed FLOPs without LM head (GEMMs + causal attention) / 2.5 PFLOP/s",
        "config": {"workload": "GPT-2 124M forward, fp16 storage / fp32 accumulate, batch 512 x "
                               "seqlen 300, hidden-state output (no LM head)",
                   "tokens_per_step": tokens, "n_layer": 12, "n_embd": 768, "n_head": 12},
        "roofline": {"kernel": "gemm_kernel (ffn1: M=153600 N=3072 K=768, bias+GELU epilogue)",
                     "bound": "mfma", "achieved": round(achieved, 1), "peak": PEAK_FP16 / 1e12,
                     "unit": "TFLOP/s", "frac": round(achieved * 1e12 / PEAK_FP16, 4),
                     "avg_ms": round(ffn1_ms, 4), "launches": len(ffn1_events),
                     "traffic": FFN1_TRAFFIC_BYTES},
    }
    line["cpu_baseline"] = None if args.no_cpu_baseline else cpu_baseline()
    if args.traffic_calibration:
        copy_calibration(dev)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
