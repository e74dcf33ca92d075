#!/usr/bin/env python3
"""Headline benchmark: GPT-2 124M forward, fp16 storage / fp32 accumulate, batch 512 x seqlen 300,
synthetic N(0, 0.02) weights and uniform token ids, one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]
                    [--workload headline|batch2048|xl|config0|ops] [--lm-head]

The default (and the only line the contract asks for) is `headline`; `batch2048` is the same model
at the max-batch memory point 2048 x 300, `xl` the GPT-2 XL shape (48 x 1600, 25 heads, batch 64 x
seqlen 1024), `config0` the same model at 2 x 64 tokens (bound by its launches; `--graph` times
replays of the captured forward, `--no-ln-prologue` runs the LayerNorms as launches of their own),
`ops` times the single operators at the headline sizes (mean and median of event-timed
repetitions, one JSON line).  `--lm-head` adds the tied LM head (logits) to the step.

A step is one forward pass (hidden state [512, 300, 768], like the reference's forward, which
stops at the final LayerNorm) with the token ids already resident in HBM.  Prints ONE JSON
line.  Beside the whole-forward numbers it carries
  * "roofline": the dominant kernel (the ffn1 GEMM, M=153600 N=3072 K=768, GELU epilogue) timed
    live with events around each of its calls inside the timed region (a call is one launch of
    the persistent kernel plus, at this shape, one of the small-tile kernel for the last 768
    rows); achieved = 2*M*N*K / mean duration against the 2.5 PFLOP/s dense fp16 MFMA peak;
  * "cpu_baseline": the plain PyTorch fp32 forward of the same architecture (the stand-in for the
    reference's CPU-side comparator, HF GPT2Model in fp32) on this box's host cores, at the
    same 512 x 300 batch (1 warm-up + 3 timed forwards, about two minutes on 16 cores;
    `--cpu-sample-batch 64` bounds it for profile runs).
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
ARCH_XL = dict(vocab_size=50257, block_size=1024, n_layer=48, n_head=25, n_embd=1600)
WORKLOADS = {  # name -> (architecture, batch, seqlen, description)
    "headline": (ARCH, 512, 300, "GPT-2 124M forward, fp16 storage / fp32 accumulate, batch 512 x "
                                 "seqlen 300"),
    "batch2048": (ARCH, 2048, 300, "GPT-2 124M forward, fp16 storage / fp32 accumulate, batch 2048 "
                                   "x seqlen 300 (max-batch memory point)"),
    "xl": (ARCH_XL, 64, 1024, "GPT-2 XL-shape forward (48 layers, d_model 1600, 25 heads x 64, FFN "
                              "6400), fp16 storage / fp32 accumulate, batch 64 x seqlen 1024"),
}
WORKLOADS["config0"] = (ARCH, 2, 64, "GPT-2 124M forward, fp16 storage / fp32 accumulate, batch 2 x "
                                     "seqlen 64 (the size of the reference's CPU-runnable case: "
                                     "bound by its launches)")
PEAK_FP16 = 2.5e15       # MI355X dense fp16 MFMA, FLOP/s
PEAK_HBM = 8.0e12        # bytes/s
# HBM-side bytes of one ffn1 call come from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs (scaled
# by the copy kernel of --traffic-calibration); the counters cannot be read from inside this
# process, so the figure is the one the profile summary states in its `ffn1_call_hbm_bytes:` line
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "gemm_ffn1_hbm_traffic_pmc.md")


def ffn1_traffic_bytes():
    """The `ffn1_call_hbm_bytes: <number>` line of the traffic profile, or None without it."""
    try:
        for line in open(TRAFFIC_PROFILE):
            if line.startswith("ffn1_call_hbm_bytes:"):
                return float(line.split(":", 1)[1].split()[0])
    except (OSError, ValueError):
        pass
    return None


def forward_flops(tokens, seqlen, arch=ARCH, lm_head=False):
    """Executed FLOPs of one forward: the four GEMMs per layer plus the causal half of the
    attention products (+ the tied LM head when asked for)."""
    h, L = arch["n_embd"], arch["n_layer"]
    gemm = 2 * tokens * h * (3 * h + h + 4 * h + 4 * h)
    attn = 4 * (tokens // seqlen) * arch["n_head"] * (h // arch["n_head"]) * seqlen * (seqlen + 1) // 2
    return L * (gemm + attn) + (2 * tokens * h * arch["vocab_size"] if lm_head else 0)


def cpu_model_name():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown CPU"


def cpu_baseline(sample_batch=BATCH, reps=3):
    """PyTorch fp32 eager forward of the same 124M model on the host cores: 1 warm-up + `reps`
    timed forwards of `sample_batch` x 300 tokens (the whole 512 x 300 step by default: about
    30 s per forward on 16 cores)."""
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
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        gpt2_forward_fp32(params, ids, ARCH["n_head"])
        times.append(time.perf_counter() - t0)
    mean, best = sum(times) / reps, min(times)
    tokens = sample_batch * SEQLEN
    return {"value": round(tokens / mean, 1), "unit": "tokens/s", "cores": threads,
            "kind": "port", "cpu_model": cpu_model_name(), "logical_cores": cores,
            "cpu_ms_mean": round(mean * 1e3, 1), "cpu_ms_min": round(best * 1e3, 1),
            "cpu_tokens_per_s_best": round(tokens / best, 1),
            "sample": f"PyTorch fp32 eager forward of the same 124M model on the host CPU "
                      f"({threads} torch threads), batch {sample_batch} x seqlen {SEQLEN} "
                      f"({tokens} tokens" + ("" if sample_batch == BATCH else f"; the full 512 x 300 step would take ~{mean * BATCH / sample_batch:.0f} s") + "), "
                      f"1 warm-up + {reps} timed forwards: mean {mean * 1e3:.0f} ms, min {best * 1e3:.0f} ms"}


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


def time_op(fn, flush=None, min_ms=100.0, warm_ms=25.0):
    """Mean and median duration (ms) of fn() from one event pair per repetition, after at
    least warm_ms of warm-up and over at least min_ms of repetitions; `flush` (a callable) runs
    before every repetition, outside the timed pair, to push the operands out of L2 / the
    memory-side cache for the bandwidth-bound operators."""
    import torch

    def once():
        if flush is not None:
            flush()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        return e0, e1

    e0, e1 = once()
    torch.cuda.synchronize()
    est = max(e0.elapsed_time(e1), 1e-3)
    for _ in range(max(1, int(warm_ms / est))):
        once()
    pairs = [once() for _ in range(max(5, int(min_ms / est)))]
    torch.cuda.synchronize()
    ts = sorted(a.elapsed_time(b) for a, b in pairs)
    return sum(ts) / len(ts), ts[len(ts) // 2], len(ts)


def bench_ops(dev):
    """Single operators at the headline sizes (M = 512 * 300 tokens)."""
    import torch

    from gpt_triton_amd import kernels as K

    M, h = BATCH * SEQLEN, 768
    g = torch.Generator(device=dev).manual_seed(1337)
    rn = lambda *shape, std=1.0: (std * torch.randn(*shape, device=dev, generator=g)).half()
    x, x4 = rn(M, h), rn(M, 4 * h)
    w1, b1 = K.pack_weight(rn(h, 4 * h, std=0.02)), rn(4 * h, std=0.02)
    w2, b2 = K.pack_weight(rn(4 * h, h, std=0.02)), rn(h, std=0.02)
    wq, bq = K.pack_weight(rn(h, 3 * h, std=0.02)), rn(3 * h, std=0.02)
    wo, bo = K.pack_weight(rn(h, h, std=0.02)), rn(h, std=0.02)
    lw, lb = torch.ones(h, device=dev).half(), torch.zeros(h, device=dev).half()
    q, k, v = (rn(BATCH, 12, SEQLEN, 64) for _ in range(3))
    ids = torch.randint(0, ARCH["vocab_size"], (BATCH, SEQLEN), device=dev, generator=g)
    wte, wpe = rn(ARCH["vocab_size"], h, std=0.02), rn(1024, h, std=0.02)
    # all-zero operands: the same instructions on data that toggles no bits -- what the schedule
    # alone allows when the chip's power management has no reason to lower the clock
    xz, x4z = torch.zeros_like(x), torch.zeros_like(x4)
    w1z, w2z = K.pack_weight(torch.zeros(h, 4 * h, device=dev).half()), K.pack_weight(torch.zeros(4 * h, h, device=dev).half())
    wqz = K.pack_weight(torch.zeros(h, 3 * h, device=dev).half())
    b1z, b2z, bqz = torch.zeros_like(b1), torch.zeros_like(b2), torch.zeros_like(bq)
    spill = torch.empty(1 << 29, dtype=torch.uint8, device=dev)  # 512 MB > L2 + memory-side cache
    flush = lambda: spill.add_(1)
    gemm = lambda n, k_: 2 * M * n * k_
    ops = [
        ("ffn1 768->3072 +bias+GELU", lambda: K.fused_ffn(x, w1, bias=b1, add_gelu=True), gemm(3072, 768), None, None),
        # the same products with parts of the epilogue left out: the differences are what the
        # bias, the GELU and the residual cost
        ("ffn1 768->3072 +bias (no GELU)", lambda: K.fused_ffn(x, w1, bias=b1), gemm(3072, 768), None, None),
        ("ffn1 768->3072 (no bias, no GELU)", lambda: K.fused_ffn(x, w1), gemm(3072, 768), None, None),
        ("ffn2 3072->768 +bias", lambda: K.fused_ffn(x4, w2, bias=b2), gemm(768, 3072), None, None),
        ("ffn2 3072->768 +bias+residual", lambda: K.fused_ffn(x4, w2, bias=b2, residual=x), gemm(768, 3072), None, None),
        ("qkv 768->2304 +bias, head-major split", lambda: K.matmul_and_split_qkv(x.view(BATCH, SEQLEN, h), wq, bq, 12), gemm(2304, 768), None, None),
        ("attention projection 768->768 +bias+residual", lambda: K.fused_ffn(x, wo, bias=bo, residual=x), gemm(768, 768), None, None),
        ("attention projection 768->768 +bias (no residual)", lambda: K.fused_ffn(x, wo, bias=bo), gemm(768, 768), None, None),
        ("ffn1 768->3072 +bias+GELU, all-zero operands", lambda: K.fused_ffn(xz, w1z, bias=b1z, add_gelu=True), gemm(3072, 768), None, None),
        ("ffn2 3072->768 +bias+residual, all-zero operands", lambda: K.fused_ffn(x4z, w2z, bias=b2z, residual=xz), gemm(768, 3072), None, None),
        ("qkv 768->2304 +bias, head-major split, all-zero operands", lambda: K.matmul_and_split_qkv(xz.view(BATCH, SEQLEN, h), wqz, bqz, 12), gemm(2304, 768), None, None),
        ("flash attention 512x12x300x64 causal", lambda: K.flash_attention_v1(q, k, v), 4 * BATCH * 12 * 64 * SEQLEN * (SEQLEN + 1) // 2, 4 * BATCH * 12 * SEQLEN * 64 * 2, flush),
        ("layernorm 153600x768", lambda: K.fused_layer_norm(x, lw, lb), None, 2 * M * h * 2, flush),
        ("softmax 153600x768", lambda: K.fused_softmax(x), None, 2 * M * h * 2, flush),
        ("embedding 512x300x768", lambda: K.fused_embeddings(ids, wte, wpe), None, M * 8 + 2 * M * h * 2 + SEQLEN * h * 2, flush),
        ("embedding + first LayerNorm 512x300x768", lambda: K.fused_embeddings_layer_norm(ids, wte, wpe, lw, lb), None, M * 8 + 3 * M * h * 2 + SEQLEN * h * 2, flush),
    ]
    # where the streamed operand comes from: a product whose activations (201 MB) fit the 256 MB
    # memory-side cache, repeated with the cache left alone and with it flushed (HBM) in between,
    # on N(0, 1) and on all-zero operands
    Mc = 32768
    xc, wc, bc = rn(Mc, 4 * h), K.pack_weight(rn(4 * h, 2 * h, std=0.02)), rn(2 * h, std=0.02)
    xcz, wcz, bcz = torch.zeros_like(xc), K.pack_weight(torch.zeros(4 * h, 2 * h, device=dev).half()), torch.zeros_like(bc)
    gc = 2 * Mc * 2 * h * 4 * h
    ops += [
        ("32768x3072 -> 1536 +bias, activations in the memory-side cache", lambda: K.fused_ffn(xc, wc, bias=bc), gc, None, None),
        ("32768x3072 -> 1536 +bias, activations from HBM", lambda: K.fused_ffn(xc, wc, bias=bc), gc, None, flush),
        ("32768x3072 -> 1536 +bias, all-zero operands, activations in the memory-side cache", lambda: K.fused_ffn(xcz, wcz, bias=bcz), gc, None, None),
        ("32768x3072 -> 1536 +bias, all-zero operands, activations from HBM", lambda: K.fused_ffn(xcz, wcz, bias=bcz), gc, None, flush),
    ]
    # the MLP (ffn1 + GELU -> ffn2 + residual) in one piece and in row chunks whose 3072-wide
    # intermediate (134 / 267 MB) could stay in the 256 MB memory-side cache between the two
    # products; 85 row tiles fill whole rounds of the persistent kernels (1020 and 255 tiles)
    mid = torch.empty(M, 4 * h, device=dev, dtype=torch.float16)
    mlp_out = torch.empty(M, h, device=dev, dtype=torch.float16)

    def mlp(rows):
        for r0 in range(0, M, rows):
            r1 = min(M, r0 + rows)
            K._linear(x[r0:r1], w1, b1, None, mid[r0:r1], True, 0.0, K._lib.GPTMI_W_PACKED, "ffn1")
            K._linear(mid[r0:r1], w2, b2, x[r0:r1], mlp_out[r0:r1], False, 0.0,
                      K._lib.GPTMI_W_PACKED, "ffn2")

    for tiles in (600, 85, 170):
        ops.append((f"MLP ffn1+GELU -> ffn2+residual in row chunks of {tiles} x 256 rows",
                    (lambda t: lambda: mlp(t * 256))(tiles), gemm(3072, 768) + gemm(768, 3072), None, flush))
    # the other head sizes the reference accepts (kernels.py:490), same number of (batch, head)
    # pairs x head size as the headline so that the rows compare: 128 -> 6 heads, 256 -> 3 heads
    for d, heads in ((128, 6), (256, 3)):
        for Bq, Lq in ((BATCH, SEQLEN), (64, 1024)):
            qa, ka, va = (rn(Bq, heads, Lq, d) for _ in range(3))
            ops.append((f"flash attention {Bq}x{heads}x{Lq}x{d} causal",
                        (lambda a, b, c: lambda: K.flash_attention_v1(a, b, c))(qa, ka, va),
                        4 * Bq * heads * d * Lq * (Lq + 1) // 2, 4 * Bq * heads * Lq * d * 2, flush))
    # LayerNorm followed by ffn1 + GELU as two launches and as one (the LayerNorm in the GEMM's
    # operand prologue), at the headline's rows and at the 128 rows of a 2 x 64 batch: the one
    # launch is for few rows, where a launch costs more than normalising a row block per column tile
    xs = rn(128, h)
    for rows_, xin in ((M, x), (128, xs)):
        fl_ = 2 * rows_ * 3072 * 768
        ops.append((f"LayerNorm -> ffn1+GELU, two launches, {rows_} rows",
                    (lambda t: lambda: K.fused_ffn(K.fused_layer_norm(t, lw, lb), w1, bias=b1, add_gelu=True))(xin),
                    fl_, None, None))
        ops.append((f"LayerNorm -> ffn1+GELU, one launch (LayerNorm in the GEMM prologue), {rows_} rows",
                    (lambda t: lambda: K.layer_norm_ffn(t, lw, lb, w1, bias=b1, add_gelu=True))(xin),
                    fl_, None, None))
    rows = []
    for name, fn, flops, nbytes, fl in ops:
        mean, med, n = time_op(fn, fl)
        row = {"op": name, "mean_ms": round(mean, 4), "median_ms": round(med, 4), "reps": n}
        if flops:
            row["tflops"] = round(flops / (mean * 1e-3) / 1e12, 1)
            row["frac_mfma_peak"] = round(flops / (mean * 1e-3) / PEAK_FP16, 4)
        if nbytes:
            row["gbps"] = round(nbytes / (mean * 1e-3) / 1e9, 1)
            row["frac_hbm_peak"] = round(nbytes / (mean * 1e-3) / PEAK_HBM, 4)
        rows.append(row)
    print(json.dumps({"metric": "operators_at_headline_sizes", "dtype": "f16", "data": "synthetic",
                      "n_gpus": 1, "ops": rows}), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", choices=sorted(WORKLOADS) + ["ops"], default="headline")
    ap.add_argument("--lm-head", action="store_true",
                    help="include the tied LM head (logits [T, 50257]) in the step")
    ap.add_argument("--no-cpu-baseline", action="store_true",
                    help="skip the host-CPU leg (used under rocprofv3)")
    ap.add_argument("--cpu-sample-batch", type=int, default=BATCH,
                    help="sequences in the host-CPU forward (default: the whole batch of 512; "
                         "64 keeps a profile run short)")
    ap.add_argument("--no-zero-operands", action="store_true",
                    help="skip the ffn1 run on all-zero operands behind the timed region (used "
                         "under rocprofv3, so that the trace holds the forward's launches only)")
    ap.add_argument("--ablate-layernorm", action="store_true",
                    help="timing experiment, WRONG results: the 24 LayerNorm kernels between the "
                         "GEMMs are skipped (identity), which bounds what fusing them into "
                         "neighbouring kernels could return; prints an ablation line, not the "
                         "benchmark line")
    ap.add_argument("--no-ln-prologue", action="store_true",
                    help="small batches: run every LayerNorm as a launch of its own instead of "
                         "inside the following GEMM (gpt.LN_PROLOGUE_MAX_ROWS = 0), for comparison")
    ap.add_argument("--ln-prologue-under-capture", action="store_true",
                    help="with --graph: keep the LayerNorm-in-GEMM form inside the captured graph "
                         "(the model takes the two launches there), for comparison")
    ap.add_argument("--graph", action="store_true",
                    help="time replays of the forward captured into a HIP graph (gpt.GraphedForward)")
    ap.add_argument("--traffic-calibration", action="store_true",
                    help="also launch a plain copy kernel of known size (1 GiB read, 1 GiB "
                         "written) so that FETCH_SIZE / WRITE_SIZE counters of the same "
                         "rocprofv3 --pmc run can be scaled to bytes")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU's full share of the forward; "
                 "--gpus must be 1 (the forward shards over the batch with no exchange between GPUs)")

    import torch

    from gpt_triton_amd import gpt as G
    from gpt_triton_amd import kernels as K

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.workload == "ops":
        return bench_ops(dev)

    arch, batch, seqlen, what = WORKLOADS[args.workload]
    headline = args.workload == "headline" and not args.lm_head
    cfg = G.GPTConfig(dropout=0.1, **arch)
    model = G.FusedGPT(cfg).init_synthetic_(seed=1337).to(device=dev, dtype=torch.float16).eval()
    gen = torch.Generator(device="cpu").manual_seed(1338)
    ids = torch.randint(0, arch["vocab_size"], (batch, seqlen), generator=gen).to(dev)

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
    if args.ablate_layernorm:
        final_ln, calls = G.fused_layer_norm, [0]

        def skipped_ln(x, weight, bias):
            # the model's last call (the final LayerNorm, its output) stays; the others vanish
            calls[0] += 1
            return final_ln(x, weight, bias) if calls[0] % (2 * arch["n_layer"]) == 0 else x

        G.fused_layer_norm = skipped_ln
    if args.no_ln_prologue:
        G.LN_PROLOGUE_MAX_ROWS = 0
    if args.ln_prologue_under_capture:
        G.LN_PROLOGUE_UNDER_CAPTURE = True
    step = (lambda: model(ids, return_logits=True)) if args.lm_head else (lambda: model(ids))
    if args.graph:
        graphed = G.GraphedForward(model, ids, return_logits=args.lm_head)
        step = lambda: graphed(ids)

    with torch.no_grad():
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        recording[0] = True
        t0 = time.perf_counter()
        for _ in range(args.steps):
            out = step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
    recording[0] = False
    if args.ablate_layernorm:
        print(json.dumps({"metric": "ablation_forward_ms_with_the_layernorms_between_gemms_skipped",
                          "value": round(dt / args.steps * 1e3, 3), "unit": "ms",
                          "results": "wrong (timing only)", "n_gpus": 1, "steps": args.steps,
                          "warmup": args.warmup, "config": {"workload": what}}), flush=True)
        return
    if args.lm_head:
        out, logits = out
        assert logits.shape == (batch, seqlen, arch["vocab_size"])
        # every logit finite, and the last token row equal to the plain product of its hidden
        # state with wte (fp32 torch): the rows past 2^32 bytes of the logits are real results
        assert bool(torch.isfinite(logits).all())
        ref = out[-1, -4:].float() @ model.wte_weight.data.float().t()
        assert float((logits[-1, -4:].float() - ref).abs().max()) <= 2e-2
    assert out.shape == (batch, seqlen, arch["n_embd"]) and bool(torch.isfinite(out).all())

    ms = dt / args.steps * 1e3
    tokens = batch * seqlen
    flops = forward_flops(tokens, seqlen, arch, args.lm_head)
    h = arch["n_embd"]
    ffn1_flops = 2 * tokens * 4 * h * h
    if ffn1_events:
        ffn1_ms = sum(a.elapsed_time(b) for a, b in ffn1_events) / len(ffn1_events)
    else:
        # no ffn1 launch of its own was seen: the LayerNorm-prologue form (few rows) or a graph
        # replay; time the call by itself
        xs = torch.randn(tokens, h, device=dev).half()
        w1 = model.blocks[0][1]._weight("ffn1_weight")
        b1 = model.blocks[0][1].ffn1_bias.data
        ffn1_ms = time_op(lambda: inner(xs, w1, b1, None, True, 0.0), min_ms=20.0, warm_ms=5.0)[0]
    achieved = ffn1_flops / (ffn1_ms * 1e-3) / 1e12

    line = {
        "metric": "gpt2_124m_forward_tokens_per_s" if arch is ARCH else "gpt2_xl_forward_tokens_per_s",
        "baseline_metric": "GPT-2 124M fwd ms @512x300 fp16; tokens/s; MFU vs MI355X peak",
        "value": round(tokens / (ms * 1e-3), 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms, 3),
        "higher_is_better": True,
        "scaling": "weak",
        # the reference's published number for the headline forward is 273 ms on one A100-40GB
        # (README.md:17, bench.py:87-89); other hardware, so reported as a ratio of step times
        "vs_baseline": round(273.0 / ms, 3) if headline else None,
        "vs_baseline_ref": "273 ms, gpt-triton mixed fp16, 1x A100 40GB (README.md:17)",
        "dtype": "f16",
        "data": "synthetic",
        "mfu": round(flops / (ms * 1e-3) / PEAK_FP16, 4),
        "mfu_flops": flops,
        "mfu_note": ("executed FLOPs with the tied LM head" if args.lm_head else
                     "executed FLOPs without LM head") + " (GEMMs + causal attention) / 2.5 PFLOP/s",
        "config": {"workload": what + (", logits output (tied LM head)" if args.lm_head
                                       else ", hidden-state output (no LM head)") +
                               (", replays of a captured HIP graph" if args.graph else "") +
                               (", LayerNorms as launches of their own" if args.no_ln_prologue else "") +
                               (", LayerNorm-in-GEMM form kept under capture"
                                if args.ln_prologue_under_capture else ""),
                   "tokens_per_step": tokens, "n_layer": arch["n_layer"], "n_embd": h,
                   "n_head": arch["n_head"]},
        # one ffn1 call = gemm_stream_kernel on the row tiles that fill whole rounds of the
        # persistent workgroups + gemm_kernel<128,128> on the rows left over (none for some shapes)
        "roofline": {"kernel": f"ffn1 GEMM, both launches of a call (gemm_stream_kernel + small-tile gemm_kernel for the last rows: M={tokens} N={4 * h} K={h}, bias+GELU epilogue)",
                     "bound": "mfma", "achieved": round(achieved, 1), "peak": PEAK_FP16 / 1e12,
                     "unit": "TFLOP/s", "frac": round(achieved * 1e12 / PEAK_FP16, 4),
                     "avg_ms": round(ffn1_ms, 4), "calls": len(ffn1_events),
                     "traffic": ffn1_traffic_bytes() if arch is ARCH and batch == BATCH else None},
    }
    if headline and not args.no_zero_operands:
        # the same ffn1 call on all-zero operands (outside the timed region): identical
        # instructions, no bit toggling, so the clock stays up -- the rate the kernel's schedule
        # allows, beside the rate the chip sustains on real data
        xz = torch.zeros(tokens, h, device=dev, dtype=torch.float16)
        wz = K.pack_weight(torch.zeros(h, 4 * h, device=dev, dtype=torch.float16))
        bz = torch.zeros(4 * h, device=dev, dtype=torch.float16)
        zmean, _, _ = time_op(lambda: inner(xz, wz, bz, None, True, 0.0), min_ms=40.0, warm_ms=10.0)
        line["roofline"]["zero_operands"] = {
            "avg_ms": round(zmean, 4), "frac": round(ffn1_flops / (zmean * 1e-3) / PEAK_FP16, 4),
            "note": "same launches on all-zero x, W, bias: the schedule's own rate; the difference "
                    "to `frac` is the clock the chip gives up on operands that toggle bits"}
    line["cpu_baseline"] = (None if (args.no_cpu_baseline or not headline)
                            else cpu_baseline(args.cpu_sample_batch))
    if args.traffic_calibration:
        copy_calibration(dev)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
