"""Model layer: GPTConfig / FusedGPT / FusedAttention / FusedMLP and the FLOP helpers, with the
class names, constructor arguments and state_dict keys of the reference's gpt.py so that a
checkpoint or calling code written for it works unchanged:

    FusedAttention(hidden_size, num_heads, dropout_prob=0.0)     gpt.py:21-67
    FusedMLP(hidden_size, dropout_prob=0.0)                      gpt.py:70-119
    GPTConfig                                                    gpt.py:122-129
    FusedGPT(config)                                             gpt.py:132-196
    convert_huggingface_to_triton(hf_sd, hf_config)              gpt.py:199-237
    estimate_days / get_num_parameters / compute_mfu             gpt.py:250-263

Differences, all additive: GPU_TO_FLOPS knows "mi355x"; FusedGPT.forward takes
`return_logits=True` for the tied LM head the reference leaves commented out
(gpt.py:159-161, 172-179); `init_synthetic_` draws the N(0, 0.02) benchmark weights;
`FusedGPT.forward` reads `config.dropout` (the reference reads a `dropout_prob` attribute the
dataclass does not have, gpt.py:165, and so only works in eval mode).
"""
import re
from dataclasses import dataclass

import torch
import torch.nn as nn

from .kernels import (flash_attention_v1, fused_embeddings, fused_embeddings_layer_norm, fused_ffn,
                      fused_layer_norm, layer_norm_ffn, layer_norm_linear_supported,
                      layer_norm_matmul_and_split_qkv, lm_head, matmul_and_split_qkv, pack_lm_head,
                      pack_weight)

# Up to this many token rows the blocks run their LayerNorm inside the following GEMM
# (layer_norm_ffn, layer_norm_matmul_and_split_qkv: one launch instead of two, same bits): such
# a forward is bound by its launches.  Above, the LayerNorm kernel and the big-tile GEMMs are
# faster -- the fused form normalises a row block once per column tile and runs on small tiles --
# and so are the two launches inside a captured graph, where a launch costs next to nothing.
LN_PROLOGUE_MAX_ROWS = 1024
LN_PROLOGUE_UNDER_CAPTURE = False  # measurement switch (bench.py --ln-prologue-under-capture)


def _ln_in_gemm(x, weight):
    return (x.numel() // x.shape[-1] <= LN_PROLOGUE_MAX_ROWS and
            layer_norm_linear_supported(x, weight) and
            (LN_PROLOGUE_UNDER_CAPTURE or not torch.cuda.is_current_stream_capturing()))

# dense fp16/bf16 tensor throughput, FLOP/s
GPU_TO_FLOPS = {
    "v100": 130 * 10**12,
    "a100": 312 * 10**12,
    "h100": 989 * 10**12,
    "mi355x": 2500 * 10**12,
}


class _PackedWeights:
    """Per-module cache of the GEMM's packed weight images, used in eval mode only.  An entry
    is rebuilt when the parameter's storage, dtype or version counter changes (optimizer steps,
    load_state_dict, .to()); in-place edits made through `param.data` bypass the version
    counter -- call `clear()` (or `model.train()`) after those."""

    def __init__(self):
        self._entries = {}

    def get(self, name, param, pack=pack_weight):
        key = (param.data_ptr(), param._version, param.dtype, tuple(param.shape))
        hit = self._entries.get(name)
        if hit is None or hit[0] != key:
            hit = (key, pack(param.data))
            self._entries[name] = hit
        return hit[1]

    def clear(self):
        self._entries.clear()


def _linear_flops(tokens, fan_in, fan_out):
    # multiply-adds of the product plus the bias add, as gpt.py:62-67 / 113-119 count them
    return tokens * fan_out * (2 * fan_in) + tokens * fan_out


def _norm_flops(tokens, width):
    return 2 * tokens * width


class FusedAttention(nn.Module):
    """Pre-LN causal self-attention block: x + proj(attention(qkv(LN(x))))."""

    def __init__(self, hidden_size, num_heads, dropout_prob=0.0):
        super().__init__()
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.dropout_prob = dropout_prob
        h = hidden_size
        self.layer_norm_weight = nn.Parameter(torch.ones(h))
        self.layer_norm_bias = nn.Parameter(torch.zeros(h))
        self.c_attn_weight = nn.Parameter(torch.rand(h, 3 * h))
        self.c_attn_bias = nn.Parameter(torch.rand(3 * h))
        self.c_proj_weight = nn.Parameter(torch.rand(h, h))
        self.c_proj_bias = nn.Parameter(torch.rand(h))
        self._packed = _PackedWeights()

    def _weight(self, name):
        prm = getattr(self, name)
        if self.training or (self.hidden_size // self.num_heads) % 8 != 0:
            return prm.data
        return self._packed.get(name, prm)

    def train(self, mode=True):
        self._packed.clear()
        return super().train(mode)

    def forward(self, x, normed=None):
        """`normed`: LayerNorm(x) with this block's weights, if the caller already has it (the
        first block of FusedGPT gets it from the embedding kernel)."""
        p = self.dropout_prob if self.training else 0.0
        skip = x
        y = normed
        w_attn = self._weight("c_attn_weight")
        if y is None and p == 0.0 and _ln_in_gemm(x, w_attn):
            q, k, v = layer_norm_matmul_and_split_qkv(x, self.layer_norm_weight.data,
                                                      self.layer_norm_bias.data, w_attn,
                                                      self.c_attn_bias.data, self.num_heads)
        else:
            if y is None:
                y = fused_layer_norm(x, self.layer_norm_weight.data, self.layer_norm_bias.data)
            q, k, v = matmul_and_split_qkv(y, w_attn, self.c_attn_bias.data, self.num_heads)
        # [B, N, L, d] values in a [B, L, N, d] buffer: the head merge below copies nothing
        y = flash_attention_v1(q, k, v, dropout_prob=p, merged_heads_layout=True)
        y = y.transpose(1, 2).contiguous().view(skip.shape)
        return fused_ffn(y, self._weight("c_proj_weight"), bias=self.c_proj_bias.data,
                         residual=skip, add_gelu=False, dropout_prob=p)

    def get_fwd_flops(self, num_tokens):
        h = self.hidden_size
        return (_norm_flops(num_tokens, h) + _linear_flops(num_tokens, h, 3 * h) +
                _linear_flops(num_tokens, h, h))


class FusedMLP(nn.Module):
    """Pre-LN feed-forward block: x + ffn2(gelu(ffn1(LN(x)))), inner width 4h."""

    def __init__(self, hidden_size, dropout_prob=0.0):
        super().__init__()
        self.hidden_size = hidden_size
        self.intermediate_size = 4 * hidden_size
        self.dropout_prob = dropout_prob
        h, mid = hidden_size, self.intermediate_size
        self.layer_norm_weight = nn.Parameter(torch.ones((h,)))
        self.layer_norm_bias = nn.Parameter(torch.zeros((h,)))
        self.ffn1_weight = nn.Parameter(torch.rand(h, mid))
        self.ffn1_bias = nn.Parameter(torch.rand(mid))
        self.ffn2_weight = nn.Parameter(torch.rand(mid, h))
        self.ffn2_bias = nn.Parameter(torch.rand(h))
        self._packed = _PackedWeights()

    def _weight(self, name):
        prm = getattr(self, name)
        return prm.data if self.training else self._packed.get(name, prm)

    def train(self, mode=True):
        self._packed.clear()
        return super().train(mode)

    def forward(self, x):
        p = self.dropout_prob if self.training else 0.0
        skip = x
        w1 = self._weight("ffn1_weight")
        if p == 0.0 and _ln_in_gemm(x, w1):
            y = layer_norm_ffn(x, self.layer_norm_weight.data, self.layer_norm_bias.data, w1,
                               bias=self.ffn1_bias.data, add_gelu=True)
        else:
            y = fused_layer_norm(x, self.layer_norm_weight.data, self.layer_norm_bias.data)
            y = fused_ffn(y, w1, bias=self.ffn1_bias.data, residual=None, add_gelu=True,
                          dropout_prob=p)
        return fused_ffn(y, self._weight("ffn2_weight"), bias=self.ffn2_bias.data, residual=skip,
                         add_gelu=False, dropout_prob=p)

    def get_fwd_flops(self, num_tokens):
        h, mid = self.hidden_size, self.intermediate_size
        return (_norm_flops(num_tokens, h) + _linear_flops(num_tokens, h, mid) +
                _linear_flops(num_tokens, mid, h))


@dataclass
class GPTConfig:
    vocab_size: int = 50304
    block_size: int = 512
    n_layer: int = 12
    n_head: int = 12
    n_embd: int = 768
    dropout: float = 0.1


class FusedGPT(nn.Module):
    """Token + position embeddings, n_layer x (FusedAttention, FusedMLP), final LayerNorm.
    forward(x) returns the final hidden state [B, L, n_embd], like the reference."""

    def __init__(self, config):
        super().__init__()
        self.config = config
        h = config.n_embd
        self.wte_weight = nn.Parameter(torch.rand(config.vocab_size, h))
        self.wpe_weight = nn.Parameter(torch.rand(config.block_size, h))
        self.blocks = nn.ModuleList([
            nn.Sequential(FusedAttention(h, config.n_head, dropout_prob=config.dropout),
                          FusedMLP(h, dropout_prob=config.dropout))
            for _ in range(config.n_layer)
        ])
        self.layer_norm_weight = nn.Parameter(torch.ones((h,)))
        self.layer_norm_bias = nn.Parameter(torch.zeros((h,)))
        self._packed = _PackedWeights()

    def train(self, mode=True):
        self._packed.clear()
        return super().train(mode)

    def _lm_head_weight(self):
        # In eval mode the LM head multiplies with a packed image of wte whose vocabulary is
        # zero-padded to a multiple of 64 (GPT-2's 50257 -> 50304): the logits' rows are then
        # whole 128-byte lines and the product runs on the persistent GEMM kernel, and the image
        # is built once instead of on every call; see kernels.pack_lm_head.
        w = self.wte_weight
        if self.training:
            return w.data
        return self._packed.get("lm_head", w, pack_lm_head)

    def forward(self, x, return_logits=False):
        # causal by construction; no attention or padding mask is taken
        p = self.config.dropout if self.training else 0.0
        if p == 0.0 and len(self.blocks) > 0:
            # eval mode: the first block's LayerNorm comes out of the embedding kernel.  The two
            # modules of blocks[0] are called one by one, so forward hooks registered on that
            # nn.Sequential container itself do not fire (hooks on its two modules do).
            first = self.blocks[0]
            x, y = fused_embeddings_layer_norm(x, self.wte_weight.data, self.wpe_weight.data,
                                               first[0].layer_norm_weight.data,
                                               first[0].layer_norm_bias.data)
            x = first[1](first[0](x, normed=y))
            rest = self.blocks[1:]
        else:
            x = fused_embeddings(x, self.wte_weight.data, self.wpe_weight.data, dropout_prob=p)
            rest = self.blocks
        for block in rest:
            x = block(x)
        x = fused_layer_norm(x, self.layer_norm_weight.data, self.layer_norm_bias.data)
        if return_logits:
            return x, lm_head(x, self._lm_head_weight())
        return x

    def get_fwd_flops(self, num_tokens):
        cfg = self.config
        # the embedding lookups are counted as if they were matmuls (gpt.py:182-196)
        lookups = num_tokens * cfg.n_embd * 2 * (cfg.vocab_size + cfg.block_size)
        body = sum(m.get_fwd_flops(num_tokens) for blk in self.blocks for m in blk)
        return body + _norm_flops(num_tokens, cfg.n_embd) + lookups

    @torch.no_grad()
    def init_synthetic_(self, seed=1337, std=0.02):
        """Benchmark initialisation: matrices N(0, std), biases 0, LayerNorm (1, 0).  The
        constructors' U[0,1) values overflow fp16 within a layer."""
        gen = torch.Generator(device="cpu").manual_seed(seed)
        for name, prm in self.named_parameters():
            if "layer_norm_weight" in name:
                prm.fill_(1.0)
            elif name.endswith("_bias"):
                prm.zero_()
            else:
                prm.copy_(torch.randn(prm.shape, generator=gen, dtype=torch.float32) * std)
        return self


_MASK_BUFFER = re.compile(r"h\.\d+\.attn\.(bias|masked_bias)")  # HF's causal-mask buffers


def convert_huggingface_to_triton(hf_sd, hf_config):
    """Renames a HuggingFace GPT2Model state dict to FusedGPT's keys.  HF's Conv1D weights are
    already [in, out], so no tensor is transposed; the causal-mask buffers are dropped."""
    n_pos = getattr(hf_config, "n_ctx", None) or hf_config.n_positions
    config = GPTConfig(vocab_size=hf_config.vocab_size, block_size=n_pos,
                       n_layer=hf_config.n_layer, n_head=hf_config.n_head,
                       n_embd=hf_config.n_embd, dropout=0.1)
    rename = {"wte.weight": "wte_weight", "wpe.weight": "wpe_weight",
              "ln_f.weight": "layer_norm_weight", "ln_f.bias": "layer_norm_bias"}
    per_layer = {
        "ln_1.weight": "0.layer_norm_weight", "ln_1.bias": "0.layer_norm_bias",
        "attn.c_attn.weight": "0.c_attn_weight", "attn.c_attn.bias": "0.c_attn_bias",
        "attn.c_proj.weight": "0.c_proj_weight", "attn.c_proj.bias": "0.c_proj_bias",
        "ln_2.weight": "1.layer_norm_weight", "ln_2.bias": "1.layer_norm_bias",
        "mlp.c_fc.weight": "1.ffn1_weight", "mlp.c_fc.bias": "1.ffn1_bias",
        "mlp.c_proj.weight": "1.ffn2_weight", "mlp.c_proj.bias": "1.ffn2_bias",
    }
    for i in range(config.n_layer):
        for src, dst in per_layer.items():
            rename[f"h.{i}.{src}"] = f"blocks.{i}.{dst}"
    sd = {}
    for key, tensor in hf_sd.items():
        if _MASK_BUFFER.fullmatch(key):
            continue
        sd[rename[key]] = tensor
    return sd, config


def convert_hf_and_load_model(model_id, device):
    """Loads HF GPT-2 weights (a hub name, or a local directory when offline) into a FusedGPT;
    returns (model, hf_model), both in eval mode on `device`."""
    from transformers import GPT2Model

    hf_model = GPT2Model.from_pretrained(model_id)
    state_dict, config = convert_huggingface_to_triton(hf_model.state_dict(), hf_model.config)
    model = FusedGPT(config)
    model.load_state_dict(state_dict)
    return model.to(device).eval(), hf_model.to(device).eval()


class GraphedForward:
    """The forward of an eval-mode FusedGPT for one input shape, captured once into a HIP graph
    and replayed per call: the ~110 launches of a forward become one graph launch, which is what
    a small batch is bound by (2 x 64 tokens, 124M: 1.76 -> 1.06 ms).  Nothing in the library
    allocates or synchronises, so capture needs no special path; the operators' output tensors
    come from the graph's private pool.  The result of a call is overwritten by the next call --
    clone it to keep it.  No counterpart in the reference (Triton launches kernel by kernel)."""

    def __init__(self, model, example_ids, return_logits=False, warmup=3):
        assert not model.training, "capture an eval-mode model (weights are packed once)"
        self.ids = example_ids.clone()
        side = torch.cuda.Stream(device=example_ids.device)
        side.wait_stream(torch.cuda.current_stream(example_ids.device))
        with torch.cuda.stream(side):
            for _ in range(warmup):  # packs the weights, sets kernel attributes, fills the pools
                model(self.ids, return_logits=return_logits)
        torch.cuda.current_stream(example_ids.device).wait_stream(side)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.out = model(self.ids, return_logits=return_logits)

    @torch.no_grad()
    def __call__(self, ids):
        assert ids.shape == self.ids.shape and ids.dtype == self.ids.dtype
        self.ids.copy_(ids)
        self.graph.replay()
        return self.out


def estimate_days(flops, mfu=0.45, gpu="h100", num_gpus=1):
    assert gpu in GPU_TO_FLOPS
    return flops / (mfu * GPU_TO_FLOPS[gpu] * 3600 * 24 * num_gpus)


def get_num_parameters(model):
    return sum(p.numel() for p in model.parameters())


def compute_mfu(flops_per_second, gpu="h100"):
    assert gpu in GPU_TO_FLOPS
    return flops_per_second / GPU_TO_FLOPS[gpu]
