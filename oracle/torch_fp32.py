"""Plain PyTorch fp32 GPT-2 forward on the CPU: the stand-in for the reference's CPU-side
comparator, HuggingFace GPT2Model run eagerly in fp32 (bench.py:42-49, test.py:129), whose
files and weights cannot travel to the GPU box.  Same block order as HF GPT-2
(ln_1 -> attention -> +residual -> ln_2 -> MLP -> +residual -> ln_f), true fp32 products.

TEST / CPU-BASELINE INFRASTRUCTURE ONLY: used by bench.py's cpu_baseline leg and by tests; the
product never imports it.
"""
import math

import torch
import torch.nn.functional as F


@torch.no_grad()
def gpt2_forward_fp32(params, ids, n_head):
    """params: dict of fp32 torch tensors keyed like FusedGPT.state_dict(); ids int64 [B, L]."""
    B, L = ids.shape
    h = params["wte_weight"].shape[1]
    d = h // n_head
    n_layer = 1 + max(int(k.split(".")[1]) for k in params if k.startswith("blocks."))
    x = params["wte_weight"][ids] + params["wpe_weight"][:L]
    mask = torch.tril(torch.ones(L, L, dtype=torch.bool))
    for i in range(n_layer):
        a, m = f"blocks.{i}.0.", f"blocks.{i}.1."
        y = F.layer_norm(x, (h,), params[a + "layer_norm_weight"], params[a + "layer_norm_bias"],
                         1e-5)
        qkv = torch.addmm(params[a + "c_attn_bias"], y.view(-1, h), params[a + "c_attn_weight"])
        q, k, v = (t.view(B, L, n_head, d).transpose(1, 2) for t in qkv.view(B, L, 3 * h).split(h, -1))
        s = (q @ k.transpose(-1, -2)) / math.sqrt(d)
        s = s.masked_fill(~mask, float("-inf"))
        o = (s.softmax(-1) @ v).transpose(1, 2).reshape(B * L, h)
        x = x + torch.addmm(params[a + "c_proj_bias"], o, params[a + "c_proj_weight"]).view(B, L, h)
        y = F.layer_norm(x, (h,), params[m + "layer_norm_weight"], params[m + "layer_norm_bias"],
                         1e-5)
        y = F.gelu(torch.addmm(params[m + "ffn1_bias"], y.view(-1, h), params[m + "ffn1_weight"]),
                   approximate="tanh")
        x = x + torch.addmm(params[m + "ffn2_bias"], y, params[m + "ffn2_weight"]).view(B, L, h)
    return F.layer_norm(x, (h,), params["layer_norm_weight"], params["layer_norm_bias"], 1e-5)
