"""Writes tests/golden/dropout.npz: inputs and outputs of the REFERENCE's fused_embeddings,
fused_ffn and flash_attention_v1 (kernels.py:75-101, 260-315, 477-525) with dropout_prob > 0,
run under Triton's CPU interpreter.

Run in the authoring container only (the reference tree does not travel):

    TRITON_INTERPRET=1 python tests/golden/make_dropout_vectors.py /root/reference

Generated from the reference because nothing else pins how its kernels feed tl.rand: which
offsets reach the generator (column only / flat m*N+n / lq*Lk+lk), the default seed, the
`rand > p` comparison and the place of the dropout in each epilogue.  Inputs are
fp16-representable fp32 values, stored as fp16; tensors are fp32 so that the interpreter's
treatment of the Python-float `p` (weakly typed there, an fp32 scalar on a device) cannot matter.
`add_gelu` is passed as numpy.bool_: triton 3.6's interpreter cannot wrap a Python bool kernel
argument (it builds an int1 handle over int32 data and raises), a numpy bool passes through.
"""
import os
import sys

os.environ.setdefault("TRITON_INTERPRET", "1")

import numpy as np
import torch


def t32(a):
    return torch.from_numpy(a.astype(np.float32))


def main(ref_root):
    sys.path.insert(0, ref_root)
    import kernels as ref  # the reference's kernels.py

    out = {}
    rng = np.random.default_rng(20240611)

    def h(*shape, scale=1.0):
        return (rng.standard_normal(shape) * scale).astype(np.float16)

    # embeddings: p = 0.25 and the always-on p = 0 path
    ids = rng.integers(0, 50, size=(2, 7), dtype=np.int64)
    wte, wpe = h(50, 200), h(16, 200)
    out["emb_ids"], out["emb_wte"], out["emb_wpe"] = ids, wte, wpe
    out["emb_p"] = np.float32(0.25)
    out["emb_out"] = ref.fused_embeddings(torch.from_numpy(ids), t32(wte), t32(wpe), dropout_prob=0.25).numpy()
    out["emb_out_p0"] = ref.fused_embeddings(torch.from_numpy(ids), t32(wte), t32(wpe)).numpy()

    # ffn: bias + GELU + dropout + residual, ragged against the 128 x 128 tile
    x, w, b, r = h(70, 48), h(48, 136, scale=0.2), h(136, scale=0.2), h(70, 136)
    out["ffn_x"], out["ffn_w"], out["ffn_b"], out["ffn_r"] = x, w, b, r
    out["ffn_p"] = np.float32(0.1)
    out["ffn_out"] = ref.fused_ffn(t32(x), t32(w), bias=t32(b), residual=t32(r),
                                   add_gelu=np.bool_(True), dropout_prob=0.1).numpy()
    out["ffn_out_plain"] = ref.fused_ffn(t32(x), t32(w), add_gelu=np.bool_(False),
                                         dropout_prob=0.5).numpy()

    # attention: two heads (the mask must repeat), two key tiles
    q, k, v = h(1, 2, 100, 64), h(1, 2, 100, 64), h(1, 2, 100, 64)
    out["att_q"], out["att_k"], out["att_v"] = q, k, v
    out["att_p"] = np.float32(0.2)
    out["att_out"] = ref.flash_attention_v1(t32(q), t32(k), t32(v), dropout_prob=0.2).numpy()

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "dropout.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, {k: getattr(v, "shape", v) for k, v in out.items()})


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
