"""Writes tests/golden/flash_attention_v1_lq_lk.npz: inputs and outputs of the REFERENCE's
flash_attention_v1 (kernels.py:477-525) for query and key sequences of DIFFERENT lengths, run
under Triton's CPU interpreter.

Run in the authoring container only (the reference tree does not travel):

    TRITON_INTERPRET=1 python tests/golden/make_flash_lqlk_vectors.py /root/reference

What these vectors pin, and nothing else does: the reference masks by `query >= key` alone
(kernels.py:436) and loads key rows past Lk as zeros (kernels.py:421-424, 462), so with Lq > Lk
the queries at or past Lk also attend to the zero rows that pad the last key tile (score 0,
value 0); with Lq < Lk the keys past the last query are never visible.
Inputs are fp16-representable fp32 values, stored as fp16 to keep the fixture small.
"""
import os
import sys

os.environ.setdefault("TRITON_INTERPRET", "1")

import numpy as np
import torch

CASES = {  # name -> (B, N, Lq, Lk, D)
    "short_q": (1, 2, 70, 150, 64),
    "long_q": (1, 2, 150, 70, 64),      # keys 70..127 are zero padding, visible to queries >= 70
    "long_q_whole_tile": (1, 1, 200, 64, 64),  # no padding rows: queries >= 64 see all 64 keys
    "long_q_d128": (1, 1, 100, 37, 128),
}


def main(ref_root):
    sys.path.insert(0, ref_root)
    import kernels as ref  # the reference's kernels.py

    out = {}
    rng = np.random.default_rng(20240611)
    for name, (B, N, Lq, Lk, D) in CASES.items():
        q = rng.standard_normal((B, N, Lq, D)).astype(np.float16)
        k, v = (rng.standard_normal((B, N, Lk, D)).astype(np.float16) for _ in range(2))
        z = ref.flash_attention_v1(*(torch.from_numpy(t.astype(np.float32)) for t in (q, k, v)))
        out[f"{name}_q"], out[f"{name}_k"], out[f"{name}_v"] = q, k, v
        out[f"{name}_out"] = z.numpy().astype(np.float32)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "flash_attention_v1_lq_lk.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
