"""Writes tests/golden/flash_attention_v1.npz: inputs and outputs of the REFERENCE's
flash_attention_v1 (kernels.py:477-525) run under Triton's CPU interpreter.

Run in the authoring container only (the reference tree does not travel):

    TRITON_INTERPRET=1 python tests/golden/make_flash_vectors.py /root/reference

Only this operator is generated from the reference: it is the one function of the path whose
last bits (the fp16 rounding of P relative to the per-tile running max) no closed form pins.
Inputs are fp16-representable fp32 values, stored as fp16 to keep the fixture small.
"""
import os
import sys

os.environ.setdefault("TRITON_INTERPRET", "1")

import numpy as np
import torch


def main(ref_root):
    sys.path.insert(0, ref_root)
    import kernels as ref  # the reference's kernels.py

    out = {}
    rng = np.random.default_rng(20240607)
    for name, (B, N, L, D) in {"a": (1, 3, 150, 64), "b": (1, 2, 63, 128), "c": (1, 1, 300, 64)}.items():
        q, k, v = (rng.standard_normal((B, N, L, D)).astype(np.float16) for _ in range(3))
        z = ref.flash_attention_v1(*(torch.from_numpy(t.astype(np.float32)) for t in (q, k, v)))
        out[f"{name}_q"], out[f"{name}_k"], out[f"{name}_v"] = q, k, v
        out[f"{name}_out"] = z.numpy().astype(np.float32)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "flash_attention_v1.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
