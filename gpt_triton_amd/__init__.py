"""MI355X-native GPT-2 forward hot path: hand-written gfx950 HIP kernels behind a C ABI
(libgptmi.so, include/gptmi.h), driven through the operator functions of `kernels` and the
model classes of `gpt`, which keep the names and signatures of thevasudevgupta/gpt-triton's
kernels.py and gpt.py."""

__all__ = ["kernels", "gpt", "build"]
