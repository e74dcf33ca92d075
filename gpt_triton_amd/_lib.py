"""ctypes binding of libgptmi.so (include/gptmi.h).  There is no fallback: if the library
has not been built, importing the operators fails with instructions."""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libgptmi.so")

GPTMI_F32, GPTMI_F16 = 0, 1
GPTMI_W_KN, GPTMI_W_NK, GPTMI_W_PACKED = 0, 1, 2
GPTMI_O_BNLD, GPTMI_O_BLND = 0, 1

_vp, _i64, _int, _f32, _u64, _sz = (ctypes.c_void_p, ctypes.c_int64, ctypes.c_int,
                                   ctypes.c_float, ctypes.c_uint64, ctypes.c_size_t)

# name -> (restype, argtypes); mirrors include/gptmi.h one to one
SIGNATURES = {
    "gptmi_version": (_int, []),
    "gptmi_last_error": (ctypes.c_char_p, []),
    "gptmi_embed": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _f32, _u64, _int,
                           _vp]),
    "gptmi_embed_layernorm": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64,
                                     _i64, _f32, _int, _vp]),
    "gptmi_layernorm": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _f32, _int, _vp]),
    "gptmi_softmax": (_int, [_vp, _vp, _i64, _i64, _int, _vp]),
    "gptmi_linear_workspace_bytes": (_sz, [_i64, _i64, _i64, _int, _int]),
    "gptmi_packed_weight_bytes": (_sz, [_i64, _i64]),
    "gptmi_pack_weight": (_int, [_vp, _vp, _i64, _i64, _int, _int, _vp]),
    "gptmi_linear": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _f32, _u64, _int,
                            _vp, _sz, _int, _vp]),
    "gptmi_linear_static_capacity": (_sz, []),
    "gptmi_linear_static": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _f32, _u64,
                                   _int, _int, _vp]),
    "gptmi_linear_qkv": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _int,
                                _vp, _sz, _int, _vp]),
    "gptmi_layernorm_linear_supported": (_int, [_i64, _i64, _int]),
    "gptmi_layernorm_linear": (_int, [_vp, _vp, _vp, _f32, _vp, _vp, _vp, _i64, _i64, _i64, _int,
                                      _int, _vp]),
    "gptmi_layernorm_linear_qkv": (_int, [_vp, _vp, _vp, _f32, _vp, _vp, _vp, _vp, _vp, _i64,
                                          _i64, _i64, _i64, _i64, _int, _vp]),
    "gptmi_flash_attn": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _f32, _f32,
                                _u64, _int, _int, _vp]),
}

_lib = None


def load():
    """Loads libgptmi.so once and declares every entry point's prototype."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build the HIP extension first "
            "(`python -m gpt_triton_amd.build`, needs hipcc); there is no CPU fallback")
    # PyTorch ships its own HIP runtime; it must be in the process before libgptmi.so is, so
    # that the library binds to that copy (the one whose streams and allocations it is handed)
    # instead of pulling in a second runtime from /opt/rocm.
    import torch  # noqa: F401

    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc, what):
    if rc != 0:
        msg = load().gptmi_last_error().decode("utf-8", "replace")
        if rc == -2:
            raise NotImplementedError(f"{what}: {msg}")
        raise RuntimeError(f"{what} failed (status {rc}): {msg}")
