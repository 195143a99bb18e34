"""ctypes interface to libturbogpt.so.

Mirrors the reference's tests/bridge.py (Config / OneCycle / StepRates / Native over the tg_* ABI,
bridge.py:7-81) and adds the kernel-level tgk_* entry points.  There is no fallback: if the HIP
library is missing or a symbol is absent, loading raises.
"""
import ctypes as C
import os
from pathlib import Path

_HERE = Path(__file__).resolve().parent
_LIB = None

vp, i32, i64, f32, sz = C.c_void_p, C.c_int, C.c_int64, C.c_float, C.c_size_t

# name -> (restype, argtypes); every symbol include/tgk_kernels.h declares
KERNEL_ABI = {
    "tgk_error": (C.c_char_p, []),
    "tgk_gemm_fwd": (i32, [vp, i32, i32, i32, vp, i32, vp, i32, vp, i32, vp, i32, vp, i32]),
    "tgk_gemm_dgrad": (i32, [vp, i32, i32, i32, vp, i32, vp, i32, vp, i32, vp, i32]),
    "tgk_gemm_wgrad": (i32, [vp, i32, i32, i32, vp, i32, vp, i32, vp, i32, i32, vp, sz]),
    "tgk_gemm_wgrad_workspace": (sz, [i32, i32, i32]),
    "tgk_attn_fwd": (i32, [vp, i32, i32, i32, i32, vp, vp, vp, i32, vp, i32, vp, f32]),
    "tgk_attn_bwd": (i32, [vp, i32, i32, i32, i32, vp, vp, vp, i32, vp, i32, vp, vp, i32, vp, vp, vp, i32,
                           f32, vp, sz]),
    "tgk_attn_bwd_workspace": (sz, [i32, i32, i32]),
    "tgk_embed_fwd": (i32, [vp, i32, i32, i32, vp, vp, vp, vp]),
    "tgk_embed_bwd": (i32, [vp, i32, i32, i32, i32, vp, vp, vp, vp, i32]),
    "tgk_layernorm_fwd": (i32, [vp, i32, i32, vp, vp, vp, vp, vp, vp, f32]),
    "tgk_layernorm_bwd": (i32, [vp, i32, i32, vp, vp, vp, vp, vp, vp, vp, f32, i32, i32, vp, sz]),
    "tgk_layernorm_bwd_workspace": (sz, [i32, i32]),
    "tgk_cross_entropy": (i32, [vp, i32, i32, vp, vp, vp, vp, f32, i32]),
    "tgk_sumsq_partials": (i32, [vp, vp, sz, vp, i32]),
    "tgk_adamw": (i32, [vp, sz, vp, vp, vp, vp, vp, vp, i32, vp, vp, i32, f32, f32, f32, f32, f32, f32,
                        C.c_uint64]),
    "tgk_sample_batch": (i32, [vp, vp, i64, C.c_uint64, C.c_uint64, i32, i32, vp, vp]),
    "tgk_position_means": (i32, [vp, vp, i32, i32, vp]),
}
ENGINE_ABI = {
    "tg_error": (C.c_char_p, []),
}


def library_path():
    return Path(os.environ.get("TURBOGPT_LIBRARY", str(_HERE / "libturbogpt.so")))


def library():
    """The loaded C-ABI library with argument types declared."""
    global _LIB
    if _LIB is None:
        path = library_path()
        if not path.exists():
            raise RuntimeError(f"{path} is missing: build it with `python -m turbogpt_amd.build` "
                               "(there is no CPU or PyTorch fallback)")
        lib = C.CDLL(str(path))
        for name, (restype, argtypes) in {**KERNEL_ABI, **ENGINE_ABI}.items():
            fn = getattr(lib, name)  # AttributeError if the symbol is not exported
            fn.restype, fn.argtypes = restype, argtypes
        _LIB = lib
    return _LIB


def check(status):
    if status < 0:
        raise RuntimeError(library().tg_error().decode())
    return status
