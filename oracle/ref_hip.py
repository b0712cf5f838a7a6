"""ctypes view of oracle/_ref/libref_hip.so: the reference's own HIP kernel library
(cccc-hip/hip_functions.cpp) compiled for gfx950 by oracle/Makefile.  TEST INFRASTRUCTURE ONLY: the
GPU-side checker of the BF16 neighbour ops and the kernels of the reference-style decode baseline in
bench.py.  Every entry point takes device pointers and synchronises the device before it returns
(cccc-hip/hip_functions.cpp:32-42).  The library has no FP8 / FP4 code (its hip_convert, .cpp:2683-2690,
knows float, half and bfloat16 only)."""
from __future__ import annotations

import ctypes
from pathlib import Path

HERE = Path(__file__).resolve().parent
_lib = None

BF16 = 3


def lib():
    """The loaded library, or None when it was never built (no reference tree at build time)."""
    global _lib
    if _lib is None:
        path = HERE / "_ref" / "libref_hip.so"
        if not path.exists():
            return None
        L = ctypes.CDLL(str(path))          # RTLD_LOCAL: its hip_* names do not collide with the product library's
        vp, i32, u32, f32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_uint, ctypes.c_float
        sigs = {
            "hip_rms_norm_fwd": [i32, vp, vp, vp, vp, u32, u32, f32],          # hip_functions.h:79-80
            "hip_rope_fwd": [i32, vp, vp, vp, vp, u32, u32, u32, u32],         # :91-94
            "hip_embed_fwd": [i32, vp, vp, vp, i32, i32, i32],                 # :112-113
            "hip_softmax_bf16": [vp, vp, u32, u32, f32, f32],                  # :57
            "hip_sigmoid_bf16": [vp, vp, u32, f32, f32],                       # :54
            "hip_add": [i32, vp, vp, vp, u32, f32, f32],                       # :27
            "hip_mul": [i32, vp, vp, vp, u32, f32, f32],                       # :28
            "hip_causal_mask": [i32, vp, i32, i32, i32, i32],                  # :126
            "hip_tile_fwd": [i32, vp, vp] + [i32] * 8,                         # :117-119
            "hip_convert": [vp, i32, vp, i32, u32, f32],
        }
        for name, args in sigs.items():
            fn = getattr(L, name)
            fn.restype = i32
            fn.argtypes = args
        _lib = L
    return _lib
