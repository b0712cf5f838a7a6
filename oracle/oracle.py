"""Python face of the CPU oracle.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module, and
only as the checker.  It wraps oracle/liboracle.so (cccc_oracle.c, the scalar C restatement of the
reference) with ctypes and adds vectorised NumPy forms of the same functions for large inputs.
Each function names the reference lines it follows (paths relative to the reference tree).
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent

FLOAT, DOUBLE, HALF, BF16, E4M3, E5M2, FP4 = 0, 1, 2, 3, 4, 5, 6   # cccc/types.h:24-34

_lib = None
_ref = None


def build(force: bool = False) -> None:
    """Compile liboracle.so (and oracle/_ref when the reference tree is present)."""
    if force or not (HERE / "liboracle.so").exists():
        subprocess.run(["make", "-C", str(HERE), "-B", "liboracle.so"], check=True, capture_output=True)
    if Path(os.environ.get("CCCC_REFERENCE", "/root/reference")).joinpath("cccc/types.h").exists():
        if force or not (HERE / "_ref" / "libref_types.so").exists() or not (HERE / "_ref" / "libref_hip.so").exists():
            subprocess.run(["make", "-C", str(HERE), "ref"], check=True, capture_output=True)


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        path = HERE / "liboracle.so"
        if not path.exists():
            build()
        L = ctypes.CDLL(str(path))
        f32, u8, u16, i32, u32 = ctypes.c_float, ctypes.c_uint8, ctypes.c_uint16, ctypes.c_int, ctypes.c_uint
        vp = ctypes.c_void_p
        L.orc_e5m2_to_float.restype = f32; L.orc_e5m2_to_float.argtypes = [u8]
        L.orc_e4m3_to_float.restype = f32; L.orc_e4m3_to_float.argtypes = [u8]
        L.orc_fp4_to_float.restype = f32; L.orc_fp4_to_float.argtypes = [u8]
        L.orc_f32_to_bf16_rne.restype = u16; L.orc_f32_to_bf16_rne.argtypes = [f32]
        L.orc_f32_to_half_rne.restype = u16; L.orc_f32_to_half_rne.argtypes = [f32]
        L.orc_half_to_float.restype = f32; L.orc_half_to_float.argtypes = [u16]
        L.orc_float_to_e5m2_trunc.restype = u8; L.orc_float_to_e5m2_trunc.argtypes = [f32, f32]
        L.orc_float_to_e4m3_trunc.restype = u8; L.orc_float_to_e4m3_trunc.argtypes = [f32, f32]
        L.orc_float_to_fp4.restype = u8; L.orc_float_to_fp4.argtypes = [f32]
        L.orc_float_to_e5m2_rne.restype = u8; L.orc_float_to_e5m2_rne.argtypes = [f32]
        L.orc_convert.restype = i32; L.orc_convert.argtypes = [vp, i32, vp, i32, u32, f32]
        L.orc_fp4_blockscale_to_bf16.restype = i32; L.orc_fp4_blockscale_to_bf16.argtypes = [vp, vp, vp, u32, u32]
        L.orc_float_to_fp4_blockscale.restype = i32; L.orc_float_to_fp4_blockscale.argtypes = [vp, vp, vp, u32, u32]
        L.orc_quant_gemm.restype = i32
        L.orc_quant_gemm.argtypes = [i32, i32, i32, i32, i32, f32, vp, i32, i32, f32, vp, i32, i32, f32,
                                     f32, vp, i32, i32, vp, vp, u32, i32]
        L.orc_cpu_linear.restype = i32
        L.orc_cpu_linear.argtypes = [vp, i32, f32, vp, u32, vp, vp, i32, i32, i32, vp, i32,
                                     ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)]
        L.orc_decode_table.restype = None; L.orc_decode_table.argtypes = [i32, vp]
        L.orc_encode_e5m2_rne_bulk.restype = None; L.orc_encode_e5m2_rne_bulk.argtypes = [vp, vp, ctypes.c_size_t]
        _lib = L
    return _lib


def ref():
    """oracle/_ref/libref_types.so: the reference's own cccc/types.h, or None if it was never built."""
    global _ref
    if _ref is None:
        path = HERE / "_ref" / "libref_types.so"
        if not path.exists():
            return None
        R = ctypes.CDLL(str(path))
        f32, u8 = ctypes.c_float, ctypes.c_uint8
        for name in ("ref_e5m2_to_float", "ref_e4m3_to_float", "ref_fp4_to_float"):
            getattr(R, name).restype = f32
            getattr(R, name).argtypes = [u8]
        for name in ("ref_float_to_e5m2", "ref_float_to_e4m3", "ref_float_to_fp4"):
            getattr(R, name).restype = u8
            getattr(R, name).argtypes = [f32]
        R.ref_fp4_get.restype = f32; R.ref_fp4_get.argtypes = [ctypes.c_void_p, ctypes.c_int]
        R.ref_float_to_bf16_host.restype = ctypes.c_uint16; R.ref_float_to_bf16_host.argtypes = [f32]
        _ref = R
    return _ref


def _ptr(a: np.ndarray) -> int:
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data


# ----------------------------------------------------------------------------- tables / roundings

def decode_table(dtype: int) -> np.ndarray:
    """float32[256] (FP4: entry i = value of nibble i & 15).  cccc/types.h:72-90, :139-166, :208-216."""
    out = np.empty(256, dtype=np.float32)
    lib().orc_decode_table(dtype, _ptr(out))
    return out


def f32_to_bf16(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even float32 -> bf16 bits (uint16): cccc-cuda/cuda_functions.cu:2761-2764."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = u + 0x7FFF + ((u >> 16) & 1)
    return ((u >> 16) & 0xFFFF).astype(np.uint16)


def bf16_to_f32(h: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(h, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


# ----------------------------------------------------------------------------- dequantisation

def dequant_fp8_to_bf16(codes: np.ndarray, dtype: int, inv_scale: float = 1.0) -> np.ndarray:
    """bf16 bits of decode(code) * inv_scale: cuda_functions.cu:2566-2577 (E4M3), :2756-2766 (E5M2)."""
    with np.errstate(invalid="ignore", over="ignore"):
        f = decode_table(dtype)[np.ascontiguousarray(codes, dtype=np.uint8)] * np.float32(inv_scale)
    return f32_to_bf16(f)


def dequant_fp8_to_half(codes: np.ndarray, dtype: int, inv_scale: float = 1.0) -> np.ndarray:
    """half_rne(decode(code) * inv_scale) as float16: the workspace of the reference's HALF route
    (cccc/cublas_real.h:921-938 -> cuda_convert(.., HALF, .., invScaleA)).  NumPy's float32 -> float16
    cast rounds to nearest even; with inv_scale 1 every FP8 value is a half exactly (E5M2 is the high
    byte of an IEEE half, which tests/test_oracle_formats.py checks)."""
    table = decode_table(dtype)
    with np.errstate(over="ignore", invalid="ignore"):
        return (table[np.asarray(codes, dtype=np.uint8)] * np.float32(inv_scale)).astype(np.float16)


def contract_exact(W: np.ndarray, X: np.ndarray, chunk: int = 8192) -> np.ndarray:
    """float64 X @ W^T for W [n_out, K] and X [tokens, K] of any float type."""
    out = np.empty((X.shape[0], W.shape[0]), dtype=np.float64)
    X64 = X.astype(np.float64)
    for r0 in range(0, W.shape[0], chunk):
        out[:, r0:r0 + chunk] = X64 @ W[r0:r0 + chunk].astype(np.float64).T
    return out


def unpack_fp4(nibbles: np.ndarray, n: int) -> np.ndarray:
    """uint8 codes of n elements: low nibble = even element (cccc/types.h:257-261)."""
    b = np.ascontiguousarray(nibbles, dtype=np.uint8).ravel()
    out = np.empty(b.size * 2, dtype=np.uint8)
    out[0::2] = b & 15
    out[1::2] = b >> 4
    return out[:n]


def dequant_fp4_blockscale_to_bf16(nibbles: np.ndarray, scales: np.ndarray, n: int, block: int = 16) -> np.ndarray:
    """bf16 bits of fp4(i) * e4m3(scales[i // block]) over the flat index: cuda_functions.cu:2926-2939."""
    codes = unpack_fp4(nibbles, n)
    vals = decode_table(FP4)[codes]
    s = decode_table(E4M3)[np.ascontiguousarray(scales, dtype=np.uint8).ravel()]
    with np.errstate(invalid="ignore"):
        f = vals * np.repeat(s, block)[:n]
    return f32_to_bf16(f.astype(np.float32))


def dequant_fp4_to_bf16(nibbles: np.ndarray, n: int, inv_scale: float) -> np.ndarray:
    """Per-tensor scale FP4: cuda_functions.cu:2872-2884."""
    f = decode_table(FP4)[unpack_fp4(nibbles, n)] * np.float32(inv_scale)
    return f32_to_bf16(f)


def convert(src: np.ndarray, src_type: int, dst_type: int, n: int, scale: float = 1.0):
    """Scalar C orc_convert (cuda_functions.cu:3066-3090).  Returns (rc, dst array)."""
    item = {FLOAT: np.float32, HALF: np.uint16, BF16: np.uint16, E4M3: np.uint8, E5M2: np.uint8, FP4: np.uint8}
    if dst_type not in item:
        return -1, None
    cnt = (n + 1) // 2 if dst_type == FP4 else n
    dst = np.zeros(max(cnt, 1), dtype=item[dst_type])
    src = np.ascontiguousarray(src)
    rc = lib().orc_convert(_ptr(src), src_type, _ptr(dst), dst_type, n, scale)
    return rc, dst[:cnt]


# ----------------------------------------------------------------------------- encoders (data makers)

def encode_e5m2_rne(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even float32 -> E5M2 codes.  Not a reference function (the reference
    truncates, cccc/types.h:168-199); it makes the synthetic weights and is pinned against
    torch.float8_e5m2 in the tests."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint8)
    lib().orc_encode_e5m2_rne_bulk(_ptr(x), _ptr(out), x.size)
    return out


def encode_e4m3_rne(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even, saturating-to-NaN float32 -> OCP E4M3 codes, the cast the converter
    applies to FP4 block scales (scripts/convert_weights.py:368: .to(torch.float8_e4m3fn))."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    table = decode_table(E4M3).astype(np.float64)
    pos = table[:0x7F]                                  # 0 .. 448, increasing
    a = np.abs(x.astype(np.float64))
    hi = np.searchsorted(pos, a, side="left").clip(1, 0x7E)
    lo = hi - 1
    d_lo, d_hi = a - pos[lo], pos[hi] - a
    pick_hi = (d_hi < d_lo) | ((d_hi == d_lo) & (hi % 2 == 0))
    code = np.where(pick_hi, hi, lo).astype(np.uint8)
    code = np.where(a > 464.0, 0x7F, code)              # beyond the rounding range of 448 -> NaN
    code = np.where(np.isnan(x), 0x7F, code)
    return (code | (np.signbit(x).astype(np.uint8) << 7)).astype(np.uint8)


FP4_BOUNDS = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0], dtype=np.float32)


def quantize_fp4_blockscale_converter(data: np.ndarray, group: int = 16):
    """The offline converter's packer: scripts/convert_weights.py:346-370.  Returns (nibble bytes,
    scale bytes).  Codes come from the unrounded 6/absmax; boundaries go to the lower code
    (searchsorted side='left'); the scale byte is the RNE E4M3 cast of absmax/6."""
    data = np.ascontiguousarray(data, dtype=np.float32).ravel()
    n = data.size
    pad = (-n) % group
    if pad:
        data = np.concatenate([data, np.zeros(pad, dtype=np.float32)])
    blocks = data.reshape(-1, group)
    amax = np.abs(blocks).max(axis=1)
    scales = np.where(amax > 1e-10, amax / np.float32(6.0), np.float32(1.0)).astype(np.float32)
    with np.errstate(divide="ignore"):
        fwd = np.where(amax > 1e-10, np.float32(6.0) / amax, np.float32(1.0)).astype(np.float32)
    scaled = (blocks * fwd[:, None]).ravel()
    sign = (scaled < 0).astype(np.uint8) * 8
    code = np.searchsorted(FP4_BOUNDS, np.abs(scaled)).astype(np.uint8) | sign
    packed = (code[0::2] | (code[1::2] << 4)).astype(np.uint8)[: (n + 1) // 2]
    scales = scales[: (n + group - 1) // group]
    return packed, encode_e4m3_rne(scales)


def quantize_fp4_blockscale_kernel(data: np.ndarray, block: int = 16):
    """The on-the-fly quantiser: cuda_functions.cu:2896-2923 (truncating E4M3 scale, boundary to the
    upper code).  Scalar C."""
    data = np.ascontiguousarray(data, dtype=np.float32).ravel()
    n = data.size
    nib = np.zeros((n + 1) // 2, dtype=np.uint8)
    sc = np.zeros((n + block - 1) // block, dtype=np.uint8)
    rc = lib().orc_float_to_fp4_blockscale(_ptr(data), _ptr(nib), _ptr(sc), n, block)
    assert rc == 0
    return nib, sc


# ----------------------------------------------------------------------------- linear / GEMM

def dequant_weight(W: np.ndarray, w_type: int, n_out: int, K: int, inv_scale: float = 1.0,
                   blk_sc: np.ndarray | None = None, block: int = 16) -> np.ndarray:
    """bf16 bits [n_out, K] of a K-contiguous quantized weight."""
    if w_type == FP4:
        if blk_sc is not None:
            return dequant_fp4_blockscale_to_bf16(W, blk_sc, n_out * K, block).reshape(n_out, K)
        return dequant_fp4_to_bf16(W, n_out * K, inv_scale).reshape(n_out, K)
    return dequant_fp8_to_bf16(np.asarray(W).ravel()[: n_out * K], w_type, inv_scale).reshape(n_out, K)


def linear_exact(W_bf16: np.ndarray, X_bf16: np.ndarray, chunk: int = 8192) -> np.ndarray:
    """float64 [tokens, n_out] = X @ W^T over bf16 bit arrays: the exact value of the contraction the
    reference hands to its BF16 GEMM (cccc/cublas_real.h:957-961)."""
    X = bf16_to_f32(X_bf16).astype(np.float64)
    out = np.empty((X.shape[0], W_bf16.shape[0]), dtype=np.float64)
    for r0 in range(0, W_bf16.shape[0], chunk):
        Wc = bf16_to_f32(W_bf16[r0:r0 + chunk]).astype(np.float64)
        out[:, r0:r0 + chunk] = X @ Wc.T
    return out


def linear_oracle(W_bf16: np.ndarray, X_bf16: np.ndarray, alpha: float = 1.0, beta: float = 0.0,
                  Y_old: np.ndarray | None = None) -> np.ndarray:
    """bf16 bits [tokens, n_out]: exact contraction, alpha/beta, one rounding to BF16."""
    acc = np.float64(alpha) * linear_exact(W_bf16, X_bf16)
    if beta != 0.0:
        acc = acc + np.float64(beta) * bf16_to_f32(Y_old).astype(np.float64)
    return f32_to_bf16(acc.astype(np.float32))


def quant_gemm(transA, transB, M, N, K, alpha, A, typeA, lda, invA, B, typeB, ldb, invB, beta, C, ldc,
               blk_scA=None, blk_scB=None, block=16, acc64=True) -> int:
    """Scalar C orc_quant_gemm (cccc/cublas_real.h:875-881, :943-964, :1066-1087); C is updated in place."""
    return lib().orc_quant_gemm(transA, transB, M, N, K, alpha, _ptr(A), typeA, lda, invA, _ptr(B), typeB, ldb, invB,
                                beta, _ptr(C), BF16, ldc,
                                _ptr(blk_scA) if blk_scA is not None else None,
                                _ptr(blk_scB) if blk_scB is not None else None, block, 1 if acc64 else 0)


# ----------------------------------------------------------------------------- CPU baseline

def find_cblas_sgemm():
    """(function pointer, library name) of a cblas_sgemm found at run time, or (None, 'builtin')."""
    import glob
    candidates = []
    for name in ("libopenblas.so", "libopenblas.so.0"):
        candidates.append((name, "cblas_sgemm"))
    try:
        import scipy
        base = Path(scipy.__file__).resolve().parent.parent
        for p in sorted(glob.glob(str(base / "scipy.libs" / "libscipy_openblas*.so"))):
            candidates.append((p, "scipy_cblas_sgemm"))
    except Exception:
        pass
    try:
        base = Path(np.__file__).resolve().parent.parent
        for p in sorted(glob.glob(str(base / "numpy.libs" / "libscipy_openblas*.so"))):
            candidates.append((p, "scipy_cblas_sgemm"))
    except Exception:
        pass
    candidates.append(("/opt/conda/lib/libmkl_rt.so", "cblas_sgemm"))
    for path, sym in candidates:
        try:
            L = ctypes.CDLL(path)
            fn = getattr(L, sym)
            return ctypes.cast(fn, ctypes.c_void_p), f"{Path(path).name}:{sym}"
        except (OSError, AttributeError):
            continue
    return None, "builtin"


def cpu_linear(W: np.ndarray, w_type: int, inv_scale: float, blk_sc, block: int, X_bf16: np.ndarray,
               n_out: int, tokens: int, K: int, sgemm=None, threads: int = 1):
    """Reference CPU route (whole-weight dequant + cblas_sgemm + bf16 round).  Returns
    (Y bf16 [tokens, n_out], seconds dequant, seconds gemm)."""
    Y = np.zeros((tokens, n_out), dtype=np.uint16)
    td, tg = ctypes.c_double(0), ctypes.c_double(0)
    W = np.ascontiguousarray(W)
    X = np.ascontiguousarray(X_bf16, dtype=np.uint16)
    rc = lib().orc_cpu_linear(_ptr(W), w_type, inv_scale, _ptr(blk_sc) if blk_sc is not None else None, block,
                              _ptr(X), _ptr(Y), n_out, tokens, K, sgemm, threads, ctypes.byref(td), ctypes.byref(tg))
    assert rc == 0, rc
    return Y, td.value, tg.value
