"""The C-ABI library loads without a GPU and exports every entry point include/*.h declares; the
argument checks that run before any HIP call behave as documented."""
import ctypes
import re
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent


def declared_symbols():
    names = []
    for header in sorted((ROOT / "include").glob("*.h")):
        text = header.read_text()
        names += re.findall(r"C_EXPORT\s+[\w\s\*]+?\b(hip_\w+)\s*\(", text)
    return names


def test_header_declares_the_expected_entry_points(pkg):
    names = declared_symbols()
    assert set(pkg.capi.EXPORTS) <= set(names), set(pkg.capi.EXPORTS) - set(names)
    assert "hip_convert" in names and "hip_quant_gemm" in names and "hip_fp4_blockscale_to_bf16" in names


def test_library_exports_every_declared_symbol(pkg):
    assert pkg.library_path().exists(), "build the library first: make -C cccc-lite_amd"
    raw = ctypes.CDLL(str(pkg.library_path()))
    for name in declared_symbols():
        assert hasattr(raw, name), name


def test_missing_library_fails_loudly(pkg, tmp_path):
    import pytest
    with pytest.raises(FileNotFoundError):
        pkg.QuantLibrary(tmp_path / "nope.so")


def test_argument_checks_need_no_gpu(pkg):
    lib = pkg.QuantLibrary()
    buf = np.zeros(256, dtype=np.uint8)
    p = buf.ctypes.data
    D = pkg.DataType
    # unsupported conversion pairs are refused before anything is launched
    for st, dt in ((D.DOUBLE, D.FLOAT), (D.FP8_E5M2, D.FP8_E4M3), (D.FP4_E2M1, D.HALF), (9, D.BFLOAT16), (D.BFLOAT16, -3)):
        assert lib.convert(p, st, p, dt, 16, 1.0) == -1
    assert lib.fp4_blockscale_to_bf16(p, p, p, 16, 0) == -1
    assert lib.float_to_fp4_blockscale(p, p, p, 16, 3) == -1
    # unified GEMM: only "exactly one operand quantized, the other BF16, C BF16" is implemented
    assert lib.quant_gemm(1, 0, 16, 1, 16, 1.0, p, D.FP8_E5M2, 16, 1.0, p, D.FP8_E5M2, 16, 1.0, 0.0, p, D.BFLOAT16, 16) == -1
    assert lib.quant_gemm(1, 0, 16, 1, 16, 1.0, p, D.BFLOAT16, 16, 1.0, p, D.BFLOAT16, 16, 1.0, 0.0, p, D.BFLOAT16, 16) == -1
    assert lib.quant_gemm(1, 0, 16, 1, 16, 1.0, p, D.FP8_E5M2, 16, 1.0, p, D.BFLOAT16, 16, 1.0, 0.0, p, D.HALF, 16) == -1
    assert lib.quant_gemm(1, 3, 16, 1, 16, 1.0, p, D.FP8_E5M2, 16, 1.0, p, D.BFLOAT16, 16, 1.0, 0.0, p, D.BFLOAT16, 16) == -1
    assert lib.quant_gemm(1, 0, 16, 1, 16, 1.0, None, D.FP8_E5M2, 16, 1.0, p, D.BFLOAT16, 16, 1.0, 0.0, p, D.BFLOAT16, 16) == -1
    assert lib.quant_gemm(1, 0, 0, 1, 16, 1.0, p, D.FP8_E5M2, 16, 1.0, p, D.BFLOAT16, 16, 1.0, 0.0, p, D.BFLOAT16, 16) == 0
    before = lib.set_sync(True)                                          # returns the previous setting
    assert before in (0, 1) and lib.set_sync(False) == 1 and lib.set_sync(False) == 0
    lib.set_sync(bool(before))
    assert lib.set_stream(None) == 0 and lib.get_stream() == 0
    assert not buf.any()
