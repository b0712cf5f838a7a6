"""ctypes access to libcccc_host.so: the C++ host mirror (Matrix / MatrixData / GpuControl /
Rocblas look-alikes of the reference, HIP only) that calls the kernel library the way cccc's
Matrix::mul / Matrix::mulBatched do (reference cccc/Matrix.cpp:1107-1268)."""
from __future__ import annotations

import ctypes
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent


class HostLibrary:
    def __init__(self, path: Path | None = None):
        path = Path(path) if path else HERE / "libcccc_host.so"
        if not path.exists():
            raise FileNotFoundError(f"{path} is missing: build it with `make -C {HERE}`")
        self.path = path
        L = ctypes.CDLL(str(path))
        vp, i32, f32, i64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_longlong
        L.cccc_host_init.restype = i32; L.cccc_host_init.argtypes = [i32]
        L.cccc_matrix_create.restype = vp; L.cccc_matrix_create.argtypes = [i32, i32, i32, i32, i32]
        L.cccc_matrix_destroy.restype = None; L.cccc_matrix_destroy.argtypes = [vp]
        L.cccc_matrix_data.restype = vp; L.cccc_matrix_data.argtypes = [vp]
        L.cccc_matrix_upload.restype = i32; L.cccc_matrix_upload.argtypes = [vp, vp, ctypes.c_size_t]
        L.cccc_matrix_download.restype = i32; L.cccc_matrix_download.argtypes = [vp, vp, ctypes.c_size_t]
        L.cccc_matrix_load_quantized.restype = i32; L.cccc_matrix_load_quantized.argtypes = [vp, vp, i64, f32, i32]
        L.cccc_matrix_set_block_scale.restype = i32; L.cccc_matrix_set_block_scale.argtypes = [vp, vp, i64]
        L.cccc_matrix_quantize.restype = i32; L.cccc_matrix_quantize.argtypes = [vp, i32]
        L.cccc_host_set_repack.restype = None; L.cccc_host_set_repack.argtypes = [i32]
        L.cccc_matrix_prepare_tiled.restype = i32; L.cccc_matrix_prepare_tiled.argtypes = [vp]
        L.cccc_matrix_dtype.restype = i32; L.cccc_matrix_dtype.argtypes = [vp]
        L.cccc_matrix_quant_scale.restype = f32; L.cccc_matrix_quant_scale.argtypes = [vp]
        L.cccc_matrix_block_scale_data.restype = vp; L.cccc_matrix_block_scale_data.argtypes = [vp]
        L.cccc_matrix_get_block_scale.restype = i64; L.cccc_matrix_get_block_scale.argtypes = [vp, vp, i64]
        L.cccc_matrix_mul.restype = i32; L.cccc_matrix_mul.argtypes = [vp, vp, vp, f32, f32, i32, i32]
        L.cccc_matrix_mul_batched.restype = i32; L.cccc_matrix_mul_batched.argtypes = [vp, vp, vp, i32, i32, f32, f32]
        L.cccc_gpu_allocated_bytes.restype = ctypes.c_ulonglong; L.cccc_gpu_allocated_bytes.argtypes = []
        L.cccc_bench_linear_chain.restype = ctypes.c_double
        L.cccc_bench_linear_chain.argtypes = [i32, ctypes.POINTER(vp), ctypes.POINTER(vp), ctypes.POINTER(vp), i32, i32, i32]
        L.cccc_bench_fp4_chain.restype = ctypes.c_double
        L.cccc_bench_fp4_chain.argtypes = [i32, ctypes.POINTER(vp), ctypes.POINTER(vp), vp, vp, i32, i32, i32, ctypes.c_uint, i32, i32]
        self.c = L

    def init(self, device: int = 0) -> None:
        if self.c.cccc_host_init(device) != 0:
            raise RuntimeError("cccc_host_init failed")

    def set_repack(self, enabled: bool) -> None:
        self.c.cccc_host_set_repack(1 if enabled else 0)

    def matrix(self, w, h, c, n, dtype) -> "HostMatrix":
        return HostMatrix(self, self.c.cccc_matrix_create(w, h, c, n, dtype))

    def bench_linear_chain(self, W, X, R, steps, warmup, use_graph) -> float:
        n = len(W)
        arr = lambda ms: (ctypes.c_void_p * n)(*[m.handle for m in ms])
        return float(self.c.cccc_bench_linear_chain(n, arr(W), arr(X), arr(R), steps, warmup, 1 if use_graph else 0))


    def bench_fp4_chain(self, W_ptrs, S_ptrs, X_ptr, Y_ptr, n_out, tokens, K, block, iters, warmup) -> float:
        n = len(W_ptrs)
        return float(self.c.cccc_bench_fp4_chain(n, (ctypes.c_void_p * n)(*W_ptrs), (ctypes.c_void_p * n)(*S_ptrs), X_ptr, Y_ptr,
                                                 n_out, tokens, K, block, iters, warmup))


class HostMatrix:
    def __init__(self, lib: HostLibrary, handle):
        self.lib, self.handle = lib, handle

    def __del__(self):
        if getattr(self, "handle", None):
            self.lib.c.cccc_matrix_destroy(self.handle)
            self.handle = None

    @property
    def data_ptr(self) -> int:
        return self.lib.c.cccc_matrix_data(self.handle)

    @property
    def dtype(self) -> int:
        return self.lib.c.cccc_matrix_dtype(self.handle)

    @property
    def quant_scale(self) -> float:
        return self.lib.c.cccc_matrix_quant_scale(self.handle)

    @property
    def block_scale_ptr(self):
        return self.lib.c.cccc_matrix_block_scale_data(self.handle)

    def upload(self, a: np.ndarray) -> None:
        a = np.ascontiguousarray(a)
        assert self.lib.c.cccc_matrix_upload(self.handle, a.ctypes.data, a.nbytes) == 0

    def download(self, dtype, count) -> np.ndarray:
        out = np.empty(count, dtype=dtype)
        assert self.lib.c.cccc_matrix_download(self.handle, out.ctypes.data, out.nbytes) == 0
        return out

    def load_quantized(self, codes: np.ndarray, scale: float, dtype: int) -> None:
        codes = np.ascontiguousarray(codes)
        self.lib.c.cccc_matrix_load_quantized(self.handle, codes.ctypes.data, codes.nbytes, scale, dtype)

    def set_block_scale(self, scales: np.ndarray) -> None:
        scales = np.ascontiguousarray(scales)
        assert self.lib.c.cccc_matrix_set_block_scale(self.handle, scales.ctypes.data, scales.nbytes) == 0

    def block_scales(self) -> np.ndarray:
        n = -self.lib.c.cccc_matrix_get_block_scale(self.handle, None, 0)
        out = np.empty(max(n, 0), dtype=np.uint8)
        if n > 0:
            assert self.lib.c.cccc_matrix_get_block_scale(self.handle, out.ctypes.data, n) == n
        return out

    def prepare_tiled(self) -> bool:
        return self.lib.c.cccc_matrix_prepare_tiled(self.handle) == 0

    def quantize(self, dtype: int) -> None:
        self.lib.c.cccc_matrix_quantize(self.handle, dtype)


def mul_batched(A: HostMatrix, B: HostMatrix, R: HostMatrix, ta=0, tb=0, a=1.0, r=0.0) -> int:
    return A.lib.c.cccc_matrix_mul_batched(A.handle, B.handle, R.handle, ta, tb, a, r)


def mul(A: HostMatrix, B: HostMatrix, R: HostMatrix, a=1.0, r=0.0, ta=0, tb=0) -> int:
    return A.lib.c.cccc_matrix_mul(A.handle, B.handle, R.handle, a, r, ta, tb)


_host = None


def host() -> HostLibrary:
    global _host
    if _host is None:
        _host = HostLibrary()
    return _host
