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
        L.cccc_matrix_set_quant_scale.restype = None; L.cccc_matrix_set_quant_scale.argtypes = [vp, f32]
        L.cccc_matrix_block_scale_data.restype = vp; L.cccc_matrix_block_scale_data.argtypes = [vp]
        L.cccc_matrix_get_block_scale.restype = i64; L.cccc_matrix_get_block_scale.argtypes = [vp, vp, i64]
        L.cccc_matrix_mul.restype = i32; L.cccc_matrix_mul.argtypes = [vp, vp, vp, f32, f32, i32, i32]
        L.cccc_matrix_mul_batched.restype = i32; L.cccc_matrix_mul_batched.argtypes = [vp, vp, vp, i32, i32, f32, f32]
        L.cccc_gpu_allocated_bytes.restype = ctypes.c_ulonglong; L.cccc_gpu_allocated_bytes.argtypes = []
        u64 = ctypes.c_ulonglong
        L.cccc_decode_create.restype = vp; L.cccc_decode_create.argtypes = [i32] * 8 + [f32, f32]
        L.cccc_decode_destroy.restype = None; L.cccc_decode_destroy.argtypes = [vp]
        L.cccc_decode_set_tensor.restype = i32; L.cccc_decode_set_tensor.argtypes = [vp, i32, i32, vp, u64, i32, f32]
        L.cccc_decode_set_block_scales.restype = i32; L.cccc_decode_set_block_scales.argtypes = [vp, i32, i32, vp, u64]
        L.cccc_decode_tensor_data.restype = vp; L.cccc_decode_tensor_data.argtypes = [vp, i32, i32]
        L.cccc_decode_reset.restype = i32; L.cccc_decode_reset.argtypes = [vp, i32, i32]
        L.cccc_decode_step.restype = i32; L.cccc_decode_step.argtypes = [vp]
        L.cccc_decode_run.restype = ctypes.c_double; L.cccc_decode_run.argtypes = [vp, i32, i32]
        L.cccc_decode_token.restype = i32; L.cccc_decode_token.argtypes = [vp]
        L.cccc_decode_pos.restype = i32; L.cccc_decode_pos.argtypes = [vp]
        L.cccc_decode_logits.restype = i32; L.cccc_decode_logits.argtypes = [vp, vp, u64]
        L.cccc_decode_activation.restype = i32; L.cccc_decode_activation.argtypes = [vp, i32, vp, u64]
        L.cccc_decode_kv.restype = i32; L.cccc_decode_kv.argtypes = [vp, i32, i32, vp, u64]
        L.cccc_decode_cos_table.restype = i32; L.cccc_decode_cos_table.argtypes = [vp, vp, u64]
        L.cccc_decode_weight_bytes.restype = u64; L.cccc_decode_weight_bytes.argtypes = [vp]
        L.cccc_weightfile_open.restype = vp; L.cccc_weightfile_open.argtypes = [ctypes.c_char_p, ctypes.POINTER(i32)]
        L.cccc_weightfile_close.restype = None; L.cccc_weightfile_close.argtypes = [vp]
        L.cccc_weightfile_count.restype = i32; L.cccc_weightfile_count.argtypes = [vp]
        L.cccc_weightfile_key.restype = ctypes.c_char_p; L.cccc_weightfile_key.argtypes = [vp, i32]
        L.cccc_weightfile_get.restype = ctypes.c_longlong; L.cccc_weightfile_get.argtypes = [vp, ctypes.c_char_p, vp, u64]
        L.cccc_weightfile_resolve.restype = i32; L.cccc_weightfile_resolve.argtypes = [vp, ctypes.c_char_p, ctypes.c_char_p, i32]
        L.cccc_weightfile_load_named_group.restype = i32; L.cccc_weightfile_load_named_group.argtypes = [vp, vp, ctypes.c_char_p]
        L.cccc_matrix_rows_view.restype = vp; L.cccc_matrix_rows_view.argtypes = [vp, i32, i32]
        L.cccc_weightfile_load_named.restype = i32; L.cccc_weightfile_load_named.argtypes = [vp, vp, ctypes.c_char_p]
        L.cccc_host_float_to_e4m3.restype = ctypes.c_ubyte; L.cccc_host_float_to_e4m3.argtypes = [f32]
        L.cccc_host_half_to_bf16.restype = ctypes.c_ushort; L.cccc_host_half_to_bf16.argtypes = [ctypes.c_ushort]
        L.cccc_decode_load_named.restype = i32; L.cccc_decode_load_named.argtypes = [vp, vp, i32, ctypes.c_char_p, i32]
        L.cccc_decode_save_named.restype = i32; L.cccc_decode_save_named.argtypes = [vp, ctypes.c_char_p]
        L.cccc_matrix_save_named.restype = i32; L.cccc_matrix_save_named.argtypes = [vp, ctypes.c_char_p, ctypes.c_char_p]
        L.cccc_decode_set_exact_attention.restype = None; L.cccc_decode_set_exact_attention.argtypes = [vp, i32]
        L.cccc_decode_prefill.restype = i32; L.cccc_decode_prefill.argtypes = [vp, ctypes.POINTER(ctypes.c_int), i32, i32]
        L.cccc_decode_set_qk_norm.restype = None; L.cccc_decode_set_qk_norm.argtypes = [vp, i32]
        L.cccc_decode_qk_norm.restype = i32; L.cccc_decode_qk_norm.argtypes = [vp]
        L.cccc_decode_set_repack_linears.restype = None; L.cccc_decode_set_repack_linears.argtypes = [vp, i32]
        L.cccc_decode_set_tied_lm_head.restype = None; L.cccc_decode_set_tied_lm_head.argtypes = [vp, i32]
        L.cccc_decode_tied_lm_head.restype = i32; L.cccc_decode_tied_lm_head.argtypes = [vp]
        L.cccc_decode_tensor_prepare.restype = i32; L.cccc_decode_tensor_prepare.argtypes = [vp, i32, i32]
        L.cccc_decode_quantize_linear.restype = i32; L.cccc_decode_quantize_linear.argtypes = [vp, i32, i32, vp, i32]
        L.cccc_decode_tensor_scale.restype = f32; L.cccc_decode_tensor_scale.argtypes = [vp, i32, i32]
        L.cccc_decode_kv_data.restype = vp; L.cccc_decode_kv_data.argtypes = [vp, i32, i32]
        self.c = L

    def init(self, device: int = 0) -> None:
        if self.c.cccc_host_init(device) != 0:
            raise RuntimeError("cccc_host_init failed")

    def set_repack(self, enabled: bool) -> None:
        self.c.cccc_host_set_repack(1 if enabled else 0)

    def matrix(self, w, h, c, n, dtype) -> "HostMatrix":
        return HostMatrix(self, self.c.cccc_matrix_create(w, h, c, n, dtype))


class WeightFile:
    """host/WeightFile.h: memory-mapped reader of a CFG_BIN INI container (no GPU needed to open or query it)."""

    def __init__(self, lib: HostLibrary, path):
        self.lib = lib
        status = ctypes.c_int(0)
        self.handle = lib.c.cccc_weightfile_open(str(path).encode(), ctypes.byref(status))
        self.status = status.value
        if not self.handle:
            raise OSError(f"cannot read weight file {path}: status {self.status}")

    def close(self) -> None:
        if getattr(self, "handle", None):
            self.lib.c.cccc_weightfile_close(self.handle)
            self.handle = None

    __del__ = close

    def keys(self) -> list[str]:
        return [self.lib.c.cccc_weightfile_key(self.handle, i).decode() for i in range(self.lib.c.cccc_weightfile_count(self.handle))]

    def get(self, key: str):
        n = self.lib.c.cccc_weightfile_get(self.handle, key.encode(), None, 0)
        if n < 0:
            return None
        buf = ctypes.create_string_buffer(max(int(n), 1))
        self.lib.c.cccc_weightfile_get(self.handle, key.encode(), buf, n)
        return buf.raw[:n]

    def resolve(self, name: str):
        """(key, dtype, is_quantized) or None."""
        buf = ctypes.create_string_buffer(256)
        rc = self.lib.c.cccc_weightfile_resolve(self.handle, name.encode(), buf, 256)
        return None if rc < 0 else (buf.value.decode(), rc & 0xFFFF, bool(rc & 0x10000))

    def load_named(self, m: "HostMatrix", name: str) -> int:
        return self.lib.c.cccc_weightfile_load_named(self.handle, m.handle, name.encode())

    def load_named_group(self, m: "HostMatrix", names) -> int:
        """Several quantized linears sharing their input into one storage, row ranges in the order given."""
        packed = b"".join(n.encode() + b"\0" for n in names) + b"\0"
        return self.lib.c.cccc_weightfile_load_named_group(self.handle, m.handle, packed)


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

    @quant_scale.setter
    def quant_scale(self, scale: float) -> None:
        """Matrix::setQuantScale: the per-tensor dequantisation multiplier that goes with the codes already in the storage."""
        self.lib.c.cccc_matrix_set_quant_scale(self.handle, scale)

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

    def rows_view(self, row0: int, n_rows: int) -> "HostMatrix":
        """Rows [row0, row0 + n_rows) as a matrix of their own on the same storage (Matrix::rowsView)."""
        handle = self.lib.c.cccc_matrix_rows_view(self.handle, row0, n_rows)
        if not handle:
            raise ValueError("row range does not fit")
        return HostMatrix(self.lib, handle)

    def save_named(self, name: str, path) -> None:
        if self.lib.c.cccc_matrix_save_named(self.handle, name.encode(), str(path).encode()) != 0:
            raise OSError(f"cannot write {path}")

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


# tensor ids of DecodeModel::Tensor
LAYER_TENSORS = {"rms_attn": 0, "wq": 1, "wk": 2, "wv": 3, "q_norm": 4, "k_norm": 5, "wo": 6, "rms_ffn": 7,
                 "w_gate": 8, "w_up": 9, "w_down": 10}
GLOBAL_TENSORS = {"emb": 100, "rms_final": 101, "lm_head": 102}
QUANTIZED = {"wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down", "lm_head"}


class DecodeModel:
    """The C++ DecodeModel (host/DecodeModel.h): a Qwen3-style batch-1 decode step on the fused kernels."""

    def __init__(self, lib: HostLibrary, layers, hidden, n_q, n_kv, head_dim, inter, vocab, t_kv, theta=1e6, eps=1e-6):
        self.lib = lib
        self.cfg = dict(layers=layers, hidden=hidden, n_q=n_q, n_kv=n_kv, head_dim=head_dim, inter=inter, vocab=vocab, t_kv=t_kv)
        self.handle = lib.c.cccc_decode_create(layers, hidden, n_q, n_kv, head_dim, inter, vocab, t_kv, theta, eps)
        if not self.handle:
            raise ValueError("unsupported decode configuration")

    def __del__(self):
        if getattr(self, "handle", None):
            self.lib.c.cccc_decode_destroy(self.handle)
            self.handle = None

    def set_tensor(self, layer: int, name: str, a: np.ndarray, dtype: int, scale: float = 1.0) -> None:
        which = LAYER_TENSORS.get(name, GLOBAL_TENSORS.get(name))
        a = np.ascontiguousarray(a)
        rc = self.lib.c.cccc_decode_set_tensor(self.handle, layer, which, a.ctypes.data, a.nbytes, dtype, scale)
        if rc != 0:
            raise ValueError(f"set_tensor({layer}, {name}) failed: {rc}")

    def set_block_scales(self, layer: int, name: str, scales: np.ndarray) -> None:
        which = LAYER_TENSORS.get(name, GLOBAL_TENSORS.get(name))
        scales = np.ascontiguousarray(scales, dtype=np.uint8)
        rc = self.lib.c.cccc_decode_set_block_scales(self.handle, layer, which, scales.ctypes.data, scales.size)
        if rc != 0:
            raise ValueError(f"set_block_scales({layer}, {name}) failed: {rc}")

    def tensor_ptr(self, layer: int, name: str) -> int:
        return self.lib.c.cccc_decode_tensor_data(self.handle, layer, LAYER_TENSORS.get(name, GLOBAL_TENSORS.get(name)))

    def prepare_tiled(self, layer: int, name: str) -> bool:
        """Builds the tiled copy of a linear whose bytes were written through tensor_ptr (set_tensor and
        load_named do this themselves)."""
        return self.lib.c.cccc_decode_tensor_prepare(self.handle, layer, LAYER_TENSORS.get(name, GLOBAL_TENSORS.get(name))) == 0

    def quantize_linear(self, layer: int, name: str, device_bf16_ptr: int, to: int = 5) -> None:
        """Quantizes a linear on the device from BF16 values ([n_out][K]) already in device memory (DecodeModel::quantizeLinear:
        per-tensor absmax scale for FP8, block scales for FP4)."""
        rc = self.lib.c.cccc_decode_quantize_linear(self.handle, layer, LAYER_TENSORS.get(name, GLOBAL_TENSORS.get(name)), device_bf16_ptr, to)
        if rc != 0:
            raise ValueError(f"quantize_linear({layer}, {name}) failed: {rc}")

    def tensor_scale(self, layer: int, name: str) -> float:
        return float(self.lib.c.cccc_decode_tensor_scale(self.handle, layer, LAYER_TENSORS.get(name, GLOBAL_TENSORS.get(name))))

    def load(self, model: dict, fp8_dtype: int = 5) -> None:
        """model: the dict layout of oracle.decode_oracle.make_model (uint8 codes / uint16 bf16 bits); a quantized
        tensor given as a (packed FP4 nibbles, E4M3 block scales) pair is loaded as FP4_E2M1."""
        def put(li, name, value):
            if isinstance(value, tuple):
                self.set_tensor(li, name, value[0], 6)
                self.set_block_scales(li, name, value[1])
            else:
                self.set_tensor(li, name, value, fp8_dtype if name in QUANTIZED else 3)
        self.set_tied_lm_head("lm_head" not in model)
        for name in GLOBAL_TENSORS:
            if name in model:
                put(0, name, model[name])
        self.set_qk_norm(all("q_norm" in L for L in model["layers"]))
        for li, L in enumerate(model["layers"]):
            for name in LAYER_TENSORS:
                if name in L:
                    put(li, name, L[name])

    def load_named(self, wf: WeightFile, quantize_to: int = 5) -> None:
        """Every tensor from a converted model file by the converter's names; plain linears are quantized on load."""
        failed = ctypes.create_string_buffer(128)
        rc = self.lib.c.cccc_decode_load_named(self.handle, wf.handle, quantize_to, failed, 128)
        if rc != 0:
            raise ValueError(f"loading {failed.value.decode()!r} failed: {rc}")

    def save_named(self, path) -> None:
        """Every tensor under the converter's names, bytes as they sit on the device (DecodeModel::saveNamedWeights)."""
        if self.lib.c.cccc_decode_save_named(self.handle, str(path).encode()) != 0:
            raise OSError(f"cannot write {path}")

    def set_exact_attention(self, exact: bool) -> None:
        """True: separate norm / RoPE / append launch and BF16 probabilities (the reference's rounding
        points); False (default): the two-launch attention with FP32 probabilities."""
        self.lib.c.cccc_decode_set_exact_attention(self.handle, 1 if exact else 0)

    def set_qk_norm(self, on: bool) -> None:
        """Per-head RMSNorm of q and k in front of the rotation (Qwen3: on, the default; Llama-3.1: off)."""
        self.lib.c.cccc_decode_set_qk_norm(self.handle, 1 if on else 0)

    def set_repack_linears(self, on: bool) -> None:
        """Keep the tiled copy of every linear set or loaded from now on (faster prompt-phase GEMMs, twice the weight memory)."""
        self.lib.c.cccc_decode_set_repack_linears(self.handle, 1 if on else 0)

    def set_tied_lm_head(self, tied: bool) -> None:
        """Tied embeddings: the head reads the BF16 embedding table, no separate lm_head is stored."""
        self.lib.c.cccc_decode_set_tied_lm_head(self.handle, 1 if tied else 0)

    @property
    def tied_lm_head(self) -> bool:
        return self.lib.c.cccc_decode_tied_lm_head(self.handle) != 0

    @property
    def qk_norm(self) -> bool:
        return self.lib.c.cccc_decode_qk_norm(self.handle) != 0

    def reset(self, token: int, pos: int) -> None:
        assert self.lib.c.cccc_decode_reset(self.handle, token, pos) == 0

    def prefill(self, tokens, pos0: int = 0) -> int:
        """The prompt phase (DecodeModel::prefill): the caches take the prompt at positions pos0 .., the greedy pick after its
        last token becomes the current token.  Returns that token."""
        arr = (ctypes.c_int * len(tokens))(*[int(t) for t in tokens])
        rc = self.lib.c.cccc_decode_prefill(self.handle, arr, len(tokens), pos0)
        if rc != 0:
            raise RuntimeError(f"prefill failed: {rc}")
        return self.token

    def step(self) -> int:
        rc = self.lib.c.cccc_decode_step(self.handle)
        if rc != 0:
            raise RuntimeError(f"decode step failed: {rc}")
        return self.token

    def run(self, n_steps: int, use_graph: bool) -> float:
        ms = float(self.lib.c.cccc_decode_run(self.handle, n_steps, 1 if use_graph else 0))
        if ms < 0:
            raise RuntimeError(f"decode run failed: {ms}")
        return ms

    @property
    def token(self) -> int:
        return self.lib.c.cccc_decode_token(self.handle)

    @property
    def pos(self) -> int:
        return self.lib.c.cccc_decode_pos(self.handle)

    def logits(self) -> np.ndarray:
        out = np.empty(self.cfg["vocab"], dtype=np.uint16)
        assert self.lib.c.cccc_decode_logits(self.handle, out.ctypes.data, out.nbytes) == 0
        return out

    ACTIVATIONS = {"x": 0, "r1": 1, "q": 2, "k": 3, "v": 4, "att": 5, "gated": 6}

    def activation(self, name: str) -> np.ndarray:
        """BF16 bits of an intermediate vector as the last layer that ran left it."""
        c = self.cfg
        n = {"x": c["hidden"], "r1": c["hidden"], "q": c["n_q"] * c["head_dim"], "k": c["n_kv"] * c["head_dim"],
             "v": c["n_kv"] * c["head_dim"], "att": c["n_q"] * c["head_dim"], "gated": c["inter"]}[name]
        out = np.empty(n, dtype=np.uint16)
        assert self.lib.c.cccc_decode_activation(self.handle, self.ACTIVATIONS[name], out.ctypes.data, out.nbytes) == 0
        return out

    def kv(self, layer: int, is_v: bool) -> np.ndarray:
        c = self.cfg
        out = np.empty((c["n_kv"], c["t_kv"], c["head_dim"]), dtype=np.uint16)
        assert self.lib.c.cccc_decode_kv(self.handle, layer, 1 if is_v else 0, out.ctypes.data, out.nbytes) == 0
        return out

    def cos_table(self) -> np.ndarray:
        c = self.cfg
        out = np.empty((c["t_kv"], c["head_dim"] // 2), dtype=np.uint16)
        assert self.lib.c.cccc_decode_cos_table(self.handle, out.ctypes.data, out.nbytes) == 0
        return out

    def kv_ptr(self, layer: int, is_v: bool) -> int:
        return self.lib.c.cccc_decode_kv_data(self.handle, layer, 1 if is_v else 0)

    @property
    def weight_bytes(self) -> int:
        return int(self.lib.c.cccc_decode_weight_bytes(self.handle))
