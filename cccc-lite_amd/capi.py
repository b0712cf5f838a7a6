"""ctypes binding of include/cccc_hip_quant.h (the drop-in C-ABI)."""
from __future__ import annotations

import ctypes
from pathlib import Path

HERE = Path(__file__).resolve().parent


class DataType:
    """cccc::DataType values (reference cccc/types.h:24-34)."""
    FLOAT = 0
    DOUBLE = 1
    HALF = 2
    BFLOAT16 = 3
    FP8_E4M3 = 4
    FP8_E5M2 = 5
    FP4_E2M1 = 6


NO_TRANS, TRANS = 0, 1


class FusedLinear(ctypes.Structure):
    """struct hip_fused_linear of include/cccc_hip_quant.h."""
    _fields_ = [("w_type", ctypes.c_int), ("K", ctypes.c_int), ("n_segments", ctypes.c_int), ("pair", ctypes.c_int),
                ("W", ctypes.c_void_p * 3), ("n_out", ctypes.c_int * 3), ("w_scale", ctypes.c_float * 3),
                ("Y", ctypes.c_void_p * 3), ("X", ctypes.c_void_p), ("norm_weight", ctypes.c_void_p),
                ("norm_eps", ctypes.c_float), ("residual", ctypes.c_void_p),
                ("blk_sc", ctypes.c_void_p * 3), ("block_size", ctypes.c_uint), ("argmax_workspace", ctypes.c_void_p)]


def make_fused_linear(w_type, K, W, n_out, Y, X, scales=None, norm_weight=None, norm_eps=1e-6, residual=None, pair=False,
                      blk_sc=None, block_size=16, argmax_workspace=None) -> FusedLinear:
    d = FusedLinear()
    d.block_size = block_size
    d.argmax_workspace = argmax_workspace
    for s, p in enumerate(blk_sc or []):
        d.blk_sc[s] = p
    d.w_type, d.K, d.n_segments, d.pair = w_type, K, len(W), 1 if pair else 0
    for s in range(len(W)):
        d.W[s], d.n_out[s], d.Y[s] = W[s], n_out[s], Y[s]
        d.w_scale[s] = scales[s] if scales else 1.0
    d.X, d.norm_weight, d.norm_eps, d.residual = X, norm_weight, norm_eps, residual
    return d

EXPORTS = (
    "hip_convert",
    "hip_fp4_blockscale_to_bf16",
    "hip_float_to_fp4_blockscale",
    "hip_absmax",
    "hip_quant_gemm",
    "hip_quant_gemm_noalloc",
    "hip_quant_tiled_size",
    "hip_quant_weight_prepare",
    "hip_quant_weight_prepare_fp4",
    "hip_quant_weight_release",
    "hip_quant_linear_fused",
    "hip_rms_norm_fwd",
    "hip_rope_fwd",
    "hip_embed_fwd",
    "hip_embed_token_bf16",
    "hip_qk_norm_rope_kv_bf16",
    "hip_attention_decode_bf16",
    "hip_attention_decode_workspace_bytes",
    "hip_attention_decode_fused_bf16",
    "hip_attention_decode_exact_bf16",
    "hip_qk_norm_rope_kv_rows_bf16",
    "hip_attention_prefill_bf16",
    "hip_add_bf16",
    "hip_swiglu_bf16",
    "hip_add_rms_norm_bf16",
    "hip_quant_gemm_swiglu",
    "hip_quant_gemm_add_rms_norm",
    "hip_quant_gemm_segments",
    "hip_argmax_workspace_bytes",
    "hip_argmax_bf16",
    "hip_argmax_pick_embed_bf16",
    "hip_quant_workspace_reserve",
    "hip_quant_set_sync",
    "hip_quant_set_stream",
    "hip_quant_get_stream",
    "hip_quant_last_kernel",
)


def library_path() -> Path:
    return HERE / "libcccc_hip_quant.so"


class QuantLibrary:
    """The loaded shared library with typed entry points.  Pointers are plain integers (device
    addresses, e.g. torch.Tensor.data_ptr())."""

    def __init__(self, path: Path | None = None):
        path = Path(path) if path else library_path()
        if not path.exists():
            raise FileNotFoundError(
                f"{path} is missing: build it with `make -C {HERE}` (or __graft_entry__.build()); "
                "there is no CPU or PyTorch fallback for this path")
        self.path = path
        L = ctypes.CDLL(str(path))
        vp, i32, u32, f32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_uint, ctypes.c_float
        L.hip_convert.restype = i32
        L.hip_convert.argtypes = [vp, i32, vp, i32, u32, f32]
        L.hip_fp4_blockscale_to_bf16.restype = i32
        L.hip_fp4_blockscale_to_bf16.argtypes = [vp, vp, vp, u32, u32]
        L.hip_float_to_fp4_blockscale.restype = i32
        L.hip_float_to_fp4_blockscale.argtypes = [vp, vp, vp, u32, u32]
        L.hip_absmax.restype = i32
        L.hip_absmax.argtypes = [vp, i32, u32, vp]
        L.hip_quant_gemm.restype = i32
        L.hip_quant_gemm.argtypes = [i32, i32, i32, i32, i32, f32,
                                     vp, i32, i32, f32,
                                     vp, i32, i32, f32,
                                     f32, vp, i32, i32, f32,
                                     vp, vp, u32]
        L.hip_quant_gemm_noalloc.restype = i32
        L.hip_quant_gemm_noalloc.argtypes = L.hip_quant_gemm.argtypes
        L.hip_quant_tiled_size.restype = ctypes.c_ulonglong
        L.hip_quant_tiled_size.argtypes = [i32, i32, i32]
        L.hip_quant_weight_prepare.restype = i32
        L.hip_quant_weight_prepare.argtypes = [vp, i32, i32, i32, i32, vp]
        L.hip_quant_weight_prepare_fp4.restype = i32
        L.hip_quant_weight_prepare_fp4.argtypes = [vp, vp, u32, i32, i32, vp]
        L.hip_quant_weight_release.restype = i32
        L.hip_quant_weight_release.argtypes = [vp]
        L.hip_quant_linear_fused.restype = i32
        L.hip_quant_linear_fused.argtypes = [ctypes.POINTER(FusedLinear)]
        L.hip_rms_norm_fwd.restype = i32
        L.hip_rms_norm_fwd.argtypes = [i32, vp, vp, vp, vp, u32, u32, f32]
        L.hip_rope_fwd.restype = i32
        L.hip_rope_fwd.argtypes = [i32, vp, vp, vp, vp, u32, u32, u32, u32]
        L.hip_embed_fwd.restype = i32
        L.hip_embed_fwd.argtypes = [i32, vp, vp, vp, i32, i32, i32]
        L.hip_embed_token_bf16.restype = i32
        L.hip_embed_token_bf16.argtypes = [vp, vp, vp, i32, i32]
        L.hip_qk_norm_rope_kv_bf16.restype = i32
        L.hip_qk_norm_rope_kv_bf16.argtypes = [vp] * 10 + [i32, i32, i32, i32, vp, f32]
        L.hip_attention_decode_bf16.restype = i32
        L.hip_attention_decode_bf16.argtypes = [vp] * 5 + [ctypes.c_ulonglong, i32, i32, i32, i32, vp]
        L.hip_attention_decode_fused_bf16.restype = i32
        L.hip_attention_decode_fused_bf16.argtypes = [vp] * 11 + [ctypes.c_ulonglong, i32, i32, i32, i32, vp, f32]
        L.hip_attention_decode_exact_bf16.restype = i32
        L.hip_attention_decode_exact_bf16.argtypes = [vp] * 11 + [ctypes.c_ulonglong, i32, i32, i32, i32, vp, f32]
        L.hip_qk_norm_rope_kv_rows_bf16.restype = i32
        L.hip_qk_norm_rope_kv_rows_bf16.argtypes = [vp] * 10 + [i32, i32, i32, i32, i32, i32, f32]
        L.hip_attention_prefill_bf16.restype = i32
        L.hip_attention_prefill_bf16.argtypes = [vp] * 4 + [i32, i32, i32, i32, i32, i32]
        L.hip_add_bf16.restype = i32
        L.hip_add_bf16.argtypes = [vp, vp, vp, ctypes.c_ulonglong]
        L.hip_swiglu_bf16.restype = i32
        L.hip_swiglu_bf16.argtypes = [vp, vp, vp, ctypes.c_ulonglong]
        L.hip_quant_gemm_segments.restype = i32
        L.hip_quant_gemm_segments.argtypes = [i32, vp, vp, vp, vp, vp, i32, i32, i32, i32, vp, i32]
        L.hip_quant_gemm_add_rms_norm.restype = i32
        L.hip_quant_gemm_add_rms_norm.argtypes = [i32, i32, i32, vp, i32, i32, ctypes.c_float, vp, i32, vp, vp, vp, vp, ctypes.c_float]
        L.hip_quant_gemm_swiglu.restype = i32
        L.hip_quant_gemm_swiglu.argtypes = [i32, i32, i32, vp, vp, i32, i32, ctypes.c_float, ctypes.c_float, vp, i32, vp, i32]
        L.hip_add_rms_norm_bf16.restype = i32
        L.hip_add_rms_norm_bf16.argtypes = [vp, vp, vp, vp, vp, u32, u32, ctypes.c_float]
        L.hip_attention_decode_workspace_bytes.restype = ctypes.c_ulonglong
        L.hip_attention_decode_workspace_bytes.argtypes = [i32, i32, i32]
        L.hip_argmax_workspace_bytes.restype = ctypes.c_ulonglong
        L.hip_argmax_workspace_bytes.argtypes = [u32]
        L.hip_argmax_bf16.restype = i32
        L.hip_argmax_bf16.argtypes = [vp, u32, vp, vp, vp]
        L.hip_argmax_pick_embed_bf16.restype = i32
        L.hip_argmax_pick_embed_bf16.argtypes = [vp, u32, vp, vp, vp, vp, i32, i32]
        L.hip_quant_set_sync.restype = i32
        L.hip_quant_set_sync.argtypes = [i32]
        L.hip_quant_set_stream.restype = i32
        L.hip_quant_set_stream.argtypes = [vp]
        L.hip_quant_workspace_reserve.restype = i32
        L.hip_quant_workspace_reserve.argtypes = [ctypes.c_ulonglong]
        L.hip_quant_get_stream.restype = vp
        L.hip_quant_get_stream.argtypes = []
        L.hip_quant_last_kernel.restype = ctypes.c_char_p
        L.hip_quant_last_kernel.argtypes = []
        self.c = L

    # -- thin, argument-for-argument wrappers ------------------------------------------------
    def convert(self, src, src_type, dst, dst_type, n, scale=1.0) -> int:
        return self.c.hip_convert(src, src_type, dst, dst_type, n, scale)

    def fp4_blockscale_to_bf16(self, nibbles, scales, dst, n_elems, block_size=16) -> int:
        return self.c.hip_fp4_blockscale_to_bf16(nibbles, scales, dst, n_elems, block_size)

    def float_to_fp4_blockscale(self, src, nibbles, scales, n_elems, block_size=16) -> int:
        return self.c.hip_float_to_fp4_blockscale(src, nibbles, scales, n_elems, block_size)

    def absmax(self, src, src_type, n, d_result) -> int:
        return self.c.hip_absmax(src, src_type, n, d_result)

    def quant_gemm(self, transA, transB, M, N, K, alpha, A, typeA, lda, invScaleA,
                   B, typeB, ldb, invScaleB, beta, C, typeC, ldc, act_scale=0.0,
                   blk_scA=None, blk_scB=None, block_size=16, noalloc=False) -> int:
        entry = self.c.hip_quant_gemm_noalloc if noalloc else self.c.hip_quant_gemm
        return entry(transA, transB, M, N, K, alpha, A, typeA, lda, invScaleA,
                                     B, typeB, ldb, invScaleB, beta, C, typeC, ldc, act_scale,
                                     blk_scA, blk_scB, block_size)

    def tiled_size(self, w_type, n_out, K) -> int:
        return int(self.c.hip_quant_tiled_size(w_type, n_out, K))

    def weight_prepare(self, W, w_type, n_out, K, ldw, dst_tiled) -> int:
        return self.c.hip_quant_weight_prepare(W, w_type, n_out, K, ldw, dst_tiled)

    def weight_prepare_fp4(self, W, blk_sc, block_size, n_out, K, dst_tiled) -> int:
        return self.c.hip_quant_weight_prepare_fp4(W, blk_sc, block_size, n_out, K, dst_tiled)

    def weight_release(self, W) -> int:
        return self.c.hip_quant_weight_release(W)

    def quant_linear_fused(self, desc: FusedLinear) -> int:
        return self.c.hip_quant_linear_fused(ctypes.byref(desc))

    def set_sync(self, enabled: bool) -> int:
        return self.c.hip_quant_set_sync(1 if enabled else 0)

    def set_stream(self, stream_handle: int | None) -> int:
        return self.c.hip_quant_set_stream(stream_handle)

    def workspace_reserve(self, nbytes: int) -> int:
        return self.c.hip_quant_workspace_reserve(nbytes)

    def get_stream(self) -> int:
        return int(self.c.hip_quant_get_stream() or 0)

    def last_kernel(self) -> str:
        return (self.c.hip_quant_last_kernel() or b"").decode()

    # -- the call the LLM graph makes --------------------------------------------------------
    def linear(self, W, w_type, X, Y, n_out, tokens, K, inv_scale=1.0, blk_sc=None, block_size=16,
               alpha=1.0, beta=0.0, act_type=DataType.BFLOAT16, noalloc=False) -> int:
        """y[t][o] = sum_k W[o][k] x[t][k], argument layout of Matrix::mulBatched(W, X, Y, TRANS,
        NO_TRANS) for a linear layer (reference cccc/Matrix.cpp:1162-1203): BLAS M = n_out,
        BLAS N = tokens, lda = ldb = K, ldc = n_out."""
        return self.quant_gemm(TRANS, NO_TRANS, n_out, tokens, K, alpha, W, w_type, K, inv_scale,
                               X, act_type, K, 1.0, beta, Y, act_type, n_out, 0.0,
                               blk_sc, None, block_size, noalloc=noalloc)


_library = None


def library() -> QuantLibrary:
    global _library
    if _library is None:
        _library = QuantLibrary()
    return _library
