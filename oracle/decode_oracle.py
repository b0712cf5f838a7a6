"""CPU oracle of one batch-1 decode step of a Qwen3-style transformer as the reference's graph runs
it.  TEST INFRASTRUCTURE ONLY (see oracle.py).

Op sequence and rounding points follow the script the reference's converter emits and the kernels
its HIP library runs (paths relative to the reference tree):
  graph                scripts/convert_weights.py:488-692 (has_qknorm, GQA via tile), decode variant
                       cccc-llm/cccc-llm.cpp:589-618
  embed                cccc-hip/hip_functions.cpp:2027-2043 (row copy)
  rmsNorm              cccc-hip/hip_functions.cpp:1506-1535: y = bf16(x * rsqrtf(mean(x^2) + eps) * w), eps 1e-6
                       (cccc/NetCifa.cpp:388)
  linear               oracle.linear_oracle (dequantised BF16 weights, exact sum, one BF16 rounding)
  rope                 cccc-hip/hip_functions.cpp:1719-1738, tables oracle C orc_rope_tables
  kv cache             cccc/MatrixOp.cpp:237-280 (append at row pos)
  attention            cccc/MatrixEx.cpp:3018-3104: scores = bf16(K^T q / sqrt(d)), mask k > pos -> -1e9,
                       softmax cccc-hip/hip_functions.cpp:776-804 -> bf16, y = bf16(V p)
  silu / mul / add     cccc/MatrixEx.cpp:756-762, cccc-hip/hip_functions.cpp:722-732, :953-966, :895-908
Every intermediate tensor is BF16; math inside an op is float32 (sums in float64, then float32,
which only removes accumulation-order noise).

Pinning: (1) on the GPU, tests/test_gpu_ref_hip.py runs the reference's own HIP kernels
(oracle/_ref/libref_hip.so, compiled from cccc-hip/hip_functions.cpp where it lies) for RMSNorm, RoPE,
causal mask, softmax, sigmoid / mul / add and the whole attention sequence of MatrixEx.cpp:3018-3104
(with BF16 GEMMs) and compares them with the functions below: identical, or one BF16 ulp apart where
the summation order or the device's expf differ; (2) on the CPU, tests/test_oracle_decode.py checks
closed forms (a constant vector normalises to +-w, RoPE preserves pair norms and is the identity at
position 0, a one-hot softmax, SiLU(0) = 0) and an independent float64 torch implementation of the
same step without intermediate rounding (agreement within BF16 noise).  The reference holds no
golden vectors for these ops.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass

import numpy as np

from . import oracle as o


@dataclass
class DecodeConfig:
    layers: int = 2
    hidden: int = 256
    n_q: int = 4
    n_kv: int = 2
    head_dim: int = 128
    inter: int = 512
    vocab: int = 1000
    t_kv: int = 64
    theta: float = 1e6
    eps: float = 1e-6

    @property
    def q_out(self):
        return self.n_q * self.head_dim

    @property
    def kv_out(self):
        return self.n_kv * self.head_dim


QWEN3_8B = DecodeConfig(layers=36, hidden=4096, n_q=32, n_kv=8, head_dim=128, inter=12288, vocab=151936, t_kv=4096)


def rope_tables(cfg: DecodeConfig):
    L = o.lib()
    L.orc_rope_tables.restype = None
    L.orc_rope_tables.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_void_p]
    cos = np.zeros((cfg.t_kv, cfg.head_dim // 2), dtype=np.uint16)
    sin = np.zeros_like(cos)
    L.orc_rope_tables(cfg.t_kv, cfg.head_dim, cfg.theta, cos.ctypes.data, sin.ctypes.data)
    return cos, sin


def r(x) -> np.ndarray:
    """float -> nearest-even BF16 value, as float32."""
    return o.bf16_to_f32(o.f32_to_bf16(np.asarray(x, dtype=np.float32)))


def f(bits) -> np.ndarray:
    return o.bf16_to_f32(bits)


def rms_norm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    """x, w float32 holding BF16 values; last axis is normalised."""
    ms = (x.astype(np.float64) ** 2).mean(axis=-1, keepdims=True).astype(np.float32)
    invstd = (np.float32(1.0) / np.sqrt(ms + np.float32(eps))).astype(np.float32)
    return r((x * invstd) * w)


def rope(x: np.ndarray, cos_row: np.ndarray, sin_row: np.ndarray) -> np.ndarray:
    """x [..., head_dim] float32 (BF16 values); tables are BF16 values of one position."""
    half = x.shape[-1] // 2
    xl, xr = x[..., :half], x[..., half:]
    return np.concatenate([r(xl * cos_row - xr * sin_row), r(xr * cos_row + xl * sin_row)], axis=-1)


def linear(Wd_bits: np.ndarray, x: np.ndarray) -> np.ndarray:
    """bf16(W x): Wd_bits = dequantised BF16 weight bits [n_out, K]; x float32 BF16 values [K]."""
    return f(o.linear_oracle(Wd_bits, o.f32_to_bf16(x)[None, :])[0])


def silu_mul(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    with np.errstate(over="ignore"):
        sig = r(np.float32(1.0) / (np.float32(1.0) + np.exp(-gate, dtype=np.float32)))
    return r(r(gate * sig) * up)


def softmax(scores: np.ndarray) -> np.ndarray:
    """One row: bf16(expf(x - max) * (1 / sum)), cccc-hip/hip_functions.cpp:776-804 with a = 1, r = 0."""
    e = np.exp(scores - scores.max(), dtype=np.float32)
    inv = np.float32(1.0) / np.float32(e.astype(np.float64).sum())
    return r(e * inv)


def attention(q: np.ndarray, k_cache: np.ndarray, v_cache: np.ndarray, pos: int, n_q: int, n_kv: int) -> np.ndarray:
    """q [n_q, d]; caches [n_kv, t_kv, d] (float32 BF16 values).  Returns [n_q, d]."""
    d = q.shape[-1]
    t_kv = k_cache.shape[1]
    scale = np.float32(1.0 / np.sqrt(np.float32(d)))
    out = np.zeros_like(q)
    for h in range(n_q):
        kv = h // (n_q // n_kv)
        scores = r(scale * (k_cache[kv].astype(np.float64) @ q[h].astype(np.float64)).astype(np.float32))
        scores[np.arange(t_kv) > pos] = r(np.float32(-1e9))
        p = softmax(scores)
        out[h] = r((p.astype(np.float64) @ v_cache[kv].astype(np.float64)).astype(np.float32))
    return out


def dequant_linear(W) -> np.ndarray:
    """BF16 bits [n_out, K] of a linear weight of the model dict: uint8 E5M2 codes [n_out, K], a
    (packed FP4 nibbles [n_out, K / 2], E4M3 block scales [n_out, K / 16]) pair, or uint16 BF16 bits as they are."""
    if not isinstance(W, tuple) and W.dtype == np.uint16:
        return W                                            # already BF16 bits: a weight the reference leaves unquantized
    if isinstance(W, tuple):
        nib, sc = W
        n_out, K = nib.shape[0], nib.shape[1] * 2
        return o.dequant_fp4_blockscale_to_bf16(nib, sc, n_out * K, K // sc.shape[1]).reshape(n_out, K)
    return o.dequant_fp8_to_bf16(W, o.E5M2).reshape(W.shape)


def make_model(cfg: DecodeConfig, seed: int = 0, fmt: str = "fp8_e5m2", qk_norm: bool = True, tied: bool = False):
    """Random-init model: linears from N(0, 0.02) as FP8_E5M2 codes (round to nearest) or, fmt = "fp4_e2m1", as the
    converter's FP4 block-scale packing (blocks of 16); BF16 norms near 1, BF16 embedding N(0, 1).
    qk_norm = False: no per-head norm weights (has_qknorm = False in scripts/convert_weights.py:488-530, Llama-style)."""
    rng = np.random.default_rng(seed)

    def q8(n_out, K):
        w = f(o.f32_to_bf16(rng.standard_normal((n_out, K), dtype=np.float32) * np.float32(0.02)))
        if fmt == "fp4_e2m1":
            nib, sc = o.quantize_fp4_blockscale_converter(w, 16)
            return nib.reshape(n_out, K // 2), sc.reshape(n_out, K // 16)
        return o.encode_e5m2_rne(w)

    def norm_w(n):
        return o.f32_to_bf16((1.0 + 0.1 * rng.standard_normal(n)).astype(np.float32))

    model = {"emb": o.f32_to_bf16(rng.standard_normal((cfg.vocab, cfg.hidden), dtype=np.float32)), "layers": []}
    for _ in range(cfg.layers):
        model["layers"].append({
            "rms_attn": norm_w(cfg.hidden), "wq": q8(cfg.q_out, cfg.hidden), "wk": q8(cfg.kv_out, cfg.hidden),
            "wv": q8(cfg.kv_out, cfg.hidden), "q_norm": norm_w(cfg.head_dim), "k_norm": norm_w(cfg.head_dim),
            "wo": q8(cfg.hidden, cfg.q_out), "rms_ffn": norm_w(cfg.hidden), "w_gate": q8(cfg.inter, cfg.hidden),
            "w_up": q8(cfg.inter, cfg.hidden), "w_down": q8(cfg.hidden, cfg.inter)})
    model["rms_final"] = norm_w(cfg.hidden)
    model["lm_head"] = q8(cfg.vocab, cfg.hidden)
    if not qk_norm:
        for L in model["layers"]:
            del L["q_norm"], L["k_norm"]
    if tied:                                                # tie_word_embeddings: no separate head (scripts/convert_weights.py:230-260)
        del model["lm_head"]
    return model


class DecodeOracle:
    def __init__(self, cfg: DecodeConfig, model: dict):
        self.cfg, self.model = cfg, model
        cos, sin = rope_tables(cfg)
        self.cos, self.sin = f(cos), f(sin)
        self.k = np.zeros((cfg.layers, cfg.n_kv, cfg.t_kv, cfg.head_dim), dtype=np.float32)
        self.v = np.zeros_like(self.k)
        self._deq = {}

    def deq(self, layer, name):
        key = (layer, name)
        if key not in self._deq:
            W = self.model[name] if layer is None else self.model["layers"][layer][name]
            self._deq[key] = dequant_linear(W)
        return self._deq[key]

    def step(self, token: int, pos: int, trace: dict | None = None, logit_rows=None):
        """One decode step.  `trace`, when given, receives the intermediate tensors of every layer
        (keys suffixed with the layer index; layer 0 also under the bare names).  `logit_rows` limits
        the lm_head to those output rows (a full-size vocabulary is then affordable); the returned
        token is the arg-max over the rows computed."""
        c = self.cfg
        x = f(self.model["emb"][token])
        for li, L in enumerate(self.model["layers"]):
            xn = rms_norm(x, f(L["rms_attn"]), c.eps)
            q = linear(self.deq(li, "wq"), xn).reshape(c.n_q, c.head_dim)
            k = linear(self.deq(li, "wk"), xn).reshape(c.n_kv, c.head_dim)
            v = linear(self.deq(li, "wv"), xn).reshape(c.n_kv, c.head_dim)
            if "q_norm" in L:            # Q_hHT -> rmsNorm -> permute -> rope, or straight to the rotation (scripts/convert_weights.py:494-503)
                q, k = rms_norm(q, f(L["q_norm"]), c.eps), rms_norm(k, f(L["k_norm"]), c.eps)
            q = rope(q, self.cos[pos], self.sin[pos])
            k = rope(k, self.cos[pos], self.sin[pos])
            self.k[li, :, pos], self.v[li, :, pos] = k, v
            att = attention(q, self.k[li], self.v[li], pos, c.n_q, c.n_kv).reshape(-1)
            r1 = r(x + linear(self.deq(li, "wo"), att))
            rn = rms_norm(r1, f(L["rms_ffn"]), c.eps)
            gated = silu_mul(linear(self.deq(li, "w_gate"), rn), linear(self.deq(li, "w_up"), rn))
            x = r(r1 + linear(self.deq(li, "w_down"), gated))
            if trace is not None:
                trace[f"x{li}"] = x.copy()
                trace.update({f"xn{li}": xn, f"q{li}": q.copy(), f"att{li}": att.copy(), f"r1_{li}": r1, f"gated{li}": gated})
                if li == 0:
                    trace.update(xn=xn, q=q.copy(), att=att.copy(), r1=r1, gated=gated)
        xf = rms_norm(x, f(self.model["rms_final"]), c.eps)
        # tied embeddings (no "lm_head" in the model): the head multiplies by the BF16 embedding table (cccc/Net.cpp:1158-1190)
        head = "lm_head" if "lm_head" in self.model else "emb"
        if logit_rows is not None:
            logits = linear(dequant_linear(self.model[head][np.asarray(logit_rows)]), xf)
            return logits, int(np.asarray(logit_rows)[int(np.argmax(logits))])
        logits = linear(self.deq(None, head), xf)
        return logits, int(np.argmax(logits))
