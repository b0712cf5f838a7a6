#!/usr/bin/env python3
"""Benchmark of the MI355X weight-only quantized linear path (one GPU).

A step is one pass of the hot path over one batch of synthetic input.  Default workload
(`decode_step`): one greedy batch-1 decode step of a random-init Qwen3-8B-shaped W8A16 model -- 36
layers, FP8_E5M2 linears, BF16 activations and KV cache holding 4096 positions -- run by the C++
DecodeModel on the fused kernels; `value` = tokens per second.  The same line then carries the GEMV
half of the metric: the 253 linears of one token issued through Matrix::mulBatched exactly as
cccc's graph issues them (`quant_gemv`), the per-shape sweep over M in {1, 4, 16} (`sweep`) and the
FP4 block-scale sweep (`fp4_sweep`); GB/s figures are algorithmic bytes (K*N + 2*M*K + 2*M*N per
GEMV) / elapsed.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload decode_step|decode_linears|gemv|prefill|prompt_attention]
                    [--shape K,N] [--tokens M] [--no-graph] [--no-cpu] [--no-sweep]

Prints ONE JSON line.  `roofline` is measured live on the dominant kernel (the fused RMSNorm +
gate/up SwiGLU GEMV for decode_step, the gate/up-shaped GEMV K=4096 N=12288 for decode_linears)
with HIP events on the stream it runs on; `cpu_baseline` times the CPU restatement of the
reference's CPU route (scalar dequant of the whole weight + cblas_sgemm) on a bounded sample.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published
# HBM bytes per launch of the gate/up-shaped GEMV (K=4096, N=12288, M=1) from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE, each scaled by the same counter on a 256 MiB device copy (factors 1.99977 and 1.0)
GEMV_GATE_UP_TRAFFIC_BYTES = 50450876
# the same two counters for one launch of the fused RMSNorm + gate/up SwiGLU GEMV (two 4096 x 12288 weights)
GEMV_FUSED_GATE_UP_TRAFFIC_BYTES = 101017770

# `roofline.traffic` is a constant from a counter run, not measured by this script (rocprofv3 --pmc needs a run of its own)
TRAFFIC_SOURCE = "constant copied from the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs summarised in profiles/"

FLOAT, HALF, BF16, E4M3, E5M2, FP4 = 0, 2, 3, 4, 5, 6

QWEN3_8B = dict(layers=36, hidden=4096, n_q=32, n_kv=8, q_out=4096, kv_out=1024, inter=12288, vocab=151936)
QWEN_SHAPES = [(4096, 4096), (4096, 1024), (4096, 12288), (12288, 4096), (4096, 151936)]     # (K, N)


def gemv_bytes(K, N, M):
    return K * N + 2 * M * K + 2 * M * N


class BenchLibrary:
    """libcccc_bench.so: the timing loops (host/bench_capi.cpp), native so that Python call overhead stays out
    of microsecond kernels.  Only this script loads it."""

    def __init__(self, pkg_dir: Path):
        import ctypes
        path = pkg_dir / "libcccc_bench.so"
        if not path.exists():
            raise FileNotFoundError(f"{path} is missing: build it with `make -C {pkg_dir}`")
        L = ctypes.CDLL(str(path))
        vp, i32 = ctypes.c_void_p, ctypes.c_int
        L.cccc_bench_linear_chain.restype = ctypes.c_double
        L.cccc_bench_linear_chain.argtypes = [i32, ctypes.POINTER(vp), ctypes.POINTER(vp), ctypes.POINTER(vp), i32, i32, i32]
        L.cccc_bench_fp4_chain.restype = ctypes.c_double
        L.cccc_bench_fp4_chain.argtypes = [i32, ctypes.POINTER(vp), ctypes.POINTER(vp), vp, vp, i32, i32, i32, ctypes.c_uint, i32, i32]
        L.cccc_decode_bench_gate_up.restype = ctypes.c_double
        L.cccc_decode_bench_gate_up.argtypes = [vp, i32]
        L.cccc_bench_floor_read.restype = ctypes.c_double
        L.cccc_bench_floor_read.argtypes = [i32, ctypes.POINTER(vp), ctypes.c_ulonglong, i32, i32, i32, i32, i32]
        L.cccc_bench_launch_us.restype = ctypes.c_double
        L.cccc_bench_launch_us.argtypes = [i32, i32, i32]
        L.cccc_bench_gemm_ablation.restype = ctypes.c_double
        L.cccc_bench_gemm_ablation.argtypes = [i32, i32, i32, ctypes.POINTER(i32)]
        L.cccc_bench_gemm_variant.restype = ctypes.c_double
        L.cccc_bench_gemm_variant.argtypes = [i32, i32, i32, ctypes.POINTER(vp), vp, vp, i32, i32, i32, ctypes.c_float, vp, i32, i32, ctypes.POINTER(ctypes.c_double)]
        self.c, self.ctypes = L, ctypes

    def gemm_ablation_tflops(self, flags: int, trips=2048, launches=40) -> float:
        """TFLOP/s of the prefill GEMM's k-tile with only some of its ingredients (host/bench_gemm_variants.hip,
        gemm_ablation_kernel): 0 = the 64 matrix-core instructions on register operands; +1 FP8 -> BF16 conversions,
        +2 fragment reads from LDS, +4 barrier, +8 LDS stores, +16 weight loads, +32 activation loads (L2-resident windows)."""
        n = self.ctypes.c_int(0)
        us = float(self.c.cccc_bench_gemm_ablation(flags, trips, launches, self.ctypes.byref(n)))
        if us < 0:
            raise RuntimeError(f"gemm ablation {flags} failed: {us}")
        return n.value * 4.0 * trips * 64 * 16384 / us * 1e-6

    def gemm_variant(self, variant, tile, tiled_ptrs, X_ptr, Y_ptr, n_out, tokens, K, inv_scale=1.0, partial_ptr=None, iters=64, warmup=8):
        """Microseconds per launch of one experimental variant of the FP8 prefill GEMM (host/bench_gemm_variants.hip)
        and, for the tracing variants, the share of a workgroup's ticks spent converting / at the barrier / in the rest."""
        n = len(tiled_ptrs)
        phases = (self.ctypes.c_double * 4)()
        us = float(self.c.cccc_bench_gemm_variant(variant, tile, n, (self.ctypes.c_void_p * n)(*tiled_ptrs), X_ptr, Y_ptr, n_out, tokens, K,
                                                  inv_scale, partial_ptr, iters, warmup, phases))
        if us < 0:
            raise RuntimeError(f"gemm variant {variant}/{tile} failed: {us}")
        return us, ([round(phases[j] / phases[3], 4) for j in range(3)] if (variant & 4) and phases[3] > 0 else None)

    def floor_read_us(self, ptrs, nbytes, iters=None, wgs_per_cu=8, contiguous=False, pipelined=True) -> float:
        """Microseconds per launch of a kernel that only streams `nbytes` with 16-byte loads, rotating over the buffers
        `ptrs` (host/bench_kernels.hip): the floor of any weight-streaming launch of that size on this GPU.  contiguous:
        every workgroup reads one contiguous range instead of KiB pieces at a grid stride; pipelined: eight KiB pieces
        in flight per wave instead of four."""
        n = len(ptrs)
        iters = iters or max(20, min(400, (4 << 30) // max(nbytes, 1)))
        us = float(self.c.cccc_bench_floor_read(n, (self.ctypes.c_void_p * n)(*ptrs), nbytes, wgs_per_cu, iters, min(5, n), 1 if contiguous else 0, 1 if pipelined else 0))
        if us < 0:
            raise RuntimeError(f"floor read failed: {us}")
        return us

    def floor_us(self, ptrs, nbytes) -> float:
        """The fastest of the streaming-read forms: 2, 4 or 8 workgroups per CU, pieces at a grid stride or one contiguous
        range per workgroup, four or eight KiB pieces in flight per wave."""
        return min(self.floor_read_us(ptrs, nbytes, wgs_per_cu=w, contiguous=c, pipelined=p) for w in (2, 4, 8) for c in (False, True) for p in (False, True))

    def launch_us(self, kind=0, n_launches=200, reps=20) -> float:
        """Microseconds per launch of `n_launches` dependent launches inside one hipGraph (0: empty kernel, 1: one wave
        with one dependent trip to memory)."""
        us = float(self.c.cccc_bench_launch_us(n_launches, reps, kind))
        if us < 0:
            raise RuntimeError(f"launch timing failed: {us}")
        return us

    def linear_chain(self, W, X, R, steps, warmup, use_graph) -> float:
        n = len(W)
        arr = lambda ms: (self.ctypes.c_void_p * n)(*[m.handle for m in ms])
        return float(self.c.cccc_bench_linear_chain(n, arr(W), arr(X), arr(R), steps, warmup, 1 if use_graph else 0))

    def fp4_chain(self, W_ptrs, S_ptrs, X_ptr, Y_ptr, n_out, tokens, K, block, iters, warmup) -> float:
        n = len(W_ptrs)
        vp = self.ctypes.c_void_p
        return float(self.c.cccc_bench_fp4_chain(n, (vp * n)(*W_ptrs), (vp * n)(*S_ptrs), X_ptr, Y_ptr, n_out, tokens, K, block, iters, warmup))

    def gate_up_us(self, model, reps: int) -> float:
        """Average microseconds per fused gate/up launch over all layers' distinct weights."""
        us = float(self.c.cccc_decode_bench_gate_up(model.handle, reps))
        if us < 0:
            raise RuntimeError(f"gate/up timing failed: {us}")
        return us


class Workspace:
    """Weights, activations and outputs of the benchmark as host-mirror matrices on cuda:0."""

    def __init__(self, pkg, torch):
        self.pkg, self.torch = pkg, torch
        self.lib = pkg.library()
        self.host = pkg.host_api.host()
        self.host.init(0)
        self.bench = BenchLibrary(ROOT / "cccc-lite_amd")
        self.dev = torch.device("cuda:0")
        self.gen = torch.Generator(device=self.dev).manual_seed(1234)
        self.keep = []
        self.repack = False

    def weight_e5m2(self, n_out, K):
        return self.weight_fp8(n_out, K, E5M2)

    def weight_fp8(self, n_out, K, dtype=E5M2, inv_scale=1.0):
        """FP8 codes of N(0, 0.02) weights (bf16, then round to nearest).  inv_scale != 1: the codes are those of
        w / inv_scale and the matrix carries inv_scale as its per-tensor dequantisation multiplier, as a weight quantized by
        Matrix::quantizeWeights does (cccc/Matrix.cpp:338-352)."""
        t = self.torch
        f8 = t.float8_e5m2 if dtype == E5M2 else t.float8_e4m3fn
        m = self.host.matrix(K, n_out, 1, 1, dtype)
        rows = max(1, min(n_out, (1 << 27) // K))
        for r0 in range(0, n_out, rows):
            r = min(rows, n_out - r0)
            w = ((t.randn(r, K, device=self.dev, generator=self.gen) * (0.02 / inv_scale)).to(t.bfloat16)).to(f8)
            assert self.lib.convert(w.data_ptr(), dtype, m.data_ptr + r0 * K, dtype, r * K, 1.0) == 0
            t.cuda.synchronize()
        if inv_scale != 1.0:
            m.quant_scale = inv_scale
        if self.repack:
            m.prepare_tiled()        # what Matrix::loadQuantizedDirect does after uploading file bytes
        return m

    def activation(self, tokens, K, dtype=BF16):
        t = self.torch
        m = self.host.matrix(K, tokens, 1, 1, dtype)
        x = t.randn(tokens, K, device=self.dev, generator=self.gen).to(t.bfloat16 if dtype == BF16 else t.float16)
        assert self.lib.convert(x.data_ptr(), dtype, m.data_ptr, dtype, tokens * K * 2, 1.0) == 0
        t.cuda.synchronize()
        return m

    def output(self, tokens, n_out, dtype=BF16):
        return self.host.matrix(n_out, tokens, 1, 1, dtype)


def build_decode_model(ws: Workspace, tokens: int):
    """Returns (ops, weights_by_shape): ops = list of (W, X, Y, K, N) in graph order."""
    c = QWEN3_8B
    x_h, x_i = ws.activation(tokens, c["hidden"]), ws.activation(tokens, c["inter"])
    y = {n: ws.output(tokens, n) for n in (c["q_out"], c["kv_out"], c["inter"], c["vocab"])}
    y_up = ws.output(tokens, c["inter"])
    y_v = ws.output(tokens, c["kv_out"])
    ops, by_shape = [], {}

    def add(K, N, X, Y):
        W = ws.weight_e5m2(N, K)
        by_shape.setdefault((K, N), []).append(W)
        ops.append((W, X, Y, K, N))

    for _ in range(c["layers"]):
        add(c["hidden"], c["q_out"], x_h, y[c["q_out"]])
        add(c["hidden"], c["kv_out"], x_h, y[c["kv_out"]])
        add(c["hidden"], c["kv_out"], x_h, y_v)
        add(c["hidden"], c["q_out"], x_h, y[c["q_out"]])          # o
        add(c["hidden"], c["inter"], x_h, y[c["inter"]])          # gate
        add(c["hidden"], c["inter"], x_h, y_up)                   # up
        add(c["inter"], c["hidden"], x_i, y[c["q_out"]])          # down
    add(c["hidden"], c["vocab"], x_h, y[c["vocab"]])              # lm_head
    return ops, by_shape


def build_grouped_model(ws: Workspace, tokens: int):
    """The same linears with the projections that share an input stored together, as WeightFile::loadNamedGroup
    stores them: q, k, v in one storage (N = 6144), gate and up in one (N = 24576).  A graph that multiplies the
    grouped storage once and hands out row views of the result issues 4 launches per layer instead of 7."""
    c = QWEN3_8B
    x_h, x_i = ws.activation(tokens, c["hidden"]), ws.activation(tokens, c["inter"])
    n_qkv, n_gu = c["q_out"] + 2 * c["kv_out"], 2 * c["inter"]
    y = {n: ws.output(tokens, n) for n in (n_qkv, c["q_out"], n_gu, c["vocab"])}
    ops = []

    def add(K, N, X, Y):
        ops.append((ws.weight_e5m2(N, K), X, Y, K, N))

    for _ in range(c["layers"]):
        add(c["hidden"], n_qkv, x_h, y[n_qkv])
        add(c["hidden"], c["q_out"], x_h, y[c["q_out"]])          # o
        add(c["hidden"], n_gu, x_h, y[n_gu])
        add(c["inter"], c["hidden"], x_i, y[c["q_out"]])          # down
    add(c["hidden"], c["vocab"], x_h, y[c["vocab"]])              # lm_head
    return ops


DECODE_CTX = 4096


def build_decode_step(ws: Workspace, ctx: int, quantize_on_device: bool = False):
    """The full random-init Qwen3-8B W8A16 model of the C++ DecodeModel, tensors generated on the GPU:
    FP8_E5M2 linears from N(0, 0.02) (bf16, then round to nearest), norms near 1, BF16 embedding and
    a KV cache already holding `ctx` positions of N(0, 1) keys and values.
    quantize_on_device: the linears are generated as BF16 and quantized by Matrix::quantizeWeights, the reference's route for
    a model stored unquantized (cccc/Matrix.cpp:301-355): truncating encoder, per-tensor scale absmax / 57344 -- every
    linear then carries a dequantisation multiplier other than 1."""
    t, c = ws.torch, QWEN3_8B
    model = ws.pkg.host_api.DecodeModel(ws.host, c["layers"], c["hidden"], 32, 8, 128, c["inter"], c["vocab"], ctx)

    def fill_fp8(ptr, n_out, K):
        rows = max(1, min(n_out, (1 << 27) // K))
        for r0 in range(0, n_out, rows):
            r = min(rows, n_out - r0)
            w = (t.randn(r, K, device=ws.dev, generator=ws.gen) * 0.02).to(t.bfloat16).to(t.float8_e5m2)
            assert ws.lib.convert(w.data_ptr(), E5M2, ptr + r0 * K, E5M2, r * K, 1.0) == 0
            t.cuda.synchronize()

    def quantize(li, name, n_out, K):
        w = t.empty(n_out, K, dtype=t.bfloat16, device=ws.dev)
        rows = max(1, min(n_out, (1 << 26) // K))
        for r0 in range(0, n_out, rows):
            r = min(rows, n_out - r0)
            w[r0:r0 + r] = (t.randn(r, K, device=ws.dev, generator=ws.gen) * 0.02).to(t.bfloat16)
        t.cuda.synchronize()
        model.quantize_linear(li, name, w.data_ptr(), E5M2)
        t.cuda.synchronize()
        del w

    def fill_bf16(ptr, n, mean, std):
        step = 1 << 26
        for i0 in range(0, n, step):
            m = min(step, n - i0)
            v = (t.randn(m, device=ws.dev, generator=ws.gen) * std + mean).to(t.bfloat16)
            assert ws.lib.convert(v.data_ptr(), BF16, ptr + i0 * 2, BF16, m * 2, 1.0) == 0
            t.cuda.synchronize()

    shapes = {"wq": (c["q_out"], c["hidden"]), "wk": (c["kv_out"], c["hidden"]), "wv": (c["kv_out"], c["hidden"]),
              "wo": (c["hidden"], c["q_out"]), "w_gate": (c["inter"], c["hidden"]), "w_up": (c["inter"], c["hidden"]),
              "w_down": (c["hidden"], c["inter"])}
    for li in range(c["layers"]):
        for name, (n_out, K) in shapes.items():
            if quantize_on_device:
                quantize(li, name, n_out, K)
            else:
                fill_fp8(model.tensor_ptr(li, name), n_out, K)
        for name, n in (("rms_attn", c["hidden"]), ("rms_ffn", c["hidden"]), ("q_norm", 128), ("k_norm", 128)):
            fill_bf16(model.tensor_ptr(li, name), n, 1.0, 0.1)
        for is_v in (False, True):
            fill_bf16(model.kv_ptr(li, is_v), 8 * ctx * 128, 0.0, 1.0)
    if quantize_on_device:
        quantize(0, "lm_head", c["vocab"], c["hidden"])        # (quantizeLinear keeps the head's tiled copy itself)
    else:
        fill_fp8(model.tensor_ptr(0, "lm_head"), c["vocab"], c["hidden"])
        model.prepare_tiled(0, "lm_head")              # what loading through set_tensor / load_named does
    fill_bf16(model.tensor_ptr(0, "rms_final"), c["hidden"], 1.0, 0.1)
    fill_bf16(model.tensor_ptr(0, "emb"), c["vocab"] * c["hidden"], 0.0, 1.0)
    return model


LLAMA31_8B = dict(layers=32, hidden=4096, n_q=32, n_kv=8, q_out=4096, kv_out=1024, inter=14336, vocab=128256, theta=5e5)


def build_llama_fp4_step(ws: Workspace, ctx: int, block: int = 16, repack: bool = False):
    """Random-init Llama-3.1-8B-shaped model with FP4_E2M1 block-scale linears (the reference's Llama FP4 route: codes and
    one E4M3 scale byte per 16 elements as scripts/convert_weights.py:346-370 packs them), no per-head q/k norms, RoPE
    theta 5e5, BF16 embedding and a KV cache already holding `ctx` positions.  Codes and scale bytes are uniform random
    (scales in [2^-5, 2) so that no NaN code occurs); every layer gets its own device buffers, filled from one host
    pattern rotated per layer."""
    import numpy as np
    t, c = ws.torch, LLAMA31_8B
    model = ws.pkg.host_api.DecodeModel(ws.host, c["layers"], c["hidden"], c["n_q"], c["n_kv"], 128, c["inter"], c["vocab"], ctx, theta=c["theta"])
    model.set_qk_norm(False)
    model.set_repack_linears(repack)            # tiled copies beside the file layout: what the prompt phase's FP4 GEMM reads
    rng = np.random.default_rng(4321)
    shapes = {"wq": (c["q_out"], c["hidden"]), "wk": (c["kv_out"], c["hidden"]), "wv": (c["kv_out"], c["hidden"]),
              "wo": (c["hidden"], c["q_out"]), "w_gate": (c["inter"], c["hidden"]), "w_up": (c["inter"], c["hidden"]),
              "w_down": (c["hidden"], c["inter"]), "lm_head": (c["vocab"], c["hidden"])}
    biggest = max(n * k for n, k in shapes.values())
    codes = rng.integers(0, 256, size=biggest // 2 + 4096, dtype=np.uint8)
    scales = rng.integers(0x10, 0x40, size=biggest // block + 4096, dtype=np.uint8)

    def put(li, name):
        n_out, K = shapes[name]
        off = (li * 131 + len(name) * 17) % 4096
        model.set_tensor(li, name, codes[off:off + n_out * K // 2], FP4)
        model.set_block_scales(li, name, scales[off:off + n_out * K // block])

    def fill_bf16(ptr, n, mean, std):
        step = 1 << 26
        for i0 in range(0, n, step):
            m = min(step, n - i0)
            v = (t.randn(m, device=ws.dev, generator=ws.gen) * std + mean).to(t.bfloat16)
            assert ws.lib.convert(v.data_ptr(), BF16, ptr + i0 * 2, BF16, m * 2, 1.0) == 0
            t.cuda.synchronize()

    for li in range(c["layers"]):
        for name in ("wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down"):
            put(li, name)
        for name in ("rms_attn", "rms_ffn"):
            fill_bf16(model.tensor_ptr(li, name), c["hidden"], 1.0, 0.1)
        for is_v in (False, True):
            fill_bf16(model.kv_ptr(li, is_v), c["n_kv"] * ctx * 128, 0.0, 1.0)
    put(0, "lm_head")
    fill_bf16(model.tensor_ptr(0, "rms_final"), c["hidden"], 1.0, 0.1)
    fill_bf16(model.tensor_ptr(0, "emb"), c["vocab"] * c["hidden"], 0.0, 1.0)
    return model


def llama_fp4_step_bytes(ctx_mean: float, block: int = 16) -> int:
    """Bytes one FP4 decode step must move: codes and scale bytes of every linear once, the keys and values attended to,
    the embedding row, the norm weights and the logits."""
    c = LLAMA31_8B
    elems = c["layers"] * (c["hidden"] * (c["q_out"] + 2 * c["kv_out"]) + c["q_out"] * c["hidden"] + 3 * c["hidden"] * c["inter"]) + c["hidden"] * c["vocab"]
    kv = int(c["layers"] * 2 * c["kv_out"] * 2 * ctx_mean)
    small = c["layers"] * 2 * 2 * c["hidden"] + 2 * c["hidden"] * 2 + c["vocab"] * 2
    return elems // 2 + elems // block + kv + small


def llama_fp4_decode(ws: Workspace, steps: int, warmup: int, use_graph: bool, repack: bool = False):
    """The FP4 decode step as a benchmark entry: tokens / s of the Llama-3.1-8B-shaped model at context DECODE_CTX."""
    model = build_llama_fp4_step(ws, DECODE_CTX, repack=repack)
    start = DECODE_CTX - steps - warmup
    ws.torch.cuda.synchronize()
    model.reset(1, start)
    if warmup:
        model.run(warmup, use_graph)
    ms = model.run(steps, use_graph) / steps
    assert model.pos == DECODE_CTX
    nbytes = llama_fp4_step_bytes(DECODE_CTX - (steps - 1) / 2.0)
    c = LLAMA31_8B
    entry = {"workload": ("full random-init Llama-3.1-8B-shaped FP4_E2M1 block-16 decode step, batch 1, greedy: 32 layers, hidden 4096, 32 q / 8 kv heads x 128, "
                          f"no qk norm, RoPE theta 5e5, SwiGLU 14336, vocab 128256, bf16 KV cache holding {DECODE_CTX} positions"),
             "tok_s": round(1000.0 / ms, 1), "ms_per_step": round(ms, 4), "launch_mode": "hipGraph" if use_graph else "stream",
             "bytes_per_token": nbytes, "GBps": round(nbytes / ms * 1e-6, 1), "frac_of_hbm_bound": round(nbytes / ms * 1e-6 / HBM_PEAK_GBS, 4),
             "launches_per_step": 6 * c["layers"] + 2, "last_token": model.token}
    return entry, model


def prompt_phase(ws: Workspace, model, token_counts=(512, 2048), reps: int = 3, layout: str = "row-major", c=None):
    """The prompt phase of the same model (DecodeModel::prefill, positions 0 .. T - 1): every linear is one quantized GEMM
    with T columns -- the prefill-GEMM kernel of the `prefill` entry on all seven shapes of a layer, on the row-major file bytes (a batch-1
    DecodeModel keeps no tiled copies) -- with the row kernels and the causal attention between them.  Wall clock around the
    call, device synchronised on both sides; best of `reps` after one warm-up call (which also allocates the activations)."""
    import numpy as np
    t, c = ws.torch, (c or QWEN3_8B)
    lin_elems = c["layers"] * (c["hidden"] * (c["q_out"] + 2 * c["kv_out"]) + c["q_out"] * c["hidden"] + 3 * c["hidden"] * c["inter"])
    out = []
    for T in token_counts:
        prompt = [int(v) for v in np.random.default_rng(T).integers(0, c["vocab"], size=T)]
        model.prefill(prompt)
        best = None
        for _ in range(reps):
            t.cuda.synchronize()
            t0 = time.perf_counter()
            model.prefill(prompt)
            t.cuda.synchronize()
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
        # linears 2 T K N each; attention 2 * 2 * 128 * n_q per (token, visible key) pair
        flops = 2.0 * T * lin_elems + 4.0 * 128 * c["n_q"] * c["layers"] * (T * (T + 1) / 2) + 2.0 * c["hidden"] * c["vocab"]
        out.append({"tokens": T, "weights": layout, "ms": round(best * 1e3, 3), "tok_s": round(T / best, 1), "TFLOPs": round(flops / best * 1e-12, 1),
                    "frac_of_bf16_mfma_peak": round(flops / best * 1e-12 / MFMA_BF16_PEAK_TFLOPS, 4)})
    return out


def generate_run(ws: Workspace, model, use_graph: bool, prompt_tokens: int = 2048, new_tokens: int = 128):
    """Prompt and generation together, as a chat turn runs them: DecodeModel::prefill on a prompt from an empty cache, then
    greedy decode steps that carry on from it (one captured step replayed; the capture is inside the clock).  Wall clock,
    device synchronised around each phase; the model keeps the tiled copies of its linears at this point of the run."""
    import numpy as np
    t = ws.torch
    prompt = [int(v) for v in np.random.default_rng(prompt_tokens + 1).integers(0, QWEN3_8B["vocab"], size=prompt_tokens)]
    model.prefill(prompt)                                       # warm-up
    t.cuda.synchronize()
    t0 = time.perf_counter()
    model.prefill(prompt)
    t.cuda.synchronize()
    t1 = time.perf_counter()
    model.run(new_tokens, use_graph)
    t.cuda.synchronize()
    t2 = time.perf_counter()
    assert model.pos == prompt_tokens + new_tokens
    return {"workload": f"{prompt_tokens}-token prompt, then {new_tokens} greedy tokens, Qwen3-8B W8A16, batch 1",
            "time_to_first_token_ms": round((t1 - t0) * 1e3, 3), "decode_ms": round((t2 - t1) * 1e3, 3),
            "decode_tok_s": round(new_tokens / (t2 - t1), 1), "total_ms": round((t2 - t0) * 1e3, 3), "last_token": model.token}


def decode_step_bytes(ctx_mean: float) -> int:
    """Bytes one decode step must move: every linear weight once, the keys and values of the positions
    attended to, the embedding row, the norm weights and the logits."""
    c = QWEN3_8B
    weights = c["layers"] * (c["hidden"] * (c["q_out"] + 2 * c["kv_out"]) + c["q_out"] * c["hidden"] + 3 * c["hidden"] * c["inter"]) + c["hidden"] * c["vocab"]
    kv = int(c["layers"] * 2 * c["kv_out"] * 2 * ctx_mean)
    small = c["layers"] * 2 * (2 * c["hidden"] + 128) + 2 * c["hidden"] * 2 + c["vocab"] * 2
    return weights + kv + small


def gpu_baselines(ws: Workspace, ctx: int, steps_ref: int = 3, steps_torch: int = 10):
    """Two same-GPU baselines of the decode step on a BF16 copy of the model shape (random init):
    (1) reference HIP style: the reference's own HIP kernels (oracle/_ref/libref_hip.so, compiled from
        cccc-hip/hip_functions.cpp) for embedding, RMSNorm, RoPE, causal mask, softmax, sigmoid / mul /
        add, each followed by the device synchronisation that library does, one launch per graph op as in
        scripts/convert_weights.py:488-692, K / V tiled to the query heads, BF16 weights (that build has
        no FP8), GEMMs by torch.matmul (rocBLAS / hipBLASLt, what its Rocblas wrapper calls), driven from
        Python;  (2) plain PyTorch BF16 eager (rms_norm, matmul, scaled_dot_product_attention), no syncs.
    Returns a dict, or None when the reference library was not built."""
    import ctypes
    from oracle import ref_hip
    t, c = ws.torch, QWEN3_8B
    R = ref_hip.lib()
    dev, bf = ws.dev, t.bfloat16
    H, NQ, NKV, D, I, V = c["hidden"], 32, 8, 128, c["inter"], c["vocab"]

    def w(n_out, k):
        return (t.randn(n_out, k, device=dev, generator=ws.gen) * 0.02).to(bf)

    layers = [dict(wq=w(NQ * D, H), wk=w(NKV * D, H), wv=w(NKV * D, H), wo=w(H, NQ * D), wg=w(I, H), wu=w(I, H), wd=w(H, I),
                   n1=t.ones(H, device=dev, dtype=bf), n2=t.ones(H, device=dev, dtype=bf), qn=t.ones(D, device=dev, dtype=bf), kn=t.ones(D, device=dev, dtype=bf),
                   kc=t.randn(NKV, ctx, D, device=dev, generator=ws.gen).to(bf), vc=t.randn(NKV, ctx, D, device=dev, generator=ws.gen).to(bf))
              for _ in range(c["layers"])]
    emb = t.randn(V, H, device=dev, generator=ws.gen).to(bf)
    lm, nf = w(V, H), t.ones(H, device=dev, dtype=bf)
    inv_freq = 1.0 / (1e6 ** (t.arange(0, D, 2, device=dev, dtype=t.float32) / D))
    ang = t.arange(ctx, device=dev, dtype=t.float32)[:, None] * inv_freq[None, :]
    cos, sin = ang.cos().to(bf).contiguous(), ang.sin().to(bf).contiguous()
    scale = 1.0 / 128.0 ** 0.5
    p = lambda x: ctypes.c_void_p(x.data_ptr())
    f32 = ctypes.c_float
    out = {}

    if R is not None:
        kt, vt = t.empty(NQ, ctx, D, device=dev, dtype=bf), t.empty(NQ, ctx, D, device=dev, dtype=bf)

        def rms(x, wgt, outer, inner):
            y = t.empty_like(x)
            assert R.hip_rms_norm_fwd(3, p(x), p(y), p(wgt), None, outer, inner, f32(1e-6)) == 0
            return y

        def ref_step(token, pos):
            ids = t.tensor([float(token)], device=dev)
            x = t.empty(H, device=dev, dtype=bf)
            assert R.hip_embed_fwd(3, p(ids), p(emb), p(x), H, 1, 1) == 0
            for L in layers:
                xn = rms(x, L["n1"], 1, H)
                q, k, v = L["wq"] @ xn, L["wk"] @ xn, L["wv"] @ xn
                qn, kn = rms(q, L["qn"], NQ, D), rms(k, L["kn"], NKV, D)
                qr, kr = t.empty_like(qn), t.empty_like(kn)
                assert R.hip_rope_fwd(3, p(qn), p(qr), p(cos), p(sin), D, 1, NQ, pos) == 0
                assert R.hip_rope_fwd(3, p(kn), p(kr), p(cos), p(sin), D, 1, NKV, pos) == 0
                L["kc"][:, pos] = kr.view(NKV, D)
                L["vc"][:, pos] = v.view(NKV, D)
                kt.view(NKV, NQ // NKV, ctx, D).copy_(L["kc"][:, None])           # GQA by tiling K and V to the query heads
                vt.view(NKV, NQ // NKV, ctx, D).copy_(L["vc"][:, None])
                scores = (t.bmm(kt, qr.view(NQ, D, 1)) * scale).view(NQ, ctx)
                assert R.hip_causal_mask(3, p(scores), 1, ctx, NQ, pos) == 0
                assert R.hip_softmax_bf16(p(scores), p(scores), ctx, NQ, f32(1.0), f32(0.0)) == 0
                att = t.bmm(scores.view(NQ, 1, ctx), vt).view(NQ * D)
                o = L["wo"] @ att
                r1 = t.empty_like(x)
                assert R.hip_add(3, p(x), p(o), p(r1), H, f32(1.0), f32(1.0)) == 0
                rn = rms(r1, L["n2"], 1, H)
                g, u = L["wg"] @ rn, L["wu"] @ rn
                sg, si, ga = t.empty_like(g), t.empty_like(g), t.empty_like(g)
                assert R.hip_sigmoid_bf16(p(sg), p(g), I, f32(1.0), f32(0.0)) == 0
                assert R.hip_mul(3, p(g), p(sg), p(si), I, f32(1.0), f32(0.0)) == 0
                assert R.hip_mul(3, p(si), p(u), p(ga), I, f32(1.0), f32(0.0)) == 0
                dn = L["wd"] @ ga
                x = t.empty_like(r1)
                assert R.hip_add(3, p(r1), p(dn), p(x), H, f32(1.0), f32(1.0)) == 0
            logits = lm @ rms(x, nf, 1, H)
            return int(logits.argmax())

        tok = ref_step(1, ctx - steps_ref - 1)
        t.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps_ref):
            tok = ref_step(tok, ctx - steps_ref + i)
        t.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / steps_ref
        out["reference_hip_style"] = {"tok_s": round(1e3 / ms, 2), "ms_per_step": round(ms, 3), "steps": steps_ref, "weights": "bf16",
                                      "what": "reference's own HIP kernels (norm, rope, mask, softmax, silu, add; each syncs the device) + rocBLAS/hipBLASLt GEMMs via torch.matmul, one launch per graph op, driven from Python"}
        del kt, vt

    F = t.nn.functional

    def torch_step(token, pos):
        x = emb[token]
        for L in layers:
            xn = F.rms_norm(x, (H,), L["n1"], 1e-6)
            q, k, v = (L["wq"] @ xn).view(NQ, D), (L["wk"] @ xn).view(NKV, D), L["wv"] @ xn
            q, k = F.rms_norm(q, (D,), L["qn"], 1e-6), F.rms_norm(k, (D,), L["kn"], 1e-6)
            cs, sn = cos[pos], sin[pos]
            q = t.cat([q[:, :64] * cs - q[:, 64:] * sn, q[:, 64:] * cs + q[:, :64] * sn], dim=1)
            k = t.cat([k[:, :64] * cs - k[:, 64:] * sn, k[:, 64:] * cs + k[:, :64] * sn], dim=1)
            L["kc"][:, pos] = k
            L["vc"][:, pos] = v.view(NKV, D)
            att = F.scaled_dot_product_attention(q.view(1, NQ, 1, D), L["kc"][None, :, :pos + 1], L["vc"][None, :, :pos + 1], enable_gqa=True).view(NQ * D)
            r1 = x + L["wo"] @ att
            rn = F.rms_norm(r1, (H,), L["n2"], 1e-6)
            x = r1 + L["wd"] @ (F.silu(L["wg"] @ rn) * (L["wu"] @ rn))
        return (lm @ F.rms_norm(x, (H,), nf, 1e-6)).argmax()

    with t.no_grad():
        tok = torch_step(1, ctx - steps_torch - 1)
        t.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps_torch):
            tok = torch_step(tok, ctx - steps_torch + i)
        t.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / steps_torch
    out["torch_bf16_eager"] = {"tok_s": round(1e3 / ms, 2), "ms_per_step": round(ms, 3), "steps": steps_torch, "weights": "bf16",
                               "what": "PyTorch-ROCm eager BF16 (rms_norm, matmul, scaled_dot_product_attention), no device syncs inside a step"}

    def rope_rows(x, n):                                        # x [n, heads, D], positions 0 .. n - 1
        cs, sn = cos[:n, None, :], sin[:n, None, :]
        return t.cat([x[..., :64] * cs - x[..., 64:] * sn, x[..., 64:] * cs + x[..., :64] * sn], dim=-1)

    def torch_prompt(tokens):
        n = tokens.numel()
        x = emb[tokens]
        for L in layers:
            xn = F.rms_norm(x, (H,), L["n1"], 1e-6)
            q, k, v = (xn @ L["wq"].T).view(n, NQ, D), (xn @ L["wk"].T).view(n, NKV, D), (xn @ L["wv"].T).view(n, NKV, D)
            q, k = rope_rows(F.rms_norm(q, (D,), L["qn"], 1e-6), n), rope_rows(F.rms_norm(k, (D,), L["kn"], 1e-6), n)
            L["kc"][:, :n] = k.transpose(0, 1)
            L["vc"][:, :n] = v.transpose(0, 1)
            att = F.scaled_dot_product_attention(q.transpose(0, 1)[None], L["kc"][None, :, :n], L["vc"][None, :, :n], is_causal=True, enable_gqa=True)
            r1 = x + att[0].transpose(0, 1).reshape(n, NQ * D) @ L["wo"].T
            rn = F.rms_norm(r1, (H,), L["n2"], 1e-6)
            x = r1 + (F.silu(rn @ L["wg"].T) * (rn @ L["wu"].T)) @ L["wd"].T
        return (lm @ F.rms_norm(x[-1], (H,), nf, 1e-6)).argmax()

    n_prompt = min(2048, ctx)
    prompt = t.randint(0, V, (n_prompt,), device=dev, generator=ws.gen)
    with t.no_grad():
        torch_prompt(prompt)
        best = None
        for _ in range(3):
            t.cuda.synchronize()
            t0 = time.perf_counter()
            torch_prompt(prompt)
            t.cuda.synchronize()
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
    out["torch_bf16_eager_prompt"] = {"tokens": n_prompt, "ms": round(best * 1e3, 3), "tok_s": round(n_prompt / best, 1), "weights": "bf16",
                                      "what": "the prompt phase in PyTorch-ROCm eager BF16 (rms_norm, matmul = hipBLASLt, causal scaled_dot_product_attention with GQA)"}
    return out


def time_chain(ws, ops, steps, warmup, use_graph):
    ms = ws.bench.linear_chain([o[0] for o in ops], [o[1] for o in ops], [o[2] for o in ops], steps, warmup, use_graph)
    if ms < 0:
        raise RuntimeError(f"bench chain failed with code {ms}")
    return ms


def shape_sweep(ws, by_shape, token_counts, use_graph, comparators=True):
    """Per-shape GEMV rates with weights rotating over distinct buffers (no cache reuse).  floor_us: a launch that only
    streams the same weight buffers with 16-byte loads (host/bench_kernels.hip), i.e. what the memory side alone costs."""
    out = []
    for (K, N) in QWEN_SHAPES:
        weights = by_shape[(K, N)]
        floor_us = ws.bench.floor_us([W.data_ptr for W in weights], K * N)
        for M in token_counts:
            X, Y = ws.activation(M, K), ws.output(M, N)
            reps = max(1, min(8, (2 << 30) // (K * N * len(weights))))
            ops = [(W, X, Y, K, N) for W in weights] * reps
            ms = time_chain(ws, ops, 3, 1, use_graph)
            us = ms * 1000.0 / (3 * len(ops))
            gbs = gemv_bytes(K, N, M) / us * 1e-3
            assert ws.lib.linear(weights[0].data_ptr, E5M2, X.data_ptr, Y.data_ptr, N, M, K) == 0
            row = {"K": K, "N": N, "M": M, "us": round(us, 2), "floor_us": round(floor_us, 2), "floor_over_us": round(floor_us / us, 3),
                   "GBps": round(gbs, 1), "frac": round(gbs / HBM_PEAK_GBS, 4), "launch_mode": "hipGraph" if use_graph else "stream",
                   "kernel": ws.lib.last_kernel(), "distinct_weight_MB": round(K * N * len(weights) / 2 ** 20)}
            if M == 1 and comparators:
                row.update(same_gpu_comparators(ws, weights, K, N, M))
            out.append(row)
    return out


SCALED_INV_SCALE = 0.2 / 57344.0       # absmax / max_code of a weight whose largest element is 0.2 (cccc/Matrix.cpp:338-352): ten sigma, no Inf codes


def variant_sweep(ws, by_shape, token_counts=(1, 16), use_graph=False):
    """The routes of the same GEMV that a model quantized by the reference takes instead of `sweep`'s (scale 1, E5M2, BF16):
    "e5m2_scaled" -- the same E5M2 weights with a per-tensor dequantisation multiplier other than 1 (every weight
    Matrix::quantizeWeights produces carries absmax / 57344, cccc/Matrix.cpp:338-352): the kernels then decode to FP32,
    multiply and round to BF16 instead of one hardware conversion; "e4m3_scaled" -- FP8_E4M3 codes with a scale (the hy-mt2
    files, scripts/convert_weights.py:272-313); "e5m2_half" -- HALF activations and outputs (the reference's Qwen3 inis
    default to data_type = half, scripts/convert_weights.py:728-729; branch cccc/cublas_real.h:921-938).  Each row carries
    the time of the plain route on the same shape (`base_us`, from `sweep`) when it was measured."""
    out = []
    for (K, N) in QWEN_SHAPES:
        base = by_shape[(K, N)]
        n_w = len(base) if K * N * len(base) <= (1 << 30) else max(1, (1 << 30) // (K * N))
        e4 = [ws.weight_fp8(N, K, E4M3, SCALED_INV_SCALE * 128.0) for _ in range(n_w)]       # 448 instead of 57344
        for route, weights, act in (("e5m2_scaled", base, BF16), ("e4m3_scaled", e4, BF16), ("e5m2_half", base, HALF)):
            if route == "e5m2_scaled":
                for W in weights:
                    W.quant_scale = SCALED_INV_SCALE
            for M in token_counts:
                X, Y = ws.activation(M, K, act), ws.output(M, N, act)
                reps = max(1, min(8, (2 << 30) // (K * N * len(weights))))
                ops = [(W, X, Y, K, N) for W in weights] * reps
                ms = time_chain(ws, ops, 3, 1, use_graph)
                us = ms * 1000.0 / (3 * len(ops))
                gbs = gemv_bytes(K, N, M) / us * 1e-3
                assert ws.lib.linear(weights[0].data_ptr, weights[0].dtype, X.data_ptr, Y.data_ptr, N, M, K, inv_scale=weights[0].quant_scale, act_type=act) == 0
                out.append({"route": route, "K": K, "N": N, "M": M, "us": round(us, 2), "GBps": round(gbs, 1), "frac": round(gbs / HBM_PEAK_GBS, 4),
                            "kernel": ws.lib.last_kernel()})
            if route == "e5m2_scaled":
                for W in weights:
                    W.quant_scale = 1.0
        ws.keep.append(e4)                 # freed with everything else (freeing mid-run slows what runs next)
    return out


def same_gpu_comparators(ws, weights, K, N, M, max_ops=24):
    """The same linear on the same GPU the way the reference's unified GEMM does it (cccc/cublas_real.h:943-964
    expressed with HIP calls): dequantise the whole weight to a BF16 workspace, then a BF16 GEMM with FP32
    accumulation (rocBLAS / hipBLASLt through torch), with the device synchronisation the reference's kernel
    wrappers make after each step -- and the plain BF16 GEMM alone, which is what the reference's HIP build
    (no FP8 support) would run on BF16 weights.  Microseconds per linear over rotating weights."""
    t = ws.torch
    wsb = t.empty(N, K, dtype=t.bfloat16, device=ws.dev)
    x = t.randn(M, K, device=ws.dev, generator=ws.gen).to(t.bfloat16)
    ops = weights[:max_ops]
    out = {}
    for name, sync in (("ref_style_us", True), ("ref_style_nosync_us", False)):
        for rep in range(2):                                   # first pass warms up
            t.cuda.synchronize()
            t0 = time.perf_counter()
            for W in ops:
                assert ws.lib.convert(W.data_ptr, E5M2, wsb.data_ptr(), BF16, N * K, 1.0) == 0
                if sync:
                    t.cuda.synchronize()
                y = x @ wsb.T
                if sync:
                    t.cuda.synchronize()
            t.cuda.synchronize()
            out[name] = round((time.perf_counter() - t0) * 1e6 / len(ops), 2)
    n_bf = max(2, min(8, (1 << 30) // (2 * K * N)))
    bf = [t.randn(N, K, device=ws.dev, generator=ws.gen).to(t.bfloat16) for _ in range(n_bf)]
    for rep in range(2):
        t.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(4 * n_bf):
            y = x @ bf[i % n_bf].T
        t.cuda.synchronize()
        out["bf16_gemm_us"] = round((time.perf_counter() - t0) * 1e6 / (4 * n_bf), 2)
    ws.keep.append((wsb, bf, x))           # freed with everything else (freeing GBs mid-run slows what is timed next)
    return out


def prefill_cases(ws, by_shape):
    """The W8A16 prefill GEMM workload: M in {512, 2048} x the two MLP shapes, with the plain BF16 GEMM
    of the vendor library (torch.matmul) on the same shape beside it.  Three passes over the four cases -- this build's
    kernel, the same with a per-tensor multiplier, the vendor GEMM -- because seconds of dense vendor GEMMs, and freeing
    their operands, depress whatever is timed next by several per cent; nothing is freed until the last case is done."""
    t = ws.torch
    cases = [(K, N, M) for (K, N) in ((4096, 12288), (12288, 4096)) for M in (512, 2048)]
    rows, chains = {}, {}
    for (K, N, M) in cases:
        weights = by_shape[(K, N)][:16]
        X, Y = ws.activation(M, K), ws.output(M, N)
        ops = [(W, X, Y, K, N) for W in weights]
        steps = 40 if M <= 512 else 12                  # 30 ms or more per figure: shorter bursts run at other clocks
        chains[(K, N, M)] = (ops, steps, weights)
        us = time_chain(ws, ops, steps, steps // 4, False) * 1000.0 / (steps * len(ops))
        tf = 2.0 * M * K * N / us * 1e-6
        rows[(K, N, M)] = {"K": K, "N": N, "M": M, "us": round(us, 2), "TFLOPs": round(tf, 1), "frac_of_bf16_mfma_peak": round(tf / MFMA_BF16_PEAK_TFLOPS, 4),
                           "kernel": ws.lib.last_kernel()}
    # the same launches with a per-tensor dequantisation multiplier (the route of a weight quantized on load)
    for (K, N, M) in cases:
        ops, steps, weights = chains[(K, N, M)]
        for W in weights:
            W.quant_scale = SCALED_INV_SCALE
        us_scaled = time_chain(ws, ops, steps, steps // 4, False) * 1000.0 / (steps * len(ops))
        for W in weights:
            W.quant_scale = 1.0
        tf_scaled = 2.0 * M * K * N / us_scaled * 1e-6
        rows[(K, N, M)].update({"scaled_us": round(us_scaled, 2), "scaled_TFLOPs": round(tf_scaled, 1),
                                "scaled_frac_of_bf16_mfma_peak": round(tf_scaled / MFMA_BF16_PEAK_TFLOPS, 4)})
    bf = {}
    for (K, N, M) in cases:
        if (K, N) not in bf:
            bf[(K, N)] = [t.randn(N, K, device=ws.dev, generator=ws.gen).to(t.bfloat16) for _ in range(4)]
        x = t.randn(M, K, device=ws.dev, generator=ws.gen).to(t.bfloat16)
        for rep in range(2):
            t.cuda.synchronize()
            t0 = time.perf_counter()
            for i in range(16):
                y = x @ bf[(K, N)][i % 4].T
            t.cuda.synchronize()
            lib_us = (time.perf_counter() - t0) * 1e6 / 16
        rows[(K, N, M)].update({"vendor_bf16_gemm_us": round(lib_us, 2), "vendor_bf16_gemm_TFLOPs": round(2.0 * M * K * N / lib_us * 1e-6, 1)})
        ws.keep.append((x, y))
    ws.keep.append((bf, chains))
    return [rows[c] for c in cases]


LLAMA_SHAPES = [(4096, 4096), (4096, 1024), (4096, 14336), (14336, 4096), (4096, 128256)]     # (K, N)


def fp4_bytes(K, N, M, block):
    return K * N // 2 + K * N // block + 2 * M * K + 2 * M * N


def fp4_sweep(ws, token_counts=(1, 4, 16), prefill_tokens=(512, 2048)):
    """The FP4 workload: Llama-3.1-8B-shaped FP4 block-scale GEMVs, block 16 (the reference's format) and 32, weights
    rotating over at least 512 MiB of distinct buffers, with their load-time tiled copies registered as the host mirror
    registers them (unless --no-repack); M = 1 is the configuration's own row, 4 and 16 ride along.  Second list: the
    FP4 prefill GEMM on the two MLP shapes (FLOPs 2 M K N against the BF16 matrix-core peak)."""
    t = ws.torch
    out, prefill, keep = [], [], []                 # buffers stay allocated until the sweep is over (freeing slows what runs next)
    pool = t.randint(0, 255, (800 << 20,), dtype=t.uint8, device=ws.dev)        # what the streaming floor reads
    keep.append(([], [], [pool]))
    for (K, N) in LLAMA_SHAPES:
        for block in (16, 32):
            per = K * N // 2 + K * N // block
            n_w = max(2, min(48, (768 << 20) // per))
            span = (per + 4095) // 4096 * 4096
            floor_ptrs = [pool.data_ptr() + i * span for i in range(max(1, min(n_w, (800 << 20) // span)))]
            floor_us = ws.bench.floor_us(floor_ptrs, per)
            nib = [t.randint(0, 256, (N, K // 2), dtype=t.uint8, device=ws.dev, generator=ws.gen) for _ in range(n_w)]
            sc = [t.randint(0x10, 0x40, (N, K // block), dtype=t.uint8, device=ws.dev, generator=ws.gen) for _ in range(n_w)]
            tiled = []
            if ws.repack:
                for w, s_ in zip(nib, sc):
                    tiled.append(t.empty(ws.lib.tiled_size(FP4, N, K), dtype=t.uint8, device=ws.dev))
                    assert ws.lib.weight_prepare_fp4(w.data_ptr(), s_.data_ptr(), block, N, K, tiled[-1].data_ptr()) == 0
            iters = max(20, min(400, (4 << 30) // per))
            mlp = (K, N) in ((4096, 14336), (14336, 4096))
            for M in tuple(token_counts) + (tuple(prefill_tokens) if mlp and block == 16 else ()):
                X, Y = ws.activation(M, K), ws.output(M, N)
                n_it = iters if M <= 16 else 96
                ms = ws.bench.fp4_chain([w.data_ptr() for w in nib], [s_.data_ptr() for s_ in sc], X.data_ptr, Y.data_ptr, N, M, K, block, n_it, 5)
                if ms < 0:
                    raise RuntimeError(f"fp4 chain failed: {ms}")
                us = ms * 1000.0 / n_it
                if M <= 16:
                    gbs = fp4_bytes(K, N, M, block) / us * 1e-3
                    out.append({"K": K, "N": N, "M": M, "block": block, "us": round(us, 2), "floor_us": round(floor_us, 2), "floor_over_us": round(floor_us / us, 3),
                                "GBps": round(gbs, 1), "frac": round(gbs / HBM_PEAK_GBS, 4),
                                "kernel": ws.lib.last_kernel(), "distinct_weight_MB": round(per * n_w / 2 ** 20)})
                else:
                    tf = 2.0 * M * K * N / us * 1e-6
                    prefill.append({"K": K, "N": N, "M": M, "block": block, "us": round(us, 2), "TFLOPs": round(tf, 1),
                                    "frac_of_bf16_mfma_peak": round(tf / MFMA_BF16_PEAK_TFLOPS, 4), "kernel": ws.lib.last_kernel()})
                del X, Y
            keep.append((nib, sc, tiled))
    for nib, sc, tiled in keep:
        for w in nib:
            ws.lib.weight_release(w.data_ptr())
    return out, prefill


def cpu_baseline(pkg, threads, unit):
    """The reference CPU route (scalar dequantisation of the whole weight to float32 + cblas_sgemm, cccc/Matrix.cpp:1258-1267)
    on the linear layers of the decode workload at M=1, on a bounded sample: 24 of the 36 layers (the same seven
    weights walked 24 times: 4.6 GB of codes per walk, far beyond the host caches), timed three times -- about
    ten seconds of CPU work."""
    import numpy as np
    from oracle import oracle, synth
    c = QWEN3_8B
    shapes = [(c["hidden"], c["q_out"]), (c["hidden"], c["kv_out"]), (c["hidden"], c["kv_out"]), (c["hidden"], c["q_out"]),
              (c["hidden"], c["inter"]), (c["hidden"], c["inter"]), (c["inter"], c["hidden"])]
    fn, blas = oracle.find_cblas_sgemm()
    rng = np.random.default_rng(7)
    data = []
    for K, N in shapes:
        W = rng.integers(0, 0x7C, size=(N, K), dtype=np.uint8)
        X = synth.activations(7, 1, K)
        data.append((W, X, K, N))
    layers_sampled = 24
    runs = []
    t_end = time.time() + 30.0
    for rep in range(4):
        td = tg = 0.0
        for _ in range(1 if rep == 0 else layers_sampled):         # pass 0 warms up
            for W, X, K, N in data:
                _, a, b = oracle.cpu_linear(W, oracle.E5M2, 1.0, None, 16, X, N, 1, K, sgemm=fn, threads=threads)
                td, tg = td + a, tg + b
        if rep:
            runs.append((td + tg, td, tg))
        if time.time() > t_end and runs:
            break
    runs.sort()
    total, td, tg = runs[len(runs) // 2]
    layer_bytes = sum(gemv_bytes(K, N, 1) for _, _, K, N in data)
    gbs = layers_sampled * layer_bytes / total * 1e-9
    model_bytes = c["layers"] * layer_bytes + gemv_bytes(c["hidden"], c["vocab"], 1)
    out = {"cores": threads, "kind": "port",
           "sample": f"{layers_sampled} of 36 Qwen3-8B layers (q,k,v,o,gate,up,down) at M=1, {layers_sampled * layer_bytes} bytes, median of {len(runs)} timed walks after a warm-up",
           "linears_GBps": round(gbs, 3), "dequant_s": round(td, 4), "gemm_s": round(tg, 4), "blas": blas}
    if unit == "tok/s":
        # the linear layers of one token at the sampled rate; attention, norms and the rest of the CPU route are not timed, so this is an upper bound
        out.update({"value": round(gbs * 1e9 / model_bytes, 4), "unit": "tok/s",
                    "scaled": "linear layers of one token (7.57 GB of codes) at the sampled rate; upper bound for the CPU route"})
    else:
        out.update({"value": round(gbs, 3), "unit": "GB/s"})
    return out


def north_star_summary(line):
    """The headline figures of the line once more, compact and last, so that they survive a reader that keeps only the tail of
    the output: fractions of the 8 TB/s HBM peak for the GEMVs (rows = K x N, columns = token counts), fractions of the
    2.5 PFLOP/s BF16 matrix-core peak for the prefill GEMMs, the decode step against its HBM bound."""
    def grid(rows, key="frac", extra=lambda r: True):
        out = {}
        for r in rows:
            if extra(r):
                out.setdefault(f"{r['K']}x{r['N']}", {})[f"M{r['M']}"] = r[key]
        return out
    # least important first: a reader that keeps only the last characters still gets the decode, GEMV and prefill figures
    ns = {}
    if "fp4_decode_step" in line:
        ns["fp4_decode_tok_s"] = line["fp4_decode_step"]["tok_s"]
    if "fp4_prefill" in line:
        ns["fp4_prefill_frac"] = grid(line["fp4_prefill"], "frac_of_bf16_mfma_peak")
    if "fp4_sweep" in line:
        ns["fp4_b16_gemv_frac"] = grid(line["fp4_sweep"], extra=lambda r: r["block"] == 16)
    if "sweep_variants" in line:
        for route in ("e5m2_half", "e4m3_scaled", "e5m2_scaled"):
            ns["gemv_frac_" + route] = grid(line["sweep_variants"], extra=lambda r, route=route: r["route"] == route)
    if "sweep" in line:
        ns["gemv_floor_us"] = {f"{r['K']}x{r['N']}": r["floor_us"] for r in line["sweep"] if r["M"] == line["sweep"][0]["M"]}
        ns["gemv_us"] = grid(line["sweep"], "us")
    if "prefill" in line:
        ns["prefill_frac_scaled"] = grid(line["prefill"], "scaled_frac_of_bf16_mfma_peak")
        ns["prefill_frac"] = grid(line["prefill"], "frac_of_bf16_mfma_peak")
    if "sweep" in line:
        ns["gemv_frac"] = grid(line["sweep"])
    if "quant_gemv" in line:
        ns["gemv_chain_frac"] = line["quant_gemv"]["frac_of_hbm_peak"]
        ns["gemv_chain_grouped_frac"] = line.get("quant_gemv_grouped", {}).get("frac_of_hbm_peak")
    if "scaled_decode_step" in line:
        ns["decode_ms_scaled_weights"] = line["scaled_decode_step"]["ms_per_step"]
    ns.update({"decode_ms_exact_attention": line.get("ms_per_step_exact_attention"), "dominant_kernel_frac": line["roofline"]["frac"],
               "decode_frac_of_hbm_bound": line.get("decode_step_frac_of_hbm_bound"), "decode_ms": line["ms_per_step"], "decode_tok_s": line["value"]})
    return ns


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="decode_step", choices=["decode_step", "decode_linears", "gemv", "prefill", "copy", "prompt_attention", "floor", "prefill_variants"])
    ap.add_argument("--shape", default="4096,12288", help="K,N for --workload gemv / prefill")
    ap.add_argument("--tokens", type=int, default=1)
    ap.add_argument("--weights", default="fp8", choices=["fp8", "fp4"], help="weight format of --workload gemv / prefill (fp4: E2M1 codes + E4M3 block scales)")
    ap.add_argument("--block", type=int, default=16, choices=[16, 32], help="FP4 block length")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-sweep", action="store_true")
    ap.add_argument("--no-fp4-step", action="store_true", help="skip the Llama-3.1-8B-shaped FP4 decode step")
    ap.add_argument("--no-prompt", action="store_true", help="skip the prompt-phase (prefill) measurement of the decode model")
    ap.add_argument("--sweep-tokens", default="1,4,16", help="token counts of the per-shape GEMV sweep")
    ap.add_argument("--no-baselines", action="store_true", help="skip the same-GPU BF16 baselines of the decode step")
    ap.add_argument("--no-scaled-step", action="store_true", help="skip the decode step on weights quantized on the device (per-tensor scales)")
    ap.add_argument("--no-repack", action="store_true", help="do not build the load-time tiled weight copies (tokens 3..16 then use the row-major kernels)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this path runs on one GPU (no sharding, no collectives); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    import __graft_entry__
    pkg = __graft_entry__.load_package()
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    if args.workload == "copy":
        # counter calibration: a plain device copy kernel of known size (reads and writes 256 MiB per launch)
        n = 256 << 20
        src = torch.randint(0, 255, (n,), dtype=torch.uint8, device="cuda:0")
        dst = torch.empty_like(src)
        for _ in range(args.steps):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"workload": "copy", "bytes_read_per_launch": n, "bytes_written_per_launch": n, "launches": args.steps}))
        return
    if args.workload == "prompt_attention":
        # the prompt phase's causal attention kernel alone (for counter runs): --tokens query tokens from position 0,
        # Qwen3-8B heads (32 q / 8 kv x 128), --steps launches after --warmup
        import ctypes
        lib, dev = pkg.library(), torch.device("cuda:0")
        T = max(args.tokens, 16)
        q = torch.randn(T, 32, 128, device=dev).to(torch.bfloat16)
        kc, vc = torch.randn(8, T, 128, device=dev).to(torch.bfloat16), torch.randn(8, T, 128, device=dev).to(torch.bfloat16)
        y = torch.zeros(T, 32, 128, device=dev, dtype=torch.bfloat16)
        p = lambda x: ctypes.c_void_p(x.data_ptr())
        launch = lambda: lib.c.hip_attention_prefill_bf16(p(q), p(kc), p(vc), p(y), 32, 8, 128, T, T, 0)
        for _ in range(args.warmup):
            assert launch() == 0
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(args.steps):
            launch()
        e1.record()
        torch.cuda.synchronize()
        print(json.dumps({"workload": "prompt_attention", "tokens": T, "launches": args.steps, "us_per_launch": round(e0.elapsed_time(e1) * 1e3 / args.steps, 2)}))
        return
    ws = Workspace(pkg, torch)
    ws.repack = not args.no_repack
    use_graph = not args.no_graph
    extra = {}
    if args.workload == "floor":
        # What a launch costs on this GPU when it only streams its bytes, for the byte counts of the GEMV sweeps (FP8 Qwen3-8B
        # shapes, FP4 block-16 Llama-3.1-8B shapes), over rotating buffers of at least 512 MiB in total; and what a launch
        # costs when it does nothing (dependent launches inside one hipGraph).
        rows = []
        sizes = ([("fp8", K, N, K * N) for K, N in QWEN_SHAPES] + [("fp8 q,k,v together", 4096, 6144, 4096 * 6144), ("fp8 gate,up together", 4096, 24576, 4096 * 24576)]
                 + [("fp4_b16", K, N, K * N // 2 + K * N // 16) for K, N in LLAMA_SHAPES])
        pool = torch.randint(0, 255, (1 << 30,), dtype=torch.uint8, device=ws.dev)
        for fmt, K, N, nbytes in sizes:
            span = (nbytes + 4095) // 4096 * 4096
            n_buf = max(1, min(64, (1 << 30) // span))
            ptrs = [pool.data_ptr() + i * span for i in range(n_buf)]
            best = {f"{'contiguous' if c else 'strided'}_{'8' if p else '4'}KiB_{w}": round(min(ws.bench.floor_read_us(ptrs, nbytes, wgs_per_cu=w, contiguous=c, pipelined=p) for _ in range(2)), 2)
                    for c in (False, True) for p in (True, False) for w in (2, 4, 8)}
            us = min(best.values())
            rows.append({"weights": fmt, "K": K, "N": N, "bytes": nbytes, "floor_us": us, "GBps": round(nbytes / us * 1e-3, 1),
                         "frac_of_hbm_peak": round(nbytes / us * 1e-3 / HBM_PEAK_GBS, 4), "us_by_pattern_bytes_in_flight_per_wave_and_workgroups_per_cu": best})
        print(json.dumps({"workload": "floor", "what": "streaming read of the sweep byte counts with 16-byte non-temporal loads, KiB pieces at a grid stride or one contiguous range per workgroup, rotating buffers (1 GiB pool); "
                                                       "empty and one-trip launches inside a hipGraph",
                          "launch_us_empty": round(ws.bench.launch_us(0), 3), "launch_us_one_trip": round(ws.bench.launch_us(1), 3), "rows": rows}))
        return

    if args.workload == "prefill_variants":
        # The FP8 prefill GEMM against the variants of it that were tried and not adopted (host/bench_gemm_variants.hip):
        # conversions spread between the matrix-core instructions, a 4 x 2 blocking of the tiles over the XCDs, other
        # tile shapes; and where a workgroup's time goes (wave 0's clock: conversion + wait for weight bytes / barrier /
        # rest of the k-tile).  Same weights (tiled copies of 8 distinct E5M2 matrices), activations and launch count
        # for every row; every variant's output is compared with its tile's "block" variant (bit for bit) and the product entry's.
        rows = []
        for (K, N) in ((4096, 12288), (12288, 4096)):
            codes = [torch.randn(N, K, device=ws.dev, generator=ws.gen).mul_(0.02).to(torch.bfloat16).to(torch.float8_e5m2) for _ in range(8)]
            tiled = [torch.empty(ws.lib.tiled_size(E5M2, N, K), dtype=torch.uint8, device=ws.dev) for _ in codes]
            for c_, t_ in zip(codes, tiled):
                assert ws.lib.weight_prepare(c_.data_ptr(), E5M2, N, K, K, t_.data_ptr()) == 0
            ptrs = [t_.data_ptr() for t_ in tiled]
            for M in (512, 2048):
                x = torch.randn(M, K, device=ws.dev, generator=ws.gen).to(torch.bfloat16)
                y, y_ref = torch.zeros(M, N, device=ws.dev, dtype=torch.bfloat16), torch.zeros(M, N, device=ws.dev, dtype=torch.bfloat16)
                partial = torch.empty(4 * M * N, device=ws.dev, dtype=torch.float32)
                rm_ptrs = [c_.data_ptr() for c_ in codes]
                n_it = 600 if M <= 512 else 200                 # 30 ms or more per figure: shorter bursts run at other clocks
                us, _ = ws.bench.gemm_variant(8, 0, rm_ptrs, x.data_ptr(), y_ref.data_ptr(), N, M, K, iters=n_it, warmup=n_it // 4)
                row = {"K": K, "N": N, "M": M, "product_us": round(us, 2), "product_kernel": ws.lib.last_kernel(), "variants": {}}
                names = {0: "block", 1: "spread", 2: "raster4x2", 3: "spread+raster4x2"}
                tiles = {0: "128x256", 3: "64x256", 4: "128x192", 1: "64x192", 5: "128x256_split2", 6: "64x256_split2", 2: "128x256_split4"}
                for tile in tiles:
                    if tile in (1, 4) and N % 192 != 0:
                        continue
                    for variant in (0, 1, 2, 3):
                        y.zero_()
                        us, _ = ws.bench.gemm_variant(variant, tile, ptrs, x.data_ptr(), y.data_ptr(), N, M, K, partial_ptr=partial.data_ptr(), iters=n_it, warmup=n_it // 4)
                        if variant == 0:
                            y_block = y.clone()         # same k order for every variant of one tile: they must agree bit for bit
                        row["variants"][f"{tiles[tile]}/{names[variant]}"] = {
                            "us": round(us, 2), "equal_to_block_variant": bool(torch.equal(y, y_block)),
                            "max_abs_diff_to_product": float((y.float() - y_ref.float()).abs().max())}
                    for code, label in ((16, "memory_spread"), (17, "memory_spread_wide"), (18, "memory_spread_weights_first")):
                        if tile not in (0, 1, 2, 3, 4):
                            continue
                        y.zero_()
                        us, _ = ws.bench.gemm_variant(code, tile, ptrs, x.data_ptr(), y.data_ptr(), N, M, K, partial_ptr=partial.data_ptr(), iters=n_it, warmup=n_it // 4)
                        row["variants"][f"{tiles[tile]}/{label}"] = {"us": round(us, 2), "equal_to_block_variant": bool(torch.equal(y, y_block)),
                                                                     "max_abs_diff_to_product": float((y.float() - y_ref.float()).abs().max())}
                    for variant in (4, 5):
                        _, ph = ws.bench.gemm_variant(variant, tile, ptrs, x.data_ptr(), y.data_ptr(), N, M, K, partial_ptr=partial.data_ptr(), iters=8, warmup=2)
                        row["variants"][f"{tiles[tile]}/{names[variant - 4]}"]["ticks_cvt_barrier_rest"] = ph
                # the product kernel with other tile shapes, k splits and weight prefetch distances (PD k-tiles ahead)
                shapes = {0: "64x192", 1: "64x256", 2: "128x192", 3: "64x256_split4", 4: "128x256_split4", 5: "64x256_split2", 6: "64x256_split3", 7: "128x192_split2",
                          8: "128x256_one_wg_per_cu", 9: "128x256_split4_one_wg_per_cu", 20: "128x128_split4", 21: "128x128"}
                row["product_kernel_by_tile_and_prefetch"] = {}
                for code in (101, 102, 103, 111, 112, 113, 121, 122, 131, 132, 133, 141, 151, 153, 161, 163, 171, 172, 181, 182, 183, 191, 192, 193, 201, 202, 211):
                    if code < 200 and (code // 10) % 10 in (0, 2, 7) and N % 192 != 0:
                        continue
                    us, _ = ws.bench.gemm_variant(0, code, ptrs, x.data_ptr(), y.data_ptr(), N, M, K, partial_ptr=partial.data_ptr(), iters=n_it, warmup=n_it // 4)
                    row["product_kernel_by_tile_and_prefetch"][f"{shapes[(code // 10) % 10 if code < 200 else code // 10]}/pd{code % 10}"] = {
                        "us": round(us, 2), "max_abs_diff_to_product": float((y.float() - y_ref.float()).abs().max())}
                us0, _ = ws.bench.gemm_variant(0, 0, ptrs, x.data_ptr(), y.data_ptr(), N, M, K, inv_scale=SCALED_INV_SCALE, iters=n_it, warmup=n_it // 4)
                us1, _ = ws.bench.gemm_variant(1, 0, ptrs, x.data_ptr(), y.data_ptr(), N, M, K, inv_scale=SCALED_INV_SCALE, iters=n_it, warmup=n_it // 4)
                row["scaled_128x256"] = {"block_us": round(us0, 2), "spread_us": round(us1, 2)}
                us, _ = ws.bench.gemm_variant(8, 0, rm_ptrs, x.data_ptr(), y_ref.data_ptr(), N, M, K, iters=n_it, warmup=n_it // 4)
                row["product_us_after_the_variants"] = round(us, 2)
                rows.append(row)
                del x, y, y_ref, partial
            for c_ in codes:
                ws.lib.weight_release(c_.data_ptr())
            del codes, tiled
        names = {0: "mfma_only", 1: "+conversions", 3: "+fragment_reads_from_lds", 7: "+barrier", 15: "+lds_stores (all four mid-tile)",
                 31: "+weight_loads (all four behind the barrier)", 63: "+activation_loads (all four mid-tile) = the whole k-tile, memory instructions in bursts",
                 1307: "the whole k-tile in the product's order (one memory instruction per token block)",
                 1507: "the same with 5 fragments read ahead instead of 3", 6: "mfma+fragment_reads+barrier", 17: "mfma+conversions+weight_loads"}
        ceiling = {"TFLOPs": {names[f]: round(ws.bench.gemm_ablation_tflops(f), 1) for f in names},
                   "what": "the 128 x 256 tile's k-tile (64 matrix-core instructions per wave, two workgroups per CU, operands in registers or in "
                           "windows that stay in L2: no HBM traffic) with its ingredients switched on one after the other, ~30-50 ms per figure"}
        print(json.dumps({"workload": "prefill_variants", "k_tile_ablation": ceiling, "what": "W8A16 prefill GEMM: the product kernel and the variants measured against it "
                          "(us per launch over 600 (M 512) / 200 (M 2048) launches on 8 distinct weights; ticks = shares of wave 0's clock per workgroup)", "rows": rows}))
        return

    metric, unit = "quant GEMV HBM GB/s (Qwen3-8B W8A16 decode linears, bs=1)", "GB/s"
    if args.workload == "decode_step":
        # full decode step: tokens / s at context DECODE_CTX; then the GEMV half of the metric on the
        # same shapes through Matrix::mulBatched (decode linears chain and the per-shape sweep)
        if args.steps + args.warmup > DECODE_CTX:
            sys.exit("bench.py: --steps + --warmup must not exceed the context length")
        model = build_decode_step(ws, DECODE_CTX)
        start = DECODE_CTX - args.steps - args.warmup
        torch.cuda.synchronize()
        model.reset(1, start)
        if args.warmup:
            model.run(args.warmup, use_graph)
        ms = model.run(args.steps, use_graph)
        assert model.pos == DECODE_CTX
        model.reset(1, start + args.warmup)
        ms_other = model.run(args.steps, not use_graph)
        # the same steps on the attention path that keeps every rounding point of the reference (BF16 probabilities)
        model.set_exact_attention(True)
        model.reset(1, start)
        if args.warmup:
            model.run(args.warmup, use_graph)
        ms_exact = model.run(args.steps, use_graph)
        model.set_exact_attention(False)
        ms_step = ms / args.steps
        value = 1000.0 / ms_step
        extra["ms_per_step_exact_attention"] = round(ms_exact / args.steps, 4)
        extra["launch_us"] = {"empty_in_graph": round(ws.bench.launch_us(0), 3), "one_trip_in_graph": round(ws.bench.launch_us(1), 3)}
        metric, unit = "decode tok/s Qwen3-8B W8A16 bs=1", "tok/s"
        step_bytes = decode_step_bytes(DECODE_CTX - (args.steps - 1) / 2.0)
        extra["launch_mode"] = "hipGraph" if use_graph else "stream"
        extra["ms_per_step_" + ("stream" if use_graph else "hipGraph")] = round(ms_other / args.steps, 4)
        extra["bytes_per_token"] = step_bytes
        extra["decode_step_GBps"] = round(step_bytes / ms_step * 1e-6, 1)
        extra["decode_step_frac_of_hbm_bound"] = round(step_bytes / ms_step * 1e-6 / HBM_PEAK_GBS, 4)
        extra["launches_per_step"] = 6 * QWEN3_8B["layers"] + 2
        extra["last_token"] = model.token
        workload = ("full random-init Qwen3-8B W8A16 decode step, batch 1, greedy: 36 layers, hidden 4096, 32 q / 8 kv heads x 128, qk RMSNorm, "
                    f"RoPE theta 1e6, SwiGLU 12288, vocab 151936, bf16 KV cache holding {DECODE_CTX} positions; FP8_E5M2 weights with scale 1; "
                    "attention with FP32 softmax probabilities (ms_per_step_exact_attention: BF16 probabilities, the reference's rounding point)")
        # dominant kernel: the fused RMSNorm + gate/up SwiGLU launch (two 4096 x 12288 weights), timed over the 36 layers' distinct weights
        K, N, M = 4096, 2 * 12288, 1
        dom_us = ws.bench.gate_up_us(model, 10)
        dom_bytes = K * N + 2 * K + 2 * K + 2 * 12288
        if not args.no_scaled_step:
            # the same step on linears quantized on the device by Matrix::quantizeWeights (per-tensor scales absmax / 57344)
            model_q = build_decode_step(ws, DECODE_CTX, quantize_on_device=True)
            torch.cuda.synchronize()
            model_q.reset(1, start)
            if args.warmup:
                model_q.run(args.warmup, use_graph)
            ms_q = model_q.run(args.steps, use_graph) / args.steps
            extra["scaled_decode_step"] = {"workload": "the same decode step with every linear quantized on the device by Matrix::quantizeWeights "
                                                       "(FP8_E5M2, truncating encoder, per-tensor scale absmax / 57344): the reference's weight_data_type = fp8_e5m2 route",
                                           "ms_per_step": round(ms_q, 4), "tok_s": round(1000.0 / ms_q, 1), "vs_scale_1": round(ms_q / ms_step, 4),
                                           "example_scale": model_q.tensor_scale(0, "wq"), "last_token": model_q.token}
            ws.keep.append(model_q)
        if not args.no_fp4_step:
            extra["fp4_decode_step"], fp4_model = llama_fp4_decode(ws, args.steps, args.warmup, use_graph, repack=not args.no_prompt)
        if not args.no_sweep:
            # Nothing is freed until the last sweep has run: on this driver, freeing a few GB of device memory slows the
            # kernels that stream through the buffers still allocated (the 253-linear chain: 1.79 -> 1.91 ms per step
            # after the decode model is released, and it stays there)
            ops, by_shape = build_decode_model(ws, 1)
            lin_bytes = sum(gemv_bytes(k, n, 1) for *_, k, n in ops)
            lin_ms = time_chain(ws, ops, args.steps, args.warmup, use_graph) / args.steps
            extra["quant_gemv"] = {"workload": "the 253 FP8_E5M2 linears of one decode token through Matrix::mulBatched", "ms_per_step": round(lin_ms, 4),
                                   "GBps": round(lin_bytes / lin_ms * 1e-6, 1), "frac_of_hbm_peak": round(lin_bytes / lin_ms * 1e-6 / HBM_PEAK_GBS, 4)}
            extra["sweep"] = shape_sweep(ws, by_shape, tuple(int(v) for v in args.sweep_tokens.split(",")), use_graph)
            extra["sweep_variants"] = variant_sweep(ws, by_shape, use_graph=use_graph)
            extra["prefill"] = prefill_cases(ws, by_shape)
            gops = build_grouped_model(ws, 1)
            g_ms = time_chain(ws, gops, args.steps, args.warmup, use_graph) / args.steps
            extra["quant_gemv_grouped"] = {"workload": "the same weights with q,k,v and gate,up stored together (loader-level grouping): 145 launches through Matrix::mulBatched",
                                           "ms_per_step": round(g_ms, 4), "GBps": round(lin_bytes / g_ms * 1e-6, 1),
                                           "frac_of_hbm_peak": round(lin_bytes / g_ms * 1e-6 / HBM_PEAK_GBS, 4)}
            extra["fp4_sweep"], extra["fp4_prefill"] = fp4_sweep(ws)
            del ops, by_shape, gops
        if not args.no_prompt:
            # after the sweeps: a third of a second of dense matrix-core work lowers what is measured right behind it
            extra["prompt_phase"] = {"workload": "prompt phase of the same Qwen3-8B W8A16 model from an empty cache (DecodeModel::prefill): per layer seven "
                                                 "quantized GEMMs with T columns on the row-major weights, RMSNorm / RoPE / append rows, causal attention, "
                                                 "residual adds, SwiGLU; then the head on the last token",
                                     "cases": prompt_phase(ws, model, token_counts=(32, 128, 512, 2048))}
            # the same with the load-time tiled copy of every linear (DecodeModel::setRepackLinears: twice the weight memory)
            for li in range(QWEN3_8B["layers"]):
                for name in ("wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down"):
                    assert model.prepare_tiled(li, name)
            extra["prompt_phase"]["cases"] += prompt_phase(ws, model, token_counts=(32, 128, 512, 2048, DECODE_CTX), layout="tiled copies")
            extra["generate"] = generate_run(ws, model, use_graph)
            extra["generate_short_prompt"] = generate_run(ws, model, use_graph, prompt_tokens=128)
            if not args.no_fp4_step:
                # the Llama-3.1-8B-shaped FP4 model, whose linears were loaded with their tiled copies (the FP4 GEMM reads those)
                extra["fp4_decode_step"]["prompt_phase"] = prompt_phase(ws, fp4_model, token_counts=(32, 128, 512, 2048), layout="tiled copies", c=LLAMA31_8B)
        del model
        if not args.no_baselines:
            torch.cuda.empty_cache()
            extra["gpu_baselines"] = gpu_baselines(ws, DECODE_CTX)
            for name, b in extra["gpu_baselines"].items():
                if name == "torch_bf16_eager_prompt":
                    ours = [c for c in extra.get("prompt_phase", {}).get("cases", []) if c["tokens"] == b["tokens"]]
                    if ours:
                        b["speedup_of_this_build"] = {c["weights"]: round(c["tok_s"] / b["tok_s"], 2) for c in ours}
                else:
                    b["speedup_of_this_build"] = round(value / b["tok_s"], 2)
            torch.cuda.empty_cache()
    elif args.workload == "decode_linears":
        ops, by_shape = build_decode_model(ws, 1)
        step_bytes = sum(gemv_bytes(K, N, 1) for *_, K, N in ops)
        torch.cuda.synchronize()
        ms = time_chain(ws, ops, args.steps, args.warmup, use_graph)
        torch.cuda.synchronize()
        ms_other = time_chain(ws, ops, args.steps, 1, not use_graph)
        ms_step = ms / args.steps
        value = step_bytes / ms_step * 1e-6
        extra["launch_mode"] = "hipGraph" if use_graph else "stream"
        extra["ms_per_step_" + ("stream" if use_graph else "hipGraph")] = round(ms_other / args.steps, 4)
        extra["decode_linears_tok_s"] = round(1000.0 / ms_step, 1)
        extra["launches_per_step"] = len(ops)
        workload = "qwen3-8b W8A16 decode linears, batch 1: 36x(q,k,v,o,gate,up,down)+lm_head, 7568097280 B of distinct FP8_E5M2 weights per step"
        # dominant kernel: gate/up-shaped GEMV over the 72 distinct gate/up weights
        K, N, M = 4096, 12288, 1
        dom_ops = [o for o in ops if (o[3], o[4]) == (K, N)]
        dom_ms = time_chain(ws, dom_ops, 10, 2, False)
        dom_us = dom_ms * 1000.0 / (10 * len(dom_ops))
        if not args.no_sweep:
            extra["sweep"] = shape_sweep(ws, by_shape, tuple(int(v) for v in args.sweep_tokens.split(",")), False)
            extra["fp4_sweep"], extra["fp4_prefill"] = fp4_sweep(ws)
    else:
        K, N = (int(v) for v in args.shape.split(","))
        M = args.tokens if args.workload == "gemv" else max(args.tokens, 512)
        X, Y = ws.activation(M, K), ws.output(M, N)
        if args.weights == "fp4":
            t, block = torch, args.block
            per = K * N // 2 + K * N // block
            n_w = max(2, min(48, (768 << 20) // per))
            nib = [t.randint(0, 256, (N, K // 2), dtype=t.uint8, device=ws.dev, generator=ws.gen) for _ in range(n_w)]
            sc = [t.randint(0x10, 0x40, (N, K // block), dtype=t.uint8, device=ws.dev, generator=ws.gen) for _ in range(n_w)]
            tiled = []
            if ws.repack:
                for w, s_ in zip(nib, sc):
                    tiled.append(t.empty(ws.lib.tiled_size(FP4, N, K), dtype=t.uint8, device=ws.dev))
                    assert ws.lib.weight_prepare_fp4(w.data_ptr(), s_.data_ptr(), block, N, K, tiled[-1].data_ptr()) == 0
            torch.cuda.synchronize()
            ms = ws.bench.fp4_chain([w.data_ptr() for w in nib], [s_.data_ptr() for s_ in sc], X.data_ptr, Y.data_ptr, N, M, K, block, args.steps * n_w, args.warmup * n_w)
            if ms < 0:
                raise RuntimeError(f"fp4 chain failed: {ms}")
            ms_step = ms / args.steps
            step_bytes = n_w * fp4_bytes(K, N, M, block)
            ops = []
        else:
            n_w = max(2, min(64, (1 << 30) // (K * N)))
            weights = [ws.weight_e5m2(N, K) for _ in range(n_w)]
            ops = [(W, X, Y, K, N) for W in weights]
            torch.cuda.synchronize()
            ms = time_chain(ws, ops, args.steps, args.warmup, False)
            torch.cuda.synchronize()
            ms_step = ms / args.steps
            step_bytes = sum(gemv_bytes(K, N, M) for _ in ops)
        value = step_bytes / ms_step * 1e-6
        dom_us = ms_step * 1000.0 / n_w
        extra["launch_mode"] = "stream"
        workload = f"{args.workload} K={K} N={N} M={M} over {n_w} distinct " + (f"FP4_E2M1 block-{args.block} weights" if args.weights == "fp4" else "FP8_E5M2 weights")

    if args.workload != "decode_step" and ops:
        assert ws.lib.linear(ops[0][0].data_ptr, E5M2, ops[0][1].data_ptr, ops[0][2].data_ptr, ops[0][4], M if args.workload != "decode_linears" else 1, ops[0][3]) == 0
    if args.workload == "decode_step":
        achieved = dom_bytes / dom_us * 1e-3
        roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                    "traffic": GEMV_FUSED_GATE_UP_TRAFFIC_BYTES, "traffic_source": TRAFFIC_SOURCE + "decode_step_qwen3_8b_ctx4096.md",
                    "kernel": "gemv8_fused_kernel (RMSNorm + gate/up SwiGLU pair)",
                    "shape": {"K": K, "N": N, "M": M}, "us_per_launch": round(dom_us, 3), "bytes_per_launch": dom_bytes}
    elif args.workload == "prefill":
        flops = 2.0 * M * K * N
        achieved = flops / dom_us * 1e-6
        roofline = {"bound": "mfma", "achieved": round(achieved, 2), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                    "frac": round(achieved / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None,
                    "kernel": ("gemm4_mfma_direct_kernel" if args.weights == "fp4" and ws.lib.last_kernel() == "gemm_mfma_tiled" else
                               "gemm_mfma_direct_kernel" if args.weights == "fp8" and (ws.lib.last_kernel() == "gemm_mfma_tiled" or (K % 64 == 0 and M >= 48)) else "gemm_mfma_kernel"),
                    "weight_layout": "tiled copy" if ws.lib.last_kernel() == "gemm_mfma_tiled" else "row-major", "shape": {"K": K, "N": N, "M": M}, "us_per_launch": round(dom_us, 3)}
    else:
        achieved = (fp4_bytes(K, N, M, args.block) if args.weights == "fp4" else gemv_bytes(K, N, M)) / dom_us * 1e-3
        roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": round(achieved / HBM_PEAK_GBS, 4),
                    "traffic": GEMV_GATE_UP_TRAFFIC_BYTES if (K, N, M, args.weights) == (4096, 12288, 1, "fp8") else None,
                    "traffic_source": TRAFFIC_SOURCE + "gemv8_mfma_tiled_K4096_N12288_M1.md" if (K, N, M, args.weights) == (4096, 12288, 1, "fp8") else None,
                    "kernel": ws.lib.last_kernel(), "shape": {"K": K, "N": N, "M": M}, "us_per_launch": round(dom_us, 3),
                    "bytes_per_launch": fp4_bytes(K, N, M, args.block) if args.weights == "fp4" else gemv_bytes(K, N, M)}

    line = {
        "metric": metric if args.workload != "prefill" else ("W4A16" if args.weights == "fp4" else "W8A16") + " prefill GEMM algorithmic GB/s",
        "value": round(value, 1), "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic", "config": {"workload": workload},
        "roofline": roofline,
    }
    if unit == "GB/s":
        line["frac_of_hbm_peak"] = round(value / HBM_PEAK_GBS, 4)
    if not args.no_cpu:
        threads = min(16, len(os.sched_getaffinity(0)))
        line["cpu_baseline"] = cpu_baseline(pkg, threads, unit if args.workload != "prefill" else "GB/s")
    line.update(extra)
    if args.workload == "decode_step":
        line["north_star"] = north_star_summary(line)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
