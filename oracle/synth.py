"""Synthetic weights and activations of the benchmark configurations (seeded, reproducible).  DATA MAKER for tests,
the smoke test and the benchmark's CPU leg; not part of the shipped package.

Weights: float32 N(0, 0.02) -> BF16 (RNE) -> FP8_E5M2 (RNE) with no extra scale, or the offline
converter's FP4 block-scale packing (reference scripts/convert_weights.py:346-370, restated here
with the same library calls).  Activations: float32 N(0, 1) -> BF16 (RNE).  The reference's own
encoders truncate (cccc/types.h:168-199); round-to-nearest is what the benchmark configuration
asks for, so the encoders here are this package's own.
"""
from __future__ import annotations

import numpy as np
import torch

FP4_BOUNDS = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0], dtype=np.float32)


def seed_for(config_index: int, shape_index: int) -> int:
    return 1234 + 1000 * config_index + shape_index


def bf16_bits(x: torch.Tensor) -> np.ndarray:
    return x.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def activations(seed: int, tokens: int, K: int) -> np.ndarray:
    """bf16 bits [tokens, K] of N(0, 1)."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((tokens, K), dtype=np.float32)
    return bf16_bits(torch.from_numpy(x))


def weights_f32(seed: int, n_out: int, K: int) -> np.ndarray:
    """N(0, 0.02) rounded to BF16, as float32 [n_out, K]."""
    rng = np.random.default_rng(seed + 500)
    w = rng.standard_normal((n_out, K), dtype=np.float32) * np.float32(0.02)
    return torch.from_numpy(w).to(torch.bfloat16).to(torch.float32).numpy()


def weights_e5m2(seed: int, n_out: int, K: int) -> np.ndarray:
    """uint8 E5M2 codes [n_out, K], round-to-nearest-even."""
    w = torch.from_numpy(weights_f32(seed, n_out, K))
    return w.to(torch.float8_e5m2).view(torch.uint8).numpy()


def weights_e4m3(seed: int, n_out: int, K: int, amax_to_448: bool = True):
    """(uint8 E4M3 codes [n_out, K], inv_scale): per-tensor absmax scaling onto the E4M3 range."""
    w = torch.from_numpy(weights_f32(seed, n_out, K))
    inv_scale = float(w.abs().max()) / 448.0 if amax_to_448 else 1.0
    q = (w / inv_scale).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    return q, inv_scale


def pack_fp4_blockscale(data: np.ndarray, group: int = 16):
    """(nibble bytes, E4M3 scale bytes) of a flat float32 array, as the offline converter packs."""
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
    code = np.searchsorted(FP4_BOUNDS, np.abs(scaled)).astype(np.uint8) | ((scaled < 0).astype(np.uint8) * 8)
    packed = (code[0::2] | (code[1::2] << 4)).astype(np.uint8)[: (n + 1) // 2]
    scales = scales[: (n + group - 1) // group]
    scale_bytes = torch.from_numpy(scales).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    return packed, scale_bytes


def weights_fp4(seed: int, n_out: int, K: int, group: int = 16):
    """(nibbles [n_out, K/2], scales [n_out, K/group]) for N(0, 0.02) weights."""
    nib, sc = pack_fp4_blockscale(weights_f32(seed, n_out, K), group)
    return nib.reshape(n_out, K // 2), sc.reshape(n_out, K // group)
