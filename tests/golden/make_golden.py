"""Writes the golden fixtures of tests/golden/ from library routines that share no code with the
oracle: torch's float8 / bfloat16 casts and float64 matmul.  The reference tree holds no test
vectors for this path, so these are this repository's own known answers.

    python tests/golden/make_golden.py

Special cases written by hand because no library states them: every FP8 NaN code decodes to the
canonical +qNaN 0x7FC00000 (sign dropped) and stays 0x7FC0 in BF16 for every scale (a NaN operand
passes through the FP32 multiply unchanged on x86 and on gfx950, and the integer rounding keeps
0x7FC0), and FP4 code 8 is +0.0.
"""
from pathlib import Path

import numpy as np
import torch

HERE = Path(__file__).resolve().parent
SCALES = np.array([1.0, 0.5, 2.0 ** -7, 3.0, 0.1, 1.0 / 448.0, 0.02 / 57344.0, 1.7e-3, 1.0e30, -0.75], dtype=np.float32)
FP4_VALUES = np.array([0, 0.5, 1, 1.5, 2, 3, 4, 6, 0, -0.5, -1, -1.5, -2, -3, -4, -6], dtype=np.float32)


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def decode_fp8(torch_dtype) -> np.ndarray:
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    f = codes.view(torch_dtype).to(torch.float32).numpy().copy()
    bits = f.view(np.uint32)
    bits[np.isnan(f)] = 0x7FC00000
    return bits.view(np.float32)


def main() -> None:
    e5 = decode_fp8(torch.float8_e5m2)
    e4 = decode_fp8(torch.float8_e4m3fn)
    with np.errstate(all="ignore"):
        e5_bf16 = np.stack([bf16_bits(torch.from_numpy(e5) * torch.tensor(s)) for s in SCALES])
        e4_bf16 = np.stack([bf16_bits(torch.from_numpy(e4) * torch.tensor(s)) for s in SCALES])
        fp4_bf16 = np.stack([bf16_bits(torch.from_numpy(FP4_VALUES) * torch.tensor(s)) for s in SCALES])
        # every (scale byte, nibble) product of the block-scale format
        prod = torch.from_numpy(e4)[:, None] * torch.from_numpy(FP4_VALUES)[None, :]
        blockscale_bf16 = bf16_bits(prod)
    e5_bf16[:, np.isnan(e5)] = 0x7FC0
    e4_bf16[:, np.isnan(e4)] = 0x7FC0
    blockscale_bf16[np.isnan(e4), :] = 0x7FC0
    np.savez(HERE / "dequant_tables.npz", scales=SCALES, e5m2_f32_bits=e5.view(np.uint32), e4m3_f32_bits=e4.view(np.uint32),
             e5m2_bf16=e5_bf16, e4m3_bf16=e4_bf16, fp4_bf16=fp4_bf16, blockscale_bf16=blockscale_bf16)

    # tiny linears with float64 answers (inputs are exactly representable, so float64 is exact)
    rng = np.random.default_rng(20240607)
    cases = {}
    for name, n_out, K, tokens in (("fp8_a", 24, 64, 1), ("fp8_b", 17, 48, 3), ("fp4_a", 8, 64, 2)):
        x = torch.from_numpy(rng.standard_normal((tokens, K), dtype=np.float32)).to(torch.bfloat16)
        if name.startswith("fp8"):
            w = torch.from_numpy((rng.standard_normal((n_out, K), dtype=np.float32) * 0.02).astype(np.float32)).to(torch.float8_e5m2)
            wf = w.to(torch.float64)
            cases[name + "_w"] = w.view(torch.uint8).numpy()
        else:
            nib = rng.integers(0, 256, size=(n_out, K // 2), dtype=np.uint8)
            sc = rng.integers(0x08, 0x60, size=(n_out, K // 16), dtype=np.uint8)
            codes = np.empty((n_out, K), dtype=np.uint8)
            codes[:, 0::2] = nib & 15
            codes[:, 1::2] = nib >> 4
            sf = torch.from_numpy(sc).view(torch.float8_e4m3fn).to(torch.float64)
            wf = torch.from_numpy(FP4_VALUES[codes]).to(torch.float64) * sf.repeat_interleave(16, dim=1)
            cases[name + "_w"] = nib
            cases[name + "_s"] = sc
        y = x.to(torch.float64) @ wf.T
        cases[name + "_x"] = x.view(torch.int16).numpy().view(np.uint16)
        cases[name + "_y_f64"] = y.numpy()
        cases[name + "_y_bf16"] = bf16_bits(y.to(torch.float32))
    np.savez(HERE / "linear_cases.npz", **cases)
    print("wrote", [p.name for p in HERE.glob("*.npz")])


if __name__ == "__main__":
    main()
