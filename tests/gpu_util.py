"""Helpers shared by the GPU parity tests: device buffers from NumPy arrays and the tolerance of
the benchmark definition (max relative error 1e-2, per-row L2 relative error 2e-3), both measured
against the exact float64 contraction of the bit-exact dequantized weights."""
import numpy as np

MAX_REL = 1e-2
ROW_L2_REL = 2e-3


def to_dev(torch, dev, a: np.ndarray):
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).to(dev)
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32)).to(dev)
    return torch.from_numpy(a).to(dev)


def from_dev(t, dtype):
    return t.cpu().numpy().view(dtype)


def round_to_bf16(x_f64: np.ndarray) -> np.ndarray:
    """float64 -> nearest-even BF16 value (as float64): the reference's own output of an exact sum."""
    u = np.ascontiguousarray(x_f64, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return u.astype(np.uint32).view(np.float32).astype(np.float64)


def check_rows(got_f64: np.ndarray, exact_f64: np.ndarray, label=""):
    """Rows = tokens.  The tolerance is stated against the reference's own output, which is a BF16
    tensor, so the exact contraction is rounded to BF16 first (otherwise the comparison would
    mostly measure the output rounding itself, about 1.1e-3 RMS).  Returns (max rel, worst row L2
    rel) and asserts the tolerance."""
    assert got_f64.shape == exact_f64.shape
    want_f64 = round_to_bf16(exact_f64)
    worst_max, worst_l2 = 0.0, 0.0
    for r in range(want_f64.shape[0]):
        ref = want_f64[r]
        diff = np.abs(got_f64[r] - ref)
        scale = max(np.abs(ref).max(), 1e-30)
        worst_max = max(worst_max, diff.max() / scale)
        worst_l2 = max(worst_l2, np.linalg.norm(diff) / max(np.linalg.norm(ref), 1e-30))
    assert worst_max <= MAX_REL, f"{label}: max rel err {worst_max:.3e} > {MAX_REL}"
    assert worst_l2 <= ROW_L2_REL, f"{label}: row L2 rel err {worst_l2:.3e} > {ROW_L2_REL}"
    return worst_max, worst_l2


def check_bf16_close(got_bits: np.ndarray, want_f64: np.ndarray, label="", slack_ulp=1.0, abs_floor=0.0):
    """Tighter than the benchmark tolerance: every output is within slack_ulp BF16 ulps of the exact
    value plus the FP32 accumulation noise floor `abs_floor`."""
    got = (got_bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    ulp = np.maximum(np.abs(want_f64), 2.0 ** -126) * 2.0 ** -8
    bad = np.abs(got - want_f64) > slack_ulp * ulp + abs_floor
    assert not bad.any(), f"{label}: {bad.sum()} outputs off by more than {slack_ulp} ulp; worst {np.abs(got - want_f64)[bad].max()}"
