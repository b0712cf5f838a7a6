"""FP8 weights against IEEE-half activations (the reference's HALF route, cccc/cublas_real.h:921-938):
weight dequantised to half, FP32 accumulation, half out.  Checked against the exact float64
contraction of the half-rounded weights."""
import numpy as np
import pytest

from gpu_util import MAX_REL, ROW_L2_REL, from_dev, to_dev

pytestmark = pytest.mark.gpu
HALF, BF16, E4M3, E5M2, FP4 = 2, 3, 4, 5, 6


def make_case(oracle, rng, w_type, n_out, K, tokens, scale):
    w = (rng.standard_normal((n_out, K)) * 0.02 / scale).astype(np.float32)
    codes = oracle.encode_e5m2_rne(w) if w_type == E5M2 else oracle.encode_e4m3_rne(w)
    x = rng.standard_normal((tokens, K)).astype(np.float16)
    Wh = oracle.dequant_fp8_to_half(codes, w_type, scale)
    return codes, x, oracle.contract_exact(Wh, x)


def check_half(got_bits, exact, alpha=1.0, extra=None, label=""):
    want = alpha * exact + (0.0 if extra is None else extra)
    got = got_bits.view(np.float16).astype(np.float64).reshape(want.shape)
    want_h = want.astype(np.float16).astype(np.float64)                       # the reference's output is a half tensor
    for r in range(want.shape[0]):
        scale = max(np.abs(want_h[r]).max(), 1e-30)
        assert np.abs(got[r] - want_h[r]).max() / scale <= MAX_REL, label
        assert np.linalg.norm(got[r] - want_h[r]) / max(np.linalg.norm(want_h[r]), 1e-30) <= ROW_L2_REL, label
    # tighter: within one half ulp of the exact value plus FP32 accumulation noise
    ulp = np.maximum(np.abs(want), 2.0 ** -14) * 2.0 ** -10
    assert (np.abs(got - want) <= 1.0 * ulp + 3e-6 * np.sqrt(exact.shape[1]) * np.abs(want).max()).all(), label


@pytest.mark.parametrize("w_type", [E5M2, E4M3])
@pytest.mark.parametrize("tokens,kernel", [(1, "gemv_dot2_half"), (3, "gemv_dot2_half"), (4, "gemv_dot2_half"), (7, "gemv_mfma_half"), (16, "gemv_mfma_half"),
                                           (17, "gemm_mfma_half"), (40, "gemm_mfma_half"), (200, "gemm_mfma_half")])
@pytest.mark.parametrize("scale", [1.0, 0.37])
def test_half_activations(gpu, oracle, w_type, tokens, kernel, scale):
    torch, dev, lib = gpu
    rng = np.random.default_rng(tokens * 10 + w_type)
    n_out, K = 320, 2064                                                      # ragged against the 1 KiB k step and the 128-row tile
    codes, x, exact = make_case(oracle, rng, w_type, n_out, K, tokens, scale)
    wd, xd = to_dev(torch, dev, codes), to_dev(torch, dev, x.view(np.uint16))
    y = torch.zeros(tokens * n_out + 16, dtype=torch.int16, device=dev)
    assert lib.linear(wd.data_ptr(), w_type, xd.data_ptr(), y.data_ptr(), n_out, tokens, K, inv_scale=scale, act_type=HALF) == 0
    assert lib.last_kernel() == kernel
    out = from_dev(y, np.uint16)
    assert not out[tokens * n_out:].any()
    check_half(out[:tokens * n_out].reshape(tokens, n_out), exact, label=f"{w_type} {tokens} {scale}")


@pytest.mark.parametrize("w_type", [E5M2, E4M3])
@pytest.mark.parametrize("tokens", [64, 200])
def test_half_gemm_with_weights_kept_out_of_lds(gpu, oracle, w_type, tokens):
    """K % 64 == 0 and 48 tokens or more: the GEMM that converts weights in registers, row-major and tiled."""
    torch, dev, lib = gpu
    rng = np.random.default_rng(tokens + w_type)
    n_out, K, scale = 328, 1024, 0.37
    codes, x, exact = make_case(oracle, rng, w_type, n_out, K, tokens, scale)
    wd, xd = to_dev(torch, dev, codes), to_dev(torch, dev, x.view(np.uint16))
    td = torch.zeros(lib.tiled_size(w_type, n_out, K), dtype=torch.uint8, device=dev)
    outs = []
    for tiled in (False, True):
        if tiled:
            assert lib.weight_prepare(wd.data_ptr(), w_type, n_out, K, K, td.data_ptr()) == 0
        try:
            y = torch.zeros(tokens * n_out + 16, dtype=torch.int16, device=dev)
            assert lib.linear(wd.data_ptr(), w_type, xd.data_ptr(), y.data_ptr(), n_out, tokens, K, inv_scale=scale, act_type=HALF) == 0
            assert lib.last_kernel() == "gemm_mfma_half"
        finally:
            if tiled:
                assert lib.weight_release(wd.data_ptr()) == 0
        out = from_dev(y, np.uint16)
        assert not out[tokens * n_out:].any()
        outs.append(out[:tokens * n_out].reshape(tokens, n_out))
        check_half(outs[-1], exact, label=f"{w_type} {tokens} tiled={tiled}")
    assert np.array_equal(outs[0], outs[1])


@pytest.mark.parametrize("w_type", [E5M2, E4M3])
@pytest.mark.parametrize("n_out,K", [(328, 1024), (4200, 2112), (1040, 8448)])
def test_half_matrix_core_gemv_on_the_tiled_copy(gpu, oracle, w_type, n_out, K):
    """1..16 tokens of HALF activations on a weight with a registered tiled copy: the matrix-core GEMV reads the copy (from
    three tokens on for a weight this small), with and without a per-tensor scale, alpha / beta included; every
    configuration of its launch table that these shapes reach (few / many row tiles, short / long rows)."""
    torch, dev, lib = gpu
    rng = np.random.default_rng(n_out + w_type)
    for tokens, scale, alpha, beta in ((3, 1.0, 1.0, 0.0), (4, 0.37, 1.0, 0.0), (8, 0.37, 0.5, -2.0), (16, 1.0, 1.0, 0.0), (13, 0.37, 1.0, 0.0)):
        codes, x, exact = make_case(oracle, rng, w_type, n_out, K, tokens, scale)
        c0 = rng.standard_normal((tokens, n_out)).astype(np.float16)
        wd, xd = to_dev(torch, dev, codes), to_dev(torch, dev, x.view(np.uint16))
        td = torch.zeros(lib.tiled_size(w_type, n_out, K), dtype=torch.uint8, device=dev)
        assert lib.weight_prepare(wd.data_ptr(), w_type, n_out, K, K, td.data_ptr()) == 0
        try:
            y = to_dev(torch, dev, np.concatenate([c0.view(np.uint16).ravel(), np.zeros(16, dtype=np.uint16)]))
            assert lib.linear(wd.data_ptr(), w_type, xd.data_ptr(), y.data_ptr(), n_out, tokens, K, inv_scale=scale, alpha=alpha, beta=beta, act_type=HALF) == 0
            assert lib.last_kernel() == "gemv_mfma_tiled_half"
        finally:
            assert lib.weight_release(wd.data_ptr()) == 0
        out = from_dev(y, np.uint16)
        assert not out[tokens * n_out:].any()
        check_half(out[:tokens * n_out].reshape(tokens, n_out), exact, alpha=alpha, extra=beta * c0.astype(np.float64) if beta else None,
                   label=f"{w_type} {n_out}x{K} {tokens} tokens")


def test_half_alpha_beta_tall_and_generic(gpu, oracle):
    torch, dev, lib = gpu
    rng = np.random.default_rng(5)
    # alpha / beta, tall weight (8-wave configuration)
    n_out, K, tokens = 33000, 256, 2
    codes, x, exact = make_case(oracle, rng, E5M2, n_out, K, tokens, 1.0)
    c0 = rng.standard_normal((tokens, n_out)).astype(np.float16)
    wd, xd, y = to_dev(torch, dev, codes), to_dev(torch, dev, x.view(np.uint16)), to_dev(torch, dev, c0.view(np.uint16).reshape(-1))
    assert lib.linear(wd.data_ptr(), E5M2, xd.data_ptr(), y.data_ptr(), n_out, tokens, K, alpha=0.5, beta=-2.0, act_type=HALF) == 0
    check_half(from_dev(y, np.uint16).reshape(tokens, n_out), exact, alpha=0.5, extra=-2.0 * c0.astype(np.float64), label="alpha beta")
    # a row length the fast kernels refuse (K % 16 != 0) goes through the generic kernel
    n_out, K, tokens = 24, 40, 3
    codes, x, exact = make_case(oracle, rng, E4M3, n_out, K, tokens, 0.5)
    wd, xd = to_dev(torch, dev, codes), to_dev(torch, dev, x.view(np.uint16))
    y = torch.zeros(tokens * n_out, dtype=torch.int16, device=dev)
    assert lib.linear(wd.data_ptr(), E4M3, xd.data_ptr(), y.data_ptr(), n_out, tokens, K, inv_scale=0.5, act_type=HALF) == 0
    assert lib.last_kernel() == "generic"
    check_half(from_dev(y, np.uint16).reshape(tokens, n_out), exact, label="generic")
    # refused combinations: FP4 with HALF, mixed 16-bit types
    p = wd.data_ptr()
    assert lib.quant_gemm(1, 0, 16, 1, 32, 1.0, p, FP4, 32, 1.0, p, HALF, 32, 1.0, 0.0, p, HALF, 16) == -1
    assert lib.quant_gemm(1, 0, 16, 1, 32, 1.0, p, E5M2, 32, 1.0, p, HALF, 32, 1.0, 0.0, p, BF16, 16) == -1
    assert lib.quant_gemm(1, 0, 16, 1, 32, 1.0, p, E5M2, 32, 1.0, p, BF16, 32, 1.0, 0.0, p, HALF, 16) == -1


def test_half_dequant_inside_the_kernel_is_exact(gpu, oracle):
    """One-hot half activations pick out single dequantised weights: all 256 codes, with and without a scale."""
    torch, dev, lib = gpu
    for w_type in (E5M2, E4M3):
        for scale in (1.0, 0.37):
            codes = np.arange(256, dtype=np.uint8).reshape(16, 16)
            x = np.eye(16, dtype=np.float16)
            wd, xd = to_dev(torch, dev, codes), to_dev(torch, dev, x.view(np.uint16))
            y = torch.zeros(16 * 16, dtype=torch.int16, device=dev)
            assert lib.linear(wd.data_ptr(), w_type, xd.data_ptr(), y.data_ptr(), 16, 16, 16, inv_scale=scale, act_type=HALF) == 0
            got = from_dev(y, np.uint16).reshape(16, 16).T                     # [token k][row o] -> W[o][k]
            want = oracle.dequant_fp8_to_half(codes, w_type, scale).view(np.uint16)
            # a row holding an Inf or NaN code turns every output of that row into NaN (Inf * 0): leave those rows out
            ok_rows = np.isfinite(oracle.decode_table(w_type)[codes]).all(axis=1) & np.isfinite(want.view(np.float16)).all(axis=1)
            assert ok_rows.sum() >= 12
            # (numeric comparison: the sum -0 * 1 + 0 * 0 + ... is +0, so code 0x80 comes back without its sign)
            assert (got[ok_rows].view(np.float16) == want[ok_rows].view(np.float16)).all(), (w_type, scale)
