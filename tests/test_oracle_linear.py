"""Pins the oracle's GEMM / block-scale / packer logic on the CPU: the scalar C dispatcher against
the vectorised NumPy contraction and the float64 golden answers, one-hot and all-ones activations,
and the converter-faithful FP4 packer against hand-computed blocks."""
import numpy as np
from oracle import synth
import pytest
import torch


def f64(oracle, bits):
    return oracle.bf16_to_f32(bits).astype(np.float64)


def test_golden_linear_cases(oracle, golden_linear):
    g = golden_linear
    for name, n_out, K, tokens, wt in (("fp8_a", 24, 64, 1, 5), ("fp8_b", 17, 48, 3, 5), ("fp4_a", 8, 64, 2, 6)):
        sc = g[name + "_s"] if wt == 6 else None
        Wd = oracle.dequant_weight(g[name + "_w"], wt, n_out, K, blk_sc=sc)
        exact = oracle.linear_exact(Wd, g[name + "_x"])
        assert np.array_equal(exact, g[name + "_y_f64"])                       # every product and sum is exact in float64
        assert np.array_equal(oracle.linear_oracle(Wd, g[name + "_x"]), g[name + "_y_bf16"])
        C = np.zeros((tokens, n_out), dtype=np.uint16)                          # column-major [n_out x tokens]
        W = np.ascontiguousarray(g[name + "_w"])
        rc = oracle.quant_gemm(1, 0, n_out, tokens, K, 1.0, W, wt, K, 1.0, g[name + "_x"], oracle.BF16, K, 1.0, 0.0, C, n_out,
                               blk_scA=np.ascontiguousarray(sc) if sc is not None else None)
        assert rc == 0 and np.array_equal(C, g[name + "_y_bf16"])
        C32 = np.zeros_like(C)                                                  # float accumulation: within one ulp
        oracle.quant_gemm(1, 0, n_out, tokens, K, 1.0, W, wt, K, 1.0, g[name + "_x"], oracle.BF16, K, 1.0, 0.0, C32, n_out,
                          blk_scA=np.ascontiguousarray(sc) if sc is not None else None, acc64=False)
        assert np.abs(f64(oracle, C32) - exact).max() <= 2.0 ** -8 * np.abs(exact).max()


def test_one_hot_and_all_ones_activations(oracle):
    rng = np.random.default_rng(1)
    n_out, K = 32, 64
    W = rng.integers(0, 0x7C, size=(n_out, K), dtype=np.uint8) | (rng.integers(0, 2, size=(n_out, K), dtype=np.uint8) << 7)
    Wd = oracle.dequant_weight(W, oracle.E5M2, n_out, K, 0.37)
    for k in (0, 13, 63):
        X = np.zeros((1, K), dtype=np.uint16); X[0, k] = 0x3F80
        C = np.zeros((1, n_out), dtype=np.uint16)
        assert oracle.quant_gemm(1, 0, n_out, 1, K, 1.0, W, oracle.E5M2, K, 0.37, X, oracle.BF16, K, 1.0, 0.0, C, n_out) == 0
        a, b = C[0].copy(), Wd[:, k].copy()
        a[a == 0x8000] = 0; b[b == 0x8000] = 0
        assert np.array_equal(a, b)
    X = np.full((1, K), 0x3F80, dtype=np.uint16)
    C = np.zeros((1, n_out), dtype=np.uint16)
    oracle.quant_gemm(1, 0, n_out, 1, K, 1.0, W, oracle.E5M2, K, 0.37, X, oracle.BF16, K, 1.0, 0.0, C, n_out)
    sums = f64(oracle, Wd).sum(axis=1)
    assert np.array_equal(C[0], oracle.f32_to_bf16(sums.astype(np.float32)))


def test_dispatcher_layouts_and_alpha_beta_vs_numpy(oracle):
    rng = np.random.default_rng(2)
    n_out, tokens, K = 12, 3, 32
    Wq = oracle.encode_e5m2_rne((rng.standard_normal((n_out, K)) * 0.02).astype(np.float32))
    Xb = oracle.f32_to_bf16(rng.standard_normal((tokens, K)).astype(np.float32))
    Wd = f64(oracle, oracle.dequant_weight(Wq, oracle.E5M2, n_out, K, 0.5))
    Y = f64(oracle, Xb) @ Wd.T                                                   # [tokens, n_out]
    for weight_is_a in (True, False):
        for ta in (0, 1):
            for tb in (0, 1):
                if weight_is_a:
                    M, N = n_out, tokens
                    A = Wq if ta else np.ascontiguousarray(Wq.T)
                    B = np.ascontiguousarray(Xb.T) if tb else Xb
                    tA, tB, sA, sB = oracle.E5M2, oracle.BF16, 0.5, 1.0
                    want = Y                                                     # C memory [N][M] = [tokens][n_out]
                else:
                    M, N = tokens, n_out
                    A = Xb if ta else np.ascontiguousarray(Xb.T)
                    B = np.ascontiguousarray(Wq.T) if tb else Wq
                    tA, tB, sA, sB = oracle.BF16, oracle.E5M2, 1.0, 0.5
                    want = Y.T
                lda, ldb = (K if ta else M), (N if tb else K)
                C0 = oracle.f32_to_bf16(rng.standard_normal((N, M)).astype(np.float32))
                C = C0.copy()
                assert oracle.quant_gemm(ta, tb, M, N, K, 2.0, A, tA, lda, sA, B, tB, ldb, sB, -0.5, C, M) == 0
                expect = oracle.f32_to_bf16((2.0 * want - 0.5 * f64(oracle, C0)).astype(np.float32))
                assert np.array_equal(C, expect), (weight_is_a, ta, tb)
    # unsupported combinations
    assert oracle.quant_gemm(1, 0, 4, 1, 4, 1.0, Wq, oracle.E5M2, 4, 1.0, Wq, oracle.E5M2, 4, 1.0, 0.0, np.zeros(4, np.uint16), 4) == -1
    assert oracle.quant_gemm(1, 0, 4, 1, 4, 1.0, Xb, oracle.BF16, 4, 1.0, Xb, oracle.BF16, 4, 1.0, 0.0, np.zeros(4, np.uint16), 4) == -1


def test_converter_packer_by_hand(oracle, pkg):
    # one block, absmax 6 -> scale 1.0 (0x38), values on the grid map to themselves
    grid = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, -0.0, -.5, -1, -1.5, -2, -3, -4, -6], dtype=np.float32)
    for packer in (oracle.quantize_fp4_blockscale_converter, synth.pack_fp4_blockscale):
        nib, sc = packer(grid, 16)
        assert sc.tolist() == [0x38]
        assert oracle.unpack_fp4(nib, 16).tolist() == [0, 1, 2, 3, 4, 5, 6, 7, 0, 9, 10, 11, 12, 13, 14, 15]   # sign of -0.0 is 0
        # exact boundaries go to the lower code (searchsorted side='left'), unlike the on-the-fly kernel
        edge = np.array([6, .25, .75, 1.25, 1.75, 2.5, 3.5, 5.0, -.25, -5.0, 0, 0, 0, 0, 0, 0], dtype=np.float32)
        nib, sc = packer(edge, 16)
        assert oracle.unpack_fp4(nib, 16).tolist()[:10] == [7, 0, 1, 2, 3, 4, 5, 6, 8, 14]
        # all-zero block: scale 1.0; a second block with absmax 0.012 -> 0.002 -> E4M3 subnormal 1 * 2^-9 (RNE)
        two = np.zeros(32, dtype=np.float32); two[16] = 0.012; two[17] = -0.006
        nib, sc = packer(two, 16)
        assert sc.tolist() == [0x38, 0x01]
        assert oracle.unpack_fp4(nib, 32).tolist()[16:18] == [7, 13]            # 6/absmax scaling: 6 and -3
        # ragged tail: zero padded, outputs trimmed
        nib, sc = packer(np.array([1, 2, 3], dtype=np.float32), 16)
        assert nib.size == 2 and sc.size == 1
    kn, ks = oracle.quantize_fp4_blockscale_kernel(edge, 16)
    assert oracle.unpack_fp4(kn, 16).tolist()[:10] == [7, 1, 2, 3, 4, 5, 6, 7, 9, 15]


def test_on_the_fly_fp4_quantiser_scale_byte_by_hand(oracle):
    """The scale byte of the on-the-fly quantiser (cccc-cuda/cuda_functions.cu:2896-2923) is absmax / 6
    through the TRUNCATING E4M3 encoder (:2383-2412), worked out by hand below; the cases marked (*) are
    the ones where round-to-nearest would give the next byte up."""
    step = 2.0 ** -9                                              # E4M3 subnormal spacing
    cases = [
        # absmax, absmax / 6,           byte
        (0.0, "scale 1.0 for an all-zero block", 0x38),
        (6.0, "1.0 = 2^0: e = 7, m = 0", 0x38),
        (1.5, "0.25 = 2^-2: e = 5, m = 0", 0x28),
        (10.5, "1.75 = 1.110b: e = 7, m = 6", 0x3E),
        (11.0, "1.8333 = 1.110101..b: m = 6 (*) nearest is m = 7", 0x3E),
        (0.021, "0.0035 = 1.79 subnormal steps: 1 (*) nearest is 2", 0x01),
        (0.06, "0.01 = 5.12 subnormal steps: 5", 0x05),
        (0.0115, "0.00192 = 0.98 subnormal steps: 0 (*) nearest is 1", 0x00),
        (6 * 7 * step, "7 subnormal steps exactly", 0x07),
        (6 * 2.0 ** -6, "smallest normal 2^-6: e = 1, m = 0", 0x08),
        (6 * 448.0, "largest finite 448: e = 15, m = 6", 0x7E),
        (6 * 1000.0, "beyond the range: saturates at 448", 0x7E),
    ]
    for amax, why, byte in cases:
        block = np.zeros(16, dtype=np.float32)
        block[5], block[9] = -amax, amax / 2
        nib, sc = oracle.quantize_fp4_blockscale_kernel(block, 16)
        assert sc.tolist() == [byte], (amax, why, hex(int(sc[0])))
        if amax > 0:
            # codes come from 6 / absmax: the extreme element is -6 (code 15), half of it 3 (code 5)
            codes = oracle.unpack_fp4(nib, 16).tolist()
            assert codes[5] == 15 and codes[9] == 5 and sum(codes) == 20, (amax, codes)
    # the same bytes through round-to-nearest differ exactly at the marked cases
    rne = oracle.encode_e4m3_rne(np.array([11.0 / 6, 0.021 / 6, 0.0115 / 6], dtype=np.float32))
    assert rne.tolist() == [0x3F, 0x02, 0x01]
    # blocks of 32, two blocks, ragged tail (3 elements in the last block)
    x = np.zeros(35, dtype=np.float32)
    x[31], x[34] = 3.0, -0.75
    nib, sc = oracle.quantize_fp4_blockscale_kernel(x, 32)
    assert sc.tolist() == [0x30, 0x20] and nib.size == 18              # 0.5 = 2^-1: e = 6; 0.125 = 2^-3: e = 4
    assert oracle.unpack_fp4(nib, 35).tolist()[31] == 7 and oracle.unpack_fp4(nib, 35).tolist()[34] == 15


def test_packers_agree_and_round_trip_is_bounded(oracle, pkg):
    w = synth.weights_f32(3, 64, 256)
    a = oracle.quantize_fp4_blockscale_converter(w, 16)
    b = synth.pack_fp4_blockscale(w, 16)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
    deq = oracle.bf16_to_f32(oracle.dequant_fp4_blockscale_to_bf16(a[0], a[1], w.size, 16)).reshape(w.shape)
    # scales land in E4M3's subnormal range (step 2^-9), so the error is bounded by the block scale error
    s = oracle.decode_table(oracle.E4M3)[a[1]].reshape(64, 16)
    assert np.all(np.abs(deq.reshape(64, 16, 16)) <= 6.0 * s[:, :, None])
    assert np.abs(deq - w).max() < 0.02


def test_synthetic_e5m2_weights_are_rne(oracle, pkg):
    w = synth.weights_f32(4, 32, 128)
    q = synth.weights_e5m2(4, 32, 128)
    assert np.array_equal(q, oracle.encode_e5m2_rne(w))
    assert np.array_equal(q, torch.from_numpy(w).to(torch.float8_e5m2).view(torch.uint8).numpy())
    back = oracle.decode_table(oracle.E5M2)[q]
    assert np.all(np.abs(back - w) <= np.abs(w) * 0.125 + 2.0 ** -17)


def test_cpu_baseline_route_matches_the_oracle(oracle, pkg):
    n_out, tokens, K = 96, 2, 256
    W = synth.weights_e5m2(5, n_out, K)
    X = synth.activations(5, tokens, K)
    want = oracle.linear_exact(oracle.dequant_weight(W, oracle.E5M2, n_out, K), X)
    fn, name = oracle.find_cblas_sgemm()
    for sgemm in (None, fn):
        Y, td, tg = oracle.cpu_linear(W, oracle.E5M2, 1.0, None, 16, X, n_out, tokens, K, sgemm=sgemm, threads=2)
        assert np.abs(f64(oracle, Y) - want).max() <= 2.0 ** -7 * np.abs(want).max(), name
    nib, sc = synth.weights_fp4(6, n_out, K)
    want = oracle.linear_exact(oracle.dequant_weight(nib, oracle.FP4, n_out, K, blk_sc=sc), X)
    Y, _, _ = oracle.cpu_linear(nib, oracle.FP4, 1.0, sc, 16, X, n_out, tokens, K, sgemm=fn, threads=2)
    assert np.abs(f64(oracle, Y) - want).max() <= 2.0 ** -7 * np.abs(want).max()
