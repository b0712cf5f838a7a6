"""Parity of hip_quant_gemm (decode GEMV family, prefill GEMM, generic fallback) against the
oracle, through the C-ABI.  Expected values are the exact float64 contraction of the bit-exact
dequantized BF16 weights (oracle.linear_exact); tolerances are the benchmark's (gpu_util)."""
import numpy as np
from oracle import synth
import pytest

from gpu_util import check_bf16_close, check_rows, from_dev, to_dev

pytestmark = pytest.mark.gpu


def bf16_f64(oracle, bits):
    return oracle.bf16_to_f32(bits).astype(np.float64)


def run_linear(gpu, pkg, W, w_type, X, n_out, tokens, K, inv_scale=1.0, blk_sc=None, block=16, alpha=1.0, beta=0.0, Y0=None):
    torch, dev, lib = gpu
    wd, xd = to_dev(torch, dev, W), to_dev(torch, dev, X)
    sd = to_dev(torch, dev, blk_sc) if blk_sc is not None else None
    y0 = Y0 if Y0 is not None else np.zeros((tokens, n_out), dtype=np.uint16)
    yd = to_dev(torch, dev, np.concatenate([y0.ravel(), np.zeros(64, dtype=np.uint16)]))
    rc = lib.linear(wd.data_ptr(), w_type, xd.data_ptr(), yd.data_ptr(), n_out, tokens, K, inv_scale,
                    sd.data_ptr() if sd is not None else None, block, alpha, beta)
    assert rc == 0
    out = from_dev(yd, np.uint16)
    assert not out[tokens * n_out:].any(), "wrote past the end"
    return out[: tokens * n_out].reshape(tokens, n_out), lib.last_kernel()


# ------------------------------------------------------------------------------------------ golden

def test_golden_linear_cases(gpu, pkg, oracle, golden_linear):
    g = golden_linear
    for name, n_out, K, tokens in (("fp8_a", 24, 64, 1), ("fp8_b", 17, 48, 3)):
        y, _ = run_linear(gpu, pkg, g[name + "_w"], oracle.E5M2, g[name + "_x"], n_out, tokens, K)
        check_rows(bf16_f64(oracle, y), g[name + "_y_f64"], name)
        check_bf16_close(y, g[name + "_y_f64"], name, slack_ulp=1.0, abs_floor=1e-6)
    y, _ = run_linear(gpu, pkg, g["fp4_a_w"], oracle.FP4, g["fp4_a_x"], 8, 2, 64, blk_sc=g["fp4_a_s"])
    check_rows(bf16_f64(oracle, y), g["fp4_a_y_f64"], "fp4_a")


# ------------------------------------------------------------------------------------------ FP8 GEMV

@pytest.mark.parametrize("tokens", [1, 2, 3, 4, 5, 8, 16])
@pytest.mark.parametrize("n_out,K", [(4096, 4096), (1024, 4096), (768, 12288), (1000, 2064), (7, 16)])
def test_fp8_gemv_vs_oracle(gpu, pkg, oracle, tokens, n_out, K):
    seed = synth.seed_for(2, n_out % 97 + tokens)
    W = synth.weights_e5m2(seed, n_out, K)
    X = synth.activations(seed, tokens, K)
    y, kernel = run_linear(gpu, pkg, W, oracle.E5M2, X, n_out, tokens, K)
    want = oracle.linear_exact(oracle.dequant_weight(W, oracle.E5M2, n_out, K), X)
    check_rows(bf16_f64(oracle, y), want, f"{kernel} {n_out}x{K} M={tokens}")
    check_bf16_close(y, want, kernel, slack_ulp=1.0, abs_floor=2e-5)
    assert kernel in ("gemv_dot2", "gemv_mfma")


@pytest.mark.parametrize("tokens", [1, 4, 16])
def test_every_code_dequantizes_exactly_inside_the_gemv(gpu, pkg, oracle, tokens):
    """One-hot activations pick single dequantized weights out of the GEMV: with x = e_k the output
    row is bf16(decode(W[:, k])) bit for bit, for all 256 codes (NaN codes: NaN)."""
    for w_type, K in ((oracle.E5M2, 256), (oracle.E4M3, 256)):
        n_out = 256
        W = np.empty((n_out, K), dtype=np.uint8)
        for o in range(n_out):
            W[o] = np.roll(np.arange(256, dtype=np.uint8), o)        # W[o][k] = (k - o) mod 256
        ks = [0, 5, 255][:max(1, min(tokens, 3))]
        X = np.zeros((tokens, K), dtype=np.uint16)
        for t in range(tokens):
            X[t, ks[t % len(ks)]] = 0x3F80                            # 1.0
        # Inf / NaN codes would poison their whole row through 0 * Inf; give them a separate pass
        tab = oracle.decode_table(w_type)
        special = ~np.isfinite(tab)
        Wf = W.copy()
        Wf[special[W]] = 0
        y, kernel = run_linear(gpu, pkg, Wf, w_type, X, n_out, tokens, K)
        for t in range(tokens):
            k = ks[t % len(ks)]
            want = oracle.dequant_fp8_to_bf16(Wf[:, k], w_type, 1.0)
            got = y[t].copy()
            got[got == 0x8000] = 0                                    # -0.0 + 0.0 accumulates to +0.0
            want = want.copy(); want[want == 0x8000] = 0
            assert np.array_equal(got, want), (kernel, w_type, t)
    # Inf and NaN codes propagate
    W = np.full((16, 64), 0x3C, dtype=np.uint8)
    W[3, 7] = 0x7C; W[5, 9] = 0x7E; W[6, 0] = 0xFC
    X = np.full((tokens, 64), 0x3F80, dtype=np.uint16)
    y, _ = run_linear(gpu, pkg, W, oracle.E5M2, X, 16, tokens, 64)
    f = bf16_f64(oracle, y)
    assert np.all(f[:, 3] == np.inf) and np.all(np.isnan(f[:, 5])) and np.all(f[:, 6] == -np.inf) and np.all(f[:, 0] == 64.0)


@pytest.mark.parametrize("tokens", [1, 3, 16, 40])
@pytest.mark.parametrize("w_type_name", ["e5m2", "e4m3"])
def test_per_tensor_scale_rounds_the_weight_to_bf16(gpu, pkg, oracle, tokens, w_type_name):
    """With invScale != 1 the weight entering the product is bf16(decode * invScale)."""
    n_out, K = 512, 1024
    seed = synth.seed_for(2, 40 + tokens)
    X = synth.activations(seed, tokens, K)
    if w_type_name == "e5m2":
        wf = synth.weights_f32(seed, n_out, K)
        inv = float(np.abs(wf).max()) / 57344.0
        W, w_type = oracle.encode_e5m2_rne(wf / np.float32(inv)), oracle.E5M2
    else:
        W, inv = synth.weights_e4m3(seed, n_out, K)
        w_type = oracle.E4M3
    y, kernel = run_linear(gpu, pkg, W, w_type, X, n_out, tokens, K, inv_scale=inv)
    want = oracle.linear_exact(oracle.dequant_weight(W, w_type, n_out, K, inv), X)
    check_rows(bf16_f64(oracle, y), want, kernel)
    check_bf16_close(y, want, kernel, slack_ulp=1.0, abs_floor=2e-5)
    # and it is measurably different from scaling after the sum (so the rounding point is tested)
    unrounded = oracle.linear_exact(oracle.dequant_weight(W, w_type, n_out, K, 1.0), X) * inv
    assert np.abs(unrounded - want).max() > 0


def test_alpha_beta_epilogue(gpu, pkg, oracle):
    n_out, K = 640, 2048
    for tokens in (1, 4, 12, 48):
        seed = synth.seed_for(2, 60 + tokens)
        W = synth.weights_e5m2(seed, n_out, K)
        X = synth.activations(seed, tokens, K)
        Y0 = synth.activations(seed + 1, tokens, n_out)
        y, kernel = run_linear(gpu, pkg, W, oracle.E5M2, X, n_out, tokens, K, alpha=0.5, beta=-2.0, Y0=Y0)
        want = 0.5 * oracle.linear_exact(oracle.dequant_weight(W, oracle.E5M2, n_out, K), X) - 2.0 * bf16_f64(oracle, Y0)
        check_rows(bf16_f64(oracle, y), want, kernel)


# ------------------------------------------------------------------------------------------ FP4

@pytest.mark.parametrize("block", [16, 32])
@pytest.mark.parametrize("tokens", [1, 2, 4, 7, 16])
@pytest.mark.parametrize("n_out,K", [(4096, 4096), (1024, 4096), (512, 14336), (33, 64)])
def test_fp4_gemv_vs_oracle(gpu, pkg, oracle, tokens, n_out, K, block):
    seed = synth.seed_for(3, n_out % 89 + tokens + block)
    nib, sc = synth.weights_fp4(seed, n_out, K, block)
    X = synth.activations(seed, tokens, K)
    y, kernel = run_linear(gpu, pkg, nib, oracle.FP4, X, n_out, tokens, K, blk_sc=sc, block=block)
    want = oracle.linear_exact(oracle.dequant_weight(nib, oracle.FP4, n_out, K, blk_sc=sc, block=block), X)
    check_rows(bf16_f64(oracle, y), want, f"{kernel} fp4 {n_out}x{K} M={tokens} b={block}")
    assert kernel == "gemv_dot2"


@pytest.mark.parametrize("tokens", [1, 3, 4, 7, 16])
@pytest.mark.parametrize("n_out,K", [(8, 48), (257, 144), (130, 2064), (64, 4112)])
def test_fp4_rows_of_half_a_load_more(gpu, pkg, oracle, tokens, n_out, K):
    """K % 32 == 16 with blocks of 16 -- legal in the reference, whose blocks run over the flat element index
    (cccc-cuda/cuda_functions.cu:2926-2939): every other row starts in the middle of a 16-byte load and at an odd scale
    byte, and a row's last load is half this row, half the next.  Up to 16 tokens stay on the dot2 kernel; the neighbours'
    codes and scales must not leak in (the buffers end with the last row: nothing past them may be read either), and
    blocks of 32 on such rows, which straddle rows, take the generic kernel."""
    seed = synth.seed_for(3, 700 + tokens + n_out % 11)
    X = synth.activations(seed, tokens, K)
    nib, sc = synth.pack_fp4_blockscale(synth.weights_f32(seed, n_out, K), 16)
    y, kernel = run_linear(gpu, pkg, nib, oracle.FP4, X, n_out, tokens, K, blk_sc=sc, block=16)
    assert kernel == "gemv_dot2"
    Wd = oracle.dequant_weight(nib, oracle.FP4, n_out, K, blk_sc=sc, block=16)
    want = oracle.linear_exact(Wd, X)
    check_rows(bf16_f64(oracle, y), want, f"ragged fp4 {tokens}x{n_out}x{K}")
    check_bf16_close(y, want, kernel, slack_ulp=1.0, abs_floor=2e-5)
    if tokens == 1 and (n_out * K) % 32 == 0:
        nib32, sc32 = synth.pack_fp4_blockscale(synth.weights_f32(seed, n_out, K), 32)
        y, kernel = run_linear(gpu, pkg, nib32, oracle.FP4, X, n_out, tokens, K, blk_sc=sc32, block=32)
        assert kernel == "generic"
        check_rows(bf16_f64(oracle, y), oracle.linear_exact(oracle.dequant_weight(nib32, oracle.FP4, n_out, K, blk_sc=sc32, block=32), X), "ragged block 32")


def test_fp4_every_nibble_and_scale_inside_the_gemv(gpu, pkg, oracle):
    """x = one-hot: the output is bf16(fp4 * e4m3 scale) exactly, for all 16 nibbles x all finite
    scale bytes."""
    K, n_out = 64, 256
    nib_row = (np.arange(16, dtype=np.uint8)[0::2] | (np.arange(16, dtype=np.uint8)[1::2] << 4)).astype(np.uint8)
    nib = np.tile(nib_row, (n_out, K // 16))                            # element k of every row = nibble k % 16
    sc = np.repeat(np.arange(256, dtype=np.uint8)[:, None], K // 16, axis=1)
    sc[sc == 0x7F] = 0x38; sc[sc == 0xFF] = 0xB8
    Wd = oracle.dequant_weight(nib, oracle.FP4, n_out, K, blk_sc=sc, block=16)
    for k in (0, 9, 15, 16 + 3, 63):
        X = np.zeros((1, K), dtype=np.uint16); X[0, k] = 0x3F80
        y, _ = run_linear(gpu, pkg, nib, oracle.FP4, X, n_out, 1, K, blk_sc=sc, block=16)
        got, want = y[0].copy(), Wd[:, k].copy()
        got[got == 0x8000] = 0; want[want == 0x8000] = 0
        assert np.array_equal(got, want), k


# ------------------------------------------------------------------------------------------ prefill GEMM

@pytest.mark.parametrize("tokens,n_out,K", [(128, 256, 512), (512, 768, 1024), (130, 200, 144), (17, 128, 64), (2048, 256, 256)])
@pytest.mark.parametrize("fmt", ["e5m2", "fp4_16", "fp4_32"])
def test_prefill_gemm_vs_oracle(gpu, pkg, oracle, tokens, n_out, K, fmt):
    seed = synth.seed_for(4, tokens % 83 + n_out % 7)
    X = synth.activations(seed, tokens, K)
    expect = "gemm_mfma"
    if fmt == "e5m2":
        W = synth.weights_e5m2(seed, n_out, K)
        y, kernel = run_linear(gpu, pkg, W, oracle.E5M2, X, n_out, tokens, K)
        Wd = oracle.dequant_weight(W, oracle.E5M2, n_out, K)
    else:
        block = int(fmt[-2:])
        if K % 32:
            # rows that are not whole 32-element loads (with blocks of 32 they even straddle rows: the scales run over
            # the flat element index) are served by the generic kernel
            expect = "generic"
            nib, sc = synth.pack_fp4_blockscale(synth.weights_f32(seed, n_out, K), block)
        else:
            nib, sc = synth.weights_fp4(seed, n_out, K, block)
        y, kernel = run_linear(gpu, pkg, nib, oracle.FP4, X, n_out, tokens, K, blk_sc=sc, block=block)
        Wd = oracle.dequant_weight(nib, oracle.FP4, n_out, K, blk_sc=sc, block=block)
    want = oracle.linear_exact(Wd, X)
    check_rows(bf16_f64(oracle, y), want, f"{kernel} {fmt} {tokens}x{n_out}x{K}")
    check_bf16_close(y, want, kernel, slack_ulp=1.0, abs_floor=2e-5)
    assert kernel == expect


@pytest.mark.parametrize("tokens", [48, 64, 65, 128, 200, 513])
@pytest.mark.parametrize("n_out,K", [(256, 64), (1000, 192), (250, 1024), (1536, 2048), (512, 8192)])
@pytest.mark.parametrize("w_type_name", ["e5m2", "e4m3"])
def test_prefill_gemm_with_weights_kept_out_of_lds(gpu, pkg, oracle, tokens, n_out, K, w_type_name):
    """FP8 GEMM kernel for K % 64 == 0 and 48 tokens or more (64- and 128-token tiles, ragged token and
    row counts, one k-tile and many), on the row-major weight and on its tiled copy, with and without a
    per-tensor scale and with alpha / beta, against the exact contraction.  The two long-K shapes have so
    few output tiles that the k range is split over workgroups (2 and 8 ranges) and a second kernel adds
    the partial sums; n_out = 250 is not a multiple of 4 and never splits."""
    torch, dev, lib = gpu
    seed = synth.seed_for(4, 300 + tokens % 89 + n_out % 13)
    if w_type_name == "e5m2":
        w_type, W = oracle.E5M2, synth.weights_e5m2(seed, n_out, K)
    else:
        w_type, W = oracle.E4M3, synth.weights_e4m3(seed, n_out, K)[0]
    X = synth.activations(seed, tokens, K)
    want = oracle.linear_exact(oracle.dequant_weight(W, w_type, n_out, K), X)
    want_s = oracle.linear_exact(oracle.dequant_weight(W, w_type, n_out, K, 0.37), X)
    c0 = synth.activations(seed + 1, tokens, n_out)
    wd, xd = to_dev(torch, dev, W), to_dev(torch, dev, X)
    td = torch.zeros(lib.tiled_size(w_type, n_out, K), dtype=torch.uint8, device=dev)

    def run(label, expect_kernel):
        y = torch.zeros(tokens * n_out + 64, dtype=torch.int16, device=dev)
        assert lib.linear(wd.data_ptr(), w_type, xd.data_ptr(), y.data_ptr(), n_out, tokens, K) == 0
        assert lib.last_kernel() == expect_kernel
        out = from_dev(y, np.uint16)
        assert not out[tokens * n_out:].any(), "wrote past the end"
        got = out[: tokens * n_out].reshape(tokens, n_out)
        check_rows(bf16_f64(oracle, got), want, f"{label} {w_type_name} {tokens}x{n_out}x{K}")
        # one BF16 ulp plus the FP32 accumulation noise, which grows with the size of the terms (E4M3 codes reach 448)
        check_bf16_close(got, want, label, slack_ulp=1.0, abs_floor=max(2e-5, 1e-6 * np.sqrt(K) * np.abs(want).max()))
        ys = torch.zeros(tokens * n_out, dtype=torch.int16, device=dev)
        assert lib.linear(wd.data_ptr(), w_type, xd.data_ptr(), ys.data_ptr(), n_out, tokens, K, inv_scale=0.37) == 0
        check_rows(bf16_f64(oracle, from_dev(ys, np.uint16).reshape(tokens, n_out)), want_s, label + " scaled")
        yb = to_dev(torch, dev, c0.reshape(-1))
        assert lib.linear(wd.data_ptr(), w_type, xd.data_ptr(), yb.data_ptr(), n_out, tokens, K, alpha=0.5, beta=-2.0) == 0
        want_b = 0.5 * want - 2.0 * bf16_f64(oracle, c0)
        check_rows(bf16_f64(oracle, from_dev(yb, np.uint16).reshape(tokens, n_out)), want_b, label + " alpha beta")
        return got

    plain = run("row-major", "gemm_mfma")
    assert lib.weight_prepare(wd.data_ptr(), w_type, n_out, K, K, td.data_ptr()) == 0
    try:
        tiled = run("tiled", "gemm_mfma_tiled")
    finally:
        assert lib.weight_release(wd.data_ptr()) == 0
    # same products, same order of summation: the two layouts agree to the bit
    assert np.array_equal(plain, tiled)


# ------------------------------------------------------------------------------------------ dispatcher

def test_weight_as_B_and_transposed_layouts_match_the_scalar_oracle(gpu, pkg, oracle):
    """All eight (which operand is quantized) x (transA) x (transB) layouts of the unified call
    against the scalar C restatement of the dispatcher."""
    torch, dev, lib = gpu
    rng = np.random.default_rng(77)
    n_out, tokens, K = 48, 5, 64
    Wq = oracle.encode_e5m2_rne((rng.standard_normal((n_out, K)) * 0.02).astype(np.float32))
    Xb = oracle.f32_to_bf16(rng.standard_normal((tokens, K)).astype(np.float32))
    for weight_is_a in (True, False):
        for ta in (0, 1):
            for tb in (0, 1):
                if weight_is_a:
                    M, N = n_out, tokens
                    A = Wq if ta else np.ascontiguousarray(Wq.T)           # trans: stored [M][K] (lda=K); no-trans: [K][M] (lda=M)
                    B = np.ascontiguousarray(Xb.T) if tb else Xb           # no-trans: stored [N][K] (ldb=K); trans: [K][N] (ldb=N)
                    lda, ldb = (K if ta else M), (N if tb else K)
                    tA, tB, sA = oracle.E5M2, oracle.BF16, 0.25
                else:
                    M, N = tokens, n_out
                    A = Xb if ta else np.ascontiguousarray(Xb.T)
                    B = np.ascontiguousarray(Wq.T) if tb else Wq
                    lda, ldb = (K if ta else M), (N if tb else K)
                    tA, tB, sA = oracle.BF16, oracle.E5M2, 1.0
                sB = 0.25 if not weight_is_a else 1.0
                C0 = oracle.f32_to_bf16(rng.standard_normal((N, M)).astype(np.float32))
                want = C0.copy()
                assert oracle.quant_gemm(ta, tb, M, N, K, 1.5, A, tA, lda, sA, B, tB, ldb, sB, 0.5, want, M) == 0
                Ad, Bd, Cd = to_dev(torch, dev, A), to_dev(torch, dev, B), to_dev(torch, dev, C0)
                rc = lib.quant_gemm(ta, tb, M, N, K, 1.5, Ad.data_ptr(), tA, lda, sA, Bd.data_ptr(), tB, ldb, sB, 0.5,
                                    Cd.data_ptr(), oracle.BF16, M)
                assert rc == 0
                got = from_dev(Cd, np.uint16).reshape(N, M)
                diff = np.abs(bf16_f64(oracle, got) - bf16_f64(oracle, want))
                assert diff.max() <= 2.0 ** -7 * np.abs(bf16_f64(oracle, want)).max(), (weight_is_a, ta, tb, lib.last_kernel())


@pytest.mark.parametrize("case", range(36))
def test_random_shapes_with_padded_strides(gpu, pkg, oracle, case):
    """Seeded random FP8 problems in the two LLM layouts (weight as A with TRANS / NO_TRANS, weight as B
    mirrored) with row strides larger than the rows -- lda, ldb and ldc padded, the padding filled with NaN
    codes or NaN values -- against the scalar C restatement of the dispatcher; token counts straddle every
    kernel family (GEMV, matrix-core GEMV, both GEMMs, k-split).  The padding of C must come back untouched."""
    torch, dev, lib = gpu
    rng = np.random.default_rng(1000 + case)
    tokens = int(rng.choice([1, 2, 3, 5, 9, 16, 17, 40, 48, 63, 64, 65, 100, 129, 200, 260]))
    n_out = int(rng.choice([16, 40, 64, 250, 256, 300, 512, 1000]))
    K = int(rng.choice([64, 128, 192, 448, 1024, 2048]) if case % 3 else rng.choice([16, 48, 80, 272, 1040]))
    if tokens * n_out * K > 6e7:
        K = 128
    w_type = oracle.E5M2 if case % 2 else oracle.E4M3
    pad_w, pad_x, pad_c = int(rng.choice([0, 16, 64])), int(rng.choice([0, 8, 24])), int(rng.choice([0, 4, 5, 12]))
    ldw, ldx = K + pad_w, K + pad_x
    scale = float(rng.choice([1.0, 0.37]))
    alpha, beta = float(rng.choice([1.0, 0.5])), float(rng.choice([0.0, 0.0, -1.5]))
    enc = oracle.encode_e5m2_rne if w_type == oracle.E5M2 else oracle.encode_e4m3_rne
    W = np.full((n_out, ldw), 0x7F, dtype=np.uint8)                         # NaN code in both FP8 formats
    W[:, :K] = enc((rng.standard_normal((n_out, K)) * 0.02 / scale).astype(np.float32))
    X = np.full((tokens, ldx), 0x7FC0, dtype=np.uint16)                     # BF16 NaN
    X[:, :K] = oracle.f32_to_bf16(rng.standard_normal((tokens, K)).astype(np.float32))
    weight_is_a = bool(case % 4 < 2)
    if weight_is_a:                                                          # C is [tokens][ldc >= n_out]
        M, N, ldc = n_out, tokens, n_out + pad_c
        args = lambda a, b: (1, 0, M, N, K, alpha, a, w_type, ldw, scale, b, oracle.BF16, ldx, 1.0, beta)
        A, B = W, X
        C0 = oracle.f32_to_bf16(rng.standard_normal((tokens, ldc)).astype(np.float32))
        rows, cols = tokens, n_out
    else:                                                                    # C is [n_out][ldc >= tokens]
        M, N, ldc = tokens, n_out, tokens + pad_c
        args = lambda a, b: (1, 0, M, N, K, alpha, a, oracle.BF16, ldx, 1.0, b, w_type, ldw, scale, beta)
        A, B = X, W
        C0 = oracle.f32_to_bf16(rng.standard_normal((n_out, ldc)).astype(np.float32))
        rows, cols = n_out, tokens
    want = C0.copy()
    assert oracle.quant_gemm(*args(A, B), want, ldc) == 0
    Ad, Bd, Cd = to_dev(torch, dev, A), to_dev(torch, dev, B), to_dev(torch, dev, C0)
    assert lib.quant_gemm(*args(Ad.data_ptr(), Bd.data_ptr()), Cd.data_ptr(), oracle.BF16, ldc) == 0
    kernel = lib.last_kernel()
    got = from_dev(Cd, np.uint16).reshape(rows, ldc)
    assert np.array_equal(got[:, cols:], C0[:, cols:]), f"{kernel}: padding of C was written"
    g, w = bf16_f64(oracle, got[:, :cols]), bf16_f64(oracle, want[:, :cols])
    assert np.isfinite(g).all(), f"{kernel}: padding leaked into the result"
    assert np.abs(g - w).max() <= 2.0 ** -7 * np.abs(w).max() + 1e-6, (kernel, tokens, n_out, K, ldw, ldx, ldc, weight_is_a)


def test_fp4_weight_as_B_with_block_scales(gpu, pkg, oracle):
    torch, dev, lib = gpu
    n_out, tokens, K = 64, 3, 128
    nib, sc = synth.weights_fp4(5, n_out, K, 16)
    Xb = synth.activations(5, tokens, K)
    C0 = np.zeros((n_out, tokens), dtype=np.uint16)
    want = C0.copy()
    assert oracle.quant_gemm(1, 0, tokens, n_out, K, 1.0, Xb, oracle.BF16, K, 1.0, nib, oracle.FP4, K, 1.0, 0.0, want, tokens, None, sc, 16) == 0
    Ad, Bd, Sd, Cd = to_dev(torch, dev, Xb), to_dev(torch, dev, nib), to_dev(torch, dev, sc), to_dev(torch, dev, C0)
    rc = lib.quant_gemm(1, 0, tokens, n_out, K, 1.0, Ad.data_ptr(), oracle.BF16, K, 1.0, Bd.data_ptr(), oracle.FP4, K, 1.0, 0.0,
                        Cd.data_ptr(), oracle.BF16, tokens, 0.0, None, Sd.data_ptr(), 16)
    assert rc == 0
    got = from_dev(Cd, np.uint16).reshape(n_out, tokens)
    diff = np.abs(bf16_f64(oracle, got) - bf16_f64(oracle, want))
    assert diff.max() <= 2.0 ** -7 * np.abs(bf16_f64(oracle, want)).max()


def test_odd_sizes_fall_back_to_the_generic_kernel(gpu, pkg, oracle):
    rng = np.random.default_rng(78)
    n_out, tokens, K = 37, 3, 50                                         # K % 16 != 0
    W = oracle.encode_e5m2_rne((rng.standard_normal((n_out, K)) * 0.02).astype(np.float32))
    X = oracle.f32_to_bf16(rng.standard_normal((tokens, K)).astype(np.float32))
    y, kernel = run_linear(gpu, pkg, W, oracle.E5M2, X, n_out, tokens, K, inv_scale=0.3)
    assert kernel == "generic"
    want = oracle.linear_exact(oracle.dequant_weight(W, oracle.E5M2, n_out, K, 0.3), X)
    check_rows(bf16_f64(oracle, y), want, kernel)
    # FP4 with a per-tensor scale and no block scales
    nib = rng.integers(0, 256, size=(n_out, 32), dtype=np.uint8)
    X = oracle.f32_to_bf16(rng.standard_normal((tokens, 64)).astype(np.float32))
    y, kernel = run_linear(gpu, pkg, nib, oracle.FP4, X, n_out, tokens, 64, inv_scale=0.01)
    assert kernel == "generic"
    want = oracle.linear_exact(oracle.dequant_weight(nib, oracle.FP4, n_out, 64, 0.01), X)
    check_rows(bf16_f64(oracle, y), want, kernel)


def test_rejected_argument_combinations(gpu, oracle):
    torch, dev, lib = gpu
    b = torch.zeros(4096, dtype=torch.uint8, device=dev)
    p = b.data_ptr()
    BF, E5 = oracle.BF16, oracle.E5M2
    assert lib.quant_gemm(1, 0, 16, 1, 16, 1.0, p, E5, 16, 1.0, p, E5, 16, 1.0, 0.0, p, BF, 16) == -1       # both quantized (W8A8 route)
    assert lib.quant_gemm(1, 0, 16, 1, 16, 1.0, p, BF, 16, 1.0, p, BF, 16, 1.0, 0.0, p, BF, 16) == -1       # nothing quantized
    assert lib.quant_gemm(1, 0, 16, 1, 16, 1.0, p, E5, 16, 1.0, p, oracle.HALF, 16, 1.0, 0.0, p, BF, 16) == -1       # mixed 16-bit types
    assert lib.quant_gemm(1, 0, 16, 1, 16, 1.0, p, oracle.FP4, 16, 1.0, p, oracle.HALF, 16, 1.0, 0.0, p, oracle.HALF, 16) == -1   # FP4 has no HALF route
    assert lib.quant_gemm(1, 0, 16, 1, 16, 1.0, p, E5, 16, 1.0, p, BF, 16, 1.0, 0.0, p, oracle.FLOAT, 16) == -1
    assert lib.quant_gemm(2, 0, 16, 1, 16, 1.0, p, E5, 16, 1.0, p, BF, 16, 1.0, 0.0, p, BF, 16) == -1
    assert lib.quant_gemm(1, 0, 0, 1, 16, 1.0, p, E5, 16, 1.0, p, BF, 16, 1.0, 0.0, p, BF, 16) == 0         # empty output
    assert not b.cpu().numpy().any()
    # K == 0: the sum is empty, C = beta * C
    c = to_dev(torch, dev, np.full(16, 0x4000, dtype=np.uint16))
    assert lib.quant_gemm(1, 0, 16, 1, 0, 1.0, p, E5, 16, 1.0, p, BF, 16, 1.0, 0.5, c.data_ptr(), BF, 16) == 0
    assert np.all(from_dev(c, np.uint16) == 0x3F80)


# ------------------------------------------------------------------------------------------ full-size properties

def test_full_size_gemv_properties(gpu, pkg, oracle):
    """At the benchmark's real shapes (too big for the scalar oracle in a test): (1) rows sampled at
    random agree with the exact contraction; (2) linearity in x; (3) all-ones x gives row sums."""
    torch, dev, lib = gpu
    for n_out, K in ((12288, 4096), (4096, 12288), (151936, 4096)):
        g = torch.Generator(device="cpu").manual_seed(n_out + K)
        W = (torch.randn(n_out, K, generator=g) * 0.02).to(torch.bfloat16).to(torch.float8_e5m2).view(torch.uint8).numpy()
        wd = to_dev(torch, dev, W)
        rows = np.random.default_rng(n_out).choice(n_out, size=257, replace=False)
        Wd_rows = oracle.dequant_fp8_to_bf16(W[rows], oracle.E5M2)
        for tokens in (1, 4, 16):
            X = synth.activations(n_out + tokens, tokens, K)
            xd = to_dev(torch, dev, X)
            yd = torch.zeros(tokens, n_out, dtype=torch.int16, device=dev)
            assert lib.linear(wd.data_ptr(), oracle.E5M2, xd.data_ptr(), yd.data_ptr(), n_out, tokens, K) == 0
            y = from_dev(yd, np.uint16)
            want = oracle.linear_exact(Wd_rows, X)
            check_rows(bf16_f64(oracle, y[:, rows]), want, f"{lib.last_kernel()} {n_out}x{K} M={tokens}")
        ones = np.full((1, K), 0x3F80, dtype=np.uint16)
        yd = torch.zeros(1, n_out, dtype=torch.int16, device=dev)
        assert lib.linear(wd.data_ptr(), oracle.E5M2, to_dev(torch, dev, ones).data_ptr(), yd.data_ptr(), n_out, 1, K) == 0
        sums = oracle.decode_table(oracle.E5M2).astype(np.float64)[W[rows]].sum(axis=1)
        got = bf16_f64(oracle, from_dev(yd, np.uint16))[0, rows]
        assert np.all(np.abs(got - sums) <= 2.0 ** -8 * np.abs(sums) + 1e-5)
        del wd


def test_full_size_prefill_gemm_sampled(gpu, pkg, oracle):
    """The benchmark's four prefill shapes at full size, on the row-major weight and on its tiled copy (the
    last shape has 64 output tiles, so its k range is split over workgroups): 192 sampled features of
    every token against the exact contraction, and the two layouts against each other."""
    torch, dev, lib = gpu
    for tokens, n_out, K in ((512, 12288, 4096), (2048, 12288, 4096), (2048, 4096, 12288), (512, 4096, 12288)):
        g = torch.Generator(device="cpu").manual_seed(tokens + K)
        W = (torch.randn(n_out, K, generator=g) * 0.02).to(torch.bfloat16).to(torch.float8_e5m2).view(torch.uint8).numpy()
        X = synth.activations(tokens, tokens, K)
        wd, xd = to_dev(torch, dev, W), to_dev(torch, dev, X)
        rows = np.random.default_rng(tokens).choice(n_out, size=192, replace=False)
        want = oracle.linear_exact(oracle.dequant_fp8_to_bf16(W[rows], oracle.E5M2), X)
        yd = torch.zeros(tokens, n_out, dtype=torch.int16, device=dev)
        assert lib.linear(wd.data_ptr(), oracle.E5M2, xd.data_ptr(), yd.data_ptr(), n_out, tokens, K) == 0
        assert lib.last_kernel() == "gemm_mfma"
        y = from_dev(yd, np.uint16)
        check_rows(bf16_f64(oracle, y[:, rows]), want, f"gemm {tokens}x{n_out}x{K}")
        td = torch.zeros(lib.tiled_size(oracle.E5M2, n_out, K), dtype=torch.uint8, device=dev)
        assert lib.weight_prepare(wd.data_ptr(), oracle.E5M2, n_out, K, K, td.data_ptr()) == 0
        try:
            yt = torch.zeros(tokens, n_out, dtype=torch.int16, device=dev)
            assert lib.linear(wd.data_ptr(), oracle.E5M2, xd.data_ptr(), yt.data_ptr(), n_out, tokens, K) == 0
            assert lib.last_kernel() == "gemm_mfma_tiled"
        finally:
            assert lib.weight_release(wd.data_ptr()) == 0
        assert np.array_equal(from_dev(yt, np.uint16), y), "tiled and row-major weights give different outputs"
        del wd, xd, yd, yt, td


# ------------------------------------------------------------------------------------------ load-time repack

def tiled_reference(W, n_out, K):
    """NumPy construction of the tiled layout: KiB (t, b) holds at lane l = i + 16 g the 16 codes
    W[16 t + i][64 b + 16 g ..]; rows / codes beyond the matrix are zero."""
    n_tiles, kb = (n_out + 15) // 16, (K + 63) // 64
    pad = np.zeros((n_tiles * 16, kb * 64), dtype=np.uint8)
    pad[:n_out, :K] = W
    t = pad.reshape(n_tiles, 16, kb, 4, 16)            # [t][i][b][g][16]
    return np.ascontiguousarray(t.transpose(0, 2, 3, 1, 4)).ravel()   # [t][b][g][i][16]


@pytest.mark.parametrize("n_out,K", [(64, 128), (100, 2064), (4096, 4096)])
def test_weight_prepare_builds_the_tiled_layout(gpu, pkg, oracle, n_out, K):
    torch, dev, lib = gpu
    W = np.random.default_rng(5).integers(0, 256, size=(n_out, K), dtype=np.uint8)
    wd = to_dev(torch, dev, W)
    size = lib.tiled_size(oracle.E5M2, n_out, K)
    assert size == ((n_out + 15) // 16) * ((K + 63) // 64) * 1024
    td = torch.full((size + 64,), 0xAA, dtype=torch.uint8, device=dev)
    assert lib.weight_prepare(wd.data_ptr(), oracle.E5M2, n_out, K, K, td.data_ptr()) == 0
    got = td.cpu().numpy()
    assert np.array_equal(got[:size], tiled_reference(W, n_out, K)) and np.all(got[size:] == 0xAA)
    assert lib.weight_release(wd.data_ptr()) == 0
    # refused: FP4 through the FP8 entry point, K not a multiple of 16, null pointers
    assert lib.weight_prepare(wd.data_ptr(), oracle.FP4, n_out, K, K, td.data_ptr()) == -1
    assert lib.weight_prepare(wd.data_ptr(), oracle.E5M2, n_out, 24, 24, td.data_ptr()) == -1
    assert lib.weight_prepare(None, oracle.E5M2, n_out, K, K, td.data_ptr()) == -1


@pytest.mark.parametrize("tokens", [1, 2, 3, 4, 5, 9, 16])
@pytest.mark.parametrize("n_out,K", [(300, 528), (4096, 2048), (12288, 1024), (1024, 12288), (65530, 272), (70000, 16), (151936, 1024)])
def test_prepared_weights_give_the_same_gemv(gpu, pkg, oracle, tokens, n_out, K):
    """Every launch configuration of the matrix-core kernel on the tiled copy (few / several / many row
    tiles per CU, short and long rows, ragged row counts and row lengths) against the exact contraction."""
    torch, dev, lib = gpu
    seed = synth.seed_for(2, 200 + n_out % 91 + tokens)
    W = synth.weights_e5m2(seed, n_out, K)
    X = synth.activations(seed, tokens, K)
    wd, xd = to_dev(torch, dev, W), to_dev(torch, dev, X)
    y0 = torch.zeros(tokens * n_out, dtype=torch.int16, device=dev)
    assert lib.linear(wd.data_ptr(), oracle.E5M2, xd.data_ptr(), y0.data_ptr(), n_out, tokens, K) == 0
    plain_kernel = lib.last_kernel()
    assert plain_kernel != "gemv_mfma_tiled"
    td = torch.zeros(lib.tiled_size(oracle.E5M2, n_out, K), dtype=torch.uint8, device=dev)
    assert lib.weight_prepare(wd.data_ptr(), oracle.E5M2, n_out, K, K, td.data_ptr()) == 0
    uses_tiled = tokens >= 3 or n_out * K >= (8 << 20)          # one or two tokens on a small weight stay on the dot2 kernels
    try:
        y1 = torch.zeros(tokens * n_out + 64, dtype=torch.int16, device=dev)
        assert lib.linear(wd.data_ptr(), oracle.E5M2, xd.data_ptr(), y1.data_ptr(), n_out, tokens, K) == 0
        assert lib.last_kernel() == ("gemv_mfma_tiled" if uses_tiled else plain_kernel)
        y2 = torch.zeros(tokens * n_out, dtype=torch.int16, device=dev)
        assert lib.linear(wd.data_ptr(), oracle.E5M2, xd.data_ptr(), y2.data_ptr(), n_out, tokens, K, inv_scale=0.37) == 0
    finally:
        assert lib.weight_release(wd.data_ptr()) == 0
    out = from_dev(y1, np.uint16)
    assert not out[tokens * n_out:].any()
    want = oracle.linear_exact(oracle.dequant_weight(W, oracle.E5M2, n_out, K), X)
    got = out[: tokens * n_out].reshape(tokens, n_out)
    check_rows(bf16_f64(oracle, got), want, f"tiled {n_out}x{K} M={tokens}")
    check_bf16_close(got, want, "tiled", slack_ulp=1.0, abs_floor=2e-5)
    # the plain path computed the same thing (summation order may differ by an ulp)
    plain = from_dev(y0, np.uint16).reshape(tokens, n_out)
    assert np.abs(bf16_f64(oracle, plain) - bf16_f64(oracle, got)).max() <= 2.0 ** -7 * np.abs(want).max()
    want_s = oracle.linear_exact(oracle.dequant_weight(W, oracle.E5M2, n_out, K, 0.37), X)
    check_rows(bf16_f64(oracle, from_dev(y2, np.uint16).reshape(tokens, n_out)), want_s, "tiled scaled")
    # after release the same call goes back to the plain kernels
    assert lib.linear(wd.data_ptr(), oracle.E5M2, xd.data_ptr(), y0.data_ptr(), n_out, tokens, K) == 0
    assert lib.last_kernel() == plain_kernel


# ------------------------------------------------------------------------------------------ FP4 tiled copy

def tiled_reference_fp4(nib, sc, n_out, K, block):
    """NumPy construction of the FP4 tiled copy: per row tile t (16 rows) and chunk c (128 elements) a KiB of codes
    in which lane l = n + 16 g owns 16 bytes, byte pair m holding row 16 t + n, elements 128 c + 16 m + 4 g .. + 3;
    after all code KiBs the scales, 16 * (128 / block) bytes per (t, c), row by row."""
    n_tiles, chunks, ns = (n_out + 15) // 16, (K + 127) // 128, 128 // block
    codes = np.zeros((n_tiles * 16, chunks * 64), dtype=np.uint8)
    codes[:n_out, :K // 2] = nib.reshape(n_out, K // 2)
    pieces = codes.view(np.uint16).reshape(n_tiles, 16, chunks, 8, 4)                    # [t][n][c][m][g]
    codes_t = np.ascontiguousarray(pieces.transpose(0, 2, 4, 1, 3)).view(np.uint8)        # [t][c][g][n][m]
    scales = np.zeros((n_tiles * 16, chunks * ns), dtype=np.uint8)
    scales[:n_out, :K // block] = sc.reshape(n_out, K // block)
    scales_t = np.ascontiguousarray(scales.reshape(n_tiles, 16, chunks, ns).transpose(0, 2, 1, 3))
    return np.concatenate([codes_t.ravel(), scales_t.ravel()])


@pytest.mark.parametrize("block", [16, 32])
@pytest.mark.parametrize("n_out,K", [(64, 128), (100, 2080), (4096, 4096)])
def test_weight_prepare_fp4_builds_the_tiled_layout(gpu, oracle, n_out, K, block):
    torch, dev, lib = gpu
    rng = np.random.default_rng(6)
    nib = rng.integers(0, 256, size=(n_out, K // 2), dtype=np.uint8)
    sc = rng.integers(0, 0x7F, size=(n_out, K // block), dtype=np.uint8)
    nd, sd = to_dev(torch, dev, nib), to_dev(torch, dev, sc)
    size = lib.tiled_size(oracle.FP4, n_out, K)
    assert size == ((n_out + 15) // 16) * ((K + 127) // 128) * (1024 + 128)
    td = torch.full((size + 64,), 0xAA, dtype=torch.uint8, device=dev)
    assert lib.weight_prepare_fp4(nd.data_ptr(), sd.data_ptr(), block, n_out, K, td.data_ptr()) == 0
    want = tiled_reference_fp4(nib, sc, n_out, K, block)
    got = td.cpu().numpy()
    assert np.array_equal(got[:want.size], want) and np.all(got[size:] == 0xAA)
    assert lib.weight_release(nd.data_ptr()) == 0
    assert lib.weight_prepare_fp4(nd.data_ptr(), None, block, n_out, K, td.data_ptr()) == -1
    assert lib.weight_prepare_fp4(nd.data_ptr(), sd.data_ptr(), 8, n_out, K, td.data_ptr()) == -1
    assert lib.weight_prepare_fp4(nd.data_ptr(), sd.data_ptr(), block, n_out, 48, td.data_ptr()) == -1


@pytest.mark.parametrize("block", [16, 32])
@pytest.mark.parametrize("tokens", [1, 2, 4, 5, 9, 16])
@pytest.mark.parametrize("n_out,K", [(300, 544), (4096, 4096), (1024, 4096), (512, 14336), (70000, 32), (8200, 1024), (65600, 160)])
def test_prepared_fp4_weights_on_the_matrix_cores(gpu, pkg, oracle, tokens, n_out, K, block):
    """Every launch shape of the FP4 matrix-core kernel on the tiled copy (few / several / many row tiles per CU, short
    and long rows, ragged row counts, rows that end inside a 128-element chunk), 1..16 tokens, against the exact
    contraction; alpha / beta; after release the call is back on the row-major kernel."""
    torch, dev, lib = gpu
    seed = synth.seed_for(3, 400 + n_out % 91 + tokens + block)
    nib, sc = synth.weights_fp4(seed, n_out, K, block)
    X = synth.activations(seed, tokens, K)
    nd, sd, xd = to_dev(torch, dev, nib), to_dev(torch, dev, sc), to_dev(torch, dev, X)
    td = torch.zeros(lib.tiled_size(oracle.FP4, n_out, K), dtype=torch.uint8, device=dev)
    want = oracle.linear_exact(oracle.dequant_weight(nib, oracle.FP4, n_out, K, blk_sc=sc, block=block), X)
    c0 = synth.activations(seed + 1, tokens, n_out)
    assert lib.weight_prepare_fp4(nd.data_ptr(), sd.data_ptr(), block, n_out, K, td.data_ptr()) == 0
    try:
        y = torch.zeros(tokens * n_out + 64, dtype=torch.int16, device=dev)
        assert lib.linear(nd.data_ptr(), oracle.FP4, xd.data_ptr(), y.data_ptr(), n_out, tokens, K, blk_sc=sd.data_ptr(), block_size=block) == 0
        # one or two tokens stay on the dot2 kernel unless the rows are long and the row tiles few (256 CUs on the test GPU)
        pays = tokens >= 3 or (K > 8192 and ((n_out + 15) // 16) // 256 < 2)
        assert lib.last_kernel() == ("gemv_mfma_tiled" if pays else "gemv_dot2")
        out = from_dev(y, np.uint16)
        assert not out[tokens * n_out:].any(), "wrote past the end"
        got = out[: tokens * n_out].reshape(tokens, n_out)
        check_rows(bf16_f64(oracle, got), want, f"fp4 tiled {n_out}x{K} M={tokens} b={block}")
        check_bf16_close(got, want, "fp4 tiled", slack_ulp=1.0, abs_floor=2e-5)
        yb = to_dev(torch, dev, c0.reshape(-1))
        assert lib.linear(nd.data_ptr(), oracle.FP4, xd.data_ptr(), yb.data_ptr(), n_out, tokens, K, blk_sc=sd.data_ptr(), block_size=block,
                          alpha=0.5, beta=-2.0) == 0
        check_rows(bf16_f64(oracle, from_dev(yb, np.uint16).reshape(tokens, n_out)), 0.5 * want - 2.0 * bf16_f64(oracle, c0), "fp4 tiled alpha beta")
        # other block scales behind the same codes: the copy no longer applies
        other = to_dev(torch, dev, sc)
        assert lib.linear(nd.data_ptr(), oracle.FP4, xd.data_ptr(), y.data_ptr(), n_out, tokens, K, blk_sc=other.data_ptr(), block_size=block) == 0
        assert lib.last_kernel() == "gemv_dot2"
    finally:
        assert lib.weight_release(nd.data_ptr()) == 0
    assert lib.linear(nd.data_ptr(), oracle.FP4, xd.data_ptr(), y.data_ptr(), n_out, tokens, K, blk_sc=sd.data_ptr(), block_size=block) == 0
    assert lib.last_kernel() == "gemv_dot2"


@pytest.mark.parametrize("block", [16, 32])
@pytest.mark.parametrize("tokens,n_out,K", [(48, 256, 128), (64, 300, 384), (130, 776, 1152), (512, 1024, 2048), (200, 520, 4096),
                                            (256, 4096, 1024), (1000, 12288, 256)])
def test_prepared_fp4_weights_in_the_prefill_gemm(gpu, pkg, oracle, tokens, n_out, K, block):
    """FP4 prefill on the tiled copy (codes and block scales fed to the matrix cores from registers): every tile shape
    (64 / 128 tokens x 192 / 256 features), the k split (few output tiles, long K) and its combine, ragged token and
    feature counts, against the exact contraction; alpha / beta; without whole 128-element chunks, or after release, the
    two-operand kernel takes the call."""
    torch, dev, lib = gpu
    seed = synth.seed_for(3, 900 + n_out % 89 + tokens + block)
    nib, sc = synth.weights_fp4(seed, n_out, K, block)
    X = synth.activations(seed, tokens, K)
    nd, sd, xd = to_dev(torch, dev, nib), to_dev(torch, dev, sc), to_dev(torch, dev, X)
    td = torch.zeros(lib.tiled_size(oracle.FP4, n_out, K), dtype=torch.uint8, device=dev)
    want = oracle.linear_exact(oracle.dequant_weight(nib, oracle.FP4, n_out, K, blk_sc=sc, block=block), X)
    c0 = synth.activations(seed + 1, tokens, n_out)
    assert lib.weight_prepare_fp4(nd.data_ptr(), sd.data_ptr(), block, n_out, K, td.data_ptr()) == 0
    try:
        y = torch.zeros(tokens * n_out + 64, dtype=torch.int16, device=dev)
        assert lib.linear(nd.data_ptr(), oracle.FP4, xd.data_ptr(), y.data_ptr(), n_out, tokens, K, blk_sc=sd.data_ptr(), block_size=block) == 0
        assert lib.last_kernel() == "gemm_mfma_tiled"
        out = from_dev(y, np.uint16)
        assert not out[tokens * n_out:].any(), "wrote past the end"
        got = out[: tokens * n_out].reshape(tokens, n_out)
        check_rows(bf16_f64(oracle, got), want, f"fp4 prefill {n_out}x{K} M={tokens} b={block}")
        check_bf16_close(got, want, "fp4 prefill", slack_ulp=1.0, abs_floor=2e-5)
        yb = to_dev(torch, dev, c0.reshape(-1))
        assert lib.linear(nd.data_ptr(), oracle.FP4, xd.data_ptr(), yb.data_ptr(), n_out, tokens, K, blk_sc=sd.data_ptr(), block_size=block,
                          alpha=0.5, beta=-2.0) == 0
        check_rows(bf16_f64(oracle, from_dev(yb, np.uint16).reshape(tokens, n_out)), 0.5 * want - 2.0 * bf16_f64(oracle, c0), "fp4 prefill alpha beta")
        # the entry point that allocates nothing takes the same route (its k split uses the static scratch)
        yn = torch.zeros(tokens * n_out, dtype=torch.int16, device=dev)
        assert lib.linear(nd.data_ptr(), oracle.FP4, xd.data_ptr(), yn.data_ptr(), n_out, tokens, K, blk_sc=sd.data_ptr(), block_size=block, noalloc=True) == 0
        assert lib.last_kernel() == "gemm_mfma_tiled"
        assert np.array_equal(from_dev(yn, np.uint16), out[: tokens * n_out])
    finally:
        assert lib.weight_release(nd.data_ptr()) == 0
    assert lib.linear(nd.data_ptr(), oracle.FP4, xd.data_ptr(), y.data_ptr(), n_out, tokens, K, blk_sc=sd.data_ptr(), block_size=block) == 0
    assert lib.last_kernel() == "gemm_mfma"
    check_rows(bf16_f64(oracle, from_dev(y, np.uint16)[: tokens * n_out].reshape(tokens, n_out)), want, "fp4 prefill, row-major")


def test_fp4_prefill_without_whole_chunks_stays_on_the_two_operand_kernel(gpu, pkg, oracle):
    torch, dev, lib = gpu
    tokens, n_out, K, block = 64, 256, 160, 16
    nib, sc = synth.weights_fp4(77, n_out, K, block)
    X = synth.activations(77, tokens, K)
    nd, sd, xd = to_dev(torch, dev, nib), to_dev(torch, dev, sc), to_dev(torch, dev, X)
    td = torch.zeros(lib.tiled_size(oracle.FP4, n_out, K), dtype=torch.uint8, device=dev)
    assert lib.weight_prepare_fp4(nd.data_ptr(), sd.data_ptr(), block, n_out, K, td.data_ptr()) == 0
    try:
        y = torch.zeros(tokens * n_out, dtype=torch.int16, device=dev)
        assert lib.linear(nd.data_ptr(), oracle.FP4, xd.data_ptr(), y.data_ptr(), n_out, tokens, K, blk_sc=sd.data_ptr(), block_size=block) == 0
        assert lib.last_kernel() == "gemm_mfma"
        want = oracle.linear_exact(oracle.dequant_weight(nib, oracle.FP4, n_out, K, blk_sc=sc, block=block), X)
        check_rows(bf16_f64(oracle, from_dev(y, np.uint16).reshape(tokens, n_out)), want, "fp4 K=160")
    finally:
        assert lib.weight_release(nd.data_ptr()) == 0


def test_reserved_workspace_keeps_the_k_split_under_capture(gpu, pkg, oracle):
    """hip_quant_workspace_reserve: a k-split GEMM captured into a graph on a stream whose scratch buffer was sized
    beforehand gives the bits of the eager call (same kernels, same FP32 order); the library allocates nothing while
    the stream is capturing, and the reserve call itself is refused there."""
    torch, dev, lib = gpu
    tokens, n_out, K = 512, 4096, 4096                  # 64 tiles of 128 x 256 on 256 CUs: the k range splits in four
    seed = synth.seed_for(7, 33)
    W, X = synth.weights_e5m2(seed, n_out, K), synth.activations(seed, tokens, K)
    wd, xd = to_dev(torch, dev, W), to_dev(torch, dev, X)
    y_eager = torch.zeros(tokens * n_out, dtype=torch.int16, device=dev)
    y_graph = torch.zeros_like(y_eager)
    assert lib.linear(wd.data_ptr(), oracle.E5M2, xd.data_ptr(), y_eager.data_ptr(), n_out, tokens, K) == 0
    torch.cuda.synchronize()
    stream = torch.cuda.Stream(device=dev)
    graph = torch.cuda.CUDAGraph()
    lib.set_sync(False)
    try:
        assert lib.set_stream(stream.cuda_stream) == 0
        assert lib.workspace_reserve(8 * tokens * n_out * 4) == 0        # this thread's buffer for this stream
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream, capture_error_mode="thread_local"):
            assert lib.workspace_reserve(1 << 30) == -1                   # never while capturing
            assert lib.linear(wd.data_ptr(), oracle.E5M2, xd.data_ptr(), y_graph.data_ptr(), n_out, tokens, K) == 0
        for _ in range(2):
            y_graph.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(y_graph, y_eager)
    finally:
        lib.set_stream(None)
        lib.set_sync(True)
    want = oracle.linear_exact(oracle.dequant_weight(W, oracle.E5M2, n_out, K), X[:16])
    check_rows(bf16_f64(oracle, from_dev(y_graph, np.uint16).reshape(tokens, n_out)[:16]), want, "captured k-split GEMM")
