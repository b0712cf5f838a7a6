"""The C++ host mirror (Matrix / MatrixData / GpuControl / Rocblas) drives the kernel library the
way cccc's graph does: Matrix::mulBatched(W, X, R, TRANS, NO_TRANS) on a weight loaded with
loadQuantizedDirect / setBlockScaleFromHost, or quantized in place with quantizeWeights."""
import numpy as np
from oracle import synth
import pytest

from gpu_util import check_rows

pytestmark = pytest.mark.gpu

FLOAT, HALF, BF16, E4M3, E5M2, FP4 = 0, 2, 3, 4, 5, 6
NO_TRANS, TRANS = 0, 1


@pytest.fixture(scope="module")
def host(gpu, pkg):
    h = pkg.host_api.host()
    h.init(0)
    return h


def f64(oracle, bits):
    return oracle.bf16_to_f32(bits).astype(np.float64)


@pytest.mark.parametrize("tokens", [1, 4, 16, 64])
def test_mul_batched_fp8_linear(host, pkg, oracle, tokens):
    n_out, K = 768, 1024
    Wq = synth.weights_e5m2(11, n_out, K)
    X = synth.activations(11, tokens, K)
    W = host.matrix(K, n_out, 1, 1, BF16)                     # allocated as the activation type, re-typed on load
    W.load_quantized(Wq, 1.0, E5M2)
    assert W.dtype == E5M2 and W.quant_scale == 1.0
    Xm = host.matrix(K, tokens, 1, 1, BF16); Xm.upload(X)
    R = host.matrix(n_out, tokens, 1, 1, BF16)
    assert pkg.host_api.mul_batched(W, Xm, R, TRANS, NO_TRANS) == 0
    y = R.download(np.uint16, tokens * n_out).reshape(tokens, n_out)
    check_rows(f64(oracle, y), oracle.linear_exact(oracle.dequant_weight(Wq, oracle.E5M2, n_out, K), X), f"host M={tokens}")
    # the 2-D form (rows x number) reaches the same dispatcher
    W2 = host.matrix(K, 1, 1, n_out, BF16); W2.load_quantized(Wq, 1.0, E5M2)
    X2 = host.matrix(K, 1, 1, tokens, BF16); X2.upload(X)
    R2 = host.matrix(n_out, 1, 1, tokens, BF16)
    assert pkg.host_api.mul(W2, X2, R2, 1.0, 0.0, TRANS, NO_TRANS) == 0
    # (this storage is N x 1-column, so it keeps no tiled copy: same products on the row-major bytes, possibly summed in another order)
    y2 = R2.download(np.uint16, tokens * n_out).reshape(tokens, n_out)
    check_rows(f64(oracle, y2), oracle.linear_exact(oracle.dequant_weight(Wq, oracle.E5M2, n_out, K), X), f"host 2-D M={tokens}")
    assert np.abs(f64(oracle, y2) - f64(oracle, y)).max() <= 2.0 ** -7 * np.abs(f64(oracle, y)).max()
    # shapes that do not fit come back as an error code before anything is launched
    assert pkg.host_api.mul(W, Xm, R, 1.0, 0.0, TRANS, NO_TRANS) == -1
    if tokens > 1:
        assert pkg.host_api.mul_batched(W, Xm, R2, TRANS, NO_TRANS) == -1


def test_mul_batched_fp4_two_batches_use_per_batch_offsets(host, pkg, oracle):
    n_out, K, tokens, batch = 128, 256, 3, 2
    nib, sc, Wd = [], [], []
    for b in range(batch):
        n, s = synth.weights_fp4(20 + b, n_out, K)
        nib.append(n); sc.append(s)
        Wd.append(oracle.dequant_weight(n, oracle.FP4, n_out, K, blk_sc=s))
    X = synth.activations(21, tokens * batch, K).reshape(batch, tokens, K)
    W = host.matrix(K, n_out, 1, batch, BF16)
    W.load_quantized(np.concatenate([n.ravel() for n in nib]), 1.0, FP4)
    W.set_block_scale(np.concatenate([s.ravel() for s in sc]))
    assert W.dtype == FP4 and W.block_scale_ptr
    Xm = host.matrix(K, tokens, 1, batch, BF16); Xm.upload(X)
    R = host.matrix(n_out, tokens, 1, batch, BF16)
    assert pkg.host_api.mul_batched(W, Xm, R, TRANS, NO_TRANS) == 0
    y = R.download(np.uint16, batch * tokens * n_out).reshape(batch, tokens, n_out)
    for b in range(batch):
        check_rows(f64(oracle, y[b]), oracle.linear_exact(Wd[b], X[b]), f"batch {b}")


def test_quantize_weights_in_place(host, pkg, oracle):
    n_out, K = 96, 128
    w = synth.weights_f32(30, n_out, K)                   # exactly representable in BF16
    wb = oracle.f32_to_bf16(w)
    # FP8: per-tensor absmax scale, truncating encoder
    for target, top in ((E5M2, 57344.0), (E4M3, 448.0)):
        W = host.matrix(K, n_out, 1, 1, BF16); W.upload(wb)
        W.quantize(target)
        amax = np.float32(np.abs(w).max())
        assert W.dtype == target
        assert np.float32(W.quant_scale) == amax / np.float32(top)
        fwd = np.float32(top) / amax
        rc, want = oracle.convert(w, oracle.FLOAT, target, w.size, float(fwd))
        assert rc == 0 and np.array_equal(W.download(np.uint8, w.size), want)
    # FP4: block scales, quant_scale stays 1
    W = host.matrix(K, n_out, 1, 1, BF16); W.upload(wb)
    W.quantize(FP4)
    wn, ws = oracle.quantize_fp4_blockscale_kernel(w, 16)
    assert W.dtype == FP4 and W.quant_scale == 1.0
    assert np.array_equal(W.download(np.uint8, w.size // 2), wn)
    assert np.array_equal(W.block_scales(), ws)
    # small views are left alone (either dim < 64), as the reference's policy
    small = host.matrix(32, 128, 1, 1, BF16); small.upload(wb.ravel()[:32 * 128])
    small.quantize(E5M2)
    assert small.dtype == BF16


def test_quantized_then_multiplied_matches_the_oracle(host, pkg, oracle):
    n_out, K, tokens = 256, 512, 2
    w = synth.weights_f32(31, n_out, K)
    X = synth.activations(31, tokens, K)
    W = host.matrix(K, n_out, 1, 1, BF16); W.upload(oracle.f32_to_bf16(w))
    W.quantize(E5M2)
    codes = W.download(np.uint8, w.size).reshape(n_out, K)
    Xm = host.matrix(K, tokens, 1, 1, BF16); Xm.upload(X)
    R = host.matrix(n_out, tokens, 1, 1, BF16)
    assert pkg.host_api.mul_batched(W, Xm, R, TRANS, NO_TRANS) == 0
    y = R.download(np.uint16, tokens * n_out).reshape(tokens, n_out)
    want = oracle.linear_exact(oracle.dequant_weight(codes, oracle.E5M2, n_out, K, W.quant_scale), X)
    check_rows(f64(oracle, y), want, "quantize+mul")
    # and the quantized product is close to the unquantized one (E5M2 truncation: <= 25 % per weight, averaged out)
    full = oracle.linear_exact(oracle.f32_to_bf16(w), X)
    assert np.linalg.norm(f64(oracle, y) - full) / np.linalg.norm(full) < 0.15


def test_tracked_allocations_are_released(host, pkg):
    base = host.c.cccc_gpu_allocated_bytes()
    m = host.matrix(1024, 1024, 1, 1, BF16)
    assert host.c.cccc_gpu_allocated_bytes() == base + 2 * 1024 * 1024
    del m
    assert host.c.cccc_gpu_allocated_bytes() == base


def test_rewriting_a_prepared_weight_drops_its_tiled_copy(gpu, pkg, oracle):
    """The tiled copy is keyed on the weight's pointer: every host path that writes the storage (a second
    loadQuantizedDirect into the same allocation, a raw upload) must drop it, or the matrix-core GEMV would keep
    computing from the old bytes."""
    torch, dev, lib = gpu
    host = pkg.host_api.host()
    host.init(0)
    host.set_repack(True)
    n_out, K, tokens = 1024, 2048, 4
    X = synth.activations(51, tokens, K)
    xm = host.matrix(K, tokens, 1, 1, BF16)
    xm.upload(X)
    ym = host.matrix(n_out, tokens, 1, 1, BF16)
    first, second, third = (synth.weights_e5m2(52 + i, n_out, K) for i in range(3))
    wm = host.matrix(K, n_out, 1, 1, E5M2)

    def run(codes, expect_kernel):
        assert pkg.host_api.mul_batched(wm, xm, ym, ta=1, tb=0) == 0
        assert lib.last_kernel() == expect_kernel
        want = oracle.linear_exact(oracle.dequant_weight(codes, oracle.E5M2, n_out, K), X)
        check_rows(oracle.bf16_to_f32(ym.download(np.uint16, tokens * n_out).reshape(tokens, n_out)).astype(np.float64), want, expect_kernel)

    wm.load_quantized(first, 1.0, E5M2)
    ptr = wm.data_ptr
    run(first, "gemv_mfma_tiled")
    wm.load_quantized(second, 1.0, E5M2)                 # same allocation, new bytes: a new tiled copy of the new bytes
    assert wm.data_ptr == ptr
    run(second, "gemv_mfma_tiled")
    wm.upload(third)                                     # raw write: the copy is dropped, the row-major kernel reads the new bytes
    run(third, "gemv_dot2")
    assert wm.prepare_tiled()
    run(third, "gemv_mfma_tiled")
