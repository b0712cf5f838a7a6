"""hip_quant_gemm_noalloc -- the entry point that allocates nothing -- against hip_quant_gemm through the
C-ABI: same kernels, so the outputs must agree bit for bit; its k-split partial sums live in a static
device array that every call on the GPU shares, so the cases run back to back, a smaller one after a larger
one, and a stale partial sum from the earlier call would show."""
import numpy as np
from oracle import synth
import pytest

from gpu_util import check_rows, from_dev, to_dev

pytestmark = pytest.mark.gpu

E5M2, E4M3, FP4 = 5, 4, 6


HALF = 2


def both_ways(gpu, pkg, oracle, tokens, n_out, K, w_type=E5M2, expect=None, tiled=False, half=False, **kw):
    """half: IEEE-half activations and outputs (bit-for-bit comparison of the two entry points only; the half route's
    own parity tests check it against the oracle).  tiled: the weight's load-time tiled copy is registered first."""
    torch, dev, lib = gpu
    seed = synth.seed_for(7, tokens % 61 + n_out % 17)
    X = synth.activations(seed, tokens, K)
    blk = {}
    scd = None
    if w_type == FP4:
        W, sc = synth.weights_fp4(seed, n_out, K, 16)
        scd = to_dev(torch, dev, sc)
        blk = dict(blk_sc=scd.data_ptr(), block_size=16)
        Wd = oracle.dequant_weight(W, oracle.FP4, n_out, K, blk_sc=sc, block=16)
    else:
        W = synth.weights_e5m2(seed, n_out, K)
        Wd = oracle.dequant_weight(W, oracle.E5M2, n_out, K, kw.get("inv_scale", 1.0))
    if half:
        X = np.random.default_rng(seed).standard_normal((tokens, K)).astype(np.float16).view(np.uint16)
        kw = dict(kw, act_type=HALF)
    wd, xd = to_dev(torch, dev, W), to_dev(torch, dev, X)
    c0 = synth.activations(seed + 1, tokens, n_out)
    td = None
    if tiled:
        td = torch.zeros(lib.tiled_size(w_type, n_out, K), dtype=torch.uint8, device=dev)
        if w_type == FP4:
            assert lib.weight_prepare_fp4(wd.data_ptr(), scd.data_ptr(), 16, n_out, K, td.data_ptr()) == 0
        else:
            assert lib.weight_prepare(wd.data_ptr(), w_type, n_out, K, K, td.data_ptr()) == 0
    outs = []
    try:
        for noalloc in (False, True):
            y = to_dev(torch, dev, np.concatenate([c0.ravel(), np.zeros(64, dtype=np.uint16)]))
            assert lib.linear(wd.data_ptr(), w_type, xd.data_ptr(), y.data_ptr(), n_out, tokens, K, noalloc=noalloc, **blk, **kw) == 0
            if expect:
                assert lib.last_kernel() == expect
            out = from_dev(y, np.uint16)
            assert not out[tokens * n_out:].any(), "wrote past the end"
            outs.append(out[: tokens * n_out].reshape(tokens, n_out))
    finally:
        if tiled:
            assert lib.weight_release(wd.data_ptr()) == 0
    assert np.array_equal(outs[0], outs[1]), f"{tokens}x{n_out}x{K}: the two entry points differ"
    if half:
        return
    want = kw.get("alpha", 1.0) * oracle.linear_exact(Wd, X) + kw.get("beta", 0.0) * oracle.bf16_to_f32(c0).astype(np.float64)
    check_rows(oracle.bf16_to_f32(outs[1]).astype(np.float64), want, f"noalloc {tokens}x{n_out}x{K}")


def test_noalloc_entry_point_matches_hip_quant_gemm(gpu, pkg, oracle):
    torch, dev, lib = gpu
    # k split over four workgroup ranges: 4 * 512 * 4096 floats = the whole 32 MiB of static scratch
    both_ways(gpu, pkg, oracle, 512, 4096, 12288, expect="gemm_mfma")
    # a smaller k-split right after it (two ranges), with alpha / beta and a per-tensor scale: reuses the same array
    both_ways(gpu, pkg, oracle, 128, 1536, 2048, expect="gemm_mfma", alpha=0.5, beta=-2.0, inv_scale=0.37)
    # the paths that need no scratch: GEMV, matrix-core GEMV, unsplit GEMM, FP4, generic
    both_ways(gpu, pkg, oracle, 1, 1024, 4096, expect="gemv_dot2")
    both_ways(gpu, pkg, oracle, 16, 768, 2048, expect="gemv_mfma")
    both_ways(gpu, pkg, oracle, 256, 4096, 1024, expect="gemm_mfma")
    both_ways(gpu, pkg, oracle, 3, 512, 2048, w_type=FP4, expect="gemv_dot2")
    both_ways(gpu, pkg, oracle, 3, 40, 50, expect="generic", inv_scale=0.3)
    # the other routes that split K through the static array: FP4 on its tiled copy (eight ranges: 16.8 MB of partial
    # sums) and HALF activations (eight ranges of a short prompt)
    both_ways(gpu, pkg, oracle, 128, 4096, 14336, w_type=FP4, tiled=True, expect="gemm_mfma_tiled")
    both_ways(gpu, pkg, oracle, 64, 1024, 4096, half=True, expect="gemm_mfma_half", inv_scale=0.37)
    # the first shape again, after the others
    both_ways(gpu, pkg, oracle, 512, 4096, 12288, expect="gemm_mfma")


def test_noalloc_entry_point_refuses_what_does_not_fit(gpu, pkg, oracle, capfd):
    """512 tokens x 4352 features split K in four: 4 * 512 * 4352 * 4 bytes = 35.7 MB of partial sums, more than
    the static 32 MiB.  The call says so, launches nothing and leaves C alone; hip_quant_gemm takes the shape."""
    torch, dev, lib = gpu
    tokens, n_out, K = 512, 4352, 12288
    w = torch.zeros(n_out * K, dtype=torch.uint8, device=dev)
    x = torch.zeros(tokens * K, dtype=torch.int16, device=dev)
    y = torch.full((tokens * n_out,), 0x1234, dtype=torch.int16, device=dev)
    assert lib.linear(w.data_ptr(), E5M2, x.data_ptr(), y.data_ptr(), n_out, tokens, K, noalloc=True) == -1
    assert "static scratch" in capfd.readouterr().err
    assert bool((y == 0x1234).all())
    assert lib.linear(w.data_ptr(), E5M2, x.data_ptr(), y.data_ptr(), n_out, tokens, K) == 0
    assert lib.last_kernel() == "gemm_mfma" and not bool(y.any())
    # argument checks come first, as in hip_quant_gemm
    p = w.data_ptr()
    assert lib.quant_gemm(1, 0, 16, 1, 16, 1.0, p, E5M2, 16, 1.0, p, E5M2, 16, 1.0, 0.0, p, 3, 16, noalloc=True) == -1
