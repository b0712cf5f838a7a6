"""Prompt-phase neighbours (T tokens at once) against the CPU oracle of the one-token step, through the C-ABI."""
import ctypes

import numpy as np
import pytest

from gpu_util import check_rows, from_dev, to_dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dec():
    from oracle import decode_oracle
    return decode_oracle


def ulp_close(got_bits, want_vals, ulps=1.0, floor=1e-6):
    got = (got_bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    want = np.asarray(want_vals, dtype=np.float64)
    tol = ulps * np.maximum(np.abs(want), 2.0 ** -120) * 2.0 ** -8 + floor
    return np.abs(got - want) <= tol


ptr = lambda t: ctypes.c_void_p(t.data_ptr())


@pytest.mark.parametrize("n_q,n_kv,normed", [(4, 2, True), (8, 2, True), (2, 2, False)])
def test_rows_norm_rope_append_equals_the_one_token_kernel(gpu, oracle, dec, n_q, n_kv, normed):
    """T tokens through hip_qk_norm_rope_kv_rows_bf16 leave the bytes T calls of hip_qk_norm_rope_kv_bf16 leave."""
    torch, dev, lib = gpu
    rng = np.random.default_rng(3)
    t_kv, T, pos0 = 96, 37, 11
    cfg = dec.DecodeConfig(n_q=n_q, n_kv=n_kv, t_kv=t_kv)
    cos, sin = dec.rope_tables(cfg)
    q = oracle.f32_to_bf16((2 * rng.standard_normal((T, n_q, 128))).astype(np.float32))
    k = oracle.f32_to_bf16((2 * rng.standard_normal((T, n_kv, 128))).astype(np.float32))
    v = oracle.f32_to_bf16(rng.standard_normal((T, n_kv, 128)).astype(np.float32))
    qw = oracle.f32_to_bf16((1 + 0.1 * rng.standard_normal(128)).astype(np.float32))
    kw = oracle.f32_to_bf16((1 + 0.1 * rng.standard_normal(128)).astype(np.float32))
    qd, kd, vd, qwd, kwd, cd, sd = (to_dev(torch, dev, a) for a in (q, k, v, qw, kw, cos, sin))
    nq_w, nk_w = (ptr(qwd), ptr(kwd)) if normed else (ctypes.c_void_p(0), ctypes.c_void_p(0))
    base = oracle.f32_to_bf16(rng.standard_normal((n_kv, t_kv, 128)).astype(np.float32))
    kc, vc = to_dev(torch, dev, base), to_dev(torch, dev, base[::-1].copy())
    q_out = torch.zeros(T * n_q * 128, dtype=torch.int16, device=dev)
    assert lib.c.hip_qk_norm_rope_kv_rows_bf16(ptr(qd), ptr(kd), ptr(vd), nq_w, nk_w, ptr(cd), ptr(sd), ptr(q_out), ptr(kc), ptr(vc),
                                               n_q, n_kv, 128, t_kv, T, pos0, ctypes.c_float(1e-6)) == 0
    kc2, vc2 = to_dev(torch, dev, base), to_dev(torch, dev, base[::-1].copy())
    q_ref = np.zeros((T, n_q, 128), dtype=np.uint16)
    for t in range(T):
        q1 = torch.zeros(n_q * 128, dtype=torch.int16, device=dev)
        pd = torch.tensor([pos0 + t], dtype=torch.int32, device=dev)
        qt, kt, vt = (to_dev(torch, dev, a[t]) for a in (q, k, v))
        assert lib.c.hip_qk_norm_rope_kv_bf16(ptr(qt), ptr(kt), ptr(vt), nq_w, nk_w, ptr(cd), ptr(sd), ptr(q1), ptr(kc2), ptr(vc2),
                                              n_q, n_kv, 128, t_kv, ptr(pd), ctypes.c_float(1e-6)) == 0
        q_ref[t] = from_dev(q1, np.uint16).reshape(n_q, 128)
    assert np.array_equal(from_dev(q_out, np.uint16).reshape(T, n_q, 128), q_ref)
    assert np.array_equal(from_dev(kc, np.uint16), from_dev(kc2, np.uint16))
    assert np.array_equal(from_dev(vc, np.uint16), from_dev(vc2, np.uint16))
    # a prompt that would run past the cache is refused
    assert lib.c.hip_qk_norm_rope_kv_rows_bf16(ptr(qd), ptr(kd), ptr(vd), nq_w, nk_w, ptr(cd), ptr(sd), ptr(q_out), ptr(kc), ptr(vc),
                                               n_q, n_kv, 128, t_kv, T, t_kv - T + 1, ctypes.c_float(1e-6)) == -1


@pytest.mark.parametrize("n_q,n_kv,t_kv,T,pos0", [(4, 2, 200, 1, 0), (4, 2, 200, 5, 0), (4, 2, 200, 16, 3), (8, 2, 200, 17, 0), (8, 2, 300, 100, 70),
                                                     (2, 2, 200, 64, 64), (8, 2, 1024, 130, 800), (2, 1, 128, 33, 95)])
def test_prefill_attention_follows_the_oracle_token_by_token(gpu, oracle, dec, n_q, n_kv, t_kv, T, pos0):
    """Every token of the prompt attends to the cache rows up to its own position: the oracle's one-token attention,
    token by token, on the same caches.  Rows past the prompt hold NaN patterns and must not leak."""
    torch, dev, lib = gpu
    rng = np.random.default_rng(T + pos0)
    q = oracle.f32_to_bf16(rng.standard_normal((T, n_q, 128)).astype(np.float32))
    kc = oracle.f32_to_bf16(rng.standard_normal((n_kv, t_kv, 128)).astype(np.float32))
    vc = oracle.f32_to_bf16(rng.standard_normal((n_kv, t_kv, 128)).astype(np.float32))
    kc[:, pos0 + T:] = 0x7FC1
    vc[:, pos0 + T:] = 0xFFFF
    qd, kd, vd = to_dev(torch, dev, q), to_dev(torch, dev, kc), to_dev(torch, dev, vc)
    y = torch.zeros(T * n_q * 128 + 64, dtype=torch.int16, device=dev)
    assert lib.c.hip_attention_prefill_bf16(ptr(qd), ptr(kd), ptr(vd), ptr(y), n_q, n_kv, 128, t_kv, T, pos0) == 0
    out = from_dev(y, np.uint16)
    assert not out[T * n_q * 128:].any()
    got = out[:T * n_q * 128].reshape(T, n_q, 128)
    kf, vf = dec.f(kc), dec.f(vc)
    kf[:, pos0 + T:], vf[:, pos0 + T:] = 0.0, 0.0               # masked in the oracle too; NaN * 0 would poison its matrix products
    for t in range(T):
        want = dec.attention(dec.f(q[t]), kf, vf, pos0 + t, n_q, n_kv)
        assert np.isfinite(dec.f(got[t])).all(), t
        assert ulp_close(got[t], want, ulps=2.0, floor=2e-3 * np.abs(want).max()).all(), t
        assert np.linalg.norm(dec.f(got[t]) - want) <= 4e-3 * np.linalg.norm(want), t
    assert lib.c.hip_attention_prefill_bf16(ptr(qd), ptr(kd), ptr(vd), ptr(y), n_q, n_kv, 128, t_kv, T, t_kv - T + 1) == -1
    assert lib.c.hip_attention_prefill_bf16(ptr(qd), ptr(kd), ptr(vd), ptr(y), 3 * n_kv, n_kv, 128, t_kv, T, pos0) == -1


@pytest.mark.parametrize("w_type,tiled", [("e5m2", False), ("e5m2", True), ("e4m3", True)])
@pytest.mark.parametrize("tokens,widths,K", [(60, (512, 256, 256), 256), (130, (1000, 72), 1024), (300, (2048, 512, 512), 512), (48, (64,), 64), (20, (512, 256), 256),
                                             (7, (512, 256, 256), 2048), (2, (1000, 72), 1024)])
def test_linears_that_share_their_input_in_one_launch_equal_the_separate_calls(gpu, oracle, w_type, tiled, tokens, widths, K):
    """hip_quant_gemm_segments (the q, k, v projections of a prompt as one launch) against one hip_quant_gemm call per
    weight and against the exact contraction, on the file layout and on tiled copies, with a different per-tensor scale per
    weight for E4M3.  Byte for byte where K is too short for a k split (under 1024); at K = 1024 the joint launch splits
    its few tiles in two k ranges with one combine for all segments, the separate calls do not, and the two differ by
    the order of the FP32 sums only (as they do up to 16 tokens, where a separate call is a matrix-vector kernel).
    Unsupported arguments are refused."""
    torch, dev, lib = gpu
    rng = np.random.default_rng(tokens + K + len(widths))
    wt = oracle.E5M2 if w_type == "e5m2" else oracle.E4M3
    scales = [1.0] * len(widths) if w_type == "e5m2" else [0.011, 0.017, 0.023][:len(widths)]
    X = oracle.f32_to_bf16((rng.standard_normal((tokens, K)) * (0.05 if w_type == "e5m2" else 1.0)).astype(np.float32))
    xd = to_dev(torch, dev, X)
    wds, keep, sep, one, host_w = [], [], [], [], []
    for n_out in widths:
        W = rng.integers(0, 256, size=(n_out, K), dtype=np.uint8)
        if w_type == "e5m2": W[(W & 0x7C) == 0x7C] = 0x3C
        else: W[(W & 0x7F) == 0x7F] = 0x38
        host_w.append(W)
        wds.append(to_dev(torch, dev, W))
        if tiled:
            t = torch.zeros(lib.tiled_size(wt, n_out, K), dtype=torch.uint8, device=dev)
            assert lib.weight_prepare(wds[-1].data_ptr(), wt, n_out, K, K, t.data_ptr()) == 0
            keep.append(t)
        sep.append(torch.zeros(tokens * n_out + 64, dtype=torch.int16, device=dev))
        one.append(torch.zeros(tokens * n_out + 64, dtype=torch.int16, device=dev))
    try:
        for wd, y, n_out, sc in zip(wds, sep, widths, scales):
            assert lib.linear(wd.data_ptr(), wt, xd.data_ptr(), y.data_ptr(), n_out, tokens, K, sc) == 0
        n = len(widths)
        arr_i = (ctypes.c_int * n)(*widths)
        arr_w = (ctypes.c_void_p * n)(*[w.data_ptr() for w in wds])
        arr_s = (ctypes.c_float * n)(*scales)
        arr_y = (ctypes.c_void_p * n)(*[y.data_ptr() for y in one])
        call = lambda toks, k, typ: lib.c.hip_quant_gemm_segments(n, arr_i, arr_w, arr_s, arr_y, arr_i, typ, toks, k, K, ptr(xd), K)
        assert call(tokens, K, wt) == 0
        assert lib.last_kernel() == ("gemm_segments_tiled" if tiled else "gemm_segments")
        for y1, y3, n_out, W, sc in zip(one, sep, widths, host_w, scales):
            got = from_dev(y1, np.uint16)
            assert got[:tokens * n_out].any() and not got[tokens * n_out:].any()
            if K < 1024:
                assert np.array_equal(got, from_dev(y3, np.uint16))
            have = oracle.bf16_to_f32(got[:tokens * n_out].reshape(tokens, n_out)).astype(np.float64)
            other = oracle.bf16_to_f32(from_dev(y3, np.uint16)[:tokens * n_out].reshape(tokens, n_out)).astype(np.float64)
            want = oracle.linear_exact(oracle.dequant_fp8_to_bf16(W, wt, sc), X)
            check_rows(have, want, f"segment of {n_out} features")
            assert (np.linalg.norm(have - other, axis=1) <= 2e-3 * np.linalg.norm(want, axis=1)).all()
        assert call(1, K, wt) == -1 and call(tokens, K - 32, wt) == -1 and call(tokens, K, oracle.FP4) == -1
    finally:
        if tiled:
            for wd in wds:
                assert lib.weight_release(wd.data_ptr()) == 0


@pytest.mark.parametrize("block", [16, 32])
@pytest.mark.parametrize("tokens,widths,K", [(60, (512, 256, 256), 256), (130, (1000, 72), 1024), (300, (2048, 512, 512), 512), (5, (512, 256, 256), 1024)])
def test_fp4_linears_that_share_their_input_in_one_launch(gpu, oracle, block, tokens, widths, K):
    """hip_quant_gemm_segments on FP4 block-scale weights (tiled copies registered, which is what the FP4 GEMM reads) against
    one hip_quant_gemm call per weight -- byte for byte where K is too short for a k split (under 1024), within the order of
    the FP32 sums at K = 1024, where the joint launch splits its few tiles in two k ranges -- and against the exact
    contraction; without the tiled copies the call is refused."""
    torch, dev, lib = gpu
    rng = np.random.default_rng(tokens + K + block)
    X = oracle.f32_to_bf16(rng.standard_normal((tokens, K)).astype(np.float32))
    xd = to_dev(torch, dev, X)
    wds, sds, keep, sep, one, host_w, host_s = [], [], [], [], [], [], []
    for n_out in widths:
        host_w.append(rng.integers(0, 256, size=(n_out, K // 2), dtype=np.uint8))
        host_s.append(rng.integers(0x20, 0x40, size=(n_out, K // block), dtype=np.uint8))
        wds.append(to_dev(torch, dev, host_w[-1]))
        sds.append(to_dev(torch, dev, host_s[-1]))
        sep.append(torch.zeros(tokens * n_out + 64, dtype=torch.int16, device=dev))
        one.append(torch.zeros(tokens * n_out + 64, dtype=torch.int16, device=dev))
    n = len(widths)
    arr_i = (ctypes.c_int * n)(*widths)
    arr_w = (ctypes.c_void_p * n)(*[w.data_ptr() for w in wds])
    arr_s = (ctypes.c_float * n)(*([1.0] * n))
    arr_y = (ctypes.c_void_p * n)(*[y.data_ptr() for y in one])
    call = lambda: lib.c.hip_quant_gemm_segments(n, arr_i, arr_w, arr_s, arr_y, arr_i, oracle.FP4, tokens, K, K, ptr(xd), K)
    assert call() == -1                                         # no tiled copies yet
    for wd, sd, n_out in zip(wds, sds, widths):
        t = torch.zeros(lib.tiled_size(oracle.FP4, n_out, K), dtype=torch.uint8, device=dev)
        assert lib.weight_prepare_fp4(wd.data_ptr(), sd.data_ptr(), block, n_out, K, t.data_ptr()) == 0
        keep.append(t)
    try:
        for wd, sd, y, n_out in zip(wds, sds, sep, widths):
            assert lib.linear(wd.data_ptr(), oracle.FP4, xd.data_ptr(), y.data_ptr(), n_out, tokens, K, 1.0, sd.data_ptr(), block) == 0
            assert lib.last_kernel() == ("gemm_mfma_tiled" if tokens >= 17 else "gemv_mfma_tiled")
        assert call() == 0
        assert lib.last_kernel() == "gemm_segments_tiled"
        for y1, y3, n_out, W, sc in zip(one, sep, widths, host_w, host_s):
            got = from_dev(y1, np.uint16)
            assert got[:tokens * n_out].any() and not got[tokens * n_out:].any()
            if K < 1024:
                assert np.array_equal(got, from_dev(y3, np.uint16))
            have = oracle.bf16_to_f32(got[:tokens * n_out].reshape(tokens, n_out)).astype(np.float64)
            other = oracle.bf16_to_f32(from_dev(y3, np.uint16)[:tokens * n_out].reshape(tokens, n_out)).astype(np.float64)
            want = oracle.linear_exact(oracle.dequant_weight(W.reshape(-1), oracle.FP4, n_out, K, blk_sc=sc.reshape(-1), block=block), X)
            check_rows(have, want, f"FP4 segment of {n_out} features")
            assert (np.linalg.norm(have - other, axis=1) <= 2e-3 * np.linalg.norm(want, axis=1)).all()
    finally:
        for wd in wds:
            assert lib.weight_release(wd.data_ptr()) == 0


@pytest.mark.parametrize("w_type,tiled", [("e5m2", False), ("e5m2", True), ("e4m3", False), ("e4m3", True)])
@pytest.mark.parametrize("tokens,n_out,K", [(60, 512, 256), (130, 200, 1024), (300, 1536, 512), (9, 256, 2048), (2, 200, 1024)])
def test_gate_up_pair_gemm_with_swiglu_equals_the_three_calls(gpu, oracle, dec, w_type, tiled, tokens, n_out, K):
    """hip_quant_gemm_swiglu against two hip_quant_gemm calls and hip_swiglu_bf16 on the same inputs -- byte for byte where K
    is too short for a k split (under 1024), so every sum runs in the same order; at K = 1024 the pair launch splits its
    few tiles in two k ranges and its combine launch writes the product, which may then differ from the three calls where
    a gate or up sum lands on the other side of a BF16 rounding boundary -- and against the oracle's exact contraction, on
    the file layout and on the tiled copies, with the per-tensor scales of an E4M3 file differing between gate and up.
    Unsupported arguments are refused with -1."""
    torch, dev, lib = gpu
    rng = np.random.default_rng(tokens + n_out + K)
    wt = oracle.E5M2 if w_type == "e5m2" else oracle.E4M3
    sg, su = (1.0, 1.0) if w_type == "e5m2" else (0.011, 0.017)
    Wg = rng.integers(0, 256, size=(n_out, K), dtype=np.uint8)
    Wu = rng.integers(0, 256, size=(n_out, K), dtype=np.uint8)
    for W in (Wg, Wu):                                          # no NaN / Inf codes
        if w_type == "e5m2": W[(W & 0x7C) == 0x7C] = 0x3C
        else: W[(W & 0x7F) == 0x7F] = 0x38
    X = oracle.f32_to_bf16((rng.standard_normal((tokens, K)) * (0.05 if w_type == "e5m2" else 1.0)).astype(np.float32))
    gd, ud, xd = to_dev(torch, dev, Wg), to_dev(torch, dev, Wu), to_dev(torch, dev, X)
    keep = []
    if tiled:
        for wd in (gd, ud):
            t = torch.zeros(lib.tiled_size(wt, n_out, K), dtype=torch.uint8, device=dev)
            assert lib.weight_prepare(wd.data_ptr(), wt, n_out, K, K, t.data_ptr()) == 0
            keep.append(t)
    try:
        g, u, y3, y1 = (torch.zeros(tokens * n_out + 64, dtype=torch.int16, device=dev) for _ in range(4))
        assert lib.linear(gd.data_ptr(), wt, xd.data_ptr(), g.data_ptr(), n_out, tokens, K, sg) == 0
        assert lib.linear(ud.data_ptr(), wt, xd.data_ptr(), u.data_ptr(), n_out, tokens, K, su) == 0
        assert lib.c.hip_swiglu_bf16(ptr(g), ptr(u), ptr(y3), tokens * n_out) == (0 if (tokens * n_out) % 8 == 0 else -1)
        assert lib.c.hip_quant_gemm_swiglu(n_out, tokens, K, ptr(gd), ptr(ud), wt, K, ctypes.c_float(sg), ctypes.c_float(su),
                                           ptr(xd), K, ptr(y1), n_out) == 0
        assert lib.last_kernel() == ("gemm_swiglu_tiled" if tiled else "gemm_swiglu")
        got = from_dev(y1, np.uint16)
        assert not got[tokens * n_out:].any()
        if (tokens * n_out) % 8 == 0 and K < 1024:
            assert np.array_equal(got, from_dev(y3, np.uint16))
        elif (tokens * n_out) % 8 == 0:
            assert np.mean(got != from_dev(y3, np.uint16)) < 0.02
        gate = oracle.f32_to_bf16(oracle.linear_exact(oracle.dequant_fp8_to_bf16(Wg, wt, sg), X).astype(np.float32))
        up = oracle.f32_to_bf16(oracle.linear_exact(oracle.dequant_fp8_to_bf16(Wu, wt, su), X).astype(np.float32))
        want = dec.silu_mul(dec.f(gate), dec.f(up))
        have = dec.f(got[:tokens * n_out].reshape(tokens, n_out))
        assert np.linalg.norm(have - want) <= 1e-2 * np.linalg.norm(want)
        bad = lambda *a: lib.c.hip_quant_gemm_swiglu(*a)
        assert bad(n_out, 1, K, ptr(gd), ptr(ud), wt, K, ctypes.c_float(sg), ctypes.c_float(su), ptr(xd), K, ptr(y1), n_out) == -1
        assert bad(n_out, tokens, K, ptr(gd), ptr(ud), oracle.FP4, K, ctypes.c_float(sg), ctypes.c_float(su), ptr(xd), K, ptr(y1), n_out) == -1
        assert bad(n_out, tokens, K - 32, ptr(gd), ptr(ud), wt, K, ctypes.c_float(sg), ctypes.c_float(su), ptr(xd), K, ptr(y1), n_out) == -1
    finally:
        if tiled:
            assert lib.weight_release(gd.data_ptr()) == 0 and lib.weight_release(ud.data_ptr()) == 0


@pytest.mark.parametrize("block", [16, 32])
@pytest.mark.parametrize("tokens,n_out,K", [(60, 512, 256), (130, 200, 1024), (300, 1536, 512), (5, 256, 1024)])
def test_fp4_gate_up_pair_gemm_with_swiglu(gpu, oracle, dec, block, tokens, n_out, K):
    """hip_quant_gemm_swiglu on FP4 block-scale weights (tiled copies registered) against two hip_quant_gemm calls and
    hip_swiglu_bf16 -- byte for byte where K is too short for a k split (under 1024) -- and against the oracle's exact
    contraction; without the tiled copies the call is refused."""
    torch, dev, lib = gpu
    rng = np.random.default_rng(tokens + n_out + K + block)
    X = oracle.f32_to_bf16(rng.standard_normal((tokens, K)).astype(np.float32))
    xd = to_dev(torch, dev, X)
    Wg, Wu = (rng.integers(0, 256, size=(n_out, K // 2), dtype=np.uint8) for _ in range(2))
    Sg, Su = (rng.integers(0x20, 0x40, size=(n_out, K // block), dtype=np.uint8) for _ in range(2))
    gd, ud, sgd, sud = (to_dev(torch, dev, v) for v in (Wg, Wu, Sg, Su))
    g, u, y3, y1 = (torch.zeros(tokens * n_out + 64, dtype=torch.int16, device=dev) for _ in range(4))
    call = lambda: lib.c.hip_quant_gemm_swiglu(n_out, tokens, K, ptr(gd), ptr(ud), oracle.FP4, K, ctypes.c_float(1.0), ctypes.c_float(1.0),
                                               ptr(xd), K, ptr(y1), n_out)
    assert call() == -1                                         # no tiled copies yet
    keep = []
    for wd, sd in ((gd, sgd), (ud, sud)):
        t = torch.zeros(lib.tiled_size(oracle.FP4, n_out, K), dtype=torch.uint8, device=dev)
        assert lib.weight_prepare_fp4(wd.data_ptr(), sd.data_ptr(), block, n_out, K, t.data_ptr()) == 0
        keep.append(t)
    try:
        assert lib.linear(gd.data_ptr(), oracle.FP4, xd.data_ptr(), g.data_ptr(), n_out, tokens, K, 1.0, sgd.data_ptr(), block) == 0
        assert lib.linear(ud.data_ptr(), oracle.FP4, xd.data_ptr(), u.data_ptr(), n_out, tokens, K, 1.0, sud.data_ptr(), block) == 0
        assert lib.c.hip_swiglu_bf16(ptr(g), ptr(u), ptr(y3), tokens * n_out) == 0
        assert call() == 0
        assert lib.last_kernel() == "gemm_swiglu_tiled"
        got = from_dev(y1, np.uint16)
        assert got[:tokens * n_out].any() and not got[tokens * n_out:].any()
        if K < 1024:
            assert np.array_equal(got, from_dev(y3, np.uint16))
        else:
            assert np.mean(got != from_dev(y3, np.uint16)) < 0.02
        deq = lambda W, S: oracle.dequant_weight(W.reshape(-1), oracle.FP4, n_out, K, blk_sc=S.reshape(-1), block=block)
        gate = oracle.f32_to_bf16(oracle.linear_exact(deq(Wg, Sg), X).astype(np.float32))
        up = oracle.f32_to_bf16(oracle.linear_exact(deq(Wu, Su), X).astype(np.float32))
        want = dec.silu_mul(dec.f(gate), dec.f(up))
        have = dec.f(got[:tokens * n_out].reshape(tokens, n_out))
        assert np.linalg.norm(have - want) <= 1e-2 * np.linalg.norm(want)
    finally:
        assert lib.weight_release(gd.data_ptr()) == 0 and lib.weight_release(ud.data_ptr()) == 0


@pytest.mark.parametrize("w_type,tiled", [("e5m2", False), ("e4m3", True), ("fp4", True)])
@pytest.mark.parametrize("tokens,n_out,K", [(20, 256, 1024), (60, 4096, 2048), (130, 1000, 4096), (300, 512, 8192), (6, 1024, 2048)])
def test_linear_residual_add_and_norm_in_the_combine_launch(gpu, oracle, w_type, tiled, tokens, n_out, K):
    """hip_quant_gemm_add_rms_norm on shapes whose GEMM splits its k range against hip_quant_gemm, hip_add_bf16 and
    hip_rms_norm_fwd on the same inputs: both outputs byte for byte (from 17 tokens on, where the separate GEMM is the same
    kernel; below that it is a matrix-vector kernel with another order of the FP32 sums, and a few sums land on the other
    side of a BF16 rounding boundary), nothing written past them; a shape that does not split and unsupported arguments
    return -1 and write nothing."""
    torch, dev, lib = gpu
    rng = np.random.default_rng(tokens + n_out + K)
    X = oracle.f32_to_bf16((rng.standard_normal((tokens, K)) * (0.05 if w_type == "e5m2" else 1.0)).astype(np.float32))
    R = oracle.f32_to_bf16(rng.standard_normal((tokens, n_out)).astype(np.float32))
    Wn = oracle.f32_to_bf16((1.0 + 0.1 * rng.standard_normal(n_out)).astype(np.float32))
    xd, rd, nd = to_dev(torch, dev, X), to_dev(torch, dev, R), to_dev(torch, dev, Wn)
    sd, block, sc = None, 16, 1.0
    if w_type == "fp4":
        wt = oracle.FP4
        wd = to_dev(torch, dev, rng.integers(0, 256, size=(n_out, K // 2), dtype=np.uint8))
        sd = to_dev(torch, dev, rng.integers(0x20, 0x40, size=(n_out, K // block), dtype=np.uint8))
    else:
        wt = oracle.E5M2 if w_type == "e5m2" else oracle.E4M3
        sc = 1.0 if w_type == "e5m2" else 0.013
        W = rng.integers(0, 256, size=(n_out, K), dtype=np.uint8)
        if w_type == "e5m2": W[(W & 0x7C) == 0x7C] = 0x3C
        else: W[(W & 0x7F) == 0x7F] = 0x38
        wd = to_dev(torch, dev, W)
    keep = None
    if tiled:
        keep = torch.zeros(lib.tiled_size(wt, n_out, K), dtype=torch.uint8, device=dev)
        if w_type == "fp4": assert lib.weight_prepare_fp4(wd.data_ptr(), sd.data_ptr(), block, n_out, K, keep.data_ptr()) == 0
        else: assert lib.weight_prepare(wd.data_ptr(), wt, n_out, K, K, keep.data_ptr()) == 0
    try:
        o, s3, y3, s1, y1 = (torch.zeros(tokens * n_out + 64, dtype=torch.int16, device=dev) for _ in range(5))
        if w_type == "fp4": assert lib.linear(wd.data_ptr(), wt, xd.data_ptr(), o.data_ptr(), n_out, tokens, K, 1.0, sd.data_ptr(), block) == 0
        else: assert lib.linear(wd.data_ptr(), wt, xd.data_ptr(), o.data_ptr(), n_out, tokens, K, sc) == 0
        assert lib.c.hip_add_bf16(ptr(rd), ptr(o), ptr(s3), tokens * n_out) == 0
        assert lib.c.hip_rms_norm_fwd(oracle.BF16, ptr(s3), ptr(y3), ptr(nd), None, tokens, n_out, ctypes.c_float(1e-6)) == 0
        call = lambda toks, n, k: lib.c.hip_quant_gemm_add_rms_norm(n, toks, k, ptr(wd), wt, K, ctypes.c_float(sc), ptr(xd), K,
                                                                    ptr(rd), ptr(s1), ptr(nd), ptr(y1), ctypes.c_float(1e-6))
        assert call(tokens, n_out, K) == 0
        assert lib.last_kernel() == ("gemm_add_rms_norm_tiled" if tiled else "gemm_add_rms_norm")
        got_s, got_y = from_dev(s1, np.uint16), from_dev(y1, np.uint16)
        assert got_y[:tokens * n_out].any() and not got_y[tokens * n_out:].any() and not got_s[tokens * n_out:].any()
        if tokens >= 17:
            assert np.array_equal(got_s, from_dev(s3, np.uint16))
            assert np.array_equal(got_y, from_dev(y3, np.uint16))
        else:
            assert np.mean(got_s != from_dev(s3, np.uint16)) < 0.02
            a, b = (oracle.bf16_to_f32(v[:tokens * n_out].reshape(tokens, n_out)).astype(np.float64) for v in (got_y, from_dev(y3, np.uint16)))
            assert (np.linalg.norm(a - b, axis=1) <= 2e-3 * np.linalg.norm(b, axis=1)).all()
        s1.zero_(); y1.zero_()
        assert call(1, n_out, K) == -1 and call(tokens, n_out - 4, K) == -1 and call(tokens, n_out, K - 32) == -1
        assert not from_dev(s1, np.uint16).any() and not from_dev(y1, np.uint16).any()
    finally:
        if tiled:
            assert lib.weight_release(wd.data_ptr()) == 0


def test_linear_add_norm_refuses_a_shape_that_does_not_split(gpu, oracle):
    """2048 tokens x 4096 features fill the GPU without a k split: hip_quant_gemm_add_rms_norm returns -1 and launches nothing."""
    torch, dev, lib = gpu
    tokens, n_out, K = 2048, 4096, 256
    w = torch.zeros(n_out * K, dtype=torch.uint8, device=dev)
    x = torch.zeros(tokens * K, dtype=torch.int16, device=dev)
    r, s, y = (torch.zeros(tokens * n_out, dtype=torch.int16, device=dev) for _ in range(3))
    nw = torch.zeros(n_out, dtype=torch.int16, device=dev)
    assert lib.c.hip_quant_gemm_add_rms_norm(n_out, tokens, K, ptr(w), oracle.E5M2, K, ctypes.c_float(1.0), ptr(x), K,
                                             ptr(r), ptr(s), ptr(nw), ptr(y), ctypes.c_float(1e-6)) == -1


@pytest.mark.parametrize("rows,inner", [(1, 256), (7, 4096), (130, 1024), (5, 136)])
def test_add_and_rms_norm_in_one_pass_equals_the_two_calls(gpu, oracle, dec, rows, inner):
    """hip_add_rms_norm_bf16 against hip_add_bf16 followed by hip_rms_norm_fwd on the same inputs: both outputs byte for
    byte; rows that do not fit the kernel (longer than 4096, not a multiple of 8) are refused."""
    torch, dev, lib = gpu
    rng = np.random.default_rng(rows + inner)
    a = oracle.f32_to_bf16(rng.standard_normal((rows, inner)).astype(np.float32))
    b = oracle.f32_to_bf16((rng.standard_normal((rows, inner)) * 3).astype(np.float32))
    w = oracle.f32_to_bf16((1.0 + 0.1 * rng.standard_normal(inner)).astype(np.float32))
    ad, bd, wd = to_dev(torch, dev, a), to_dev(torch, dev, b), to_dev(torch, dev, w)
    s1, y1, s2, y2 = (torch.zeros(rows * inner + 64, dtype=torch.int16, device=dev) for _ in range(4))
    assert lib.c.hip_add_bf16(ptr(ad), ptr(bd), ptr(s1), rows * inner) == 0
    assert lib.c.hip_rms_norm_fwd(oracle.BF16, ptr(s1), ptr(y1), ptr(wd), None, rows, inner, ctypes.c_float(1e-6)) == 0
    assert lib.c.hip_add_rms_norm_bf16(ptr(ad), ptr(bd), ptr(s2), ptr(wd), ptr(y2), rows, inner, ctypes.c_float(1e-6)) == 0
    assert np.array_equal(from_dev(s1, np.uint16), from_dev(s2, np.uint16))
    assert np.array_equal(from_dev(y1, np.uint16), from_dev(y2, np.uint16))
    assert from_dev(y2, np.uint16)[:rows * inner].any() and not from_dev(y2, np.uint16)[rows * inner:].any()
    assert lib.c.hip_add_rms_norm_bf16(ptr(ad), ptr(bd), ptr(s2), ptr(wd), ptr(y2), 1, 4104, ctypes.c_float(1e-6)) == -1
    assert lib.c.hip_add_rms_norm_bf16(ptr(ad), ptr(bd), ptr(s2), ptr(wd), ptr(y2), 1, 100, ctypes.c_float(1e-6)) == -1


def test_residual_add_and_swiglu_rows(gpu, oracle, dec):
    torch, dev, lib = gpu
    rng = np.random.default_rng(9)
    n = 8 * 4099
    a = oracle.f32_to_bf16((3 * rng.standard_normal(n)).astype(np.float32))
    b = oracle.f32_to_bf16((3 * rng.standard_normal(n)).astype(np.float32))
    a[:4] = (0x7F80, 0xFF80, 0x0000, 0x8000)                    # +-inf and zeros ride along
    ad, bd = to_dev(torch, dev, a), to_dev(torch, dev, b)
    y = torch.zeros(n, dtype=torch.int16, device=dev)
    assert lib.c.hip_add_bf16(ptr(ad), ptr(bd), ptr(y), n) == 0
    with np.errstate(invalid="ignore"):
        want = oracle.f32_to_bf16(dec.f(a) + dec.f(b))
    assert np.array_equal(from_dev(y, np.uint16), want)
    assert lib.c.hip_swiglu_bf16(ptr(ad), ptr(bd), ptr(y), n) == 0
    got = from_dev(y, np.uint16)
    want = dec.silu_mul(dec.f(a[4:]), dec.f(b[4:]))
    # expf on the device and in numpy may differ in the last bit: one BF16 ulp at the two roundings behind it
    assert ulp_close(got[4:], want, ulps=3.0, floor=1e-30).all()
    assert (got[4:] == oracle.f32_to_bf16(want)).mean() > 0.99
    assert lib.c.hip_add_bf16(ptr(ad), ptr(bd), ptr(y), n - 1) == -1


# ------------------------------------------------------------------------------------------ the whole prompt phase

def _fresh(pkg, host, cfg):
    return pkg.host_api.DecodeModel(host, cfg.layers, cfg.hidden, cfg.n_q, cfg.n_kv, cfg.head_dim, cfg.inter, cfg.vocab, cfg.t_kv, theta=cfg.theta)


@pytest.mark.parametrize("variant", ["qwen3 fp8", "llama fp4", "tied fp8", "qwen3 fp8 tiled", "llama fp4 tiled"])
@pytest.mark.parametrize("T", [1, 5, 20, 60])
def test_prompt_phase_of_the_decode_model_follows_the_oracle(gpu, pkg, oracle, dec, variant, T):
    """DecodeModel::prefill (linears through the GEMM face with T columns, row kernels between them) against the oracle
    fed the same prompt token by token: the cache rows of every layer and position, the logits after the last token and
    the greedy pick; then three decode steps carry on from the prompt and still follow the oracle.  "tiled": every linear
    keeps its load-time tiled copy, which the GEMMs and GEMVs of the prompt phase then read."""
    host = pkg.host_api.host()
    host.init(0)
    fp4, tied, tiled = variant.startswith("llama fp4"), variant == "tied fp8", variant.endswith("tiled")
    cfg = dec.DecodeConfig(layers=2, hidden=256, n_q=4, n_kv=2, inter=512, vocab=1000, t_kv=96, theta=5e5 if fp4 else 1e6)
    weights = dec.make_model(cfg, 53, fmt="fp4_e2m1" if fp4 else "fp8_e5m2", qk_norm=not fp4, tied=tied)
    model = _fresh(pkg, host, cfg)
    model.set_repack_linears(tiled)
    model.load(weights)
    assert model.prepare_tiled(1, "w_up") == tiled
    model.set_exact_attention(True)
    rng = np.random.default_rng(T)
    prompt = [int(t) for t in rng.integers(0, cfg.vocab, size=T)]
    orc = dec.DecodeOracle(cfg, weights)
    for pos, tok in enumerate(prompt):
        want_logits, want_next = orc.step(tok, pos)
    got_next = model.prefill(prompt)
    assert model.pos == T
    for li in range(cfg.layers):
        for is_v, want_c in ((False, orc.k[li]), (True, orc.v[li])):
            got_c = dec.f(model.kv(li, is_v)[:, :T])
            assert np.isfinite(got_c).all()
            err = np.linalg.norm(got_c - want_c[:, :T]) / np.linalg.norm(want_c[:, :T])
            assert err <= (2e-3 if li == 0 else 1e-2), (li, is_v, err)
    got = dec.f(model.logits())
    assert np.linalg.norm(got - want_logits) <= 1e-2 * np.linalg.norm(want_logits)
    top2 = np.sort(want_logits)[-2:]
    if top2[1] - top2[0] > 2 * np.abs(got - want_logits).max():
        assert got_next == want_next
    token = want_next
    for pos in range(T, T + 3):
        model.reset(token, pos)
        got_token = model.step()
        want_logits, want_token = orc.step(token, pos)
        got = dec.f(model.logits())
        assert np.linalg.norm(got - want_logits) <= 1e-2 * np.linalg.norm(want_logits), pos
        token = want_token


def test_prompt_in_pieces_and_bad_arguments(gpu, pkg, oracle, dec):
    """A prompt fed in two calls (the second at pos0 = length of the first) leaves what one call leaves, up to the
    summation order of the linears (a piece of 7 tokens takes the GEMV kernels, one of 53 the GEMM); a prompt that does not fit
    the cache, an empty one and a token outside the vocabulary are refused."""
    host = pkg.host_api.host()
    host.init(0)
    cfg = dec.DecodeConfig(layers=2, hidden=256, n_q=4, n_kv=2, inter=512, vocab=1000, t_kv=64)
    weights = dec.make_model(cfg, 59)
    prompt = [int(t) for t in np.random.default_rng(5).integers(0, cfg.vocab, size=60)]
    a, b = _fresh(pkg, host, cfg), _fresh(pkg, host, cfg)
    b.set_repack_linears(True)                                 # the second model also reads its linears through their tiled copies
    a.load(weights); b.load(weights)
    assert b.prepare_tiled(0, "w_down") and not a.prepare_tiled(0, "w_down")      # only b's linears may carry the copy
    a.prefill(prompt)
    b.prefill(prompt[:7])
    b.prefill(prompt[7:], pos0=7)
    assert a.pos == b.pos == 60
    for li in range(cfg.layers):
        for is_v in (False, True):
            ca, cb = dec.f(a.kv(li, is_v)[:, :60]), dec.f(b.kv(li, is_v)[:, :60])
            assert np.linalg.norm(ca - cb) <= 1e-2 * np.linalg.norm(ca)
    la, lb = dec.f(a.logits()), dec.f(b.logits())
    assert np.linalg.norm(la - lb) <= 1e-2 * np.linalg.norm(la)
    with pytest.raises(RuntimeError):
        a.prefill(prompt + [1, 2, 3, 4, 5])                    # 65 positions in a cache of 64
    with pytest.raises(RuntimeError):
        a.prefill([])
    with pytest.raises(RuntimeError):
        a.prefill([3, cfg.vocab, 4])
    with pytest.raises(RuntimeError):
        a.prefill([1, 2], pos0=63)


def test_prompt_and_steps_on_a_non_blocking_stream(gpu, pkg, oracle, dec):
    """The prompt phase and the decode steps behind it with the library's launches on a stream created with
    hipStreamNonBlocking (which the null stream's blocking copies do not order with) and no device synchronisation after the
    launches: cache rows, logits and tokens equal those of the same model driven on the null stream.  A prompt in two pieces
    and a reset between steps go through the host copies (token ids, step state, last row) that must be ordered with the
    launches by the model itself."""
    torch, dev, lib = gpu
    host = pkg.host_api.host()
    host.init(0)
    cfg = dec.DecodeConfig(layers=2, hidden=256, n_q=4, n_kv=2, inter=512, vocab=1000, t_kv=96)
    weights = dec.make_model(cfg, 71)
    prompt = [int(t) for t in np.random.default_rng(9).integers(0, cfg.vocab, size=70)]

    def drive(model):
        model.load(weights)
        out = [model.prefill(prompt[:40]), model.prefill(prompt[40:], pos0=40)]
        for _ in range(3):
            out.append(model.step())
        model.reset(out[-1], model.pos)
        out.append(model.step())
        return out, model.logits().copy(), [model.kv(li, v).copy() for li in range(cfg.layers) for v in (False, True)]

    want = drive(_fresh(pkg, host, cfg))
    stream = torch.cuda.Stream(device=dev)                     # torch creates its streams non-blocking
    lib.set_sync(False)
    try:
        assert lib.set_stream(stream.cuda_stream) == 0
        assert lib.get_stream() == stream.cuda_stream
        got = drive(_fresh(pkg, host, cfg))
        stream.synchronize()
    finally:
        lib.set_stream(None)
        lib.set_sync(True)
    assert lib.get_stream() == 0
    assert got[0] == want[0]
    assert np.array_equal(got[1], want[1])
    for a, b in zip(got[2], want[2]):
        assert np.array_equal(a[:, :75], b[:, :75])
