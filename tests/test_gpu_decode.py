"""Decode-step neighbours and the fused step against the CPU oracle (oracle/decode_oracle.py),
through the C-ABI and the C++ DecodeModel."""
import ctypes

import numpy as np
import pytest

from gpu_util import from_dev, to_dev

pytestmark = pytest.mark.gpu

BF16, E4M3, E5M2 = 3, 4, 5


@pytest.fixture(scope="module")
def dec():
    from oracle import decode_oracle
    return decode_oracle


def ulp_close(got_bits, want_vals, ulps=1.0, floor=1e-6):
    got = (got_bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    want = np.asarray(want_vals, dtype=np.float64)
    tol = ulps * np.maximum(np.abs(want), 2.0 ** -120) * 2.0 ** -8 + floor
    return np.abs(got - want) <= tol


def test_rms_norm_and_rope_match_the_oracle(gpu, oracle, dec):
    torch, dev, lib = gpu
    rng = np.random.default_rng(0)
    for outer, inner in ((1, 4096), (40, 128), (3, 1000)):
        x = oracle.f32_to_bf16((rng.standard_normal((outer, inner)) * 3).astype(np.float32))
        w = oracle.f32_to_bf16((1 + 0.1 * rng.standard_normal(inner)).astype(np.float32))
        xd, wd = to_dev(torch, dev, x), to_dev(torch, dev, w)
        yd = torch.zeros(outer * inner, dtype=torch.int16, device=dev)
        inv = torch.zeros(outer, dtype=torch.float32, device=dev)
        assert lib.c.hip_rms_norm_fwd(BF16, ctypes.c_void_p(xd.data_ptr()), ctypes.c_void_p(yd.data_ptr()), ctypes.c_void_p(wd.data_ptr()),
                                      ctypes.c_void_p(inv.data_ptr()), outer, inner, ctypes.c_float(1e-6)) == 0
        want = dec.rms_norm(dec.f(x), dec.f(w), 1e-6)
        got = from_dev(yd, np.uint16).reshape(outer, inner)
        ok = ulp_close(got, want)
        assert ok.all()
        assert (got == oracle.f32_to_bf16(want)).mean() > 0.99          # bit-identical except rare rsqrt rounding flips
        ms = (dec.f(x).astype(np.float64) ** 2).mean(axis=1)
        assert np.allclose(inv.cpu().numpy(), 1 / np.sqrt(ms + 1e-6), rtol=1e-5)
    assert lib.c.hip_rms_norm_fwd(0, None, None, None, None, 1, 16, ctypes.c_float(1e-6)) == 1
    cfg = dec.DecodeConfig(t_kv=64)
    cos, sin = dec.rope_tables(cfg)
    x = oracle.f32_to_bf16(rng.standard_normal((6, 128)).astype(np.float32))
    xd, cd, sd = to_dev(torch, dev, x), to_dev(torch, dev, cos), to_dev(torch, dev, sin)
    for pos in (0, 1, 37, 63):
        yd = torch.zeros(6 * 128, dtype=torch.int16, device=dev)
        assert lib.c.hip_rope_fwd(BF16, ctypes.c_void_p(xd.data_ptr()), ctypes.c_void_p(yd.data_ptr()), ctypes.c_void_p(cd.data_ptr()),
                                  ctypes.c_void_p(sd.data_ptr()), 128, 1, 6, pos) == 0
        want = dec.rope(dec.f(x), dec.f(cos[pos]), dec.f(sin[pos]))
        assert ulp_close(from_dev(yd, np.uint16).reshape(6, 128), want).all(), pos
    assert lib.c.hip_rope_fwd(BF16, None, None, None, None, 127, 1, 1, 0) == 1


def fused_desc(pkg, **kw):
    lib = pkg.library()
    d = pkg.capi.FusedLinear()
    for k, v in kw.items():
        setattr(d, k, v)
    return d


class TiledCopies:
    """Registers load-time tiled copies for device weights (hip_quant_weight_prepare) and releases them."""

    def __init__(self, torch, dev, lib, weights, w_type, K):
        self.lib, self.keys, self.bufs = lib, [], []
        for w in weights:
            n_out = w.numel() // K
            t = torch.zeros(lib.tiled_size(w_type, n_out, K), dtype=torch.uint8, device=dev)
            assert lib.weight_prepare(w.data_ptr(), w_type, n_out, K, K, t.data_ptr()) == 0
            self.keys.append(w.data_ptr())
            self.bufs.append(t)

    def release(self):
        for k in self.keys:
            assert self.lib.weight_release(k) == 0


@pytest.mark.parametrize("tiled", [False, True])
def test_fused_linear_variants(gpu, pkg, oracle, dec, tiled):
    torch, dev, lib = gpu
    rng = np.random.default_rng(1)
    K, n0, n1, n2 = 2048, 512, 128, 130
    x = oracle.f32_to_bf16(rng.standard_normal(K).astype(np.float32))
    nw = oracle.f32_to_bf16((1 + 0.1 * rng.standard_normal(K)).astype(np.float32))
    Ws = [oracle.encode_e5m2_rne((rng.standard_normal((n, K)) * 0.02).astype(np.float32)) for n in (n0, n1, n2)]
    Wd = [oracle.dequant_fp8_to_bf16(W, oracle.E5M2).reshape(W.shape) for W in Ws]
    xd, nwd = to_dev(torch, dev, x), to_dev(torch, dev, nw)
    wds = [to_dev(torch, dev, W) for W in Ws]
    xn = dec.rms_norm(dec.f(x), dec.f(nw), 1e-6)

    Wu = oracle.encode_e5m2_rne((rng.standard_normal((n0, K)) * 0.02).astype(np.float32))
    wud = to_dev(torch, dev, Wu)
    copies = TiledCopies(torch, dev, lib, wds + [wud], E5M2, K) if tiled else None

    def run(desc, outs, pair=False):
        assert lib.quant_linear_fused(desc) == 0
        # these weights are not tall: tiled copies or not, they stay on the row-major kernel
        assert lib.last_kernel() == "gemv_fused"
        return [from_dev(o_, np.uint16) for o_ in outs]

    # (1) norm + three segments
    ys = [torch.zeros(n + 8, dtype=torch.int16, device=dev) for n in (n0, n1, n2)]
    d = pkg.capi.make_fused_linear(E5M2, K, [w.data_ptr() for w in wds], [n0, n1, n2], [y.data_ptr() for y in ys], xd.data_ptr(),
                                   norm_weight=nwd.data_ptr(), norm_eps=1e-6)
    outs = run(d, ys)
    for s, n in enumerate((n0, n1, n2)):
        assert not outs[s][n:].any()
        want = dec.linear(Wd[s], xn)
        assert ulp_close(outs[s][:n], want, ulps=1.0, floor=2e-5).all(), s
    # (2) plain single segment with residual and a per-tensor scale
    res = oracle.f32_to_bf16(rng.standard_normal(n0).astype(np.float32))
    rd = to_dev(torch, dev, res)
    y = torch.zeros(n0, dtype=torch.int16, device=dev)
    d = pkg.capi.make_fused_linear(E5M2, K, [wds[0].data_ptr()], [n0], [y.data_ptr()], xd.data_ptr(), scales=[0.5], residual=rd.data_ptr())
    out, = run(d, [y])
    lin = dec.linear(oracle.dequant_fp8_to_bf16(Ws[0], oracle.E5M2, 0.5).reshape(n0, K), dec.f(x))
    assert ulp_close(out, dec.r(lin + dec.f(res)), ulps=1.0, floor=2e-5).all()
    # (3) SwiGLU pair with norm: gate = W0, up = another n0-row weight
    y = torch.zeros(n0, dtype=torch.int16, device=dev)
    d = pkg.capi.make_fused_linear(E5M2, K, [wds[0].data_ptr(), wud.data_ptr()], [n0, n0], [y.data_ptr(), None], xd.data_ptr(),
                                   norm_weight=nwd.data_ptr(), norm_eps=1e-6, pair=True)
    out, = run(d, [y], pair=True)
    gate = dec.linear(Wd[0], xn)
    up = dec.linear(oracle.dequant_fp8_to_bf16(Wu, oracle.E5M2).reshape(n0, K), xn)
    want = dec.silu_mul(gate, up)
    # the product of two rounded factors moves by up to ~2 ulp when a factor flips by one
    assert ulp_close(out, want, ulps=3.0, floor=1e-4).all()
    assert (out == oracle.f32_to_bf16(want)).mean() > 0.97
    # rejected descriptors
    bad = pkg.capi.make_fused_linear(E5M2, 24, [wds[0].data_ptr()], [n0], [y.data_ptr()], xd.data_ptr())
    assert lib.quant_linear_fused(bad) == -1
    bad = pkg.capi.make_fused_linear(6, K, [wds[0].data_ptr()], [n0], [y.data_ptr()], xd.data_ptr())
    assert lib.quant_linear_fused(bad) == -1
    if copies:
        copies.release()


@pytest.mark.parametrize("K,n_out", [(1520, 37), (16400, 64), (8192, 33), (8208, 16), (272, 70000), (1040, 65550), (2064, 65600)])
@pytest.mark.parametrize("norm", [False, True])
@pytest.mark.parametrize("tiled", [False, True])
def test_fused_linear_ragged_lengths(gpu, pkg, oracle, dec, K, n_out, norm, tiled):
    """Row lengths that are not a multiple of 1 KiB, longer than the register-staged part of the
    activation, and odd row counts."""
    torch, dev, lib = gpu
    rng = np.random.default_rng(K + n_out)
    x = oracle.f32_to_bf16(rng.standard_normal(K).astype(np.float32))
    nw = oracle.f32_to_bf16((1 + 0.1 * rng.standard_normal(K)).astype(np.float32))
    W = oracle.encode_e5m2_rne((rng.standard_normal((n_out, K)) * 0.02).astype(np.float32))
    res = oracle.f32_to_bf16(rng.standard_normal(n_out).astype(np.float32))
    xd, nwd, wd, rd = (to_dev(torch, dev, v) for v in (x, nw, W, res))
    y = torch.zeros(n_out + 8, dtype=torch.int16, device=dev)
    d = pkg.capi.make_fused_linear(E5M2, K, [wd.data_ptr()], [n_out], [y.data_ptr()], xd.data_ptr(),
                                   norm_weight=nwd.data_ptr() if norm else None, norm_eps=1e-6, residual=rd.data_ptr())
    copies = TiledCopies(torch, dev, lib, [wd], E5M2, K) if tiled else None
    assert lib.quant_linear_fused(d) == 0
    assert lib.last_kernel() == ("gemv_fused_mfma" if tiled and n_out >= 65536 else "gemv_fused")      # tall weights only
    if copies:
        copies.release()
    out = from_dev(y, np.uint16)
    assert not out[n_out:].any()
    xin = dec.rms_norm(dec.f(x), dec.f(nw), 1e-6) if norm else dec.f(x)
    lin = dec.linear(oracle.dequant_fp8_to_bf16(W, oracle.E5M2).reshape(n_out, K), xin)
    # bf16(bf16(lin) + res): a one-ulp flip of lin (summation order) carries into the sum at lin's magnitude, not the sum's
    want = dec.r(lin + dec.f(res))
    got = dec.f(out[:n_out]).astype(np.float64)
    tol = np.maximum(np.maximum(np.abs(lin), np.abs(dec.f(res))), np.abs(want)) * 2.0 ** -7 + 1e-4      # one BF16 spacing of the largest term
    bad = np.abs(got - want) > tol
    assert not bad.any(), (int(bad.sum()), float((np.abs(got - want) / tol).max()), np.flatnonzero(bad)[:5], got[bad][:5], want[bad][:5], lin[bad][:5])
    assert (out[:n_out] == oracle.f32_to_bf16(want)).mean() > 0.98


@pytest.mark.parametrize("n_out,tiled", [(96, False), (66000, False), (66000, True)])
def test_fused_linear_e4m3_with_a_per_tensor_scale(gpu, pkg, oracle, dec, n_out, tiled):
    """FP8_E4M3 weights with scale_<name> (the hy-mt2 file layout) through both forms of the fused kernel."""
    torch, dev, lib = gpu
    rng = np.random.default_rng(n_out)
    K, scale = 1024, 0.0123
    x = oracle.f32_to_bf16(rng.standard_normal(K).astype(np.float32))
    nw = oracle.f32_to_bf16((1 + 0.1 * rng.standard_normal(K)).astype(np.float32))
    W = oracle.encode_e4m3_rne((rng.standard_normal((n_out, K)) * 0.02 / scale).astype(np.float32))
    xd, nwd, wd = (to_dev(torch, dev, v) for v in (x, nw, W))
    y = torch.zeros(n_out, dtype=torch.int16, device=dev)
    d = pkg.capi.make_fused_linear(E4M3, K, [wd.data_ptr()], [n_out], [y.data_ptr()], xd.data_ptr(), scales=[scale],
                                   norm_weight=nwd.data_ptr(), norm_eps=1e-6)
    copies = TiledCopies(torch, dev, lib, [wd], E4M3, K) if tiled else None
    assert lib.quant_linear_fused(d) == 0
    assert lib.last_kernel() == ("gemv_fused_mfma" if tiled else "gemv_fused")
    if copies:
        copies.release()
    want = dec.linear(oracle.dequant_fp8_to_bf16(W, oracle.E4M3, scale).reshape(n_out, K), dec.rms_norm(dec.f(x), dec.f(nw), 1e-6))
    got = dec.f(from_dev(y, np.uint16))
    assert np.linalg.norm(got - want) <= 2e-3 * np.linalg.norm(want)
    assert (np.abs(got - want) <= np.abs(want) * 2.0 ** -7 + 1e-4).all()


@pytest.mark.parametrize("n_q,n_kv,t_kv", [(4, 2, 200), (8, 2, 200), (2, 2, 200), (8, 2, 1024)])
def test_attention_decode_matches_the_oracle(gpu, oracle, dec, n_q, n_kv, t_kv):
    torch, dev, lib = gpu
    rng = np.random.default_rng(2)
    q = oracle.f32_to_bf16(rng.standard_normal((n_q, 128)).astype(np.float32))
    kc = oracle.f32_to_bf16(rng.standard_normal((n_kv, t_kv, 128)).astype(np.float32))
    vc = oracle.f32_to_bf16(rng.standard_normal((n_kv, t_kv, 128)).astype(np.float32))
    qd, kd, vd = to_dev(torch, dev, q), to_dev(torch, dev, kc), to_dev(torch, dev, vc)
    ws_bytes = lib.c.hip_attention_decode_workspace_bytes(n_q, n_kv, t_kv)
    assert ws_bytes >= n_q * t_kv * 2 and ws_bytes % 256 == 0
    ws = torch.full((ws_bytes,), 0x5A, dtype=torch.uint8, device=dev)       # content between calls must not matter
    positions = (0, 1, 63, 64, 127, 128, 130, 199) if t_kv == 200 else (511, 1000, 1023)
    for pos in positions:
        pd = torch.tensor([pos], dtype=torch.int32, device=dev)
        y = torch.zeros(n_q * 128, dtype=torch.int16, device=dev)
        rc = lib.c.hip_attention_decode_bf16(ctypes.c_void_p(qd.data_ptr()), ctypes.c_void_p(kd.data_ptr()), ctypes.c_void_p(vd.data_ptr()),
                                             ctypes.c_void_p(y.data_ptr()), ctypes.c_void_p(ws.data_ptr()), ws_bytes,
                                             n_q, n_kv, 128, t_kv, ctypes.c_void_p(pd.data_ptr()))
        assert rc == 0
        want = dec.attention(dec.f(q), dec.f(kc), dec.f(vc), pos, n_q, n_kv)
        got = from_dev(y, np.uint16).reshape(n_q, 128)
        assert ulp_close(got, want, ulps=2.0, floor=2e-3 * np.abs(want).max()).all(), pos
        # the BF16 scores themselves (launch 1, first n_q * t_kv BF16 values of the workspace) are the reference's rounding point
        s = ws[:n_q * t_kv * 2].cpu().numpy().view(np.uint16).reshape(n_q, t_kv)[:, :pos + 1]
        for h in range(n_q):
            exact = dec.f(kc)[h // (n_q // n_kv), :pos + 1].astype(np.float64) @ dec.f(q)[h].astype(np.float64)
            ref = dec.r(np.float32(1 / np.sqrt(np.float32(128))) * exact.astype(np.float32))
            assert ulp_close(s[h], ref, ulps=1.0, floor=1e-5).all()
    # too small a workspace and an unsupported head grouping are refused
    args = [ctypes.c_void_p(t.data_ptr()) for t in (qd, kd, vd, y, ws)]
    assert lib.c.hip_attention_decode_bf16(*args, ws_bytes - 256, n_q, n_kv, 128, t_kv, ctypes.c_void_p(pd.data_ptr())) == -1
    assert lib.c.hip_attention_decode_bf16(*args, ws_bytes, 3 * n_kv, n_kv, 128, t_kv, ctypes.c_void_p(pd.data_ptr())) == -1


@pytest.mark.parametrize("n_q,n_kv,t_kv", [(4, 2, 200), (8, 2, 300), (2, 2, 130), (4, 2, 6000)])
def test_fused_attention_appends_and_attends(gpu, oracle, dec, n_q, n_kv, t_kv):
    """q/k norm + RoPE + cache append + attention in two launches: cache rows as the oracle's, outputs
    within a few BF16 ulps (the probabilities are not rounded to BF16 on this path).  The 6000-row cache has
    94 blocks, more than the merge kernel requests up front, and its workspace starts out as NaN patterns."""
    torch, dev, lib = gpu
    rng = np.random.default_rng(5)
    cfg = dec.DecodeConfig(n_q=n_q, n_kv=n_kv, t_kv=t_kv)
    cos, sin = dec.rope_tables(cfg)
    qw = oracle.f32_to_bf16((1 + 0.1 * rng.standard_normal(128)).astype(np.float32))
    kw = oracle.f32_to_bf16((1 + 0.1 * rng.standard_normal(128)).astype(np.float32))
    kc = oracle.f32_to_bf16(rng.standard_normal((n_kv, t_kv, 128)).astype(np.float32))
    vc = oracle.f32_to_bf16(rng.standard_normal((n_kv, t_kv, 128)).astype(np.float32))
    kd, vd = to_dev(torch, dev, kc), to_dev(torch, dev, vc)
    # a second pair of caches whose rows were never written: NaN patterns everywhere; it is filled position by position below
    kn = torch.full((n_kv * t_kv * 128,), -1, dtype=torch.int16, device=dev)
    vn = torch.full((n_kv * t_kv * 128,), 0x7FC1, dtype=torch.int16, device=dev)
    ws_bytes = lib.c.hip_attention_decode_workspace_bytes(n_q, n_kv, t_kv)
    ws = torch.full((ws_bytes,), 0xFF if t_kv > 4096 else 0xA5, dtype=torch.uint8, device=dev)
    consts = [to_dev(torch, dev, a) for a in (qw, kw, cos, sin)]
    k_ref, v_ref = dec.f(kc).copy(), dec.f(vc).copy()
    for pos in ((0, 4095, 4096, 4160, t_kv - 1) if t_kv > 4096 else (0, 1, 127, 128, 129, t_kv - 1)):
        q = oracle.f32_to_bf16((2 * rng.standard_normal((n_q, 128))).astype(np.float32))
        k = oracle.f32_to_bf16((2 * rng.standard_normal((n_kv, 128))).astype(np.float32))
        v = oracle.f32_to_bf16(rng.standard_normal((n_kv, 128)).astype(np.float32))
        qd, knd, vnd = (to_dev(torch, dev, a) for a in (q, k, v))
        pd = torch.tensor([pos], dtype=torch.int32, device=dev)
        y = torch.zeros(n_q * 128, dtype=torch.int16, device=dev)
        ptr = lambda t: ctypes.c_void_p(t.data_ptr())
        rc = lib.c.hip_attention_decode_fused_bf16(ptr(qd), ptr(knd), ptr(vnd), ptr(consts[0]), ptr(consts[1]), ptr(consts[2]), ptr(consts[3]),
                                                   ptr(kd), ptr(vd), ptr(y), ptr(ws), ws_bytes, n_q, n_kv, 128, t_kv, ptr(pd), ctypes.c_float(1e-6))
        assert rc == 0
        qr = dec.rope(dec.rms_norm(dec.f(q), dec.f(qw), 1e-6), dec.f(cos[pos]), dec.f(sin[pos]))
        k_ref[:, pos] = dec.rope(dec.rms_norm(dec.f(k), dec.f(kw), 1e-6), dec.f(cos[pos]), dec.f(sin[pos]))
        v_ref[:, pos] = dec.f(v)
        got_k = from_dev(kd, np.uint16).reshape(n_kv, t_kv, 128)
        got_v = from_dev(vd, np.uint16).reshape(n_kv, t_kv, 128)
        assert ulp_close(got_k, k_ref, ulps=2.0, floor=1e-6).all()            # the new row within rsqrt rounding, every other row untouched
        assert np.array_equal(dec.f(got_v), v_ref)
        # attend over the cache as the GPU holds it, so that a one-ulp difference in the new key does not leak into this check
        want = dec.attention(qr, dec.f(got_k), dec.f(got_v), pos, n_q, n_kv)
        got = from_dev(y, np.uint16).reshape(n_q, 128)
        assert ulp_close(got, want, ulps=3.0, floor=4e-3 * np.abs(want).max()).all(), pos
        # two BF16 tensors rounded from slightly different exact values: about 1.6e-3 from the roundings alone
        assert np.linalg.norm(dec.f(got) - want) <= 4e-3 * np.linalg.norm(want)
        k_ref = dec.f(got_k).copy()
        if pos <= 2:
            # the same call on the never-written caches (positions 0, 1 in order): rows past the position must not leak into the output
            y2 = torch.zeros(n_q * 128, dtype=torch.int16, device=dev)
            rc = lib.c.hip_attention_decode_fused_bf16(ptr(qd), ptr(knd), ptr(vnd), ptr(consts[0]), ptr(consts[1]), ptr(consts[2]), ptr(consts[3]),
                                                       ptr(kn), ptr(vn), ptr(y2), ptr(ws), ws_bytes, n_q, n_kv, 128, t_kv, ptr(pd), ctypes.c_float(1e-6))
            assert rc == 0
            got2 = dec.f(from_dev(y2, np.uint16).reshape(n_q, 128))
            assert np.isfinite(got2).all()
            want2 = dec.attention(qr, dec.f(from_dev(kn, np.uint16).reshape(n_kv, t_kv, 128))[:, :pos + 1], dec.f(from_dev(vn, np.uint16).reshape(n_kv, t_kv, 128))[:, :pos + 1], pos, n_q, n_kv)
            assert ulp_close(from_dev(y2, np.uint16).reshape(n_q, 128), want2, ulps=3.0, floor=4e-3 * np.abs(want2).max()).all()


def test_argmax_and_embed(gpu, oracle):
    torch, dev, lib = gpu
    rng = np.random.default_rng(3)
    x = oracle.f32_to_bf16(rng.standard_normal(151936).astype(np.float32))
    x[[777, 90000]] = 0x4120                                   # two equal maxima (10.0): the lower index wins
    xd = to_dev(torch, dev, x)
    st = torch.tensor([0, 41], dtype=torch.int32, device=dev)
    aws = torch.zeros(lib.c.hip_argmax_workspace_bytes(151936), dtype=torch.uint8, device=dev)
    assert lib.c.hip_argmax_bf16(ctypes.c_void_p(xd.data_ptr()), 151936, ctypes.c_void_p(st.data_ptr()), ctypes.c_void_p(st.data_ptr() + 4),
                                 ctypes.c_void_p(aws.data_ptr())) == 0
    assert st.cpu().tolist() == [777, 42]
    for n, hot in ((1, 0), (2049, 2048), (5000, 4999)):                       # block boundaries, last element
        x2 = np.full(n, 0xBF80, dtype=np.uint16)
        x2[hot] = 0x3F80
        assert lib.c.hip_argmax_bf16(ctypes.c_void_p(to_dev(torch, dev, x2).data_ptr()), n, ctypes.c_void_p(st.data_ptr()), None,
                                     ctypes.c_void_p(aws.data_ptr())) == 0
        assert st.cpu().tolist() == [hot, 42]
    W = oracle.f32_to_bf16(rng.standard_normal((50, 256)).astype(np.float32))
    wd = to_dev(torch, dev, W)
    y = torch.zeros(256, dtype=torch.int16, device=dev)
    tok = torch.tensor([17], dtype=torch.int32, device=dev)
    assert lib.c.hip_embed_token_bf16(ctypes.c_void_p(tok.data_ptr()), ctypes.c_void_p(wd.data_ptr()), ctypes.c_void_p(y.data_ptr()), 256, 50) == 0
    assert np.array_equal(from_dev(y, np.uint16), W[17])
    ids = torch.tensor([3.0, 49.0], dtype=torch.float32, device=dev)
    y2 = torch.zeros(2 * 256, dtype=torch.int16, device=dev)
    assert lib.c.hip_embed_fwd(BF16, ctypes.c_void_p(ids.data_ptr()), ctypes.c_void_p(wd.data_ptr()), ctypes.c_void_p(y2.data_ptr()), 256, 2, 1) == 0
    assert np.array_equal(from_dev(y2, np.uint16).reshape(2, 256), W[[3, 49]])


@pytest.fixture(scope="module", params=["fused attention", "reference rounding points"])
def small_model(request, gpu, pkg, dec):
    host = pkg.host_api.host()
    host.init(0)
    cfg = dec.DecodeConfig(layers=2, hidden=256, n_q=4, n_kv=2, inter=512, vocab=1000, t_kv=64)
    weights = dec.make_model(cfg, 11)
    model = pkg.host_api.DecodeModel(host, cfg.layers, cfg.hidden, cfg.n_q, cfg.n_kv, cfg.head_dim, cfg.inter, cfg.vocab, cfg.t_kv)
    model.load(weights)
    model.set_exact_attention(request.param == "reference rounding points")
    return cfg, weights, model


def test_rope_tables_of_the_host_model(small_model, dec):
    cfg, _, model = small_model
    cos, _ = dec.rope_tables(cfg)
    assert np.array_equal(model.cos_table(), cos)


def test_decode_steps_follow_the_oracle(small_model, oracle, dec):
    cfg, weights, model = small_model
    orc = dec.DecodeOracle(cfg, weights)
    token = 5
    agree = 0
    for pos in range(12):
        model.reset(token, pos)
        got_token = model.step()
        assert model.pos == pos + 1
        want_logits, want_token = orc.step(token, pos)
        got = dec.f(model.logits())
        err = np.linalg.norm(got - want_logits) / np.linalg.norm(want_logits)
        assert err < 1e-2, (pos, err)
        assert np.abs(got - want_logits).max() <= 2e-2 * np.abs(want_logits).max()
        # the caches hold the rotated keys / raw values of this position
        # (layer 0 sees identical inputs: within rsqrt rounding; deeper layers inherit the BF16-level differences of the layers before)
        assert ulp_close(model.kv(0, False)[:, pos], orc.k[0, :, pos], ulps=2.0, floor=2e-3).all()
        assert ulp_close(model.kv(0, True)[:, pos], orc.v[0, :, pos], ulps=2.0, floor=2e-3).all()
        for li in range(cfg.layers):
            for got_c, want_c in ((dec.f(model.kv(li, False)[:, pos]), orc.k[li, :, pos]), (dec.f(model.kv(li, True)[:, pos]), orc.v[li, :, pos])):
                assert np.linalg.norm(got_c - want_c) <= 1e-2 * np.linalg.norm(want_c), (pos, li)
        # greedy token: identical unless the oracle's top two logits are within the error
        top2 = np.sort(want_logits)[-2:]
        if top2[1] - top2[0] > 2 * np.abs(got - want_logits).max():
            assert got_token == want_token, pos
            agree += 1
        token = want_token
    assert agree >= 8


def test_graph_replay_equals_eager_steps(small_model, dec):
    cfg, _, model = small_model
    model.reset(3, 0)
    eager = []
    for _ in range(10):
        eager.append(model.step())
    logits_eager = model.logits().copy()
    model.reset(3, 0)
    assert model.run(10, True) > 0                       # one captured step replayed ten times
    assert model.pos == 10
    assert model.token == eager[-1]
    assert np.array_equal(model.logits(), logits_eager)
    model.reset(3, 0)
    assert model.run(10, False) > 0
    assert model.token == eager[-1] and np.array_equal(model.logits(), logits_eager)


# ------------------------------------------------------------------------------------------ FP4 block-scale weights

@pytest.mark.parametrize("block", [16, 32])
def test_fused_linear_fp4_variants(gpu, pkg, oracle, dec, block):
    """hip_quant_linear_fused on FP4_E2M1 weights with E4M3 block scales: norm + three segments, single segment with
    residual and no norm, the SwiGLU pair, rows longer than one k-step and row counts that are odd."""
    from oracle import synth
    torch, dev, lib = gpu
    rng = np.random.default_rng(block)
    for K, (n0, n1, n2) in ((2048, (512, 128, 130)), (4608, (96, 33, 64)), (14336, (70, 16, 16))):
        x = oracle.f32_to_bf16(rng.standard_normal(K).astype(np.float32))
        nw = oracle.f32_to_bf16((1 + 0.1 * rng.standard_normal(K)).astype(np.float32))
        packed = [synth.weights_fp4(int(rng.integers(1 << 20)), n, K, block) for n in (n0, n1, n2, n0)]
        Wd = [oracle.dequant_weight(nib, oracle.FP4, nib.shape[0], K, blk_sc=sc, block=block) for nib, sc in packed]
        nd = [to_dev(torch, dev, nib) for nib, _ in packed]
        sd = [to_dev(torch, dev, sc) for _, sc in packed]
        xd, nwd = to_dev(torch, dev, x), to_dev(torch, dev, nw)
        xn = dec.rms_norm(dec.f(x), dec.f(nw), 1e-6)
        # (1) norm + three segments
        ys = [torch.zeros(n + 8, dtype=torch.int16, device=dev) for n in (n0, n1, n2)]
        d = pkg.capi.make_fused_linear(6, K, [w.data_ptr() for w in nd[:3]], [n0, n1, n2], [y.data_ptr() for y in ys], xd.data_ptr(),
                                       norm_weight=nwd.data_ptr(), norm_eps=1e-6, blk_sc=[s_.data_ptr() for s_ in sd[:3]], block_size=block)
        assert lib.quant_linear_fused(d) == 0 and lib.last_kernel() == "gemv_fused_fp4"
        for s_, n in enumerate((n0, n1, n2)):
            out = from_dev(ys[s_], np.uint16)
            assert not out[n:].any()
            assert ulp_close(out[:n], dec.linear(Wd[s_], xn), ulps=1.0, floor=2e-5).all(), (K, s_)
        # (2) one segment, no norm, residual
        res = oracle.f32_to_bf16(rng.standard_normal(n0).astype(np.float32))
        rd = to_dev(torch, dev, res)
        y = torch.zeros(n0, dtype=torch.int16, device=dev)
        d = pkg.capi.make_fused_linear(6, K, [nd[0].data_ptr()], [n0], [y.data_ptr()], xd.data_ptr(), residual=rd.data_ptr(),
                                       blk_sc=[sd[0].data_ptr()], block_size=block)
        assert lib.quant_linear_fused(d) == 0
        lin = dec.linear(Wd[0], dec.f(x))
        want = dec.r(lin + dec.f(res))
        tol = np.maximum(np.maximum(np.abs(lin), np.abs(dec.f(res))), np.abs(want)) * 2.0 ** -7 + 1e-4
        assert (np.abs(dec.f(from_dev(y, np.uint16)).astype(np.float64) - want) <= tol).all()
        # (3) SwiGLU pair behind the norm
        y = torch.zeros(n0, dtype=torch.int16, device=dev)
        d = pkg.capi.make_fused_linear(6, K, [nd[0].data_ptr(), nd[3].data_ptr()], [n0, n0], [y.data_ptr(), None], xd.data_ptr(),
                                       norm_weight=nwd.data_ptr(), norm_eps=1e-6, pair=True, blk_sc=[sd[0].data_ptr(), sd[3].data_ptr()], block_size=block)
        assert lib.quant_linear_fused(d) == 0
        want = dec.silu_mul(dec.linear(Wd[0], xn), dec.linear(Wd[3], xn))
        out = from_dev(y, np.uint16)
        assert ulp_close(out, want, ulps=3.0, floor=1e-4).all()
        assert (out == oracle.f32_to_bf16(want)).mean() > 0.97
    # refused: no block scales, a block length the kernels do not have, rows that are not whole 32-element loads
    d = pkg.capi.make_fused_linear(6, K, [nd[0].data_ptr()], [n0], [y.data_ptr()], xd.data_ptr(), block_size=block)
    assert lib.quant_linear_fused(d) == -1
    d = pkg.capi.make_fused_linear(6, K, [nd[0].data_ptr()], [n0], [y.data_ptr()], xd.data_ptr(), blk_sc=[sd[0].data_ptr()], block_size=8)
    assert lib.quant_linear_fused(d) == -1
    d = pkg.capi.make_fused_linear(6, 48, [nd[0].data_ptr()], [n0], [y.data_ptr()], xd.data_ptr(), blk_sc=[sd[0].data_ptr()], block_size=block)
    assert lib.quant_linear_fused(d) == -1


def test_decode_steps_with_fp4_linears_follow_the_oracle(gpu, pkg, oracle, dec):
    """The Llama-3.1-8B route of the reference (FP4_E2M1 block-scale linears, cccc/Net.cpp:1460-1481) through the
    fused decode step: eight steps of a two-layer model against the oracle on the same nibbles and scale bytes."""
    host = pkg.host_api.host()
    host.init(0)
    cfg = dec.DecodeConfig(layers=2, hidden=256, n_q=4, n_kv=2, inter=512, vocab=1000, t_kv=32)
    weights = dec.make_model(cfg, 17, fmt="fp4_e2m1")
    model = pkg.host_api.DecodeModel(host, cfg.layers, cfg.hidden, cfg.n_q, cfg.n_kv, cfg.head_dim, cfg.inter, cfg.vocab, cfg.t_kv)
    model.load(weights)
    model.set_exact_attention(True)
    orc = dec.DecodeOracle(cfg, weights)
    token = 9
    for pos in range(8):
        model.reset(token, pos)
        got_token = model.step()
        want_logits, want_token = orc.step(token, pos)
        got = dec.f(model.logits())
        assert np.linalg.norm(got - want_logits) <= 1e-2 * np.linalg.norm(want_logits), pos
        top2 = np.sort(want_logits)[-2:]
        if top2[1] - top2[0] > 2 * np.abs(got - want_logits).max():
            assert got_token == want_token, pos
        token = want_token
    # graph replay == eager on this path too
    model.reset(3, 0)
    eager = [model.step() for _ in range(6)]
    logits_eager = model.logits().copy()
    model.reset(3, 0)
    assert model.run(6, True) > 0 and model.token == eager[-1] and np.array_equal(model.logits(), logits_eager)


@pytest.mark.parametrize("n_q,n_kv,t_kv,normed", [(4, 2, 200, True), (8, 2, 300, True), (2, 2, 130, True), (8, 2, 300, False), (4, 2, 6000, True)])
def test_three_launch_attention_keeps_the_reference_rounding_points(gpu, oracle, dec, n_q, n_kv, t_kv, normed):
    """hip_attention_decode_exact_bf16: norm, rotation and append in the scores launch.  The appended rows are the
    oracle's, the BF16 scores it leaves in the workspace are the reference's rounding point (within one ulp of the exact
    product sum: the summation order is the matrix cores'), and the outputs agree with the four-launch route
    (hip_qk_norm_rope_kv_bf16 + hip_attention_decode_bf16) on the same inputs as closely as with the oracle."""
    torch, dev, lib = gpu
    rng = np.random.default_rng(41)
    cfg = dec.DecodeConfig(n_q=n_q, n_kv=n_kv, t_kv=t_kv)
    cos, sin = dec.rope_tables(cfg)
    qw = oracle.f32_to_bf16((1 + 0.1 * rng.standard_normal(128)).astype(np.float32))
    kw = oracle.f32_to_bf16((1 + 0.1 * rng.standard_normal(128)).astype(np.float32))
    kc = oracle.f32_to_bf16(rng.standard_normal((n_kv, t_kv, 128)).astype(np.float32))
    vc = oracle.f32_to_bf16(rng.standard_normal((n_kv, t_kv, 128)).astype(np.float32))
    ws_bytes = lib.c.hip_attention_decode_workspace_bytes(n_q, n_kv, t_kv)
    ws = torch.full((ws_bytes,), 0xFF, dtype=torch.uint8, device=dev)
    ws2 = torch.full((ws_bytes,), 0x5A, dtype=torch.uint8, device=dev)
    qwd, kwd, cd, sd = (to_dev(torch, dev, a) for a in (qw, kw, cos, sin))
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())
    nq_w, nk_w = (ptr(qwd), ptr(kwd)) if normed else (ctypes.c_void_p(0), ctypes.c_void_p(0))
    for pos in ((0, 4095, 4096, 4160, t_kv - 1) if t_kv > 4096 else (0, 1, 63, 64, 127, 128, t_kv - 1)):
        q = oracle.f32_to_bf16((2 * rng.standard_normal((n_q, 128))).astype(np.float32))
        k = oracle.f32_to_bf16((2 * rng.standard_normal((n_kv, 128))).astype(np.float32))
        v = oracle.f32_to_bf16(rng.standard_normal((n_kv, 128)).astype(np.float32))
        qd, knd, vnd = (to_dev(torch, dev, a) for a in (q, k, v))
        pd = torch.tensor([pos], dtype=torch.int32, device=dev)
        kd, vd = to_dev(torch, dev, kc), to_dev(torch, dev, vc)
        y = torch.zeros(n_q * 128, dtype=torch.int16, device=dev)
        assert lib.c.hip_attention_decode_exact_bf16(ptr(qd), ptr(knd), ptr(vnd), nq_w, nk_w, ptr(cd), ptr(sd), ptr(kd), ptr(vd), ptr(y), ptr(ws), ws_bytes,
                                                     n_q, n_kv, 128, t_kv, ptr(pd), ctypes.c_float(1e-6)) == 0
        # the four-launch route on copies of the same caches
        kd2, vd2 = to_dev(torch, dev, kc), to_dev(torch, dev, vc)
        q_rot = torch.zeros(n_q * 128, dtype=torch.int16, device=dev)
        y2 = torch.zeros(n_q * 128, dtype=torch.int16, device=dev)
        assert lib.c.hip_qk_norm_rope_kv_bf16(ptr(qd), ptr(knd), ptr(vnd), nq_w, nk_w, ptr(cd), ptr(sd), ptr(q_rot), ptr(kd2), ptr(vd2),
                                              n_q, n_kv, 128, t_kv, ptr(pd), ctypes.c_float(1e-6)) == 0
        assert lib.c.hip_attention_decode_bf16(ptr(q_rot), ptr(kd2), ptr(vd2), ptr(y2), ptr(ws2), ws_bytes, n_q, n_kv, 128, t_kv, ptr(pd)) == 0
        got_k = from_dev(kd, np.uint16).reshape(n_kv, t_kv, 128)
        # the appended rows: both routes run the same arithmetic on the same bytes
        assert np.array_equal(got_k, from_dev(kd2, np.uint16).reshape(n_kv, t_kv, 128)), pos
        assert np.array_equal(from_dev(vd, np.uint16), from_dev(vd2, np.uint16)), pos
        qr = dec.f(from_dev(q_rot, np.uint16).reshape(n_q, 128))
        # scores: BF16 of the exact sum, up to the last bit of an FP32 sum taken in another order
        s = ws[:n_q * t_kv * 2].cpu().numpy().view(np.uint16).reshape(n_q, t_kv)[:, :pos + 1]
        for h in range(n_q):
            exact = dec.f(got_k)[h // (n_q // n_kv), :pos + 1].astype(np.float64) @ qr[h].astype(np.float64)
            ref = dec.r(np.float32(1 / np.sqrt(np.float32(128))) * exact.astype(np.float32))
            # (ulp_close measures in units of |want| * 2^-8, i.e. half a BF16 ulp at the bottom of a binade: 2.0 = one rounding flip)
            assert ulp_close(s[h], ref, ulps=2.0, floor=1e-5).all(), (pos, h)
            assert (s[h] == oracle.f32_to_bf16(ref)).mean() > 0.99
        want = dec.attention(qr, dec.f(got_k), dec.f(from_dev(vd, np.uint16).reshape(n_kv, t_kv, 128)), pos, n_q, n_kv)
        got = from_dev(y, np.uint16).reshape(n_q, 128)
        assert ulp_close(got, want, ulps=2.0, floor=2e-3 * np.abs(want).max()).all(), pos
        assert ulp_close(got, dec.f(from_dev(y2, np.uint16).reshape(n_q, 128)), ulps=2.0, floor=2e-3 * np.abs(want).max()).all(), pos
    args = [ptr(qd), ptr(knd), ptr(vnd), nq_w, nk_w, ptr(cd), ptr(sd), ptr(kd), ptr(vd), ptr(y), ptr(ws)]
    assert lib.c.hip_attention_decode_exact_bf16(*args, ws_bytes - 256, n_q, n_kv, 128, t_kv, ptr(pd), ctypes.c_float(1e-6)) == -1
    assert lib.c.hip_attention_decode_exact_bf16(*args, ws_bytes, 3 * n_kv, n_kv, 128, t_kv, ptr(pd), ctypes.c_float(1e-6)) == -1


@pytest.mark.parametrize("n_q,n_kv,t_kv", [(4, 2, 200), (8, 2, 300)])
def test_attention_without_per_head_norms(gpu, oracle, dec, n_q, n_kv, t_kv):
    """Llama-style heads (has_qknorm = False, scripts/convert_weights.py:488-530): NULL norm weights make both attention
    routes rotate the raw projections.  The appended key row is then exactly rope(k) -- no rsqrt in its way -- and both
    routes follow the oracle; one NULL norm weight alone is refused."""
    torch, dev, lib = gpu
    rng = np.random.default_rng(31)
    cfg = dec.DecodeConfig(n_q=n_q, n_kv=n_kv, t_kv=t_kv, theta=5e5)
    cos, sin = dec.rope_tables(cfg)
    kc = oracle.f32_to_bf16(rng.standard_normal((n_kv, t_kv, 128)).astype(np.float32))
    vc = oracle.f32_to_bf16(rng.standard_normal((n_kv, t_kv, 128)).astype(np.float32))
    ws_bytes = lib.c.hip_attention_decode_workspace_bytes(n_q, n_kv, t_kv)
    ws = torch.full((ws_bytes,), 0xA5, dtype=torch.uint8, device=dev)
    cd, sd = to_dev(torch, dev, cos), to_dev(torch, dev, sin)
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())
    null = ctypes.c_void_p(0)
    for pos in (0, 63, 64, 130, t_kv - 1):
        q = oracle.f32_to_bf16((2 * rng.standard_normal((n_q, 128))).astype(np.float32))
        k = oracle.f32_to_bf16((2 * rng.standard_normal((n_kv, 128))).astype(np.float32))
        v = oracle.f32_to_bf16(rng.standard_normal((n_kv, 128)).astype(np.float32))
        qd, knd, vnd = (to_dev(torch, dev, a) for a in (q, k, v))
        pd = torch.tensor([pos], dtype=torch.int32, device=dev)
        qr = dec.rope(dec.f(q), dec.f(cos[pos]), dec.f(sin[pos]))
        k_ref, v_ref = dec.f(kc).copy(), dec.f(vc).copy()
        k_ref[:, pos] = dec.rope(dec.f(k), dec.f(cos[pos]), dec.f(sin[pos]))
        v_ref[:, pos] = dec.f(v)
        want = dec.attention(qr, k_ref, v_ref, pos, n_q, n_kv)
        # two-launch route
        kd, vd = to_dev(torch, dev, kc), to_dev(torch, dev, vc)
        y = torch.zeros(n_q * 128, dtype=torch.int16, device=dev)
        assert lib.c.hip_attention_decode_fused_bf16(ptr(qd), ptr(knd), ptr(vnd), null, null, ptr(cd), ptr(sd), ptr(kd), ptr(vd), ptr(y), ptr(ws), ws_bytes,
                                                     n_q, n_kv, 128, t_kv, ptr(pd), ctypes.c_float(1e-6)) == 0
        assert np.array_equal(dec.f(from_dev(kd, np.uint16).reshape(n_kv, t_kv, 128)), k_ref), pos
        assert np.array_equal(dec.f(from_dev(vd, np.uint16).reshape(n_kv, t_kv, 128)), v_ref), pos
        got = from_dev(y, np.uint16).reshape(n_q, 128)
        assert ulp_close(got, want, ulps=3.0, floor=4e-3 * np.abs(want).max()).all(), pos
        # the route with the reference's rounding points
        kd2, vd2 = to_dev(torch, dev, kc), to_dev(torch, dev, vc)
        q_rot = torch.zeros(n_q * 128, dtype=torch.int16, device=dev)
        y2 = torch.zeros(n_q * 128, dtype=torch.int16, device=dev)
        assert lib.c.hip_qk_norm_rope_kv_bf16(ptr(qd), ptr(knd), ptr(vnd), null, null, ptr(cd), ptr(sd), ptr(q_rot), ptr(kd2), ptr(vd2),
                                              n_q, n_kv, 128, t_kv, ptr(pd), ctypes.c_float(1e-6)) == 0
        assert np.array_equal(dec.f(from_dev(q_rot, np.uint16).reshape(n_q, 128)), qr), pos
        assert np.array_equal(dec.f(from_dev(kd2, np.uint16).reshape(n_kv, t_kv, 128)), k_ref), pos
        assert lib.c.hip_attention_decode_bf16(ptr(q_rot), ptr(kd2), ptr(vd2), ptr(y2), ptr(ws), ws_bytes, n_q, n_kv, 128, t_kv, ptr(pd)) == 0
        assert ulp_close(from_dev(y2, np.uint16).reshape(n_q, 128), want, ulps=2.0, floor=2e-3 * np.abs(want).max()).all(), pos
    # one norm weight without the other describes no model
    w1 = to_dev(torch, dev, oracle.f32_to_bf16(np.ones(128, dtype=np.float32)))
    assert lib.c.hip_attention_decode_fused_bf16(ptr(qd), ptr(knd), ptr(vnd), ptr(w1), null, ptr(cd), ptr(sd), ptr(kd), ptr(vd), ptr(y), ptr(ws), ws_bytes,
                                                 n_q, n_kv, 128, t_kv, ptr(pd), ctypes.c_float(1e-6)) == -1
    assert lib.c.hip_qk_norm_rope_kv_bf16(ptr(qd), ptr(knd), ptr(vnd), null, ptr(w1), ptr(cd), ptr(sd), ptr(q_rot), ptr(kd2), ptr(vd2),
                                          n_q, n_kv, 128, t_kv, ptr(pd), ctypes.c_float(1e-6)) == -1


@pytest.mark.parametrize("fmt,exact", [("fp4_e2m1", True), ("fp4_e2m1", False), ("fp8_e5m2", False)])
def test_decode_steps_of_a_model_without_qk_norm(gpu, pkg, oracle, dec, fmt, exact):
    """A Llama-3.1-shaped graph (no W_qnorm / W_knorm, RoPE theta 5e5; FP4 block-scale linears are the reference's Llama
    route, cccc/Net.cpp:1460-1481) through the fused decode step against the oracle, then graph replay == eager."""
    host = pkg.host_api.host()
    host.init(0)
    cfg = dec.DecodeConfig(layers=2, hidden=256, n_q=4, n_kv=2, inter=512, vocab=1000, t_kv=32, theta=5e5)
    weights = dec.make_model(cfg, 29, fmt=fmt, qk_norm=False)
    assert "q_norm" not in weights["layers"][0]
    model = pkg.host_api.DecodeModel(host, cfg.layers, cfg.hidden, cfg.n_q, cfg.n_kv, cfg.head_dim, cfg.inter, cfg.vocab, cfg.t_kv, theta=cfg.theta)
    model.load(weights)
    assert not model.qk_norm
    model.set_exact_attention(exact)
    orc = dec.DecodeOracle(cfg, weights)
    token = 9
    for pos in range(8):
        model.reset(token, pos)
        got_token = model.step()
        want_logits, want_token = orc.step(token, pos)
        got = dec.f(model.logits())
        assert np.linalg.norm(got - want_logits) <= 1e-2 * np.linalg.norm(want_logits), pos
        # layer 0 sees the oracle's inputs up to the GEMV's summation order: its rotated key row within BF16 rounding
        assert ulp_close(model.kv(0, False)[:, pos], orc.k[0, :, pos], ulps=2.0, floor=2e-3).all()
        top2 = np.sort(want_logits)[-2:]
        if top2[1] - top2[0] > 2 * np.abs(got - want_logits).max():
            assert got_token == want_token, pos
        token = want_token
    # graph replay == eager on this route too
    model.reset(3, 0)
    eager = [model.step() for _ in range(6)]
    logits_eager = model.logits().copy()
    model.reset(3, 0)
    assert model.run(6, True) > 0 and model.token == eager[-1] and np.array_equal(model.logits(), logits_eager)


@pytest.mark.parametrize("K,n_out", [(2048, 512), (1520, 37), (272, 70000), (4096, 1000)])
def test_fused_linear_on_an_unquantized_bf16_weight(gpu, pkg, oracle, dec, K, n_out):
    """w_type 3: a weight the reference leaves in BF16 (a tied lm_head is the embedding table, cccc/Net.cpp:1158-1190).
    Norm in front, plain, with a residual, the greedy candidates of a tall weight, and three segments; a one-hot
    activation returns the weight's own column bit for bit.  A per-tensor scale is refused."""
    torch, dev, lib = gpu
    rng = np.random.default_rng(K + n_out)
    x = oracle.f32_to_bf16(rng.standard_normal(K).astype(np.float32))
    nw = oracle.f32_to_bf16((1 + 0.1 * rng.standard_normal(K)).astype(np.float32))
    W = oracle.f32_to_bf16((rng.standard_normal((n_out, K)) * 0.05).astype(np.float32))
    xd, nwd, wd = to_dev(torch, dev, x), to_dev(torch, dev, nw), to_dev(torch, dev, W)
    xn = dec.rms_norm(dec.f(x), dec.f(nw), 1e-6)
    # norm in front + candidates
    ws_bytes = lib.c.hip_argmax_workspace_bytes(n_out)
    ws = torch.zeros(ws_bytes, dtype=torch.uint8, device=dev)
    y = torch.zeros(n_out + 8, dtype=torch.int16, device=dev)
    d = pkg.capi.make_fused_linear(BF16, K, [wd.data_ptr()], [n_out], [y.data_ptr()], xd.data_ptr(), norm_weight=nwd.data_ptr(), norm_eps=1e-6,
                                   argmax_workspace=ws.data_ptr())
    assert lib.quant_linear_fused(d) == 0 and lib.last_kernel() == "gemv_fused_bf16"
    out = from_dev(y, np.uint16)
    assert not out[n_out:].any()
    want = dec.linear(W, xn)
    assert ulp_close(out[:n_out], want, ulps=1.0, floor=2e-5).all()
    idx = torch.zeros(2, dtype=torch.int32, device=dev)
    assert lib.c.hip_argmax_pick_embed_bf16(ctypes.c_void_p(ws.data_ptr()), n_out, ctypes.c_void_p(idx.data_ptr()), None, None, None, 0, 0) == 0
    got = dec.f(out[:n_out])
    assert int(idx[0].item()) == int(np.flatnonzero(got == got.max())[0])
    # plain + residual
    res = oracle.f32_to_bf16(rng.standard_normal(n_out).astype(np.float32))
    rd = to_dev(torch, dev, res)
    y = torch.zeros(n_out, dtype=torch.int16, device=dev)
    d = pkg.capi.make_fused_linear(BF16, K, [wd.data_ptr()], [n_out], [y.data_ptr()], xd.data_ptr(), residual=rd.data_ptr())
    assert lib.quant_linear_fused(d) == 0
    assert ulp_close(from_dev(y, np.uint16), dec.r(dec.linear(W, dec.f(x)) + dec.f(res)), ulps=1.0, floor=2e-5).all()
    # one-hot activations: y = W[:, k] exactly
    for k in (0, 7, K // 2 + 3, K - 1):
        e = np.zeros(K, dtype=np.uint16)
        e[k] = 0x3F80
        ed = to_dev(torch, dev, e)
        y = torch.zeros(n_out, dtype=torch.int16, device=dev)
        d = pkg.capi.make_fused_linear(BF16, K, [wd.data_ptr()], [n_out], [y.data_ptr()], ed.data_ptr())
        assert lib.quant_linear_fused(d) == 0
        assert np.array_equal(from_dev(y, np.uint16), W[:, k]), k
    if n_out >= 96:
        # three segments of one weight's rows
        cuts = (0, n_out // 2, n_out // 2 + 33, n_out)
        ys = [torch.zeros(cuts[i + 1] - cuts[i], dtype=torch.int16, device=dev) for i in range(3)]
        d = pkg.capi.make_fused_linear(BF16, K, [wd.data_ptr() + cuts[i] * K * 2 for i in range(3)], [cuts[i + 1] - cuts[i] for i in range(3)],
                                       [t.data_ptr() for t in ys], xd.data_ptr(), norm_weight=nwd.data_ptr(), norm_eps=1e-6)
        # (segment starts are whole rows of K * 2 bytes: 16-byte aligned because K is a multiple of 16)
        assert lib.quant_linear_fused(d) == 0
        assert ulp_close(np.concatenate([from_dev(t, np.uint16) for t in ys]), want, ulps=1.0, floor=2e-5).all()
    bad = pkg.capi.make_fused_linear(BF16, K, [wd.data_ptr()], [n_out], [y.data_ptr()], xd.data_ptr(), scales=[0.5])
    assert lib.quant_linear_fused(bad) == -1


def test_decode_steps_with_tied_embeddings(gpu, pkg, oracle, dec):
    """tie_word_embeddings (Hy-MT2, small Qwen3 models): no separate head -- the logits are the BF16 embedding table times the
    normalised state, as in the reference, which never quantizes an EMBED table (cccc/Net.cpp:1158-1190)."""
    host = pkg.host_api.host()
    host.init(0)
    cfg = dec.DecodeConfig(layers=2, hidden=256, n_q=4, n_kv=2, inter=512, vocab=1000, t_kv=32)
    weights = dec.make_model(cfg, 43, tied=True)
    assert "lm_head" not in weights
    model = pkg.host_api.DecodeModel(host, cfg.layers, cfg.hidden, cfg.n_q, cfg.n_kv, cfg.head_dim, cfg.inter, cfg.vocab, cfg.t_kv)
    model.load(weights)
    assert model.tied_lm_head
    orc = dec.DecodeOracle(cfg, weights)
    token = 9
    for pos in range(8):
        model.reset(token, pos)
        got_token = model.step()
        want_logits, want_token = orc.step(token, pos)
        got = dec.f(model.logits())
        assert np.linalg.norm(got - want_logits) <= 1e-2 * np.linalg.norm(want_logits), pos
        top2 = np.sort(want_logits)[-2:]
        if top2[1] - top2[0] > 2 * np.abs(got - want_logits).max():
            assert got_token == want_token, pos
        token = want_token
    model.reset(3, 0)
    eager = [model.step() for _ in range(6)]
    logits_eager = model.logits().copy()
    model.reset(3, 0)
    assert model.run(6, True) > 0 and model.token == eager[-1] and np.array_equal(model.logits(), logits_eager)
    # an untied head of the same values quantized to FP8 answers differently: the tied route really reads the BF16 table
    untied = dict(weights)
    untied["lm_head"] = oracle.encode_e5m2_rne(dec.f(weights["emb"]))
    other = pkg.host_api.DecodeModel(host, cfg.layers, cfg.hidden, cfg.n_q, cfg.n_kv, cfg.head_dim, cfg.inter, cfg.vocab, cfg.t_kv)
    other.load(untied)
    assert not other.tied_lm_head
    other.reset(3, 0)
    model.reset(3, 0)
    other.step(); model.step()
    assert not np.array_equal(other.logits(), model.logits())


@pytest.mark.parametrize("n_out,K,fmt", [(300, 1024, "e5m2"), (5000, 2048, "e5m2"), (70000, 1024, "e5m2 tiled"), (151936, 256, "e5m2 tiled"),
                                         (4100, 2048, "fp4"), (66000, 512, "fp4")])
def test_greedy_pick_from_the_linear_epilogue(gpu, pkg, oracle, n_out, K, fmt):
    """hip_quant_linear_fused leaves the greedy candidates of its outputs, hip_argmax_pick_embed_bf16 picks among them,
    advances the position and copies the embedding row: the token is the lowest index of the largest stored logit."""
    from oracle import synth
    torch, dev, lib = gpu
    rng = np.random.default_rng(n_out)
    x = oracle.f32_to_bf16(rng.standard_normal(K).astype(np.float32))
    xd = to_dev(torch, dev, x)
    kw = {}
    if fmt == "fp4":
        nib, sc = synth.weights_fp4(n_out, n_out, K, 16)
        wd, sd = to_dev(torch, dev, nib), to_dev(torch, dev, sc)
        w_type, kw = 6, dict(blk_sc=[sd.data_ptr()], block_size=16)
    else:
        W = synth.weights_e5m2(n_out, n_out, K)
        W[n_out - 1] = W[3]                                        # two equal rows: equal logits, the lower index must win if they are the maximum
        wd, w_type = to_dev(torch, dev, W), E5M2
    copies = TiledCopies(torch, dev, lib, [wd], E5M2, K) if fmt.endswith("tiled") else None
    ws = torch.full((lib.c.hip_argmax_workspace_bytes(n_out),), 0xEE, dtype=torch.uint8, device=dev)
    y = torch.zeros(n_out, dtype=torch.int16, device=dev)
    D = 64
    emb = oracle.f32_to_bf16(rng.standard_normal((n_out, D)).astype(np.float32))
    ed = to_dev(torch, dev, emb)
    ey = torch.zeros(D, dtype=torch.int16, device=dev)
    st = torch.tensor([-1, 41], dtype=torch.int32, device=dev)
    d = pkg.capi.make_fused_linear(w_type, K, [wd.data_ptr()], [n_out], [y.data_ptr()], xd.data_ptr(), argmax_workspace=ws.data_ptr(), **kw)
    assert lib.quant_linear_fused(d) == 0
    assert lib.last_kernel() == {"e5m2": "gemv_fused", "e5m2 tiled": "gemv_fused_mfma", "fp4": "gemv_fused_fp4"}[fmt]
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())
    assert lib.c.hip_argmax_pick_embed_bf16(ptr(ws), n_out, ptr(st), ctypes.c_void_p(st.data_ptr() + 4), ptr(ed), ptr(ey), D, n_out) == 0
    if copies:
        copies.release()
    logits = oracle.bf16_to_f32(from_dev(y, np.uint16))
    want = int(np.argmax(logits))                                    # first occurrence of the maximum
    assert st.cpu().tolist() == [want, 42]
    assert np.array_equal(from_dev(ey, np.uint16), emb[want])
    # forced tie at the top: rows 3 and n_out - 1 of the logits made the largest by scaling x would need new weights; instead check
    # the tie rule on the stored values directly: equal maxima -> lowest index
    ties = np.flatnonzero(logits == logits.max())
    assert want == ties[0]
    # without an embedding table the launch only picks
    assert lib.c.hip_argmax_pick_embed_bf16(ptr(ws), n_out, ptr(st), None, None, None, 0, 0) == 0
    assert st.cpu().tolist() == [want, 42]
    # refused: a candidate list on a multi-segment or pair launch
    bad = pkg.capi.make_fused_linear(w_type, K, [wd.data_ptr(), wd.data_ptr()], [n_out, n_out], [y.data_ptr(), y.data_ptr()], xd.data_ptr(),
                                     argmax_workspace=ws.data_ptr(), **({} if fmt != "fp4" else dict(blk_sc=[sd.data_ptr(), sd.data_ptr()], block_size=16)))
    assert lib.quant_linear_fused(bad) == -1
