"""Parity at the benchmark's full sizes, on the kernels the benchmark launches: the tiled matrix-core
GEMV at the five Qwen3-8B shapes, the FP4 block-scale GEMV at the Llama-3.1-8B shapes, the fused decode
linears at their Qwen3-8B instantiations and a whole decode step at Qwen3-8B widths with a filled KV
cache.  Weights are drawn on the GPU (a full-size weight takes seconds to draw on the host); the oracle
sees the very bytes the kernels read, downloaded for the sampled rows."""
import ctypes

import numpy as np
from oracle import synth
import pytest

from gpu_util import check_bf16_close, check_rows, from_dev, to_dev

pytestmark = pytest.mark.gpu

BF16, E4M3, E5M2, FP4 = 3, 4, 5, 6
QWEN_SHAPES = [(4096, 4096), (4096, 1024), (4096, 12288), (12288, 4096), (4096, 151936)]      # (K, n_out)
LLAMA_SHAPES = [(4096, 14336), (14336, 4096), (4096, 128256)]


@pytest.fixture(scope="module")
def dec():
    from oracle import decode_oracle
    return decode_oracle


def bf16_f64(oracle, bits):
    return oracle.bf16_to_f32(bits).astype(np.float64)


def draw_e5m2(torch, dev, gen, n_out, K):
    """uint8 E5M2 codes [n_out, K] on the device: N(0, 0.02) -> BF16 -> FP8 (round to nearest)."""
    out = torch.empty(n_out, K, dtype=torch.uint8, device=dev)
    rows = max(1, (1 << 27) // K)
    for r0 in range(0, n_out, rows):
        r = min(rows, n_out - r0)
        out[r0:r0 + r] = (torch.randn(r, K, device=dev, generator=gen) * 0.02).to(torch.bfloat16).to(torch.float8_e5m2).view(torch.uint8)
    return out


def draw_bf16(torch, dev, gen, shape, mean=0.0, std=1.0):
    return (torch.randn(*shape, device=dev, generator=gen) * std + mean).to(torch.bfloat16).view(torch.int16)


def host_bits(t):
    return t.cpu().numpy().view(np.uint16)


# ------------------------------------------------------------------------------------------ FP8, tiled copy

@pytest.mark.parametrize("K,n_out", QWEN_SHAPES)
def test_tiled_gemv_at_the_qwen3_8b_shapes(gpu, pkg, oracle, K, n_out):
    """hip_quant_gemm with the load-time tiled copy registered, 1 / 4 / 16 tokens: sampled rows against the
    exact contraction, all-ones activations against the row sums of the decoded weight."""
    torch, dev, lib = gpu
    gen = torch.Generator(device=dev).manual_seed(K + n_out)
    wd = draw_e5m2(torch, dev, gen, n_out, K)
    td = torch.zeros(lib.tiled_size(E5M2, n_out, K), dtype=torch.uint8, device=dev)
    assert lib.weight_prepare(wd.data_ptr(), E5M2, n_out, K, K, td.data_ptr()) == 0
    try:
        rows = np.sort(np.random.default_rng(n_out).choice(n_out, size=257, replace=False))
        W_rows = wd[torch.from_numpy(rows).to(dev)].cpu().numpy()
        Wd_rows = oracle.dequant_fp8_to_bf16(W_rows, oracle.E5M2).reshape(W_rows.shape)
        for tokens in (1, 4, 16):
            X = synth.activations(n_out + tokens, tokens, K)
            xd = to_dev(torch, dev, X)
            yd = torch.zeros(tokens * n_out + 64, dtype=torch.int16, device=dev)
            assert lib.linear(wd.data_ptr(), E5M2, xd.data_ptr(), yd.data_ptr(), n_out, tokens, K) == 0
            small = tokens <= 2 and n_out * K < (8 << 20)               # one or two tokens on a few MiB stay on the pipelined dot2 kernel
            assert lib.last_kernel() == ("gemv_dot2" if small else "gemv_mfma_tiled")
            out = from_dev(yd, np.uint16)
            assert not out[tokens * n_out:].any(), "wrote past the end"
            y = out[:tokens * n_out].reshape(tokens, n_out)
            want = oracle.linear_exact(Wd_rows, X)
            check_rows(bf16_f64(oracle, y[:, rows]), want, f"tiled {n_out}x{K} M={tokens}")
            check_bf16_close(y[:, rows], want, "tiled", slack_ulp=1.0, abs_floor=2e-5)
        ones = np.full((1, K), 0x3F80, dtype=np.uint16)
        yd = torch.zeros(n_out, dtype=torch.int16, device=dev)
        assert lib.linear(wd.data_ptr(), E5M2, to_dev(torch, dev, ones).data_ptr(), yd.data_ptr(), n_out, 1, K) == 0
        sums = oracle.decode_table(oracle.E5M2).astype(np.float64)[W_rows].sum(axis=1)
        got = bf16_f64(oracle, from_dev(yd, np.uint16))[rows]
        assert np.all(np.abs(got - sums) <= 2.0 ** -8 * np.abs(sums) + 1e-5)
    finally:
        assert lib.weight_release(wd.data_ptr()) == 0


def draw_fp8_scaled(torch, dev, gen, n_out, K, w_type, inv_scale):
    """uint8 codes [n_out, K] of w / inv_scale for N(0, 0.02) weights w: what a weight quantized with the per-tensor scale
    inv_scale holds (cccc/Matrix.cpp:338-352), rounded to nearest."""
    f8 = torch.float8_e5m2 if w_type == E5M2 else torch.float8_e4m3fn
    out = torch.empty(n_out, K, dtype=torch.uint8, device=dev)
    rows = max(1, (1 << 27) // K)
    for r0 in range(0, n_out, rows):
        r = min(rows, n_out - r0)
        out[r0:r0 + r] = (torch.randn(r, K, device=dev, generator=gen) * (0.02 / inv_scale)).to(torch.bfloat16).to(f8).view(torch.uint8)
    return out


@pytest.mark.parametrize("w_type,inv_scale", [(E5M2, 0.2 / 57344.0), (E4M3, 0.2 / 448.0)])      # ten sigma of headroom: no Inf / NaN codes
@pytest.mark.parametrize("K,n_out", QWEN_SHAPES)
def test_scaled_weights_at_the_qwen3_8b_shapes(gpu, pkg, oracle, K, n_out, w_type, inv_scale):
    """The routes of the benchmark's `sweep_variants` and scaled prefill rows at full size: weights with a per-tensor
    dequantisation multiplier (every weight Matrix::quantizeWeights makes carries absmax / 57344 or / 448), E5M2 and E4M3,
    1 and 16 tokens on the tiled copy, and 512 tokens (the register-fed GEMM; the two MLP shapes only) -- the weight that
    enters a product is bf16(decode(code) * inv_scale), rounded once, as the oracle rounds it."""
    torch, dev, lib = gpu
    gen = torch.Generator(device=dev).manual_seed(K + n_out + w_type)
    wd = draw_fp8_scaled(torch, dev, gen, n_out, K, w_type, inv_scale)
    td = torch.zeros(lib.tiled_size(w_type, n_out, K), dtype=torch.uint8, device=dev)
    assert lib.weight_prepare(wd.data_ptr(), w_type, n_out, K, K, td.data_ptr()) == 0
    try:
        rows = np.sort(np.random.default_rng(n_out + w_type).choice(n_out, size=193, replace=False))
        W_rows = wd[torch.from_numpy(rows).to(dev)].cpu().numpy()
        Wd_rows = oracle.dequant_fp8_to_bf16(W_rows, oracle.E5M2 if w_type == E5M2 else oracle.E4M3, inv_scale).reshape(W_rows.shape)
        counts = (1, 16, 512) if (K, n_out) in ((4096, 12288), (12288, 4096)) else (1, 16)
        for tokens in counts:
            X = synth.activations(n_out + tokens + w_type, tokens, K)
            xd = to_dev(torch, dev, X)
            yd = torch.zeros(tokens * n_out + 64, dtype=torch.int16, device=dev)
            assert lib.linear(wd.data_ptr(), w_type, xd.data_ptr(), yd.data_ptr(), n_out, tokens, K, inv_scale=inv_scale) == 0
            small = tokens <= 2 and n_out * K < (8 << 20)
            assert lib.last_kernel() == ("gemm_mfma_tiled" if tokens > 16 else "gemv_dot2" if small else "gemv_mfma_tiled")
            out = from_dev(yd, np.uint16)
            assert not out[tokens * n_out:].any(), "wrote past the end"
            y = out[:tokens * n_out].reshape(tokens, n_out)
            want = oracle.linear_exact(Wd_rows, X)
            check_rows(bf16_f64(oracle, y[:, rows]), want, f"scaled type {w_type} {n_out}x{K} M={tokens}")
            check_bf16_close(y[:, rows], want, "scaled", slack_ulp=1.0, abs_floor=2e-5)
    finally:
        assert lib.weight_release(wd.data_ptr()) == 0


# ------------------------------------------------------------------------------------------ FP4

FP4_BOUNDS = (0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0)


def pack_fp4_on_device(torch, w, block):
    """The converter's packing (absmax / 6 -> E4M3 by round to nearest, codes from the unrounded 6 / absmax,
    boundaries to the lower code, low nibble = even element) on a float32 device tensor [n_out, K]; the
    test below checks it against the host packer on a slab before trusting it."""
    n_out, K = w.shape
    b = w.reshape(-1, block)
    amax = b.abs().amax(dim=1)
    live = amax > 1e-10
    one = torch.ones_like(amax)
    # float32 quotients as the host computes them: divided in float64 and rounded once (a float32 division on the
    # device need not be correctly rounded)
    scales = torch.where(live, (amax.double() / 6.0).float(), one)
    fwd = torch.where(live, (6.0 / amax.double()).float(), one)
    scaled = (b * fwd[:, None]).reshape(-1)
    bounds = torch.tensor(FP4_BOUNDS, dtype=torch.float32, device=w.device)
    code = torch.bucketize(scaled.abs(), bounds, right=False).to(torch.uint8) | ((scaled < 0).to(torch.uint8) << 3)
    nib = (code[0::2] | (code[1::2] << 4)).reshape(n_out, K // 2)
    sc = scales.to(torch.float8_e4m3fn).view(torch.uint8).reshape(n_out, K // block)
    return nib, sc


@pytest.mark.parametrize("block", [16, 32])
@pytest.mark.parametrize("K,n_out", LLAMA_SHAPES)
def test_fp4_gemv_at_the_llama_8b_shapes(gpu, pkg, oracle, K, n_out, block):
    torch, dev, lib = gpu
    gen = torch.Generator(device=dev).manual_seed(K + n_out + block)
    nib = torch.empty(n_out, K // 2, dtype=torch.uint8, device=dev)
    sc = torch.empty(n_out, K // block, dtype=torch.uint8, device=dev)
    slab = max(1, (1 << 26) // K)
    for r0 in range(0, n_out, slab):
        r = min(slab, n_out - r0)
        w = (torch.randn(r, K, device=dev, generator=gen) * 0.02).to(torch.bfloat16).to(torch.float32)
        nib[r0:r0 + r], sc[r0:r0 + r] = pack_fp4_on_device(torch, w, block)
        if r0 == 0:
            want_nib, want_sc = synth.pack_fp4_blockscale(w[:64].cpu().numpy(), block)
            bad_nib = int((nib[:64].cpu().numpy().ravel() != want_nib).sum())
            bad_sc = int((sc[:64].cpu().numpy().ravel() != want_sc).sum())
            assert bad_nib == 0 and bad_sc == 0, f"device packer differs from the host packer: {bad_nib} code bytes, {bad_sc} scale bytes"
    rows = np.sort(np.random.default_rng(n_out + block).choice(n_out, size=257, replace=False))
    ridx = torch.from_numpy(rows).to(dev)
    nib_rows, sc_rows = nib[ridx].cpu().numpy(), sc[ridx].cpu().numpy()
    Wd_rows = oracle.dequant_weight(nib_rows, oracle.FP4, len(rows), K, blk_sc=sc_rows, block=block)
    # first on the bytes as the file holds them (dot2 kernel), then with the load-time tiled copy registered
    # (matrix cores from three tokens on, and at one token for the long-row shape)
    td = torch.zeros(lib.tiled_size(FP4, n_out, K), dtype=torch.uint8, device=dev)
    for tiled in (False, True):
        if tiled:
            assert lib.weight_prepare_fp4(nib.data_ptr(), sc.data_ptr(), block, n_out, K, td.data_ptr()) == 0
        try:
            for tokens in (1, 4, 16):
                X = synth.activations(n_out + tokens, tokens, K)
                xd = to_dev(torch, dev, X)
                yd = torch.zeros(tokens * n_out + 64, dtype=torch.int16, device=dev)
                assert lib.linear(nib.data_ptr(), FP4, xd.data_ptr(), yd.data_ptr(), n_out, tokens, K, blk_sc=sc.data_ptr(), block_size=block) == 0
                kernel = lib.last_kernel()
                on_cores = tiled and (tokens >= 3 or K > 8192)
                assert kernel == ("gemv_mfma_tiled" if on_cores else "gemv_dot2")
                out = from_dev(yd, np.uint16)
                assert not out[tokens * n_out:].any(), "wrote past the end"
                y = out[:tokens * n_out].reshape(tokens, n_out)
                want = oracle.linear_exact(Wd_rows, X)
                check_rows(bf16_f64(oracle, y[:, rows]), want, f"{kernel} fp4 {n_out}x{K} M={tokens} block {block}")
                check_bf16_close(y[:, rows], want, kernel, slack_ulp=1.0, abs_floor=2e-5)
        finally:
            if tiled:
                assert lib.weight_release(nib.data_ptr()) == 0
    ones = np.full((1, K), 0x3F80, dtype=np.uint16)
    yd = torch.zeros(n_out, dtype=torch.int16, device=dev)
    assert lib.linear(nib.data_ptr(), FP4, to_dev(torch, dev, ones).data_ptr(), yd.data_ptr(), n_out, 1, K, blk_sc=sc.data_ptr(), block_size=block) == 0
    sums = bf16_f64(oracle, Wd_rows).sum(axis=1)
    got = bf16_f64(oracle, from_dev(yd, np.uint16))[rows]
    assert np.all(np.abs(got - sums) <= 2.0 ** -8 * np.abs(sums) + 1e-5)


# ------------------------------------------------------------------------------------------ fused decode linears

def ulp_close(got_bits, want_vals, ulps=1.0, floor=1e-6):
    got = (got_bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    want = np.asarray(want_vals, dtype=np.float64)
    return np.abs(got - want) <= ulps * np.maximum(np.abs(want), 2.0 ** -120) * 2.0 ** -8 + floor


@pytest.mark.parametrize("case", ["o", "down", "qkv", "gate_up", "lm_head"])
def test_fused_linears_at_their_qwen3_8b_instantiations(gpu, pkg, oracle, dec, case):
    """hip_quant_linear_fused with the arguments DecodeModel::step passes at Qwen3-8B widths: unscaled
    E5M2 weights, o and down without a norm (activation requested with the weights) and with the residual,
    q/k/v as three segments behind an RMSNorm, the SwiGLU pair behind an RMSNorm, lm_head behind the final
    norm on its tiled copy."""
    torch, dev, lib = gpu
    gen = torch.Generator(device=dev).manual_seed(len(case) * 7919)
    K = {"o": 4096, "down": 12288, "qkv": 4096, "gate_up": 4096, "lm_head": 4096}[case]
    n_outs = {"o": [4096], "down": [4096], "qkv": [4096, 1024, 1024], "gate_up": [12288, 12288], "lm_head": [151936]}[case]
    norm = case in ("qkv", "gate_up", "lm_head")
    wds = [draw_e5m2(torch, dev, gen, n, K) for n in n_outs]
    x_std = 0.3 if case == "down" else 1.0
    xd = draw_bf16(torch, dev, gen, (K,), std=x_std)
    nwd = draw_bf16(torch, dev, gen, (K,), mean=1.0, std=0.1)
    x, nw = dec.f(host_bits(xd)), dec.f(host_bits(nwd))
    xin = dec.rms_norm(x, nw, 1e-6) if norm else x
    tiled = None
    if case == "lm_head":
        tiled = torch.zeros(lib.tiled_size(E5M2, n_outs[0], K), dtype=torch.uint8, device=dev)
        assert lib.weight_prepare(wds[0].data_ptr(), E5M2, n_outs[0], K, K, tiled.data_ptr()) == 0

    def sampled(w, n, count=512):
        rows = np.sort(np.random.default_rng(n).choice(n, size=min(count, n), replace=False))
        codes = w[torch.from_numpy(rows).to(dev)].cpu().numpy()
        return rows, dec.linear(oracle.dequant_fp8_to_bf16(codes, oracle.E5M2).reshape(codes.shape), xin)

    try:
        if case == "gate_up":
            y = torch.zeros(n_outs[0] + 8, dtype=torch.int16, device=dev)
            d = pkg.capi.make_fused_linear(E5M2, K, [w.data_ptr() for w in wds], n_outs, [y.data_ptr(), None], xd.data_ptr(),
                                           norm_weight=nwd.data_ptr(), norm_eps=1e-6, pair=True)
            assert lib.quant_linear_fused(d) == 0 and lib.last_kernel() == "gemv_fused"
            out = from_dev(y, np.uint16)
            assert not out[n_outs[0]:].any()
            rows, gate = sampled(wds[0], n_outs[0], 1024)
            _, up = sampled(wds[1], n_outs[0], 1024)
            want = dec.silu_mul(gate, up)
            assert ulp_close(out[rows], want, ulps=3.0, floor=1e-4).all()
            assert (out[rows] == oracle.f32_to_bf16(want)).mean() > 0.97
            return
        ys = [torch.zeros(n + 8, dtype=torch.int16, device=dev) for n in n_outs]
        resd = draw_bf16(torch, dev, gen, (n_outs[0],)) if case in ("o", "down") else None
        d = pkg.capi.make_fused_linear(E5M2, K, [w.data_ptr() for w in wds], n_outs, [y.data_ptr() for y in ys], xd.data_ptr(),
                                       norm_weight=nwd.data_ptr() if norm else None, norm_eps=1e-6,
                                       residual=resd.data_ptr() if resd is not None else None)
        assert lib.quant_linear_fused(d) == 0
        assert lib.last_kernel() == ("gemv_fused_mfma" if case == "lm_head" else "gemv_fused")
        for s, n in enumerate(n_outs):
            out = from_dev(ys[s], np.uint16)
            assert not out[n:].any()
            rows, lin = sampled(wds[s], n)
            if resd is not None:
                res = dec.f(host_bits(resd))[rows]
                want = dec.r(lin + res)
                tol = np.maximum(np.maximum(np.abs(lin), np.abs(res)), np.abs(want)) * 2.0 ** -7 + 1e-4
                assert (np.abs(dec.f(out[rows]).astype(np.float64) - want) <= tol).all()
                assert (out[rows] == oracle.f32_to_bf16(want)).mean() > 0.98
            else:
                assert ulp_close(out[rows], lin, ulps=1.0, floor=2e-5).all(), s
    finally:
        if tiled is not None:
            assert lib.weight_release(wds[0].data_ptr()) == 0


# ------------------------------------------------------------------------------------------ decode step

@pytest.mark.parametrize("exact_attention", [False, True])
@pytest.mark.parametrize("arch", ["qwen3_8b_fp8", "llama31_8b_fp4"])
def test_decode_step_at_qwen3_8b_widths(gpu, pkg, oracle, dec, exact_attention, arch):
    """Two layers of the Qwen3-8B shape (hidden 4096, 32 / 8 heads, intermediate 12288, vocabulary 151936,
    4096 cache rows) with caches already holding 4090 positions, two steps from position 4090: every launch
    configuration the benchmark's 36-layer model uses is reached.  The last layer's intermediate vectors, the
    appended cache rows of both layers and 4096 sampled logits against the CPU oracle on the same bytes.
    llama31_8b_fp4: the same at the Llama-3.1-8B shape (intermediate 14336, vocabulary 128256, RoPE theta 5e5, no
    per-head norms) with FP4_E2M1 block-16 linears packed as the converter packs them -- the launches of the
    benchmark's fp4_decode_step."""
    torch, dev, lib = gpu
    host = pkg.host_api.host()
    host.init(0)
    fp4 = arch == "llama31_8b_fp4"
    if fp4:
        cfg = dec.DecodeConfig(layers=2, hidden=4096, n_q=32, n_kv=8, inter=14336, vocab=128256, t_kv=4096, theta=5e5)
    else:
        cfg = dec.DecodeConfig(layers=2, hidden=4096, n_q=32, n_kv=8, inter=12288, vocab=151936, t_kv=4096)
    model = pkg.host_api.DecodeModel(host, cfg.layers, cfg.hidden, cfg.n_q, cfg.n_kv, cfg.head_dim, cfg.inter, cfg.vocab, cfg.t_kv, theta=cfg.theta)
    model.set_exact_attention(exact_attention)
    model.set_qk_norm(not fp4)
    gen = torch.Generator(device=dev).manual_seed(8)
    copy = lambda src, dst, nbytes: lib.convert(src.data_ptr(), BF16, dst, BF16, nbytes, 1.0)      # same type: a byte copy on the device

    def draw_fp4(n_out, K):
        """(packed codes, E4M3 block scales) on the device, from N(0, 0.02) rounded to BF16, in slabs of rows"""
        nibs, scs = [], []
        rows = max(1, (1 << 25) // K)
        for r0 in range(0, n_out, rows):
            w = (torch.randn(min(rows, n_out - r0), K, device=dev, generator=gen) * 0.02).to(torch.bfloat16).float()
            nib, sc = pack_fp4_on_device(torch, w, 16)
            nibs.append(nib)
            scs.append(sc)
        return torch.cat(nibs), torch.cat(scs)

    def put_linear(li, name, n_out, K):
        """Draws one linear, hands it to the model, returns what the oracle's model dict holds for it"""
        if fp4:
            nib, sc = draw_fp4(n_out, K)
            nib_h, sc_h = nib.cpu().numpy(), sc.cpu().numpy()
            model.set_tensor(li, name, nib_h, 6)
            model.set_block_scales(li, name, sc_h)
            return (nib_h, sc_h), (nib, sc)
        w = draw_e5m2(torch, dev, gen, n_out, K)
        assert copy(w, model.tensor_ptr(li, name), n_out * K) == 0
        return w.cpu().numpy(), w

    weights = {"layers": []}
    lin_shapes = {"wq": (cfg.q_out, cfg.hidden), "wk": (cfg.kv_out, cfg.hidden), "wv": (cfg.kv_out, cfg.hidden), "wo": (cfg.hidden, cfg.q_out),
                  "w_gate": (cfg.inter, cfg.hidden), "w_up": (cfg.inter, cfg.hidden), "w_down": (cfg.hidden, cfg.inter)}
    norm_sizes = {"rms_attn": cfg.hidden, "rms_ffn": cfg.hidden}
    if not fp4:
        norm_sizes.update(q_norm=128, k_norm=128)
    start = 4090
    k_host = np.zeros((cfg.layers, cfg.n_kv, cfg.t_kv, 128), dtype=np.float32)
    v_host = np.zeros_like(k_host)
    for li in range(cfg.layers):
        L = {}
        for name, (n_out, K) in lin_shapes.items():
            L[name], _ = put_linear(li, name, n_out, K)
        for name, n in norm_sizes.items():
            v = draw_bf16(torch, dev, gen, (n,), mean=1.0, std=0.1)
            assert copy(v, model.tensor_ptr(li, name), n * 2) == 0
            L[name] = host_bits(v)
        weights["layers"].append(L)
        for is_v, dst in ((False, k_host), (True, v_host)):
            c = draw_bf16(torch, dev, gen, (cfg.n_kv, cfg.t_kv, 128))
            c[:, start:] = 0x7FC1                                    # rows not written yet hold NaN patterns
            assert copy(c, model.kv_ptr(li, is_v), c.numel() * 2) == 0
            dst[li] = dec.f(host_bits(c))
    lm_host, lm = put_linear(0, "lm_head", cfg.vocab, cfg.hidden)
    if not fp4:
        assert model.prepare_tiled(0, "lm_head")
    fin = draw_bf16(torch, dev, gen, (cfg.hidden,), mean=1.0, std=0.1)
    assert copy(fin, model.tensor_ptr(0, "rms_final"), cfg.hidden * 2) == 0
    emb_rows = {}
    emb = draw_bf16(torch, dev, gen, (cfg.vocab, cfg.hidden))
    assert copy(emb, model.tensor_ptr(0, "emb"), cfg.vocab * cfg.hidden * 2) == 0
    torch.cuda.synchronize()

    logit_rows = np.sort(np.random.default_rng(3).choice(cfg.vocab, size=4096, replace=False))
    if fp4:
        lm_rows = (lm_host[0][logit_rows], lm_host[1][logit_rows])
    else:
        lm_rows = lm[torch.from_numpy(logit_rows).to(dev)].cpu().numpy()

    class Rows:
        """Stands in for a [vocab, hidden] array of which only a few rows were downloaded."""

        def __init__(self, fetch):
            self.fetch = fetch

        def __getitem__(self, i):
            return self.fetch(i)

    weights["emb"] = Rows(lambda t: host_bits(emb[int(t)]))
    weights["rms_final"] = host_bits(fin)
    pick = lambda idx: np.searchsorted(logit_rows, np.asarray(idx))
    weights["lm_head"] = Rows((lambda idx: (lm_rows[0][pick(idx)], lm_rows[1][pick(idx)])) if fp4 else (lambda idx: lm_rows[pick(idx)]))
    del emb_rows
    orc = dec.DecodeOracle(cfg, weights)
    orc.k[:], orc.v[:] = k_host, v_host
    orc.k[:, :, start:], orc.v[:, :, start:] = 0.0, 0.0              # the oracle masks them; NaN * 0 would poison its matrix products

    token = 1234
    for pos in (start, start + 1):
        model.reset(token, pos)
        got_token = model.step()
        assert model.pos == pos + 1
        trace = {}
        want_logits, _ = orc.step(token, pos, trace=trace, logit_rows=logit_rows)
        last = cfg.layers - 1
        # (the step ends by fetching the next token's embedding into x, so the last layer's output is checked through the logits)
        for name, want in (("att", trace[f"att{last}"]), ("r1", trace[f"r1_{last}"]), ("gated", trace[f"gated{last}"])):
            got = dec.f(model.activation(name))
            assert np.isfinite(got).all(), name
            err = np.linalg.norm(got - want.reshape(-1)) / np.linalg.norm(want)
            # The second layer's inputs already differ from the oracle's by the first layer's BF16 roundings (r1 of a
            # single layer: 1e-3), which the softmax amplifies; on the route that keeps FP32 probabilities every element
            # may sit one more ulp away (a single layer measures 3e-3 .. 4e-3 there, two layers up to 1.1e-2).
            assert err < (2e-2 if name == "att" and not exact_attention else 1e-2), (pos, name, err)
        for li in range(cfg.layers):
            gk, gv = dec.f(model.kv(li, False)[:, pos]), dec.f(model.kv(li, True)[:, pos])
            tol = 2e-3 if li == 0 else 1e-2                          # layer 0 sees identical inputs
            assert np.linalg.norm(gk - orc.k[li, :, pos]) <= tol * np.linalg.norm(orc.k[li, :, pos]), (pos, li)
            assert np.linalg.norm(gv - orc.v[li, :, pos]) <= tol * np.linalg.norm(orc.v[li, :, pos]), (pos, li)
        logits = model.logits()
        got = dec.f(logits[logit_rows])
        assert np.linalg.norm(got - want_logits) <= 1e-2 * np.linalg.norm(want_logits), pos
        assert np.abs(got - want_logits).max() <= 2e-2 * np.abs(want_logits).max()
        # greedy pick = lowest index of the largest logit the kernel itself produced
        all_logits = dec.f(logits)
        assert got_token == int(np.argmax(all_logits))
        token = got_token


# ------------------------------------------------------------------------------------------ prompt phase

@pytest.mark.parametrize("tiled", [False, True])
def test_fused_prompt_gemms_at_qwen3_8b_shapes_equal_the_separate_calls(gpu, pkg, oracle, tiled):
    """2048 tokens at Qwen3-8B widths: q, k, v as one launch against three hip_quant_gemm calls, and gate / up / SwiGLU as
    one launch against two calls and hip_swiglu_bf16 -- byte for byte (none of these shapes splits its k range), on the
    file layout and on tiled copies; sampled features of the q output against the exact contraction."""
    torch, dev, lib = gpu
    gen = torch.Generator(device=dev).manual_seed(77)
    T, K = 2048, 4096
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())
    x = draw_bf16(torch, dev, gen, (T, K))
    widths = (4096, 1024, 1024, 12288, 12288)                  # q, k, v, gate, up
    ws = [draw_e5m2(torch, dev, gen, n, K) for n in widths]
    keep = []
    if tiled:
        for w, n in zip(ws, widths):
            td = torch.zeros(lib.tiled_size(E5M2, n, K), dtype=torch.uint8, device=dev)
            assert lib.weight_prepare(w.data_ptr(), E5M2, n, K, K, td.data_ptr()) == 0
            keep.append(td)
    try:
        sep = [torch.zeros(T * n, dtype=torch.int16, device=dev) for n in widths]
        for w, y, n in zip(ws, sep, widths):
            assert lib.linear(w.data_ptr(), E5M2, x.data_ptr(), y.data_ptr(), n, T, K) == 0
            assert lib.last_kernel() == ("gemm_mfma_tiled" if tiled else "gemm_mfma")
        one = [torch.zeros(T * n, dtype=torch.int16, device=dev) for n in widths[:3]]
        arr_i = (ctypes.c_int * 3)(*widths[:3])
        arr_w = (ctypes.c_void_p * 3)(*[w.data_ptr() for w in ws[:3]])
        arr_s = (ctypes.c_float * 3)(1.0, 1.0, 1.0)
        arr_y = (ctypes.c_void_p * 3)(*[y.data_ptr() for y in one])
        assert lib.c.hip_quant_gemm_segments(3, arr_i, arr_w, arr_s, arr_y, arr_i, E5M2, T, K, K, ptr(x), K) == 0
        for a, b in zip(one, sep[:3]):
            assert torch.equal(a, b)
        rows = np.random.default_rng(3).choice(4096, size=96, replace=False)
        want = oracle.linear_exact(oracle.dequant_fp8_to_bf16(ws[0][torch.as_tensor(rows, device=dev)].cpu().numpy(), E5M2), host_bits(x).reshape(T, K))
        check_rows(bf16_f64(oracle, host_bits(one[0]).reshape(T, 4096)[:, rows]), want, "q of the q,k,v launch")
        prod, fused = torch.zeros(T * 12288, dtype=torch.int16, device=dev), torch.zeros(T * 12288, dtype=torch.int16, device=dev)
        assert lib.c.hip_swiglu_bf16(ptr(sep[3]), ptr(sep[4]), ptr(prod), T * 12288) == 0
        assert lib.c.hip_quant_gemm_swiglu(12288, T, K, ptr(ws[3]), ptr(ws[4]), E5M2, K, ctypes.c_float(1.0), ctypes.c_float(1.0),
                                           ptr(x), K, ptr(fused), 12288) == 0
        assert lib.last_kernel() == ("gemm_swiglu_tiled" if tiled else "gemm_swiglu")
        assert torch.equal(fused, prod) and bool(fused.any())
    finally:
        if tiled:
            for w in ws:
                assert lib.weight_release(w.data_ptr()) == 0


@pytest.mark.parametrize("tiled", [False, True])
@pytest.mark.parametrize("T", [32, 128])
def test_fused_prompt_gemms_of_a_short_prompt_at_qwen3_8b_shapes(gpu, pkg, oracle, dec, tiled, T):
    """32 and 128 tokens at Qwen3-8B widths, where the q,k,v launch (24 feature tiles) and the gate / up pair (96) split
    their k range over workgroups and a combine launch finishes them -- for the pair with the SwiGLU product: sampled
    features of q, k, v and of the product against the exact contraction, nothing written past the outputs."""
    torch, dev, lib = gpu
    gen = torch.Generator(device=dev).manual_seed(78 + T)
    K = 4096
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())
    x = draw_bf16(torch, dev, gen, (T, K))
    widths = (4096, 1024, 1024, 12288, 12288)                  # q, k, v, gate, up
    ws = [draw_e5m2(torch, dev, gen, n, K) for n in widths]
    keep = []
    if tiled:
        for w, n in zip(ws, widths):
            td = torch.zeros(lib.tiled_size(E5M2, n, K), dtype=torch.uint8, device=dev)
            assert lib.weight_prepare(w.data_ptr(), E5M2, n, K, K, td.data_ptr()) == 0
            keep.append(td)
    try:
        X = host_bits(x).reshape(T, K)
        exact = lambda w, rows: oracle.linear_exact(oracle.dequant_fp8_to_bf16(w[torch.as_tensor(rows, device=dev)].cpu().numpy(), E5M2), X)
        one = [torch.zeros(T * n + 64, dtype=torch.int16, device=dev) for n in widths[:3]]
        arr_i = (ctypes.c_int * 3)(*widths[:3])
        arr_w = (ctypes.c_void_p * 3)(*[w.data_ptr() for w in ws[:3]])
        arr_s = (ctypes.c_float * 3)(1.0, 1.0, 1.0)
        arr_y = (ctypes.c_void_p * 3)(*[y.data_ptr() for y in one])
        assert lib.c.hip_quant_gemm_segments(3, arr_i, arr_w, arr_s, arr_y, arr_i, E5M2, T, K, K, ptr(x), K) == 0
        assert lib.last_kernel() == ("gemm_segments_tiled" if tiled else "gemm_segments")
        for y, w, n, name in zip(one, ws, widths, "qkv"):
            bits = host_bits(y)
            assert not bits[T * n:].any(), name
            rows = np.random.default_rng(n + T).choice(n, size=64, replace=False)
            check_rows(bf16_f64(oracle, bits[:T * n].reshape(T, n)[:, rows]), exact(w, rows), f"{name} of the q,k,v launch, {T} tokens")
        fused = torch.zeros(T * 12288 + 64, dtype=torch.int16, device=dev)
        assert lib.c.hip_quant_gemm_swiglu(12288, T, K, ptr(ws[3]), ptr(ws[4]), E5M2, K, ctypes.c_float(1.0), ctypes.c_float(1.0),
                                           ptr(x), K, ptr(fused), 12288) == 0
        assert lib.last_kernel() == ("gemm_swiglu_tiled" if tiled else "gemm_swiglu")
        bits = host_bits(fused)
        assert not bits[T * 12288:].any()
        rows = np.random.default_rng(5 + T).choice(12288, size=64, replace=False)
        gate = oracle.f32_to_bf16(exact(ws[3], rows).astype(np.float32))
        up = oracle.f32_to_bf16(exact(ws[4], rows).astype(np.float32))
        want = dec.silu_mul(dec.f(gate), dec.f(up))
        have = dec.f(bits[:T * 12288].reshape(T, 12288)[:, rows])
        assert np.isfinite(have).all() and have.any()
        assert np.linalg.norm(have - want) <= 1e-2 * np.linalg.norm(want)
    finally:
        if tiled:
            for w in ws:
                assert lib.weight_release(w.data_ptr()) == 0


@pytest.mark.parametrize("arch", ["qwen3_8b_fp8", "llama31_8b_fp4"])
def test_prompt_phase_at_full_widths_equals_token_by_token_decoding(gpu, pkg, oracle, dec, arch):
    """DecodeModel::prefill at the benchmark's widths (two layers): 130 prompt tokens from position 0 in one call against the
    same tokens fed one at a time through the decode step on the attention route with the reference's rounding points
    (which the tests above hold against the CPU oracle at these widths).  Both read the same weight bytes; the linears run
    as GEMMs with 130 columns here and as GEMVs there, so agreement is to summation order: cache rows, last logits,
    and the greedy pick when its margin allows."""
    torch, dev, lib = gpu
    host = pkg.host_api.host()
    host.init(0)
    fp4 = arch == "llama31_8b_fp4"
    if fp4:
        cfg = dec.DecodeConfig(layers=2, hidden=4096, n_q=32, n_kv=8, inter=14336, vocab=128256, t_kv=256, theta=5e5)
    else:
        cfg = dec.DecodeConfig(layers=2, hidden=4096, n_q=32, n_kv=8, inter=12288, vocab=151936, t_kv=256)
    gen = torch.Generator(device=dev).manual_seed(21)
    copy = lambda src, dst, nbytes: lib.convert(src.data_ptr(), BF16, dst, BF16, nbytes, 1.0)
    models = [pkg.host_api.DecodeModel(host, cfg.layers, cfg.hidden, cfg.n_q, cfg.n_kv, cfg.head_dim, cfg.inter, cfg.vocab, cfg.t_kv, theta=cfg.theta)
              for _ in range(2)]
    for m in models:
        m.set_qk_norm(not fp4)
        m.set_exact_attention(True)
    lin_shapes = {"wq": (cfg.q_out, cfg.hidden), "wk": (cfg.kv_out, cfg.hidden), "wv": (cfg.kv_out, cfg.hidden), "wo": (cfg.hidden, cfg.q_out),
                  "w_gate": (cfg.inter, cfg.hidden), "w_up": (cfg.inter, cfg.hidden), "w_down": (cfg.hidden, cfg.inter)}

    def put_linear(li, name, n_out, K):
        if fp4:
            nibs, scs = [], []
            rows = max(1, (1 << 25) // K)
            for r0 in range(0, n_out, rows):
                w = (torch.randn(min(rows, n_out - r0), K, device=dev, generator=gen) * 0.02).to(torch.bfloat16).float()
                nib, sc = pack_fp4_on_device(torch, w, 16)
                nibs.append(nib); scs.append(sc)
            nib_h, sc_h = torch.cat(nibs).cpu().numpy(), torch.cat(scs).cpu().numpy()
            for m in models:
                m.set_tensor(li, name, nib_h, 6)
                m.set_block_scales(li, name, sc_h)
        else:
            w = draw_e5m2(torch, dev, gen, n_out, K)
            for m in models:
                assert copy(w, m.tensor_ptr(li, name), n_out * K) == 0

    def put_plain(li, name, shape, mean, std):
        v = draw_bf16(torch, dev, gen, shape, mean=mean, std=std)
        for m in models:
            assert copy(v, m.tensor_ptr(li, name), v.numel() * 2) == 0

    for li in range(cfg.layers):
        for name, (n_out, K) in lin_shapes.items():
            put_linear(li, name, n_out, K)
        for name in ("rms_attn", "rms_ffn"):
            put_plain(li, name, (cfg.hidden,), 1.0, 0.1)
        if not fp4:
            for name in ("q_norm", "k_norm"):
                put_plain(li, name, (128,), 1.0, 0.1)
    put_linear(0, "lm_head", cfg.vocab, cfg.hidden)
    if not fp4:
        for m in models:
            assert m.prepare_tiled(0, "lm_head")
    put_plain(0, "rms_final", (cfg.hidden,), 1.0, 0.1)
    put_plain(0, "emb", (cfg.vocab, cfg.hidden), 0.0, 1.0)
    torch.cuda.synchronize()

    T = 130
    prompt = [int(t) for t in np.random.default_rng(11).integers(0, cfg.vocab, size=T)]
    a, b = models
    next_a = a.prefill(prompt)
    for pos, tok in enumerate(prompt):
        b.reset(tok, pos)
        next_b = b.step()
    assert a.pos == b.pos == T
    for li in range(cfg.layers):
        for is_v in (False, True):
            ca, cb = dec.f(a.kv(li, is_v)[:, :T]), dec.f(b.kv(li, is_v)[:, :T])
            assert np.isfinite(ca).all()
            err = np.linalg.norm(ca - cb) / np.linalg.norm(cb)
            assert err <= (2e-3 if li == 0 else 1e-2), (li, is_v, err)
            # per position too: no row may be off by more than BF16 noise
            rows = np.linalg.norm((ca - cb).reshape(cfg.n_kv, T, -1), axis=2) / np.linalg.norm(cb.reshape(cfg.n_kv, T, -1), axis=2)
            assert rows.max() <= 3e-2, (li, is_v, rows.max())
    la, lb = dec.f(a.logits()), dec.f(b.logits())
    assert np.linalg.norm(la - lb) <= 1e-2 * np.linalg.norm(lb)
    top2 = np.sort(lb)[-2:]
    if top2[1] - top2[0] > 2 * np.abs(la - lb).max():
        assert next_a == next_b
