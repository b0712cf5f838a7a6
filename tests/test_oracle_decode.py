"""Pins the decode-step oracle on the CPU: closed forms of each op and an independent float64 torch
implementation of the whole step (no intermediate rounding), which the BF16-rounded oracle must
follow within BF16 noise."""
import numpy as np
import pytest
import torch


def test_rms_norm_closed_forms(oracle):
    from oracle import decode_oracle as d
    w = d.f(oracle.f32_to_bf16(np.linspace(0.5, 1.5, 128).astype(np.float32)))
    x = np.full(128, 3.0, dtype=np.float32)
    assert np.array_equal(d.rms_norm(x, w, 0.0), w)                     # a constant vector normalises to the weights
    assert np.array_equal(d.rms_norm(-x, w, 0.0), -w)
    y = d.rms_norm(np.array([3.0, 4.0, 0.0, 0.0], dtype=np.float32), np.ones(4, dtype=np.float32), 0.0)
    assert np.allclose(y, np.array([3.0, 4.0, 0, 0]) / 2.5, rtol=2 ** -8)   # rms of (3,4,0,0) is 2.5
    rows = d.rms_norm(np.stack([x, 2 * x]), w, 0.0)                     # scale invariance, row by row
    assert np.array_equal(rows[0], rows[1])


def test_rope_closed_forms(oracle):
    from oracle import decode_oracle as d
    cfg = d.DecodeConfig(t_kv=32)
    cos, sin = d.rope_tables(cfg)
    c, s = d.f(cos), d.f(sin)
    assert np.all(cos[0] == 0x3F80) and np.all(sin[0] == 0)             # position 0: identity
    x = d.r(np.random.default_rng(0).standard_normal((3, 128)).astype(np.float32))
    assert np.array_equal(d.rope(x, c[0], s[0]), x)
    # tables: truncated (not rounded) float32 cos / sin of t * theta^(-2d/128)
    t, k = 7, 5
    angle = np.float32(t) * np.float32(np.float32(1e6) ** (np.float32(-2.0 * k) / np.float32(128)))
    want = np.float32(np.cos(angle)).view(np.uint32) >> 16
    assert abs(int(cos[t, k]) - int(want)) <= 1
    assert (d.f(cos[t]) ** 2 + d.f(sin[t]) ** 2 <= 1.0 + 1e-6).all()    # truncation never overshoots the unit circle
    # pair norms are preserved up to BF16 rounding
    y = d.rope(x, c[9], s[9])
    n0 = x[:, :64] ** 2 + x[:, 64:] ** 2
    n1 = y[:, :64] ** 2 + y[:, 64:] ** 2
    assert np.allclose(n0, n1, rtol=0.03, atol=1e-3)


def test_attention_and_silu_closed_forms(oracle):
    from oracle import decode_oracle as d
    rng = np.random.default_rng(1)
    k = np.zeros((1, 8, 128), dtype=np.float32)
    v = d.r(rng.standard_normal((1, 8, 128)).astype(np.float32))
    q = np.zeros((2, 128), dtype=np.float32)
    # all-zero keys: uniform weights over the positions <= pos, the rest is masked out
    out = d.attention(q, k, v, 3, 2, 1)
    assert np.allclose(out[0], v[0, :4].mean(axis=0), atol=2 ** -7 * np.abs(v).max())
    # a key aligned with the query dominates: the output is that value row
    k[0, 2] = 8.0
    q[:] = 8.0
    out = d.attention(q, k, v, 5, 2, 1)
    assert np.array_equal(out[1], v[0, 2])
    # position 0 attends to itself only
    assert np.array_equal(d.attention(q, k, v, 0, 2, 1)[0], v[0, 0])
    z = np.zeros(4, dtype=np.float32)
    assert np.array_equal(d.silu_mul(z, np.ones(4, dtype=np.float32)), z)
    g = np.array([20.0, -20.0, 1.0], dtype=np.float32)
    s = d.silu_mul(g, np.ones(3, dtype=np.float32))
    assert s[0] == 20.0 and abs(s[1]) < 1e-6 and abs(s[2] - 0.731) < 4e-3


def torch_step(model, cfg, oracle, d, tokens):
    """The same decode steps in float64 without intermediate rounding (independent implementation)."""
    T = torch.float64
    cos, sin = d.rope_tables(cfg)
    cos, sin = torch.from_numpy(d.f(cos)).to(T), torch.from_numpy(d.f(sin)).to(T)

    def W(a):
        return torch.from_numpy(oracle.decode_table(oracle.E5M2)[a]).to(T)

    def B(a):
        return torch.from_numpy(d.f(a)).to(T)

    def norm(x, w):
        return x * torch.rsqrt((x * x).mean(-1, keepdim=True) + cfg.eps) * w

    def rot(x, pos):
        xl, xr = x[..., :64], x[..., 64:]
        return torch.cat([xl * cos[pos] - xr * sin[pos], xr * cos[pos] + xl * sin[pos]], -1)

    ks = [torch.zeros(cfg.n_kv, cfg.t_kv, 128, dtype=T) for _ in range(cfg.layers)]
    vs = [torch.zeros(cfg.n_kv, cfg.t_kv, 128, dtype=T) for _ in range(cfg.layers)]
    outs = []
    for pos, tok in enumerate(tokens):
        x = B(model["emb"][tok])
        for li, L in enumerate(model["layers"]):
            xn = norm(x, B(L["rms_attn"]))
            q, k = (W(L["wq"]) @ xn).view(cfg.n_q, 128), (W(L["wk"]) @ xn).view(cfg.n_kv, 128)
            if "q_norm" in L:
                q, k = norm(q, B(L["q_norm"])), norm(k, B(L["k_norm"]))
            q, k = rot(q, pos), rot(k, pos)
            ks[li][:, pos], vs[li][:, pos] = k, (W(L["wv"]) @ xn).view(cfg.n_kv, 128)
            rep = cfg.n_q // cfg.n_kv
            kk, vv = ks[li][:, :pos + 1].repeat_interleave(rep, 0), vs[li][:, :pos + 1].repeat_interleave(rep, 0)
            p = torch.softmax(torch.einsum("htd,hd->ht", kk, q) / np.sqrt(128.0), -1)
            att = torch.einsum("ht,htd->hd", p, vv).reshape(-1)
            r1 = x + W(L["wo"]) @ att
            rn = norm(r1, B(L["rms_ffn"]))
            x = r1 + W(L["w_down"]) @ (torch.nn.functional.silu(W(L["w_gate"]) @ rn) * (W(L["w_up"]) @ rn))
        outs.append((W(model["lm_head"]) @ norm(x, B(model["rms_final"]))).numpy())
    return outs


@pytest.mark.parametrize("qk_norm", [True, False])
def test_oracle_follows_an_unrounded_float64_model(oracle, qk_norm):
    """qk_norm = False is the graph without per-head norms (Llama-style, scripts/convert_weights.py:494-503): the two
    cases must also differ from each other, or the switch would not be in the oracle's path."""
    from oracle import decode_oracle as d
    cfg = d.DecodeConfig(layers=2, hidden=256, n_q=4, n_kv=2, inter=512, vocab=500, t_kv=16, theta=1e6 if qk_norm else 5e5)
    model = d.make_model(cfg, 3, qk_norm=qk_norm)
    assert ("q_norm" in model["layers"][0]) == qk_norm
    tokens = [7, 123, 42, 499, 0]
    want = torch_step(model, cfg, oracle, d, tokens)
    orc = d.DecodeOracle(cfg, model)
    for pos, tok in enumerate(tokens):
        logits, nxt = orc.step(tok, pos)
        err = np.linalg.norm(logits - want[pos]) / np.linalg.norm(want[pos])
        assert err < 2e-2, (pos, err)                       # BF16 rounding at ~25 points per layer
        assert np.corrcoef(logits, want[pos])[0, 1] > 0.999
