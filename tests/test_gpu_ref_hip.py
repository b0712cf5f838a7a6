"""The BF16 neighbour ops against the reference's own HIP kernels (oracle/_ref/libref_hip.so, built
from cccc-hip/hip_functions.cpp where it lies): the product's entry points of the same name must
agree with them, and so must the CPU decode oracle -- this is what pins oracle/decode_oracle.py."""
import ctypes

import numpy as np
import pytest

from gpu_util import from_dev, to_dev

pytestmark = pytest.mark.gpu
BF16 = 3


@pytest.fixture(scope="module")
def ref(gpu):
    from oracle import ref_hip
    L = ref_hip.lib()
    if L is None:
        pytest.skip("oracle/_ref/libref_hip.so was not built (no reference tree at build time)")
    return L


@pytest.fixture(scope="module")
def dec():
    from oracle import decode_oracle
    return decode_oracle


def p(t):
    return ctypes.c_void_p(t.data_ptr())


def bits(oracle, a):
    return oracle.f32_to_bf16(np.asarray(a, dtype=np.float32))


def ulps_apart(oracle, a_bits, b_bits):
    a, b = oracle.bf16_to_f32(a_bits).astype(np.float64), oracle.bf16_to_f32(b_bits).astype(np.float64)
    return np.abs(a - b) / (np.maximum(np.abs(b), 2.0 ** -120) * 2.0 ** -8)


@pytest.mark.parametrize("outer,inner", [(1, 4096), (40, 128), (3, 1000), (2, 12288)])
def test_rms_norm_product_reference_and_oracle_agree(gpu, ref, oracle, dec, outer, inner):
    torch, dev, lib = gpu
    rng = np.random.default_rng(outer * inner)
    x = bits(oracle, rng.standard_normal((outer, inner)) * 3)
    w = bits(oracle, 1 + 0.1 * rng.standard_normal(inner))
    xd, wd = to_dev(torch, dev, x), to_dev(torch, dev, w)
    out = {}
    for name, L in (("product", lib.c), ("reference", ref)):
        y = torch.zeros(outer * inner, dtype=torch.int16, device=dev)
        inv = torch.zeros(outer, dtype=torch.float32, device=dev)
        assert L.hip_rms_norm_fwd(BF16, p(xd), p(y), p(wd), p(inv), outer, inner, ctypes.c_float(1e-6)) == 0
        out[name] = (from_dev(y, np.uint16), inv.cpu().numpy())
    want = oracle.f32_to_bf16(dec.rms_norm(dec.f(x), dec.f(w), 1e-6)).reshape(-1)
    for name in ("product", "oracle"):
        got = out[name][0] if name == "product" else want
        # the reference adds the squares one thread per row in index order; a different order can move
        # invstd by an FP32 ulp, which flips a BF16 rounding now and then, never more than one ulp
        assert ulps_apart(oracle, got, out["reference"][0]).max() <= 1.0, name
        assert (got == out["reference"][0]).mean() > 0.995, name
    assert np.allclose(out["product"][1], out["reference"][1], rtol=2e-6)


@pytest.mark.parametrize("pos", [0, 3, 63])
def test_rope_product_reference_and_oracle_agree(gpu, ref, oracle, dec, pos):
    torch, dev, lib = gpu
    rng = np.random.default_rng(pos)
    cfg = dec.DecodeConfig(t_kv=64)
    cos, sin = dec.rope_tables(cfg)
    x = bits(oracle, rng.standard_normal((2, 5, 128)))              # B = 2 "heads", T = 5 positions
    xd, cd, sd = to_dev(torch, dev, x), to_dev(torch, dev, cos), to_dev(torch, dev, sin)
    t_len = 5 if pos + 5 <= 64 else 1
    out = {}
    for name, L in (("product", lib.c), ("reference", ref)):
        y = torch.zeros(x.size, dtype=torch.int16, device=dev)
        assert L.hip_rope_fwd(BF16, p(xd), p(y), p(cd), p(sd), 128, t_len, 2 * 5 // t_len, pos) == 0
        out[name] = from_dev(y, np.uint16)
    assert np.array_equal(out["product"], out["reference"])
    if t_len == 5:
        want = np.stack([[dec.rope(dec.f(x[b, t]), dec.f(cos[pos + t]), dec.f(sin[pos + t])) for t in range(5)] for b in range(2)])
        assert np.array_equal(oracle.f32_to_bf16(want).reshape(-1), out["reference"])


def test_embed_product_and_reference_agree(gpu, ref, oracle):
    torch, dev, lib = gpu
    rng = np.random.default_rng(9)
    W = bits(oracle, rng.standard_normal((50, 256)))
    wd = to_dev(torch, dev, W)
    ids = torch.tensor([3.0, 49.0, 0.0, 17.0], dtype=torch.float32, device=dev)
    out = {}
    for name, L in (("product", lib.c), ("reference", ref)):
        y = torch.zeros(4 * 256, dtype=torch.int16, device=dev)
        assert L.hip_embed_fwd(BF16, p(ids), p(wd), p(y), 256, 2, 2) == 0
        out[name] = from_dev(y, np.uint16)
    assert np.array_equal(out["product"], out["reference"])
    assert np.array_equal(out["reference"].reshape(4, 256), W[[3, 49, 0, 17]])


def test_oracle_softmax_mask_silu_residual_match_the_reference_kernels(gpu, ref, oracle, dec):
    torch, dev, _ = gpu
    rng = np.random.default_rng(4)
    # causal mask + softmax over a (T_k = 300) row per head, query at position 200
    n_heads, t_k, pos = 4, 300, 200
    s = bits(oracle, rng.standard_normal((n_heads, t_k)) * 3)
    sd = to_dev(torch, dev, s)
    assert ref.hip_causal_mask(BF16, p(sd), 1, t_k, n_heads, pos) == 0
    masked = from_dev(sd, np.uint16).reshape(n_heads, t_k)
    want_masked = s.copy()
    want_masked[:, pos + 1:] = oracle.f32_to_bf16(np.float32([-1e9]))[0]
    assert np.array_equal(masked, want_masked)
    assert ref.hip_softmax_bf16(p(sd), p(sd), t_k, n_heads, ctypes.c_float(1.0), ctypes.c_float(0.0)) == 0
    probs = from_dev(sd, np.uint16).reshape(n_heads, t_k)
    for h in range(n_heads):
        want = oracle.f32_to_bf16(dec.softmax(dec.f(want_masked[h])))
        assert ulps_apart(oracle, want, probs[h])[probs[h] != 0].max() <= 1.0
        assert (want == probs[h]).mean() > 0.99
        assert not probs[h, pos + 1:].any()
    # SiLU as the graph runs it: sigmoid -> mul -> mul, each a BF16 tensor
    n = 5000
    gate, up = bits(oracle, rng.standard_normal(n) * 4), bits(oracle, rng.standard_normal(n))
    gd, ud = to_dev(torch, dev, gate), to_dev(torch, dev, up)
    sig = torch.zeros(n, dtype=torch.int16, device=dev)
    assert ref.hip_sigmoid_bf16(p(sig), p(gd), n, ctypes.c_float(1.0), ctypes.c_float(0.0)) == 0
    silu = torch.zeros(n, dtype=torch.int16, device=dev)
    assert ref.hip_mul(BF16, p(gd), p(sig), p(silu), n, ctypes.c_float(1.0), ctypes.c_float(0.0)) == 0
    gated = torch.zeros(n, dtype=torch.int16, device=dev)
    assert ref.hip_mul(BF16, p(silu), p(ud), p(gated), n, ctypes.c_float(1.0), ctypes.c_float(0.0)) == 0
    want = oracle.f32_to_bf16(dec.silu_mul(dec.f(gate), dec.f(up)))
    got = from_dev(gated, np.uint16)
    assert ulps_apart(oracle, want, got)[got != 0].max() <= 2.0          # expf of the device vs the host: an ulp of sigmoid can carry through two products
    assert (want == got).mean() > 0.99
    # residual add
    a, b = bits(oracle, rng.standard_normal(n)), bits(oracle, rng.standard_normal(n))
    ad, bd = to_dev(torch, dev, a), to_dev(torch, dev, b)
    r = torch.zeros(n, dtype=torch.int16, device=dev)
    assert ref.hip_add(BF16, p(ad), p(bd), p(r), n, ctypes.c_float(1.0), ctypes.c_float(1.0)) == 0
    assert np.array_equal(from_dev(r, np.uint16), oracle.f32_to_bf16(dec.f(a) + dec.f(b)))


def test_attention_oracle_matches_the_reference_sequence(gpu, ref, oracle, dec):
    """The reference's attention (cccc/MatrixEx.cpp:3018-3104) with its own mask and softmax kernels and
    BF16 GEMMs (FP32 accumulate, BF16 out) for K^T q and V p, against the CPU oracle and the product."""
    torch, dev, lib = gpu
    rng = np.random.default_rng(6)
    n_q, n_kv, t_kv, pos = 8, 2, 256, 180
    q = bits(oracle, rng.standard_normal((n_q, 128)))
    kc = bits(oracle, rng.standard_normal((n_kv, t_kv, 128)))
    vc = bits(oracle, rng.standard_normal((n_kv, t_kv, 128)))
    qt = to_dev(torch, dev, q).view(torch.bfloat16).reshape(n_q, 128)
    kt = to_dev(torch, dev, kc).view(torch.bfloat16).reshape(n_kv, t_kv, 128).repeat_interleave(n_q // n_kv, dim=0)   # the graph tiles K / V per query head
    vt = to_dev(torch, dev, vc).view(torch.bfloat16).reshape(n_kv, t_kv, 128).repeat_interleave(n_q // n_kv, dim=0)
    scale = 1.0 / np.sqrt(np.float32(128.0))
    scores = torch.baddbmm(torch.zeros(n_q, t_kv, 1, dtype=torch.bfloat16, device=dev), kt, qt.unsqueeze(2), beta=0.0, alpha=float(scale)).squeeze(2).contiguous()
    assert ref.hip_causal_mask(BF16, p(scores), 1, t_kv, n_q, pos) == 0
    assert ref.hip_softmax_bf16(p(scores), p(scores), t_kv, n_q, ctypes.c_float(1.0), ctypes.c_float(0.0)) == 0
    y_ref = torch.bmm(scores.unsqueeze(1), vt).squeeze(1).contiguous()
    got_ref = y_ref.view(torch.int16).cpu().numpy().view(np.uint16)
    want = dec.attention(dec.f(q), dec.f(kc), dec.f(vc), pos, n_q, n_kv)
    scale_abs = 2e-3 * np.abs(want).max()
    assert (np.abs(dec.f(got_ref) - want) <= 2 * np.abs(want) * 2.0 ** -8 + scale_abs).all()
    # the product's reference-rounding path against the same reference sequence
    ws_bytes = lib.c.hip_attention_decode_workspace_bytes(n_q, n_kv, t_kv)
    ws = torch.zeros(ws_bytes, dtype=torch.uint8, device=dev)
    pd = torch.tensor([pos], dtype=torch.int32, device=dev)
    y = torch.zeros(n_q * 128, dtype=torch.int16, device=dev)
    qd, kd, vd = to_dev(torch, dev, q), to_dev(torch, dev, kc), to_dev(torch, dev, vc)
    assert lib.c.hip_attention_decode_bf16(p(qd), p(kd), p(vd), p(y), p(ws), ws_bytes, n_q, n_kv, 128, t_kv, p(pd)) == 0
    got = dec.f(from_dev(y, np.uint16).reshape(n_q, 128))
    assert (np.abs(got - dec.f(got_ref)) <= 2 * np.abs(dec.f(got_ref)) * 2.0 ** -8 + scale_abs).all()
