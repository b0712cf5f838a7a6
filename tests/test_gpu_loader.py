"""Loading converted model files into the host mirror: WeightFile::loadNamed into a Matrix and
DecodeModel::loadNamedWeights, against tensors set directly and against the CPU oracle."""
import struct

import numpy as np
import pytest

from gpu_util import check_rows

pytestmark = pytest.mark.gpu
BF16, E4M3, E5M2, FP4 = 3, 4, 5, 6


@pytest.fixture(scope="module")
def host(gpu, pkg):
    h = pkg.host_api.host()
    h.init(0)
    return h


def linear_out(pkg, host, W, x_bits, n_out, K):
    X = host.matrix(K, 1, 1, 1, BF16)
    X.upload(x_bits)
    Y = host.matrix(n_out, 1, 1, 1, BF16)
    assert pkg.host_api.mul_batched(W, X, Y, ta=1, tb=0) == 0
    return Y.download(np.uint16, n_out)


def test_fp8_and_fp4_weights_load_like_direct_uploads(tmp_path, gpu, pkg, host, oracle):
    rng = np.random.default_rng(0)
    K, n_out = 512, 96
    x = oracle.f32_to_bf16(rng.standard_normal(K).astype(np.float32))
    w = pkg.weight_file.BinWriter()
    codes8 = oracle.encode_e5m2_rne((rng.standard_normal((n_out, K)) * 0.02).astype(np.float32))
    w.add("weight_fp8_e5m2_W_a", codes8); w.add_float("scale_W_a", 0.5); w.add_float("input_scale_W_a", 0.25)
    w.add("weight_W_legacy", codes8 & 0x7E)                                           # legacy key: FP8_E4M3, no scale entry -> 1.0
    nib, sc = pkg.synth.pack_fp4_blockscale((rng.standard_normal((n_out, K)) * 0.02).astype(np.float32), 16)
    w.add("weight_fp4_e2m1_W_b", nib); w.add("blockscale_W_b", sc)
    w.add("weight_fp4_e2m1_W_c", nib); w.add("blockscale_W_c", np.concatenate([sc, np.full(sc.size, 0x7E, np.uint8)]))   # twice the scale bytes, as the reference's own writer leaves them
    sc_f32 = oracle.decode_table(E4M3)[sc].astype(np.float32)
    w.add("weight_fp4_e2m1_W_d", np.concatenate([nib, np.zeros(nib.size, np.uint8)])); w.add("blockscale_W_d", sc_f32)     # blob sized by elements, legacy float32 scales
    w.add("weight_fp8_e5m2_W_short", codes8[:-1])
    path = tmp_path / "w.bin"
    w.save(path)
    f = pkg.host_api.WeightFile(host, path)

    m = host.matrix(K, n_out, 1, 1, BF16)                                             # allocated as BF16, re-typed by the load
    assert f.load_named(m, "W_a") == 0
    assert m.dtype == E5M2 and m.quant_scale == 0.5
    Wd = oracle.dequant_fp8_to_bf16(codes8, oracle.E5M2, 0.5).reshape(n_out, K)       # scale_W_a reached the kernel
    check_rows(oracle.bf16_to_f32(linear_out(pkg, host, m, x, n_out, K))[None, :].astype(np.float64), oracle.linear_exact(Wd, x[None, :]))
    m2 = host.matrix(K, n_out, 1, 1, E4M3)
    assert f.load_named(m2, "W_legacy") == 0 and m2.dtype == E4M3 and m2.quant_scale == 1.0
    assert np.array_equal(m2.download(np.uint8, n_out * K), (codes8 & 0x7E).reshape(-1))

    direct = host.matrix(K, n_out, 1, 1, BF16)
    direct.load_quantized(nib, 1.0, FP4)
    direct.set_block_scale(sc)
    y_direct = linear_out(pkg, host, direct, x, n_out, K)
    for name in ("W_b", "W_c", "W_d"):
        mf = host.matrix(K, n_out, 1, 1, BF16)
        assert f.load_named(mf, name) == 0, name
        assert mf.dtype == FP4
        assert np.array_equal(mf.block_scales(), sc), name
        assert np.array_equal(linear_out(pkg, host, mf, x, n_out, K), y_direct), name
    assert f.load_named(host.matrix(K, n_out, 1, 1, BF16), "W_short") == -1
    assert f.load_named(host.matrix(K, n_out, 1, 1, BF16), "W_absent") == 1


def test_plain_weights_keep_or_convert_their_type(tmp_path, gpu, pkg, host, oracle):
    rng = np.random.default_rng(1)
    n = 4096
    vals = rng.standard_normal(n).astype(np.float32)
    w = pkg.weight_file.BinWriter()
    w.add("weight_bf16_P", oracle.f32_to_bf16(vals))
    w.add("weight_half_Q", vals.astype(np.float16))
    w.add("weight_float_R", vals)
    path = tmp_path / "p.bin"
    w.save(path)
    f = pkg.host_api.WeightFile(host, path)
    m = host.matrix(n, 1, 1, 1, BF16)
    assert f.load_named(m, "P") == 0 and np.array_equal(m.download(np.uint16, n), oracle.f32_to_bf16(vals))
    m = host.matrix(n, 1, 1, 1, BF16)                                                 # HALF file into a BF16 tensor: converted on the host by truncation
    assert f.load_named(m, "Q") == 0 and m.dtype == BF16
    want = (vals.astype(np.float16).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    assert np.array_equal(m.download(np.uint16, n), want)
    m = host.matrix(n, 1, 1, 1, BF16)                                                 # FLOAT file: the tensor takes the file's type
    assert f.load_named(m, "R") == 0 and m.dtype == 0
    assert np.array_equal(m.download(np.float32, n), vals)


@pytest.fixture(scope="module")
def dec():
    from oracle import decode_oracle
    return decode_oracle


def make_model(pkg, host, cfg):
    return pkg.host_api.DecodeModel(host, cfg.layers, cfg.hidden, cfg.n_q, cfg.n_kv, cfg.head_dim, cfg.inter, cfg.vocab, cfg.t_kv)


def test_decode_model_from_an_fp8_file_equals_direct_tensors(tmp_path, gpu, pkg, host, dec):
    cfg = dec.DecodeConfig(layers=2, hidden=256, n_q=4, n_kv=2, inter=512, vocab=1000, t_kv=64)
    weights = dec.make_model(cfg, 21)
    path = tmp_path / "model_fp8.bin"
    pkg.weight_file.write_decode_model(path, weights, "fp8_e5m2")
    a, b = make_model(pkg, host, cfg), make_model(pkg, host, cfg)
    a.load(weights)
    b.load_named(pkg.host_api.WeightFile(host, path))
    for m in (a, b):
        m.reset(7, 0)
    for _ in range(5):
        assert a.step() == b.step()
    assert np.array_equal(a.logits(), b.logits())
    # a file without some tensor is refused with its name
    w = pkg.weight_file
    path2 = tmp_path / "broken.bin"
    full = w.read_index(path)[0]
    bw = w.BinWriter()
    for k in full:
        if k != "weight_fp8_e5m2_W_up_1":
            bw.add(k, w.read_entry(path, k))
    bw.save(path2)
    with pytest.raises(ValueError, match="W_up_1"):
        make_model(pkg, host, cfg).load_named(pkg.host_api.WeightFile(host, path2))


def test_decode_model_quantizes_a_bf16_file_on_load(tmp_path, gpu, pkg, host, oracle, dec):
    """BF16 linears are quantized on load with the reference's per-tensor rule: scale = absmax / 57344,
    codes = truncating E5M2 of w / scale (cccc/Matrix.cpp:301-355); the step then follows the oracle run on
    exactly those codes and scales."""
    cfg = dec.DecodeConfig(layers=1, hidden=256, n_q=4, n_kv=2, inter=512, vocab=500, t_kv=32)
    rng = np.random.default_rng(3)
    base = dec.make_model(cfg, 5)
    linears = {"wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down"}

    def bf16_weight(shape):
        return oracle.f32_to_bf16((rng.standard_normal(shape) * 0.02).astype(np.float32))

    file_model = {"emb": base["emb"], "rms_final": base["rms_final"], "lm_head": bf16_weight(base["lm_head"].shape),
                  "layers": [{k: (bf16_weight(v.shape) if k in linears else v) for k, v in base["layers"][0].items()}]}
    path = tmp_path / "model_bf16.bin"
    pkg.weight_file.write_decode_model(path, file_model, "bf16")
    model = make_model(pkg, host, cfg)
    model.load_named(pkg.host_api.WeightFile(host, path), E5M2)

    def quantize(bits):
        w = oracle.bf16_to_f32(bits)
        amax = np.float32(np.abs(w).max())
        fwd = np.float32(57344.0) / amax
        rc, codes = oracle.convert((w.reshape(-1)), 0, 5, w.size, float(fwd))
        assert rc == 0
        return codes.reshape(bits.shape), float(amax / np.float32(57344.0))

    q_model = {"emb": base["emb"], "rms_final": base["rms_final"], "layers": [dict(file_model["layers"][0])]}
    scales = {}
    q_model["lm_head"], scales["lm_head"] = quantize(file_model["lm_head"])
    for k in linears:
        q_model["layers"][0][k], scales[k] = quantize(file_model["layers"][0][k])
    # the device holds exactly these codes
    got = np.empty(q_model["lm_head"].size, dtype=np.uint8)
    import torch
    src = model.tensor_ptr(0, "lm_head")
    t = torch.empty(got.size, dtype=torch.uint8, device="cuda:0")
    assert pkg.library().convert(src, E5M2, t.data_ptr(), E5M2, got.size, 1.0) == 0
    assert np.array_equal(t.cpu().numpy(), q_model["lm_head"].reshape(-1))

    class ScaledOracle(dec.DecodeOracle):
        def deq(self, layer, name):
            W = self.model[name] if layer is None else self.model["layers"][layer][name]
            return oracle.dequant_fp8_to_bf16(W, oracle.E5M2, scales[name]).reshape(W.shape)

    orc = ScaledOracle(cfg, q_model)
    model.set_exact_attention(True)
    token = 3
    for pos in range(4):
        model.reset(token, pos)
        model.step()
        want_logits, token = orc.step(token, pos)
        got_logits = dec.f(model.logits())
        assert np.linalg.norm(got_logits - want_logits) <= 1e-2 * np.linalg.norm(want_logits), pos
