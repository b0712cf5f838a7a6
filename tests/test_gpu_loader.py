"""Loading converted model files into the host mirror: WeightFile::loadNamed into a Matrix and
DecodeModel::loadNamedWeights, against tensors set directly and against the CPU oracle."""
import struct

import numpy as np
from oracle import synth, weight_file
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
    w = weight_file.BinWriter()
    codes8 = oracle.encode_e5m2_rne((rng.standard_normal((n_out, K)) * 0.02).astype(np.float32))
    w.add("weight_fp8_e5m2_W_a", codes8); w.add_float("scale_W_a", 0.5); w.add_float("input_scale_W_a", 0.25)
    w.add("weight_W_legacy", codes8 & 0x7E)                                           # legacy key: FP8_E4M3, no scale entry -> 1.0
    nib, sc = synth.pack_fp4_blockscale((rng.standard_normal((n_out, K)) * 0.02).astype(np.float32), 16)
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
    w = weight_file.BinWriter()
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
    weight_file.write_decode_model(path, weights, "fp8_e5m2")
    a, b = make_model(pkg, host, cfg), make_model(pkg, host, cfg)
    a.load(weights)
    b.load_named(pkg.host_api.WeightFile(host, path))
    for m in (a, b):
        m.reset(7, 0)
    for _ in range(5):
        assert a.step() == b.step()
    assert np.array_equal(a.logits(), b.logits())
    # a file without some tensor is refused with its name
    w = weight_file
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
    weight_file.write_decode_model(path, file_model, "bf16")
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


def test_quantize_on_load_then_save_then_reload_is_identical(tmp_path, gpu, pkg, host, oracle, dec):
    """The weight_data_type + save_fp8_file route (cccc/MainProcess.cpp:362-378): a BF16 file is quantized on load,
    DecodeModel::saveNamedWeights writes the cache, and a second model loaded from the cache holds the same bytes and
    scales and decodes the same tokens without quantizing anything."""
    cfg = dec.DecodeConfig(layers=2, hidden=256, n_q=4, n_kv=2, inter=512, vocab=500, t_kv=32)
    rng = np.random.default_rng(9)
    base = dec.make_model(cfg, 6)
    linears = {"wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down"}
    bf16_weight = lambda shape: oracle.f32_to_bf16((rng.standard_normal(shape) * 0.02).astype(np.float32))
    file_model = {"emb": base["emb"], "rms_final": base["rms_final"], "lm_head": bf16_weight(base["lm_head"].shape),
                  "layers": [{k: (bf16_weight(v.shape) if k in linears else v) for k, v in L.items()} for L in base["layers"]]}
    src = tmp_path / "model_bf16.bin"
    weight_file.write_decode_model(src, file_model, "bf16")
    a = make_model(pkg, host, cfg)
    a.load_named(pkg.host_api.WeightFile(host, src), E5M2)
    cache = tmp_path / "cache_fp8.bin"
    a.save_named(cache)

    # what the cache holds: header, typed keys, one float32 scale per quantized tensor, raw sizes
    index, _ = weight_file.read_index(cache)
    assert list(index)[:2] == ["data_type", "named_weights"] and weight_file.read_entry(cache, "data_type") == b"fp8_e5m2"
    assert index["weight_bf16_W_emb"][1] == cfg.vocab * cfg.hidden * 2
    assert index["weight_fp8_e5m2_W_lm_head"][1] == cfg.vocab * cfg.hidden and index["scale_W_lm_head"][1] == 4
    for i in range(cfg.layers):
        for name, n in (("W_q", cfg.q_out * cfg.hidden), ("W_k", cfg.kv_out * cfg.hidden), ("W_down", cfg.hidden * cfg.inter)):
            assert index[f"weight_fp8_e5m2_{name}_{i}"][1] == n and index[f"scale_{name}_{i}"][1] == 4
        assert index[f"weight_bf16_W_rms_attn_{i}"][1] == cfg.hidden * 2 and f"scale_W_rms_attn_{i}" not in index
    # the saved scale is absmax / 57344 of the BF16 tensor, the saved codes its truncating quantization
    w = oracle.bf16_to_f32(file_model["layers"][1]["w_down"])
    amax = np.float32(np.abs(w).max())
    assert struct.unpack("<f", weight_file.read_entry(cache, "scale_W_down_1"))[0] == np.float32(amax / np.float32(57344.0))
    rc, codes = oracle.convert(w.reshape(-1), 0, 5, w.size, float(np.float32(57344.0) / amax))
    assert rc == 0 and weight_file.read_entry(cache, "weight_fp8_e5m2_W_down_1") == codes.tobytes()

    b = make_model(pkg, host, cfg)
    b.load_named(pkg.host_api.WeightFile(host, cache), E5M2)
    recache = tmp_path / "cache_again.bin"
    b.save_named(recache)
    assert cache.read_bytes() == recache.read_bytes()                     # same bytes, same scales, same order
    for m in (a, b):
        m.reset(11, 0)
    for _ in range(6):
        assert a.step() == b.step()
    assert np.array_equal(a.logits(), b.logits())


def test_fp4_matrix_saves_packed_codes_and_block_scales(tmp_path, gpu, pkg, host, oracle):
    """quantizeWeights(FP4) on the device, then the named-weight writer: packed nibbles sized (elements + 1) / 2,
    one E4M3 byte per 16 elements, both equal to the oracle's on-the-fly quantiser; reloading gives the same GEMV."""
    K, n_out = 256, 80
    w = synth.weights_f32(41, n_out, K)
    m = host.matrix(K, n_out, 1, 1, BF16)
    m.upload(oracle.f32_to_bf16(w))
    m.quantize(FP4)
    assert m.dtype == FP4
    path = tmp_path / "fp4.bin"
    m.save_named("W_x", path)
    index, _ = weight_file.read_index(path)
    assert index["weight_fp4_e2m1_W_x"][1] == n_out * K // 2 and index["blockscale_W_x"][1] == n_out * K // 16 and "scale_W_x" not in index
    nib, sc = oracle.quantize_fp4_blockscale_kernel(w, 16)
    assert weight_file.read_entry(path, "weight_fp4_e2m1_W_x") == nib.tobytes()
    assert weight_file.read_entry(path, "blockscale_W_x") == sc.tobytes()
    back = host.matrix(K, n_out, 1, 1, BF16)
    assert pkg.host_api.WeightFile(host, path).load_named(back, "W_x") == 0 and back.dtype == FP4
    x = synth.activations(41, 1, K)[0]
    assert np.array_equal(linear_out(pkg, host, m, x, n_out, K), linear_out(pkg, host, back, x, n_out, K))


def test_mixed_fp8_formats_in_one_file(tmp_path, gpu, pkg, host, oracle, dec):
    """k stored as FP8_E4M3 with a scale next to E5M2 q and v: the step decodes each projection with its own format
    (three launches instead of one).  Gate and up in two formats likewise: every tensor keeps the format the file gives
    it (cccc/Net.cpp:1444-1481), the step runs the two linears and the SwiGLU product as launches of their own, and the
    prompt phase takes its separate calls."""
    cfg = dec.DecodeConfig(layers=1, hidden=256, n_q=4, n_kv=2, inter=512, vocab=300, t_kv=16)
    weights = dec.make_model(cfg, 31)
    path = tmp_path / "mixed.bin"
    weight_file.write_decode_model(path, weights, "fp8_e5m2")
    wk_f32 = oracle.decode_table(oracle.E5M2)[weights["layers"][0]["wk"]]
    scale = float(np.abs(wk_f32).max()) / 448.0
    wk_e4m3 = oracle.encode_e4m3_rne((wk_f32 / np.float32(scale)).astype(np.float32))

    def rewrite(replace_key, new_key, codes, scale_key):
        bw = weight_file.BinWriter()
        for k in weight_file.read_index(path)[0]:
            if k == replace_key:
                bw.add(new_key, codes)
                bw.add_float(scale_key, scale)
            else:
                bw.add(k, weight_file.read_entry(path, k))
        out = tmp_path / (new_key + ".bin")
        bw.save(out)
        return out

    mixed = rewrite("weight_fp8_e5m2_W_k_0", "weight_fp8_e4m3_W_k_0", wk_e4m3, "scale_W_k_0")
    model = make_model(pkg, host, cfg)
    model.load_named(pkg.host_api.WeightFile(host, mixed))
    model.set_exact_attention(True)

    class MixedOracle(dec.DecodeOracle):
        def deq(self, layer, name):
            if name == "wk":
                return oracle.dequant_fp8_to_bf16(wk_e4m3, oracle.E4M3, scale).reshape(wk_e4m3.shape)
            return super().deq(layer, name)

    orc = MixedOracle(cfg, weights)
    token = 4
    for pos in range(3):
        model.reset(token, pos)
        model.step()
        want_logits, token = orc.step(token, pos)
        got = dec.f(model.logits())
        assert np.linalg.norm(got - want_logits) <= 1e-2 * np.linalg.norm(want_logits), pos
    up_f32 = oracle.decode_table(oracle.E5M2)[weights["layers"][0]["w_up"]]
    up_scale = float(np.abs(up_f32).max()) / 448.0
    up_e4m3 = oracle.encode_e4m3_rne((up_f32 / np.float32(up_scale)).astype(np.float32))
    scale = up_scale
    both = rewrite("weight_fp8_e5m2_W_up_0", "weight_fp8_e4m3_W_up_0", up_e4m3, "scale_W_up_0")

    class MixedUpOracle(dec.DecodeOracle):
        def deq(self, layer, name):
            if name == "w_up":
                return oracle.dequant_fp8_to_bf16(up_e4m3, oracle.E4M3, up_scale).reshape(up_e4m3.shape)
            return super().deq(layer, name)

    model = make_model(pkg, host, cfg)
    model.load_named(pkg.host_api.WeightFile(host, both))
    model.set_exact_attention(True)
    orc = MixedUpOracle(cfg, weights)
    token = 4
    for pos in range(3):
        model.reset(token, pos)
        model.step()
        want_logits, token = orc.step(token, pos)
        got = dec.f(model.logits())
        assert np.linalg.norm(got - want_logits) <= 1e-2 * np.linalg.norm(want_logits), pos
        gated = dec.f(model.activation("gated"))
        assert np.isfinite(gated).all()
    # the prompt phase of the same model (separate gate / up calls), then a step behind it
    orc = MixedUpOracle(cfg, weights)
    prompt = [5, 17, 250, 3, 9, 11]
    for pos, tok in enumerate(prompt):
        want_logits, want_next = orc.step(tok, pos)
    model.prefill(prompt)
    got = dec.f(model.logits())
    assert np.linalg.norm(got - want_logits) <= 1e-2 * np.linalg.norm(want_logits)


def test_decode_model_from_an_fp4_file(tmp_path, gpu, pkg, host, oracle, dec):
    """weight_fp4_e2m1_<name> + blockscale_<name> entries, as the converter writes a Llama FP4 model
    (scripts/convert_weights.py:318-392): loading them gives the same steps as tensors set directly, and
    saveNamedWeights writes the same entries back."""
    cfg = dec.DecodeConfig(layers=1, hidden=256, n_q=4, n_kv=2, inter=512, vocab=400, t_kv=16)
    weights = dec.make_model(cfg, 23, fmt="fp4_e2m1")
    names = {"rms_attn": "W_rms_attn", "wq": "W_q", "wk": "W_k", "wv": "W_v", "q_norm": "W_qnorm", "k_norm": "W_knorm", "wo": "W_o",
             "rms_ffn": "W_rms_ffn", "w_gate": "W_gate", "w_up": "W_up", "w_down": "W_down"}
    w = weight_file.BinWriter()
    w.add("data_type", b"fp4_e2m1")
    w.add("named_weights", b"1")

    def put(name, value):
        if isinstance(value, tuple):
            w.add(f"weight_fp4_e2m1_{name}", value[0])
            w.add(f"blockscale_{name}", value[1])
        else:
            w.add(f"weight_bf16_{name}", value)

    put("W_emb", weights["emb"]); put("W_rms_final", weights["rms_final"]); put("W_lm_head", weights["lm_head"])
    for short, value in weights["layers"][0].items():
        put(f"{names[short]}_0", value)
    path = tmp_path / "model_fp4.bin"
    w.save(path)
    a, b = make_model(pkg, host, cfg), make_model(pkg, host, cfg)
    a.load(weights)
    b.load_named(pkg.host_api.WeightFile(host, path))
    for m in (a, b):
        m.reset(7, 0)
    for _ in range(5):
        assert a.step() == b.step()
    assert np.array_equal(a.logits(), b.logits())
    again = tmp_path / "model_fp4_again.bin"
    b.save_named(again)
    for key in weight_file.read_index(path)[0]:
        assert weight_file.read_entry(again, key) == weight_file.read_entry(path, key), key
    # an FP4 linear without its block scales cannot run on the fused kernels: refused by name
    bw = weight_file.BinWriter()
    for key in weight_file.read_index(path)[0]:
        if key != "blockscale_W_o_0":
            bw.add(key, weight_file.read_entry(path, key))
    broken = tmp_path / "model_fp4_noscale.bin"
    bw.save(broken)
    with pytest.raises(ValueError, match="W_o_0"):
        make_model(pkg, host, cfg).load_named(pkg.host_api.WeightFile(host, broken))


@pytest.mark.parametrize("fmt", ["fp8_e5m2", "fp4_e2m1"])
def test_projections_sharing_an_input_load_into_one_storage(tmp_path, gpu, pkg, host, oracle, fmt):
    """q, k, v of one layer in ONE storage (WeightFile::loadNamedGroup): a single GEMV on it gives the three
    projections back to back, bit for bit what three separately loaded weights give, and Matrix::rowsView hands
    each projection out as a tensor of its own (codes, and for FP4 the block scales, at the right offsets)."""
    torch, dev, lib = gpu
    rng = np.random.default_rng(12)
    K, rows = 1024, (512, 128, 128)
    names = ("W_q_0", "W_k_0", "W_v_0")
    w = weight_file.BinWriter()
    packed = []
    for name, n in zip(names, rows):
        wf = (rng.standard_normal((n, K)) * 0.02).astype(np.float32)
        if fmt == "fp4_e2m1":
            nib, sc = synth.pack_fp4_blockscale(wf, 16)
            w.add(f"weight_fp4_e2m1_{name}", nib); w.add(f"blockscale_{name}", sc)
            packed.append((nib, sc))
        else:
            codes = oracle.encode_e5m2_rne(wf)
            w.add(f"weight_fp8_e5m2_{name}", codes)
            packed.append((codes, None))
    w.add("weight_fp8_e4m3_W_other", np.zeros((128, K), np.uint8))
    w.add("weight_fp8_e5m2_W_scaled", np.zeros((128, K), np.uint8)); w.add_float("scale_W_scaled", 0.5)
    path = tmp_path / "group.bin"
    w.save(path)
    f = pkg.host_api.WeightFile(host, path)
    dtype = FP4 if fmt == "fp4_e2m1" else E5M2

    total = sum(rows)
    group = host.matrix(K, total, 1, 1, BF16)
    assert f.load_named_group(group, names) == 0 and group.dtype == dtype
    for tokens in (1, 4):
        X = synth.activations(70 + tokens, tokens, K)
        xm = host.matrix(K, tokens, 1, 1, BF16); xm.upload(X)
        y_all = host.matrix(total, tokens, 1, 1, BF16)
        assert pkg.host_api.mul_batched(group, xm, y_all, ta=1, tb=0) == 0
        got = y_all.download(np.uint16, tokens * total).reshape(tokens, total)
        row0 = 0
        for name, n, (codes, sc) in zip(names, rows, packed):
            single = host.matrix(K, n, 1, 1, BF16)
            assert f.load_named(single, name) == 0
            y1 = host.matrix(n, tokens, 1, 1, BF16)
            assert pkg.host_api.mul_batched(single, xm, y1, ta=1, tb=0) == 0
            want_bits = y1.download(np.uint16, tokens * n).reshape(tokens, n)
            Wd = oracle.dequant_weight(codes, oracle.FP4 if sc is not None else oracle.E5M2, n, K, blk_sc=sc)
            check_rows(oracle.bf16_to_f32(got[:, row0:row0 + n]).astype(np.float64), oracle.linear_exact(Wd, X), name)
            assert np.abs(oracle.bf16_to_f32(got[:, row0:row0 + n]).astype(np.float64) - oracle.bf16_to_f32(want_bits).astype(np.float64)).max() \
                <= 2.0 ** -7 * np.abs(oracle.bf16_to_f32(want_bits)).max()
            # the projection as a tensor of its own on the shared storage
            view = group.rows_view(row0, n)
            assert view.dtype == dtype and view.data_ptr == group.data_ptr + (row0 * K // 2 if sc is not None else row0 * K)
            yv = host.matrix(n, tokens, 1, 1, BF16)
            assert pkg.host_api.mul_batched(view, xm, yv, ta=1, tb=0) == 0
            check_rows(oracle.bf16_to_f32(yv.download(np.uint16, tokens * n).reshape(tokens, n)).astype(np.float64), oracle.linear_exact(Wd, X), name + " view")
            row0 += n
    # A row view saved under a name of its own holds exactly its rows: codes, and for FP4 the block scales of those rows
    # (not the storage's whole scale array); a view can neither replace the storage's scales nor build a tiled copy.
    row0 = rows[0]
    view = group.rows_view(row0, rows[1])
    saved = tmp_path / f"view_{fmt}.bin"
    view.save_named("W_k_0", saved)
    codes, sc = packed[1]
    key = "weight_fp4_e2m1_W_k_0" if sc is not None else "weight_fp8_e5m2_W_k_0"
    assert weight_file.read_entry(saved, key) == codes.tobytes()
    if sc is not None:
        assert weight_file.read_entry(saved, "blockscale_W_k_0") == sc.tobytes()
        assert np.array_equal(view.block_scales(), sc.ravel())
        all_scales = group.block_scales()
        view.set_block_scale(np.zeros(sc.size, np.uint8))          # ignored on a view
        assert np.array_equal(group.block_scales(), all_scales)
    had = group.prepare_tiled()
    assert view.prepare_tiled() == had                              # (reports the storage's copy; builds none of its own)
    # members of different types or scales, a missing name, a storage of the wrong size
    if fmt == "fp8_e5m2":
        assert f.load_named_group(host.matrix(K, 512 + 128, 1, 1, BF16), ("W_q_0", "W_other")) == -1
        assert f.load_named_group(host.matrix(K, 512 + 128, 1, 1, BF16), ("W_q_0", "W_scaled")) == -1
    assert f.load_named_group(host.matrix(K, total, 1, 1, BF16), ("W_q_0", "W_k_0", "W_nope")) == 1
    assert f.load_named_group(host.matrix(K, total + 16, 1, 1, BF16), names) == -1
    with pytest.raises(ValueError):
        group.rows_view(total - 8, 16)


def test_a_file_without_qk_norm_weights_loads_as_a_model_without_them(tmp_path, gpu, pkg, host, oracle, dec):
    """The converter writes no W_qnorm / W_knorm for Llama (scripts/convert_weights.py:195-216): such a file loads, runs the
    steps of the same tensors set directly with the per-head norm switched off, and is saved back without those entries."""
    cfg = dec.DecodeConfig(layers=2, hidden=256, n_q=4, n_kv=2, inter=512, vocab=400, t_kv=16, theta=5e5)
    weights = dec.make_model(cfg, 37, fmt="fp4_e2m1", qk_norm=False)
    names = {"rms_attn": "W_rms_attn", "wq": "W_q", "wk": "W_k", "wv": "W_v", "wo": "W_o",
             "rms_ffn": "W_rms_ffn", "w_gate": "W_gate", "w_up": "W_up", "w_down": "W_down"}
    w = weight_file.BinWriter()
    w.add("data_type", b"fp4_e2m1")
    w.add("named_weights", b"1")

    def put(name, value):
        if isinstance(value, tuple):
            w.add(f"weight_fp4_e2m1_{name}", value[0])
            w.add(f"blockscale_{name}", value[1])
        else:
            w.add(f"weight_bf16_{name}", value)

    put("W_emb", weights["emb"]); put("W_rms_final", weights["rms_final"]); put("W_lm_head", weights["lm_head"])
    for li, L in enumerate(weights["layers"]):
        for short, value in L.items():
            put(f"{names[short]}_{li}", value)
    path = tmp_path / "llama_like.bin"
    w.save(path)

    def fresh():
        return pkg.host_api.DecodeModel(host, cfg.layers, cfg.hidden, cfg.n_q, cfg.n_kv, cfg.head_dim, cfg.inter, cfg.vocab, cfg.t_kv, theta=cfg.theta)

    a, b = fresh(), fresh()
    a.load(weights)
    assert b.qk_norm
    b.load_named(pkg.host_api.WeightFile(host, path))
    assert not a.qk_norm and not b.qk_norm
    for m in (a, b):
        m.reset(7, 0)
    for _ in range(5):
        assert a.step() == b.step()
    assert np.array_equal(a.logits(), b.logits())
    again = tmp_path / "llama_like_again.bin"
    b.save_named(again)
    keys = weight_file.read_index(again)[0]
    assert not any("norm_" in k and ("qnorm" in k or "knorm" in k) for k in keys)
    for key in weight_file.read_index(path)[0]:
        assert weight_file.read_entry(again, key) == weight_file.read_entry(path, key), key


def test_a_file_without_lm_head_loads_with_tied_embeddings(tmp_path, gpu, pkg, host, oracle, dec):
    """tie_word_embeddings: the converter writes no W_lm_head (scripts/convert_weights.py:256-260).  The model then multiplies
    by the BF16 embedding table (cccc/Net.cpp:1158-1190 keeps EMBED tables unquantized), steps as the same tensors set
    directly, and is saved back without a head entry."""
    cfg = dec.DecodeConfig(layers=1, hidden=256, n_q=4, n_kv=2, inter=512, vocab=400, t_kv=16)
    weights = dec.make_model(cfg, 47, tied=True)
    names = {"rms_attn": "W_rms_attn", "wq": "W_q", "wk": "W_k", "wv": "W_v", "q_norm": "W_qnorm", "k_norm": "W_knorm", "wo": "W_o",
             "rms_ffn": "W_rms_ffn", "w_gate": "W_gate", "w_up": "W_up", "w_down": "W_down"}
    w = weight_file.BinWriter()
    w.add("data_type", b"fp8_e5m2")
    w.add("named_weights", b"1")
    w.add("weight_bf16_W_emb", weights["emb"])
    w.add("weight_bf16_W_rms_final", weights["rms_final"])
    for short, value in weights["layers"][0].items():
        w.add(("weight_fp8_e5m2_" if value.dtype == np.uint8 else "weight_bf16_") + f"{names[short]}_0", value)
    path = tmp_path / "tied.bin"
    w.save(path)
    a, b = make_model(pkg, host, cfg), make_model(pkg, host, cfg)
    a.load(weights)
    assert not b.tied_lm_head
    b.load_named(pkg.host_api.WeightFile(host, path))
    assert a.tied_lm_head and b.tied_lm_head
    for m in (a, b):
        m.reset(7, 0)
    for _ in range(5):
        assert a.step() == b.step()
    assert np.array_equal(a.logits(), b.logits())
    again = tmp_path / "tied_again.bin"
    b.save_named(again)
    keys = weight_file.read_index(again)[0]
    assert not any("W_lm_head" in k for k in keys)
    for key in weight_file.read_index(path)[0]:
        assert weight_file.read_entry(again, key) == weight_file.read_entry(path, key), key
