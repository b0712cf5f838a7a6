"""Pins the oracle's scalar formats against evidence that shares no code with it: torch's float8
and bfloat16 casts, the IEEE fp16 view of E5M2, the literal FP4 table, the reference's own
cccc/types.h compiled as oracle/_ref (when present), closed forms and brute force."""
import numpy as np
import pytest
import torch

ALL = np.arange(256, dtype=np.uint8)


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def test_e5m2_decode_matches_torch_and_fp16_view(oracle):
    tab = oracle.decode_table(oracle.E5M2)
    t = torch.from_numpy(ALL.copy()).view(torch.float8_e5m2).to(torch.float32).numpy()
    h = (ALL.astype(np.uint16) << 8).view(np.float16).astype(np.float32)
    ok = ~np.isnan(t)
    assert ok.sum() == 250
    assert np.array_equal(bits(tab[ok]), bits(t[ok]))
    assert np.array_equal(bits(tab[ok]), bits(h[ok]))
    # NaN rule of the reference: every NaN code -> +qNaN, sign dropped; Inf keeps its sign
    assert np.all(bits(tab[~ok]) == 0x7FC00000)
    assert bits(tab[0x7C:0x7D])[0] == 0x7F800000 and bits(tab[0xFC:0xFD])[0] == 0xFF800000
    # closed forms: subnormals m * 2^-16, max normal 57344
    assert tab[1] == 2.0 ** -16 and tab[3] == 3 * 2.0 ** -16 and tab[0x7B] == 57344.0 and tab[0x80 | 0x3C] == -1.0


def test_e4m3_decode_matches_torch(oracle):
    tab = oracle.decode_table(oracle.E4M3)
    t = torch.from_numpy(ALL.copy()).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    ok = ~np.isnan(t)
    assert ok.sum() == 254
    assert np.array_equal(bits(tab[ok]), bits(t[ok]))
    assert np.all(bits(tab[~ok]) == 0x7FC00000)
    assert tab[1] == 2.0 ** -9 and tab[0x7E] == 448.0 and tab[0x38] == 1.0 and tab[0x08] == 2.0 ** -6


def test_fp4_table_literal(oracle):
    tab = oracle.decode_table(oracle.FP4)[:16]
    want = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, 0, -.5, -1, -1.5, -2, -3, -4, -6], dtype=np.float32)
    assert np.array_equal(bits(tab), bits(want))     # code 8 is +0.0, not -0.0
    nib = np.array([0x21, 0xF8], dtype=np.uint8)
    assert list(oracle.unpack_fp4(nib, 4)) == [1, 2, 8, 15]    # low nibble = even element


def test_golden_tables(oracle, golden_tables):
    g = golden_tables
    assert np.array_equal(bits(oracle.decode_table(oracle.E5M2)), g["e5m2_f32_bits"])
    assert np.array_equal(bits(oracle.decode_table(oracle.E4M3)), g["e4m3_f32_bits"])
    for i, s in enumerate(g["scales"]):
        assert np.array_equal(oracle.dequant_fp8_to_bf16(ALL, oracle.E5M2, float(s)), g["e5m2_bf16"][i]), s
        assert np.array_equal(oracle.dequant_fp8_to_bf16(ALL, oracle.E4M3, float(s)), g["e4m3_bf16"][i]), s
        nib = (np.arange(16, dtype=np.uint8)[0::2] | (np.arange(16, dtype=np.uint8)[1::2] << 4)).astype(np.uint8)
        assert np.array_equal(oracle.dequant_fp4_to_bf16(nib, 16, float(s)), g["fp4_bf16"][i]), s
        # the scalar C convert agrees with the vectorised form
        rc, c = oracle.convert(ALL, oracle.E5M2, oracle.BF16, 256, float(s))
        assert rc == 0 and np.array_equal(c, g["e5m2_bf16"][i])
        rc, c = oracle.convert(ALL, oracle.E4M3, oracle.BF16, 256, float(s))
        assert rc == 0 and np.array_equal(c, g["e4m3_bf16"][i])


def test_golden_blockscale_all_products(oracle, golden_tables):
    want = golden_tables["blockscale_bf16"]            # [scale byte][nibble]
    # one block of 16 elements per scale byte holding nibbles 0..15
    nib = np.tile((np.arange(16, dtype=np.uint8)[0::2] | (np.arange(16, dtype=np.uint8)[1::2] << 4)).astype(np.uint8), 256)
    got = oracle.dequant_fp4_blockscale_to_bf16(nib, ALL, 256 * 16, 16).reshape(256, 16)
    assert np.array_equal(got, want)
    out = np.zeros(256 * 16, dtype=np.uint16)
    rc = oracle.lib().orc_fp4_blockscale_to_bf16(nib.ctypes.data, ALL.ctypes.data, out.ctypes.data, 256 * 16, 16)
    assert rc == 0 and np.array_equal(out.reshape(256, 16), want)
    # invariant: fp4 * e4m3 needs at most 6 significant bits, so the BF16 rounding is exact
    t4 = oracle.decode_table(oracle.FP4)[:16].astype(np.float64)
    t8 = oracle.decode_table(oracle.E4M3).astype(np.float64)
    exact = t8[:, None] * t4[None, :]
    fin = np.isfinite(exact)
    assert np.array_equal(oracle.bf16_to_f32(got)[fin].astype(np.float64), exact[fin])


def test_bf16_rounding_is_rne(oracle):
    rng = np.random.default_rng(7)
    x = np.concatenate([rng.standard_normal(200000).astype(np.float32) * np.float32(10.0) ** rng.integers(-30, 30, 200000).astype(np.float32),
                        np.array([1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, 3.3895314e38, np.inf, -np.inf, 0.0, -0.0, 1e-40], dtype=np.float32)])
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(oracle.f32_to_bf16(x), want)
    got_c = np.array([oracle.lib().orc_f32_to_bf16_rne(float(v)) for v in x[:2000]], dtype=np.uint16)
    assert np.array_equal(got_c, want[:2000])
    # ties go to even: 1 + 2^-8 -> 1.0 (0x3F80), 1 + 3*2^-8 -> 1 + 2^-6 (0x3F82)
    assert oracle.f32_to_bf16(np.array([1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8], dtype=np.float32)).tolist() == [0x3F80, 0x3F82]


def test_power_of_two_scale_is_exact(oracle):
    tab = oracle.decode_table(oracle.E5M2).astype(np.float64)
    fin = np.isfinite(tab)
    for k in (-7, -3, 1, 5):
        got = oracle.bf16_to_f32(oracle.dequant_fp8_to_bf16(ALL, oracle.E5M2, 2.0 ** k)).astype(np.float64)
        assert np.array_equal(got[fin], tab[fin] * 2.0 ** k)


def test_half_conversions_match_numpy(oracle):
    rng = np.random.default_rng(3)
    x = np.concatenate([rng.standard_normal(20000).astype(np.float32) * np.float32(2.0) ** rng.integers(-30, 18, 20000).astype(np.float32),
                        np.array([65504.0, 65519.9, 65520.0, 70000.0, 2.0 ** -24, 2.0 ** -25, 1.5 * 2.0 ** -25, 0.0, -0.0, np.inf], dtype=np.float32)])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = np.array([oracle.lib().orc_f32_to_half_rne(float(v)) for v in x], dtype=np.uint16)
    assert np.array_equal(got, want)
    allh = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    back = np.array([oracle.lib().orc_half_to_float(int(h)) for h in allh[::7]], dtype=np.float32)
    ref = allh[::7].view(np.float16).astype(np.float32)
    ok = ~np.isnan(ref)
    assert np.array_equal(bits(back[ok]), bits(ref[ok])) and np.all(np.isnan(back[~ok]))


def test_e5m2_rne_encoder_matches_torch(oracle):
    rng = np.random.default_rng(11)
    x = np.concatenate([(rng.standard_normal(300000) * 0.02).astype(np.float32),
                        rng.standard_normal(100000).astype(np.float32) * np.float32(2.0) ** rng.integers(-22, 18, 100000).astype(np.float32),
                        np.array([1.49, 1.375, 1.125, 57344.0, 61439.0, 61440.0, 65536.0, 2.0 ** -17, 1.0001 * 2.0 ** -17, 0.0, -0.0, np.inf, -np.inf], dtype=np.float32)])
    want = torch.from_numpy(x).to(torch.float8_e5m2).view(torch.uint8).numpy()
    got = oracle.encode_e5m2_rne(x)
    assert np.array_equal(got, want)
    # every code round-trips
    tab = oracle.decode_table(oracle.E5M2)
    fin = np.isfinite(tab)
    rt = oracle.encode_e5m2_rne(tab[fin])
    assert np.array_equal(rt & 0x7F, ALL[fin] & 0x7F)


def test_e4m3_rne_encoder_matches_torch(oracle):
    rng = np.random.default_rng(12)
    x = np.concatenate([(np.abs(rng.standard_normal(200000)) * 0.01).astype(np.float32),
                        rng.standard_normal(100000).astype(np.float32) * np.float32(2.0) ** rng.integers(-14, 9, 100000).astype(np.float32),
                        np.array([0.0075, 448.0, 463.9, 1.0, 2.0 ** -10, 3 * 2.0 ** -10, 0.0], dtype=np.float32)])
    want = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = oracle.encode_e4m3_rne(x)
    assert np.array_equal(got, want)


def test_truncating_encoders_brute_force(oracle):
    """Closed form of a truncating encoder: the code whose value is the largest representable
    magnitude <= |x| (saturating).  Checked by brute force over the decode tables."""
    L = oracle.lib()
    rng = np.random.default_rng(5)
    for enc, dtype, top in ((L.orc_float_to_e5m2_trunc, oracle.E5M2, 0x7B), (L.orc_float_to_e4m3_trunc, oracle.E4M3, 0x7E)):
        tab = oracle.decode_table(dtype)[: top + 1].astype(np.float64)       # non-negative finite codes, increasing
        xs = np.concatenate([rng.standard_normal(3000) * 2.0 ** rng.integers(-20, 17, 3000), tab, tab * 1.01, tab * 0.99, [1e9, -1e9]])
        for v in xs.astype(np.float32):
            code = enc(float(v), 1.0)
            want = int(np.searchsorted(tab, abs(np.float64(v)), side="right") - 1)
            want = max(want, 0) | (0x80 if np.signbit(v) else 0)
            assert code == want, (float(v), hex(code), hex(want))
    assert L.orc_float_to_e5m2_trunc(1.49, 1.0) == 0x3D          # the reference truncates (RNE would give 0x3E)
    assert L.orc_float_to_e5m2_trunc(float("nan"), 1.0) == 0x7C and L.orc_float_to_e4m3_trunc(float("nan"), 1.0) == 0x7F
    assert L.orc_float_to_e5m2_trunc(float("inf"), 1.0) == 0x7C and L.orc_float_to_e5m2_trunc(float("-inf"), 1.0) == 0xFC
    assert L.orc_float_to_e4m3_trunc(3.0, 100.0) == 0x79         # value * scale is what gets encoded: 300 -> 288


def test_fp4_encoder_thresholds(oracle):
    L = oracle.lib()
    for v, code in ((0.0, 0), (0.2499, 0), (0.25, 1), (0.75, 2), (1.25, 3), (1.75, 4), (2.5, 5), (3.5, 6), (5.0, 7), (100.0, 7), (-0.25, 9), (-6.0, 15), (-0.0, 0)):
        assert L.orc_float_to_fp4(v) == code, v


def test_against_reference_types_header(oracle):
    R = oracle.ref()
    if R is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    L = oracle.lib()
    for b in range(256):
        for mine, theirs in ((L.orc_e5m2_to_float, R.ref_e5m2_to_float), (L.orc_e4m3_to_float, R.ref_e4m3_to_float)):
            a, r = np.float32(mine(b)), np.float32(theirs(b))
            assert a.view(np.uint32) == r.view(np.uint32), b
    for n in range(16):
        assert np.float32(L.orc_fp4_to_float(n)).view(np.uint32) == np.float32(R.ref_fp4_to_float(n)).view(np.uint32)
    buf = np.array([0x21, 0xF8], dtype=np.uint8)
    assert [R.ref_fp4_get(buf.ctypes.data, i) for i in range(4)] == [0.5, 1.0, 0.0, -6.0]
    rng = np.random.default_rng(9)
    xs = np.concatenate([rng.standard_normal(20000) * 2.0 ** rng.integers(-24, 18, 20000), [0.0, -0.0, 1.49, 448.0, 57344.0, 1e9, -1e9, np.inf, -np.inf, np.nan]]).astype(np.float32)
    for v in xs:
        v = float(v)
        assert L.orc_float_to_e5m2_trunc(v, 1.0) == R.ref_float_to_e5m2(v), v
        assert L.orc_float_to_e4m3_trunc(v, 1.0) == R.ref_float_to_e4m3(v), v
        if v == v:
            assert L.orc_float_to_fp4(v) == R.ref_float_to_fp4(v), v
