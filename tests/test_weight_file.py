"""The CFG_BIN INI container reader of the host library (host/WeightFile.cpp) and its name-resolution
rules, on files written by oracle/weight_file.py in the converter's layout
(scripts/convert_weights.py:54-83).  Host code only: no GPU call is made."""
import struct

import numpy as np
from oracle import weight_file
import pytest


@pytest.fixture(scope="module")
def host(pkg):
    return pkg.host_api.host()


def test_container_round_trip_and_key_order(tmp_path, pkg, host):
    wf_mod = weight_file
    w = wf_mod.BinWriter()
    rng = np.random.default_rng(0)
    blobs = {"data_type": b"fp8_e4m3", "named_weights": b"1", "weight_fp8_e5m2_W_q_0": rng.integers(0, 255, 4096, dtype=np.uint8),
             "scale_W_q_0": struct.pack("<f", 0.125), "weight_bf16_W_rms_attn_0": rng.integers(0, 65535, 64, dtype=np.uint16), "empty": b""}
    for k, v in blobs.items():
        w.add(k, v)
    path = tmp_path / "m.bin"
    total = w.save(path)
    assert path.stat().st_size == total
    raw = path.read_bytes()
    assert raw[:11] == b"CFG_BIN INI" and raw[11:32] == bytes(21)                 # the converter's header
    (ini_len,) = struct.unpack("<Q", raw[32:40])
    assert raw[40:40 + ini_len].decode("ascii").splitlines()[0] == "data_type = 0,8"
    f = pkg.host_api.WeightFile(host, path)
    assert f.keys() == list(blobs)
    for k, v in blobs.items():
        want = v.tobytes() if isinstance(v, np.ndarray) else v
        assert f.get(k) == want == wf_mod.read_entry(path, k)
    assert f.get("missing") is None
    f.close()


def test_name_resolution_follows_the_reference_order(tmp_path, pkg, host):
    D = pkg.DataType
    w = weight_file.BinWriter()
    one = np.zeros(16, dtype=np.uint8)
    w.add("weight_bf16_A", one); w.add("weight_fp8_e5m2_A", one)          # a quantized typed key is found through the suffix list in its order
    w.add("weight_half_B", one); w.add("weight_B", one)                   # legacy untyped key beats a plain typed key
    w.add("weight_fp8_C", one); w.add("weight_fp8_e5m2_C", one)           # "fp8" comes before "fp8_e5m2" in the list
    w.add("weight_float_D", one)
    w.add("weight_fp4_e2m1_E", one); w.add("weight_bfloat16_E", one)      # bf16 aliases come before fp4 in the list: the plain key is what is found
    w.add("weight_fp4_e2m1_F", one)
    w.add("weight_G", one)
    path = tmp_path / "r.bin"
    w.save(path)
    f = pkg.host_api.WeightFile(host, path)
    assert f.resolve("A") == ("weight_bf16_A", D.BFLOAT16, False)          # first suffix that exists is bf16 -> not quantized, no legacy key
    assert f.resolve("B") == ("weight_B", D.FP8_E4M3, True)
    assert f.resolve("C") == ("weight_fp8_C", D.FP8_E4M3, True)
    assert f.resolve("D") == ("weight_float_D", D.FLOAT, False)
    assert f.resolve("E") == ("weight_bfloat16_E", D.BFLOAT16, False)
    assert f.resolve("F") == ("weight_fp4_e2m1_F", D.FP4_E2M1, True)
    assert f.resolve("G") == ("weight_G", D.FP8_E4M3, True)
    assert f.resolve("H") is None


def test_malformed_files_are_refused(tmp_path, pkg, host):
    good = tmp_path / "g.bin"
    w = weight_file.BinWriter()
    w.add("k", b"12345678")
    w.save(good)
    raw = bytearray(good.read_bytes())

    def status_of(data, name):
        p = tmp_path / name
        p.write_bytes(bytes(data))
        with pytest.raises(OSError) as e:
            pkg.host_api.WeightFile(host, p)
        return int(str(e.value).rsplit(" ", 1)[1])

    assert status_of(b"short", "a.bin") == -2
    assert status_of(b"NOT_A_BIN XX" + bytes(raw[12:]), "b.bin") == -2
    bad_len = bytearray(raw); bad_len[32:40] = struct.pack("<Q", 1 << 40)
    assert status_of(bad_len, "c.bin") == -3
    assert status_of(raw[:-3], "d.bin") == -4                                # the entry now reaches past the end of the file
    garbled = bytes(raw).replace(b"k = 0,8", b"k = x,8")
    assert status_of(garbled, "e.bin") == -3
    with pytest.raises(OSError):
        pkg.host_api.WeightFile(host, tmp_path / "absent.bin")


def test_host_scalar_conversions_match_the_reference_types(pkg, host, oracle):
    """Legacy float32 block scales go through the reference's host E4M3 encoder; HALF files through its
    host bfloat16 (truncation).  Checked against the reference's own cccc/types.h where that was built,
    and against the oracle's restatement."""
    rng = np.random.default_rng(1)
    vals = np.concatenate([rng.standard_normal(4000).astype(np.float32) * s for s in (1e-3, 0.1, 1, 30, 600)]
                          + [np.float32([0, -0.0, 448, 449, 479.9, 480, 511.9, 512, 1e9, np.inf, -np.inf, np.nan, 2.0 ** -6, 2.0 ** -9, 2.0 ** -10, 1.7e-3])])
    got = np.array([host.c.cccc_host_float_to_e4m3(float(v)) for v in vals], dtype=np.uint8)
    R = oracle.ref()
    if R is not None:
        assert np.array_equal(got, np.array([R.ref_float_to_e4m3(float(v)) for v in vals], dtype=np.uint8))
    rc, want = oracle.convert(vals, 0, 4, vals.size, 1.0)                  # the device-side truncating encoder: same bytes inside the E4M3 range
    inside = np.isfinite(vals) & (np.abs(vals) <= 448)
    assert rc == 0 and np.array_equal(got[inside], want[inside])
    halves = np.arange(0, 65536, dtype=np.uint16)
    got_bf = np.array([host.c.cccc_host_half_to_bf16(int(h)) for h in halves], dtype=np.uint16)
    f32 = halves.view(np.float16).astype(np.float32)
    want_bf = (f32.view(np.uint32) >> 16).astype(np.uint16)
    nan = np.isnan(f32)
    assert np.array_equal(got_bf[~nan], want_bf[~nan])
    assert (((got_bf[nan] & 0x7F80) == 0x7F80) & ((got_bf[nan] & 0x7F) != 0) | ((got_bf[nan] & 0x7FFF) == 0x7F80)).all()
