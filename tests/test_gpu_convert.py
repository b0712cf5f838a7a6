"""Bit-exact parity of hip_convert / hip_fp4_blockscale_to_bf16 against the oracle and the golden
tables, through the C-ABI."""
import numpy as np
import pytest

from gpu_util import from_dev, to_dev

pytestmark = pytest.mark.gpu

ALL = np.arange(256, dtype=np.uint8)


def run_convert(gpu, src, src_type, dst_type, n, scale, dst_dtype, dst_count=None, src_offset=0, dst_offset=0):
    torch, dev, lib = gpu
    s = to_dev(torch, dev, src)
    count = dst_count if dst_count is not None else n
    item = np.dtype(dst_dtype).itemsize
    d = torch.zeros(count * item + dst_offset + 64, dtype=torch.uint8, device=dev)
    rc = lib.convert(s.data_ptr() + src_offset, src_type, d.data_ptr() + dst_offset, dst_type, n, scale)
    out = d.cpu().numpy()[dst_offset:dst_offset + count * item].copy().view(dst_dtype)
    tail = d.cpu().numpy()[dst_offset + count * item:]
    assert not tail.any(), "wrote past the end"
    return rc, out


def test_all_codes_all_scales_golden(gpu, golden_tables, oracle):
    g = golden_tables
    reps = np.tile(ALL, 5)[:1237]                      # not a multiple of 16: exercises vector body + scalar tail
    for i, s in enumerate(g["scales"]):
        for dtype, key in ((oracle.E5M2, "e5m2_bf16"), (oracle.E4M3, "e4m3_bf16")):
            rc, out = run_convert(gpu, reps, dtype, oracle.BF16, reps.size, float(s), np.uint16)
            assert rc == 0
            assert np.array_equal(out, g[key][i][reps]), (key, s)
        nib = (np.arange(16, dtype=np.uint8)[0::2] | (np.arange(16, dtype=np.uint8)[1::2] << 4)).astype(np.uint8)
        nib = np.tile(nib, 9)[:67]
        n = 133                                        # odd element count
        rc, out = run_convert(gpu, nib, oracle.FP4, oracle.BF16, n, float(s), np.uint16)
        assert rc == 0
        assert np.array_equal(out, oracle.dequant_fp4_to_bf16(nib, n, float(s))), s


@pytest.mark.parametrize("dst", ["float", "half", "bf16"])
@pytest.mark.parametrize("src", ["e5m2", "e4m3"])
def test_fp8_dequant_random_vs_oracle(gpu, oracle, src, dst):
    rng = np.random.default_rng(100)
    st = {"e5m2": oracle.E5M2, "e4m3": oracle.E4M3}[src]
    dt, npdt = {"float": (oracle.FLOAT, np.uint32), "half": (oracle.HALF, np.uint16), "bf16": (oracle.BF16, np.uint16)}[dst]
    for n, scale in ((1 << 20, 1.0), (100003, 0.0371), (15, 2.0), (1, 1.0)):
        codes = rng.integers(0, 256, size=n, dtype=np.uint8)
        rc, out = run_convert(gpu, codes, st, dt, n, scale, npdt)
        assert rc == 0
        rc2, want = oracle.convert(codes, st, dt, n, scale)
        assert rc2 == 0
        want = want.view(npdt)
        if dst == "float":
            nan = np.isnan(want.view(np.float32))
            assert np.array_equal(out[~nan], want[~nan]) and np.all(np.isnan(out.view(np.float32)[nan]))
        elif dst == "half":
            nan = np.isnan(want.view(np.float16))
            assert np.array_equal(out[~nan], want[~nan]) and np.all(np.isnan(out.view(np.float16)[nan]))
        else:
            assert np.array_equal(out, want)


def test_misaligned_pointers_take_the_scalar_path(gpu, oracle):
    rng = np.random.default_rng(101)
    codes = rng.integers(0, 256, size=5000 + 3, dtype=np.uint8)
    rc, out = run_convert(gpu, codes, oracle.E5M2, oracle.BF16, 5000, 0.3, np.uint16, src_offset=3, dst_offset=2)
    assert rc == 0
    assert np.array_equal(out, oracle.dequant_fp8_to_bf16(codes[3:], oracle.E5M2, 0.3))


@pytest.mark.parametrize("block", [16, 32, 8, 2, 64])
def test_fp4_blockscale_vs_oracle_and_golden(gpu, oracle, golden_tables, block):
    torch, dev, lib = gpu
    rng = np.random.default_rng(102 + block)
    for n in (256 * 16, 4096 * 64, 16 * 1000 + block * 3, block * 5 + (block // 2) * 2 - 1):
        nib = rng.integers(0, 256, size=(n + 1) // 2, dtype=np.uint8)
        sc = rng.integers(0, 256, size=(n + block - 1) // block, dtype=np.uint8)
        nd, sd = to_dev(torch, dev, nib), to_dev(torch, dev, sc)
        out = torch.zeros(n + 32, dtype=torch.int16, device=dev)
        rc = lib.fp4_blockscale_to_bf16(nd.data_ptr(), sd.data_ptr(), out.data_ptr(), n, block)
        assert rc == 0
        got = from_dev(out, np.uint16)
        assert not got[n:].any()
        assert np.array_equal(got[:n], oracle.dequant_fp4_blockscale_to_bf16(nib, sc, n, block)), (block, n)
    if block == 16:
        nib = np.tile((np.arange(16, dtype=np.uint8)[0::2] | (np.arange(16, dtype=np.uint8)[1::2] << 4)).astype(np.uint8), 256)
        nd, sd = to_dev(torch, dev, nib), to_dev(torch, dev, ALL)
        out = torch.zeros(4096, dtype=torch.int16, device=dev)
        assert lib.fp4_blockscale_to_bf16(nd.data_ptr(), sd.data_ptr(), out.data_ptr(), 4096, 16) == 0
        assert np.array_equal(from_dev(out, np.uint16).reshape(256, 16), golden_tables["blockscale_bf16"])


def test_fp4_blockscale_bad_arguments(gpu):
    torch, dev, lib = gpu
    buf = torch.zeros(64, dtype=torch.uint8, device=dev)
    assert lib.fp4_blockscale_to_bf16(buf.data_ptr(), buf.data_ptr(), buf.data_ptr(), 16, 0) == -1
    assert lib.fp4_blockscale_to_bf16(buf.data_ptr(), None, buf.data_ptr(), 16, 16) == -1
    assert lib.fp4_blockscale_to_bf16(buf.data_ptr(), buf.data_ptr(), buf.data_ptr(), 0, 16) == 0


def test_other_pairs_of_the_table(gpu, oracle):
    rng = np.random.default_rng(103)
    n = 70001
    x = (rng.standard_normal(n) * 2.0 ** rng.integers(-12, 12, n)).astype(np.float32)
    x[:6] = [0.0, -0.0, 1e9, -1e9, 448.0, 57344.0]
    xb = oracle.f32_to_bf16(x)
    xh = x.astype(np.float16).view(np.uint16)
    cases = [
        (x, oracle.FLOAT, oracle.BF16, np.uint16, 1.0),
        (xh, oracle.HALF, oracle.FLOAT, np.uint32, 1.0),
        (xh, oracle.HALF, oracle.BF16, np.uint16, 1.0),
        (xb, oracle.BF16, oracle.FLOAT, np.uint32, 1.0),
        (xb, oracle.BF16, oracle.HALF, np.uint16, 1.0),
        (x, oracle.FLOAT, oracle.E4M3, np.uint8, 3.7),
        (x, oracle.FLOAT, oracle.E5M2, np.uint8, 0.9),
        (xb, oracle.BF16, oracle.E4M3, np.uint8, 1.0),
    ]
    for src, st, dt, npdt, scale in cases:
        rc, out = run_convert(gpu, src, st, dt, n, scale, npdt)
        rc2, want = oracle.convert(src, st, dt, n, scale)
        assert rc == 0 and rc2 == 0
        assert np.array_equal(out, want.view(npdt)), (st, dt)
    rc, out = run_convert(gpu, x, oracle.FLOAT, oracle.FP4, n, 1.3, np.uint8, dst_count=(n + 1) // 2)
    rc2, want = oracle.convert(x, oracle.FLOAT, oracle.FP4, n, 1.3)
    assert rc == 0 and np.array_equal(out, want)


def test_unsupported_pairs_and_same_type_copy(gpu, oracle):
    torch, dev, lib = gpu
    buf = to_dev(torch, dev, np.arange(64, dtype=np.uint8))
    dst = torch.zeros(64, dtype=torch.uint8, device=dev)
    for st, dt in ((oracle.DOUBLE, oracle.FLOAT), (oracle.E5M2, oracle.E4M3), (oracle.FP4, oracle.HALF), (7, 3), (3, -1), (oracle.HALF, oracle.E4M3)):
        assert lib.convert(buf.data_ptr(), st, dst.data_ptr(), dt, 16, 1.0) == -1, (st, dt)
    assert not dst.cpu().numpy().any()
    # same type, scale 1: copies n BYTES whatever the type (reference behaviour)
    assert lib.convert(buf.data_ptr(), oracle.BF16, dst.data_ptr(), oracle.BF16, 10, 1.0) == 0
    got = dst.cpu().numpy()
    assert np.array_equal(got[:10], np.arange(10, dtype=np.uint8)) and not got[10:].any()
    assert lib.convert(buf.data_ptr(), oracle.E5M2, dst.data_ptr(), oracle.BF16, 0, 1.0) == 0


def test_float_to_fp4_blockscale_vs_oracle(gpu, oracle):
    torch, dev, lib = gpu
    rng = np.random.default_rng(104)
    for n, block in ((4096, 16), (1000, 16), (999, 16), (4096, 32), (64, 2)):
        x = (rng.standard_normal(n) * 0.02).astype(np.float32)
        x[: min(n, 32)] = 0.0                           # an all-zero block: scale 1.0 -> 0x38
        xd = to_dev(torch, dev, x)
        nib = torch.zeros((n + 1) // 2, dtype=torch.uint8, device=dev)
        sc = torch.zeros((n + block - 1) // block, dtype=torch.uint8, device=dev)
        assert lib.float_to_fp4_blockscale(xd.data_ptr(), nib.data_ptr(), sc.data_ptr(), n, block) == 0
        wn, ws = oracle.quantize_fp4_blockscale_kernel(x, block)
        assert np.array_equal(nib.cpu().numpy(), wn) and np.array_equal(sc.cpu().numpy(), ws), (n, block)
    assert lib.float_to_fp4_blockscale(xd.data_ptr(), nib.data_ptr(), sc.data_ptr(), 16, 3) == -1


@pytest.mark.parametrize("src_type", ["float", "half", "bf16"])
@pytest.mark.parametrize("n,offset", [(1, 0), (7, 0), (4099, 0), (4099, 1), (1 << 20, 0), ((1 << 22) + 5, 3)])
def test_absmax_of_a_tensor(gpu, oracle, src_type, n, offset):
    """hip_absmax (the per-tensor scale of the on-the-fly FP8 quantiser, cccc-cuda/cuda_functions.cu:2694-2733) against
    numpy on FLOAT / HALF / BF16 tensors, including a start that is not 16-byte aligned, a ragged tail, a NaN (skipped)
    and the largest value in the last element; the result buffer is cleared by the call."""
    torch, dev, lib = gpu
    rng = np.random.default_rng(n + offset)
    x = (rng.standard_normal(n + offset) * 3).astype(np.float32)
    if n > 4:
        x[offset + 2] = np.nan
    x[offset + n - 1] = -77.5 if n > 1 else 0.25
    if src_type == "float":
        host, code, vals = x, oracle.FLOAT, x
    elif src_type == "half":
        host = x.astype(np.float16)
        code, vals = oracle.HALF, host.astype(np.float32)
    else:
        bits = oracle.f32_to_bf16(np.nan_to_num(x, nan=0.0))
        if n > 4:
            bits[offset + 2] = 0x7FC0
        host, code, vals = bits, oracle.BF16, oracle.bf16_to_f32(bits)
    d = to_dev(torch, dev, host)
    res = torch.full((2,), 123.0, dtype=torch.float32, device=dev)
    assert lib.absmax(d.data_ptr() + offset * host.dtype.itemsize, code, n, res.data_ptr()) == 0
    got = res.cpu().numpy()
    assert got[1] == 123.0
    assert got[0] == np.nanmax(np.abs(vals[offset:offset + n]))
