"""Pins the oracle's input generator and narrow-format conversions against outside
knowledge: published SplitMix64 outputs, numpy's float16, torch's float8/bfloat16, the
OCP MX value tables.  None of these checks re-derives the oracle's own formulas."""
import numpy as np
import pytest

from oracle import pyoracle as orc


# SplitMix64 (Steele/Lea/Flood; Vigna's splitmix64.c), first outputs for state 1234567:
# the vector that test suites of the JDK's SplittableRandom ports use.
SPLITMIX_1234567 = [6457827717110365317, 3203168211198807973, 9817491932198370423,
                    4593380528125082431, 16408922859458223821]


def test_rng_stream0_is_splitmix64():
    got = [orc.rng_word(1234567, 0, i) for i in range(5)]
    assert got == SPLITMIX_1234567


def test_rng_streams_are_distinct_and_counter_based():
    a = [orc.rng_word(42, 0, i) for i in range(64)]
    b = [orc.rng_word(42, 1, i) for i in range(64)]
    assert len(set(a) | set(b)) == 128
    # element i does not depend on how many elements were drawn before it
    assert orc.fill_f32(16, 42, 3, 0, first=100)[5] == orc.fill_f32(1, 42, 3, 0, first=105)[0]


def test_uniform_ranges_and_moments():
    u = orc.fill_f32(1 << 20, 7, 0, 0)
    s = orc.fill_f32(1 << 20, 7, 0, 1)
    assert u.min() >= 0.0 and u.max() < 1.0 and s.min() >= -1.0 and s.max() < 1.0
    assert abs(u.mean() - 0.5) < 2e-3 and abs(u.var() - 1 / 12) < 1e-3
    assert abs(s.mean()) < 3e-3 and abs(s.var() - 1 / 3) < 2e-3
    # values sit on the 2^-24 / 2^-23 lattices, i.e. are exact in fp32
    assert np.all(u * 2 ** 24 == np.round(u * 2 ** 24)) and np.all(s * 2 ** 23 == np.round(s * 2 ** 23))
    # the two distributions are the same draws: s = 2u - 1
    assert np.array_equal(s, u * 2 - 1)


def test_normal_moments():
    z = orc.lib()
    x = np.array([z.orc_normal(11, 2, i) for i in range(200000)])
    assert abs(x.mean()) < 0.01 and abs(x.std() - 1) < 0.01
    assert abs(((x - x.mean()) ** 3).mean()) < 0.03             # skewness ~ 0
    assert abs(((x - x.mean()) ** 4).mean() - 3) < 0.1            # kurtosis ~ 3
    assert abs((np.abs(x) < 1.959964).mean() - 0.95) < 0.003


def test_f16_decode_all_codes_against_numpy():
    codes = np.arange(65536, dtype=np.uint16)
    ref = codes.view(np.float16).astype(np.float64)
    got = orc.decode(orc.FMT_F16, codes)
    nan = np.isnan(ref)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan], ref[~nan])


def test_f16_encode_against_numpy():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(20000) * 10.0 ** rng.integers(-8, 5, 20000),
                        [0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e9, -1e9, 2.0 ** -24, 2.0 ** -25, 3 * 2.0 ** -25,
                         1 + 2.0 ** -11, 1 + 3 * 2.0 ** -11]])
    with np.errstate(over="ignore"):
        ref = x.astype(np.float16).view(np.uint16)  # float64 -> float16 is a single RNE rounding in numpy
    got = orc.encode(orc.FMT_F16, x).astype(np.uint16)
    assert np.array_equal(got, ref)


def test_bf16_against_torch():
    torch = pytest.importorskip("torch")
    codes = np.arange(65536, dtype=np.int64)
    t = torch.tensor(codes.astype(np.int16) if False else codes, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    ref = t.to(torch.float64).numpy()
    got = orc.decode(orc.FMT_BF16, codes)
    ok = ~np.isnan(ref)
    assert np.array_equal(np.isnan(got), ~ok) and np.array_equal(got[ok], ref[ok])
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(20000) * 10.0 ** rng.integers(-20, 20, 20000)).astype(np.float32)
    ref_c = torch.tensor(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(orc.encode(orc.FMT_BF16, x.astype(np.float64)).astype(np.uint16), ref_c)


@pytest.mark.parametrize("fmt,tname", [(orc.FMT_E4M3, "float8_e4m3fn"), (orc.FMT_E5M2, "float8_e5m2")])
def test_fp8_against_torch(fmt, tname):
    torch = pytest.importorskip("torch")
    tdt = getattr(torch, tname)
    codes = np.arange(256, dtype=np.uint8)
    ref = torch.tensor(codes).view(tdt).to(torch.float64).numpy()
    got = orc.decode(fmt, codes)
    ok = ~np.isnan(ref)
    assert np.array_equal(np.isnan(got), ~ok) and np.array_equal(got[ok], ref[ok])
    # encode: torch rounds to nearest even; stay inside the finite range (torch does not saturate)
    fmax = np.nanmax(np.where(np.isinf(ref), np.nan, ref))
    rng = np.random.default_rng(2)
    x = (rng.standard_normal(20000) * 10.0 ** rng.integers(-6, 3, 20000)).astype(np.float32)
    x = x[np.abs(x) <= fmax]
    ref_c = torch.tensor(x).to(tdt).view(torch.uint8).numpy()
    assert np.array_equal(orc.encode(fmt, x.astype(np.float64)).astype(np.uint8), ref_c)
    # saturation instead of inf/nan beyond the range (OCP saturating conversion)
    assert orc.decode(fmt, orc.encode(fmt, [1e9]))[0] == fmax and orc.decode(fmt, orc.encode(fmt, [-1e9]))[0] == -fmax


def test_mx_value_tables():
    """OCP Microscaling Formats (MX) v1.0, tables of the element formats."""
    e2m1 = orc.decode(orc.FMT_E2M1, np.arange(16))
    assert list(e2m1[:8]) == [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    assert list(e2m1[8:]) == [-0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0]
    e2m3 = orc.decode(orc.FMT_E2M3, np.arange(64))
    assert e2m3[:32].max() == 7.5 and e2m3[1] == 0.125 and e2m3[8] == 1.0 and e2m3[0b01111] == 1.875
    e3m2 = orc.decode(orc.FMT_E3M2, np.arange(64))
    assert e3m2[:32].max() == 28.0 and e3m2[1] == 0.0625 and e3m2[0b00100] == 0.25 and e3m2[0b01100] == 1.0
    e4m3 = orc.decode(orc.FMT_E4M3, np.arange(256))
    assert np.nanmax(e4m3) == 448.0 and e4m3[1] == 2.0 ** -9 and np.isnan(e4m3[0x7f]) and e4m3[0x38] == 1.0
    e5m2 = orc.decode(orc.FMT_E5M2, np.arange(256))
    assert e5m2[0x7b] == 57344.0 and np.isinf(e5m2[0x7c]) and e5m2[1] == 2.0 ** -16 and e5m2[0x3c] == 1.0
    L = orc.lib()
    assert L.orc_e8m0(127) == 1.0 and L.orc_e8m0(0) == 2.0 ** -127 and L.orc_e8m0(254) == 2.0 ** 127
    assert np.isnan(L.orc_e8m0(255))


@pytest.mark.parametrize("fmt,ncodes", [(orc.FMT_E2M3, 64), (orc.FMT_E3M2, 64), (orc.FMT_E2M1, 16)])
def test_small_format_encode_is_nearest_even(fmt, ncodes):
    """Brute force: for a dense sweep of reals, the chosen code is a nearest one and
    ties go to the even code."""
    table = orc.decode(fmt, np.arange(ncodes // 2))
    xs = np.linspace(0, table.max() * 1.2, 4001)
    got = orc.encode(fmt, xs)
    for x, c in zip(xs, got):
        d = np.abs(table - min(x, table.max()))
        best = np.flatnonzero(d == d.min())
        assert c in best
        if len(best) == 2:
            assert c % 2 == 0
    assert np.array_equal(orc.encode(fmt, -xs[1:]), got[1:] + ncodes // 2)


def test_operand_builders():
    n = 4096
    i8 = orc.fill_int8(5, 2, n)
    assert i8.min() == -8 and i8.max() == 7 and abs(i8.mean() + 0.5) < 0.3
    e = orc.fill_e8m0(5, 4, n).astype(int) - 127
    assert e.min() == -4 and e.max() == 4 and len(np.unique(e)) == 9
    m = orc.fill_sparse_meta(5, 6, n)
    p0, p1 = m & 3, (m >> 2) & 3
    assert np.all(p0 < p1) and len(np.unique(m)) == 6 and np.all(m < 16)
    codes = (np.arange(64) % 64).astype(np.uint8)
    packed6 = orc.pack_bits(codes, 6)
    bits = np.unpackbits(packed6, bitorder="little")
    assert np.array_equal(bits.reshape(-1, 6) @ (1 << np.arange(6)), codes)
    packed4 = orc.pack_bits(codes % 16, 4)
    assert np.array_equal(packed4 & 15, (codes % 16)[0::2]) and np.array_equal(packed4 >> 4, (codes % 16)[1::2])
    # sigma-scaled normal codes decode to values with the requested spread
    c = orc.fill_normal_codes(orc.FMT_F16, 0.01, 9, 2, 20000)
    v = c.view(np.float16).astype(np.float64)
    assert abs(v.std() - 0.01) < 3e-4 and abs(v.mean()) < 3e-4


# ---- the committed fixture of the seeded streams ------------------------------------------------------
def _golden_streams():
    import json
    import os
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "seeded_streams.json")
    with open(path) as f:
        return json.load(f)


def test_oracle_reproduces_the_committed_streams():
    """tests/golden/seeded_streams.json was written once by tests/golden/make_seeded_streams.py; building it
    again must give the same document, value for value."""
    import importlib.util
    import os
    spec = importlib.util.spec_from_file_location(
        "make_seeded_streams", os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "make_seeded_streams.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    assert mod.build() == _golden_streams()


def test_host_generator_reproduces_the_committed_streams():
    """The backend's own host-side generator (what Mi355Peak uploads, what bench.py measures on) against the
    same fixture, without the oracle in between."""
    from clpeak_amd import workloads as pw
    g = _golden_streams()
    n, seed = g["count"], g["seed"]
    assert seed == pw.DEFAULT_SEED
    for name, fmt, sigma in (("f16", pw.F16, 0.01), ("bf16", pw.BF16, 0.01), ("e4m3", pw.E4M3, 1.0), ("e5m2", pw.E5M2, 1.0)):
        got = pw.operand(fmt, sigma, seed, pw.STREAM_MFMA_A, n)
        codes = got.view(np.uint16) if fmt in (pw.F16, pw.BF16) else got
        assert [int(x) for x in codes] == g["operands"][name], name
    # 6- and 4-bit codes come packed: unpack little-endian bit fields
    for name, fmt, bits in (("e2m3", pw.E2M3, 6), ("e3m2", pw.E3M2, 6), ("e2m1", pw.E2M1, 4)):
        packed = pw.operand(fmt, 1.0, seed, pw.STREAM_MFMA_A, n)
        word = int.from_bytes(bytes(packed), "little")
        assert [(word >> (bits * i)) & ((1 << bits) - 1) for i in range(n)] == g["operands"][name], name
    assert [int(x) for x in pw.operand(pw.I8, 0.0, seed, pw.STREAM_MFMA_B, n).view(np.int8)] == g["operands"]["int8"]
    assert [int(x) for x in pw.e8m0_scales(seed, pw.STREAM_SCALE_A, n)] == g["bytes"]["e8m0_scale_a"]
    assert [int(x) for x in pw.sparse_meta(seed, pw.STREAM_SPARSE, n)] == g["bytes"]["sparse_meta"]
