"""Pins the oracle's binary16 conversions and its seeded generator."""
import numpy as np


def test_half_to_float_exhaustive(orc):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.empty(65536, dtype=np.float32)
    orc.lib().miwo_half_to_float_n(orc._p(bits), orc._p(got), 65536)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.isnan(got[np.isnan(want)]).all()


def test_float_to_half_every_half_and_midpoints(orc):
    # every finite half, its neighbours' midpoints (ties) and values a hair to either side
    h = np.arange(0x7C00, dtype=np.uint16).view(np.float16).astype(np.float64)
    mid = (h[:-1] + h[1:]) / 2
    pts = np.concatenate([h, mid, np.nextafter(mid.astype(np.float32), np.float32(np.inf)).astype(np.float64),
                          np.nextafter(mid.astype(np.float32), np.float32(-np.inf)).astype(np.float64),
                          [65504.0, 65519.99, 65520.0, 65536.0, 1e9, 2.0 ** -24, 2.0 ** -25, 2.0 ** -26, 3e-8]])
    pts = np.concatenate([pts, -pts]).astype(np.float32)
    want = pts.astype(np.float16)
    got = np.empty(pts.size, dtype=np.uint16)
    orc.lib().miwo_float_to_half_n(orc._p(pts), orc._p(got), pts.size)
    assert np.array_equal(got, want.view(np.uint16))


def test_float_to_half_random_bits(orc):
    rng = np.random.default_rng(1)
    bits = rng.integers(0, 2 ** 32, 2_000_000, dtype=np.uint64).astype(np.uint32)
    f = bits.view(np.float32)
    f = f[~np.isnan(f)]
    with np.errstate(over="ignore"):
        want = f.astype(np.float16)
    got = np.empty(f.size, dtype=np.uint16)
    orc.lib().miwo_float_to_half_n(orc._p(f), orc._p(got), f.size)
    assert np.array_equal(got, want.view(np.uint16))


def test_double_to_half_single_rounding(orc):
    # a double just above a half tie rounds up in one step; through float it would tie to even
    lib = orc.lib()
    tie = 1.0 + 2.0 ** -11               # midpoint between 1 and 1 + 2^-10
    above = tie + 2.0 ** -40             # not representable in float: (float) rounds it to the tie
    assert np.float32(above) == np.float32(tie)
    assert lib.miwo_double_to_half(tie) == np.float16(1.0).view(np.uint16)
    assert lib.miwo_double_to_half(above) == np.float16(1.0 + 2.0 ** -10).view(np.uint16)
    assert lib.miwo_double_to_half(-above) == np.float16(-(1.0 + 2.0 ** -10)).view(np.uint16)
    rng = np.random.default_rng(2)
    xs = rng.uniform(-70000, 70000, 20000)
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)   # numpy converts double->half directly
    got = np.array([lib.miwo_double_to_half(float(x)) for x in xs], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_splitmix64_known_answers(orc):
    # SplitMix64 from seed 0: published first outputs (Vigna's reference stream)
    want = [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F]
    got = [orc.lib().miwo_splitmix64_at(0, i) for i in range(3)]
    assert got == want
    idx = np.arange(1000, dtype=np.uint64)
    v = orc.np_splitmix64(12345, idx)
    assert [int(x) for x in v[:50]] == [orc.lib().miwo_splitmix64_at(12345, i) for i in range(50)]


def test_fill_c_equals_numpy(orc):
    for seed in (0, 1, 7):
        for dt in (np.float16, np.float32):
            a = orc.fill_uniform(4099, seed, -1.0, 1.0, dt)
            b = orc.np_fill_uniform(4099, seed, -1.0, 1.0, dt)
            assert np.array_equal(a.view(np.uint16 if dt == np.float16 else np.uint32),
                                  b.view(np.uint16 if dt == np.float16 else np.uint32))
            assert a.min() >= -1 and a.max() <= 1 and abs(float(a.astype(np.float64).mean())) < 0.05
    n = orc.fill_normal(20000, 3, 0.02, np.float32)
    assert abs(float(n.mean())) < 1e-3 and abs(float(n.std()) - 0.02) < 1e-3
    # libm's log/cos vs numpy's: allow the last float ulp before rounding to half
    n2 = orc.np_fill_normal(20000, 3, 0.02, np.float32)
    assert np.allclose(n, n2, rtol=1e-6, atol=1e-9)
