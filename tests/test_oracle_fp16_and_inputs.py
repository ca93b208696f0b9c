"""Pins the oracle's fp16 conversion and input generator against independent sources:
numpy's IEEE binary16, the published SplitMix64 known-answer vector, and a numpy
restatement of the generator."""
import numpy as np
import pytest

MASK = (1 << 64) - 1


def test_f16_to_f32_all_bit_patterns(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([oracle.f16_to_f32(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f32_to_f16_roundtrip_all_halves(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    f = bits.view(np.float16).astype(np.float32)
    for b, v in zip(bits.tolist(), f.tolist()):
        if (b & 0x7FFF) > 0x7C00:
            continue
        assert oracle.f32_to_f16(v) == b


def test_f32_to_f16_matches_numpy_rne(oracle):
    rng = np.random.default_rng(7)
    # random bit patterns cover all exponents, plus dense samples around the
    # subnormal/normal/overflow boundaries and exact ties
    raw = rng.integers(0, 1 << 32, size=1 << 18, dtype=np.uint64).astype(np.uint32).view(np.float32)
    near = np.concatenate([
        rng.uniform(-70000, 70000, 1 << 17), rng.uniform(-1e-4, 1e-4, 1 << 17), rng.uniform(-2, 2, 1 << 17),
    ]).astype(np.float32)
    halves = np.arange(0x7C00, dtype=np.uint16).view(np.float16).astype(np.float64)
    ties = ((halves[:-1] + halves[1:]) / 2).astype(np.float32)  # exact midpoints are fp32-representable
    ties = np.concatenate([ties, -ties, np.float32([65520.0, 65519.996, 65504.0, 2.0 ** -25, 2.0 ** -24, 0.0, -0.0])])
    vals = np.concatenate([raw, near, ties])
    vals = vals[~np.isnan(vals)]
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([oracle.f32_to_f16(v) for v in vals.tolist()], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_convert_f32_to_f16_array_matches_numpy_rne(oracle):
    """The element-wise conversion (the reference's convertFp32ToFp16, src/utils/cuda_helpers.cuh:116-121)
    against numpy's IEEE round-to-nearest-even cast, NaNs by class."""
    rng = np.random.default_rng(8)
    raw = rng.integers(0, 1 << 32, size=1 << 18, dtype=np.uint64).astype(np.uint32).view(np.float32)
    halves = np.arange(0x7C00, dtype=np.uint16).view(np.float16).astype(np.float64)
    ties = ((halves[:-1] + halves[1:]) / 2).astype(np.float32)
    vals = np.concatenate([raw, ties, -ties, np.nextafter(ties, np.float32(np.inf)), np.nextafter(ties, np.float32(-np.inf)),
                           np.float32([65520.0, -65520.0, 65519.996, 65504.0, 2.0 ** -25, 2.0 ** -24, 0.0, -0.0, np.inf, -np.inf, 0.001])])
    got = oracle.f32_to_f16_array(vals)
    with np.errstate(over="ignore", invalid="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    nan = np.isnan(vals)
    assert np.array_equal(got[~nan], want[~nan])
    assert ((got[nan] & 0x7C00) == 0x7C00).all() and ((got[nan] & 0x03FF) != 0).all()
    assert oracle.f32_to_f16_array(np.float32([0.001]))[0] == 0x1419  # the reference's fill value
    assert oracle.f32_to_f16_array(np.empty(0, np.float32)).size == 0


def test_f64_to_f16_single_rounding(oracle):
    rng = np.random.default_rng(11)
    vals = np.concatenate([rng.uniform(-70000, 70000, 20000), rng.uniform(-1e-4, 1e-4, 20000), rng.uniform(-4, 4, 20000)])
    halves = np.arange(0x7C00, dtype=np.uint16).view(np.float16).astype(np.float64)
    mids = (halves[:-1] + halves[1:]) / 2
    # a hair above/below a tie must round away from / toward it: double rounding through
    # fp32 would get these wrong
    vals = np.concatenate([vals, mids, np.nextafter(mids, np.inf), np.nextafter(mids, -np.inf), -mids])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([oracle.f64_to_f16(v) for v in vals.tolist()], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_ulp_f16(oracle):
    for v, u in [(0.0, 2.0 ** -24), (1e-6, 2.0 ** -24), (2.0 ** -14, 2.0 ** -24), (1.0, 2.0 ** -10), (1.999, 2.0 ** -10),
                 (2.0, 2.0 ** -9), (-3.0, 2.0 ** -9), (1024.0, 1.0), (40000.0, 32.0), (70000.0, 32.0)]:
        assert oracle.ulp_f16(v) == u
    # agrees with numpy's spacing on every positive normal half
    h = np.arange(0x0400, 0x7BFF, dtype=np.uint16).view(np.float16)  # spacing(65504) overflows in fp16
    want = np.spacing(h).astype(np.float64)
    got = np.array([oracle.ulp_f16(float(x)) for x in h.astype(np.float64)])
    assert np.array_equal(got, want)


def test_splitmix64_known_answer_vector(oracle):
    # first outputs of SplitMix64 (Steele/Lea/Vigna) seeded with 1234567
    want = [6457827717110365317, 3203168211198807973, 9817491932198370423, 4593380528125082431, 16408922859458223821]
    assert [oracle.splitmix64(1234567, i) for i in range(5)] == want


def _np_splitmix(seed, idx):
    with np.errstate(over="ignore"):
        z = np.uint64(seed & MASK) + (idx.astype(np.uint64) + np.uint64(1)) * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


@pytest.mark.parametrize("seed", [0, 1, 0xDEADBEEFCAFEF00D])
def test_generator_matches_numpy_restatement(oracle, seed):
    n = 1 << 16
    idx = np.arange(n, dtype=np.uint64)
    z = _np_splitmix(seed, idx)
    # uniform [-1,1)
    u = (z >> np.uint64(40)).astype(np.float32)
    h = (u * np.float32(2.0 ** -23) - np.float32(1.0)).astype(np.float16).view(np.uint16)
    h = np.where(h == 0x3C00, np.uint16(0x3BFF), h)
    assert np.array_equal(oracle.generate_f16(n, seed, oracle.DIST_UNIFORM), h)
    # exact grid
    k = (z >> np.uint64(52)).astype(np.int64) - 2048
    g = (k.astype(np.float64) / 2048.0).astype(np.float16)
    assert np.array_equal(g.astype(np.float64) * 2048, k)  # exactly representable
    assert np.array_equal(oracle.generate_f16(n, seed, oracle.DIST_GRID), g.view(np.uint16))
    # small ints
    s = ((z >> np.uint64(33)) % np.uint64(3)).astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.generate_f16(n, seed, oracle.DIST_SMALLINT), s)
    # range form is consistent with the whole
    part = oracle.generate_f16(1000, seed, oracle.DIST_UNIFORM, first=12345)
    assert np.array_equal(part, h[12345:13345])


def test_generator_distribution_sanity(oracle):
    n = 1 << 20
    x = oracle.generate_f16(n, 0, oracle.DIST_UNIFORM).view(np.float16).astype(np.float64)
    assert x.min() >= -1.0 and x.max() < 1.0
    assert abs(x.mean()) < 3e-3 and abs(x.var() - 1.0 / 3.0) < 3e-3
    z = oracle.generate_f16(n, 1, oracle.DIST_NORMAL).view(np.float16).astype(np.float64)
    assert abs(z.mean()) < 5e-3 and abs(z.var() - 1.0) < 1e-2
    assert abs((np.abs(z) < 1.0).mean() - 0.682689) < 3e-3
    g = oracle.generate_f16(n, 1, oracle.DIST_GRID).view(np.float16).astype(np.float64)
    assert g.min() >= -1.0 and g.max() <= 2047 / 2048


def test_constant_fill_is_the_reference_fixture(oracle):
    # the reference fills every input with (half) 0.001f = 0x1419
    x = oracle.fill_f16(1000, 0.001)
    assert np.all(x == 0x1419)
    assert float(x[:1].view(np.float16)[0]) == 0.00100040435791015625
