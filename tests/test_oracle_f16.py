"""f32<->f16 conversion and FNV KATs for the CPU oracle: the theorem tests of
crates/wgpu-compute/tests/kv_f16.rs:81-173, a numpy.float16 cross-check (IEEE RNE), and
the hash constants of crates/itak-kv/src/hash.rs."""
import numpy as np

import oracle


def test_every_finite_half_round_trips_exactly():
    # kv_f16.rs:87-98: 63,488 finite bit patterns.
    bits = np.concatenate([np.arange(0x0000, 0x7C00), np.arange(0x8000, 0xFC00)]).astype(np.uint16)
    assert bits.size == 63_488
    values = oracle.f16_to_f32_array(bits)
    assert np.all(np.isfinite(values))
    assert np.array_equal(oracle.f32_to_f16_array(values), bits)
    # The decoder agrees with numpy's IEEE half on every pattern, infinities included.
    allbits = np.arange(0, 0x10000, dtype=np.uint32).astype(np.uint16)
    ours = oracle.f16_to_f32_array(allbits)
    theirs = allbits.view(np.float16).astype(np.float32)
    finite = ~np.isnan(theirs)
    assert np.array_equal(ours[finite].view(np.uint32), theirs[finite].view(np.uint32))
    assert np.all(np.isnan(ours[~finite]))


class Rng:
    """kv_f16.rs:247-256 (the fixture LCG)."""

    def __init__(self, seed):
        self.s = seed

    def next_u8(self):
        self.s = (self.s * 6364136223846793005 + 1442695040888963407) % 2**64
        return self.s >> 56


def test_round_trip_stays_inside_the_half_ulp_bound():
    # kv_f16.rs:100-162.
    xs = []
    for e in range(-20, 16):
        for m in (1.0, 1.0009766, 1.5, 1.9990234, 0.5, 0.75):
            x = np.float32(m) * np.float32(2.0) ** np.float32(e)
            xs += [x, -x]
    rng = Rng(0x0F160BAD)
    for _ in range(200_000):
        sign = 1.0 if rng.next_u8() & 1 == 0 else -1.0
        e = (rng.next_u8() % 36) - 20
        mant = np.float32(1.0) + (np.float32(rng.next_u8()) / np.float32(256.0)
                                  + np.float32(rng.next_u8()) / np.float32(65536.0))
        xs.append(np.float32(sign) * mant * np.float32(2.0) ** np.float32(e))
    x = np.array(xs, dtype=np.float32)
    x = x[np.isfinite(x) & (np.abs(x) < 65504.0)]
    assert x.size > 200_000
    rt = oracle.round_through_f16(x)
    err = np.abs(rt.astype(np.float64) - x.astype(np.float64))
    normal = np.abs(x) >= np.float32(2.0) ** -14
    rel = err[normal] / np.abs(x[normal].astype(np.float64))
    assert rel.max() <= 2.0 ** -11
    assert rel.max() > 0.0
    assert err[~normal].max() <= 2.0 ** -25


def test_packed_word_layout_is_even_low_odd_high():
    # kv_f16.rs:164-173: consecutive little-endian halves are the packed pair.
    for lo, hi in ((1.5, -0.25), (0.0, 65504.0)):
        halves = oracle.f32_to_f16_array(np.array([lo, hi], dtype=np.float32))
        word = int(halves.view(np.uint32)[0])
        assert word == int(halves[0]) | (int(halves[1]) << 16)
        back = oracle.f16_to_f32_array(halves)
        assert back.tolist() == [lo, hi]


def test_encoder_matches_ieee_rne_everywhere_numpy_defines_it():
    rng = np.random.default_rng(20261125)
    bits = rng.integers(0, 2**32, size=2_000_000, dtype=np.uint64).astype(np.uint32)
    # Dense sweeps around every rounding boundary class: ties, subnormals, overflow edge.
    edges = []
    for e in range(0, 256):
        base = e << 23
        for frac in (0, 1, 0xFFF, 0x1000, 0x1001, 0x1FFF, 0x2000, 0x2FFF, 0x3000, 0x3001,
                     0x7FEFFF, 0x7FF000, 0x7FF001, 0x7FFFFF):
            edges += [base | frac, 0x80000000 | base | frac]
    bits = np.concatenate([bits, np.array(edges, dtype=np.uint32)])
    x = bits.view(np.float32)
    ours = oracle.f32_to_f16_array(x)
    with np.errstate(over="ignore", invalid="ignore"):
        theirs = x.astype(np.float16).view(np.uint16)
    nan = np.isnan(x)
    assert np.array_equal(ours[~nan], theirs[~nan])
    # NaN canonicalisation (k1_q4k_gemv.rs:290-293): sign kept, payload dropped.
    sign = ((bits[nan] >> 16) & 0x8000).astype(np.uint16)
    assert np.array_equal(ours[nan], sign | np.uint16(0x7E00))


def test_named_special_cases():
    f = oracle.f32_to_f16_bits
    assert f(65504.0) == 0x7BFF
    assert f(65519.996) == 0x7BFF       # below the halfway point to 65536
    assert f(65520.0) == 0x7C00         # the tie rounds to even = infinity
    assert f(-65520.0) == 0xFC00
    assert f(2.0 ** -24) == 0x0001      # smallest subnormal
    assert f(2.0 ** -25) == 0x0000      # tie to even (zero)
    assert f(np.nextafter(np.float32(2.0 ** -25), np.float32(1))) == 0x0001
    assert f(-0.0) == 0x8000
    assert f(1.0 + 2.0 ** -11) == 0x3C00  # tie to even stays
    assert f(1.0 + 3 * 2.0 ** -11) == 0x3C02  # tie to even goes up
    assert f(float("inf")) == 0x7C00
    assert oracle.f32_bits_to_f16_bits(0xFFC12345) == 0xFE00


def test_fnv1a_constants_and_vectors():
    # hash.rs:14,72,83-87 and the published FNV-1a 64 test vectors.
    assert oracle.checksum(b"") == 0xCBF29CE484222325
    assert oracle.prefix_hash([]) == 0xCBF29CE484222325
    assert oracle.checksum(b"a") == 0xAF63DC4C8601EC8C
    assert oracle.checksum(b"foobar") == 0x85944171F73967E8
    assert oracle.prefix_hash([1, 2, 3]) != oracle.prefix_hash([3, 2, 1])
    assert oracle.prefix_hash([0x64636261]) == oracle.checksum(b"abcd")


def test_rope_is_a_rotation_with_float64_angles():
    # rope.rs:99-116: position 0 is the identity, norms are preserved, pair i uses
    # angle p * base^(-2i/d).
    rng = np.random.default_rng(1)
    x = rng.standard_normal(128).astype(np.float32)
    assert np.array_equal(oracle.rope_half_split(x, 0, 1e6), x)
    y = oracle.rope_half_split(x, 4095, 1e6)
    assert abs(np.linalg.norm(y) - np.linalg.norm(x)) < 1e-4
    i = 5
    ang = 4095 * (1e6 ** (-2 * i / 128))
    assert abs(y[i] - (x[i] * np.cos(ang) - x[i + 64] * np.sin(ang))) < 1e-6
    assert abs(y[i + 64] - (x[i] * np.sin(ang) + x[i + 64] * np.cos(ang))) < 1e-6
    rows = rng.standard_normal((3, 2, 128)).astype(np.float32)
    batch = oracle.rope_rows(rows, 10, 1e6)
    for r in range(3):
        for h in range(2):
            assert np.array_equal(batch[r, h], oracle.rope_half_split(rows[r, h], 10 + r, 1e6))
