"""Checks that pin oracle/hash_rng.py without retyping its formulas: both hashes are permutations (inverted
here with modular inverses from pow() and by undoing each xor-shift), no collisions, avalanche, and the two
float distributions against scipy.stats."""
import numpy as np
import pytest
from scipy import stats

from oracle import hash_rng

M = 1 << 32


def _unxorshift(y, s):
    """Inverse of x -> x ^ (x >> s) on 32 bits."""
    x = y
    for _ in range(32 // s + 1):
        x = y ^ (x >> s)
    return x


def _invert_hash_u32(h):
    word = _unxorshift(h, 22)
    mixed = (word * pow(277803737, -1, M)) % M
    # the data-dependent shift is at least 4, so the top four bits of the state survive it
    state = _unxorshift(mixed, (mixed >> 28) + 4)
    return ((state - 2891336453) * pow(747796405, -1, M)) % M


def _invert_hash_u32x2(x, y):
    k, c = 1664525, 1013904223
    kinv = pow(k, -1, M)
    x, y = _unxorshift(x, 16), _unxorshift(y, 16)
    y = (y - x * k) % M
    x = (x - y * k) % M
    x, y = _unxorshift(x, 16), _unxorshift(y, 16)
    y = (y - x * k) % M
    x = (x - y * k) % M
    return ((x - c) * kinv) % M, ((y - c) * kinv) % M


def test_hash_u32_is_inverted_by_the_permutation_steps():
    rng = np.random.default_rng(1)
    vs = np.concatenate([np.array([0, 1, 2, M - 1, M // 2]), rng.integers(0, M, 2000)]).astype(np.uint64)
    hs = hash_rng.hash_u32(vs)
    for v, h in zip(vs.tolist(), hs.tolist()):
        assert _invert_hash_u32(int(h)) == int(v)


def test_hash_u32x2_is_inverted_by_the_permutation_steps():
    rng = np.random.default_rng(2)
    xs = rng.integers(0, M, 2000).astype(np.uint64)
    ys = np.concatenate([np.ones(1000, dtype=np.uint64), rng.integers(0, M, 1000).astype(np.uint64)])
    hx, hy = hash_rng.hash_u32x2(xs, ys)
    for x, y, a, b in zip(xs.tolist(), ys.tolist(), hx.tolist(), hy.tolist()):
        assert _invert_hash_u32x2(int(a), int(b)) == (int(x), int(y))


def test_hash_u32_has_no_collisions_on_consecutive_counters():
    # a random function on 32 bits would collide about n^2 / 2^33 = 2048 times here
    n = 1 << 22
    h = hash_rng.hash_u32(np.arange(n, dtype=np.uint64) + np.uint64(0xFFF00000))   # spans the 2^32 wrap
    assert np.unique(h).size == n


@pytest.mark.parametrize('bit', [0, 7, 16, 31])
def test_single_bit_avalanche(bit):
    v = np.arange(1 << 16, dtype=np.uint64) * np.uint64(2654435761) & np.uint64(M - 1)
    a, b = hash_rng.hash_u32(v), hash_rng.hash_u32(v ^ np.uint64(1 << bit))
    flipped = np.unpackbits((a ^ b).view(np.uint8)).sum() / v.size
    assert 13.0 < flipped < 19.0
    ax, ay = hash_rng.hash_u32x2(v, np.ones_like(v))
    bx, by = hash_rng.hash_u32x2(v ^ np.uint64(1 << bit), np.ones_like(v))
    # the 2-D hash mixes less in its low bits than the 1-D one; a changed counter must still move both halves
    assert np.unpackbits((ax ^ bx).view(np.uint8)).sum() / v.size > 8.0
    assert np.unpackbits((ay ^ by).view(np.uint8)).sum() / v.size > 8.0


def test_counter_wraps_modulo_2_32():
    seed = 0xFFFFFFF0
    a = hash_rng.random_uniform(64, seed)
    b = hash_rng.random_uniform(48, 0)
    assert np.array_equal(a[16:], b)          # element 16 has counter (16 + seed) mod 2^32 = 0


def test_uniform_distribution_and_affine_map():
    n = 1 << 20
    u = hash_rng.random_uniform(n, 12345)
    assert u.dtype == np.float32 and u.min() >= 0.0 and u.max() <= 1.0
    assert abs(u.mean() - 0.5) < 2e-3 and abs(u.var() - 1 / 12) < 1e-3
    assert stats.kstest(u[:200000].astype(np.float64), 'uniform').pvalue > 1e-3
    w = hash_rng.random_uniform(n, 12345, -0.25, 0.75)
    assert np.allclose(w, u.astype(np.float64) - 0.25, rtol=0, atol=1e-7)
    assert w.dtype == np.float32
    # neighbouring seeds shift the stream by one element: the value depends on counter + seed only
    assert np.array_equal(hash_rng.random_uniform(100, 8)[:-1], hash_rng.random_uniform(100, 7)[1:])


def test_normal_distribution_and_affine_map():
    n = 1 << 20
    z = hash_rng.random_normal(n, 999)
    z = z[np.isfinite(z)]
    assert z.size >= n - 2
    assert abs(z.mean()) < 4e-3 and abs(z.std() - 1.0) < 4e-3
    assert abs(stats.skew(z.astype(np.float64))) < 0.02 and abs(stats.kurtosis(z.astype(np.float64))) < 0.05
    assert stats.kstest(z[:200000].astype(np.float64), 'norm').pvalue > 1e-3
    w = hash_rng.random_normal(n, 999, 1.5, 0.1)
    ok = np.isfinite(w)
    assert np.allclose(w[ok], 1.5 + 0.1 * hash_rng.random_normal(n, 999)[ok].astype(np.float64), rtol=0, atol=1e-6)


def test_fma32_rounds_once():
    """The single-precision affine stage of both initialisers is one fused multiply-add: compare the helper with
    exact rational arithmetic, including products that sit exactly half-way between two floats before the addend
    breaks the tie (where rounding the product or the double sum first would go the other way)."""
    from fractions import Fraction
    rng = np.random.default_rng(7)
    a = rng.standard_normal(4000).astype(np.float32)
    b = rng.standard_normal(4000).astype(np.float32)
    c = (rng.standard_normal(4000) * 10.0 ** rng.integers(-12, 3, 4000)).astype(np.float32)
    # ties: (1 + 2^-12)^2 = 1 + 2^-11 + 2^-24 is half-way between two floats near 1; a tiny addend decides
    t = np.float32(1 + 2.0 ** -12)
    a = np.concatenate([a, np.full(4, t, np.float32)])
    b = np.concatenate([b, np.full(4, t, np.float32)])
    c = np.concatenate([c, np.array([2.0 ** -60, -2.0 ** -60, 0.0, 2.0 ** -100], np.float32)])
    got = hash_rng.fma32(a, b, c)

    def nearest_f32(q):
        lo = np.float32(float(q))                      # within one ulp of the answer
        cands = {float(lo), float(np.nextafter(lo, np.float32(np.inf))), float(np.nextafter(lo, np.float32(-np.inf)))}
        best = min(cands, key=lambda v: (abs(Fraction(v) - q), int(np.float32(v).view(np.uint32)) & 1))
        return np.float32(best)

    for x, y, z, g in zip(a.tolist(), b.tolist(), c.tolist(), got.tolist()):
        assert np.float32(g) == nearest_f32(Fraction(x) * Fraction(y) + Fraction(z)), (x, y, z)
    assert got[-4] != got[-3]      # the 2^-60 addends break the tie in opposite directions


def test_lr_dropout_mask_is_the_uniform_stream_against_a_threshold():
    """Optimizer.py:199-202 compares hash_float_uint(gid + seed) with lr_dropout: the mask is the uniform initialiser's
    unit stream (low 0, high 1) cut at the threshold, with the expected share of elements dropped; the counter wraps
    modulo 2**32 like the initialisers'."""
    n = 200000
    for seed, p in ((3, 0.25), (2147483647, 0.5), (4294967295 - 50, 0.9)):
        mask = hash_rng.lr_dropout_mask(n, seed, p)
        assert np.array_equal(mask, hash_rng.random_uniform(n, seed, 0.0, 1.0) <= np.float32(p))
        assert abs(mask.mean() - p) < 0.01
    assert not hash_rng.lr_dropout_mask(1000, 1, 0.0).any() or hash_rng.random_uniform(1000, 1).min() == 0.0
    assert hash_rng.lr_dropout_mask(1000, 1, 1.0).all()
