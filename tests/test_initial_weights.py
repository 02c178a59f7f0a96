"""Initial weights of new keys (init_range > 0): the oracle's formula against an integer-only
restatement, MurmurHash3's published finalizer value, the bounds and moments of the uniform
distribution, and the operator semantics around it (a pull that misses answers the weights an
insertion would store). The reference leaves the initial value to the user hook init_store_value
(pico-ps/operator/SparsePullOperator.h:307-310, SparsePushOperator.h:250-251) and ships only zeros,
so the formula is pinned by these checks, not by the reference. Runs without a GPU."""
import numpy as np
import pytest

M64 = (1 << 64) - 1


def fmix64(k):
    k ^= k >> 33
    k = k * 0xFF51AFD7ED558CCD & M64
    k ^= k >> 33
    k = k * 0xC4CEB9FE1A85EC53 & M64
    k ^= k >> 33
    return k


def model_weight(init_range, key, col):
    """Integers up to the 24-bit draw; then exactly two fp32 roundings (the draw maps to [-1, 1)
    without rounding: it is a multiple of 2^-23 below 2 in magnitude)."""
    h = fmix64(key ^ ((col + 1) * 0x9E3779B97F4A7C15 & M64))
    top = h >> 40
    unit = np.float32((top - (1 << 23)) / float(1 << 23))
    assert float(unit) == (top - (1 << 23)) / float(1 << 23)   # exact in fp32
    return np.float32(unit * np.float32(init_range))


def test_finalizer_matches_the_published_value():
    assert fmix64(0) == 0
    assert fmix64(1) == 0xB456BCFC34C2CB2C


def test_oracle_formula_matches_the_integer_model(orc):
    rng = np.random.default_rng(5)
    keys = [0, 1, 2, (1 << 64) - 3, 1 << 63, 0x9E3779B97F4A7C15] + [int(k) for k in rng.integers(0, 1 << 63, 300, dtype=np.uint64)]
    for r in (1.0, 0.01, 0.25, 3.0e-5, 1000.0, float(np.float32(0.1))):
        for k in keys:
            for c in (0, 1, 7, 63, 16383):
                assert np.float32(orc.init_weight(r, k, c)) == model_weight(r, k, c), (r, k, c)


def test_library_host_function_matches_the_oracle(ps, orc):
    rng = np.random.default_rng(6)
    for _ in range(2000):
        k = int(rng.integers(0, 1 << 63, dtype=np.uint64)) * 2 + int(rng.integers(0, 2))
        c = int(rng.integers(0, 16384))
        r = float(np.float32(rng.uniform(1e-4, 2.0)))
        assert ps.init_weight(r, k, c) == orc.init_weight(r, k, c)


def test_bounds_and_moments(orc):
    r = 0.05
    o = orc.Oracle(64, capacity=4096, init_range=r)
    keys = np.arange(1, 4097, dtype=np.uint64) * np.uint64(0x100000001B3)
    st, rows, hit = o.pull(keys)
    assert st == 0 and not hit.any()
    w = rows.astype(np.float64).ravel()
    assert (w >= -r).all() and (w < r).all()
    n = w.size
    # uniform on [-r, r): mean 0 (sd r / sqrt(3 n)), variance r^2 / 3
    assert abs(w.mean()) < 5 * r / np.sqrt(3 * n)
    assert abs(w.var() / (r * r / 3) - 1) < 0.02
    # columns and keys decorrelate: neighbouring columns, neighbouring keys
    assert abs(np.corrcoef(rows[:, 0], rows[:, 1])[0, 1]) < 0.08
    assert abs(np.corrcoef(rows[:-1, 3], rows[1:, 3])[0, 1]) < 0.08
    # no two keys share a row
    assert np.unique(rows, axis=0).shape[0] == keys.size


@pytest.mark.parametrize("optimizer,extra", [(1, dict(lr=0.5)), (2, dict(lr=0.5, init_acc=0.1)),
                                             (3, dict(alpha=0.05, beta=1.0, l1=0.0, l2=0.0))])
def test_operator_semantics(orc, optimizer, extra):
    dim, r = 8, 0.25
    o = orc.Oracle(dim, optimizer=optimizer, capacity=64, init_range=r, **extra)
    keys = np.array([11, 22, 33], np.uint64)
    w0 = np.array([[orc.init_weight(r, int(k), c) for c in range(dim)] for k in keys], np.float32)
    st, rows, hit = o.pull(keys)                               # a miss answers the initial weights
    assert st == 0 and not hit.any() and o.size() == 0
    np.testing.assert_array_equal(rows, w0)
    st, rows, hit = o.pull(keys[:2], orc.PULL_INSERT_ON_MISS)  # ... and an inserting pull stores them
    assert st == 0 and o.size() == 2
    np.testing.assert_array_equal(rows, w0[:2])
    g = np.zeros((3, dim), np.float32)
    assert o.push(keys, g) == 0                                # key 33 is inserted by the push
    st, rows, hit = o.pull(keys)
    assert hit.all()
    if optimizer != 3:                                         # a zero gradient leaves SGD / Adagrad weights alone
        np.testing.assert_array_equal(rows, w0)
    rec = np.sort(o.dump()[1], order="key")
    if optimizer == 2:
        np.testing.assert_array_equal(rec["value"][:, dim:], np.full((3, dim), 0.1, np.float32))
    if optimizer == 1:                                         # one SGD step from the initial weights
        g[:] = 1.0
        assert o.push(keys, g) == 0
        np.testing.assert_array_equal(o.pull(keys)[1], w0 - np.float32(0.5))


def test_zero_range_is_zero_weights(orc):
    o = orc.Oracle(4, capacity=16)
    st, rows, hit = o.pull(np.array([5, 6], np.uint64))
    assert not rows.any()
    with pytest.raises(ValueError):
        orc.Oracle(4, capacity=16, init_range=-1.0)
    with pytest.raises(ValueError):
        orc.Oracle(4, capacity=16, init_range=float("inf"))
