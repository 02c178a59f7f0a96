"""Pins the optimizer arithmetic of the oracle (no GPU). The reference ships no optimizer, so the
formulas are this repository's; what pins them here: hand-computed single-key numbers, algebraic
identities that a dropped term, a wrong sign or a swapped state block would break, and an
independent float64 evaluation."""
import math

import numpy as np
import pytest

K = np.array([42], np.uint64)


def one(orc, opt, w0, g, state=None, **kw):
    """value after one push of gradient g on a key holding w0 (+state)"""
    o = orc.Oracle(1, opt, capacity=4, **kw)
    v0 = [w0] + list(state or [])
    assert o.set(K, np.array([v0], np.float32)) == 0
    assert o.push(K, np.array([[g]], np.float32)) == 0
    return o.dump()[1]["value"][0]


def test_sgd_hand_computed(orc):
    v = one(orc, orc.OPT_SGD, 1.0, 0.5, lr=0.01)
    assert v[0] == pytest.approx(0.995, rel=1e-7)
    assert v[0] == np.float32(1.0) - np.float32(0.01) * np.float32(0.5)  # two roundings, no fma


def test_adagrad_hand_computed(orc):
    v = one(orc, orc.OPT_ADAGRAD, 1.0, 0.3, state=[0.1], lr=0.05, init_acc=0.1)
    assert v[1] == pytest.approx(0.19, rel=1e-6)          # n = 0.1 + 0.3^2
    assert v[0] == pytest.approx(0.96558764, rel=1e-6)    # 1 - 0.05*0.3/sqrt(0.19)


def test_ftrl_hand_computed_from_zero_state(orc):
    kw = dict(alpha=0.05, beta=1.0, l1=1e-4, l2=1e-5)
    v = one(orc, orc.OPT_FTRL, 0.0, 0.5, state=[0.0, 0.0], **kw)
    # n = 0.25, sigma = 0.5/0.05 = 10, z = 0.5 - 10*0 = 0.5, w = -(0.5-1e-4)/((1+0.5)/0.05 + 1e-5)
    assert v[2] == pytest.approx(0.25, rel=1e-7)
    assert v[1] == pytest.approx(0.5, rel=1e-7)
    assert v[0] == pytest.approx(-0.016663327779, rel=1e-6)
    # |z| <= l1 gives exactly zero weight (the sparsity FTRL exists for)
    v = one(orc, orc.OPT_FTRL, 0.0, 5e-5, state=[0.0, 0.0], **kw)
    assert v[0] == 0.0 and v[1] == pytest.approx(5e-5, rel=1e-6)


def test_fresh_key_starts_from_zero_weights_and_init_state(orc):
    g = np.array([[0.25, -0.5]], np.float32)
    o = orc.Oracle(2, orc.OPT_ADAGRAD, lr=0.1, init_acc=0.1, capacity=4)
    assert o.push(K, g) == 0
    v = o.dump()[1]["value"][0]
    np.testing.assert_allclose(v[2:], [0.1 + 0.0625, 0.1 + 0.25], rtol=1e-6)
    np.testing.assert_allclose(v[:2], [-0.1 * 0.25 / math.sqrt(0.1625), 0.1 * 0.5 / math.sqrt(0.35)], rtol=1e-6)
    # a pull-inserted key holds zeros and the initial accumulator, and pulls zeros
    st, rows, hit = o.pull(np.array([7], np.uint64), orc.PULL_INSERT_ON_MISS)
    np.testing.assert_array_equal(rows, 0)
    rec = o.dump()[1]
    np.testing.assert_array_equal(rec[rec["key"] == 7]["value"][0], [0, 0, np.float32(0.1), np.float32(0.1)])


@pytest.mark.parametrize("opt,kw,state", [
    ("OPT_SGD", dict(lr=0.3), []),
    ("OPT_ADAGRAD", dict(lr=0.3, init_acc=0.1), [0.7]),
])
def test_zero_gradient_leaves_the_row_bit_identical(orc, opt, kw, state):
    v = one(orc, getattr(orc, opt), 0.123456789, 0.0, state=state, **kw)
    np.testing.assert_array_equal(v, np.array([0.123456789] + state, np.float32))


def test_sgd_is_linear_in_the_gradient(orc):
    rng = np.random.default_rng(0)
    g1, g2 = rng.normal(0, 1e-3, (2, 8)).astype(np.float32)
    a = orc.Oracle(8, orc.OPT_SGD, lr=0.01, capacity=4)
    b = orc.Oracle(8, orc.OPT_SGD, lr=0.01, capacity=4)
    a.push(K, g1[None]); a.push(K, g2[None])
    b.push(np.array([42, 42], np.uint64), np.stack([g1, g2]))   # aggregated in one batch
    np.testing.assert_allclose(a.dump()[1]["value"], b.dump()[1]["value"], rtol=1e-6, atol=1e-9)
    # direction and size: w = -lr * (g1 + g2)
    np.testing.assert_allclose(b.dump()[1]["value"][0], -0.01 * (g1.astype(np.float64) + g2), rtol=1e-6)


def test_adagrad_accumulates_squares_and_steps_against_the_gradient(orc):
    rng = np.random.default_rng(1)
    gs = rng.normal(0, 1e-2, (20, 4)).astype(np.float32)
    o = orc.Oracle(4, orc.OPT_ADAGRAD, lr=0.05, init_acc=0.1, capacity=4)
    w = np.zeros(4); n = np.full(4, 0.1)
    for g in gs:
        o.push(K, g[None])
        n = n + g.astype(np.float64) ** 2
        w = w - 0.05 * g / np.sqrt(n)
    v = o.dump()[1]["value"][0]
    np.testing.assert_allclose(v[4:], n, rtol=1e-6)
    np.testing.assert_allclose(v[:4], w, rtol=1e-5, atol=1e-8)


def test_ftrl_without_regularisation_is_per_coordinate_gradient_descent(orc):
    # McMahan et al. 2013: with l1 = l2 = beta = 0, FTRL-proximal is online gradient descent with
    # the learning rate alpha/sqrt(n_t). Adagrad with init_acc = 0 and lr = alpha is that descent.
    rng = np.random.default_rng(2)
    gs = rng.normal(0, 0.1, (30, 6)).astype(np.float32)
    f = orc.Oracle(6, orc.OPT_FTRL, alpha=0.07, beta=0.0, l1=0.0, l2=0.0, capacity=4)
    a = orc.Oracle(6, orc.OPT_ADAGRAD, lr=0.07, init_acc=0.0, capacity=4)
    for g in gs:
        f.push(K, g[None]); a.push(K, g[None])
    vf, va = f.dump()[1]["value"][0], a.dump()[1]["value"][0]
    np.testing.assert_allclose(vf[:6], va[:6], rtol=2e-4, atol=1e-6)   # weights
    np.testing.assert_allclose(vf[12:], va[6:], rtol=1e-6)             # n == sum of squares


def test_ftrl_float64_reevaluation(orc):
    rng = np.random.default_rng(3)
    al, be, l1, l2 = 0.05, 1.0, 1e-4, 1e-5
    o = orc.Oracle(5, orc.OPT_FTRL, alpha=al, beta=be, l1=l1, l2=l2, capacity=4)
    w = np.zeros(5); z = np.zeros(5); n = np.zeros(5)
    for _ in range(25):
        g = rng.normal(0, 1e-2, 5).astype(np.float32)
        o.push(K, g[None])
        g = g.astype(np.float64)
        sigma = (np.sqrt(n + g * g) - np.sqrt(n)) / al
        z = z + g - sigma * w
        n = n + g * g
        w = np.where(np.abs(z) <= l1, 0.0, -(z - np.sign(z) * l1) / ((be + np.sqrt(n)) / al + l2))
    v = o.dump()[1]["value"][0]
    np.testing.assert_allclose(v[:5], w, rtol=1e-4, atol=1e-7)
    np.testing.assert_allclose(v[5:10], z, rtol=1e-4, atol=1e-7)
    np.testing.assert_allclose(v[10:], n, rtol=1e-5)


def test_aggregation_is_sequential_input_order_sum(orc):
    # SparsePushOperator.h:134-141: occurrences are added in input order starting from zero
    g = np.array([[1e8], [1.0], [-1e8], [1.0]], np.float32)
    k = np.array([5, 5, 5, 5], np.uint64)
    uk, us = orc.aggregate(1, k, g)
    assert uk.tolist() == [5]
    expect = np.float32(0)
    for x in g[:, 0]:
        expect = np.float32(expect + x)
    assert us[0, 0] == expect == 1.0   # (1e8 + 1) rounds to 1e8; then -1e8; then + 1
    # integer test operator of the reference: arg = key pushed c times -> sum = key*c, count = c
    keys = np.repeat(np.arange(1, 50, dtype=np.uint64), 3)
    grads = np.stack([keys.astype(np.float32), np.ones(keys.size, np.float32)], axis=1)
    uk, us = orc.aggregate(2, keys, grads)
    np.testing.assert_array_equal(us[:, 0], uk.astype(np.float32) * 3)
    np.testing.assert_array_equal(us[:, 1], 3)


def test_user_rule_momentum_hand_computed(orc):
    """The rule shipped as the library's user hook (parameter-server_amd/csrc/user_opt.h), which the
    oracle mirrors: SGD with momentum, v = beta * v + g; w = w - lr * v. Parity unpinned by the
    reference (its update rule is user code); pinned by hand-computed steps, the closed form of a
    constant gradient, and the identity beta = 0 => plain SGD."""
    kw = dict(lr=0.1, beta=0.9)
    v = one(orc, orc.OPT_USER, 1.0, 0.5, state=[0.25], **kw)
    assert v[1] == pytest.approx(0.9 * 0.25 + 0.5, rel=1e-7)           # v = 0.725
    assert v[0] == pytest.approx(1.0 - 0.1 * 0.725, rel=1e-7)          # w = 0.9275
    # a fresh key starts at rest; n pushes of a constant g: v_n = g (1 - beta^n) / (1 - beta)
    o = orc.Oracle(1, orc.OPT_USER, capacity=4, **kw)
    w, vel = 0.0, 0.0
    for n in range(1, 6):
        assert o.push(K, np.array([[0.2]], np.float32)) == 0
        vel = 0.9 * vel + 0.2
        w -= 0.1 * vel
        got = o.dump()[1]["value"][0]
        assert got[1] == pytest.approx(0.2 * (1 - 0.9 ** n) / (1 - 0.9), rel=1e-6)
        assert got[0] == pytest.approx(w, rel=1e-6)
    # beta = 0: the weight follows plain SGD bit for bit
    a = one(orc, orc.OPT_USER, 0.3, -0.7, state=[123.0], lr=0.05, beta=0.0)
    b = one(orc, orc.OPT_SGD, 0.3, -0.7, lr=0.05)
    assert a[0] == b[0] and a[1] == np.float32(-0.7)
    assert orc.lib().pso_value_floats(8, orc.OPT_USER) == 16
