"""The increment: which keys pushes touched since the last take (the reference's second storage,
pico-ps/operator/SparsePushOperator.h:253-266,394-407, read and emptied by the sync operator,
pico-ps/service/IncrementStorage.h:29-36)."""
import numpy as np
import pytest


def _run(make, wl, mod):
    rng = np.random.default_rng(5)
    dim = 4
    b = make(dim)
    keys = wl.table_keys_np(0, 3000, seed=3)
    vals = rng.integers(-5, 6, (3000, dim)).astype(np.float32)
    assert b.set(keys, vals) == 0
    assert b.increment_size() == (0, 0)                      # set is not part of the increment
    st, rows, hit = b.pull(wl.fresh_keys_np(rng, 50), mod.PULL_INSERT_ON_MISS)
    assert b.increment_size() == (0, 0)                      # neither is an inserting pull
    model = {int(k): v.astype(np.float64) for k, v in zip(keys, vals)}
    touched = set()

    def push(q, g, flags=0, store=False):
        if store:
            assert b.queue(q, g) == 0 and b.store(flags) == 0
        else:
            assert b.push(q, g, flags) == 0
        for k, x in zip(q, g):
            k = int(k)
            if k not in model:
                if flags & mod.PUSH_NO_INSERT:
                    continue
                model[k] = np.zeros(dim)
            model[k] = model[k] + x
            touched.add(k)

    def take_and_check():
        st, n = b.increment_size()
        assert st == 0 and n == len(touched)
        st, rec = b.take_increment()
        assert st == 0 and rec.size == len(touched)
        assert set(rec["key"].tolist()) == touched
        for k, v in zip(rec["key"], rec["value"]):
            np.testing.assert_array_equal(v, model[int(k)].astype(np.float32))
        touched.clear()
        assert b.increment_size() == (0, 0)
        assert b.take_increment()[1].size == 0

    q = np.concatenate([keys[rng.integers(0, 3000, 4000)], wl.fresh_keys_np(rng, 200)])
    push(q, rng.integers(-3, 4, (q.size, dim)).astype(np.float32))
    take_and_check()
    # two pushes and a store between takes; a push that may not insert drops its new keys
    q = keys[rng.integers(0, 3000, 500)]
    push(q, rng.integers(-3, 4, (q.size, dim)).astype(np.float32))
    q = np.concatenate([keys[:100], wl.fresh_keys_np(rng, 30)])
    push(q, rng.integers(-3, 4, (q.size, dim)).astype(np.float32), mod.PUSH_NO_INSERT)
    q = np.concatenate([keys[2000:2300], keys[2000:2100]])
    push(q, rng.integers(-3, 4, (q.size, dim)).astype(np.float32), store=True)
    # too little room: nothing is taken
    st, rec = b.take_increment(capacity=3)
    assert st != 0 and b.increment_size()[1] == len(touched)
    take_and_check()
    # erased keys leave the increment; the marks of the rows that move follow them
    q = keys[rng.integers(0, 3000, 1500)]
    push(q, rng.integers(-3, 4, (q.size, dim)).astype(np.float32))
    victims = keys[::3]
    st, gone = b.erase(victims)
    assert st == 0
    for k in victims:
        model.pop(int(k), None)
        touched.discard(int(k))
    take_and_check()
    assert b.clear() == 0 and b.increment_size() == (0, 0)
    b.close()


def test_oracle_increment(orc, wl):
    _run(lambda dim: orc.Oracle(dim, orc.OPT_SUM, capacity=8000, track_increment=True), wl, orc)


@pytest.mark.gpu
def test_gpu_increment(ps, wl):
    _run(lambda dim: ps.Table(dim, ps.OPT_SUM, capacity=8000, track_increment=True), wl, ps)


@pytest.mark.gpu
def test_gpu_increment_needs_the_option(ps):
    t = ps.Table(4, ps.OPT_SUM, capacity=100)
    assert t.increment_size()[0] != 0 and t.take_increment(10)[0] != 0
    t.close()
