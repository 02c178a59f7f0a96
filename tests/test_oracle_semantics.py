"""Pins the CPU oracle's container semantics (no GPU): the reference's known answers, a
brute-force dict model, and the invariants the reference's tests assert."""
import numpy as np
import pytest

import scenario


@pytest.mark.parametrize("scn", scenario.load_scenarios(), ids=lambda s: s["name"])
def test_reference_known_answers(orc, scn):
    scenario.run(scn, lambda dim, opt: orc.Oracle(dim, opt, capacity=1 << 16), orc.predicate)


class DictModel:
    """Straight-line Python model of one shard under the SUM operator (pico-ps/test/TestOps.h:87-118)."""

    def __init__(self, dim):
        self.dim, self.d = dim, {}

    def pull(self, keys, insert=False):
        entry = set(self.d)
        rows, hit = [], []
        for k in keys:
            k = int(k)
            if k in self.d:
                rows.append(self.d[k].copy())
                hit.append(1 if k in entry else 0)
            else:
                rows.append(np.zeros(self.dim, np.float32))
                hit.append(0)
                if insert:
                    self.d[k] = np.zeros(self.dim, np.float32)
        return np.array(rows, np.float32).reshape(len(keys), self.dim), np.array(hit, np.uint8)

    def push(self, keys, grads, insert=True):
        agg = {}
        for k, g in zip(keys, grads):
            agg.setdefault(int(k), np.zeros(self.dim, np.float32))
            agg[int(k)] = agg[int(k)] + g
        for k, g in agg.items():
            if k not in self.d:
                if not insert:
                    continue
                self.d[k] = np.zeros(self.dim, np.float32)
            self.d[k] = self.d[k] + g


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_oracle_against_dict_model(orc, seed):
    rng = np.random.default_rng(seed)
    dim = 3
    o = orc.Oracle(dim, orc.OPT_SUM, capacity=4096)
    m = DictModel(dim)
    for it in range(40):
        n = int(rng.integers(1, 60))
        keys = rng.integers(0, 80, size=n).astype(np.uint64)  # small range: many duplicates
        kind = rng.integers(0, 4)
        if kind == 0:
            grads = rng.integers(-8, 9, size=(n, dim)).astype(np.float32)  # integers: sums exact
            assert o.push(keys, grads) == 0
            m.push(keys, grads)
        elif kind == 1:
            grads = rng.integers(-8, 9, size=(n, dim)).astype(np.float32)
            assert o.push(keys, grads, orc.PUSH_NO_INSERT) == 0
            m.push(keys, grads, insert=False)
        else:
            ins = kind == 3
            st, rows, hit = o.pull(keys, orc.PULL_INSERT_ON_MISS if ins else 0)
            er, eh = m.pull(keys, insert=ins)
            assert st == 0
            np.testing.assert_array_equal(rows, er)
            np.testing.assert_array_equal(hit, eh)
        assert o.size() == len(m.d)
    st, rec = o.dump()
    assert st == 0 and set(rec["key"].tolist()) == set(m.d)
    for r in rec:
        np.testing.assert_array_equal(r["value"], m.d[int(r["key"])])


def test_pull_is_readonly_by_default_and_idempotent(orc):
    o = orc.Oracle(4, orc.OPT_SUM, capacity=100)
    keys = np.arange(10, dtype=np.uint64)
    o.push(keys[:5], np.ones((5, 4), np.float32))
    for _ in range(3):  # pico-ps/test/ps_service_test.cpp:204-213: repeated pulls agree
        st, rows, hit = o.pull(keys)
        assert st == 0 and o.size() == 5
        np.testing.assert_array_equal(hit, [1] * 5 + [0] * 5)
        np.testing.assert_array_equal(rows[5:], 0)
        np.testing.assert_array_equal(rows[:5], 1)
    st, rows, hit = o.pull(np.array([7, 7, 8, 1], np.uint64), orc.PULL_INSERT_ON_MISS)
    np.testing.assert_array_equal(hit, [0, 0, 0, 1])  # mask is taken against the table at entry
    assert o.size() == 7
    st, rows, hit = o.pull(np.array([7, 8], np.uint64))
    np.testing.assert_array_equal(hit, [1, 1])


def test_read_only_table_never_inserts_on_pull(orc):
    o = orc.Oracle(2, orc.OPT_SUM, capacity=100, read_only=True)
    st, rows, hit = o.pull(np.array([1, 2], np.uint64), orc.PULL_INSERT_ON_MISS)
    assert st == 0 and o.size() == 0


def test_capacity_is_all_or_nothing(orc):
    o = orc.Oracle(2, orc.OPT_SUM, capacity=8)
    keys = np.arange(6, dtype=np.uint64)
    assert o.push(keys, np.ones((6, 2), np.float32)) == 0
    before = o.dump()[1].copy()
    # 2 present + 3 new > 8 - 6 free
    assert o.push(np.array([0, 1, 10, 11, 12], np.uint64), np.ones((5, 2), np.float32)) == orc.OUT_OF_MEMORY
    assert o.pull(np.array([20, 21, 22], np.uint64), orc.PULL_INSERT_ON_MISS)[0] == orc.OUT_OF_MEMORY
    assert o.set(np.array([30, 31, 32], np.uint64), np.ones((3, 2), np.float32)) == orc.OUT_OF_MEMORY
    after = o.dump()[1]
    np.testing.assert_array_equal(before, after)
    # exactly filling the table is fine; present keys never count
    assert o.push(np.array([0, 10, 11, 10], np.uint64), np.ones((4, 2), np.float32)) == 0
    assert o.size() == 8
    assert o.push(keys, np.ones((6, 2), np.float32)) == 0


def test_sync_store_equals_async_push_of_concatenation(orc):
    # pico-ps/operator/SparsePushOperator.h:374-409: store merges all queued blocks, then applies once
    rng = np.random.default_rng(5)
    a = orc.Oracle(2, orc.OPT_SUM, capacity=1000)
    b = orc.Oracle(2, orc.OPT_SUM, capacity=1000)
    ks, gs = [], []
    for _ in range(4):
        k = rng.integers(0, 50, size=30).astype(np.uint64)
        g = rng.integers(-4, 5, size=(30, 2)).astype(np.float32)
        assert a.queue(k, g) == 0
        ks.append(k)
        gs.append(g)
    assert a.size() == 0 and a.queued() == 120  # queued blocks do not touch the table
    assert a.store() == 0 and a.queued() == 0
    assert b.push(np.concatenate(ks), np.concatenate(gs)) == 0
    ra, rb = a.dump()[1], b.dump()[1]
    np.testing.assert_array_equal(np.sort(ra, order="key"), np.sort(rb, order="key"))
    assert a.store() == 0  # empty store is a no-op ack


def test_set_is_upsert_and_load_unique_rejects_present_keys(orc):
    o = orc.Oracle(2, orc.OPT_ADAGRAD, lr=0.1, init_acc=0.5, capacity=100)
    assert o.value_floats == 4
    keys = np.array([3, 4], np.uint64)
    vals = np.arange(8, dtype=np.float32).reshape(2, 4)
    assert o.set(keys, vals) == 0
    assert o.set(keys[:1], vals[1:]) == 0  # overwrite (safe_set, KVShardStorage.h:804-814)
    st, rec = o.dump()
    rec = np.sort(rec, order="key")
    np.testing.assert_array_equal(rec["value"], [vals[1], vals[1]])
    assert o.load(rec, orc.LOAD_UNIQUE) == orc.ERROR  # LoadOperator.h:194,210
    assert o.load(rec) == 0
    st, part = o.iterate(1, 5)
    assert st == 0 and part.size == 1  # a short batch marks the end (KVShardStorage.h:64-87)


def test_reserved_keys_are_rejected(orc):
    o = orc.Oracle(1, orc.OPT_SUM, capacity=10)
    bad = np.array([1, 0xFFFFFFFFFFFFFFFF], np.uint64)
    assert o.push(bad, np.ones((2, 1), np.float32)) == orc.ERROR
    assert o.pull(bad)[0] == orc.ERROR
    assert o.size() == 0


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_for_each_and_erase_against_dict_model(orc, seed):
    """for_each / erase_if / erase against a plain dict; the hooks are the reference's test
    operators generalised: count + column sums (pico-ps/test/TestOps.h:159-185), erase by a
    comparison on the key or a value column (TestOps.h:138-150 erases the odd keys)."""
    rng = np.random.default_rng(seed)
    dim = 3
    o = orc.Oracle(dim, orc.OPT_SUM, capacity=5000)
    model = {}
    keys = rng.integers(0, 3000, 2000).astype(np.uint64)
    vals = rng.integers(-9, 10, (2000, dim)).astype(np.float32)
    assert o.set(keys, vals) == 0
    for k, v in zip(keys, vals):
        model[int(k)] = v.copy()

    def check(where, fn):
        st, cnt, sums = o.for_each(where)
        sel = [v for k, v in model.items() if fn(k, v)]
        assert st == 0 and cnt == len(sel)
        np.testing.assert_array_equal(sums, np.sum(np.array(sel, dtype=np.float64).reshape(-1, dim), axis=0))

    check(None, lambda k, v: True)
    check(orc.predicate((orc.COL_KEY, orc.CMP_MOD_EQ, (2, 1))), lambda k, v: k % 2 == 1)
    check(orc.predicate((1, orc.CMP_GE, 3.0), (orc.COL_KEY, orc.CMP_LT, 1500)), lambda k, v: v[1] >= 3 and k < 1500)
    check(orc.predicate((0, orc.CMP_NE, 0.0), (2, orc.CMP_LE, -1.0), (1, orc.CMP_EQ, 2.0)),
          lambda k, v: v[0] != 0 and v[2] <= -1 and v[1] == 2)
    # erase_if: the odd keys (the reference's own hook), then a value column
    st, gone = o.erase_if(orc.predicate((orc.COL_KEY, orc.CMP_MOD_EQ, (2, 1))))
    odd = [k for k in model if k % 2 == 1]
    assert st == 0 and gone == len(odd)
    for k in odd:
        del model[k]
    st, gone = o.erase_if(orc.predicate((2, orc.CMP_GT, 4.0)))
    big = [k for k, v in model.items() if v[2] > 4]
    assert gone == len(big)
    for k in big:
        del model[k]
    # erase of chosen keys: repeats and absent keys are ignored
    victims = np.array(list(model)[:300] + list(model)[:5] + [999_999, 888_888], dtype=np.uint64)
    st, gone = o.erase(victims)
    assert st == 0 and gone == 300
    for k in list(model)[:300]:
        del model[k]
    assert o.size() == len(model)
    st, rec = o.dump()
    assert sorted(rec["key"].tolist()) == sorted(model)
    for k, v in zip(rec["key"], rec["value"]):
        np.testing.assert_array_equal(v, model[int(k)])
    st, rows, hit = o.pull(np.array(odd[:50] + list(model)[:50], dtype=np.uint64))
    assert not hit[:50].any() and hit[50:].all() and not rows[:50].any()
    check(None, lambda k, v: True)
    assert o.erase_if(None) == (0, len(model)) and o.size() == 0
    o.close()
