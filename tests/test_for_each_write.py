"""Writing for-each (pico-ps/operator/ForEachOperator.h:277-359) with the declarative hook: an
affine map or a clamp on a column range of the records that satisfy a predicate."""
import numpy as np
import pytest


def _cases(mod, vf):
    return [
        (mod.update(mod.UPD_AFFINE, 0, vf, 0.5, 0.0), None),                                   # decay everything
        (mod.update(mod.UPD_AFFINE, vf - 1, 1, 0.0, 0.125), mod.predicate((0, mod.CMP_GT, 0.0))),  # reset one column
        (mod.update(mod.UPD_CLAMP, 0, min(2, vf), -1.5, 2.25), mod.predicate((mod.COL_KEY, mod.CMP_MOD_EQ, (3, 2)))),
        (mod.update(mod.UPD_AFFINE, 1 % vf, 1, -3.0, 7.0), mod.predicate((mod.COL_KEY, mod.CMP_EQ, 1))),   # no record
        (mod.update(mod.UPD_AFFINE, 0, 0, 2.0, 2.0), None),                                     # no column
    ]


def _model(vals, keys, what, where_fn):
    out = vals.copy()
    sel = np.array([where_fn(int(k), v) for k, v in zip(keys, vals)], dtype=bool)
    c0, c1 = what.first_column, what.first_column + what.n_columns
    if what.op == 0:
        out[sel, c0:c1] = (np.float32(what.a) * vals[sel, c0:c1]).astype(np.float32) + np.float32(what.b)
    else:
        out[sel, c0:c1] = np.minimum(np.maximum(vals[sel, c0:c1], np.float32(what.a)), np.float32(what.b))
    return out.astype(np.float32), int(sel.sum())


WHERE = [
    lambda k, v: True,
    lambda k, v: v[0] > 0.0,
    lambda k, v: k % 3 == 2,
    lambda k, v: k == 1,
    lambda k, v: True,
]


def _run(make, mod, wl, dim):
    rng = np.random.default_rng(dim)
    b = make(dim)
    vf = b.value_floats
    n = 5003
    keys = wl.table_keys_np(0, n, seed=7)
    vals = rng.normal(0, 2.0, (n, vf)).astype(np.float32)
    assert b.set(keys, vals) == 0
    for (what, where), fn in zip(_cases(mod, vf), WHERE):
        st, rec = b.dump()
        order = np.argsort(rec["key"])
        before_k, before_v = rec["key"][order], rec["value"][order]
        want, cnt = _model(before_v, before_k, what, fn)
        assert b.for_each_write(what, where) == (0, cnt)
        st, rec = b.dump()
        order = np.argsort(rec["key"])
        np.testing.assert_array_equal(rec["key"][order], before_k)
        np.testing.assert_array_equal(rec["value"][order].view(np.uint32), want.view(np.uint32))
    # refused: columns out of range, unknown operation
    assert b.for_each_write(mod.update(mod.UPD_AFFINE, vf, 1, 1.0, 0.0))[0] == 1
    assert b.for_each_write(mod.update(7, 0, 1, 1.0, 0.0))[0] == 1
    b.close()


@pytest.mark.parametrize("dim", [1, 6])
def test_oracle_for_each_write(orc, wl, dim):
    _run(lambda d: orc.Oracle(d, orc.OPT_ADAGRAD, lr=0.1, init_acc=0.1, capacity=8000), orc, wl, dim)


@pytest.mark.gpu
@pytest.mark.parametrize("dim", [1, 6, 16, 130])
def test_gpu_for_each_write(ps, wl, dim):
    _run(lambda d: ps.Table(d, ps.OPT_ADAGRAD, lr=0.1, init_acc=0.1, capacity=8000), ps, wl, dim)
