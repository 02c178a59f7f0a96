"""Row handles (pshbm_pull_dev_handles -> pshbm_push_dev_handles), through the C ABI: a push that
takes the rows an earlier pull of the same keys found must leave the table exactly as the oracle's
pull + push of that batch does (the reference looks every key up both times,
pico-ps/operator/SparsePullOperator.h:214 and SparsePushOperator.h:248), whatever happened to the
table in between. Bars as everywhere: key sets and pulled rows bit-exact, pushed values bit-exact
with integer gradients and within 1e-6 relative / 1e-7 absolute of the exactly aggregated result
otherwise."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-6, 1e-7
OPTS = {
    "sum": dict(optimizer=0),
    "sgd": dict(optimizer=1, lr=0.01),
    "adagrad": dict(optimizer=2, lr=0.05, init_acc=0.1),
    "ftrl": dict(optimizer=3, alpha=0.05, beta=1.0, l1=1e-4, l2=1e-5),
}


def sorted_dump(b):
    st, rec = b.dump()
    assert st == 0
    return np.sort(rec, order="key")


def same(t, r, exact):
    a, b = sorted_dump(t), sorted_dump(r)
    np.testing.assert_array_equal(a["key"], b["key"])
    if exact:
        np.testing.assert_array_equal(a["value"], b["value"])
    else:
        np.testing.assert_allclose(a["value"], b["value"], rtol=RTOL, atol=ATOL)


def fill(t, r, wl, rng, n_table, opt, dim, seed):
    keys = wl.table_keys_np(0, n_table, seed=seed)
    vals = rng.normal(0, 0.01, (n_table, t.value_floats)).astype(np.float32)
    if opt == "adagrad":
        vals[:, dim:] = 0.1
    if opt == "ftrl":
        vals[:, 2 * dim:] = vals[:, dim:2 * dim] ** 2
    assert t.set(keys, vals) == 0 and r.set(keys, vals) == 0
    return keys


class Dev:
    """A batch on the device: keys, gradients, room for the pulled rows and the handles."""

    def __init__(self, q, g, dim):
        self.n = len(q)
        self.keys = torch.from_numpy(q.view(np.int64)).cuda()
        self.grads = torch.from_numpy(g).cuda()
        self.rows = torch.empty(self.n, dim, device="cuda")
        self.hit = torch.empty(self.n, dtype=torch.uint8, device="cuda")
        self.handles = torch.empty(self.n, dtype=torch.int32, device="cuda")
        self.stream = torch.cuda.current_stream().cuda_stream

    def pull(self, t, flags=0):
        st, epoch = t.pull_dev_handles(self.keys.data_ptr(), self.n, self.rows.data_ptr(), self.handles.data_ptr(),
                                       self.hit.data_ptr(), flags, self.stream)
        assert st == 0, t.last_error()
        torch.cuda.synchronize()
        return epoch

    def push(self, t, epoch, flags=0):
        st = t.push_dev_handles(self.keys.data_ptr(), self.grads.data_ptr(), self.handles.data_ptr(), epoch, self.n,
                                flags, self.stream)
        assert st == 0, t.last_error()
        torch.cuda.synchronize()


def batch(wl, rng, n_table, n, s, dim, seed, fresh, integer=False):
    q = wl.zipf_batch_np(rng, n_table, s, n, seed=seed)
    nf = int(n * fresh)
    if nf:
        q[:nf] = wl.fresh_keys_np(rng, nf)         # keys the pull misses and the push inserts
        q[nf:nf + nf // 4] = q[:nf // 4]           # some of them more than once
        rng.shuffle(q)
    if integer:
        g = rng.integers(-3, 4, (n, dim)).astype(np.float32)
    else:
        g = rng.normal(0, 1e-3, (n, dim)).astype(np.float32)
    return q, g


@pytest.mark.parametrize("opt,dim,s,fresh", [("sgd", 16, 1.05, 0.0), ("adagrad", 64, 1.2, 0.1), ("ftrl", 8, 1.1, 0.05),
                                             ("sgd", 3, 1.3, 0.1), ("adagrad", 128, 1.1, 0.0)])
@pytest.mark.parametrize("verify", [False, True])
def test_pull_then_push_with_handles(ps, orc, wl, opt, dim, s, fresh, verify):
    rng = np.random.default_rng(dim + 7)
    n_table, n = 60000, 40000 if dim <= 64 else 20000
    t = ps.Table(dim, capacity=n_table + 3 * n, max_batch=n, **OPTS[opt])
    r = orc.Oracle(dim, capacity=n_table + 3 * n, **OPTS[opt])
    fill(t, r, wl, rng, n_table, opt, dim, seed=5)
    for step in range(3):
        q, g = batch(wl, rng, n_table, n, s, dim, 5, fresh)
        d = Dev(q, g, dim)
        epoch = d.pull(t)
        st, rows, hit = r.pull(q)
        assert st == 0
        if step == 0:   # the tables are bit-identical until the first push of floating-point sums
            np.testing.assert_array_equal(d.rows.cpu().numpy().view(np.uint32), rows.view(np.uint32))
        else:
            np.testing.assert_allclose(d.rows.cpu().numpy(), rows, rtol=RTOL, atol=ATOL)
        np.testing.assert_array_equal(d.hit.cpu().numpy(), hit)
        # a handle is a row number for a key the table holds, "none" for the others
        h = d.handles.cpu().numpy().view(np.uint32)
        assert ((h != 0xFFFFFFFF) == hit.astype(bool)).all()
        flags = (ps.PUSH_NO_INSERT if step == 2 else 0)
        d.push(t, epoch, flags | (ps.PUSH_VERIFY_HANDLES if verify else 0))
        assert r.push(q, g, flags | orc.PUSH_EXACT_AGGREGATION) == 0
        same(t, r, exact=False)
        assert t.size() == r.size()
    t.close()


@pytest.mark.parametrize("dim", [4, 16])
def test_handles_with_integer_gradients_bit_exact(ps, orc, wl, dim):
    """Integer sums are exact in any order (pico-ps/test/TestOps.h:98-117): every value bit for bit."""
    rng = np.random.default_rng(dim + 31)
    n_table, n = 50000, 70000
    t = ps.Table(dim, capacity=n_table + 2 * n, max_batch=n, **OPTS["sum"])
    r = orc.Oracle(dim, capacity=n_table + 2 * n, **OPTS["sum"])
    fill(t, r, wl, rng, n_table, "sum", dim, seed=6)
    for step in range(2):
        q, g = batch(wl, rng, n_table, n, 1.2, dim, 6, 0.08, integer=True)
        q[::5] = q[0]                                 # one key fills a fifth of the batch
        d = Dev(q, g, dim)
        epoch = d.pull(t)
        d.push(t, epoch)
        assert r.push(q, g) == 0
        same(t, r, exact=True)
    t.close()


def test_handles_survive_insertions_and_die_with_an_erase(ps, orc, wl):
    """Between the pull and the push: other keys are inserted (rows never move: the handles stay
    good, the epoch is the same), then keys are erased (rows move into the holes: a new epoch, and
    the push must look every key up again -- with the old handles it would update other keys'
    rows)."""
    dim, opt = 16, "sgd"
    rng = np.random.default_rng(3)
    n_table, n = 60000, 30000
    t = ps.Table(dim, capacity=n_table + 4 * n, max_batch=n, **OPTS[opt])
    r = orc.Oracle(dim, capacity=n_table + 4 * n, **OPTS[opt])
    keys = fill(t, r, wl, rng, n_table, opt, dim, seed=8)

    q, g = batch(wl, rng, n_table, n, 1.1, dim, 8, 0.0)
    d = Dev(q, g, dim)
    epoch = d.pull(t)
    extra = wl.fresh_keys_np(rng, 5000)
    ev = rng.normal(0, 0.01, (5000, t.value_floats)).astype(np.float32)
    assert t.set(extra, ev) == 0 and r.set(extra, ev) == 0
    d2 = Dev(q[:16], g[:16], dim)
    assert d2.pull(t) == epoch                       # insertions begin no new epoch
    d.push(t, epoch)
    assert r.push(q, g, orc.PUSH_EXACT_AGGREGATION) == 0
    same(t, r, exact=False)

    q, g = batch(wl, rng, n_table, n, 1.1, dim, 8, 0.0)
    d = Dev(q, g, dim)
    epoch = d.pull(t)
    gone = keys[1000:9000]                           # low rows: the last rows of the slab move into them
    st, erased = t.erase(gone)
    assert st == 0 and erased == len(gone)
    assert r.erase(gone)[1] == len(gone)
    assert d2.pull(t) != epoch
    d.push(t, epoch)                                 # stale handles: ignored; erased keys come back as new ones
    assert r.push(q, g, orc.PUSH_EXACT_AGGREGATION) == 0
    same(t, r, exact=False)
    assert t.size() == r.size()
    t.close()


def test_verify_rejects_handles_of_other_keys(ps, orc, wl):
    """A handle array that belongs to another key array: with PSHBM_PUSH_VERIFY_HANDLES the push
    notices (the row's key is not the batch key) and looks those keys up instead."""
    dim, opt = 8, "adagrad"
    rng = np.random.default_rng(11)
    n_table, n = 40000, 20000
    t = ps.Table(dim, capacity=n_table + 2 * n, max_batch=n, **OPTS[opt])
    r = orc.Oracle(dim, capacity=n_table + 2 * n, **OPTS[opt])
    fill(t, r, wl, rng, n_table, opt, dim, seed=9)
    q, g = batch(wl, rng, n_table, n, 1.1, dim, 9, 0.05)
    d = Dev(q, g, dim)
    epoch = d.pull(t)
    d.handles = torch.roll(d.handles, 1)              # every handle now names the row of the key before
    d.push(t, epoch, ps.PUSH_VERIFY_HANDLES)
    assert r.push(q, g, orc.PUSH_EXACT_AGGREGATION) == 0
    same(t, r, exact=False)
    t.close()


def test_handles_are_ignored_by_small_batches(ps, orc, wl):
    dim, opt = 16, "ftrl"
    rng = np.random.default_rng(12)
    n_table = 20000
    t = ps.Table(dim, capacity=n_table + 20000, **OPTS[opt])
    r = orc.Oracle(dim, capacity=n_table + 20000, **OPTS[opt])
    fill(t, r, wl, rng, n_table, opt, dim, seed=10)
    for n in (300, 6000):                             # the one-launch push, the sorted push
        q, g = batch(wl, rng, n_table, n, 1.1, dim, 10, 0.1, integer=True)   # exact sums: bit for bit
        d = Dev(q, g, dim)
        epoch = d.pull(t)
        d.push(t, epoch)
        assert r.push(q, g) == 0
        same(t, r, exact=True)
    t.close()


@pytest.mark.parametrize("verify", [False, True])
def test_handles_in_partitions_that_need_several_passes(ps, orc, wl, verify):
    """With the pass capacity turned down every partition takes the several-passes path (entries
    chosen by hash class, a class at a time): the handles travel with the chosen entries."""
    dim, opt = 16, "sgd"
    rng = np.random.default_rng(14)
    n_table, n = 40000, 60000
    t = ps.Table(dim, capacity=n_table + n, max_batch=n, **OPTS[opt])
    r = orc.Oracle(dim, capacity=n_table + n, **OPTS[opt])
    fill(t, r, wl, rng, n_table, opt, dim, seed=15)
    q, g = batch(wl, rng, n_table, n, 1.05, dim, 15, 0.05, integer=True)
    d = Dev(q, g, dim)
    epoch = d.pull(t)
    try:
        ps.debug_part_pass_capacity(256)
        d.push(t, epoch, ps.PUSH_VERIFY_HANDLES if verify else 0)
    finally:
        ps.debug_part_pass_capacity(0)
    assert r.push(q, g) == 0
    same(t, r, exact=True)
    assert t.size() == r.size()
    t.close()


def test_handles_with_track_increment_and_a_second_table(ps, orc, wl):
    """Two tables on the device, each with its own handles and epoch; pushes mark what they touch."""
    dim, opt = 8, "adagrad"
    rng = np.random.default_rng(16)
    n_table, n = 30000, 20000
    tabs = [ps.Table(dim, capacity=n_table + n, max_batch=n, track_increment=True, **OPTS[opt]) for _ in range(2)]
    refs = [orc.Oracle(dim, capacity=n_table + n, track_increment=True, **OPTS[opt]) for _ in range(2)]
    for t, r, seed in zip(tabs, refs, (17, 18)):
        fill(t, r, wl, rng, n_table, opt, dim, seed=seed)
        t.take_increment(), r.take_increment()
    work = []
    for t, seed in zip(tabs, (17, 18)):
        q, g = batch(wl, rng, n_table, n, 1.1, dim, seed, 0.02)
        d = Dev(q, g, dim)
        work.append((d, d.pull(t), q, g))
    for (d, epoch, q, g), t, r in zip(work, tabs, refs):      # the pushes after both pulls
        d.push(t, epoch)
        assert r.push(q, g, orc.PUSH_EXACT_AGGREGATION) == 0
        same(t, r, exact=False)
        st, rec = t.take_increment()
        st2, rec2 = r.take_increment()
        assert st == st2 == 0
        np.testing.assert_array_equal(np.sort(rec["key"]), np.sort(rec2["key"]))
    for t in tabs:
        t.close()
