"""Parity of the HIP path with the CPU oracle, through the C ABI (needs an MI355X).

Bars: pulled rows, hit masks and stored key sets bit-exact; pushed values within 1e-6 relative /
1e-7 absolute of the oracle (aggregation order differs), and bit-exact wherever every key of a
batch is distinct or the gradients are integers.
"""
import numpy as np
import pytest

import scenario

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-6, 1e-7

OPTS = {
    "sum": dict(optimizer=0),
    "sgd": dict(optimizer=1, lr=0.01),
    "adagrad": dict(optimizer=2, lr=0.05, init_acc=0.1),
    "ftrl": dict(optimizer=3, alpha=0.05, beta=1.0, l1=1e-4, l2=1e-5),
    "user": dict(optimizer=4, lr=0.05, beta=0.9),   # the rule of csrc/user_opt.h: SGD with momentum
}


@pytest.fixture(autouse=True, params=["default", "sorted"])
def push_path(request, ps):
    """Every test of this file runs twice: with the library's own choice of push path (one launch up
    to 512 keys, the partitioned push above) and with mid-size and large batches sent through the
    sorted push (locate, radix sort, segmented reduce, fix-up), which otherwise only serves batches
    of more than 4M keys, nearly full tables and the entry point that allocates nothing."""
    ps.debug_part_min_keys((1 << 40) if request.param == "sorted" else 0)
    yield request.param
    ps.debug_part_min_keys(0)


def pair(ps, orc, dim, opt, capacity=1 << 16, **kw):
    o = OPTS[opt]
    t = ps.Table(dim, capacity=capacity, **o, **kw)
    r = orc.Oracle(dim, capacity=capacity, **o, **kw)
    return t, r


def sorted_dump(b):
    st, rec = b.dump()
    assert st == 0
    return np.sort(rec, order="key")


def assert_same_table(t, r, exact):
    a, b = sorted_dump(t), sorted_dump(r)
    np.testing.assert_array_equal(a["key"], b["key"])
    if exact:
        np.testing.assert_array_equal(a["value"], b["value"])
    else:
        np.testing.assert_allclose(a["value"], b["value"], rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("scn", scenario.load_scenarios(), ids=lambda s: s["name"])
def test_reference_known_answers(ps, scn):
    scenario.run(scn, lambda dim, opt: ps.Table(dim, opt, capacity=1 << 12), ps.predicate)


@pytest.mark.parametrize("dim", [1, 3, 4, 8, 16, 64, 128, 260])
def test_pull_bit_exact(ps, orc, wl, dim):
    rng = np.random.default_rng(dim)
    t, r = pair(ps, orc, dim, "sgd", capacity=5000)
    keys = wl.table_keys_np(0, 3000, seed=dim)
    vals = rng.normal(0, 0.01, (3000, dim)).astype(np.float32)
    assert t.set(keys, vals) == 0 and r.set(keys, vals) == 0
    assert t.size() == r.size() == 3000
    # hits, misses and duplicates, in a length that is not a multiple of the wave's 16 keys
    q = np.concatenate([keys[rng.integers(0, 3000, 777)], wl.fresh_keys_np(rng, 100), keys[:5], keys[:5]])
    rng.shuffle(q)
    st, rows, hit = t.pull(q)
    st2, rows2, hit2 = r.pull(q)
    assert st == st2 == 0
    np.testing.assert_array_equal(hit, hit2)
    np.testing.assert_array_equal(rows.view(np.uint32), rows2.view(np.uint32))
    assert t.size() == 3000  # a pull without the insert flag never inserts
    for n in (1, 15, 16, 17):
        st, rows, hit = t.pull(q[:n])
        np.testing.assert_array_equal(rows, rows2[:n])
        np.testing.assert_array_equal(hit, hit2[:n])
    t.close()


def test_pull_empty_and_all_miss(ps, orc):
    t, r = pair(ps, orc, 8, "sum", capacity=64)
    st, rows, hit = t.pull(np.array([], np.uint64))
    assert st == 0 and rows.shape == (0, 8)
    st, rows, hit = t.pull(np.arange(40, dtype=np.uint64))
    assert st == 0 and not rows.any() and not hit.any() and t.size() == 0
    t.close()


@pytest.mark.parametrize("dim", [2, 16])
def test_pull_insert_on_miss(ps, orc, wl, dim):
    rng = np.random.default_rng(3)
    t, r = pair(ps, orc, dim, "adagrad", capacity=4000)
    keys = wl.table_keys_np(0, 1000, seed=9)
    vals = rng.normal(0, 0.01, (1000, 2 * dim)).astype(np.float32)
    t.set(keys, vals), r.set(keys, vals)
    fresh = wl.fresh_keys_np(rng, 300)
    q = np.concatenate([keys[:200], fresh, fresh[:50], keys[100:150]])
    rng.shuffle(q)
    a = t.pull(q, ps.PULL_INSERT_ON_MISS)
    b = r.pull(q, orc.PULL_INSERT_ON_MISS)
    assert a[0] == b[0] == 0
    np.testing.assert_array_equal(a[1], b[1])
    np.testing.assert_array_equal(a[2], b[2])  # mask against the table at entry; duplicates share it
    assert t.size() == r.size() == 1300
    assert_same_table(t, r, exact=True)        # fresh rows: zero weights, accumulator = init_acc
    a, b = t.pull(q), r.pull(q)
    np.testing.assert_array_equal(a[2], b[2])
    assert a[2].all()
    # a read-only table ignores the flag
    t2 = ps.Table(dim, capacity=100, read_only=True)
    st, rows, hit = t2.pull(q[:50], ps.PULL_INSERT_ON_MISS)
    assert st == 0 and t2.size() == 0
    t.close(), t2.close()


@pytest.mark.parametrize("opt", ["sum", "sgd", "adagrad", "ftrl", "user"])
@pytest.mark.parametrize("dim", [1, 3, 8, 16, 64, 128, 260])
def test_push_unique_keys_bit_exact(ps, orc, wl, opt, dim):
    """With distinct keys there is nothing to aggregate: every value must match bit for bit."""
    rng = np.random.default_rng(dim * 7 + len(opt))
    t, r = pair(ps, orc, dim, opt, capacity=4000)
    keys = wl.table_keys_np(0, 1500, seed=1)
    for it in range(3):
        sel = rng.permutation(1500)[: 700 + it]
        g = rng.normal(0, 1e-2, (sel.size, dim)).astype(np.float32)
        assert t.push(keys[sel], g) == 0 and r.push(keys[sel], g) == 0
    assert t.push(keys[:300], g[:300], ps.PUSH_ASSUME_UNIQUE) == 0 and r.push(keys[:300], g[:300]) == 0
    assert_same_table(t, r, exact=True)
    t.close()


@pytest.mark.parametrize("dim", [1, 2, 3, 16, 64, 260])
def test_aggregation_exact_with_integer_gradients(ps, orc, dim):
    """The reference's own test operator: integer sums do not depend on the order of addition
    (pico-ps/test/TestOps.h:98-117), so heavy duplication must still match bit for bit."""
    rng = np.random.default_rng(dim)
    t, r = pair(ps, orc, dim, "sum", capacity=3000)
    for it in range(4):
        n = 5000 + 17 * it
        keys = rng.zipf(1.3, n).astype(np.uint64) % np.uint64(2000)   # a few keys repeat thousands of times
        g = rng.integers(-3, 4, (n, dim)).astype(np.float32)
        assert t.push(keys, g) == 0 and r.push(keys, g) == 0
    assert_same_table(t, r, exact=True)
    # one key only: a single run spanning every chunk of the segmented reduction; the long one also
    # spans many 64-chunk windows of the border fix-up, and shares the batch with two more long runs
    for n in (9000, 40000, 150000):
        keys = np.full(n, 77, np.uint64)
        keys[n // 2: n // 2 + n // 5] = 78
        keys[: n // 7] = 1999
        g = rng.integers(-3, 4, (n, dim)).astype(np.float32)
        assert t.push(keys, g) == 0 and r.push(keys, g) == 0
        assert_same_table(t, r, exact=True)
    t.close()


@pytest.mark.parametrize("n", [(1 << 20) + 1, 1_300_000, 2_500_000])
def test_aggregation_exact_large_batch(ps, orc, n):
    """Batches beyond 2^20 pairs take the sort's three-launch passes; the batch mixes one key that
    fills a tenth of it, skewed repeats, keys pushed for the first time more than once, and keys
    that are not stored and must be dropped (second push, no insertion)."""
    rng = np.random.default_rng(n)
    dim = 4
    t = ps.Table(dim, capacity=700_000, max_batch=n, **OPTS["sum"])
    r = orc.Oracle(dim, capacity=700_000, **OPTS["sum"])
    keys = (rng.zipf(1.1, n).astype(np.uint64) * np.uint64(2654435761)) % np.uint64(400_000)
    keys[rng.integers(0, n, n // 10)] = 123456789
    fresh = rng.integers(1 << 40, 1 << 41, 50_000).astype(np.uint64)
    keys[rng.integers(0, n, 120_000)] = fresh[rng.integers(0, fresh.size, 120_000)]
    g = rng.integers(-3, 4, (n, dim)).astype(np.float32)
    assert t.push(keys, g) == 0 and r.push(keys, g) == 0
    assert_same_table(t, r, exact=True)
    keys2 = keys.copy()
    keys2[::3] += np.uint64(1 << 50)                   # not stored
    g2 = rng.integers(-3, 4, (n, dim)).astype(np.float32)
    assert t.push(keys2, g2, ps.PUSH_NO_INSERT) == 0
    assert r.push(keys2, g2, orc.PUSH_NO_INSERT) == 0
    assert_same_table(t, r, exact=True)
    # smaller batches on the workspace of the large one: both sort schemes, and a tiny batch
    for m in (1 << 20, 300_000, 77):
        assert t.push(keys[:m], g[:m]) == 0 and r.push(keys[:m], g[:m]) == 0
    assert_same_table(t, r, exact=True)
    t.close()


def assert_push_parity(gpu, seq, exact, multiplicity=None, report=None):
    """gpu / seq / exact: key-sorted dumps after the same push from the same state, through the
    kernels, the oracle (sums duplicates sequentially in fp32, the reference's order:
    pico-ps/operator/SparsePushOperator.h:134-141) and the oracle with exactly rounded sums.
    Every value must be within RTOL/ATOL of the reference-order result or of the exactly rounded
    one: the sequential fp32 sum of thousands of terms is itself further than the tolerance from
    the exact sum, and an implementation that adds in another order cannot (and should not)
    follow it there. No value is excused. `report` collects how many values needed the second
    clause and how far both implementations are from the exact result."""
    np.testing.assert_array_equal(gpu["key"], seq["key"])
    np.testing.assert_array_equal(gpu["key"], exact["key"])
    g, s, e = (x["value"].astype(np.float64) for x in (gpu, seq, exact))
    near_seq = np.abs(g - s) <= ATOL + RTOL * np.abs(s)
    near_exact = np.abs(g - e) <= ATOL + RTOL * np.abs(e)
    if report is not None:
        report["values"] = report.get("values", 0) + g.size
        report["beyond_reference_order_tolerance"] = report.get("beyond_reference_order_tolerance", 0) + int((~near_seq).sum())
        report["worst_gpu_minus_exact"] = max(report.get("worst_gpu_minus_exact", 0.0), float(np.abs(g - e).max()))
        report["worst_reference_minus_exact"] = max(report.get("worst_reference_minus_exact", 0.0), float(np.abs(s - e).max()))
        if multiplicity is not None and (~near_seq).any():
            rows = np.unique(np.nonzero(~near_seq)[0])
            report["least_multiplicity_beyond"] = min(report.get("least_multiplicity_beyond", 1 << 60),
                                                      int(multiplicity[rows].min()))
    assert (near_seq | near_exact).all(), \
        "a pushed value is within the tolerance of neither the reference-order nor the exact result"


@pytest.mark.parametrize("opt", ["sgd", "adagrad", "ftrl", "user"])
@pytest.mark.parametrize("dim,s", [(16, 1.05), (64, 1.2), (8, 1.1), (128, 1.1)])
@pytest.mark.parametrize("batch", [30000, 800, 450])  # 450: the one-launch push
def test_push_zipf_within_tolerance(ps, orc, wl, opt, dim, s, batch):
    rng = np.random.default_rng(11)
    n_table = 20000
    t, r = pair(ps, orc, dim, opt, capacity=n_table + 4000)
    x = orc.Oracle(dim, capacity=n_table + 4000, **OPTS[opt])   # exactly rounded aggregation
    keys = wl.table_keys_np(0, n_table, seed=2)
    vf = t.value_floats
    vals = rng.normal(0, 0.01, (n_table, vf)).astype(np.float32)
    if opt == "adagrad":
        vals[:, dim:] = 0.1
    if opt == "ftrl":
        vals[:, 2 * dim:] = vals[:, dim:2 * dim] ** 2
    for b in (t, r, x):
        assert b.set(keys, vals) == 0
    for step in range(3):
        q = wl.zipf_batch_np(rng, n_table, s, batch, seed=2)
        nf = min(500, batch // 4)
        q[:nf] = wl.fresh_keys_np(rng, nf)              # insert-on-miss inside a push
        q[nf:nf + nf // 5] = q[:nf // 5]                # duplicated fresh keys
        g = rng.normal(0, 1e-3, (batch, dim)).astype(np.float32)
        assert t.push(q, g) == 0 and r.push(q, g) == 0
        assert x.push(q, g, orc.PUSH_EXACT_AGGREGATION) == 0
        st, rows, hit = t.pull(q[:4000])
        st2, rows2, hit2 = r.pull(q[:4000])
        np.testing.assert_array_equal(hit, hit2)
        a, b, c = sorted_dump(t), sorted_dump(r), sorted_dump(x)
        uk, cnt = np.unique(q, return_counts=True)
        mult = np.zeros(a.size, np.int64)
        mult[np.searchsorted(a["key"], uk)] = cnt
        assert_push_parity(a, b, c, mult)
        # whatever the multiplicity, the kernels stay within the tolerance of the exact result
        np.testing.assert_allclose(a["value"], c["value"], rtol=RTOL, atol=ATOL)
        # next step: everyone restarts from the reference-order state
        assert t.set(b["key"], b["value"]) == 0, t.last_error()
        assert x.set(b["key"], b["value"]) == 0
    assert t.size() == r.size()
    t.close()


def test_push_no_insert_drops_missing_keys(ps, orc, wl):
    rng = np.random.default_rng(4)
    t, r = pair(ps, orc, 4, "sgd", capacity=1000)
    keys = wl.table_keys_np(0, 100, seed=3)
    t.set(keys, np.zeros((100, 4), np.float32)), r.set(keys, np.zeros((100, 4), np.float32))
    q = np.concatenate([keys[:50], wl.fresh_keys_np(rng, 50)])
    g = rng.normal(0, 1, (100, 4)).astype(np.float32)
    assert t.push(q, g, ps.PUSH_NO_INSERT) == 0 and r.push(q, g, orc.PUSH_NO_INSERT) == 0
    assert t.size() == 100
    assert_same_table(t, r, exact=True)
    t.close()


def test_capacity_is_all_or_nothing(ps, orc):
    t, r = pair(ps, orc, 2, "sum", capacity=8)
    keys = np.arange(6, dtype=np.uint64)
    ones = lambda n: np.ones((n, 2), np.float32)
    assert t.push(keys, ones(6)) == 0 and r.push(keys, ones(6)) == 0
    for b in (t, r):
        assert b.push(np.array([0, 1, 10, 11, 12], np.uint64), ones(5)) == 3
        assert b.pull(np.array([20, 21, 22], np.uint64), 1)[0] == 3
        assert b.set(np.array([30, 31, 32], np.uint64), ones(3)) == 3
    assert "capacity" in t.last_error()
    assert_same_table(t, r, exact=True)
    for b in (t, r):
        assert b.push(np.array([0, 10, 11, 10], np.uint64), ones(4)) == 0
        assert b.size() == 8
        assert b.push(keys, ones(6)) == 0                      # present keys always fit
        assert b.push(np.array([99], np.uint64), ones(1)) == 3
    assert_same_table(t, r, exact=True)
    # the table keeps working after refusals: missing keys pull zeros
    st, rows, hit = t.pull(np.array([10, 12, 99], np.uint64))
    np.testing.assert_array_equal(hit, [1, 0, 0])
    t.close()


def test_sync_push_and_store(ps, orc, wl):
    rng = np.random.default_rng(6)
    t, r = pair(ps, orc, 8, "sgd", capacity=4000)
    for _ in range(5):
        k = rng.integers(0, 900, 1000).astype(np.uint64)
        g = rng.normal(0, 1e-3, (1000, 8)).astype(np.float32)
        assert t.queue(k, g) == 0 and r.queue(k, g) == 0
    assert t.size() == 0 and t.queued() == r.queued() == 5000
    assert t.store() == 0 and r.store() == 0
    assert t.queued() == 0
    assert_same_table(t, r, exact=False)
    assert t.store() == 0   # nothing queued: a plain acknowledgement
    t.close()


@pytest.mark.parametrize("n", [300, 60000])     # a block split on the host; one split on the device (2.5 MB)
def test_push_pairs_wire_layout(ps, orc, n):
    rng = np.random.default_rng(8)
    t, r = pair(ps, orc, 6, "sgd", capacity=4 * n)
    dt = np.dtype([("key", "<u8"), ("value", "<f4", (6,))])
    pairs = np.zeros(n, dtype=dt)
    pairs["key"] = rng.permutation(3 * n)[:n] + 1
    pairs["value"] = rng.normal(0, 1, (n, 6))
    assert t.push_pairs(pairs) == 0 and r.push(pairs["key"], pairs["value"]) == 0
    assert_same_table(t, r, exact=True)
    # the sync path takes the same blocks; padded pairs (a stride beyond the value) are allowed
    wide = np.zeros(n, dtype=np.dtype([("key", "<u8"), ("value", "<f4", (6,)), ("pad", "<u4", (3,))]))
    wide["key"], wide["value"] = pairs["key"], pairs["value"]
    assert t.queue_pairs(pairs) == 0 and t.queue_pairs(wide) == 0 and t.queued() == 2 * n
    assert r.queue(pairs["key"], pairs["value"]) == 0 and r.queue(pairs["key"], pairs["value"]) == 0
    assert t.store() == 0 and r.store() == 0
    assert_same_table(t, r, exact=False)
    bad = pairs[:10].copy()
    bad["key"][4] = 0xFFFFFFFFFFFFFFFF
    assert t.push_pairs(bad) == ps.ERROR and t.queue_pairs(bad) == ps.ERROR and t.queued() == 0
    t.close()


@pytest.mark.parametrize("opt,dim", [("sgd", 16), ("ftrl", 8), ("adagrad", 128)])
def test_dump_load_iterate_roundtrip(ps, orc, wl, opt, dim):
    rng = np.random.default_rng(12)
    n = 90000 if dim == 128 else 20000       # 90000 x 1032 B = 3 staging chunks
    t, r = pair(ps, orc, dim, opt, capacity=n + 10)
    keys = wl.table_keys_np(0, n, seed=5)
    vals = rng.normal(0, 0.01, (n, t.value_floats)).astype(np.float32)
    assert t.set(keys, vals) == 0
    rec = sorted_dump(t)
    order = np.argsort(keys)
    np.testing.assert_array_equal(rec["key"], keys[order])
    np.testing.assert_array_equal(rec["value"], vals[order])
    # iterate in slices reproduces the dump, a short slice marks the end
    st, whole = t.dump()
    got, off = [], 0
    while True:
        st, part = t.iterate(off, 7001)
        assert st == 0
        got.append(part.copy())
        off += part.size
        if part.size < 7001:
            break
    np.testing.assert_array_equal(np.concatenate(got), whole)
    # load into a new table; restore semantics refuse keys that are already there
    t2 = ps.Table(dim, capacity=n + 10, **OPTS[opt])
    assert t2.load(whole, ps.LOAD_UNIQUE) == 0
    np.testing.assert_array_equal(sorted_dump(t2), rec)
    assert t2.load(whole[:10], ps.LOAD_UNIQUE) == ps.ERROR
    assert t2.load(whole[:10]) == 0 and t2.size() == n
    assert t2.clear() == 0 and t2.size() == 0
    st, rows, hit = t2.pull(keys[:100])
    assert not hit.any()
    assert t2.load(whole[:100], ps.LOAD_UNIQUE) == 0 and t2.size() == 100
    t.close(), t2.close()


def test_bulk_transfers_through_page_locked_buffers(ps, orc, wl):
    """Dump into and Load from page-locked memory take the path without staging copies; the
    records are the same as through pageable buffers (6 staging chunks here)."""
    rng = np.random.default_rng(21)
    dim, n = 128, 200000                       # 200000 x 520 B = 104 MB
    t = ps.Table(dim, ps.OPT_SGD, lr=0.5, capacity=n)
    keys = wl.table_keys_np(0, n, seed=8)
    vals = rng.normal(0, 1, (n, dim)).astype(np.float32)
    assert t.set(keys, vals) == 0
    st, plain = t.dump()
    st2, locked = t.dump(pinned=True)
    assert st == 0 and st2 == 0
    np.testing.assert_array_equal(plain, locked)
    order = np.argsort(keys)
    srt = np.sort(locked, order="key")
    np.testing.assert_array_equal(srt["key"], keys[order])
    np.testing.assert_array_equal(srt["value"], vals[order])
    t2 = ps.Table(dim, ps.OPT_SGD, lr=0.5, capacity=n)
    assert t2.load(locked, ps.LOAD_UNIQUE) == 0 and t2.size() == n
    np.testing.assert_array_equal(np.sort(t2.dump()[1], order="key"), srt)
    # a slice that starts inside the page-locked buffer is page-locked too
    assert t2.clear() == 0 and t2.load(locked[1000:151000], ps.LOAD_UNIQUE) == 0 and t2.size() == 150000
    t.close(), t2.close()


def test_load_leaves_out_records_with_reserved_keys(ps, orc):
    dim = 4
    t = ps.Table(dim, capacity=100)
    r = orc.Oracle(dim, capacity=100)
    rec = np.zeros(10, dtype=ps.record_dtype(dim))
    rec["key"] = np.arange(10, dtype=np.uint64) + 5
    rec["key"][3] = 0xFFFFFFFFFFFFFFFF
    rec["key"][7] = 0xFFFFFFFFFFFFFFFE
    rec["value"] = np.arange(40, dtype=np.float32).reshape(10, dim)
    assert t.load(rec) == ps.ERROR and r.load(rec) == orc.ERROR
    assert "reserved" in t.last_error()
    assert t.size() == 8 and r.size() == 8
    np.testing.assert_array_equal(np.sort(t.dump()[1], order="key"), np.sort(r.dump()[1], order="key"))
    t.close()


def test_reserved_keys_and_stats(ps, orc, wl):
    t = ps.Table(4, capacity=20000, max_load_factor=0.8)
    bad = np.array([1, 0xFFFFFFFFFFFFFFFF], np.uint64)
    assert t.push(bad, np.ones((2, 4), np.float32)) == ps.ERROR
    assert t.pull(bad)[0] == ps.ERROR and t.size() == 0
    keys = wl.table_keys_np(0, 20000, seed=7)
    assert t.set(keys, np.zeros((20000, 4), np.float32)) == 0
    s = t.stats()
    assert s.size == 20000 and s.capacity == 20000 and s.slots == 32768
    assert sum(s.probe_hist) == 20000 and s.probe_hist[0] > 15000
    assert abs(s.load_factor - 20000 / 32768) < 1e-9
    assert t.memory_usage() == s.memory_usage == 32768 * 16 + 20000 * (16 + 8)
    t.close()


def test_device_pointer_entry_points(ps, orc, wl):
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(21)
    dim, n_table, batch = 16, 50000, 40000
    t, r = pair(ps, orc, dim, "sgd", capacity=n_table + batch)
    keys = wl.table_keys_np(0, n_table, seed=4)
    vals = rng.normal(0, 0.01, (n_table, dim)).astype(np.float32)
    dk = torch.from_numpy(keys.view(np.int64)).cuda()
    dv = torch.from_numpy(vals).cuda()
    stream = torch.cuda.current_stream().cuda_stream
    assert t.set_dev(dk.data_ptr(), dv.data_ptr(), n_table, stream) == 0
    assert r.set(keys, vals) == 0
    q = wl.zipf_batch_np(rng, n_table, 1.05, batch, seed=4)
    g = rng.normal(0, 1e-3, (batch, dim)).astype(np.float32)
    dq = torch.from_numpy(q.view(np.int64)).cuda()
    dg = torch.from_numpy(g).cuda()
    out = torch.empty(batch, dim, device="cuda")
    hit = torch.empty(batch, dtype=torch.uint8, device="cuda")
    for step in range(2):
        assert t.pull_dev(dq.data_ptr(), batch, out.data_ptr(), hit.data_ptr(), 0, stream) == 0
        assert t.push_dev(dq.data_ptr(), dg.data_ptr(), batch, 0, stream) == 0
        torch.cuda.synchronize()
        st, rows, h = r.pull(q)
        np.testing.assert_allclose(out.cpu().numpy(), rows, rtol=RTOL, atol=ATOL)
        assert hit.all()
        assert r.push(q, g) == 0
    # queue_dev / store_dev on another stream: the table orders itself across streams
    s2 = torch.cuda.Stream()
    assert t.queue_dev(dq.data_ptr(), dg.data_ptr(), batch, s2.cuda_stream) == 0
    assert t.store_dev(0, s2.cuda_stream) == 0
    assert t.pull_dev(dq.data_ptr(), batch, out.data_ptr(), None, 0, stream) == 0
    torch.cuda.synchronize()
    assert r.queue(q, g) == 0 and r.store() == 0
    np.testing.assert_allclose(out.cpu().numpy(), r.pull(q)[1], rtol=RTOL, atol=ATOL)
    assert_same_table(t, r, exact=False)
    t.close()


def _random_predicates(mod, rng, vf):
    """a few predicates on the key and on value columns, built for module `mod`"""
    col = int(rng.integers(0, vf))
    return [
        None,
        mod.predicate((mod.COL_KEY, mod.CMP_MOD_EQ, (3, 1))),
        mod.predicate((col, mod.CMP_LT, -0.002)),
        mod.predicate((mod.COL_KEY, mod.CMP_GE, 1 << 62), (col, mod.CMP_GT, 0.0)),
        mod.predicate((0, mod.CMP_LE, 0.004), (vf - 1, mod.CMP_NE, 0.0), (mod.COL_KEY, mod.CMP_MOD_EQ, (2, 0))),
        mod.predicate((mod.COL_KEY, mod.CMP_EQ, 12345)),          # nothing matches
    ]


@pytest.mark.parametrize("opt,dim", [("sum", 2), ("sgd", 16), ("adagrad", 8), ("ftrl", 100), ("sgd", 300)])
def test_for_each_counts_and_sums(ps, orc, wl, opt, dim):
    """Read-only for-each (pico-ps/operator/ForEachOperator.h:180-190) with the count / sum
    reduction: counts are exact; the column sums are float64 sums of fp32 values added in another
    order than the oracle's, so they agree to 1e-12 relative."""
    rng = np.random.default_rng(dim)
    t, r = pair(ps, orc, dim, opt, capacity=40000)
    n = 30011
    keys = wl.table_keys_np(0, n, seed=4)
    vals = rng.normal(0, 0.01, (n, t.value_floats)).astype(np.float32)
    assert t.set(keys, vals) == 0 and r.set(keys, vals) == 0
    for pg, po in zip(_random_predicates(ps, np.random.default_rng(1), t.value_floats),
                      _random_predicates(orc, np.random.default_rng(1), t.value_floats)):
        st, cnt, sums = t.for_each(pg)
        st2, cnt2, sums2 = r.for_each(po)
        assert st == st2 == 0 and cnt == cnt2
        np.testing.assert_allclose(sums, sums2, rtol=1e-12, atol=1e-15)
        again = t.for_each(pg)
        assert again[1] == cnt and np.array_equal(again[2], sums)     # fixed order of additions
    # an empty table, and a predicate that the library must refuse
    t.clear()
    assert t.for_each()[1:2] == (0,)
    assert t.for_each(ps.predicate((t.value_floats, ps.CMP_LT, 0.0)))[0] == 1     # no such column
    assert t.for_each(ps.predicate((0, ps.CMP_MOD_EQ, 1.0)))[0] == 1              # MOD_EQ needs the key
    t.close()


@pytest.mark.parametrize("opt,dim", [("sum", 2), ("sgd", 16), ("adagrad", 64), ("ftrl", 5)])
def test_erase_if_and_erase_keep_the_table_consistent(ps, orc, wl, opt, dim):
    """erase_if (pico-ps/operator/EraseIfOperator.h:38-47) by predicate and erase of chosen keys:
    after every step the stored set equals the oracle's, the rows are dense (dump, iterate, size
    agree), erased keys miss, survivors keep their values bit for bit, pushes and inserts after
    the erase behave as on a table that never held the erased keys."""
    rng = np.random.default_rng(dim + 100)
    t, r = pair(ps, orc, dim, opt, capacity=60000)
    n = 40000
    keys = wl.table_keys_np(0, n, seed=6)
    vals = rng.normal(0, 0.01, (n, t.value_floats)).astype(np.float32)
    if opt == "adagrad":
        vals[:, dim:] = 0.1
    if opt == "ftrl":
        vals[:, 2 * dim:] = vals[:, dim:2 * dim] ** 2
    assert t.set(keys, vals) == 0 and r.set(keys, vals) == 0

    def check():
        assert t.size() == r.size()
        assert_same_table(t, r, exact=True)
        st, rec = t.iterate(0, t.size() + 10)
        assert st == 0 and rec.size == t.size() and np.unique(rec["key"]).size == rec.size
        q = np.concatenate([keys[:3000], keys[-3000:]])
        a, b = t.pull(q), r.pull(q)
        np.testing.assert_array_equal(a[2], b[2])
        np.testing.assert_array_equal(a[1], b[1])

    # by predicate: a third of the keys, then a value column
    for pg, po in ((ps.predicate((ps.COL_KEY, ps.CMP_MOD_EQ, (3, 0))), orc.predicate((orc.COL_KEY, orc.CMP_MOD_EQ, (3, 0)))),
                   (ps.predicate((0, ps.CMP_GT, 0.005)), orc.predicate((0, orc.CMP_GT, 0.005)))):
        a, b = t.erase_if(pg), r.erase_if(po)
        assert a == b and a[0] == 0 and a[1] > 0
        check()
    # chosen keys, with repeats and keys that are not stored
    victims = np.concatenate([keys[rng.integers(0, n, 5000)], wl.fresh_keys_np(rng, 300), keys[:10], keys[:10]])
    a, b = t.erase(victims), r.erase(victims)
    assert a == b and a[0] == 0
    check()
    # the table keeps working: push with duplicates re-inserts some erased keys, then more erases
    q = np.concatenate([keys[rng.integers(0, n, 20000)], wl.fresh_keys_np(rng, 500)])
    g = rng.integers(-3, 4, (q.size, dim)).astype(np.float32) if opt == "sum" else rng.normal(0, 1e-3, (q.size, dim)).astype(np.float32)
    uq, first = np.unique(q, return_index=True)              # distinct keys: bit-exact for every optimizer
    assert t.push(uq, g[first]) == 0 and r.push(uq, g[first]) == 0
    check()
    assert t.compact() == 0
    check()
    a, b = t.erase_if(ps.predicate((ps.COL_KEY, ps.CMP_MOD_EQ, (2, 1)))), r.erase_if(orc.predicate((orc.COL_KEY, orc.CMP_MOD_EQ, (2, 1))))
    assert a == b
    check()
    # erase everything, in two ways
    a, b = t.erase_if(None), r.erase_if(None)
    assert a == b and t.size() == 0
    assert t.set(keys[:100], vals[:100]) == 0 and t.erase(keys[:100]) == (0, 100) and t.size() == 0
    st, cnt, sums = t.for_each()
    assert cnt == 0 and not sums.any()
    t.close()


def test_erase_many_rounds_triggers_rebuild(ps, orc, wl):
    """Markers of erased keys pile up in the slots until the hash array is rebuilt by itself (an
    eighth of the slots); lookups, inserts and erases must not notice."""
    rng = np.random.default_rng(9)
    t, r = pair(ps, orc, 4, "sum", capacity=4000)
    for it in range(12):
        keys = wl.table_keys_np(it * 2500, 2500, seed=8)
        vals = rng.integers(-5, 6, (2500, 4)).astype(np.float32)
        assert t.set(keys, vals) == 0 and r.set(keys, vals) == 0
        assert t.erase(keys[:2400]) == r.erase(keys[:2400]) == (0, 2400)
        assert t.erase_if(ps.predicate((ps.COL_KEY, ps.CMP_EQ, int(keys[2400])))) == (0, 1)
        assert r.erase_if(orc.predicate((orc.COL_KEY, orc.CMP_EQ, int(keys[2400])))) == (0, 1)
        assert_same_table(t, r, exact=True)
    assert t.size() == r.size() == 12 * 99
    t.close()


def test_fill_erase_refill_on_a_tight_hash_array(ps, orc, wl):
    """A capacity that puts the hash array at 90 % load (940,000 keys in 2^20 slots): filled to the
    brim, an eighth of the slots' worth of keys erased, as many new keys inserted. Markers of
    erased keys are not reused by inserts, so without an earlier rebuild live keys + markers would
    fill every slot and a probe could neither end nor insert."""
    rng = np.random.default_rng(21)
    cap = 940_000
    t = ps.Table(2, capacity=cap, max_load_factor=0.9, **OPTS["sum"])
    r = orc.Oracle(2, capacity=cap, **OPTS["sum"])
    assert t.stats().slots == 1 << 20
    keys = wl.table_keys_np(0, cap, seed=12)
    vals = rng.integers(-5, 6, (cap, 2)).astype(np.float32)
    for lo in range(0, cap, 235_000):
        assert t.set(keys[lo:lo + 235_000], vals[lo:lo + 235_000]) == 0
        assert r.set(keys[lo:lo + 235_000], vals[lo:lo + 235_000]) == 0
    assert t.size() == cap
    n = (1 << 20) // 8
    gone = keys[rng.permutation(cap)[:n]]
    assert t.erase(gone) == r.erase(gone) == (0, n)
    fresh = wl.fresh_keys_np(rng, n)
    g = rng.integers(-3, 4, (n, 2)).astype(np.float32)
    assert t.push(fresh, g) == 0, t.last_error()       # insert-on-miss through the partitioned push
    assert r.push(fresh, g) == 0
    assert t.size() == r.size() == cap
    q = np.concatenate([fresh[:5000], gone[:5000], keys[:5000]])
    st, rows, hit = t.pull(q)
    st2, rows2, hit2 = r.pull(q)
    assert st == st2 == 0
    np.testing.assert_array_equal(hit, hit2)
    np.testing.assert_array_equal(rows, rows2)
    assert t.push(wl.fresh_keys_np(rng, 20000), np.ones((20000, 2), np.float32)) == ps.OUT_OF_MEMORY
    assert_same_table(t, r, exact=True)
    t.close()


@pytest.mark.parametrize("opt,dim", [("ftrl", 16384), ("adagrad", 4097), ("sum", 16384)])
def test_largest_rows(ps, orc, wl, opt, dim):
    """The largest dim the library takes (16384: rows of up to 192 KB with FTRL state) and an odd one
    just past a power of two: every entry point on a small table, against the oracle."""
    rng = np.random.default_rng(dim)
    n = 120
    t, r = pair(ps, orc, dim, opt, capacity=400)
    keys = wl.table_keys_np(0, n, seed=2)
    vf = t.value_floats
    vals = rng.integers(-3, 4, (n, vf)).astype(np.float32)
    if opt != "sum":
        vals[:, dim:] = np.abs(vals[:, dim:]) + 1.0
    assert t.set(keys, vals) == 0 and r.set(keys, vals) == 0
    q = np.concatenate([keys[rng.integers(0, n, 150)], wl.fresh_keys_np(rng, 20)])
    g = rng.integers(-2, 3, (q.size, dim)).astype(np.float32)
    if opt != "sum":
        q = np.unique(q)                      # inexact optimizers: distinct keys compare bit for bit
        g = g[: q.size]
    a, b = t.pull(q), r.pull(q)
    np.testing.assert_array_equal(a[1].view(np.uint32), b[1].view(np.uint32))
    np.testing.assert_array_equal(a[2], b[2])
    assert t.push(q, g) == 0 and r.push(q, g) == 0
    assert_same_table(t, r, exact=True)
    a, b = t.for_each(), r.for_each()
    assert a[:2] == b[:2]
    np.testing.assert_allclose(a[2], b[2], rtol=1e-12, atol=1e-9)
    where = [(-1, 6, (3, 1))]
    assert t.erase_if(ps.predicate(*where)) == r.erase_if(orc.predicate(*where))
    assert_same_table(t, r, exact=True)
    st, rec = t.dump()
    t2 = ps.Table(dim, capacity=400, **OPTS[opt])
    assert t2.load(rec, ps.LOAD_UNIQUE) == 0
    np.testing.assert_array_equal(np.sort(t2.dump()[1], order="key"), np.sort(rec, order="key"))
    t.close(), t2.close()


@pytest.mark.parametrize("opt,dim", [("sgd", 16), ("ftrl", 6), ("adagrad", 64)])
def test_reserve_grows_a_full_table(ps, orc, wl, opt, dim):
    """A table that refuses a batch for lack of room takes it after pshbm_reserve; keys, values,
    marks and the order of the slab survive the move, erased slots' markers do not."""
    rng = np.random.default_rng(77)
    cap = 3000
    t, r = pair(ps, orc, dim, opt, capacity=cap, track_increment=True)
    keys = wl.table_keys_np(0, 20000, seed=4)
    g = rng.integers(-3, 4, (20000, dim)).astype(np.float32)
    assert t.push(keys[:2500], g[:2500]) == 0 and r.push(keys[:2500], g[:2500]) == 0
    assert t.erase(keys[:400]) == r.erase(keys[:400])
    before = t.dump()[1]
    assert t.push(keys[2500:6000], g[2500:6000]) == ps.OUT_OF_MEMORY == r.push(keys[2500:6000], g[2500:6000])
    np.testing.assert_array_equal(t.dump()[1], before)            # all or nothing
    assert t.reserve(100) == 0 and t.stats().capacity == cap      # never shrinks
    assert t.reserve(12000) == 0 and r.reserve(12000) == 0
    s = t.stats()
    assert s.capacity == 12000 and s.size == 2100 and sum(s.probe_hist) == 2100
    np.testing.assert_array_equal(t.dump()[1], before)            # same slab, same order
    assert t.push(keys[2500:6000], g[2500:6000]) == 0 and r.push(keys[2500:6000], g[2500:6000]) == 0
    assert t.push(keys[:9000], g[:9000]) == 0 and r.push(keys[:9000], g[:9000]) == 0
    assert_same_table(t, r, exact=True)
    a, b = t.take_increment(), r.take_increment()
    np.testing.assert_array_equal(np.sort(a[1], order="key"), np.sort(b[1], order="key"))
    a, b = t.pull(keys[:12000]), r.pull(keys[:12000])
    np.testing.assert_array_equal(a[1].view(np.uint32), b[1].view(np.uint32))
    np.testing.assert_array_equal(a[2], b[2])
    assert t.reserve(1 << 33) == ps.INVALID_CONFIG
    t.close()


@pytest.mark.parametrize("dim", [1, 4, 16, 100, 260])
@pytest.mark.parametrize("n", [1, 33, 257, 500, 512, 513, 1000, 4096, 4097, 8193])
def test_one_launch_push_heavy_repeats(ps, orc, dim, n):
    """Batches of up to 512 keys take the one-launch push, larger ones the partitioned push (one
    tile up to 4096 keys, then two, then three): a few keys repeated hundreds of times (runs added by
    the whole workgroup), keys that are new and repeated inside the batch, keys not stored under
    PUSH_NO_INSERT; integer gradients, so the sums are exact in any order."""
    rng = np.random.default_rng(dim * 1000 + n)
    t, r = pair(ps, orc, dim, "sum", capacity=5000 + 4 * n)
    base = np.arange(1, 41, dtype=np.uint64) * 7919
    assert t.set(base[:20], np.ones((20, dim), np.float32)) == 0
    assert r.set(base[:20], np.ones((20, dim), np.float32)) == 0
    for it in range(4):
        hot = base[rng.integers(0, 3, n)]                         # three keys take most of the batch
        cold = base[rng.integers(0, 40, n)]                       # stored and new ones
        fresh = rng.integers(1 << 40, 1 << 41, n).astype(np.uint64)
        pick = rng.random(n)
        q = np.where(pick < 0.6, hot, np.where(pick < 0.9, cold, fresh)).astype(np.uint64)
        q[rng.integers(0, n)] = q[0]                              # at least one repeat of a maybe-new key
        g = rng.integers(-4, 5, (n, dim)).astype(np.float32)
        flags = ps.PUSH_NO_INSERT if it == 2 else 0
        assert t.push(q, g, flags) == 0 and r.push(q, g, flags) == 0
        assert_same_table(t, r, exact=True)
    t.close()


@pytest.mark.parametrize("opt", ["sgd", "adagrad", "ftrl"])
def test_hyperparameters_change_between_pushes(ps, orc, wl, opt):
    """A learning-rate schedule (or a newly registered push operator, pico-ps/operator/Operator.h:53-57):
    the pushes after pshbm_set_hyperparameters take the new values, keys inserted afterwards the new
    initial accumulator; distinct keys per batch, so every value compares bit for bit."""
    rng = np.random.default_rng(3)
    dim = 12
    t, r = pair(ps, orc, dim, opt, capacity=6000)
    keys = wl.table_keys_np(0, 5000, seed=6)
    schedules = [dict(lr=0.5, init_acc=0.25, alpha=0.1, beta=0.5, l1=1e-3, l2=1e-2),
                 dict(lr=0.03125, init_acc=1.0, alpha=0.7, beta=2.0, l1=0.0, l2=0.0)]
    for it in range(4):
        q = keys[rng.permutation(5000)[: 400 + 700 * it]]          # one-launch and chained pushes
        g = rng.normal(0, 0.1, (q.size, dim)).astype(np.float32)
        assert t.push(q, g) == 0 and r.push(q, g) == 0
        if it < 2:
            hp = schedules[it]
            assert t.set_hyperparameters(**hp) == 0 and r.set_hyperparameters(**hp) == 0
    assert_same_table(t, r, exact=True)
    if opt == "ftrl":
        assert t.set_hyperparameters(alpha=0.0) == ps.INVALID_CONFIG
    t.close()


@pytest.mark.parametrize("opt", ["sum", "sgd", "adagrad", "ftrl"])
@pytest.mark.parametrize("dim", [5, 8, 128])
@pytest.mark.parametrize("n", [300, 20000])      # the one-launch push; the chain of kernels
def test_initial_weights_of_new_keys(ps, orc, wl, opt, dim, n):
    """init_range > 0: a miss answers the weights an insertion would store, a push and an inserting
    pull store them, bit for bit the oracle's (a pure function of key and column)."""
    rng = np.random.default_rng(17)
    rg = 0.05
    t, r = pair(ps, orc, dim, opt, capacity=4 * n + 64, init_range=rg)
    keys = wl.fresh_keys_np(rng, 3 * n)
    a, b = t.pull(keys[:n]), r.pull(keys[:n])                  # nothing stored: every key misses
    assert a[0] == b[0] == 0 and not a[2].any() and t.size() == 0
    np.testing.assert_array_equal(a[1], b[1])
    assert np.abs(a[1]).max() <= rg and a[1].std() > rg / 4
    spot = rng.integers(0, n, 5)
    for i in spot:
        assert a[1][i, dim - 1] == np.float32(ps.init_weight(rg, int(keys[i]), dim - 1))
    g = rng.normal(0, 1e-2, (n, dim)).astype(np.float32)
    assert t.push(keys[:n], g) == 0 and r.push(keys[:n], g) == 0     # distinct keys: bit-exact
    assert_same_table(t, r, exact=True)
    q = np.concatenate([keys[: n // 2], keys[n: n + n // 4], keys[n: n + n // 4]])  # stored, new twice
    rng.shuffle(q)
    g = rng.normal(0, 1e-2, (q.size, dim)).astype(np.float32)
    assert t.push(q, g) == 0 and r.push(q, g) == 0
    assert_same_table(t, r, exact=False)
    assert t.set(*(lambda d: (d["key"], d["value"]))(sorted_dump(r))) == 0
    q = np.concatenate([keys[2 * n:], keys[:n // 3], keys[2 * n: 2 * n + 7]])
    rng.shuffle(q)
    a, b = t.pull(q, ps.PULL_INSERT_ON_MISS), r.pull(q, orc.PULL_INSERT_ON_MISS)
    assert a[0] == b[0] == 0
    np.testing.assert_array_equal(a[1], b[1])
    np.testing.assert_array_equal(a[2], b[2])
    assert_same_table(t, r, exact=True)
    assert t.size() == r.size() == n + n // 4 + n
    # the hyperparameters may change, the range stays
    if opt != "sum":
        o = dict(OPTS[opt]); o.pop("optimizer")
        assert t.set_hyperparameters(**o) == 0
        extra = wl.fresh_keys_np(rng, 40)
        a, b = t.pull(extra), r.pull(extra)
        np.testing.assert_array_equal(a[1], b[1])
    t.close()


def test_initial_weights_config_is_validated(ps):
    for bad in (-0.5, float("inf"), float("nan")):
        with pytest.raises(ps.PshbmError):
            ps.Table(4, capacity=16, init_range=bad)


def test_device_memory_limit(ps, orc, wl):
    """A budget of device memory for the library (the hard limit of the reference's
    ShardStorageMemory, pico-ps/storage/Storage.cpp:93-98, for the device): what would pass it fails
    with OUT_OF_MEMORY and changes nothing; what is released is given back."""
    import gc
    gc.collect()                                   # tables of earlier tests that nobody holds any more
    base, limit = ps.device_memory(0)
    assert limit == 0
    dim = 16
    t, r = pair(ps, orc, dim, "sgd", capacity=100_000)
    used, _ = ps.device_memory(0)
    assert used - base >= t.memory_usage() > 100_000 * (dim * 4 + 8)
    keys = wl.table_keys_np(0, 60_000, seed=8)
    g = np.random.default_rng(2).normal(0, 1, (60_000, dim)).astype(np.float32)
    assert t.push(keys[:50_000], g[:50_000]) == 0 and r.push(keys[:50_000], g[:50_000]) == 0
    assert_same_table(t, r, exact=True)            # (the first dump allocates the staging buffers)
    used, _ = ps.device_memory(0)
    ps.set_memory_limit(0, used + (1 << 20))
    try:
        assert ps.device_memory(0) == (used, used + (1 << 20))
        with pytest.raises(ps.PshbmError) as e:
            ps.Table(dim, capacity=1_000_000)
        assert e.value.status == ps.OUT_OF_MEMORY and "limit" in str(e.value)
        assert ps.device_memory(0)[0] == used                     # nothing of the failed table is left
        assert t.reserve(1_000_000) == ps.OUT_OF_MEMORY and "limit" in t.last_error()
        assert ps.device_memory(0)[0] == used and t.stats().capacity == 100_000
        small = ps.Table(2, capacity=100, max_batch=64)           # what fits is still granted
        small.close()
        # the table works on as it was
        assert t.push(keys[40_000:], g[40_000:]) == 0 and r.push(keys[40_000:], g[40_000:]) == 0
        assert_same_table(t, r, exact=True)
    finally:
        ps.set_memory_limit(0, 0)
    assert t.reserve(300_000) == 0 and r.reserve(300_000) == 0
    assert_same_table(t, r, exact=True)
    t.close()
    assert ps.device_memory(0)[0] <= base
    with pytest.raises(ps.PshbmError):
        ps.set_memory_limit(64, 1)


@pytest.mark.parametrize("n", [300, 5000, 40000])   # the one-launch push; the chain; beyond 1 MB: staged
def test_page_locked_request_buffers_are_used_in_place(ps, orc, wl, n):
    """Small pulls and pushes whose buffers lie in page-locked memory (pshbm_host_alloc) hand them to
    the kernels as they are; the results are those of pageable buffers."""
    rng = np.random.default_rng(31)
    dim = 16
    t, r = pair(ps, orc, dim, "adagrad", capacity=4 * n + 1000)
    keys = wl.fresh_keys_np(rng, 2 * n)
    q = np.concatenate([keys[:n // 2], keys[:n // 2]])
    rng.shuffle(q)
    pk = ps.pinned_empty(q.size, np.uint64)
    pg = ps.pinned_empty((q.size, dim), np.float32)
    out = ps.pinned_empty((q.size, dim), np.float32)
    hit = ps.pinned_empty(q.size, np.uint8)
    for step in range(3):
        pk[:] = q
        pg[:] = rng.integers(-3, 4, (q.size, dim)).astype(np.float32)
        assert t.push(pk, pg) == 0 and r.push(q, np.array(pg)) == 0
        out[:] = -7.0
        st, rows, h = t.pull(pk, 0, out=out, hit=hit)
        b = r.pull(q)
        assert st == 0 and rows is out
        np.testing.assert_allclose(out, b[1], rtol=RTOL, atol=ATOL)
        np.testing.assert_array_equal(hit, b[2])
        # mixed: page-locked keys, pageable rows -> the staged path
        st, rows2, h2 = t.pull(pk)
        np.testing.assert_array_equal(rows2, out)
        q = np.concatenate([keys[step * 10: step * 10 + n // 2], keys[n: n + n // 2]])
    assert_same_table(t, r, exact=False)
    m = min(n, 3000)                                   # set from page-locked buffers, in place when small
    pv = ps.pinned_empty((m, t.value_floats), np.float32)
    pv[:] = rng.integers(1, 9, (m, t.value_floats)).astype(np.float32)
    pk[:m] = keys[:m]
    assert t.set(pk[:m], pv) == 0 and r.set(keys[:m], np.array(pv)) == 0
    assert_same_table(t, r, exact=False)
    t.close()


def test_iterate_keys_follows_the_record_order(ps, orc, wl):
    """The keys-only walk names the records of pshbm_iterate, slice by slice, also after erasures
    have moved rows; past the end it returns nothing."""
    rng = np.random.default_rng(41)
    t, r = pair(ps, orc, 8, "sgd", capacity=20000)
    keys = wl.fresh_keys_np(rng, 12000)
    g = rng.normal(0, 1, (12000, 8)).astype(np.float32)
    assert t.push(keys, g) == 0 and r.push(keys, g) == 0
    assert t.erase(keys[::3]) == r.erase(keys[::3])
    n = t.size()
    seen = []
    for off in range(0, n + 3000, 2500):
        st, k = t.iterate_keys(off, 2500)
        st2, rec = t.iterate(off, 2500)
        assert st == 0 and st2 == 0
        np.testing.assert_array_equal(k, rec["key"])
        assert k.size == max(0, min(2500, n - off))
        seen.append(k)
    seen = np.concatenate(seen)
    assert seen.size == n and np.array_equal(np.sort(seen), np.sort(r.dump()[1]["key"]))
    assert t.iterate_keys(0, 0)[1].size == 0
    t.close()


def test_sort_that_gives_up_applies_nothing(ps, orc, wl, push_path):
    """A tile of the aggregation sort that gives up its bounded wait raises a flag; the kernels
    after the sort then leave the rows alone and the table reports FATAL until it is cleared. The
    host makes the wait give up (a limit of zero polls): every kernel still runs to its end."""
    if push_path != "sorted":
        pytest.skip("the sorted push only")
    rng = np.random.default_rng(21)
    n_table, dim, n = 30000, 8, 14000          # 4 tiles of 4096 pairs: one-launch passes that wait
    t = ps.Table(dim, capacity=n_table + n, optimizer=1, lr=0.5)
    keys = wl.table_keys_np(0, n_table, seed=7)
    vals = rng.normal(0, 0.01, (n_table, dim)).astype(np.float32)
    assert t.set(keys, vals) == 0
    q = keys[rng.integers(0, n_table, n)]
    g = rng.normal(0, 1.0, (n, dim)).astype(np.float32)
    try:
        ps.debug_sort_spin_limit(0)
        assert t.push(q, g) == 0                # enqueued; the failure shows at the next counter read
    finally:
        ps.debug_sort_spin_limit()
    with pytest.raises(ps.PshbmError) as e:
        t.size()
    assert e.value.status == ps.FATAL and "not applied" in str(e.value)
    assert t.push(q, g) == 0                    # later pushes are refused on the device as well
    st, rows, hit = t.pull(keys)
    assert st == 0 and hit.all()
    np.testing.assert_array_equal(rows, vals)   # no row was touched
    assert t.clear() == 0 and t.size() == 0
    assert t.set(keys, vals) == 0 and t.push(q, g) == 0 and t.size() == n_table
    st, rows, hit = t.pull(keys)
    assert not np.array_equal(rows, vals)
    t.close()


def test_c2_shaped_push_against_reference_order_and_exact_sums(ps, orc, wl, capsys, push_path):
    """The headline workload at a table size the oracle reaches: 1M-key Zipf(1.05) batches (the
    hottest key repeats about 100,000 times) over 10M keys, dim 16, SGD, gradients N(0, 1e-3).
    Every value must be within 1e-6 / 1e-7 of the exactly rounded result; the report says how many
    are further than that from the reference-order result, which drifts from the exact one itself."""
    rng = np.random.default_rng(17)
    n_table, n, dim = 10_000_000, 1_000_000, 16
    # (room for a whole batch of new keys: a table that might not hold the batch would take the
    # sorted push, which can be undone, whatever the path this run asks for)
    t = ps.Table(dim, capacity=n_table + n + 16, max_batch=n, **OPTS["sgd"])
    r = orc.Oracle(dim, capacity=n_table + 16, **OPTS["sgd"])
    x = orc.Oracle(dim, capacity=n_table + 16, **OPTS["sgd"])
    chunk = 1_000_000
    for start in range(0, n_table, chunk):
        keys = wl.table_keys_np(start, chunk, seed=11)
        vals = rng.normal(0, 0.01, (chunk, dim)).astype(np.float32)
        for b in (t, r, x):
            assert b.set(keys, vals) == 0
    report = {}
    for step in range(2):
        q = wl.zipf_batch_np(rng, n_table, 1.05, n, seed=11)
        g = rng.normal(0, 1e-3, (n, dim)).astype(np.float32)
        assert t.push(q, g) == 0 and r.push(q, g) == 0
        assert x.push(q, g, orc.PUSH_EXACT_AGGREGATION) == 0
        uk, cnt = np.unique(q, return_counts=True)
        # compare the rows the batch touched (the others are bit-identical by construction)
        a, b, c = (bb.pull(uk)[1] for bb in (t, r, x))
        dt = np.dtype([("key", "<u8"), ("value", "<f4", (dim,))])
        pack = lambda rows: np.rec.fromarrays([uk, rows], dtype=dt)
        assert_push_parity(pack(a), pack(b), pack(c), cnt, report)
        np.testing.assert_allclose(a, c, rtol=RTOL, atol=ATOL)
        report["top_multiplicity"] = max(report.get("top_multiplicity", 0), int(cnt.max()))
        # both oracles restart from the reference-order state, as the table does
        assert t.set(uk, b) == 0 and x.set(uk, b) == 0
    with capsys.disabled():
        print(f"\nC2-shaped push parity report ({push_path} push):", report)
    t.close()
