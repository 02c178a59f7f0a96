"""Several host threads on one table: the host-pointer entry points are synchronous and
thread-safe (pulls share the table, everything else takes it exclusively, the discipline of
pico-ps/operator/SparsePullOperator.h:188-192 and SparsePushOperator.h:220; the reference's server
calls the operator halves from 4 + 4 threads, pico-ps/service/Server.h:24-26)."""
import threading

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_concurrent_pushes_pulls_and_scans(ps, orc, wl):
    rng = np.random.default_rng(12)
    dim, n = 8, 20000
    t = ps.Table(dim, ps.OPT_SUM, capacity=60000)
    r = orc.Oracle(dim, orc.OPT_SUM, capacity=60000)
    keys = wl.table_keys_np(0, n, seed=5)
    vals = rng.integers(-5, 6, (n, dim)).astype(np.float32)
    assert t.set(keys, vals) == 0 and r.set(keys, vals) == 0
    n_threads, rounds = 6, 12
    work = []
    for w in range(n_threads):
        mine = []
        for it in range(rounds):
            q = np.concatenate([keys[rng.integers(0, n, 3000)], wl.fresh_keys_np(rng, 40)])
            g = rng.integers(-3, 4, (q.size, dim)).astype(np.float32)   # integer sums: order-free
            mine.append((q, g))
        work.append(mine)
    errors = []

    def worker(w):
        try:
            for q, g in work[w]:
                assert t.push(q, g) == 0
                st, rows, hit = t.pull(q[:500])
                assert st == 0 and hit.all()           # the thread's own pushed keys are there
                st, cnt, sums = t.for_each()
                assert st == 0 and cnt >= n
                if w == 0:
                    assert t.size() >= n
        except Exception as e:  # noqa: BLE001 - reported by the main thread
            errors.append(repr(e))

    threads = [threading.Thread(target=worker, args=(w,)) for w in range(n_threads)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors
    for mine in work:                                   # any order gives the same integer sums
        for q, g in mine:
            assert r.push(q, g) == 0
    a = np.sort(t.dump()[1], order="key")
    b = np.sort(r.dump()[1], order="key")
    np.testing.assert_array_equal(a["key"], b["key"])
    np.testing.assert_array_equal(a["value"], b["value"])
    t.close()


def test_pulls_on_several_streams_between_pushes(ps, orc, wl):
    """Pulls enqueued on four streams overlap on the device; each must still see every push that
    was made before it and none that was made after it."""
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(31)
    dim, n, batch = 16, 200000, 50000
    t = ps.Table(dim, ps.OPT_SUM, capacity=n + 1000, max_batch=batch)
    r = orc.Oracle(dim, orc.OPT_SUM, capacity=n + 1000)
    keys = wl.table_keys_np(0, n, seed=9)
    vals = rng.integers(-5, 6, (n, dim)).astype(np.float32)
    assert t.set(keys, vals) == 0 and r.set(keys, vals) == 0
    streams = [torch.cuda.Stream() for _ in range(4)]
    push_stream = torch.cuda.Stream()
    plan = []
    for it in range(6):                                  # inputs first: nothing waits in the loop below
        q = keys[rng.integers(0, n, batch)]
        g = rng.integers(-3, 4, (batch, dim)).astype(np.float32)
        pulls = []
        for s in streams:
            pq = keys[rng.integers(0, n, batch)]
            pulls.append((pq, torch.from_numpy(pq.view(np.int64)).cuda(),
                          torch.empty(batch, dim, device="cuda"),
                          torch.empty(batch, dtype=torch.uint8, device="cuda")))
        plan.append((q, g, torch.from_numpy(q.view(np.int64)).cuda(), torch.from_numpy(g).cuda(), pulls))
    torch.cuda.synchronize()
    for q, g, dq, dg, pulls in plan:
        assert t.push_dev(dq.data_ptr(), dg.data_ptr(), batch, 0, push_stream.cuda_stream) == 0
        for s, (pq, dpq, out, hit) in zip(streams, pulls):
            assert t.pull_dev(dpq.data_ptr(), batch, out.data_ptr(), hit.data_ptr(), 0, s.cuda_stream) == 0
    torch.cuda.synchronize()
    for q, g, dq, dg, pulls in plan:
        assert r.push(q, g) == 0
        for pq, dpq, out, hit in pulls:
            st, rows, rhit = r.pull(pq)
            np.testing.assert_array_equal(out.cpu().numpy(), rows)
            np.testing.assert_array_equal(hit.cpu().numpy(), rhit)
    t.close()


def test_concurrent_erasers_with_overlapping_ranges(ps):
    """pico-ps/test/ps_pmem_test.cpp:159-193 with its threads: ten rounds of inserting keys 0..99 and
    ten threads erasing the overlapping ranges [10 i, 10 i + 20) at once; afterwards no key is found
    and the table is empty. Every key is erased exactly once, whichever thread gets there first."""
    t = ps.Table(1, ps.OPT_SUM, capacity=256)
    keys = np.arange(100, dtype=np.uint64)
    vals = keys.astype(np.float32).reshape(-1, 1)
    for _ in range(10):
        assert t.set(keys, vals) == 0 and t.size() == 100
        erased = [0] * 10
        errors = []

        def eraser(i):
            try:
                st, n = t.erase(np.arange(10 * i, 10 * i + 20, dtype=np.uint64))
                assert st == 0
                erased[i] = n
            except Exception as e:  # noqa: BLE001 - reported by the main thread
                errors.append(repr(e))

        threads = [threading.Thread(target=eraser, args=(i,)) for i in range(10)]
        for th in threads:
            th.start()
        for th in threads:
            th.join()
        assert not errors, errors
        assert sum(erased) == 100
        st, rows, hit = t.pull(keys)
        assert st == 0 and not hit.any() and not rows.any() and t.size() == 0
    t.close()


def test_several_tables_pushed_at_once(ps, orc, wl):
    """A server holds several shards, each a table of its own, and its threads push to them at the
    same time (pico-ps/service/Server.h:24-26): three tables of different shapes, one thread each,
    batches of one sort tile up to more than 2^20 keys, so that sort passes of different tables --
    whose tiles wait for each other's counts -- share the device."""
    shapes = [(16, dict(optimizer=ps.OPT_SGD, lr=0.5)), (8, dict(optimizer=ps.OPT_SUM)),
              (64, dict(optimizer=ps.OPT_SGD, lr=0.25))]
    n = 400_000
    sizes = [300_000, 3000, 70_000, 1_200_000, 20_000, 300_000]
    tables, oracles, work = [], [], []
    for w, (dim, opt) in enumerate(shapes):
        rng = np.random.default_rng(40 + w)
        t = ps.Table(dim, capacity=n + 50_000, **opt)
        r = orc.Oracle(dim, capacity=n + 50_000, **opt)
        keys = wl.table_keys_np(0, n, seed=20 + w)
        vals = rng.integers(-8, 9, (n, dim)).astype(np.float32)
        assert t.set(keys, vals) == 0 and r.set(keys, vals) == 0
        mine = []
        for b in sizes:
            q = wl.zipf_batch_np(rng, n, 1.1, b, seed=20 + w)
            q[:50] = wl.fresh_keys_np(rng, 50)
            g = rng.integers(-2, 3, (b, dim)).astype(np.float32)   # integer sums, steps of 1/2 or 1/4: exact
            mine.append((q, g))
        tables.append(t), oracles.append(r), work.append(mine)
    errors = []

    def worker(w):
        try:
            for q, g in work[w]:
                assert tables[w].push(q, g) == 0
                st, rows, hit = tables[w].pull(q[:2000])
                assert st == 0 and hit.all()
        except Exception as e:  # noqa: BLE001 - reported by the main thread
            errors.append(repr(e))

    threads = [threading.Thread(target=worker, args=(w,)) for w in range(len(shapes))]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors
    for w, (t, r) in enumerate(zip(tables, oracles)):
        for q, g in work[w]:
            assert r.push(q, g) == 0
        a = np.sort(t.dump()[1], order="key")
        b = np.sort(r.dump()[1], order="key")
        np.testing.assert_array_equal(a["key"], b["key"])
        np.testing.assert_array_equal(a["value"], b["value"])
        t.close()


def test_several_tables_on_their_own_streams(ps, orc, wl):
    """The same with device buffers: pushes to three tables are enqueued on three streams without
    waiting in between, so their kernels really run side by side; the sort's bounded waits must not
    time out (a time-out would surface as PSHBM_FATAL in size())."""
    import torch
    dims = [16, 8, 32]
    n, b = 500_000, 1_000_000                       # 245 sort tiles per push: one tile per compute unit
    tables, oracles, streams, bufs = [], [], [], []
    for w, dim in enumerate(dims):
        rng = np.random.default_rng(60 + w)
        t = ps.Table(dim, ps.OPT_SGD, lr=0.5, capacity=n + 1000, max_batch=b)
        r = orc.Oracle(dim, orc.OPT_SGD, lr=0.5, capacity=n + 1000)
        keys = wl.table_keys_np(0, n, seed=30 + w)
        vals = rng.integers(-8, 9, (n, dim)).astype(np.float32)
        assert t.set(keys, vals) == 0 and r.set(keys, vals) == 0
        rounds = []
        for _ in range(4):
            q = wl.zipf_batch_np(rng, n, 1.05, b, seed=30 + w)
            g = rng.integers(-2, 3, (b, dim)).astype(np.float32)
            rounds.append((q, g, torch.from_numpy(q.view(np.int64)).cuda(), torch.from_numpy(g).cuda()))
        tables.append(t), oracles.append(r), bufs.append(rounds)
        streams.append(torch.cuda.Stream())
    torch.cuda.synchronize()
    for k in range(4):
        for w, t in enumerate(tables):
            q, g, dq, dg = bufs[w][k]
            assert t.push_dev(dq.data_ptr(), dg.data_ptr(), b, 0, streams[w].cuda_stream) == 0
    torch.cuda.synchronize()
    for w, (t, r) in enumerate(zip(tables, oracles)):
        assert t.size() == n                        # (also reads the sort's error flag)
        for q, g, _, _ in bufs[w]:
            assert r.push(q, g) == 0
        a = np.sort(t.dump()[1], order="key")
        bb = np.sort(r.dump()[1], order="key")
        np.testing.assert_array_equal(a["key"], bb["key"])
        np.testing.assert_array_equal(a["value"], bb["value"])
        t.close()
