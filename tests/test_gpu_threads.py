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
