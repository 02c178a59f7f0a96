"""The push entry point that allocates nothing (pshbm_push_dev_noalloc), through the C ABI: its
results must be those of pshbm_push_dev from the same state, on two calls in a row, the second
with a smaller batch (the fixed scratch keeps what the first call left in it)."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-6, 1e-7


def dump_sorted(t):
    st, rec = t.dump()
    assert st == 0
    return np.sort(rec, order="key")


@pytest.mark.parametrize("dim,opt", [(16, dict(optimizer=2, lr=0.05, init_acc=0.1)),
                                      (64, dict(optimizer=3, alpha=0.05, beta=1.0, l1=1e-4, l2=1e-5)),
                                      (3, dict(optimizer=1, lr=0.01))])
def test_noalloc_push_matches_push_dev(ps, wl, dim, opt):
    rng = np.random.default_rng(dim)
    n_table = 20000
    a = ps.Table(dim, capacity=n_table + 40000, **opt)
    b = ps.Table(dim, capacity=n_table + 40000, **opt)
    keys = wl.table_keys_np(0, n_table, seed=4)
    vals = rng.normal(0, 0.01, (n_table, a.value_floats)).astype(np.float32)
    if opt["optimizer"] == 2:
        vals[:, dim:] = 0.1
    if opt["optimizer"] == 3:
        vals[:, 2 * dim:] = vals[:, dim:2 * dim] ** 2
    assert a.set(keys, vals) == 0 and b.set(keys, vals) == 0
    stream = torch.cuda.current_stream().cuda_stream
    # 16384 keys is the entry point's limit (dim 64: also its limit of 2^20 gradient floats);
    # then smaller batches, down to the one-launch push, on the scratch the larger ones used
    for n in (16384, 5000, 16000, 300):
        q = wl.zipf_batch_np(rng, n_table, 1.1, n, seed=4)
        q[: n // 8] = wl.fresh_keys_np(rng, n // 8)       # insert-on-miss
        q[n // 8: n // 8 + n // 40] = q[: n // 40]         # new keys that repeat in the batch
        g = rng.normal(0, 1e-3, (n, dim)).astype(np.float32)
        dk = torch.from_numpy(q.view(np.int64)).cuda()
        dg = torch.from_numpy(g).cuda()
        assert a.push_dev_noalloc(dk.data_ptr(), dg.data_ptr(), n, 0, stream) == 0, a.last_error()
        assert b.push_dev(dk.data_ptr(), dg.data_ptr(), n, 0, stream) == 0, b.last_error()
        torch.cuda.synchronize()
        x, y = dump_sorted(a), dump_sorted(b)
        np.testing.assert_array_equal(x["key"], y["key"])
        np.testing.assert_allclose(x["value"], y["value"], rtol=RTOL, atol=ATOL)
    assert a.size() == b.size()
    a.close(), b.close()


def test_noalloc_push_rejects_what_does_not_fit(ps):
    t = ps.Table(128, capacity=1000, optimizer=1, lr=0.1)
    dk = torch.zeros(20000, dtype=torch.int64, device="cuda")
    dg = torch.zeros(20000, 128, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    assert t.push_dev_noalloc(dk.data_ptr(), dg.data_ptr(), 16385, 0, stream) == ps.ERROR
    assert "16384" in t.last_error()
    assert t.push_dev_noalloc(dk.data_ptr(), dg.data_ptr(), 8193, 0, stream) == ps.ERROR   # 8193 x 128 > 2^20
    assert t.push_dev_noalloc(dk.data_ptr(), dg.data_ptr(), 0, 0, stream) == 0
    assert t.size() == 0
    t.close()
