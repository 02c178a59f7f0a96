"""Properties of the HIP path at the full sizes of the benchmark's configurations (needs an MI355X).

At 10^8 keys the CPU oracle is out of reach, so these tests use what the domain fixes without it:
  * stored values are a closed form of the key's index, so any pulled row is known in advance;
  * with a step of 0.5 and integer gradients SGD is exact in fp32, so a pushed value is the closed
    form minus half the integer sum of the key's gradients, whatever the order of the additions
    (the reference's own test operator relies on the same fact, pico-ps/test/TestOps.h:98-117);
  * pushing g and then -g restores the table bit for bit; a zero gradient changes nothing;
  * rows are numbered in insertion order, so the shard iterator returns the keys in the order the
    table was built.
Everything goes through the device-pointer entry points of the C ABI with torch tensors as the
device buffers.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def closed_form(idx, dim, vf):
    """value row of key index idx (int64 tensor): small integers, exact in fp32"""
    c = torch.arange(vf, device=idx.device, dtype=torch.int64)
    v = ((idx[:, None] + 7 * c[None, :]) % 251 - 125).to(torch.float32)
    return v


def build(ps, wl, n_table, dim, opt, batch, extra_capacity, state_fill=None, square_last=False):
    t = ps.Table(dim, capacity=n_table + extra_capacity, max_batch=batch, **opt)
    vf = t.value_floats
    stream = torch.cuda.current_stream().cuda_stream
    chunk = 4_000_000
    for start in range(0, n_table, chunk):
        cnt = min(chunk, n_table - start)
        idx = torch.arange(start, start + cnt, dtype=torch.int64, device="cuda")
        keys = wl.keys_of_index_torch(idx, 0)
        vals = closed_form(idx, dim, vf)
        if state_fill is not None:
            vals[:, dim:] = state_fill
        if square_last:                                  # FTRL: n = z^2, so that n >= 0
            vals[:, 2 * dim:] = vals[:, dim:2 * dim] ** 2
        assert t.set_dev(keys.data_ptr(), vals.data_ptr(), cnt, stream) == 0, t.last_error()
        torch.cuda.synchronize()
    assert t.size() == n_table
    return t


def pull(t, keys, dim):
    n = keys.numel()
    out = torch.empty(n, dim, device="cuda")
    hit = torch.empty(n, dtype=torch.uint8, device="cuda")
    st = t.pull_dev(keys.data_ptr(), n, out.data_ptr(), hit.data_ptr(), 0,
                    torch.cuda.current_stream().cuda_stream)
    assert st == 0, t.last_error()
    torch.cuda.synchronize()
    return out, hit


def push(t, keys, grads, flags=0):
    st = t.push_dev(keys.data_ptr(), grads.data_ptr(), keys.numel(), flags,
                    torch.cuda.current_stream().cuda_stream)
    assert st == 0, t.last_error()
    torch.cuda.synchronize()


def zipf_indices(wl, gen, n_table, s, count):
    return wl.rank_to_index_torch(wl.zipf_ranks_torch(gen, n_table, s, count, "cuda"), n_table)


def summed_by_index(idx, grads):
    """(distinct indices, integer sum of the gradients of each) -- exact whatever the order"""
    uniq, inv = torch.unique(idx, return_inverse=True)
    acc = torch.zeros(uniq.numel(), grads.shape[1], device="cuda", dtype=torch.float64)
    acc.index_add_(0, inv, grads.to(torch.float64))
    return uniq, acc


def test_c2_size_exact_properties(ps, wl):
    """C2: 100M keys, dim 16, SGD, 1M-key Zipf(1.05) batches."""
    n_table, dim, batch = 100_000_000, 16, 1_000_000
    t = build(ps, wl, n_table, dim, dict(optimizer=1, lr=0.5), batch, 8 * batch)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(3)
    idx = zipf_indices(wl, gen, n_table, 1.05, batch)
    keys = wl.keys_of_index_torch(idx, 0)

    # pull: closed form, every key found; twice the same; absent keys give zeros and no insert
    out, hit = pull(t, keys, dim)
    assert bool(hit.all())
    assert torch.equal(out, closed_form(idx, dim, dim))
    out2, _ = pull(t, keys, dim)
    assert torch.equal(out, out2)
    absent = wl.keys_of_index_torch(torch.arange(n_table, n_table + batch, device="cuda"), 0)
    out3, hit3 = pull(t, absent, dim)
    assert not bool(hit3.any()) and not bool(out3.any()) and t.size() == n_table

    # push: value = closed form - 0.5 * integer sum over the key's occurrences
    g = torch.randint(-3, 4, (batch, dim), device="cuda", generator=gen).to(torch.float32)
    push(t, keys, g)
    uniq, acc = summed_by_index(idx, g)
    ukeys = wl.keys_of_index_torch(uniq, 0)
    got, hit = pull(t, ukeys, dim)
    want = (closed_form(uniq, dim, dim).to(torch.float64) - 0.5 * acc).to(torch.float32)
    assert bool(hit.all()) and torch.equal(got, want)
    assert t.size() == n_table                       # nothing was inserted

    # keys the batch did not touch are untouched (a uniform sample; touched ones are skipped)
    sample = torch.randint(0, n_table, (batch,), device="cuda", generator=gen)
    pos = torch.searchsorted(uniq, sample).clamp(max=uniq.numel() - 1)
    untouched = uniq[pos] != sample
    got, _ = pull(t, wl.keys_of_index_torch(sample, 0), dim)
    assert torch.equal(got[untouched], closed_form(sample, dim, dim)[untouched])

    # a zero gradient changes nothing; -g undoes g bit for bit
    push(t, keys, torch.zeros_like(g))
    got, _ = pull(t, ukeys, dim)
    assert torch.equal(got, want)
    push(t, keys, -g)
    got, _ = pull(t, ukeys, dim)
    assert torch.equal(got, closed_form(uniq, dim, dim))

    # insert-on-miss inside a push: new keys start from zero weights, repeated new keys are summed
    fresh_idx = torch.randint(n_table, n_table + 50_000, (200_000,), device="cuda", generator=gen)
    mixed_idx = torch.cat([idx[: batch - 200_000], fresh_idx])
    mixed_keys = wl.keys_of_index_torch(mixed_idx, 0)
    push(t, mixed_keys, g)
    uniq2, acc2 = summed_by_index(mixed_idx, g)
    n_new = int((uniq2 >= n_table).sum())
    assert t.size() == n_table + n_new
    base = closed_form(uniq2, dim, dim).to(torch.float64)
    base[uniq2 >= n_table] = 0.0
    got, hit = pull(t, wl.keys_of_index_torch(uniq2, 0), dim)
    assert bool(hit.all()) and torch.equal(got, (base - 0.5 * acc2).to(torch.float32))

    # the shard iterator walks the rows in insertion order
    st, rec = t.iterate(n_table - 1000, 1000)
    assert st == 0 and rec.size == 1000
    np.testing.assert_array_equal(rec["key"], wl.table_keys_np(n_table - 1000, 1000, seed=0))
    st, rec = t.iterate(12_345_678, 500)
    np.testing.assert_array_equal(rec["key"], wl.table_keys_np(12_345_678, 500, seed=0))
    t.close()


def test_c5_size_properties(ps, wl):
    """C5, the largest table of the configs: 200M keys, dim 128 + 128 accumulators (215 GB),
    Adagrad, 4M-key Zipf(1.1) batches. Adagrad is not exact in fp32, so the pushed values are
    compared with a float64 evaluation of the update at the tolerance of the parity tests."""
    n_table, dim, batch = 200_000_000, 128, 4_000_000
    lr, acc0 = 0.05, 0.1
    torch.cuda.empty_cache()
    free_b, _ = torch.cuda.mem_get_info()
    if free_b < 240e9:
        pytest.skip("needs 240 GB of free HBM")
    t = build(ps, wl, n_table, dim, dict(optimizer=2, lr=lr, init_acc=acc0), batch, 2 * batch,
              state_fill=acc0)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(4)
    idx = zipf_indices(wl, gen, n_table, 1.1, batch)
    keys = wl.keys_of_index_torch(idx, 0)
    out, hit = pull(t, keys, dim)
    assert bool(hit.all()) and torch.equal(out, closed_form(idx, dim, dim))
    del out
    # the very last row of the slab is where a 32-bit byte offset would have wrapped long ago
    last = torch.arange(n_table - 1000, n_table, device="cuda")
    out, hit = pull(t, wl.keys_of_index_torch(last, 0), dim)
    assert bool(hit.all()) and torch.equal(out, closed_form(last, dim, dim))

    g = torch.randint(-3, 4, (batch, dim), device="cuda", generator=gen).to(torch.float32) * 0.25
    push(t, keys, g)
    uniq, acc = summed_by_index(idx, g)               # exact: multiples of 0.25
    del g
    n_acc = acc0 + acc * acc
    want = closed_form(uniq, dim, dim).to(torch.float64) - lr * acc / torch.sqrt(n_acc)
    got, hit = pull(t, wl.keys_of_index_torch(uniq, 0), dim)
    assert bool(hit.all())
    err = (got.to(torch.float64) - want).abs()
    assert bool((err <= 1e-7 + 1e-6 * want.abs()).all()), float(err.max())
    assert t.size() == n_table
    t.close()


def test_c4_size_aggregation_matches_presummed(ps, wl):
    """C4: 500M keys, dim 8, FTRL (w, z, n), 4M-key batches with keys pushed for the first time.
    FTRL is not exact in fp32, but two keys with the same state that receive the same total
    gradient must end bit-identical: key index i and i + 251,000,000 hold the same closed-form
    state; the batch pushes the first with its Zipf duplicates and the second once with the
    integer sum of those gradients."""
    n_table, dim, batch = 500_000_000, 8, 4_000_000
    twin = 251_000_000
    t = build(ps, wl, n_table, dim, dict(optimizer=3, alpha=0.05, beta=1.0, l1=1e-4, l2=1e-5), batch,
              2 * batch, square_last=True)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(5)
    half = 1_900_000
    idx_a = zipf_indices(wl, gen, n_table - twin, 1.1, half)
    g_a = torch.randint(-3, 4, (half, dim), device="cuda", generator=gen).to(torch.float32)
    uniq, acc = summed_by_index(idx_a, g_a)
    idx_b = uniq + twin
    g_b = acc.to(torch.float32)
    n_fresh = batch - half - uniq.numel()
    assert n_fresh > 100_000
    idx_f = torch.randint(n_table, n_table + 60_000, (n_fresh,), device="cuda", generator=gen)
    g_f = torch.randint(-3, 4, (n_fresh, dim), device="cuda", generator=gen).to(torch.float32)
    idx = torch.cat([idx_a, idx_b, idx_f])
    g = torch.cat([g_a, g_b, g_f])
    perm = torch.randperm(batch, device="cuda", generator=gen)
    idx, g = idx[perm], g[perm].contiguous()
    push(t, wl.keys_of_index_torch(idx, 0), g)
    assert t.size() == n_table + int(torch.unique(idx_f).numel())
    got_a, hit_a = pull(t, wl.keys_of_index_torch(uniq, 0), dim)
    got_b, hit_b = pull(t, wl.keys_of_index_torch(idx_b, 0), dim)
    assert bool(hit_a.all()) and bool(hit_b.all())
    assert torch.equal(got_a, got_b)
    changed = (got_a != closed_form(uniq, dim, dim)).any(dim=1)
    assert float(changed.float().mean()) > 0.9      # the push did something
    # fresh keys pushed several times equal the same keys pushed once with the summed gradient
    uf, accf = summed_by_index(idx_f, g_f)
    twin_f = uf + 1_000_000                           # not stored either
    push(t, wl.keys_of_index_torch(twin_f, 0), accf.to(torch.float32))
    got_f, _ = pull(t, wl.keys_of_index_torch(uf, 0), dim)
    got_tf, _ = pull(t, wl.keys_of_index_torch(twin_f, 0), dim)
    assert torch.equal(got_f, got_tf)
    # a push that may not insert drops absent keys and leaves the table as it is
    absent = wl.keys_of_index_torch(torch.arange(n_table + 5_000_000, n_table + 5_000_000 + batch,
                                                 device="cuda"), 0)
    size_before = t.size()
    push(t, absent, g, ps.PUSH_NO_INSERT)
    assert t.size() == size_before
    again, _ = pull(t, wl.keys_of_index_torch(uniq, 0), dim)
    assert torch.equal(again, got_a)
    t.close()


def test_c2_size_for_each_and_erase_if(ps, wl):
    """For-each and erase-if over 100M keys: the column sums of the closed form are integers, so
    the float64 sums are exact in any order; erasing the keys with an odd index-derived column
    leaves exactly the others, dense, with their values, and the table keeps working."""
    import time
    n_table, dim, batch = 100_000_000, 16, 1_000_000
    t = build(ps, wl, n_table, dim, dict(optimizer=1, lr=0.5), batch, 8 * batch)
    # expected column sums of the closed form, in chunks (exact integers in float64)
    want = torch.zeros(dim, dtype=torch.float64, device="cuda")
    n_sel = 0
    sel_sum = torch.zeros(dim, dtype=torch.float64, device="cuda")
    for start in range(0, n_table, 10_000_000):
        idx = torch.arange(start, start + 10_000_000, device="cuda")
        v = closed_form(idx, dim, dim).to(torch.float64)
        want += v.sum(0)
        m = v[:, 3] > 100.0                       # column 3 above 100: about a tenth of the keys
        n_sel += int(m.sum())
        sel_sum += v[m].sum(0)
    torch.cuda.synchronize()
    st, cnt, sums = t.for_each()                  # the first call also allocates the scratch
    t0 = time.perf_counter()
    st, cnt, sums = t.for_each()
    dt_all = time.perf_counter() - t0
    assert st == 0 and cnt == n_table
    np.testing.assert_array_equal(sums, want.cpu().numpy())
    where = ps.predicate((3, ps.CMP_GT, 100.0))
    st, cnt, sums = t.for_each(where)
    assert st == 0 and cnt == n_sel
    np.testing.assert_array_equal(sums, sel_sum.cpu().numpy())

    t0 = time.perf_counter()
    st, erased = t.erase_if(where)
    dt_erase = time.perf_counter() - t0
    assert st == 0 and erased == n_sel and t.size() == n_table - n_sel
    st, cnt, sums = t.for_each()
    assert cnt == n_table - n_sel
    np.testing.assert_array_equal(sums, (want - sel_sum).cpu().numpy())
    assert t.for_each(where)[1] == 0
    # erased keys miss, the others keep their rows; the slab is dense again
    gen = torch.Generator(device="cuda")
    gen.manual_seed(6)
    idx = torch.randint(0, n_table, (batch,), device="cuda", generator=gen)
    v = closed_form(idx, dim, dim)
    gone = v[:, 3] > 100.0
    out, hit = pull(t, wl.keys_of_index_torch(idx, 0), dim)
    assert torch.equal(hit.bool(), ~gone)
    assert torch.equal(out[~gone], v[~gone]) and not bool(out[gone].any())
    st, rec = t.iterate(n_table - n_sel - 1000, 2000)
    assert st == 0 and rec.size == 1000 and not (rec["value"][:, 3] > 100.0).any()
    # pushes after the erase: erased keys come back as new keys (zero weights), others update
    g = torch.ones(batch, dim, device="cuda")
    uniq = torch.unique(idx)
    push(t, wl.keys_of_index_torch(uniq, 0), g[: uniq.numel()])
    vu = closed_form(uniq, dim, dim)
    vu[vu[:, 3] > 100.0] = 0.0
    out, hit = pull(t, wl.keys_of_index_torch(uniq, 0), dim)
    assert bool(hit.all()) and torch.equal(out, vu - 0.5)
    print(f"\nfor_each over {n_table} rows: {dt_all * 1e3:.2f} ms; erase_if of {n_sel} rows: {dt_erase * 1e3:.2f} ms")
    t.close()


def test_c1_size_pulls_match_the_closed_form(ps, wl):
    """C1: 1M keys, dim 8, read-only serving: 100 pulls of 65,536 uniform keys each, a tenth of
    them absent, every pulled row and every hit flag against the closed form; then the same keys
    again (a pull changes nothing)."""
    n_table, dim, batch = 1_000_000, 8, 65_536
    t = build(ps, wl, n_table, dim, dict(optimizer=1, lr=0.01), batch, 16)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(7)
    first = None
    for step in range(100):
        idx = torch.randint(0, n_table + n_table // 9, (batch,), device="cuda", generator=gen)   # a tenth absent
        keys = wl.keys_of_index_torch(idx, 0)
        out, hit = pull(t, keys, dim)
        present = idx < n_table
        assert torch.equal(hit.bool(), present)
        want = closed_form(idx, dim, dim)
        want[~present] = 0.0
        assert torch.equal(out, want)
        if step == 0:
            first = (keys, out)
    out, _ = pull(t, first[0], dim)
    assert torch.equal(out, first[1]) and t.size() == n_table
    t.close()


def test_c3_size_adagrad_against_float64(ps, wl):
    """C3: 50M keys, dim 64 + 64 accumulators, Adagrad, 2M-key Zipf(1.2) batches (the hottest key
    about 200,000 times). The gradients are multiples of 0.25, so their sums are exact in any order
    and the update is one float64 formula per element; the pull before and after goes with row
    handles, the second push takes them."""
    n_table, dim, batch = 50_000_000, 64, 2_000_000
    lr, acc0 = 0.05, 0.1
    t = build(ps, wl, n_table, dim, dict(optimizer=2, lr=lr, init_acc=acc0), batch, 2 * batch, state_fill=acc0)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(8)
    stream = torch.cuda.current_stream().cuda_stream
    idx = zipf_indices(wl, gen, n_table, 1.2, batch)
    keys = wl.keys_of_index_torch(idx, 0)
    out = torch.empty(batch, dim, device="cuda")
    handles = torch.empty(batch, dtype=torch.int32, device="cuda")
    st, epoch = t.pull_dev_handles(keys.data_ptr(), batch, out.data_ptr(), handles.data_ptr(), None, 0, stream)
    assert st == 0, t.last_error()
    torch.cuda.synchronize()
    assert torch.equal(out, closed_form(idx, dim, dim))

    g = torch.randint(-3, 4, (batch, dim), device="cuda", generator=gen).to(torch.float32) * 0.25
    push(t, keys, g)                                   # the plain push
    uniq, acc = summed_by_index(idx, g)
    n1 = acc0 + acc * acc
    w1 = closed_form(uniq, dim, dim).to(torch.float64) - lr * acc / torch.sqrt(n1)
    got, hit = pull(t, wl.keys_of_index_torch(uniq, 0), dim)
    assert bool(hit.all())
    err = (got.to(torch.float64) - w1).abs()
    assert bool((err <= 1e-7 + 1e-6 * w1.abs()).all()), float(err.max())

    # the same batch again through the handles of the first pull (rows have not moved)
    st = t.push_dev_handles(keys.data_ptr(), g.data_ptr(), handles.data_ptr(), epoch, batch, 0, stream)
    assert st == 0, t.last_error()
    torch.cuda.synchronize()
    n2 = n1 + acc * acc
    w2 = w1 - lr * acc / torch.sqrt(n2)
    got, hit = pull(t, wl.keys_of_index_torch(uniq, 0), dim)
    err = (got.to(torch.float64) - w2).abs()
    assert bool((err <= 2e-7 + 2e-6 * w2.abs()).all()), float(err.max())   # two rounded steps
    assert t.size() == n_table
    t.close()
