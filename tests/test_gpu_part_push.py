"""The partitioned push (batches of 16,384 keys and more: tiles, partitions, one probe per distinct
key) against the CPU oracle, through the C ABI. Bars as everywhere: stored key sets bit-exact,
values bit-exact with integer gradients, within 1e-6 relative / 1e-7 absolute otherwise."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-6, 1e-7
OPTS = {
    "sum": dict(optimizer=0),
    "sgd": dict(optimizer=1, lr=0.01),
    "adagrad": dict(optimizer=2, lr=0.05, init_acc=0.1),
    "ftrl": dict(optimizer=3, alpha=0.05, beta=1.0, l1=1e-4, l2=1e-5),
    "user": dict(optimizer=4, lr=0.05, beta=0.9),   # the rule of csrc/user_opt.h: SGD with momentum
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


def test_value_floats_of_the_user_rule(ps, orc):
    assert ps.value_floats(8, ps.OPT_USER) == orc.lib().pso_value_floats(8, orc.OPT_USER) == 16


@pytest.mark.parametrize("opt,dim,s", [("sgd", 16, 1.05), ("adagrad", 64, 1.2), ("ftrl", 8, 1.1),
                                       ("adagrad", 128, 1.1), ("sgd", 3, 1.3), ("ftrl", 260, 1.1),
                                       ("sum", 1, 1.5), ("user", 16, 1.1), ("user", 6, 1.2)])
def test_zipf_batches_with_fresh_keys(ps, orc, wl, opt, dim, s):
    """Exact aggregation in the oracle (float64 sums, rounded once): the kernels add in double
    precision too, so the tolerance only covers the rounding of the tiles' partial sums."""
    rng = np.random.default_rng(dim)
    n_table, n = 50000, 40000 if dim <= 64 else 20000
    t = ps.Table(dim, capacity=n_table + 3 * n, max_batch=n, **OPTS[opt])
    r = orc.Oracle(dim, capacity=n_table + 3 * n, **OPTS[opt])
    fill(t, r, wl, rng, n_table, opt, dim, seed=3)
    for step in range(3):
        q = wl.zipf_batch_np(rng, n_table, s, n, seed=3)
        nf = n // 10
        q[:nf] = wl.fresh_keys_np(rng, nf)                 # keys the push inserts
        q[nf:nf + nf // 4] = q[:nf // 4]                    # some of them more than once
        rng.shuffle(q)
        g = rng.normal(0, 1e-3, (n, dim)).astype(np.float32)
        flags = ps.PUSH_NO_INSERT if step == 2 else 0
        assert t.push(q, g, flags) == 0, t.last_error()
        assert r.push(q, g, flags | orc.PUSH_EXACT_AGGREGATION) == 0
        same(t, r, exact=False)
        assert t.size() == r.size()
    t.close()


@pytest.mark.parametrize("dim", [1, 4, 16, 36])
def test_integer_gradients_bit_exact(ps, orc, dim):
    """Integer sums are exact in any order (pico-ps/test/TestOps.h:98-117): heavy repetition, one
    key that fills a fifth of the batch, keys inserted several times, all bit for bit."""
    rng = np.random.default_rng(dim + 100)
    t = ps.Table(dim, capacity=200_000, max_batch=150_000, **OPTS["sum"])
    r = orc.Oracle(dim, capacity=200_000, **OPTS["sum"])
    for n in (16384, 16385, 50_000, 150_000):
        keys = (rng.zipf(1.2, n).astype(np.uint64) * np.uint64(2654435761)) % np.uint64(60_000)
        keys[rng.integers(0, n, n // 5)] = 424242
        g = rng.integers(-3, 4, (n, dim)).astype(np.float32)
        assert t.push(keys, g) == 0 and r.push(keys, g) == 0
        same(t, r, exact=True)
    n = 70_000                       # one key only, then two keys
    for keys in (np.full(n, 7, np.uint64), np.where(np.arange(n) % 3 == 0, 8, 9).astype(np.uint64)):
        g = rng.integers(-3, 4, (n, dim)).astype(np.float32)
        assert t.push(keys, g) == 0 and r.push(keys, g) == 0
        same(t, r, exact=True)
    t.close()


def test_all_keys_distinct_and_all_new(ps, orc, wl):
    rng = np.random.default_rng(5)
    n, dim = 100_000, 8
    t = ps.Table(dim, capacity=2 * n, max_batch=n, **OPTS["adagrad"])
    r = orc.Oracle(dim, capacity=2 * n, **OPTS["adagrad"])
    keys = wl.fresh_keys_np(rng, n)
    g = rng.normal(0, 1e-2, (n, dim)).astype(np.float32)
    assert t.push(keys, g) == 0 and r.push(keys, g) == 0      # every key inserted by the push
    same(t, r, exact=True)                                    # nothing to aggregate: bit-exact
    assert t.push(keys, g) == 0 and r.push(keys, g) == 0      # every key present
    same(t, r, exact=True)
    assert t.size() == n
    t.close()


def test_partitions_that_need_several_passes(ps, orc, wl):
    """With the pass capacity turned down every partition of an ordinary batch takes the path of a
    partition crowded by hot keys: passes over its entries by hash class."""
    rng = np.random.default_rng(9)
    n_table, n, dim = 40000, 60000, 16
    t = ps.Table(dim, capacity=n_table + n, max_batch=n, **OPTS["sgd"])
    r = orc.Oracle(dim, capacity=n_table + n, **OPTS["sgd"])
    fill(t, r, wl, rng, n_table, "sgd", dim, seed=6)
    q = wl.zipf_batch_np(rng, n_table, 1.05, n, seed=6)
    q[:3000] = wl.fresh_keys_np(rng, 3000)
    g = rng.integers(-3, 4, (n, dim)).astype(np.float32)
    try:
        ps.debug_part_pass_capacity(256)
        assert t.push(q, g) == 0 and r.push(q, g) == 0
    finally:
        ps.debug_part_pass_capacity(0)
    same(t, r, exact=True)
    assert t.size() == r.size()
    t.close()


M64 = (1 << 64) - 1
C1, C2, GOLD = 0xff51afd7ed558ccd, 0xc4ceb9fe1a85ec53, 0x9E3779B97F4A7C15


def unmix64(h):
    """Inverse of MurmurHash3's 64-bit finaliser (the table's hash), on numpy uint64 arrays."""
    i1, i2 = np.uint64(pow(C1, -1, 1 << 64)), np.uint64(pow(C2, -1, 1 << 64))
    h = h ^ (h >> np.uint64(33))
    h = h * i2
    h = h ^ (h >> np.uint64(33))
    h = h * i1
    return h ^ (h >> np.uint64(33))


def test_hot_keys_that_agree_in_partition_and_class_bits(ps, orc, wl):
    """Five keys met in every one of 700 tiles, made to share one bucket of the hash array (hence
    the partition) and the low 30 bits of the hash by which a crowded partition is taken in passes:
    their 3,500 entries do not fit a pass, and the classes split thirty times before they part."""
    rng = np.random.default_rng(21)
    n_table, dim, tiles, tile = 40000, 4, 700, 4096
    n = tiles * tile
    # (room for a row per key of the batch: a table that might fill takes the sorted push)
    t = ps.Table(dim, capacity=n_table + n + 1000, max_batch=n, **OPTS["sgd"])
    r = orc.Oracle(dim, capacity=n_table + n + 1000, **OPTS["sgd"])
    table_keys = fill(t, r, wl, rng, n_table, "sgd", dim, seed=8)
    bucket_mask = np.uint64(t.stats().slots // 4 - 1)
    hot = np.zeros(0, dtype=np.uint64)
    with np.errstate(over="ignore"):
        for chunk in range(64):
            if len(hot) >= 5:
                break
            i = np.arange(chunk << 22, (chunk + 1) << 22, dtype=np.uint64) + np.uint64(1)
            c = (i << np.uint64(30)) | np.uint64(0x2AAAAAAA)
            h = unmix64(c) ^ np.uint64(GOLD)       # hash of the key whose class hash is c
            hot = np.concatenate([hot, unmix64(h[(h & bucket_mask) == np.uint64(77)])])
    hot = hot[:5]
    assert len(hot) == 5 and len(set(hot.tolist()) | set(table_keys.tolist())) == n_table + 5
    q = table_keys[rng.integers(0, n_table, (tiles, tile))]
    q[:, :5] = hot
    q = np.ascontiguousarray(q.reshape(-1))
    g = rng.integers(-3, 4, (n, dim)).astype(np.float32)
    assert t.push(q, g) == 0 and r.push(q, g) == 0
    assert t.size() == r.size() == n_table + 5
    same(t, r, exact=True)
    # The next pushes find that partition in the order the first one left: shared by several
    # workgroups from the start, a class of keys each. New keys of that partition (their buckets are
    # near the hot keys') then park where the workgroup that meets them has reserved room.
    bucket_bits = int(bucket_mask + 1).bit_length() - 1
    assert bucket_bits >= 19            # buckets 0 .. 127 share a partition however the push is cut (at most 4096 ways)
    for step in range(2):
        with np.errstate(over="ignore"):
            k = np.arange(300, dtype=np.uint64)
            near = unmix64(((k + np.uint64(1000 * (step + 1))) << np.uint64(40)) | (k % np.uint64(50) + np.uint64(70)))
        q2 = q.copy()
        q2[rng.choice(n, 300, replace=False)] = near
        g2 = rng.integers(-3, 4, (n, dim)).astype(np.float32)
        assert t.push(q2, g2) == 0 and r.push(q2, g2) == 0
        assert t.size() == r.size()
        same(t, r, exact=True)
    t.close()


def test_batches_of_changing_size_follow_and_drop_the_order(ps, orc, wl):
    """Pushes of 0.3M to 2.9M keys in turn, so that the number of partitions changes from push to
    push: the order a push leaves (fullest partitions first, crowded ones shared) is followed by the
    next push with the same cut and by no other. Integer gradients: bit for bit against the oracle,
    new keys in every batch, the last push without inserts."""
    rng = np.random.default_rng(77)
    n_table, dim = 120_000, 4
    sizes = [1_400_000, 1_400_000, 300_000, 2_900_000, 1_400_000, 700_000, 2_900_000, 2_900_000]
    cap = n_table + sum(sizes) // 50 + max(sizes) + 1000
    t = ps.Table(dim, capacity=cap, max_batch=max(sizes), **OPTS["sgd"])
    r = orc.Oracle(dim, capacity=cap, **OPTS["sgd"])
    fill(t, r, wl, rng, n_table, "sgd", dim, seed=12)
    for step, n in enumerate(sizes):
        q = wl.zipf_batch_np(rng, n_table, 1.15, n, seed=12)
        nf = n // 100
        q[rng.choice(n, nf, replace=False)] = wl.fresh_keys_np(rng, nf)
        g = rng.integers(-3, 4, (n, dim)).astype(np.float32)
        flags = ps.PUSH_NO_INSERT if step == len(sizes) - 1 else 0
        assert t.push(q, g, flags) == 0, t.last_error()
        assert r.push(q, g, flags) == 0
        assert t.size() == r.size()
        if step % 2 == 1 or step == len(sizes) - 1:
            same(t, r, exact=True)
    t.close()


def test_work_items_left_for_the_next_push_cover_every_partition(ps, wl):
    """What a push of 1024 partitions or more leaves for the next one (pshbm_debug_part_order): every
    partition once, or 2, 4 or 8 times with one class of keys each; spare slots marked; the crowded
    partition built here is among the shared ones. No oracle needed: an invariant of the order."""
    rng = np.random.default_rng(31)
    n_table, dim, tiles, tile = 60000, 4, 400, 4096
    n = tiles * tile
    t = ps.Table(dim, capacity=n_table + n + 1000, max_batch=n, **OPTS["sum"])
    keys = wl.table_keys_np(0, n_table, seed=4)
    assert t.set(keys, np.zeros((n_table, dim), np.float32)) == 0
    items, parts = t.debug_part_order()
    assert parts == 0 and items.size == 0
    q = keys[rng.integers(0, n_table, (tiles, tile))]
    with np.errstate(over="ignore"):                # six keys met in every tile, made to lie in buckets 0 .. 5:
        hot = unmix64(((np.arange(6, dtype=np.uint64) + np.uint64(1)) << np.uint64(40)) | np.arange(6, dtype=np.uint64))
    q[:, :6] = hot                                  # one partition holds their 2,400 entries
    q = np.ascontiguousarray(q.reshape(-1))
    g = np.ones((n, dim), np.float32)
    for step in range(2):
        assert t.push(q, g) == 0
        items, parts = t.debug_part_order()
        assert parts >= 1024 and items.size == parts + parts // 8
        live = items[items != 0xFFFFFFFF]
        p, lg, cls = live & 0xFFFF, (live >> 16) & 3, live >> 20
        assert (p < parts).all() and (cls < (1 << lg)).all()
        seen = {}
        for pi, li, ci in zip(p.tolist(), lg.tolist(), cls.tolist()):
            seen.setdefault(pi, []).append((li, ci))
        assert sorted(seen) == list(range(parts))                       # every partition
        assert len(seen[0]) > 1                                          # the crowded one shared
        for pi, lst in seen.items():
            l0 = lst[0][0]
            assert sorted(lst) == [(l0, c) for c in range(1 << l0)]     # once, or every class once
        # slot x belongs to run x & 7 of parts / 8 consecutive partitions
        x = np.flatnonzero(items != 0xFFFFFFFF)
        assert ((items[x] & 0xFFFF) // (parts // 8) == (x & 7)).all()
    st, rows, hit = t.pull(hot)
    times = np.array([(q == k).sum() for k in hot], dtype=np.float32)
    assert st == 0 and hit.all() and (rows == 2 * times[:, None]).all()    # both pushes, every occurrence once
    t.close()


def test_track_increment_through_the_partitioned_push(ps, orc, wl):
    rng = np.random.default_rng(13)
    n_table, n, dim = 30000, 20000, 4
    t = ps.Table(dim, capacity=n_table + n, max_batch=n, track_increment=True, **OPTS["sgd"])
    keys = wl.table_keys_np(0, n_table, seed=8)
    assert t.set(keys, np.zeros((n_table, dim), np.float32)) == 0
    q = np.concatenate([keys[rng.integers(0, n_table, n - 500)], wl.fresh_keys_np(rng, 500)])
    g = rng.normal(0, 1, (n, dim)).astype(np.float32)
    assert t.push(q, g) == 0
    st, rec = t.take_increment()
    assert st == 0
    np.testing.assert_array_equal(np.sort(rec["key"]), np.unique(q))
    t.close()
