"""The key partitioner: partition = jump_consistent_hash(murmur_hash(key), n), the shape of the
reference's DefaultPartitioner<uint64_t> (pico-ps/common/Partitioner.h:43-61). Both functions live
in pico-core, which the reference tree does not hold, so parity with the reference's own numbers is
unpinned; what is pinned here is that the oracle (and, byte for byte, the library's host function)
computes the two PUBLISHED functions: MurmurHash3's 64-bit finalizer and the jump consistent hash of
Lamping and Veach (arXiv:1406.2294)."""
import numpy as np
import pytest

M64 = (1 << 64) - 1


def fmix64(k):                     # MurmurHash3 finalizer, integers only
    k ^= k >> 33
    k = (k * 0xFF51AFD7ED558CCD) & M64
    k ^= k >> 33
    k = (k * 0xC4CEB9FE1A85EC53) & M64
    k ^= k >> 33
    return k


def jump(key, n):                  # the paper's loop; Python floats are IEEE doubles
    b, j = -1, 0
    while j < n:
        b = j
        key = (key * 2862933555777941757 + 1) & M64
        j = int((b + 1) * (float(1 << 31) / float((key >> 33) + 1)))
    return b


def test_jump_consistent_hash_published_vectors():
    """Test vectors of github.com/dgryski/go-jump (the widely used Go port of the paper's code)."""
    for key, n, want in [(1, 1, 0), (42, 57, 43), (0xDEAD10CC, 1, 0), (0xDEAD10CC, 666, 361), (256, 1024, 520)]:
        assert jump(key, n) == want


def test_oracle_and_library_compute_the_published_functions(orc, ps):
    rng = np.random.default_rng(5)
    keys = [0, 1, 2, 42, 0xDEAD10CC, M64 - 2] + [int(x) for x in rng.integers(0, 1 << 63, 400, dtype=np.uint64)]
    for n in (1, 2, 3, 7, 64, 1000, 65536, (1 << 31) - 1):
        for k in keys:
            want = jump(fmix64(k), n)
            assert orc.partition(k, n) == want
            assert ps.partition(k, n) == want       # host function of the C ABI: no device needed
    assert orc.partition(5, 0) == -1 and ps.partition(5, 0) == -1 and ps.partition(5, -3) == -1


def test_properties_of_a_consistent_hash(orc):
    """What the paper proves: with one bucket everything is in bucket 0; when a bucket is added a key
    stays where it is or moves to the NEW bucket; about 1/(n+1) of the keys move; even spread."""
    rng = np.random.default_rng(6)
    keys = [int(x) for x in rng.integers(0, 1 << 63, 20000, dtype=np.uint64)]
    assert all(orc.partition(k, 1) == 0 for k in keys[:200])
    for n in (1, 2, 5, 16, 100):
        a = np.array([orc.partition(k, n) for k in keys])
        b = np.array([orc.partition(k, n + 1) for k in keys])
        assert a.min() >= 0 and a.max() < n
        moved = a != b
        assert (b[moved] == n).all()
        assert abs(moved.mean() - 1.0 / (n + 1)) < 0.02
        counts = np.bincount(a, minlength=n)
        mean = len(keys) / n
        assert np.abs(counts - mean).max() < 5 * np.sqrt(mean)          # binomial spread, five sigma


def test_partition_terms_of_the_oracle_predicate(orc):
    o = orc.Oracle(2, capacity=5000)
    keys = np.arange(1, 3001, dtype=np.uint64) * np.uint64(0x9E3779B97F4A7C15)
    keys = keys[keys < np.uint64(M64 - 1)]
    vals = np.ones((keys.size, 2), np.float32)
    assert o.set(keys, vals) == 0
    n = 7
    mine = np.array([jump(fmix64(int(k)), n) for k in keys])
    total = 0
    for p in range(n):
        st, cnt, _ = o.for_each(orc.predicate((orc.COL_KEY, orc.CMP_PART_EQ, (n, p))))
        assert st == 0 and cnt == int((mine == p).sum())
        total += cnt
    assert total == keys.size
    st, gone = o.erase_if(orc.predicate((orc.COL_KEY, orc.CMP_PART_NE, (n, 3))))   # the purge of shard 3
    assert st == 0 and gone == int((mine != 3).sum()) and o.size() == int((mine == 3).sum())
    o.close()


@pytest.mark.gpu
def test_device_partition_terms_match_the_oracle(ps, orc, wl):
    """for_each by partition and the purge of a shard (erase every key whose partition is not this
    shard's: pico-ps/operator/UpdateContextOperator.h:143-196) on the device, against the oracle."""
    rng = np.random.default_rng(7)
    n_keys, dim = 200_000, 4
    t = ps.Table(dim, capacity=n_keys + 16, optimizer=0)
    r = orc.Oracle(dim, capacity=n_keys + 16, optimizer=0)
    keys = wl.table_keys_np(0, n_keys, seed=13)
    vals = rng.integers(-4, 5, (n_keys, dim)).astype(np.float32)
    assert t.set(keys, vals) == 0 and r.set(keys, vals) == 0
    for n, p in ((1, 0), (3, 2), (16, 5), (1000, 999), ((1 << 31) - 1, 12345)):
        a = t.for_each(ps.predicate((ps.COL_KEY, ps.CMP_PART_EQ, (n, p))))
        b = r.for_each(orc.predicate((orc.COL_KEY, orc.CMP_PART_EQ, (n, p))))
        assert a[0] == b[0] == 0 and a[1] == b[1]
        np.testing.assert_array_equal(a[2], b[2])
    sample = keys[:2000]
    assert [ps.partition(int(k), 16) for k in sample] == [orc.partition(int(k), 16) for k in sample]
    a = t.erase_if(ps.predicate((ps.COL_KEY, ps.CMP_PART_NE, (16, 5))))
    b = r.erase_if(orc.predicate((orc.COL_KEY, orc.CMP_PART_NE, (16, 5))))
    assert a == b and a[0] == 0 and 0 < t.size() == r.size() < n_keys // 8
    st, rec = t.dump()
    assert all(ps.partition(int(k), 16) == 5 for k in rec["key"][:500])
    x, y = np.sort(rec, order="key"), np.sort(r.dump()[1], order="key")
    np.testing.assert_array_equal(x["key"], y["key"])
    np.testing.assert_array_equal(x["value"], y["value"])
    assert t.for_each(ps.predicate((0, ps.CMP_PART_EQ, 1.0)))[0] == ps.INVALID_CONFIG      # a partition test needs the key
    assert t.for_each(ps.predicate((ps.COL_KEY, ps.CMP_PART_EQ, (0, 0))))[0] == ps.INVALID_CONFIG   # ... and partitions
    t.close()
