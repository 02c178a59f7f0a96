"""Writes tests/golden/reference_known_answers.json: the scenarios of the reference's own tests
for the sparse-table path, restated as operation lists with the results those tests assert.

Nothing here runs the reference or the oracle: every expected number is the closed form that the
cited reference test checks (all integer valued). The reference's TestValue{sum,count}
(pico-ps/test/TestOps.h:53-58) is modelled as a dim-2 row [sum, count] under the SUM optimizer, and
a push of arg=key (apply_push_arg: sum += arg, count += 1, TestOps.h:98-103) as the gradient
[key, 1].

Run from the repository root:  python tests/golden/make_reference_known_answers.py
"""
import json
import os

TEST_KEY_NUM = 100  # pico-ps/test/TestOps.h:12


def test_sparse(num_process):
    """pico-ps/test/ps_service_test.cpp:77-184 (test_sparse) on one shard."""
    ops = []
    all_keys = []
    for rank in range(num_process):
        keys = list(range(rank * TEST_KEY_NUM, (rank + 1) * TEST_KEY_NUM))
        grads = [[k, 1] for k in keys]
        all_keys += keys
        ops.append({"op": "push", "keys": keys, "grads": grads})          # async_push, :104
        ops.append({"op": "queue", "keys": keys, "grads": grads})         # sync_push, :106
        if rank % 2 == 0:
            ops.append({"op": "queue", "keys": keys, "grads": grads})     # even ranks again, :108-111
    ops.append({"op": "store"})                                           # :120
    ops.append({"op": "expect_size", "value": TEST_KEY_NUM * num_process})  # :122

    def row(k):
        count = 2 + (1 if (k // TEST_KEY_NUM) % 2 == 0 else 0)  # TestOps.h:170-172
        return [k * count, count]

    # dump, load into a new storage, clear, restore (:125-156): same size, same pulls
    ops.append({"op": "dump_load_roundtrip", "expect_size": TEST_KEY_NUM * num_process})
    ops.append({"op": "expect_pull", "keys": all_keys, "rows": [row(k) for k in all_keys],
                "hit": [1] * len(all_keys)})                              # :204-213 (x5: idempotent)
    ops.append({"op": "expect_pull", "keys": all_keys, "rows": [row(k) for k in all_keys],
                "hit": [1] * len(all_keys)})
    # a key that is not stored pulls the default value 0 and is not inserted
    # (pico-ps/operator/SparsePullOperator.h:307-310; ps_service_test.cpp:176-184 for erased keys)
    missing = [TEST_KEY_NUM * num_process + i for i in range(10)]
    ops.append({"op": "expect_pull", "keys": missing, "rows": [[0, 0]] * len(missing),
                "hit": [0] * len(missing)})
    ops.append({"op": "expect_size", "value": TEST_KEY_NUM * num_process})
    # for-each over every record: num = records, and the merged sum / count columns
    # (TestForEachOperator, TestOps.h:159-185; ps_service_test.cpp:158-161)
    ops.append({"op": "expect_for_each", "where": [], "count": len(all_keys),
                "sums": [sum(row(k)[0] for k in all_keys), sum(row(k)[1] for k in all_keys)]})
    # erase_if(key % 2) (TestEraseIfOperator, TestOps.h:138-150), then half the records are left
    # (ps_service_test.cpp:163-166) and an erased key pulls 0 (:176-184)
    odd = [[-1, 6, [2, 1]]]   # key % 2 == 1
    even_keys = [k for k in all_keys if k % 2 == 0]
    ops.append({"op": "erase_if", "where": odd, "erased": len(all_keys) - len(even_keys)})
    ops.append({"op": "expect_for_each", "where": [], "count": len(even_keys),
                "sums": [sum(row(k)[0] for k in even_keys), sum(row(k)[1] for k in even_keys)]})
    ops.append({"op": "expect_size", "value": len(even_keys)})
    ops.append({"op": "expect_pull", "keys": all_keys,
                "rows": [row(k) if k % 2 == 0 else [0, 0] for k in all_keys],
                "hit": [1 if k % 2 == 0 else 0 for k in all_keys]})
    ops.append({"op": "clear"})                                           # :153
    ops.append({"op": "expect_size", "value": 0})                         # :154
    return {"name": f"test_sparse_{num_process}", "dim": 2, "optimizer": "SUM",
            "cite": "pico-ps/test/ps_service_test.cpp:77-184, pico-ps/test/TestOps.h:87-136,159-185",
            "ops": ops}


def pmem_three_pushes(num_keys=120):
    """pico-ps/test/ps_pmem_test.cpp:395-439: key 2k is pushed arg=k three times (async), dumped
    and loaded; pulling keys 0..NUM_KEYS-1 gives i odd ? 0 : i/2*3."""
    keys = [2 * k for k in range(num_keys)]
    grads = [[k, 1] for k in range(num_keys)]
    ops = [{"op": "push", "keys": keys, "grads": grads} for _ in range(3)]
    ops.append({"op": "dump_load_roundtrip", "expect_size": num_keys})
    pull_keys = list(range(num_keys))
    rows = [[0, 0] if i % 2 else [i // 2 * 3, 3] for i in pull_keys]
    ops.append({"op": "expect_pull", "keys": pull_keys, "rows": rows,
                "hit": [0 if i % 2 else 1 for i in pull_keys]})
    return {"name": "pmem_three_pushes", "dim": 2, "optimizer": "SUM",
            "cite": "pico-ps/test/ps_pmem_test.cpp:395-439", "ops": ops}


def native_ps_roundtrip(num_process=2, per_rank=150):
    """pico-ps/test/ps_predictor_native_ps_test.cpp:108-170: each key is pushed once with the value
    (key+1, key+2), dumped, loaded through the in-process path; the pulled value is key+2.
    (The reference uses 1000 keys per rank; the fixture keeps the stride and fewer keys.)"""
    ops = []
    keys = []
    for rank in range(num_process):
        ks = list(range(rank * 1000, rank * 1000 + per_rank))
        keys += ks
        ops.append({"op": "push", "keys": ks, "grads": [[k + 1, k + 2] for k in ks]})
    ops.append({"op": "dump_load_roundtrip", "expect_size": len(keys)})
    for _ in range(2):
        ops.append({"op": "expect_pull", "keys": keys, "rows": [[k + 1, k + 2] for k in keys],
                    "hit": [1] * len(keys)})
    return {"name": "native_ps_roundtrip", "dim": 2, "optimizer": "SUM",
            "cite": "pico-ps/test/ps_predictor_native_ps_test.cpp:108-170", "ops": ops}


def ha_load_pull(num_keys=2500):
    """pico-ps/test/ps_ha_loader_puller_test.cpp:86-183: keys 0 .. N-1 are pushed once with the value
    (key+1, key+2) in one batch, dumped, loaded into a new storage (LoadOperator::restore: every key
    must be new) and pulled repeatedly; every pull answers key+2 in the value's second field.
    (The reference uses 10000 keys and five pulls; the fixture keeps the key range dense from 0 and
    the single push, with fewer keys and two pulls.)"""
    keys = list(range(num_keys))
    ops = [{"op": "push", "keys": keys, "grads": [[k + 1, k + 2] for k in keys]},
           {"op": "expect_size", "value": num_keys},
           {"op": "dump_load_roundtrip", "expect_size": num_keys}]
    for _ in range(2):
        ops.append({"op": "expect_pull", "keys": keys, "rows": [[k + 1, k + 2] for k in keys],
                    "hit": [1] * num_keys})
    return {"name": "ha_load_pull", "dim": 2, "optimizer": "SUM",
            "cite": "pico-ps/test/ps_ha_loader_puller_test.cpp:86-183", "ops": ops}


def hash_map_contract():
    """pico-ps/test/ps_pmem_test.cpp:110-157: the map contract the operators use (lock_find,
    safe_insert, safe_set, safe_erase; storage/KVShardStorage.h:786-834) on int -> int. The test's
    `it->second = 3` through an accessor and its safe_set calls are upserts here; its second
    safe_insert of key 0, which must leave the stored 2 alone, is a pull of key 0."""
    def pull(keys, vals):
        return {"op": "expect_pull", "keys": keys, "rows": [[v if v is not None else 0] for v in vals],
                "hit": [int(v is not None) for v in vals]}
    ops = [{"op": "set", "keys": [0], "values": [[2]]},           # safe_insert(mp, 0, 2)
           pull([0, 1], [2, None]),                               # the value stays 2; key 1 is absent
           {"op": "set", "keys": [0], "values": [[3]]},           # it->second = 3
           {"op": "set", "keys": [1], "values": [[4]]},
           {"op": "set", "keys": [2], "values": [[5]]},
           {"op": "set", "keys": [3], "values": [[6]]},
           {"op": "set", "keys": [4], "values": [[7]]},
           pull([5], [None]),
           {"op": "expect_values", "values": [3, 4, 5, 6, 7]},
           {"op": "set", "keys": [3], "values": [[6666]]},
           pull([3], [6666]),
           {"op": "erase", "keys": [3], "erased": 1},
           pull([3], [None]),
           {"op": "expect_values", "values": [3, 4, 5, 7]},
           {"op": "expect_size", "value": 4}]
    return {"name": "hash_map_contract", "dim": 1, "optimizer": "SUM",
            "cite": "pico-ps/test/ps_pmem_test.cpp:110-157", "ops": ops}


def concurrent_erase():
    """pico-ps/test/ps_pmem_test.cpp:159-193: ten rounds of: insert keys 0..99 with value = key,
    size 100, ten erasers take the overlapping ranges [10 i, 10 i + 20) -- every key from 10 on is
    erased twice, keys 100..109 were never there --, afterwards no key is found and the size is 0.
    The ten ranges arrive as one batch (the reference's threads race; the outcome is the same)."""
    ops = []
    keys = list(range(100))
    ranges = [k for i in range(10) for k in range(10 * i, 10 * i + 20)]
    for _ in range(10):
        ops.append({"op": "set", "keys": keys, "values": [[k] for k in keys]})
        ops.append({"op": "expect_size", "value": 100})
        ops.append({"op": "erase", "keys": ranges, "erased": 100})
        ops.append({"op": "expect_pull", "keys": keys, "rows": [[0]] * 100, "hit": [0] * 100})
        ops.append({"op": "expect_size", "value": 0})
    return {"name": "concurrent_erase", "dim": 1, "optimizer": "SUM",
            "cite": "pico-ps/test/ps_pmem_test.cpp:159-193", "ops": ops}


DENSE_BLOCK_SIZE = 5  # pico-ps/test/TestOps.h:270


def test_dense(num_process=3, per_rank=3):
    """pico-ps/test/ps_service_test.cpp:241-409 (test_dense). The dense parameter of key k is the
    vector {k, k+1, ..., 2k-1} (:262-266), cut into slices of DENSE_BLOCK_SIZE (TestValuePartitioner,
    TestOps.h:307-319); the test operator adds what is pushed (TestOps.h:351-377). A slice
    {id, slice_id} (pico-ps/common/dense_common.h:67-104) is the table row of key id << 24 | slice_id,
    the last slice of a parameter padded with zeros. (The reference uses 100 keys per rank; the
    fixture keeps the stride of 100 and the first `per_rank` keys of every rank.)"""
    def slices(k):
        arg = [k + i for i in range(k)]
        out = []
        for s in range(0, k, DENSE_BLOCK_SIZE):
            part = arg[s:s + DENSE_BLOCK_SIZE]
            out.append(((k << 24) | (s // DENSE_BLOCK_SIZE), part + [0] * (DENSE_BLOCK_SIZE - len(part))))
        return out

    ranks = []
    for rank in range(num_process):
        items = [it for k in range(rank * TEST_KEY_NUM, rank * TEST_KEY_NUM + per_rank) for it in slices(k)]
        ranks.append(([it[0] for it in items], [it[1] for it in items]))
    ops = []
    for keys, grads in ranks:                                             # :259-272
        ops.append({"op": "push", "keys": keys, "grads": grads})
        ops.append({"op": "queue", "keys": keys, "grads": grads})
    ops.append({"op": "store"})                                           # :274-277
    for rank, (keys, grads) in enumerate(ranks):                          # :280-291
        if rank % 2 == 0:
            ops.append({"op": "queue", "keys": keys, "grads": grads})
    ops.append({"op": "store"})                                           # :296-298
    for rank, (keys, grads) in enumerate(ranks):                          # :307-326
        ops.append({"op": "push", "keys": keys, "grads": grads})
        ops.append({"op": "queue", "keys": keys, "grads": grads})
        if rank % 2 == 0:
            ops.append({"op": "queue", "keys": keys, "grads": grads})

    def expect(factor):
        keys, rows = [], []
        for rank, (ks, gs) in enumerate(ranks):
            keys += ks
            rows += [[v * factor(rank) for v in g] for g in gs]
        return {"op": "expect_pull", "keys": keys, "rows": rows, "hit": [1] * len(keys)}

    ops.append(expect(lambda rank: 3 + (rank % 2 == 0)))                  # :332-347: queued pushes not applied yet
    ops.append({"op": "store"})                                           # :356-357
    n_slices = sum(len(ks) for ks, _ in ranks)
    ops.append({"op": "dump_load_roundtrip", "expect_size": n_slices})   # :359-390
    for _ in range(2):
        ops.append(expect(lambda rank: (2 + (rank % 2 == 0)) * 2))       # :393-409
    return {"name": f"test_dense_{num_process}", "dim": DENSE_BLOCK_SIZE, "optimizer": "SUM",
            "cite": "pico-ps/test/ps_service_test.cpp:241-409, pico-ps/test/TestOps.h:270-399", "ops": ops}


def main():
    scenarios = [test_sparse(1), test_sparse(3), pmem_three_pushes(), native_ps_roundtrip(), ha_load_pull(),
                 hash_map_contract(), concurrent_erase(), test_dense()]
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_known_answers.json")
    with open(out, "w") as f:
        json.dump({"scenarios": scenarios}, f, separators=(",", ":"))
    print(out, os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()
