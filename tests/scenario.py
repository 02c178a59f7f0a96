"""Runs a golden scenario (tests/golden/reference_known_answers.json) against a backend.

A backend is anything with the method set shared by oracle.Oracle and the product's Table:
pull / push / queue / store / set / erase / dump / load / for_each / erase_if / clear / size. `make` builds a fresh backend of the
scenario's shape (used for the dump -> load round trip into a new storage).
"""
import json
import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                      "reference_known_answers.json")
OPT = {"SUM": 0, "SGD": 1, "ADAGRAD": 2, "FTRL": 3}


def load_scenarios():
    with open(GOLDEN) as f:
        return json.load(f)["scenarios"]


def _where(predicate, terms):
    """[[column, cmp, operand], ...] of the fixture -> predicate object (None = every record)"""
    if not terms:
        return None
    return predicate(*[(c, m, tuple(o) if isinstance(o, list) else o) for c, m, o in terms])


def run(scn, make, predicate):
    """make(dim, optimizer) -> backend; predicate(*terms) -> the backend's predicate object.
    Asserts every expectation of the scenario."""
    dim, opt = scn["dim"], OPT[scn["optimizer"]]
    b = make(dim, opt)
    for step, op in enumerate(scn["ops"]):
        where = f"{scn['name']} step {step} ({op['op']})"
        kind = op["op"]
        if kind == "push":
            assert b.push(np.array(op["keys"], dtype=np.uint64),
                          np.array(op["grads"], dtype=np.float32)) == 0, where
        elif kind == "queue":
            assert b.queue(np.array(op["keys"], dtype=np.uint64),
                           np.array(op["grads"], dtype=np.float32)) == 0, where
        elif kind == "store":
            assert b.store() == 0, where
            assert b.queued() == 0, where
        elif kind == "set":
            assert b.set(np.array(op["keys"], dtype=np.uint64),
                         np.array(op["values"], dtype=np.float32)) == 0, where
        elif kind == "erase":
            st, erased = b.erase(np.array(op["keys"], dtype=np.uint64))
            assert st == 0 and erased == op["erased"], where
        elif kind == "expect_values":
            # every stored value, in ascending order (the reference walks the map and sorts)
            st, rec = b.dump()
            assert st == 0, where
            np.testing.assert_array_equal(np.sort(rec["value"][:, 0]),
                                          np.array(op["values"], dtype=np.float32), err_msg=where)
        elif kind == "expect_size":
            assert b.size() == op["value"], where
        elif kind == "clear":
            assert b.clear() == 0, where
        elif kind == "expect_pull":
            st, rows, hit = b.pull(np.array(op["keys"], dtype=np.uint64))
            assert st == 0, where
            np.testing.assert_array_equal(rows, np.array(op["rows"], dtype=np.float32), err_msg=where)
            np.testing.assert_array_equal(hit, np.array(op["hit"], dtype=np.uint8), err_msg=where)
        elif kind == "expect_for_each":
            st, count, sums = b.for_each(_where(predicate, op["where"]))
            assert st == 0 and count == op["count"], where
            np.testing.assert_array_equal(sums, np.array(op["sums"], dtype=np.float64), err_msg=where)
        elif kind == "erase_if":
            st, erased = b.erase_if(_where(predicate, op["where"]))
            assert st == 0 and erased == op["erased"], where
        elif kind == "dump_load_roundtrip":
            # dump, load into a new storage; then clear that one and restore it (unique load)
            st, rec = b.dump()
            assert st == 0 and rec.size == op["expect_size"], where
            assert np.unique(rec["key"]).size == rec.size, where
            b2 = make(dim, opt)
            assert b2.load(rec) == 0, where
            assert b2.size() == op["expect_size"], where
            assert b2.clear() == 0 and b2.size() == 0, where
            assert b2.load(rec, 1) == 0, where  # restore: keys must be new
            assert b2.size() == op["expect_size"], where
            b.close()
            b = b2
        else:
            raise AssertionError(f"unknown op {kind}")
    b.close()
