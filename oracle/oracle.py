"""ctypes front end of the CPU oracle (oracle/libps_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by bench.py's
cpu_baseline leg. The product library never loads it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libps_oracle.so")

OK, INVALID_CONFIG, OUT_OF_MEMORY, ERROR = 0, 1, 3, 10
OPT_SUM, OPT_SGD, OPT_ADAGRAD, OPT_FTRL, OPT_USER = 0, 1, 2, 3, 4
PULL_INSERT_ON_MISS = 1
PUSH_NO_INSERT = 1
PUSH_EXACT_AGGREGATION = 0x100  # oracle only: float64 sums, rounded once
LOAD_UNIQUE = 1


class _Config(C.Structure):
    _fields_ = [
        ("dim", C.c_uint32),
        ("optimizer", C.c_int32),
        ("lr", C.c_float),
        ("init_acc", C.c_float),
        ("alpha", C.c_float),
        ("beta", C.c_float),
        ("l1", C.c_float),
        ("l2", C.c_float),
        ("capacity", C.c_uint64),
        ("read_only", C.c_int32),
        ("track_increment", C.c_int32),
        ("init_range", C.c_float),
    ]


COL_KEY = -1
CMP_LT, CMP_LE, CMP_GT, CMP_GE, CMP_EQ, CMP_NE, CMP_MOD_EQ, CMP_PART_EQ, CMP_PART_NE = range(9)


class _Term(C.Structure):
    _fields_ = [("column", C.c_int32), ("cmp", C.c_int32), ("f", C.c_float), ("reserved", C.c_uint32),
                ("u", C.c_uint64), ("u2", C.c_uint64)]


class Predicate(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("n_terms", C.c_uint32), ("term", _Term * 4)]


def predicate(*terms):
    """The same constructor as the product binding's: (column, cmp, operand) terms."""
    p = Predicate()
    p.struct_size = C.sizeof(Predicate)
    p.n_terms = len(terms)
    for i, (col, cmp_, operand) in enumerate(terms):
        p.term[i].column, p.term[i].cmp = col, cmp_
        if col == COL_KEY:
            if cmp_ in (CMP_MOD_EQ, CMP_PART_EQ, CMP_PART_NE):
                p.term[i].u, p.term[i].u2 = operand
            else:
                p.term[i].u = operand
        else:
            p.term[i].f = operand
    return p


UPD_AFFINE, UPD_CLAMP = 0, 1


class Update(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("op", C.c_int32), ("first_column", C.c_uint32),
                ("n_columns", C.c_uint32), ("a", C.c_float), ("b", C.c_float)]


def update(op, first_column, n_columns, a, b):
    return Update(C.sizeof(Update), op, first_column, n_columns, a, b)


def build():
    """Compiles the oracle with g++ (a few seconds)."""
    subprocess.run(["make", "-C", _HERE, "-B", "libps_oracle.so"], check=True, capture_output=True)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        vp, u64p, f32p, u8p = C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p
        L.pso_value_floats.restype = C.c_uint32
        L.pso_value_floats.argtypes = [C.c_uint32, C.c_int32]
        L.pso_create.argtypes = [C.POINTER(_Config), C.POINTER(vp)]
        L.pso_partition.restype = C.c_int32
        L.pso_partition.argtypes = [C.c_uint64, C.c_int32]
        L.pso_init_weight.restype = C.c_float
        L.pso_init_weight.argtypes = [C.c_float, C.c_uint64, C.c_uint32]
        L.pso_destroy.argtypes = [vp]
        L.pso_pull.argtypes = [vp, u64p, C.c_size_t, f32p, u8p, C.c_uint32]
        L.pso_aggregate.argtypes = [C.c_uint32, u64p, f32p, C.c_size_t, u64p, f32p,
                                    C.POINTER(C.c_size_t)]
        L.pso_push.argtypes = [vp, u64p, f32p, C.c_size_t, C.c_uint32]
        L.pso_queue.argtypes = [vp, u64p, f32p, C.c_size_t]
        L.pso_queued.argtypes = [vp, C.POINTER(C.c_uint64)]
        L.pso_store.argtypes = [vp, C.c_uint32]
        L.pso_set.argtypes = [vp, u64p, f32p, C.c_size_t]
        L.pso_load.argtypes = [vp, vp, C.c_size_t, C.c_uint32]
        L.pso_iterate.argtypes = [vp, C.c_size_t, C.c_size_t, vp, C.POINTER(C.c_size_t)]
        L.pso_dump.argtypes = [vp, vp, C.c_size_t, C.POINTER(C.c_size_t)]
        L.pso_for_each.argtypes = [vp, vp, C.POINTER(C.c_uint64), vp]
        L.pso_for_each_write.argtypes = [vp, vp, vp, C.POINTER(C.c_uint64)]
        L.pso_erase_if.argtypes = [vp, vp, C.POINTER(C.c_uint64)]
        L.pso_erase.argtypes = [vp, vp, C.c_size_t, C.POINTER(C.c_uint64)]
        L.pso_reserve.argtypes = [vp, C.c_uint64]
        L.pso_set_hyperparameters.argtypes = [vp] + [C.c_float] * 6
        L.pso_increment_size.argtypes = [vp, C.POINTER(C.c_uint64)]
        L.pso_take_increment.argtypes = [vp, vp, C.c_size_t, C.POINTER(C.c_size_t)]
        L.pso_clear.argtypes = [vp]
        L.pso_size.argtypes = [vp, C.POINTER(C.c_uint64)]
        _lib = L
    return _lib


def _keys(a):
    a = np.ascontiguousarray(a, dtype=np.uint64)
    return a, a.ctypes.data


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data


def record_dtype(value_floats):
    """Layout of one Load/Dump record: uint64 key then the value's floats, packed."""
    return np.dtype([("key", "<u8"), ("value", "<f4", (value_floats,))])


def init_weight(init_range, key, column):
    """Weight `column` of a new key of a table that draws initial weights in [-init_range, init_range)."""
    return lib().pso_init_weight(init_range, key, column)


def partition(key, n):
    """Partition of `key` among n (DefaultPartitioner<uint64_t>'s shape with the published functions)."""
    return lib().pso_partition(key, n)


class Oracle:
    """One shard of the reference's KV storage with the operator loops on top (CPU, scalar)."""

    def __init__(self, dim, optimizer=OPT_SUM, lr=0.0, init_acc=0.0, alpha=0.0, beta=0.0, l1=0.0,
                 l2=0.0, capacity=1 << 20, read_only=False, track_increment=False, init_range=0.0):
        self.dim = dim
        self.optimizer = optimizer
        self.value_floats = lib().pso_value_floats(dim, optimizer)
        cfg = _Config(dim, optimizer, lr, init_acc, alpha, beta, l1, l2, capacity, int(read_only),
                      int(track_increment), init_range)
        self._h = C.c_void_p()
        st = lib().pso_create(C.byref(cfg), C.byref(self._h))
        if st != OK:
            raise ValueError(f"pso_create failed with status {st}")

    def close(self):
        if self._h:
            lib().pso_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def pull(self, keys, flags=0):
        k, kp = _keys(keys)
        out = np.empty((k.size, self.dim), dtype=np.float32)
        hit = np.empty(k.size, dtype=np.uint8)
        st = lib().pso_pull(self._h, kp, k.size, out.ctypes.data, hit.ctypes.data, flags)
        return st, out, hit

    def push(self, keys, grads, flags=0):
        k, kp = _keys(keys)
        g, gp = _f32(grads)
        assert g.size == k.size * self.dim
        return lib().pso_push(self._h, kp, gp, k.size, flags)

    def queue(self, keys, grads):
        k, kp = _keys(keys)
        g, gp = _f32(grads)
        assert g.size == k.size * self.dim
        return lib().pso_queue(self._h, kp, gp, k.size)

    def queued(self):
        n = C.c_uint64()
        lib().pso_queued(self._h, C.byref(n))
        return n.value

    def store(self, flags=0):
        return lib().pso_store(self._h, flags)

    def set(self, keys, values):
        k, kp = _keys(keys)
        v, vp = _f32(values)
        assert v.size == k.size * self.value_floats
        return lib().pso_set(self._h, kp, vp, k.size)

    def load(self, records, flags=0):
        r = np.ascontiguousarray(records, dtype=record_dtype(self.value_floats))
        return lib().pso_load(self._h, r.ctypes.data, r.size, flags)

    def dump(self):
        n = self.size()
        rec = np.empty(n, dtype=record_dtype(self.value_floats))
        got = C.c_size_t()
        st = lib().pso_dump(self._h, rec.ctypes.data, n, C.byref(got))
        return st, rec[: got.value]

    def iterate(self, offset, batch):
        rec = np.empty(batch, dtype=record_dtype(self.value_floats))
        got = C.c_size_t()
        st = lib().pso_iterate(self._h, offset, batch, rec.ctypes.data, C.byref(got))
        return st, rec[: got.value]

    def increment_size(self):
        n = C.c_uint64()
        lib().pso_increment_size(self._h, C.byref(n))
        return OK, n.value

    def take_increment(self, capacity=None):
        if capacity is None:
            capacity = self.increment_size()[1]
        rec = np.empty(max(capacity, 1), dtype=record_dtype(self.value_floats))
        got = C.c_size_t()
        st = lib().pso_take_increment(self._h, rec.ctypes.data, capacity, C.byref(got))
        return st, rec[: got.value if st == OK else 0]

    def for_each(self, where=None):
        n = C.c_uint64()
        sums = np.zeros(self.value_floats, dtype=np.float64)
        st = lib().pso_for_each(self._h, C.byref(where) if where is not None else None, C.byref(n),
                                sums.ctypes.data)
        return st, n.value, sums

    def for_each_write(self, what, where=None):
        n = C.c_uint64()
        st = lib().pso_for_each_write(self._h, C.byref(where) if where is not None else None,
                                      C.byref(what), C.byref(n))
        return st, n.value

    def erase_if(self, where=None):
        n = C.c_uint64()
        st = lib().pso_erase_if(self._h, C.byref(where) if where is not None else None, C.byref(n))
        return st, n.value

    def erase(self, keys):
        k, kp = _keys(keys)
        n = C.c_uint64()
        st = lib().pso_erase(self._h, kp, k.size, C.byref(n))
        return st, n.value

    def compact(self):
        return OK

    def set_hyperparameters(self, lr=0.0, init_acc=0.0, alpha=0.0, beta=0.0, l1=0.0, l2=0.0):
        return lib().pso_set_hyperparameters(self._h, lr, init_acc, alpha, beta, l1, l2)

    def reserve(self, capacity):
        return lib().pso_reserve(self._h, capacity)

    def clear(self):
        return lib().pso_clear(self._h)

    def size(self):
        n = C.c_uint64()
        lib().pso_size(self._h, C.byref(n))
        return n.value


def aggregate(dim, keys, grads):
    """Duplicate aggregation alone; returns (unique keys in first-occurrence order, sums)."""
    k, kp = _keys(keys)
    g, gp = _f32(grads)
    uk = np.empty(k.size, dtype=np.uint64)
    us = np.empty((k.size, dim), dtype=np.float32)
    nu = C.c_size_t()
    lib().pso_aggregate(dim, kp, gp, k.size, uk.ctypes.data, us.ctypes.data, C.byref(nu))
    return uk[: nu.value], us[: nu.value]
