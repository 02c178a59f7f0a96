"""ctypes binding of libpshbm.so, the HBM-resident sparse table behind the Pull / Push / Load /
Dump operators of one pico-ps server shard.

The directory name contains a hyphen, so load it with
``importlib.import_module("parameter-server_amd")``.

There is no CPU fallback: if the library has not been built, or no HIP device answers, the calls
raise.
"""
import ctypes as C
import os
import subprocess
import weakref

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libpshbm.so")
CSRC = os.path.join(_HERE, "csrc")

OK, INVALID_CONFIG, INVALID_ID, OUT_OF_MEMORY, ERROR, FATAL = 0, 1, 2, 3, 10, 11
OPT_SUM, OPT_SGD, OPT_ADAGRAD, OPT_FTRL, OPT_USER = 0, 1, 2, 3, 4
PULL_INSERT_ON_MISS = 1
PUSH_NO_INSERT = 1
PUSH_ASSUME_UNIQUE = 2
PUSH_VERIFY_HANDLES = 4
LOAD_UNIQUE = 1

# every symbol include/pshbm.h declares
SYMBOLS = [
    "pshbm_create", "pshbm_destroy", "pshbm_last_error", "pshbm_value_floats", "pshbm_init_weight",
    "pshbm_pull", "pshbm_pull_dev", "pshbm_push", "pshbm_push_dev", "pshbm_push_pairs",
    "pshbm_queue", "pshbm_queue_dev", "pshbm_queue_pairs", "pshbm_queued", "pshbm_store", "pshbm_store_dev",
    "pshbm_set", "pshbm_set_dev", "pshbm_load", "pshbm_dump", "pshbm_iterate", "pshbm_iterate_keys",
    "pshbm_increment_size", "pshbm_take_increment", "pshbm_for_each", "pshbm_for_each_write", "pshbm_erase_if", "pshbm_erase", "pshbm_erase_dev", "pshbm_compact", "pshbm_reserve", "pshbm_set_hyperparameters", "pshbm_set_memory_limit", "pshbm_device_memory",
    "pshbm_clear", "pshbm_size", "pshbm_memory_usage", "pshbm_get_stats",
    "pshbm_host_alloc", "pshbm_host_free", "pshbm_profile_enable", "pshbm_profile_read",
    "pshbm_push_dev_noalloc", "pshbm_pull_dev_handles", "pshbm_push_dev_handles", "pshbm_debug_sort_spin_limit", "pshbm_debug_part_pass_capacity", "pshbm_debug_part_min_keys",
    "pshbm_debug_tombstone_limit", "pshbm_debug_sort_pairs", "pshbm_debug_part_order", "pshbm_partition",
]
PHASES = ["pull", "locate", "sort_hist", "segreduce", "fixup", "update_unique", "gather", "sort_pass",
          "fixup_windows", "assign_rows", "push_small", "part_tile", "part_apply", "part_insert"]


class Config(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("device", C.c_int32),
        ("dim", C.c_uint32),
        ("optimizer", C.c_int32),
        ("lr", C.c_float),
        ("init_acc", C.c_float),
        ("alpha", C.c_float),
        ("beta", C.c_float),
        ("l1", C.c_float),
        ("l2", C.c_float),
        ("expected_max_items", C.c_uint64),
        ("max_load_factor", C.c_float),
        ("read_only", C.c_int32),
        ("max_batch", C.c_uint64),
        ("track_increment", C.c_int32),
        ("init_range", C.c_float),
    ]


class Hyperparameters(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("lr", C.c_float),
        ("init_acc", C.c_float),
        ("alpha", C.c_float),
        ("beta", C.c_float),
        ("l1", C.c_float),
        ("l2", C.c_float),
    ]


class Stats(C.Structure):
    _fields_ = [
        ("size", C.c_uint64),
        ("capacity", C.c_uint64),
        ("slots", C.c_uint64),
        ("memory_usage", C.c_uint64),
        ("load_factor", C.c_double),
        ("probe_hist", C.c_uint64 * 16),
        ("max_probe", C.c_uint64),
    ]


COL_KEY = -1
CMP_LT, CMP_LE, CMP_GT, CMP_GE, CMP_EQ, CMP_NE, CMP_MOD_EQ, CMP_PART_EQ, CMP_PART_NE = range(9)


class Term(C.Structure):
    _fields_ = [("column", C.c_int32), ("cmp", C.c_int32), ("f", C.c_float), ("reserved", C.c_uint32),
                ("u", C.c_uint64), ("u2", C.c_uint64)]


class Predicate(C.Structure):
    """pshbm_predicate: up to four terms that must all hold."""
    _fields_ = [("struct_size", C.c_uint32), ("n_terms", C.c_uint32), ("term", Term * 4)]


def predicate(*terms):
    """predicate((column, cmp, operand), ...): column COL_KEY compares the key with an integer
    operand -- (COL_KEY, CMP_MOD_EQ, (modulus, remainder)) for key % modulus == remainder,
    (COL_KEY, CMP_PART_EQ / CMP_PART_NE, (partitions, partition)) for the key's partition --,
    any other column compares that value column with a float."""
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
    """pshbm_update: what a writing for-each does to columns [first_column, first_column + n_columns)."""
    _fields_ = [("struct_size", C.c_uint32), ("op", C.c_int32), ("first_column", C.c_uint32),
                ("n_columns", C.c_uint32), ("a", C.c_float), ("b", C.c_float)]


def update(op, first_column, n_columns, a, b):
    return Update(C.sizeof(Update), op, first_column, n_columns, a, b)


class Profile(C.Structure):
    _fields_ = [("ms", C.c_double * len(PHASES)), ("launches", C.c_uint64 * len(PHASES))]


class PshbmError(RuntimeError):
    def __init__(self, status, message):
        super().__init__(f"pshbm status {status}: {message}")
        self.status = status


def build(verbose=False):
    """Compiles the HIP sources for gfx950 into libpshbm.so (hipcc; works without a GPU)."""
    r = subprocess.run(["make", "-C", CSRC, "-B", "-j4"], capture_output=True, text=True)
    if verbose or r.returncode != 0:
        print(r.stdout[-4000:])
        print(r.stderr[-4000:])
    if r.returncode != 0:
        raise RuntimeError("building libpshbm.so failed")


_lib = None


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(
                f"{LIB_PATH} is missing: build it with __graft_entry__.build() "
                f"(make -C {CSRC}); there is no CPU fallback")
        # PyTorch wheels bundle their own HIP runtime under the same SONAME. A process must hold
        # one runtime only (streams and device pointers are handed between torch and this
        # library), and whichever loads first wins: let torch load first when it is installed.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        L = C.CDLL(LIB_PATH)
        vp, sz, u32, i32 = C.c_void_p, C.c_size_t, C.c_uint32, C.c_int32
        L.pshbm_create.argtypes = [C.POINTER(Config), C.POINTER(vp)]
        L.pshbm_destroy.argtypes = [vp]
        L.pshbm_last_error.argtypes = [vp]
        L.pshbm_last_error.restype = C.c_char_p
        L.pshbm_value_floats.argtypes = [u32, i32]
        L.pshbm_value_floats.restype = u32
        L.pshbm_init_weight.argtypes = [C.c_float, C.c_uint64, u32]
        L.pshbm_init_weight.restype = C.c_float
        L.pshbm_pull.argtypes = [vp, vp, sz, vp, vp, u32]
        L.pshbm_pull_dev.argtypes = [vp, vp, sz, vp, vp, u32, vp]
        L.pshbm_push.argtypes = [vp, vp, vp, sz, u32]
        L.pshbm_push_dev.argtypes = [vp, vp, vp, sz, u32, vp]
        L.pshbm_push_dev_noalloc.argtypes = [vp, vp, vp, sz, u32, vp]
        L.pshbm_pull_dev_handles.argtypes = [vp, vp, sz, vp, vp, vp, C.POINTER(C.c_uint64), u32, vp]
        L.pshbm_push_dev_handles.argtypes = [vp, vp, vp, vp, C.c_uint64, sz, u32, vp]
        L.pshbm_debug_sort_spin_limit.argtypes = [u32]
        L.pshbm_debug_part_pass_capacity.argtypes = [u32]
        L.pshbm_debug_part_min_keys.argtypes = [C.c_uint64]
        L.pshbm_partition.argtypes = [C.c_uint64, C.c_int32]
        L.pshbm_partition.restype = C.c_int32
        L.pshbm_debug_sort_pairs.argtypes = [C.c_int32, vp, vp, vp, vp, sz, u32, C.POINTER(C.c_int32), vp]
        L.pshbm_debug_part_order.argtypes = [vp, vp, sz, C.POINTER(sz), C.POINTER(u32)]
        L.pshbm_debug_tombstone_limit.argtypes = [C.c_uint64, C.c_uint64]
        L.pshbm_debug_tombstone_limit.restype = C.c_uint64
        L.pshbm_push_pairs.argtypes = [vp, vp, sz, sz, u32]
        L.pshbm_queue.argtypes = [vp, vp, vp, sz]
        L.pshbm_queue_dev.argtypes = [vp, vp, vp, sz, vp]
        L.pshbm_queue_pairs.argtypes = [vp, vp, sz, sz]
        L.pshbm_queued.argtypes = [vp, C.POINTER(C.c_uint64)]
        L.pshbm_store.argtypes = [vp, u32]
        L.pshbm_store_dev.argtypes = [vp, u32, vp]
        L.pshbm_set.argtypes = [vp, vp, vp, sz]
        L.pshbm_set_dev.argtypes = [vp, vp, vp, sz, vp]
        L.pshbm_load.argtypes = [vp, vp, sz, u32]
        L.pshbm_dump.argtypes = [vp, vp, sz, C.POINTER(sz)]
        L.pshbm_iterate.argtypes = [vp, sz, sz, vp, C.POINTER(sz)]
        L.pshbm_for_each.argtypes = [vp, vp, C.POINTER(C.c_uint64), vp]
        L.pshbm_for_each_write.argtypes = [vp, vp, vp, C.POINTER(C.c_uint64)]
        L.pshbm_erase_if.argtypes = [vp, vp, C.POINTER(C.c_uint64)]
        L.pshbm_erase.argtypes = [vp, vp, sz, C.POINTER(C.c_uint64)]
        L.pshbm_erase_dev.argtypes = [vp, vp, sz, C.POINTER(C.c_uint64), vp]
        L.pshbm_compact.argtypes = [vp]
        L.pshbm_reserve.argtypes = [vp, C.c_uint64]
        L.pshbm_set_hyperparameters.argtypes = [vp, C.POINTER(Hyperparameters)]
        L.pshbm_increment_size.argtypes = [vp, C.POINTER(C.c_uint64)]
        L.pshbm_take_increment.argtypes = [vp, vp, sz, C.POINTER(sz)]
        L.pshbm_clear.argtypes = [vp]
        L.pshbm_size.argtypes = [vp, C.POINTER(C.c_uint64)]
        L.pshbm_memory_usage.argtypes = [vp, C.POINTER(C.c_uint64)]
        L.pshbm_get_stats.argtypes = [vp, C.POINTER(Stats)]
        L.pshbm_iterate_keys.argtypes = [vp, sz, sz, vp, C.POINTER(sz)]
        L.pshbm_set_memory_limit.argtypes = [i32, C.c_uint64]
        L.pshbm_device_memory.argtypes = [i32, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]
        L.pshbm_host_alloc.argtypes = [C.POINTER(vp), sz]
        L.pshbm_host_free.argtypes = [vp]
        L.pshbm_profile_enable.argtypes = [vp, i32]
        L.pshbm_profile_read.argtypes = [vp, C.POINTER(Profile)]
        for name in SYMBOLS:
            if getattr(L, name).restype is C.c_int:
                getattr(L, name).restype = i32
        _lib = L
    return _lib


def value_floats(dim, optimizer):
    return lib().pshbm_value_floats(dim, optimizer)


def set_memory_limit(device, nbytes):
    """Budget of device memory for everything the library allocates on `device` (0 = none)."""
    st = lib().pshbm_set_memory_limit(device, nbytes)
    if st != OK:
        raise PshbmError(st, "set_memory_limit: bad device")


def device_memory(device=0):
    """(bytes the library holds on the device, limit or 0)."""
    a, b = C.c_uint64(), C.c_uint64()
    st = lib().pshbm_device_memory(device, C.byref(a), C.byref(b))
    if st != OK:
        raise PshbmError(st, "device_memory: bad device")
    return a.value, b.value


def debug_sort_spin_limit(polls=0xFFFFFFFF):
    """Test hook: polls a sort tile grants its predecessors (default 2^24; 0 = give up at once)."""
    return lib().pshbm_debug_sort_spin_limit(polls)


def debug_part_pass_capacity(entries=0):
    """Test hook: entries one pass of the partitioned push's apply kernel takes (0 = default)."""
    return lib().pshbm_debug_part_pass_capacity(entries)


def debug_part_min_keys(keys=0):
    """Test hook: smallest batch that takes the partitioned push (0 = default); a large value sends
    mid-size batches through the sorted push."""
    return lib().pshbm_debug_part_min_keys(keys)


def partition(key, n_partitions):
    """Partition of a key among n_partitions: jump_consistent_hash(fmix64(key), n) (pshbm_partition)."""
    return lib().pshbm_partition(key, n_partitions)


def init_weight(init_range, key, column):
    """Weight `column` that a table with this init_range gives a new key (host side of the kernels' formula)."""
    return lib().pshbm_init_weight(init_range, key, column)


def record_dtype(vf):
    """Layout of one Load/Dump record: uint64 key then the value's floats, packed."""
    return np.dtype([("key", "<u8"), ("value", "<f4", (vf,))])


def pinned_empty(shape, dtype):
    """An uninitialised numpy array in page-locked host memory (pshbm_host_alloc), freed when the
    array and its views are gone. Load and Dump move such buffers without staging copies."""
    dtype = np.dtype(dtype)
    n = int(np.prod(shape)) if not np.isscalar(shape) else int(shape)
    nbytes = max(n * dtype.itemsize, 1)
    p = C.c_void_p()
    st = lib().pshbm_host_alloc(C.byref(p), nbytes)
    if st != OK:
        raise PshbmError(st, "pshbm_host_alloc failed")
    buf = (C.c_char * nbytes).from_address(p.value)
    weakref.finalize(buf, lib().pshbm_host_free, C.c_void_p(p.value))
    return np.frombuffer(buf, dtype=dtype, count=n).reshape(shape)


def _u64(a):
    return np.ascontiguousarray(a, dtype=np.uint64)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


class Table:
    """One shard's storage in HBM. Methods return the status code (and outputs); they raise only
    on misuse. Host-array methods are synchronous; the ``*_dev`` methods take raw device pointers
    and a hipStream_t value and enqueue."""

    def __init__(self, dim, optimizer=OPT_SUM, lr=0.0, init_acc=0.0, alpha=0.0, beta=0.0, l1=0.0,
                 l2=0.0, capacity=1 << 20, max_load_factor=0.0, read_only=False, max_batch=0,
                 device=0, track_increment=False, init_range=0.0):
        self.dim = dim
        self.optimizer = optimizer
        self._h = C.c_void_p()
        cfg = Config(C.sizeof(Config), device, dim, optimizer, lr, init_acc, alpha, beta, l1, l2,
                     capacity, max_load_factor, int(read_only), max_batch, int(track_increment), init_range)
        st = lib().pshbm_create(C.byref(cfg), C.byref(self._h))
        if st != OK:
            raise PshbmError(st, (lib().pshbm_last_error(None) or b"").decode())
        self.value_floats = value_floats(dim, optimizer)

    # -- lifetime
    def close(self):
        if self._h:
            lib().pshbm_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def last_error(self):
        return (lib().pshbm_last_error(self._h) or b"").decode()

    # -- host-array entry points
    def pull(self, keys, flags=0, out=None, hit=None):
        """(status, rows, hit mask). `out` / `hit`: arrays of the caller to fill; when they and the
        keys lie in page-locked memory (pinned_empty) a small pull uses them without a copy."""
        k = _u64(keys)
        if out is None:
            out = np.empty((k.size, self.dim), dtype=np.float32)
        if hit is None:
            hit = np.empty(k.size, dtype=np.uint8)
        if out.dtype != np.float32 or out.size != k.size * self.dim or not out.flags.c_contiguous or \
                hit.dtype != np.uint8 or hit.size != k.size or not hit.flags.c_contiguous:
            raise ValueError("out: contiguous float32 n x dim; hit: contiguous uint8 n")
        st = lib().pshbm_pull(self._h, k.ctypes.data, k.size, out.ctypes.data, hit.ctypes.data, flags)
        return st, out, hit

    def push(self, keys, grads, flags=0):
        k, g = _u64(keys), _f32(grads)
        assert g.size == k.size * self.dim
        return lib().pshbm_push(self._h, k.ctypes.data, g.ctypes.data, k.size, flags)

    def push_pairs(self, pairs, flags=0):
        """pairs: structured array {key u8, value f4[dim]} (the wire layout of a push block)."""
        p = np.ascontiguousarray(pairs)
        return lib().pshbm_push_pairs(self._h, p.ctypes.data, p.size, p.dtype.itemsize, flags)

    def queue(self, keys, grads):
        k, g = _u64(keys), _f32(grads)
        assert g.size == k.size * self.dim
        return lib().pshbm_queue(self._h, k.ctypes.data, g.ctypes.data, k.size)

    def queue_pairs(self, pairs):
        p = np.ascontiguousarray(pairs)
        return lib().pshbm_queue_pairs(self._h, p.ctypes.data, p.size, p.dtype.itemsize)

    def queued(self):
        n = C.c_uint64()
        lib().pshbm_queued(self._h, C.byref(n))
        return n.value

    def store(self, flags=0):
        return lib().pshbm_store(self._h, flags)

    def set(self, keys, values):
        k, v = _u64(keys), _f32(values)
        assert v.size == k.size * self.value_floats
        return lib().pshbm_set(self._h, k.ctypes.data, v.ctypes.data, k.size)

    def load(self, records, flags=0):
        r = np.ascontiguousarray(records, dtype=record_dtype(self.value_floats))
        return lib().pshbm_load(self._h, r.ctypes.data, r.size, flags)

    def dump(self, pinned=False, out=None):
        """(status, records). pinned=True returns them in page-locked memory, which the copy
        engine writes directly; `out` reuses a record array of the caller (page-locking a large
        buffer costs more than the dump itself)."""
        n = self.size()
        if out is not None:
            if out.dtype != record_dtype(self.value_floats) or out.size < n or not out.flags.c_contiguous:
                raise ValueError("out: a contiguous record array of at least size() records")
            rec = out
        else:
            rec = (pinned_empty if pinned else np.empty)(n, dtype=record_dtype(self.value_floats))
        got = C.c_size_t()
        st = lib().pshbm_dump(self._h, rec.ctypes.data, rec.size, C.byref(got))
        return st, rec[: got.value]

    def iterate(self, offset, batch):
        rec = np.empty(batch, dtype=record_dtype(self.value_floats))
        got = C.c_size_t()
        st = lib().pshbm_iterate(self._h, offset, batch, rec.ctypes.data, C.byref(got))
        return st, rec[: got.value]

    def iterate_keys(self, offset, batch):
        """(status, keys of records [offset, offset + batch)): the keys alone, in record order."""
        keys = np.empty(batch, dtype=np.uint64)
        got = C.c_size_t()
        st = lib().pshbm_iterate_keys(self._h, offset, batch, keys.ctypes.data, C.byref(got))
        return st, keys[: got.value]

    def increment_size(self):
        n = C.c_uint64()
        st = lib().pshbm_increment_size(self._h, C.byref(n))
        return st, n.value

    def take_increment(self, capacity=None):
        """(status, records of the keys pushes touched since the last take)."""
        if capacity is None:
            st, capacity = self.increment_size()
            if st != OK:
                return st, np.empty(0, dtype=record_dtype(self.value_floats))
        rec = np.empty(max(capacity, 1), dtype=record_dtype(self.value_floats))
        got = C.c_size_t()
        st = lib().pshbm_take_increment(self._h, rec.ctypes.data, capacity, C.byref(got))
        return st, rec[: got.value if st == OK else 0]

    def for_each(self, where=None):
        """(status, count, column sums) over the records that satisfy `where` (a Predicate)."""
        n = C.c_uint64()
        sums = np.zeros(self.value_floats, dtype=np.float64)
        st = lib().pshbm_for_each(self._h, C.byref(where) if where is not None else None, C.byref(n),
                                  sums.ctypes.data)
        return st, n.value, sums

    def for_each_write(self, what, where=None):
        """(status, records rewritten): columns rewritten by `what` (an Update) where `where` holds."""
        n = C.c_uint64()
        st = lib().pshbm_for_each_write(self._h, C.byref(where) if where is not None else None,
                                        C.byref(what), C.byref(n))
        return st, n.value

    def erase_if(self, where=None):
        n = C.c_uint64()
        st = lib().pshbm_erase_if(self._h, C.byref(where) if where is not None else None, C.byref(n))
        return st, n.value

    def erase(self, keys):
        k = _u64(keys)
        n = C.c_uint64()
        st = lib().pshbm_erase(self._h, k.ctypes.data, k.size, C.byref(n))
        return st, n.value

    def erase_dev(self, d_keys, n, stream=0):
        got = C.c_uint64()
        st = lib().pshbm_erase_dev(self._h, d_keys, n, C.byref(got), stream)
        return st, got.value

    def compact(self):
        return lib().pshbm_compact(self._h)

    def set_hyperparameters(self, lr=0.0, init_acc=0.0, alpha=0.0, beta=0.0, l1=0.0, l2=0.0):
        """The optimizer's hyperparameters for the pushes and stores that follow; status."""
        hp = Hyperparameters(C.sizeof(Hyperparameters), lr, init_acc, alpha, beta, l1, l2)
        return lib().pshbm_set_hyperparameters(self._h, C.byref(hp))

    def reserve(self, capacity):
        """Grows the table to hold `capacity` keys; status."""
        return lib().pshbm_reserve(self._h, capacity)

    def clear(self):
        return lib().pshbm_clear(self._h)

    def size(self):
        n = C.c_uint64()
        st = lib().pshbm_size(self._h, C.byref(n))
        if st != OK:
            raise PshbmError(st, self.last_error())
        return n.value

    def memory_usage(self):
        n = C.c_uint64()
        lib().pshbm_memory_usage(self._h, C.byref(n))
        return n.value

    def debug_part_order(self):
        """(work items the last inserting push of 1024 partitions or more left for the next one, the
        number of partitions they are for): pshbm_debug_part_order; (empty array, 0) before any."""
        items = np.empty(4608, dtype=np.uint32)
        n, parts = C.c_size_t(0), C.c_uint32(0)
        st = lib().pshbm_debug_part_order(self._h, items.ctypes.data, items.size, C.byref(n), C.byref(parts))
        if st != OK:
            raise PshbmError(st, self.last_error())
        return items[: n.value].copy(), parts.value

    def stats(self):
        s = Stats()
        st = lib().pshbm_get_stats(self._h, C.byref(s))
        if st != OK:
            raise PshbmError(st, self.last_error())
        return s

    def profile_enable(self, on=True):
        return lib().pshbm_profile_enable(self._h, int(on))

    def profile_read(self):
        """{phase: (total ms, launches)} since the last read."""
        p = Profile()
        st = lib().pshbm_profile_read(self._h, C.byref(p))
        if st != OK:
            raise PshbmError(st, self.last_error())
        return {name: (p.ms[i], p.launches[i]) for i, name in enumerate(PHASES)}

    # -- device-pointer entry points (pointers and stream as integers)
    def pull_dev(self, d_keys, n, d_out, d_hit=None, flags=0, stream=0):
        return lib().pshbm_pull_dev(self._h, d_keys, n, d_out, d_hit, flags, stream)

    def push_dev(self, d_keys, d_grads, n, flags=0, stream=0):
        return lib().pshbm_push_dev(self._h, d_keys, d_grads, n, flags, stream)

    def pull_dev_handles(self, d_keys, n, d_out, d_handles, d_hit=None, flags=0, stream=0):
        """pull_dev that also writes a row handle per key (n uint32 on the device); returns
        (status, epoch) for push_dev_handles."""
        epoch = C.c_uint64(0)
        st = lib().pshbm_pull_dev_handles(self._h, d_keys, n, d_out, d_hit, d_handles, C.byref(epoch), flags, stream)
        return st, epoch.value

    def push_dev_handles(self, d_keys, d_grads, d_handles, epoch, n, flags=0, stream=0):
        """push_dev of the key array a pull_dev_handles answered, with that call's handles and epoch."""
        return lib().pshbm_push_dev_handles(self._h, d_keys, d_grads, d_handles, epoch, n, flags, stream)

    def push_dev_noalloc(self, d_keys, d_grads, n, flags=0, stream=0):
        """push_dev with its scratch in the library's fixed device array: allocates nothing."""
        return lib().pshbm_push_dev_noalloc(self._h, d_keys, d_grads, n, flags, stream)

    def queue_dev(self, d_keys, d_grads, n, stream=0):
        return lib().pshbm_queue_dev(self._h, d_keys, d_grads, n, stream)

    def store_dev(self, flags=0, stream=0):
        return lib().pshbm_store_dev(self._h, flags, stream)

    def set_dev(self, d_keys, d_values, n, stream=0):
        return lib().pshbm_set_dev(self._h, d_keys, d_values, n, stream)
