#!/usr/bin/env python3
"""Benchmark of the sparse-table hot path on one MI355X.

A step = one pull of a key batch followed by one push of gradients for the same batch, both
through the device-pointer C ABI with every input already resident in HBM. The default workload
is the headline configuration ("c2": 100M uint64 keys, dim-16 fp32 rows, plain SGD lr 0.01, 1M-key
Zipf(1.05) batches, duplicates summed before the update).

Prints ONE JSON line: metric/value (pulled + pushed keys per second) of the headline
configuration, the roofline of the kernel that takes the most time per step, the same workload
timed on the host CPU with the oracle, and -- under "configs" -- the same measurements for the
other configurations of the benchmark (each on its own table at full size, a shorter run), with
the load factor and probe-distance histogram of every table.
"""
import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published

CONFIGS = {
    # name: table keys, dim, optimizer kwargs, batch, zipf s, fresh fraction, grad sigma
    "c1": dict(n=1_000_000, dim=8, opt=dict(optimizer=1, lr=0.01), batch=65_536, s=None, fresh=0.0,
               sigma=1e-3, pull_only=True,
               desc="C1: 1M keys dim8, pull only, 65536-key uniform batches"),
    "c2": dict(n=100_000_000, dim=16, opt=dict(optimizer=1, lr=0.01), batch=1_000_000, s=1.05,
               fresh=0.0, sigma=1e-3, pull_only=False,
               desc="C2: 100M keys dim16 SGD lr0.01, pull+push of 1M-key Zipf(1.05) batches"),
    "c3": dict(n=50_000_000, dim=64, opt=dict(optimizer=2, lr=0.05, init_acc=0.1), batch=2_000_000,
               s=1.2, fresh=0.0, sigma=1e-3, pull_only=False,
               desc="C3: 50M keys dim64 Adagrad, pull+push of 2M-key Zipf(1.2) batches"),
    "c4": dict(n=500_000_000, dim=8, opt=dict(optimizer=3, alpha=0.05, beta=1.0, l1=1e-4, l2=1e-5),
               batch=4_000_000, s=1.1, fresh=0.05, sigma=1e-2, pull_only=False,
               desc="C4: 500M keys dim8 FTRL, pull+push of 4M-key batches (95% Zipf(1.1), 5% fresh)"),
    "c5": dict(n=200_000_000, dim=128, opt=dict(optimizer=2, lr=0.05, init_acc=0.1), batch=4_000_000,
               s=1.1, fresh=0.0, sigma=1e-3, pull_only=False,
               desc="C5: 200M keys dim128 Adagrad, pull+push of 4M-key Zipf(1.1) batches"),
}
STATE_BLOCKS = {0: 1, 1: 1, 2: 2, 3: 3}
KERNEL_OF_PHASE = {"pull": "pull_kernel", "locate": "locate_kernel", "sort_hist": "sort_hist_kernel",
                   "sort_pass": "sort_pass_kernel", "segreduce": "segreduce_kernel",
                   "fixup": "fixup_kernel", "fixup_windows": "fixup_windows_kernel",
                   "assign_rows": "assign_rows_kernel", "update_unique": "update_unique_kernel",
                   "push_small": "push_small_kernel",
                   "gather": "gather_slots_kernel", "part_tile": "part_tile_kernel",
                   "part_apply": "part_apply_kernel", "part_insert": "part_insert_kernel"}
# HBM bytes per launch as rocprofv3 --pmc counted them on an MI355X (FETCH_SIZE and WRITE_SIZE, each
# scaled by what the same counter reads for a plain copy of known size): NOT measured by this run.
# Every figure names the summary under profiles/ it was copied from; a kernel that has changed since
# must be counted again.
TRAFFIC_FROM_PROFILES = {
    # (config, phase): (bytes, summary)
    ("c1", "pull"): (19226624, "profiles/c1_pull_trace_and_hbm_counters.md"),
    ("c2", "pull"): (196078592, "profiles/c2_pull_push_trace_and_hbm_counters.md"),
    ("c2", "part_tile"): (78201856, "profiles/c2_pull_push_trace_and_hbm_counters.md"),
    ("c2", "part_apply"): (146975744, "profiles/c2_pull_push_trace_and_hbm_counters.md"),
    ("c3", "pull"): (703205376, "profiles/c3_pull_push_trace_and_hbm_counters.md"),
    ("c3", "part_tile"): (450809856, "profiles/c3_pull_push_trace_and_hbm_counters.md"),
    ("c3", "part_apply"): (367959040, "profiles/c3_pull_push_trace_and_hbm_counters.md"),
    ("c4", "pull"): (558414848, "profiles/c4_pull_push_trace_and_hbm_counters.md"),
    ("c4", "part_tile"): (234421248, "profiles/c4_pull_push_trace_and_hbm_counters.md"),
    ("c4", "part_apply"): (640694272, "profiles/c4_pull_push_trace_and_hbm_counters.md"),
    ("c5", "pull"): (3204195328, "profiles/c5_pull_push_trace_and_hbm_counters.md"),
    ("c5", "part_tile"): (1380374528, "profiles/c5_pull_push_trace_and_hbm_counters.md"),
    ("c5", "part_apply"): (2679222272, "profiles/c5_pull_push_trace_and_hbm_counters.md"),
}


def algorithmic_bytes(cfg, phase, k, u, k_alone=None):
    """Bytes of keys, gradients, rows and state one launch must move (probe, partitioning and
    scratch traffic excluded): k = keys in the batch, u = distinct keys, k_alone = keys that do
    not repeat inside their tile of 4096 keys. Over the kernels of a push the figures add up to
    k * (8 + 4 * dim) + u * 2 * row bytes."""
    d4 = 4 * cfg["dim"]
    r = d4 * STATE_BLOCKS[cfg["opt"]["optimizer"]]
    if phase == "pull":
        return k * (8 + d4 + d4)            # key, row read (weights), response write
    if phase == "locate":
        return k * 8                        # key read
    if phase == "segreduce":
        return k * d4 + u * 2 * r           # gradient read, row+state read and write
    if phase == "part_tile":                # keys; the gradient rows of the keys that repeat in their tile
        return k * 8 + (k - (k_alone if k_alone is not None else k)) * d4
    if phase == "part_apply":               # the other gradient rows; row+state read and write
        return (k_alone if k_alone is not None else k) * d4 + u * 2 * r
    return 0                                # sort, scan, scatter, fix-up, row numbering: pure overhead


def build_table(ps, wl, torch, cfg, n_table, seed=0):
    dim = cfg["dim"]
    cap = n_table + max(n_table // 16, 8 * cfg["batch"])   # room for keys that pushes insert
    t = ps.Table(dim, capacity=cap, max_batch=cfg["batch"], **cfg["opt"])
    vf = t.value_floats
    stream = torch.cuda.current_stream().cuda_stream
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1)
    chunk = 4_000_000
    for start in range(0, n_table, chunk):
        cnt = min(chunk, n_table - start)
        keys = wl.table_keys_torch(start, cnt, seed=seed)
        vals = torch.randn(cnt, vf, device="cuda", generator=gen) * 0.01
        if cfg["opt"]["optimizer"] == 2:
            vals[:, dim:] = cfg["opt"]["init_acc"]
        if cfg["opt"]["optimizer"] == 3:   # self-consistent FTRL state: n = z^2
            vals[:, 2 * dim:] = vals[:, dim:2 * dim] ** 2
        st = t.set_dev(keys.data_ptr(), vals.data_ptr(), cnt, stream)
        if st != 0:
            raise RuntimeError(f"set_dev failed: {st} {t.last_error()}")
        torch.cuda.synchronize()
    assert t.size() == n_table, (t.size(), n_table)
    return t


def make_batches(wl, torch, cfg, n_table, n_batches, seed=0):
    gen = torch.Generator(device="cuda")
    gen.manual_seed(2)
    out = []
    for b in range(n_batches):
        k = cfg["batch"]
        if cfg["s"] is None:
            idx = torch.randint(0, n_table, (k,), device="cuda", generator=gen)
            keys = wl.keys_of_index_torch(idx, seed)
        else:
            keys = wl.zipf_batch_torch(gen, n_table, cfg["s"], k, seed=seed)
        nf = int(k * cfg["fresh"])
        if nf:
            fresh = torch.randint(0, 1 << 62, (nf,), device="cuda", generator=gen) * 2 + 1
            pos = torch.randperm(k, device="cuda", generator=gen)[:nf]
            keys[pos] = fresh
        grads = torch.randn(k, cfg["dim"], device="cuda", generator=gen) * cfg["sigma"]
        out.append((keys.contiguous(), grads.contiguous(), int(torch.unique(keys).numel()),
                    keys_alone_in_tile(torch, keys)))
    return out


def keys_alone_in_tile(torch, keys, tile=4096):
    """Keys of the batch that do not repeat inside their tile of `tile` consecutive keys (the
    partitioned push reads their gradient rows in its apply kernel, the others in its tile kernel)."""
    k = keys.numel()
    pad = (-k) % tile
    x = keys
    if pad:   # distinct fillers that equal no key of their tile
        x = torch.cat([keys, torch.arange(pad, device=keys.device, dtype=keys.dtype) - (1 << 62)])
    x = x.view(-1, tile).sort(dim=1).values
    same_next = torch.zeros_like(x, dtype=torch.bool)
    same_next[:, :-1] = x[:, :-1] == x[:, 1:]
    same_prev = torch.zeros_like(same_next)
    same_prev[:, 1:] = same_next[:, :-1]
    return int((~(same_next | same_prev)).sum().item()) - pad


def run_steps(t, torch, cfg, batches, out, steps, first=0, handles=None):
    """`steps` steps: the pull of a batch, then the push of gradients for the same keys. With
    `handles` (a device array of one word per key) the pull tells the push where the rows lie
    (pshbm_pull_dev_handles / pshbm_push_dev_handles), so that the push does not look the keys up
    a second time; without, the plain pshbm_pull_dev / pshbm_push_dev."""
    stream = torch.cuda.current_stream().cuda_stream
    k = cfg["batch"]
    for i in range(first, first + steps):
        keys, grads = batches[i % len(batches)][:2]
        if handles is None or cfg["pull_only"]:
            st = t.pull_dev(keys.data_ptr(), k, out.data_ptr(), None, 0, stream)
            if st == 0 and not cfg["pull_only"]:
                st = t.push_dev(keys.data_ptr(), grads.data_ptr(), k, 0, stream)
        else:
            st, epoch = t.pull_dev_handles(keys.data_ptr(), k, out.data_ptr(), handles.data_ptr(), None, 0, stream)
            if st == 0:
                st = t.push_dev_handles(keys.data_ptr(), grads.data_ptr(), handles.data_ptr(), epoch, k, 0, stream)
        if st != 0:
            raise RuntimeError(f"step {i} failed: {st} {t.last_error()}")


def scan_table(ps, t, cfg, n_table):
    """Whole-table operations at the table's full size: every row and key is read once, so the
    algorithmic bytes of a for-each are rows * (8 + 4 * value floats). Median of 5 calls (the first
    call, which allocates scratch, is not counted); the erase-if runs once, last."""
    rec = 8 + 4 * t.value_floats
    where = ps.predicate((3 % cfg["dim"], ps.CMP_GT, 0.0128))   # weights are N(0, 0.01): about a tenth

    def timed(f, reps):
        f()
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            r = f()
            ts.append(time.perf_counter() - t0)
        return sorted(ts)[len(ts) // 2], r

    rows = t.size()
    dt_all, (st, cnt, _) = timed(lambda: t.for_each(), 5)
    assert st == 0 and cnt == rows
    dt_sel, (st, n_sel, _) = timed(lambda: t.for_each(where), 5)
    assert st == 0
    # the writing for-each with the identity map 1 * v + 0 on every column: rows read and written
    ident = ps.update(ps.UPD_AFFINE, 0, t.value_floats, 1.0, 0.0)
    dt_write, (st, n_written) = timed(lambda: t.for_each_write(ident), 3)
    assert st == 0 and n_written == rows
    t0 = time.perf_counter()
    st, erased = t.erase_if(where)
    dt_erase = time.perf_counter() - t0
    assert st == 0 and erased == n_sel and t.size() == rows - n_sel
    return {"rows": rows, "record_bytes": rec,
            "for_each_ms": round(dt_all * 1e3, 3), "for_each_GBps": round(rows * rec / dt_all / 1e9, 1),
            "for_each_where_ms": round(dt_sel * 1e3, 3), "selected": int(n_sel),
            "for_each_write_ms": round(dt_write * 1e3, 3),
            "for_each_write_GBps": round(rows * (rec + rec - 8) / dt_write / 1e9, 1),
            "erase_if_ms": round(dt_erase * 1e3, 3), "erased": int(erased),
            "note": "wall clock of the synchronous calls, read-back of the result included"}


def bulk_transfers(ps, t, cfg):
    """Dump of the whole table into page-locked host memory and Load of the same records into a
    second, empty table (a restore: every key is new), timed as the synchronous calls they are. The
    records cross the link once each way; the rate is record bytes over wall clock."""
    rows = t.size()
    rec = ps.pinned_empty(rows, ps.record_dtype(t.value_floats))   # page-locking is not timed
    t0 = time.perf_counter()
    st, got = t.dump(out=rec)
    dt_dump = time.perf_counter() - t0
    assert st == 0 and got.size == rows
    t2 = ps.Table(cfg["dim"], capacity=rows + 16, max_batch=1 << 20, **cfg["opt"])
    t0 = time.perf_counter()
    st = t2.load(got, ps.LOAD_UNIQUE)
    dt_load = time.perf_counter() - t0
    assert st == 0 and t2.size() == rows
    t2.close()
    nbytes = rows * rec.dtype.itemsize
    return {"rows": rows, "record_bytes": rec.dtype.itemsize, "bytes": nbytes,
            "dump_ms": round(dt_dump * 1e3, 2), "dump_GBps": round(nbytes / dt_dump / 1e9, 1),
            "load_ms": round(dt_load * 1e3, 2), "load_GBps": round(nbytes / dt_load / 1e9, 1),
            "note": "host buffer page-locked; PCIe-inclusive by nature, never part of `value`"}


def cpu_baseline(cfg, wl, budget_keys):
    """The oracle (a scalar port of the reference's operator loops) on a bounded sample of the same
    workload: a table of budget_keys keys and a few batches of the configured size, one thread."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import numpy as np
    import oracle
    n = min(cfg["n"], budget_keys)
    dim, k = cfg["dim"], cfg["batch"]
    o = oracle.Oracle(dim, capacity=n + 8 * k, **cfg["opt"])
    vf = o.value_floats
    rng = np.random.default_rng(1)
    chunk = 1_000_000
    for start in range(0, n, chunk):
        cnt = min(chunk, n - start)
        vals = (rng.standard_normal((cnt, vf), dtype=np.float32) * np.float32(0.01))
        if cfg["opt"]["optimizer"] == 2:
            vals[:, dim:] = cfg["opt"]["init_acc"]
        if cfg["opt"]["optimizer"] == 3:
            vals[:, 2 * dim:] = vals[:, dim:2 * dim] ** 2
        assert o.set(wl.table_keys_np(start, cnt, seed=0), vals) == 0
        if (start // chunk) % 10 == 9:
            print(f"cpu_baseline: {start + cnt} of {n} keys stored", file=sys.stderr, flush=True)
    steps, times = 4, []
    for s in range(steps):
        if cfg["s"] is None:
            keys = wl.keys_of_index_np(rng.integers(0, n, k), 0)
        else:
            keys = wl.zipf_batch_np(rng, n, cfg["s"], k, seed=0)
        grads = rng.standard_normal((k, dim), dtype=np.float32) * np.float32(cfg["sigma"])
        t0 = time.perf_counter()
        st, rows, hit = o.pull(keys)
        if not cfg["pull_only"]:
            assert o.push(keys, grads) == 0
        times.append(time.perf_counter() - t0)
    per_step = sorted(times[1:])[len(times[1:]) // 2]   # first step warms the caches
    keys_per_step = k * (1 if cfg["pull_only"] else 2)
    o.close()
    return {
        "value": keys_per_step / per_step, "unit": "keys/s", "cores": 1, "kind": "port",
        "sample": (f"the full {n}-key table" if n == cfg["n"] else
                   f"{n}-key table (of {cfg['n']}: the two full tables of this leg take 3.5 minutes to build in "
                   f"std::unordered_map, so the default run is bounded to about 30 s of CPU work; a smaller table "
                   f"only helps the CPU's caches -- C2 measured once with --cpu-keys 100000000 on the same host: "
                   f"8.0 M keys/s on one thread, 87.8 M keys/s on 16 shards)") +
                  f", median of {steps - 1} steps of {k}-key batches, oracle/ps_oracle.cpp single thread",
        "sharded": cpu_baseline_sharded(cfg, wl, n, oracle, np),
    }


def cpu_baseline_sharded(cfg, wl, n, oracle, np):
    """The same sample on S shards, one applying thread per shard (a push takes its shard
    exclusively, pico-ps/operator/SparsePushOperator.h:220, so a shard never has more): the table
    and every batch are split by key, as the reference's client does before it sends
    (SparsePushOperator.h:161-184); the split is not timed, the shards run concurrently."""
    from concurrent.futures import ThreadPoolExecutor
    S = max(1, min(16, os.cpu_count() or 1))
    dim, k = cfg["dim"], cfg["batch"]
    shards = [oracle.Oracle(dim, capacity=2 * n // S + 8 * k, **cfg["opt"]) for _ in range(S)]
    vf = shards[0].value_floats
    rng = np.random.default_rng(1)
    chunk = 1_000_000
    for start in range(0, n, chunk):
        cnt = min(chunk, n - start)
        keys = wl.table_keys_np(start, cnt, seed=0)
        vals = (rng.standard_normal((cnt, vf), dtype=np.float32) * np.float32(0.01))
        if cfg["opt"]["optimizer"] == 2:
            vals[:, dim:] = cfg["opt"]["init_acc"]
        if cfg["opt"]["optimizer"] == 3:
            vals[:, 2 * dim:] = vals[:, dim:2 * dim] ** 2
        which = keys % np.uint64(S)
        for s in range(S):
            m = which == s
            assert shards[s].set(keys[m], vals[m]) == 0
        if (start // chunk) % 10 == 9:
            print(f"cpu_baseline, {S} shards: {start + cnt} of {n} keys stored", file=sys.stderr, flush=True)

    def apply(job):
        o, keys, grads = job
        o.pull(keys)
        if not cfg["pull_only"]:
            assert o.push(keys, grads) == 0

    steps, times = 4, []
    with ThreadPoolExecutor(S) as pool:
        for _ in range(steps):
            if cfg["s"] is None:
                keys = wl.keys_of_index_np(rng.integers(0, n, k), 0)
            else:
                keys = wl.zipf_batch_np(rng, n, cfg["s"], k, seed=0)
            grads = rng.standard_normal((k, dim), dtype=np.float32) * np.float32(cfg["sigma"])
            which = keys % np.uint64(S)
            jobs = [(shards[s], np.ascontiguousarray(keys[which == s]),
                     np.ascontiguousarray(grads[which == s])) for s in range(S)]
            t0 = time.perf_counter()
            list(pool.map(apply, jobs))
            times.append(time.perf_counter() - t0)
    for o in shards:
        o.close()
    per_step = sorted(times[1:])[len(times[1:]) // 2]
    return {"value": k * (1 if cfg["pull_only"] else 2) / per_step, "unit": "keys/s", "cores": S,
            "sample": f"the same table and batches split over {S} shards by key, one thread per shard"}


def table_stats(t):
    """Load factor and probe-distance histogram of the table (pshbm_get_stats): keys whose bucket
    lies h buckets past their home bucket, h = 0..14, then 15 and more."""
    st = t.stats()
    return {"keys": int(st.size), "slots": int(st.slots), "load_factor": round(st.load_factor, 4),
            "probe_hist": [int(x) for x in st.probe_hist], "max_probe": int(st.max_probe)}


def bulk_slice(ps, t, cfg, max_bytes):
    """The Dump + Load leg on as large a slice of the table as `max_bytes` of page-locked host memory
    hold: the first records of the dump sequence (pshbm_iterate) into a pinned buffer, then Load of
    those records into a second, empty table. Synchronous calls; the rate is record bytes over wall
    clock, so the whole table would take its record bytes at that rate."""
    dt = ps.record_dtype(t.value_floats)
    rows = t.size()
    n = int(min(rows, max_bytes // dt.itemsize))
    lib = ps.lib()
    import ctypes as C
    rec = ps.pinned_empty(n, dt)                      # page-locking is not timed
    got = C.c_size_t()
    t0 = time.perf_counter()
    st = lib.pshbm_iterate(t._h, 0, n, rec.ctypes.data, C.byref(got))
    dt_dump = time.perf_counter() - t0
    assert st == 0 and got.value == n, (st, got.value, t.last_error())
    t2 = ps.Table(cfg["dim"], capacity=n + 16, max_batch=1 << 20, **cfg["opt"])
    t0 = time.perf_counter()
    st = t2.load(rec, ps.LOAD_UNIQUE)
    dt_load = time.perf_counter() - t0
    assert st == 0 and t2.size() == n, (st, t2.last_error())
    t2.close()
    nbytes = n * dt.itemsize
    full = rows * dt.itemsize
    return {"records": n, "of_records": rows, "record_bytes": dt.itemsize, "bytes": nbytes,
            "dump_ms": round(dt_dump * 1e3, 2), "dump_GBps": round(nbytes / dt_dump / 1e9, 1),
            "load_ms": round(dt_load * 1e3, 2), "load_GBps": round(nbytes / dt_load / 1e9, 1),
            "whole_table_dump_s_at_this_rate": round(full / (nbytes / dt_dump), 2),
            "whole_table_load_s_at_this_rate": round(full / (nbytes / dt_load), 2),
            "note": "a slice of the table through a page-locked buffer of this size (pshbm_iterate, then "
                    "pshbm_load into an empty table); PCIe-inclusive by nature, never part of `value`"}


def measure(name, args, torch, ps, wl, steps, warmup, headline):
    """One configuration on its own table at full size: W warm-up steps, K timed steps between two
    device synchronisations, then the same K steps with HIP events around every kernel launch."""
    cfg = dict(CONFIGS[name])
    n_table = (args.table_keys if headline else 0) or cfg["n"]
    t = build_table(ps, wl, torch, cfg, n_table)
    # Eight batches in turn -- except where batches bring fresh keys (c4): there every step of the
    # warm-up, of the timed run and of the run under events gets a batch of its own, so that each
    # step really inserts its fresh keys (a batch that comes round again would find them stored).
    n_batches = (warmup + 2 * steps) if cfg["fresh"] > 0 else 8
    batches = make_batches(wl, torch, cfg, n_table, n_batches=n_batches)
    out = torch.empty(cfg["batch"], cfg["dim"], device="cuda")
    k = cfg["batch"]
    keys_per_step = k * (1 if cfg["pull_only"] else 2)
    handles = None if args.no_handles else torch.empty(k, dtype=torch.int32, device="cuda")

    run_steps(t, torch, cfg, batches, out, warmup, handles=handles)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    run_steps(t, torch, cfg, batches, out, steps, first=warmup, handles=handles)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / steps

    t.profile_enable(True)
    run_steps(t, torch, cfg, batches, out, steps, first=warmup + (steps if cfg["fresh"] > 0 else 0), handles=handles)
    torch.cuda.synchronize()
    prof = t.profile_read()
    t.profile_enable(False)
    u_mean = sum(b[2] for b in batches) / len(batches)
    alone_mean = sum(b[3] for b in batches) / len(batches)
    phases = {}
    for phase, (ms, launches) in prof.items():
        if launches:
            avg_ms = ms / launches
            by = algorithmic_bytes(cfg, phase, k, u_mean, alone_mean)
            phases[phase] = {"kernel": KERNEL_OF_PHASE[phase], "avg_ms": round(avg_ms, 5), "launches": int(launches),
                             "ms_per_step": round(ms / steps, 5),
                             "algorithmic_GBps": round(by / avg_ms / 1e6, 1)}
    # the kernel that takes the most time per step (all its launches of a step together)
    dominant = max(phases, key=lambda p: phases[p]["ms_per_step"])
    achieved = phases[dominant]["algorithmic_GBps"]
    # (the profiled runs were at full table size, with row handles)
    profiled = n_table == cfg["n"] and (handles is not None or cfg["pull_only"])
    traffic = TRAFFIC_FROM_PROFILES.get((name, dominant)) if profiled else None
    step_traffic = [TRAFFIC_FROM_PROFILES.get((name, ph)) for ph in phases if ph != "part_insert"]
    step_traffic = sum(x[0] for x in step_traffic) if profiled and all(step_traffic) else None
    roofline = {"kernel": KERNEL_OF_PHASE[dominant], "bound": "hbm", "achieved": achieved,
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                "traffic": traffic[0] if traffic else None,
                "traffic_from_profile": traffic[1] if traffic else None,
                "avg_ms": phases[dominant]["avg_ms"],
                "algorithmic_bytes": int(algorithmic_bytes(cfg, dominant, k, u_mean, alone_mean)),
                "note": "achieved = algorithmic bytes of one launch / its average duration (HIP events on the "
                        "launch stream, this run); traffic = HBM bytes per launch counted by rocprofv3 --pmc in "
                        "the run the named summary describes, not in this one"}
    step_bytes = algorithmic_bytes(cfg, "pull", k, u_mean)
    if not cfg["pull_only"]:
        step_bytes += algorithmic_bytes(cfg, "segreduce", k, u_mean) + 8 * k   # = k (8 + 4 dim) + u 2 R
    res = {
        "value": keys_per_step * steps / elapsed, "ms_per_step": ms_per_step, "steps": steps, "warmup": warmup,
        "config": {"workload": cfg["desc"], "table_keys": n_table, "batch": k, "dim": cfg["dim"],
                   "unique_keys_per_batch": round(u_mean), "keys_alone_in_their_tile": round(alone_mean),
                   "row_handles": handles is not None and not cfg["pull_only"],
                   "batches": n_batches},
        "step_algorithmic_bytes": int(step_bytes),
        "step_algorithmic_GBps": round(step_bytes / (ms_per_step * 1e6), 1),
        "step_frac_of_hbm_peak": round(step_bytes / (ms_per_step * 1e6) / HBM_PEAK_GBS, 4),
        "kernel_ms_per_step": round(sum(p["ms_per_step"] for p in phases.values()), 5),
        "step_traffic_bytes_from_profiles": step_traffic,
        "step_traffic_over_algorithmic": round(step_traffic / step_bytes, 2) if step_traffic else None,
        "roofline": roofline,
        "phases": phases,
        "table_stats": table_stats(t),
    }
    if headline and args.bulk:
        res["bulk"] = bulk_transfers(ps, t, cfg)
    if name == "c5" and not args.no_bulk_slice:
        res["bulk"] = bulk_slice(ps, t, cfg, args.bulk_slice_bytes)
    if headline and args.scan:
        res["scan"] = scan_table(ps, t, cfg, n_table)
    t.close()
    del out, batches
    torch.cuda.empty_cache()
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", default="c2", choices=sorted(CONFIGS),
                    help="the headline configuration (value, ms_per_step, roofline, cpu_baseline)")
    ap.add_argument("--only", action="store_true",
                    help="measure the headline configuration only (profiling runs); by default the other "
                         "configurations follow, 20 steps each, and are reported under \"configs\"")
    ap.add_argument("--table-keys", type=int, default=0, help="override the headline table size (testing)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-handles", action="store_true",
                    help="plain pshbm_pull_dev / pshbm_push_dev: the push looks every key up again instead of "
                         "taking the rows the pull of the same batch found")
    ap.add_argument("--cpu-keys", type=int, default=10_000_000, help="table size of the CPU sample")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run one 256 MiB device copy, a kernel of known HBM traffic that "
                         "rocprofv3 --pmc runs of this script use to scale FETCH_SIZE / WRITE_SIZE")
    ap.add_argument("--scan", action="store_true",
                    help="after the steps, also time the whole-table operations on the same table: "
                         "for-each (count + column sums), for-each under a predicate on a value "
                         "column, erase-if of about a tenth of the keys; reported under \"scan\"")
    ap.add_argument("--bulk", action="store_true",
                    help="after the steps, also time Dump of the whole headline table into page-locked host "
                         "memory and Load of those records into an empty table; reported under \"bulk\"")
    ap.add_argument("--bulk-slice-bytes", type=int, default=16 << 30,
                    help="page-locked bytes of the Dump + Load leg of c5 (a slice of its 215 GB table)")
    ap.add_argument("--no-bulk-slice", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (--gpus must be 1)")

    import torch
    ps = importlib.import_module("parameter-server_amd")
    wl = importlib.import_module("parameter-server_amd.workload")
    ps.lib()  # fails loudly if the HIP library has not been built
    torch.cuda.set_device(0)

    if args.calibration_copy:
        a = torch.empty(64 << 20, dtype=torch.float32, device="cuda").normal_()
        b = torch.empty_like(a)
        for _ in range(3):
            b.copy_(a)
        torch.cuda.synchronize()
        del a, b
    head = measure(args.config, args, torch, ps, wl, args.steps, args.warmup, headline=True)
    result = {
        "metric": "pulled+pushed keys/sec on 1 MI355X; achieved HBM GB/s as % of peak",
        "value": head.pop("value"), "unit": "keys/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": head.pop("ms_per_step"), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
    }
    head.pop("steps"), head.pop("warmup")
    result.update(head)
    if not args.only:
        result["configs"] = {}
        for other in sorted(CONFIGS):
            if other != args.config:
                result["configs"][other] = measure(other, args, torch, ps, wl, min(args.steps, 20),
                                                   min(args.warmup, 3), headline=False)
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(dict(CONFIGS[args.config]), wl, args.cpu_keys)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
