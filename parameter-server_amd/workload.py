"""Seeded synthetic workloads of the benchmark configurations: table keys, initial rows, Zipf key
batches and gradients. Every generator exists for numpy (host) and torch (device) arrays; the
two draw from different random streams but from the same distributions.

Keys of a table are mix64(i) for i = 0..N-1: mix64 is a bijection of the 64-bit integers, so the
keys are distinct without any bookkeeping and look uniformly random.
Batches draw a rank r in [1, N] from Zipf(s) by rejection-inversion (Hormann & Derflinger 1996)
and map it to the table index (r * STRIDE) mod N, so that popular keys are scattered over the
row slab instead of sitting next to each other.
"""
import numpy as np

GOLDEN = 0x9E3779B97F4A7C15
MASK64 = (1 << 64) - 1
RANK_STRIDE = 2654435761  # odd prime; coprime to every table size used here


def mix64_int(x):
    """splitmix64 finalizer on a Python int."""
    x = (x + GOLDEN) & MASK64
    x ^= x >> 30
    x = (x * 0xBF58476D1CE4E5B9) & MASK64
    x ^= x >> 27
    x = (x * 0x94D049BB133111EB) & MASK64
    x ^= x >> 31
    return x


def mix64_np(x):
    x = np.asarray(x, dtype=np.uint64)
    with np.errstate(over="ignore"):
        x = x + np.uint64(GOLDEN)
        x = x ^ (x >> np.uint64(30))
        x = x * np.uint64(0xBF58476D1CE4E5B9)
        x = x ^ (x >> np.uint64(27))
        x = x * np.uint64(0x94D049BB133111EB)
        x = x ^ (x >> np.uint64(31))
    return x


def _lsr_t(x, s):
    """logical shift right of an int64 torch tensor"""
    return (x >> s) & ((1 << (64 - s)) - 1)


def _as_i64(c):
    return c - (1 << 64) if c >= (1 << 63) else c


def mix64_torch(x):
    """mix64 on an int64 tensor holding the bit patterns of uint64 values (wrapping arithmetic)."""
    x = x + _as_i64(GOLDEN)
    x = x ^ _lsr_t(x, 30)
    x = x * _as_i64(0xBF58476D1CE4E5B9)
    x = x ^ _lsr_t(x, 27)
    x = x * _as_i64(0x94D049BB133111EB)
    x = x ^ _lsr_t(x, 31)
    return x


def table_keys_np(start, count, seed=0):
    """keys start .. start+count of the table generated with `seed` (uint64)."""
    i = np.arange(start, start + count, dtype=np.uint64)
    with np.errstate(over="ignore"):
        return mix64_np(i ^ (np.uint64(seed) * np.uint64(0xD6E8FEB86659FD93)))


def table_keys_torch(start, count, seed=0, device="cuda"):
    import torch
    i = torch.arange(start, start + count, dtype=torch.int64, device=device)
    return mix64_torch(i ^ _as_i64((seed * 0xD6E8FEB86659FD93) & MASK64))


def keys_of_index_np(idx, seed=0):
    with np.errstate(over="ignore"):
        return mix64_np(np.asarray(idx, dtype=np.uint64) ^ (np.uint64(seed) * np.uint64(0xD6E8FEB86659FD93)))


def keys_of_index_torch(idx, seed=0):
    return mix64_torch(idx ^ _as_i64((seed * 0xD6E8FEB86659FD93) & MASK64))


# ---- Zipf by rejection-inversion -------------------------------------------------------------
class _Zipf:
    def __init__(self, n, s, xp, f64):
        self.n, self.s, self.xp, self.f64 = float(n), float(s), xp, f64
        self.h_x1 = self._h_integral_s(1.5) - 1.0
        self.h_n = self._h_integral_s(self.n + 0.5)
        self.sp = 2.0 - self._h_inv_s(self._h_integral_s(2.5) - 2.0 ** (-self.s))

    # scalar versions (Python floats) for the constants
    def _h_integral_s(self, x):
        lx = np.log(x)
        t = (1.0 - self.s) * lx
        return (np.expm1(t) / t if abs(t) > 1e-8 else 1.0 + t / 2) * lx

    def _h_inv_s(self, x):
        t = max(x * (1.0 - self.s), -1.0)
        return float(np.exp((np.log1p(t) / t if abs(t) > 1e-8 else 1.0 - t / 2) * x))

    # array versions
    def h_integral(self, x):
        xp = self.xp
        lx = xp.log(x)
        t = (1.0 - self.s) * lx
        small = xp.abs(t) < 1e-8
        ts = xp.where(small, t * 0 + 1.0, t)
        return xp.where(small, 1.0 + t / 2, xp.expm1(ts) / ts) * lx

    def h(self, x):
        return self.xp.exp(-self.s * self.xp.log(x))

    def h_inv(self, x):
        xp = self.xp
        t = x * (1.0 - self.s)
        t = xp.where(t < -1.0, t * 0 - 1.0, t)
        small = xp.abs(t) < 1e-8
        ts = xp.where(small, t * 0 + 1.0, t)
        return xp.exp(xp.where(small, 1.0 - t / 2, xp.log1p(ts) / ts) * x)

    def accept(self, u):
        """for uniforms u in (0,1): candidate ranks and their acceptance mask"""
        xp = self.xp
        v = self.h_n + u * (self.h_x1 - self.h_n)
        x = self.h_inv(v)
        k = xp.floor(x + 0.5)
        k = xp.where(k < 1.0, k * 0 + 1.0, k)
        k = xp.where(k > self.n, k * 0 + self.n, k)
        ok = (k - x <= self.sp) | (v >= self.h_integral(k + 0.5) - self.h(k))
        return k, ok


def zipf_ranks_np(rng, n_table, s, count):
    z = _Zipf(n_table, s, np, np.float64)
    out = np.empty(count, dtype=np.int64)
    todo = np.arange(count)
    while todo.size:
        k, ok = z.accept(rng.random(todo.size))
        out[todo[ok]] = k[ok].astype(np.int64)
        todo = todo[~ok]
    return out


def zipf_ranks_torch(gen, n_table, s, count, device="cuda"):
    import torch
    z = _Zipf(n_table, s, torch, torch.float64)
    out = torch.empty(count, dtype=torch.int64, device=device)
    todo = torch.arange(count, device=device)
    while todo.numel():
        u = torch.rand(todo.numel(), dtype=torch.float64, device=device, generator=gen)
        k, ok = z.accept(u)
        out[todo[ok]] = k[ok].to(torch.int64)
        todo = todo[~ok]
    return out


def rank_to_index_np(rank, n_table):
    return (rank.astype(np.uint64) * np.uint64(RANK_STRIDE)) % np.uint64(n_table)


def rank_to_index_torch(rank, n_table):
    return (rank * RANK_STRIDE) % n_table


def zipf_batch_np(rng, n_table, s, count, seed=0):
    """`count` keys of the table generated with `seed`, popularity ~ Zipf(s)."""
    return keys_of_index_np(rank_to_index_np(zipf_ranks_np(rng, n_table, s, count), n_table), seed)


def zipf_batch_torch(gen, n_table, s, count, seed=0, device="cuda"):
    return keys_of_index_torch(
        rank_to_index_torch(zipf_ranks_torch(gen, n_table, s, count, device), n_table), seed)


def fresh_keys_np(rng, count):
    """uniform random uint64 keys that are not in any generated table with overwhelming probability"""
    k = rng.integers(0, 1 << 63, size=count, dtype=np.uint64) * np.uint64(2) + np.uint64(1)
    return np.minimum(k, np.uint64(0xFFFFFFFFFFFFFFFD))
