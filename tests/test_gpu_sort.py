"""The library's radix sort of (key, value) pairs on its own, through a test-only export, against
numpy's stable sort: sizes from one tile to 16M pairs (the one-launch-per-pass scheme up to 2^20
pairs, the three-launches-per-pass scheme above), 6 to 30 key bits, inputs with heavy repeats.
Stability is part of the contract: the values (batch indices) of equal keys keep their input
order, which is what makes the segmented sums of the sorted push add in batch order."""
import ctypes as C

import numpy as np
import pytest

torch = pytest.importorskip("torch")

pytestmark = pytest.mark.gpu


def device_sort(ps, keys, vals, bits):
    n = keys.size
    dk = torch.from_numpy(keys.view(np.int32)).cuda()
    dv = torch.from_numpy(vals.view(np.int32)).cuda()
    tk, tv = torch.empty_like(dk), torch.empty_like(dv)
    in_tmp = C.c_int32(-1)
    stream = torch.cuda.current_stream().cuda_stream
    st = ps.lib().pshbm_debug_sort_pairs(0, dk.data_ptr(), dv.data_ptr(), tk.data_ptr(), tv.data_ptr(), n, bits,
                                         C.byref(in_tmp), stream)
    assert st == 0, st
    ok, ov = (tk, tv) if in_tmp.value == 1 else (dk, dv)
    return ok.cpu().numpy().view(np.uint32), ov.cpu().numpy().view(np.uint32)


def make_keys(rng, n, bits, shape):
    top = (1 << bits) - 1
    if shape == "uniform":
        k = rng.integers(0, top + 1, n, dtype=np.uint64)
    elif shape == "hot":          # one key in 8 % of the positions, 50,000 warm keys in 40 %, the rest anywhere
        u = rng.random(n)
        k = rng.integers(0, top + 1, n, dtype=np.uint64)
        warm = (rng.integers(0, 50000, n, dtype=np.uint64) * np.uint64(5003)) & np.uint64(top)
        k = np.where(u < 0.5, warm, k)
        k = np.where(u < 0.08, np.uint64(12345677 & top), k)
    else:                          # few distinct keys: long runs everywhere
        k = rng.integers(0, min(top + 1, 37), n, dtype=np.uint64)
    return k.astype(np.uint32)


@pytest.mark.parametrize("n,bits", [(1, 8), (63, 6), (4096, 12), (4097, 20), (65_536, 27), (100_003, 9),
                                    (1 << 20, 27), ((1 << 20) + 1, 27), (2_500_000, 30), (4_000_000, 28),
                                    (16_000_000, 30)])
@pytest.mark.parametrize("shape", ["uniform", "hot", "runs"])
def test_sort_is_numpys_stable_sort(ps, n, bits, shape):
    rng = np.random.default_rng(n % 9973 + bits)
    keys = make_keys(rng, n, bits, shape)
    vals = np.arange(n, dtype=np.uint32)
    got_k, got_v = device_sort(ps, keys.copy(), vals.copy(), bits)
    order = np.argsort(keys, kind="stable")
    np.testing.assert_array_equal(got_k, keys[order])
    np.testing.assert_array_equal(got_v, vals[order])
