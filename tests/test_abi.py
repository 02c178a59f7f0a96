"""The C-ABI library loads and exports every symbol include/pshbm.h declares (no GPU needed)."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "pshbm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pshbm_[a-z_]+)\s*\(", text)))


def test_header_and_binding_agree(ps):
    assert declared_symbols() == sorted(ps.SYMBOLS)


def test_library_exports_every_declared_symbol(ps):
    lib = ctypes.CDLL(ps.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(lib, name), name


def test_value_floats(ps):
    assert ps.value_floats(16, ps.OPT_SGD) == 16
    assert ps.value_floats(16, ps.OPT_SUM) == 16
    assert ps.value_floats(64, ps.OPT_ADAGRAD) == 128
    assert ps.value_floats(8, ps.OPT_FTRL) == 24
    assert ps.value_floats(8, 99) == 0


def test_status_codes_match_the_reference_enum(ps):
    # pico-ps/common/Status.h:15-29
    assert (ps.OK, ps.INVALID_CONFIG, ps.INVALID_ID, ps.OUT_OF_MEMORY, ps.ERROR, ps.FATAL) == (0, 1, 2, 3, 10, 11)


@pytest.mark.parametrize("kw", [
    dict(dim=0), dict(dim=1 << 20), dict(dim=4, optimizer=7), dict(dim=4, capacity=0),
    dict(dim=4, max_load_factor=0.95), dict(dim=4, optimizer=3, alpha=0.0),
])
def test_invalid_config_is_refused_before_any_device_work(ps, kw):
    with pytest.raises(ps.PshbmError) as e:
        ps.Table(**kw)
    assert e.value.status == ps.INVALID_CONFIG


def test_null_handle_is_invalid_id(ps):
    n = ctypes.c_uint64()
    assert ps.lib().pshbm_size(None, ctypes.byref(n)) == ps.INVALID_ID
    assert ps.lib().pshbm_pull(None, None, 0, None, None, 0) == ps.INVALID_ID


def test_record_layout(ps):
    dt = ps.record_dtype(6)
    assert dt.itemsize == 8 + 24 and dt.fields["value"][1] == 8


def test_memory_limit_is_kept_per_device_without_a_gpu(ps):
    assert ps.device_memory(3) == (0, 0)
    ps.set_memory_limit(3, 1 << 30)
    assert ps.device_memory(3) == (0, 1 << 30) and ps.device_memory(2) == (0, 0)
    ps.set_memory_limit(3, 0)
    assert ps.device_memory(3) == (0, 0)
    for bad in (-1, 64):
        try:
            ps.set_memory_limit(bad, 1)
        except ps.PshbmError as e:
            assert e.status == ps.INVALID_ID
        else:
            raise AssertionError("a device ordinal out of range was accepted")


def test_marker_limit_keeps_room_in_the_hash_array(ps):
    """Markers of erased keys are never reused by inserts: a full table plus its markers must stay
    below 95 % of the slots whatever max_load_factor (up to 0.9) put the capacity at."""
    lim = ps.lib().pshbm_debug_tombstone_limit
    assert lim(1 << 20, 1 << 19) == (1 << 20) // 8                 # load factor 0.5: an eighth of the slots
    assert lim(1 << 20, 940_000) == (1 << 20) - (1 << 20) // 20 - 940_000   # 0.9: what is left below 95 %
    assert lim(1 << 20, 1 << 20) == 0
    for slots in (1 << 10, 1 << 20, 1 << 28):
        for lf in (0.1, 0.5, 0.75, 0.875, 0.9):
            rows = int(slots * lf)
            assert rows + lim(slots, rows) <= slots - slots // 20
            assert lim(slots, rows) <= slots // 8
