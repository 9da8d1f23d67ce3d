"""The C ABI library loads without a GPU and exports every symbol that
include/hkv_c_api.h declares; the Python binding covers the same set."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "hkv_c_api.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b(hkv_[a-z0-9_]+)\s*\(", text)
    # function-pointer members of hkv_allocator are not symbols
    return sorted(set(n for n in names if n not in ("hkv_allocator",)))


def test_every_declared_symbol_is_exported():
    from hierarchicalkv_amd import _capi
    lib = ctypes.CDLL(_capi.LIB_PATH)
    names = declared_functions()
    assert len(names) >= 35
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in hkv_c_api.h but not exported"
    assert set(names) == set(_capi.SIGNATURES), set(names) ^ set(_capi.SIGNATURES)


def test_library_reports_version_and_defaults():
    from hierarchicalkv_amd import _capi
    assert b"gfx950" in _capi.lib.hkv_version()
    o = _capi.Options()
    _capi.lib.hkv_options_default(ctypes.byref(o))
    # HashTableOptions defaults, merlin_hashtable.cuh:103-136
    assert (o.max_bucket_size, o.dim, o.block_size, o.io_block_size, o.device_id) == (128, 64, 128, 1024, -1)
    assert abs(o.max_load_factor - 0.5) < 1e-9 and o.api_lock == 1 and o.num_of_buckets_per_alloc == 1
    assert o.reserved_key_start_bit == 0 and o.io_by_cpu == 0 and o.table_mode == 0


def test_option_checks_need_no_gpu():
    """init's argument checks (merlin_hashtable.cuh:1016-1048) run before any
    device call, so they are observable on a machine without a GPU."""
    from hierarchicalkv_amd import HashTable, MerlinException, default_options
    for bad in (dict(reserved_key_start_bit=63), dict(max_bucket_size=100),
                dict(num_of_buckets_per_alloc=3)):
        t = HashTable()
        with pytest.raises(MerlinException):
            t.init(default_options(init_capacity=1024, max_capacity=1024, **bad))
    # dual-bucket mode has checks of its own (merlin_hashtable.cuh:992-1014)
    for bad in (dict(init_capacity=1024, max_capacity=2048), dict(max_hbm_for_vectors=1 << 30),
                dict(dim=225), dict(init_capacity=128, max_capacity=128)):
        kw = dict(init_capacity=1024, max_capacity=1024, max_hbm_for_vectors=0, dim=4, table_mode=1)
        kw.update(bad)
        with pytest.raises(MerlinException):
            HashTable().init(default_options(**kw))
    t = HashTable()
    with pytest.raises(ValueError):
        t.init(default_options(init_capacity=1024, max_capacity=1024, table_mode=2))
    with pytest.raises(NotImplementedError):
        t.init(default_options(init_capacity=1024, max_capacity=1024, score_size=4))
