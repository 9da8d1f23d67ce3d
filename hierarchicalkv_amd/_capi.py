"""ctypes binding of the C ABI declared in include/hkv_c_api.h.

The native library is the product; there is no Python or CPU fallback.  If
libhkv.so is missing the import of this module raises, with the build command
in the message.
"""
import ctypes as C
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("HKV_LIB_PATH") or os.path.join(_PKG, "libhkv.so")

HKV_SUCCESS = 0
HKV_ERROR_CHECK = 1
HKV_ERROR_HIP = 2
HKV_ERROR_RUNTIME = 3
HKV_ERROR_ARGUMENT = 4
HKV_ERROR_UNSUPPORTED = 5


class Options(C.Structure):
    """struct hkv_options (HashTableOptions, merlin_hashtable.cuh:103-136)."""
    _fields_ = [
        ("init_capacity", C.c_uint64),
        ("max_capacity", C.c_uint64),
        ("max_hbm_for_vectors", C.c_uint64),
        ("max_bucket_size", C.c_uint64),
        ("dim", C.c_uint64),
        ("max_load_factor", C.c_float),
        ("block_size", C.c_int32),
        ("io_block_size", C.c_int32),
        ("device_id", C.c_int32),
        ("io_by_cpu", C.c_int32),
        ("use_constant_memory", C.c_int32),
        ("reserved_key_start_bit", C.c_int32),
        ("num_of_buckets_per_alloc", C.c_uint64),
        ("api_lock", C.c_int32),
        ("table_mode", C.c_int32),
        ("evict_strategy", C.c_int32),
        ("value_kind", C.c_int32),
        ("value_size", C.c_uint32),
        ("score_size", C.c_uint32),
    ]


class TableView(C.Structure):
    """struct hkv_table_view."""
    _fields_ = [
        ("digests", C.c_void_p),
        ("keys", C.c_void_p),
        ("scores", C.c_void_p),
        ("sizes", C.c_void_p),
        ("values", C.c_void_p),
        ("host_values", C.c_void_p),
        ("hbm_slots", C.c_uint64),
        ("buckets_num", C.c_uint64),
        ("capacity", C.c_uint64),
        ("value_bytes", C.c_uint32),
        ("dim", C.c_uint32),
        ("empty_key", C.c_uint64),
        ("reclaim_key", C.c_uint64),
        ("locked_key", C.c_uint64),
        ("reserved_mask1", C.c_uint64),
        ("reserved_mask2", C.c_uint64),
        ("empty_digest", C.c_uint8),
        ("reclaim_digest", C.c_uint8),
        ("pow2_buckets", C.c_uint8),
        ("dual_bucket", C.c_uint8),
        ("pad_", C.c_uint8 * 4),
        ("bounds", C.c_void_p),
    ]


_u64 = C.c_uint64
_p = C.c_void_p
_i = C.c_int
_T = C.c_void_p  # hkv_table*

# name -> (restype, argtypes); every symbol include/hkv_c_api.h declares
SIGNATURES = {
    "hkv_options_default": (None, [C.POINTER(Options)]),
    "hkv_last_error": (C.c_char_p, []),
    "hkv_version": (C.c_char_p, []),
    "hkv_table_create": (_i, [C.POINTER(Options), C.POINTER(_T)]),
    "hkv_table_create_with_allocator": (_i, [C.POINTER(Options), _p, C.POINTER(_T)]),
    "hkv_table_destroy": (_i, [_T]),
    "hkv_insert_or_assign": (_i, [_T, _u64, _p, _p, _p, _p, _i, _i]),
    "hkv_insert_or_assign_noalloc": (_i, [_T, _u64, _p, _p, _p, _p, _i]),
    "hkv_insert_and_evict": (_i, [_T, _u64, _p, _p, _p, _p, _p, _p, _p, _p, _i, _i]),
    "hkv_insert_and_evict_count": (_i, [_T, _u64, _p, _p, _p, _p, _p, _p, _p, _i, _i, C.POINTER(_u64)]),
    "hkv_accum_or_assign": (_i, [_T, _u64, _p, _p, _p, _p, _p, _i]),
    "hkv_find_or_insert": (_i, [_T, _u64, _p, _p, _p, _p, _i, _i]),
    "hkv_find_or_insert_ptr": (_i, [_T, _u64, _p, _p, _p, _p, _p, _i, _i]),
    "hkv_find_or_insert_ptr_lock": (_i, [_T, _u64, _p, _p, _p, _p, _p, _p, _i]),
    "hkv_assign": (_i, [_T, _u64, _p, _p, _p, _p, _i]),
    "hkv_assign_scores": (_i, [_T, _u64, _p, _p, _p, _i]),
    "hkv_assign_values": (_i, [_T, _u64, _p, _p, _p, _i]),
    "hkv_find": (_i, [_T, _u64, _p, _p, _p, _p, _p]),
    "hkv_find_missed": (_i, [_T, _u64, _p, _p, _p, _p, _p, _p, _p]),
    "hkv_find_ptr": (_i, [_T, _u64, _p, _p, _p, _p, _p, _i]),
    "hkv_contains": (_i, [_T, _u64, _p, _p, _p]),
    "hkv_erase": (_i, [_T, _u64, _p, _p]),
    "hkv_clear": (_i, [_T, _p]),
    "hkv_lock_keys": (_i, [_T, _u64, _p, _p, _p, _p, _p]),
    "hkv_unlock_keys": (_i, [_T, _u64, _p, _p, _p, _p]),
    "hkv_find_and_update": (_i, [_T, _u64, _p, _p, _p, _p, _p]),
    "hkv_reserve": (_i, [_T, C.c_uint64, _p]),
    "hkv_set_max_capacity": (_i, [_T, C.c_uint64]),
    "hkv_export_batch": (_i, [_T, _u64, _u64, _p, _p, _p, _p, _p]),
    "hkv_export_batch_if": (_i, [_T, _i, _u64, _u64, _u64, _u64, _p, _p, _p, _p, _p]),
    "hkv_size_if": (_i, [_T, _i, _u64, _u64, _p, C.POINTER(_u64)]),
    "hkv_size": (_i, [_T, _p, C.POINTER(_u64)]),
    "hkv_empty": (_i, [_T, _p, C.POINTER(_i)]),
    "hkv_capacity": (_u64, [_T]),
    "hkv_load_factor": (_i, [_T, _p, C.POINTER(C.c_float)]),
    "hkv_dim": (_u64, [_T]),
    "hkv_max_bucket_size": (_u64, [_T]),
    "hkv_bucket_count": (_u64, [_T]),
    "hkv_is_pure_hbm": (_i, [_T]),
    "hkv_set_global_epoch": (_i, [_T, _u64]),
    "hkv_table_get_view": (_i, [_T, C.POINTER(TableView)]),
    "hkv_lock_begin": (_i, [_T, _i, _p]),
    "hkv_lock_end": (_i, [_T, _i, _p]),
    "hkv_set_clock": (_i, [_T, _i, _u64]),
    "hkv_scores_changed": (_i, [_T]),
    "hkv_time_next_kernel": (_i, [C.c_void_p, C.c_void_p]),
}


def load(path=LIB_PATH):
    if not os.path.exists(path):
        raise ImportError(
            f"{path} is missing: the HIP library has not been built. Run "
            "`python -c 'import __graft_entry__ as g; g.build()'` (or "
            "`python hierarchicalkv_amd/build.py lib`) in the repository root.")
    # A process must hold one HIP runtime only.  PyTorch wheels bundle their own
    # libamdhip64 (same soname as the system one); when torch is going to be used
    # for the device buffers it has to be loaded first, so that this library binds
    # to the runtime torch already brought in instead of loading a second one.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    lib = C.CDLL(path)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


lib = load()
