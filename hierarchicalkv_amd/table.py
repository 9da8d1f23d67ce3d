"""Host-side mirror of nv::merlin::HashTable over the C ABI, for Python callers.

Method names, argument order and defaults follow the reference class
(include/merlin_hashtable.cuh:187-885); torch is used only to own device
buffers and streams.  Every method takes raw device pointers (ints) or torch
CUDA tensors and forwards them to libhkv.so unchanged.
"""
import ctypes as C

from . import _capi
from ._capi import Options, TableView, lib


class MerlinException(RuntimeError):
    """MERLIN_CHECK failure (debug.hpp:50-72)."""


class HipException(RuntimeError):
    """HIP runtime failure (CudaException, debug.hpp:27-48)."""


class EvictStrategy:
    """nv::merlin::EvictStrategy (merlin_hashtable.cuh:79-87)."""
    kLru = 0
    kLfu = 1
    kEpochLru = 2
    kEpochLfu = 3
    kCustomized = 4


class ValueKind:
    kBytes = 0
    kF32 = 1
    kF64 = 2
    kI32 = 3
    kI64 = 4
    kI8 = 5
    kI16 = 6


class Predicate:
    kAlways = 0
    kScoreLt = 1
    kScoreLe = 2
    kScoreGt = 3
    kScoreGe = 4
    kKeyHigh16EqAndScoreLt = 5


def _raise(rc):
    msg = lib.hkv_last_error().decode()
    if rc == _capi.HKV_ERROR_CHECK:
        raise MerlinException(msg)
    if rc == _capi.HKV_ERROR_HIP:
        raise HipException(msg)
    if rc == _capi.HKV_ERROR_ARGUMENT:
        raise ValueError(msg)
    if rc == _capi.HKV_ERROR_UNSUPPORTED:
        raise NotImplementedError(msg)
    raise RuntimeError(msg)


def _check(rc):
    if rc != _capi.HKV_SUCCESS:
        _raise(rc)


def _ptr(x):
    """Device address of a torch tensor, an int, or None."""
    if x is None:
        return None
    if isinstance(x, int):
        return x
    return x.data_ptr()


def _stream(s):
    if s is None:
        import torch
        return torch.cuda.current_stream().cuda_stream
    if isinstance(s, int):
        return s
    return s.cuda_stream


def default_options(**kw):
    o = Options()
    lib.hkv_options_default(C.byref(o))
    for k, v in kw.items():
        if not hasattr(o, k):
            raise AttributeError(f"hkv_options has no field {k}")
        setattr(o, k, v)
    return o


class HashTable:
    """HashTable<K=uint64, V, S=uint64, Strategy> over libhkv.so."""

    def __init__(self):
        self._h = None
        self.options = None

    def init(self, options):
        if self._h is not None:
            return
        h = C.c_void_p()
        _check(lib.hkv_table_create(C.byref(options), C.byref(h)))
        self._h = h
        self.options = options

    def close(self):
        if self._h is not None:
            lib.hkv_table_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # -- writers ---------------------------------------------------------------
    def insert_or_assign(self, n, keys, values, scores=None, stream=None,
                         unique_key=True, ignore_evict_strategy=False):
        _check(lib.hkv_insert_or_assign(self._h, n, _ptr(keys), _ptr(values), _ptr(scores),
                                        _stream(stream), int(unique_key), int(ignore_evict_strategy)))

    def insert_or_assign_noalloc(self, n, keys, values, scores=None, stream=None,
                                 ignore_evict_strategy=False):
        """insert_or_assign on the library's static scratch area: allocates nothing."""
        _check(lib.hkv_insert_or_assign_noalloc(self._h, n, _ptr(keys), _ptr(values), _ptr(scores),
                                                _stream(stream), int(ignore_evict_strategy)))

    def insert_and_evict(self, n, keys, values, scores, evicted_keys, evicted_values,
                         evicted_scores, d_evicted_counter=None, stream=None,
                         unique_key=True, ignore_evict_strategy=False):
        """With d_evicted_counter=None this is the count-returning overload."""
        if d_evicted_counter is None:
            out = C.c_uint64(0)
            _check(lib.hkv_insert_and_evict_count(
                self._h, n, _ptr(keys), _ptr(values), _ptr(scores), _ptr(evicted_keys),
                _ptr(evicted_values), _ptr(evicted_scores), _stream(stream),
                int(unique_key), int(ignore_evict_strategy), C.byref(out)))
            return out.value
        _check(lib.hkv_insert_and_evict(
            self._h, n, _ptr(keys), _ptr(values), _ptr(scores), _ptr(evicted_keys),
            _ptr(evicted_values), _ptr(evicted_scores), _ptr(d_evicted_counter),
            _stream(stream), int(unique_key), int(ignore_evict_strategy)))
        return None

    def accum_or_assign(self, n, keys, value_or_deltas, accum_or_assigns, scores=None,
                        stream=None, ignore_evict_strategy=False):
        _check(lib.hkv_accum_or_assign(self._h, n, _ptr(keys), _ptr(value_or_deltas),
                                       _ptr(accum_or_assigns), _ptr(scores), _stream(stream),
                                       int(ignore_evict_strategy)))

    def find_or_insert(self, n, keys, values, scores=None, stream=None, unique_key=True,
                       ignore_evict_strategy=False):
        _check(lib.hkv_find_or_insert(self._h, n, _ptr(keys), _ptr(values), _ptr(scores),
                                      _stream(stream), int(unique_key), int(ignore_evict_strategy)))

    def find_or_insert_ptr(self, n, keys, value_ptrs, founds, scores=None, stream=None,
                           unique_key=True, ignore_evict_strategy=False, locked_key_ptrs=None):
        if locked_key_ptrs is not None:
            if not unique_key:
                raise ValueError("unique_key should be true and max_bucket_size should be larger.")
            _check(lib.hkv_find_or_insert_ptr_lock(self._h, n, _ptr(keys), _ptr(value_ptrs),
                                                   _ptr(founds), _ptr(scores), _ptr(locked_key_ptrs),
                                                   _stream(stream), int(ignore_evict_strategy)))
            return
        _check(lib.hkv_find_or_insert_ptr(self._h, n, _ptr(keys), _ptr(value_ptrs), _ptr(founds),
                                          _ptr(scores), _stream(stream), int(unique_key),
                                          int(ignore_evict_strategy)))

    def assign(self, n, keys, values, scores=None, stream=None, unique_key=True):
        _check(lib.hkv_assign(self._h, n, _ptr(keys), _ptr(values), _ptr(scores),
                              _stream(stream), int(unique_key)))

    def assign_scores(self, n, keys, scores=None, stream=None, unique_key=True):
        _check(lib.hkv_assign_scores(self._h, n, _ptr(keys), _ptr(scores), _stream(stream),
                                     int(unique_key)))

    def assign_values(self, n, keys, values, stream=None, unique_key=True):
        _check(lib.hkv_assign_values(self._h, n, _ptr(keys), _ptr(values), _stream(stream),
                                     int(unique_key)))

    def lock_keys(self, n, keys, locked_key_ptrs, success=None, stream=None, scores=None):
        _check(lib.hkv_lock_keys(self._h, n, _ptr(keys), _ptr(locked_key_ptrs), _ptr(success),
                                 _ptr(scores), _stream(stream)))

    def unlock_keys(self, n, locked_key_ptrs, keys, success=None, stream=None):
        _check(lib.hkv_unlock_keys(self._h, n, _ptr(locked_key_ptrs), _ptr(keys), _ptr(success),
                                   _stream(stream)))

    def find_and_update(self, n, keys, value_ptrs, founds, scores=None, stream=None, unique_key=True):
        _check(lib.hkv_find_and_update(self._h, n, _ptr(keys), _ptr(value_ptrs), _ptr(founds),
                                       _ptr(scores), _stream(stream)))

    def erase(self, n, keys, stream=None):
        _check(lib.hkv_erase(self._h, n, _ptr(keys), _stream(stream)))

    def clear(self, stream=None):
        _check(lib.hkv_clear(self._h, _stream(stream)))

    def set_max_capacity(self, new_max_capacity):
        _check(lib.hkv_set_max_capacity(self._h, new_max_capacity))

    def reserve(self, new_capacity, stream=None):
        _check(lib.hkv_reserve(self._h, new_capacity, _stream(stream)))

    # -- readers ---------------------------------------------------------------
    def find(self, n, keys, values, founds, scores=None, stream=None):
        _check(lib.hkv_find(self._h, n, _ptr(keys), _ptr(values), _ptr(founds), _ptr(scores),
                            _stream(stream)))

    def find_missed(self, n, keys, values, missed_keys, missed_indices, missed_size,
                    scores=None, stream=None):
        _check(lib.hkv_find_missed(self._h, n, _ptr(keys), _ptr(values), _ptr(missed_keys),
                                   _ptr(missed_indices), _ptr(missed_size), _ptr(scores),
                                   _stream(stream)))

    def find_ptr(self, n, keys, value_ptrs, founds, scores=None, stream=None, unique_key=True):
        _check(lib.hkv_find_ptr(self._h, n, _ptr(keys), _ptr(value_ptrs), _ptr(founds),
                                _ptr(scores), _stream(stream), int(unique_key)))

    def contains(self, n, keys, founds, stream=None):
        _check(lib.hkv_contains(self._h, n, _ptr(keys), _ptr(founds), _stream(stream)))

    def export_batch(self, n, offset, d_counter, keys, values, scores=None, stream=None):
        _check(lib.hkv_export_batch(self._h, n, offset, _ptr(d_counter), _ptr(keys), _ptr(values),
                                    _ptr(scores), _stream(stream)))

    def export_batch_if(self, predicate, pattern, threshold, n, offset, d_counter, keys, values,
                        scores=None, stream=None):
        _check(lib.hkv_export_batch_if(self._h, predicate, pattern, threshold, n, offset,
                                       _ptr(d_counter), _ptr(keys), _ptr(values), _ptr(scores),
                                       _stream(stream)))

    def size_if(self, predicate, pattern, threshold, stream=None):
        out = C.c_uint64(0)
        _check(lib.hkv_size_if(self._h, predicate, pattern, threshold, _stream(stream), C.byref(out)))
        return out.value

    def size(self, stream=None):
        out = C.c_uint64(0)
        _check(lib.hkv_size(self._h, _stream(stream), C.byref(out)))
        return out.value

    def empty(self, stream=None):
        out = C.c_int(0)
        _check(lib.hkv_empty(self._h, _stream(stream), C.byref(out)))
        return bool(out.value)

    def load_factor(self, stream=None):
        out = C.c_float(0)
        _check(lib.hkv_load_factor(self._h, _stream(stream), C.byref(out)))
        return out.value

    def capacity(self):
        return lib.hkv_capacity(self._h)

    def dim(self):
        return lib.hkv_dim(self._h)

    def max_bucket_size(self):
        return lib.hkv_max_bucket_size(self._h)

    def bucket_count(self):
        return lib.hkv_bucket_count(self._h)

    def is_pure_hbm(self):
        return bool(lib.hkv_is_pure_hbm(self._h))

    def set_global_epoch(self, epoch):
        _check(lib.hkv_set_global_epoch(self._h, epoch))

    def set_clock(self, mode, base=0):
        _check(lib.hkv_set_clock(self._h, mode, base))

    def view(self):
        v = TableView()
        _check(lib.hkv_table_get_view(self._h, C.byref(v)))
        return v
