"""ctypes binding of the CPU oracle (oracle/libhkv_oracle.so) for the tests.

Test infrastructure: only tests, the smoke test and the benchmark's CPU
baseline may import this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
LIB = os.path.join(ORACLE_DIR, "libhkv_oracle.so")

from hierarchicalkv_amd._capi import Options  # same struct layout (hkv_options)

if not os.path.exists(LIB):
    subprocess.check_call(["make", "-C", ORACLE_DIR, "libhkv_oracle.so"])
_lib = C.CDLL(LIB)

_u64 = C.c_uint64
_p = C.c_void_p
_i = C.c_int
_SIG = {
    "hkvo_murmur3_fmix64": (_u64, [_u64]),
    "hkvo_reserved_keys": (_i, [_i, C.POINTER(_u64)]),
    "hkvo_locate": (None, [_u64, _u64, C.POINTER(_u64), C.POINTER(C.c_uint32), C.POINTER(C.c_uint8)]),
    "hkvo_locate_dual": (None, [_u64, _u64, C.POINTER(_u64), C.POINTER(C.c_uint32), C.POINTER(C.c_uint8)]),
    "hkvo_create": (_i, [C.POINTER(Options), _i, C.POINTER(_p)]),
    "hkvo_destroy": (None, [_p]),
    "hkvo_last_error": (C.c_char_p, []),
    "hkvo_set_global_epoch": (_i, [_p, _u64]),
    "hkvo_set_clock": (_i, [_p, _i, _u64]),
    "hkvo_insert_or_assign": (_i, [_p, _u64, _p, _p, _p, _i]),
    "hkvo_insert_and_evict": (_i, [_p, _u64, _p, _p, _p, _p, _p, _p, _p, _i]),
    "hkvo_accum_or_assign": (_i, [_p, _u64, _p, _p, _p, _p, _i]),
    "hkvo_find_or_insert": (_i, [_p, _u64, _p, _p, _p, _i]),
    "hkvo_find_or_insert_slot": (_i, [_p, _u64, _p, _p, _p, _p, _i]),
    "hkvo_assign": (_i, [_p, _u64, _p, _p, _p]),
    "hkvo_assign_scores": (_i, [_p, _u64, _p, _p]),
    "hkvo_assign_values": (_i, [_p, _u64, _p, _p]),
    "hkvo_find": (_i, [_p, _u64, _p, _p, _p, _p]),
    "hkvo_find_slot": (_i, [_p, _u64, _p, _p, _p, _p]),
    "hkvo_contains": (_i, [_p, _u64, _p, _p]),
    "hkvo_lock_keys": (_i, [_p, _u64, _p, _p, _p, _p]),
    "hkvo_unlock_keys": (_i, [_p, _u64, _p, _p, _p]),
    "hkvo_find_and_update": (_i, [_p, _u64, _p, _p, _p, _p]),
    "hkvo_erase": (_i, [_p, _u64, _p]),
    "hkvo_clear": (_i, [_p]),
    "hkvo_reserve": (_i, [_p, _u64]),
    "hkvo_set_max_capacity": (_i, [_p, _u64]),
    "hkvo_export_batch_if": (_i, [_p, _i, _u64, _u64, _u64, _u64, _p, _p, _p, _p]),
    "hkvo_size_if": (_u64, [_p, _i, _u64, _u64]),
    "hkvo_size": (_u64, [_p]),
    "hkvo_capacity": (_u64, [_p]),
    "hkvo_bucket_count": (_u64, [_p]),
    "hkvo_bucket_size": (C.c_int32, [_p, _u64]),
    "hkvo_find_mt": (_i, [_p, _u64, _p, _p, _p, _p, _i]),
    "hkvo_insert_or_assign_mt": (_i, [_p, _u64, _p, _p, _p, _i, _i]),
    "hkvo_online_cores": (_i, []),
}
for _n, (_r, _a) in _SIG.items():
    _f = getattr(_lib, _n)
    _f.restype = _r
    _f.argtypes = _a


class OracleError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(msg)
        self.code = code


def _check(rc):
    if rc != 0:
        raise OracleError(rc, _lib.hkvo_last_error().decode())


def _np(a):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data


def fmix64(k):
    return _lib.hkvo_murmur3_fmix64(k)


def reserved_keys(bit):
    out = (_u64 * 7)()
    rc = _lib.hkvo_reserved_keys(bit, out)
    if rc != 0:
        raise ValueError(bit)
    return list(out)


def locate(key, buckets_num):
    b = _u64()
    s = C.c_uint32()
    d = C.c_uint8()
    _lib.hkvo_locate(key, buckets_num, C.byref(b), C.byref(s), C.byref(d))
    return b.value, s.value, d.value


def locate_dual(key, buckets_num):
    """((b1, b2), (start1, start2), digest) of a key in dual-bucket mode."""
    b = (_u64 * 2)()
    s = (C.c_uint32 * 2)()
    d = C.c_uint8()
    _lib.hkvo_locate_dual(key, buckets_num, b, s, C.byref(d))
    return (b[0], b[1]), (s[0], s[1]), d.value


def online_cores():
    return _lib.hkvo_online_cores()


class OracleTable:
    """Host table with the reference's semantics; numpy arrays in and out."""

    def __init__(self, options, hybrid=False):
        self._h = None
        h = _p()
        _check(_lib.hkvo_create(C.byref(options), int(hybrid), C.byref(h)))
        self._h = h
        self.dim = options.dim
        self.vb = options.dim * options.value_size

    def close(self):
        if self._h:
            _lib.hkvo_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def set_global_epoch(self, e):
        _check(_lib.hkvo_set_global_epoch(self._h, e))

    def set_clock(self, mode, base=0):
        _check(_lib.hkvo_set_clock(self._h, mode, base))

    def insert_or_assign(self, keys, values, scores=None, ignore=False):
        _check(_lib.hkvo_insert_or_assign(self._h, len(keys), _np(keys), _np(values), _np(scores), int(ignore)))

    def insert_or_assign_mt(self, keys, values, scores=None, ignore=False, threads=0):
        _check(_lib.hkvo_insert_or_assign_mt(self._h, len(keys), _np(keys), _np(values), _np(scores),
                                             int(ignore), threads))

    def insert_and_evict(self, keys, values, scores=None, ignore=False):
        n = len(keys)
        ek = np.zeros(n, np.uint64)
        ev = np.zeros((n, self.vb), np.uint8)
        es = np.zeros(n, np.uint64)
        cnt = np.zeros(1, np.uint64)
        _check(_lib.hkvo_insert_and_evict(self._h, n, _np(keys), _np(values), _np(scores), _np(ek), _np(ev),
                                          _np(es), _np(cnt), int(ignore)))
        c = int(cnt[0])
        return ek[:c], ev[:c], es[:c]

    def accum_or_assign(self, keys, values, flags, scores=None, ignore=False):
        _check(_lib.hkvo_accum_or_assign(self._h, len(keys), _np(keys), _np(values), _np(flags), _np(scores),
                                         int(ignore)))

    def find_or_insert(self, keys, values, scores=None, ignore=False):
        _check(_lib.hkvo_find_or_insert(self._h, len(keys), _np(keys), _np(values), _np(scores), int(ignore)))

    def find_or_insert_slot(self, keys, scores=None, ignore=False):
        n = len(keys)
        slots = np.full(n, 0x5555555555555555, np.uint64)
        founds = np.full(n, 2, np.uint8)
        _check(_lib.hkvo_find_or_insert_slot(self._h, n, _np(keys), _np(slots), _np(founds), _np(scores), int(ignore)))
        return slots, founds

    def assign(self, keys, values, scores=None):
        _check(_lib.hkvo_assign(self._h, len(keys), _np(keys), _np(values), _np(scores)))

    def assign_scores(self, keys, scores=None):
        _check(_lib.hkvo_assign_scores(self._h, len(keys), _np(keys), _np(scores)))

    def assign_values(self, keys, values):
        _check(_lib.hkvo_assign_values(self._h, len(keys), _np(keys), _np(values)))

    def find(self, keys, values=None, want_scores=True, threads=None):
        """values: (n, vb) uint8 array that is updated in place for hits."""
        n = len(keys)
        if values is None:
            values = np.zeros((n, self.vb), np.uint8)
        founds = np.zeros(n, np.uint8)
        scores = np.zeros(n, np.uint64) if want_scores else None
        if threads is None:
            _check(_lib.hkvo_find(self._h, n, _np(keys), _np(values), _np(founds), _np(scores)))
        else:
            _check(_lib.hkvo_find_mt(self._h, n, _np(keys), _np(values), _np(founds), _np(scores), threads))
        return values, founds.astype(bool), scores

    def find_slot(self, keys):
        n = len(keys)
        slots = np.zeros(n, np.uint64)
        founds = np.zeros(n, np.uint8)
        scores = np.zeros(n, np.uint64)
        _check(_lib.hkvo_find_slot(self._h, n, _np(keys), _np(slots), _np(founds), _np(scores)))
        return slots, founds.astype(bool), scores

    def lock_keys(self, keys, scores=None):
        n = len(keys)
        slots = np.zeros(n, np.uint64)
        ok = np.zeros(n, np.uint8)
        _check(_lib.hkvo_lock_keys(self._h, n, _np(keys), _np(slots), _np(ok), _np(scores)))
        return slots, ok.astype(bool)

    def unlock_keys(self, slots, keys):
        ok = np.zeros(len(keys), np.uint8)
        _check(_lib.hkvo_unlock_keys(self._h, len(keys), _np(slots), _np(keys), _np(ok)))
        return ok.astype(bool)

    def find_and_update(self, keys, scores=None):
        """scores: in/out array or None; returns (slots, founds, scores)."""
        n = len(keys)
        slots = np.zeros(n, np.uint64)
        founds = np.zeros(n, np.uint8)
        sc = None if scores is None else np.ascontiguousarray(scores).copy()
        _check(_lib.hkvo_find_and_update(self._h, n, _np(keys), _np(slots), _np(founds), _np(sc)))
        return slots, founds.astype(bool), sc

    def contains(self, keys):
        founds = np.zeros(len(keys), np.uint8)
        _check(_lib.hkvo_contains(self._h, len(keys), _np(keys), _np(founds)))
        return founds.astype(bool)

    def erase(self, keys):
        _check(_lib.hkvo_erase(self._h, len(keys), _np(keys)))

    def clear(self):
        _check(_lib.hkvo_clear(self._h))

    def reserve(self, new_capacity):
        _check(_lib.hkvo_reserve(self._h, new_capacity))

    def set_max_capacity(self, new_max_capacity):
        _check(_lib.hkvo_set_max_capacity(self._h, new_max_capacity))

    def export_batch_if(self, pred=0, pattern=0, threshold=0, n=None, offset=0):
        cap = self.capacity()
        if n is None:
            n = cap
        m = min(n, max(cap - offset, 0)) if offset < cap else 0
        keys = np.zeros(m, np.uint64)
        values = np.zeros((m, self.vb), np.uint8)
        scores = np.zeros(m, np.uint64)
        cnt = np.zeros(1, np.uint64)
        _check(_lib.hkvo_export_batch_if(self._h, pred, pattern, threshold, n, offset, _np(cnt), _np(keys),
                                         _np(values), _np(scores)))
        c = int(cnt[0])
        return keys[:c], values[:c], scores[:c]

    def export_all(self):
        return self.export_batch_if()

    def size_if(self, pred, pattern, threshold):
        return _lib.hkvo_size_if(self._h, pred, pattern, threshold)

    def size(self):
        return _lib.hkvo_size(self._h)

    def capacity(self):
        return _lib.hkvo_capacity(self._h)

    def bucket_count(self):
        return _lib.hkvo_bucket_count(self._h)

    def bucket_size(self, b):
        return _lib.hkvo_bucket_size(self._h, b)
