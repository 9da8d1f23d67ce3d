"""Helpers for the GPU parity tests: device buffers, raw device reads, table
export and table-vs-oracle comparison.  Everything goes through the C ABI."""
import ctypes as C

import numpy as np
import torch

from hierarchicalkv_amd import HashTable, Predicate

DEV = "cuda:0"
_hip = None


def hip():
    global _hip
    if _hip is None:
        _hip = C.CDLL("libamdhip64.so")
        _hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        _hip.hipMemcpy.restype = C.c_int
    return _hip


def read_device(ptr, nbytes):
    """Copy nbytes from a raw device (or mapped host) address to a numpy array."""
    out = np.empty(nbytes, np.uint8)
    rc = hip().hipMemcpy(out.ctypes.data, C.c_void_p(ptr), nbytes, 2)  # hipMemcpyDeviceToHost
    assert rc == 0, rc
    return out


def dev(a):
    """numpy -> device tensor (uint64 travels as int64 bit patterns)."""
    if a is None:
        return None
    if a.dtype == np.uint64:
        a = a.view(np.int64)
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def host_u64(t):
    return t.cpu().numpy().view(np.uint64)


def host_bytes(t, n, vb):
    return t.cpu().numpy().view(np.uint8).reshape(n, vb)


def export_table(table: HashTable, vb, pred=Predicate.kAlways, pattern=0, threshold=0, chunk=1 << 20):
    """All (key, value bytes, score) entries matching pred, via export_batch_if in windows."""
    cap = table.capacity()
    keys, vals, scores = [], [], []
    dk = torch.zeros(chunk, dtype=torch.int64, device=DEV)
    dv = torch.zeros(chunk * vb, dtype=torch.uint8, device=DEV)
    ds = torch.zeros(chunk, dtype=torch.int64, device=DEV)
    dc = torch.zeros(1, dtype=torch.int64, device=DEV)
    for off in range(0, cap, chunk):
        table.export_batch_if(pred, pattern, threshold, chunk, off, dc, dk, dv, ds)
        torch.cuda.synchronize()
        c = int(dc.item())
        keys.append(host_u64(dk[:c]).copy())
        vals.append(dv[:c * vb].cpu().numpy().reshape(c, vb).copy())
        scores.append(host_u64(ds[:c]).copy())
    return np.concatenate(keys), np.concatenate(vals), np.concatenate(scores)


def sort_by_key(keys, vals, scores):
    o = np.argsort(keys, kind="stable")
    return keys[o], vals[o], scores[o]


def assert_same_table(table, oracle, vb):
    """Resident map (key -> value bytes, score) and size, bit-exact."""
    gk, gv, gs = sort_by_key(*export_table(table, vb))
    ok, ov, os_ = sort_by_key(*oracle.export_all())
    assert len(gk) == len(ok), (len(gk), len(ok))
    assert len(np.unique(gk)) == len(gk), "duplicate keys in the GPU table"
    assert (gk == ok).all()
    assert (gs == os_).all()
    assert (gv == ov).all()
    assert table.size() == oracle.size() == len(gk)


def canonical_evicted(ek, ev, es, resident_keys):
    """Evicted entries whose key is not resident afterwards, sorted by key."""
    keep = ~np.isin(ek, resident_keys)
    return sort_by_key(ek[keep], ev[keep], es[keep])
