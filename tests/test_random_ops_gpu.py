"""Seeded random sequences of calls against the oracle: whatever the mix of operations and
batch sizes, the GPU table and the oracle must agree after every call (outputs of the call)
and every few calls (the whole resident map).  The order-independence preconditions hold by
construction: keys unique per batch, scores distinct and growing from call to call,
accum_or_assign flags taken from a find just before."""
import numpy as np
import pytest
import torch

import workloads as w
from gpu_util import (DEV, assert_same_table, canonical_evicted, dev, export_table, host_bytes,
                      host_u64, sort_by_key)
from hierarchicalkv_amd import EvictStrategy, HashTable, Predicate, default_options

pytestmark = pytest.mark.gpu


def bytes_of(a):
    return np.ascontiguousarray(a).view(np.uint8).reshape(len(a), -1)


@pytest.mark.parametrize("seed,dim,cap,strategy,hybrid", [
    (1, 4, 1 << 13, EvictStrategy.kCustomized, False),
    (2, 16, 1 << 13, EvictStrategy.kCustomized, False),
    (3, 5, 12345 // 128 * 128 + 128, EvictStrategy.kCustomized, False),
    (4, 64, 1 << 12, EvictStrategy.kCustomized, False),
    (5, 8, 1 << 13, EvictStrategy.kLru, False),       # scores from the deterministic clock
    (6, 32, 1 << 12, EvictStrategy.kEpochLru, False),
    # three quarters of the rows in host memory: the upserts of a batch hold their slots, as the
    # oracle's model of the reference's lock-key and write kernels does; no insert_and_evict there
    (7, 16, 1 << 12, EvictStrategy.kCustomized, True),
    (8, 8, 1 << 13, EvictStrategy.kLru, True),
])
def test_random_call_sequences(oracle, seed, dim, cap, strategy, hybrid):
    o = default_options(init_capacity=cap, max_capacity=cap, max_hbm_for_vectors=cap * dim if hybrid else 1 << 30,
                        dim=dim, evict_strategy=strategy)
    t = HashTable()
    t.init(o)
    assert t.is_pure_hbm() != hybrid
    ot = oracle.OracleTable(o, hybrid=hybrid)
    clocked = strategy != EvictStrategy.kCustomized
    if clocked:
        t.set_clock(1, 1 << 44)
        ot.set_clock(1, 1 << 44)
    if strategy == EvictStrategy.kEpochLru:
        t.set_global_epoch(1)
        ot.set_global_epoch(1)
    rng = np.random.default_rng(1000 + seed)
    universe = w.unique_keys(500 + seed, 0, 3 * cap)
    vb = dim * 4
    seq = 0
    counts = {}
    for step in range(160):
        n = int(rng.choice([1, 7, 64, 65, 500, 1500, 3000]))
        keys = rng.choice(universe, size=n, replace=False)
        if rng.random() < 0.3:  # a reserved key now and then
            keys[rng.integers(0, n)] = np.uint64((1 << 64) - 1 - int(rng.integers(0, 4)))
        vals = rng.random((n, dim), dtype=np.float32)
        seq += 1
        sc = None if clocked else w.monotone_scores(seq, n, seed=seed)
        if strategy == EvictStrategy.kEpochLru and step % 16 == 15:
            t.set_global_epoch(1 + step // 16)
            ot.set_global_epoch(1 + step // 16)
        op = rng.choice(["insert_or_assign", "find", "find_or_insert", "insert_and_evict", "assign",
                         "accum_or_assign", "erase", "contains", "export_if"],
                        p=[0.35, 0.12, 0.17, 0.0, 0.08, 0.1, 0.08, 0.05, 0.05] if hybrid else
                        [0.25, 0.12, 0.12, 0.15, 0.08, 0.1, 0.08, 0.05, 0.05])
        counts[op] = counts.get(op, 0) + 1
        if op in ("find_or_insert", "accum_or_assign"):
            # A resident key of the batch can be pushed out by a new key of the same batch before
            # its own turn; what it then reads back (or whether its delta is dropped) depends on
            # the order, so these two calls get batches that are all resident or all new.
            present = ot.contains(keys)
            keep = present if (rng.random() < 0.5 and present.sum() > 0) else ~present
            if keep.sum() == 0:
                keep = ~keep
            keys, vals = keys[keep], vals[keep]
            sc = None if sc is None else sc[keep]
            n = len(keys)
        dk, dv, ds = dev(keys), dev(vals), dev(sc)
        if op == "insert_or_assign":
            t.insert_or_assign(n, dk, dv, ds)
            ot.insert_or_assign(keys, bytes_of(vals), sc)
        elif op == "find":
            out = torch.zeros(n, dim, dtype=torch.float32, device=DEV)
            f = torch.zeros(n, dtype=torch.bool, device=DEV)
            s = torch.zeros(n, dtype=torch.int64, device=DEV)
            t.find(n, dk, out, f, s)
            torch.cuda.synchronize()
            ov, of, os_ = ot.find(keys)
            gf = f.cpu().numpy()
            assert np.array_equal(gf, of), (step, op)
            assert np.array_equal(bytes_of(out.cpu().numpy())[of], ov[of]), (step, op)
            assert np.array_equal(host_u64(s)[of], os_[of]), (step, op)
        elif op == "find_or_insert":
            io = dv.clone()
            t.find_or_insert(n, dk, io, ds)
            torch.cuda.synchronize()
            ovals = bytes_of(vals).copy()
            ot.find_or_insert(keys, ovals, sc)
            assert np.array_equal(bytes_of(io.cpu().numpy()), ovals), (step, op)
        elif op == "insert_and_evict":
            ek = torch.zeros(n, dtype=torch.int64, device=DEV)
            ev = torch.zeros(n, dim, dtype=torch.float32, device=DEV)
            es = torch.zeros(n, dtype=torch.int64, device=DEV)
            c = t.insert_and_evict(n, dk, dv, ds, ek, ev, es)
            oek, oev, oes = ot.insert_and_evict(keys, bytes_of(vals), sc)
            gk, _, _ = export_table(t, vb)
            a = canonical_evicted(host_u64(ek[:c]), host_bytes(ev[:c], c, vb), host_u64(es[:c]), gk)
            b = canonical_evicted(oek, oev, oes, gk)
            assert all(np.array_equal(x, y) for x, y in zip(a, b)), (step, op)
        elif op == "assign":
            t.assign(n, dk, dv, ds)
            ot.assign(keys, bytes_of(vals), sc)
        elif op == "accum_or_assign":
            f = torch.zeros(n, dtype=torch.bool, device=DEV)
            t.contains(n, dk, f)
            torch.cuda.synchronize()
            flags = f.cpu().numpy()
            assert np.array_equal(flags, ot.contains(keys)), (step, op)
            delta = (rng.integers(-8, 8, (n, dim)) * 0.25).astype(np.float32)  # exact in fp32 sums
            t.accum_or_assign(n, dk, dev(delta), f, ds)
            ot.accum_or_assign(keys, bytes_of(delta), flags.astype(np.uint8), sc)
        elif op == "erase":
            t.erase(n, dk)
            ot.erase(keys)
        elif op == "contains":
            f = torch.zeros(n, dtype=torch.bool, device=DEV)
            t.contains(n, dk, f)
            torch.cuda.synchronize()
            assert np.array_equal(f.cpu().numpy(), ot.contains(keys)), (step, op)
        elif op == "export_if":
            thr = int(w.monotone_scores(max(1, seq - 5), 1, seed=seed)[0])
            if clocked:  # somewhere inside the range of scores the clock has handed out
                _, _, alls = ot.export_all()
                thr = int(np.median(alls)) if len(alls) else 0
            got = sort_by_key(*export_table(t, vb, Predicate.kScoreGe, 0, thr, chunk=1000))
            want = sort_by_key(*ot.export_batch_if(int(Predicate.kScoreGe), 0, thr))
            assert all(np.array_equal(x, y) for x, y in zip(got, want)), (step, op)
            assert t.size_if(Predicate.kScoreGe, 0, thr) == len(want[0])
        assert t.size() == ot.size(), (step, op)
        if step % 10 == 9:
            assert_same_table(t, ot, vb)
    assert_same_table(t, ot, vb)
    assert len(counts) >= (6 if hybrid else 7)
    t.close()
    ot.close()
