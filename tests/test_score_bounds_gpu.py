"""The score bounds of LRU tables (hkv_table_view::bounds): for every line of 16 slots a value that
is not above any score in the line, which the LRU upserts use to find a bucket's lowest score from
one or two of its eight score lines.  Checked here:
  * the invariant itself, read back from device memory after mixed call sequences, on the
    deterministic and on the hardware clock (a bound above a score would send an eviction to the
    wrong slot sooner or later);
  * that erase and the calls which may lower scores (upserts with ignore_evict_strategy,
    set_clock) leave the bounds right;
  * parity with the oracle through all of this (deterministic clock), which is the parity of the
    bounded search with the full scan: the oracle scans all 128 scores."""
import numpy as np
import pytest
import torch

import workloads as w
from gpu_util import DEV, assert_same_table, dev, read_device
from hierarchicalkv_amd import EvictStrategy, HashTable, default_options

import os

pytestmark = [pytest.mark.gpu,
              pytest.mark.skipif(os.environ.get("HKV_SCORE_BOUNDS") == "0", reason="score bounds switched off")]


def bytes_of(a):
    return np.ascontiguousarray(a).view(np.uint8).reshape(len(a), -1)


def bounds_hold(t):
    """bound[line] <= the score of every key (or tombstone) of the line, for all lines of the table.
    A free slot does not count: it gets a score of the time when it is taken."""
    torch.cuda.synchronize()
    v = t.view()
    cap = v.capacity
    scores = read_device(v.scores, cap * 8).view(np.uint64).reshape(cap // 16, 16).copy()
    keys = read_device(v.keys, cap * 8).view(np.uint64).reshape(cap // 16, 16)
    bounds = read_device(v.bounds, cap // 16 * 8).view(np.uint64)
    scores[keys == np.uint64(v.empty_key)] = np.uint64((1 << 64) - 1)
    bad = np.flatnonzero(bounds > scores.min(axis=1))
    return len(bad) == 0, bad[:5], int((bounds > 0).sum())


def make(cap, dim, **kw):
    o = default_options(init_capacity=cap, max_capacity=cap, max_hbm_for_vectors=1 << 30, dim=dim,
                        evict_strategy=EvictStrategy.kLru, **kw)
    t = HashTable()
    t.init(o)
    return t, o


@pytest.mark.parametrize("clock", ["deterministic", "hardware"])
def test_bounds_stay_below_the_scores(oracle, clock):
    cap, dim = 1 << 13, 8
    t, o = make(cap, dim)
    ot = oracle.OracleTable(o)
    det = clock == "deterministic"
    if det:
        t.set_clock(1, 1 << 44)
        ot.set_clock(1, 1 << 44)
    rng = np.random.default_rng(77)
    universe = w.unique_keys(610, 0, 4 * cap)
    tight = 0
    for step in range(60):
        n = int(rng.choice([64, 700, 3000]))
        keys = rng.choice(universe, size=n, replace=False)
        vals = rng.random((n, dim), dtype=np.float32)
        op = rng.choice(["insert_or_assign", "find_or_insert", "insert_and_evict", "assign", "erase"],
                        p=[0.4, 0.15, 0.2, 0.1, 0.15])
        if op == "find_or_insert":  # all resident or all new: see test_random_ops_gpu.py
            present = ot.contains(keys) if det else np.ones(n, bool)
            keep = present if present.sum() else ~present
            keys, vals = keys[keep], vals[keep]
            n = len(keys)
        dk, dv = dev(keys), dev(vals)
        if op == "insert_or_assign":
            t.insert_or_assign(n, dk, dv)
            ot.insert_or_assign(keys, bytes_of(vals), None)
        elif op == "find_or_insert":
            t.find_or_insert(n, dk, dv.clone())
            ot.find_or_insert(keys, bytes_of(vals).copy(), None)
        elif op == "insert_and_evict":
            ek = torch.zeros(n, dtype=torch.int64, device=DEV)
            ev = torch.zeros(n, dim, dtype=torch.float32, device=DEV)
            t.insert_and_evict(n, dk, dv, None, ek, ev, None)
            ot.insert_and_evict(keys, bytes_of(vals), None)
        elif op == "assign":
            t.assign(n, dk, dv)
            ot.assign(keys, bytes_of(vals), None)
        else:
            t.erase(n, dk)
            ot.erase(keys)
        ok, bad, n_tight = bounds_hold(t)
        assert ok, (step, op, bad)
        tight = max(tight, n_tight)
        if det:
            assert t.size() == ot.size(), (step, op)
            if step % 10 == 9:
                assert_same_table(t, ot, dim * 4)
    assert tight > cap // 16 // 4  # the bounds are in use, not all zero
    if det:
        assert_same_table(t, ot, dim * 4)
    t.close()


def test_scores_from_outside_the_clock(oracle):
    """An upsert with ignore_evict_strategy (what load() uses) writes the caller's scores into an
    LRU table, lower than what is there; the clock can be set back.  Evictions afterwards must
    still take the lowest score of the bucket."""
    cap, dim = 1 << 12, 4
    t, o = make(cap, dim)
    ot = oracle.OracleTable(o)
    t.set_clock(1, 1 << 44)
    ot.set_clock(1, 1 << 44)
    keys = w.unique_keys(620, 0, 8 * cap)
    for b in range(6):  # fill and evict: the bounds tighten
        k = keys[b * 2000:(b + 1) * 2000]
        v = w.values_from_keys(k, dim)
        t.insert_or_assign(len(k), dev(k), dev(v))
        ot.insert_or_assign(k, bytes_of(v), None)
    assert bounds_hold(t)[0]
    # caller's scores, far below the clock's
    k = keys[500:2500]
    v = w.uniform_values(621, 0, len(k), dim)
    sc = np.arange(1, len(k) + 1, dtype=np.uint64)
    t.insert_or_assign(len(k), dev(k), dev(v), dev(sc), ignore_evict_strategy=True)
    ot.insert_or_assign(k, bytes_of(v), sc, ignore=True)
    assert_same_table(t, ot, dim * 4)
    # the next clocked upserts evict those low scores first
    for b in range(6, 9):
        k = keys[b * 2000:(b + 1) * 2000]
        v = w.values_from_keys(k, dim)
        t.insert_or_assign(len(k), dev(k), dev(v))
        ot.insert_or_assign(k, bytes_of(v), None)
        assert bounds_hold(t)[0]
        assert_same_table(t, ot, dim * 4)
    # the clock goes back: new scores below the old ones
    t.set_clock(1, 1 << 30)
    ot.set_clock(1, 1 << 30)
    for b in range(9, 12):
        k = keys[18000 + (b - 9) * 1000:18000 + (b - 8) * 1000]
        v = w.values_from_keys(k, dim)
        t.insert_or_assign(len(k), dev(k), dev(v))
        ot.insert_or_assign(k, bytes_of(v), None)
        assert bounds_hold(t)[0]
        assert_same_table(t, ot, dim * 4)
    t.close()
