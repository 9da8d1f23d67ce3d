"""hkv_insert_or_assign_noalloc (the two-phase insert_or_assign on the library's static scratch
array, for callers that must not allocate) against hkv_insert_or_assign, through the C ABI:
the same batches go into twin tables, one per entry point, and after every call the two tables
must hold the same keys, rows and scores, bit for bit; the oracle is held to the same."""
import numpy as np
import pytest
import torch

import workloads as w
from gpu_util import DEV, assert_same_table, dev, export_table, sort_by_key
from hierarchicalkv_amd import (EvictStrategy, HashTable, MerlinException, default_options)

pytestmark = pytest.mark.gpu


def same_tables(a, b, vb):
    ka, va, sa = sort_by_key(*export_table(a, vb))
    kb, vb_, sb = sort_by_key(*export_table(b, vb))
    assert np.array_equal(ka, kb) and np.array_equal(va, vb_) and np.array_equal(sa, sb)
    assert a.size() == b.size() == len(ka)


@pytest.mark.parametrize("strategy", [EvictStrategy.kCustomized, EvictStrategy.kLru])
def test_noalloc_equals_insert_or_assign_on_two_calls_in_a_row(oracle, strategy):
    cap, dim = 1 << 15, 16
    vb = dim * 4
    opts = default_options(init_capacity=cap, max_capacity=cap, dim=dim, max_hbm_for_vectors=1 << 30,
                           evict_strategy=strategy)
    plain, noalloc = HashTable(), HashTable()
    plain.init(opts)
    noalloc.init(opts)
    o = oracle.OracleTable(opts)
    if strategy == EvictStrategy.kLru:
        for t in (plain, noalloc, o):
            t.set_clock(1, 1 << 40)  # the deterministic clock: scores do not depend on the run

    def scores_of(batch, n):
        return w.monotone_scores(batch, n) if strategy == EvictStrategy.kCustomized else None

    # fill past load factor 1.0 through the ordinary entry point on all three, so that the calls
    # under test meet full buckets: hits, evictions and refusals
    for b in range(5):
        keys = w.unique_keys(501, b * 8192, 8192)
        vals = w.values_from_keys(keys, dim)
        sc = scores_of(b + 1, 8192)
        for t in (plain, noalloc):
            t.insert_or_assign(8192, dev(keys), dev(vals), dev(sc))
        o.insert_or_assign(keys, vals.view(np.uint8).reshape(8192, vb), sc)
    same_tables(plain, noalloc, vb)

    # two calls in a row on the entry point under test, the second with a smaller input; half of
    # each batch is resident already
    for call, n in enumerate((50000, 7001)):
        old = w.unique_keys(501, 20000 + call * 3000, n // 2)
        new = w.unique_keys(502 + call, 0, n - n // 2)
        keys = np.concatenate([old, new])
        vals = w.values_from_keys(keys, dim) + np.float32(call + 1)
        sc = scores_of(10 + call, n)
        plain.insert_or_assign(n, dev(keys), dev(vals), dev(sc))
        noalloc.insert_or_assign_noalloc(n, dev(keys), dev(vals), dev(sc))
        o.insert_or_assign(keys, vals.view(np.uint8).reshape(n, vb), sc)
        torch.cuda.synchronize()
        same_tables(plain, noalloc, vb)
        assert_same_table(noalloc, o, vb)
    for t in (plain, noalloc, o):
        t.close()


@pytest.mark.parametrize("dim,strategy", [(3, EvictStrategy.kCustomized), (8, EvictStrategy.kLfu),
                                          (64, EvictStrategy.kEpochLru), (128, EvictStrategy.kEpochLfu),
                                          (300, EvictStrategy.kLru)])
def test_noalloc_row_sizes_strategies_and_long_lists(oracle, dim, strategy):
    """The two-phase path by itself against the oracle: rows of 12 bytes (4-byte units), 32, 256, 512
    and 1200 bytes (more than one pass of a tile), every strategy, a table of 32 buckets so that a
    bucket takes dozens of keys of one call (lists longer than one staging round), free slots left
    by erase, hits and new keys mixed."""
    cap = 1 << 12
    vb = dim * 4
    opts = default_options(init_capacity=cap, max_capacity=cap, dim=dim, max_hbm_for_vectors=1 << 30,
                           evict_strategy=strategy)
    t = HashTable()
    t.init(opts)
    o = oracle.OracleTable(opts)
    clocked = strategy in (EvictStrategy.kLru, EvictStrategy.kEpochLru)
    if clocked:
        t.set_clock(1, 1 << 44)
        o.set_clock(1, 1 << 44)
    if strategy in (EvictStrategy.kEpochLru, EvictStrategy.kEpochLfu):
        t.set_global_epoch(2)
        o.set_global_epoch(2)
    seed, pos, batch = 700 + dim, 0, 1

    def call(keys, bump=0.0):
        nonlocal batch
        n = len(keys)
        vals = w.values_from_keys(keys, dim) + np.float32(bump)
        # distinct, growing from call to call, and below 2^32 (EpochLFU keeps the low half only)
        sc = None if clocked else ((np.uint64(batch) << np.uint64(20)) +
                                   np.random.Generator(np.random.PCG64(batch)).permutation(n).astype(np.uint64))
        batch += 1
        t.insert_or_assign_noalloc(n, dev(keys), dev(vals), dev(sc))
        o.insert_or_assign(keys, vals.view(np.uint8).reshape(n, vb), sc)
        torch.cuda.synchronize()
        assert_same_table(t, o, vb)

    for n in (1500, 3000, 3000):  # past load factor 1.0 from an empty table: free slots, then victims
        call(w.unique_keys(seed, pos, n))
        pos += n
    gone = w.unique_keys(seed, pos - 1000, 700)
    t.erase(len(gone), dev(gone))
    o.erase(gone)
    assert_same_table(t, o, vb)
    for rep in range(3):
        # hits are keys of the latest call (the highest scores: no key of the batch can evict one
        # of them before its turn; under LFU they only gain), the rest is new
        old = w.unique_keys(seed, pos - 600, 600)
        old = old[o.contains(old)]
        new = w.unique_keys(seed, pos, 2001)
        pos += 2001
        call(np.concatenate([old, new]), bump=rep + 1.0)
    t.close()
    o.close()


def test_noalloc_refuses_what_it_cannot_do():
    dim = 4
    grow = HashTable()
    grow.init(default_options(init_capacity=1 << 12, max_capacity=1 << 16, dim=dim, max_hbm_for_vectors=1 << 30))
    keys = dev(w.unique_keys(9, 0, 128))
    vals = torch.zeros(128, dim, dtype=torch.float32, device=DEV)
    with pytest.raises(Exception, match="grow"):
        grow.insert_or_assign_noalloc(128, keys, vals)
    grow.close()
    t = HashTable()
    t.init(default_options(init_capacity=1 << 12, max_capacity=1 << 12, dim=dim, max_hbm_for_vectors=1 << 30))
    big = (1 << 20) + 64
    with pytest.raises(Exception, match="limit"):
        t.insert_or_assign_noalloc(big, keys, vals)  # refused before any key is read
    t.insert_or_assign_noalloc(0, keys, vals)        # an empty batch is fine
    t.insert_or_assign_noalloc(128, keys, vals)
    assert t.size() == 128
    t.close()
