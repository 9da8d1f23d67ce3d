"""Host-thread tests after tests/merlin_hashtable_test.cc.cu:3180-3625
(test_insert_or_assign_multi_threads): 64 host threads, each on a stream of its own, call
insert_or_assign, find and size() on one table at the same time."""
import threading
import time

import numpy as np
import pytest
import torch

import workloads as w
from gpu_util import DEV, assert_same_table, dev
from hierarchicalkv_amd import EvictStrategy, HashTable, default_options

pytestmark = pytest.mark.gpu


def test_sixty_four_threads_insert_find_and_size(oracle):
    """Every thread owns a disjoint key range: before its insert none of its keys is found,
    afterwards all are with their rows; size() never reads less than what the thread itself has
    inserted nor more than all threads together will; at the end the table equals the oracle
    (no bucket fills up at this load, so the order of the batches does not matter).  The count
    readers are what this test is for: each size() takes a device word, zeroes it, has a kernel
    add to it and reads it back, and with 64 callers two of them must never share a word."""
    n_threads, rounds, n, dim = 64, 6, 2048, 8
    cap = 1 << 21
    total = n_threads * rounds * n
    opts = default_options(init_capacity=cap, max_capacity=cap, dim=dim, max_hbm_for_vectors=1 << 34,
                           evict_strategy=EvictStrategy.kLru)
    t = HashTable()
    t.init(opts)
    errors = []
    stop = threading.Event()

    def worker(tid):
        try:
            torch.cuda.set_device(0)
            st = torch.cuda.Stream()
            mine = 0
            for r in range(rounds):
                if stop.is_set():
                    return
                keys = w.unique_keys(7000 + tid, r * n, n)
                vals = w.values_from_keys(keys, dim)
                dk, dv = dev(keys), dev(vals)
                out = torch.zeros(n, dim, dtype=torch.float32, device=DEV)
                founds = torch.zeros(n, dtype=torch.bool, device=DEV)
                torch.cuda.current_stream().synchronize()
                t.find(n, dk, out, founds, None, stream=st)
                st.synchronize()
                assert not bool(founds.any()), ("found before insert", tid, r)
                t.insert_or_assign(n, dk, dv, None, stream=st)
                mine += n
                s1 = t.size(stream=st)
                assert mine <= s1 <= total, ("size after insert", tid, r, s1, mine)
                t.find(n, dk, out, founds, None, stream=st)
                s2 = t.size(stream=st)
                st.synchronize()
                assert s1 <= s2 <= total, ("size went down", tid, r, s1, s2)
                assert bool(founds.all()), ("not found after insert", tid, r)
                assert np.array_equal(out.cpu().numpy(), vals), ("row", tid, r)
        except BaseException as e:  # noqa: BLE001 - reported by the main thread
            errors.append((tid, repr(e)))
            stop.set()  # the other threads stop at their next round

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(n_threads)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors[:3]
    assert t.size() == total

    # the same keys through the oracle: the resident key set, rows and size must agree
    # (LRU scores are clock readings and differ)
    o = oracle.OracleTable(opts)
    for tid in range(n_threads):
        for r in range(rounds):
            keys = w.unique_keys(7000 + tid, r * n, n)
            o.insert_or_assign(keys, w.values_from_keys(keys, dim).view(np.uint8).reshape(n, dim * 4))
    from gpu_util import export_table, sort_by_key
    gk, gv, _ = sort_by_key(*export_table(t, dim * 4))
    ok, ov, _ = sort_by_key(*o.export_all())
    assert np.array_equal(gk, ok) and np.array_equal(gv, ov)
    assert o.size() == total
    o.close()
    t.close()


def test_lru_scores_are_unix_epoch_nanoseconds():
    """The reference's LRU score is %globaltimer, nanoseconds since the Unix epoch
    (utils.cuh:75-80): a fresh key's score lies between host clock readings taken around the
    call, give or take the accuracy of the table's tie between device counter and host clock."""
    n, dim = 4096, 8
    t = HashTable()
    t.init(default_options(init_capacity=1 << 16, max_capacity=1 << 16, dim=dim,
                           max_hbm_for_vectors=1 << 30, evict_strategy=EvictStrategy.kLru))
    keys = w.unique_keys(31, 0, n)
    dk, dv = dev(keys), dev(w.values_from_keys(keys, dim))
    torch.cuda.synchronize()
    before = time.time_ns()
    t.insert_or_assign(n, dk, dv)
    torch.cuda.synchronize()
    after = time.time_ns()
    out = torch.zeros(n, dim, dtype=torch.float32, device=DEV)
    founds = torch.zeros(n, dtype=torch.bool, device=DEV)
    scores = torch.zeros(n, dtype=torch.int64, device=DEV)
    t.find(n, dk, out, founds, scores)
    torch.cuda.synchronize()
    s = scores.cpu().numpy().view(np.uint64)
    assert bool(founds.all())
    slack = 50_000_000  # 50 ms: far above the sampling error, far below any wrong epoch
    assert int(s.min()) >= before - slack and int(s.max()) <= after + slack, (before, int(s.min()), int(s.max()), after)
    t.close()
