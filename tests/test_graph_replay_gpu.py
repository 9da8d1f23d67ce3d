"""Calls that return nothing to the host launch kernels only (no allocation, no memset, no host
synchronisation on a table that cannot grow), so a serving loop can capture them into a HIP
graph: find and insert_or_assign in the first test, contains, assign, find_or_insert,
insert_and_evict with a device counter and erase in the second.  The graph is replayed several
times with new contents in its static buffers, with eager calls and synchronisations in between,
and every replay is checked against the oracle stepping through the same sequence."""
import numpy as np
import pytest
import torch

import workloads as w
from gpu_util import DEV, assert_same_table, dev, host_u64
from hierarchicalkv_amd import EvictStrategy, HashTable, default_options

pytestmark = pytest.mark.gpu


def bytes_of(a):
    return np.ascontiguousarray(a).view(np.uint8).reshape(len(a), -1)


def test_find_and_insert_or_assign_replay_from_a_graph(oracle):
    # one stream for everything: the table's group lock then has nothing to order, and the
    # captured calls see the stream they were warmed up on
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        _run(oracle, stream)
    torch.cuda.synchronize()


def _run(oracle, stream):
    cap, dim, n = 1 << 14, 16, 2048
    o = default_options(init_capacity=cap, max_capacity=cap, max_hbm_for_vectors=1 << 30, dim=dim,
                        evict_strategy=EvictStrategy.kCustomized)
    t = HashTable()
    t.init(o)
    ot = oracle.OracleTable(o)
    seq = 0

    def batch(start):
        keys = w.unique_keys(77, start, n)
        vals = w.uniform_values(77, start, n, dim)
        return keys, vals

    # eager pre-fill to a full table
    for b in range(12):
        seq += 1
        k, v = batch(b * n)
        sc = w.monotone_scores(seq, n)
        t.insert_or_assign(n, dev(k), dev(v), dev(sc))
        ot.insert_or_assign(k, bytes_of(v), sc)
    assert_same_table(t, ot, dim * 4)

    # static buffers of the graph
    fk = torch.zeros(n, dtype=torch.int64, device=DEV)
    fout = torch.zeros(n, dim, dtype=torch.float32, device=DEV)
    ffound = torch.zeros(n, dtype=torch.bool, device=DEV)
    fsc = torch.zeros(n, dtype=torch.int64, device=DEV)
    ik = torch.zeros(n, dtype=torch.int64, device=DEV)
    iv = torch.zeros(n, dim, dtype=torch.float32, device=DEV)
    isc = torch.zeros(n, dtype=torch.int64, device=DEV)

    def load_inputs(step):
        nonlocal seq
        seq += 1
        qk = np.concatenate([w.unique_keys(77, (8 + step) * n, n // 2),      # residents or evicted
                             w.unique_keys(78, step * n, n // 2)])            # never seen
        k, v = batch((12 + step) * n)
        k[: n // 4] = w.unique_keys(77, (10 + step) * n, n // 4)              # a quarter are updates
        sc = w.monotone_scores(seq, n)
        fk.copy_(dev(qk))
        ik.copy_(dev(k))
        iv.copy_(dev(v))
        isc.copy_(dev(sc))
        return qk, k, v, sc

    # warm-up of the exact calls, then capture on the same stream
    qk, k, v, sc = load_inputs(0)
    torch.cuda.synchronize()
    t.find(n, fk, fout, ffound, fsc)
    t.insert_or_assign(n, ik, iv, isc)
    torch.cuda.synchronize()
    ov, of, os_ = ot.find(qk)
    ot.insert_or_assign(k, bytes_of(v), sc)
    assert np.array_equal(ffound.cpu().numpy(), of)

    g = torch.cuda.CUDAGraph()
    qk, k, v, sc = load_inputs(1)
    torch.cuda.synchronize()
    with torch.cuda.graph(g, stream=stream):
        t.find(n, fk, fout, ffound, fsc)
        t.insert_or_assign(n, ik, iv, isc)
    # capture does not run the work: the table still equals the oracle's
    assert_same_table(t, ot, dim * 4)

    for step in range(1, 5):
        if step > 1:
            qk, k, v, sc = load_inputs(step)
        fout.zero_()
        ffound.zero_()
        g.replay()
        torch.cuda.synchronize()
        ov, of, os_ = ot.find(qk)
        ot.insert_or_assign(k, bytes_of(v), sc)
        gf = ffound.cpu().numpy()
        assert np.array_equal(gf, of), step
        assert np.array_equal(bytes_of(fout.cpu().numpy())[of], ov[of]), step
        assert np.array_equal(host_u64(fsc)[of], os_[of]), step
        assert_same_table(t, ot, dim * 4)
        # eager work between the replays
        seq += 1
        ek, ev = batch((40 + step) * n)
        esc = w.monotone_scores(seq, n)
        t.insert_or_assign(n, dev(ek), dev(ev), dev(esc))
        ot.insert_or_assign(ek, bytes_of(ev), esc)
        torch.cuda.synchronize()
        assert t.size() == ot.size()
    t.close()
    ot.close()


def test_writers_with_device_counters_replay_from_a_graph(oracle):
    """The other calls that return nothing to the host: contains, assign, find_or_insert,
    insert_and_evict with a device counter (cleared inside the graph by a fill kernel), erase."""
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        _run_writers(oracle, stream)
    torch.cuda.synchronize()


def _run_writers(oracle, stream):
    cap, dim, n = 1 << 14, 8, 1024
    o = default_options(init_capacity=cap, max_capacity=cap, max_hbm_for_vectors=1 << 30, dim=dim,
                        evict_strategy=EvictStrategy.kCustomized)
    t = HashTable()
    t.init(o)
    ot = oracle.OracleTable(o)
    seq = 0
    for b in range(20):  # a full table
        seq += 1
        k, v, sc = w.unique_keys(91, b * n, n), w.uniform_values(91, b * n, n, dim), w.monotone_scores(seq, n)
        t.insert_or_assign(n, dev(k), dev(v), dev(sc))
        ot.insert_or_assign(k, bytes_of(v), sc)
    assert_same_table(t, ot, dim * 4)

    def buf(shape, dtype):
        return torch.zeros(shape, dtype=dtype, device=DEV)
    ak, av, asc = buf(n, torch.int64), buf((n, dim), torch.float32), buf(n, torch.int64)      # assign
    fk, fio, fsc = buf(n, torch.int64), buf((n, dim), torch.float32), buf(n, torch.int64)     # find_or_insert
    ek, ev, esc = buf(n, torch.int64), buf((n, dim), torch.float32), buf(n, torch.int64)      # insert_and_evict
    ok_, ov_, os_, cnt = buf(n, torch.int64), buf((n, dim), torch.float32), buf(n, torch.int64), buf(1, torch.int64)
    rk, cf = buf(n // 4, torch.int64), buf(n // 4, torch.bool)                                # erase, contains

    def load_inputs(step):
        nonlocal seq
        a_keys = w.unique_keys(91, 19 * n, n)  # resident throughout: its scores are raised every step
        seq += 1
        a_sc = w.monotone_scores(seq, n)
        f_keys = w.unique_keys(92, step * n, n)  # all new
        seq += 1
        f_sc = w.monotone_scores(seq, n)
        e_keys = w.unique_keys(93, step * n, n)  # all new
        seq += 1
        e_sc = w.monotone_scores(seq, n)
        r_keys = f_keys[: n // 4]  # erase a quarter of what find_or_insert has just put in
        vals = [w.uniform_values(94 + i, step * n, n, dim) for i in range(3)]
        for d, h in ((ak, a_keys), (asc, a_sc), (fk, f_keys), (fsc, f_sc), (ek, e_keys), (esc, e_sc), (rk, r_keys)):
            d.copy_(dev(h))
        for d, h in ((av, vals[0]), (fio, vals[1]), (ev, vals[2])):
            d.copy_(dev(h))
        return a_keys, a_sc, f_keys, f_sc, e_keys, e_sc, r_keys, vals

    def calls():
        t.assign(n, ak, av, asc)
        t.find_or_insert(n, fk, fio, fsc)
        cnt.zero_()
        t.insert_and_evict(n, ek, ev, esc, ok_, ov_, os_, cnt)
        t.erase(n // 4, rk)
        t.contains(n // 4, rk, cf)

    def check(inp, step):
        a_keys, a_sc, f_keys, f_sc, e_keys, e_sc, r_keys, vals = inp
        ot.assign(a_keys, bytes_of(vals[0]), a_sc)
        fio_want = bytes_of(vals[1]).copy()
        ot.find_or_insert(f_keys, fio_want, f_sc)
        oek, oev, oes = ot.insert_and_evict(e_keys, bytes_of(vals[2]), e_sc)
        ot.erase(r_keys)
        assert np.array_equal(bytes_of(fio.cpu().numpy()), fio_want), step
        c = int(cnt.item())
        assert c == len(oek), step
        a = np.argsort(host_u64(ok_)[:c], kind="stable")
        b = np.argsort(oek, kind="stable")
        assert np.array_equal(host_u64(ok_)[:c][a], oek[b]), step
        assert np.array_equal(bytes_of(ov_.cpu().numpy())[:c][a], oev[b]), step
        assert np.array_equal(host_u64(os_)[:c][a], oes[b]), step
        assert not cf.cpu().numpy().any(), step
        assert_same_table(t, ot, dim * 4)

    inp = load_inputs(0)
    torch.cuda.synchronize()
    calls()  # warm-up of the exact calls
    torch.cuda.synchronize()
    check(inp, 0)
    g = torch.cuda.CUDAGraph()
    inp = load_inputs(1)
    torch.cuda.synchronize()
    with torch.cuda.graph(g, stream=stream):
        calls()
    assert_same_table(t, ot, dim * 4)  # capture has not run anything
    for step in range(1, 5):
        if step > 1:
            inp = load_inputs(step)
        g.replay()
        torch.cuda.synchronize()
        check(inp, step)
        seq += 1  # eager work between the replays
        k, v, sc = w.unique_keys(95, step * n, n), w.uniform_values(95, step * n, n, dim), w.monotone_scores(seq, n)
        t.insert_or_assign(n, dev(k), dev(v), dev(sc))
        ot.insert_or_assign(k, bytes_of(v), sc)
        torch.cuda.synchronize()
    t.close()
    ot.close()


@pytest.mark.skipif(__import__("os").environ.get("HKV_SCORE_BOUNDS") == "0", reason="score bounds switched off")
def test_replays_after_scores_from_outside_the_clock():
    """An LRU table on the hardware clock whose upserts search victims through the score bounds: an
    insert_or_assign recorded into a graph must go on evicting the lowest score of a bucket after
    a call that writes scores from outside the clock (ignore_evict_strategy) has made the bounds
    stale, replay after replay, with eager upserts (which make the bounds again) in between.
    Without an oracle (the scores are the time of day): the keys that were given the lowest scores
    are the first to go, every row that is found is its key's, and the bounds hold at the end."""
    from test_score_bounds_gpu import bounds_hold
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        cap, dim, n = 1 << 14, 16, 2048
        o = default_options(init_capacity=cap, max_capacity=cap, max_hbm_for_vectors=1 << 30, dim=dim,
                            evict_strategy=EvictStrategy.kLru)
        t = HashTable()
        t.init(o)
        pos = 0
        for _ in range(12):  # past load factor 1.0: the last calls use the bounds
            k = w.unique_keys(55, pos, n)
            t.insert_or_assign(n, dev(k), dev(w.values_from_keys(k, dim)))
            pos += n
        torch.cuda.synchronize()
        assert bounds_hold(t)[0] and bounds_hold(t)[2] > 0
        ik = torch.zeros(n, dtype=torch.int64, device=DEV)
        iv = torch.zeros(n, dim, dtype=torch.float32, device=DEV)

        def load(start):
            k = w.unique_keys(55, start, n)
            ik.copy_(dev(k))
            iv.copy_(dev(w.values_from_keys(k, dim)))
            return k
        load(pos)
        pos += n
        t.insert_or_assign(n, ik, iv)  # warm-up of the exact call
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        load(pos)
        torch.cuda.synchronize()
        with torch.cuda.graph(g, stream=stream):
            t.insert_or_assign(n, ik, iv)
        founds = torch.zeros(n, dtype=torch.bool, device=DEV)
        out = torch.zeros(n, dim, dtype=torch.float32, device=DEV)
        for rnd in range(3):
            # residents get scores far below the clock's
            low = w.unique_keys(55, pos - 2 * n, n)
            t.contains(n, dev(low), founds)
            torch.cuda.synchronize()
            low = low[founds.cpu().numpy()]
            assert len(low) > n // 2
            t.insert_or_assign(len(low), dev(low), dev(w.values_from_keys(low, dim)),
                               dev(np.arange(1, len(low) + 1, dtype=np.uint64)), ignore_evict_strategy=True)
            # three replays and an eager upsert: 64 new keys for each of the 128 buckets on average,
            # at least about 40 for every one, against at most about 30 low-scored keys in a bucket:
            # they all go if every eviction takes the bucket's lowest score, and most of them stay
            # if victims are taken from elsewhere
            for r in range(3):
                load(pos)
                pos += n
                g.replay()
                if r == 1:  # an eager upsert between replays rebuilds the bounds and uses them
                    k = w.unique_keys(56, pos, n)
                    t.insert_or_assign(n, dev(k), dev(w.values_from_keys(k, dim)))
            torch.cuda.synchronize()
            f2 = torch.zeros(len(low), dtype=torch.bool, device=DEV)
            t.contains(len(low), dev(low), f2)
            torch.cuda.synchronize()
            assert not f2.cpu().numpy().any(), "keys with the lowest scores outlived 64 new keys per bucket"
            assert t.size() == cap
            last = w.unique_keys(55, pos - n, n)
            t.find(n, dev(last), out, founds)
            torch.cuda.synchronize()
            f = founds.cpu().numpy()
            assert f.all()
            assert np.array_equal(out.cpu().numpy(), w.values_from_keys(last, dim))
        k = w.unique_keys(57, 0, n)
        t.insert_or_assign(n, dev(k), dev(w.values_from_keys(k, dim)))
        torch.cuda.synchronize()
        ok, bad, _ = bounds_hold(t)
        assert ok, bad
        t.close()
    torch.cuda.synchronize()
