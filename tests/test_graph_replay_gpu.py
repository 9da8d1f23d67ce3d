"""find and insert_or_assign launch kernels only (no allocation, no memset, no host
synchronisation on a table that cannot grow), so a serving loop can capture them into a HIP
graph.  The graph is replayed several times with new contents in its static buffers, with
eager calls and synchronisations in between, and every replay is checked against the oracle
stepping through the same sequence."""
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
