"""The benchmark configurations 2 to 5 at their full sizes.

No host oracle finishes at these sizes, so the checks are properties that do
not depend on size: every row that comes back (found, evicted or exported)
must be the function of its key that was stored, evicted scores must be the
score function of the evicted key, counts must be conserved, accumulation must
be linear, erased keys must be gone.  Keys, scores and values are generated on
the device (a 64-bit mixing bijection of a counter), so a 2^28-slot table is
filled in seconds.  Sizes, strategies, batch and dims follow the workload
descriptions of configurations 2-5; the small configuration 1 runs in
test_parity_gpu.py against the oracle line by line.

Run with -s to see the timings these tests print (hybrid mode: host-link GB/s).
"""
import time

import numpy as np
import pytest
import torch

import workloads as w
from gpu_util import DEV
from hierarchicalkv_amd import EvictStrategy, HashTable, Predicate, ValueKind, default_options

pytestmark = pytest.mark.gpu

from workloads_device import M63, _lsr, dev_keys, mix64, score_of, value_of  # noqa: E402,F401


def make_table(**kw):
    t = HashTable()
    t.init(default_options(**kw))
    return t


def fill(t, cap, n, dim, seed, scores_fn=None, factor=1.0):
    """insert_or_assign batches of fresh keys until about factor * cap keys went in."""
    pos = 0
    while pos < int(factor * cap):
        k = dev_keys(seed, pos, n)
        t.insert_or_assign(n, k, value_of(k, dim), None if scores_fn is None else scores_fn(k))
        pos += n
    return pos


def device_unique_count(chunks):
    allk = torch.cat(chunks)
    return int(torch.unique(allk).numel()), int(allk.numel())


def export_keys(t, vb_unused, pred=Predicate.kAlways, pattern=0, threshold=0, with_values_dim=None,
                window=1 << 22):
    """Keys (and optionally a check of every exported row) of all entries matching pred."""
    cap = t.capacity()
    dk = torch.zeros(window, dtype=torch.int64, device=DEV)
    ds = torch.zeros(window, dtype=torch.int64, device=DEV)
    dv = None
    if with_values_dim:
        dv = torch.zeros(window, with_values_dim, dtype=torch.float32, device=DEV)
    dc = torch.zeros(1, dtype=torch.int64, device=DEV)
    keys, scores = [], []
    for off in range(0, cap, window):
        t.export_batch_if(pred, pattern, threshold, window, off, dc, dk, dv, ds)
        c = int(dc.item())
        keys.append(dk[:c].clone())
        scores.append(ds[:c].clone())
        if dv is not None and c:
            assert torch.equal(dv[:c], value_of(dk[:c], with_values_dim)), "exported row is not its key's row"
    return keys, scores


# ---- configuration 2: 2^26 slots, dim 8, LRU; load factors 0.50 / 0.75 / 1.00 -----------------------------

def test_config2_throughput_shape_full_size():
    cap, dim, n, seed = 1 << 26, 8, 1 << 20, 2
    t = make_table(init_capacity=cap, max_capacity=cap, max_hbm_for_vectors=cap * dim * 4, dim=dim,
                   evict_strategy=EvictStrategy.kLru)
    out = torch.empty(n, dim, dtype=torch.float32, device=DEV)
    founds = torch.empty(n, dtype=torch.bool, device=DEV)
    pos = 0
    for lf in (0.50, 0.75, 1.00):
        while pos < int(lf * cap):
            k = dev_keys(seed, pos, n)
            t.insert_or_assign(n, k, value_of(k, dim))
            pos += n
        size = t.size()
        assert size <= cap
        if lf == 0.50:
            assert size == pos  # half full: no bucket of 128 overflows, nothing has been evicted
        else:
            assert size > 0.95 * min(pos, cap)  # uniform hashing: some buckets overflow before others fill
        # find, 100 % hits: the newest batch is resident under LRU
        newest = dev_keys(seed, pos - n, n)
        t.find(n, newest, out, founds)
        assert bool(founds.all())
        assert torch.equal(out, value_of(newest, dim))
        # insert_or_assign, 50 % new keys; the assigned half gets new rows
        half_old, fresh = newest[: n // 2], dev_keys(seed, pos, n // 2)
        pos += n // 2
        batch = torch.cat([half_old, fresh])
        rows = value_of(batch, dim) + 0.5
        t.insert_or_assign(n, batch, rows)
        t.find(n, batch, out, founds)
        assert bool(founds.all())
        assert torch.equal(out, rows)
        # find_or_insert: present keys return the stored row, absent keys keep and store their own
        fresh2 = dev_keys(seed, pos, n // 2)
        pos += n // 2
        batch2 = torch.cat([fresh, fresh2])
        io = torch.cat([torch.full((n // 2, dim), -7.0, device=DEV), value_of(fresh2, dim)])
        t.find_or_insert(n, batch2, io)
        assert torch.equal(io[: n // 2], rows[n // 2:])
        assert torch.equal(io[n // 2:], value_of(fresh2, dim))
        t.find(n // 2, fresh2, out[: n // 2], founds[: n // 2])
        assert bool(founds[: n // 2].all()) and torch.equal(out[: n // 2], value_of(fresh2, dim))
        # assign (no slot locks: the updater is alone on the table): present keys get the new
        # rows, absent keys are not inserted
        absent = dev_keys(seed + 17, pos, n // 2)
        batch3 = torch.cat([fresh2, absent])
        rows3 = value_of(batch3, dim) + 0.25
        before = t.size()
        t.assign(n, batch3, rows3)
        assert t.size() == before
        t.find(n, batch3, out, founds)
        assert bool(founds[: n // 2].all()) and not bool(founds[n // 2:].any())
        assert torch.equal(out[: n // 2], rows3[: n // 2])
        # find_or_insert*: pointers to the rows of present and new keys
        fresh3 = dev_keys(seed, pos, n // 2)
        pos += n // 2
        batch4 = torch.cat([fresh2, fresh3])
        ptrs = torch.zeros(n, dtype=torch.int64, device=DEV)
        t.find_or_insert_ptr(n, batch4, ptrs, founds)
        assert bool(founds[: n // 2].all()) and not bool(founds[n // 2:].any())
        assert bool((ptrs != 0).all())
        v = t.view()
        off = ptrs - v.values
        assert bool(((off >= 0) & (off < cap * dim * 4) & (off % (dim * 4) == 0)).all())
        assert int(torch.unique(off).numel()) == n  # one row per key
        t.assign_values(n // 2, fresh3, value_of(fresh3, dim))  # rows of the new keys, as a caller would
        t.find(n, batch4, out, founds)
        assert bool(founds.all())
        assert torch.equal(out, torch.cat([rows3[: n // 2], value_of(fresh3, dim)]))
    # the table holds each key once, and as many as it says
    keys, _ = export_keys(t, dim * 4)
    uniq, total = device_unique_count(keys)
    assert uniq == total == t.size()
    assert t.size() > 0.95 * cap
    t.close()


# ---- configuration 3: 2^27 slots, dim 64 (32 GB of rows), Customized, Zipf insert_and_evict ------------------

def test_config3_insert_and_evict_full_size():
    cap, dim, n, seed = 1 << 27, 64, 1 << 20, 3
    t = make_table(init_capacity=cap, max_capacity=cap, max_hbm_for_vectors=cap * dim * 4, dim=dim,
                   evict_strategy=EvictStrategy.kCustomized)
    fill(t, cap, n, dim, seed, scores_fn=score_of, factor=1.4)
    assert t.size() > 0.999 * cap
    ek = torch.zeros(n, dtype=torch.int64, device=DEV)
    ev = torch.zeros(n, dim, dtype=torch.float32, device=DEV)
    es = torch.zeros(n, dtype=torch.int64, device=DEV)
    out = torch.empty(n, dim, dtype=torch.float32, device=DEV)
    founds = torch.empty(n, dtype=torch.bool, device=DEV)
    before = torch.empty(n, dtype=torch.bool, device=DEV)
    zpos = 0
    for b in range(3):
        hk, zpos = w.zipf_unique_keys(seed, zpos, n)  # alpha 1.05 over 2^31 keys, unique in the batch
        k = torch.from_numpy(hk.view(np.int64)).to(DEV)
        t.contains(n, k, before)
        size0 = t.size()
        cnt = t.insert_and_evict(n, k, value_of(k, dim), score_of(k), ek, ev, es)
        assert 0 < cnt <= n
        # whatever leaves - evicted or refused - leaves whole: key, its row, its score
        assert torch.equal(ev[:cnt], value_of(ek[:cnt], dim))
        assert torch.equal(es[:cnt], score_of(ek[:cnt]))
        # (a key can leave twice: a resident key of the batch that a batch-mate evicts and whose
        # own upsert is then refused - one of the legal serial orders)
        left = torch.unique(ek[:cnt])
        t.find(n, k, out, founds)
        assert torch.equal(out[founds], value_of(k[founds], dim))
        # a key of the batch that is absent afterwards was refused (it is in the output), or was
        # admitted and then displaced by a later key of the batch (also in the output)
        gone = k[~founds]
        assert bool(torch.isin(gone, ek[:cnt]).all())
        # conservation: keys that were not there and are now, minus those that left for good
        still = torch.empty(left.numel(), dtype=torch.bool, device=DEV)
        t.contains(left.numel(), left, still)
        assert not bool(still.any())
        new_in = int((founds & ~before).sum())
        was_in_and_left = left.numel() - int((~founds & ~before).sum())  # outputs that were resident before
        assert t.size() == size0 + new_in - was_in_and_left
    t.close()


# ---- configuration 4: 2^28 slots, dim 64 (64 GB of rows), 16 GB in HBM, the rest pinned; LFU -------------------

def test_config4_hybrid_full_size():
    cap, dim, n, seed = 1 << 28, 64, 1 << 20, 4
    hbm = 16 << 30
    t0 = time.time()
    t = make_table(init_capacity=cap, max_capacity=cap, max_hbm_for_vectors=hbm, dim=dim,
                   evict_strategy=EvictStrategy.kLfu)
    assert not t.is_pure_hbm()
    print(f"\n[hybrid] table created in {time.time() - t0:.1f} s", flush=True)
    ones = torch.ones(n, dtype=torch.int64, device=DEV)
    t0 = time.time()
    pos = 0
    while pos < cap + cap // 8:
        k = dev_keys(seed, pos, n)
        t.insert_or_assign(n, k, value_of(k, dim), ones)
        pos += n
    torch.cuda.synchronize()
    size = t.size()
    print(f"[hybrid] filled to {size / cap:.4f} in {time.time() - t0:.1f} s", flush=True)
    assert size > 0.99 * cap
    # With equal counts LFU evicts the lowest slot of a full bucket, i.e. mostly the keys that came
    # last; keys of an early stretch went into free slots and are mostly still there.
    out = torch.empty(n, dim, dtype=torch.float32, device=DEV)
    founds = torch.empty(n, dtype=torch.bool, device=DEV)
    cand = torch.cat([dev_keys(seed, (10 + i) * n, n) for i in range(4)])
    res = torch.empty(cand.numel(), dtype=torch.bool, device=DEV)
    t.contains(cand.numel(), cand, res)
    resident = cand[res]
    assert resident.numel() >= int(0.8 * n)
    absent = dev_keys(seed + 1, 0, n - int(0.8 * n))
    q = torch.cat([resident[: int(0.8 * n)], absent])  # 80 % hits
    ptrs = torch.zeros(n, dtype=torch.int64, device=DEV)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
    t.find(n, q, out, founds)  # warm-up
    ev[0].record()
    t.find(n, q, out, founds)
    ev[1].record()
    t.find_ptr(n, q, ptrs, founds)
    ev[2].record()
    torch.cuda.synchronize()
    hits = int(founds.sum())
    assert hits == int(0.8 * n)
    assert torch.equal(out[founds], value_of(q[founds], dim))
    view = t.view()
    host_lo = view.host_values
    host_hi = host_lo + (cap - view.hbm_slots) * dim * 4
    p = ptrs[founds]
    in_host = int(((p >= host_lo) & (p < host_hi)).sum())
    in_hbm = int(((p >= view.values) & (p < view.values + view.hbm_slots * dim * 4)).sum())
    assert in_host + in_hbm == hits
    find_ms = ev[0].elapsed_time(ev[1])
    ptr_ms = ev[1].elapsed_time(ev[2])
    print(f"[hybrid] find 80% hits: {find_ms:.3f} ms, {hits / find_ms / 1e6:.3f} bKV/s; rows from host memory "
          f"{in_host} ({in_host * dim * 4 / find_ms / 1e6:.1f} GB/s over the host link), from HBM {in_hbm} "
          f"({in_hbm * dim * 4 / find_ms / 1e6:.1f} GB/s); find* {ptr_ms:.3f} ms", flush=True)
    # insert_or_assign with 20 % new keys; the assigned rows change, counts go up by one
    fresh = dev_keys(seed + 2, 0, n - int(0.8 * n))
    batch = torch.cat([resident[: int(0.8 * n)], fresh])
    rows = value_of(batch, dim) + 0.25
    ev[0].record()
    t.insert_or_assign(n, batch, rows, ones)
    ev[1].record()
    torch.cuda.synchronize()
    print(f"[hybrid] insert_or_assign 20% new: {ev[0].elapsed_time(ev[1]):.3f} ms", flush=True)
    sc = torch.zeros(n, dtype=torch.int64, device=DEV)
    t.find(n, batch, out, founds, sc)
    # Every count in the table is 1, so the new keys displace whatever sits lowest in their
    # bucket; an assigned key that a batch-mate displaced before its own turn came is inserted
    # again (count 1) and may be displaced again.  Nearly all keep their slot and count up.
    n_old = int(0.8 * n)
    old = founds[:n_old]
    assert int(old.sum()) > 0.99 * n_old
    assert torch.equal(out[:n_old][old], rows[:n_old][old])
    so = sc[:n_old][old]
    assert bool(((so == 2) | (so == 1)).all()) and int((so == 2).sum()) > 0.99 * n_old
    newf = founds[int(0.8 * n):]
    assert torch.equal(out[int(0.8 * n):][newf], rows[int(0.8 * n):][newf])
    assert t.size() <= cap
    t.close()


# ---- configuration 5: 2^25 slots, dim 128, EpochLRU; accum_or_assign, export_batch_if, erase ------------------

def test_config5_update_export_full_size():
    cap, dim, n, seed = 1 << 25, 128, 1 << 20, 5
    t = make_table(init_capacity=cap, max_capacity=cap, max_hbm_for_vectors=cap * dim * 4, dim=dim,
                   evict_strategy=EvictStrategy.kEpochLru)
    t.set_clock(1, 1 << 40)  # deterministic clock: scores are (epoch << 32) | ticks
    epoch, batches, pos = 1, 0, 0
    t.set_global_epoch(epoch)

    def tick():
        nonlocal epoch, batches
        batches += 1
        if batches % 10 == 0:  # the epoch moves every 10 batches
            epoch += 1
            t.set_global_epoch(epoch)

    while pos < cap + cap // 4:
        k = dev_keys(seed, pos, n)
        t.insert_or_assign(n, k, value_of(k, dim))
        pos += n
        tick()
    assert t.size() > 0.999 * cap
    out = torch.empty(n, dim, dtype=torch.float32, device=DEV)
    founds = torch.empty(n, dtype=torch.bool, device=DEV)
    # accum_or_assign, 70 % existing keys: existing ones accumulate a delta, new ones are assigned
    n_old = int(0.7 * n)
    recent = dev_keys(seed, pos - n, n)[:n_old]
    delta = 0.125  # exact in fp32 on top of the small integers stored, so sums are exact
    for rep in range(1, 3):
        fresh = dev_keys(seed + 7, (rep - 1) * n, n - n_old)
        batch = torch.cat([recent, fresh])
        rows = torch.cat([torch.full((n_old, dim), delta, device=DEV), value_of(fresh, dim)])
        flags = torch.cat([torch.ones(n_old, dtype=torch.bool, device=DEV),
                           torch.zeros(n - n_old, dtype=torch.bool, device=DEV)])
        t.accum_or_assign(n, batch, rows, flags)
        tick()
        t.find(n, batch, out, founds)
        assert bool(founds.all())
        assert torch.equal(out[:n_old], value_of(recent, dim) + rep * delta)  # linear in the repeats
        assert torch.equal(out[n_old:], value_of(fresh, dim))
    # export_batch_if, score >= threshold: the threshold is the score quantile that keeps about a quarter
    keys, scores = export_keys(t, dim * 4)
    allk, alls = torch.cat(keys), torch.cat(scores)
    assert allk.numel() == t.size() == int(torch.unique(allk).numel())
    thr = int(torch.sort(alls).values[int(0.75 * alls.numel())].item())
    want = int((alls >= thr).sum())
    assert 0.2 * alls.numel() < want < 0.3 * alls.numel()
    assert t.size_if(Predicate.kScoreGe, 0, thr) == want
    k2, s2 = export_keys(t, dim * 4, Predicate.kScoreGe, 0, thr)
    k2, s2 = torch.cat(k2), torch.cat(s2)
    assert k2.numel() == want and bool((s2 >= thr).all())
    assert torch.equal(torch.sort(k2).values, torch.sort(allk[alls >= thr]).values)
    # erase 2^18 keys, half of them resident
    m = 1 << 18
    victims = torch.cat([recent[: m // 2], dev_keys(seed + 9, 0, m // 2)])
    size0 = t.size()
    t.erase(m, victims)
    t.contains(m, victims, founds[:m])
    assert not bool(founds[:m].any())
    assert t.size() == size0 - m // 2
    # a tombstone is the first victim of its bucket: new keys go in without the size passing capacity
    k = dev_keys(seed + 11, 0, n)
    t.insert_or_assign(n, k, value_of(k, dim))
    t.find(n, k, out, founds)
    assert bool(founds.all()) and torch.equal(out, value_of(k, dim))
    assert t.size() <= cap
    t.close()


# ---- closed-form scenarios of the reference's own tests at (nearly) their sizes --------------------------

def _ref_rows(keys, dim):
    """test_util.cuh:160-163: every element of a key's row is float(key * 0.00001)."""
    return np.repeat((keys.astype(np.float64) * 0.00001).astype(np.float32)[:, None], dim, axis=1)


def test_basic_when_full_scenario():
    """tests/merlin_hashtable_test.cc.cu:799-925 (test_basic_when_full): as many random keys as
    the table has slots in one call; what stays can be found with its row, erasing everything
    empties the table, and inserting the same batch again fills it to the same size."""
    from gpu_util import dev
    cap, dim = 1 << 20, 16
    t = make_table(init_capacity=cap, max_capacity=cap, max_hbm_for_vectors=1 << 34, dim=dim,
                   reserved_key_start_bit=3, num_of_buckets_per_alloc=32,
                   evict_strategy=EvictStrategy.kCustomized)
    rng = np.random.default_rng(7)
    keys = np.unique(rng.integers(0, 1 << 62, cap + 4096, dtype=np.uint64))[:cap]
    rng.shuffle(keys)
    scores = rng.integers(1, 1 << 62, cap, dtype=np.uint64)
    dk, dv, ds = dev(keys), dev(_ref_rows(keys, dim)), dev(scores)
    t.insert_or_assign(cap, dk, dv, ds)
    size_after_insert = t.size()
    assert 0.9 * cap < size_after_insert < cap  # some buckets get more than 128 of the keys
    out = torch.zeros(cap, dim, dtype=torch.float32, device=DEV)
    founds = torch.zeros(cap, dtype=torch.bool, device=DEV)
    t.find(cap, dk, out, founds, None)
    assert int(founds.sum()) == size_after_insert
    assert bool((out[founds] == dv[founds]).all())
    # the survivors of a bucket are its highest scores: the table holds sum(min(128, n_b)) keys
    t.erase(cap, dk)
    assert t.size() == 0
    t.insert_or_assign(cap, dk, dv, ds)
    assert t.size() == size_after_insert
    t.close()


def test_customized_correct_rate_scenario():
    """tests/merlin_hashtable_test.cc.cu:3055-3178 (test_evict_strategy_customized_correct_rate) at
    1/16 of its size: consecutive keys with score = key, three times the capacity in 128 batches
    per round; after every round at least 96.4 % of the slots hold keys of that round."""
    from gpu_util import dev, export_table
    batch, steps, dim, rounds = 1 << 16, 128, 4, 3
    cap = batch * steps
    t = make_table(init_capacity=cap, max_capacity=cap, max_hbm_for_vectors=1 << 34, dim=dim,
                   reserved_key_start_bit=17, num_of_buckets_per_alloc=128,
                   evict_strategy=EvictStrategy.kCustomized)
    start = 100000
    for r in range(rounds):
        expected_min, expected_max = start + cap * r, start + cap * (r + 1) - 1
        for s in range(steps):
            k = np.arange(start + (r * steps + s) * batch, start + (r * steps + s + 1) * batch, dtype=np.uint64)
            t.insert_or_assign(batch, dev(k), dev(_ref_rows(k, dim)), dev(k.copy()))
        size = t.size()
        assert size >= (int(0.964 * cap) if r == 0 else cap)
        assert t.capacity() == cap
        ek, ev, es = export_table(t, dim * 4)
        assert len(ek) == size and np.array_equal(ek, es)
        assert np.array_equal(ev.view(np.float32), _ref_rows(ek, dim))
        rate = float((es >= expected_min).sum()) / cap
        print(f"[round {r}] correct rate {rate:.4f}, size {size / cap:.4f}")
        assert int(ek.max()) >= expected_max
        assert rate >= 0.964
    t.close()


@pytest.mark.parametrize("hbm", [1 << 34, 0])
def test_insert_or_assign_values_check_scenario(hbm):
    """tests/merlin_hashtable_test.cc.cu:3621-3660 (test_insert_or_assign_values_check): an LRU table
    that grows from 1024 slots to 2^19, batches of 2^19 + 13 random keys out of a range 16 times
    as large (more keys than the table can ever hold, and many of them met before); after every
    call the export has as many entries as size() says and every row is the row of its key."""
    from gpu_util import dev, export_table
    cap, dim = 524288, 64
    n = cap + 13
    t = make_table(init_capacity=1024, max_capacity=cap, max_hbm_for_vectors=hbm, dim=dim,
                   evict_strategy=EvictStrategy.kLru)
    rng = np.random.default_rng(11)
    for it in range(6):
        keys = rng.choice(n * 16, size=n, replace=False).astype(np.uint64)
        if it % 2 == 0:
            t.insert_or_assign(n, dev(keys), dev(_ref_rows(keys, dim)))
        else:
            # find_or_insert_test.cc.cu (test_find_or_insert_values_check): keys that are there hand
            # their row back, new keys store theirs; either way the caller holds the key's row
            io = dev(_ref_rows(keys, dim))
            t.find_or_insert(n, dev(keys), io)
            assert np.array_equal(io.cpu().numpy(), _ref_rows(keys, dim))
        size = t.size()
        ek, ev, es = export_table(t, dim * 4)
        assert len(ek) == size and len(np.unique(ek)) == size
        assert np.array_equal(ev.view(np.float32), _ref_rows(ek, dim))
        assert t.capacity() == cap and size > 0.9 * cap
        assert np.isin(ek, keys).mean() > 0.9  # LRU: what stays is mostly the newest batch
    t.close()
