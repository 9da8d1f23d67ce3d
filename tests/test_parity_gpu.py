"""GPU parity: the HIP table (through the C ABI) against the CPU oracle on the
same seeded inputs.  Bit-exact: found flags, returned values and scores,
resident (key -> value, score) maps, sizes, evicted sets.

Preconditions that make the concurrent kernels' result order-independent (and
therefore comparable with the oracle's sequential pass): keys are unique per
batch, scores are pairwise distinct and never lower a resident key's score
(deterministic clock for LRU strategies, batch-monotone scores for Customized).
"""
import numpy as np
import pytest
import torch

import workloads as w
from gpu_util import (DEV, assert_same_table, canonical_evicted, dev, export_table, host_bytes,
                      host_u64, read_device, sort_by_key)
from hierarchicalkv_amd import (EvictStrategy, HashTable, MerlinException, Predicate, ValueKind,
                                default_options)

pytestmark = pytest.mark.gpu


def make_pair(oracle, hybrid=False, **kw):
    kw.setdefault("max_hbm_for_vectors", 1 << 34)
    o = default_options(**kw)
    t = HashTable()
    t.init(o)
    return t, oracle.OracleTable(o, hybrid=hybrid), o


def bytes_of(vals):
    return np.ascontiguousarray(vals).view(np.uint8).reshape(len(vals), -1)


def gpu_find(table, keys, dim, dtype=torch.float32, fill=0):
    n = len(keys)
    out = torch.full((n, dim), fill, dtype=dtype, device=DEV)
    founds = torch.zeros(n, dtype=torch.bool, device=DEV)
    scores = torch.zeros(n, dtype=torch.int64, device=DEV)
    table.find(n, dev(keys), out, founds, scores)
    torch.cuda.synchronize()
    return out.cpu().numpy(), founds.cpu().numpy(), host_u64(scores)


def check_find(table, oracle, keys, dim):
    gv, gf, gs = gpu_find(table, keys, dim)
    ov, of, os_ = oracle.find(keys)
    assert (gf == of).all()
    assert (bytes_of(gv)[gf] == ov[of]).all()
    assert (gs[gf] == os_[of]).all()
    assert (gv[~gf] == 0).all()  # misses leave the output untouched
    return gf


# ---- config 1: the small verification table, exactly as specified ------------------------------

def test_config1_lru_insert_then_find(oracle):
    cap, dim, bs = 1 << 20, 16, 65536
    t, o, _ = make_pair(oracle, init_capacity=cap, max_capacity=cap, dim=dim, evict_strategy=EvictStrategy.kLru)
    t.set_clock(1, 1 << 40)
    o.set_clock(1, 1 << 40)
    seed = 0x484B5601
    for b in range(12):  # 12 * 65536 = 0.75 * 2^20
        keys = w.unique_keys(seed, b * bs, bs)
        vals = w.values_from_keys(keys, dim)
        t.insert_or_assign(bs, dev(keys), dev(vals))
        o.insert_or_assign(keys, bytes_of(vals))
    torch.cuda.synchronize()
    assert t.size() == o.size()
    assert abs(t.load_factor() - o.size() / cap) < 1e-6
    q = np.concatenate([w.unique_keys(seed, 3 * bs + 5, bs // 2), w.unique_keys(seed, 100 * bs, bs // 2)])
    gf = check_find(t, o, q, dim)
    assert gf[: bs // 2].sum() > 0 and not gf[bs // 2:].any()
    assert_same_table(t, o, dim * 4)
    t.close()


# ---- config 2 at reduced capacity: find / insert_or_assign / find_or_insert at three load factors ----

def test_config2_load_factor_sweep(oracle):
    cap, dim, bs = 1 << 20, 8, 1 << 16
    t, o, _ = make_pair(oracle, init_capacity=cap, max_capacity=cap, dim=dim, evict_strategy=EvictStrategy.kLru)
    t.set_clock(1, 1 << 40)
    o.set_clock(1, 1 << 40)
    seed = 0x484B5602
    filled = 0
    for lf in (0.50, 0.75, 1.00):
        while filled < int(cap * lf):
            keys = w.unique_keys(seed, filled, bs)
            vals = w.uniform_values(seed, filled, bs, dim)
            t.insert_or_assign(bs, dev(keys), dev(vals))
            o.insert_or_assign(keys, bytes_of(vals))
            filled += bs
        assert t.size() == o.size()
        # find, 100 % resident candidates (some were evicted or never fitted at lf 1.0)
        q = w.unique_keys(seed, filled - bs, bs)
        check_find(t, o, q, dim)
        # insert_or_assign, 50 % new keys
        keys = np.concatenate([w.unique_keys(seed, filled - bs // 2, bs // 2),
                               w.unique_keys(seed + 1000, filled, bs // 2)])
        vals = w.uniform_values(seed + 1, filled, bs, dim)
        t.insert_or_assign(bs, dev(keys), dev(vals))
        o.insert_or_assign(keys, bytes_of(vals))
        assert t.size() == o.size()
        # find_or_insert on a half-known batch: hits read, misses insert
        # (the known half is recent, i.e. high-scored: a hit that another key of
        # the same batch could evict first would make the outcome order-dependent)
        keys = np.concatenate([w.unique_keys(seed, filled - bs, bs // 2),
                               w.unique_keys(seed + 2000, filled, bs // 2)])
        vals = w.uniform_values(seed + 2, filled, bs, dim)
        d_vals = dev(vals)
        t.find_or_insert(bs, dev(keys), d_vals)
        ovals = bytes_of(vals).copy()
        o.find_or_insert(keys, ovals)
        torch.cuda.synchronize()
        assert (host_bytes(d_vals, bs, dim * 4) == ovals).all()
        assert_same_table(t, o, dim * 4)
    t.close()


# ---- config 3 at reduced capacity: Zipf keys, Customized scores, insert_and_evict at lf 1.0 -------------

def test_config3_insert_and_evict_zipf(oracle):
    cap, dim, bs = 1 << 18, 64, 1 << 15
    t, o, _ = make_pair(oracle, init_capacity=cap, max_capacity=cap, dim=dim,
                        evict_strategy=EvictStrategy.kCustomized)
    seed = 0x484B5603
    pos = 0
    ek = torch.zeros(bs, dtype=torch.int64, device=DEV)
    ev = torch.zeros(bs, dim, dtype=torch.float32, device=DEV)
    es = torch.zeros(bs, dtype=torch.int64, device=DEV)
    total_evicted = 0
    for b in range(16):  # 16 * 32768 = 2 * capacity worth of (partly repeated) keys
        keys, pos = w.zipf_unique_keys(seed, pos, bs, universe_bits=22)
        vals = w.values_from_keys(keys, dim)
        scores = w.monotone_scores(b + 1, bs, seed=3)
        cnt = t.insert_and_evict(bs, dev(keys), dev(vals), dev(scores), ek, ev, es)
        oek, oev, oes = o.insert_and_evict(keys, bytes_of(vals), scores)
        assert t.size() == o.size()
        gk, gv, gs = sort_by_key(*export_table(t, dim * 4))
        a = canonical_evicted(host_u64(ek[:cnt]), host_bytes(ev[:cnt], cnt, dim * 4), host_u64(es[:cnt]), gk)
        bb = canonical_evicted(oek, oev, oes, gk)
        assert len(a[0]) == len(bb[0])
        assert (a[0] == bb[0]).all() and (a[1] == bb[1]).all() and (a[2] == bb[2]).all()
        total_evicted += cnt
    assert total_evicted > 0
    assert_same_table(t, o, dim * 4)
    # find on the same Zipf stream
    q, _ = w.zipf_unique_keys(seed, 0, bs, universe_bits=22)
    check_find(t, o, q, dim)
    t.close()


@pytest.mark.parametrize("strategy", [EvictStrategy.kLru, EvictStrategy.kCustomized])
def test_insert_and_evict_ragged_batches_on_a_full_table(oracle, strategy):
    """On a full table the kernel runs two wavefronts of 64 keys per workgroup that claim their
    entries of the evicted-keys output together: batches that fill neither, one, or one and a
    bit of a workgroup, and larger ragged ones."""
    cap, dim = 1 << 14, 8
    t, o, _ = make_pair(oracle, init_capacity=cap, max_capacity=cap, dim=dim, evict_strategy=strategy)
    lru = strategy == EvictStrategy.kLru
    if lru:
        t.set_clock(1, 1 << 40)
        o.set_clock(1, 1 << 40)
    seed, pos, batch = 0x484B5611, 0, 1

    def scores_for(n):
        return None if lru else w.monotone_scores(batch, n, seed=11)

    while pos < 2 * cap:  # twice the capacity: every bucket is full
        keys = w.unique_keys(seed, pos, 4096)
        vals = w.values_from_keys(keys, dim)
        sc = scores_for(4096)
        t.insert_or_assign(4096, dev(keys), dev(vals), None if sc is None else dev(sc))
        o.insert_or_assign(keys, bytes_of(vals), sc)
        pos += 4096
        batch += 1
    assert t.size() == o.size()
    for n in (1, 63, 64, 65, 127, 128, 129, 1000, 4097):
        # half resident (from the last batches), half new
        keys = np.concatenate([w.unique_keys(seed, pos - n, n // 2), w.unique_keys(seed, pos, n - n // 2)])
        pos += n
        vals = w.values_from_keys(keys, dim) + np.float32(batch)
        sc = scores_for(n)
        ek = torch.zeros(n, dtype=torch.int64, device=DEV)
        ev = torch.zeros(n, dim, dtype=torch.float32, device=DEV)
        es = torch.zeros(n, dtype=torch.int64, device=DEV)
        cnt = t.insert_and_evict(n, dev(keys), dev(vals), None if sc is None else dev(sc), ek, ev, es)
        oek, oev, oes = o.insert_and_evict(keys, bytes_of(vals), sc)
        assert cnt == len(oek), n
        gk, _, _ = sort_by_key(*export_table(t, dim * 4))
        a = canonical_evicted(host_u64(ek[:cnt]), host_bytes(ev[:cnt], cnt, dim * 4), host_u64(es[:cnt]), gk)
        b = canonical_evicted(oek, oev, oes, gk)
        assert (a[0] == b[0]).all() and (a[1] == b[1]).all() and (a[2] == b[2]).all(), n
        assert len(np.unique(host_u64(ek[:cnt]))) == cnt, n  # no entry claimed twice, none left out
        batch += 1
    assert_same_table(t, o, dim * 4)
    t.close()


# ---- config 5 at reduced capacity: EpochLRU, accum_or_assign, export_batch_if, erase -----------------------

def test_config5_accum_export_erase(oracle):
    cap, dim, bs = 1 << 16, 128, 1 << 13
    t, o, _ = make_pair(oracle, init_capacity=cap, max_capacity=cap, dim=dim,
                        evict_strategy=EvictStrategy.kEpochLru)
    t.set_clock(1, 1 << 40)
    o.set_clock(1, 1 << 40)
    seed = 0x484B5605
    filled = 0
    batch = 0

    def epoch():
        t.set_global_epoch(batch // 10)
        o.set_global_epoch(batch // 10)

    while filled < cap + 2 * bs:  # past lf 1.0
        epoch()
        keys = w.unique_keys(seed, filled, bs)
        vals = w.uniform_values(seed, filled, bs, dim)
        t.insert_or_assign(bs, dev(keys), dev(vals))
        o.insert_or_assign(keys, bytes_of(vals))
        filled += bs
        batch += 1
    for rep in range(6):
        epoch()
        # 70 % candidates from a recent insert batch (high scores, so no other key
        # of this batch can evict them first), 30 % new; flags from a preceding find
        old = w.unique_keys(seed, filled - 2 * bs, bs)[: bs * 7 // 10]
        keys = np.concatenate([old, w.unique_keys(seed + 50, rep * bs, bs - len(old))])
        deltas = (w.uniform_values(seed + 7, rep * bs, bs, dim) * np.float32(0.01)).astype(np.float32)
        founds = torch.zeros(bs, dtype=torch.bool, device=DEV)
        t.contains(bs, dev(keys), founds)
        torch.cuda.synchronize()
        flags = founds.cpu().numpy()
        assert (flags == o.contains(keys)).all()
        t.accum_or_assign(bs, dev(keys), dev(deltas), founds)
        o.accum_or_assign(keys, bytes_of(deltas), flags.astype(np.uint8))
        batch += 1
        assert t.size() == o.size()
        assert o.contains(keys[flags]).all(), "input hazard: an accum key was evicted inside its batch"
    assert_same_table(t, o, dim * 4)
    # export_batch_if with score >= threshold keeping about a quarter
    _, _, os_ = o.export_all()
    thr = int(np.sort(os_)[len(os_) * 3 // 4])
    gk, gv, gs = sort_by_key(*export_table(t, dim * 4, Predicate.kScoreGe, 0, thr))
    ok, ov, oss = sort_by_key(*o.export_batch_if(Predicate.kScoreGe, 0, thr))
    assert len(gk) == len(ok) and abs(len(gk) / len(os_) - 0.25) < 0.01
    assert (gk == ok).all() and (gv == ov).all() and (gs == oss).all()
    assert t.size_if(Predicate.kScoreGe, 0, thr) == len(ok)
    # erase
    gone = np.concatenate([w.unique_keys(seed, filled - 3 * bs, bs), w.unique_keys(seed + 99, 0, bs)])
    t.erase(len(gone), dev(gone))
    o.erase(gone)
    assert t.size() == o.size()
    assert_same_table(t, o, dim * 4)
    # the tombstones are reused
    keys = w.unique_keys(seed + 123, 0, bs)
    vals = w.uniform_values(seed + 9, 0, bs, dim)
    t.insert_or_assign(bs, dev(keys), dev(vals))
    o.insert_or_assign(keys, bytes_of(vals))
    assert_same_table(t, o, dim * 4)
    t.clear()
    o.clear()
    assert t.size() == 0 and t.empty()
    assert_same_table(t, o, dim * 4)
    t.close()
