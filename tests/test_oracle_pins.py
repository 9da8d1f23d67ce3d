"""Pins for the CPU oracle (no GPU needed).

The reference cannot be executed here and its tests hold no golden vectors
(their inputs are unseeded), so every check below is either a known answer
that the mathematics fixes, a closed-form scenario taken from one of the
reference's own tests (cited), or an independent brute-force model written
differently from the oracle (python dicts and sorting instead of buckets).
"""
import numpy as np
import pytest

import workloads as w
from hierarchicalkv_amd import EvictStrategy, Predicate, ValueKind, default_options

M64 = (1 << 64) - 1


# ---- hash --------------------------------------------------------------------

def test_fmix64_known_answers(oracle):
    # closed-form evaluations of MurmurHash3's 64-bit finaliser
    # (reference: utils.cuh:127-135; host twin tests/test_util.cuh:272-280)
    assert oracle.fmix64(0) == 0
    assert oracle.fmix64(1) == 0xB456BCFC34C2CB2C
    assert oracle.fmix64(2) == 0x3ABF2A20650683E7
    assert oracle.fmix64(0x0123456789ABCDEF) == 0x87CBFBFE89022CEA
    assert oracle.fmix64(M64) == 0x64B5720B4B825F21
    assert oracle.fmix64(M64 - 1) == 0x3A8593886C55A02B


def test_fmix64_is_inverted_by_the_published_inverse(oracle):
    # fmix64 is a bijection; its inverse uses the modular inverses of the two
    # multipliers.  A wrong constant or shift in the oracle breaks the round trip.
    def unxorshift33(x):
        return x ^ (x >> 33)  # shift >= 32: one application undoes itself

    def inverse(h):
        h = unxorshift33(h)
        h = (h * 0x9CB4B2F8129337DB) & M64
        h = unxorshift33(h)
        h = (h * 0x4F74430C22A54005) & M64
        return unxorshift33(h)

    assert (0xFF51AFD7ED558CCD * 0x4F74430C22A54005) & M64 == 1
    assert (0xC4CEB9FE1A85EC53 * 0x9CB4B2F8129337DB) & M64 == 1
    for k in [0, 1, 2, 12345, 0xDEADBEEFCAFEF00D, M64, M64 - 7] + [int(x) for x in w.stream(7, 0, 200)]:
        assert inverse(oracle.fmix64(k)) == k


def test_sentinel_digests(oracle):
    # digest = hash bits 32..39 (kernel_utils.cuh:72-96)
    assert (oracle.fmix64(M64) >> 32) & 0xFF == 0x0B       # EMPTY
    assert (oracle.fmix64(M64 - 1) >> 32) & 0xFF == 0x88   # RECLAIM


# ---- addressing ----------------------------------------------------------------

def test_locate_matches_test_util_bucket_formula(oracle):
    # tests/test_util.cuh:296-331: bkt = (hash & (capacity - 1)) / 128 for a
    # power-of-two capacity; start = (global % 128) rounded down to 4
    cap = 1 << 20
    assert oracle.locate(1, cap // 128) == (1430, 44, 0xFC)
    for k in [int(x) for x in w.stream(11, 0, 500)]:
        h = oracle.fmix64(k)
        g = h & (cap - 1)
        b, s, d = oracle.locate(k, cap // 128)
        assert b == g // 128
        assert s == (g % 128) // 4 * 4
        assert d == (h >> 32) & 0xFF


def test_locate_uses_modulo_for_other_capacities(oracle):
    nb = 524287
    for k in [int(x) for x in w.stream(13, 0, 300)]:
        h = oracle.fmix64(k)
        g = h % (nb * 128)
        assert oracle.locate(k, nb)[:2] == (g // 128, (g % 128) // 4 * 4)


def test_bucket_count_rule(oracle):
    # tests/merlin_hashtable_test.cc.cu:180-182, 242: capacity 64M - 129 with
    # init == max gives 524287 buckets (no rounding to a power of two)
    o = default_options(init_capacity=64 * 1024 * 1024 - 129, max_capacity=64 * 1024 * 1024 - 129,
                        dim=1, value_size=1, value_kind=ValueKind.kBytes, reserved_key_start_bit=2,
                        num_of_buckets_per_alloc=32, evict_strategy=EvictStrategy.kCustomized)
    t = oracle.OracleTable(o)
    assert t.bucket_count() == 524287
    assert t.capacity() == 524287 * 128
    t.close()
    # growable table (init * 2 <= max): next power of two of init / 128
    o = default_options(init_capacity=1000, max_capacity=1 << 20, dim=1, value_size=1,
                        value_kind=ValueKind.kBytes)
    t = oracle.OracleTable(o)
    assert t.bucket_count() == 8
    t.close()


# ---- reserved keys ---------------------------------------------------------------

def test_reserved_key_truth_table(oracle):
    # tests/reserved_keys_test.cc.cu:84-97
    for bit in range(0, 63):
        empty, reclaim, locked, rm1, rm2, vm1, vm2 = oracle.reserved_keys(bit)
        is_reserved = lambda k: (k & rm1) == rm2
        assert is_reserved(empty) and is_reserved(reclaim) and is_reserved(locked)
        assert not is_reserved(0) and not is_reserved(0x10)
        assert is_reserved(M64) == (bit == 0)
        assert len({empty, reclaim, locked}) == 3
        is_vacant = lambda k: (k & vm1) == vm2
        assert is_vacant(empty) and is_vacant(reclaim) and not is_vacant(locked)
    assert oracle.reserved_keys(0)[:3] == [M64, M64 - 1, M64 - 2]
    with pytest.raises(ValueError):
        oracle.reserved_keys(63)


def test_reserved_keys_are_skipped_by_every_op(oracle):
    o = default_options(init_capacity=1024, max_capacity=1024, dim=2, evict_strategy=EvictStrategy.kCustomized)
    t = oracle.OracleTable(o)
    keys = np.array([M64, M64 - 1, M64 - 2, M64 - 3, 5], np.uint64)
    vals = np.arange(10, dtype=np.float32).reshape(5, 2).view(np.uint8).reshape(5, 8)
    t.insert_or_assign(keys, vals, np.arange(5, dtype=np.uint64) + 1)
    assert t.size() == 1
    _, founds, _ = t.find(keys)
    assert founds.tolist() == [False, False, False, False, True]
    t.close()


# ---- helpers ------------------------------------------------------------------------

def keys_in_bucket(oracle, n, nb, bucket, seed, lo=0, hi=M64 - 3):
    """Rejection sampling as create_keys_in_one_buckets (test_util.cuh:296-331)."""
    out = []
    pos = 0
    seen = set()
    while len(out) < n:
        for k in w.stream(seed, pos, 4096):
            k = int(k) % (hi - lo) + lo
            if k in seen:
                continue
            if oracle.locate(k, nb)[0] == bucket:
                seen.add(k)
                out.append(k)
                if len(out) == n:
                    break
        pos += 4096
    return np.array(out, np.uint64)


def vals_of(keys, dim):
    """v[i][j] = float(key * 0.00001) (test_util.cuh:160-163)."""
    v = (keys.astype(np.float64) * 0.00001).astype(np.float32)
    return np.repeat(v[:, None], dim, axis=1).copy().view(np.uint8).reshape(len(keys), dim * 4)


def as_map(keys, values, scores):
    return {int(k): (values[i].tobytes(), int(scores[i])) for i, k in enumerate(keys)}


# ---- eviction scenarios from the reference's tests -----------------------------------------

def test_customized_basic(oracle):
    # tests/merlin_hashtable_test.cc.cu:2674-2849
    o = default_options(init_capacity=1024, max_capacity=1024, dim=4, reserved_key_start_bit=15,
                        num_of_buckets_per_alloc=8, evict_strategy=EvictStrategy.kCustomized)
    base = keys_in_bucket(oracle, 128, 8, 1, 21, 0, 0x3FFFFFFFFFFFFFFF)
    test = keys_in_bucket(oracle, 128, 8, 1, 22, 0x3FFFFFFFFFFFFFFF, 0xFFFFFFFFFFFFFFFD)
    test[64:] = base[64:]
    bs = np.arange(1000, 1128, dtype=np.uint64)
    ts = np.arange(1128, 1256, dtype=np.uint64)
    t = oracle.OracleTable(o)
    assert t.size() == 0
    t.insert_or_assign(base, vals_of(base, 4), bs)
    assert t.size() == 128
    k, v, s = t.export_all()
    assert sorted(s.tolist()) == list(range(1000, 1128))
    assert (v == vals_of(k, 4)).all()
    t.insert_or_assign(test, vals_of(test, 4), ts)
    assert t.size() == 128
    k, v, s = t.export_all()
    assert len(k) == 128
    assert sorted(s.tolist()) == list(range(1128, 1256))
    assert (v == vals_of(k, 4)).all()
    t.close()


def test_customized_advanced(oracle):
    # tests/merlin_hashtable_test.cc.cu:2851-3053: four low-score keys are
    # refused, four resident keys are re-scored (one of them downwards)
    o = default_options(init_capacity=1024, max_capacity=1024, dim=4, reserved_key_start_bit=16,
                        num_of_buckets_per_alloc=8, evict_strategy=EvictStrategy.kCustomized)
    base = keys_in_bucket(oracle, 128, 8, 1, 31, 0, 0x3FFFFFFFFFFFFFFF)
    test = keys_in_bucket(oracle, 8, 8, 1, 32, 0x3FFFFFFFFFFFFFFF, 0xFFFFFFFFFFFFFFFD)
    test[4:8] = base[72:76]
    ts = np.array([20, 78, 97, 98, 99, 1010, 1020, 1035], np.uint64)
    t = oracle.OracleTable(o)
    assert t.bucket_count() == 8
    t.insert_or_assign(base, vals_of(base, 4), np.arange(1000, 1128, dtype=np.uint64))
    t.insert_or_assign(test, vals_of(test, 4), ts)
    assert t.size() == 128
    k, v, s = t.export_all()
    resident = as_map(k, v, s)
    for i in range(4):
        assert int(test[i]) not in resident
    for i in range(4, 8):
        assert resident[int(test[i])][1] == int(ts[i])
    assert (v == vals_of(k, 4)).all()
    t.close()


def test_full_bucket_keeps_the_top_128_scores(oracle):
    """Brute force: with distinct scores that never go down, the residents of a
    full bucket are the 128 best of (old residents + batch), whatever the order
    inside the batch.  The model below knows nothing about slots or digests."""
    nb = 4
    o = default_options(init_capacity=nb * 128, max_capacity=nb * 128, dim=2,
                        evict_strategy=EvictStrategy.kCustomized)
    rng = np.random.Generator(np.random.PCG64(5))
    for trial in range(6):
        t = oracle.OracleTable(o)
        model = {}  # key -> (value bytes, score), per bucket resident sets derived by sorting
        universe = w.unique_keys(100 + trial, 0, 3000)
        for batch in range(8):
            keys = rng.choice(universe, size=400, replace=False)
            scores = w.monotone_scores(batch + 1, len(keys), seed=trial)
            vals = rng.integers(0, 255, size=(len(keys), 8), dtype=np.uint8)
            order = rng.permutation(len(keys))
            t.insert_or_assign(keys[order].copy(), vals[order].copy(), scores[order].copy())
            for i in range(len(keys)):
                model[int(keys[i])] = (vals[i].tobytes(), int(scores[i]))
            # keep the best 128 per bucket
            by_bucket = {}
            for k, (vv, sc) in model.items():
                by_bucket.setdefault(oracle.locate(k, nb)[0], []).append((sc, k))
            model = {k: model[k] for b in by_bucket.values() for sc, k in sorted(b, reverse=True)[:128]}
            k, v, s = t.export_all()
            assert as_map(k, v, s) == model
            assert t.size() == len(model)
        t.close()


def test_refusal_rule_strict_vs_hybrid(oracle):
    # pure HBM refuses on score < min (upsert.cuh:188), hybrid on score <= min (upsert.cuh:1524)
    o = default_options(init_capacity=128, max_capacity=128, dim=1, evict_strategy=EvictStrategy.kCustomized)
    base = w.unique_keys(1, 0, 128)
    vals = np.zeros((128, 4), np.uint8)
    extra = w.unique_keys(2, 0, 1)
    for hybrid, expect_in in ((False, True), (True, False)):
        t = oracle.OracleTable(o, hybrid=hybrid)
        t.insert_or_assign(base, vals, np.arange(10, 138, dtype=np.uint64))
        t.insert_or_assign(extra, vals[:1], np.array([10], np.uint64))  # equal to the minimum
        assert t.contains(extra)[0] == expect_in
        assert t.size() == 128
        t.close()


def test_hybrid_batch_holds_every_slot_it_took(oracle):
    # upsert.cuh:1350-1595 (find_or_insert.cuh:1417-1676): the lock kernel of the hybrid upsert
    # leaves the slot of every key of the batch LOCKED until the write kernel has run, and its
    # victim scan passes LOCKED slots over.  Worked by hand for one full bucket whose residents
    # score 100, 110, ... and the batch 105, 200, 115, 125, 99 in this order:
    #   105 > 100: takes the slot of 100          200: lowest visible is 110, takes it
    #   115: lowest visible is 120, refused        125 > 120: takes the slot of 120
    #   99: lowest visible is 130, refused
    # One key at a time (each call releases its slot) the same keys end differently:
    #   105 takes 100's slot, 200 takes 105's, 115 takes 110's, 125 takes 115's, 99 is refused.
    o = default_options(init_capacity=128, max_capacity=128, dim=1, max_hbm_for_vectors=0,
                        evict_strategy=EvictStrategy.kCustomized)
    base = w.unique_keys(1, 0, 128)
    vals = np.zeros((128, 4), np.uint8)
    sc = np.arange(100, 100 + 10 * 128, 10, dtype=np.uint64)
    batch = w.unique_keys(2, 0, 5)
    bsc = np.array([105, 200, 115, 125, 99], np.uint64)

    def scores_of(t):
        _, _, s = t.export_all()
        return sorted(s.tolist())

    t = oracle.OracleTable(o, hybrid=True)
    t.insert_or_assign(base, vals, sc)
    t.insert_or_assign(batch, vals[:5], bsc)
    assert scores_of(t) == sorted([x for x in sc.tolist() if x not in (100, 110, 120)] + [105, 200, 125])
    assert list(t.contains(batch)) == [True, True, False, True, False]
    t.close()
    t = oracle.OracleTable(o, hybrid=True)
    t.insert_or_assign(base, vals, sc)
    for i in range(5):
        t.insert_or_assign(batch[i:i + 1], vals[:1], bsc[i:i + 1])
    assert scores_of(t) == sorted([x for x in sc.tolist() if x not in (100, 110)] + [200, 125])
    t.close()
    # find_or_insert follows the same kernels
    t = oracle.OracleTable(o, hybrid=True)
    t.insert_or_assign(base, vals, sc)
    t.find_or_insert(batch, vals[:5].copy(), bsc)
    assert scores_of(t) == sorted([x for x in sc.tolist() if x not in (100, 110, 120)] + [105, 200, 125])
    t.close()


# ---- insert_and_evict ------------------------------------------------------------------------

def test_insert_and_evict_conservation(oracle):
    # tests/insert_and_evict_test.cc.cu:34-48, 94, 115, 287-311:
    # table_before + batch == table_after + evicted (as key -> value maps) and
    # n_evicted + size_after == size_before + n_new.  Batches of never-seen keys,
    # as in the reference's test, so no key is updated and evicted in one batch.
    o = default_options(init_capacity=1024, max_capacity=1024, dim=2, evict_strategy=EvictStrategy.kCustomized)
    t = oracle.OracleTable(o)
    for batch in range(10):
        keys = w.unique_keys(9, batch * 700, 700)
        vals = vals_of(keys, 2)
        scores = w.monotone_scores(batch + 1, len(keys), seed=3)
        bk, bv, bs = t.export_all()
        before = as_map(bk, bv, bs)
        size_before = t.size()
        ek, ev, es = t.insert_and_evict(keys, vals, scores)
        ak, av, as_ = t.export_all()
        after = as_map(ak, av, as_)
        assert len(ek) + t.size() == size_before + len(keys)
        union_in = {k: v[0] for k, v in before.items()}
        union_in.update({int(k): vals[i].tobytes() for i, k in enumerate(keys)})
        union_out = {k: v[0] for k, v in after.items()}
        assert not (set(union_out) & set(int(k) for k in ek))
        union_out.update({int(k): ev[i].tobytes() for i, k in enumerate(ek)})
        assert union_in == union_out
        # every evicted or refused key scores below everything left in its bucket
        mins = {}
        for k, (_, sc) in after.items():
            b = oracle.locate(k, 8)[0]
            mins[b] = min(mins.get(b, M64), sc)
        for i, k in enumerate(ek):
            assert int(es[i]) < mins[oracle.locate(int(k), 8)[0]]
        # evicted scores are the scores those keys had (or were offered)
        offered = {int(k): int(scores[i]) for i, k in enumerate(keys)}
        for i, k in enumerate(ek):
            k = int(k)
            assert int(es[i]) == (before[k][1] if k in before else offered[k])
    t.close()


def test_insert_and_evict_with_updates_is_conservative_after_canonicalisation(oracle):
    """Keys that are updated by a batch may be evicted earlier in the same batch
    (with their old row) and come back; such entries are dropped before
    comparing, everything else is conserved."""
    o = default_options(init_capacity=1024, max_capacity=1024, dim=2, evict_strategy=EvictStrategy.kCustomized)
    t = oracle.OracleTable(o)
    universe = w.unique_keys(9, 0, 6000)
    rng = np.random.Generator(np.random.PCG64(1))
    for batch in range(10):
        keys = rng.choice(universe, size=700, replace=False)
        vals = rng.integers(0, 255, size=(700, 8), dtype=np.uint8)
        scores = w.monotone_scores(batch + 1, len(keys), seed=3)
        bk, bv, bs = t.export_all()
        before = as_map(bk, bv, bs)
        ek, ev, es = t.insert_and_evict(keys, vals, scores)
        ak, av, as_ = t.export_all()
        after = as_map(ak, av, as_)
        gone = {int(k): ev[i].tobytes() for i, k in enumerate(ek) if int(k) not in after}
        final_in = {k: v[0] for k, v in before.items()}
        final_in.update({int(k): vals[i].tobytes() for i, k in enumerate(keys)})
        final_out = {k: v[0] for k, v in after.items()}
        final_out.update(gone)
        assert final_in == final_out
    t.close()


def test_reclaimed_slots_are_reused_without_eviction_output(oracle):
    o = default_options(init_capacity=128, max_capacity=128, dim=1, evict_strategy=EvictStrategy.kCustomized)
    t = oracle.OracleTable(o)
    base = w.unique_keys(4, 0, 128)
    vals = np.zeros((128, 4), np.uint8)
    t.insert_or_assign(base, vals, np.arange(100, 228, dtype=np.uint64))
    t.erase(base[:10])
    assert t.size() == 118
    new = w.unique_keys(5, 0, 12)
    ek, ev, es = t.insert_and_evict(new, vals[:12], np.arange(300, 312, dtype=np.uint64))
    # ten tombstones absorb ten keys silently; the other two evict scores 110, 111
    assert t.size() == 128
    assert sorted(es.tolist()) == [110, 111]
    assert sorted(ek.tolist()) == sorted(base[10:12].tolist())
    t.close()


# ---- score strategies ------------------------------------------------------------------------------

def test_lfu_scores_add_up(oracle):
    # tests/insert_and_evict_test.cc.cu:541-556: score after == increment + score before
    o = default_options(init_capacity=1024, max_capacity=1024, dim=1, evict_strategy=EvictStrategy.kLfu)
    t = oracle.OracleTable(o)
    keys = w.unique_keys(6, 0, 300)
    vals = np.zeros((300, 4), np.uint8)
    t.insert_or_assign(keys, vals, np.full(300, 3, np.uint64))
    t.insert_or_assign(keys[:100], vals[:100], np.full(100, 5, np.uint64))
    _, f, s = t.find(keys)
    assert f.all()
    assert (s[:100] == 8).all() and (s[100:] == 3).all()
    with pytest.raises(oracle.OracleError):
        t.insert_or_assign(keys, vals, None)  # LFU needs scores (merlin_hashtable.cuh:3840-3845)
    t.close()


def test_epoch_lfu_score_format(oracle):
    # tests/test_util.cuh:371-376: (epoch << 32) | min(freq, 0xFFFFFFFF)
    o = default_options(init_capacity=1024, max_capacity=1024, dim=1, evict_strategy=EvictStrategy.kEpochLfu)
    t = oracle.OracleTable(o)
    keys = w.unique_keys(7, 0, 4)
    vals = np.zeros((4, 4), np.uint8)
    with pytest.raises(oracle.OracleError):
        t.insert_or_assign(keys, vals, np.ones(4, np.uint64))  # epoch not set (:3853-3860)
    t.set_global_epoch(7)
    t.insert_or_assign(keys, vals, np.array([1, 2, 0xFFFFFFF0, 0x1FFFFFFFF], np.uint64))
    _, _, s = t.find(keys)
    assert s.tolist() == [(7 << 32) | 1, (7 << 32) | 2, (7 << 32) | 0xFFFFFFF0, (7 << 32) | 0xFFFFFFFF]
    t.set_global_epoch(9)
    t.insert_or_assign(keys, vals, np.array([1, 2, 0x20, 5], np.uint64))
    _, _, s = t.find(keys)
    # low half adds and saturates, high half takes the new epoch
    assert s.tolist() == [(9 << 32) | 2, (9 << 32) | 4, (9 << 32) | 0xFFFFFFFF, (9 << 32) | 0xFFFFFFFF]
    t.close()


def test_lru_and_epoch_lru_with_deterministic_clock(oracle):
    for strat in (EvictStrategy.kLru, EvictStrategy.kEpochLru):
        o = default_options(init_capacity=1024, max_capacity=1024, dim=1, evict_strategy=strat)
        t = oracle.OracleTable(o)
        t.set_clock(1, 5 << 40)
        if strat == EvictStrategy.kEpochLru:
            t.set_global_epoch(3)
        keys = w.unique_keys(8, 0, 8)
        vals = np.zeros((8, 4), np.uint8)
        with pytest.raises(oracle.OracleError):
            t.insert_or_assign(keys, vals, np.ones(8, np.uint64))  # LRU takes no scores
        t.insert_or_assign(keys, vals)
        _, _, s = t.find(keys)
        now = [(5 << 40) + (i << 20) for i in range(8)]
        if strat == EvictStrategy.kLru:
            assert s.tolist() == now
        else:
            assert s.tolist() == [(3 << 32) | ((x >> 20) & 0xFFFFFFFF) for x in now]
        t.close()


# ---- accum_or_assign -------------------------------------------------------------------------------------

def test_accum_or_assign_truth_table(oracle):
    # tests/accum_or_assign_test.cc.cu:2818-2845
    o = default_options(init_capacity=1024, max_capacity=1024, dim=3, evict_strategy=EvictStrategy.kCustomized)
    t = oracle.OracleTable(o)
    keys = w.unique_keys(10, 0, 8)
    base = np.arange(24, dtype=np.float32).reshape(8, 3)
    t.insert_or_assign(keys[:4], base[:4].copy().view(np.uint8).reshape(4, 12), np.arange(1, 5, dtype=np.uint64))
    delta = np.full((8, 3), 0.5, np.float32)
    flags = np.array([1, 0, 1, 0, 1, 0, 1, 0], np.uint8)  # accum / assign alternating
    t.accum_or_assign(keys, delta.view(np.uint8).reshape(8, 12), flags, np.arange(11, 19, dtype=np.uint64))
    v, f, s = t.find(keys)
    v = v.view(np.float32).reshape(8, 3)
    # existed & accum -> old + delta ; existed & assign -> unchanged
    assert f.tolist() == [True, True, True, True, False, True, False, True]
    assert (v[0] == base[0] + 0.5).all() and s[0] == 11
    assert (v[1] == base[1]).all() and s[1] == 2
    assert (v[2] == base[2] + 0.5).all() and s[2] == 13
    assert (v[3] == base[3]).all() and s[3] == 4
    # missing & assign -> inserted with the delta as value ; missing & accum -> nothing
    assert (v[5] == 0.5).all() and s[5] == 16
    assert (v[7] == 0.5).all() and s[7] == 18
    assert t.size() == 6
    t.close()


# ---- find_or_insert, assign family -------------------------------------------------------------------------

def test_find_or_insert_reads_hits_and_writes_misses(oracle):
    o = default_options(init_capacity=1024, max_capacity=1024, dim=2, evict_strategy=EvictStrategy.kCustomized)
    t = oracle.OracleTable(o)
    keys = w.unique_keys(12, 0, 6)
    old = np.arange(6, dtype=np.float32).reshape(3, 2)
    t.insert_or_assign(keys[:3], old.copy().view(np.uint8).reshape(3, 8), np.array([5, 6, 7], np.uint64))
    io = np.full((6, 2), 9.0, np.float32).view(np.uint8).reshape(6, 8).copy()
    t.find_or_insert(keys, io, np.arange(20, 26, dtype=np.uint64))
    got = io.view(np.float32).reshape(6, 2)
    assert (got[:3] == old).all() and (got[3:] == 9.0).all()
    v, f, s = t.find(keys)
    assert f.all()
    assert s.tolist() == [20, 21, 22, 23, 24, 25]  # Customized: hit re-scores (kernel_utils.cuh:581-593)
    assert (v.view(np.float32).reshape(6, 2)[3:] == 9.0).all()
    t.close()


def test_assign_family_never_inserts(oracle):
    o = default_options(init_capacity=1024, max_capacity=1024, dim=2, evict_strategy=EvictStrategy.kCustomized)
    t = oracle.OracleTable(o)
    keys = w.unique_keys(14, 0, 6)
    z = np.zeros((6, 8), np.uint8)
    t.insert_or_assign(keys[:3], z[:3], np.array([1, 2, 3], np.uint64))
    ones = np.ones((6, 2), np.float32).view(np.uint8).reshape(6, 8)
    t.assign(keys, ones, np.arange(10, 16, dtype=np.uint64))
    assert t.size() == 3
    v, f, s = t.find(keys)
    assert f.tolist() == [True] * 3 + [False] * 3
    assert (v[:3] == ones[:3]).all() and s[:3].tolist() == [10, 11, 12]
    t.assign_scores(keys, np.arange(30, 36, dtype=np.uint64))
    t.assign_values(keys, z)
    v, f, s = t.find(keys)
    assert (v[:3] == 0).all() and s[:3].tolist() == [30, 31, 32]
    t.close()


# ---- export / size_if / erase / clear -----------------------------------------------------------------------------

def test_export_batch_if_and_size_if_agree(oracle):
    # tests/export_batch_if_test.cc.cu:214-222, 268-296
    o = default_options(init_capacity=4096, max_capacity=4096, dim=2, evict_strategy=EvictStrategy.kCustomized)
    t = oracle.OracleTable(o)
    keys = w.unique_keys(15, 0, 3000)
    scores = (w.stream(16, 0, 3000) % np.uint64(1000)).astype(np.uint64)
    t.insert_or_assign(keys, vals_of(keys, 2), scores)
    kk, vv, ss = t.export_all()
    resident = as_map(kk, vv, ss)
    for pred, fn in ((Predicate.kScoreLt, lambda s: s < 400), (Predicate.kScoreGe, lambda s: s >= 400),
                     (Predicate.kScoreGt, lambda s: s > 400), (Predicate.kScoreLe, lambda s: s <= 400)):
        k, v, s = t.export_batch_if(pred, 0, 400)
        assert len(set(k.tolist())) == len(k)
        assert t.size_if(pred, 0, 400) == len(k)
        assert all(fn(int(x)) for x in s)
        assert as_map(k, v, s) == {a: b for a, b in resident.items() if fn(b[1])}
    # windows of the slot range partition the table
    total = 0
    for off in range(0, 4096, 1000):
        k, _, _ = t.export_batch_if(Predicate.kAlways, 0, 0, n=1000, offset=off)
        total += len(k)
    assert total == t.size()
    assert len(t.export_batch_if(Predicate.kAlways, 0, 0, n=10, offset=4096)[0]) == 0
    t.close()


def test_erase_and_clear_counts(oracle):
    # tests/merlin_hashtable_test.cc.cu:336-344
    o = default_options(init_capacity=4096, max_capacity=4096, dim=1, evict_strategy=EvictStrategy.kCustomized)
    t = oracle.OracleTable(o)
    keys = w.unique_keys(17, 0, 2000)
    z = np.zeros((2000, 4), np.uint8)
    t.insert_or_assign(keys, z, np.arange(1, 2001, dtype=np.uint64))
    n0 = t.size()
    present = t.contains(keys)
    t.erase(keys[:1000])
    assert t.size() == n0 - int(present[:1000].sum())
    assert not t.contains(keys[:1000]).any()
    t.erase(keys[:1000])  # erasing twice changes nothing
    assert t.size() == n0 - int(present[:1000].sum())
    t.clear()
    assert t.size() == 0
    assert len(t.export_all()[0]) == 0
    t.insert_or_assign(keys, z, np.arange(1, 2001, dtype=np.uint64))
    assert t.size() == n0
    t.close()


# ---- argument checks ----------------------------------------------------------------------------------------------------

def test_init_checks(oracle):
    # merlin_hashtable.cuh:1016-1048
    with pytest.raises(oracle.OracleError):
        oracle.OracleTable(default_options(init_capacity=1024, max_capacity=1024, reserved_key_start_bit=63))
    with pytest.raises(oracle.OracleError):
        oracle.OracleTable(default_options(init_capacity=1024, max_capacity=1024, max_bucket_size=100))
    with pytest.raises(oracle.OracleError):
        oracle.OracleTable(default_options(init_capacity=1024, max_capacity=1024, num_of_buckets_per_alloc=3))
    with pytest.raises(oracle.OracleError):
        oracle.OracleTable(default_options(init_capacity=128, max_capacity=128, num_of_buckets_per_alloc=2))


def test_multithreaded_baseline_equals_sequential(oracle):
    o = default_options(init_capacity=1 << 14, max_capacity=1 << 14, dim=4, evict_strategy=EvictStrategy.kCustomized)
    a = oracle.OracleTable(o)
    b = oracle.OracleTable(o)
    for batch in range(4):
        keys = w.unique_keys(20, batch * 9000, 9000)
        vals = vals_of(keys, 4)
        sc = w.monotone_scores(batch + 1, 9000)
        a.insert_or_assign(keys, vals, sc)
        b.insert_or_assign_mt(keys, vals, sc, threads=4)
    ka, va, sa = a.export_all()
    kb, vb, sb = b.export_all()
    assert as_map(ka, va, sa) == as_map(kb, vb, sb)
    q = w.unique_keys(20, 20000, 9000)
    v1, f1, s1 = a.find(q)
    v2, f2, s2 = b.find(q, threads=4)
    assert (f1 == f2).all() and (v1 == v2).all() and (s1 == s2).all()
    a.close()
    b.close()


# ---- growth ----------------------------------------------------------------------

def test_rehash_scenario_of_the_reference_test(oracle):
    # tests/merlin_hashtable_test.cc.cu:1078-1200 (test_rehash): one bucket to start with, room
    # for four; 256 keys arrive at once.  The growth loop at the head of insert_or_assign
    # (fast_load_factor = 256/128 > 0.5, then 256/256 > 0.5) takes the table to 512 slots
    # before the first key goes in, so nothing is evicted.
    o = default_options(init_capacity=128, max_capacity=512, dim=4, reserved_key_start_bit=5,
                        evict_strategy=EvictStrategy.kCustomized)
    t = oracle.OracleTable(o)
    assert t.capacity() == 128
    keys = w.unique_keys(7, 0, 256)
    keys = keys[(keys & np.uint64(0x60)) != np.uint64(0x60)][:200]  # keep clear of the reserved patterns at bit 5
    t.insert_or_assign(keys, vals_of(keys, 4), keys.copy())
    assert t.capacity() == 512
    per_bucket = np.bincount([int(oracle.locate(int(k), 4)[0]) for k in keys], minlength=4)
    assert per_bucket.max() <= 128  # so every key fits: the size is the number of keys
    assert t.size() == len(keys)
    t.reserve(512)
    assert t.capacity() == 512 and t.size() == len(keys)
    v, f, sc = t.find(keys)
    assert f.all() and (sc == keys).all() and (v == vals_of(keys, 4)).all()
    t.close()


def test_reserve_keeps_the_map_and_doubles_until_the_limit(oracle):
    # reserve (merlin_hashtable.cuh:3503-3541) against a python dict: same entries before and
    # after, every key in the bucket its hash names for the new bucket count, tombstones
    # still not counted, and no doubling past max_capacity.
    o = default_options(init_capacity=1024, max_capacity=8192, dim=2, max_load_factor=2.0,
                        evict_strategy=EvictStrategy.kCustomized)  # load factor 2: no growth on its own
    t = oracle.OracleTable(o)
    keys = w.unique_keys(11, 0, 900)
    sc = w.monotone_scores(1, 900)
    t.insert_or_assign(keys, vals_of(keys, 2), sc)
    t.erase(keys[:50])
    before = dict(zip(*[x.tolist() for x in (t.export_all()[0], t.export_all()[2])]))
    assert t.capacity() == 1024 and t.size() == len(before)
    t.reserve(2048)
    assert t.capacity() == 2048
    t.reserve(3000)  # next power of two
    assert t.capacity() == 4096
    t.reserve(1 << 20)  # beyond max_capacity: ignored (merlin_hashtable.cuh:3508-3511)
    assert t.capacity() == 4096
    t.reserve(8192)
    assert t.capacity() == 8192
    t.reserve(16384)
    assert t.capacity() == 8192
    k, v, s = t.export_all()
    assert dict(zip(k.tolist(), s.tolist())) == before
    assert (v == vals_of(k, 2)).all()
    assert t.size() == len(before)
    sizes = np.zeros(64, np.int64)
    for key in k.tolist():
        sizes[oracle.locate(key, 64)[0]] += 1
    assert [t.bucket_size(b) for b in range(64)] == sizes.tolist()
    _, f, _ = t.find(keys)
    assert not f[:50].any()
    assert f.tolist() == [k_ in before for k_ in keys.tolist()]  # (a few were evicted at 1024 slots)
    t.close()


def test_set_max_capacity_scenario_of_the_reference(oracle):
    # set_max_capacity (merlin_hashtable.cuh:3561-3579) by the reference's own scenario
    # (tests/dynamic_max_capacity_test.cc.cu:39-134): fill a table of 2^12 slots that may grow to
    # 2^14 with consecutive integer keys through insert_and_evict until it is 98 % full, raise the
    # limit, reserve up to it (the capacity then equals the new limit and the load factor is at most
    # a half), go on until the limit would pass 2^17; every key ever inserted is then either in the
    # table or among the evicted ones, each with the row made from it, and the closed forms of the
    # text: a limit that is not a power of two raises, one below the capacity changes nothing.
    dim, n = 2, 2500
    cap_limit, uplimit = 1 << 14, 1 << 17
    o = default_options(init_capacity=1 << 12, max_capacity=cap_limit, dim=dim, max_load_factor=0.5,
                        evict_strategy=EvictStrategy.kLru)
    t = oracle.OracleTable(o)
    t.set_clock(1, 1 << 40)
    seen = {}
    offset = 0
    while True:
        keys = np.arange(offset, offset + n, dtype=np.uint64)
        ek, ev, _ = t.insert_and_evict(keys, vals_of(keys, dim), None)
        offset += n
        assert offset <= 2 * uplimit, "too many keys without filling the table"
        for k, v in zip(ek.tolist(), ev):
            seen[k] = v.tobytes()
        if t.size() / t.capacity() >= 0.98:
            assert t.capacity() == cap_limit  # grown by itself up to the limit, not past it
            with pytest.raises(oracle.OracleError):
                t.set_max_capacity(cap_limit * 2 + 2)  # not a power of two
            t.set_max_capacity(cap_limit // 4)  # below the capacity: ignored
            t.reserve(cap_limit * 2)
            assert t.capacity() == cap_limit
            cap_limit *= 2
            if cap_limit > uplimit:
                break
            t.set_max_capacity(cap_limit)
            t.reserve(cap_limit)
            assert t.capacity() == cap_limit
            assert t.size() / t.capacity() <= 0.5
    k, v, _ = t.export_all()
    for key, row in zip(k.tolist(), v):
        seen[key] = row.tobytes()
    assert t.capacity() * 2 == cap_limit
    assert len(seen) >= t.capacity() * 0.98
    assert sorted(seen) == list(range(offset))  # nothing lost, nothing made up
    want = vals_of(np.array(sorted(seen), dtype=np.uint64), dim)
    assert all(seen[key] == want[i].tobytes() for i, key in enumerate(sorted(seen)))
    t.close()


# ---- lock_keys / unlock_keys / find_and_update ---------------------------------------

def test_lock_unlock_truth_table(oracle):
    # lock_kernel_with_filter / unlock_keys_kernel (core_kernels.cuh:1180-1204, 1248-1362):
    # present -> LOCKED + score touched + address; absent or reserved -> null, false;
    # unlock succeeds exactly once per locked address
    o = default_options(init_capacity=1024, max_capacity=1024, dim=2, evict_strategy=EvictStrategy.kCustomized)
    t = oracle.OracleTable(o)
    keys = w.unique_keys(21, 0, 300)
    t.insert_or_assign(keys, vals_of(keys, 2), np.arange(1000, 1300, dtype=np.uint64))
    assert t.size() == 300
    batch = np.concatenate([keys[:60], w.unique_keys(22, 0, 10), np.array([M64, M64 - 2], np.uint64)])
    new_sc = np.arange(5000, 5000 + len(batch), dtype=np.uint64)
    slots, ok = t.lock_keys(batch, new_sc)
    assert ok.tolist() == [True] * 60 + [False] * 12
    assert (slots[60:] == np.uint64(M64)).all() and len(set(slots[:60].tolist())) == 60
    _, f, _ = t.find(keys)
    assert not f[:60].any() and f[60:].all()        # a locked key is invisible to lookups
    assert t.size() == 300                          # ... but still counted
    assert len(t.export_all()[0]) == 240            # ... and not exported (its key word is reserved)
    again, ok2 = t.lock_keys(batch[:5], new_sc[:5])
    assert not ok2.any()                            # cannot be found, so cannot be locked twice
    ok3 = t.unlock_keys(slots, batch)
    assert ok3.tolist() == [True] * 60 + [False] * 12
    assert not t.unlock_keys(slots[:60], batch[:60]).any()
    v, f, sc = t.find(keys)
    assert f.all() and (v == vals_of(keys, 2)).all()
    assert (sc[:60] == new_sc[:60]).all() and (sc[60:] == np.arange(1060, 1300, dtype=np.uint64)).all()
    t.close()


def test_locked_slot_is_never_the_victim(oracle):
    o = default_options(init_capacity=128, max_capacity=128, dim=1, evict_strategy=EvictStrategy.kCustomized)
    t = oracle.OracleTable(o)
    keys = w.unique_keys(23, 0, 128)
    sc = np.arange(100, 228, dtype=np.uint64)
    t.insert_or_assign(keys, vals_of(keys, 1), sc)
    slots, ok = t.lock_keys(keys[:1], np.array([100], np.uint64))  # the minimum-score key
    assert ok.all()
    newk = w.unique_keys(24, 0, 1)
    t.insert_or_assign(newk, vals_of(newk, 1), np.array([500], np.uint64))
    assert t.unlock_keys(slots, keys[:1]).all()
    _, f, s2 = t.find(np.concatenate([keys[:2], newk]))
    assert f.tolist() == [True, False, True]        # the second lowest score went instead
    t.close()


def test_find_and_update_touches_scores(oracle):
    # tlp_lookup_ptr_kernel_with_filter, update_score = true (lookup_ptr.cuh:93-110)
    o = default_options(init_capacity=1024, max_capacity=1024, dim=2, evict_strategy=EvictStrategy.kLfu)
    t = oracle.OracleTable(o)
    keys = w.unique_keys(25, 0, 200)
    t.insert_or_assign(keys, vals_of(keys, 2), np.full(200, 3, np.uint64))
    q = np.concatenate([keys[:50], w.unique_keys(26, 0, 5)])
    slots, f, sc = t.find_and_update(q, np.full(55, 4, np.uint64))
    assert f.tolist() == [True] * 50 + [False] * 5
    assert (sc[:50] == 7).all() and (sc[50:] == 4).all()  # LFU adds; misses keep their input
    assert (slots[50:] == np.uint64(M64)).all()
    _, _, s2 = t.find(keys)
    assert (s2[:50] == 7).all() and (s2[50:] == 3).all()
    with pytest.raises(Exception):
        t.find_and_update(q, None)  # LFU needs scores (check_evict_strategy)
    t.close()


def test_find_or_insert_pointer_truth_table(oracle):
    # find_or_insert_ptr_kernel_lock_key (find_ptr_or_insert.cuh:27-246), one full bucket, Customized:
    #   reserved key     -> value pointer and found flag left as they were (:66-70)
    #   present          -> found, its own slot, score := input (update_with_digest, :108-113)
    #   absent, score > min          -> not found, takes the slot of the minimum score (:195-224)
    #   absent, score == min or less -> refused: null pointer, not found (:196-199, "<=")
    untouched_slot, untouched_flag = 0x5555555555555555, 2   # what the binding pre-fills
    o = default_options(init_capacity=128, max_capacity=128, dim=1, evict_strategy=EvictStrategy.kCustomized)
    t = oracle.OracleTable(o)
    keys = w.unique_keys(41, 0, 128)
    sc = np.arange(1000, 1128, dtype=np.uint64)
    t.insert_or_assign(keys, vals_of(keys, 1), sc)
    where, f, _ = t.find_slot(keys)
    assert f.all() and sorted(where.tolist()) == list(range(128))
    fresh = w.unique_keys(42, 0, 3)
    batch = np.concatenate([np.array([M64, M64 - 1, M64 - 2, M64 - 3], np.uint64),  # the four reserved keys
                            keys[5:7],            # present
                            fresh])               # absent: above the minimum, equal to it, below it
    # key 0 holds the minimum (1000); after fresh[0] has taken its slot with 5000 the minimum is 1001
    bsc = np.array([1, 1, 1, 1, 7005, 7006, 5000, 1001, 3], np.uint64)
    slots, founds = t.find_or_insert_slot(batch, bsc)
    assert (slots[:4] == np.uint64(untouched_slot)).all() and (founds[:4] == untouched_flag).all()
    assert founds[4:6].tolist() == [1, 1] and slots[4:6].tolist() == where[5:7].tolist()
    assert founds[6] == 0 and slots[6] == where[0]          # victim = the minimum score's slot
    assert founds[7] == 0 and slots[7] == np.uint64(M64)    # equal to the minimum: refused
    assert founds[8] == 0 and slots[8] == np.uint64(M64)    # below the minimum: refused
    _, f, s2 = t.find(np.concatenate([keys[:1], keys[5:7], fresh]))
    assert f.tolist() == [False, True, True, True, False, False]
    assert s2[1:4].tolist() == [7005, 7006, 5000]
    assert t.size() == 128
    t.close()


def test_find_or_insert_pointer_never_takes_locked_or_empty_slots(oracle):
    # the victim scan of the lock-key kernels skips slots whose key word is LOCKED or EMPTY
    # (find_ptr_or_insert.cuh:170-180): with the two lowest scores locked, the third goes
    o = default_options(init_capacity=128, max_capacity=128, dim=1, evict_strategy=EvictStrategy.kCustomized)
    t = oracle.OracleTable(o)
    keys = w.unique_keys(43, 0, 128)
    sc = np.arange(100, 228, dtype=np.uint64)
    t.insert_or_assign(keys, vals_of(keys, 1), sc)
    where, _, _ = t.find_slot(keys)
    locked, ok = t.lock_keys(keys[:2], sc[:2].copy())
    assert ok.all() and locked.tolist() == where[:2].tolist()
    newk = w.unique_keys(44, 0, 1)
    slots, founds = t.find_or_insert_slot(newk, np.array([900], np.uint64))
    assert founds[0] == 0 and slots[0] == where[2]
    # a key that cannot beat the lowest visible score (102 left; 103 is next) is refused, not parked
    # on a locked slot
    again = w.unique_keys(45, 0, 1)
    slots2, founds2 = t.find_or_insert_slot(again, np.array([103], np.uint64))
    assert founds2[0] == 0 and slots2[0] == np.uint64(M64)
    assert t.unlock_keys(locked, keys[:2]).all()
    _, f, _ = t.find(np.concatenate([keys[:3], newk, again]))
    assert f.tolist() == [True, True, False, True, False]
    # free slots come before victims: erase one key, the next absent key lands in that slot
    t.erase(keys[10:11])
    third = w.unique_keys(46, 0, 1)
    slots3, founds3 = t.find_or_insert_slot(third, np.array([1], np.uint64))  # the lowest score of all
    assert founds3[0] == 0 and slots3[0] == where[10]
    t.close()


def test_find_pointer_truth_table(oracle):
    # tlp_lookup_ptr_kernel_with_filter / lookup_ptr_kernel (lookup_ptr.cuh:25-152, 379-435):
    # present -> its slot, found, its score; absent -> null, not found, score output untouched;
    # reserved keys and keys held by lock_keys are not found; the table does not change
    o = default_options(init_capacity=1024, max_capacity=1024, dim=2, evict_strategy=EvictStrategy.kCustomized)
    t = oracle.OracleTable(o)
    keys = w.unique_keys(47, 0, 300)
    sc = np.arange(2000, 2300, dtype=np.uint64)
    t.insert_or_assign(keys, vals_of(keys, 2), sc)
    q = np.concatenate([keys[:40], w.unique_keys(48, 0, 8), np.array([M64, M64 - 1, M64 - 2, M64 - 3], np.uint64)])
    slots, f, s = t.find_slot(q)
    assert f.tolist() == [True] * 40 + [False] * 12
    assert (slots[40:] == np.uint64(M64)).all() and (s[40:] == 0).all()
    assert (s[:40] == sc[:40]).all()
    # the slot is where the key's row lives: bucket of the key, and distinct per key
    nb = 1024 // 128
    assert [int(x) // 128 for x in slots[:40]] == [oracle.locate(int(k), nb)[0] for k in keys[:40]]
    assert len(set(slots[:40].tolist())) == 40
    locked, ok = t.lock_keys(keys[:3], sc[:3].copy())
    assert ok.all()
    _, f2, _ = t.find_slot(keys[:5])
    assert f2.tolist() == [False, False, False, True, True]
    assert t.unlock_keys(locked, keys[:3]).all()
    slots3, f3, s3 = t.find_slot(keys[:5])
    assert f3.all() and slots3.tolist() == slots[:5].tolist() and (s3 == sc[:5]).all()
    assert t.size() == 300
    t.close()


# ---- dual-bucket mode (TableMode::kMemory) -------------------------------------------------

def dual_options(capacity, dim=4, strategy=EvictStrategy.kCustomized, **kw):
    # create_memory_mode_table, tests/dual_bucket_test.cc.cu:42-52
    return default_options(init_capacity=capacity, max_capacity=capacity, max_hbm_for_vectors=0,
                           dim=dim, table_mode=1, evict_strategy=strategy, **kw)


def test_dual_addressing_closed_form(oracle):
    # dual_bucket_utils.cuh:36-74: b1 from the low hash word, b2 from the high one,
    # moved on by one when they collide; digest = the top byte
    rng = np.random.default_rng(77)
    for nb in (2, 4, 7, 128, 524287, 1 << 21):
        for key in [0, 1, 2, 0x0123456789ABCDEF] + rng.integers(0, M64 - 4, 40, dtype=np.uint64).tolist():
            h = oracle.fmix64(int(key))
            lo, hi = h & 0xFFFFFFFF, h >> 32
            b1, b2 = lo % nb, hi % nb
            if b2 == b1:
                b2 = (b2 + 1) % nb
            (g1, g2), (s1, s2), d = oracle.locate_dual(int(key), nb)
            assert (g1, g2) == (b1, b2) and g1 != g2
            assert (s1, s2) == ((lo % 128) & ~3, (hi % 128) & ~3)
            assert d == h >> 56
    # known answers from the closed form of fmix64 (h(1) = 0xb456bcfc34c2cb2c)
    assert oracle.locate_dual(1, 8192) == ((0x34c2cb2c % 8192, 0xb456bcfc % 8192), (0x2c & ~3, 0x7c), 0xb4)


def test_dual_init_checks_and_guards(oracle):
    # tests/dual_bucket_test.cc.cu:641-661, 1051-1107, 1187-1196 and :471-515, 941-1049
    for bad in (dict(init_capacity=1024, max_capacity=2048), dict(max_hbm_for_vectors=1 << 30),
                dict(dim=225), dict(init_capacity=128, max_capacity=128)):
        kw = dict(init_capacity=1024, max_capacity=1024, max_hbm_for_vectors=0, dim=4, table_mode=1,
                  evict_strategy=EvictStrategy.kCustomized)
        kw.update(bad)
        with pytest.raises(oracle.OracleError):
            oracle.OracleTable(default_options(**kw))
    oracle.OracleTable(dual_options(256, dim=224)).close()
    t = oracle.OracleTable(dual_options(1024))
    keys = np.arange(1, 9, dtype=np.uint64)
    vals = vals_of(keys, 4)
    sc = np.arange(1, 9, dtype=np.uint64)
    t.insert_or_assign(keys, vals, sc)
    flags = np.ones(8, dtype=np.uint8)
    for call in (lambda: t.erase(keys), lambda: t.contains(keys), lambda: t.reserve(2048),
                 lambda: t.find_or_insert(keys, vals.copy(), sc), lambda: t.insert_and_evict(keys, vals, sc),
                 lambda: t.accum_or_assign(keys, vals, flags, sc), lambda: t.assign_scores(keys, sc),
                 lambda: t.assign_values(keys, vals), lambda: t.assign(keys, vals, sc),
                 lambda: t.find_slot(keys), lambda: t.lock_keys(keys, sc)):
        with pytest.raises(oracle.OracleError):
            call()
    assert t.size() == 8
    t.close()


def test_dual_basic_update_and_b1_equals_b2(oracle):
    # tests/dual_bucket_test.cc.cu:74-237 and :663-742 (4 buckets: b1 == b2 before the
    # adjustment for about a quarter of the keys)
    t = oracle.OracleTable(dual_options(4 * 128, dim=16))
    keys = np.arange(1, 257, dtype=np.uint64)
    as_bytes = lambda a: np.ascontiguousarray(a, dtype=np.float32).view(np.uint8).reshape(len(a), -1)
    fvals = np.repeat(keys.astype(np.float32)[:, None], 16, axis=1)
    vals = as_bytes(fvals)
    t.insert_or_assign(keys, vals, keys.copy())
    assert t.size() == 256
    collide = sum(1 for k in keys.tolist()
                  if (oracle.fmix64(k) & 0xFFFFFFFF) % 4 == (oracle.fmix64(k) >> 32) % 4)
    assert collide > 20
    v, f, s = t.find(keys)
    assert f.all() and (v == vals).all() and (s == keys).all()
    # update in place: no duplicates, wherever the key lives
    t.insert_or_assign(keys, as_bytes(fvals * 2), keys + 1000)
    assert t.size() == 256
    v, f, s = t.find(keys)
    assert f.all() and (v == as_bytes(fvals * 2)).all() and (s == keys + 1000).all()
    ek, ev, es = t.export_all()
    assert sorted(ek.tolist()) == keys.tolist()
    # every key sits in one of its two buckets
    v, f, s = t.find(np.arange(1000, 1100, dtype=np.uint64))
    assert not f.any()
    # clear and re-insert (tests/dual_bucket_test.cc.cu:1841-1900)
    t.clear()
    assert t.size() == 0
    _, f, _ = t.find(keys)
    assert not f.any()
    t.insert_or_assign(keys, vals, keys.copy())
    v, f, s = t.find(keys)
    assert f.all() and (v == vals).all() and t.size() == 256
    t.close()


def test_dual_two_choice_fills_the_emptier_bucket(oracle):
    # a brute-force model of phase 1 (dict of bucket -> count) predicts the size of every
    # bucket while nothing is evicted
    nb = 64
    t = oracle.OracleTable(dual_options(nb * 128, dim=1))
    rng = np.random.default_rng(5)
    keys = np.unique(rng.integers(1, 1 << 62, 5000, dtype=np.uint64))
    rng.shuffle(keys)
    model = [0] * nb
    where = {}
    for k in keys.tolist():
        (b1, b2), _, _ = oracle.locate_dual(k, nb)
        b = b1 if model[b1] <= model[b2] else b2
        assert model[b] < 128
        model[b] += 1
        where[k] = b
    t.insert_or_assign(keys, vals_of(keys, 1), np.arange(1, len(keys) + 1, dtype=np.uint64))
    assert [t.bucket_size(b) for b in range(nb)] == model
    ek, _, _ = t.export_batch_if(n=128, offset=128 * 3)
    assert sorted(ek.tolist()) == sorted(k for k, b in where.items() if b == 3)
    t.close()


def test_dual_eviction_takes_the_minimum_of_both_buckets(oracle):
    # 2 buckets: every key has the candidates {0, 1}; once both are full the table holds
    # the 256 highest scores seen so far, whatever the order (scores distinct)
    t = oracle.OracleTable(dual_options(256, dim=1))
    rng = np.random.default_rng(9)
    keys = np.arange(1, 1025, dtype=np.uint64)
    scores = rng.permutation(np.arange(1, 1025, dtype=np.uint64))
    for lo in range(0, 1024, 64):
        t.insert_or_assign(keys[lo:lo + 64], vals_of(keys[lo:lo + 64], 1), scores[lo:lo + 64])
        ek, _, es = t.export_all()
        seen = scores[:lo + 64]
        want = np.sort(seen)[-256:]
        assert np.array_equal(np.sort(es), want)
    # a score below the minimum is refused, one equal to it is accepted
    ek, _, es = t.export_all()
    m = int(es.min())
    newk = np.array([5000], dtype=np.uint64)
    t.insert_or_assign(newk, vals_of(newk, 1), np.array([m - 1], dtype=np.uint64))
    assert not t.find(newk)[1][0]
    t.insert_or_assign(newk, vals_of(newk, 1), np.array([m], dtype=np.uint64))
    assert t.find(newk)[1][0] and t.size() == 256
    t.close()


def test_dual_first_eviction_load_factor(oracle):
    # tests/dual_bucket_test.cc.cu:399-465: keys 1, 2, ... with score = key in batches of
    # 128; the first eviction must come after load factor 0.98 (about 0.982 at 10 M slots)
    cap = 10 * 1024 * 1024
    t = oracle.OracleTable(dual_options(cap, dim=1))
    nxt, inserted, first = 1, 0, None
    step = 128 * 512
    while inserted < cap:
        # below 0.97 nothing can have been evicted unless the two-choice rule is broken:
        # check in big steps there, then batch by batch as the reference's test does
        n = step if inserted + step < int(cap * 0.97) else 128
        keys = np.arange(nxt, nxt + n, dtype=np.uint64)
        t.insert_or_assign(keys, vals_of(keys, 1), keys.copy())
        nxt += n
        inserted += n
        size = t.size()
        if size < inserted:
            first = size / cap
            break
    assert first is not None and first > 0.980
    assert first < 0.995
    t.close()


def test_dual_eviction_quality(oracle):
    # tests/dual_bucket_test.cc.cu:1406-1520: 5 x capacity keys with random scores in
    # batches of one capacity; the survivors overlap the ideal top set by >= 99.5 %
    cap = 128 * 1024
    t = oracle.OracleTable(dual_options(cap, dim=1))
    total = 5 * cap
    rng = np.random.default_rng(42)
    keys = np.arange(1, total + 1, dtype=np.uint64)
    scores = (rng.integers(0, 1 << 63, total, dtype=np.uint64) >> np.uint64(1)) | np.uint64(1)
    for lo in range(0, total, cap):
        t.insert_or_assign(keys[lo:lo + cap], vals_of(keys[lo:lo + cap], 1), scores[lo:lo + cap])
    ek, _, es = t.export_all()
    assert len(ek) == t.size() and len(ek) > 0.99 * cap
    ideal = set(keys[np.argsort(scores)[::-1][:len(ek)]].tolist())
    overlap = sum(1 for k in ek.tolist() if k in ideal)
    assert overlap / len(ek) >= 0.995
    assert np.array_equal(es, scores[ek.astype(np.int64) - 1])
    t.close()


def test_rehash_on_big_batch_scenario_of_the_reference(oracle):
    # merlin_hashtable_test.cc.cu:1223-1367: init 1024, max 16384, load factor 0.6; 1024 keys
    # bring the capacity to 2048, the 2048 keys that contain them to 8192, and the table then
    # holds 2048 keys (re-inserting keys that a rehash has moved must find them: the reference
    # compacts buckets after a rehash, here the key is looked for in the whole bucket)
    o = default_options(init_capacity=1024, max_capacity=16 * 1024, dim=2, reserved_key_start_bit=6,
                        num_of_buckets_per_alloc=8, max_load_factor=0.6, max_hbm_for_vectors=1 << 30,
                        evict_strategy=EvictStrategy.kCustomized)
    t = oracle.OracleTable(o)
    keys = w.unique_keys(151, 0, 2048)
    vals = np.zeros((2048, 8), np.uint8)
    for n, cap in ((1024, 2048), (2048, 8192)):
        t.insert_or_assign(keys[:n], vals[:n], keys[:n].copy())
        assert t.size() == n and t.capacity() == cap
    ek, _, es = t.export_all()
    assert len(ek) == 2048 and len(np.unique(ek)) == 2048 and np.array_equal(np.sort(ek), np.sort(keys))
    assert np.array_equal(es, ek)
    # merlin_hashtable_test.cc.cu:1369-1439: 50 000 asked for, 100 000 allowed: 512 buckets, no doubling
    o = default_options(init_capacity=50000, max_capacity=100000, dim=2, max_load_factor=0.6,
                        max_hbm_for_vectors=1 << 30, evict_strategy=EvictStrategy.kLru)
    t = oracle.OracleTable(o)
    t.set_clock(1, 1 << 40)
    k = w.unique_keys(152, 0, 50000)
    t.insert_or_assign(k, np.zeros((50000, 8), np.uint8))
    assert t.capacity() == 65536


def test_accum_wraps_in_the_element_type(oracle):
    # accum_or_assign_vector (accum_or_assign.cuh:24-35) adds in V: 8- and 16-bit elements wrap at
    # their own width, independently of their neighbours in the row
    for dtype, kind in ((np.uint8, ValueKind.kI8), (np.int16, ValueKind.kI16)):
        dim = 7
        o = default_options(init_capacity=1024, max_capacity=1024, dim=dim, value_size=np.dtype(dtype).itemsize,
                            value_kind=kind, max_hbm_for_vectors=1 << 30, evict_strategy=EvictStrategy.kCustomized)
        t = oracle.OracleTable(o)
        rng = np.random.default_rng(5)
        info = np.iinfo(dtype)
        keys = w.unique_keys(171, 0, 64)
        base = rng.integers(info.min, info.max, size=(64, dim), dtype=dtype, endpoint=True)
        delta = rng.integers(info.min, info.max, size=(64, dim), dtype=dtype, endpoint=True)
        sc = np.arange(1, 65, dtype=np.uint64)
        as_bytes = lambda a: np.ascontiguousarray(a).view(np.uint8).reshape(len(a), -1)  # noqa: E731
        t.insert_or_assign(keys, as_bytes(base), sc)
        t.accum_or_assign(keys, as_bytes(delta), np.ones(64, np.uint8), sc)
        vals, founds, _ = t.find(keys)
        assert founds.all()
        with np.errstate(over="ignore"):
            want = (base.astype(np.int64) + delta.astype(np.int64)).astype(dtype)  # modulo 2^bits
        assert np.array_equal(vals, as_bytes(want))
