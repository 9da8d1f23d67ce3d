"""Many keys of one call in every bucket: tables of a few dozen buckets take calls of up to 1500
keys, so that every lock, every free slot and every victim is fought over by keys in flight
at the same moment (at the benchmark's sizes two keys of a call rarely meet).  The outcome of
such a call depends on the order in which its keys get their turn, so there is no oracle here;
what must hold in any order is checked after every call:
  * no key is in the table twice, size() is the number of keys an export hands out, and it
    never exceeds the capacity;
  * the table holds nothing but keys it held before and keys of the call; erase removes
    exactly its keys; assign, find and the lock calls change no key;
  * insert_and_evict hands back every key that left, once, and every key of the call that
    did not get in;
  * a key that is found carries a row that was written for it last (with repeated keys in
    a call: one of that call's rows for the key);
  * find agrees with the export.
One case per table shape the kernels are instantiated for: row sizes from 4 to 1200 bytes,
rows in host memory, host threads moving the rows, a capacity that is not a power of two, a
table that grows, reserved keys elsewhere in the key space, calls that repeat keys, and the
two-bucket mode."""
import numpy as np
import pytest
import torch

import workloads as w
from gpu_util import DEV, dev, export_table, host_u64, read_device
from hierarchicalkv_amd import EvictStrategy, HashTable, default_options

pytestmark = pytest.mark.gpu

UPSERTS = ["insert_or_assign", "find_or_insert", "insert_and_evict", "accum_or_assign"]
OTHERS = ["assign", "assign_scores", "erase", "find"]


def run_calls(t, strategy, dim, seed, steps, universe, sizes, ops, probs, repeat_keys=False, grows=False,
              hidden=0):
    rng = np.random.default_rng(seed)
    from_clock = strategy in (EvictStrategy.kLru, EvictStrategy.kEpochLru)
    vb = dim * 4
    rows_of = {}  # key -> list of rows one of which the key must carry (absent: not tracked)
    resident = set()
    for step in range(steps):
        n = int(rng.choice(sizes))
        op = str(rng.choice(ops, p=probs))
        repeated = repeat_keys and op in ("insert_or_assign", "find_or_insert", "assign") and rng.random() < 0.5
        keys = rng.choice(universe, size=n, replace=repeated)
        vals = rng.random((n, dim), dtype=np.float32)
        sc = rng.integers(1, 1 << int(rng.choice([4, 20, 40])), size=n, dtype=np.uint64)
        dk, dv, ds = dev(keys), dev(vals), (None if from_clock else dev(sc))
        where = (step, op, n)
        evicted = None
        if op == "insert_or_assign":
            t.insert_or_assign(n, dk, dv, ds, unique_key=not repeated)
        elif op == "find_or_insert":
            t.find_or_insert(n, dk, dv, ds, unique_key=not repeated)
        elif op == "insert_and_evict":
            ek = torch.zeros(n, dtype=torch.int64, device=DEV)
            ev = torch.zeros(n, dim, dtype=torch.float32, device=DEV)
            es = torch.zeros(n, dtype=torch.int64, device=DEV)
            cnt = t.insert_and_evict(n, dk, dv, ds, ek, ev, es)
            evicted = host_u64(ek[:cnt]).tolist()
        elif op == "accum_or_assign":
            flags = torch.from_numpy(rng.random(n) < 0.5).to(DEV)
            t.accum_or_assign(n, dk, dv, flags, ds)
        elif op == "assign":
            t.assign(n, dk, dv, ds, unique_key=not repeated)
        elif op == "assign_scores":
            t.assign_scores(n, dk, ds)
        elif op == "erase":
            t.erase(n, dk)
        elif op == "find":
            out = torch.zeros(n, dim, dtype=torch.float32, device=DEV)
            founds = torch.zeros(n, dtype=torch.bool, device=DEV)
            t.find(n, dk, out, founds)
        if op in ("insert_or_assign", "insert_and_evict", "assign"):
            fresh = {}
            for k, v in zip(keys.tolist(), vals):
                fresh.setdefault(k, []).append(v)
            for k, c in fresh.items():
                if op == "assign" and k not in rows_of:
                    continue  # nothing known about the row it had; if the key is absent nothing happens
                rows_of[k] = c
        elif op in ("find_or_insert", "accum_or_assign", "erase"):
            for k in keys.tolist():
                rows_of.pop(k, None)  # (the row depends on whether the key was there: not tracked)
        gk, gv, _ = export_table(t, vb)
        now = set(gk.tolist())
        batch = set(keys.tolist())
        # (`hidden`: slots held by lock_keys, which no export shows but size() counts)
        assert len(now) == len(gk) == t.size() - hidden <= t.capacity() - hidden, where
        if op == "erase":
            assert now == resident - batch, where
        elif op not in UPSERTS:
            assert now == resident, where
        else:
            assert now <= resident | batch, where
            if grows and fullest_bucket(t) < 128:
                # nothing is evicted or refused while no bucket is full (one that was full during
                # the call still is: an upsert frees nothing)
                if op != "accum_or_assign":
                    assert now == resident | batch, where
            elif strategy == EvictStrategy.kLru and op != "accum_or_assign":
                assert batch <= now, where  # the scores of the call are the highest: none is refused or evicted
        if evicted is not None:
            left = [k for k in evicted if k not in batch]
            assert len(set(left)) == len(left) and set(left) <= resident, where
            assert now - batch == (resident - batch) - set(left), where
            assert batch - now <= set(evicted), where
        resident = now
        rows = gv.view(np.float32).reshape(len(gk), dim)
        by_key = dict(zip(gk.tolist(), rows))
        for k, row in by_key.items():
            c = rows_of.get(k)
            if c is not None:
                assert any(np.array_equal(row, r) for r in c), (where, k)
        if op == "find":
            torch.cuda.synchronize()
            f = founds.cpu().numpy()
            o = out.cpu().numpy()
            for i, k in enumerate(keys.tolist()):
                assert f[i] == (k in by_key), (where, k)
                if f[i]:
                    assert np.array_equal(o[i], by_key[k]), (where, k)
    return resident


def fullest_bucket(t):
    torch.cuda.synchronize()
    v = t.view()
    keys = read_device(v.keys, v.capacity * 8).view(np.uint64).reshape(-1, 128)
    return int((keys != np.uint64(v.empty_key)).sum(axis=1).max())


def table(strategy, dim, cap, **kw):
    kw.setdefault("max_capacity", cap)
    kw.setdefault("max_hbm_for_vectors", 1 << 30)
    o = default_options(init_capacity=cap, dim=dim, evict_strategy=strategy, **kw)
    t = HashTable()
    t.init(o)
    return t


ALL = UPSERTS + OTHERS
P_ALL = [0.3, 0.1, 0.15, 0.1, 0.08, 0.07, 0.1, 0.1]


@pytest.mark.parametrize("dim", [1, 3, 64, 300])
@pytest.mark.parametrize("strategy", [EvictStrategy.kLru, EvictStrategy.kCustomized])
def test_row_sizes(strategy, dim):
    cap = 1 << 12
    t = table(strategy, dim, cap)
    run_calls(t, strategy, dim, 700 + dim, 40, w.unique_keys(701, 0, 3 * cap), [17, 300, 1500], ALL, P_ALL)
    t.close()


@pytest.mark.parametrize("strategy", [EvictStrategy.kLfu, EvictStrategy.kCustomized, EvictStrategy.kLru])
def test_rows_in_host_memory(strategy):
    """Hybrid mode: a quarter of the rows in HBM; the upserts follow the lock-key kernels' rule
    (a key whose score equals the bucket's lowest is refused, and no key takes the slot of
    another key of its call)."""
    cap, dim = 1 << 12, 8
    t = table(strategy, dim, cap, max_hbm_for_vectors=cap * dim * 4 // 4)
    assert not t.is_pure_hbm()
    ops = [o for o in ALL if o != "insert_and_evict"]  # (pure HBM only, as in the reference)
    # 4000 keys: more than 128 of a call in some buckets, whose slots are then all held by the call
    # (insert_or_assign and find_or_insert keep their slots locked to the end of the launch) and
    # refuse the rest; under LRU every key of a call gets in as long as that does not happen
    sizes = [17, 300, 1500] if strategy == EvictStrategy.kLru else [17, 300, 1500, 4000]
    run_calls(t, strategy, dim, 710 + int(strategy), 40, w.unique_keys(711, 0, 3 * cap), sizes,
              ops, [0.45, 0.1, 0.1, 0.08, 0.07, 0.1, 0.1])
    t.close()


def test_rows_moved_by_host_threads():
    cap, dim = 1 << 12, 8
    strategy = EvictStrategy.kCustomized
    t = table(strategy, dim, cap, max_hbm_for_vectors=0, io_by_cpu=True)
    ops = ["insert_or_assign", "find_or_insert", "assign", "erase", "find"]
    run_calls(t, strategy, dim, 720, 30, w.unique_keys(721, 0, 3 * cap), [17, 300, 1500], ops,
              [0.45, 0.2, 0.1, 0.1, 0.15])
    t.close()


def test_capacity_that_is_no_power_of_two():
    cap, dim = 37 * 128, 4
    strategy = EvictStrategy.kLru
    t = table(strategy, dim, cap)
    run_calls(t, strategy, dim, 730, 40, w.unique_keys(731, 0, 3 * cap), [17, 300, 1500], ALL, P_ALL)
    t.close()


def test_table_that_grows():
    """From 8 buckets to 128 in four doublings, rehashed between calls (load factor limit
    0.75); until the last size is reached no key may be lost."""
    dim = 4
    strategy = EvictStrategy.kCustomized
    t = table(strategy, dim, 1 << 10, max_capacity=1 << 14, max_load_factor=0.75)
    left = run_calls(t, strategy, dim, 740, 50, w.unique_keys(741, 0, 3 << 14), [17, 300, 1500], ALL, P_ALL,
                     grows=True)
    assert t.capacity() == 1 << 14 and len(left) > (1 << 13)
    t.close()


def test_reserved_keys_elsewhere():
    cap, dim = 1 << 12, 4
    strategy = EvictStrategy.kLru
    t = table(strategy, dim, cap, reserved_key_start_bit=17)
    # types.cuh:80-109: reserved now are the keys with bit 0 clear and every other bit but 17 and 18
    # set; the rest of the top of the key space, the all-ones key included, is ordinary
    universe = np.concatenate([w.unique_keys(751, 0, 3 * cap),
                               np.array([(1 << 64) - 1, (1 << 64) - 3, (1 << 64) - 4], np.uint64)])
    run_calls(t, strategy, dim, 750, 40, universe, [17, 300, 1500], ALL, P_ALL)
    t.close()


@pytest.mark.parametrize("strategy", [EvictStrategy.kLru, EvictStrategy.kCustomized])
def test_calls_that_repeat_keys(strategy):
    cap, dim = 1 << 12, 4
    t = table(strategy, dim, cap)
    run_calls(t, strategy, dim, 760 + int(strategy), 40, w.unique_keys(761, 0, cap), [17, 300, 1500], ALL, P_ALL,
              repeat_keys=True)
    t.close()


def test_two_bucket_mode():
    cap, dim = 1 << 12, 4
    strategy = EvictStrategy.kCustomized
    t = table(strategy, dim, cap, max_hbm_for_vectors=0, table_mode=1)
    run_calls(t, strategy, dim, 770, 40, w.unique_keys(771, 0, 3 * cap), [17, 300, 1500],
              ["insert_or_assign", "find"], [0.8, 0.2])
    t.close()


@pytest.mark.parametrize("api_lock", [0, 1])
@pytest.mark.parametrize("strategy", [EvictStrategy.kLru, EvictStrategy.kCustomized])
def test_four_streams_at_once(strategy, api_lock):
    """api_lock = false: calls on different streams run at the same time, kept apart by the
    slot locks alone.  The caller keeps the key sets of calls that may overlap apart (two calls
    that bring the same new key at the same moment each give it a slot, in the reference as
    here): four streams, each with keys of its own, all on one table of 32 buckets, so that
    the calls take each other's victims, free slots (erase runs beside the upserts) and locks.
    After every round: no key twice, size() = keys exported, and every key carries, whole, the
    row its stream wrote for it last (or, after a find_or_insert, the one before).
    (Upserts and finds only: an erase or an assign that runs beside an upsert takes a key whose
    slot another launch holds at that moment for absent, as the reference's kernels do — without
    the group lock the caller keeps such calls apart.)
    api_lock = true: upserts, assign, erase and find, ordered by their roles between the streams
    (events; an upsert runs alone and searches through the score bounds)."""
    cap, dim = 1 << 12, 8
    t = table(strategy, dim, cap, api_lock=api_lock)
    rng = np.random.default_rng(780 + int(strategy))
    streams = [torch.cuda.Stream() for _ in range(4)]
    universes = [w.unique_keys(781 + s, 0, 6 * cap) for s in range(4)]
    assert len(np.unique(np.concatenate(universes))) == 24 * cap
    from_clock = strategy == EvictStrategy.kLru
    rows_of = {}
    version = 0
    for rnd in range(10):
        # all inputs of the round first, then its twenty calls back to back, so that they overlap
        calls = []
        for call in range(5):
            for s, st in enumerate(streams):
                n = int(rng.choice([1500, 6000, 20000]))
                op = str(rng.choice(["insert_or_assign", "find_or_insert", "assign", "erase", "find"],
                                    p=[0.45, 0.15, 0.1, 0.15, 0.15] if api_lock else [0.65, 0.2, 0.0, 0.0, 0.15]))
                keys = rng.choice(universes[s], size=n, replace=False)
                version += 1
                vals = np.full((n, dim), version, np.float32)
                sc = rng.integers(1, 1 << 20, size=n, dtype=np.uint64)
                out = torch.zeros(n, dim, dtype=torch.float32, device=DEV)
                founds = torch.zeros(n, dtype=torch.bool, device=DEV)
                calls.append((op, st, n, keys, version, dev(keys), dev(vals), None if from_clock else dev(sc),
                              out, founds))
        torch.cuda.synchronize()
        for op, st, n, keys, ver, dk, dv, ds, out, founds in calls:
            if op == "insert_or_assign":
                t.insert_or_assign(n, dk, dv, ds, stream=st)
            elif op == "find_or_insert":
                t.find_or_insert(n, dk, dv, ds, stream=st)
            elif op == "assign":
                t.assign(n, dk, dv, ds, stream=st)
            elif op == "erase":
                t.erase(n, dk, stream=st)
            else:
                t.find(n, dk, out, founds, stream=st)
        for op, st, n, keys, ver, *_ in calls:  # (the calls of one stream run in this order)
            if op == "insert_or_assign":
                for k in keys.tolist():
                    rows_of[k] = [ver]
            elif op == "find_or_insert":
                for k in keys.tolist():
                    rows_of[k] = rows_of.get(k, []) + [ver]
            elif op == "assign":
                for k in keys.tolist():
                    if k in rows_of:  # (a key that is absent stays so; one that is there has been written)
                        rows_of[k] = [ver]
            elif op == "erase":
                for k in keys.tolist():
                    rows_of.pop(k, None)
        torch.cuda.synchronize()
        gk, gv, _ = export_table(t, dim * 4)
        assert len(set(gk.tolist())) == len(gk) == t.size() <= cap, rnd
        rows = gv.view(np.float32).reshape(len(gk), dim)
        assert (rows == rows[:, :1]).all(), rnd  # one call's row, not a mixture
        for k, row in zip(gk.tolist(), rows):
            assert k in rows_of and int(row[0]) in rows_of[k], (rnd, k, row[0], rows_of.get(k))
    t.close()


@pytest.mark.parametrize("strategy", [EvictStrategy.kLru, EvictStrategy.kCustomized])
def test_slots_held_by_lock_keys_survive(strategy):
    """A quarter of every bucket is held by lock_keys while calls of 1500 other keys fill the
    table and evict: the victim search reads the key words beside the scores and passes the held
    slots over, so after unlock_keys every held key is there with its row, whatever its score."""
    cap, dim = 1 << 12, 4
    t = table(strategy, dim, cap)
    rng = np.random.default_rng(790 + int(strategy))
    from_clock = strategy == EvictStrategy.kLru
    held = w.unique_keys(791, 0, 1000)
    hv = rng.random((1000, dim), dtype=np.float32)
    ones = np.ones(1000, np.uint64)  # the lowest scores of the table: first in line for eviction
    t.insert_or_assign(1000, dev(held), dev(hv), None if from_clock else dev(ones))
    ptrs = torch.zeros(1000, dtype=torch.int64, device=DEV)
    ok = torch.zeros(1000, dtype=torch.bool, device=DEV)
    t.lock_keys(1000, dev(held), ptrs, ok, scores=None if from_clock else dev(ones))
    assert bool(ok.all())
    others = w.unique_keys(792, 0, 4 * cap)
    run_calls(t, strategy, dim, 793 + int(strategy), 25, others, [300, 1500],
              ["insert_or_assign", "find_or_insert", "insert_and_evict", "accum_or_assign", "erase"],
              [0.4, 0.15, 0.2, 0.1, 0.15], hidden=len(held))
    ok2 = torch.zeros(1000, dtype=torch.bool, device=DEV)
    t.unlock_keys(1000, ptrs, dev(held), ok2)
    assert bool(ok2.all())
    out = torch.zeros(1000, dim, dtype=torch.float32, device=DEV)
    founds = torch.zeros(1000, dtype=torch.bool, device=DEV)
    t.find(1000, dev(held), out, founds)
    torch.cuda.synchronize()
    assert bool(founds.all()) and np.array_equal(out.cpu().numpy(), hv)
    gk, _, _ = export_table(t, dim * 4)
    assert len(set(gk.tolist())) == len(gk) == t.size() <= cap
    t.close()


@pytest.mark.parametrize("strategy", [EvictStrategy.kLru, EvictStrategy.kCustomized])
def test_pointer_overload_that_keeps_its_slots(strategy):
    """find_or_insert by pointer with locked_key_ptrs: every key the call settles keeps its slot
    LOCKED until unlock_keys, so the 47 keys that meet in a bucket see more and more slots that
    are neither theirs nor anybody's victim.  After unlock_keys: no key twice, the pointers of
    the keys that got in are pairwise different and those keys are found, and under LRU (whose
    new scores are the highest) every key got in."""
    cap, dim = 1 << 12, 4
    t = table(strategy, dim, cap)
    rng = np.random.default_rng(795 + int(strategy))
    from_clock = strategy == EvictStrategy.kLru
    universe = w.unique_keys(796, 0, 3 * cap)
    run_calls(t, strategy, dim, 797, 8, universe, [1500], ["insert_or_assign"], [1.0])  # full by now
    for rnd in range(6):
        n = 1500
        keys = rng.choice(universe, size=n, replace=False)
        sc = rng.integers(1, 1 << 20, size=n, dtype=np.uint64)
        ptrs = torch.zeros(n, dtype=torch.int64, device=DEV)
        founds = torch.zeros(n, dtype=torch.bool, device=DEV)
        kptrs = torch.zeros(n, dtype=torch.int64, device=DEV)
        t.find_or_insert_ptr(n, dev(keys), ptrs, founds, None if from_clock else dev(sc), locked_key_ptrs=kptrs)
        ok = torch.zeros(n, dtype=torch.bool, device=DEV)
        t.unlock_keys(n, kptrs, dev(keys), ok)
        torch.cuda.synchronize()
        p = ptrs.cpu().numpy()
        got_in = p != 0
        assert np.array_equal(ok.cpu().numpy(), got_in), rnd
        assert len(np.unique(p[got_in])) == got_in.sum(), rnd
        if from_clock:
            assert got_in.all(), rnd
        gk, _, _ = export_table(t, dim * 4)
        now = set(gk.tolist())
        assert len(now) == len(gk) == t.size() <= cap, rnd
        assert set(keys[got_in].tolist()) <= now and not (set(keys[~got_in].tolist()) & now), rnd
    t.close()
