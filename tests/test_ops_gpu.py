"""GPU parity for the remaining entry points and edge cases: pointer lookups,
contains, missed-keys find, assign family, find_or_insert pointers, value type
and dim matrix, ragged and empty batches, reserved keys, non-power-of-two
capacity, LFU / EpochLFU arithmetic, hybrid mode, error behaviour, streams."""
import numpy as np
import pytest
import torch

import workloads as w
from gpu_util import (DEV, assert_same_table, dev, export_table, host_bytes, host_u64,
                      read_device, sort_by_key)
from hierarchicalkv_amd import (EvictStrategy, HashTable, MerlinException, Predicate, ValueKind,
                                default_options)

pytestmark = pytest.mark.gpu
M64 = (1 << 64) - 1


def make_pair(oracle, hybrid=False, **kw):
    kw.setdefault("max_hbm_for_vectors", 1 << 34)
    o = default_options(**kw)
    t = HashTable()
    t.init(o)
    return t, oracle.OracleTable(o, hybrid=hybrid), o


def bytes_of(vals):
    return np.ascontiguousarray(vals).view(np.uint8).reshape(len(vals), -1)


def fill(t, o, seed, nbatch, bs, dim, scores_fn=None, start=0):
    for b in range(nbatch):
        keys = w.unique_keys(seed, start + b * bs, bs)
        vals = w.uniform_values(seed, start + b * bs, bs, dim)
        sc = scores_fn(b, bs) if scores_fn else None
        t.insert_or_assign(bs, dev(keys), dev(vals), dev(sc))
        o.insert_or_assign(keys, bytes_of(vals), sc)


def test_find_ptr_contains_and_missed(oracle):
    cap, dim, bs = 1 << 16, 24, 5000  # 96-byte rows, ragged batch size
    t, o, _ = make_pair(oracle, init_capacity=cap, max_capacity=cap, dim=dim,
                        evict_strategy=EvictStrategy.kCustomized)
    fill(t, o, 41, 10, bs, dim, lambda b, n: w.monotone_scores(b + 1, n))
    q = np.concatenate([w.unique_keys(41, 2 * bs + 17, 3001), w.unique_keys(42, 0, 2000),
                        np.array([M64, M64 - 1, M64 - 2, M64 - 3], np.uint64)])
    n = len(q)
    # find* : pointers to the rows
    ptrs = torch.zeros(n, dtype=torch.int64, device=DEV)
    founds = torch.zeros(n, dtype=torch.bool, device=DEV)
    scores = torch.zeros(n, dtype=torch.int64, device=DEV)
    t.find_ptr(n, dev(q), ptrs, founds, scores)
    torch.cuda.synchronize()
    ov, of, osc = o.find(q)
    gf = founds.cpu().numpy()
    gp = ptrs.cpu().numpy()
    assert (gf == of).all() and not gf[-4:].any()
    assert ((gp != 0) == of).all()
    assert (host_u64(scores)[gf] == osc[of]).all()
    for i in np.flatnonzero(gf)[:: 97]:
        assert (read_device(int(gp[i]), dim * 4) == ov[i]).all()
    # contains
    c = torch.zeros(n, dtype=torch.bool, device=DEV)
    t.contains(n, dev(q), c)
    torch.cuda.synchronize()
    assert (c.cpu().numpy() == of).all()
    # find with the missed-keys outputs
    out = torch.zeros(n, dim, dtype=torch.float32, device=DEV)
    mk = torch.zeros(n, dtype=torch.int64, device=DEV)
    mi = torch.zeros(n, dtype=torch.int32, device=DEV)
    ms = torch.full((1,), 77, dtype=torch.int32, device=DEV)
    t.find_missed(n, dev(q), out, mk, mi, ms)
    torch.cuda.synchronize()
    m = int(ms.item())
    assert m == int((~of).sum())  # missed + found == n (find_with_missed_keys_test.cc.cu:32-212)
    idx = np.sort(mi[:m].cpu().numpy())
    assert (idx == np.flatnonzero(~of)).all()
    order = np.argsort(mi[:m].cpu().numpy())
    assert (host_u64(mk[:m])[order] == q[~of]).all()
    assert (bytes_of(out.cpu().numpy())[of] == ov[of]).all()
    t.close()


@pytest.mark.parametrize("np_dtype,torch_dtype,kind,dim", [
    (np.int8, torch.int8, ValueKind.kBytes, 3),
    (np.uint8, torch.uint8, ValueKind.kBytes, 129),
    (np.int16, torch.int16, ValueKind.kBytes, 66),
    (np.int8, torch.int8, ValueKind.kI8, 3),       # 1-byte units
    (np.uint8, torch.uint8, ValueKind.kI8, 129),
    (np.int8, torch.int8, ValueKind.kI8, 64),      # 16-byte units
    (np.int16, torch.int16, ValueKind.kI16, 33),   # 2-byte units
    (np.uint16, torch.int16, ValueKind.kI16, 66),  # 4-byte units
    (np.int32, torch.int32, ValueKind.kI32, 202),  # 8-byte units
    (np.float32, torch.float32, ValueKind.kF32, 224),
    (np.float32, torch.float32, ValueKind.kF32, 3),
    (np.float64, torch.float64, ValueKind.kF64, 128),
    (np.float64, torch.float64, ValueKind.kF64, 63),  # 8-byte units
    (np.int64, torch.int64, ValueKind.kI64, 5),
    (np.float32, torch.float32, ValueKind.kF32, 520),   # 2080-byte rows: several passes of 16-byte units
    (np.float32, torch.float32, ValueKind.kF32, 1025),  # 4100-byte rows, 4-byte units
    (np.int16, torch.int16, ValueKind.kI16, 2051),      # 4102-byte rows, 2-byte units
    (np.float64, torch.float64, ValueKind.kF64, 257),   # 2056-byte rows, 8-byte units
])
def test_value_types_and_dims(oracle, np_dtype, torch_dtype, kind, dim):
    # the matrix of test_find_using_pipeline (merlin_hashtable_test.cc.cu:675-798, 3816-3830)
    cap, bs = 1 << 14, 3000
    esz = np.dtype(np_dtype).itemsize
    t, o, _ = make_pair(oracle, init_capacity=cap, max_capacity=cap, dim=dim, value_size=esz,
                        value_kind=kind, evict_strategy=EvictStrategy.kCustomized)
    rng = np.random.Generator(np.random.PCG64(dim))
    for b in range(7):  # past capacity: evictions with odd row sizes
        keys = w.unique_keys(50, b * bs, bs)
        vals = rng.integers(0, 256, size=(bs, dim * esz), dtype=np.uint8)
        sc = w.monotone_scores(b + 1, bs)
        t.insert_or_assign(bs, dev(keys), dev(vals), dev(sc))
        o.insert_or_assign(keys, vals, sc)
    assert_same_table(t, o, dim * esz)
    q = w.unique_keys(50, 5 * bs, 2 * bs)
    out = torch.zeros(len(q), dim * esz, dtype=torch.uint8, device=DEV)
    founds = torch.zeros(len(q), dtype=torch.bool, device=DEV)
    t.find(len(q), dev(q), out, founds, None)
    torch.cuda.synchronize()
    ov, of, _ = o.find(q)
    assert (founds.cpu().numpy() == of).all() and of.any()
    assert (out.cpu().numpy()[of] == ov[of]).all()
    if kind != ValueKind.kBytes:
        # accum_or_assign on every arithmetic element type
        keys = q[: bs]
        if np.issubdtype(np_dtype, np.integer):
            # the whole range: carries between the bytes of an element, wrap-around at its top
            info = np.iinfo(np_dtype)
            delta = rng.integers(info.min, info.max, size=(bs, dim), dtype=np_dtype, endpoint=True)
        else:
            delta = (rng.standard_normal(size=(bs, dim)) * 1000).astype(np_dtype)
        flags = o.contains(keys)
        t.accum_or_assign(bs, dev(keys), dev(bytes_of(delta)), dev(flags.astype(np.uint8)),
                          dev(w.monotone_scores(9, bs)))
        o.accum_or_assign(keys, bytes_of(delta), flags.astype(np.uint8), w.monotone_scores(9, bs))
        assert_same_table(t, o, dim * esz)
    t.close()


def test_empty_ragged_and_reserved_batches(oracle):
    cap, dim = 1 << 12, 8
    t, o, _ = make_pair(oracle, init_capacity=cap, max_capacity=cap, dim=dim,
                        evict_strategy=EvictStrategy.kCustomized)
    t.insert_or_assign(0, None, None, None)  # n == 0: nothing is dereferenced
    t.find(0, None, None, None)
    t.erase(0, None)
    assert t.size() == 0 and t.empty()
    for n in (1, 63, 64, 65, 127, 1000):
        keys = w.unique_keys(60 + n, 0, n)
        keys[0] = np.uint64(M64 - (n % 4))  # a reserved key in every batch
        vals = w.uniform_values(60, 0, n, dim)
        sc = w.monotone_scores(n, n)
        t.insert_or_assign(n, dev(keys), dev(vals), dev(sc))
        o.insert_or_assign(keys, bytes_of(vals), sc)
        out = torch.zeros(n, dim, dtype=torch.float32, device=DEV)
        founds = torch.ones(n, dtype=torch.bool, device=DEV)
        t.find(n, dev(keys), out, founds, None)
        torch.cuda.synchronize()
        ov, of, _ = o.find(keys)
        assert (founds.cpu().numpy() == of).all() and not of[0] and of[1:].all()
        assert (bytes_of(out.cpu().numpy()) == ov).all()
    assert_same_table(t, o, dim * 4)
    t.close()


def test_non_power_of_two_capacity_and_reserved_bit(oracle):
    cap, dim, bs = 1000 * 128 - 129 + 128, 4, 1 << 13  # 1000 buckets
    t, o, _ = make_pair(oracle, init_capacity=cap, max_capacity=cap, dim=dim, reserved_key_start_bit=17,
                        evict_strategy=EvictStrategy.kCustomized)
    assert t.bucket_count() == o.bucket_count() == 1000
    assert t.capacity() == 128000
    fill(t, o, 70, 20, bs, dim, lambda b, n: w.monotone_scores(b + 1, n))
    # with start bit 17 the sentinels move: EMPTY is all ones but bit 0 (the old RECLAIM
    # value), while the old EMPTY and LOCKED values become ordinary keys
    rk = oracle.reserved_keys(17)
    assert rk[0] == M64 - 1
    special = np.array([M64, M64 - 2, M64 - 4] + rk[:3], np.uint64)
    vals = w.uniform_values(71, 0, 6, dim)
    sc = w.monotone_scores(30, 6)
    t.insert_or_assign(6, dev(special), dev(vals), dev(sc))
    o.insert_or_assign(special, bytes_of(vals), sc)
    c = torch.zeros(6, dtype=torch.bool, device=DEV)
    t.contains(6, dev(special), c)
    torch.cuda.synchronize()
    assert c.cpu().numpy().tolist() == o.contains(special).tolist() == [True] * 3 + [False] * 3
    assert_same_table(t, o, dim * 4)
    t.close()


def test_assign_family_and_find_or_insert_ptr(oracle):
    cap, dim, bs = 1 << 15, 16, 1 << 12
    t, o, _ = make_pair(oracle, init_capacity=cap, max_capacity=cap, dim=dim,
                        evict_strategy=EvictStrategy.kCustomized)
    fill(t, o, 80, 6, bs, dim, lambda b, n: w.monotone_scores(b + 1, n))
    keys = np.concatenate([w.unique_keys(80, 3 * bs, bs // 2), w.unique_keys(81, 0, bs // 2)])
    vals = w.uniform_values(82, 0, bs, dim)
    sc = w.monotone_scores(20, bs)
    t.assign(bs, dev(keys), dev(vals), dev(sc))
    o.assign(keys, bytes_of(vals), sc)
    assert t.size() == o.size()
    assert_same_table(t, o, dim * 4)
    sc = w.monotone_scores(21, bs)
    t.assign_scores(bs, dev(keys), dev(sc))
    o.assign_scores(keys, sc)
    vals = w.uniform_values(83, 0, bs, dim)
    t.assign_values(bs, dev(keys), dev(vals))
    o.assign_values(keys, bytes_of(vals))
    assert_same_table(t, o, dim * 4)
    # pointer overload of find_or_insert: hits report found, misses get a row to fill
    keys = np.concatenate([w.unique_keys(80, 4 * bs, bs // 2), w.unique_keys(84, 0, bs // 2)])
    sc = w.monotone_scores(22, bs)
    ptrs = torch.zeros(bs, dtype=torch.int64, device=DEV)
    founds = torch.zeros(bs, dtype=torch.bool, device=DEV)
    t.find_or_insert_ptr(bs, dev(keys), ptrs, founds, dev(sc))
    torch.cuda.synchronize()
    oslots, ofounds = o.find_or_insert_slot(keys, sc)
    gf = founds.cpu().numpy()
    assert (gf == ofounds.astype(bool)).all()
    gp = ptrs.cpu().numpy()
    assert ((gp != 0) == (oslots != np.uint64(M64))).all()
    assert t.size() == o.size()
    # every returned pointer is the row of its key: write through it, read back with find
    vals = w.uniform_values(85, 0, bs, dim)
    view = t.view()
    slots = (gp - view.values) // (dim * 4)
    assert (slots[gp != 0] >= 0).all() and (slots[gp != 0] < cap).all()
    t.assign_values(bs, dev(keys), dev(vals))
    torch.cuda.synchronize()
    for i in range(0, bs, 211):
        if gp[i]:
            assert (read_device(int(gp[i]), dim * 4) == bytes_of(vals)[i]).all()
    o.assign_values(keys, bytes_of(vals))
    # rows of the new keys held whatever was there before; make both sides equal first
    assert_same_table(t, o, dim * 4)
    t.close()


@pytest.mark.parametrize("strategy", [EvictStrategy.kLfu, EvictStrategy.kEpochLfu])
def test_frequency_strategies(oracle, strategy):
    cap, dim, bs = 1 << 14, 4, 1 << 12
    t, o, _ = make_pair(oracle, init_capacity=cap, max_capacity=cap, dim=dim, evict_strategy=strategy)
    with pytest.raises(MerlinException):
        t.insert_or_assign(4, dev(w.unique_keys(1, 0, 4)), dev(np.zeros((4, dim), np.float32)), None)
    if strategy == EvictStrategy.kEpochLfu:
        with pytest.raises(MerlinException):  # epoch not set
            t.insert_or_assign(4, dev(w.unique_keys(1, 0, 4)), dev(np.zeros((4, dim), np.float32)),
                               dev(np.ones(4, np.uint64)))
        t.set_global_epoch(3)
        o.set_global_epoch(3)
    # distinct frequencies, larger for later batches, so victims are well defined and
    # the keys re-used below are never the minimum of their bucket
    freq = lambda b, n: np.uint64(1000 * (b + 1)) + np.arange(n, dtype=np.uint64) * np.uint64(7919) % np.uint64(997)
    def distinct(b, n):
        return (np.uint64(b + 1) << np.uint64(20)) + np.random.Generator(np.random.PCG64(b)).permutation(n).astype(np.uint64)
    fill(t, o, 90, 6, bs, dim, distinct)
    assert_same_table(t, o, dim * 4)
    if strategy == EvictStrategy.kEpochLfu:
        t.set_global_epoch(4)
        o.set_global_epoch(4)
    keys = np.concatenate([w.unique_keys(90, 5 * bs, bs // 2), w.unique_keys(91, 0, bs // 2)])
    vals = w.uniform_values(92, 0, bs, dim)
    sc = distinct(8, bs)
    t.insert_or_assign(bs, dev(keys), dev(vals), dev(sc))
    o.insert_or_assign(keys, bytes_of(vals), sc)
    assert_same_table(t, o, dim * 4)
    # saturation of the 32-bit frequency (kernel_utils.cuh:499-512)
    if strategy == EvictStrategy.kEpochLfu:
        k4 = keys[:4].copy()
        big = np.array([0xFFFFFFF0, 0xFFFFFFFF, 0x1FFFFFFFF, 5], np.uint64)
        t.insert_or_assign(4, dev(k4), dev(vals[:4]), dev(big))
        o.insert_or_assign(k4, bytes_of(vals[:4]), big)
        assert_same_table(t, o, dim * 4)
    t.close()


def test_hybrid_mode(oracle):
    """Config 4 at reduced size: most value rows in pinned host memory, LFU,
    find / find* with 80 % hits and insert_or_assign with 20 % new keys."""
    cap, dim, bs = 1 << 16, 64, 1 << 12
    t, o, opts = make_pair(oracle, hybrid=True, init_capacity=cap, max_capacity=cap, dim=dim,
                           max_hbm_for_vectors=cap * dim * 4 // 4, evict_strategy=EvictStrategy.kLfu)
    assert not t.is_pure_hbm()
    v = t.view()
    assert v.hbm_slots == cap // 4 and v.host_values

    def distinct(b, n):
        return (np.uint64(b + 1) << np.uint64(24)) + np.random.Generator(np.random.PCG64(100 + b)).permutation(n).astype(np.uint64)
    nb = (cap + 4 * bs) // bs
    fill(t, o, 95, nb, bs, dim, distinct)
    assert t.size() == o.size()
    assert_same_table(t, o, dim * 4)
    recent = w.unique_keys(95, (nb - 2) * bs, bs)
    q = np.concatenate([recent[: bs * 8 // 10], w.unique_keys(96, 0, bs - bs * 8 // 10)])
    out = torch.zeros(bs, dim, dtype=torch.float32, device=DEV)
    founds = torch.zeros(bs, dtype=torch.bool, device=DEV)
    sc = torch.zeros(bs, dtype=torch.int64, device=DEV)
    t.find(bs, dev(q), out, founds, sc)
    ptrs = torch.zeros(bs, dtype=torch.int64, device=DEV)
    f2 = torch.zeros(bs, dtype=torch.bool, device=DEV)
    t.find_ptr(bs, dev(q), ptrs, f2, None)
    torch.cuda.synchronize()
    ov, of, osc = o.find(q)
    gf = founds.cpu().numpy()
    assert (gf == of).all() and (f2.cpu().numpy() == of).all()
    assert abs(of.mean() - 0.8) < 0.02
    assert (bytes_of(out.cpu().numpy())[of] == ov[of]).all()
    assert (host_u64(sc)[of] == osc[of]).all()
    gp = ptrs.cpu().numpy()
    in_host = (gp >= v.host_values) & (gp < v.host_values + (cap - v.hbm_slots) * dim * 4)
    in_hbm = (gp >= v.values) & (gp < v.values + v.hbm_slots * dim * 4)
    assert (in_host | in_hbm)[of].all() and in_host[of].mean() > 0.6
    for i in np.flatnonzero(of)[:: 151]:
        assert (read_device(int(gp[i]), dim * 4) == ov[i]).all()
    # insert_or_assign with 20 % new keys
    keys = np.concatenate([recent[: bs * 8 // 10], w.unique_keys(97, 0, bs - bs * 8 // 10)])
    vals = w.uniform_values(98, 0, bs, dim)
    s2 = distinct(nb + 3, bs)
    t.insert_or_assign(bs, dev(keys), dev(vals), dev(s2))
    o.insert_or_assign(keys, bytes_of(vals), s2)
    assert_same_table(t, o, dim * 4)
    # find_or_insert, and the refusal of insert_and_evict (merlin_hashtable.cuh:1384-1386)
    keys = np.concatenate([recent[bs // 2: bs], w.unique_keys(99, 0, bs // 2)])
    io = w.uniform_values(101, 0, bs, dim)
    d_io = dev(io)
    s3 = distinct(nb + 4, bs)
    t.find_or_insert(bs, dev(keys), d_io, dev(s3))
    oio = bytes_of(io).copy()
    o.find_or_insert(keys, oio, s3)
    torch.cuda.synchronize()
    assert (host_bytes(d_io, bs, dim * 4) == oio).all()
    assert_same_table(t, o, dim * 4)
    with pytest.raises(RuntimeError):
        t.insert_and_evict(bs, dev(keys), dev(io), dev(s3), torch.zeros(bs, dtype=torch.int64, device=DEV),
                           torch.zeros(bs, dim, device=DEV), torch.zeros(bs, dtype=torch.int64, device=DEV))
    t.close()


def test_hybrid_batch_holds_its_locks(oracle):
    """The reference's hybrid upsert holds every slot lock of a batch from its lock kernel to its
    write kernel (upsert.cuh:1350-1595), so an absent key never takes the slot of another key of
    its own batch: each takes the lowest-scored resident that is still visible, or is refused
    when its score is not above that.  On a one-bucket table with a batch whose scores interleave
    with the lowest resident scores the outcome depends on which key of the batch comes first, in
    the reference as here, but not in the way it would if the keys were handed over one call at
    a time (then the key with score 105 always loses its slot again to a later key; under the
    batch's locks it keeps it whenever it got one).  The GPU's result must be what the oracle's
    batch model gives for some order of the batch (all 120 are tried).  Then a batch that tells
    the two apart: 64 keys whose scores all lie between the lowest and the second lowest
    resident.  One key at a time the highest of them always ends up as the only survivor (each
    key evicts the lower one before it); under the batch's locks the survivor is whichever key
    locked the lowest resident first, and the 63 others, which see nothing below 2000, are
    refused."""
    import itertools
    dim = 4
    opts = default_options(init_capacity=128, max_capacity=128, dim=dim, max_hbm_for_vectors=0,
                           evict_strategy=EvictStrategy.kCustomized)
    keys = w.unique_keys(311, 0, 128)
    vals = w.values_from_keys(keys, dim)
    sc = np.arange(100, 100 + 10 * 128, 10, dtype=np.uint64)
    batch = w.unique_keys(312, 0, 5)
    bvals = w.values_from_keys(batch, dim)
    bsc = np.array([105, 200, 115, 125, 99], np.uint64)

    def resident_map(table):
        ek, _, es = table.export_all()
        return frozenset(zip(ek.tolist(), es.tolist()))

    serial, batched = set(), set()
    for order in itertools.permutations(range(5)):
        o = oracle.OracleTable(opts, hybrid=True)
        o.insert_or_assign(keys, bytes_of(vals), sc)
        for i in order:
            o.insert_or_assign(batch[i:i + 1], bytes_of(bvals[i:i + 1]), bsc[i:i + 1])
        serial.add(resident_map(o))
        o.close()
        o = oracle.OracleTable(opts, hybrid=True)
        o.insert_or_assign(keys, bytes_of(vals), sc)
        p = list(order)
        o.insert_or_assign(batch[p], bytes_of(bvals[p]), bsc[p])
        batched.add(resident_map(o))
        o.close()
    assert len(batched) > len(serial) == 1

    for rep in range(5):
        t = HashTable()
        t.init(opts)
        assert not t.is_pure_hbm()
        t.insert_or_assign(128, dev(keys), dev(vals), dev(sc))
        t.insert_or_assign(5, dev(batch), dev(bvals), dev(bsc))
        gk, gv, gs = export_table(t, dim * 4)
        assert frozenset(zip(gk.tolist(), gs.tolist())) in batched
        allv = {int(k): v for k, v in zip(np.concatenate([keys, batch]), np.concatenate([bytes_of(vals), bytes_of(bvals)]))}
        assert all((gv[i] == allv[int(k)]).all() for i, k in enumerate(gk))  # every resident carries its own row
        assert t.size() == 128
        # find_or_insert follows the same kernels (find_or_insert.cuh:1417-1676)
        io = dev(bvals.copy())
        t.find_or_insert(5, dev(batch), io, dev(bsc))
        torch.cuda.synchronize()
        assert t.size() == 128
        t.close()

    sc = np.arange(1000, 1000 * 129, 1000, dtype=np.uint64)
    crowd = w.unique_keys(313, 0, 64)
    cvals = w.values_from_keys(crowd, dim)
    survivors = []
    for top_at in (0, 63, 31, 62):  # where the highest score of the batch sits
        csc = np.arange(1001, 1065, dtype=np.uint64)
        csc[[top_at, 63]] = csc[[63, top_at]]
        for call in ("insert_or_assign", "find_or_insert"):
            t = HashTable()
            t.init(opts)
            t.insert_or_assign(128, dev(keys), dev(vals), dev(sc))
            if call == "insert_or_assign":
                t.insert_or_assign(64, dev(crowd), dev(cvals), dev(csc))
            else:
                t.find_or_insert(64, dev(crowd), dev(cvals.copy()), dev(csc))
            gk, gv, gs = export_table(t, dim * 4)
            mine = np.isin(gk, crowd)
            assert mine.sum() == 1 and t.size() == 128 and keys[0] not in gk
            who = int(np.flatnonzero(crowd == gk[mine][0])[0])
            assert gs[mine][0] == csc[who] and (gv[mine][0] == bytes_of(cvals)[who]).all()
            survivors.append(csc[who] == 1064)
            t.close()
    assert not all(survivors)  # one key at a time it would be the highest score every time



def test_io_by_cpu(oracle):
    """io_by_cpu (merlin_hashtable.cuh:1275-1292, 1820-1841, 2175-2192, 2414-2431): all rows in
    pinned host memory, host threads move the rows of insert_or_assign, find_or_insert, assign
    and assign_values; the upserts follow the plain kernels' rule (refuse when score < min)."""
    cap, dim, bs = 1 << 15, 16, 1 << 12
    with pytest.raises(MerlinException):  # merlin_hashtable.cuh:1071-1073
        HashTable().init(default_options(init_capacity=cap, max_capacity=cap, dim=dim,
                                         max_hbm_for_vectors=1 << 20, io_by_cpu=1))
    t, o, _ = make_pair(oracle, hybrid=False, init_capacity=cap, max_capacity=cap, dim=dim,
                        max_hbm_for_vectors=0, io_by_cpu=1, evict_strategy=EvictStrategy.kCustomized)
    assert not t.is_pure_hbm() and t.view().hbm_slots == 0

    def distinct(b, n):
        return (np.uint64(b + 1) << np.uint64(24)) + np.random.Generator(np.random.PCG64(300 + b)).permutation(n).astype(np.uint64)
    nb = (cap + 3 * bs) // bs  # past load factor 1.0: the last batches evict
    fill(t, o, 131, nb, bs, dim, distinct)
    assert t.size() == o.size()
    assert_same_table(t, o, dim * 4)
    recent = w.unique_keys(131, (nb - 2) * bs, bs)
    # insert_or_assign, half hits; a refusal at score == min would show (plain rule: accepted)
    keys = np.concatenate([recent[: bs // 2], w.unique_keys(132, 0, bs // 2),
                           np.array([M64, M64 - 2], np.uint64)])
    n = len(keys)
    vals = w.uniform_values(133, 0, n, dim)
    sc = distinct(nb + 2, n)
    t.insert_or_assign(n, dev(keys), dev(vals), dev(sc))
    o.insert_or_assign(keys, bytes_of(vals), sc)
    assert_same_table(t, o, dim * 4)
    # find_or_insert: hits read, new keys write
    keys = np.concatenate([recent[bs // 2:], w.unique_keys(134, 0, bs // 2)])
    io = w.uniform_values(135, 0, bs, dim)
    d_io = dev(io)
    sc = distinct(nb + 3, bs)
    t.find_or_insert(bs, dev(keys), d_io, dev(sc))
    oio = bytes_of(io).copy()
    o.find_or_insert(keys, oio, sc)
    torch.cuda.synchronize()
    assert (host_bytes(d_io, bs, dim * 4) == oio).all()
    assert_same_table(t, o, dim * 4)
    # assign (rows + scores) and assign_values (rows only), 50 % present
    keys = np.concatenate([recent[: bs // 2], w.unique_keys(136, 0, bs // 2)])
    vals = w.uniform_values(137, 0, bs, dim)
    sc = distinct(nb + 4, bs)
    t.assign(bs, dev(keys), dev(vals), dev(sc))
    o.assign(keys, bytes_of(vals), sc)
    assert_same_table(t, o, dim * 4)
    vals = w.uniform_values(138, 0, bs, dim)
    t.assign_values(bs, dev(keys), dev(vals))
    o.assign_values(keys, bytes_of(vals))
    assert_same_table(t, o, dim * 4)
    # the reading calls are the ordinary ones
    out = torch.zeros(bs, dim, dtype=torch.float32, device=DEV)
    founds = torch.zeros(bs, dtype=torch.bool, device=DEV)
    t.find(bs, dev(keys), out, founds, None)
    torch.cuda.synchronize()
    ov, of, _ = o.find(keys)
    assert (founds.cpu().numpy() == of).all() and (bytes_of(out.cpu().numpy())[of] == ov[of]).all()
    t.close()


def test_calls_on_two_streams_are_ordered_by_role(oracle):
    """Writers and readers on different streams: the group lock orders them the
    way the calls were issued (group_lock.cuh:43-56), without host syncs."""
    cap, dim, bs = 1 << 16, 32, 1 << 14
    t, o, _ = make_pair(oracle, init_capacity=cap, max_capacity=cap, dim=dim,
                        evict_strategy=EvictStrategy.kCustomized)
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    outs = []
    keep = []
    for b in range(6):
        keys = w.unique_keys(110, b * bs, bs)
        vals = w.uniform_values(110, b * bs, bs, dim)
        sc = w.monotone_scores(b + 1, bs)
        dk, dv, ds = dev(keys), dev(vals), dev(sc)
        torch.cuda.synchronize()
        t.insert_or_assign(bs, dk, dv, ds, stream=s1)
        o.insert_or_assign(keys, bytes_of(vals), sc)
        out = torch.zeros(bs, dim, dtype=torch.float32, device=DEV)
        founds = torch.zeros(bs, dtype=torch.bool, device=DEV)
        t.find(bs, dk, out, founds, None, stream=s2)  # must see the insert issued just before
        ov, of, _ = o.find(keys)
        outs.append((out, founds, ov, of))
        keep.append((dk, dv, ds))
    torch.cuda.synchronize()
    for out, founds, ov, of in outs:
        gf = founds.cpu().numpy()
        assert (gf == of).all()
        assert (bytes_of(out.cpu().numpy())[of] == ov[of]).all()
    assert_same_table(t, o, dim * 4)
    t.close()


def test_assign_family_on_two_streams_and_with_repeated_keys(oracle):
    """Updaters issued on different streams take effect in the order of the calls (each is
    alone on the table, which is what lets the assign kernels run without slot locks);
    unique_key=False keeps the slot locks: a repeated key gets one of its rows, whole."""
    cap, dim, bs = 1 << 15, 64, 1 << 13
    t, o, _ = make_pair(oracle, init_capacity=cap, max_capacity=cap, dim=dim,
                        evict_strategy=EvictStrategy.kCustomized)
    fill(t, o, 141, 3, bs, dim, lambda b, n: w.monotone_scores(b + 1, n))
    keys = np.concatenate([w.unique_keys(141, bs, bs // 2), w.unique_keys(142, 0, bs // 2)])
    dk = dev(keys)
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    keep = []
    torch.cuda.synchronize()
    for r in range(6):
        vals = w.uniform_values(143 + r, 0, bs, dim)
        sc = w.monotone_scores(10 + r, bs)
        dv, ds = dev(vals), dev(sc)
        keep.append((dv, ds))
        torch.cuda.synchronize()
        if r % 3 == 0:
            t.assign(bs, dk, dv, ds, stream=(s1, s2)[r % 2])
            o.assign(keys, bytes_of(vals), sc)
        elif r % 3 == 1:
            t.assign_values(bs, dk, dv, stream=(s1, s2)[r % 2])
            o.assign_values(keys, bytes_of(vals))
        else:
            t.assign_scores(bs, dk, ds, stream=(s1, s2)[r % 2])
            o.assign_scores(keys, sc)
    torch.cuda.synchronize()
    assert_same_table(t, o, dim * 4)
    # repeated keys: 64 copies of each of 128 resident keys, every copy with its own row
    base = w.unique_keys(141, 2 * bs, 128)
    rep = np.repeat(base, 64)
    rows = np.arange(len(rep), dtype=np.float32)[:, None] + np.zeros((1, dim), np.float32)
    t.assign_values(len(rep), dev(rep), dev(rows), unique_key=False)
    out = torch.zeros(128, dim, dtype=torch.float32, device=DEV)
    founds = torch.zeros(128, dtype=torch.bool, device=DEV)
    t.find(128, dev(base), out, founds, None)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert founds.cpu().numpy().all()
    assert (got == got[:, :1]).all()  # one writer's row, not a mixture
    assert ((got[:, 0] // 64).astype(np.int64) == np.arange(128)).all()
    t.close()


def test_error_classes(oracle):
    t = HashTable()
    t.init(default_options(init_capacity=1024, max_capacity=1024, max_hbm_for_vectors=1 << 30, dim=4,
                           evict_strategy=EvictStrategy.kLru))
    k = dev(w.unique_keys(1, 0, 8))
    v = dev(np.zeros((8, 4), np.float32))
    with pytest.raises(MerlinException):  # LRU takes no scores (merlin_hashtable.cuh:3834-3839)
        t.insert_or_assign(8, k, v, dev(np.ones(8, np.uint64)))
    t.insert_or_assign(8, k, v, dev(np.ones(8, np.uint64)), ignore_evict_strategy=True)
    assert t.size() == 8
    with pytest.raises(ValueError):
        t.export_batch_if(99, 0, 0, 10, 0, torch.zeros(1, dtype=torch.int64, device=DEV), k, v)
    t2 = HashTable()
    t2.init(default_options(init_capacity=1024, max_capacity=1024, max_hbm_for_vectors=1 << 30, dim=4,
                            value_kind=ValueKind.kBytes, evict_strategy=EvictStrategy.kLru))
    with pytest.raises(ValueError):
        t2.accum_or_assign(8, k, v, torch.zeros(8, dtype=torch.bool, device=DEV))
    t.close()
    t2.close()


def test_growth_reserve_and_rehash(oracle):
    # reserve / rehash and the growth loop at the head of the inserting calls
    # (merlin_hashtable.cuh:3503-3541, 1151-1154); scenario of test_rehash
    # (merlin_hashtable_test.cc.cu:1078-1200) at a larger size, plus evictions once
    # max_capacity is reached
    dim, bs = 8, 3000
    t, o, _ = make_pair(oracle, init_capacity=1 << 12, max_capacity=1 << 15, dim=dim,
                        max_load_factor=0.5, evict_strategy=EvictStrategy.kCustomized)
    assert t.capacity() == o.capacity() == 1 << 12
    caps = []
    for b in range(16):  # 48000 keys into at most 32768 slots
        keys = w.unique_keys(77, b * bs, bs)
        vals = w.values_from_keys(keys, dim)
        sc = w.monotone_scores(b + 1, bs)
        t.insert_or_assign(bs, dev(keys), dev(vals), dev(sc))
        o.insert_or_assign(keys, vals.view(np.uint8).reshape(bs, -1), sc)
        assert t.capacity() == o.capacity()
        assert t.size() == o.size()
        caps.append(t.capacity())
    assert caps[0] > 1 << 12 and caps[-1] == 1 << 15 and sorted(caps) == caps
    assert_same_table(t, o, dim * 4)
    t.close()
    # explicit reserve on a table that does not grow by itself
    t, o, _ = make_pair(oracle, init_capacity=1 << 12, max_capacity=1 << 14, dim=dim,
                        max_load_factor=4.0, evict_strategy=EvictStrategy.kLru)
    t.set_clock(1, 1 << 40)
    o.set_clock(1, 1 << 40)
    for b in range(2):  # 6000 keys into 4096 slots: evictions, then tombstones
        keys = w.unique_keys(78, b * bs, bs)
        vals = w.values_from_keys(keys, dim)
        t.insert_or_assign(bs, dev(keys), dev(vals))
        o.insert_or_assign(keys, vals.view(np.uint8).reshape(bs, -1))
    gone = w.unique_keys(78, bs, 500)
    t.erase(500, dev(gone))
    o.erase(gone)
    for want in (5000, 1 << 14, 1 << 20):
        t.reserve(want)
        o.reserve(want)
        assert t.capacity() == o.capacity()
        assert t.size() == o.size()
        assert_same_table(t, o, dim * 4)
    assert t.capacity() == 1 << 14
    keys = w.unique_keys(78, 2 * bs, bs)
    vals = w.values_from_keys(keys, dim)
    t.insert_or_assign(bs, dev(keys), dev(vals))
    o.insert_or_assign(keys, vals.view(np.uint8).reshape(bs, -1))
    assert_same_table(t, o, dim * 4)
    t.close()


def test_lock_keys_unlock_keys_find_and_update(oracle):
    # merlin_hashtable.cuh:1982-2044, 2811-2843
    cap, dim, bs = 1 << 13, 8, 6000
    t, o, _ = make_pair(oracle, init_capacity=cap, max_capacity=cap, dim=dim,
                        evict_strategy=EvictStrategy.kCustomized)
    keys = w.unique_keys(91, 0, bs)
    vals = w.values_from_keys(keys, dim)
    sc = w.monotone_scores(1, bs)
    t.insert_or_assign(bs, dev(keys), dev(vals), dev(sc))
    o.insert_or_assign(keys, vals.view(np.uint8).reshape(bs, -1), sc)
    n = 1500
    batch = np.concatenate([keys[:1200], w.unique_keys(92, 0, n - 1200)])
    new_sc = w.monotone_scores(2, n)
    ptrs = torch.zeros(n, dtype=torch.int64, device=DEV)
    ok = torch.zeros(n, dtype=torch.bool, device=DEV)
    t.lock_keys(n, dev(batch), ptrs, ok, scores=dev(new_sc))
    oslots, ook = o.lock_keys(batch, new_sc)
    assert (ok.cpu().numpy() == ook).all() and ook[:1200].all() and not ook[1200:].any()
    assert bool(((ptrs != 0) == ok).all())
    founds = torch.zeros(bs, dtype=torch.bool, device=DEV)
    t.contains(bs, dev(keys), founds)
    assert (founds.cpu().numpy() == o.contains(keys)).all() and not bool(founds[:1200].any())
    assert t.size() == o.size()
    # inserting while keys are locked: locked slots are never victims
    more = w.unique_keys(93, 0, 4000)
    mv = w.values_from_keys(more, dim)
    ms = w.monotone_scores(3, 4000)
    t.insert_or_assign(4000, dev(more), dev(mv), dev(ms))
    o.insert_or_assign(more, mv.view(np.uint8).reshape(4000, -1), ms)
    assert t.size() == o.size()
    ok2 = torch.zeros(n, dtype=torch.bool, device=DEV)
    t.unlock_keys(n, ptrs, dev(batch), ok2)
    assert (ok2.cpu().numpy() == o.unlock_keys(oslots, batch)).all()
    t.unlock_keys(n, ptrs, dev(batch), ok2)
    assert not bool(ok2.any())
    assert_same_table(t, o, dim * 4)
    t.close()
    # find_and_update under LFU: rows through the returned addresses, scores after the touch
    t, o, _ = make_pair(oracle, init_capacity=cap, max_capacity=cap, dim=dim, evict_strategy=EvictStrategy.kLfu)
    cnt = (np.arange(bs, dtype=np.uint64) % 7) + 1
    t.insert_or_assign(bs, dev(keys), dev(vals), dev(cnt))
    o.insert_or_assign(keys, vals.view(np.uint8).reshape(bs, -1), cnt)
    add = (np.arange(n, dtype=np.uint64) % 5) + 1
    dsc = dev(add.copy())
    vp = torch.zeros(n, dtype=torch.int64, device=DEV)
    fd = torch.zeros(n, dtype=torch.bool, device=DEV)
    t.find_and_update(n, dev(batch), vp, fd, dsc)
    oslots, of, osc = o.find_and_update(batch, add)
    assert (fd.cpu().numpy() == of).all() and of[:1200].all() and not of[1200:].any()
    assert (host_u64(dsc) == osc).all()
    vpn = vp.cpu().numpy()
    assert (vpn[1200:] == 0).all()
    for i in (0, 7, 1199):
        row = read_device(int(vpn[i]), dim * 4)
        assert (row == vals[i].view(np.uint8)).all()
    assert_same_table(t, o, dim * 4)
    t.close()


def test_batches_with_repeated_keys(oracle):
    """unique_key = false: every key ends up in the table once, whatever the call
    (tests/find_or_insert_ptr_test.cc.cu:3390-3475: 1024 copies of one key leave one entry);
    which occurrence wins is unspecified, so values and scores are checked against the set of
    the key's occurrences."""
    cap, dim = 1 << 14, 8
    o = default_options(init_capacity=cap, max_capacity=cap, max_hbm_for_vectors=1 << 30, dim=dim,
                        evict_strategy=EvictStrategy.kCustomized)
    rng = np.random.default_rng(314)
    # the reference's scenario: one key, 1024 times, through the pointer overload
    t = HashTable()
    t.init(o)
    n = 1024
    same = np.full(n, 0x0101010101010101, dtype=np.uint64)
    ptrs = torch.zeros(n, dtype=torch.int64, device=DEV)
    founds = torch.ones(n, dtype=torch.bool, device=DEV)
    sc = np.arange(1, n + 1, dtype=np.uint64)
    t.find_or_insert_ptr(n, dev(same), ptrs, founds, dev(sc), unique_key=False)
    torch.cuda.synchronize()
    assert t.size() == 1
    p = ptrs.cpu().numpy()
    assert p[0] != 0 and (p == p[0]).all() and not founds.cpu().numpy().any()
    t.find_or_insert_ptr(n, dev(same), ptrs, founds, dev(sc), unique_key=False)
    torch.cuda.synchronize()
    assert t.size() == 1 and (ptrs.cpu().numpy() == p[0]).all() and founds.cpu().numpy().all()
    t.close()

    # insert_or_assign: 4096 occurrences of 1000 keys
    t = HashTable()
    t.init(o)
    uniq = w.unique_keys(61, 0, 1000)
    n = 4096
    pick = rng.integers(0, 1000, n)
    pick[:1000] = np.arange(1000)  # every key at least once
    keys = uniq[pick]
    vals = rng.random((n, dim), dtype=np.float32)
    sc = rng.permutation(n).astype(np.uint64) + np.uint64(10)
    t.insert_or_assign(n, dev(keys), dev(vals), dev(sc), unique_key=False)
    assert t.size() == 1000
    ek, ev, es = sort_by_key(*export_table(t, dim * 4))
    assert np.array_equal(ek, np.sort(uniq))
    vb = bytes_of(vals)
    for i in range(0, 1000, 37):
        occ = np.flatnonzero(keys == ek[i])
        hit = [j for j in occ if np.array_equal(vb[j], ev[i]) and sc[j] == es[i]]
        assert hit, "the resident row and score must come from one occurrence of the key"
    # find_or_insert with values: all occurrences of a key read the same row, the table's
    q = np.concatenate([keys[:2000], w.unique_keys(62, 0, 500), w.unique_keys(62, 0, 500)])
    m = len(q)
    io = torch.from_numpy(rng.random((m, dim), dtype=np.float32)).to(DEV)
    qs = rng.permutation(m).astype(np.uint64) + np.uint64(100000)
    t.find_or_insert(m, dev(q), io, dev(qs), unique_key=False)
    torch.cuda.synchronize()
    assert t.size() == 1500
    got = bytes_of(io.cpu().numpy())
    out = torch.zeros(m, dim, dtype=torch.float32, device=DEV)
    f = torch.zeros(m, dtype=torch.bool, device=DEV)
    t.find(m, dev(q), out, f)
    torch.cuda.synchronize()
    assert f.cpu().numpy().all()
    assert np.array_equal(got, bytes_of(out.cpu().numpy()))
    t.close()

    # insert_and_evict on a full table: what left + what stayed == what was there + new keys
    t = HashTable()
    t.init(o)
    for b in range(5):
        k = w.unique_keys(63, b * 4096, 4096)
        t.insert_or_assign(4096, dev(k), dev(rng.random((4096, dim), dtype=np.float32)),
                           dev(w.monotone_scores(b + 1, 4096)))
    before = t.size()
    fresh = w.unique_keys(64, 0, 1500)
    keys = np.concatenate([fresh, fresh[:700], fresh[100:400]])
    n = len(keys)
    ek = torch.zeros(n, dtype=torch.int64, device=DEV)
    evv = torch.zeros(n, dim, dtype=torch.float32, device=DEV)
    es = torch.zeros(n, dtype=torch.int64, device=DEV)
    c = t.insert_and_evict(n, dev(keys), dev(rng.random((n, dim), dtype=np.float32)),
                           dev(w.monotone_scores(9, n)), ek, evv, es, unique_key=False)
    assert c + t.size() == before + 1500
    assert len(np.unique(host_u64(ek)[:c])) == c
    gk, _, _ = export_table(t, dim * 4)
    assert len(np.unique(gk)) == len(gk)
    t.close()


def test_find_or_insert_with_locked_key_pointers(oracle):
    """find_or_insert(…, locked_key_ptrs): the accepted keys stay LOCKED (invisible to lookups)
    until unlock_keys, and the table then equals what the plain pointer overload leaves
    (merlin_hashtable.cuh:1878-1927, find_ptr_or_insert.cuh:27-245)."""
    cap, dim, bs = 1 << 13, 8, 7000
    t, o, _ = make_pair(oracle, init_capacity=cap, max_capacity=cap, dim=dim,
                        evict_strategy=EvictStrategy.kCustomized)
    keys = w.unique_keys(95, 0, bs)
    vals = w.values_from_keys(keys, dim)
    sc = w.monotone_scores(1, bs)
    # the keys that the batch below finds again hold the highest scores: a key of that batch that
    # evicts cannot take one of them before its own turn (it would come back as a new key, which is
    # one of the outcomes a concurrent batch may have, but not the one the oracle's order gives)
    sc[:1000] += np.uint64(1 << 39)
    t.insert_or_assign(bs, dev(keys), dev(vals), dev(sc))
    o.insert_or_assign(keys, vals.view(np.uint8).reshape(bs, -1), sc)
    n = 3000
    batch = np.concatenate([keys[:1000], w.unique_keys(96, 0, n - 1000),
                            np.array([M64, M64 - 1], np.uint64)])
    n = len(batch)
    bsc = w.monotone_scores(2, n)
    vptrs = torch.zeros(n, dtype=torch.int64, device=DEV)
    kptrs = torch.zeros(n, dtype=torch.int64, device=DEV)
    founds = torch.zeros(n, dtype=torch.bool, device=DEV)
    t.find_or_insert_ptr(n, dev(batch), vptrs, founds, dev(bsc), locked_key_ptrs=kptrs)
    torch.cuda.synchronize()
    oslots, of = o.find_or_insert_slot(batch, bsc)
    accepted = (of != 2) & (oslots != np.uint64(M64))  # reserved keys are not looked at at all
    assert np.array_equal(founds.cpu().numpy()[accepted], of[accepted].astype(bool))
    vp, kp = vptrs.cpu().numpy(), kptrs.cpu().numpy()
    assert np.array_equal(vp != 0, accepted) and np.array_equal(kp != 0, accepted)
    assert accepted[:n - 2].sum() > 2000 and not accepted[-2:].any()
    assert t.size() == o.size()
    # every accepted key is invisible while locked, the rest of the table is not
    c = torch.zeros(n, dtype=torch.bool, device=DEV)
    t.contains(n, dev(batch), c)
    torch.cuda.synchronize()
    assert not c.cpu().numpy().any()
    c2 = torch.zeros(bs, dtype=torch.bool, device=DEV)
    t.contains(bs, dev(keys), c2)
    untouched = o.contains(keys)
    untouched[:1000] = False
    assert np.array_equal(c2.cpu().numpy(), untouched)
    # rows are written through the value pointers, then the keys are released
    newrows = w.values_from_keys(batch, dim) + np.float32(0.5)
    import ctypes as C
    from gpu_util import hip
    for i in np.flatnonzero(accepted)[::41]:
        row = np.ascontiguousarray(newrows[i])
        assert hip().hipMemcpy(C.c_void_p(int(vp[i])), row.ctypes.data, dim * 4, 1) == 0
    ok = torch.zeros(n, dtype=torch.bool, device=DEV)
    t.unlock_keys(n, kptrs, dev(batch), ok)
    torch.cuda.synchronize()
    assert np.array_equal(ok.cpu().numpy(), accepted)
    out = torch.zeros(n, dim, dtype=torch.float32, device=DEV)
    f = torch.zeros(n, dtype=torch.bool, device=DEV)
    s = torch.zeros(n, dtype=torch.int64, device=DEV)
    t.find(n, dev(batch), out, f, s)
    torch.cuda.synchronize()
    assert np.array_equal(f.cpu().numpy(), accepted)
    outn = out.cpu().numpy()
    for i in np.flatnonzero(accepted)[::41]:
        assert np.array_equal(outn[i], newrows[i])
    # keys and scores equal the oracle's table (rows of new keys are the caller's business)
    gk, _, gs = sort_by_key(*export_table(t, dim * 4))
    ok_, _, os_ = sort_by_key(*o.export_all())
    assert np.array_equal(gk, ok_) and np.array_equal(gs, os_)
    t.close()


def test_growth_under_host_threads():
    """tests/merlin_hashtable_test.cc.cu:1441-1580 (test_dynamic_rehash_on_multi_threads): eight
    host threads, each on its own stream, insert and look up 256 keys at a time while the table
    grows from 32 buckets by repeated rehash; every thread finds what it has just inserted."""
    import threading
    init_cap, dim, n, n_threads = 4 * 1024 - 128 - 1, 16, 256, 8
    max_cap = 1024 * init_cap
    t = HashTable()
    t.init(default_options(init_capacity=init_cap, max_capacity=max_cap, dim=dim, reserved_key_start_bit=8,
                           num_of_buckets_per_alloc=16, max_load_factor=0.5, max_hbm_for_vectors=1 << 34,
                           evict_strategy=EvictStrategy.kLru))
    assert t.bucket_count() == 32
    errors, rounds = [], [0] * n_threads

    def worker(tid):
        try:
            torch.cuda.set_device(0)
            st = torch.cuda.Stream()
            pos = 0
            while t.capacity() * 2 < max_cap:
                keys = w.unique_keys(1000 + tid, pos, n)
                pos += n
                vals = w.values_from_keys(keys, dim)
                dk, dv = dev(keys), dev(vals)
                out = torch.zeros(n, dim, dtype=torch.float32, device=DEV)
                founds = torch.zeros(n, dtype=torch.bool, device=DEV)
                f2 = torch.zeros(n, dtype=torch.bool, device=DEV)
                torch.cuda.current_stream().synchronize()
                t.insert_or_assign(n, dk, dv, None, stream=st)
                st.synchronize()
                t.find(n, dk, out, founds, None, stream=st)
                t.contains(n, dk, f2, stream=st)
                st.synchronize()
                assert bool(founds.all()) and bool(f2.all()), (tid, rounds[tid])
                assert np.array_equal(out.cpu().numpy(), vals), (tid, rounds[tid])
                rounds[tid] += 1
        except BaseException as e:  # noqa: BLE001 - reported by the main thread
            errors.append((tid, repr(e)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(n_threads)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors[:3]
    assert t.capacity() * 2 >= max_cap and min(rounds) > 0
    assert t.size() <= sum(rounds) * n
    t.close()


@pytest.mark.parametrize("hbm", [1 << 34, 0, 1024 * 8 * 4])
def test_rehash_on_big_batches(oracle, hbm):
    """tests/merlin_hashtable_test.cc.cu:1223-1367 (test_rehash_on_big_batch) and :1369-1439
    (test_rehash_on_big_batch_specific): the capacities the growth loop arrives at; with all rows
    in HBM, all in host memory (the reference runs its rehash tests both ways) and with an HBM
    budget that the growing table leaves behind."""
    dim = 8
    t, o, _ = make_pair(oracle, hybrid=hbm < (1 << 34), init_capacity=1024, max_capacity=16 * 1024, dim=dim,
                        reserved_key_start_bit=6, num_of_buckets_per_alloc=8, max_load_factor=0.6,
                        max_hbm_for_vectors=hbm, evict_strategy=EvictStrategy.kCustomized)
    keys = w.unique_keys(151, 0, 2048)
    keys = keys[(keys & np.uint64(~(3 << 6) & M64 & ~1)) != np.uint64(~(3 << 6) & M64 & ~1)]
    assert len(keys) == 2048
    vals = w.values_from_keys(keys, dim)
    for n, cap in ((1024, 2048), (2048, 8192)):
        t.insert_or_assign(n, dev(keys[:n]), dev(vals[:n]), dev(keys[:n].copy()))
        o.insert_or_assign(keys[:n], bytes_of(vals[:n]), keys[:n].copy())
        assert t.size() == o.size() == n
        assert t.capacity() == o.capacity() == cap
    ek, ev, es = export_table(t, dim * 4)
    assert len(ek) == 2048
    out = torch.zeros(2048, dim, dtype=torch.float32, device=DEV)
    founds = torch.zeros(2048, dtype=torch.bool, device=DEV)
    sc = torch.zeros(2048, dtype=torch.int64, device=DEV)
    t.find(2048, dev(keys), out, founds, sc)
    torch.cuda.synchronize()
    assert bool(founds.all()) and np.array_equal(host_u64(sc), keys)
    assert np.array_equal(out.cpu().numpy(), vals)
    assert_same_table(t, o, dim * 4)
    t.close()
    # 50 000 slots asked for, 100 000 allowed: 512 buckets, and no room to double
    t, o, _ = make_pair(oracle, hybrid=hbm < (1 << 34), init_capacity=50000, max_capacity=100000, dim=dim,
                        reserved_key_start_bit=7, num_of_buckets_per_alloc=16, max_load_factor=0.6,
                        max_hbm_for_vectors=hbm, evict_strategy=EvictStrategy.kLru)
    t.set_clock(1, 1 << 40)
    o.set_clock(1, 1 << 40)
    keys = w.unique_keys(152, 0, 50000)
    vals = w.values_from_keys(keys, dim)
    t.insert_or_assign(50000, dev(keys), dev(vals))
    o.insert_or_assign(keys, bytes_of(vals))
    assert t.capacity() == o.capacity() == 65536
    assert t.size() == o.size()
    assert_same_table(t, o, dim * 4)
    t.close()


def test_tombstones_are_never_reported_as_evicted(oracle):
    """tests/insert_and_evict_test.cc.cu:1654-1710 (test_insert_and_evict_bugfix_no_zero_eviction):
    fill a 2048-slot LRU table, erase half, insert 2048 new keys with insert_and_evict: slots of
    erased keys are taken without an eviction being reported, and every reported key is a key
    that was resident."""
    cap, dim = 2048, 8
    t, o, _ = make_pair(oracle, init_capacity=cap, max_capacity=cap, dim=dim, num_of_buckets_per_alloc=16,
                        evict_strategy=EvictStrategy.kLru)
    t.set_clock(1, 1 << 40)
    o.set_clock(1, 1 << 40)

    def evict_call(keys):
        n = len(keys)
        vals = w.values_from_keys(keys, dim)
        ek = torch.zeros(n, dtype=torch.int64, device=DEV)
        ev = torch.zeros(n, dim, dtype=torch.float32, device=DEV)
        got = t.insert_and_evict(n, dev(keys), dev(vals), None, ek, ev, None)  # count-returning overload
        oek, oev, _ = o.insert_and_evict(keys, bytes_of(vals))
        torch.cuda.synchronize()
        gk = host_u64(ek)[:got]
        gv = host_bytes(ev, n, dim * 4)[:got]
        assert got == len(oek)
        a, b = np.argsort(gk, kind="stable"), np.argsort(oek, kind="stable")
        assert np.array_equal(gk[a], oek[b]) and np.array_equal(gv[a], oev[b])
        return gk

    first = np.arange(1, cap + 1, dtype=np.uint64)
    evict_call(first)
    t.erase(1024, dev(first[:1024]))
    o.erase(first[:1024])
    assert t.size() == o.size()
    resident = set(export_table(t, dim * 4)[0].tolist())
    new = np.arange(3000, 3000 + cap, dtype=np.uint64)
    gone = evict_call(new)
    assert 0 not in set(gone.tolist())
    assert set(gone.tolist()) <= resident | set(new.tolist())  # residents, or refused new keys
    assert not (set(gone.tolist()) & set(first[:1024].tolist()))  # nothing that had been erased
    assert_same_table(t, o, dim * 4)
    t.close()


def test_insert_and_evict_beside_find_on_another_thread():
    """tests/insert_and_evict_test.cc.cu:1713-1790 (test_insert_and_evict_run_with_batch_find): one
    host thread inserts with eviction, another looks keys up on a stream of its own; the group lock
    keeps the two kinds of call apart.  Checked here: every lookup sees whole rows, and keys are
    conserved (inserted = resident + evicted)."""
    import threading
    cap, dim, bs, batches = 1 << 18, 16, 1 << 14, 48
    t = HashTable()
    t.init(default_options(init_capacity=cap, max_capacity=cap, dim=dim, max_hbm_for_vectors=1 << 34,
                           num_of_buckets_per_alloc=128, evict_strategy=EvictStrategy.kLru))
    keys = [w.unique_keys(161, b * bs, bs) for b in range(batches)]
    step, errors, evicted_total = [0], [], [0]

    def inserter():
        try:
            st = torch.cuda.Stream()
            ek = torch.zeros(bs, dtype=torch.int64, device=DEV)
            ev = torch.zeros(bs, dim, dtype=torch.float32, device=DEV)
            for b in range(batches):
                dk, dv = dev(keys[b]), dev(w.values_from_keys(keys[b], dim))
                torch.cuda.current_stream().synchronize()
                got = t.insert_and_evict(bs, dk, dv, None, ek, ev, None, stream=st)
                st.synchronize()
                gk = host_u64(ek)[:got]
                rows = ev.cpu().numpy()[:got]
                assert np.array_equal(rows, w.values_from_keys(gk, dim)), b  # evicted rows are whole
                evicted_total[0] += got
                step[0] = b + 1
        except BaseException as e:  # noqa: BLE001
            errors.append(("insert", repr(e)))
            step[0] = batches

    def finder():
        try:
            st = torch.cuda.Stream()
            out = torch.zeros(bs, dim, dtype=torch.float32, device=DEV)
            founds = torch.zeros(bs, dtype=torch.bool, device=DEV)
            rounds = 0
            while step[0] < batches or rounds == 0:
                b = max(step[0] - 1, 0)
                dk = dev(keys[b])
                torch.cuda.current_stream().synchronize()
                t.find(bs, dk, out, founds, None, stream=st)
                st.synchronize()
                f = founds.cpu().numpy()
                rows = out.cpu().numpy()
                assert np.array_equal(rows[f], w.values_from_keys(keys[b], dim)[f]), b
                rounds += 1
        except BaseException as e:  # noqa: BLE001
            errors.append(("find", repr(e)))

    th = [threading.Thread(target=finder), threading.Thread(target=inserter)]
    for x in th:
        x.start()
    for x in th:
        x.join()
    assert not errors, errors
    assert t.size() + evicted_total[0] == batches * bs
    assert t.size() > 0.95 * cap
    t.close()


def test_insert_and_evict_with_export_batch_scenario():
    """tests/insert_and_evict_test.cc.cu:1311-1385: 4096 + 13 consecutive keys (row = key) in one
    insert_and_evict call into an LRU table that grows from 2048 to its maximum of 4096 slots;
    what was evicted and what export_batch finds, window by window, is every key once with its row."""
    dim, n = 16, 4096 + 13
    t = HashTable()
    t.init(default_options(init_capacity=2048, max_capacity=4096, dim=dim, max_hbm_for_vectors=1 << 30,
                           num_of_buckets_per_alloc=16, evict_strategy=EvictStrategy.kLru))
    keys = np.arange(n, dtype=np.uint64)
    rows = np.repeat(keys.astype(np.float32)[:, None], dim, axis=1)
    ek = torch.zeros(n, dtype=torch.int64, device=DEV)
    ev = torch.zeros(n, dim, dtype=torch.float32, device=DEV)
    got = t.insert_and_evict(n, dev(keys), dev(rows), None, ek, ev, None)
    torch.cuda.synchronize()
    assert t.capacity() == 4096
    seen = {}
    gk, gv = host_u64(ek)[:got], ev.cpu().numpy()[:got]
    for k, r in zip(gk.tolist(), gv):
        assert k not in seen
        seen[k] = r
    window = t.capacity() >> 2
    dk = torch.zeros(window, dtype=torch.int64, device=DEV)
    dv = torch.zeros(window, dim, dtype=torch.float32, device=DEV)
    dc = torch.zeros(1, dtype=torch.int64, device=DEV)
    total = 0
    for off in range(0, t.capacity(), window):
        t.export_batch(window, off, dc, dk, dv, None)
        torch.cuda.synchronize()
        c = int(dc.item())
        total += c
        for k, r in zip(host_u64(dk)[:c].tolist(), dv.cpu().numpy()[:c]):
            assert k not in seen
            seen[k] = r
    assert total == t.size() and got + total == n
    assert sorted(seen) == list(range(n))
    assert all((r == np.float32(k)).all() for k, r in seen.items())
    t.close()


@pytest.mark.parametrize("row_bytes", [3, 66, 256, 520 * 4, 1025 * 4])
def test_every_row_moving_call_with_odd_and_long_rows(oracle, row_bytes):
    """Row sizes that take the 1-, 4- and 16-byte units and more than one pass of a tile: every call
    that moves rows (insert_or_assign, find_or_insert, insert_and_evict, assign, assign_values,
    find, export) against the oracle."""
    cap, bs = 1 << 12, 700
    t, o, _ = make_pair(oracle, init_capacity=cap, max_capacity=cap, dim=row_bytes, value_size=1,
                        value_kind=ValueKind.kBytes, evict_strategy=EvictStrategy.kCustomized)
    rng = np.random.Generator(np.random.PCG64(row_bytes))
    rows = lambda n: rng.integers(0, 256, size=(n, row_bytes), dtype=np.uint8)  # noqa: E731
    seq = 0
    for b in range(8):  # past capacity
        seq += 1
        k, v, sc = w.unique_keys(181, b * bs, bs), rows(bs), w.monotone_scores(seq, bs)
        t.insert_or_assign(bs, dev(k), dev(v), dev(sc))
        o.insert_or_assign(k, v, sc)
    assert_same_table(t, o, row_bytes)
    recent = w.unique_keys(181, 7 * bs, bs)
    # find_or_insert: residents hand their rows back
    io = rows(bs)
    d_io = dev(io)
    seq += 1
    sc = w.monotone_scores(seq, bs)
    t.find_or_insert(bs, dev(recent), d_io, dev(sc))
    oio = io.copy()
    o.find_or_insert(recent, oio, sc)
    torch.cuda.synchronize()
    assert np.array_equal(d_io.cpu().numpy(), oio) and not np.array_equal(oio, io)
    # find_or_insert: new keys store theirs
    fresh = w.unique_keys(182, 0, bs)
    io = rows(bs)
    d_io = dev(io)
    seq += 1
    sc = w.monotone_scores(seq, bs)
    t.find_or_insert(bs, dev(fresh), d_io, dev(sc))
    oio = io.copy()
    o.find_or_insert(fresh, oio, sc)
    torch.cuda.synchronize()
    assert np.array_equal(d_io.cpu().numpy(), oio)
    assert_same_table(t, o, row_bytes)
    # insert_and_evict: the evicted rows come out whole
    k2, v2 = w.unique_keys(183, 0, bs), rows(bs)
    seq += 1
    sc = w.monotone_scores(seq, bs)
    ek = torch.zeros(bs, dtype=torch.int64, device=DEV)
    ev = torch.zeros(bs, row_bytes, dtype=torch.uint8, device=DEV)
    es = torch.zeros(bs, dtype=torch.int64, device=DEV)
    c = t.insert_and_evict(bs, dev(k2), dev(v2), dev(sc), ek, ev, es)
    oek, oev, oes = o.insert_and_evict(k2, v2, sc)
    torch.cuda.synchronize()
    assert c == len(oek) and c > 0
    a, b = np.argsort(host_u64(ek)[:c], kind="stable"), np.argsort(oek, kind="stable")
    assert np.array_equal(host_u64(ek)[:c][a], oek[b])
    assert np.array_equal(ev.cpu().numpy()[:c][a], oev[b])
    assert np.array_equal(host_u64(es)[:c][a], oes[b])
    # assign and assign_values on a half-resident batch
    mixed = np.concatenate([k2[: bs // 2], w.unique_keys(184, 0, bs - bs // 2)])
    v3 = rows(bs)
    seq += 1
    sc = w.monotone_scores(seq, bs)
    t.assign(bs, dev(mixed), dev(v3), dev(sc))
    o.assign(mixed, v3, sc)
    v4 = rows(bs)
    t.assign_values(bs, dev(mixed), dev(v4))
    o.assign_values(mixed, v4)
    assert_same_table(t, o, row_bytes)
    # find and find* read what is there
    out = torch.zeros(bs, row_bytes, dtype=torch.uint8, device=DEV)
    founds = torch.zeros(bs, dtype=torch.bool, device=DEV)
    ptrs = torch.zeros(bs, dtype=torch.int64, device=DEV)
    f2 = torch.zeros(bs, dtype=torch.bool, device=DEV)
    t.find(bs, dev(mixed), out, founds, None)
    t.find_ptr(bs, dev(mixed), ptrs, f2, None)
    torch.cuda.synchronize()
    ov, of, _ = o.find(mixed)
    assert np.array_equal(founds.cpu().numpy(), of) and np.array_equal(f2.cpu().numpy(), of)
    assert np.array_equal(out.cpu().numpy()[of], ov[of])
    gp = ptrs.cpu().numpy()
    for i in np.flatnonzero(of)[:: 53]:
        assert np.array_equal(read_device(int(gp[i]), row_bytes), ov[i])
    t.close()


def test_one_digest_for_a_whole_bucket(oracle):
    """Every key of a bucket carries the same digest byte, so every probe sees 128 candidates,
    16 per lane of its tile: the candidate order (the lane of the key's start slot first), the
    second step, the second candidate of a lane and the loop over the rest are all taken, by
    readers and writers alike.  Two buckets, 300 such keys: fill, find (present and absent),
    find*, contains, erase and insert again, insert_and_evict, all against the oracle."""
    dim = 4
    t, o, _ = make_pair(oracle, init_capacity=256, max_capacity=256, dim=dim,
                        evict_strategy=EvictStrategy.kCustomized)
    cand = w.unique_keys(901, 0, 1 << 17)
    dig = np.array([oracle.locate(int(k), 2)[2] for k in cand[:1 << 17]], np.uint8)
    same = cand[dig == dig[0]][:300]
    assert len(same) == 300
    vals = w.values_from_keys(same, dim)
    sc = np.arange(1000, 1300, dtype=np.uint64)

    def check_lookups(q):
        n = len(q)
        out = torch.zeros(n, dim, dtype=torch.float32, device=DEV)
        f = torch.zeros(n, dtype=torch.bool, device=DEV)
        s = torch.zeros(n, dtype=torch.int64, device=DEV)
        t.find(n, dev(q), out, f, s)
        p = torch.zeros(n, dtype=torch.int64, device=DEV)
        f2 = torch.zeros(n, dtype=torch.bool, device=DEV)
        t.find_ptr(n, dev(q), p, f2)
        c = torch.zeros(n, dtype=torch.bool, device=DEV)
        t.contains(n, dev(q), c)
        torch.cuda.synchronize()
        ov, of, osc = o.find(q)
        gf = f.cpu().numpy()
        assert (gf == of).all() and (f2.cpu().numpy() == of).all() and (c.cpu().numpy() == of).all()
        assert (bytes_of(out.cpu().numpy())[of] == ov[of]).all()
        assert (host_u64(s)[of] == osc[of]).all()
        return int(of.sum())

    # 200 keys into 256 slots (free slots everywhere), then 100 more: the buckets fill up and evict
    t.insert_or_assign(200, dev(same[:200]), dev(vals[:200]), dev(sc[:200]))
    o.insert_or_assign(same[:200], bytes_of(vals[:200]), sc[:200])
    assert check_lookups(same) == 200
    assert_same_table(t, o, dim * 4)
    t.insert_or_assign(100, dev(same[200:]), dev(vals[200:]), dev(sc[200:]))
    o.insert_or_assign(same[200:], bytes_of(vals[200:]), sc[200:])
    assert t.size() == o.size() == 256
    assert check_lookups(same) == 256
    assert_same_table(t, o, dim * 4)
    # erase every third resident key, look again, put some back with new rows
    gone = np.ascontiguousarray(same[44::3][:60])
    t.erase(len(gone), dev(gone))
    o.erase(gone)
    assert t.size() == o.size()
    check_lookups(same)
    back = np.concatenate([gone[:30], same[:10]])
    bv = w.uniform_values(902, 0, len(back), dim)
    bs_ = np.arange(2000, 2000 + len(back), dtype=np.uint64)
    t.insert_or_assign(len(back), dev(back), dev(bv), dev(bs_))
    o.insert_or_assign(back, bytes_of(bv), bs_)
    check_lookups(same)
    assert_same_table(t, o, dim * 4)
    # assign on present and absent keys of the same digest
    av = w.uniform_values(903, 0, 300, dim)
    as_ = np.arange(3000, 3300, dtype=np.uint64)
    t.assign(300, dev(same), dev(av), dev(as_))
    o.assign(same, bytes_of(av), as_)
    assert_same_table(t, o, dim * 4)
    t.close()


@pytest.mark.parametrize("bounds", ["on", "off"])
def test_accum_flags_that_disagree_in_nearly_full_buckets(oracle, monkeypatch, bounds):
    """accum_or_assign with some thirty new keys per bucket and a handful of free slots in each:
    half of the new keys are flagged "accumulate" and so change nothing, the other half share
    the free slots and then evict.  A key whose flag disagrees with its presence takes no slot,
    not even for a moment: a slot that is taken and handed back looks taken to the bucket's other
    new keys, which then search a victim in a bucket that is not full (and, with the handed-back
    slot still holding score 0, find that very slot over and over).  With the bounded search
    and with the full scan, against the oracle."""
    if bounds == "off":
        monkeypatch.setenv("HKV_SCORE_BOUNDS", "0")
    cap, dim = 1 << 12, 4  # 32 buckets
    t, o, _ = make_pair(oracle, init_capacity=cap, max_capacity=cap, dim=dim)
    t.set_clock(1, 1 << 44)
    o.set_clock(1, 1 << 44)
    vb = dim * 4
    rng = np.random.default_rng(91)
    fill(t, o, 91, 3, 1000, dim)  # old keys: the victims
    pos = 3000
    for rep in range(4):
        # the latest keys (highest scores: no eviction of this repetition reaches them)
        recent = w.unique_keys(91, pos, 800)
        rv = w.uniform_values(91, pos, 800, dim)
        t.insert_or_assign(800, dev(recent), dev(rv))
        o.insert_or_assign(recent, bytes_of(rv), None)
        pos += 800
        if rep:  # free slots again: some of the oldest keys leave
            gone = w.unique_keys(91, (rep - 1) * 700, 300)
            t.erase(300, dev(gone))
            o.erase(gone)
        assert_same_table(t, o, vb)
        keys = np.concatenate([recent[:450], w.unique_keys(91, pos, 1050)])
        pos += 1050
        keys = keys[rng.permutation(len(keys))]
        n = len(keys)
        deltas = w.uniform_values(92 + rep, 0, n, dim)
        flags = rng.random(n) < 0.5
        t.accum_or_assign(n, dev(keys), dev(deltas), dev(flags.astype(np.uint8)))
        o.accum_or_assign(keys, bytes_of(deltas), flags.astype(np.uint8))
        assert t.size() == o.size()
        assert_same_table(t, o, vb)
    t.close()
