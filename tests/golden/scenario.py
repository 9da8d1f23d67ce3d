"""The call sequence behind tests/golden/scenario_customized.npz, written once against an
abstract `Driver` so that the fixture generator (host oracle), the CPU regression test and
the GPU parity test all run the very same calls.

Table: capacity 2048 (16 buckets), dim 2 fp32, Customized scores, pure HBM.  The sequence
goes past load factor 1.0, so evictions, refusals, tombstones and their reuse all occur.
Inputs are stored in the fixture itself (no generator needs to be trusted when reading it).
"""
import numpy as np

CAPACITY, DIM, BATCH = 2048, 2, 512
M64 = (1 << 64) - 1


def make_inputs():
    """Seeded inputs (numpy PCG64): distinct keys per batch, distinct scores overall."""
    rng = np.random.Generator(np.random.PCG64(0x484B56))
    pool = rng.choice(1 << 40, size=8 * BATCH, replace=False).astype(np.uint64) * np.uint64(2654435761) + np.uint64(17)
    pool = pool[(pool & np.uint64(M64 - 3)) != np.uint64(M64 - 3)]
    assert len(np.unique(pool)) == len(pool)
    inp = {}
    for b in range(5):  # fill past load factor 1.0
        inp[f"fill{b}_keys"] = pool[b * BATCH:(b + 1) * BATCH].copy()
        inp[f"fill{b}_vals"] = rng.uniform(-1, 1, (BATCH, DIM)).astype(np.float32)
        inp[f"fill{b}_scores"] = (np.uint64(b + 1) << np.uint64(24)) + rng.permutation(BATCH).astype(np.uint64)
    # find: 256 keys of the last batches + 256 never inserted + the reserved keys
    inp["find_keys"] = np.concatenate([pool[4 * BATCH:4 * BATCH + 256], pool[6 * BATCH:6 * BATCH + 256],
                                       np.array([M64, M64 - 1, M64 - 2, M64 - 3], np.uint64)])
    # insert_and_evict: 256 resident keys of the newest batch (never a bucket's minimum) with
    # raised scores, 256 new keys whose scores straddle the resident range, so that some evict
    # and some are refused.  With these choices the outcome does not depend on the order in
    # which the keys of the batch are handled (a bucket keeps its 128 highest scores).
    inp["evict_keys"] = np.concatenate([pool[4 * BATCH:4 * BATCH + 256], pool[5 * BATCH:5 * BATCH + 256]])
    inp["evict_vals"] = rng.uniform(-1, 1, (BATCH, DIM)).astype(np.float32)
    inp["evict_scores"] = np.concatenate([
        (np.uint64(6) << np.uint64(24)) + rng.permutation(256).astype(np.uint64),
        (np.uint64(1) << np.uint64(24)) + np.uint64(1000) + rng.permutation(1 << 20)[:256].astype(np.uint64) * np.uint64(61)])
    inp["erase_keys"] = np.concatenate([pool[4 * BATCH + 100:4 * BATCH + 228], pool[7 * BATCH:7 * BATCH + 32]])
    # accum_or_assign: flags partly right, partly wrong (accum_or_assign.cuh:139-156)
    inp["accum_keys"] = np.concatenate([pool[4 * BATCH + 300:4 * BATCH + 428], pool[7 * BATCH + 64:7 * BATCH + 192]])
    inp["accum_vals"] = rng.uniform(-1, 1, (256, DIM)).astype(np.float32)
    inp["accum_flags"] = (rng.integers(0, 4, 256) != 0) ^ (np.arange(256) >= 128)
    inp["accum_scores"] = (np.uint64(9) << np.uint64(24)) + rng.permutation(256).astype(np.uint64)
    # tombstones are reused: a last insert of new keys
    inp["last_keys"] = pool[7 * BATCH + 200:7 * BATCH + 456].copy()
    inp["last_vals"] = rng.uniform(-1, 1, (256, DIM)).astype(np.float32)
    inp["last_scores"] = (np.uint64(10) << np.uint64(24)) + rng.permutation(256).astype(np.uint64)
    return inp


def run(driver, inp):
    """driver: insert_or_assign(keys, vals, scores), find(keys) -> (value bytes, founds, scores),
    insert_and_evict(keys, vals, scores) -> (keys, value bytes, scores) of the evicted entries,
    erase(keys), accum_or_assign(keys, vals, flags, scores), size(), export_all() ->
    (keys, value bytes, scores).  Returns the observable outputs, canonically ordered."""
    out = {}
    for b in range(5):
        driver.insert_or_assign(inp[f"fill{b}_keys"], inp[f"fill{b}_vals"], inp[f"fill{b}_scores"])
        out[f"size_after_fill{b}"] = np.array([driver.size()], np.uint64)
    v, f, s = driver.find(inp["find_keys"])
    out["find_founds"] = np.asarray(f, bool)
    out["find_vals"] = np.where(out["find_founds"][:, None], v, 0).astype(np.uint8)
    out["find_scores"] = np.where(out["find_founds"], s, 0).astype(np.uint64)
    ek, ev, es = driver.insert_and_evict(inp["evict_keys"], inp["evict_vals"], inp["evict_scores"])
    o = np.argsort(ek, kind="stable")
    out["evicted_keys"], out["evicted_vals"], out["evicted_scores"] = ek[o], ev[o], es[o]
    out["size_after_evict"] = np.array([driver.size()], np.uint64)
    driver.erase(inp["erase_keys"])
    out["size_after_erase"] = np.array([driver.size()], np.uint64)
    driver.accum_or_assign(inp["accum_keys"], inp["accum_vals"], inp["accum_flags"], inp["accum_scores"])
    driver.insert_or_assign(inp["last_keys"], inp["last_vals"], inp["last_scores"])
    k, v, s = driver.export_all()
    o = np.argsort(k, kind="stable")
    out["table_keys"], out["table_vals"], out["table_scores"] = k[o], v[o], s[o]
    out["size_final"] = np.array([driver.size()], np.uint64)
    return out
