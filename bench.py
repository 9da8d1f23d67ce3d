#!/usr/bin/env python
"""Benchmark of the hot path on one MI355X.

Workload (the shape the headline metric is quoted on): capacity 2^26 keys, uint64 keys, fp32
values dim 64 (16 GiB of value rows, all in HBM), uint64 scores, LRU, batch
2^20, table pre-filled to load factor 1.0.  One step = find on 2^20 resident
keys (100 % hits) followed by insert_or_assign of 2^20 keys, half resident and
half new (every new key evicts the bucket's minimum).  Inputs and outputs are
resident in HBM when the timed region starts.

The resident keys of a step come from old pre-fill batches, a different batch
per step, so their rows are neither in the L2s nor in the 256 MB Infinity Cache
when the step touches them (--warm-keys takes them from the previous step's
insert instead, as the reference's benchmark does).

Prints one JSON line: whole-step throughput in 10^9 KV/s, per-op figures, the
HBM roofline of each kernel from HIP-event timings inside the timed region, and
a CPU baseline (the multithreaded host oracle on a bounded sample).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0
# algorithmic bytes per key (minimum traffic the mandated layout implies):
#   find hit   = 8 key + 128 digest line + 8 key verify + VB read + VB write + 1 found
#   upsert hit = 8 + 128 + 8 lock + VB in + VB out + 8 score + 1 digest + 8 unlock
#   upsert miss in a full bucket = upsert hit + 1024 (score scan)
def find_bytes(vb):
    return 145 + 2 * vb


def upsert_bytes(vb, new_fraction):
    return (1.0 - new_fraction) * (161 + 2 * vb) + new_fraction * (1185 + 2 * vb)


# HBM bytes per launch on the default workload come from rocprofv3 --pmc FETCH_SIZE and
# --pmc WRITE_SIZE runs of this very command (KiB per dispatch, each scaled by what the same
# counter reads for a 1 GiB device-to-device copy in the same run).  Counters cannot be read
# from inside this process, so `--profile-summary` writes them to a file beside the profile
# summaries and the default run reports what that file holds; it applies to the default
# workload only.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic_cap2p26_dim64_batch2p20.json")


class HipEvent:
    """A HIP event for timing only, created with hipEventDisableSystemFence: recording it does not
    write the caches back and invalidate them, as the events torch creates do, so the kernel after
    it starts as it would with no event there (hip_runtime_api.h says as much of the flag).  The
    timed region ends with a device synchronisation, after which the time stamps are read.
    Two uses: record() puts the event on the stream between two calls; a pair handed to the
    library (hkv_time_next_kernel) is attached to one kernel launch and gets the start and the end
    of that kernel's execution, which is what a profiler's trace reports for it."""
    _hip = None

    def __init__(self, torch):
        import ctypes as C
        if HipEvent._hip is None:
            HipEvent._hip = C.CDLL("libamdhip64.so")
            HipEvent._hip.hipEventCreateWithFlags.argtypes = [C.POINTER(C.c_void_p), C.c_uint]
            HipEvent._hip.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
            HipEvent._hip.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
            HipEvent._hip.hipEventDestroy.argtypes = [C.c_void_p]
        self._C = C
        self._torch = torch
        self._e = C.c_void_p()
        rc = HipEvent._hip.hipEventCreateWithFlags(C.byref(self._e), 0x20000000)  # hipEventDisableSystemFence
        if rc:
            raise RuntimeError("hipEventCreateWithFlags: %d" % rc)

    @property
    def handle(self):
        return self._e

    def record(self):
        rc = HipEvent._hip.hipEventRecord(self._e, self._C.c_void_p(self._torch.cuda.current_stream().cuda_stream))
        if rc:
            raise RuntimeError("hipEventRecord: %d" % rc)

    def elapsed_time(self, later):
        ms = self._C.c_float()
        rc = HipEvent._hip.hipEventElapsedTime(self._C.byref(ms), self._e, later._e)
        if rc:
            raise RuntimeError("hipEventElapsedTime: %d" % rc)
        return ms.value

    def __del__(self):
        try:
            if self._e:
                HipEvent._hip.hipEventDestroy(self._e)
                self._e = None
        except Exception:  # interpreter shutdown: the library may be gone already
            pass


def measured_traffic(kernel):
    try:
        with open(TRAFFIC_FILE) as f:
            return json.load(f)["kernels"][kernel]["traffic_bytes"]
    except (OSError, KeyError, ValueError):
        return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--capacity-log2", type=int, default=26)
    ap.add_argument("--dim", type=int, default=64)
    ap.add_argument("--batch-log2", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--strategy", choices=["lru", "customized", "epochlru"], default="lru",
                    help="eviction strategy of the table (the headline workload is LRU; customized: scores "
                         "(call number << 40) | index from the caller, epochlru: one epoch)")
    ap.add_argument("--kernel-events", action="store_true",
                    help="time each kernel by an event pair it is launched with (hkv_time_next_kernel: start and "
                         "end of its execution, what a profiler's trace reports) instead of by events recorded "
                         "on the stream between the calls; launches made that way cost the step about 8 us")
    ap.add_argument("--warm-keys", action="store_true",
                    help="resident keys of a step = keys written by the previous step")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run one plain 1 GiB device copy (reference point for "
                         "FETCH_SIZE / WRITE_SIZE when profiling)")
    ap.add_argument("--cpu-capacity-log2", type=int, default=26,
                    help="capacity of the host oracle's table for the CPU baseline (the benchmark's own 2^26 by "
                         "default: 17 GiB of host memory)")
    ap.add_argument("--matrix", action="store_true",
                    help="instead of the one-line benchmark: the reference's own benchmark table "
                         "(README.md:245-317, benchmark/merlin_hashtable_benchmark.cc.cu), every API "
                         "at load factor 0.50 / 0.75 / 1.00 for dim 8, 32 and 64, printed as markdown")
    ap.add_argument("--ops", action="store_true",
                    help="instead of the one-line benchmark: every entry point at the metric shape "
                         "(capacity 2^26, dim 64, batch 2^20, load factor 1.0), kernel time by HIP "
                         "events and algorithmic GB/s against the 8 TB/s peak, printed as markdown")
    ap.add_argument("--config", type=int, choices=[2, 3, 4, 5], default=0,
                    help="instead of the one-line benchmark: the measurement protocol of one of the other "
                         "workload configurations at its full size (2: dim 8 at load factor 0.50 / 0.75 / 1.00; "
                         "3: Zipf insert_and_evict + find at 2^27, dim 64; 4: hybrid HBM + pinned host rows at "
                         "2^28 with HBM and host-link GB/s apart; 5: accum_or_assign / export_batch_if / erase "
                         "at 2^25, dim 128); a markdown table and one JSON line")
    ap.add_argument("--load-factor", type=float, default=0.0,
                    help="with --config 2: only this load factor (0.5, 0.75 or 1.0) instead of all three in turn, so "
                         "that a profiler's last dispatches of each kernel are the timed calls at that load factor")
    ap.add_argument("--group-lock", action="store_true",
                    help="instead of the one-line benchmark: what the API-level group lock costs the host per call, "
                         "as built (stream events, never blocks) against a host-blocking acquisition as the "
                         "reference does it (a one-thread kernel on a side stream plus a stream synchronisation)")
    ap.add_argument("--profile-summary", metavar="DIR", default=None,
                    help="no GPU needed: condense rocprofv3 output (DIR/<bench|ops>_<trace|fetch|write|l2|rd|wr|sq|tcp>/"
                         "out_*.csv, made by the commands the summaries list) into profiles/*.md and "
                         "profiles/traffic_cap2p26_dim64_batch2p20.json, which the default run reports as "
                         "roofline.traffic")
    ap.add_argument("--ceilings", action="store_true",
                    help="instead of the one-line benchmark: what the memory system needs for the access "
                         "patterns of find and insert_or_assign at the same shape with no table logic "
                         "(hierarchicalkv_amd/csrc/hkv_ceilings.hip), and the streaming / gather / scatter / "
                         "small-access rates they are made of; one JSON line and a markdown table")
    ap.add_argument("--matrix-hybrid", action="store_true",
                    help="with --matrix: the hybrid table of README.md:289-303 (dim 64, capacity "
                         "128M, 16 GB of the rows in HBM, the rest in pinned host memory)")
    args = ap.parse_args()
    if args.profile_summary:
        summarize_profiles(args.profile_summary)
        return
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path "
              "(one table per device, as in the reference); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import workloads as w
    from hierarchicalkv_amd import EvictStrategy, HashTable, default_options

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    if args.matrix:
        run_matrix(args, np, torch, dev)
        return
    if args.ops:
        run_ops(args, np, torch, dev, w)
        return
    if args.ceilings:
        run_ceilings(args)
        return
    if args.config:
        run_config(args, torch)
        return
    if args.group_lock:
        run_group_lock(torch)
        return
    cap = 1 << args.capacity_log2
    dim = args.dim
    n = 1 << args.batch_log2
    vb = dim * 4
    seed = 0x484B5600
    K, W = args.steps, args.warmup

    strategy = {"lru": EvictStrategy.kLru, "customized": EvictStrategy.kCustomized,
                "epochlru": EvictStrategy.kEpochLru}[args.strategy]
    opts = default_options(init_capacity=cap, max_capacity=cap, max_hbm_for_vectors=cap * vb,
                           dim=dim, evict_strategy=strategy)
    table = HashTable()
    table.init(opts)
    assert table.is_pure_hbm()
    if args.strategy == "epochlru":
        table.set_global_epoch(1)
    call_no = [0]
    index = torch.arange(n, dtype=torch.int64, device=dev)

    def next_scores():
        """Customized: distinct scores that grow from call to call, made on the device."""
        if args.strategy != "customized":
            return None
        call_no[0] += 1
        return index + (call_no[0] << 40)

    def d64(a):
        return torch.from_numpy(a.view(np.int64)).to(dev)

    # ---- prefill to load factor 1.0 (untimed) ------------------------------------
    t0 = time.time()
    pos = 0
    vals = torch.empty(n, dim, dtype=torch.float32, device=dev)
    size0 = 0
    prefill_starts = []
    # uniform hashing fills the last slots slowly: keep inserting (the fullest
    # buckets evict meanwhile) until 99.9 % of the slots hold a key
    while size0 < 0.999 * cap and pos < 3 * cap:
        for _ in range(max(1, (cap // n) // 8)):
            keys = w.unique_keys(seed, pos, n)
            vals.uniform_(-1.0, 1.0)
            table.insert_or_assign(n, d64(keys), vals, next_scores())
            prefill_starts.append(pos)
            pos += n
        size0 = table.size()
    prefill_s = time.time() - t0

    # ---- per-step inputs, resident in HBM ------------------------------------------
    # step s: find the keys inserted by step s-1 (all resident, highest LRU scores);
    #         insert_or_assign half of those again + as many never-seen keys.
    steps = K + W
    nb = len(prefill_starts)
    find_keys, ins_keys = [], []
    if args.warm_keys:
        # step s: find the keys inserted by step s-1; insert half of them again
        prev = w.unique_keys(seed, pos - n, n)
        for s in range(steps):
            find_keys.append(d64(prev))
            fresh = w.unique_keys(seed, pos, n // 2)
            pos += n // 2
            batch = np.concatenate([prev[: n // 2], fresh])
            ins_keys.append(d64(batch))
            prev = batch
    else:
        # A bucket holds the newest 128 of the ~2 keys per batch it received, i.e.
        # the last ~64 pre-fill batches, and loses about one key per step.  Batches
        # 9..(9+steps) from the end serve find, half batches further back serve the
        # resident half of insert_or_assign; all stay resident for the whole run.
        assert steps <= 26 and nb >= 9 + steps + (steps + 1) // 2 + 2, "too many steps for cold keys"
        for s in range(steps):
            find_keys.append(d64(w.unique_keys(seed, prefill_starts[nb - 9 - s], n)))
            old = w.unique_keys(seed, prefill_starts[nb - 10 - steps - s // 2], n)
            half = old[: n // 2] if s % 2 == 0 else old[n // 2:]
            fresh = w.unique_keys(seed, pos, n // 2)
            pos += n // 2
            ins_keys.append(d64(np.concatenate([half, fresh])))
    ins_vals = torch.empty(n, dim, dtype=torch.float32, device=dev).uniform_(-1.0, 1.0)
    out_vals = torch.empty(n, dim, dtype=torch.float32, device=dev)
    founds = torch.empty(n, dtype=torch.bool, device=dev)

    # The calls of a step are timed by events recorded on the stream between them (one after each
    # call; the one after a step's insert_or_assign is the one before the next step's find), so
    # each figure holds one gap between launches, 2 to 3 us.  With --kernel-events every kernel
    # is launched with an event pair of its own instead (hkv_time_next_kernel): the runtime stamps
    # it with the start and the end of the kernel's execution, which is what rocprofv3's trace
    # reports, but launches made that way cost the step about 8 us of wall time.
    from hierarchicalkv_amd._capi import lib as hkv_lib
    ev_find = [(HipEvent(torch), HipEvent(torch)) for _ in range(steps)]
    ev_ins = [(HipEvent(torch), HipEvent(torch)) for _ in range(steps)]
    ev_edge = [HipEvent(torch) for _ in range(steps + 1)]
    ev_mid = [HipEvent(torch) for _ in range(steps)]

    step_scores = [next_scores() for _ in range(steps)]

    def step(s):
        if (not args.kernel_events):
            table.find(n, find_keys[s], out_vals, founds)
            ev_mid[s].record()
            table.insert_or_assign(n, ins_keys[s], ins_vals, step_scores[s])
            ev_edge[s + 1].record()
            return
        hkv_lib.hkv_time_next_kernel(ev_find[s][0].handle, ev_find[s][1].handle)
        table.find(n, find_keys[s], out_vals, founds)
        hkv_lib.hkv_time_next_kernel(ev_ins[s][0].handle, ev_ins[s][1].handle)
        table.insert_or_assign(n, ins_keys[s], ins_vals, step_scores[s])

    if args.calibrate:
        cal = torch.empty(2, 1 << 28, dtype=torch.float32, device=dev)
        cal[0].fill_(1.0)
        torch.cuda.synchronize()
        cal[1].copy_(cal[0])  # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del cal
    ev_edge[0].record()
    for s in range(W):
        step(s)
    torch.cuda.synchronize()
    hit_rate = float(founds.float().mean().item())
    t_start = time.perf_counter()
    ev_edge[W].record()
    for s in range(W, steps):
        step(s)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t_start

    if (not args.kernel_events):
        find_ms = [ev_edge[s].elapsed_time(ev_mid[s]) for s in range(W, steps)]
        ups_ms = [ev_mid[s].elapsed_time(ev_edge[s + 1]) for s in range(W, steps)]
    else:
        find_ms = [ev_find[s][0].elapsed_time(ev_find[s][1]) for s in range(W, steps)]
        ups_ms = [ev_ins[s][0].elapsed_time(ev_ins[s][1]) for s in range(W, steps)]
    find_avg = sum(find_ms) / K
    ups_avg = sum(ups_ms) / K
    size1 = table.size()

    value = 2.0 * n * K / wall / 1e9
    fb = find_bytes(vb) * n
    ub = upsert_bytes(vb, 0.5) * n
    find_gbs = fb / (find_avg * 1e-3) / 1e9
    ups_gbs = ub / (ups_avg * 1e-3) / 1e9

    default_workload = (args.capacity_log2 == 26 and dim == 64 and args.batch_log2 == 20
                        and not args.warm_keys and args.strategy == "lru")
    ups_traffic = measured_traffic("upsert_kernel") if default_workload else None
    find_traffic = measured_traffic("lookup_kernel") if default_workload else None
    timed_by = ("events on the stream around each call" if (not args.kernel_events) else
                "the event pair each kernel is launched with (start and end of its execution)")

    def traffic_frac(traffic, ms):
        return None if traffic is None else round(traffic / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)

    result = {
        "metric": "billion-KV/s for find & insert_or_assign, dim 64, load factor 1.0, 1 GPU",
        "value": round(value, 4),
        "unit": "billion-KV/s (10^9 keys/s, find + insert_or_assign per step)",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": round(wall / K * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u64 keys/scores, fp32 values copied as bytes",
        "data": "synthetic",
        "config": {
            "workload": f"capacity 2^{args.capacity_log2}, dim {dim} fp32, batch 2^{args.batch_log2}, "
                        f"{args.strategy.upper() if args.strategy == 'lru' else args.strategy}, load factor 1.0; "
                        "step = find (100% hit) + insert_or_assign (50% new)",
            "load_factor": round(size0 / cap, 4),
            "find_hit_rate": round(hit_rate, 4),
            "size_before": size0,
            "size_after": size1,
            "prefill_s": round(prefill_s, 1),
            "resident_keys": "warm (previous step)" if args.warm_keys else "cold (old pre-fill batches)",
        },
        "find": {"ms": round(find_avg, 4), "bkvs": round(n / (find_avg * 1e-3) / 1e9, 4),
                 "bkvs_2p30": round(n / (find_avg * 1e-3) / 2**30, 4)},
        "insert_or_assign": {"ms": round(ups_avg, 4), "bkvs": round(n / (ups_avg * 1e-3) / 1e9, 4),
                             "bkvs_2p30": round(n / (ups_avg * 1e-3) / 2**30, 4)},
        # frac: algorithmic bytes / kernel time / peak; traffic_frac: the bytes the counters saw
        # moving (FETCH_SIZE + WRITE_SIZE of the same workload, profiles/) / kernel time / peak.
        # The bounded victim search moves fewer bytes than the algorithmic figure bills (it reads
        # one or two of a bucket's eight score lines), find moves more (whole 128-byte lines for
        # 8-byte key verifications).
        "roofline": {"kernel": "upsert_kernel<insert_or_assign>", "bound": "hbm",
                     "achieved": round(ups_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(ups_gbs / HBM_PEAK_GBS, 4), "traffic": ups_traffic,
                     "traffic_frac": traffic_frac(ups_traffic, ups_avg),
                     "bytes_per_key": upsert_bytes(vb, 0.5), "timed_by": timed_by},
        "roofline_find": {"kernel": "lookup_kernel<values>", "bound": "hbm",
                          "achieved": round(find_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": round(find_gbs / HBM_PEAK_GBS, 4), "traffic": find_traffic,
                          "traffic_frac": traffic_frac(find_traffic, find_avg),
                          "bytes_per_key": find_bytes(vb), "timed_by": timed_by},
    }
    table.close()
    del find_keys, ins_keys, ins_vals, out_vals
    torch.cuda.empty_cache()

    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(args, np, w)
    print(json.dumps(result))


def run_matrix(args, np, torch, dev):
    """The reference's benchmark protocol (benchmark/merlin_hashtable_benchmark.cc.cu:75-420):
    LRU table, consecutive integer keys up to the load factor, then ONE timed call of 2^20 keys
    per API, 60 % of them from the last inserted batch and 40 % never seen
    (benchmark_util.cuh:135-177), wall clock from the call to the end of the stream, best of two,
    in units of 2^30 KV/s.  One table per (dim, load factor) serves all APIs here, read-only ones
    first (the reference builds a fresh table per API; an insert of 0.4 M new keys moves the load
    factor of a 64 M table by 0.6 %)."""
    from hierarchicalkv_amd import EvictStrategy, HashTable, default_options, Predicate

    n = 1 << 20
    M = 1 << 20
    if args.matrix_hybrid:
        configs = [(64, 128 * M, 16 << 30)]
    else:
        configs = [(8, 128 * M, 4 << 30), (32, 128 * M, 16 << 30), (64, 64 * M, 16 << 30)]
    apis = ["insert_or_assign", "find", "find_or_insert", "assign", "find*", "find_or_insert*",
            "insert_and_evict", "export_batch", "export_batch_if", "contains"]
    order = ["find", "find*", "contains", "export_batch", "export_batch_if", "assign",
             "find_or_insert", "find_or_insert*", "insert_or_assign", "insert_and_evict"]
    if args.matrix_hybrid:
        # insert_and_evict needs a pure-HBM table, as in the reference (merlin_hashtable.cuh:1373-1375)
        apis.remove("insert_and_evict")
        order.remove("insert_and_evict")

    def d64(a):
        return torch.from_numpy(a.view(np.int64)).to(dev)

    print("| dim | capacity | HBM for rows | load factor | " + " | ".join(apis) + " |")
    print("|---|---|---|---|" + "---|" * len(apis))
    for dim, cap, hbm in configs:
        for lf in (0.50, 0.75, 1.00):
            table = HashTable()
            table.init(default_options(init_capacity=cap, max_capacity=cap, max_hbm_for_vectors=hbm,
                                       dim=dim, evict_strategy=EvictStrategy.kLru))
            vals = torch.ones(n, dim, dtype=torch.float32, device=dev)
            defv = torch.full((n, dim), 2.0, dtype=torch.float32, device=dev)
            ptrs = torch.zeros(n, dtype=torch.int64, device=dev)
            founds = torch.zeros(n, dtype=torch.bool, device=dev)
            scores = torch.zeros(n, dtype=torch.int64, device=dev)
            ek = torch.zeros(n, dtype=torch.int64, device=dev)
            es = torch.zeros(n, dtype=torch.int64, device=dev)
            cnt = torch.zeros(1, dtype=torch.int64, device=dev)
            # step 1 and 2 of the reference: consecutive keys, then top up to the load factor
            start = 0
            target = int(cap * lf)
            while start < target:
                m = min(n, target - start)
                table.insert_or_assign(m, d64(np.arange(start, start + m, dtype=np.uint64)), vals)
                start += m
            while True:
                short = target - table.size()
                if short <= cap * 1e-3 or start > 3 * cap:
                    break
                m = min(n, short)
                table.insert_or_assign(m, d64(np.arange(start, start + m, dtype=np.uint64)), vals)
                start += m
            threshold = 0  # the reference's threshold is the device clock before the prefill: keeps all
            res = {}
            fresh = (1 << 64) - 5  # never-seen keys count down from the top, below the reserved ones
            for api in order:
                best = float("inf")
                for rep in range(2):
                    hit = np.arange(start - n, start - n + int(n * 0.6), dtype=np.uint64)
                    m_new = n - len(hit)
                    new = np.arange(fresh - m_new + 1, fresh + 1, dtype=np.uint64)[::-1]
                    fresh -= m_new
                    keys = d64(np.concatenate([hit, new]))
                    cnt.zero_()
                    torch.cuda.synchronize()
                    t0 = time.perf_counter()
                    if api == "find":
                        table.find(n, keys, vals, founds)  # LRU: no scores asked for (:108)
                    elif api == "find*":
                        table.find_ptr(n, keys, ptrs, founds)
                    elif api == "contains":
                        table.contains(n, keys, founds)
                    elif api == "export_batch":
                        table.export_batch(int(n / lf * 0.995), 0, cnt, keys, vals)
                    elif api == "export_batch_if":
                        table.export_batch_if(Predicate.kScoreGt, 0, threshold, int(n / lf * 0.995), 0,
                                              cnt, keys, vals)
                    elif api == "assign":
                        table.assign(n, keys, defv)
                    elif api == "find_or_insert":
                        table.find_or_insert(n, keys, vals)
                    elif api == "find_or_insert*":
                        table.find_or_insert_ptr(n, keys, ptrs, founds)
                    elif api == "insert_or_assign":
                        table.insert_or_assign(n, keys, vals)
                    elif api == "insert_and_evict":
                        table.insert_and_evict(n, keys, vals, None, ek, defv, es, cnt)
                    torch.cuda.synchronize()
                    best = min(best, time.perf_counter() - t0)
                res[api] = n / best / float(1 << 30)
            print("| %d | %dM | %d GB | %.2f | " % (dim, cap // M, hbm >> 30, table.size() / cap)
                  + " | ".join("%.3f" % res[a] for a in apis) + " |", flush=True)
            table.close()
            del table, vals, defv
            torch.cuda.empty_cache()


def run_ops(args, np, torch, dev, w):
    """Every entry point at the metric shape, one row each: average HIP-event time of 6 calls
    after 2 warm-up calls, 10^9 KV/s, algorithmic bytes per key and their rate against the
    8 TB/s peak.  Bytes per key, VB = 256: find hit 145 + 2 VB; find* hit 153; contains hit 145;
    upsert hit 161 + 2 VB, upsert into a full bucket 1185 + 2 VB; find_or_insert hit 169 + 2 VB;
    insert_and_evict evicting 1201 + 4 VB; accum hit 161 + 3 VB; assign hit 161 + 2 VB;
    export 16 per scanned slot + (2 VB + 16) per match; erase hit 165."""
    from hierarchicalkv_amd import EvictStrategy, HashTable, default_options, Predicate

    cap, dim, n = 1 << args.capacity_log2, args.dim, 1 << args.batch_log2
    vb = dim * 4
    seed = 0x484B5600
    table = HashTable()
    table.init(default_options(init_capacity=cap, max_capacity=cap, max_hbm_for_vectors=cap * vb,
                               dim=dim, evict_strategy=EvictStrategy.kLru))

    def d64(a):
        return torch.from_numpy(a.view(np.int64)).to(dev)

    vals = torch.empty(n, dim, dtype=torch.float32, device=dev).uniform_(-1.0, 1.0)
    pos, starts, size = 0, [], 0
    while size < 0.999 * cap and pos < 3 * cap:
        for _ in range(max(1, (cap // n) // 8)):
            table.insert_or_assign(n, d64(w.unique_keys(seed, pos, n)), vals)
            starts.append(pos)
            pos += n
        size = table.size()
    nb = len(starts)
    out = torch.empty(n, dim, dtype=torch.float32, device=dev)
    ev_vals = torch.empty(n, dim, dtype=torch.float32, device=dev)
    founds = torch.empty(n, dtype=torch.bool, device=dev)
    flags = torch.empty(n, dtype=torch.bool, device=dev)
    ptrs = torch.zeros(n, dtype=torch.int64, device=dev)
    ek = torch.zeros(n, dtype=torch.int64, device=dev)
    es = torch.zeros(n, dtype=torch.int64, device=dev)
    cnt = torch.zeros(1, dtype=torch.int64, device=dev)
    state = {"old": 0, "pos": pos}

    def resident():
        # an old pre-fill batch that is still resident and cold in the caches: the batches 8 to 31
        # from the end take turns (the table holds the newest ~64, and every upsert row below
        # pushes out half a batch)
        state["old"] += 1
        return w.unique_keys(seed, starts[nb - 8 - state["old"] % 24], n)

    def mixed(new_fraction=0.5):
        m = int(n * new_fraction)
        fresh = w.unique_keys(seed, state["pos"], m)
        state["pos"] += m
        return np.concatenate([resident()[: n - m], fresh])

    hit, full = 161 + 2 * vb, 1185 + 2 * vb
    rows = [
        ("find (100 % hit)", lambda k: table.find(n, k, out, founds), resident, 145 + 2 * vb),
        ("find* (100 % hit)", lambda k: table.find_ptr(n, k, ptrs, founds), resident, 153),
        ("contains (100 % hit)", lambda k: table.contains(n, k, founds), resident, 145),
        ("assign (100 % hit)", lambda k: table.assign(n, k, vals), resident, hit),
        ("insert_or_assign (50 % new)", lambda k: table.insert_or_assign(n, k, vals), mixed,
         0.5 * hit + 0.5 * full),
        ("find_or_insert (50 % new)", lambda k: table.find_or_insert(n, k, out), mixed,
         0.5 * (169 + 2 * vb) + 0.5 * full),
        ("find_or_insert* (50 % new)", lambda k: table.find_or_insert_ptr(n, k, ptrs, founds), mixed,
         0.5 * 177 + 0.5 * (1185 + 16)),
        ("insert_and_evict (50 % new)",
         lambda k: (cnt.zero_(), table.insert_and_evict(n, k, vals, None, ek, ev_vals, es, cnt)), mixed,
         0.5 * hit + 0.5 * (1201 + 4 * vb)),
        ("accum_or_assign (50 % new, flags from find)", None, mixed, 0.5 * (161 + 3 * vb) + 0.5 * (full + 1)),
        ("export_batch_if (2^20 slots, all match)",
         lambda k: table.export_batch_if(Predicate.kAlways, 0, 0, n, (state["old"] % 32) * n, cnt, ek, out, es),
         resident, 16 + 2 * vb + 16),
        ("erase (100 % hit)", lambda k: table.erase(n, k), resident, 165),
        # the calls that hand out addresses and hold key words (after erase: their kernels are not
        # among those the profile summary looks up by dispatch order).  Bytes per key: the digest
        # line, the key word read and locked (three times 8), the score read and written, the
        # address and the flag out; unlock_keys: address and key in, the key word read and written,
        # the flag out
        ("lock_keys (100 % hit)", lambda k: table.lock_keys(n, k, ptrs, founds), resident, 128 + 8 + 24 + 16 + 9),
        ("unlock_keys (the same keys)", None, None, 8 + 8 + 16 + 1),
        ("find_and_update (100 % hit)", lambda k: table.find_and_update(n, k, ptrs, founds), resident,
         128 + 8 + 32 + 16 + 8 + 9),
    ]
    print("| call | ms per 2^20 keys | 10^9 KV/s | algorithmic bytes per key | algorithmic GB/s | fraction of 8 TB/s |")
    print("|---|---|---|---|---|---|")
    locked = []  # (keys, key addresses) of the lock_keys calls, for the unlock_keys row
    for name, fn, gen, bpk in rows:
        times = []
        for rep in range(8):
            if name.startswith("unlock_keys"):
                k, kp = locked[rep]
                call = lambda: table.unlock_keys(n, kp, k, founds)
            else:
                k = d64(gen())
            if name.startswith("unlock_keys"):
                pass
            elif name.startswith("lock_keys"):
                kp = torch.zeros(n, dtype=torch.int64, device=dev)
                locked.append((k, kp))
                call = lambda: table.lock_keys(n, k, kp, founds)
            elif fn is None:  # accum_or_assign: the flags say which keys are there (as config 5 does)
                table.find(n, k, out, flags)
                torch.cuda.synchronize()
                call = lambda: table.accum_or_assign(n, k, vals, flags)
            else:
                call = lambda: fn(k)
            torch.cuda.synchronize()
            a = HipEvent(torch)
            b = HipEvent(torch)
            a.record()
            call()
            b.record()
            torch.cuda.synchronize()
            if rep >= 2:
                times.append(a.elapsed_time(b))
        ms = sum(times) / len(times)
        gbs = bpk * n / (ms * 1e-3) / 1e9
        print("| %s | %.4f | %.2f | %.0f | %.0f | %.3f |" % (name, ms, n / ms / 1e6, bpk, gbs, gbs / HBM_PEAK_GBS),
              flush=True)
    table.close()


def run_group_lock(torch):
    """Host time per API call, small batches so that the GPU work is negligible (1024 keys, dim 8):
    api_lock off / on with one stream (nothing to wait for, nothing recorded) / on with readers and
    an inserter alternating on two streams (every call records one event and waits for one) / a
    host-blocking acquisition in front of every call, which is what group_lock.cuh:130-166 costs
    (lock kernel <<<1,1>>> on a side stream, then cudaStreamSynchronize)."""
    import workloads_device as wd
    from hierarchicalkv_amd import EvictStrategy, HashTable, default_options

    dev = wd.DEV
    n, dim, calls = 1024, 8, 2000
    keys = wd.dev_keys(7, 0, n)
    vals = torch.zeros(n, dim, dtype=torch.float32, device=dev)
    out = torch.zeros(n, dim, dtype=torch.float32, device=dev)
    founds = torch.zeros(n, dtype=torch.bool, device=dev)
    side = torch.cuda.Stream()
    flag = torch.zeros(1, dtype=torch.int32, device=dev)
    rows = []

    def table(api_lock):
        t = HashTable()
        t.init(default_options(init_capacity=1 << 16, max_capacity=1 << 16, dim=dim, max_hbm_for_vectors=1 << 30,
                               api_lock=api_lock, evict_strategy=EvictStrategy.kLru))
        t.insert_or_assign(n, keys, vals)
        torch.cuda.synchronize()
        return t

    def per_call(fn):
        for _ in range(50):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(calls):
            fn()
        host = (time.perf_counter() - t0) / calls
        torch.cuda.synchronize()
        total = (time.perf_counter() - t0) / calls
        return host * 1e6, total * 1e6

    t = table(False)
    rows.append(("api_lock off, one stream", *per_call(lambda: t.find(n, keys, out, founds))))
    t.close()
    t = table(True)
    rows.append(("group lock as built, one stream", *per_call(lambda: t.find(n, keys, out, founds))))
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    state = [0]

    def two_streams():
        state[0] ^= 1
        if state[0]:
            t.find(n, keys, out, founds, stream=s1)
        else:
            t.insert_or_assign(n, keys, vals, stream=s2)
    rows.append(("group lock as built, find on one stream and insert_or_assign on another in turn", *per_call(two_streams)))

    def blocking():
        with torch.cuda.stream(side):
            flag.add_(1)          # stands for the lock kernel <<<1,1>>>
        side.synchronize()        # the host waits for it, as group_lock.cuh:146-166 does
        t.find(n, keys, out, founds)
    rows.append(("host-blocking acquisition before every call (as the reference)", *per_call(blocking)))
    t.close()
    print("| lock | host time per call, us | wall time per call incl. the GPU work, us |")
    print("|---|---|---|")
    for name, host, total in rows:
        print("| %s | %.1f | %.1f |" % (name, host, total), flush=True)
    print(json.dumps({"group_lock": [{"lock": r[0], "host_us": round(r[1], 2), "wall_us": round(r[2], 2)} for r in rows]}))


PROFILE_GROUPS = [
    ("trace", "--kernel-trace --stats"),
    ("fetch", "--kernel-trace --pmc FETCH_SIZE TCC_EA0_RDREQ_DRAM_sum"),
    ("write", "--kernel-trace --pmc WRITE_SIZE TCC_EA0_ATOMIC_sum TCC_ATOMIC_sum"),
    ("l2", "--kernel-trace --pmc TCC_HIT_sum TCC_MISS_sum TCC_REQ_sum TCC_EA0_RDREQ_32B_sum"),
    ("rd", "--kernel-trace --pmc TCC_EA0_RDREQ_sum TCC_EA0_RDREQ_64B_sum TCC_EA0_RDREQ_128B_sum TCC_BUBBLE_sum"),
    ("wr", "--kernel-trace --pmc TCC_EA0_WRREQ_sum TCC_EA0_WRREQ_64B_sum TCC_WRITE_sum TCC_READ_sum"),
    ("sq", "--kernel-trace --pmc OccupancyPercent SQ_WAVES SQ_LDS_BANK_CONFLICT SQ_INSTS_LDS SQ_WAIT_INST_ANY "
           "SQ_INSTS_VMEM_RD SQ_INSTS_VMEM_WR"),
    ("tcp", "--kernel-trace --pmc TCP_TCC_READ_REQ_sum TCP_TCC_WRITE_REQ_sum TCP_TCC_ATOMIC_WITH_RET_REQ_sum "
            "TCP_UTCL1_TRANSLATION_MISS_sum"),
    ("lat", "--kernel-trace --pmc TCP_TCC_READ_REQ_LATENCY_sum TCP_TCC_READ_REQ_sum TCP_PENDING_STALL_CYCLES_sum "
            "SQ_BUSY_CYCLES SQ_INSTS_VALU SQ_INSTS_SALU SQ_WAVE_CYCLES SQ_WAIT_ANY"),
]

# the part these figures are taken on: SQ_BUSY_CYCLES is summed over the shader engines
N_SHADER_ENGINES = 32
N_CUS = 256


def in_flight_row(label, c):
    """Row of the requests-in-flight table from one kernel's counters of the `lat` group."""
    busy = c["SQ_BUSY_CYCLES"] / N_SHADER_ENGINES
    reqs = max(1.0, c["TCP_TCC_READ_REQ_sum"])
    lat = c["TCP_TCC_READ_REQ_LATENCY_sum"]
    return "| %s | %.2f | %.0f | %.1f | %.2f | %.1f | %.1f | %.2f |" % (
        label, reqs / 1e6, lat / reqs, lat / busy / N_CUS, c["TCP_PENDING_STALL_CYCLES_sum"] / N_CUS / busy,
        c["SQ_INSTS_VALU"] / 1e6, c["SQ_INSTS_SALU"] / 1e6, c["SQ_WAIT_ANY"] / max(1.0, c["SQ_WAVE_CYCLES"]))


IN_FLIGHT_HEAD = (
    "| kernel | L1 -> L2 read requests (M) | average latency of one (cycles) | of them in flight per CU | share of the run "
    "in which a CU's L1 has its pending-request queue full | vector instructions (M) | scalar instructions (M) | "
    "share of wavefront time spent waiting |\n|---|---|---|---|---|---|---|---|")
# kernels of bench.py --ops, in the order of its table: (substring of the kernel name, call, algorithmic bytes per key)
OPS_KERNELS = [
    ("lookup_kernel<0, 16", "find (100 % hit)", 657),
    ("lookup_kernel<1, 16", "find* (100 % hit)", 153),
    ("lookup_kernel<2, 16", "contains (100 % hit)", 145),
    ("assign_kernel<16, 2, true>", "assign (100 % hit)", 673),
    ("upsert_kernel<0, 16, 2, false", "insert_or_assign (50 % new)", 1185),
    ("upsert_kernel<2, 16, 2, false", "find_or_insert (50 % new)", 1189),
    ("upsert_kernel<4, 16, 1, false", "find_or_insert* (50 % new)", 689),
    ("upsert_kernel<1, 16, 2, false", "insert_and_evict (50 % new)", 1449),
    ("upsert_kernel<3, 16, 2, false", "accum_or_assign (50 % new)", 1314),
    ("export_if_kernel", "export_batch_if (2^20 slots, all match)", 544),
    ("erase_kernel<true>", "erase (100 % hit)", 165),
    ("touch_kernel<true>", "lock_keys (100 % hit)", 185),
    ("unlock_keys_kernel", "unlock_keys (the same keys)", 33),
    ("touch_kernel<false>", "find_and_update (100 % hit)", 201),
]


# bench.py --config N under rocprofv3: (run tag, command, title, [(kernel needle, call, which dispatches)]).
# "last3": the timed calls are the kernel's last three dispatches; "mid3": the middle one of each
# of its last three triples (configuration 4 looks up row addresses before and after its timed
# find*); "sum8": one call is eight dispatches, added up.
CONFIG_PROFILES = [
    ("cfg2_lf050", "python3 bench.py --config 2 --load-factor 0.5", "configuration 2 (capacity 2^26, dim 8, LRU) at load factor 0.50",
     [("lookup_kernel<0, 16", "find (100 % hit)", "last3"), ("upsert_kernel<0, 16, 1, false", "insert_or_assign (50 % new)", "last3"),
      ("upsert_kernel<2, 16, 1, false", "find_or_insert (50 % new)", "last3")]),
    ("cfg2_lf075", "python3 bench.py --config 2 --load-factor 0.75", "configuration 2 at load factor 0.75",
     [("lookup_kernel<0, 16", "find (100 % hit)", "last3"), ("upsert_kernel<0, 16, 1, false", "insert_or_assign (50 % new)", "last3"),
      ("upsert_kernel<2, 16, 1, false", "find_or_insert (50 % new)", "last3")]),
    ("cfg2_lf100", "python3 bench.py --config 2 --load-factor 1.0", "configuration 2 at load factor 1.00",
     [("lookup_kernel<0, 16", "find (100 % hit)", "last3"), ("upsert_kernel<0, 16, 1, false", "insert_or_assign (50 % new)", "last3"),
      ("upsert_kernel<2, 16, 1, false", "find_or_insert (50 % new)", "last3")]),
    ("cfg3", "python3 bench.py --config 3", "configuration 3 (capacity 2^27, dim 64, Customized, Zipf keys, load factor 1.0)",
     [("upsert_kernel<1, 16, 2, false", "insert_and_evict", "last3"), ("lookup_kernel<0, 16", "find on the same keys", "last3")]),
    ("cfg4", "python3 bench.py --config 4", "configuration 4 (capacity 2^28, dim 64, 16 GiB of rows in HBM + 48 GiB pinned, LFU)",
     [("lookup_kernel<0, 16", "find (about 80 % hit)", "last3"), ("lookup_kernel<1, 16", "find*", "mid3"),
      ("upsert_kernel<0, 16, 2, false", "insert_or_assign (about 20 % new): the kernel that settles the keys, moves the rows and leaves the slots locked", "last3"),
      ("open_held_kernel", "insert_or_assign: the launch that opens the slots", "last3")]),
    ("cfg5", "python3 bench.py --config 5", "configuration 5 (capacity 2^25, dim 128, EpochLRU, load factor 1.0)",
     [("upsert_kernel<3, 16, 4, false", "accum_or_assign (70 % existing)", "last3"),
      ("export_if_kernel", "export_batch_if over the whole table (8 windows)", "sum8"),
      ("erase_kernel<true>", "erase (2^18 keys)", "last3")]),
]
CONFIG_GROUPS = ["trace", "fetch", "write", "wr", "tcp"]


def summarize_configs(root, pick, counters, durations):
    """profiles/config<N>_*.md and .json from rocprofv3 runs of bench.py --config N (see CONFIG_PROFILES)."""
    groups = dict(PROFILE_GROUPS)
    for tag, cmd, title, kernels in CONFIG_PROFILES:
        dur = durations(tag)
        if not dur:
            continue
        cnt = {g: counters(tag, g)[0] for g in CONFIG_GROUPS if g != "trace"}

        def take(values, how):
            if how == "mid3":
                v = [values[i] for i in (-2, -5, -8) if len(values) >= -i]
            elif how == "sum8":
                return sum(values[-8:])
            else:
                v = values[-3:]
            return sum(v) / len(v) if v else float("nan")

        def cval(g, needle, name, how):
            k = pick(cnt[g], needle)
            return take(cnt[g][k][name], how) if k and name in cnt[g][k] else float("nan")

        o = ["# rocprofv3: %s\n" % title,
             "One MI355X.  Commands, from the repository root after `cd /tmp && export TMPDIR=/tmp && cd -`, one run each "
             "(the output of the first is kept beside this file as %s.json):\n" % ("config" + tag[3:])]
        for g in CONFIG_GROUPS:
            o.append("    rocprofv3 %s --output-format csv -d gpurun_out/prof/%s_%s -o out -- %s" % (groups[g], tag, g, cmd))
        o.append("    python3 bench.py --profile-summary gpurun_out/prof\n")
        o.append("Per call: the average over the kernel's timed dispatches (the last three of the run; find* of "
                 "configuration 4: the middle one of each of the last three triples; export_batch_if: eight windows "
                 "added up).  FETCH_SIZE is scaled by 2.0 and WRITE_SIZE by 1.0 (what they read for a plain 1 GiB "
                 "device copy, profiles/lookup_kernel_upsert_kernel_cap2p26_dim64_batch2p20.md).  Durations are those of "
                 "the trace run; a counter run serialises and slows the kernels.  Rows that a kernel reads or writes in "
                 "pinned host memory do not pass the HBM counters.\n")
        o.append("| call | kernel | us (trace) | FETCH MB | WRITE MB | traffic GB/s | writes to memory (M) | of them partial, "
                 "below 64 B (M) | atomics to memory (M) | L1 -> L2 read / write requests (M) | returning atomics (M) | "
                 "L1 TLB misses (M) |\n|---|---|---|---|---|---|---|---|---|---|---|---|")
        for needle, call, how in kernels:
            k = pick(dur, needle)
            if not k:
                continue
            us = take(dur[k], how)
            fmb = cval("fetch", needle, "FETCH_SIZE", how) * 2.0 * 1024 / 1e6
            wmb = cval("write", needle, "WRITE_SIZE", how) * 1024 / 1e6
            wreq = cval("wr", needle, "TCC_EA0_WRREQ_sum", how)
            w64 = cval("wr", needle, "TCC_EA0_WRREQ_64B_sum", how)
            short = k.split("(")[0].replace("void ", "").replace("hkv::", "")
            o.append("| %s | `%s` | %.1f | %.1f | %.1f | %.0f | %.2f | %.2f | %.2f | %.2f / %.2f | %.2f | %.2f |" % (
                call, short, us, fmb, wmb, (fmb + wmb) / us * 1e3, wreq / 1e6, (wreq - w64) / 1e6,
                cval("write", needle, "TCC_EA0_ATOMIC_sum", how) / 1e6,
                cval("tcp", needle, "TCP_TCC_READ_REQ_sum", how) / 1e6, cval("tcp", needle, "TCP_TCC_WRITE_REQ_sum", how) / 1e6,
                cval("tcp", needle, "TCP_TCC_ATOMIC_WITH_RET_REQ_sum", how) / 1e6,
                cval("tcp", needle, "TCP_UTCL1_TRANSLATION_MISS_sum", how) / 1e6))
        # the benchmark's own table and JSON line of the trace run
        log = os.path.join(root, "%s_trace.log" % tag)
        line = None
        if os.path.exists(log):
            o.append("\n## What `%s` printed in the trace run (HIP-event times per call, algorithmic bytes)\n" % cmd)
            for ln in open(log):
                if ln.startswith("|"):
                    o.append(ln.rstrip())
                if ln.startswith("{") and '"config"' in ln:
                    line = ln.strip()
        if line:
            try:
                peak = json.loads(line).get("host_link_peak")
            except ValueError:
                peak = None
            if peak:
                o.append("\nHost link in the same run, pinned host memory <-> device copies of 1 GiB: %.1f GB/s host to "
                         "device, %.1f GB/s device to host; `host_link_gbs` above is the bytes of the rows that live "
                         "in pinned host memory over the call's time, `hbm_gbs` the rest of the call's algorithmic "
                         "bytes over the same time." % (peak["h2d_gbs"], peak["d2h_gbs"]))
        name = "config" + tag[3:]
        path = os.path.join(ROOT, "profiles", name + ".md")
        with open(path, "w") as f:
            f.write("\n".join(o) + "\n")
        print("wrote", path)
        if line:
            with open(os.path.join(ROOT, "profiles", name + ".json"), "w") as f:
                f.write(line + "\n")


def summarize_profiles(root):
    """rocprofv3 CSVs -> profiles/*.md + the traffic file.  Per kernel: the average over its last
    dispatches (the timed calls: the launches of the table fill come first), durations from the
    --kernel-trace --stats run, counters from the --pmc runs, FETCH_SIZE / WRITE_SIZE scaled by what
    they read for the 1 GiB device copy of the same run (--calibrate)."""
    import collections
    import csv
    import glob

    def csv_of(tag, group, kind):
        hits = glob.glob(os.path.join(root, "%s_%s" % (tag, group), "**", "*%s.csv" % kind), recursive=True)
        return hits[0] if hits else None

    def counters(tag, group):
        by = collections.defaultdict(lambda: collections.defaultdict(list))
        meta = {}
        f = csv_of(tag, group, "counter_collection")
        if not f:
            return by, meta
        for r in csv.DictReader(open(f)):
            by[r["Kernel_Name"]][r["Counter_Name"]].append(float(r["Counter_Value"]))
            meta[r["Kernel_Name"]] = (int(r["VGPR_Count"]), int(r["Accum_VGPR_Count"]), int(r["LDS_Block_Size"]),
                                      int(r["Scratch_Size"]), int(r["Workgroup_Size"]), int(r["Grid_Size"]))
        return by, meta

    def durations(tag):
        by = collections.defaultdict(list)
        f = csv_of(tag, "trace", "kernel_trace")
        if f:
            for r in csv.DictReader(open(f)):
                by[r["Kernel_Name"]].append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
        return by

    def pick(table, needle):
        # of an upsert kernel the form with score bounds (template argument true, before the number
        # of wavefronts per workgroup) is the one the timed calls run on an LRU table; the plain form
        # fills the table before that
        for want in ((needle + ", true, ", needle + ", false, ") if needle.startswith("upsert_kernel") else (needle,)):
            for name in table:
                if want in name:
                    return name
        return None

    # bench.py --ops launches lookup_kernel<values> twice: 8 times for its find row (the first 8
    # dispatches, 2 of them warm-up) and again, at a 50 % hit rate, to make accum_or_assign's flags
    first_eight = {"find (100 % hit)"}

    def last(values, k, call=None):
        v = values[2:8] if call in first_eight and k == 6 else values[-k:]
        return sum(v) / len(v) if v else float("nan")

    n = 1 << 20
    traffic = {"workload": "capacity 2^26, dim 64 fp32, batch 2^20, LRU, load factor 1.0", "kernels": {}}
    for tag, cmd, take, kernels, fname, title in [
        ("bench", "python3 bench.py --steps 4 --warmup 1 --no-cpu-baseline --calibrate", 3,
         [("lookup_kernel<0, 16", "find (100 % hit)", 657), ("upsert_kernel<0, 16, 2, false", "insert_or_assign (50 % new)", 1185)],
         "lookup_kernel_upsert_kernel_cap2p26_dim64_batch2p20.md",
         "lookup_kernel (find) and upsert_kernel (insert_or_assign) on the benchmark's workload"),
        ("ops", "python3 bench.py --ops", 6, OPS_KERNELS, "all_entry_points_cap2p26_dim64_batch2p20.md",
         "every entry point at the benchmark's shape (bench.py --ops)"),
    ]:
        dur = durations(tag)
        if not dur:
            continue
        groups = {g: counters(tag, g) for g, _ in PROFILE_GROUPS if g != "trace"}
        fe, _ = groups["fetch"]
        wr, _ = groups["write"]
        copyk = pick(fe, "copyBuffer")
        cal_f = cal_w = None
        if copyk and tag == "bench":
            cal_f = (1 << 20) / max(fe[copyk]["FETCH_SIZE"])      # KiB of a 1 GiB copy / counter
            cal_w = (1 << 20) / max(wr[pick(wr, "copyBuffer")]["WRITE_SIZE"])
            traffic["calibration"] = {"fetch_factor": round(cal_f, 4), "write_factor": round(cal_w, 4),
                                      "by": "1 GiB device-to-device copy in the same rocprofv3 run"}
        else:
            cal = traffic.get("calibration", {"fetch_factor": 2.0, "write_factor": 1.0})
            cal_f, cal_w = cal["fetch_factor"], cal["write_factor"]
        o = ["# rocprofv3: %s\n" % title,
             "Workload: capacity 2^26, dim 64 fp32 (16 GiB of rows in HBM), batch 2^20 unique keys, LRU, load factor 1.0.",
             "One MI355X.  Commands, from the repository root after `cd /tmp && export TMPDIR=/tmp && cd -`, one run each:\n"]
        bench_cmd = "python3 bench.py --steps 10 --warmup 3 --no-cpu-baseline" if tag == "bench" else cmd
        for g, pargs in PROFILE_GROUPS:
            o.append("    rocprofv3 %s --output-format csv -d gpurun_out/prof/%s_%s -o out -- %s" % (
                pargs, tag, g, bench_cmd if g == "trace" else cmd))
        o.append("    python3 bench.py --profile-summary gpurun_out/prof\n")
        o.append("Every figure is the average over the last %d dispatches of the kernel in its run (the timed calls; the "
                 "launches that fill the table come first).  FETCH_SIZE and WRITE_SIZE are scaled by what they read for a "
                 "plain 1 GiB device copy (factors %.3f and %.3f).  Counter runs serialise the kernels and slow them "
                 "down; durations are those of the trace run.\n" % (take, cal_f, cal_w))
        o.append("## Time and HBM traffic\n")
        o.append("| call | kernel | avg us | algorithmic MB | FETCH MB | WRITE MB | traffic / algorithmic | algorithmic GB/s | "
                 "fraction of 8 TB/s | traffic GB/s |\n|---|---|---|---|---|---|---|---|---|---|")
        detail = []
        for needle, call, bpk in kernels:
            k = pick(dur, needle)
            if not k:
                continue
            us = last(dur[k], take, call)
            alg = bpk * n / 1e6
            kf, kw = pick(fe, needle), pick(wr, needle)
            fmb = last(fe[kf]["FETCH_SIZE"], take, call) * cal_f * 1024 / 1e6 if kf else float("nan")
            wmb = last(wr[kw]["WRITE_SIZE"], take, call) * cal_w * 1024 / 1e6 if kw else float("nan")
            short = k.split("(")[0].replace("void ", "").replace("hkv::", "")
            o.append("| %s | `%s` | %.1f | %.1f | %.1f | %.1f | %.2f | %.0f | %.3f | %.0f |" % (
                call, short, us, alg, fmb, wmb, (fmb + wmb) / alg, alg / us * 1e3, alg / us * 1e3 / HBM_PEAK_GBS,
                (fmb + wmb) / us * 1e3))
            if tag == "bench":
                key = "lookup_kernel" if "lookup" in needle else "upsert_kernel"
                traffic["kernels"][key] = {"kernel": short, "traffic_bytes": round((fmb + wmb) * 1e6),
                                           "fetch_bytes": round(fmb * 1e6), "write_bytes": round(wmb * 1e6),
                                           "avg_us": round(us, 1), "algorithmic_bytes": round(alg * 1e6)}
            row = {"call": call}
            for g in ("write", "l2", "rd", "wr", "sq", "tcp"):
                by, meta = groups[g]
                kk = pick(by, needle)
                if kk:
                    for c, v in by[kk].items():
                        row[c] = last(v, take, call)
                    row["meta"] = meta[kk]
            detail.append(row)

        def col(r, c, scale=1.0, fmt="%.2f"):
            return fmt % (r[c] * scale) if c in r else "-"

        o.append("\n## L2 (TCC) and its requests to memory, millions per launch\n")
        o.append("| call | L2 requests | L2 hit rate | reads to memory | of them 128 B | 64 B | 32 B | writes to memory | of them full 64 B | "
                 "partial (below 64 B: read-modify-write at the memory side) | atomics to memory |\n|---|---|---|---|---|---|---|---|---|---|---|")
        for r in detail:
            hit = "%.3f" % (r["TCC_HIT_sum"] / max(1.0, r["TCC_REQ_sum"])) if "TCC_HIT_sum" in r else "-"
            part = "%.2f" % ((r["TCC_EA0_WRREQ_sum"] - r["TCC_EA0_WRREQ_64B_sum"]) / 1e6) if "TCC_EA0_WRREQ_sum" in r else "-"
            o.append("| %s | %s | %s | %s | %s | %s | %s | %s | %s | %s | %s |" % (
                r["call"], col(r, "TCC_REQ_sum", 1e-6), hit, col(r, "TCC_EA0_RDREQ_sum", 1e-6),
                col(r, "TCC_EA0_RDREQ_128B_sum", 1e-6), col(r, "TCC_EA0_RDREQ_64B_sum", 1e-6, "%.3f"),
                col(r, "TCC_EA0_RDREQ_32B_sum", 1e-6, "%.3f"), col(r, "TCC_EA0_WRREQ_sum", 1e-6),
                col(r, "TCC_EA0_WRREQ_64B_sum", 1e-6), part, col(r, "TCC_EA0_ATOMIC_sum", 1e-6)))
        o.append("\n## Wavefronts, LDS, vector memory, address translation\n")
        o.append("Registers per lane: twice rocprofv3's VGPR_Count field, which counts register pairs on this part "
                 "(registers are allocated in blocks of 8: the compiler's resource report for `lookup_kernel<0, 16>` reads "
                 "114, for the bounded `upsert_kernel<0, 16, 2>` 125).\n")
        o.append("| call | wavefronts | vector registers per lane | LDS bytes per workgroup | scratch | occupancy % of the maximum | vector memory reads "
                 "/ writes (M instructions) | L1 -> L2 read / write requests (M) | returning atomics (M) | L1 TLB misses (M) | "
                 "LDS instructions (M) | LDS bank-conflict cycles (M) |\n|---|---|---|---|---|---|---|---|---|---|---|---|")
        for r in detail:
            m = r.get("meta", (0, 0, 0, 0, 0, 0))
            o.append("| %s | %s | %d | %d | %d | %s | %s / %s | %s / %s | %s | %s | %s | %s |" % (
                r["call"], col(r, "SQ_WAVES", 1.0, "%.0f"), 2 * (m[0] + m[1]), m[2], m[3], col(r, "OccupancyPercent", 1.0, "%.1f"),
                col(r, "SQ_INSTS_VMEM_RD", 1e-6), col(r, "SQ_INSTS_VMEM_WR", 1e-6), col(r, "TCP_TCC_READ_REQ_sum", 1e-6),
                col(r, "TCP_TCC_WRITE_REQ_sum", 1e-6), col(r, "TCP_TCC_ATOMIC_WITH_RET_REQ_sum", 1e-6),
                col(r, "TCP_UTCL1_TRANSLATION_MISS_sum", 1e-6), col(r, "SQ_INSTS_LDS", 1e-6),
                col(r, "SQ_LDS_BANK_CONFLICT", 1e-6)))
        lat_by, _ = groups["lat"]
        if lat_by:
            o.append("\n## Read requests in flight\n")
            o.append("What bounds these kernels is the number of read requests a CU keeps in flight and how long one "
                     "takes: latency sum / busy cycles (SQ_BUSY_CYCLES is summed over the %d shader engines of the "
                     "part, %d CUs).\n" % (N_SHADER_ENGINES, N_CUS))
            o.append(IN_FLIGHT_HEAD)
            for needle, call, _ in kernels:
                kk = pick(lat_by, needle)
                if kk:
                    o.append(in_flight_row(call, {c: last(v, take, call) for c, v in lat_by[kk].items()}))
        if tag == "bench":
            stats = csv_of(tag, "trace", "kernel_stats")
            if stats:
                o.append("\n## `--stats` of the trace run (whole process, table fill included)\n")
                o.append("| kernel | calls | avg us | min us | max us | % of GPU time |\n|---|---|---|---|---|---|")
                for r in csv.DictReader(open(stats)):
                    if "hkv::" in r["Name"]:
                        o.append("| `%s` | %s | %.1f | %.1f | %.1f | %s |" % (
                            r["Name"].split("(")[0].replace("void ", "").replace("hkv::", ""), r["Calls"],
                            float(r["AverageNs"]) / 1e3, float(r["MinNs"]) / 1e3, float(r["MaxNs"]) / 1e3, r["Percentage"]))
        path = os.path.join(ROOT, "profiles", fname)
        with open(path, "w") as f:
            f.write("\n".join(o) + "\n")
        print("wrote", path)
    summarize_configs(root, pick, counters, durations)
    dur = durations("ceil")
    lat_by, _ = counters("ceil", "lat")
    if dur and lat_by:
        reps = 21  # launches per pattern: one untimed, twenty timed
        # kernel, which of its launches (patterns run in the order of CEILING_PATTERNS), label
        rows = [("k_stream_read", (1, reps), "stream_read"),
                ("k_row_gather", (1, reps), "row_gather"),
                ("k_find_pattern<false>", (reps + 1, 2 * reps), "find_pattern (1.44 key lines)"),
                ("k_find_pattern<true>", (1, reps), "find_pattern_chained, launched behind itself"),
                ("k_find_pattern<true>", (2 * reps + 1, 3 * reps), "the same in the step (step_find)"),
                ("k_upsert_pattern<false>", (reps + 1, 2 * reps), "upsert_pattern_locks"),
                ("k_upsert_pattern<true>", (1, reps), "upsert_pattern_chained, launched behind itself"),
                ("k_upsert_pattern<true>", (reps + 1, 2 * reps), "upsert_pattern_bounds, launched behind itself"),
                ("k_upsert_pattern<true>", (4 * reps + 1, 5 * reps), "upsert_pattern_chained in the step (step_upsert)")]
        o = ["# rocprofv3: the no-logic pattern kernels of bench.py --ceilings\n",
             "Workload: capacity 2^26, dim 64 fp32, batch 2^20; one MI355X.  Commands, from the repository root after "
             "`cd /tmp && export TMPDIR=/tmp && cd -`:\n",
             "    rocprofv3 --kernel-trace --stats --output-format csv -d gpurun_out/prof/ceil_trace -o out -- python3 bench.py --ceilings",
             "    rocprofv3 %s --output-format csv -d gpurun_out/prof/ceil_lat -o out -- python3 bench.py --ceilings" % dict(PROFILE_GROUPS)["lat"],
             "    python3 bench.py --profile-summary gpurun_out/prof\n",
             "Averages over the named launches of each kernel (the counter run serialises kernels: its durations are "
             "not used).  Compare with the same table for the product kernels in "
             "lookup_kernel_upsert_kernel_cap2p26_dim64_batch2p20.md.\n",
             "| kernel | avg us (trace) | L1 -> L2 read requests (M) | average latency of one (cycles) | of them in flight per CU | "
             "share of the run in which a CU's L1 has its pending-request queue full | vector instructions (M) | scalar "
             "instructions (M) | share of wavefront time spent waiting |\n|---|---|---|---|---|---|---|---|---|"]
        for needle, (lo, hi), label in rows:
            kd, kl = pick(dur, needle), pick(lat_by, needle)
            if not kd or not kl:
                continue
            us = dur[kd][lo:hi]
            c = {name: sum(v[lo:hi]) / max(1, len(v[lo:hi])) for name, v in lat_by[kl].items()}
            if not us or not c.get("SQ_BUSY_CYCLES"):
                continue
            o.append(in_flight_row("%s | %.1f" % (label, sum(us) / len(us)), c))
        path = os.path.join(ROOT, "profiles", "ceiling_kernels_cap2p26_dim64_batch2p20.md")
        with open(path, "w") as f:
            f.write("\n".join(o) + "\n")
        print("wrote", path)
    if traffic["kernels"]:
        with open(TRAFFIC_FILE, "w") as f:
            json.dump(traffic, f, indent=1)
            f.write("\n")
        print("wrote", TRAFFIC_FILE)


def run_config(args, torch):
    """Configurations 2 to 5 at full size: every call is timed by HIP events around it on the
    stream the library launches on, the median of `reps` isolated calls per figure (a
    synchronisation before each, fresh keys every time, so nothing of a call's working set is in
    the caches).
    Algorithmic bytes per key, VB = row bytes: find hit 145 + 2 VB, miss 137; find* hit 153;
    upsert of a key that is present 161 + 2 VB (find_or_insert: 169 + 2 VB), of an absent key into
    a free slot 169 + 2 VB, into a full bucket 1185 + 2 VB; insert_and_evict evicting 1201 + 4 VB;
    accum_or_assign accumulating 161 + 3 VB; export 16 per scanned slot + (2 VB + 16) per match;
    erase 165.  Mixes are priced by the outcome fractions the run itself observes."""
    import workloads_device as wd
    from hierarchicalkv_amd import EvictStrategy, HashTable, Predicate, default_options

    dev = wd.DEV
    n = 1 << 20
    reps = 3
    rows = []

    def timed(fn):
        torch.cuda.synchronize()
        a, b = HipEvent(torch), HipEvent(torch)
        a.record()
        fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b)

    def add(name, ms_list, bpk, keys=n, extra=None):
        # the median: a call that does something once per table (the first insert that uses the
        # score bounds builds them from the scores, a pass over the whole table) does not count
        ms = sorted(ms_list)[len(ms_list) // 2]
        gbs = bpk * keys / (ms * 1e-3) / 1e9
        r = {"op": name, "ms": round(ms, 4), "bkvs": round(keys / (ms * 1e-3) / 1e9, 3),
             "bytes_per_key": round(bpk, 1), "algorithmic_gbs": round(gbs, 1),
             "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)}
        if extra:
            r.update(extra)
        rows.append(r)
        print("| %s | %.4f | %.2f | %.0f | %.0f | %.3f | %s |" % (
            name, ms, r["bkvs"], bpk, gbs, gbs / HBM_PEAK_GBS,
            "; ".join("%s %s" % kv for kv in (extra or {}).items())), flush=True)

    print("| call | ms per call | 10^9 KV/s | algorithmic bytes per key | algorithmic GB/s | fraction of 8 TB/s | notes |")
    print("|---|---|---|---|---|---|---|")
    founds = torch.empty(n, dtype=torch.bool, device=dev)
    info = {}

    if args.config == 2:
        cap, dim, seed = 1 << 26, 8, 2
        vb = dim * 4
        t = HashTable()
        t.init(default_options(init_capacity=cap, max_capacity=cap, max_hbm_for_vectors=cap * vb, dim=dim,
                               evict_strategy=EvictStrategy.kLru))
        out = torch.empty(n, dim, dtype=torch.float32, device=dev)
        vals = torch.empty(n, dim, dtype=torch.float32, device=dev).uniform_(-1.0, 1.0)
        pos, fresh, old = 0, 1 << 36, 0
        for lf in ((args.load_factor,) if args.load_factor else (0.50, 0.75, 1.00)):
            while pos < int(lf * cap) or (lf == 1.0 and t.size() < 0.999 * cap and pos < 3 * cap):
                t.insert_or_assign(n, wd.dev_keys(seed, pos, n), vals)
                pos += n
            size = t.size()

            def resident():  # an old batch: still resident (inserted within the last capacity's worth), cold
                nonlocal old
                old += 1
                return wd.dev_keys(seed, pos - (8 + old % 16) * n, n)

            def mixed():
                nonlocal fresh
                k = torch.cat([resident()[: n // 2], wd.dev_keys(seed, fresh, n // 2)])
                fresh += n // 2
                return k

            full = size > 0.99 * cap
            miss = (1185 if full else 169) + 2 * vb
            ms = []
            for r in range(reps + 1):  # the first call of each kind is not timed
                k = resident()
                x = timed(lambda: t.find(n, k, out, founds))
                if r:
                    ms.append(x)
            add("find (100 %% hit), load factor %.2f" % (size / cap), ms, 145 + 2 * vb,
                extra={"hit_rate": round(float(founds.float().mean().item()), 4)})
            ms = []
            for r in range(reps + 1):
                k = mixed()
                x = timed(lambda: t.insert_or_assign(n, k, vals))
                if r:
                    ms.append(x)
            add("insert_or_assign (50 %% new), load factor %.2f" % (size / cap), ms,
                0.5 * (161 + 2 * vb) + 0.5 * miss)
            ms = []
            for r in range(reps + 1):
                k = mixed()
                x = timed(lambda: t.find_or_insert(n, k, out))
                if r:
                    ms.append(x)
            add("find_or_insert (50 %% new), load factor %.2f" % (size / cap), ms,
                0.5 * (169 + 2 * vb) + 0.5 * miss, extra={"load_factor_after": round(t.size() / cap, 4)})
        info = {"workload": "capacity 2^26, dim 8 fp32, LRU, batch 2^20, uniform keys"}
        t.close()

    elif args.config == 3:
        cap, dim, seed = 1 << 27, 64, 3
        vb = dim * 4
        t = HashTable()
        t.init(default_options(init_capacity=cap, max_capacity=cap, max_hbm_for_vectors=cap * vb, dim=dim,
                               evict_strategy=EvictStrategy.kCustomized))
        gen = torch.Generator(device=dev)
        gen.manual_seed(0x484B5603)
        batch = 1
        # uniform keys up to load factor 1.0 (the lowest scores), then 24 batches of the Zipf
        # stream so that the timed calls meet the steady state: hot keys resident, tail evicted
        vals = torch.empty(n, dim, dtype=torch.float32, device=dev).uniform_(-1.0, 1.0)
        pos = 0
        while pos < cap or (t.size() < 0.999 * cap and pos < 3 * cap):
            k = wd.dev_keys(seed, pos, n)
            t.insert_or_assign(n, k, vals, wd.batch_scores(k, batch))
            pos += n
            batch += 1
        for _ in range(24):
            k = wd.zipf_keys(gen, n)
            t.insert_or_assign(n, k, vals, wd.batch_scores(k, batch))
            batch += 1
        size0 = t.size()
        ek = torch.zeros(n, dtype=torch.int64, device=dev)
        es = torch.zeros(n, dtype=torch.int64, device=dev)
        ev = torch.zeros(n, dim, dtype=torch.float32, device=dev)
        out = torch.empty(n, dim, dtype=torch.float32, device=dev)
        cnt = torch.zeros(1, dtype=torch.int64, device=dev)
        ms_i, ms_f, hits, evs = [], [], [], []
        for _ in range(reps + 2):
            k = wd.zipf_keys(gen, n)
            sc = wd.batch_scores(k, batch)
            batch += 1
            t.contains(n, k, founds)
            hit = float(founds.float().mean().item())
            cnt.zero_()
            ms = timed(lambda: t.insert_and_evict(n, k, vals, sc, ek, ev, es, cnt))
            evicted = int(cnt.item())
            msf = timed(lambda: t.find(n, k, out, founds))
            if _ >= 2:
                ms_i.append(ms)
                ms_f.append(msf)
                hits.append(hit)
                evs.append(evicted / n)
        h = sum(hits) / len(hits)
        e = sum(evs) / len(evs)
        add("insert_and_evict (Zipf 1.05 over 2^31, load factor 1.0)", ms_i,
            h * (161 + 2 * vb) + e * (1201 + 4 * vb) + max(0.0, 1.0 - h - e) * (169 + 2 * vb),
            extra={"present": round(h, 4), "evicting": round(e, 4)})
        add("find on the same keys (all resident)", ms_f, 145 + 2 * vb,
            extra={"hit_rate": round(float(founds.float().mean().item()), 4)})
        info = {"workload": "capacity 2^27, dim 64 fp32 (32 GiB of rows in HBM), Customized scores "
                            "(batch << 40 | mix), batch 2^20 unique keys with power-law ranks (alpha 1.05) "
                            "over 2^31; table filled with uniform keys, then 24 batches of the same stream",
                "size": size0, "fill_batches": batch}
        t.close()

    elif args.config == 4:
        cap, dim, seed = 1 << 28, 64, 4
        vb = dim * 4
        hbm = 16 << 30
        t = HashTable()
        t0 = time.time()
        t.init(default_options(init_capacity=cap, max_capacity=cap, max_hbm_for_vectors=hbm, dim=dim,
                               evict_strategy=EvictStrategy.kLfu))
        assert not t.is_pure_hbm()
        init_s = time.time() - t0
        # host-link peak: pinned host <-> device copies of 1 GiB, both directions, in this run
        pin = torch.empty(1 << 28, dtype=torch.float32, pin_memory=True)
        dbuf = torch.empty(1 << 28, dtype=torch.float32, device=dev)
        h2d = min(timed(lambda: dbuf.copy_(pin, non_blocking=True)) for _ in range(3))
        d2h = min(timed(lambda: pin.copy_(dbuf, non_blocking=True)) for _ in range(3))
        link = {"h2d_gbs": round((1 << 30) / (h2d * 1e-3) / 1e9, 1), "d2h_gbs": round((1 << 30) / (d2h * 1e-3) / 1e9, 1)}
        del pin, dbuf
        ones = torch.ones(n, dtype=torch.int64, device=dev)
        vals = torch.empty(n, dim, dtype=torch.float32, device=dev).uniform_(-1.0, 1.0)
        pos = 0
        while pos < cap or (t.size() < 0.999 * cap and pos < 3 * cap):
            t.insert_or_assign(n, wd.dev_keys(seed, pos, n), vals, ones)
            pos += n
        size0 = t.size()
        view = t.view()
        hbm_lo, hbm_hi = int(view.values), int(view.values) + int(view.hbm_slots) * vb
        out = torch.empty(n, dim, dtype=torch.float32, device=dev)
        ptrs = torch.zeros(n, dtype=torch.int64, device=dev)
        fresh, old = 1 << 40, 0

        def mixed(new_fraction):
            nonlocal fresh, old
            m = int(n * new_fraction)
            old += 1
            # LFU with every frequency equal: a full bucket gives up its lowest slot, so what
            # stays resident are the keys that found a free slot, i.e. the early batches of the
            # fill; the hit rate is measured, and the bytes are priced by it
            k = torch.cat([wd.dev_keys(seed, (old % 160) * n, n)[: n - m], wd.dev_keys(seed, fresh, m)])
            fresh += m
            return k

        def host_rows(k):
            t.find_ptr(n, k, ptrs, founds)
            torch.cuda.synchronize()
            f = founds
            in_hbm = (ptrs >= hbm_lo) & (ptrs < hbm_hi)
            return int((f & ~in_hbm).sum().item()), int(f.sum().item())

        ms_f, ms_p, ms_i = [], [], []
        lf, lp, li, hf = [], [], [], []
        for _ in range(reps):
            k = mixed(0.2)
            hostn, foundn = host_rows(k)
            ms = timed(lambda: t.find(n, k, out, founds))
            ms_f.append(ms)
            lf.append(hostn * vb / (ms * 1e-3) / 1e9)
            hf.append(foundn / n)
            k = mixed(0.2)
            ms_p.append(timed(lambda: t.find_ptr(n, k, ptrs, founds)))
            k = mixed(0.2)
            ms = timed(lambda: t.insert_or_assign(n, k, vals, ones))
            hostn, foundn = host_rows(k)   # where the accepted keys' rows are now
            ms_i.append(ms)
            li.append(hostn * vb / (ms * 1e-3) / 1e9)
        hit = sum(hf) / len(hf)
        alg_find = hit * (145 + 2 * vb) + (1 - hit) * 137
        add("find (%.0f %% hit)" % (100 * hit), ms_f, alg_find,
            extra={"host_link_gbs": round(sum(lf) / len(lf), 1),
                   "hbm_gbs": round((alg_find * n - sum(lf) / len(lf) * 1e9 * (sum(ms_f) / len(ms_f)) * 1e-3)
                                    / ((sum(ms_f) / len(ms_f)) * 1e-3) / 1e9, 1)})
        add("find* (%.0f %% hit)" % (100 * hit), ms_p, hit * 153 + (1 - hit) * 137, extra={"host_link_gbs": 0.0})
        alg_ins = hit * (169 + 2 * vb) + (1 - hit) * (1185 + 8 + 2 * vb)
        add("insert_or_assign (%.0f %% new)" % (100 * (1 - hit)), ms_i, alg_ins,
            extra={"host_link_gbs": round(sum(li) / len(li), 1),
                   "hbm_gbs": round((alg_ins * n - sum(li) / len(li) * 1e9 * (sum(ms_i) / len(ms_i)) * 1e-3)
                                    / ((sum(ms_i) / len(ms_i)) * 1e-3) / 1e9, 1)})
        info = {"workload": "capacity 2^28, dim 64 fp32: 16 GiB of the 64 GiB of rows in HBM, 48 GiB in pinned host "
                            "memory; LFU; batch 2^20 uniform keys; load factor 1.0",
                "size": size0, "init_s": round(init_s, 1), "host_link_peak": link}
        t.close()

    else:
        cap, dim, seed = 1 << 25, 128, 5
        vb = dim * 4
        t = HashTable()
        t.init(default_options(init_capacity=cap, max_capacity=cap, max_hbm_for_vectors=cap * vb, dim=dim,
                               evict_strategy=EvictStrategy.kEpochLru))
        vals = torch.empty(n, dim, dtype=torch.float32, device=dev).uniform_(-0.01, 0.01)
        flags = torch.empty(n, dtype=torch.bool, device=dev)
        out = torch.empty(n, dim, dtype=torch.float32, device=dev)
        pos, batch = 0, 0
        while pos < cap or (t.size() < 0.999 * cap and pos < 3 * cap):
            t.set_global_epoch(batch // 10)
            t.insert_or_assign(n, wd.dev_keys(seed, pos, n), vals)
            pos += n
            batch += 1
        size0 = t.size()
        fresh, old = 1 << 40, 0
        ms, hits = [], []
        for _ in range(reps):
            old += 1
            m = int(0.3 * n)
            k = torch.cat([wd.dev_keys(seed, pos - (4 + old % 8) * n, n)[: n - m], wd.dev_keys(seed, fresh, m)])
            fresh += m
            t.set_global_epoch(batch // 10)
            batch += 1
            t.contains(n, k, flags)   # accumulate what is there, assign what is not
            hits.append(float(flags.float().mean().item()))
            ms.append(timed(lambda: t.accum_or_assign(n, k, vals, flags)))
        h = sum(hits) / len(hits)
        add("accum_or_assign (%.0f %% existing)" % (100 * h), ms, h * (161 + 3 * vb) + (1 - h) * (1185 + 1 + 2 * vb))
        # threshold that keeps about a quarter of the entries: the 75th percentile of a sample of scores
        sc = torch.zeros(n, dtype=torch.int64, device=dev)
        t.find(n, wd.dev_keys(seed, pos - 5 * n, n), out, founds, sc)
        torch.cuda.synchronize()
        sample = torch.cat([sc[founds]])
        for back in (1, 9, 13, 17, 21, 25, 29):
            t.find(n, wd.dev_keys(seed, pos - back * n, n), out, founds, sc)
            torch.cuda.synchronize()
            sample = torch.cat([sample, sc[founds]])
        thr = int(torch.quantile(sample[:: max(1, sample.numel() // (1 << 20))].to(torch.float64), 0.75).item())
        window = 1 << 22
        dk = torch.zeros(window, dtype=torch.int64, device=dev)
        ds = torch.zeros(window, dtype=torch.int64, device=dev)
        dv = torch.zeros(window, dim, dtype=torch.float32, device=dev)
        dc = torch.zeros(1, dtype=torch.int64, device=dev)
        total_ms, matched = 0.0, 0
        for off in range(0, cap, window):
            total_ms += timed(lambda: t.export_batch_if(Predicate.kScoreGe, 0, thr, window, off, dc, dk, dv, ds))
            matched += int(dc.item())
        add("export_batch_if (score >= threshold, whole table)", [total_ms],
            (16 * cap + (2 * vb + 16) * matched) / cap, keys=cap,
            extra={"kept": round(matched / max(1, size0), 4), "windows": cap // window})
        ms = []
        ne = 1 << 18
        for r in range(reps):
            k = wd.dev_keys(seed, pos - (2 + r) * n, ne)
            ms.append(timed(lambda: t.erase(ne, k)))
        add("erase (2^18 keys)", ms, 165, keys=ne)
        info = {"workload": "capacity 2^25, dim 128 fp32, EpochLRU (epoch = batch / 10), batch 2^20 uniform keys, "
                            "deltas in [-0.01, 0.01], load factor 1.0", "size": size0}
    print(json.dumps({"config": args.config, **info, "ops": rows}))


CEILING_PATTERNS = [
    # name, what one launch does, unit of the rate
    ("stream_read", "16-byte streaming loads over 1 GiB", "GB/s"),
    ("stream_write", "16-byte streaming stores over 1 GiB", "GB/s"),
    ("stream_copy", "1 GiB read + 1 GiB written", "GB/s"),
    ("row_gather", "random table rows -> dense array (read + written bytes)", "GB/s"),
    ("row_scatter", "dense array -> random table rows, write-through stores (read + written bytes)", "GB/s"),
    ("find_pattern_1line", "find's accesses, one key line per key, no logic (algorithmic bytes)", "GB/s"),
    ("find_pattern", "find's accesses, 1.44 key lines per key (false digest matches), no logic "
                     "(algorithmic bytes)", "GB/s"),
    ("find_pattern_chained", "find's accesses, 1.1 key lines per key, each group of addresses known only when the "
                             "group before has arrived (batch key -> digest line -> key word -> row), no logic "
                             "(algorithmic bytes)", "GB/s"),
    ("upsert_pattern", "insert_or_assign's accesses, 50 % absent keys into full buckets, no locks, no logic "
                       "(algorithmic bytes)", "GB/s"),
    ("upsert_pattern_locks", "the same plus the slot-lock protocol's atomics, re-reads and unlock stores "
                             "(algorithmic bytes)", "GB/s"),
    ("upsert_pattern_chained", "upsert_pattern_locks with 1.1 key lines per key and every group of addresses known "
                               "only when the group before has arrived (batch key -> digest line -> key word and "
                               "compare-and-swap -> score scan -> exchange and score re-read -> stores -> unlock)", "GB/s"),
    ("upsert_pattern_bounds", "upsert_pattern_chained with the bucket's 8 score bounds (64 bytes) and one score line "
                              "read per absent key instead of all 8 lines, and one more 8-byte store", "GB/s"),
    ("step_pattern", "find_pattern_chained, then upsert_pattern_chained on other keys: the benchmark's step "
                     "(algorithmic bytes of both)", "GB/s"),
    ("step_find", "the find half of step_pattern, timed launch by launch", "GB/s"),
    ("step_upsert", "the insert_or_assign half of step_pattern, timed launch by launch", "GB/s"),
    ("small_load8", "8-byte loads, one per random 128-byte line", "G ops/s"),
    ("small_store8", "8-byte write-through stores, one per random line", "G ops/s"),
    ("small_store1", "1-byte write-through stores, one per random line", "G ops/s"),
    ("small_store16", "16-byte write-through stores, one per random line", "G ops/s"),
    ("small_chunk64", "aligned 64-byte chunks written by 4 lanes, one per random line", "G ops/s"),
    ("small_cas64", "64-bit compare-and-swap, one per random line", "G ops/s"),
    ("small_xchg64", "64-bit exchange, one per random line", "G ops/s"),
    ("small_xchg32_side", "32-bit exchange on a 4-byte-per-bucket array (fits the Infinity Cache)", "G ops/s"),
    # (new patterns go to the end: --profile-summary finds the launches of the ones above by their order)
    ("upsert_pattern_free", "insert_or_assign's accesses on a table with free slots, chained: 50 % absent keys that "
                            "take a free slot with a compare-and-swap, no score reads (algorithmic bytes)", "GB/s"),
    ("findptr_pattern", "find* / contains: batch key -> digest line -> key word (1.1 lines per key) -> 8-byte result "
                        "and flag (algorithmic bytes: 153 per key)", "GB/s"),
    ("erase_pattern", "erase with the table to itself: batch key -> digest line -> key word -> key store, digest "
                      "store (algorithmic bytes: 165 per key)", "GB/s"),
]


def run_ceilings(args):
    """Access-pattern ceilings at the benchmark's shape; see hkv_ceilings.hip."""
    import ctypes

    path = os.path.join(ROOT, "hierarchicalkv_amd", "libhkv_ceilings.so")
    if not os.path.exists(path):
        raise SystemExit("libhkv_ceilings.so is not built: run python hierarchicalkv_amd/build.py ceilings")
    lib = ctypes.CDLL(path)
    lib.hkv_ceilings_last_error.restype = ctypes.c_char_p
    lib.hkv_ceilings_setup.argtypes = [ctypes.c_uint64, ctypes.c_uint32, ctypes.c_uint64]
    lib.hkv_ceilings_run.argtypes = [ctypes.c_char_p, ctypes.c_int, ctypes.POINTER(ctypes.c_double),
                                     ctypes.POINTER(ctypes.c_double)]
    buckets = (1 << args.capacity_log2) // 128
    vb = args.dim * 4
    n = 1 << args.batch_log2
    if lib.hkv_ceilings_setup(buckets, vb, n):
        raise SystemExit(lib.hkv_ceilings_last_error().decode())
    reps = max(args.steps, 5)
    out = {}
    print("| pattern | what one launch does | ms per launch | rate | fraction of 8 TB/s |")
    print("|---|---|---|---|---|")
    for name, what, unit in CEILING_PATTERNS:
        ms, moved = ctypes.c_double(), ctypes.c_double()
        if lib.hkv_ceilings_run(name.encode(), reps, ctypes.byref(ms), ctypes.byref(moved)):
            raise SystemExit(lib.hkv_ceilings_last_error().decode())
        rate = moved.value / (ms.value * 1e-3) / 1e9
        out[name] = {"ms": round(ms.value, 5), "rate": round(rate, 2), "unit": unit}
        frac = "%.3f" % (rate / HBM_PEAK_GBS) if unit == "GB/s" else ""
        print("| %s | %s | %.4f | %.1f %s | %s |" % (name, what, ms.value, rate, unit, frac), flush=True)
    lib.hkv_ceilings_release()
    print(json.dumps({"ceilings": out, "config": {"workload": f"capacity 2^{args.capacity_log2}, dim "
                                                  f"{args.dim} fp32, batch 2^{args.batch_log2}",
                                                  "launches_per_pattern": reps}}))


def cpu_baseline(args, np, w):
    """The host oracle (multithreaded variant, a port of the same semantics) on a
    bounded sample: same dim / batch / load factor 1.0 at a smaller capacity."""
    import oracle_binding as ob
    from hierarchicalkv_amd import EvictStrategy, default_options

    cap = 1 << args.cpu_capacity_log2
    dim = args.dim
    n = 1 << args.batch_log2
    threads = min(ob.online_cores(), 16)
    seed = 0x484B5600
    opts = default_options(init_capacity=cap, max_capacity=cap, dim=dim, evict_strategy=EvictStrategy.kLru)
    t = ob.OracleTable(opts)
    vals = np.random.default_rng(1).random((n, dim), dtype=np.float32).view(np.uint8).reshape(n, dim * 4)
    pos = 0
    while pos < cap:
        t.insert_or_assign_mt(w.unique_keys(seed, pos, n), vals, threads=threads)
        pos += n
    prev = w.unique_keys(seed, pos - n, n)
    reps = 100  # about 10 s of host work
    tf = ti = 0.0
    out = np.zeros((n, dim * 4), np.uint8)
    for r in range(reps):
        a = time.perf_counter()
        t.find(prev, out, want_scores=False, threads=threads)
        b = time.perf_counter()
        batch = np.concatenate([prev[: n // 2], w.unique_keys(seed, pos, n // 2)])
        pos += n // 2
        c = time.perf_counter()
        t.insert_or_assign_mt(batch, vals, threads=threads)
        d = time.perf_counter()
        tf += b - a
        ti += d - c
        prev = batch
    t.close()
    return {
        "value": round(2.0 * n * reps / (tf + ti) / 1e9, 5),
        "unit": "billion-KV/s (10^9 keys/s, find + insert_or_assign per step)",
        "cores": threads,
        "kind": "port",
        "find_bkvs": round(n * reps / tf / 1e9, 5),
        "insert_or_assign_bkvs": round(n * reps / ti / 1e9, 5),
        "sample": f"{reps} steps of the same workload at capacity 2^{args.cpu_capacity_log2} "
                  f"(dim {dim}, batch 2^{args.batch_log2}, load factor 1.0), host oracle with "
                  f"{threads} threads; table pre-filled by the same code",
    }


if __name__ == "__main__":
    main()
