"""The committed fixture tests/golden/scenario_customized.npz against the host oracle (CPU) and
against the library through the C ABI (GPU).  The fixture holds its own inputs; what it freezes
and why is said in tests/golden/make_golden.py."""
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))

import scenario  # noqa: E402


def load_fixture():
    z = np.load(os.path.join(HERE, "golden", "scenario_customized.npz"))  # allow_pickle stays False
    inp = {k[3:]: z[k] for k in z.files if k.startswith("in_")}
    out = {k[4:]: z[k] for k in z.files if k.startswith("out_")}
    return inp, out


def compare(got, want):
    assert set(got) == set(want)
    for name in sorted(want):
        assert got[name].shape == want[name].shape, name
        assert (got[name] == want[name]).all(), name


def test_fixture_inputs_are_the_seeded_ones():
    inp, _ = load_fixture()
    again = scenario.make_inputs()
    assert set(inp) == set(again)
    for k in inp:
        assert (inp[k] == again[k]).all(), k


def test_oracle_reproduces_the_fixture(oracle):
    import make_golden
    inp, want = load_fixture()
    compare(scenario.run(make_golden.OracleDriver(), inp), want)


class LibraryDriver:
    """The same calls through hierarchicalkv_amd (ctypes over the C ABI), device buffers from torch."""

    def __init__(self):
        import torch
        from gpu_util import DEV, dev, export_table, host_bytes, host_u64
        from hierarchicalkv_amd import EvictStrategy, HashTable, default_options
        self.torch, self.DEV, self.dev = torch, DEV, dev
        self.export_table, self.host_bytes, self.host_u64 = export_table, host_bytes, host_u64
        self.vb = scenario.DIM * 4
        self.t = HashTable()
        self.t.init(default_options(init_capacity=scenario.CAPACITY, max_capacity=scenario.CAPACITY,
                                    dim=scenario.DIM, max_hbm_for_vectors=1 << 30,
                                    evict_strategy=EvictStrategy.kCustomized))

    def insert_or_assign(self, k, v, s):
        self.t.insert_or_assign(len(k), self.dev(k), self.dev(v), self.dev(s))

    def find(self, k):
        torch = self.torch
        n = len(k)
        out = torch.zeros(n, scenario.DIM, dtype=torch.float32, device=self.DEV)
        founds = torch.zeros(n, dtype=torch.bool, device=self.DEV)
        sc = torch.zeros(n, dtype=torch.int64, device=self.DEV)
        self.t.find(n, self.dev(k), out, founds, sc)
        torch.cuda.synchronize()
        return self.host_bytes(out, n, self.vb), founds.cpu().numpy(), self.host_u64(sc)

    def insert_and_evict(self, k, v, s):
        torch = self.torch
        n = len(k)
        ek = torch.zeros(n, dtype=torch.int64, device=self.DEV)
        ev = torch.zeros(n, scenario.DIM, dtype=torch.float32, device=self.DEV)
        es = torch.zeros(n, dtype=torch.int64, device=self.DEV)
        cnt = torch.zeros(1, dtype=torch.int64, device=self.DEV)
        self.t.insert_and_evict(n, self.dev(k), self.dev(v), self.dev(s), ek, ev, es, cnt)
        torch.cuda.synchronize()
        c = int(cnt.item())
        return self.host_u64(ek)[:c].copy(), self.host_bytes(ev, n, self.vb)[:c].copy(), self.host_u64(es)[:c].copy()

    def erase(self, k):
        self.t.erase(len(k), self.dev(k))

    def accum_or_assign(self, k, v, f, s):
        self.t.accum_or_assign(len(k), self.dev(k), self.dev(v), self.dev(np.asarray(f, bool)), self.dev(s))

    def size(self):
        return self.t.size()

    def export_all(self):
        return self.export_table(self.t, self.vb)


@pytest.mark.gpu
def test_library_reproduces_the_fixture():
    inp, want = load_fixture()
    d = LibraryDriver()
    compare(scenario.run(d, inp), want)
    d.t.close()
