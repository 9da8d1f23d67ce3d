"""Writes tests/golden/scenario_customized.npz: the inputs of tests/golden/scenario.py and
the outputs the host oracle gives for them.

The reference cannot be built or run without CUDA, so this fixture is not a recording of the
reference: it freezes what the oracle answered once its functions had been pinned by
tests/test_oracle_pins.py (known answers, closed-form scenarios of the reference's own tests,
brute-force models).  Its job is to catch a later change that moves the oracle and the library
together.  Usage (from the repository root, after building the oracle):

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, HERE)

import oracle_binding  # noqa: E402
import scenario  # noqa: E402
from hierarchicalkv_amd import EvictStrategy, default_options  # noqa: E402


class OracleDriver:
    def __init__(self):
        o = default_options(init_capacity=scenario.CAPACITY, max_capacity=scenario.CAPACITY, dim=scenario.DIM,
                            max_hbm_for_vectors=1 << 30, evict_strategy=EvictStrategy.kCustomized)
        self.t = oracle_binding.OracleTable(o)

    @staticmethod
    def _b(vals):
        return np.ascontiguousarray(vals).view(np.uint8).reshape(len(vals), -1)

    def insert_or_assign(self, k, v, s):
        self.t.insert_or_assign(k, self._b(v), s)

    def find(self, k):
        return self.t.find(k)

    def insert_and_evict(self, k, v, s):
        return self.t.insert_and_evict(k, self._b(v), s)

    def erase(self, k):
        self.t.erase(k)

    def accum_or_assign(self, k, v, f, s):
        self.t.accum_or_assign(k, self._b(v), np.asarray(f, np.uint8), s)

    def size(self):
        return self.t.size()

    def export_all(self):
        return self.t.export_all()


if __name__ == "__main__":
    inp = scenario.make_inputs()
    out = scenario.run(OracleDriver(), inp)
    data = {f"in_{k}": v for k, v in inp.items()}
    data.update({f"out_{k}": v for k, v in out.items()})
    path = os.path.join(HERE, "scenario_customized.npz")
    np.savez_compressed(path, **data)
    print("wrote", path, os.path.getsize(path), "bytes;",
          "final size", int(out["size_final"][0]), "evicted", len(out["evicted_keys"]),
          "found", int(out["find_founds"].sum()))
