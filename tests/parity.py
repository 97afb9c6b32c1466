"""Shared helpers for the parity tests: run one routine through the CPU checker (oracle/) and
through the HIP library on identical host buffers, and compare."""
from __future__ import annotations

from typing import Dict, Mapping, Optional, Sequence

import numpy as np

from ocannl_amd import llir as L
from ocannl_amd import workloads as W
from oracle import cc_oracle


def oracle_buffers(routine: L.Routine, init: Mapping[int, np.ndarray]) -> Dict[int, np.ndarray]:
    bufs = {}
    for n in routine.param_nodes():
        if n.id in init:
            a = np.array(init[n.id], copy=True)
            assert a.nbytes == n.size_in_bytes, (n, a.shape, a.dtype)
            bufs[n.id] = np.ascontiguousarray(a)
        else:
            bufs[n.id] = cc_oracle.host_array(n)
    return bufs


class OracleRun:
    """Compiled checker + live host buffers (parameters persist across steps, like a context)."""

    def __init__(self, routine: L.Routine, init: Mapping[int, np.ndarray]):
        self.routine = routine
        self.lib = cc_oracle.CompiledOracle([routine])
        self.bufs = oracle_buffers(routine, init)

    def step(self, static: Optional[Mapping[int, int]] = None):
        self.lib.run(self.routine.name, self.bufs, static or {})

    def get(self, node: L.Node) -> np.ndarray:
        return self.bufs[node.id]


from ocannl_amd.backend import HipRun  # noqa: E402,F401  (the GPU side lives in the package)


def rel_err(got: np.ndarray, want: np.ndarray, prec: str) -> float:
    """max |got - want| / max(|want|_inf, tiny): relative to the tensor's scale."""
    g, w = W.to_float(got, prec), W.to_float(want, prec)
    scale = max(float(np.max(np.abs(w))), 1e-30)
    return float(np.max(np.abs(g - w))) / scale
