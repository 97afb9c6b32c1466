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


def _rows(a: np.ndarray) -> np.ndarray:
    a = np.asarray(a, np.float64)
    return a.reshape(-1, a.shape[-1]) if a.ndim >= 2 else a.reshape(1, -1)


def rel_err(got: np.ndarray, want: np.ndarray, prec: str) -> float:
    """Largest |got - want| relative to the scale of the ROW the element sits in (the tensor's last
    axis; a vector or scalar is one row): max over rows of max|diff| / max|want| of that row.  So an
    element is judged against max(|want|, its row's scale): a row of small gradients is not excused by
    large values elsewhere in the tensor.  A row whose expected values are all (nearly) zero is judged
    at a thousandth of the tensor's scale -- below that a deviation is the noise of sums that cancel,
    whatever computes them."""
    g, w = _rows(W.to_float(got, prec)), _rows(W.to_float(want, prec))
    assert g.shape == w.shape, (g.shape, w.shape)
    tensor = max(float(np.max(np.abs(w))), 1e-30)
    scale = np.maximum(np.max(np.abs(w), axis=1), 1e-3 * tensor)
    return float(np.max(np.max(np.abs(g - w), axis=1) / scale))


def tensor_err(got: np.ndarray, want: np.ndarray, prec: str) -> float:
    """max |got - want| / max |want| over the whole tensor (looser than rel_err: kept for reporting)."""
    g, w = W.to_float(got, prec), W.to_float(want, prec)
    scale = max(float(np.max(np.abs(w))), 1e-30)
    return float(np.max(np.abs(g - w))) / scale
