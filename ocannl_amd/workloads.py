"""The benchmark configurations as routines in the loop IR, with seeded synthetic data.

Each builder returns a :class:`Workload`: the routine(s) a ``Train.to_routine`` call would compile
(forward + backprop + optimiser update as ONE routine, as in test/training/moons_demo.ml:61), the
nodes to upload, and the nodes to read back.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from . import llir as L
from .frontend import ConstT, Graph, T, make_routine


@dataclass
class Workload:
    name: str
    routine: L.Routine
    init: Dict[int, np.ndarray]                 # node id -> host values to upload before step 0
    nodes: Dict[str, L.Node]                    # named nodes (params, loss, ...)
    statics: Dict[str, L.StaticSymbol] = field(default_factory=dict)
    outputs: List[L.Node] = field(default_factory=list)
    description: str = ""


def to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """float32 -> bfloat16 bit patterns, round to nearest even (arrayjit/lib/builtins.c:620-627)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF).astype(np.uint16)


def from_bf16_bits(b: np.ndarray) -> np.ndarray:
    return (b.astype(np.uint32) << 16).view(np.float32)


def as_prec(x: np.ndarray, prec: str) -> np.ndarray:
    if prec == "bfloat16":
        return to_bf16_bits(x)
    return np.ascontiguousarray(x, dtype={"single": np.float32, "double": np.float64, "half": np.float16}[prec])


def to_float(a: np.ndarray, prec: str) -> np.ndarray:
    if prec == "bfloat16":
        return from_bf16_bits(a).astype(np.float64)
    return a.astype(np.float64)


# ------------------------------------------------------------------------------------------------
# config 1: half-moons MLP
# ------------------------------------------------------------------------------------------------

def half_moons(n: int, noise: float, seed: int):
    """1024-point half-moons as BASELINE config 1 defines them: two unit-radius half circles, the
    second shifted by (1, -0.5) and flipped, N(0, noise) jitter, labels +-1."""
    rng = np.random.default_rng(seed)
    half = n // 2
    t = rng.uniform(0.0, np.pi, size=n)
    x = np.empty((n, 2), np.float32)
    y = np.empty((n,), np.float32)
    x[:half, 0] = np.cos(t[:half]); x[:half, 1] = np.sin(t[:half]); y[:half] = 1.0
    x[half:, 0] = 1.0 - np.cos(t[half:]); x[half:, 1] = 0.5 - np.sin(t[half:]); y[half:] = -1.0
    x += rng.normal(0.0, noise, size=x.shape).astype(np.float32)
    perm = rng.permutation(n)
    return x[perm], y[perm]


def moons_mlp(batch: int = 20, n_points: int = 1024, hidden: int = 16, lr: float = 0.1, momentum: float = 0.9,
              weight_decay: float = 0.0, seed: int = 0, inline: bool = True, prec: str = "single") -> Workload:
    """MLP 2->16->16->1 ReLU, hinge loss ``mean relu(1 - y f(x))``, SGD with momentum; the batch is a
    slice ``data @| batch_n`` of the resident data set (test/training/moons_demo.ml:42-61)."""
    L.reset_symbols(0)
    g = Graph(prec, prec)
    n_batches = n_points // batch
    batch_n = L.StaticSymbol(L.fresh_symbol(), n_batches)
    data = g.input("moons_flat", ("n", "b", "i"), (n_batches, batch, 2))
    classes = g.input("moons_classes", ("n", "b"), (n_batches, batch))
    w1 = g.param("w1", ("h1", "i"), (hidden, 2)); b1 = g.param("b1", ("h1",), (hidden,))
    w2 = g.param("w2", ("h2", "h1"), (hidden, hidden)); b2 = g.param("b2", ("h2",), (hidden,))
    w3 = g.param("w3", ("o", "h2"), (1, hidden))
    lrate = g.input("learning_rate", ("one",), (1,))
    # the slice views: leading index is the static symbol (assignments.ml:226-232)
    x = T(data.value, ("b", "i"), None, label="moons_input")
    x_get = lambda idx: L.Get(data.value, (L.It(batch_n.sym), idx["b"], idx["i"]))
    y_get = lambda idx: L.Get(classes.value, (L.It(batch_n.sym), idx["b"]))
    xs = _SliceT(data.value, ("b", "i"), (batch, 2), x_get)
    ys = _SliceT(classes.value, ("b",), (batch,), y_get)
    h1 = g.unary("relu", g.add(b1, g.einsum(w1, xs, ("b", "h1"), ident="w1x"), ("b", "h1")))
    h2 = g.unary("relu", g.add(b2, g.einsum(w2, h1, ("b", "h2"), ident="w2h"), ("b", "h2")))
    f = g.einsum(w3, h2, ("b", "o"), ident="mlp")
    margin = g.unary("relu", g.sub(ConstT(1.0), g.mul(ys, f, ("b", "o")), ("b", "o")), ident="margin_loss")
    total = g.reduce(margin, ("l",), ident="loss_sum")
    loss = g.div(total, ConstT(float(batch)), ("l",), ident="scalar_loss")
    loss.label = "scalar_loss"
    params = [w1, b1, w2, b2, w3]
    body = g.grad_update(loss) + g.sgd_update(params, lrate, momentum=momentum, weight_decay=weight_decay)
    routine = make_routine(g, "moons_sgd_step", body, [batch_n], inline=inline, outputs=[loss.value])
    rng = np.random.default_rng(seed + 1)
    xd, yd = half_moons(n_points, 0.1, seed)
    init = {
        data.value.id: as_prec(xd[: n_batches * batch].reshape(n_batches, batch, 2), prec),
        classes.value.id: as_prec(yd[: n_batches * batch].reshape(n_batches, batch), prec),
        lrate.value.id: as_prec(np.array([lr], np.float32), prec),
    }
    for p in params:
        fan_in = p.dims[-1] if len(p.dims) > 1 else 1
        lim = np.sqrt(6.0 / (fan_in + p.dims[0])) if len(p.dims) > 1 else 0.0
        init[p.value.id] = as_prec(rng.uniform(-lim, lim, size=p.dims).astype(np.float32), prec)
    nodes = {p.label: p.value for p in params}
    nodes.update({"loss": loss.value, "data": data.value, "classes": classes.value})
    for p in params:
        nodes["mom_" + p.label] = p.sgd_momentum
    return Workload("moons_mlp", routine, init, nodes, {"batch_n": batch_n}, [loss.value],
                    f"MLP 2->{hidden}->{hidden}->1 relu, hinge, SGD lr {lr} momentum {momentum}, batch {batch}")


class _SliceT(T):
    """A read-only view whose element read is an arbitrary index expression (slice by a static
    symbol).  Only usable as an operand."""

    def __init__(self, node, axes, dims, getter):
        super().__init__(node, tuple(axes), None)
        self._dims = tuple(dims)
        self._getter = getter

    @property
    def dims(self):
        return self._dims


# ------------------------------------------------------------------------------------------------
# config 3: dense-layer contraction, forward and both gradients
# ------------------------------------------------------------------------------------------------

def dense_contraction(b: int = 8192, i: int = 4096, o: int = 4096, prec: str = "single", out_prec: str = "single",
                      seed: int = 0, which: Sequence[str] = ("fwd", "dx", "dw"), reduce_order: str = "last") -> Workload:
    """``Y[b,o] = sum_i X[b,i] W[o,i]`` plus ``dX[b,i] += sum_o dY[b,o] W[o,i]`` and
    ``dW[o,i] += sum_b dY[b,o] X[b,i]``: the matmul of tensor/operation.ml:96-99 and its gradient
    assignments (operation.ml:77-83).  ``prec`` is the operand precision, results are ``out_prec``
    (bf16 operands with a single-precision destination = "bf16 with fp32 accumulation")."""
    L.reset_symbols(0)
    g = Graph(prec, out_prec, reduce_order=reduce_order)
    X = g.node("x", (b, i), prec, "ctx"); W = g.node("w", (o, i), prec, "ctx")
    Y = g.node("y", (b, o), out_prec, "ctx"); dY = g.node("dy", (b, o), prec, "ctx")
    dX = g.node("dx", (b, i), out_prec, "ctx"); dW = g.node("dw", (o, i), out_prec, "ctx")
    body: List[L.Stmt] = []
    sp = [("b", b), ("o", o), ("i", i)]
    if "fwd" in which:
        body.append(L.Comment("y fwd"))
        body += g.lower(Y, ("b", "o"), sp, lambda ix: L.Binop("mul", L.Get(X, (ix["b"], ix["i"])), L.Get(W, (ix["o"], ix["i"]))))
    if "dx" in which:
        body.append(L.Comment("dx"))
        body += g.lower(dX, ("b", "i"), [("b", b), ("i", i), ("o", o)],
                        lambda ix: L.Binop("mul", L.Get(dY, (ix["b"], ix["o"])), L.Get(W, (ix["o"], ix["i"]))), init_neutral=False)
    if "dw" in which:
        body.append(L.Comment("dw"))
        body += g.lower(dW, ("o", "i"), [("o", o), ("i", i), ("b", b)],
                        lambda ix: L.Binop("mul", L.Get(dY, (ix["b"], ix["o"])), L.Get(X, (ix["b"], ix["i"]))), init_neutral=False)
    routine = L.Routine(f"dense_{prec}", body)
    rng = np.random.default_rng(seed)
    init = {
        X.id: as_prec(rng.uniform(-1, 1, (b, i)).astype(np.float32), prec),
        W.id: as_prec(rng.uniform(-1, 1, (o, i)).astype(np.float32), prec),
        dY.id: as_prec(rng.uniform(-1, 1, (b, o)).astype(np.float32), prec),
    }
    nodes = {"x": X, "w": W, "y": Y, "dy": dY, "dx": dX, "dw": dW}
    outs = [n for k, n in (("fwd", Y), ("dx", dX), ("dw", dW)) if k in which]
    return Workload(f"dense_{prec}", routine, init, nodes, {}, outs,
                    f"b|i->o contraction b={b} i={i} o={o} {prec} (dest {out_prec}), fwd+dX+dW")
