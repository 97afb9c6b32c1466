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
    """1024-point half-moons as benchmark configuration 1 defines them: two unit-radius half circles, the
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


def plain_copy(n: int = 1 << 26, prec: str = "single") -> Workload:
    """``y[i] = x[i]`` over ``n`` elements: one generated kernel that reads and writes a known
    number of bytes -- the yardstick for memory-traffic counters."""
    L.reset_symbols(0)
    x = L.Node(1, "x", prec, (n,)); y = L.Node(2, "y", prec, (n,))
    i = L.fresh_symbol()
    routine = L.Routine("plain_copy", [L.For(i, 0, n - 1, [L.Set(y, (L.It(i),), L.Get(x, (L.It(i),)))])])
    rng = np.random.default_rng(0)
    init = {1: as_prec(rng.uniform(-1, 1, n).astype(np.float32), prec)}
    return Workload("plain_copy", routine, init, {"x": x, "y": y}, {}, [y],
                    f"copy of {n} {prec} elements ({2 * x.size_in_bytes} bytes of traffic)")


# ------------------------------------------------------------------------------------------------
# config 2: character-level MLP language model
# ------------------------------------------------------------------------------------------------

def char_mlp(batch: int = 32, vocab: int = 27, context: int = 3, embed: int = 10, hidden: int = 200,
             lr: float = 1e-3, seed: int = 0, inline: bool = True, n_batches: int = 16) -> Workload:
    """test/training/mlp_names.ml:145-168 with synthetic tokens: ids -> embedding gather ->
    ``tanh(emb +* w1 + b1)`` -> logits -> stable log-softmax cross entropy; Adam update.  A fresh
    batch is a slice of a resident id/target set selected by the static index ``batch_n``."""
    L.reset_symbols(0)
    g = Graph("single", "single")
    batch_n = L.StaticSymbol(L.fresh_symbol(), n_batches)
    ids_all = g.input("input_batch", ("n", "b", "s"), (n_batches, batch, context))
    tgt_all = g.input("target_batch", ("n", "b", "v"), (n_batches, batch, vocab))
    ids = _SliceT(ids_all.value, ("b", "s"), (batch, context),
                  lambda idx: L.Get(ids_all.value, (L.It(batch_n.sym), idx["b"], idx["s"])))
    ids.value_prec = "single"
    tgt = _SliceT(tgt_all.value, ("b", "v"), (batch, vocab),
                  lambda idx: L.Get(tgt_all.value, (L.It(batch_n.sym), idx["b"], idx["v"])))
    c = g.param("c", ("e", "v"), (embed, vocab))
    w1 = g.param("w1", ("h", "s", "e"), (hidden, context, embed)); b1 = g.param("b1", ("h",), (hidden,))
    w2 = g.param("w2", ("v", "h"), (vocab, hidden)); b2 = g.param("b2", ("v",), (vocab,))
    # the gather reads the ids through the slice's getter
    emb = _gather_rows_with_getter(g, c, ids, (batch, context), "v")
    hid = g.unary("tanh", g.add(g.einsum(emb, w1, ("b", "h"), ident="emb_w1"), b1, ("b", "h")), ident="hidden")
    logits = g.add(g.einsum(w2, hid, ("b", "v"), ident="w2h"), b2, ("b", "v"), ident="logits")
    max_l = g.reduce(logits, ("b",), accum="max", ident="max_l")
    shifted = g.sub(logits, max_l, ("b", "v"), ident="shifted")
    lse = g.unary("log", g.reduce(g.unary("exp", shifted), ("b",), ident="sumexp"), ident="lse")
    log_probs = g.sub(shifted, lse, ("b", "v"), ident="log_probs")
    nll = g.unary("neg", g.reduce(g.mul(tgt, log_probs, ("b", "v")), ("l",), ident="tgt_lp"), ident="nll")
    loss = g.div(nll, ConstT(float(batch)), ("l",), ident="batch_loss")
    loss.label = "batch_loss"
    params = [c, w1, b1, w2, b2]
    body = g.grad_update(loss) + g.adam_update(params, lr=lr)
    routine = make_routine(g, "char_mlp_adam_step", body, [batch_n], inline=inline, outputs=[loss.value])
    rng = np.random.default_rng(seed)
    toks = rng.integers(0, vocab, size=(n_batches, batch, context + 1))
    onehot = np.zeros((n_batches, batch, vocab), np.float32)
    np.put_along_axis(onehot, toks[..., -1:], 1.0, axis=-1)
    init = {ids_all.value.id: toks[..., :context].astype(np.float32), tgt_all.value.id: onehot}
    for p in params:
        fan = int(np.prod(p.dims[1:])) if len(p.dims) > 1 else p.dims[0]
        init[p.value.id] = (rng.uniform(-1, 1, p.dims) / np.sqrt(fan)).astype(np.float32)
    nodes = {p.label: p.value for p in params}
    nodes["loss"] = loss.value
    for p in params:
        nodes["m_" + p.label] = p.adam_m
        nodes["v_" + p.label] = p.adam_v
    return Workload("char_mlp", routine, init, nodes, {"batch_n": batch_n}, [loss.value],
                    f"char MLP LM vocab {vocab} ctx {context} emb {embed} hid {hidden} batch {batch}, Adam lr {lr}")


def _gather_rows_with_getter(g, table, ids, ids_dims, table_axis, ident="embed"):
    out_axes = tuple(ids.axes) + tuple(a for a in table.axes if a != table_axis)
    ext = dict(zip(ids.axes, ids_dims))
    ext.update(dict(zip(table.axes, table.dims)))
    classes = ext[table_axis]
    v, gr = g._result(ident, out_axes, ext, None, True)
    res = T(v, out_axes, gr, (table,), label=ident)
    dyn_axis = table.axes.index(table_axis)

    def value(idx):
        iv = ids._getter(idx)
        guard = L.Binop("and", L.Binop("and", L.Binop("lt", L.Const(-1.0), iv), L.Binop("lt", iv, L.Const(float(classes)))),
                        L.Binop("eq", iv, L.Unop("trunc", iv, "double")))
        tix = tuple(L.Fixed(0) if a == table_axis else idx[a] for a in table.axes)
        return L.Ternop("where", guard, L.GetDynamic(table.value, tix, dyn_axis, iv, "single"), L.Const(0.0), "double")

    space = [(a, ext[a]) for a in out_axes]
    res.fwd = g.lower(v, out_axes, space, value)

    def bwd():
        sp = space + [(table_axis, classes)]
        return g.lower(table.grad, table.axes, sp, lambda idx: L.Binop(
            "mul", L.Get(gr, tuple(idx[a] for a in out_axes)),
            L.Binop("eq", L.EmbedIndex(idx[table_axis]), ids._getter(idx))), accum="add", init_neutral=False)

    res.bwd = bwd
    return res


# ------------------------------------------------------------------------------------------------
# config 5: batched attention, forward and backward
# ------------------------------------------------------------------------------------------------

def attention(b: int = 16, h: int = 16, q: int = 1024, k: int = 1024, d: int = 64, prec: str = "bfloat16",
              grad_prec: str = "single", seed: int = 0, inline: bool = True, backward: bool = True) -> Workload:
    """``scores[b,s,h,t] = sum_d Q[b,s,h,d] K[b,t,h,d] / sqrt(d)``, softmax over ``t``,
    ``out[b,s,h,e] = sum_t attn[b,s,h,t] V[b,t,h,e]`` (lib/nn_blocks.ml:222-236) and the backward
    contractions from a supplied ``d out``."""
    from .frontend import softmax
    L.reset_symbols(0)
    g = Graph(prec, grad_prec)
    Q = g.param("q", ("b", "s", "h", "d"), (b, q, h, d)); K = g.param("k", ("b", "t", "h", "d"), (b, k, h, d))
    V = g.param("v", ("b", "t", "h", "e"), (b, k, h, d))
    for t in (Q, K, V):
        t.grad.mode = "ctx"
    scores = g.div(g.einsum(Q, K, ("b", "s", "h", "t"), ident="qk"), ConstT(float(np.sqrt(d))), ("b", "s", "h", "t"),
                   ident="scores")
    attn = softmax(g, scores, "t", ident="attn")
    out = g.einsum(attn, V, ("b", "s", "h", "e"), ident="attn_out")
    out.label = "attn_out"
    body = g.forward(out)
    outputs = [out.value]
    if backward:
        body += g.backprop_from(out)
        outputs += [Q.grad, K.grad, V.grad]
    routine = make_routine(g, "attention_fwd_bwd" if backward else "attention_fwd", body, [], inline=inline, outputs=outputs)
    rng = np.random.default_rng(seed)
    init = {t.value.id: as_prec(rng.standard_normal(t.dims).astype(np.float32), prec) for t in (Q, K, V)}
    if backward:
        init[out.grad.id] = as_prec(rng.standard_normal(out.dims).astype(np.float32), grad_prec)
    nodes = {"q": Q.value, "k": K.value, "v": V.value, "out": out.value, "attn": attn.value,
             "dq": Q.grad, "dk": K.grad, "dv": V.grad, "dout": out.grad}
    return Workload("attention", routine, init, nodes, {}, outputs,
                    f"attention b={b} h={h} q={q} k={k} d={d} {prec}, fwd{'+bwd' if backward else ''}")


# ------------------------------------------------------------------------------------------------
# config 4: decoder-only transformer training step
# ------------------------------------------------------------------------------------------------

def transformer(batch: int = 32, seq: int = 256, d_model: int = 512, heads: int = 8, d_ff: int = 2048,
                layers: int = 4, vocab: int = 4096, prec: str = "bfloat16", grad_prec: str = "single",
                lr: float = 0.01, seed: int = 0, inline: bool = True) -> Workload:
    """Decoder-only transformer: ``Nn_blocks.decoder_only`` (lib/nn_blocks.ml:274-296: post-norm
    blocks of masked multi-head attention and a 2-layer ReLU FFN), wired as in
    test/training/fsm_transformer.ml:122-139 -- one-hot token input times an embedding matrix plus
    a learned positional encoding, a final projection to the vocabulary, softmax cross entropy --
    with ``Train.grad_update`` + ``Train.sgd_update`` compiled as one routine."""
    from .frontend import layer_norm, rename, softmax
    L.reset_symbols(0)
    g = Graph(prec, grad_prec)
    dk = d_model // heads
    x_in = g.input("input_batch", ("b", "s", "v"), (batch, seq, vocab))
    target = g.input("target_batch", ("b", "s", "v"), (batch, seq, vocab))
    mask = g.input("mask", ("s", "t"), (seq, seq), "single")
    lrate = g.input("learning_rate", ("one",), (1,), "single")
    params: List[T] = []

    def P(name, axes, dims):
        p = g.param(name, axes, dims)
        params.append(p)
        return p

    w_embed = P("w_embed", ("m", "v"), (d_model, vocab))
    pos = P("pos_encoding", ("s", "m"), (seq, d_model))
    x = g.add(g.einsum(w_embed, x_in, ("b", "s", "m"), ident="embed"), pos, ("b", "s", "m"), ident="embedded")
    for li in range(layers):
        lb = f"l{li}"
        w_q = P(f"w_q_{lb}", ("h", "d", "m"), (heads, dk, d_model))
        w_k = P(f"w_k_{lb}", ("h", "d", "m"), (heads, dk, d_model))
        w_v = P(f"w_v_{lb}", ("h", "e", "m"), (heads, dk, d_model))
        w_o = P(f"w_o_{lb}", ("m", "h", "e"), (d_model, heads, dk))
        q = g.einsum(w_q, x, ("b", "s", "h", "d"), ident=f"q_{lb}")
        k = rename(g.einsum(w_k, x, ("b", "s", "h", "d"), ident=f"k_{lb}"), {"s": "t"})
        v = rename(g.einsum(w_v, x, ("b", "s", "h", "e"), ident=f"v_{lb}"), {"s": "t"})
        scores = g.div(g.einsum(q, k, ("b", "s", "h", "t"), ident=f"qk_{lb}"), ConstT(float(np.sqrt(dk))),
                       ("b", "s", "h", "t"), ident=f"scores_{lb}")
        masked = g.where(mask, scores, ConstT(-1e9), ident=f"masked_{lb}")
        attn = softmax(g, _reorder(g, masked, ("b", "s", "h", "t")), "t", ident=f"attn_{lb}")
        att_out = g.einsum(attn, v, ("b", "s", "h", "e"), ident=f"attn_out_{lb}")
        mha = g.einsum(w_o, att_out, ("b", "s", "m"), ident=f"mha_{lb}")
        x1, ln1p = layer_norm(g, g.add(x, mha, ("b", "s", "m")), "m", f"ln1_{lb}")
        params += ln1p
        w_f1 = P(f"w_ffn1_{lb}", ("f", "m"), (d_ff, d_model)); b_f1 = P(f"b_ffn1_{lb}", ("f",), (d_ff,))
        w_f2 = P(f"w_ffn2_{lb}", ("m", "f"), (d_model, d_ff))
        hid = g.unary("relu", g.add(g.einsum(w_f1, x1, ("b", "s", "f"), ident=f"ffn1_{lb}"), b_f1, ("b", "s", "f")),
                      ident=f"ffn_hid_{lb}")
        ffn = g.einsum(w_f2, hid, ("b", "s", "m"), ident=f"ffn_{lb}")
        x, ln2p = layer_norm(g, g.add(x1, ffn, ("b", "s", "m")), "m", f"ln2_{lb}")
        params += ln2p
    w_out = P("w_out", ("v", "m"), (vocab, d_model))
    logits = g.einsum(w_out, x, ("b", "s", "v"), ident="logits")
    counts = g.unary("exp", logits, ident="counts")
    probs = g.div(counts, g.reduce(counts, ("b", "s"), ident="counts_sum"), ("b", "s", "v"), ident="probs")
    # the loss reduction is kept in single precision (Tn.update_prec on the loss nodes): a bfloat16
    # running sum of 8192 token losses saturates
    output_probs = g.reduce(g.mul(probs, target, ("b", "s", "v")), ("b", "s"), ident="output_probs", prec="single")
    tok_loss = g.unary("neg", g.unary("log", output_probs, prec="single"), ident="loss", prec="single")
    batch_loss = g.div(g.reduce(tok_loss, ("l",), ident="loss_sum", prec="single"), ConstT(float(batch * seq)), ("l",),
                       ident="batch_loss", prec="single")
    batch_loss.label = "batch_loss"
    body = g.grad_update(batch_loss) + g.sgd_update(params, lrate)
    routine = make_routine(g, "transformer_sgd_step", body, [], inline=inline, outputs=[batch_loss.value])
    rng = np.random.default_rng(seed)
    toks = rng.integers(0, vocab, size=(batch, seq + 1))
    oh_in = np.zeros((batch, seq, vocab), np.float32); oh_tg = np.zeros((batch, seq, vocab), np.float32)
    np.put_along_axis(oh_in, toks[:, :seq, None], 1.0, axis=-1)
    np.put_along_axis(oh_tg, toks[:, 1:, None], 1.0, axis=-1)
    init = {x_in.value.id: as_prec(oh_in, prec), target.value.id: as_prec(oh_tg, prec),
            mask.value.id: np.tril(np.ones((seq, seq), np.float32)),
            lrate.value.id: np.array([lr], np.float32)}
    for p in params:
        if p.label.startswith("gamma"):
            vals = np.ones(p.dims, np.float32)
        elif p.label.startswith(("beta", "b_")):
            vals = np.zeros(p.dims, np.float32)
        else:
            fan_in = int(np.prod([d_ for a, d_ in zip(p.axes, p.dims) if a in ("m", "v", "f", "e") and a != p.axes[0]])) or p.dims[-1]
            vals = (rng.uniform(-1, 1, p.dims) * np.sqrt(3.0 / max(fan_in, 1))).astype(np.float32)
        init[p.value.id] = as_prec(vals, prec)
    nodes = {p.label: p.value for p in params}
    nodes.update({"loss": batch_loss.value, "logits": logits.value})
    wl = Workload("transformer", routine, init, nodes, {}, [batch_loss.value],
                  f"decoder-only transformer x{layers}: d_model {d_model}, {heads} heads, d_ff {d_ff}, seq {seq}, "
                  f"batch {batch}, vocab {vocab}, {prec} values / {grad_prec} grads, SGD lr {lr}")
    wl.params = params
    return wl


def _reorder(g: Graph, t: T, axes):
    """Guarantee the axis order of a tensor (a copy only when it differs)."""
    if tuple(t.axes) == tuple(axes):
        return t
    return g.nary(t.label + "_perm", [t], axes, lambda x: x, [lambda gr, v, x: gr])
