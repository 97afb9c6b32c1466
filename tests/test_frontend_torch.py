"""The harness that builds the benchmark routines (ocannl_amd/frontend.py: forward code, reverse-mode
differentiation, SGD update, lowering to the loop IR) pinned against PyTorch autograd: the transformer
training step of benchmark configuration 4 at a small size, executed by the CPU checker in fp32, has
to give the loss and the updated parameters that the same architecture gives in PyTorch. Both sides of
the GPU parity tests consume the same IR, so a mistake in the harness's derivatives would pass them
unnoticed; this test is what catches it."""
import numpy as np
import pytest

from ocannl_amd import workloads as W
from parity import OracleRun

torch = pytest.importorskip("torch")


def _layer_norm(x, gamma, beta, eps=1e-5):
    # Nn_blocks.layer_norm as written (lib/nn_blocks.ml:251-258): "mean" is the sum over the axis
    d = x.shape[-1]
    centered = (x - x.sum(-1, keepdim=True)) / d
    std = torch.sqrt((centered * centered).sum(-1, keepdim=True) + eps)
    return gamma * (centered / std) + beta


def _torch_step(w, P, steps, kw):
    layers, heads, dk = kw["layers"], kw["heads"], kw["d_model"] // kw["heads"]
    x_in = torch.tensor(w.init[w.routine_inputs["input_batch"]]); target = torch.tensor(w.init[w.routine_inputs["target_batch"]])
    mask = torch.tensor(w.init[w.routine_inputs["mask"]])
    losses = []
    for _ in range(steps):
        for p in P.values():
            p.grad = None
        x = torch.einsum("mv,bsv->bsm", P["w_embed"], x_in) + P["pos_encoding"]
        for li in range(layers):
            lb = f"l{li}"
            q = torch.einsum("hdm,bsm->bshd", P[f"w_q_{lb}"], x)
            k = torch.einsum("hdm,btm->bthd", P[f"w_k_{lb}"], x)
            v = torch.einsum("hem,btm->bthe", P[f"w_v_{lb}"], x)
            scores = torch.einsum("bshd,bthd->bsht", q, k) / float(np.sqrt(dk))
            masked = torch.where(mask[None, :, None, :] != 0, scores, torch.tensor(-1e9))
            attn = torch.softmax(masked, dim=-1)
            mha = torch.einsum("mhe,bshe->bsm", P[f"w_o_{lb}"], torch.einsum("bsht,bthe->bshe", attn, v))
            x1 = _layer_norm(x + mha, P[f"gamma_ln1_{lb}"], P[f"beta_ln1_{lb}"])
            hid = torch.relu(torch.einsum("fm,bsm->bsf", P[f"w_ffn1_{lb}"], x1) + P[f"b_ffn1_{lb}"])
            x = _layer_norm(x1 + torch.einsum("mf,bsf->bsm", P[f"w_ffn2_{lb}"], hid), P[f"gamma_ln2_{lb}"], P[f"beta_ln2_{lb}"])
        logits = torch.einsum("vm,bsm->bsv", P["w_out"], x)
        counts = torch.exp(logits)
        probs = counts / counts.sum(-1, keepdim=True)
        loss = (-torch.log((probs * target).sum(-1))).sum() / (x_in.shape[0] * x_in.shape[1])
        loss.backward()
        losses.append(float(loss.detach()))
        with torch.no_grad():
            for p in P.values():
                p -= kw["lr"] * p.grad
    return losses


def test_transformer_step_of_the_harness_equals_pytorch_autograd():
    kw = dict(batch=2, seq=16, d_model=32, heads=2, d_ff=64, layers=2, vocab=64, lr=0.05)
    w = W.transformer(prec="single", grad_prec="single", **kw)
    by_ident = {n.ident.rsplit("_", 1)[0]: n.id for n in w.routine.param_nodes()}
    w.routine_inputs = {k: by_ident[k] for k in ("input_batch", "target_batch", "mask")}
    P = {label: torch.tensor(np.array(w.init[node.id]), dtype=torch.float32, requires_grad=True)
         for label, node in w.nodes.items() if label not in ("loss", "logits")}
    steps = 3
    want = _torch_step(w, P, steps, kw)
    ora = OracleRun(w.routine, w.init)
    got = []
    for _ in range(steps):
        ora.step()
        got.append(float(ora.get(w.nodes["loss"])[0]))
    assert np.allclose(got, want, rtol=2e-5), (got, want)
    for label, p in P.items():
        a, b = ora.get(w.nodes[label]), p.detach().numpy()
        assert np.max(np.abs(a - b)) <= 2e-5 * max(1.0, float(np.max(np.abs(b)))), label


def test_char_mlp_adam_step_of_the_harness_equals_pytorch():
    # benchmark configuration 2: embedding gather -> tanh layer -> logits -> log-softmax cross entropy,
    # Adam exactly as the reference documents it (docs/migration_guide.md:639-652: no bias correction,
    # epsilon added to sqrt(v)); a fresh batch per step through the static index
    w = W.char_mlp()
    by_ident = {n.ident.rsplit("_", 1)[0]: n.id for n in w.routine.param_nodes()}
    ids_all = torch.tensor(w.init[by_ident["input_batch"]]).long()
    tgt_all = torch.tensor(w.init[by_ident["target_batch"]])
    P = {k: torch.tensor(np.array(w.init[w.nodes[k].id]), requires_grad=True) for k in ("c", "w1", "b1", "w2", "b2")}
    M = {k: torch.zeros_like(p) for k, p in P.items()}; V = {k: torch.zeros_like(p) for k, p in P.items()}
    ora = OracleRun(w.routine, w.init)
    sym = w.statics["batch_n"].sym
    for step in range(4):
        n = step % w.statics["batch_n"].range
        ora.step({sym: n})
        for p in P.values():
            p.grad = None
        emb = P["c"].t()[ids_all[n]]                                   # [b, s, e]
        hid = torch.tanh(torch.einsum("bse,hse->bh", emb, P["w1"]) + P["b1"])
        logits = torch.einsum("vh,bh->bv", P["w2"], hid) + P["b2"]
        loss = -(tgt_all[n] * torch.log_softmax(logits, dim=-1)).sum() / ids_all.shape[1]
        loss.backward()
        with torch.no_grad():
            for k, p in P.items():
                M[k] = 0.9 * M[k] + (1.0 - 0.9) * p.grad
                V[k] = 0.999 * V[k] + (1.0 - 0.999) * p.grad * p.grad
                p -= 1e-3 * M[k] / (torch.sqrt(V[k]) + 1e-8)
        assert abs(float(ora.get(w.nodes["loss"])[0]) - float(loss.detach())) <= 2e-5 * float(loss.detach()), step
    for k, p in P.items():
        a, b = ora.get(w.nodes[k]), p.detach().numpy()
        assert np.max(np.abs(a - b)) <= 1e-4 * max(1.0, float(np.max(np.abs(b)))), k
        assert np.allclose(ora.get(w.nodes["m_" + k]), M[k].numpy(), rtol=1e-3, atol=1e-7), k


def test_moons_sgd_momentum_step_of_the_harness_equals_pytorch():
    # benchmark configuration 1: MLP 2->16->16->1, hinge loss mean relu(1 - y f(x)), Train.sgd_one with
    # momentum (lib/train.ml:76-90): delta = g + wd p; m = mu m + delta; p -= lr m -- which is
    # torch.optim.SGD(momentum=mu, dampening=0)
    w = W.moons_mlp()
    data = torch.tensor(np.array(w.init[w.nodes["data"].id])); cls = torch.tensor(np.array(w.init[w.nodes["classes"].id]))
    P = {k: torch.tensor(np.array(w.init[w.nodes[k].id]), requires_grad=True) for k in ("w1", "b1", "w2", "b2", "w3")}
    opt = torch.optim.SGD(list(P.values()), lr=0.1, momentum=0.9)
    ora = OracleRun(w.routine, w.init)
    sym = w.statics["batch_n"].sym
    for step in range(6):
        n = step % w.statics["batch_n"].range
        ora.step({sym: n})
        opt.zero_grad()
        h1 = torch.relu(data[n] @ P["w1"].t() + P["b1"])
        h2 = torch.relu(h1 @ P["w2"].t() + P["b2"])
        f = (h2 @ P["w3"].t())[:, 0]
        loss = torch.relu(1.0 - cls[n] * f).mean()
        loss.backward()
        opt.step()
        assert abs(float(ora.get(w.nodes["loss"])[0]) - float(loss.detach())) <= 2e-5 * max(1.0, float(loss.detach())), step
    for k, p in P.items():
        a, b = ora.get(w.nodes[k]), p.detach().numpy()
        assert np.max(np.abs(a - b)) <= 1e-4 * max(1.0, float(np.max(np.abs(b)))), k
