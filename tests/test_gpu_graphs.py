"""Replay of a routine's kernel list from a captured HIP graph (one graph per combination of static-index
values; fills recorded as kernels, never as memsets; the side queue as a branch of the graph): every
replay has to leave exactly what launching the kernels one by one leaves (`graphs=0`), step after step,
with reads of results and synchronisations of the program's own between the replays.  (`graphs=1`; the
default is off: on this ROCm the replay pays only for routines of about ten tiny kernels.)"""
import numpy as np
import pytest

from ocannl_amd import backend as B
from ocannl_amd import workloads as W
from parity import HipRun

pytestmark = pytest.mark.gpu


def _same_after_every_step(w, steps, statics_of, names, options=None):
    opt = (options + ";" if options else "")
    replay, direct = HipRun(w.routine, w.init, opt + "graphs=1"), HipRun(w.routine, w.init, opt + "graphs=0")
    for step in range(steps):
        st = statics_of(step)
        replay.step(st); direct.step(st)
        for name in names:   # (reading a result synchronises the device: eager work between two replays)
            assert np.array_equal(replay.get(w.nodes[name]), direct.get(w.nodes[name])), (step, name)
    replay.close(); direct.close()


def test_moons_steps_replayed_per_static_index_value():
    w = W.moons_mlp()
    sym, nb = w.statics["batch_n"].sym, w.statics["batch_n"].range
    # serial=0: dozens of kernels per step; batches revisited, so that every graph is replayed several times
    _same_after_every_step(w, 24, lambda s: {sym: (s * 7) % 5}, ("loss", "w1", "b2", "w3", "mom_w2"), "serial=0")
    _same_after_every_step(w, 8, lambda s: {sym: s % nb}, ("loss", "w1"), "serial=0;parallel=0")


def test_char_mlp_adam_steps_replayed():
    w = W.char_mlp()
    sym, nb = w.statics["batch_n"].sym, w.statics["batch_n"].range
    _same_after_every_step(w, 3 * nb, lambda s: {sym: s % nb}, ("loss", "c", "w1", "b2", "m_w1", "v_w2"))


def test_transformer_steps_with_fills_side_queue_and_split_k_replayed():
    kw = dict(batch=8, seq=128, d_model=256, heads=4, d_ff=512, layers=2, vocab=512, prec="bfloat16", grad_prec="single", lr=0.05)
    w = W.transformer(**kw)
    ks = B.compile(w.routine, "side_queue=1").kernels()
    assert any(k["kind"] == "mfma" for k in ks)
    _same_after_every_step(w, 5, lambda s: None, ("loss", "w_q_l0", "w_ffn2_l1", "w_out", "b_ffn1_l0", "beta_ln2_l1"), "side_queue=1")


def test_attention_replayed_and_bad_static_index_still_refused():
    w = W.attention(b=2, h=4, q=64, k=128, d=32, prec="bfloat16", grad_prec="single")
    _same_after_every_step(w, 4, lambda s: None, ("out", "dq", "dk", "dv"), "min_mfma_flops=1")
    m = W.moons_mlp()
    h = HipRun(m.routine, m.init, "serial=0;graphs=1")
    sym = m.statics["batch_n"].sym
    for _ in range(3):
        h.step({sym: 1})
    with pytest.raises(B.User_error):
        h.step({sym: m.statics["batch_n"].range})   # out of range: refused, nothing captured or launched
    h.step({sym: 2})
    h.close()
