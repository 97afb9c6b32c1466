"""In-routine logging (debug_log_from_routines: arrayjit/lib/c_syntax.ml:493-535, utils.ml:591): a routine
compiled with debug_log=1 prints from the device what every statement computes, in the reference's line
format and in program order.  The run happens in a child process whose standard output is captured, as
the reference's tests capture theirs (test/operations/micrograd_demo_logging.ml)."""
import os
import re
import subprocess
import sys

import numpy as np
import pytest

from conftest import ROOT

pytestmark = pytest.mark.gpu

CHILD = r"""
import sys
sys.path.insert(0, {root!r}); sys.path.insert(0, {tests!r})
import numpy as np
from ocannl_amd import backend as B
from test_kat_routines import micrograd
r, init, nodes = micrograd()
h = B.HipRun(r, init, "debug_log=1")
h.step()
B.await_(h.ctx.dev)
print("LOGID", h.rt.log_id(), flush=True)
print("RESULT", float(h.get(nodes["g"])[0]), float(h.get(nodes["a_grad"])[0]), float(h.get(nodes["b_grad"])[0]), flush=True)
h.step()
B.await_(h.ctx.dev)
print("LOGID2", h.rt.log_id(), flush=True)
h.close()
"""


def test_micrograd_log_lines_from_the_device():
    from ocannl_amd import backend as B
    from ocannl_amd import llir as L
    from test_kat_routines import micrograd
    p = subprocess.run([sys.executable, "-c", CHILD.format(root=ROOT, tests=os.path.join(ROOT, "tests"))],
                       capture_output=True, text=True, timeout=240)
    assert p.returncode == 0, p.stderr[-2000:]
    out = p.stdout
    log_id = int(re.search(r"LOGID (\d+)", out).group(1))
    g, ag, bg = (float(x) for x in re.search(r"RESULT (\S+) (\S+) (\S+)", out).groups())
    assert int(g * 1000) == 24704 and int(ag * 1000) == 138833 and int(bg * 1000) == 645577   # logging leaves results alone
    lines = B.routine_log_lines(out, log_id)
    r, init, nodes = micrograd()
    # one `# statement` line per Set of the routine, in program order, each followed by its value line;
    # a Zero_out logs `# <ident> := 0` per element (c_syntax.ml:476-479)
    expected = []

    def walk(body):
        for c in body:
            if isinstance(c, L.For):
                walk(c.body)
            elif isinstance(c, L.Set):
                expected.append("# " + L.ll_statement(c))
            elif isinstance(c, L.ZeroOut):
                # (the first function-scope Zero_out of a routine-local node that its declaration already
                # zeroes prints nothing: c_syntax.ml:424-432)
                if not (c.node.mode == "local" and c.node.zero_initialized_by_code and c.node.id not in seen):
                    expected.extend(["# " + c.node.ident + " := 0"] * c.node.num_elems)
                seen.add(c.node.id)
    seen = set()
    walk(r.body)
    stmt_lines = [l for l in lines if l.startswith("# ") and not l.startswith("# local")]
    assert stmt_lines == expected
    comments = [l for l in lines if l.startswith("COMMENT: ")]
    assert comments[0] == "COMMENT: g forward and gradient update" and "COMMENT: g zero grads and backprop" in comments
    # value lines: lhs[offset]{=old} = new = expression with the value of every read in braces
    first = lines[lines.index(stmt_lines[0]) + 1]
    m = re.fullmatch(r"(\w+)\[0\]\{=(\S+)\} = (\S+) = \((\w+)\[0\]\{=(\S+)\} \+ (\w+)\[0\]\{=(\S+)\}\)", first)
    assert m, first
    assert float(m.group(3)) == -2.0 and float(m.group(5)) == -4.0 and float(m.group(7)) == 2.0   # c = a + b
    # the final value of g appears on the line of the statement that computes it (24.7041 as %g)
    g_line = [l for l in lines if l.startswith(nodes["g"].ident + "[0]{=")]
    assert g_line and abs(float(re.search(r"\} = (\S+) = ", g_line[-1]).group(1)) - 24.7041) < 1e-3
    # a second run logs under the next id
    assert int(re.search(r"LOGID2 (\d+)", out).group(1)) == log_id + 1
    assert len(B.routine_log_lines(out, log_id + 1)) == len(lines)


CHILD_VS_CHECKER = r"""
import sys
sys.path.insert(0, {root!r}); sys.path.insert(0, {tests!r})
import numpy as np
from ocannl_amd import backend as B
from test_kat_routines import micrograd
from test_oracle_emit import _log_stmt_format
which = {which!r}
if which == "micrograd":
    r, init, nodes = micrograd()
else:
    r, (a, b, c) = _log_stmt_format()
    init = {{a.id: np.array([1.0], np.float32), b.id: np.array([1.0], np.float32)}}
h = B.HipRun(r, init, "debug_log=1")
h.step()
B.await_(h.ctx.dev)
print("LOGID", h.rt.log_id(), flush=True)
h.close()
"""


def _normalise(lines):
    # what the reference's own test does to a log before comparing it with the golden
    # (test/operations/dune:55-75): addresses and the old value of a one-element lhs are masked
    out = []
    for ln in lines:
        ln = re.sub(r" = 0x[0-9a-fA-F]+$| = \(nil\)$", " = 0xNNNN", ln)
        ln = re.sub(r"^([a-z0-9_]+)\[0\]\{=[-+.e0-9naif]+\} = ", r"\1[0]{=MAYBE UNINITIALIZED} = ", ln)
        out.append(ln)
    return out


@pytest.mark.parametrize("which", ["log_stmt_format", "micrograd"])
def test_device_log_equals_the_checkers_log_line_for_line(which, tmp_path):
    # The checker's generated C logs through fprintf exactly as the reference's does (pinned token for
    # token by test_oracle_emit.py::test_text_log_stmt_format); the device has to print the same lines:
    # the parameter header, comments, `# statement`, value lines with the value of every read.
    from ocannl_amd import backend as B
    from oracle import cc_oracle
    from test_kat_routines import micrograd
    from test_oracle_emit import _log_stmt_format
    p = subprocess.run([sys.executable, "-c", CHILD_VS_CHECKER.format(root=ROOT, tests=os.path.join(ROOT, "tests"), which=which)],
                       capture_output=True, text=True, timeout=240)
    assert p.returncode == 0, p.stderr[-2000:]
    log_id = int(re.search(r"LOGID (\d+)", p.stdout).group(1))
    device = B.routine_log_lines(p.stdout, log_id)
    if which == "micrograd":
        r, init, _ = micrograd()
    else:
        r, (a, b, c) = _log_stmt_format()
        init = {a.id: np.array([1.0], np.float32), b.id: np.array([1.0], np.float32)}
    from parity import oracle_buffers
    bufs = oracle_buffers(r, init)
    log = tmp_path / "checker.log"
    cc_oracle.CompiledOracle([r], debug_log=True).run(r.name, bufs, log_file=str(log))
    checker = log.read_text().splitlines()
    assert len(checker) > 5
    assert _normalise(device) == _normalise(checker)
