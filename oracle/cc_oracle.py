"""TEST INFRASTRUCTURE -- CPU checker, not part of the shipped product path.

Compiles the C text of :mod:`oracle.cc_emit` the way ``Cc_backend.c_compile_and_load`` does
(arrayjit/lib/cc_backend.ml:62-153: ``cc <file> -O3 -march=native -o <lib> -shared -fPIC``, no
``-ffast-math``), loads it with ``dlopen`` and calls routines on caller-owned numpy buffers,
one core, in-process -- the ``sync_cc`` execution model (arrayjit/lib/schedulers.ml:231-287).
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import subprocess
import sys
import tempfile
from typing import Dict, Mapping, Sequence

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(_HERE))
from ocannl_amd import llir as L  # noqa: E402
from oracle import cc_emit  # noqa: E402

NP_DTYPE = {
    "byte": np.uint8, "uint16": np.uint16, "int32": np.int32, "uint32": np.uint32,
    "int64": np.int64, "uint64": np.uint64, "half": np.float16, "bfloat16": np.uint16,
    "fp8": np.uint8, "single": np.float32, "double": np.float64,
}

CC_FLAGS = ["-O3", "-march=native", "-shared", "-fPIC"]  # cc_backend.ml:17-21,82,87-96


def np_dtype(prec: str):
    if prec == "uint4x32":
        return np.dtype((np.uint32, 4))
    return np.dtype(NP_DTYPE[prec])


def host_array(node: L.Node, fill=None) -> np.ndarray:
    if node.prec == "uint4x32":
        a = np.zeros(node.dims + (4,), dtype=np.uint32)
    else:
        a = np.zeros(node.dims, dtype=NP_DTYPE[node.prec])
    if fill is not None:
        a[...] = fill
    return a


class CompiledOracle:
    """A loaded translation unit holding one or more routines."""

    def __init__(self, routines: Sequence[L.Routine], keep_dir: str | None = None, debug_log: bool = False,
                 full_printf: bool = True):
        """``debug_log``: the routines log every computed value (``debug_log_from_routines``); ``run``
        then takes the name of the file to write (cc_backend.ml: the log file per run)."""
        self.routines = {r.name: r for r in routines}
        self.debug_log = debug_log
        self.source = cc_emit.emit_translation_unit(routines, debug_log, full_printf)
        tag = hashlib.sha1(self.source.encode()).hexdigest()[:16]
        d = keep_dir or os.path.join(tempfile.gettempdir(), "ocannl_oracle_cc")
        os.makedirs(d, exist_ok=True)
        self.c_path = os.path.join(d, f"r_{tag}.c")
        self.so_path = os.path.join(d, f"r_{tag}.so")
        if not os.path.exists(self.so_path):
            with open(self.c_path, "w") as f:
                f.write(self.source)
            tmp = self.so_path + f".{os.getpid()}.tmp"
            cmd = [os.environ.get("CC", "cc"), self.c_path] + CC_FLAGS + ["-o", tmp, "-lm"]
            p = subprocess.run(cmd, capture_output=True, text=True)
            if p.returncode != 0:
                # cc_backend.ml:105-117: compile failure is an internal error with the output
                raise ValueError(
                    f"oracle: generated code failed to compile (exit {p.returncode})\n"
                    f"{' '.join(cmd)}\n{p.stderr}")
            os.replace(tmp, self.so_path)
        self.lib = ctypes.CDLL(self.so_path)

    def run(self, name: str, buffers: Mapping[int, np.ndarray],
            static: Mapping[int, int] | None = None, merge: np.ndarray | None = None,
            log_file: str | None = None) -> None:
        """Call routine ``name``; ``buffers`` maps node id -> C-contiguous array (mutated in
        place); ``static`` maps static symbol -> value; ``log_file``: where a routine built with
        ``debug_log`` writes its log (None: it logs nothing)."""
        r = self.routines[name]
        static = static or {}
        args = []
        for _decl, src in cc_emit.kernel_params(r, self.debug_log):
            if src == "log":
                args.append(ctypes.c_char_p(log_file.encode() if log_file else None))
            elif isinstance(src, L.Node):
                a = buffers[src.id]
                assert a.flags["C_CONTIGUOUS"] and a.nbytes == src.size_in_bytes, (src, a.shape)
                args.append(ctypes.c_void_p(a.ctypes.data))
            elif isinstance(src, L.StaticSymbol):
                v = int(static[src.sym])
                if v < 0 or (src.range is not None and v >= src.range):
                    raise ValueError(f"static index {L.sym_ident(src.sym)}={v} out of range")
                args.append((ctypes.c_uint64 if cc_emit.LARGE_MODELS else ctypes.c_uint32)(v))
            else:
                args.append(ctypes.c_void_p(merge.ctypes.data))
        fn = getattr(self.lib, name)
        fn.restype = None
        fn(*args)


def run_routine(r: L.Routine, buffers: Dict[int, np.ndarray],
                static: Mapping[int, int] | None = None) -> None:
    CompiledOracle([r]).run(r.name, buffers, static)
