"""Phase timestamps of the fused forward kernel.

``python -m connect6_amd.profiling --build`` compiles a copy of the library with ``-DC6_TRACE``
(``lib/libconnect6_amd_trace.so``: the kernels record the shader cycle counter at phase
boundaries of the third board of every workgroup); ``python -m connect6_amd.profiling bf16f6 bf16``
then runs B=4096 forwards on the GPU through that copy and prints, per arithmetic mode, the mean
cycles per phase over all workgroups and waves and the shader clock during the traced board.
The shipped library contains none of this.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
import sys
from pathlib import Path

from . import _lib

TRACE_SO = _lib._LIBDIR / "libconnect6_amd_trace.so"

# marks of the pipelined kernel (c6_forward.hip, C6_MARK): per 3x3 layer l = 1..7 (the 2nd..8th
# convolution): start of its K-loop, end of the phases in front of its low-order pass, end of that
# pass, end of its last phase
_PIPE_MARKS = [0, 1, 2] + sum([[3 if l == 1 else 3 + 2 * l, 30 + l, 40 + l, 4 + 2 * l] for l in range(1, 8)], []) + [19, 20]
_PIPE_NAMES = ["stage input", "conv1 K-loop"] + sum(
    [[f"conv{l} -> conv{l + 1} boundary", f"conv{l + 1} phases before the low-order pass",
      f"conv{l + 1} low-order pass", f"conv{l + 1} last phase (parts A, B)"] for l in range(1, 8)], []) + ["heads", "write out"]


def build_traced() -> Path:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-DC6_TRACE",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-function",
           "-o", str(TRACE_SO)] + [str(_lib._CSRC / s) for s in _lib._SOURCES]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise _lib.C6Error(f"hipcc failed ({proc.returncode}):\n{proc.stderr[-4000:]}")
    return TRACE_SO


def phase_table(precision: str, batch: int = 4096, launches: int = 150) -> str:
    """Run `launches` forwards of `batch` boards through the traced library and format the marks
    of the last one.  Must be the first use of the library in the process."""
    import numpy as np
    import torch

    if not TRACE_SO.exists():
        raise _lib.C6Error(f"{TRACE_SO} is missing: python -m connect6_amd.profiling --build")
    if _lib._lib is not None and Path(_lib._SO) != TRACE_SO:
        raise _lib.C6Error("the untraced library is already loaded in this process")
    _lib._SO = TRACE_SO
    import connect6_amd as c6
    from connect6_amd.synthetic import gen_boards

    dev = torch.device("cuda:0")
    lib = c6.load()
    lib.c6_debug_trace.restype = ctypes.c_int
    lib.c6_debug_trace.argtypes = [ctypes.c_void_p]
    torch.manual_seed(1234)
    model = c6.PolicyValueNet().to(dev).eval()
    model.precision = precision
    x = gen_boards(batch, 200, 2025)[0].to(dev)
    with torch.inference_mode():
        for _ in range(launches):
            model.forward_masked(x)
    torch.cuda.synchronize()
    buf = np.zeros(256 * 4 * 64, dtype=np.int64)
    rc = lib.c6_debug_trace(buf.ctypes.data_as(ctypes.c_void_p))
    if rc != 0:
        raise _lib.C6Error(f"c6_debug_trace failed with HIP error {rc}")
    raw = buf.reshape(256, 4, 64).astype(np.float64)
    if precision not in ("bf16f6", "bf16", "fp16"):
        raise _lib.C6Error("phase names are defined for the pipelined kernel (bf16f6, bf16, fp16)")
    t = raw[:, :, _PIPE_MARKS]
    d = np.diff(t, axis=2)
    tot = t[:, :, -1] - t[:, :, 0]
    seconds = (raw[:, :, 51] - raw[:, :, 50]) / 100e6     # the constant 100 MHz counter at marks 0 and 20
    lines = [f"{precision}: one board = {tot.mean():.0f} shader cycles (min {tot.min():.0f}, max {tot.max():.0f} over "
             f"256 workgroups x 4 waves) = {seconds.mean() * 1e6:.1f} us at {(tot / seconds).mean() / 1e9:.3f} GHz",
             "", "| phase | cycles | % |", "|---|---|---|"]
    mean = d.mean(axis=(0, 1))
    for name, v in zip(_PIPE_NAMES, mean):
        lines.append(f"| {name} | {v:.0f} | {100 * v / tot.mean():.1f} |")
    return "\n".join(lines)


def main(argv: list[str]) -> int:
    if argv and argv[0] == "--build":
        print(build_traced())
        return 0
    for i, prec in enumerate(argv or ["bf16f6"]):
        if i:   # one process per mode keeps every run the library's first use
            out = subprocess.run([sys.executable, "-m", "connect6_amd.profiling", prec], capture_output=True, text=True)
            print(out.stdout.rstrip() or out.stderr[-2000:])
        else:
            print(phase_table(prec))
        print()
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
