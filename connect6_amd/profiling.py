"""Phase timestamps of the fused forward kernel.

``python -m connect6_amd.profiling --build`` compiles a copy of the library with ``-DC6_TRACE``
(``lib/libconnect6_amd_trace.so``: the kernels record the shader cycle counter at phase
boundaries of the third board of every workgroup); ``python -m connect6_amd.profiling bf16f6 bf16``
then runs B=4096 forwards on the GPU through that copy and prints, per arithmetic mode, the mean
cycles per phase over all workgroups and waves and the shader clock during the traced board.
The shipped library contains none of this.

``python -m connect6_amd.profiling --threshold-sweep`` (the ordinary library) prints, for a range
of cascade thresholds, how many boards are evaluated twice and what that costs in argmax agreement
with the fp32 kernel, over 32 random networks of either initialisation.

``python -m connect6_amd.profiling --build-ablations`` compiles further traced copies (the
corrected mode without the low-order pass of some layers; with idle cycles added) and
``python -m connect6_amd.profiling --ablations`` measures them back to back: cycles per board, shader
clock, time per launch, agreement with fp32.
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


def _traced_build_command(out: Path, defines=()) -> list[str]:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    return ([hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-DC6_TRACE"]
            + [f"-D{d}" for d in defines]
            + ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-function",
               "-o", str(out)] + [str(_lib._CSRC / s) for s in _lib._SOURCES])


def build_traced() -> Path:
    proc = subprocess.run(_traced_build_command(TRACE_SO), capture_output=True, text=True)
    if proc.returncode != 0:
        raise _lib.C6Error(f"hipcc failed ({proc.returncode}):\n{proc.stderr[-4000:]}")
    return TRACE_SO


# Ablation copies of the traced library: the corrected mode ("bf16f6") with the low-order pass of
# some layers left out (their results then differ: these price the layers, they are not modes),
# and with idle cycles added at every layer end.  name -> (what it is, extra compiler defines)
ABLATIONS = {
    "all": ("low-order pass on the input of every 3x3 layer (the library as shipped)", ()),
    "no8": ("without the last layer's", ("C6_LO_MASK=0x7e",)),
    "no78": ("without the last two layers'", ("C6_LO_MASK=0x3e",)),
    "no678": ("without the last three layers'", ("C6_LO_MASK=0x1e",)),
    "no23": ("without layers 2 and 3", ("C6_LO_MASK=0xf8",)),
    "none": ("no low-order pass, no low-order part computed (bf16 arithmetic in this mode's record layout)",
             ("C6_LO_MASK=0x00",)),
    "idle": ("every layer, plus 40 x 64 idle cycles at the end of each 3x3 layer", ("C6_IDLE_PER_LAYER=40",)),
}


def _ablation_so(name: str) -> Path:
    return TRACE_SO if name == "all" else _lib._LIBDIR / f"libconnect6_amd_trace_{name}.so"


def build_ablations(jobs: int = 4) -> list[Path]:
    """Compile every ablation copy (``jobs`` compilers at a time; each takes a few minutes)."""
    pending = [(n, subprocess.Popen(_traced_build_command(_ablation_so(n), ABLATIONS[n][1]), stdout=subprocess.PIPE,
                                    stderr=subprocess.PIPE, text=True)) for n in list(ABLATIONS)[:jobs]]
    todo = list(ABLATIONS)[jobs:]
    built = []
    while pending:
        name, proc = pending.pop(0)
        _, err = proc.communicate()
        if proc.returncode != 0:
            raise _lib.C6Error(f"hipcc failed for ablation {name} ({proc.returncode}):\n{err[-4000:]}")
        built.append(_ablation_so(name))
        if todo:
            n = todo.pop(0)
            pending.append((n, subprocess.Popen(_traced_build_command(_ablation_so(n), ABLATIONS[n][1]),
                                                stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)))
    return built


def ablation_row(name: str, batch: int = 4096, launches: int = 150) -> str:
    """One row of the ablation table, measured in this process (which must not have loaded the
    library yet): cycles per board and shader clock from the traced board, time per launch from
    HIP events over the last 20 launches, argmax agreement with the fp32 kernel."""
    import numpy as np
    import torch

    global TRACE_SO
    TRACE_SO = _ablation_so(name)
    table = phase_table("bf16f6", batch=batch, launches=launches)
    head = table.splitlines()[0]
    import connect6_amd as c6
    from connect6_amd.synthetic import gen_boards

    dev = torch.device("cuda:0")
    torch.manual_seed(1234)
    model = c6.PolicyValueNet().to(dev).eval()
    x = gen_boards(batch, 200, 2025)[0].to(dev)
    with torch.inference_mode():
        model.precision = "fp32"
        want = model.forward_masked(x)[0].argmax(1)
        model.precision = "bf16f6"
        got = model.forward_masked(x)[0].argmax(1)
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(20)]
        for a, b in evs:
            a.record()
            model.forward_masked(x)
            b.record()
        torch.cuda.synchronize()
    ms = float(np.mean([a.elapsed_time(b) for a, b in evs]))
    cycles = head.split("one board = ")[1].split(" shader")[0]
    clock = head.rsplit(" at ", 1)[1]
    agree = float((got == want).float().mean())
    return (f"| {name} | {ABLATIONS[name][0]} | {cycles} | {clock} | {ms:.4f} | "
            f"{batch * 269554368 / (ms * 1e-3) / 2.5e15 * 100:.1f} | {agree:.4f} |")


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
    if precision not in ("bf16f6w", "bf16f6", "bf16", "fp16"):
        raise _lib.C6Error("phase names are defined for the pipelined kernel (bf16f6w, bf16f6, bf16, fp16)")
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


def threshold_sweep(thresholds=(0.01, 0.015, 0.02, 0.025, 0.03, 0.04), seeds=range(1000, 1032), batch: int = 4096) -> str:
    """Cascade mode: boards evaluated twice and argmax agreement with the fp32 kernel per
    threshold, beside the second pass's arithmetic on every board (bf16f6w), the activation
    correction alone (bf16f6) and plain bf16."""
    import torch

    import connect6_amd as c6
    from connect6_amd.synthetic import gen_boards

    dev = torch.device("cuda:0")
    lines = []
    for stones in (200, 20):
        x = gen_boards(batch, stones, 2025 + stones)[0].to(dev)
        for init in ("reference", "torch_default"):
            acc = {t: [] for t in thresholds}
            frac = {t: [] for t in thresholds}
            other = {"bf16f6w": [], "bf16f6": [], "bf16": []}
            for seed in seeds:
                torch.manual_seed(seed)
                m = c6.PolicyValueNet().to(dev).eval()
                if init == "torch_default":
                    for mod in m.modules():
                        if isinstance(mod, torch.nn.Conv2d):
                            mod.reset_parameters()
                    m.refresh_weights()
                with torch.inference_mode():
                    m.precision = "fp32"
                    want = m.forward_masked(x)[0].argmax(1)
                    agree = lambda: float((m.forward_masked(x)[0].argmax(1) == want).float().mean())
                    for name in other:
                        m.precision = name
                        other[name].append(agree())
                    m.precision = "bf16c"
                    for t in thresholds:
                        m.cascade_threshold = t
                        acc[t].append(agree())
                        frac[t].append(int(m.cascade_stats["second_pass"].item()) / batch)
            o = {k: torch.tensor(v) for k, v in other.items()}
            lines += [f"stones <= {stones}, {init} initialisation, {len(o['bf16'])} networks x {batch} boards; argmax agreement "
                      f"with fp32, mean (worst network): bf16f6w {o['bf16f6w'].mean():.4f} ({o['bf16f6w'].min():.4f}), "
                      f"bf16f6 {o['bf16f6'].mean():.4f} ({o['bf16f6'].min():.4f}), bf16 {o['bf16'].mean():.4f} ({o['bf16'].min():.4f})",
                      "", "| threshold | evaluated twice, mean (max) | agreement, mean | worst network | networks under 99 % | under 99.5 % |",
                      "|---|---|---|---|---|---|"]
            for t in thresholds:
                a, f = torch.tensor(acc[t]), torch.tensor(frac[t])
                lines.append(f"| {t:g} | {f.mean():.3f} ({f.max():.3f}) | {a.mean():.4f} | {a.min():.4f} | "
                             f"{int((a < 0.99).sum())} / {len(a)} | {int((a < 0.995).sum())} / {len(a)} |")
            lines.append("")
    return "\n".join(lines)


def main(argv: list[str]) -> int:
    if argv and argv[0] == "--build":
        print(build_traced())
        return 0
    if argv and argv[0] == "--threshold-sweep":
        print(threshold_sweep())
        return 0
    if argv and argv[0] == "--build-ablations":
        for so in build_ablations():
            print(so)
        return 0
    if argv and argv[0] == "--ablation-row":
        print(ablation_row(argv[1]))
        return 0
    if argv and argv[0] == "--ablations":
        print("| build | low-order passes | cycles per board | shader clock | ms per 4096 boards | % of 2.5 PFLOP/s | argmax agreement with fp32 |")
        print("|---|---|---|---|---|---|---|")
        for name in ABLATIONS:   # one process per copy: each must be the first library the process loads
            out = subprocess.run([sys.executable, "-m", "connect6_amd.profiling", "--ablation-row", name],
                                 capture_output=True, text=True)
            print(out.stdout.strip().splitlines()[-1] if out.returncode == 0 and out.stdout.strip() else
                  f"| {name} | failed: {out.stderr[-300:]!r} | | | | | |")
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
