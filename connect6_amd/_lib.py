"""Build and load ``libconnect6_amd.so`` (hand-written HIP for gfx950) via ctypes.

The library is the only compute backend of this package: there is no PyTorch
or CPU fallback.  ``load()`` raises if the shared object is missing.
"""
from __future__ import annotations

import ctypes
import os
import re
import subprocess
import warnings
from pathlib import Path

_PKG = Path(__file__).resolve().parent
_CSRC = _PKG / "csrc"
_LIBDIR = _PKG / "lib"
_SO = _LIBDIR / "libconnect6_amd.so"
_SOURCES = ("c6_forward.hip", "c6_tail.hip", "c6_generic.hip", "c6_env.hip", "c6_api.hip")
_RESOURCES = _LIBDIR / "resource_usage.txt"   # registers, scratch and LDS of every kernel, written by build()

# arithmetic modes (include/connect6_amd.h)
PREC_F32, PREC_BF16, PREC_F16, PREC_BF16F6, PREC_BF16C, PREC_BF16F6W, PREC_BF16C6 = 0, 1, 2, 3, 4, 5, 6
PREC_BY_NAME = {"fp32": PREC_F32, "bf16": PREC_BF16, "fp16": PREC_F16, "bf16f6": PREC_BF16F6, "bf16c": PREC_BF16C,
                "bf16f6w": PREC_BF16F6W, "bf16c6": PREC_BF16C6}
CASCADES = (PREC_BF16C, PREC_BF16C6)   # the modes that go through the cascade entry points
# cascade mode: a board is evaluated a second time (low parts of activations and weights carried) when its best free
# square leads the second best by less than this many standard deviations of its logits, or two
# other free squares lie within twice that.  The plain pass's error on a difference of two logits
# has a standard deviation of about 0.01 standard deviations of the logits: the threshold is two
# of those.
CASCADE_THRESHOLD = 0.02
DT_F32, DT_BF16, DT_F16 = 0, 1, 2
MASK_NONE, MASK_INPUT, MASK_LEGAL = 0, 1, 2

# every symbol include/connect6_amd.h declares
EXPORTS = (
    "c6_version",
    "c6_last_error",
    "c6_packed_bytes",
    "c6_pack_weights",
    "c6_pack_weights_grouped",
    "c6_forward",
    "c6_forward_boards",
    "c6_cascade_workspace_bytes",
    "c6_forward_cascade",
    "c6_forward_boards_cascade",
    "c6_generic_workspace_bytes",
    "c6_forward_generic",
    "c6_forward_generic_grouped",
    "c6_forward_generic_static",
    "c6_mask_logits",
    "c6_softmax_sample",
    "c6_d4_expand",
    "c6_d4_reduce",
    "c6_env_step",
    "c6_canonical_input",
)


class C6Error(RuntimeError):
    pass


def build(verbose: bool = False) -> Path:
    """Compile the HIP sources for gfx950 into ``lib/libconnect6_amd.so``."""
    _LIBDIR.mkdir(exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [
        hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
        # packed-fp32 VALU forms are disabled for every kernel in this library
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        "-Wall", "-Wno-unused-function",
        "-Rpass-analysis=kernel-resource-usage",
        "-o", str(_SO),
    ] + [str(_CSRC / s) for s in _SOURCES]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    remarks, other = [], []
    excerpt = 0   # a resource-usage remark is followed by a source excerpt of two lines: drop those
    for line in proc.stderr.splitlines():   # (and only those: excerpts of errors and warnings stay)
        if "-Rpass-analysis=kernel-resource-usage" in line:
            remarks.append(line)
            excerpt = 2
        elif excerpt and re.match(r"\s*\d*\s*\|", line):
            excerpt -= 1
        else:
            excerpt = 0
            other.append(line)
    if verbose or proc.returncode != 0:
        print(proc.stdout)
        print("\n".join(other))
    if proc.returncode != 0:
        raise C6Error(f"hipcc failed ({proc.returncode}):\n" + "\n".join(other)[-4000:])
    _RESOURCES.write_text("\n".join(r.split("remark:", 1)[1].rsplit("[", 1)[0].rstrip() for r in remarks) + "\n")
    try:   # the probe is a measurement aid of bench.py, not part of the library
        build_probe()
    except C6Error as exc:
        warnings.warn(f"the MFMA probe did not build (bench.py will report it as missing): {exc}")
    return _SO


_PROBE_SO = _LIBDIR / "libc6_probe.so"


def build_probe() -> Path:
    """Compile the measurement aid ``csrc/probe/mfma_probe.hip`` (sustained bf16 MFMA rate of
    the GPU, used by bench.py only) into ``lib/libc6_probe.so``."""
    _LIBDIR.mkdir(exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-o", str(_PROBE_SO), str(_CSRC / "probe" / "mfma_probe.hip")]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise C6Error(f"hipcc failed ({proc.returncode}):\n{proc.stderr[-4000:]}")
    return _PROBE_SO


def probe_mfma_rate(iters: int = 60000, zero_operands: bool = False) -> dict[str, float]:
    """Sustained rate of back-to-back bf16 MFMAs on every CU of the current GPU (random operand
    bits unless ``zero_operands``), and the shader clock the card holds under that load."""
    if not _PROBE_SO.exists():
        raise C6Error(f"{_PROBE_SO} is missing: build it with connect6_amd.build()")
    lib = ctypes.CDLL(str(_PROBE_SO))
    dbl = ctypes.POINTER(ctypes.c_double)
    lib.c6_probe_mfma_rate.restype = ctypes.c_int
    lib.c6_probe_mfma_rate.argtypes = [ctypes.c_int, ctypes.c_int, dbl, dbl, dbl]
    tf, ghz, cyc = ctypes.c_double(), ctypes.c_double(), ctypes.c_double()
    rc = lib.c6_probe_mfma_rate(iters, int(zero_operands), ctypes.byref(tf), ctypes.byref(ghz), ctypes.byref(cyc))
    if rc != 0:
        raise C6Error(f"c6_probe_mfma_rate failed with HIP error {rc}")
    return {"tflops": tf.value, "clock_ghz": ghz.value, "cycles_per_mfma": cyc.value}


def resource_usage(rebuild_if_missing: bool = True) -> dict[str, dict[str, int]]:
    """Per kernel (mangled name): registers, scratch bytes per lane, spills and LDS as the
    compiler reported them in the last ``build()``."""
    if not _RESOURCES.exists():
        if not rebuild_if_missing:
            raise C6Error(f"{_RESOURCES} is missing: run connect6_amd.build()")
        build()
    out: dict[str, dict[str, int]] = {}
    cur = None
    for line in _RESOURCES.read_text().splitlines():
        key, _, val = line.strip().partition(":")
        key = key.strip()
        if key == "Function Name":
            cur = out.setdefault(val.strip(), {})
        elif cur is not None and val.strip().lstrip("-").isdigit():
            cur[key.split(" [")[0]] = int(val)
    return out


_lib = None


def load() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not _SO.exists():
        raise C6Error(
            f"{_SO} is missing: build it with connect6_amd.build() "
            "(hipcc --offload-arch=gfx950); there is no fallback path"
        )
    lib = ctypes.CDLL(str(_SO))
    vp, i32, i64, f32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float
    lib.c6_version.restype = i32
    lib.c6_version.argtypes = []
    lib.c6_last_error.restype = ctypes.c_char_p
    lib.c6_last_error.argtypes = []
    lib.c6_packed_bytes.restype = i32
    lib.c6_packed_bytes.argtypes = [i32, ctypes.POINTER(ctypes.c_size_t)]
    lib.c6_pack_weights.restype = i32
    lib.c6_pack_weights.argtypes = [ctypes.POINTER(vp), ctypes.POINTER(vp), vp, vp, vp, vp, i32, vp, vp]
    lib.c6_forward.restype = i32
    lib.c6_forward.argtypes = [vp, i32, i64, i64, vp, ctypes.c_size_t, i32, vp, vp, i32, vp, f32,
                               vp, f32, vp, vp, vp]
    lib.c6_forward_boards.restype = i32
    lib.c6_forward_boards.argtypes = [vp, vp, vp, i64, vp, i32, i64, vp, i32, vp, vp, i32, f32, vp, f32,
                                      vp, vp, vp]
    lib.c6_cascade_workspace_bytes.restype = i32
    lib.c6_cascade_workspace_bytes.argtypes = [i64, ctypes.POINTER(ctypes.c_size_t)]
    lib.c6_forward_cascade.restype = i32
    lib.c6_pack_weights_grouped.restype = i32
    lib.c6_pack_weights_grouped.argtypes = [ctypes.POINTER(vp), ctypes.POINTER(vp), vp, vp, vp, vp, i64, i32, vp,
                                            ctypes.c_size_t, vp]
    lib.c6_forward_cascade.argtypes = [vp, i32, i64, i64, vp, ctypes.c_size_t, i32, vp, i32, vp, i32, vp, f32,
                                       vp, f32, vp, vp, f32, vp, ctypes.c_size_t, vp]
    lib.c6_forward_boards_cascade.restype = i32
    lib.c6_forward_boards_cascade.argtypes = [vp, vp, vp, i64, vp, i32, i64, vp, i32, vp, i32, vp, i32, f32, vp, f32,
                                              vp, vp, f32, vp, ctypes.c_size_t, vp]
    ip = ctypes.POINTER(ctypes.c_int)
    lib.c6_generic_workspace_bytes.restype = i32
    lib.c6_generic_workspace_bytes.argtypes = [i64, i32, i32, ip, ctypes.POINTER(ctypes.c_size_t)]
    lib.c6_forward_generic.restype = i32
    lib.c6_forward_generic.argtypes = [vp, i32, i64, i32, i32, ip, ip, ctypes.POINTER(vp),
                                       ctypes.POINTER(vp), vp, vp, vp, vp, i32, vp,
                                       ctypes.c_size_t, vp, vp, i32, vp, f32, vp]
    lib.c6_forward_generic_grouped.restype = i32
    lib.c6_forward_generic_grouped.argtypes = [vp, i32, i64, i64, i32, i32, ip, ip, ctypes.POINTER(vp),
                                               ctypes.POINTER(vp), vp, vp, vp, vp, i32, vp,
                                               ctypes.c_size_t, vp, vp, i32, vp, f32, vp]
    lib.c6_forward_generic_static.restype = i32
    lib.c6_forward_generic_static.argtypes = [vp, i32, i64, i32, i32, ip, ip, ctypes.POINTER(vp),
                                              ctypes.POINTER(vp), vp, vp, vp, vp, i32, vp, vp,
                                              i32, vp, f32, vp]
    lib.c6_mask_logits.restype = i32
    lib.c6_mask_logits.argtypes = [vp, vp, i32, i64, ctypes.c_uint32, vp, vp]
    lib.c6_softmax_sample.restype = i32
    lib.c6_softmax_sample.argtypes = [vp, vp, vp, f32, i64, vp, vp, vp]
    lib.c6_d4_expand.restype = i32
    lib.c6_d4_expand.argtypes = [vp, i32, i64, vp, vp]
    lib.c6_d4_reduce.restype = i32
    lib.c6_d4_reduce.argtypes = [vp, vp, i64, vp, vp, vp]
    lib.c6_env_step.restype = i32
    lib.c6_env_step.argtypes = [vp, vp, vp, vp, vp, vp, i32, i64, i32, i32, vp, vp, vp, vp, vp, vp]
    lib.c6_canonical_input.restype = i32
    lib.c6_canonical_input.argtypes = [vp, vp, vp, i64, i32, vp, vp]
    _lib = lib
    return lib


def check(rc: int, what: str) -> None:
    """Map a library return code to the exception the reference would raise:
    bad shapes/dtypes are ValueError (connect6/model.py:98-102), anything the
    device reports is RuntimeError."""
    if rc == 0:
        return
    msg = load().c6_last_error().decode("utf-8", "replace")
    if rc == -1:
        raise ValueError(f"{what}: {msg}")
    raise C6Error(f"{what}: {msg} (code {rc})")


def packed_bytes(prec: int) -> int:
    n = ctypes.c_size_t(0)
    check(load().c6_packed_bytes(prec, ctypes.byref(n)), "c6_packed_bytes")
    return int(n.value)


def cascade_workspace_bytes(boards: int) -> int:
    n = ctypes.c_size_t(0)
    check(load().c6_cascade_workspace_bytes(int(boards), ctypes.byref(n)), "c6_cascade_workspace_bytes")
    return int(n.value)


def torch_dtype_code(dtype) -> int:
    import torch

    if dtype == torch.float32:
        return DT_F32
    if dtype == torch.bfloat16:
        return DT_BF16
    if dtype == torch.float16:
        return DT_F16
    raise ValueError(f"unsupported tensor dtype {dtype}; expected float32, bfloat16 or float16")


def stream_ptr(device) -> int:
    import torch

    return int(torch.cuda.current_stream(device).cuda_stream)
