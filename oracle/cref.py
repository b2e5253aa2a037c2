"""ctypes binding of ``conv_ref.c`` (test infrastructure only)."""
from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path

import numpy as np
import torch

_HERE = Path(__file__).resolve().parent
_SO = _HERE / "_build" / "libc6ref.so"


def build(force: bool = False) -> Path:
    if force or not _SO.exists():
        subprocess.run(["make", "-C", str(_HERE), "-B" if force else "-s", "all"], check=True)
    return _SO


def _fp(a: np.ndarray):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def forward(state, x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Brute-force forward of the network described by ``state`` on x[B,Cin,n,n]."""
    lib = ctypes.CDLL(str(build()))
    lib.c6ref_forward.restype = ctypes.c_int
    layers = 0
    while f"convs.{layers}.weight" in state:
        layers += 1
    ws = [state[f"convs.{i}.weight"].detach().float().contiguous().numpy() for i in range(layers)]
    bs = [state[f"convs.{i}.bias"].detach().float().contiguous().numpy() for i in range(layers)]
    kernels = (ctypes.c_int * layers)(*[int(w.shape[-1]) for w in ws])
    channels = (ctypes.c_int * layers)(*[int(w.shape[0]) for w in ws])
    conv_w = np.concatenate([w.ravel() for w in ws]).astype(np.float32)
    conv_b = np.concatenate([b.ravel() for b in bs]).astype(np.float32)
    pw = state["policy_output.weight"].detach().float().contiguous().numpy().ravel().copy()
    pb = state["policy_output.bias"].detach().float().contiguous().numpy().ravel().copy()
    vw = state["value_output.weight"].detach().float().contiguous().numpy().ravel().copy()
    vb = state["value_output.bias"].detach().float().contiguous().numpy().ravel().copy()
    xn = np.ascontiguousarray(x.detach().float().numpy())
    b, cin, n, _ = xn.shape
    logits = np.zeros((b, n * n), dtype=np.float32)
    value = np.zeros((b,), dtype=np.float32)
    rc = lib.c6ref_forward(_fp(xn), ctypes.c_long(b), n, cin, layers, kernels, channels,
                           _fp(conv_w), _fp(conv_b), _fp(pw), _fp(pb), _fp(vw), _fp(vb),
                           _fp(logits), _fp(value))
    if rc != 0:
        raise RuntimeError(f"c6ref_forward failed with {rc}")
    return torch.from_numpy(logits), torch.from_numpy(value)
