"""Collector-side helpers around the forward: sampling and D4 views.

Mirrors the small pure functions of the reference's connect6/train.py that the
forward path's callers use: ``_sample_actions`` (:195-213),
``_symmetry_for_phase`` (:216-219), ``_transform_boards`` (:222-230),
``_transform_actions`` (:233-253) and ``_inverse_transform_actions``
(:256-277).  The batched pieces (sampling, the 8-view gather and the
inverse-map-and-average) are HIP kernels; the scalar index maps are integer
tensor arithmetic.
"""
from __future__ import annotations

import torch

from . import _lib
from .model import _require_device_tensor


def symmetry_for_phase(phase: int) -> tuple[int, bool]:
    """Eight-step D4 cycle: 0/90/180/270 degrees, then the same four mirrored."""
    phase = int(phase) % 8
    return phase % 4, phase >= 4


def transform_actions(actions: torch.Tensor, board_size: int, k: int, flip: bool) -> torch.Tensor:
    """Map canonical actions into the coordinates of ``transform_boards``."""
    n = int(board_size)
    k = int(k) % 4
    r = torch.div(actions, n, rounding_mode="floor")
    c = actions.remainder(n)
    if k == 1:
        r, c = n - 1 - c, r
    elif k == 2:
        r, c = n - 1 - r, n - 1 - c
    elif k == 3:
        r, c = c, n - 1 - r
    if flip:
        c = n - 1 - c
    return r * n + c


def inverse_transform_actions(actions: torch.Tensor, board_size: int, k: int, flip: bool) -> torch.Tensor:
    """Map policy-view actions back into canonical coordinates: undo the
    mirror first, then the rotation."""
    n = int(board_size)
    k = int(k) % 4
    r = torch.div(actions, n, rounding_mode="floor")
    c = actions.remainder(n)
    if flip:
        c = n - 1 - c
    if k == 1:
        r, c = c, n - 1 - r
    elif k == 2:
        r, c = n - 1 - r, n - 1 - c
    elif k == 3:
        r, c = n - 1 - c, r
    return r * n + c


def transform_boards(boards: torch.Tensor, k: int, flip: bool) -> torch.Tensor:
    """One D4 view of ``[..., n, n]`` boards: rotate by ``k`` quarter turns,
    then mirror the columns -- a gather through ``inverse_transform_actions``."""
    n = int(boards.shape[-1])
    src = inverse_transform_actions(torch.arange(n * n, device=boards.device), n, k, flip)
    flat = boards.reshape(*boards.shape[:-2], n * n)
    return flat.index_select(-1, src).reshape(boards.shape)


def sample_actions(
    logits: torch.Tensor,
    legal: torch.Tensor | None,
    temperature: float,
    u: torch.Tensor,
    return_logprob: bool = True,
):
    """Categorical draw from ``mask_logits(logits.float(), legal) / max(T, 1e-4)``
    by inverse CDF on the supplied uniforms ``u[B]`` (one HIP kernel, one wave
    per board).  Returns ``(actions, logprob)`` or only ``actions``."""
    _require_device_tensor(logits, "logits")
    if logits.ndim != 2 or logits.shape[1] != 361:
        raise ValueError(f"logits must have shape [B, 361], got {tuple(logits.shape)}")
    lib = _lib.load()
    dev = logits.device
    src = logits.float().contiguous()
    b = int(src.shape[0])
    if legal is not None:
        if legal.shape != src.shape or legal.dtype != torch.bool:
            raise ValueError("legal must be a bool tensor of the logits' shape")
        legal = legal.to(dev).contiguous().view(torch.uint8)
    u = u.to(device=dev, dtype=torch.float32).contiguous()
    if u.shape != (b,):
        raise ValueError(f"u must have shape ({b},), got {tuple(u.shape)}")
    actions = torch.empty((b,), dtype=torch.int64, device=dev)
    logprob = torch.empty((b,), dtype=torch.float32, device=dev) if return_logprob else None
    with torch.cuda.device(dev):
        rc = lib.c6_softmax_sample(src.data_ptr(), legal.data_ptr() if legal is not None else None,
                                   u.data_ptr(), float(temperature), b, actions.data_ptr(),
                                   logprob.data_ptr() if logprob is not None else None,
                                   _lib.stream_ptr(dev))
    _lib.check(rc, "c6_softmax_sample")
    return (actions, logprob) if return_logprob else actions


def d4_expand(x: torch.Tensor) -> torch.Tensor:
    """``[B,3,19,19]`` -> ``[8,B,3,19,19]``; view ``p`` equals
    ``transform_boards(x, *symmetry_for_phase(p))``."""
    _require_device_tensor(x, "boards")
    if x.ndim != 4 or tuple(x.shape[1:]) != (3, 19, 19):
        raise ValueError(f"boards must have shape [B, 3, 19, 19], got {tuple(x.shape)}")
    lib = _lib.load()
    x = x.contiguous()
    out = torch.empty((8,) + tuple(x.shape), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        rc = lib.c6_d4_expand(x.data_ptr(), _lib.torch_dtype_code(x.dtype), int(x.shape[0]),
                              out.data_ptr(), _lib.stream_ptr(x.device))
    _lib.check(rc, "c6_d4_expand")
    return out


def d4_reduce(view_logits: torch.Tensor, view_values: torch.Tensor | None):
    """``[8,B,361]`` view logits (+ ``[8,B]`` values) -> logits mapped back to
    the canonical orientation and averaged over the views (+ mean values)."""
    _require_device_tensor(view_logits, "view logits")
    if view_logits.ndim != 3 or view_logits.shape[0] != 8 or view_logits.shape[2] != 361:
        raise ValueError(f"view logits must have shape [8, B, 361], got {tuple(view_logits.shape)}")
    lib = _lib.load()
    dev = view_logits.device
    vl = view_logits.float().contiguous()
    b = int(vl.shape[1])
    vv = None
    if view_values is not None:
        if tuple(view_values.shape) != (8, b):
            raise ValueError(f"view values must have shape [8, {b}], got {tuple(view_values.shape)}")
        vv = view_values.float().contiguous()
    logits = torch.empty((b, 361), dtype=torch.float32, device=dev)
    values = torch.empty((b,), dtype=torch.float32, device=dev) if vv is not None else None
    with torch.cuda.device(dev):
        rc = lib.c6_d4_reduce(vl.data_ptr(), vv.data_ptr() if vv is not None else None, b,
                              logits.data_ptr(), values.data_ptr() if values is not None else None,
                              _lib.stream_ptr(dev))
    _lib.check(rc, "c6_d4_reduce")
    return logits, values


def evaluate_d4(model, x: torch.Tensor):
    """Evaluate every board in its 8 rotations/reflections in one batched
    forward and average the policy logits (mapped back to the canonical
    orientation) and the values over the views."""
    views = d4_expand(x)
    b = int(x.shape[0])
    logits, value = model(views.view(8 * b, 3, 19, 19))
    return d4_reduce(logits.view(8, b, 361), value.view(8, b))
