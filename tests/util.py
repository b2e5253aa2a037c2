"""Shared helpers of the parity tests."""
from __future__ import annotations

import torch


def rel_l2(a: torch.Tensor, b: torch.Tensor) -> float:
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))


def argmax_agreement(masked_a: torch.Tensor, masked_b: torch.Tensor) -> float:
    return float((masked_a.cpu().argmax(1) == masked_b.cpu().argmax(1)).float().mean())


def load_state(model, state):
    model.load_state_dict({k: v.clone() for k, v in state.items()})
    return model
