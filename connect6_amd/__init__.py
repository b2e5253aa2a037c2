"""connect6_amd: the Connect6 policy/value CNN forward path on MI355X (gfx950).

Host-side mirror of the reference's operator interface for this path
(connect6/model.py and connect6/history.py:186-303) over a C-ABI library of
hand-written HIP kernels.
"""
from ._lib import C6Error, build, load
from .history import HistoricalCheckpoint, HistoricalPolicyEnsemble
from .model import PolicyValueNet, build_model, mask_logits
from .selfplay import (
    d4_expand,
    d4_reduce,
    evaluate_d4,
    inverse_transform_actions,
    sample_actions,
    symmetry_for_phase,
    transform_actions,
    transform_boards,
)

__all__ = [
    "C6Error",
    "HistoricalCheckpoint",
    "HistoricalPolicyEnsemble",
    "PolicyValueNet",
    "build",
    "build_model",
    "d4_expand",
    "d4_reduce",
    "evaluate_d4",
    "inverse_transform_actions",
    "load",
    "mask_logits",
    "sample_actions",
    "symmetry_for_phase",
    "transform_actions",
    "transform_boards",
]
