"""connect6_amd: the Connect6 policy/value CNN forward path on MI355X (gfx950).

Host-side mirror of the reference's operator interface for this path
(connect6/model.py, connect6/history.py:186-303 and connect6/vector_env.py) over
a C-ABI library of hand-written HIP kernels.
"""
from ._lib import CASCADE_THRESHOLD, C6Error, build, load, probe_mfma_rate
from .history import HistoricalCheckpoint, HistoricalPolicyEnsemble, history_dtype
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
from .vector_env import StepBatch, VectorConnect6, canonical_network_input, canonical_observation

__all__ = [
    "CASCADE_THRESHOLD",
    "C6Error",
    "HistoricalCheckpoint",
    "HistoricalPolicyEnsemble",
    "PolicyValueNet",
    "StepBatch",
    "VectorConnect6",
    "build",
    "build_model",
    "canonical_network_input",
    "canonical_observation",
    "d4_expand",
    "d4_reduce",
    "evaluate_d4",
    "history_dtype",
    "inverse_transform_actions",
    "load",
    "mask_logits",
    "probe_mfma_rate",
    "sample_actions",
    "symmetry_for_phase",
    "transform_actions",
    "transform_boards",
]
