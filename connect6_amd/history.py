"""Grouped forward of many frozen checkpoints in one launch.

Mirrors ``HistoricalCheckpoint`` and ``HistoricalPolicyEnsemble`` of the
reference (connect6/history.py:26-32 and :186-303).  Where the reference folds
the M models into ``F.conv2d(groups=M)`` once per layer, here the M weight
sets sit side by side in one packed buffer and the fused forward kernel picks
the set from the board index -- one launch for all models and all layers.
Policy only, no masking, as in the reference.
"""
from __future__ import annotations

from dataclasses import dataclass
from pathlib import Path
from typing import Any

import torch

from . import _lib
from .model import _require_device_tensor, pack_state, run_forward, run_forward_generic


@dataclass(slots=True)
class HistoricalCheckpoint:
    path: Path
    update: int
    model_state: dict[str, torch.Tensor]
    model_config: dict[str, Any]
    game_config: dict[str, Any]


def _normalized_model_cfg(cfg: dict[str, Any]) -> dict[str, Any]:
    out = dict(cfg)
    out.pop("compile", None)
    out.pop("compile_mode", None)
    return out


_PREC_OF_DTYPE = {
    torch.float32: _lib.PREC_F32,
    torch.bfloat16: _lib.PREC_BF16,
    torch.float16: _lib.PREC_F16,
}


class HistoricalPolicyEnsemble:
    """Many frozen CNN policies evaluated together.

    Input ``[MODELS, TABLES, 3, H, W]`` -> policy logits ``[MODELS, TABLES,
    H*W]`` in the ensemble dtype.  ``dtype`` selects the arithmetic as in the
    reference's ``_history_dtype`` (connect6/train.py:133-145): float32,
    bfloat16 or float16.  ``precision`` may override it with ``"bf16x2"``.
    """

    def __init__(
        self,
        checkpoints: list[HistoricalCheckpoint],
        device: torch.device,
        *,
        dtype: torch.dtype | None = None,
        precision: str | None = None,
    ) -> None:
        if not checkpoints:
            raise ValueError("HistoricalPolicyEnsemble needs at least 1 checkpoint")
        self.device = torch.device(device)
        self.dtype = dtype or torch.float32
        if self.dtype not in _PREC_OF_DTYPE:
            raise ValueError("ensemble dtype must be one of: bfloat16 | float16 | float32")
        self.num_models = len(checkpoints)
        self.updates = [cp.update for cp in checkpoints]
        self.paths = [cp.path for cp in checkpoints]

        first_cfg = _normalized_model_cfg(checkpoints[0].model_config)
        self.board_size = int(checkpoints[0].game_config["board_size"])
        self.kernels = tuple(int(v) for v in first_cfg.get("kernels", (23, 3, 3, 3, 3, 3, 3, 3)))
        self.channels = tuple(int(v) for v in first_cfg.get("channels", (32, 32, 64, 64, 64, 96, 96, 96)))
        self.input_channels = 3
        for cp in checkpoints[1:]:
            if int(cp.game_config["board_size"]) != self.board_size:
                raise ValueError("historical checkpoints use different board sizes")
            if _normalized_model_cfg(cp.model_config) != first_cfg:
                raise ValueError("historical checkpoints have different CNN architectures")

        states = [cp.model_state for cp in checkpoints]
        # same attributes as the reference (history.py:224-233), on `device` in `dtype`
        self.conv_weights: list[torch.Tensor] = []
        self.conv_biases: list[torch.Tensor | None] = []
        for i in range(len(self.kernels)):
            self.conv_weights.append(self._stack(states, f"convs.{i}.weight"))
            self.conv_biases.append(self._stack_optional(states, f"convs.{i}.bias"))
        self.policy_weight = self._stack(states, "policy_output.weight")
        self.policy_bias = self._stack_optional(states, "policy_output.bias")
        self.action_size = self.board_size * self.board_size

        self._prec = _PREC_OF_DTYPE[self.dtype] if precision is None else _lib.PREC_BY_NAME[precision]
        self._packed: torch.Tensor | None = None
        self._states = states

    def _stack(self, states, key: str) -> torch.Tensor:
        try:
            tensor = torch.stack([state[key].detach().cpu() for state in states], dim=0)
        except KeyError as exc:
            raise KeyError(f"parameter {key} is missing from the historical checkpoints") from exc
        return tensor.to(device=self.device, dtype=self.dtype, non_blocking=True)

    def _stack_optional(self, states, key: str) -> torch.Tensor | None:
        if key not in states[0]:
            return None
        return self._stack(states, key)

    @property
    def is_default_architecture(self) -> bool:
        return (
            self.board_size == 19
            and self.kernels == (23, 3, 3, 3, 3, 3, 3, 3)
            and self.channels == (32, 32, 64, 64, 64, 96, 96, 96)
        )

    def _model_state(self, m: int) -> dict[str, torch.Tensor]:
        """Parameters of model ``m`` as the ensemble holds them (rounded to ``dtype``)."""
        state = {}
        for i in range(len(self.kernels)):
            state[f"convs.{i}.weight"] = self.conv_weights[i][m]
            if self.conv_biases[i] is not None:
                state[f"convs.{i}.bias"] = self.conv_biases[i][m]
        state["policy_output.weight"] = self.policy_weight[m]
        if self.policy_bias is not None:
            state["policy_output.bias"] = self.policy_bias[m]
        return state

    def _packed_weights(self) -> torch.Tensor:
        if self._packed is None:
            one = _lib.packed_bytes(self._prec)
            buf = torch.empty((self.num_models, one), dtype=torch.uint8, device=self.device)
            for m in range(self.num_models):
                pack_state(self._model_state(m), self._prec, buf[m])
            self._packed = buf
        return self._packed

    def forward_grouped(self, x: torch.Tensor) -> torch.Tensor:
        if x.ndim != 5:
            raise ValueError("history ensemble expects input [MODELS, TABLES, 3, H, W]")
        expected_tail = (self.input_channels, self.board_size, self.board_size)
        if x.shape[0] != self.num_models or tuple(x.shape[2:]) != expected_tail:
            raise ValueError(
                f"bad history batch {tuple(x.shape)}; expected "
                f"[{self.num_models}, T, {expected_tail[0]}, {expected_tail[1]}, {expected_tail[2]}]"
            )
        if self.device.type != "cuda":
            raise RuntimeError(
                f"ensemble device is {self.device}: connect6_amd computes only on an MI355X "
                "(HIP) device; there is no CPU path"
            )
        if x.device != self.device or x.dtype != self.dtype:
            x = x.to(device=self.device, dtype=self.dtype, non_blocking=True)
        _require_device_tensor(x, "history input")
        m, t = int(x.shape[0]), int(x.shape[1])
        if t == 0:
            return torch.empty((m, 0, self.action_size), dtype=self.dtype, device=self.device)
        if self.is_default_architecture:
            logits, _, _, _ = run_forward(x.reshape(m * t, *expected_tail), self._packed_weights(),
                                          self._prec, m, t, want_value=False)
        else:  # other architectures: layer by layer, one model after the other
            logits = torch.cat([
                run_forward_generic(x[i], self._model_state(i), self.kernels, self.channels,
                                    self._prec, want_value=False)[0]
                for i in range(m)
            ])
        logits = logits.view(m, t, self.action_size)
        return logits if self.dtype == torch.float32 else logits.to(self.dtype)
