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


# bfloat16 selects the cascade (plain bf16 layer boundaries, then the boards whose decision is
# close again with the low parts of activations and weights carried), the fastest bf16 mode that
# keeps the argmax of fp32; the literal "round everything to bf16" arithmetic stays available as
# precision="bf16", the corrections on every board as precision="bf16f6" / "bf16f6w".
_PREC_OF_DTYPE = {
    torch.float32: _lib.PREC_F32,
    torch.bfloat16: _lib.PREC_BF16C6,   # (parameters held in bf16 have no low part: the second pass is bf16f6)
    torch.float16: _lib.PREC_F16,
}


def history_dtype(device: torch.device, dtype_name: str) -> torch.dtype:
    """Ensemble dtype from the config's ``historical_inference_dtype``
    (connect6/train.py:133-145): always float32 off the GPU, else by name."""
    if torch.device(device).type != "cuda":
        return torch.float32
    name = dtype_name.lower()
    if name == "bfloat16":
        return torch.bfloat16
    if name == "float16":
        return torch.float16
    if name == "float32":
        return torch.float32
    raise ValueError("historical_inference_dtype must be one of: bfloat16 | float16 | float32")


class HistoricalPolicyEnsemble:
    """Many frozen CNN policies evaluated together.

    Input ``[MODELS, TABLES, 3, H, W]`` -> policy logits ``[MODELS, TABLES,
    H*W]`` in the ensemble dtype.  ``dtype`` selects the arithmetic as in the
    reference's ``_history_dtype`` (connect6/train.py:133-145): float32,
    bfloat16 or float16.  bfloat16 runs the cascade (``"bf16c6"``);
    ``precision`` may name any other mode, e.g. ``"bf16"`` for the literal
    bf16 rounding of every activation.

    ``conv_weights``, ``conv_biases``, ``policy_weight`` and ``policy_bias``
    (the reference's stacked ``[M, ...]`` tensors, connect6/history.py:224-233)
    are built on first access: the forward reads only the packed copy.
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
        required = [f"convs.{i}.weight" for i in range(len(self.kernels))] + ["policy_output.weight"]
        for key in required:  # the KeyError of the reference's _stack (history.py:235-240)
            for state in states:
                if key not in state:
                    raise KeyError(f"parameter {key} is missing from the historical checkpoints")
        self.action_size = self.board_size * self.board_size

        self._prec = _PREC_OF_DTYPE[self.dtype] if precision is None else _lib.PREC_BY_NAME[precision]
        self._packed: tuple | None = None   # (buffer, stream it was packed on, event)
        self._states = states
        self._stacked: dict[str, torch.Tensor | None] = {}
        self._stacked32: dict[str, torch.Tensor] | None = None

    # -- the reference's stacked attributes, on `device` in `dtype`, built when first read --
    def _stacked_attr(self, key: str, optional: bool) -> torch.Tensor | None:
        if key not in self._stacked:
            self._stacked[key] = (self._stack_optional if optional else self._stack)(self._states, key)
        return self._stacked[key]

    @property
    def conv_weights(self) -> list[torch.Tensor]:
        return [self._stacked_attr(f"convs.{i}.weight", False) for i in range(len(self.kernels))]

    @property
    def conv_biases(self) -> list[torch.Tensor | None]:
        return [self._stacked_attr(f"convs.{i}.bias", True) for i in range(len(self.kernels))]

    @property
    def policy_weight(self) -> torch.Tensor:
        return self._stacked_attr("policy_output.weight", False)

    @property
    def policy_bias(self) -> torch.Tensor | None:
        return self._stacked_attr("policy_output.bias", True)

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
        keys = [f"convs.{i}.{kind}" for i in range(len(self.kernels)) for kind in ("weight", "bias")]
        keys += ["policy_output.weight", "policy_output.bias"]
        src = self._states[m]
        return {k: src[k].detach().to(device=self.device, dtype=self.dtype) for k in keys if k in src}

    def _packed_weights(self) -> torch.Tensor:
        stream = torch.cuda.current_stream(self.device)
        if self._packed is None:
            one = _lib.packed_bytes(self._prec)
            buf = torch.empty((self.num_models, one), dtype=torch.uint8, device=self.device)
            # one call for all models, from the stacked tensors (rounded to `dtype`, as the
            # ensemble holds its parameters): two launches, however many models
            keys = [f"convs.{i}.{kind}" for i in range(len(self.kernels)) for kind in ("weight", "bias")]
            keys += ["policy_output.weight", "policy_output.bias"]
            stacked = {k: self._stacked_attr(k, optional=k.endswith("bias")) for k in keys}
            pack_state(stacked, self._prec, buf, groups=self.num_models)
            done = torch.cuda.Event()
            done.record(stream)
            self._packed = (buf, stream.cuda_stream, done)
        buf, packed_on, done = self._packed
        if packed_on != stream.cuda_stream:   # packed on another stream: wait for it, and tell the
            stream.wait_event(done)           # allocator that this stream reads the buffer too
            buf.record_stream(stream)
        return buf

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
            # (the cascade's entry point writes the logits in the ensemble's type itself)
            direct = self._prec in _lib.CASCADES and self.dtype != torch.float32
            logits, _, _, _ = run_forward(x.reshape(m * t, *expected_tail), self._packed_weights(),
                                          self._prec, m, t, want_value=False,
                                          logits_dtype=self.dtype if direct else torch.float32)
        else:  # other architectures: layer by layer, every layer one launch for all models
            keys = [f"convs.{i}.{kind}" for i in range(len(self.kernels)) for kind in ("weight", "bias")]
            keys += ["policy_output.weight", "policy_output.bias"]
            if self._stacked32 is None:   # the layer-by-layer kernels read fp32 parameters
                self._stacked32 = {k: v.float().contiguous() for k in keys
                                   if (v := self._stacked_attr(k, optional=k.endswith("bias"))) is not None}
            stacked = self._stacked32
            logits = run_forward_generic(x.reshape(m * t, *expected_tail), stacked, self.kernels, self.channels,
                                         self._prec, want_value=False, groups=m)[0]
        logits = logits.view(m, t, self.action_size)
        return logits if self.dtype == torch.float32 else logits.to(self.dtype)
