"""Batched Connect6 environment on a HIP device: the reference's ``VectorConnect6``
(connect6/vector_env.py:17-226) with ``step`` and ``network_input`` as one HIP launch each.

Same constructor, same state tensors (``boards``, ``current_player``, ``stones_left``,
``empty_count``, ``move_count``: dtypes and shapes of connect6/vector_env.py:33-53), same
``StepBatch`` result.  There is no CPU path: the tensors live on the HIP device and a missing
library is an error.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from . import _lib


@dataclass(slots=True)
class StepBatch:
    """connect6/vector_env.py:8-14."""

    reward: torch.Tensor
    done: torch.Tensor
    winner: torch.Tensor
    transition_sign: torch.Tensor
    game_lengths: torch.Tensor


def _require_state(boards: torch.Tensor, current_player: torch.Tensor, stones_left: torch.Tensor) -> int:
    if boards.device.type != "cuda":
        raise RuntimeError("connect6_amd environment kernels need tensors on a HIP device")
    if boards.dim() != 3 or boards.shape[-1] != boards.shape[-2]:
        raise ValueError(f"expected boards [N, n, n], got {tuple(boards.shape)}")
    n_env = boards.shape[0]
    for name, t in (("boards", boards), ("current_player", current_player), ("stones_left", stones_left)):
        if t.dtype != torch.int8:
            raise ValueError(f"{name} must be int8, got {t.dtype}")
        if t.device != boards.device:
            raise ValueError(f"{name} is on {t.device}, boards on {boards.device}")
    if current_player.shape != (n_env,) or stones_left.shape != (n_env,):
        raise ValueError("current_player and stones_left must have shape [N]")
    return n_env


def canonical_network_input(
    boards: torch.Tensor, current_player: torch.Tensor, stones_left: torch.Tensor
) -> torch.Tensor:
    """connect6/vector_env.py:196-218: [N, 3, n, n] float32, planes = own stones, the other
    side's stones, "this decision is the last stone of the turn"."""
    n_env = _require_state(boards, current_player, stones_left)
    size = boards.shape[-1]
    boards, current_player, stones_left = boards.contiguous(), current_player.contiguous(), stones_left.contiguous()
    out = torch.empty((n_env, 3, size, size), dtype=torch.float32, device=boards.device)
    with torch.cuda.device(boards.device):
        rc = _lib.load().c6_canonical_input(boards.data_ptr(), current_player.data_ptr(), stones_left.data_ptr(),
                                            n_env, size, out.data_ptr(), _lib.stream_ptr(boards.device))
    _lib.check(rc, "c6_canonical_input")
    return out


def canonical_observation(
    boards: torch.Tensor, current_player: torch.Tensor, stones_left: torch.Tensor
) -> torch.Tensor:
    """connect6/vector_env.py:221-226."""
    return canonical_network_input(boards, current_player, stones_left)


class VectorConnect6:
    """connect6/vector_env.py:17-193."""

    def __init__(
        self,
        num_envs: int,
        board_size: int = 19,
        win_length: int = 6,
        device: str | torch.device = "cuda",
        debug_checks: bool = False,
    ) -> None:
        self.num_envs = int(num_envs)
        self.board_size = int(board_size)
        self.win_length = int(win_length)
        self.device = torch.device(device)
        self.debug_checks = bool(debug_checks)
        if self.device.type != "cuda":
            raise RuntimeError(
                f"connect6_amd.VectorConnect6 runs on a HIP device only (got {self.device}); "
                "use the reference's connect6.vector_env on the CPU"
            )
        if self.num_envs < 0 or self.board_size < 1 or self.board_size > 181 or self.win_length < 1:
            raise ValueError("num_envs >= 0, 1 <= board_size <= 181 and win_length >= 1 are required")
        _lib.load()  # fail here, loudly, when the library is missing
        n = self.board_size
        self.boards = torch.zeros((self.num_envs, n, n), dtype=torch.int8, device=self.device)
        self.current_player = torch.ones(self.num_envs, dtype=torch.int8, device=self.device)
        self.stones_left = torch.ones(self.num_envs, dtype=torch.int8, device=self.device)
        self.empty_count = torch.full((self.num_envs,), n * n, dtype=torch.int16, device=self.device)
        self.move_count = torch.zeros(self.num_envs, dtype=torch.int16, device=self.device)

    @property
    def action_size(self) -> int:
        return self.board_size * self.board_size

    @property
    def input_channels(self) -> int:
        return 3

    def reset(self, indices: torch.Tensor | None = None) -> None:
        """connect6/vector_env.py:77-93."""
        if indices is None:
            self.boards.zero_()
            self.current_player.fill_(1)
            self.stones_left.fill_(1)
            self.empty_count.fill_(self.action_size)
            self.move_count.zero_()
            return
        if indices.numel() == 0:
            return
        self.boards[indices] = 0
        self.current_player[indices] = 1
        self.stones_left[indices] = 1
        self.empty_count[indices] = self.action_size
        self.move_count[indices] = 0

    def legal_mask(self) -> torch.Tensor:
        return self.boards.view(self.num_envs, -1).eq(0)

    def network_input(self) -> torch.Tensor:
        return canonical_network_input(self.boards, self.current_player, self.stones_left)

    def observation(self) -> torch.Tensor:
        return self.network_input()

    @torch.no_grad()
    def step(self, actions: torch.Tensor, view: int = 0) -> StepBatch:
        """connect6/vector_env.py:106-161, one launch.  ``view`` (beyond the reference's
        signature): the D4 view the actions are expressed in; the kernel maps them back as
        ``_inverse_transform_actions`` does (connect6/train.py:854-862) before placing the stone."""
        view = int(view)
        if not 0 <= view < 8:
            raise ValueError(f"view must be 0..7, got {view}")
        actions = actions.to(device=self.device, dtype=torch.long, non_blocking=True)
        if actions.shape != (self.num_envs,):
            raise ValueError(f"expected actions of shape {(self.num_envs,)}, got {tuple(actions.shape)}")
        actions = actions.contiguous()
        if self.debug_checks:
            if self.num_envs and (int(actions.min()) < 0 or int(actions.max()) >= self.action_size):
                raise IndexError("action outside the board")
            from .selfplay import inverse_transform_actions

            placed = inverse_transform_actions(actions, self.board_size, view % 4, view >= 4)
            occupied = self.boards.view(self.num_envs, -1).gather(1, placed.view(-1, 1)).ne(0).flatten()
            if bool(occupied.any()):
                bad = int(torch.nonzero(occupied, as_tuple=False).flatten()[0])
                raise RuntimeError(f"stone placed on an occupied square in env {bad}")
        dev = self.device
        n_env = self.num_envs
        reward = torch.empty(n_env, dtype=torch.float32, device=dev)
        done = torch.empty(n_env, dtype=torch.bool, device=dev)
        winner = torch.empty(n_env, dtype=torch.int8, device=dev)
        sign = torch.empty(n_env, dtype=torch.int8, device=dev)
        lengths = torch.empty(n_env, dtype=torch.int16, device=dev)
        with torch.cuda.device(dev):
            rc = _lib.load().c6_env_step(
                self.boards.data_ptr(), self.current_player.data_ptr(), self.stones_left.data_ptr(),
                self.empty_count.data_ptr(), self.move_count.data_ptr(), actions.data_ptr(), view, n_env,
                self.board_size, self.win_length, reward.data_ptr(), done.data_ptr(), winner.data_ptr(),
                sign.data_ptr(), lengths.data_ptr(), _lib.stream_ptr(dev))
        _lib.check(rc, "c6_env_step")
        return StepBatch(reward=reward, done=done, winner=winner, transition_sign=sign, game_lengths=lengths)
