"""Seeded synthetic Connect6 positions for benchmarks and parity tests.

The reference has no such generator: real inputs come from
``canonical_network_input`` (connect6/vector_env.py:196-218 of the reference),
whose planes are exactly 0.0/1.0 -- channel 0 own stones, channel 1 opponent
stones, channel 2 a constant plane telling whether this is the last stone of
the turn.  The generator reproduces that input format from a seed.
"""
from __future__ import annotations

import torch


def gen_boards(batch: int, max_stones: int = 200, seed: int = 2025, board_size: int = 19):
    """Returns ``(x, legal)``: x fp32 ``[B,3,n,n]`` with values in {0,1} and
    legal bool ``[B,n*n]``.

    Per board: stone count ``s`` uniform in ``0..max_stones``; ``s`` distinct
    squares drawn uniformly; the first ``s//2`` go to channel 0 (side to move)
    and the remaining ``s - s//2`` to channel 1, so the opponent holds the odd
    stone; channel 2 is all ones with probability 1/2, else all zeros.
    """
    nn_ = board_size * board_size
    g = torch.Generator(device="cpu").manual_seed(int(seed))
    count = torch.randint(0, int(max_stones) + 1, (batch,), generator=g)
    order = torch.rand(batch, nn_, generator=g).argsort(dim=1)
    rank = torch.empty_like(order)
    rank.scatter_(1, order, torch.arange(nn_).expand(batch, nn_))
    own = rank < (count // 2).view(-1, 1)
    stone = rank < count.view(-1, 1)
    opp = stone & ~own
    last = torch.rand(batch, generator=g) < 0.5
    x = torch.zeros(batch, 3, nn_, dtype=torch.float32)
    x[:, 0] = own.float()
    x[:, 1] = opp.float()
    x[:, 2] = last.float().view(-1, 1).expand(batch, nn_)
    legal = ~stone
    return x.view(batch, 3, board_size, board_size), legal


def gen_uniform(batch: int, seed: int = 7) -> torch.Tensor:
    """Seeded uniform draws in [0,1), one per board, for inverse-CDF sampling."""
    g = torch.Generator(device="cpu").manual_seed(int(seed))
    return torch.rand(batch, generator=g)
