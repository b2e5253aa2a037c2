#!/usr/bin/env python3
"""Writes tests/golden/default_arch_golden.npz (seeded inputs and the fp32 oracle's outputs)
and tests/golden/env_rollout_golden.npz (a seeded random self-play rollout through the
environment oracle: actions in, every StepBatch field and the final state out).

The reference repository holds no numeric vectors for this path (it was not imported or run);
these fixtures come from THIS repository's oracle (oracle/torch_ref.py, itself pinned by the
brute-force C convolution and closed forms in tests/test_oracle.py).  They guard against drift
of the oracle across PyTorch versions and give the GPU tests a file-based target.

    python tests/golden/make_golden.py
"""
import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parent.parent.parent
sys.path.insert(0, str(ROOT))

from connect6_amd.synthetic import gen_boards, gen_uniform  # noqa: E402
from oracle import env_ref as E  # noqa: E402
from oracle import torch_ref as R  # noqa: E402


def main() -> None:
    torch.set_num_threads(1)          # fixed summation order
    out = {}
    x, legal = gen_boards(6, 200, 2025)
    u = gen_uniform(6, 7)
    out["x"] = x.numpy()
    out["legal"] = legal.numpy()
    out["u"] = u.numpy()
    for init in ("reference", "torch_default"):
        st = R.init_state(1234, init)
        with torch.inference_mode():
            logits, value = R.forward(st, x)
            actions, logprob = R.sample_inverse_cdf(logits, legal, u, 1.0)
        out[f"{init}_logits"] = logits.numpy()
        out[f"{init}_value"] = value.numpy()
        out[f"{init}_actions"] = actions.numpy()
        out[f"{init}_logprob"] = logprob.numpy()
    np.savez_compressed(Path(__file__).resolve().parent / "default_arch_golden.npz", **out)
    print("wrote default_arch_golden.npz", {k: v.shape for k, v in out.items()})

    # environment rollout: 48 games on the default board, 160 steps, finished games reset
    gen = torch.Generator().manual_seed(77)
    st = E.new_state(48, 19, 6)
    rec = {k: [] for k in ("actions", "reward", "done", "winner", "transition_sign", "game_lengths")}
    for _ in range(160):
        legal = st.boards.view(48, -1).eq(0)
        # mostly play next to existing stones so that lines (and wins) actually form
        near = torch.nn.functional.max_pool2d(st.boards.ne(0).float().unsqueeze(1), 3, 1, 1).view(48, -1)
        score = torch.rand(legal.shape, generator=gen) + 2.0 * near
        actions = score.masked_fill(~legal, -1.0).argmax(1)
        step = E.step(st, actions)
        rec["actions"].append(actions.numpy())
        for k in ("reward", "done", "winner", "transition_sign", "game_lengths"):
            rec[k].append(getattr(step, k).numpy())
        E.reset(st, torch.nonzero(step.done).flatten())
    env = {k: np.stack(v) for k, v in rec.items()}
    env.update(boards=st.boards.numpy(), current_player=st.current_player.numpy(),
               stones_left=st.stones_left.numpy(), empty_count=st.empty_count.numpy(),
               move_count=st.move_count.numpy())
    np.savez_compressed(Path(__file__).resolve().parent / "env_rollout_golden.npz", **env)
    print("wrote env_rollout_golden.npz", int(env["done"].sum()), "finished games,", int(env["reward"].sum()), "wins")


if __name__ == "__main__":
    main()
