"""Parity of the environment kernels (c6_env_step, c6_canonical_input) with the oracle:
bit-exact on every state tensor and every result, step by step, through whole games."""
import pytest
import torch

import connect6_amd as c6
from oracle import env_ref as E
from oracle import torch_ref as R

pytestmark = pytest.mark.gpu


def _assert_same_state(env: c6.VectorConnect6, st: E.EnvState):
    assert torch.equal(env.boards.cpu(), st.boards)
    assert torch.equal(env.current_player.cpu(), st.current_player)
    assert torch.equal(env.stones_left.cpu(), st.stones_left)
    assert torch.equal(env.empty_count.cpu(), st.empty_count)
    assert torch.equal(env.move_count.cpu(), st.move_count)


def _assert_same_step(got: c6.StepBatch, want: E.StepOut):
    assert got.reward.dtype == torch.float32 and got.done.dtype == torch.bool
    assert got.winner.dtype == torch.int8 and got.transition_sign.dtype == torch.int8
    assert got.game_lengths.dtype == torch.int16
    assert torch.equal(got.reward.cpu(), want.reward)
    assert torch.equal(got.done.cpu(), want.done)
    assert torch.equal(got.winner.cpu(), want.winner)
    assert torch.equal(got.transition_sign.cpu(), want.transition_sign)
    assert torch.equal(got.game_lengths.cpu(), want.game_lengths)


def _random_legal_actions(boards: torch.Tensor, gen: torch.Generator) -> torch.Tensor:
    legal = boards.view(boards.shape[0], -1).eq(0)
    return torch.rand(legal.shape, generator=gen).masked_fill(~legal, -1.0).argmax(1)


@pytest.mark.parametrize("num,board,win,steps", [(2048, 19, 6, 380), (512, 9, 6, 120), (257, 7, 4, 80), (64, 3, 6, 20), (1, 19, 6, 40)])
def test_rollouts_match_oracle_bit_exact(cuda, num, board, win, steps):
    gen = torch.Generator().manual_seed(board * 1000 + num)
    env = c6.VectorConnect6(num, board, win, device=cuda)
    st = E.new_state(num, board, win)
    finished = wins = draws = 0
    for _ in range(steps):
        actions = _random_legal_actions(st.boards, gen)
        want = E.step(st, actions)
        got = env.step(actions.to(cuda))
        _assert_same_step(got, want)
        _assert_same_state(env, st)
        finished += int(want.done.sum())
        wins += int(want.reward.sum())
        draws += int((want.done & (want.winner == 0)).sum())
        idx = torch.nonzero(want.done).flatten()
        E.reset(st, idx)
        env.reset(idx.to(cuda))
    if num > 1:
        assert finished > 0 and (wins > 0 or draws > 0)


def test_reference_known_answers(cuda):
    # reference tests/test_game.py:9-44 through the product class
    env = c6.VectorConnect6(1, 19, 6, device=cuda)
    out = env.step(torch.tensor([9 * 19 + 9]))
    assert (env.current_player.item(), env.stones_left.item(), out.transition_sign.item()) == (-1, 2, -1)
    out = env.step(torch.tensor([0], device=cuda))
    assert (env.current_player.item(), env.stones_left.item(), out.transition_sign.item()) == (-1, 1, 1)
    out = env.step(torch.tensor([1], device=cuda, dtype=torch.int32))      # any integer dtype, any device
    assert (env.current_player.item(), env.stones_left.item(), out.transition_sign.item()) == (1, 2, -1)

    env = c6.VectorConnect6(2, 9, 6, device=cuda)
    env.boards[0, 4, 1:6] = 1
    for i in range(5):
        env.boards[1, i, i] = -1
    env.current_player[1] = -1
    out = env.step(torch.tensor([4 * 9 + 6, 5 * 9 + 5], device=cuda))
    assert out.done.tolist() == [True, True] and out.winner.tolist() == [1, -1]
    assert out.reward.tolist() == [1.0, 1.0]


def test_lines_at_the_board_edge_and_longer_than_six(cuda):
    # wins along all four directions touching the border, and an overline (7) counts as a win
    env = c6.VectorConnect6(5, 19, 6, device=cuda)
    st = E.new_state(5, 19, 6)
    for s, b in ((st, st.boards), (env, env.boards)):
        b[0, 0, 0:5] = 1            # row 0, completes at column 5
        b[1, 14:19, 18] = 1         # last column, completes at row 13
        b[2, 13, 5] = b[2, 14, 4] = b[2, 15, 3] = b[2, 16, 2] = b[2, 17, 1] = 1   # anti-diagonal to the corner
        b[3, 5, 5:8] = 1
        b[3, 5, 9:12] = 1           # xxx_xxx: the middle stone makes seven
        b[4, 0, 0:4] = 1            # only five after the move: no win
    actions = torch.tensor([5, 13 * 19 + 18, 18 * 19 + 0, 5 * 19 + 8, 4])
    want = E.step(st, actions)
    got = env.step(actions.to(cuda))
    _assert_same_step(got, want)
    assert want.done.tolist() == [True, True, True, True, False]
    _assert_same_state(env, st)


def test_debug_checks_and_argument_errors(cuda):
    env = c6.VectorConnect6(4, 9, 6, device=cuda, debug_checks=True)
    result = env.step(torch.tensor([0, 1, 2, 3]))          # reference tests/test_game.py:62-75
    assert result.done.shape == (4,)
    x = env.network_input()
    assert x.shape == (4, 3, 9, 9) and x.dtype == torch.float32
    with pytest.raises(RuntimeError, match="occupied"):
        env.step(torch.tensor([5, 1, 6, 7]))
    with pytest.raises(ValueError):
        env.step(torch.zeros(3, dtype=torch.long))
    assert env.action_size == 81 and env.input_channels == 3
    assert torch.equal(env.legal_mask().cpu(), env.boards.cpu().view(4, -1).eq(0))


def test_empty_environment_batch(cuda):
    env = c6.VectorConnect6(0, 19, 6, device=cuda)
    out = env.step(torch.zeros(0, dtype=torch.long))
    assert out.done.shape == (0,) and env.network_input().shape == (0, 3, 19, 19)


@pytest.mark.parametrize("num,board", [(1, 19), (1000, 19), (33, 9)])
def test_canonical_input_matches_oracle(cuda, num, board):
    gen = torch.Generator().manual_seed(num)
    boards = torch.randint(-1, 2, (num, board, board), generator=gen, dtype=torch.int8)
    player = (torch.randint(0, 2, (num,), generator=gen) * 2 - 1).to(torch.int8)
    stones = torch.randint(1, 3, (num,), generator=gen).to(torch.int8)
    want = R.canonical_network_input(boards, player, stones)       # connect6/vector_env.py:196-218
    got = c6.canonical_network_input(boards.to(cuda), player.to(cuda), stones.to(cuda))
    assert got.dtype == torch.float32 and torch.equal(got.cpu(), want)
    assert torch.equal(c6.canonical_observation(boards.to(cuda), player.to(cuda), stones.to(cuda)).cpu(), want)


def test_full_size_batch_is_periodic_in_the_small_one(cuda):
    # 262144 games driven by the first 1024 games' actions repeated: every block of 1024 must
    # reproduce the oracle-checked small batch bit for bit, at every step
    small, reps, steps = 1024, 256, 60
    gen = torch.Generator().manual_seed(5)
    st = E.new_state(small, 19, 6)
    env = c6.VectorConnect6(small * reps, 19, 6, device=cuda)
    for _ in range(steps):
        actions = _random_legal_actions(st.boards, gen)
        want = E.step(st, actions)
        got = env.step(actions.to(cuda).repeat(reps))
        for name in ("reward", "done", "winner", "transition_sign", "game_lengths"):
            g = getattr(got, name).view(reps, small)
            assert torch.equal(g[0].cpu(), getattr(want, name))
            assert bool((g == g[0:1]).all())
    b = env.boards.view(reps, small, 19, 19)
    assert torch.equal(b[0].cpu(), st.boards) and bool((b == b[0:1]).all())
    # conservation: stones on the board == moves made == 361 - empty squares
    stones = env.boards.ne(0).flatten(1).sum(1)
    assert torch.equal(stones.to(torch.int16), env.move_count)
    assert torch.equal(361 - env.empty_count, env.move_count)


@pytest.mark.parametrize("board", [19, 9])
def test_actions_given_in_a_d4_view(cuda, board):
    # the collector samples in view coordinates and maps back (connect6/train.py:854-862)
    gen = torch.Generator().manual_seed(3)
    for view in range(8):
        env = c6.VectorConnect6(64, board, 6, device=cuda, debug_checks=True)
        st = E.new_state(64, board, 6)
        for _ in range(12):
            canonical = _random_legal_actions(st.boards, gen)
            in_view = R.transform_actions(canonical, board, view % 4, view >= 4)
            want = E.step(st, canonical)
            got = env.step(in_view.to(cuda), view=view)
            _assert_same_step(got, want)
            _assert_same_state(env, st)


def test_collector_loop_plays_legal_games_to_the_end(cuda):
    # forward from int8 state -> sample -> step, all in view coordinates; debug_checks would raise
    # on any stone placed on an occupied square
    model = c6.PolicyValueNet().to(cuda).eval()
    env = c6.VectorConnect6(256, 19, 6, device=cuda, debug_checks=True)
    gen = torch.Generator().manual_seed(1)
    finished = 0
    with torch.inference_mode():
        for it in range(400):
            view = it % 8
            u = torch.rand(256, generator=gen).to(cuda)
            actions, logprob, value = model.selfplay_step_boards(env.boards, env.current_player, env.stones_left,
                                                                 u, 1.0, view=view)
            step = env.step(actions, view=view)
            finished += int(step.done.sum())
            env.reset(torch.nonzero(step.done).flatten())
            assert bool(torch.isfinite(logprob).all()) and bool(value.abs().le(1).all())
    assert finished > 0
    assert bool((env.boards.ne(0).flatten(1).sum(1).to(torch.int16) == env.move_count).all())


def test_committed_env_rollout(cuda):
    import numpy as np
    from pathlib import Path

    g = np.load(Path(__file__).resolve().parent / "golden" / "env_rollout_golden.npz")
    env = c6.VectorConnect6(48, 19, 6, device=cuda)
    for i in range(g["actions"].shape[0]):
        out = env.step(torch.from_numpy(g["actions"][i]).to(cuda))
        for k in ("reward", "done", "winner", "transition_sign", "game_lengths"):
            assert np.array_equal(getattr(out, k).cpu().numpy(), g[k][i]), (k, i)
        env.reset(torch.nonzero(out.done).flatten())
    for k in ("boards", "current_player", "stones_left", "empty_count", "move_count"):
        assert np.array_equal(getattr(env, k).cpu().numpy(), g[k])
