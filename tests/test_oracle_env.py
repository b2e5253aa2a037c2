"""Pins oracle/env_ref.py (CPU only): the reference's known answers and an independent scalar game."""
import numpy as np
import pytest
import torch

from oracle import env_ref as E


def test_initial_state_and_reset():
    st = E.new_state(3, 9, 6)
    assert st.boards.shape == (3, 9, 9) and st.boards.dtype == torch.int8
    assert st.current_player.tolist() == [1, 1, 1] and st.stones_left.tolist() == [1, 1, 1]
    assert st.empty_count.tolist() == [81] * 3 and st.move_count.tolist() == [0] * 3
    E.step(st, torch.tensor([0, 1, 2]))
    E.reset(st, torch.tensor([1]))
    assert st.boards[1].abs().sum() == 0 and st.boards[0].abs().sum() == 1
    assert st.current_player.tolist() == [-1, 1, -1] and st.empty_count.tolist() == [80, 81, 80]
    E.reset(st, torch.tensor([], dtype=torch.long))
    E.reset(st)
    assert st.boards.abs().sum() == 0 and st.move_count.tolist() == [0, 0, 0]


def test_turn_order_known_answer():
    # reference tests/test_game.py:9-25: Black places one stone, then everybody two
    st = E.new_state(1, 19, 6)
    out = E.step(st, torch.tensor([9 * 19 + 9]))
    assert (st.current_player.item(), st.stones_left.item(), out.transition_sign.item()) == (-1, 2, -1)
    out = E.step(st, torch.tensor([0]))
    assert (st.current_player.item(), st.stones_left.item(), out.transition_sign.item()) == (-1, 1, 1)
    out = E.step(st, torch.tensor([1]))
    assert (st.current_player.item(), st.stones_left.item(), out.transition_sign.item()) == (1, 2, -1)
    assert out.game_lengths.item() == 3 and not out.done.item() and out.reward.item() == 0.0


def test_horizontal_and_diagonal_win_known_answers():
    # reference tests/test_game.py:28-44
    st = E.new_state(2, 9, 6)
    st.boards[0, 4, 1:6] = 1
    st.current_player[0], st.stones_left[0] = 1, 1
    for i in range(5):
        st.boards[1, i, i] = -1
    st.current_player[1] = -1
    out = E.step(st, torch.tensor([4 * 9 + 6, 5 * 9 + 5]))
    assert out.done.tolist() == [True, True] and out.winner.tolist() == [1, -1]
    assert out.reward.tolist() == [1.0, 1.0] and out.transition_sign.tolist() == [0, 0]
    # a finished game keeps its side to move and stones_left (connect6/vector_env.py:140-146)
    assert st.current_player.tolist() == [1, -1] and st.stones_left.tolist() == [1, 1]


def test_five_is_not_six_and_gaps_do_not_count():
    st = E.new_state(2, 19, 6)
    st.boards[0, 3, 2:6] = 1                 # four in a row; a fifth does not win
    st.boards[1, 3, 2:5] = 1
    st.boards[1, 3, 6:8] = 1                 # xxx_xx: filling the gap makes six
    out = E.step(st, torch.tensor([3 * 19 + 6, 3 * 19 + 9]))
    assert out.done.tolist() == [False, False]
    st.current_player[:] = 1
    out = E.step(st, torch.tensor([3 * 19 + 1, 3 * 19 + 5]))
    assert out.done.tolist() == [True, True] and out.winner.tolist() == [1, 1]


def _random_games(n_envs, board, win, seed, steps):
    g = torch.Generator().manual_seed(seed)
    st = E.new_state(n_envs, board, win)
    games = [E.ScalarGame(board, win) for _ in range(n_envs)]
    finished = 0
    for _ in range(steps):
        legal = st.boards.view(n_envs, -1).eq(0)
        scores = torch.rand(legal.shape, generator=g).masked_fill(~legal, -1.0)
        actions = scores.argmax(1)
        out = E.step(st, actions)
        for i, game in enumerate(games):
            r, d, w, s, length = game.step(int(actions[i]))
            assert (out.reward[i].item(), out.done[i].item(), out.winner[i].item(),
                    out.transition_sign[i].item(), out.game_lengths[i].item()) == (r, d, w, s, length)
            if d:
                finished += 1
                games[i] = E.ScalarGame(board, win)
        E.reset(st, torch.nonzero(out.done).flatten())
        for i, game in enumerate(games):
            assert np.array_equal(st.boards[i].numpy(), game.board)
            assert (st.current_player[i].item(), st.stones_left[i].item()) == (game.player, game.stones_left)
            assert st.move_count[i].item() == game.moves
            assert st.empty_count[i].item() == board * board - game.moves
    return finished


@pytest.mark.parametrize("board,win,steps", [(19, 6, 400), (9, 6, 200), (7, 4, 120), (3, 6, 30)])
def test_step_matches_independent_scalar_game(board, win, steps):
    finished = _random_games(12, board, win, 100 + board, steps)
    assert finished >= 12          # every board size sees whole games, wins and (3x3) draws


def test_draw_on_board_without_room_for_a_line():
    st = E.new_state(1, 3, 6)
    for a in range(8):
        out = E.step(st, torch.tensor([a]))
        assert not out.done.item()
    out = E.step(st, torch.tensor([8]))
    assert out.done.item() and out.winner.item() == 0 and out.reward.item() == 0.0
    assert out.transition_sign.item() == 0 and out.game_lengths.item() == 9


def test_bad_action_shape_raises():
    with pytest.raises(ValueError):
        E.step(E.new_state(4, 9, 6), torch.zeros(3, dtype=torch.long))


def test_oracle_reproduces_committed_env_rollout():
    from pathlib import Path

    g = np.load(Path(__file__).resolve().parent / "golden" / "env_rollout_golden.npz")
    st = E.new_state(48, 19, 6)
    for i in range(g["actions"].shape[0]):
        out = E.step(st, torch.from_numpy(g["actions"][i]))
        for k in ("reward", "done", "winner", "transition_sign", "game_lengths"):
            assert np.array_equal(getattr(out, k).numpy(), g[k][i]), (k, i)
        E.reset(st, torch.nonzero(out.done).flatten())
    for k in ("boards", "current_player", "stones_left", "empty_count", "move_count"):
        assert np.array_equal(getattr(st, k).numpy(), g[k])
    assert g["done"].sum() >= 50 and g["reward"].sum() >= 50      # the fixture holds real wins
