"""Pins the CPU oracle (oracle/) without any GPU: brute force, closed forms,
known answers and the reference's own invariants."""
import math

import pytest
import torch

from connect6_amd.synthetic import gen_boards, gen_uniform
from oracle import cref
from oracle import torch_ref as R

TINY = dict(kernels=(3, 3, 3), channels=(8, 8, 16))  # tests/test_training_features.py:122-129


def test_init_state_keys_shapes_and_scale():
    st = R.init_state(0, "reference")
    assert len(st) == 20
    cin = 3
    for i, (k, c) in enumerate(zip(R.DEFAULT_KERNELS, R.DEFAULT_CHANNELS)):
        assert st[f"convs.{i}.weight"].shape == (c, cin, k, k)
        assert st[f"convs.{i}.bias"].shape == (c,)
        assert torch.count_nonzero(st[f"convs.{i}.bias"]) == 0
        want = math.sqrt(2.0 / (cin * k * k))
        assert abs(st[f"convs.{i}.weight"].std().item() / want - 1) < 0.05
        cin = c
    assert st["policy_output.weight"].shape == (1, 96, 1, 1)
    assert st["value_output.weight"].shape == (1, 96, 1, 1)
    assert abs(st["policy_output.weight"].std().item() / 0.01 - 1) < 0.3
    n_params = sum(v.numel() for v in st.values())
    assert n_params == 374082
    td = R.init_state(0, "torch_default")
    assert td["convs.3.bias"].abs().max() <= 1 / math.sqrt(64 * 9)


def test_forward_matches_bruteforce_c_tiny():
    st = R.init_state(5, "torch_default", **TINY)
    x = torch.randn(3, 3, 5, 5, generator=torch.Generator().manual_seed(1))
    lt, vt = R.forward(st, x)
    lc, vc = cref.forward(st, x)
    assert lt.shape == (3, 25) and vt.shape == (3,)
    assert torch.allclose(lt, lc, atol=1e-6, rtol=1e-5)
    assert torch.allclose(vt, vc, atol=1e-6, rtol=1e-5)


def test_forward_matches_bruteforce_c_default_architecture():
    st = R.init_state(1234, "torch_default")
    x, _ = gen_boards(2, 200, 11)
    lt, vt = R.forward(st, x)
    lc, vc = cref.forward(st, x)
    assert float((lt - lc).norm() / lc.norm()) < 1e-5
    assert torch.allclose(vt, vc, atol=1e-6)


def test_forward_one_layer_hand_computed():
    # 1x1 conv with weight 2 and bias 1 on a single plane, heads = identity / 0.5
    st = {
        "convs.0.weight": torch.tensor([[[[2.0]], [[0.0]], [[0.0]]]]),
        "convs.0.bias": torch.tensor([1.0]),
        "policy_output.weight": torch.tensor([[[[1.0]]]]),
        "policy_output.bias": torch.tensor([0.25]),
        "value_output.weight": torch.tensor([[[[0.5]]]]),
        "value_output.bias": torch.tensor([0.0]),
    }
    x = torch.zeros(1, 3, 2, 2)
    x[0, 0] = torch.tensor([[0.0, 1.0], [2.0, -1.0]])
    z = 2 * x[0, 0] + 1
    a = z / (1 + torch.exp(-z))
    logits, value = R.forward(st, x)
    assert torch.allclose(logits, (a + 0.25).reshape(1, 4))       # row-major flatten
    assert torch.allclose(value, torch.tanh((0.5 * a).mean()).reshape(1))


def test_zero_input_known_answer_and_value_range():
    st = R.init_state(3, "reference")
    logits, value = R.forward(st, torch.zeros(3, 3, 19, 19))      # tests/test_model.py:13-17
    assert logits.shape == (3, 361) and value.shape == (3,)
    assert torch.count_nonzero(logits) == 0 and torch.count_nonzero(value) == 0
    x, _ = gen_boards(16, 200, 2)
    _, v = R.forward(R.init_state(3, "torch_default"), x)
    assert torch.all(v <= 1) and torch.all(v >= -1)


def test_forward_rejects_bad_shape():
    st = R.init_state(3, "reference")
    with pytest.raises(ValueError):
        R.forward(st, torch.zeros(3, 2, 19, 19))
    with pytest.raises(ValueError):
        R.forward(st, torch.zeros(3, 19, 19))


def test_grouped_equals_individual_models():
    # the reference's invariant, tests/test_training_features.py:120-151
    states = [R.init_state(100 + i, "reference", **TINY) for i in range(2)]
    x = torch.randn(2, 5, 3, 5, 5, generator=torch.Generator().manual_seed(123))
    grouped = R.forward_grouped(states, x)
    assert grouped.shape == (2, 5, 25)
    for i, s in enumerate(states):
        assert torch.allclose(grouped[i], R.forward(s, x[i])[0], atol=1e-5, rtol=1e-5)
    states = [R.init_state(7 + i, "torch_default") for i in range(2)]
    xb, _ = gen_boards(4, 200, 5)
    xg = xb.view(2, 2, 3, 19, 19)
    assert torch.allclose(R.forward_grouped(states, xg), R.forward_grouped_loop(states, xg), atol=1e-5)
    with pytest.raises(ValueError):
        R.forward_grouped([], xg)


def test_mask_logits_bit_patterns():
    logits = torch.randn(4, 361)
    _, legal = gen_boards(4, 200, 9)
    out = R.mask_logits(logits, legal)
    lowest = torch.tensor(torch.finfo(torch.float32).min)
    assert torch.equal(out[~legal].view(torch.int32), lowest.view(torch.int32).expand(int((~legal).sum())))
    assert torch.equal(out[legal].view(torch.int32), logits[legal].view(torch.int32))
    assert torch.all(torch.isneginf(R.mask_logits(logits, legal, float("-inf"))[~legal]))
    x, lg = gen_boards(4, 200, 9)
    assert torch.equal(R.legal_from_input(x), lg)


def _sample_loop(logits, legal, u, temperature):
    out = []
    for b in range(logits.shape[0]):
        z = [(logits[b, i].item() / max(temperature, 1e-4)) if legal[b, i] else -math.inf for i in range(logits.shape[1])]
        m = max(z)
        e = [math.exp(v - m) for v in z]
        total = sum(e)
        run, pick = 0.0, None
        for i, v in enumerate(e):
            run += v
            if legal[b, i] and run > u[b].item() * total:
                pick = i
                break
        if pick is None:
            pick = max(i for i in range(len(z)) if legal[b, i])
        out.append((pick, z[pick] - m - math.log(total)))
    return out


def test_sample_inverse_cdf_matches_python_loop_and_respects_mask():
    g = torch.Generator().manual_seed(4)
    logits = torch.randn(64, 361, generator=g) * 2
    _, legal = gen_boards(64, 300, 17)
    u = gen_uniform(64, 3)
    a, lp = R.sample_inverse_cdf(logits, legal, u, 0.7)
    want = _sample_loop(logits, legal, u, 0.7)
    assert [int(v) for v in a] == [w[0] for w in want]
    assert torch.allclose(lp, torch.tensor([w[1] for w in want], dtype=torch.float32), atol=1e-4)
    assert bool(legal.gather(1, a.view(-1, 1)).all())
    # u -> 1 picks the last legal square, u = 0 the first with non-zero mass
    a1, _ = R.sample_inverse_cdf(logits, legal, torch.full((64,), 0.99999994), 1.0)
    assert bool(legal.gather(1, a1.view(-1, 1)).all())
    a0, _ = R.sample_inverse_cdf(logits, legal, torch.zeros(64), 1.0)
    assert torch.equal(a0, legal.float().argmax(1))


def test_sample_inverse_cdf_distribution():
    logits = torch.tensor([[0.0, 1.0, 2.0, -1.0] + [0.0] * 357])
    legal = torch.zeros(1, 361, dtype=torch.bool)
    legal[0, :4] = True
    legal[0, 2] = False
    n = 20000
    u = torch.rand(n, generator=torch.Generator().manual_seed(0))
    a, _ = R.sample_inverse_cdf(logits.expand(n, -1), legal.expand(n, -1), u, 1.0)
    p = torch.softmax(torch.tensor([0.0, 1.0, -1.0]), 0)
    freq = torch.tensor([(a == 0).float().mean(), (a == 1).float().mean(), (a == 3).float().mean()])
    assert int((a == 2).sum()) == 0 and int((a > 3).sum()) == 0
    assert torch.allclose(freq, p, atol=0.015)


def test_symmetry_cycle_order():
    # tests/test_training_features.py:154-166
    want = [(0, False), (1, False), (2, False), (3, False), (0, True), (1, True), (2, True), (3, True)]
    assert [R.symmetry_for_phase(i) for i in range(8)] == want
    assert R.symmetry_for_phase(8) == want[0]


@pytest.mark.parametrize("n", [3, 7, 19])
def test_d4_maps_match_rot90_flip_and_invert(n):
    board = torch.arange(n * n, dtype=torch.int64).reshape(1, n, n)
    actions = torch.arange(n * n)
    for phase in range(8):
        k, flip = R.symmetry_for_phase(phase)
        lib = torch.rot90(board, k=k, dims=(-2, -1)) if k else board      # train.py:228-230
        lib = torch.flip(lib, dims=(-1,)) if flip else lib
        view = R.transform_boards(board, k, flip)
        assert torch.equal(view, lib)
        ta = R.transform_actions(actions, n, k, flip)
        # tests/test_training_features.py:169-187: a stone stays under its transformed action
        assert torch.equal(view.reshape(-1)[ta], board.reshape(-1)[actions])
        assert torch.equal(R.inverse_transform_actions(ta, n, k, flip), actions)
        assert sorted(ta.tolist()) == list(range(n * n))


def test_d4_single_stone_follows_action():
    # tests/test_model.py:40-53
    n = 7
    board = torch.zeros(1, n, n, dtype=torch.int8)
    board[0, 1, 2] = 1
    action = torch.tensor([1 * n + 2])
    for k in range(4):
        for flip in (False, True):
            ob = R.transform_boards(board, k, flip)
            oa = int(R.transform_actions(action, n, k, flip))
            assert int(ob[0, oa // n, oa % n]) == 1
            assert torch.equal(R.inverse_transform_actions(torch.tensor([oa]), n, k, flip), action)


def test_d4_average_recovers_equivariant_map():
    base = torch.randn(5, 361)
    vals = torch.randn(8, 5)
    views = R.d4_expand(base.view(5, 1, 19, 19)).view(8, 5, 361)   # view p shows base through D4 map p
    logits, values = R.d4_average(views, vals)
    assert torch.allclose(logits, base, atol=1e-6)
    assert torch.allclose(values, vals.mean(0))
    # brute force for one entry
    b, a = 2, 123
    s = sum(views[p, b, int(R.transform_actions(torch.tensor([a]), 19, *R.symmetry_for_phase(p)))] for p in range(8))
    assert abs(float(s) / 8 - float(logits[b, a])) < 1e-6


def test_bf16_emulation_is_close_to_fp32():
    st = R.init_state(1234, "reference")
    x, legal = gen_boards(64, 200, 2025)
    l32, v32 = R.forward(st, x)
    l16, v16 = R.forward_bf16_emulated(st, x)
    assert float((l16 - l32).norm() / l32.norm()) < 2e-2
    assert float((v16 - v32).norm() / v32.norm()) < 2e-2


def test_generator_properties():
    x, legal = gen_boards(512, 200, 2025)
    assert x.shape == (512, 3, 19, 19) and x.dtype == torch.float32
    assert set(torch.unique(x).tolist()) <= {0.0, 1.0}
    own, opp = x[:, 0].flatten(1).sum(1), x[:, 1].flatten(1).sum(1)
    assert float((x[:, 0] * x[:, 1]).sum()) == 0            # no overlaps
    assert torch.all((opp - own == 0) | (opp - own == 1))    # split as evenly as possible
    assert int((own + opp).max()) <= 200 and int((own + opp).min()) >= 0
    plane = x[:, 2].flatten(1)
    assert torch.all((plane.min(1).values == plane.max(1).values))
    assert 0.35 < float(plane[:, 0].mean()) < 0.65
    assert torch.equal(legal, (x[:, 0] + x[:, 1] == 0).flatten(1))
    x2, _ = gen_boards(512, 200, 2025)
    assert torch.equal(x, x2)
    x3, _ = gen_boards(64, 300, 1)
    assert int((x3[:, 0] + x3[:, 1]).flatten(1).sum(1).max()) > 200


def test_canonical_network_input_channel_meaning():
    # tests/test_game.py:46-59 of the reference: plane 0 = side to move, plane 1 = opponent,
    # plane 2 = "this is the last stone of the turn"
    boards = torch.zeros(2, 19, 19, dtype=torch.int8)
    boards[0, 9, 9] = 1
    boards[0, 3, 4] = -1
    boards[1, 0, 0] = -1
    boards[1, 18, 18] = 1
    player = torch.tensor([1, -1], dtype=torch.int8)
    left = torch.tensor([1, 2], dtype=torch.int8)
    x = R.canonical_network_input(boards, player, left)
    assert x.shape == (2, 3, 19, 19) and x.dtype == torch.float32
    assert x[0, 0, 9, 9] == 1 and x[0, 0].sum() == 1
    assert x[0, 1, 3, 4] == 1 and x[0, 1].sum() == 1
    assert torch.all(x[0, 2] == 1) and torch.all(x[1, 2] == 0)
    assert x[1, 0, 0, 0] == 1 and x[1, 1, 18, 18] == 1          # colours swap with the side to move
    assert torch.equal(R.legal_from_input(x), boards.view(2, -1).eq(0))   # vector_env.py:95-96


def test_oracle_reproduces_committed_golden_vectors():
    import numpy as np
    from pathlib import Path

    g = np.load(Path(__file__).resolve().parent / "golden" / "default_arch_golden.npz")
    x, legal = gen_boards(6, 200, 2025)
    assert np.array_equal(g["x"], x.numpy()) and np.array_equal(g["legal"], legal.numpy())
    for init in ("reference", "torch_default"):
        logits, value = R.forward(R.init_state(1234, init), x)
        assert np.allclose(g[f"{init}_logits"], logits.numpy(), rtol=1e-5, atol=1e-7)
        assert np.allclose(g[f"{init}_value"], value.numpy(), rtol=1e-5, atol=1e-7)
        a, lp = R.sample_inverse_cdf(logits, legal, torch.from_numpy(g["u"]), 1.0)
        assert np.array_equal(g[f"{init}_actions"], a.numpy())


# --------------------------------------------------------------------------
# oracle/lowprec_ref.py: the bf16 + fp6 contract and the cascade's rule
# --------------------------------------------------------------------------
from oracle import lowprec_ref as Q


def _e2m3_codes_by_hand():
    """All 32 non-negative code points from their bit fields, no library involved."""
    out = []
    for code in range(32):
        e, m = code >> 3, code & 7
        out.append((m / 8.0) if e == 0 else (1.0 + m / 8.0) * (2.0 ** (e - 1)))
    return out


def test_e2m3_grid_is_the_enumerated_format():
    grid = Q.e2m3_grid().tolist()
    assert grid == _e2m3_codes_by_hand()
    assert grid == sorted(grid) and len(set(grid)) == 32
    assert grid[0] == 0.0 and grid[1] == 0.125 and grid[8] == 1.0 and grid[-1] == 7.5


def test_quant_e2m3_is_round_to_nearest_even_with_saturation():
    grid = _e2m3_codes_by_hand()
    mids = torch.tensor([(a + b) / 2 for a, b in zip(grid, grid[1:])])   # the ties, exactly representable
    xs = torch.cat([torch.linspace(-9.0, 9.0, 28801), mids, -mids])
    got = Q.quant_e2m3(xs)
    for x, g in zip(xs.tolist(), got.tolist()):
        a = min(abs(x), 7.5)
        best = min(abs(a - v) for v in grid)
        cands = [i for i, v in enumerate(grid) if abs(abs(a - v) - best) < 1e-12]
        want = grid[cands[0]] if len(cands) == 1 else grid[[i for i in cands if i % 2 == 0][0]]  # tie: even mantissa
        assert abs(g) == want and (g == 0 or (g > 0) == (x > 0)), (x, g, want)
    on_grid = torch.tensor(grid + [-v for v in grid])
    assert torch.equal(Q.quant_e2m3(on_grid), on_grid)               # idempotent
    assert Q.quant_e2m3(torch.tensor([7.74, 8.0, 1e9, -1e9])).tolist() == [7.5, 7.5, 7.5, -7.5]


def test_block_scale_is_the_power_of_two_that_puts_the_largest_in_4_to_8():
    m = torch.cat([torch.rand(4000).mul(40).sub(20).exp2(), torch.tensor([1.0, 2.0, 0.5, 2.0 ** -20, 3.999999, 4.0])])
    sc = Q.block_scale(m)
    assert torch.equal(torch.log2(sc), torch.log2(sc).round())       # powers of two
    r = m / sc
    assert bool(((r >= 4.0) & (r < 8.0)).all())
    for v, s in zip(m.tolist()[-6:], sc.tolist()[-6:]):
        assert s == 2.0 ** (math.floor(math.log2(v)) - 2)
    assert float(Q.block_scale(torch.tensor([0.0]))) == 2.0 ** -126  # an all-zero block


def test_quant_lo_blocks_error_is_half_a_step_of_the_block_scale():
    g = torch.Generator().manual_seed(3)
    lo = torch.randn(2, 64, 5, 5, generator=g) * torch.rand(2, 1, 5, 5, generator=g).mul(12).sub(12).exp2()
    lo[0, :32, 0, 0] = 0.0
    q = Q.quant_lo_blocks(lo)
    assert torch.count_nonzero(q[0, :32, 0, 0]) == 0
    v, qv = lo.view(2, 2, 32, 5, 5), q.view(2, 2, 32, 5, 5)
    sc = Q.block_scale(v.abs().amax(2, keepdim=True))
    r = (v / sc).abs()
    step = torch.where(r < 2, 0.125, torch.where(r < 4, 0.25, 0.5))
    ok = ((qv - v).abs() <= 0.5 * step * sc * (1 + 1e-6)) | (r > 7.5)   # saturated elements aside
    assert bool(ok.all())
    assert bool(((qv / sc).abs() <= 7.5).all())


def test_bf16f6_emulation_reduces_to_the_bf16_emulation_and_to_bf16_weights():
    st = R.init_state(4, "reference")
    x, legal = gen_boards(6, 200, 3)
    x[1, 2] = torch.rand(19, 19, generator=torch.Generator().manual_seed(1))     # a varying third plane too
    with torch.inference_mode():
        # no layer corrected: exactly the plain bf16 contract
        l0, v0 = Q.forward_bf16f6_emulated(st, x, lo_mask=0)
        le, ve = R.forward_bf16_emulated(st, x, act_scale=Q.ACT_SCALE, exact_constant_plane=True)
        assert torch.equal(l0, le) and torch.equal(v0, ve)
        # exact low-order parts: the forward with bf16 weights and unrounded activations (the
        # first layer's constant plane aside, which the kernels keep unrounded: both forms here)
        lx, _ = Q.forward_bf16f6_emulated(st, x, exact_lo=True, exact_constant_plane=False)
        stq = {k: (v.to(torch.bfloat16).float() if k.startswith("convs.") and k.endswith("weight") else v)
               for k, v in st.items()}
        # (the first layer's weights are rounded after the activation scale is folded into them)
        stq["convs.0.weight"] = (st["convs.0.weight"] * Q.ACT_SCALE).to(torch.bfloat16).float() / Q.ACT_SCALE
        lw, _ = R.forward(stq, x.to(torch.bfloat16).float())
        assert float((lx - lw).norm() / lw.norm()) < 2e-5
        # the fp6 correction sits between the two
        l6, _ = Q.forward_bf16f6_emulated(st, x, exact_constant_plane=False)
        e_plain = float((le - lw).norm() / lw.norm())
        e_f6 = float((l6 - lw).norm() / lw.norm())
        assert e_f6 < 0.25 * e_plain
        # with the weights' low part as well ("bf16f6w"): exact low-order parts give the fp32
        # forward up to the second rounding of the weights (2^-16 relative each), ...
        # (input planes are bf16 operands of the first layer in every 16-bit mode: stones are exact)
        lf, vf = R.forward(st, x.to(torch.bfloat16).float())
        ly, vy = Q.forward_bf16f6_emulated(st, x, exact_lo=True, weights_lo=True, exact_constant_plane=False)
        assert float((ly - lf).norm() / lf.norm()) < 3e-5 and float((vy - vf).norm() / vf.norm()) < 3e-5
        # ... and the e2m3 roundings of the activations' low part leave a few 1e-4
        lz, _ = Q.forward_bf16f6_emulated(st, x, weights_lo=True, exact_constant_plane=False)
        e_w = float((lz - lf).norm() / lf.norm())
        assert 2e-5 < e_w < 5e-4 and e_w < 0.1 * float((l6 - lf).norm() / lf.norm())


def test_cascade_rule_against_a_plain_python_loop():
    g = torch.Generator().manual_seed(9)
    logits = torch.randn(40, 361, generator=g) * torch.rand(40, 1, generator=g) + 3.0 * torch.randn(40, 1, generator=g)
    free = torch.rand(40, 361, generator=g) < 0.6
    logits[0] = 0.25                                   # flat: no spread, no second pass
    free[1] = False; free[1, 17] = True                # one free square: nothing to decide
    free[2] = False                                    # none
    logits[3, 5] = logits[3, 200] = 50.0; free[3, 5] = free[3, 200] = True   # a tie at the top
    free[4] = False; free[4, 3] = free[4, 300] = True  # two free squares: no third to look at
    logits[5] = 0.0; free[5] = True; logits[5, 360] = 1.0                      # a clear lead of the best ...
    logits[5, 359] = logits[5, 358] = 1.0 - 0.0041                             # ... but two others close behind
    for thr in (0.0, 0.03, 0.5, -1.0):
        got = Q.cascade_second_pass(logits, free, thr).tolist()
        for b in range(40):
            z = sorted((float(logits[b, i]) for i in range(361) if bool(free[b, i])), reverse=True)
            if len(z) < 2:
                want = False
            elif thr < 0:
                want = True
            else:
                mean = sum(z) / len(z)
                std = math.sqrt(sum((v - mean) ** 2 for v in z) / len(z))
                want = (z[0] - z[1]) < thr * std or (len(z) >= 3 and (z[0] - z[2]) < 2 * thr * std)
            assert got[b] == want, (thr, b)
    assert Q.cascade_second_pass(logits, free, 0.03)[3] and not Q.cascade_second_pass(logits, free, 0.03)[0]
    # board 5: lead 0.0041 = 0.045 standard deviations: not below 0.03, but two squares within 0.06
    assert Q.cascade_second_pass(logits, free, 0.03)[5] and not Q.cascade_second_pass(logits, free, 0.02)[5]
