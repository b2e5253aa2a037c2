"""The cascade mode ("bf16c") through the C ABI: every board in plain bf16, the boards whose
decision is closer than the rounding noise again with the low parts of activations and weights
carried ("bf16f6w").

What is checked: the two extremes of the threshold reproduce the two modes bit for bit; every
output row is one of the two modes' rows and the choice follows the stated rule
(oracle.lowprec_ref.cascade_second_pass on the first pass's logits); the parity gates of the
16-bit paths (<= 2e-2 relative L2, >= 99 % argmax agreement on masked logits against the fp32
oracle); a board's result does not depend on the batch around it; grouped weight sets, int8
board-state input and the fused sampling go through the same two passes.
"""
import ctypes

import pytest
import torch

import connect6_amd as c6
from connect6_amd import _lib
from connect6_amd.synthetic import gen_boards, gen_uniform
from oracle import lowprec_ref as Q
from oracle import torch_ref as R
from tests.util import argmax_agreement, rel_l2

pytestmark = pytest.mark.gpu

BF16_TOL = 2e-2
ARGMAX_MIN = 0.99


def make_model(dev, state, precision, threshold=None):
    m = c6.PolicyValueNet().to(dev).eval()
    m.load_state_dict(state)
    m.precision = precision
    m.cascade_threshold = threshold
    return m


def second_pass(model) -> int:
    return int(model.cascade_stats["second_pass"].item())


def test_threshold_extremes_reproduce_the_two_modes(cuda):
    st = R.init_state(1234, "reference")
    x, legal = gen_boards(700, 200, 2025)
    u = gen_uniform(700, 3)
    xd, ud = x.to(cuda), u.to(cuda)
    with torch.inference_mode():
        plain = make_model(cuda, st, "bf16")
        fine = make_model(cuda, st, "bf16f6w")
        for thr, other in ((0.0, plain), (-1.0, fine)):
            m = make_model(cuda, st, "bf16c", thr)
            for call in (lambda mm: mm(xd), lambda mm: mm.forward_masked(xd),
                         lambda mm: mm.forward_masked(xd, legal.to(cuda), fill=float("-inf"))):
                got, want = call(m), call(other)
                assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
                assert second_pass(m) == (0 if thr == 0.0 else 700)
            got, want = m.selfplay_step(xd, ud, 0.7), other.selfplay_step(xd, ud, 0.7)
            assert all(torch.equal(a, b) for a, b in zip(got, want))


@pytest.mark.parametrize("init", ["reference", "torch_default"])
def test_rows_follow_the_rule_and_keep_the_gates_b4096(cuda, init):
    torch.set_num_threads(16)
    st = R.init_state(1234, init)
    x, legal = gen_boards(4096, 200, 2025)
    xd = x.to(cuda)
    with torch.inference_mode():
        lo, vo = R.forward(st, x)
        lb, vb = make_model(cuda, st, "bf16")(xd)
        lf, vf = make_model(cuda, st, "bf16f6w")(xd)
        m = make_model(cuda, st, "bf16c")              # default threshold
        lc, vc = m(xd)
    lb, lf, lc, vb, vf, vc = (t.cpu() for t in (lb, lf, lc, vb, vf, vc))
    n2 = second_pass(m)
    # every row is the first pass's or the second pass's, value included
    from_f6 = (lc == lf).all(1) & (vc == vf)
    from_b = (lc == lb).all(1) & (vc == vb)
    assert bool((from_f6 | from_b).all())
    # ... chosen by the rule, judged on the first pass's logits (boards within 2 % of a
    # threshold aside: the kernel sums in fp32 and in another order)
    gap2, gap3, std = Q.cascade_margin(lb, legal)
    thr = _lib.CASCADE_THRESHOLD
    want = Q.cascade_second_pass(lb, legal, thr)
    near = lambda g, t: (g > 0.98 * t * std) & (g < 1.02 * t * std)
    clear = ~(near(gap2, thr) | near(gap3, 2 * thr))
    took_second = from_f6 & ~from_b                    # (rows equal in both modes tell nothing)
    took_first = from_b & ~from_f6
    assert not bool((took_second & ~want & clear).any())
    assert not bool((took_first & want & clear).any())
    assert abs(n2 - int(want.sum())) <= int((~clear).sum())
    # the gates
    assert rel_l2(lc, lo) <= BF16_TOL and rel_l2(vc, vo) <= BF16_TOL
    masked = lambda t: R.mask_logits(t, legal)
    agree = argmax_agreement(masked(lc), masked(lo))
    agree_f6 = argmax_agreement(masked(lf), masked(lo))
    print(f"{init}: second pass {n2} of 4096 ({n2 / 4096:.3f}); argmax agreement cascade {agree:.4f}, "
          f"second pass's arithmetic on every board {agree_f6:.4f}, bf16 {argmax_agreement(masked(lb), masked(lo)):.4f}")
    assert agree >= ARGMAX_MIN
    assert agree >= agree_f6 - 0.003                   # what the threshold is allowed to cost
    if init == "reference":
        assert agree >= 0.996                          # (measured 0.9988)
    if init == "reference":
        assert n2 <= 0.10 * 4096                       # the cascade pays: few boards go twice


def test_cascade_for_parameters_held_in_bf16(cuda):
    """"bf16c6": the cascade whose second pass leaves the weights' low part out, for parameters that
    are exact in bf16 (what a bf16 module or ensemble holds).  Its extremes are bf16 and bf16f6;
    on such parameters "bf16c" lists the same boards and its second pass multiplies the
    activations with low parts that are all zero -- except in the first layer, whose weights are
    rounded after the activation scale is folded in: that is all that separates the two."""
    st = {k: v.to(torch.bfloat16).float() for k, v in R.init_state(1234, "reference").items()}
    x, legal = gen_boards(1500, 200, 2025)
    xd = x.to(cuda)
    with torch.inference_mode():
        plain, fine = make_model(cuda, st, "bf16"), make_model(cuda, st, "bf16f6")
        for thr, other in ((0.0, plain), (-1.0, fine)):
            m = make_model(cuda, st, "bf16c6", thr)
            got, want = m.forward_masked(xd), other.forward_masked(xd)
            assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
        a, b = make_model(cuda, st, "bf16c6"), make_model(cuda, st, "bf16c")
        la, va = a.forward_masked(xd)
        lb, vb = b.forward_masked(xd)
        assert 0 < second_pass(a) == second_pass(b) < 150
        once = (la == make_model(cuda, st, "bf16").forward_masked(xd)[0]).all(1)
        assert torch.equal(la[once], lb[once]) and int((~once).sum()) <= second_pass(a)
        assert rel_l2(la[~once].cpu().masked_fill(~legal[~once.cpu()], 0), lb[~once].cpu().masked_fill(~legal[~once.cpu()], 0)) <= 3e-3
        assert rel_l2(va, vb) <= 3e-3
        # a module that holds its parameters in bf16 picks it by itself
        held = c6.PolicyValueNet().to(cuda).eval()
        held.load_state_dict(st)
        held = held.to(torch.bfloat16)
        assert held.resolve_precision() == _lib.PREC_BF16C6
        lh, vh = held.forward_masked(xd.to(torch.bfloat16))
        assert torch.equal(lh, la) and torch.equal(vh, va)


def test_a_boards_result_does_not_depend_on_the_batch(cuda):
    st = R.init_state(11, "reference")
    x, legal = gen_boards(1000, 200, 77)
    xd, ld = x.to(cuda), legal.to(cuda)
    u = gen_uniform(1000, 5).to(cuda)
    m = make_model(cuda, st, "bf16c", 0.2)             # a wide threshold: many boards go twice
    with torch.inference_mode():
        lg, vg = m.forward_masked(xd, ld)
        assert 50 < second_pass(m) < 950
        ag, pg, _ = m.selfplay_step(xd, u, 0.8, legal=ld)
        for n in (1, 3, 255, 257, 513, 999):
            l, v = m.forward_masked(xd[:n], ld[:n])
            assert torch.equal(l, lg[:n]) and torch.equal(v, vg[:n]), n
            a, p, _ = m.selfplay_step(xd[:n], u[:n], 0.8, legal=ld[:n])
            assert torch.equal(a, ag[:n]) and torch.equal(p, pg[:n]), n
        # the same from int8 board states
        boards = (x[:, 0] - x[:, 1]).to(torch.int8).to(cuda)
        player = torch.ones(1000, dtype=torch.int8, device=cuda)
        left = (x[:, 2, 0, 0] == 1).to(torch.int8).to(cuda)   # plane 2 = (stones_left == 1)
        lb, vb = m.forward_boards(boards, player, left)
        assert torch.equal(lb, m.forward_masked(xd)[0]) and torch.equal(vb, vg)


def test_grouped_sets_go_through_both_passes(cuda):
    from pathlib import Path

    torch.set_num_threads(16)
    cfg = {"architecture_version": 4, "kernels": list(R.DEFAULT_KERNELS), "channels": list(R.DEFAULT_CHANNELS)}
    cps = [c6.HistoricalCheckpoint(path=Path(f"model_update_{i + 1:08d}.pt"), update=i + 1,
                                   model_state=R.init_state(1234 + i, "reference"), model_config=cfg,
                                   game_config={"board_size": 19, "win_length": 6}) for i in range(8)]
    x, legal = gen_boards(4096, 200, 2025)
    xg, lg = x.view(8, 512, 3, 19, 19), legal.view(8, 512, 361)
    ens = c6.HistoricalPolicyEnsemble(cps, cuda, dtype=torch.bfloat16, precision="bf16c")
    with torch.inference_mode():
        from connect6_amd.model import run_forward

        stats = {}
        raw, _, _, _ = run_forward(xg.to(cuda).reshape(4096, 3, 19, 19).to(torch.bfloat16), ens._packed_weights(),
                                   ens._prec, 8, 512, want_value=False, stats=stats)
        grouped = ens.forward_grouped(xg.to(cuda))
        assert torch.equal(grouped, raw.view(8, 512, 361).to(torch.bfloat16))
        n2 = int(stats["second_pass"].item())
        assert 0 < n2 < 0.10 * 4096
        raw = raw.view(8, 512, 361).cpu()
        for i, cp in enumerate(cps):
            st16 = {k: v.to(torch.bfloat16).float() for k, v in cp.model_state.items()}
            expected, _ = R.forward(st16, xg[i])
            assert rel_l2(raw[i], expected) <= BF16_TOL
            assert argmax_agreement(R.mask_logits(raw[i], lg[i]), R.mask_logits(expected, lg[i])) >= ARGMAX_MIN
            # group i of the grouped launch == the single-model launch on its boards
            single = make_model(cuda, st16, "bf16c")(xg[i].to(cuda))[0]
            assert torch.equal(single.cpu(), raw[i])


def test_cascade_entry_points_check_their_workspace(cuda):
    lib = c6.load()
    n = ctypes.c_size_t(0)
    assert lib.c6_cascade_workspace_bytes(100, ctypes.byref(n)) == 0 and n.value >= 16 + 400 and n.value % 16 == 0
    st = R.init_state(1, "reference")
    m = make_model(cuda, st, "bf16c")
    packed = m.packed_weights(_lib.PREC_BF16C)
    x = gen_boards(100, 200, 1)[0].to(cuda)
    out = torch.empty(100, 361, device=cuda)
    small = torch.empty(16, dtype=torch.int32, device=cuda)
    args = (x.data_ptr(), _lib.DT_F32, 1, 100, packed.data_ptr(), packed.numel(), _lib.PREC_BF16C, out.data_ptr(),
            _lib.DT_F32, None, _lib.MASK_NONE, None, 0.0, None, 1.0, None, None, 0.03)
    rc = lib.c6_forward_cascade(*args, small.data_ptr(), small.numel() * 4, _lib.stream_ptr(cuda))
    assert rc == -1 and b"workspace" in lib.c6_last_error()
    rc = lib.c6_forward_cascade(*args, None, 1 << 20, _lib.stream_ptr(cuda))
    assert rc == -1
    # the plain entry point refuses the cascade's mode (it has no workspace to give it)
    rc = lib.c6_forward(x.data_ptr(), _lib.DT_F32, 1, 100, packed.data_ptr(), packed.numel(), _lib.PREC_BF16C,
                        out.data_ptr(), None, _lib.MASK_NONE, None, 0.0, None, 1.0, None, None, _lib.stream_ptr(cuda))
    assert rc == -1 and b"c6_forward_cascade" in lib.c6_last_error()


def test_grouped_pack_equals_one_pack_per_model(cuda):
    """c6_pack_weights_grouped (all checkpoints of an ensemble in two launches, from the stacked
    tensors) writes what c6_pack_weights writes model by model, in every arithmetic mode."""
    from pathlib import Path

    from connect6_amd.model import pack_state

    cfg = {"architecture_version": 4, "kernels": list(R.DEFAULT_KERNELS), "channels": list(R.DEFAULT_CHANNELS)}
    cps = [c6.HistoricalCheckpoint(path=Path(f"m{i}.pt"), update=i + 1, model_state=R.init_state(50 + i, "torch_default"),
                                   model_config=cfg, game_config={"board_size": 19, "win_length": 6}) for i in range(5)]
    first = _lib.packed_bytes(_lib.PREC_BF16)
    second_at = (first + 255) // 256 * 256
    for name, dtype in (("fp32", torch.float32), ("bf16", torch.bfloat16), ("fp16", torch.float16),
                        ("bf16f6", torch.bfloat16), ("bf16f6w", torch.bfloat16), ("bf16c", torch.bfloat16),
                        ("bf16c6", torch.bfloat16)):
        ens = c6.HistoricalPolicyEnsemble(cps, cuda, dtype=dtype, precision=name)
        packed = ens._packed_weights()
        one = _lib.packed_bytes(ens._prec)
        assert packed.shape == (5, one)
        # bytes every mode defines: all fragments and the fp32 tail; the eight scale words behind
        # it only where a low-order copy exists; the cascade's alignment gap not at all
        if name in ("bf16c", "bf16c6"):
            spans = [(0, first - 32), (second_at, one)]
        else:
            spans = [(0, one if name in ("bf16f6", "bf16f6w") else one - 32)]
        for m in range(5):
            alone = torch.empty(one, dtype=torch.uint8, device=cuda)
            pack_state(ens._model_state(m), ens._prec, alone)
            for a, b in spans:
                assert torch.equal(packed[m, a:b], alone[a:b]), (name, m, a, b)
