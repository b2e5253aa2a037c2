"""Parity of the HBM-bound kernels around the forward: stand-alone masking,
sampling, the fused self-play step and the D4 view kernels."""
import pytest
import torch

import connect6_amd as c6
from connect6_amd.synthetic import gen_boards, gen_uniform
from oracle import torch_ref as R
from tests.util import rel_l2

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("batch", [1, 7, 4096])
def test_mask_logits_bit_exact(cuda, dtype, batch):
    g = torch.Generator().manual_seed(batch)
    logits = torch.randn(batch, 361, generator=g).to(dtype)
    _, legal = gen_boards(batch, 300, batch + 1)
    out = c6.mask_logits(logits.to(cuda), legal.to(cuda)).cpu()
    want = R.mask_logits(logits, legal)          # connect6/model.py:123-125
    itype = torch.int32 if dtype == torch.float32 else torch.int16
    assert out.dtype == dtype
    assert torch.equal(out.view(itype), want.view(itype))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mask_logits_takes_row_slices(cuda, dtype):
    """A contiguous row slice starts 361 elements into its tensor, so it is not 16-byte aligned;
    the reference's torch.where accepts it (connect6/model.py:123-125) and so does this."""
    logits = torch.randn(9, 361, generator=torch.Generator().manual_seed(3)).to(dtype)
    _, legal = gen_boards(9, 300, 4)
    lg, ll = logits.to(cuda), legal.to(cuda)
    for lo in (1, 2, 3):
        out = c6.mask_logits(lg[lo:], ll[lo:]).cpu()
        want = R.mask_logits(logits[lo:], legal[lo:])
        itype = torch.int32 if dtype == torch.float32 else torch.int16
        assert torch.equal(out.view(itype), want.view(itype))


def _check_samples(actions, logprob, logits, legal, u, temperature):
    a_ref, lp_ref = R.sample_inverse_cdf(logits, legal, u, temperature)
    actions, logprob = actions.cpu(), logprob.cpu()
    assert bool(legal.gather(1, actions.view(-1, 1)).all())        # never an occupied square
    same = actions == a_ref
    assert float(same.float().mean()) >= 0.999
    # a disagreement is only legitimate when u sits on a CDF step (summation order differs)
    z = R.mask_logits(logits.float(), legal) / max(temperature, 1e-4)
    p = torch.softmax(z.double(), 1)
    cdf = torch.cumsum(p, 1)
    for b in torch.nonzero(~same).flatten().tolist():
        lo, hi = sorted((int(actions[b]), int(a_ref[b])))
        edge = cdf[b, lo:hi]
        assert float((edge - float(u[b])).abs().min()) < 1e-5
    assert torch.allclose(logprob[same], lp_ref[same], atol=2e-4, rtol=1e-4)


@pytest.mark.parametrize("temperature", [1.0, 0.35])
def test_softmax_sample_matches_oracle(cuda, temperature):
    b = 4096
    logits = torch.randn(b, 361, generator=torch.Generator().manual_seed(1)) * 3
    _, legal = gen_boards(b, 300, 3)
    u = gen_uniform(b, 7)
    actions, logprob = c6.sample_actions(logits.to(cuda), legal.to(cuda), temperature, u.to(cuda))
    assert actions.dtype == torch.int64 and actions.shape == (b,)
    _check_samples(actions, logprob, logits, legal, u, temperature)
    only = c6.sample_actions(logits.to(cuda), legal.to(cuda), temperature, u.to(cuda), return_logprob=False)
    assert torch.equal(only, actions)
    nomask = c6.sample_actions(logits.to(cuda), None, temperature, u.to(cuda), return_logprob=False)
    a_ref, _ = R.sample_inverse_cdf(logits, torch.ones_like(legal), u, temperature)
    assert float((nomask.cpu() == a_ref).float().mean()) >= 0.999


def test_sample_edge_cases(cuda):
    logits = torch.zeros(4, 361)
    legal = torch.zeros(4, 361, dtype=torch.bool)
    legal[0, 360] = True                 # a single legal square, the last one
    legal[1, 0] = True                   # a single legal square, the first one
    legal[2, 100] = legal[2, 200] = True
    legal[3, :] = True
    u = torch.tensor([0.5, 0.999, 0.75, 0.0])
    a, lp = c6.sample_actions(logits.to(cuda), legal.to(cuda), 1.0, u.to(cuda))
    assert a.cpu().tolist() == [360, 0, 200, 0]
    assert torch.allclose(lp.cpu(), torch.log(torch.tensor([1.0, 1.0, 0.5, 1 / 361])), atol=1e-5)


@pytest.mark.parametrize("prec", ["bf16f6", "bf16c"])
def test_fused_selfplay_step_cfg4(cuda, prec):
    """B=16384, stones 0..300: forward + mask + softmax + draw in one launch, in the headline
    arithmetic mode (the one the benchmark times) and in the hi+lo bf16 mode."""
    b = 16384
    st = R.init_state(1234, "reference")
    x, legal = gen_boards(b, 300, 2025)
    u = gen_uniform(b, 7)
    model = c6.PolicyValueNet().to(cuda).eval()
    model.load_state_dict(st)
    model.precision = prec
    with torch.inference_mode():
        actions, logprob, value, masked = model.selfplay_step(x.to(cuda), u.to(cuda), 1.0, return_logits=True)
        a2, lp2, v2 = model.selfplay_step(x.to(cuda), u.to(cuda), 1.0)
        plain, v3 = model(x.to(cuda))
    assert torch.equal(actions, a2) and torch.equal(value, v2) and torch.equal(value, v3)
    assert torch.equal(masked.cpu(), R.mask_logits(plain.cpu(), legal))
    # the draw is the oracle's inverse CDF applied to the logits the kernel produced
    _check_samples(actions, logprob, plain.cpu(), legal, u, 1.0)
    # and the stand-alone kernel agrees with the fused one on the same logits
    a3, lp3 = c6.sample_actions(plain, legal.to(cuda), 1.0, u.to(cuda))
    assert torch.equal(a3, actions) and torch.allclose(lp3, logprob, atol=1e-6)
    # a small fp32 slice end-to-end against the fp32 oracle forward
    model.precision = None
    with torch.inference_mode():
        a4, lp4, v4 = model.selfplay_step(x[:256].to(cuda), u[:256].to(cuda), 0.8)
        lo, vo = R.forward(st, x[:256])
    a_ref, lp_ref = R.sample_inverse_cdf(lo, legal[:256], u[:256], 0.8)
    assert float((a4.cpu() == a_ref).float().mean()) >= 0.98   # logits differ by ~1e-6 relative
    assert rel_l2(v4, vo) <= 1e-4
    # the 16-bit mode's own logits and value against the fp32 oracle on a slice the CPU does quickly
    with torch.inference_mode():
        lo2, vo2 = R.forward(st, x[:1024])
    assert rel_l2(plain[:1024].cpu()[legal[:1024]], lo2[legal[:1024]]) <= 2e-2
    assert rel_l2(value[:1024], vo2) <= 2e-2


@pytest.mark.parametrize("batch", [37, 44, 64])   # views not 16-byte aligned / whole groups of 32 planes + a partial one / whole groups
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_d4_expand_matches_oracle(cuda, dtype, batch):
    x = torch.randn(batch, 3, 19, 19, generator=torch.Generator().manual_seed(2)).to(dtype)
    views = c6.d4_expand(x.to(cuda)).cpu()
    assert views.shape == (8, batch, 3, 19, 19)
    assert torch.equal(views, R.d4_expand(x))
    for p in range(8):    # and the library routines the reference uses (train.py:222-230)
        k, flip = R.symmetry_for_phase(p)
        lib = torch.rot90(x, k=k, dims=(-2, -1)) if k else x
        lib = torch.flip(lib, dims=(-1,)) if flip else lib
        assert torch.equal(views[p], lib)


def test_d4_reduce_matches_oracle(cuda):
    vl = torch.randn(8, 129, 361, generator=torch.Generator().manual_seed(3))
    vv = torch.randn(8, 129, generator=torch.Generator().manual_seed(4))
    logits, values = c6.d4_reduce(vl.to(cuda), vv.to(cuda))
    lo, vo = R.d4_average(vl, vv)
    assert torch.allclose(logits.cpu(), lo, atol=1e-6) and torch.allclose(values.cpu(), vo, atol=1e-6)
    only, none = c6.d4_reduce(vl.to(cuda), None)
    assert none is None and torch.equal(only, logits)


@pytest.mark.parametrize("prec", ["bf16f6", "bf16c"])
def test_d4_evaluation_cfg5(cuda, prec):
    st = R.init_state(1234, "reference")
    model = c6.PolicyValueNet().to(cuda).eval()
    model.load_state_dict(st)
    # small slice in fp32 against the oracle pipeline
    x, _ = gen_boards(64, 200, 2025)
    with torch.inference_mode():
        lg, vg = c6.evaluate_d4(model, x.to(cuda))
        views = R.d4_expand(x)
        lv, vv = R.forward(st, views.reshape(8 * 64, 3, 19, 19))
        lo, vo = R.d4_average(lv.view(8, 64, 361), vv.view(8, 64))
    assert rel_l2(lg, lo) <= 1e-4 and rel_l2(vg, vo) <= 1e-4
    # full size (8192 base boards -> 65536 views) through a size-independent property:
    # the D4 average is invariant to presenting the board in another orientation
    model.precision = prec
    x, _ = gen_boards(8192, 200, 2025)
    xd = x.to(cuda)
    with torch.inference_mode():
        base_l, base_v = c6.evaluate_d4(model, xd)
        k, flip = R.symmetry_for_phase(5)
        rot_l, rot_v = c6.evaluate_d4(model, c6.transform_boards(xd, k, flip).contiguous())
        # ... and a slice of the 16-bit result against the fp32 oracle pipeline
        views = R.d4_expand(x[:128])
        lv, vv = R.forward(st, views.reshape(8 * 128, 3, 19, 19))
        lo, vo = R.d4_average(lv.view(8, 128, 361), vv.view(8, 128))
    a = torch.arange(361, device=cuda)
    back = rot_l[:, c6.transform_actions(a, 19, k, flip)]
    assert torch.allclose(back, base_l, atol=1e-6) and torch.allclose(rot_v, base_v, atol=1e-6)
    assert rel_l2(base_l[:128], lo) <= 2e-2 and rel_l2(base_v[:128], vo) <= 2e-2


def _random_states(n, seed):
    g = torch.Generator().manual_seed(seed)
    x, _ = gen_boards(n, 250, seed)
    player = (torch.randint(0, 2, (n,), generator=g) * 2 - 1).to(torch.int8)
    # planes are side-to-move relative; rebuild absolute colours
    boards = ((x[:, 0] - x[:, 1]) * player.view(-1, 1, 1).float()).to(torch.int8)
    left = torch.randint(1, 3, (n,), generator=g).to(torch.int8)
    return boards, player, left


@pytest.mark.parametrize("view", [0, 3, 6])
def test_forward_from_board_states(cuda, view):
    """Collector step from the environment's int8 state: view, canonical input, gather, forward, mask."""
    st = R.init_state(1234, "reference")
    model = c6.PolicyValueNet().to(cuda).eval()
    model.load_state_dict(st)
    boards, player, left = _random_states(300, 5)
    index = torch.randperm(300, generator=torch.Generator().manual_seed(1))[:200]
    k, flip = R.symmetry_for_phase(view)
    view_boards = R.transform_boards(boards, k, flip)               # train.py:730-741
    x = R.canonical_network_input(view_boards, player, left)        # train.py:743-747
    legal = view_boards.reshape(300, -1).eq(0)                      # train.py:748
    with torch.inference_mode():
        lo, vo = R.forward(st, x[index])                            # train.py:791-794
        lg, vg = model.forward_boards(boards.to(cuda), player.to(cuda), left.to(cuda),
                                      index=index.to(cuda), view=view)
        plain, _ = model.forward_boards(boards.to(cuda), player.to(cuda), left.to(cuda),
                                        index=index.to(cuda), view=view, masked=False)
        same, vsame = model.forward_masked(x[index].to(cuda))      # float-plane entry point, same kernel
    assert rel_l2(plain, lo) <= 1e-4 and rel_l2(vg, vo) <= 1e-4
    assert torch.equal(lg.cpu(), R.mask_logits(plain.cpu(), legal[index]))   # bit-exact masking
    assert torch.equal(lg, same) and torch.equal(vg, vsame)
    # whole batch, no gather, with the fused draw
    u = gen_uniform(300, 2)
    model.precision = "bf16f6"
    with torch.inference_mode():
        a, lp, v = model.selfplay_step_boards(boards.to(cuda), player.to(cuda), left.to(cuda), u.to(cuda),
                                              0.9, view=view)
        a2, lp2, v2 = model.selfplay_step(x.to(cuda), u.to(cuda), 0.9)
    assert torch.equal(a, a2) and torch.equal(lp, lp2) and torch.equal(v, v2)
    assert bool(legal.gather(1, a.cpu().view(-1, 1)).all())
    back = c6.inverse_transform_actions(a.cpu(), 19, k, flip)       # train.py:854-862
    assert bool((boards.reshape(300, -1).gather(1, back.view(-1, 1)) == 0).all())


def test_forward_boards_argument_checks(cuda):
    model = c6.PolicyValueNet().to(cuda).eval()
    boards, player, left = (t.to(cuda) for t in _random_states(4, 1))
    with torch.inference_mode():
        with pytest.raises(ValueError):
            model.forward_boards(boards.float(), player, left)
        with pytest.raises(ValueError):
            model.forward_boards(boards, player[:3], left)
        with pytest.raises(ValueError):
            model.forward_boards(boards, player, left, view=8)
        # rows outside [0, N) are clamped into range by the kernel (never read out of bounds)
        lc, _ = model.forward_boards(boards, player, left, index=torch.tensor([-3, 9], device=cuda))
        le, _ = model.forward_boards(boards, player, left, index=torch.tensor([0, 3], device=cuda))
        assert torch.equal(lc, le)
        logits, value = model.forward_boards(boards, player, left, index=torch.zeros(0, dtype=torch.int64, device=cuda))
        assert logits.shape == (0, 361) and value.shape == (0,)
