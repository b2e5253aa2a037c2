"""Non-default architectures (any board / kernels / channels the reference's
PolicyValueNet accepts) run through the layer-by-layer HIP path."""
from pathlib import Path

import pytest
import torch

import connect6_amd as c6
from oracle import cref
from oracle import torch_ref as R
from tests.util import rel_l2

pytestmark = pytest.mark.gpu


def _lib_prec(dtype):
    from connect6_amd import _lib
    return _lib.PREC_F32 if dtype == torch.float32 else _lib.PREC_BF16


def test_grouped_history_matches_individual_models_reference_test_shape(cuda):
    # tests/test_training_features.py:120-151 of the reference, on the GPU
    torch.manual_seed(123)
    board_size = 5
    model_cfg = {"architecture_version": 4, "kernels": [3, 3, 3], "channels": [8, 8, 16],
                 "compile": False, "compile_mode": "default"}
    game_cfg = {"board_size": board_size, "win_length": 3}
    models = [c6.build_model(model_cfg, board_size).to(cuda) for _ in range(2)]
    checkpoints = [
        c6.HistoricalCheckpoint(path=Path(f"model_update_{i + 1:08d}.pt"), update=i + 1,
                                model_state=model.state_dict(), model_config=model_cfg,
                                game_config=game_cfg)
        for i, model in enumerate(models)
    ]
    ensemble = c6.HistoricalPolicyEnsemble(checkpoints, cuda)
    x = torch.randn(2, 5, 3, board_size, board_size)
    with torch.inference_mode():
        grouped = ensemble.forward_grouped(x.to(cuda))
        assert grouped.shape == (2, 5, 25)
        for i, model in enumerate(models):
            model.eval()
            got, value = model(x[i].to(cuda))
            assert torch.allclose(grouped[i], got, atol=1e-5, rtol=1e-5)
            state = {k: v.cpu() for k, v in model.state_dict().items()}
            expected, vexp = R.forward(state, x[i])
            assert torch.allclose(grouped[i].cpu(), expected, atol=1e-5, rtol=1e-5)
            assert torch.allclose(value.cpu(), vexp, atol=1e-5, rtol=1e-5)
            assert torch.all(value <= 1) and torch.all(value >= -1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_grouped_generic_is_one_launch_per_layer_and_equals_model_by_model(cuda, dtype):
    """An ensemble of a non-default architecture goes through c6_forward_generic_grouped (the
    stacked parameters, every layer one launch for all models, as connect6/history.py:263-273) and
    gives, bit for bit, what c6_forward_generic gives model by model."""
    from connect6_amd.model import run_forward_generic

    board, kernels, channels = 9, [5, 3, 1], [16, 24, 7]
    cfg = {"architecture_version": 4, "kernels": kernels, "channels": channels}
    cps = [c6.HistoricalCheckpoint(path=Path(f"m{i}.pt"), update=i + 1,
                                   model_state=R.init_state(70 + i, "torch_default", kernels=kernels, channels=channels),
                                   model_config=cfg, game_config={"board_size": board, "win_length": 6})
           for i in range(5)]
    ens = c6.HistoricalPolicyEnsemble(cps, cuda, dtype=dtype)
    assert not ens.is_default_architecture
    x = torch.randn(5, 7, 3, board, board, generator=torch.Generator().manual_seed(9))
    x[:, :, :2] = (x[:, :, :2] > 0.8).float()
    with torch.inference_mode():
        grouped = ens.forward_grouped(x.to(cuda))
        assert grouped.shape == (5, 7, board * board) and grouped.dtype == dtype
        for i, cp in enumerate(cps):
            single = run_forward_generic(x[i].to(cuda).to(dtype), ens._model_state(i), kernels, channels, ens._prec,
                                         want_value=False)[0]
            assert torch.equal(grouped[i], single.to(dtype)), i
            want, _ = R.forward({k: v.to(dtype).float() for k, v in cp.model_state.items()}, x[i].to(dtype).float())
            assert rel_l2(grouped[i].float().cpu(), want) <= (1e-5 if dtype == torch.float32 else 2e-2)
    # the value head of every weight set too (an ensemble asks for policies only): stacked
    # parameters of three models through the grouped entry point against model-by-model calls
    states = [R.init_state(90 + i, "torch_default", kernels=kernels, channels=channels) for i in range(3)]
    stacked = {k: torch.stack([st[k] for st in states]).to(cuda) for k in states[0]}
    xs = x[:3].to(cuda)
    with torch.inference_mode():
        lg, vg = run_forward_generic(xs.reshape(21, 3, board, board), stacked, kernels, channels, _lib_prec(dtype),
                                     groups=3, mask_mode=1)
        for i, st in enumerate(states):
            l1, v1 = run_forward_generic(xs[i], {k: v.to(cuda) for k, v in st.items()}, kernels, channels,
                                         _lib_prec(dtype), mask_mode=1)
            assert torch.equal(lg[7 * i:7 * i + 7], l1) and torch.equal(vg[7 * i:7 * i + 7], v1), i
    # argument checks of the grouped entry point
    import ctypes

    from connect6_amd import _lib
    lib = c6.load()
    ints = ctypes.c_int * 3
    rc = lib.c6_forward_generic_grouped(None, 0, 0, 7, board, 3, ints(*kernels), ints(*channels), None, None, None,
                                        None, None, None, 0, None, 0, None, None, 0, None, 0.0, None)
    assert rc == -1 and b"groups" in lib.c6_last_error()
    rc = lib.c6_forward_generic_grouped(None, 0, 5, 0, board, 3, ints(*kernels), ints(*channels), None, None, None,
                                        None, None, None, 0, None, 0, None, None, 0, None, 0.0, None)
    assert rc == 0                                          # no boards: nothing to do


@pytest.mark.parametrize("board,kernels,channels", [(9, [5, 3, 1], [16, 24, 7]), (19, [7, 3], [5, 33])])
def test_other_architectures_match_oracle_and_bruteforce(cuda, board, kernels, channels):
    st = R.init_state(11, "torch_default", kernels=kernels, channels=channels)
    model = c6.PolicyValueNet(board_size=board, kernels=kernels, channels=channels).to(cuda).eval()
    model.load_state_dict(st)
    assert not model.is_default_architecture
    x = torch.randn(6, 3, board, board, generator=torch.Generator().manual_seed(3))
    x[:, :2] = (x[:, :2] > 0.8).float()                    # stone planes
    legal = ((x[:, 0] == 0) & (x[:, 1] == 0)).flatten(1)
    with torch.inference_mode():
        lo, vo = R.forward(st, x)
        lc, vc = cref.forward(st, x[:2])
        lg, vg = model(x.to(cuda))
        lm, _ = model.forward_masked(x.to(cuda))
        ll, _ = model.forward_masked(x.to(cuda), legal.to(cuda), fill=float("-inf"))
    assert lg.shape == (6, board * board) and vg.shape == (6,)
    assert rel_l2(lg, lo) <= 1e-5 and rel_l2(vg, vo) <= 1e-5
    assert rel_l2(lg[:2], lc) <= 1e-5 and rel_l2(vg[:2], vc) <= 1e-5
    assert torch.equal(lm.cpu(), R.mask_logits(lg.cpu(), legal))            # bit-exact fill / pass-through
    assert torch.equal(torch.isneginf(ll.cpu()), ~legal)
    # 16-bit contracts: same roundings as the emulation in the oracle
    model.precision = "bf16"
    with torch.inference_mode():
        lb, vb = model(x.to(cuda))
        le, ve = R.forward_bf16_emulated(st, x)
    assert rel_l2(lb, le) <= 2e-3 and rel_l2(lb, lo) <= 2e-2 and rel_l2(vb, vo) <= 2e-2


def test_generic_path_edge_cases(cuda):
    model = c6.PolicyValueNet(board_size=5, kernels=[3], channels=[4]).to(cuda).eval()
    with torch.inference_mode():
        logits, value = model(torch.zeros(0, 3, 5, 5, device=cuda))
        assert logits.shape == (0, 25) and value.shape == (0,)
        logits, value = model(torch.zeros(3, 3, 5, 5, device=cuda))     # tests/test_model.py:11-18
        assert torch.count_nonzero(logits) == 0 and torch.count_nonzero(value) == 0
        with pytest.raises(NotImplementedError):
            model.selfplay_step(torch.zeros(1, 3, 5, 5, device=cuda), torch.zeros(1, device=cuda))
    with pytest.raises(ValueError):
        model(torch.zeros(2, 3, 6, 6, device=cuda))
