"""Host-side logic of the drop-in modules and the C-ABI surface, no GPU needed
(no compute entry point is launched here)."""
import ctypes
import re
from pathlib import Path

import pytest
import torch

import connect6_amd as c6
from connect6_amd import _lib
from oracle import torch_ref as R

ROOT = Path(__file__).resolve().parent.parent


def test_library_exports_every_declared_symbol():
    header = (ROOT / "include" / "connect6_amd.h").read_text()
    declared = set(re.findall(r"\b(c6_[a-z0-9_]+)\s*\(", header))
    assert declared == set(_lib.EXPORTS)
    lib = _lib.load()
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.c6_version() == 1


def test_fused_kernels_stay_within_their_scratch_budget():
    """One wave per SIMD: every scratch access of the fused kernel is latency next to the MFMAs.
    The compiler's report from the last build bounds the spill bytes per lane of each
    arithmetic mode (headline and plain 16-bit modes tight, the others a ceiling)."""
    usage = _lib.resource_usage()
    fused = {name: u for name, u in usage.items() if "fused_forward_kernel" in name or "fused_pipe_kernel" in name}
    assert len(fused) == 5
    # bytes per lane; the pipelined kernels (bf16f6w, bf16f6, bf16, fp16) keep two layers'
    # accumulators live and still spill nothing: per-lane addresses are recomputed per board, not kept
    limit = {"PrecBF16F6W": 0, "PrecBF16F6E": 0, "PrecBF16E": 0, "PrecF16": 0, "PrecF32": 32}
    seen = set()
    for name, u in fused.items():
        for tag, cap in limit.items():
            if tag in name:
                seen.add(tag)
                assert u["ScratchSize"] <= cap, (name, u)
                assert u["VGPRs"] <= 256 and u["AGPRs"] <= 256 and u["Occupancy"] >= 1
    assert seen == set(limit)


def test_history_dtype_follows_the_reference_policy():
    # connect6/train.py:133-145
    cpu, gpu = torch.device("cpu"), torch.device("cuda", 0)
    assert c6.history_dtype(cpu, "bfloat16") is torch.float32
    assert c6.history_dtype(gpu, "bfloat16") is torch.bfloat16
    assert c6.history_dtype(gpu, "Float16") is torch.float16
    assert c6.history_dtype(gpu, "float32") is torch.float32
    with pytest.raises(ValueError):
        c6.history_dtype(gpu, "int8")


def test_packed_sizes_follow_the_layout():
    # 1 KiB fragments: first layer 35 rows x (24/E) per half, 3x3 layers 9*Cin/KSTEP x Cout/32
    def frags(e):
        kstep = 2 * e
        n = 35 * (24 // e)
        for cin, cout in zip((32, 32, 64, 64, 64, 96, 96), (32, 64, 64, 64, 96, 96, 96)):
            n += (9 * cin // kstep) * (cout // 32)
        return n + 24
    tail = (544 + 96 + 96 + 4 + 8) * 4
    # pipelined modes: plus the first layer's two-plane copy (23 rows x 3 fragments, 8 over-read)
    # and the third plane's table as the lanes hold it (4 waves x 3 pixel tiles x 4 quads)
    fast1 = 23 * 3 + 8 + 4 * 3 * 4
    assert _lib.packed_bytes(_lib.PREC_BF16) == (frags(8) + fast1) * 1024 + tail
    assert _lib.packed_bytes(_lib.PREC_F16) == (frags(8) + fast1) * 1024 + tail
    assert _lib.packed_bytes(_lib.PREC_F32) == frags(4) * 1024 + tail
    # bf16 + fp6: plus the e2m3 copy of the 3x3 layers (64-wide chunks, two fragments per chunk and
    # cout tile: 16 bytes per lane, then 8 bytes per lane packed densely) and its over-read padding
    lo = 0
    for cin, cout in zip((32, 32, 64, 64, 64, 96, 96), (32, 64, 64, 64, 96, 96, 96)):
        lo += ((9 * cin // 32 + 1) // 2) * (cout // 32) * 2
    assert _lib.packed_bytes(_lib.PREC_BF16F6) == (frags(8) + lo + 18 + fast1) * 1024 + tail
    # ... and with the weights' low part: every fragment of the main pass twice (the first layer's
    # two-plane copy too), the over-read padding and the rest as before
    main = frags(8) - 24
    fast1w = 2 * 23 * 3 + 8 + 4 * 3 * 4
    assert _lib.packed_bytes(_lib.PREC_BF16F6W) == (2 * main + 24 + lo + 18 + fast1w) * 1024 + tail
    # cascade: the bf16 set, then (256-byte aligned) the second pass's set
    first = (_lib.packed_bytes(_lib.PREC_BF16) + 255) // 256 * 256
    assert _lib.packed_bytes(_lib.PREC_BF16C) == first + _lib.packed_bytes(_lib.PREC_BF16F6W)
    # ... or, for parameters that are exact in bf16, the bf16 + fp6 set
    assert _lib.packed_bytes(_lib.PREC_BF16C6) == first + _lib.packed_bytes(_lib.PREC_BF16F6)
    # workspace: 4 ints, 1024 per-run counts, per-run lists with room for boards + 1024 entries
    assert _lib.cascade_workspace_bytes(0) == 16 + 8192 and _lib.cascade_workspace_bytes(5) == 16 + 8192 + 32
    with pytest.raises(ValueError):
        _lib.packed_bytes(9)


def test_entry_points_reject_bad_arguments_before_touching_the_device():
    lib = _lib.load()
    assert lib.c6_forward(None, 0, 1, 4, None, 0, 1, None, None, 0, None, 0.0, None, 1.0, None, None, None) == -1
    assert b"null" in lib.c6_last_error()
    assert lib.c6_forward(None, 7, 1, 4, None, 0, 1, None, None, 0, None, 0.0, None, 1.0, None, None, None) == -1
    assert lib.c6_forward(None, 0, 1, 4, None, 0, 5, None, None, 0, None, 0.0, None, 1.0, None, None, None) == -1
    assert lib.c6_forward(None, 0, 0, 4, None, 0, 1, None, None, 0, None, 0.0, None, 1.0, None, None, None) == -1
    # an empty batch is a no-op, not an error
    assert lib.c6_forward(None, 0, 1, 0, None, 0, 1, None, None, 0, None, 0.0, None, 1.0, None, None, None) == 0
    # the cascade's mode only through the entry points that take its workspace, and those only it
    assert lib.c6_forward(None, 0, 1, 4, None, 0, _lib.PREC_BF16C, None, None, 0, None, 0.0, None, 1.0, None, None,
                          None) == -1
    assert b"c6_forward_cascade" in lib.c6_last_error()
    C, C6 = _lib.PREC_BF16C, _lib.PREC_BF16C6
    assert lib.c6_forward_cascade(None, 0, 1, 4, None, 0, C, None, 0, None, 0, None, 0.0, None, 1.0, None, None, 0.03,
                                  None, 0, None) == -1
    assert lib.c6_forward_cascade(None, 0, 1, 0, None, 0, C6, None, 0, None, 0, None, 0.0, None, 1.0, None, None, 0.03,
                                  None, 0, None) == 0
    assert lib.c6_forward_cascade(None, 0, 1, 4, None, 0, C, None, 9, None, 0, None, 0.0, None, 1.0, None, None, 0.03,
                                  None, 0, None) == -1                  # unknown element type of the logits
    assert lib.c6_forward_cascade(None, 0, 1, 4, None, 0, _lib.PREC_BF16, None, 0, None, 0, None, 0.0, None, 1.0, None,
                                  None, 0.03, None, 0, None) == -1      # not a cascade mode
    assert b"c6_forward" in lib.c6_last_error()
    assert lib.c6_forward_boards_cascade(None, None, None, 4, None, 0, 4, None, C, None, 0, None, 1, 0.0, None, 1.0,
                                         None, None, 0.03, None, 0, None) == -1
    assert lib.c6_pack_weights_grouped(None, None, None, None, None, None, 0, 1, None, 0, None) == -1
    size = ctypes.c_size_t(0)
    assert lib.c6_cascade_workspace_bytes(-1, ctypes.byref(size)) == -1
    assert lib.c6_cascade_workspace_bytes(4096, ctypes.byref(size)) == 0 and size.value == 16 + 8192 + 4 * 4096
    assert lib.c6_mask_logits(None, None, 0, 3, 0, None, None) == -1
    assert lib.c6_mask_logits(None, None, 0, 0, 0, None, None) == 0
    assert lib.c6_softmax_sample(None, None, None, 1.0, 2, None, None, None) == -1
    assert lib.c6_d4_expand(None, 0, 2, None, None) == -1
    assert lib.c6_d4_reduce(None, None, 2, None, None, None) == -1
    assert lib.c6_pack_weights(None, None, None, None, None, None, 1, None, None) == -1
    assert lib.c6_forward_boards(None, None, None, 4, None, 0, 4, None, 1, None, None, 1, 0.0, None, 1.0,
                                 None, None, None) == -1
    assert lib.c6_forward_boards(None, None, None, 4, None, 9, 4, None, 1, None, None, 1, 0.0, None, 1.0,
                                 None, None, None) == -1
    assert lib.c6_forward_boards(None, None, None, 4, None, 0, 0, None, 1, None, None, 1, 0.0, None, 1.0,
                                 None, None, None) == 0
    none14 = [None] * 5
    assert lib.c6_env_step(*none14, None, 0, 4, 19, 6, None, None, None, None, None, None) == -1  # null state
    assert lib.c6_env_step(*none14, None, 0, 4, 0, 6, None, None, None, None, None, None) == -1   # board size
    assert lib.c6_env_step(*none14, None, 0, 4, 19, 0, None, None, None, None, None, None) == -1  # win length
    assert lib.c6_env_step(*none14, None, 8, 4, 19, 6, None, None, None, None, None, None) == -1  # view
    assert lib.c6_env_step(*none14, None, 0, 0, 19, 6, None, None, None, None, None, None) == 0   # no games
    assert lib.c6_canonical_input(None, None, None, 3, 19, None, None) == -1
    assert lib.c6_canonical_input(None, None, None, 0, 19, None, None) == 0
    n = ctypes.c_size_t(0)
    ch = (ctypes.c_int * 3)(8, 8, 16)
    ks = (ctypes.c_int * 3)(3, 3, 3)
    assert lib.c6_generic_workspace_bytes(4, 5, 3, ch, ctypes.byref(n)) == 0
    assert n.value == 2 * 4 * 16 * 25 * 4
    assert lib.c6_generic_workspace_bytes(4, 0, 3, ch, ctypes.byref(n)) == -1
    bad = (ctypes.c_int * 3)(3, 4, 3)      # even kernel, as connect6/model.py:44-45 rejects
    assert lib.c6_forward_generic(None, 0, 2, 5, 3, bad, ch, None, None, None, None, None, None, 0,
                                  None, 0, None, None, 0, None, 0.0, None) == -1
    assert lib.c6_forward_generic(None, 0, 2, 5, 3, ks, ch, None, None, None, None, None, None, 0,
                                  None, 0, None, None, 0, None, 0.0, None) == -1
    assert lib.c6_forward_generic(None, 0, 0, 5, 3, ks, ch, None, None, None, None, None, None, 0,
                                  None, 0, None, None, 0, None, 0.0, None) == 0


def test_model_attributes_match_reference_contract():
    # tests/test_model.py:11-37 of the reference, minus the CPU forward
    model = c6.PolicyValueNet(board_size=19)
    assert model.receptive_field == 37
    assert model.board_size == 19 and model.action_size == 361 and model.input_channels == 3
    cfg = {
        "architecture_version": 4,
        "kernels": [23, 3, 3, 3, 3, 3, 3, 3],
        "channels": [32, 32, 64, 64, 64, 96, 96, 96],
        "compile": False,
        "compile_mode": "default",
    }
    model = c6.build_model(cfg, 19)
    assert [m.kernel_size[0] for m in model.convs] == [23, 3, 3, 3, 3, 3, 3, 3]
    assert [m.out_channels for m in model.convs] == [32, 32, 64, 64, 64, 96, 96, 96]
    assert model.convs[0].in_channels == 3
    assert model.policy_output.kernel_size == (1, 1)
    assert model.policy_output.in_channels == 96
    assert model.policy_output.out_channels == 1
    assert model.value_output.kernel_size == (1, 1)
    assert model.receptive_field == 37
    assert model.kernels == (23, 3, 3, 3, 3, 3, 3, 3)
    assert isinstance(model.activation, torch.nn.SiLU)


def test_state_dict_is_interchangeable_with_the_oracle():
    model = c6.PolicyValueNet()
    st = R.init_state(1, "reference")
    assert set(model.state_dict().keys()) == set(st.keys())
    for k, v in model.state_dict().items():
        assert v.shape == st[k].shape, k
    model.load_state_dict(st)
    # reference init: zero biases, small heads (connect6/model.py:83-94)
    fresh = c6.PolicyValueNet()
    assert all(torch.count_nonzero(c.bias) == 0 for c in fresh.convs)
    assert torch.count_nonzero(fresh.policy_output.bias) == 0
    assert fresh.policy_output.weight.std() < 0.02 and fresh.value_output.weight.std() < 0.02
    assert abs(fresh.convs[7].weight.std().item() / (2.0 / 864) ** 0.5 - 1) < 0.05


def test_constructor_validation():
    for bad in (
        dict(kernels=[3, 3], channels=[8]),
        dict(kernels=[], channels=[]),
        dict(kernels=[2], channels=[8]),
        dict(kernels=[-1], channels=[8]),
        dict(kernels=[3], channels=[0]),
    ):
        with pytest.raises(ValueError):
            c6.PolicyValueNet(board_size=5, **bad)
    small = c6.PolicyValueNet(board_size=5, kernels=[3, 3, 3], channels=[8, 8, 16])
    assert small.receptive_field == 7 and not small.is_default_architecture


def test_forward_errors():
    model = c6.PolicyValueNet()
    with pytest.raises(ValueError):          # shape errors first, as connect6/model.py:97-102
        model(torch.zeros(2, 4, 19, 19))
    with pytest.raises(ValueError):
        model(torch.zeros(3, 19, 19))
    with pytest.raises(RuntimeError, match="no CPU path"):
        with torch.no_grad():
            model(torch.zeros(2, 3, 19, 19))
    model.precision = "int4"
    with pytest.raises(ValueError):
        model.resolve_precision()


def test_precision_resolution_follows_torch_rules():
    model = c6.PolicyValueNet()
    assert model.resolve_precision() == _lib.PREC_F32
    model.precision = "bf16f6"
    assert model.resolve_precision() == _lib.PREC_BF16F6
    model.precision = "bf16f6w"
    assert model.resolve_precision() == _lib.PREC_BF16F6W
    model.precision = None
    # bf16 parameters (or bf16 autocast) select the cascade (plain bf16, corrected where the
    # decision is close); the two modes it is made of are by name only
    # (under bf16 autocast, which needs the GPU, fp32 parameters select "bf16c": the GPU tests hold
    # that; parameters held in bf16 have no low part for the second pass to carry)
    assert model.to(torch.bfloat16).resolve_precision() == _lib.PREC_BF16C6
    assert model.to(torch.float16).resolve_precision() == _lib.PREC_F16
    model.precision = "bf16"
    assert model.resolve_precision() == _lib.PREC_BF16


def test_mask_logits_argument_checks():
    with pytest.raises(RuntimeError, match="no CPU path"):
        c6.mask_logits(torch.zeros(2, 361), torch.ones(2, 361, dtype=torch.bool))


def _checkpoints(n, **kw):
    cfg = {"architecture_version": 4, "kernels": list(R.DEFAULT_KERNELS),
           "channels": list(R.DEFAULT_CHANNELS), "compile": False, "compile_mode": "default"}
    return [
        c6.HistoricalCheckpoint(path=Path(f"model_update_{i + 1:08d}.pt"), update=i + 1,
                                model_state=R.init_state(50 + i, "reference"),
                                model_config=dict(cfg, **kw), game_config={"board_size": 19, "win_length": 6})
        for i in range(n)
    ]


def test_history_ensemble_construction_and_validation():
    with pytest.raises(ValueError):
        c6.HistoricalPolicyEnsemble([], torch.device("cpu"))
    cps = _checkpoints(2)
    ens = c6.HistoricalPolicyEnsemble(cps, torch.device("cpu"))
    assert ens.num_models == 2 and ens.updates == [1, 2] and ens.board_size == 19
    assert ens.kernels == R.DEFAULT_KERNELS and ens.channels == R.DEFAULT_CHANNELS
    assert ens.action_size == 361 and ens.input_channels == 3 and ens.dtype == torch.float32
    assert ens.conv_weights[0].shape == (2, 32, 3, 23, 23)
    assert ens.conv_biases[7].shape == (2, 96)
    assert ens.policy_weight.shape == (2, 1, 96, 1, 1) and ens.policy_bias.shape == (2, 1)
    assert ens._prec == _lib.PREC_F32
    ens16 = c6.HistoricalPolicyEnsemble(cps, torch.device("cpu"), dtype=torch.bfloat16)
    assert ens16._prec == _lib.PREC_BF16C6 and ens16.conv_weights[3].dtype == torch.bfloat16
    assert c6.HistoricalPolicyEnsemble(cps, torch.device("cpu"), dtype=torch.bfloat16, precision="bf16")._prec == _lib.PREC_BF16
    # compile keys are ignored when comparing architectures (history.py:69-73)
    cps[1].model_config["compile"] = True
    c6.HistoricalPolicyEnsemble(cps, torch.device("cpu"))
    bad = _checkpoints(2)
    bad[1].game_config = {"board_size": 15}
    with pytest.raises(ValueError):
        c6.HistoricalPolicyEnsemble(bad, torch.device("cpu"))
    bad = _checkpoints(2)
    bad[1].model_config["channels"] = [32] * 8
    with pytest.raises(ValueError):
        c6.HistoricalPolicyEnsemble(bad, torch.device("cpu"))
    bad = _checkpoints(2)
    del bad[1].model_state["convs.3.weight"]
    with pytest.raises(KeyError):
        c6.HistoricalPolicyEnsemble(bad, torch.device("cpu"))
    with pytest.raises(ValueError):   # shape errors as history.py:277-286
        ens.forward_grouped(torch.zeros(2, 3, 19, 19))
    with pytest.raises(ValueError):
        ens.forward_grouped(torch.zeros(3, 4, 3, 19, 19))
    with pytest.raises(RuntimeError, match="no CPU path"):
        ens.forward_grouped(torch.zeros(2, 4, 3, 19, 19))


def test_symmetry_helpers_on_host():
    # tests/test_training_features.py:154-187 and tests/test_model.py:40-53 of the reference
    want = [(0, False), (1, False), (2, False), (3, False), (0, True), (1, True), (2, True), (3, True)]
    assert [c6.symmetry_for_phase(i) for i in range(8)] == want
    assert c6.symmetry_for_phase(8) == want[0]
    board = torch.arange(9, dtype=torch.int8).reshape(1, 3, 3)
    actions = torch.arange(9, dtype=torch.long)
    for phase in range(8):
        k, flip = c6.symmetry_for_phase(phase)
        tb = c6.transform_boards(board, k, flip)
        ta = c6.transform_actions(actions, 3, k, flip)
        assert torch.equal(tb.reshape(-1)[ta], board.reshape(-1)[actions])
        assert torch.equal(c6.inverse_transform_actions(ta, board_size=3, k=k, flip=flip), actions)
        assert torch.equal(tb, R.transform_boards(board, k, flip))
    n = 7
    b = torch.zeros(1, n, n, dtype=torch.int8)
    b[0, 1, 2] = 1
    a = torch.tensor([1 * n + 2])
    for k in range(4):
        for flip in (False, True):
            ob, oa = c6.transform_boards(b, k, flip), int(c6.transform_actions(a, n, k, flip))
            assert int(ob[0, oa // n, oa % n]) == 1
            assert torch.equal(c6.inverse_transform_actions(torch.tensor([oa]), n, k, flip), a)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    # there is no fallback path: without the built shared object every entry raises
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "_SO", tmp_path / "libconnect6_amd.so")
    with pytest.raises(c6.C6Error, match="no fallback"):
        _lib.load()
    with pytest.raises(c6.C6Error):
        _lib.packed_bytes(_lib.PREC_BF16)


def test_vector_env_refuses_cpu_device():
    import connect6_amd as c6

    with pytest.raises(RuntimeError, match="HIP device only"):
        c6.VectorConnect6(4, 9, 6, device="cpu")
    with pytest.raises(RuntimeError, match="HIP device"):
        c6.canonical_network_input(torch.zeros(1, 9, 9, dtype=torch.int8), torch.ones(1, dtype=torch.int8),
                                   torch.ones(1, dtype=torch.int8))


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys

    proc = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert proc.returncode != 0
    assert "one GPU" in proc.stderr and proc.stdout.strip() == ""


def test_probe_library_loads_and_exports_its_symbol():
    # the measurement aid bench.py uses (sustained bf16 MFMA rate); no compute without a GPU
    import ctypes

    assert _lib._PROBE_SO.exists(), "run connect6_amd.build()"
    probe = ctypes.CDLL(str(_lib._PROBE_SO))
    assert hasattr(probe, "c6_probe_mfma_rate")
