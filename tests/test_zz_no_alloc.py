"""``c6_forward_generic_static``: the generic forward through the library's built-in
workspace (for callers that cannot allocate device memory) against
``c6_forward_generic`` with a caller workspace.  Both run the same kernels, so the
outputs must be bit-identical; the second call uses a smaller batch, so it also shows
that what the first call left in the shared array does not leak into the next."""
import ctypes

import pytest
import torch

import connect6_amd as c6
from connect6_amd import _lib
from connect6_amd.model import run_forward_generic
from oracle import torch_ref as R
from tests.util import rel_l2

pytestmark = pytest.mark.gpu

KERNELS, CHANNELS, BOARD = [5, 3, 1], [16, 24, 7], 9


def _inputs(batch, seed):
    x = torch.randn(batch, 3, BOARD, BOARD, generator=torch.Generator().manual_seed(seed))
    x[:, :2] = (x[:, :2] > 0.8).float()
    return x


def test_static_workspace_forward_matches_caller_workspace_forward(cuda):
    st = R.init_state(11, "torch_default", kernels=KERNELS, channels=CHANNELS)
    dev_state = {k: v.to(cuda) for k, v in st.items()}
    # the first launch on a device loads the library's device image (which holds the array)
    run_forward_generic(_inputs(1, 0).to(cuda), dev_state, KERNELS, CHANNELS, _lib.PREC_F32,
                        static_workspace=True)
    for prec_name in ("fp32", "bf16"):
        prec = _lib.PREC_BY_NAME[prec_name]
        for batch, seed in ((48, 3), (5, 4)):          # two calls in a row, the second smaller
            x = _inputs(batch, seed).to(cuda)
            out = (torch.full((batch, BOARD * BOARD), float("nan"), device=cuda),
                   torch.full((batch,), float("nan"), device=cuda))
            torch.cuda.synchronize()
            free_before = torch.cuda.mem_get_info()[0]
            lg, vg = run_forward_generic(x, dev_state, KERNELS, CHANNELS, prec, mask_mode=_lib.MASK_INPUT,
                                         static_workspace=True, out=out)
            torch.cuda.synchronize()
            # (parameters are already fp32 on the device and the outputs are preallocated:
            # nothing in this call may have taken device memory)
            assert torch.cuda.mem_get_info()[0] == free_before
            lw, vw = run_forward_generic(x, dev_state, KERNELS, CHANNELS, prec, mask_mode=_lib.MASK_INPUT)
            assert torch.equal(lg, lw) and torch.equal(vg, vw)
            if prec_name == "fp32":
                lo, vo = R.forward(st, x.cpu())
                legal = ((x[:, 0] == 0) & (x[:, 1] == 0)).flatten(1).cpu()
                assert torch.equal(lg.cpu() == torch.finfo(torch.float32).min, ~legal)
                assert rel_l2(lg.cpu()[legal], lo[legal]) <= 1e-5 and rel_l2(vg, vo) <= 1e-5


def test_static_workspace_rejects_batches_beyond_its_size(cuda):
    lib = c6.load()
    ints = ctypes.c_int * 3
    ks, ch = ints(*KERNELS), ints(*CHANNELS)
    need = ctypes.c_size_t(0)
    # 16 MiB / (2 buffers * 24 channels * 81 squares * 4 bytes) = 1078.8 boards
    assert lib.c6_generic_workspace_bytes(1078, BOARD, 3, ch, ctypes.byref(need)) == 0
    assert need.value <= 16 << 20
    assert lib.c6_generic_workspace_bytes(1079, BOARD, 3, ch, ctypes.byref(need)) == 0
    assert need.value > 16 << 20
    rc = lib.c6_forward_generic_static(None, 0, 1079, BOARD, 3, ks, ch, None, None, None, None, None,
                                       None, 0, None, None, 0, None, 0.0, None)
    assert rc == -1 and b"built-in" in lib.c6_last_error()
    st = R.init_state(11, "torch_default", kernels=KERNELS, channels=CHANNELS)
    dev_state = {k: v.to(cuda) for k, v in st.items()}
    with pytest.raises(ValueError):
        run_forward_generic(_inputs(1079, 1).to(cuda), dev_state, KERNELS, CHANNELS, _lib.PREC_F32,
                            static_workspace=True)
    lg, _ = run_forward_generic(_inputs(1078, 1).to(cuda), dev_state, KERNELS, CHANNELS, _lib.PREC_F32,
                                static_workspace=True)
    lw, _ = run_forward_generic(_inputs(1078, 1).to(cuda), dev_state, KERNELS, CHANNELS, _lib.PREC_F32)
    assert torch.equal(lg, lw)
