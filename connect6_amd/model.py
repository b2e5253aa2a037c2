"""Drop-in ``PolicyValueNet`` whose forward runs hand-written HIP kernels.

Mirrors the operator interface of the reference's connect6/model.py
(``PolicyValueNet``, ``build_model``, ``mask_logits``): same constructor,
validation, attributes, ``state_dict`` keys and error behaviour.  The forward
pass itself is one fused gfx950 kernel launched through the C ABI in
``include/connect6_amd.h``; PyTorch only owns the memory and the stream.
"""
from __future__ import annotations

import ctypes
from typing import Any

import torch
from torch import nn

from . import _lib

_FILL_LOWEST = float(torch.finfo(torch.float32).min)


def _require_device_tensor(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(
            f"{what} is on {t.device}: connect6_amd computes only on an MI355X (HIP) device; "
            "there is no CPU path"
        )


def pack_state(state: dict[str, torch.Tensor], prec: int, out: torch.Tensor, groups: int | None = None) -> None:
    """Repack one checkpoint (reference ``state_dict`` keys, device tensors)
    into ``out`` (uint8 device buffer of ``_lib.packed_bytes(prec)`` bytes).

    With ``groups`` = G every tensor of ``state`` is G checkpoints' tensors stacked along a
    new first dimension (what ``HistoricalPolicyEnsemble._stack`` builds) and ``out`` is
    ``[G, packed_bytes]``: all sets are packed by one call."""
    lib = _lib.load()
    keep = []  # keep fp32 staging copies alive until the launch is enqueued
    lead = () if groups is None else (int(groups),)

    def dev32(key: str, required: bool = True):
        if key not in state or state[key] is None:
            if required:
                raise KeyError(f"missing parameter {key}")
            return None
        t = state[key].detach().to(device=out.device, dtype=torch.float32).contiguous()
        keep.append(t)
        return t

    ws = [dev32(f"convs.{i}.weight") for i in range(8)]
    bs = [dev32(f"convs.{i}.bias", required=False) for i in range(8)]
    expect_in = 3
    for i, (k, c) in enumerate(zip(PolicyValueNet.DEFAULT_KERNELS, PolicyValueNet.DEFAULT_CHANNELS)):
        if tuple(ws[i].shape) != lead + (c, expect_in, k, k):
            raise ValueError(
                f"convs.{i}.weight has shape {tuple(ws[i].shape)}; the fused kernels are built for "
                f"the default architecture and need {lead + (c, expect_in, k, k)}"
            )
        expect_in = c
    pw, pb = dev32("policy_output.weight"), dev32("policy_output.bias", required=False)
    vw, vb = dev32("value_output.weight", required=False), dev32("value_output.bias", required=False)
    vp = ctypes.c_void_p
    wptrs = (vp * 8)(*[t.data_ptr() for t in ws])
    bptrs = (vp * 8)(*[(t.data_ptr() if t is not None else None) for t in bs])

    def ptr(t):
        return t.data_ptr() if t is not None else None

    with torch.cuda.device(out.device):
        if groups is None:
            rc = lib.c6_pack_weights(wptrs, bptrs, ptr(pw), ptr(pb), ptr(vw), ptr(vb), prec,
                                     out.data_ptr(), _lib.stream_ptr(out.device))
        else:
            if out.ndim != 2 or out.shape[0] != groups or not out.is_contiguous():
                raise ValueError(f"out must be a contiguous [{groups}, packed_bytes] buffer")
            rc = lib.c6_pack_weights_grouped(wptrs, bptrs, ptr(pw), ptr(pb), ptr(vw), ptr(vb), int(groups), prec,
                                             out.data_ptr(), int(out.shape[1]), _lib.stream_ptr(out.device))
    _lib.check(rc, "c6_pack_weights")
    # the staging copies are freed by the caching allocator in stream order, after the kernel


def run_forward(
    x: torch.Tensor,
    packed: torch.Tensor,
    prec: int,
    groups: int,
    boards_per_group: int,
    *,
    want_logits: bool = True,
    want_value: bool = True,
    mask_mode: int = _lib.MASK_NONE,
    legal: torch.Tensor | None = None,
    fill: float = _FILL_LOWEST,
    u: torch.Tensor | None = None,
    temperature: float = 1.0,
    want_logprob: bool = False,
    threshold: float | None = None,
    stats: dict | None = None,
    logits_dtype: torch.dtype = torch.float32,
):
    """Launch ``c6_forward`` (``c6_forward_cascade`` for the cascade mode, with ``threshold``
    and a workspace tensor of its own); returns (logits, value, actions, logprob), each None
    when not requested.  ``stats``, if given, receives ``second_pass`` for the cascade mode: a
    one-element int32 device tensor, the number of boards that were evaluated twice.
    ``logits_dtype`` other than float32 (the cascade mode's entry point only) makes the kernel
    write the logits rounded to that type."""
    lib = _lib.load()
    dev = x.device
    total = groups * boards_per_group
    x = x.contiguous()
    if logits_dtype != torch.float32 and prec not in _lib.CASCADES:
        raise ValueError("only the cascade mode's entry point writes logits in another type than float32")
    logits = torch.empty((total, 361), dtype=logits_dtype, device=dev) if want_logits else None
    value = torch.empty((total,), dtype=torch.float32, device=dev) if want_value else None
    actions = logprob = None
    if u is not None:
        u = u.to(device=dev, dtype=torch.float32).contiguous()
        if u.shape != (total,):
            raise ValueError(f"u must have shape ({total},), got {tuple(u.shape)}")
        actions = torch.empty((total,), dtype=torch.int64, device=dev)
        if want_logprob:
            logprob = torch.empty((total,), dtype=torch.float32, device=dev)
    if legal is not None:
        if legal.shape != (total, 361):
            raise ValueError(f"legal mask must have shape ({total}, 361), got {tuple(legal.shape)}")
        if legal.dtype == torch.bool:
            legal = legal.contiguous().view(torch.uint8)
        elif legal.dtype != torch.uint8:
            raise ValueError("legal mask must be a bool or uint8 tensor")
        legal = legal.to(dev).contiguous()

    def ptr(t):
        return t.data_ptr() if t is not None else None

    stride = packed.numel() // groups if groups > 1 else packed.numel()
    with torch.cuda.device(dev):
        if prec in _lib.CASCADES:
            ws = torch.empty(_lib.cascade_workspace_bytes(total) // 4, dtype=torch.int32, device=dev)
            rc = lib.c6_forward_cascade(
                x.data_ptr(), _lib.torch_dtype_code(x.dtype), groups, boards_per_group, packed.data_ptr(),
                stride, prec, ptr(logits), _lib.torch_dtype_code(logits_dtype), ptr(value), mask_mode, ptr(legal), fill,
                ptr(u), float(temperature), ptr(actions), ptr(logprob),
                float(_lib.CASCADE_THRESHOLD if threshold is None else threshold),
                ws.data_ptr(), ws.numel() * 4, _lib.stream_ptr(dev))
            if stats is not None:
                stats["second_pass"] = ws[:1]
            _lib.check(rc, "c6_forward_cascade")
            return logits, value, actions, logprob
        rc = lib.c6_forward(x.data_ptr(), _lib.torch_dtype_code(x.dtype), groups, boards_per_group,
                            packed.data_ptr(), stride, prec, ptr(logits), ptr(value), mask_mode,
                            ptr(legal), fill, ptr(u), float(temperature), ptr(actions),
                            ptr(logprob), _lib.stream_ptr(dev))
    _lib.check(rc, "c6_forward")
    return logits, value, actions, logprob


def run_forward_generic(
    x: torch.Tensor,
    state: dict[str, torch.Tensor],
    kernels,
    channels,
    prec: int,
    *,
    want_value: bool = True,
    mask_mode: int = _lib.MASK_NONE,
    legal: torch.Tensor | None = None,
    fill: float = _FILL_LOWEST,
    static_workspace: bool = False,
    out: tuple[torch.Tensor, torch.Tensor | None] | None = None,
    groups: int = 1,
):
    """Launch ``c6_forward_generic`` for one weight set of any architecture:
    x ``[B,3,n,n]`` -> (logits ``[B,n*n]``, value ``[B]`` or None).

    ``groups = G > 1``: ``state`` holds G weight sets stacked along a leading dimension (as
    ``HistoricalPolicyEnsemble._stack`` lays them out, connect6/history.py:224-240), x is
    ``[G*T,3,n,n]`` and board b uses set ``b // T`` -- ``c6_forward_generic_grouped``, one launch
    per layer for all sets.

    ``static_workspace`` routes the layer-boundary activations through the
    library's built-in 16 MiB array (``c6_forward_generic_static``) instead of
    a workspace tensor; with ``out=(logits, value)`` preallocated the call then
    allocates no device memory for the forward itself."""
    lib = _lib.load()
    dev = x.device
    x = x.contiguous()
    b, n = int(x.shape[0]), int(x.shape[-1])
    layers = len(kernels)
    keep = []
    if groups < 1 or b % groups or (groups > 1 and static_workspace):
        raise ValueError(f"{b} boards do not split into {groups} groups (or groups with the static workspace)")

    def dev32(key, required=True):
        if key not in state:
            if required:
                raise KeyError(f"missing parameter {key}")
            return None
        t = state[key].detach().to(device=dev, dtype=torch.float32).contiguous()
        keep.append(t)
        return t

    ws = [dev32(f"convs.{i}.weight") for i in range(layers)]
    bs = [dev32(f"convs.{i}.bias", required=False) for i in range(layers)]
    pw, pb = dev32("policy_output.weight"), dev32("policy_output.bias", required=False)
    vw = dev32("value_output.weight", required=False) if want_value else None
    vb = dev32("value_output.bias", required=False) if want_value else None
    ints = ctypes.c_int * layers
    ck, cc = ints(*[int(k) for k in kernels]), ints(*[int(c) for c in channels])
    vp = ctypes.c_void_p
    wptrs = (vp * layers)(*[t.data_ptr() for t in ws])
    bptrs = (vp * layers)(*[(t.data_ptr() if t is not None else None) for t in bs])
    workspace = None
    if not static_workspace:
        nbytes = ctypes.c_size_t(0)
        _lib.check(lib.c6_generic_workspace_bytes(b, n, layers, cc, ctypes.byref(nbytes)),
                   "c6_generic_workspace_bytes")
        workspace = torch.empty(max(int(nbytes.value), 16), dtype=torch.uint8, device=dev)
    if out is not None:
        logits, value = out
        if logits.shape != (b, n * n) or logits.dtype != torch.float32 or not logits.is_contiguous():
            raise ValueError(f"out[0] must be a contiguous float32 tensor of shape ({b}, {n * n})")
        if want_value and (value is None or value.shape != (b,) or value.dtype != torch.float32):
            raise ValueError(f"out[1] must be a float32 tensor of shape ({b},)")
    else:
        logits = torch.empty((b, n * n), dtype=torch.float32, device=dev)
        value = torch.empty((b,), dtype=torch.float32, device=dev) if want_value else None
    if legal is not None:
        if legal.shape != (b, n * n):
            raise ValueError(f"legal mask must have shape ({b}, {n * n}), got {tuple(legal.shape)}")
        legal = legal.to(dev).contiguous()
        legal = legal.view(torch.uint8) if legal.dtype == torch.bool else legal

    def ptr(t):
        return t.data_ptr() if t is not None else None

    with torch.cuda.device(dev):
        if static_workspace:
            rc = lib.c6_forward_generic_static(x.data_ptr(), _lib.torch_dtype_code(x.dtype), b, n,
                                               layers, ck, cc, wptrs, bptrs, ptr(pw), ptr(pb),
                                               ptr(vw), ptr(vb), prec, ptr(logits), ptr(value),
                                               mask_mode, ptr(legal), fill, _lib.stream_ptr(dev))
        elif groups > 1:
            rc = lib.c6_forward_generic_grouped(x.data_ptr(), _lib.torch_dtype_code(x.dtype), groups,
                                                b // groups, n, layers, ck, cc, wptrs, bptrs, ptr(pw),
                                                ptr(pb), ptr(vw), ptr(vb), prec, workspace.data_ptr(),
                                                workspace.numel(), ptr(logits), ptr(value), mask_mode,
                                                ptr(legal), fill, _lib.stream_ptr(dev))
        else:
            rc = lib.c6_forward_generic(x.data_ptr(), _lib.torch_dtype_code(x.dtype), b, n, layers,
                                        ck, cc, wptrs, bptrs, ptr(pw), ptr(pb), ptr(vw), ptr(vb),
                                        prec, workspace.data_ptr(), workspace.numel(), ptr(logits),
                                        ptr(value), mask_mode, ptr(legal), fill,
                                        _lib.stream_ptr(dev))
    _lib.check(rc, "c6_forward_generic_static" if static_workspace else "c6_forward_generic")
    return logits, value


class PolicyValueNet(nn.Module):
    """Fully convolutional policy + value network for Connect6
    (reference: connect6/model.py:9-111).

    Input ``[B, 3, H, W]``: 0 = own stones, 1 = opponent stones, 2 = whether
    this decision is the last stone of the turn.  Returns ``(logits[B, H*W],
    value[B])``, both fp32.

    ``precision`` selects the arithmetic of the HIP path: ``None`` follows
    PyTorch's own rules (bf16/fp16 under ``torch.autocast`` or when the
    parameters are held in that dtype, else fp32), where bf16 means the
    cascade ``"bf16c"``: every board with plain bf16 layer boundaries, then
    the boards whose decision is closer than that pass's rounding noise (the
    best free square leads the second best by less than ``cascade_threshold``
    standard deviations of the board's logits, default ``CASCADE_THRESHOLD``
    = 0.02, or two others lie within twice that) once more with the low parts
    of the activations and of the weights carried (``"bf16f6w"``: within 3e-4
    of fp32).  Over random networks with the reference's initialisation its
    argmax agrees with fp32's on 99.9 % of the boards (worst of 32 networks
    99.7 %) while about 6 % of the boards are evaluated twice (a quarter, or
    all, when a network's logits are nearly flat; a module whose parameters
    are held in bf16 runs ``"bf16c6"``, the same cascade without the weights'
    low part, of which there is none).  The modes it is made of
    have to be asked for by name: ``"bf16"`` (every activation and weight
    rounded to bf16 and nothing else, 98.8-98.9 % agreement), ``"bf16f6w"``
    (on every board: twice the matrix work), and ``"bf16f6"`` (bf16 MFMA plus
    a correction pass on the activations' low-order part alone, held in
    block-scaled fp6, on every board); also ``"fp32"`` and ``"fp16"``.
    """

    DEFAULT_KERNELS = (23, 3, 3, 3, 3, 3, 3, 3)
    DEFAULT_CHANNELS = (32, 32, 64, 64, 64, 96, 96, 96)
    INPUT_CHANNELS = 3

    def __init__(
        self,
        board_size: int = 19,
        kernels: list[int] | tuple[int, ...] | None = None,
        channels: list[int] | tuple[int, ...] | None = None,
    ) -> None:
        super().__init__()
        self.board_size = int(board_size)
        self.action_size = self.board_size * self.board_size
        self.input_channels = self.INPUT_CHANNELS

        kernels = tuple(self.DEFAULT_KERNELS if kernels is None else kernels)
        channels = tuple(self.DEFAULT_CHANNELS if channels is None else channels)
        # same checks, same order, same exception type as connect6/model.py:40-47
        if len(kernels) != len(channels):
            raise ValueError("kernels and channels must have the same number of elements")
        if not kernels:
            raise ValueError("the CNN needs at least one layer")
        if any(k <= 0 or k % 2 == 0 for k in kernels):
            raise ValueError("every kernel must be a positive odd number")
        if any(c <= 0 for c in channels):
            raise ValueError("channel counts must be positive")
        self.kernels = kernels
        self.channels = channels

        convs = []
        cin = self.input_channels
        for k, cout in zip(kernels, channels):
            convs.append(nn.Conv2d(cin, cout, kernel_size=k, stride=1, padding=k // 2, bias=True))
            cin = cout
        self.convs = nn.ModuleList(convs)
        self.activation = nn.SiLU(inplace=True)
        self.policy_output = nn.Conv2d(cin, 1, kernel_size=1, bias=True)
        self.value_output = nn.Conv2d(cin, 1, kernel_size=1, bias=True)
        self.value_tanh = nn.Tanh()
        self._init_weights()

        self.precision: str | None = None
        self.cascade_threshold: float | None = None   # None: _lib.CASCADE_THRESHOLD
        self.cascade_stats: dict = {}                 # "second_pass": boards evaluated twice (last call)
        self._packed: dict[int, tuple] = {}
        self._epoch = 0
        self.register_load_state_dict_post_hook(lambda module, _keys: module.refresh_weights())

    @property
    def receptive_field(self) -> int:
        return 1 + sum(k - 1 for k in self.kernels)

    def _init_weights(self) -> None:
        """connect6/model.py:83-94: Kaiming-normal (ReLU gain) convs with zero
        bias; both heads N(0, 0.01) with zero bias."""
        for conv in self.convs:
            nn.init.kaiming_normal_(conv.weight, nonlinearity="relu")
            if conv.bias is not None:
                nn.init.zeros_(conv.bias)
        for head in (self.policy_output, self.value_output):
            nn.init.normal_(head.weight, mean=0.0, std=0.01)
            nn.init.zeros_(head.bias)

    # -- precision / weights ------------------------------------------------
    @property
    def is_default_architecture(self) -> bool:
        return (
            self.board_size == 19
            and self.kernels == self.DEFAULT_KERNELS
            and self.channels == self.DEFAULT_CHANNELS
        )

    def resolve_precision(self) -> int:
        if self.precision is not None:
            try:
                return _lib.PREC_BY_NAME[self.precision]
            except KeyError:
                raise ValueError(
                    f"precision must be one of {sorted(_lib.PREC_BY_NAME)} or None, got {self.precision!r}"
                ) from None
        held = self.convs[0].weight.dtype
        dtype = held
        if torch.is_autocast_enabled("cuda"):  # reference: train.py:126-130 wraps calls in autocast
            dtype = torch.get_autocast_dtype("cuda")
        if dtype == torch.bfloat16:
            # the cascade: plain "bf16" alone misses the 99 % argmax agreement with fp32.  Parameters
            # that are held in bf16 have no low part for the second pass to carry.
            return _lib.PREC_BF16C6 if held == torch.bfloat16 else _lib.PREC_BF16C
        if dtype == torch.float16:
            return _lib.PREC_F16
        return _lib.PREC_F32

    def refresh_weights(self) -> None:
        """Force a repack on the next forward.  ``load_state_dict``, ``.to()`` and in-place
        updates of the parameters themselves (``p.add_()``, an optimizer step) are noticed
        through the tensors' version counters; edits through ``p.data`` (``p.data.copy_()``)
        and edits of parameters created under ``torch.inference_mode()`` bump no counter:
        call this after them."""
        self._epoch += 1

    def packed_weights(self, prec: int) -> torch.Tensor:
        """Kernel-layout copy of the parameters; rebuilt whenever a parameter
        was modified in place, replaced or moved."""
        params = list(self.parameters())
        # inference tensors carry no version counter; load_state_dict / refresh_weights bump the epoch
        key = (self._epoch,) + tuple(
            (p.data_ptr(), -1 if p.is_inference() else p._version, p.dtype) for p in params
        )
        dev = params[0].device
        stream = torch.cuda.current_stream(dev)
        hit = self._packed.get(prec)
        if hit is not None and hit[0] == key:
            _, buf, packed_on, done = hit
            if packed_on != stream.cuda_stream:
                stream.wait_event(done)  # the pack kernel ran on another stream
                # ... whose allocator owns the buffer: a repack drops it, and without this note the
                # memory could be handed out again while a forward here still reads it
                buf.record_stream(stream)
            return buf
        buf = torch.empty(_lib.packed_bytes(prec), dtype=torch.uint8, device=dev)
        pack_state({k: v for k, v in self.state_dict().items()}, prec, buf)
        done = torch.cuda.Event()
        done.record(stream)
        self._packed[prec] = (key, buf, stream.cuda_stream, done)
        return buf

    # -- forward --------------------------------------------------------------
    def _check_input(self, x: torch.Tensor) -> None:
        expected = (self.input_channels, self.board_size, self.board_size)
        if x.ndim != 4 or tuple(x.shape[1:]) != expected:
            raise ValueError(
                f"model input must have shape [B, {expected[0]}, {expected[1]}, {expected[2]}], "
                f"got {tuple(x.shape)}."
            )
        _require_device_tensor(x, "model input")
        _require_device_tensor(self.convs[0].weight, "model parameters")
        if torch.is_grad_enabled() and (
            x.requires_grad or any(p.requires_grad for p in self.parameters())
        ):
            raise RuntimeError(
                "connect6_amd.PolicyValueNet is the inference forward only: call it under "
                "torch.no_grad() / torch.inference_mode() (training stays on a PyTorch module "
                "sharing this state_dict)"
            )

    def _generic(self, x, prec, **kw):
        """Non-default architectures run layer by layer (``c6_forward_generic``)."""
        if int(x.shape[0]) == 0:
            return (torch.empty((0, self.action_size), dtype=torch.float32, device=x.device),
                    torch.empty((0,), dtype=torch.float32, device=x.device))
        return run_forward_generic(x, self.state_dict(), self.kernels, self.channels, prec, **kw)

    def forward(self, x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        self._check_input(x)
        prec = self.resolve_precision()
        if not self.is_default_architecture:
            return self._generic(x, prec)
        logits, value, _, _ = run_forward(x, self.packed_weights(prec), prec, 1, int(x.shape[0]),
                                          threshold=self.cascade_threshold, stats=self.cascade_stats)
        return logits, value

    def forward_masked(
        self,
        x: torch.Tensor,
        legal: torch.Tensor | None = None,
        fill: float | None = None,
    ) -> tuple[torch.Tensor, torch.Tensor]:
        """Forward with the occupied-square masking fused into the head:
        equals ``mask_logits(forward(x)[0].float(), legal)``.  With
        ``legal=None`` a square is occupied iff plane 0 or plane 1 of ``x`` is
        non-zero there.  ``fill`` defaults to ``finfo(float32).min``."""
        self._check_input(x)
        prec = self.resolve_precision()
        mask_mode = _lib.MASK_INPUT if legal is None else _lib.MASK_LEGAL
        fill = _FILL_LOWEST if fill is None else float(fill)
        if not self.is_default_architecture:
            return self._generic(x, prec, mask_mode=mask_mode, legal=legal, fill=fill)
        logits, value, _, _ = run_forward(
            x, self.packed_weights(prec), prec, 1, int(x.shape[0]),
            mask_mode=mask_mode, legal=legal, fill=fill,
            threshold=self.cascade_threshold, stats=self.cascade_stats,
        )
        return logits, value

    def selfplay_step(
        self,
        x: torch.Tensor,
        u: torch.Tensor,
        temperature: float = 1.0,
        legal: torch.Tensor | None = None,
        return_logits: bool = False,
    ):
        """Fused collector step: forward, occupied-square mask, masked softmax
        at ``temperature`` and one categorical draw per board by inverse CDF
        on ``u[b]`` in [0,1) -- the work of ``_sample_actions`` in the
        reference (connect6/train.py:195-203) without materialising logits.
        Returns ``(actions int64[B], logprob[B], value[B])`` (+ masked logits)."""
        self._check_input(x)
        if not self.is_default_architecture:
            raise NotImplementedError(
                "the fused self-play step is built for the default architecture on a 19x19 board; "
                "use forward_masked() followed by sample_actions() elsewhere"
            )
        prec = self.resolve_precision()
        logits, value, actions, logprob = run_forward(
            x, self.packed_weights(prec), prec, 1, int(x.shape[0]), want_logits=return_logits,
            mask_mode=_lib.MASK_INPUT if legal is None else _lib.MASK_LEGAL, legal=legal,
            u=u, temperature=temperature, want_logprob=True,
            threshold=self.cascade_threshold, stats=self.cascade_stats,
        )
        if return_logits:
            return actions, logprob, value, logits
        return actions, logprob, value

    def forward_boards(
        self,
        boards: torch.Tensor,
        current_player: torch.Tensor,
        stones_left: torch.Tensor,
        *,
        index: torch.Tensor | None = None,
        view: int = 0,
        masked: bool = True,
        fill: float | None = None,
    ) -> tuple[torch.Tensor, torch.Tensor]:
        """Forward straight from the environment's int8 state
        (``VectorConnect6.boards / .current_player / .stones_left``): one launch
        does what the reference's collector does per step with
        ``_transform_boards`` (D4 ``view`` 0..7, connect6/train.py:730-741),
        ``canonical_network_input`` (connect6/vector_env.py:196-218), the row
        gather ``network_input[index]``, the forward and -- with ``masked`` --
        ``mask_logits(logits.float(), view_boards == 0)``.  Logits are in view
        coordinates, as in the reference."""
        logits, value, _, _ = _forward_boards(self, boards, current_player, stones_left, index=index,
                                              view=view, masked=masked, fill=fill, u=None,
                                              temperature=1.0, want_logits=True)
        return logits, value

    def selfplay_step_boards(
        self,
        boards: torch.Tensor,
        current_player: torch.Tensor,
        stones_left: torch.Tensor,
        u: torch.Tensor,
        temperature: float = 1.0,
        *,
        index: torch.Tensor | None = None,
        view: int = 0,
    ):
        """``forward_boards`` + masked softmax + one inverse-CDF draw per board
        (``_sample_actions``, connect6/train.py:195-203) in the same launch.
        Returns ``(actions, logprob, value)``; actions are in view coordinates
        (map them back with ``inverse_transform_actions``)."""
        _, value, actions, logprob = _forward_boards(self, boards, current_player, stones_left,
                                                     index=index, view=view, masked=True, fill=None,
                                                     u=u, temperature=temperature, want_logits=False)
        return actions, logprob, value


def _state_tensor(t: torch.Tensor, name: str, shape, dev) -> torch.Tensor:
    if t.dtype != torch.int8:
        raise ValueError(f"{name} must be an int8 tensor (as VectorConnect6 holds it), got {t.dtype}")
    if tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")
    return t.to(dev).contiguous()


def _forward_boards(
    model: "PolicyValueNet",
    boards: torch.Tensor,
    current_player: torch.Tensor,
    stones_left: torch.Tensor,
    *,
    index: torch.Tensor | None,
    view: int,
    masked: bool,
    fill: float | None,
    u: torch.Tensor | None,
    temperature: float,
    want_logits: bool,
):
    _require_device_tensor(boards, "boards")
    _require_device_tensor(model.convs[0].weight, "model parameters")
    if not model.is_default_architecture:
        raise NotImplementedError("board-state input is built for the default architecture on a 19x19 board")
    if torch.is_grad_enabled() and any(p.requires_grad for p in model.parameters()):
        raise RuntimeError("connect6_amd.PolicyValueNet is the inference forward only: call it under "
                           "torch.no_grad() / torch.inference_mode()")
    if boards.ndim != 3 or tuple(boards.shape[1:]) != (19, 19):
        raise ValueError(f"boards must have shape [N, 19, 19], got {tuple(boards.shape)}")
    if not 0 <= int(view) <= 7:
        raise ValueError(f"view must be a D4 phase 0..7, got {view}")
    dev = boards.device
    n = int(boards.shape[0])
    boards = _state_tensor(boards, "boards", (n, 19, 19), dev)
    current_player = _state_tensor(current_player, "current_player", (n,), dev)
    stones_left = _state_tensor(stones_left, "stones_left", (n,), dev)
    if index is not None:
        if index.dtype != torch.int64 or index.ndim != 1:
            raise ValueError("index must be a 1-D int64 tensor of board rows")
        index = index.to(dev).contiguous()   # entries outside [0, N) are clamped by the kernel
    b = n if index is None else int(index.numel())
    prec = model.resolve_precision()
    packed = model.packed_weights(prec)
    logits = torch.empty((b, 361), dtype=torch.float32, device=dev) if want_logits else None
    value = torch.empty((b,), dtype=torch.float32, device=dev)
    actions = logprob = None
    if u is not None:
        u = u.to(device=dev, dtype=torch.float32).contiguous()
        if u.shape != (b,):
            raise ValueError(f"u must have shape ({b},), got {tuple(u.shape)}")
        actions = torch.empty((b,), dtype=torch.int64, device=dev)
        logprob = torch.empty((b,), dtype=torch.float32, device=dev)

    def ptr(t):
        return t.data_ptr() if t is not None else None

    with torch.cuda.device(dev):
        if prec in _lib.CASCADES:
            ws = torch.empty(_lib.cascade_workspace_bytes(b) // 4, dtype=torch.int32, device=dev)
            thr = _lib.CASCADE_THRESHOLD if model.cascade_threshold is None else model.cascade_threshold
            rc = _lib.load().c6_forward_boards_cascade(
                boards.data_ptr(), current_player.data_ptr(), stones_left.data_ptr(), n, ptr(index),
                int(view), b, packed.data_ptr(), prec, ptr(logits), _lib.DT_F32, value.data_ptr(),
                _lib.MASK_INPUT if masked else _lib.MASK_NONE,
                _FILL_LOWEST if fill is None else float(fill), ptr(u), float(temperature),
                ptr(actions), ptr(logprob), float(thr), ws.data_ptr(), ws.numel() * 4, _lib.stream_ptr(dev))
            model.cascade_stats["second_pass"] = ws[:1]
            _lib.check(rc, "c6_forward_boards_cascade")
            return logits, value, actions, logprob
        rc = _lib.load().c6_forward_boards(
            boards.data_ptr(), current_player.data_ptr(), stones_left.data_ptr(), n, ptr(index),
            int(view), b, packed.data_ptr(), prec, ptr(logits), value.data_ptr(),
            _lib.MASK_INPUT if masked else _lib.MASK_NONE,
            _FILL_LOWEST if fill is None else float(fill), ptr(u), float(temperature),
            ptr(actions), ptr(logprob), _lib.stream_ptr(dev))
    _lib.check(rc, "c6_forward_boards")
    return logits, value, actions, logprob


def build_model(model_cfg: dict[str, Any], board_size: int) -> PolicyValueNet:
    """Build the CNN from the ``model`` section of the YAML config
    (connect6/model.py:114-120): the three bookkeeping keys are ignored."""
    cfg = dict(model_cfg)
    cfg.pop("compile", None)
    cfg.pop("compile_mode", None)
    cfg.pop("architecture_version", None)
    return PolicyValueNet(board_size=board_size, **cfg)


def mask_logits(logits: torch.Tensor, legal_mask: torch.Tensor) -> torch.Tensor:
    """Block occupied squares so that a softmax can never choose them
    (connect6/model.py:123-125): out-of-place, fill = ``finfo(dtype).min``."""
    _require_device_tensor(logits, "logits")
    if logits.ndim != 2 or logits.shape[1] != 361 or legal_mask.shape != logits.shape:
        raise ValueError(
            f"mask_logits expects logits and legal mask of shape [B, 361], got "
            f"{tuple(logits.shape)} and {tuple(legal_mask.shape)}"
        )
    if legal_mask.dtype != torch.bool:
        raise ValueError("legal mask must be a bool tensor")
    lib = _lib.load()
    src = logits.contiguous()
    legal = legal_mask.to(logits.device).contiguous().view(torch.uint8)
    out = torch.empty_like(src)
    fill = torch.tensor(torch.finfo(src.dtype).min, dtype=src.dtype)
    if src.dtype == torch.float32:
        fill_bits = int(fill.view(torch.int32).item()) & 0xFFFFFFFF
    else:
        fill_bits = int(fill.view(torch.int16).item()) & 0xFFFF
    with torch.cuda.device(src.device):
        rc = lib.c6_mask_logits(src.data_ptr(), legal.data_ptr(), _lib.torch_dtype_code(src.dtype),
                                int(src.shape[0]), fill_bits, out.data_ptr(),
                                _lib.stream_ptr(src.device))
    _lib.check(rc, "c6_mask_logits")
    return out
