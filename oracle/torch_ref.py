"""Plain-PyTorch fp32 restatement of the reference's batched CNN forward path.

TEST INFRASTRUCTURE ONLY -- the product (``connect6_amd``) never imports this.

Every function cites the reference file:line it follows (paths are relative to
the reference repository root).  All arithmetic lives in PyTorch library
routines, exactly as in the reference (which is pure PyTorch); the reference
holds no numeric golden vectors for this path, so the oracle is pinned by:

=====================  =====================================================
function               pinned by (tests/test_oracle.py)
=====================  =====================================================
``init_state``         shapes/keys (tests/test_model.py:21-37 of the
                       reference); fan-in std of the Kaiming-normal init;
                       zero biases.  RNG stream identity with the reference
                       is NOT needed: parity always loads one state dict on
                       both sides.
``forward``            brute-force double-precision direct convolution in
                       plain C (``conv_ref.c``) on tiny and default shapes;
                       zero-input known answer (logits == policy bias,
                       value == tanh(value bias)); -1 <= value <= 1;
                       hand-computed 1-layer 1x1 case.
``forward_grouped``    the reference's own invariant grouped[i] ==
                       single(model_i, x[i]) (tests/test_training_features.py
                       :120-151 of the reference).
``mask_logits``        closed form; bit-pattern check of fill / untouched.
``canonical_network_   channel meaning as the reference tests it (tests/test_game.py
input``                :46-59, :62-75): hand-built position, values exactly {0,1}.
``sample_inverse_cdf`` brute-force python loop on tiny inputs; empirical
                       distribution vs softmax; never picks a masked square.
``transform_*``        the reference's property tests (tests/test_model.py
                       :40-53, tests/test_training_features.py:154-187) and
                       the library routines ``torch.rot90``/``torch.flip``;
                       exhaustive over 8 views x all actions.
``d4_average``         identity when the network is replaced by an
                       equivariant map; brute-force loop.
=====================  =====================================================
"""
from __future__ import annotations

import math
from typing import Mapping, Sequence

import torch
import torch.nn.functional as F

DEFAULT_KERNELS = (23, 3, 3, 3, 3, 3, 3, 3)      # connect6/model.py:22
DEFAULT_CHANNELS = (32, 32, 64, 64, 64, 96, 96, 96)  # connect6/model.py:23
INPUT_CHANNELS = 3                                # connect6/model.py:24


# --------------------------------------------------------------------------
# parameters
# --------------------------------------------------------------------------
def init_state(
    seed: int,
    init: str = "reference",
    kernels: Sequence[int] = DEFAULT_KERNELS,
    channels: Sequence[int] = DEFAULT_CHANNELS,
) -> dict[str, torch.Tensor]:
    """Seeded fp32 parameters with the reference's state_dict key names.

    ``init="reference"`` follows connect6/model.py:83-94: conv weights
    Kaiming-normal for ReLU gain (std = sqrt(2 / fan_in)), conv biases zero,
    both 1x1 heads N(0, 0.01) with zero bias.  ``init="torch_default"`` is
    what ``nn.Conv2d`` does on construction (connect6/model.py:56-63 before
    the override): weights and biases uniform in +-1/sqrt(fan_in).
    """
    g = torch.Generator(device="cpu").manual_seed(int(seed))
    state: dict[str, torch.Tensor] = {}
    cin = INPUT_CHANNELS
    for i, (k, cout) in enumerate(zip(kernels, channels)):
        fan_in = cin * k * k
        if init == "reference":
            w = torch.randn(cout, cin, k, k, generator=g) * math.sqrt(2.0 / fan_in)
            b = torch.zeros(cout)
        elif init == "torch_default":
            bound = 1.0 / math.sqrt(fan_in)
            w = (torch.rand(cout, cin, k, k, generator=g) * 2 - 1) * bound
            b = (torch.rand(cout, generator=g) * 2 - 1) * bound
        else:
            raise ValueError(f"unknown init {init!r}")
        state[f"convs.{i}.weight"] = w
        state[f"convs.{i}.bias"] = b
        cin = cout
    for head in ("policy_output", "value_output"):
        if init == "reference":
            w = torch.randn(1, cin, 1, 1, generator=g) * 0.01
            b = torch.zeros(1)
        else:
            bound = 1.0 / math.sqrt(cin)
            w = (torch.rand(1, cin, 1, 1, generator=g) * 2 - 1) * bound
            b = (torch.rand(1, generator=g) * 2 - 1) * bound
        state[f"{head}.weight"] = w
        state[f"{head}.bias"] = b
    return state


def _num_layers(state: Mapping[str, torch.Tensor]) -> int:
    n = 0
    while f"convs.{n}.weight" in state:
        n += 1
    return n


# --------------------------------------------------------------------------
# single-model forward
# --------------------------------------------------------------------------
def forward(
    state: Mapping[str, torch.Tensor], x: torch.Tensor
) -> tuple[torch.Tensor, torch.Tensor]:
    """connect6/model.py:96-111: 8 x (same-padded conv + bias, SiLU), then the
    1x1 policy conv flattened row-major to [B, H*W] and the 1x1 value conv ->
    mean over the board -> tanh -> [B]."""
    n = _num_layers(state)
    w0 = state["convs.0.weight"]
    board = x.shape[-1]
    expected = (w0.shape[1], board, board)
    if x.ndim != 4 or tuple(x.shape[1:]) != expected or x.shape[-2] != board:
        raise ValueError(f"input must be [B, {expected}], got {tuple(x.shape)}")
    f = x
    for i in range(n):
        w = state[f"convs.{i}.weight"]
        f = F.conv2d(f, w, state[f"convs.{i}.bias"], stride=1, padding=w.shape[-1] // 2)
        f = F.silu(f)
    logits = F.conv2d(f, state["policy_output.weight"], state["policy_output.bias"]).flatten(1)
    vmap = F.conv2d(f, state["value_output.weight"], state["value_output.bias"])
    value = torch.tanh(vmap.mean(dim=(-2, -1))).squeeze(1)
    return logits, value


def _bf16_round(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.bfloat16).to(torch.float32)


def forward_bf16_emulated(
    state: Mapping[str, torch.Tensor], x: torch.Tensor, act_scale: float = 1.0,
    exact_constant_plane: bool = False,
) -> tuple[torch.Tensor, torch.Tensor]:
    """The arithmetic contract of the bf16 HIP paths, emulated in fp32 torch:
    conv weights and layer inputs rounded to bf16 (RNE), fp32 accumulation,
    bias + SiLU in fp32, ONE rounding to bf16 at each layer boundary, last
    layer's activations and the two heads kept in fp32.

    ``act_scale`` c != 1 models the fused kernel, which carries c * activation
    between layers (c = -log2 e): first-layer weights are rounded AFTER the
    scaling, later layers see bf16(c * silu), biases are c * b in fp32, and the
    heads divide the factor out again.  Mathematically the same network.

    ``exact_constant_plane`` models the pipelined kernel's first layer: on a board whose last
    input plane is one constant, that plane's weights are summed per output square in fp32
    (unrounded) instead of going through the bf16 contraction."""
    n = _num_layers(state)
    c = float(act_scale)
    f = _bf16_round(x)
    for i in range(n):
        w = state[f"convs.{i}.weight"]
        wq = _bf16_round(w * c) if i == 0 else _bf16_round(w)
        if i == 0 and exact_constant_plane:
            last = x[:, -1]
            const = (last == last[:, :1, :1]).flatten(1).all(dim=1).view(-1, 1, 1, 1)
            wmix = wq.clone()
            wmix[:, -1] = w[:, -1] * c      # the constant plane's weights unrounded ...
            u_exact = F.conv2d(torch.cat((f[:, :-1], x[:, -1:]), 1), wmix, state["convs.0.bias"] * c,
                               stride=1, padding=w.shape[-1] // 2)   # ... times its unrounded value
            u_plain = F.conv2d(f, wq, state["convs.0.bias"] * c, stride=1, padding=w.shape[-1] // 2)
            u = torch.where(const, u_exact, u_plain)
            f = c * F.silu(u / c)
            f = _bf16_round(f)
            continue
        u = F.conv2d(f, wq, state[f"convs.{i}.bias"] * c, stride=1, padding=w.shape[-1] // 2)
        f = c * F.silu(u / c)
        if i + 1 < n:
            f = _bf16_round(f)
    logits = F.conv2d(f, state["policy_output.weight"] / c, state["policy_output.bias"]).flatten(1)
    vmap = F.conv2d(f, state["value_output.weight"] / c, state["value_output.bias"])
    value = torch.tanh(vmap.mean(dim=(-2, -1))).squeeze(1)
    return logits, value


# --------------------------------------------------------------------------
# grouped history forward
# --------------------------------------------------------------------------
def _grouped_conv(x, weight, bias, padding):
    """connect6/history.py:251-274: fold the M models into conv groups."""
    m, t, c, h, w = x.shape
    o, k = int(weight.shape[1]), int(weight.shape[-1])
    gx = x.permute(1, 0, 2, 3, 4).reshape(t, m * c, h, w)
    gw = weight.reshape(m * o, c, k, k)
    gb = bias.reshape(m * o) if bias is not None else None
    y = F.conv2d(gx, gw, gb, stride=1, padding=padding, groups=m)
    return y.reshape(t, m, o, h, w).permute(1, 0, 2, 3, 4)


def forward_grouped(
    states: Sequence[Mapping[str, torch.Tensor]], x: torch.Tensor
) -> torch.Tensor:
    """connect6/history.py:276-303: x [M,T,3,H,W] -> policy logits [M,T,H*W].
    Policy only: no value head, no masking."""
    m = len(states)
    if m == 0:
        raise ValueError("at least one checkpoint is required")  # history.py:202-203
    if x.ndim != 5 or x.shape[0] != m:
        raise ValueError(f"expected [M={m},T,3,H,W], got {tuple(x.shape)}")
    n = _num_layers(states[0])
    for i in range(n):
        w = torch.stack([s[f"convs.{i}.weight"] for s in states])   # history.py:224-236
        b = torch.stack([s[f"convs.{i}.bias"] for s in states])
        x = F.silu(_grouped_conv(x, w, b, w.shape[-1] // 2))
    pw = torch.stack([s["policy_output.weight"] for s in states])
    pb = torch.stack([s["policy_output.bias"] for s in states])
    return _grouped_conv(x, pw, pb, 0).squeeze(2).flatten(2)


def forward_grouped_loop(states, x):
    """The invariant the reference tests (tests/test_training_features.py
    :146-151): group i equals model i applied to x[i]."""
    return torch.stack([forward(s, x[i])[0] for i, s in enumerate(states)])


# --------------------------------------------------------------------------
# mask + sampling
# --------------------------------------------------------------------------
def mask_logits(logits: torch.Tensor, legal: torch.Tensor, fill: float | None = None) -> torch.Tensor:
    """connect6/model.py:123-125.  ``fill=None`` is the reference's
    ``finfo(dtype).min``; benchmarks may ask for ``-inf``."""
    if fill is None:
        fill = torch.finfo(logits.dtype).min
    return logits.masked_fill(~legal, fill)


def legal_from_input(x: torch.Tensor) -> torch.Tensor:
    """connect6/vector_env.py:95-96 with :212-214: a square is legal iff
    neither the own-stone nor the opponent-stone plane is set."""
    return ((x[:, 0] == 0) & (x[:, 1] == 0)).flatten(1)


def sample_inverse_cdf(
    logits: torch.Tensor, legal: torch.Tensor, u: torch.Tensor, temperature: float = 1.0
) -> tuple[torch.Tensor, torch.Tensor]:
    """Categorical draw from ``mask_logits(logits.float(), legal) / max(T,1e-4)``
    (connect6/train.py:195-203) by inverse CDF on a supplied uniform ``u[B]``:
    action = first index whose running probability sum exceeds ``u * total``;
    log-prob = log-softmax at that index (what ``Categorical.log_prob``
    returns, train.py:203)."""
    z = mask_logits(logits.float(), legal) / max(float(temperature), 1e-4)
    zmax = z.max(dim=1, keepdim=True).values
    e = torch.exp(z - zmax)
    c = torch.cumsum(e, dim=1)
    total = c[:, -1:]
    target = u.float().view(-1, 1) * total
    a = (c <= target).sum(dim=1)
    last_legal = (legal.shape[1] - 1) - torch.flip(legal, dims=(1,)).float().argmax(dim=1)
    a = torch.minimum(a, last_legal)
    logp = z.gather(1, a.view(-1, 1)).squeeze(1) - zmax.squeeze(1) - torch.log(total.squeeze(1))
    return a, logp


def canonical_network_input(boards: torch.Tensor, current_player: torch.Tensor,
                            stones_left: torch.Tensor) -> torch.Tensor:
    """connect6/vector_env.py:196-218: int8 boards [N,n,n] (+1/-1/0), side to move [N],
    stones left [N] -> fp32 planes [N,3,n,n]: own stones, opponent stones, "last stone of
    the turn" flag broadcast over the board."""
    player = current_player.view(-1, 1, 1)
    me = boards.eq(player).to(torch.float32)
    opp = boards.eq(-player).to(torch.float32)
    last = stones_left.eq(1).to(torch.float32).view(-1, 1, 1).expand(-1, boards.shape[-2], boards.shape[-1])
    return torch.stack((me, opp, last), dim=1)


# --------------------------------------------------------------------------
# D4 views
# --------------------------------------------------------------------------
def symmetry_for_phase(phase: int) -> tuple[int, bool]:
    """connect6/train.py:216-219."""
    phase = int(phase) % 8
    return phase % 4, phase >= 4


def transform_actions(actions: torch.Tensor, n: int, k: int, flip: bool) -> torch.Tensor:
    """connect6/train.py:233-253: canonical (r,c) -> coordinates in the view."""
    k = int(k) % 4
    r, c = actions // n, actions % n
    if k == 1:
        r, c = n - 1 - c, r
    elif k == 2:
        r, c = n - 1 - r, n - 1 - c
    elif k == 3:
        r, c = c, n - 1 - r
    if flip:
        c = n - 1 - c
    return r * n + c


def inverse_transform_actions(actions: torch.Tensor, n: int, k: int, flip: bool) -> torch.Tensor:
    """connect6/train.py:256-277: undo the mirror, then the rotation."""
    k = int(k) % 4
    r, c = actions // n, actions % n
    if flip:
        c = n - 1 - c
    if k == 1:
        r, c = c, n - 1 - r
    elif k == 2:
        r, c = n - 1 - r, n - 1 - c
    elif k == 3:
        r, c = n - 1 - c, r
    return r * n + c


def transform_boards(boards: torch.Tensor, k: int, flip: bool) -> torch.Tensor:
    """connect6/train.py:222-230 stated as one gather: the view's square
    ``transform_actions(a)`` shows what the canonical board has at ``a``."""
    n = boards.shape[-1]
    a = torch.arange(n * n)
    src = inverse_transform_actions(a, n, k, flip)      # view index -> canonical index
    flat = boards.reshape(*boards.shape[:-2], n * n)
    return flat[..., src].reshape(boards.shape)


def d4_expand(x: torch.Tensor) -> torch.Tensor:
    """[B,C,n,n] -> [8,B,C,n,n], view ``p`` = transform_boards(x, *symmetry_for_phase(p))."""
    return torch.stack([transform_boards(x, *symmetry_for_phase(p)) for p in range(8)])


def d4_average(view_logits: torch.Tensor, view_values: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """view_logits [8,B,n*n], view_values [8,B] -> canonical mean logits and
    values: canonical[b, a] = mean_p view_logits[p, b, transform_actions(a; p)]."""
    nn_ = view_logits.shape[-1]
    n = int(round(math.sqrt(nn_)))
    a = torch.arange(nn_)
    acc = torch.zeros_like(view_logits[0], dtype=torch.float32)
    for p in range(8):
        k, flip = symmetry_for_phase(p)
        acc += view_logits[p].float()[:, transform_actions(a, n, k, flip)]
    return acc / 8.0, view_values.float().mean(dim=0)
