"""fp32-PyTorch emulation of the arithmetic contracts of the 16-bit HIP modes that go beyond plain
bf16 rounding: the bf16 + block-scaled-fp6 correction (``"bf16f6"``), the same with the weights'
low part (``"bf16f6w"``), and the decision rule of the cascade (``"bf16c"``).

TEST INFRASTRUCTURE ONLY -- the product (``connect6_amd``) never imports this.

These functions restate what the kernels in ``connect6_amd/csrc/c6_forward.hip`` are specified
to compute; the reference repository has no counterpart (its only 16-bit arithmetic is
``torch.autocast``, connect6/train.py:126-130), so nothing here cites a reference line.  What
anchors them to the reference is ``torch_ref.forward`` (connect6/model.py:96-111): with the
rounding steps removed every function below reduces to it, and the tests check that.

=========================  ====================================================================
function                   pinned by (tests/test_oracle.py)
=========================  ====================================================================
``e2m3_grid`` /            the 64 code points enumerated bit by bit in plain Python (sign,
``quant_e2m3``             2 exponent bits with bias 1, 3 mantissa bits, subnormals); round to
                           nearest with ties to the even mantissa checked against a brute-force
                           search over the grid; saturation at +-7.5; idempotence on the grid.
``block_scale``            power of two; the block's largest magnitude lands in [4, 8); the
                           closed form 2^(floor(log2 m) - 2) on random and on exact powers of two.
``quant_lo_blocks``        error <= half a grid step of the block's scale for every element that
                           does not saturate; all-zero blocks stay zero.
``forward_bf16f6_emulated``  with ``lo_mask=0`` it equals ``torch_ref.forward_bf16_emulated``
                           bit for bit; with exact (unquantised) low-order parts and weights it
                           equals the forward with bf16 weights and unrounded activations to
                           fp32 rounding; its distance to fp32 is below plain bf16's;
                           ``weights_lo`` with exact low-order parts equals the fp32 forward to
                           2^-16 relative (the weights' second rounding), and with the e2m3
                           roundings stays within 5e-4 of it.
``cascade_margin`` /       brute-force double-precision loop over the legal squares of small
``cascade_second_pass``    hand-made boards (ties, one or two legal squares, flat logits).
=========================  ====================================================================
"""
from __future__ import annotations

from typing import Mapping

import torch
import torch.nn.functional as F

from . import torch_ref as R

ACT_SCALE = -1.4426950408889634      # the 16-bit kernels carry -log2(e) x activation between layers
E2M3_MAX = 7.5


def e2m3_grid() -> torch.Tensor:
    """The non-negative values of the 6-bit float with 2 exponent bits (bias 1) and 3 mantissa
    bits (OCP MX "FP6 E2M3"), ascending: 0, 0.125 .. 0.875 (subnormal), 1 .. 1.875, 2 .. 3.75,
    4 .. 7.5."""
    vals = []
    for e in range(4):
        for m in range(8):
            vals.append(m / 8.0 if e == 0 else (1.0 + m / 8.0) * 2.0 ** (e - 1))
    return torch.tensor(vals, dtype=torch.float32)


def quant_e2m3(x: torch.Tensor) -> torch.Tensor:
    """Round to the nearest e2m3 value, ties to the even mantissa, saturating at +-7.5."""
    a = x.abs().clamp(max=E2M3_MAX)
    # grid step: 1/8 below 2, 1/4 in [2, 4), 1/2 in [4, 8)
    step = torch.where(a < 2.0, torch.full_like(a, 0.125), torch.where(a < 4.0, torch.full_like(a, 0.25),
                                                                      torch.full_like(a, 0.5)))
    q = torch.round(a / step) * step          # torch.round: half to even, and the grid's multiples
    return torch.copysign(q.clamp(max=E2M3_MAX), x)   # of `step` alternate even / odd mantissas


def block_scale(maxabs: torch.Tensor) -> torch.Tensor:
    """Power-of-two scale of a block whose largest magnitude is ``maxabs``: 2^(E-2) for a
    magnitude in [2^E, 2^(E+1)), so that the largest element lands in [4, 8); never below 2^-126
    (the smallest scale the matrix instruction's exponent byte can express besides 2^-127)."""
    m = maxabs.clamp_min(2.0 ** -126)
    e = torch.floor(torch.log2(m))
    # log2 of a float just below a power of two may round up: fix with an exact comparison
    e = torch.where(torch.pow(2.0, e) > m, e - 1, e)
    return torch.pow(2.0, (e - 2).clamp_min(-126.0))


def quant_lo_blocks(lo: torch.Tensor) -> torch.Tensor:
    """Block-scaled e2m3 of low-order parts ``lo[B, C, H, W]``: the 32 channels [32t, 32t+32) of
    one position share ``block_scale`` of their largest magnitude."""
    b, c, h, w = lo.shape
    assert c % 32 == 0
    v = lo.reshape(b, c // 32, 32, h, w)
    sc = block_scale(v.abs().amax(dim=2, keepdim=True))
    return (quant_e2m3(v / sc) * sc).reshape(b, c, h, w)


def lo_weight_copy(w: torch.Tensor) -> torch.Tensor:
    """The correction pass's copy of a 3x3 layer's weights: the bf16 weights times 2^sw (sw from
    the layer's largest |w| so that it lands just below 7.5, |sw| <= 20), as e2m3, scaled back."""
    m = float(w.abs().max())
    sw = 0
    if 0.0 < m < float("inf"):
        sw = int(torch.floor(torch.log2(torch.tensor(E2M3_MAX / m))).item())
    sw = max(-20, min(20, sw))
    wb = w.to(torch.bfloat16).to(torch.float32)
    return quant_e2m3(wb * 2.0 ** sw) / 2.0 ** sw


def forward_bf16f6_emulated(
    state: Mapping[str, torch.Tensor], x: torch.Tensor, lo_mask: int = 0xFE,
    act_scale: float = ACT_SCALE, exact_constant_plane: bool = True, exact_lo: bool = False,
    weights_lo: bool = False,
) -> tuple[torch.Tensor, torch.Tensor]:
    """The ``"bf16f6"`` contract: as ``torch_ref.forward_bf16_emulated`` (bf16 weights and layer
    inputs, fp32 accumulation, fp32 bias + SiLU, last layer and heads in fp32), plus, for every
    3x3 layer l with bit l of ``lo_mask`` set, a second contraction of what the bf16 rounding of
    the layer's input dropped (``lo = a - bf16(a)``, block-scaled e2m3) with the e2m3 copy of
    the layer's weights.  ``exact_lo`` skips both e2m3 roundings (what the correction
    approximates).  ``weights_lo`` is the ``"bf16f6w"`` contract (the cascade's second pass): every
    layer's bf16 input is also contracted with what the weights' rounding to bf16 dropped, itself
    rounded to bf16 (``w = bf16(w) + bf16(w - bf16(w))`` to 16 mantissa bits)."""
    n = R._num_layers(state)
    c = float(act_scale)
    f = x
    for i in range(n):
        w = state[f"convs.{i}.weight"]
        b = state[f"convs.{i}.bias"] * c
        pad = w.shape[-1] // 2
        if i == 0:
            wq = R._bf16_round(w * c)
            if weights_lo:
                wq = wq + R._bf16_round(w * c - wq)
            xin = R._bf16_round(f)
            u = F.conv2d(xin, wq, b, padding=pad)
            if exact_constant_plane:
                last = x[:, -1]
                const = (last == last[:, :1, :1]).flatten(1).all(dim=1).view(-1, 1, 1, 1)
                wmix = wq.clone()
                wmix[:, -1] = w[:, -1] * c
                u_exact = F.conv2d(torch.cat((xin[:, :-1], x[:, -1:]), 1), wmix, b, padding=pad)
                u = torch.where(const, u_exact, u)
        else:
            wq = R._bf16_round(w)
            hi = R._bf16_round(f)
            u = F.conv2d(hi, wq, b, padding=pad)
            if weights_lo:
                u = u + F.conv2d(hi, R._bf16_round(w - wq), None, padding=pad)
            if (lo_mask >> i) & 1:
                lo = f - hi
                if exact_lo:
                    u = u + F.conv2d(lo, wq, None, padding=pad)
                else:
                    u = u + F.conv2d(quant_lo_blocks(lo), lo_weight_copy(w), None, padding=pad)
        f = c * F.silu(u / c)
    logits = F.conv2d(f, state["policy_output.weight"] / c, state["policy_output.bias"]).flatten(1)
    vmap = F.conv2d(f, state["value_output.weight"] / c, state["value_output.bias"])
    value = torch.tanh(vmap.mean(dim=(-2, -1))).squeeze(1)
    return logits, value


def cascade_margin(logits: torch.Tensor, free: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Per board, over the free squares only and in double precision: (lead of the largest logit
    over the second largest, lead over the third largest, standard deviation of the logits).
    Missing entries (fewer than two / three free squares) are inf, the deviation then 0."""
    z = logits.double()
    neg = torch.full_like(z, float("-inf"))
    zf = torch.where(free, z, neg)
    top3 = zf.topk(3, dim=1).values
    cnt = free.sum(dim=1)
    gap2 = top3[:, 0] - top3[:, 1]          # (inf where the second entry is a masked square)
    gap3 = top3[:, 0] - top3[:, 2]
    zero = torch.zeros_like(z)
    mean = torch.where(free, z, zero).sum(1) / cnt.clamp_min(1)
    var = torch.where(free, (z - mean[:, None]) ** 2, zero).sum(1) / cnt.clamp_min(1)
    few = cnt < 2
    inf = torch.full_like(gap2, float("inf"))
    gap2 = torch.where(few, inf, gap2)
    gap3 = torch.where(cnt < 3, inf, gap3)
    std = torch.where(few, torch.zeros_like(var), var.sqrt())
    return gap2, gap3, std


def cascade_second_pass(logits: torch.Tensor, free: torch.Tensor, threshold: float) -> torch.Tensor:
    """The cascade's rule: a board is evaluated a second time iff it has at least two free
    squares and either the lead of its best free square over the second best is below
    ``threshold`` standard deviations of its free squares' logits, or at least two other free
    squares (so also the third best) lie within twice that of the best.  ``threshold < 0``:
    every board with two free squares."""
    gap2, gap3, std = cascade_margin(logits, free)
    enough = free.sum(dim=1) >= 2
    if threshold < 0:
        return enough
    return enough & ((gap2 < threshold * std) | (gap3 < 2 * threshold * std))
