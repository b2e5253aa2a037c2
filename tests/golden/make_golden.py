#!/usr/bin/env python3
"""Writes tests/golden/default_arch_golden.npz: seeded inputs and the fp32 oracle's outputs.

The reference repository holds no numeric vectors for this path (it was not imported or run);
these fixtures come from THIS repository's oracle (oracle/torch_ref.py, itself pinned by the
brute-force C convolution and closed forms in tests/test_oracle.py).  They guard against drift
of the oracle across PyTorch versions and give the GPU tests a file-based target.

    python tests/golden/make_golden.py
"""
import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parent.parent.parent
sys.path.insert(0, str(ROOT))

from connect6_amd.synthetic import gen_boards, gen_uniform  # noqa: E402
from oracle import torch_ref as R  # noqa: E402


def main() -> None:
    torch.set_num_threads(1)          # fixed summation order
    out = {}
    x, legal = gen_boards(6, 200, 2025)
    u = gen_uniform(6, 7)
    out["x"] = x.numpy()
    out["legal"] = legal.numpy()
    out["u"] = u.numpy()
    for init in ("reference", "torch_default"):
        st = R.init_state(1234, init)
        with torch.inference_mode():
            logits, value = R.forward(st, x)
            actions, logprob = R.sample_inverse_cdf(logits, legal, u, 1.0)
        out[f"{init}_logits"] = logits.numpy()
        out[f"{init}_value"] = value.numpy()
        out[f"{init}_actions"] = actions.numpy()
        out[f"{init}_logprob"] = logprob.numpy()
    np.savez_compressed(Path(__file__).resolve().parent / "default_arch_golden.npz", **out)
    print("wrote default_arch_golden.npz", {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
