"""Writes tests/golden/ring_small.npz: seeded inputs and the fp64 oracle's outputs for two tiny
ring shares (one per model family, zigzag layout). The reference ships no vectors for this path
(its tests regenerate inputs from seeds), so these fixtures come from this repository's own oracle
(oracle/ring_oracle.py, pinned in tests/test_oracle.py) and guard against silent drift of the
oracle; the GPU tests also compare the HIP kernels with them. Run from the repository root:

    python tests/golden/make_golden.py
"""

import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import ring_oracle as R  # noqa: E402

CASES = {  # name: (Hq, Hkv, Dqk, Dv, S_local, C, rank)
    "gqa": (2, 1, 128, 128, 32, 2, 1),
    "mla": (1, 1, 192, 128, 32, 2, 0),
}


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.to(torch.bfloat16).view(torch.int16).numpy()


def main():
    out = {}
    for name, (hq, hkv, dqk, dv, s_l, c, r) in CASES.items():
        g = torch.Generator().manual_seed(42)
        q = torch.randn(1, s_l, hq, dqk, generator=g).to(torch.bfloat16)
        ks = [torch.randn(1, s_l, hkv, dqk, generator=g).to(torch.bfloat16) for _ in range(c)]
        vs = [torch.randn(1, s_l, hkv, dv, generator=g).to(torch.bfloat16) for _ in range(c)]
        dout = torch.randn(1, s_l, hq, dv, generator=g).to(torch.bfloat16)
        scale = dqk**-0.5
        o, lse = R.ring_forward(q, ks, vs, scale, r, c, "zigzag")
        dq, dks, dvs = R.ring_backward(dout, q, o, lse, ks, vs, scale, r, c, "zigzag")
        out[f"{name}_q"], out[f"{name}_dout"] = bf16_bits(q), bf16_bits(dout)
        out[f"{name}_k"] = np.stack([bf16_bits(t) for t in ks])
        out[f"{name}_v"] = np.stack([bf16_bits(t) for t in vs])
        out[f"{name}_o"], out[f"{name}_lse"], out[f"{name}_dq"] = (t.float().numpy() for t in (o, lse, dq))
        out[f"{name}_dk"] = np.stack([t.float().numpy() for t in dks])
        out[f"{name}_dv"] = np.stack([t.float().numpy() for t in dvs])
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ring_small.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
