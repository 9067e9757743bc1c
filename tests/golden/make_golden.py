"""Writes tests/golden/ring_small.npz: seeded inputs and the fp64 oracle's outputs for two tiny
ring shares (one per model family, zigzag layout), and tests/golden/prologue_small.npz: the same
for the two layer prologues (q/k RMSNorm + rotary embedding; MLA rotary + q/k/v assembly). The reference ships no vectors for this path
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
from oracle import prologue_oracle as P  # noqa: E402
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
    prologue()


def prologue():
    out = {}
    g = torch.Generator().manual_seed(123)
    bf = torch.bfloat16
    # q/k RMSNorm + rotary embedding (GQA layer): x [1, 12, 3, 128]
    x = torch.randn(1, 12, 3, 128, generator=g).to(bf)
    w = (torch.rand(128, generator=g) + 0.5).to(bf)
    dout = torch.randn(1, 12, 3, 128, generator=g).to(bf)
    cos, sin = P.cos_sin_table(torch.arange(12).unsqueeze(0) + 5000, 128, dtype=bf)
    y = P.norm_rope_fwd(x, w, cos, sin, 1e-6)
    dx, dw = P.norm_rope_bwd(x, w, cos, sin, dout, 1e-6)
    for k, t in (("x", x), ("w", w), ("dout", dout), ("cos", cos), ("sin", sin)):
        out[f"nr_{k}"] = bf16_bits(t)
    for k, t in (("y", y), ("dx", dx), ("dw", dw)):
        out[f"nr_{k}"] = t.numpy()
    # MLA layer: q [1, 10, 2, 192], kv [1, 10, 2, 256], k_pe [1, 10, 64], tables [32, 64]
    q = torch.randn(1, 10, 2, 192, generator=g).to(bf)
    kv = torch.randn(1, 10, 2, 256, generator=g).to(bf)
    k_pe = torch.randn(1, 10, 64, generator=g).to(bf)
    ang = torch.rand(32, 32, generator=g) * 6.283
    tab = torch.cat((ang, ang), -1)
    tcos, tsin = (tab.cos() * 1.07).to(bf), (tab.sin() * 1.07).to(bf)
    pos = torch.randint(0, 32, (1, 10), generator=g)
    outs = P.mla_assemble_fwd(q, kv, k_pe, tcos, tsin, pos, 128)
    grads = [torch.randn(t.shape, generator=g).to(bf) for t in outs]
    gin = P.mla_assemble_bwd(*grads, tcos, tsin, pos, 128)
    for k, t in (("q", q), ("kv", kv), ("k_pe", k_pe), ("cos", tcos), ("sin", tsin),
                 ("gq", grads[0]), ("gk", grads[1]), ("gv", grads[2])):  # fmt: skip
        out[f"ma_{k}"] = bf16_bits(t)
    out["ma_pos"] = pos.numpy()
    for k, t in zip(("query", "key", "value", "dq", "dkv", "dk_pe"), (*outs, *gin)):
        out[f"ma_{k}"] = t.numpy()
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "prologue_small.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
