"""Committed fixtures (tests/golden/ring_small.npz, written by tests/golden/make_golden.py from the
fp64 oracle): the oracle still reproduces them (CPU), and the HIP ring share matches them (GPU)."""

import os

import numpy as np
import pytest
import torch

from helpers import check_bf16_result, check_lse
from oracle import ring_oracle as R

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ring_small.npz")
CASES = {"gqa": (2, 1, 128, 128, 32, 2, 1), "mla": (1, 1, 192, 128, 32, 2, 0)}


def _load(name):
    z = np.load(GOLDEN)  # allow_pickle=False by default
    bf = lambda a: torch.from_numpy(a.copy()).view(torch.bfloat16)  # noqa: E731
    c = CASES[name][5]
    return dict(
        q=bf(z[f"{name}_q"]), dout=bf(z[f"{name}_dout"]),
        ks=[bf(z[f"{name}_k"][j]) for j in range(c)], vs=[bf(z[f"{name}_v"][j]) for j in range(c)],
        o=torch.from_numpy(z[f"{name}_o"]), lse=torch.from_numpy(z[f"{name}_lse"]), dq=torch.from_numpy(z[f"{name}_dq"]),
        dk=torch.from_numpy(z[f"{name}_dk"]), dv=torch.from_numpy(z[f"{name}_dv"]),
    )  # fmt: skip


@pytest.mark.parametrize("name", list(CASES))
def test_oracle_reproduces_fixtures(name):
    hq, hkv, dqk, dv, s_l, c, r = CASES[name]
    d = _load(name)
    o, lse = R.ring_forward(d["q"], d["ks"], d["vs"], dqk**-0.5, r, c, "zigzag")
    dq, dks, dvs = R.ring_backward(d["dout"], d["q"], o, lse, d["ks"], d["vs"], dqk**-0.5, r, c, "zigzag")
    assert torch.allclose(o.float(), d["o"], rtol=1e-6, atol=1e-7)
    assert torch.allclose(lse.float(), d["lse"], rtol=1e-6, atol=1e-6)
    assert torch.allclose(dq.float(), d["dq"], rtol=1e-5, atol=1e-6)
    for j in range(c):
        assert torch.allclose(dks[j].float(), d["dk"][j], rtol=1e-5, atol=1e-6)
        assert torch.allclose(dvs[j].float(), d["dv"][j], rtol=1e-5, atol=1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(CASES))
def test_hip_ring_matches_fixtures(gpu, name):
    from pithtrain_amd.operators.ring_attention.local import ring_backward_local, ring_forward_local

    hq, hkv, dqk, dv, s_l, c, r = CASES[name]
    d = _load(name)
    q, dout = d["q"].to(gpu), d["dout"].to(gpu)
    ks, vs = [t.to(gpu) for t in d["ks"]], [t.to(gpu) for t in d["vs"]]
    out, lse = ring_forward_local(q, ks, vs, dqk**-0.5, r, c, "zigzag")
    dq, dks, dvs = ring_backward_local(dout, q, out, lse, ks, vs, dqk**-0.5, r, c, "zigzag")
    check_bf16_result(out, d["o"], "O")
    check_lse(lse, d["lse"], "LSE2")
    check_bf16_result(dq, d["dq"], "dQ", otol=1e-3)
    for j in range(c):
        check_bf16_result(dks[j], d["dk"][j], f"dK{j}", otol=1e-3)
        check_bf16_result(dvs[j], d["dv"][j], f"dV{j}", otol=1e-3)
