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


# ---------------------------------------------------------------------------------------------
# layer prologues (tests/golden/prologue_small.npz)

PROLOGUE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "prologue_small.npz")


def _prologue():
    z = np.load(PROLOGUE)
    bf = lambda a: torch.from_numpy(a.copy()).view(torch.bfloat16)  # noqa: E731
    bits = {"nr_x", "nr_w", "nr_dout", "nr_cos", "nr_sin", "ma_q", "ma_kv", "ma_k_pe", "ma_cos", "ma_sin", "ma_gq", "ma_gk", "ma_gv"}
    return {k: (bf(z[k]) if k in bits else torch.from_numpy(z[k])) for k in z.files}


def test_prologue_oracle_reproduces_fixtures():
    from oracle import prologue_oracle as P

    d = _prologue()
    y = P.norm_rope_fwd(d["nr_x"], d["nr_w"], d["nr_cos"], d["nr_sin"], 1e-6)
    dx, dw = P.norm_rope_bwd(d["nr_x"], d["nr_w"], d["nr_cos"], d["nr_sin"], d["nr_dout"], 1e-6)
    for got, want in ((y, d["nr_y"]), (dx, d["nr_dx"]), (dw, d["nr_dw"])):
        assert torch.allclose(got, want, rtol=1e-12, atol=1e-12)
    outs = P.mla_assemble_fwd(d["ma_q"], d["ma_kv"], d["ma_k_pe"], d["ma_cos"], d["ma_sin"], d["ma_pos"], 128)
    gin = P.mla_assemble_bwd(d["ma_gq"], d["ma_gk"], d["ma_gv"], d["ma_cos"], d["ma_sin"], d["ma_pos"], 128)
    for got, name in zip((*outs, *gin), ("query", "key", "value", "dq", "dkv", "dk_pe")):
        assert torch.allclose(got, d[f"ma_{name}"], rtol=1e-12, atol=1e-12), name


@pytest.mark.gpu
def test_hip_prologues_match_fixtures(gpu):
    from helpers import assert_close
    from pithtrain_amd.operators.mla_assemble import mla_assemble_bwd_into, mla_assemble_fwd_into
    from pithtrain_amd.operators.norm_rope import norm_rope_bwd_into, norm_rope_fwd_into

    d = _prologue()
    g = {k: v.to(gpu) for k, v in d.items()}
    tol = lambda want: dict(rtol=2.0**-8, atol=1e-5 * want.abs().max().item())  # noqa: E731
    y, dx, dw = torch.empty_like(g["nr_x"]), torch.empty_like(g["nr_x"]), torch.empty(128, device=gpu)
    norm_rope_fwd_into(g["nr_x"], g["nr_w"], g["nr_cos"], g["nr_sin"], y, 1e-6)
    norm_rope_bwd_into(g["nr_x"], g["nr_w"], g["nr_cos"], g["nr_sin"], g["nr_dout"], dx, dw, 1e-6)
    assert_close(y, d["nr_y"], what="y", **tol(d["nr_y"]))
    assert_close(dx, d["nr_dx"], what="dx", **tol(d["nr_dx"]))
    assert_close(dw, d["nr_dw"], rtol=1e-4, atol=1e-4 * d["nr_dw"].abs().max().item(), what="dweight")
    bf = torch.bfloat16
    outs = [torch.empty(d[f"ma_{n}"].shape, dtype=bf, device=gpu) for n in ("query", "key", "value")]
    mla_assemble_fwd_into(g["ma_q"], g["ma_kv"], g["ma_k_pe"], g["ma_cos"], g["ma_sin"], g["ma_pos"], *outs)
    gin = [torch.empty(d[f"ma_{n}"].shape, dtype=bf, device=gpu) for n in ("dq", "dkv", "dk_pe")]
    mla_assemble_bwd_into(g["ma_gq"], g["ma_gk"], g["ma_gv"], g["ma_cos"], g["ma_sin"], g["ma_pos"], *gin)
    for got, name in zip((*outs, *gin), ("query", "key", "value", "dq", "dkv", "dk_pe")):
        assert_close(got, d[f"ma_{name}"], what=name, **tol(d[f"ma_{name}"]))
