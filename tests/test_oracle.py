"""Pins the CPU oracle (oracle/ring_oracle.py) before anything is checked against it.

The reference holds no golden vectors for this path (every one of its tests regenerates inputs
from a seed and compares against an in-process implementation), so the oracle is pinned by what
the mathematics fixes: library routines, brute force, closed forms and invariants, plus the
reference's own three combine properties (tests/test_online_softmax_combine_log2.py:44-106) and
the ring-vs-full-sequence design of tests/test_ring_mla_attention.py:79-108.
"""

import math

import pytest
import torch
import torch.nn.functional as F

from oracle import ring_oracle as R

F64 = torch.float64


def _rand(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=F64) * scale


def _qkv(B, Sq, Skv, Hq, Hkv, Dqk, Dv, seed):
    return _rand((B, Sq, Hq, Dqk), seed), _rand((B, Skv, Hkv, Dqk), seed + 1), _rand((B, Skv, Hkv, Dv), seed + 2)


SHAPES = [  # B, Sq, Skv, Hq, Hkv, Dqk, Dv, causal
    (1, 24, 24, 2, 2, 16, 16, True),
    (2, 16, 40, 4, 2, 24, 8, False),
    (1, 33, 33, 6, 2, 8, 8, True),
]


@pytest.mark.parametrize("B,Sq,Skv,Hq,Hkv,Dqk,Dv,causal", SHAPES)
def test_chunk_fwd_against_sdpa_and_logsumexp(B, Sq, Skv, Hq, Hkv, Dqk, Dv, causal):
    q, k, v = _qkv(B, Sq, Skv, Hq, Hkv, Dqk, Dv, seed=11)
    scale = 0.37
    o, lse = R.chunk_fwd(q, k, v, scale, causal)
    g = Hq // Hkv
    ke, ve = k.repeat_interleave(g, dim=2), v.repeat_interleave(g, dim=2)
    ref = F.scaled_dot_product_attention(
        q.transpose(1, 2), ke.transpose(1, 2), ve.transpose(1, 2), is_causal=causal, scale=scale
    ).transpose(1, 2)
    assert torch.allclose(o, ref, rtol=1e-10, atol=1e-12)
    # LSE2 = log2 sum_j exp(scale * s_ij), from the natural-log routine
    s = torch.einsum("bihd,bjhd->bhij", q, ke) * scale
    if causal:
        s = s.masked_fill(torch.ones(Sq, Skv, dtype=torch.bool).triu(1), float("-inf"))
    assert torch.allclose(lse, torch.logsumexp(s, dim=-1) / math.log(2.0), rtol=1e-12, atol=1e-12)


def test_chunk_fwd_brute_force_rows():
    """Scalar loops over one head: catches a transposed operand or a wrong mask direction."""
    B, S, H, D = 1, 7, 1, 5
    q, k, v = _qkv(B, S, S, H, H, D, D, seed=5)
    scale = 0.5
    o, lse = R.chunk_fwd(q, k, v, scale, True)
    for i in range(S):
        w = [math.exp(scale * sum(q[0, i, 0, d].item() * k[0, j, 0, d].item() for d in range(D))) for j in range(i + 1)]
        z = sum(w)
        for d in range(D):
            expect = sum(w[j] * v[0, j, 0, d].item() for j in range(i + 1)) / z
            assert abs(o[0, i, 0, d].item() - expect) < 1e-12
        assert abs(lse[0, 0, i].item() - math.log2(z)) < 1e-12


def test_chunk_fwd_causal_first_row_closed_form():
    q, k, v = _qkv(2, 9, 9, 4, 2, 12, 6, seed=3)
    scale = 12**-0.5
    o, lse = R.chunk_fwd(q, k, v, scale, True)
    ve = v.repeat_interleave(2, dim=2)
    ke = k.repeat_interleave(2, dim=2)
    assert torch.allclose(o[:, 0], ve[:, 0], rtol=0, atol=1e-14)
    expect = (q[:, 0] * ke[:, 0]).sum(-1) * scale * R.LOG2E
    assert torch.allclose(lse[:, :, 0], expect, rtol=1e-13, atol=1e-13)


def _dense_attention(q, k, v, scale, causal):
    """Independent dense attention used for autograd (natural softmax, explicit head loop)."""
    B, Sq, Hq, _ = q.shape
    g = Hq // k.shape[2]
    outs = []
    for h in range(Hq):
        s = q[:, :, h] @ k[:, :, h // g].transpose(-1, -2) * scale
        if causal:
            s = s + torch.full((Sq, k.shape[1]), float("-inf"), dtype=s.dtype).triu(1)
        outs.append(torch.softmax(s, dim=-1) @ v[:, :, h // g])
    return torch.stack(outs, dim=2)


@pytest.mark.parametrize("B,Sq,Skv,Hq,Hkv,Dqk,Dv,causal", SHAPES)
def test_chunk_bwd_against_autograd(B, Sq, Skv, Hq, Hkv, Dqk, Dv, causal):
    q, k, v = _qkv(B, Sq, Skv, Hq, Hkv, Dqk, Dv, seed=21)
    dout = _rand((B, Sq, Hq, Dv), 99)
    scale = 0.41
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
    _dense_attention(qa, ka, va, scale, causal).backward(dout)
    o, lse = R.chunk_fwd(q, k, v, scale, causal)
    delta = R.bwd_delta(o, dout)
    dq, dk, dv = R.chunk_bwd(q, k, v, dout, lse, delta, scale, causal)
    assert torch.allclose(dq, qa.grad, rtol=1e-9, atol=1e-11)
    assert torch.allclose(dk, ka.grad, rtol=1e-9, atol=1e-11)
    assert torch.allclose(dv, va.grad, rtol=1e-9, atol=1e-11)


def test_delta_identity():
    """delta_i = sum_j P_ij dP_ij with dP = dO V^T."""
    q, k, v = _qkv(1, 12, 20, 2, 2, 8, 6, seed=8)
    dout = _rand((1, 12, 2, 6), 77)
    o, lse = R.chunk_fwd(q, k, v, 0.3, False)
    s = torch.einsum("bihd,bjhd->bhij", q, k) * 0.3
    p = torch.softmax(s, dim=-1)
    dp = torch.einsum("bihd,bjhd->bhij", dout, v)
    assert torch.allclose(R.bwd_delta(o, dout), (p * dp).sum(-1), rtol=1e-11, atol=1e-12)
    assert torch.allclose(p.sum(-1), torch.ones_like(p.sum(-1)), atol=1e-13)


# ---------------------------------------------------------------------------------------------
# combine


def _combine_independent(o1, l1, o2, l2, base):
    """logaddexp formulation: lse = log(b^l1 + b^l2), out = o1*b^(l1-lse) + o2*b^(l2-lse)."""
    ln = math.log(base)
    lse = torch.logaddexp(l1 * ln, l2 * ln) / ln
    w1 = torch.exp((l1 - lse) * ln).transpose(1, 2).unsqueeze(-1)
    w2 = torch.exp((l2 - lse) * ln).transpose(1, 2).unsqueeze(-1)
    return w1 * o1 + w2 * o2, lse


@pytest.mark.parametrize("fn,base", [(R.combine_log2, 2.0), (R.combine_ln, math.e)])
def test_combine_against_logaddexp(fn, base):
    B, S, H, D = 2, 17, 3, 8
    o1, o2 = _rand((B, S, H, D), 1), _rand((B, S, H, D), 2)
    g = torch.Generator().manual_seed(3)
    l1 = torch.rand((B, H, S), generator=g, dtype=F64) * 16 - 4
    l2 = torch.rand((B, H, S), generator=g, dtype=F64) * 16 - 4
    out, lse = fn(o1, l1, o2, l2)
    eo, el = _combine_independent(o1, l1, o2, l2, base)
    assert torch.allclose(out, eo, rtol=1e-12, atol=1e-13)
    assert torch.allclose(lse, el, rtol=1e-12, atol=1e-13)


def test_combine_two_halves_equals_full():
    """Reference property 1 (tests/test_online_softmax_combine_log2.py:44-65), shapes and seed kept."""
    B, S, H, DQ, DV = 1, 256, 16, 192, 128
    scale = DQ**-0.5
    torch.manual_seed(123)
    q = torch.randn(B, S // 2, H, DQ, dtype=torch.bfloat16)
    k1, v1 = torch.randn(B, S // 2, H, DQ, dtype=torch.bfloat16), torch.randn(B, S // 2, H, DV, dtype=torch.bfloat16)
    k2, v2 = torch.randn(B, S // 2, H, DQ, dtype=torch.bfloat16), torch.randn(B, S // 2, H, DV, dtype=torch.bfloat16)
    o1, l1 = R.chunk_fwd(q, k1, v1, scale, False)
    o2, l2 = R.chunk_fwd(q, k2, v2, scale, False)
    out, lse = R.combine_log2(o1, l1, o2, l2)
    full, full_lse = R.chunk_fwd(q, torch.cat([k1, k2], 1), torch.cat([v1, v2], 1), scale, False)
    assert torch.allclose(out, full, rtol=1e-10, atol=1e-12)
    assert torch.allclose(lse, full_lse, rtol=1e-12, atol=1e-12)


def test_combine_identity_and_initial_state():
    """Reference property 2 (:68-84) and the ring's initial state (ring_attention/mla.py:49-52)."""
    o, l = _rand((1, 128, 16, 128), 7), _rand((1, 16, 128), 8) * 5
    zeros = torch.zeros_like(o)
    for empty in (float("-inf"), torch.finfo(torch.float32).min):
        e = torch.full_like(l, empty)
        out, lse = R.combine_log2(o, l, zeros, e)
        assert torch.equal(out, o) and torch.equal(lse, l)
        out, lse = R.combine_log2(zeros, e, o, l)
        assert torch.equal(out, o) and torch.equal(lse, l)


def test_combine_commutes():
    """Reference property 3 (:87-106)."""
    o1, o2 = _rand((1, 128, 16, 128), 99), _rand((1, 128, 16, 128), 100)
    l1, l2 = _rand((1, 16, 128), 101) * 4, _rand((1, 16, 128), 102) * 4
    ab, lab = R.combine_log2(o1, l1, o2, l2)
    ba, lba = R.combine_log2(o2, l2, o1, l1)
    assert torch.allclose(ab, ba, rtol=0, atol=1e-14) and torch.allclose(lab, lba, rtol=0, atol=1e-14)


def test_combine_promotes_to_fp32_like_the_reference():
    o1 = torch.randn(1, 8, 2, 8).to(torch.bfloat16)
    o2 = torch.randn(1, 8, 2, 8).to(torch.bfloat16)
    l1, l2 = torch.randn(1, 2, 8), torch.randn(1, 2, 8)
    out, lse = R.combine_log2(o1, l1, o2, l2)
    assert out.dtype == torch.float32 and lse.dtype == torch.float32 and out.is_contiguous()


# ---------------------------------------------------------------------------------------------
# ring: exact decomposition of full-sequence causal attention


RING_CASES = [  # B, S, Hq, Hkv, Dqk, Dv, C  — reference ring test shapes scaled down, both families
    (1, 64, 4, 4, 16, 16, 2),
    (2, 96, 8, 2, 16, 16, 3),
    (1, 128, 4, 4, 24, 16, 4),
]


@pytest.mark.parametrize("layout", ["contiguous", "zigzag"])
@pytest.mark.parametrize("B,S,Hq,Hkv,Dqk,Dv,C", RING_CASES)
def test_ring_equals_full_sequence(layout, B, S, Hq, Hkv, Dqk, Dv, C):
    q, k, v = _qkv(B, S, S, Hq, Hkv, Dqk, Dv, seed=42)
    dout = _rand((B, S, Hq, Dv), 43)
    scale = Dqk**-0.5
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
    full = _dense_attention(qa, ka, va, scale, True)
    full.backward(dout)
    _, full_lse = R.chunk_fwd(q, k, v, scale, True)

    split = R.zigzag_split if layout == "zigzag" else R.contiguous_split
    qs, ks, vs, dos = split(q, C), split(k, C), split(v, C), split(dout, C)
    dk_sum = [torch.zeros_like(c) for c in ks]
    dv_sum = [torch.zeros_like(c) for c in vs]
    for r in range(C):
        pos = R.token_positions(r, C, S // C, layout)
        out, lse = R.ring_forward(qs[r], ks, vs, scale, r, C, layout)
        assert torch.allclose(out, full.detach()[:, pos], rtol=1e-9, atol=1e-11)
        assert torch.allclose(lse, full_lse[:, :, pos], rtol=1e-11, atol=1e-11)
        dq, dks, dvs = R.ring_backward(dos[r], qs[r], out, lse, ks, vs, scale, r, C, layout)
        assert torch.allclose(dq, qa.grad[:, pos], rtol=1e-8, atol=1e-11)
        for j in range(C):
            if dks[j] is not None:
                dk_sum[j] += dks[j]
                dv_sum[j] += dvs[j]
            elif layout == "zigzag":
                raise AssertionError("zigzag visits every chunk")
    for j in range(C):
        pos = R.token_positions(j, C, S // C, layout)
        assert torch.allclose(dk_sum[j], ka.grad[:, pos], rtol=1e-8, atol=1e-11)
        assert torch.allclose(dv_sum[j], va.grad[:, pos], rtol=1e-8, atol=1e-11)


def test_zigzag_work_is_balanced_and_contiguous_is_not():
    C, S = 4, 64
    for layout, balanced in (("zigzag", True), ("contiguous", False)):
        work = []
        for r in range(C):
            w = 0
            for _, causal, (a, b), (n0, n1) in R._steps(r, C, S, layout):
                w += (b - a) * (n1 - n0) // (2 if causal else 1)
            work.append(w)
        assert (len(set(work)) == 1) == balanced, (layout, work)
        if balanced:
            assert work[0] == C * S * S // 2


def test_cpu_baseline_matches_oracle():
    """The blocked fp32 baseline that bench.py times computes the same ring share."""
    B, S, Hq, Hkv, D, C, r = 1, 64, 4, 2, 16, 4, 1
    q, k, v = _qkv(B, S * C, S * C, Hq, Hkv, D, D, seed=4)
    dout = _rand((B, S * C, Hq, D), 6)
    qs, ks, vs, dos = (R.zigzag_split(t.to(torch.bfloat16), C) for t in (q, k, v, dout))
    scale = D**-0.5
    out, lse = R.ring_forward(qs[r], ks, vs, scale, r, C, "zigzag")
    dq, dks, dvs = R.ring_backward(dos[r], qs[r], out.to(torch.bfloat16), lse, ks, vs, scale, r, C, "zigzag")
    bo, bl, bdq, bdk, bdv = R.cpu_ring_fwd_bwd(qs[r], ks, vs, dos[r], scale, r, C, "zigzag", q_block=24)
    assert torch.allclose(bo.double(), out, rtol=1e-4, atol=1e-5)
    assert torch.allclose(bl.double(), lse, rtol=1e-5, atol=1e-5)
    assert torch.allclose(bdq.double(), dq, rtol=1e-3, atol=1e-4)
    for j in range(C):
        assert torch.allclose(bdk[j].double(), dks[j], rtol=1e-3, atol=1e-4)
        assert torch.allclose(bdv[j].double(), dvs[j], rtol=1e-3, atol=1e-4)
    # a head sub-range (whole kv groups) reproduces the matching slice
    ho, hl, hdq, _, _ = R.cpu_ring_fwd_bwd(qs[r], ks, vs, dos[r], scale, r, C, "zigzag", heads=(2, 4), q_block=64)
    assert torch.allclose(ho, bo[:, :, 2:4], rtol=1e-5, atol=1e-6)
    assert torch.allclose(hdq, bdq[:, :, 2:4], rtol=1e-4, atol=1e-5)
