"""Pins oracle/prologue_oracle.py (q/k RMSNorm + rotary embedding) on the CPU against library
routines and what the mathematics fixes; no test here restates the oracle's own formula."""

import math

import pytest
import torch

from oracle import prologue_oracle as P

torch.manual_seed(0)
F64 = torch.float64


def _angles(b, s, d, seed=0):
    g = torch.Generator().manual_seed(seed)
    theta = torch.rand(b, s, d // 2, generator=g, dtype=F64) * 2 * math.pi
    full = torch.cat((theta, theta), -1)
    return theta, full.cos(), full.sin()


def test_rms_norm_against_library_routine():
    x = torch.randn(2, 5, 3, 64, dtype=F64)
    w = torch.randn(64, dtype=F64)
    for eps in (0.0, 1e-6, 0.3):
        want = torch.nn.functional.rms_norm(x, (64,), w, eps)
        assert torch.allclose(P.rms_norm(x, w, eps), want, rtol=1e-13, atol=1e-13)


def test_rms_norm_invariants():
    x = torch.randn(3, 4, 2, 32, dtype=F64)
    y = P.rms_norm(x, None, 0.0)
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(3, 4, 2, dtype=F64), atol=1e-13)
    assert torch.allclose(P.rms_norm(7.5 * x, None, 0.0), y, atol=1e-13)  # scale invariance
    assert torch.allclose(P.rms_norm(-x, None, 0.0), -y, atol=1e-13)


def test_rope_is_complex_multiplication():
    b, s, h, d = 2, 7, 3, 16
    x = torch.randn(b, s, h, d, dtype=F64)
    theta, cos, sin = _angles(b, s, d)
    z = torch.complex(x[..., : d // 2], x[..., d // 2 :]) * torch.polar(torch.ones_like(theta), theta).unsqueeze(2)
    want = torch.cat((z.real, z.imag), -1)
    assert torch.allclose(P.rope(x, cos, sin), want, atol=1e-13)


def test_rope_invariants():
    b, s, h, d = 1, 6, 2, 8
    x = torch.randn(b, s, h, d, dtype=F64)
    theta, cos, sin = _angles(b, s, d, seed=1)
    y = P.rope(x, cos, sin)
    pair = lambda t: t[..., : d // 2] ** 2 + t[..., d // 2 :] ** 2  # noqa: E731
    assert torch.allclose(pair(y), pair(x), atol=1e-13)  # each pair keeps its length
    assert torch.equal(P.rope(x, torch.ones(b, s, d, dtype=F64), torch.zeros(b, s, d, dtype=F64)), x)
    assert torch.allclose(P.rope(y, cos, -sin), x, atol=1e-13)  # rotate back
    # quarter turn: (lo, hi) -> (-hi, lo)
    q = P.rope(x, torch.zeros(b, s, d, dtype=F64), torch.ones(b, s, d, dtype=F64))
    assert torch.equal(q, torch.cat((-x[..., d // 2 :], x[..., : d // 2]), -1))


def test_rope_scores_depend_on_relative_position_only():
    d = 32
    q = torch.randn(1, 1, 1, d, dtype=F64)
    k = torch.randn(1, 1, 1, d, dtype=F64)

    def score(m, n):
        cm, sm = P.cos_sin_table(torch.tensor([[m]]), d)
        cn, sn = P.cos_sin_table(torch.tensor([[n]]), d)
        return (P.rope(q, cm, sm) * P.rope(k, cn, sn)).sum().item()

    assert abs(score(5, 3) - score(105, 103)) < 1e-9
    assert abs(score(17, 0) - score(40, 23)) < 1e-9
    assert abs(score(5, 3) - score(6, 3)) > 1e-6  # and it does depend on the difference


def test_cos_sin_table_known_values():
    cos, sin = P.cos_sin_table(torch.tensor([0, 1, 2]), 4, base=10000.0)
    assert torch.equal(cos[0], torch.ones(4, dtype=F64)) and torch.equal(sin[0], torch.zeros(4, dtype=F64))
    # inv_freq = [1, 1/100]
    want = torch.tensor([math.cos(2.0), math.cos(0.02), math.cos(2.0), math.cos(0.02)], dtype=F64)
    assert torch.allclose(cos[2], want, atol=1e-15)
    assert torch.allclose(sin[1], torch.tensor([math.sin(1.0), math.sin(0.01)] * 2, dtype=F64), atol=1e-15)


def _library_forward(x, w, theta, eps):
    """Independent forward: library rms_norm, rotation in complex arithmetic."""
    d = x.shape[-1]
    y = x if w is None else torch.nn.functional.rms_norm(x, (d,), w, eps)
    z = torch.complex(y[..., : d // 2], y[..., d // 2 :]) * torch.polar(torch.ones_like(theta), theta).unsqueeze(2)
    return torch.cat((z.real, z.imag), -1)


@pytest.mark.parametrize("with_weight", [True, False])
def test_backward_against_autograd_of_an_independent_forward(with_weight):
    b, s, h, d = 2, 5, 3, 16
    x = torch.randn(b, s, h, d, dtype=F64, requires_grad=True)
    w = torch.randn(d, dtype=F64, requires_grad=True) if with_weight else None
    theta, cos, sin = _angles(b, s, d, seed=2)
    dout = torch.randn(b, s, h, d, dtype=F64)
    eps = 1e-3
    out = _library_forward(x, w, theta, eps)
    assert torch.allclose(P.norm_rope_fwd(x.detach(), None if w is None else w.detach(), cos, sin, eps), out.detach(), atol=1e-13)
    out.backward(dout)
    dx, dw = P.norm_rope_bwd(x.detach(), None if w is None else w.detach(), cos, sin, dout, eps)
    assert torch.allclose(dx, x.grad, atol=1e-12)
    if with_weight:
        assert torch.allclose(dw, w.grad, atol=1e-12)
    else:
        assert dw is None


def test_backward_against_finite_differences():
    b, s, h, d = 1, 3, 2, 8
    x = torch.randn(b, s, h, d, dtype=F64)
    w = torch.randn(d, dtype=F64)
    # cos/sin that are NOT a rotation and differ between the halves: the gradient must not rely on either
    cos = torch.randn(b, s, d, dtype=F64)
    sin = torch.randn(b, s, d, dtype=F64)
    dout = torch.randn(b, s, h, d, dtype=F64)
    eps = 1e-2
    dx, dw = P.norm_rope_bwd(x, w, cos, sin, dout, eps)
    f = lambda xx, ww: (P.norm_rope_fwd(xx, ww, cos, sin, eps) * dout).sum().item()  # noqa: E731
    hstep = 1e-6
    for idx in [(0, 0, 0, 0), (0, 1, 1, 3), (0, 2, 0, 7), (0, 2, 1, 4)]:
        xp, xm = x.clone(), x.clone()
        xp[idx] += hstep
        xm[idx] -= hstep
        assert abs((f(xp, w) - f(xm, w)) / (2 * hstep) - dx[idx].item()) < 1e-6
    for j in range(d):
        wp, wm = w.clone(), w.clone()
        wp[j] += hstep
        wm[j] -= hstep
        assert abs((f(x, wp) - f(x, wm)) / (2 * hstep) - dw[j].item()) < 1e-6


def test_eager_bf16_composite_is_close_to_the_oracle():
    """The reference's own evaluation order (nn.RMSNorm, then the bf16 expression of
    qwen3_30b_a3b.py:132-136, run here on the CPU) stays within bf16 rounding of the oracle."""
    b, s, h, d = 1, 16, 4, 128
    x = torch.randn(b, s, h, d).bfloat16()
    norm = torch.nn.RMSNorm(d, eps=1e-6).bfloat16()
    with torch.no_grad():
        norm.weight.copy_(torch.rand(d) + 0.5)
    cos, sin = P.cos_sin_table(torch.arange(s).unsqueeze(0) + 1000, d, dtype=torch.bfloat16)
    with torch.no_grad():
        y = norm(x)
        c, sn = cos.unsqueeze(2), sin.unsqueeze(2)
        half = d // 2
        eager = (y * c) + (torch.cat((-y[..., half:], y[..., :half]), dim=-1) * sn)
    want = P.norm_rope_fwd(x, norm.weight.detach(), cos, sin, 1e-6)
    err = (eager.double() - want).abs().max().item() / want.abs().max().item()
    assert err < 2e-2


# ---------------------------------------------------------------------------------------------
# MLA layer assembly


def _mla_inputs(b, s, h, dn, dr, dv, seed=0, dtype=F64):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(b, s, h, dn + dr, generator=g, dtype=dtype)
    kv = torch.randn(b, s, h, dn + dv, generator=g, dtype=dtype)
    k_pe = torch.randn(b, s, dr, generator=g, dtype=dtype)
    theta = torch.rand(64, dr // 2, generator=g, dtype=dtype) * 2 * math.pi  # table of 64 positions
    pos = torch.randint(0, 64, (b, s), generator=g)
    return q, kv, k_pe, theta, pos


def _independent_mla_forward(q, kv, k_pe, theta, pos, dn):
    """Index-based de-interleave, rotation in complex arithmetic, slice assignment as in the reference."""
    b, s, h, _ = q.shape
    dr = k_pe.shape[-1]
    phase = torch.polar(torch.ones_like(theta), theta)[pos]  # [B,S,dr/2]

    def rot(pe):  # [..., dr] interleaved pairs
        z = torch.complex(pe[..., 0::2], pe[..., 1::2]) * (phase if pe.dim() == 3 else phase.unsqueeze(2))
        return torch.cat((z.real, z.imag), -1)

    query = torch.zeros(b, s, h, dn + dr, dtype=q.dtype)
    query[..., :dn] = q[..., :dn]
    query[..., dn:] = rot(q[..., dn:])
    key = torch.zeros(b, s, h, dn + dr, dtype=q.dtype)
    key[..., :dn] = kv[..., :dn]
    key[..., dn:] = rot(k_pe).unsqueeze(2)
    return query, key, kv[..., dn:]


def test_mla_assemble_forward_against_complex_rotation():
    dn, dr, dv = 16, 8, 24
    q, kv, k_pe, theta, pos = _mla_inputs(2, 5, 3, dn, dr, dv)
    full = torch.cat((theta, theta), -1)
    got = P.mla_assemble_fwd(q, kv, k_pe, full.cos(), full.sin(), pos, dn)
    want = _independent_mla_forward(q, kv, k_pe, theta, pos, dn)
    for g_, w_ in zip(got, want):
        assert torch.allclose(g_, w_, atol=1e-13)
    assert torch.equal(got[0][..., :dn], q[..., :dn]) and torch.equal(got[2], kv[..., dn:])
    assert torch.equal(got[1][:, :, 0, dn:], got[1][:, :, 2, dn:])  # the rope part is shared by the heads
    # positions default to 0..S-1
    a = P.mla_assemble_fwd(q, kv, k_pe, full.cos(), full.sin(), None, dn)
    bb = P.mla_assemble_fwd(q, kv, k_pe, full.cos(), full.sin(), torch.arange(5).expand(2, 5), dn)
    assert all(torch.equal(x, y) for x, y in zip(a, bb))


def test_deinterleave_known_values():
    x = torch.arange(8.0).unsqueeze(0)
    assert P.deinterleave(x).tolist() == [[0, 2, 4, 6, 1, 3, 5, 7]]
    assert torch.equal(P._interleave(P.deinterleave(x)), x)


def test_mla_assemble_backward_against_autograd_of_an_independent_forward():
    dn, dr, dv = 8, 8, 16
    q, kv, k_pe, theta, pos = _mla_inputs(2, 4, 3, dn, dr, dv, seed=4)
    q.requires_grad_(), kv.requires_grad_(), k_pe.requires_grad_()
    query, key, value = _independent_mla_forward(q, kv, k_pe, theta, pos, dn)
    g = torch.Generator().manual_seed(5)
    dquery, dkey, dvalue = (torch.randn(t.shape, generator=g, dtype=F64) for t in (query, key, value))
    torch.autograd.backward([query, key, value], [dquery, dkey, dvalue])
    full = torch.cat((theta, theta), -1)
    dq, dkv, dk_pe = P.mla_assemble_bwd(dquery, dkey, dvalue, full.cos(), full.sin(), pos, dn)
    assert torch.allclose(dq, q.grad, atol=1e-12)
    assert torch.allclose(dkv, kv.grad, atol=1e-12)
    assert torch.allclose(dk_pe, k_pe.grad, atol=1e-12)


def test_mla_assemble_backward_with_tables_that_are_not_rotations():
    """cos/sin scaled (YaRN mscale) and different in the two halves: autograd through the oracle's
    own forward, which the previous tests pin, must agree with the closed form."""
    dn, dr, dv = 8, 16, 8
    q, kv, k_pe, _, pos = _mla_inputs(1, 6, 2, dn, dr, dv, seed=6)
    g = torch.Generator().manual_seed(7)
    cos, sin = torch.randn(64, dr, generator=g, dtype=F64), torch.randn(64, dr, generator=g, dtype=F64)
    q.requires_grad_(), kv.requires_grad_(), k_pe.requires_grad_()
    outs = P.mla_assemble_fwd(q, kv, k_pe, cos, sin, pos, dn)
    grads = [torch.randn(t.shape, generator=g, dtype=F64) for t in outs]
    torch.autograd.backward(list(outs), grads)
    dq, dkv, dk_pe = P.mla_assemble_bwd(*grads, cos, sin, pos, dn)
    assert torch.allclose(dq, q.grad, atol=1e-12) and torch.allclose(dkv, kv.grad, atol=1e-12)
    assert torch.allclose(dk_pe, k_pe.grad, atol=1e-12)
