"""HIP prologue of the MLA layer (rotary embedding of the rope parts + assembly of query / key /
value states) against the fp64 oracle, through the C-ABI library. Copied parts must be
bit-identical; rotated parts are one bf16 rounding of the exact result."""

import pytest
import torch

from helpers import assert_close
from oracle import prologue_oracle as P

pytestmark = pytest.mark.gpu

RTOL = 2.0**-8
BF = torch.bfloat16


def _inputs(b, s, h, dn, dr, dv, seed, positions=64, wide_kpe=True):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(b, s, h, dn + dr, generator=g).to(BF)
    kv = torch.randn(b, s, h, dn + dv, generator=g).to(BF)
    # k_pe is a column slice of a wider projection (kv_lora_rank + dr columns), as in the layer
    lora = 32 if wide_kpe else 0
    a_proj = torch.randn(b, s, lora + dr, generator=g).to(BF)
    pos = torch.randint(0, positions, (b, s), generator=g)
    ang = torch.rand(positions, dr // 2, generator=g) * 6.283
    table = torch.cat((ang, ang), -1)
    cos, sin = (table.cos() * 1.07).to(BF), (table.sin() * 1.07).to(BF)  # YaRN-style magnitude scale
    return q, kv, a_proj, lora, cos, sin, pos


def _check(actual, expected, what):
    assert_close(actual, expected, rtol=RTOL, atol=1e-5 * expected.abs().max().item(), what=what)


CASES = [
    # b, s, h, dn, dr, dv
    (1, 64, 16, 128, 64, 128),  # DeepSeek-V2-Lite
    (2, 37, 16, 128, 64, 128),
    (2, 5, 3, 8, 16, 8),
    (1, 1, 1, 16, 16, 24),
    (1, 9, 40, 64, 32, 64),     # more pieces per token than one pass of the block covers
]


@pytest.mark.parametrize("b,s,h,dn,dr,dv", CASES)
@pytest.mark.parametrize("use_positions", [True, False])
def test_forward_and_backward_match_the_oracle(gpu, b, s, h, dn, dr, dv, use_positions):
    from pithtrain_amd.operators.mla_assemble import mla_assemble_bwd_into, mla_assemble_fwd_into

    q, kv, a_proj, lora, cos, sin, pos = _inputs(b, s, h, dn, dr, dv, seed=s * 7 + h, positions=max(64, s))
    if not use_positions:
        pos = None
    k_pe = a_proj[..., lora:]
    want = P.mla_assemble_fwd(q, kv, k_pe, cos, sin, pos, dn)

    qd, kvd, ad, cd, sd = (t.to(gpu) for t in (q, kv, a_proj, cos, sin))
    pd = None if pos is None else pos.to(gpu)
    outs = [torch.full(w.shape, float("nan"), dtype=BF, device=gpu) for w in want]
    mla_assemble_fwd_into(qd, kvd, ad[..., lora:], cd, sd, pd, *outs)
    for o, w, name in zip(outs, want, ("query", "key", "value")):
        _check(o, w, name)
    assert torch.equal(outs[0][..., :dn].cpu(), q[..., :dn]), "q_nope must be copied bit-exactly"
    assert torch.equal(outs[1][..., :dn].cpu(), kv[..., :dn]), "k_nope must be copied bit-exactly"
    assert torch.equal(outs[2].cpu(), kv[..., dn:]), "value must be copied bit-exactly"
    assert torch.equal(outs[1][:, :, :1, dn:].expand(b, s, h, dr), outs[1][..., dn:]), "rope part differs between heads"

    g = torch.Generator().manual_seed(99)
    grads = [torch.randn(w.shape, generator=g).to(BF) for w in want]
    want_dq, want_dkv, want_dkpe = P.mla_assemble_bwd(*grads, cos, sin, pos, dn)
    dq = torch.full((b, s, h, dn + dr), float("nan"), dtype=BF, device=gpu)
    dkv = torch.full((b, s, h, dn + dv), float("nan"), dtype=BF, device=gpu)
    dkpe = torch.full((b, s, dr), float("nan"), dtype=BF, device=gpu)
    mla_assemble_bwd_into(*(t.to(gpu) for t in grads), cd, sd, pd, dq, dkv, dkpe)
    _check(dq, want_dq, "dq")
    _check(dkpe, want_dkpe, "dk_pe")
    assert torch.equal(dkv.cpu(), want_dkv.to(BF)), "dkv is a pure copy of the nope and value gradients"
    assert torch.equal(dq[..., :dn].cpu(), grads[0][..., :dn])


def test_autograd_with_the_layers_views(gpu):
    """q / kv / k_pe as the layer produces them (k_pe [b, s, 1, dr] sliced from the kv_a projection);
    gradients reach the projections' outputs."""
    from pithtrain_amd.operators.mla_assemble import mla_assemble_qkv

    b, s, h, dn, dr, dv = 2, 48, 16, 128, 64, 128
    q, kv, a_proj, lora, cos, sin, pos = _inputs(b, s, h, dn, dr, dv, seed=5)
    qd = q.to(gpu).requires_grad_()
    kvd = kv.to(gpu).requires_grad_()
    ad = a_proj.to(gpu).requires_grad_()
    k_pe = ad[..., lora:].view(b, s, 1, dr)
    query, key, value = mla_assemble_qkv(qd, kvd, k_pe, cos.to(gpu), sin.to(gpu), pos.to(gpu))
    want = P.mla_assemble_fwd(q, kv, a_proj[..., lora:], cos, sin, pos, dn)
    for o, w, name in zip((query, key, value), want, ("query", "key", "value")):
        _check(o, w, name)
    g = torch.Generator().manual_seed(6)
    grads = [torch.randn(w.shape, generator=g).to(BF) for w in want]
    torch.autograd.backward([query, key, value], [t.to(gpu) for t in grads])
    want_dq, want_dkv, want_dkpe = P.mla_assemble_bwd(*grads, cos, sin, pos, dn)
    _check(qd.grad, want_dq, "dq")
    _check(kvd.grad, want_dkv, "dkv")
    _check(ad.grad[..., lora:], want_dkpe, "dk_pe")
    assert ad.grad[..., :lora].abs().max().item() == 0.0  # the compressed-kv columns get no gradient from here


def test_matches_the_reference_statements_run_eagerly(gpu):
    """The reference's statements (deepseek_v2_lite.py:173-187, 446-454) written with torch ops on
    the GPU in bf16: nope parts identical, rope parts within bf16 rounding of each other."""
    from pithtrain_amd.operators.mla_assemble import mla_assemble_qkv

    b, s, h, dn, dr, dv = 1, 128, 16, 128, 64, 128
    q, kv, a_proj, lora, cos, sin, pos = (t.to(gpu) if torch.is_tensor(t) else t for t in _inputs(b, s, h, dn, dr, dv, seed=8))
    k_pe = a_proj[..., lora:].view(b, s, 1, dr)
    query, key, value = mla_assemble_qkv(q, kv, k_pe, cos, sin, pos)

    c, sn = cos[pos].unsqueeze(2), sin[pos].unsqueeze(2)

    def rot(x):
        bb, ss, hh, d = x.shape
        x = x.view(bb, ss, hh, d // 2, 2).transpose(4, 3).reshape(bb, ss, hh, d)
        return (x * c) + (torch.cat((-x[..., d // 2 :], x[..., : d // 2]), dim=-1) * sn)

    ref_q = torch.empty_like(query)
    ref_q[..., :dn] = q[..., :dn]
    ref_q[..., dn:] = rot(q[..., dn:])
    ref_k = torch.empty_like(key)
    ref_k[..., :dn] = kv[..., :dn]
    ref_k[..., dn:] = rot(k_pe)
    assert torch.equal(query[..., :dn], ref_q[..., :dn]) and torch.equal(key[..., :dn], ref_k[..., :dn])
    assert torch.equal(value, kv[..., dn:])
    assert_close(query[..., dn:], ref_q[..., dn:], rtol=3e-2, atol=3e-2, what="rope(q_pe)")
    assert_close(key[..., dn:], ref_k[..., dn:], rtol=3e-2, atol=3e-2, what="rope(k_pe)")


def test_positions_outside_the_table_are_clamped(gpu):
    from pithtrain_amd.operators.mla_assemble import mla_assemble_qkv

    b, s, h, dn, dr, dv = 1, 8, 2, 16, 16, 16
    q, kv, a_proj, lora, cos, sin, _ = _inputs(b, s, h, dn, dr, dv, seed=9, positions=16)
    pos = torch.tensor([[0, 15, 16, 1000, -1, -7, 3, 2**40]])
    clamped = pos.clamp(0, 15)
    got = mla_assemble_qkv(q.to(gpu), kv.to(gpu), a_proj[..., lora:].to(gpu), cos.to(gpu), sin.to(gpu), pos.to(gpu))
    want = mla_assemble_qkv(q.to(gpu), kv.to(gpu), a_proj[..., lora:].to(gpu), cos.to(gpu), sin.to(gpu), clamped.to(gpu))
    assert all(torch.equal(a, c) for a, c in zip(got, want))


def test_full_size_deepseek_share(gpu):
    """One rank's 4096 tokens of the 16K MLA configuration, every element against the oracle."""
    from pithtrain_amd.operators.mla_assemble import mla_assemble_bwd_into, mla_assemble_fwd_into

    b, s, h, dn, dr, dv = 1, 4096, 16, 128, 64, 128
    q, kv, a_proj, lora, cos, sin, _ = _inputs(b, s, h, dn, dr, dv, seed=12, positions=16384)
    pos = (torch.arange(s) + 8192).unsqueeze(0)
    k_pe = a_proj[..., lora:]
    want = P.mla_assemble_fwd(q, kv, k_pe, cos, sin, pos, dn)
    dev = [t.to(gpu) for t in (q, kv, a_proj, cos, sin, pos)]
    outs = [torch.empty(w.shape, dtype=BF, device=gpu) for w in want]
    mla_assemble_fwd_into(dev[0], dev[1], dev[2][..., lora:], dev[3], dev[4], dev[5], *outs)
    for o, w, name in zip(outs, want, ("query", "key", "value")):
        _check(o, w, name)
    grads = [w.to(BF) for w in want]  # any tensors of the right shapes
    want_grads = P.mla_assemble_bwd(*grads, cos, sin, pos, dn)
    res = [torch.empty(w.shape, dtype=BF, device=gpu) for w in want_grads]
    mla_assemble_bwd_into(*(t.to(gpu) for t in grads), dev[3], dev[4], dev[5], *res)
    for o, w, name in zip(res, want_grads, ("dq", "dkv", "dk_pe")):
        _check(o, w, name)
