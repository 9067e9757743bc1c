"""HIP chunk attention (forward, delta, dK/dV, dQ) against the fp64 oracle, through the C ABI.

Shapes, seeds and tolerances follow the reference's operator tests
(tests/operators/mla/test_triton_non_causal.py:31-32,70,99-108 and tests/operators/mla/test_triton.py:58,83-85):
H16 192/128 at (B1,S512), (B2,S1024), seed 42, isclose(rtol=1e-2, atol=2e-2) with at most 0.1 %
outliers on gradients; plus the GQA / D=64 / ragged / unequal-length cases the ring needs."""

import pytest
import torch

from helpers import check_bf16_result, check_lse
from oracle import ring_oracle as R
from pithtrain_amd import _C
from pithtrain_amd.operators.mla.hip import (
    MLA,
    _mla_bwd_dk_dv,
    _mla_bwd_dq,
    _mla_bwd_preprocess,
    _mla_fwd,
    attn_bwd_dkdv_into,
    attn_bwd_dq_into,
)

pytestmark = pytest.mark.gpu

CASES = [  # B, Sq, Skv, Hq, Hkv, Dqk, Dv, causal
    pytest.param(1, 512, 512, 16, 16, 192, 128, True, id="mla-b1-s512-causal"),
    pytest.param(1, 512, 512, 16, 16, 192, 128, False, id="mla-b1-s512"),
    pytest.param(2, 1024, 1024, 16, 16, 192, 128, True, id="mla-b2-s1024-causal"),
    pytest.param(2, 1024, 1024, 16, 16, 192, 128, False, id="mla-b2-s1024"),
    pytest.param(1, 512, 512, 12, 4, 128, 128, True, id="gqa-12/4-d128-causal"),
    pytest.param(2, 256, 256, 8, 2, 64, 64, True, id="gqa-8/2-d64-causal"),
    pytest.param(1, 128, 128, 4, 4, 64, 64, False, id="mha-d64"),
    pytest.param(1, 1024, 512, 8, 1, 128, 128, False, id="gqa-8/1-sq1024-skv512"),
    pytest.param(1, 256, 768, 4, 2, 128, 128, False, id="gqa-sq256-skv768"),
    pytest.param(1, 333, 333, 4, 2, 128, 128, True, id="ragged-333-causal"),
    pytest.param(2, 100, 333, 4, 2, 128, 128, False, id="ragged-100x333"),
    pytest.param(1, 77, 77, 2, 2, 192, 128, True, id="ragged-mla-77-causal"),
    pytest.param(1, 1, 1, 1, 1, 64, 64, True, id="single-token"),
    pytest.param(1, 2048, 2048, 4, 1, 128, 128, True, id="gqa-4/1-s2048-causal"),
    # edges of the pipelined 128-dim kernels: one / two / three tiles, tile boundaries +- 1
    pytest.param(1, 1, 1, 1, 1, 128, 128, True, id="d128-single-token"),
    pytest.param(1, 64, 64, 2, 2, 128, 128, True, id="d128-one-tile-causal"),
    pytest.param(1, 65, 65, 2, 1, 128, 128, True, id="d128-65-causal"),
    pytest.param(1, 129, 64, 2, 2, 128, 128, False, id="d128-sq129-skv64"),
    pytest.param(1, 64, 129, 4, 4, 128, 128, False, id="d128-sq64-skv129"),
    pytest.param(1, 193, 193, 8, 1, 128, 128, True, id="d128-193-causal-gqa8"),
    pytest.param(2, 320, 448, 8, 2, 128, 128, False, id="d128-b2-320x448"),
    pytest.param(1, 640, 640, 2, 2, 128, 128, True, id="d128-640-causal"),
    # enough workgroups for the 8-wavefront variants of the general kernels (shorter query ranges
    # take the 4-wavefront ones): ceil(Sq/256) * Hq * B >= 192
    pytest.param(1, 1024, 1024, 48, 48, 192, 128, True, id="mla-h48-s1024-causal-8waves"),
    pytest.param(1, 1000, 300, 48, 16, 192, 128, False, id="mla-h48-1000x300-8waves"),
    pytest.param(2, 1536, 1536, 16, 4, 64, 64, True, id="d64-b2-s1536-causal-8waves"),
]


def _inputs(B, Sq, Skv, Hq, Hkv, Dqk, Dv, seed=42):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Sq, Hq, Dqk, generator=g).to(torch.bfloat16)
    k = torch.randn(B, Skv, Hkv, Dqk, generator=g).to(torch.bfloat16)
    v = torch.randn(B, Skv, Hkv, Dv, generator=g).to(torch.bfloat16)
    dout = torch.randn(B, Sq, Hq, Dv, generator=g).to(torch.bfloat16)
    return q, k, v, dout


@pytest.mark.parametrize("B,Sq,Skv,Hq,Hkv,Dqk,Dv,causal", CASES)
def test_forward_and_backward_match_oracle(gpu, B, Sq, Skv, Hq, Hkv, Dqk, Dv, causal):
    q, k, v, dout = _inputs(B, Sq, Skv, Hq, Hkv, Dqk, Dv)
    scale = Dqk**-0.5
    ref_o, ref_lse = R.chunk_fwd(q, k, v, scale, causal)
    qd, kd, vd, dod = (t.to(gpu) for t in (q, k, v, dout))

    o, lse = _mla_fwd(qd, kd, vd, scale, causal=causal)
    assert o.dtype == torch.bfloat16 and o.shape == (B, Sq, Hq, Dv)
    assert lse.dtype == torch.float32 and lse.shape == (B, Hq, Sq)
    check_bf16_result(o, ref_o, "O")
    check_lse(lse, ref_lse, "LSE2")

    # backward against the kernel's own O/LSE (what a caller has), compared with exact gradients
    delta = _mla_bwd_preprocess(o, dod)
    ref_delta = R.bwd_delta(o.cpu(), dout)
    assert (delta.double().cpu() - ref_delta).abs().max() < 1e-4 * max(1.0, ref_delta.abs().max().item())
    ref_dq, ref_dk, ref_dv = R.chunk_bwd(q, k, v, dout, ref_lse, R.bwd_delta(ref_o, dout), scale, causal)
    dk, dv = _mla_bwd_dk_dv(qd, kd, vd, dod, lse, delta, scale, causal=causal)
    dq = _mla_bwd_dq(qd, kd, vd, dod, lse, delta, scale, causal=causal)
    assert dq.dtype == dk.dtype == dv.dtype == torch.bfloat16
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape
    check_bf16_result(dq, ref_dq, "dQ", otol=1e-3)
    check_bf16_result(dk, ref_dk, "dK", otol=1e-3)
    check_bf16_result(dv, ref_dv, "dV", otol=1e-3)


def test_baseline_input_scaling(gpu):
    """The benchmark inputs are N(0,1)/sqrt(D): outputs are small, so the normalised error is what bites."""
    B, S, Hq, Hkv, D = 1, 1024, 8, 1, 128
    q, k, v, dout = _inputs(B, S, S, Hq, Hkv, D, D, seed=1)
    q, k, v = ((t.float() * D**-0.5).to(torch.bfloat16) for t in (q, k, v))
    scale = D**-0.5
    ref_o, ref_lse = R.chunk_fwd(q, k, v, scale, True)
    o, lse = _mla_fwd(q.to(gpu), k.to(gpu), v.to(gpu), scale, causal=True)
    check_bf16_result(o, ref_o, "O (scaled inputs)")
    check_lse(lse, ref_lse, "LSE2 (scaled inputs)")


def test_sliced_arguments_and_fp32_accumulation(gpu):
    """Row ranges of larger tensors are used in place (zigzag half-chunk steps) and the fp32
    accumulate mode adds to what the output already holds."""
    B, S, Hq, Hkv, D = 2, 256, 4, 2, 128
    q, k, v, dout = _inputs(B, S, S, Hq, Hkv, D, D, seed=3)
    scale = D**-0.5
    half = S // 2
    qd, kd, vd, dod = (t.to(gpu) for t in (q, k, v, dout))
    # second half of the queries against the first half of the keys, non-causal
    qs, ks, vs, ds = qd[:, half:], kd[:, :half], vd[:, :half], dod[:, half:]
    o_full = torch.zeros(B, S, Hq, D, dtype=torch.bfloat16, device=gpu)
    lse_full = torch.zeros(B, Hq, S, device=gpu)
    from pithtrain_amd.operators.mla.hip import attn_fwd_into

    attn_fwd_into(qs, ks, vs, o_full[:, half:], lse_full[:, :, half:], scale, False)
    ref_o, ref_lse = R.chunk_fwd(q[:, half:], k[:, :half], v[:, :half], scale, False)
    check_bf16_result(o_full[:, half:], ref_o, "sliced O")
    check_lse(lse_full[:, :, half:], ref_lse, "sliced LSE2")
    assert not o_full[:, :half].any() and not lse_full[:, :, :half].any(), "rows outside the slice were written"

    delta_full = torch.zeros(B, Hq, S, device=gpu)
    from pithtrain_amd.operators.mla.hip import attn_bwd_delta_into

    attn_bwd_delta_into(o_full[:, half:], ds, delta_full[:, :, half:])
    ref_dq, ref_dk, ref_dv = R.chunk_bwd(q[:, half:], k[:, :half], v[:, :half], dout[:, half:], ref_lse,
                                         R.bwd_delta(ref_o, dout[:, half:]), scale, False)  # fmt: skip
    dq_acc = torch.full((B, S, Hq, D), 1.0, dtype=torch.float32, device=gpu)
    attn_bwd_dq_into(qs, ks, vs, ds, lse_full[:, :, half:], delta_full[:, :, half:], dq_acc[:, half:], scale, False,
                     accumulate=True)  # fmt: skip
    assert torch.equal(dq_acc[:, :half], torch.ones_like(dq_acc[:, :half]))
    check_bf16_result(dq_acc[:, half:] - 1.0, ref_dq, "accumulated fp32 dQ", otol=1e-3)
    dk = torch.zeros(B, S, Hkv, D, dtype=torch.float32, device=gpu)
    dv = torch.zeros(B, S, Hkv, D, dtype=torch.float32, device=gpu)
    for _ in range(2):  # accumulate twice -> twice the gradient
        attn_bwd_dkdv_into(qs, ks, vs, ds, lse_full[:, :, half:], delta_full[:, :, half:], dk[:, :half], dv[:, :half],
                           scale, False, accumulate=True)  # fmt: skip
    assert not dk[:, half:].any() and not dv[:, half:].any()
    check_bf16_result(dk[:, :half] / 2, ref_dk, "accumulated fp32 dK", otol=1e-3)
    check_bf16_result(dv[:, :half] / 2, ref_dv, "accumulated fp32 dV", otol=1e-3)


def test_mla_module_autograd(gpu):
    """MLA(h, dq, dv, scale).forward + autograd, as tests/operators/mla/test_triton.py drives it."""
    B, S, H, DQ, DV = 1, 384, 4, 192, 128
    q, k, v, dout = _inputs(B, S, S, H, H, DQ, DV, seed=42)
    scale = DQ**-0.5
    MLA.autotune(B, S, H, DQ, DV, scale, include_non_causal=True)
    qd, kd, vd = (t.to(gpu).requires_grad_(True) for t in (q, k, v))
    out = MLA(H, DQ, DV, scale).to(gpu)(qd, kd, vd)
    out.backward(dout.to(gpu))
    ref_o, ref_lse = R.chunk_fwd(q, k, v, scale, True)
    ref_dq, ref_dk, ref_dv = R.chunk_bwd(q, k, v, dout, ref_lse, R.bwd_delta(ref_o, dout), scale, True)
    check_bf16_result(out, ref_o, "MLA O")
    check_bf16_result(qd.grad, ref_dq, "MLA dQ", otol=1e-3)
    check_bf16_result(kd.grad, ref_dk, "MLA dK", otol=1e-3)
    check_bf16_result(vd.grad, ref_dv, "MLA dV", otol=1e-3)


def test_error_paths(gpu):
    z = lambda *s: torch.zeros(*s, dtype=torch.bfloat16, device=gpu)  # noqa: E731
    with pytest.raises(AssertionError, match="support"):
        _mla_fwd(z(1, 64, 2, 96), z(1, 64, 2, 96), z(1, 64, 2, 96), 0.1)
    with pytest.raises(AssertionError, match="causal"):
        _mla_fwd(z(1, 64, 2, 128), z(1, 32, 2, 128), z(1, 32, 2, 128), 0.1, causal=True)
    with pytest.raises(AssertionError, match="not contiguous"):
        _mla_fwd(z(1, 64, 4, 128)[:, :, ::2], z(1, 64, 2, 128), z(1, 64, 2, 128), 0.1)
    with pytest.raises(AssertionError, match="multiple"):
        _mla_fwd(z(1, 64, 3, 128), z(1, 64, 2, 128), z(1, 64, 2, 128), 0.1)
    with pytest.raises(AssertionError, match="bfloat16"):
        _mla_fwd(z(1, 64, 2, 128).float(), z(1, 64, 2, 128), z(1, 64, 2, 128), 0.1)
    assert _C.lib().pith_last_error() is not None


def _random_cases(n, seed):
    """Seeded sweep over shapes no hand-picked case covers: odd lengths around and far from tile
    boundaries, every head-dim family, group sizes 1..8, one or two batch elements."""
    import random

    rng = random.Random(seed)
    cases = []
    for i in range(n):
        dqk, dv = rng.choice([(128, 128), (128, 128), (192, 128), (64, 64)])
        causal = rng.random() < 0.5
        sq = rng.choice([rng.randint(1, 70), rng.randint(60, 270), rng.randint(250, 600)])
        skv = sq if causal else rng.choice([rng.randint(1, 70), rng.randint(60, 270), rng.randint(250, 600)])
        hkv = rng.choice([1, 2, 3])
        group = rng.choice([1, 2, 4, 8])
        b = rng.choice([1, 1, 2])
        cases.append(pytest.param(b, sq, skv, hkv * group, hkv, dqk, dv, causal, 1000 + i,
                                  id=f"rand{i}-b{b}-{sq}x{skv}-h{hkv * group}/{hkv}-d{dqk}-{'c' if causal else 'n'}"))  # fmt: skip
    return cases


@pytest.mark.parametrize("B,Sq,Skv,Hq,Hkv,Dqk,Dv,causal,seed", _random_cases(36, seed=2024))
def test_random_shapes_match_oracle(gpu, B, Sq, Skv, Hq, Hkv, Dqk, Dv, causal, seed):
    q, k, v, dout = _inputs(B, Sq, Skv, Hq, Hkv, Dqk, Dv, seed=seed)
    scale = Dqk**-0.5
    ref_o, ref_lse = R.chunk_fwd(q, k, v, scale, causal)
    ref_dq, ref_dk, ref_dv = R.chunk_bwd(q, k, v, dout, ref_lse, R.bwd_delta(ref_o, dout), scale, causal)
    qd, kd, vd, dod = (t.to(gpu) for t in (q, k, v, dout))
    o, lse = _mla_fwd(qd, kd, vd, scale, causal=causal)
    delta = _mla_bwd_preprocess(o, dod)
    dk, dv = _mla_bwd_dk_dv(qd, kd, vd, dod, lse, delta, scale, causal=causal)
    dq = _mla_bwd_dq(qd, kd, vd, dod, lse, delta, scale, causal=causal)
    check_bf16_result(o, ref_o, "O")
    check_lse(lse, ref_lse, "LSE2")
    # gradients sum hundreds of bf16-rounded terms: elements much smaller than their row's scale may
    # miss isclose; allow 0.2 % of them (at least 8 elements of a tiny tensor). The normalised
    # max-abs and cosine bounds inside check_bf16_result apply to every element.
    for name, got, want in (("dQ", dq, ref_dq), ("dK", dk, ref_dk), ("dV", dv, ref_dv)):
        check_bf16_result(got, want, name, otol=max(2e-3, 8.0 / want.numel()))


@pytest.mark.parametrize("causal", [True, False])
def test_error_is_within_twice_an_eager_bf16_restatement(gpu, causal):
    """Inputs at the benchmark scale (N(0,1)/sqrt(D)): the normalised max-abs error of every result
    against the fp64 oracle is at most twice that of the reference's numerics restated with eager
    torch ops on the same GPU (fp32 scores from bf16 operands, P and dS rounded to bf16 before
    the second product, bf16 results)."""
    from helpers import norm_max_err

    B, S, Hq, Hkv, D = 1, 1024, 8, 2, 128
    q, k, v, dout = _inputs(B, S, S, Hq, Hkv, D, D, seed=77)
    q, k, v = ((t.float() * D**-0.5).to(torch.bfloat16) for t in (q, k, v))
    scale = D**-0.5
    ref_o, ref_lse = R.chunk_fwd(q, k, v, scale, causal)
    ref_dq, ref_dk, ref_dv = R.chunk_bwd(q, k, v, dout, ref_lse, R.bwd_delta(ref_o, dout), scale, causal)

    qd, kd, vd, dod = (t.to(gpu) for t in (q, k, v, dout))
    o, lse = _mla_fwd(qd, kd, vd, scale, causal=causal)
    delta = _mla_bwd_preprocess(o, dod)
    dk, dv = _mla_bwd_dk_dv(qd, kd, vd, dod, lse, delta, scale, causal=causal)
    dq = _mla_bwd_dq(qd, kd, vd, dod, lse, delta, scale, causal=causal)

    # eager restatement, heads first: [B, H, S, D]
    g = Hq // Hkv
    qe, doe = qd.transpose(1, 2).float(), dod.transpose(1, 2).float()
    ke = kd.transpose(1, 2).repeat_interleave(g, dim=1).float()
    ve = vd.transpose(1, 2).repeat_interleave(g, dim=1).float()
    s = (qe @ ke.transpose(-1, -2)) * scale
    if causal:
        s = s.masked_fill(torch.ones(S, S, dtype=torch.bool, device=gpu).triu(1), float("-inf"))
    p = torch.softmax(s, dim=-1)
    p16 = p.to(torch.bfloat16).float()
    oe = (p16 @ ve).to(torch.bfloat16)
    de = (oe.float() * doe).sum(-1, keepdim=True)
    dve = (p16.transpose(-1, -2) @ doe).to(torch.bfloat16)
    ds16 = (p * (doe @ ve.transpose(-1, -2) - de) * scale).to(torch.bfloat16).float()
    dqe = (ds16 @ ke).to(torch.bfloat16)
    dke = (ds16.transpose(-1, -2) @ qe).to(torch.bfloat16)
    fold = lambda t: t.float().view(B, Hkv, g, S, D).sum(2).to(torch.bfloat16).transpose(1, 2)  # noqa: E731
    eager = {"O": oe.transpose(1, 2), "dQ": dqe.transpose(1, 2), "dK": fold(dke), "dV": fold(dve)}
    ours = {"O": o, "dQ": dq, "dK": dk, "dV": dv}
    want = {"O": ref_o, "dQ": ref_dq, "dK": ref_dk, "dV": ref_dv}
    for name in ours:
        e_ours, e_eager = norm_max_err(ours[name], want[name]), norm_max_err(eager[name], want[name])
        assert e_ours <= 2 * e_eager + 1e-4, f"{name}: error {e_ours:.3e} against {e_eager:.3e} of the eager restatement"


@pytest.mark.parametrize("Dqk,Hq,Hkv,Sq,causal", [
    (128, 8, 2, 512, False), (128, 8, 2, 512, True), (128, 32, 4, 2048, False),  # 128-row and 256-row workgroups
    (192, 4, 4, 384, True), (192, 48, 48, 1024, False), (64, 4, 2, 320, True),
])  # fmt: skip
@pytest.mark.parametrize("ramp", ["climbing", "huge-jump", "falling"])
def test_forward_when_the_running_maximum_moves(gpu, Dqk, Hq, Hkv, Sq, causal, ramp):
    """The forward refreshes its running row maximum lazily (a stale maximum is kept while no P value exceeds 2^8).
    Scores that climb from key tile to key tile, that jump by far more than fp32's exponent range allows
    exp2(kappa * (s - m_stale)) to hold, or that fall (first tile dominates, everything after underflows) must
    give the same O and LSE2 as the oracle."""
    Dv = min(Dqk, 128)
    q, k, v, _ = _inputs(1, Sq, Sq, Hq, Hkv, Dqk, Dv, seed=17)
    # keys along a direction every query has a positive component on, growing (or shrinking) with the position
    direction = torch.zeros(Dqk)
    direction[0] = 1.0
    q = q.float()
    q[..., 0] = q[..., 0].abs() + 1.0
    pos = torch.arange(Sq, dtype=torch.float32) / Sq
    gain = {"climbing": 60.0 * pos, "huge-jump": 4000.0 * (pos > 0.5).float(), "falling": 300.0 * (1 - pos)}[ramp]
    k = (k.float() + gain[None, :, None, None] * direction).to(torch.bfloat16)
    q = q.to(torch.bfloat16)
    scale = Dqk**-0.5
    ref_o, ref_lse = R.chunk_fwd(q, k, v, scale, causal)
    o, lse = _mla_fwd(q.to(gpu), k.to(gpu), v.to(gpu), scale, causal=causal)
    check_bf16_result(o, ref_o, f"O ({ramp})")
    # LSE2 is large here (up to thousands): 1e-3 absolute is below fp32 resolution of such values, so the bound is
    # relative to the magnitude for them
    err = (lse.double().cpu() - ref_lse).abs()
    assert (err <= 1e-3 + 2e-7 * ref_lse.abs()).all(), f"LSE2 ({ramp}): max error {err.max().item():.3e}"
