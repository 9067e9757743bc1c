"""HIP combine kernel against the oracle (closed form in fp64) and the reference's own three
properties (tests/test_online_softmax_combine_log2.py:44-106 of the reference: shapes, seeds and
tolerances kept), through the C ABI."""

import pytest
import torch

from helpers import assert_close, check_lse
from oracle import ring_oracle as R
from pithtrain_amd import _C
from pithtrain_amd.operators.mla.hip import _mla_fwd
from pithtrain_amd.operators.ring_attention.combine import cast_f32_bf16_into, combine_into
from pithtrain_amd.operators.ring_attention.mla import _online_softmax_combine_log2
from pithtrain_amd.operators.ring_attention.standard import _online_softmax_combine

pytestmark = pytest.mark.gpu


def _partials(B, S, H, D, seed, dt1=torch.bfloat16, dt2=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    o1 = torch.randn(B, S, H, D, generator=g).to(dt1)
    o2 = torch.randn(B, S, H, D, generator=g).to(dt2)
    l1 = torch.rand(B, H, S, generator=g) * 16 - 4
    l2 = torch.rand(B, H, S, generator=g) * 16 - 4
    return o1, l1, o2, l2


@pytest.mark.parametrize("dt1", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("dt2", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("B,S,H,D", [(1, 256, 16, 128), (2, 77, 3, 64), (1, 4096, 32, 128)])
def test_combine_log2_matches_oracle(gpu, dt1, dt2, B, S, H, D):
    o1, l1, o2, l2 = _partials(B, S, H, D, 5, dt1, dt2)
    out, lse = _online_softmax_combine_log2(o1.to(gpu), l1.to(gpu), o2.to(gpu), l2.to(gpu))
    assert out.dtype == torch.float32 and lse.dtype == torch.float32 and out.is_contiguous()
    ro, rl = R.combine_log2(o1.double(), l1.double(), o2.double(), l2.double())
    # fp32 result of fp32 arithmetic on exactly representable inputs: a few ulp
    assert_close(out, ro, rtol=2e-6, atol=2e-6, what="combined out")
    check_lse(lse, rl, "combined lse", tol=1e-5)


def test_combine_natural_log_matches_oracle(gpu):
    o1, l1, o2, l2 = _partials(2, 130, 4, 128, 9)
    out, lse = _online_softmax_combine(o1.to(gpu), l1.to(gpu), o2.to(gpu), l2.to(gpu))
    ro, rl = R.combine_ln(o1.double(), l1.double(), o2.double(), l2.double())
    assert_close(out, ro, rtol=5e-6, atol=5e-6, what="combined out (base e)")
    check_lse(lse, rl, "combined lse (base e)", tol=1e-5)


def test_combine_two_halves(gpu):
    """Split KV in half, compute partial attentions, combine, compare to full."""
    B, S, H, DQ, DV = 1, 256, 16, 192, 128
    scale = DQ**-0.5
    S_half = S // 2
    torch.manual_seed(123)
    q = torch.randn(B, S_half, H, DQ, dtype=torch.bfloat16, device=gpu)
    k1 = torch.randn(B, S_half, H, DQ, dtype=torch.bfloat16, device=gpu)
    v1 = torch.randn(B, S_half, H, DV, dtype=torch.bfloat16, device=gpu)
    k2 = torch.randn(B, S_half, H, DQ, dtype=torch.bfloat16, device=gpu)
    v2 = torch.randn(B, S_half, H, DV, dtype=torch.bfloat16, device=gpu)
    out1, lse1 = _mla_fwd(q, k1, v1, scale, causal=False)
    out2, lse2 = _mla_fwd(q, k2, v2, scale, causal=False)
    combined_out, combined_lse = _online_softmax_combine_log2(out1, lse1, out2, lse2)
    ref_out, ref_lse = R.chunk_fwd(q.cpu(), torch.cat([k1, k2], 1).cpu(), torch.cat([v1, v2], 1).cpu(), scale, False)
    assert_close(combined_out.to(torch.bfloat16), ref_out.to(torch.bfloat16), rtol=1e-2, atol=2e-2)
    check_lse(combined_lse, ref_lse, "two-halves lse")


def test_combine_identity(gpu):
    """Combining with a -inf LSE (or the ring's finfo.min initial state) is the identity."""
    B, S, H, DQ, DV = 1, 128, 16, 192, 128
    scale = DQ**-0.5
    torch.manual_seed(7)
    q = torch.randn(B, S, H, DQ, dtype=torch.bfloat16, device=gpu)
    k = torch.randn(B, S, H, DQ, dtype=torch.bfloat16, device=gpu)
    v = torch.randn(B, S, H, DV, dtype=torch.bfloat16, device=gpu)
    out, lse = _mla_fwd(q, k, v, scale, causal=False)
    zeros = torch.zeros_like(out)
    for empty in (float("-inf"), torch.finfo(torch.float32).min):
        e = torch.full_like(lse, empty)
        co, cl = _online_softmax_combine_log2(out, lse, zeros, e)
        assert_close(co.to(torch.bfloat16), out, rtol=0, atol=1e-5)
        assert torch.equal(cl, lse)
        co, cl = _online_softmax_combine_log2(zeros, e, out, lse)
        assert torch.equal(co.to(torch.bfloat16), out) and torch.equal(cl, lse)


def test_combine_both_empty_is_empty(gpu):
    """Defined here as (0, -inf); the reference yields NaN and never meets the case."""
    z = torch.zeros(1, 8, 2, 64, dtype=torch.bfloat16, device=gpu)
    e = torch.full((1, 2, 8), float("-inf"), device=gpu)
    co, cl = _online_softmax_combine_log2(z, e, z, e)
    assert torch.equal(co, torch.zeros_like(co)) and torch.isinf(cl).all() and (cl < 0).all()


def test_combine_commutes(gpu):
    """Combining A then B equals combining B then A (the reference's 'associativity' test)."""
    B, S, H, DQ, DV = 1, 128, 16, 192, 128
    scale = DQ**-0.5
    torch.manual_seed(99)
    q = torch.randn(B, S, H, DQ, dtype=torch.bfloat16, device=gpu)
    k1 = torch.randn(B, S, H, DQ, dtype=torch.bfloat16, device=gpu)
    v1 = torch.randn(B, S, H, DV, dtype=torch.bfloat16, device=gpu)
    k2 = torch.randn(B, S, H, DQ, dtype=torch.bfloat16, device=gpu)
    v2 = torch.randn(B, S, H, DV, dtype=torch.bfloat16, device=gpu)
    out1, lse1 = _mla_fwd(q, k1, v1, scale, causal=False)
    out2, lse2 = _mla_fwd(q, k2, v2, scale, causal=False)
    comb_ab, lse_ab = _online_softmax_combine_log2(out1, lse1, out2, lse2)
    comb_ba, lse_ba = _online_softmax_combine_log2(out2, lse2, out1, lse1)
    assert_close(comb_ab.to(torch.bfloat16), comb_ba.to(torch.bfloat16), rtol=0, atol=1e-5)
    assert_close(lse_ab, lse_ba, rtol=0, atol=1e-5)


def test_combine_row_range_in_place_and_bf16_out(gpu):
    """The ring's usage: merge a half-chunk result into rows [S/2, S) of the running state in
    place (fp32), and emit bf16 on the last merge; rows outside the range stay untouched."""
    B, S, H, D = 2, 64, 4, 128
    o1, l1, o2, l2 = _partials(B, S, H, D, 21, torch.float32, torch.bfloat16)
    run, run_lse = o1.to(gpu), l1.to(gpu)
    keep, keep_lse = run.clone(), run_lse.clone()
    half = S // 2
    step, step_lse = o2[:, half:].contiguous().to(gpu), l2[:, :, half:].contiguous().to(gpu)
    combine_into(run[:, half:], run_lse[:, :, half:], step, step_lse, run[:, half:], run_lse[:, :, half:])
    ro, rl = R.combine_log2(o1[:, half:].double(), l1[:, :, half:].double(), o2[:, half:].double(), l2[:, :, half:].double())
    assert torch.equal(run[:, :half], keep[:, :half]) and torch.equal(run_lse[:, :, :half], keep_lse[:, :, :half])
    assert_close(run[:, half:], ro, rtol=2e-6, atol=2e-6)
    check_lse(run_lse[:, :, half:], rl, "row-range lse", tol=1e-5)
    out_bf16 = torch.zeros(B, S, H, D, dtype=torch.bfloat16, device=gpu)
    lse_o = torch.empty_like(keep_lse)
    combine_into(keep, keep_lse, o2.to(gpu), l2.to(gpu), out_bf16, lse_o)
    full, _ = R.combine_log2(o1.double(), l1.double(), o2.double(), l2.double())
    assert torch.equal(out_bf16.cpu(), full.to(torch.float32).to(torch.bfloat16)) or (
        (out_bf16.cpu().float() - full.float()).abs() <= full.float().abs() * 2**-8 + 1e-30
    ).all()


@pytest.mark.parametrize("dts", [("bf16", "bf16", "f32"), ("bf16", "bf16", "bf16"), ("f32", "bf16", "f32"),
                                 ("f32", "bf16", "bf16"), ("bf16", "f32", "f32"), ("f32", "f32", "f32")])
@pytest.mark.parametrize("B,S,H,D", [
    (1, 96, 32, 128),   # fp32 chunks: 32 rows x 32 chunks = 256 x 4 per position
    (2, 40, 64, 128),   # 64 heads: 256 x 8 (the long-context shape)
    (1, 64, 16, 128),   # 16 heads (MLA): two positions per tile
    (1, 24, 8, 64),     # 8 positions per tile
    (1, 1000, 32, 128),  # more tiles than one round of blocks covers on a 256-CU device, ragged last round
])
def test_combine_front_walk_equals_per_tile_kernel(gpu, dts, B, S, H, D):
    """Shapes that take the front-walking kernel (one block per compute unit, tiles of 256 x U chunks) in
    every dtype combination and unroll, in place and out of place, against the oracle, and bit for bit
    against the per-tile kernel: the same problem with one position appended no longer divides into
    front tiles evenly (S odd -> one position per tile is still possible, so a head is appended instead:
    H+1 heads never give 256 x U chunks) and is served by the per-tile kernel."""
    dt = {"bf16": torch.bfloat16, "f32": torch.float32}
    d1, d2, do = (dt[x] for x in dts)
    o1, l1, o2, l2 = _partials(B, S, H + 1, D, 31, d1, d2)
    # per-tile kernel on H+1 heads, then compare heads [0, H)
    big = [t.to(gpu) for t in (o1, l1, o2, l2)]
    out_big = torch.empty(B, S, H + 1, D, dtype=do, device=gpu)
    lse_big = torch.empty(B, H + 1, S, dtype=torch.float32, device=gpu)
    combine_into(*big, out_big, lse_big)
    small = [o1[:, :, :H].contiguous().to(gpu), l1[:, :H].contiguous().to(gpu),
             o2[:, :, :H].contiguous().to(gpu), l2[:, :H].contiguous().to(gpu)]  # fmt: skip
    out = torch.full((B, S, H, D), float("nan"), dtype=do, device=gpu)
    lse = torch.full((B, H, S), float("nan"), dtype=torch.float32, device=gpu)
    combine_into(*small, out, lse)
    assert torch.equal(out, out_big[:, :, :H]) and torch.equal(lse, lse_big[:, :H])
    ro, rl = R.combine_log2(small[0].double().cpu(), small[1].double().cpu(), small[2].double().cpu(), small[3].double().cpu())
    if do == torch.float32:
        assert_close(out, ro, rtol=2e-6, atol=2e-6, what="combined out")
    else:
        assert_close(out, ro, rtol=2**-8 * 1.01, atol=1e-6, what="combined out (bf16)")  # one rounding to bf16: half an ulp
    check_lse(lse, rl, "combined lse", tol=1e-5)
    # in place: out aliases the partial of its dtype, lse_out aliases lse1
    if do in (d1, d2):
        tgt = small[0] if do == d1 else small[2]
        combine_into(*small, tgt, small[1])
        assert torch.equal(tgt, out) and torch.equal(small[1], lse)


def test_cast_f32_bf16_is_round_to_nearest_even(gpu):
    g = torch.Generator().manual_seed(0)
    x = torch.randn(4096, generator=g) * 100
    x[:8] = torch.tensor([1.00390625, 1.01171875, -1.00390625, 0.0, 3.0e38, 1e-40, -0.0, 65504.0])  # ties and extremes
    y = torch.empty(4096, dtype=torch.bfloat16, device=gpu)
    cast_f32_bf16_into(x.to(gpu), y)
    assert torch.equal(y.cpu(), x.to(torch.bfloat16))


def test_combine_full_size_properties(gpu):
    """The benchmark combine shape [1, 4096, 32, 128]: oracle comparison in full (seconds on the CPU),
    commutativity and the identity."""
    o1, l1, o2, l2 = _partials(1, 4096, 32, 128, 42)
    d = [t.to(gpu) for t in (o1, l1, o2, l2)]
    ab, lab = _online_softmax_combine_log2(*d)
    ba, lba = _online_softmax_combine_log2(d[2], d[3], d[0], d[1])
    assert_close(ab, ba, rtol=0, atol=1e-6)
    assert_close(lab, lba, rtol=0, atol=1e-6)
    ro, rl = R.combine_log2(o1.float(), l1, o2.float(), l2)
    assert_close(ab, ro, rtol=3e-6, atol=3e-6)
    check_lse(lab, rl, "full-size lse", tol=1e-5)
    e = torch.full_like(d[1], torch.finfo(torch.float32).min)
    ident, _ = _online_softmax_combine_log2(torch.zeros_like(d[0]), e, d[2], d[3])
    assert torch.equal(ident, d[2].float())


def test_combine_error_paths(gpu):
    o = torch.zeros(1, 8, 2, 64, dtype=torch.bfloat16, device=gpu)
    l = torch.zeros(1, 2, 8, device=gpu)
    with pytest.raises(AssertionError):
        combine_into(o, l, o[:, :4], l, o, l)
    with pytest.raises(TypeError):
        combine_into(o.half(), l, o, l, o, l)
    with pytest.raises(_C.PithError) as e:
        bad = torch.zeros(1, 8, 2, 60, dtype=torch.bfloat16, device=gpu)
        combine_into(bad, l, bad, l, bad, l)
    assert e.value.code == _C.PITH_ERR_BAD_SHAPE
