"""HIP attention prologue (per-head RMSNorm + rotary embedding) against the fp64 oracle, through
the C-ABI library. The kernel rounds to bf16 once, so the bound is one bf16 rounding of the exact
result (relative 2^-8) plus a small absolute term for fp32 cancellation; dweight is an fp32 sum."""

import pytest
import torch

from helpers import assert_close
from oracle import prologue_oracle as P

pytestmark = pytest.mark.gpu

RTOL = 2.0**-8


def _inputs(b, s, h, d, seed, weight_dtype=torch.bfloat16, per_batch_positions=True, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(b, s, h, d, generator=g) * scale).bfloat16()
    w = (torch.rand(d, generator=g) + 0.5).to(weight_dtype)
    if per_batch_positions:
        pos = torch.stack([torch.arange(s) + 977 * i for i in range(b)])
    else:
        pos = torch.arange(s).unsqueeze(0) + 31
    cos, sin = P.cos_sin_table(pos, d, dtype=torch.bfloat16)
    dout = torch.randn(b, s, h, d, generator=g).bfloat16()
    return x, w, cos, sin, dout


def _check(actual, expected, what):
    tol = 1e-5 * expected.abs().max().item()
    assert_close(actual, expected, rtol=RTOL, atol=tol, what=what)


CASES = [
    # b, s, h, d
    (1, 64, 32, 128),  # Qwen3 q heads
    (1, 64, 4, 128),   # Qwen3 kv heads
    (2, 37, 8, 128),   # ragged token count, two batch elements
    (1, 5, 5, 128),    # heads not a multiple of the head-group count
    (2, 19, 40, 128),  # more heads than one pass of a slot covers
    (1, 33, 12, 64),
    (1, 9, 3, 256),
    (1, 7, 2, 512),
    (1, 1, 1, 8),
    (3, 1, 16, 128),
]


@pytest.mark.parametrize("b,s,h,d", CASES)
@pytest.mark.parametrize("with_weight", [True, False])
def test_forward_and_backward_match_the_oracle(gpu, b, s, h, d, with_weight):
    from pithtrain_amd.operators.norm_rope import norm_rope_bwd_into, norm_rope_fwd_into

    x, w, cos, sin, dout = _inputs(b, s, h, d, seed=b * 1000 + s * 10 + h)
    if not with_weight:
        w = None
    eps = 1e-6
    want = P.norm_rope_fwd(x, w, cos, sin, eps)
    want_dx, want_dw = P.norm_rope_bwd(x, w, cos, sin, dout, eps)

    xd, cd, sd, dd = x.to(gpu), cos.to(gpu), sin.to(gpu), dout.to(gpu)
    wd = None if w is None else w.to(gpu)
    out = torch.full_like(xd, float("nan"))
    norm_rope_fwd_into(xd, wd, cd, sd, out, eps)
    _check(out, want, "out")

    dx = torch.full_like(xd, float("nan"))
    dw = None if w is None else torch.full((d,), float("nan"), device=gpu)
    norm_rope_bwd_into(xd, wd, cd, sd, dd, dx, dw, eps)
    _check(dx, want_dx, "dx")
    if w is not None:
        assert_close(dw, want_dw, rtol=1e-4, atol=1e-4 * want_dw.abs().max().item(), what="dweight")


def test_fp32_weight_and_shared_cos_sin_tables(gpu):
    from pithtrain_amd.operators.norm_rope import norm_rope_bwd_into, norm_rope_fwd_into

    b, s, h, d = 3, 21, 8, 128
    x, w, cos, sin, dout = _inputs(b, s, h, d, seed=5, weight_dtype=torch.float32, per_batch_positions=False)
    want = P.norm_rope_fwd(x, w, cos, sin, 1e-5)
    want_dx, want_dw = P.norm_rope_bwd(x, w, cos, sin, dout, 1e-5)
    xd, wd, dd = x.to(gpu), w.to(gpu), dout.to(gpu)
    for c, sn in ((cos.to(gpu), sin.to(gpu)), (cos[0].to(gpu), sin[0].to(gpu))):  # [1,S,D] and [S,D]
        out = torch.empty_like(xd)
        norm_rope_fwd_into(xd, wd, c, sn, out, 1e-5)
        _check(out, want, "out")
        dx, dw = torch.empty_like(xd), torch.empty(d, device=gpu)
        norm_rope_bwd_into(xd, wd, c, sn, dd, dx, dw, 1e-5)
        _check(dx, want_dx, "dx")
        assert_close(dw, want_dw, rtol=1e-4, atol=1e-4 * want_dw.abs().max().item(), what="dweight")


def test_eps_matters_for_small_rows_and_zero_rows_stay_finite(gpu):
    from pithtrain_amd.operators.norm_rope import norm_rope_bwd_into, norm_rope_fwd_into

    b, s, h, d = 1, 8, 4, 128
    x, w, cos, sin, dout = _inputs(b, s, h, d, seed=9, scale=1e-3)  # mean square ~1e-6 = eps
    x[0, 3] = 0  # a token of exact zeros
    want = P.norm_rope_fwd(x, w, cos, sin, 1e-6)
    want_dx, want_dw = P.norm_rope_bwd(x, w, cos, sin, dout, 1e-6)
    xd, wd, cd, sd, dd = (t.to(gpu) for t in (x, w, cos, sin, dout))
    out, dx, dw = torch.empty_like(xd), torch.empty_like(xd), torch.empty(d, device=gpu)
    norm_rope_fwd_into(xd, wd, cd, sd, out, 1e-6)
    norm_rope_bwd_into(xd, wd, cd, sd, dd, dx, dw, 1e-6)
    assert torch.isfinite(out.float()).all() and torch.isfinite(dx.float()).all()
    assert out[0, 3].abs().max().item() == 0.0
    _check(out, want, "out")
    _check(dx, want_dx, "dx")
    assert_close(dw, want_dw, rtol=1e-4, atol=1e-4 * want_dw.abs().max().item(), what="dweight")


def test_in_place_and_batch_strided_views(gpu):
    from pithtrain_amd.operators.norm_rope import norm_rope_bwd_into, norm_rope_fwd_into

    b, s, h, d = 2, 16, 4, 128
    x, w, cos, sin, dout = _inputs(b, s, h, d, seed=3)
    want = P.norm_rope_fwd(x, w, cos, sin, 1e-6)
    want_dx, _ = P.norm_rope_bwd(x, w, cos, sin, dout, 1e-6)
    wd, cd, sd = w.to(gpu), cos.to(gpu), sin.to(gpu)
    # x is the first S rows of a longer buffer: the batch stride exceeds S*H*D
    big = torch.zeros(b, 2 * s, h, d, dtype=torch.bfloat16, device=gpu)
    big[:, :s] = x.to(gpu)
    view = big[:, :s]
    norm_rope_fwd_into(view, wd, cd, sd, view, 1e-6)  # in place
    _check(view, want, "out (in place)")
    assert big[:, s:].abs().max().item() == 0.0  # nothing written past the view
    grad = dout.to(gpu).clone()
    dw = torch.empty(d, device=gpu)
    norm_rope_bwd_into(x.to(gpu), wd, cd, sd, grad, grad, dw, 1e-6)  # dx over dout
    _check(grad, want_dx, "dx (in place)")


def test_dweight_is_reproducible(gpu):
    from pithtrain_amd.operators.norm_rope import norm_rope_bwd_into

    b, s, h, d = 2, 1024, 32, 128
    x, w, cos, sin, dout = (t.to(gpu) for t in _inputs(b, s, h, d, seed=11))
    results = []
    for _ in range(3):
        dx, dw = torch.empty_like(x), torch.empty(d, device=gpu)
        norm_rope_bwd_into(x, w, cos, sin, dout, dx, dw, 1e-6)
        results.append((dx.clone(), dw.clone()))
    for dx, dw in results[1:]:
        assert torch.equal(dx, results[0][0]) and torch.equal(dw, results[0][1])


def test_autograd_and_reference_named_functions(gpu):
    from pithtrain_amd.operators.norm_rope import apply_rotary_pos_emb, qk_norm_rope

    b, s, d = 2, 48, 128
    q, wq, cos, sin, dq_out = _inputs(b, s, 8, d, seed=21)
    k, wk, _, _, dk_out = _inputs(b, s, 2, d, seed=22)
    want_q = P.norm_rope_fwd(q, wq, cos, sin, 1e-6)
    want_k = P.norm_rope_fwd(k, wk, cos, sin, 1e-6)
    want_dq, want_dwq = P.norm_rope_bwd(q, wq, cos, sin, dq_out, 1e-6)
    want_dk, want_dwk = P.norm_rope_bwd(k, wk, cos, sin, dk_out, 1e-6)

    qd = q.to(gpu).requires_grad_()
    kd = k.to(gpu).requires_grad_()
    wqd = wq.to(gpu).requires_grad_()
    wkd = wk.to(gpu).requires_grad_()
    cd, sd = cos.to(gpu), sin.to(gpu)
    oq, ok = qk_norm_rope(qd, kd, wqd, wkd, cd, sd, 1e-6)
    _check(oq, want_q, "q")
    _check(ok, want_k, "k")
    torch.autograd.backward([oq, ok], [dq_out.to(gpu), dk_out.to(gpu)])
    _check(qd.grad, want_dq, "dq")
    _check(kd.grad, want_dk, "dk")
    assert wqd.grad.dtype == torch.bfloat16
    assert_close(wqd.grad, want_dwq, rtol=1e-2, atol=1e-2 * want_dwq.abs().max().item(), what="dwq")
    assert_close(wkd.grad, want_dwk, rtol=1e-2, atol=1e-2 * want_dwk.abs().max().item(), what="dwk")

    # rotary embedding alone, under the reference's name
    rq, rk = apply_rotary_pos_emb(q.to(gpu), k.to(gpu), cd, sd)
    _check(rq, P.norm_rope_fwd(q, None, cos, sin, 0.0), "rope(q)")
    _check(rk, P.norm_rope_fwd(k, None, cos, sin, 0.0), "rope(k)")


@pytest.mark.parametrize("with_weight", [True, False])
def test_pair_launch_equals_two_single_launches(gpu, with_weight):
    """q and k in one launch: bit-identical to the single-tensor entry points, including dweight."""
    from pithtrain_amd.operators.norm_rope import (
        norm_rope_bwd_into, norm_rope_fwd_into, qk_norm_rope_bwd_into, qk_norm_rope_fwd_into,
    )  # fmt: skip

    b, s, d = 2, 301, 128
    q, wq, cos, sin, gq = (t.to(gpu) for t in _inputs(b, s, 32, d, seed=51))
    k, wk, _, _, gk = (t.to(gpu) for t in _inputs(b, s, 4, d, seed=52, weight_dtype=torch.float32))
    if not with_weight:
        wq = wk = None
    new = lambda t: torch.full_like(t, float("nan"))  # noqa: E731
    dw = lambda: torch.full((d,), float("nan"), device=gpu) if with_weight else None  # noqa: E731
    single = {"q": new(q), "k": new(k), "dq": new(q), "dk": new(k), "dwq": dw(), "dwk": dw()}
    norm_rope_fwd_into(q, wq, cos, sin, single["q"], 1e-6)
    norm_rope_fwd_into(k, wk, cos, sin, single["k"], 1e-6)
    norm_rope_bwd_into(q, wq, cos, sin, gq, single["dq"], single["dwq"], 1e-6)
    norm_rope_bwd_into(k, wk, cos, sin, gk, single["dk"], single["dwk"], 1e-6)
    pair = {"q": new(q), "k": new(k), "dq": new(q), "dk": new(k), "dwq": dw(), "dwk": dw()}
    qk_norm_rope_fwd_into(q, k, wq, wk, cos, sin, pair["q"], pair["k"], 1e-6)
    qk_norm_rope_bwd_into(q, k, wq, wk, cos, sin, gq, gk, pair["dq"], pair["dk"], pair["dwq"], pair["dwk"], 1e-6)
    for name in single:
        if single[name] is not None:
            assert torch.equal(single[name], pair[name]), name


def test_pair_with_different_head_dims_and_lengths(gpu):
    """The two tensors of a pair only share B: different S, H, D and cos/sin tables are allowed."""
    from pithtrain_amd.operators.norm_rope import norm_rope_fwd_into
    from pithtrain_amd import _C
    from pithtrain_amd.operators import norm_rope as NR

    xa, wa, ca, sa, _ = (t.to(gpu) for t in _inputs(1, 50, 6, 64, seed=61))
    xb, wb, cb, sb, _ = (t.to(gpu) for t in _inputs(1, 9, 3, 256, seed=62))
    oa, ob = torch.empty_like(xa), torch.empty_like(xb)
    a = NR._args(xa, wa, ca, sa, oa, 1e-6)
    b = NR._args(xb, wb, cb, sb, ob, 1e-5)
    _C.check(_C.lib().pith_norm_rope_fwd_pair(_C.byref(a), _C.byref(b), _C.current_stream(xa)))
    ra, rb = torch.empty_like(xa), torch.empty_like(xb)
    norm_rope_fwd_into(xa, wa, ca, sa, ra, 1e-6)
    norm_rope_fwd_into(xb, wb, cb, sb, rb, 1e-5)
    assert torch.equal(oa, ra) and torch.equal(ob, rb)


def test_at_least_as_accurate_as_the_eager_bf16_expression(gpu):
    """The reference's evaluation (nn.RMSNorm, then the bf16 expression of
    pithtrain/models/qwen3_30b_a3b.py:132-136) run eagerly on the GPU: the fused kernel's error
    against the oracle is no larger."""
    from pithtrain_amd.operators.norm_rope import norm_rope

    b, s, h, d = 1, 256, 32, 128
    x, w, cos, sin, _ = _inputs(b, s, h, d, seed=33)
    want = P.norm_rope_fwd(x, w, cos, sin, 1e-6)
    xd, wd, cd, sd = (t.to(gpu) for t in (x, w, cos, sin))
    y = torch.nn.functional.rms_norm(xd, (d,), wd, 1e-6)
    c, sn = cd.unsqueeze(2), sd.unsqueeze(2)
    eager = (y * c) + (torch.cat((-y[..., d // 2 :], y[..., : d // 2]), dim=-1) * sn)
    ours = norm_rope(xd, wd, cd, sd, 1e-6)
    err = lambda t: (t.double().cpu() - want).abs().mean().item()  # noqa: E731
    assert err(ours) <= err(eager)
    assert_close(ours, eager, rtol=3e-2, atol=3e-2, what="ours vs eager")


def test_full_size_qwen3_share(gpu):
    """The benchmark's shape (one rank's 8192 tokens, 32 q heads + 4 kv heads of 128): forward and
    backward against the oracle on every row, and the rotation keeps each pair's length."""
    from pithtrain_amd.operators.norm_rope import norm_rope_bwd_into, norm_rope_fwd_into

    s, d = 8192, 128
    for h, seed in ((32, 41), (4, 42)):
        x, w, cos, sin, dout = _inputs(1, s, h, d, seed=seed)
        xd, wd, cd, sd, dd = (t.to(gpu) for t in (x, w, cos, sin, dout))
        out, dx, dw = torch.empty_like(xd), torch.empty_like(xd), torch.empty(d, device=gpu)
        norm_rope_fwd_into(xd, wd, cd, sd, out, 1e-6)
        norm_rope_bwd_into(xd, wd, cd, sd, dd, dx, dw, 1e-6)
        want = P.norm_rope_fwd(x, w, cos, sin, 1e-6)
        want_dx, want_dw = P.norm_rope_bwd(x, w, cos, sin, dout, 1e-6)
        _check(out, want, "out")
        _check(dx, want_dx, "dx")
        assert_close(dw, want_dw, rtol=1e-4, atol=1e-4 * want_dw.abs().max().item(), what="dweight")
        # rope only: pair lengths are preserved up to the bf16 rounding of cos/sin and of the result
        rot = torch.empty_like(xd)
        norm_rope_fwd_into(xd, None, cd, sd, rot, 0.0)
        pair = lambda t: (t[..., : d // 2].double() ** 2 + t[..., d // 2 :].double() ** 2)  # noqa: E731
        assert_close(pair(rot.cpu()), pair(x), rtol=2e-2, atol=1e-3, what="pair lengths")
