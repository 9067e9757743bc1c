"""Two conveniences of the backward entry points that spare the ring separate launches: the dK/dV call that also
clears the rows of dk / dv behind the visible part of a chunk (the reference allocates zeroed gradients per step,
pithtrain/operators/ring_attention/standard.py:131-133), and the dQ call that emits finished rows as bf16 beside the
fp32 accumulator (the reference adds bf16 partials, mla.py:116; here the sum is rounded once). Both must give, bit
for bit, what the separate fill / cast launches give."""

import pytest
import torch

from helpers import check_bf16_result
from oracle import ring_oracle as R
from pithtrain_amd import _C
from pithtrain_amd.operators.mla import hip as H
from pithtrain_amd.operators.ring_attention import local as L

pytestmark = pytest.mark.gpu


def _inputs(B, Sq, Skv, Hq, Hkv, Dqk, seed=42):
    g = torch.Generator().manual_seed(seed)
    scale = Dqk**-0.5
    q = (torch.randn(B, Sq, Hq, Dqk, generator=g) * scale).to(torch.bfloat16)
    k = (torch.randn(B, Skv, Hkv, Dqk, generator=g) * scale).to(torch.bfloat16)
    v = (torch.randn(B, Skv, Hkv, min(Dqk, 128), generator=g) * scale).to(torch.bfloat16)
    dout = torch.randn(B, Sq, Hq, min(Dqk, 128), generator=g).to(torch.bfloat16)
    return q, k, v, dout, scale


@pytest.mark.parametrize("Dqk,Hq,Hkv", [(128, 8, 2), (128, 4, 4), (192, 4, 4), (64, 4, 2)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_dkdv_clears_the_rows_behind_the_visible_part(gpu, Dqk, Hq, Hkv, dtype):
    B, Sq, S_chunk, Skv = 2, 320, 400, 200  # the step sees rows [0, 200) of a 400-row chunk
    q, k, v, dout, scale = _inputs(B, Sq, S_chunk, Hq, Hkv, Dqk)
    qd, kd, vd, dod = (t.to(gpu) for t in (q, k, v, dout))
    ks, vs = kd[:, :Skv], vd[:, :Skv]
    o, lse = H._mla_fwd(qd, ks, vs, scale, False)
    delta = H._mla_bwd_preprocess(o, dod)
    want_dk = torch.zeros(kd.shape, dtype=dtype, device=gpu)
    want_dv = torch.zeros(vd.shape, dtype=dtype, device=gpu)
    H.attn_bwd_dkdv_into(qd, ks, vs, dod, lse, delta, want_dk[:, :Skv], want_dv[:, :Skv], scale, False)
    dk = torch.full(kd.shape, float("nan"), dtype=dtype, device=gpu)
    dv = torch.full(vd.shape, float("nan"), dtype=dtype, device=gpu)
    H.attn_bwd_dkdv_into(qd, ks, vs, dod, lse, delta, dk[:, :Skv], dv[:, :Skv], scale, False, zero_tail=S_chunk - Skv)
    assert torch.equal(dk, want_dk) and torch.equal(dv, want_dv)
    # accumulating calls leave the rows alone
    dk2, dv2 = torch.ones_like(dk), torch.ones_like(dv)
    H.attn_bwd_dkdv_into(qd, ks, vs, dod, lse, delta, dk2[:, :Skv], dv2[:, :Skv], scale, False, accumulate=True,
                         zero_tail=S_chunk - Skv)  # fmt: skip
    assert (dk2[:, Skv:] == 1).all() and (dv2[:, Skv:] == 1).all()


# (Sq, Skv, Hq, Hkv, hand-over, Dqk): the three dQ kernels for head dims (128, 128) and the one for (192, 128)
DQ_KERNELS = [
    pytest.param(2048, 1024, 32, 4, True, 128, id="from-dS-images"),
    pytest.param(2048, 1024, 32, 4, False, 128, id="recomputing-256-row"),
    pytest.param(640, 320, 4, 2, False, 128, id="recomputing-128-row"),
    pytest.param(1000, 520, 8, 2, False, 128, id="ragged"),
    pytest.param(1024, 512, 16, 16, False, 192, id="mla-192"),
    pytest.param(333, 200, 4, 4, False, 192, id="mla-192-ragged"),
]


@pytest.mark.parametrize("Sq,Skv,Hq,Hkv,handover,Dqk", DQ_KERNELS)
@pytest.mark.parametrize("accumulate", [True, False])
def test_dq_final_rows_equal_accumulate_then_cast(gpu, Sq, Skv, Hq, Hkv, handover, Dqk, accumulate):
    B = 1
    q, k, v, dout, scale = _inputs(B, Sq, Skv, Hq, Hkv, Dqk, seed=5)
    qd, kd, vd, dod = (t.to(gpu) for t in (q, k, v, dout))
    o, lse = H._mla_fwd(qd, kd, vd, scale, False)
    delta = H._mla_bwd_preprocess(o, dod)
    old = torch.randn(qd.shape, device=gpu) * 0.01
    ds = torch.empty(H.attn_bwd_ds_bytes(qd, kd, vd, False), dtype=torch.uint8, device=gpu) if handover else None
    dk, dv = torch.empty_like(kd), torch.empty_like(vd)
    H.attn_bwd_dkdv_into(qd, kd, vd, dod, lse, delta, dk, dv, scale, False, ds=ds)
    acc = old.clone()
    H.attn_bwd_dq_into(qd, kd, vd, dod, lse, delta, acc, scale, False, accumulate=accumulate, ds=ds)
    want = acc.to(torch.bfloat16)
    r0, r1 = (Sq // 2) // 32 * 32, Sq  # the second part of the rows is finished by this call
    acc2 = old.clone()
    fin = torch.full(qd.shape, 3.0, dtype=torch.bfloat16, device=gpu)
    H.attn_bwd_dq_into(qd, kd, vd, dod, lse, delta, acc2, scale, False, accumulate=accumulate, ds=ds,
                       dq_final=fin, dq_final_rows=(r0, r1))  # fmt: skip
    assert torch.equal(fin[:, r0:r1], want[:, r0:r1]), "finished rows must equal accumulate + cast"
    assert (fin[:, :r0] == 3.0).all(), "rows outside dq_final_rows must stay untouched"
    assert torch.equal(acc2[:, :r0], acc[:, :r0]), "unfinished rows go to the fp32 tensor as before"
    assert torch.equal(acc2[:, r0:r1], old[:, r0:r1]), "finished rows leave the fp32 tensor alone"
    with pytest.raises(_C.PithError, match="PITH_ERR_BAD_SHAPE"):
        H.attn_bwd_dq_into(qd, kd, vd, dod, lse, delta, acc2, scale, False, dq_final=fin, dq_final_rows=(8, 40))
    with pytest.raises(_C.PithError, match="PITH_ERR_UNSUPPORTED"):  # a bf16 dq has nothing to finish
        H.attn_bwd_dq_into(qd, kd, vd, dod, lse, delta, fin.clone(), scale, False, dq_final=fin)


@pytest.mark.parametrize("layout", ["contiguous", "zigzag"])
@pytest.mark.parametrize("Hq,Hkv,S,D", [(8, 2, 2048, 128), (32, 4, 4096, 128), (4, 4, 1000, 128), (4, 4, 2048, 192)])
def test_ring_backward_with_and_without_the_fused_epilogues(gpu, layout, Hq, Hkv, S, D, monkeypatch):
    """Every rank of a ring of 4: dQ, dK, dV bit for bit the same whether the fill and the cast are separate
    launches or folded into the dK/dV and dQ launches, and equal to the oracle's ring share."""
    B, C = 1, 4
    g = torch.Generator().manual_seed(13)
    scale = D**-0.5
    full = [torch.randn(B, S, h, d, generator=g).to(torch.bfloat16) for h, d in ((Hq, D), (Hkv, D), (Hkv, 128), (Hq, 128))]
    split = (lambda x: R.zigzag_split(x, C)) if layout == "zigzag" else (lambda x: [c.contiguous() for c in x.chunk(C, 1)])
    if layout == "zigzag" and S % (2 * C):
        pytest.skip("zigzag needs 2 * cp_size blocks")
    qs, ks, vs, dos = (split(t) for t in full)
    kd, vd = [c.to(gpu) for c in ks], [c.to(gpu) for c in vs]
    for r in range(C):
        res = {}
        for fused in (True, False):
            monkeypatch.setattr(L, "FUSE_FINAL_DQ", fused)
            monkeypatch.setattr(L, "FUSE_ZERO_TAIL", fused)
            qd = qs[r].to(gpu)
            out, lse = L.ring_forward_local(qd, kd, vd, scale, r, C, layout)
            res[fused] = L.ring_backward_local(dos[r].to(gpu), qd, out, lse, kd, vd, scale, r, C, layout)
        dq1, dk1, dv1 = res[True]
        dq0, dk0, dv0 = res[False]
        assert torch.equal(dq1, dq0), f"rank {r}: dQ differs"
        for a, b in zip(dk1 + dv1, dk0 + dv0):
            assert (a is None and b is None) or torch.equal(a, b), f"rank {r}: dK / dV differ"
        ro, rl = R.ring_forward(qs[r], ks, vs, scale, r, C, layout)
        rdq, _, _ = R.ring_backward(dos[r], qs[r], ro, rl, ks, vs, scale, r, C, layout)
        check_bf16_result(dq1, rdq, f"ring dQ rank {r}", otol=1e-3)
