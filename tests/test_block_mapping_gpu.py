"""Launches with many tiles and more than 8 kv heads take their heads in chunks of 8 kv heads (attn_tiles.h,
decode_block; attn_bwd_common.h, decode_dkdv_block) instead of level by level over all heads. Which workgroup
computes which (tile, head) must not change any result: every kernel is run on 16 heads x 16384 rows (64 or more
tiles: the chunked order) and on the two halves of the heads separately (8 heads: the plain order), and the results
are compared. The halves may pick another workgroup shape (the launch heuristics look at the grid size), so the
comparison is to rounding, not bit for bit: a workgroup on a wrong tile or head, or a tile nobody computes (the
outputs start as NaN), is off by the size of the values themselves."""

import pytest
import torch

from pithtrain_amd.operators.mla import hip as H

pytestmark = pytest.mark.gpu

S, HEADS = 16384, 16


def _close(got, want, what, tol=2e-2):
    got, want = got.float(), want.float()
    assert torch.isfinite(got).all(), f"{what}: not finite (a tile was not computed)"
    err = (got - want).abs().max().item() / want.abs().max().item()
    assert err < tol, f"{what}: {err:.3e} of the largest value"


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("Dqk", [128, 192])
def test_chunked_head_order_changes_no_result(gpu, Dqk, causal):
    Dv = 128
    g = torch.Generator().manual_seed(5)
    scale = Dqk**-0.5
    q = (torch.randn(1, S, HEADS, Dqk, generator=g) * scale).to(torch.bfloat16).to(gpu)
    k = (torch.randn(1, S, HEADS, Dqk, generator=g) * scale).to(torch.bfloat16).to(gpu)
    v = (torch.randn(1, S, HEADS, Dv, generator=g) * scale).to(torch.bfloat16).to(gpu)
    dout = torch.randn(1, S, HEADS, Dv, generator=g).to(torch.bfloat16).to(gpu)

    def run(qs, ks, vs, dos):
        o = torch.full(dos.shape, float("nan"), dtype=torch.bfloat16, device=gpu)
        lse = torch.full((1, qs.shape[2], S), float("nan"), device=gpu)
        H.attn_fwd_into(qs, ks, vs, o, lse, scale, causal)
        delta = torch.empty_like(lse)
        H.attn_bwd_delta_into(o, dos, delta)
        dq = torch.full(qs.shape, float("nan"), device=gpu)
        dk = torch.full(ks.shape, float("nan"), dtype=torch.bfloat16, device=gpu)
        dv = torch.full(vs.shape, float("nan"), dtype=torch.bfloat16, device=gpu)
        H.attn_bwd_dkdv_into(qs, ks, vs, dos, lse, delta, dk, dv, scale, causal)
        H.attn_bwd_dq_into(qs, ks, vs, dos, lse, delta, dq, scale, causal)
        return o, lse, dq, dk, dv

    whole = run(q, k, v, dout)
    for h0 in (0, 8):
        part = run(*(t[:, :, h0 : h0 + 8].contiguous() for t in (q, k, v, dout)))
        tag = f"heads {h0}..{h0 + 8}"
        _close(whole[0][:, :, h0 : h0 + 8], part[0], f"o, {tag}")
        assert (whole[1][:, h0 : h0 + 8] - part[1]).abs().max().item() < 2e-3, f"lse, {tag}"
        _close(whole[2][:, :, h0 : h0 + 8], part[2], f"dq, {tag}")
        _close(whole[3][:, :, h0 : h0 + 8], part[3], f"dk, {tag}")
        _close(whole[4][:, :, h0 : h0 + 8], part[4], f"dv, {tag}")


def test_descending_query_walk_of_the_causal_dkdv_kernel(gpu):
    """Causal dK/dV for head dims (128, 128) walks the query tiles from the last one down once Q and dO exceed
    192 MB (attn_bwd_dkdv.hip, kWalkDescBytes): 16384 rows x 32 query heads x 256 features x 2 bytes x 2 tensors =
    256 MiB. Reference: the same kv heads two at a time (16 query heads: 128 MiB, ascending walk). The sums run in
    another order, so the comparison is to rounding. The dS tiles the descending walk stores must serve the dQ
    kernel like those of the ascending one."""
    Sq, Hq, Hkv, D = 16384, 32, 4, 128
    g = torch.Generator().manual_seed(9)
    scale = D**-0.5
    q = (torch.randn(1, Sq, Hq, D, generator=g) * scale).to(torch.bfloat16).to(gpu)
    k = (torch.randn(1, Sq, Hkv, D, generator=g) * scale).to(torch.bfloat16).to(gpu)
    v = (torch.randn(1, Sq, Hkv, D, generator=g) * scale).to(torch.bfloat16).to(gpu)
    dout = torch.randn(1, Sq, Hq, D, generator=g).to(torch.bfloat16).to(gpu)
    o = torch.empty_like(dout)
    lse = torch.empty((1, Hq, Sq), device=gpu)
    H.attn_fwd_into(q, k, v, o, lse, scale, True)
    delta = torch.empty_like(lse)
    H.attn_bwd_delta_into(o, dout, delta)

    dk = torch.full(k.shape, float("nan"), dtype=torch.bfloat16, device=gpu)
    dv = torch.full(v.shape, float("nan"), dtype=torch.bfloat16, device=gpu)
    ds = torch.full((H.attn_bwd_ds_bytes(q, k, v, True),), 0x7F, dtype=torch.uint8, device=gpu)
    H.attn_bwd_dkdv_into(q, k, v, dout, lse, delta, dk, dv, scale, True, ds=ds)
    dq_ds = torch.full(q.shape, float("nan"), device=gpu)
    H.attn_bwd_dq_into(q, k, v, dout, lse, delta, dq_ds, scale, True, ds=ds)
    del ds
    dq = torch.empty(q.shape, device=gpu)
    H.attn_bwd_dq_into(q, k, v, dout, lse, delta, dq, scale, True)
    _close(dq_ds, dq, "dq from the stored dS tiles", tol=6e-3)
    group = Hq // Hkv
    for h0 in (0, 2):
        qs, dos = (t[:, :, h0 * group : (h0 + 2) * group].contiguous() for t in (q, dout))
        ks, vs = (t[:, :, h0 : h0 + 2].contiguous() for t in (k, v))
        ls, des = (t[:, h0 * group : (h0 + 2) * group].contiguous() for t in (lse, delta))
        dk2, dv2 = torch.empty_like(ks), torch.empty_like(vs)
        H.attn_bwd_dkdv_into(qs, ks, vs, dos, ls, des, dk2, dv2, scale, True)
        _close(dk[:, :, h0 : h0 + 2], dk2, f"dk, kv heads {h0}, {h0 + 1}", tol=1e-2)
        _close(dv[:, :, h0 : h0 + 2], dv2, f"dv, kv heads {h0}, {h0 + 1}", tol=1e-2)


def test_chunked_order_with_a_batch_dimension(gpu):
    """Two batch elements of 8 heads are 16 (batch, head) combinations per tile level: chunked order again, now
    with a chunk boundary between the batch elements; each element alone (8 combinations) runs in plain order."""
    Dqk, Dv, B, heads = 128, 128, 2, 8
    g = torch.Generator().manual_seed(6)
    scale = Dqk**-0.5
    q = (torch.randn(B, S, heads, Dqk, generator=g) * scale).to(torch.bfloat16).to(gpu)
    k = (torch.randn(B, S, heads, Dqk, generator=g) * scale).to(torch.bfloat16).to(gpu)
    v = (torch.randn(B, S, heads, Dv, generator=g) * scale).to(torch.bfloat16).to(gpu)
    dout = torch.randn(B, S, heads, Dv, generator=g).to(torch.bfloat16).to(gpu)

    def run(qs, ks, vs, dos):
        o = torch.full(dos.shape, float("nan"), dtype=torch.bfloat16, device=gpu)
        lse = torch.full((qs.shape[0], heads, S), float("nan"), device=gpu)
        H.attn_fwd_into(qs, ks, vs, o, lse, scale, True)
        delta = torch.empty_like(lse)
        H.attn_bwd_delta_into(o, dos, delta)
        dq = torch.full(qs.shape, float("nan"), device=gpu)
        dk = torch.full(ks.shape, float("nan"), dtype=torch.bfloat16, device=gpu)
        dv = torch.full(vs.shape, float("nan"), dtype=torch.bfloat16, device=gpu)
        H.attn_bwd_dkdv_into(qs, ks, vs, dos, lse, delta, dk, dv, scale, True)
        H.attn_bwd_dq_into(qs, ks, vs, dos, lse, delta, dq, scale, True)
        return o, dq, dk, dv

    whole = run(q, k, v, dout)
    for b in range(B):
        part = run(*(t[b : b + 1] for t in (q, k, v, dout)))
        for name, w, p in zip(("o", "dq", "dk", "dv"), whole, part):
            _close(w[b : b + 1], p, f"{name}, batch element {b}")
