"""dS hand-over between the two backward kernels of one chunk pair (head dims 128/128): with a `ds`
buffer the dK/dV kernel stores the dS tiles it forms and the dQ kernel computes dQ = scale * dS K from
them instead of recomputing S and dP (pithtrain/operators/mla/triton.py:205-266 recomputes). Expected
values come from the fp64 oracle; the recomputing dQ kernel is compared as well (the same bf16 dS values
summed in another order), and dK/dV must not change by a bit when the tiles are also stored."""

import pytest
import torch

from helpers import check_bf16_result, norm_max_err
from oracle import ring_oracle as R
from pithtrain_amd.operators.mla.hip import (
    _mla_bwd_preprocess,
    _mla_fwd,
    attn_bwd_dkdv_into,
    attn_bwd_dq_into,
    attn_bwd_ds_bytes,
    ds_buffer,
)
from pithtrain_amd.operators.ring_attention.local import ring_attention_local

pytestmark = pytest.mark.gpu

SHAPES = [
    # B, Sq, Skv, Hq, Hkv
    (1, 256, 256, 4, 4),
    (1, 512, 512, 8, 2),
    (2, 384, 384, 4, 1),
    (1, 333, 333, 4, 2),      # ragged last query tile and key block
    (1, 1000, 1000, 2, 1),
    (1, 2048, 2048, 16, 2),   # head split of the dK/dV kernel
    (1, 65, 65, 2, 2),        # one row beyond a query tile: two tiles, one key block
    (1, 129, 129, 4, 1),      # one row beyond a key block
    (2, 777, 777, 8, 2),
]
NONCAUSAL_SHAPES = SHAPES + [(1, 512, 256, 8, 2), (1, 256, 768, 4, 4), (1, 200, 450, 4, 2), (1, 65, 129, 2, 2)]


def _inputs(B, Sq, Skv, Hq, Hkv, seed=42, dqk=128):
    g = torch.Generator().manual_seed(seed)
    scale = dqk**-0.5
    q = (torch.randn(B, Sq, Hq, dqk, generator=g) * scale).to(torch.bfloat16)
    k = (torch.randn(B, Skv, Hkv, dqk, generator=g) * scale).to(torch.bfloat16)
    v = (torch.randn(B, Skv, Hkv, 128, generator=g) * scale).to(torch.bfloat16)
    dout = torch.randn(B, Sq, Hq, 128, generator=g).to(torch.bfloat16)
    return q, k, v, dout, scale


def _run(gpu, causal, shape, dq_dtype, dqk=128):
    q, k, v, dout, scale = _inputs(*shape, dqk=dqk)
    qd, kd, vd, dod = (t.to(gpu) for t in (q, k, v, dout))
    o, lse = _mla_fwd(qd, kd, vd, scale, causal)
    delta = _mla_bwd_preprocess(o, dod)
    o_ref, lse_ref = R.chunk_fwd(q, k, v, scale, causal)
    dq_ref, dk_ref, dv_ref = R.chunk_bwd(q, k, v, dout, lse_ref, R.bwd_delta(o_ref, dout), scale, causal)

    dk0, dv0 = torch.empty_like(kd), torch.empty_like(vd)
    dq0 = torch.empty(qd.shape, dtype=dq_dtype, device=gpu)
    attn_bwd_dkdv_into(qd, kd, vd, dod, lse, delta, dk0, dv0, scale, causal)
    attn_bwd_dq_into(qd, kd, vd, dod, lse, delta, dq0, scale, causal)

    need = attn_bwd_ds_bytes(qd, kd, vd, causal)
    n_qt, n_kb = (shape[1] + 63) // 64, (shape[2] + 127) // 128
    # 16 KB per (64-row query tile, 128-key block); under the mask tile t keeps its first t // 2 + 1 key blocks
    blocks = sum(t // 2 + 1 for t in range(n_qt)) if causal else n_qt * n_kb
    assert need == shape[0] * shape[3] * blocks * 16384
    # poisoned buffer: whatever the dQ kernel reads must have been written by the dK/dV kernel
    ds = torch.full((need,), 0x7F, dtype=torch.uint8, device=gpu)
    dk1, dv1 = torch.empty_like(kd), torch.empty_like(vd)
    dq1 = torch.empty(qd.shape, dtype=dq_dtype, device=gpu)
    attn_bwd_dkdv_into(qd, kd, vd, dod, lse, delta, dk1, dv1, scale, causal, ds=ds)
    attn_bwd_dq_into(qd, kd, vd, dod, lse, delta, dq1, scale, causal, ds=ds)
    torch.cuda.synchronize()
    assert torch.equal(dk0, dk1) and torch.equal(dv0, dv1), "storing dS changed dK/dV"
    check_bf16_result(dq1, dq_ref, "dQ from dS", otol=1e-3)
    # two bf16 results of the same sums in different orders: up to one bf16 step (2^-8) of the largest element
    assert norm_max_err(dq1.float().cpu(), dq0.float().cpu()) < 6e-3, "dQ from dS vs recomputing kernel"
    return qd, kd, vd, dod, lse, delta, dq1, ds, scale


@pytest.mark.parametrize("shape", SHAPES)
def test_causal_dq_from_ds(gpu, shape):
    _run(gpu, True, shape, torch.bfloat16)


@pytest.mark.parametrize("shape", NONCAUSAL_SHAPES)
def test_noncausal_dq_from_ds(gpu, shape):
    _run(gpu, False, shape, torch.bfloat16)


@pytest.mark.parametrize("causal", [True, False])
def test_fp32_output_and_accumulation(gpu, causal):
    qd, kd, vd, dod, lse, delta, dq1, ds, scale = _run(gpu, causal, (1, 512, 512, 8, 2), torch.float32)
    acc = torch.full_like(dq1, 0.25)
    attn_bwd_dq_into(qd, kd, vd, dod, lse, delta, acc, scale, causal, accumulate=True, ds=ds)
    assert torch.equal(acc, dq1 + 0.25)


def test_small_buffer_falls_back_to_recomputation(gpu):
    q, k, v, dout, scale = _inputs(1, 256, 256, 4, 4)
    qd, kd, vd, dod = (t.to(gpu) for t in (q, k, v, dout))
    o, lse = _mla_fwd(qd, kd, vd, scale, True)
    delta = _mla_bwd_preprocess(o, dod)
    dq0, dq1 = torch.empty_like(qd), torch.empty_like(qd)
    attn_bwd_dq_into(qd, kd, vd, dod, lse, delta, dq0, scale, True)
    small = torch.zeros(attn_bwd_ds_bytes(qd, kd, vd, True) - 1024, dtype=torch.uint8, device=gpu)
    attn_bwd_dq_into(qd, kd, vd, dod, lse, delta, dq1, scale, True, ds=small)
    assert torch.equal(dq0, dq1)
    # head dims without a hand-over path report 0 bytes and get no buffer
    for d in (64, 192):
        qx = torch.empty(1, 128, 4, d, dtype=torch.bfloat16, device=gpu)
        vx = torch.empty(1, 128, 4, min(d, 128), dtype=torch.bfloat16, device=gpu)
        assert attn_bwd_ds_bytes(qx, qx, vx) == 0 and ds_buffer(qx, qx, vx) is None


@pytest.mark.parametrize("layout", ["contiguous", "zigzag"])
def test_ring_share_uses_the_handover(gpu, layout, monkeypatch):
    """The ring backward with the hand-over equals the ring backward without it (dK/dV bit for bit, dQ up to
    summation order) and the oracle's ring share."""
    from pithtrain_amd.operators.ring_attention import local as L

    B, S, Hq, Hkv, C, rank = 1, 2048, 8, 2, 4, 1
    q_full, k_full, v_full, dout_full, scale = _inputs(B, S, S, Hq, Hkv, seed=7)
    split = (lambda x: R.zigzag_split(x, C)) if layout == "zigzag" else (lambda x: list(x.chunk(C, 1)))
    qs, ks, vs, dos = (split(t) for t in (q_full, k_full, v_full, dout_full))

    def run():
        q = qs[rank].to(gpu).requires_grad_(True)
        kc = [t.to(gpu).requires_grad_(True) for t in ks]
        vc = [t.to(gpu).requires_grad_(True) for t in vs]
        out = ring_attention_local(q, kc, vc, scale, rank, C, layout)
        out.backward(dos[rank].to(gpu))
        return q.grad, [t.grad for t in kc], [t.grad for t in vc]

    calls = []

    def always(q, k, v, causal=False):  # the default policy would decline a share this small
        calls.append(1)
        return torch.empty(attn_bwd_ds_bytes(q, k, v, causal), dtype=torch.uint8, device=q.device)

    monkeypatch.setattr(L, "ds_buffer", always)
    dq1, dk1, dv1 = run()
    assert calls, "the ring backward did not ask for a hand-over buffer"
    monkeypatch.setattr(L, "ds_buffer", lambda *a: None)
    dq0, dk0, dv0 = run()
    for a, b in zip(dk0 + dv0, dk1 + dv1):
        assert (a is None and b is None) or torch.equal(a, b)
    assert norm_max_err(dq1.float().cpu(), dq0.float().cpu()) < 6e-3
    o_ref, lse_ref = R.ring_forward(qs[rank], ks, vs, scale, rank, C, layout)
    dq_ref, _, _ = R.ring_backward(dos[rank], qs[rank], o_ref, lse_ref, ks, vs, scale, rank, C, layout)
    check_bf16_result(dq1, dq_ref, "ring dQ", otol=1e-3)


def test_default_policy_of_the_buffer(gpu, monkeypatch):
    """ds_buffer hands out a buffer only when it stays under the size limit and the dS-reading dQ kernel
    would fill the device; otherwise the ring backward recomputes."""
    from pithtrain_amd.operators.mla import hip as H

    def shaped(b, s, hq, hkv):
        q = torch.empty(b, s, hq, 128, dtype=torch.bfloat16, device=gpu)
        k = torch.empty(b, s, hkv, 128, dtype=torch.bfloat16, device=gpu)
        return q, k, k

    assert ds_buffer(*shaped(1, 512, 8, 2)) is None  # 1 x 8 workgroups: too few
    big = shaped(1, 4096, 32, 4)  # 8 x 32 workgroups, 1 GiB
    assert attn_bwd_ds_bytes(*big) == 1 << 30
    buf = ds_buffer(*big)
    assert buf is not None and buf.numel() == 1 << 30 and buf.data_ptr() % 256 == 0
    del buf
    monkeypatch.setattr(H, "DS_BUFFER_LIMIT_BYTES", (1 << 30) - 1)
    assert ds_buffer(*big) is None
