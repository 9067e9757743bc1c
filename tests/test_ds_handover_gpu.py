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

    from pithtrain_amd.operators.mla import hip as H

    used = []
    real_plan = H.ds_plan

    def always(q, k, v, causal=False):  # the default policy would decline a share this small
        used.append(1)
        return k.shape[2], attn_bwd_ds_bytes(q, k, v, causal)

    monkeypatch.setattr(H, "ds_plan", always)
    dq1, dk1, dv1 = run()
    assert used, "the ring backward did not ask for a hand-over plan"
    monkeypatch.setattr(H, "ds_plan", lambda *a: None)
    dq0, dk0, dv0 = run()
    monkeypatch.setattr(H, "ds_plan", real_plan)
    for a, b in zip(dk0 + dv0, dk1 + dv1):
        assert (a is None and b is None) or torch.equal(a, b)
    assert norm_max_err(dq1.float().cpu(), dq0.float().cpu()) < 6e-3
    o_ref, lse_ref = R.ring_forward(qs[rank], ks, vs, scale, rank, C, layout)
    dq_ref, _, _ = R.ring_backward(dos[rank], qs[rank], o_ref, lse_ref, ks, vs, scale, rank, C, layout)
    check_bf16_result(dq1, dq_ref, "ring dQ", otol=1e-3)


def _shaped(gpu, b, s, hq, hkv):
    q = torch.empty(b, s, hq, 128, dtype=torch.bfloat16, device=gpu)
    k = torch.empty(b, s, hkv, 128, dtype=torch.bfloat16, device=gpu)
    return q, k, k


def test_default_policy_of_the_buffer(gpu, monkeypatch):
    """ds_plan takes the hand-over only when the dS-reading dQ kernel would fill the device, keeps the buffer
    under the configured limit and under a fraction of the free memory by going through the kv heads in slabs,
    and gives up (both kernels recompute) when not even one kv head fits."""
    from pithtrain_amd.operators.mla import hip as H

    assert H.DS_BUFFER_LIMIT_BYTES <= 4 << 30, "the default limit must stay modest"
    assert H.ds_plan(*_shaped(gpu, 1, 512, 8, 2)) is None  # 1 x 8 workgroups: too few
    big = _shaped(gpu, 1, 4096, 32, 4)  # 8 x 32 workgroups, 1 GiB
    assert attn_bwd_ds_bytes(*big) == 1 << 30
    assert H.ds_plan(*big) == (4, 1 << 30)
    buf = ds_buffer(*big)
    assert buf is not None and buf.numel() == 1 << 30 and buf.data_ptr() % 256 == 0
    del buf
    monkeypatch.setattr(H, "DS_BUFFER_LIMIT_BYTES", (1 << 30) - 1)
    assert H.ds_plan(*big) is None and ds_buffer(*big) is None  # slabs of 2 kv heads: 8 x 16 workgroups, too few
    # 16384 x 16384 rows, 32 / 4 heads: 4 GiB per kv head, 32 x 8 workgroups of the dQ kernel per kv head
    q = torch.empty(1, dtype=torch.bfloat16, device=gpu).as_strided((1, 16384, 32, 128), (0, 0, 0, 0))
    k = torch.empty(1, dtype=torch.bfloat16, device=gpu).as_strided((1, 16384, 4, 128), (0, 0, 0, 0))
    monkeypatch.setattr(H, "DS_BUFFER_LIMIT_BYTES", 16 << 30)
    assert H.ds_plan(q, k, k) == (4, 16 << 30)
    monkeypatch.setattr(H, "DS_BUFFER_LIMIT_BYTES", (16 << 30) - 1)
    assert H.ds_plan(q, k, k) == (2, 8 << 30) and ds_buffer(q, k, k) is None  # two slabs of two kv heads
    monkeypatch.setattr(H, "DS_BUFFER_LIMIT_BYTES", (4 << 30) + 5)
    assert H.ds_plan(q, k, k) == (1, 4 << 30)
    monkeypatch.setattr(H, "DS_BUFFER_LIMIT_BYTES", (4 << 30) - 1)
    assert H.ds_plan(q, k, k) is None
    # the 131072-token configuration (64 / 4 heads, 16384 x 8192 rows per ring step): one kv head at a time
    monkeypatch.setattr(H, "DS_BUFFER_LIMIT_BYTES", 4 << 30)
    q64 = torch.empty(1, dtype=torch.bfloat16, device=gpu).as_strided((1, 16384, 64, 128), (0, 0, 0, 0))
    k8k = torch.empty(1, dtype=torch.bfloat16, device=gpu).as_strided((1, 8192, 4, 128), (0, 0, 0, 0))
    assert H.ds_plan(q64, k8k, k8k) == (1, 4 << 30)
    # little free memory: the budget follows it
    monkeypatch.setattr(H, "DS_BUFFER_LIMIT_BYTES", 16 << 30)
    monkeypatch.setattr(H.torch.cuda, "mem_get_info", lambda dev=None: (8 << 30, 1 << 38))
    monkeypatch.setattr(H.torch.cuda, "memory_reserved", lambda dev=None: 0)
    monkeypatch.setattr(H.torch.cuda, "memory_allocated", lambda dev=None: 0)
    assert H.ds_plan(q, k, k) == (1, 4 << 30)


@pytest.mark.parametrize("causal", [False, True])
def test_slabs_of_kv_heads_equal_the_whole_call(gpu, causal, monkeypatch):
    """attn_bwd_pair_into through a buffer that holds one or two kv heads at a time (head ranges of the full
    tensors, passed in place) gives dK/dV bit for bit and dQ bit for bit what the whole-pair hand-over gives."""
    from pithtrain_amd.operators.mla import hip as H

    B, Sq, Hq, Hkv = 2, 1024, 16, 4
    Skv = Sq if causal else 640
    q, k, v, dout, scale = _inputs(B, Sq, Skv, Hq, Hkv, seed=11)
    qd, kd, vd, dod = (t.to(gpu) for t in (q, k, v, dout))
    o, lse = _mla_fwd(qd, kd, vd, scale, causal)
    delta = _mla_bwd_preprocess(o, dod)
    need = attn_bwd_ds_bytes(qd, kd, vd, causal)
    results = []
    for heads in (4, 2, 1):
        monkeypatch.setattr(H, "ds_plan", lambda *a, heads=heads: (heads, need // Hkv * heads))
        dq = torch.full(qd.shape, 0.25, dtype=torch.float32, device=gpu)
        dk, dv = torch.empty_like(kd), torch.empty_like(vd)
        used = H.attn_bwd_pair_into(qd, kd, vd, dod, lse, delta, dq, dk, dv, scale, causal, accumulate_dq=True)
        assert used == need // Hkv * heads
        results.append((dq, dk, dv))
    for dq, dk, dv in results[1:]:
        assert torch.equal(dq, results[0][0]) and torch.equal(dk, results[0][1]) and torch.equal(dv, results[0][2])
    rdq, rdk, rdv = R.chunk_bwd(q, k, v, dout, lse.double().cpu(), delta.double().cpu(), scale, causal)
    check_bf16_result(results[2][0] - 0.25, rdq, "slab dQ", otol=1e-3)
    check_bf16_result(results[2][1], rdk, "slab dK", otol=1e-3)
    check_bf16_result(results[2][2], rdv, "slab dV", otol=1e-3)


def test_head_range_calls_without_handover(gpu):
    """The recomputing kernels accept a head range of wider tensors too (all three head-dim families)."""
    for d_q, d_v in ((128, 128), (192, 128), (64, 64)):
        B, S, Hq, Hkv = 1, 320, 8, 4
        g = torch.Generator().manual_seed(5)
        q = (torch.randn(B, S, Hq, d_q, generator=g) * d_q**-0.5).to(torch.bfloat16).to(gpu)
        k = (torch.randn(B, S, Hkv, d_q, generator=g) * d_q**-0.5).to(torch.bfloat16).to(gpu)
        v = torch.randn(B, S, Hkv, d_v, generator=g).to(torch.bfloat16).to(gpu)
        dout = torch.randn(B, S, Hq, d_v, generator=g).to(torch.bfloat16).to(gpu)
        scale = d_q**-0.5
        o, lse = _mla_fwd(q, k, v, scale, True)
        delta = _mla_bwd_preprocess(o, dout)
        dq0, dk0, dv0 = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        from pithtrain_amd.operators.mla import hip as H_

        H_.attn_bwd_pair_into(q, k, v, dout, lse, delta, dq0, dk0, dv0, scale, True, handover=False)
        dq1, dk1, dv1 = torch.zeros_like(q), torch.zeros_like(k), torch.zeros_like(v)
        for h0 in range(0, Hkv, 2):
            kv_h, q_h = slice(h0, h0 + 2), slice(2 * h0, 2 * h0 + 4)
            H_.attn_bwd_pair_into(q[:, :, q_h], k[:, :, kv_h], v[:, :, kv_h], dout[:, :, q_h], lse[:, q_h], delta[:, q_h],
                                  dq1[:, :, q_h], dk1[:, :, kv_h], dv1[:, :, kv_h], scale, True, handover=False)  # fmt: skip
        assert torch.equal(dq0, dq1) and torch.equal(dk0, dk1) and torch.equal(dv0, dv1), (d_q, d_v)


def test_allocation_failure_falls_back_to_recomputation(gpu, monkeypatch):
    """When the hand-over buffer cannot be allocated the pair recomputes: dK/dV bit-identical to the hand-over
    path (the dK/dV kernel's arithmetic does not depend on the stores), dQ within oracle parity."""
    from pithtrain_amd.operators.mla import hip as H

    B, Sq, Skv, Hq, Hkv = 1, 1024, 768, 8, 2
    q, k, v, dout, scale = _inputs(B, Sq, Skv, Hq, Hkv, seed=3)
    qd, kd, vd, dod = (t.to(gpu) for t in (q, k, v, dout))
    o, lse = _mla_fwd(qd, kd, vd, scale, False)
    delta = _mla_bwd_preprocess(o, dod)
    monkeypatch.setattr(H, "ds_plan", lambda *a: (Hkv, attn_bwd_ds_bytes(qd, kd, vd, False)))
    need = attn_bwd_ds_bytes(qd, kd, vd, False)
    real_empty = torch.empty

    def failing_empty(*a, **kw):  # only the hand-over buffer's allocation fails
        if a and a[0] == need and kw.get("dtype") == torch.uint8:
            raise torch.cuda.OutOfMemoryError("forced by the test")
        return real_empty(*a, **kw)

    out = {}
    for name in ("handover", "oom"):
        with monkeypatch.context() as m:
            if name == "oom":
                m.setattr(torch, "empty", failing_empty)
            dq, dk, dv = torch.empty_like(qd), torch.empty_like(kd), torch.empty_like(vd)
            used = H.attn_bwd_pair_into(qd, kd, vd, dod, lse, delta, dq, dk, dv, scale, False)
        out[name] = (dq, dk, dv, used)
    assert out["handover"][3] > 0 and out["oom"][3] == 0
    assert torch.equal(out["handover"][1], out["oom"][1]) and torch.equal(out["handover"][2], out["oom"][2])
    rdq, _, _ = R.chunk_bwd(q, k, v, dout, lse.double().cpu(), delta.double().cpu(), scale, False)
    check_bf16_result(out["oom"][0], rdq, "recomputed dQ after allocation failure", otol=1e-3)
    check_bf16_result(out["handover"][0], rdq, "hand-over dQ", otol=1e-3)
