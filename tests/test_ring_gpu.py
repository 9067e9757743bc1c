"""One GPU's ring share (forward + backward through autograd) against full-sequence causal
attention, for every rank of the ring looped locally, in both token layouts.

Design, shapes, seed, the dO = ones loss and the 1 - cos < 1e-5 gate are those of the reference's
two-GPU tests (tests/test_ring_attention.py:48-106, tests/test_ring_mla_attention.py:61-134); the
ring there is split over real ranks, here rank r's work runs on one device and the sum over
r = 0..C-1 of the returned dK/dV is compared with the full-sequence gradient."""

import pytest
import torch

from helpers import check_bf16_result, check_lse, cosine_error
from oracle import ring_oracle as R
from pithtrain_amd.operators.ring_attention.local import (
    ring_attention_local,
    ring_forward_local,
    zigzag_merge,
    zigzag_split,
)
from pithtrain_amd.operators.ring_attention.mla import ring_mla_attention_func
from pithtrain_amd.operators.ring_attention.standard import ring_attention_func

pytestmark = pytest.mark.gpu

CONFIGS = [  # B, S, H, Hkv, DQ, DV, C
    pytest.param(1, 128, 4, 4, 64, 64, 2, id="MHA S=128"),
    pytest.param(2, 256, 8, 2, 64, 64, 2, id="GQA S=256"),
    pytest.param(1, 512, 12, 4, 128, 128, 2, id="GQA S=512 D=128"),
    pytest.param(1, 256, 16, 16, 192, 128, 2, id="MLA S=256"),
    pytest.param(2, 512, 16, 16, 192, 128, 2, id="MLA S=512 B=2"),
    pytest.param(1, 1024, 16, 16, 192, 128, 2, id="MLA S=1024"),
    pytest.param(1, 2048, 8, 2, 128, 128, 4, id="GQA S=2048 C=4"),
    pytest.param(1, 1536, 4, 4, 192, 128, 3, id="MLA S=1536 C=3"),
]


def _full_reference(q, k, v, dout, scale):
    o, lse = R.chunk_fwd(q, k, v, scale, True)
    dq, dk, dv = R.chunk_bwd(q, k, v, dout, lse, R.bwd_delta(o, dout), scale, True)
    return o, lse, dq, dk, dv


@pytest.mark.parametrize("layout", ["contiguous", "zigzag"])
@pytest.mark.parametrize("B,S,H,Hkv,DQ,DV,C", CONFIGS)
def test_forward_backward(gpu, layout, B, S, H, Hkv, DQ, DV, C):
    scale = DQ**-0.5
    torch.manual_seed(42)
    q_full = torch.randn(B, S, H, DQ, dtype=torch.bfloat16)
    k_full = torch.randn(B, S, Hkv, DQ, dtype=torch.bfloat16)
    v_full = torch.randn(B, S, Hkv, DV, dtype=torch.bfloat16)
    dout = torch.ones(B, S, H, DV, dtype=torch.bfloat16)  # loss = out.sum()
    o_ref, lse_ref, dq_ref, dk_ref, dv_ref = _full_reference(q_full, k_full, v_full, dout, scale)

    split = (lambda t: zigzag_split(t, C)) if layout == "zigzag" else (lambda t: [c.contiguous() for c in t.chunk(C, 1)])
    k_chunks = [c.to(gpu).requires_grad_(True) for c in split(k_full)]
    v_chunks = [c.to(gpu).requires_grad_(True) for c in split(v_full)]
    dk_sum = [torch.zeros(c.shape, dtype=torch.float32) for c in k_chunks]
    dv_sum = [torch.zeros(c.shape, dtype=torch.float32) for c in v_chunks]
    for r in range(C):
        pos = R.token_positions(r, C, S // C, layout)
        q_chunk = split(q_full)[r].to(gpu).requires_grad_(True)
        for t in k_chunks + v_chunks:
            t.grad = None
        out_ring = ring_attention_local(q_chunk, k_chunks, v_chunks, scale, r, C, layout)
        out_ring.sum().backward()
        assert cosine_error(out_ring, o_ref[:, pos]) < 1e-5
        assert cosine_error(q_chunk.grad, dq_ref[:, pos]) < 1e-5
        check_bf16_result(out_ring, o_ref[:, pos], f"rank {r} O")
        check_bf16_result(q_chunk.grad, dq_ref[:, pos], f"rank {r} dQ", otol=1e-3)
        for j in range(C):
            if k_chunks[j].grad is not None:
                dk_sum[j] += k_chunks[j].grad.float().cpu()
                dv_sum[j] += v_chunks[j].grad.float().cpu()
        if layout == "contiguous":  # chunks of higher ranks are never visited
            assert all(k_chunks[j].grad is None for j in range(r + 1, C))
    for j in range(C):
        pos = R.token_positions(j, C, S // C, layout)
        assert cosine_error(dk_sum[j], dk_ref[:, pos]) < 1e-5
        assert cosine_error(dv_sum[j], dv_ref[:, pos]) < 1e-5
        check_bf16_result(dk_sum[j], dk_ref[:, pos], f"chunk {j} dK", otol=1e-3)
        check_bf16_result(dv_sum[j], dv_ref[:, pos], f"chunk {j} dV", otol=1e-3)


@pytest.mark.parametrize("layout", ["contiguous", "zigzag"])
def test_ring_lse_is_base2_and_global(gpu, layout):
    B, S, H, Hkv, D, C = 1, 1024, 8, 2, 128, 4
    torch.manual_seed(0)
    q, k, v = (torch.randn(B, S, h, D, dtype=torch.bfloat16) for h in (H, Hkv, Hkv))
    scale = D**-0.5
    _, lse_ref = R.chunk_fwd(q, k, v, scale, True)
    split = (lambda t: zigzag_split(t, C)) if layout == "zigzag" else (lambda t: [c.contiguous() for c in t.chunk(C, 1)])
    ks, vs = [c.to(gpu) for c in split(k)], [c.to(gpu) for c in split(v)]
    for r in range(C):
        out, lse = ring_forward_local(split(q)[r].to(gpu), ks, vs, scale, r, C, layout)
        check_lse(lse, lse_ref[:, :, R.token_positions(r, C, S // C, layout)], f"rank {r} LSE2")
        oo, ol = R.ring_forward(split(q)[r], split(k), split(v), scale, r, C, layout)
        check_bf16_result(out, oo, f"rank {r} O vs oracle ring")


def test_zigzag_split_roundtrip():
    x = torch.arange(2 * 24 * 3).reshape(2, 24, 3)
    for C in (1, 2, 3, 4):
        assert torch.equal(zigzag_merge(zigzag_split(x, C)), x)
        assert [c.tolist() for c in zigzag_split(x, C)] == [c.tolist() for c in R.zigzag_split(x, C)]


@pytest.mark.parametrize("rerotate", [False, True])
def test_reference_entry_points_with_a_group_of_one(gpu, rerotate):
    """ring_attention_func / ring_mla_attention_func keep the reference's positional signature;
    with cp_group=None (a context-parallel group of one) they are plain causal attention.
    rerotate=True takes the backward whose dK/dV go through an fp32 accumulator that the kernel
    adds to (the form that travels around a real ring)."""
    for fn, (H, Hkv, DQ, DV) in ((ring_attention_func, (8, 2, 128, 128)), (ring_mla_attention_func, (4, 4, 192, 128))):
        B, S = 2, 320
        torch.manual_seed(1)
        q = torch.randn(B, S, H, DQ, dtype=torch.bfloat16)
        k = torch.randn(B, S, Hkv, DQ, dtype=torch.bfloat16)
        v = torch.randn(B, S, Hkv, DV, dtype=torch.bfloat16)
        dout = torch.randn(B, S, H, DV, dtype=torch.bfloat16)
        scale = DQ**-0.5
        qd, kd, vd = (t.to(gpu).requires_grad_(True) for t in (q, k, v))
        out = fn(qd, kd, vd, scale, None, rerotate=rerotate)
        out.backward(dout.to(gpu))
        o_ref, lse_ref, dq_ref, dk_ref, dv_ref = _full_reference(q, k, v, dout, scale)
        check_bf16_result(out, o_ref, "O")
        check_bf16_result(qd.grad, dq_ref, "dQ", otol=1e-3)
        check_bf16_result(kd.grad, dk_ref, "dK", otol=1e-3)
        check_bf16_result(vd.grad, dv_ref, "dV", otol=1e-3)


@pytest.fixture
def one_rank_group(tmp_path):
    """A real torch.distributed ProcessGroup with a single member (file rendezvous, gloo): the object the
    model code hands to ring_attention_func. A ring of one issues no collective."""
    import torch.distributed as dist

    assert not dist.is_initialized()
    dist.init_process_group("gloo", init_method=f"file://{tmp_path}/rendezvous", rank=0, world_size=1)
    try:
        yield dist.new_group([0])
    finally:
        dist.destroy_process_group()


def test_reference_entry_points_with_a_process_group(gpu, one_rank_group):
    """Positional call exactly as the reference's layers make it (qwen3_30b_a3b.py:432-438,
    deepseek_v2_lite.py:456-465): ring_attention_func(q, k, v, softmax_scale, cp_group) with a
    ProcessGroup object, so that cp_group.rank() / size() / get_global_rank are exercised on the GPU path."""
    assert one_rank_group.size() == 1 and one_rank_group.rank() == 0
    for fn, (H, Hkv, DQ, DV) in ((ring_attention_func, (8, 2, 128, 128)), (ring_mla_attention_func, (4, 4, 192, 128))):
        B, S = 1, 384
        torch.manual_seed(3)
        q = torch.randn(B, S, H, DQ, dtype=torch.bfloat16)
        k = torch.randn(B, S, Hkv, DQ, dtype=torch.bfloat16)
        v = torch.randn(B, S, Hkv, DV, dtype=torch.bfloat16)
        dout = torch.randn(B, S, H, DV, dtype=torch.bfloat16)
        scale = DQ**-0.5
        qd, kd, vd = (t.to(gpu).requires_grad_(True) for t in (q, k, v))
        out = fn(qd, kd, vd, scale, one_rank_group)
        out.backward(dout.to(gpu))
        o_ref, lse_ref, dq_ref, dk_ref, dv_ref = _full_reference(q, k, v, dout, scale)
        check_bf16_result(out, o_ref, "O")
        check_bf16_result(qd.grad, dq_ref, "dQ", otol=1e-3)
        check_bf16_result(kd.grad, dk_ref, "dK", otol=1e-3)
        check_bf16_result(vd.grad, dv_ref, "dV", otol=1e-3)


def test_autograd_functions_with_the_references_seven_arguments(gpu):
    """RingAttentionFunc.apply / RingMLAAttentionFunc.apply called with exactly the reference's seven positional
    arguments (q, k, v, softmax_scale, cp_rank, cp_size, global_ranks: standard.py:73, mla.py:47); the backward
    returns seven gradients (standard.py:189, mla.py:149): dq, dk, dv and four None."""
    from pithtrain_amd.operators.ring_attention.mla import RingMLAAttentionFunc
    from pithtrain_amd.operators.ring_attention.standard import RingAttentionFunc

    for base, (H, Hkv, DQ, DV) in ((RingAttentionFunc, (8, 2, 128, 128)), (RingMLAAttentionFunc, (4, 4, 192, 128))):
        returned = []

        class Probe(base):
            @staticmethod
            def backward(ctx, dout):
                grads = base.backward(ctx, dout)
                returned.append(grads)
                return grads

        B, S = 2, 320
        torch.manual_seed(5)
        q = torch.randn(B, S, H, DQ, dtype=torch.bfloat16)
        k = torch.randn(B, S, Hkv, DQ, dtype=torch.bfloat16)
        v = torch.randn(B, S, Hkv, DV, dtype=torch.bfloat16)
        dout = torch.randn(B, S, H, DV, dtype=torch.bfloat16)
        scale = DQ**-0.5
        qd, kd, vd = (t.to(gpu).requires_grad_(True) for t in (q, k, v))
        out = Probe.apply(qd, kd, vd, scale, 0, 1, [0])
        assert out.dtype == torch.bfloat16 and tuple(out.shape) == (B, S, H, DV)
        out.backward(dout.to(gpu))
        (grads,) = returned
        assert len(grads) == 7 and all(g is None for g in grads[3:]), "backward must return the reference's 7-tuple"
        o_ref, lse_ref, dq_ref, dk_ref, dv_ref = _full_reference(q, k, v, dout, scale)
        check_bf16_result(out, o_ref, "O")
        check_bf16_result(qd.grad, dq_ref, "dQ", otol=1e-3)
        check_bf16_result(kd.grad, dk_ref, "dK", otol=1e-3)
        check_bf16_result(vd.grad, dv_ref, "dV", otol=1e-3)
