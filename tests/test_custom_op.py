"""The single-device attention entry points (custom ops): shape propagation without a GPU, and
parity / torch.compile on the GPU. The reference wraps its launches as custom ops so that layers
compiled with fullgraph=True keep working (pithtrain/operators/mla/triton.py:445-508); the
non-context-parallel call it replaces is flash_attn_func at pithtrain/models/qwen3_30b_a3b.py:424-430."""

import pytest
import torch

from pithtrain_amd.operators.mla import MLA
from pithtrain_amd.operators.mla.hip import attention_func


def _meta(*shape):
    return torch.empty(*shape, dtype=torch.bfloat16, device="meta", requires_grad=True)


def test_fake_implementations_propagate_shapes():
    q, k, v = _meta(2, 64, 8, 128), _meta(2, 96, 2, 128), _meta(2, 96, 2, 128)
    o = attention_func(q, k, v, None, False)
    assert o.shape == (2, 64, 8, 128) and o.dtype == torch.bfloat16
    o.sum().backward()
    assert q.grad.shape == q.shape and k.grad.shape == k.shape and v.grad.shape == v.shape


def test_fullgraph_compile_traces_through_the_ops():
    m = MLA(4, 192, 128)
    f = torch.compile(lambda q, k, v: m(q, k, v) * 2, backend="aot_eager", fullgraph=True)
    q, k, v = _meta(1, 64, 4, 192), _meta(1, 64, 4, 192), _meta(1, 64, 4, 128)
    o = f(q, k, v)
    assert o.shape == (1, 64, 4, 128)
    o.sum().backward()
    assert q.grad.shape == q.shape and v.grad.shape == v.shape


def test_cpu_tensors_are_refused():
    x = torch.zeros(1, 4, 2, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="need tensors on a GPU"):
        attention_func(x, x, x)


@pytest.mark.gpu
@pytest.mark.parametrize("causal,sq,skv", [(True, 384, 384), (False, 256, 640)])
def test_attention_func_matches_oracle(gpu, causal, sq, skv):
    from helpers import check_bf16_result
    from oracle import ring_oracle as R

    g = torch.Generator().manual_seed(7)
    q = torch.randn(1, sq, 8, 128, generator=g).to(torch.bfloat16)
    k = torch.randn(1, skv, 2, 128, generator=g).to(torch.bfloat16)
    v = torch.randn(1, skv, 2, 128, generator=g).to(torch.bfloat16)
    dout = torch.randn(1, sq, 8, 128, generator=g).to(torch.bfloat16)
    scale = 128**-0.5
    o_ref, lse_ref = R.chunk_fwd(q, k, v, scale, causal)
    delta = R.bwd_delta(o_ref, dout)
    dq_ref, dk_ref, dv_ref = R.chunk_bwd(q, k, v, dout, lse_ref, delta, scale, causal)

    qd, kd, vd = (t.to(gpu).requires_grad_() for t in (q, k, v))
    o = attention_func(qd, kd, vd, scale, causal)
    o.backward(dout.to(gpu))
    check_bf16_result(o.detach().cpu(), o_ref, "o")
    check_bf16_result(qd.grad.cpu(), dq_ref, "dq", otol=1e-3)
    check_bf16_result(kd.grad.cpu(), dk_ref, "dk", otol=1e-3)
    check_bf16_result(vd.grad.cpu(), dv_ref, "dv", otol=1e-3)


@pytest.mark.gpu
def test_compiled_module_matches_eager(gpu):
    m = MLA(16, 192, 128)
    g = torch.Generator().manual_seed(42)
    q = torch.randn(1, 512, 16, 192, generator=g).to(torch.bfloat16).to(gpu)
    k = torch.randn(1, 512, 16, 192, generator=g).to(torch.bfloat16).to(gpu)
    v = torch.randn(1, 512, 16, 128, generator=g).to(torch.bfloat16).to(gpu)
    f = torch.compile(m, backend="aot_eager", fullgraph=True)
    qa, ka, va = (t.clone().requires_grad_() for t in (q, k, v))
    qb, kb, vb = (t.clone().requires_grad_() for t in (q, k, v))
    oa, ob = m(qa, ka, va), f(qb, kb, vb)
    assert torch.equal(oa, ob)
    oa.float().square().sum().backward()
    ob.float().square().sum().backward()
    assert torch.equal(qa.grad, qb.grad) and torch.equal(ka.grad, kb.grad) and torch.equal(va.grad, vb.grad)
