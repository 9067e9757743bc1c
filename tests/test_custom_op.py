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


def test_prologue_fake_implementations_and_fullgraph_compile():
    """The q/k RMSNorm + rotary embedding ops trace without a GPU: a compiled attention layer's
    prologue + attention chain, shapes and gradients (weights included) on meta tensors."""
    from pithtrain_amd.operators.norm_rope import apply_rotary_pos_emb, qk_norm_rope

    def layer(q, k, v, wq, wk, cos, sin):
        q, k = qk_norm_rope(q, k, wq, wk, cos, sin, 1e-6)
        return attention_func(q, k, v, None, True)

    f = torch.compile(layer, backend="aot_eager", fullgraph=True)
    q, k, v = _meta(2, 64, 8, 128), _meta(2, 64, 2, 128), _meta(2, 64, 2, 128)
    wq, wk = _meta(128), _meta(128)
    cos = torch.empty(2, 64, 128, dtype=torch.bfloat16, device="meta")
    o = f(q, k, v, wq, wk, cos, cos)
    assert o.shape == (2, 64, 8, 128)
    o.sum().backward()
    assert q.grad.shape == q.shape and k.grad.shape == k.shape
    assert wq.grad.shape == (128,) and wq.grad.dtype == torch.bfloat16 and wk.grad.shape == (128,)
    rq, rk = apply_rotary_pos_emb(q.detach(), k.detach(), cos, cos)
    assert rq.shape == q.shape and rk.shape == k.shape


@pytest.mark.gpu
def test_compiled_prologue_matches_eager(gpu):
    from pithtrain_amd.operators.norm_rope import qk_norm_rope

    g = torch.Generator().manual_seed(3)
    mk = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16).to(gpu)  # noqa: E731
    q, k, wq, wk, cos, sin = mk(1, 200, 32, 128), mk(1, 200, 4, 128), mk(128), mk(128), mk(1, 200, 128), mk(1, 200, 128)
    f = torch.compile(qk_norm_rope, backend="aot_eager", fullgraph=True)
    a = [t.clone().requires_grad_() for t in (q, k, wq, wk)]
    b = [t.clone().requires_grad_() for t in (q, k, wq, wk)]
    qa, ka = qk_norm_rope(*a, cos, sin, 1e-6)
    qb, kb = f(*b, cos, sin, 1e-6)
    assert torch.equal(qa, qb) and torch.equal(ka, kb)
    (qa.float().square().sum() + ka.float().sum()).backward()
    (qb.float().square().sum() + kb.float().sum()).backward()
    for x, y in zip(a, b):
        assert torch.equal(x.grad, y.grad)
