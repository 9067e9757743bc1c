"""Keys in two parts (the MLA layer's k_nope [B,S,H,128] and the rotary k_pe [B,S,64] shared by all heads,
pithtrain/models/deepseek_v2_lite.py:448-454): the chunk kernels and the ring share must give what the
assembled 192-feature key gives. Expected values come from the oracle on the assembled key
(dk_nope = dk[..., :128], dk_pe = sum over heads of dk[..., 128:]); the assembled-key path of the
library is compared as well (same kernels reading the same numbers: O, LSE, dQ, dk_nope, dV bit for bit)."""

import pytest
import torch

from helpers import check_bf16_result, check_lse
from oracle import ring_oracle as R
from pithtrain_amd.operators.mla.hip import _mla_bwd_dk_dv, _mla_bwd_dq, _mla_bwd_preprocess, _mla_fwd
from pithtrain_amd.operators.ring_attention.local import ring_attention_local

pytestmark = pytest.mark.gpu


def _parts(B, S, H, seed):
    g = torch.Generator().manual_seed(seed)
    scale = 192**-0.5
    k_nope = (torch.randn(B, S, H, 128, generator=g) * scale).to(torch.bfloat16)
    # k_pe as the model has it: a column slice of a wider projection output ([b, s, 512 + 64])
    wide = (torch.randn(B, S, 576, generator=g) * scale).to(torch.bfloat16)
    v = (torch.randn(B, S, H, 128, generator=g) * scale).to(torch.bfloat16)
    return k_nope, wide, v


def _assemble(k_nope, k_pe):
    return torch.cat([k_nope, k_pe.unsqueeze(2).expand(-1, -1, k_nope.shape[2], -1)], -1).contiguous()


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("B,Sq,Skv,H", [(1, 512, 512, 16), (2, 1024, 1024, 16), (1, 333, 333, 4), (1, 4096, 4096, 16)])
def test_chunk_kernels_with_keys_in_two_parts(gpu, causal, B, Sq, Skv, H):
    scale = 192**-0.5
    g = torch.Generator().manual_seed(42)
    q = (torch.randn(B, Sq, H, 192, generator=g) * scale).to(torch.bfloat16)
    dout = torch.randn(B, Sq, H, 128, generator=g).to(torch.bfloat16)
    k_nope, wide, v = _parts(B, Skv, H, 43)
    k_pe = wide[..., 512:]
    k_full = _assemble(k_nope, k_pe)
    qd, dod, knd, wided, vd, kfd = (t.to(gpu) for t in (q, dout, k_nope, wide, v, k_full))
    kped = wided[..., 512:]  # strided view: row stride 576

    o, lse = _mla_fwd(qd, knd, vd, scale, causal, k_pe=kped)
    o_ref, lse_ref = R.chunk_fwd(q, k_full, v, scale, causal)
    check_bf16_result(o, o_ref, "O")
    check_lse(lse, lse_ref, "LSE2")
    o_full, lse_full = _mla_fwd(qd, kfd, vd, scale, causal)
    assert torch.equal(o, o_full) and torch.equal(lse, lse_full)

    delta = _mla_bwd_preprocess(o, dod)
    dk_nope, dv, dk_pe = _mla_bwd_dk_dv(qd, knd, vd, dod, lse, delta, scale, causal, k_pe=kped)
    dq = _mla_bwd_dq(qd, knd, vd, dod, lse, delta, scale, causal, k_pe=kped)
    dq_ref, dk_ref, dv_ref = R.chunk_bwd(q, k_full, v, dout, lse_ref, R.bwd_delta(o_ref, dout), scale, causal)
    check_bf16_result(dq, dq_ref, "dQ", otol=1e-3)
    check_bf16_result(dv, dv_ref, "dV", otol=1e-3)
    check_bf16_result(dk_nope, dk_ref[..., :128], "dK nope", otol=1e-3)
    check_bf16_result(dk_pe, dk_ref[..., 128:].sum(2), "dK pe (summed over heads)", otol=1e-3)
    dk_full, dv_full = _mla_bwd_dk_dv(qd, kfd, vd, dod, lse, delta, scale, causal)
    dq_full = _mla_bwd_dq(qd, kfd, vd, dod, lse, delta, scale, causal)
    assert torch.equal(dq, dq_full) and torch.equal(dv, dv_full) and torch.equal(dk_nope, dk_full[..., :128])
    # the head sum of the assembled path's bf16 gradients differs from dk_pe only by their rounding
    check_bf16_result(dk_pe, dk_full[..., 128:].float().sum(2), "dK pe vs assembled path", otol=1e-3)


@pytest.mark.parametrize("layout", ["contiguous", "zigzag"])
def test_ring_share_with_keys_in_two_parts(gpu, layout):
    B, S, H, C = 1, 1024, 8, 4
    S_l = S // C
    scale = 192**-0.5
    g = torch.Generator().manual_seed(42)
    q_full = (torch.randn(B, S, H, 192, generator=g) * scale).to(torch.bfloat16)
    dout_full = torch.randn(B, S, H, 128, generator=g).to(torch.bfloat16)
    k_nope, wide, v = _parts(B, S, H, 44)
    k_pe = wide[..., 512:].contiguous()
    split = (lambda x: R.zigzag_split(x, C)) if layout == "zigzag" else (lambda x: list(x.chunk(C, 1)))
    qs, dos, kns, kps, vs = (split(t) for t in (q_full, dout_full, k_nope, k_pe, v))
    k_asm = [_assemble(a, b) for a, b in zip(kns, kps)]
    for r in range(C):
        qd = qs[r].contiguous().to(gpu).requires_grad_(True)
        knd = [c.contiguous().to(gpu).requires_grad_(True) for c in kns]
        kpd = [c.contiguous().to(gpu).requires_grad_(True) for c in kps]
        vd = [c.contiguous().to(gpu).requires_grad_(True) for c in vs]
        out = ring_attention_local(qd, knd, vd, scale, r, C, layout, k_pe_chunks=kpd)
        out.backward(dos[r].contiguous().to(gpu))
        ro, rl = R.ring_forward(qs[r], k_asm, vs, scale, r, C, layout)
        rdq, rdk, rdv = R.ring_backward(dos[r], qs[r], ro, rl, k_asm, vs, scale, r, C, layout)
        check_bf16_result(out, ro, f"O rank {r}")
        check_bf16_result(qd.grad, rdq, f"dQ rank {r}", otol=1e-3)
        for j in range(C):
            if rdk[j] is None:
                assert knd[j].grad is None and kpd[j].grad is None
                continue
            check_bf16_result(knd[j].grad, rdk[j][..., :128], f"dK nope rank {r} chunk {j}", otol=2e-3)
            check_bf16_result(kpd[j].grad, rdk[j][..., 128:].sum(2), f"dK pe rank {r} chunk {j}", otol=2e-3)
            check_bf16_result(vd[j].grad, rdv[j], f"dV rank {r} chunk {j}", otol=2e-3)


@pytest.mark.parametrize("rerotate", [False, True])
def test_public_wrapper_with_keys_in_two_parts(gpu, rerotate):
    """ring_mla_attention_func(q, k_nope, v, scale, group, k_pe=...) with a group of one: plain causal
    attention on the key [k_nope | k_pe]; gradients for k_nope and for k_pe in the shape it was given."""
    from pithtrain_amd.operators.ring_attention.mla import ring_mla_attention_func

    B, S, H = 2, 320, 8
    scale = 192**-0.5
    g = torch.Generator().manual_seed(5)
    q = (torch.randn(B, S, H, 192, generator=g) * scale).to(torch.bfloat16)
    dout = torch.randn(B, S, H, 128, generator=g).to(torch.bfloat16)
    k_nope, wide, v = _parts(B, S, H, 6)
    k_pe = wide[..., 512:].unsqueeze(2).contiguous()  # [B, S, 1, 64] as the model holds it
    qd, knd, vd, kpd = (t.to(gpu).requires_grad_(True) for t in (q, k_nope, v, k_pe))
    out = ring_mla_attention_func(qd, knd, vd, scale, None, rerotate=rerotate, k_pe=kpd)
    out.backward(dout.to(gpu))
    k_full = _assemble(k_nope, k_pe[:, :, 0])
    o_ref, lse_ref = R.chunk_fwd(q, k_full, v, scale, True)
    dq_ref, dk_ref, dv_ref = R.chunk_bwd(q, k_full, v, dout, lse_ref, R.bwd_delta(o_ref, dout), scale, True)
    assert kpd.grad.shape == k_pe.shape
    check_bf16_result(out, o_ref, "O")
    check_bf16_result(qd.grad, dq_ref, "dQ", otol=1e-3)
    check_bf16_result(vd.grad, dv_ref, "dV", otol=1e-3)
    check_bf16_result(knd.grad, dk_ref[..., :128], "dK nope", otol=1e-3)
    check_bf16_result(kpd.grad[:, :, 0], dk_ref[..., 128:].sum(2), "dK pe", otol=1e-3)
