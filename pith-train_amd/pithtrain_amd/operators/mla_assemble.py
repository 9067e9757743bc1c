"""
Attention prologue of the MLA layer backed by libpith_hip.so: rotary embedding of the rope parts
of q and of the shared k_pe, and assembly of query / key / value states, one HIP kernel per direction.

Replaces, at pithtrain/models/deepseek_v2_lite.py:446-454 and the `.contiguous()` of :462/:467,

    q_pe, k_pe = apply_rotary_pos_emb(q_pe, k_pe, cos, sin, position_ids, unsqueeze_dim=2)   # :173-187
    query_states = k_pe.new_empty(bsz, q_len, self.num_heads, self.q_head_dim)
    query_states[:, :, :, : self.qk_nope_head_dim] = q_nope
    query_states[:, :, :, self.qk_nope_head_dim :] = q_pe
    key_states = k_pe.new_empty(bsz, q_len, self.num_heads, self.q_head_dim)
    key_states[:, :, :, : self.qk_nope_head_dim] = k_nope
    key_states[:, :, :, self.qk_nope_head_dim :] = k_pe
    ... value_states.contiguous()

with  `query_states, key_states, value_states = mla_assemble_qkv(q, kv, k_pe, cos, sin, position_ids)`
where q is the q_proj output viewed [b, s, h, dn + dr], kv the kv_b_proj output viewed [b, s, h, dn + dv]
(before the reference splits them) and k_pe the [b, s, 1, dr] (or [b, s, dr]) slice of the kv_a projection.

 b : batch size, s : sequence length, h : heads, dn : nope dim, dr : rope dim, dv : value dim.
cos, sin are the rotary module's [positions, dr] tables (bf16); position_ids [b, s] int64 or None.
"""

import os
from typing import Optional, Tuple

import torch

from pithtrain_amd import _C


def _tables(cos: torch.Tensor, sin: torch.Tensor, dr: int) -> int:
    assert cos.dtype == sin.dtype == torch.bfloat16, "cos and sin must be bfloat16"
    assert cos.dim() == 2 and cos.shape == sin.shape and cos.shape[1] == dr, f"cos and sin must be [positions, {dr}]"
    assert cos.is_contiguous() and sin.is_contiguous(), "cos or sin is not contiguous"
    return cos.shape[0]


def _positions(position_ids: Optional[torch.Tensor], b: int, s: int, table_rows: int):
    """Pointer and batch stride of position_ids. The rotary tables must cover every position: the
    reference indexes them with `cos[position_ids]` (pithtrain/models/deepseek_v2_lite.py:173-187, tables
    sized at :443-445), which raises on a position beyond the table; the kernel clamps such a position
    to the table edge to stay inside memory, so a too-short table is rejected here where it can be seen
    without reading device memory (position_ids=None means positions 0..s-1). With explicit positions the
    caller sizes the table to max(position_ids)+1 as the reference does; PITHTRAIN_AMD_CHECK_POSITIONS=1
    adds that check at the price of a device synchronisation."""
    if position_ids is None:
        assert table_rows >= s, f"rotary tables hold {table_rows} positions, the sequence has {s}"
        return None, 0
    if os.environ.get("PITHTRAIN_AMD_CHECK_POSITIONS") == "1":
        lo, hi = int(position_ids.min()), int(position_ids.max())
        assert 0 <= lo and hi < table_rows, f"position_ids span [{lo}, {hi}], the rotary tables hold {table_rows} positions"
    assert position_ids.dtype == torch.int64, "position_ids must be int64"
    assert position_ids.dim() == 2 and position_ids.shape[0] in (1, b) and position_ids.shape[1] == s, (
        f"position_ids of shape {tuple(position_ids.shape)} does not match [b={b} or 1, s={s}]"
    )
    assert s == 1 or position_ids.stride(1) == 1, "position_ids is not contiguous"
    return position_ids.data_ptr(), (position_ids.stride(0) if position_ids.shape[0] > 1 else 0)


def mla_assemble_fwd_into(q, kv, k_pe, cos, sin, position_ids, q_out, k_out, v_out) -> None:
    """q_out [b,s,h,dn+dr], k_out [b,s,h,dn+dr], v_out [b,s,h,dv] (contiguous) are written."""
    _C.require_device(q, kv, k_pe, cos, sin, q_out, k_out, v_out)
    assert q.dtype == kv.dtype == k_pe.dtype == torch.bfloat16, "q, kv, k_pe must be bfloat16"
    assert q.dim() == 4 and kv.dim() == 4, "q and kv must be [B, S, H, D]"
    b, s, h, dqk = q.shape
    if k_pe.dim() == 4:
        assert k_pe.shape[2] == 1, "k_pe must have a single head"
        k_pe = k_pe[:, :, 0]
    dr = k_pe.shape[-1]
    dn = dqk - dr
    dv = kv.shape[-1] - dn
    assert dn > 0 and dv > 0 and tuple(kv.shape[:3]) == (b, s, h) and tuple(k_pe.shape) == (b, s, dr), (
        f"shapes do not fit: q {tuple(q.shape)}, kv {tuple(kv.shape)}, k_pe {tuple(k_pe.shape)}"
    )
    assert k_pe.stride(2) == 1, "k_pe is not contiguous along its last dim"
    for name, t, shape in (("q_out", q_out, (b, s, h, dqk)), ("k_out", k_out, (b, s, h, dqk)), ("v_out", v_out, (b, s, h, dv))):
        assert t.dtype == torch.bfloat16 and tuple(t.shape) == shape and t.is_contiguous(), f"{name} has the wrong dtype, shape or layout"
    table_rows = _tables(cos, sin, dr)
    pos_ptr, pos_bs = _positions(position_ids, b, s, table_rows)
    if position_ids is not None:
        _C.require_device(q, position_ids)
    args = _C.MlaAssembleArgs(
        q=q.data_ptr(), kv=kv.data_ptr(), k_pe=k_pe.data_ptr(), cos=cos.data_ptr(), sin=sin.data_ptr(),
        position_ids=pos_ptr, q_out=q_out.data_ptr(), k_out=k_out.data_ptr(), v_out=v_out.data_ptr(),
        dq_out=None, dk_out=None, dv_out=None, B=b, S=s, H=h, Dn=dn, Dr=dr, Dv=dv, P=_tables(cos, sin, dr),
        q_bs=_C.bshd_batch_stride(q, "q"), kv_bs=_C.bshd_batch_stride(kv, "kv"),
        k_pe_bs=k_pe.stride(0) if b > 1 else s * k_pe.stride(1), k_pe_rs=k_pe.stride(1) if s > 1 else dr, pos_bs=pos_bs,
    )  # fmt: skip
    _C.check(_C.lib().pith_mla_assemble_fwd(_C.byref(args), _C.current_stream(q)))


def mla_assemble_bwd_into(dq_out, dk_out, dv_out, cos, sin, position_ids, dq, dkv, dk_pe) -> None:
    """dq [b,s,h,dn+dr], dkv [b,s,h,dn+dv], dk_pe [b,s,dr] (contiguous) <- gradients of the inputs."""
    _C.require_device(dq_out, dk_out, dv_out, cos, sin, dq, dkv, dk_pe)
    b, s, h, dqk = dq_out.shape
    dr, dv = dk_pe.shape[-1], dv_out.shape[-1]
    dn = dqk - dr
    for name, t, shape in (("dq_out", dq_out, (b, s, h, dqk)), ("dk_out", dk_out, (b, s, h, dqk)),
                           ("dv_out", dv_out, (b, s, h, dv)), ("dq", dq, (b, s, h, dqk)),
                           ("dkv", dkv, (b, s, h, dn + dv)), ("dk_pe", dk_pe, (b, s, dr))):  # fmt: skip
        assert t.dtype == torch.bfloat16 and tuple(t.shape) == shape and t.is_contiguous(), f"{name} has the wrong dtype, shape or layout"
    pos_ptr, pos_bs = _positions(position_ids, b, s, _tables(cos, sin, dr))
    args = _C.MlaAssembleArgs(
        q=None, kv=None, k_pe=None, cos=cos.data_ptr(), sin=sin.data_ptr(), position_ids=pos_ptr,
        q_out=dq.data_ptr(), k_out=dkv.data_ptr(), v_out=dk_pe.data_ptr(),
        dq_out=dq_out.data_ptr(), dk_out=dk_out.data_ptr(), dv_out=dv_out.data_ptr(),
        B=b, S=s, H=h, Dn=dn, Dr=dr, Dv=dv, P=_tables(cos, sin, dr), q_bs=0, kv_bs=0, k_pe_bs=0, k_pe_rs=0, pos_bs=pos_bs,
    )  # fmt: skip
    _C.check(_C.lib().pith_mla_assemble_bwd(_C.byref(args), _C.current_stream(dq_out)))


@torch.library.custom_op("pithtrain_amd::mla_assemble_fwd", mutates_args=())
def _mla_assemble_fwd_op(q: torch.Tensor, kv: torch.Tensor, k_pe: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                         position_ids: Optional[torch.Tensor]) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:  # fmt: skip
    b, s, h, dqk = q.shape
    dv = kv.shape[-1] - (dqk - k_pe.shape[-1])
    q_out = q.new_empty((b, s, h, dqk))
    k_out = q.new_empty((b, s, h, dqk))
    v_out = q.new_empty((b, s, h, dv))
    mla_assemble_fwd_into(q.contiguous(), kv.contiguous(), k_pe, cos, sin, position_ids, q_out, k_out, v_out)
    return q_out, k_out, v_out


@_mla_assemble_fwd_op.register_fake
def _(q, kv, k_pe, cos, sin, position_ids):
    b, s, h, dqk = q.shape
    dv = kv.shape[-1] - (dqk - k_pe.shape[-1])
    return q.new_empty((b, s, h, dqk)), q.new_empty((b, s, h, dqk)), q.new_empty((b, s, h, dv))


@torch.library.custom_op("pithtrain_amd::mla_assemble_bwd", mutates_args=())
def _mla_assemble_bwd_op(dq_out: torch.Tensor, dk_out: torch.Tensor, dv_out: torch.Tensor, cos: torch.Tensor,
                         sin: torch.Tensor, position_ids: Optional[torch.Tensor],
                         k_pe_heads: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:  # fmt: skip
    b, s, h, dqk = dq_out.shape
    dr, dv = cos.shape[1], dv_out.shape[-1]
    dq = dq_out.new_empty((b, s, h, dqk))
    dkv = dq_out.new_empty((b, s, h, dqk - dr + dv))
    dk_pe = dq_out.new_empty((b, s, dr))
    mla_assemble_bwd_into(dq_out.contiguous(), dk_out.contiguous(), dv_out.contiguous(), cos, sin, position_ids,
                          dq, dkv, dk_pe)  # fmt: skip
    return dq, dkv, (dk_pe.unsqueeze(2) if k_pe_heads else dk_pe)


@_mla_assemble_bwd_op.register_fake
def _(dq_out, dk_out, dv_out, cos, sin, position_ids, k_pe_heads):
    b, s, h, dqk = dq_out.shape
    dr, dv = cos.shape[1], dv_out.shape[-1]
    dk_pe = dq_out.new_empty((b, s, 1, dr) if k_pe_heads else (b, s, dr))
    return dq_out.new_empty((b, s, h, dqk)), dq_out.new_empty((b, s, h, dqk - dr + dv)), dk_pe


def _setup_context(ctx, inputs, output):
    q, kv, k_pe, cos, sin, position_ids = inputs
    ctx.save_for_backward(cos, sin, position_ids)
    ctx.k_pe_heads = 1 if k_pe.dim() == 4 else 0


def _backward(ctx, dq_out, dk_out, dv_out):
    cos, sin, position_ids = ctx.saved_tensors
    dq, dkv, dk_pe = _mla_assemble_bwd_op(dq_out, dk_out, dv_out, cos, sin, position_ids, ctx.k_pe_heads)
    return dq, dkv, dk_pe, None, None, None


_mla_assemble_fwd_op.register_autograd(_backward, setup_context=_setup_context)


def mla_assemble_qkv(q: torch.Tensor, kv: torch.Tensor, k_pe: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                     position_ids: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:  # fmt: skip
    """(query_states, key_states, value_states) of the MLA layer, with autograd to q, kv and k_pe."""
    return _mla_assemble_fwd_op(q, kv, k_pe, cos, sin, position_ids)


__all__ = ["mla_assemble_qkv", "mla_assemble_fwd_into", "mla_assemble_bwd_into"]
