"""
Attention prologue of the GQA layer backed by libpith_hip.so: per-head RMSNorm of the projected
q / k followed by the rotary position embedding, one HIP kernel per direction
(q and k share a launch).

Replaces, at pithtrain/models/qwen3_30b_a3b.py:417-421,

    query_states = self.q_norm(query_states)          # nn.RMSNorm(head_dim), :381-382
    key_states = self.k_norm(key_states)
    query_states, key_states = apply_rotary_pos_emb(query_states, key_states, cos, sin)   # :107-136

with  `qk_norm_rope(query_states, key_states, self.q_norm.weight, self.k_norm.weight, cos, sin, eps)`.
`apply_rotary_pos_emb` keeps the reference's name and signature for call sites without a norm.

 b : batch size, s : sequence length, h : heads, d : head dim.
x [b, s, h, d] bf16; cos, sin [b, s, d] (or [1, s, d] / [s, d], shared by the batch) bf16;
weight [d] bf16 or fp32. Arithmetic is fp32 with a single rounding to bf16 (the reference's eager
bf16 expression rounds after every elementwise op). Wrapped as torch.library custom ops with fake
implementations and an autograd formula, so compiled layers keep working.
"""

from typing import Optional, Tuple

import torch

from pithtrain_amd import _C


def _cos_sin_stride(cos: torch.Tensor, sin: torch.Tensor, b: int, s: int, d: int) -> int:
    assert cos.dtype == sin.dtype == torch.bfloat16, "cos and sin must be bfloat16"
    assert cos.shape == sin.shape and cos.stride() == sin.stride(), "cos and sin must share shape and strides"
    if cos.dim() == 2:
        assert tuple(cos.shape) == (s, d), f"cos of shape {tuple(cos.shape)} does not match [s={s}, d={d}]"
        assert cos.is_contiguous(), "cos is not contiguous"
        return 0
    assert cos.dim() == 3 and cos.shape[0] in (1, b) and tuple(cos.shape[1:]) == (s, d), (
        f"cos of shape {tuple(cos.shape)} does not match [b={b} or 1, s={s}, d={d}]"
    )
    assert cos.stride(2) == 1 and (s == 1 or cos.stride(1) == d), "cos is not contiguous"
    return cos.stride(0) if (cos.shape[0] > 1) else 0


def _args(x, weight, cos, sin, out, eps) -> _C.NormRopeArgs:
    _C.require_device(x, cos, sin, out)
    assert x.dtype == torch.bfloat16 and x.dim() == 4, "x must be a bfloat16 [B, S, H, D] tensor"
    assert out.dtype == torch.bfloat16 and out.shape == x.shape, "out must match x"
    b, s, h, d = x.shape
    if weight is not None:
        _C.require_device(x, weight)
        assert tuple(weight.shape) == (d,) and weight.is_contiguous(), f"weight must be a contiguous [{d}] tensor"
    return _C.NormRopeArgs(
        x=x.data_ptr(), weight=None if weight is None else weight.data_ptr(),
        cos=cos.data_ptr(), sin=sin.data_ptr(), dout=None, out=out.data_ptr(), dweight=None,
        workspace=None, workspace_bytes=0, B=b, S=s, H=h, D=d,
        x_bs=_C.bshd_batch_stride(x, "x"), out_bs=_C.bshd_batch_stride(out, "out"), dout_bs=0,
        cs_bs=_cos_sin_stride(cos, sin, b, s, d), eps=float(eps),
        weight_dtype=_C.PITH_BF16 if weight is None else _C.dtype_code(weight),
    )  # fmt: skip


def norm_rope_fwd_into(x: torch.Tensor, weight: Optional[torch.Tensor], cos: torch.Tensor, sin: torch.Tensor,
                       out: torch.Tensor, eps: float) -> None:  # fmt: skip
    """out <- rope(rms_norm(x) * weight) (weight None: rope(x)). out may be x itself."""
    args = _args(x, weight, cos, sin, out, eps)
    _C.check(_C.lib().pith_norm_rope_fwd(_C.byref(args), _C.current_stream(x)))


def norm_rope_bwd_into(x: torch.Tensor, weight: Optional[torch.Tensor], cos: torch.Tensor, sin: torch.Tensor,
                       dout: torch.Tensor, dx: torch.Tensor, dweight: Optional[torch.Tensor], eps: float) -> None:  # fmt: skip
    """dx <- gradient w.r.t. x; dweight [d] fp32 <- gradient w.r.t. weight (ignored without weight)."""
    args = _args(x, weight, cos, sin, dx, eps)
    _C.require_device(x, dout)
    assert dout.dtype == torch.bfloat16 and dout.shape == x.shape, "dout must match x"
    args.dout, args.dout_bs = dout.data_ptr(), _C.bshd_batch_stride(dout, "dout")
    workspace = None
    if weight is not None:
        assert dweight is not None and dweight.dtype == torch.float32 and dweight.shape == weight.shape, (
            "dweight must be a float32 tensor shaped like weight"
        )
        _C.require_device(x, dweight)
        assert dweight.is_contiguous(), "dweight is not contiguous"
        args.dweight = dweight.data_ptr()
        need = _C.lib().pith_norm_rope_bwd_workspace_bytes(_C.byref(args))
        workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
        args.workspace, args.workspace_bytes = workspace.data_ptr(), need
    _C.check(_C.lib().pith_norm_rope_bwd(_C.byref(args), _C.current_stream(x)))


@torch.library.custom_op("pithtrain_amd::norm_rope_fwd", mutates_args=())
def _norm_rope_fwd_op(x: torch.Tensor, weight: Optional[torch.Tensor], cos: torch.Tensor, sin: torch.Tensor,
                      eps: float) -> torch.Tensor:  # fmt: skip
    x = x.contiguous()
    out = torch.empty_like(x)
    norm_rope_fwd_into(x, weight, cos.contiguous(), sin.contiguous(), out, eps)
    return out


@_norm_rope_fwd_op.register_fake
def _(x, weight, cos, sin, eps):
    return torch.empty_like(x, memory_format=torch.contiguous_format)


@torch.library.custom_op("pithtrain_amd::norm_rope_bwd", mutates_args=())
def _norm_rope_bwd_op(x: torch.Tensor, weight: Optional[torch.Tensor], cos: torch.Tensor, sin: torch.Tensor,
                      dout: torch.Tensor, eps: float) -> Tuple[torch.Tensor, torch.Tensor]:  # fmt: skip
    x, dout = x.contiguous(), dout.contiguous()
    dx = torch.empty_like(x)
    # without a weight the second result is an empty placeholder (custom ops cannot return None)
    dweight = x.new_empty((x.shape[-1] if weight is not None else 0,), dtype=torch.float32)
    norm_rope_bwd_into(x, weight, cos.contiguous(), sin.contiguous(), dout, dx,
                       dweight if weight is not None else None, eps)  # fmt: skip
    return dx, dweight


@_norm_rope_bwd_op.register_fake
def _(x, weight, cos, sin, dout, eps):
    dx = torch.empty_like(x, memory_format=torch.contiguous_format)
    return dx, x.new_empty((x.shape[-1] if weight is not None else 0,), dtype=torch.float32)


def _setup_context(ctx, inputs, output):
    x, weight, cos, sin, eps = inputs
    ctx.save_for_backward(x, weight, cos, sin)
    ctx.eps = eps


def _backward(ctx, grad_out):
    x, weight, cos, sin = ctx.saved_tensors
    dx, dweight = _norm_rope_bwd_op(x, weight, cos, sin, grad_out, ctx.eps)
    return dx, (None if weight is None else dweight.to(weight.dtype)), None, None, None


_norm_rope_fwd_op.register_autograd(_backward, setup_context=_setup_context)


def norm_rope(x: torch.Tensor, weight: Optional[torch.Tensor], cos: torch.Tensor, sin: torch.Tensor,
              eps: float = 1e-6) -> torch.Tensor:  # fmt: skip
    """rope(rms_norm(x, eps) * weight) over the last dim of x [b, s, h, d], with autograd."""
    return _norm_rope_fwd_op(x, weight, cos, sin, eps)


# ---------------------------------------------------------------------------------------------
# q and k of a layer together: one launch forward, one (plus the dweight sums) backward.


def _workspace_for(args: _C.NormRopeArgs, device) -> Optional[torch.Tensor]:
    need = _C.lib().pith_norm_rope_bwd_workspace_bytes(_C.byref(args))
    if need == 0:
        return None
    workspace = torch.empty(need, dtype=torch.uint8, device=device)
    args.workspace, args.workspace_bytes = workspace.data_ptr(), need
    return workspace


def qk_norm_rope_fwd_into(q, k, q_weight, k_weight, cos, sin, q_out, k_out, eps: float) -> None:
    """q_out, k_out <- rope(rms_norm(q) * q_weight), rope(rms_norm(k) * k_weight); weights may both be None."""
    a = _args(q, q_weight, cos, sin, q_out, eps)
    b = _args(k, k_weight, cos, sin, k_out, eps)
    _C.check(_C.lib().pith_norm_rope_fwd_pair(_C.byref(a), _C.byref(b), _C.current_stream(q)))


def qk_norm_rope_bwd_into(q, k, q_weight, k_weight, cos, sin, dq_out, dk_out, dq, dk, dq_weight, dk_weight,
                          eps: float) -> None:  # fmt: skip
    """dq, dk <- gradients w.r.t. q, k; dq_weight, dk_weight [d] fp32 <- gradients w.r.t. the weights."""
    a = _args(q, q_weight, cos, sin, dq, eps)
    b = _args(k, k_weight, cos, sin, dk, eps)
    keep = []
    for args, x, w, dout, dweight in ((a, q, q_weight, dq_out, dq_weight), (b, k, k_weight, dk_out, dk_weight)):
        _C.require_device(x, dout)
        assert dout.dtype == torch.bfloat16 and dout.shape == x.shape, "a gradient does not match its tensor"
        args.dout, args.dout_bs = dout.data_ptr(), _C.bshd_batch_stride(dout, "dout")
        if w is not None:
            assert dweight is not None and dweight.dtype == torch.float32 and dweight.shape == w.shape, (
                "dweight must be a float32 tensor shaped like weight"
            )
            _C.require_device(x, dweight)
            assert dweight.is_contiguous(), "dweight is not contiguous"
            args.dweight = dweight.data_ptr()
            keep.append(_workspace_for(args, x.device))
    _C.check(_C.lib().pith_norm_rope_bwd_pair(_C.byref(a), _C.byref(b), _C.current_stream(q)))


@torch.library.custom_op("pithtrain_amd::qk_norm_rope_fwd", mutates_args=())
def _qk_norm_rope_fwd_op(q: torch.Tensor, k: torch.Tensor, q_weight: Optional[torch.Tensor],
                         k_weight: Optional[torch.Tensor], cos: torch.Tensor, sin: torch.Tensor,
                         eps: float) -> Tuple[torch.Tensor, torch.Tensor]:  # fmt: skip
    q, k = q.contiguous(), k.contiguous()
    q_out, k_out = torch.empty_like(q), torch.empty_like(k)
    qk_norm_rope_fwd_into(q, k, q_weight, k_weight, cos.contiguous(), sin.contiguous(), q_out, k_out, eps)
    return q_out, k_out


@_qk_norm_rope_fwd_op.register_fake
def _(q, k, q_weight, k_weight, cos, sin, eps):
    fmt = torch.contiguous_format
    return torch.empty_like(q, memory_format=fmt), torch.empty_like(k, memory_format=fmt)


@torch.library.custom_op("pithtrain_amd::qk_norm_rope_bwd", mutates_args=())
def _qk_norm_rope_bwd_op(q: torch.Tensor, k: torch.Tensor, q_weight: Optional[torch.Tensor],
                         k_weight: Optional[torch.Tensor], cos: torch.Tensor, sin: torch.Tensor,
                         dq_out: torch.Tensor, dk_out: torch.Tensor,
                         eps: float) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:  # fmt: skip
    q, k, dq_out, dk_out = q.contiguous(), k.contiguous(), dq_out.contiguous(), dk_out.contiguous()
    dq, dk = torch.empty_like(q), torch.empty_like(k)
    # without weights the last two results are empty placeholders (custom ops cannot return None)
    n = q.shape[-1] if q_weight is not None else 0
    dwq, dwk = q.new_empty((n,), dtype=torch.float32), q.new_empty((n,), dtype=torch.float32)
    qk_norm_rope_bwd_into(q, k, q_weight, k_weight, cos.contiguous(), sin.contiguous(), dq_out, dk_out, dq, dk,
                          dwq if n else None, dwk if n else None, eps)  # fmt: skip
    return dq, dk, dwq, dwk


@_qk_norm_rope_bwd_op.register_fake
def _(q, k, q_weight, k_weight, cos, sin, dq_out, dk_out, eps):
    fmt = torch.contiguous_format
    n = q.shape[-1] if q_weight is not None else 0
    return (torch.empty_like(q, memory_format=fmt), torch.empty_like(k, memory_format=fmt),
            q.new_empty((n,), dtype=torch.float32), q.new_empty((n,), dtype=torch.float32))  # fmt: skip


def _qk_setup_context(ctx, inputs, output):
    q, k, q_weight, k_weight, cos, sin, eps = inputs
    ctx.save_for_backward(q, k, q_weight, k_weight, cos, sin)
    ctx.eps = eps


def _qk_backward(ctx, grad_q, grad_k):
    q, k, q_weight, k_weight, cos, sin = ctx.saved_tensors
    dq, dk, dwq, dwk = _qk_norm_rope_bwd_op(q, k, q_weight, k_weight, cos, sin, grad_q, grad_k, ctx.eps)
    if q_weight is None:
        return dq, dk, None, None, None, None, None
    return dq, dk, dwq.to(q_weight.dtype), dwk.to(k_weight.dtype), None, None, None


_qk_norm_rope_fwd_op.register_autograd(_qk_backward, setup_context=_qk_setup_context)


def qk_norm_rope(q: torch.Tensor, k: torch.Tensor, q_weight: torch.Tensor, k_weight: torch.Tensor,
                 cos: torch.Tensor, sin: torch.Tensor, eps: float = 1e-6) -> Tuple[torch.Tensor, torch.Tensor]:  # fmt: skip
    """The three statements at pithtrain/models/qwen3_30b_a3b.py:417-421 as one kernel launch."""
    return _qk_norm_rope_fwd_op(q, k, q_weight, k_weight, cos, sin, eps)


def apply_rotary_pos_emb(q: torch.Tensor, k: torch.Tensor, cos: torch.Tensor,
                         sin: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:  # fmt: skip
    """pithtrain/models/qwen3_30b_a3b.py:107-136 — same name, arguments and results."""
    return _qk_norm_rope_fwd_op(q, k, None, None, cos, sin, 0.0)


__all__ = [
    "norm_rope", "qk_norm_rope", "apply_rotary_pos_emb", "norm_rope_fwd_into", "norm_rope_bwd_into",
    "qk_norm_rope_fwd_into", "qk_norm_rope_bwd_into",
]  # fmt: skip
