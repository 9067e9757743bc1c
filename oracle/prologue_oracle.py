"""
CPU oracle for the attention prologue (q/k RMSNorm + rotary embedding) — TEST INFRASTRUCTURE ONLY.

Restates, in dense PyTorch on the CPU (float64 by default), what the GQA layer does to the
projected q and k before the attention call. Imported only by tests/, __graft_entry__.smoke()
and the cpu_baseline leg of bench.py; the product package never imports it.

Reference lines followed (paths relative to the PithTrain tree):
  pithtrain/models/qwen3_30b_a3b.py:381-382,417-418  q_norm / k_norm = nn.RMSNorm(head_dim, eps) -> rms_norm
  pithtrain/models/qwen3_30b_a3b.py:100-104          rotate_half                                  -> rotate_half
  pithtrain/models/qwen3_30b_a3b.py:107-136          apply_rotary_pos_emb (one tensor of the two)  -> rope
  pithtrain/models/qwen3_30b_a3b.py:54-71            cos/sin table                                 -> cos_sin_table
  pithtrain/models/deepseek_v2_lite.py:173-187       apply_rotary_pos_emb with the pair de-interleave -> deinterleave + rope
  pithtrain/models/deepseek_v2_lite.py:446-454,462   q/k/v assembly of the MLA layer               -> mla_assemble_fwd
torch.nn.RMSNorm is PyTorch's (y = x / sqrt(mean(x^2) + eps) * weight over the last dim); the
reference runs it and the rotation in bf16 with a rounding after every elementwise op, the
oracle is the exact function those roundings approximate. Tolerances live in the tests.

How each function is pinned (tests/test_prologue_oracle.py), none by retyping its own formula:
  rms_norm      : against torch.nn.functional.rms_norm (library routine); rows of the result with
                  unit weight have mean square 1 (eps = 0); invariance to scaling x.
  rope          : against complex multiplication, (x[j] + i x[j+D/2]) * exp(i theta_j), when cos/sin
                  come from angles; pairwise norm preservation; angle 0 is the identity; rotating
                  by theta then -theta is the identity; <rope(q,m), rope(k,n)> depends on m-n only.
  norm_rope_bwd : against torch.autograd through the library rms_norm and a complex-arithmetic
                  rotation, and against central finite differences of norm_rope_fwd.
  mla_assemble_fwd : rope parts against complex multiplication of the (even, odd) pairs; nope parts and
                  values are exact copies; every head of key_states carries the same rope part.
  mla_assemble_bwd : against torch.autograd through an independently written forward (index-based
                  de-interleave, complex rotation, slice assignment as in the reference).
"""

from typing import Optional, Tuple

import torch


def cos_sin_table(positions: torch.Tensor, dim: int, base: float = 1000000.0, dtype=torch.float64):
    """[..., dim] cos and sin of positions * inv_freq with the two halves equal (qwen3_30b_a3b.py:54-71)."""
    inv_freq = 1.0 / (base ** (torch.arange(0, dim, 2, dtype=torch.float64) / dim))
    freqs = positions.to(torch.float64).unsqueeze(-1) * inv_freq
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def rms_norm(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2, -1) + eps) * weight."""
    y = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x [B,S,H,D]; cos, sin [B,S,D] (or broadcastable to it): x*cos + rotate_half(x)*sin."""
    cos = cos.unsqueeze(-2)
    sin = sin.unsqueeze(-2)
    return x * cos + rotate_half(x) * sin


def norm_rope_fwd(x, weight, cos, sin, eps: float, dtype=torch.float64) -> torch.Tensor:
    x, cos, sin = x.to(dtype), cos.to(dtype), sin.to(dtype)
    y = x if weight is None else rms_norm(x, weight.to(dtype), eps)
    return rope(y, cos, sin)


def norm_rope_bwd(x, weight, cos, sin, dout, eps: float, dtype=torch.float64) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Closed-form gradients of norm_rope_fwd: (dx, dweight)."""
    x, cos, sin, dout = x.to(dtype), cos.to(dtype), sin.to(dtype), dout.to(dtype)
    cos = cos.unsqueeze(-2)
    sin = sin.unsqueeze(-2)
    half = x.shape[-1] // 2
    z = dout * sin
    # transpose of rotate_half: component j < half receives z[j + half], j >= half receives -z[j - half]
    dy = dout * cos + torch.cat((z[..., half:], -z[..., :half]), dim=-1)
    if weight is None:
        return dy, None
    w = weight.to(dtype)
    rstd = torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    xhat = x * rstd
    dweight = (dy * xhat).reshape(-1, x.shape[-1]).sum(0)
    dxhat = dy * w
    dx = rstd * (dxhat - xhat * (dxhat * xhat).mean(-1, keepdim=True))
    return dx, dweight


# ---------------------------------------------------------------------------------------------
# MLA layer (pithtrain/models/deepseek_v2_lite.py:446-454; apply_rotary_pos_emb :173-187)


def deinterleave(x: torch.Tensor) -> torch.Tensor:
    """[..., d] -> [..., d]: even-indexed elements first, then odd-indexed (deepseek_v2_lite.py:179-183)."""
    return torch.cat((x[..., 0::2], x[..., 1::2]), dim=-1)


def mla_assemble_fwd(q, kv, k_pe, cos_table, sin_table, position_ids, dn: int, dtype=torch.float64):
    """q [B,S,H,dn+dr], kv [B,S,H,dn+dv], k_pe [B,S,dr]; tables [P,dr]; position_ids [B,S] or None.
    Returns (query_states [B,S,H,dn+dr], key_states [B,S,H,dn+dr], value_states [B,S,H,dv])."""
    q, kv, k_pe = q.to(dtype), kv.to(dtype), k_pe.to(dtype)
    b, s, h, _ = q.shape
    if position_ids is None:
        position_ids = torch.arange(s).unsqueeze(0).expand(b, s)
    cos = cos_table.to(dtype)[position_ids]  # [B,S,dr]
    sin = sin_table.to(dtype)[position_ids]
    q_rot = rope(deinterleave(q[..., dn:]), cos, sin)
    k_rot = rope(deinterleave(k_pe).unsqueeze(2), cos, sin)  # [B,S,1,dr]
    query = torch.cat((q[..., :dn], q_rot), dim=-1)
    key = torch.cat((kv[..., :dn], k_rot.expand(b, s, h, k_rot.shape[-1])), dim=-1)
    return query, key, kv[..., dn:].contiguous()


def _interleave(x: torch.Tensor) -> torch.Tensor:
    """Inverse of deinterleave."""
    half = x.shape[-1] // 2
    return torch.stack((x[..., :half], x[..., half:]), dim=-1).flatten(-2)


def mla_assemble_bwd(dquery, dkey, dvalue, cos_table, sin_table, position_ids, dn: int, dtype=torch.float64):
    """Closed-form gradients of mla_assemble_fwd: (dq, dkv, dk_pe [B,S,dr])."""
    dquery, dkey, dvalue = dquery.to(dtype), dkey.to(dtype), dvalue.to(dtype)
    b, s, h, _ = dquery.shape
    if position_ids is None:
        position_ids = torch.arange(s).unsqueeze(0).expand(b, s)
    cos = cos_table.to(dtype)[position_ids].unsqueeze(2)
    sin = sin_table.to(dtype)[position_ids].unsqueeze(2)

    def unrotate(g):  # transpose of x -> x*cos + rotate_half(x)*sin, then of the de-interleave
        half = g.shape[-1] // 2
        z = g * sin
        return _interleave(g * cos + torch.cat((z[..., half:], -z[..., :half]), dim=-1))

    dq = torch.cat((dquery[..., :dn], unrotate(dquery[..., dn:])), dim=-1)
    dkv = torch.cat((dkey[..., :dn], dvalue), dim=-1)
    dk_pe = unrotate(dkey[..., dn:].sum(dim=2, keepdim=True))[:, :, 0]
    return dq, dkv, dk_pe
