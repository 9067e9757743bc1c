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
