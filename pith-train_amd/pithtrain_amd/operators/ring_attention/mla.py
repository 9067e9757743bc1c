"""
Ring MLA attention for context parallelism (asymmetric head dims: q/k 192, v 128).

Drop-in for pithtrain/operators/ring_attention/mla.py: `ring_mla_attention_func`,
`RingMLAAttentionFunc` and `_online_softmax_combine_log2` keep their names and argument order.
The chunk kernels store LSE in log2 scale, so the combine works with exp2/log2.
"""

import torch
import torch.distributed as dist

from pithtrain_amd import _C
from pithtrain_amd.operators.ring_attention.combine import _combine_new
from pithtrain_amd.operators.ring_attention.distributed import (
    RingAttentionDistributedFunc,
    ring_attention_group_func,
)


def _online_softmax_combine_log2(out1, lse1, out2, lse2):
    """Combine two partial attention outputs via online softmax rescaling.

    Operates in log2 scale to match the chunk kernels.
    out: [B, S, H, D],  lse: [B, H, S]  (float32, log2 scale). Returns fp32 (out, lse).
    """
    return _combine_new(out1, lse1, out2, lse2, _C.PITH_BASE_2)


class RingMLAAttentionFunc(RingAttentionDistributedFunc):
    """Causal ring MLA attention with HIP chunk kernels; forward(ctx, q, k, v, softmax_scale,
    cp_rank, cp_size, global_ranks) as in the reference."""


def ring_mla_attention_func(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    softmax_scale: float,
    cp_group: dist.ProcessGroup,
    *,
    layout: str = "contiguous",
    rerotate: bool = False,
    k_pe: torch.Tensor = None,
):
    """Causal ring MLA attention across context-parallel ranks.

    Keyword k_pe: keys in two parts. Pass k = k_nope [B, S_l, H, 128] and k_pe [B, S_l, 64] (or
    [B, S_l, 1, 64]), the rotary key part that the reference broadcasts to all heads when it assembles
    key_states (pithtrain/models/deepseek_v2_lite.py:448-454); the kernels read both in place, both
    rotate around the ring, and autograd returns a gradient for each."""
    return ring_attention_group_func(q, k, v, softmax_scale, cp_group, layout, rerotate, k_pe)


__all__ = ["ring_mla_attention_func", "RingMLAAttentionFunc", "_online_softmax_combine_log2"]
