"""
Ring attention for context parallelism, GQA / MHA variant (equal q/k and v head dims).

Drop-in for pithtrain/operators/ring_attention/standard.py: `ring_attention_func`,
`RingAttentionFunc` and `_online_softmax_combine` keep their names and argument order. The chunk
attention is the HIP forward/backward of pithtrain_amd.operators.mla.hip instead of flash-attn's
_flash_attn_forward/_flash_attn_backward (standard.py:91-93, 134-153); inside the ring the LSE is
kept in base 2 (LSE_2 = LSE_e * log2(e)), which leaves O, dQ, dK, dV unchanged.

`layout="zigzag"` (keyword only, default "contiguous" as in the reference) selects the
load-balanced token layout described in local.py.
"""

import torch
import torch.distributed as dist

from pithtrain_amd import _C
from pithtrain_amd.operators.ring_attention.combine import _combine_new
from pithtrain_amd.operators.ring_attention.distributed import (
    RingAttentionDistributedFunc,
    _ring_send_recv_kv,
    ring_attention_group_func,
)


def _online_softmax_combine(out1, lse1, out2, lse2):
    """Combine two partial attention outputs via online softmax rescaling.

    out: [B, S, H, D],  lse: [B, H, S]  (float32, natural-log scale). Returns fp32 (out, lse).
    """
    return _combine_new(out1, lse1, out2, lse2, _C.PITH_BASE_E)


class RingAttentionFunc(RingAttentionDistributedFunc):
    """Causal ring attention with HIP chunk kernels; forward(ctx, q, k, v, softmax_scale, cp_rank,
    cp_size, global_ranks) as in the reference."""


def ring_attention_func(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    softmax_scale: float,
    cp_group: dist.ProcessGroup,
    *,
    layout: str = "contiguous",
    rerotate: bool = False,
):
    """Causal ring attention across context-parallel ranks."""
    assert q.shape[-1] == v.shape[-1], "ring_attention_func expects equal q/k and v head dims"
    return ring_attention_group_func(q, k, v, softmax_scale, cp_group, layout, rerotate)


__all__ = ["ring_attention_func", "RingAttentionFunc", "_online_softmax_combine", "_ring_send_recv_kv"]
