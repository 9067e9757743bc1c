"""
Ring attention across context-parallel ranks: the K/V rotation and the return of dK/dV around
torch.distributed point-to-point calls (backend "nccl", which is RCCL on ROCm), with the per-step
compute shared with the one-GPU driver (local.py).

Communication pattern of the reference (pithtrain/operators/ring_attention/standard.py:29-50,
164-187): forward sends the held K/V chunk to rank+1 and receives from rank-1, cp_size-1 times;
backward returns, at distance d = 1..cp_size-1, the gradient computed for the chunk of rank
r-d and receives the one computed by rank r+d. With the zigzag layout every rank visits every
chunk, so both directions are taken modulo cp_size.

Only the cp_size == 1 path of this module runs on a one-GPU machine; the exchange code keeps the
call sites of the reference working unchanged on a multi-GPU node.
"""

from typing import List

import torch
import torch.distributed as dist

from pithtrain_amd.operators.ring_attention.local import RingBackward, RingForward, ring_schedule


def _ring_send_recv_kv(send_k: torch.Tensor, send_v: torch.Tensor, next_global: int, prev_global: int):
    """Passes the held chunk to the next rank and returns the one arriving from the previous rank."""
    assert send_k.is_contiguous() and send_v.is_contiguous(), "ring attention send_k or send_v is not contiguous"
    recv_k, recv_v = torch.empty_like(send_k), torch.empty_like(send_v)
    ops = [
        dist.P2POp(dist.isend, send_k, next_global),
        dist.P2POp(dist.isend, send_v, next_global),
        dist.P2POp(dist.irecv, recv_k, prev_global),
        dist.P2POp(dist.irecv, recv_v, prev_global),
    ]
    for req in dist.batch_isend_irecv(ops):
        req.wait()
    return recv_k, recv_v


class RingAttentionDistributedFunc(torch.autograd.Function):
    """Causal ring attention of one rank inside a context-parallel group (any supported head dims)."""

    @staticmethod
    def forward(ctx, q, k, v, softmax_scale, cp_rank, cp_size, global_ranks, layout="contiguous"):
        assert k.is_contiguous() and v.is_contiguous(), "ring attention k or v is not contiguous"
        steps = {st.kv_rank: st for st in ring_schedule(cp_rank, cp_size, q.shape[1], layout)}
        order = [st for st in ring_schedule(cp_rank, cp_size, q.shape[1], layout)]
        fwd = RingForward(q, v.shape[-1], softmax_scale, order, layout)
        next_global = global_ranks[(cp_rank + 1) % cp_size]
        prev_global = global_ranks[(cp_rank - 1) % cp_size]
        cur_k, cur_v = k, v
        saved_k, saved_v, saved_ranks = [], [], []
        for step in range(cp_size):
            kv_rank = (cp_rank - step) % cp_size
            if kv_rank in steps:
                fwd.run_step(steps[kv_rank], cur_k, cur_v)
                saved_k.append(cur_k)
                saved_v.append(cur_v)
                saved_ranks.append(kv_rank)
            if step < cp_size - 1:
                cur_k, cur_v = _ring_send_recv_kv(cur_k, cur_v, next_global, prev_global)
        out, lse = fwd.result()
        ctx.save_for_backward(q, out, lse, *saved_k, *saved_v)
        ctx.conf = (softmax_scale, cp_rank, cp_size, list(global_ranks), layout)
        ctx.saved_ranks = saved_ranks
        return out

    @staticmethod
    def backward(ctx, dout):
        softmax_scale, cp_rank, cp_size, global_ranks, layout = ctx.conf
        saved = ctx.saved_tensors
        q, out, lse = saved[0], saved[1], saved[2]
        n = len(ctx.saved_ranks)
        all_k, all_v = list(saved[3 : 3 + n]), list(saved[3 + n : 3 + 2 * n])
        order = ring_schedule(cp_rank, cp_size, q.shape[1], layout)
        bwd = RingBackward(dout, q, out, lse, softmax_scale, order)
        local_dk = local_dv = None
        remote_dk, remote_dv = {}, {}
        for st, k_j, v_j in zip(order, all_k, all_v):
            dk_j, dv_j = bwd.run_step(st, k_j, v_j)
            if st.kv_rank == cp_rank:
                local_dk, local_dv = dk_j, dv_j
            else:
                remote_dk[st.kv_rank], remote_dv[st.kv_rank] = dk_j, dv_j
        dq = bwd.finish()

        wrap = layout == "zigzag"  # every rank visits every chunk, so distances wrap around
        for d in range(1, cp_size):
            target, source = cp_rank - d, cp_rank + d
            if wrap:
                target, source = target % cp_size, source % cp_size
            ops: List[dist.P2POp] = []
            recv_dk = recv_dv = None
            if 0 <= target and target in remote_dk:
                assert remote_dk[target].is_contiguous() and remote_dv[target].is_contiguous(), (
                    "ring attention remote_dk or remote_dv is not contiguous"
                )
                ops.append(dist.P2POp(dist.isend, remote_dk[target], global_ranks[target]))
                ops.append(dist.P2POp(dist.isend, remote_dv[target], global_ranks[target]))
            if source < cp_size:
                recv_dk, recv_dv = torch.empty_like(local_dk), torch.empty_like(local_dv)
                ops.append(dist.P2POp(dist.irecv, recv_dk, global_ranks[source]))
                ops.append(dist.P2POp(dist.irecv, recv_dv, global_ranks[source]))
            if ops:
                for req in dist.batch_isend_irecv(ops):
                    req.wait()
            if recv_dk is not None:
                local_dk += recv_dk
                local_dv += recv_dv
        return dq, local_dk, local_dv, None, None, None, None, None


def ring_attention_group_func(q, k, v, softmax_scale: float, cp_group, layout: str = "contiguous"):
    """Resolves rank, size and global ranks of `cp_group` (None = a group of one) and applies the ring."""
    if cp_group is None:
        cp_rank, cp_size, global_ranks = 0, 1, [0]
    else:
        cp_rank, cp_size = cp_group.rank(), cp_group.size()
        global_ranks = [dist.distributed_c10d.get_global_rank(cp_group, r) for r in range(cp_size)]
    return RingAttentionDistributedFunc.apply(q, k, v, softmax_scale, cp_rank, cp_size, global_ranks, layout)
