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


def _post_kv_exchange(send_k: torch.Tensor, send_v: torch.Tensor, next_global: int, prev_global: int):
    """Starts passing the held chunk to the next rank and receiving the previous rank's chunk.
    Returns (requests, recv_k, recv_v); the receive buffers are valid after the requests are waited on."""
    assert send_k.is_contiguous() and send_v.is_contiguous(), "ring attention send_k or send_v is not contiguous"
    recv_k, recv_v = torch.empty_like(send_k), torch.empty_like(send_v)
    ops = [
        dist.P2POp(dist.isend, send_k, next_global),
        dist.P2POp(dist.isend, send_v, next_global),
        dist.P2POp(dist.irecv, recv_k, prev_global),
        dist.P2POp(dist.irecv, recv_v, prev_global),
    ]
    return dist.batch_isend_irecv(ops), recv_k, recv_v


def _ring_send_recv_kv(send_k: torch.Tensor, send_v: torch.Tensor, next_global: int, prev_global: int):
    """Passes the held chunk to the next rank and returns the one arriving from the previous rank
    (the reference's blocking helper, pithtrain/operators/ring_attention/standard.py:29-50)."""
    reqs, recv_k, recv_v = _post_kv_exchange(send_k, send_v, next_global, prev_global)
    for req in reqs:
        req.wait()
    return recv_k, recv_v


class RingAttentionDistributedFunc(torch.autograd.Function):
    """Causal ring attention of one rank inside a context-parallel group (any supported head dims).

    The exchange of a step is posted BEFORE the step's kernels are enqueued and waited on after
    them: with the RCCL backend the transfer runs on the communicator's stream while the
    attention kernels run on the compute stream, so the next chunk (8-25 MB over one xGMI link)
    arrives behind the current step's compute. The reference waits for each exchange before it
    computes (standard.py:95-98); the data each step sees is the same."""

    @staticmethod
    def forward(ctx, q, k, v, softmax_scale, cp_rank, cp_size, global_ranks, layout="contiguous", rerotate=False):
        assert k.is_contiguous() and v.is_contiguous(), "ring attention k or v is not contiguous"
        order = ring_schedule(cp_rank, cp_size, q.shape[1], layout)
        steps = {st.kv_rank: st for st in order}
        fwd = RingForward(q, v.shape[-1], softmax_scale, order, layout)
        next_global = global_ranks[(cp_rank + 1) % cp_size]
        prev_global = global_ranks[(cp_rank - 1) % cp_size]
        cur_k, cur_v = k, v
        saved_k, saved_v, saved_ranks = [], [], []
        for step in range(cp_size):
            pending = None
            if step < cp_size - 1:
                pending = _post_kv_exchange(cur_k, cur_v, next_global, prev_global)
            kv_rank = (cp_rank - step) % cp_size
            if kv_rank in steps:
                fwd.run_step(steps[kv_rank], cur_k, cur_v)
                saved_k.append(cur_k)
                saved_v.append(cur_v)
                saved_ranks.append(kv_rank)
            if pending is not None:
                reqs, cur_k, cur_v = pending
                for req in reqs:
                    req.wait()
        out, lse = fwd.result()
        if rerotate:  # keep only the local chunk; backward sends the chunks around again
            saved_k, saved_v, saved_ranks = [k], [v], [cp_rank]
        ctx.save_for_backward(q, out, lse, *saved_k, *saved_v)
        ctx.conf = (softmax_scale, cp_rank, cp_size, list(global_ranks), layout)
        ctx.saved_ranks = saved_ranks
        ctx.rerotate = rerotate
        return out

    @staticmethod
    def backward(ctx, dout):
        softmax_scale, cp_rank, cp_size, global_ranks, layout = ctx.conf
        saved = ctx.saved_tensors
        q, out, lse = saved[0], saved[1], saved[2]
        if ctx.rerotate:
            dq, dk, dv = _backward_rerotating(dout, q, out, lse, saved[3], saved[4], softmax_scale, cp_rank, cp_size,
                                              global_ranks, layout)  # fmt: skip
            return dq, dk, dv, None, None, None, None, None, None
        n = len(ctx.saved_ranks)
        chunks = {j: (saved[3 + i], saved[3 + n + i]) for i, j in enumerate(ctx.saved_ranks)}
        order = ring_schedule(cp_rank, cp_size, q.shape[1], layout)
        by_rank = {st.kv_rank: st for st in order}
        bwd = RingBackward(dout, q, out, lse, softmax_scale, order)

        # Distance 0 is the local chunk. At distance d >= 1 this rank has computed (if the chunk of
        # rank r-d was visible to it) the gradient that belongs to rank r-d, and rank r+d the one
        # that belongs here (standard.py:164-187). With the zigzag layout every rank visits every
        # chunk, so distances wrap around. The exchange of distance d is posted right after the
        # step that produced its payload and overlaps the next step's kernels; arrivals are added
        # in order of distance, so the sum does not depend on timing.
        wrap = layout == "zigzag"
        local_dk, local_dv = bwd.run_step(by_rank[cp_rank], *chunks[cp_rank])
        in_flight = []  # (requests, recv_dk, recv_dv, payload kept alive until the send has completed)
        for d in range(1, cp_size):
            target, source = cp_rank - d, cp_rank + d
            if wrap:
                target, source = target % cp_size, source % cp_size
            ops: List[dist.P2POp] = []
            payload = recv_dk = recv_dv = None
            if 0 <= target and target in by_rank:
                payload = bwd.run_step(by_rank[target], *chunks[target])
                assert payload[0].is_contiguous() and payload[1].is_contiguous(), (
                    "ring attention remote_dk or remote_dv is not contiguous"
                )
                ops.append(dist.P2POp(dist.isend, payload[0], global_ranks[target]))
                ops.append(dist.P2POp(dist.isend, payload[1], global_ranks[target]))
            if source < cp_size:
                recv_dk, recv_dv = torch.empty_like(local_dk), torch.empty_like(local_dv)
                ops.append(dist.P2POp(dist.irecv, recv_dk, global_ranks[source]))
                ops.append(dist.P2POp(dist.irecv, recv_dv, global_ranks[source]))
            if ops:
                in_flight.append((dist.batch_isend_irecv(ops), recv_dk, recv_dv, payload))
        dq = bwd.finish()
        for reqs, recv_dk, recv_dv, _payload in in_flight:
            for req in reqs:
                req.wait()
            if recv_dk is not None:
                local_dk += recv_dk
                local_dv += recv_dv
        return dq, local_dk, local_dv, None, None, None, None, None, None


def _backward_rerotating(dout, q, out, lse, k, v, softmax_scale, cp_rank, cp_size, global_ranks, layout):
    """Backward that keeps one K/V chunk per rank instead of the cp_size chunks the forward saw
    (the memory cost noted at pithtrain/operators/ring_attention/standard.py:19-21): the chunks
    go around the ring a second time, each with an fp32 (dK, dV) accumulator travelling beside
    it. A rank adds its contribution inside the dK/dV kernel's epilogue and passes chunk and
    accumulator on; after cp_size hops the accumulator is back at the chunk's owner with every
    rank's share, added in ring order (deterministic). The next K/V chunk is requested before the
    step's kernels run; the accumulator can only leave after them.
    Traffic per hop: K, V (bf16) and dK, dV (fp32), against bf16 dK, dV once per remote chunk in
    the saving variant: memory is traded for link time."""
    order = ring_schedule(cp_rank, cp_size, q.shape[1], layout)
    by_rank = {st.kv_rank: st for st in order}
    bwd = RingBackward(dout, q, out, lse, softmax_scale, order)
    next_global = global_ranks[(cp_rank + 1) % cp_size]
    prev_global = global_ranks[(cp_rank - 1) % cp_size]
    cur_k, cur_v = k, v
    acc_dk = torch.zeros(k.shape, dtype=torch.float32, device=k.device)
    acc_dv = torch.zeros(v.shape, dtype=torch.float32, device=v.device)
    for step in range(cp_size):
        pending_kv = None
        if step < cp_size - 1:
            pending_kv = _post_kv_exchange(cur_k, cur_v, next_global, prev_global)
        kv_rank = (cp_rank - step) % cp_size
        if kv_rank in by_rank:
            bwd.run_step(by_rank[kv_rank], cur_k, cur_v, add_to=(acc_dk, acc_dv))
        if cp_size > 1:
            recv_dk, recv_dv = torch.empty_like(acc_dk), torch.empty_like(acc_dv)
            ops = [
                dist.P2POp(dist.isend, acc_dk, next_global),
                dist.P2POp(dist.isend, acc_dv, next_global),
                dist.P2POp(dist.irecv, recv_dk, prev_global),
                dist.P2POp(dist.irecv, recv_dv, prev_global),
            ]
            for req in dist.batch_isend_irecv(ops):
                req.wait()
            acc_dk, acc_dv = recv_dk, recv_dv
        if pending_kv is not None:
            reqs, cur_k, cur_v = pending_kv
            for req in reqs:
                req.wait()
    dq = bwd.finish()
    # after cp_size hops the accumulators held here belong to the local chunk
    return dq, acc_dk.to(k.dtype), acc_dv.to(v.dtype)


def ring_attention_group_func(q, k, v, softmax_scale: float, cp_group, layout: str = "contiguous",
                              rerotate: bool = False):
    """Resolves rank, size and global ranks of `cp_group` (None = a group of one) and applies the ring.
    rerotate=True selects the backward that keeps one K/V chunk per rank (_backward_rerotating)."""
    if cp_group is None:
        cp_rank, cp_size, global_ranks = 0, 1, [0]
    else:
        cp_rank, cp_size = cp_group.rank(), cp_group.size()
        global_ranks = [dist.distributed_c10d.get_global_rank(cp_group, r) for r in range(cp_size)]
    return RingAttentionDistributedFunc.apply(q, k, v, softmax_scale, cp_rank, cp_size, global_ranks, layout, rerotate)
