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

from typing import List, Sequence

import torch
import torch.distributed as dist

from pithtrain_amd.operators.ring_attention.local import RingBackward, RingForward, ring_schedule


def _post_exchange(send: Sequence[torch.Tensor], next_global: int, prev_global: int):
    """Starts passing the held tensors to the next rank and receiving the previous rank's.
    Returns (requests, received); the receive buffers are valid after the requests are waited on."""
    for t in send:
        assert t.is_contiguous(), "ring attention send_k or send_v is not contiguous"
    recv = [torch.empty_like(t) for t in send]
    ops = [dist.P2POp(dist.isend, t, next_global) for t in send]
    ops += [dist.P2POp(dist.irecv, t, prev_global) for t in recv]
    return dist.batch_isend_irecv(ops), recv


def _post_kv_exchange(send_k: torch.Tensor, send_v: torch.Tensor, next_global: int, prev_global: int):
    """The K/V pair of the reference's helper; returns (requests, recv_k, recv_v)."""
    reqs, (recv_k, recv_v) = _post_exchange([send_k, send_v], next_global, prev_global)
    return reqs, recv_k, recv_v


def _ring_send_recv_kv(send_k: torch.Tensor, send_v: torch.Tensor, next_global: int, prev_global: int):
    """Passes the held chunk to the next rank and returns the one arriving from the previous rank
    (the reference's blocking helper, pithtrain/operators/ring_attention/standard.py:29-50)."""
    reqs, recv_k, recv_v = _post_kv_exchange(send_k, send_v, next_global, prev_global)
    for req in reqs:
        req.wait()
    return recv_k, recv_v


def _wait(reqs) -> None:
    for req in reqs:
        req.wait()


class RingAttentionDistributedFunc(torch.autograd.Function):
    """Causal ring attention of one rank inside a context-parallel group (any supported head dims).

    The exchange of a step is posted BEFORE the step's kernels are enqueued and waited on after
    them: with the RCCL backend the transfer can then run on the communicator's stream while the
    attention kernels run on the compute stream, so the next chunk (8-25 MB over one xGMI link)
    may arrive behind the current step's compute (by construction; this build has no second GPU to
    measure it on). The reference waits for each exchange before it computes (standard.py:95-98);
    the data each step sees is the same.

    The first seven arguments are the reference's (standard.py:73, mla.py:47) and may be all that is
    passed; the backward then returns the reference's seven gradients (standard.py:189, mla.py:149).
    Up to three more may follow: layout ("contiguous"), rerotate (False) and k_pe (None).

    k_pe: keys in two parts. k is then the 128-feature k_nope and k_pe
    [B, S_l, 64] the rotary part shared by all heads; both travel around the ring (16.5 MB instead
    of the assembled key's 24 MB per chunk of 4096 tokens and 16 heads), and the backward returns
    gradients for both."""

    @staticmethod
    def forward(ctx, q, k, v, softmax_scale, cp_rank, cp_size, global_ranks, *extra):
        assert len(extra) <= 3, "at most layout, rerotate and k_pe may follow the reference's seven arguments"
        layout, rerotate, k_pe = (*extra, *("contiguous", False, None)[len(extra) :])
        ctx.n_extra = len(extra)
        assert k.is_contiguous() and v.is_contiguous(), "ring attention k or v is not contiguous"
        order = ring_schedule(cp_rank, cp_size, q.shape[1], layout)
        steps = {st.kv_rank: st for st in order}
        fwd = RingForward(q, v.shape[-1], softmax_scale, order, layout)
        next_global = global_ranks[(cp_rank + 1) % cp_size]
        prev_global = global_ranks[(cp_rank - 1) % cp_size]
        two_part = k_pe is not None
        ctx.k_pe_4d = two_part and k_pe.dim() == 4
        if two_part:
            k_pe = (k_pe[:, :, 0] if k_pe.dim() == 4 else k_pe).contiguous()
        cur = [k, v] + ([k_pe] if two_part else [])
        saved, saved_ranks = [], []
        for step in range(cp_size):
            pending = None
            if step < cp_size - 1:
                pending = _post_exchange(cur, next_global, prev_global)
            kv_rank = (cp_rank - step) % cp_size
            if kv_rank in steps:
                fwd.run_step(steps[kv_rank], cur[0], cur[1], cur[2] if two_part else None)
                saved.append(cur)
                saved_ranks.append(kv_rank)
            if pending is not None:
                reqs, cur = pending
                _wait(reqs)
        out, lse = fwd.result()
        if rerotate:  # keep only the local chunk; backward sends the chunks around again
            saved, saved_ranks = [[k, v] + ([k_pe] if two_part else [])], [cp_rank]
        ctx.save_for_backward(q, out, lse, *[t for kind in range(len(cur)) for t in (c[kind] for c in saved)])
        ctx.conf = (softmax_scale, cp_rank, cp_size, list(global_ranks), layout)
        ctx.saved_ranks = saved_ranks
        ctx.rerotate = rerotate
        ctx.two_part = two_part
        return out

    @staticmethod
    def backward(ctx, dout):
        softmax_scale, cp_rank, cp_size, global_ranks, layout = ctx.conf
        saved = ctx.saved_tensors
        q, out, lse = saved[0], saved[1], saved[2]
        n, kinds = len(ctx.saved_ranks), 3 if ctx.two_part else 2
        # chunks[j] = [k_j, v_j(, k_pe_j)]
        chunks = {j: [saved[3 + kind * n + i] for kind in range(kinds)] for i, j in enumerate(ctx.saved_ranks)}
        if ctx.rerotate:
            grads = _backward_rerotating(dout, q, out, lse, chunks[cp_rank], softmax_scale, cp_rank, cp_size,
                                         global_ranks, layout)  # fmt: skip
            dk_pe = (grads[3].unsqueeze(2) if ctx.k_pe_4d else grads[3]) if ctx.two_part else None
            return (grads[0], grads[1], grads[2], None, None, None, None, *(None, None, dk_pe)[: ctx.n_extra])
        order = ring_schedule(cp_rank, cp_size, q.shape[1], layout)
        by_rank = {st.kv_rank: st for st in order}
        bwd = RingBackward(dout, q, out, lse, softmax_scale, order)

        def run(j):  # -> [dk_j, dv_j(, dk_pe_j)]
            c = chunks[j]
            return list(bwd.run_step(by_rank[j], c[0], c[1], k_pe_j=c[2] if ctx.two_part else None))

        # Distance 0 is the local chunk. At distance d >= 1 this rank has computed (if the chunk of
        # rank r-d was visible to it) the gradient that belongs to rank r-d, and rank r+d the one
        # that belongs here (standard.py:164-187). With the zigzag layout every rank visits every
        # chunk, so distances wrap around. The exchange of distance d is posted right after the
        # step that produced its payload and overlaps the next step's kernels; arrivals are added
        # in order of distance, so the sum does not depend on timing.
        wrap = layout == "zigzag"
        local = run(cp_rank)
        in_flight = []  # (requests, received gradients, payload kept alive until the send has completed)
        for d in range(1, cp_size):
            target, source = cp_rank - d, cp_rank + d
            if wrap:
                target, source = target % cp_size, source % cp_size
            ops: List[dist.P2POp] = []
            payload = recv = None
            if 0 <= target and target in by_rank:
                payload = run(target)
                for t in payload:
                    assert t.is_contiguous(), "ring attention remote_dk or remote_dv is not contiguous"
                    ops.append(dist.P2POp(dist.isend, t, global_ranks[target]))
            if source < cp_size:
                recv = [torch.empty_like(t) for t in local]
                ops += [dist.P2POp(dist.irecv, t, global_ranks[source]) for t in recv]
            if ops:
                in_flight.append((dist.batch_isend_irecv(ops), recv, payload))
        dq = bwd.finish()
        for reqs, recv, _payload in in_flight:
            _wait(reqs)
            if recv is not None:
                for mine, theirs in zip(local, recv):
                    mine += theirs
        dk_pe = (local[2].unsqueeze(2) if ctx.k_pe_4d else local[2]) if ctx.two_part else None
        # one gradient per forward argument: the reference's seven, then those of the optional ones passed
        return (dq, local[0], local[1], None, None, None, None, *(None, None, dk_pe)[: ctx.n_extra])


def _backward_rerotating(dout, q, out, lse, chunk, softmax_scale, cp_rank, cp_size, global_ranks, layout):
    """Backward that keeps one K/V chunk per rank instead of the cp_size chunks the forward saw
    (the memory cost noted at pithtrain/operators/ring_attention/standard.py:19-21): the chunks
    go around the ring a second time, each with an fp32 (dK, dV) accumulator travelling beside
    it. A rank adds its contribution inside the dK/dV kernel's epilogue and passes chunk and
    accumulator on; after cp_size hops the accumulator is back at the chunk's owner with every
    rank's share, added in ring order (deterministic). The next K/V chunk is requested before the
    step's kernels run; the accumulator can only leave after them.
    Traffic per hop: K, V (bf16) and dK, dV (fp32), against bf16 dK, dV once per remote chunk in
    the saving variant: memory is traded for link time.
    `chunk` = [k, v] or [k_nope, v, k_pe]; returns (dq, dk, dv[, dk_pe])."""
    order = ring_schedule(cp_rank, cp_size, q.shape[1], layout)
    by_rank = {st.kv_rank: st for st in order}
    bwd = RingBackward(dout, q, out, lse, softmax_scale, order)
    next_global = global_ranks[(cp_rank + 1) % cp_size]
    prev_global = global_ranks[(cp_rank - 1) % cp_size]
    two_part = len(chunk) == 3
    cur = list(chunk)
    like = [chunk[0], chunk[1]] + ([chunk[2]] if two_part else [])  # accumulators mirror k, v(, k_pe)
    acc = [torch.zeros(t.shape, dtype=torch.float32, device=t.device) for t in like]
    for step in range(cp_size):
        pending = None
        if step < cp_size - 1:
            pending = _post_exchange(cur, next_global, prev_global)
        kv_rank = (cp_rank - step) % cp_size
        if kv_rank in by_rank:
            bwd.run_step(by_rank[kv_rank], cur[0], cur[1], add_to=tuple(acc), k_pe_j=cur[2] if two_part else None)
        if cp_size > 1:
            reqs, acc = _post_exchange(acc, next_global, prev_global)
            _wait(reqs)
        if pending is not None:
            reqs, cur = pending
            _wait(reqs)
    dq = bwd.finish()
    # after cp_size hops the accumulators held here belong to the local chunk
    return (dq, *[a.to(t.dtype) for a, t in zip(acc, like)])


def ring_attention_group_func(q, k, v, softmax_scale: float, cp_group, layout: str = "contiguous",
                              rerotate: bool = False, k_pe=None):
    """Resolves rank, size and global ranks of `cp_group` (None = a group of one) and applies the ring.
    rerotate=True selects the backward that keeps one K/V chunk per rank (_backward_rerotating);
    k_pe: keys in two parts (k = k_nope), see RingAttentionDistributedFunc."""
    if cp_group is None:
        cp_rank, cp_size, global_ranks = 0, 1, [0]
    else:
        cp_rank, cp_size = cp_group.rank(), cp_group.size()
        global_ranks = [dist.distributed_c10d.get_global_rank(cp_group, r) for r in range(cp_size)]
    return RingAttentionDistributedFunc.apply(q, k, v, softmax_scale, cp_rank, cp_size, global_ranks, layout, rerotate, k_pe)
