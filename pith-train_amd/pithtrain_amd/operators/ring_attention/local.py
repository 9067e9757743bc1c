"""
One GPU's share of causal ring attention, computed without collectives.

The reference ring (pithtrain/operators/ring_attention/standard.py:73-189, mla.py:47-149) runs
cp_size steps on every rank; at each step the rank holds one K/V chunk, attends its local Q
against it, merges the partial result into a running (out, lse) pair, and passes the chunk on.
Here the chunks a rank would receive are handed in as a list (indexed by the rank that owns
them), and the same per-step work runs back to back on one device: chunk attention forward,
log2-domain combine, and in backward the per-chunk dQ/dK/dV against the combined LSE and
delta = rowsum(dO*O) computed once.

Two token layouts:

  "contiguous"  the reference's: rank r owns tokens [r*S_l, (r+1)*S_l). It computes the causal
                diagonal chunk and full attention against chunks 0..r-1 (standard.py:86-93), so
                work grows with the rank (the imbalance noted at standard.py:16-18).
  "zigzag"      the sequence is cut into 2C blocks and rank r owns blocks r and 2C-1-r, in that
                order. Step 0 is plain causal attention over the local chunk. For a chunk of a
                lower rank j < r only its first block is visible, to every local query; for a
                chunk of a higher rank j > r the whole chunk is visible, but only to the second
                local block. Every rank does the same amount of work.

Running state follows the reference: partial results are merged in fp32 (the type promotion at
mla.py:38) and rounded to bf16 once at the end (mla.py:78); here the last combine that touches a
row range writes bf16 directly, which is the same single rounding. dQ is accumulated over steps
in fp32 inside the dQ kernel's epilogue and rounded once (the reference adds bf16 partials,
mla.py:116). dK/dV of every visited chunk are returned separately, zero where a chunk's rows were
not visible; on a real ring those are what travels back to the owning ranks (standard.py:164-187).

Keys in two parts (MLA): every function below takes optional `k_pe` chunks ([B, S_l, 64], the
rotary key part shared by all heads) beside 128-feature `k` chunks (k_nope). The chunk kernels
then read [k_nope | k_pe] in place of the assembled 192-feature key that the reference builds at
pithtrain/models/deepseek_v2_lite.py:448-454 (with k_pe broadcast to all heads: 24 MB instead of
16.5 MB per chunk of 4096 tokens and 16 heads, also on the wire of a real ring), and the
backward returns dk_nope and the head-summed dk_pe per chunk.
"""

from dataclasses import dataclass
from typing import List, Sequence, Tuple

import torch

from pithtrain_amd import _C
from pithtrain_amd.operators.mla.hip import (
    FINAL_DQ_HEAD_DIMS,
    MERGING_HEAD_DIMS,
    attn_bwd_delta_into,
    attn_bwd_pair_into,
    attn_fwd_into,
)
from pithtrain_amd.operators.ring_attention.combine import cast_f32_bf16_into, combine_into

LAYOUTS = ("contiguous", "zigzag")
# Ring steps after the first merge inside the forward kernel (one launch per step) where the kernels support it;
# False restores chunk forward + combine launch per step (kept for comparison runs).
FUSE_MERGE = True
# The ring backward lets the dQ launch that completes a row range write its bf16 rows (no cast pass at the end)
# where the kernels support it; False restores the fp32 accumulator + cast (kept for comparison runs).
FUSE_FINAL_DQ = True
# The dK/dV launch of a step that sees only the first rows of a chunk clears the other rows of dk / dv itself;
# False restores separate fill launches.
FUSE_ZERO_TAIL = True


@dataclass(frozen=True)
class RingStep:
    """One step of a rank's ring: which chunk, which rows of each side take part, and the mask."""

    kv_rank: int
    causal: bool
    q_rows: Tuple[int, int]  # [start, stop) within the local chunk
    kv_rows: Tuple[int, int]  # [start, stop) within the visited chunk


def ring_schedule(cp_rank: int, cp_size: int, s_local: int, layout: str = "contiguous") -> List[RingStep]:
    """Steps rank `cp_rank` performs, in ring arrival order kv_rank = (cp_rank - step) % cp_size."""
    assert layout in LAYOUTS, f"layout must be one of {LAYOUTS}, got {layout!r}"
    assert 0 <= cp_rank < cp_size
    full = (0, s_local)
    steps = []
    if layout == "zigzag":
        assert s_local % 2 == 0, "zigzag needs an even local sequence length"
        half = s_local // 2
    for step in range(cp_size):
        j = (cp_rank - step) % cp_size
        if j == cp_rank:
            steps.append(RingStep(j, True, full, full))
        elif layout == "contiguous":
            if j < cp_rank:
                steps.append(RingStep(j, False, full, full))
        elif j < cp_rank:
            steps.append(RingStep(j, False, full, (0, half)))
        else:
            steps.append(RingStep(j, False, (half, s_local), full))
    return steps


def zigzag_split(x: torch.Tensor, cp_size: int, dim: int = 1) -> List[torch.Tensor]:
    """Cuts a full-sequence tensor into the per-rank zigzag chunks [block r ; block 2C-1-r]."""
    blocks = x.chunk(2 * cp_size, dim=dim)
    assert len(blocks) == 2 * cp_size, "sequence length must be a multiple of 2 * cp_size"
    return [torch.cat([blocks[r], blocks[2 * cp_size - 1 - r]], dim=dim).contiguous() for r in range(cp_size)]


def zigzag_merge(chunks: Sequence[torch.Tensor], dim: int = 1) -> torch.Tensor:
    """Inverse of zigzag_split."""
    cp_size = len(chunks)
    blocks = [None] * (2 * cp_size)
    for r, c in enumerate(chunks):
        first, second = c.chunk(2, dim=dim)
        blocks[r], blocks[2 * cp_size - 1 - r] = first, second
    return torch.cat(blocks, dim=dim)


def cp_local_slice(x: torch.Tensor, cp_rank: int, cp_size: int, layout: str = "contiguous", dim: int = 1) -> torch.Tensor:
    """The part of a full-sequence tensor (tokens, labels, hidden states) that rank `cp_rank` owns.

    "contiguous" is the reference's slicing (pithtrain/tasks/pretrain_language_model.py:128-133);
    "zigzag" is what the zigzag ring expects: blocks cp_rank and 2*cp_size-1-cp_rank of 2*cp_size."""
    assert layout in LAYOUTS, f"layout must be one of {LAYOUTS}, got {layout!r}"
    n = x.shape[dim]
    if layout == "contiguous":
        assert n % cp_size == 0, "sequence length must be a multiple of cp_size"
        chunk = n // cp_size
        return x.narrow(dim, cp_rank * chunk, chunk)
    assert n % (2 * cp_size) == 0, "sequence length must be a multiple of 2 * cp_size"
    block = n // (2 * cp_size)
    return torch.cat([x.narrow(dim, cp_rank * block, block), x.narrow(dim, (2 * cp_size - 1 - cp_rank) * block, block)], dim=dim)


def cp_position_ids(cp_rank: int, cp_size: int, s_local: int, layout: str = "contiguous", device=None) -> torch.Tensor:
    """[1, s_local] positions, in the full sequence, of the tokens rank `cp_rank` owns: what the
    rotary embedding must see. "contiguous" is the reference's offset
    (pithtrain/models/qwen3_30b_a3b.py:816-821); "zigzag" follows cp_local_slice."""
    full = torch.arange(cp_size * s_local, device=device).unsqueeze(0)
    return cp_local_slice(full, cp_rank, cp_size, layout, dim=1)


def _rows(t: torch.Tensor, rows: Tuple[int, int]) -> torch.Tensor:
    """Row range of a [B, S, H, D] tensor (a view)."""
    return t if rows == (0, t.shape[1]) else t[:, rows[0] : rows[1]]


def _pe_rows(t, rows: Tuple[int, int]):
    """Row range of a [B, S, 64] (or [B, S, 1, 64]) tensor (a view); None passes through."""
    return t if t is None or rows == (0, t.shape[1]) else t[:, rows[0] : rows[1]]


def _lse_rows(t: torch.Tensor, rows: Tuple[int, int]) -> torch.Tensor:
    """Row range of a [B, H, S] tensor (a view)."""
    return t if rows == (0, t.shape[2]) else t[:, :, rows[0] : rows[1]]


class RingForward:
    """Running (out, lse) of one rank's forward; feed it the schedule's steps in order."""

    def __init__(self, q: torch.Tensor, dv_dim: int, softmax_scale: float, steps: Sequence[RingStep], layout: str):
        assert q.is_contiguous(), "ring attention q is not contiguous"
        B, S, H, _ = q.shape
        self.q, self.scale, self.steps = q, softmax_scale, list(steps)
        self.out = torch.empty((B, S, H, dv_dim), dtype=torch.bfloat16, device=q.device)
        self.lse = torch.empty((B, H, S), dtype=torch.float32, device=q.device)
        # Row ranges are merged independently. `pending[r]` counts the merges still to come for
        # range r; while it is non-zero the running value of the range lives in the fp32
        # accumulator (or still in `out`, in bf16, before its first merge); the last merge of a
        # range writes bf16 into `out`.
        self.ranges = [(0, S)] if layout == "contiguous" else [(0, S // 2), (S // 2, S)]
        self.pending = {r: sum(self._covers(st, r) for st in self.steps[1:]) for r in self.ranges}
        self.in_acc = {r: False for r in self.ranges}
        self.acc = None
        if any(n > 1 for n in self.pending.values()):
            self.acc = torch.empty((B, S, H, dv_dim), dtype=torch.float32, device=q.device)
        # Steps after the first merge into the running state inside the forward kernel's epilogue where the
        # kernels for these head dims can (fuse_merge); otherwise the chunk result goes to step_out / step_lse
        # and a combine launch merges it.
        self.fuse_merge = FUSE_MERGE and (q.shape[-1], dv_dim) in MERGING_HEAD_DIMS
        self.dv_dim = dv_dim
        self.step_out = self.step_lse = None
        self.done = 0

    def _step_buffers(self):
        if self.step_out is None:
            B, S, H, _ = self.q.shape
            self.step_out = torch.empty((B, S, H, self.dv_dim), dtype=torch.bfloat16, device=self.q.device)
            self.step_lse = torch.empty(B * H * S, dtype=torch.float32, device=self.q.device)
        return self.step_out, self.step_lse

    @staticmethod
    def _covers(step: RingStep, r: Tuple[int, int]) -> bool:
        return step.q_rows[0] <= r[0] and r[1] <= step.q_rows[1]

    def run_step(self, st: RingStep, k_j: torch.Tensor, v_j: torch.Tensor, k_pe_j: torch.Tensor = None) -> None:
        assert st == self.steps[self.done], "ring steps must be fed in schedule order"
        assert k_j.is_contiguous() and v_j.is_contiguous(), "ring attention k or v is not contiguous"
        B, S, H, _ = self.q.shape
        self.done += 1
        if self.done == 1:
            # Step 0 is the diagonal chunk and covers every local row: merging it into the
            # reference's initial state (zeros, finfo.min) returns it unchanged, so it is written
            # straight into the running tensors.
            assert st.causal and st.q_rows == (0, S)
            attn_fwd_into(self.q, k_j, v_j, self.out, self.lse, self.scale, True, k_pe_j)
            return
        covered = [r for r in self.ranges if self._covers(st, r)]
        assert covered and (covered[0][0], covered[-1][1]) == st.q_rows, "a step's query rows must be whole row ranges"
        if self.fuse_merge and len({self.in_acc[r] for r in covered}) == 1:
            # One launch: chunk attention + merge. The running value of all covered ranges sits in the same tensor
            # (the schedule merges them equally often up to here); ranges that are merged again later get the fp32
            # result, ranges whose last merge this is get bf16. A launch that covers both kinds tells the kernel
            # which rows go where when the boundaries allow it (multiples of 32 rows); otherwise it writes both
            # outputs for every row, and the surplus rows of either tensor are overwritten later or never read.
            prev = self.acc if self.in_acc[covered[0]] else self.out
            last = [r for r in covered if self.pending[r] == 1]
            more = [r for r in covered if self.pending[r] > 1]
            o_rows = acc_rows = None
            if last and more:
                spans = [(rs[0][0] - st.q_rows[0], rs[-1][1] - st.q_rows[0]) for rs in (last, more)]
                whole = all(sum(r[1] - r[0] for r in rs) == sp[1] - sp[0] for rs, sp in zip((last, more), spans))
                if whole and all(sp[0] % 32 == 0 and (sp[1] % 32 == 0 or sp[1] == st.q_rows[1] - st.q_rows[0]) for sp in spans):
                    o_rows, acc_rows = spans
            attn_fwd_into(_rows(self.q, st.q_rows), _rows(k_j, st.kv_rows), _rows(v_j, st.kv_rows),
                          _rows(self.out, st.q_rows) if last else None, _lse_rows(self.lse, st.q_rows), self.scale, False,
                          _pe_rows(k_pe_j, st.kv_rows), prev_o=_rows(prev, st.q_rows),
                          acc_o=_rows(self.acc, st.q_rows) if more else None, o_rows=o_rows, acc_o_rows=acc_rows)  # fmt: skip
            for r in covered:
                self.pending[r] -= 1
                self.in_acc[r] = self.pending[r] > 0
            return
        n_q = st.q_rows[1] - st.q_rows[0]
        step_out, step_lse = self._step_buffers()
        so = step_out[:, :n_q]
        sl = step_lse[: B * H * n_q].view(B, H, n_q)
        attn_fwd_into(_rows(self.q, st.q_rows), _rows(k_j, st.kv_rows), _rows(v_j, st.kv_rows), so, sl,
                      self.scale, False, _pe_rows(k_pe_j, st.kv_rows))  # fmt: skip
        # Ranges in the same state are merged by one launch.
        groups = {}
        for r in self.ranges:
            if self._covers(st, r):
                groups.setdefault((self.in_acc[r], self.pending[r] == 1), []).append(r)
        for (from_acc, last), rs in groups.items():
            lo, hi = rs[0][0], rs[-1][1]
            rel = (lo - st.q_rows[0], hi - st.q_rows[0])
            src = _rows(self.acc if from_acc else self.out, (lo, hi))
            dst = _rows(self.out if last else self.acc, (lo, hi))
            run_lse = _lse_rows(self.lse, (lo, hi))
            combine_into(src, run_lse, _rows(so, rel), _lse_rows(sl, rel), dst, run_lse, _C.PITH_BASE_2)
            for r in rs:
                self.pending[r] -= 1
                self.in_acc[r] = not last

    def result(self) -> Tuple[torch.Tensor, torch.Tensor]:
        assert self.done == len(self.steps), "not every ring step has run"
        return self.out, self.lse


class RingBackward:
    """Gradient state of one rank's backward; feed it the schedule's steps in order."""

    def __init__(self, dout, q, out, lse, softmax_scale: float, steps: Sequence[RingStep]):
        self.dout = dout.contiguous()
        self.q, self.lse, self.scale, self.steps = q, lse, softmax_scale, list(steps)
        B, S, H, _ = q.shape
        # Rows between two boundaries of the steps' query ranges receive the same contributions; `dq_left` counts
        # those still to come. Where the kernels can, the step that brings a range's last contribution writes its
        # bf16 rows of dq itself (and leaves them out of the fp32 accumulator); ranges finished that way need no
        # cast at the end.
        cuts = sorted({0, S} | {r for st in self.steps for r in st.q_rows})
        self.dq_ranges = list(zip(cuts[:-1], cuts[1:]))
        self.dq_left = {r: sum(st.q_rows[0] <= r[0] and r[1] <= st.q_rows[1] for st in self.steps) for r in self.dq_ranges}
        self.dq_done_in_kernel = set()
        self.final_in_kernel = FUSE_FINAL_DQ and (q.shape[-1], out.shape[-1]) in FINAL_DQ_HEAD_DIMS and len(self.steps) > 1
        # delta from the COMBINED output, once (pithtrain/operators/ring_attention/mla.py:101).
        self.delta = torch.empty((B, H, S), dtype=torch.float32, device=q.device)
        attn_bwd_delta_into(out, self.dout, self.delta)
        self.dq = torch.empty_like(q)
        single = len(self.steps) == 1
        self.dq_acc = self.dq if single else torch.empty(q.shape, dtype=torch.float32, device=q.device)
        self.done = 0
        self.handover = True  # False: every step's two kernels recompute the scores (no dS scratch)
        self.scratch_bytes = 0  # largest dS hand-over buffer a step has used so far

    def run_step(self, st: RingStep, k_j: torch.Tensor, v_j: torch.Tensor, add_to=None, k_pe_j: torch.Tensor = None):
        """Returns (dk_j, dv_j), this rank's contribution to chunk st.kv_rank's gradients; with
        k_pe_j (keys in two parts) (dk_nope_j, dv_j, dk_pe_j).

        With add_to=(dk_acc, dv_acc[, dk_pe_acc]) (tensors shaped like the chunk, bf16 or fp32) the
        contribution is ADDED to them inside the kernel epilogue instead, and they are returned: the
        form a gradient accumulator that travels around the ring with its chunk needs."""
        assert st == self.steps[self.done], "ring steps must be fed in schedule order"
        if k_pe_j is not None and k_pe_j.dim() == 4:
            k_pe_j = k_pe_j[:, :, 0]
        dk_pe_j = None
        zero_tail = 0
        if add_to is None:
            dk_j, dv_j = torch.empty_like(k_j), torch.empty_like(v_j)
            outs = [dk_j, dv_j]
            if k_pe_j is not None:
                dk_pe_j = torch.empty((k_j.shape[0], k_j.shape[1], k_pe_j.shape[-1]), dtype=k_j.dtype, device=k_j.device)
                outs.append(dk_pe_j)
            if st.kv_rows != (0, k_j.shape[1]):  # rows of the chunk this rank cannot see get no gradient
                # rows behind the visible ones are cleared by the dK/dV launch itself; anything else here
                in_kernel = FUSE_ZERO_TAIL and st.kv_rows[0] == 0
                zero_tail = k_j.shape[1] - st.kv_rows[1] if in_kernel else 0
                for t in outs if not in_kernel else outs[2:]:  # (the launch does not clear dk_pe)
                    t[:, : st.kv_rows[0]].zero_()
                    t[:, st.kv_rows[1] :].zero_()
        else:
            dk_j, dv_j = add_to[0], add_to[1]
            dk_pe_j = add_to[2] if k_pe_j is not None else None
            assert dk_j.shape == k_j.shape and dv_j.shape == v_j.shape, "accumulators must be shaped like the chunk"
        qs, ds = _rows(self.q, st.q_rows), _rows(self.dout, st.q_rows)
        ks, vs = _rows(k_j, st.kv_rows), _rows(v_j, st.kv_rows)
        ls, dl = _lse_rows(self.lse, st.q_rows), _lse_rows(self.delta, st.q_rows)
        pes = _pe_rows(k_pe_j, st.kv_rows)
        # dK/dV, then dQ; the pair helper decides whether the dK/dV kernel leaves its dS tiles for the dQ
        # kernel (head dims 128/128, bounded scratch) or both kernels recompute the scores.
        # Step 0 covers every row and initialises the dQ accumulator; later steps add to their rows.
        covered = [r for r in self.dq_ranges if st.q_rows[0] <= r[0] and r[1] <= st.q_rows[1]]
        for r in covered:
            self.dq_left[r] -= 1
        final = final_rows = None
        if self.final_in_kernel:
            last = [r for r in covered if self.dq_left[r] == 0]
            span = (last[0][0] - st.q_rows[0], last[-1][1] - st.q_rows[0]) if last else None
            n_q = st.q_rows[1] - st.q_rows[0]
            if last and sum(r[1] - r[0] for r in last) == span[1] - span[0] and span[0] % 32 == 0 and (
                span[1] % 32 == 0 or span[1] == n_q
            ):
                final, final_rows = _rows(self.dq, st.q_rows), span
                self.dq_done_in_kernel.update(last)
        self.scratch_bytes = max(self.scratch_bytes, attn_bwd_pair_into(
            qs, ks, vs, ds, ls, dl, _rows(self.dq_acc, st.q_rows), _rows(dk_j, st.kv_rows), _rows(dv_j, st.kv_rows),
            self.scale, st.causal, accumulate_dq=self.done > 0, accumulate_dkv=add_to is not None, k_pe=pes,
            dk_pe=_pe_rows(dk_pe_j, st.kv_rows), handover=self.handover, zero_tail=zero_tail,
            dq_final=final, dq_final_rows=final_rows))  # fmt: skip
        self.done += 1
        return (dk_j, dv_j) if k_pe_j is None else (dk_j, dv_j, dk_pe_j)

    def finish(self) -> torch.Tensor:
        assert self.done == len(self.steps), "not every ring step has run"
        if self.dq_acc is not self.dq:
            todo = [r for r in self.dq_ranges if r not in self.dq_done_in_kernel]
            if len(todo) == len(self.dq_ranges):
                cast_f32_bf16_into(self.dq_acc, self.dq)
            else:
                for r in todo:  # ranges no launch could finish (boundaries off the 32-row grid)
                    for b in range(self.dq.shape[0]):
                        cast_f32_bf16_into(self.dq_acc[b, r[0] : r[1]], self.dq[b, r[0] : r[1]])
        return self.dq


def ring_forward_local(
    q: torch.Tensor, k_chunks: Sequence[torch.Tensor], v_chunks: Sequence[torch.Tensor],
    softmax_scale: float, cp_rank: int, cp_size: int, layout: str = "contiguous",
    k_pe_chunks: Sequence[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:  # fmt: skip
    """Forward of rank `cp_rank`: returns (out bf16 [B, S_l, Hq, Dv], lse fp32 base-2 [B, Hq, S_l]).

    k_chunks[j] / v_chunks[j] are the K/V chunks owned by rank j (entries the schedule never
    visits may be None); with k_pe_chunks the keys come in two parts (k_chunks = k_nope)."""
    steps = ring_schedule(cp_rank, cp_size, q.shape[1], layout)
    fwd = RingForward(q, v_chunks[cp_rank].shape[-1], softmax_scale, steps, layout)
    for st in steps:
        fwd.run_step(st, k_chunks[st.kv_rank], v_chunks[st.kv_rank],
                     None if k_pe_chunks is None else k_pe_chunks[st.kv_rank])  # fmt: skip
    return fwd.result()


def ring_backward_local(
    dout: torch.Tensor, q: torch.Tensor, out: torch.Tensor, lse: torch.Tensor,
    k_chunks: Sequence[torch.Tensor], v_chunks: Sequence[torch.Tensor],
    softmax_scale: float, cp_rank: int, cp_size: int, layout: str = "contiguous",
    k_pe_chunks: Sequence[torch.Tensor] = None,
):  # fmt: skip
    """Backward of rank `cp_rank`. Returns (dq, dk_list, dv_list): dq bf16 like q; dk_list[j] and
    dv_list[j] are this rank's contribution to the gradients of chunk j (None if never visited).
    With k_pe_chunks (keys in two parts) a fourth list holds the contributions to every k_pe chunk."""
    steps = ring_schedule(cp_rank, cp_size, q.shape[1], layout)
    bwd = RingBackward(dout, q, out, lse, softmax_scale, steps)
    dk_list: List[torch.Tensor] = [None] * cp_size
    dv_list: List[torch.Tensor] = [None] * cp_size
    dpe_list: List[torch.Tensor] = [None] * cp_size
    for st in steps:
        j = st.kv_rank
        if k_pe_chunks is None:
            dk_list[j], dv_list[j] = bwd.run_step(st, k_chunks[j], v_chunks[j])
        else:
            dk_list[j], dv_list[j], dpe_list[j] = bwd.run_step(st, k_chunks[j], v_chunks[j], k_pe_j=k_pe_chunks[j])
    if k_pe_chunks is None:
        return bwd.finish(), dk_list, dv_list
    return bwd.finish(), dk_list, dv_list, dpe_list


class RingAttentionLocalFunc(torch.autograd.Function):
    """autograd wrapper of one rank's ring share; gradients flow to q and to every visited chunk.
    *kv holds cp_size K chunks and cp_size V chunks, optionally followed by cp_size k_pe chunks
    (keys in two parts)."""

    @staticmethod
    def forward(ctx, q, softmax_scale, cp_rank, cp_size, layout, *kv):
        assert len(kv) in (2 * cp_size, 3 * cp_size), "expected cp_size K chunks, cp_size V chunks[, cp_size k_pe chunks]"
        k_chunks, v_chunks = list(kv[:cp_size]), list(kv[cp_size : 2 * cp_size])
        pe_chunks = list(kv[2 * cp_size :]) if len(kv) == 3 * cp_size else None
        out, lse = ring_forward_local(q, k_chunks, v_chunks, softmax_scale, cp_rank, cp_size, layout, pe_chunks)
        visited = sorted({st.kv_rank for st in ring_schedule(cp_rank, cp_size, q.shape[1], layout)})
        kinds = [k_chunks, v_chunks] + ([pe_chunks] if pe_chunks is not None else [])
        ctx.save_for_backward(q, out, lse, *[kind[j] for kind in kinds for j in visited])
        ctx.visited = visited
        ctx.n_kinds = len(kinds)
        ctx.conf = (softmax_scale, cp_rank, cp_size, layout)
        return out

    @staticmethod
    def backward(ctx, dout):
        softmax_scale, cp_rank, cp_size, layout = ctx.conf
        saved = ctx.saved_tensors
        q, out, lse = saved[0], saved[1], saved[2]
        n = len(ctx.visited)
        kinds = [[None] * cp_size for _ in range(ctx.n_kinds)]
        for which in range(ctx.n_kinds):
            for i, j in enumerate(ctx.visited):
                kinds[which][j] = saved[3 + which * n + i]
        grads = ring_backward_local(
            dout, q, out, lse, kinds[0], kinds[1], softmax_scale, cp_rank, cp_size, layout,
            kinds[2] if ctx.n_kinds == 3 else None,
        )
        return (grads[0], None, None, None, None, *[g for kind in grads[1:] for g in kind])


def ring_attention_local(
    q: torch.Tensor, k_chunks: Sequence[torch.Tensor], v_chunks: Sequence[torch.Tensor],
    softmax_scale: float, cp_rank: int, cp_size: int, layout: str = "contiguous",
    k_pe_chunks: Sequence[torch.Tensor] = None,
) -> torch.Tensor:  # fmt: skip
    """Differentiable one-GPU ring share for either model family (head dims pick the kernels).
    With k_pe_chunks the keys come in two parts (k_chunks = k_nope, see the module docstring)."""
    assert len(k_chunks) == cp_size and len(v_chunks) == cp_size
    assert k_pe_chunks is None or len(k_pe_chunks) == cp_size
    # Chunks the schedule never visits may be None; autograd needs tensors, so they are replaced
    # by empty placeholders that receive no gradient.
    visited = {st.kv_rank for st in ring_schedule(cp_rank, cp_size, q.shape[1], layout)}
    empty = q.new_empty(0)
    ks = [k_chunks[j] if j in visited else empty for j in range(cp_size)]
    vs = [v_chunks[j] if j in visited else empty for j in range(cp_size)]
    pes = [] if k_pe_chunks is None else [k_pe_chunks[j] if j in visited else empty for j in range(cp_size)]
    return RingAttentionLocalFunc.apply(q, softmax_scale, cp_rank, cp_size, layout, *ks, *vs, *pes)
