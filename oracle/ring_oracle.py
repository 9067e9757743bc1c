"""
CPU oracle for the ring-attention hot path — TEST INFRASTRUCTURE ONLY.

This module restates, in plain dense PyTorch on the CPU, the algorithm of PithTrain's
context-parallel ring attention so that the HIP kernels can be checked against it. It is imported
only by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of bench.py; the product
package (pith-train_amd/) never imports it and has no CPU fallback.

Reference files followed (paths relative to the PithTrain tree):
  pithtrain/operators/ring_attention/mla.py:27-40      _online_softmax_combine_log2  -> combine_log2
  pithtrain/operators/ring_attention/standard.py:53-66 _online_softmax_combine       -> combine_ln
  pithtrain/operators/mla/triton.py:32-93, 274-323     chunk forward (exp2 domain)   -> chunk_fwd
  pithtrain/operators/mla/triton.py:101-122            delta = rowsum(O*dO)          -> bwd_delta
  pithtrain/operators/mla/triton.py:130-197, 205-266   chunk backward                -> chunk_bwd
  pithtrain/operators/ring_attention/mla.py:47-88      ring forward loop             -> ring_forward
  pithtrain/operators/ring_attention/mla.py:91-149     ring backward loop            -> ring_backward
The GQA chunk attention of the reference lives in flash-attn (Dao-AILab/flash-attention, version
not pinned by the reference's pyproject.toml; call sites standard.py:91-93,134-153): its published
algorithm is the same softmax attention with kv head = q head // group and a natural-log LSE.

The reference is tiled and rounds P and dS to bf16 before the second matmul; the oracle is dense
and keeps full precision in `dtype` (float64 by default), i.e. it is the exact function the
kernels approximate. Tolerances live in the tests.

How each function is pinned (tests/test_oracle.py), none by retyping its own formula:
  chunk_fwd   : O against torch.nn.functional.scaled_dot_product_attention (library routine) and
                against a per-row brute-force loop; LSE2 against torch.logsumexp; causal row 0 gives
                O[0] = V[0], LSE2[0] = kappa * q0.k0; rows of P sum to one.
  chunk_bwd   : against torch.autograd through an independently written dense attention.
  bwd_delta   : against the identity delta_i = sum_j P_ij dP_ij.
  combine_*   : against an independent logaddexp formulation; the reference's three properties
                (two halves == full, identity with -inf, commutativity); finfo.min initial state.
  ring_*      : O/LSE2/dQ of a rank equal full-sequence causal attention restricted to the rank's
                tokens, and dK/dV summed over ranks equal the full-sequence gradients, for both
                layouts (the design of the reference's tests/test_ring_mla_attention.py:79-108).
"""

import math
from typing import List, Optional, Sequence, Tuple

import torch

LOG2E = math.log2(math.e)


# ---------------------------------------------------------------------------------------------
# combine


def combine_log2(out1, lse1, out2, lse2):
    """mla.py:27-40. out: [B,S,H,D], lse: [B,H,S] (base 2). Result dtype by promotion, as there."""
    max_lse = torch.maximum(lse1, lse2)
    exp1 = torch.exp2(lse1 - max_lse)
    exp2 = torch.exp2(lse2 - max_lse)
    e1 = exp1.transpose(1, 2).unsqueeze(-1)
    e2 = exp2.transpose(1, 2).unsqueeze(-1)
    new_out = ((e1 * out1 + e2 * out2) / (e1 + e2)).contiguous()
    new_lse = max_lse + torch.log2(exp1 + exp2)
    return new_out, new_lse


def combine_ln(out1, lse1, out2, lse2):
    """standard.py:53-66. Same with natural exp/log."""
    max_lse = torch.maximum(lse1, lse2)
    exp1 = torch.exp(lse1 - max_lse)
    exp2 = torch.exp(lse2 - max_lse)
    e1 = exp1.transpose(1, 2).unsqueeze(-1)
    e2 = exp2.transpose(1, 2).unsqueeze(-1)
    new_out = (e1 * out1 + e2 * out2) / (e1 + e2)
    new_lse = max_lse + torch.log(exp1 + exp2)
    return new_out, new_lse


# ---------------------------------------------------------------------------------------------
# chunk attention


def _expand_kv(x: torch.Tensor, hq: int) -> torch.Tensor:
    """[B,S,Hkv,D] -> [B,S,Hq,D]: q head h reads kv head h // (Hq/Hkv)."""
    hkv = x.shape[2]
    return x if hkv == hq else x.repeat_interleave(hq // hkv, dim=2)


def _scores(q, k, scale, causal):
    """kappa-scaled scores in the exp2 domain, [B,H,Sq,Skv]; masked entries are -inf."""
    s = torch.einsum("bihd,bjhd->bhij", q, k) * (scale * LOG2E)
    if causal:
        sq, skv = s.shape[-2:]
        assert sq == skv, "the causal mask of the reference assumes equal lengths (triton.py:75-77)"
        mask = torch.ones(sq, skv, dtype=torch.bool).triu(1)  # key index > query index
        s = s.masked_fill(mask, float("-inf"))
    return s


def chunk_fwd(q, k, v, scale: float, causal: bool, dtype=torch.float64):
    """triton.py:32-93 / 274-323 without tiling. q [B,Sq,Hq,Dqk], k [B,Skv,Hkv,Dqk], v [B,Skv,Hkv,Dv].
    Returns (o [B,Sq,Hq,Dv], lse2 [B,Hq,Sq]) in `dtype`."""
    hq = q.shape[2]
    qd, kd, vd = q.to(dtype), _expand_kv(k.to(dtype), hq), _expand_kv(v.to(dtype), hq)
    s = _scores(qd, kd, scale, causal)
    m = s.amax(dim=-1, keepdim=True)  # running max at the end of the loop (:80-81)
    p = torch.exp2(s - m)  # :83
    l = p.sum(dim=-1, keepdim=True)  # :84-85
    o = torch.einsum("bhij,bjhd->bihd", p / l, vd)  # :88-90
    lse = (torch.log2(l) + m).squeeze(-1)  # :92  (m is already kappa-scaled here)
    return o, lse


def bwd_delta(o, dout, dtype=torch.float64):
    """triton.py:101-122: delta[b,h,s] = sum_d o*do."""
    return (o.to(dtype) * dout.to(dtype)).sum(dim=-1).transpose(1, 2).contiguous()


def chunk_bwd(q, k, v, dout, lse, delta, scale: float, causal: bool, dtype=torch.float64):
    """triton.py:130-197 (dk, dv) and :205-266 (dq) without tiling, against EXTERNAL lse/delta.
    Returns (dq [B,Sq,Hq,Dqk], dk [B,Skv,Hkv,Dqk], dv [B,Skv,Hkv,Dv]); with Hq > Hkv the kv
    gradients are summed over each group."""
    hq, hkv = q.shape[2], k.shape[2]
    qd, dod = q.to(dtype), dout.to(dtype)
    kd, vd = _expand_kv(k.to(dtype), hq), _expand_kv(v.to(dtype), hq)
    s = _scores(qd, kd, scale, causal)
    p = torch.exp2(s - lse.to(dtype).unsqueeze(-1))  # :181 / :253 ; masked entries become 0 (:184)
    dv = torch.einsum("bhij,bihd->bjhd", p, dod)  # :186
    dp = torch.einsum("bihd,bjhd->bhij", dod, vd)  # :188 / :258
    ds = p * (dp - delta.to(dtype).unsqueeze(-1)) * scale  # :189 / :259
    dq = torch.einsum("bhij,bjhd->bihd", ds, kd)  # :262-263
    dk = torch.einsum("bhij,bihd->bjhd", ds, qd)  # :192-193
    if hkv != hq:
        g = hq // hkv
        dk = dk.reshape(*dk.shape[:2], hkv, g, dk.shape[-1]).sum(dim=3)
        dv = dv.reshape(*dv.shape[:2], hkv, g, dv.shape[-1]).sum(dim=3)
    return dq, dk, dv


# ---------------------------------------------------------------------------------------------
# ring schedules


def zigzag_split(x: torch.Tensor, cp_size: int, dim: int = 1) -> List[torch.Tensor]:
    """Rank r owns blocks r and 2C-1-r of the 2C equal blocks of the sequence, in that order."""
    blocks = x.chunk(2 * cp_size, dim=dim)
    return [torch.cat([blocks[r], blocks[2 * cp_size - 1 - r]], dim=dim) for r in range(cp_size)]


def contiguous_split(x: torch.Tensor, cp_size: int, dim: int = 1) -> List[torch.Tensor]:
    """Rank r owns tokens [r*S_l, (r+1)*S_l) (pithtrain/tasks/pretrain_language_model.py:128-133)."""
    return list(x.chunk(cp_size, dim=dim))


def token_positions(cp_rank: int, cp_size: int, s_local: int, layout: str) -> torch.Tensor:
    """Global token index of every local row of rank `cp_rank`."""
    if layout == "contiguous":
        return torch.arange(cp_rank * s_local, (cp_rank + 1) * s_local)
    half = s_local // 2
    return torch.cat(
        [torch.arange(cp_rank * half, (cp_rank + 1) * half),
         torch.arange((2 * cp_size - 1 - cp_rank) * half, (2 * cp_size - cp_rank) * half)]
    )  # fmt: skip


def _steps(cp_rank: int, cp_size: int, s_local: int, layout: str):
    """(kv_rank, causal, q row range, kv row range) per ring step, in arrival order
    kv_rank = (cp_rank - step) % cp_size (mla.py:62-66). Contiguous: only kv_rank <= cp_rank is
    computed (mla.py:64). Zigzag: a lower rank's chunk shows its first half to all local queries;
    a higher rank's chunk is fully visible, but only to the second half of the local queries."""
    half = s_local // 2
    out = []
    for step in range(cp_size):
        j = (cp_rank - step) % cp_size
        if j == cp_rank:
            out.append((j, True, (0, s_local), (0, s_local)))
        elif layout == "contiguous":
            if j < cp_rank:
                out.append((j, False, (0, s_local), (0, s_local)))
        elif j < cp_rank:
            out.append((j, False, (0, s_local), (0, half)))
        else:
            out.append((j, False, (half, s_local), (0, s_local)))
    return out


# ---------------------------------------------------------------------------------------------
# ring forward / backward of one rank, all chunks given (no communication)


def ring_forward(q, k_chunks: Sequence, v_chunks: Sequence, scale: float, cp_rank: int, cp_size: int,
                 layout: str = "contiguous", dtype=torch.float64):  # fmt: skip
    """mla.py:47-88 for one rank. Returns (combined_out [B,S_l,Hq,Dv], combined_lse [B,Hq,S_l]) in `dtype`."""
    B, S, H = q.shape[0], q.shape[1], q.shape[2]
    DV = v_chunks[cp_rank].shape[-1]
    combined_out = torch.zeros((B, S, H, DV), dtype=dtype)  # :49
    combined_lse = torch.full((B, H, S), torch.finfo(torch.float32).min, dtype=dtype)  # :50-52
    for j, causal, (q0, q1), (n0, n1) in _steps(cp_rank, cp_size, S, layout):
        step_out, step_lse = chunk_fwd(q[:, q0:q1], k_chunks[j][:, n0:n1], v_chunks[j][:, n0:n1], scale, causal, dtype)
        new_out, new_lse = combine_log2(combined_out[:, q0:q1], combined_lse[:, :, q0:q1], step_out, step_lse)  # :68-70
        combined_out[:, q0:q1] = new_out
        combined_lse[:, :, q0:q1] = new_lse
    return combined_out, combined_lse


def ring_backward(dout, q, combined_out, combined_lse, k_chunks: Sequence, v_chunks: Sequence, scale: float,
                  cp_rank: int, cp_size: int, layout: str = "contiguous", dtype=torch.float64):  # fmt: skip
    """mla.py:91-122 for one rank (the P2P return of dk/dv, :124-147, is left to the caller).
    Returns (dq, dk_list, dv_list); dk_list[j] is this rank's contribution to chunk j (None when
    the chunk is never visited), zero on rows the rank cannot see."""
    S = q.shape[1]
    delta = bwd_delta(combined_out, dout, dtype)  # :101
    dq = torch.zeros(q.shape, dtype=dtype)  # :103
    dk_list: List[Optional[torch.Tensor]] = [None] * cp_size
    dv_list: List[Optional[torch.Tensor]] = [None] * cp_size
    for j, causal, (q0, q1), (n0, n1) in _steps(cp_rank, cp_size, S, layout):
        dq_s, dk_s, dv_s = chunk_bwd(
            q[:, q0:q1], k_chunks[j][:, n0:n1], v_chunks[j][:, n0:n1], dout[:, q0:q1],
            combined_lse[:, :, q0:q1], delta[:, :, q0:q1], scale, causal, dtype,
        )  # :110-115  # fmt: skip
        dq[:, q0:q1] += dq_s  # :116
        dk_j = torch.zeros(k_chunks[j].shape, dtype=dtype)
        dv_j = torch.zeros(v_chunks[j].shape, dtype=dtype)
        dk_j[:, n0:n1] = dk_s
        dv_j[:, n0:n1] = dv_s
        dk_list[j], dv_list[j] = dk_j, dv_j
    return dq, dk_list, dv_list


# ---------------------------------------------------------------------------------------------
# the timed CPU baseline: the same ring share in fp32 eager PyTorch, blocked to bound memory


def cpu_ring_fwd_bwd(q, k_chunks, v_chunks, dout, scale, cp_rank, cp_size, layout,
                     heads: Optional[Tuple[int, int]] = None, q_block: int = 1024, backward: bool = True):  # fmt: skip
    """Forward + backward of one rank in fp32 on bf16-rounded inputs, for query heads
    [heads[0], heads[1]) only (all when None). Score tiles are [heads, q_block, Skv] at most.
    Returns (out, lse, dq, dk_list, dv_list) restricted to those heads (kv gradients hold only the
    contribution of those query heads). backward=False stops after the forward (the gradients
    returned are then meaningless)."""
    hq, hkv = q.shape[2], k_chunks[cp_rank].shape[2]
    g = hq // hkv
    h0, h1 = heads if heads is not None else (0, hq)
    whole_groups = h0 % g == 0 and h1 % g == 0
    assert whole_groups or h0 // g == (h1 - 1) // g, "head range must cover whole kv groups or lie within one"
    kv0, kv1 = h0 // g, (h1 - 1) // g + 1
    f32 = torch.float32
    qh, doh = q[:, :, h0:h1].to(f32), dout[:, :, h0:h1].to(f32)
    ks = [None if c is None else c[:, :, kv0:kv1].to(f32) for c in k_chunks]
    vs = [None if c is None else c[:, :, kv0:kv1].to(f32) for c in v_chunks]
    S = q.shape[1]
    out = torch.empty((q.shape[0], S, h1 - h0, vs[cp_rank].shape[-1]), dtype=f32)
    lse = torch.empty((q.shape[0], h1 - h0, S), dtype=f32)
    dq = torch.empty_like(qh)
    dk_list = [None if c is None else torch.zeros_like(c) for c in ks]
    dv_list = [None if c is None else torch.zeros_like(c) for c in vs]
    for r0 in range(0, S, q_block):
        r1 = min(S, r0 + q_block)
        # a causal step needs no key beyond the block's last row
        sub = [(j, c, (max(a, r0), min(b, r1)), (n0, min(n1, r1) if c else n1))
               for j, c, (a, b), (n0, n1) in _steps(cp_rank, cp_size, S, layout) if max(a, r0) < min(b, r1)]  # fmt: skip
        # forward over the row block: per-chunk attention merged by the log2 combine
        co = torch.zeros((q.shape[0], r1 - r0, h1 - h0, out.shape[-1]), dtype=f32)
        cl = torch.full((q.shape[0], h1 - h0, r1 - r0), torch.finfo(f32).min, dtype=f32)
        for j, causal, (a, b), (n0, n1) in sub:
            so, sl = _cpu_chunk_fwd(qh[:, a:b], ks[j][:, n0:n1], vs[j][:, n0:n1], scale, causal, a)
            no, nl = combine_log2(co[:, a - r0 : b - r0], cl[:, :, a - r0 : b - r0], so, sl)
            co[:, a - r0 : b - r0], cl[:, :, a - r0 : b - r0] = no, nl
        out[:, r0:r1], lse[:, :, r0:r1] = co, cl
        if not backward:
            continue
        delta = bwd_delta(co.to(torch.bfloat16), doh[:, r0:r1], f32)
        dq[:, r0:r1] = 0
        for j, causal, (a, b), (n0, n1) in sub:
            dq_s, dk_s, dv_s = _cpu_chunk_bwd(qh[:, a:b], ks[j][:, n0:n1], vs[j][:, n0:n1], doh[:, a:b],
                                              cl[:, :, a - r0 : b - r0], delta[:, :, a - r0 : b - r0], scale, causal, a)  # fmt: skip
            dq[:, a:b] += dq_s
            dk_list[j][:, n0:n1] += dk_s
            dv_list[j][:, n0:n1] += dv_s
    return out, lse, dq, dk_list, dv_list


def _cpu_scores(q, k, scale, causal, q_row0):
    s = torch.einsum("bihd,bjhd->bhij", q, k) * (scale * LOG2E)
    if causal:  # rows of a row block sit at q_row0.. inside the chunk; keys start at 0
        qi = torch.arange(q_row0, q_row0 + q.shape[1]).unsqueeze(1)
        kj = torch.arange(k.shape[1]).unsqueeze(0)
        s = s.masked_fill(kj > qi, float("-inf"))
    return s


def _cpu_chunk_fwd(q, k, v, scale, causal, q_row0):
    hq = q.shape[2]
    k, v = _expand_kv(k, hq), _expand_kv(v, hq)
    s = _cpu_scores(q, k, scale, causal, q_row0)
    m = s.amax(dim=-1, keepdim=True)
    p = torch.exp2(s - m)
    l = p.sum(dim=-1, keepdim=True)
    o = torch.einsum("bhij,bjhd->bihd", p / l, v)
    return o, (torch.log2(l) + m).squeeze(-1)


def _cpu_chunk_bwd(q, k, v, dout, lse, delta, scale, causal, q_row0):
    hq, hkv = q.shape[2], k.shape[2]
    ke, ve = _expand_kv(k, hq), _expand_kv(v, hq)
    p = torch.exp2(_cpu_scores(q, ke, scale, causal, q_row0) - lse.unsqueeze(-1))
    dv = torch.einsum("bhij,bihd->bjhd", p, dout)
    ds = p * (torch.einsum("bihd,bjhd->bhij", dout, ve) - delta.unsqueeze(-1)) * scale
    dq = torch.einsum("bhij,bjhd->bihd", ds, ke)
    dk = torch.einsum("bhij,bihd->bjhd", ds, q)
    if hkv != hq:
        g = hq // hkv
        dk = dk.reshape(*dk.shape[:2], hkv, g, dk.shape[-1]).sum(dim=3)
        dv = dv.reshape(*dv.shape[:2], hkv, g, dv.shape[-1]).sum(dim=3)
    return dq, dk, dv
