"""
Per-chunk attention operators backed by libpith_hip.so (HIP kernels for gfx950).

Drop-in for the raw helpers of pithtrain/operators/mla/triton.py:552-603 (same names, argument
order and return values), generalised beyond the reference's dq=192/dv=128 MHA case to what the
ring needs on both model families:

  * head dims (Dqk, Dv) in {(64, 64), (128, 128), (192, 128)};
  * grouped-query attention (k/v with fewer heads than q; dk/dv sum over the group);
  * non-causal calls with different query and key lengths (zigzag half-chunk steps);
  * arguments that are slices along S of contiguous tensors (no copies are made).

 b : batch size, s : sequence length, h : heads, dq : query/key head dim, dv : value head dim.
Layouts: q/k/v/o/do/dq/dk/dv are BSHD bf16; lse and delta are [b, h, s] fp32; lse is base-2.

The `*_into` functions write into caller-provided tensors and are what the ring drivers use;
the underscore helpers allocate their outputs like the reference does.
"""

import math
import os

import torch
import torch.nn as nn

from pithtrain_amd import _C

SUPPORTED_HEAD_DIMS = ((64, 64), (128, 128), (192, 128))


def _k_pe_strides(k: torch.Tensor, k_pe: torch.Tensor):
    """Checks the shared rotary key part k_pe ([b, s, 64] or [b, s, 1, 64], unit stride along the
    features; it may be a column slice of a wider tensor) against k_nope and returns
    (tensor viewed as [b, s, 64], batch stride, row stride) in elements."""
    if k_pe.dim() == 4:
        assert k_pe.shape[2] == 1, "k_pe must have a single head"
        k_pe = k_pe[:, :, 0]
    b, s = k.shape[0], k.shape[1]
    assert k_pe.dtype == torch.bfloat16 and tuple(k_pe.shape) == (b, s, 64), (
        f"k_pe of shape {tuple(k_pe.shape)} does not match [b={b}, s={s}, 64]"
    )
    assert k_pe.stride(2) == 1, "k_pe is not contiguous along its last dim"
    rs = k_pe.stride(1) if s > 1 else 64
    return k_pe, (k_pe.stride(0) if b > 1 else s * rs), rs


def _check_qkv(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, causal: bool, k_pe=None) -> None:
    _C.require_device(q, k, v)
    assert q.dtype == k.dtype == v.dtype == torch.bfloat16, "q, k, v must be bfloat16"
    assert q.dim() == 4 and k.dim() == 4 and v.dim() == 4, "q, k, v must be [B, S, H, D]"
    d_q, d_v = q.shape[-1], v.shape[-1]
    assert (d_q, d_v) in SUPPORTED_HEAD_DIMS, (
        f"HIP attention kernels support (dq, dv) in {SUPPORTED_HEAD_DIMS}, got dq={d_q} and dv={d_v}"
    )
    if k_pe is not None:
        _C.require_device(q, k_pe)
        assert (d_q, d_v) == (192, 128) and k.shape[-1] == 128, (
            "keys in two parts (k_nope, k_pe) need dq=192, dv=128 and a 128-feature k_nope"
        )
        assert q.shape[2] == k.shape[2], "keys in two parts need as many kv heads as query heads"
    else:
        assert k.shape[-1] == d_q, f"k head dim {k.shape[-1]} != q head dim {d_q}"
    assert k.shape[0] == q.shape[0] and v.shape[0] == q.shape[0], "batch sizes differ"
    assert k.shape[1] == v.shape[1] and k.shape[2] == v.shape[2], "k and v disagree on sequence length or heads"
    assert q.shape[2] % k.shape[2] == 0, f"q heads {q.shape[2]} not a multiple of kv heads {k.shape[2]}"
    if causal:
        assert q.shape[1] == k.shape[1], "causal attention needs equal query and key lengths"


MERGING_HEAD_DIMS = ((128, 128), (192, 128))  # forward kernels that can merge with a running result
FINAL_DQ_HEAD_DIMS = ((128, 128), (192, 128))  # dQ kernels that can emit finished rows as bf16 beside an fp32 accumulator


def attn_fwd_into(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, o: torch.Tensor, lse: torch.Tensor,
    softmax_scale: float, causal: bool, k_pe: torch.Tensor = None,
    prev_o: torch.Tensor = None, acc_o: torch.Tensor = None, o_rows=None, acc_o_rows=None,
) -> None:  # fmt: skip
    """o, lse <- attention(q, k, v). o [b, sq, hq, dv] bf16 and lse [b, hq, sq] fp32 are written.

    With k_pe ([b, skv, 64], the MLA layer's rotary key part, one vector per position shared by all
    heads) k is the 128-feature k_nope and the key of head h is [k[:, :, h] | k_pe]: what
    pithtrain/models/deepseek_v2_lite.py:448-454 materialises is read in place instead.

    With prev_o (bf16 or fp32, shaped like o) the call is a whole ring step: the chunk's result is merged in
    the kernel's epilogue with the running (prev_o, lse) as _online_softmax_combine_log2 would merge them
    (pithtrain/operators/ring_attention/mla.py:27-40); lse is read and overwritten, the merged output goes to
    o (bf16; may be None) and / or acc_o (fp32; may be None); either may be prev_o itself. o_rows / acc_o_rows
    ((begin, end) query rows of this call on multiples of 32, None = all) restrict which rows each output
    receives. Head dims in MERGING_HEAD_DIMS, causal=False only."""
    _check_qkv(q, k, v, causal, k_pe)
    _C.require_device(q, lse)
    b, sq, hq, d_q = q.shape
    _, skv, hkv, d_v = v.shape
    assert lse.dtype == torch.float32 and tuple(lse.shape) == (b, hq, sq), "lse has the wrong dtype or shape"
    lse_bs, lse_hs = _C.bhs_strides(lse, "lse")
    args = _C.AttnFwdArgs(
        q=q.data_ptr(), k=k.data_ptr(), v=v.data_ptr(), o=None, lse=lse.data_ptr(),
        B=b, Sq=sq, Skv=skv, Hq=hq, Hkv=hkv, Dqk=d_q, Dv=d_v,
        q_bs=_C.bshd_batch_stride(q, "q"), k_bs=_C.bshd_batch_stride(k, "k"),
        v_bs=_C.bshd_batch_stride(v, "v"), o_bs=0,
        lse_bs=lse_bs, lse_hs=lse_hs, scale=float(softmax_scale), causal=int(bool(causal)),
        k_pe=None, k_pe_bs=0, k_pe_rs=0,
    )  # fmt: skip
    if o is not None:
        _C.require_device(q, o)
        assert o.dtype == torch.bfloat16 and tuple(o.shape) == (b, sq, hq, d_v), "o has the wrong dtype or shape"
        args.o, args.o_bs = o.data_ptr(), _C.bshd_batch_stride(o, "o")
    if prev_o is not None:
        _C.require_device(q, prev_o)
        assert tuple(prev_o.shape) == (b, sq, hq, d_v), "prev_o has the wrong shape"
        assert o is not None or acc_o is not None, "a merging call needs o or acc_o"
        args.prev_o, args.prev_o_bs, args.prev_o_dtype = prev_o.data_ptr(), _C.bshd_batch_stride(prev_o, "prev_o"), _C.dtype_code(prev_o)
        if acc_o is not None:
            _C.require_device(q, acc_o)
            assert acc_o.dtype == torch.float32 and tuple(acc_o.shape) == (b, sq, hq, d_v), "acc_o has the wrong dtype or shape"
            args.acc_o, args.acc_o_bs = acc_o.data_ptr(), _C.bshd_batch_stride(acc_o, "acc_o")
        if o_rows is not None:
            args.o_rows[0], args.o_rows[1] = o_rows
        if acc_o_rows is not None:
            args.acc_o_rows[0], args.acc_o_rows[1] = acc_o_rows
    else:
        assert o is not None and acc_o is None, "o is required (and acc_o unused) without prev_o"
    if k_pe is not None:
        k_pe, args.k_pe_bs, args.k_pe_rs = _k_pe_strides(k, k_pe)
        args.k_pe = k_pe.data_ptr()
    _C.check(_C.lib().pith_attn_fwd(_C.byref(args), _C.current_stream(q)))


def attn_bwd_delta_into(out: torch.Tensor, dout: torch.Tensor, delta: torch.Tensor) -> None:
    """delta[b, h, s] <- sum_d out * dout (fp32)."""
    _C.require_device(out, dout, delta)
    assert out.dtype == dout.dtype == torch.bfloat16 and out.shape == dout.shape, "out/dout mismatch"
    b, s, h, d_v = out.shape
    assert delta.dtype == torch.float32 and tuple(delta.shape) == (b, h, s), "delta has the wrong dtype or shape"
    d_bs, d_hs = _C.bhs_strides(delta, "delta")
    args = _C.AttnDeltaArgs(
        o=out.data_ptr(), dout=dout.data_ptr(), delta=delta.data_ptr(), B=b, S=s, H=h, D=d_v,
        o_bs=_C.bshd_batch_stride(out, "out"), dout_bs=_C.bshd_batch_stride(dout, "dout"),
        delta_bs=d_bs, delta_hs=d_hs,
    )  # fmt: skip
    _C.check(_C.lib().pith_attn_bwd_delta(_C.byref(args), _C.current_stream(out)))


def _bwd_args(q, k, v, dout, lse, delta, softmax_scale, causal, k_pe=None) -> _C.AttnBwdArgs:
    _check_qkv(q, k, v, causal, k_pe)
    _C.require_device(q, dout, lse, delta)
    b, sq, hq, d_q = q.shape
    _, skv, hkv, d_v = v.shape
    assert dout.dtype == torch.bfloat16 and tuple(dout.shape) == (b, sq, hq, d_v), "dout has the wrong dtype or shape"
    for name, t in (("lse", lse), ("delta", delta)):
        assert t.dtype == torch.float32 and tuple(t.shape) == (b, hq, sq), f"{name} has the wrong dtype or shape"
    lse_bs, lse_hs = _C.bhs_strides(lse, "lse")
    assert _C.bhs_strides(delta, "delta") == (lse_bs, lse_hs), "lse and delta must share strides"
    kpe_ptr, kpe_bs, kpe_rs = None, 0, 0
    if k_pe is not None:
        k_pe, kpe_bs, kpe_rs = _k_pe_strides(k, k_pe)
        kpe_ptr = k_pe.data_ptr()
    # q / dout (and k / v) may be the same range of consecutive heads of wider tensors
    (q_bs, q_rh), (dout_bs, do_rh) = _C.bshd_head_range_strides(q, "q"), _C.bshd_head_range_strides(dout, "dout")
    (k_bs, k_rh), (v_bs, v_rh) = _C.bshd_head_range_strides(k, "k"), _C.bshd_head_range_strides(v, "v")
    assert q_rh == do_rh and k_rh == v_rh, "q / dout (k / v) must be the same head range of equally wide tensors"
    assert k_pe is None or (q_rh == hq and k_rh == hkv), "keys in two parts cannot be combined with a head range"
    return _C.AttnBwdArgs(
        k_pe=kpe_ptr, k_pe_bs=kpe_bs, k_pe_rs=kpe_rs, dk_pe=None, dk_pe_bs=0,
        q=q.data_ptr(), k=k.data_ptr(), v=v.data_ptr(), dout=dout.data_ptr(),
        lse=lse.data_ptr(), delta=delta.data_ptr(), dq=None, dk=None, dv=None,
        B=b, Sq=sq, Skv=skv, Hq=hq, Hkv=hkv, Dqk=d_q, Dv=d_v,
        q_bs=q_bs, k_bs=k_bs, v_bs=v_bs, dout_bs=dout_bs,
        dq_bs=0, dk_bs=0, dv_bs=0, lse_bs=lse_bs, lse_hs=lse_hs,
        scale=float(softmax_scale), causal=int(bool(causal)),
        dq_dtype=_C.PITH_BF16, dkv_dtype=_C.PITH_BF16, accumulate_dq=0, accumulate_dkv=0,
        workspace=None, workspace_bytes=0, ds=None, ds_bytes=0,
        q_row_heads=q_rh, kv_row_heads=k_rh,
    )  # fmt: skip


def attn_bwd_ds_bytes(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, causal: bool = False) -> int:
    """Bytes of the dS hand-over buffer for one chunk pair (0: these head dims have no hand-over path,
    both backward calls then recompute the scores). A causal pair needs about half: only the tiles at
    or below the diagonal are kept."""
    b, sq, hq, d_q = q.shape
    args = _C.AttnBwdArgs(B=b, Sq=sq, Skv=k.shape[1], Hq=hq, Hkv=k.shape[2], Dqk=d_q, Dv=v.shape[-1], causal=int(bool(causal)))
    return int(_C.lib().pith_attn_bwd_ds_bytes(_C.byref(args)))


def _set_ds(args, ds: torch.Tensor, like: torch.Tensor) -> None:
    if ds is None:
        return
    _C.require_device(like, ds)
    assert ds.dtype == torch.uint8 and ds.is_contiguous() and ds.data_ptr() % 256 == 0, "ds must be a contiguous, 256-byte aligned uint8 buffer"
    args.ds, args.ds_bytes = ds.data_ptr(), ds.numel()


# The dS hand-over (head dims 128/128) makes the backward of a chunk pair 3-6 % faster at the price of a
# transient buffer of Sq*Skv*Hq*B*2 bytes while the pair's two kernels run (about half under the causal mask).
# Policy: the buffer never exceeds DS_BUFFER_LIMIT_BYTES nor DS_BUFFER_FREE_FRACTION of the device memory that is
# free right now; a chunk pair that needs more is processed one group of kv heads (with their query heads) after
# the other through one buffer of the bounded size; when not even one kv head fits, or the allocation fails, the
# two kernels recompute the scores as the reference's do (pithtrain/operators/mla/triton.py:130-266), which needs
# no scratch at all.
DS_BUFFER_LIMIT_BYTES = int(float(os.environ.get("PITHTRAIN_AMD_DS_BUFFER_LIMIT_GB", "4")) * (1 << 30))
DS_BUFFER_FREE_FRACTION = 0.5
_DS_ROWS_PER_WORKGROUP = 512  # query rows a workgroup of the dS-reading dQ kernel owns
_compute_units = {}


def _device_compute_units(device: torch.device) -> int:
    idx = device.index if device.index is not None else torch.cuda.current_device()
    if idx not in _compute_units:
        info = _C.DeviceInfo()
        _C.check(_C.lib().pith_device_info(idx, _C.byref(info)))
        _compute_units[idx] = max(int(info.compute_units), 1)
    return _compute_units[idx]


def _ds_budget_bytes(device: torch.device) -> int:
    """What a hand-over buffer may take right now: the configured limit, and at most a fraction of the
    memory that is free on the device or cached (unused) by torch's allocator."""
    free, _ = torch.cuda.mem_get_info(device)
    cached = torch.cuda.memory_reserved(device) - torch.cuda.memory_allocated(device)
    return min(DS_BUFFER_LIMIT_BYTES, int((free + max(cached, 0)) * DS_BUFFER_FREE_FRACTION))


def ds_plan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, causal: bool = False):
    """How the backward of one chunk pair uses the dS hand-over: (kv heads per slab, bytes of the buffer),
    or None when both kernels should recompute (no hand-over path for these head dims, the dS-reading dQ
    kernel would have fewer workgroups than the device has compute units, or not even one kv head fits the
    budget)."""
    need = attn_bwd_ds_bytes(q, k, v, causal)
    if need == 0:
        return None
    b, sq, hq, _ = q.shape
    hkv = k.shape[2]
    budget = _ds_budget_bytes(q.device)
    per_kv_head = need // hkv
    heads = hkv
    while heads > 1 and per_kv_head * heads > budget:
        heads -= 1
        while hkv % heads:
            heads -= 1
    if per_kv_head * heads > budget:
        return None
    if -(-sq // _DS_ROWS_PER_WORKGROUP) * (hq // hkv) * heads * b < _device_compute_units(q.device):
        return None
    return heads, per_kv_head * heads


def ds_buffer(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, causal: bool = False):
    """A dS hand-over buffer for the WHOLE chunk pair from torch's caching allocator, or None when
    ds_plan says the pair should recompute or be processed in slabs, or when the allocation fails."""
    plan = ds_plan(q, k, v, causal)
    if plan is None or plan[0] != k.shape[2]:
        return None
    return _try_alloc(plan[1], q.device)


def _try_alloc(nbytes: int, device: torch.device):
    try:
        return torch.empty(nbytes, dtype=torch.uint8, device=device)
    except torch.cuda.OutOfMemoryError:
        return None


def attn_bwd_pair_into(
    q, k, v, dout, lse, delta, dq: torch.Tensor, dk: torch.Tensor, dv: torch.Tensor, softmax_scale: float, causal: bool,
    accumulate_dq: bool = False, accumulate_dkv: bool = False, k_pe: torch.Tensor = None, dk_pe: torch.Tensor = None,
    handover: bool = True, zero_tail: int = 0, dq_final: torch.Tensor = None, dq_final_rows=None,
) -> int:  # fmt: skip
    """Both backward calls of one chunk pair: dk, dv, then dq (see attn_bwd_dkdv_into / attn_bwd_dq_into).
    The dS hand-over between them is decided here (ds_plan), so a buffer can never reach the dQ call without
    the dK/dV call that fills it. Returns the bytes of hand-over scratch used (0: both kernels recomputed)."""
    plan = ds_plan(q, k, v, causal) if handover and k_pe is None else None
    buf = _try_alloc(plan[1], q.device) if plan is not None else None
    hkv = k.shape[2]
    if buf is None or plan[0] == hkv:
        attn_bwd_dkdv_into(q, k, v, dout, lse, delta, dk, dv, softmax_scale, causal, accumulate=accumulate_dkv,
                           k_pe=k_pe, dk_pe=dk_pe, ds=buf, zero_tail=zero_tail)  # fmt: skip
        attn_bwd_dq_into(q, k, v, dout, lse, delta, dq, softmax_scale, causal, accumulate=accumulate_dq, k_pe=k_pe, ds=buf,
                         dq_final=dq_final, dq_final_rows=dq_final_rows)  # fmt: skip
        return 0 if buf is None else buf.numel()
    # one group of kv heads after the other, each with its query heads, through the same buffer (the
    # kernels of successive slabs are ordered by the stream)
    group = q.shape[2] // hkv
    for h0 in range(0, hkv, plan[0]):
        kv_h, q_h = slice(h0, h0 + plan[0]), slice(h0 * group, (h0 + plan[0]) * group)
        qs, ds_, ls, dl = q[:, :, q_h], dout[:, :, q_h], lse[:, q_h], delta[:, q_h]
        attn_bwd_dkdv_into(qs, k[:, :, kv_h], v[:, :, kv_h], ds_, ls, dl, dk[:, :, kv_h], dv[:, :, kv_h],
                           softmax_scale, causal, accumulate=accumulate_dkv, ds=buf, zero_tail=zero_tail)  # fmt: skip
        attn_bwd_dq_into(qs, k[:, :, kv_h], v[:, :, kv_h], ds_, ls, dl, dq[:, :, q_h], softmax_scale, causal,
                         accumulate=accumulate_dq, ds=buf, dq_final=None if dq_final is None else dq_final[:, :, q_h],
                         dq_final_rows=dq_final_rows)  # fmt: skip
    return buf.numel()


def attn_bwd_dkdv_into(
    q, k, v, dout, lse, delta, dk: torch.Tensor, dv: torch.Tensor, softmax_scale: float, causal: bool,
    accumulate: bool = False, k_pe: torch.Tensor = None, dk_pe: torch.Tensor = None, ds: torch.Tensor = None,
    zero_tail: int = 0,
) -> None:  # fmt: skip
    """dk, dv <- (or +=, with accumulate) the gradients of this chunk pair; bf16 or fp32 outputs.
    zero_tail: dk and dv are row ranges [:skv] of tensors with at least skv + zero_tail rows, and the kernel
    also clears those rows behind them (not with accumulate, not dk_pe).
    With k_pe (see attn_fwd_into) dk is the gradient of k_nope and dk_pe [b, skv, 64] (contiguous rows,
    same dtype as dk) receives the gradient of k_pe, summed over heads in head order.
    ds: uint8 buffer of attn_bwd_ds_bytes(q, k, v, causal) bytes; the kernel leaves its dS tiles there for an
    attn_bwd_dq_into call on the same chunk pair with the same buffer."""
    args = _bwd_args(q, k, v, dout, lse, delta, softmax_scale, causal, k_pe)
    _set_ds(args, ds, q)
    _C.require_device(q, dk, dv)
    assert dk.shape == k.shape and dv.shape == v.shape and dk.dtype == dv.dtype, "dk/dv must match k/v"
    if k_pe is not None:
        assert dk_pe is not None, "keys in two parts need a dk_pe tensor"
        _C.require_device(q, dk_pe)
        b, s = k.shape[0], k.shape[1]
        assert tuple(dk_pe.shape) == (b, s, 64) and dk_pe.dtype == dk.dtype, "dk_pe must be [b, skv, 64] in dk's dtype"
        assert dk_pe.stride(2) == 1 and (s == 1 or dk_pe.stride(1) == 64), "dk_pe rows are not contiguous"
        args.dk_pe = dk_pe.data_ptr()
        args.dk_pe_bs = dk_pe.stride(0) if b > 1 else s * 64
    args.dk, args.dv = dk.data_ptr(), dv.data_ptr()
    (args.dk_bs, dk_rh), (args.dv_bs, dv_rh) = _C.bshd_head_range_strides(dk, "dk"), _C.bshd_head_range_strides(dv, "dv")
    assert dk_rh == dv_rh == args.kv_row_heads, "dk / dv must be laid out like k / v"
    args.dkv_dtype = _C.dtype_code(dk)
    args.accumulate_dkv = int(bool(accumulate))
    args.dkv_zero_tail = int(zero_tail)
    # Scratch for the head-split partial sums; the caching allocator makes this a pointer bump,
    # and stream ordering keeps the block alive until the kernels that use it have run.
    need = _C.lib().pith_attn_bwd_dkdv_workspace_bytes(_C.byref(args))
    workspace = None
    if need > 0:
        workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
        args.workspace, args.workspace_bytes = workspace.data_ptr(), need
    _C.check(_C.lib().pith_attn_bwd_dkdv(_C.byref(args), _C.current_stream(q)))


def attn_bwd_dq_into(
    q, k, v, dout, lse, delta, dq: torch.Tensor, softmax_scale: float, causal: bool, accumulate: bool = False,
    k_pe: torch.Tensor = None, ds: torch.Tensor = None, dq_final: torch.Tensor = None, dq_final_rows=None,
) -> None:  # fmt: skip
    """dq <- (or +=, with accumulate) the query gradient of this chunk pair; bf16 or fp32 output.
    dq_final (bf16, laid out like an fp32 dq; head dims in FINAL_DQ_HEAD_DIMS): rows dq_final_rows ((begin, end)
    on multiples of 32, None = all) receive their complete value, what dq held included when accumulating,
    rounded to bf16 in dq_final instead of dq.
    ds: the buffer an attn_bwd_dkdv_into call on the same chunk pair has just filled; dq is then
    computed from those dS tiles without recomputing the scores."""
    args = _bwd_args(q, k, v, dout, lse, delta, softmax_scale, causal, k_pe)
    _set_ds(args, ds, q)
    _C.require_device(q, dq)
    assert dq.shape == q.shape, "dq must match q"
    args.dq = dq.data_ptr()
    args.dq_bs, dq_rh = _C.bshd_head_range_strides(dq, "dq")
    assert dq_rh == args.q_row_heads, "dq must be laid out like q"
    args.dq_dtype = _C.dtype_code(dq)
    args.accumulate_dq = int(bool(accumulate))
    if dq_final is not None:
        _C.require_device(q, dq_final)
        assert dq_final.dtype == torch.bfloat16 and dq_final.shape == q.shape, "dq_final must be a bf16 tensor shaped like q"
        args.dq_final_bs, fin_rh = _C.bshd_head_range_strides(dq_final, "dq_final")
        assert fin_rh == args.q_row_heads, "dq_final must be laid out like q"
        args.dq_final = dq_final.data_ptr()
        if dq_final_rows is not None:
            args.dq_final_rows[0], args.dq_final_rows[1] = dq_final_rows
    _C.check(_C.lib().pith_attn_bwd_dq(_C.byref(args), _C.current_stream(q)))


# ---------------------------------------------------------------------------------------------
# Reference-named helpers (pithtrain/operators/mla/triton.py:552-603)


def _mla_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, softmax_scale: float, causal: bool = True,
             *, k_pe: torch.Tensor = None):  # fmt: skip
    """Raw attention forward. Returns (out, lse) with lse in log2 scale. Keyword k_pe: keys in two
    parts (k = k_nope), see attn_fwd_into."""
    (b, s, h, _), dv_dim = q.shape, v.shape[-1]
    o = torch.empty((b, s, h, dv_dim), dtype=torch.bfloat16, device=q.device)
    lse = torch.empty((b, h, s), dtype=torch.float32, device=q.device)
    attn_fwd_into(q, k, v, o, lse, softmax_scale, causal, k_pe)
    return o, lse


def _mla_bwd_preprocess(out: torch.Tensor, dout: torch.Tensor):
    """Phase 1: delta = rowsum(out * dout). Called once with combined_out."""
    b, s, h, _ = out.shape
    delta = torch.empty((b, h, s), dtype=torch.float32, device=out.device)
    attn_bwd_delta_into(out, dout, delta)
    return delta


def _mla_bwd_dk_dv(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, dout: torch.Tensor,
                   lse: torch.Tensor, delta: torch.Tensor, softmax_scale: float, causal: bool = True,
                   *, k_pe: torch.Tensor = None):  # fmt: skip
    """Phase 2: compute dK and dV using external lse and delta. Returns (dk, dv), or with keyword k_pe
    (keys in two parts, k = k_nope) (dk_nope, dv, dk_pe)."""
    dk = torch.empty_like(k)
    dv_out = torch.empty_like(v)
    if k_pe is None:
        attn_bwd_dkdv_into(q, k, v, dout, lse, delta, dk, dv_out, softmax_scale, causal)
        return dk, dv_out
    dk_pe = torch.empty((k.shape[0], k.shape[1], 64), dtype=k.dtype, device=k.device)
    attn_bwd_dkdv_into(q, k, v, dout, lse, delta, dk, dv_out, softmax_scale, causal, k_pe=k_pe, dk_pe=dk_pe)
    return dk, dv_out, dk_pe


def _mla_bwd_dq(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, dout: torch.Tensor,
                lse: torch.Tensor, delta: torch.Tensor, softmax_scale: float, causal: bool = True,
                *, k_pe: torch.Tensor = None):  # fmt: skip
    """Phase 3: compute dQ using external lse and delta. Returns dq."""
    dq_out = torch.empty_like(q)
    attn_bwd_dq_into(q, k, v, dout, lse, delta, dq_out, softmax_scale, causal, k_pe=k_pe)
    return dq_out


# ---------------------------------------------------------------------------------------------
# Single-device attention as torch.library custom ops, so that layers compiled with
# torch.compile(fullgraph=True) keep working: the reference wraps its Triton launches the same
# way (pithtrain/operators/mla/triton.py:445-508). Two ops (forward, backward), fake
# implementations that only produce shapes, and an autograd formula tying them together.


@torch.library.custom_op("pithtrain_amd::attn_fwd", mutates_args=())
def _attn_fwd_op(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, softmax_scale: float,
                 causal: bool) -> tuple[torch.Tensor, torch.Tensor]:  # fmt: skip
    return _mla_fwd(q.contiguous(), k.contiguous(), v.contiguous(), softmax_scale, causal)


@_attn_fwd_op.register_fake
def _(q, k, v, softmax_scale, causal):
    b, sq, hq, _ = q.shape
    return q.new_empty((b, sq, hq, v.shape[-1])), q.new_empty((b, hq, sq), dtype=torch.float32)


@torch.library.custom_op("pithtrain_amd::attn_bwd", mutates_args=())
def _attn_bwd_op(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, o: torch.Tensor, lse: torch.Tensor,
                 dout: torch.Tensor, softmax_scale: float,
                 causal: bool) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:  # fmt: skip
    q, k, v, o, dout = q.contiguous(), k.contiguous(), v.contiguous(), o.contiguous(), dout.contiguous()
    delta = _mla_bwd_preprocess(o, dout)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    attn_bwd_pair_into(q, k, v, dout, lse, delta, dq, dk, dv, softmax_scale, causal)
    return dq, dk, dv


@_attn_bwd_op.register_fake
def _(q, k, v, o, lse, dout, softmax_scale, causal):
    return torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)


def _attn_setup_context(ctx, inputs, output):
    q, k, v, softmax_scale, causal = inputs
    o, lse = output
    ctx.save_for_backward(q, k, v, o, lse)
    ctx.softmax_scale = softmax_scale
    ctx.causal = causal


def _attn_backward(ctx, grad_o, grad_lse):
    q, k, v, o, lse = ctx.saved_tensors
    dq, dk, dv = _attn_bwd_op(q, k, v, o, lse, grad_o, ctx.softmax_scale, ctx.causal)
    return dq, dk, dv, None, None


_attn_fwd_op.register_autograd(_attn_backward, setup_context=_attn_setup_context)


def attention_func(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, softmax_scale: float | None = None,
                   causal: bool = False) -> torch.Tensor:  # fmt: skip
    """Attention on one device (no context parallelism) with autograd: the call that replaces
    flash_attn_func(q, k, v, softmax_scale=..., causal=...) at pithtrain/models/qwen3_30b_a3b.py:424-430.
    q [b, sq, hq, d], k/v [b, skv, hkv, d] bf16 (hq a multiple of hkv); returns o [b, sq, hq, dv] bf16."""
    if softmax_scale is None:
        softmax_scale = q.shape[-1] ** -0.5
    o, _ = _attn_fwd_op(q, k, v, softmax_scale, causal)
    return o


class MLA(nn.Module):
    """
    HIP implementation of the MLA operator (causal, BSHD layout); constructor and forward follow
    pithtrain/operators/mla/pytorch.py:8-34 and pithtrain/operators/mla/triton.py:510-549.
    """

    def __init__(self, h: int, dq: int, dv: int, softmax_scale: float = 0.0):
        super().__init__()
        self.h = h
        self.dq = dq
        self.dv = dv
        self.softmax_scale = softmax_scale if softmax_scale != 0.0 else math.sqrt(1.0 / dq)

    @staticmethod
    def autotune(b: int, s: int, h: int, dq: int, dv: int, softmax_scale: float,
                 include_non_causal: bool = False) -> None:  # fmt: skip
        """Kept for call-site compatibility (pithtrain/tasks/pretrain_language_model.py:497-501):
        the HIP kernels are compiled ahead of time with fixed tilings, so there is nothing to tune;
        only the head dims are validated, as the reference asserts them."""
        assert (dq, dv) in SUPPORTED_HEAD_DIMS, (
            f"HIP attention kernels support (dq, dv) in {SUPPORTED_HEAD_DIMS}, got dq={dq} and dv={dv}"
        )

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
        o, _ = _attn_fwd_op(q, k, v, self.softmax_scale, True)
        return o


__all__ = [
    "MLA", "attention_func", "_mla_fwd", "_mla_bwd_preprocess", "_mla_bwd_dk_dv", "_mla_bwd_dq",
    "attn_fwd_into", "attn_bwd_delta_into", "attn_bwd_dkdv_into", "attn_bwd_dq_into", "attn_bwd_pair_into",
    "ds_plan", "ds_buffer",
]  # fmt: skip
