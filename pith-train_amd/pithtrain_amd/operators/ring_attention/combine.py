"""Online-softmax combine of two partial attention results on the HIP combine kernel.

Both bases of the reference are served by one kernel: base 2 for
pithtrain/operators/ring_attention/mla.py:27-40 and base e for
pithtrain/operators/ring_attention/standard.py:53-66.
"""

import torch

from pithtrain_amd import _C


def combine_into(
    out1: torch.Tensor, lse1: torch.Tensor, out2: torch.Tensor, lse2: torch.Tensor,
    out: torch.Tensor, lse_out: torch.Tensor, base: int = _C.PITH_BASE_2,
) -> None:  # fmt: skip
    """out, lse_out <- merge of (out1, lse1) and (out2, lse2).

    out*: [B, S, H, D] bf16 or fp32 (any mix), lse*: [B, H, S] fp32. All tensors may be slices
    along S of larger contiguous tensors. `out` may be out1 or out2 itself when dtypes match, and
    lse_out may be lse1 or lse2 (every element is read before it is written by the same thread).
    """
    _C.require_device(out1, lse1, out2, lse2, out, lse_out)
    b, s, h, d = out1.shape
    assert out2.shape == out1.shape and out.shape == out1.shape, "out tensors disagree on shape"
    for name, t in (("lse1", lse1), ("lse2", lse2), ("lse_out", lse_out)):
        assert t.dtype == torch.float32 and tuple(t.shape) == (b, h, s), f"{name} must be fp32 [B, H, S]"
    l1, l2, lo = _C.bhs_strides(lse1, "lse1"), _C.bhs_strides(lse2, "lse2"), _C.bhs_strides(lse_out, "lse_out")
    args = _C.CombineArgs(
        out1=out1.data_ptr(), lse1=lse1.data_ptr(), out2=out2.data_ptr(), lse2=lse2.data_ptr(),
        out=out.data_ptr(), lse_out=lse_out.data_ptr(),
        dtype1=_C.dtype_code(out1), dtype2=_C.dtype_code(out2), dtype_out=_C.dtype_code(out), base=base,
        B=b, S=s, H=h, D=d,
        out1_bs=_C.bshd_batch_stride(out1, "out1"), out2_bs=_C.bshd_batch_stride(out2, "out2"),
        out_bs=_C.bshd_batch_stride(out, "out"),
        lse1_bs=l1[0], lse1_hs=l1[1], lse2_bs=l2[0], lse2_hs=l2[1], lse_out_bs=lo[0], lse_out_hs=lo[1],
    )  # fmt: skip
    _C.check(_C.lib().pith_combine(_C.byref(args), _C.current_stream(out1)))


def _combine_new(out1, lse1, out2, lse2, base):
    """Reference calling convention: fresh fp32 outputs whatever the input dtypes."""
    assert lse1.is_contiguous() or lse1.stride(-1) == 1
    new_out = torch.empty(out1.shape, dtype=torch.float32, device=out1.device)
    new_lse = torch.empty(lse1.shape, dtype=torch.float32, device=lse1.device)
    combine_into(out1, lse1, out2, lse2, new_out, new_lse, base)
    return new_out, new_lse


def cast_f32_bf16_into(src: torch.Tensor, dst: torch.Tensor) -> None:
    """dst <- bf16(src), both contiguous with the same number of elements."""
    _C.require_device(src, dst)
    assert src.dtype == torch.float32 and dst.dtype == torch.bfloat16 and src.numel() == dst.numel()
    assert src.is_contiguous() and dst.is_contiguous()
    _C.check(_C.lib().pith_cast_f32_bf16(src.data_ptr(), dst.data_ptr(), src.numel(), _C.current_stream(src)))
