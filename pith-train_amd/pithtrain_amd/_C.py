"""ctypes binding of libpith_hip.so (declarations in include/pith_hip.h).

There is no fallback: if the library has not been built, or a call returns an error code, an
exception is raised. PyTorch is used only for device memory and streams; every tensor argument
is handed to C as a raw device pointer plus sizes and strides.
"""

import ctypes
import os
from ctypes import POINTER, Structure, byref, c_char_p, c_float, c_int, c_int32, c_int64, c_void_p

import torch

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libpith_hip.so")

PITH_BF16, PITH_F32 = 0, 1
PITH_BASE_2, PITH_BASE_E = 0, 1

PITH_OK = 0
PITH_ERR_NULL_POINTER = -1
PITH_ERR_BAD_SHAPE = -2
PITH_ERR_BAD_DTYPE = -3
PITH_ERR_UNSUPPORTED = -4
PITH_ERR_MISALIGNED = -5
PITH_ERR_LAUNCH = -6


class PithError(RuntimeError):
    """A libpith_hip.so entry point returned a negative status."""

    def __init__(self, code: int, name: str, message: str):
        super().__init__(f"{name} ({code}): {message}")
        self.code = code
        self.name = name


class CombineArgs(Structure):
    _fields_ = [
        ("out1", c_void_p), ("lse1", c_void_p), ("out2", c_void_p), ("lse2", c_void_p),
        ("out", c_void_p), ("lse_out", c_void_p),
        ("dtype1", c_int32), ("dtype2", c_int32), ("dtype_out", c_int32), ("base", c_int32),
        ("B", c_int64), ("S", c_int64), ("H", c_int64), ("D", c_int64),
        ("out1_bs", c_int64), ("out2_bs", c_int64), ("out_bs", c_int64),
        ("lse1_bs", c_int64), ("lse1_hs", c_int64), ("lse2_bs", c_int64), ("lse2_hs", c_int64),
        ("lse_out_bs", c_int64), ("lse_out_hs", c_int64),
    ]  # fmt: skip


class AttnFwdArgs(Structure):
    _fields_ = [
        ("q", c_void_p), ("k", c_void_p), ("v", c_void_p), ("o", c_void_p), ("lse", c_void_p),
        ("B", c_int64), ("Sq", c_int64), ("Skv", c_int64), ("Hq", c_int64), ("Hkv", c_int64),
        ("Dqk", c_int64), ("Dv", c_int64),
        ("q_bs", c_int64), ("k_bs", c_int64), ("v_bs", c_int64), ("o_bs", c_int64),
        ("lse_bs", c_int64), ("lse_hs", c_int64),
        ("scale", c_float), ("causal", c_int32),
        ("k_pe", c_void_p), ("k_pe_bs", c_int64), ("k_pe_rs", c_int64),
        ("prev_o", c_void_p), ("prev_o_bs", c_int64), ("acc_o", c_void_p), ("acc_o_bs", c_int64),
        ("prev_o_dtype", c_int32), ("reserved0", c_int32),
        ("o_rows", c_int64 * 2), ("acc_o_rows", c_int64 * 2),
    ]  # fmt: skip


class AttnDeltaArgs(Structure):
    _fields_ = [
        ("o", c_void_p), ("dout", c_void_p), ("delta", c_void_p),
        ("B", c_int64), ("S", c_int64), ("H", c_int64), ("D", c_int64),
        ("o_bs", c_int64), ("dout_bs", c_int64), ("delta_bs", c_int64), ("delta_hs", c_int64),
    ]  # fmt: skip


class AttnBwdArgs(Structure):
    _fields_ = [
        ("q", c_void_p), ("k", c_void_p), ("v", c_void_p), ("dout", c_void_p),
        ("lse", c_void_p), ("delta", c_void_p), ("dq", c_void_p), ("dk", c_void_p), ("dv", c_void_p),
        ("B", c_int64), ("Sq", c_int64), ("Skv", c_int64), ("Hq", c_int64), ("Hkv", c_int64),
        ("Dqk", c_int64), ("Dv", c_int64),
        ("q_bs", c_int64), ("k_bs", c_int64), ("v_bs", c_int64), ("dout_bs", c_int64),
        ("dq_bs", c_int64), ("dk_bs", c_int64), ("dv_bs", c_int64),
        ("lse_bs", c_int64), ("lse_hs", c_int64),
        ("scale", c_float), ("causal", c_int32),
        ("dq_dtype", c_int32), ("dkv_dtype", c_int32),
        ("accumulate_dq", c_int32), ("accumulate_dkv", c_int32),
        ("workspace", c_void_p), ("workspace_bytes", c_int64),
        ("k_pe", c_void_p), ("k_pe_bs", c_int64), ("k_pe_rs", c_int64),
        ("dk_pe", c_void_p), ("dk_pe_bs", c_int64),
        ("ds", c_void_p), ("ds_bytes", c_int64),
        ("q_row_heads", c_int64), ("kv_row_heads", c_int64),
        ("dkv_zero_tail", c_int64), ("dq_final", c_void_p), ("dq_final_bs", c_int64), ("dq_final_rows", c_int64 * 2),
    ]  # fmt: skip


class NormRopeArgs(Structure):
    _fields_ = [
        ("x", c_void_p), ("weight", c_void_p), ("cos", c_void_p), ("sin", c_void_p), ("dout", c_void_p),
        ("out", c_void_p), ("dweight", c_void_p), ("workspace", c_void_p), ("workspace_bytes", c_int64),
        ("B", c_int64), ("S", c_int64), ("H", c_int64), ("D", c_int64),
        ("x_bs", c_int64), ("out_bs", c_int64), ("dout_bs", c_int64), ("cs_bs", c_int64),
        ("eps", c_float), ("weight_dtype", c_int32),
    ]  # fmt: skip


class MlaAssembleArgs(Structure):
    _fields_ = [
        ("q", c_void_p), ("kv", c_void_p), ("k_pe", c_void_p), ("cos", c_void_p), ("sin", c_void_p),
        ("position_ids", c_void_p), ("q_out", c_void_p), ("k_out", c_void_p), ("v_out", c_void_p),
        ("dq_out", c_void_p), ("dk_out", c_void_p), ("dv_out", c_void_p),
        ("B", c_int64), ("S", c_int64), ("H", c_int64), ("Dn", c_int64), ("Dr", c_int64), ("Dv", c_int64),
        ("P", c_int64), ("q_bs", c_int64), ("kv_bs", c_int64), ("k_pe_bs", c_int64), ("k_pe_rs", c_int64),
        ("pos_bs", c_int64),
    ]  # fmt: skip


class DeviceInfo(Structure):
    _fields_ = [
        ("arch_name", ctypes.c_char * 64), ("compute_units", c_int32), ("lds_bytes_per_workgroup", c_int32),
        ("clock_khz", c_int32), ("supported", c_int32), ("hbm_bytes", c_int64),
    ]  # fmt: skip


# name -> (restype, argtypes); must list every symbol declared in include/pith_hip.h
SYMBOLS = {
    "pith_version": (c_int, []),
    "pith_last_error": (c_char_p, []),
    "pith_error_name": (c_char_p, [c_int]),
    "pith_device_info": (c_int, [c_int, POINTER(DeviceInfo)]),
    "pith_combine": (c_int, [POINTER(CombineArgs), c_void_p]),
    "pith_attn_fwd": (c_int, [POINTER(AttnFwdArgs), c_void_p]),
    "pith_attn_bwd_delta": (c_int, [POINTER(AttnDeltaArgs), c_void_p]),
    "pith_attn_bwd_dkdv": (c_int, [POINTER(AttnBwdArgs), c_void_p]),
    "pith_attn_bwd_dq": (c_int, [POINTER(AttnBwdArgs), c_void_p]),
    "pith_attn_bwd_dkdv_static": (c_int, [POINTER(AttnBwdArgs), c_void_p]),
    "pith_attn_bwd_dkdv_workspace_bytes": (c_int64, [POINTER(AttnBwdArgs)]),
    "pith_attn_bwd_ds_bytes": (c_int64, [POINTER(AttnBwdArgs)]),
    "pith_cast_f32_bf16": (c_int, [c_void_p, c_void_p, c_int64, c_void_p]),
    "pith_norm_rope_fwd": (c_int, [POINTER(NormRopeArgs), c_void_p]),
    "pith_norm_rope_bwd": (c_int, [POINTER(NormRopeArgs), c_void_p]),
    "pith_norm_rope_bwd_workspace_bytes": (c_int64, [POINTER(NormRopeArgs)]),
    "pith_norm_rope_fwd_pair": (c_int, [POINTER(NormRopeArgs), POINTER(NormRopeArgs), c_void_p]),
    "pith_norm_rope_bwd_pair": (c_int, [POINTER(NormRopeArgs), POINTER(NormRopeArgs), c_void_p]),
    "pith_mla_assemble_fwd": (c_int, [POINTER(MlaAssembleArgs), c_void_p]),
    "pith_mla_assemble_bwd": (c_int, [POINTER(MlaAssembleArgs), c_void_p]),
}

_lib = None


def lib() -> ctypes.CDLL:
    """Loads libpith_hip.so once (after torch, so the HIP runtime torch loaded is reused)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m pithtrain_amd.build` "
                "(there is no non-HIP fallback for these operators)"
            )
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SYMBOLS.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


def check(code: int) -> None:
    if code != PITH_OK:
        handle = lib()
        raise PithError(code, handle.pith_error_name(code).decode(), handle.pith_last_error().decode())


def dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return PITH_BF16
    if t.dtype == torch.float32:
        return PITH_F32
    raise TypeError(f"expected a bfloat16 or float32 tensor, got {t.dtype}")


def current_stream(t: torch.Tensor) -> c_void_p:
    return c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def require_device(*tensors: torch.Tensor) -> None:
    dev = tensors[0].device
    if dev.type != "cuda":
        raise RuntimeError(
            f"pithtrain_amd operators run HIP kernels and need tensors on a GPU, got device '{dev}'"
        )
    for t in tensors:
        if t.device != dev:
            raise RuntimeError(f"tensors on different devices: {dev} and {t.device}")


def bshd_batch_stride(t: torch.Tensor, what: str) -> int:
    """Checks that a [B,S,H,D] tensor is contiguous within each batch element (a slice along S
    of a contiguous tensor qualifies) and returns its batch stride in elements."""
    B, S, H, D = t.shape
    sb, ss, sh, sd = t.stride()
    ok = (D == 1 or sd == 1) and (H == 1 or sh == D) and (S == 1 or ss == H * D)
    assert ok, f"{what} is not contiguous"
    return sb if B > 1 else S * H * D


def bshd_head_range_strides(t: torch.Tensor, what: str):
    """Like bshd_batch_stride for a tensor that may also be a range of consecutive heads of a wider
    [B,S,H_total,D] tensor (t = wide[:, s0:s1, h0:h1]); returns (batch stride in elements, heads per row)."""
    B, S, H, D = t.shape
    sb, ss, sh, sd = t.stride()
    row_heads = H if S == 1 else ss // D
    ok = (D == 1 or sd == 1) and (H == 1 or sh == D) and (S == 1 or (ss % D == 0 and row_heads >= H))
    assert ok, f"{what} is not contiguous"
    return (sb if B > 1 else S * row_heads * D), row_heads


def bhs_strides(t: torch.Tensor, what: str):
    """Checks that a [B,H,S] tensor has unit stride along S; returns (batch, head) strides."""
    B, H, S = t.shape
    sb, sh, ss = t.stride()
    assert S == 1 or ss == 1, f"{what} is not contiguous along the sequence"
    return (sb if B > 1 else H * max(sh, S)), (sh if H > 1 else S)


__all__ = [
    "lib", "check", "PithError", "CombineArgs", "AttnFwdArgs", "AttnDeltaArgs", "AttnBwdArgs", "NormRopeArgs", "MlaAssembleArgs", "DeviceInfo", "SYMBOLS",
    "dtype_code", "current_stream", "require_device", "bshd_batch_stride", "bshd_head_range_strides", "bhs_strides", "byref",
]  # fmt: skip
