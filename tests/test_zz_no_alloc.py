"""pith_attn_bwd_dkdv_static, the entry point that allocates nothing: called through the C ABI,
its dK/dV must equal, bit for bit, what pith_attn_bwd_dkdv writes with a caller-provided
workspace (same kernels, same fixed summation order), on two calls in a row, the second with a
smaller input (the built-in scratch then still holds the first call's partial sums)."""

import ctypes
import gc

import pytest
import torch

from pithtrain_amd import _C
from pithtrain_amd.operators.mla.hip import _bwd_args

pytestmark = pytest.mark.gpu


def _inputs(dev, seed, B, Sq, Skv, Hq, Hkv, D):
    g = torch.Generator().manual_seed(seed)
    scale = D**-0.5
    q = (torch.randn(B, Sq, Hq, D, generator=g) * scale).to(torch.bfloat16).to(dev)
    k = (torch.randn(B, Skv, Hkv, D, generator=g) * scale).to(torch.bfloat16).to(dev)
    v = (torch.randn(B, Skv, Hkv, D, generator=g) * scale).to(torch.bfloat16).to(dev)
    dout = torch.randn(B, Sq, Hq, D, generator=g).to(torch.bfloat16).to(dev)
    # any finite lse / delta will do for a comparison of two entry points: realistic magnitudes
    lse = (torch.rand(B, Hq, Sq, generator=g) * 2 + 3).to(dev)
    delta = (torch.randn(B, Hq, Sq, generator=g) * 0.1).to(dev)
    return q, k, v, dout, lse, delta, scale


def _call(entry, args, dk, dv, workspace):
    args.dk, args.dv = dk.data_ptr(), dv.data_ptr()
    args.dk_bs, args.dv_bs = dk[0].numel(), dv[0].numel()
    args.dkv_dtype = _C.dtype_code(dk)
    if workspace is not None:
        args.workspace, args.workspace_bytes = workspace.data_ptr(), workspace.numel()
    else:
        args.workspace, args.workspace_bytes = None, 0
    _C.check(entry(ctypes.byref(args), _C.current_stream(dk)))


@pytest.mark.parametrize("D", [128, 64])
def test_static_scratch_entry_matches_the_workspace_entry(gpu, D):
    lib = _C.lib()
    # (B, Sq, Skv, Hq, Hkv): grouped heads and few key tiles, so the head split is in use; the
    # second call is smaller in every dimension and ragged
    shapes = [(2, 384, 512, 8, 2), (1, 200, 130, 8, 2)]
    for n, (B, Sq, Skv, Hq, Hkv) in enumerate(shapes):
        q, k, v, dout, lse, delta, scale = _inputs(gpu, 42 + n, B, Sq, Skv, Hq, Hkv, D)
        for out_dtype in (torch.bfloat16, torch.float32):
            args = _bwd_args(q, k, v, dout, lse, delta, scale, False)
            need = lib.pith_attn_bwd_dkdv_workspace_bytes(ctypes.byref(args))
            assert need > 0, "the shape was chosen so that the head split (and its scratch) is used"
            ws = torch.empty(need, dtype=torch.uint8, device=gpu)
            want_dk = torch.empty(k.shape, dtype=out_dtype, device=gpu)
            want_dv = torch.empty(v.shape, dtype=out_dtype, device=gpu)
            _call(lib.pith_attn_bwd_dkdv, args, want_dk, want_dv, ws)
            got_dk = torch.full(k.shape, float("nan"), dtype=out_dtype, device=gpu)
            got_dv = torch.full(v.shape, float("nan"), dtype=out_dtype, device=gpu)
            if n == 0 and out_dtype is torch.bfloat16:
                # the address of the built-in scratch is looked up at the first call on a device; make that
                # call before measuring, as a caller under graph capture would
                _call(lib.pith_attn_bwd_dkdv_static, args, got_dk, got_dv, None)
            gc.collect()  # garbage of earlier tests must not be released in the middle of the measurement
            torch.cuda.synchronize()
            free_before, _ = torch.cuda.mem_get_info(gpu)
            torch_before = torch.cuda.memory_allocated(gpu), torch.cuda.memory_reserved(gpu)
            peak_before = torch.cuda.max_memory_allocated(gpu)
            torch.cuda.reset_peak_memory_stats(gpu)
            _call(lib.pith_attn_bwd_dkdv_static, args, got_dk, got_dv, None)
            torch.cuda.synchronize()
            # the call's stated property: it allocates nothing, neither through torch nor from the device
            assert torch.cuda.max_memory_allocated(gpu) <= torch_before[0], "the call allocated through torch"
            assert torch.cuda.memory_reserved(gpu) == torch_before[1]
            assert torch.cuda.mem_get_info(gpu)[0] >= free_before, "device memory was taken during the call"
            del peak_before
            assert torch.isfinite(want_dk.float()).all() and want_dk.float().abs().max() > 0
            assert torch.equal(got_dk, want_dk), f"dK differs (call {n}, {out_dtype})"
            assert torch.equal(got_dv, want_dv), f"dV differs (call {n}, {out_dtype})"


def test_static_scratch_entry_causal_and_accumulate(gpu):
    lib = _C.lib()
    B, S, Hq, Hkv, D = 1, 320, 16, 2, 128
    q, k, v, dout, lse, delta, scale = _inputs(gpu, 7, B, S, S, Hq, Hkv, D)
    # a causal call needs an lse no smaller than the row's true one for P <= 1; take a generous one
    lse = lse + 4
    args = _bwd_args(q, k, v, dout, lse, delta, scale, True)
    args.accumulate_dkv = 1
    need = lib.pith_attn_bwd_dkdv_workspace_bytes(ctypes.byref(args))
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device=gpu)
    base_dk = torch.randn(k.shape, device=gpu)
    base_dv = torch.randn(v.shape, device=gpu)
    want_dk, want_dv = base_dk.clone(), base_dv.clone()
    _call(lib.pith_attn_bwd_dkdv, args, want_dk, want_dv, ws)
    got_dk, got_dv = base_dk.clone(), base_dv.clone()
    _call(lib.pith_attn_bwd_dkdv_static, args, got_dk, got_dv, None)
    torch.cuda.synchronize()
    assert not torch.equal(want_dk, base_dk)
    assert torch.equal(got_dk, want_dk) and torch.equal(got_dv, want_dv)


def test_static_scratch_entry_rejects_what_does_not_fit(gpu):
    lib = _C.lib()
    # A causal call whose head-split partial sums exceed the 64 MiB scratch. How far the heads are split depends
    # on the device's compute-unit count, so the shape is searched for: 4 kv heads x 4 query heads each, growing
    # key counts (on 256 compute units: 6144 keys, 48 key tiles cut 4 ways, 96 MiB). Nothing is launched.
    B, Hq, Hkv, D = 1, 16, 4, 128
    found = None
    for S in range(2048, 16385, 1024):
        q = torch.empty(B, S, Hq, D, dtype=torch.bfloat16, device=gpu)
        k = torch.empty(B, S, Hkv, D, dtype=torch.bfloat16, device=gpu)
        stat = torch.empty(B, Hq, S, device=gpu)
        args = _bwd_args(q, k, k, q, stat, stat, D**-0.5, True)
        if lib.pith_attn_bwd_dkdv_workspace_bytes(ctypes.byref(args)) > 64 << 20:
            found = (S, args, q, k)
            break
    if found is None:
        pytest.skip("no probed shape needs more than the built-in scratch on this device")
    S, args, q, k = found
    dk, dv = torch.empty_like(k), torch.empty_like(k)
    args.dk, args.dv = dk.data_ptr(), dv.data_ptr()
    args.dk_bs, args.dv_bs = dk[0].numel(), dv[0].numel()
    rc = lib.pith_attn_bwd_dkdv_static(ctypes.byref(args), _C.current_stream(dk))
    assert rc == _C.PITH_ERR_UNSUPPORTED
    assert b"built-in scratch" in lib.pith_last_error()
