"""The forward kernel's merging epilogue: one launch computes a chunk's attention and merges it with the running
(output, LSE2) of the same rows, which the reference does as attention call + _online_softmax_combine_log2
(pithtrain/operators/ring_attention/mla.py:27-40, 64-70). Expected values: the fp64 oracle's chunk forward followed
by the oracle's combine."""

import ctypes

import pytest
import torch

from helpers import check_bf16_result, check_lse, norm_max_err
from oracle import ring_oracle as R
from pithtrain_amd import _C
from pithtrain_amd.operators.mla.hip import attn_fwd_into
from pithtrain_amd.operators.ring_attention.combine import combine_into

pytestmark = pytest.mark.gpu

SHAPES = [  # B, Sq, Skv, Hq, Hkv, Dqk
    (1, 256, 256, 4, 2, 128),      # 128-row workgroups (wave pairs split the keys)
    (2, 333, 200, 4, 4, 128),      # ragged rows and keys
    (1, 2048, 512, 32, 4, 128),    # 256-row workgroups
    (1, 1000, 320, 40, 8, 128),    # 256-row workgroups, ragged last block
    (1, 384, 384, 4, 4, 192),      # MLA, 128-row workgroups
    (1, 1024, 300, 48, 48, 192),   # MLA, 256-row workgroups
    (1, 1, 1, 1, 1, 128),
]


def _case(B, Sq, Skv, Hq, Hkv, Dqk, seed=42):
    g = torch.Generator().manual_seed(seed)
    scale = Dqk**-0.5
    q = torch.randn(B, Sq, Hq, Dqk, generator=g).to(torch.bfloat16)
    k = torch.randn(B, Skv, Hkv, Dqk, generator=g).to(torch.bfloat16)
    v = torch.randn(B, Skv, Hkv, 128, generator=g).to(torch.bfloat16)
    prev = torch.randn(B, Sq, Hq, 128, generator=g)
    prev_lse = torch.rand(B, Hq, Sq, generator=g) * 16 - 4
    return q, k, v, prev, prev_lse, scale


@pytest.mark.parametrize("prev_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("B,Sq,Skv,Hq,Hkv,Dqk", SHAPES)
def test_merging_forward_matches_oracle(gpu, B, Sq, Skv, Hq, Hkv, Dqk, prev_dtype):
    q, k, v, prev, prev_lse, scale = _case(B, Sq, Skv, Hq, Hkv, Dqk)
    prev = prev.to(prev_dtype)
    co, cl = R.chunk_fwd(q, k, v, scale, False)
    # centre the running LSE on the chunk's so that both sides carry weight
    prev_lse = prev_lse - 6 + cl.float().mean()
    want_o, want_l = R.combine_log2(prev.double(), prev_lse.double(), co, cl)
    qd, kd, vd = q.to(gpu), k.to(gpu), v.to(gpu)
    for outs in ("both", "bf16", "fp32"):
        pd, ld = prev.to(gpu), prev_lse.to(gpu)
        o = torch.full((B, Sq, Hq, 128), float("nan"), dtype=torch.bfloat16, device=gpu) if outs != "fp32" else None
        acc = torch.full((B, Sq, Hq, 128), float("nan"), dtype=torch.float32, device=gpu) if outs != "bf16" else None
        attn_fwd_into(qd, kd, vd, o, ld, scale, False, prev_o=pd, acc_o=acc)
        check_lse(ld, want_l, f"merged LSE2 ({outs})")
        if o is not None:
            check_bf16_result(o, want_o, f"merged O bf16 ({outs})")
        if acc is not None:
            check_bf16_result(acc, want_o, f"merged O fp32 ({outs})")
            if o is not None:  # the bf16 copy is the rounded fp32 copy
                assert torch.equal(acc.to(torch.bfloat16), o)


@pytest.mark.parametrize("Dqk", [128, 192])
def test_merging_in_place_and_against_the_two_launch_path(gpu, Dqk):
    """Outputs may be the running tensors themselves; the result agrees with chunk forward + combine launch to
    fp32 rounding (the combine then sees a bf16-rounded chunk result, the fused epilogue the fp32 accumulators:
    the fused form is the closer one to the exact value)."""
    B, Sq, Skv, Hq, Hkv = 1, 777, 512, 8, 8 if Dqk == 192 else 2
    q, k, v, prev, prev_lse, scale = _case(B, Sq, Skv, Hq, Hkv, Dqk, seed=9)
    co, cl = R.chunk_fwd(q, k, v, scale, False)
    prev_lse = prev_lse - 6 + cl.float().mean()
    want_o, want_l = R.combine_log2(prev.double(), prev_lse.double(), co, cl)
    qd, kd, vd = q.to(gpu), k.to(gpu), v.to(gpu)
    # fp32 running output merged in place
    acc, ld = prev.to(gpu), prev_lse.to(gpu)
    attn_fwd_into(qd, kd, vd, None, ld, scale, False, prev_o=acc, acc_o=acc)
    check_bf16_result(acc, want_o, "in-place fp32")
    check_lse(ld, want_l, "in-place LSE2")
    # bf16 running output merged in place
    pb = prev.to(torch.bfloat16)
    want_b, _ = R.combine_log2(pb.double(), prev_lse.double(), co, cl)
    ob, lb = pb.to(gpu), prev_lse.to(gpu)
    attn_fwd_into(qd, kd, vd, ob, lb, scale, False, prev_o=ob)
    check_bf16_result(ob, want_b, "in-place bf16")
    # two launches: forward into a chunk result, then the combine kernel
    so = torch.empty(B, Sq, Hq, 128, dtype=torch.bfloat16, device=gpu)
    sl = torch.empty(B, Hq, Sq, dtype=torch.float32, device=gpu)
    attn_fwd_into(qd, kd, vd, so, sl, scale, False)
    two = torch.empty(B, Sq, Hq, 128, dtype=torch.float32, device=gpu)
    l2 = prev_lse.to(gpu)
    combine_into(prev.to(gpu), l2, so, sl, two, l2, _C.PITH_BASE_2)
    assert norm_max_err(acc, two) < 6e-3
    assert (ld - l2).abs().max().item() < 1e-4
    assert norm_max_err(acc, want_o) <= norm_max_err(two, want_o) * 1.05 + 1e-6


@pytest.mark.parametrize("Sq,split", [(1024, 512), (800, 544), (320, 32)])
def test_row_ranges_send_each_row_to_one_output(gpu, Sq, split):
    """o_rows / acc_o_rows: the first rows get the bf16 output only, the others the fp32 output only; rows outside
    an output's range keep what they held."""
    B, Skv, Hq, Hkv, Dqk = 1, 256, 8, 2, 128
    q, k, v, prev, prev_lse, scale = _case(B, Sq, Skv, Hq, Hkv, Dqk, seed=5)
    co, cl = R.chunk_fwd(q, k, v, scale, False)
    prev_lse = prev_lse - 6 + cl.float().mean()
    pb = prev.to(torch.bfloat16)
    want_o, want_l = R.combine_log2(pb.double(), prev_lse.double(), co, cl)
    o, ld = pb.to(gpu), prev_lse.to(gpu)
    acc = torch.full((B, Sq, Hq, 128), 7.0, dtype=torch.float32, device=gpu)
    attn_fwd_into(q.to(gpu), k.to(gpu), v.to(gpu), o, ld, scale, False, prev_o=o, acc_o=acc,
                  o_rows=(0, split), acc_o_rows=(split, Sq))  # fmt: skip
    check_lse(ld, want_l, "LSE2")
    check_bf16_result(o[:, :split], want_o[:, :split], "bf16 rows")
    check_bf16_result(acc[:, split:], want_o[:, split:], "fp32 rows")
    assert torch.equal(o[:, split:].cpu(), pb[:, split:]), "rows outside o_rows must stay untouched"
    assert (acc[:, :split] == 7.0).all(), "rows outside acc_o_rows must stay untouched"
    with pytest.raises(_C.PithError, match="PITH_ERR_BAD_SHAPE"):
        attn_fwd_into(q.to(gpu), k.to(gpu), v.to(gpu), o, ld, scale, False, prev_o=o, acc_o=acc, o_rows=(0, 17))


def test_initial_state_and_empty_sides(gpu):
    """Merging into the reference's initial state (zeros, finfo.min: mla.py:49-52) returns the chunk result; a
    running side with LSE -inf likewise (tests/test_online_softmax_combine_log2.py:68-84 of the reference)."""
    B, Sq, Skv, Hq, Hkv, Dqk = 1, 320, 192, 4, 2, 128
    q, k, v, _, _, scale = _case(B, Sq, Skv, Hq, Hkv, Dqk, seed=3)
    qd, kd, vd = q.to(gpu), k.to(gpu), v.to(gpu)
    so = torch.empty(B, Sq, Hq, 128, dtype=torch.bfloat16, device=gpu)
    sl = torch.empty(B, Hq, Sq, dtype=torch.float32, device=gpu)
    attn_fwd_into(qd, kd, vd, so, sl, scale, False)
    for init in (torch.finfo(torch.float32).min, float("-inf")):
        acc = torch.zeros(B, Sq, Hq, 128, dtype=torch.float32, device=gpu)
        o = torch.empty(B, Sq, Hq, 128, dtype=torch.bfloat16, device=gpu)
        lse = torch.full((B, Hq, Sq), init, dtype=torch.float32, device=gpu)
        attn_fwd_into(qd, kd, vd, o, lse, scale, False, prev_o=acc, acc_o=acc)
        assert torch.equal(o, so), "merging into the empty initial state must return the chunk result"
        assert (lse - sl).abs().max().item() < 1e-5


def test_merging_is_refused_where_no_kernel_has_it(gpu):
    lib = _C.lib()
    t = torch.zeros(1, 64, 2, 64, dtype=torch.bfloat16, device=gpu)
    lse = torch.zeros(1, 2, 64, device=gpu)
    with pytest.raises(_C.PithError, match="PITH_ERR_UNSUPPORTED"):
        attn_fwd_into(t, t, t, t.clone(), lse, 0.1, False, prev_o=t.clone())  # head dims (64, 64)
    q = torch.zeros(1, 64, 2, 128, dtype=torch.bfloat16, device=gpu)
    with pytest.raises(_C.PithError, match="PITH_ERR_UNSUPPORTED"):
        attn_fwd_into(q, q, q, q.clone(), lse, 0.1, True, prev_o=q.clone())  # causal
    args = _C.AttnFwdArgs(q=q.data_ptr(), k=q.data_ptr(), v=q.data_ptr(), o=None, lse=lse.data_ptr(), B=1, Sq=64, Skv=64,
                          Hq=2, Hkv=2, Dqk=128, Dv=128, q_bs=64 * 256, k_bs=64 * 256, v_bs=64 * 256, o_bs=64 * 256, lse_bs=128,
                          lse_hs=64, scale=0.1, causal=0)  # fmt: skip
    assert lib.pith_attn_fwd(ctypes.byref(args), None) == _C.PITH_ERR_NULL_POINTER  # neither o nor (prev_o, acc_o)
    args.prev_o, args.prev_o_bs, args.prev_o_dtype = q.data_ptr(), 64 * 256, 7
    args.o = q.data_ptr()
    assert lib.pith_attn_fwd(ctypes.byref(args), None) == _C.PITH_ERR_BAD_DTYPE


@pytest.mark.parametrize("layout", ["contiguous", "zigzag"])
@pytest.mark.parametrize("Dqk,Hq,Hkv", [(128, 8, 2), (192, 4, 4)])
def test_ring_forward_fused_equals_unfused(gpu, layout, Dqk, Hq, Hkv):
    """The ring forward with merging launches against the same ring with chunk forward + combine launches, every
    rank of a ring of 4."""
    from pithtrain_amd.operators.ring_attention import local as L

    B, S, C = 1, 2048, 4
    g = torch.Generator().manual_seed(21)
    scale = Dqk**-0.5
    q_full = torch.randn(B, S, Hq, Dqk, generator=g).to(torch.bfloat16)
    k_full = torch.randn(B, S, Hkv, Dqk, generator=g).to(torch.bfloat16)
    v_full = torch.randn(B, S, Hkv, 128, generator=g).to(torch.bfloat16)
    split = (lambda x: R.zigzag_split(x, C)) if layout == "zigzag" else (lambda x: [c.contiguous() for c in x.chunk(C, 1)])
    qs, ks, vs = split(q_full), [c.to(gpu) for c in split(k_full)], [c.to(gpu) for c in split(v_full)]
    for r in range(C):
        res = {}
        for fused in (True, False):
            steps = L.ring_schedule(r, C, S // C, layout)
            fwd = L.RingForward(qs[r].to(gpu), 128, scale, steps, layout)
            assert fwd.fuse_merge
            fwd.fuse_merge = fused
            for st in steps:
                fwd.run_step(st, ks[st.kv_rank], vs[st.kv_rank])
            res[fused] = fwd.result()
        ro, rl = R.ring_forward(qs[r], split(k_full), split(v_full), scale, r, C, layout)
        check_bf16_result(res[True][0], ro, f"fused ring O rank {r}")
        check_lse(res[True][1], rl, f"fused ring LSE2 rank {r}")
        assert norm_max_err(res[True][0], res[False][0].float()) < 1.2e-2  # two bf16 roundings apart at most
        assert (res[True][1] - res[False][1]).abs().max().item() < 1e-4
