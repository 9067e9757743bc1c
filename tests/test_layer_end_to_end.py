"""Sharding helpers on the CPU, and on the GPU the whole attention core of a GQA layer under
context parallelism: shard the projected q/k/v of a full sequence the way a rank's data loader
would, run the prologue (RMSNorm + rotary with the rank's positions) and the ring share of every
rank on one device, and compare the merged result with the same layer on the unsharded sequence
(which is checked against the fp64 oracle)."""

import pytest
import torch

from pithtrain_amd.operators.ring_attention.local import (
    cp_local_slice,
    cp_position_ids,
    zigzag_merge,
    zigzag_split,
)


@pytest.mark.parametrize("cp_size", [1, 2, 4])
def test_contiguous_slices_match_the_reference_slicing(cp_size):
    x = torch.arange(2 * 24 * 3).view(2, 24, 3)
    chunk = 24 // cp_size
    for r in range(cp_size):
        want = x[:, r * chunk : (r + 1) * chunk]  # pretrain_language_model.py:131-133
        assert torch.equal(cp_local_slice(x, r, cp_size, "contiguous"), want)
        assert torch.equal(cp_position_ids(r, cp_size, chunk, "contiguous"), torch.arange(r * chunk, (r + 1) * chunk).unsqueeze(0))


@pytest.mark.parametrize("cp_size", [1, 2, 3, 4])
def test_zigzag_slices_partition_the_sequence_and_agree_with_zigzag_split(cp_size):
    n = 12 * cp_size
    x = torch.randn(2, n, 5)
    parts = [cp_local_slice(x, r, cp_size, "zigzag") for r in range(cp_size)]
    for a, b in zip(parts, zigzag_split(x, cp_size)):
        assert torch.equal(a, b)
    assert torch.equal(zigzag_merge(parts), x)
    pos = torch.cat([cp_position_ids(r, cp_size, n // cp_size, "zigzag") for r in range(cp_size)], dim=1)
    assert sorted(pos.flatten().tolist()) == list(range(n))  # every position exactly once
    for r in range(cp_size):
        ids = cp_position_ids(r, cp_size, n // cp_size, "zigzag")[0]
        assert torch.equal(x[:, ids], parts[r])  # a rank's positions index its own tokens
        # balanced causal work: sum over a rank's tokens of (position + 1) is the same for every rank
        assert (ids + 1).sum().item() == (n * (n + 1) // 2) // cp_size
    # sequence dimension other than 1
    y = torch.randn(n, 3)
    assert torch.equal(cp_local_slice(y, 0, cp_size, "zigzag", dim=0), cp_local_slice(y.unsqueeze(0), 0, cp_size, "zigzag")[0])


def test_slicing_rejects_indivisible_lengths():
    with pytest.raises(AssertionError):
        cp_local_slice(torch.zeros(1, 10), 0, 4, "contiguous")
    with pytest.raises(AssertionError):
        cp_local_slice(torch.zeros(1, 12), 0, 4, "zigzag")
    with pytest.raises(AssertionError):
        cp_local_slice(torch.zeros(1, 16), 0, 4, "diagonal")


@pytest.mark.gpu
@pytest.mark.parametrize("layout", ["contiguous", "zigzag"])
def test_sharded_layer_core_equals_the_unsharded_layer(gpu, layout):
    from helpers import check_bf16_result
    from oracle import prologue_oracle as P
    from oracle import ring_oracle as R
    from pithtrain_amd.operators.mla.hip import attention_func
    from pithtrain_amd.operators.norm_rope import qk_norm_rope
    from pithtrain_amd.operators.ring_attention.local import ring_attention_local

    B, S, Hq, Hkv, D, C = 1, 1024, 8, 2, 128, 4
    g = torch.Generator().manual_seed(17)
    bf = torch.bfloat16
    q_raw = torch.randn(B, S, Hq, D, generator=g).to(bf)
    k_raw = torch.randn(B, S, Hkv, D, generator=g).to(bf)
    v = (torch.randn(B, S, Hkv, D, generator=g) * D**-0.5).to(bf)
    wq, wk = (torch.rand(D, generator=g) + 0.5).to(bf), (torch.rand(D, generator=g) + 0.5).to(bf)
    dout = torch.randn(B, S, Hq, D, generator=g).to(bf)
    cos_t, sin_t = P.cos_sin_table(torch.arange(S), D, dtype=bf)  # [S, D] tables
    scale = D**-0.5

    # ---- unsharded layer on the GPU
    leaves = [t.to(gpu).requires_grad_() for t in (q_raw, k_raw, v, wq, wk)]
    qf, kf, vf, wqf, wkf = leaves
    qn, kn = qk_norm_rope(qf, kf, wqf, wkf, cos_t.unsqueeze(0).to(gpu), sin_t.unsqueeze(0).to(gpu), 1e-6)
    out_full = attention_func(qn, kn, vf, scale, causal=True)
    out_full.backward(dout.to(gpu))

    # the unsharded layer against the fp64 oracle (prologue rounded to bf16 as the kernels do)
    q_ref = P.norm_rope_fwd(q_raw, wq, cos_t.unsqueeze(0), sin_t.unsqueeze(0), 1e-6).to(bf)
    k_ref = P.norm_rope_fwd(k_raw, wk, cos_t.unsqueeze(0), sin_t.unsqueeze(0), 1e-6).to(bf)
    o_ref, _ = R.chunk_fwd(q_ref, k_ref, v, scale, True)
    check_bf16_result(out_full, o_ref, "unsharded O")

    # ---- the same layer, every rank's share computed from its own slices
    sh_leaves = [t.to(gpu).requires_grad_() for t in (q_raw, k_raw, v, wq, wk)]
    qs, ks, vs, wqs, wks = sh_leaves
    q_loc, k_loc, v_loc = [], [], []
    for r in range(C):
        pos = cp_position_ids(r, C, S // C, layout, device=gpu)  # [1, S_l]
        cos, sin = cos_t.to(gpu)[pos], sin_t.to(gpu)[pos]         # what the rotary module returns for these positions
        qr, kr = qk_norm_rope(cp_local_slice(qs, r, C, layout).contiguous(), cp_local_slice(ks, r, C, layout).contiguous(),
                              wqs, wks, cos, sin, 1e-6)  # fmt: skip
        q_loc.append(qr)
        k_loc.append(kr)
        v_loc.append(cp_local_slice(vs, r, C, layout).contiguous())
    outs = [ring_attention_local(q_loc[r], k_loc, v_loc, scale, r, C, layout) for r in range(C)]
    merged = zigzag_merge(outs) if layout == "zigzag" else torch.cat(outs, dim=1)
    dout_loc = [cp_local_slice(dout.to(gpu), r, C, layout).contiguous() for r in range(C)]
    torch.autograd.backward(outs, dout_loc)

    check_bf16_result(merged, o_ref, "sharded O")
    check_bf16_result(merged, out_full.double().cpu(), "sharded vs unsharded O", nerr_tol=1e-2)
    names = ("dq_raw", "dk_raw", "dv", "dwq", "dwk")
    for name, a, b in zip(names, sh_leaves, leaves):
        # the weights are bf16 parameters: autograd adds the four ranks' bf16-rounded contributions
        # in bf16, so their gradients carry a few more roundings than the unsharded one
        cos_tol = 1e-4 if name.startswith("dw") else 1e-5
        check_bf16_result(a.grad, b.grad.double().cpu(), f"sharded vs unsharded {name}", otol=2e-3, nerr_tol=2e-2,
                          cos_tol=cos_tol)
