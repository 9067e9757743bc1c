"""The multi-rank driver's communication logic on the CPU: ranks are gloo processes, and the HIP
entry points the driver calls are replaced, inside this test only, by CPU stand-ins built from the
oracle. What is tested is the part no one-GPU run reaches: which chunk is where at each ring step
(K/V rotation), which gradients travel back to which rank (distance loop, with and without
wrap-around; or the accumulator that travels with its chunk in the re-rotating backward), and
the reference-named entry points on a real process group. Every rank's O, dQ
and its own chunk's dK/dV must equal full-sequence causal attention restricted to its tokens."""

import socket

import pytest
import torch
import torch.distributed as dist
import torch.multiprocessing as mp

from oracle import ring_oracle as R


def _install_cpu_stand_ins():
    from pithtrain_amd.operators.ring_attention import local as L

    def full_key(k, k_pe):  # keys in two parts: [k_nope | k_pe for every head]
        return k if k_pe is None else torch.cat([k, k_pe.unsqueeze(2).expand(-1, -1, k.shape[2], -1)], -1)

    def attn_fwd_into(q, k, v, o, lse, scale, causal, k_pe=None, prev_o=None, acc_o=None):
        ro, rl = R.chunk_fwd(q, full_key(k, k_pe), v, scale, causal)
        if prev_o is not None:  # the merging form: one ring step
            ro, rl = R.combine_log2(prev_o.double(), lse.double(), ro, rl)
        if o is not None:
            o.copy_(ro)
        if acc_o is not None:
            acc_o.copy_(ro)
        lse.copy_(rl)

    def attn_bwd_delta_into(out, dout, delta):
        delta.copy_(R.bwd_delta(out, dout))

    def attn_bwd_dkdv_into(q, k, v, dout, lse, delta, dk, dv, scale, causal, accumulate=False, k_pe=None, dk_pe=None, ds=None):
        _, rdk, rdv = R.chunk_bwd(q, full_key(k, k_pe), v, dout, lse.double(), delta.double(), scale, causal)
        if k_pe is not None:
            rpe, rdk = rdk[..., k.shape[-1] :].sum(2), rdk[..., : k.shape[-1]]
            dk_pe.copy_(dk_pe.double() + rpe if accumulate else rpe)
        dk.copy_(dk.double() + rdk if accumulate else rdk)
        dv.copy_(dv.double() + rdv if accumulate else rdv)

    def attn_bwd_dq_into(q, k, v, dout, lse, delta, dq, scale, causal, accumulate=False, k_pe=None, ds=None):
        rdq, _, _ = R.chunk_bwd(q, full_key(k, k_pe), v, dout, lse.double(), delta.double(), scale, causal)
        dq.copy_(dq.double() + rdq if accumulate else rdq)

    def attn_bwd_pair_into(q, k, v, dout, lse, delta, dq, dk, dv, scale, causal, accumulate_dq=False,
                           accumulate_dkv=False, k_pe=None, dk_pe=None, handover=True, zero_tail=0, dq_final=None,
                           dq_final_rows=None):  # fmt: skip
        assert zero_tail == 0 and dq_final is None, "the stand-ins do not implement the fused conveniences"
        attn_bwd_dkdv_into(q, k, v, dout, lse, delta, dk, dv, scale, causal, accumulate_dkv, k_pe, dk_pe)
        attn_bwd_dq_into(q, k, v, dout, lse, delta, dq, scale, causal, accumulate_dq, k_pe)
        return 0  # no dS hand-over between the stand-ins

    L.FUSE_FINAL_DQ = L.FUSE_ZERO_TAIL = False  # per-process (the ranks are spawned): fill and cast stay separate calls

    def combine_into(out1, lse1, out2, lse2, out, lse_out, base=0):
        o, l = R.combine_log2(out1.double(), lse1.double(), out2.double(), lse2.double())
        out.copy_(o)
        lse_out.copy_(l)

    def cast_f32_bf16_into(src, dst):
        dst.copy_(src)

    for name, fn in list(locals().items()):
        if callable(fn) and hasattr(L, name):
            setattr(L, name, fn)


def _worker(rank, world, port, layout, variant, rerotate, results):
    dist.init_process_group("gloo", init_method=f"tcp://127.0.0.1:{port}", rank=rank, world_size=world)
    try:
        _install_cpu_stand_ins()
        from pithtrain_amd.operators.ring_attention.local import cp_local_slice
        from pithtrain_amd.operators.ring_attention.mla import ring_mla_attention_func
        from pithtrain_amd.operators.ring_attention.standard import ring_attention_func

        B, s_l, Hq, Hkv = 1, 16, 4, 2
        dqk, dv = (24, 16) if variant.startswith("mla") else (16, 16)
        if variant.startswith("mla"):
            Hkv = Hq
        S = s_l * world
        g = torch.Generator().manual_seed(1234)  # every rank draws the same full sequence
        bf = torch.bfloat16
        q = torch.randn(B, S, Hq, dqk, generator=g).to(bf)
        k = torch.randn(B, S, Hkv, dqk, generator=g).to(bf)
        v = torch.randn(B, S, Hkv, dv, generator=g).to(bf)
        dout = torch.randn(B, S, Hq, dv, generator=g).to(bf)
        scale = dqk**-0.5

        mine = lambda t: cp_local_slice(t, rank, world, layout).contiguous()  # noqa: E731
        group = dist.group.WORLD
        if variant == "mla-two-part":
            # keys in two parts: the last 8 features are one vector per position shared by all heads
            k_pe = k[:, :, 0, dqk - 8 :].contiguous()
            k = torch.cat([k[..., : dqk - 8], k_pe.unsqueeze(2).expand(-1, -1, Hkv, -1)], -1).contiguous()
            ql, kl, vl, pl = (mine(t).requires_grad_() for t in (q, k[..., : dqk - 8], v, k_pe))
            out = ring_mla_attention_func(ql, kl, vl, scale, group, layout=layout, rerotate=rerotate, k_pe=pl)
        else:
            ql, kl, vl = (mine(t).requires_grad_() for t in (q, k, v))
            fn = ring_mla_attention_func if variant == "mla" else ring_attention_func
            out = fn(ql, kl, vl, scale, group, layout=layout, rerotate=rerotate)
        out.backward(mine(dout))

        ro, rl = R.chunk_fwd(q, k, v, scale, True)
        rdq, rdk, rdv = R.chunk_bwd(q, k, v, dout, rl, R.bwd_delta(ro, dout), scale, True)
        errs = {}
        checks = [("O", out, ro), ("dQ", ql.grad, rdq), ("dK", kl.grad, rdk), ("dV", vl.grad, rdv)]
        if variant == "mla-two-part":
            checks[2] = ("dK nope", kl.grad, rdk[..., : dqk - 8])
            checks.append(("dK pe", pl.grad, rdk[..., dqk - 8 :].sum(2)))
        for name, got, want in checks:
            w = mine(want)
            errs[name] = ((got.double() - w).abs().max() / w.abs().max()).item()
        results[rank] = errs
    finally:
        dist.destroy_process_group()


def _free_port():
    with socket.socket() as s:
        s.bind(("127.0.0.1", 0))
        return s.getsockname()[1]


@pytest.mark.timeout(300)
@pytest.mark.parametrize(
    "world,layout,variant,rerotate",
    [
        (2, "contiguous", "gqa", False), (2, "zigzag", "gqa", False), (3, "zigzag", "mla", False),
        (4, "contiguous", "mla", False), (4, "zigzag", "gqa", False),
        # backward that keeps one K/V chunk per rank and sends the chunks around again
        (2, "zigzag", "gqa", True), (3, "contiguous", "gqa", True), (4, "zigzag", "mla", True),
        # keys in two parts: k_nope and the shared k_pe both rotate, both receive gradients
        (3, "zigzag", "mla-two-part", False), (2, "contiguous", "mla-two-part", True),
    ],
)  # fmt: skip
def test_ring_over_gloo_matches_full_sequence_attention(world, layout, variant, rerotate):
    torch.set_num_threads(1)
    with mp.Manager() as manager:
        results = manager.dict()
        mp.spawn(_worker, args=(world, _free_port(), layout, variant, rerotate, results), nprocs=world, join=True)
        assert sorted(results.keys()) == list(range(world))
        for rank in range(world):
            for name, err in results[rank].items():
                # stand-ins compute in fp64; what remains is the bf16 rounding of O, of the saved
                # tensors and of the gradients that travel between ranks
                assert err < 2e-2, f"rank {rank} {name}: normalised max-abs error {err:.3e}"
