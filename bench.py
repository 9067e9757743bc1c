#!/usr/bin/env python3
"""Benchmark of the ring-attention hot path on ONE MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-extra-configs]
    python bench.py --config mla16k|long131k [--steps K]     (one of the other configurations alone)

A step is one forward + backward pass of one GPU's share of causal ring attention at the
Qwen3-30B-A3B shape (32 q heads / 4 kv heads, head dim 128, 32768 tokens as 4 zigzag chunks of 8192,
rank 1 of 4): 4 chunk-attention forwards, 3 log2 combines, delta, 4 dK/dV and 4 dQ launches.
Inputs are synthetic (CPU generator, seed 42; q/k/v ~ N(0,1)/sqrt(Dqk), dO ~ N(0,1)) and resident in
HBM before the timed region. One JSON line is printed; everything in it is measured in this run
except the block under "from_profiles", which quotes hardware-counter figures of earlier rocprofv3
runs by file:

  value      algorithmic TFLOP/s of the whole step: 2*(Dqk+Dv)*E*Hq forward + 2*(3Dqk+2Dv)*E*Hq backward
             with E = C*S_l^2/2 score entries per head (5 backward matmuls; recomputation not counted)
  fwd_only   the forward alone (the forward-only configuration of the same shape)
  roofline   the dominant kernel (non-causal dK/dV), timed per launch with events on the launch stream
  mla16k     the same ring driver at the MLA shape (16 heads, 192/128, 16384 tokens as 4 zigzag chunks)
  long131k   the same at the long-context shape (64 q / 4 kv heads, 131072 tokens as 8 zigzag chunks, rank 3)
  combine    the log2 combine at [1,4096,32,128] bf16+bf16 -> fp32 over rotating buffers, GB/s of
             algorithmic bytes against the 8 TB/s HBM peak: timed as replays of a captured HIP graph
             (kernel time, no host launch cost in between) and, beside it, launched eagerly
  norm_rope  the layer's prologue (per-head RMSNorm + rotary embedding of q [1,8192,32,128] and
             k [1,8192,4,128], forward and backward) over rotating buffers, GB/s of algorithmic bytes
  mla_assemble  the MLA layer's prologue (rotary embedding of the rope parts + assembly of query / key /
             value states, forward and backward) at [1,4096,16,128+64 | 128], GB/s of algorithmic bytes
  cpu_baseline  the oracle's eager-PyTorch restatement of the same ring share (all heads, once), timed
             on the host cores
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "pith-train_amd"))

MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16
HBM_PEAK_GBPS = 8000.0

HQ, HKV, DQK, DV, S_LOCAL, CP, RANK = 32, 4, 128, 128, 8192, 4, 1
LAYOUT = "zigzag"
COMBINE_TRAFFIC = 135_900_000


# Figures that are NOT measured by this program: hardware-counter results of rocprofv3 --pmc runs over
# `bench.py --counter-pass`, kept here only so that the JSON line can point at them. They describe the
# kernels as they were when the named summary was written.
FROM_PROFILES = {
    "note": "quoted from committed rocprofv3 summaries, not measured in this run",
    "attn_bwd_dkdv_d128_kernel<non-causal>": {
        "file": "profiles/attn_bwd_dkdv_d128_qwen3_step_hbm_counters.txt",
        # with the dS stores: 153.4 MB fetched + 2169.9 MB written (2147.5 MB of dS, the rest dK / dV or their head-split partials)
        "hbm_bytes_per_launch": 2_323_000_000,
        "hbm_bytes_per_launch_without_ds_stores": 175_700_000,  # 153.4 MB fetched + 22.4 MB written (mean of the three launches)
        "mfma_file": "profiles/attn_kernels_mfma_lds_counters.txt",
        "mfma_busy_fraction": 0.58,  # SQ_VALU_MFMA_BUSY_CYCLES / (GRBM_GUI_ACTIVE / 8 x 1024 SIMDs); 0.68 without the stores
        "sustained_clock_ghz": 1.75,  # GRBM_GUI_ACTIVE / 8 XCDs / launch duration (2.4 GHz nominal); 1.85 without the stores
    },
    "combine_front_kernel": {"file": "profiles/combine_norm_rope_mla_assemble_hbm_counters.txt", "hbm_bytes_per_launch": COMBINE_TRAFFIC},
    "norm_rope_kernels": {"file": "profiles/combine_norm_rope_mla_assemble_hbm_counters.txt", "hbm_bytes_fwd_plus_bwd": 159_400_000 + 235_200_000},
    "mla_assemble_kernels": {"file": "profiles/combine_norm_rope_mla_assemble_hbm_counters.txt", "hbm_bytes_fwd_plus_bwd": 128_000_000 + 128_000_000},
}


class RingConfig:
    """One GPU's share of a ring: head counts, head dims, local chunk, ring size, rank (zigzag layout)."""

    def __init__(self, name, hq, hkv, dqk, dv, s_local, cp, rank):
        self.name, self.hq, self.hkv, self.dqk, self.dv, self.s_local, self.cp, self.rank = name, hq, hkv, dqk, dv, s_local, cp, rank

    def flops(self):
        entries = self.cp * self.s_local * self.s_local // 2  # per head, this rank's zigzag share
        return 2 * (self.dqk + self.dv) * entries * self.hq, 2 * (3 * self.dqk + 2 * self.dv) * entries * self.hq

    def make_inputs(self, torch, device, host=False):
        g = torch.Generator().manual_seed(42)
        s = self.dqk**-0.5
        q = (torch.randn(1, self.s_local, self.hq, self.dqk, generator=g) * s).to(torch.bfloat16)
        ks = [(torch.randn(1, self.s_local, self.hkv, self.dqk, generator=g) * s).to(torch.bfloat16) for _ in range(self.cp)]
        vs = [(torch.randn(1, self.s_local, self.hkv, self.dv, generator=g) * s).to(torch.bfloat16) for _ in range(self.cp)]
        dout = torch.randn(1, self.s_local, self.hq, self.dv, generator=g).to(torch.bfloat16)
        dev = (q.to(device), [c.to(device) for c in ks], [c.to(device) for c in vs], dout.to(device))
        return ((q, ks, vs, dout) if host else None), dev


QWEN3 = RingConfig("qwen3-32k", HQ, HKV, DQK, DV, S_LOCAL, CP, RANK)
MLA16K = RingConfig("mla-16k", 16, 16, 192, 128, 4096, 4, 1)
LONG131K = RingConfig("long-131k", 64, 4, 128, 128, 16384, 8, 3)


def make_inputs(torch, device):
    return QWEN3.make_inputs(torch, device, host=True)


def flops_per_step():
    return QWEN3.flops()


def time_events(torch, fn, reps):
    """Average milliseconds of fn() over `reps` calls, bracketed by events on the current stream."""
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(reps):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / reps


def time_ring_share(torch, cfg, dev_inputs, steps, warmup):
    """(ms per fwd+bwd step by wall clock around synchronised steps, ms forward, ms backward by events)."""
    from pithtrain_amd.operators.ring_attention.local import ring_backward_local, ring_forward_local

    q, ks, vs, dout = dev_inputs
    scale = cfg.dqk**-0.5

    def forward():
        return ring_forward_local(q, ks, vs, scale, cfg.rank, cfg.cp, LAYOUT)

    def step():
        out, lse = forward()
        return ring_backward_local(dout, q, out, lse, ks, vs, scale, cfg.rank, cfg.cp, LAYOUT)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / steps
    ms_fwd = time_events(torch, forward, steps)
    out, lse = forward()
    ms_bwd = time_events(torch, lambda: ring_backward_local(dout, q, out, lse, ks, vs, scale, cfg.rank, cfg.cp, LAYOUT), steps)
    return ms_step, ms_fwd, ms_bwd, out, lse


def ring_summary(cfg, ms_step, ms_fwd, ms_bwd):
    fwd_flops, bwd_flops = cfg.flops()
    tf = lambda fl, ms: fl / (ms * 1e-3) / 1e12  # noqa: E731
    step_tf = tf(fwd_flops + bwd_flops, ms_step)
    return {
        "workload": f"{cfg.hq} q / {cfg.hkv} kv heads, head dims {cfg.dqk}/{cfg.dv}, S={cfg.cp * cfg.s_local} as {cfg.cp} zigzag "
                    f"chunks of {cfg.s_local} looped locally (rank {cfg.rank}), B=1, fwd+bwd incl. combines and delta",
        "ms_per_step": round(ms_step, 4), "tflops": round(step_tf, 2), "frac_mfma_peak": round(step_tf / MFMA_BF16_PEAK_TFLOPS, 4),
        "fwd": {"ms": round(ms_fwd, 4), "tflops": round(tf(fwd_flops, ms_fwd), 2)},
        "bwd": {"ms": round(ms_bwd, 4), "tflops": round(tf(bwd_flops, ms_bwd), 2)},
    }  # fmt: skip


def bench_recompute(torch, dev_inputs, steps, warmup):
    """The headline share once more with the dS hand-over between the two backward kernels switched off:
    both kernels recompute S and dP (7 matrix products executed for the 5 counted), no scratch."""
    from pithtrain_amd.operators.mla import hip

    limit = hip.DS_BUFFER_LIMIT_BYTES
    hip.DS_BUFFER_LIMIT_BYTES = 0
    try:
        ms_step, ms_fwd, ms_bwd, _, _ = time_ring_share(torch, QWEN3, dev_inputs, steps, warmup)
    finally:
        hip.DS_BUFFER_LIMIT_BYTES = limit
    fwd_flops, bwd_flops = QWEN3.flops()
    return {
        "what": "the same share with the dS hand-over off (PITHTRAIN_AMD_DS_BUFFER_LIMIT_GB=0): dQ and dK/dV kernels both "
                "recompute S and dP",
        "ms_per_step": round(ms_step, 4), "tflops": round((fwd_flops + bwd_flops) / (ms_step * 1e-3) / 1e12, 2),
        "bwd_ms": round(ms_bwd, 4),
    }  # fmt: skip


def handover_scratch_bytes(cfg, dev):
    """Largest dS hand-over scratch the ring backward takes in a ring step of `cfg` (0: it recomputes in all of them)."""
    from pithtrain_amd.operators.mla import hip
    from pithtrain_amd.operators.ring_attention.local import ring_schedule

    q, ks, vs, _ = dev
    most = 0
    for s in ring_schedule(cfg.rank, cfg.cp, cfg.s_local, LAYOUT):
        rows = slice(s.kv_rows[0], s.kv_rows[1])
        plan = hip.ds_plan(q[:, s.q_rows[0] : s.q_rows[1]], ks[s.kv_rank][:, rows], vs[s.kv_rank][:, rows], s.causal)
        most = max(most, plan[1] if plan else 0)
    return most


def bench_other_config(torch, device, cfg, steps, warmup):
    _, dev = cfg.make_inputs(torch, device)
    ms_step, ms_fwd, ms_bwd, _, _ = time_ring_share(torch, cfg, dev, steps, warmup)
    out = ring_summary(cfg, ms_step, ms_fwd, ms_bwd)
    out["ds_handover_scratch_bytes_per_ring_step"] = handover_scratch_bytes(cfg, dev)
    del dev
    torch.cuda.empty_cache()
    return out


def bench_ring(torch, args, dev_inputs):
    from pithtrain_amd.operators.mla.hip import attn_bwd_delta_into, attn_bwd_dkdv_into, ds_buffer
    from pithtrain_amd.operators.ring_attention.local import ring_schedule

    q, ks, vs, dout = dev_inputs
    scale = DQK**-0.5
    ms_step, ms_fwd, ms_bwd, out, lse = time_ring_share(torch, QWEN3, dev_inputs, args.steps, args.warmup)

    # Dominant kernel: the non-causal dK/dV launch (3 per step; every one covers S_l^2/2 score
    # entries per query head and performs 4 of the 5 algorithmic backward products).
    delta = torch.empty_like(lse)
    attn_bwd_delta_into(out, dout, delta)
    st = [s for s in ring_schedule(RANK, CP, S_LOCAL, LAYOUT) if not s.causal]
    launches = []
    for s in st:
        k_j, v_j = ks[s.kv_rank][:, s.kv_rows[0] : s.kv_rows[1]], vs[s.kv_rank][:, s.kv_rows[0] : s.kv_rows[1]]
        rows = slice(s.q_rows[0], s.q_rows[1])
        dk, dv = torch.empty_like(k_j), torch.empty_like(v_j)
        launches.append((q[:, rows], k_j, v_j, dout[:, rows], lse[:, :, rows], delta[:, :, rows], dk, dv))
    # the same kernel variant as in the step: with the dS hand-over buffer whenever the ring driver would use one
    hand = ds_buffer(*launches[0][:3])

    def dkdv_launches():
        for a in launches:
            attn_bwd_dkdv_into(*a, scale, False, ds=hand)

    dkdv_launches()
    if args.counter_pass:
        # rocprofv3 --pmc run: a few more launches of the roofline kernel and a plain elementwise
        # copy of known size (256 MiB read, 256 MiB written) to calibrate the counter against
        dkdv_launches()
        src = torch.ones(64 << 20, dtype=torch.float32, device=q.device)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.mul(src, 1.0, out=dst)
        torch.cuda.synchronize()
        return None
    ms_dkdv = time_events(torch, dkdv_launches, args.steps) / len(launches)
    entries = (S_LOCAL * S_LOCAL // 2) * HQ
    dkdv_flops = 2 * (2 * DQK + 2 * DV) * entries
    return ms_step, ms_fwd, ms_bwd, ms_dkdv, dkdv_flops, hand is not None


def bench_combine(torch, device, reps=50, graph=True):
    from pithtrain_amd.operators.ring_attention.combine import combine_into

    B, S, H, D = 1, 4096, 32, 128
    g = torch.Generator().manual_seed(42)
    sets = []
    for _ in range(5):  # 5 x 129.5 MiB > the 256 MiB last-level cache
        o1 = torch.randn(B, S, H, D, generator=g).to(torch.bfloat16).to(device)
        o2 = torch.randn(B, S, H, D, generator=g).to(torch.bfloat16).to(device)
        l1 = (torch.rand(B, H, S, generator=g) * 16 - 4).to(device)
        l2 = (torch.rand(B, H, S, generator=g) * 16 - 4).to(device)
        out = torch.empty(B, S, H, D, dtype=torch.float32, device=device)
        lse = torch.empty(B, H, S, dtype=torch.float32, device=device)
        sets.append((o1, l1, o2, l2, out, lse))
    nbytes = sum(t.numel() * t.element_size() for t in sets[0])
    it = [0]

    def one():
        combine_into(*sets[it[0] % len(sets)])
        it[0] += 1

    for _ in range(8):
        one()
    ms_eager = time_events(torch, one, reps)
    if not graph:
        return ms_eager, ms_eager, nbytes, None
    # The same rotating sequence captured once in a HIP graph: a replay enqueues the launches back to
    # back without the host-side cost of each call (the kernel lasts ~25 us, about what the Python
    # binding spends per call), so the time per launch is the kernel's. The library records no memset
    # and allocates nothing, which is what makes the capture legal.
    per_graph = 4 * len(sets)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        one()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    it[0] = 0
    with torch.cuda.graph(graph):
        for _ in range(per_graph):
            one()
    graph.replay()
    ms_graph = time_events(torch, graph.replay, max(1, reps // 4)) / per_graph
    host = [t.cpu() for t in sets[0][:4]]
    return ms_graph, ms_eager, nbytes, host


def bench_norm_rope(torch, device, reps=40):
    """Forward and backward of the q and k prologue at one rank's shape; every buffer is read or
    written once per launch, so algorithmic bytes = sum of the tensors' sizes."""
    from pithtrain_amd.operators.norm_rope import qk_norm_rope_bwd_into, qk_norm_rope_fwd_into

    g = torch.Generator().manual_seed(7)
    bf = torch.bfloat16
    cos = torch.randn(1, S_LOCAL, DQK, generator=g).to(bf).to(device)
    sin = torch.randn(1, S_LOCAL, DQK, generator=g).to(bf).to(device)
    sets = []
    for _ in range(5):  # 5 x 302 MB of q-sized tensors > the 256 MiB last-level cache
        per_tensor = []
        for h in (HQ, HKV):
            x = torch.randn(1, S_LOCAL, h, DQK, generator=g).to(bf).to(device)
            dout = torch.randn(1, S_LOCAL, h, DQK, generator=g).to(bf).to(device)
            w = (torch.rand(DQK, generator=g) + 0.5).to(bf).to(device)
            per_tensor.append((x, w, dout, torch.empty_like(x), torch.empty_like(x),
                               torch.empty(DQK, dtype=torch.float32, device=device)))  # fmt: skip
        sets.append(per_tensor)
    size = lambda *ts: sum(t.numel() * t.element_size() for t in ts)  # noqa: E731
    fwd_bytes = sum(size(x, w, out) for x, w, _, out, _, _ in sets[0]) + size(cos, sin)
    bwd_bytes = sum(size(x, w, dout, dx, dw) for x, w, dout, _, dx, dw in sets[0]) + size(cos, sin)
    it = [0]

    def forward():  # q and k in one launch
        (q, wq, _, q_out, _, _), (k, wk, _, k_out, _, _) = sets[it[0] % len(sets)]
        qk_norm_rope_fwd_into(q, k, wq, wk, cos, sin, q_out, k_out, 1e-6)
        it[0] += 1

    def backward():  # one launch plus the fixed-order sum of the dweight partials
        (q, wq, gq, _, dq, dwq), (k, wk, gk, _, dk, dwk) = sets[it[0] % len(sets)]
        qk_norm_rope_bwd_into(q, k, wq, wk, cos, sin, gq, gk, dq, dk, dwq, dwk, 1e-6)
        it[0] += 1

    for _ in range(5):
        forward()
        backward()
    ms_f = time_events(torch, forward, reps)
    ms_b = time_events(torch, backward, reps)
    host = [t.cpu() for t in sets[0][0][:3]] + [cos.cpu(), sin.cpu()]
    return ms_f, fwd_bytes, ms_b, bwd_bytes, host


def bench_mla_assemble(torch, device, reps=40):
    """Forward and backward of the MLA prologue at one rank's share of the 16K configuration."""
    from pithtrain_amd.operators.mla_assemble import mla_assemble_bwd_into, mla_assemble_fwd_into

    b, s, h, dn, dr, dv, lora = 1, 4096, 16, 128, 64, 128, 512
    g = torch.Generator().manual_seed(11)
    bf = torch.bfloat16
    table = torch.rand(16384, dr // 2, generator=g) * 6.283
    table = torch.cat((table, table), -1)
    cos, sin = table.cos().to(bf).to(device), table.sin().to(bf).to(device)
    pos = (torch.arange(s) + 4096).unsqueeze(0).to(device)
    sets = []
    for _ in range(5):  # 5 x 127 MB of tensors touched per direction, well beyond the 256 MiB last-level cache
        q = torch.randn(b, s, h, dn + dr, generator=g).to(bf).to(device)
        kv = torch.randn(b, s, h, dn + dv, generator=g).to(bf).to(device)
        a_proj = torch.randn(b, s, lora + dr, generator=g).to(bf).to(device)
        outs = [torch.empty(b, s, h, d, dtype=bf, device=device) for d in (dn + dr, dn + dr, dv)]
        grads = [torch.empty(b, s, h, dn + dr, dtype=bf, device=device), torch.empty(b, s, h, dn + dv, dtype=bf, device=device),
                 torch.empty(b, s, dr, dtype=bf, device=device)]  # fmt: skip
        sets.append((q, kv, a_proj[..., lora:], outs, grads))
    size = lambda *ts: sum(t.numel() * t.element_size() for t in ts)  # noqa: E731
    q, kv, k_pe, outs, grads = sets[0]
    touched_tables = 2 * s * dr * 2  # the cos and sin rows of this share
    fwd_bytes = size(q, kv, k_pe, pos, *outs) + touched_tables
    bwd_bytes = size(pos, *outs, *grads) + touched_tables
    it = [0]

    def forward():
        q, kv, k_pe, outs, _ = sets[it[0] % len(sets)]
        mla_assemble_fwd_into(q, kv, k_pe, cos, sin, pos, *outs)
        it[0] += 1

    def backward():  # the forward outputs stand in for their gradients (same shapes)
        _, _, _, outs, grads = sets[it[0] % len(sets)]
        mla_assemble_bwd_into(*outs, cos, sin, pos, *grads)
        it[0] += 1

    for _ in range(5):
        forward()
        backward()
    ms_f = time_events(torch, forward, reps)
    ms_b = time_events(torch, backward, reps)
    return ms_f, fwd_bytes, ms_b, bwd_bytes


def cpu_baseline_norm_rope(torch, host, reps=3):
    """The oracle's fp32 forward + backward of the q tensor on the host cores; GB/s of the same
    algorithmic byte count."""
    from oracle import prologue_oracle as P

    x, w, dout, cos, sin = host
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        P.norm_rope_fwd(x, w, cos, sin, 1e-6, dtype=torch.float32)
        P.norm_rope_bwd(x, w, cos, sin, dout, 1e-6, dtype=torch.float32)
        times.append(time.perf_counter() - t0)
    times.sort()
    nbytes = 5 * x.numel() * 2 + 4 * cos.numel() * 2  # x, out | x, dout, dx; cos and sin twice
    return nbytes / times[len(times) // 2] / 1e9


def cpu_baseline_ring(torch, host_inputs):
    """The whole configuration once on the host cores: every head, every row."""
    from oracle import ring_oracle as R

    q, ks, vs, dout = host_inputs
    t0 = time.perf_counter()
    R.cpu_ring_fwd_bwd(q, ks, vs, dout, DQK**-0.5, RANK, CP, LAYOUT, heads=(0, HQ), q_block=1024)
    dt = time.perf_counter() - t0
    fwd, bwd = flops_per_step()
    return (fwd + bwd) / dt / 1e12, dt


def cpu_baseline_combine(torch, host, nbytes, reps=5):
    from oracle import ring_oracle as R

    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        R.combine_log2(*host)
        times.append(time.perf_counter() - t0)
    times.sort()
    return nbytes / times[len(times) // 2] / 1e9


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra-configs", action="store_true",
                    help="skip the MLA 16K and long 131K configurations (sub-objects mla16k, long131k)")
    ap.add_argument("--config", choices=["mla16k", "long131k"], default=None,
                    help="time only this configuration's ring share and print its sub-object (for kernel traces)")
    ap.add_argument("--no-handover", action="store_true",
                    help="run everything with the dS hand-over between the backward kernels switched off (for traces)")
    ap.add_argument("--counter-pass", action="store_true",
                    help="run only the roofline kernel and a calibration copy (for rocprofv3 --pmc), print no JSON")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit(
            "bench.py measures one GPU's share of the ring (no collectives are part of this build); "
            f"--gpus {args.gpus} is not supported, run with --gpus 1"
        )
    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py needs an MI355X: no GPU is visible")
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)

    if args.no_handover:
        from pithtrain_amd.operators.mla import hip

        hip.DS_BUFFER_LIMIT_BYTES = 0
    if args.config:
        cfg = MLA16K if args.config == "mla16k" else LONG131K
        print(json.dumps({args.config: bench_other_config(torch, device, cfg, args.steps, args.warmup)}))
        return
    host_inputs, dev_inputs = make_inputs(torch, device)
    ring = bench_ring(torch, args, dev_inputs)
    if ring is None:
        # the HBM-bound kernels, a few dispatches each, for the same counters
        del dev_inputs
        bench_other_config(torch, device, MLA16K, 1, 0)  # the 192/128 kernels, for the same counters
        bench_combine(torch, device, reps=4, graph=False)
        bench_norm_rope(torch, device, reps=3)
        bench_mla_assemble(torch, device, reps=3)
        print("counter pass done")
        return
    ms_step, ms_fwd, ms_bwd, ms_dkdv, dkdv_flops, handover_on = ring
    recompute = None
    if not args.no_extra_configs and handover_on:
        recompute = bench_recompute(torch, dev_inputs, args.steps, args.warmup)
    scratch = handover_scratch_bytes(QWEN3, dev_inputs) if handover_on else 0
    del dev_inputs
    torch.cuda.empty_cache()
    fwd_flops, bwd_flops = flops_per_step()
    tflops = (fwd_flops + bwd_flops) / (ms_step * 1e-3) / 1e12
    mla16k = long131k = None
    if not args.no_extra_configs:
        mla16k = bench_other_config(torch, device, MLA16K, args.steps, args.warmup)
        long131k = bench_other_config(torch, device, LONG131K, max(2, args.steps // 5), 1)
    ms_comb, ms_comb_eager, comb_bytes, comb_host = bench_combine(torch, device)
    comb_gbps = comb_bytes / (ms_comb * 1e-3) / 1e9
    nr_ms_f, nr_bytes_f, nr_ms_b, nr_bytes_b, nr_host = bench_norm_rope(torch, device)
    nr_gbps = (nr_bytes_f + nr_bytes_b) / ((nr_ms_f + nr_ms_b) * 1e-3) / 1e9
    ma_ms_f, ma_bytes_f, ma_ms_b, ma_bytes_b = bench_mla_assemble(torch, device)
    ma_gbps = (ma_bytes_f + ma_bytes_b) / ((ma_ms_f + ma_ms_b) * 1e-3) / 1e9

    cores = torch.get_num_threads()
    cpu = None
    combine_cpu = None
    norm_rope_cpu = None
    if not args.no_cpu_baseline:
        cpu_tflops, cpu_s = cpu_baseline_ring(torch, host_inputs)
        cpu = {
            "value": round(cpu_tflops, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"the whole workload once (all {HQ} query heads, all rows, forward + backward), fp32 eager PyTorch "
                      f"on bf16-rounded inputs, {cpu_s:.1f} s; os.cpu_count()={os.cpu_count()}",
        }  # fmt: skip
        combine_cpu = {
            "value": round(cpu_baseline_combine(torch, comb_host, comb_bytes), 2), "unit": "GB/s", "cores": cores,
            "kind": "port", "sample": "full [1,4096,32,128] combine, eager PyTorch, median of 5",
        }  # fmt: skip
        norm_rope_cpu = {
            "value": round(cpu_baseline_norm_rope(torch, nr_host), 2), "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": "q tensor [1,8192,32,128] only, forward + backward, fp32 eager PyTorch, median of 3",
        }  # fmt: skip

    dkdv_tflops = dkdv_flops / (ms_dkdv * 1e-3) / 1e12
    dkdv_prof = FROM_PROFILES["attn_bwd_dkdv_d128_kernel<non-causal>"]
    line = {
        "metric": "ring-attn fwd+bwd causal TFLOP/s (Qwen3-30B-A3B, 32K)",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "GQA ring share fwd+bwd: 32 q / 4 kv heads, head dim 128, S=32768 as 4 zigzag chunks of "
                        "8192 looped locally (rank 1), B=1, incl. log2 combines and delta",
            "layout": LAYOUT, "cp_size": CP, "cp_rank": RANK, "s_local": S_LOCAL,
        },  # fmt: skip
        "frac_mfma_peak": round(tflops / MFMA_BF16_PEAK_TFLOPS, 4),
        "fwd": {"ms": round(ms_fwd, 4), "tflops": round(fwd_flops / (ms_fwd * 1e-3) / 1e12, 2)},
        "bwd": {"ms": round(ms_bwd, 4), "tflops": round(bwd_flops / (ms_bwd * 1e-3) / 1e12, 2)},
        "fwd_only": {
            "workload": "the same share, forward only (4 chunk-attention launches + 3 combines): O and the base-2 LSE",
            "ms": round(ms_fwd, 4), "tflops": round(fwd_flops / (ms_fwd * 1e-3) / 1e12, 2),
            "frac_mfma_peak": round(fwd_flops / (ms_fwd * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
        },
        "roofline": {
            "kernel": "attn_bwd_dkdv_d128_kernel<non-causal> (S, dP, dV, dK of one ring step"
                      + ("; also stores its dS tiles for the dQ kernel)" if handover_on else ")"),
            "bound": "mfma", "achieved": round(dkdv_tflops, 2), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round(dkdv_tflops / MFMA_BF16_PEAK_TFLOPS, 4),
            "traffic": dkdv_prof["hbm_bytes_per_launch" if handover_on else "hbm_bytes_per_launch_without_ds_stores"],
            "traffic_from": dkdv_prof["file"],
            "ms_per_launch": round(ms_dkdv, 4),
        },  # fmt: skip
        "ds_handover": {
            "on": handover_on,
            "what": "the dK/dV kernel hands its dS tiles to the dQ kernel (5 matrix products executed instead of 7)",
            "scratch_bytes_per_ring_step": scratch,
            "recompute_backward": recompute,
        },
        "mla16k": mla16k,
        "long131k": long131k,
        "combine": {
            "metric": "online_softmax_combine_log2 GB/s ([1,4096,32,128] bf16 x2 -> fp32)",
            "value": round(comb_gbps, 1), "unit": "GB/s", "us_per_launch": round(ms_comb * 1e3, 2),
            "timing": "replays of a captured HIP graph of 20 launches over 5 rotating buffer sets",
            "us_per_launch_eager": round(ms_comb_eager * 1e3, 2),
            "gbps_eager": round(comb_bytes / (ms_comb_eager * 1e-3) / 1e9, 1),
            "bytes": comb_bytes,
            "roofline": {"bound": "hbm", "achieved": round(comb_gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                         "frac": round(comb_gbps / HBM_PEAK_GBPS, 4),
                         "traffic": FROM_PROFILES["combine_front_kernel"]["hbm_bytes_per_launch"],
                         "traffic_from": FROM_PROFILES["combine_front_kernel"]["file"]},
            "cpu_baseline": combine_cpu,
        },  # fmt: skip
        "norm_rope": {
            "metric": "q/k RMSNorm + rotary embedding fwd+bwd GB/s (q [1,8192,32,128] + k [1,8192,4,128] bf16)",
            "value": round(nr_gbps, 1), "unit": "GB/s",
            "fwd": {"us": round(nr_ms_f * 1e3, 2), "bytes": nr_bytes_f,
                    "gbps": round(nr_bytes_f / (nr_ms_f * 1e-3) / 1e9, 1)},
            "bwd": {"us": round(nr_ms_b * 1e3, 2), "bytes": nr_bytes_b,
                    "gbps": round(nr_bytes_b / (nr_ms_b * 1e-3) / 1e9, 1)},
            "roofline": {"bound": "hbm", "achieved": round(nr_gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                         "frac": round(nr_gbps / HBM_PEAK_GBPS, 4)},
            "cpu_baseline": norm_rope_cpu,
        },  # fmt: skip
        "mla_assemble": {
            "metric": "MLA rotary + q/k/v assembly fwd+bwd GB/s ([1,4096,16,192] q, [1,4096,16,256] kv, bf16)",
            "value": round(ma_gbps, 1), "unit": "GB/s",
            "fwd": {"us": round(ma_ms_f * 1e3, 2), "bytes": ma_bytes_f,
                    "gbps": round(ma_bytes_f / (ma_ms_f * 1e-3) / 1e9, 1)},
            "bwd": {"us": round(ma_ms_b * 1e3, 2), "bytes": ma_bytes_b,
                    "gbps": round(ma_bytes_b / (ma_ms_b * 1e-3) / 1e9, 1)},
            "roofline": {"bound": "hbm", "achieved": round(ma_gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                         "frac": round(ma_gbps / HBM_PEAK_GBPS, 4)},
        },  # fmt: skip
        "from_profiles": FROM_PROFILES,
        "cpu_baseline": cpu,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
