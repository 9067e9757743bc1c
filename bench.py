#!/usr/bin/env python3
"""Benchmark of the ring-attention hot path on ONE MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-extra-configs]
    python bench.py --config mla16k|long131k|mla_op [--steps K]     (one of the other configurations alone)

A step is one forward + backward pass of one GPU's share of causal ring attention at the
Qwen3-30B-A3B shape (32 q heads / 4 kv heads, head dim 128, 32768 tokens as 4 zigzag chunks of 8192,
rank 1 of 4): 4 chunk-attention forwards, 3 log2 combines, delta, 4 dK/dV and 4 dQ launches.
Inputs are synthetic (CPU generator, seed 42; q/k/v ~ N(0,1)/sqrt(Dqk), dO ~ N(0,1)) and resident in
HBM before the timed region. One JSON line is printed; everything in it is measured in this run except
`roofline.traffic` (HBM bytes per launch need a rocprofv3 --pmc run: the figure is read from the committed summary
named beside it in `traffic_from`, null when that summary has none):

  value      algorithmic TFLOP/s of the whole step: 2*(Dqk+Dv)*E*Hq forward + 2*(3Dqk+2Dv)*E*Hq backward
             with E = C*S_l^2/2 score entries per head (5 backward matmuls; recomputation not counted)
  roofline   the dominant kernel (non-causal dK/dV), timed per launch with events on the launch stream
  fwd_only   the forward alone (the forward-only configuration of the same shape), with its dominant kernel
             (the non-causal forward launch) and its own CPU baseline
  mla16k     the same ring driver at the MLA shape (16 heads, 192/128, 16384 tokens as 4 zigzag chunks), with the
             roofline of its dominant kernel and the CPU port on the whole workload
  long131k   the same at the long-context shape (64 q / 4 kv heads, 131072 tokens as 8 zigzag chunks, rank 3);
             CPU port on 4 of the 64 query heads
  mla_op     the reference's own MLA operator benchmark matrix (h in {16,128} x s in {4096,32768}, causal,
             forward and backward) with its FLOP and byte models
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


def profile_figure(name, key):
    """A figure quoted from a committed rocprofv3 summary: the value of the line `bench.py <key> = <number>` in
    profiles/<name>, or None when the file or the line is missing. HBM traffic cannot be measured by this
    program (it needs a rocprofv3 --pmc run), so `roofline.traffic` is read from the summary of that run."""
    try:
        with open(os.path.join(ROOT, "profiles", name)) as f:
            for line in f:
                parts = line.split()
                if len(parts) >= 4 and parts[0] == "bench.py" and parts[1] == key and parts[2] == "=":
                    return int(float(parts[3]))
    except OSError:
        pass
    return None


HBM_COUNTERS = "attn_bwd_dkdv_d128_qwen3_step_hbm_counters.txt"
STREAM_COUNTERS = "combine_norm_rope_mla_assemble_hbm_counters.txt"


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


def roofline_entry(kernel, flops_per_launch, ms_per_launch, launches, traffic=None, traffic_from=None, note=None):
    tf = flops_per_launch / (ms_per_launch * 1e-3) / 1e12
    out = {
        "kernel": kernel, "bound": "mfma", "achieved": round(tf, 2), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
        "frac": round(tf / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": traffic, "traffic_from": traffic_from,
        "ms_per_launch": round(ms_per_launch, 4), "flop_per_launch": flops_per_launch, "launches_per_step": launches,
    }  # fmt: skip
    if note:
        out["note"] = note
    return out


def noncausal_steps(cfg):
    from pithtrain_amd.operators.ring_attention.local import ring_schedule

    return [s for s in ring_schedule(cfg.rank, cfg.cp, cfg.s_local, LAYOUT) if not s.causal]


def dominant_dkdv(torch, cfg, dev, out, lse, reps, counter_pass=False):
    """The non-causal dK/dV launches of one step of `cfg`, launched exactly as the ring backward launches them
    (with the dS hand-over buffer, whole or one slab of kv heads at a time, whenever its policy takes one) and
    timed with events on the launch stream. Returns (ms per launch, FLOP per launch, launches per step, bytes of
    hand-over scratch)."""
    from pithtrain_amd.operators.mla import hip

    q, ks, vs, dout = dev
    scale = cfg.dqk**-0.5
    delta = torch.empty_like(lse)
    hip.attn_bwd_delta_into(out, dout, delta)
    launches, buf, flops = [], None, 0
    for s in noncausal_steps(cfg):
        kr, qr = slice(*s.kv_rows), slice(*s.q_rows)
        k_j, v_j = ks[s.kv_rank][:, kr], vs[s.kv_rank][:, kr]
        dk, dv = torch.empty_like(k_j), torch.empty_like(v_j)
        plan = hip.ds_plan(q[:, qr], k_j, v_j, False)
        if plan is not None and buf is None:
            buf = hip._try_alloc(plan[1], q.device)
        heads = plan[0] if plan is not None and buf is not None else cfg.hkv
        g = cfg.hq // cfg.hkv
        for h0 in range(0, cfg.hkv, heads):
            kv_h, q_h = slice(h0, h0 + heads), slice(h0 * g, (h0 + heads) * g)
            launches.append((q[:, qr, q_h], k_j[:, :, kv_h], v_j[:, :, kv_h], dout[:, qr, q_h], lse[:, q_h, qr],
                             delta[:, q_h, qr], dk[:, :, kv_h], dv[:, :, kv_h]))  # fmt: skip
        flops = 2 * (2 * cfg.dqk + 2 * cfg.dv) * (qr.stop - qr.start) * (kr.stop - kr.start) * heads * g

    def run():
        for a in launches:
            hip.attn_bwd_dkdv_into(*a, scale, False, ds=buf)

    run()
    if counter_pass:
        run()
        torch.cuda.synchronize()
        return None
    ms = time_events(torch, run, reps) / len(launches)
    return ms, flops, len(launches), (0 if buf is None else buf.numel())


def dominant_fwd(torch, cfg, dev, reps):
    """The non-causal chunk-attention forward launches of one step of `cfg`, timed like dominant_dkdv."""
    from pithtrain_amd.operators.mla import hip

    q, ks, vs, _ = dev
    scale = cfg.dqk**-0.5
    launches, flops = [], 0
    for s in noncausal_steps(cfg):
        kr, qr = slice(*s.kv_rows), slice(*s.q_rows)
        n_q = qr.stop - qr.start
        o = torch.empty((1, n_q, cfg.hq, cfg.dv), dtype=torch.bfloat16, device=q.device)
        l = torch.empty((1, cfg.hq, n_q), dtype=torch.float32, device=q.device)
        launches.append((q[:, qr], ks[s.kv_rank][:, kr], vs[s.kv_rank][:, kr], o, l))
        flops = 2 * (cfg.dqk + cfg.dv) * n_q * (kr.stop - kr.start) * cfg.hq

    def run():
        for a in launches:
            hip.attn_fwd_into(*a, scale, False)

    run()
    return time_events(torch, run, reps) / len(launches), flops, len(launches)


def bench_other_config(torch, device, cfg, steps, warmup, cpu_heads=None, counter_pass=False):
    """Step time of another configuration through the same ring driver, its dominant kernel (the non-causal dK/dV
    launch) against the MFMA roofline, and (cpu_heads = (first, last+1) query heads, or "all") the oracle's CPU port
    on that sample of the same workload."""
    host, dev = cfg.make_inputs(torch, device, host=cpu_heads is not None)
    ms_step, ms_fwd, ms_bwd, o, lse = time_ring_share(torch, cfg, dev, steps, warmup)
    if counter_pass:
        dominant_dkdv(torch, cfg, dev, o, lse, 1, counter_pass=True)
        return None
    out = ring_summary(cfg, ms_step, ms_fwd, ms_bwd)
    ms, flops, n, scratch = dominant_dkdv(torch, cfg, dev, o, lse, steps)
    kname = "attn_bwd_dkdv_d192_kernel" if cfg.dqk == 192 else "attn_bwd_dkdv_d128_kernel"
    slabs = n // len(noncausal_steps(cfg))
    out["roofline"] = roofline_entry(
        f"{kname}<non-causal> (S, dP, dV, dK of one ring step" + (f", one of {slabs} kv-head slabs per launch" if slabs > 1 else "")
        + ("; also stores its dS tiles for the dQ kernel)" if scratch else ")"),
        flops, ms, n, profile_figure(HBM_COUNTERS, f"{cfg.name}.dkdv_traffic_bytes_per_launch"), "profiles/" + HBM_COUNTERS)  # fmt: skip
    out["ds_handover_scratch_bytes_per_ring_step"] = handover_scratch_bytes(cfg, dev)
    del dev, o, lse
    torch.cuda.empty_cache()
    if cpu_heads is not None:
        out["cpu_baseline"] = cpu_baseline_ring(torch, cfg, host, None if cpu_heads == "all" else cpu_heads)
    return out


def bench_mla_op(torch, device, reps=5):
    """The reference's own operator benchmark matrix (benchmarks/operators/mla/test_triton.py:41-48): the causal
    MLA operator, b=1, h in {16, 128}, s in {4096, 32768}, head dims 192/128, forward and backward, with its FLOP
    and byte models (:7-28, :77-78, :116-118): forward b*h*s^2*(dq+dv), backward 2.5x that."""
    from pithtrain_amd.operators.mla.hip import MLA

    dq, dv = 192, 128
    rows = []
    for h in (16, 128):
        for s in (4096, 32768):
            torch.manual_seed(42)
            q = torch.randn((1, s, h, dq), dtype=torch.bfloat16, device=device, requires_grad=True)
            k = torch.randn((1, s, h, dq), dtype=torch.bfloat16, device=device, requires_grad=True)
            v = torch.randn((1, s, h, dv), dtype=torch.bfloat16, device=device, requires_grad=True)
            do = torch.randn((1, s, h, dv), dtype=torch.bfloat16, device=device)
            op = MLA(h, dq, dv, dq**-0.5)

            def fwd():
                with torch.no_grad():
                    return op.forward(q, k, v)

            o = op.forward(q, k, v)

            def bwd():
                q.grad = k.grad = v.grad = None
                o.backward(do, retain_graph=True)

            fwd(), bwd()
            n = reps if s > 4096 else 4 * reps
            ms_f, ms_b = time_events(torch, fwd, n), time_events(torch, bwd, n)
            f_flops = h * s * s * (dq + dv)
            b_flops = int(2.5 * f_flops)
            f_bytes = s * h * (dq * 4 + dv * 4) + h * s * 4
            b_bytes = s * h * (dq * 8 + dv * 6) + h * s * 8
            rows.append({
                "b": 1, "s": s, "h": h, "dq": dq, "dv": dv,
                "fwd": {"ms": round(ms_f, 4), "tflops": round(f_flops / ms_f / 1e9, 1), "tbps": round(f_bytes / ms_f / 1e9, 3),
                        "frac_mfma_peak": round(f_flops / ms_f / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4)},
                "bwd": {"ms": round(ms_b, 4), "tflops": round(b_flops / ms_b / 1e9, 1), "tbps": round(b_bytes / ms_b / 1e9, 3),
                        "frac_mfma_peak": round(b_flops / ms_b / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4)},
            })  # fmt: skip
            del q, k, v, do, o
            torch.cuda.empty_cache()
    return {
        "what": "causal MLA operator (module MLA, autograd backward = delta + dK/dV + dQ), the reference's benchmark "
                "matrix and FLOP / byte models (benchmarks/operators/mla/test_triton.py)",
        "rows": rows,
    }  # fmt: skip


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


def cpu_baseline_ring(torch, cfg, host_inputs, heads=None, backward=True):
    """The oracle's blocked fp32 eager-PyTorch port of the same ring share on the host cores, once: all query
    heads, or the sample heads = (first, last + 1) (whole kv-head groups), whose work is a fixed fraction of the
    configuration's (every head does the same work) and is counted as such."""
    from oracle import ring_oracle as R

    q, ks, vs, dout = host_inputs
    h0, h1 = heads if heads is not None else (0, cfg.hq)
    t0 = time.perf_counter()
    R.cpu_ring_fwd_bwd(q, ks, vs, dout, cfg.dqk**-0.5, cfg.rank, cfg.cp, LAYOUT, heads=(h0, h1), q_block=1024, backward=backward)
    dt = time.perf_counter() - t0
    fwd, bwd = cfg.flops()
    work = (fwd + (bwd if backward else 0)) * (h1 - h0) / cfg.hq
    what = "forward + backward" if backward else "forward only"
    sample = (f"the whole workload once (all {cfg.hq} query heads, all rows, {what})" if (h0, h1) == (0, cfg.hq) else
              f"query heads {h0}..{h1 - 1} of {cfg.hq} (of kv head {h0 // (cfg.hq // cfg.hkv)}), all rows, {what}: "
              f"{h1 - h0}/{cfg.hq} of the workload's FLOP, counted as such (the whole is not extrapolated from it)")  # fmt: skip
    return {
        "value": round(work / dt / 1e12, 4), "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"{sample}, fp32 eager PyTorch on bf16-rounded inputs, {dt:.1f} s; os.cpu_count()={os.cpu_count()}",
    }  # fmt: skip


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
    ap.add_argument("--config", choices=["mla16k", "long131k", "mla_op"], default=None,
                    help="time only this configuration (ring share, or the MLA operator matrix) and print its sub-object "
                         "(for kernel traces)")
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
    cpu_on = not args.no_cpu_baseline
    if args.config:
        if args.config == "mla_op":
            print(json.dumps({"mla_op": bench_mla_op(torch, device)}))
            return
        cfg = MLA16K if args.config == "mla16k" else LONG131K
        res = bench_other_config(torch, device, cfg, args.steps, args.warmup, counter_pass=args.counter_pass)
        print(json.dumps({args.config: res}) if res is not None else "counter pass done")
        return
    host_inputs, dev_inputs = make_inputs(torch, device)
    ms_step, ms_fwd, ms_bwd, out, lse = time_ring_share(torch, QWEN3, dev_inputs, args.steps, args.warmup)
    if args.counter_pass:
        # rocprofv3 --pmc run: a few more launches of the roofline kernel, a plain elementwise copy of known size
        # (256 MiB read, 256 MiB written) to calibrate the counter against, and the other kernels a few times each
        dominant_dkdv(torch, QWEN3, dev_inputs, out, lse, 1, counter_pass=True)
        src = torch.ones(64 << 20, dtype=torch.float32, device=device)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.mul(src, 1.0, out=dst)
        torch.cuda.synchronize()
        del dev_inputs, out, lse, src, dst
        bench_other_config(torch, device, MLA16K, 1, 0, counter_pass=True)
        bench_combine(torch, device, reps=4, graph=False)
        bench_norm_rope(torch, device, reps=3)
        bench_mla_assemble(torch, device, reps=3)
        print("counter pass done")
        return
    ms_dkdv, dkdv_flops, dkdv_n, scratch = dominant_dkdv(torch, QWEN3, dev_inputs, out, lse, args.steps)
    ms_fwdk, fwdk_flops, fwdk_n = dominant_fwd(torch, QWEN3, dev_inputs, args.steps)
    handover_on = scratch > 0
    scratch = handover_scratch_bytes(QWEN3, dev_inputs)
    recompute = None
    if not args.no_extra_configs and handover_on:
        recompute = bench_recompute(torch, dev_inputs, args.steps, args.warmup)
    del dev_inputs, out, lse
    torch.cuda.empty_cache()
    fwd_flops, bwd_flops = flops_per_step()
    tflops = (fwd_flops + bwd_flops) / (ms_step * 1e-3) / 1e12
    mla16k = long131k = mla_op = None
    if not args.no_extra_configs:
        mla16k = bench_other_config(torch, device, MLA16K, args.steps, args.warmup, cpu_heads="all" if cpu_on else None)
        # CPU sample of the long configuration: 4 of its 64 query heads (a quarter of one kv-head group; a whole
        # group would be ~90 s of host time)
        long131k = bench_other_config(torch, device, LONG131K, max(2, args.steps // 5), 1, cpu_heads=(0, 4) if cpu_on else None)
        mla_op = bench_mla_op(torch, device)
    ms_comb, ms_comb_eager, comb_bytes, comb_host = bench_combine(torch, device)
    comb_gbps = comb_bytes / (ms_comb * 1e-3) / 1e9
    nr_ms_f, nr_bytes_f, nr_ms_b, nr_bytes_b, nr_host = bench_norm_rope(torch, device)
    nr_gbps = (nr_bytes_f + nr_bytes_b) / ((nr_ms_f + nr_ms_b) * 1e-3) / 1e9
    ma_ms_f, ma_bytes_f, ma_ms_b, ma_bytes_b = bench_mla_assemble(torch, device)
    ma_gbps = (ma_bytes_f + ma_bytes_b) / ((ma_ms_f + ma_ms_b) * 1e-3) / 1e9

    cores = torch.get_num_threads()
    cpu = fwd_cpu = combine_cpu = norm_rope_cpu = None
    if cpu_on:
        cpu = cpu_baseline_ring(torch, QWEN3, host_inputs)
        fwd_cpu = cpu_baseline_ring(torch, QWEN3, host_inputs, backward=False)
        combine_cpu = {
            "value": round(cpu_baseline_combine(torch, comb_host, comb_bytes), 2), "unit": "GB/s", "cores": cores,
            "kind": "port", "sample": "full [1,4096,32,128] combine, eager PyTorch, median of 5",
        }  # fmt: skip
        norm_rope_cpu = {
            "value": round(cpu_baseline_norm_rope(torch, nr_host), 2), "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": "q tensor [1,8192,32,128] only, forward + backward, fp32 eager PyTorch, median of 3",
        }  # fmt: skip

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
            "workload": "the same share, forward only (4 chunk-attention launches and the log2 merges): O and the base-2 LSE",
            "ms": round(ms_fwd, 4), "tflops": round(fwd_flops / (ms_fwd * 1e-3) / 1e12, 2),
            "frac_mfma_peak": round(fwd_flops / (ms_fwd * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
            "roofline": roofline_entry(
                "attn_fwd_direct_kernel<128, non-causal> (S, P, O of one ring step)", fwdk_flops, ms_fwdk, fwdk_n,
                profile_figure(HBM_COUNTERS, "qwen3-32k.fwd_traffic_bytes_per_launch"), "profiles/" + HBM_COUNTERS),
            "cpu_baseline": fwd_cpu,
        },  # fmt: skip
        "roofline": roofline_entry(
            "attn_bwd_dkdv_d128_kernel<non-causal> (S, dP, dV, dK of one ring step"
            + ("; also stores its dS tiles for the dQ kernel)" if handover_on else ")"), dkdv_flops, ms_dkdv, dkdv_n,
            profile_figure(HBM_COUNTERS, "qwen3-32k.dkdv_traffic_bytes_per_launch" if handover_on
                           else "qwen3-32k.dkdv_traffic_bytes_per_launch_without_ds_stores"), "profiles/" + HBM_COUNTERS),  # fmt: skip
        "ds_handover": {
            "on": handover_on,
            "what": "the dK/dV kernel hands its dS tiles to the dQ kernel (5 matrix products executed instead of 7)",
            "scratch_bytes_per_ring_step": scratch,
            "recompute_backward": recompute,
        },
        "mla16k": mla16k,
        "long131k": long131k,
        "mla_op": mla_op,
        "combine": {
            "metric": "online_softmax_combine_log2 GB/s ([1,4096,32,128] bf16 x2 -> fp32)",
            "value": round(comb_gbps, 1), "unit": "GB/s", "us_per_launch": round(ms_comb * 1e3, 2),
            "timing": "replays of a captured HIP graph of 20 launches over 5 rotating buffer sets",
            "us_per_launch_eager": round(ms_comb_eager * 1e3, 2),
            "gbps_eager": round(comb_bytes / (ms_comb_eager * 1e-3) / 1e9, 1),
            "bytes": comb_bytes,
            "roofline": {"bound": "hbm", "achieved": round(comb_gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                         "frac": round(comb_gbps / HBM_PEAK_GBPS, 4),
                         "traffic": profile_figure(STREAM_COUNTERS, "combine.traffic_bytes_per_launch"),
                         "traffic_from": "profiles/" + STREAM_COUNTERS},
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
        "cpu_baseline": cpu,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
