"""Headline benchmark: ring-attention forward on ONE MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg4]

A step is one full forward of the workload: every ring step of every virtual rank, with Q/K/V
already resident in HBM -- one launch (ring_walk64_kernel at d = 128, else ring_walk_kernel) in which a
workgroup walks all ring steps of its 256 query rows with the softmax state in registers and writes O
and LSE at the end.
Prints one JSON line.  `value` is algorithmic TFLOP/s (4*B*H*d*visible (q,k) pairs per forward)
over the wall time of K steps; `roofline` prices the block-attention launch of the same forward
against the dense MFMA peak, timed by an event pair on the launch stream (a second pass of K
forwards on a plan with the timing flag); `sustained` is the same forward run back to back for a few
seconds more, the figure of its last second; `forward_with_step_partials` is the same forward on a
plan that keeps the ring steps apart (a fp32 partial (O, LSE) per step in a workspace, merged at
the end of each workgroup: another instantiation of the kernel, so a kernel trace keeps the two
apart; --step-partials makes that one the headline, --one-forward skips the other one); `merge`
times the merge kernel alone, on
caller-held per-step partials, against HBM bandwidth; `cpu_baseline` is the CPU oracle timed on
this host on a bounded sample of the same workload's rows.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# Published MI355X dense peaks used for the roofline (not the 2:1-sparsity figures)
PEAK_TFLOPS = {"bf16": 2500.0, "fp16": 2500.0}
PEAK_HBM_GBS = 8000.0
# HBM bytes per launch of the default forward's kernel measured with rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE): workload ->
# (bytes, summary under profiles/, kernel, kernel_source_id(kernel) when it was measured).  The figure is only printed
# while the forward still runs that kernel and its source is still the one that was profiled.
MEASURED_TRAFFIC = {
    "cfg4": (2243e6, "profiles/ring_walk64_kernel_cfg4.md", "ring_walk64_kernel", "4f2da51b8ee24e2d"),
    "cfg3": (2328e6, "profiles/ring_walk64_kernel_other_workloads.md", "ring_walk64_kernel", "4f2da51b8ee24e2d"),
    "cfg5": (48980e6, "profiles/ring_walk64_kernel_other_workloads.md", "ring_walk64_kernel", "4f2da51b8ee24e2d"),
    "cfg2": (34.3e6, "profiles/ring_walk64_kernel_other_workloads.md", "ring_walk64_kernel", "4f2da51b8ee24e2d"),
}
KERNEL_SOURCES = {
    "ring_walk64_kernel": ("ringattn_walk64.hip", "ringattn_walk64_loop.inc", "ringattn_walk64_loop_d64.inc", "ringattn_device.h"),
    "ring_walk_kernel": ("ringattn_walk.hip", "ringattn_device.h"),
}
BASELINE_METRIC = "ring-attn fwd TFLOP/s + % bf16 MFMA peak, S=32K d=128 8-step ring, 1 GPU"


def kernel_source_id(kernel):
    """Hash of the sources of one of the attention kernels."""
    import hashlib
    h = hashlib.sha256()
    try:
        for name in KERNEL_SOURCES[kernel]:
            with open(os.path.join(ROOT, "ringattention_amd", "csrc", name), "rb") as f:
                h.update(f.read())
    except (OSError, KeyError):
        return None
    return h.hexdigest()[:16]


def describe(w):
    return (f"{w.name}: {'causal' if w.causal else 'non-causal'} fwd, B={w.batch} H={w.heads} d={w.dim}, "
            f"{w.npes} virtual ranks x {w.chunk} tokens (S={w.seq}), {w.dtype}, N(0,{w.sigma_qk:g}^2) Q/K seed {w.seed}")


def visible_pairs(item):
    """(q, k) pairs of one work item (q_start, q_len, kv_start, kv_len, diag_off, slot)."""
    _, q_len, _, kv_len, diag_off, _ = item
    if diag_off < 0:
        return q_len * kv_len
    return q_len * diag_off + q_len * (q_len + 1) // 2


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="cfg4")
    ap.add_argument("--layout", default="contiguous", choices=["contiguous", "zigzag"],
                    help="placement of the sequence on the ranks (zigzag: load-balanced causal ring)")
    ap.add_argument("--rank-local", action="store_true",
                    help="also time the ring rank by rank on rank-local buffers (one launch per rank and step)")
    ap.add_argument("--per-step", action="store_true", help="also time one block-attention launch per ring step")
    ap.add_argument("--one-forward", action="store_true",
                    help="skip the forward of the other kind (see --step-partials), which is timed as well by default")
    ap.add_argument("--step-partials", action="store_true",
                    help="time the forward that keeps the ring steps apart (per-step partials in a workspace, merged at "
                         "the end) instead of the one that carries the softmax state through the steps")
    ap.add_argument("--operands", default="workload", choices=["workload", "zeros"],
                    help="diagnostic: 'zeros' runs the same launches on all-zero Q, K, V (same instruction stream, no operand "
                         "toggling: shows what the power manager leaves of the clock); not a valid headline")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="target CPU time of the cpu_baseline sample (0 = skip)")
    ap.add_argument("--sustain-seconds", type=float, default=2.5,
                    help="after the timed steps, run the same forward back to back for this long and report the last second (0 = skip)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (P virtual ring ranks on one MI355X); use --gpus 1")

    import numpy as np
    import torch
    from ringattention_amd import WORKLOADS, _lib, api
    _lib.load()   # fails loudly if the HIP extension is missing
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    torch.cuda.set_device(0)
    w = WORKLOADS[args.workload]

    q, k, v = api.make_qkv_bits(w)
    qd, kd, vd = (api.bits_to_tensor(x, w.dtype) for x in (q, k, v))
    if args.operands == "zeros":
        for t in (qd, kd, vd):
            t.zero_()
    plan = api.RingAttention(w.npes, w.chunk, w.dim, w.batch, w.heads, w.dtype, w.causal, graph=w.graph, layout=args.layout,
                             half_partials=w.half_partials, step_partials=args.step_partials)
    out = torch.empty_like(qd)
    lse = torch.empty((w.batch, w.heads, w.seq), dtype=torch.float32, device="cuda")
    stream = torch.cuda.current_stream()

    for _ in range(args.warmup):
        plan.forward(qd, kd, vd, out, lse, stream)
    torch.cuda.synchronize()
    # K steps between two synchronisations on the host clock, and the same K steps between an
    # event pair on the launch stream (the protocol of the reference harness, csrc/ring_attention.cu:772-783)
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record(stream)
    for _ in range(args.steps):
        plan.forward(qd, kd, vd, out, lse, stream)
    ev1.record(stream)
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    ms_per_step_events = ev0.elapsed_time(ev1) / args.steps
    tflops = w.flops / (ms_per_step * 1e-3) / 1e12

    # ---- what is sustained: the same forward back to back for --sustain-seconds more, in batches timed by event
    # pairs; reported: the batches of the last second (the first second of a process runs a few percent fast, before
    # the part's power manager has settled)
    sustained = None
    if args.sustain_seconds > 0:
        per_batch = max(1, int(round(0.1 / (ms_per_step * 1e-3))))    # about 0.1 s of forwards per batch
        batch_ms, t_start = [], time.perf_counter()
        while time.perf_counter() - t_start < args.sustain_seconds:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(per_batch):
                plan.forward(qd, kd, vd, out, lse, stream)
            e1.record(stream)
            torch.cuda.synchronize()
            batch_ms.append(e0.elapsed_time(e1) / per_batch)
        total_s = time.perf_counter() - t_start
        tail, acc = [], 0.0
        for x in reversed(batch_ms):     # the batches that make up the last second
            tail.append(x)
            acc += x * per_batch * 1e-3
            if acc >= 1.0:
                break
        last_ms = float(np.mean(tail))
        sustained = {"seconds": round(total_s, 2), "forwards": per_batch * len(batch_ms),
                     "ms_per_step_last_second": round(last_ms, 4),
                     "tflops_last_second": round(w.flops / (last_ms * 1e-3) / 1e12, 2),
                     "pct_mfma_peak_last_second": round(100.0 * w.flops / (last_ms * 1e-3) / 1e12 / PEAK_TFLOPS[w.dtype], 2),
                     "ms_per_step_first_batch": round(batch_ms[0], 4),
                     "clock_evidence": "profiles/ring_walk64_kernel_cfg4.md"}

    bh = w.batch * w.heads
    peak = PEAK_TFLOPS[w.dtype]
    # ---- attention kernel: the same forward on a plan that records an event pair around its
    # block-attention launch, on the stream it is launched on.  The launch is the whole ring (every
    # step of every rank).
    timed = api.RingAttention(w.npes, w.chunk, w.dim, w.batch, w.heads, w.dtype, w.causal, graph=False,
                              layout=args.layout, timing=True, half_partials=w.half_partials, step_partials=args.step_partials)
    timed.forward(qd, kd, vd, out, lse, stream)
    launch_ms = []
    for _ in range(args.steps):
        timed.forward(qd, kd, vd, out, lse, stream)
        launch_ms.append(timed.launch_times())
    launch_ms = np.array(launch_ms)                       # [steps, launches per forward]
    n_launch = launch_ms.shape[1]
    avg_launch_ms = float(launch_ms.mean())
    block_tflops = w.flops / n_launch / (avg_launch_ms * 1e-3) / 1e12
    traffic, traffic_source = None, "not measured for this workload / layout"
    kernel = timed.forward_kernel()
    if args.layout == "contiguous" and not args.step_partials and w.name in MEASURED_TRAFFIC:
        t_bytes, t_profile, t_kernel, t_src = MEASURED_TRAFFIC[w.name]
        if t_kernel == kernel and t_src == kernel_source_id(kernel):
            traffic, traffic_source = t_bytes, t_profile
        else:
            traffic_source = (f"stale: {t_profile} was measured on {t_kernel} with source {t_src}, this is {kernel} "
                              f"with source {kernel_source_id(kernel)}")
    roofline = {
        "kernel": kernel, "bound": "mfma",
        "achieved": round(block_tflops, 2), "peak": peak, "unit": "TFLOP/s", "frac": round(block_tflops / peak, 4),
        "traffic": traffic, "traffic_source": traffic_source,
        "launches_per_step": n_launch, "avg_launch_ms": round(avg_launch_ms, 4),
        "avg_launch_flop": w.flops / n_launch,
        "launch_ms": [round(float(x), 4) for x in launch_ms.mean(axis=0)],
    }
    timed.close()

    # ---- the other forward (steps kept apart unless --step-partials, which swaps the two)
    other_leg = None
    if not args.one_forward:
        other = api.RingAttention(w.npes, w.chunk, w.dim, w.batch, w.heads, w.dtype, w.causal, graph=w.graph, layout=args.layout,
                                  half_partials=w.half_partials, step_partials=not args.step_partials)
        for _ in range(2):
            other.forward(qd, kd, vd, out, lse, stream)
        ev0.record(stream)
        for _ in range(args.steps):
            other.forward(qd, kd, vd, out, lse, stream)
        ev1.record(stream)
        torch.cuda.synchronize()
        other_ms = ev0.elapsed_time(ev1) / args.steps
        other_leg = {"ms_per_step_events": round(other_ms, 4), "tflops": round(w.flops / (other_ms * 1e-3) / 1e12, 2),
                     "workspace_bytes": int(other.lib.ringattn_workspace_bytes(other.params)),
                     "partials": "none" if args.step_partials else ("fp16" if w.half_partials else "fp32")}
        other.close()

    # ---- merge kernel alone: the ring merge on caller-held partials (random numbers: only the
    # bytes matter), events on the launch stream
    eager = api.RingAttention(w.npes, w.chunk, w.dim, w.batch, w.heads, w.dtype, w.causal, graph=False, layout=args.layout,
                              half_partials=w.half_partials)
    o_parts = torch.empty((w.npes, w.batch, w.heads, w.seq, w.dim), dtype=eager.part_dtype, device="cuda").normal_()
    l_parts = torch.empty((w.npes, w.batch, w.heads, w.seq), dtype=torch.float32, device="cuda").normal_()
    reps = max(3, min(args.steps, 10))
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(reps + 1)]
    eager.merge_ring(o_parts, l_parts, out, lse, stream)
    for r in range(reps):
        ev[r].record(stream)
        eager.merge_ring(o_parts, l_parts, out, lse, stream)
    ev[reps].record(stream)
    torch.cuda.synchronize()
    merge_ms = float(np.mean([ev[r].elapsed_time(ev[r + 1]) for r in range(reps)]))
    # algorithmic bytes = active parts * (4 d + 4) read (2 d + 4 with fp16 partials) + (2 d + 4) written, per row
    part_row = (2 if w.half_partials else 4) * w.dim + 4
    merge_bytes = bh * sum(ln * (bin(act).count("1") * part_row + 2 * w.dim + 4) for _, ln, act in eager.merge_regions())
    merge = {"kernel": "merge_kernel", "bound": "hbm", "achieved": round(merge_bytes / (merge_ms * 1e-3) / 1e9, 1),
             "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(merge_bytes / (merge_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
             "ms": round(merge_ms, 4), "bytes": merge_bytes, "launches": 1, "regions": len(eager.merge_regions())}

    # ---- optional: one launch per ring step (what ringattn_block_fwd runs), to show how the work
    # spreads over the steps of the ring
    per_step = None
    if args.per_step:
        evs = [[torch.cuda.Event(enable_timing=True) for _ in range(w.npes + 1)] for _ in range(reps)]
        for rep in range(-1, reps):   # rep -1 warms up
            for s in range(w.npes):
                if rep >= 0:
                    evs[rep][s].record(stream)
                eager.block_forward(s, qd, kd, vd, o_parts[s], l_parts[s], stream)
            if rep >= 0:
                evs[rep][w.npes].record(stream)
        torch.cuda.synchronize()
        step_ms = [np.mean([evs[r][s].elapsed_time(evs[r][s + 1]) for r in range(reps)]) for s in range(w.npes)]
        step_flops = [4.0 * w.dim * bh * sum(visible_pairs(it) for it in eager.work_items(s)) for s in range(w.npes)]
        assert abs(sum(step_flops) - w.flops) <= 1e-9 * w.flops
        per_step = {"ms": [round(float(x), 4) for x in step_ms],
                    "tflops": [round(f / (t * 1e-3) / 1e12, 1) for f, t in zip(step_flops, step_ms)]}
    del o_parts, l_parts
    # the same merge with a row's steps next to each other (RINGATTN_FLAG_ROW_PARTIALS): same bytes, one run per row
    rowp = api.RingAttention(w.npes, w.chunk, w.dim, w.batch, w.heads, w.dtype, w.causal, graph=False, layout=args.layout,
                             half_partials=w.half_partials, row_partials=True)
    o_shape, l_shape = rowp.parts_shapes()
    o_parts = torch.empty(o_shape, dtype=rowp.part_dtype, device="cuda").normal_()
    l_parts = torch.empty(l_shape, dtype=torch.float32, device="cuda").normal_()
    rowp.merge_ring(o_parts, l_parts, out, lse, stream)
    for r in range(reps):
        ev[r].record(stream)
        rowp.merge_ring(o_parts, l_parts, out, lse, stream)
    ev[reps].record(stream)
    torch.cuda.synchronize()
    row_ms = float(np.mean([ev[r].elapsed_time(ev[r + 1]) for r in range(reps)]))
    merge["row_major_partials"] = {"achieved": round(merge_bytes / (row_ms * 1e-3) / 1e9, 1), "ms": round(row_ms, 4),
                                   "frac": round(merge_bytes / (row_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)}
    rowp.close()
    del o_parts, l_parts

    # ---- optional: the ring as one process per GPU would run it, replayed rank by rank on this
    # GPU with rank-local buffers (ringattn_rank_step_fwd / ringattn_rank_merge): every launch is one
    # (rank, step), i.e. the kernel on one GPU's share at its real shape.  In a real ring the ranks
    # move in lockstep (one K/V exchange per step), so a step costs what its slowest rank costs.
    ring = None
    if args.rank_local:
        P, c = w.npes, w.chunk
        kvh = w.heads
        t_step = np.zeros((P, P))
        t_merge = np.zeros(P)
        for r in range(P):
            q_r = qd[:, :, r * c:(r + 1) * c].contiguous()
            op = torch.zeros((P, w.batch, w.heads, c, w.dim), dtype=eager.part_dtype, device="cuda")
            lp = torch.full((P, w.batch, w.heads, c), float("-inf"), dtype=torch.float32, device="cuda")
            o_r = torch.empty((w.batch, w.heads, c, w.dim), dtype=qd.dtype, device="cuda")
            l_r = torch.empty((w.batch, w.heads, c), dtype=torch.float32, device="cuda")
            chunks = [(kd[:, :, j * c:(j + 1) * c].contiguous(), vd[:, :, j * c:(j + 1) * c].contiguous()) for j in range(P)]
            e = [[torch.cuda.Event(enable_timing=True) for _ in range(P + 2)] for _ in range(reps)]
            for rep in range(-1, reps):
                for st in range(P):
                    if rep >= 0:
                        e[rep][st].record(stream)
                    kj, vj = chunks[(r + st) % P]
                    eager.rank_step_forward(r, st, q_r, kj, vj, op[st], lp[st], stream)
                if rep >= 0:
                    e[rep][P].record(stream)
                eager.rank_merge(r, op, lp, o_r, l_r, stream)
                if rep >= 0:
                    e[rep][P + 1].record(stream)
            torch.cuda.synchronize()
            for st in range(P):
                t_step[r, st] = np.mean([e[k][st].elapsed_time(e[k][st + 1]) for k in range(reps)])
            t_merge[r] = np.mean([e[k][P].elapsed_time(e[k][P + 1]) for k in range(reps)])
            del q_r, op, lp, o_r, l_r, chunks
        lockstep = float(t_step.max(axis=0).sum() + t_merge.max())
        ring = {"per_rank_ms": [round(float(x), 4) for x in (t_step.sum(axis=1) + t_merge)],
                "per_step_slowest_rank_ms": [round(float(x), 4) for x in t_step.max(axis=0)],
                "lockstep_ms": round(lockstep, 4),
                "per_gpu_tflops_in_lockstep": round(w.flops / P / (lockstep * 1e-3) / 1e12, 1)}
    eager.close()
    plan_ws = plan.lib.ringattn_workspace_bytes(plan.params)
    plan.close()

    # ---- CPU baseline: the oracle (a port; the reference has no CPU attention path) on a
    # bounded, seeded sample of rows of the same workload
    cpu = None
    if args.cpu_seconds > 0:
        from oracle import oracle
        rng = np.random.default_rng(12345)
        per_row = 4.0 * w.dim * (np.arange(w.seq) + 1 if w.causal else np.full(w.seq, w.seq))   # FLOP per row index
        n, dt = 2048, 0.0
        for _ in range(4):   # grow the sample until it costs about --cpu-seconds of CPU work
            rows = rng.integers(0, w.rows, n)
            t = time.perf_counter()
            oracle.attention_rows(q, k, v, w.dtype, causal=w.causal, rows=rows)
            dt = time.perf_counter() - t
            if dt >= 0.6 * args.cpu_seconds or n >= w.rows:
                break
            n = int(min(w.rows, n * min(32.0, args.cpu_seconds / max(dt, 1e-3))))
        fl = float(per_row[rows % w.seq].sum())
        cpu = {"value": round(fl / dt / 1e12, 5), "unit": "TFLOP/s", "cores": oracle.num_threads(), "kind": "port",
               "sample": f"{n} seeded random query rows of {w.name} ({fl:.3e} FLOP) in {dt:.1f} s, fp64 oracle; "
                         f"full forward extrapolates to {w.flops / (fl / dt):.0f} s"}

    print(json.dumps({
        "metric": BASELINE_METRIC if (w.name == "cfg4" and args.layout == "contiguous" and args.operands == "workload")
        else f"ring-attn fwd TFLOP/s + % {w.dtype} MFMA peak, {describe(w)}, {args.layout} layout, 1 GPU"
        + ("" if args.operands == "workload" else ", ALL-ZERO OPERANDS (diagnostic)"),
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "ms_per_step_events": round(ms_per_step_events, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": w.dtype, "data": "synthetic" if args.operands == "workload" else "all-zero operands (diagnostic, not the workload)",
        "config": {"workload": describe(w), "algorithmic_flop": w.flops, "graph": bool(w.graph), "layout": args.layout,
                   "partials": ("fp16" if w.half_partials else "fp32") if args.step_partials
                   else "none: softmax state carried through the ring steps in registers",
                   "workspace_bytes": int(plan_ws)},
        "pct_mfma_peak": round(100.0 * tflops / peak, 2),
        "sustained": sustained,
        "roofline": roofline,
        ("forward_with_carried_state" if args.step_partials else "forward_with_step_partials"): other_leg,
        "merge": merge, "per_ring_step": per_step, "rank_local_ring": ring, "cpu_baseline": cpu,
    }))


if __name__ == "__main__":
    main()
