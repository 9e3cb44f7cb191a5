#!/usr/bin/env python3
"""Benchmark of the bidirectional GLA forward on one MI355X.

A step = one bidirectional GLA forward (both directions, one library call) over
one batch of synthetic inputs of the named workload, inputs resident in HBM.
Input sets are rotated (>= 3 sets, > 256 MB in total) so that timed launches read
HBM rather than the 256 MB Infinity Cache.

Prints ONE JSON line on stdout; everything else goes to stderr.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 MFMA, published


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def cpu_baseline(shape, seed, budget_s=20.0):
    """Times the float32 torch port of the reference's recurrent routine on the host cores.

    The sample is the named workload with the batch cut so one run stays near `budget_s`.
    """
    import torch

    from oracle import gla_oracle as O
    from vig_amd.synthetic import make_gla_inputs

    threads = torch.get_num_threads()
    # probe at batch 4 to size the sample
    probe_B = min(4, shape.B)
    q, k, v, gf, gb = make_gla_inputs(probe_B, shape.H, shape.L, shape.Dk, shape.Dv, seed, torch.float32)
    t0 = time.perf_counter()
    O.bidir_naive_recurrent_gla_f32(q, k, v, gf, gb)
    t_probe = time.perf_counter() - t0
    per_b = t_probe / probe_B
    B = int(max(1, min(shape.B, budget_s / 3 / max(per_b, 1e-9))))
    q, k, v, gf, gb = make_gla_inputs(B, shape.H, shape.L, shape.Dk, shape.Dv, seed, torch.float32)
    O.bidir_naive_recurrent_gla_f32(q, k, v, gf, gb)  # warm-up
    ts = []
    t_begin = time.perf_counter()
    while len(ts) < 3 or (time.perf_counter() - t_begin < budget_s / 2 and len(ts) < 200):
        t0 = time.perf_counter()
        O.bidir_naive_recurrent_gla_f32(q, k, v, gf, gb)
        ts.append(time.perf_counter() - t0)
    t = sorted(ts)[len(ts) // 2]
    tokens = B * shape.H * shape.L
    flops = tokens * 8 * shape.Dk * shape.Dv
    return {
        "value": flops / t / 1e12,
        "unit": "TFLOP/s",
        "cores": threads,
        "kind": "port",
        "sample": f"B={B} of {shape.B} (H={shape.H} L={shape.L} Dk={shape.Dk} Dv={shape.Dv}, fp32 torch recurrent port, "
                  f"two sweeps summed), median of {len(ts)} runs, {t:.3f} s",
        "tokens_per_s": tokens / t,
    }


def model_throughput(dev, batch=256, warmup=10, iters=30, tune_gemm=True, use_graph=True):
    """Full ViG-S eval forward (random init, synthetic images, bf16): images/s the way the reference's
    throughput() measures it (classification/main.py:389-406: timed forwards of one resident batch)."""
    import torch

    from vig_amd import layers

    tuned = _enable_gemm_tuning(tune_gemm)
    torch.manual_seed(0)
    model = layers.vig_small().eval().to(dev, torch.bfloat16)
    images = torch.randn(batch, 3, 224, 224, device=dev, dtype=torch.bfloat16)
    from vig_amd import evaluate
    ips = evaluate.throughput(model, images, warmup=warmup, iters=iters)
    dt = iters * batch / ips
    out = {"images_per_s": iters * batch / dt, "batch": batch, "dtype": "bf16", "iters": iters,
           "ms_per_forward": dt / iters * 1e3, "gemm_solution_tuning": "torch.cuda.tunable" if tuned else None}
    # the same forward as one HIP graph (one submission instead of ~190 launches), if it replays bit for bit
    if use_graph:
        if tuned:
            torch.cuda.tunable.tuning_enable(False)  # every shape has its solution by now; none is tried under capture
        graphed = evaluate.graphed_forward_checked(model, images)
        if graphed is not None:
            ips_g = evaluate.throughput(graphed, images, warmup=warmup, iters=iters)
            out["hip_graph"] = {"images_per_s": ips_g, "ms_per_forward": batch / ips_g * 1e3,
                                "replays_checked_against_eager": 4}
        else:
            out["hip_graph"] = None
        # a small batch is bound by the ~190 launches, not by the kernels: there the graph is what counts
        small = images[:16].contiguous()
        ips_e = evaluate.throughput(model, small, warmup=warmup, iters=iters)
        g16 = evaluate.graphed_forward_checked(model, small)
        out["batch16_latency_ms"] = {"eager": 16 / ips_e * 1e3,
                                     "hip_graph": 16 / evaluate.throughput(g16, small, warmup=warmup, iters=iters) * 1e3
                                     if g16 is not None else None}
    return out


def _enable_gemm_tuning(tune_gemm):
    """The GEMMs are hipBLASLt calls made by torch; let torch pick the fastest solution per shape."""
    try:
        if not tune_gemm:
            raise RuntimeError("switched off")
        import tempfile

        import torch.cuda.tunable as tunable
        tunable.enable(True)
        tunable.tuning_enable(True)
        tunable.set_max_tuning_duration(200)
        tunable.set_filename(os.path.join(tempfile.gettempdir(), "vig_bench_gemm_solutions.csv"))
        return True
    except Exception as e:  # noqa: BLE001 - tuning is optional plumbing
        log(f"GEMM tuning unavailable: {e}")
        return False


def train_step_throughput(dev, batch=128, warmup=3, iters=10, tune_gemm=True):
    """ViG-S training steps (forward, cross-entropy, backward, AdamW update) on synthetic images: the differentiable
    path of the shell, whose kernels between the GEMMs are the library's in both directions.  fp32 as the reference's
    configs train (vig-s.yaml: AMP off), and bf16 autocast."""
    import torch

    from vig_amd import layers

    tuned = _enable_gemm_tuning(tune_gemm)
    out = {"batch": batch, "iters": iters, "gemm_solution_tuning": "torch.cuda.tunable" if tuned else None}
    images = torch.randn(batch, 3, 224, 224, device=dev)
    target = torch.randint(0, 1000, (batch,), device=dev)
    for name, amp in (("fp32", False), ("bf16_autocast", True)):
        torch.manual_seed(0)
        model = layers.vig_small().to(dev).train()
        opt = torch.optim.AdamW(model.parameters(), lr=1e-4)

        def step():
            opt.zero_grad(set_to_none=True)
            with torch.autocast("cuda", dtype=torch.bfloat16, enabled=amp):
                loss = torch.nn.functional.cross_entropy(model(images).float(), target)
            loss.backward()
            opt.step()
            return loss

        for _ in range(warmup):
            step()
        torch.cuda.synchronize(dev)
        t0 = time.perf_counter()
        for _ in range(iters):
            loss = step()
        torch.cuda.synchronize(dev)
        dt = (time.perf_counter() - t0) / iters
        out[name] = {"images_per_s": batch / dt, "ms_per_step": dt * 1e3, "loss": float(loss.detach())}
        del model, opt
    return out


def backward_time(lib, sets, s, io_dt, scale, sp, stream, dev, iters=60):
    """Event-bracketed time of vig_gla_bidir_bwd, rotating over the input sets like the forward loop does."""
    import torch

    q, k, v, gf, gb, o = sets[0]
    d_os = [torch.randn_like(t[2]) for t in sets]
    dq, dk, dv, dgf, dgb = (torch.empty_like(t) for t in (q, k, v, gf, gb))
    n = lib.vig_gla_bidir_bwd_workspace(s.B, s.H, s.L, s.Dk, s.Dv, 1)
    if n == 0:
        return None
    ws = torch.empty(n, dtype=torch.uint8, device=dev)

    def run(i):
        q, k, v, gf, gb, _ = sets[i % len(sets)]
        d_o = d_os[i % len(sets)]
        rc = lib.vig_gla_bidir_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), gf.data_ptr(), gb.data_ptr(), d_o.data_ptr(),
                                   dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), dgf.data_ptr(), dgb.data_ptr(),
                                   ws.data_ptr(), n, s.B, s.H, s.L, s.Dk, s.Dv, scale, 1.0, io_dt, io_dt, sp)
        if rc != 0:
            raise RuntimeError(f"vig_gla_bidir_bwd rc={rc}")

    for i in range(3):
        run(i)
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    for i, (a, b) in enumerate(evs):
        a.record(stream)
        run(i)
        b.record(stream)
    torch.cuda.synchronize()
    us = sum(a.elapsed_time(b) for a, b in evs) / iters * 1e3
    esz = 4 if s.dtype == "f32" else 2
    mfma = s.dtype != "f32" and s.Dk in (32, 64) and s.Dv == 64
    alg = s.tokens * esz * ((2 * s.Dk + 2 * s.Dv) + 2 * s.Dk + (2 * s.Dk + s.Dv) + 2 * s.Dk)
    return {"us": us, "algorithmic_bytes": alg, "algorithmic_GBps": alg / (us * 1e-6) / 1e9,
            "frac_of_hbm_peak": alg / (us * 1e-6) / 1e9 / HBM_PEAK_GBPS,
            "kernel": ("fp32 token-recurrent" if not mfma else
                       "matrix cores (whole-slab quadratic form), bf16 operands" if s.L <= 256 else
                       "matrix cores (segments of <= 256 tokens linked by states), bf16 operands")}



def other_workload_time(lib, idx, dev, stream, steps=20, warmup=5):
    """Event-bracketed time of one more named workload (op only): inputs of the workload's shape and distributions drawn
    on the device (timing only: the parity tests use the seeded CPU draws), >= 3 sets and > 256 MB rotated."""
    import torch
    import torch.nn.functional as F

    from vig_amd import _lib
    from vig_amd.synthetic import CONFIGS, make_locality_weight

    s = CONFIGS[idx]
    g = torch.Generator(device=dev)
    g.manual_seed(1000 + idx)
    nsets = max(3, int(300e6 // s.alg_bytes()) + 1)
    sets = []
    for _ in range(nsets):
        q = torch.randn(s.B, s.H, s.L, s.Dk, device=dev, generator=g)
        k = torch.randn(s.B, s.H, s.L, s.Dk, device=dev, generator=g) * s.Dk ** -0.5
        v = torch.randn(s.B, s.H, s.L, s.Dv, device=dev, generator=g)
        gf = F.logsigmoid(torch.randn(s.B, s.H, s.L, s.Dk, device=dev, generator=g)) / 16
        gb = F.logsigmoid(torch.randn(s.B, s.H, s.L, s.Dk, device=dev, generator=g)) / 16
        sets.append(tuple(t.bfloat16() for t in (q, k, v, gf, gb)) + (torch.empty(s.B, s.H, s.L, s.Dv, dtype=torch.bfloat16, device=dev),))
    ws_bytes = lib.vig_gla_bidir_fwd_workspace(s.B, s.H, s.L, s.Dk, s.Dv, _lib.VIG_BF16)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    sp = stream.cuda_stream
    scale = s.Dk ** -0.5
    gate_w = None
    if idx == 2:
        gate_w = make_locality_weight(s.H * s.Dv, 2002).reshape(s.H * s.Dv, 9).float().contiguous().to(dev)

    def step(i):
        q, k, v, gf, gb, o = sets[i % nsets]
        if gate_w is not None:
            rc = lib.vig_gla_bidir_locgate_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), gf.data_ptr(), gb.data_ptr(),
                                               gate_w.data_ptr(), o.data_ptr(), s.B, s.H, s.L, s.Dk, s.Dv, s.grid[0],
                                               s.grid[1], scale, 1.0, _lib.VIG_BF16, _lib.VIG_BF16, sp)
        else:
            rc = lib.vig_gla_bidir_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), gf.data_ptr(), gb.data_ptr(), o.data_ptr(),
                                       ws.data_ptr(), ws_bytes, s.B, s.H, s.L, s.Dk, s.Dv, scale, 1.0, _lib.VIG_BF16,
                                       _lib.VIG_BF16, sp)
        if rc != 0:
            raise RuntimeError(f"workload {idx}: rc={rc}")

    for i in range(warmup):
        step(i)
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for i, (a, b) in enumerate(evs):
        a.record(stream)
        step(i)
        b.record(stream)
    torch.cuda.synchronize()
    durs = sorted(a.elapsed_time(b) * 1e3 for a, b in evs)
    us = sum(durs) / len(durs)
    gbps = s.alg_bytes() / (us * 1e-6) / 1e9
    out = {"workload": s.name, "steps": steps, "us": us, "us_min": durs[0], "algorithmic_bytes": s.alg_bytes(),
           "achieved_GBps": gbps, "frac": gbps / HBM_PEAK_GBPS, "tflops_algorithmic": s.alg_flops() / (us * 1e-6) / 1e12,
           "inputs": "the workload's shape and distributions, drawn on the device", "traffic": None}
    out.update(_measured_traffic(s.name, "traffic"))
    if idx == 2:
        out["locality_gate"] = "inside the GLA kernel"
    del sets
    return out


def _measured_traffic(key, field="traffic"):
    """HBM bytes per launch from the rocprofv3 counter runs kept under profiles/ (FETCH_SIZE / WRITE_SIZE scaled by a
    copy kernel of known size), with the source commit and date of that counter run."""
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            t = json.load(f)
        e = t.get(key)
        if not e:
            return {field: None}
        return {field: e.get("bytes_per_launch"),
                field + "_measured": {"commit": e.get("commit", t.get("_commit")), "date": e.get("date", t.get("_date")),
                                      "kernels": e.get("kernels")}}
    except (OSError, ValueError):
        return {field: None}

def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", type=int, default=1, help="named workload index (1 = ViG-S shape, the headline)")
    ap.add_argument("--sets", type=int, default=0, help="input sets to rotate (0 = enough to exceed 256 MB, >= 3)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--exact", action="store_true", help="time the fp32-arithmetic recurrent kernel instead")
    ap.add_argument("--model", action="store_true",
                    help="also time the full ViG-S eval forward (images/s); on by default for the headline workload")
    ap.add_argument("--backward", action="store_true",
                    help="also time the backward of the op on the same workload; on by default for the headline workload")
    ap.add_argument("--op-only", action="store_true", help="no model forward and no backward, whatever the workload")
    ap.add_argument("--no-gemm-tuning", action="store_true",
                    help="with --model / --train: leave torch's GEMM solution tuning off (clean kernel traces)")
    ap.add_argument("--train", action="store_true",
                    help="also time ViG-S training steps (differentiable path of the shell; fp32 and bf16 autocast)")
    ap.add_argument("--train-only", action="store_true",
                    help="time only the ViG-S training steps and print their JSON line (clean kernel traces)")
    ap.add_argument("--no-graph", action="store_true",
                    help="with --model: eager forwards only (no HIP graph capture, no batch-16 latency)")
    ap.add_argument("--unfused-gate", action="store_true",
                    help="workload 2: run the locality gate as a second kernel instead of inside the GLA kernel")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run plain device copies of known size (q -> o), so that FETCH_SIZE / WRITE_SIZE "
                         "counters of a profiled run can be scaled to bytes")
    args = ap.parse_args()

    if args.gpus != 1:
        log("bench.py: this build runs on ONE GPU; (batch, head) pairs are independent, so more GPUs would only "
            "shard the batch. --gpus must be 1.")
        sys.exit(2)

    import torch

    import vig_amd
    from vig_amd import _lib
    from vig_amd.synthetic import CONFIGS, make_gla_inputs, torch_dtype

    if not os.path.exists(_lib.LIB_PATH):
        from vig_amd.build import build_library
        build_library()
    lib = _lib.load()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.train_only:
        res = train_step_throughput(dev, tune_gemm=not args.no_gemm_tuning)
        print(json.dumps({"metric": "ViG-S training step images/sec @224^2 (forward + backward + AdamW)",
                          "value": res["bf16_autocast"]["images_per_s"], "unit": "images/s", "n_gpus": 1,
                          "ms_per_step": res["bf16_autocast"]["ms_per_step"], "higher_is_better": True,
                          "dtype": "bf16 autocast", "data": "synthetic", "vs_baseline": None,
                          "config": {"workload": "vig_s_train_step_B128_224"}, "detail": res}))
        return

    s = CONFIGS[args.config]
    dt = torch_dtype(s.dtype)
    alg_bytes = s.alg_bytes()
    alg_flops = s.alg_flops()
    nsets = args.sets or max(3, int(300e6 // alg_bytes) + 1)
    log(f"workload {s.name}: tokens={s.tokens} alg_bytes={alg_bytes/1e6:.1f} MB alg_flops={alg_flops/1e9:.2f} GF, "
        f"{nsets} input sets")

    sets = []
    for i in range(nsets):
        q, k, v, gf, gb = make_gla_inputs(s.B, s.H, s.L, s.Dk, s.Dv, 1000 + args.config + 17 * i, dt)
        sets.append(tuple(t.to(dev) for t in (q, k, v, gf, gb)) + (torch.empty(s.B, s.H, s.L, s.Dv, dtype=dt, device=dev),))
    io_dt = _lib.VIG_F32 if s.dtype == "f32" else _lib.VIG_BF16
    ws_bytes = lib.vig_gla_bidir_fwd_workspace(s.B, s.H, s.L, s.Dk, s.Dv, io_dt)
    if args.exact and s.dtype != "f32":
        ws_bytes = max(ws_bytes, s.B * s.H * s.L * s.Dv * 4)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev)
    sp = stream.cuda_stream
    fn = lib.vig_gla_bidir_fwd_exact if args.exact else lib.vig_gla_bidir_fwd
    scale = s.Dk ** -0.5

    # workload 2 adds the sigmoid locality gate on the 14x14 grid of the GLA output: inside the GLA kernel, or with
    # --unfused-gate as a second (stencil) kernel over the stored output
    with_gate = args.config == 2
    fused_gate = with_gate and not args.unfused_gate and not args.exact
    if with_gate:
        from vig_amd.synthetic import make_locality_weight
        gate_w = make_locality_weight(s.H * s.Dv, 2002).reshape(s.H * s.Dv, 9).float().contiguous().to(dev)
        gate_out = [torch.empty_like(t[5]) for t in sets]

    def step(i):
        q, k, v, gf, gb, o = sets[i % nsets]
        if fused_gate:
            rc = lib.vig_gla_bidir_locgate_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), gf.data_ptr(), gb.data_ptr(),
                                               gate_w.data_ptr(), gate_out[i % nsets].data_ptr(), s.B, s.H, s.L, s.Dk,
                                               s.Dv, s.grid[0], s.grid[1], scale, 1.0, io_dt, io_dt, sp)
            if rc != 0:
                raise RuntimeError(f"vig_gla_bidir_locgate_fwd rc={rc}")
            return
        rc = fn(q.data_ptr(), k.data_ptr(), v.data_ptr(), gf.data_ptr(), gb.data_ptr(), o.data_ptr(),
                ws.data_ptr(), ws_bytes, s.B, s.H, s.L, s.Dk, s.Dv, scale, 1.0, io_dt, io_dt, sp)
        if rc != 0:
            raise RuntimeError(f"vig_gla_bidir_fwd rc={rc}")
        if with_gate:
            rc = lib.vig_locality_gate_fwd(o.data_ptr(), gate_w.data_ptr(), gate_out[i % nsets].data_ptr(), s.B, s.H,
                                           s.grid[0], s.grid[1], s.Dv, io_dt, sp)
            if rc != 0:
                raise RuntimeError(f"vig_locality_gate_fwd rc={rc}")

    if args.copy_calibration:
        # a copy kernel whose traffic is known exactly: numel*2 bytes read, numel*2 bytes written per call
        for i in range(4):
            sets[i % nsets][5].copy_(sets[i % nsets][2])
        torch.cuda.synchronize()
        log(f"copy calibration: {sets[0][2].numel() * sets[0][2].element_size()} bytes read and written per copy kernel")

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()

    # whole-loop wall clock: K steps between two synchronisations
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / args.steps * 1e3

    # per-launch device time: HIP events recorded on the launch stream around each launch
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    for i in range(args.steps):
        evs[i][0].record(stream)
        step(i)
        evs[i][1].record(stream)
    torch.cuda.synchronize()
    durs = sorted(a.elapsed_time(b) for a, b in evs)  # ms
    k_avg = sum(durs) / len(durs)
    k_med = durs[len(durs) // 2]
    k_min = durs[0]
    log(f"wall {ms_per_step*1e3:.1f} us/step; event-bracketed launch avg {k_avg*1e3:.1f} us, median {k_med*1e3:.1f}, min {k_min*1e3:.1f}")

    # what this box's memory system gives a plain device-to-device copy that moves the same number of bytes (half read,
    # half written), timed the same way on rotating buffers: the practical ceiling beside the published 8 TB/s
    copy_ref = None
    if not args.exact:
        half = alg_bytes // 2
        bufs = [(torch.empty(half, dtype=torch.uint8, device=dev), torch.empty(half, dtype=torch.uint8, device=dev))
                for _ in range(max(3, int(300e6 // alg_bytes) + 1))]
        for i in range(10):
            bufs[i % len(bufs)][1].copy_(bufs[i % len(bufs)][0])
        cev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(50)]
        for i, (a, b) in enumerate(cev):
            a.record(stream)
            bufs[i % len(bufs)][1].copy_(bufs[i % len(bufs)][0])
            b.record(stream)
        torch.cuda.synchronize()
        c_us = sum(a.elapsed_time(b) for a, b in cev) / len(cev) * 1e3
        copy_ref = {"bytes": 2 * half, "us": c_us, "GBps": 2 * half / (c_us * 1e-6) / 1e9,
                    "what": "torch copy_ of alg_bytes/2 (read) into alg_bytes/2 (written), event-bracketed, rotating buffers"}
        log(f"device copy of the same bytes: {c_us:.1f} us ({copy_ref['GBps']:.0f} GB/s)")
        del bufs

    # HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE / WRITE_SIZE, scaled by a copy kernel of known
    # size); the figures live with the profile summaries, keyed by workload, with the commit and date they were taken at
    traffic = _measured_traffic(s.name)

    tflops = alg_flops / (ms_per_step * 1e-3) / 1e12
    achieved_gbps = alg_bytes / (k_avg * 1e-3) / 1e9
    exec_flops_tok = 2 * (2 * 64 * (s.Dk + s.Dv) + 4 * s.Dk * s.Dv)  # executed MFMA FLOPs/token at chunk 64

    out = {
        "metric": "bidir GLA fwd TFLOP/s (algorithmic 8*Dk*Dv FLOP/token, both directions, 1 GPU)",
        "value": tflops,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": s.dtype,
        "data": "synthetic",
        "config": {"workload": s.name, "B": s.B, "H": s.H, "L": s.L, "Dk": s.Dk, "Dv": s.Dv,
                   "input_sets_rotated": nsets, "kernel_path": "recurrent_fp32" if args.exact else "default",
                   "locality_gate": ("inside the GLA kernel" if fused_gate else "separate stencil kernel after the GLA")
                   if with_gate else None},
        "tokens_per_s": s.tokens / (ms_per_step * 1e-3),
        "mfma_frac_algorithmic": tflops / MFMA_BF16_PEAK_TFLOPS,
        "executed_tflops_chunk64": s.tokens * exec_flops_tok / (ms_per_step * 1e-3) / 1e12,
        "kernel_us": {"avg": k_avg * 1e3, "median": k_med * 1e3, "min": k_min * 1e3},
        "roofline": {"bound": "hbm", "achieved": achieved_gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved_gbps / HBM_PEAK_GBPS, **traffic},
        "device_copy_same_bytes": copy_ref,
    }
    # the headline run (config 1) also reports the other half of the metric (ViG-S images/s) and the backward
    # (--backward --op-only: the forward and the backward of the op, nothing else)
    want_backward = (args.backward or (args.config == 1 and not args.op_only)) and not args.exact
    want_model = (args.model or args.config == 1) and not args.op_only and not args.exact
    if want_backward:
        out["backward"] = backward_time(lib, sets, s, io_dt, scale, sp, stream, dev)
        if out["backward"] is not None:
            out["backward"].update(_measured_traffic(s.name + ":backward"))
    if args.config == 1 and not args.op_only and not args.exact:
        # the other named workloads, op only, 20 steps each: every roofline figure of the report is timed by this run
        others = {}
        for idx in (2, 3, 4):
            others[f"cfg{idx}"] = other_workload_time(lib, idx, dev, stream)
            log(f"workload {idx}: {others[f'cfg{idx}']['us']:.1f} us, {100 * others[f'cfg{idx}']['frac']:.1f} % of HBM peak")
        out["other_workloads"] = others
        out["long_sequence"] = others["cfg3"]  # the 4096-token workload: the second named target
    if want_model:
        if args.train:
            out["vig_s_train_step"] = train_step_throughput(dev, tune_gemm=not args.no_gemm_tuning)
        out["vig_s_forward"] = model_throughput(dev, tune_gemm=not args.no_gemm_tuning, use_graph=not args.no_graph)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(s, 1000 + args.config)
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
