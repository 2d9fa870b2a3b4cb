#!/usr/bin/env python3
"""Benchmark of the Q8_0 mul_mat hot path on one MI355X.

A step is one call of the fused Q8_0 linear (activation quantize + int8 MFMA + per-block scale
settlement) over one batch of synthetic activations already resident in HBM.  The workload is the
MSA-track QKV projection: X 26368 x 256 f32 ~N(0,1), W 768 x 256 Q8_0 from N(0,0.02), Y 26368 x 768
f32.  Consecutive steps rotate through several X/Y buffer pairs whose total size exceeds the 256 MB
last-level cache, so every step streams its operands from HBM.

Prints ONE JSON line.  ``value`` is int8 TOPS (2*M*N*K per step / time); ``roofline`` prices the
same kernel against HBM, its binding roof (algorithmic bytes: X once, W once, Y once);
``cpu_baseline`` is the CPU oracle timed on this box's host cores on the same workload.
``extra`` lists the other configured shapes, each measured the same way.
"""
from __future__ import annotations

import argparse
import json
import os
import re
import sys
import time

METRIC = "Q8_0 mul_mat TOPS + GB/s (% of int8 MFMA / HBM roofline), 1 MI355X"
HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
INT8_PEAK_TOPS = 5000.0      # dense int8 MFMA, published
FP32_MFMA_PEAK_TFLOPS = 157.3
BF16_MFMA_PEAK_TFLOPS = 2500.0

PREHEAT_MS = 40.0            # untimed load ahead of every timed region: the chip needs 25-30 ms of continuous load to settle
EVENT_REGION_MS = 5.0        # least length of each of the three event-timed regions
PROFILES = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles")
TRAFFIC_PROFILE = os.path.join(PROFILES, "q8_linear_msa_qkv_hbm_traffic.md")
TRAFFIC_PROFILE_OTHERS = os.path.join(PROFILES, "hbm_traffic_other_configured_shapes.md")


def measured_traffic_bytes(name=None):
    """HBM bytes per launch as the committed rocprofv3 --pmc summaries state them (FETCH_SIZE + WRITE_SIZE, each
    scaled by the same counter's reading for a 1 GiB copy).  The dominant kernel: the line
    ``traffic_bytes_per_launch: <integer>`` of profiles/q8_linear_msa_qkv_hbm_traffic.md; another configured
    shape: the line ``traffic_bytes_per_launch[<name>]: <integer>`` of
    profiles/hbm_traffic_other_configured_shapes.md.  None when the summary or the line is not there."""
    path = TRAFFIC_PROFILE if name is None else TRAFFIC_PROFILE_OTHERS
    key = r"traffic_bytes_per_launch" + ("" if name is None else r"\[" + re.escape(name) + r"\]")
    try:
        with open(path) as f:
            m = re.search(r"^" + key + r":\s*(\d+)", f.read(), flags=re.M)
        return int(m.group(1)) if m else None
    except OSError:
        return None


def q8_bytes(rows, K, N):
    """Algorithmic HBM bytes of one Q8_0 linear: f32 activations in, Q8_0 weights in, f32 out."""
    return rows * K * 4 + N * K * 34 // 32 + rows * N * 4


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=500,
                    help="untimed steps; the shader clock needs 1-2 ms of load to reach its steady value")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the other configured shapes")
    ap.add_argument("--configured-shapes-only", action="store_true",
                    help="of the other shapes, measure only the five HBM-bound configured ones (the short run that the "
                         "rocprofv3 --pmc traffic passes use)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a 1 GiB device copy, the kernel of known size against which the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run are scaled")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (no collectives, no sharding); "
              "run with --gpus 1", file=sys.stderr)
        return 2

    import torch

    from proteinpredictmachinelearning_amd import ops

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the backend has no CPU path", file=sys.stderr)
        return 3
    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(1)

    def time_op(fn, nsets, steps, warmup):
        """Two clocks, both reported; neither depends on the other's length.
        Pre-heat: PREHEAT_MS of untimed launches of the same step.  After any pause of 10 ms or more the chip runs
        a load at full speed for about a millisecond, then 15-50 % slower for some 15 ms, and is back at its steady
        rate after 25-30 ms of continuous load; both clocks below start behind that.
        Wall: `warmup` untimed steps, one device synchronisation, then exactly `steps` steps up to the next
        synchronisation (the whole-job figure: it contains the launch latency of the first step).
        Events: three consecutive regions of `event_steps` launches each between HIP events on the launch stream,
        event_steps = max(steps, EVENT_REGION_MS / step time) -- a region of fixed length in time, whatever `steps`
        is -- queued directly behind more untimed launches so that the queue is deep when the first event is
        reached; the figure is the median region.  Returns (wall s / step, event s / step); details in
        time_op.last."""
        for i in range(3):
            fn(i % nsets)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(5):
            fn(i % nsets)
        torch.cuda.synchronize()
        est = max((time.perf_counter() - t0) / 5, 1e-6)
        heat = min(40000, int(PREHEAT_MS * 1e-3 / est) + 1)
        for i in range(heat):
            fn(i % nsets)
        for i in range(warmup):
            fn(i % nsets)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            fn(i % nsets)
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) / steps
        event_steps = max(steps, min(40000, int(EVENT_REGION_MS * 1e-3 / max(wall, 1e-7)) + 1))
        marks = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
        for i in range(max(warmup, min(heat, event_steps))):
            fn(i % nsets)
        marks[0].record()
        for r in range(3):
            for i in range(event_steps):
                fn(i % nsets)
            marks[r + 1].record()
        torch.cuda.synchronize()
        regions = sorted(marks[r].elapsed_time(marks[r + 1]) * 1e-3 / event_steps for r in range(3))
        time_op.last = {"event_steps": event_steps, "event_regions_us": [round(t * 1e6, 2) for t in regions],
                        "preheat_launches": heat}
        return wall, regions[1]

    # the event machinery's first use in a process costs some 150 us inside the region that contains it
    first = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    first[0].record()
    first[1].record()
    torch.cuda.synchronize()
    first[0].elapsed_time(first[1])

    # ------------------------------------------------------------------ what the bytes alone cost
    import ctypes as C
    probe_path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "bench_probe", "libppml_probe.so")
    probe = C.CDLL(probe_path) if os.path.exists(probe_path) else None
    if probe is not None:
        probe.ppml_probe_stream.restype = C.c_int
        probe.ppml_probe_stream.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int, C.c_int, C.c_void_p]

    def bytes_only_us(read_bytes, write_bytes, steps, warmup):
        """Time per launch of a kernel that only reads `read_bytes` and writes `write_bytes` (16 bytes per lane,
        coalesced, buffers rotated past the last-level cache), measured in the same loop as everything else: the
        practical floor of a launch with that HBM traffic on this box, launch latency included.  The best of
        streaming / ordinary stores and of a one-pass / persistent grid."""
        if probe is None:
            return None
        read_bytes, write_bytes = (int(read_bytes) + 15) // 16 * 16, (int(write_bytes) + 15) // 16 * 16
        ns = max(2, int(640e6 // (read_bytes + write_bytes)) + 1)
        srcs = [torch.randn(max(read_bytes, 16) // 4, device=dev, generator=gen) for _ in range(ns)]
        dsts = [torch.empty(max(write_bytes, 16) // 4, device=dev) for _ in range(ns)]
        stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        best = None
        for nt in (1, 0):
            for groups in (0, 2048):
                def fn(i, nt=nt, groups=groups):
                    probe.ppml_probe_stream(C.c_void_p(srcs[i].data_ptr()), C.c_void_p(dsts[i].data_ptr()), read_bytes, write_bytes,
                                            nt, groups, stream)
                _, ev_ = time_op(fn, ns, steps, warmup)
                best = ev_ if best is None else min(best, ev_)
        return round(best * 1e6, 2)

    def q8_case(rows, K, N, relu=False, packed=True):
        nbytes = q8_bytes(rows, K, N)
        nsets = max(2, int(640e6 // nbytes) + 1)
        w = torch.randn(N, K, device=dev, generator=gen) * 0.02
        W = ops.Q8Weight.from_f32(w)                    # block_q8_0 records, as the reference's loader leaves them
        if packed:
            W = W.pack()
        xs = [torch.randn(rows, K, device=dev, generator=gen) for _ in range(nsets)]
        ys = [torch.empty(rows, N, device=dev) for _ in range(nsets)]
        lib, cabi = ops._lib(), ops.cabi
        stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        wp = C.c_void_p(W.data.data_ptr())
        xp = [C.c_void_p(x.data_ptr()) for x in xs]
        yp = [C.c_void_p(y.data_ptr()) for y in ys]
        flags = 1 if relu else 0

        def fn(i):
            rc = lib.mul_mat_q8_ex_hip(wp, xp[i], yp[i], N, rows, K, W.wtype, 1, flags, None, None, stream)
            if rc:
                cabi.check("mul_mat_q8_ex_hip", rc)
        return fn, nsets, nbytes, 2.0 * rows * K * N, (w, xs[0])

    # ------------------------------------------------------------------ headline: MSA QKV
    rows, K, N = 26368, 256, 768
    fn, nsets, nbytes, nops, (w0, x0) = q8_case(rows, K, N)
    wall, ev = time_op(fn, nsets, args.steps, args.warmup)
    value = nops / wall / 1e12
    achieved = nbytes / ev / 1e9
    out = {
        "metric": METRIC,
        "value": round(value, 3),
        "unit": "TOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall * 1e3, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic (seeded normal draws made on the device)",
        "config": {"workload": "MSA-track QKV Q8_0 linear: X 26368x256 f32 -> Q8_0 on the fly, "
                               "W 768x256 Q8_0, Y 26368x768 f32",
                   "buffer_rotation": nsets, "weight_layout": "Q8_0M (MFMA fragments)"},
        "preheat_ms": PREHEAT_MS,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": measured_traffic_bytes(),
                     "kernel": "q8_linear_ws_kernel", "algorithmic_bytes_per_launch": nbytes,
                     "kernel_us": round(ev * 1e6, 2),
                     "clock": "HIP events on the launch stream: median of three consecutive regions of event_steps launches, "
                              "queued behind preheat_ms of load",
                     "event_steps": time_op.last["event_steps"], "event_regions_us": time_op.last["event_regions_us"],
                     "wall_us": round(wall * 1e6, 2), "frac_wall_clock": round(nbytes / wall / 1e9 / HBM_PEAK_GBS, 4),
                     "clocks_differ_by_more_than_10_percent": bool(abs(ev - wall) > 0.1 * min(ev, wall)),
                     "int8_mfma_frac": round(nops / ev / 1e12 / INT8_PEAK_TOPS, 4),
                     "bytes_only_us": bytes_only_us(rows * K * 4 + N * K * 34 // 32, rows * N * 4, max(20, args.steps // 4), 5)},
    }

    # ------------------------------------------------------------------ CPU baseline (oracle, rank 0)
    cpu_pair = None
    if not args.no_cpu:
        import numpy as np
        import oracle   # the checker, timed here as a reported baseline only

        threads = min(len(os.sched_getaffinity(0)), 16)

        def cpu_leg(run, nthreads, budget_s):
            reps, t_cpu = 0, 0.0
            while t_cpu < budget_s and reps < 50:
                t0 = time.perf_counter()
                run(nthreads)
                t_cpu += time.perf_counter() - t0
                reps += 1
            return reps, t_cpu

        def cpu_pair(run, work, unit, what, budget_all=3.0, budget_ref=2.5):
            """The CPU oracle on `threads` host threads and on the reference's own default of 4
            (PPML_N_THREADS, src/model/PPML.cpp:3828-3833); `work` = operations of one pass of `run`."""
            reps, t_cpu = cpu_leg(run, threads, budget_all)
            reps4, t_cpu4 = cpu_leg(run, min(4, threads), budget_ref)
            return {"value": round(work * reps / t_cpu / 1e12, 5), "unit": unit, "cores": threads, "kind": "port",
                    "sample": f"{reps} passes of {what}, {t_cpu:.1f} s of CPU time",
                    "reference_default_threads": {"value": round(work * reps4 / t_cpu4 / 1e12, 5), "unit": unit,
                                                  "cores": min(4, threads),
                                                  "sample": f"{reps4} passes, {t_cpu4:.1f} s of CPU time"}}

        def q8_cpu(w_dev, x_dev, relu, work, what, **budgets):
            xh = x_dev.cpu().numpy()
            wq = oracle.quantize_q8_0(w_dev.cpu().numpy())
            if relu:
                return cpu_pair(lambda nt: oracle.mul_mat_q8(wq, np.maximum(xh, 0.0), wtype=0, c_trans=1, fma=1, nthreads=nt),
                                work, "TOPS", what + " (ReLU + quantize rows + block dot)", **budgets)
            return cpu_pair(lambda nt: oracle.mul_mat_q8(wq, xh, wtype=0, c_trans=1, fma=1, nthreads=nt),
                            work, "TOPS", what + " (quantize rows + block dot)", **budgets)

        out["cpu_baseline"] = q8_cpu(w0, x0, False, nops, "the whole 26368x256->768 workload", budget_all=10.0, budget_ref=8.0)

    # ------------------------------------------------------------------ the other configured shapes
    if not args.no_extra:
        extra = {}
        steps, warm = max(20, args.steps // 2), max(5, args.warmup // 2)
        for name, (r, k, n, relu) in {
            "dev_linear_408x256_256": (408, 256, 256, False),
            "pair_ff_up_10609x128_512": (10609, 128, 512, False),
            "pair_ff_down_relu_10609x512_128": (10609, 512, 128, True),
        }.items():
            f, ns, nb, no, (w_dev, x_dev) = q8_case(r, k, n, relu)
            w_, e_ = time_op(f, ns, steps, warm)
            extra[name] = {"us": round(e_ * 1e6, 2), "TOPS": round(no / e_ / 1e12, 2), "GBps": round(nb / e_ / 1e9, 1),
                           "hbm_frac": round(nb / e_ / 1e9 / HBM_PEAK_GBS, 4), "kernel": ops.last_q8_path(),
                           "event_steps": time_op.last["event_steps"], "algorithmic_bytes_per_launch": nb,
                           "traffic": measured_traffic_bytes(name),
                           "bytes_only_us": bytes_only_us(r * k * 4 + n * k * 34 // 32, r * n * 4, steps, warm)}
            if cpu_pair is not None:
                extra[name]["cpu_baseline"] = q8_cpu(w_dev, x_dev, relu, no, f"the whole {r}x{k}->{n} workload")

        # the headline shape on a weight in the reference's own layout (block_q8_0 records): the library packs it into
        # its workspace per call and runs the same kernel
        if not args.configured_shapes_only:
            f, ns, nb, no, _ = q8_case(26368, 256, 768, packed=False)
            w_, e_ = time_op(f, ns, steps, warm)
            extra["msa_qkv_on_a_block_q8_0_weight_26368x256_768"] = {
                "us": round(e_ * 1e6, 2), "TOPS": round(no / e_ / 1e12, 2), "GBps": round(nb / e_ / 1e9, 1),
                "hbm_frac": round(nb / e_ / 1e9 / HBM_PEAK_GBS, 4), "kernel": ops.last_q8_path(), "event_steps": time_op.last["event_steps"]}

        # a compute-bound shape of the same operator (no shape of the reference's model is one: its quantized
        # projections all have K <= 512): large weights take the tiled kernel, measured against the int8 matrix peak
        if not args.configured_shapes_only:
            r, k, n = 4096, 4096, 4096
            f, ns, nb, no, _ = q8_case(r, k, n)
            w_, e_ = time_op(f, ns, max(10, steps // 4), 3)
            extra["q8_linear_large_4096x4096_4096"] = {"us": round(e_ * 1e6, 2), "TOPS": round(no / e_ / 1e12, 2),
                                                       "int8_mfma_frac": round(no / e_ / 1e12 / INT8_PEAK_TOPS, 4),
                                                       "kernel": ops.last_q8_path(), "event_steps": time_op.last["event_steps"]}

        rest = {"skip": False}

        def f32_case(make, nbytes, flops, name, pipe="fp32", rw=None, cpu=None):
            if rest["skip"]:
                return
            # pipe: "fp32" = fp32 MFMA; "bf16x3" = binary32 operands split three ways, six bf16 MFMA
            # products per binary32 product (TFLOPS counts binary32 products, the fraction bf16 ones)
            fn_, ns = make()
            w_, e_ = time_op(fn_, ns, steps, warm)
            extra[name] = {"us": round(e_ * 1e6, 2), "TFLOPS": round(flops / e_ / 1e12, 2),
                           "GBps": round(nbytes / e_ / 1e9, 1), "hbm_frac": round(nbytes / e_ / 1e9 / HBM_PEAK_GBS, 4)}
            if pipe == "bf16x3":
                extra[name]["bf16_mfma_frac"] = round(6.0 * flops / e_ / 1e12 / BF16_MFMA_PEAK_TFLOPS, 4)
            elif pipe == "f16":                         # halves straight to the matrix pipe (same published peak as bf16)
                extra[name]["f16_mfma_frac"] = round(flops / e_ / 1e12 / BF16_MFMA_PEAK_TFLOPS, 4)
            else:
                extra[name]["fp32_mfma_frac"] = round(flops / e_ / 1e12 / FP32_MFMA_PEAK_TFLOPS, 4)
            if rw is not None:                          # (bytes read, bytes written) of an HBM-bound shape
                extra[name]["bytes_only_us"] = bytes_only_us(rw[0], rw[1], steps, warm)
                extra[name]["algorithmic_bytes_per_launch"] = nbytes
                extra[name]["traffic"] = measured_traffic_bytes(name)
            extra[name]["event_steps"] = time_op.last["event_steps"]
            if cpu is not None and cpu_pair is not None:
                extra[name]["cpu_baseline"] = cpu()

        keep = []

        def logits(planes, L, D):
            def make():
                nb = (2 * planes * D * L + planes * L * L) * 4
                ns = max(2, int(640e6 // nb) + 1)
                ks = [torch.randn(1, planes, D, L, device=dev, generator=gen) for _ in range(ns)]
                qs = [torch.randn(1, planes, D, L, device=dev, generator=gen) for _ in range(ns)]
                outs = [torch.empty(1, planes, L, L, device=dev) for _ in range(ns)]
                # straight through the C ABI on preallocated outputs: the Python operator's own bookkeeping
                # (shape checks, output allocation) costs more host time per call than the small shape takes on the GPU
                lib, cabi = ops._lib(), ops.cabi
                stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
                dims = [L, D, planes, 1, L, D, planes, 1, L, L, planes, 1]
                argsets = [(C.c_void_p(ks[i].data_ptr()), C.c_void_p(qs[i].data_ptr()), C.c_void_p(outs[i].data_ptr()), *dims,
                            1.0 / D ** 0.5, stream) for i in range(ns)]

                def fn(i):
                    rc = lib.out_prod_scaled_hip(*argsets[i])
                    if rc:
                        cabi.check("out_prod_scaled_hip", rc)
                keep.append((ks, qs, outs))
                return fn, ns
            return make
        def logits_cpu(planes, L, D):
            # the reference's two nodes on the CPU: kernel_out_prod then kernel_scale (CPUKernels.cpp:787-887, 1737-1754)
            def cpu():
                ks, qs, _ = keep[-1]
                kh, qh = ks[0].cpu().numpy(), qs[0].cpu().numpy()
                s = float(np.float32(1.0) / np.sqrt(np.float32(D)))
                return cpu_pair(lambda nt: oracle.scale(oracle.out_prod(kh, qh, nthreads=nt), s, nthreads=nt),
                                2.0 * planes * L * L * D, "TFLOPS", f"the whole {planes} x {L} x {L} x {D} workload (out_prod + scale)")
            return cpu
        f32_case(logits(412, 103, 32), (2 * 412 * 32 * 103 + 412 * 103 * 103) * 4, 2.0 * 412 * 103 * 103 * 32,
                 "attn_logits_pair_412x103x103x32", pipe="bf16x3", rw=(2 * 412 * 32 * 103 * 4, 412 * 103 * 103 * 4),
                 cpu=logits_cpu(412, 103, 32))
        f32_case(logits(824, 256, 32), (2 * 824 * 32 * 256 + 824 * 256 * 256) * 4, 2.0 * 824 * 256 * 256 * 32,
                 "attn_logits_msa_824x256x256x32", pipe="bf16x3", rw=(2 * 824 * 32 * 256 * 4, 824 * 256 * 256 * 4),
                 cpu=logits_cpu(824, 256, 32))

        rest["skip"] = args.configured_shapes_only         # everything below is beyond the configured shapes
        def attention(planes, L, D, with_bias, layout=0):
            def make():
                import ctypes as C
                nb = (4 * planes * L * D + planes * L + (planes * L * L if with_bias else 0)) * 4
                ns = max(2, int(640e6 // nb) + 1)
                qkv = [[torch.randn(1, planes, L, D, device=dev, generator=gen) for _ in range(3)] for _ in range(ns)]
                bs = [torch.randn(1, planes, L, L, device=dev, generator=gen) if with_bias else None for _ in range(ns)]
                outs = [(torch.empty(1, planes, L, D, device=dev), torch.empty(1, planes, L, device=dev)) for _ in range(ns)]
                lib, cabi = ops._lib(), ops.cabi
                stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
                ptr = lambda t: C.c_void_p(t.data_ptr()) if t is not None else None      # noqa: E731
                argsets = [(1, planes, L, D, 0, 0.0, 1e-9, 64, ptr(qkv[i][0]), ptr(qkv[i][1]), ptr(qkv[i][2]), ptr(bs[i]),
                            ptr(outs[i][0]), ptr(outs[i][1]), layout, stream) for i in range(ns)]

                def fn(i):
                    rc = lib.flash_attn_forward_ex_hip(*argsets[i])
                    if rc:
                        cabi.check("flash_attn_forward_ex_hip", rc)
                keep.append((qkv, bs, outs))
                return fn, ns
            return make
        # layout 3: Q, K, V and O in the graph's [L, D, h, B] layout, i.e. without the four permutation copies
        for planes, L, D, wb, lay, tag in [(412, 103, 32, True, 0, "pair_412x103x32_bias"), (824, 256, 32, True, 0, "msa_824x256x32_bias"),
                                           (824, 256, 32, False, 0, "msa_824x256x32"),
                                           (824, 256, 32, True, 3, "msa_824x256x32_bias_graph_layout")]:
            f32_case(attention(planes, L, D, wb, lay), (4 * planes * L * D + planes * L + (planes * L * L if wb else 0)) * 4,
                     4.0 * planes * L * L * D, "fused_attention_" + tag, pipe="bf16x3")

        def attention_back(planes, L, D):
            def make():
                import ctypes as C
                nb = (8 * planes * L * D + planes * L + 2 * planes * L * L) * 4
                ns = max(2, int(640e6 // nb) + 1)
                t = lambda *shape: torch.randn(*shape, device=dev, generator=gen)      # noqa: E731
                sets = []
                for _ in range(ns):
                    q, k, v, do, b = t(1, planes, L, D), t(1, planes, L, D), t(1, planes, L, D), t(1, planes, L, D), t(1, planes, L, L)
                    o, lse = ops.flash_attn_forward(q, k, v, b)
                    sets.append((q, k, v, b, o, do, lse, torch.empty_like(q), torch.empty_like(q), torch.empty_like(q), torch.empty_like(b)))
                lib, cabi = ops._lib(), ops.cabi
                stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
                argsets = [(1, planes, L, D, 0, 0.0) + tuple(C.c_void_p(x.data_ptr()) for x in s_) + (stream,) for s_ in sets]

                def fn(i):
                    rc = lib.flash_attn_backward_hip(*argsets[i])
                    if rc:
                        cabi.check("flash_attn_backward_hip", rc)
                keep.append(sets)
                return fn, ns
            return make
        # flops: five 2*L*L*D contractions per plane in exact terms (S, dP, dQ, dK, dV); S and dP are computed twice
        f32_case(attention_back(824, 256, 32), (8 * 824 * 256 * 32 + 824 * 256 + 2 * 824 * 256 * 256) * 4,
                 10.0 * 824 * 256 * 256 * 32, "fused_attention_backward_msa_824x256x32_bias", pipe="bf16x3")

        def bridge():
            # the [L, D, h, B] -> [D, L, h, B] copy in front of the fused attention node, MSA-track size
            import ctypes as C
            ns = 12
            xs = [torch.randn(824, 32, 256, device=dev, generator=gen) for _ in range(ns)]
            ys = [torch.empty(824, 256, 32, device=dev) for _ in range(ns)]
            lib, cabi = ops._lib(), ops.cabi
            stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
            argsets = [(C.c_void_p(xs[i].data_ptr()), C.c_void_p(ys[i].data_ptr()), 824 * 32 * 256, 3, 1, 0, 2, 3,
                        256, 32, 824, 1, 32, 256, 824, 1, stream) for i in range(ns)]

            def fn(i):
                rc = lib.permute_hip(*argsets[i])
                if rc:
                    cabi.check("permute_hip", rc)
            keep.append((xs, ys))
            return fn, ns
        f32_case(bridge, 2 * 824 * 32 * 256 * 4, 0.0, "permute_attention_bridge_824x256x32", rw=(824 * 32 * 256 * 4, 824 * 32 * 256 * 4))

        def trimul():
            # triangle multiplication (outgoing) of the pair track: 128 channels x 103 x 103, contracted length 103
            import ctypes as C
            Dc, Lr = 128, 103
            ns = 40
            ls = [torch.randn(Dc * Lr * Lr, device=dev, generator=gen) for _ in range(ns)]
            rs = [torch.randn(Dc * Lr * Lr, device=dev, generator=gen) for _ in range(ns)]
            os_ = [torch.empty(Dc * Lr * Lr, device=dev) for _ in range(ns)]
            lib, cabi = ops._lib(), ops.cabi
            stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
            argsets = [(C.c_void_p(ls[i].data_ptr()), C.c_void_p(rs[i].data_ptr()), C.c_void_p(os_[i].data_ptr()),
                        Dc, Lr, Lr, Lr, 1, 1.0 / Lr, 1, stream) for i in range(ns)]

            def fn(i):
                rc = lib.tri_mul_hip(*argsets[i])
                if rc:
                    cabi.check("tri_mul_hip", rc)
            keep.append((ls, rs, os_))
            return fn, ns
        f32_case(trimul, 3 * 128 * 103 * 103 * 4, 2.0 * 128 * 103 ** 3, "tri_mul_outgoing_128x103x103x103")

        opm_operands = []

        def opm():
            a = torch.randn(256, 12288, device=dev, generator=gen) * 0.1
            b = torch.randn(256, 12288, device=dev, generator=gen) * 0.1
            opm_operands[:] = [a, b]
            return (lambda i: ops.mul_mat_tn(a, b, 1.0 / 256)), 1

        def opm_cpu():
            # the reference's CPU mul_mat (CPUKernels.cpp:763-771) on the transposed operands, on a sample of the output
            # rows: 768 of 12288 (one sixteenth of the 77.3 GFLOP), every column, followed by the 1/N scale
            rows_sample = 768
            at = np.ascontiguousarray(opm_operands[0][:, :rows_sample].cpu().numpy().T)
            bt = np.ascontiguousarray(opm_operands[1].cpu().numpy().T)
            inv = float(np.float32(1.0) / np.float32(256))
            return cpu_pair(lambda nt: oracle.scale(oracle.mul_mat_f32(at, bt, nthreads=nt), inv, nthreads=nt),
                            2.0 * rows_sample * 12288 * 256, "TFLOPS",
                            f"{rows_sample} of the 12288 output rows x all 12288 columns x K = 256 (1/16 of the workload)")
        steps, warm = 50, 10
        f32_case(opm, (2 * 256 * 12288 + 12288 * 12288) * 4, 2.0 * 12288 * 12288 * 256, "opm_dense_12288x256x12288", pipe="bf16x3",
                 cpu=opm_cpu)

        def dense():
            a = torch.randn(4096, 4096, device=dev, generator=gen)
            b = torch.randn(4096, 4096, device=dev, generator=gen)
            return (lambda i: ops.mul_mat(a, b)), 1
        f32_case(dense, 3 * 4096 * 4096 * 4, 2.0 * 4096 ** 3, "mul_mat_f32_4096x4096x4096", pipe="bf16x3")

        # the same two contractions on the fp32 matrix pipe (the library's other arithmetic for binary32 operands)
        ops.set_f32_arithmetic("fp32")
        try:
            steps, warm = 20, 5
            f32_case(opm, (2 * 256 * 12288 + 12288 * 12288) * 4, 2.0 * 12288 * 12288 * 256,
                     "opm_dense_12288x256x12288_fp32_pipe", pipe="fp32")
            f32_case(dense, 3 * 4096 * 4096 * 4, 2.0 * 4096 ** 3, "mul_mat_f32_4096x4096x4096_fp32_pipe", pipe="fp32")
        finally:
            ops.set_f32_arithmetic("split")

        def opm_back():
            # both gradients of the graph-form outer-product-mean at D = 32, L = 384, N = 256: two contractions
            # 12288 x 12288 -> 256 over a compound index of the 604 MB gradient tensor, cut into K slices
            Dc, Lc, Nc = 32, 384, 256
            left = torch.randn(Dc * Lc * Nc, device=dev, generator=gen) * 0.1
            right = torch.randn(Dc * Lc * Nc, device=dev, generator=gen) * 0.1
            grad = torch.randn(Dc * Dc * Lc * Lc, device=dev, generator=gen) * 0.1
            return (lambda i: ops.outer_prod_mean_back(grad, left, right, Dc, Lc, Nc, 1)), 1
        steps, warm = 20, 5
        f32_case(opm_back, (2 * 12288 * 12288 + 4 * 12288 * 256) * 4, 4.0 * 12288 * 12288 * 256,
                 "opm_backward_D32_L384_N256", pipe="bf16x3")

        def weight_grad():
            # dW = X^T dY of the headline projection's f32 twin (src/core/ComputeGraph.cpp:708-773): 256 x 768 outputs,
            # contraction over the 26368 tokens, cut into K slices
            ns = 3
            xs = [torch.randn(26368, 256, device=dev, generator=gen) for _ in range(ns)]
            dys = [torch.randn(26368, 768, device=dev, generator=gen) for _ in range(ns)]
            keep.append((xs, dys))
            return (lambda i: ops.mul_mat_tn(xs[i], dys[i])), ns
        steps, warm = 50, 10
        f32_case(weight_grad, (26368 * 256 + 26368 * 768 + 256 * 768) * 4, 2.0 * 26368 * 256 * 768,
                 "linear_weight_gradient_26368x256_768", pipe="bf16x3")

        def f16_linear():
            # the headline projection with both operands in halves (F16 x F16 -> F32, src/backend/CPUKernels.cpp:646-672)
            ns = 8
            xs = [torch.randn(26368, 256, device=dev, generator=gen).half() for _ in range(ns)]
            w16 = (torch.randn(768, 256, device=dev, generator=gen) * 0.05).half()
            keep.append((xs, w16))
            return (lambda i: ops.mul_mat_f16(xs[i], w16)), ns
        f32_case(f16_linear, 26368 * 256 * 2 + 768 * 256 * 2 + 26368 * 768 * 4, 2.0 * 26368 * 256 * 768,
                 "mul_mat_f16_26368x256_768", pipe="f16")

        def bias_grad():
            # dbias[n] = sum over the tokens of dY[token][n] (OP_REPEAT_BACK, src/backend/CPUKernels.cpp:2091-2148)
            ns = 6
            dys = [torch.randn(26368, 768, device=dev, generator=gen) for _ in range(ns)]
            keep.append(dys)
            return (lambda i: ops.repeat_back(dys[i], (768,))), ns
        f32_case(bias_grad, (26368 * 768 + 768) * 4, 0.0, "linear_bias_gradient_26368x768")
        out["extra"] = extra

    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_(generator=gen)   # 1 GiB
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        out["copy_calibration"] = {"bytes_read": src.numel() * 4, "bytes_written": dst.numel() * 4, "launches": 5}

    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
