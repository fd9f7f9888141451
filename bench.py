#!/usr/bin/env python3
"""Benchmark of the eclat kernel path on one MI355X.

A step is one pass of the hot path (execute the compiled Program) over one batch
of synthetic input.  The headline workload is benchmark configuration 2 -- row softmax of
fp32 [4096, 4096], compiled from the reference's five-kernel lowering into one
fused launch -- reported as HBM GB/s of algorithmic traffic (one read + one
write).  The same JSON line carries configs 3, 1, 4 and 5 under "extra", each with a
roofline object; for configs 1, 2, 4 and 5 also the per-kernel path (what the reference's
unmodified executor would drive: one synchronous launch per lowered kernel); and the CPU
baseline (the oracle's C kernels, unfused, on host cores).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--options key=value,...]
"""

from __future__ import annotations

import argparse
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--options", default="")
    ap.add_argument("--no-tuned", action="store_true", help="do not load harp_amd/tuned_gfx950.txt")
    ap.add_argument("--sets", type=int, default=4)
    ap.add_argument("--only", default="", help="softmax | matmul | config1 | mlp | cnn (default: all)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-per-kernel", action="store_true", help="skip the per-kernel (unfused, synchronous) path")
    ap.add_argument("--no-check", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this path runs on one GPU (every kernel here works on one GPU's "
                 "share at its real shape); run with --gpus 1")
    if args.steps < 1 or args.warmup < 0:
        sys.exit("bench.py: --steps must be >= 1 and --warmup >= 0")

    from harp_amd import backend as hb
    from harp_amd import measure
    from harp_amd import workloads as wl
    from harp_amd.measure import FP32_MFMA_PEAK_TFLOPS, HBM_PEAK_GBS      # MI355X published peaks
    if hb.device_count() == 0:
        sys.exit("bench.py: no HIP device present; the HIP backend has no CPU path")
    dev = hb.HipDevice(0)
    props = dev.props
    log(f"[bench] device: {props['name']} {props['arch']} CUs={props['compute_units']} "
        f"clock={props['clock_khz'] / 1e6:.2f} GHz LDS/CU={props['local_memory_size']}")
    options = args.options or None
    # what the measured schedule search filed for gfx950 (programs and single launches, by key) applies
    # unless the caller names another file; explicit --options still go on top
    tuned_file = os.environ.get("ECLAT_HIP_TUNE", "")
    shipped = os.path.join(os.path.dirname(os.path.abspath(hb.__file__)), "tuned_gfx950.txt")
    if not tuned_file and os.path.exists(shipped) and not args.no_tuned:
        os.environ["ECLAT_HIP_TUNE"] = tuned_file = shipped
    want = lambda n: not args.only or args.only == n
    extra = {}

    def roofline(bound, achieved, unit, algo, launch=None):
        """Roofline object of one kernel (`launch` given) or of a whole step: `achieved` is
        algorithmic work over measured time."""
        peak = HBM_PEAK_GBS if bound == "hbm" else FP32_MFMA_PEAK_TFLOPS
        r = {"bound": bound, "achieved": round(achieved, 2), "peak": peak, "unit": unit,
             "frac": round(achieved / peak, 4), "traffic": None,
             "algorithmic_bytes" if bound == "hbm" else "algorithmic_flops": algo}
        if launch is not None:
            traffic, stale = (None, False) if args.options else measure.measured_traffic(launch["entry"], launch["source"])
            r["traffic"] = traffic
            if stale:
                r["traffic_stale"] = True    # the kernel's source changed since the counters were read
            r["traffic_source"] = ("profiles/traffic.json: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE per dispatch, scaled by "
                                   "the same counters on this backend's plain copy kernel of known size (assumed free "
                                   "of wasted traffic); counted only for the kernel source hash it was read on")
            r["kernel"], r["schedule"] = launch["entry"], launch["schedule"]
        return r

    def unfused(prog_ast, arg_names, consts, arrays, steps, warmup, check=None):
        """The per-kernel path: every lowered kernel compiled and launched on its own,
        synchronously, every intermediate buffer in memory (src/backend/executor.rs:245-372)."""
        if args.no_per_kernel:
            return None
        path = measure.PerKernelPath(dev, prog_ast, options)
        inputs = measure.upload_inputs(dev, prog_ast, arg_names, consts, arrays)
        ms = path.time(inputs, steps, warmup)
        queued = path.time(inputs, steps, warmup, sync=False)
        if check is not None and not args.no_check:
            check(path.step(inputs))
            check(path.step(inputs, sync=False))
        dev.trim()
        return {"ms_per_step": round(ms, 4), "ms_per_step_queued": round(queued, 4), "steps": steps, "launches": len(path.launches),
                "lowered_kernels": len(path.kernels),
                "algorithmic_bytes": sum(l["algo_bytes"] for l in path.launches),
                "timing": "host wall clock; ms_per_step: every launch waits for completion, as the reference's own "
                          "Kernel::execute does; ms_per_step_queued: launches only queued, one wait at the end (the "
                          "binding's default: every buffer read is ordered behind them on the device's stream)"}

    # ---- config 2: row softmax 4096 x 4096 (headline) --------------------------------
    softmax = None
    if want("softmax"):
        arrays = wl.config2_inputs()
        prog_ast, arg_names, out_name, consts, _ = wl.lower_with_table([(4096, 4096)], wl.config2_graph)
        prog = hb.HipProgram(dev, prog_ast, options)
        sets = measure.make_sets(dev, prog, arg_names, consts, arrays, args.sets)
        ms, wall_ms = measure.time_steps(dev, prog, sets, args.steps, args.warmup)
        algo = sum(l["algo_bytes"] for l in prog.launches)
        softmax = {"ms": ms, "gbs": algo / (ms * 1e-3) / 1e9, "algo_bytes": algo, "launch": prog.launches[0],
                   "n_launches": len(prog.launches)}
        softmax["each"] = measure.time_each_step(dev, prog, sets, max(20, min(args.steps, 200)), max(5, min(args.warmup, 20)))
        log(f"[bench] softmax 4096^2: {ms * 1e3:.1f} us/step -> {softmax['gbs']:.0f} GB/s "
            f"({softmax['gbs'] / HBM_PEAK_GBS:.1%} of 8 TB/s); {[(l['entry'], l['schedule']) for l in prog.launches]}")

        def check_softmax(got):
            x = arrays[0].astype(np.float64)
            e = np.exp(x[:64] - x[:64].max(1, keepdims=True))
            assert np.allclose(got[:64], e / e.sum(1, keepdims=True), rtol=1e-5, atol=1e-12), "softmax result check failed"
            assert np.allclose(got.sum(1), 1.0, atol=1e-5), "softmax rows do not sum to 1"
        if not args.no_check:
            check_softmax(sets[0][1][out_name].read_array(np.float32, (4096, 4096)))
        del sets
        softmax["per_kernel"] = unfused(prog_ast, arg_names, consts, arrays, max(5, min(args.steps, 50)), 3,
                                        lambda named: check_softmax(named[out_name].read_array(np.float32, (4096, 4096))))
        if softmax["per_kernel"]:
            log(f"[bench] softmax, per-kernel path: {softmax['per_kernel']['ms_per_step'] * 1e3:.1f} us/step, "
                f"{softmax['per_kernel']['launches']} launches")

    # ---- config 3: 4096^3 fp32 matmul --------------------------------------------------
    matmul = None
    if want("matmul"):
        arrays = wl.config3_inputs()
        prog_ast, arg_names, out_name, consts, _ = wl.lower_with_table([(4096, 4096)] * 2, wl.config3_graph)
        prog = hb.HipProgram(dev, prog_ast, options)
        sets = measure.make_sets(dev, prog, arg_names, consts, arrays, 2)
        k = max(50, min(args.steps, 100))
        wu = max(10, args.warmup)
        ms, _ = measure.time_steps(dev, prog, sets, k, wu)
        flops = sum(l["flops"] for l in prog.launches)
        matmul = {"ms": ms, "tflops": flops / (ms * 1e-3) / 1e12, "steps": k, "warmup": wu, "flops": flops, "launch": prog.launches[0]}
        matmul["each"] = measure.time_each_step(dev, prog, sets, k, wu)
        log(f"[bench] matmul 4096^3: {ms:.3f} ms/step over {k} launches -> {matmul['tflops']:.1f} TFLOP/s "
            f"({matmul['tflops'] / FP32_MFMA_PEAK_TFLOPS:.1%} of FP32 MFMA peak); per launch median "
            f"{matmul['each'][0]:.3f} min {matmul['each'][1]:.3f} mean {matmul['each'][2]:.3f} ms; "
            f"{[(l['entry'], l['schedule']) for l in prog.launches]}")
        if not args.no_check:
            got = sets[0][1][out_name].read_array(np.float32, (4096, 4096))
            a, b = arrays
            ref = a[:32].astype(np.float64) @ b.astype(np.float64)
            scale = np.abs(a[:32]).astype(np.float64) @ np.abs(b).astype(np.float64)
            assert np.all(np.abs(got[:32] - ref) <= 1e-3 * scale), "matmul result check failed"
        del sets

    # ---- config 1: fused elementwise + reduce, 1024 x 1024 ------------------------------
    cfg1 = None
    if want("config1"):
        arrays = wl.config1_inputs()
        prog_ast, arg_names, out_name, consts, _ = wl.lower_with_table([(1024, 1024)] * 3, wl.config1_graph)
        prog = hb.HipProgram(dev, prog_ast, options)
        sets = measure.make_sets(dev, prog, arg_names, consts, arrays, max(args.sets, 24))
        ms, wall_ms = measure.time_steps(dev, prog, sets, args.steps, args.warmup)
        algo = sum(l["algo_bytes"] for l in prog.launches)
        cfg1 = {"us": ms * 1e3, "wall_us": wall_ms * 1e3, "gbs": algo / (ms * 1e-3) / 1e9, "algo_bytes": algo,
                "launch": prog.launches[0], "floor_us": measure.launch_floor_us(dev, prog.launches[0]["grid"][0])}
        log(f"[bench] config1 relu-sum 1024^2: {cfg1['us']:.2f} us/step -> {cfg1['gbs']:.0f} GB/s")

        def check_cfg1(got):
            a, b, c = [x.astype(np.float64) for x in arrays]
            assert np.allclose(got.ravel(), np.maximum(a * b + c, 0).sum(1), rtol=1e-5, atol=1e-4), "config1 check failed"
        if not args.no_check:
            check_cfg1(sets[0][1][out_name].read_array(np.float32, (1024,)))
        del sets
        cfg1["per_kernel"] = unfused(prog_ast, arg_names, consts, arrays, max(5, min(args.steps, 100)), 5,
                                     lambda named: check_cfg1(named[out_name].read_array(np.float32, (1024,))))

    # ---- config 4: MLP 1024-4096-4096-1024, batch 8192, forward + backward + SGD ---------
    mlp = None
    if want("mlp"):
        batch, dims = wl.mlp_sizes(True)
        arrays = wl.config4_inputs(batch, dims)
        from harp_amd.frontend import Tensor
        ts = [Tensor.input(list(a.shape)) for a in arrays]
        roots = wl.config4_graph(*ts)
        prog_ast, arg_names, outs, consts, plain = wl.lower_multi(ts, roots)
        prog = hb.HipProgram(dev, prog_ast, options)
        sets = measure.make_sets(dev, prog, arg_names, consts, arrays, 1)
        k = max(3, min(args.steps, 20))
        ms, wall_ms = measure.time_steps(dev, prog, sets, k, min(args.warmup, 3))
        flops = sum(l["flops"] for l in prog.launches)
        algo = sum(l["algo_bytes"] for l in prog.launches)
        mlp = {"ms": ms, "steps": k, "flops": flops, "algo_bytes": algo,
               "lowered_kernels": len(plain.args), "launches": len(prog.launches),
               "gemm_launches": sum(l["schedule"].count("mfma") for l in prog.launches)}
        log(f"[bench] mlp step (batch {batch}, {dims}): {ms:.2f} ms/step -> {flops / ms / 1e9:.1f} TFLOP/s, "
            f"{batch / ms * 1e3:.0f} samples/s; {mlp['lowered_kernels']} kernels -> {mlp['launches']} launches")

        mlp_want = []

        def check_mlp(named):
            # loss and every updated parameter against the float64 statement of the step
            from harp_amd.checks import mlp_step
            if not mlp_want:
                mlp_want.extend(mlp_step(arrays)[:2])
            loss, grads = mlp_want
            got_loss = float(named[outs[-1]].read_array(np.float32, (1,))[0])
            assert abs(got_loss - loss) <= 1e-5 * abs(loss), f"mlp loss check failed: {got_loss} vs {loss}"
            for name, p, g in zip(outs[:-1], arrays[2:], grads):
                got = named[name].read_array(np.float32, p.shape)
                assert np.allclose(got, p - 1e-3 * g, rtol=1e-5, atol=1e-7), f"mlp update of {p.shape} check failed"
            return got_loss
        if not args.no_check:
            mlp["loss"] = check_mlp(sets[0][1])
        del sets
        dev.trim()
        mlp["per_kernel"] = unfused(prog_ast, arg_names, consts, arrays, 3, 1, check_mlp)
        if mlp["per_kernel"]:
            log(f"[bench] mlp step, per-kernel path: {mlp['per_kernel']['ms_per_step']:.2f} ms/step, "
                f"{mlp['per_kernel']['launches']} launches")

    # ---- config 5: MNIST-shaped CNN, batch 256, forward + backward + SGD update ------------
    cnn = None
    if want("cnn"):
        sizes = wl.cnn_sizes(True)
        arrays = wl.config5_inputs(*sizes)
        from harp_amd.frontend import Tensor
        ts = [Tensor.input(list(a.shape)) for a in arrays]
        roots = wl.config5_graph(*ts, lr=1e-2)
        prog_ast, arg_names, outs, consts, plain = wl.lower_multi(ts, roots)
        prog = hb.HipProgram(dev, prog_ast, options)
        sets = measure.make_sets(dev, prog, arg_names, consts, arrays, 1)
        k = max(3, min(args.steps, 50))
        ms, wall_ms = measure.time_steps(dev, prog, sets, k, min(args.warmup, 5))
        cnn = {"ms": ms, "steps": k, "flops": sum(l["flops"] for l in prog.launches),
               "algo_bytes": sum(l["algo_bytes"] for l in prog.launches),
               "lowered_kernels": len(plain.args), "launches": len(prog.launches),
               "gemm_launches": sum(l["schedule"].count("mfma") for l in prog.launches)}
        gms, gwall = measure.time_replays(dev, prog, sets, k, min(args.warmup, 5))
        cnn["graph_ms"], cnn["graph_wall_ms"], cnn["wall_ms"] = gms, gwall, wall_ms
        log(f"[bench] cnn step replayed as one HIP graph: {gms:.3f} ms/step (host wall {gwall:.3f} ms; "
            f"eager host wall {wall_ms:.3f} ms)")
        log(f"[bench] cnn step (batch {sizes[0]}): {ms:.3f} ms/step -> {sizes[0] / ms * 1e3:.0f} images/s; "
            f"{cnn['lowered_kernels']} kernels -> {cnn['launches']} launches, {cnn['gemm_launches']} MFMA contractions")

        cnn_want = []

        def check_cnn(named):
            # loss and every updated parameter against the float64 statement of the step
            from harp_amd.checks import cnn_step
            if not cnn_want:
                cnn_want.extend(cnn_step(arrays[0], arrays[1], arrays[2:]))
            loss, grads = cnn_want
            got_loss = float(named[outs[-1]].read_array(np.float32, (1,))[0])
            assert abs(got_loss - loss) <= 1e-5 * abs(loss), f"cnn loss check failed: {got_loss} vs {loss}"
            for name, p, g in zip(outs[:-1], arrays[2:], grads):
                got = named[name].read_array(np.float32, p.shape)
                assert np.allclose(got, p - 1e-2 * g, rtol=1e-4, atol=1e-6), f"cnn update of {p.shape} check failed"
            return got_loss
        if not args.no_check:
            cnn["loss"] = check_cnn(sets[0][1])
        del sets
        cnn["per_kernel"] = unfused(prog_ast, arg_names, consts, arrays, 5, 2, check_cnn)
        if cnn["per_kernel"]:
            log(f"[bench] cnn step, per-kernel path: {cnn['per_kernel']['ms_per_step']:.3f} ms/step, "
                f"{cnn['per_kernel']['launches']} launches")

    # ---- CPU baseline: the oracle's unfused C kernels on host cores -------------------------
    cpu = None
    if not args.no_cpu_baseline and softmax is not None:
        from oracle import baseline
        arrays = wl.config2_inputs()
        sec, reps, _ = baseline.time_graph(wl.config2_graph, arrays, min_seconds=8.0, max_reps=40)
        cpu = {"value": softmax["algo_bytes"] / sec / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
               "sample": f"full 4096x4096 softmax, unfused R,E,E,R,E kernels (gcc -O3 -ffast-math), "
                         f"median of {reps} passes, {sec * 1e3:.0f} ms/pass"}
        log(f"[bench] cpu baseline softmax: {sec * 1e3:.0f} ms/pass -> {cpu['value']:.2f} GB/s (1 core)")
        # the OpenMP variant of the same kernels on the cores this process may use
        cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
        cores = max(1, min(cores, int(os.environ.get("OMP_NUM_THREADS", cores))))
        os.environ["OMP_NUM_THREADS"] = str(cores)
        sec_o, reps_o, _ = baseline.time_graph(wl.config2_graph, arrays, min_seconds=4.0, max_reps=40, openmp=True)
        extra["cpu_baseline_openmp"] = {
            "value": softmax["algo_bytes"] / sec_o / 1e9, "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": f"full 4096x4096 softmax, the same five kernels with '#pragma omp parallel for' on the "
                      f"outer loop (gcc -O3 -ffast-math -fopenmp), median of {reps_o} passes, {sec_o * 1e3:.1f} ms/pass"}
        log(f"[bench] cpu baseline softmax, OpenMP: {sec_o * 1e3:.1f} ms/pass -> "
            f"{extra['cpu_baseline_openmp']['value']:.1f} GB/s ({cores} cores)")
        if matmul is not None:
            a, b = wl.config3_inputs()
            sub = 8
            sec_m, reps_m, _ = baseline.time_graph(wl.config3_graph, [a[:sub].copy(), b],
                                                   min_seconds=4.0, max_reps=10)
            gflops = 2.0 * sub * 4096 * 4096 / sec_m / 1e9
            extra["cpu_baseline_matmul"] = {
                "value": gflops / 1e3, "unit": "TFLOP/s", "cores": 1, "kind": "port",
                "sample": f"{sub} of 4096 rows of A through the reference's ijk kernel "
                          f"(gcc -O3 -ffast-math), median of {reps_m} passes, {sec_m * 1e3:.0f} ms/pass"}
            log(f"[bench] cpu baseline matmul: {gflops:.2f} GFLOP/s (1 core, {sub}-row sample)")

        if mlp is not None:
            from harp_amd.frontend import exact_mode
            sub = 4
            arrays = wl.config4_inputs(sub, wl.mlp_sizes(True)[1])
            with exact_mode():
                sec_p, reps_p, _ = baseline.time_graph(lambda *ts: wl.config4_graph(*ts), arrays,
                                                       min_seconds=4.0, max_reps=3)
            extra["cpu_baseline_mlp"] = {
                "value": sub / sec_p, "unit": "samples/s", "cores": 1, "kind": "port",
                "sample": f"batch {sub} of 8192 through the same lowered kernels, unfused "
                          f"(gcc -O3 -ffast-math), median of {reps_p} passes, {sec_p * 1e3:.0f} ms/pass"}
            log(f"[bench] cpu baseline mlp: {sub / sec_p:.2f} samples/s (1 core, batch {sub})")

        if cnn is not None:
            from harp_amd.frontend import exact_mode
            sub = 64
            sizes = wl.cnn_sizes(True)
            arrays = wl.config5_inputs(sub, *sizes[1:])
            with exact_mode():
                sec_c, reps_c, _ = baseline.time_graph(lambda *ts: wl.config5_graph(*ts, lr=1e-2), arrays,
                                                       min_seconds=4.0, max_reps=10)
            extra["cpu_baseline_cnn"] = {
                "value": sub / sec_c, "unit": "images/s", "cores": 1, "kind": "port",
                "sample": f"batch {sub} of 256 through the same lowered kernels, unfused "
                          f"(gcc -O3 -ffast-math), median of {reps_c} passes, {sec_c * 1e3:.0f} ms/pass"}
            log(f"[bench] cpu baseline cnn: {sub / sec_c:.1f} images/s (1 core, batch {sub})")

    head = softmax
    out = {
        "metric": "fused-kernel HBM GB/s (softmax 4096²)" + (" + fp32 matmul TFLOP/s (4096³)" if matmul else ""),
        "value": round(head["gbs"], 1) if head else None,
        "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(head["ms"], 6) if head else None,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic (seeded N(0, std 2) fp32 [4096,4096])",
        "config": {"workload": "config2: row softmax fp32 [4096,4096], one fused launch",
                   "buffer_sets": args.sets, "options": args.options,
                   "tuned_options_file": os.path.relpath(tuned_file, os.path.dirname(os.path.abspath(__file__))) if tuned_file else None},
    }
    each_note = ("one HIP event pair per launch on the launch stream, same buffer rotation; the events sit between "
                 "launches, so ms_mean can exceed ms_per_step, which is measured over launches queued back to back")
    if head:
        out["ms_median"], out["ms_min"], out["ms_mean"] = (round(v, 6) for v in head["each"])
        out["per_launch_timing"] = each_note
        out["roofline"] = roofline("hbm", head["gbs"], "GB/s", head["algo_bytes"], head["launch"])
        if head["per_kernel"]:
            extra["per_kernel_path"] = {"config2_softmax_4096": head["per_kernel"]}
    if cpu:
        out["cpu_baseline"] = cpu
    if matmul:
        extra["matmul_4096"] = {
            "value": round(matmul["tflops"], 2), "unit": "TFLOP/s", "ms_per_step": round(matmul["ms"], 4),
            "steps": matmul["steps"], "warmup": matmul["warmup"], "dtype": "f32",
            "ms_median": round(matmul["each"][0], 4), "ms_min": round(matmul["each"][1], 4), "ms_mean": round(matmul["each"][2], 4),
            "tflops_at_median": round(matmul["flops"] / (matmul["each"][0] * 1e-3) / 1e12, 2),
            "per_launch_timing": each_note,
            "roofline": roofline("mfma", matmul["tflops"], "TFLOP/s", matmul["flops"], matmul["launch"]),
            "per_kernel_path": "the same single kernel on both paths"}
    if cfg1:
        extra["config1_relu_sum_1024"] = {
            "us_per_step": round(cfg1["us"], 2), "host_us_per_step": round(cfg1["wall_us"], 2),
            "value": round(cfg1["gbs"], 1), "unit": "GB/s", "schedule": cfg1["launch"]["schedule"],
            "roofline": roofline("hbm", cfg1["gbs"], "GB/s", cfg1["algo_bytes"], cfg1["launch"]),
            "empty_kernel_us_per_launch": round(cfg1["floor_us"], 2),
            "us_above_empty_kernel": round(cfg1["us"] - cfg1["floor_us"], 2),
            "note": "12.6 MB per launch is 1.6 us at peak; empty_kernel_us_per_launch is the same grid of a kernel that "
                    "does nothing, queued back to back the same way: the part of the step that is launch and drain"}
        if cfg1["per_kernel"]:
            extra.setdefault("per_kernel_path", {})["config1_relu_sum_1024"] = cfg1["per_kernel"]
    if mlp:
        tflops = mlp["flops"] / mlp["ms"] / 1e9
        extra["config4_mlp_step"] = {
            "value": round(8192 / mlp["ms"] * 1e3, 1), "unit": "samples/s", "ms_per_step": round(mlp["ms"], 3),
            "steps": mlp["steps"], "tflops": round(tflops, 2),
            "algorithmic_bytes": mlp["algo_bytes"], "lowered_kernels": mlp["lowered_kernels"],
            "launches": mlp["launches"], "gemm_launches": mlp["gemm_launches"], "loss": mlp.get("loss"),
            "roofline": roofline("mfma", tflops, "TFLOP/s", mlp["flops"]),
            "workload": "MLP 1024-4096-4096-1024, batch 8192: forward, MSE, exact backward, SGD update, one Program"}
        if mlp["per_kernel"]:
            extra.setdefault("per_kernel_path", {})["config4_mlp_step"] = mlp["per_kernel"]
    if cnn:
        # the step's roofline: whichever of its algorithmic bytes at HBM peak and its flops at MFMA
        # peak takes longer
        t_hbm = cnn["algo_bytes"] / (HBM_PEAK_GBS * 1e9)
        t_mfma = cnn["flops"] / (FP32_MFMA_PEAK_TFLOPS * 1e12)
        if t_hbm >= t_mfma:
            roof = roofline("hbm", cnn["algo_bytes"] / (cnn["ms"] * 1e-3) / 1e9, "GB/s", cnn["algo_bytes"])
        else:
            roof = roofline("mfma", cnn["flops"] / cnn["ms"] / 1e9, "TFLOP/s", cnn["flops"])
        extra["config5_cnn_step"] = {
            "value": round(256 / cnn["ms"] * 1e3, 1), "unit": "images/s", "ms_per_step": round(cnn["ms"], 4),
            "steps": cnn["steps"], "algorithmic_bytes": cnn["algo_bytes"], "algorithmic_flops": cnn["flops"],
            "lowered_kernels": cnn["lowered_kernels"], "launches": cnn["launches"],
            "gemm_launches": cnn["gemm_launches"], "loss": cnn.get("loss"), "roofline": roof,
            "ms_per_step_hip_graph": round(cnn["graph_ms"], 4),
            "host_ms_per_step": {"eager": round(cnn["wall_ms"], 4), "hip_graph": round(cnn["graph_wall_ms"], 4)},
            "workload": "CNN 1x28x28: conv3x3(32)+relu+pool, conv3x3(64)+relu+pool, fc 3136-128-10, "
                        "cross-entropy; batch 256 forward + exact backward, plus the SGD update (more than the "
                        "configuration asks for, inside the timed region), one Program"}
        if cnn["per_kernel"]:
            extra.setdefault("per_kernel_path", {})["config5_cnn_step"] = cnn["per_kernel"]
    extra["device"] = {"name": props["name"] or "MI355X (name not reported by the runtime)", "arch": props["arch"],
                       "compute_units": props["compute_units"], "clock_khz": props["clock_khz"]}
    out["extra"] = extra
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
