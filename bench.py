#!/usr/bin/env python3
"""Benchmark of the eclat kernel path on one MI355X.

A step is one pass of the hot path (execute the compiled Program) over one batch
of synthetic input.  The headline workload is benchmark configuration 2 -- row softmax of
fp32 [4096, 4096], compiled from the reference's five-kernel lowering into one
fused launch -- reported as HBM GB/s of algorithmic traffic (one read + one
write).  The same JSON line carries config 3 (4096^3 fp32 matmul, TFLOP/s on the
FP32 MFMA schedule) and config 1 under "extra", a roofline object per dominant
kernel, and the CPU baseline (the oracle's C kernels, unfused, on host cores).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--options key=value,...]
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E bandwidth
FP32_MFMA_PEAK_TFLOPS = 157.3  # MI355X published dense FP32 matrix peak


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def measured_traffic(kernel):
    """HBM bytes per launch from the committed counter summary (rocprofv3 --pmc FETCH_SIZE /
    WRITE_SIZE, scaled by a copy kernel of known size); None when the kernel is not in it."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            return json.load(f)["kernels"][kernel]["traffic_bytes"]
    except (OSError, KeyError, ValueError):
        return None


def build(dev, hb, wl, name, shapes, options):
    inputs_fn, graph_fn = wl.CONFIGS[name]
    prog_ast, arg_names, out_name, const_inputs, _ = wl.lower_with_table(shapes, graph_fn)
    prog = hb.HipProgram(dev, prog_ast, options)
    return prog, arg_names, out_name, const_inputs


def make_sets(dev, hb, prog, arg_names, const_inputs, arrays, nsets):
    from harp_amd import measure
    return measure.make_sets(dev, prog, arg_names, const_inputs, arrays, nsets)


def time_steps(dev, hb, prog, sets, steps, warmup):
    from harp_amd import measure
    return measure.time_steps(dev, prog, sets, steps, warmup)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--options", default="")
    ap.add_argument("--sets", type=int, default=4)
    ap.add_argument("--only", default="", help="softmax | matmul | config1 | mlp | cnn | copy | mfma_peak (default: all but copy)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-check", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this path runs on one GPU (every kernel here works on one GPU's "
                 "share at its real shape); run with --gpus 1")
    if args.steps < 1 or args.warmup < 0:
        sys.exit("bench.py: --steps must be >= 1 and --warmup >= 0")

    from harp_amd import backend as hb
    from harp_amd import workloads as wl
    if hb.device_count() == 0:
        sys.exit("bench.py: no HIP device present; the HIP backend has no CPU path")
    dev = hb.HipDevice(0)
    props = dev.props
    log(f"[bench] device: {props['name']} {props['arch']} CUs={props['compute_units']} "
        f"clock={props['clock_khz'] / 1e6:.2f} GHz LDS/CU={props['local_memory_size']}")
    options = args.options or None
    want = lambda n: not args.only or args.only == n
    result_extra = {}

    # ---- config 2: row softmax 4096 x 4096 (headline) --------------------------------
    softmax = None
    if want("softmax"):
        shapes = [(4096, 4096)]
        arrays = wl.config2_inputs()
        prog, arg_names, out_name, consts = build(dev, hb, wl, "config2_softmax", shapes, options)
        sets = make_sets(dev, hb, prog, arg_names, consts, arrays, args.sets)
        ms, wall_ms = time_steps(dev, hb, prog, sets, args.steps, args.warmup)
        algo = sum(l["algo_bytes"] for l in prog.launches)
        softmax = {"ms": ms, "wall_ms": wall_ms, "gbs": algo / (ms * 1e-3) / 1e9, "algo_bytes": algo,
                   "launches": [(l["entry"], l["schedule"]) for l in prog.launches]}
        log(f"[bench] softmax 4096^2: {ms * 1e3:.1f} us/step -> {softmax['gbs']:.0f} GB/s "
            f"({softmax['gbs'] / HBM_PEAK_GBS:.1%} of 8 TB/s); {softmax['launches']}")
        if not args.no_check:
            got = sets[0][1][out_name].read_array(np.float32, (4096, 4096))
            x = arrays[0].astype(np.float64)
            e = np.exp(x[:64] - x[:64].max(1, keepdims=True))
            assert np.allclose(got[:64], e / e.sum(1, keepdims=True), rtol=1e-5, atol=1e-12), \
                "softmax result check failed"
            assert np.allclose(got.sum(1), 1.0, atol=1e-5), "softmax rows do not sum to 1"
        del sets

    # ---- calibration: plain copy of the same size (for counter scaling, not a result) ------
    if args.only == "copy":
        wl.CONFIGS["copy"] = (wl.config2_inputs, lambda x: x.contiguous())
        arrays = wl.config2_inputs()
        prog, arg_names, out_name, consts = build(dev, hb, wl, "copy", [(4096, 4096)], options)
        sets = make_sets(dev, hb, prog, arg_names, consts, arrays, args.sets)
        ms, _ = time_steps(dev, hb, prog, sets, args.steps, args.warmup)
        log(f"[bench] copy 4096^2 ({prog.launches[0]['entry']}, {prog.launches[0]['schedule']}): "
            f"{ms * 1e3:.1f} us/step -> {2 * 4096 * 4096 * 4 / (ms * 1e-3) / 1e9:.0f} GB/s")
        return

    # ---- calibration: MFMA issue rate with operands in registers (not a result) -------------
    if args.only == "mfma_peak":
        iters, waves_per_cu = 4096, 8
        src = """
typedef float f16v __attribute__((ext_vector_type(16)));
extern "C" __global__ void __launch_bounds__(256) eh_mfma_peak(float* out) {
  f16v acc[4];
  for (int i = 0; i < 4; ++i) for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;
  float a = threadIdx.x * 1e-3f, b = blockIdx.x * 1e-3f;
  for (int it = 0; it < %d; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[i], 0, 0, 0);
  }
  float s = 0.0f;
  for (int i = 0; i < 4; ++i) for (int r = 0; r < 16; ++r) s += acc[i][r];
  out[blockIdx.x * 256 + threadIdx.x] = s;
}
""" % iters
        blocks = props["compute_units"] * waves_per_cu // 4
        mod = hb.HipModule(dev, hb.compile_source(src), "eh_mfma_peak")
        out = hb.HipBuffer(dev, [blocks * 256 * 4], None, nbytes=blocks * 256 * 4)
        for _ in range(3):
            mod.launch([blocks, 1, 1], [256, 1, 1], [out], sync=False)
        dev.sync()
        e0, e1 = hb.Event(dev), hb.Event(dev)
        e0.record()
        reps = 20
        for _ in range(reps):
            mod.launch([blocks, 1, 1], [256, 1, 1], [out], sync=False)
        e1.record()
        e1.sync()
        ms = e0.elapsed_ms(e1) / reps
        flops = blocks * 4 * iters * 4 * (32 * 32 * 2 * 2)
        log(f"[bench] MFMA f32 32x32x2 issue-rate ceiling: {flops / ms / 1e9:.1f} TFLOP/s "
            f"({flops / ms / 1e9 / FP32_MFMA_PEAK_TFLOPS:.1%} of the published {FP32_MFMA_PEAK_TFLOPS}); "
            f"{blocks} workgroups x 4 waves, {ms * 1e3:.0f} us/launch")
        return

    # ---- config 3: 4096^3 fp32 matmul --------------------------------------------------
    matmul = None
    if want("matmul"):
        shapes = [(4096, 4096), (4096, 4096)]
        arrays = wl.config3_inputs()
        prog, arg_names, out_name, consts = build(dev, hb, wl, "config3_matmul", shapes, options)
        sets = make_sets(dev, hb, prog, arg_names, consts, arrays, 2)
        k = max(5, min(args.steps, 50))
        ms, wall_ms = time_steps(dev, hb, prog, sets, k, min(args.warmup, 5))
        flops = sum(l["flops"] for l in prog.launches)
        matmul = {"ms": ms, "tflops": flops / (ms * 1e-3) / 1e12, "steps": k,
                  "launches": [(l["entry"], l["schedule"]) for l in prog.launches]}
        log(f"[bench] matmul 4096^3: {ms:.3f} ms/step -> {matmul['tflops']:.1f} TFLOP/s "
            f"({matmul['tflops'] / FP32_MFMA_PEAK_TFLOPS:.1%} of FP32 MFMA peak); {matmul['launches']}")
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
        shapes = [(1024, 1024)] * 3
        arrays = wl.config1_inputs()
        prog, arg_names, out_name, consts = build(dev, hb, wl, "config1_relu_sum", shapes, options)
        sets = make_sets(dev, hb, prog, arg_names, consts, arrays, args.sets)
        ms, _ = time_steps(dev, hb, prog, sets, args.steps, args.warmup)
        algo = sum(l["algo_bytes"] for l in prog.launches)
        cfg1 = {"us": ms * 1e3, "gbs": algo / (ms * 1e-3) / 1e9, "algo_bytes": algo,
                "launches": [(l["entry"], l["schedule"]) for l in prog.launches]}
        log(f"[bench] config1 relu-sum 1024^2: {cfg1['us']:.1f} us/step -> {cfg1['gbs']:.0f} GB/s")
        del sets

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
        sets = make_sets(dev, hb, prog, arg_names, consts, arrays, 1)
        k = max(3, min(args.steps, 20))
        ms, wall_ms = time_steps(dev, hb, prog, sets, k, min(args.warmup, 3))
        flops = sum(l["flops"] for l in prog.launches)
        algo = sum(l["algo_bytes"] for l in prog.launches)
        mlp = {"ms": ms, "steps": k, "flops": flops, "algo_bytes": algo,
               "lowered_kernels": len(plain.args), "launches": len(prog.launches),
               "gemm_launches": sum(1 for l in prog.launches if l["schedule"].startswith("mfma"))}
        log(f"[bench] mlp step (batch {batch}, {dims}): {ms:.2f} ms/step -> {flops / ms / 1e9:.1f} TFLOP/s, "
            f"{batch / ms * 1e3:.0f} samples/s; {mlp['lowered_kernels']} kernels -> {mlp['launches']} launches")
        if not args.no_check:
            named = sets[0][1]
            x, t, params = arrays[0], arrays[1], arrays[2:]
            h = x
            for i in range(len(params) // 2):
                h = h @ params[2 * i].T + params[2 * i + 1]
                if i + 1 < len(params) // 2:
                    h = np.tanh(h)
            d = h.astype(np.float64) - t
            loss = float((d * d).mean())
            got_loss = float(named[outs[-1]].read_array(np.float32, (1,))[0])
            assert abs(got_loss - loss) <= 1e-3 * abs(loss), f"mlp loss check failed: {got_loss} vs {loss}"
            nb = params[-1].astype(np.float64) - 1e-3 * (2.0 * d / d.size).sum(0)
            got_b = named[outs[-2]].read_array(np.float32, (dims[-1],))
            assert np.allclose(got_b, nb, rtol=1e-4, atol=1e-7), "mlp bias update check failed"
            mlp["loss"] = got_loss
        del sets

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
        sets = make_sets(dev, hb, prog, arg_names, consts, arrays, 1)
        k = max(3, min(args.steps, 50))
        ms, wall_ms = time_steps(dev, hb, prog, sets, k, min(args.warmup, 5))
        cnn = {"ms": ms, "steps": k, "flops": sum(l["flops"] for l in prog.launches),
               "algo_bytes": sum(l["algo_bytes"] for l in prog.launches),
               "lowered_kernels": len(plain.args), "launches": len(prog.launches),
               "gemm_launches": sum(1 for l in prog.launches if l["schedule"].startswith("mfma"))}
        from harp_amd import measure
        gms, gwall = measure.time_replays(dev, prog, sets, k, min(args.warmup, 5))
        cnn["graph_ms"], cnn["graph_wall_ms"], cnn["wall_ms"] = gms, gwall, wall_ms
        log(f"[bench] cnn step replayed as one HIP graph: {gms:.3f} ms/step (host wall {gwall:.3f} ms; "
            f"eager host wall {wall_ms:.3f} ms)")
        log(f"[bench] cnn step (batch {sizes[0]}): {ms:.3f} ms/step -> {sizes[0] / ms * 1e3:.0f} images/s; "
            f"{cnn['lowered_kernels']} kernels -> {cnn['launches']} launches ({cnn['gemm_launches']} MFMA)")
        if not args.no_check:
            named = sets[0][1]
            got_loss = float(named[outs[-1]].read_array(np.float32, (1,))[0])
            assert np.isfinite(got_loss) and abs(got_loss - np.log(10.0)) < 0.5, f"cnn loss {got_loss}"
            cnn["loss"] = got_loss
        del sets

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
        result_extra["cpu_baseline_openmp"] = {
            "value": softmax["algo_bytes"] / sec_o / 1e9, "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": f"full 4096x4096 softmax, the same five kernels with '#pragma omp parallel for' on the "
                      f"outer loop (gcc -O3 -ffast-math -fopenmp), median of {reps_o} passes, {sec_o * 1e3:.1f} ms/pass"}
        log(f"[bench] cpu baseline softmax, OpenMP: {sec_o * 1e3:.1f} ms/pass -> "
            f"{result_extra['cpu_baseline_openmp']['value']:.1f} GB/s ({cores} cores)")
        if matmul is not None:
            a, b = wl.config3_inputs()
            sub = 8
            sec_m, reps_m, _ = baseline.time_graph(wl.config3_graph, [a[:sub].copy(), b],
                                                   min_seconds=4.0, max_reps=10)
            gflops = 2.0 * sub * 4096 * 4096 / sec_m / 1e9
            result_extra["cpu_baseline_matmul"] = {
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
            result_extra["cpu_baseline_mlp"] = {
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
            result_extra["cpu_baseline_cnn"] = {
                "value": sub / sec_c, "unit": "images/s", "cores": 1, "kind": "port",
                "sample": f"batch {sub} of 256 through the same lowered kernels, unfused "
                          f"(gcc -O3 -ffast-math), median of {reps_c} passes, {sec_c * 1e3:.0f} ms/pass"}
            log(f"[bench] cpu baseline cnn: {sub / sec_c:.1f} images/s (1 core, batch {sub})")

    head = softmax
    out = {
        "metric": "fused-kernel HBM GB/s (softmax 4096\u00b2)" + (" + fp32 matmul TFLOP/s (4096\u00b3)" if matmul else ""),
        "value": round(head["gbs"], 1) if head else None,
        "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(head["ms"], 6) if head else None,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic (seeded N(0, std 2) fp32 [4096,4096])",
        "config": {"workload": "config2: row softmax fp32 [4096,4096], one fused launch",
                   "buffer_sets": args.sets, "options": args.options},
    }
    if head:
        out["roofline"] = {"bound": "hbm", "achieved": round(head["gbs"], 1), "peak": HBM_PEAK_GBS,
                           "unit": "GB/s", "frac": round(head["gbs"] / HBM_PEAK_GBS, 4),
                           "traffic": measured_traffic(head["launches"][0][0]) if not args.options else None,
                           "algorithmic_bytes": head["algo_bytes"],
                           "kernel": head["launches"][0][0], "schedule": head["launches"][0][1]}
    if cpu:
        out["cpu_baseline"] = cpu
    if matmul:
        result_extra["matmul_4096"] = {
            "value": round(matmul["tflops"], 2), "unit": "TFLOP/s", "ms_per_step": round(matmul["ms"], 4),
            "steps": matmul["steps"], "dtype": "f32",
            "roofline": {"bound": "mfma", "achieved": round(matmul["tflops"], 2), "peak": FP32_MFMA_PEAK_TFLOPS,
                         "unit": "TFLOP/s", "frac": round(matmul["tflops"] / FP32_MFMA_PEAK_TFLOPS, 4),
                         "traffic": measured_traffic(matmul["launches"][0][0]) if not args.options else None,
                         "kernel": matmul["launches"][0][0],
                         "schedule": matmul["launches"][0][1]}}
    if cfg1:
        result_extra["config1_relu_sum_1024"] = {"us_per_step": round(cfg1["us"], 2),
                                                 "value": round(cfg1["gbs"], 1), "unit": "GB/s",
                                                 "schedule": cfg1["launches"][0][1]}
    if mlp:
        result_extra["config4_mlp_step"] = {
            "value": round(8192 / mlp["ms"] * 1e3, 1), "unit": "samples/s", "ms_per_step": round(mlp["ms"], 3),
            "steps": mlp["steps"], "tflops": round(mlp["flops"] / mlp["ms"] / 1e9, 2),
            "algorithmic_bytes": mlp["algo_bytes"], "lowered_kernels": mlp["lowered_kernels"],
            "launches": mlp["launches"], "gemm_launches": mlp["gemm_launches"], "loss": mlp.get("loss"),
            "workload": "MLP 1024-4096-4096-1024, batch 8192: forward, MSE, exact backward, SGD update, one Program"}
    if cnn:
        result_extra["config5_cnn_step"] = {
            "value": round(256 / cnn["ms"] * 1e3, 1), "unit": "images/s", "ms_per_step": round(cnn["ms"], 4),
            "steps": cnn["steps"], "algorithmic_bytes": cnn["algo_bytes"],
            "lowered_kernels": cnn["lowered_kernels"], "launches": cnn["launches"],
            "gemm_launches": cnn["gemm_launches"], "loss": cnn.get("loss"),
            "ms_per_step_hip_graph": round(cnn["graph_ms"], 4),
            "host_ms_per_step": {"eager": round(cnn["wall_ms"], 4), "hip_graph": round(cnn["graph_wall_ms"], 4)},
            "workload": "CNN 1x28x28: conv3x3(32)+relu+pool, conv3x3(64)+relu+pool, fc 3136-128-10, "
                        "cross-entropy; batch 256 forward + exact backward, plus the SGD update (more than the "
                        "configuration asks for, inside the timed region), one Program"}
    result_extra["device"] = {"name": props["name"] or "MI355X (name not reported by the runtime)", "arch": props["arch"],
                              "compute_units": props["compute_units"], "clock_khz": props["clock_khz"]}
    out["extra"] = result_extra
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
