"""Timing of compiled programs on the device: buffer sets and event-bracketed launches.

Shared by the benchmark and the option search, so both measure the same way: inputs resident
in device memory, several independent bindings rotated between launches so that a launch does
not find its operands in the last-level cache, W untimed launches, then K launches between two
events on the launch stream with a device synchronisation on both sides.
"""

from __future__ import annotations

import hashlib
import json
import os
import time

import numpy as np

from . import backend as hb

HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E bandwidth
FP32_MFMA_PEAK_TFLOPS = 157.3  # MI355X published dense FP32 matrix peak
TRAFFIC_FILE = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "profiles", "traffic.json")


def make_sets(dev, prog, arg_names, const_inputs, arrays, nsets):
    """`nsets` independent bindings of `prog`: inputs filled from `arrays` (in the order of
    `arg_names`), synthesised constants filled with their value, outputs allocated; temps are
    kept by the program itself.  Returns [(binding, {name: buffer})]."""
    sets = []
    for _ in range(nsets):
        named = {}
        for b in prog.buffers:
            if b["elided"] or b["role"] == "temp":
                continue
            buf = hb.HipBuffer(dev, [b["bytes"]], None, nbytes=b["bytes"])
            if b["name"] in arg_names:
                buf.write_array(np.ascontiguousarray(arrays[arg_names.index(b["name"])]))
            elif b["name"] in const_inputs:
                fill = {"ones": 1.0, "zeros": 0.0, "scalar": 1.0}[const_inputs[b["name"]]]
                buf.write_array(np.full(b["bytes"] // 4, fill, dtype=np.float32))
            named[b["name"]] = buf
        sets.append((prog.bind(named), named))
    return sets


def time_steps(dev, prog, sets, steps, warmup):
    """(event ms, wall ms) per step over exactly `steps` launches after `warmup` untimed ones."""
    for i in range(warmup):
        prog.run(sets[i % len(sets)][0], sync=False)
    dev.sync()
    e0, e1 = hb.Event(dev), hb.Event(dev)
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        prog.run(sets[i % len(sets)][0], sync=False)
    e1.record()
    e1.sync()
    dev.sync()
    wall = (time.perf_counter() - t0) * 1e3
    return e0.elapsed_ms(e1) / steps, wall / steps


def time_each_step(dev, prog, sets, steps, warmup):
    """Per-step durations in ms: an event before the first launch and one behind every step, all on
    the launch stream, read after the last one completed.  Returns (median, min, mean) over `steps`
    steps after `warmup` untimed ones.  The events sit between the steps, so the mean here can
    exceed what `time_steps` measures over the same steps queued back to back."""
    for i in range(warmup):
        prog.run(sets[i % len(sets)][0], sync=False)
    dev.sync()
    events = [hb.Event(dev) for _ in range(steps + 1)]
    events[0].record()
    for i in range(steps):
        prog.run(sets[i % len(sets)][0], sync=False)
        events[i + 1].record()
    events[-1].sync()
    dev.sync()
    ms = np.array([events[i].elapsed_ms(events[i + 1]) for i in range(steps)])
    return float(np.median(ms)), float(ms.min()), float(ms.mean())


def time_replays(dev, prog, sets, steps, warmup):
    """As `time_steps`, with each binding recorded once as a HIP graph and a step = one replay."""
    graphs = [prog.record(b) for b, _ in sets]
    for i in range(warmup):
        graphs[i % len(graphs)].replay(sync=False)
    dev.sync()
    e0, e1 = hb.Event(dev), hb.Event(dev)
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        graphs[i % len(graphs)].replay(sync=False)
    e1.record()
    e1.sync()
    dev.sync()
    wall = (time.perf_counter() - t0) * 1e3
    return e0.elapsed_ms(e1) / steps, wall / steps


# ---------------------------------------------------------------------------
# the per-kernel path: what the reference's unmodified executor drives
# ---------------------------------------------------------------------------

class PerKernelPath:
    """The kernels of a lowered Program compiled one by one (`compile_ast`) and run as
    `execute_graph` runs them (src/backend/executor.rs:245-372): per kernel, allocate the
    outputs zero-filled, `Kernel::execute(inputs, outputs)` synchronously, publish the outputs
    by name for the kernels that follow.  Nothing is fused across kernels and every
    intermediate buffer exists."""

    def __init__(self, dev, program_ast, options=None):
        from .frontend import AstNode
        self.dev = dev
        self.table = {b["name"]: b for b in program_ast.attrs["buffers"]}
        self.kernels = []
        for k in program_ast.args:
            params = [p for p in k.attrs["params"] if p.dtype.is_ptr()]
            kern = hb.HipKernel(dev, AstNode.program([k]), options)
            self.kernels.append((kern, [p.name for p in params if not p.mutable],
                                 [p.name for p in params if p.mutable]))
        self.launches = [l for kern, _, _ in self.kernels for l in kern.launches]

    def _nbytes(self, name):
        b = self.table[name]
        n = b["dtype"].itemsize()
        for d in b["shape"]:
            n *= int(d)
        return n

    def step(self, inputs, sync=True):
        """One pass; `inputs` maps buffer name -> HipBuffer.  Returns all buffers by name.
        `sync=False`: launches are only queued (the Rust binding's default)."""
        named = dict(inputs)
        for kern, ins, outs in self.kernels:
            out_bufs = [self.dev.alloc(self._nbytes(n)) for n in outs]
            kern.execute([named[n] for n in ins], out_bufs, sync)
            named.update(zip(outs, out_bufs))
        return named

    def time(self, inputs, steps, warmup, sync=True):
        """Wall-clock ms per step.  With `sync` every launch waits for completion, so wall time is
        device time plus what the host spends between launches, as it would be for the reference's
        own backends; without, launches are queued and the device is waited for once at the end."""
        for _ in range(warmup):
            self.step(inputs, sync)
        self.dev.sync()
        t0 = time.perf_counter()
        for _ in range(steps):
            self.step(inputs, sync)
        self.dev.sync()
        return (time.perf_counter() - t0) * 1e3 / steps


def upload_inputs(dev, program_ast, arg_names, const_inputs, arrays):
    """Device buffers for every input row of the program's table, by name."""
    named = {}
    for b in program_ast.attrs["buffers"]:
        if b["role"] not in ("input", "ones", "zeros"):
            continue
        n = b["dtype"].itemsize()
        for d in b["shape"]:
            n *= int(d)
        buf = dev.alloc(n)
        if b["name"] in arg_names:
            buf.write_array(np.ascontiguousarray(arrays[arg_names.index(b["name"])]))
        else:
            fill = {"ones": 1.0, "zeros": 0.0, "scalar": 1.0}[const_inputs.get(b["name"], b["role"])]
            buf.write_array(np.full(n // 4, fill, dtype=np.float32))
        named[b["name"]] = buf
    return named


# ---------------------------------------------------------------------------
# counter-derived traffic, tied to the kernel source it was measured on
# ---------------------------------------------------------------------------

def source_hash(source: str) -> str:
    return hashlib.sha1(source.encode()).hexdigest()


def measured_traffic(entry: str, source: str):
    """(HBM bytes per launch, stale?) for kernel `entry` from profiles/traffic.json (rocprofv3 --pmc
    FETCH_SIZE / WRITE_SIZE, scaled by a copy kernel of known size).  The figure counts only
    while the generated source is the one it was measured on: otherwise (None, True).
    (None, False): the kernel is not in the file."""
    try:
        with open(TRAFFIC_FILE) as f:
            rec = json.load(f)["kernels"][entry]
    except (OSError, KeyError, ValueError):
        return None, False
    if rec.get("source_sha1") != source_hash(source):
        return None, True
    return rec["traffic_bytes"], False


# ---------------------------------------------------------------------------
# calibration kernels (ceilings the profiles quote; not results)
# ---------------------------------------------------------------------------

MFMA_PEAK_SOURCE = """
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
"""


def mfma_issue_rate(dev, iters=4096, waves_per_cu=8, reps=20):
    """TFLOP/s of v_mfma_f32_32x32x2_f32 issued back to back with operands in registers."""
    blocks = dev.props["compute_units"] * waves_per_cu // 4
    mod = hb.HipModule(dev, hb.compile_source(MFMA_PEAK_SOURCE % iters), "eh_mfma_peak")
    out = hb.HipBuffer(dev, [blocks * 256 * 4], None, nbytes=blocks * 256 * 4)
    for _ in range(3):
        mod.launch([blocks, 1, 1], [256, 1, 1], [out], sync=False)
    dev.sync()
    e0, e1 = hb.Event(dev), hb.Event(dev)
    e0.record()
    for _ in range(reps):
        mod.launch([blocks, 1, 1], [256, 1, 1], [out], sync=False)
    e1.record()
    e1.sync()
    ms = e0.elapsed_ms(e1) / reps
    flops = blocks * 4 * iters * 4 * (32 * 32 * 2 * 2)
    return flops / ms / 1e9, blocks, ms


EMPTY_SOURCE = """
extern "C" __global__ void __launch_bounds__(256) eh_empty(float* out) {
  if (out == nullptr) out[0] = 0.0f;
}
"""


def launch_floor_us(dev, blocks=256, reps=2000):
    """Microseconds per launch of a kernel that does nothing (`blocks` workgroups of 256), queued
    back to back on the device's stream: what one kernel boundary costs whatever the kernel
    computes -- the floor under any step made of one small grid."""
    mod = hb.HipModule(dev, hb.compile_source(EMPTY_SOURCE), "eh_empty")
    out = hb.HipBuffer(dev, [64], None, nbytes=256)
    for _ in range(50):
        mod.launch([blocks, 1, 1], [256, 1, 1], [out], sync=False)
    dev.sync()
    e0, e1 = hb.Event(dev), hb.Event(dev)
    e0.record()
    for _ in range(reps):
        mod.launch([blocks, 1, 1], [256, 1, 1], [out], sync=False)
    e1.record()
    e1.sync()
    return e0.elapsed_ms(e1) / reps * 1e3


def copy_rate(dev, shape=(4096, 4096), steps=200, warmup=20, nsets=4, options=None):
    """GB/s of a plain fp32 copy of `shape` (read + write), rotating buffer sets: the ceiling a
    memory-bound kernel of that size can reach, and the kernel the traffic counters are scaled by."""
    from . import workloads as wl
    x = np.zeros(shape, np.float32)
    ast, arg_names, _out, consts, _ = wl.lower_with_table([shape], lambda t: t.contiguous())
    prog = hb.HipProgram(dev, ast, options)
    sets = make_sets(dev, prog, arg_names, consts, [x], nsets)
    ms, _ = time_steps(dev, prog, sets, steps, warmup)
    return 2 * x.nbytes / (ms * 1e-3) / 1e9, prog.launches[0], ms


# ---------------------------------------------------------------------------
# profiles/traffic.json from rocprofv3 counter runs
# ---------------------------------------------------------------------------

def _counter_per_dispatch(directory: str, counter: str):
    """{kernel name: (mean of `counter` per dispatch, dispatches)} from the counter_collection CSV
    files rocprofv3 --pmc wrote under `directory` (one row per dispatch and counter dimension)."""
    import csv
    import glob
    per = {}
    for f in glob.glob(os.path.join(directory, "**", "*counter_collection.csv"), recursive=True):
        with open(f) as fh:
            for r in csv.DictReader(fh):
                if r["Counter_Name"] != counter:
                    continue
                d = per.setdefault(r["Kernel_Name"], {})
                d[r["Dispatch_Id"]] = d.get(r["Dispatch_Id"], 0.0) + float(r["Counter_Value"])
    return {k: (sum(v.values()) / len(v), len(v)) for k, v in per.items()}


def write_traffic_file(root: str, out_path: str = TRAFFIC_FILE):
    """Builds profiles/traffic.json from `root`/<workload>_{fetch,write} (workloads: copy, softmax,
    matmul, config1), each the output directory of
        rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE -d <dir> -o pmc --output-format csv -- \
            python3 bench.py --only <workload> --steps 10 --warmup 2 --no-cpu-baseline --no-per-kernel --no-check
    (for the copy kernel: -- python3 -m harp_amd.measure copy)
    FETCH_SIZE / WRITE_SIZE are scaled so that the plain 64 MiB copy kernel reads and writes exactly
    its 65536 KiB (it is assumed to waste nothing); every entry carries the SHA-1 of the generated
    source it was measured on, which bench.py compares with the source it times."""
    from . import workloads as wl
    copy_ast = wl.lower_with_table([(4096, 4096)], lambda t: t.contiguous())[0]
    copy_entry = hb.render_program(copy_ast).launches[0]["entry"]
    cf = _counter_per_dispatch(os.path.join(root, "copy_fetch"), "FETCH_SIZE")[copy_entry][0]
    cw = _counter_per_dispatch(os.path.join(root, "copy_write"), "WRITE_SIZE")[copy_entry][0]
    kib = 4096 * 4096 * 4 / 1024
    rec = {"calibration": {"kernel": f"{copy_entry} (plain copy, {kib:.0f} KiB read + {kib:.0f} KiB written, assumed free of wasted traffic)",
                           "FETCH_SIZE_reading": round(cf, 1), "WRITE_SIZE_reading": round(cw, 1),
                           "fetch_factor": round(kib / cf, 4), "write_factor": round(kib / cw, 4)},
           "kernels": {}}
    plans = {"softmax": wl.lower_with_table([(4096, 4096)], wl.config2_graph)[0],
             "matmul": wl.lower_with_table([(4096, 4096)] * 2, wl.config3_graph)[0],
             "config1": wl.lower_with_table([(1024, 1024)] * 3, wl.config1_graph)[0]}
    for name, ast in plans.items():
        fetch = _counter_per_dispatch(os.path.join(root, name + "_fetch"), "FETCH_SIZE")
        write = _counter_per_dispatch(os.path.join(root, name + "_write"), "WRITE_SIZE")
        for l in hb.render_program(ast).launches:
            if l["entry"] not in fetch or l["entry"] not in write:
                continue
            rd = fetch[l["entry"]][0] * kib / cf * 1024
            wr = write[l["entry"]][0] * kib / cw * 1024
            rec["kernels"][l["entry"]] = {
                "workload": name, "schedule": l["schedule"], "source_sha1": source_hash(l["source"]),
                "FETCH_SIZE_reading": round(fetch[l["entry"]][0], 1), "WRITE_SIZE_reading": round(write[l["entry"]][0], 1),
                "dispatches": [fetch[l["entry"]][1], write[l["entry"]][1]],
                "read_bytes": int(rd), "written_bytes": int(wr), "traffic_bytes": int(rd + wr),
                "algorithmic_bytes": int(l["algo_bytes"])}
    with open(out_path, "w") as f:
        json.dump(rec, f, indent=1)
        f.write("\n")
    return rec


if __name__ == "__main__":
    import sys
    usage = ("usage: python -m harp_amd.measure traffic <directory holding <workload>_fetch and <workload>_write>\n"
             "       python -m harp_amd.measure copy        (HBM rate of this backend's plain 64 MiB copy kernel)\n"
             "       python -m harp_amd.measure mfma_peak   (issue rate of v_mfma_f32_32x32x2_f32 from registers)")
    if len(sys.argv) == 3 and sys.argv[1] == "traffic":
        print(json.dumps(write_traffic_file(sys.argv[2]), indent=1))
    elif len(sys.argv) >= 2 and sys.argv[1] in ("copy", "mfma_peak"):
        if hb.device_count() == 0:
            sys.exit("harp_amd.measure: no HIP device present")
        _dev = hb.HipDevice(0)
        if sys.argv[1] == "copy":
            gbs, launch, ms = copy_rate(_dev)
            print(f"copy 4096^2 ({launch['entry']}, {launch['schedule']}): {ms * 1e3:.1f} us/step -> {gbs:.0f} GB/s")
        else:
            tflops, blocks, ms = mfma_issue_rate(_dev)
            print(f"MFMA f32 32x32x2 issue-rate ceiling: {tflops:.1f} TFLOP/s ({tflops / FP32_MFMA_PEAK_TFLOPS:.1%} of the "
                  f"published {FP32_MFMA_PEAK_TFLOPS}); {blocks} workgroups x 4 waves, {ms * 1e3:.0f} us/launch")
    else:
        sys.exit(usage)
