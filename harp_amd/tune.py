"""Beam search over the HIP generator's gfx950 schedule space, with the device as the estimator.

The reference optimises every lowered AST with `BeamSearchOptimizer`
(`src/opt/ast/optimizer/beam_search.rs:34-66, 235-410`): a beam of candidate ASTs, suggesters
that propose rewrites (tiling, vectorisation, parallelisation: `src/opt/ast/suggesters/`), a
static cost estimator (`src/opt/ast/estimator.rs`) that ranks them, stop after `max_steps` or
when nothing improves.  This backend does not rewrite ASTs: its generator picks a schedule
from the kernel's structure, and what remains open is the schedule's parameters.  The search
here keeps the reference's shape -- states, suggesters proposing neighbours, a beam, early
stop -- over that parameter space (contraction tile, wave tile, waves per SIMD, K split;
threads and elements per row; block size, vectors per thread, streaming stores), and ranks
states by running them: event-timed launches of the compiled Program on the GPU.

    python -m harp_amd.tune --config config3_matmul [--beam 3] [--steps 4]
    python -m harp_amd.tune --config config5_cnn_step --save tuned.txt
    python -m harp_amd.tune --config config5_cnn_step --per-launch --save tuned.txt

prints the best options as the "key=value,..." string `eh_program_compile` takes.  With `--save`
the result is also filed under the program's key (`backend.tune_key`) in the given file; a process
that runs with ECLAT_HIP_TUNE=<that file> then compiles this program with these options (explicit
options still win), as the reference's optimiser applies what its search found.
"""

from __future__ import annotations

import argparse
import json
import sys
from typing import Callable, Dict, Iterable, List, Optional, Sequence, Tuple

import numpy as np

from . import backend as hb
from . import measure

Options = Tuple[Tuple[str, int], ...]          # sorted (key, value) pairs: hashable state


def _freeze(d: Dict[str, int]) -> Options:
    return tuple(sorted(d.items()))


def options_string(opts: Options) -> str:
    return ",".join(f"{k}={v}" for k, v in opts)


# -- suggesters: each proposes neighbours of a state, given the schedules the plan uses ----------

GEMM_TILES = [  # (bm, bn, bk, wm, wn): macro tile, k step, wave tile; LDS 2*bk*(bm+bn+8)*4 <= 160 KiB
    (256, 256, 16, 64, 64), (256, 256, 16, 128, 64), (256, 128, 16, 64, 64), (128, 256, 16, 64, 64),
    (128, 128, 16, 64, 64), (128, 128, 16, 32, 64), (128, 128, 32, 64, 64), (128, 64, 16, 64, 32),
    (64, 64, 16, 32, 32), (64, 64, 32, 32, 32),
]


def suggest_gemm(state: Dict[str, int], schedules: Sequence[str]) -> Iterable[Dict[str, int]]:
    """Tile shapes, register budget (waves per SIMD) and K split of the MFMA contraction."""
    if not any("mfma" in s for s in schedules):
        return
    cur = tuple(state.get(k, 0) for k in ("gemm_bm", "gemm_bn", "gemm_bk", "gemm_wm", "gemm_wn"))
    for t in GEMM_TILES:
        if t != cur:
            yield {**state, **dict(zip(("gemm_bm", "gemm_bn", "gemm_bk", "gemm_wm", "gemm_wn"), t))}
    if state.get("gemm_bm", 0):
        threads = (state["gemm_bm"] // state["gemm_wm"]) * (state["gemm_bn"] // state["gemm_wn"]) * 64
        per_simd = max(1, threads // 256)
        for w in (per_simd, 2 * per_simd, 4 * per_simd):
            if w <= 8 and w != state.get("gemm_waves", 0):
                yield {**state, "gemm_waves": w}
    # (1: never; a requested split goes down to two k-steps a chunk; unset leaves it to the planner)
    for sk in (1, 2, 4, 8, 16, 32):
        if sk != state.get("gemm_split_k", -1):
            yield {**state, "gemm_split_k": sk}
    for p in (0, 1):
        if p != state.get("gemm_setprio", 0):
            yield {**state, "gemm_setprio": p}


def suggest_row(state: Dict[str, int], schedules: Sequence[str]) -> Iterable[Dict[str, int]]:
    """Threads cooperating on a row and elements per thread of row programs."""
    if not any(s.startswith("row(") for s in schedules):
        return
    for t in (32, 64, 128, 256, 512, 1024):
        if t != state.get("row_threads", 0):
            yield {**state, "row_threads": t}
    for e in (4, 8, 16):
        if e != state.get("row_elems", 8) and not state.get("row_threads", 0):
            yield {**state, "row_elems": e}


def suggest_flat(state: Dict[str, int], schedules: Sequence[str]) -> Iterable[Dict[str, int]]:
    """Block size and vectors per thread of flat elementwise kernels."""
    if not any(s.startswith("flat(") for s in schedules):
        return
    for b in (128, 256, 512, 1024):
        if b != state.get("flat_block", 256):
            yield {**state, "flat_block": b}
    for it in (1, 2, 4, 8):
        if it != state.get("flat_iters", 4):
            yield {**state, "flat_iters": it}


def suggest_streaming(state: Dict[str, int], schedules: Sequence[str]) -> Iterable[Dict[str, int]]:
    """Non-temporal stores / loads for the memory-bound schedules."""
    if not any(s.startswith(("row(", "flat(")) for s in schedules):
        return
    for nt in (0, 1, 2):
        if nt != state.get("nontemporal", -1):
            yield {**state, "nontemporal": nt}


def suggest_pipeline(state: Dict[str, int], schedules: Sequence[str]) -> Iterable[Dict[str, int]]:
    """How far ahead of their use a contraction's tiles are loaded (register stages), whether they
    go through registers or straight into LDS, and how many streams a program's independent
    launches are spread over: the register, LDS and queue budgets of a plan."""
    if any("mfma" in s for s in schedules):
        for p in (1, 3, 5):
            if p != state.get("gemm_prefetch", 0):
                yield {**state, "gemm_prefetch": p}
        for d in (0, 1):
            if d != state.get("gemm_dma", 2):
                yield {**state, "gemm_dma": d}
    if len(schedules) >= 8:
        for n in (1, 2, 3):
            if n != state.get("lanes", 1):
                yield {**state, "lanes": n}


def suggest_window(state: Dict[str, int], schedules: Sequence[str]) -> Iterable[Dict[str, int]]:
    """Passes over k of the LDS-staged window contractions (stores of one pass drain behind the
    next), their interleaving of LDS reads with MFMAs, or the tile-loader schedule instead."""
    if not any("mfma16x16x4(window," in s for s in schedules) and not state.get("gemm_window", 1) == 0:
        return
    for p in (1, 2, 3, 4):
        if p != state.get("window_passes", 0):
            yield {**state, "window_passes": p}
    for m in (0, 1):
        if m != state.get("gemm_mix", 1):
            yield {**state, "gemm_mix": m}
    if state.get("gemm_window", 1):
        yield {"gemm_window": 0}


SUGGESTERS: List[Callable] = [suggest_gemm, suggest_row, suggest_flat, suggest_streaming, suggest_pipeline]
LAUNCH_SUGGESTERS: List[Callable] = [suggest_gemm, suggest_window, suggest_row, suggest_flat, suggest_streaming]


def save_tuned(path: str, key: str, options: str, note: str = "") -> None:
    """Appends "<key> <options>  # note" to `path` (the last line for a key counts)."""
    if not options:
        options = "fuse=1"                    # an entry that changes nothing still records the search
    with open(path, "a") as f:
        f.write(f"{key} {options}" + (f"  # {note}" if note else "") + "\n")


# -- the search --------------------------------------------------------------------------------

class MeasuredEstimator:
    """Cost of a state = event-timed milliseconds per launch of the Program compiled with it.
    States the generator or hiprtc rejects cost infinity."""

    def __init__(self, dev, prog_ast, arg_names, consts, arrays, steps=20, warmup=3, sets=2):
        self.dev, self.ast = dev, prog_ast
        self.arg_names, self.consts, self.arrays = arg_names, consts, arrays
        self.steps, self.warmup, self.nsets = steps, warmup, sets
        self.cache: Dict[Options, float] = {}
        self.key = hb.tune_key(prog_ast)

    def schedules(self, opts: Options) -> List[str]:
        return [l["schedule"] for l in hb.render_program(self.ast, dict(opts) or None).launches]

    def cost(self, opts: Options) -> float:
        if opts in self.cache:
            return self.cache[opts]
        try:
            prog = hb.HipProgram(self.dev, self.ast, dict(opts) or None)
            sets = measure.make_sets(self.dev, prog, self.arg_names, self.consts, self.arrays, self.nsets)
            ms, _ = measure.time_steps(self.dev, prog, sets, self.steps, self.warmup)
        except hb.EhError:
            ms = float("inf")
        self.cache[opts] = ms
        return ms


def beam_search(estimator, start: Optional[Dict[str, int]] = None, beam_width: int = 3, max_steps: int = 4,
                no_improvement_limit: int = 1, suggesters: Sequence[Callable] = SUGGESTERS, log=None):
    """Returns (best options, best cost, history).  history: [(step, options string, cost)]
    for every state measured, in measurement order."""
    first = _freeze(start or {})
    beam = [(estimator.cost(first), first)]
    history = [(0, options_string(first), beam[0][0])]
    best_cost, best = beam[0]
    stale = 0
    seen = {first}
    for step in range(1, max_steps + 1):
        candidates = []
        for _, state in beam:
            schedules = estimator.schedules(state)
            for sg in suggesters:
                for nxt in sg(dict(state), schedules):
                    f = _freeze(nxt)
                    if f in seen:
                        continue
                    seen.add(f)
                    c = estimator.cost(f)
                    history.append((step, options_string(f), c))
                    if log:
                        log(f"[tune] step {step}: {options_string(f) or '(defaults)'} -> {c:.4f} ms")
                    candidates.append((c, f))
        if not candidates:
            break
        beam = sorted(beam + candidates)[:beam_width]
        if beam[0][0] < best_cost * 0.995:
            best_cost, best = beam[0]
            stale = 0
        else:
            stale += 1
            if stale >= no_improvement_limit:
                break
    return best, best_cost, history


def per_launch_search(estimator, base: Optional[Dict[str, int]] = None, max_launches: int = 12, log=None):
    """One sweep over the launches of the plan, in the order of their share of the step's work: each
    launch's own options (suggesters applied to that launch's schedule alone) are tried with
    everything else as it stands, and kept when the whole step gains 0.5 %.  Options for a launch
    are filed under its key (`launch["tune_key"]`), so they follow the launch's lowered kernel into
    any program.  Returns ({key: options}, cost, history)."""
    base = dict(base or {})
    plan = hb.render_program(estimator.ast, base or None)
    launches = {}
    for l in plan.launches:            # (the two launches of a split contraction share a key)
        k = l["tune_key"]
        w = launches.setdefault(k, {"schedule": l["schedule"], "weight": 0.0, "entry": l["entry"]})
        w["weight"] += 4.0 + max(l["algo_bytes"] / 4.0e6, l["flops"] / 5.0e7)
    order = sorted(launches, key=lambda k: -launches[k]["weight"])[:max_launches]
    chosen: Dict[str, Dict[str, int]] = {}

    def state_of(extra_key=None, extra=None):
        st = dict(base)
        for k, o in list(chosen.items()) + ([(extra_key, extra)] if extra_key else []):
            for name, v in o.items():
                st[f"@{k}:{name}"] = v
        return _freeze(st)

    best_cost = estimator.cost(state_of())
    history = [(0, "", best_cost)]
    for k in order:
        sched = [launches[k]["schedule"].replace("together(", "")]
        mine = dict(chosen.get(k, {}))
        tried = {_freeze(mine)}
        for sg in LAUNCH_SUGGESTERS:
            for nxt in sg(dict(mine), sched):
                f = _freeze(nxt)
                if f in tried:
                    continue
                tried.add(f)
                c = estimator.cost(state_of(k, nxt))
                history.append((k, options_string(f), c))
                if log:
                    log(f"[tune] {launches[k]['entry']} ({k}): {options_string(f)} -> {c:.4f} ms (best {best_cost:.4f})")
                if c < best_cost * 0.995:
                    best_cost, mine = c, dict(nxt)
                    chosen[k] = mine
    return {k: options_string(_freeze(o)) for k, o in chosen.items() if o}, best_cost, history


def tune_config(name: str, shapes=None, beam_width=3, max_steps=4, steps=20, log=None, save=None, per_launch=False):
    """Searches the options of one benchmark configuration on device 0: one of
    `workloads.CONFIGS`, or a whole training step (`config4_mlp_step`, `config5_cnn_step`),
    where one option set serves every launch of the step."""
    from . import workloads as wl
    from .frontend import Tensor
    dev = hb.HipDevice(0)
    if name in ("config4_mlp_step", "config5_cnn_step"):
        mlp = name == "config4_mlp_step"
        arrays = wl.config4_inputs(*wl.mlp_sizes(True)) if mlp else wl.config5_inputs(*wl.cnn_sizes(True))
        ts = [Tensor.input(list(a.shape)) for a in arrays]
        roots = wl.config4_graph(*ts) if mlp else wl.config5_graph(*ts, lr=1e-2)
        prog_ast, arg_names, _outs, consts, _ = wl.lower_multi(ts, roots)
        est = MeasuredEstimator(dev, prog_ast, arg_names, consts, arrays, steps=steps, sets=1)
        if per_launch:
            chosen, cost, history = per_launch_search(est, log=log)
            if save:
                for k, o in chosen.items():
                    save_tuned(save, k, o, f"{name}, one launch: step {cost:.4f} ms (defaults {history[0][2]:.4f} ms)")
            return _freeze({f"@{k}:{n}": int(v) for k, o in chosen.items() for n, v in (i.split("=") for i in o.split(","))}), cost, history
        return _search_and_file(est, name, beam_width, max_steps, log, save)
    default_shapes = {"config1_relu_sum": [(1024, 1024)] * 3, "config2_softmax": [(4096, 4096)],
                      "config3_matmul": [(4096, 4096)] * 2}
    shapes = shapes or default_shapes[name]
    inputs_fn, graph_fn = wl.CONFIGS[name]
    rng = np.random.default_rng(7)
    arrays = [rng.uniform(-1, 1, s).astype(np.float32) for s in shapes]
    prog_ast, arg_names, _out, consts, _ = wl.lower_with_table(shapes, graph_fn)
    est = MeasuredEstimator(dev, prog_ast, arg_names, consts, arrays, steps=steps)
    return _search_and_file(est, name, beam_width, max_steps, log, save)


def _search_and_file(est, name, beam_width, max_steps, log, save):
    best, cost, history = beam_search(est, beam_width=beam_width, max_steps=max_steps, log=log)
    if save:
        save_tuned(save, est.key, options_string(best), f"{name}: {cost:.4f} ms (defaults {history[0][2]:.4f} ms)")
    return best, cost, history


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--config", default="config3_matmul")
    ap.add_argument("--beam", type=int, default=3)
    ap.add_argument("--steps", type=int, default=4, help="search steps (beam expansions)")
    ap.add_argument("--launches", type=int, default=20, help="timed launches per state")
    ap.add_argument("--save", default=None, help="file to append the result to (read back through ECLAT_HIP_TUNE)")
    ap.add_argument("--per-launch", action="store_true",
                    help="training steps: search each launch's own options, filed under the launch's key")
    args = ap.parse_args(argv)
    if hb.device_count() == 0:
        sys.exit("tune: no HIP device present")
    best, cost, history = tune_config(args.config, beam_width=args.beam, max_steps=args.steps,
                                      steps=args.launches, log=lambda m: print(m, file=sys.stderr, flush=True),
                                      save=args.save, per_launch=args.per_launch)
    print(json.dumps({"config": args.config, "options": options_string(best), "ms": cost,
                      "default_ms": history[0][2], "states_measured": len(history)}))
    return 0


if __name__ == "__main__":
    sys.exit(main())
