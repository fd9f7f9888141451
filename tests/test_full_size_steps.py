"""Benchmark configurations 4 and 5 at the sizes bench.py times, through the very Programs it
times: the schedules asserted here (256x256x16 MFMA tiles, contractions with epilogues, split-K
with a summing launch, implicit-GEMM loaders) are the ones that run, and every updated
parameter and the loss are compared with a float64 numpy step; the C oracle covers what it can
finish in seconds (for the CNN the whole batch-256 step; for the MLP a row subset of the forward
pass at full widths).
"""

import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

pytestmark = pytest.mark.gpu


def _compile_and_run(hb, graph_fn, arrays, **kw):
    """bench.py's own sequence: lower_multi, one HipProgram, one execute.  Returns
    ({root name: flat float32 array} in root order, launches)."""
    from harp_amd import measure
    from harp_amd import workloads as wl
    from harp_amd.frontend import Tensor
    dev = hb.HipDevice(0)
    ts = [Tensor.input(list(a.shape)) for a in arrays]
    prog_ast, arg_names, outs, consts, _plain = wl.lower_multi(ts, graph_fn(*ts, **kw))
    prog = hb.HipProgram(dev, prog_ast, None)
    (binding, named), = measure.make_sets(dev, prog, arg_names, consts, arrays, 1)
    prog.run(binding, sync=True)
    results = [named[o].read_array(np.float32) for o in outs]
    del named, binding
    dev.trim()
    return results, prog.launches


def test_config4_mlp_step_at_benchmark_size(frontend, hip):
    """Batch 8192, 1024-4096-4096-1024.  lr = 1e-3 is the benchmarked step; at that rate an
    update is far below one ulp of most weights, so the same Program with lr = 1000 (one literal
    differs) is what exposes the gradients themselves."""
    from harp_amd import workloads as wl
    from harp_amd.checks import mlp_step
    batch, dims = wl.mlp_sizes(True)
    arrays = wl.config4_inputs(batch, dims)
    loss, grads, _ = mlp_step(arrays)
    for lr in (1e-3, 1e3):
        got, launches = _compile_and_run(hip, wl.config4_graph, arrays, lr=lr)
        scheds = [l["schedule"] for l in launches]
        big = [s for s in scheds if s.startswith("mfma32x32x2(tile=256x256x16")]
        assert len(big) >= 8, scheds                                   # 3 forward, 2 + 3 backward, at least
        assert any("epilogue=" in s for s in scheds), scheds
        assert any(s.startswith("split-k-final(") for s in scheds), scheds
        assert len(launches) <= 24, len(launches)
        assert abs(float(got[-1][0]) - loss) <= 1e-5 * abs(loss)
        for p, g, new in zip(arrays[2:], grads, got[:-1]):
            want = p.astype(np.float64) - lr * g
            # a gradient entry is a sum of `batch` (or batch * width) products: reduction class,
            # relative to the largest entry of the tensor
            tol = 1e-5 * float(np.abs(lr * g).max()) + 2.0 ** -23 * np.abs(want)
            assert np.all(np.abs(new.reshape(p.shape) - want) <= tol), (lr, p.shape)


def test_config4_forward_rows_against_the_c_oracle(frontend, hip):
    """The forward pass of config 4 at full batch and widths on HIP (its three contractions are
    the 256x256x16 schedules with the bias and tanh chain as epilogue) against the C oracle on 16
    of the 8192 rows (0.8 GFLOP of the reference's ijk loops)."""
    from conftest import realize_on
    from harp_amd import workloads as wl
    from harp_amd.checks import mlp_step
    batch, dims = wl.mlp_sizes(True)
    arrays = wl.config4_inputs(batch, dims)
    x, params = arrays[0], arrays[2:]

    def forward(xt, *ps):
        with frontend.exact_mode():
            h = xt
            for i in range(len(ps) // 2):
                h = frontend.nn.linear(h, ps[2 * i], ps[2 * i + 1])
                if i + 1 < len(ps) // 2:
                    h = wl.tanh_exact(h)
        return h
    got = realize_on(frontend, "hip", forward, [x] + params).reshape(batch, dims[-1])
    rows = np.sort(np.random.default_rng(4).choice(batch, 16, replace=False))
    ref = realize_on(frontend, "c", forward, [x[rows].copy()] + params).reshape(16, dims[-1])
    _, _, exact = mlp_step(arrays)
    assert np.allclose(got[rows], ref, rtol=1e-4, atol=1e-5)
    assert np.allclose(got, exact, rtol=1e-4, atol=1e-5)


def test_config5_cnn_step_at_benchmark_size(frontend, hip):
    """Batch 256 of 1x28x28, the SGD step bench.py times (lr = 1e-2) and the gradients-only
    form: against the C oracle running the same exact-mode graph at the same size, and against
    the float64 numpy CNN."""
    from harp_amd.checks import cnn_step
    from test_hip_parity import _cnn_step_on
    from harp_amd import workloads as wl
    sizes = wl.cnn_sizes(True)
    arrays = wl.config5_inputs(*sizes)
    loss, grads = cnn_step(arrays[0], arrays[1], arrays[2:])
    ref = _cnn_step_on(frontend, "c", arrays, lr=1e-2)
    got, launches = _compile_and_run(hip, wl.config5_graph, arrays, lr=1e-2)
    scheds = [l["schedule"] for l in launches]
    # (a layer's input gradient and weight gradient, independent contractions, go out as one launch)
    assert sum(s.count("mfma") for s in scheds) >= 11, scheds
    assert sum(s.startswith("together(mfma") for s in scheds) == 3, scheds
    # im2col never materialised: staged in LDS once per image; the second convolution's input gradient sums its nine shifts there too
    assert sum(s.count("mfma16x16x4(window,") for s in scheds) == 5 and sum("shifts=9" in s for s in scheds) == 1, scheds
    assert len(launches) <= 50, len(launches)
    assert abs(float(got[-1][0]) - float(ref[-1][0])) <= 1e-5 * abs(float(ref[-1][0]))
    assert abs(float(got[-1][0]) - loss) <= 1e-5 * abs(loss)
    for new, r, p, g in zip(got[:-1], ref[:-1], arrays[2:], grads):
        assert np.allclose(new, r, rtol=1e-5, atol=1e-6), p.shape
        assert np.allclose(new.reshape(p.shape), p - 1e-2 * g, rtol=1e-4, atol=1e-6), p.shape
    # the gradients themselves
    ref_g = _cnn_step_on(frontend, "c", arrays)
    got_g, _ = _compile_and_run(hip, wl.config5_graph, arrays)
    # Three evaluations of one step in three arithmetics.  Where a pre-activation lies within
    # rounding of zero, or two pooled values within rounding of each other, the ReLU and max-pool
    # masks of the float32 runs and of the float64 run differ, and each flipped position moves a
    # gradient entry by a whole term of its sum: observed up to 1e-3 of a tensor's largest entry
    # for either float32 run against float64, at this batch size.  A dropped or doubled term
    # would show as an error of the order of the entries themselves.
    for g_hip, g_c, g64 in zip(got_g[:-1], ref_g[:-1], grads):
        scale = max(float(np.abs(g64).max()), 1e-6)
        err_hip = float(np.abs(g_hip.reshape(g64.shape) - g64).max()) / scale
        err_c = float(np.abs(g_c.reshape(g64.shape) - g64).max()) / scale
        print(f"gradient {g64.shape}: HIP {err_hip:.2e}, oracle {err_c:.2e} of the largest entry")
        assert err_hip <= 3e-3, (g64.shape, err_hip)
        assert err_c <= 3e-3, (g64.shape, err_c)
        assert np.allclose(g_hip, g_c, rtol=1e-3, atol=3e-3 * scale)
