"""Parity of the HIP backend with the CPU oracle on identical seeded inputs.
Every case goes through the C ABI (ctypes -> libeclat_hip.so).

Tolerance classes (written where they are applied):
  * add / mul / max / select / compare / cast / copies / indexing: bit-exact
    (up to the sign of zero and flushed denormals: the oracle is gcc -ffast-math);
  * recip / sqrt / exp2 / log2 / sin: 4 ulp-class, rtol 1e-6 (libm vs device libm);
  * reductions (incl. softmax): rtol 1e-5;
  * K=4096 MFMA matmul: rtol 1e-3 of the row scale.
"""

import numpy as np
import pytest

import golden_ops
from conftest import bits_equal_mod_zero, realize_on

pytestmark = pytest.mark.gpu

RNG = np.random.default_rng


def both(fe, build, arrays, fuse=True):
    ref = realize_on(fe, "c", build, arrays)
    got = realize_on(fe, "hip", build, arrays, fuse=fuse)
    return ref, got


@pytest.mark.parametrize("fuse", [False, True])
def test_reference_known_answers(frontend, hip, fuse):
    a = np.array([1, 2, 3, 4], dtype=np.float32)
    b = np.array([5, 6, 7, 8], dtype=np.float32)
    assert realize_on(frontend, "hip", lambda x, y: x + y, [a, b], fuse=fuse).tolist() == [6, 8, 10, 12]
    b2 = np.array([2, 3, 4, 5], dtype=np.float32)
    assert realize_on(frontend, "hip", lambda x, y: x * y, [a, b2], fuse=fuse).tolist() == [2, 6, 12, 20]
    m1 = np.array([[1, 2], [3, 4]], dtype=np.float32)
    m2 = np.array([[5, 6], [7, 8]], dtype=np.float32)
    out = realize_on(frontend, "hip", lambda x, y: frontend.nn.matmul(x, y), [m1, m2], fuse=fuse)
    assert out.tolist() == [19, 22, 43, 50]


_FX = golden_ops.load()


@pytest.mark.parametrize("case", _FX["forward"], ids=lambda c: c["id"])
@pytest.mark.parametrize("fuse", [False, True])
def test_fixture_forward_known_answers(frontend, hip, case, fuse):
    """The reference's own known answers (tests/golden/) through the HIP backend."""
    arrays = [golden_ops.array(v, s) for v, s in zip(case["inputs"], case["shapes"])]
    out = realize_on(frontend, "hip", golden_ops.graph(frontend, case["op"]), arrays, fuse=fuse)
    golden_ops.check_forward(case, out)


def test_fixture_gradients_and_properties(frontend, hip):
    from harp_amd.frontend.tensor import _INPUT_BUFFER_CACHE
    for case in _FX["properties"]:
        arrays = [golden_ops.array(v, s) for v, s in zip(case["inputs"], case["shapes"])]
        out = realize_on(frontend, "hip", golden_ops.graph(frontend, case["op"]), arrays)
        assert out.size == case["length"] and abs(float(out.sum()) - case["sum"]) < case["atol"]
    frontend.set_device_str("hip")
    for case in _FX["gradients"]:
        try:
            ts = []
            for v, s in zip(case["inputs"], case["shapes"]):
                t = frontend.Tensor.input(s).requires_grad_(True)
                t.set_data(golden_ops.array(v, s))
                ts.append(t)
            golden_ops.graph(frontend, case["op"])(*ts).backward_with_params(ts)
            got = [t.grad().realize().to_numpy().tolist() for t in ts]
        finally:
            _INPUT_BUFFER_CACHE.clear()
        assert got == [[float(v) for v in e] for e in case["expected"]], case["id"]


ELEMENTWISE = {
    "mul_add": lambda a, b, c: a * b + c,
    "relu_chain": lambda a, b, c: (a * b + c).maximum(c) - a,
    "neg_min": lambda a, b, c: (-a).minimum(b) * c,
    "where": lambda a, b, c: a.where_cond(a.lt(b), c),
    "abs": lambda a, b, c: a.abs() + b * c,
}


@pytest.mark.parametrize("shape", [(1,), (7,), (37, 53), (64, 128), (3, 5, 8), (1000, 1024)])
@pytest.mark.parametrize("name", sorted(ELEMENTWISE))
@pytest.mark.parametrize("fuse", [False, True])
def test_elementwise_bit_exact(frontend, hip, shape, name, fuse):
    rng = RNG(hash((shape, name)) % 2**32)
    arrs = [rng.normal(0, 1, shape).astype(np.float32) for _ in range(3)]
    ref, got = both(frontend, ELEMENTWISE[name], arrs, fuse)
    assert bits_equal_mod_zero(ref, got)


@pytest.mark.parametrize("shapes", [[(33, 7, 2), (33, 7)], [(129, 5, 6), (129, 5)], [(1, 1, 2), (1, 1)], [(64, 14, 2, 14, 2), (64, 14, 2, 14)]])
@pytest.mark.parametrize("fuse", [False, True])
def test_elementwise_in_pairs_bit_exact(frontend, hip, shapes, fuse):
    """A contiguous extent two (or six) wide next to an operand that does not move along it (a
    pooling window put back over its image): the flat schedule works in pairs, 64-bit accesses
    for what moves and one read for what does not.  Bit-exact against the oracle."""
    rng = RNG(sum(sum(s) for s in shapes))
    arrs = [rng.normal(0, 1, s).astype(np.float32) for s in shapes]
    fn = lambda x, y: x * y.unsqueeze(len(shapes[0]) - 1) + x
    if fuse:
        from harp_amd import workloads as wl
        plan = hip.render_program(wl.lower_with_table(shapes, fn)[0])
        assert [l["schedule"] for l in plan.launches] == ["flat(V=2,block=256)"]
    ref, got = both(frontend, fn, arrs, fuse)
    assert bits_equal_mod_zero(ref, got)


@pytest.mark.parametrize("op", ["sqrt", "recip", "exp", "ln", "sin", "cos", "exp2", "log2"])
@pytest.mark.parametrize("fuse", [False, True])
def test_transcendental_elementwise(frontend, hip, op, fuse):
    x = RNG(5).uniform(0.1, 9.0, (33, 65)).astype(np.float32)
    ref, got = both(frontend, lambda t: getattr(t, op)(), [x], fuse)
    assert np.allclose(got, ref, rtol=1e-6, atol=1e-6)


def test_floor_and_cast_bit_exact(frontend, hip):
    x = RNG(6).normal(0, 50, (17, 19)).astype(np.float32)
    ref, got = both(frontend, lambda t: t.floor(), [x])
    assert bits_equal_mod_zero(ref, got)


OTHER_TYPES = {
    # name: (graph, numpy dtype, value range, exact?)
    "i32_mul_add": (lambda a, b: a * b + a, np.int32, 1000, True),
    "i32_row_sum": (lambda a, b: (a * b).sum(1), np.int32, 1000, True),
    "i32_max": (lambda a, b: a.maximum(b).max(1), np.int32, 1000, True),
    "i64_add": (lambda a, b: a + b, np.int64, 2 ** 40, True),
    "f64_mul_add": (lambda a, b: a * b + a, np.float64, 3.0, True),
    "f64_row_sum": (lambda a, b: (a * b).sum(1), np.float64, 3.0, False),
    # the C renderer names the float functions whatever the element type
    # (crates/backend-c/src/renderer.rs:182-201), so the oracle's double sqrt and max go
    # through single precision; the device code uses the double forms
    "f64_sqrt": (lambda a, b: (a * a + b * b).sqrt(), np.float64, 3.0, False),
    "f64_max": (lambda a, b: a.maximum(b), np.float64, 3.0, False),
}


@pytest.mark.parametrize("shape", [(5, 7), (64, 128), (33, 1000)])
@pytest.mark.parametrize("name", sorted(OTHER_TYPES))
def test_other_element_types(frontend, hip, name, shape):
    """i32, i64 and f64 tensors through the same schedules (the benchmark configurations
    are all fp32).  Integer results and double add/mul are bit-exact; what the oracle
    computes in single precision, or sums in another order, is held to 1e-6."""
    fn, dt, lim, exact = OTHER_TYPES[name]
    rng = RNG(hash((name, shape)) % 2**32)
    if np.issubdtype(dt, np.integer):
        arrs = [rng.integers(-lim, lim, shape).astype(dt) for _ in range(2)]
    else:
        arrs = [rng.uniform(-lim, lim, shape).astype(dt) for _ in range(2)]
    for fuse in (False, True):
        ref, got = both(frontend, fn, arrs, fuse)
        assert got.dtype == ref.dtype == dt
        if exact:
            assert np.array_equal(got, ref), (name, fuse)
        else:
            assert np.allclose(got, ref, rtol=1e-6, atol=1e-6), (name, fuse)


def test_double_contraction_keeps_double_precision(frontend, hip):
    """The MFMA schedule is fp32 only: a double contraction takes a generic reduce schedule
    and keeps double accuracy."""
    rng = RNG(9)
    a, b = rng.uniform(-1, 1, (37, 64)), rng.uniform(-1, 1, (64, 29))
    ref, got = both(frontend, lambda x, y: frontend.nn.matmul(x, y), [a, b])
    assert got.dtype == np.float64
    assert np.allclose(got, ref, rtol=1e-12, atol=1e-13)
    assert np.allclose(got.reshape(37, 29), a @ b, rtol=1e-12, atol=1e-13)


def test_cast_round_trip_bit_exact(frontend, hip):
    x = RNG(8).normal(0, 50, (64, 96)).astype(np.float32)
    ref, got = both(frontend, lambda t: t.cast(frontend.I32).cast(frontend.F32), [x])
    assert np.array_equal(got, ref) and np.array_equal(got.reshape(x.shape), np.trunc(x))


@pytest.mark.parametrize("shape,axis", [((8, 10), 1), ((33, 1000), 1), ((16, 4096), 1), ((5, 7, 64), 2),
                                        ((64, 48), 0), ((9, 130, 6), 1), ((1, 17), 1), ((17, 1), 1),
                                        ((300, 70000), 1)])
@pytest.mark.parametrize("op", ["sum", "max", "min", "prod"])
@pytest.mark.parametrize("fuse", [False, True])
def test_reductions(frontend, hip, shape, axis, op, fuse):
    rng = RNG(hash((shape, axis, op)) % 2**32)
    if op == "prod":
        x = rng.uniform(0.97, 1.03, shape).astype(np.float32)
    else:
        x = rng.normal(0, 1, shape).astype(np.float32)
    ref, got = both(frontend, lambda t: getattr(t, op)(axis), [x], fuse)
    if op in ("max", "min"):
        assert bits_equal_mod_zero(ref, got)          # order-independent, exact
    else:
        scale = np.abs(x).sum(axis).ravel() if op == "sum" else np.abs(ref)
        # rel-err 1e-5; a product's rounding error grows with the number of factors on both
        # sides (each is ~sqrt(K)*2^-24 from the exact value), so long products get K/4096 of it
        tol = 1e-5 * (max(1.0, shape[axis] / 4096.0) if op == "prod" else 1.0)
        assert np.all(np.abs(got - ref) <= tol * np.maximum(scale, 1e-30))


@pytest.mark.parametrize("shape", [(8, 10), (33, 1000), (128, 4096), (4, 6, 50), (2, 100000)])
@pytest.mark.parametrize("fuse", [False, True])
def test_softmax_and_log_softmax(frontend, hip, shape, fuse):
    x = RNG(len(shape) * 1000 + shape[-1]).normal(0, 2, shape).astype(np.float32)
    ax = len(shape) - 1
    ref, got = both(frontend, lambda t: frontend.nn.softmax(t, ax), [x], fuse)
    assert np.allclose(got, ref, rtol=1e-5, atol=1e-9)             # reduction class
    assert np.allclose(got.reshape(-1, shape[-1]).sum(1), 1.0, atol=1e-5)
    ref, got = both(frontend, lambda t: frontend.nn.log_softmax(t, ax), [x], fuse)
    assert np.allclose(got, ref, rtol=1e-5, atol=2e-5)


@pytest.mark.parametrize("shape", [(32, 512), (7, 33), (512, 4096)])
@pytest.mark.parametrize("fuse", [False, True])
def test_layer_norm_rows(frontend, hip, shape, fuse):
    """The graph of `crates/cli/examples/layer_norm.ecl`: two row sums, a square root and an
    affine map.  The tensor API has no scalar constants, so 1/C and eps come in as vectors.
    Fused, the ten lowered kernels are one row launch."""
    R, C = shape
    rng = RNG(R * 100 + C)
    x = rng.normal(0.5, 2, shape).astype(np.float32)
    gamma, beta = (rng.normal(1, 0.2, (C,)).astype(np.float32) for _ in range(2))
    inv = np.full((R,), 1.0 / C, np.float32)
    eps = np.full((R,), 1e-5, np.float32)

    def layer_norm(t, g, b, inv_n, e):
        mean = t.sum(1) * inv_n
        centred = t - mean.unsqueeze(1).expand(1, C)
        var = (centred * centred).sum(1) * inv_n
        std = (var + e).sqrt()
        return centred / std.unsqueeze(1).expand(1, C) * g.unsqueeze(0).expand(0, R) + b.unsqueeze(0).expand(0, R)

    ref, got = both(frontend, layer_norm, [x, gamma, beta, inv, eps], fuse)
    assert np.allclose(got, ref, rtol=1e-5, atol=1e-5)             # reduction class
    x64 = x.astype(np.float64)
    want = (x64 - x64.mean(1, keepdims=True)) / np.sqrt(x64.var(1, keepdims=True) + 1e-5) * gamma + beta
    assert np.allclose(got.reshape(shape), want, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("fuse", [False, True])
def test_config1_fused_elementwise_reduce(frontend, hip, fuse):
    """benchmark configuration 1: s = sum(relu(a*b + c), -1), fp32 [1024,1024], N(0,1)."""
    rng = RNG(1234)
    a, b, c = (rng.normal(0, 1, (1024, 1024)).astype(np.float32) for _ in range(3))
    ref, got = both(frontend, lambda x, y, z: frontend.nn.relu(x * y + z).sum(1), [a, b, c], fuse)
    assert np.allclose(got, ref, rtol=1e-5)
    assert np.all(got >= 0)


def test_config2_row_softmax_full_size(frontend, hip):
    """benchmark configuration 2: row softmax of fp32 [4096,4096], N(0, std 2)."""
    x = RNG(1235).normal(0, 2, (4096, 4096)).astype(np.float32)
    ref, got = both(frontend, lambda t: frontend.nn.softmax(t, 1), [x])
    assert np.allclose(got, ref, rtol=1e-5, atol=1e-12)
    got2 = got.reshape(4096, 4096)
    assert np.allclose(got2.sum(1), 1.0, atol=1e-5)
    assert np.array_equal(got2.argmax(1), x.argmax(1))


@pytest.mark.parametrize("m,k,n", [(4, 3, 2), (64, 64, 64), (128, 256, 128), (256, 96, 192), (100, 60, 36),
                                   (512, 1024, 256)])
@pytest.mark.parametrize("fuse", [False, True])
def test_matmul_small(frontend, hip, m, k, n, fuse):
    rng = RNG(m * 7 + k * 3 + n)
    a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    ref, got = both(frontend, lambda x, y: frontend.nn.matmul(x, y), [a, b], fuse)
    scale = (np.abs(a) @ np.abs(b)).ravel()
    assert np.all(np.abs(got - ref) <= 1e-5 * scale + 1e-30)


@pytest.mark.parametrize("batch,kin,kout", [(8, 12, 5), (256, 128, 64), (128, 320, 192)])
def test_linear_layer(frontend, hip, batch, kin, kout):
    rng = RNG(batch + kin + kout)
    x = rng.uniform(-1, 1, (batch, kin)).astype(np.float32)
    w = rng.uniform(-1, 1, (kout, kin)).astype(np.float32)
    bias = rng.uniform(-1, 1, (kout,)).astype(np.float32)
    ref, got = both(frontend, lambda t, u, v: frontend.nn.linear(t, u, v), [x, w, bias])
    scale = (np.abs(x) @ np.abs(w.T) + np.abs(bias)).ravel()
    assert np.all(np.abs(got - ref) <= 1e-5 * scale)


def test_config3_matmul_4096(frontend, hip):
    """benchmark configuration 3: C = A@B, fp32 4096^3, U(-1,1).  The C oracle runs a row subset
    (64 rows of A, 2 GFLOP); float64 numpy covers every row."""
    rng = RNG(1236)
    a = rng.uniform(-1, 1, (4096, 4096)).astype(np.float32)
    b = rng.uniform(-1, 1, (4096, 4096)).astype(np.float32)
    got = realize_on(frontend, "hip", lambda x, y: frontend.nn.matmul(x, y), [a, b]).reshape(4096, 4096)
    rows = np.sort(rng.choice(4096, 64, replace=False))
    ref_rows = realize_on(frontend, "c", lambda x, y: frontend.nn.matmul(x, y), [a[rows].copy(), b])
    ref_rows = ref_rows.reshape(64, 4096)
    scale = np.abs(a[rows]) @ np.abs(b)
    assert np.all(np.abs(got[rows] - ref_rows) <= 1e-3 * scale)                   # north-star bound
    assert np.max(np.abs(got[rows] - ref_rows) / scale) < 1e-5                    # what is observed
    ref64 = a.astype(np.float64) @ b.astype(np.float64)
    err = np.abs(got - ref64) / (np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64))
    assert err.max() < 1e-5


INDEX_FORMS = {
    "transpose": lambda t: t.permute([1, 0]).contiguous(),
    "broadcast": lambda t: t.unsqueeze(0).expand(0, 3).contiguous(),
    "pad": lambda t: t.pad([(1, 2), (0, 1)]).contiguous(),
    "reshape_sum": lambda t: t.reshape([3, 8]).sum(1),
    "cumsum": lambda t: t.cumsum(1),
    "cummax": lambda t: t.cummax(0),
    "unfold": lambda t: t.unfold([0, 1], [2, 3], [1, 1], [1, 1]).contiguous(),
    "fold_unfold": lambda t: t.unfold([0, 1], [2, 2], [2, 2], [1, 1]).fold([4, 6], [0, 1], [2, 2], [2, 2], [1, 1]),
    "neg_transposed": lambda t: (-t.permute([1, 0])).contiguous(),
}


@pytest.mark.parametrize("name", sorted(INDEX_FORMS))
@pytest.mark.parametrize("fuse", [False, True])
def test_index_forms_bit_exact(frontend, hip, name, fuse):
    x = RNG(11).normal(0, 1, (4, 6)).astype(np.float32)
    ref, got = both(frontend, INDEX_FORMS[name], [x], fuse)
    if name in ("cumsum", "reshape_sum"):          # sums: reduction class
        assert np.allclose(got, ref, rtol=1e-6)
    else:
        assert bits_equal_mod_zero(ref, got)


GATHER_FORMS = {
    "transpose": lambda t: t.permute([1, 0]).contiguous(),
    "pad": lambda t: t.pad([(1, 2), (3, 1)]).contiguous(),
    "windows": lambda t: t.unfold([0, 1], [3, 3], [1, 1], [1, 1]).contiguous(),
    "tiles_interleaved": lambda t: t.unfold([0, 1], [2, 2], [2, 2], [1, 1]).permute([0, 2, 1, 3]).contiguous(),
    "flip_neg": lambda t: (-type(t).from_graph(t.graph.flip(1))).contiguous(),   # flip exists on graph nodes only
    "repeat_rows": lambda t: t.unsqueeze(0).expand(0, 5).contiguous(),
}


@pytest.mark.parametrize("name", sorted(GATHER_FORMS))
@pytest.mark.parametrize("shape", [(64, 96), (50, 82)])
def test_gathering_copies_bit_exact(frontend, hip, name, shape):
    """Copies through permuted, padded, windowed and repeated views, thousands of elements
    (several workgroups of the flat schedule, ragged last block)."""
    x = RNG(shape[0]).normal(0, 1, shape).astype(np.float32)
    fn = GATHER_FORMS[name]
    t = frontend.Tensor.input(list(shape))
    with frontend.exact_mode():
        prog, _, _ = frontend.lower_graph([fn(t).graph])
        scheds = [l["schedule"] for l in hip.render_program(prog).launches]
        ref, got = both(frontend, fn, [x], True)
    assert any(s.startswith("flat(") for s in scheds), scheds
    assert bits_equal_mod_zero(ref, got)


def test_tensor_beyond_32_bit_indices(frontend, hip):
    """2^31 + 262 144 elements (8.6 GB of fp32): element and row indices leave the 32-bit
    range, so the generated kernels must switch to 64-bit index arithmetic.  Elementwise
    result bit-exact, row maxima exact, row sums in the reduction class."""
    rows, cols = 65544, 32768
    block = RNG(31).normal(0, 1, (rows // 8, cols)).astype(np.float32)
    x = np.tile(block, (8, 1))
    del block
    ref, got = both(frontend, lambda t: t * t + t, [x])
    assert got.size == rows * cols > 2 ** 31
    assert bits_equal_mod_zero(ref, got)
    assert np.array_equal(got[-cols:], (x[-1] * x[-1] + x[-1]))          # the very last row
    del ref, got
    ref, got = both(frontend, lambda t: t.max(1), [x])
    assert np.array_equal(ref, got) and np.array_equal(got, x.max(1))
    ref, got = both(frontend, lambda t: t.sum(1), [x])
    assert np.allclose(got, ref, rtol=1e-5, atol=1e-5 * np.abs(x[:64]).sum(1).max())


@pytest.mark.parametrize("name", ["attention", "attention_masked", "avg_pool2d", "conv1d", "elu", "gelu",
                                  "leaky_relu", "prelu", "silu"])
@pytest.mark.parametrize("fuse", [False, True])
def test_nn_functions(frontend, hip, name, fuse):
    """Activations, 1-D convolution, average pooling and scaled dot-product attention
    (tests/nn_cases.py): HIP against the oracle, and against the formula in float64."""
    import nn_cases
    fn, arrays, want = nn_cases.cases(frontend)[name]
    with frontend.exact_mode():
        ref, got = both(frontend, fn, arrays, fuse)
    assert np.allclose(got, ref, rtol=2e-5, atol=2e-6)
    assert np.allclose(got.reshape(want.shape), want, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("optimizer", ["sgd", "momentum", "adam"])
def test_training_loop_on_the_device(frontend, hip, optimizer):
    """Six optimizer steps of a small MLP (tests/train_loop.py); every step is one Program
    (forward, exact backward, update of parameters and optimizer state), the new parameters
    stay on the device.  HIP against the oracle and against float64 numpy."""
    import train_loop
    ref_losses, ref_params = train_loop.run(frontend, "c", optimizer, 6)
    losses, params = train_loop.run(frontend, "hip", optimizer, 6)
    np_losses, np_params = train_loop.run_numpy(frontend, optimizer, 6)
    assert np.allclose(losses, ref_losses, rtol=1e-5) and np.allclose(losses, np_losses, rtol=1e-4)
    for a, b, c in zip(params, ref_params, np_params):
        assert np.allclose(a, b, rtol=1e-4, atol=1e-6) and np.allclose(a, c, rtol=1e-3, atol=1e-5)


GROUP_PARALLEL_ADD = """
(program (kernel "E_1000_0" (params ("gidx0" i64 imm (group_id 0)) ("buf0" (ptr f32 global) imm normal)
    ("buf2" (ptr f32 global) imm normal) ("buf4" (ptr f32 global) mut normal))
  (grid (const i64 1000) (const i64 1) (const i64 1)) (tg (const i64 1) (const i64 1) (const i64 1))
  (block (decls) (store (var "buf4") (var "gidx0")
     (add (load (var "buf0") (var "gidx0") 1 f32) (load (var "buf2") (var "gidx0") 1 f32))))))
"""

GROUP_AND_LOCAL_ADD = """
(program (kernel "E_1000_0" (params ("gidx0" i64 imm (group_id 0)) ("lidx0" i64 imm (local_id 0))
    ("buf0" (ptr f32 global) imm normal) ("buf2" (ptr f32 global) imm normal) ("buf4" (ptr f32 global) mut normal))
  (grid (idiv (add (const i64 1000) (const i64 63)) (const i64 64)) (const i64 1) (const i64 1))
  (tg (const i64 64) (const i64 1) (const i64 1))
  (block (decls)
    (if (lt (add (mul (var "gidx0") (const i64 64)) (var "lidx0")) (const i64 1000))
      (store (var "buf4") (add (mul (var "gidx0") (const i64 64)) (var "lidx0"))
        (add (load (var "buf0") (add (mul (var "gidx0") (const i64 64)) (var "lidx0")) 1 f32)
             (load (var "buf2") (add (mul (var "gidx0") (const i64 64)) (var "lidx0")) 1 f32)))))))
"""


@pytest.mark.parametrize("text,grid,block", [(GROUP_PARALLEL_ADD, [1000, 1, 1], [1, 1, 1]),
                                             (GROUP_AND_LOCAL_ADD, [16, 1, 1], [64, 1, 1])])
def test_kernels_parallelised_by_the_reference_run_as_written(hip, text, grid, block):
    """Kernels the reference's own suggesters have already parallelised carry group / local id
    parameters and their dispatch size (`src/opt/ast/suggesters/parallelization.rs:186-232`:
    one workgroup per iteration, then a local axis with a bounds check and a `ceil_div` grid
    size, evaluated as `src/backend/pipeline.rs:505-553` does).  They are launched with exactly
    that size, ids bound to blockIdx / threadIdx."""
    dev = hip.HipDevice(0)
    k = hip.HipKernel(dev, text)
    l, = k.launches
    assert l["schedule"] == "as-written" and l["grid"] == grid and l["block"] == block
    rng = RNG(3)
    a, b = (rng.normal(0, 1, 1000).astype(np.float32) for _ in range(2))
    bufs = [dev.alloc(4000) for _ in range(3)]
    bufs[0].write_array(a)
    bufs[1].write_array(b)
    k.execute(bufs[:2], bufs[2:])
    assert np.array_equal(bufs[2].read_array(np.float32), a + b)


def test_concurrent_compile_and_execute(frontend, hip):
    """Four threads share one device handle; each compiles its own programs and runs them on
    its own buffers while the others do the same (ctypes drops the interpreter lock inside
    every call).  Every result must equal the single-threaded one."""
    import threading
    from harp_amd import measure, workloads as wl
    dev = hip.HipDevice(0)
    jobs = []
    for i in range(4):                      # lowering shares front-end counters: do it up front
        shape = (200 + 37 * i, 96 + 8 * i)
        x = RNG(i).normal(0, 1, shape).astype(np.float32)
        ast, names, out, consts, _ = wl.lower_with_table([shape], lambda t: frontend.nn.softmax(t * t, 1))
        e = np.exp((x * x) - (x * x).max(1, keepdims=True))
        jobs.append((ast, names, out, consts, x, e / e.sum(1, keepdims=True)))
    errors = []

    def work(job):
        ast, names, out, consts, x, want = job
        try:
            for _ in range(3):
                prog = hip.HipProgram(dev, ast, None)
                (binding, named), = measure.make_sets(dev, prog, names, consts, [x], 1)
                for _ in range(10):
                    prog.run(binding, sync=True)
                got = named[out].read_array(np.float32, want.shape)
                if not np.allclose(got, want, rtol=1e-5, atol=1e-7):
                    errors.append("wrong result")
        except Exception as exc:            # noqa: BLE001 - reported below
            errors.append(repr(exc))

    threads = [threading.Thread(target=work, args=(j,)) for j in jobs]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors


def test_corrupt_disk_cache_entry_is_replaced(frontend, hip, tmp_path, monkeypatch):
    """A code object in the disk cache that does not load (truncated file) is compiled afresh
    and overwritten instead of failing every later run."""
    import os
    import subprocess
    import sys
    code = (
        "import sys, os, numpy as np\n"
        "sys.path.insert(0, %r)\n"
        "from harp_amd import backend as hb, workloads as wl\n"
        "ast, names, out, consts, _ = wl.lower_with_table([(64, 96)], lambda t: t * t + t)\n"
        "dev = hb.HipDevice(0)\n"
        "prog = hb.HipProgram(dev, ast, None)\n"
        "x = np.arange(64 * 96, dtype=np.float32).reshape(64, 96) / 100\n"
        "b = dev.alloc(x.nbytes); b.write_array(x)\n"
        "res = prog.execute({names[0]: b})[out].read_array(np.float32, x.shape)\n"
        "assert np.array_equal(res, x * x + x)\n"
        "print('ok')\n") % os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, HARP_CACHE_DIR=str(tmp_path))
    env.pop("HARP_NO_DISK_CACHE", None)
    run = lambda: subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=120)
    first = run()
    assert first.returncode == 0, first.stderr
    bins = [os.path.join(dp, f) for dp, _, fs in os.walk(tmp_path) for f in fs if f.endswith(".bin")]
    assert bins, "nothing was cached"
    sizes = {}
    for path in bins:
        sizes[path] = os.path.getsize(path)
        with open(path, "r+b") as f:
            f.truncate(100)
    second = run()                                     # fresh process: only the disk cache is left
    assert second.returncode == 0, second.stderr
    assert all(os.path.getsize(p) == n for p, n in sizes.items())


def test_c_client_runs_the_known_answer(hip):
    """The plain-C client (tests/capi_client.c, built with the library) computes the
    reference's [1,2,3,4] + [5,6,7,8] through the C ABI alone, from the compiled program and
    again from its binary."""
    import os
    import subprocess
    from harp_amd import build as hb_build
    exe = hb_build.CLIENT if os.path.exists(hb_build.CLIENT) else hb_build.build_capi_client()
    r = subprocess.run([exe, "run"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    assert "run ok" in r.stdout


TRANSPOSING = {
    "transpose_2d_ragged": ((300, 500), lambda t: t.permute([1, 0]).contiguous()),
    "swap_last_two_of_three": ((9, 130, 70), lambda t: t.permute([0, 2, 1]).contiguous()),
    "transpose_plus_aligned": ((257, 257), lambda t: (t.permute([1, 0]) + t) * t),
    "rotate_three_axes": ((40, 64, 96), lambda t: t.permute([2, 0, 1]).contiguous()),
    # the contiguous axes are pairs of loops here: (h, w) of the operand, (h, w) of the output
    "nchw_to_nhwc": ((9, 40, 14, 14), lambda t: t.permute([0, 2, 3, 1]).contiguous()),
    "nhwc_to_nchw_relu": ((9, 14, 14, 40), lambda t: t.permute([0, 3, 1, 2]).maximum(t.permute([0, 3, 1, 2]) * t.permute([0, 3, 1, 2]))),
}


@pytest.mark.parametrize("name", sorted(TRANSPOSING))
def test_transposing_copies_through_lds_tiles(frontend, hip, name):
    """Elementwise kernels whose operand is contiguous along a row loop of the output take the
    64x64 tile schedule (coalesced on both sides); bit-exact with the oracle, ragged edges
    included, and identical with the schedule switched off."""
    shape, fn = TRANSPOSING[name]
    x = RNG(len(name)).normal(0, 1, shape).astype(np.float32)
    t = frontend.Tensor.input(list(shape))
    prog, _, _ = frontend.lower_graph([fn(t).graph])
    assert any(l["schedule"].startswith("transpose(") for l in hip.render_program(prog).launches)
    assert not any(l["schedule"].startswith("transpose(")
                   for l in hip.render_program(prog, {"transpose": 0}).launches)
    for fuse in (True, False):
        ref, got = both(frontend, fn, [x], fuse)
        assert bits_equal_mod_zero(ref, got), (name, fuse)


def test_buffer_roundtrip_and_size_check(hip):
    dev = hip.HipDevice(0)
    from harp_amd.frontend import F32
    buf = hip.HipBuffer(dev, [5, 3], F32)
    assert buf.read_array(np.float32).tolist() == [0.0] * 15            # zero-filled
    data = np.arange(15, dtype=np.float32)
    buf.write_from_host(data.tobytes())
    assert np.array_equal(buf.read_array(np.float32), data)
    clone = buf.clone_buffer()
    assert np.array_equal(clone.read_array(np.float32), data)
    with pytest.raises(hip.EhError) as e:
        buf.write_from_host(b"\0" * 8)
    assert "Buffer size mismatch" in str(e.value)
    assert dev.props["arch"].startswith("gfx9") and dev.props["warp_size"] == 64


def test_released_memory_is_reused_and_zero_filled(hip):
    """A released buffer's block serves the next allocation of the same size; the new buffer
    is zero-filled all the same.  Trimming hands the kept blocks back."""
    dev = hip.HipDevice(0)
    dev.trim()
    n = 1 << 20
    a = dev.alloc(n)
    a.write_array(np.full(n, 0xAB, np.uint8))
    ptr = a.device_ptr()
    del a
    b = dev.alloc(n)
    assert b.device_ptr() == ptr
    assert not b.read_array(np.uint8).any()
    c = dev.alloc(n)                      # b still lives: another block
    assert c.device_ptr() != ptr
    del b, c
    assert dev.trim() == 2 * n and dev.trim() == 0


def test_a_new_buffer_reads_as_zeros_whenever_its_fill_happens(frontend, hip):
    """The zero fill of a new buffer is put off until its contents are needed.  On recycled
    memory full of 0xAB: a kernel that writes every element cancels the fill (and is right), a
    kernel that reads the buffer or writes only part of it gets zeros first, a read or a copy
    before any write gives zeros, and an execute that fails before its launch leaves a buffer
    that still reads as zeros."""
    dev = hip.HipDevice(0)
    F32 = frontend.F32
    n = 64 * 64

    def dirty(count=4):
        bufs = [dev.alloc(4 * n) for _ in range(count)]
        for b in bufs:
            b.write_array(np.full(4 * n, 0xAB, np.uint8))
        del bufs                                            # back to the pool, contents kept

    a = frontend.Tensor.input([64, 64])
    prog, _, _ = frontend.lower_graph([(a + a).graph])
    k = hip.HipKernel(dev, prog)
    assert [l["overwrites"] for l in hip.render_program(prog).launches] == [[False, True]]
    x = hip.HipBuffer(dev, [64, 64], F32)
    data = RNG(7).normal(0, 1, (64, 64)).astype(np.float32)
    x.write_array(data)
    dirty()
    out = hip.HipBuffer(dev, [64, 64], F32)
    k.execute([x], [out])                                   # overwrites all of `out`: no fill
    assert np.array_equal(out.read_array(np.float32), (data + data).ravel())
    dirty()
    fresh = hip.HipBuffer(dev, [64, 64], F32)
    out2 = hip.HipBuffer(dev, [64, 64], F32)
    k.execute([fresh], [out2])                              # reads a buffer nothing wrote: zeros
    assert not out2.read_array(np.float32).any() and not fresh.read_array(np.float32).any()
    dirty()
    never = hip.HipBuffer(dev, [64, 64], F32)
    assert not never.read_array(np.float32).any()           # read before any write
    assert not never.clone_buffer().read_array(np.float32).any()
    dirty()
    big = hip.HipBuffer(dev, [2 * n], F32)                  # larger than the kernel's output: only half is written
    k.execute([x], [big])
    got = big.read_array(np.float32)
    assert np.array_equal(got[:n], (data + data).ravel()) and not got[n:].any()
    dirty()
    out3 = hip.HipBuffer(dev, [64, 64], F32)
    with pytest.raises(hip.EhError):
        k.execute([hip.HipBuffer(dev, [16], F32)], [out3])  # refused before the launch
    assert not out3.read_array(np.float32).any()
    dirty()
    handed_out = hip.HipBuffer(dev, [64, 64], F32)          # asking for the address queues the fill
    assert handed_out.device_ptr() and not handed_out.read_array(np.float32).any()


def test_undersized_buffer_is_rejected_before_launch(frontend, hip):
    dev = hip.HipDevice(0)
    a = frontend.Tensor.input([64, 64])
    prog, _, _ = frontend.lower_graph([(a + a).graph])
    k = hip.HipKernel(dev, prog)
    small = hip.HipBuffer(dev, [16], frontend.F32)
    full = hip.HipBuffer(dev, [64, 64], frontend.F32)
    with pytest.raises(hip.EhError) as e:
        k.execute([small], [full])
    assert "Buffer size mismatch" in str(e.value)
    with pytest.raises(hip.EhError):
        k.execute([full, full], [full])                      # wrong argument count


def test_kernel_binary_round_trip(frontend, hip):
    dev = hip.HipDevice(0)
    a = frontend.Tensor.input([256])
    prog, _, _ = frontend.lower_graph([(a * a).graph])
    k = hip.HipKernel(dev, prog)
    blob = k.get_binary()
    assert blob[:4] == b"\x7fELF" and len(blob) > 1000
    # compile_from_binary: load the code object again and launch it with explicit sizes
    l = k.launches[0]
    mod = hip.HipModule(dev, blob, l["entry"])
    x = np.arange(256, dtype=np.float32)
    src, dst = hip.HipBuffer(dev, [256], frontend.F32), hip.HipBuffer(dev, [256], frontend.F32)
    src.write_array(x)
    mod.launch(l["grid"], l["block"], [src, dst])
    assert np.array_equal(dst.read_array(np.float32), x * x)
    with pytest.raises(hip.EhError):
        hip.HipModule(dev, b"not a code object", "k")
    with pytest.raises(hip.EhError):
        hip.HipModule(dev, blob, "no_such_entry")


def _train_step_on(fe, kind, arrays, fuse=True):
    """Config 4 graph (forward, MSE, exact backward, SGD update) realized with one
    execute_graph call; returns [new parameters..., loss] as flat arrays."""
    import os
    from harp_amd import workloads as wl
    from harp_amd.frontend.tensor import _INPUT_BUFFER_CACHE
    fe.set_device_str(kind)
    old = os.environ.get("ECLAT_HIP_FUSE")
    os.environ["ECLAT_HIP_FUSE"] = "1" if fuse else "0"
    try:
        with fe.exact_mode():
            ts = []
            for a in arrays:
                t = fe.Tensor.input(list(a.shape))
                t.set_data(a)
                ts.append(t)
            roots = wl.config4_graph(*ts)
            fe.realize_many(roots)
            return [r.to_numpy() for r in roots]
    finally:
        _INPUT_BUFFER_CACHE.clear()
        if old is None:
            os.environ.pop("ECLAT_HIP_FUSE", None)
        else:
            os.environ["ECLAT_HIP_FUSE"] = old


@pytest.mark.parametrize("batch,dims", [(64, (32, 64, 64, 32)), (256, (128, 256, 128, 128)), (50, (12, 20, 12))])
@pytest.mark.parametrize("fuse", [False, True])
def test_config4_mlp_training_step(frontend, hip, batch, dims, fuse):
    """benchmark configuration 4 at oracle-sized shapes: every updated parameter and the loss match
    the C oracle running the same graph; the step also matches a float64 numpy MLP."""
    from harp_amd import workloads as wl
    arrays = wl.config4_inputs(batch, dims, seed=99)
    if dims[0] != dims[-1]:
        arrays[1] = arrays[1][:, :dims[-1]]
    ref = _train_step_on(frontend, "c", arrays)
    got = _train_step_on(frontend, "hip", arrays, fuse)
    for r, g, a in zip(ref, got, arrays[2:] + [np.zeros(1, np.float32)]):
        assert r.shape == g.shape
        # gradients are sums over the batch of products: reduction class, scaled by |param|+lr*|grad|
        assert np.allclose(g, r, rtol=1e-5, atol=1e-6 * max(1.0, float(np.abs(r).max())))
    # numpy float64 reference of the whole step
    x, t = arrays[0].astype(np.float64), arrays[1].astype(np.float64)
    ps = [p.astype(np.float64) for p in arrays[2:]]
    hs, pre = [x], []
    nl = len(ps) // 2
    for i in range(nl):
        z = hs[-1] @ ps[2 * i].T + ps[2 * i + 1]
        pre.append(z)
        hs.append(np.tanh(z) if i + 1 < nl else z)
    d = hs[-1] - t
    loss = (d * d).mean()
    gz = 2 * d / d.size
    grads = [None] * len(ps)
    for i in range(nl - 1, -1, -1):
        grads[2 * i] = gz.T @ hs[i]
        grads[2 * i + 1] = gz.sum(0)
        if i > 0:
            gz = (gz @ ps[2 * i]) * (1 - np.tanh(pre[i - 1]) ** 2)
    assert abs(float(got[-1][0]) - loss) <= 1e-4 * abs(loss)
    for p, gr, g in zip(ps, grads, got[:-1]):
        assert np.allclose(g.reshape(p.shape), p - 1e-3 * gr, rtol=1e-4, atol=1e-6)


def test_compiled_step_fed_back_matches_eager_steps(frontend, hip):
    """`CompiledStep` lowers and compiles the MLP step once and is then called three times with
    its own outputs (the updated parameters, still on the device) as the next inputs; the
    oracle runs the same three steps through the eager path, re-lowering each time."""
    from harp_amd import workloads as wl
    from harp_amd.step import CompiledStep
    arrays = wl.config4_inputs(64, (32, 64, 64, 32), seed=5)
    step = CompiledStep(lambda *ts: wl.config4_graph(*ts, lr=0.05), [a.shape for a in arrays])
    assert len(step.launches) < step.lowered_kernels // 2
    bufs = [step.upload(a) for a in arrays]
    ref_arrays = list(arrays)
    for _ in range(3):
        outs = step(*bufs)
        bufs = bufs[:2] + outs[:-1]
        frontend.set_device_str("c")
        ref = _train_step_with_lr(frontend, ref_arrays, 0.05)
        ref_arrays = ref_arrays[:2] + [r.reshape(a.shape) for r, a in zip(ref[:-1], arrays[2:])]
        got_loss = float(outs[-1].read_array(np.float32)[0])
        assert abs(got_loss - float(ref[-1][0])) <= 1e-5 * abs(float(ref[-1][0]))
    for b, r in zip(bufs[2:], ref_arrays[2:]):
        assert np.allclose(b.read_array(np.float32, r.shape), r, rtol=1e-4, atol=1e-6)
    with pytest.raises(ValueError):
        step(*bufs[:-1])
    with pytest.raises(ValueError):
        step(*(bufs[:-1] + [bufs[0]]))                  # wrong size for the last parameter


def _train_step_with_lr(fe, arrays, lr):
    from harp_amd import workloads as wl
    from harp_amd.frontend.tensor import _INPUT_BUFFER_CACHE
    try:
        with fe.exact_mode():
            ts = []
            for a in arrays:
                t = fe.Tensor.input(list(a.shape))
                t.set_data(a)
                ts.append(t)
            roots = wl.config4_graph(*ts, lr=lr)
            fe.realize_many(roots)
            return [r.to_numpy() for r in roots]
    finally:
        _INPUT_BUFFER_CACHE.clear()


def _cnn_step_on(fe, kind, arrays, fuse=True, lr=None):
    import os
    from harp_amd import workloads as wl
    from harp_amd.frontend.tensor import _INPUT_BUFFER_CACHE
    fe.set_device_str(kind)
    old = os.environ.get("ECLAT_HIP_FUSE")
    os.environ["ECLAT_HIP_FUSE"] = "1" if fuse else "0"
    try:
        with fe.exact_mode():
            ts = []
            for a in arrays:
                t = fe.Tensor.input(list(a.shape))
                t.set_data(a)
                ts.append(t)
            roots = wl.config5_graph(*ts, lr=lr)
            fe.realize_many(roots)
            return [r.to_numpy() for r in roots]
    finally:
        _INPUT_BUFFER_CACHE.clear()
        if old is None:
            os.environ.pop("ECLAT_HIP_FUSE", None)
        else:
            os.environ["ECLAT_HIP_FUSE"] = old


@pytest.mark.parametrize("sizes", [(4, 8, 4, 8, 16, 10), (8, 28, 32, 64, 128, 10)])
@pytest.mark.parametrize("fuse", [False, True])
def test_config5_cnn_training_step(frontend, hip, sizes, fuse):
    """benchmark configuration 5 (second case: the real channel/image sizes at batch 8): every
    parameter gradient and the loss match the C oracle running the same exact-mode graph,
    and a float64 numpy CNN."""
    from harp_amd import workloads as wl
    from harp_amd.checks import cnn_step
    arrays = wl.config5_inputs(*sizes, seed=77)
    ref = _cnn_step_on(frontend, "c", arrays)
    got = _cnn_step_on(frontend, "hip", arrays, fuse)
    loss, grads = cnn_step(arrays[0], arrays[1], arrays[2:])
    assert abs(float(got[-1][0]) - float(ref[-1][0])) <= 1e-5 * abs(float(ref[-1][0]))
    assert abs(float(got[-1][0]) - loss) <= 1e-5 * abs(loss)
    for g, r, n in zip(got[:-1], ref[:-1], grads):
        scale = max(float(np.abs(r).max()), 1e-6)
        assert np.allclose(g, r, rtol=1e-4, atol=1e-5 * scale)
        assert np.allclose(g.reshape(n.shape), n, rtol=1e-3, atol=1e-5 * scale)


def test_config5_cnn_step_with_sgd_update(frontend, hip):
    """The form the benchmark times: the same step with p - lr * gradient for every parameter
    as the roots (the updates ride on the gradient contractions where they can)."""
    from harp_amd import workloads as wl
    from harp_amd.checks import cnn_step
    arrays = wl.config5_inputs(8, 28, 32, 64, 128, 10, seed=78)
    ref = _cnn_step_on(frontend, "c", arrays, lr=0.05)
    got = _cnn_step_on(frontend, "hip", arrays, lr=0.05)
    loss, grads = cnn_step(arrays[0], arrays[1], arrays[2:])
    assert abs(float(got[-1][0]) - loss) <= 1e-5 * abs(loss)
    for g, r, p, n in zip(got[:-1], ref[:-1], arrays[2:], grads):
        assert np.allclose(g, r, rtol=1e-5, atol=1e-6)
        assert np.allclose(g.reshape(p.shape), p - 0.05 * n, rtol=1e-4, atol=1e-6)


def _run_program(fe, hb, graph_fn, arrays, options=None):
    """Lowers graph_fn with a buffer table, compiles it as one HIP program with `options`,
    runs it and returns (flat result, launch schedules)."""
    from harp_amd import workloads as wl
    dev = hb.HipDevice(0)
    prog_ast, arg_names, out, consts, _ = wl.lower_with_table([a.shape for a in arrays], graph_fn)
    prog = hb.HipProgram(dev, prog_ast, options)
    named = {}
    for name, a in zip(arg_names, arrays):
        b = hb.HipBuffer(dev, list(a.shape), fe.F32)
        b.write_array(np.ascontiguousarray(a))
        named[name] = b
    for b in prog.buffers:
        if b["name"] in consts and not b["elided"]:
            cb = hb.HipBuffer(dev, [b["bytes"] // 4], fe.F32)
            cb.write_array(np.full(b["bytes"] // 4, 0.0 if consts[b["name"]] == "zeros" else 1.0, np.float32))
            named[b["name"]] = cb
    outs = prog.execute(named)
    return outs[out].read_array(np.float32), [l["schedule"] for l in prog.launches]


def _contract(fe, kind):
    """Contractions as the front end writes them (unsqueeze/expand, multiply, sum)."""
    if kind == "matmul":                      # a [M,K] @ b [K,N]
        return lambda a, b: fe.nn.matmul(a, b)
    if kind == "linear":                      # x [B,K] . w [O,K]
        return lambda x, w: fe.nn.linear(x, w)
    if kind == "rows3d":                      # x [G,R,K] . w [O,K] -> [G,R,O]: (G,R) walk as one axis
        return lambda x, w: (x.unsqueeze(2) * w.unsqueeze(0).unsqueeze(0)).sum(3)
    if kind == "per_group":                   # g [G,R,O], c [G,R,K] -> [G,O,K], reduce over R
        return lambda g, c: (g.unsqueeze(3) * c.unsqueeze(2)).sum(1)
    raise KeyError(kind)


CONTRACTIONS = [
    # kind, shapes, options, expected in schedule
    ("matmul", [(100, 60), (60, 36)], None, "edges"),
    ("matmul", [(70, 50), (50, 30)], None, "/scalar"),
    ("matmul", [(64, 2048), (2048, 64)], None, "split-k="),
    ("matmul", [(96, 1000), (1000, 40)], None, "split-k="),
    ("matmul", [(256, 512), (512, 256)], {"gemm_split_k": 3}, "split-k=3"),
    ("matmul", [(256, 64), (64, 128)], {"gemm_dma": 1}, "B>lds"),
    ("per_group", [(3, 64, 64), (3, 64, 128)], {"gemm_dma": 1}, "A>lds,B>lds"),
    ("matmul", [(192, 160), (160, 320)], {"gemm_bm": 128, "gemm_bn": 128, "gemm_bk": 16, "gemm_wm": 64, "gemm_wn": 64}, "tile=128x128x16"),
    ("matmul", [(192, 160), (160, 320)], {"gemm_transpose": 1}, "mfma"),
    ("per_group", [(3, 64, 64), (3, 64, 128)], {"gemm_transpose": 1, "gemm_prefetch": 1}, "mfma"),
    ("matmul", [(256, 512), (512, 256)], {"gemm_prefetch": 3, "gemm_bm": 128, "gemm_bn": 128, "gemm_bk": 16, "gemm_wm": 64, "gemm_wn": 64}, "tile=128x128x16"),
    ("linear", [(130, 72), (50, 72)], None, "edges"),
    ("linear", [(33, 18), (7, 18)], None, "/scalar"),
    ("rows3d", [(6, 50, 36), (20, 36)], None, "mfma"),
    ("rows3d", [(4, 49, 288), (64, 288)], None, "mfma"),
    ("per_group", [(6, 50, 20), (6, 50, 36)], None, "mfma"),
    ("per_group", [(3, 196, 64), (3, 196, 288)], None, "mfma"),
]


@pytest.mark.parametrize("kind,shapes,options,expect", CONTRACTIONS)
def test_contraction_variants_on_mfma(frontend, hip, kind, shapes, options, expect):
    """Ragged sizes, operands that cannot be read as 128-bit vectors, K split over
    workgroups, row axes that merge, and per-group contractions all take the MFMA schedule
    and match the C oracle (sum order differs: reduction tolerance) and float64 numpy."""
    rng = RNG(sum(sum(s) for s in shapes))
    arrays = [rng.uniform(-1, 1, s).astype(np.float32) for s in shapes]
    fn = _contract(frontend, kind)
    got, scheds = _run_program(frontend, hip, fn, arrays, options)
    assert any(s.startswith("mfma32x32x2(") and expect in s for s in scheds), scheds
    ref = realize_on(frontend, "c", fn, arrays)
    a64 = [a.astype(np.float64) for a in arrays]
    if kind == "matmul":
        exact, scale = a64[0] @ a64[1], np.abs(a64[0]) @ np.abs(a64[1])
    elif kind == "linear":
        exact, scale = a64[0] @ a64[1].T, np.abs(a64[0]) @ np.abs(a64[1]).T
    elif kind == "rows3d":
        exact, scale = a64[0] @ a64[1].T, np.abs(a64[0]) @ np.abs(a64[1]).T
    else:
        exact = np.einsum("gro,grk->gok", a64[0], a64[1])
        scale = np.einsum("gro,grk->gok", np.abs(a64[0]), np.abs(a64[1]))
    assert got.shape == ref.shape == (exact.size,)
    assert np.all(np.abs(got - ref) <= 1e-5 * scale.ravel() + 1e-30)
    assert np.all(np.abs(got - exact.ravel()) <= 1e-5 * scale.ravel() + 1e-30)


@pytest.mark.parametrize("shapes,options,expect", [
    ([(5, 50, 36), (20, 36), (20,)], None, "C:split"),
    ([(3, 50, 2048), (24, 2048), (24,)], None, "split-k="),
    ([(3, 50, 2048), (24, 2048), (24,)], {"gemm_split_k": 4}, "split-k=4"),
    ([(4, 196, 72), (64, 72), (64,)], None, "C:split"),
])
def test_contraction_rows_across_groups_into_a_permuted_result(frontend, hip, shapes, options, expect):
    """x [G,R,K] . w [O,K] written as [G,O,R] with a bias per O (a convolution's NCHW output): R
    is no multiple of the tile, so (G,R) is one row axis of the contraction and only the
    result's address keeps the two extents; with K split the summing launch computes that
    address.  Against the C oracle and float64 numpy."""
    rng = RNG(sum(sum(s) for s in shapes))
    arrays = [rng.uniform(-1, 1, s).astype(np.float32) for s in shapes]

    def fn(x, w, b):
        y = (x.unsqueeze(2) * w.unsqueeze(0).unsqueeze(0)).sum(3)
        return y.permute([0, 2, 1]).contiguous() + b.unsqueeze(0).unsqueeze(2)

    got, scheds = _run_program(frontend, hip, fn, arrays, options)
    assert any(s.startswith("mfma32x32x2(") and "C:split" in s and expect in s for s in scheds), scheds
    assert len(scheds) == (2 if "split-k" in expect else 1), scheds
    ref = realize_on(frontend, "c", fn, arrays)
    a64 = [a.astype(np.float64) for a in arrays]
    exact = np.einsum("grk,ok->gor", a64[0], a64[1]) + a64[2][None, :, None]
    scale = np.einsum("grk,ok->gor", np.abs(a64[0]), np.abs(a64[1])) + np.abs(a64[2])[None, :, None]
    assert got.shape == ref.shape == (exact.size,)
    assert np.all(np.abs(got - ref) <= 1e-5 * scale.ravel() + 1e-30)
    assert np.all(np.abs(got - exact.ravel()) <= 1e-5 * scale.ravel() + 1e-30)


@pytest.mark.parametrize("shape", [(64, 32, 14, 14), (40, 32, 7, 5), (33, 64, 28, 28)])
def test_bias_gradient_chain_matches_the_oracle(frontend, hip, shape):
    """b - lr * sum over (columns, rows, batch) of x: the sums over columns and rows run as one sum
    along memory and the update in the launch that finishes the sum over the batch; against the
    oracle's kernel-by-kernel result (reduction tolerance) and float64 numpy."""
    from test_host_cpu import _bias_gradient_step
    rng = RNG(sum(shape))
    arrays = [rng.normal(0, 1, shape).astype(np.float32), rng.normal(0, 1, shape[1]).astype(np.float32),
              np.full(shape[1], 0.01, np.float32)]
    got, scheds = _run_program(frontend, hip, _bias_gradient_step, arrays)
    assert len(scheds) == 2 and "epilogue=2" in scheds[1], scheds
    ref = realize_on(frontend, "c", _bias_gradient_step, arrays)
    exact = arrays[1].astype(np.float64) - arrays[0].astype(np.float64).sum((0, 2, 3)) * 0.01
    scale = np.abs(arrays[0]).astype(np.float64).sum((0, 2, 3)) * 0.01 + np.abs(arrays[1])
    assert np.all(np.abs(got - ref) <= 1e-5 * scale) and np.all(np.abs(got - exact) <= 1e-5 * scale)


def _independent_roots(a, b, c, d, e):
    """Three results over different index spaces that have nothing to do with each other, and a
    column sum that needs the first."""
    x = a * b + a
    y = (c - d).maximum(d)
    z = e.sum(1)
    return [x, y, z, x.sum(0)]


def test_independent_launches_issued_together_match_the_oracle(frontend, hip):
    """Roots that do not depend on each other become one launch (each part with its own range of
    workgroups and its own grid-stride loop, several iterations per work-item at this size); the
    root that needs one of them follows.  Bit-exact against the oracle for the elementwise
    roots, reduction tolerance for the sums; merge_launches=0 plans them one by one."""
    import os
    from harp_amd import workloads as wl
    from harp_amd.frontend.tensor import _INPUT_BUFFER_CACHE
    shapes = [(1500, 1024), (1500, 1024), (1100, 2048), (1100, 2048), (700, 512)]
    rng = RNG(77)
    arrays = [rng.normal(0, 1, s).astype(np.float32) for s in shapes]
    ts = [frontend.Tensor.input(list(s)) for s in shapes]
    ast = wl.lower_multi(ts, _independent_roots(*ts))[0]
    plan = hip.render_program(ast)
    apart = hip.render_program(ast, {"merge_launches": 0})
    together = [l for l in plan.launches if l["schedule"].startswith("together(")]
    assert len(together) == 1 and together[0]["schedule"].count("flat(") == 2 and len(plan.launches) < len(apart.launches), \
        [l["schedule"] for l in plan.launches]
    assert together[0]["grid"][0] > 500                      # real grid-stride loops, not one workgroup each

    def run(kind):
        frontend.set_device_str(kind)
        old = os.environ.get("ECLAT_HIP_FUSE")
        os.environ["ECLAT_HIP_FUSE"] = "1"
        try:
            tensors = []
            for a in arrays:
                t = frontend.Tensor.input(list(a.shape))
                t.set_data(a)
                tensors.append(t)
            roots = _independent_roots(*tensors)
            frontend.realize_many(roots)
            return [r.to_numpy() for r in roots]
        finally:
            _INPUT_BUFFER_CACHE.clear()
            if old is None:
                os.environ.pop("ECLAT_HIP_FUSE", None)
            else:
                os.environ["ECLAT_HIP_FUSE"] = old

    ref, got = run("c"), run("hip")
    for i in (0, 1):
        assert bits_equal_mod_zero(ref[i], got[i]), i
    assert np.all(np.abs(got[2].astype(np.float64) - ref[2]) <= 1e-5 * np.abs(arrays[4]).astype(np.float64).sum(1))
    x = np.abs(arrays[0] * arrays[1] + arrays[0]).astype(np.float64)
    assert np.all(np.abs(got[3].astype(np.float64) - ref[3]) <= 1e-5 * x.sum(0))


def test_config5_with_implicit_gemm_loader(frontend, hip):
    """im2col gathers and layout copies that only contractions read are evaluated inside the
    contractions' tile loaders (no launch, no buffer); option gemm_fold=0 materialises them.
    Same results either way."""
    from harp_amd import workloads as wl
    from harp_amd.frontend.device import _BACKENDS
    sizes = (8, 28, 32, 64, 128, 10)
    arrays = wl.config5_inputs(*sizes, seed=78)
    ts = [frontend.Tensor.input(list(a.shape)) for a in arrays]
    prog_ast = wl.lower_multi(ts, wl.config5_graph(*ts))[0]
    plain = hip.render_program(prog_ast, {"gemm_fold": 0})
    folded = hip.render_program(prog_ast)
    assert len(folded.launches) < len(plain.launches)
    assert sum("/folded" in l["schedule"] or "(window," in l["schedule"] for l in folded.launches) >= 3
    assert sum("(window," in l["schedule"] for l in folded.launches) >= 2
    assert not any("(window," in l["schedule"] for l in hip.render_program(prog_ast, {"gemm_window": 0}).launches)
    assert sum(b["elided"] for b in folded.buffers) > sum(b["elided"] for b in plain.buffers)
    ref = _cnn_step_on(frontend, "c", arrays)
    reg = _BACKENDS["hip"]
    old = reg.options
    reg.options = {"gemm_fold": 0}
    try:
        got_plain = _cnn_step_on(frontend, "hip", arrays, True)
    finally:
        reg.options = old
    got = _cnn_step_on(frontend, "hip", arrays, True)
    for g, p in zip(got, got_plain):
        assert np.allclose(g, p, rtol=1e-4, atol=1e-7)
    # the gathers evaluated per element in the tile loader instead of staged in LDS: same sums in another order
    reg.options = {"gemm_window": 0}
    try:
        got_loader = _cnn_step_on(frontend, "hip", arrays, True)
    finally:
        reg.options = old
    for g, p in zip(got, got_loader):
        assert np.allclose(g, p, rtol=1e-4, atol=1e-7)
    # guarded reads (padding) through a buffer resource, out of range where the guard fails
    # (default), or at a clamped index with a select behind them (ranged_loads=0): same bits
    # (in the plan without the LDS-staged schedules: there the shifted sums of the input gradient are a kernel of their own)
    assert any("eh_ranged_load(eh_rs_" in l["source"] for l in hip.render_program(prog_ast, {"gemm_window": 0}).launches)
    assert not any("eh_ranged_load" in l["source"]
                   for l in hip.render_program(prog_ast, {"ranged_loads": 0, "gemm_window": 0}).launches)
    reg.options = {"ranged_loads": 0, "gemm_window": 0}
    try:
        got_clamped = _cnn_step_on(frontend, "hip", arrays, True)
    finally:
        reg.options = old
    for g, c in zip(got_loader, got_clamped):
        assert np.array_equal(g, c)
    # option gemm_merge_batch=1: per-image weight-gradient contractions and the sum over images
    # that follows become one contraction with the batch folded into k
    merged = hip.render_program(prog_ast, {"gemm_merge_batch": 1})
    assert [l["entry"] for l in merged.launches] != [l["entry"] for l in folded.launches]
    assert sum(l["grid"][2] > 1 for l in merged.launches) < sum(l["grid"][2] > 1 for l in folded.launches)   # no per-image contractions left
    reg.options = {"gemm_merge_batch": 1}
    try:
        got_merged = _cnn_step_on(frontend, "hip", arrays, True)
    finally:
        reg.options = old
    for g, r in zip(got_merged[:-1], ref[:-1]):
        scale = max(float(np.abs(r).max()), 1e-6)
        assert np.allclose(g, r, rtol=1e-4, atol=1e-5 * scale)
    assert abs(float(got[-1][0]) - float(ref[-1][0])) <= 1e-5 * abs(float(ref[-1][0]))
    for g, r in zip(got[:-1], ref[:-1]):
        scale = max(float(np.abs(r).max()), 1e-6)
        assert np.allclose(g, r, rtol=1e-4, atol=1e-5 * scale)


def test_measured_option_search(frontend, hip, tmp_path, monkeypatch):
    """One expansion of the beam search on a 512^3 matmul: every proposed state compiles or is
    rejected cleanly, the winner is no slower than the defaults, and it computes the same C.  The
    result is filed, and a compile under ECLAT_HIP_TUNE plans the program with it."""
    from harp_amd import tune
    from harp_amd import workloads as wl
    msgs = []
    saved = tmp_path / "tuned.txt"
    best, cost, history = tune.tune_config("config3_matmul", shapes=[(512, 512), (512, 512)],
                                           beam_width=2, max_steps=1, steps=10, log=msgs.append, save=str(saved))
    ast = wl.lower_with_table([(512, 512), (512, 512)], wl.config3_graph)[0]
    assert saved.read_text().startswith(hip.tune_key(ast) + " ")
    monkeypatch.setenv("ECLAT_HIP_TUNE", str(saved))
    filed = [l["schedule"] for l in hip.render_program(ast).launches]
    monkeypatch.delenv("ECLAT_HIP_TUNE")
    assert filed == [l["schedule"] for l in hip.render_program(ast, dict(best) or None).launches]
    assert len(history) > 5 and history[0][1] == ""
    assert cost <= history[0][2] * 1.02 and np.isfinite(cost)
    rng = RNG(5)
    a = rng.uniform(-1, 1, (512, 512)).astype(np.float32)
    b = rng.uniform(-1, 1, (512, 512)).astype(np.float32)
    got, scheds = _run_program(frontend, hip, lambda x, y: frontend.nn.matmul(x, y), [a, b], dict(best) or None)
    exact = a.astype(np.float64) @ b.astype(np.float64)
    scale = np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64)
    assert np.all(np.abs(got.reshape(512, 512) - exact) <= 1e-5 * scale)


SPREAD_FORMS = {
    # name: (shape, graph, schedule expected somewhere in the plan, sums keep the oracle's order)
    "cumsum_rows": ((300, 257), lambda t: t.cumsum(1), "outer-parallel(work-items=300)"),
    # as lowered, the accumulator of a mid-axis scan runs on over the inner axis too: only axis 0 is free
    "cumprod_mid": ((6, 50, 9), lambda t: t.cumprod(1), "outer-parallel(work-items=6)"),
    "cummax_rows": ((128, 300), lambda t: t.cummax(1), "outer-parallel(work-items=128)"),
    # lines of 512 elements and more get a workgroup each: tiles of 1024, carry between tiles
    "cummax_long": ((128, 1000), lambda t: t.cummax(1), "scan-row(lines=128,length=1000)"),
    "cumsum_long": ((37, 5000), lambda t: t.cumsum(1), "scan-row(lines=37,length=5000)"),
    "cumprod_long": ((8, 3001), lambda t: t.cumprod(1), "scan-row(lines=8,length=3001)"),
    "cumsum_mid_long": ((3, 200, 9), lambda t: t.cumsum(1), "scan-row(lines=3,length=1800)"),
    # a scan over axis 0 is lowered with one accumulator for the whole tensor: one long line
    "cummax_axis0": ((300, 50), lambda t: t.cummax(0), "scan-row(lines=1,length=15000)"),
    "fold_tiles": ((64, 96), lambda t: t.unfold([0, 1], [2, 3], [2, 3], [1, 1])
                   .fold([64, 96], [0, 1], [2, 3], [2, 3], [1, 1]), "outer-parallel(work-items=6144)"),
    "fold_overlapping": ((20, 30), lambda t: t.unfold([0, 1], [3, 3], [1, 1], [1, 1])
                         .fold([20, 30], [0, 1], [3, 3], [1, 1], [1, 1]), "outer-parallel(work-items=4536,atomics)"),
    "fold_overlapping_large": ((300, 500), lambda t: t.unfold([0, 1], [3, 3], [1, 1], [1, 1])
                               .fold([300, 500], [0, 1], [3, 3], [1, 1], [1, 1]),
                               "outer-parallel(work-items=1335636,atomics)"),
}


@pytest.mark.parametrize("name", sorted(SPREAD_FORMS))
def test_scan_and_scatter_kernels_spread_over_work_items(frontend, hip, name):
    """Prefix scans run one work-item per scanned line, scatter-adds one per window element:
    bit-exact with the oracle where every sum keeps the sequential order; running sums and
    products, and the atomic additions of overlapping windows (whose order is open), are held
    to the reduction tolerance, as everywhere."""
    shape, fn, expect = SPREAD_FORMS[name]
    lo, hi = (0.995, 1.005) if name == "cumprod_long" else (0.5, 1.5)      # a long product must stay finite
    x = RNG(len(name)).uniform(lo, hi, shape).astype(np.float32)
    t = frontend.Tensor.input(list(shape))
    prog, _, _ = frontend.lower_graph([fn(t).graph])
    scheds = [l["schedule"] for l in hip.render_program(prog).launches]
    assert expect in scheds, scheds
    ref, got = both(frontend, fn, [x], False)
    if name.startswith(("cumsum", "cumprod", "fold_overlapping")):   # order of the additions is open: reduction class
        assert np.allclose(got, ref, rtol=1e-5 if name.endswith("_long") else 1e-6)
        if name == "cumsum_long":
            assert np.allclose(got.reshape(shape), np.cumsum(x.astype(np.float64), 1), rtol=1e-5)
    else:
        assert bits_equal_mod_zero(ref, got)


@pytest.mark.parametrize("shapes,family", [(((1, 1000), (1000, 3000)), "-reduce("), (((3000, 1000), (1000, 1)), "row("),
                                           (((1, 4096), (4096, 512)), "-reduce(")])
def test_vector_times_matrix_follows_the_matrix_layout(frontend, hip, shapes, family):
    """x[1,K] @ W[K,N]: the vector is contiguous along the reduce axis but the matrix, which is
    all the traffic, is contiguous along the outputs, so the contraction is scheduled as a
    reduce over a non-contiguous axis (coalesced rows of W); W[N,K] @ x[K,1] stays a row reduce."""
    from harp_amd import workloads as wl
    fn = lambda a, b: frontend.nn.matmul(a, b)
    scheds = [l["schedule"] for l in hip.render_program(wl.lower_with_table(list(shapes), fn)[0]).launches]
    assert scheds[0].split("(")[0] + "(" in (family, "split" + family, "column" + family, "serial" + family), scheds
    rng = RNG(sum(shapes[0]))
    a = rng.uniform(-1, 1, shapes[0]).astype(np.float32)
    b = rng.uniform(-1, 1, shapes[1]).astype(np.float32)
    ref, got = both(frontend, fn, [a, b], True)
    exact = (a.astype(np.float64) @ b.astype(np.float64)).ravel()
    scale = (np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64)).ravel()
    assert np.all(np.abs(got.ravel() - exact) <= 1e-5 * scale)
    assert np.all(np.abs(ref.ravel() - exact) <= 1e-5 * scale)


CONVS_AS_WRITTEN = {
    # name: (input shape, weight shape, graph)
    "3x3_pad1": ((3, 5, 12, 10), (7, 5, 3, 3), lambda nn, x, w: nn.conv2d(x, w, None, (1, 1), (1, 1))),
    "1x1": ((2, 16, 9, 9), (8, 16, 1, 1), lambda nn, x, w: nn.conv2d(x, w)),
    "5x5_stride2": ((2, 3, 21, 19), (6, 3, 5, 5), lambda nn, x, w: nn.conv2d(x, w, None, (2, 2), (2, 2))),
    "conv1d_k5": ((4, 6, 100), (9, 6, 5), lambda nn, x, w: nn.conv1d(x, w)),
    "3x3_64ch": ((2, 64, 14, 14), (64, 64, 3, 3), lambda nn, x, w: nn.conv2d(x, w, None, (1, 1), (1, 1))),
}


@pytest.mark.parametrize("name", sorted(CONVS_AS_WRITTEN))
def test_convolution_as_the_reference_lowers_it_has_no_gather_launch(frontend, hip, name):
    """As the reference lowers a convolution, the unfold view is applied twice: a gather writes
    the windows, a second gather reads that buffer through the same view, the contraction
    reads the second.  Both gathers are evaluated in the contraction's tile loader (the first
    as a device function the second calls) and neither buffer exists; results equal the
    oracle's, which runs the three kernels, and the per-kernel HIP path's."""
    from harp_amd import workloads as wl
    xs, ws, graph = CONVS_AS_WRITTEN[name]
    fn = lambda x, w: graph(frontend.nn, x, w)
    plan = hip.render_program(wl.lower_with_table([xs, ws], fn)[0])
    assert len(plan.launches) <= 2 and "/folded" in plan.launches[0]["schedule"], [l["schedule"] for l in plan.launches]
    assert all(l["schedule"].startswith(("mfma", "split-k-final")) for l in plan.launches)
    assert sum(b["elided"] for b in plan.buffers) == 2 and "eh_win_" in plan.launches[0]["source"]
    rng = RNG(len(name))
    x = rng.uniform(-1, 1, xs).astype(np.float32)
    w = rng.uniform(-1, 1, ws).astype(np.float32)
    ref, got = both(frontend, fn, [x, w], True)
    off = realize_on(frontend, "hip", fn, [x, w], fuse=False)
    scale = max(1.0, float(np.abs(ref).max()))
    assert np.allclose(got, ref, rtol=1e-5, atol=1e-5 * scale) and np.allclose(got, off, rtol=1e-5, atol=1e-5 * scale)


POOLS = {
    # name: (input shape, graph, exact mode, numpy statement or None)
    "max2": ((3, 5, 12, 16), lambda nn, t: nn.max_pool2d(t, (2, 2)), True,
             lambda x: x.reshape(3, 5, 6, 2, 8, 2).max((3, 5))),
    "max2_as_written": ((3, 5, 12, 16), lambda nn, t: nn.max_pool2d(t, (2, 2)), False, None),
    "max3s2p1": ((2, 4, 15, 13), lambda nn, t: nn.max_pool2d(t, (3, 3), (2, 2), (1, 1)), True, None),
    "max3s1d2": ((2, 3, 17, 17), lambda nn, t: nn.max_pool2d(t, (3, 3), (1, 1), (0, 0), (2, 2)), True, None),
    "avg2": ((4, 3, 10, 14), lambda nn, t: nn.avg_pool2d(t, (2, 2), exact=True), True,
             lambda x: x.reshape(4, 3, 5, 2, 7, 2).mean((3, 5))),
    "avg3s2p1": ((2, 3, 9, 9), lambda nn, t: nn.avg_pool2d(t, (3, 3), (2, 2), (1, 1), exact=True), True, None),
    "avg3s2p1_as_written": ((2, 3, 9, 9), lambda nn, t: nn.avg_pool2d(t, (3, 3), (2, 2), (1, 1)), False, None),
}


@pytest.mark.parametrize("name", sorted(POOLS))
def test_pooling_reads_its_windows_from_the_source(frontend, hip, name):
    """Pooling is lowered as unfold (a gather that lays the windows out), sometimes a copy, then a
    short reduce over the window axis (src/tensor/nn/pool.rs:146-160 in the reference).  With a
    buffer table the reduce reads the source through the gathers' index maps, one work-item
    per output, and the window buffers are never written; results match the oracle, which
    runs the kernels as lowered, and numpy where the case has a closed form."""
    from harp_amd import workloads as wl
    import contextlib
    shape, graph, exact, closed = POOLS[name]
    fn = lambda t: graph(frontend.nn, t)
    with (frontend.exact_mode() if exact else contextlib.nullcontext()):
        plan = hip.render_program(wl.lower_with_table([shape], fn)[0])
        scheds = [l["schedule"] for l in plan.launches]
        assert any(s.startswith("window-reduce(") for s in scheds), scheds
        win = [l for l in plan.launches if l["schedule"].startswith("window-reduce(")][0]
        elided = {b["name"] for b in plan.buffers if b["elided"]}
        assert len(elided) == len(win["kernels"]) - 1 and not elided & set(win["args"])
        x = RNG(len(name)).uniform(-2, 2, shape).astype(np.float32)
        ref, got = both(frontend, fn, [x], True)
        off = realize_on(frontend, "hip", fn, [x], fuse=False)
    if "max" in name:
        assert bits_equal_mod_zero(ref, got) and bits_equal_mod_zero(off, got)
    else:
        assert np.allclose(got, ref, rtol=1e-5, atol=1e-6) and np.allclose(got, off, rtol=1e-5, atol=1e-6)
    if closed is not None:
        assert np.allclose(got, closed(x.astype(np.float64)).ravel(), rtol=1e-5, atol=1e-6)


LONG_LINES = {
    # name: (shape, graph, float64 statement of the same, entry of the kernel that cuts the lines)
    "sum_4x10M": ((4, 10_000_000), lambda t: t.sum(1), lambda x: x.sum(1), "row"),
    "sum_all_16M": ((1 << 24,), lambda t: t.sum(0), lambda x: x.sum(0, keepdims=True), "row"),
    "max_2x4M": ((2, 1 << 22), lambda t: t.max(1), lambda x: x.max(1), "row"),
    "min_3x2x2M": ((3, 2, 1 << 21), lambda t: t.min(2), lambda x: x.min(2), "row"),
    "mean_sq_2x3M": ((2, 3 << 20), lambda t: (t * t).sum(1), lambda x: (x * x).sum(1), "row"),
    "max_32x256k": ((32, 1 << 18), lambda t: t.max(1), lambda x: x.max(1), "row"),
    "sum_8x300k": ((8, 300_000), lambda t: t.sum(1), lambda x: x.sum(1), "row"),
}


@pytest.mark.parametrize("name", sorted(LONG_LINES))
def test_few_very_long_reduce_lines_are_cut_over_workgroups(frontend, hip, name):
    """A reduce with a handful of lines of millions of elements is planned as two reduces (pieces
    of a line, then the pieces): max and min stay bit-exact with the oracle; a sum is held to
    the reduction tolerance against float64, since the oracle's own sequential float32 sum of
    10^7 terms is only good to about 1e-4."""
    from harp_amd import workloads as wl
    shape, fn, exact_fn, sched = LONG_LINES[name]
    launches = hip.render_program(wl.lower_with_table([shape], fn)[0]).launches
    cut = [l for l in launches if l["entry"].endswith("_rows")]
    assert len(cut) == 1 and cut[0]["schedule"].startswith(sched) and cut[0]["grid"][0] >= 128, launches
    x = RNG(len(name)).uniform(-1.0, 1.5, shape).astype(np.float32)
    ref, got = both(frontend, fn, [x], True)
    if name.startswith(("max", "min")):
        assert bits_equal_mod_zero(ref, got)
        return
    x64 = x.astype(np.float64)
    exact, scale = exact_fn(x64).ravel(), exact_fn(np.abs(x64)).ravel()
    assert np.all(np.abs(got.ravel() - exact) <= 1e-5 * scale)
    assert np.all(np.abs(ref.ravel() - exact) <= 1e-3 * scale)


LONG_SCANS = {
    # name: (shape, graph, float64 statement, schedule of the scanning launch)
    "cummax_axis0": ((2048, 512), lambda t: t.cummax(0), None, "scan-row(lines=1,length=1048576,chunks=256)"),
    "cumsum_ragged": ((3, 700001), lambda t: t.cumsum(1), lambda x: np.cumsum(x, 1), "scan-row(lines=3,length=700001,chunks=171)"),
    "cumsum_2x1M": ((2, 1 << 20), lambda t: (t * t).cumsum(1), lambda x: np.cumsum(x * x, 1), "scan-row(lines=2,length=1048576,chunks=256)"),
    "cumsum_100x20k": ((100, 20_000), lambda t: t.cumsum(1), lambda x: np.cumsum(x, 1), "scan-row(lines=100,length=20000,chunks=5)"),
    "cummax_mid_7x3000x11": ((7, 3000, 11), lambda t: t.cummax(1), None, "scan-row(lines=7,length=33000,chunks=9)"),
    "cumprod_1x600k": ((1, 600_000), lambda t: t.cumprod(1), lambda x: np.cumprod(x, 1), "scan-row(lines=1,length=600000,chunks=147)"),
}


@pytest.mark.parametrize("name", sorted(LONG_SCANS))
def test_few_very_long_scan_lines_are_cut_over_workgroups(frontend, hip, name):
    """A prefix scan with a handful of lines of a million elements: a first launch totals chunks
    of whole tiles, the scanning launch starts every chunk from the totals ahead of it.  Max is
    bit-exact with the oracle; sums and products are held to the reduction tolerance against
    float64 (the oracle's sequential float32 scan over 10^6 terms is itself only good to about 1e-4)."""
    from harp_amd import workloads as wl
    shape, fn, exact_fn, sched = LONG_SCANS[name]
    launches = hip.render_program(wl.lower_with_table([shape], fn)[0]).launches
    scheds = [l["schedule"] for l in launches]
    assert sched in scheds and any(s.startswith("scan-row-totals(") for s in scheds), scheds
    x = RNG(len(name)).uniform(-1.0, 1.5, shape).astype(np.float32)
    if name.startswith("cumprod"):
        x = np.exp(RNG(len(name)).uniform(-0.05, 0.05, shape)).astype(np.float32)
    ref, got = both(frontend, fn, [x], True)
    if exact_fn is None:
        assert bits_equal_mod_zero(ref, got)
        return
    x64 = x.astype(np.float64)
    exact, scale = exact_fn(x64).ravel(), exact_fn(np.abs(x64)).ravel()
    if name.startswith("cumprod"):
        # every rounding of a product reaches the result at full weight, whatever the order:
        # n roundings of 2^-24 each walk to about sqrt(n) * 2^-24 on either side
        bound = 8 * np.sqrt(x.size) * 2.0 ** -24
        assert np.all(np.abs(got.ravel() - exact) <= bound * scale)
        assert np.all(np.abs(ref.ravel() - exact) <= bound * scale)
        return
    assert np.all(np.abs(got.ravel() - exact) <= 1e-5 * scale)
    assert np.all(np.abs(ref.ravel() - exact) <= 1e-3 * scale)


def test_scratch_temps_of_a_plan_may_be_left_unbound(frontend, hip):
    """A plan may append scratch temps to the caller's buffer table (the pieces of cut lines);
    through the C ABI the caller may bind its own entries only, or all of them."""
    import ctypes
    from harp_amd import workloads as wl
    from harp_amd._lib import lib, check
    shape = (4, 300_000)
    x = RNG(11).uniform(-1, 1, shape).astype(np.float32)
    ast, names, out, consts, _ = wl.lower_with_table([shape], lambda t: t.max(1))
    dev = hip.HipDevice(0)
    prog = hip.HipProgram(dev, ast, None)
    assert [b["name"].startswith("eh_rowpart_") for b in prog.buffers] == [False, False, True]
    xin, res = dev.alloc(x.nbytes), dev.alloc(16)
    xin.write_array(x)
    by_name = {names[0]: xin, out: res}
    for n in (2, 3):
        arr = (ctypes.c_void_p * n)()
        for i in range(2):
            arr[i] = by_name[prog.buffers[i]["name"]]._h
        check(lib.eh_program_execute(prog._h, arr, n, 1))
        assert np.array_equal(res.read_array(np.float32), x.max(1))
    arr = (ctypes.c_void_p * 1)()
    arr[0] = xin._h
    with pytest.raises(Exception, match="binds 3 buffers, 1 given"):
        check(lib.eh_program_execute(prog._h, arr, 1, 1))


def test_softmax_over_two_rows_of_millions(frontend, hip):
    """Row softmax whose rows are too long for one workgroup each: every reduce in it is cut."""
    shape = (2, 1 << 22)
    x = RNG(77).uniform(-3, 3, shape).astype(np.float32)
    fn = lambda t: frontend.nn.softmax(t, 1)
    ref, got = both(frontend, fn, [x], True)
    e = np.exp(x.astype(np.float64) - x.max(1, keepdims=True))
    exact = e / e.sum(1, keepdims=True)
    assert np.allclose(got.reshape(shape), exact, rtol=1e-5, atol=0)
    assert np.allclose(ref.reshape(shape), exact, rtol=1e-3, atol=0)


def _held_to_error_bounds(frontend, seed, desc, fn, fn64, arrays, fuses=(True,)):
    """HIP against the oracle and against float64, per element, by what float32 rounding can do to
    the graph (tests/np_frontend.py): two float32 evaluations may differ by twice the bound."""
    import np_frontend
    exact, bound = np_frontend.evaluate(fn64, arrays)
    for fuse in fuses:
        ref, got = both(frontend, fn, arrays, fuse)
        assert ref.shape == got.shape and ref.size == exact.size, desc
        exact, bound = exact.reshape(ref.shape), bound.reshape(ref.shape)
        tol = 2.0 * bound + 4 * np_frontend.U * np.abs(exact)
        assert np.all(np.abs(got.astype(np.float64) - ref) <= tol), (desc, fuse, float(np.max(np.abs(got.astype(np.float64) - ref) / tol)))
        assert np.all(np.abs(got.astype(np.float64) - exact) <= 0.5 * tol + 2 * np_frontend.U * np.abs(exact)), (desc, fuse)


@pytest.mark.parametrize("seed", list(range(64)) + [1211])
def test_random_graphs_match_the_oracle(frontend, hip, seed):
    """Differential test on seeded random graphs (tests/graph_fuzz.py): elementwise chains,
    views, reductions over any axis, row normalisations, small contractions.  Held per element to
    the running error bound of a float64 evaluation of the same graph: seed 1211 ends in an
    element of 0.0033 that the graph computes as a difference of values near one -- the oracle is
    3.7e-6 off the float64 value there, more than a relative 2e-5 plus 2e-6 allows either side,
    and the bound says 1.3e-4 is what float32 can do."""
    import graph_fuzz, np_frontend
    shapes, fn, desc = graph_fuzz.build(seed, frontend)
    _, fn64, _ = graph_fuzz.build(seed, np_frontend.Frontend)
    rng = RNG(seed)
    arrays = [rng.uniform(-1.5, 1.5, s).astype(np.float32) for s in shapes]
    _held_to_error_bounds(frontend, seed, desc, fn, fn64, arrays)


@pytest.mark.parametrize("seed", range(600, 624))
def test_random_graphs_with_scans_selects_and_windows(frontend, hip, seed):
    """The same generator ending in a prefix scan, a select on a comparison, sliding windows
    (unfold) or a batched contraction; small and large axes alternate."""
    import graph_fuzz
    large = seed % 2 == 1
    shapes, fn, desc = graph_fuzz.build(seed, frontend, kinds=(8, 12),
                                        dims=graph_fuzz.LARGE_DIMS if large else graph_fuzz.SMALL_DIMS,
                                        max_rank=2 if large else 3)
    rng = RNG(seed)
    arrays = [rng.uniform(-1.5, 1.5, s).astype(np.float32) for s in shapes]
    # Lowered in exact mode: as the reference lowers it, a reader of a materialised unfold
    # indexes the window buffer with the unfold's input-space view and runs past its end
    # (`lower.rs:344-348` vs `:221-224`); the HIP backend refuses such a launch on the host.
    # A prefix sum near zero has lost the digits its terms cancelled: scans are held to the
    # size of the largest prefix instead.
    rtol = 2e-4 if "kind 8" in desc else 2e-5
    with frontend.exact_mode():
        for fuse in (True, False):
            ref, got = both(frontend, fn, arrays, fuse)
            assert ref.shape == got.shape, desc
            scale = max(1.0, float(np.abs(ref).max()))
            assert np.allclose(got, ref, rtol=rtol, atol=2e-6 * scale), (desc, fuse)


def test_out_of_bounds_reader_of_a_materialised_unfold_is_refused(frontend, hip):
    """Lowered as the reference does, max over sliding windows reads the contiguous window
    buffer [257,128,2] through the unfold's own view (row stride 257) and would run 255
    elements past its end; the launch is rejected on the host instead of faulting."""
    x = RNG(1).normal(0, 1, (257, 257)).astype(np.float32)
    with pytest.raises(hip.EhError, match="needs at least"):
        realize_on(frontend, "hip", lambda t: t.unfold([1], [2], [2], [1]).contiguous().max(2), [x])


@pytest.mark.parametrize("seed", range(5000, 5020))
def test_random_large_graphs_match_the_oracle(frontend, hip, seed):
    """The same generator with one or two axes of up to 2048 elements: vectorised accesses,
    rows held in registers or LDS, multi-block reductions, MFMA contractions with edges.
    The tolerance is per element and follows the arithmetic (tests/np_frontend.py: a float64
    evaluation of the same graph with a running bound on what float32 rounding can do to it,
    sums counted with their condition): two float32 evaluations may differ by twice the bound.
    A sum of 2048 values that nearly cancel (seed 5012: -0.30470 from terms of size 1) is judged
    by sum|x|, everything well conditioned more tightly than a fixed relative tolerance would."""
    import graph_fuzz, np_frontend
    shapes, fn, desc = graph_fuzz.build(seed, frontend, dims=graph_fuzz.LARGE_DIMS, max_rank=2)
    _, fn64, _ = graph_fuzz.build(seed, np_frontend.Frontend, dims=graph_fuzz.LARGE_DIMS, max_rank=2)
    rng = RNG(seed)
    arrays = [rng.uniform(-1.5, 1.5, s).astype(np.float32) for s in shapes]
    _held_to_error_bounds(frontend, seed, desc, fn, fn64, arrays, fuses=(True, False))


LONG_LINE_SEEDS = [(7007, 0), (7052, 0), (7084, 0), (7092, 0), (7229, 0), (7264, 0), (7282, 0), (7284, 0), (7296, 0),
                   (7024, 8), (7028, 8), (7087, 8), (7107, 8), (7154, 8), (7373, 8)]


@pytest.mark.parametrize("seed,first_kind", LONG_LINE_SEEDS)
def test_random_graphs_with_few_long_lines_match_the_oracle(frontend, hip, seed, first_kind):
    """The same generator over one to twenty lines of 40 000 or 300 000 elements, seeds chosen
    so that the plan cuts a reduce or a scan line over workgroups (totals, row normalisations,
    gathers before a reduce, prefix scans after elementwise chains)."""
    import graph_fuzz
    from harp_amd import workloads as wl
    dims = (1, 2, 3, 7, 20, 40000, 300000)
    with frontend.exact_mode():
        shapes, fn, desc = graph_fuzz.build(seed, frontend, dims=dims, max_rank=2, kinds=(first_kind, first_kind + (8 if first_kind == 0 else 4)))
        launches = hip.render_program(wl.lower_with_table(shapes, fn)[0]).launches
        assert any(l["entry"].endswith("_rows") or l["schedule"].startswith("scan-row-totals(") for l in launches), desc
        rng = RNG(seed)
        arrays = [rng.uniform(-1.5, 1.5, s).astype(np.float32) for s in shapes]
        rtol = 2e-4 if "kind 8" in desc else 2e-5
        for fuse in (True, False):
            ref, got = both(frontend, fn, arrays, fuse)
            assert ref.shape == got.shape, desc
            scale = max(1.0, float(np.abs(ref).max()))
            assert np.allclose(got, ref, rtol=rtol, atol=rtol / 10 * scale), (desc, fuse)


@pytest.mark.parametrize("seed", range(400, 420))
def test_random_small_cnns_match_the_oracle(frontend, hip, seed):
    """Random conv + pool + linear classifiers (tests/graph_fuzz.py): forward with the fused
    and the per-kernel path, then every gradient of the summed output in exact mode."""
    import graph_fuzz
    shapes, fn, desc = graph_fuzz.build_cnn(seed, frontend)
    rng = RNG(seed)
    arrays = [rng.uniform(-1, 1, s).astype(np.float32) for s in shapes]
    for fuse in (True, False):
        ref, got = both(frontend, fn, arrays, fuse)
        assert ref.shape == got.shape, desc
        assert np.allclose(got, ref, rtol=2e-5, atol=2e-5), (desc, fuse)
    ref = _grads_on(frontend, "c", shapes, fn, arrays)
    got = _grads_on(frontend, "hip", shapes, fn, arrays)
    assert ref is not None and len(ref) == len(got) == len(shapes) + 1, desc
    for r, g in zip(ref, got):
        assert r.shape == g.shape, desc
        scale = max(1.0, float(np.abs(r).max()))
        close = np.isclose(g, r, rtol=1e-4, atol=1e-5 * scale)
        # a relu or max-pool tie that falls differently moves one window's gradient
        assert int((~close).sum()) <= (2 if "pool True" in desc else 0), desc


CONV_DX_CASES = [((3, 8, 10, 12), (16, 8, 3, 3), (1, 1), (1, 1), 9),
                 ((2, 4, 9, 7), (8, 4, 5, 5), (2, 2), (1, 1), 25),
                 ((2, 6, 8, 8), (12, 6, 2, 2), (0, 0), (1, 1), 4),
                 ((2, 4, 6, 20), (8, 4, 1, 3), (0, 1), (1, 1), 3),
                 ((2, 32, 14, 14), (64, 32, 3, 3), (1, 1), (1, 1), 9),
                 ((5, 3, 10, 10), (8, 3, 3, 3), (0, 0), (1, 1), 9),
                 ((2, 4, 12, 12), (8, 4, 3, 3), (2, 2), (2, 2), 0),
                 ((1, 16, 30, 30), (8, 16, 3, 3), (1, 1), (1, 1), 9),
                 ((1, 64, 20, 20), (64, 64, 3, 3), (1, 1), (1, 1), 0)]


@pytest.mark.parametrize("xs,ws,pad,dil,shifts", CONV_DX_CASES)
def test_convolution_input_gradients_as_one_window_contraction(frontend, hip, xs, ws, pad, dil, shifts):
    """d/dx of sum(conv2d(x, w) * g): the product dY x W and the kernels that add up its shifted
    reads run as one window contraction (3x3, 5x5, 2x2 and 1x3 kernels, with and without
    padding; a dilated window and a weight tile too large for one workgroup's LDS keep the
    separate launches).  All three gradients and the loss against the oracle."""
    from harp_amd import workloads as wl
    fe = frontend

    def fn(x, w, g):
        return fe.nn.conv2d(x, w, None, padding=pad, dilation=dil) * g

    ho = xs[2] + 2 * pad[0] - dil[0] * (ws[2] - 1)
    wo = xs[3] + 2 * pad[1] - dil[1] * (ws[3] - 1)
    shapes = [xs, ws, (xs[0], ws[0], ho, wo)]
    with fe.exact_mode():
        ts = [fe.Tensor.input(list(sh)) for sh in shapes]
        loss = fn(*ts)
        while loss.ndim() > 0:
            loss = loss.sum(loss.ndim() - 1)
        loss.backward_with_params(ts)
        plan = hip.render_program(wl.lower_multi(ts[1:], [ts[0].grad().contiguous()])[0])
    fused = [l for l in plan.launches if "shifts=" in l["schedule"]]
    assert len(fused) == (1 if shifts else 0), [l["schedule"] for l in plan.launches]
    if shifts:
        assert fused[0]["schedule"].endswith(",shifts=%d)" % shifts)
    rng = RNG(sum(xs) + sum(ws))
    arrays = [rng.uniform(-1, 1, sh).astype(np.float32) for sh in shapes]
    ref = _grads_on(fe, "c", shapes, fn, arrays)
    got = _grads_on(fe, "hip", shapes, fn, arrays)
    assert ref is not None and len(ref) == len(got) == 4
    for r, g in zip(ref, got):
        assert r.shape == g.shape
        scale = max(1.0, float(np.abs(r).max()))
        assert np.allclose(g, r, rtol=1e-4, atol=1e-5 * scale)


@pytest.mark.parametrize("seed", range(430, 438))
def test_random_small_cnn_training_steps_match_the_oracle(frontend, hip, seed):
    """The same random classifiers as one SGD step: every input after `x - 0.05 * dloss/dx` and
    the loss, realized together (as many roots as inputs plus one)."""
    import graph_fuzz
    shapes, fn, desc = graph_fuzz.build_cnn(seed, frontend)
    rng = RNG(seed)
    arrays = [rng.uniform(-1, 1, s).astype(np.float32) for s in shapes]
    ref = _grads_on(frontend, "c", shapes, fn, arrays, lr=0.05)
    got = _grads_on(frontend, "hip", shapes, fn, arrays, lr=0.05)
    assert ref is not None and len(ref) == len(got) == len(shapes) + 1, desc
    for r, g in zip(ref, got):
        assert r.shape == g.shape, desc
        scale = max(1.0, float(np.abs(r).max()))
        close = np.isclose(g, r, rtol=1e-4, atol=1e-5 * scale)
        assert int((~close).sum()) <= (2 if "pool True" in desc else 0), desc


def _grads_on(fe, kind, shapes, fn, arrays, lr=None):
    """Exact-mode gradients of sum(fn(inputs)) with respect to every input, plus the sum,
    realized together (with `lr`: the inputs after a gradient step instead of the gradients).
    Returns None when the graph uses an op without an exact VJP."""
    from harp_amd.frontend.tensor import _INPUT_BUFFER_CACHE
    fe.set_device_str(kind)
    try:
        with fe.exact_mode():
            ts = []
            for a in arrays:
                t = fe.Tensor.input(list(a.shape))
                t.set_data(a)
                ts.append(t)
            loss = fn(*ts)
            while loss.ndim() > 0:
                loss = loss.sum(loss.ndim() - 1)
            try:
                loss.backward_with_params(ts)
            except NotImplementedError:
                return None
            if lr is None:
                roots = [t.grad().contiguous() for t in ts if t.grad() is not None] + [loss]
            else:
                roots = [(t - t.grad().scale_exact(lr)).contiguous() for t in ts if t.grad() is not None] + [loss]
            fe.realize_many(roots)
            return [r.to_numpy() for r in roots]
    finally:
        _INPUT_BUFFER_CACHE.clear()


@pytest.mark.parametrize("seed", list(range(200, 232)) + [392])
def test_random_graph_gradients_match_the_oracle(frontend, hip, seed):
    """The same random graphs, differentiated: loss = sum of the output, exact-mode VJPs,
    all gradients and the loss as roots of one Program.  HIP against the C oracle -- compiled
    with the reference's flags and -mno-recip (kind "c-exactdiv"): the gradient of a max / min
    tests a value for equality with its recomputation in another kernel, and gcc's vectorised
    reciprocal under -ffast-math breaks that equality inside the oracle itself (seed 392: eleven
    of 24 rows lose their gradient; tests/test_oracle_golden.py shows it without a GPU)."""
    import graph_fuzz
    shapes, fn, desc = graph_fuzz.build(seed, frontend)
    rng = RNG(seed)
    arrays = [rng.uniform(-1.5, 1.5, s).astype(np.float32) for s in shapes]
    ref = _grads_on(frontend, "c-exactdiv", shapes, fn, arrays)
    if ref is None:
        pytest.skip("graph uses an op without an exact VJP: " + desc)
    got = _grads_on(frontend, "hip", shapes, fn, arrays)
    assert len(ref) == len(got), desc
    for r, g in zip(ref, got):
        assert r.shape == g.shape, desc
        scale = max(1.0, float(np.abs(r).max()))
        close = np.isclose(g, r, rtol=1e-4, atol=1e-5 * scale)
        # the gradient of a max/min goes to the elements equal to it: where two candidates
        # differ by an ulp of sinf/exp2f on one side and tie on the other, one element's
        # gradient legitimately differs (the function is not differentiable there)
        allowed = 1 if ("(max)" in desc or "(min)" in desc) else 0
        assert int((~close).sum()) <= allowed, desc


@pytest.mark.parametrize("seed", sorted(set(range(22100, 22124)) | {22112, 22119, 23078}))
def test_random_gradients_of_graphs_with_scans_selects_and_windows(frontend, hip, seed):
    """The generator's other final stages (prefix scans, selects on comparisons, sliding windows,
    batched contractions), differentiated where exact VJPs exist.  Seeds 22112 and 22119: a reduce
    whose epilogue reads a buffer the reduce reads as well listed that buffer twice among its
    kernel's parameters, and the launch did not compile."""
    import graph_fuzz
    shapes, fn, desc = graph_fuzz.build(seed, frontend, kinds=(8, 12))
    rng = RNG(seed)
    arrays = [rng.uniform(-1.5, 1.5, s).astype(np.float32) for s in shapes]
    # HIP first: where a window buffer has two readers (the forward reduce and its gradient's
    # mask), the lowering -- the reference's, mirrored -- materialises the unfold contiguously and
    # lets the readers index it through the unfold's input-space view, past its end
    # (`lower.rs:344-348` vs `:221-224`).  The backend refuses such a launch on the host; the
    # oracle, like backend-c, would read out of bounds, so it is not run on such a program.
    try:
        got = _grads_on(frontend, "hip", shapes, fn, arrays)
    except hip.EhError as e:
        if "Buffer size mismatch" in str(e):
            pytest.skip("the lowered program reads a window buffer out of bounds and is refused: " + desc)
        raise
    if got is None:
        pytest.skip("graph uses an op without an exact VJP: " + desc)
    ref = _grads_on(frontend, "c-exactdiv", shapes, fn, arrays)
    assert len(ref) == len(got), desc
    for r, g in zip(ref, got):
        assert r.shape == g.shape, desc
        scale = max(1.0, float(np.abs(r).max()))
        assert np.allclose(g, r, rtol=2e-4, atol=2e-5 * scale), desc


def test_producers_read_through_another_index_space(frontend, hip):
    """A squared tensor, permuted, made contiguous and regrouped, feeding a kernel over the new
    axes: planned as one launch (the producers are evaluated where they are read), as three with
    reindex=0; both equal the oracle bit for bit (elementwise arithmetic only) and numpy."""
    from test_host_cpu import _regrouped_chain
    rng = RNG(77)
    x = rng.uniform(-2, 2, (8, 6, 4)).astype(np.float32)
    y = rng.uniform(-2, 2, (4, 12)).astype(np.float32)
    got, scheds = _run_program(frontend, hip, _regrouped_chain, [x, y])
    apart, scheds0 = _run_program(frontend, hip, _regrouped_chain, [x, y], "reindex=0")
    assert len(scheds) == 1 and len(scheds0) == 3
    ref = realize_on(frontend, "c", _regrouped_chain, [x, y])
    a = (x * x).transpose(2, 0, 1).reshape(4, 4, 12)
    want = (a * y[None] + a).ravel()
    assert np.array_equal(got, apart) and np.array_equal(got, ref)
    assert np.allclose(got, want, rtol=1e-6)


@pytest.mark.parametrize("threads", [16, 32, 64, 128, 256, 512, 1024])
def test_row_programs_with_every_thread_count(frontend, hip, threads):
    """Softmax and a fused relu-sum with the threads per row forced to each power of two the
    schedule takes: one wave or less per row (lane reductions), two waves per row with two rows in
    a workgroup (each row needs LDS slots of its own), and whole workgroups per row."""
    from harp_amd import workloads as wl
    rng = RNG(threads)
    x = rng.uniform(-4, 4, (96, 2048)).astype(np.float32)
    got, scheds = _run_program(frontend, hip, wl.config2_graph, [x], f"row_threads={threads}")
    assert f"row(T={min(threads, 512)}," in scheds[0], scheds
    e = np.exp(x.astype(np.float64) - x.max(1, keepdims=True))
    assert np.allclose(got.reshape(x.shape), e / e.sum(1, keepdims=True), rtol=1e-5, atol=1e-12)
    a, b, c = [rng.uniform(-1, 1, (200, 1024)).astype(np.float32) for _ in range(3)]
    got, scheds = _run_program(frontend, hip, wl.config1_graph, [a, b, c], f"row_threads={threads}")
    want = np.maximum(a.astype(np.float64) * b + c, 0).sum(1)
    assert np.allclose(got, want, rtol=1e-5, atol=1e-4)


def test_stored_value_read_back_by_a_later_reduction(frontend, hip):
    """The elementwise root and the row sums of the same expression (tests/test_host_cpu.py): with
    the stored value read back and with reindex=0, both against numpy."""
    from harp_amd import measure
    from harp_amd import workloads as wl
    from harp_amd.frontend import Tensor
    from test_host_cpu import _value_and_its_row_sums
    rng = RNG(5)
    x = rng.uniform(-1, 1, (64, 256)).astype(np.float32)
    m = rng.uniform(-1, 1, (64, 256)).astype(np.float32)
    dev = hip.HipDevice(0)
    ts = [Tensor.input([64, 256]), Tensor.input([64, 256])]
    ast, arg_names, outs, consts, _ = wl.lower_multi(ts, _value_and_its_row_sums(*ts))
    want = [(x * m + x).ravel(), (x.astype(np.float64) * m + x).sum(1)]
    for options in (None, "reindex=0"):
        prog = hip.HipProgram(dev, ast, options)
        (binding, named), = measure.make_sets(dev, prog, arg_names, consts, [x, m], 1)
        prog.run(binding, sync=True)
        got = [named[o].read_array(np.float32) for o in outs]
        assert np.array_equal(got[0], want[0])
        assert np.allclose(got[1], want[1], rtol=1e-5, atol=1e-5)
