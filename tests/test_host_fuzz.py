"""The AST reader, the normaliser and the planner under AddressSanitizer and
UndefinedBehaviorSanitizer (host code only, no GPU): every lowered and rewritten kernel of a set
of graphs goes through unharmed, and thousands of mutated texts -- bytes dropped and replaced,
atoms swapped for hostile ones (INT64 extremes, NaN bit patterns, wrong keywords), expressions
duplicated, the text cut short -- are either refused with an error or planned, never a crash, an
out-of-bounds read, a signed overflow or a planner that does not return."""

import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _corpus(fe):
    from harp_amd import workloads as wl
    from harp_amd.frontend import AstNode, optimize
    nn = fe.nn
    graphs = [
        ([(6, 23), (23,)], lambda a, b: a * b.unsqueeze(0).expand(0, 6) + a),
        ([(5, 37)], lambda a: (a * a).sum(1)),
        ([(9, 16)], lambda a: a.max(0)),
        ([(7, 19)], lambda a: nn.softmax(a, 1)),
        ([(10, 21), (21, 8)], lambda a, b: nn.matmul(a, b)),
        ([(4, 9, 8)], lambda a: a.permute([2, 0, 1]).contiguous() + a.permute([2, 0, 1])),
        ([(5, 11)], lambda a: a.pad([(1, 2), (3, 0)]) * a.pad([(1, 2), (3, 0)])),
        ([(4, 29)], lambda a: a.cumsum(1)),
        ([(4, 6)], lambda t: t.unfold([0, 1], [2, 2], [2, 2], [1, 1]).fold([4, 6], [0, 1], [2, 2], [2, 2], [1, 1])),
        ([(2, 3, 8, 8), (4, 3, 3, 3), (4,)],
         lambda x, w, b: nn.max_pool2d(nn.relu(nn.conv2d(x, w, b, padding=(1, 1))), (2, 2))),
    ]
    out = []
    for shapes, fn in graphs:
        table, _, _, _, plain = wl.lower_with_table(shapes, fn)
        out.append(table.to_sexpr())
        for k in plain.args:
            out.append(AstNode.program([k]).to_sexpr())
            for tf in (["tile=3"], ["guard=5", "unroll"], ["tile_all=2", "unroll"], ["interchange"]):
                out.append(optimize.optimize_kernel(k, tf).to_sexpr())
    # whole training steps (exact mode): many kernels behind one buffer table, which is what the
    # program-level passes work on (producers inlined through re-indexing, stored values read
    # back, transposed temps, epilogues, lanes)
    from harp_amd.frontend import Tensor
    steps = []
    for arrays, fn in ((wl.config5_inputs(2, 8, 4, 4, 8, 10), lambda *t: wl.config5_graph(*t, lr=1e-2)),
                       (wl.config4_inputs(8, [16, 32, 32, 16]), lambda *t: wl.config4_graph(*t, lr=1e-3))):
        ts = [Tensor.input(list(a.shape)) for a in arrays]
        steps.append(wl.lower_multi(ts, fn(*ts))[0].to_sexpr())
    # the reference's search drops candidates above 10 000 nodes (src/opt/ast/optimizer/beam_search.rs:67):
    # texts beyond that (a convolution unrolled at every level) are left out
    return [o for o in out if len(o) < 100_000] + steps


def test_reader_normaliser_and_planner_survive_mutated_asts_under_sanitizers(frontend, tmp_path):
    from harp_amd import build
    exe = build.build_host_fuzz()
    corpus = _corpus(frontend)
    assert len(corpus) > 100
    path = tmp_path / "corpus.txt"
    path.write_text("\n".join(corpus) + "\n")
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    r = subprocess.run([exe, str(path), "40", "20261125"], capture_output=True, text=True, timeout=900, env=env)
    assert r.returncode == 0, (r.stdout[-2000:], r.stderr[-6000:])
    last = r.stdout.strip().splitlines()[-1]
    assert last.startswith(f"host_fuzz: {len(corpus)} corpus entries") and last.endswith(" 0 odd"), last
    accepted, rejected = int(last.split()[4]), int(last.split()[7])
    assert accepted > 100 and rejected > 1000, last
