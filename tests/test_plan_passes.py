"""One plan test per pass of plan_program over the kernels in canonical form
(harp_amd/csrc/rewrites.cpp, run in this order by harp_amd/csrc/plan.cpp), on the CNN training
step of config 5 at benchmark size: what the pass does to the plan, and that switching it off
gives the plan without it.  No GPU involved: plans are made and their sources compiled."""
import pytest

pytestmark = []


@pytest.fixture(scope="module")
def cnn_ast(frontend):
    from harp_amd import workloads as wl
    from harp_amd.frontend import Tensor
    arrays = wl.config5_inputs(*wl.cnn_sizes(True))
    ts = [Tensor.input(list(a.shape)) for a in arrays]
    return wl.lower_multi(ts, wl.config5_graph(*ts, lr=1e-2))[0]


def _plan(ast, options=None):
    from harp_amd import backend as hb
    return hb.render_program(ast, options)


def _covering(plan, kernel):
    (l,) = [l for l in plan.launches if kernel in l["kernels"]]
    return l


def _gone(plan):
    return {b["name"] for b in plan.buffers if b["elided"]}


def test_move_elementwise_behind_producers(cnn_ast):
    """E_256_128_23 prepares the second fully connected layer's operand from the first layer's
    activation, but is lowered behind kernels of the loss (another root of the step): it moves
    up behind its producer and rides on the first layer's contraction with the rest of that
    chain.  Without re-indexing passes it stays where it was lowered, a launch of its own."""
    plan = _plan(cnn_ast)
    fc1 = _covering(plan, "E_256_128_23")
    assert "R_256_1_128_16" in fc1["kernels"] and "epilogue=4" in fc1["schedule"]
    off = _plan(cnn_ast, "reindex=0")
    assert "R_256_1_128_16" not in _covering(off, "E_256_128_23")["kernels"]


def test_merge_batch_sums_into_contractions(cnn_ast):
    """gemm_merge_batch=1: a convolution's weight gradient, lowered as one contraction per image
    and a sum over the images, becomes one contraction with the batch folded into k; the kernel
    that summed and the per-image results go."""
    plan = _plan(cnn_ast, "gemm_merge_batch=1,gemm_window=0")
    wg2 = [l for l in plan.launches if "R_256_1_64_288_88" in l["kernels"]][0]       # (K is split then: a part and a final launch)
    assert "R_1_1_64_288_89" in wg2["kernels"] and wg2["grid"][2] == 1 and "split-k=256" in wg2["schedule"]
    default = _plan(cnn_ast, "gemm_window=0")
    per_image = _covering(default, "R_256_1_64_288_88")
    assert "R_1_1_64_288_89" not in per_image["kernels"] and per_image["grid"][2] == 256
    assert len(_gone(plan)) > len(_gone(default))


def test_merge_sums_over_neighbouring_axes(cnn_ast):
    """A bias gradient is lowered as a sum over the image's columns, then its rows, then the
    batch.  The first two are one sum along memory: R_256_32_1_1_84 disappears into
    R_256_32_28_1_83 (and R_256_64_1_1_93 into R_256_64_14_1_92), with the buffer between."""
    plan = _plan(cnn_ast)
    for first, second in (("R_256_32_28_1_83", "R_256_32_1_1_84"), ("R_256_64_14_1_92", "R_256_64_1_1_93")):
        l = _covering(plan, first)
        assert second in l["kernels"]
        part = [s for s in l["schedule"].replace("together(", "").split(" + ") if s.startswith("row(")]
        assert part, l["schedule"]
    off = _plan(cnn_ast, "reindex=0")
    assert len(off.launches) > len(plan.launches) and len(_gone(off)) < len(_gone(plan))


def test_fold_gathers_into_contractions(cnn_ast):
    """The im2col gathers and the layout copies that only contractions read are not launched and
    their buffers never exist: the contractions evaluate them (staged in LDS, or in the tile
    loader with gemm_window=0).  gemm_fold=0 launches the gathers and keeps the buffers."""
    plan = _plan(cnn_ast)
    assert not any(l["kernels"][0].startswith("E_256_14_14_32_3_3") for l in plan.launches)
    assert "E_256_14_14_32_3_3_8" not in [k for l in plan.launches for k in l["kernels"]]
    off = _plan(cnn_ast, "gemm_fold=0")
    assert "E_256_14_14_32_3_3_8" in [k for l in off.launches for k in l["kernels"]]
    assert len(off.launches) > len(plan.launches) and len(_gone(off)) < len(_gone(plan))
    loader = _plan(cnn_ast, "gemm_window=0")
    assert any("/folded" in l["schedule"] or "B:source" in l["schedule"] or "A:source" in l["schedule"] for l in loader.launches)


def test_read_windows_through_their_gathers(cnn_ast):
    """Max pooling is lowered as unfold, copy, reduce over the window axis.  The reduce reads the
    convolution's output through the gathers' index maps: one launch, no window buffer.  What the
    gather reads is max(z, 0) of a pre-activation z that the backward pass needs anyway: the
    reduce applies that as well, and the convolution stores z only.  window=0 launches the
    gather; rematerialize=0 keeps the stored activation.  (gemm_tail=0: the pooling as a launch
    of its own.)"""
    plan = _plan(cnn_ast, "gemm_tail=0")
    pool = _covering(plan, "R_256_32_14_14_1_7")
    assert pool["kernels"][:3] == ["E_256_32_28_28_5", "E_256_32_14_14_2_2_6", "R_256_32_14_14_1_7"]
    assert "window-reduce(window=4,gathers=2)" in pool["schedule"] and "fmaxf(buf31[" in pool["source"]
    conv = _covering(plan, "R_256_784_32_1_1")
    assert "E_256_32_28_28_5" not in conv["kernels"] and sum(conv["written"]) == 1
    assert any(b["name"] == "buf37" and b["elided"] for b in plan.buffers)
    stored = _plan(cnn_ast, "rematerialize=0,gemm_tail=0")
    assert "E_256_32_28_28_5" in _covering(stored, "R_256_784_32_1_1")["kernels"]
    assert "window-reduce(window=4,gathers=1)" in _covering(stored, "R_256_32_14_14_1_7")["schedule"]
    off = _plan(cnn_ast, "window=0,gemm_tail=0")
    assert "E_256_32_14_14_2_2_6" not in _covering(off, "R_256_32_14_14_1_7")["kernels"]
    assert len(off.launches) > len(plan.launches)


def test_join_shifted_sums_with_their_contraction(cnn_ast):
    """The second convolution's input gradient: dY x W, then eight kernels adding up nine shifted,
    guarded reads of the product.  One window contraction over (channel, shift) covers all nine
    kernels; gemm_window=0 keeps the product and the sums apart."""
    plan = _plan(cnn_ast, "merge_templates=0,gemm_tail=0")
    dx = _covering(plan, "R_256_196_1_288_59")
    assert dx["kernels"][1:] == ["E_256_32_16_16_%d" % q for q in range(60, 68)] and "shifts=9" in dx["schedule"]
    off = _plan(cnn_ast, "gemm_window=0,merge_templates=0")
    assert _covering(off, "R_256_196_1_288_59")["kernels"] == ["R_256_196_1_288_59"]
    assert len(off.launches) == len(plan.launches) + 1


def test_issue_independent_contractions_together(cnn_ast):
    """A layer's input gradient and weight gradient are contractions that read the same dY and
    nothing of each other.  Each is an instance of a kernel template; compiled as parts (a device
    function of the launch's linear workgroup id and of the launch's one block of LDS) they go out
    as one launch, the longer part first: the second convolution's, and both fully connected
    layers'.  merge_templates=0 launches them one by one."""
    from harp_amd import backend as hb
    plan = _plan(cnn_ast)
    pairs = [l for l in plan.launches if l["schedule"].startswith("together(mfma")]
    assert [sorted(k for k in l["kernels"] if k.startswith("R_")) for l in pairs] == [
        ["R_1_128_10_103", "R_256_128_1_44"], ["R_1_3136_128_97", "R_256_3136_1_47"], ["R_256_196_1_288_59", "R_256_1_64_288_88"]]
    conv = pairs[2]
    assert conv["grid"] == [512, 1, 1] and conv["block"] == [256, 1, 1]
    src = conv["source"]
    assert src.count("#define EH_PART 1") == 2 and src.count("#undef EW_ENTRY") == 2
    assert "float eh_lds[eh_max2(eh_part0::eh_lds_floats, eh_max2(eh_part1::eh_lds_floats, 4))];" in src
    assert src.index("eh_part0::eh_run(blockIdx.x - 0u, eh_lds") < src.index("eh_part1::eh_run(blockIdx.x - 256u, eh_lds")
    assert len(hb.compile_source(src)) > 1000
    # split K over the second grid axis: the part decodes it from the linear id
    fc = pairs[1]
    assert "split-k=2" in fc["schedule"] and fc["grid"] == [196 + 98 * 2, 1, 1] and "#define EH_PART_GY 2u" in fc["source"]
    apart = _plan(cnn_ast, "merge_templates=0")
    assert len(apart.launches) == len(plan.launches) + 3 and not any(l["schedule"].startswith("together(mfma") for l in apart.launches)


def test_pooling_runs_in_the_convolution_launch(cnn_ast):
    """The pooling reduce reads the convolution's stored pre-activation through its gathers, and one
    image's pooled outputs read only that image's block, which is what one workgroup of the window
    schedule stores.  The reduce is offered to the contraction as a tail: the epilogue keeps the
    block in LDS as well (beside the tiles: 158 812 of 163 840 bytes for the second convolution),
    and behind a barrier that waits for LDS only the workgroup computes its image's pooled outputs.
    Two launches less; gemm_tail=0 keeps the poolings as launches."""
    from harp_amd import backend as hb
    plan = _plan(cnn_ast)
    for conv, pool, z, per_image, block in (("R_256_784_32_1_1", "R_256_32_14_14_1_7", "buf31", 6272, 25088),
                                            ("R_256_196_64_1_9", "R_256_64_7_7_1_15", "buf47", 3136, 12544)):
        l = _covering(plan, conv)
        assert l is _covering(plan, pool) and ",tail=window-reduce(window=4,gathers=2)" in l["schedule"]
        src = l["source"]
        assert "#define EH_TAIL_PER_GROUP %d\n" % per_image in src and "#define EH_TAIL_BLOCK %d\n" % block in src
        # every store of the pre-activation has its twin into LDS, and the tail reads LDS
        assert src.count("eh_tail_lds[eh_e - EH_TAIL_BASE] = eh_v_" + z) == 2
        assert src.count("*reinterpret_cast<EhQ<float>*>(eh_tail_lds + (eh_e - EH_TAIL_BASE))") == 1
        assert "fmaxf(%s[-(idx_t)EH_TAIL_BASE + " % z in src and "#define EH_TAIL_ARGS , eh_tail_lds, " in src
        assert int(l["schedule"].split("lds=")[1].split("B")[0]) <= 160 * 1024
        assert len(hb.compile_source(src)) > 1000
    apart = _plan(cnn_ast, "gemm_tail=0")
    assert len(apart.launches) == len(plan.launches) + 2 and not any(",tail=" in l["schedule"] for l in apart.launches)
