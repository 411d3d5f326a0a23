"""Host-side tests that need no GPU: the C ABI loads and exports what the headers
declare, misuse returns status codes (where the reference panics), layouts are
decoded on the host, and the fusion pass produces the kernels the reference's
rules produce.  They run on a plan-only device: kernels are generated and
JIT-compiled for gfx950 but nothing is launched and nothing is computed."""
import ctypes
import os
import re

import numpy as np
import pytest

from helpers import ROOT


def _declared_symbols():
    names = set()
    for header in ("wkf_hip.h", "wkf_tensor.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(wkf_[a-z0-9_]+)\s*\(", text))
    return names


def test_library_exports_every_declared_symbol(wkf):
    lib = ctypes.CDLL(wkf.LIB_PATH)
    declared = _declared_symbols()
    assert len(declared) > 60
    missing = [n for n in sorted(declared) if not hasattr(lib, n)]
    assert not missing, missing
    assert declared == set(wkf.EXPORTS), declared ^ set(wkf.EXPORTS)


def test_headers_cite_the_reference_interface():
    for header in ("wkf_hip.h", "wkf_tensor.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        assert len(re.findall(r"src/[a-z_/]+\.rs:\d+", text)) >= 15, header


def test_planner_device_props(planner):
    p = planner.props()
    assert planner.is_planner and p.ordinal == -1 and p.wave_size == 64 and p.arch == b"gfx950"


def test_leaf_roundtrip_and_host_side_view_decoding(wkf, planner):
    data = np.array([[1, 2], [3, 4], [5, 6]], dtype=np.float32)
    t = wkf.Tensor.new(planner, data)
    assert t.shape() == (3, 2) and t.rank() == 2 and t.datatype() == wkf.F32
    assert np.array_equal(t.to_numpy(), data)
    # test_tensor_slice, src/tensor.rs:646-666 of the reference: the whole buffer comes back, the view is decoded on the host
    s = t.slice([(0, 2), (0, 1)]).as_slice()
    assert s.shape == (2, 1) and s.strides == (2, 1) and s.offset == 0 and s.buffer.size == 6
    assert s[0, 0] == 1.0 and s[1, 0] == 3.0
    assert s.get([0, 1]) is None and s.get([1, 1]) is None and s.get([2, 0]) is None
    tr = t.transpose(0, 1).as_slice()
    assert tr.shape == (2, 3) and tr.strides == (1, 2)
    assert np.array_equal(tr.to_numpy(), data.T)
    b = wkf.Tensor.new(planner, np.array([[1, 2], [3, 4]], dtype=np.float32)).broadcast([2, 2, 3]).as_slice()
    assert b.shape == (2, 2, 3) and b.strides == (2, 1, 0)
    n = t.narrow(0, 1, 2).as_slice()
    assert n.offset == 2 and np.array_equal(n.to_numpy(), data[1:])
    # test_tensor_compare, src/tensor.rs:786-815
    cube = wkf.Tensor.new(planner, np.arange(24, dtype=np.float32).reshape(6, 2, 2))
    a = cube.slice([(0, 2), (0, 1), (0, 1)]).as_slice()
    assert a == a
    assert a != cube.slice([(0, 1), (0, 1), (0, 1)]).as_slice()
    assert a != cube.slice([(1, 3), (0, 1), (0, 1)]).as_slice()
    h = wkf.Tensor.new(planner, data.astype(np.float16))
    assert h.datatype() == wkf.F16 and np.array_equal(h.to_numpy(), data.astype(np.float16))


def test_computed_values_are_refused_without_a_gpu(wkf, planner):
    t = wkf.Tensor.new(planner, np.ones((4, 4), dtype=np.float32)) + 1.0
    t.materialize()  # planning and compiling is fine
    with pytest.raises(wkf.WkfError) as e:
        t.as_slice()
    assert e.value.code == 5 and "plan-only" in str(e.value)


def test_misuse_returns_status_codes(wkf, planner):
    T = wkf.Tensor
    a = T.new(planner, np.ones((3, 2), dtype=np.float32))
    b = T.new(planner, np.ones((2, 3), dtype=np.float32))
    h = T.new(planner, np.ones((3, 2), dtype=np.float16))
    cases = [
        lambda: a + b,                       # src/pair_wise.rs:92
        lambda: a + h,                       # dtype mismatch (a compile error in Rust)
        lambda: a.sum(2),                    # axis out of range
        lambda: a.mat_mul(a),                # src/matmul.rs:194
        lambda: a.narrow(0, 2, 2),           # src/composite/narrow.rs:6
        lambda: a.narrow(2, 0, 1),           # src/composite/narrow.rs:7
        lambda: a.broadcast([3, 2]),         # rank must grow by one
        lambda: a.broadcast([3, 5, 7]),      # src/map_layout.rs:78-79
        lambda: a.reshape([4, 2]),           # src/resize.rs:132-135
        lambda: a.slice([(0, 4), (0, 2)]),   # range outside the tensor
        lambda: a.slice_assign([(0, 2), (0, 2)], b),  # src/slice_assign.rs:69
        lambda: T.cat([a, b], 0),            # src/composite/cat.rs:12-19
        lambda: T.cat([a, a], 2),
        lambda: a.softmax(),                 # rank 1 only
        lambda: a.layer_norm(T.new(planner, np.ones(3, dtype=np.float32)), 1e-5),
        lambda: T.arange_step(planner, 0.0, 1.0, 0.0),
    ]
    for i, f in enumerate(cases):
        with pytest.raises(wkf.WkfError) as e:
            f()
        assert e.value.code == 3, (i, str(e.value))
    with pytest.raises(ValueError):
        T.new(planner, [[1.0, 2.0], [3.0]])  # ragged input: the reference panics in IntoTensor
    with pytest.raises(wkf.WkfError):
        wkf.Device.new(99)
    # level 0: an argument block cut short of its tail padding would reach the kernel without its last member
    lib = wkf.load()
    k = ctypes.c_void_p()
    src = b'struct Args { float* p; unsigned n; }; extern "C" __global__ void k0(const Args a) { if (a.n) a.p[0] = 1.0f; }'
    assert lib.wkf_module_get(planner._h, b"test|unpadded args", src, b"k0", ctypes.byref(k)) == 0, lib.wkf_last_error()
    one = (ctypes.c_uint32 * 3)(1, 1, 1)
    assert lib.wkf_launch(planner._h, k, one, one, 0, bytes(12), 12, None) == 3
    assert b"multiple of 8" in lib.wkf_last_error()
    assert lib.wkf_launch(planner._h, k, one, one, 0, bytes(16), 16, None) == 0


def test_layout_view_algebra(wkf, planner):
    # test_contiguous, src/layout.rs:96-102
    layout = wkf.Layout.contiguous([2, 3])
    assert (layout.offset(), layout.shape(), layout.strides(), layout.rank()) == (0, (2, 3), (3, 1), 2)
    assert layout.is_contiguous()
    assert not layout.slice([range(0, 1), range(0, 1)]).is_contiguous()   # strides (3, 1) are not those of a [1, 1] tensor
    assert not layout.slice([range(1, 2), range(0, 3)]).is_contiguous()   # offset 3
    # slice keeps the strides, moves the offset and takes the range lengths as the shape (src/layout.rs:15-31,62-71)
    cube = wkf.Layout.contiguous([4, 5, 6])
    assert cube.strides() == (30, 6, 1)
    view = cube.slice([(1, 3), (2, 5), (0, 6)])
    assert (view.offset(), view.shape(), view.strides()) == (30 + 12, (2, 3, 6), (30, 6, 1))
    again = view.slice([(1, 2), (1, 3), (4, 6)])                             # ranges are relative to the view
    assert (again.offset(), again.shape()) == (42 + 30 + 6 + 4, (1, 2, 2))
    # whole-range slices of a contiguous layout stay contiguous; a leading-dimension prefix does too
    assert cube.slice([(0, 4), (0, 5), (0, 6)]).is_contiguous()
    assert cube.slice([(0, 2), (0, 5), (0, 6)]).is_contiguous()
    assert not cube.slice([(0, 4), (0, 4), (0, 6)]).is_contiguous()
    # from_parts takes anything; transposed and broadcast strides are not contiguous, rank 0 is
    assert not wkf.Layout.from_parts(0, [3, 2], [1, 3]).is_contiguous()
    assert not wkf.Layout.from_parts(0, [2, 3], [0, 1]).is_contiguous()
    assert wkf.Layout.contiguous([]).is_contiguous() and wkf.Layout.contiguous([]).rank() == 0
    assert wkf.Layout.contiguous([7]).strides() == (1,)
    # the layouts the library hands out are these: a sliced tensor's view has the layout Layout::slice gives
    t = wkf.Tensor.new(planner, np.arange(24, dtype=np.float32).reshape(4, 6))
    got = t.slice([(1, 3), (2, 5)]).as_slice()
    want = wkf.Layout.contiguous([4, 6]).slice([(1, 3), (2, 5)])
    assert (got.offset, got.shape, got.strides) == (want.offset(), want.shape(), want.strides())
    for bad in ([(0, 5), (0, 5), (0, 6)], [(3, 2), (0, 5), (0, 6)], [(0, 4), (0, 5)]):
        with pytest.raises(wkf.WkfError) as e:
            cube.slice(bad)
        assert e.value.code == wkf.ERR_INVALID_ARG


def test_a_new_device_starts_with_default_settings(wkf):
    # per-device state is dropped with the device: a later device (the allocator tends to hand out the same
    # address again) must not inherit the fusion mode of one that was destroyed
    for _ in range(8):
        d = wkf.Device.planner()
        assert d.fusion() == wkf.FUSION_TREE
        d.set_fusion(wkf.FUSION_REFERENCE)
        assert d.fusion() == wkf.FUSION_REFERENCE
        d.close()


def test_graphs_sharing_nodes_resolve_from_several_threads(wkf, planner):
    # nodes are immutable and a resolution keeps its state to itself, so graphs that share nodes may be
    # materialised from different threads (one handle per thread); the device layer serialises the launches
    import threading
    base = wkf.Tensor.new(planner, np.arange(64 * 64, dtype=np.float32).reshape(64, 64))
    shared = base.mat_mul(base)
    roots = [(shared + float(i)).sum(1) for i in range(32)]
    errors = []

    def work(ts):
        try:
            for t in ts:
                t.materialize()
                assert [k.kind for k in t.kernels()] == ["gemm", "red_row"]
        except Exception as e:  # noqa: BLE001
            errors.append(e)

    threads = [threading.Thread(target=work, args=(roots[i::4],)) for i in range(4)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors


def test_hiprtc_failure_is_reported_with_the_log(wkf, planner):
    lib = wkf.load()
    k = ctypes.c_void_p()
    rc = lib.wkf_module_get(planner._h, b"test|bad-source", b"extern \"C\" __global__ void k() { this is not HIP }", b"k",
                            ctypes.byref(k))
    assert rc == 2
    msg = lib.wkf_last_error().decode()
    assert "hiprtc" in msg and "error" in msg


def test_graphvis_is_the_reference_dot_format(wkf, planner):
    # node ids `<name> ([shape] dtype) #<n>`, edges input -> consumer, shared nodes once (src/compute_graph/visualize.rs:13-271)
    x = wkf.Tensor.new(planner, np.ones((3, 2), dtype=np.float32))
    y = wkf.Tensor.new(planner, np.ones((3, 2), dtype=np.float16))
    m = x * 2.0
    t = (m + m.exp()).cast(wkf.F16).transpose(0, 1).mat_mul(y).sum(1)
    dot = t.graphvis()
    lines = [l.strip() for l in dot.strip().splitlines()]
    assert lines[0] == 'digraph "ComputeGraph" {' and lines[-1] == "}"
    nodes = [l for l in lines[1:-1] if "->" not in l]
    edges = [l for l in lines[1:-1] if "->" in l]
    names = [n.split(" (")[0].strip('"') for n in nodes]
    assert names == ["tensor", "multiply_const", "exp", "add", "cast", "slice", "tensor", "matmul", "sum"]
    assert '"slice ([2, 3] f16) #5";' in nodes and '"matmul ([2, 2] f16) #7";' in nodes and '"sum ([2] f16) #8";' in nodes
    assert len(edges) == 9  # multiply_const feeds both exp and add and is listed once
    assert '"multiply_const ([3, 2] f32) #1" -> "exp ([3, 2] f32) #2";' in edges
    assert '"multiply_const ([3, 2] f32) #1" -> "add ([3, 2] f32) #3";' in edges
    t.materialize()
    assert t.graphvis() == dot  # resolving keeps the graph (src/compute_graph/mod.rs:241-248)


def test_arange_is_a_host_loop(wkf, planner):
    assert np.array_equal(wkf.Tensor.arange(planner, 0.0, 10.0).to_numpy(), np.arange(10, dtype=np.float32))
    assert np.array_equal(wkf.Tensor.arange_step(planner, 0.0, 10.0, 2.0).to_numpy(), np.array([0, 2, 4, 6, 8], dtype=np.float32))
    assert np.array_equal(wkf.Tensor.arange_step(planner, 3.0, 0.0, -1.0).to_numpy(), np.array([3, 2, 1], dtype=np.float32))
    h = wkf.Tensor.arange_step(planner, 0.0, 1.0, 0.25, dtype=wkf.F16)
    assert h.datatype() == wkf.F16 and np.array_equal(h.to_numpy(), np.array([0, 0.25, 0.5, 0.75], dtype=np.float16))


# ---- the fusion pass (src/compute_graph/resolve.rs:49-196 of the reference) ---------------------

def _kinds(t):
    t.materialize()
    return [k.kind for k in t.kernels()]


def _x(wkf, dev, shape=(64, 64), dtype=np.float32, seed=0):
    return wkf.Tensor.new(dev, np.random.default_rng(seed).standard_normal(shape).astype(dtype))


@pytest.mark.parametrize("mode", [0, 1])
def test_fusion_rules_shared_by_both_modes(wkf, planner, mode):
    planner.set_fusion(mode)
    try:
        x, y = _x(wkf, planner), _x(wkf, planner, seed=1)
        # (1) a chain of element-wise nodes is one kernel (test_merge_add_const, src/element_wise.rs:422-443)
        t = ((x * 2.0) + 1.0).sin().exp()
        assert _kinds(t) == ["map"]
        sig = t.kernels()[0].signature
        assert "multiply_const" in sig and "add_const" in sig and "sin" in sig and "exp" in sig
        assert not t.kernels()[0].detail.endswith("in_place")  # a leaf is never overwritten (tests/inplace_clone.rs)
        # (3) chains below both operands of a pair-wise op fuse into it (src/pair_wise.rs:292-317)
        assert _kinds((x + 1.0) + (y * 2.0)) == ["map"]
        # (2) a chain above a pair-wise op fuses into it (src/pair_wise.rs:321-346)
        assert _kinds((x + y) - 1.0) == ["map"]
        # (3) pre-fused reduce (src/reduce.rs:570-600) and (2) post-fused reduce (:604-631)
        assert _kinds((x + 1.0).sum(0)) == ["red_col"]
        assert _kinds((x + 1.0).sum(1)) == ["red_row"]
        r = x.sum(1) + 1.0
        assert _kinds(r) == ["red_row"] and "post:load:f32@0;add_const" in r.kernels()[0].signature
        # (4) views cost nothing; a reduce of a sliced view still is one kernel
        assert _kinds(x.slice([(0, 64), (0, 1)]).sum(0)) == ["red_col"]
        assert _kinds(x.transpose(0, 1)) == []
        # (5) reduce <-> reduce never fuse
        assert _kinds(x.sum(1).sum(0)) == ["red_row", "red_row"]
        # resize, slice_assign and cat are copies
        assert _kinds(x.resize([70, 80])) == ["map"]
        # reshape always copies in the reference (src/resize.rs:131-144); in tree mode a dense tensor is re-viewed
        # instead, and the copy of a computed or strided one is fused with what produces it
        assert _kinds(x.reshape([32, 128])) == (["map"] if mode == 0 else [])
        assert _kinds(x.transpose(0, 1).reshape([32, 128])) == ["map"]
        assert _kinds((x + 1.0).reshape([32, 128])) == (["map", "map"] if mode == 0 else ["map"])
    finally:
        planner.set_fusion(1)


def test_reference_mode_is_the_reference_decomposition(wkf, planner):
    planner.set_fusion(wkf.FUSION_REFERENCE)
    try:
        a, b = _x(wkf, planner, (4, 8, 16)), _x(wkf, planner, (4, 8, 16), seed=1)
        bias = _x(wkf, planner, (16,), seed=2)
        bias3 = bias.broadcast([8, 16]).broadcast([4, 8, 16])
        out = a.silu() * (b + bias3)
        # silu's div, the strided add, then the mul in place into the div's result (src/pair_wise.rs:95-107)
        assert _kinds(out) == ["map", "map", "map"]
        ks = out.kernels()
        assert "in_place" not in ks[0].detail and "in_place" not in ks[1].detail and ks[2].detail.endswith("in_place")
        # RMSNorm = one reduce (pre [sqr], post [/H, +eps, sqrt]) + two strided pair-wise kernels
        x, w = _x(wkf, planner, (32, 64)), _x(wkf, planner, (64,), seed=3)
        ln = x.layer_norm(w, 1e-5)
        assert _kinds(ln) == ["red_row", "map", "map"]
        sig = ln.kernels()[0].signature
        assert "pre:load:f32@0;sqr" in sig and "divide_const" in sig and "add_const" in sig and "sqrt" in sig
        # no memoisation: the exp under softmax is computed in both kernels (src/tensor.rs:286-288)
        v = _x(wkf, planner, (128,))
        assert _kinds(v.softmax()) == ["red_row", "map"]
        # (5) pair-wise <-> pair-wise do not fuse: (a + b) is materialised, then multiplied in place
        t = (a + b) * a
        assert _kinds(t) == ["map", "map"] and t.kernels()[1].detail.endswith("in_place")
    finally:
        planner.set_fusion(wkf.FUSION_TREE)


def test_tree_mode_fuses_pair_wise_trees_and_copies(wkf, planner):
    a, b = _x(wkf, planner, (4, 8, 16)), _x(wkf, planner, (4, 8, 16), seed=1)
    bias3 = _x(wkf, planner, (16,), seed=2).broadcast([8, 16]).broadcast([4, 8, 16])
    out = a.silu() * (b + bias3)
    assert _kinds(out) == ["map"]
    k = out.kernels()[0]
    assert "operands=4" in k.detail  # a (read once although silu uses it twice), b, bias, out
    assert "shape=[32,16]" in k.detail  # the two leading dims merge for every operand
    x, w = _x(wkf, planner, (32, 64)), _x(wkf, planner, (64,), seed=3)
    # last-axis reductions that are used again on the same rows run as ONE row kernel (row held in registers)
    ln = x.layer_norm(w, 1e-5)
    assert _kinds(ln) == ["row"] and "stages=1" in ln.kernels()[0].detail
    s = _x(wkf, planner, (4, 8, 32)).softmax_last_dim()
    assert _kinds(s) == ["row"] and "stages=2" in s.kernels()[0].detail  # max, sum(exp(x - max)), exp(x - max) / sum
    # a row length that is not a multiple of the 16-byte vector takes narrower vectors in the same kernel
    odd = _x(wkf, planner, (8, 30)).softmax_last_dim()
    assert _kinds(odd) == ["row"] and "vec=2" in odd.kernels()[0].detail
    q = _x(wkf, planner, (2, 8, 16))
    cos, sin = _x(wkf, planner, (8, 8), seed=4), _x(wkf, planner, (8, 8), seed=5)
    # rope = ONE kernel: the cats of rotate_half and of the duplicated tables are cut at the seam, both halves of the
    # result are stored by the same kernel, and x1, x2, cos, sin are each loaded once (the reference: about 10 kernels)
    r = q.rope(cos, sin)
    assert _kinds(r) == ["map"]
    assert "outputs=2" in r.kernels()[0].detail and "operands=6" in r.kernels()[0].detail
    # a cat that is itself the result: one copy kernel per piece (each fused with what produces the piece), no padding pass
    c3 = wkf.Tensor.cat([q, q * 2.0, _x(wkf, planner, (5, 8, 16), seed=8)], 0)
    assert _kinds(c3) == ["map", "map", "map"] and c3.shape() == (9, 8, 16)
    planner.set_fusion(wkf.FUSION_REFERENCE)
    try:
        assert len(_kinds(wkf.Tensor.cat([q, q * 2.0], 0))) == 3  # the reference: resize, the product, slice_assign
    finally:
        planner.set_fusion(wkf.FUSION_TREE)
    # pieces of different widths: one kernel per piece
    odd = _x(wkf, planner, (2, 8, 10)).narrow(2, 0, 3)
    assert _kinds(wkf.Tensor.cat([odd, _x(wkf, planner, (2, 8, 5), seed=6)], 2) * _x(wkf, planner, (2, 8, 8), seed=7)) == ["map", "map"]


def test_few_outputs_over_a_long_axis_fold_in_two_launches(wkf, planner):
    # the reference always puts one workgroup on one output (src/reduce.rs:316-346); here a long axis with too
    # few outputs to fill the chip is cut into slices whose f32 partial folds a second launch finishes
    x = wkf.Tensor.new(planner, np.zeros((8192, 512), dtype=np.float32))
    t = (x * 2.0).sum(0) + 1.0
    assert _kinds(t) == ["red_col", "red_col"]
    first, second = t.kernels()
    assert first.detail.endswith("partial") and "vec=4" in first.detail and "|raw" in first.signature
    assert "multiply_const" in first.signature and "add_const" not in first.signature
    assert "pre:load:f32@0->0|" in second.signature and "add_const" in second.signature and "fold:f32" in second.signature
    h = wkf.Tensor.new(planner, np.zeros((4, 262144), dtype=np.float16)).max(1)
    assert _kinds(h) == ["red_row", "red_row"]
    assert "fold:f16" in h.kernels()[1].signature and "in:f32" in h.kernels()[1].signature
    # an axis length without a power-of-two factor is not cut
    assert _kinds(wkf.Tensor.new(planner, np.zeros((3, 100003), dtype=np.float32)).sum(1)) == ["red_row"]
    planner.set_fusion(wkf.FUSION_REFERENCE)
    try:
        assert _kinds(wkf.Tensor.new(planner, np.zeros((8192, 512), dtype=np.float32)).sum(0)) == ["red_col"]
    finally:
        planner.set_fusion(wkf.FUSION_TREE)


def test_sibling_row_reductions_share_one_pass(wkf, planner):
    # README.md:20 of the reference lists "parallel reduces" as to-do; here several tensors are materialised together
    x = wkf.Tensor.new(planner, np.zeros((512, 2048), dtype=np.float32))
    a, b, c = x.max(1), (x.clone() - 1.0).exp().sum(1) + 2.0, x.min(1)
    wkf.materialize_many([a, b, c])
    ks = a.kernels()
    assert [k.kind for k in ks] == ["row"] and "reductions=3" in ks[0].detail and "|scalars" in ks[0].signature
    assert b.kernels() == [] and c.kernels() == []  # the pass is recorded on the first tensor
    # alone, each is an ordinary reduce
    assert _kinds(a) == ["red_row"]
    # a shared producer is computed once for all of its consumers; reductions over other axes run one by one
    g = x.mat_mul(wkf.Tensor.new(planner, np.zeros((2048, 256), dtype=np.float32)))
    s0, s1, m = g.sum(0), g.sum(1), g.max(1) * 3.0
    wkf.materialize_many([s0, s1, m])
    kinds = [k.kind for k in s0.kernels()]
    assert kinds.count("gemm") == 1 and kinds.count("row") == 1 and kinds.count("red_col") >= 1 and len(kinds) <= 4
    # rows too long for the registers of one block: separate (two-launch) reduces
    y = wkf.Tensor.new(planner, np.zeros((64, 400000), dtype=np.float32))
    p, q = y.max(1), y.sum(1)
    wkf.materialize_many([p, q])
    assert [k.kind for k in p.kernels()] == ["red_row"] * 4
    planner.set_fusion(wkf.FUSION_REFERENCE)
    try:
        wkf.materialize_many([a, c])
        assert [k.kind for k in a.kernels()] == ["red_row", "red_row"]
    finally:
        planner.set_fusion(wkf.FUSION_TREE)
    with pytest.raises(wkf.WkfError):
        wkf.materialize_many([])


def test_row_kernel_takes_rows_that_do_not_split_evenly(wkf, planner):
    def detail(shape, dtype, f):
        t = f(_x(wkf, planner, shape, dtype))
        assert _kinds(t) == ["row"], [k.detail for k in t.kernels()]
        return t.kernels()[0].detail

    sm = lambda t: t.softmax_last_dim()  # noqa: E731
    # an even split keeps the exact kernel (no masking) ...
    assert "ragged" not in detail((8, 4096), np.float32, sm)
    assert "ragged" not in detail((8, 5120), np.float32, sm)                      # 1280 vectors = 256 lanes x 5
    # ... anything else gets the widest layout with the tail lanes masked in their last vector
    assert detail((8, 2880), np.float32, sm).endswith("vec=4 threads_per_row=256 vectors_per_lane=3 stages=2 operands=2 ragged")
    assert "vec=2" in detail((8, 1002), np.float32, sm) and "vec=1" in detail((8, 50257), np.float32, sm)
    assert "vec=8" in detail((8, 2880), np.float16, sm) and "vec=4" in detail((8, 11004), np.float16, sm)
    # rows of a view that start off the vector grid take narrower vectors instead of three kernels
    assert "vec=1" in detail((8, 4096), np.float32, lambda t: t.slice([(0, 8), (1, 4095)]).softmax_last_dim())
    # beyond what 1024 lanes hold in registers a row is spread over the registers of a team of blocks that exchange
    # their folds: one launch, the row read once; the grid never exceeds four blocks per compute unit (1024 here)
    assert detail((2, 65537), np.float32, sm).endswith(
        "vectors_per_lane=8 stages=2 operands=2, max and sum in one exchange, rows in the registers of teams of 33 blocks, 2 teams")
    assert detail((256, 65537), np.float32, sm).endswith("rows in the registers of teams of 33 blocks, 29 teams")
    assert detail((64, 262144), np.float32, sm).endswith("rows in the registers of teams of 32 blocks, 32 teams")
    team = _x(wkf, planner, (3, 200000), np.float16).softmax_last_dim()
    assert _kinds(team) == ["row"] and team.kernels()[0].signature.endswith("|online|team") and team.kernels()[0].detail.endswith("teams of 13 blocks, 3 teams")
    # two operands: half the vectors per lane each; a stage that does not pair with the next: one exchange per stage
    two = _x(wkf, planner, (4, 80000), np.float32)
    two = (two + _x(wkf, planner, (4, 80000), np.float32, seed=1)).softmax_last_dim()
    assert _kinds(two) == ["row"] and "vectors_per_lane=4" in two.kernels()[0].detail and "teams of 20 blocks" in two.kernels()[0].detail
    norm = _x(wkf, planner, (4, 80000), np.float32).layer_norm(_x(wkf, planner, (80000,), np.float32, seed=2), 1e-5)
    assert _kinds(norm) == ["row"], [k.detail for k in norm.kernels()]
    assert "in one exchange" not in norm.kernels()[0].detail and "teams of" in norm.kernels()[0].detail
    # rows of more than 256 parts (2 M floats) and devices with teams switched off keep the kernels below
    planner.set_row_teams(False)
    try:
        # a few rows are split into parts: one launch for the online pair of max and sum over every part, one that
        # folds a row's parts and writes the result
        long_rows = _x(wkf, planner, (2, 65537), np.float32).softmax_last_dim()
        assert _kinds(long_rows) == ["row", "row"]
        details = [k.detail for k in long_rows.kernels()]
        assert details[0].endswith("streamed (max and sum in one pass), rows split in 65 parts of 1024 vectors: launch 1 of 2"), details
        assert details[1].endswith("launch 2 of 2") and long_rows.kernels()[0].signature.endswith("|split0")
        assert long_rows.kernels()[1].signature.endswith("|split2")
        # 256 rows or more stream with a block per row, in one launch
        many = _x(wkf, planner, (256, 65537), np.float32).softmax_last_dim()
        assert _kinds(many) == ["row"] and many.kernels()[0].detail.endswith("streamed (max and sum in one pass)")
    finally:
        planner.set_row_teams(True)
    wide = _x(wkf, planner, (2, (1 << 21) + 4096), np.float32).softmax_last_dim()
    assert _kinds(wide) == ["row", "row"] and "rows split in" in wide.kernels()[0].detail
    # rows that are short but too many vectors for the lanes' registers (fewer than 1024 vectors never are) stay decomposed
    assert _kinds(_x(wkf, planner, (2, 70000), np.float32).max(1)) == ["red_row", "red_row"]


def test_f16_column_max_with_a_post_op_compiles(wkf, planner):
    # this kernel (8 f16 columns per lane, 16 waves, four loads in flight, c - max) once hit a fatal "cannot select"
    # error inside the compiler's backend, which ends the process; kernels are compiled without the SLP vectoriser since
    t = 1.0 - _x(wkf, planner, (512, 8), np.float16).max(0)
    assert _kinds(t) == ["red_col"] and t.shape() == (8,)
    assert "|v8|" in t.kernels()[0].signature and "const_subtract" in t.kernels()[0].signature


def test_mat_mul_kernel_choice(wkf, planner):
    def detail(m, n, k, dtype):
        t = _x(wkf, planner, (m, k), dtype).mat_mul(_x(wkf, planner, (k, n), dtype, seed=1))
        assert _kinds(t) in (["gemm"], ["gemm", "red_col"])  # (K in slices: the f32 partial sums are folded by a second launch)
        return t.kernels()[0].detail

    # full f16 tiles: the operands go from memory straight into the LDS (whole tiles and a last round in half tiles)
    assert detail(4096, 4096, 192, np.float16).endswith("mfma 256x256 tiles, operands loaded straight into the LDS")
    assert detail(4096, 4352, 192, np.float16).endswith("operands loaded straight into the LDS, last round: 16 tiles as 32 halves of 128 rows")
    assert detail(512, 256, 96, np.float32).endswith("mfma 256x256 tiles")
    # not a multiple of the tile but every row 16-byte aligned: the same MFMA kernel with edge handling
    assert detail(4000, 4000, 72, np.float16).endswith("mfma 256x256 tiles edge")
    # ... and a partly filled last round of it runs in half tiles like that of a full shape (16 x 17 tiles)
    assert detail(4000, 4104, 72, np.float16).endswith("mfma 256x256 tiles edge, last round: 16 tiles as 32 halves of 128 rows")
    assert detail(300, 260, 68, np.float32).endswith("mfma 256x256 tiles edge")
    assert detail(4096, 4352, 64, np.float32).endswith("mfma 256x256 tiles, last round: 16 tiles as 32 halves of 128 rows")
    # f16 products whose large tiles would fill at most half of the chip take 128 x 128 tiles, two workgroups per compute unit
    # (K a multiple of 64: a tile of 64 NI x 64 NJ chosen by a cost model, operands loaded straight into the LDS; else 128 x 128)
    assert detail(512, 256, 128, np.float16).endswith("mfma 64x192 tiles, operands loaded straight into the LDS, 4 stages")
    assert detail(512, 11008, 4096, np.float16).endswith("mfma 128x192 tiles, operands loaded straight into the LDS, 4 stages")
    assert detail(128, 4096, 4096, np.float16).endswith("mfma 64x128 tiles, operands loaded straight into the LDS, 5 stages slices=4")
    assert detail(512, 264, 136, np.float16).endswith("mfma 128x128 tiles")
    assert detail(300, 264, 72, np.float16).endswith("mfma 128x128 tiles")
    assert detail(1024, 11008, 512, np.float16).endswith("mfma 256x256 tiles, operands loaded straight into the LDS")
    # unaligned rows or tiny problems: the generic kernel
    assert detail(300, 262, 72, np.float16).endswith("generic")
    assert detail(3, 7, 5, np.float32).endswith("generic")
    # ... unless the product is large: then one transposed copy of B (rows aligned again) keeps it on the MFMA kernels
    t = _x(wkf, planner, (300, 512), np.float16).mat_mul(_x(wkf, planner, (512, 1001), np.float16, seed=1))
    assert _kinds(t) == ["map", "gemm"] and "tiled" in t.kernels()[0].detail and t.kernels()[1].detail.endswith("tiles B^T")
    # ... and when K is off the vector grid, zero-padded copies of both operands do
    t = _x(wkf, planner, (300, 515), np.float16).mat_mul(_x(wkf, planner, (515, 1000), np.float16, seed=1))
    assert _kinds(t) == ["map", "map", "gemm"] and "k=520" in t.kernels()[2].detail and t.shape() == (300, 1000)
    # a handful of rows: the bandwidth kernel over slices of K, then one reduce over the slices
    s = _x(wkf, planner, (4, 4096), np.float16).mat_mul(_x(wkf, planner, (4096, 2048), np.float16, seed=1))
    assert _kinds(s) == ["gemm", "red_col"] and "skinny" in s.kernels()[0].detail and s.shape() == (4, 2048)
    assert s.datatype() == wkf.F16 and "fold:f16" in s.kernels()[1].signature
    # a transposed A is copied into a dense buffer first (tiled copy), then multiplied
    t = _x(wkf, planner, (256, 512), np.float16).transpose(0, 1).mat_mul(_x(wkf, planner, (256, 256), np.float16, seed=1))
    assert _kinds(t) == ["map", "gemm"] and "tiled" in t.kernels()[0].detail
    # x * W^T for a dense W [N, K] needs no copy: the MFMA kernels read W as it lies ...
    w = _x(wkf, planner, (512, 256), np.float16, seed=2)
    t = _x(wkf, planner, (256, 256), np.float16).mat_mul(w.transpose(0, 1))
    assert _kinds(t) == ["gemm"] and "tiles B^T" in t.kernels()[0].detail and "|bt" in t.kernels()[0].signature
    big_w = _x(wkf, planner, (4096, 256), np.float16, seed=2)
    t = _x(wkf, planner, (4096, 256), np.float16).mat_mul(big_w.transpose(0, 1))
    assert _kinds(t) == ["gemm"] and "B^T" in t.kernels()[0].detail and t.kernels()[0].signature.endswith("|bt|direct to LDS")
    # ... and with a handful of rows W is streamed once through MFMA operands (decode)
    t = _x(wkf, planner, (2, 256), np.float16).mat_mul(w.transpose(0, 1))
    assert _kinds(t)[0] == "gemm" and "skinny B^T" in t.kernels()[0].detail and t.shape() == (2, 512)
    # in f32 up to 16 rows take the vector ALUs instead (the f32 matrix instruction cannot keep up with the memory), more the MFMAs
    w32 = _x(wkf, planner, (512, 256), np.float32, seed=2)
    t = _x(wkf, planner, (16, 256), np.float32).mat_mul(w32.transpose(0, 1))
    # (rows of A that fit the LDS whole: one launch, no K slices; here 16 x 256 floats; a wave walks one row of W)
    assert _kinds(t) == ["gemm"] and t.kernels()[0].detail.endswith("skinny B^T valu whole K, 1 rows a wave")
    assert t.kernels()[0].signature == "gemm|gfx950|f32|skinny_bt|valu|m16|c1024|r1"
    big = _x(wkf, planner, (16, 4096), np.float32).mat_mul(_x(wkf, planner, (512, 4096), np.float32, seed=2).transpose(0, 1))
    assert len(_kinds(big)) == 2 and "skinny B^T valu slices=" in big.kernels()[0].detail  # 256 KiB of A: K in slices, then the fold
    # 5 to 16 rows of f16 against enough rows of W to give every compute unit a block: one launch, the eight waves of a block share K
    wide16 = _x(wkf, planner, (8, 1024), np.float16).mat_mul(_x(wkf, planner, (8192, 1024), np.float16, seed=2).transpose(0, 1))
    assert _kinds(wide16) == ["gemm"] and wide16.kernels()[0].detail.endswith("skinny B^T, K over the 8 waves of a block")
    t = _x(wkf, planner, (17, 256), np.float32).mat_mul(w32.transpose(0, 1))
    assert _kinds(t)[0] == "gemm" and "skinny B^T slices" in t.kernels()[0].detail
    planner.set_fusion(wkf.FUSION_REFERENCE)
    try:
        assert _kinds(_x(wkf, planner, (256, 256), np.float16).mat_mul(w.transpose(0, 1))) == ["map", "gemm"]
    finally:
        planner.set_fusion(wkf.FUSION_TREE)


def test_batched_mat_mul_is_one_launch(wkf, planner):
    # beyond the reference (rank 2 only, src/matmul.rs:25-29): equal leading dimensions are a batch
    q = _x(wkf, planner, (8, 512, 128), np.float16)
    k = _x(wkf, planner, (8, 512, 128), np.float16, seed=1)
    scores = q.mat_mul(k.transpose(1, 2))                      # q k^T per head: k is read as it lies
    assert scores.shape() == (8, 512, 512) and _kinds(scores) == ["gemm"]
    assert "tiles B^T" in scores.kernels()[0].detail and scores.kernels()[0].detail.endswith("batch=8") and "|bt" in scores.kernels()[0].signature
    v = _x(wkf, planner, (8, 512, 128), np.float16, seed=2)
    out = scores.softmax_last_dim().mat_mul(v)
    assert out.shape() == (8, 512, 128) and _kinds(out) == ["gemm", "row", "gemm"]
    # n = 128: the small tile, nothing wasted; one column of tiles over K = 512: every workgroup starts at its own K tile
    assert out.kernels()[2].detail.endswith("128x128 tiles K start rotated batch=8") and out.kernels()[2].signature.endswith("|rotk")
    r4 = _x(wkf, planner, (2, 3, 17, 33), np.float32).mat_mul(_x(wkf, planner, (2, 3, 33, 5), np.float32, seed=1))
    assert r4.shape() == (2, 3, 17, 5) and _kinds(r4) == ["gemm"] and r4.kernels()[0].detail.endswith("generic batch=6")
    # decode: one query row per head streams k and v once (the bandwidth kernels), one fold for all heads
    q1 = _x(wkf, planner, (8, 1, 128), np.float16, seed=3)
    kv = _x(wkf, planner, (8, 2048, 128), np.float16, seed=4)
    s1 = q1.mat_mul(kv.transpose(1, 2))
    # (one launch: the vector-ALU kernel for one row of f16 folds its K slices itself, the last wave to finish 32 rows)
    assert _kinds(s1) == ["gemm"]
    assert "skinny B^T valu" in s1.kernels()[0].detail and s1.kernels()[0].detail.endswith("batch=8")
    s8 = _x(wkf, planner, (8, 8, 128), np.float16, seed=3).mat_mul(kv.transpose(1, 2))
    assert _kinds(s8)[0] == "gemm" and len(_kinds(s8)) == 2 and "skinny B^T slices" in s8.kernels()[0].detail  # more rows: MFMAs, then the fold
    o1 = s1.mat_mul(kv)
    assert o1.shape() == (8, 1, 128) and _kinds(o1)[-2:] == ["gemm", "red_col"]
    # (128 columns: a narrow B, whose rows the lanes of a block share among themselves)
    assert "skinny narrow slices" in o1.kernels()[-2].detail and o1.kernels()[-2].detail.endswith("batch=8")
    assert o1.kernels()[-2].signature.endswith("|skinny|m1|v8|narrow16")
    # the same kernel source as a single product (the tile may differ: it is chosen for the number of workgroups)
    before = planner.module_stats()
    _x(wkf, planner, (3, 256, 64), np.float16).mat_mul(_x(wkf, planner, (3, 64, 256), np.float16, seed=1)).materialize()
    _x(wkf, planner, (256, 64), np.float16).mat_mul(_x(wkf, planner, (64, 256), np.float16, seed=1)).materialize()
    after = planner.module_stats()
    assert (after["compiled"] + after["disk_hits"]) - (before["compiled"] + before["disk_hits"]) <= 2
    for bad_a, bad_b in (((2, 4, 8), (3, 8, 4)), ((2, 4, 8), (8, 4)), ((2, 4, 8), (2, 7, 4)), ((8,), (8,))):
        with pytest.raises(wkf.WkfError) as e:
            _x(wkf, planner, bad_a, np.float32).mat_mul(_x(wkf, planner, bad_b, np.float32, seed=1))
        assert e.value.code == wkf.ERR_INVALID_ARG


def test_one_binary_serves_every_size_and_constant(wkf, planner):
    before = planner.module_stats()
    t1 = (_x(wkf, planner, (256, 256)) * 3.0) + 5.0
    t2 = (_x(wkf, planner, (128, 512)) * -7.5) + 0.25
    t1.materialize()
    t2.materialize()
    assert t1.kernels()[0].signature == t2.kernels()[0].signature
    after = planner.module_stats()
    assert after["compiled"] + after["disk_hits"] - before["compiled"] - before["disk_hits"] <= 1
    assert after["mem_hits"] >= before["mem_hits"] + 1


def test_generated_source_keeps_every_op_rounded_on_its_own(wkf, planner):
    t = ((_x(wkf, planner, (64, 64), np.float16) * 2.0) + 1.0).exp()
    t.materialize()
    src = wkf.kernel_source(t.kernels()[0].signature)
    assert "const _Float16 v1 = v0 * (_Float16)c[0];" in src
    assert "const _Float16 v2 = v1 + (_Float16)c[1];" in src
    assert "wkf_f16x8" in src  # 128-bit vectors of f16
    f = ((_x(wkf, planner, (64, 64)) * 2.0) + 1.0).sin().exp()
    f.materialize()
    src = wkf.kernel_source(f.kernels()[0].signature)
    assert "wkf_sin(v2, far)" in src and "expf(v3)" in src  # interior op: f64 core; last op: f32 library
    assert "wkf_expr_far" in src and "wkf_f32x4" in src
    planner.set_exact_math(True)
    try:
        f.materialize()
        assert "wkf_exp(v3)" in wkf.kernel_source(f.kernels()[0].signature)
    finally:
        planner.set_exact_math(False)


def test_reduce_into_plans_without_allocating_and_refuses_the_rest(wkf):
    # the allocation-free variant of reduce + materialize, on a device of its own (fresh kernel table)
    dev = wkf.Device.planner()
    T = wkf.Tensor
    x = T.new(dev, np.zeros((64, 262144), dtype=np.float32))
    out = T.new(dev, np.zeros((64,), dtype=np.float32))
    # its kernels are not loaded yet: loading one would allocate, so the call names the kernel and stops
    with pytest.raises(wkf.WkfError, match="is not loaded"):
        x.reduce_into("sum", 1, out)
    lazy = x.sum(1)
    lazy.materialize()
    assert len(lazy.kernels()) == 2  # few rows over a long axis: partial results, then the fold
    before = dev.module_stats()
    x.reduce_into("sum", 1, out)
    after = dev.module_stats()
    assert (after["compiled"], after["disk_hits"]) == (before["compiled"], before["disk_hits"])
    # partial results beyond the static scratch array (1 MiB): refused with the sizes in the message
    big = T.new(dev, np.zeros((4096, 32768), dtype=np.float16))
    big.sum(0).materialize()
    with pytest.raises(wkf.WkfError, match="static scratch array holds 1048576"):
        big.reduce_into("sum", 0, T.new(dev, np.zeros((32768,), dtype=np.float16)))
    with pytest.raises(wkf.WkfError, match="hold data"):
        (x + 1.0).reduce_into("sum", 1, out)
    with pytest.raises(wkf.WkfError, match="shape"):
        x.reduce_into("sum", 1, T.new(dev, np.zeros((63,), dtype=np.float32)))
    dev.close()


def test_reference_compat_changes_only_the_square_layer_norm(wkf):
    # the flag is per device and acts when the tensor is built: for a square input the weight's broadcast lands on
    # dimension 1, as the reference's text reads, so along a row the weight is ONE value (axis stride 0 in the row
    # kernel's signature) instead of a row of values (axis stride 1); a non-square input plans the same kernel either way
    dev = wkf.Device.planner()
    T = wkf.Tensor
    w = T.new(dev, np.ones((8,), dtype=np.float32))
    sq, rect = T.new(dev, np.ones((8, 8), dtype=np.float32)), T.new(dev, np.ones((4, 8), dtype=np.float32))

    def plan(x):
        t = x.layer_norm(w, 1e-5).materialize()
        return [k.signature for k in t.kernels()]

    meant, rect_meant = plan(sq), plan(rect)
    dev.set_reference_compat(True)
    written, rect_written = plan(sq), plan(rect)
    dev.set_reference_compat(False)
    assert len(meant) == len(written) == 1
    assert "|in:f32a1,f32a1,|" in meant[0] and "|in:f32a1,f32a0,|" in written[0]
    assert rect_written == rect_meant and plan(sq) == meant
    dev.close()


@pytest.mark.parametrize("dtype", [np.float16, np.float32], ids=["f16", "f32"])
def test_every_unary_op_compiles_where_its_value_feeds_further_work(wkf, dtype):
    # the generator picks a different evaluation for an op whose value is read again (f64 cores, f16 roundings decided in
    # f32, ...): every unary op, followed by a literal op, inside a reduction's chain and in front of a cast, must give a
    # kernel that compiles (an interior sqrt on f16 once named a helper its kernel did not include)
    dev = wkf.Device.planner()
    x = wkf.Tensor.new(dev, np.ones((64, 64), dtype=dtype))
    ops = ["exp", "exp2", "log", "log2", "sqr", "sqrt", "sin", "cos", "tan", "asin", "acos", "atan", "sinh", "cosh", "tanh",
           "asinh", "acosh", "atanh", "abs"]
    for op in ops:
        for graph in (getattr(x, op)() * 2.0, getattr(x, op)().sum(1), getattr(x, op)().cast(wkf.F32 if dtype == np.float16 else wkf.F16) + 1.0):
            graph.materialize()
            assert len(graph.kernels()) == 1, op
    dev.close()


def test_a_costly_value_of_one_f16_operand_is_cut_out_as_a_table(wkf):
    # silu(a) * (b + bias) on f16: silu(a) depends on `a` alone, so from the table threshold on the planner cuts it out of
    # the fused program, plans a kernel that fills the table (the cut program, marked "!" because its result fed further
    # arithmetic and keeps the rounding of an interior op) and a map kernel with a `lookup` in its place and the table as
    # one more argument; below the threshold, with tables off, or on f32 nothing changes
    dev = wkf.Device.planner()
    T = wkf.Tensor
    n = (512, 512)

    def plan(dtype, least):
        dev.set_map_table(least)
        a, b = T.new(dev, np.ones(n, dtype=dtype)), T.new(dev, np.ones(n, dtype=dtype))
        bias = T.new(dev, np.ones((512,), dtype=dtype))
        t = (a.silu() * (b + bias.broadcast(list(n)))).materialize()
        return [(k.signature, k.detail) for k in t.kernels()]

    cut = plan(np.float16, 1 << 17)
    assert len(cut) == 2
    assert cut[0][0].endswith("load:f16@0;neg:f16(0);exp:f16(1);add_const:f16(2,c0);div:f16(0,3)->4!") and "shape=[65536]" in cut[0][1]
    assert "lookup:f16(0)" in cut[1][0] and cut[1][0].endswith("|table") and "exp" not in cut[1][0].split("|m0|")[1]
    assert "table lookup: 65536 values of" in cut[1][1]
    again = plan(np.float16, 1 << 17)
    assert len(again) == 1 and again[0][0] == cut[1][0]            # the table is kept per device
    for other in (plan(np.float16, 1 << 25), plan(np.float16, 0), plan(np.float32, 1 << 17)):
        assert len(other) == 1 and "lookup" not in other[0][0] and "|table" not in other[0][0]
    dev.close()


def test_a_timer_outlives_its_device_handle(wkf):
    # A timer keeps its device alive like a buffer does (its events go back to that device's pool): destroying the
    # device first and the timer afterwards must find the device still there, and the device goes with the timer.
    import ctypes
    lib = wkf.load()
    lib.wkf_timer_create.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p)]
    lib.wkf_timer_destroy.argtypes = [ctypes.c_void_p]
    lib.wkf_timer_destroy.restype = None
    for _ in range(4):
        dev = wkf.Device.planner()
        x = wkf.Tensor.new(dev, np.zeros((8,), dtype=np.float32))
        stats = dev.alloc_stats()
        assert stats["live_buffers"] >= 1 and stats["buffer_allocs"] >= 1
        timers = [ctypes.c_void_p() for _ in range(3)]
        for t in timers:
            assert lib.wkf_timer_create(dev._h, ctypes.byref(t)) == 0
        assert dev.alloc_stats()["timers"] == stats["timers"] + 3
        dev.close()            # deferred: a buffer and three timers are alive
        del x                  # the tensor's buffer goes first ...
        for t in timers:       # ... and the last timer takes the device with it
            lib.wkf_timer_destroy(t)


def _code_object_kernels(path):
    """The kernel records of the AMDGPU metadata note of one code object (ELF note type 32, MessagePack)."""
    import struct

    import msgpack
    b = open(path, "rb").read()
    assert b[:4] == b"\x7fELF"
    shoff = struct.unpack_from("<Q", b, 0x28)[0]
    shentsize, shnum, _ = struct.unpack_from("<HHH", b, 0x3A)
    kernels = []
    for i in range(shnum):
        sh = struct.unpack_from("<IIQQQQIIQQ", b, shoff + i * shentsize)
        if sh[1] != 7:  # SHT_NOTE
            continue
        p, end = sh[4], sh[4] + sh[5]
        while p < end:
            namesz, descsz, typ = struct.unpack_from("<III", b, p)
            p += 12
            name = b[p:p + namesz]
            p += (namesz + 3) & ~3
            desc = b[p:p + descsz]
            p += (descsz + 3) & ~3
            if name.startswith(b"AMDGPU") and typ == 32:
                kernels += msgpack.unpackb(desc, raw=False)["amdhsa.kernels"]
    return kernels


def test_gemm_kernels_use_no_scratch_memory(tmp_path):
    # A GEMM kernel that spills its accumulators to scratch memory still gives right results, only several times
    # slower: every mat_mul kernel variant is compiled into an empty cache directory and the compiler's own record
    # in each code object must show no private segment and no spilled register.
    import glob
    import subprocess
    import sys
    script = (
        "import sys, numpy as np\n"
        f"sys.path.insert(0, {os.path.join(ROOT, 'tests')!r})\n"
        "from helpers import load_package\n"
        "w = load_package(); dev = w.Device.planner(); T = w.Tensor\n"
        "def mm(m, n, k, dt, bt=False, lead=()):\n"
        "    a = T.new(dev, np.zeros(lead + (m, k), dtype=dt))\n"
        "    b = T.new(dev, np.zeros(lead + ((n, k) if bt else (k, n)), dtype=dt))\n"
        "    r = len(lead) + 2\n"
        "    a.mat_mul(b.transpose(r - 2, r - 1) if bt else b).materialize()\n"
        "for dt in (np.float16, np.float32):\n"
        "    for bt in (False, True):\n"
        "        mm(4096, 4096, 128, dt, bt)    # full 256 x 256 tiles\n"
        "        mm(4096, 4352, 128, dt, bt)    # 272 tiles: the last round in half tiles (f16)\n"
        "        mm(4000, 4104, 136, dt, bt)    # 256 x 256 tiles with ragged edges (f16, B as it lies: the last round in half tiles)\n"
        "        mm(4000, 4000, 136, dt, bt)    # ... in whole tiles\n"
        "        mm(512, 512, 256, dt, bt)      # few tiles\n"
        "        mm(300, 264, 2048, dt, bt)     # few ragged tiles, K in slices\n"
        "        mm(256, 256, 4096, dt, bt)     # K in slices\n"
        "        mm(128, 384, 4096, dt, bt)     # 128 x 128 tiles (f16), K in slices\n"
        "        mm(512, 1024, 512, dt, bt)     # 128 x 128 tiles (f16)\n"
        "        mm(1, 1024, 512, dt, bt); mm(8, 520, 1000, dt, bt); mm(20, 264, 4096, dt, bt)  # decode sizes\n"
        "    mm(4000, 4001, 136, dt, True)      # rows of C off the 16-byte grid: the ragged kernel that addresses with pointers\n"
        "    mm(3, 5, 7, dt)                    # the generic kernel\n"
        "    mm(64, 64, 32, dt, lead=(3,))\n"
        "    for k in (128, 192, 256):          # many full tiles over a short K: a tile's stores under the next tile's MFMAs (f16)\n"
        "        mm(2048, 2048, k, dt, True, lead=(16,)); mm(2048, 2048, k, dt, False, lead=(16,))\n"
        "import os\n"
        "for cfg in ('2,3,4,1', '2,3,4,3', '2,3,3,2', '2,2,2,1', '2,2,2,4', '1,3,4,1', '1,3,4,2', '1,4,4,1', '1,2,5,2', '1,2,5,4'):\n"
        "    os.environ['WKF_GEMM_FLEX'] = cfg     # every tile of the flexible f16 kernel, forced on a device of its own\n"
        "    dev = w.Device.planner()\n"
        "    mm(300, 1000, 2048, np.float16); mm(300, 1000, 2048, np.float16, True)\n"
        "del os.environ['WKF_GEMM_FLEX']\n"
    )
    env = dict(os.environ, WKF_CACHE_DIR=str(tmp_path))
    subprocess.run([sys.executable, "-c", script], check=True, env=env, timeout=900)
    checked = 0
    for path in glob.glob(os.path.join(str(tmp_path), "*.hsaco")):
        for k in _code_object_kernels(path):
            if not k[".name"].startswith("wkf_gemm"):
                continue
            checked += 1
            assert k[".private_segment_fixed_size"] == 0 and not k[".uses_dynamic_stack"], (k[".name"], k[".private_segment_fixed_size"])
            # (a scalar register parked in a lane of a vector register outside the loop costs nothing and touches no memory)
            assert k[".vgpr_spill_count"] == 0 and k[".sgpr_spill_count"] <= 8, (k[".name"], k[".vgpr_spill_count"], k[".sgpr_spill_count"])
            assert k[".vgpr_count"] <= 512
    assert checked >= 40, f"only {checked} GEMM kernels were compiled: the shapes above no longer reach the variants"


def test_team_row_kernels_fit_four_workgroups_per_compute_unit(tmp_path):
    # The workgroups of a team wait for each other, so the host sizes the grid for four resident workgroups of 256
    # lanes per compute unit.  That holds when a kernel needs at most 128 vector registers and no scratch memory;
    # the launch bounds ask the compiler for exactly that, and its own record in each code object must show it.
    import glob
    import subprocess
    import sys
    script = (
        "import sys, numpy as np\n"
        f"sys.path.insert(0, {os.path.join(ROOT, 'tests')!r})\n"
        "from helpers import load_package\n"
        "w = load_package(); dev = w.Device.planner(); T = w.Tensor\n"
        "for dt, n in ((np.float32, 100003), (np.float32, 131072), (np.float16, 262144), (np.float16, 140002)):\n"
        "    x = T.new(dev, np.zeros((8, n), dtype=dt)); wt = T.new(dev, np.zeros((n,), dtype=dt))\n"
        "    for t in (x.softmax_last_dim(), x.layer_norm(wt, 1e-5)):\n"
        "        t.materialize()\n"
        "        assert any('teams of' in k.detail for k in t.kernels()), [k.detail for k in t.kernels()]\n"
        "dev.set_row_teams(True, (1 << 31) | 64)\n"
        "T.new(dev, np.zeros((8, 100003), dtype=np.float32)).softmax_last_dim().materialize()\n"
    )
    env = dict(os.environ, WKF_CACHE_DIR=str(tmp_path))
    subprocess.run([sys.executable, "-c", script], check=True, env=env, timeout=900)
    checked = 0
    for path in glob.glob(os.path.join(str(tmp_path), "*.hsaco")):
        for k in _code_object_kernels(path):
            if not k[".name"].startswith("wkf_row"):
                continue
            checked += 1
            assert k[".private_segment_fixed_size"] == 0 and not k[".uses_dynamic_stack"], (k[".name"], k[".private_segment_fixed_size"])
            assert k[".vgpr_spill_count"] == 0 and k[".sgpr_spill_count"] == 0, (k[".name"], k[".vgpr_spill_count"])
            assert k[".vgpr_count"] <= 128, (k[".name"], k[".vgpr_count"])
            assert k[".max_flat_workgroup_size"] == 256
    assert checked >= 6, f"only {checked} team kernels were compiled"
