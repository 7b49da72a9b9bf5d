"""Host-side logic of libdeepracin.so that needs no GPU: exported C-ABI, stored-format reader/writer,
execution order, buffer planner, error behaviour, list cursor rules.  No compute call is made here.
"""
import ctypes
import filecmp
import os
import re

import numpy as np
import pytest

import deepracin_amd as dr
from deepracin_amd import configs
from conftest import GOLDEN, ROOT

MODEL = os.path.join(GOLDEN, "squeezenet_whole")


# ---------------------------------------------------------------------------------------------
# C-ABI surface
# ---------------------------------------------------------------------------------------------

def declared_symbols():
    names = set()
    for header in ("deepRACIN.h", "dR_nodes.h", "dr_hip.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        for m in re.finditer(r"\b((?:dR|drhip)_\w+)\s*\(", text):
            names.add(m.group(1))
    return sorted(names)


def test_library_exports_every_declared_symbol(lib):
    syms = declared_symbols()
    assert len(syms) > 60
    raw = ctypes.CDLL(dr.LIB_PATH)
    missing = [s for s in syms if not hasattr(raw, s)]
    assert not missing, "declared in include/*.h but not exported: %s" % missing
    for must in ("dR_NewGraph", "dR_loadGraph", "dR_feedData", "dR_prepare", "dR_apply", "dR_getOutputBuffers",
                 "dR_downloadArray", "drhip_conv3x3_winograd_f32", "drhip_conv1x1_f32", "drhip_fc_f32"):
        assert must in syms


def test_every_symbol_the_reference_python_wrapper_looks_up_resolves(lib):
    """tests/golden/ref_wrapper_symbols.txt lists the lib.dR_* names of the reference's ctypes front-end
    (python/deepracin/__init__.py.in:36-218 bind at import; a few more are looked up when called).  All
    must resolve, or the unmodified wrapper stops with AttributeError before any graph is built."""
    names = open(os.path.join(GOLDEN, "ref_wrapper_symbols.txt")).read().split()
    assert len(names) >= 35 and "dR_MaskDependentFilter" in names and "dR_apply" in names
    raw = ctypes.CDLL(dr.LIB_PATH)
    missing = [s for s in names if not hasattr(raw, s)]
    assert not missing, "looked up by the reference wrapper but not exported: %s" % missing


def test_constructors_outside_the_layer_path_refuse(lib, capfd):
    """Image-filter, two-tensor, RoI, colour, upscaling, label and crop constructors exist for the wrapper's
    import only: they append nothing and return NULL."""
    raw = ctypes.CDLL(dr.LIB_PATH)
    g = lib.dR_NewGraph()
    sh = (ctypes.c_int * 4)(3, 3, 1, 1)
    for name, args in (("dR_RGB2gray", (g, None)), ("dR_ResolveRoI", (g, None, sh)), ("dR_CropOrPad", (g, None, sh)),
                       ("dR_ElemWise2Operation", (g, None, None, 0)), ("dR_Upscaling", (g, None, 0, 2, 2)),
                       ("dR_MaskDependentFilter", (g, None, None, sh)), ("dR_PerPixelFilter", (g, None, None, sh, sh)),
                       ("dR_LabelCreation", (g, None, 0, ctypes.c_float(0), ctypes.c_float(0), ctypes.c_float(0)))):
        f = getattr(raw, name)
        f.restype = ctypes.c_void_p
        assert f(*args) is None, name
    raw.dR_MaskDependentFilter_setVariables.restype = None
    raw.dR_MaskDependentFilter_setVariables(None, None, None)
    out = capfd.readouterr().out
    assert out.count("outside the CNN layer path") == 9


def test_no_device_is_reported_not_faked(lib):
    # on a machine without a GPU the device layer says so; on a GPU box it initialises
    info = dr.DeviceInfo()
    rc = lib.drhip_init(0, info)
    if lib.drhip_device_count() == 0:
        assert rc == -3 and b"no HIP device" in lib.drhip_last_error()
    else:
        assert rc == 0 and info.arch.startswith(b"gfx950")


# ---------------------------------------------------------------------------------------------
# stored format
# ---------------------------------------------------------------------------------------------

def test_load_stored_model_and_roundtrip_bytes(lib, tmp_path):
    with dr.Environment() as env:
        g = env.create_graph()
        nodes, feeds = dr.load_graph(g, MODEL)
        assert len(nodes) == 48 and len(feeds) == 1 and feeds[0].shape == [224, 224, 3]
        types = [dr.node_struct(n).type for n in nodes]
        assert types.count(3) == 26 and types.count(16) == 9 and types.count(15) == 3      # conv, concat, slice
        assert [dr.node_struct(n).layerID for n in nodes] == list(range(48))
        dr.save_graph(g, str(tmp_path))
    out = tmp_path / "dr_graph_export"
    assert filecmp.cmp(str(out / "graph.dr"), os.path.join(MODEL, "graph.dr"), shallow=False)
    for i in range(52):
        assert filecmp.cmp(str(out / ("%d.var" % i)), os.path.join(MODEL, "%d.var" % i), shallow=False)
    # and the written model loads again into the same topology
    with dr.Environment() as env:
        g = env.create_graph()
        nodes2, _ = dr.load_graph(g, str(out))
        assert len(nodes2) == 48


def test_saved_synthetic_graph_has_reference_grammar(lib, tmp_path):
    spec, _, outs = configs.fire_module(seed=3, size=9, cin=8, squeeze=4, expand=8)
    with dr.Environment() as env:
        g = env.create_graph()
        configs.build_graph(g, spec, outs)
        dr.save_graph(g, str(tmp_path))
    text = open(tmp_path / "dr_graph_export" / "graph.dr").read()
    lines = text.split("\n")
    assert lines[0] == "deepRACIN graph: 5 nodes, 1 feed nodes" and text.endswith("\n")
    assert lines[1:6] == ["Node 0: DataFeedNode", "params: 9 9 8", "previous_nodes:", "next_nodes: 1", "variable_files:"]
    assert lines[6:11] == ["Node 1: Conv2D", "params: 1 1 1 1 8 4 1 1 1 1", "previous_nodes: 0", "next_nodes: 2 3",
                           "variable_files: 0.var 1.var"]
    assert lines[21:26] == ["Node 4: Concat", "params: 2 2", "previous_nodes: 2 3", "next_nodes:", "variable_files:"]
    w = np.fromfile(tmp_path / "dr_graph_export" / "0.var", dtype="<f4")
    assert np.array_equal(w, spec[1]["w"].reshape(-1))


def _expect_load_failure(tmp_path, text, files=()):
    d = tmp_path / "m"
    d.mkdir(exist_ok=True)
    (d / "graph.dr").write_text(text)
    for name, arr in files:
        np.asarray(arr, "<f4").tofile(d / name)
    with dr.Environment() as env:
        g = env.create_graph()
        with pytest.raises(RuntimeError):
            dr.load_graph(g, str(d))


def test_loader_error_paths(lib, tmp_path):
    feed = "Node 0: DataFeedNode\nparams: 4 4 2\nprevious_nodes:\nnext_nodes: 1\nvariable_files:\n"
    # missing file
    with dr.Environment() as env:
        g = env.create_graph()
        with pytest.raises(RuntimeError):
            dr.load_graph(g, str(tmp_path / "nowhere"))
    # unknown node type
    _expect_load_failure(tmp_path, "deepRACIN graph: 2 nodes, 1 feed nodes\n" + feed +
                         "Node 1: Bogus\nparams:\nprevious_nodes: 0\nnext_nodes:\nvariable_files:\n")
    # node type of the reference that is outside the CNN layer path
    _expect_load_failure(tmp_path, "deepRACIN graph: 2 nodes, 1 feed nodes\n" + feed +
                         "Node 1: RGB2Gray\nparams:\nprevious_nodes: 0\nnext_nodes:\nvariable_files:\n")
    # wrong parameter count for a conv
    _expect_load_failure(tmp_path, "deepRACIN graph: 2 nodes, 1 feed nodes\n" + feed +
                         "Node 1: Conv2D\nparams: 1 1 3 3 2\nprevious_nodes: 0\nnext_nodes:\nvariable_files: 0.var 1.var\n",
                         [("0.var", np.zeros(36)), ("1.var", np.zeros(2))])
    # variable file shorter than the tensor it should hold
    _expect_load_failure(tmp_path, "deepRACIN graph: 2 nodes, 1 feed nodes\n" + feed +
                         "Node 1: Conv2D\nparams: 1 1 3 3 2 2 1 1 1 1\nprevious_nodes: 0\nnext_nodes:\nvariable_files: 0.var 1.var\n",
                         [("0.var", np.zeros(10)), ("1.var", np.zeros(2))])
    # forward reference
    _expect_load_failure(tmp_path, "deepRACIN graph: 2 nodes, 1 feed nodes\n" + feed +
                         "Node 1: Softmax\nparams:\nprevious_nodes: 1\nnext_nodes:\nvariable_files:\n")
    # a loader only fills an empty graph
    with dr.Environment() as env:
        g = env.create_graph()
        dr.feed_node(g, [4, 4, 2])
        with pytest.raises(RuntimeError):
            dr.load_graph(g, MODEL)


def test_normalization_node_format_roundtrip(lib, tmp_path):
    """graph.dr grammar of the Normalization node: 3 parameters `type mean dev` written with %d %f %f
    (reference src/dR_nodes_misc.c:1103-1105), read back into the same node."""
    with dr.Environment() as env:
        g = env.create_graph()
        f = dr.feed_node(g, [6, 5, 3])
        n = dr.Normalization(f, "target_mean_dev", 0.25, 2.0)
        dr.Softmax(n)
        dr.save_graph(g, str(tmp_path))
    lines = open(tmp_path / "dr_graph_export" / "graph.dr").read().split("\n")
    assert lines[6:11] == ["Node 1: Normalization", "params: 2 0.250000 2.000000", "previous_nodes: 0", "next_nodes: 2", "variable_files:"]
    with dr.Environment() as env:
        g = env.create_graph()
        nodes, feeds = dr.load_graph(g, str(tmp_path / "dr_graph_export"))
        assert [dr.node_struct(x).type for x in nodes] == [12, 7, 14]          # feed, normalization, softmax
        assert lib.dR_propagateShapesAndSchedule(g.ptr) == 1
        s = dr.node_struct(nodes[1]).oshape
        f0 = dr.node_struct(nodes[0]).oshape
        assert (s.s0, s.s1, s.s2) == (f0.s0, f0.s1, f0.s2) and sorted((s.s0, s.s1, s.s2)) == [3, 5, 6]
        dr.save_graph(g, str(tmp_path / "again"))
    assert filecmp.cmp(str(tmp_path / "again" / "dr_graph_export" / "graph.dr"), str(tmp_path / "dr_graph_export" / "graph.dr"), shallow=False)
    # wrong parameter count / unknown type are refused
    feed = "Node 0: DataFeedNode\nparams: 4 4 2\nprevious_nodes:\nnext_nodes: 1\nvariable_files:\n"
    _expect_load_failure(tmp_path, "deepRACIN graph: 2 nodes, 1 feed nodes\n" + feed +
                         "Node 1: Normalization\nparams: 2 0.0\nprevious_nodes: 0\nnext_nodes:\nvariable_files:\n")
    _expect_load_failure(tmp_path, "deepRACIN graph: 2 nodes, 1 feed nodes\n" + feed +
                         "Node 1: Normalization\nparams: 5 0.0 1.0\nprevious_nodes: 0\nnext_nodes:\nvariable_files:\n")


# ---------------------------------------------------------------------------------------------
# prepare-time errors (host side only: fail before any device call)
# ---------------------------------------------------------------------------------------------

def test_prepare_and_shape_errors(lib):
    with dr.Environment() as env:
        g = env.create_graph()
        assert lib.dR_propagateShapesAndSchedule(g.ptr) == 0            # no feed node
        mem = (ctypes.c_void_p * 10)()
        assert lib.dR_getOutputBuffers(g.ptr, mem) == 0                 # not prepared
        assert lib.dR_apply(g.ptr) == 0
    rng = np.random.default_rng(0)
    w = rng.standard_normal((2, 3, 3, 3)).astype(np.float32)
    with dr.Environment() as env:                                       # conv stride larger than the image -> zero shape
        g = env.create_graph()
        spec = [{"op": "feed", "shape": (2, 2, 2)}, {"op": "conv", "in": 0, "w": w, "b": None, "stride": (4, 4), "relu": False}]
        configs.build_graph(g, spec, [1])
        assert lib.dR_propagateShapesAndSchedule(g.ptr) == 0
    with dr.Environment() as env:                                       # FC input size mismatch
        g = env.create_graph()
        spec = [{"op": "feed", "shape": (2, 2, 2)}, {"op": "fc", "in": 0, "w": np.zeros((9, 4), np.float32), "b": None, "relu": False}]
        configs.build_graph(g, spec, [1])
        assert lib.dR_propagateShapesAndSchedule(g.ptr) == 0
    with dr.Environment() as env:                                       # conv channel mismatch
        g = env.create_graph()
        spec = [{"op": "feed", "shape": (4, 4, 3)}, {"op": "conv", "in": 0, "w": w, "b": None, "stride": (1, 1), "relu": False}]
        configs.build_graph(g, spec, [1])
        assert lib.dR_propagateShapesAndSchedule(g.ptr) == 0


def test_shape_rules(lib):
    # conv: floor(in/stride); pool: ceil(in/stride); fc: (N,1,1)   (reference conv2d.c:115, pooling.c:201, fc.c:302)
    spec, _, outs = configs.squeezenet11(seed=1)
    with dr.Environment() as env:
        g = env.create_graph()
        nodes = configs.build_graph(g, spec, outs)
        assert lib.dR_propagateShapesAndSchedule(g.ptr) == 1
        shapes = [(dr.node_struct(n).oshape.s0, dr.node_struct(n).oshape.s1, dr.node_struct(n).oshape.s2) for n in nodes]
    _, want = configs.flops(spec)
    assert shapes == [tuple(s) for s in want]
    assert shapes[1] == (112, 112, 64) and shapes[2] == (56, 56, 64) and shapes[-1] == (1, 1, 1000)
    with dr.Environment() as env:
        g = env.create_graph()
        spec = [{"op": "feed", "shape": (55, 55, 4)}, {"op": "pool", "in": 0, "window": (3, 3, 1), "stride": (2, 2, 1), "kind": 0}]
        nodes = configs.build_graph(g, spec, [1])
        assert lib.dR_propagateShapesAndSchedule(g.ptr) == 1
        s = dr.node_struct(nodes[1]).oshape
        assert (s.s0, s.s1, s.s2) == (28, 28, 4)


# ---------------------------------------------------------------------------------------------
# execution order and buffer plan
# ---------------------------------------------------------------------------------------------

def reference_order(spec):
    """The reference's work-list walk (src/dR_core.c:121-211) restated over a layer list."""
    consumers = {i: [] for i in range(len(spec))}
    inputs = {}
    for i, n in enumerate(spec):
        ins = n.get("ins", [n["in"]] if "in" in n else [])
        inputs[i] = ins
        for j in ins:
            consumers[j].append(i)
    done, queued, work, order = set(), set(), [], []
    for i, n in enumerate(spec):
        if n["op"] == "feed":
            done.add(i)
            for c in consumers[i]:
                if c not in queued:
                    queued.add(c); work.append(c)
    while work:
        n = work.pop(0)
        if not all(j in done for j in inputs[n]):
            work.append(n)
            continue
        done.add(n); order.append(n)
        for c in consumers[n]:
            if c not in queued:
                queued.add(c); work.append(c)
    return order


class FullHandler(ctypes.Structure):
    pass


FullHandler._fields_ = [("outputFor", ctypes.c_void_p), ("size", ctypes.c_int), ("numberOfDependencies", ctypes.c_int),
                        ("bufptr", ctypes.c_void_p), ("buf", ctypes.c_void_p), ("outputBuf", ctypes.c_int),
                        ("regionOfInterest", ctypes.c_int), ("useIndexBufferForRoI", ctypes.c_int),
                        ("indexBuffer", ctypes.c_void_p), ("index", ctypes.c_int), ("roiOrigin", dr.Shape3),
                        ("drViewOf", ctypes.POINTER(FullHandler)), ("drViewOffset", ctypes.c_int),
                        ("drFirstDef", ctypes.c_int), ("drLastUse", ctypes.c_int), ("drPinned", ctypes.c_int)]


def plan_of(graph, nodes):
    """[(physical id, offset, size)] per node after dR_planBuffers."""
    out = []
    for n in nodes:
        hp = ctypes.cast(dr.node_struct(n).outputBuf, ctypes.POINTER(FullHandler))
        h = hp.contents
        if h.drViewOf:
            out.append((ctypes.addressof(h.drViewOf.contents), h.drViewOffset, h.size, h.drViewOf.contents.size))
        else:
            out.append((ctypes.addressof(h), 0, None, h.size))
    return out


@pytest.mark.parametrize("name", ["fire", "vgg_conv3", "squeezenet", "stored"])
def test_schedule_order_and_buffer_plan(lib, oracle, name):
    with dr.Environment() as env:
        g = env.create_graph()
        if name == "stored":
            nodes, _ = dr.load_graph(g, MODEL)
            spec = oracle.parse_graph_dir(MODEL)
            outs = [47]
            dr.mark_as_output(nodes[47])
        else:
            kw = {"size": 32} if name == "squeezenet" else {}
            spec, _, outs = configs.CONFIGS[name](seed=2, **kw)
            nodes = configs.build_graph(g, spec, outs)
        assert lib.dR_propagateShapesAndSchedule(g.ptr) == 1
        pos = [dr.node_struct(n).drSchedulePos for n in nodes]
        order = [i for _, i in sorted((p, i) for i, p in enumerate(pos) if p >= 0)]
        assert order == reference_order(spec)
        assert lib.dR_planBuffers(g.ptr) == 1
        plan = plan_of(g, nodes)
        vol = [dr.node_struct(n).oshape.s0 * dr.node_struct(n).oshape.s1 * dr.node_struct(n).oshape.s2 for n in nodes]

    inputs = {i: n.get("ins", [n["in"]] if "in" in n else []) for i, n in enumerate(spec)}
    last_use = {i: pos[i] for i in range(len(spec))}
    for i, ins in inputs.items():
        for j in ins:
            last_use[j] = max(last_use[j], pos[i])
    # a 1x1 layer behind a 3x3/2 max pool that nobody else reads pools while it loads: it reads the tensor
    # in FRONT of the pooling node, which therefore has to stay intact until that layer has run
    for i, n in enumerate(spec):
        if n["op"] == "conv" and tuple(n["w"].shape[2:]) == (1, 1) and spec[n["in"]]["op"] == "pool":
            pl = spec[n["in"]]
            if tuple(pl["window"]) == (3, 3, 1) and tuple(pl["stride"]) == (2, 2, 1) and pl["kind"] == 0:
                last_use[pl["in"]] = max(last_use[pl["in"]], pos[i])
    fused_into = {}
    # a max pool stored by the convolution in front of it: the convolution then owns no tensor of
    # its own, only the pooled one in the pooling node's buffer
    for i, n in enumerate(spec):
        if n["op"] == "pool" and plan[n["in"]][0] == plan[i][0]:
            j = n["in"]
            # 2x2/2 behind a Winograd convolution, or 3x3/2 behind a first layer (3x3 filter, <= 4 input channels)
            assert spec[j]["op"] == "conv" and tuple(n["stride"]) == (2, 2, 1) and n["kind"] == 0
            k = spec[j]["w"].shape
            assert tuple(n["window"]) == (2, 2, 1) or (tuple(n["window"]) == (3, 3, 1) and k[0] <= 4 and tuple(k[2:]) == (3, 3))
            assert plan[j][1] == plan[i][1] == 0 and j not in outs
            assert sum(1 for k in inputs if j in inputs[k]) == 1
            fused_into[j] = i
            vol[j] = vol[i]
    if name == "vgg_conv3":
        assert any(spec[i]["op"] == "pool" for i in fused_into.values()), "max pools should be absorbed by their convolutions"
    region = {i: (plan[i][0], plan[i][1], plan[i][1] + vol[i]) for i in range(len(spec))}
    for i in range(len(spec)):
        assert plan[i][3] >= plan[i][1] + vol[i], "node %d does not fit its buffer" % i
    for i, n in enumerate(spec):
        if n["op"] == "concat" and all(plan[j][0] == plan[i][0] for j in n["ins"]):
            off = 0
            for j in n["ins"]:
                assert plan[j][1] == off, "producer %d not at its channel offset" % j
                off += vol[j]
                fused_into[j] = i
    if name in ("fire", "squeezenet", "stored"):
        assert fused_into, "channel concats should absorb their producers"

    def overlaps(a, b):
        return a[0] == b[0] and a[1] < b[2] and b[1] < a[2]

    # brute-force liveness: when node i writes, no other tensor that is still needed may share its bytes
    for i in range(len(spec)):
        if pos[i] < 0:
            continue
        for j in range(len(spec)):
            if j == i or fused_into.get(j) == i or fused_into.get(i) == j:
                continue
            if j in fused_into and i in fused_into and fused_into[i] == fused_into[j]:
                assert not overlaps(region[i], region[j])
                continue
            live = (pos[j] < pos[i] <= last_use[j]) or spec[j]["op"] == "feed" or j in outs
            if live and pos[j] <= pos[i]:
                assert not overlaps(region[i], region[j]), "node %d overwrites live tensor %d" % (i, j)
    # feed and output tensors own their storage
    pinned = [i for i, n in enumerate(spec) if n["op"] == "feed"] + list(outs)
    for i in pinned:
        assert sum(1 for j in range(len(spec)) if plan[j][0] == plan[i][0] and fused_into.get(j) != i) == 1
    # and recycling does happen on the deep nets
    if name in ("squeezenet", "stored"):
        assert len({p[0] for p in plan}) < len(spec) // 2


def _odd_offset_norm_spec():
    """feed 5x5x3 -> {1x1 conv to 3 channels (75 floats), Normalization} -> channel concat."""
    rng = np.random.default_rng(5)
    w = rng.standard_normal((3, 3, 1, 1)).astype(np.float32)
    spec = [{"op": "feed", "shape": (5, 5, 3)},
            {"op": "conv", "in": 0, "w": w, "b": None, "stride": (1, 1), "relu": False},
            {"op": "norm", "in": 0, "kind": 2, "mean": 0.0, "dev": 1.0},
            {"op": "concat", "ins": [1, 2], "dim": 2}]
    x = rng.standard_normal((3, 5, 5)).astype(np.float32)
    return spec, x


def test_normalization_is_never_planned_at_an_unaligned_concat_offset(lib):
    """The normalization kernels move 16 bytes per lane.  Behind a producer of 75 floats the fused concat
    would put the Normalization node at byte offset 300: the planner must not fuse such a concat (and may
    fuse it when the normalization comes first, at offset 0)."""
    spec, _ = _odd_offset_norm_spec()
    for ins, fused in (([1, 2], False), ([2, 1], True)):
        spec[3] = {"op": "concat", "ins": ins, "dim": 2}
        with dr.Environment() as env:
            g = env.create_graph()
            nodes = configs.build_graph(g, spec, [3])
            assert lib.dR_propagateShapesAndSchedule(g.ptr) == 1 and lib.dR_planBuffers(g.ptr) == 1
            plan = plan_of(g, nodes)
        assert (plan[2][0] == plan[3][0]) == fused
        if plan[2][0] == plan[3][0]:
            assert plan[2][1] % 4 == 0


def test_second_prepare_is_refused_not_silently_empty(lib, capfd):
    """A graph is prepared once.  A second walk would find every node already queued and schedule nothing:
    the call must say so and return FALSE, and the first schedule must still stand."""
    spec, _, outs = configs.CONFIGS["fire"](seed=3)
    with dr.Environment() as env:
        g = env.create_graph()
        nodes = configs.build_graph(g, spec, outs)
        assert lib.dR_propagateShapesAndSchedule(g.ptr) == 1
        first = [dr.node_struct(n).drSchedulePos for n in nodes]
        capfd.readouterr()
        assert lib.dR_prepare(g.ptr) == 0
        out = capfd.readouterr().out
        assert "scheduled before" in out and "prepared already" not in out      # (scheduled by hand, never prepared)
        assert [dr.node_struct(n).drSchedulePos for n in nodes] == first


# ---------------------------------------------------------------------------------------------
# list cursor rules and helpers
# ---------------------------------------------------------------------------------------------

def test_list_cursor_rules():
    raw = ctypes.CDLL(dr.LIB_PATH)
    vp = ctypes.c_void_p
    raw.dR_list_createEmptyList.restype = vp
    raw.dR_list_next.restype = vp
    raw.dR_list_pop.restype = vp
    for f in (raw.dR_list_append, raw.dR_list_removeFirstOcc):
        f.argtypes = [vp, vp]
    for f in (raw.dR_list_next, raw.dR_list_pop, raw.dR_list_resetIt, raw.dR_list_cleanup):
        f.argtypes = [vp]
    l = raw.dR_list_createEmptyList()
    for v in (11, 22, 33, 44):
        raw.dR_list_append(l, v)
    assert [raw.dR_list_next(l) for _ in range(5)] == [11, 22, 33, 44, None]      # wraps to reset after the end
    assert raw.dR_list_next(l) == 11 and raw.dR_list_next(l) == 22
    assert raw.dR_list_removeFirstOcc(l, 22) == 1                                  # remove under the cursor
    assert raw.dR_list_next(l) == 33                                               # successor comes next
    raw.dR_list_resetIt(l)
    assert raw.dR_list_next(l) == 11
    assert raw.dR_list_removeFirstOcc(l, 11) == 1                                  # remove the head under the cursor
    assert raw.dR_list_next(l) == 33
    assert raw.dR_list_pop(l) == 33 and raw.dR_list_pop(l) == 44 and raw.dR_list_pop(l) is None
    assert raw.dR_list_removeFirstOcc(l, 5) == 0
    raw.dR_list_cleanup(l)


def test_matmul_helpers():
    raw = ctypes.CDLL(dr.LIB_PATH)
    fp = ctypes.POINTER(ctypes.c_float)
    rng = np.random.default_rng(1)
    a, b = rng.standard_normal((4, 3)).astype(np.float32), rng.standard_normal((3, 5)).astype(np.float32)
    out = np.zeros((4, 5), np.float32)
    assert raw.dR_matmul(a.ctypes.data_as(fp), 4, 3, b.ctypes.data_as(fp), 3, 5, out.ctypes.data_as(fp)) == 1
    assert np.allclose(out, a @ b, atol=1e-6)
    bt = rng.standard_normal((6, 3)).astype(np.float32)
    out2 = np.zeros((4, 6), np.float32)
    assert raw.dR_matmulT(a.ctypes.data_as(fp), 4, 3, bt.ctypes.data_as(fp), 6, 3, out2.ctypes.data_as(fp)) == 1
    assert np.allclose(out2, a @ bt.T, atol=1e-6)
    assert raw.dR_matmul(a.ctypes.data_as(fp), 4, 3, bt.ctypes.data_as(fp), 6, 3, out2.ctypes.data_as(fp)) == 0


def _kernel_line(node):
    """The 'Kernel: ...' line of a conv node's printLayer text (which algorithm schedule() settled on)."""
    fn = ctypes.CFUNCTYPE(ctypes.c_void_p, ctypes.c_void_p)(dr.node_struct(node).printLayer)
    text = ctypes.string_at(fn(node.ptr)).decode()
    return [l for l in text.splitlines() if "Kernel:" in l][0]


def test_layers_beyond_the_packed_argument_fields_take_the_general_kernel(lib):
    """The matrix-core convolution kernels carry W, H, I and O in 16-bit fields: a 3x3 layer with a dimension above
    65535 is scheduled onto the general direct kernel, and a first layer of that size is not fused with its pool."""
    rng = np.random.default_rng(0)
    for width, expect in ((64, "Winograd"), (70000, "direct")):
        with dr.Environment() as env:
            g = env.create_graph()
            x = dr.feed_node(g, [2, width, 1])                                   # HWC: 2 rows, `width` columns
            c = dr.Conv2d_raw(x, rng.standard_normal((1, 2, 3, 3)), None, (1, 1), "relu")
            p = dr.Pooling(c, "max", [1, 3, 3, 1], [1, 2, 2, 1])
            dr.mark_as_output(p)
            assert lib.dR_propagateShapesAndSchedule(g.ptr) == 1
            assert expect in _kernel_line(c), _kernel_line(c)
            assert lib.dR_planBuffers(g.ptr) == 1
            # (the conv is a "first layer": with the stride-1 3x3 filter it is a Winograd node, never the fused
            # first-layer + pool kernel; the wide one, now direct, must not be fused either)
            plan = plan_of(g, [c, p])
            if width > 65535:
                assert plan[0][0] != plan[1][0]                  # the convolution keeps a tensor of its own


def test_layers_beyond_32_bit_byte_offsets_take_the_general_kernels(lib):
    """Every dimension fits the 16-bit argument fields, but the input holds 2^29 elements or more: the matrix-core
    3x3 kernels and the pooling-on-load 1x1 kernel (32-bit byte offsets) are not scheduled for such a layer."""
    rng = np.random.default_rng(0)
    for width, bank in ((64, True), (65000, False)):
        with dr.Environment() as env:                                         # strided 3x3: direct kernel, with or without its filter bank
            g = env.create_graph()
            x = dr.feed_node(g, [1033, width, 8])
            c = dr.Conv2d_raw(x, rng.standard_normal((8, 2, 3, 3)), None, (2, 2), "relu")
            dr.mark_as_output(c)
            assert lib.dR_propagateShapesAndSchedule(g.ptr) == 1
            line = _kernel_line(c)
            assert "direct" in line and (("variant 0" not in line) == bank), line
    class PoolData(ctypes.Structure):                                         # dR_Pooling_Data (include/dR_nodes.h)
        _fields_ = [("ishape", ctypes.c_int * 3), ("shape", ctypes.c_int * 4), ("stride", ctypes.c_int * 4), ("poolingType", ctypes.c_int),
                    ("shaderSrc", ctypes.c_void_p), ("useLMEM", ctypes.c_int), ("drFused", ctypes.c_int)]
    for width, fused in ((64, True), (65000, False)):
        with dr.Environment() as env:                                         # 3x3/2 max pool -> 1x1 conv
            g = env.create_graph()
            x = dr.feed_node(g, [1033, width, 8])
            p = dr.Pooling(x, "max", [1, 3, 3, 1], [1, 2, 2, 1])
            c = dr.Conv2d_raw(p, rng.standard_normal((8, 2, 1, 1)), None, (1, 1), "relu")
            dr.mark_as_output(c)
            assert lib.dR_propagateShapesAndSchedule(g.ptr) == 1
            assert lib.dR_planBuffers(g.ptr) == 1
            pd = ctypes.cast(dr.node_struct(p).layer, ctypes.POINTER(PoolData)).contents
            assert bool(pd.drFused) == fused, (width, pd.drFused)


def test_c_host_program_compiles_against_the_public_headers(lib, tmp_path):
    """tests/c_caller.c: plain C11 against include/deepRACIN.h, with one _Static_assert per field of the structs a
    host program of the reference reaches into (offsets from the reference's own header, tests/golden/
    ref_struct_offsets.h).  Compiling it is the layout check; it links against the library without a GPU."""
    from deepracin_amd import build
    exe = build.build_c_caller(out=str(tmp_path / "c_caller"), verbose=False)
    import subprocess
    r = subprocess.run([exe], capture_output=True, text=True, timeout=60)
    assert r.returncode == 2 and "usage" in r.stderr


def test_pick_variants_are_launchable(lib):
    for (W, H, I, O) in [(224, 224, 3, 64), (224, 224, 64, 64), (56, 56, 256, 256), (14, 14, 512, 512), (55, 55, 16, 64), (1, 1, 1, 1)]:
        v = lib.drhip_conv3x3_winograd_pick_variant(W, H, I, O)
        assert v >= 1
        c = lib.drhip_conv1x1_pick_variant(W * H, I, O)          # waves per tile | 0x100 for 16x16 tiles
        assert (c in (1, 2, 4, 8)) or (c & 0x100 and (c & 0xff) in (1, 2, 4, 8, 16) and c >> 9 == 0)


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU: any other --gpus value ends with a message, not with a number."""
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "exactly one GPU" in (r.stdout + r.stderr)
    assert not r.stdout.strip().startswith("{")
