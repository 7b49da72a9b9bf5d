"""End-to-end parity through the deepRacin C graph API (dR_NewGraph ... dR_downloadArray) on the GPU.

Every benchmark configuration is built from seeded synthetic tensors, run through libdeepracin.so and
compared with the CPU oracle evaluating the same layer list.  Bars (north star): per-layer max
relative error <= 1e-4 (max|gpu-oracle| / max|oracle| of that layer), final logits max abs error
<= 1e-3 with identical argmax, pooling bit-exact given equal inputs.
"""
import ctypes
import os

import numpy as np
import pytest

import deepracin_amd as dr
from deepracin_amd import configs
from conftest import GOLDEN, assert_close, rel_err, spec_terms

pytestmark = pytest.mark.gpu

LAYER_TOL = 1e-4
LOGIT_TOL = 1e-3


class _Handler(ctypes.Structure):
    _fields_ = [("outputFor", ctypes.c_void_p), ("size", ctypes.c_int), ("numberOfDependencies", ctypes.c_int),
                ("bufptr", ctypes.POINTER(ctypes.c_void_p)), ("buf", ctypes.c_void_p)]


class _NodeHead(ctypes.Structure):
    _fields_ = [("oshape", dr.Shape3), ("layerID", ctypes.c_int32), ("previous_layers", ctypes.c_void_p),
                ("next_layers", ctypes.c_void_p), ("clKernel", ctypes.c_void_p), ("outputBuf", ctypes.POINTER(_Handler))]


def node_output(graph, node):
    """Download a node's buffer via the public struct layout (include/dR_types.h) as [C][H][W]."""
    head = ctypes.cast(node.ptr, ctypes.POINTER(_NodeHead)).contents
    s = head.oshape
    flat = np.empty(s.s0 * s.s1 * s.s2, np.float32)
    graph.lib.dR_downloadArray(graph.ptr, b"", head.outputBuf.contents.bufptr, 0, flat.nbytes, flat.ctypes.data_as(ctypes.c_void_p))
    return flat.reshape(s.s2, s.s1, s.s0)


def run_config(name, outputs=None, env_vars=None, **kw):
    spec, feeds, outs = configs.CONFIGS[name](**kw)
    outs = outputs(spec, outs) if callable(outputs) else (outputs or outs)
    old = {k: os.environ.get(k) for k in (env_vars or {})}
    os.environ.update(env_vars or {})
    try:
        with dr.Environment() as env:
            g = env.create_graph()
            nodes = configs.build_graph(g, spec, outs)
            dr.prepare(g)
            for i, a in feeds.items():
                configs.feed_chw(nodes[i], a)
            assert g.lib.dR_apply(g.ptr)
            got = {i: node_output(g, nodes[i]) for i in outs}
            # a second pass over the same buffers must reproduce the first bit for bit
            assert g.lib.dR_apply(g.ptr)
            again = {i: node_output(g, nodes[i]) for i in outs}
    finally:
        for k, v in old.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
    for i in outs:
        assert np.array_equal(got[i], again[i]), "node %d differs between two applies" % i
    return spec, feeds, got


def all_compute_nodes(spec, outs):
    return [i for i, n in enumerate(spec) if n["op"] != "feed"]


def check_layers(oracle, spec, feeds, got, force_direct=False):
    """Two comparisons with the oracle.  End to end (the oracle's own chain of layers): norm-wise 1e-4 per
    node.  Layer by layer (the oracle evaluates every node on the tensors the GPU produced for its
    inputs): norm-wise 1e-4 and element-wise |gpu-oracle| <= 1e-4*|oracle| + 1e-6*max|oracle| -- applied
    to the nodes all of whose inputs are feeds or downloaded tensors."""
    want = oracle.run_spec(spec, feeds, force_direct=force_direct)
    for i, g in got.items():
        assert g.shape == want[i].shape, "node %d shape %s vs %s" % (i, g.shape, want[i].shape)
        e = rel_err(g, want[i])
        assert e <= LAYER_TOL, "node %d (%s): rel err %.3g" % (i, spec[i]["op"], e)
    step = oracle.run_spec(spec, feeds, force_direct=force_direct, inputs_from=got)
    for i, g in got.items():
        ins = spec[i].get("ins", [spec[i]["in"]] if "in" in spec[i] else [])
        if all(j in got or spec[j]["op"] == "feed" for j in ins):
            assert_close(g, step[i], "node %d (%s) on the GPU's own inputs" % (i, spec[i]["op"]), LAYER_TOL, spec_terms(spec[i]))
    return want


def test_config1_conv3x3_winograd_and_direct(oracle, gpu):
    spec, feeds, got = run_config("conv3x3")
    check_layers(oracle, spec, feeds, got)
    spec, feeds, got_d = run_config("conv3x3", env_vars={"DR_CONV3X3": "direct"})
    check_layers(oracle, spec, feeds, got_d, force_direct=True)
    truth = oracle.run_spec(spec, feeds, f64=True)[1]
    assert rel_err(got[1], truth) <= LAYER_TOL and rel_err(got_d[1], truth) <= LAYER_TOL


def test_config2_fire_module(oracle, gpu):
    # default: only the concat is an output -> producers write straight into the concat buffer
    spec, feeds, got = run_config("fire")
    want = check_layers(oracle, spec, feeds, got)
    assert got[4].shape == (128, 55, 55)
    # every node an output -> nothing is fused, the concat copies; same numbers
    spec, feeds, got_all = run_config("fire", outputs=all_compute_nodes)
    check_layers(oracle, spec, feeds, got_all)
    # default run: the 1x1 expand rides along in the 3x3 expand's Winograd launch (centre taps), so its
    # channels round differently at the 1e-6 level; with that fusion off the runs agree bit for bit
    assert np.array_equal(got_all[4][64:], got[4][64:]) and rel_err(got[4], got_all[4]) <= 1e-5
    _, _, apart = run_config("fire", env_vars={"DR_FUSE_EXPAND": "0"})
    assert np.array_equal(got_all[4], apart[4])
    assert np.array_equal(got_all[4][:64], got_all[2]) and np.array_equal(got_all[4][64:], got_all[3])
    assert rel_err(got[4], oracle.run_spec(spec, feeds, f64=True)[4]) <= LAYER_TOL
    del want


def test_config3_vgg_conv3_block(oracle, gpu):
    spec, feeds, got = run_config("vgg_conv3", outputs=all_compute_nodes)
    want = check_layers(oracle, spec, feeds, got)
    assert got[4].shape == (256, 28, 28)
    # pooling is bit-exact given the same input: pool the GPU's own conv output on the CPU
    assert np.array_equal(got[4], oracle.pool(got[3], (2, 2, 1), (2, 2, 1), 0))
    del want


def test_maxpool_fused_into_convolution(oracle, gpu):
    """With only the final tensor requested, the last convolution of the block stores the pooled
    tensor itself (no pooling launch); the numbers equal the unfused run bit for bit."""
    spec, feeds, fused = run_config("vgg_conv3")
    _, _, plain = run_config("vgg_conv3", env_vars={"DR_FUSE_POOL": "0"})
    assert np.array_equal(fused[4], plain[4]) and fused[4].shape == (256, 28, 28)
    want = oracle.run_spec(spec, feeds)
    assert_close(fused[4], want[4], "fused pool")
    # the pooling node of the fused run launches nothing
    with dr.Environment() as env:
        g = env.create_graph()
        nodes = configs.build_graph(g, spec, [4])
        dr.prepare(g)
        configs.feed_chw(nodes[0], feeds[0])
        dr.graph_config(g).profilingGPU = 1
        assert g.lib.dR_apply(g.ptr)
        assert dr.node_struct(nodes[4]).drLastKernelMs == 0.0 and dr.node_struct(nodes[3]).drLastKernelMs > 0.0


def test_maxpool_taken_on_load_by_the_1x1_layer_behind_it(oracle, gpu):
    """SqueezeNet's pool3 / pool5 pattern: fire module -> 3x3/2 max pool -> squeeze 1x1.  With only the last
    tensor requested the squeeze layer pools while it loads (no pooling launch, no pooled tensor); with
    DR_FUSE_POOLIN=0 the two kernels run.  Same values to rounding (the channel sum is dealt to a different
    number of waves), and the layer bar against the oracle either way."""
    spec, feeds, outs = configs.fire_module(seed=21, size=27, cin=24, squeeze=8, expand=16)
    st = configs._Streams(22)
    spec.append(configs._maxpool(outs[0], 3, 2)); pool = len(spec) - 1
    spec.append(configs._conv(st, pool, 1, 32, 12)); sq = len(spec) - 1
    want = oracle.run_spec(spec, feeds)
    res = {}
    for flag in ("1", "0"):
        os.environ["DR_FUSE_POOLIN"] = flag
        try:
            with dr.Environment() as env:
                g = env.create_graph()
                nodes = configs.build_graph(g, spec, [sq])
                dr.prepare(g)
                for i, a in feeds.items():
                    configs.feed_chw(nodes[i], a)
                dr.graph_config(g).profilingGPU = 1
                assert g.lib.dR_apply(g.ptr)
                pool_ms = dr.node_struct(nodes[pool]).drLastKernelMs
                dr.graph_config(g).profilingGPU = 0
                assert g.lib.dR_apply(g.ptr) and g.lib.dR_apply(g.ptr)       # recorded, then replayed
                res[flag] = (configs.fetch_chw(g)[0], pool_ms)
        finally:
            os.environ.pop("DR_FUSE_POOLIN", None)
    assert res["1"][1] == 0.0 and res["0"][1] > 0.0, "the pooling node must launch nothing when fused"
    assert res["1"][0].shape == (12, 14, 14)
    assert_close(res["1"][0], want[sq], "squeeze behind pool, fused")
    assert_close(res["0"][0], want[sq], "squeeze behind pool, unfused")
    assert rel_err(res["1"][0], res["0"][0]) <= 1e-5
    # the pooled tensor requested as an output: nothing is fused, and it is there
    with dr.Environment() as env:
        g = env.create_graph()
        nodes = configs.build_graph(g, spec, [pool, sq])
        dr.prepare(g)
        for i, a in feeds.items():
            configs.feed_chw(nodes[i], a)
        assert g.lib.dR_apply(g.ptr)
        got_pool, got_sq = configs.fetch_chw(g)
    assert_close(got_pool, want[pool], "pool as output")
    assert_close(got_sq, want[sq], "squeeze, pool as output")


def test_fc_chain_fused(oracle, gpu):
    """FC -> FC -> softmax: the finishing kernels of the two GEMVs disappear into their consumers
    (3 launches instead of 5) and the probabilities do not change by a bit."""
    rng = np.random.default_rng(5)
    spec = [{"op": "feed", "shape": (4, 4, 64)},
            {"op": "fc", "in": 0, "w": (rng.standard_normal((1024, 2048)) * 0.04).astype(np.float32), "b": (rng.standard_normal(2048) * 0.01).astype(np.float32), "relu": True},
            {"op": "fc", "in": 1, "w": (rng.standard_normal((2048, 1000)) * 0.03).astype(np.float32), "b": (rng.standard_normal(1000) * 0.01).astype(np.float32), "relu": False},
            {"op": "softmax", "in": 2}]
    x = rng.random((64, 4, 4), dtype=np.float32)
    res, launches = {}, {}
    for mode in ("1", "0"):
        os.environ["DR_FUSE_FC"] = mode
        try:
            with dr.Environment() as env:
                g = env.create_graph()
                nodes = configs.build_graph(g, spec, [3])
                dr.prepare(g)
                configs.feed_chw(nodes[0], x)
                assert g.lib.dR_apply(g.ptr) and g.lib.dR_apply(g.ptr)          # captured pass, then its replay
                res[mode] = configs.fetch_chw(g)[0].copy()
                dr.graph_config(g).profilingGPU = 1
                assert g.lib.dR_apply(g.ptr)
                launches[mode] = g.lib.drhip_timing_count()
                assert np.array_equal(configs.fetch_chw(g)[0], res[mode])
        finally:
            os.environ.pop("DR_FUSE_FC", None)
    assert launches == {"1": 3, "0": 5}
    assert np.array_equal(res["1"], res["0"])
    want = oracle.run_spec(spec, {0: x})
    assert rel_err(res["1"], want[3]) <= LAYER_TOL and int(res["1"].argmax()) == int(want[3].argmax())
    # Both GEMV outputs wanted by the caller as well: still 3 launches, the consumers store the
    # finished vectors into the producers' output buffers on the way.
    with dr.Environment() as env:
        g = env.create_graph()
        nodes = configs.build_graph(g, spec, [1, 2, 3])
        dr.prepare(g)
        configs.feed_chw(nodes[0], x)
        assert g.lib.dR_apply(g.ptr) and g.lib.dR_apply(g.ptr)
        outs = [a.copy() for a in configs.fetch_chw(g)]
        dr.graph_config(g).profilingGPU = 1
        assert g.lib.dR_apply(g.ptr) and g.lib.drhip_timing_count() == 3
    assert np.array_equal(outs[2], res["0"])
    for k in range(3):
        assert_close(outs[k], want[k + 1], "fc chain %d" % k)


def test_conv_global_average_softmax_fused(oracle, gpu):
    """1x1 conv -> global average pooling -> softmax (SqueezeNet's tail): the pooling kernel and the
    convolution's tensor disappear; the pooled tensor, an output here, is stored by the softmax."""
    rng = np.random.default_rng(9)
    for tail in ("softmax", "fc"):
        spec = [{"op": "feed", "shape": (13, 11, 24)},
                {"op": "conv", "in": 0, "w": (rng.standard_normal((24, 70, 1, 1)) * 0.3).astype(np.float32), "b": (rng.standard_normal(70) * 0.05).astype(np.float32), "stride": (1, 1), "relu": True},
                {"op": "pool", "in": 1, "window": (13, 11, 1), "stride": (13, 11, 1), "kind": 1}]
        if tail == "softmax":
            spec.append({"op": "softmax", "in": 2})
        else:
            spec.append({"op": "fc", "in": 2, "w": (rng.standard_normal((70, 300)) * 0.2).astype(np.float32), "b": (rng.standard_normal(300) * 0.05).astype(np.float32), "relu": False})
        x = rng.random((24, 11, 13), dtype=np.float32)
        want = oracle.run_spec(spec, {0: x})
        res, launches = {}, {}
        for mode in ("1", "0"):
            os.environ["DR_FUSE_AVGPOOL"] = mode
            try:
                with dr.Environment() as env:
                    g = env.create_graph()
                    nodes = configs.build_graph(g, spec, [2, 3])
                    dr.prepare(g)
                    configs.feed_chw(nodes[0], x)
                    assert g.lib.dR_apply(g.ptr) and g.lib.dR_apply(g.ptr)
                    res[mode] = [a.copy() for a in configs.fetch_chw(g)]
                    dr.graph_config(g).profilingGPU = 1
                    assert g.lib.dR_apply(g.ptr)
                    launches[mode] = g.lib.drhip_timing_count()
            finally:
                os.environ.pop("DR_FUSE_AVGPOOL", None)
        assert launches["0"] - launches["1"] == 1, launches
        for k in range(2):
            assert rel_err(res["1"][k], want[2 + k]) <= LAYER_TOL and rel_err(res["1"][k], res["0"][k]) <= 1e-5


def test_squeezenet_with_normalization_node(oracle, gpu):
    """Config 4 with its per-image normalisation moved into the graph: raw U[0,255) image in, a
    Normalization node (mean 0, deviation 1) in front of conv1."""
    spec, feeds, got = run_config("squeezenet", size=96, normalise_in_graph=True)
    assert spec[1]["op"] == "norm" and float(feeds[0].max()) > 100.0
    want = oracle.run_spec(spec, feeds)
    for i in got:
        assert_close(got[i], want[i], "node %d" % i)
    assert int(got[len(spec) - 1].argmax()) == int(want[-1].argmax())
    # the node alone, as an output
    _, _, only = run_config("squeezenet", outputs=[1], size=96, normalise_in_graph=True)
    assert_close(only[1], want[1], "normalization node")
    assert abs(float(only[1].astype(np.float64).mean())) < 1e-4 and abs(float(only[1].astype(np.float64).std()) - 1.0) < 1e-4


def test_normalization_behind_an_odd_volume_producer_in_a_concat(oracle, gpu):
    """feed 5x5x3 -> {1x1 conv (75 floats), Normalization} -> channel concat: a fused concat would put the
    Normalization node 300 bytes into the buffer, where its 16-byte accesses cannot go; the graph is valid
    in the reference (src/dR_nodes_transform.c:238-281) and must run here in either input order."""
    rng = np.random.default_rng(5)
    w = rng.standard_normal((3, 3, 1, 1)).astype(np.float32)
    x = rng.standard_normal((3, 5, 5)).astype(np.float32)
    for ins in ([1, 2], [2, 1]):
        spec = [{"op": "feed", "shape": (5, 5, 3)},
                {"op": "conv", "in": 0, "w": w, "b": None, "stride": (1, 1), "relu": False},
                {"op": "norm", "in": 0, "kind": 2, "mean": 0.0, "dev": 1.0},
                {"op": "concat", "ins": ins, "dim": 2}]
        want = oracle.run_spec(spec, {0: x})
        with dr.Environment() as env:
            g = env.create_graph()
            nodes = configs.build_graph(g, spec, [3])
            dr.prepare(g)
            configs.feed_chw(nodes[0], x)
            assert g.lib.dR_apply(g.ptr)
            got = configs.fetch_chw(g)[0]
            assert not g.lib.dR_prepare(g.ptr)               # one prepare per graph; refused, the plan stands
            assert g.lib.dR_apply(g.ptr)
            assert np.array_equal(configs.fetch_chw(g)[0], got)
        assert_close(got, want[3], "concat %s" % ins)


def test_layer_wider_than_the_packed_argument_fields(oracle, gpu):
    """A 3x3 layer on a 70000 x 2 map (a width beyond the 16-bit fields the matrix-core kernels carry their shapes
    in) runs on the general direct kernel and gives the oracle's values, with a pooling behind it unfused."""
    rng = np.random.default_rng(6)
    W, H = 70000, 2
    w = (rng.standard_normal((1, 2, 3, 3)) * 0.3).astype(np.float32)
    b = (rng.standard_normal(2) * 0.1).astype(np.float32)
    x = rng.standard_normal((1, H, W)).astype(np.float32)
    spec = [{"op": "feed", "shape": (W, H, 1)},
            {"op": "conv", "in": 0, "w": w, "b": b, "stride": (1, 1), "relu": True},
            {"op": "pool", "in": 1, "window": (3, 3, 1), "stride": (2, 2, 1), "kind": 0}]
    want = oracle.run_spec(spec, {0: x})
    with dr.Environment() as env:
        g = env.create_graph()
        nodes = configs.build_graph(g, spec, [2])
        dr.prepare(g)
        configs.feed_chw(nodes[0], x)
        assert g.lib.dR_apply(g.ptr)
        got = configs.fetch_chw(g)[0]
    assert_close(got, want[2], "pool behind a 70000-wide 3x3 layer", terms=9)


def test_config4_squeezenet(oracle, gpu):
    spec, feeds, got = run_config("squeezenet", outputs=all_compute_nodes)
    want = check_layers(oracle, spec, feeds, got)
    probs, logits = got[len(spec) - 1].reshape(-1), got[len(spec) - 2].reshape(-1)
    wl = want[len(spec) - 2].reshape(-1)
    assert np.abs(logits - wl).max() <= LOGIT_TOL
    assert int(logits.argmax()) == int(wl.argmax()) and int(probs.argmax()) == int(want[-1].argmax())
    assert abs(float(probs.sum()) - 1) < 1e-4
    # fused-concat production run gives the same final numbers as the all-outputs run (the two fusions
    # that change a summation order switched off)
    _, _, prod = run_config("squeezenet", env_vars={"DR_FUSE_EXPAND": "0", "DR_FUSE_AVGPOOL": "0", "DR_FUSE_POOLIN": "0"})
    assert np.array_equal(prod[len(spec) - 1], got[len(spec) - 1])
    # and with the expand pairs of the 8 fire modules fused into single Winograd launches
    _, _, fused = run_config("squeezenet")
    assert rel_err(fused[len(spec) - 1], got[len(spec) - 1]) <= LAYER_TOL
    assert np.abs(fused[len(spec) - 2] - got[len(spec) - 2]).max() <= LOGIT_TOL
    assert int(fused[len(spec) - 1].argmax()) == int(got[len(spec) - 1].argmax())


def test_config5_vgg16(oracle, gpu):
    spec, feeds, got = run_config("vgg16", outputs=all_compute_nodes)
    want = check_layers(oracle, spec, feeds, got)
    logits, wl = got[len(spec) - 2].reshape(-1), want[len(spec) - 2].reshape(-1)
    assert np.abs(logits - wl).max() <= LOGIT_TOL
    assert int(logits.argmax()) == int(wl.argmax())
    probs = got[len(spec) - 1].reshape(-1)
    assert int(probs.argmax()) == int(want[-1].argmax()) and abs(float(probs.sum()) - 1) < 1e-4


@pytest.mark.parametrize("name,cls", [("tiger", 292), ("puzzle", 611)])
def test_stored_squeezenet_known_answer(oracle, gpu, name, cls):
    """The reference's only known answers: its stored SqueezeNet v1.1 on its two example images
    (examples/squeezenet-v1.1/squeezenet_deployed.c:199-207), loaded with dR_loadGraph."""
    img = np.load(os.path.join(GOLDEN, "%s_224_rgb_u8.npy" % name))
    chw = np.ascontiguousarray(img.transpose(2, 0, 1).astype(np.float32))
    with dr.Environment() as env:
        g = env.create_graph()
        nodes, feeds = dr.load_graph(g, os.path.join(GOLDEN, "squeezenet_whole"))
        assert len(nodes) == 48 and feeds[0].shape == [224, 224, 3]
        dr.mark_as_output(nodes[-1])
        dr.mark_as_output(nodes[-2])
        dr.prepare(g)
        configs.feed_chw(feeds[0], chw)
        assert g.lib.dR_apply(g.ptr)
        probs, pooled = [a.reshape(-1) for a in configs.fetch_chw(g)]
    want = oracle.run_graph_dir(os.path.join(GOLDEN, "squeezenet_whole"), chw)
    assert int(probs.argmax()) == cls
    assert np.abs(pooled - want[-2].reshape(-1)).max() <= LOGIT_TOL
    assert rel_err(probs, want[-1].reshape(-1)) <= LAYER_TOL


def test_python_frontend_hwc_roundtrip(oracle, gpu):
    """The wrapper's layout rules: HWC in, HWIO weights, HWC out (reference python wrapper :444-497,:559-562)."""
    rng = np.random.default_rng(3)
    x = rng.random((10, 12, 5), dtype=np.float32)                     # H, W, C
    w = (rng.standard_normal((3, 3, 5, 6)) * 0.2).astype(np.float32)  # H, W, I, O
    b = (rng.standard_normal(6) * 0.1).astype(np.float32)
    with dr.Environment() as env:
        g = env.create_graph("HWC")
        f = dr.feed_node(g, [10, 12, 5])
        c = dr.Conv2d(f, (3, 3, 5, 6), (1, 1, 1, 1), "relu", w, b)
        p = dr.Pooling(c, "max", (1, 2, 2, 1), (1, 2, 2, 1))
        dr.mark_as_output(p)
        dr.prepare(g)
        dr.feed_data(f, x)
        out = dr.apply(g)[0]
    want = oracle.pool(oracle.conv_winograd(x.transpose(2, 0, 1), w.transpose(2, 3, 0, 1), b, relu=True), (2, 2, 1), (2, 2, 1), 0)
    assert out.shape == (5, 6, 6)
    assert rel_err(out, want.transpose(1, 2, 0)) <= LAYER_TOL


def test_feed_and_download_through_pinned_staging(oracle, gpu):
    """dR_feedData goes through the graph's pinned staging area and does not wait for the bus: the caller's
    array must have been read when the call returns (it is overwritten right after each call here), feeds
    with an offset and back-to-back feeds must land where and in the order they were made, and
    DR_STAGING=0 (plain blocking copies) must give the same bytes."""
    spec, feeds, outs = configs.CONFIGS["conv3x3"](seed=5)
    x = feeds[0]
    want = oracle.run_spec(spec, feeds)[outs[0]]
    res = {}
    for flag in ("1", "0"):
        os.environ["DR_STAGING"] = flag
        try:
            with dr.Environment() as env:
                g = env.create_graph()
                nodes = configs.build_graph(g, spec, outs)
                dr.prepare(g)
                assert bool(dr.graph_struct(g).drStaging) == (flag == "1")
                lib, feed = g.lib, nodes[0]
                scratch = np.empty_like(x)
                fp = scratch.ctypes.data_as(dr.POINTER(dr.c_float))
                outs_seen = []
                for rep in range(3):
                    # garbage first, then the real image in two halves from ONE reused host array
                    scratch[...] = -1e30
                    lib.dR_feedData(g.ptr, feed.ptr, fp, 0, x.size)
                    half = x.size // 2
                    flat = scratch.reshape(-1)
                    flat[:half] = x.reshape(-1)[:half] * (rep + 1)
                    lib.dR_feedData(g.ptr, feed.ptr, fp, 0, half)
                    flat[:x.size - half] = x.reshape(-1)[half:] * (rep + 1)          # overwrites what was just fed
                    lib.dR_feedData(g.ptr, feed.ptr, fp, half, x.size - half)
                    scratch[...] = 7e30                                               # and again before the pass runs
                    assert lib.dR_apply(g.ptr)
                    outs_seen.append(configs.fetch_chw(g)[0])
                res[flag] = outs_seen
        finally:
            os.environ.pop("DR_STAGING", None)
    for rep in range(3):
        assert np.array_equal(res["1"][rep], res["0"][rep])
    assert_close(res["1"][0], want, "pass fed through the staging area")
    assert not np.array_equal(res["1"][0], res["1"][1])              # the scaled images really arrived


def test_linearity_at_full_size(gpu):
    """Size-independent property at VGG scale: a bias-free linear conv commutes with scaling and adds."""
    rng = np.random.default_rng(5)
    I, O, S = 128, 256, 56
    w = (rng.standard_normal((I, O, 3, 3)) * np.sqrt(2.0 / (9 * I))).astype(np.float32)
    spec = [{"op": "feed", "shape": (S, S, I)}, {"op": "conv", "in": 0, "w": w, "b": None, "stride": (1, 1), "relu": False}]
    a, b = rng.random((I, S, S), dtype=np.float32), rng.random((I, S, S), dtype=np.float32)
    with dr.Environment() as env:
        g = env.create_graph()
        nodes = configs.build_graph(g, spec, [1])
        dr.prepare(g)
        res = []
        for inp in (a, b, a + 2 * b):
            configs.feed_chw(nodes[0], inp)
            assert g.lib.dR_apply(g.ptr)
            res.append(configs.fetch_chw(g)[0])
    assert rel_err(res[2], res[0] + 2 * res[1]) <= LAYER_TOL


def _run_many(spec, outs, inputs, graph_mode, branches=False):
    old = os.environ.get("DR_HIPGRAPH")
    os.environ["DR_HIPGRAPH"] = "1" if graph_mode else "0"
    os.environ["DR_BRANCHES"] = "1" if branches else "0"
    try:
        with dr.Environment() as env:
            g = env.create_graph()
            nodes = configs.build_graph(g, spec, outs)
            dr.prepare(g)
            res = []
            for x in inputs:
                configs.feed_chw(nodes[0], x)          # eager blocking copy between the replays
                assert g.lib.dR_apply(g.ptr)
                res.append([a.copy() for a in configs.fetch_chw(g)])   # blocking download = sync
            tail = dr.graph_struct(g)
            used_graph = bool(tail.drGraphExec)
            _run_many.groups = tail.drBranchGroups
    finally:
        os.environ.pop("DR_BRANCHES", None)
        if old is None:
            os.environ.pop("DR_HIPGRAPH", None)
        else:
            os.environ["DR_HIPGRAPH"] = old
    return res, used_graph


@pytest.mark.parametrize("name", ["squeezenet", "vgg_conv3"])
def test_launch_graph_replays_equal_node_by_node(gpu, name):
    """dR_apply replays a captured hipGraph after the first pass.  Every replay -- with blocking copies
    and synchronisations of the program in between -- must equal the node-by-node result bit for bit."""
    spec, feeds, outs = configs.CONFIGS[name](seed=9)
    rng = np.random.default_rng(10)
    inputs = [feeds[0]] + [rng.random(feeds[0].shape, dtype=np.float32) for _ in range(4)] + [feeds[0]]
    eager, g0 = _run_many(spec, outs, inputs, graph_mode=False)
    replay, g1 = _run_many(spec, outs, inputs, graph_mode=True)
    assert not g0 and g1, "graph mode flags: eager run used a graph=%s, graph run used a graph=%s" % (g0, g1)
    assert _run_many.groups == 0
    if name == "squeezenet":
        # opt-in: the two expand convolutions of each of the 8 fire modules forked onto side streams
        forked, g2 = _run_many(spec, outs, inputs, graph_mode=True, branches=True)
        assert g2 and _run_many.groups == 8
        for a, b in zip(eager, forked):
            for x, y in zip(a, b):
                assert np.array_equal(x, y)
    for k, (a, b) in enumerate(zip(eager, replay)):
        for x, y in zip(a, b):
            assert np.array_equal(x, y), "replay %d differs from the node-by-node pass" % k
    assert np.array_equal(replay[0][0], replay[-1][0])


# ---------------------------------------------------------------------------------------------
# Random topologies: the buffer planner (live intervals, fused concats, pooled convolutions, joint
# expand launches, deferred GEMV reductions) must give the oracle's values whatever the graph looks
# like and whichever subset of nodes the caller reads.

def _random_spec(seed):
    rng = np.random.default_rng(seed)
    W, H, C = int(rng.integers(5, 30)), int(rng.integers(5, 30)), int(rng.integers(1, 9))
    spec = [{"op": "feed", "shape": (W, H, C)}]
    shapes = [(W, H, C)]

    def conv(src, k, cout, stride=1, relu=True):
        cin = shapes[src][2]
        w = (rng.standard_normal((cin, cout, k, k)) * np.sqrt(2.0 / (k * k * cin))).astype(np.float32)
        b = (rng.standard_normal(cout) * 0.05).astype(np.float32) if rng.random() < 0.8 else None
        spec.append({"op": "conv", "in": src, "w": w, "b": b, "stride": (stride, stride), "relu": relu})
        shapes.append((shapes[src][0] // stride, shapes[src][1] // stride, cout))
        return len(spec) - 1

    cur = 0
    for _ in range(int(rng.integers(3, 8))):
        w_, h_, c_ = shapes[cur]
        kind = rng.choice(["conv3", "conv1", "conv5", "pool2", "pool3", "fire", "branch3", "slice", "scalar", "norm"])
        if kind == "conv3":
            cur = conv(cur, 3, int(rng.integers(1, 40)), relu=bool(rng.integers(0, 2)))
        elif kind == "conv1":
            cur = conv(cur, 1, int(rng.integers(1, 40)))
        elif kind == "conv5" and min(w_, h_) >= 4:
            cur = conv(cur, 5, int(rng.integers(1, 12)), stride=int(rng.integers(1, 3)))
        elif kind in ("pool2", "pool3") and min(w_, h_) >= 2:
            k, s = (2, 2) if kind == "pool2" else (3, 2)
            spec.append({"op": "pool", "in": cur, "window": (k, k, 1), "stride": (s, s, 1), "kind": int(rng.integers(0, 2))})
            shapes.append((-(-w_ // s), -(-h_ // s), c_)); cur = len(spec) - 1
        elif kind == "fire":
            s = conv(cur, 1, int(rng.integers(1, 12)))
            e = int(rng.integers(1, 40))
            a, b = conv(s, 1, e), conv(s, 3, e)
            spec.append({"op": "concat", "ins": [a, b], "dim": 2}); shapes.append((w_, h_, 2 * e)); cur = len(spec) - 1
        elif kind == "branch3":                      # three producers, one of them read twice
            a, b = conv(cur, 3, int(rng.integers(1, 10))), conv(cur, 1, int(rng.integers(1, 10)))
            ins = [a, b, cur] if rng.random() < 0.5 else [b, a, a]
            spec.append({"op": "concat", "ins": ins, "dim": 2})
            shapes.append((w_, h_, sum(shapes[i][2] for i in ins))); cur = len(spec) - 1
        elif kind == "slice" and c_ >= 2:
            z0 = int(rng.integers(0, c_ - 1)); cz = int(rng.integers(1, c_ - z0 + 1))
            x0 = int(rng.integers(0, w_)); cw = int(rng.integers(1, w_ - x0 + 1))
            spec.append({"op": "slice", "in": cur, "origin": (x0, 0, z0), "shape": (cw, h_, cz)})
            shapes.append((cw, h_, cz)); cur = len(spec) - 1
        elif kind == "scalar":
            spec.append({"op": "scalar", "in": cur, "kind": int(rng.integers(0, 3)), "value": float(rng.uniform(0.5, 2.0))})
            shapes.append(shapes[cur]); cur = len(spec) - 1
        elif kind == "norm" and w_ * h_ * c_ > 1:
            spec.append({"op": "norm", "in": cur, "kind": int(rng.integers(0, 3)), "mean": 0.25, "dev": 1.5})
            shapes.append(shapes[cur]); cur = len(spec) - 1
    if rng.random() < 0.6:                           # classifier tail
        w_, h_, c_ = shapes[cur]
        for n_out, relu in ((int(rng.integers(200, 700)), True), (int(rng.integers(2, 300)), False)):
            k = shapes[cur][0] * shapes[cur][1] * shapes[cur][2]
            spec.append({"op": "fc", "in": cur, "w": (rng.standard_normal((k, n_out)) * np.sqrt(2.0 / k)).astype(np.float32),
                         "b": (rng.standard_normal(n_out) * 0.05).astype(np.float32), "relu": relu})
            shapes.append((n_out, 1, 1)); cur = len(spec) - 1
        spec.append({"op": "softmax", "in": cur}); shapes.append(shapes[cur]); cur = len(spec) - 1
    x = rng.random((C, H, W), dtype=np.float32) + np.float32(0.1)
    compute = [i for i in range(1, len(spec))]
    some = sorted(set([cur] + [int(i) for i in rng.choice(compute, size=min(2, len(compute)), replace=False)]))
    return spec, x, some


@pytest.mark.parametrize("seed", range(48 * int(os.environ.get("DR_SWEEP_SCALE", "1"))))    # (a one-off wider run: DR_SWEEP_SCALE=n)
def test_random_topologies(oracle, gpu, seed):
    spec, x, some = _random_spec(1000 + seed)
    want = oracle.run_spec(spec, {0: x})
    if not all(np.isfinite(a).all() for a in want if a is not None):
        pytest.skip("degenerate draw: a Normalization node met a constant tensor (deviation 0)")
    for outs in (some, [i for i in range(1, len(spec))]):
        with dr.Environment() as env:
            g = env.create_graph()
            nodes = configs.build_graph(g, spec, outs)
            dr.prepare(g)
            configs.feed_chw(nodes[0], x)
            for rep in range(2):                         # the captured pass, then a replay
                assert g.lib.dR_apply(g.ptr)
                got = configs.fetch_chw(g)
                for i, a in zip(outs, got):
                    assert a.shape == want[i].shape, (seed, i, spec[i]["op"], a.shape, want[i].shape)
                    if rel_err(a, want[i]) > LAYER_TOL:
                        k = int(np.abs(a - want[i]).argmax())
                        raise AssertionError("seed %d, %d outputs, pass %d: node %d (%s) of %s: element %d of %d is %r, the oracle has %r; "
                                             "%d elements differ by more than 1e-4 of the largest" % (
                                                 seed, len(outs), rep, i, spec[i]["op"], [s["op"] for s in spec], k, a.size, a.reshape(-1)[k],
                                                 want[i].reshape(-1)[k], int((np.abs(a - want[i]) > 1e-4 * np.abs(want[i]).max()).sum())))
                if len(outs) == len(spec) - 1:           # every tensor downloaded: judge each layer on the GPU's own inputs
                    step = oracle.run_spec(spec, {0: x}, inputs_from=dict(zip(outs, got)))
                    for i, a in zip(outs, got):
                        assert_close(a, step[i], "seed %d node %d (%s) of %s" % (seed, i, spec[i]["op"], [s["op"] for s in spec]),
                                     terms=spec_terms(spec[i]))
