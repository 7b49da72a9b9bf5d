"""The drop-in boundary beyond the seven calls of a plain forward pass: the library bound exactly as the
reference's own ctypes wrapper declares it, and the exported calls a host program may use to bring its
own buffers, stream, debug download and profiling switches (reference include/deepRACIN.h:72,126,242,
src/deepRACIN.c:204-270).  Everything goes through the C-ABI of libdeepracin.so and is checked against
the CPU oracle.
"""
import ctypes
import os
from ctypes import POINTER, c_bool, c_char_p, c_float, c_int, c_void_p, pointer

import numpy as np
import pytest

import deepracin_amd as dr
from deepracin_amd import configs
from conftest import GOLDEN, assert_close

pytestmark = pytest.mark.gpu

_CTYPES = {"c_void_p": c_void_p, "c_bool": c_bool, "c_int": c_int, "c_float": c_float, "c_char_p": c_char_p, "None": None}


def small_spec(seed, size=12, classes=7):
    """feed -> 3x3 conv + ReLU -> 2x2/2 max pool -> FC -> softmax, seeded."""
    rng = np.random.default_rng(seed)
    I, O = 3, 8
    w = (rng.standard_normal((I, O, 3, 3)) * np.sqrt(2.0 / (9 * I))).astype(np.float32)
    b = (rng.standard_normal(O) * 0.01).astype(np.float32)
    K = (size // 2) * (size // 2) * O
    fw = (rng.standard_normal((K, classes)) * np.sqrt(2.0 / K)).astype(np.float32)
    fb = (rng.standard_normal(classes) * 0.01).astype(np.float32)
    spec = [{"op": "feed", "shape": (size, size, I)},
            {"op": "conv", "in": 0, "w": w, "b": b, "relu": True},
            {"op": "pool", "in": 1, "kind": 0, "window": (2, 2, 1), "stride": (2, 2, 1)},
            {"op": "fc", "in": 2, "w": fw, "b": fb, "relu": False},
            {"op": "softmax", "in": 3}]
    feeds = {0: rng.random((I, size, size), dtype=np.float32)}
    return spec, feeds


def bind_like_the_reference_wrapper():
    """A fresh handle of libdeepracin.so whose functions carry exactly the argtypes / restype the reference's
    wrapper gives them (tests/golden/ref_wrapper_signatures.txt, written from the wrapper's text)."""
    lib = ctypes.CDLL(dr.LIB_PATH)
    n = 0
    for line in open(os.path.join(GOLDEN, "ref_wrapper_signatures.txt")):
        name, restype, argtypes = [s.strip() for s in line.split("|")]
        f = getattr(lib, name)
        if restype != "-":
            f.restype = _CTYPES[restype]
        if argtypes != "-":
            f.argtypes = [_CTYPES[a.strip()] for a in argtypes.split(",")]
        n += 1
    assert n >= 30
    return lib


def build_with(lib, g, spec):
    """The node constructors called the way the reference's wrapper calls them (python/deepracin/__init__.py.in)."""
    keep, nodes = [], []
    for n in spec:
        if n["op"] == "feed":
            sh = dr.Shape3(*n["shape"])
            keep.append(sh)
            nodes.append(lib.dR_Datafeednode(c_void_p(g), pointer(sh)))
        elif n["op"] == "conv":
            w, b = np.ascontiguousarray(n["w"]), np.ascontiguousarray(n["b"])
            I, O, kh, kw = w.shape
            sh, st = dr.Shape4(kw, kh, I, O), dr.Shape4(1, 1, 1, 1)
            node = lib.dR_Conv2d(c_void_p(g), c_void_p(nodes[n["in"]]), pointer(sh), pointer(st), c_int(1 if n["relu"] else 0), c_bool(True))
            lib.dR_Conv2d_setVariables(c_void_p(node), w.ctypes.data_as(POINTER(c_float)), b.ctypes.data_as(POINTER(c_float)))
            keep += [w, b, sh, st]
            nodes.append(node)
        elif n["op"] == "pool":
            sh, st = dr.Shape4(1, *n["window"]), dr.Shape4(1, *n["stride"])
            keep += [sh, st]
            nodes.append(lib.dR_Pooling(c_void_p(g), c_void_p(nodes[n["in"]]), pointer(sh), pointer(st), c_int(n["kind"])))
        elif n["op"] == "fc":
            w, b = np.ascontiguousarray(n["w"]), np.ascontiguousarray(n["b"])
            sh = dr.Shape2(*w.shape)
            node = lib.dR_FullyConnected(c_void_p(g), c_void_p(nodes[n["in"]]), pointer(sh), c_int(1 if n["relu"] else 0), c_bool(True))
            lib.dR_FullyConnected_setVariables(c_void_p(node), w.ctypes.data_as(POINTER(c_float)), b.ctypes.data_as(POINTER(c_float)))
            keep += [w, b, sh]
            nodes.append(node)
        elif n["op"] == "softmax":
            nodes.append(lib.dR_Softmax(c_void_p(g), c_void_p(nodes[n["in"]])))
        assert nodes[-1], n["op"]
    return nodes, keep


def test_library_bound_with_the_reference_wrappers_own_declarations(oracle, gpu, tmp_path):
    """The sequence of the reference wrapper's prepare() / apply() (python/deepracin/__init__.py.in:405-465) with
    its declared ctypes signatures: dR_config with c_bool switches, dR_initCL read as a c_bool that must be
    true, a second graph of the same environment taking the first one's device through
    dR_getClEnvironmentFrom, dR_prepare, dR_getOutputShape read as three ints, feed, apply, download.
    (The wrapper declares no argtypes for dR_getClEnvironmentFrom and hands it a bare integer, which ctypes
    passes as a 32-bit int; a pointer is passed here.)"""
    lib = bind_like_the_reference_wrapper()
    graphs, keep = [], []
    try:
        for k in range(2):
            spec, feeds = small_spec(seed=10 + k, size=12 + 4 * k)
            g = lib.dR_NewGraph()
            assert g
            nodes, kp = build_with(lib, g, spec)
            keep.append(kp)
            assert lib.dR_setAsOutput(c_void_p(g), c_void_p(nodes[-1]))
            if k == 0:
                plat, mdir = ctypes.create_string_buffer(b""), ctypes.create_string_buffer(str(tmp_path).encode())
                keep += [plat, mdir]
                lib.dR_config(c_void_p(g), plat, c_bool(True), c_bool(False), c_bool(False), c_bool(False), mdir)
                ret = True
                ret &= lib.dR_initCL(c_void_p(g))
                assert ret, "dR_initCL read as c_bool must be true (the reference wrapper raises otherwise)"
            else:
                cfg = ctypes.cast(g, POINTER(dr.GraphStruct)).contents.config.contents
                cfg.silent = 1
                lib.dR_getClEnvironmentFrom(c_void_p(g), c_void_p(graphs[0][0]))
            assert lib.dR_prepare(c_void_p(g))
            graphs.append((g, nodes, spec, feeds))
        # both graphs live on the first one's stream
        cc = [ctypes.cast(g, POINTER(dr.GraphStruct)).contents.clConfig for g, _, _, _ in graphs]
        for g, nodes, spec, feeds in graphs:
            shape = ctypes.cast(lib.dR_getOutputShape(c_void_p(nodes[-1])), POINTER(c_int * 3)).contents
            out_shape = [shape[0], shape[1], shape[2]]
            assert out_shape == [spec[3]["w"].shape[1], 1, 1]
            x = np.ascontiguousarray(feeds[0])
            lib.dR_feedData(c_void_p(g), c_void_p(nodes[0]), x.ctypes.data_as(POINTER(c_float)), 0, x.size)
        for g, nodes, spec, feeds in graphs:            # interleaved: apply both, then download both
            assert lib.dR_apply(c_void_p(g))
        for g, nodes, spec, feeds in graphs:
            memptr = (c_void_p * 1)()
            assert lib.dR_getOutputBuffers(c_void_p(g), memptr) == 1
            n = spec[3]["w"].shape[1]
            data = (c_float * n)()
            lib.dR_downloadArray(c_void_p(g), ctypes.create_string_buffer(b"output0"), memptr[0], 0, n * 4, data)
            got = np.frombuffer(data, dtype=np.float32)
            want = oracle.run_spec(spec, feeds)[4].reshape(-1)
            assert_close(got, want, "softmax through the reference-declared bindings")
            assert int(got.argmax()) == int(want.argmax())
        del cc
    finally:
        for g, _, _, _ in reversed(graphs):             # the first graph owns the stream the second one borrowed
            lib.dR_cleanup(c_void_p(g), c_bool(True))


def _graph(env, spec, outs):
    g = env.create_graph()
    nodes = configs.build_graph(g, spec, outs)
    return g, nodes


def test_caller_owned_feed_buffer(lib, dev, oracle):
    """dR_setDataFeedNodeBuffer (reference include/deepRACIN.h:72): the feed node reads a device buffer the caller
    allocated and filled; dR_feedData is never called and the graph does not free the buffer."""
    spec, feeds = small_spec(seed=3)
    x = feeds[0]
    with dr.Environment() as env:
        g, nodes = _graph(env, spec, [1, 4])
        buf = dev.put(x)                                  # caller's device memory, [C][H][W]
        handle = c_void_p(buf.value)
        lib.dR_setDataFeedNodeBuffer.argtypes = [c_void_p, c_void_p, POINTER(c_void_p)]
        lib.dR_setDataFeedNodeBuffer.restype = c_int
        assert lib.dR_setDataFeedNodeBuffer(g.ptr, nodes[0].ptr, ctypes.byref(handle)) == 1
        assert lib.dR_setDataFeedNodeBuffer(g.ptr, nodes[1].ptr, ctypes.byref(handle)) == 0      # not a feed node
        dr.prepare(g)
        assert dr.node_struct(nodes[0]).outputBuf.contents.buf == buf.value
        for _ in range(2):                                # plain pass, then the replayed launch graph
            assert lib.dR_apply(g.ptr)
            conv, soft = configs.fetch_chw(g)
            want = oracle.run_spec(spec, feeds)
            assert_close(conv, want[1], "conv on a caller-owned feed buffer")
            assert_close(soft.reshape(-1), want[4].reshape(-1), "softmax on a caller-owned feed buffer")
        # new contents of the caller's buffer are seen by the next pass
        x2 = np.ascontiguousarray(x[:, ::-1, :])
        assert lib.drhip_upload(buf, 0, x2.ctypes.data_as(c_void_p), x2.nbytes, None) == 0
        assert lib.dR_apply(g.ptr)
        conv2, _ = configs.fetch_chw(g)
        assert_close(conv2, oracle.run_spec(spec, {0: x2})[1], "conv after the caller rewrote its buffer")
    # the graph is gone; the caller's buffer is still the caller's to read and free
    assert np.array_equal(dev.get(buf, x.shape), x2)


def test_preexisting_output_buffer(lib, dev, oracle):
    """dR_setPreexistingOutputBuffer (reference include/deepRACIN.h:126, src/deepRACIN.c:122-129): a node writes into
    device memory the caller owns and becomes an output of the graph.  On an inner node whose tensor a fusion would otherwise do away with (the convolution in front of a
    2x2/2 max pool), and on the last node.  The planner neither recycles nor frees such a buffer."""
    spec, feeds = small_spec(seed=4, size=16)
    want = oracle.run_spec(spec, feeds)
    lib.dR_setPreexistingOutputBuffer.argtypes = [c_void_p, c_void_p, POINTER(c_void_p)]
    lib.dR_setPreexistingOutputBuffer.restype = c_int
    with dr.Environment() as env:
        g, nodes = _graph(env, spec, [])
        conv_buf = dev.put(np.full(want[1].shape, 7.0, np.float32))
        soft_buf = dev.put(np.full(want[4].size, 7.0, np.float32))
        h1, h2 = c_void_p(conv_buf.value), c_void_p(soft_buf.value)
        assert lib.dR_setPreexistingOutputBuffer(g.ptr, nodes[1].ptr, ctypes.byref(h1)) == 1
        assert lib.dR_setPreexistingOutputBuffer(g.ptr, nodes[4].ptr, ctypes.byref(h2)) == 1
        g.outnodes, g.num_outputs = [nodes[1], nodes[4]], 2      # the call makes the node an output of the graph, like the reference's
        dr.prepare(g)
        x = feeds[0]
        configs.feed_chw(nodes[0], x)
        for _ in range(2):
            assert lib.dR_apply(g.ptr)
            conv, soft = configs.fetch_chw(g)
            assert_close(conv, want[1], "convolution (graph's own download)")
            assert_close(soft.reshape(-1), want[4].reshape(-1), "softmax (graph's own download)")
            assert_close(dev.get(conv_buf, want[1].shape), want[1], "unpooled convolution in the caller's buffer")
            assert_close(dev.get(soft_buf, (want[4].size,)), want[4].reshape(-1), "softmax in the caller's buffer")
    assert_close(dev.get(conv_buf, want[1].shape), want[1], "caller's buffer after dR_cleanup")


def test_caller_stream_through_set_cl_environment(lib, dev, oracle):
    """dR_setClEnvironment (reference include/deepRACIN.h:242): the graph runs on the command queue -- here the HIP
    stream -- the caller hands over, and leaves it alive at dR_cleanup."""
    spec, feeds = small_spec(seed=5)
    want = oracle.run_spec(spec, feeds)
    stream = c_void_p()
    assert lib.drhip_stream_create(ctypes.byref(stream)) == 0
    lib.dR_setClEnvironment.argtypes = [c_void_p] * 5
    lib.dR_setClEnvironment.restype = None
    try:
        with dr.Environment() as env:
            g, nodes = _graph(env, spec, [4])
            lib.dR_setClEnvironment(g.ptr, None, None, stream, None)
            dr.prepare(g)
            cc = ctypes.cast(dr.graph_struct(g).clConfig, POINTER(c_void_p * 3)).contents      # clContext, clPlatformId, clCommandQueue
            assert cc[2] == stream.value
            configs.feed_chw(nodes[0], feeds[0])
            assert lib.dR_apply(g.ptr)
            assert lib.drhip_stream_sync(stream) == 0   # the caller's own handle orders behind the pass
            (soft,) = configs.fetch_chw(g)
            assert_close(soft.reshape(-1), want[4].reshape(-1), "softmax on the caller's stream")
        # still usable after the graph is gone
        buf = dev.put(np.arange(8, dtype=np.float32))
        assert lib.drhip_fill_f32(buf, 2.5, 8, stream) == 0 and lib.drhip_stream_sync(stream) == 0
        assert np.all(dev.get(buf, (8,)) == 2.5)
    finally:
        assert lib.drhip_stream_destroy(stream) == 0


def test_debug_layer_download_and_profiling_switches(lib, dev, oracle, capfd):
    """debugLayer: dR_apply copies the first channel plane (width x height floats, as the reference does,
    src/deepRACIN.c:235-238) of the chosen layer into hostDebugBuffer, the host array the graph allocates for this at
    dR_prepare and frees at dR_cleanup (src/dR_core.c:322,493).  Set before dR_prepare, the layer keeps a tensor of
    its own although a fusion would do away with it (the convolution in front of a 2x2/2 max pool); set afterwards on
    such a layer, the pass says so and leaves the array alone.
    profilingCPU: the pass is timed on the host and waited for; profilingGPU: per-node kernel times."""
    spec, feeds = small_spec(seed=6)
    want = oracle.run_spec(spec, feeds)
    for early in (True, False):
        with dr.Environment() as env:
            g, nodes = _graph(env, spec, [4])
            gs = dr.graph_struct(g)
            conv = dr.node_struct(nodes[1])
            if early:
                gs.debugLayer = conv.layerID
            dr.prepare(g)
            assert gs.hostDebugBuffer                       # the graph's own array, large enough for its largest tensor
            n = conv.oshape.s0 * conv.oshape.s1
            plane = np.ctypeslib.as_array(ctypes.cast(gs.hostDebugBuffer, POINTER(c_float)), shape=(n,))
            plane[:] = -1.0
            configs.feed_chw(nodes[0], feeds[0])
            gs.debugLayer = conv.layerID
            capfd.readouterr()
            assert lib.dR_apply(g.ptr)
            (soft,) = configs.fetch_chw(g)
            assert_close(soft.reshape(-1), want[4].reshape(-1), "softmax of a pass with a debug download")
            if early:
                assert_close(plane.reshape(conv.oshape.s1, conv.oshape.s0).copy(), want[1][0], "debug download of the convolution's first plane")
                continue
            assert np.all(plane == -1.0)
            assert "its tensor is never stored" in capfd.readouterr().out
            gs.debugLayer = -1
            cfg = dr.graph_config(g)
            cfg.profilingCPU = 1
            capfd.readouterr()
            assert lib.dR_apply(g.ptr)
            assert gs.drLastApplyMs > 0.0
            assert "CPU Profiling: Whole graph took" in capfd.readouterr().out
            cfg.profilingCPU = 0
            cfg.profilingGPU = 1
            assert lib.dR_apply(g.ptr)
            assert "GPU Profiling: Sum of all kernel run times" in capfd.readouterr().out
            assert dr.node_struct(nodes[1]).drLastKernelMs > 0.0
            cfg.profilingGPU = 0
            assert lib.dR_apply(g.ptr)
            (soft,) = configs.fetch_chw(g)
            assert_close(soft.reshape(-1), want[4].reshape(-1), "softmax after the switches were turned off again")
            del plane


def test_compiled_c_host_program_classifies_the_reference_images(gpu, tmp_path):
    """tests/c_caller.c, compiled with gcc against the public headers (by build(); compiled here if it is missing),
    run as a child process: the reference example's sequence -- switches poked into net->config / net->clConfig,
    dR_loadGraph of the stored SqueezeNet v1.1, feed / apply / download per image -- must name the classes the
    reference documents for its two images (examples/squeezenet-v1.1/squeezenet_deployed.c:199-207)."""
    import subprocess
    from deepracin_amd import build
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = os.path.join(root, "tests", "bin", "c_caller")
    if not os.path.exists(exe):
        exe = build.build_c_caller(verbose=False)
    files = []
    for name in ("tiger", "puzzle"):
        img = np.load(os.path.join(GOLDEN, "%s_224_rgb_u8.npy" % name))
        f = tmp_path / (name + ".f32")
        np.ascontiguousarray(img.transpose(2, 0, 1).astype(np.float32)).tofile(str(f))
        files.append(str(f))
    r = subprocess.run([exe, os.path.join(GOLDEN, "squeezenet_whole") + "/", files[0], files[1], files[0]],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    classes = [int(l.split()[1]) for l in r.stdout.splitlines() if l.startswith("class ")]
    assert classes == [292, 611, 292], r.stdout
    assert "GPU Profiling: Sum of all kernel run times" in r.stdout and "CPU Profiling: Whole graph took" in r.stdout
