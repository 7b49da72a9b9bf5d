"""deepracin_amd -- Python front-end over libdeepracin.so (the MI355X / gfx950 build of deepRacin).

Mirrors the reference's ctypes wrapper for the CNN layer path (python/deepracin/__init__.py.in):
same function names, same argument meaning, same layout conversions
  * feed_data:   HWC numpy -> [C][H][W] buffer           (reference :475-497)
  * apply:       [C][H][W] buffer -> HWC numpy, squeezed (reference :444-465)
  * Conv2d:      HWIO weights -> [I][O][kh][kw]          (reference :559-562)
so a script written against `import deepracin as dr` runs with `import deepracin_amd as dr`.

All compute happens in hand-written HIP kernels inside the shared library; this module only
marshals arguments.  Importing it never builds anything: run `python -m deepracin_amd.build` (or
__graft_entry__.build()) first.  A missing library is an ImportError-style failure, not a fallback.
"""
import ctypes
import os
from ctypes import POINTER, Structure, byref, c_char_p, c_float, c_int, c_size_t, c_void_p, pointer

import numpy as np

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "lib", "libdeepracin.so")


class Shape2(Structure):
    _fields_ = [("s0", c_int), ("s1", c_int)]


class Shape3(Structure):
    _fields_ = [("s0", c_int), ("s1", c_int), ("s2", c_int)]


class Shape4(Structure):
    _fields_ = [("s0", c_int), ("s1", c_int), ("s2", c_int), ("s3", c_int)]


class DeviceInfo(Structure):
    _fields_ = [("name", ctypes.c_char * 256), ("arch", ctypes.c_char * 64), ("device", c_int), ("num_cu", c_int),
                ("wavefront", c_int), ("lds_bytes", c_int), ("clock_khz", c_int), ("hbm_bytes", c_size_t),
                ("l2_bytes", c_int)]


_FN = c_void_p      # function-pointer slots of the node vtable


class MemoryHandlerStruct(Structure):
    """Head of dR_MemoryHandler (include/dR_types.h)."""
    _fields_ = [("outputFor", c_void_p), ("size", c_int), ("numberOfDependencies", c_int),
                ("bufptr", POINTER(c_void_p)), ("buf", c_void_p)]


class NodeStruct(Structure):
    """dR_Node (include/dR_types.h): lets Python read shapes, buffers and per-node profile times."""
    _fields_ = [("oshape", Shape3), ("layerID", ctypes.c_int32), ("previous_layers", c_void_p), ("next_layers", c_void_p),
                ("clKernel", c_void_p), ("outputBuf", POINTER(MemoryHandlerStruct)), ("layer", c_void_p), ("type", c_int),
                ("propagated", c_int), ("output", c_int), ("queued", c_int)] + \
               [(n, _FN) for n in ("compute", "schedule", "propagateShape", "getRequiredOutputBufferSize", "createKernel",
                                   "allocateBuffers", "fillBuffers", "cleanupBuffers", "cleanupLayer", "printLayer",
                                   "serializeNode", "parseAppendNode", "generateKernel", "createKernelName", "setVariables")] + \
               [("drSchedulePos", c_int), ("drLastKernelMs", c_float)]


class ConfigStruct(Structure):
    """dR_Config (include/dR_types.h)."""
    _fields_ = [("silent", c_int), ("profilingGPU", c_int), ("profilingCPU", c_int), ("debugInfo", c_int),
                ("totalNodeCPUTime", ctypes.c_double), ("convLocalWorkSizeWindow", c_int), ("modelPath", c_char_p)]


class GraphStruct(Structure):
    """dR_Graph (include/dR_types.h): the reference's fields, then the ones this library appends."""
    _fields_ = [("prepared", c_int), ("swapBuffer1", c_void_p), ("swapBuffer2", c_void_p),
                ("config", POINTER(ConfigStruct)), ("clConfig", c_void_p), ("feed_layers", c_void_p),
                ("output_layers", c_void_p), ("streamBufferHandlers", c_void_p),
                ("number_of_layers", ctypes.c_int32), ("maxBufferSize", ctypes.c_int32), ("hostDebugBuffer", c_void_p),
                ("scheduledLayers", c_void_p), ("allNodes", c_void_p), ("debugLayer", c_int),
                ("drViewHandlers", c_void_p), ("drLastApplyMs", ctypes.c_double), ("drGraphExec", c_void_p),
                ("drGraphOff", c_int), ("drSideStreams", c_void_p * 3), ("drBranchEvents", c_void_p * 4),
                ("drBranchGroups", c_int), ("drStaging", c_void_p)]


def graph_struct(graph):
    return ctypes.cast(graph.ptr, POINTER(GraphStruct)).contents


def node_struct(node):
    return ctypes.cast(node.ptr, POINTER(NodeStruct)).contents


def graph_config(graph):
    return ctypes.cast(graph.ptr, POINTER(GraphStruct)).contents.config.contents


_lib = None


def load_library(path=None):
    """ctypes handle of libdeepracin.so with argument types declared.  Raises if it is not built."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = path or LIB_PATH
    if not os.path.exists(p):
        raise OSError("libdeepracin.so not found at %s -- build it with `python -m deepracin_amd.build`" % p)
    lib = ctypes.CDLL(p)
    vp, fp, ip = c_void_p, POINTER(c_float), POINTER(c_int)
    sig = {
        # graph API
        "dR_NewGraph": (vp, []),
        "dR_config": (None, [vp, c_char_p, c_int, c_int, c_int, c_int, c_char_p]),
        "dR_initCL": (c_int, [vp]),
        "dR_getClEnvironmentFrom": (None, [vp, vp]),
        "dR_setAsOutput": (c_int, [vp, vp]),
        "dR_prepare": (c_int, [vp]),
        "dR_getOutputBuffers": (c_int, [vp, POINTER(vp)]),
        "dR_feedData": (None, [vp, vp, fp, c_int, c_int]),
        "dR_apply": (c_int, [vp]),
        "dR_cleanup": (None, [vp, c_int]),
        "dR_saveGraph": (c_int, [vp, c_char_p]),
        "dR_loadGraph": (vp, [vp, c_char_p, POINTER(POINTER(vp)), ip, POINTER(POINTER(vp)), ip]),
        "dR_printNetObject": (None, [vp, c_char_p]),
        "dR_getOutputShape": (POINTER(Shape3), [vp]),
        "dR_getFeedNodeInputShape": (POINTER(Shape3), [vp]),
        "dR_downloadArray": (None, [vp, c_char_p, vp, c_size_t, c_size_t, vp]),
        "dR_uploadArray": (c_int, [vp, c_char_p, vp, c_size_t, c_size_t, vp]),
        "dR_createFloatBuffer": (c_int, [vp, POINTER(vp), c_int, c_int]),
        "dR_propagateShapesAndSchedule": (c_int, [vp]),
        "dR_planBuffers": (c_int, [vp]),
        # nodes
        "dR_Datafeednode": (vp, [vp, POINTER(Shape3)]),
        "dR_Conv2d": (vp, [vp, vp, POINTER(Shape4), POINTER(Shape4), c_int, c_int]),
        "dR_Conv2d_setVariables": (None, [vp, fp, fp]),
        "dR_Pooling": (vp, [vp, vp, POINTER(Shape4), POINTER(Shape4), c_int]),
        "dR_FullyConnected": (vp, [vp, vp, POINTER(Shape2), c_int, c_int]),
        "dR_FullyConnected_setVariables": (None, [vp, fp, fp]),
        "dR_Softmax": (vp, [vp, vp]),
        "dR_Concat": (vp, [vp, POINTER(vp), c_int, c_int]),
        "dR_Slice": (vp, [vp, vp, POINTER(Shape4), POINTER(Shape4)]),
        "dR_ElemWise1Operation": (vp, [vp, vp, c_int, c_float]),
        "dR_Normalization": (vp, [vp, vp, c_int, c_float, c_float]),
        # device layer
        "drhip_init": (c_int, [c_int, POINTER(DeviceInfo)]),
        "drhip_last_error": (c_char_p, []),
        "drhip_device_count": (c_int, []),
        "drhip_stream_sync": (c_int, [vp]),
        "drhip_graph_capture_begin": (c_int, [vp]),
        "drhip_graph_capture_end": (c_int, [vp, POINTER(vp)]),
        "drhip_graph_launch": (c_int, [vp, vp]),
        "drhip_graph_destroy": (c_int, [vp]),
        "drhip_malloc": (c_int, [POINTER(vp), c_size_t]),
        "drhip_free": (c_int, [vp]),
        "drhip_upload": (c_int, [vp, c_size_t, vp, c_size_t, vp]),
        "drhip_download": (c_int, [vp, vp, c_size_t, c_size_t, vp]),
        "drhip_fill_f32": (c_int, [vp, c_float, c_size_t, vp]),
        "drhip_event_create": (c_int, [POINTER(vp)]),
        "drhip_event_destroy": (c_int, [vp]),
        "drhip_event_record": (c_int, [vp, vp]),
        "drhip_event_elapsed_ms": (c_int, [vp, vp, POINTER(c_float)]),
        "drhip_stream_wait_event": (c_int, [vp, vp]),
        "drhip_fc_slices": (c_int, [c_int, c_int]),
        "drhip_fc_ex_f32": (c_int, [vp, vp, vp, vp, vp, vp, c_int, c_int, c_int, c_int, vp]),
        "drhip_softmax_ex_f32": (c_int, [vp, vp, vp, c_int, vp]),
        "drhip_normalize_scratch_floats": (c_size_t, [c_size_t]),
        "drhip_normalize_f32": (c_int, [vp, vp, c_size_t, c_int, c_float, c_float, vp, vp]),
        "drhip_timing_begin": (c_int, []),
        "drhip_timing_count": (c_int, []),
        "drhip_timing_end": (c_int, [POINTER(c_float), c_int, POINTER(c_int)]),
        "drhip_conv2d_direct_f32": (c_int, [vp, vp, vp, vp] + [c_int] * 9 + [vp]),
        "drhip_conv3x3_pool3s2_f32": (c_int, [vp, vp, vp, vp] + [c_int] * 7 + [vp]),
        "drhip_conv1x1_poolsum_f32": (c_int, [vp, vp, vp, vp, c_int, c_int, c_int, c_int, vp]),
        "drhip_conv1x1_poolsum_slices": (c_int, [c_int]),
        "drhip_winograd_filter_transform_f32": (c_int, [vp, vp, c_int, c_int, vp]),
        "drhip_conv3x3_winograd_f32": (c_int, [vp, vp, vp, vp] + [c_int] * 6 + [vp, vp]),
        "drhip_conv3x3_winograd_filter_floats": (c_size_t, [c_int, c_int]),
        "drhip_conv3x3_winograd_workspace_floats": (c_size_t, [c_int] * 5),
        "drhip_conv3x3_winograd_pick_variant": (c_int, [c_int] * 4),
        "drhip_conv3x3_winograd_workspace_prepare_f32": (c_int, [vp, c_size_t, vp]),
        "drhip_conv3x3_winograd_join_timeouts": (c_int, [POINTER(ctypes.c_uint)]),
        "drhip_conv1x1_f32": (c_int, [vp, vp, vp, vp] + [c_int] * 5 + [vp]),
        "drhip_conv1x1_pick_variant": (c_int, [c_int] * 3),
        "drhip_conv3x3_direct_filter_floats": (c_size_t, [c_int, c_int]),
        "drhip_conv3x3_direct_filter_layout_f32": (c_int, [vp, vp, c_int, c_int, vp]),
        "drhip_conv3x3_direct_pick_variant": (c_int, [c_int] * 4),
        "drhip_conv3x3_direct_mfma_f32": (c_int, [vp, vp, vp, vp] + [c_int] * 7 + [vp]),
        "drhip_conv1x1_pooled3s2_f32": (c_int, [vp, vp, vp, vp] + [c_int] * 5 + [vp]),
        "drhip_pool_f32": (c_int, [vp, vp, vp] + [c_int] * 10 + [vp]),
        "drhip_fc_scratch_floats": (c_size_t, [c_int, c_int]),
        "drhip_fc_f32": (c_int, [vp] * 5 + [c_int] * 3 + [vp]),
        "drhip_fc_noalloc_f32": (c_int, [vp] * 4 + [c_int] * 3 + [vp]),
        "drhip_fc_noalloc_max_scratch_floats": (c_size_t, []),
        "drhip_staging_create": (c_int, [POINTER(vp), c_size_t]),
        "drhip_staging_destroy": (c_int, [vp]),
        "drhip_staging_upload_capacity": (c_size_t, [vp]),
        "drhip_staging_download_capacity": (c_size_t, [vp]),
        "drhip_upload_staged": (c_int, [vp, vp, c_size_t, vp, c_size_t, vp]),
        "drhip_download_staged": (c_int, [vp, vp, vp, c_size_t, c_size_t, vp]),
        "drhip_fc_permute_rows_f32": (c_int, [vp, vp] + [c_int] * 4 + [vp]),
        "drhip_softmax_f32": (c_int, [vp, vp, c_int, vp]),
        "drhip_copy3d_f32": (c_int, [vp] + [c_int] * 5 + [vp] + [c_int] * 8 + [vp]),
        "drhip_scalar_op_f32": (c_int, [vp, vp, c_size_t, c_int, c_float, vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    if path is None:
        _lib = lib
    return lib


def device_available():
    """True when a HIP device is visible (does not initialise a context)."""
    try:
        return load_library().drhip_device_count() > 0
    except OSError:
        return False


act_dict = {"linear": 0, "relu": 1}
pool_dict = {"max": 0, "average": 1}


def _fptr(a):
    return a.ctypes.data_as(POINTER(c_float)) if a is not None else None


class Node:
    """Handle of a graph node (the reference's Node, python/deepracin/__init__.py.in:253)."""

    def __init__(self, ptr, graph, desc, params, variables=None):
        if not ptr:
            raise RuntimeError("DR Error: creating a %s node failed" % desc)
        self.ptr = ptr
        self.graph = graph
        self.desc = desc
        self.params = params
        self.variables = variables
        self.out_shape = None
        self.shape = None


class Graph:
    def __init__(self, gid, layout, env):
        self.lib = load_library()
        self.ptr = self.lib.dR_NewGraph()
        self.id = gid
        self.layout = layout
        self.env = env
        self.feed_nodes = []
        self.outnodes = []
        self.num_outputs = 0
        self.model_path = None
        self.prepared = False
        self._keep = []         # keeps byte strings handed to the C side alive


class Environment:
    """Context manager owning the graphs, like the reference's Environment (:339-381)."""

    def __init__(self, preferred_platform=""):
        self.preferred_platform_name = preferred_platform
        self.graphs = []
        self.graph_with_cl_context = -1
        self.id_counter = 0
        self.silent = True
        self.debuginfo = False
        self.profileGPU = False
        self.profileCPU = False
        self.model_path = os.environ.get("DR_MODEL_PATH", "/tmp/deepracin_amd")

    def __enter__(self):
        return self

    def __exit__(self, exc_type, exc, tb):
        self.close()
        return False

    def close(self):
        for g in reversed(self.graphs):         # (the first prepared graph owns the stream the later ones borrowed)
            if g.ptr:
                g.lib.dR_cleanup(g.ptr, 1)
                g.ptr = None
        self.graphs = []
        self.graph_with_cl_context = -1

    def create_graph(self, interface_layout="HWC"):
        g = Graph(self.id_counter, interface_layout, self)
        self.id_counter += 1
        self.graphs.append(g)
        return g


def _dr_shape3(layout, shape):
    if layout == "WHC":
        return [shape[0], shape[1], shape[2]]
    if layout == "CHW":
        return [shape[2], shape[1], shape[0]]
    if layout == "HWC":
        return [shape[1], shape[0], shape[2]]
    raise NotImplementedError("DR Error: Graphs's layout " + layout + " not supported!")


def feed_node(graph, shape):
    if len(shape) != 3 or not all(isinstance(s, (int, np.integer)) for s in shape):
        raise TypeError("DR Error: feed_node()'s shape parameter needs to be a list with 3 ints!")
    d = _dr_shape3(graph.layout, [int(s) for s in shape])
    sh = Shape3(*d)
    node = Node(graph.lib.dR_Datafeednode(graph.ptr, pointer(sh)), graph, "DataFeedNode", d)
    node.shape = d
    graph.feed_nodes.append(node)
    return node


def prepare(graph):
    env = graph.env
    model_path = graph.model_path or env.model_path
    os.makedirs(model_path, exist_ok=True)
    plat, mdir = env.preferred_platform_name.encode(), model_path.encode()
    graph._keep += [plat, mdir]
    graph.lib.dR_config(graph.ptr, plat, int(env.silent), int(env.debuginfo), int(env.profileGPU), int(env.profileCPU), mdir)
    # the first graph of an environment brings the device up, the others take its device and stream (reference :408-428)
    first = next((g for g in env.graphs if g.id == env.graph_with_cl_context and g.ptr), None)
    if first is None:
        if not graph.lib.dR_initCL(graph.ptr):
            raise RuntimeError("DR Error: deepRACIN initCL failed!")
        env.graph_with_cl_context = graph.id
    elif first is not graph:
        graph.lib.dR_getClEnvironmentFrom(graph.ptr, first.ptr)
    if not graph.lib.dR_prepare(graph.ptr):
        raise RuntimeError("DR Error: deepRACIN prepare failed!")
    for node in graph.outnodes:
        s = graph.lib.dR_getOutputShape(node.ptr).contents
        node.out_shape = [s.s0, s.s1, s.s2]
    for node in graph.feed_nodes:
        s = graph.lib.dR_getOutputShape(node.ptr).contents
        node.shape = [s.s0, s.s1, s.s2]
    graph.prepared = True


def _from_chw(graph, flat, shape):
    arr = flat.reshape([shape[2], shape[1], shape[0]])
    if graph.layout == "WHC":
        arr = arr.transpose([2, 1, 0])
    elif graph.layout == "HWC":
        arr = arr.transpose([1, 2, 0])
    return arr


def download_outputs(graph, squeeze=True):
    """Fetch every output buffer (blocking) in the graph's interface layout."""
    lib = graph.lib
    mem = (c_void_p * max(graph.num_outputs, 1))()
    n = lib.dR_getOutputBuffers(graph.ptr, mem)
    outs = []
    for i in range(n):
        s = graph.outnodes[i].out_shape
        flat = np.empty(s[0] * s[1] * s[2], np.float32)
        lib.dR_downloadArray(graph.ptr, b"output", mem[i], 0, flat.nbytes, flat.ctypes.data_as(c_void_p))
        arr = _from_chw(graph, flat, s)
        outs.append(np.squeeze(arr) if squeeze else arr)
    return outs


def apply(graph):
    """Run the graph once and return the outputs (reference :444-465)."""
    if not graph.lib.dR_apply(graph.ptr):
        raise RuntimeError("DR Error: deepRACIN apply failed!")
    return download_outputs(graph)


def mark_as_output(node):
    node.graph.lib.dR_setAsOutput(node.graph.ptr, node.ptr)
    node.graph.num_outputs += 1
    node.graph.outnodes.append(node)


def feed_data(node, data):
    if data.ndim != 3:
        raise TypeError("DR Error: data fed to a feed_node needs to be an array with 3 dimensions!")
    if data.dtype != np.float32:
        raise TypeError("DR Error: data fed to a feed_node is " + str(data.dtype) + " but needs to be an array of type float32!")
    layout = node.graph.layout
    d = _dr_shape3(layout, list(data.shape))
    if layout == "WHC":
        data = data.transpose([2, 1, 0])
    elif layout == "HWC":
        data = data.transpose([2, 0, 1])
    data = np.ascontiguousarray(data)
    if d != list(node.shape):
        raise ValueError("DR Error: data array's dimensions %s do not match node's dimensions %s!" % (d, node.shape))
    node.graph.lib.dR_feedData(node.graph.ptr, node.ptr, _fptr(data), 0, d[0] * d[1] * d[2])


def load_graph(graph, path):
    """Fill an empty graph from <path>/graph.dr; returns (nodes, feed nodes)."""
    if not isinstance(path, str):
        raise TypeError("DR Error: path needs to be a string!")
    lib = graph.lib
    nodes, feeds = POINTER(c_void_p)(), POINTER(c_void_p)()
    nn, nf = c_int(0), c_int(0)
    bpath = path.encode()
    graph._keep.append(bpath)
    last = lib.dR_loadGraph(graph.ptr, bpath, byref(nodes), byref(nn), byref(feeds), byref(nf))
    if not last:
        raise RuntimeError("DR Error: loading graph from %s failed!" % path)
    out = [Node(nodes[i], graph, "loaded", []) for i in range(nn.value)]
    feed = []
    for i in range(nf.value):
        n = next(x for x in out if x.ptr == feeds[i])
        s = lib.dR_getFeedNodeInputShape(n.ptr).contents
        n.shape = [s.s0, s.s1, s.s2]
        feed.append(n)
        graph.feed_nodes.append(n)
    graph.model_path = path
    return out, feed


def save_graph(graph, path):
    os.makedirs(path, exist_ok=True)
    if not graph.lib.dR_saveGraph(graph.ptr, path.encode()):
        raise RuntimeError("DR Error: saving graph to %s failed!" % path)


def print_graph(graph):
    graph.lib.dR_printNetObject(graph.ptr, None)


def Conv2d(input_node, shape, stride, activation, weights, biases=None):
    """shape (kh?, kw, I, O) as in the reference: quadratic odd filters; weights HWIO."""
    if not (shape[0] == shape[1] and shape[0] % 2 == 1):
        raise TypeError("DR Error: Conv2d' currently only supports quadratic filter sizes with odd side length!")
    if not (stride[0] == stride[3] == 1 and stride[1] == stride[2]):
        raise TypeError("DR Error: Conv2d' currently only strides of from (1,x,x,1)!")
    use_bias = biases is not None
    if weights is not None:
        weights = np.ascontiguousarray(np.asarray(weights, np.float32).transpose([2, 3, 0, 1]))
    sh, st = Shape4(*shape), Shape4(*stride)
    g = input_node.graph
    params = [act_dict[activation], int(use_bias)] + list(shape) + list(stride)
    node = Node(g.lib.dR_Conv2d(g.ptr, input_node.ptr, pointer(sh), pointer(st), act_dict[activation], int(use_bias)),
                g, "Conv2D", params, [weights, biases])
    if weights is not None:
        b = np.ascontiguousarray(biases, np.float32) if use_bias else None
        g.lib.dR_Conv2d_setVariables(node.ptr, _fptr(weights), _fptr(b))
    return node


def Conv2d_raw(input_node, weights_iohw, biases, stride, activation):
    """Conv2d from weights already in the C API's [I][O][kh][kw] layout (no transpose)."""
    w = np.ascontiguousarray(weights_iohw, np.float32)
    I, O, kh, kw = w.shape
    sh, st = Shape4(kw, kh, I, O), Shape4(1, stride[0], stride[1], 1)
    use_bias = biases is not None
    g = input_node.graph
    node = Node(g.lib.dR_Conv2d(g.ptr, input_node.ptr, pointer(sh), pointer(st), act_dict[activation], int(use_bias)),
                g, "Conv2D", [])
    b = np.ascontiguousarray(biases, np.float32) if use_bias else None
    g.lib.dR_Conv2d_setVariables(node.ptr, _fptr(w), _fptr(b))
    return node


def Fully_Connected(input_node, shape, activation, weights, biases=None):
    use_bias = biases is not None
    g = input_node.graph
    sh = Shape2(*shape)
    node = Node(g.lib.dR_FullyConnected(g.ptr, input_node.ptr, pointer(sh), act_dict[activation], int(use_bias)),
                g, "FullyConnected", [act_dict[activation], int(use_bias), shape[0], shape[1]])
    if weights is not None:
        w = np.ascontiguousarray(weights, np.float32)
        b = np.ascontiguousarray(biases, np.float32) if use_bias else None
        g.lib.dR_FullyConnected_setVariables(node.ptr, _fptr(w), _fptr(b))
    return node


def Pooling(input_node, pooling_type, shape, stride):
    g = input_node.graph
    sh, st = Shape4(*shape), Shape4(*stride)
    return Node(g.lib.dR_Pooling(g.ptr, input_node.ptr, pointer(sh), pointer(st), pool_dict[pooling_type]),
                g, "Pooling", [pool_dict[pooling_type]] + list(shape) + list(stride))


def Softmax(input_node):
    g = input_node.graph
    return Node(g.lib.dR_Softmax(g.ptr, input_node.ptr), g, "Softmax", [])


norm_dict = {"target_mean": 0, "target_dev": 1, "target_mean_dev": 2}


def Normalization(input_node, normalization_type, target_mean=0.0, target_dev=1.0):
    """Reference wrapper :889-898; normalization_type is a key of norm_dict (or its number)."""
    g = input_node.graph
    kind = norm_dict.get(normalization_type, normalization_type)
    return Node(g.lib.dR_Normalization(g.ptr, input_node.ptr, int(kind), c_float(target_mean), c_float(target_dev)), g,
                "Normalization", [kind, target_mean, target_dev])


def Slice(input_node, origin, shape):
    g = input_node.graph
    o = _dr_shape3(g.layout, list(origin)) + [0]
    s = _dr_shape3(g.layout, list(shape)) + [0]
    return Node(g.lib.dR_Slice(g.ptr, input_node.ptr, pointer(Shape4(*o)), pointer(Shape4(*s))), g, "Slice", o + s)


def Concat(input_nodes, concat_dim):
    n = len(input_nodes)
    if n <= 1:
        raise ValueError("DR Error: Concat with one or less nodes not allowed!")
    g = input_nodes[0].graph
    dr_dim = {"WHC": [0, 1, 2], "CHW": [2, 1, 0], "HWC": [1, 0, 2]}[g.layout][concat_dim]
    ptrs = (c_void_p * n)(*[x.ptr for x in input_nodes])
    return Node(g.lib.dR_Concat(g.ptr, ptrs, n, dr_dim), g, "Concat", [n, dr_dim])


def _scalar(input_node, op, scalar):
    g = input_node.graph
    return Node(g.lib.dR_ElemWise1Operation(g.ptr, input_node.ptr, op, c_float(scalar)), g, "ElemWise1Op", [op, scalar])


def Add_Scalar(input_node, scalar):
    return _scalar(input_node, 0, scalar)


def Sub_Scalar(input_node, scalar):
    return _scalar(input_node, 1, scalar)


def Mul_Scalar(input_node, scalar):
    return _scalar(input_node, 2, scalar)


def Div_Scalar(input_node, scalar):
    return _scalar(input_node, 3, scalar)
