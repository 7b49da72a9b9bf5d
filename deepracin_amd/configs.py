"""Seeded synthetic workloads of the CNN layer path (the five benchmark configurations).

A workload is a *spec*: a list of node dicts in creation order, each referring to earlier nodes by
index.  The same spec is (a) turned into a deepRacin graph through the C API by `build_graph`, and
(b) evaluated by the CPU oracle in the tests -- so both sides see bit-identical weights and inputs.

    {"op": "feed", "shape": (W, H, C)}
    {"op": "conv", "in": i, "w": [I,O,kh,kw] f32, "b": [O] f32 | None, "stride": (sx, sy), "relu": bool}
    {"op": "pool", "in": i, "window": (sx, sy, sz), "stride": (stx, sty, stz), "kind": 0 max | 1 average}
    {"op": "fc", "in": i, "w": [K,N] f32 (k counts the input in [H][W][C] order), "b": [N] | None, "relu": bool}
    {"op": "softmax", "in": i}
    {"op": "concat", "ins": [i, j, ...], "dim": 2}
    {"op": "norm", "in": i, "kind": 0 mean | 1 deviation | 2 both, "mean": target, "dev": target}

Random numbers: numpy PCG64 from one seed, one sub-stream per tensor.  Tensors are drawn in the
logical interface layout (HWC images, HWIO filters) and converted to the C API layouts exactly as
the reference's Python wrapper does (HWC -> CHW, HWIO -> [I][O][kh][kw]).
"""
import numpy as np

import deepracin_amd as dr


class _Streams:
    """One independent PCG64 sub-stream per tensor, in creation order."""

    def __init__(self, seed):
        self._seq = np.random.SeedSequence(seed)

    def next(self):
        return np.random.Generator(np.random.PCG64(self._seq.spawn(1)[0]))


def _normal_f32(rng, shape, std, chunk=1 << 24):
    n = int(np.prod(shape))
    out = np.empty(n, np.float32)
    for s in range(0, n, chunk):                  # chunked: FC6 of VGG16 is 103 M weights
        e = min(n, s + chunk)
        out[s:e] = rng.standard_normal(e - s, dtype=np.float32) * np.float32(std)
    return out.reshape(shape)


def _conv(st, src, k, cin, cout, stride=1, relu=True, bias=True):
    w_hwio = _normal_f32(st.next(), (k, k, cin, cout), np.sqrt(2.0 / (k * k * cin)))     # He-normal
    w = np.ascontiguousarray(w_hwio.transpose(2, 3, 0, 1))                                # [I][O][kh][kw]
    b = _normal_f32(st.next(), (cout,), 0.01) if bias else None
    return {"op": "conv", "in": src, "w": w, "b": b, "stride": (stride, stride), "relu": relu}


def _fc(st, src, k, n, relu):
    w = _normal_f32(st.next(), (k, n), np.sqrt(2.0 / k))
    b = _normal_f32(st.next(), (n,), 0.01)
    return {"op": "fc", "in": src, "w": w, "b": b, "relu": relu}


def _maxpool(src, k, s):
    return {"op": "pool", "in": src, "window": (k, k, 1), "stride": (s, s, 1), "kind": 0}


def image_input(st, w, h, c, scale=1.0, normalise=False):
    """HWC image drawn U[0,scale), optionally normalised per image, returned as CHW float32."""
    img = st.next().random((h, w, c), dtype=np.float32) * np.float32(scale)
    if normalise:
        img = ((img - img.mean()) / img.std()).astype(np.float32)
    return np.ascontiguousarray(img.transpose(2, 0, 1))


def _fire(st, spec, src, cin, squeeze, expand):
    spec.append(_conv(st, src, 1, cin, squeeze)); s = len(spec) - 1
    spec.append(_conv(st, s, 1, squeeze, expand)); e1 = len(spec) - 1
    spec.append(_conv(st, s, 3, squeeze, expand)); e3 = len(spec) - 1
    spec.append({"op": "concat", "ins": [e1, e3], "dim": 2})
    return len(spec) - 1


def conv3x3_single(seed=0, size=56, cin=64, cout=64):
    """Config 1: one 3x3 stride-1 conv with bias + ReLU on a size x size x cin input."""
    st = _Streams(seed)
    spec = [{"op": "feed", "shape": (size, size, cin)}, _conv(st, 0, 3, cin, cout)]
    return spec, {0: image_input(st, size, size, cin)}, [1]


def fire_module(seed=0, size=55, cin=128, squeeze=16, expand=64):
    """Config 2: SqueezeNet fire module (squeeze 1x1 -> expand 1x1 || expand 3x3 -> channel concat)."""
    st = _Streams(seed)
    spec = [{"op": "feed", "shape": (size, size, cin)}]
    out = _fire(st, spec, 0, cin, squeeze, expand)
    return spec, {0: image_input(st, size, size, cin)}, [out]


def vgg_conv3_block(seed=0, size=56, cin=128, cout=256):
    """Config 3: three 3x3 convs to cout channels + 2x2/2 max pool."""
    st = _Streams(seed)
    spec = [{"op": "feed", "shape": (size, size, cin)}]
    spec.append(_conv(st, 0, 3, cin, cout))
    spec.append(_conv(st, 1, 3, cout, cout))
    spec.append(_conv(st, 2, 3, cout, cout))
    spec.append(_maxpool(3, 2, 2))
    return spec, {0: image_input(st, size, size, cin)}, [4]


def squeezenet11(seed=0, size=224, classes=1000, normalise_in_graph=False):
    """Config 4: SqueezeNet v1.1 topology, random He-normal weights, per-image normalised input.

    normalise_in_graph: feed the raw U[0,255) image and let a Normalization node (mean 0, deviation 1)
    in front of conv1 do what the generator otherwise does on the host."""
    st = _Streams(seed)
    spec = [{"op": "feed", "shape": (size, size, 3)}]
    if normalise_in_graph:
        spec.append({"op": "norm", "in": 0, "kind": 2, "mean": 0.0, "dev": 1.0})
    spec.append(_conv(st, len(spec) - 1, 3, 3, 64, stride=2))
    spec.append(_maxpool(len(spec) - 1, 3, 2)); cur, cin = len(spec) - 1, 64
    plan = [(16, 64), (16, 64), "pool", (32, 128), (32, 128), "pool", (48, 192), (48, 192), (64, 256), (64, 256)]
    for item in plan:
        if item == "pool":
            spec.append(_maxpool(cur, 3, 2)); cur = len(spec) - 1
        else:
            cur = _fire(st, spec, cur, cin, item[0], item[1]); cin = 2 * item[1]
    spec.append(_conv(st, cur, 1, cin, classes)); cur = len(spec) - 1
    fin = size // 2                                  # conv1 /2, then three ceil-mode /2 pools
    for _ in range(3):
        fin = -(-fin // 2)
    spec.append({"op": "pool", "in": cur, "window": (fin, fin, 1), "stride": (fin, fin, 1), "kind": 1}); cur = len(spec) - 1
    spec.append({"op": "softmax", "in": cur})
    return spec, {0: image_input(st, size, size, 3, scale=255.0, normalise=not normalise_in_graph)}, [len(spec) - 1, len(spec) - 2]


def vgg16(seed=0, size=224, classes=1000, fc_width=4096):
    """Config 5: VGG16 (13 convs, 5 pools, 3 FC, softmax).  Outputs: softmax and the FC8 logits."""
    st = _Streams(seed)
    spec = [{"op": "feed", "shape": (size, size, 3)}]
    cur, cin = 0, 3
    for cout, reps in [(64, 2), (128, 2), (256, 3), (512, 3), (512, 3)]:
        for _ in range(reps):
            spec.append(_conv(st, cur, 3, cin, cout)); cur, cin = len(spec) - 1, cout
        spec.append(_maxpool(cur, 2, 2)); cur = len(spec) - 1
    side = size // 32
    spec.append(_fc(st, cur, side * side * 512, fc_width, True)); cur = len(spec) - 1
    spec.append(_fc(st, cur, fc_width, fc_width, True)); cur = len(spec) - 1
    spec.append(_fc(st, cur, fc_width, classes, False)); cur = len(spec) - 1
    spec.append({"op": "softmax", "in": cur})
    return spec, {0: image_input(st, size, size, 3)}, [len(spec) - 1, len(spec) - 2]


CONFIGS = {
    "conv3x3": conv3x3_single,
    "fire": fire_module,
    "vgg_conv3": vgg_conv3_block,
    "squeezenet": squeezenet11,
    "vgg16": vgg16,
}


def build_graph(graph, spec, outputs):
    """Create the spec's nodes in `graph` through the C API; returns the node handles.

    Tensors cross this boundary in the C API's own layouts ([C][H][W] / [I][O][kh][kw]); create the
    graph with interface layout 'CHW'-agnostic calls only (no transposes happen here).
    """
    lib = graph.lib
    nodes = []
    for n in spec:
        op = n["op"]
        if op == "feed":
            sh = dr.Shape3(*n["shape"])
            node = dr.Node(lib.dR_Datafeednode(graph.ptr, dr.pointer(sh)), graph, "DataFeedNode", list(n["shape"]))
            node.shape = list(n["shape"])
            graph.feed_nodes.append(node)
        elif op == "conv":
            node = dr.Conv2d_raw(nodes[n["in"]], n["w"], n.get("b"), n.get("stride", (1, 1)), "relu" if n.get("relu") else "linear")
        elif op == "pool":
            node = dr.Pooling(nodes[n["in"]], "max" if n["kind"] == 0 else "average", (1,) + tuple(n["window"]), (1,) + tuple(n["stride"]))
        elif op == "fc":
            node = dr.Fully_Connected(nodes[n["in"]], n["w"].shape, "relu" if n.get("relu") else "linear", n["w"], n.get("b"))
        elif op == "softmax":
            node = dr.Softmax(nodes[n["in"]])
        elif op == "concat":
            ptrs = (dr.c_void_p * len(n["ins"]))(*[nodes[i].ptr for i in n["ins"]])
            node = dr.Node(lib.dR_Concat(graph.ptr, ptrs, len(n["ins"]), n["dim"]), graph, "Concat", [])
        elif op == "slice":
            o, s = dr.Shape4(*n["origin"], 0), dr.Shape4(*n["shape"], 0)
            node = dr.Node(lib.dR_Slice(graph.ptr, nodes[n["in"]].ptr, dr.pointer(o), dr.pointer(s)), graph, "Slice", [])
        elif op == "norm":
            node = dr.Normalization(nodes[n["in"]], n["kind"], n["mean"], n["dev"])
        elif op == "scalar":
            node = dr.Node(lib.dR_ElemWise1Operation(graph.ptr, nodes[n["in"]].ptr, n["kind"], dr.c_float(n["value"])), graph, "ElemWise1Op", [])
        else:
            raise ValueError("unknown op %r" % op)
        nodes.append(node)
    for i in outputs:
        dr.mark_as_output(nodes[i])
    return nodes


def feed_chw(node, chw):
    """Feed a [C][H][W] float32 array as is (the C API's own layout)."""
    a = np.ascontiguousarray(chw, np.float32)
    node.graph.lib.dR_feedData(node.graph.ptr, node.ptr, a.ctypes.data_as(dr.POINTER(dr.c_float)), 0, a.size)


def fetch_chw(graph):
    """All outputs as [C][H][W] arrays (blocking)."""
    lib = graph.lib
    mem = (dr.c_void_p * max(graph.num_outputs, 1))()
    n = lib.dR_getOutputBuffers(graph.ptr, mem)
    outs = []
    for i in range(n):
        s = graph.outnodes[i].out_shape
        flat = np.empty(s[0] * s[1] * s[2], np.float32)
        lib.dR_downloadArray(graph.ptr, b"output", mem[i], 0, flat.nbytes, flat.ctypes.data_as(dr.c_void_p))
        outs.append(flat.reshape(s[2], s[1], s[0]))
    return outs


def flops(spec):
    """Direct-equivalent FLOPs (2*MAC) per node index; shapes are propagated with the reference's rules."""
    shapes, out = [], {}
    for i, n in enumerate(spec):
        op = n["op"]
        if op == "feed":
            shapes.append(tuple(n["shape"]))
        elif op == "conv":
            W, H, _ = shapes[n["in"]]
            I, O, kh, kw = n["w"].shape
            sx, sy = n.get("stride", (1, 1))
            shapes.append((W // sx, H // sy, O))
            out[i] = 2 * (W // sx) * (H // sy) * I * O * kh * kw
        elif op == "pool":
            W, H, C = shapes[n["in"]]
            stx, sty, stz = n["stride"]
            shapes.append((-(-W // stx), -(-H // sty), -(-C // stz)))
        elif op == "fc":
            K, N = n["w"].shape
            shapes.append((N, 1, 1))
            out[i] = 2 * K * N
        elif op == "concat":
            W, H, _ = shapes[n["ins"][0]]
            shapes.append((W, H, sum(shapes[j][2] for j in n["ins"])))
        else:
            shapes.append(shapes[n["in"]])
    return out, shapes
