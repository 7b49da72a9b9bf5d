"""CPU oracle for the deepRacin CNN layer path.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module; the
product (deepracin_amd, libdeepracin.so) never does.

Three layers of checking live here:
  * `lib` functions (conv_direct, conv_winograd, conv1x1, pool, fc, softmax ...): ctypes bindings to
    oracle/libdr_oracle.so, the scalar-C restatement of the reference's kernels in their own
    accumulation order (fp32);
  * `*_f64` functions: closed forms in float64 numpy, the mathematical truth the restatement itself
    is pinned against;
  * `run_spec` / `run_graph_dir`: evaluate a whole network (a layer list, or a stored graph.dr
    directory read by an independent pure-Python parser) with the lib functions, choosing the same
    algorithm per node as the reference's dispatch (src/dR_nodes_conv2d.c:37-81).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libdr_oracle.so")
_lib = None

_f = ctypes.POINTER(ctypes.c_float)
_i = ctypes.POINTER(ctypes.c_int)


def build(force=False):
    """Compile oracle/dr_oracle.c (gcc, OpenMP)."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)
    return _LIB_PATH


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_num_threads.restype = ctypes.c_int
    return _lib


def _p(a):
    return a.ctypes.data_as(_f) if a is not None else None


def _c(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def num_threads():
    return load().oracle_num_threads()


def set_threads(n):
    load().oracle_set_threads(int(n))


# ---------------------------------------------------------------------------------------------
# fp32 restatements (C)
# ---------------------------------------------------------------------------------------------

def conv_direct(x, w, b=None, stride=(1, 1), relu=False):
    """x [I,H,W]; w [I,O,kh,kw]; stride (sx, sy) -> [O, H//sy, W//sx]."""
    x, w = _c(x), _c(w)
    b = _c(b) if b is not None else None
    I, H, W = x.shape
    _, O, kh, kw = w.shape
    sx, sy = stride
    out = np.empty((O, H // sy, W // sx), np.float32)
    load().oracle_conv_direct(_p(x), _p(w), _p(b), _p(out), W, H, I, O, kw, kh, sx, sy, int(relu))
    return out


def wino_filter(w):
    """w [I,O,3,3] -> U in the reference layout [I,16,O]."""
    w = _c(w)
    I, O = w.shape[:2]
    U = np.empty((I, 16, O), np.float32)
    load().oracle_wino_filter(_p(w), _p(U), I, O)
    return U


def conv_winograd(x, w, b=None, relu=False):
    x = _c(x)
    b = _c(b) if b is not None else None
    U = wino_filter(w)
    I, H, W = x.shape
    O = U.shape[2]
    out = np.empty((O, H, W), np.float32)
    load().oracle_conv_winograd(_p(x), _p(U), _p(b), _p(out), W, H, I, O, int(relu))
    return out


def conv1x1(x, w, b=None, relu=False):
    """x [I,H,W]; w [I,O,1,1] or [I,O]."""
    x = _c(x)
    w = _c(w).reshape(w.shape[0], w.shape[1])
    b = _c(b) if b is not None else None
    I, H, W = x.shape
    O = w.shape[1]
    out = np.empty((O, H, W), np.float32)
    load().oracle_conv1x1(_p(x), _p(w), _p(b), _p(out), H * W, I, O, int(relu))
    return out


def conv2d(x, w, b=None, stride=(1, 1), relu=False, force_direct=False):
    """Algorithm dispatch of dR_Conv2d (reference src/dR_nodes_conv2d.c:37-81)."""
    kh, kw = w.shape[2], w.shape[3]
    if kh == 3 and kw == 3 and tuple(stride) == (1, 1) and not force_direct:
        return conv_winograd(x, w, b, relu)
    if kh == 1 and kw == 1 and tuple(stride) == (1, 1):
        return conv1x1(x, w, b, relu)
    return conv_direct(x, w, b, stride, relu)


def pool(x, window, stride, kind=0, want_argmax=False):
    """x [C,H,W]; window (sx,sy,sz); stride (stx,sty,stz); kind 0 max / 1 average."""
    x = _c(x)
    C, H, W = x.shape
    sx, sy, sz = window
    stx, sty, stz = stride
    out = np.empty((-(-C // stz), -(-H // sty), -(-W // stx)), np.float32)
    arg = np.empty(out.shape, np.int32) if want_argmax else None
    load().oracle_pool(_p(x), _p(out), arg.ctypes.data_as(_i) if arg is not None else None,
                       W, H, C, sx, sy, sz, stx, sty, stz, int(kind))
    return (out, arg) if want_argmax else out


def fc(x, Wt, b=None, relu=False, partition=0):
    """x [C,H,W]; Wt [K,N] with k counting x in [H][W][C] order."""
    x, Wt = _c(x), _c(Wt)
    b = _c(b) if b is not None else None
    C, H, W = x.shape
    N = Wt.shape[1]
    y = np.empty((N,), np.float32)
    load().oracle_fc(_p(x), _p(Wt), _p(b), _p(y), W, H, C, N, int(relu), int(partition))
    return y.reshape(1, 1, N)


def softmax(x):
    x = _c(x)
    y = np.empty_like(x)
    load().oracle_softmax(_p(x), _p(y), x.size)
    return y


def scalar_op(x, op, s):
    x = _c(x)
    y = np.empty_like(x)
    load().oracle_scalar_op(_p(x), _p(y), ctypes.c_size_t(x.size), int(op), ctypes.c_float(s))
    return y


def normalize(x, kind, target_mean=0.0, target_dev=1.0):
    """Normalization node on x [C,H,W]: kind 0 mean, 1 deviation, 2 both (reference tree-sum order)."""
    x = _c(x)
    C, H, W = x.shape
    y = np.empty_like(x)
    load().oracle_normalize(_p(x), _p(y), W, H, C, int(kind), ctypes.c_float(target_mean), ctypes.c_float(target_dev))
    return y


def normalize_f64(x, kind, target_mean=0.0, target_dev=1.0):
    """Closed form in float64: population mean / standard deviation over the whole tensor."""
    x64 = np.asarray(x, np.float64)
    add = target_mean - x64.mean() if kind != 1 else 0.0
    mul = target_dev / x64.std() if kind != 0 else 1.0
    return (x64 + add) * mul


def slice3d(x, origin, shape):
    """origin (x,y,z), shape (w,h,c) on x [C,H,W]."""
    x = _c(x)
    C, H, W = x.shape
    w, h, c = shape
    out = np.empty((c, h, w), np.float32)
    load().oracle_copy3d(_p(x), W, H, origin[0], origin[1], origin[2], _p(out), w, h, 0, 0, 0, w, h, c)
    return out


def concat(xs, dim):
    """dim in the reference's (W,H,C) numbering: 0 = W, 1 = H, 2 = C."""
    axis = {0: 2, 1: 1, 2: 0}[dim]
    return np.concatenate([_c(a) for a in xs], axis=axis)


# ---------------------------------------------------------------------------------------------
# float64 closed forms (numpy) -- what the restatements are pinned against
# ---------------------------------------------------------------------------------------------

def conv_f64(x, w, b=None, stride=(1, 1), relu=False):
    """Zero-padded cross-correlation, window of output (x,y) centred on input (x*sx, y*sy)."""
    x = np.asarray(x, np.float64)
    w = np.asarray(w, np.float64)
    I, H, W = x.shape
    _, O, kh, kw = w.shape
    sx, sy = stride
    Wo, Ho = W // sx, H // sy
    xp = np.zeros((I, H + kh - 1 + sy, W + kw - 1 + sx))
    xp[:, kh // 2:kh // 2 + H, kw // 2:kw // 2 + W] = x
    out = np.zeros((O, Ho, Wo))
    for j in range(kh):
        for i in range(kw):
            patch = xp[:, j:j + Ho * sy:sy, i:i + Wo * sx:sx]      # [I,Ho,Wo]
            out += np.einsum("chw,co->ohw", patch, w[:, :, j, i])
    if b is not None:
        out += np.asarray(b, np.float64)[:, None, None]
    return np.maximum(out, 0) if relu else out


def pool_f64(x, window, stride, kind=0):
    x = np.asarray(x, np.float64)
    C, H, W = x.shape
    sx, sy, sz = window
    stx, sty, stz = stride
    Co, Ho, Wo = -(-C // stz), -(-H // sty), -(-W // stx)
    xp = np.zeros((Co * stz + sz, Ho * sty + sy, Wo * stx + sx))
    xp[:C, :H, :W] = x
    out = np.full((Co, Ho, Wo), -np.inf) if kind == 0 else np.zeros((Co, Ho, Wo))
    for dz in range(sz):
        for dy in range(sy):
            for dx in range(sx):
                v = xp[dz:dz + Co * stz:stz, dy:dy + Ho * sty:sty, dx:dx + Wo * stx:stx]
                out = np.maximum(out, v) if kind == 0 else out + v
    return out if kind == 0 else out / (sx * sy * sz)


def fc_f64(x, Wt, b=None, relu=False):
    x = np.asarray(x, np.float64)
    xh = x.transpose(1, 2, 0).reshape(-1)          # [H][W][C] order
    y = xh @ np.asarray(Wt, np.float64)
    if b is not None:
        y = y + np.asarray(b, np.float64)
    return (np.maximum(y, 0) if relu else y).reshape(1, 1, -1)


def softmax_f64(x):
    x = np.asarray(x, np.float64)
    e = np.exp(x - x.max())
    return e / e.sum()


# ---------------------------------------------------------------------------------------------
# whole networks
# ---------------------------------------------------------------------------------------------

def run_spec(spec, feeds, force_direct=False, f64=False, inputs_from=None):
    """Evaluate a layer list (see deepracin_amd.configs) on the CPU.

    spec: list of dicts; node i may reference earlier nodes by index ('in' / 'ins').
    feeds: {node index: array [C,H,W]}.  Returns the list of all node outputs.
    f64=True evaluates with the closed forms instead of the fp32 restatements.
    inputs_from: {node index: array}; a node that reads one of these nodes is given that array instead of
    this evaluation's own result, so that every layer can be judged on the inputs the implementation
    under test actually had (per-layer error without the drift of the layers in front).
    """
    class _Inputs(list):
        def __getitem__(self, k):
            if inputs_from is not None and k in inputs_from and spec[k]["op"] != "feed":
                return np.asarray(inputs_from[k], np.float64 if f64 else np.float32)
            return list.__getitem__(self, k)

    outs = _Inputs()
    for idx, n in enumerate(spec):
        op = n["op"]
        if op == "feed":
            v = np.asarray(feeds[idx], np.float64 if f64 else np.float32)
        elif op == "conv":
            x = outs[n["in"]]
            if f64:
                v = conv_f64(x, n["w"], n.get("b"), n.get("stride", (1, 1)), n.get("relu", False))
            else:
                v = conv2d(x, n["w"], n.get("b"), n.get("stride", (1, 1)), n.get("relu", False), force_direct)
        elif op == "pool":
            fn = pool_f64 if f64 else pool
            v = fn(outs[n["in"]], n["window"], n["stride"], n["kind"])
        elif op == "fc":
            fn = fc_f64 if f64 else fc
            v = fn(outs[n["in"]], n["w"], n.get("b"), n.get("relu", False))
        elif op == "softmax":
            x = outs[n["in"]]
            v = softmax_f64(x) if f64 else softmax(x)
        elif op == "concat":
            v = concat([outs[i] for i in n["ins"]], n["dim"])
            if f64:
                v = v.astype(np.float64)
        elif op == "slice":
            v = slice3d(outs[n["in"]], n["origin"], n["shape"])
        elif op == "scalar":
            v = scalar_op(outs[n["in"]], n["kind"], n["value"])
        elif op == "norm":
            v = normalize_f64(outs[n["in"]], n["kind"], n["mean"], n["dev"]).astype(np.float32) if f64 else \
                normalize(outs[n["in"]], n["kind"], n["mean"], n["dev"])
        else:
            raise ValueError("unknown op %r" % op)
        outs.append(v)
    return list(outs)


def parse_graph_dir(path):
    """Independent pure-Python reader of the stored format (graph.dr + N.var) -> layer list."""
    with open(os.path.join(path, "graph.dr"), "rb") as fh:
        lines = [l for l in fh.read().decode("ascii").replace("\r", "\n").split("\n") if l]
    head = lines[0].split()
    n_nodes = int(head[2])
    spec = [None] * n_nodes
    for k in range(n_nodes):
        rec = lines[1 + 5 * k: 6 + 5 * k]
        nid = int(rec[0].split()[1].rstrip(":"))
        desc = rec[0].split()[2]
        params = rec[1].split()[1:]
        prev = [int(t) for t in rec[2].split()[1:]]
        files = rec[4].split()[1:]
        var = [np.fromfile(os.path.join(path, f), dtype="<f4") for f in files]
        if desc.startswith("DataFeedNode"):
            node = {"op": "feed", "shape": tuple(int(p) for p in params)}
        elif desc.startswith("Conv2D"):
            act, use_b, kw, kh, ci, co, _, sx, sy, _ = [int(p) for p in params]
            node = {"op": "conv", "in": prev[0], "w": var[0][:ci * co * kh * kw].reshape(ci, co, kh, kw),
                    "b": var[1][:co] if use_b else None, "stride": (sx, sy), "relu": act == 1}
        elif desc.startswith("Pooling"):
            t, _, sx, sy, sz, _, stx, sty, stz = [int(p) for p in params]
            node = {"op": "pool", "in": prev[0], "window": (sx, sy, sz), "stride": (stx, sty, stz), "kind": t}
        elif desc.startswith("FullyConnected"):
            act, use_b, K, N = [int(p) for p in params]
            node = {"op": "fc", "in": prev[0], "w": var[0][:K * N].reshape(K, N), "b": var[1][:N] if use_b else None,
                    "relu": act == 1}
        elif desc.startswith("Softmax"):
            node = {"op": "softmax", "in": prev[0]}
        elif desc.startswith("Slice"):
            p = [int(t) for t in params]
            node = {"op": "slice", "in": prev[0], "origin": tuple(p[0:3]), "shape": tuple(p[4:7])}
        elif desc.startswith("Concat"):
            node = {"op": "concat", "ins": prev, "dim": int(params[1])}
        elif desc.startswith("ElemWise1Op"):
            node = {"op": "scalar", "in": prev[0], "kind": int(params[0]), "value": float(params[1])}
        elif desc.startswith("Normalization"):
            node = {"op": "norm", "in": prev[0], "kind": int(params[0]), "mean": float(params[1]), "dev": float(params[2])}
        else:
            raise ValueError("node type %s not part of the CNN layer path" % desc)
        spec[nid] = node
    return spec


def run_graph_dir(path, feed):
    spec = parse_graph_dir(path)
    feeds = {i: feed for i, n in enumerate(spec) if n["op"] == "feed"}
    return run_spec(spec, feeds)
