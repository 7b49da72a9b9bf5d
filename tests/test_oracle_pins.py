"""Pins the CPU oracle (oracle/dr_oracle.c) before anything is compared against it.

The reference ships no unit tests; its only known answers are the two class ids of its SqueezeNet
example.  Every oracle function is therefore checked against something it was NOT written from:
float64 closed forms, library routines (torch, scipy), textbook identities and special cases chosen
so that a dropped term, a wrong sign/index or a transposed operand fails.  CPU only.
"""
import os

import numpy as np
import pytest
import scipy.special
import torch
import torch.nn.functional as F

from conftest import GOLDEN, rel_err

RNG = np.random.default_rng(1234)


def rnd(*shape):
    return RNG.standard_normal(shape).astype(np.float32)


# ---------------------------------------------------------------------------------------------
# direct convolution
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("I,O,H,W,k", [(3, 5, 9, 11, 3), (4, 2, 7, 7, 5), (2, 3, 6, 5, 1), (5, 4, 8, 8, 7)])
def test_conv_direct_matches_torch_and_closed_form(oracle, I, O, H, W, k):
    x, w, b = rnd(I, H, W), rnd(I, O, k, k), rnd(O)
    got = oracle.conv_direct(x, w, b, (1, 1), relu=False)
    lib_ref = F.conv2d(torch.from_numpy(x).double()[None], torch.from_numpy(w).double().permute(1, 0, 2, 3),
                       torch.from_numpy(b).double(), padding=k // 2)[0].numpy()
    assert rel_err(got, lib_ref) < 2e-6
    assert rel_err(oracle.conv_f64(x, w, b), lib_ref) < 1e-12      # the closed form agrees with the library


def test_conv_direct_delta_filter_shifts(oracle):
    # a filter that is 1 at tap (j,i) copies the input shifted by (j-1, i-1): pins the tap order/sign
    x = rnd(1, 6, 7)
    for j in range(3):
        for i in range(3):
            w = np.zeros((1, 1, 3, 3), np.float32)
            w[0, 0, j, i] = 1
            got = oracle.conv_direct(x, w)[0]
            want = np.zeros_like(x[0])
            for y in range(6):
                for xx in range(7):
                    yy, xs = y + j - 1, xx + i - 1
                    if 0 <= yy < 6 and 0 <= xs < 7:
                        want[y, xx] = x[0, yy, xs]
            assert np.array_equal(got, want)


def test_conv_direct_ones_counts_zero_padding(oracle):
    # all-ones 3x3 on all-ones image: 4 at corners, 6 on edges, 9 inside -> pins the zero padding
    got = oracle.conv_direct(np.ones((1, 5, 6), np.float32), np.ones((1, 1, 3, 3), np.float32))[0]
    assert got[0, 0] == 4 and got[0, -1] == 4 and got[-1, 0] == 4 and got[-1, -1] == 4
    assert np.all(got[0, 1:-1] == 6) and np.all(got[1:-1, 0] == 6)
    assert np.all(got[1:-1, 1:-1] == 9)


def test_conv_direct_channel_and_filter_indexing(oracle):
    # weights [I][O][kh][kw]: output o only sees w[:, o]; a transposed I/O layout would fail
    x = rnd(3, 4, 4)
    w = np.zeros((3, 2, 1, 1), np.float32)
    w[2, 1, 0, 0] = 2.0
    got = oracle.conv_direct(x, w)
    assert np.all(got[0] == 0) and np.allclose(got[1], 2 * x[2])


@pytest.mark.parametrize("H,W,s", [(8, 8, 2), (9, 7, 2), (12, 10, 3)])
def test_conv_direct_stride_follows_header_formula(oracle, H, W, s):
    # window of output (x,y) centred on input (x*s, y*s), output floor(in/s)
    # (reference include/dR_nodes_conv2d.h:47-54): brute force in float64
    I, O = 2, 3
    x, w = rnd(I, H, W), rnd(I, O, 3, 3)
    got = oracle.conv_direct(x, w, None, (s, s))
    want = np.zeros((O, H // s, W // s))
    for o in range(O):
        for y in range(H // s):
            for xx in range(W // s):
                acc = 0.0
                for c in range(I):
                    for j in range(3):
                        for i in range(3):
                            yy, xs = y * s + j - 1, xx * s + i - 1
                            if 0 <= yy < H and 0 <= xs < W:
                                acc += float(x[c, yy, xs]) * float(w[c, o, j, i])
                want[o, y, xx] = acc
    assert got.shape == want.shape
    assert rel_err(got, want) < 2e-6
    assert rel_err(oracle.conv_f64(x, w, None, (s, s)), want) < 1e-12
    # equals a stride-1 convolution sampled at multiples of s
    full = oracle.conv_direct(x, w)
    assert np.allclose(got, full[:, ::s, ::s][:, :H // s, :W // s], atol=1e-6)


def test_conv_bias_and_relu(oracle):
    x, w, b = rnd(2, 5, 5), rnd(2, 3, 3, 3), rnd(3)
    lin = oracle.conv_direct(x, w, b, relu=False)
    assert np.allclose(lin - oracle.conv_direct(x, w, None), b[:, None, None], atol=1e-6)
    assert np.array_equal(oracle.conv_direct(x, w, b, relu=True), np.maximum(lin, 0))


# ---------------------------------------------------------------------------------------------
# Winograd F(2x2,3x3)
# ---------------------------------------------------------------------------------------------

def test_winograd_filter_transform_is_GgGt(oracle):
    G = np.array([[1, 0, 0], [.5, .5, .5], [.5, -.5, .5], [0, 0, 1]], np.float64)
    w = rnd(3, 2, 3, 3)
    U = oracle.wino_filter(w)                   # [I,16,O]
    for c in range(3):
        for o in range(2):
            want = G @ w[c, o].astype(np.float64) @ G.T
            assert np.allclose(U[c, :, o].reshape(4, 4), want, atol=1e-6)


def test_winograd_single_tile_identity(oracle):
    # A^T[(G g G^T) .* (B^T d B)]A == valid 3x3 correlation of a 4x4 block (Lavin & Gray),
    # with the reference's sign convention (4th row of B^T and 4th column of A^T negated)
    Bt = np.array([[1, 0, -1, 0], [0, 1, 1, 0], [0, -1, 1, 0], [0, -1, 0, 1]], np.float64)
    At = np.array([[1, 1, 1, 0], [0, 1, -1, 1]], np.float64)
    G = np.array([[1, 0, 0], [.5, .5, .5], [.5, -.5, .5], [0, 0, 1]], np.float64)
    d, g = RNG.standard_normal((4, 4)), RNG.standard_normal((3, 3))
    Y = At @ ((G @ g @ G.T) * (Bt @ d @ Bt.T)) @ At.T
    want = np.array([[np.sum(d[y:y + 3, x:x + 3] * g) for x in range(2)] for y in range(2)])
    assert np.allclose(Y, want, atol=1e-12)
    # and the oracle reproduces it on a 2x2 image whose padded window is d's interior
    x = np.zeros((1, 2, 2), np.float32)
    x[0] = d[1:3, 1:3]
    got = oracle.conv_winograd(x, g.astype(np.float32).reshape(1, 1, 3, 3))
    dz = np.zeros((4, 4)); dz[1:3, 1:3] = x[0]
    wantz = np.array([[np.sum(dz[y:y + 3, xx:xx + 3] * g.astype(np.float32)) for xx in range(2)] for y in range(2)])
    assert np.allclose(got[0], wantz, atol=1e-5)


@pytest.mark.parametrize("I,O,H,W", [(4, 3, 8, 8), (3, 5, 7, 9), (16, 8, 11, 5), (1, 1, 1, 1), (2, 2, 2, 3)])
def test_winograd_equals_direct(oracle, I, O, H, W):
    x, w, b = rnd(I, H, W), rnd(I, O, 3, 3), rnd(O)
    a = oracle.conv_winograd(x, w, b, relu=True)
    d = oracle.conv_direct(x, w, b, relu=True)
    truth = oracle.conv_f64(x, w, b, relu=True)
    assert a.shape == d.shape == (O, H, W)
    assert rel_err(a, truth) < 1e-5 and rel_err(d, truth) < 1e-5


def test_conv1x1_matches_einsum(oracle):
    x, w, b = rnd(7, 5, 6), rnd(7, 4, 1, 1), rnd(4)
    got = oracle.conv1x1(x, w, b, relu=True)
    want = np.maximum(np.einsum("chw,co->ohw", x.astype(np.float64), w[:, :, 0, 0].astype(np.float64)) + b[:, None, None], 0)
    assert rel_err(got, want) < 2e-6
    assert rel_err(oracle.conv_direct(x, w, b, relu=True), want) < 2e-6


# ---------------------------------------------------------------------------------------------
# pooling
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("H,W,k,s", [(8, 8, 2, 2), (9, 7, 3, 2), (112, 112, 3, 2), (14, 14, 14, 14), (5, 6, 2, 3)])
def test_pool_matches_torch_on_zero_padded_input(oracle, H, W, k, s):
    x = np.abs(rnd(3, H, W))          # non-negative: zero padding == -inf padding for max
    Ho, Wo = -(-H // s), -(-W // s)
    padded = np.zeros((3, max(H, (Ho - 1) * s + k), max(W, (Wo - 1) * s + k)), np.float32)
    padded[:, :H, :W] = x
    t = torch.from_numpy(padded)[None]
    mx = F.max_pool2d(t, k, s)[0].numpy()
    av = F.avg_pool2d(t, k, s)[0].numpy()
    got_max = oracle.pool(x, (k, k, 1), (s, s, 1), 0)
    got_avg = oracle.pool(x, (k, k, 1), (s, s, 1), 1)
    assert got_max.shape == (3, Ho, Wo)
    assert np.array_equal(got_max, mx)
    assert np.allclose(got_avg, av, rtol=1e-6, atol=1e-7)
    assert np.allclose(got_avg, oracle.pool_f64(x, (k, k, 1), (s, s, 1), 1), rtol=1e-6)


@pytest.mark.parametrize("C,H,W,win,st", [(8, 6, 6, (2, 2, 2), (2, 2, 2)), (7, 5, 9, (3, 2, 3), (2, 2, 2)),
                                          (6, 4, 4, (1, 1, 3), (1, 1, 1)), (5, 7, 3, (2, 3, 2), (1, 2, 3))])
def test_pool_with_depth_window_matches_torch_3d(oracle, C, H, W, win, st):
    """Windows that span channels (sz > 1): torch's max_pool3d / avg_pool3d on the input zero-padded at the
    far end of every axis are the library routines this reduces to (window anchored at out*stride, samples
    outside read 0.0, the average divides by the full window).  A window walking the wrong axis, a stride
    applied to the wrong axis or a divisor that forgets sz would fail."""
    sx, sy, sz = win
    stx, sty, stz = st
    x = np.abs(rnd(C, H, W)) + 0.1       # positive: zero padding == -inf padding for max
    Co, Ho, Wo = -(-C // stz), -(-H // sty), -(-W // stx)
    padded = np.zeros((max(C, (Co - 1) * stz + sz), max(H, (Ho - 1) * sty + sy), max(W, (Wo - 1) * stx + sx)), np.float32)
    padded[:C, :H, :W] = x
    t = torch.from_numpy(padded)[None, None]
    mx = F.max_pool3d(t, (sz, sy, sx), (stz, sty, stx))[0, 0].numpy()
    av = F.avg_pool3d(t.double(), (sz, sy, sx), (stz, sty, stx))[0, 0].numpy()
    got_max, arg = oracle.pool(x, win, st, 0, want_argmax=True)
    got_avg = oracle.pool(x, win, st, 1)
    assert got_max.shape == (Co, Ho, Wo) == mx.shape
    assert np.array_equal(got_max, mx)
    assert np.array_equal(x.reshape(-1)[arg.reshape(-1)], got_max.reshape(-1))      # the index points at the maximum
    assert np.allclose(got_avg, av, rtol=1e-6, atol=1e-7)


def test_pool_max_pads_with_zero_not_minus_inf(oracle):
    # a window hanging over the border sees 0.0f: with negative inputs the result is 0, not the max
    x = -np.ones((1, 3, 3), np.float32)
    got, arg = oracle.pool(x, (2, 2, 1), (2, 2, 1), 0, want_argmax=True)
    assert got.shape == (1, 2, 2)
    assert got[0, 0, 0] == -1 and got[0, 0, 1] == 0 and got[0, 1, 0] == 0 and got[0, 1, 1] == 0
    assert arg[0, 0, 0] == 0 and arg[0, 1, 1] == -1


def test_pool_argmax_is_first_max_in_scan_order(oracle):
    x = np.zeros((1, 4, 4), np.float32)
    x[0, 0, 1] = 5; x[0, 1, 0] = 5            # two equal maxima in window (0,0): first in y,x order wins
    _, arg = oracle.pool(x, (2, 2, 1), (2, 2, 1), 0, want_argmax=True)
    assert arg[0, 0, 0] == 1


# ---------------------------------------------------------------------------------------------
# fully connected, softmax
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("C,H,W,N,P", [(4, 3, 2, 5, 0), (8, 1, 1, 3, 0), (3, 2, 2, 7, 5), (16, 7, 7, 10, 64)])
def test_fc_reads_input_in_hwc_order(oracle, C, H, W, N, P):
    x, Wt, b = rnd(C, H, W), rnd(C * H * W, N), rnd(N)
    got = oracle.fc(x, Wt, b, relu=False, partition=P).reshape(-1)
    xh = x.transpose(1, 2, 0).reshape(-1)
    want = F.linear(torch.from_numpy(xh).double(), torch.from_numpy(Wt).double().t(), torch.from_numpy(b).double()).numpy()
    assert rel_err(got, want) < 5e-6
    if H * W > 1 and C > 1:                      # reading in CHW order instead must NOT match
        wrong = x.reshape(-1).astype(np.float64) @ Wt.astype(np.float64) + b
        assert rel_err(wrong, want) > 1e-3
    assert np.array_equal(oracle.fc(x, Wt, b, relu=True).reshape(-1), np.maximum(oracle.fc(x, Wt, b).reshape(-1), 0))


def test_softmax_matches_scipy(oracle):
    x = rnd(1000) * 3
    got = oracle.softmax(x)
    want = scipy.special.softmax(x.astype(np.float64))
    assert rel_err(got, want) < 1e-5
    assert abs(float(got.sum()) - 1.0) < 1e-5
    assert int(got.argmax()) == int(x.argmax())


@pytest.mark.parametrize("C,H,W", [(3, 224, 224), (1, 5, 7), (4, 17, 33), (2, 8, 16), (5, 1, 1)])
def test_normalize_matches_numpy_mean_and_std(oracle, C, H, W):
    """Normalization node: mean and POPULATION standard deviation over the whole tensor (numpy's
    float64 mean / std are the library routines the closed form reduces to), deviation about the mean
    for type 1 too.  A sample deviation (n-1), a per-channel statistic or a dropped mean would fail."""
    rng = np.random.default_rng(C * 100 + H)
    x = (rng.random((C, H, W), dtype=np.float32) * 255.0 + np.arange(C, dtype=np.float32)[:, None, None] * 40.0).astype(np.float32)
    x64 = x.astype(np.float64)
    n = x.size
    y0 = oracle.normalize(x, 0, 3.0, 1.0)
    assert abs(float(y0.astype(np.float64).mean()) - 3.0) < 1e-3 and np.allclose(y0, x64 + (3.0 - x64.mean()), rtol=1e-5, atol=1e-3)
    if n > 1:
        y1 = oracle.normalize(x, 1, 0.0, 2.0)
        assert np.allclose(y1, x64 * (2.0 / x64.std()), rtol=1e-4, atol=1e-4)
        assert abs(float(y1.astype(np.float64).std()) - 2.0) < 1e-3
        y2 = oracle.normalize(x, 2, 0.5, 1.5)
        # (x + (0.5 - mean)) * (1.5 / std), Kernels/dR_math.cl:143: the target mean is scaled as well
        want = (x64 - x64.mean()) / x64.std() * 1.5 + 0.5 * 1.5 / x64.std()
        assert np.allclose(y2, want, rtol=1e-4, atol=1e-4)
        assert np.allclose(y2, oracle.normalize_f64(x, 2, 0.5, 1.5), rtol=1e-4, atol=1e-4)
        assert abs(float(y2.astype(np.float64).std()) - 1.5) < 1e-3
        if C > 1:     # one statistic for the whole tensor, not one per channel
            assert abs(float(y2[0].astype(np.float64).mean()) - float(y2[-1].astype(np.float64).mean())) > 0.1
    # invariances that fix signs: shifting the input does not change a mean-normalised output
    assert np.allclose(oracle.normalize(x + np.float32(10.0), 0, 0.0, 1.0), oracle.normalize(x, 0, 0.0, 1.0), atol=2e-3)


def test_scalar_concat_slice(oracle):
    x = rnd(4, 3, 5)
    assert np.array_equal(oracle.scalar_op(x, 1, 2.5), x - np.float32(2.5))
    assert np.array_equal(oracle.scalar_op(x, 0, 2.5), x + np.float32(2.5))
    # the remaining operations of dR_ElemWise1OperationType against numpy's float32 routines
    # (Kernels/dR_math.cl:170-341): 2 x*s, 3 x/s, 4 log x, 5 exp x, 6 sqrt x, 7 s, 8 pow(x, s)
    assert np.array_equal(oracle.scalar_op(x, 2, -1.75), x * np.float32(-1.75))
    assert np.array_equal(oracle.scalar_op(x, 3, 3.0), x / np.float32(3.0))
    assert np.array_equal(oracle.scalar_op(x, 7, 0.625), np.full_like(x, 0.625))
    pos = np.abs(x) + np.float32(0.5)
    assert np.allclose(oracle.scalar_op(pos, 4, 0.0), np.log(pos.astype(np.float64)), rtol=1e-6, atol=1e-7)
    assert np.allclose(oracle.scalar_op(x, 5, 0.0), np.exp(x.astype(np.float64)), rtol=1e-6)
    assert np.allclose(oracle.scalar_op(pos, 6, 0.0), np.sqrt(pos.astype(np.float64)), rtol=1e-6)
    assert np.allclose(oracle.scalar_op(pos, 8, 1.5), pos.astype(np.float64) ** 1.5, rtol=1e-6)
    assert not np.array_equal(oracle.scalar_op(x, 3, 3.0), np.float32(3.0) / x)         # x/s, not s/x
    assert np.array_equal(oracle.slice3d(x, (1, 0, 2), (3, 2, 1)), x[2:3, 0:2, 1:4])
    assert np.array_equal(oracle.concat([x, x * 2], 2), np.concatenate([x, x * 2], 0))


# ---------------------------------------------------------------------------------------------
# the reference's own known answers: stored SqueezeNet v1.1 + two images
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("name,cls", [("tiger", 292), ("puzzle", 611)])
def test_stored_squeezenet_known_answers(oracle, name, cls):
    # examples/squeezenet-v1.1/squeezenet_deployed.c:153-157,199-207: feed RGB [c,h,w] floats 0..255,
    # expect argmax 292 (tiger) / 611 (jigsaw puzzle)
    img = np.load(os.path.join(GOLDEN, "%s_224_rgb_u8.npy" % name))
    chw = np.ascontiguousarray(img.transpose(2, 0, 1).astype(np.float32))
    outs = oracle.run_graph_dir(os.path.join(GOLDEN, "squeezenet_whole"), chw)
    p = outs[-1].reshape(-1)
    assert p.shape == (1000,)
    assert int(p.argmax()) == cls
    assert abs(float(p.sum()) - 1.0) < 1e-4


def test_stored_model_variable_sizes_match_params(oracle):
    spec = oracle.parse_graph_dir(os.path.join(GOLDEN, "squeezenet_whole"))
    assert len(spec) == 48 and spec[0]["op"] == "feed" and spec[0]["shape"] == (224, 224, 3)
    files = 0
    for n in spec:
        if n["op"] == "conv":
            files += 2
            assert n["w"].size == np.prod(n["w"].shape) and n["b"].size == n["w"].shape[1]
    assert files == 52
    assert os.path.getsize(os.path.join(GOLDEN, "squeezenet_whole", "0.var")) == 3 * 64 * 3 * 3 * 4
    assert os.path.getsize(os.path.join(GOLDEN, "squeezenet_whole", "50.var")) == 512 * 1000 * 4
