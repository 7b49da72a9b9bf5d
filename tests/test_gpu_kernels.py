"""Parity of every hand-written HIP kernel against the CPU oracle, called through the C-ABI
device layer (include/dr_hip.h) with plain device pointers.

Tolerances (north star): fp32 layers max relative error <= 1e-4, measured as
max|gpu - oracle| / max|oracle| over the layer; pooling values and max-indices bit-exact.
"""
import ctypes
import os

import numpy as np
import pytest

from conftest import Dev, assert_close, rel_err

pytestmark = pytest.mark.gpu

TOL = 1e-4
RNG = np.random.default_rng(7)


def rnd(*shape, scale=1.0):
    return (RNG.standard_normal(shape) * scale).astype(np.float32)


def ok(lib, rc):
    assert rc == 0, lib.drhip_last_error().decode()


# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("W,H,I,O,k,s", [
    (56, 56, 64, 64, 3, 1),      # config 1, direct variant
    (224, 224, 3, 64, 3, 2),     # SqueezeNet conv1
    (17, 13, 5, 7, 3, 1), (20, 18, 4, 20, 5, 1), (33, 31, 3, 9, 3, 2), (16, 16, 2, 3, 7, 3), (9, 9, 1, 1, 1, 2),
    (37, 21, 4, 33, 3, 1), (8, 5, 1, 16, 3, 3), (2, 2, 3, 2, 3, 1),     # I <= 4 with a 3x3 filter: the no-LDS first-layer kernel
    (112, 110, 24, 40, 3, 1), (61, 37, 17, 70, 3, 2), (30, 9, 8, 32, 3, 1),   # 3x3 with raw weights and more than 4 channels: the LDS-tiled kernel
])
def test_conv_direct(lib, dev, oracle, W, H, I, O, k, s):
    x, w, b = np.abs(rnd(I, H, W)), rnd(I, O, k, k, scale=np.sqrt(2.0 / (k * k * I))), rnd(O, scale=0.01)
    want = oracle.conv_direct(x, w, b, (s, s), relu=True)
    out = dev.empty(want.size)
    ok(lib, lib.drhip_conv2d_direct_f32(dev.put(x), dev.put(w), dev.put(b), out, W, H, I, O, k, k, s, s, 1, None))
    got = dev.get(out, want.shape)
    assert_close(got, want)
    # linear, no bias
    want2 = oracle.conv_direct(x, w, None, (s, s), relu=False)
    ok(lib, lib.drhip_conv2d_direct_f32(dev.put(x), dev.put(w), None, out, W, H, I, O, k, k, s, s, 0, None))
    assert_close(dev.get(out, want2.shape), want2)


@pytest.mark.parametrize("variant", [0, 1, 2, 4, 8, 0x11, 0x14, 0x18])
@pytest.mark.parametrize("W,H,I,O,s", [
    (56, 56, 64, 64, 1),         # config 1, direct variant
    (56, 56, 128, 256, 1),       # config 3's first layer
    (112, 110, 24, 40, 1), (61, 37, 17, 70, 2), (30, 9, 8, 32, 1), (55, 55, 16, 64, 1), (7, 9, 5, 3, 1), (1, 1, 9, 1, 1),
    (2, 3, 33, 65, 2), (28, 28, 40, 48, 2), (3, 1, 6, 2, 1),
])
def test_conv3x3_direct_mfma(lib, dev, oracle, variant, W, H, I, O, s):
    """The implicit-GEMM 3x3 kernel over the prepared filter bank: oracle (same algorithm, direct order), the
    float64 closed form, and the filter bank's layout itself.  Signed inputs, so every padding sample matters."""
    x, w, b = rnd(I, H, W), rnd(I, O, 3, 3, scale=np.sqrt(2.0 / (9 * I))), rnd(O, scale=0.01)
    n = lib.drhip_conv3x3_direct_filter_floats(I, O)
    chunks, opad = -(-I // 8), -(-O // 32) * 32
    assert n == 9 * chunks * 8 * opad
    F = dev.empty(n)
    ok(lib, lib.drhip_conv3x3_direct_filter_layout_f32(dev.put(w), F, I, O, None))
    if variant == 0:
        expect = np.zeros((9, chunks, opad, 8), np.float32)       # [tap][c/8][o][pos], pos = (c&1)*4 + (c%8)/2
        for c in range(I):
            expect[:, c // 8, :O, (c & 1) * 4 + (c % 8) // 2] = w[c].reshape(O, 9).T
        assert np.array_equal(dev.get(F, expect.shape), expect)
    want = oracle.conv_direct(x, w, b, (s, s), relu=True)
    out = dev.empty(want.size)
    xd, bd = dev.put(x), dev.put(b)
    ok(lib, lib.drhip_conv3x3_direct_mfma_f32(xd, F, bd, out, W, H, I, O, s, 1, variant, None))
    got = dev.get(out, want.shape)
    assert_close(got, want, terms=9 * I)
    assert_close(got, oracle.conv_f64(x, w, b, stride=(s, s), relu=True), terms=9 * I)
    want2 = oracle.conv_direct(x, w, None, (s, s), relu=False)      # linear, no bias: sign-sensitive
    ok(lib, lib.drhip_conv3x3_direct_mfma_f32(xd, F, None, out, W, H, I, O, s, 0, variant, None))
    assert_close(dev.get(out, want2.shape), want2, terms=9 * I)
    if variant == 0:
        assert lib.drhip_conv3x3_direct_mfma_f32(xd, F, None, out, W, H, I, O, 3, 0, 0, None) == -1      # stride 3
        assert lib.drhip_conv3x3_direct_mfma_f32(xd, F, None, out, W, H, I, O, s, 0, 3, None) == -1      # 3 waves


@pytest.mark.parametrize("W,H,I,O,sx,sy", [(224, 224, 3, 64, 2, 2), (33, 31, 3, 9, 2, 2), (17, 13, 1, 5, 1, 1), (20, 18, 4, 70, 1, 2),
                                            (8, 5, 2, 16, 3, 1), (2, 2, 3, 2, 1, 1), (9, 9, 4, 33, 2, 2), (64, 48, 3, 32, 1, 1)])
@pytest.mark.parametrize("relu", [1, 0])
def test_first_layer_conv_with_maxpool(lib, dev, oracle, W, H, I, O, sx, sy, relu):
    """3x3 first-layer convolution + 3x3/2 max pooling in one kernel against the two oracle steps.
    Without ReLU the convolution has negative outputs, so the pooling's zero padding is visible."""
    x, w, b = rnd(I, H, W), rnd(I, O, 3, 3, scale=np.sqrt(2.0 / (9 * I))), rnd(O, scale=0.05)
    conv = oracle.conv_direct(x, w, b, (sx, sy), relu=bool(relu))
    want = oracle.pool(conv, (3, 3, 1), (2, 2, 1), 0)
    out = dev.empty(want.size)
    ok(lib, lib.drhip_conv3x3_pool3s2_f32(dev.put(x), dev.put(w), dev.put(b), out, W, H, I, O, sx, sy, relu, None))
    got = dev.get(out, want.shape)
    assert_close(got, want)
    assert_close(got, oracle.pool_f64(oracle.conv_f64(x, w, b, stride=(sx, sy), relu=bool(relu)), (3, 3, 1), (2, 2, 1), 0))
    # no bias
    want2 = oracle.pool(oracle.conv_direct(x, w, None, (sx, sy), relu=bool(relu)), (3, 3, 1), (2, 2, 1), 0)
    ok(lib, lib.drhip_conv3x3_pool3s2_f32(dev.put(x), dev.put(w), None, out, W, H, I, O, sx, sy, relu, None))
    assert_close(dev.get(out, want2.shape), want2)
    assert lib.drhip_conv3x3_pool3s2_f32(dev.put(x), dev.put(w), None, out, W, H, 5, O, sx, sy, relu, None) == -1


def test_conv_direct_valu_kernels(lib, dev, oracle):
    """DR_DIRECT_VALU=1: the LDS-tiled / first-layer VALU kernels behind the matrix-core forms."""
    import os
    os.environ["DR_DIRECT_VALU"] = "1"
    try:
        for (W, H, I, O, s) in [(56, 56, 64, 64, 1), (224, 224, 3, 64, 2), (33, 31, 3, 9, 2), (30, 9, 8, 32, 1)]:
            x, w, b = rnd(I, H, W), rnd(I, O, 3, 3, scale=np.sqrt(2.0 / (9 * I))), rnd(O, scale=0.01)
            want = oracle.conv_direct(x, w, b, (s, s), relu=True)
            out = dev.empty(want.size)
            ok(lib, lib.drhip_conv2d_direct_f32(dev.put(x), dev.put(w), dev.put(b), out, W, H, I, O, 3, 3, s, s, 1, None))
            assert_close(dev.get(out, want.shape), want)
    finally:
        os.environ.pop("DR_DIRECT_VALU", None)


def wino_filters(lib, dev, w):
    I, O = w.shape[:2]
    n = lib.drhip_conv3x3_winograd_filter_floats(I, O)
    U = dev.empty(n)
    ok(lib, lib.drhip_winograd_filter_transform_f32(dev.put(w), U, I, O, None))
    return U, n


def wino_workspace(lib, dev, W, H, I, O, variant):
    n = lib.drhip_conv3x3_winograd_workspace_floats(W, H, I, O, variant)
    if not n:
        return None
    ws = dev.put(np.full(n, np.nan, np.float32))          # poison: nothing may be read before it is written
    if variant & 0x800:                                   # joined splits watch the slots for a marker
        ok(lib, lib.drhip_conv3x3_winograd_workspace_prepare_f32(ws, n, None))
    return ws


def test_winograd_filter_transform(lib, dev, oracle):
    I, O = 19, 37
    w = rnd(I, O, 3, 3)
    U, n = wino_filters(lib, dev, w)
    chunks, opad = -(-I // 8), -(-O // 32) * 32
    assert n == 16 * chunks * 8 * opad
    got = dev.get(U, (16, chunks, opad, 8))
    want = oracle.wino_filter(w)                          # reference layout [I,16,O]
    # device layout: [xi][c/8][o][pos], channel c%8 at pos (c&1)*4 + (c%8)/2; c and o zero padded
    expect = np.zeros((16, chunks, opad, 8), np.float32)
    for c in range(I):
        expect[:, c // 8, :O, (c & 1) * 4 + (c % 8) // 2] = want[c]
    assert np.allclose(got, expect, rtol=1e-6, atol=1e-7)


@pytest.mark.parametrize("variant", [1, 2, 3, 0x11, 0x21, 0x12, 0x33, 0x101, 0x102, 0x103, 0x111, 0x122,
                                     0x401, 0x402, 0x411, 0x432, 0x501, 0x502, 0x503, 0x512])
@pytest.mark.parametrize("W,H,I,O", [
    (56, 56, 64, 64),        # config 1
    (55, 55, 16, 64),        # fire expand3x3: odd size, two stages of 8 channels
    (28, 28, 24, 40),        # I not a multiple of 8, O not a multiple of 32
    (14, 14, 48, 96), (7, 9, 3, 5), (1, 1, 1, 1), (2, 3, 9, 33), (224, 224, 3, 64),
])
def test_winograd_conv(lib, dev, oracle, variant, W, H, I, O):
    x, w, b = np.abs(rnd(I, H, W)), rnd(I, O, 3, 3, scale=np.sqrt(2.0 / (9 * I))), rnd(O, scale=0.01)
    U, _ = wino_filters(lib, dev, w)
    ws = wino_workspace(lib, dev, W, H, I, O, variant)
    want = oracle.conv_winograd(x, w, b, relu=True)
    floor = float(np.abs(b).max())                    # tiny tensors: the output can be what is left of bias against conv sum
    out = dev.empty(want.size)
    xd, bd = dev.put(x), dev.put(b)
    for _ in range(2):                       # twice: a split layer must leave its counters at zero
        ok(lib, lib.drhip_conv3x3_winograd_f32(xd, U, bd, out, W, H, I, O, 1, variant, ws, None))
        got = dev.get(out, want.shape)
        assert_close(got, want, floor=floor)
    truth = oracle.conv_f64(x, w, b, relu=True)
    assert_close(got, truth, floor=floor)
    # linear, no bias (pre-activation values, sign-sensitive)
    want2 = oracle.conv_winograd(x, w, None, relu=False)
    ok(lib, lib.drhip_conv3x3_winograd_f32(xd, U, None, out, W, H, I, O, 0, variant, ws, None))
    assert_close(dev.get(out, want2.shape), want2)


@pytest.mark.parametrize("variant", [1, 2, 0x11, 0x22, 0x101, 0x112, 0x401, 0x412, 0x502])
@pytest.mark.parametrize("W,H,I,O", [(56, 56, 64, 64), (28, 12, 24, 40), (2, 2, 1, 1), (224, 224, 3, 64)])
def test_winograd_fused_maxpool(lib, dev, oracle, variant, W, H, I, O):
    """Epilogue flag 2: the kernel stores the 2x2/2 maximum of every output tile -- bit for bit what
    the pooling kernel makes of the kernel's own unpooled output."""
    x, w, b = rnd(I, H, W), rnd(I, O, 3, 3, scale=np.sqrt(2.0 / (9 * I))), rnd(O, scale=0.01)
    U, _ = wino_filters(lib, dev, w)
    ws = wino_workspace(lib, dev, W, H, I, O, variant)
    xd, bd = dev.put(x), dev.put(b)
    for relu in (1, 0):
        full = dev.empty(O * H * W)
        ok(lib, lib.drhip_conv3x3_winograd_f32(xd, U, bd, full, W, H, I, O, relu, variant, ws, None))
        want = oracle.pool(dev.get(full, (O, H, W)), (2, 2, 1), (2, 2, 1), 0)
        pooled = dev.empty(want.size)
        ok(lib, lib.drhip_conv3x3_winograd_f32(xd, U, bd, pooled, W, H, I, O, relu | 2, variant, ws, None))
        assert np.array_equal(dev.get(pooled, want.shape), want)
        ref = oracle.pool(oracle.conv_winograd(x, w, b, relu=bool(relu)), (2, 2, 1), (2, 2, 1), 0)
        assert_close(dev.get(pooled, want.shape), ref)
    p = dev.empty(64)
    assert lib.drhip_conv3x3_winograd_f32(p, U, None, p, 3, 4, I, O, 2, 1, None, None) == -1      # odd width
    assert lib.drhip_conv3x3_winograd_f32(p, U, None, p, 4, 4, I, O, 4, 1, None, None) == -1      # unknown flag


@pytest.mark.parametrize("variant", [0x811, 0x812, 0x821, 0x831, 0xc11, 0xc12, 0xc21, 0xc22, 0xc31])
@pytest.mark.parametrize("W,H,I,O", [
    (56, 56, 64, 64), (14, 14, 64, 96), (28, 20, 32, 40), (13, 9, 16, 33), (2, 2, 128, 3), (14, 14, 512, 512),
])
def test_winograd_joined_splits(lib, dev, oracle, variant, W, H, I, O):
    """Variant bit 0x800: the splits of a panel add their partial tiles up inside the one launch.  Same sums in the
    same order as the two-kernel form, so the results must be bit-identical to it; the workspace must be left
    holding the marker again; several launches in a row; the pooling epilogue."""
    chunks = -(-I // 8)
    per_split = -(-chunks // min(1 << ((variant >> 4) & 0xf), chunks))
    splits = -(-chunks // per_split)                      # what the launcher makes of the request: no empty split
    x, w, b = rnd(I, H, W), rnd(I, O, 3, 3, scale=np.sqrt(2.0 / (9 * I))), rnd(O, scale=0.01)
    U, _ = wino_filters(lib, dev, w)
    xd, bd = dev.put(x), dev.put(b)
    out = dev.empty(O * H * W)
    n = lib.drhip_conv3x3_winograd_workspace_floats(W, H, I, O, variant)
    nt, two_sets = variant & 0xf, bool(variant & 0x400)
    groups = -(-(-(-W // 2) * -(-H // 2)) // 32) * -(-O // (32 * nt)) * splits
    resident = groups <= 256 * (1 if two_sets else {1: 3, 2: 2}[nt])     # MI355X: 256 CUs
    if splits * per_split != chunks or splits & (splits - 1) or not resident:     # unequal splits, or more workgroups than fit at once: refused
        assert n > 0
        assert lib.drhip_conv3x3_winograd_f32(xd, U, bd, out, W, H, I, O, 1, variant, dev.empty(n), None) == -1
        return
    ws = wino_workspace(lib, dev, W, H, I, O, variant)
    plain = variant & ~0x800
    ws2 = wino_workspace(lib, dev, W, H, I, O, plain)
    ref = dev.empty(O * H * W)
    ok(lib, lib.drhip_conv3x3_winograd_f32(xd, U, bd, ref, W, H, I, O, 1, plain, ws2, None))
    want = dev.get(ref, (O, H, W))
    assert_close(want, oracle.conv_winograd(x, w, b, relu=True), floor=float(np.abs(b).max()))
    for _ in range(3):
        ok(lib, lib.drhip_fill_f32(out, 7.0, O * H * W, None))
        ok(lib, lib.drhip_conv3x3_winograd_f32(xd, U, bd, out, W, H, I, O, 1, variant, ws, None))
        assert np.array_equal(dev.get(out, want.shape), want)
        assert np.all(dev.get(ws, (n,)).view(np.uint32) == 0xffa5c3e1)
    if W % 2 == 0 and H % 2 == 0:
        ok(lib, lib.drhip_conv3x3_winograd_f32(xd, U, bd, ref, W, H, I, O, 2, plain, ws2, None))
        ok(lib, lib.drhip_conv3x3_winograd_f32(xd, U, bd, out, W, H, I, O, 2, variant, ws, None))
        assert np.array_equal(dev.get(out, (O, H // 2, W // 2)), dev.get(ref, (O, H // 2, W // 2)))
    late = ctypes.c_uint(123)
    ok(lib, lib.drhip_conv3x3_winograd_join_timeouts(ctypes.byref(late)))
    assert late.value == 0


def test_winograd_joined_refused_when_not_resident(lib, dev):
    """A joined split needs every workgroup of the launch resident at once; a layer with more panels is refused."""
    p = dev.empty(64)
    n = lib.drhip_conv3x3_winograd_workspace_floats(224, 224, 16, 64, 0x811)
    assert n > 0
    assert lib.drhip_conv3x3_winograd_f32(p, p, None, p, 224, 224, 16, 64, 0, 0x811, p, None) == -1
    assert b"resident" in lib.drhip_last_error()
    assert lib.drhip_conv3x3_winograd_f32(p, p, None, p, 8, 8, 16, 16, 0, 0x801, p, None) == -1     # joined, but unsplit
    assert lib.drhip_conv3x3_winograd_f32(p, p, None, p, 8, 8, 16, 16, 0, 0x911, p, None) == -1     # 16-tile blocks


@pytest.mark.parametrize("variant", [0x1801, 0x1802])
@pytest.mark.parametrize("W,H,I,O", [
    (112, 112, 128, 128),    # 49 panels per XCD: one cut into 16, 16 halved, 32 whole
    (112, 112, 64, 128),     # 8 stages: the finest cut is 8
    (56, 56, 64, 64), (28, 20, 32, 40), (13, 9, 16, 33), (2, 2, 128, 3), (14, 14, 512, 512),
    (28, 28, 24, 40),        # 3 stages: nothing to halve, the launch stays unsplit
    (7, 9, 3, 5),
])
def test_winograd_tiered_splits(lib, dev, oracle, variant, W, H, I, O):
    """Variant bits 0x1800: the panels of an XCD go out in tiers of whole, halved, quartered ... panels whose pieces
    add their partial tiles up inside the launch.  Against the oracle; repeated launches bit-identical; the
    workspace left holding the marker; the pooling epilogue equal to the pooled unpooled output."""
    x, w, b = rnd(I, H, W), rnd(I, O, 3, 3, scale=np.sqrt(2.0 / (9 * I))), rnd(O, scale=0.01)
    U, _ = wino_filters(lib, dev, w)
    xd, bd = dev.put(x), dev.put(b)
    out = dev.empty(O * H * W)
    n = lib.drhip_conv3x3_winograd_workspace_floats(W, H, I, O, variant)
    chunks = -(-I // 8)
    assert (n > 0) == (chunks % 2 == 0)
    ws = wino_workspace(lib, dev, W, H, I, O, variant)
    want = oracle.conv_winograd(x, w, b, relu=True)
    first = None
    for _ in range(3):
        ok(lib, lib.drhip_fill_f32(out, 7.0, O * H * W, None))
        ok(lib, lib.drhip_conv3x3_winograd_f32(xd, U, bd, out, W, H, I, O, 1, variant, ws, None))
        got = dev.get(out, want.shape)
        assert_close(got, want, floor=float(np.abs(b).max()))
        first = got if first is None else first
        assert np.array_equal(got, first)
        if n:
            assert np.all(dev.get(ws, (n,)).view(np.uint32) == 0xffa5c3e1)
    assert_close(first, oracle.conv_f64(x, w, b, relu=True), floor=float(np.abs(b).max()))
    if W % 2 == 0 and H % 2 == 0:
        pooled = dev.empty(O * H * W // 4)
        ok(lib, lib.drhip_conv3x3_winograd_f32(xd, U, bd, pooled, W, H, I, O, 1 | 2, variant, ws, None))
        assert np.array_equal(dev.get(pooled, (O, H // 2, W // 2)), oracle.pool(first, (2, 2, 1), (2, 2, 1), 0))
    late = ctypes.c_uint(123)
    ok(lib, lib.drhip_conv3x3_winograd_join_timeouts(ctypes.byref(late)))
    assert late.value == 0
    if n:       # the pieces wait for each other through the workspace: none offered, refused
        assert lib.drhip_conv3x3_winograd_f32(xd, U, bd, out, W, H, I, O, 1, variant, None, None) == -1


def test_winograd_tiered_refused_combinations(lib, dev):
    p = dev.empty(64)
    for variant in (0x1001, 0x1901, 0x1c01, 0x1811, 0x1803, 0x2801):     # not joined, 16-tile blocks, two wave sets, split bits, 128 channels, unknown bit
        assert lib.drhip_conv3x3_winograd_workspace_floats(8, 8, 16, 16, variant) == 0
        assert lib.drhip_conv3x3_winograd_f32(p, p, None, p, 8, 8, 16, 16, 0, variant, p, None) == -1, hex(variant)


def test_winograd_auto_variant_vgg_shapes(lib, dev, oracle):
    assert lib.drhip_conv3x3_winograd_pick_variant(112, 112, 128, 128) == 0x1801      # (MI355X: 32 CUs per XCD)
    assert lib.drhip_conv3x3_winograd_pick_variant(14, 14, 512, 512) == 0x831
    assert lib.drhip_conv3x3_winograd_pick_variant(224, 224, 3, 64) == 1           # an image layer: 32-channel blocks
    assert lib.drhip_conv3x3_winograd_pick_variant(224, 224, 64, 64) == 2
    for (W, I, O) in [(224, 3, 64), (224, 64, 64), (112, 128, 128), (56, 128, 256), (28, 256, 512), (14, 512, 512)]:
        x, w, b = np.abs(rnd(I, W, W)), rnd(I, O, 3, 3, scale=np.sqrt(2.0 / (9 * I))), rnd(O, scale=0.01)
        U, _ = wino_filters(lib, dev, w)
        variant = lib.drhip_conv3x3_winograd_pick_variant(W, W, I, O)
        ws = wino_workspace(lib, dev, W, W, I, O, variant)
        want = oracle.conv_winograd(x, w, b, relu=True)
        out = dev.empty(want.size)
        ok(lib, lib.drhip_conv3x3_winograd_f32(dev.put(x), U, dev.put(b), out, W, W, I, O, 1, variant, ws, None))
        assert_close(dev.get(out, want.shape), want)
        # variant 0 without a workspace falls back to an unsplit configuration
        ok(lib, lib.drhip_conv3x3_winograd_f32(dev.put(x), U, dev.put(b), out, W, W, I, O, 1, 0, None, None))
        assert_close(dev.get(out, want.shape), want)
        dev.close()


def test_winograd_rejects_bad_arguments(lib, dev):
    p = dev.empty(64)
    assert lib.drhip_conv3x3_winograd_f32(p, p, None, p, 0, 4, 1, 1, 0, 0, None, None) == -1
    assert lib.drhip_conv3x3_winograd_f32(p, p, None, p, 4, 4, 1, 1, 0, 9, None, None) == -1
    assert lib.drhip_conv3x3_winograd_f32(p, p, None, p, 4, 4, 1, 1, 0, 4, None, None) == -1      # panel codes are 1..3
    assert lib.drhip_conv3x3_winograd_f32(None, p, None, p, 4, 4, 1, 1, 0, 0, None, None) == -1
    assert lib.drhip_conv3x3_winograd_f32(p, p, None, p, 4, 4, 32, 1, 0, 0x11, None, None) == -1    # split without workspace
    assert b"workspace" in lib.drhip_last_error()


@pytest.mark.parametrize("variant", [0, 1, 2, 4, 8, 0x101, 0x102, 0x108, 0x110])
@pytest.mark.parametrize("P,I,O", [(3025, 128, 16), (3025, 16, 64), (196, 512, 1000), (196, 512, 64), (784, 256, 32), (50, 7, 5), (1, 1, 1), (33, 9, 65), (70, 24, 40)])
def test_conv1x1(lib, dev, oracle, variant, P, I, O):
    x, w, b = np.abs(rnd(I, 1, P)), rnd(I, O, 1, 1, scale=np.sqrt(2.0 / I)), rnd(O, scale=0.01)
    want = oracle.conv1x1(x, w, b, relu=True)
    out = dev.empty(want.size)
    ok(lib, lib.drhip_conv1x1_f32(dev.put(x), dev.put(w), dev.put(b), out, P, I, O, 1, variant, None))
    assert_close(dev.get(out, want.shape), want)
    want2 = oracle.conv1x1(x, w, None, relu=False)
    ok(lib, lib.drhip_conv1x1_f32(dev.put(x), dev.put(w), None, out, P, I, O, 0, variant, None))
    assert_close(dev.get(out, want2.shape), want2)


@pytest.mark.parametrize("W,H,C,k,s", [(56, 56, 256, 2, 2), (112, 112, 64, 3, 2), (55, 55, 7, 3, 2), (14, 14, 1000, 14, 14), (9, 7, 3, 2, 3), (5, 5, 2, 5, 1),
                                         (13, 13, 5, 8, 8), (20, 17, 3, 9, 4), (30, 30, 2, 16, 16)])   # >= 64 samples: one wavefront per output
def test_pool_bit_exact(lib, dev, oracle, W, H, C, k, s):
    x = rnd(C, H, W)                     # signed values: the zero padding is observable
    x[:, ::3, ::2] = x[0, 0, 0]          # ties: the first maximum in scan order must win
    for kind in (0, 1):
        want, warg = oracle.pool(x, (k, k, 1), (s, s, 1), kind, want_argmax=True) if kind == 0 else (oracle.pool(x, (k, k, 1), (s, s, 1), kind), None)
        out = dev.empty(want.size)
        arg = dev.empty(want.size, np.int32) if kind == 0 else None
        ok(lib, lib.drhip_pool_f32(dev.put(x), out, arg, W, H, C, k, k, 1, s, s, 1, kind, None))
        got = dev.get(out, want.shape)
        if kind == 0:
            assert np.array_equal(got, want)                                   # values bit-exact
            assert np.array_equal(dev.get(arg, want.shape, np.int32), warg)    # max-indices bit-exact
        else:
            assert rel_err(got, want) <= 1e-6


def test_pool_depth_window(lib, dev, oracle):
    x = rnd(6, 5, 4)
    want = oracle.pool(x, (2, 2, 2), (2, 2, 2), 0)
    out = dev.empty(want.size)
    ok(lib, lib.drhip_pool_f32(dev.put(x), out, None, 4, 5, 6, 2, 2, 2, 2, 2, 2, 0, None))
    assert np.array_equal(dev.get(out, want.shape), want)


@pytest.mark.parametrize("C,H,W,N,relu", [(512, 7, 7, 4096, 1), (4096, 1, 1, 1000, 0), (16, 3, 5, 10, 1), (3, 2, 2, 7, 0), (64, 1, 1, 130, 1), (1, 1, 1, 1, 0)])
def test_fc(lib, dev, oracle, C, H, W, N, relu):
    K = C * H * W
    x, Wt, b = np.abs(rnd(C, H, W)), rnd(K, N, scale=np.sqrt(2.0 / K)), rnd(N, scale=0.01)
    want = oracle.fc(x, Wt, b, relu=bool(relu)).reshape(-1)
    truth = oracle.fc_f64(x, Wt, b, relu=bool(relu)).reshape(-1)
    raw, perm = dev.put(Wt), dev.empty(K * N)
    ok(lib, lib.drhip_fc_permute_rows_f32(raw, perm, W, H, C, N, None))
    nparts = lib.drhip_fc_scratch_floats(K, N)
    parts = dev.empty(nparts) if nparts else None
    y = dev.empty(N)
    xd, bd = dev.put(x), dev.put(b)
    first = None
    for _ in range(2):                     # the scratch needs no reset between calls
        ok(lib, lib.drhip_fc_f32(xd, perm, bd, y, parts, K, N, relu, None))
        got = dev.get(y, (N,))
        assert_close(got, want, terms=K)
        assert_close(got, truth, terms=K)
        assert first is None or np.array_equal(first, got)      # fixed summation order
        first = got


@pytest.mark.parametrize("Win,Hin,I,O", [(56, 56, 128, 32), (28, 28, 256, 48), (55, 27, 20, 7), (9, 6, 3, 17), (2, 2, 1, 1), (1, 1, 5, 3)])
def test_conv1x1_with_pooled_input(lib, dev, oracle, Win, Hin, I, O):
    """3x3/2 max pooling taken while the 1x1 layer loads its input: the same values as the pooling kernel
    followed by the 1x1 GEMM (to rounding: the channel sum may be dealt to a different number of waves),
    and the oracle's pool -> conv1x1 within the layer bar.
    Signed inputs: windows hanging over the border must see 0.0, not -inf and not the edge sample."""
    x, w, b = rnd(I, Hin, Win), rnd(I, O, 1, 1, scale=np.sqrt(2.0 / I)), rnd(O, scale=0.01)
    Wp, Hp = -(-Win // 2), -(-Hin // 2)
    pooled = oracle.pool(x, (3, 3, 1), (2, 2, 1), 0)
    assert pooled.shape == (I, Hp, Wp)
    xd, wd, bd = dev.put(x), dev.put(w), dev.put(b)
    for relu in (1, 0):
        want = oracle.conv1x1(pooled, w, b, relu=bool(relu))
        out = dev.empty(want.size)
        ok(lib, lib.drhip_conv1x1_pooled3s2_f32(xd, wd, bd, out, Win, Hin, I, O, relu, None))
        got = dev.get(out, want.shape)
        assert_close(got, want, "pooled-input 1x1 %dx%dx%d->%d" % (Win, Hin, I, O))
        # against the two kernels it replaces
        mid, two = dev.empty(pooled.size), dev.empty(want.size)
        ok(lib, lib.drhip_pool_f32(xd, mid, None, Win, Hin, I, 3, 3, 1, 2, 2, 1, 0, None))
        assert np.array_equal(dev.get(mid, pooled.shape), pooled)
        ok(lib, lib.drhip_conv1x1_f32(mid, wd, bd, two, Wp * Hp, I, O, relu, 0, None))
        assert_close(got, dev.get(two, want.shape), "pooled-input 1x1 vs pool + 1x1 kernels")
    assert lib.drhip_conv1x1_pooled3s2_f32(xd, wd, bd, None, Win, Hin, I, O, 0, None) == -1


class DeferredVec(ctypes.Structure):
    """drhip_deferred_vec (include/dr_hip.h)."""
    _fields_ = [("partials", ctypes.c_void_p), ("bias", ctypes.c_void_p), ("slices", ctypes.c_int), ("n", ctypes.c_int), ("relu", ctypes.c_int), ("finished", ctypes.c_void_p),
                ("divisor", ctypes.c_float)]


@pytest.mark.parametrize("N2", [1000, 2500])        # softmax with the vector in registers / re-read from memory
def test_fc_chain_without_finishing_kernels(lib, dev, oracle, N2):
    """FC -> FC -> softmax where each consumer sums the producer's split-K partials itself: every
    result equals the one of the three separate calls bit for bit."""
    K, N1 = 1024, 2048
    x, W1, b1 = np.abs(rnd(K)), rnd(K, N1, scale=np.sqrt(2.0 / K)), rnd(N1, scale=0.01)
    W2, b2 = rnd(N1, N2, scale=np.sqrt(2.0 / N1)), rnd(N2, scale=0.01)
    xd, W1d, b1d, W2d, b2d = dev.put(x), dev.put(W1), dev.put(b1), dev.put(W2), dev.put(b2)
    s1, s2 = lib.drhip_fc_slices(K, N1), lib.drhip_fc_slices(N1, N2)
    assert s1 > 1 and s2 > 1 and lib.drhip_fc_scratch_floats(K, N1) == s1 * N1
    p1, p2 = dev.empty(s1 * N1), dev.empty(s2 * N2)
    y1, y2, prob = dev.empty(N1), dev.empty(N2), dev.empty(N2)
    # plain chain
    ok(lib, lib.drhip_fc_f32(xd, W1d, b1d, y1, p1, K, N1, 1, None))
    ok(lib, lib.drhip_fc_f32(y1, W2d, b2d, y2, p2, N1, N2, 0, None))
    ok(lib, lib.drhip_softmax_f32(y2, prob, N2, None))
    want1, want2, wantp = dev.get(y1, (N1,)), dev.get(y2, (N2,)), dev.get(prob, (N2,))
    assert_close(want2, oracle.fc(oracle.fc(x.reshape(K, 1, 1), W1, b1, relu=True), W2, b2, relu=False).reshape(-1))
    # deferred chain: y1 and y2 are never written
    q1, q2, prob2 = dev.empty(s1 * N1), dev.empty(s2 * N2), dev.empty(N2)
    ok(lib, lib.drhip_fc_ex_f32(xd, None, W1d, b1d, None, q1, K, N1, 1, 1, None))
    d1 = DeferredVec(q1.value, b1d.value, s1, N1, 1, None)
    y2b = dev.empty(N2)
    ok(lib, lib.drhip_fc_ex_f32(None, ctypes.byref(d1), W2d, b2d, y2b, q2, N1, N2, 0, 0, None))
    assert np.array_equal(dev.get(y2b, (N2,)), want2)
    ok(lib, lib.drhip_fc_ex_f32(None, ctypes.byref(d1), W2d, b2d, None, q2, N1, N2, 0, 1, None))
    d2 = DeferredVec(q2.value, b2d.value, s2, N2, 0, None)
    ok(lib, lib.drhip_softmax_ex_f32(None, ctypes.byref(d2), prob2, N2, None))
    assert np.array_equal(dev.get(prob2, (N2,)), wantp)
    # ... and with the consumers also storing the finished vectors (producers whose output is wanted too)
    fin1, fin2 = dev.put(np.full(N1, -7.0, np.float32)), dev.put(np.full(N2, -7.0, np.float32))
    d1f = DeferredVec(q1.value, b1d.value, s1, N1, 1, fin1.value)
    ok(lib, lib.drhip_fc_ex_f32(None, ctypes.byref(d1f), W2d, b2d, None, q2, N1, N2, 0, 1, None))
    assert np.array_equal(dev.get(fin1, (N1,)), want1)
    d2f = DeferredVec(q2.value, b2d.value, s2, N2, 0, fin2.value)
    ok(lib, lib.drhip_softmax_ex_f32(None, ctypes.byref(d2f), prob2, N2, None))
    assert np.array_equal(dev.get(prob2, (N2,)), wantp) and np.array_equal(dev.get(fin2, (N2,)), want2)
    d2bad = DeferredVec(q2.value, b2d.value, s2, N2, 0, prob2.value)
    assert lib.drhip_softmax_ex_f32(None, ctypes.byref(d2bad), prob2, N2, None) == -1
    # argument checks
    bad = DeferredVec(q1.value, b1d.value, s1, N1 + 1, 1, None)
    assert lib.drhip_fc_ex_f32(None, ctypes.byref(bad), W2d, b2d, y2b, q2, N1, N2, 0, 0, None) == -1
    assert lib.drhip_fc_ex_f32(xd, None, W1d, b1d, None, None, 64, 8, 0, 1, None) == -1        # unsplit layers cannot defer


@pytest.mark.parametrize("P,I,O,relu", [(196, 512, 1000, 1), (196, 64, 40, 0), (33, 9, 65, 1), (1, 1, 1, 0), (70, 24, 31, 1)])
def test_conv1x1_with_global_average(lib, dev, oracle, P, I, O, relu):
    """1x1 convolution whose epilogue leaves per-tile pixel sums; the softmax in front of which the
    pooled vector is needed adds the tiles and divides (drhip_deferred_vec.divisor)."""
    x, w, b = rnd(I, 1, P), rnd(I, O, 1, 1, scale=np.sqrt(2.0 / I)), rnd(O, scale=0.05)
    conv = oracle.conv1x1(x, w, b, relu=bool(relu))                      # [O, 1, P]
    pooled = oracle.pool(conv, (P, 1, 1), (P, 1, 1), 1).reshape(-1)       # global average
    slices = lib.drhip_conv1x1_poolsum_slices(P)
    assert slices == (P + 31) // 32
    parts = dev.empty(slices * O)
    ok(lib, lib.drhip_conv1x1_poolsum_f32(dev.put(x), dev.put(w), dev.put(b), parts, P, I, O, relu, None))
    got = dev.get(parts, (slices, O)).astype(np.float64).sum(axis=0) / P
    assert_close(got, pooled)
    fin, prob = dev.empty(O), dev.empty(O)
    d = DeferredVec(parts.value, None, slices, O, 0, fin.value, float(P))
    ok(lib, lib.drhip_softmax_ex_f32(None, ctypes.byref(d), prob, O, None))
    assert_close(dev.get(fin, (O,)), pooled)
    assert_close(dev.get(prob, (O,)), oracle.softmax(pooled))


@pytest.mark.parametrize("C,H,W", [(3, 224, 224), (1, 5, 7), (4, 17, 33), (64, 56, 56), (1, 1, 2)])
def test_normalize(lib, dev, oracle, C, H, W):
    x = (np.random.default_rng(C + H).random((C, H, W), dtype=np.float32) * 255.0).astype(np.float32)
    n = x.size
    scratch = dev.empty(lib.drhip_normalize_scratch_floats(n))
    xd, y = dev.put(x), dev.empty(n)
    for kind, tm, td in [(0, 3.0, 1.0), (1, 0.0, 2.0), (2, 0.0, 1.0), (2, 0.5, 1.5)]:
        first = None
        for _ in range(2):                   # the scratch needs no reset between calls; fixed summation order
            ok(lib, lib.drhip_normalize_f32(xd, y, n, kind, tm, td, scratch, None))
            got = dev.get(y, x.shape)
            assert first is None or np.array_equal(first, got)
            first = got
        assert_close(got, oracle.normalize(x, kind, tm, td))
        assert_close(got, oracle.normalize_f64(x, kind, tm, td))
    assert lib.drhip_normalize_f32(xd, y, n, 3, 0.0, 1.0, scratch, None) == -1
    assert lib.drhip_normalize_f32(xd, y, 0, 2, 0.0, 1.0, scratch, None) == -1


def test_softmax(lib, dev, oracle):
    for n, scale in [(1000, 3.0), (10, 1.0), (5000, 5.0), (1, 1.0), (2048, 2.0), (2049, 2.0), (257, 1.0)]:
        x = rnd(n, scale=scale)
        y = dev.empty(n)
        ok(lib, lib.drhip_softmax_f32(dev.put(x), y, n, None))
        got = dev.get(y, (n,))
        assert_close(got, oracle.softmax(x))
        assert_close(got, oracle.softmax_f64(x))
        assert abs(float(got.sum()) - 1) < 1e-5 and int(got.argmax()) == int(x.argmax())
    # logits that overflow exp() unshifted still give a distribution here
    big = np.array([100.0, 101.0, 99.0], np.float32)
    y = dev.empty(3)
    ok(lib, lib.drhip_softmax_f32(dev.put(big), y, 3, None))
    assert_close(dev.get(y, (3,)), oracle.softmax_f64(big))


@pytest.mark.parametrize("env", [{}, {"DR_SPIN_US": "0"}, {"DR_UPLOAD_KERNEL": "0"}])
def test_staged_transfers_carry_every_byte(lib, dev, env):
    """Uploads through the pinned area (by kernel and by the DMA engine: odd destination offsets and sizes
    take the latter) and downloads through the flagged copy kernel, many times over with new contents and
    sizes each time: a flag seen before its data, or data left in the area from the call before, would show."""
    import os
    os.environ.update(env)
    try:
        h = ctypes.c_void_p()
        ok(lib, lib.drhip_staging_create(ctypes.byref(h), 1 << 20))
    finally:
        for k in env:
            os.environ.pop(k, None)
    assert lib.drhip_staging_upload_capacity(h) == 1 << 20 and lib.drhip_staging_download_capacity(h) == 65536
    rng = np.random.default_rng(11)
    buf = dev.empty(1 << 18)
    vp = ctypes.c_void_p
    try:
        for it in range(300):
            n = int(rng.choice([1, 3, 4, 250, 1000, 4096, 16383, 16384, 75001, 131072]))     # (from 256 KiB on an upload goes in two pieces)
            off = int(rng.integers(0, 64)) * int(rng.choice([1, 4]))          # floats; some 16-byte aligned, some not
            a = rng.standard_normal(n).astype(np.float32) + it
            ok(lib, lib.drhip_upload_staged(h, buf, 4 * off, a.ctypes.data_as(vp), a.nbytes, None))
            a_copy = a.copy()
            a[...] = np.nan                                                    # the caller's array is free again
            if a.nbytes <= 65536:
                back = np.full(n, -1.0, np.float32)
                ok(lib, lib.drhip_download_staged(h, back.ctypes.data_as(vp), buf, 4 * off, back.nbytes, None))
            else:                                                              # (beyond the download area: the plain blocking copy)
                back = dev.get(buf, (off + n,))[off:]
            assert np.array_equal(back, a_copy), (it, n, off)
        # many uploads in a row with no download in between (the two pinned areas are reused while earlier uploads
        # may still be in flight), the caller's array overwritten after every call
        n, rows = 4096, 24
        src = np.empty(n, np.float32)
        want = np.empty((rows, n), np.float32)
        for k in range(rows):
            src[...] = rng.standard_normal(n).astype(np.float32) + 100 * k
            want[k] = src
            ok(lib, lib.drhip_upload_staged(h, buf, 4 * k * n, src.ctypes.data_as(vp), src.nbytes, None))
            src[...] = np.nan
        for k in range(rows):
            back = np.full(n, -1.0, np.float32)
            ok(lib, lib.drhip_download_staged(h, back.ctypes.data_as(vp), buf, 4 * k * n, back.nbytes, None))
            assert np.array_equal(back, want[k]), k
        # bytes that are not whole floats go through the DMA engine both ways
        raw = rng.integers(0, 256, 1001, dtype=np.uint8)
        ok(lib, lib.drhip_upload_staged(h, buf, 3, raw.ctypes.data_as(vp), raw.nbytes, None))
        got = np.zeros_like(raw)
        ok(lib, lib.drhip_download_staged(h, got.ctypes.data_as(vp), buf, 3, got.nbytes, None))
        assert np.array_equal(got, raw)
        assert lib.drhip_download_staged(h, got.ctypes.data_as(vp), buf, 0, 65537, None) == -1
        assert lib.drhip_upload_staged(h, buf, 0, raw.ctypes.data_as(vp), (1 << 20) + 1, None) == -1
    finally:
        lib.drhip_staging_destroy(h)


def test_copy3d_and_scalar(lib, dev, oracle):
    x = rnd(6, 9, 11)
    out = dev.empty(3 * 4 * 5)
    ok(lib, lib.drhip_copy3d_f32(dev.put(x), 11, 9, 2, 3, 1, out, 5, 4, 0, 0, 0, 5, 4, 3, None))
    assert np.array_equal(dev.get(out, (3, 4, 5)), x[1:4, 3:7, 2:7])
    assert lib.drhip_copy3d_f32(dev.put(x), 11, 9, 8, 0, 0, out, 5, 4, 0, 0, 0, 5, 4, 3, None) == -1   # box leaves the source
    for op, s in [(0, 1.5), (1, 123.68), (2, 0.5), (3, 4.0), (7, 2.0)]:
        y = dev.empty(x.size)
        ok(lib, lib.drhip_scalar_op_f32(dev.put(x), y, x.size, op, s, None))
        assert np.array_equal(dev.get(y, x.shape), oracle.scalar_op(x, op, s))


# ---------------------------------------------------------------------------------------------
# Seeded sweeps over ragged shapes: sizes that are no multiple of any tile, panel, stage or vector
# width the kernels use, single rows / columns / channels included.

def _sweep(seed, count, draw):
    """`count` seeded draws; DR_SWEEP_SCALE=n in the environment multiplies the count for a one-off wider run."""
    rng = np.random.default_rng(seed)
    return [draw(rng) for _ in range(count * int(os.environ.get("DR_SWEEP_SCALE", "1")))]


@pytest.mark.parametrize("W,H,I,O,variant", _sweep(11, 40, lambda r: (
    int(r.integers(1, 41)), int(r.integers(1, 41)), int(r.integers(1, 41)), int(r.integers(1, 71)),
    int(r.choice([0, 1, 2, 3, 0x11, 0x12, 0x21, 0x31, 0x101, 0x102, 0x103, 0x111, 0x121,
                  0x401, 0x402, 0x411, 0x422, 0x501, 0x502, 0x503, 0x511, 0x521]))))
    + [(1, 37, 9, 31, 0x11), (37, 1, 8, 32, 1), (3, 3, 64, 33, 0x21), (40, 2, 17, 1, 2)])
def test_winograd_sweep(lib, dev, oracle, W, H, I, O, variant):
    x, w, b = rnd(I, H, W), rnd(I, O, 3, 3, scale=np.sqrt(2.0 / (9 * I))), rnd(O, scale=0.01)
    U, _ = wino_filters(lib, dev, w)
    ws = wino_workspace(lib, dev, W, H, I, O, variant)
    relu = (W + H + I + O) & 1
    want = oracle.conv_winograd(x, w, b, relu=bool(relu))
    out = dev.empty(want.size)
    ok(lib, lib.drhip_conv3x3_winograd_f32(dev.put(x), U, dev.put(b), out, W, H, I, O, relu, variant, ws, None))
    got = dev.get(out, want.shape)
    assert_close(got, want)
    assert_close(got, oracle.conv_f64(x, w, b, relu=bool(relu)))


@pytest.mark.parametrize("W,H,I,O,kw,kh,sx,sy", _sweep(12, 20, lambda r: (
    int(r.integers(1, 40)), int(r.integers(1, 40)), int(r.integers(1, 20)), int(r.integers(1, 40)),
    int(r.choice([1, 3, 5, 7])), int(r.choice([1, 3, 5])), int(r.integers(1, 4)), int(r.integers(1, 4)))))
def test_conv_direct_sweep(lib, dev, oracle, W, H, I, O, kw, kh, sx, sy):
    if W // sx == 0 or H // sy == 0:
        pytest.skip("empty output")
    x, w, b = rnd(I, H, W), rnd(I, O, kh, kw, scale=np.sqrt(2.0 / (kh * kw * I))), rnd(O, scale=0.01)
    want = oracle.conv_direct(x, w, b, (sx, sy), relu=False)
    out = dev.empty(want.size)
    ok(lib, lib.drhip_conv2d_direct_f32(dev.put(x), dev.put(w), dev.put(b), out, W, H, I, O, kw, kh, sx, sy, 0, None))
    got = dev.get(out, want.shape)
    assert_close(got, want)
    assert_close(got, oracle.conv_f64(x, w, b, stride=(sx, sy)))


@pytest.mark.parametrize("W,H,I,O,s,variant", _sweep(16, 32, lambda r: (
    int(r.integers(1, 41)), int(r.integers(1, 41)), int(r.integers(1, 41)), int(r.integers(1, 71)), int(r.integers(1, 3)),
    int(r.choice([0, 1, 2, 4, 8, 0x11, 0x12, 0x14, 0x18]))))
    + [(1, 40, 9, 31, 1, 0x12), (40, 1, 8, 33, 2, 4), (3, 3, 64, 65, 1, 8), (2, 2, 7, 1, 2, 0x11)])
def test_conv3x3_direct_mfma_sweep(lib, dev, oracle, W, H, I, O, s, variant):
    if W // s == 0 or H // s == 0:
        pytest.skip("empty output")
    x, w, b = rnd(I, H, W), rnd(I, O, 3, 3, scale=np.sqrt(2.0 / (9 * I))), rnd(O, scale=0.01)
    F = dev.empty(lib.drhip_conv3x3_direct_filter_floats(I, O))
    ok(lib, lib.drhip_conv3x3_direct_filter_layout_f32(dev.put(w), F, I, O, None))
    relu = (W + H + I + O) & 1
    want = oracle.conv_direct(x, w, b, (s, s), relu=bool(relu))
    out = dev.empty(want.size)
    ok(lib, lib.drhip_conv3x3_direct_mfma_f32(dev.put(x), F, dev.put(b), out, W, H, I, O, s, relu, variant, None))
    got = dev.get(out, want.shape)
    assert_close(got, want, terms=9 * I)
    assert_close(got, oracle.conv_f64(x, w, b, stride=(s, s), relu=bool(relu)), terms=9 * I)


@pytest.mark.parametrize("Win,Hin,I,O", _sweep(17, 20, lambda r: (
    int(r.integers(1, 60)), int(r.integers(1, 60)), int(r.integers(1, 140)), int(r.integers(1, 70)))))
def test_conv1x1_with_pooled_input_sweep(lib, dev, oracle, Win, Hin, I, O):
    x, w, b = rnd(I, Hin, Win), rnd(I, O, 1, 1, scale=np.sqrt(2.0 / I)), rnd(O, scale=0.01)
    pooled = oracle.pool(x, (3, 3, 1), (2, 2, 1), 0)
    relu = (Win + Hin + I + O) & 1
    want = oracle.conv1x1(pooled, w, b, relu=bool(relu))
    out = dev.empty(want.size)
    ok(lib, lib.drhip_conv1x1_pooled3s2_f32(dev.put(x), dev.put(w), dev.put(b), out, Win, Hin, I, O, relu, None))
    assert_close(dev.get(out, want.shape), want, terms=I)


@pytest.mark.parametrize("P,I,O,variant", _sweep(13, 20, lambda r: (
    int(r.integers(1, 400)), int(r.integers(1, 100)), int(r.integers(1, 100)), int(r.choice([0, 1, 2, 4, 8, 0x101, 0x104, 0x110])))))
def test_conv1x1_sweep(lib, dev, oracle, P, I, O, variant):
    x, w, b = rnd(I, 1, P), rnd(I, O, 1, 1, scale=np.sqrt(2.0 / I)), rnd(O, scale=0.01)
    want = oracle.conv1x1(x, w, b, relu=False)
    out = dev.empty(want.size)
    ok(lib, lib.drhip_conv1x1_f32(dev.put(x), dev.put(w), dev.put(b), out, P, I, O, 0, variant, None))
    assert_close(dev.get(out, want.shape), want)


@pytest.mark.parametrize("W,H,C,kx,ky,kz,sx,sy,sz", _sweep(14, 24, lambda r: (
    int(r.integers(1, 30)), int(r.integers(1, 30)), int(r.integers(1, 9)),
    int(r.integers(1, 12)), int(r.integers(1, 12)), int(r.integers(1, 3)),
    int(r.integers(1, 6)), int(r.integers(1, 6)), int(r.integers(1, 3)))))
def test_pool_sweep(lib, dev, oracle, W, H, C, kx, ky, kz, sx, sy, sz):
    x = rnd(C, H, W)
    x[:, ::2, ::3] = x.flat[0]
    for kind in (0, 1):
        want = oracle.pool(x, (kx, ky, kz), (sx, sy, sz), kind)
        out = dev.empty(want.size)
        ok(lib, lib.drhip_pool_f32(dev.put(x), out, None, W, H, C, kx, ky, kz, sx, sy, sz, kind, None))
        got = dev.get(out, want.shape)
        if kind == 0:
            assert np.array_equal(got, want)
        else:
            assert rel_err(got, want) <= 1e-6


@pytest.mark.parametrize("C,H,W,N", _sweep(15, 16, lambda r: (
    int(r.integers(1, 70)), int(r.integers(1, 6)), int(r.integers(1, 6)), int(r.integers(1, 600)))))
def test_fc_sweep(lib, dev, oracle, C, H, W, N):
    K = C * H * W
    x, Wt, b = rnd(C, H, W), rnd(K, N, scale=np.sqrt(2.0 / K)), rnd(N, scale=0.01)
    want = oracle.fc(x, Wt, b, relu=False).reshape(-1)
    perm = dev.empty(K * N)
    ok(lib, lib.drhip_fc_permute_rows_f32(dev.put(Wt), perm, W, H, C, N, None))
    n = lib.drhip_fc_scratch_floats(K, N)
    y = dev.empty(N)
    ok(lib, lib.drhip_fc_f32(dev.put(x), perm, dev.put(b), y, dev.empty(n) if n else None, K, N, 0, None))
    got = dev.get(y, (N,))
    assert_close(got, want, terms=K)
    assert_close(got, oracle.fc_f64(x, Wt, b).reshape(-1), terms=K)


def test_mfma_clock_probe(lib, gpu):
    """The measurement aid of bench.py: shader clock under a stream of fp32 MFMAs, from the two clock counters a wave
    can read.  Somewhere between idle clocks and the 2.4 GHz of the data sheet."""
    mhz, us = ctypes.c_float(0), ctypes.c_float(0)
    lib.drhip_mfma_clock_probe.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_float), ctypes.c_void_p]
    ok(lib, lib.drhip_mfma_clock_probe(100, 3, ctypes.byref(mhz), ctypes.byref(us), None))
    assert 500.0 < mhz.value < 2600.0 and us.value > 5.0, (mhz.value, us.value)
    assert lib.drhip_mfma_clock_probe(0, 1, ctypes.byref(mhz), None, None) == -1
