"""Per-element parity at the exact layer shapes of the five benchmark
configurations, with each configuration's own data distribution.

Every case is checked twice against the CPU oracle: real-valued inputs under the
per-element and normwise bounds of tests/tolerance.py (1e-4), and small-integer inputs bit for bit (fp32 sums of integers below
2^24 are exact, so any indexing mistake shows as a whole-number difference).
The whole-network tests only bound the final tensor normwise; these pin the
individual launches the networks are made of: tile grids, K lengths, XCD
banding and split-K shares differ from layer to layer.
"""
import numpy as np
import pytest
import torch

import oracle
from tolerance import REL_TOL, max_rel_err

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def ints(rng, shape, lo=-3, hi=4):
    return rng.integers(lo, hi, size=shape).astype(np.float32)


@pytest.fixture(scope="module")
def ops():
    from pet_amd import ops as _ops
    return _ops


def check_conv2d(ops, x, w, ph, pw, sh, sw, dh, dw, xi, wi):
    ref = oracle.conv2d(x, w, ph, pw, sh, sw, dh, dw)
    mag = oracle.conv2d(np.abs(x), np.abs(w), ph, pw, sh, sw, dh, dw)
    got = host(ops.conv2d(dev(x), dev(w), ph, pw, sh, sw, dh, dw))
    assert got.shape == ref.shape
    assert max_rel_err(got, ref, mag) <= REL_TOL
    refi = oracle.conv2d(xi, wi, ph, pw, sh, sw, dh, dw)
    goti = host(ops.conv2d(dev(xi), dev(wi), ph, pw, sh, sw, dh, dw))
    np.testing.assert_array_equal(goti, refi)


def test_c1_conv_64_to_64_on_56x56(ops):
    """Configuration 1: 1x64x56x56, 3x3, pad 1, inputs and weights uniform[-1, 1]."""
    rng = np.random.default_rng(0)
    x = rng.uniform(-1, 1, (1, 64, 56, 56)).astype(np.float32)
    w = rng.uniform(-1, 1, (64, 64, 3, 3)).astype(np.float32)
    check_conv2d(ops, x, w, 1, 1, 1, 1, 1, 1, ints(rng, x.shape), ints(rng, w.shape))


C2_LAYERS = [(512, 512), (512, 256), (256, 128), (128, 64)]


@pytest.mark.parametrize("cin,cout", C2_LAYERS)
@pytest.mark.parametrize("form", ["dilated", "space_to_batch"])
def test_c2_layer_both_forms(ops, cin, cout, form):
    """Configuration 2: each distinct layer as the original dilated convolution
    (1xCx64x64, dilation 2, pad 2) and as the dense convolution of the PET program
    (4xCx32x32, pad 1), activations N(0, 1), weights N(0, 0.01)."""
    rng = np.random.default_rng(cin * 7 + cout)
    w = (0.01 * rng.standard_normal((cout, cin, 3, 3))).astype(np.float32)
    wi = ints(rng, w.shape, -2, 3)
    if form == "dilated":
        x = rng.standard_normal((1, cin, 64, 64)).astype(np.float32)
        check_conv2d(ops, x, w, 2, 2, 1, 1, 2, 2, ints(rng, x.shape, -2, 3), wi)
    else:
        x = rng.standard_normal((4, cin, 32, 32)).astype(np.float32)
        check_conv2d(ops, x, w, 1, 1, 1, 1, 1, 1, ints(rng, x.shape, -2, 3), wi)


def _kaiming(rng, shape):
    return (rng.standard_normal(shape) * np.sqrt(2.0 / np.prod(shape[1:]))).astype(np.float32)


C3_LAYERS = [
    # name, c, hw, f, k, stride, pad
    ("stem 7x7/2", 3, 224, 64, 7, 2, 3),
    ("layer1 3x3", 64, 56, 64, 3, 1, 1),
    ("layer2 3x3/2", 64, 56, 128, 3, 2, 1),
    ("layer2 3x3", 128, 28, 128, 3, 1, 1),
    ("layer3 3x3/2", 128, 28, 256, 3, 2, 1),
    ("layer3 3x3", 256, 14, 256, 3, 1, 1),
    ("layer4 3x3/2", 256, 14, 512, 3, 2, 1),
    ("layer4 3x3", 512, 7, 512, 3, 1, 1),
    ("downsample 1x1/2 a", 64, 56, 128, 1, 2, 0),
    ("downsample 1x1/2 b", 128, 28, 256, 1, 2, 0),
    ("downsample 1x1/2 c", 256, 14, 512, 1, 2, 0),
]


@pytest.mark.parametrize("case", C3_LAYERS, ids=[c[0] for c in C3_LAYERS])
def test_c3_resnet18_layer(ops, case):
    """Configuration 3: every distinct convolution of ResNet-18 at batch 1, N(0, 1)
    activations, Kaiming-normal weights."""
    _, c, hw, f, k, st, pad = case
    rng = np.random.default_rng(c * 31 + hw + k)
    x = rng.standard_normal((1, c, hw, hw)).astype(np.float32)
    w = _kaiming(rng, (f, c, k, k))
    check_conv2d(ops, x, w, pad, pad, st, st, 1, 1, ints(rng, x.shape, -2, 3),
                 ints(rng, w.shape, -2, 3))


def test_c3_fc_512_to_1000(ops):
    rng = np.random.default_rng(5)
    a = rng.standard_normal((1, 1, 512)).astype(np.float32)
    b = (rng.standard_normal((1, 512, 1000)) / np.sqrt(512)).astype(np.float32)
    ref = oracle.matmul(a, b)
    mag = oracle.matmul(np.abs(a), np.abs(b))
    assert max_rel_err(host(ops.matmul(dev(a), dev(b))), ref, mag) <= REL_TOL
    ai, bi = ints(rng, a.shape), ints(rng, b.shape)
    np.testing.assert_array_equal(host(ops.matmul(dev(ai), dev(bi))), oracle.matmul(ai, bi))


C4_GEMMS = [
    # name, b, m, n, k, transB, std of B
    ("qkv merged b3", 3, 128, 768, 768, False, 0.02),
    ("projection", 1, 128, 768, 768, False, 0.02),
    ("scores b12", 12, 128, 128, 64, True, 1.0),
    ("probs x V b12", 12, 128, 64, 128, False, 1.0),
    ("ffn1", 1, 128, 3072, 768, False, 0.02),
    ("ffn2", 1, 128, 768, 3072, False, 0.02),
]


@pytest.mark.parametrize("case", C4_GEMMS, ids=[c[0] for c in C4_GEMMS])
def test_c4_bert_gemm(ops, case):
    """Configuration 4: the encoder's matmuls, activations N(0, 1), weights N(0, 0.02)."""
    _, b, m, n, k, tb, std = case
    rng = np.random.default_rng(b * 131 + n + k)
    a = rng.standard_normal((b, m, k)).astype(np.float32)
    bm = (std * rng.standard_normal((b, n, k) if tb else (b, k, n))).astype(np.float32)
    ref = oracle.matmul(a, bm, False, tb)
    mag = oracle.matmul(np.abs(a), np.abs(bm), False, tb)
    assert max_rel_err(host(ops.matmul(dev(a), dev(bm), False, tb)), ref, mag) <= REL_TOL
    ai, bi = ints(rng, a.shape, -2, 3), ints(rng, bm.shape, -2, 3)
    np.testing.assert_array_equal(host(ops.matmul(dev(ai), dev(bi), False, tb)),
                                  oracle.matmul(ai, bi, False, tb))


C5_LAYERS = [
    # name, c, t, hw, f, kernel, stride, pad  (clips shortened in time where the oracle
    # would take minutes; the spatial grid and channel counts are the network's)
    ("stem 3x7x7", 3, 4, 112, 64, (3, 7, 7), (1, 2, 2), (1, 3, 3)),
    ("layer1 3x3x3", 64, 4, 56, 64, (3, 3, 3), (1, 1, 1), (1, 1, 1)),
    ("layer2 3x3x3/2", 64, 4, 56, 128, (3, 3, 3), (2, 2, 2), (1, 1, 1)),
    ("layer3 3x3x3", 256, 4, 14, 256, (3, 3, 3), (1, 1, 1), (1, 1, 1)),
    ("layer4 3x3x3", 512, 2, 7, 512, (3, 3, 3), (1, 1, 1), (1, 1, 1)),
    ("downsample 1x1x1/2", 128, 8, 28, 256, (1, 1, 1), (2, 2, 2), (0, 0, 0)),
]


@pytest.mark.parametrize("packed", [False, True], ids=["filters as stored", "kt-major filters"])
@pytest.mark.parametrize("case", C5_LAYERS, ids=[c[0] for c in C5_LAYERS])
def test_c5_resnet3d_layer(ops, case, packed):
    """Configuration 5: Conv3d layers of ResNet3D-18 (no 3-D convolution upstream: the
    oracle is the 2-D loop nest with one more axis)."""
    _, c, t, hw, f, k, st, pad = case
    rng = np.random.default_rng(c * 17 + t + hw)
    x = rng.standard_normal((1, c, t, hw, hw)).astype(np.float32)
    w = _kaiming(rng, (f, c) + k)
    xi, wi = ints(rng, x.shape, -2, 3), ints(rng, w.shape, -2, 3)

    def run(xa, wa):
        dw = dev(wa)
        if packed:
            pk = ops.conv3d_pack_filters(dw)
            if pk is None:
                pytest.skip("this filter shape has no kt-major form")
            dw = pk
        return host(ops.conv3d(dev(xa), dw, pad, st))

    ref = oracle.conv3d(x, w, pad, st)
    mag = oracle.conv3d(np.abs(x), np.abs(w), pad, st)
    assert max_rel_err(run(x, w), ref, mag) <= REL_TOL
    np.testing.assert_array_equal(run(xi, wi), oracle.conv3d(xi, wi, pad, st))
