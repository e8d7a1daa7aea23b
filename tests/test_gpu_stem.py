"""The LDS-staged kernel for network stems (7x7 filters, stride 2, three input channels; one
time slice at a time in 3-D) against the CPU oracle: small integers bit for bit, real values
within the contraction tolerance of tests/tolerance.py. Shapes that leave its tiles ragged in
every direction, more and fewer filters than a workgroup's 64, every padding the 7x7 window
admits, batches, time strides."""
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


@pytest.fixture(scope="module")
def ops():
    from pet_amd import ops as _ops
    return _ops


STEMS_2D = [
    # n, h, w, f, pad
    (1, 224, 224, 64, 3),       # ResNet
    (1, 30, 30, 64, 3),
    (2, 37, 45, 16, 3),         # ragged tiles, fewer filters than a block, a batch
    (1, 19, 64, 100, 0),        # two filter blocks, the second ragged; no padding
    (3, 8, 9, 5, 3),            # smaller than one tile
    (1, 33, 35, 70, 1),
    (1, 64, 40, 64, 6),         # padding as wide as the window allows
]


@pytest.mark.parametrize("case", STEMS_2D)
def test_stem_2d(ops, case):
    n, h, w, f, pad = case
    rng = np.random.default_rng(sum(case))
    xi = rng.integers(-3, 4, (n, 3, h, w)).astype(np.float32)
    wi = rng.integers(-3, 4, (f, 3, 7, 7)).astype(np.float32)
    bi = rng.integers(-3, 4, (f,)).astype(np.float32)
    want = oracle.bias_act(oracle.conv2d(xi, wi, pad, pad, 2, 2), bi, "relu")
    got = host(ops.conv2d(dev(xi), dev(wi), pad, pad, 2, 2, bias=dev(bi), act="relu"))
    assert got.shape == want.shape
    np.testing.assert_array_equal(got, want)
    x = rng.standard_normal((n, 3, h, w)).astype(np.float32)
    wt = (rng.standard_normal((f, 3, 7, 7)) / np.sqrt(147)).astype(np.float32)
    ref = oracle.conv2d(x, wt, pad, pad, 2, 2)
    mag = oracle.conv2d(np.abs(x), np.abs(wt), pad, pad, 2, 2)
    assert max_rel_err(host(ops.conv2d(dev(x), dev(wt), pad, pad, 2, 2)), ref, mag) <= REL_TOL


STEMS_3D = [
    # n, t, h, w, f, kt, pt, st
    (1, 16, 112, 112, 64, 3, 1, 1),     # ResNet3D
    (1, 5, 20, 22, 64, 3, 1, 1),
    (2, 4, 18, 35, 24, 3, 1, 2),        # time stride 2, a batch, ragged
    (1, 6, 16, 16, 72, 5, 2, 1),        # five time slices, two filter blocks
    (1, 3, 14, 30, 8, 1, 0, 1),         # kt = 1 over several frames
    (1, 7, 12, 12, 16, 3, 0, 2),        # no time padding, stride 2
]


@pytest.mark.parametrize("case", STEMS_3D)
def test_stem_3d(ops, case):
    n, t, h, w, f, kt, pt, st = case
    rng = np.random.default_rng(sum(case))
    xi = rng.integers(-3, 4, (n, 3, t, h, w)).astype(np.float32)
    wi = rng.integers(-3, 4, (f, 3, kt, 7, 7)).astype(np.float32)
    bi = rng.integers(-3, 4, (f,)).astype(np.float32)
    want = oracle.conv3d(xi, wi, (pt, 3, 3), (st, 2, 2)) + bi[None, :, None, None, None]
    got = host(ops.conv3d(dev(xi), dev(wi), (pt, 3, 3), (st, 2, 2), bias=dev(bi)))
    assert got.shape == want.shape
    np.testing.assert_array_equal(got, want)
    x = rng.standard_normal((n, 3, t, h, w)).astype(np.float32)
    wt = (rng.standard_normal((f, 3, kt, 7, 7)) / np.sqrt(147 * kt)).astype(np.float32)
    ref = oracle.conv3d(x, wt, (pt, 3, 3), (st, 2, 2))
    mag = oracle.conv3d(np.abs(x), np.abs(wt), (pt, 3, 3), (st, 2, 2))
    got = host(ops.conv3d(dev(x), dev(wt), (pt, 3, 3), (st, 2, 2)))
    assert max_rel_err(got, ref, mag) <= REL_TOL


def test_stem_reads_its_input_through_a_relu_when_asked(ops):
    from pet_amd import abi
    rng = np.random.default_rng(3)
    x = rng.integers(-3, 4, (1, 3, 20, 20)).astype(np.float32)
    w = rng.integers(-3, 4, (32, 3, 7, 7)).astype(np.float32)
    want = oracle.conv2d(np.maximum(x, 0), w, 3, 3, 2, 2)
    got = host(ops.conv2d(dev(x), dev(w), 3, 3, 2, 2, flags=abi.X_RELU))
    np.testing.assert_array_equal(got, want)


def test_stem_equals_the_general_kernel(ops):
    """The same arguments with a residual go through the general kernel (the stem kernel has
    no residual operand): on integers the two must agree exactly."""
    rng = np.random.default_rng(4)
    x = dev(rng.integers(-3, 4, (2, 3, 50, 46)).astype(np.float32))
    w = dev(rng.integers(-3, 4, (64, 3, 7, 7)).astype(np.float32))
    y = ops.conv2d(x, w, 3, 3, 2, 2)
    z = ops.conv2d(x, w, 3, 3, 2, 2, residual=torch.zeros_like(y))
    assert torch.equal(y, z)


def test_stem_random_shapes(ops):
    """Thirty seeded shapes, 2-D and 3-D, small integers, bit for bit against the oracle."""
    rng = np.random.default_rng(2024)
    for _ in range(30):
        n, f = int(rng.integers(1, 4)), int(rng.integers(1, 140))
        h, w = int(rng.integers(7, 70)), int(rng.integers(7, 70))
        pad = int(rng.integers(0, 4))
        if rng.random() < 0.5:
            x = rng.integers(-3, 4, (n, 3, h, w)).astype(np.float32)
            k = rng.integers(-3, 4, (f, 3, 7, 7)).astype(np.float32)
            want = oracle.conv2d(x, k, pad, pad, 2, 2)
            got = host(ops.conv2d(dev(x), dev(k), pad, pad, 2, 2))
        else:
            t, kt = int(rng.integers(1, 7)), int(rng.integers(1, 4))
            pt, st = int(rng.integers(0, kt)), int(rng.integers(1, 3))
            if t + 2 * pt < kt:
                continue
            x = rng.integers(-3, 4, (n, 3, t, h, w)).astype(np.float32)
            k = rng.integers(-3, 4, (f, 3, kt, 7, 7)).astype(np.float32)
            want = oracle.conv3d(x, k, (pt, pad, pad), (st, 2, 2))
            got = host(ops.conv3d(dev(x), dev(k), (pt, pad, pad), (st, 2, 2)))
        assert got.shape == want.shape
        np.testing.assert_array_equal(got, want)
