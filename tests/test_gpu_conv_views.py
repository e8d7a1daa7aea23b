"""pet_hip_conv2d_view_f32: a convolution that reads x and / or writes y through strides, so
that PET's space-to-batch Transpose in front of a convolution and the batch-to-space Transpose
behind one (the dilated-to-dense mutation of src/Mutant/generator.cc; TransposeOp::compute,
src/Graph/operator.cc:2227-2245) cost no launch of their own.

Checked against the CPU oracle's convolution on operands that numpy transposes (small
integers: every summation order gives the same bits, so also launches that add partial sums
with atomics compare bit for bit), against the library's own Transpose + convolution on real
values (same kernel, same order: bit for bit where no atomics are involved), and, since space
to batch turns a dilated convolution into a dense one, against the dilated convolution itself.
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


@pytest.fixture(scope="module")
def ops():
    from pet_amd import ops as _ops
    return _ops


def to_batch(a, d):
    """[q, c, d*h, d*w] -> [(i, j, q), c, h, w], entry (i*d + j)*q + image = pixels (d*y+i, d*x+j)."""
    q, c, hh, ww = a.shape
    return np.ascontiguousarray(
        a.reshape(q, c, hh // d, d, ww // d, d).transpose(3, 5, 0, 1, 2, 4)
    ).reshape(d * d * q, c, hh // d, ww // d)


def to_space(a, d):
    b, c, h, w = a.shape
    q = b // (d * d)
    return np.ascontiguousarray(
        a.reshape(d, d, q, c, h, w).transpose(2, 3, 4, 0, 5, 1)).reshape(q, c, h * d, w * d)


# q images, channels, filters, batch-form height / width, interleave d, filter size
CASES = [
    (1, 64, 64, 16, 16, 2, 3),      # the register-fed kernel
    (1, 128, 64, 32, 32, 2, 3),     # the benchmark block's last layer
    (2, 16, 24, 6, 10, 2, 3),       # ragged tiles, two images
    (1, 8, 40, 5, 7, 4, 3),         # sixteen phases
    (3, 64, 96, 4, 4, 2, 1),        # 1x1 filters
    (1, 256, 128, 32, 32, 2, 3),    # the LDS-staged kernel, K shared between workgroups
    (1, 512, 64, 16, 16, 2, 3),
]


@pytest.mark.parametrize("q,c,f,hb,wb,d,k", CASES)
def test_views_against_the_oracle_on_transposed_operands(ops, q, c, f, hb, wb, d, k):
    rng = np.random.default_rng(q * 1000 + c + f + hb + d)
    x = rng.integers(-3, 4, (q, c, d * hb, d * wb)).astype(np.float32)
    w = rng.integers(-2, 3, (f, c, k, k)).astype(np.float32)
    bias = rng.integers(-4, 5, f).astype(np.float32)
    res = rng.integers(-9, 10, (q, f, d * hb, d * wb)).astype(np.float32)
    pad = k // 2
    xb = to_batch(x, d)
    want_b = oracle.conv2d(xb, w, pad, pad) + bias[None, :, None, None]
    want_s = to_space(want_b, d)
    view = ops.interleave_view(q, c, hb, wb, d)
    yview = ops.interleave_view(q, f, hb, wb, d)
    shape_b = (d * d * q, c, hb, wb)
    assert ops.conv2d_view_supported(shape_b, w.shape, pad, pad)
    X, XB, W, B = dev(x), dev(xb), dev(w), dev(bias)

    got = ops.conv2d(X, W, pad, pad, bias=B, x_view=view, x_shape=shape_b)
    assert np.array_equal(host(got), want_b), "x read through strides"

    out = torch.full((q, f, d * hb, d * wb), 7.0, device="cuda")
    ops.conv2d(XB, W, pad, pad, bias=B, y_view=yview, out=out)
    assert np.array_equal(host(out), want_s), "y written through strides"

    out = torch.full((q, f, d * hb, d * wb), 7.0, device="cuda")
    ops.conv2d(X, W, pad, pad, bias=B, act="relu", residual=dev(res), x_view=view,
               x_shape=shape_b, y_view=yview, out=out)
    assert np.array_equal(host(out), np.maximum(want_s + res, 0)), "both, residual laid out like y"


def test_space_to_batch_views_are_the_dilated_convolution(ops):
    """The identity the mutation rests on: a 3x3 convolution with dilation d and padding d is
    the dense one on the d*d pixel phases. The library's dilated convolution never sees a
    view; real values, so the comparison is to the contraction tolerance."""
    rng = np.random.default_rng(5)
    for q, c, f, hb, wb, d in ((1, 64, 32, 16, 16, 2), (2, 32, 48, 6, 5, 4)):
        x = rng.standard_normal((q, c, d * hb, d * wb)).astype(np.float32)
        w = (rng.standard_normal((f, c, 3, 3)) * 0.1).astype(np.float32)
        ref = oracle.conv2d(x, w, d, d, 1, 1, d, d)
        mag = oracle.conv2d(np.abs(x), np.abs(w), d, d, 1, 1, d, d)
        out = torch.empty((q, f, d * hb, d * wb), device="cuda")
        ops.conv2d(dev(x), dev(w), 1, 1, x_view=ops.interleave_view(q, c, hb, wb, d),
                   x_shape=(d * d * q, c, hb, wb), y_view=ops.interleave_view(q, f, hb, wb, d),
                   out=out)
        assert max_rel_err(host(out), ref, mag) <= REL_TOL
        direct = ops.conv2d(dev(x), dev(w), d, d, 1, 1, d, d)
        assert max_rel_err(host(direct), ref, mag) <= REL_TOL


def test_views_against_transpose_then_convolution_bit_for_bit(ops):
    """Real values: the viewed launch runs the kernel, tiling and summation order of the
    launch on the transposed copy, so where no atomics are involved the bits agree."""
    rng = np.random.default_rng(9)
    for q, c, f, hb, wb, d in ((1, 64, 64, 16, 16, 2), (1, 128, 64, 32, 32, 2), (1, 512, 512, 32, 32, 2)):
        x = dev(rng.standard_normal((q, c, d * hb, d * wb)).astype(np.float32))
        w = dev((rng.standard_normal((f, c, 3, 3)) * 0.05).astype(np.float32))
        flat, perm = [q, c, hb, d, wb, d], [3, 5, 0, 1, 2, 4]
        xb = ops.permute_flat(x, flat, perm).reshape(d * d * q, c, hb, wb)
        yb = ops.conv2d(xb, w, 1, 1, act="relu")
        ys = ops.permute_flat(yb, [d, d, q, f, hb, wb], [2, 3, 4, 0, 5, 1]).reshape(
            q, f, d * hb, d * wb)
        got_b = ops.conv2d(x, w, 1, 1, act="relu", x_view=ops.interleave_view(q, c, hb, wb, d),
                           x_shape=tuple(xb.shape))
        got_s = torch.empty_like(ys)
        ops.conv2d(xb, w, 1, 1, act="relu", y_view=ops.interleave_view(q, f, hb, wb, d), out=got_s)
        if ops.conv2d_accumulates(tuple(xb.shape), tuple(w.shape), 1, 1):
            scale = yb.abs().max().item()
            assert (got_b - yb).abs().max().item() <= 1e-5 * scale
            assert (got_s - ys).abs().max().item() <= 1e-5 * scale
        else:
            assert torch.equal(got_b, yb) and torch.equal(got_s, ys)


def test_views_that_are_refused(ops):
    from pet_amd import abi
    x = torch.zeros((1, 64, 16, 16), device="cuda")
    w = torch.zeros((32, 64, 3, 3), device="cuda")
    # strides that leave holes or visit a float twice
    for field, value in (("w_stride", 1), ("h_stride", 8), ("c_stride", 255)):
        v = ops.interleave_view(1, 64, 8, 8, 2)
        setattr(v, field, value)
        with pytest.raises(abi.PetHipError) as e:
            ops.conv2d(x, w, 1, 1, x_view=v, x_shape=(4, 64, 8, 8))
        assert e.value.status == 1
    v = ops.interleave_view(1, 64, 8, 8, 2)
    v.n_extent[1] = 3                                  # does not divide the batch
    with pytest.raises(abi.PetHipError):
        ops.conv2d(x, w, 1, 1, x_view=v, x_shape=(4, 64, 8, 8))
    # shapes the kernels that take views do not run: the caller keeps its Transpose
    x3 = torch.zeros((1, 3, 16, 16), device="cuda")
    w3 = torch.zeros((8, 3, 3, 3), device="cuda")
    assert not ops.conv2d_view_supported((4, 3, 8, 8), (8, 3, 3, 3), 1, 1)
    with pytest.raises(abi.PetHipError) as e:
        ops.conv2d(x3, w3, 1, 1, x_view=ops.interleave_view(1, 3, 8, 8, 2), x_shape=(4, 3, 8, 8))
    assert e.value.status == 2
    assert not ops.conv2d_view_supported((4, 64, 8, 8), (8, 64, 5, 5), 2, 2)
