"""Operands that start 4 bytes past a 16-byte boundary (a view into a larger buffer, which
the C ABI cannot tell from a whole allocation). The fast kernels read 16-byte words and fall
back, operand by operand, when a pointer does not allow it; inputs are small integers, so the
result must equal the aligned call's bit for bit whatever kernel ran."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from pet_amd import ops as _ops
    return _ops


def small_ints(shape, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return torch.randint(-3, 4, shape, device="cuda", generator=g).float()


def shifted(t):
    """The same values, one float past an allocation's (256-byte aligned) start."""
    buf = torch.empty(t.numel() + 1, device="cuda")
    buf[1:] = t.reshape(-1)
    view = buf[1:].reshape(t.shape)
    assert view.data_ptr() % 16 == 4
    return view


def check(call, operands, out_shape):
    """call(*operands, out) with every operand, and the output, shifted in turn."""
    want = torch.empty(out_shape, device="cuda")
    call(*operands, want)
    for i in range(len(operands)):
        if operands[i] is None:
            continue
        ops_i = list(operands)
        ops_i[i] = shifted(operands[i])
        got = torch.empty(out_shape, device="cuda")
        call(*ops_i, got)
        assert torch.equal(got, want), "operand %d shifted" % i
    got = shifted(torch.zeros(out_shape, device="cuda"))
    call(*operands, got)
    assert torch.equal(got, want), "output shifted"
    call(*[None if o is None else shifted(o) for o in operands], got)
    assert torch.equal(got, want), "everything shifted"


CONVS = [
    # n, c, h, w, f, r, s, pad, stride, dilation
    (2, 64, 16, 16, 64, 3, 3, 1, 1, 1),      # LDS-staged 3x3 tiles
    (1, 64, 12, 12, 32, 3, 3, 2, 1, 2),      # the same, dilated
    (1, 128, 7, 7, 128, 3, 3, 1, 1, 1),      # register-fed small layer
    (1, 64, 14, 14, 128, 1, 1, 0, 2, 1),     # 1x1 stride 2
    (2, 32, 9, 9, 48, 1, 1, 0, 1, 1),        # 1x1
    (1, 3, 30, 30, 16, 7, 7, 3, 2, 1),       # the general kernel
    (1, 8, 10, 11, 6, 2, 3, 1, 1, 1),
]


@pytest.mark.parametrize("case", CONVS)
def test_convolution(ops, case):
    n, c, h, w, f, r, s, pad, stride, dil = case
    x, wt, b = small_ints((n, c, h, w), 1), small_ints((f, c, r, s), 2), small_ints((f,), 3)
    oh = ops.conv_out_dim(h, r, pad, stride, dil)
    ow = ops.conv_out_dim(w, s, pad, stride, dil)
    res = small_ints((n, f, oh, ow), 4)
    check(lambda x, wt, b, res, out: ops.conv2d(x, wt, pad, pad, stride, stride, dil, dil, bias=b,
                                                act="relu", residual=res, out=out),
          [x, wt, b, res], (n, f, oh, ow))


def test_convolution_3d(ops):
    x, wt, b = small_ints((1, 32, 4, 8, 8), 1), small_ints((32, 32, 3, 3, 3), 2), small_ints((32,), 3)
    check(lambda x, wt, b, out: ops.conv3d(x, wt, (1, 1, 1), bias=b, act="relu", out=out),
          [x, wt, b], (1, 32, 4, 8, 8))


MATMULS = [
    # b, m, n, k, transA, transB
    (2, 64, 64, 64, False, False),
    (3, 128, 96, 64, False, False),
    (1, 1, 1000, 512, False, False),
    (2, 33, 17, 29, False, False),
    (2, 64, 64, 32, True, False),
    (2, 64, 48, 32, False, True),
    (1, 40, 24, 16, True, True),
]


@pytest.mark.parametrize("case", MATMULS)
def test_matmul(ops, case):
    b, m, n, k, ta, tb = case
    A = small_ints((b, k, m) if ta else (b, m, k), 5)
    B = small_ints((b, n, k) if tb else (b, k, n), 6)
    bias, res = small_ints((n,), 7), small_ints((b, m, n), 8)
    check(lambda A, B, bias, res, out: ops.matmul(A, B, ta, tb, bias=bias, act="relu",
                                                  residual=res, out=out),
          [A, B, bias, res], (b, m, n))


def test_transposed_convolution(ops):
    for n, hw, f, c in ((2, 5, 8, 12), (1, 2, 448, 64), (33, 3, 16, 8)):
        x, k, b = small_ints((n, hw, hw, f), 9), small_ints((4, 4, f, c), 10), small_ints((c,), 11)
        check(lambda x, k, b, out: ops.conv_trans(x, k, 1, 1, 2, 2, bias=b, act="relu", out=out),
              [x, k, b], (n, 2 * hw, 2 * hw, c))


def test_band_matmuls(ops):
    for bs, m, k, w, d in ((2, 100, 64, 20, 1), (1, 70, 96, 9, 2), (2, 40, 24, 5, 1)):
        q, kk = small_ints((bs, m, k), 12), small_ints((bs, m, k), 13)
        check(lambda q, kk, out: ops.g2bmm(q, kk, w, d, out=out), [q, kk], (bs, m, 2 * w + 1))
        band = small_ints((bs, m, 2 * w + 1), 14)
        check(lambda band, v, out: ops.gbmml(band, v, d, out=out), [band, q], (bs, m, k))


def test_rows_and_elements(ops):
    x = small_ints((6, 768), 15)
    g, b = small_ints((768,), 16), small_ints((768,), 17)
    # LayerNorm and softmax divide: compare within rounding of the aligned result instead
    want = ops.layernorm(x, g, b)
    for xs, gs, bs_ in ((shifted(x), g, b), (x, shifted(g), shifted(b))):
        got = ops.layernorm(xs, gs, bs_)
        assert torch.allclose(got, want, rtol=1e-6, atol=1e-6)
    got = ops.layernorm(x, g, b, out=shifted(torch.zeros_like(x)))
    assert torch.allclose(got, want, rtol=1e-6, atol=1e-6)
    want = ops.softmax(x)
    assert torch.allclose(ops.softmax(shifted(x)), want, rtol=1e-6, atol=1e-7)
    y = small_ints((6, 768), 18)
    check(lambda x, y, out: ops.eltwise("add", [x, y], out=out), [x, y], (6, 768))
    check(lambda x, out: ops.activation(x, "relu", out=out), [x], (6, 768))
    img = small_ints((2, 8, 12, 12), 19)
    check(lambda img, out: ops.pool2d(img, 3, 3, 1, 1, 2, 2, out=out), [img], (2, 8, 6, 6))
    check(lambda img, bb, out: ops.bias_act(img, bb, "relu", out=out),
          [img, small_ints((8,), 20)], (2, 8, 12, 12))


def test_attention_refuses_unaligned_rows_cleanly(ops):
    """Its Q and K rows are read as 16-byte words; the graph runtime only plans the fused
    kernel for buffers it allocated itself."""
    from pet_amd import abi
    q = small_ints((1, 16, 64), 21)
    out = ops.attention(q, q, q, 1, scale=0.125)
    got = ops.attention(q, q, shifted(q), 1, scale=0.125)       # V may sit anywhere
    assert torch.equal(got, out)
    with pytest.raises(abi.PetHipError) as e:
        ops.attention(shifted(q), q, q, 1, scale=0.125)
    assert e.value.status == 2
