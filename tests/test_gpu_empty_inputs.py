"""Empty tensors through the C ABI. The reference's loop nests simply do not run for an
extent of zero (src/Graph/operator.cc:94-158, 620-654, 1640-1662 ...); here an empty batch or
an empty output launches nothing and does not look at the pointers (torch hands out null
pointers for empty tensors), a contraction over an empty axis gives the bias, and negative
extents are still rejected."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from pet_amd import ops as _ops
    return _ops


def z(*shape):
    return torch.zeros(shape, device="cuda")


def r(*shape):
    return torch.randn(shape, device="cuda")


NO_OPS = {
    "conv2d, no images": (lambda o: o.conv2d(z(0, 8, 5, 5), r(4, 8, 3, 3), 1, 1), (0, 4, 5, 5)),
    "conv3d, no images": (lambda o: o.conv3d(z(0, 8, 4, 5, 5), r(4, 8, 3, 3, 3), (1, 1, 1)),
                          (0, 4, 4, 5, 5)),
    "matmul, no batch": (lambda o: o.matmul(z(0, 4, 8), z(0, 8, 5)), (0, 4, 5)),
    "matmul, no rows": (lambda o: o.matmul(z(2, 0, 8), r(2, 8, 5)), (2, 0, 5)),
    "matmul, no columns": (lambda o: o.matmul(r(2, 4, 8), z(2, 8, 0)), (2, 4, 0)),
    "conv_trans, no images": (lambda o: o.conv_trans(z(0, 3, 3, 8), r(3, 3, 8, 4), 1, 1, 2, 2),
                              (0, 5, 5, 4)),
    "g2bmm, no batch": (lambda o: o.g2bmm(z(0, 16, 8), z(0, 16, 8), 2, 1), (0, 16, 5)),
    "g2bmm, no rows": (lambda o: o.g2bmm(z(2, 0, 8), z(2, 0, 8), 2, 1), (2, 0, 5)),
    "gbmml, no batch": (lambda o: o.gbmml(z(0, 16, 5), z(0, 16, 8), 1), (0, 16, 8)),
    "attention, no sequences": (lambda o: o.attention(z(0, 16, 64), z(0, 16, 64), z(0, 16, 64), 2),
                                (0, 16, 64)),
    "transpose": (lambda o: o.permute_flat(z(0, 4, 6), [0, 4, 6], [2, 0, 1]), (6, 0, 4)),
    "concat of nothing": (lambda o: o.concat([z(0, 3), z(0, 3)], 0), (0, 3)),
    "pad": (lambda o: o.pad(z(0, 4), [0, 1], [0, 1]), (0, 6)),
    "slice down to nothing": (lambda o: o.slice_(r(2, 4), [1, 0], [1, 0]), (0, 4)),
    "extend": (lambda o: o.extend(z(0, 4), 1, 2), (0, 12)),
    "add": (lambda o: o.eltwise("add", [z(0, 4), z(0, 4)], out_shape=(0, 4)), (0, 4)),
    "relu": (lambda o: o.activation(z(0), "relu"), (0,)),
    "pow": (lambda o: o.pow_(z(0), 2), (0,)),
    "batchnorm": (lambda o: o.batchnorm(z(0, 4, 2, 2), r(4), r(4), r(4), r(4).abs() + 1),
                  (0, 4, 2, 2)),
    "gather of no indices": (lambda o: o.gather(r(4, 3), torch.zeros((0,), dtype=torch.int32,
                                                                      device="cuda"), 0), (0, 3)),
    "reduce_mean": (lambda o: o.reduce_mean(z(0, 4), 1), None),
    "bias_act": (lambda o: o.bias_act(z(0, 4, 2), r(4)), (0, 4, 2)),
    "pooling": (lambda o: o.pool2d(z(0, 4, 6, 6), 2, 2, 0, 0, 2, 2), (0, 4, 3, 3)),
    "softmax": (lambda o: o.softmax(z(0, 8)), (0, 8)),
    "layernorm": (lambda o: o.layernorm(z(0, 8), r(8), r(8)), (0, 8)),
}


@pytest.mark.parametrize("name", sorted(NO_OPS))
def test_an_empty_tensor_is_not_an_error(ops, name):
    fn, shape = NO_OPS[name]
    out = fn(ops)
    torch.cuda.synchronize()
    assert out.numel() == 0
    if shape is not None:
        assert tuple(out.shape) == shape


def test_split_of_an_empty_tensor(ops):
    parts = ops.split(z(0, 6, 4), 1, num=2)
    torch.cuda.synchronize()
    assert [tuple(p.shape) for p in parts] == [(0, 3, 4), (0, 3, 4)]


def test_contraction_over_an_empty_axis_gives_the_bias(ops):
    """sum over k in [0, 0) is 0: MatmulOp::compute's loop (operator.cc:620-654) leaves the
    zero it started from."""
    bias = r(5)
    got = ops.matmul(z(2, 4, 0), z(2, 0, 5))
    assert torch.equal(got, z(2, 4, 5))
    got = ops.matmul(z(2, 4, 0), z(2, 0, 5), bias=bias, act="relu")
    assert torch.equal(got, torch.relu(bias).expand(2, 4, 5))


def test_padding_around_an_empty_tensor_is_all_padding(ops):
    got = ops.pad(z(0, 4), [1, 0], [1, 0])
    torch.cuda.synchronize()
    assert torch.equal(got, z(2, 4))
    got = ops.concat([r(0, 3), torch.ones((2, 3), device="cuda")], 0)
    assert torch.equal(got, torch.ones((2, 3), device="cuda"))


def test_negative_extents_are_still_rejected():
    from pet_amd import abi
    abi.init(0)
    x = r(16)
    p = ctypes.c_void_p(x.data_ptr())
    with pytest.raises(abi.PetHipError):
        abi.call("pet_hip_g2bmm_f32", p, p, p, -1, 4, 4, 1, 1, None)
    with pytest.raises(abi.PetHipError):
        abi.call("pet_hip_g2bmm_f32", p, p, p, 1, 4, 0, 1, 1, None)      # no feature axis
    with pytest.raises(abi.PetHipError):
        abi.call("pet_hip_conv_trans_f32", p, p, None, p, -1, 2, 2, 1, 2, 2, 1, 0, 0, 1, 1, 1, 1,
                 0, 0, 0, None)
    with pytest.raises(abi.PetHipError):
        abi.call("pet_hip_conv_trans_f32", p, p, None, p, 0, 2, 2, 1, 2, 2, 1, 3, 3, 1, 1, 1, 1,
                 0, 0, 0, None)                                          # no output even so
