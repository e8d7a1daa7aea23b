"""The catalogue of transformed programs PET's mutator emits
(src/Mutant/generator.cc:1022-1552, src/nnet/nmutator.cc:529-668), each run through
the C ABI next to the operator it replaces. Inputs are small integers, so
"equivalent" means bit-equal, and the original is also checked against the oracle."""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from pet_amd import ops as _ops
    return _ops


rng = np.random.default_rng(314)


def ints(shape, lo=-3, hi=4):
    return torch.from_numpy(rng.integers(lo, hi, size=shape).astype(np.float32)).cuda()


def same(a, b):
    assert a.shape == b.shape, (a.shape, b.shape)
    assert torch.equal(a.contiguous(), b.contiguous())


def vs_oracle(t, ref):
    torch.cuda.synchronize()
    np.testing.assert_array_equal(t.cpu().numpy(), ref)


def test_w2n_with_halo_then_n2w_drop(ops):
    # generator.cc:1022-1064 (N2W / W2N) with the correction of transpose.cc:33-40, 75-88
    x, w = ints((2, 8, 12, 16)), ints((8, 8, 3, 3))
    y = ops.conv2d(x, w, 1, 1)
    vs_oracle(y, oracle.conv2d(x.cpu().numpy(), w.cpu().numpy(), 1, 1))
    # split W into two halves of 8 (+1 halo column each), halves join N
    xs = ops.trans_chain(x, [("split", 3, 8, 0, 1), ("reorder", [0, 3, 1, 2, 4]), ("fuse", 0, 0, 0)])
    assert tuple(xs.shape) == (4, 8, 12, 9)
    ys = ops.conv2d(xs, w, 1, 1)
    back = ops.trans_chain(ys, [("split", 0, 2, 0, 0), ("reorder", [0, 2, 3, 1, 4]), ("fuse", 3, 0, 1)])
    same(back, y)


def test_d2h_deinterleave_for_height_dilation(ops):
    # generator.cc:1080-1100: dilation 2 along H only
    x, w = ints((1, 8, 16, 10)), ints((8, 8, 3, 3))
    y = ops.conv2d(x, w, 2, 1, 1, 1, 2, 1)
    vs_oracle(y, oracle.conv2d(x.cpu().numpy(), w.cpu().numpy(), 2, 1, 1, 1, 2, 1))
    xs = ops.permute_flat(x, [1, 8, 8, 2, 10], [3, 0, 1, 2, 4]).reshape(2, 8, 8, 10)
    ys = ops.conv2d(xs, w, 1, 1)
    back = ops.permute_flat(ys, [2, 1, 8, 8, 10], [1, 2, 3, 0, 4]).reshape(1, 8, 16, 10)
    same(back, y)


def test_same_input_conv_merge(ops):
    # generator.cc:1327-1381: concat weights on dim 0, one conv, split on dim 1
    x, w1, w2 = ints((1, 8, 14, 14)), ints((8, 8, 3, 3)), ints((24, 8, 3, 3))
    y1, y2 = ops.conv2d(x, w1, 1, 1), ops.conv2d(x, w2, 1, 1)
    m = ops.conv2d(x, ops.concat([w1, w2], 0), 1, 1)
    a, b = ops.split(m, 1, sizes=[1, 3])
    same(a, y1)
    same(b, y2)


def test_group_merge_gcd(ops):
    # generator.cc:1159-1234: different inputs, f = 8 and 12, gcd 4 -> 5 groups
    x1, x2 = ints((1, 8, 10, 10)), ints((1, 8, 10, 10))
    w1, w2 = ints((8, 8, 3, 3)), ints((12, 8, 3, 3))
    y1, y2 = ops.conv2d(x1, w1, 1, 1), ops.conv2d(x2, w2, 1, 1)
    xin = ops.concat([ops.extend(x1, 1, 1), ops.extend(x2, 1, 2)], 1)   # 2 + 3 copies
    m = ops.conv2d(xin, ops.concat([w1, w2], 0), 1, 1)                   # cpg = 8 -> 5 groups
    a, b = ops.split(m, 1, sizes=[2, 3])
    same(a, y1)
    same(b, y2)


def test_group_merge_max_zero_padded_kernel(ops):
    # generator.cc:1236-1325: a 1x1 filter zero-padded to 3x3 joins a 3x3 conv
    x, w3, w1 = ints((1, 16, 12, 12)), ints((8, 16, 3, 3)), ints((8, 16, 1, 1))
    y3, y1 = ops.conv2d(x, w3, 1, 1), ops.conv2d(x, w1, 0, 0)
    wp = ops.pad(w1, [0, 0, 1, 1], [0, 0, 1, 1])
    m = ops.conv2d(x, ops.concat([w3, wp], 0), 1, 1)
    a, b = ops.split(m, 1, num=2)
    same(a, y3)
    same(b, y1)


def test_grouped_conv_split_into_per_group_convs(ops):
    # generator.cc:1783-1856
    x, w = ints((2, 16, 9, 9)), ints((12, 4, 3, 3))   # 4 groups
    y = ops.conv2d(x, w, 1, 1)
    vs_oracle(y, oracle.conv2d(x.cpu().numpy(), w.cpu().numpy(), 1, 1))
    xs, ws = ops.split(x, 1, num=4), ops.split(w, 0, num=4)
    same(ops.concat([ops.conv2d(a, b, 1, 1) for a, b in zip(xs, ws)], 1), y)


def test_conv1x1_as_matmul(ops):
    # generator.cc:1412-1459 / nmutator.cc:641-668: Y[f, hw] = W[f, c] X[c, hw]
    x, w = ints((1, 32, 14, 14)), ints((64, 32, 1, 1))
    y = ops.conv2d(x, w, 0, 0)
    m = ops.matmul(w.reshape(1, 64, 32), x.reshape(1, 32, 196))
    same(m.reshape(1, 64, 14, 14), y)
    # batch 3: weights as [1, f, c] against [n, c, hw] via one matmul per image merged on dim 0
    xb = ints((3, 32, 7, 7))
    yb = ops.conv2d(xb, w, 0, 0)
    mb = ops.matmul(ops.extend(w.reshape(1, 64, 32), 0, 2), xb.reshape(3, 32, 49))
    same(mb.reshape(3, 64, 7, 7), yb)


def test_transposed_operand_forms_of_matmul(ops):
    # generator.cc:1147-1155: transA / transB absorb a Transpose(-1, {0, 2, 1})
    A, B = ints((2, 24, 40)), ints((2, 40, 16))
    y = ops.matmul(A, B)
    vs_oracle(y, oracle.matmul(A.cpu().numpy(), B.cpu().numpy()))
    At, Bt = ops.transpose(A, -1, [0, 2, 1], 2), ops.transpose(B, -1, [0, 2, 1], 2)
    same(ops.matmul(At, B, True, False), y)
    same(ops.matmul(A, Bt, False, True), y)
    same(ops.matmul(At, Bt, True, True), y)


def test_pad_conv_slice(ops):
    # generator.cc:1383-1410: odd image padded to even, convolved, cropped back
    x, w = ints((1, 8, 13, 15)), ints((8, 8, 3, 3))
    y = ops.conv2d(x, w, 1, 1)
    xp = ops.pad(x, [0, 0, 0, 0], [0, 0, 1, 1])
    same(ops.slice_(ops.conv2d(xp, w, 1, 1), [0, 0, 0, 0], [0, 0, 1, 1]), y)


def test_1xk_as_kx1_through_transposes(ops):
    # generator.cc:1461-1494: Transpose(-1, {0, 1, 3, 2}) on input, weight and output
    x, w = ints((2, 4, 9, 12)), ints((6, 4, 1, 5))
    y = ops.conv2d(x, w, 0, 2)
    vs_oracle(y, oracle.conv2d(x.cpu().numpy(), w.cpu().numpy(), 0, 2))
    t = lambda a: ops.transpose(a, -1, [0, 1, 3, 2], 2)
    same(t(ops.conv2d(t(x), t(w), 2, 0)), y)


def test_batch_matmul_merge(ops):
    # generator.cc:1495-1552: concat lhs on dim 0, concat rhs on dim 0, one bmm, split
    A, W0, W1 = ints((1, 16, 24)), ints((1, 24, 8)), ints((1, 24, 8))
    m = ops.matmul(ops.concat([A, A], 0), ops.concat([W0, W1], 0))
    a, b = ops.split(m, 0, num=2)
    same(a, ops.matmul(A, W0))
    same(b, ops.matmul(A, W1))
