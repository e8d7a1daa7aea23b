"""Operands of more than 2 GiB: the fast kernels address with 32-bit byte offsets and hand
such shapes to the kernels that use 64-bit addresses. Inputs are small integers, so every
sum is exact in fp32 whatever its order and the comparisons are bit for bit: a convolution
against the same convolution run on row slices (small enough for the fast kernels), a matmul
against torch's, a transpose against torch's."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from pet_amd import ops as _ops
    free, _ = torch.cuda.mem_get_info()
    if free < 48 << 30:
        pytest.skip("needs 48 GiB of free device memory")
    return _ops


def small_ints(shape, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return torch.randint(-3, 4, shape, device="cuda", generator=g).float()


@pytest.mark.parametrize("ksize", [1, 3])
def test_convolution_of_an_input_beyond_2_gib(ops, ksize):
    c, f, h, w = 32, 32, 4608, 4608                       # 2.53 GiB in, 2.53 GiB out
    x = small_ints((1, c, h, w), 1)
    wt = small_ints((f, c, ksize, ksize), 2)
    pad = ksize // 2
    y = ops.conv2d(x, wt, pad, pad, act="relu")
    torch.cuda.synchronize()
    assert y.shape == (1, f, h, w)
    # eight rows at the top, past the first GiB, in the middle (past 2 GiB in the last
    # channels) and at the bottom, each with the halo its filter reads: the slice's own zero
    # padding then falls outside the rows compared
    for a in (0, 1000, h // 2 - 4, h - 8):
        lo, hi = max(a - pad, 0), min(a + 8 + pad, h)
        part = ops.conv2d(x[:, :, lo:hi].contiguous(), wt, pad, pad, act="relu")
        assert torch.equal(part[:, :, a - lo:a - lo + 8], y[:, :, a:a + 8])
    del x, y


def test_matmul_with_a_4_gib_operand(ops):
    m, k, n = 32768, 32768, 64                            # A: 2^30 elements
    A = small_ints((1, m, k), 3)
    B = small_ints((1, k, n), 4)
    got = ops.matmul(A, B)
    want = torch.matmul(A, B)                             # |sum| <= 9 * 32768 < 2^24: exact
    assert torch.equal(got, want)
    got = ops.matmul(A.reshape(1, k, m), B, transA=True)
    assert torch.equal(got, torch.matmul(A.reshape(1, k, m).transpose(1, 2), B))
    del A, got, want


def test_transpose_of_6_gib(ops):
    rows, cols = 3 << 9, 1 << 20                          # 1.5 * 2^30 elements
    x = small_ints((rows, cols), 5)
    got = ops.permute_flat(x, [rows, cols], [1, 0])
    assert got.shape == (cols, rows)
    assert torch.equal(got, x.t().contiguous())
    back = ops.permute_flat(got, [cols, rows], [1, 0])
    assert torch.equal(back, x)


def test_transposed_convolution_with_an_output_beyond_2_gib(ops):
    n, hw, f, c = 256, 64, 64, 128                        # out 256 x 128 x 128 x 128: 2 GiB
    x = small_ints((n, hw, hw, f), 6)
    k = small_ints((4, 4, f, c), 7)
    y = ops.conv_trans(x, k, 1, 1, 2, 2)
    assert y.shape == (n, 2 * hw, 2 * hw, c) and y.numel() * 4 >= 1 << 31
    for a in (0, 127, 254):                               # two images at a time
        assert torch.equal(ops.conv_trans(x[a:a + 2].contiguous(), k, 1, 1, 2, 2), y[a:a + 2])
    del x, y


def test_band_matmuls_with_a_band_matrix_beyond_2_gib(ops):
    bs, m, k, w = 40, 8192, 64, 1024                      # band: 40 x 8192 x 2049, 2.5 GiB
    q = small_ints((bs, m, k), 8)
    kk = small_ints((bs, m, k), 9)
    band = ops.g2bmm(q, kk, w, 1)
    assert band.shape == (bs, m, 2 * w + 1) and band.numel() * 4 >= 1 << 31
    for a in (0, 19, 38):
        assert torch.equal(ops.g2bmm(q[a:a + 2].contiguous(), kk[a:a + 2].contiguous(), w, 1),
                           band[a:a + 2])
    # band x general: |sum| <= 2049 * (9 * 64) * 3 < 2^24, still exact
    v = small_ints((bs, m, k), 10)
    out = ops.gbmml(band, v, 1)
    for a in (0, 19, 38):
        assert torch.equal(ops.gbmml(band[a:a + 2].contiguous(), v[a:a + 2].contiguous(), 1),
                           out[a:a + 2])
