"""GPU parity of ConvTrans, G2BMM and GBMML against the CPU oracle: the reference's own
ConvTranspose vectors and small-integer inputs bit for bit, real-valued inputs within the
contraction tolerance of tests/tolerance.py."""
import numpy as np
import pytest
import torch

import oracle
from convtrans_cases import reference_cases
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


def test_conv_trans_reference_vectors(ops):
    """src/Test/convtrans_test_1.cc:62-77, 120-135 through the C ABI."""
    for x, K, prm, want in reference_cases():
        got = host(ops.conv_trans(dev(x), dev(K), prm["ph"], prm["pw"], prm["sh"], prm["sw"],
                                  prm["dh"], prm["dw"]))
        np.testing.assert_array_equal(got, want)


CONV_TRANS_CASES = [
    # n, h, w, f, r, s, c, ph, pw, sh, sw, dh, dw, oph, opw
    (2, 5, 6, 4, 3, 3, 5, 1, 1, 2, 2, 1, 1, 0, 0),
    (1, 4, 4, 8, 4, 4, 40, 1, 1, 2, 2, 1, 1, 0, 0),      # 16-byte loads, two channel tiles
    (1, 7, 5, 2, 3, 2, 3, 0, 1, 1, 2, 1, 1, 0, 0),
    (1, 5, 5, 3, 3, 3, 2, 1, 1, 2, 2, 1, 1, 1, 1),       # output padding
    (1, 6, 5, 2, 4, 3, 3, 0, 0, 3, 1, 1, 1, 0, 0),       # the reference's tap skip (ah = 2)
    (1, 5, 4, 2, 5, 5, 3, 2, 2, 3, 3, 1, 1, 0, 0),
    (3, 3, 3, 16, 1, 1, 7, 0, 0, 1, 1, 1, 1, 0, 0),
    (1, 6, 6, 4, 3, 3, 4, 1, 1, 2, 2, 2, 2, 0, 0),       # dilated taps, as the loop nest reads
    (4, 16, 16, 64, 4, 4, 33, 1, 1, 2, 2, 1, 1, 0, 0),   # several pixel tiles per phase
    (16, 7, 7, 128, 4, 4, 64, 1, 1, 2, 2, 1, 1, 0, 0),   # a DCGAN / InfoGAN generator layer
    # few pixels, many features: the waves of a workgroup share the feature axis
    (1, 2, 2, 448, 4, 4, 256, 0, 0, 1, 1, 1, 1, 0, 0),   # src/Test/transposeconv_test_1.cc
    (1, 3, 3, 68, 3, 3, 40, 1, 1, 2, 2, 1, 1, 0, 0),     # the same without 16-byte loads
    (2, 5, 4, 96, 3, 3, 33, 1, 1, 2, 2, 1, 1, 1, 0),     # ragged pixel and channel tiles
    # 32 images or more: pixels numbered with the image fastest, taps skipped per wave
    (64, 1, 1, 100, 4, 4, 48, 0, 0, 1, 1, 1, 1, 0, 0),   # a generator's first layer (z = 100)
    (37, 3, 2, 12, 3, 3, 5, 1, 0, 2, 1, 1, 1, 0, 0),
]


@pytest.mark.parametrize("case", CONV_TRANS_CASES)
def test_conv_trans_both_tiers(ops, case):
    n, h, w, f, r, s, c, ph, pw, sh, sw, dh, dw, oph, opw = case
    rng = np.random.default_rng(sum(case))
    xi = rng.integers(-3, 4, (n, h, w, f)).astype(np.float32)
    Ki = rng.integers(-3, 4, (r, s, f, c)).astype(np.float32)
    want = oracle.conv_trans(xi, Ki, ph, pw, sh, sw, dh, dw, oph, opw)
    got = host(ops.conv_trans(dev(xi), dev(Ki), ph, pw, sh, sw, dh, dw, oph, opw))
    assert got.shape == want.shape
    np.testing.assert_array_equal(got, want)
    x = rng.standard_normal((n, h, w, f)).astype(np.float32)
    K = (rng.standard_normal((r, s, f, c)) / np.sqrt(f)).astype(np.float32)
    ref = oracle.conv_trans(x, K, ph, pw, sh, sw, dh, dw, oph, opw)
    mag = oracle.conv_trans(np.abs(x), np.abs(K), ph, pw, sh, sw, dh, dw, oph, opw)
    got = host(ops.conv_trans(dev(x), dev(K), ph, pw, sh, sw, dh, dw, oph, opw))
    assert max_rel_err(got, ref, mag) <= REL_TOL


def test_conv_trans_bias_and_activation(ops):
    rng = np.random.default_rng(11)
    x = rng.integers(-3, 4, (2, 4, 4, 8)).astype(np.float32)
    K = rng.integers(-3, 4, (4, 4, 8, 6)).astype(np.float32)
    b = rng.integers(-3, 4, 6).astype(np.float32)
    want = np.maximum(oracle.conv_trans(x, K, 1, 1, 2, 2) + b, 0)
    got = host(ops.conv_trans(dev(x), dev(K), 1, 1, 2, 2, bias=dev(b), act="relu"))
    np.testing.assert_array_equal(got, want)
    # the form in which waves share the feature axis has its own epilogue
    x = rng.integers(-3, 4, (1, 3, 3, 128)).astype(np.float32)
    K = rng.integers(-3, 4, (3, 3, 128, 37)).astype(np.float32)
    b = rng.integers(-3, 4, 37).astype(np.float32)
    want = np.maximum(oracle.conv_trans(x, K, 1, 1, 2, 2) + b, 0)
    got = host(ops.conv_trans(dev(x), dev(K), 1, 1, 2, 2, bias=dev(b), act="relu"))
    np.testing.assert_array_equal(got, want)


def test_conv_trans_rejects_bad_arguments(ops):
    from pet_amd import abi
    x, K = dev(np.zeros((1, 2, 2, 3), np.float32)), dev(np.zeros((2, 2, 3, 2), np.float32))
    with pytest.raises(abi.PetHipError):
        ops.conv_trans(x, K, 0, 0, 0, 1)          # stride 0
    with pytest.raises(abi.PetHipError):
        ops.conv_trans(x, K, 3, 3, 1, 1)          # padding eats the whole output


BAND_CASES = [
    # bs, m, k, w, d
    (2, 9, 5, 2, 1),
    (1, 17, 8, 3, 2),
    (3, 40, 16, 6, 4),
    (1, 5, 3, 7, 1),        # band wider than the matrix
    (2, 100, 64, 20, 1),
    (1, 257, 64, 33, 4),    # ragged row blocks in every residue class
    (8, 512, 64, 64, 1),    # a sliding-window attention head block
    (2, 70, 96, 9, 2),      # three 32-wide chunks of the feature axis
    (1, 64, 32, 40, 1),     # one chunk, band wider than the matrix
    (32, 2048, 128, 8, 1),  # many tiles: a tile per wave, 64 output columns in GBMML
    (32, 4096, 32, 4, 1),   # many tiles of 32 output columns
]


@pytest.mark.parametrize("case", BAND_CASES)
def test_g2bmm_both_tiers(ops, case):
    bs, m, k, w, d = case
    rng = np.random.default_rng(sum(case))
    Ai = rng.integers(-3, 4, (bs, m, k)).astype(np.float32)
    Bi = rng.integers(-3, 4, (bs, m, k)).astype(np.float32)
    np.testing.assert_array_equal(host(ops.g2bmm(dev(Ai), dev(Bi), w, d)),
                                  oracle.g2bmm(Ai, Bi, w, d))
    A = rng.standard_normal((bs, m, k)).astype(np.float32)
    B = rng.standard_normal((bs, m, k)).astype(np.float32)
    ref, mag = oracle.g2bmm(A, B, w, d), oracle.g2bmm(np.abs(A), np.abs(B), w, d)
    got = host(ops.g2bmm(dev(A), dev(B), w, d))
    # band entries that fall outside the matrix have no terms: exact zeros on both sides
    assert np.all(got[mag == 0] == 0)
    assert max_rel_err(got, ref, mag) <= REL_TOL


@pytest.mark.parametrize("case", BAND_CASES)
def test_gbmml_both_tiers(ops, case):
    bs, m, n, w, d = case
    rng = np.random.default_rng(sum(case) + 1)
    Ai = rng.integers(-3, 4, (bs, m, 2 * w + 1)).astype(np.float32)
    Bi = rng.integers(-3, 4, (bs, m, n)).astype(np.float32)
    np.testing.assert_array_equal(host(ops.gbmml(dev(Ai), dev(Bi), d)), oracle.gbmml(Ai, Bi, d))
    A = rng.standard_normal((bs, m, 2 * w + 1)).astype(np.float32)
    B = rng.standard_normal((bs, m, n)).astype(np.float32)
    ref, mag = oracle.gbmml(A, B, d), oracle.gbmml(np.abs(A), np.abs(B), d)
    assert max_rel_err(host(ops.gbmml(dev(A), dev(B), d)), ref, mag) <= REL_TOL


def test_band_products_compose_into_windowed_attention(ops):
    """probabilities x values over the band equals the dense masked attention: a property
    that holds at any size (here 4 x 1000 x 64, window 2 x 50 + 1, dilation 2)."""
    bs, m, k, w, d = 4, 1000, 64, 50, 2
    rng = np.random.default_rng(5)
    q = dev(rng.standard_normal((bs, m, k)).astype(np.float32))
    kk = dev(rng.standard_normal((bs, m, k)).astype(np.float32))
    v = dev(rng.standard_normal((bs, m, k)).astype(np.float32))
    s = ops.g2bmm(q, kk, w, d)
    out = host(ops.gbmml(s, v, d))
    dense = torch.bmm(q.double().cpu(), kk.double().cpu().transpose(1, 2))
    i = torch.arange(m)
    off = i[None, :] - i[:, None]
    mask = (off.abs() <= w * d) & (off % d == 0)
    want = torch.bmm(dense * mask, v.double().cpu()).numpy()
    assert np.abs(out - want).max() <= 1e-4 * np.abs(want).max()
