"""The five benchmark configurations end to end: the original network and the
PET-transformed program both run on the GPU through the C ABI and are compared
with the CPU oracle running the original network on the same seeded inputs.

Full sizes are used wherever the oracle finishes in seconds on the test box;
config 5 (81 GFLOP of naive CPU loops) is checked at full size through the
transformed == original property and against the oracle at a reduced clip.
Tolerance: normwise relative error <= 1e-4 (max|got - ref| / max|ref|): the
outputs are sums of thousands of fp32 terms pushed through up to 21 layers.
"""
import numpy as np
import pytest

import configs

pytestmark = pytest.mark.gpu

TOL = 1e-4


def norm_err(got, ref):
    return float(np.max(np.abs(got - ref)) / max(np.max(np.abs(ref)), 1e-30))


@pytest.fixture(scope="module")
def gpu():
    return configs.GpuNS()


@pytest.fixture(scope="module")
def cpu():
    return configs.OracleNS()


def check(run, params, gpu, cpu, ref=None):
    if ref is None:
        ref = cpu.numpy(run(cpu, params, False))
    y0 = gpu.numpy(run(gpu, params, False))
    y1 = gpu.numpy(run(gpu, params, True))
    assert y0.shape == ref.shape and y1.shape == ref.shape
    assert np.isfinite(y0).all() and np.isfinite(y1).all()
    assert norm_err(y0, ref) <= TOL, "original program"
    assert norm_err(y1, ref) <= TOL, "transformed program"
    return ref


def test_config1_conv_and_corrected_h2n(gpu, cpu):
    check(configs.run_c1, configs.params_c1(0), gpu, cpu)


def test_config2_dilated_block_space_to_batch(gpu, cpu):
    check(configs.run_c2, configs.params_c2(0), gpu, cpu)


def test_config3_resnet18(gpu, cpu):
    ref = check(configs.run_c3, configs.params_c3(0), gpu, cpu)
    assert ref.shape == (1, 1, 1000)


def test_config4_bert_encoder(gpu, cpu):
    ref = check(configs.run_c4, configs.params_c4(0), gpu, cpu)
    assert ref.shape == (1, 128, 768)


def test_config5_resnet3d18_reduced_vs_oracle(gpu, cpu):
    # clip 8x56x56, width 32: the same graph, 1/64 of the work for the CPU loops
    check(configs.run_c5, configs.params_c5(0, t=8, hw=56, width=32), gpu, cpu)


def test_config5_resnet3d18_full_size_property(gpu):
    p = configs.params_c5(0)
    y0 = gpu.numpy(configs.run_c5(gpu, p, False))
    y1 = gpu.numpy(configs.run_c5(gpu, p, True))
    assert y0.shape == (1, 1, 400)
    assert np.isfinite(y0).all()
    assert norm_err(y1, y0) <= TOL
    # linearity of the first layer at full size: conv(2x) == 2 conv(x) exactly
    x = gpu.tensor(p["x"])
    w = gpu.tensor(p["stem.w"])
    a = gpu.numpy(gpu.conv3d(x, w, (1, 3, 3), (1, 2, 2)))
    b = gpu.numpy(gpu.conv3d(gpu.tensor(2 * p["x"]), w, (1, 3, 3), (1, 2, 2)))
    assert np.array_equal(b, 2 * a)


def test_integer_tier_end_to_end_is_bit_exact(gpu, cpu):
    # small-integer weights and inputs through two conv layers + residual add: the
    # whole chain is exact in fp32, so GPU and oracle agree bit for bit, in both
    # the original and the corrected H2N program
    rng = np.random.default_rng(3)
    p = {"x": rng.integers(-2, 3, (1, 16, 24, 20)).astype(np.float32),
         "w": rng.integers(-2, 3, (16, 16, 3, 3)).astype(np.float32)}
    ref = cpu.numpy(configs.run_c1(cpu, p, False))
    assert np.array_equal(gpu.numpy(configs.run_c1(gpu, p, False)), ref)
    assert np.array_equal(gpu.numpy(configs.run_c1(gpu, p, True)), ref)
    assert np.array_equal(cpu.numpy(configs.run_c1(cpu, p, True)), ref)
