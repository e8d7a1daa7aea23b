"""CPU-only: the PET-transformed programs of the configurations are equivalent to
the original networks under the oracle alone (tiny sizes)."""
import numpy as np

import configs


def test_transformed_programs_equal_originals_under_the_oracle():
    cpu = configs.OracleNS()
    p1 = configs.params_c1(1, c=8, hw=12)
    np.testing.assert_allclose(configs.run_c1(cpu, p1, True), configs.run_c1(cpu, p1, False),
                               rtol=1e-5, atol=1e-5)
    p2 = configs.params_c2(1, channels=[8, 8, 4], hw=8)
    np.testing.assert_allclose(configs.run_c2(cpu, p2, True), configs.run_c2(cpu, p2, False),
                               rtol=1e-5, atol=1e-6)
    p3 = configs.params_c3(1, hw=32, width=8, classes=10)
    np.testing.assert_allclose(configs.run_c3(cpu, p3, True), configs.run_c3(cpu, p3, False),
                               rtol=1e-4, atol=1e-5)
    p4 = configs.params_c4(1, layers=2, seq=8, hidden=32, heads=4, ffn=64)
    np.testing.assert_allclose(configs.run_c4(cpu, p4, True), configs.run_c4(cpu, p4, False),
                               rtol=1e-4, atol=1e-5)
    p5 = configs.params_c5(1, t=8, hw=16, width=8, classes=10)
    np.testing.assert_allclose(configs.run_c5(cpu, p5, True), configs.run_c5(cpu, p5, False),
                               rtol=1e-4, atol=1e-5)
