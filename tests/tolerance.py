"""The error measure of the real-valued contraction tests.

The device sums in fp32, the oracle in fp64. Output i is compared as

    max(|got_i - ref_i| - 2^-23 * A_i, 0) / max(|ref_i|, 1e-3 * A_i)  <=  1e-4

with A_i = sum_k |a_ik| |b_kj|, the same contraction on absolute values (also from
the oracle), and the normwise error max|got - ref| / max|ref| must meet the same 1e-4.

* The floor 1e-3 * A_i only matters for outputs that cancel to below a thousandth of
  their own terms, where no summation order can hold a bound relative to the result;
  the reference's checker floors the denominator for the same reason
  (src/Test/dat/transpose_test/checker_tf.py:66).
* 2^-23 * A_i is one unit in the last place of an fp32 number of the size the partial
  sums can reach. 1e-4 of the floor is 1e-7 * A_i, below that unit (1.19e-7): without
  the allowance the test asks the fp32 result format for more digits than it has, and a
  plain in-order fp32 sum of 147 terms fails it on 1 output in 800 000 while being as
  good as fp32 gets. An indexing mistake moves an output by whole terms, thousands of
  times either allowance, and the small-integer tier catches it bit for bit.
"""
import numpy as np

REL_TOL = 1e-4
FLOOR = 1e-3
ULP = 2.0 ** -23


def max_rel_err(got, ref, mag):
    """mag: the contraction of |a| and |b| (term magnitude per output)."""
    if not ref.size:
        return 0.0
    got = got.astype(np.float64)
    ref = ref.astype(np.float64)
    mag = mag.astype(np.float64)
    err = np.abs(got - ref)
    # an output without terms (mag == 0) must be exactly 0: any error there divides by 1e-300
    den = np.maximum(np.maximum(np.abs(ref), FLOOR * mag), 1e-300)
    elem = np.max(np.maximum(err - ULP * mag, 0.0) / den)
    norm = np.max(err) / max(np.max(np.abs(ref)), 1e-300)
    return float(max(elem, norm))
