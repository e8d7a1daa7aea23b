"""The ConvTranspose vectors the reference's own tests hold
(tests/golden/convtrans_reference_vectors.json) as numpy arrays."""
import json
import os

import numpy as np


def reference_cases(dtype=np.float32):
    """Yields (x NHWF, K RSFC, params, expected NHWC)."""
    path = os.path.join(os.path.dirname(__file__), "golden", "convtrans_reference_vectors.json")
    for c in json.load(open(path))["cases"]:
        n, h, w, f, r, s, ch = (c[k] for k in ("n", "h", "w", "f", "r", "s", "c"))
        x = np.arange(n * h * w * f, dtype=np.int64).reshape(n, h, w, f).astype(dtype)
        ff, rr, ss, cc = np.meshgrid(np.arange(f), np.arange(r), np.arange(s), np.arange(ch),
                                     indexing="ij")
        k_frsc = ((ff * r + rr) * s + ss) * ch + cc            # value at [f, r, s, c]
        K = np.ascontiguousarray(k_frsc.transpose(1, 2, 0, 3)).astype(dtype)  # stored [r, s, f, c]
        want = np.array(c["nchw"], dtype=np.int64).reshape(c["nchw_shape"]).transpose(0, 2, 3, 1)
        prm = dict(ph=c["ph"], pw=c["pw"], sh=c["sh"], sw=c["sw"], dh=c["dh"], dw=c["dw"])
        yield x, K, prm, np.ascontiguousarray(want).astype(dtype)
