"""Golden vectors (tests/golden/golden.npz, written by tests/golden/make_golden.py
from torch CPU / numpy closed forms): the CPU oracle and the HIP path must both
reproduce them bit for bit. The inputs are small integers, so every result is
exact in fp32 and in the reference's uint32 arithmetic alike."""
import os

import numpy as np
import pytest

import oracle

G = np.load(os.path.join(os.path.dirname(__file__), "golden", "golden.npz"))
N_CONV2D, N_CONV3D = 6, 3


class OracleBackend:
    name = "oracle"

    def put(self, a):
        return np.ascontiguousarray(a)

    def get(self, a):
        return np.asarray(a)

    def put_idx(self, a):
        return np.ascontiguousarray(a)

    def div(self, a, b):
        return oracle.div(a, b, a.shape)

    def __getattr__(self, k):
        return getattr(oracle, k)


class HipBackend:
    name = "hip"

    def __init__(self):
        import torch
        from pet_amd import ops
        self.torch, self.ops = torch, ops

    def put(self, a):
        return self.torch.from_numpy(np.ascontiguousarray(a)).cuda()

    def get(self, t):
        self.torch.cuda.synchronize()
        return t.cpu().numpy()

    def put_idx(self, a):
        return self.torch.from_numpy(np.ascontiguousarray(a)).cuda()

    def div(self, a, b):
        return self.ops.eltwise("div", [a, b], tuple(a.shape))

    def __getattr__(self, k):
        return getattr(self.ops, k)


def check_all(be):
    eq = np.testing.assert_array_equal
    for i in range(N_CONV2D):
        n, c, h, w, f, cpg, r, s, ph, pw, sh, sw, dh, dw = (int(v) for v in G[f"conv2d_{i}_args"])
        y = be.get(be.conv2d(be.put(G[f"conv2d_{i}_x"]), be.put(G[f"conv2d_{i}_w"]),
                             ph, pw, sh, sw, dh, dw))
        eq(y, G[f"conv2d_{i}_y"])
    for i in range(N_CONV3D):
        a = [int(v) for v in G[f"conv3d_{i}_args"]]
        pad, st, dil = tuple(a[10:13]), tuple(a[13:16]), tuple(a[16:19])
        y = be.get(be.conv3d(be.put(G[f"conv3d_{i}_x"]), be.put(G[f"conv3d_{i}_w"]), pad, st, dil))
        eq(y, G[f"conv3d_{i}_y"])
    # the reference's batch-GEMM merge case: two matmuls == concat -> bmm -> split
    A, W0, W1 = be.put(G["mm_merge_A"]), be.put(G["mm_merge_W0"]), be.put(G["mm_merge_W1"])
    eq(be.get(be.matmul(A, W0)), G["mm_merge_Y0"])
    eq(be.get(be.matmul(A, W1)), G["mm_merge_Y1"])
    merged = be.matmul(be.concat([A, A], 0), be.concat([W0, W1], 0))
    y0, y1 = be.split(merged, 0, sizes=[1, 1])
    eq(be.get(y0), G["mm_merge_Y0"])
    eq(be.get(y1), G["mm_merge_Y1"])
    a, b, at, bt = (be.put(G[k]) for k in ("mm_t_A", "mm_t_B", "mm_t_At", "mm_t_Bt"))
    eq(be.get(be.matmul(a, b)), G["mm_t_Y"])
    eq(be.get(be.matmul(at, b, True, False)), G["mm_t_Y"])
    eq(be.get(be.matmul(a, bt, False, True)), G["mm_t_Y"])
    eq(be.get(be.matmul(at, bt, True, True)), G["mm_t_Y"])
    # transposes: operator form (TransposeOp split / after / factor) and flat form
    x = be.put(G["tr_x"])
    h2n = be.transpose(x, 2, [[0, 2], 1, -1, 3], -2)
    eq(be.get(h2n), G["tr_h2n"])
    eq(be.get(be.transpose(h2n, 0, [0, 1, [-1, 2], 3], 2)), G["tr_n2h"])
    eq(G["tr_n2h"], G["tr_x"])
    eq(be.get(be.transpose(x, 2, [0, 1, [-1, 2], 3], 2)), G["tr_d2h"])
    eq(be.get(be.permute_flat(x, [2, 4, 3, 2, 4, 2], [3, 5, 0, 1, 2, 4])).reshape(8, 4, 3, 4),
       G["tr_s2b"])
    eq(be.get(be.transpose(x, -1, [0, 2, 3, 1], 2)), G["tr_nhwc"])
    # split / concat / pad / slice / extend
    z = be.put(G["lay_x"])
    parts = be.split(z, 1, sizes=[2, 1, 3])
    for i, p in enumerate(parts):
        eq(be.get(p), G[f"lay_split_{i}"])
    eq(be.get(be.concat([z, parts[0]], 1)), G["lay_concat"])
    eq(be.get(be.pad(z, [0, 1, 2, 0], [0, 0, 1, 3])), G["lay_pad"])
    eq(be.get(be.slice_(z, [0, 1, 2, 0], [0, 1, 1, 1])), G["lay_slice"])
    eq(be.get(be.extend(z, 1, 2)), G["lay_extend"])
    # powers, division, gather (index dims first), mean over an axis
    e = be.put(G["elt_x"])
    eq(be.get(be.pow_(e, 3)), G["elt_pow3"])
    eq(be.get(be.div(e, be.put(G["elt_d"]))), G["elt_div"])
    tab, idx = be.put(G["ga_x"]), be.put_idx(G["ga_idx"])
    eq(be.get(be.gather(tab, idx, 0)), G["ga_axis0"])
    eq(be.get(be.gather(tab, idx, 1)), G["ga_axis1"])
    r = be.put(G["rm_x"])
    eq(be.get(be.reduce_mean(r, 1)), G["rm_axis1"])
    eq(be.get(be.reduce_mean(r, 2)), G["rm_axis2"])
    # transposed convolution (torch's conv_transpose2d) and the band matmuls (dense numpy)
    for i in range(3):
        n, h, w, f, r_, s, c, ph, pw, sh, sw, dh, dw, oph, opw = (
            int(v) for v in G[f"convtrans_{i}_args"])
        y = be.get(be.conv_trans(be.put(G[f"convtrans_{i}_x"]), be.put(G[f"convtrans_{i}_w"]),
                                 ph, pw, sh, sw, dh, dw, oph, opw))
        eq(y, G[f"convtrans_{i}_y"])
        bs, m, k, w_, d = (int(v) for v in G[f"band_{i}_args"])
        A, B, P = (be.put(G[f"band_{i}_{k_}"]) for k_ in ("A", "B", "P"))
        eq(be.get(be.g2bmm(A, B, w_, d)), G[f"band_{i}_g2bmm"])
        eq(be.get(be.gbmml(P, B, d)), G[f"band_{i}_gbmml"])


def test_oracle_reproduces_golden_vectors():
    check_all(OracleBackend())


def test_oracle_uint32_tier_reproduces_golden_convs():
    """The reference computes in wrapping uint32 (include/common.h:137): the same
    integers in two's complement."""
    for i in range(N_CONV2D):
        n, c, h, w, f, cpg, r, s, ph, pw, sh, sw, dh, dw = (int(v) for v in G[f"conv2d_{i}_args"])
        xu = G[f"conv2d_{i}_x"].astype(np.int64).astype(np.uint32)
        wu = G[f"conv2d_{i}_w"].astype(np.int64).astype(np.uint32)
        y = oracle.conv2d(xu, wu, ph, pw, sh, sw, dh, dw)
        np.testing.assert_array_equal(y.view(np.int32).astype(np.float32), G[f"conv2d_{i}_y"])


@pytest.mark.gpu
def test_hip_reproduces_golden_vectors():
    check_all(HipBackend())
