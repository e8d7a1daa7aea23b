"""Writes the golden vectors under tests/golden/.

Inputs are small integers (every contraction below stays exact in fp32), expected
outputs come from routines that share no code with the oracle or the HIP library:
torch's CPU convolutions and numpy's matmul / reshape / transpose / pad / split /
concatenate / tile / take / mean and integer powers, torch's conv_transpose2d, and band
products cut out of numpy's dense matmul. The transposes are the reference's own closed form
(reshape -> transpose -> reshape, src/Test/dat/transpose_test/transpose_ops.op:1-3
and src/Test/transpose_test_2.py:4-31) on an iota input (src/Test/transpose_test_2.cc:24);
the matmul triple is the reference's batch-GEMM merge case
(src/Test/batch_gemm_test.cc:9,45-50: m = n = 8, k = 4, A = iota, W0 = 3*iota, W1 = 7*iota).

Run from the repository root:  python tests/golden/make_golden.py
"""
import os

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))
rng = np.random.default_rng(20240607)


def ints(shape, lo=-3, hi=4):
    return rng.integers(lo, hi, size=shape).astype(np.float32)


def main():
    out = {}
    # ---- conv2d: (n, c, h, w, f, cpg, r, s, ph, pw, sh, sw, dh, dw)
    conv2d = [
        (1, 4, 9, 9, 6, 4, 3, 3, 1, 1, 1, 1, 1, 1),
        (1, 8, 12, 12, 8, 8, 3, 3, 2, 2, 1, 1, 2, 2),   # dilated (config 2 style)
        (1, 8, 10, 10, 12, 2, 3, 3, 1, 1, 1, 1, 1, 1),  # 4 groups
        (1, 3, 20, 20, 4, 3, 7, 7, 3, 3, 2, 2, 1, 1),   # 7x7 stride 2 stem
        (1, 5, 14, 14, 7, 5, 1, 1, 0, 0, 2, 2, 1, 1),   # 1x1 stride 2
        (2, 16, 8, 8, 8, 16, 3, 3, 1, 1, 1, 1, 1, 1),   # batch 2, 8-divisible channels
    ]
    for i, cs in enumerate(conv2d):
        n, c, h, w, f, cpg, r, s, ph, pw, sh, sw, dh, dw = cs
        x, wt = ints((n, c, h, w)), ints((f, cpg, r, s))
        y = F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(wt).double(), padding=(ph, pw),
                     stride=(sh, sw), dilation=(dh, dw), groups=c // cpg).numpy().astype(np.float32)
        out[f"conv2d_{i}_args"] = np.array(cs, np.int32)
        out[f"conv2d_{i}_x"], out[f"conv2d_{i}_w"], out[f"conv2d_{i}_y"] = x, wt, y
    # ---- conv3d: (n, c, t, h, w, f, cpg, kt, r, s) + pad, stride, dilation triples
    conv3d = [
        ((1, 3, 6, 10, 10, 4, 3, 3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),
        ((1, 8, 4, 9, 9, 8, 8, 3, 3, 3), (1, 1, 1), (2, 2, 2), (1, 1, 1)),
        ((1, 4, 6, 8, 8, 4, 2, 3, 3, 3), (2, 2, 2), (1, 1, 1), (2, 2, 2)),
    ]
    for i, (cs, pad, st, dil) in enumerate(conv3d):
        n, c, t, h, w, f, cpg, kt, r, s = cs
        x, wt = ints((n, c, t, h, w)), ints((f, cpg, kt, r, s))
        y = F.conv3d(torch.from_numpy(x).double(), torch.from_numpy(wt).double(), padding=pad,
                     stride=st, dilation=dil, groups=c // cpg).numpy().astype(np.float32)
        out[f"conv3d_{i}_args"] = np.array(list(cs) + list(pad) + list(st) + list(dil), np.int32)
        out[f"conv3d_{i}_x"], out[f"conv3d_{i}_w"], out[f"conv3d_{i}_y"] = x, wt, y
    # ---- matmul: the reference's merge case and all four transpose combinations
    m, n, k = 8, 8, 4
    A = np.arange(m * k, dtype=np.float32).reshape(1, m, k)
    W0 = 3 * np.arange(k * n, dtype=np.float32).reshape(1, k, n)
    W1 = 7 * np.arange(k * n, dtype=np.float32).reshape(1, k, n)
    out["mm_merge_A"], out["mm_merge_W0"], out["mm_merge_W1"] = A, W0, W1
    out["mm_merge_Y0"], out["mm_merge_Y1"] = np.matmul(A, W0), np.matmul(A, W1)
    a, b = ints((3, 5, 7)), ints((3, 7, 6))
    out["mm_t_A"], out["mm_t_B"], out["mm_t_Y"] = a, b, np.matmul(a, b)
    out["mm_t_At"] = np.ascontiguousarray(a.transpose(0, 2, 1))
    out["mm_t_Bt"] = np.ascontiguousarray(b.transpose(0, 2, 1))
    # ---- transposes by the reference's closed form, iota input
    x = np.arange(2 * 4 * 6 * 8, dtype=np.float32).reshape(2, 4, 6, 8)
    out["tr_x"] = x
    # H2N (nm2_hd2 in src/Test/transpose_test_2.py:26-31): split H by 2, the upper
    # factor joins N with N as the major index  ->  [2N, C, H/2, W]
    out["tr_h2n"] = x.reshape(2, 4, 2, 3, 8).transpose(0, 2, 1, 3, 4).reshape(4, 4, 3, 8)
    # N2H (nd2_hm2, transpose_test_2.py:19-24; transpose_ops.op:1-3): the inverse
    out["tr_n2h"] = out["tr_h2n"].reshape(2, 2, 4, 3, 8).transpose(0, 2, 1, 3, 4).reshape(2, 4, 6, 8)
    # D2H (h_d2_d1, transpose_test_2.py:4-9): [H/2, 2] -> [2, H/2] inside H
    out["tr_d2h"] = x.reshape(2, 4, 3, 2, 8).transpose(0, 1, 3, 2, 4).reshape(2, 4, 6, 8)
    # space-to-batch with dilation 2 on H and W  ->  [4N, C, H/2, W/2]
    out["tr_s2b"] = x.reshape(2, 4, 3, 2, 4, 2).transpose(3, 5, 0, 1, 2, 4).reshape(8, 4, 3, 4)
    # plain permutation NCHW -> NHWC
    out["tr_nhwc"] = np.ascontiguousarray(x.transpose(0, 2, 3, 1))
    # ---- split / concat / pad / slice / extend
    z = ints((2, 6, 5, 4))
    out["lay_x"] = z
    parts = np.split(z, [2, 3], axis=1)  # sizes 2, 1, 3
    for i, p in enumerate(parts):
        out[f"lay_split_{i}"] = np.ascontiguousarray(p)
    out["lay_concat"] = np.concatenate([z, z[:, :2]], axis=1)
    out["lay_pad"] = np.pad(z, [(0, 0), (1, 0), (2, 1), (0, 3)])
    out["lay_slice"] = np.ascontiguousarray(z[:, 1:5, 2:4, :3])  # begin (0,1,2,0), end (0,1,1,1)
    out["lay_extend"] = np.concatenate([z, z, z], axis=1)        # extend dim 1 by 2 copies
    # ---- element-wise powers and division, gather, mean over an axis (all exact)
    e = ints((3, 4, 5))
    d = np.array([2, -4, 0.5, 8, -1], np.float32)
    out["elt_x"], out["elt_pow3"], out["elt_d"], out["elt_div"] = e, e ** 3, d, e / d
    tab, idx = ints((7, 6)), np.array([[5, 0, 3], [2, 2, -1]], np.int32)
    out["ga_x"], out["ga_idx"] = tab, idx
    out["ga_axis0"] = tab[idx % 7]                                        # [2, 3, 6]
    out["ga_axis1"] = np.ascontiguousarray(np.moveaxis(tab[:, idx % 6], 0, 2))  # [2, 3, 7]
    r = ints((2, 8, 4))
    out["rm_x"] = r
    out["rm_axis1"], out["rm_axis2"] = r.mean(axis=1, keepdims=True), r.mean(axis=2, keepdims=True)
    # ---- transposed convolution (x NHWF, w RSFC, y NHWC) against torch's conv_transpose2d,
    # which takes NCHW input and [in, out, kh, kw] filters. Dilation 1 only: with dilation the
    # reference's loop nest (src/Graph/operator.cc:961-962) keeps the undilated offset
    # r - ph - 1 and is an operator of its own, which no library routine restates.
    # (n, h, w, f, r, s, c, ph, pw, sh, sw, dh, dw, oph, opw)
    conv_trans = [
        (1, 4, 5, 3, 3, 3, 4, 1, 1, 2, 2, 1, 1, 0, 0),
        (2, 3, 3, 8, 4, 4, 5, 1, 1, 2, 2, 1, 1, 1, 1),
        (1, 5, 4, 2, 3, 2, 3, 0, 1, 1, 1, 1, 1, 0, 0),
    ]
    for i, cs in enumerate(conv_trans):
        n, h, w, f, r, s, c, ph, pw, sh, sw, dh, dw, oph, opw = cs
        x, wt = ints((n, h, w, f)), ints((r, s, f, c))
        y = F.conv_transpose2d(torch.from_numpy(x).double().permute(0, 3, 1, 2),
                               torch.from_numpy(wt).double().permute(2, 3, 0, 1),
                               stride=(sh, sw), padding=(ph, pw), output_padding=(oph, opw),
                               dilation=(dh, dw)).permute(0, 2, 3, 1).contiguous().numpy()
        out[f"convtrans_{i}_args"] = np.array(cs, np.int32)
        out[f"convtrans_{i}_x"], out[f"convtrans_{i}_w"] = x, wt
        out[f"convtrans_{i}_y"] = y.astype(np.float32)
    # ---- band matmuls from the dense product: G2BMM[b,i,j] = (A B^T)[b, i, i + d (j - w)],
    # GBMML[b,i,:] = sum_j band[b,i,j] B[b, i + d (j - w), :], rows outside the matrix are zero
    # (bs, m, k, w, d)
    for i, (bs, m, k, w, d) in enumerate([(2, 11, 6, 2, 1), (1, 13, 8, 3, 2), (2, 40, 32, 5, 3)]):
        A, B = ints((bs, m, k)), ints((bs, m, k))
        dense = np.matmul(A, B.transpose(0, 2, 1))
        band = np.zeros((bs, m, 2 * w + 1), np.float32)
        P = ints((bs, m, 2 * w + 1))
        ctx = np.zeros((bs, m, k), np.float32)
        for r_ in range(m):
            for j in range(2 * w + 1):
                col = r_ + d * (j - w)
                if 0 <= col < m:
                    band[:, r_, j] = dense[:, r_, col]
                    ctx[:, r_, :] += P[:, r_, j:j + 1] * B[:, col, :]
        out[f"band_{i}_args"] = np.array([bs, m, k, w, d], np.int32)
        out[f"band_{i}_A"], out[f"band_{i}_B"], out[f"band_{i}_g2bmm"] = A, B, band
        out[f"band_{i}_P"], out[f"band_{i}_gbmml"] = P, ctx
    np.savez_compressed(os.path.join(HERE, "golden.npz"), **out)
    print("wrote", os.path.join(HERE, "golden.npz"), len(out), "arrays")


if __name__ == "__main__":
    main()
