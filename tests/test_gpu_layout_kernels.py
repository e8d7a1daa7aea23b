"""Bit-exact checks of every kernel the layout engine can pick, with shapes chosen
to land on each one (and on its ragged / unaligned fall-backs): direct copies
with 1 and 4 items per thread, streaming (non-temporal) variants, the 2- and
4-wide interleave kernels behind space-to-batch, the packed-store gather, and
the LDS-tiled transposes with 16-byte access on either, both or neither side."""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from pet_amd import ops as _ops
    return _ops


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def iota(shape):
    # distinct values, exact in fp32 up to 2^24 elements; beyond that a second
    # pattern keeps neighbours distinguishable
    n = int(np.prod(shape))
    a = np.arange(n, dtype=np.int64)
    return ((a % 16777213) - 8388606).astype(np.float32).reshape(shape)


def check_perm(ops, flat, perm):
    x = iota(flat)
    ref = oracle.permute_flat(x, list(flat), list(perm))
    got = host(ops.permute_flat(dev(x), list(flat), list(perm)))
    assert got.shape == ref.shape
    assert got.tobytes() == ref.tobytes()


S2B = [3, 5, 0, 1, 2, 4]   # [n, c, h/d, d, w/d, d] -> [d, d, n, c, h/d, w/d]
B2S = [2, 3, 4, 0, 5, 1]   # [d, d, n, c, h/d, w/d] -> [n, c, h/d, d, w/d, d]


@pytest.mark.parametrize("n,c,h,w,d", [
    (1, 8, 16, 16, 2),     # 2-wide interleave kernel
    (2, 3, 6, 24, 2),
    (1, 5, 4, 8, 2),
    (1, 8, 16, 12, 2),     # w/d = 6: not a multiple of 4 -> tiled / direct fall-back
    (1, 4, 6, 10, 2),
    (1, 8, 16, 16, 4),     # 4-wide interleave kernel
    (2, 3, 8, 32, 4),
    (1, 4, 8, 24, 4),      # w/d = 6 -> fall-back
    (1, 6, 12, 12, 3),     # dilation 3: never the interleave kernels
    (1, 512, 64, 64, 2),   # the bench shape
])
def test_space_to_batch_and_back(ops, n, c, h, w, d):
    check_perm(ops, [n, c, h // d, d, w // d, d], S2B)
    check_perm(ops, [d, d, n, c, h // d, w // d], B2S)


def test_interleave_streaming_variants_round_trip(ops):
    """32 Mi elements: the non-temporal variants. Checked against the oracle on the
    forward pass and by the round trip."""
    n, c, h, w, d = 2, 256, 256, 256, 2
    flat = [n, c, h // d, d, w // d, d]
    x = iota(flat)
    ref = oracle.permute_flat(x, flat, S2B)
    dx = dev(x)
    y = ops.permute_flat(dx, flat, S2B)
    assert host(y).tobytes() == ref.tobytes()
    back = ops.permute_flat(y, [d, d, n, c, h // d, w // d], B2S)
    assert torch.equal(back.reshape(-1), dx.reshape(-1))
    del y, back
    d = 4
    flat = [n, c, h // d, d, w // d, d]
    y = ops.permute_flat(dx.reshape(flat), flat, S2B)
    assert host(y).tobytes() == oracle.permute_flat(x.reshape(flat), flat, S2B).tobytes()
    back = ops.permute_flat(y, [d, d, n, c, h // d, w // d], B2S)
    assert torch.equal(back.reshape(-1), dx.reshape(-1))


@pytest.mark.parametrize("flat,perm", [
    ([33, 65], [1, 0]),                    # scalar tiled, ragged both ways
    ([64, 64], [1, 0]),                    # 16 bytes on both sides
    ([1000, 1000], [1, 0]),
    ([128, 66], [1, 0]),                   # 16 bytes on the input side only (66 % 4 != 0 out rows)
    ([66, 128], [1, 0]),                   # ... on the output side only
    ([5, 300, 70], [2, 0, 1]),
    ([12, 128, 64], [0, 2, 1]),            # matmul operand transpose
    ([7, 9, 11, 13], [3, 2, 1, 0]),        # 4 tile dims
    ([4, 6, 8, 10, 12], [4, 2, 0, 3, 1]),
    ([2048, 4100], [1, 0]),                # 8.4 Mi elements: 8192-element tiles, ragged edge
    ([64, 256, 1024], [0, 2, 1]),          # 16 Mi elements, NCHW -> NHWC
])
def test_tiled_transposes(ops, flat, perm):
    check_perm(ops, flat, perm)


@pytest.mark.parametrize("flat,perm", [
    ([4, 64, 2, 28, 56], [2, 0, 1, 3, 4]),      # H2N: outer-dim move, 16-byte direct copy
    ([128, 12, 64], [1, 0, 2]),                 # attention head split
    ([16, 64, 2, 64, 128], [2, 0, 1, 3, 4]),    # 16 Mi elements: four items per thread
    ([3, 5, 7, 9], [1, 0, 2, 3]),               # innermost extent 9: scalar direct / gather
    ([6, 10, 14, 14], [1, 0, 2, 3]),            # innermost rows of 14*14 = 196 (merged), aligned
    ([6, 10, 7, 7], [1, 0, 2, 3]),              # 49-element rows: unaligned gather
])
def test_direct_copies(ops, flat, perm):
    check_perm(ops, flat, perm)


def test_direct_streaming_variant(ops):
    flat, perm = [32, 2, 64, 64, 128], [1, 0, 2, 3, 4]   # 32 Mi elements
    check_perm(ops, flat, perm)


@pytest.mark.parametrize("shape,begin,end", [
    ((2, 3, 14, 14), (0, 0, 1, 1), (0, 0, 1, 1)),        # 16-wide output rows, 14-wide input
    ((2, 3, 13, 11), (0, 0, 2, 3), (0, 0, 0, 2)),        # 16-wide output rows, odd input
    ((4, 8, 30, 30), (0, 0, 1, 1), (0, 0, 1, 1)),
    ((1, 64, 126, 126), (0, 0, 1, 1), (0, 0, 1, 1)),     # 1 Mi outputs
    ((3, 5, 7), (1, 0, 1), (0, 2, 0)),                   # output rows of 8
    ((3, 5, 7), (1, 1, 1), (1, 1, 1)),                   # output rows of 9: scalar path
])
def test_pad_then_slice_back(ops, shape, begin, end):
    x = iota(shape)
    ref = oracle.pad(x, list(begin), list(end))
    p = ops.pad(dev(x), list(begin), list(end))
    assert host(p).tobytes() == ref.tobytes()
    back = ops.slice_(p, list(begin), list(end))
    assert host(back).tobytes() == x.tobytes()


@pytest.mark.parametrize("shape,begin,end", [
    ((8, 16, 30), (0, 0, 1), (0, 0, 1)),                 # rows of 30 -> 32: one row per 8 words
    ((8, 16, 33), (0, 0, 0), (0, 0, -1)),                # crop the last column: rows of 32 from 33
    ((4, 7, 9, 19), (0, 1, 2, -1), (1, 0, -1, -2)),      # pad and crop mixed, odd rows of 16
    ((3, 4100), (0, 2), (1, 2)),                         # rows longer than a staging tile
    ((2, 9001), (0, -1), (0, 0)),                        # ... and odd, cropped in front
    ((5, 3, 126, 126), (0, 0, 1, 1), (0, 0, 1, 1)),
    ((5, 3, 128, 128), (0, 0, -1, -1), (0, 0, -1, -1)),
    ((2, 2, 64, 130), (1, 0, 0, -3), (0, 1, 0, -3)),     # whole zero planes around cropped rows
    ((33, 257, 129), (0, 0, -1), (0, 0, 0)),             # > 1 Mi outputs
])
def test_row_staged_windows(ops, shape, begin, end):
    """Dense output whose rows are pieces of input rows at any dword alignment: the
    LDS-staged kernel (aligned 16-byte words on both global sides). Negative
    amounts crop. Also through an input that starts 4 bytes into its buffer,
    which must take the element-wise kernel and give the same bytes."""
    x = iota(shape)
    ref = x
    for d, (b, e) in enumerate(zip(begin, end)):
        idx = [slice(None)] * ref.ndim
        idx[d] = slice(max(0, -b), ref.shape[d] - max(0, -e))
        ref = ref[tuple(idx)]
        widths = [(0, 0)] * ref.ndim
        widths[d] = (max(0, b), max(0, e))
        ref = np.pad(ref, widths)
    ref = np.ascontiguousarray(ref)

    def run(xd):
        cb, ce = [max(0, -b) for b in begin], [max(0, -e) for e in end]
        pb, pe = [max(0, b) for b in begin], [max(0, e) for e in end]
        t = ops.slice_(xd, cb, ce) if any(cb) or any(ce) else xd
        return ops.pad(t, pb, pe) if any(pb) or any(pe) else t

    assert host(run(dev(x))).tobytes() == ref.tobytes()
    shifted = torch.empty(x.size + 1, dtype=torch.float32, device="cuda")
    shifted[1:] = dev(x).reshape(-1)
    assert host(run(shifted[1:].reshape(shape))).tobytes() == ref.tobytes()


def test_row_staged_streaming_variant(ops):
    x = iota((64, 64, 126, 126))                         # 65 Mi elements: non-temporal variant
    p = ops.pad(dev(x), [0, 0, 1, 1], [0, 0, 1, 1])
    back = ops.slice_(p, [0, 0, 1, 1], [0, 0, 1, 1])
    assert host(back).tobytes() == x.tobytes()
    ph = host(p)
    assert not ph[:, :, 0, :].any() and not ph[:, :, :, 127].any()
    assert ph[:, :, 1:127, 1:127].tobytes() == x.tobytes()


@pytest.mark.parametrize("shape,dim,num", [((2, 6, 7, 7), 1, 2), ((4, 8, 16), 0, 1), ((3, 5, 12), 2, 3)])
def test_extend(ops, shape, dim, num):
    x = iota(shape)
    assert host(ops.extend(dev(x), dim, num)).tobytes() == oracle.extend(x, dim, num).tobytes()


def test_halo_chain_on_width(ops):
    """W2N with a one-column halo, then N2W dropping it: the gather path with a
    window that cuts through rows."""
    x = iota((2, 4, 12, 16))
    chain = [("split", 3, 8, 0, 1), ("reorder", [0, 3, 1, 2, 4]), ("fuse", 0, 0, 0)]
    ref = oracle.trans_chain(x, chain)
    got = host(ops.trans_chain(dev(x), chain))
    assert got.shape == ref.shape and got.tobytes() == ref.tobytes()


@pytest.mark.parametrize("n,c,h,w,d", [(1, 8, 16, 16, 2), (2, 3, 12, 18, 3), (1, 64, 64, 64, 2),
                                        (3, 5, 8, 20, 4)])
def test_chained_transposes_fold_into_one_view(ops, n, c, h, w, d):
    """Space-to-batch written as two transposes in a row (rows, then columns, each
    de-interleaved into the batch) and its inverse, each sent as one micro-op
    chain: the output dim 0 is fused twice, which only the factor-wise chain
    compiler turns into a strided view. Expected values from numpy."""
    x = iota((n, c, h, w))
    fwd = [("split", 2, d, 0, 0), ("reorder", [3, 0, 1, 2, 4]), ("fuse", 0, 0, 0),
           ("split", 3, d, 0, 0), ("reorder", [4, 0, 1, 2, 3]), ("fuse", 0, 0, 0)]
    ref = (x.reshape(n, c, h // d, d, w // d, d).transpose(5, 3, 0, 1, 2, 4)
           .reshape(d * d * n, c, h // d, w // d))
    assert oracle.trans_chain(x, fwd).tobytes() == ref.tobytes()
    got = ops.trans_chain(dev(x), fwd)
    assert host(got).shape == ref.shape and host(got).tobytes() == ref.tobytes()
    # back: the column phase leaves the batch first, then the row phase
    inv = [("split", 0, d * n, 0, 0), ("reorder", [1, 2, 3, 4, 0]), ("fuse", 3, 0, 0),
           ("split", 0, n, 0, 0), ("reorder", [1, 2, 3, 0, 4]), ("fuse", 2, 0, 0)]
    back = ops.trans_chain(got, inv)
    assert host(back).shape == x.shape and host(back).tobytes() == x.tobytes()


def test_random_permutes_pads_slices_against_numpy(ops):
    """300 seeded random cases across the kernel-selection boundaries: ranks 2-6,
    extents mixing multiples of 4, of 2 and odd numbers, any permutation; then a
    random pad and the slice that undoes it. Expected values from numpy itself."""
    rng = np.random.default_rng(2024)
    pool = [1, 2, 3, 4, 5, 6, 7, 8, 12, 16, 17, 24, 32, 33, 64]
    for case in range(300):
        rank = int(rng.integers(2, 7))
        dims = [int(rng.choice(pool)) for _ in range(rank)]
        while np.prod(dims) > 1 << 18:
            dims[int(rng.integers(0, rank))] = 2
        perm = [int(v) for v in rng.permutation(rank)]
        x = iota(dims)
        ref = np.ascontiguousarray(x.transpose(perm))
        got = host(ops.permute_flat(dev(x), dims, perm))
        assert got.tobytes() == ref.tobytes(), ("permute", case, dims, perm)
        begin = [int(rng.integers(0, 3)) for _ in range(rank)]
        end = [int(rng.integers(0, 3)) for _ in range(rank)]
        refp = np.pad(x, list(zip(begin, end)))
        p = ops.pad(dev(x), begin, end)
        assert host(p).tobytes() == refp.tobytes(), ("pad", case, dims, begin, end)
        assert host(ops.slice_(p, begin, end)).tobytes() == x.tobytes(), ("slice", case, dims)
