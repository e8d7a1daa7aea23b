"""The fused attention launch against the operator sequence it stands for (head split,
scores, scale, softmax, probabilities x values, head merge), evaluated by the CPU oracle
one reference operator at a time."""
import numpy as np
import pytest
import torch

import oracle
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


CASES = [
    # heads, seq, dh
    (12, 128, 64),     # benchmark configuration 4 (BERT-base, sequence 128)
    (4, 77, 32),       # ragged query block and key block
    (2, 512, 128),     # the largest supported shape: 16 waves per workgroup
    (3, 33, 96),
    (1, 1, 64),
    (16, 256, 64),
]


@pytest.mark.parametrize("heads,seq,dh", CASES)
def test_attention_matches_the_operator_sequence(ops, heads, seq, dh):
    rng = np.random.default_rng(heads * 1000 + seq + dh)
    q, k, v = (rng.standard_normal((seq, heads * dh)).astype(np.float32) for _ in range(3))
    scale = 1.0 / np.sqrt(dh)
    ref = oracle.attention(q, k, v, heads, scale)
    mag = oracle.attention(q, k, np.abs(v), heads, scale)
    got = host(ops.attention(dev(q), dev(k), dev(v), heads, scale))
    assert got.shape == ref.shape
    assert max_rel_err(got, ref, mag) <= REL_TOL


def test_attention_over_a_batch_of_sequences(ops):
    """[batch, seq, heads*dh] operands: every batch entry is an attention of its own."""
    batch, heads, seq, dh = 3, 4, 70, 32
    rng = np.random.default_rng(5)
    q, k, v = (rng.standard_normal((batch, seq, heads * dh)).astype(np.float32) for _ in range(3))
    scale = 1.0 / np.sqrt(dh)
    got = host(ops.attention(dev(q), dev(k), dev(v), heads, scale))
    assert got.shape == (batch, seq, heads * dh)
    for b in range(batch):
        ref = oracle.attention(q[b], k[b], v[b], heads, scale)
        mag = oracle.attention(q[b], k[b], np.abs(v[b]), heads, scale)
        assert max_rel_err(got[b], ref, mag) <= REL_TOL


def test_attention_reads_the_slabs_of_a_merged_projection_in_place(ops):
    """Q, K and V as the three [seq, hidden] slabs of one [3, seq, hidden] tensor and as
    column blocks of one [seq, 3*hidden] tensor (row stride 3*hidden); the scale from a
    one-element device tensor, as the graph holds it."""
    heads, seq, dh = 12, 128, 64
    rng = np.random.default_rng(2)
    qkv = rng.standard_normal((3, seq, heads * dh)).astype(np.float32)
    ref = oracle.attention(qkv[0], qkv[1], qkv[2], heads, 0.125)
    mag = oracle.attention(qkv[0], qkv[1], np.abs(qkv[2]), heads, 0.125)
    d = dev(qkv)
    sc = dev(np.array([0.125], np.float32))
    got = host(ops.attention(d[0], d[1], d[2], heads, 1.0, scale_dev=sc))
    assert max_rel_err(got, ref, mag) <= REL_TOL
    wide = dev(np.concatenate([qkv[0], qkv[1], qkv[2]], axis=1))
    w = heads * dh
    got = host(ops.attention(wide[:, :w], wide[:, w:2 * w], wide[:, 2 * w:], heads, 0.125))
    assert max_rel_err(got, ref, mag) <= REL_TOL


def test_attention_exact_cases_pin_the_indexing(ops):
    """Two inputs whose softmax is exact in fp32. All-zero queries: every probability is
    1/seq (seq a power of two), so the output is the mean of the head's value rows, exact on
    small integers. One-hot scores: query i scores 200 against key perm[i] and 0 elsewhere,
    exp(-200) is 0 in fp32, so row i of the output is value row perm[i] bit for bit."""
    heads, seq, dh = 3, 64, 64
    rng = np.random.default_rng(4)
    v = rng.integers(-8, 9, (seq, heads * dh)).astype(np.float32)
    k = rng.standard_normal((seq, heads * dh)).astype(np.float32)
    got = host(ops.attention(dev(np.zeros_like(v)), dev(k), dev(v), heads, 1.0))
    want = np.broadcast_to(v.reshape(seq, heads, dh).mean(axis=0, keepdims=True),
                           (seq, heads, dh)).reshape(seq, heads * dh)
    np.testing.assert_array_equal(got, want.astype(np.float32))
    q = np.zeros((seq, heads * dh), np.float32)
    kk = np.zeros((seq, heads * dh), np.float32)
    want = np.empty_like(v)
    for h in range(heads):
        perm = rng.permutation(seq)
        for i in range(seq):
            kk[i, h * dh + i] = 200.0
            q[i, h * dh + perm[i]] = 1.0
            want[i, h * dh:(h + 1) * dh] = v[perm[i], h * dh:(h + 1) * dh]
    got = host(ops.attention(dev(q), dev(kk), dev(v), heads, 1.0))
    np.testing.assert_array_equal(got, want)


def test_attention_batched_and_refusals(ops):
    from pet_amd import abi
    rng = np.random.default_rng(6)
    x = rng.standard_normal((3, 3, 40, 4 * 32)).astype(np.float32)  # q/k/v, batch, seq, width
    got = host(ops.attention(dev(x[0]), dev(x[1]), dev(x[2]), 4, 0.2))
    for b in range(3):
        ref = oracle.attention(x[0, b], x[1, b], x[2, b], 4, 0.2)
        assert np.abs(got[b] - ref).max() <= 1e-4 * np.abs(ref).max()
    big = dev(np.zeros((600, 64), np.float32))
    with pytest.raises(abi.PetHipError) as err:
        ops.attention(big, big, big, 1, 1.0)
    assert err.value.status == 2
    odd = dev(np.zeros((8, 48), np.float32))
    with pytest.raises(abi.PetHipError):
        ops.attention(odd, odd, odd, 1, 1.0)   # head size 48
