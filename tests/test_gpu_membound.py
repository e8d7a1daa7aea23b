"""MemBound expressions on the GPU (pet_hip_expr_f32) against the CPU oracle's interpreter
and against numpy index maps; bad programs are refused before anything is launched."""
import numpy as np
import pytest
import torch

import oracle
from pet_amd.expr_programs import C, I, OPS, R, T, assemble
from test_oracle import _membound_cases

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


def test_expressions_match_oracle_and_numpy(ops):
    for name, shapes, top, inputs, want in _membound_cases(np.random.default_rng(9)):
        code = assemble(shapes, top)
        got = host(ops.expr(ops.ExprProgram(code), [dev(a) for a in inputs]))
        ref = oracle.expr(code, inputs)
        if inputs[0].dtype == np.float32 and np.all(inputs[0] == np.round(inputs[0])):
            np.testing.assert_array_equal(got, ref, err_msg=name)
        np.testing.assert_allclose(got, want, rtol=2e-6, atol=2e-6, err_msg=name)


def test_large_gather_is_bit_exact(ops):
    """A layout move at a real size (the dilated block's space-to-batch, 1x512x64x64) written
    as an expression equals the permute kernel's result bit for bit."""
    x = np.random.default_rng(1).standard_normal((1, 512, 64, 64)).astype(np.float32)
    top = R([("b", 0, 4), ("c", 0, 512), ("h", 0, 32), ("w", 0, 32)], [],
            T(0, [C(0), I("c"), I("h") * 2 + I("b") // 2, I("w") * 2 + I("b") % 2]))
    dx = dev(x)
    got = ops.expr(ops.ExprProgram(assemble([x.shape], top)), [dx])
    want = ops.permute_flat(dx, [1, 512, 32, 2, 32, 2], [3, 5, 0, 1, 2, 4]).view(4, 512, 32, 32)
    assert torch.equal(got, want)


def test_bad_programs_are_refused(ops):
    from pet_amd import abi
    good = assemble([(4,)], R([("i", 0, 4)], [], T(0, [I("i")])))
    for mutate in (lambda c: c[:-1],                                  # no END
                   lambda c: [0] + c[1:],                             # bad magic
                   lambda c: c[:-3] + [OPS["LOAD"], 5, OPS["END"]],   # tensor out of range
                   lambda c: c[:-1] + [99, OPS["END"]]):              # unknown opcode
        with pytest.raises(abi.PetHipError):
            ops.ExprProgram(mutate(list(good)))
