"""pet_hip_conv2d_static_f32, the entry point that allocates nothing: its split-K
scratch is a static device array inside the library. Checked through the C ABI
against pet_hip_conv2d_f32 on two calls in a row, the second on a smaller input
(the array keeps the first call's contents)."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _conv(entry, x, w, bias, pad, act):
    import torch
    from pet_amd import abi
    n, c, h, wd = x.shape
    f, cpg, r, s = w.shape
    y = torch.empty((n, f, h + 2 * pad - r + 1, wd + 2 * pad - s + 1), device=x.device)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: ctypes.c_void_p(0 if t is None else t.data_ptr())
    abi.call(entry, p(x), p(w), p(bias), p(y), n, c, h, wd, f, r, s, pad, pad, 1, 1, 1, 1,
             c // cpg, abi.ACT[act], st)
    torch.cuda.synchronize()
    return y.cpu().numpy()


def test_static_scratch_conv_matches_the_allocating_entry_point_twice_in_a_row():
    import torch
    from pet_amd import abi
    abi.init(0)
    rng = np.random.default_rng(7)
    # both shapes split their K loop (few output tiles, long K): 256->256 on 14x14,
    # then the smaller 128->128 on 14x14, whose tiles reuse the first call's scratch
    shapes = [((1, 256, 14, 14), (256, 256, 3, 3)), ((1, 128, 14, 14), (128, 128, 3, 3))]
    before = ctypes.c_int(0)
    abi.call("pet_hip_get_deterministic", ctypes.byref(before))
    try:
        for xs, wsh in shapes:
            # integer tier: every sum is exact, so the two entry points agree bit for bit
            # whatever order they add in
            xi = torch.from_numpy(rng.integers(-3, 4, xs).astype(np.float32)).cuda()
            wi = torch.from_numpy(rng.integers(-3, 4, wsh).astype(np.float32)).cuda()
            bi = torch.from_numpy(rng.integers(-3, 4, wsh[0]).astype(np.float32)).cuda()
            abi.call("pet_hip_set_deterministic", 0)
            ref = _conv("pet_hip_conv2d_f32", xi, wi, bi, 1, "relu")
            got = _conv("pet_hip_conv2d_static_f32", xi, wi, bi, 1, "relu")
            assert np.array_equal(got, ref)
            # real-valued tier: against the allocating entry point in its ordered form,
            # within the contraction tolerance of 1e-4 of the output's magnitude
            xf = torch.from_numpy(rng.standard_normal(xs).astype(np.float32)).cuda()
            wf = torch.from_numpy((0.05 * rng.standard_normal(wsh)).astype(np.float32)).cuda()
            abi.call("pet_hip_set_deterministic", 1)
            ref = _conv("pet_hip_conv2d_f32", xf, wf, None, 1, "none")
            got = _conv("pet_hip_conv2d_static_f32", xf, wf, None, 1, "none")
            assert np.abs(got - ref).max() <= 1e-4 * np.abs(ref).max()
            # ... and it is reproducible from call to call
            again = _conv("pet_hip_conv2d_static_f32", xf, wf, None, 1, "none")
            assert np.array_equal(got, again)
    finally:
        abi.call("pet_hip_set_deterministic", before.value)


REFUSAL_PROGRAM = r"""
import ctypes, sys, torch
from pet_amd import abi
abi.init(0)
x = torch.zeros((1, 512, 14, 14), device="cuda")
w = torch.zeros((512, 512, 3, 3), device="cuda")
y = torch.empty((1, 512, 14, 14), device="cuda")
st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
p = lambda t: ctypes.c_void_p(t.data_ptr())
rc = abi.status("pet_hip_conv2d_static_f32", p(x), p(w), None, p(y), 1, 512, 14, 14, 512, 3, 3,
                1, 1, 1, 1, 1, 1, 1, 0, st)
torch.cuda.synchronize()
print("rc", rc, abi.last_error())
sys.exit(0 if rc == 2 and "static scratch" in abi.last_error() else 1)
"""


def test_static_scratch_conv_refuses_what_does_not_fit():
    """With the K loop forced into 64 shares (PET_HIP_SPLITK, read when the library
    loads, hence the child process) 32 tiles need 32 MiB of partial tiles: refused with
    PET_HIP_ERR_UNSUPPORTED and the sizes in the error text, nothing launched."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, PET_HIP_SPLITK="64", PYTHONPATH=root)
    res = subprocess.run([sys.executable, "-c", REFUSAL_PROGRAM], capture_output=True, text=True,
                         timeout=300, env=env, cwd=root)
    print(res.stdout, res.stderr[-2000:])
    assert res.returncode == 0
