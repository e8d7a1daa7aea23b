"""The C-ABI library loads without a GPU and exports every symbol that
include/pet_hip.h declares; compute calls refuse to run before pet_hip_init."""
import ctypes
import os
import re

import pytest

from pet_amd import abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "pet_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pet_hip_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_a_nontrivial_surface():
    syms = declared_symbols()
    assert len(syms) >= 35
    for must in ("pet_hip_conv2d_f32", "pet_hip_conv3d_f32", "pet_hip_bmm_f32",
                 "pet_hip_transpose", "pet_hip_trans_chain", "pet_hip_split",
                 "pet_hip_concat", "pet_hip_eltwise", "pet_hip_graph_launch"):
        assert must in syms


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(abi.LIB_PATH)
    missing = [s for s in declared_symbols() if not hasattr(lib, s)]
    assert not missing, missing


def test_binding_table_matches_header():
    bound = set(abi.SIGNATURES) | {"pet_hip_last_error"}
    assert bound == set(declared_symbols())


def test_conv_out_dim_needs_no_device():
    assert abi.status("pet_hip_conv_out_dim", 224, 7, 3, 2, 1) == 112
    assert abi.status("pet_hip_conv_out_dim", 16, 3, 0, 2, 2) == 7


def test_compute_calls_refuse_before_init():
    try:
        import torch
        if torch.cuda.is_available():
            pytest.skip("a GPU is present; init may already have happened")
    except ImportError:
        pass
    rc = abi.status("pet_hip_fill_f32", None, 0.0, 16, None)
    assert rc == 4
    assert "pet_hip_init" in abi.last_error()
