"""C++ host layer (tpm::Operator / Graph / PerfEngine / CodeEngine on the C ABI).

The GPU cases run the test driver built from tests/cpp/host_tests.cc (its cases
follow the reference's src/Test programs); the CPU cases check that the host
library builds, links only against the C ABI and exports the reference's
operator classes."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "pet_amd", "lib")
DRIVER = os.path.join(LIB, "pet_host_tests")
HOST_LIB = os.path.join(LIB, "libpet_host.so")

CASES = ["conv_vs_oracle", "conv_invalid_groups", "transpose_n2h_h2n", "batch_gemm_merge",
         "pad_conv_slice_verification", "corrected_h2n_program",
         "dilated_space_to_batch_program", "code_engine_graph_runtime", "perf_engine_memo",
         "split_ratio_and_eltwise", "conv_merge_programs"]


def test_host_library_is_built_and_exports_the_operator_classes():
    assert os.path.exists(HOST_LIB), "run __graft_entry__.build() first"
    out = subprocess.run(["nm", "-DC", "--defined-only", HOST_LIB], capture_output=True,
                         text=True, check=True).stdout
    for sym in ["tpm::ConvOp::compute", "tpm::MatmulOp::perf", "tpm::TransposeOp::getTTParam",
                "tpm::SplitOp::computeV", "tpm::ConcatOp::launch", "tpm::Graph::conv",
                "tpm::SubGraph::verification", "tpm::PerfEngine::PerfEngine",
                "tpm::CodeEngine::genCode", "tpm::CodeEngine::instantiate",
                "tpm::TransposeEngine::lower"]:
        assert sym in out, sym


def test_host_library_reaches_the_device_only_through_the_c_abi():
    out = subprocess.run(["nm", "-D", "--undefined-only", HOST_LIB], capture_output=True,
                         text=True, check=True).stdout
    undefined = [l.split()[-1] for l in out.splitlines() if l.strip()]
    assert any(u.startswith("pet_hip_") for u in undefined)
    assert not [u for u in undefined if u.startswith("hip") or u.startswith("oracle_")]


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES)
def test_host_driver_case(case):
    assert os.path.exists(DRIVER), "run __graft_entry__.build() first"
    res = subprocess.run([DRIVER, case], capture_output=True, text=True, timeout=300)
    print(res.stdout)
    print(res.stderr)
    assert res.returncode == 0, res.stdout + res.stderr


@pytest.mark.gpu
def test_emitted_program_compiles_and_runs(tmp_path):
    src = tmp_path / "emitted.cpp"
    res = subprocess.run([DRIVER, "emit_program", str(src)], capture_output=True, text=True,
                         timeout=300)
    assert res.returncode == 0, res.stdout + res.stderr
    exe = tmp_path / "emitted"
    subprocess.run(["g++", "-O1", str(src), "-I", os.path.join(ROOT, "include"), "-L", LIB,
                    "-lpet_hip", "-Wl,-rpath," + LIB, "-o", str(exe)], check=True)
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stdout + run.stderr
    assert "Time(ms)" in run.stdout
