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
         "split_ratio_and_eltwise", "conv_merge_programs", "conv3d_prepacked_graph",
         "random_graphs_replay_equals_eager", "batchnorm_pow_div",
         "gather_reduce_mean", "launch_fusion_block", "alias_plan_shared_storage",
         "two_conv_verification", "convtrans_reference_vectors", "band_matmuls",
         "merged_projections", "merged_shortcut_block"]


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


# Programs under the reference's src/Test that use only the operator / graph /
# perf-engine surface this backend mirrors. Each must compile unchanged against
# pet_amd/host/include. The two headers they include for the search side
# (generator.h, search_engine.h) are outside this backend and are stood in for
# by empty files made at test time.
REFERENCE_PROGRAMS = [
    "SampleGraph3.cpp", "SampleGraph4.cpp", "batch_gemm_test.cc", "concat_test_1.cc",
    "conv_test_1.cc", "conv_test_2.cc", "conv_test_3.cc", "conv_test_4_perf.cc",
    "conv_test_5_trans_kernel.cc",
    "extend_test_1.cc", "gemm_test_1_perf.cc", "gemm_test_2_conv1x1_perf.cc",
    "group_conv_test_1.cc", "group_conv_test_2.cc", "mutant_test_2.cc", "pad_slice_test.cc",
    "perf_pool.cc", "split_test_1.cc", "split_test_2.cc", "tensor_test.cc",
    "transpose_test_1.cc", "transpose_test_2.cc", "transpose_test_3.cc", "transpose_test_4.cc",
    "transpose_test_5.cc",
]
# ... and programs that also drive the generator, the search engine and the code engine:
# they include the reference's own generator.h / search_engine.h (CMutator, nnet, ...),
# so they are only compiled where the whole search is built (pet_amd/host/Makefile) and
# run below, not syntax-checked here against empty stand-ins.
REFERENCE_TESTS = "/root/reference/src/Test"


@pytest.mark.skipif(not os.path.isdir(REFERENCE_TESTS), reason="reference sources not present")
@pytest.mark.parametrize("program", REFERENCE_PROGRAMS)
def test_reference_program_compiles_against_the_mirror_headers(program, tmp_path):
    for name in ("generator.h", "search_engine.h"):
        (tmp_path / name).write_text("#pragma once\n")
    res = subprocess.run(
        ["g++", "-std=c++17", "-fsyntax-only", "-w",
         "-I", os.path.join(ROOT, "pet_amd", "host", "include"),
         "-I", os.path.join(ROOT, "include"), "-I", str(tmp_path),
         os.path.join(REFERENCE_TESTS, program)],
        capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stderr[-2000:]


CURSOR_PROGRAM = r"""
#include "operator.h"
#include "tensor.h"
#include <cstdio>
int main() {
    tpm::Tensor t({2, 3, 4});
    size_t n = 0;
    for (t.itInit(); t.itValid(); t.itNext(), ++n)
        if (t.getOffset(t.itGet()) != n)
            return 1;
    if (n != 24)
        return 2;
    tpm::Tensor fresh;                      // no cursor before itInit on a shaped tensor
    fresh.setDims({5});
    if (fresh.itValid())
        return 3;
    tpm::Tensor in({1, 64, 162, 162});
    tpm::MaxPoolOp mp(&in, 3, 3, 1, 1, 0, 0, 2, 2);
    tpm::AvgPoolOp ap(&in, 3, 3, 0, 0, 2, 2);
    if (mp.getOutputs()[0]->getDims() != tpm::Dim{1, 64, 80, 80})
        return 4;
    if (ap.getOutputs()[0]->getDims() != tpm::Dim{1, 64, 80, 80})
        return 5;
    std::puts("ok");
    return 0;
}
"""


def test_tensor_cursor_and_pool_constructors_without_a_gpu(tmp_path):
    src = tmp_path / "cursor.cc"
    src.write_text(CURSOR_PROGRAM)
    exe = tmp_path / "cursor"
    subprocess.run(["g++", "-std=c++17", "-O1", str(src),
                    "-I", os.path.join(ROOT, "pet_amd", "host", "include"),
                    "-I", os.path.join(ROOT, "include"), "-L", LIB, "-lpet_host", "-lpet_hip",
                    "-Wl,-rpath," + LIB, "-o", str(exe)], check=True)
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert run.returncode == 0, (run.returncode, run.stdout, run.stderr)


# Prints, for every output point of a few operators, the linear offset of the
# input point the operator reports as its dependence (input index:offset).
DEPENDENCE_PROGRAM = r"""
#include "operator.h"
#include "tensor.h"
#include <cstdio>
using namespace tpm;
static void walk(const char *name, Operator *op, Tensor *out) {
    std::printf("%s", name);
    for (out->itInit(); out->itValid(); out->itNext()) {
        auto deps = op->compute(DimRange(out->itGet())).first;
        for (size_t i = 0; i < deps.size(); ++i)
            if (deps[i].isSinglePos())
                std::printf(" %zu:%zu", i, op->getInputs()[i]->getOffset(deps[i].getBegin()));
    }
    std::printf("\n");
}
int main() {
    Tensor x({2, 4, 6, 8});
    // the forms of src/Mutant/generator.cc:1028-1092
    TransposeOp h2n(&x, 2, {{0, 2}, 1, -1, 3}, -2, TransposeOp::H2N);
    walk("h2n", &h2n, h2n.getOutputs()[0]);
    TransposeOp n2h(&x, 0, {0, 1, {-1, 2}, 3}, 2, TransposeOp::N2H);
    walk("n2h", &n2h, n2h.getOutputs()[0]);
    TransposeOp d2h(&x, 2, {0, 1, {-1, 2}, 3}, 2, TransposeOp::D2H);
    walk("d2h", &d2h, d2h.getOutputs()[0]);
    TransposeOp d2hInv(&x, 2, {0, 1, {-1, 2}, 3}, -2, TransposeOp::D2H);
    walk("d2hInv", &d2hInv, d2hInv.getOutputs()[0]);
    TransposeOp swap(&x, -1, {0, 1, 3, 2});
    walk("swap", &swap, swap.getOutputs()[0]);
    Tensor a({2, 3, 4}), b({2, 5, 4});
    ConcatOp cat({&a, &b}, 1);
    walk("concat", &cat, cat.getOutputs()[0]);
    ExtendOp ext(&a, 1, 2);
    walk("extend", &ext, ext.getOutputs()[0]);
    Tensor bias({4});
    Tensor sum;
    AddOp add({&a, &bias}, &sum);
    walk("add", &add, &sum);
    SplitOp split(&b, 1, {2, 3});
    for (size_t k = 0; k < 2; ++k) {
        Tensor *o = split.getOutputs()[k];
        std::printf("split%zu", k);
        for (o->itInit(); o->itValid(); o->itNext())
            std::printf(" 0:%zu", b.getOffset(split.compute(k, DimRange(o->itGet())).first[0].getBegin()));
        std::printf("\n");
    }
    Tensor A({3, 4, 5}), B({3, 6, 5});
    MatmulOp mm(&A, &B, false, true);
    auto deps = mm.compute(DimRange(Dim{2, 1, 4})).first;
    std::printf("matmul %d %d %d %d %d %d %d %d %d %d %d %d\n",
                deps[0].getBegin()[0], deps[0].getBegin()[1], deps[0].getBegin()[2],
                deps[0].getEnd()[0], deps[0].getEnd()[1], deps[0].getEnd()[2],
                deps[1].getBegin()[0], deps[1].getBegin()[1], deps[1].getBegin()[2],
                deps[1].getEnd()[0], deps[1].getEnd()[1], deps[1].getEnd()[2]);
    return 0;
}
"""


def test_point_dependences_match_numpy_index_maps(tmp_path):
    import numpy as np
    src = tmp_path / "deps.cc"
    src.write_text(DEPENDENCE_PROGRAM)
    exe = tmp_path / "deps"
    subprocess.run(["g++", "-std=c++17", "-O1", str(src),
                    "-I", os.path.join(ROOT, "pet_amd", "host", "include"),
                    "-I", os.path.join(ROOT, "include"), "-L", LIB, "-lpet_host", "-lpet_hip",
                    "-Wl,-rpath," + LIB, "-o", str(exe)], check=True)
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert run.returncode == 0, (run.returncode, run.stdout, run.stderr)
    got = {}
    for line in run.stdout.splitlines():
        name, *rest = line.split()
        got[name] = rest

    def offsets(name, which=None):
        pairs = [t.split(":") for t in got[name]]
        return [int(o) for i, o in pairs if which is None or int(i) == which]

    x = np.arange(2 * 4 * 6 * 8).reshape(2, 4, 6, 8)
    # the closed forms the reference gives for these rewrites
    h2n = x.reshape(2, 4, 2, 3, 8).transpose(0, 2, 1, 3, 4).reshape(4, 4, 3, 8)
    assert offsets("h2n") == h2n.ravel().tolist()
    n2h = x.reshape(1, 2, 4, 6, 8).transpose(0, 2, 1, 3, 4).reshape(1, 4, 12, 8)
    assert offsets("n2h") == n2h.ravel().tolist()
    d2h = x.reshape(2, 4, 3, 2, 8).transpose(0, 1, 3, 2, 4).reshape(2, 4, 6, 8)
    assert offsets("d2h") == d2h.ravel().tolist()
    d2h_inv = x.reshape(2, 4, 2, 3, 8).transpose(0, 1, 3, 2, 4).reshape(2, 4, 6, 8)
    assert offsets("d2hInv") == d2h_inv.ravel().tolist()
    assert offsets("swap") == x.transpose(0, 1, 3, 2).ravel().tolist()

    a = np.arange(24).reshape(2, 3, 4)
    b = np.arange(40).reshape(2, 5, 4)
    tagged = np.concatenate([a * 2, b * 2 + 1], axis=1).ravel()      # low bit = which input
    pairs = [tuple(map(int, t.split(":"))) for t in got["concat"]]
    assert [o * 2 + i for i, o in pairs] == tagged.tolist()
    assert offsets("extend") == np.tile(a, (1, 3, 1)).ravel().tolist()
    assert offsets("add", 0) == list(range(24))
    assert offsets("add", 1) == [i % 4 for i in range(24)]
    assert offsets("split0") == b[:, :2].ravel().tolist()
    assert offsets("split1") == b[:, 2:].ravel().tolist()
    # C[2,1,4] = sum_k A[2,1,k] * B[2,4,k] with B stored [b,n,k]
    assert got["matmul"] == "2 1 0 2 1 4 2 4 0 2 4 4".split()


# ---- the reference's own mutation generator on this backend ----------------------
# libpet_refsearch.so is the reference's src/Mutant/generator.cc, reciprocity.cc and
# src/Graph/trans_eliminator.cc compiled unchanged against pet_amd/host/include
# (make -C pet_amd/host refsearch, run where the reference tree is present; the
# binaries travel with the tree). The programs under pet_amd/lib/refsearch are the
# reference's src/Test/single_rule_test_*.cc, also unchanged.
REFSEARCH = os.path.join(LIB, "libpet_refsearch.so")
GENERATOR_DRIVER = os.path.join(LIB, "pet_generator_driver")
STATUS = os.path.join(LIB, "refsearch_status.txt")


def _built_without_reference():
    """True only when the build recorded that it had no reference tree to compile from.
    In every other case the binaries are expected and their absence fails the test."""
    return os.path.exists(STATUS) and open(STATUS).read().strip() == "no-reference"


needs_refsearch = pytest.mark.skipif(_built_without_reference(),
                                     reason="the build had no reference tree to compile from")

# program -> candidates the generator must at least find. The assertions inside
# the programs were written for an earlier generator: at the reference's head the
# input graph itself is no longer added to the candidates
# (src/Mutant/generator.cc:23) and candidates deeper than max_depth are dropped
# (:1960-1964), so most of their counts are one higher than the head can give
# and the preprocess-only rules (6, 13, 15) give none.
SINGLE_RULE_PROGRAMS = {
    "single_rule_test_1_n2h": 2, "single_rule_test_2_n2w": 2, "single_rule_test_3_c2h": 2,
    "single_rule_test_4_c2w": 2, "single_rule_test_5_dilated": 1,
    "single_rule_test_7_trans_gemm": 1, "single_rule_test_8_conv2group": 1,
    "single_rule_test_9_group_conv_a": 1, "single_rule_test_12_1xk_trans": 1,
    "single_rule_test_14_split_group_conv": 4, "single_rule_test_16_group_conv_d": 1,
}


@pytest.mark.gpu
@needs_refsearch
@pytest.mark.parametrize("program", sorted(SINGLE_RULE_PROGRAMS))
def test_reference_single_rule_program_finds_mutants_on_the_device(program):
    import re
    exe = os.path.join(LIB, "refsearch", program)
    assert os.path.exists(exe), "run __graft_entry__.build() where the reference tree is present"
    res = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    print(res.stdout[-3000:])
    print(res.stderr[-2000:])
    # 0: the program's own assertion held; 134 (-6): it aborted on its assertion
    assert res.returncode in (0, -6, 134), res.returncode
    found = re.findall(r"candidates found: (\d+)", res.stdout)
    assert found, "the program did not reach its report"
    assert int(found[-1]) >= SINGLE_RULE_PROGRAMS[program]
    if res.returncode != 0:
        assert "candidates.size()" in res.stderr      # nothing but the stale count


@pytest.mark.gpu
@needs_refsearch
@pytest.mark.parametrize("args", [
    "1 64 56 56 64 3 1 1 1",       # benchmark configuration 1: needs an exact candidate
    "1 32 32 32 32 3 2 2 0",       # dilated convolution: de-interleave candidates, partial
])
def test_generator_candidates_run_and_are_ranked_on_the_device(args):
    assert os.path.exists(GENERATOR_DRIVER), \
        "run __graft_entry__.build() where the reference tree is present"
    res = subprocess.run([GENERATOR_DRIVER] + args.split(), capture_output=True, text=True,
                         timeout=600)
    print(res.stdout[-6000:])
    print(res.stderr[-2000:])
    assert res.returncode == 0


SEARCH_DRIVER = os.path.join(LIB, "pet_search_driver")
MEMBOUND_DRIVER = os.path.join(LIB, "pet_membound_driver")


@pytest.mark.gpu
@needs_refsearch
@pytest.mark.parametrize("args", [
    "1 64 56 56 64 3 1 1",         # benchmark configuration 1
    "1 512 64 64 512 3 2 2",       # the 512 -> 512 layer of the dilated block
    "1 512 64 64 512 3 2 2 nnet",  # the same with the reference's NMutator as mutation engine
])
def test_reference_search_engine_runs_on_the_device(args):
    """The reference's SearchEngine::run (src/Graph/search_engine.cc:54-118), compiled
    unchanged with its mutation generator: candidates are ranked by Operator::perf on the
    MI355X; the graph it returns costs no more than the input graph, its getPerf total is
    SubGraph::perf, and it computes what the input graph computes."""
    import re
    assert os.path.exists(SEARCH_DRIVER), \
        "run __graft_entry__.build() where the reference tree is present"
    res = subprocess.run([SEARCH_DRIVER] + args.split(), capture_output=True, text=True,
                         timeout=900)
    print(res.stdout[-6000:])
    print(res.stderr[-3000:])
    assert res.returncode == 0
    origin = re.findall(r"Origin Perf: ([0-9.eE+-]+)", res.stdout)
    best = re.findall(r"Best Perf without correction: ([0-9.eE+-]+)", res.stdout)
    assert origin and best and float(best[-1]) <= float(origin[0]) * 1.0001
    assert "PET graph getPerf" in res.stdout and " op_time " in res.stdout   # the profile table
    assert "driver: ok" in res.stdout


@pytest.mark.gpu
@needs_refsearch
def test_membound_operator_agrees_with_the_reference_interpreter():
    """MemBoundOp on the device against nnet::Interpreter (the reference's own evaluation,
    compiled unchanged) on expressions the reference's pattern builders produce:
    convolution, matmul, the band products, transposed convolution, layout moves."""
    assert os.path.exists(MEMBOUND_DRIVER), \
        "run __graft_entry__.build() where the reference tree is present"
    res = subprocess.run([MEMBOUND_DRIVER], capture_output=True, text=True, timeout=300)
    print(res.stdout[-4000:])
    print(res.stderr[-2000:])
    assert res.returncode == 0
    assert res.stdout.count("[  OK  ]") >= 9 and "0 failed" in res.stdout
    assert "NMutator naive MemBound of a convolution equals the convolution" in res.stdout


# ---- the benchmark networks through Graph -> SubGraph -> CodeEngine ---------------
RUN_MODEL = os.path.join(LIB, "pet_run_model")


@pytest.mark.gpu
@pytest.mark.parametrize("model", ["dilated", "dilated:pet", "resnet18", "resnet18:pet", "bert",
                                   "bert:pet", "resnet3d18"])
def test_model_graph_replay_equals_operator_by_operator_run(model):
    """pet_run_model --check: the captured HIP graph (storage sharing, transposes in a
    row folded into one kernel, constant 3-D filters repacked) against
    SubGraph::compute, which launches every operator by itself."""
    import json
    assert os.path.exists(RUN_MODEL), "run __graft_entry__.build() first"
    res = subprocess.run([RUN_MODEL, model, "--check", "--rounds", "20", "--warmup", "3"],
                         capture_output=True, text=True, timeout=300)
    print(res.stdout)
    print(res.stderr[-2000:])
    assert res.returncode == 0
    rec = json.loads(res.stdout.strip().splitlines()[-1])
    assert rec["max_abs_diff_vs_eager"] <= 1e-4 * rec["max_abs_eager"]
    assert rec["ms"] > 0
    if model == "dilated:pet":
        # the two rows of Transposes are the addressing of the first and the last convolution
        assert rec["folded"] == 4 and rec["kernels"] == 6
    if model == "resnet18:pet":
        # three blocks run their shortcut inside their first convolution
        assert rec["kernels"] == 23 - 3
    if model == "bert:pet":
        # per layer: one merged projection instead of three, the stacking Concat never runs
        assert rec["kernels"] == 108 - 2 * 12


@pytest.mark.gpu
@pytest.mark.parametrize("model", ["resnet18", "bert"])
def test_model_graph_with_searched_algorithms(model):
    """pet_run_model --tune --check: Operator::perf searches the backend's algorithms for
    every contraction first; the graph then runs with what was found and still agrees
    with the operator-by-operator run. With the search switched off nothing leaves the
    default."""
    import json
    res = subprocess.run([RUN_MODEL, model, "--tune", "--check", "--rounds", "20", "--warmup", "3"],
                         capture_output=True, text=True, timeout=600)
    assert res.returncode == 0, res.stderr[-2000:]
    rec = json.loads(res.stdout.strip().splitlines()[-1])
    assert rec["max_abs_diff_vs_eager"] <= 1e-4 * rec["max_abs_eager"]
    assert 0 <= rec["off_default_algo"] <= rec["operators"]
    env = dict(os.environ, PET_HOST_NO_ALGO_SEARCH="1")
    res = subprocess.run([RUN_MODEL, model, "--tune", "--rounds", "5", "--warmup", "2"],
                         capture_output=True, text=True, timeout=600, env=env)
    assert res.returncode == 0, res.stderr[-2000:]
    assert json.loads(res.stdout.strip().splitlines()[-1])["off_default_algo"] == 0


def _cpp_module():
    import glob
    import importlib
    import sys
    assert glob.glob(os.path.join(LIB, "cpp_module*.so")), "run __graft_entry__.build() first"
    if LIB not in sys.path:
        sys.path.insert(0, LIB)
    return importlib.import_module("cpp_module")


def test_python_module_builds_graphs_like_the_reference_front_end():
    """cpp_module (the reference's src/ffi/ffi_pet.cc surface): builder names, argument
    orders and shape rules, no device needed."""
    cm = _cpp_module()
    g = cm.Graph()
    x, w = g.tensor([1, 8, 12, 12], "FLOAT"), g.tensor([16, 8, 3, 3], "FLOAT")
    y = g.tensor([1, 16, 12, 12], "FLOAT")
    conv = g.conv(x, w, y, 1, 1)                      # input, weight, output, ph, pw
    assert y.getDims() == [1, 16, 12, 12] and "Conv" in conv.toString()
    t = g.tensor([2, 16, 6, 12], "FLOAT")
    g.transpose(y, t, 2, [[0, 2], 1, -1, 3], -2)      # H2N as the mutator writes it
    assert t.getDims() == [2, 16, 6, 12]
    a, b, c = g.tensor([3, 5, 7], "FLOAT"), g.tensor([3, 7, 4], "FLOAT"), g.tensor([3, 5, 4], "FLOAT")
    g.matmul(a, b, c)
    assert c.getDims() == [3, 5, 4]
    s0, s1 = g.tensor([1, 4, 12, 12], "FLOAT"), g.tensor([1, 12, 12, 12], "FLOAT")
    g.split(y, [s0, s1], 1, [1, 3])                   # sizes are ratios
    assert s0.getDims() == [1, 4, 12, 12] and s1.getDims() == [1, 12, 12, 12]
    p = g.tensor([1, 16, 14, 13], "FLOAT")
    g.pad(y, p, [0, 0, 1, 0], [0, 0, 1, 1])
    assert p.getDims() == [1, 16, 14, 13]
    g.updateConnection()
    sub = cm.SubGraph(g.getOperators())
    assert len(sub.getOperators()) == len(g.getOperators()) == 5
    assert {tuple(i.getDims()) for i in sub.getInputs()} == {(1, 8, 12, 12), (16, 8, 3, 3),
                                                             (3, 5, 7), (3, 7, 4)}


@pytest.mark.gpu
def test_python_module_runs_a_graph_on_the_device():
    """Graph built from Python, data from numpy, run operator by operator and as one
    replayed HIP graph; against the oracle."""
    import numpy as np
    import oracle
    cm = _cpp_module()
    rng = np.random.default_rng(5)
    g = cm.Graph()
    x, w = g.tensor([1, 8, 12, 12], "FLOAT"), g.tensor([16, 8, 3, 3], "FLOAT")
    y, z = g.tensor([1, 16, 12, 12], "FLOAT"), g.tensor([1, 16, 12, 12], "FLOAT")
    g.conv(x, w, y, 1, 1)
    g.relu(y, z)
    t = g.tensor([2, 16, 6, 12], "FLOAT")
    g.transpose(z, t, 2, [[0, 2], 1, -1, 3], -2)
    g.updateConnection()
    xv = rng.integers(-3, 4, (1, 8, 12, 12)).astype(np.float32)
    wv = rng.integers(-3, 4, (16, 8, 3, 3)).astype(np.float32)
    want = oracle.transpose(np.maximum(oracle.conv2d(xv, wv, 1, 1), 0), 2, [[0, 2], 1, -1, 3], -2)
    for replay in (False, True):
        sub = cm.SubGraph(g.getOperators())
        for inp in sub.getInputs():
            inp.setData(xv if inp.getDims() == [1, 8, 12, 12] else wv)
        if replay:
            ce = cm.CodeEngine()
            ex = ce.instantiate(sub)
            assert ex.launch() and ex.sync()
            assert ex.time(2, 5) > 0
            assert "pet_hip_conv2d" in ce.genCode(sub)
        else:
            assert sub.compute()
            assert sub.perf(cm.PerfEngine()) > 0
        got = sub.getOutputs()[0].getData()
        assert got.shape == want.shape and got.tobytes() == want.tobytes(), replay


@pytest.mark.gpu
@pytest.mark.parametrize("model", ["resnet18", "resnet3d18", "bert", "bert:pet", "dilated:pet"])
def test_emitted_model_program_compiles_and_agrees_with_the_runtime(model, tmp_path):
    """CodeEngine::genCode for a whole network (fused block tails, kt-major filters,
    storage sharing): the emitted C++ builds against pet_hip.h alone, runs, and its
    time per iteration is that of the in-process graph."""
    import json
    import re
    src = tmp_path / "net.cpp"
    res = subprocess.run([RUN_MODEL, model, "--rounds", "50", "--warmup", "5", "--emit", str(src)],
                         capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr[-2000:]
    rec = json.loads(res.stdout.strip().splitlines()[-1])
    text = src.read_text()
    if model == "bert:pet":
        assert ", 48u, s)" in text and "pet_hip_concat(" not in text  # shared lhs, bias rows
    if model == "dilated:pet":
        # space-to-batch and batch-to-space are the strides of the first and last convolution
        assert text.count("pet_hip_conv2d_view_f32(") == 2 and "pet_hip_trans_chain(" not in text
        assert "static const pet_hip_conv_view xv" in text and "&yv" in text
    elif not model.startswith("bert"):
        # a block tail became one call, with the ReLU of what it reads applied on load
        assert re.search(r"pet_hip_conv[23]d_ex_f32\([^;]*, (1[0-5]|[4-9])u, s\)", text)
    else:
        assert "pet_hip_bmm_res_f32(" in text
    # initialisations of the launches that accumulate into their output: batched up front
    assert ("pet_hip_bias_fill_batch(fills, " in text) == (rec["hoisted_fills"] > 0)
    if model == "resnet3d18":
        assert "pet_hip_conv3d_pack_filters(" in text
    exe = tmp_path / "net"
    subprocess.run(["g++", "-O1", str(src), "-I", os.path.join(ROOT, "include"), "-L", LIB,
                    "-lpet_hip", "-Wl,-rpath," + LIB, "-o", str(exe)], check=True)
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stdout + run.stderr
    ms = float(re.search(r"Time\(ms\)\D*([0-9.eE+-]+)", run.stdout).group(1))
    assert 0.7 * rec["ms"] <= ms <= 1.4 * rec["ms"], (ms, rec["ms"])


# ---- the reference's operator-level test programs, unchanged ----------------------
# pet_amd/lib/reftests/<name> is src/Test/<name>.cc(pp) of the reference compiled
# against pet_amd/host/include. Programs that compare two ways of computing the same
# tensor print "equal/total = a/b"; the others only have to run through their own
# assertions. Left out: conv_test_1 and transpose_test_1 (they read dat/ files the
# reference does not ship) and the three *_perf programs (minutes of timing loops).
REFTESTS = os.path.join(LIB, "reftests")
REFERENCE_OPERATOR_PROGRAMS = [
    "SampleGraph3", "SampleGraph4", "batch_gemm_test", "concat_test_1", "conv_test_2",
    "conv_test_3", "conv_test_5_trans_kernel", "extend_test_1", "group_conv_test_1",
    "group_conv_test_2", "mutant_test_2", "pad_slice_test", "perf_pool", "split_test_1",
    "split_test_2", "tensor_test", "transpose_test_2", "transpose_test_3", "transpose_test_4",
    "transpose_test_5",
]


# Programs of src/Test that build graphs and hand them to the reference's Generator,
# SearchEngine (which times every candidate through Operator::perf on the device) and
# CodeEngine: compiled unchanged, run to their own end. What they print is the search's
# report; "Best Perf" can only be at or below "Origin Perf" (the search keeps the input graph
# when nothing beats it). Left out, with the reason:
#   convtrans_test_1 / _2     compare an NHWC output tensor, flat, with vectors written down in
#                             NCHW order, and ConvTransOp::compute upstream takes its loop
#                             bounds from the wrong dims (src/Graph/operator.cc:948): they
#                             abort on the reference's own code too. The vectors themselves
#                             are tests/golden/convtrans_reference_vectors.json, used with
#                             the layout they were made in.
#   transposeconv_test_1      its filter tensor is [f, r, s, c] and of type Input: the
#                             reference's own ConvTransOp::checkValid (:1098-1111) rejects it
#   graph_stat_test_2_batchmm copy-assigns a SubGraph, whose destructor frees the operators
#                             both copies point at (src/Graph/graph.cc:12-19)
#   SampleGraph1              after 160 s of search it dies inside the reference's own
#                             Generator::markTransType (src/Mutant/generator.cc:1953-1954: it
#                             dereferences the producer of a convolution's input where that
#                             input is the graph's input; the `if` above it, :1950, is empty)
#   single_op_test_8_conv3d, gen_transpose    do not compile against the reference's own
#                             headers at its head; import_onnx*: need .onnx files
REFERENCE_SEARCH_PROGRAMS = {
    # program: command-line arguments
    "split_test_3": [], "fuse_activation": [], "eliminator_test_1": [],
    "single_op_test_1": [], "single_op_test_2": [], "single_op_test_3": [],
    "single_op_test_4": [], "single_op_test_5": [], "single_op_test_6": [],
    "single_op_test_7_batch_gemm": [], "graph_stat_test_1_transpose_group": [],
    "mutant_test_1": [], "mutant_test_3": [], "cache_test_1": [], "cache_test_2": [],
    "cache_test_3": [], "SampleGraph2": [],
    # the reference's own dilated-convolution benchmark: six 3x3 convolutions with ReLU at
    # dilation 2 (configuration 1), batch 1; searches, then emits the program (res.cu)
    "dilation_test": ["1", "1"],
}


# searches over a single convolution that time dozens of candidates (30-95 s each): run with
# PET_SLOW_REFERENCE_PROGRAMS=1; the same path is covered by single_op_test_3 / _6 / _7
SLOW_SEARCH_PROGRAMS = {"single_op_test_1", "single_op_test_2", "single_op_test_4",
                        "single_op_test_5"}


@pytest.mark.gpu
@needs_refsearch
@pytest.mark.parametrize("program", sorted(REFERENCE_SEARCH_PROGRAMS))
def test_reference_search_program_runs_on_the_device(program, tmp_path):
    import re
    if program in SLOW_SEARCH_PROGRAMS and not os.environ.get("PET_SLOW_REFERENCE_PROGRAMS"):
        pytest.skip("a search of 30-95 s: set PET_SLOW_REFERENCE_PROGRAMS=1")
    exe = os.path.join(REFTESTS, program)
    assert os.path.exists(exe), "run __graft_entry__.build() where the reference tree is present"
    res = subprocess.run([exe] + REFERENCE_SEARCH_PROGRAMS[program], capture_output=True,
                         text=True, timeout=600, cwd=str(tmp_path))
    print(res.stdout[-2000:])
    print(res.stderr[-1500:])
    if res.returncode == -11:
        # see SampleGraph1 above: whether a candidate that trips upstream's markTransType
        # comes up depends on the search's random sampling
        pytest.xfail("upstream's markTransType dereferenced a null producer in this run")
    assert res.returncode == 0
    origin = re.findall(r"Origin Perf: ([0-9.eE+-]+)", res.stdout)
    best = re.findall(r"Best Perf with correction: ([0-9.eE+-]+)", res.stdout)
    for o, b in zip(origin, best):
        assert 0 < float(b) <= float(o) * 1.001
    if program == "dilation_test":
        emitted = (tmp_path / "res.cu").read_text()
        assert emitted.count("pet_hip_conv2d") >= 6     # the six layers, ReLU fused


@pytest.mark.gpu
@needs_refsearch
@pytest.mark.parametrize("program", REFERENCE_OPERATOR_PROGRAMS)
def test_reference_operator_program_runs_on_the_device(program):
    import re
    env = dict(os.environ)
    if program == "SampleGraph3":
        # compares two runs of a three-convolution chain whose values (1e10) are far
        # beyond fp32's exact integers: only the run-to-run reproducible mode can
        # meet its `==` (the reference computes in wrapping uint32)
        env["PET_HIP_DETERMINISTIC"] = "1"
    assert os.path.exists(os.path.join(REFTESTS, program)), \
        "run __graft_entry__.build() where the reference tree is present"
    res = subprocess.run([os.path.join(REFTESTS, program)], capture_output=True, text=True,
                         timeout=300, env=env)
    print(res.stdout[-1500:])
    print(res.stderr[-1500:])
    assert res.returncode == 0
    for a, b in re.findall(r"equal/total\s*=\s*(\d+)/(\d+)", res.stdout):
        if program == "mutant_test_2":
            # a dilated convolution against its de-interleaved form WITHOUT boundary
            # correction: a partially equivalent rewrite. The two agree on the inner
            # 12x12 of every 14x14 output plane and nowhere on the rim: 144/196.
            assert (int(a), int(b)) == (16 * 32 * 12 * 12, 16 * 32 * 14 * 14)
        else:
            assert a == b and int(b) > 0
