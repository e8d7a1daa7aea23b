"""ONNX ingestion without the `onnx` package (pet_amd/onnx_import.py, the role of the
reference's python/cpp_plugin/import_onnx.py): parser on hand-written files, graph
building on the CPU, and on the GPU a small residual CNN and an attention-style block
against torch's CPU operators. No file written by the `onnx` package itself is
available here, so compatibility with its serialiser rests on the published field
numbers the writer (tests/onnx_writer.py) and the reader both follow."""
import glob
import os

import numpy as np
import pytest

try:
    from tests import onnx_writer as ow
except ImportError:          # collected with tests/ itself on sys.path
    import onnx_writer as ow

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
pytestmark = pytest.mark.skipif(
    not glob.glob(os.path.join(ROOT, "pet_amd", "lib", "cpp_module*.so")),
    reason="cpp_module is not built (pybind11 missing at build time)")


def cnn(rng):
    w = {"w1": rng.standard_normal((8, 3, 3, 3)) * 0.2, "b1": rng.standard_normal(8) * 0.1,
         "sc": rng.uniform(0.5, 1.5, 8), "bi": rng.standard_normal(8) * 0.1,
         "me": rng.standard_normal(8) * 0.1, "va": rng.uniform(0.5, 1.5, 8),
         "w2": rng.standard_normal((8, 8, 3, 3)) * 0.1,
         "fc": rng.standard_normal((10, 8)) * 0.3, "fb": rng.standard_normal(10) * 0.1}
    w = {k: v.astype(np.float32) for k, v in w.items()}
    nodes = [
        ow.node("Conv", ["x", "w1", "b1"], ["c1"], pads=[1, 1, 1, 1], strides=[1, 1],
                dilations=[1, 1], kernel_shape=[3, 3], group=1),
        ow.node("Relu", ["c1"], ["r1"]),
        ow.node("MaxPool", ["r1"], ["p1"], packed=True, kernel_shape=[2, 2], strides=[2, 2],
                pads=[0, 0, 0, 0]),
        ow.node("BatchNormalization", ["p1", "sc", "bi", "me", "va"], ["bn"], epsilon=1e-3),
        ow.node("Conv", ["bn", "w2"], ["c2"], pads=[1, 1, 1, 1]),
        ow.node("Add", ["c2", "bn"], ["s"]),
        ow.node("Relu", ["s"], ["r2"]),
        ow.node("GlobalAveragePool", ["r2"], ["gap"]),
        ow.node("Flatten", ["gap"], ["flat"], axis=1),
        ow.node("Gemm", ["flat", "fc", "fb"], ["logits"], transB=1, alpha=1.0, beta=1.0),
        ow.node("Softmax", ["logits"], ["prob"], axis=-1),
    ]
    data = ow.model(nodes, w, [("x", [1, 3, 16, 16])] + [(k, list(v.shape)) for k, v in w.items()],
                    [("prob", [1, 10])])
    return data, w


def cnn_reference(x, w):
    import torch
    import torch.nn.functional as F
    t = {k: torch.from_numpy(v) for k, v in w.items()}
    y = F.relu(F.conv2d(torch.from_numpy(x), t["w1"], t["b1"], padding=1))
    y = F.max_pool2d(y, 2, 2)
    bn = F.batch_norm(y, t["me"], t["va"], t["sc"], t["bi"], False, 0.1, 1e-3)
    y = F.relu(F.conv2d(bn, t["w2"], None, padding=1) + bn)
    y = F.adaptive_avg_pool2d(y, 1).flatten(1)
    return F.softmax(F.linear(y, t["fc"], t["fb"]), dim=-1).numpy()


def test_parser_reads_packed_and_unpacked_fields():
    from pet_amd import onnx_import
    data, w = cnn(np.random.default_rng(0))
    nodes, inits, inputs, outputs = onnx_import.parse(data)
    assert [n.op for n in nodes][:4] == ["Conv", "Relu", "MaxPool", "BatchNormalization"]
    assert nodes[0].attrs["pads"] == [1, 1, 1, 1] and nodes[0].inputs == ["x", "w1", "b1"]
    assert nodes[2].attrs["kernel_shape"] == [2, 2] and nodes[2].attrs["strides"] == [2, 2]  # packed
    assert abs(nodes[3].attrs["epsilon"] - 1e-3) < 1e-9 and nodes[9].attrs["transB"] == 1
    assert nodes[10].attrs["axis"] == -1                                   # negative varint
    assert set(inits) == set(w) and np.array_equal(inits["w2"], w["w2"])
    assert inputs[0] == ("x", [1, 3, 16, 16]) and outputs == ["prob"]
    # int64 initializer through int64_data as well as raw_data
    t = ow.i(1, 3) + ow.i(2, 7) + ow.s(8, "shape") + ow.ld(7, b"".join(ow.varint(v) for v in (2, -1, 4)))
    name, arr = onnx_import._tensor(t)
    assert name == "shape" and arr.tolist() == [2, -1, 4] and arr.dtype == np.int64


def test_graph_building_and_shape_rules():
    from pet_amd import onnx_import
    data, w = cnn(np.random.default_rng(0))
    m = onnx_import.load(data)
    assert m.inputs == ["x"] and set(m.weights) == set(w)
    shapes = {k: m.tensors[k].getDims() for k in ("c1", "p1", "bn", "c2", "r2", "gap")}
    assert shapes == {"c1": [1, 8, 16, 16], "p1": [1, 8, 8, 8], "bn": [1, 8, 8, 8],
                      "c2": [1, 8, 8, 8], "r2": [1, 8, 8, 8], "gap": [1, 8, 1, 1]}
    # MatmulOp gives 2-D operands a leading 1 (MatmulOp::dimExtend, operator.cc:656-662)
    assert m.tensors["flat"].getDims() == [1, 1, 8]
    assert m.tensors["prob"].size() == 10 and m.tensors["w1"].isWeight()
    assert len(m.graph.getOperators()) == 11
    with pytest.raises(ValueError):
        onnx_import.load(ow.model([ow.node("Einsum", ["x"], ["y"])], {}, [("x", [2, 2])], [("y", [2, 2])]))
    with pytest.raises(ValueError):     # channel-wise broadcast is not a trailing-dim broadcast
        onnx_import.load(ow.model([ow.node("Mul", ["x", "s"], ["y"])],
                                  {"s": np.ones((1, 3, 1, 1), np.float32)},
                                  [("x", [1, 3, 4, 4])], [("y", [1, 3, 4, 4])]))


@pytest.mark.gpu
def test_imported_cnn_matches_torch(tmp_path):
    import subprocess
    from pet_amd import onnx_import
    rng = np.random.default_rng(1)
    data, w = cnn(rng)
    x = rng.standard_normal((1, 3, 16, 16)).astype(np.float32)
    want = cnn_reference(x, w)
    m = onnx_import.load(data)
    for replay in (False, True):
        sub, feeds = m.subgraph()
        feeds["x"].setData(x)
        if replay:
            ex = m.module.CodeEngine().instantiate(sub)
            assert ex.launch() and ex.sync()
        else:
            assert sub.compute()
        got = sub.getOutputs()[0].getData().reshape(want.shape)
        np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-6)
    # the program emitted for the imported graph builds against pet_hip.h alone and runs
    src, exe = tmp_path / "net.cpp", tmp_path / "net"
    assert m.module.CodeEngine().genCode(sub, str(src)) == 0
    text = src.read_text()
    # this BatchNormalization follows the pooling, not a convolution: it stays an operator
    assert "pet_hip_conv2d" in text and "pet_hip_batchnorm(" in text
    lib = os.path.join(ROOT, "pet_amd", "lib")
    subprocess.run(["g++", "-O1", str(src), "-I", os.path.join(ROOT, "include"), "-L", lib,
                    "-lpet_hip", "-Wl,-rpath," + lib, "-o", str(exe)], check=True)
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0 and "Time(ms)" in run.stdout, run.stdout + run.stderr


def _conv_bn_model(rng):
    w = {"w": (rng.standard_normal((6, 4, 3, 3)) * 0.2), "b": rng.standard_normal(6) * 0.1,
         "sc": rng.uniform(0.5, 1.5, 6), "bi": rng.standard_normal(6) * 0.1,
         "me": rng.standard_normal(6) * 0.1, "va": rng.uniform(0.5, 1.5, 6)}
    w = {k: v.astype(np.float32) for k, v in w.items()}
    nodes = [ow.node("Conv", ["x", "w", "b"], ["c"], pads=[1, 1, 1, 1], strides=[2, 2]),
             ow.node("BatchNormalization", ["c", "sc", "bi", "me", "va"], ["n"], epsilon=1e-5),
             ow.node("Relu", ["n"], ["y"])]
    return ow.model(nodes, w, [("x", [2, 4, 9, 9])], [("y", [2, 6, 5, 5])]), w


def test_batchnorm_after_a_convolution_is_folded():
    from pet_amd import onnx_import
    data, w = _conv_bn_model(np.random.default_rng(3))
    folded = onnx_import.load(data)
    kept = onnx_import.load(data, fold_bn=False)
    assert len(folded.graph.getOperators()) == 2 and len(kept.graph.getOperators()) == 3
    factor = w["sc"] / np.sqrt(w["va"] + np.float32(1e-5))
    np.testing.assert_allclose(folded.weights["w::bn"], w["w"] * factor[:, None, None, None],
                               rtol=1e-6)
    np.testing.assert_allclose(folded.weights["c::bn_bias"], (w["b"] - w["me"]) * factor + w["bi"],
                               rtol=1e-5, atol=1e-7)


@pytest.mark.gpu
def test_folded_and_unfolded_batchnorm_match_torch():
    import torch
    import torch.nn.functional as F
    from pet_amd import onnx_import
    rng = np.random.default_rng(3)
    data, w = _conv_bn_model(rng)
    x = rng.standard_normal((2, 4, 9, 9)).astype(np.float32)
    t = {k: torch.from_numpy(v) for k, v in w.items()}
    want = F.relu(F.batch_norm(F.conv2d(torch.from_numpy(x), t["w"], t["b"], stride=2, padding=1),
                               t["me"], t["va"], t["sc"], t["bi"], False, 0.1, 1e-5)).numpy()
    for fold in (True, False):
        sub, feeds = onnx_import.load(data, fold_bn=fold).subgraph()
        feeds["x"].setData(x)
        assert sub.compute()
        np.testing.assert_allclose(sub.getOutputs()[0].getData(), want, rtol=1e-4, atol=1e-5)


@pytest.mark.gpu
def test_imported_attention_block_matches_torch():
    """MatMul / Reshape / Transpose / Softmax / Split / Concat / Gather / ReduceMean / Pow /
    LayerNormalization / Gelu."""
    import torch
    from pet_amd import onnx_import
    rng = np.random.default_rng(2)
    seq, hid, heads = 8, 16, 2
    w = {"emb": rng.standard_normal((20, hid)).astype(np.float32),
         "wqkv": (rng.standard_normal((hid, 3 * hid)) * 0.2).astype(np.float32),
         "ids": np.array([3, 19, 0, 7, 7, 1, 12, 5], dtype=np.int64),
         "shp": np.array([seq, heads, hid // heads], dtype=np.int64),
         "two": np.array([2.0], dtype=np.float32)}
    nodes = [
        ow.node("Gather", ["emb", "ids"], ["x"], axis=0),
        ow.node("MatMul", ["x", "wqkv"], ["qkv"]),
        ow.node("Split", ["qkv"], ["q", "k", "v"], axis=-1, split=[hid, hid, hid]),
    ]
    for n in "qkv":
        nodes += [ow.node("Reshape", [n, "shp"], [n + "r"]),
                  ow.node("Transpose", [n + "r"], [n + "h"], perm=[1, 0, 2])]
    nodes += [ow.node("Transpose", ["kh"], ["kt"], perm=[0, 2, 1]),
              ow.node("MatMul", ["qh", "kt"], ["sc"]),
              ow.node("Softmax", ["sc"], ["pr"], axis=-1),
              ow.node("MatMul", ["pr", "vh"], ["ctx"]),
              ow.node("Pow", ["ctx", "two"], ["sq"]),
              ow.node("ReduceMean", ["sq"], ["ms"], axes=[2], keepdims=1),
              ow.node("Concat", ["ctx", "sq"], ["cat"], axis=2),
              ow.node("LayerNormalization", ["cat", "ln_g", "ln_b"], ["ln"], axis=-1, epsilon=1e-5),
              ow.node("Gelu", ["ln"], ["act"])]
    w["ln_g"] = rng.uniform(0.5, 1.5, hid).astype(np.float32)
    w["ln_b"] = (rng.standard_normal(hid) * 0.1).astype(np.float32)
    data = ow.model(nodes, w, [], [("ms", [heads, seq, 1]), ("act", [heads, seq, hid])])
    x = torch.from_numpy(w["emb"])[torch.from_numpy(w["ids"])]
    q, k, v = (x @ torch.from_numpy(w["wqkv"])).split(hid, dim=-1)
    qh, kh, vh = (t.reshape(seq, heads, hid // heads).permute(1, 0, 2) for t in (q, k, v))
    ctx = torch.softmax(qh @ kh.transpose(1, 2), -1) @ vh
    cat = torch.cat([ctx, ctx ** 2], 2)
    act = torch.nn.functional.gelu(torch.nn.functional.layer_norm(
        cat, (hid,), torch.from_numpy(w["ln_g"]), torch.from_numpy(w["ln_b"]), 1e-5))
    want = {"ms": (ctx ** 2).mean(2, keepdim=True).numpy(), "cat": act.numpy()}
    m = onnx_import.load(data)
    sub, feeds = m.subgraph()
    assert feeds == {}
    assert sub.compute()
    outs = {tuple(t.getDims()): t.getData() for t in sub.getOutputs()}
    np.testing.assert_allclose(outs[(heads, seq, 1)], want["ms"], rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(outs[(heads, seq, hid)], want["cat"], rtol=1e-4, atol=1e-5)


def _resnet18(rng):
    """ResNet-18 as exporters write it: Conv + BatchNormalization + Relu, residual Add,
    MaxPool, GlobalAveragePool, Flatten, Gemm. Random parameters."""
    nodes, w = [], {}

    def conv_bn(name, src, cin, cout, k, stride, pad, relu):
        fan = cin * k * k
        w[name + ".w"] = (rng.standard_normal((cout, cin, k, k)) * np.sqrt(2.0 / fan)).astype(np.float32)
        for p, lo, hi in (("sc", 0.8, 1.2), ("va", 0.8, 1.2)):
            w[name + "." + p] = rng.uniform(lo, hi, cout).astype(np.float32)
        for p in ("bi", "me"):
            w[name + "." + p] = (rng.standard_normal(cout) * 0.05).astype(np.float32)
        nodes.append(ow.node("Conv", [src, name + ".w"], [name + ".c"], pads=[pad] * 4,
                             strides=[stride, stride], kernel_shape=[k, k]))
        nodes.append(ow.node("BatchNormalization",
                             [name + ".c"] + [name + "." + p for p in ("sc", "bi", "me", "va")],
                             [name + ".n"], epsilon=1e-5))
        if relu:
            nodes.append(ow.node("Relu", [name + ".n"], [name + ".r"]))
        return name + (".r" if relu else ".n")

    t = conv_bn("stem", "x", 3, 64, 7, 2, 3, True)
    nodes.append(ow.node("MaxPool", [t], ["pool"], kernel_shape=[3, 3], strides=[2, 2], pads=[1] * 4))
    t, cin = "pool", 64
    for stage, cout in enumerate((64, 128, 256, 512)):
        for blk in range(2):
            stride = 2 if (stage > 0 and blk == 0) else 1
            name = "l%d.%d" % (stage + 1, blk)
            a = conv_bn(name + ".a", t, cin, cout, 3, stride, 1, True)
            b = conv_bn(name + ".b", a, cout, cout, 3, 1, 1, False)
            skip = t if (stride == 1 and cin == cout) else conv_bn(name + ".d", t, cin, cout, 1,
                                                                   stride, 0, False)
            nodes.append(ow.node("Add", [b, skip], [name + ".s"]))
            nodes.append(ow.node("Relu", [name + ".s"], [name + ".o"]))
            t, cin = name + ".o", cout
    w["fc.w"] = (rng.standard_normal((1000, 512)) * 0.03).astype(np.float32)
    w["fc.b"] = (rng.standard_normal(1000) * 0.01).astype(np.float32)
    nodes += [ow.node("GlobalAveragePool", [t], ["gap"]), ow.node("Flatten", ["gap"], ["flat"], axis=1),
              ow.node("Gemm", ["flat", "fc.w", "fc.b"], ["logits"], transB=1)]
    return ow.model(nodes, w, [("x", [1, 3, 224, 224])], [("logits", [1, 1000])]), w


def _resnet18_torch(x, w):
    import torch
    import torch.nn.functional as F
    t = {k: torch.from_numpy(v) for k, v in w.items()}

    def conv_bn(name, src, stride, pad, relu):
        y = F.conv2d(src, t[name + ".w"], None, stride=stride, padding=pad)
        y = F.batch_norm(y, t[name + ".me"], t[name + ".va"], t[name + ".sc"], t[name + ".bi"],
                         False, 0.1, 1e-5)
        return F.relu(y) if relu else y

    y = F.max_pool2d(conv_bn("stem", torch.from_numpy(x), 2, 3, True), 3, 2, 1)
    cin = 64
    for stage, cout in enumerate((64, 128, 256, 512)):
        for blk in range(2):
            stride = 2 if (stage > 0 and blk == 0) else 1
            name = "l%d.%d" % (stage + 1, blk)
            b = conv_bn(name + ".b", conv_bn(name + ".a", y, stride, 1, True), 1, 1, False)
            skip = y if (stride == 1 and cin == cout) else conv_bn(name + ".d", y, stride, 0, False)
            y, cin = F.relu(b + skip), cout
    return F.linear(F.adaptive_avg_pool2d(y, 1).flatten(1), t["fc.w"], t["fc.b"]).numpy()


@pytest.mark.gpu
def test_imported_resnet18_matches_torch():
    """Benchmark configuration 3 end to end through the file front end: 20 convolutions
    with their BatchNormalization folded at import, replayed as one HIP graph."""
    from pet_amd import onnx_import
    rng = np.random.default_rng(18)
    data, w = _resnet18(rng)
    x = rng.standard_normal((1, 3, 224, 224)).astype(np.float32)
    want = _resnet18_torch(x, w)
    m = onnx_import.load(data)
    assert sum("Conv" in op.toString() for op in m.graph.getOperators()) == 20
    assert not any("BatchNorm" in op.toString() for op in m.graph.getOperators())
    sub, feeds = m.subgraph()
    feeds["x"].setData(x)
    ex = m.module.CodeEngine().instantiate(sub)
    assert ex.launch() and ex.sync()
    got = sub.getOutputs()[0].getData().reshape(want.shape)
    scale = np.abs(want).max()
    assert np.abs(got - want).max() <= 1e-4 * scale, (np.abs(got - want).max(), scale)
    assert ex.numKernelOps() <= 26
    assert 0.05 < ex.time(5, 20) < 5.0      # ms per inference


# ---- the same files through the host layer's own reader (Graph::importOnnx, C++) ---------
# pet_amd/lib/pet_onnx_driver (tests/cpp/onnx_driver.cc) imports a file, prints the operators
# with the shapes of their outputs and, given an input, runs the graph on the device.
DRIVER = os.path.join(ROOT, "pet_amd", "lib", "pet_onnx_driver")
REFTESTS = os.path.join(ROOT, "pet_amd", "lib", "reftests")


def _driver(*args, **kw):
    import subprocess
    assert os.path.exists(DRIVER), "run __graft_entry__.build()"
    return subprocess.run([DRIVER] + [str(a) for a in args], capture_output=True, text=True,
                          errors="replace", timeout=300, **kw)


def test_native_importer_builds_the_same_graphs(tmp_path):
    from pet_amd import onnx_import
    for name, (data, _) in (("cnn", cnn(np.random.default_rng(0))),
                            ("conv_bn", _conv_bn_model(np.random.default_rng(3))),
                            ("resnet18", _resnet18(np.random.default_rng(18)))):
        path = tmp_path / (name + ".onnx")
        path.write_bytes(data)
        res = _driver(path)
        assert res.returncode == 0, res.stderr[-1000:]
        lines = [ln for ln in res.stdout.splitlines() if "->" in ln]
        want = [op.toString() for op in onnx_import.load(data).graph.getOperators()]
        # the same operators with the same arguments, in the same order (tensor ids and the
        # hashes derived from them differ between two processes: compare without them)
        import re
        strip = lambda s: re.sub(r"\[\d{5,}\]|(input|weight|output|in|out|A|B|C)=\d+,?", "", s)
        assert [strip(ln.split("  ->")[0]) for ln in lines] == [strip(s) for s in want]
    assert sum(ln.startswith("Conv") for ln in lines) == 20            # ResNet-18, BN folded
    assert not any("BatchNorm" in ln for ln in lines)
    assert lines[-1].endswith("[1,1,1000]")


def test_both_readers_take_slice_the_way_numpy_indexes(tmp_path):
    """Slice (opset 10 on: starts / ends / axes / steps as constants): negative positions count
    from the end, positions past the end are clamped, axes may be negative or left out."""
    from pet_amd import onnx_import
    shape = [2, 6, 9, 5]
    probe = np.zeros(shape)
    for starts, ends, axes, index in (
            ([1, 2], [5, 2 ** 62], [1, 2], np.s_[:, 1:5, 2:, :]),
            ([-4, 0], [-1, 3], [-2, -1], np.s_[:, :, -4:-1, 0:3]),
            ([1, 0, 3, 2], [2, 6, 100, -1], None, np.s_[1:2, 0:6, 3:100, 2:-1])):
        w = {"st": np.array(starts, dtype=np.int64), "en": np.array(ends, dtype=np.int64)}
        ins = ["x", "st", "en"]
        if axes is not None:
            w["ax"] = np.array(axes, dtype=np.int64)
            w["sp"] = np.ones(len(axes), dtype=np.int64)
            ins += ["ax", "sp"]
        want = probe[index].shape
        data = ow.model([ow.node("Slice", ins, ["y"])], w, [("x", shape)], [("y", list(want))])
        lo = [sl.indices(n)[0] for sl, n in zip(index, shape)]
        drop = [n - sl.indices(n)[1] for sl, n in zip(index, shape)]
        text = "Slice(begin=[%s],end=[%s])" % (",".join(map(str, lo)), ",".join(map(str, drop)))
        m = onnx_import.load(data)
        assert [op.toString() for op in m.graph.getOperators()] == [text]
        assert tuple(m.tensors["y"].getDims()) == want
        (tmp_path / "slice.onnx").write_bytes(data)
        res = _driver(tmp_path / "slice.onnx")
        assert res.returncode == 0, res.stderr
        assert res.stdout.splitlines()[0] == text + "  -> [%s]" % ",".join(map(str, want))
    for bad in ({"sp": np.array([2, 1], dtype=np.int64)}, {"en": np.array([1, 9], dtype=np.int64)}):
        w = {"st": np.array([1, 2], dtype=np.int64), "en": np.array([5, 9], dtype=np.int64),
             "ax": np.array([1, 2], dtype=np.int64), "sp": np.ones(2, dtype=np.int64)}
        w.update(bad)
        data = ow.model([ow.node("Slice", ["x", "st", "en", "ax", "sp"], ["y"])], w,
                        [("x", shape)], [("y", shape)])
        with pytest.raises(ValueError):
            onnx_import.load(data)
        (tmp_path / "slice.onnx").write_bytes(data)
        assert _driver(tmp_path / "slice.onnx").returncode == 2


def test_native_importer_refuses_what_it_cannot_take(tmp_path):
    bad = tmp_path / "einsum.onnx"
    bad.write_bytes(ow.model([ow.node("Einsum", ["x"], ["y"])], {}, [("x", [2, 2])], [("y", [2, 2])]))
    res = _driver(bad)
    assert res.returncode == 2 and "Einsum is not supported" in res.stderr
    cut = tmp_path / "cut.onnx"
    cut.write_bytes(cnn(np.random.default_rng(0))[0][:-37])
    res = _driver(cut)
    assert res.returncode == 2 and "truncated" in res.stderr
    res = _driver(tmp_path / "missing.onnx")
    assert res.returncode == 2 and "cannot open" in res.stderr


@pytest.mark.gpu
def test_natively_imported_networks_match_torch(tmp_path):
    for name, (data, w), shape, ref in (
            ("cnn", cnn(np.random.default_rng(1)), (1, 3, 16, 16), cnn_reference),
            ("resnet18", _resnet18(np.random.default_rng(18)), (1, 3, 224, 224), _resnet18_torch)):
        x = np.random.default_rng(7).standard_normal(shape).astype(np.float32)
        (tmp_path / (name + ".onnx")).write_bytes(data)
        x.tofile(tmp_path / "in.bin")
        res = _driver(tmp_path / (name + ".onnx"), tmp_path / "in.bin", tmp_path / "out.bin")
        assert res.returncode == 0, res.stderr[-1000:]
        want = ref(x, w)
        got = np.fromfile(tmp_path / "out.bin", dtype=np.float32).reshape(want.shape)
        assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max()


@pytest.mark.gpu
@pytest.mark.parametrize("program", ["import_onnx", "import_onnx_nnet", "import_onnx_cmutator",
                                     "import_onnx_origin", "import_onnx_nnet_depth"])
def test_reference_import_programs_run_unchanged(program, tmp_path):
    """src/Test/import_onnx*.cpp of the reference, compiled unchanged: Graph::importOnnx on a
    model file, SearchEngine::run with the mutation generator / the nnet mutator / CMutator /
    DMutator, CodeEngine::genCode for the best graph (res.cu) and, in some, for the graph as
    given (origin.cu); import_onnx_nnet_depth repeats the nnet search at depths 0 to 8 and
    prints its statistics instead. The reference's importOnnx calls into its Python plug-in and the `onnx`
    package; here it is the host layer's own reader."""
    import subprocess
    exe = os.path.join(REFTESTS, program)
    status = os.path.join(ROOT, "pet_amd", "lib", "refsearch_status.txt")
    if os.path.exists(status) and open(status).read().strip() == "no-reference":
        pytest.skip("the build had no reference tree to compile from")
    assert os.path.exists(exe), "run __graft_entry__.build() where the reference tree is present"
    (tmp_path / "cnn.onnx").write_bytes(cnn(np.random.default_rng(1))[0])
    res = subprocess.run([exe, "cnn.onnx"], capture_output=True, text=True, timeout=600,
                         cwd=str(tmp_path))
    print(res.stdout[-2500:])
    print(res.stderr[-1500:])
    assert "Graph Imported" in res.stdout
    if res.returncode == -11:
        # Generator::markTransType / CMutator::markTransType (src/Mutant/generator.cc:1946-1957,
        # cmutator.cc likewise) dereference the producer of a convolution's input without
        # looking whether there is one; whether a candidate of that form comes up depends on
        # the search's random sampling (import_onnx_cmutator: two runs in three on this model;
        # backtrace taken with a handler linked beside the unchanged program)
        pytest.xfail("upstream's markTransType dereferenced a null producer in this run")
    assert res.returncode == 0
    if program == "import_onnx_nnet_depth":
        assert res.stdout.count("Statistics: maxdepth") == 9
        return
    emitted = (tmp_path / "res.cu").read_text()
    assert emitted.count("pet_hip_conv2d") >= 2 and "pet_hip_softmax" in emitted
    if program == "import_onnx":
        # the program ends with bestGraph->exportOnnx("pet-optimization.onnx"): the file holds
        # the optimised graph, or the exporter said on stderr which operator ONNX cannot say
        written = tmp_path / "pet-optimization.onnx"
        if "exportOnnx" in res.stderr:
            assert "ONNX" in res.stderr and not written.exists()
        else:
            again = _driver(written)
            assert again.returncode == 0, again.stderr[-1000:]
            assert again.stdout.count("Conv") >= 2 and "Softmax" in again.stdout


@pytest.mark.gpu
def test_reference_import_onnx_on_the_benchmark_block(tmp_path):
    """The reference's own pipeline at benchmark configuration 2, unchanged: the dilated
    convolution block (six 3x3 convolutions 512-512-512-512-256-128-64 with ReLU, dilation 2, on
    1x512x64x64) as a model file -> src/Test/import_onnx.cpp: Graph::importOnnx,
    SearchEngine::run (every candidate timed through Operator::perf on the device),
    CodeEngine::genCode. About 90 s of search: runs with PET_SLOW_REFERENCE_PROGRAMS=1."""
    import re
    import subprocess
    if not os.environ.get("PET_SLOW_REFERENCE_PROGRAMS"):
        pytest.skip("a search of about 90 s: set PET_SLOW_REFERENCE_PROGRAMS=1")
    exe = os.path.join(REFTESTS, "import_onnx")
    assert os.path.exists(exe), "run __graft_entry__.build() where the reference tree is present"
    rng = np.random.default_rng(0)
    ch = [512, 512, 512, 512, 256, 128, 64]
    nodes, w, t = [], {}, "x"
    for i in range(6):
        w["w%d" % i] = (rng.standard_normal((ch[i + 1], ch[i], 3, 3)) * 0.01).astype(np.float32)
        nodes.append(ow.node("Conv", [t, "w%d" % i], ["c%d" % i], pads=[2, 2, 2, 2],
                             strides=[1, 1], dilations=[2, 2], kernel_shape=[3, 3]))
        nodes.append(ow.node("Relu", ["c%d" % i], ["r%d" % i]))
        t = "r%d" % i
    (tmp_path / "dilated.onnx").write_bytes(
        ow.model(nodes, w, [("x", [1, 512, 64, 64])], [(t, [1, 64, 64, 64])]))
    res = subprocess.run([exe, "dilated.onnx"], capture_output=True, text=True, timeout=900,
                         cwd=str(tmp_path))
    print(res.stdout[-2500:])
    if res.returncode == -11:
        pytest.xfail("upstream's markTransType dereferenced a null producer in this run")
    assert res.returncode == 0 and "Search Finished" in res.stdout
    origin = float(re.findall(r"Origin Perf: ([0-9.eE+-]+)", res.stdout)[-1])
    best = float(re.findall(r"Best Perf with correction: ([0-9.eE+-]+)", res.stdout)[-1])
    assert 0.3 < best <= origin * 1.001 < 2.0          # ms for the six layers
    emitted = (tmp_path / "res.cu").read_text()
    assert emitted.count("pet_hip_conv2d_ex_f32") == 6 and "pet_hip_activation" not in emitted


def test_native_importer_survives_damaged_files(tmp_path):
    """Seeded damage to valid model files (bytes flipped, runs cut out or duplicated, the
    tail cut off): the reader either imports the result or refuses it with a message; it must
    not crash, hang or hand the builders an argument they divide by."""
    rng = np.random.default_rng(99)
    bases = [cnn(np.random.default_rng(0))[0], _conv_bn_model(np.random.default_rng(3))[0]]
    # structural bytes (keys, lengths, attributes) sit outside the big weight blobs: aim there
    outcomes = {0: 0, 2: 0}
    for trial in range(240):
        data = bytearray(bases[trial % 2])
        kind = trial % 4
        n = len(data)
        if kind == 0:
            for _ in range(int(rng.integers(1, 4))):
                data[int(rng.integers(0, n))] = int(rng.integers(0, 256))
        elif kind == 1:
            # the node list is at the front of the graph message
            for _ in range(int(rng.integers(1, 6))):
                data[int(rng.integers(0, min(n, 900)))] ^= 1 << int(rng.integers(0, 8))
        elif kind == 2:
            a = int(rng.integers(0, n - 8))
            del data[a:a + int(rng.integers(1, 40))]
        else:
            a = int(rng.integers(0, min(n, 900)))
            data[a:a] = data[a:a + int(rng.integers(1, 30))]
        path = tmp_path / "damaged.onnx"
        path.write_bytes(bytes(data))
        res = _driver(path)
        assert res.returncode in (0, 2), (trial, res.returncode, res.stderr[-300:])
        outcomes[res.returncode] += 1
    assert outcomes[2] > 20 and outcomes[0] > 20, outcomes


def test_operands_a_builder_rejects_are_a_python_error():
    """The operator constructors assert on invalid operands, as the reference's do; through the
    Python module that is a ValueError (a C++ assertion would end the interpreter)."""
    from pet_amd import onnx_import
    cm = onnx_import._module()
    g = cm.Graph()
    x, w = g.tensor([1, 3, 8, 8], "FLOAT"), g.tensor([4, 5, 3, 3], "FLOAT")
    w.setWeight()
    with pytest.raises(ValueError):
        g.conv(x, w, 1, 1, 1, 1, 1, 1, None)      # 3 input channels, filters over 5
    with pytest.raises(ValueError):                # the same through a model file
        onnx_import.load(ow.model([ow.node("Conv", ["x", "w"], ["y"], pads=[1, 1, 1, 1])],
                                  {"w": np.zeros((4, 5, 3, 3), np.float32)},
                                  [("x", [1, 3, 8, 8])], [("y", [1, 4, 8, 8])]))
