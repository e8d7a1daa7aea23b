"""GraphBase::exportOnnx (pet_amd/host/src/onnx_export.cc): the ONNX file a graph is written to.

The reference's exporter (src/Graph/graph.cc:1189-1340 with python/cpp_plugin/export_onnx.py)
needs the `onnx` package, which this image does not have: the checks here are that the file is
read back by both readers of this backend (the Python one in pet_amd/onnx_import.py and the
native one behind the driver) as the same operators, and, on the device, that the re-imported
graph computes what the exported one does and what torch computes for the same network.
"""
import os
import re
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(__file__))
from test_onnx_import import (DRIVER, _driver, _resnet18, _resnet18_torch, cnn,  # noqa: E402
                              cnn_reference)

pytestmark = pytest.mark.skipif(not os.path.exists(DRIVER), reason="host layer not built")

_IDS = re.compile(r"\[\d{5,}\]|(input|weight|output|in|out|A|B|C)=\d+,?")


def _ops(text_or_graph):
    """Operators without the tensor ids and the hashes derived from them."""
    if isinstance(text_or_graph, str):
        lines = [ln.split("  ->")[0] for ln in text_or_graph.splitlines() if "->" in ln]
    else:
        lines = [op.toString() for op in text_or_graph.getOperators()]
    return [_IDS.sub("", ln) for ln in lines]


def _mixed_graph(mod, rng):
    """A graph of the operators no importer produces as such: a convolution with a fused
    activation, an unfolded batch normalisation, pad, slice, extend, a transpose that splits
    and merges, a three-operand add, a matmul with a transposed constant and a bias."""
    g = mod.Graph()
    w = {}

    def weight(name, arr):
        t = g.tensor(list(arr.shape))
        t.setWeight()
        t.setData(np.ascontiguousarray(arr, dtype=np.float32))
        w[name] = arr.astype(np.float32)
        return t

    x = g.tensor([1, 4, 8, 8])
    conv = g.conv(x, weight("w1", rng.standard_normal((8, 4, 3, 3)) * 0.3), 1, 1, 1, 1, 1, 1,
                  weight("b1", rng.standard_normal(8) * 0.1))
    conv.setAct(1)
    t = g.batchnorm(conv.getOutput(), weight("bn_s", rng.uniform(0.5, 1.5, 8)),
                    weight("bn_b", rng.standard_normal(8) * 0.1),
                    weight("bn_m", rng.standard_normal(8) * 0.1),
                    weight("bn_v", rng.uniform(0.5, 1.5, 8))).getOutput()
    t = g.pad(t, [0, 0, 1, 1], [0, 0, 1, 1]).getOutput()            # [1, 8, 10, 10]
    t = g.slice(t, [0, 0, 1, 0], [0, 0, 1, 2]).getOutput()          # [1, 8, 8, 8]
    # rows split in two halves that move into the batch, and back (the reference's
    # batch <-> height transformation, src/Mutant/generator.cc transpose mutations)
    h2n = g.transpose(t, 2, [[0, 2], 1, -1, 3], -2).getOutput()     # [2, 8, 4, 8]
    t2 = g.transpose(h2n, 0, [0, 1, [-1, 2], 3], 2).getOutput()     # [1, 8, 8, 8]
    s = g.add([t, t2, t2]).getOutput()
    e = g.tensor([1, 24, 8, 8])
    g.extend(s, e, 1, 2)
    p = g.tensor([1, 24, 4, 4])
    g.avgpool(e, p, 2, 2, 0, 0, 2, 2)
    f = g.tensor([1, 1, 384])
    g.reshape(p, f)
    y = g.matmul(f, weight("fc", rng.standard_normal((1, 10, 384)) * 0.05), False, True,
                 weight("fc_b", rng.standard_normal(10) * 0.1)).getOutput()
    g.updateConnection()
    return g, x, y, w


def _mixed_torch(x, w):
    import torch
    import torch.nn.functional as F
    tw = {k: torch.from_numpy(v) for k, v in w.items()}
    t = F.relu(F.conv2d(torch.from_numpy(x), tw["w1"], tw["b1"], padding=1))
    t = F.batch_norm(t, tw["bn_m"], tw["bn_v"], tw["bn_s"], tw["bn_b"], False, 0.0, 1e-5)
    t = F.pad(t, (1, 1, 1, 1))[:, :, 1:9, 0:8]
    s = 3 * t
    e = torch.cat([s, s, s], 1)
    p = F.avg_pool2d(e, 2, 2)
    return (p.reshape(1, 1, 384) @ tw["fc"][0].T + tw["fc_b"]).numpy()


def test_exported_files_are_read_back_as_the_same_operators(tmp_path):
    from pet_amd import onnx_import
    for name, data in (("cnn", cnn(np.random.default_rng(0))[0]),
                       ("resnet18", _resnet18(np.random.default_rng(18))[0])):
        src, dst = tmp_path / (name + ".onnx"), tmp_path / (name + ".out.onnx")
        src.write_bytes(data)
        res = _driver(src, "--export", dst)
        assert res.returncode == 0, res.stderr[-1000:]
        first = _ops(res.stdout)
        again = _driver(dst)
        assert again.returncode == 0, again.stderr[-1000:]
        native = _ops(again.stdout)
        python = _ops(onnx_import.load(dst.read_bytes()).graph)
        assert native == python
        # the one difference: Gemm's transposed right-hand side and bias, a Matmul(A, B^T, bias)
        # in the first graph, is written as MatMul on the transposed weights followed by Add
        at = next(i for i, ln in enumerate(first) if ln.startswith("Matmul([A,B^T"))
        assert native[at].startswith("Matmul([A,B,") and native[at + 1].startswith("Add")
        assert native[:at] == first[:at] and native[at + 2:] == first[at + 1:]


def test_exporter_writes_every_layout_operator(tmp_path):
    from pet_amd import onnx_import
    mod = onnx_import._module()
    g, x, y, w = _mixed_graph(mod, np.random.default_rng(5))
    path = tmp_path / "mixed.onnx"
    assert g.exportOnnx(str(path))
    m = onnx_import.load(path.read_bytes())
    assert len(m.inputs) == 1 and m.tensors[m.inputs[0]].getDims() == [1, 4, 8, 8]
    names = [ln.split("(")[0].split("[")[0] for ln in _ops(m.graph)]
    assert names == ["Conv", "Activation", "BatchNorm", "Pad", "Slice",
                     "Reshape", "Transpose", "Reshape",             # split, reorder, merge
                     "Reshape", "Transpose", "Reshape",
                     "Add", "Add", "Concat", "AvgPool", "Reshape", "Matmul", "Add"], names
    assert m.tensors[m.outputs[0]].getDims() == [1, 1, 10]
    # the weights travel with their values
    stored = sorted(v.size for v in m.weights.values() if v.dtype == np.float32)
    assert stored[-1] == 10 * 384 and 8 * 4 * 3 * 3 in stored
    got_fc = next(v for v in m.weights.values() if v.size == 3840)
    np.testing.assert_array_equal(got_fc.reshape(384, 10), w["fc"][0].T)
    res = _driver(path)                                             # the native reader as well
    assert res.returncode == 0 and _ops(res.stdout) == _ops(m.graph)


def test_exporter_refuses_what_onnx_cannot_say(tmp_path, capfd):
    from pet_amd import onnx_import
    mod = onnx_import._module()
    g = mod.Graph()
    x = g.tensor([1, 4, 8, 8])
    g.transpose(x, 2, [[0, 2], 1, -1, 3], -2).getOutput()
    g.updateConnection()
    assert g.exportOnnx(str(tmp_path / "ok.onnx"))
    g2 = mod.Graph()
    q, k = g2.tensor([2, 16, 8]), g2.tensor([2, 16, 8])
    g2.g2bmm(q, k, g2.tensor([2, 16, 7]), 3, 1)
    g2.updateConnection()
    assert not g2.exportOnnx(str(tmp_path / "no.onnx"))
    assert "no ONNX counterpart" in capfd.readouterr().err
    assert not g.exportOnnx(str(tmp_path / "missing_dir" / "x.onnx"))


@pytest.mark.gpu
def test_exported_networks_compute_what_torch_does(tmp_path):
    for name, (data, w), shape, ref in (
            ("cnn", cnn(np.random.default_rng(1)), (1, 3, 16, 16), cnn_reference),
            ("resnet18", _resnet18(np.random.default_rng(18)), (1, 3, 224, 224), _resnet18_torch)):
        x = np.random.default_rng(7).standard_normal(shape).astype(np.float32)
        src, dst = tmp_path / (name + ".onnx"), tmp_path / (name + ".out.onnx")
        src.write_bytes(data)
        x.tofile(tmp_path / "in.bin")
        assert _driver(src, "--export", dst).returncode == 0
        res = _driver(dst, tmp_path / "in.bin", tmp_path / "out.bin")
        assert res.returncode == 0, res.stderr[-1000:]
        want = ref(x, w)
        got = np.fromfile(tmp_path / "out.bin", dtype=np.float32).reshape(want.shape)
        assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max()


@pytest.mark.gpu
def test_exported_layout_operators_compute_what_torch_does(tmp_path):
    from pet_amd import onnx_import
    mod = onnx_import._module()
    g, x, y, w = _mixed_graph(mod, np.random.default_rng(5))
    path = tmp_path / "mixed.onnx"
    assert g.exportOnnx(str(path))
    xin = np.random.default_rng(6).standard_normal((1, 4, 8, 8)).astype(np.float32)
    want = _mixed_torch(xin, w)
    m = onnx_import.load(path.read_bytes())
    sub, feeds = m.subgraph()
    assert list(feeds) == m.inputs
    feeds[m.inputs[0]].setData(xin)
    assert sub.compute()
    got = np.asarray(sub.getOutputs()[0].getData()).reshape(want.shape)
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4)
    # and through the native reader
    xin.tofile(tmp_path / "in.bin")
    res = _driver(path, tmp_path / "in.bin", tmp_path / "out.bin")
    assert res.returncode == 0, res.stderr[-1000:]
    got = np.fromfile(tmp_path / "out.bin", dtype=np.float32).reshape(want.shape)
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4)
