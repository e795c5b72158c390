"""The benchmark configurations at their full sizes through the tim::vx C++ API, whole outputs
against the oracle: MobileNetV2 at batch 64 / 224x224 (and the same network cut after single
layers, so that a wrong byte inside the network cannot hide behind the average pool), LeNet at
batch 1 and 256 with seeded synthetic parameters."""
import importlib

import numpy as np
import pytest

GF = importlib.import_module("tim-vx_amd.graphfile")
GRAPHS = importlib.import_module("tim-vx_amd.graphs")

pytestmark = pytest.mark.gpu


def _check(graphs, tmp_path, values, env=None):
    out, info, log = GF.run_graphs(graphs, str(tmp_path), env=env, timeout=900)
    for g, got in zip(graphs, out):
        assert got is not None, (g["test"], info.get(g["test"]), log[-2000:])
        want = values[g["output"]]
        assert got.dtype == want.dtype and np.array_equal(got, want), \
            (g["test"], int((got != want).sum()), np.flatnonzero(got != want)[:8])
    return log


def test_mobilenet_v2_batch64_224_bit_exact(tmp_path, oracle):
    g = GRAPHS.mobilenet_v2(batch=64, res=224)
    values = oracle.run_graph(g, keep_all=True)
    assert len(np.unique(values[g["output"]])) > 100
    log = _check([g], tmp_path / "full", values, env={"VSI_NN_LOG_LEVEL": "3"})
    plan = [l for l in log.splitlines() if "uid" in l and "->" in l]
    assert sum("pwconv_add_i8" in l or "pwconv_add_blocked_i8" in l for l in plan) == 10, plan
    # the 7 x 7 stage runs between channel-blocked tensors: the stride-2 depthwise convolution in front writes the
    # first of them (no copy), the whole-plane average leaves the stage
    assert not any("layout_to_blocked" in l for l in plan) and sum("dwconv_planes_to_blocked_i8" in l for l in plan) == 1, plan
    assert sum("_blocked_i8" in l for l in plan) == 13, plan
    # the network cut behind single operators: first convolution, expansions / depthwise / projections of every
    # resolution (112, 56, 28, 14, 7), residual Adds, the last 1x1 convolution
    cuts = []
    for i in (1, 4, 6, 8, 11, 15, 19, 22, 26, 34, 36, 39, 43, 53, 62, 72, 76, 79, 89, 94, 96, 97):
        o = g["ops"][i]
        nxt = g["ops"][i + 1] if i + 1 < len(g["ops"]) else None
        assert not (o["kind"] == "CONV2D" and nxt and nxt["kind"] == "RELU6" and nxt["inputs"][0] == o["outputs"][0]), i
        cuts.append(GRAPHS.cut_at(g, o["outputs"][0]))
    for k in range(0, len(cuts), 6):   # a few graphs per runner process: the largest outputs are 77 MB each
        _check(cuts[k:k + 6], tmp_path / ("cuts%d" % k), values)


@pytest.mark.parametrize("batch", [1, 256])
def test_lenet_with_seeded_random_parameters(tmp_path, oracle, batch):
    g = GRAPHS.lenet_random(batch=batch)
    values = oracle.run_graph(g, keep_all=True)
    ts = {t["id"]: t for t in g["tensors"]}
    assert len(np.unique(values[g["logits"]])) >= (8 if batch == 1 else 100)
    # every quantized tensor of the network, bit for bit: the graph cut behind each operator
    cuts = [GRAPHS.cut_at(g, o["outputs"][0]) for o in g["ops"][:-1] if o["kind"] != "FCL" or
            o["outputs"][0] == g["logits"]]   # (the first FullyConnected is fused with its Relu: cut behind the Relu)
    assert all(ts[c["output"]]["dtype"] == "UINT8" for c in cuts)
    _check(cuts, tmp_path, values)
    got, info, log = GF.run_graphs([g], str(tmp_path / "softmax"))
    assert got[0] is not None, (info, log[-2000:])
    assert np.allclose(got[0], values[g["output"]], rtol=0, atol=1e-6)
