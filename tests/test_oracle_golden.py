"""The CPU oracle against every golden vector the reference's own tests hold for
this path (recorded into tests/golden/*.json by tests/golden/make_fixtures.py)."""
import numpy as np
import pytest

import tvx_case as TC

CASES = TC.all_cases()


def test_fixture_inventory():
    # 24 conv2d tests (one of them loops over 66 input sizes), 16 depthwise, 3 grouped, 3 one-dimensional,
    # 2 fully-connected, 3 max-pool, 8 avg-pool, 6 softmax, 2 transpose, 3 DataConvert, 4 layout-inference source graphs, 2 DeConv2d, 2 GroupedConv1d, 3 DeConv1d (the file's fourth test needs LeakyRelu); the two int16 dynamic-fixed-point
    # conv tests of the reference are outside this path and not recorded.
    per_file = {}
    for n, c in CASES:
        per_file.setdefault(n, set()).add(c["test"])
    assert {k: len(v) for k, v in per_file.items()} == {
        "conv2d": 24, "depthwise_conv": 16, "grouped_conv2d": 3, "conv1d": 3, "fullyconnected": 2, "max_pool": 3, "avg_pool": 8, "softmax": 6,
        "transpose": 2, "dataconvert": 3, "layout_inference": 4, "deconv2d": 2, "grouped_conv1d": 2, "deconv1d": 3}
    assert len(CASES) == 146


@pytest.mark.parametrize("item", CASES, ids=TC.case_id)
def test_oracle_matches_reference_golden(item, oracle):
    _, case = item
    out = oracle.run_case(case)
    assert TC.matches(case, out), (out[:16], TC.golden_of(case)[:16])


def test_declared_shapes_equal_inferred(oracle):
    # Shapes in the fixtures are the front end's inferred/validated ones; the
    # operator's resolved padding must reproduce the declared output extent.
    for _, case in CASES:
        op = case["ops"][0]
        if op["kind"] != "CONV2D":
            continue
        t = {t["id"]: t for t in case["tensors"]}
        x, w, y = t[op["inputs"][0]], t[op["inputs"][1]], t[op["outputs"][0]]
        a = op["attrs"]
        xs, ws, ys = oracle._conv_shapes(a, x["shape"], w["shape"], y["shape"])  # Conv1d: rows of height one
        for ax in (0, 1):
            ke = (ws[ax] - 1) * a["dilation"][ax] + 1
            inferred = (xs[ax] + a["pad"][2 * ax] + a["pad"][2 * ax + 1] - ke) // a["stride"][ax] + 1
            assert ys[ax] <= inferred
