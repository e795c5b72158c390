"""The host side of the C++ runtime without a GPU: front end, compile passes (ordering, verification,
shape inference) and layout inference, linked with an executor that does nothing
(tests/host_probe/host_probe.cc). What is checked is structure - which operators the rewritten graph
holds, in which order, with which inferred shapes and pads - not tensor values."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.dirname(HERE)
PKG = os.path.join(REPO, "tim-vx_amd")


@pytest.fixture(scope="module")
def probe_output(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("host_probe") / "host_probe")
    src = [os.path.join(HERE, "host_probe", "host_probe.cc")] + [
        os.path.join(PKG, "src", f) for f in ("frontend.cc", "graph_passes.cc", "layout_inference.cc")]
    subprocess.check_call(["g++", "-std=c++17", "-O0", "-w", "-I", os.path.join(PKG, "include"),
                           "-I", os.path.join(PKG, "src")] + src + ["-o", exe])
    r = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=60)
    assert r.returncode == 0, r.stderr
    graphs, cur = {}, None
    for line in r.stdout.splitlines():
        if line.startswith("graph "):
            _, name, comp = line.split()
            cur = graphs.setdefault(name, {"compiled": comp == "compile=1", "lines": []})
        else:
            cur["lines"].append(line.strip())
    return graphs, r.stderr


def test_nhwc_network_is_rewritten_with_two_permutes(probe_output):
    graphs, _ = probe_output
    g = graphs["nhwc_net"]
    assert g["compiled"]
    # CWHN {8, 12, 10, 2} -> WHCN once in front of the convolution; conv (SAME pads resolved), Relu6 and the
    # pooling run in WHCN back to back; one permute back in front of Reshape, which wants the source order;
    # TRANSIENT tensors were declared without shapes
    assert g["lines"][:8] == [
        "TRANSPOSE perm 1 2 0 3 -> 12 10 8 2",
        "CONV2D pad 1 1 1 1 -> 12 10 16 2",
        "RELU6 -> 12 10 16 2",
        "POOL pad 0 0 0 0 -> 6 5 16 2",
        "TRANSPOSE perm 2 0 1 3 -> 16 6 5 2",
        "RESHAPE -> 480 2",
        "FCL -> 10 2",
        "SOFTMAX axis 0 -> 10 2"]
    # the graph's input and output keep the shapes the application declared
    assert g["lines"][8] == "io_map 2 input_shape 8 12 10 2 output_shape 10 2"


def test_source_graph_with_cwhn_operators_does_not_compile(probe_output):
    graphs, log = probe_output
    assert not graphs["nhwc_net_source"]["compiled"]
    assert "only WHCN activations are supported" in log


def test_softmax_axis_follows_the_layout(probe_output):
    graphs, _ = probe_output
    g = graphs["softmax_axis"]
    assert g["compiled"]
    # axis 0 of the CWHN source (channels) is axis 2 of the WHCN tensor the rewritten Softmax sees; the
    # graph OUTPUT gets its source shape back through a permute
    assert g["lines"] == ["TRANSPOSE perm 1 2 0 3 -> 8 8 6 1", "POOL pad 0 0 0 0 -> 4 4 6 1",
                          "SOFTMAX axis 2 -> 4 4 6 1", "TRANSPOSE perm 2 0 1 3 -> 6 4 4 1"]


def test_shape_inference_of_deconv_transpose_dataconvert(probe_output):
    graphs, _ = probe_output
    g = graphs["deconv_transpose_convert"]
    assert g["compiled"]
    # DeConv2d: (in - 1) * stride + k - pads + output_padding (vsi_nn_op_deconvolution.c:217-218)
    assert g["lines"] == ["DECONV2D pad 1 1 1 1 -> 10 14 6 2", "TRANSPOSE perm 2 0 1 3 -> 6 10 14 2",
                          "DATACONVERT -> 6 10 14 2"]


def test_transpose_rejects_a_non_permutation(probe_output):
    graphs, log = probe_output
    assert not graphs["bad_perm"]["compiled"]
    assert "perm is not a permutation" in log


def test_grouped_conv_same_padding_with_stride(probe_output):
    graphs, _ = probe_output
    g = graphs["grouped_same_stride2"]
    # SAME: out = ceil(9 / 2) = 5, total pad (5 - 1) * 2 + 3 - 9 = 2, split 1 / 1 (vsi_nn_util.c:221-235)
    assert g["compiled"] and g["lines"] == ["CONV2D pad 1 1 1 1 -> 5 5 8 1"]
