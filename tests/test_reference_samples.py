"""Drop-in proof on the reference's own applications: its samples are compiled WHERE THEY LIE (nothing is copied;
the test is skipped where /root/reference is absent) against this repository's tim::vx headers and linked with
libtim-vx.so. What links here is what an existing TIM-VX application needs from the library: the same namespaces,
class layouts, constructors and mangled names."""
import os
import subprocess

import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(REPO, "tim-vx_amd")
REF = os.environ.get("TVX_REFERENCE", "/root/reference")
LIB = os.path.join(PKG, "lib")

pytestmark = pytest.mark.skipif(not os.path.isdir(os.path.join(REF, "samples")) or
                                not os.path.exists(os.path.join(LIB, "libtim-vx.so")),
                                reason="needs the reference's sources and the built runtime")

CXX = ["g++", "-std=c++14", "-O0", "-I", os.path.join(PKG, "include")]
LINK = ["-L", LIB, "-ltim-vx", "-ltvx_hip", "-Wl,-rpath," + LIB, "-Wl,--no-undefined", "-pthread"]


def _run(cmd):
    p = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, " ".join(cmd) + "\n" + p.stderr[-3000:]


@pytest.mark.parametrize("sample", ["lenet/lenet_asymu8.cc", "benchmark_test/benchmark_test.cc",
                                    "multi_thread_test/multi_thread_test.cc"])
def test_sample_application_compiles_and_links(tmp_path, sample):
    """samples/lenet/lenet_asymu8.cc:117-316 (LeNet through Conv2d / Pool2d / FullyConnected / Relu / Softmax),
    samples/benchmark_test/benchmark_test.cc:33-206, samples/multi_thread_test/multi_thread_test.cc (two threads
    around the same graph builder) as whole programs."""
    src = os.path.join(REF, "samples", sample)
    _run(CXX + ["-I", os.path.dirname(src), src, "-o", str(tmp_path / "app")] + LINK)


def test_multi_device_model_builders_compile_and_link(tmp_path):
    """samples/multi_device/vx_lenet.cc and vx_mobilenet.cc (:570-700: a MobileNet of Conv2d, depthwise Conv2d, Pool2d,
    FullyConnected, Softmax, Reshape built by hand) as one shared object with no undefined symbol left, and the
    demo that drives them through the platform:: API as an object file."""
    md = os.path.join(REF, "samples", "multi_device")
    objs = []
    for name in ("vx_lenet", "vx_mobilenet", "multi_device_demo"):
        obj = str(tmp_path / (name + ".o"))
        _run(CXX + ["-fPIC", "-c", "-I", md, os.path.join(md, name + ".cc"), "-o", obj])
        objs.append(obj)
    _run(["g++", "-shared", "-o", str(tmp_path / "libmodels.so")] + objs[:2] + LINK)
