#!/usr/bin/env python3
"""Regenerate tests/golden/*.json from the reference's own operator tests.

Each reference test file is compiled in place (never copied) against this
repository's tim::vx headers and host-side front end, with a recording
Executor and a recording stand-in for the gtest macros (capture/). Running the
result executes every TEST body: the reference's helpers quantize the inline
vectors exactly as they would for the vendor simulator, and every
EXPECT_EQ / ArraysMatch becomes one JSON case holding the graph, the input and
constant data and the expected output with its tolerance.

Needs /root/reference (present only in the build container); the committed
JSON files are what the test-suite reads.
"""
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.dirname(os.path.dirname(HERE))
REF = os.environ.get("TVX_REFERENCE", "/root/reference")
PKG = os.path.join(REPO, "tim-vx_amd")

SOURCES = {
    "conv2d": "src/tim/vx/ops/conv2d_test.cc",
    "depthwise_conv": "src/tim/vx/ops/depthwiseConv_test.cc",
    "grouped_conv2d": "src/tim/vx/ops/groupedconv2d_test.cc",
    "conv1d": "src/tim/vx/ops/conv1d_test.cc",
    "grouped_conv1d": "src/tim/vx/ops/groupedconv1d_test.cc",
    "deconv1d": ("src/tim/vx/ops/deconv1d_test.cc", ["DeConv1d"]),  # (the file's other suite needs LeakyRelu)
    "fullyconnected": "src/tim/vx/ops/fullyconnected_test.cc",
    "max_pool": "src/tim/vx/ops/max_pool_test.cc",
    "avg_pool": "src/tim/vx/ops/avg_pool_test.cc",
    "softmax": "src/tim/vx/ops/softmax_test.cc",
    "transpose": "src/tim/vx/ops/transpose_test.cc",
    "deconv2d": "src/tim/vx/ops/deconv2d_test.cc",
    # (file, test suite): only the TEST(suite, ...) bodies of a file that also tests operators outside this path
    "dataconvert": ("src/tim/vx/ops/simple_operations_test.cc", ["DataConvert"]),
    # the source graphs of the layout-inference tests that stay inside this path
    "layout_inference": ("src/tim/transform/layout_inference_test.cc", ["LayoutInference", "GroupedConv2d", "FC"]),
}


def select_suite(path, suites):
    """The file's preprocessor lines plus the TEST(suite, ...) bodies of the named suites, as text for the
    compiler's stdin (nothing of the reference is written to disk)."""
    suite = "|".join(re.escape(s) for s in suites)
    text = open(path).read()
    out = [l for l in text.splitlines() if l.startswith("#include")]
    pos = 0
    while True:
        m = re.search(r"^TEST\(\s*(?:%s)\s*,[^)]*\)\s*\{" % suite, text[pos:], re.M)
        if not m:
            break
        start = pos + m.start()
        depth, i = 0, pos + m.end() - 1
        while True:
            if text[i] == "{":
                depth += 1
            elif text[i] == "}":
                depth -= 1
                if depth == 0:
                    break
            i += 1
        out.append(text[start:i + 1])
        pos = i + 1
    return "\n".join(out) + "\n"


def main():
    build = os.path.join(HERE, "capture", "_build")
    os.makedirs(build, exist_ok=True)
    cxx = ["g++", "-std=c++17", "-O1", "-w"]
    product_inc = ["-I", os.path.join(PKG, "include"), "-I", os.path.join(PKG, "src")]
    # the recording stand-ins (gtest, test_utils, the LayoutInference shim) shadow the real headers for the
    # reference's test sources and the recorder only; the runtime's own sources are built without them
    capture_inc = ["-I", os.path.join(HERE, "capture")] + product_inc + [
        "-I", REF, '-DTVX_REF_TEST_UTILS="%s"' % os.path.join(REF, "src/tim/vx/test_utils.h")]
    objs = []
    for f in ("frontend.cc", "graph_passes.cc", "layout_inference.cc"):
        obj = os.path.join(build, f.replace(".cc", ".o"))
        subprocess.check_call(cxx + product_inc + ["-c", os.path.join(PKG, "src", f), "-o", obj])
        objs.append(obj)
    main_obj = os.path.join(build, "capture_main.o")
    subprocess.check_call(cxx + capture_inc + ["-c", os.path.join(HERE, "capture", "capture_main.cc"), "-o", main_obj])
    objs.append(main_obj)
    for name, rel in SOURCES.items():
        exe = os.path.join(build, "capture_" + name)
        test_obj = os.path.join(build, "test_" + name + ".o")
        print("building", name, flush=True)
        if isinstance(rel, tuple):
            path = os.path.join(REF, rel[0])
            cmd = cxx + capture_inc + ["-I", os.path.dirname(path), "-x", "c++", "-c", "-", "-o", test_obj]
            subprocess.run(cmd, input=select_suite(path, rel[1]).encode(), check=True)
        else:
            subprocess.check_call(cxx + capture_inc + ["-c", os.path.join(REF, rel), "-o", test_obj])
        subprocess.check_call(cxx + [test_obj] + objs + ["-o", exe])
        out = os.path.join(HERE, name + ".json")
        subprocess.check_call([exe, out])
        print("wrote", out, os.path.getsize(out), "bytes", flush=True)


if __name__ == "__main__":
    sys.exit(main())
