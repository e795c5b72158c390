"""In-tree build of the HIP library (lib/libtvx_hip.so) and of the C++ tim::vx
runtime on top of it (lib/libtim-vx.so). hipcc cross-compiles gfx950 without a
GPU, so this runs in the build container; the results travel to the GPU box."""
import glob
import os
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.dirname(PKG_DIR)
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-I", os.path.join(REPO, "include"), "-I", os.path.join(PKG_DIR, "csrc"),
]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass warns that it does not know the packed-fp32 feature: harmless
    out = "\n".join(l for l in p.stdout.splitlines() if "packed-fp32-ops" not in l)
    if p.returncode != 0:
        sys.stderr.write(out + "\n")
        raise RuntimeError("build step failed: " + " ".join(cmd))
    if verbose and out.strip():
        print(out)


def build_hip(verbose=False):
    os.makedirs(os.path.join(PKG_DIR, "lib"), exist_ok=True)
    obj_dir = os.path.join(PKG_DIR, "lib", "obj")
    os.makedirs(obj_dir, exist_ok=True)
    objs = []
    procs = []
    for src in sorted(glob.glob(os.path.join(PKG_DIR, "csrc", "*.hip"))):
        obj = os.path.join(obj_dir, os.path.basename(src)[:-4] + ".o")
        objs.append(obj)
        cmd = [HIPCC] + HIP_FLAGS + ["-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    for cmd, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            sys.stderr.write(out + "\n")
            raise RuntimeError("build step failed: " + " ".join(cmd))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o",
          os.path.join(PKG_DIR, "lib", "libtvx_hip.so")] + objs, verbose)
    # the benchmark's calibration kernels: a library of their own, outside the operator library's C ABI
    _run([HIPCC] + HIP_FLAGS + ["-shared", os.path.join(PKG_DIR, "bench_aids", "calibrate.hip"), "-o",
                               os.path.join(PKG_DIR, "lib", "libtvx_calibrate.so")], verbose)


def build_runtime(verbose=False):
    """The tim::vx C++ runtime: host-only C++ that reaches the GPU through the C ABI."""
    srcs = sorted(glob.glob(os.path.join(PKG_DIR, "src", "*.cc")))
    if not any(s.endswith("hip_executor.cc") for s in srcs):
        return
    _run(["g++", "-std=c++17", "-O2", "-fPIC", "-shared", "-Wall",
          "-I", os.path.join(PKG_DIR, "include"), "-I", os.path.join(PKG_DIR, "src"),
          "-I", os.path.join(REPO, "include")] + srcs +
         ["-L", os.path.join(PKG_DIR, "lib"), "-ltvx_hip", "-Wl,-rpath,$ORIGIN",
          "-o", os.path.join(PKG_DIR, "lib", "libtim-vx.so")], verbose)
    # the graph-file runner: an application of the public API, linked like any other
    _run(["g++", "-std=c++17", "-O2", "-Wall", "-pthread", "-I", os.path.join(PKG_DIR, "include"),
          os.path.join(PKG_DIR, "src", "tools", "graph_runner.cc"),
          "-L", os.path.join(PKG_DIR, "lib"), "-ltim-vx", "-ltvx_hip", "-Wl,-rpath,$ORIGIN",
          "-o", os.path.join(PKG_DIR, "lib", "tvx_graph_runner")], verbose)


def build_all(verbose=False):
    build_hip(verbose)
    build_runtime(verbose)


if __name__ == "__main__":
    build_all(verbose=True)
