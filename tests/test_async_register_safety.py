"""The FullyConnected MFMA kernel fetches operand fragments with inline-assembly loads and waits
for them with explicit s_waitcnt (the compiler's own wait insertion would serialise the
prefetch). To the compiler such a load is complete as soon as it is issued, so nothing stops
it from giving the destination registers another job while the data is still on its way -
which corrupts whatever lands there (an address, in the worst case: a memory fault on the
GPU). This test compiles the kernel to assembly (no GPU needed) and checks every variant:
between an asynchronous load and the first read of its destination, nothing else may write
that register; loops are followed once around their back-edge."""
import os
import re
import subprocess

import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(REPO, "tim-vx_amd", "csrc")
HIPCC = "/opt/rocm/bin/hipcc"


def _regs(tok):
    tok = tok.rstrip(",")
    m = re.match(r"v\[(\d+):(\d+)\]", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"v(\d+)$", tok)
    return {int(m.group(1))} if m else set()


def unconsumed_overwrites(asm_text, kernel_pattern):
    """[(kernel, line, register)] for writes that hit a register with an asynchronous load in
    flight (issued from an inline-assembly block) before anything has read it."""
    lines = asm_text.split("\n")
    starts = [i for i, l in enumerate(lines) if re.match(r"^_ZN3tvx\S*" + kernel_pattern + r"\S*: ", l)]
    found, kernels = [], 0
    for s in starts:
        e = s
        while "s_endpgm" not in lines[e]:
            e += 1
        body = lines[s:e]
        labels = {l.split(":")[0]: i for i, l in enumerate(body) if re.match(r"^\.LBB\S+:", l)}
        unrolled = []
        for i, l in enumerate(body):
            unrolled.append(l)
            m = re.match(r"\s*s_cbranch_\S+\s+(\.LBB\S+)", l)
            if m and m.group(1) in labels and labels[m.group(1)] < i:
                unrolled.extend(body[labels[m.group(1)]:i + 1])
        kernels += 1
        in_flight = {}
        prev = ""
        for i, raw in enumerate(unrolled):
            l = raw.strip()
            if not l or l[0] in ";.":
                prev = l if l.startswith(";;#ASM") else prev
                continue
            parts = l.replace(",", " ").split()
            op = parts[0]
            is_async = prev.startswith(";;#ASMSTART") and op in ("global_load_dwordx4", "ds_read_b128")
            prev = ""
            if is_async:
                for r in _regs(parts[1]):
                    in_flight[r] = True
                continue
            if op == "s_waitcnt" and "vmcnt(0)" in l and "lgkmcnt(0)" in l:
                in_flight = {}
                continue
            for tok in parts[2:]:
                for r in _regs(tok):
                    in_flight.pop(r, None)
            if op.startswith(("v_mfma", "s_", "global_load_lds", "ds_write", "global_store", "scratch_store")):
                continue
            for r in (_regs(parts[1]) if len(parts) > 1 else ()):
                if r in in_flight:
                    found.append((lines[s].split(":")[0][-48:], l, r))
    return kernels, found


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_fc_mfma_async_loads_keep_their_registers(tmp_path):
    out = str(tmp_path / "fc.s")
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "-I", os.path.join(REPO, "include"), "-I", CSRC, "-S", "--cuda-device-only",
           os.path.join(CSRC, "fc_mfma_i8.hip"), "-o", out]
    subprocess.run(cmd, check=True, capture_output=True, timeout=600)
    kernels, found = unconsumed_overwrites(open(out).read(), "FcMfmaKernel")
    assert kernels >= 13  # every template instance of the tiled kernel
    assert not found, found[:5]


def test_checker_sees_a_planted_hazard():
    planted = "\n".join([
        "_ZN3tvx1_FcMfmaKernelIXEEv: ; @k",
        "\t;;#ASMSTART", "\tglobal_load_dwordx4 v[4:7], v[2:3], off offset:0", "\t;;#ASMEND",
        "\tv_add_u32_e32 v5, 1, v9",   # v5 is still waiting for its data
        "\tv_mfma_i32_32x32x32_i8 a[0:15], v[4:7], v[10:13], a[0:15]",
        "\ts_endpgm"])
    kernels, found = unconsumed_overwrites(planted, "FcMfmaKernel")
    assert kernels == 1 and len(found) == 1 and found[0][2] == 5
    clean = planted.replace("\tv_add_u32_e32 v5, 1, v9\n", "")
    assert unconsumed_overwrites(clean, "FcMfmaKernel") == (1, [])
