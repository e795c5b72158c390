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


def touched_in_flight(asm_text, kernel_pattern, load_ops):
    """The stricter form for loads that are waited for with a hand-placed `s_waitcnt vmcnt(0)`: from an
    inline-assembly load in `load_ops` until such a wait NOTHING may touch its destination registers, not even
    read them (a register copy would copy stale contents). Forward data flow over the kernel's basic blocks
    (the set of registers that may be in flight, united where paths meet, iterated to its fixed point).
    Returns (kernels, loads, [(kernel, instruction, register)])."""
    lines = asm_text.split("\n")
    starts = [i for i, l in enumerate(lines) if re.match(r"^_ZN3tvx\S*" + kernel_pattern + r"\S*: ", l)]
    found, loads = [], 0
    for s in starts:
        e = s
        while not lines[e].startswith(".Lfunc_end"):  # (a kernel may hold several s_endpgm)
            e += 1
        # instructions: (op, operand tokens, is_asm); labels map to instruction indices
        insts, labels, in_asm = [], {}, False
        for raw in lines[s + 1:e]:
            l = raw.strip()
            m = re.match(r"^(\.LBB\S+):", l)
            if m:
                labels[m.group(1)] = len(insts)
                continue
            if l.startswith(";;#ASMSTART"):
                in_asm = True
                continue
            if l.startswith(";;#ASMEND"):
                in_asm = False
                continue
            if not l or l[0] in ";.":
                continue
            parts = l.split(";")[0].replace(",", " ").split()
            insts.append((parts[0], parts[1:], in_asm, l))
        succ = []
        for i, (op, args, _, _) in enumerate(insts):
            if op == "s_endpgm":
                succ.append([])
            elif op == "s_branch":
                succ.append([labels[args[0]]])
            elif op.startswith("s_cbranch"):
                succ.append([labels[args[0]], i + 1])
            else:
                succ.append([i + 1] if i + 1 < len(insts) else [])
        state_in = [None] * len(insts)
        state_in[0] = frozenset()
        work, flagged = [0], set()
        while work:
            i = work.pop()
            op, args, is_asm, text = insts[i]
            cur = set(state_in[i])
            if is_asm and op in load_ops:
                for r in _regs(args[0]) & cur:  # a second load into a register whose first has not been waited for
                    flagged.add((lines[s].split(":")[0][-48:], text, r))
                cur |= _regs(args[0])
            elif op == "s_waitcnt" and "vmcnt(0)" in text:
                cur = set()
            else:
                for tok in args:
                    for r in _regs(tok) & cur:
                        flagged.add((lines[s].split(":")[0][-48:], text, r))
            out = frozenset(cur)
            for j in succ[i]:
                merged = out if state_in[j] is None else state_in[j] | out
                if merged != state_in[j]:
                    state_in[j] = merged
                    work.append(j)
        loads += sum(1 for op, _, is_asm, _ in insts if is_asm and op in load_ops)
        found.extend(sorted(flagged))
    return len(starts), loads, found


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_conv_band_async_loads_keep_their_registers(tmp_path):
    """The band convolution's loader: 8-byte loads issued one band ahead from inline assembly, waited for by a
    hand-placed s_waitcnt vmcnt(0)."""
    out = str(tmp_path / "band.s")
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "-I", os.path.join(REPO, "include"), "-I", CSRC, "-S", "--cuda-device-only",
           os.path.join(CSRC, "conv_band_i8.hip"), "-o", out]
    subprocess.run(cmd, check=True, capture_output=True, timeout=600)
    kernels, loads, found = touched_in_flight(open(out).read(), "ConvBandKernel", ("global_load_dwordx2",))
    assert kernels >= 8 and loads >= 8 * kernels  # every template instance, each with its loads
    assert not found, found[:5]


def test_strict_checker_sees_planted_hazards():
    def kernel(*body):
        return "\n".join(("_ZN3tvx1_ConvBandKernelIXEEv: ; @k",) + body + ("\ts_endpgm", ".Lfunc_end0:"))
    load = ("\t;;#ASMSTART", "\tglobal_load_dwordx2 v[4:5], v2, s[0:1]", "\t;;#ASMEND")
    wait = ("\t;;#ASMSTART", "\ts_waitcnt vmcnt(0)", "\t;;#ASMEND")
    ops = ("global_load_dwordx2",)
    # a read in front of the wait
    k, n, found = touched_in_flight(kernel(*load, "\tv_mov_b32_e32 v8, v5", *wait, "\tv_mov_b32_e32 v9, v4"), "ConvBandKernel", ops)
    assert (k, n) == (1, 1) and [f[2] for f in found] == [5]
    # clean: uses only behind the wait
    assert touched_in_flight(kernel(*load, *wait, "\tv_mov_b32_e32 v9, v4"), "ConvBandKernel", ops)[2] == []
    # a loop whose body loads at its end and waits at its head: the use behind the wait is fine, one in front is not
    loop = ("\ts_branch .LBB0_2", ".LBB0_1:", *wait, "\tv_add_u32_e32 v9, v4, v5", ".LBB0_2:", *load,
            "\ts_cbranch_scc1 .LBB0_1")
    assert touched_in_flight(kernel(*loop), "ConvBandKernel", ops)[2] == []
    bad = ("\ts_branch .LBB0_2", ".LBB0_1:", "\tv_add_u32_e32 v9, v4, v5", *wait, ".LBB0_2:", *load,
           "\ts_cbranch_scc1 .LBB0_1")
    assert sorted(f[2] for f in touched_in_flight(kernel(*bad), "ConvBandKernel", ops)[2]) == [4, 5]


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
