"""A compile-time check of the block kernel's hand-issued loads (no GPU needed).

attn_prefill_f16_kernel requests Q (and a block's new K/V rows) with `global_load_dwordx4` from
inline assembly and waits for them by count, because the compiler cannot count the loads the LDS
ring has in flight. The compiler therefore believes those registers hold their values from the
moment the load is issued: if it copied or read one of them before the `s_waitcnt` that names
them, or put a branch in between (where it may insert such copies), the kernel would compute on
whatever the registers held before. This test compiles the kernel for gfx950 and checks every
instantiation's assembly for exactly that."""
import os
import re
import subprocess
import tempfile
from concurrent.futures import ThreadPoolExecutor

import pytest

from helpers import ROOT

CSRC = os.path.join(ROOT, "itak-torch-rebuild_amd", "csrc")
# The files that instantiate the kernel (attn_prefill_f16_kernel.h), and how many instantiations
# each must at least show.
SOURCES = {"attn_prefill_f16.hip": 48, "attn_prefill_f16_dims.hip": 72}
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def registers(text):
    regs = set()
    for m in re.finditer(r"\bv\[(\d+):(\d+)\]", text):
        regs |= set(range(int(m.group(1)), int(m.group(2)) + 1))
    for m in re.finditer(r"\bv(\d+)\b", text):
        regs.add(int(m.group(1)))
    return regs


def assembly(src):
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "kernel.s")
        subprocess.run([HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature",
                        "-Xclang", "-packed-fp32-ops", "--cuda-device-only", "-S", os.path.join(CSRC, src),
                        "-o", out], check=True, capture_output=True)
        return open(out).read().split("\n")


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc is not installed")
def test_registers_of_hand_issued_loads_are_untouched_until_their_wait():
    with ThreadPoolExecutor(max_workers=len(SOURCES)) as pool:
        listings = dict(zip(SOURCES, pool.map(assembly, SOURCES)))
    for src, lines in listings.items():
        check(src, lines, SOURCES[src])


def check(src, lines, at_least):
    kernels = runs = 0
    in_kernel = False
    pending = set()      # registers with a hand-issued load in flight
    for n, raw in enumerate(lines, 1):
        line = raw.split(";")[0].strip()
        if re.match(r"^_ZN4itak.*attn_prefill_f16_kernel.*:$", line):
            in_kernel, pending = True, set()
            kernels += 1
            continue
        if not in_kernel or not line:
            continue
        if line.startswith("s_endpgm"):
            assert not pending, f"{src} line {n}: kernel ends with loads unwaited"
            in_kernel = False
            continue
        m = re.match(r"global_load_dwordx4 (v\[\d+:\d+\]), (v\[\d+:\d+\]), off", line)
        if m:  # the LDS ring's loads are global_load_lds_dwordx4 and write no register
            assert not (registers(m.group(2)) & pending), f"{src} line {n}: address in a register still in flight"
            pending |= registers(m.group(1))
            continue
        if not pending:
            continue
        if line.startswith("s_waitcnt") and "vmcnt" in line:
            pending = set()
            runs += 1
            continue
        assert not re.match(r"^(\.LBB|s_cbranch|s_branch)", line), \
            f"{src} line {n}: control flow between a hand-issued load and its wait: {line}"
        operands = line.split(None, 1)[1] if " " in line else ""
        assert not (registers(operands) & pending), \
            f"{src} line {n}: a register with a load in flight is used before the wait: {line}"
    assert kernels >= at_least and runs >= kernels, (src, kernels, runs)
