"""A property of the compiled code that no numerical test pins reliably: in the pipelined gather
kernel the registers written by the hand-issued table loads must not be read by any instruction
before the ``s_waitcnt`` that releases them (a read before it returns whatever the register held,
sometimes the right value).  The check compiles the source to gfx950 assembly and walks it."""

import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "speculators_amd", "csrc")


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc")
def test_hand_issued_loads_are_not_read_before_their_wait(tmp_path):
    out = tmp_path / "fused_loss.s"
    subprocess.run(["hipcc", "-O3", "-std=c++17", "--offload-arch=gfx950", "-Xclang", "-target-feature",
                    "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-S",
                    "--cuda-device-only", "-o", str(out), os.path.join(CSRC, "fused_loss.hip")],
                   check=True, capture_output=True)
    text = out.read_text()
    kernels = re.findall(r"^(_ZN3spx27loss_fwd_gather_pipe_kernel\w+):", text, flags=re.M)
    assert len(kernels) == 2, kernels
    for name in kernels:
        body = text[text.index(name + ":"):]
        body = body[:body.index(".Lfunc_end")].splitlines()
        pending, loads, waits = set(), 0, 0
        for line in body:
            ins = line.strip()
            m = re.match(r"buffer_load_dword (v\d+), v\d+, s\[", ins)
            if m:
                pending.add(m.group(1))
                loads += 1
                continue
            if ins.startswith("s_waitcnt") and "vmcnt" in ins:
                pending.clear()
                waits += 1
                continue
            for reg in pending:
                assert not re.search(rf"\b{reg}\b", ins), f"{name}: {reg} read before its wait: {ins}"
            # a register range that covers a pending register counts as a read too
            for lo, hi in re.findall(r"v\[(\d+):(\d+)\]", ins):
                for reg in pending:
                    assert not int(lo) <= int(reg[1:]) <= int(hi), f"{name}: {reg} inside {ins}"
        # the prologue and the two unrolled tiles issue eight loads each
        assert loads == 24 and waits >= 3, (name, loads, waits)
