"""The snapshot tracking of the split-bf16 sweep selects with v_cndmask written as inline assembly, on a lane mask that a
vector compare has just written to scalar registers. gfx940 and later need two wait states between a vector instruction that
writes a scalar register and a vector instruction that reads it; the compiler keeps that distance for the instructions it
emits itself but does not look inside inline assembly (csrc/assign_bf16_impl.h: settled_mask). This test compiles the kernels
that contain such selections to assembly (no GPU needed) and measures the distance at every place."""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "cuda-kmeans_amd", "csrc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fhip-fp32-correctly-rounded-divide-sqrt", "-fno-gpu-rdc",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC]


def instructions(path):
    out = []
    for line in open(path):
        text = line.split(";")[0].strip()
        if text and not text.startswith(".") and not text.endswith(":"):
            out.append(text)
    return out


def close_reads(code):
    """(index, text) of vector instructions that read a scalar register pair fewer than two wait states after a vector compare
    wrote it."""
    found = []
    for i, text in enumerate(code):
        m = re.match(r"v_cmp\w*_e64 (s\[\d+:\d+\])", text)
        if not m:
            continue
        reg, waited = m.group(1), 0
        for later in code[i + 1:i + 8]:
            if reg in later and later.startswith("v_"):
                if waited < 2:
                    found.append((i, text + " | " + later))
                break
            if reg in later:          # a scalar instruction took the mask over
                break
            nop = re.match(r"s_nop (\d+)", later)
            waited += int(nop.group(1)) + 1 if nop else 1
    return found


@pytest.mark.parametrize("blocks", [1, 2, 3])
def test_selections_on_a_fresh_mask_keep_two_wait_states(tmp_path, blocks):
    hipcc = "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc")
    asm = tmp_path / ("sweep_kb%d.s" % blocks)
    subprocess.check_call([hipcc] + FLAGS + ["-DKMX_KB=%d" % blocks, "-S", "--cuda-device-only",
                                             os.path.join(CSRC, "assign_bf16_inst.hip"), "-o", str(asm)],
                          stderr=subprocess.DEVNULL)
    code = instructions(str(asm))
    selections = [t for t in code if re.match(r"v_cndmask_b32_e64 v\d+, v\d+, v\d+, s\[", t)]
    assert len(selections) > 100, "the snapshot's selections are expected in this unit"
    bad = close_reads(code)
    assert not bad, "%d reads of a scalar mask within two wait states of its vector write, first: %s" % (len(bad), bad[0][1])
