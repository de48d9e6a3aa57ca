"""The snapshot tracking of the split-bf16 sweep copies under a narrowed execution mask, in statements written as inline
assembly (csrc/assign_bf16_impl.h: take_lead_where, copy_second_half_where), on a lane mask that a vector compare has just
written to scalar registers. The compiler does not look inside inline assembly: it neither keeps the distance that gfx940 and
later want between a vector instruction that writes a scalar register and a reader of that register (settled_mask writes the
wait out), nor does it know that the statement narrows the mask. This test compiles the kernels that contain such statements to assembly
(no GPU needed), finds them (narrowing, moves only, the saved mask back) and measures the distance at every one."""
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


def masked_statements(code):
    """(index, mask register, number of moves) of the statements that copy under a narrowed execution mask: s_and_saveexec, moves
    only, and the saved mask back."""
    for i, text in enumerate(code):
        m = re.match(r"s_and_saveexec_b64 (s\[\d+:\d+\]), (s\[\d+:\d+\])$", text)
        if not m:
            continue
        j = i + 1
        while j < len(code) and re.match(r"v_mov_b(32|64)(_e32)? ", code[j]):
            j += 1
        if j > i + 1 and j < len(code) and code[j] == "s_mov_b64 exec, " + m.group(1):
            yield i, m.group(2), j - i - 1


def wait_states_since_compare(code, i, reg):
    """wait states between the vector compare that wrote `reg` and instruction i (None: no compare within reach, the mask came
    from scalar instructions)"""
    waited = 0
    for earlier in reversed(code[max(0, i - 16):i]):
        if re.match(r"v_cmp\w*_e64 " + re.escape(reg), earlier):
            return waited
        nop = re.match(r"s_nop (\d+)", earlier)
        waited += int(nop.group(1)) + 1 if nop else 1
    return None


@pytest.mark.parametrize("blocks", [1, 2, 3])
def test_masked_copies_read_a_settled_mask(tmp_path, blocks):
    hipcc = "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc")
    asm = tmp_path / ("sweep_kb%d.s" % blocks)
    subprocess.check_call([hipcc] + FLAGS + ["-DKMX_KB=%d" % blocks, "-S", "--cuda-device-only",
                                             os.path.join(CSRC, "assign_bf16_inst.hip"), "-o", str(asm)],
                          stderr=subprocess.DEVNULL)
    code = instructions(str(asm))
    statements = list(masked_statements(code))
    assert len(statements) > 50, "the snapshot's masked copies are expected in this unit"
    assert {moves for _, _, moves in statements} == {4, 6}, "leader + four pairs, or four pairs"
    waits = [(i, wait_states_since_compare(code, i, reg)) for i, reg, _ in statements]
    assert any(w is not None for _, w in waits), "masks written by vector compares are expected"
    close = [(i, code[i]) for i, w in waits if w is not None and w < 2]
    assert not close, "%d masked statements within two wait states of the compare that wrote their mask, first: %s" % (len(close), close[0][1])
