"""Hazard distances in the code the compiler actually emitted.

The slot-structured kernels issue their matrix instructions through inline assembly, so the compiler adds
no wait states between such an instruction and a vector-ALU read of its result; the slot order keeps the
distance (static_asserts over the slot constants in fa_bwd.hip and fa_fwd_wide.hip).  Those asserts speak
about the source.  The compiler, however, moves side-effect-free vector work across the scheduling fences,
so this test looks at the built objects: it disassembles the gfx950 code of the two kernels' object files
and checks, for every instruction that reads a vector register (VGPR or AGPR) last written by a matrix
instruction, that enough wait states lie in between.  An 8-pass matrix instruction (32x32x16) needs its 8 passes plus 3 before the
vector ALU may read the result; an instruction counts as one wait state, `s_nop N` as N + 1, and a matrix
instruction in between as 8 (it cannot issue before the pipe has taken the one before it).
"""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BUILD = os.path.join(ROOT, "flagattention_amd", "csrc", "build")
LLVM = "/opt/rocm/llvm/bin"
NEEDED_WAIT_STATES = 11

_RANGE = re.compile(r"\b([va])\[(\d+):(\d+)\]")
_SINGLE = re.compile(r"\b([va])(\d+)\b")


def _vgprs(operand):
    """Vector registers named by an operand, both files: ('v', n) and ('a', n)."""
    regs = set()
    for file, lo, hi in _RANGE.findall(operand):
        regs.update((file, n) for n in range(int(lo), int(hi) + 1))
    for file, r in _SINGLE.findall(_RANGE.sub("", operand)):
        regs.add((file, int(r)))
    return regs


def _disassemble(obj, tmp_path):
    fat, code = str(tmp_path / "fat.bin"), str(tmp_path / "device.co")
    subprocess.run([f"{LLVM}/llvm-objcopy", f"--dump-section=.hip_fatbin={fat}", obj], check=True)
    subprocess.run([f"{LLVM}/clang-offload-bundler", "--unbundle", "--type=o", f"--input={fat}",
                    "--targets=hipv4-amdgcn-amd-amdhsa--gfx950", f"--output={code}"], check=True)
    text = subprocess.run([f"{LLVM}/llvm-objdump", "-d", "--no-show-raw-insn", code], check=True,
                          capture_output=True, text=True).stdout
    kernels, name = {}, None
    for line in text.split("\n"):
        m = re.match(r"^[0-9a-f]+ <(\w+)>:", line)
        if m:
            name = m.group(1)
            kernels[name] = []
        elif name and line.startswith("\t"):
            kernels[name].append(line.split("//")[0].strip())
    return kernels


def closest_read(instructions):
    """(wait states, reading instruction) of the read that follows the matrix instruction whose result it takes
    most closely; the body is walked twice so that reads at the top of a loop meet writes at its bottom."""
    written = {}      # register -> (wait-state clock, matrix-instruction count) at its last write by a matrix instruction
    clock = matrix = 0
    worst = (10 ** 9, None)
    checked = 0
    for _ in range(2):
        for ins in instructions:
            if not ins:
                continue
            op, _, rest = ins.partition(" ")
            operands = rest.split(",")
            if op == "s_nop":
                clock += int(operands[0]) + 1
                continue
            clock += 1
            if op.startswith("v_mfma"):
                matrix += 1
                for r in _vgprs(operands[0]):
                    written[r] = (clock, matrix)
                continue
            if not op.startswith(("v_", "ds_", "global_", "buffer_")):
                continue
            has_destination = (op.startswith("v_") and not op.startswith("v_cmp")) or \
                op.startswith(("ds_read", "global_load", "buffer_load"))
            reads = set()
            for operand in operands[1 if has_destination else 0:]:
                reads |= _vgprs(operand)
            for r in reads & written.keys():
                at, count = written[r]
                states = (clock - at - 1) + 7 * (matrix - count)
                checked += 1
                if states < worst[0]:
                    worst = (states, ins)
            if op.startswith("v_") and has_destination:
                for r in _vgprs(operands[0]):
                    written.pop(r, None)
    return worst, checked


def test_the_audit_sees_a_read_that_comes_too_early():
    early = ["v_mfma_f32_32x32x16_bf16 v[192:207], v[2:5], a[0:3], v[192:207]", "s_nop 1", "v_max_f32 v2, v192, v193"]
    (states, ins), checked = closest_read(early)
    assert checked and states == 2 and ins.startswith("v_max_f32")
    spaced = [early[0], "v_mfma_f32_32x32x16_bf16 a[0:15], v[2:5], v[6:9], a[0:15]",
              "v_mfma_f32_32x32x16_bf16 a[16:31], v[2:5], v[6:9], a[16:31]", early[2]]
    assert closest_read(spaced)[0][0] == 16
    own_accumulator = [early[0], early[0]]        # a chain reads its own accumulator back to back: not a vector-ALU read
    assert closest_read(own_accumulator)[1] == 0


@pytest.mark.parametrize("obj", ["fa_fwd_wide.o", "fa_bwd.o", "fa_fwd.o", "fa_splitkv.o", "fa_total.o"])
def test_vector_reads_of_matrix_results_keep_their_distance(obj, tmp_path):
    path = os.path.join(BUILD, obj)
    if not os.path.exists(path) or not all(shutil.which(os.path.join(LLVM, t)) for t in
                                           ("llvm-objcopy", "clang-offload-bundler", "llvm-objdump")):
        pytest.skip("needs the objects of a library build and the LLVM binary tools")
    kernels = _disassemble(path, tmp_path)
    audited = reads = 0
    for name, instructions in kernels.items():
        if not any(ins.startswith("v_mfma") for ins in instructions):
            continue
        (states, ins), checked = closest_read(instructions)
        audited += 1
        reads += checked
        assert states >= NEEDED_WAIT_STATES, f"{name}: `{ins}` reads a matrix result after {states} wait states"
    assert audited >= 2 and reads >= 100, f"{obj}: {audited} kernels with matrix instructions, {reads} reads checked"
