"""Hazard distances in the code the compiler actually emitted.

The slot-structured kernels issue their matrix instructions through inline assembly, so the compiler adds
no wait states between such an instruction and a vector-ALU read of its result; the slot order keeps the
distance (static_asserts over the slot constants in fa_bwd.hip and fa_fwd_wide.hip).  Those asserts speak
about the source.  The compiler, however, moves side-effect-free vector work across the scheduling fences,
so this test looks at the built objects: it disassembles the gfx950 code of the kernels' object files
and checks, for every instruction that reads or overwrites a vector register (VGPR or AGPR) last written by
a matrix instruction, that enough wait states lie in between on every path of the control-flow graph: on
gfx950 the instruction's passes plus 4 (12 behind a 32x32x16 product, 8 behind a 16x16x32 one).  The objects
whose matrix instructions are builtins, which the compiler pads itself, are audited too; they calibrate the
rule.
"""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BUILD = os.path.join(ROOT, "flagattention_amd", "csrc", "build")
LLVM = "/opt/rocm/llvm/bin"

_RANGE = re.compile(r"\b([va])\[(\d+):(\d+)\]")
_SINGLE = re.compile(r"\b([va])(\d+)\b")
_LABEL = re.compile(r"^[0-9a-f]+ <(L\d+)>:")
_SYMBOL = re.compile(r"^[0-9a-f]+ <(\w+)>:")
_ENDS_PATH = ("s_branch", "s_endpgm", "s_setpc_b64")
HORIZON = 24          # wait states after which no matrix result is pending any more


def _vgprs(operand):
    """Vector registers named by an operand, both files: ('v', n) and ('a', n)."""
    regs = set()
    for file, lo, hi in _RANGE.findall(operand):
        regs.update((file, n) for n in range(int(lo), int(hi) + 1))
    for file, r in _SINGLE.findall(_RANGE.sub("", operand)):
        regs.add((file, int(r)))
    return regs


def _disassemble(obj, tmp_path):
    """{kernel: [line, ...]} where a line is an instruction or a branch target `L<n>:`."""
    fat, code = str(tmp_path / "fat.bin"), str(tmp_path / "device.co")
    subprocess.run([f"{LLVM}/llvm-objcopy", f"--dump-section=.hip_fatbin={fat}", obj], check=True)
    subprocess.run([f"{LLVM}/clang-offload-bundler", "--unbundle", "--type=o", f"--input={fat}",
                    "--targets=hipv4-amdgcn-amd-amdhsa--gfx950", f"--output={code}"], check=True)
    text = subprocess.run([f"{LLVM}/llvm-objdump", "-d", "--no-show-raw-insn", "--symbolize-operands", code],
                          check=True, capture_output=True, text=True).stdout
    kernels, name = {}, None
    for line in text.split("\n"):
        label, symbol = _LABEL.match(line), _SYMBOL.match(line)
        if label and name:
            kernels[name].append(label.group(1) + ":")
        elif symbol:
            name = symbol.group(1)
            kernels[name] = []
        elif name and line.startswith("\t"):
            kernels[name].append(line.split("//")[0].strip())
    return kernels


def _passes(op):
    """Passes of 4 cycles a matrix instruction occupies the pipe for: 16 Kflop per pass on gfx950 at 16 bits."""
    m = re.match(r"v_mfma_f32_(\d+)x(\d+)x(\d+)_", op)
    rows, cols, depth = (int(g) for g in m.groups())
    return rows * cols * depth // 2048


def needed_wait_states(passes):
    """gfx950: the passes plus 4.  hipcc pads a matrix instruction it can see to exactly this distance (`s_nop 11`
    between a 32x32x16 product and a read of its result, 8 wait states behind a 16x16x32 one); the last test
    below holds the number against that padding."""
    return passes + 4


def _blocks(lines):
    """Basic blocks [(instructions, successor indices)] of one kernel."""
    starts, body = {}, []
    for line in lines:
        if not line:
            continue
        if line.endswith(":"):
            starts[line[:-1]] = len(body)
        else:
            body.append(line)
    leaders = {0} | set(starts.values())
    for i, ins in enumerate(body):
        if ins.startswith(("s_branch", "s_cbranch", "s_endpgm", "s_setpc_b64")):
            leaders.add(i + 1)
    order = sorted(l for l in leaders if l < len(body))
    index = {l: n for n, l in enumerate(order)}
    blocks = []
    for n, lead in enumerate(order):
        end = order[n + 1] if n + 1 < len(order) else len(body)
        last = body[end - 1]
        succ = []
        if last.startswith(("s_branch", "s_cbranch")):
            target = last.split()[-1]
            if target in starts and starts[target] in index:
                succ.append(index[starts[target]])
        if not last.startswith(_ENDS_PATH) and end in index:
            succ.append(index[end])
        blocks.append((body[lead:end], succ))
    return blocks


def _walk(instructions, pending, pipe_free, report):
    """One basic block.  `pending` maps a register to (issue time, passes) of the matrix instruction that wrote it
    last, times relative to the block's entry at 0; returns the same relative to its exit.  Time is counted in
    wait states: an instruction issues one after the one before it, `s_nop N` takes N + 1, and a matrix
    instruction issues no earlier than the pipe has worked off the passes of the one before it.  Other stalls
    only add to the real distance."""
    pending = dict(pending)
    now = 0
    for ins in instructions:
        op, _, rest = ins.partition(" ")
        operands = rest.split(",")
        if op == "s_nop":
            now += int(operands[0]) + 1
            continue
        if op.startswith("v_mfma"):
            now = max(now, pipe_free)
            passes = _passes(op)
            pipe_free = now + passes
            for r in _vgprs(operands[0]):     # reading its own accumulator back to back is what the pipe is built for
                pending[r] = (now, passes)
        elif op.startswith(("v_", "ds_", "global_", "buffer_")):
            has_destination = (op.startswith("v_") and not op.startswith("v_cmp")) or \
                op.startswith(("ds_read", "global_load", "buffer_load"))
            written = _vgprs(operands[0]) if has_destination else set()
            read = set()
            for operand in operands[1 if has_destination else 0:]:
                read |= _vgprs(operand)
            for kind, regs in (("read", read), ("overwrite", written - read)):
                for r in regs & pending.keys():
                    at, passes = pending[r]
                    report(kind, now - at - 1 - needed_wait_states(passes), now - at - 1, ins)
            for r in written:
                pending.pop(r, None)
        now += 1
    return {r: (at - now, p) for r, (at, p) in pending.items() if now - at <= HORIZON}, max(pipe_free - now, 0)


def closest_access(lines):
    """{"read" | "overwrite": (slack, wait states, instruction)} and the number of accesses checked: the vector or
    memory instruction that follows most closely, on any path, the matrix instruction whose result it reads, or
    overwrites without reading; slack = wait states in between minus those needed (an overwrite needs what a read
    needs)."""
    blocks = _blocks(lines)
    worst = {"read": (10 ** 9, None, None), "overwrite": (10 ** 9, None, None)}
    checked = [0]

    def report(kind, slack, states, ins):
        checked[0] += 1
        if slack < worst[kind][0]:
            worst[kind] = (slack, states, ins)

    entry = [None] * len(blocks)              # state at block entry: the most recent write of each register over all paths
    if blocks:
        entry[0] = ({}, 0)
    work = [0] if blocks else []
    while work:
        n = work.pop()
        instructions, succ = blocks[n]
        out, pipe = _walk(instructions, *entry[n], report)
        for s in succ:
            if entry[s] is None:
                entry[s] = (dict(out), pipe)
                work.append(s)
                continue
            known, known_pipe = entry[s]
            changed = pipe > known_pipe
            for r, (at, p) in out.items():
                if r not in known or at > known[r][0]:
                    known[r] = (at, p)
                    changed = True
            entry[s] = (known, max(pipe, known_pipe))
            if changed:
                work.append(s)
    return worst, checked[0]


def dma_in_flight_at(lines, stops=("s_barrier", "s_endpgm")):
    """The `stops` instructions that some path reaches while a global-to-LDS transfer may still be in flight.
    Such a transfer is counted like any vector-memory load but writes LDS, which the compiler does not know:
    the kernel itself waits for vmcnt(0) before the barrier behind which other wavefronts read the tile, and
    before it ends (the transfer must not outlive the workgroup's LDS allocation)."""
    blocks = _blocks(lines)
    found = []
    entry = [None] * len(blocks)
    if blocks:
        entry[0] = False
    work = [0] if blocks else []
    while work:
        n = work.pop()
        instructions, succ = blocks[n]
        flying = entry[n]
        for ins in instructions:
            op = ins.split(" ")[0]
            if op.startswith("global_load_lds"):
                flying = True
            elif op == "s_waitcnt" and "vmcnt(0)" in ins:
                flying = False
            elif op in stops and flying and ins not in found:
                found.append(ins)
        for s in succ:
            if entry[s] is None or (flying and not entry[s]):
                entry[s] = flying
                work.append(s)
    return found


def test_the_transfer_audit_sees_a_missing_wait():
    load = "global_load_lds_dwordx4 v1, s[2:3]"
    assert dma_in_flight_at([load, "s_waitcnt vmcnt(0)", "s_barrier", "s_endpgm"]) == []
    assert dma_in_flight_at([load, "s_waitcnt lgkmcnt(0)", "s_barrier", "s_waitcnt vmcnt(0)", "s_endpgm"]) == ["s_barrier"]
    assert dma_in_flight_at([load, "s_waitcnt vmcnt(1)", "s_endpgm"]) == ["s_endpgm"]
    loop = ["L0:", "s_barrier", load, "s_cbranch_scc1 L0", "s_waitcnt vmcnt(0)", "s_endpgm"]      # over the back edge
    assert dma_in_flight_at(loop) == ["s_barrier"]


def test_transfers_into_lds_have_landed_at_every_barrier_and_at_the_end(tmp_path):
    path = os.path.join(BUILD, "fa_fwd_wide.o")
    if not os.path.exists(path) or not all(shutil.which(os.path.join(LLVM, t)) for t in
                                           ("llvm-objcopy", "clang-offload-bundler", "llvm-objdump")):
        pytest.skip("needs the objects of a library build and the LLVM binary tools")
    audited = 0
    for name, lines in _disassemble(path, tmp_path).items():
        if any(line.startswith("global_load_lds") for line in lines):
            audited += 1
            assert dma_in_flight_at(lines) == [], name
    assert audited == 2       # the f16 and the bf16 kernel


PRODUCT = "v_mfma_f32_32x32x16_bf16 v[192:207], v[2:5], a[0:3], v[192:207]"
OTHER = "v_mfma_f32_32x32x16_bf16 a[0:15], v[2:5], v[6:9], a[0:15]"
READ = "v_max_f32 v2, v192, v193"


def closest_read(lines):
    return closest_access(lines)[0]["read"]


def test_the_audit_sees_a_read_that_comes_too_early():
    slack, states, ins = closest_read([PRODUCT, "s_nop 1", READ])
    assert states == 2 and slack == 2 - 12 and ins == READ
    assert closest_read([PRODUCT, "s_nop 11", READ])[:2] == (0, 12)
    assert closest_read([PRODUCT, OTHER, OTHER.replace("a[0:15]", "a[16:31]"), READ])[1] == 16
    short = ["v_mfma_f32_16x16x32_f16 v[172:175], v[200:203], v[14:17], v[176:179]", "s_nop 7", "v_mov_b32 v1, v172"]
    assert closest_read(short)[:2] == (0, 8)
    assert closest_access([PRODUCT, PRODUCT])[1] == 0        # a chain's own accumulator is no vector-ALU read
    overwrite = closest_access([PRODUCT, "s_nop 3", "v_mov_b32 v192, 0"])[0]
    assert overwrite["overwrite"][:2] == (4 - 12, 4) and overwrite["read"][2] is None


def test_the_audit_follows_the_branches():
    # the product at the bottom of a loop meets the read at its top over the back edge only
    loop = ["v_mov_b32 v1, 0", "L0:", READ, "s_nop 15", PRODUCT, "s_cbranch_scc1 L0", "s_nop 15", "s_endpgm"]
    assert closest_read(loop)[:2] == (1 - 12, 1)
    # code behind an unconditional branch is not reached from it
    apart = [PRODUCT, "s_branch L1", "L2:", READ, "s_endpgm", "L1:", "s_nop 15", "s_branch L2"]
    assert closest_read(apart)[1] == 18
    # of two ways into a block the shorter one counts
    merge = ["s_cbranch_scc1 L3", PRODUCT, "s_nop 1", "s_branch L4", "L3:", PRODUCT, "s_nop 13", "L4:", READ, "s_endpgm"]
    assert closest_read(merge)[1] == 3


def _audit(obj, tmp_path):
    path = os.path.join(BUILD, obj)
    if not os.path.exists(path) or not all(shutil.which(os.path.join(LLVM, t)) for t in
                                           ("llvm-objcopy", "clang-offload-bundler", "llvm-objdump")):
        pytest.skip("needs the objects of a library build and the LLVM binary tools")
    results = {}
    for name, lines in _disassemble(path, tmp_path).items():
        if any(line.startswith("v_mfma") for line in lines):
            results[name] = closest_access(lines)
    return results


# kernels whose matrix instructions the compiler does not see (hw::mfma32_vacc, pinned accumulators)
HAND_SLOTTED = ("fa_fwd_wide_kernel", "fa_bwd_dkdv_kernel")


@pytest.mark.parametrize("obj", ["fa_fwd_wide.o", "fa_bwd.o", "fa_fwd.o", "fa_splitkv.o", "fa_total.o", "paged.o"])
def test_vector_accesses_to_matrix_results_keep_their_distance(obj, tmp_path):
    """Reads everywhere; overwrites in the hand-slotted kernels.  (In compiler-scheduled code a few overwrites that
    are reached only over a taken skip branch count fewer wait states than the compiler pads to elsewhere; that
    is the compiler's bookkeeping over paths, and a taken branch costs more cycles than the count is short of.)"""
    results = _audit(obj, tmp_path)
    for name, (worst, _) in results.items():
        kinds = ("read", "overwrite") if any(h in name for h in HAND_SLOTTED) else ("read",)
        for kind in kinds:
            slack, states, ins = worst[kind]
            assert slack >= 0, f"{name}: `{ins}` ({kind}) follows the matrix instruction after {states} wait states, {-slack} too few"
    accesses = sum(checked for _, checked in results.values())
    assert len(results) >= 2 and accesses >= 100, f"{obj}: {len(results)} kernels with matrix instructions, {accesses} accesses checked"


@pytest.mark.parametrize("obj", ["fa_total.o", "fa_splitkv.o"])
def test_the_needed_distance_is_the_one_the_compiler_pads_to(obj, tmp_path):
    """These kernels issue their matrix instructions through builtins, so hipcc places the wait states itself;
    where it had nothing else to put in between, the distance it left is the requirement."""
    results = _audit(obj, tmp_path)
    assert min(worst["read"][0] for worst, _ in results.values()) == 0


def _wait_states(ins):
    return int(ins.split()[1]) + 1 if ins.startswith("s_nop") else 1


def slotted_vector_hazards(lines):
    """What the hand-placed vector instructions of the 256-row forward have to keep by themselves, because they are
    inline assembly: (a) the output tuples a[0:127] are written by matrix instructions, by the clearing writes of 0
    and by the read-scale-write triple only -- never by a copy of the compiler's; (b) the result of an exponential
    is not read by the very next instruction; (c) two wait states separate a lane exchange from the instructions
    that write or read its registers.  Returns a list of complaints; checks run inside basic blocks."""
    body = [l for l in lines if l and not l.endswith(":")]
    bad = []
    for i, ins in enumerate(body):
        op, _, rest = ins.partition(" ")
        operands = [o.strip() for o in rest.split(",")]
        if op == "v_accvgpr_write_b32":
            dst = next(iter(_vgprs(operands[0])))
            if dst[0] == "a" and dst[1] < 128 and operands[1] != "0":
                triple = body[i - 3] if i >= 3 else ""
                if triple != f"v_accvgpr_read_b32 {operands[1]}, {operands[0]}":
                    bad.append(f"(a) {ins}: a write to the output tuples that is not the scaling triple")
        elif op.startswith("v_exp_f32") and i + 1 < len(body):
            nxt = body[i + 1]
            if not nxt.startswith(("s_", "v_mfma")) and _vgprs(operands[0]) & _vgprs(nxt.partition(" ")[2].partition(",")[2]):
                bad.append(f"(b) {nxt} reads the exponential of the instruction before it")
        elif op == "v_permlane32_swap_b32":
            regs = _vgprs(rest)
            for step, seq in ((-1, body[:i][::-1]), (1, body[i + 1:])):
                states = 0
                for other in seq:
                    if states >= 2 or other.startswith(("s_branch", "s_cbranch", "s_endpgm")):
                        break
                    if not other.startswith("s_") and _vgprs(other.partition(" ")[2]) & regs:
                        bad.append(f"(c) {other} is {states} wait states {'before' if step < 0 else 'behind'} {ins}")
                    states += _wait_states(other)
    return bad


def test_the_slotted_vector_audit_sees_each_kind_of_mistake():
    ok = ["v_accvgpr_write_b32 a5, 0", "v_accvgpr_read_b32 v9, a17", "v_mul_f32_e32 v9, v9, v3", "s_nop 0",
          "v_accvgpr_write_b32 a17, v9", "v_accvgpr_write_b32 a130, v4", "v_exp_f32_e32 v7, v8", "v_add_f32_e32 v1, v1, v2",
          "v_add_f32_e32 v1, v1, v7", "v_mov_b32_e32 v20, v1", "s_nop 1", "v_permlane32_swap_b32_e32 v20, v21", "s_nop 0",
          "v_mfma_f32_32x32x16_bf16 a[0:15], v[2:5], v[6:9], a[0:15]", "v_max_f32_e32 v20, v20, v21"]
    ok = [l.replace("v_permlane32_swap_b32_e32", "v_permlane32_swap_b32") for l in ok]
    assert slotted_vector_hazards(ok) == []
    assert len(slotted_vector_hazards(["v_accvgpr_write_b32 a16, v169"])) == 1
    assert len(slotted_vector_hazards(["v_exp_f32_e32 v7, v8", "v_add_f32_e32 v1, v1, v7"])) == 1
    assert len(slotted_vector_hazards(["v_mov_b32_e32 v20, v1", "s_nop 0", "v_permlane32_swap_b32 v20, v21"])) == 1
    assert len(slotted_vector_hazards(["v_permlane32_swap_b32 v20, v21", "v_mfma_f32_32x32x16_bf16 a[0:15], v[2:5], v[6:9], a[0:15]",
                                       "v_max_f32_e32 v20, v20, v21"])) == 1


def test_hand_placed_vector_instructions_of_the_256_row_forward_keep_their_distances(tmp_path):
    path = os.path.join(BUILD, "fa_fwd_wide.o")
    if not os.path.exists(path) or not all(shutil.which(os.path.join(LLVM, t)) for t in
                                           ("llvm-objcopy", "clang-offload-bundler", "llvm-objdump")):
        pytest.skip("needs the objects of a library build and the LLVM binary tools")
    audited = 0
    for name, lines in _disassemble(path, tmp_path).items():
        if "fa_fwd_wide_kernel" in name:
            audited += 1
            lines = [re.sub(r"\bv_permlane32_swap_b32_e32\b", "v_permlane32_swap_b32", l) for l in lines]
            assert slotted_vector_hazards(lines) == [], name
            assert sum(l.startswith("v_permlane32_swap") for l in lines) >= 8
            assert sum(l.startswith("v_accvgpr_write_b32") for l in lines) >= 256
    assert audited == 2


def test_no_instruction_of_the_slotted_backward_reads_an_exponential_right_behind_it(tmp_path):
    """The slot-structured dK/dV body issues its exponentials as assembly statements, so the compiler adds no wait
    state between one and a reader of its result; the step order keeps them a slot apart."""
    path = os.path.join(BUILD, "fa_bwd.o")
    if not os.path.exists(path) or not all(shutil.which(os.path.join(LLVM, t)) for t in
                                           ("llvm-objcopy", "clang-offload-bundler", "llvm-objdump")):
        pytest.skip("needs the objects of a library build and the LLVM binary tools")
    audited = 0
    for name, lines in _disassemble(path, tmp_path).items():
        if "fa_bwd_dkdv_kernel" in name and ("Li128E" in name or "Li64E" in name):   # the head sizes with the slotted body
            audited += 1
            assert [c for c in slotted_vector_hazards(lines) if c.startswith("(b)")] == [], name
            assert sum(l.startswith("v_exp_f32") for l in lines) >= 32
    assert audited >= 16


@pytest.mark.parametrize("obj,kernel", [("fa_fwd_wide.o", "fa_fwd_wide_kernel"), ("fa_bwd.o", "fa_bwd_dkdv_kernel")])
def test_hand_slotted_kernels_spill_nothing(obj, kernel, tmp_path):
    """A spill is a memory instruction of the compiler's that reads a register wherever the allocator ran out: behind
    a matrix instruction written as assembly it would read the result without the wait states (the compiler does
    not know what the statement wrote), and in a slot it would cost what the slot was meant to hide.  The slotted
    kernels are built so that nothing spills; a change that makes the allocator spill must show up here."""
    path = os.path.join(BUILD, obj)
    if not os.path.exists(path) or not all(shutil.which(os.path.join(LLVM, t)) for t in
                                           ("llvm-objcopy", "clang-offload-bundler", "llvm-objdump")):
        pytest.skip("needs the objects of a library build and the LLVM binary tools")
    audited = 0
    for name, lines in _disassemble(path, tmp_path).items():
        if kernel in name:
            audited += 1
            spills = [l for l in lines if l.startswith(("scratch_", "buffer_store", "buffer_load"))]
            assert spills == [], f"{name}: {len(spills)} scratch accesses, e.g. {spills[0]}"
    assert audited >= 2
