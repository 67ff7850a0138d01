"""Static rules on the generated gfx950 code of the decode kernels (hipcc cross-compiles without a GPU).

The compiler inserts the wait states that matrix instructions in flight require around the instructions it
emits itself; an inline-assembly statement is opaque to it.  The kernels therefore keep their few assembly
vector instructions (the 24-bit multiplies of the input stages) away from matrix instructions, and never chain
16-deep and 32-deep fp16 matrix instructions on one accumulator.  These tests read the assembly and check both."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "rtxntc-library_amd", "csrc")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "--cuda-device-only", "-S", "-I" + os.path.join(ROOT, "include")]


def basic_blocks(path):
    """[(function, label, [(mnemonic, operands)])] of an AMDGPU assembly file."""
    blocks, function = [], None
    for line in open(path):
        if re.match(r"^_Z\w+:", line):
            function = line.split(":")[0]
            blocks.append((function, "entry", []))
        elif re.match(r"^\.LBB\d+_\d+:", line):
            blocks.append((function, line.split(":")[0], []))
        elif blocks and line.startswith("\t") and not line.strip().startswith((".", ";")):
            parts = line.strip().split(None, 1)
            blocks[-1][2].append((parts[0], parts[1] if len(parts) > 1 else ""))
    return blocks


@pytest.fixture(scope="module", params=["ntc_decode_kernel", "ntc_decode_fp8_kernel"])
def assembly(request, tmp_path_factory):
    if not shutil.which(HIPCC):
        pytest.skip("hipcc not found")
    out = tmp_path_factory.mktemp("isa") / (request.param + ".s")
    subprocess.run([HIPCC, *FLAGS, "-o", str(out), os.path.join(CSRC, request.param + ".hip")], check=True,
                   stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL, timeout=600)
    return basic_blocks(str(out))


def test_assembly_multiplies_stay_out_of_blocks_with_matrix_instructions(assembly):
    # instructions written in inline assembly print as written, without the _e32/_e64 suffix of generated ones
    for function, label, instructions in assembly:
        names = [m for m, _ in instructions]
        if any(n.startswith("v_mfma") for n in names):
            assert "v_mul_u32_u24" not in names and "v_mad_u32_u24" not in names, (function, label)
    assert any(n.startswith("v_mfma") for _, _, ins in assembly for n, _ in ins)


def test_no_accumulator_chain_mixes_16_deep_and_32_deep_matrix_instructions(assembly):
    """A matrix instruction whose accumulator input is the result of an earlier one must have the same depth
    (16x16x16 onto 16x16x16, 16x16x32 onto 16x16x32).  For every vector register the set of instructions that may have
    written it last is followed through each function's control flow: a label starts from the union of what falls
    into it and of what every branch to it carries (iterated until nothing changes, so loops are covered).  An
    accumulator input that may reach its instruction unwritten - its producer would be unknown - fails the test too."""
    def registers(operand):
        operand = operand.strip()
        m = re.match(r"v\[(\d+):(\d+)\]", operand)
        if m:
            return range(int(m.group(1)), int(m.group(2)) + 1)
        m = re.match(r"v(\d+)$", operand)
        return range(int(m.group(1)), int(m.group(1)) + 1) if m else None

    def is_f16_matrix(name):
        return isinstance(name, str) and name.startswith("v_mfma_f32_16x16x") and name.endswith("_f16")

    def merge(a, b):
        """Union of two states (register -> set of possible last writers; None = possibly unwritten)."""
        if a is None:
            return {r: set(w) for r, w in b.items()}
        out = {}
        for reg in set(a) | set(b):
            out[reg] = set(a.get(reg, {None})) | set(b.get(reg, {None}))
        return out

    functions = {}
    for fn, label, instructions in assembly:
        functions.setdefault(fn, []).append((label, instructions))
    checked = across_branches = 0
    for fn, blocks in functions.items():
        carried = {}                                          # label -> state carried by the branches that target it
        for sweep in range(8):
            before = {k: {r: frozenset(w) for r, w in v.items()} for k, v in carried.items()}
            state, final = {}, sweep > 0
            for label, instructions in blocks:
                if label in carried:
                    state = merge(state, carried[label]) if state is not None else merge(None, carried[label])
                elif state is None:
                    state = {}                                # unreachable in layout order and not (yet) a branch target
                for name, operands in instructions:
                    ops = [o.strip() for o in operands.split(",")]
                    if name.startswith(("s_cbranch", "s_branch")) and ops and ops[0].startswith(".LBB"):
                        carried[ops[0]] = merge(carried.get(ops[0]), state)
                        if name == "s_branch":
                            state = None                      # nothing falls through
                        continue
                    if name in ("s_endpgm", "s_setpc_b64"):
                        state = None
                        continue
                    if state is None:
                        state = {}
                    if final and is_f16_matrix(name) and len(ops) > 3 and registers(ops[3]) is not None:    # (a literal 0 starts a chain)
                        for reg in registers(ops[3]):
                            writers = state.get(reg, {None})
                            assert None not in writers, (fn, label, "accumulator input with a possibly unknown producer", name, operands)
                            for w in writers:
                                if is_f16_matrix(w):
                                    assert w == name, (fn, label, w, name)
                                    checked += 1
                            across_branches += len(writers) > 1
                    if ops and name.startswith(("v_", "ds_read", "global_load", "buffer_load", "scratch_load")) and registers(ops[0]) is not None:
                        for reg in registers(ops[0]):
                            state[reg] = {name}
            if sweep > 0 and before == {k: {r: frozenset(w) for r, w in v.items()} for k, v in carried.items()}:
                break
        else:
            raise AssertionError((fn, "the register states did not settle"))
    assert checked > 400                                      # four registers per chained instruction
