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
    """Within a block, a matrix instruction whose accumulator input is the result of an earlier one must have
    the same depth (16x16x16 onto 16x16x16, 16x16x32 onto 16x16x32)."""
    def registers(operand):
        m = re.match(r"v\[(\d+):(\d+)\]", operand.strip())
        return (int(m.group(1)), int(m.group(2))) if m else None
    checked = 0
    for function, label, instructions in assembly:
        producer = {}                                         # register range -> mnemonic of the matrix instruction that wrote it
        for name, operands in instructions:
            ops = [o.strip() for o in operands.split(",")]
            if name.startswith("v_mfma_f32_16x16x") and name.endswith("_f16"):
                dst, src_c = registers(ops[0]), registers(ops[3]) if len(ops) > 3 else None
                if src_c in producer:
                    assert producer[src_c] == name, (function, label, producer[src_c], name)
                    checked += 1
                producer = {r: n for r, n in producer.items() if dst is None or r[1] < dst[0] or r[0] > dst[1]}
                if dst:
                    producer[dst] = name
            elif ops and registers(ops[0]):                  # any other write to a register range ends the chain
                dst = registers(ops[0])
                producer = {r: n for r, n in producer.items() if r[1] < dst[0] or r[0] > dst[1]}
            elif ops and re.match(r"v\d+$", ops[0]):
                reg = int(ops[0][1:])
                producer = {r: n for r, n in producer.items() if not (r[0] <= reg <= r[1])}
    assert checked > 100
