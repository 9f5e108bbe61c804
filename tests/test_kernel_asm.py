"""The one-wave-per-SIMD GEMM kernel (ccglib_amd/csrc/gemm_mfma_wide.h) issues its matrix
instructions and its global -> LDS copies from inline asm statements, which the compiler does
not look into: it neither inserts the wait states such an instruction needs after what stands
in front of the statement, nor knows that the statements' explicit `s_waitcnt vmcnt(n)` counts
assume that no other memory instruction is in flight. This test compiles every instantiation
the library launches to assembly (tests/cpp/wide_kernels.hip; hipcc cross-compiles, no GPU
needed) and checks what the source can only arrange for:

* no kernel spills to scratch memory (a spill is a memory instruction of the compiler's);
* no vector-ALU instruction writes a register that a matrix instruction reads as its A or B
  operand within the two instructions before it (an operand derived from a fragment has to be
  computed several matrix instructions ahead; the hardware needs two wait states);
* the scalar base address of a copy is not written by v_readlane / v_readfirstlane within the
  three instructions before the copy's asm statement (a vector memory instruction may read a
  scalar register five wait states after a vector-ALU instruction wrote it; the statement's
  own s_mov and s_nop are two of them).
"""
import os
import re
import subprocess
import tempfile

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-command-line-argument", "--cuda-device-only", "-S"]


@pytest.fixture(scope="module")
def kernels():
    """name -> list of instructions (comments, labels and directives dropped)."""
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "wide_kernels.s")
        r = subprocess.run(["hipcc"] + FLAGS + [os.path.join(HERE, "cpp", "wide_kernels.hip"), "-o", out],
                           capture_output=True, text=True)
        assert r.returncode == 0, r.stderr[-2000:]
        text = open(out).read()
    found, name = {}, None
    scratch = dict(re.findall(r"\.amdhsa_kernel (\S+)[\s\S]*?\.amdhsa_private_segment_fixed_size (\d+)", text))
    for line in text.splitlines():
        s = line.strip()
        m = re.match(r"^(_ZN\S*complex_gemm_mfma_wide\S*):", s)
        if m:
            name = m.group(1)
            found[name] = []
        elif s.startswith(".Lfunc_end"):
            name = None
        elif name and s and not s.startswith((";", ".")) and not s.endswith(":"):
            found[name].append(s.split(";")[0].strip())
    assert len(found) == 14
    return found, scratch


def _registers(token, files):
    """'v[4:7]' -> {('v', 4), ...}; 's12' -> {('s', 12)}; other operands -> empty."""
    m = re.match(r"^([%s])\[(\d+):(\d+)\]$" % files, token)
    if m:
        return {(m.group(1), n) for n in range(int(m.group(2)), int(m.group(3)) + 1)}
    m = re.match(r"^([%s])(\d+)$" % files, token)
    return {(m.group(1), int(m.group(2)))} if m else set()


def _operands(instruction):
    parts = instruction.split(None, 1)
    return [t.strip() for t in parts[1].split(",")] if len(parts) > 1 else []


def test_no_kernel_spills_to_scratch(kernels):
    found, scratch = kernels
    for name in found:
        assert int(scratch[name]) == 0, name


def test_matrix_operands_are_not_written_right_before_their_use(kernels):
    found, _ = kernels
    for name, code in found.items():
        n_mfma = 0
        for i, ins in enumerate(code):
            if not ins.startswith("v_mfma"):
                continue
            n_mfma += 1
            ops = _operands(ins)
            sources = _registers(ops[1], "va") | _registers(ops[2], "va")
            for back in (1, 2):
                prev = code[i - back]
                if prev.startswith("v_") and not prev.startswith(("v_mfma", "v_cmp", "v_readlane",
                                                                   "v_readfirstlane")):
                    written = _registers(_operands(prev)[0], "va")
                    assert not (written & sources), (name, prev, ins)
        assert n_mfma == 4 * 192     # the four variants of a K iteration


def test_copy_base_is_not_fresh_out_of_a_vector_register(kernels):
    found, _ = kernels
    for name, code in found.items():
        copies = 0
        for i, ins in enumerate(code):
            if not ins.startswith("global_load_lds_dwordx4"):
                continue
            copies += 1
            base = _registers(_operands(ins)[1], "s")
            assert base, ins                      # a scalar register pair, not a vector one
            assert code[i - 2].startswith("s_mov_b32 m0") and code[i - 1].startswith("s_nop")
            for back in (3, 4, 5):                # the three instructions before the statement
                prev = code[i - back]
                if prev.startswith(("v_readlane_b32", "v_readfirstlane_b32")):
                    assert not (_registers(_operands(prev)[0], "s") & base), (name, prev, ins)
        assert copies >= 2 * 14 + 4 * 14          # prologue and the four iteration variants
