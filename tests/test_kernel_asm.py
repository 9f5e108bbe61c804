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
* the scalar base address of a copy is written by a scalar move inside the copy's own asm
  statement (a vector memory instruction may read a scalar register only five wait states
  after a vector-ALU instruction - a v_readlane that reads a spilled scalar back - wrote it;
  after the scalar ALU it may read it at once);
* the compiler never writes an AccVGPR itself (v_accvgpr_write / v_accvgpr_mov: it would be
  moving an accumulator out of the way or back, around matrix instructions whose wait states
  it does not know), and reads one (for a C store) no sooner than four matrix instructions
  after the last one that wrote it; the same distance holds for the accumulators that live in
  ordinary registers and whatever reads them.
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
    assert len(found) == 16
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
        # the three variants of a K iteration, for full tiles and (two copies) for short ones
        assert n_mfma == 3 * 192 + 6 * 128


def test_copy_base_goes_through_a_scalar_move(kernels):
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
            # written by the scalar ALU inside the same asm statement
            assert code[i - 3].startswith("s_mov_b64"), (name, code[i - 3])
            assert _registers(_operands(code[i - 3])[0], "s") == base, (name, code[i - 3], ins)
        assert copies >= 2 * 14 + 9 * 14          # prologue and the nine iteration variants


def test_accumulators_stay_where_they_are(kernels):
    found, _ = kernels
    for name, code in found.items():
        reads = 0
        for i, ins in enumerate(code):
            assert not ins.startswith(("v_accvgpr_write", "v_accvgpr_mov")), (name, ins)
            if not ins.startswith("v_accvgpr_read"):
                continue
            reads += 1
            source = _registers(_operands(ins)[1], "a")
            seen, k = 0, i - 1
            while seen < 4 and k >= 0 and not code[k].startswith("s_nop 15"):   # (the explicit wait)
                if code[k].startswith("v_mfma"):
                    seen += 1
                    assert not (_registers(_operands(code[k])[0], "a") & source), (name, code[k], ins)
                k -= 1
        assert reads > 0


def test_vgpr_accumulators_are_read_well_after_their_last_update(kernels):
    found, _ = kernels
    for name, code in found.items():
        recent = []       # destination registers of the last four matrix instructions
        checked = 0
        for ins in code:
            if ins.startswith("v_mfma"):
                recent = (recent + [_registers(_operands(ins)[0], "v")])[-4:]
                continue
            if ins.startswith("s_nop 15"):      # (the explicit wait before a block's last stores)
                recent = []
                continue
            live = set().union(*recent) if recent else set()
            if not live or not ins.startswith(("v_", "global_", "ds_", "buffer_", "scratch_", "flat_")):
                continue
            ops = _operands(ins)
            writes_first = not ins.startswith(("global_store", "ds_write", "ds_store", "buffer_store"))
            for token in ops[1:] if writes_first else ops:
                checked += 1
                assert not (_registers(token, "v") & live), (name, ins)
        assert checked > 0
