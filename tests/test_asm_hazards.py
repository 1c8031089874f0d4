"""Instruction-level checks of the generated gfx950 code (no GPU needed, hipcc only).

The kernels issue some instructions as asm statements: matrix products whose accumulators must stay in AGPRs, and
direct HBM -> LDS loads whose waits are placed by hand. The compiler places the wait states that the hardware wants
between dependent instructions only in front of instructions it issues itself, so two dependencies are the source's
own business and are checked here on the code of every build:

* an ordinary vector instruction must not write a register that an asm matrix instruction reads within the next three
  instructions (a v_mov materialising the all-ones operand of the row-sum product right in front of it made a quarter
  of the lanes read the old register contents);
* a vector instruction that writes a scalar register (v_readfirstlane, v_readlane, v_cmp) must be five wait states
  ahead of a memory instruction that reads that register (an unsettled pointer is read with its old high half);
* the result registers of an asm matrix instruction must not be read or written by any other kind of instruction
  within eleven wait states of it (the product has to leave the matrix core first);
* the data registers of a store of more than 8 bytes must not be written by a vector instruction within the two wait
  states behind the store (the norm+rope kernel's streaming stores are asm statements).
"""
import functools
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "iris_c_amd", "csrc")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


@functools.lru_cache(maxsize=None)
def isa(name):
    if not os.path.exists(HIPCC):
        pytest.skip("no hipcc here")
    r = subprocess.run([HIPCC, "-O3", "--offload-arch=gfx950", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
                        "-packed-fp32-ops", "-I" + CSRC, "-I" + os.path.join(ROOT, "include"), "--cuda-device-only", "-S",
                        "-o", "-", os.path.join(CSRC, name)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    ins = [l.strip() for l in r.stdout.splitlines()]
    return [l for l in ins if l and not l.startswith((";", ".")) and not l.endswith(":")]


def vregs(tok):
    m = re.match(r"([va])\[(\d+):(\d+)\]", tok)
    if m:
        return {(m.group(1), i) for i in range(int(m.group(2)), int(m.group(3)) + 1)}
    m = re.match(r"([va])(\d+)$", tok)
    return {(m.group(1), int(m.group(2)))} if m else set()


def sregs(tok):
    m = re.match(r"s\[(\d+):(\d+)\]", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"s(\d+)$", tok)
    return {int(m.group(1))} if m else set()


def operands(line):
    return [t.strip().split()[0] for t in line.split(None, 1)[1].split(",")] if " " in line else []


@pytest.mark.parametrize("name,least", [("fa_fwd_hd512_gfx950.hip", 300), ("gemm_conv_gfx950.hip", 300)])
def test_no_vector_instruction_feeds_an_asm_matrix_instruction_directly(name, least):
    """The sources whose matrix products are asm statements."""
    ins = isa(name)
    products = 0
    for i, l in enumerate(ins):
        if not l.startswith("v_mfma"):
            continue
        products += 1
        src = set().union(*[vregs(t) for t in operands(l)[1:]])
        for back in (1, 2, 3):
            p = ins[i - back]
            if p.startswith("v_") and not p.startswith("v_mfma"):
                assert not (vregs(operands(p)[0]) & src), f"{name}: {p}  feeds  {l}"
    assert products > least


@pytest.mark.parametrize("name", sorted(f for f in os.listdir(CSRC) if f.endswith(".hip")))
def test_scalar_registers_written_by_vector_instructions_settle_before_memory_instructions_read_them(name):
    """Every kernel source: the compiler's own memory instructions pass by construction, the asm ones must."""
    ins = isa(name)
    loads = 0
    for i, l in enumerate(ins):
        if not l.startswith(("global_", "buffer_", "scratch_", "flat_")):
            continue
        loads += 1
        read = set().union(*[sregs(t) for t in operands(l)])
        if not read:
            continue
        waits = 0
        for back in range(1, 7):
            p = ins[i - back]
            if waits < 5 and (p.startswith(("v_readfirstlane", "v_readlane")) or (p.startswith("v_cmp") and p.split()[1].startswith("s"))):
                assert not (sregs(operands(p)[0]) & read), f"{name}: {p}  is {waits} wait states ahead of  {l}"
            m = re.match(r"s_nop (\d+)", p)
            waits += int(m.group(1)) + 1 if m else 1
    assert loads > 0


@pytest.mark.parametrize("name", sorted(f for f in os.listdir(CSRC) if f.endswith(".hip")))
def test_data_registers_of_a_wide_store_are_left_alone_right_behind_it(name):
    ins = isa(name)
    for i, l in enumerate(ins):
        if not re.match(r"(global|flat|scratch)_store_dwordx[34]", l):
            continue
        data = vregs(operands(l)[1])
        waits = 0
        for p in ins[i + 1:i + 3]:
            if waits < 2 and p.startswith("v_"):
                assert not (vregs(operands(p)[0]) & data), f"{name}: {p}  overwrites the data of  {l}"
            m = re.match(r"s_nop (\d+)", p)
            waits += int(m.group(1)) + 1 if m else 1


@pytest.mark.parametrize("name", ["fa_fwd_hd512_gfx950.hip", "gemm_conv_gfx950.hip"])
def test_results_of_asm_matrix_instructions_are_left_alone_until_they_have_left_the_matrix_core(name):
    ins = isa(name)
    for i, l in enumerate(ins):
        if not l.startswith("v_mfma"):
            continue
        result = vregs(operands(l)[0])
        waits = 0
        for p in ins[i + 1:i + 14]:
            if waits >= 11:
                break
            if not p.startswith(("v_mfma", "s_")):
                touched = set().union(*[vregs(t) for t in operands(p)]) if operands(p) else set()
                assert not (touched & result), f"{name}: {p}  touches the result of  {l}  {waits} wait states behind it"
            m = re.match(r"s_nop (\d+)", p)
            waits += int(m.group(1)) + 1 if m else 1
