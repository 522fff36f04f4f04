"""Checks on the machine code hipcc generates for the two GEMM sources (CPU only: cross-compiles to assembly).

The direct-to-LDS loads and some matrix instructions are inline assembly, which the compiler does not look
into. Five things it would otherwise take care of are therefore checked on the generated text:

* M0 carries a load's LDS destination. Every `s_mov_b32 m0` in these files is one of ours, so the number of M0
  mentions must equal the number of direct loads, and walking back from every direct load the first M0 write
  must come before the previous direct load (each load has its own write, nothing else touches M0 in between).
* A scalar register written by the vector ALU (`v_readfirstlane`, `v_readlane`) needs five wait states before
  a vector-memory instruction reads it. The compiler inserts them for instructions it knows; in front of an
  inline-assembly load nothing does. No direct load may read such a register within five instructions unless a
  scalar instruction has rewritten it in between.
* A vector register written by the vector ALU needs wait states before a matrix instruction reads it as an
  operand; for the matrix instructions issued from inline assembly nothing inserts them. No matrix instruction
  may read a register that a vector ALU instruction wrote within the two instructions before it (`s_nop n`
  counts as n + 1).
* The result of a matrix instruction issued from inline assembly is not tracked by the compiler either. No
  instruction other than a matrix instruction may read an accumulation register (`a`) within 64 clocks of the
  in-place matrix instruction that last wrote it, counting 16 clocks per matrix instruction in between,
  n + 1 per `s_nop n` and 1 per other instruction (the write-back waits with four `s_nop 15`).
* The kernels whose K loops keep all 256 accumulation registers pinned (`gemm_bf16_early_kernel` for whole
  tiles, `sgemm_wave_tile_dma_kernel`) must not spill: a spill there means the compiler has started to move
  accumulators, which with matrix instructions in inline assembly is also a correctness hazard.
"""
import re
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

from prism_amd import build as pbuild

SOURCES = ["gemm_bf16.hip", "sgemm.hip"]


@pytest.fixture(scope="module")
def assembly(tmp_path_factory):
    out_dir = tmp_path_factory.mktemp("asm")

    def compile_one(name):
        out = out_dir / (name + ".s")
        cmd = [pbuild.hipcc_path(), *pbuild.HIPCC_FLAGS, "-S", "--cuda-device-only", "-o", str(out), str(pbuild.CSRC / name)]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        assert proc.returncode == 0, proc.stderr[-2000:]
        return out.read_text()

    with ThreadPoolExecutor(max_workers=2) as pool:
        return dict(zip(SOURCES, pool.map(compile_one, SOURCES)))


def instructions(text):
    """(kernel symbol, instruction text) for every instruction line, in order."""
    out, kernel = [], None
    for raw in text.splitlines():
        line = raw.split(";")[0].strip()
        if not line or line.startswith((".", "#")):
            continue
        if line.endswith(":"):
            if line.startswith("_Z"):
                kernel = line[:-1]
            continue
        out.append((kernel, line))
    return out


def is_direct_load(ins):
    return ins.startswith("global_load_lds_") or (ins.startswith("buffer_load_") and ins.endswith(" lds"))


def scalar_registers(text):
    regs = set()
    for m in re.finditer(r"s\[(\d+):(\d+)\]", text):
        regs |= set(range(int(m.group(1)), int(m.group(2)) + 1))
    for m in re.finditer(r"(?<![\w\[])s(\d+)\b", text):
        regs.add(int(m.group(1)))
    return regs


@pytest.mark.parametrize("source", SOURCES)
def test_every_direct_load_has_its_own_m0_write(assembly, source):
    ins = [i for _, i in instructions(assembly[source])]
    loads = [n for n, i in enumerate(ins) if is_direct_load(i)]
    m0 = [n for n, i in enumerate(ins) if re.search(r"\bm0\b", i)]
    assert loads and all(ins[n].startswith("s_mov_b32 m0,") for n in m0), "something other than s_mov_b32 touches M0"
    assert len(m0) == len(loads)
    previous = -1
    for n in loads:
        writes = [w for w in m0 if previous < w < n]
        assert len(writes) == 1, f"direct load without an M0 write of its own: {ins[n]}"
        previous = n


@pytest.mark.parametrize("source", SOURCES)
def test_no_vector_written_scalar_is_read_by_a_direct_load_too_soon(assembly, source):
    ins = [i for _, i in instructions(assembly[source])]
    for n, i in enumerate(ins):
        if not is_direct_load(i):
            continue
        wanted = scalar_registers(i)
        for back in range(1, 6):
            if n - back < 0:
                break
            p = ins[n - back]
            written = scalar_registers(p.split(",")[0]) if p.startswith(("s_", "v_readfirstlane", "v_readlane")) else set()
            if p.startswith(("v_readfirstlane", "v_readlane")):
                assert not (written & wanted), f"{p}  ...  {i}  ({back} instructions apart)"
            wanted -= written  # rewritten by a scalar instruction: the load reads that result instead


def vector_registers(text):
    regs = set()
    for m in re.finditer(r"(?<![\w])v\[(\d+):(\d+)\]", text):
        regs |= set(range(int(m.group(1)), int(m.group(2)) + 1))
    for m in re.finditer(r"(?<![\w\[])v(\d+)\b", text):
        regs.add(int(m.group(1)))
    return regs


def test_no_matrix_instruction_reads_a_register_the_vector_alu_has_just_written(assembly):
    ins = [i for _, i in instructions(assembly["gemm_bf16.hip"])]
    checked = 0
    for n, i in enumerate(ins):
        if not i.startswith("v_mfma_"):
            continue
        operands = i.split(None, 1)[1].split(",")
        sources = vector_registers(operands[1]) | vector_registers(operands[2])
        checked += 1
        distance, back = 0, 1
        while distance < 2 and n - back >= 0:
            p = ins[n - back]
            if p.startswith("s_nop"):
                distance += int(p.split()[1]) + 1
            else:
                distance += 1
                if p.startswith("v_") and not p.startswith(("v_mfma_", "v_cmp", "v_readfirstlane", "v_readlane")):
                    written = vector_registers(p.split(None, 1)[1].split(",")[0])
                    assert not (written & sources), f"{p}  ...  {i}"
            back += 1
    assert checked > 1000


def test_pinned_accumulator_kernels_do_not_spill(assembly):
    pinned = {"gemm_bf16.hip": r"gemm_bf16_early_kernelILi256ELi256ELi128ELi128ELb0E", "sgemm.hip": r"sgemm_wave_tile_dma_kernelILi256ELi256ELi\d+ELi32ELi128ELb0E"}  # the whole-tile forms
    for source, pattern in pinned.items():
        text = assembly[source]
        found = 0
        for m in re.finditer(r"^\s*\.amdhsa_kernel\s+(\S+)(.*?)\.end_amdhsa_kernel", text, re.S | re.M):
            if re.search(pattern, m.group(1)):
                found += 1
                size = re.search(r"\.amdhsa_private_segment_fixed_size\s+(\d+)", m.group(2))
                assert size and int(size.group(1)) == 0, f"{m.group(1)} uses {size.group(1) if size else '?'} bytes of scratch"
        assert found >= 2, f"no kernel matching {pattern} in {source}"


def accumulation_registers(text):
    regs = set()
    for m in re.finditer(r"\ba\[(\d+):(\d+)\]", text):
        regs |= set(range(int(m.group(1)), int(m.group(2)) + 1))
    for m in re.finditer(r"(?<![\w\[])a(\d+)\b", text):
        regs.add(int(m.group(1)))
    return regs


def test_no_accumulator_is_read_too_soon_after_an_in_place_matrix_instruction(assembly):
    """In gemm_bf16_early_kernel the accumulating v_mfma_f32_16x16x32_bf16 comes from inline assembly (between
    the compiler's ASMSTART / ASMEND marks) with its destination as addend. Reads and copies of its result by
    anything but another matrix instruction (the write-back's stores, a compiler-made copy) must keep their
    distance; results of matrix instructions the compiler issued itself are its own business."""
    reads, from_asm = 0, 0
    last_write = {}  # accumulation register -> clock of the inline-assembly matrix instruction that wrote it
    clock, kernel, in_asm = 0, None, False
    for raw in assembly["gemm_bf16.hip"].splitlines():
        if "#ASMSTART" in raw:
            in_asm = True
        elif "#ASMEND" in raw:
            in_asm = False
        i = raw.split(";")[0].strip()
        if not i or i.startswith((".", "#")):
            continue
        if i.endswith(":"):
            if i.startswith("_Z"):
                kernel, clock, last_write = i[:-1], 0, {}
            continue
        if kernel is None or "gemm_bf16_early_kernel" not in kernel:
            continue
        if i.startswith("v_mfma_"):
            clock += 16
            dest = i.split(None, 1)[1].split(",")[0]
            for r in accumulation_registers(dest):
                if in_asm:
                    last_write[r] = clock
                    from_asm += 1
                else:
                    last_write.pop(r, None)
            continue
        clock += int(i.split()[1]) + 1 if i.startswith("s_nop") else 1
        used = accumulation_registers(i.split(None, 1)[1]) if " " in i else set()
        for r in used:
            reads += 1
            assert clock - last_write.get(r, -10**9) >= 64, f"{kernel}: `{i}` reads a{r} {clock - last_write[r]} clocks after its matrix instruction"
    assert reads >= 512 and from_asm >= 512  # two instances, 256 accumulation registers each, at least
