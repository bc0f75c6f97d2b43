"""Rules the hardware does not enforce, checked on the generated code of the kernels that write instructions in
assembly (hodu_amd/csrc/gfx950_insn.hpp).  The compiler's hazard recogniser inserts wait states for the instructions
it emits itself; it does not see inside an asm statement, so for those the kernels place the wait states by hand --
and this test reads the gfx950 assembly hipcc generates for them (cross-compiled here, no GPU; the f8e4m3-weight tile
kernels through tests/isa/mi16_f8w_kernels.hip, which instantiates them alone) and holds it to the
rules:

 * results of an MFMA are not interlocked: between a matrix instruction and an instruction that reads the accumulation
   registers it wrote there must be wait states -- up to 18 for the longest instruction (an `s_nop n` is n + 1 of
   them, any other instruction one).  Inside the loops an accumulator is next touched 64 matrix instructions later;
   behind the loop the kernels place `s_nop`s, which the compiler is free to schedule reads of OLDER accumulators in
   front of: the rule checked is that the first instruction that names a register written by one of the final two
   matrix instructions comes at least 18 wait states after the last of them (anything written before those two is
   two matrix instructions, 32 cycles or more, old);
 * M0, which gives an LDS-DMA load its LDS address, is written by a scalar instruction and read by a vector memory
   instruction: one other instruction has to sit between the write and the load;
 * in the respaced-issue kernels nothing but their own `s_add_u32 m0, <base>, <literal>` writes M0, every load carries
   an immediate offset of 0 .. 3 KB on a whole KB, and per kernel the destinations (literal + immediate) of the loop's
   loads are each 1 KB piece of both ring slots exactly once per operand base.
"""
import collections
import os
import re
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

from hodu_amd.build import FLAGS as BUILD_FLAGS

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "hodu_amd", "csrc")
HIPCC = shutil.which("hipcc") or ("/opt/rocm/bin/hipcc" if os.path.exists("/opt/rocm/bin/hipcc") else None)
pytestmark = pytest.mark.skipif(HIPCC is None, reason="no hipcc to generate the assembly with")
MFMA_RESULT_WAIT_STATES = 18


SOURCES = {"tile16": os.path.join(CSRC, "gemm_mfma_mi16_bf16.hip"), "f8_tiles": os.path.join(CSRC, "gemm_mfma_f8.hip"),
           "tile16_f8w": os.path.join(ROOT, "tests", "isa", "mi16_f8w_kernels.hip"), "attention": os.path.join(CSRC, "attention.hip"),
           "builtin_offsets": os.path.join(ROOT, "tests", "isa", "lds_dma_builtin_offsets.hip")}


@pytest.fixture(scope="module")
def assembly(tmp_path_factory):
    """{name: lines of the gfx950 assembly of SOURCES[name]}, compiled side by side"""
    out_dir = tmp_path_factory.mktemp("isa")

    def one(item):
        name, source = item
        out = out_dir / (name + ".s")
        cmd = [HIPCC, *BUILD_FLAGS, "--cuda-device-only", "-S", source, "-o", str(out)]  # the library's own flags
        r = subprocess.run(cmd, capture_output=True, text=True)
        assert r.returncode == 0, r.stderr[-2000:]
        return name, out.read_text().split("\n")
    with ThreadPoolExecutor(max_workers=5) as pool:
        return dict(pool.map(one, SOURCES.items()))


def kernels_in(lines, name_part):
    """{symbol: [instruction, ..]} of the functions whose mangled name contains name_part"""
    found, name = {}, None
    for line in lines:
        text = line.split(";")[0].strip()
        m = re.match(r"^(_Z[\w$.]+):", text)
        if m and name is None:
            name = m.group(1)
            found[name] = []
            continue
        if name is not None:
            if text.startswith(".Lfunc_end"):
                name = None
            elif text and not text.startswith(".") and not text.endswith(":"):
                found[name].append(text)
    return {k: v for k, v in found.items() if name_part in k}


def agprs(operand):
    """a[4:7] -> {4, 5, 6, 7}; a19 -> {19}"""
    m = re.match(r"a\[(\d+):(\d+)\]$", operand)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"a(\d+)$", operand)
    return {int(m.group(1))} if m else set()


def wait_states_before_the_last_results_are_read(insns):
    """wait states between the last matrix instruction (in program text: the loop and its peeled copies come first) and
    the first later instruction that names a register the last TWO matrix instructions wrote"""
    mfmas = [i for i, s in enumerate(insns) if s.startswith("v_mfma")]
    fresh = set()
    for i in mfmas[-2:]:
        fresh |= agprs(insns[i].split(None, 1)[1].split(",")[0].strip())
    assert fresh
    states = 0
    for s in insns[mfmas[-1] + 1:]:
        named = set()
        for operand in re.findall(r"\ba(?:\[\d+:\d+\]|\d+)", s):
            named |= agprs(operand)
        if named & fresh:
            return states
        m = re.match(r"s_nop (\d+)", s)
        states += int(m.group(1)) + 1 if m else 1
    return states


def loads_too_close_to_an_m0_write(insns):
    bad, since_write = [], None
    for s in insns:
        if re.match(r"s_\w+ m0,", s):
            since_write = 0
            continue
        if s.startswith("global_load_lds"):
            if since_write is None or since_write < 1:
                bad.append(s)
        if since_write is not None:
            since_write += 1
    return bad


@pytest.fixture(scope="module")
def tile16(assembly):
    return assembly["tile16"]


@pytest.fixture(scope="module")
def f8_tiles(assembly):
    return assembly["f8_tiles"]


@pytest.fixture(scope="module")
def tile16_f8w(assembly):
    return assembly["tile16_f8w"]


def test_accumulators_are_read_only_after_the_wait_states(tile16, f8_tiles, tile16_f8w):
    checked = 0
    for lines, part in ((tile16, "mfma_pipe16_kernel"), (tile16, "mfma_pipe16r_kernel"), (f8_tiles, "mfma_pipe_f8x16_kernel"),
                        (tile16_f8w, "mfma_pipe16_f8w_kernel"), (tile16_f8w, "mfma_pipe16r_f8w_kernel")):
        kernels = kernels_in(lines, part)
        assert kernels, part
        for name, insns in kernels.items():
            assert wait_states_before_the_last_results_are_read(insns) >= MFMA_RESULT_WAIT_STATES, name
            checked += 1
    assert checked == 4 + 8 + 2 + 2 + 2  # four layout pairs; the respaced form with and without fused steps; e4m3 and e5m2;
    # f8e4m3 weights k-dense and row-dense, both forms


def test_an_instruction_separates_every_m0_write_from_the_load_that_uses_it(tile16, f8_tiles, tile16_f8w, assembly):
    checked = 0
    for lines, part in ((tile16, "mfma_pipe16"), (f8_tiles, "mfma_pipe_f8"), (tile16_f8w, "mfma_pipe16"),
                        (assembly["attention"], "attention_fwd_kernel")):
        for name, insns in kernels_in(lines, part).items():
            assert any(s.startswith("global_load_lds") for s in insns), name
            assert loads_too_close_to_an_m0_write(insns) == [], name
            checked += 1
    assert checked >= 12 + 4 + 4 + 8  # .. and the attention kernel: two types x two head dims, with and without a mask


def test_respaced_kernels_m0_bookkeeping(tile16):
    kernels = kernels_in(tile16, "mfma_pipe16r_kernel")
    assert len(kernels) == 8  # four layout pairs, with and without fused steps
    for name, insns in kernels.items():
        m0 = None
        per_base = collections.defaultdict(list)
        for s in insns:
            w = re.match(r"s_add_u32 m0, (s\d+), (\S+)", s)
            if w:
                m0 = (w.group(1), int(w.group(2), 0))
                continue
            assert not re.match(r"[sv]_\w+ m0,", s), (name, s)  # nothing else writes M0
            ld = re.match(r"global_load_lds_dwordx4 v\d+, s\[\d+:\d+\](?: offset:(\S+))?", s)
            if ld:
                imm = int(ld.group(1), 0) if ld.group(1) else 0
                assert m0 is not None and imm % 1024 == 0 and 0 <= imm <= 3072, (name, s)
                per_base[m0[0]].append(m0[1] + imm)
        assert len(per_base) == 2, name  # the left operand's base register and the right one's
        for base, dests in per_base.items():
            count = collections.Counter(dests)
            assert all(d % 1024 == 0 for d in count), (name, base)
            pieces = sorted(count)
            # prologue and loop each fetch every piece once; the pieces are contiguous KBs of this wavefront's share of
            # slot 0 and, one stage's bytes further on, of slot 1
            assert set(count.values()) == {2}, (name, base, count)
            half = len(pieces) // 2
            assert pieces[:half] == list(range(pieces[0], pieces[0] + half * 1024, 1024)), (name, base, pieces)
            assert pieces[half:] == list(range(pieces[half], pieces[half] + half * 1024, 1024)), (name, base, pieces)


def test_tile_kernels_keep_their_accumulators_in_registers(assembly):
    """no scratch memory in any of these kernels: a rolled loop over the accumulators, or a spill, would put them there
    (the library is built with a raised unroll threshold for that reason; this test uses its flags)"""
    seen = 0
    for lines in assembly.values():
        text = "\n".join(lines)
        for name, size in re.findall(r"\.amdhsa_kernel (\S*mfma_pipe\S*)[\s\S]*?\.amdhsa_private_segment_fixed_size (\d+)", text):
            assert int(size) == 0, (name, size)
            seen += 1
    assert seen >= 18


def test_the_compiler_reads_the_dma_immediate_as_the_respaced_kernels_do(assembly):
    """The respaced kernels rest on one reading of the ISA document: the immediate offset of global_load_lds_dwordx4
    moves the LDS address as well as the global one.  The compiler's builtin for the same instruction documents its
    offset argument as applied to both addresses, and lowers two loads from one global base to one LDS base at offsets
    of 1 and 2 KB to ONE M0 write and two instructions that differ in their immediate only -- the same reading (were
    the LDS address M0's alone, both loads would land on the same 1 KB)."""
    insns = [line.split(";")[0].strip() for line in assembly["builtin_offsets"]]
    m0_writes = [s for s in insns if re.match(r"s_\w+ m0,", s)]
    loads = [s for s in insns if s.startswith("global_load_lds_dwordx4")]
    assert len(m0_writes) == 1 and len(loads) == 2, (m0_writes, loads)
    operands = [re.match(r"global_load_lds_dwordx4 (\S+ \S+) offset:(\d+)$", s).groups() for s in loads]
    assert operands[0][0] == operands[1][0] and [int(o[1]) for o in operands] == [1024, 2048], loads
