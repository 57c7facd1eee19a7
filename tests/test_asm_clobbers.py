"""Inline assembly and the register allocator: what an asm block overwrites, it must declare.

The direct global->LDS load for a subset of lanes (tenmo_amd/csrc/gfx950_asm.hpp) narrows the execution mask with
s_and_b64, which also sets SCC.  While the block did not declare "scc", the compiler was free to keep a carry in SCC across
it, and in some instantiations of the short-reduction kernel it did: s_add_u32 before the block, s_addc_u32 behind it, the
high half of a 64-bit load address one too large — a load 4 GiB away from its operand and a GPU memory fault in exactly the
instantiations that had this schedule (never in the others, never on the CPU).  Two checks:
  * every asm statement of the kernel sources that contains an instruction writing SCC or VCC lists that register, and one
    that contains a vector-memory load keeps 5 wait states between its first instruction and that load (the load's scalar
    base may have been written by a vector instruction just before the block: the compiler pads its own loads for that
    documented hazard of the chip but does not look inside a block);
  * the generated gfx950 ISA of gemm_smallk.hip (the one unit that uses such a block) has no instruction reading SCC behind
    an asm block that overwrites it before something else sets it again.
"""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "tenmo_amd", "csrc")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# scalar instructions that set SCC (gfx9: the SOP2 / SOP1 / SOPC arithmetic, logic, shift and compare groups)
SCC_WRITERS = re.compile(r"\b(s_add_[ui]32|s_sub_[ui]32|s_addc_u32|s_subb_u32|s_cmp_\w+|s_and_b\d+|s_or_b\d+|s_xor_b\d+|s_andn2_b\d+|s_orn2_b\d+|"
                         r"s_nand_b\d+|s_nor_b\d+|s_xnor_b\d+|s_lshl_b\d+|s_lshr_b\d+|s_ashr_i\d+|s_bfe_\w+|s_abs_i32|s_min_[ui]32|s_max_[ui]32|s_not_b\d+|"
                         r"s_wqm_b\d+|s_quadmask_b\d+|s_bitcmp\d_b\d+|s_absdiff_i32|s_\w+_saveexec_b64|s_lshl[1-4]_add_u32)\b")
SCC_READERS = re.compile(r"^\s*(s_addc_u32|s_subb_u32|s_cselect_b32|s_cselect_b64|s_cbranch_scc0|s_cbranch_scc1|s_cmov_b32|s_cmov_b64)\b")
VCC_WRITERS = re.compile(r"\bv_cmp\w*_e32\b|\bvcc\s*,")


def asm_statements(text):
    """(template string, clobber string) of every asm statement with a non-empty template."""
    out = []
    for m in re.finditer(r"asm\s+volatile\s*\(", text):
        depth, i = 1, m.end()
        while depth:
            depth += {"(": 1, ")": -1}.get(text[i], 0)
            i += 1
        body = re.sub(r"//[^\n]*", "", text[m.end():i - 1])  # comments between the template's lines
        # the sections of the statement: split at the colons that are outside string literals
        sections, current, in_string, k = [], "", False, 0
        while k < len(body):
            c = body[k]
            if c == "\\" and in_string:
                current += body[k:k + 2]
                k += 2
                continue
            if c == '"':
                in_string = not in_string
            if c == ":" and not in_string:
                sections.append(current)
                current = ""
            else:
                current += c
            k += 1
        sections.append(current)
        template = "".join(re.findall(r'"((?:[^"\\]|\\.)*)"', sections[0])).replace("\\n", "\n").replace("\\t", "\t")
        clobbers = sections[3] if len(sections) > 3 else ""
        if template.strip():
            out.append((template, clobbers))
    return out


def test_asm_statements_declare_what_they_overwrite():
    seen = 0
    for name in sorted(os.listdir(CSRC)):
        for template, clobbers in asm_statements(open(os.path.join(CSRC, name)).read()):
            seen += 1
            if SCC_WRITERS.search(template):
                assert '"scc"' in clobbers, (name, template)
            if VCC_WRITERS.search(template):
                assert '"vcc"' in clobbers, (name, template)
            if "global_load" in template:
                wait_states = 0
                for instr in template.split("\n"):
                    instr = instr.strip()
                    if instr.startswith("global_load"):
                        break
                    nop = re.match(r"s_nop\s+(\d+)", instr)
                    wait_states += int(nop.group(1)) + 1 if nop else (1 if instr else 0)
                assert wait_states >= 5, (name, template, wait_states)
            if "exec" in template:  # the execution mask is saved and restored inside the block
                assert re.search(r"s_mov_b64 %\d, exec", template) and re.search(r"s_mov_b64 exec, %\d", template), (name, template)
    assert seen >= 2


def scan_isa(text):
    """SCC readers scheduled behind an asm block that overwrites SCC, before anything else sets it."""
    hits, kernel = [], None
    lines = text.split("\n")
    i = 0
    while i < len(lines):
        m = re.match(r"^(_Z\S+):", lines[i])
        if m:
            kernel = m.group(1)
        if "ASMSTART" in lines[i]:
            j = i + 1
            overwrites = False
            while "ASMEND" not in lines[j]:
                overwrites = overwrites or bool(SCC_WRITERS.search(lines[j]))
                j += 1
            if overwrites:
                k = j + 1
                while k < len(lines):
                    t = lines[k]
                    if "ASMSTART" in t or t.strip().startswith(".LBB") or "s_endpgm" in t:
                        break
                    if SCC_READERS.match(t):
                        hits.append((kernel, k + 1, t.strip()))
                        break
                    if SCC_WRITERS.search(t):
                        break
                    k += 1
            i = j
        i += 1
    return hits


def test_the_scan_finds_the_schedule_that_faulted():
    """The scanner on the sequence the compiler produced while the clobber was missing (K-major operands, one K step)."""
    bad = """_ZN5tenmo18gemm_smallk_kernelILi0ELi0ELi1ELi4ELb0EEEvNS_8GemmArgsEjjji:
	s_add_u32 s2, s17, s2
	v_readfirstlane_b32 s17, v10
	;;#ASMSTART
	s_mov_b32 m0, s17
	s_mov_b64 s[34:35], exec
	v_cmp_ne_u32_e32 vcc, 0, v7
	s_and_b64 exec, exec, vcc
	global_load_lds_dwordx4 v11, s[30:31]
	s_mov_b64 exec, s[34:35]
	;;#ASMEND
	v_add_lshl_u32 v12, v4, v12, 2
	s_addc_u32 s3, s20, s3
	s_endpgm
"""
    assert [h[2] for h in scan_isa(bad)] == ["s_addc_u32 s3, s20, s3"]
    good = bad.replace("\ts_addc_u32 s3, s20, s3\n", "").replace("\tv_readfirstlane_b32 s17, v10\n", "\ts_addc_u32 s3, s20, s3\n\tv_readfirstlane_b32 s17, v10\n")
    assert scan_isa(good) == []


# instructions that read M0 implicitly (gfx9): loads with an LDS destination, relative moves, messages, interpolation, GWS
M0_USERS = re.compile(r"\bm0\b|_lds_|\blds\b|movrel|s_sendmsg|v_interp|ds_gws|lds_direct|s_ttrace")


def scan_m0(text):
    """(line, text) of every instruction outside an asm block that names M0 or reads it implicitly, and of every asm
    block that reads M0 before writing it."""
    hits, inside, written = [], False, False
    for n, line in enumerate(text.split("\n"), 1):
        if "ASMSTART" in line:
            inside, written = True, False
            continue
        if "ASMEND" in line:
            inside = False
            continue
        code = line.split(";")[0]
        if not code.strip() or code.lstrip().startswith("."):
            continue
        if not inside:
            if M0_USERS.search(code):
                hits.append((n, code.strip()))
        else:
            if re.match(r"\s*s_mov_b32 m0,", code):
                written = True
            elif M0_USERS.search(code) and not written:
                hits.append((n, code.strip()))
    return hits


def test_the_m0_scan_sees_a_compiler_generated_user():
    ok = "\t;;#ASMSTART\n\ts_mov_b32 m0, s17\n\ts_nop 3\n\tglobal_load_lds_dwordx4 v11, s[30:31]\n\t;;#ASMEND\n\tv_add_u32 v1, v2, v3\n"
    assert scan_m0(ok) == []
    assert [h[1] for h in scan_m0(ok + "\tv_movrels_b32 v1, v2\n")] == ["v_movrels_b32 v1, v2"]
    assert [h[1] for h in scan_m0(ok + "\ts_mov_b32 m0, s3\n")] == ["s_mov_b32 m0, s3"]
    assert len(scan_m0(ok.replace("\ts_mov_b32 m0, s17\n", ""))) == 1  # a block that reads M0 without setting it


def device_units():
    """(name, extra flags, source) of every translation unit of the library, as tenmo_amd/build.py compiles them."""
    import importlib

    b = importlib.import_module("tenmo_amd.build")
    units = [("tenmo_hip", [], "tenmo_hip.hip")]
    for bm, bn, sk in b.TILES:
        units.append((f"gemm_{bm}x{bn}_{sk}", [f"-DTENMO_TILE_BM={bm}", f"-DTENMO_TILE_BN={bn}", f"-DTENMO_TILE_STREAMK={sk}"], "gemm_tiles.hip"))
    for extra in sorted(f for f in os.listdir(CSRC) if f.endswith(".hip") and f not in ("tenmo_hip.hip", "gemm_tiles.hip")):
        units.append((extra[:-4], [], extra))
    return b.FLAGS, units


@pytest.fixture(scope="module")
def device_isa():
    """name -> gfx950 assembly text of every translation unit (compiled in parallel, about a minute; kept under tests/_build/isa and
    shared with tests/test_isa_emulation.py until a source changes)."""
    import sys

    sys.path.insert(0, os.path.join(ROOT, "tests", "isa"))
    import harness

    return {name: open(path).read() for name, path in harness.compile_all().items()}


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="no hipcc")
def test_generated_isa_keeps_nothing_in_scc_across_the_masked_load(device_isa):
    text = device_isa["gemm_smallk"]
    assert text.count("global_load_lds_dwordx4") > 100 and "s_and_b64 exec, exec, vcc" in text  # the blocks are there
    for name, isa in device_isa.items():
        assert scan_isa(isa) == [], name


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="no hipcc")
def test_generated_isa_has_no_user_of_m0_outside_the_asm_blocks(device_isa):
    """The direct-load blocks write M0 without declaring it (the compiler accepts no such declaration).  That is sound as
    long as the compiler itself never uses M0 in these units: then there is no value of its own in M0 that a block could
    destroy, and nothing of its own that could read a block's value.  Checked on the generated code of every unit: no
    instruction outside an asm block names M0 or reads it implicitly, and every block that reads it sets it first."""
    blocks = 0
    for name, isa in device_isa.items():
        assert scan_m0(isa) == [], name
        blocks += isa.count("s_mov_b32 m0,")
    assert blocks > 1000


def innermost_loops(text):
    """(kernel, label, instructions) of every innermost loop: the instructions from a label to a branch back to it that
    enclose no other backward branch."""
    loops = []
    kernels, name, code = [], None, []
    for line in text.split("\n"):
        m = re.match(r"^(_Z\S+):", line)
        if m:
            if name:
                kernels.append((name, code))
            name, code = m.group(1), []
            continue
        if name is None:
            continue
        m = re.match(r"^(\.LBB\S+):", line)
        if m:
            code.append(m.group(1) + ":")
            continue
        c = line.split(";")[0].strip()
        if c and not c.startswith("."):
            code.append(c)
    if name:
        kernels.append((name, code))
    for name, code in kernels:
        at = {c[:-1]: i for i, c in enumerate(code) if c.endswith(":")}
        back = [(at[c.split()[-1]], i) for i, c in enumerate(code) if c.startswith(("s_cbranch", "s_branch")) and at.get(c.split()[-1], i) < i]
        for lo, hi in back:
            if not any((l2, h2) != (lo, hi) and lo <= l2 and h2 <= hi for l2, h2 in back):
                loops.append((name, code[lo][:-1], [c for c in code[lo:hi + 1] if not c.endswith(":")]))
    return loops


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="no hipcc")
def test_no_spilled_register_is_touched_inside_a_k_loop(device_isa):
    """Some persistent kernels (stream-K, the batch-reducing launch) keep so much state across their tiles that the compiler
    spills a few registers to scratch memory.  That is harmless as long as the spills sit in the per-tile prologue and
    epilogue: the loops that issue MFMAs — the K loops, where the time goes — must not read or write scratch memory."""
    mfma_loops = 0
    for name, isa in device_isa.items():
        for kernel, label, body in innermost_loops(isa):
            if not any(i.startswith("v_mfma") for i in body):
                continue
            mfma_loops += 1
            touched = [i for i in body if i.startswith("scratch_") or i.startswith("buffer_") and "offen" in i and "s[0:3]" in i]
            assert not touched, (name, kernel, label, touched[:3])
    assert mfma_loops > 150


def test_the_loop_scan_sees_a_spill():
    bad = "_Zkernel:\n.LBB0_1:\n\tv_mfma_f32_32x32x2_f32 a[0:15], v0, v1, a[0:15]\n\tscratch_load_dword v3, off, off offset:4\n\ts_cbranch_vccnz .LBB0_1\n\ts_endpgm\n"
    loops = innermost_loops(bad)
    assert len(loops) == 1 and any(i.startswith("scratch_") for i in loops[0][2])
    assert innermost_loops(bad.replace("s_cbranch_vccnz .LBB0_1", "s_cbranch_vccnz .LBB0_2")) == []
    # an outer loop around it is not what is checked: only the inner one counts
    nested = bad.replace(".LBB0_1:", ".LBB0_0:\n\tscratch_load_dword v9, off, off\n.LBB0_1:").replace("\ts_endpgm", "\ts_cbranch_scc1 .LBB0_0\n\ts_endpgm")
    assert [l[1] for l in innermost_loops(nested)] == [".LBB0_1"]
