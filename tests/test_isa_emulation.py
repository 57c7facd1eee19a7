"""The generated gfx950 code of the kernels, executed on the CPU.

tests/isa/gfx950.py interprets the assembly hipcc emits for the library's translation units; tests/isa/harness.py feeds it the
launches that the CPU replay records (kernel, grid, argument block, every device allocation before and after).  A case passes
when the interpreted machine code leaves in memory what the replay of the C++ source left there, with every global and LDS
access in bounds, results of loads used only after the wait that covers them, and the wait states an asm block owes kept.
This is the check that sees what the compiler made of the source: the one GPU fault of this code base — a carry parked in SCC
across an inline-assembly block that overwrote it — is invisible to the source-level replay and is found here (first test).
No GPU involved.
"""
import os
import re
import shutil
import subprocess
import sys
from concurrent.futures import ProcessPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests", "replay"))
sys.path.insert(0, os.path.join(ROOT, "tests", "isa"))
import build as replay_build  # noqa: E402
import gfx950  # noqa: E402
import harness  # noqa: E402

pytestmark = pytest.mark.skipif(not (replay_build.available() and os.path.exists(harness.HIPCC)), reason="needs the host clang++ and hipcc")


@pytest.fixture(scope="module")
def exe():
    return replay_build.build_gemm_plain()


@pytest.fixture(scope="module")
def isa():
    return harness.compile_all()


def record(exe, case, cus, where):
    shutil.rmtree(where, ignore_errors=True)
    os.makedirs(where)
    res = subprocess.run([exe, "early", case], env=dict(os.environ, REPLAY_CUS=str(cus), REPLAY_DUMP_DIR=str(where)), capture_output=True, text=True)
    assert res.returncode == 0, res.stdout[-2000:] + res.stderr[-2000:]
    return harness.launches(str(where))


def modified_unit(tmp_path, unit, old, new):
    """The unit's assembly with one piece of text of gfx950_asm.hpp changed (a copy of the sources; the library's stay as they are)."""
    os.makedirs(tmp_path, exist_ok=True)
    src = tmp_path / "csrc"
    shutil.copytree(harness.CSRC, src)
    text = (src / "gfx950_asm.hpp").read_text()
    assert old in text
    (src / "gfx950_asm.hpp").write_text(text.replace(old, new))
    return gfx950.parse_program(open(harness.compile_unit(unit, csrc=str(src), out_dir=str(tmp_path / "isa"))).read())


def test_the_fault_of_the_masked_load_is_found_without_the_fix_and_gone_with_it(exe, isa, tmp_path):
    """The short-reduction kernel on a one-step reduction with several tiles per workgroup — the launch that faulted on the GPU.  Built
    without "scc" in the clobber list of the masked direct load, the interpreted code computes a load address 4 GiB above its operand
    in the loop over further tiles (s_and_b64 inside the block sets SCC, the s_addc_u32 the compiler scheduled behind the block adds
    it into the high half); built as the library has it, every access is in bounds and the result is the replay's."""
    launch = record(exe, "260,132,12,n,t,0,0,0,gemm_smallk=3", 1, tmp_path / "dump")[0]
    assert "gemm_smallk_kernel" in launch["symbol"]
    emu, wrong = harness.run_launch(launch)
    assert not wrong and emu.opcode_counts["global_load_lds_dwordx4"] > 0
    unfixed = modified_unit(tmp_path, "gemm_smallk", ': "memory", "vcc", "scc");', ': "memory", "vcc");')
    with pytest.raises(gfx950.EmulationError) as e:
        harness.run_launch(launch, program=unfixed)
    assert "direct load to LDS" in str(e.value) and "lies outside every buffer" in str(e.value)
    operands = [(base, len(data)) for base, data in launch["before"]]
    address = int(str(e.value).split(" at 0x")[1].split()[0], 16)
    assert any(base <= address - (1 << 32) < base + size for base, size in operands), "the access is exactly 4 GiB above an operand"


def test_wait_states_owed_by_the_asm_blocks_are_checked(exe, isa, tmp_path):
    """The interpreter counts wait states.  Without the s_nop of the direct-load block, M0 is written in the instruction before the
    load that reads it (the chip needs one wait state); with `s_nop 0` in its place that is satisfied, but the load's scalar base,
    which the compiler takes out of a v_readfirstlane right before the block, is then read 3 wait states after a vector instruction
    wrote it where the chip needs 5 — the hazard the block's `s_nop 3` is there for."""
    launch = record(exe, "70,130,48,n,n,0,0,0,gemm_tile=2", 2, tmp_path / "dump")[0]
    block = "s_mov_b32 m0, %0\\n\\ts_nop 3\\n\\tglobal_load_lds_dwordx4"
    bare = modified_unit(tmp_path / "bare", "gemm_64x64_0", block, block.replace("\\ts_nop 3\\n", ""))
    with pytest.raises(gfx950.EmulationError, match="wait states after M0 was written"):
        harness.run_launch(launch, program=bare)
    short = modified_unit(tmp_path / "short", "gemm_64x64_0", block, block.replace("s_nop 3", "s_nop 0"))
    with pytest.raises(gfx950.EmulationError, match="3 wait states after a vector instruction wrote it"):
        harness.run_launch(launch, program=short)


def test_a_wait_that_is_too_lenient_gives_wrong_numbers(exe, isa, tmp_path):
    """Loads return late in the interpreter: with every vmcnt wait of the kernel relaxed to 63 the tiles in LDS are stale and the
    product is wrong — which is what makes a passing run evidence for the waits the kernels and the compiler placed."""
    launch = record(exe, "70,130,48,n,n,0,0,0,gemm_tile=2", 2, tmp_path / "dump")[0]
    program = gfx950.parse_program(open(isa["gemm_64x64_0"]).read())
    assert not harness.run_launch(launch, program=program)[1]
    for ins in program[launch["symbol"]].instructions:
        if ins.op == "s_waitcnt" and ins.mods["vm"] is not None:
            ins.mods["vm"] = 63
    assert harness.run_launch(launch, program=program)[1]


# (CUs, case): every kernel family of the library, through the entry points, at sizes the interpreter finishes in seconds
CASES = [
    # the five tiles of the ordinary kernel: operand layouts (n row-major, t transposed view, g every second element), K tails, batches, accumulate
    (2, "70,130,40,n,n,0,0,0"), (2, "70,132,40,t,n,0,0,0,gemm_tile=2"), (2, "70,130,40,n,t,0,0,1,gemm_tile=2"), (2, "72,130,40,t,t,0,0,0,gemm_tile=2"),
    (2, "70,130,40,g,g,0,0,0,gemm_tile=2"), (2, "130,260,48,n,n,0,0,0,gemm_tile=1"), (2, "128,128,40,n,n,0,0,0,gemm_tile=1"), (2, "260,132,36,t,n,0,0,0,gemm_tile=0"),
    (2, "130,68,36,n,t,2,0,0,gemm_tile=3"), (2, "68,130,36,n,n,3,1,0,gemm_tile=4"), (2, "64,64,8,n,n,0,0,0,gemm_tile=2"),
    # K slices + their reduction, stream-K + fix-up
    (2, "70,130,200,n,n,0,0,0,gemm_tile=2,gemm_splitk=3"), (4, "300,260,64,n,n,0,0,0,gemm_tile=1,gemm_streamk=1"),
    # the persistent kernels: short reduction (several steps, K tails; one step), K-stream (both tiles), resident A (both tiles)
    (1, "260,132,40,n,t,0,0,0,gemm_smallk=1"), (1, "132,260,20,t,n,2,0,1,gemm_smallk=1"), (2, "132,68,56,t,t,0,0,0,gemm_smallk=1"),
    (1, "130,260,16,n,t,0,0,0,gemm_smallk=3"), (1, "300,520,8,t,n,2,0,0,gemm_smallk=3"), (1, "132,68,4,t,t,0,0,1,gemm_smallk=3"),
    (2, "300,260,100,n,n,0,0,0,gemm_panel=1"), (2, "132,260,36,t,n,2,1,1,gemm_panel=1"), (2, "132,260,100,n,t,0,0,0,gemm_panel=3"),
    (16, "128,2052,32,n,n,0,0,0,gemm_resident=1,ran=gemm_resident_kernel"), (16, "36,1000,112,t,n,0,0,0,gemm_resident=2,ran=gemm_resident_kernel"),
    # Matmul backward: plain, broadcast parents through the batch-reducing launch (vector and element-wise loaders)
    (2, "bwd:64,48,32,n,n,3,1"), (2, "bwd:70,41,33,n,n,0,5,fold_reduce=0"), (2, "bwd:64,64,32,n,n,0,4,fold_reduce=0"), (4, "bwd:70,41,33,n,n,0,5,fold_reduce=1"), (4, "bwd:66,130,20,t,n,3,1,fold_reduce=1"), (4, "bwd:40,36,24,g,g,1,4,fold_reduce=1"),
    # Linear backward with the bias gradient in the weight-gradient launch: whole K, K slices, stream-K
    (2, "lin:300,130,70,n,n,0,0,fused=1,gemm_tile=1"), (2, "lin:300,130,70,n,n,0,0,fused=1,gemm_tile=0"),
    (4, "lin:1000,260,200,n,n,0,0,fused=1,gemm_tile=1,gemm_streamk=1"), (2, "lin:1000,200,260,n,n,0,0,fused=1,gemm_tile=2,gemm_splitk=3"),
    # matrix-vector, vector-matrix (slices joined in the launch and by a launch of their own), skinny products, dot / column sum / SGD
    (2, "mv:515,1030,n,0,1,0"), (2, "mv:70,300,t,3,0,1"), (2, "vm:1030,515,n,0,1,0,join=1"), (2, "vm:300,4099,n,3,0,1"), (2, "vm:300,515,n,-3,0,0"),
    (2, "4,2052,768,n,n,0,0,0"), (2, "3,2051,300,t,n,0,0,1"), (2, "misc:1000"), (2, "misc:4096"),
    (2, "2,2052,300,n,n,0,0,0"), (2, "2,2052,300,n,n,0,0,0,cols_join=1"), (2, "2,2051,300,n,n,0,0,0"), (2, "3,2052,300,n,n,0,0,0,cols_join=1"),
    (2, "5,2052,300,n,n,0,0,0"), (2, "5,2052,300,n,n,0,0,0,cols_join=1"), (2, "5,2051,300,n,n,0,0,0"), (2, "mv:3,5000,n,0,0,0"),
    # mv / vm through the view-level entries with their gradients: stacked, shared and element-wise (every second element) matrices
    (2, "vbw:70,33,3,0,0"), (2, "vbw:40,36,0,4,1"), (2, "vbw:64,128,2,2,0"),
    # the adjacent operators and the MLP step op by op and in three launches
    (2, "ce:33,1000,0,0"), (2, "ce:5,50257,1,10"), (2, "ce:64,10,0,0"), (2, "ce:37,9001,0,5"), (2, "ce:9,64,1,10"), (2, "ce:9,2048,0,0"), (2, "ce:9,4096,1,10"), (2, "ce:3,16384,0,0"),
    (2, "ce:9,1999,1,0"), (2, "ce:9,2047,1,0"), (2, "ce:9,4095,0,0"), (2, "ce:5,8191,1,0"), (2, "ce:3,16383,1,0"), (2, "ce:3,32767,0,0"), (2, "ce:3,32767,1,0"),
    (2, "ce:9,1000,0,0,1"), (2, "ce:9,1000,1,10,2"), (2, "ce:9,1001,0,0,3"), (2, "ce:3,70001,1,0,3"),   # arrays that are not 16-byte aligned (2, "conv:2,3,12,11,8,3,3,1,1"), (2, "conv:2,4,15,14,6,3,2,2,1"),
    (2, "mlp:64,784,128,32,10,0"), (2, "mlp:37,257,77,33,7,3"), (2, "mlp:300,40,24,16,10,0"),
]


def sweep_of_instantiations():
    """One case for every instantiation of the matrix-product kernels: the compiler allocates registers and schedules each of them
    on its own (the masked-load fault lived in some instantiations of one kernel and not in others), so each one is run."""
    a_layout = {0: "n", 1: "t", 2: "g"}   # operand mode of A (K-major rows, MN-major = transposed view, element-wise) -> layout of the case
    b_layout = {0: "t", 1: "n", 2: "g"}
    cases = []
    dims = {0: (260, 132, 40), 1: (132, 132, 40), 2: (68, 132, 24), 3: (132, 68, 24), 4: (68, 132, 24)}
    whole = {0: (512, 128), 1: (256, 128), 2: (128, 64), 3: (256, 64), 4: (128, 128)}
    for tile in range(5):                 # the ordinary kernel: every tile x every pair of operand modes
        for am in range(3):
            for bm in range(3):
                M, N, K = dims[tile]
                cases.append((2, f"{M},{N},{K},{a_layout[am]},{b_layout[bm]},0,0,{(am + bm) % 2},gemm_tile={tile}"))
                cases.append((2, f"{whole[tile][0]},{whole[tile][1]},32,{a_layout[am]},{b_layout[bm]},0,0,0,gemm_tile={tile}"))   # whole tiles, whole K steps
    for tile in range(4):                 # stream-K with a fix-up: every tile x the vector modes
        for am in range(2):
            for bm in range(2):
                M, N = {0: (700, 128), 1: (380, 128), 2: (190, 64), 3: (380, 64)}[tile]
                cases.append((2, f"{M},{N},80,{a_layout[am]},{b_layout[bm]},0,0,0,gemm_tile={tile},gemm_streamk=1"))
    for am in range(2):                   # short reduction: modes x K steps (1 .. 4, each with a K tail) x accumulate
        for bm in range(2):
            for steps, K in ((1, 12), (2, 20), (3, 48), (4, 56)):
                for acc in (0, 1):
                    cases.append((1, f"132,196,{K},{a_layout[am]},{b_layout[bm]},0,0,{acc},gemm_smallk={3 if steps == 1 else 1}"))
                    cases.append((1, f"128,192,{16 * steps},{a_layout[am]},{b_layout[bm]},0,0,{acc},gemm_smallk={3 if steps == 1 else 1}"))
    for am in range(2):                   # K-stream: modes x tile x accumulate
        for bm in range(2):
            for knob in (1, 3):
                for acc in (0, 1):
                    cases.append((2, f"132,260,36,{a_layout[am]},{b_layout[bm]},0,0,{acc},gemm_panel={knob}"))
                    cases.append((2, f"256,256,48,{a_layout[am]},{b_layout[bm]},0,0,{acc},gemm_panel={knob}"))
    for am in range(2):                   # resident A: mode of A x tile height x K range
        for knob in (1, 2):
            for K in (36, 132):
                cases.append((16, f"128,1028,{K},{a_layout[am]},n,0,0,0,gemm_resident={knob},ran=gemm_resident_kernel"))
    for la in "ntg":                      # the batch-reducing launch: layouts x which parent is shared x tile
        for lb in "ntg":
            cases.append((4, f"bwd:40,36,24,{la},{lb},1,4,fold_reduce=1"))
            cases.append((4, f"bwd:40,36,24,{la},{lb},4,1,fold_reduce=1,skip=1"))
    for la in "nt":
        for lb in "nt":
            cases.append((1, f"bwd:132,132,24,{la},{lb},1,3,fold_reduce=1"))
            cases.append((1, f"bwd:132,132,24,{la},{lb},3,1,fold_reduce=1,skip=1"))
    for tile in range(5):                 # the bias gradient in the weight-gradient launch: every tile
        cases.append((2, f"lin:300,132,68,n,n,0,0,fused=1,gemm_tile={tile}"))
    return cases


@pytest.mark.parametrize("reverse", [False, True], ids=["ascending", "descending"])
def test_every_kernel_family_on_the_generated_code(exe, isa, tmp_path, reverse):
    """Registers, LDS and scratch start as garbage (NaN as floats, far out of bounds as addresses); the workgroups of a grid and the
    wavefronts of a workgroup take their turns in ascending order and, second run, in descending order — the results are the same.
    The ascending run adds the sweep over every instantiation of the matrix-product kernels; the descending run moves every buffer so
    that a multiple of 4 GiB falls into its middle (harness.across_4gib), where every 64-bit address computation has to carry."""
    cases = CASES + ([] if reverse else sweep_of_instantiations())
    jobs = [(n, cus, case, str(tmp_path), exe, reverse, reverse) for n, (cus, case) in enumerate(cases)]   # (the descending run also relocates)
    failures, kernels, instructions = [], set(), 0
    with ProcessPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
        for case, launches in pool.map(harness.replay_and_emulate, jobs):
            for symbol, count, verdict in launches:
                kernels.add(symbol)
                instructions += count
                if verdict != "ok":
                    failures.append(f"{case}: {symbol}: {verdict}")
    assert not failures, "\n".join(failures)
    assert len(kernels) >= 70 and instructions > 5_000_000, (len(kernels), instructions)
    if not reverse:   # every instantiation of the matrix-product units has run (the rest live in tenmo_hip.hip: no assembly blocks there)
        units = harness.device_units()[1]
        not_run = [name for unit in units if unit != "tenmo_hip" for name in harness.program_of(unit) if name not in kernels]
        # (instantiated but out of reach of Matmul backward: the left operand of a folded dA and the right one of a folded dB are the dense
        # upstream gradient, so the batch-reducing launch never sees an MN-major or element-wise left operand beside a K-major or
        # element-wise right one)
        unreachable = re.compile(r"gemm_reduce_kernelILi\d+ELi\d+ELi[12]ELi[02]E")
        assert not [name for name in not_run if not unreachable.search(name)], not_run
        assert len(not_run) <= 5
        assert len(kernels) >= 170


@pytest.mark.skipif(os.environ.get("TENMO_REPLAY_FULL") != "1", reason="ten minutes of CPU time: set TENMO_REPLAY_FULL=1")
def test_the_default_dispatch_at_medium_sizes(exe, isa, tmp_path):
    """What the library picks by itself on 8 to 16 modelled CUs, at sizes where the persistent kernels walk many tiles: a 1024 x 1024 x 256
    product, attention-shaped batches, both CBOW shapes at a tenth of the vocabulary, Linear backward with the fused bias gradient, the
    broadcast-batched backward, the skinny product at its real width, mv and vm at 4096 squared."""
    cases = [(16, "1024,1024,256,n,n,0,0,0"), (16, "512,512,64,n,t,4,0,0"), (16, "256,5000,100,n,n,0,0,0"), (16, "100,5000,256,t,n,0,0,0"),
             (16, "lin:2048,768,256,n,n,0,0,fused=1"), (16, "bwd:512,768,768,n,n,4,1"), (8, "4,50257,768,n,n,0,0,0"), (8, "mv:4096,4096,n,0,0,0"),
             (8, "vm:4096,4096,n,0,0,0")]
    failures = []
    with ProcessPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
        for case, launches in pool.map(harness.replay_and_emulate, [(n, cus, case, str(tmp_path), exe) for n, (cus, case) in enumerate(cases)]):
            failures += [f"{case}: {symbol}: {verdict}" for symbol, _count, verdict in launches if verdict != "ok"]
    assert not failures, "\n".join(failures)
