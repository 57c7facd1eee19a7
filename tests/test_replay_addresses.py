"""Every GEMM kernel of the library, run on the CPU under AddressSanitizer before it ever meets a GPU.

tests/replay/ holds a CPU stand-in for the HIP runtime against which the kernel sources of tenmo_amd/csrc compile
unchanged (only the three gfx950 assembly snippets of gfx950_asm.hpp are swapped for models): a launch runs every
workgroup, every thread a fibre, wavefront-wide operations and barriers where the source has them.  Here the whole
library plus a small driver (tests/replay/replay_gemm_main.cpp) is built with -fsanitize=address and
tenmo_hip_gemm_f32 is called on operands that are heap blocks of exactly the operands' sizes: a load or store of any
kernel one byte outside an operand ends the run with the sanitizer's report, a workgroup whose wavefronts disagree
about their barriers ends it as a deadlock, and the result is compared with a float64 product.  Each group runs in both
models of the direct global->LDS loads: landing at issue ("early": a ring stage refilled too soon shows) and landing at
the s_waitcnt that covers them ("late": a wait that is too lenient shows).  No GPU involved.
"""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests", "replay"))
import build as replay_build  # noqa: E402

pytestmark = pytest.mark.skipif(not replay_build.available(), reason="no host clang++ at " + replay_build.CXX)

LAYOUTS = [("n", "n"), ("n", "t"), ("t", "n"), ("t", "t")]


@pytest.fixture(scope="module")
def exe():
    return replay_build.build_gemm_asan()


def case(M, N, K, la="n", lb="n", batch=0, b_shared=0, acc=0, **knobs):
    return ",".join([str(M), str(N), str(K), la, lb, str(batch), str(b_shared), str(acc)] + [f"{k}={v}" for k, v in knobs.items()])


def run(exe, cases, cus=256, modes=("early", "late"), timeout=600):
    env = dict(os.environ, REPLAY_CUS=str(cus), ASAN_OPTIONS="detect_leaks=0:detect_stack_use_after_return=0")
    # the cases are independent: both load models side by side, each over two halves of the list
    halves = [cases[:(len(cases) + 1) // 2], cases[(len(cases) + 1) // 2:]] if len(cases) > 3 else [cases]
    jobs = [(mode, part, subprocess.Popen([exe, mode] + part, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, env=env))
            for mode in modes for part in halves if part]
    failures = []
    for mode, part, proc in jobs:
        try:
            out, err = proc.communicate(timeout=timeout)
        except subprocess.TimeoutExpired:
            proc.kill()
            out, err = proc.communicate()
            failures.append(f"mode {mode}, {cus} CUs: no end after {timeout} s\n" + (out[-3000:] + "\n" + err[-3000:]).strip())
            continue
        tail = (out[-3000:] + "\n" + err[-6000:]).strip()
        if proc.returncode != 0:
            failures.append(f"mode {mode}, {cus} CUs:\n{tail}")
        elif out.count("relative error") != len(part):
            failures.append(tail)
    assert not failures, "\n\n".join(failures)


def test_the_checks_bite():
    """tests/replay/replay_selftest.cpp: toy kernels that are wrong on purpose, each in one way, and what becomes of them."""
    exe = replay_build.build_selftest()
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:detect_stack_use_after_return=0")
    outcome = {}
    for what in ("ok", "overread", "overwrite", "direct_overread", "divergent_collective", "lenient_wait"):
        res = subprocess.run([exe, what], capture_output=True, text=True, env=env, timeout=120)
        outcome[what] = (res.returncode, res.stdout + res.stderr)
    assert outcome["ok"][0] == 0 and "ok" in outcome["ok"][1]
    for what in ("overread", "overwrite"):   # a plain load / store one element past a device allocation
        assert outcome[what][0] != 0 and "heap-buffer-overflow" in outcome[what][1], outcome[what][1][-2000:]
    assert outcome["direct_overread"][0] != 0 and "lies outside every device allocation" in outcome["direct_overread"][1]
    assert outcome["divergent_collective"][0] != 0 and "deadlock" in outcome["divergent_collective"][1]
    assert outcome["lenient_wait"][0] == 3 and "stale data" in outcome["lenient_wait"][1]   # a wait that leaves a needed load in flight


@pytest.mark.parametrize("tile", [0, 1, 2, 3, 4])
def test_one_workgroup_per_tile_kernels(exe, tile):
    """gemm_mfma_kernel of every workgroup tile: whole and ragged tiles, K of one step, K tails (the register-staged loop
    behind the direct ring), every layout, batches with a shared B, accumulate, and both strides non-unit (the
    element-wise loader)."""
    cases = []
    for la, lb in LAYOUTS:
        for (M, N, K) in [(64, 64, 16), (130, 70, 33), (257, 129, 100), (300, 520, 48), (128, 256, 7)]:
            cases.append(case(M, N, K, la, lb, gemm_tile=tile))
        cases.append(case(132, 260, 84, la, lb, batch=3, b_shared=1, acc=1, gemm_tile=tile))
        cases.append(case(131, 77, 50, la, lb, batch=2, acc=0, gemm_tile=tile))  # extents that are no multiple of 4: an MN-major ragged tile leaves the direct path
    cases += [case(100, 90, 40, "g", "n", gemm_tile=tile), case(100, 90, 40, "n", "g", gemm_tile=tile), case(65, 130, 24, "g", "g", batch=2, acc=1, gemm_tile=tile)]
    run(exe, cases)


def test_k_slices_and_stream_k(exe):
    cases = []
    for la, lb in LAYOUTS:
        cases.append(case(200, 100, 400, la, lb, gemm_splitk=3))
        cases.append(case(130, 70, 1000, la, lb, batch=2, acc=1, gemm_splitk=8))
        for tile in (0, 1, 2, 3):
            cases.append(case(520, 300, 256, la, lb, gemm_streamk=1, gemm_tile=tile))
            cases.append(case(260, 392, 132, la, lb, batch=3, acc=1, gemm_streamk=2, gemm_tile=tile))
    run(exe, cases, cus=4)   # few CUs: every workgroup of a stream-K grid takes whole tiles and a shared piece
    run(exe, [case(1024, 768, 512), case(1000, 1000, 300, "n", "t")], cus=16, modes=("late",))  # what the automatic choice picks


def test_short_reduction_kernel(exe):
    """gemm_smallk_kernel forced on: K of 17..64 (K <= 16 goes to the ordinary kernel), every layout, K tails, ragged tiles,
    batches, a shared B, accumulate; on 2 CUs every workgroup walks many tiles, on 256 most tiles have a workgroup each."""
    cases = []
    for la, lb in LAYOUTS:
        for (M, N, K) in [(128, 192, 64), (100, 132, 36), (1000, 1000, 48), (64, 64, 20), (332, 776, 32)]:
            cases.append(case(M, N, K, la, lb, gemm_smallk=1))
        cases.append(case(256, 68, 64, la, lb, batch=6, acc=1, gemm_smallk=1))
        cases.append(case(320, 192, 32, la, lb, batch=9, b_shared=1, gemm_smallk=1))
    cases.append(case(257, 65, 64, "n", "t", batch=6, acc=1, gemm_smallk=1))   # a K-major operand may have any row count
    cases.append(case(8, 8192, 64, "n", "n", gemm_smallk=1))                  # few tile-rows, many tile-columns: column blocks per XCD
    run(exe, cases, cus=2)
    run(exe, cases[:8] + cases[-3:], cus=256, modes=("late",))
    run(exe, [case(64, 64, 16, gemm_smallk=1), case(300, 200, 12, "n", "t", gemm_smallk=1)], cus=4)  # K <= 16: not this kernel, still right


def test_k_stream_kernel(exe):
    """gemm_panel_kernel forced on: reductions of two steps to many, K tails, every layout, ragged tiles, batches, a shared
    B, accumulate (atomic adds); few CUs (long walks, the ring runs across many tile boundaries) and the real 256."""
    cases = []
    for la, lb in LAYOUTS:
        for (M, N, K) in [(128, 128, 32), (300, 520, 100), (132, 260, 20), (1000, 136, 24), (256, 384, 112), (128, 256, 36), (512, 512, 256)]:
            cases.append(case(M, N, K, la, lb, gemm_panel=1))
        cases.append(case(256, 384, 64, la, lb, batch=16, gemm_panel=1))
        cases.append(case(132, 260, 48, la, lb, batch=9, b_shared=1, acc=1, gemm_panel=1))
    cases.append(case(129, 131, 48, "n", "t", gemm_panel=1))
    cases.append(case(256, 128 * 70, 32, "n", "n", gemm_panel=1))
    run(exe, cases, cus=2)
    run(exe, cases[:9] + cases[-2:], cus=256, modes=("late",))
    run(exe, [case(128, 128, 16, gemm_panel=1), case(300, 260, 8, "t", "n", gemm_panel=1)], cus=4)  # K <= 16: not this kernel, still right
    # the 64x64-tile variant (a ring of eight stages, two operand fetches behind an MFMA for MN-major operands)
    small = []
    for la, lb in LAYOUTS:
        for (M, N, K) in [(64, 64, 32), (300, 520, 100), (132, 260, 20), (256, 384, 112), (512, 512, 256), (1024, 64, 1024)]:
            small.append(case(M, N, K, la, lb, gemm_panel=3))
        small.append(case(256, 384, 64, la, lb, batch=16, gemm_panel=3))
        small.append(case(132, 260, 48, la, lb, batch=9, b_shared=1, acc=1, gemm_panel=3))
    run(exe, small, cus=2)
    run(exe, small[:8] + [case(1024, 1024, 1024, gemm_panel=3)], cus=256, modes=("late",))


def test_resident_left_operand_kernel(exe):
    """gemm_resident_kernel forced on (both tile heights): a few tile rows of A held in LDS for all of K against a wide B
    with unit stride along N — K of two steps up to 256 and K tails, a row-major and a transposed-view A, ragged last tile
    rows and column blocks, more tile rows than one, walks of many column blocks per workgroup (few CUs) and the real 256;
    `ran=` makes the driver check that this kernel, not another one, served the case.  What it does not take (a transposed
    B, batches, accumulate, K beyond 256, a K-major A with K % 4 != 0) falls through to the other kernels and is still right."""
    cases = []
    for knob in (1, 2):
        for la in ("n", "t"):
            for (M, N, K) in [(256, 3200, 100), (100, 3204, 256), (128, 2052, 32), (64, 4096, 20), (36, 3000, 112), (200, 2500, 132), (256, 2048, 250 if la == "t" else 248)]:
                cases.append(case(M, N, K, la, "n", gemm_resident=knob, ran="gemm_resident_kernel"))
    run(exe, cases, cus=16)
    # the chip's real width: 32 or 64 workgroups per XCD, up to 32 tile rows, column blocks left over at the end of the walks
    wide = [case(256, 50000, 100, "n", "n", gemm_resident=1, ran="gemm_resident_kernel"), case(100, 50000, 256, "t", "n", gemm_resident=2, ran="gemm_resident_kernel"),
            case(1024, 6400, 48, "n", "n", gemm_resident=1, ran="gemm_resident_kernel"), case(2048, 3300, 36, "t", "n", gemm_resident=2, ran="gemm_resident_kernel")]
    run(exe, wide, cus=256, modes=("late",))
    others = [case(256, 3200, 100, "n", "t", gemm_resident=1), case(256, 3200, 100, "n", "n", batch=2, gemm_resident=1), case(256, 3200, 100, "n", "n", acc=1, gemm_resident=1),
              case(128, 3200, 272, "n", "n", gemm_resident=1), case(128, 3200, 250, "n", "n", gemm_resident=2), case(128, 3202, 64, "n", "n", gemm_resident=1),
              case(256, 128, 100, "n", "n", gemm_resident=1)]
    run(exe, others, cus=16, modes=("early",))


def test_automatic_choice_on_benchmark_shapes(exe):
    """What the dispatch picks by itself for the shapes the benchmarks run, at their real sizes (attention: 8 of the 96
    batches; the square products reduced to 1024)."""
    cases = [case(1024, 1024, 64, "n", "t", batch=8),        # Q.K^T: the short-reduction kernel
             case(1024, 64, 1024, "n", "n", batch=8),        # P.V
             case(1024, 1024, 128, "n", "t", batch=8),       # K = 128, many tiles: the K-stream kernel
             case(256, 50000, 100, "n", "n"),                # CBOW logits
             case(100, 50000, 256, "t", "n"),                # CBOW A^T.dC
             case(8, 4096, 1024, "n", "n"),                  # skinny: the column-streaming kernels
             case(1024, 1024, 1024)]
    run(exe, cases, modes=("late",), timeout=1200)


def test_gradients_of_broadcast_parents(exe):
    """tenmo_hip_matmul_backward with a parent that was broadcast over the batch: the sum over batches inside the GEMM
    launch (gemm_reduce_kernel, forced on), and the batched gradient reduced afterwards (forced off)."""
    cases = []
    for la, lb in LAYOUTS:
        for fold in (1, 0):
            cases.append(f"bwd:70,41,33,{la},{lb},0,5,fold_reduce={fold}")     # A shared by 5 batches
            cases.append(f"bwd:132,260,48,{la},{lb},4,1,fold_reduce={fold}")   # B shared (its partner's rows stack: one folded GEMM either way)
            cases.append(f"bwd:300,200,100,{la},{lb},1,3,fold_reduce={fold}")
    run(exe, cases, cus=8)
    run(exe, ["bwd:256,1024,512,n,n,0,4,fold_reduce=1", "bwd:512,256,1024,n,n,1,6"], cus=256, modes=("late",))
    # an operand without a unit stride under a broadcast: the reducing launch with the element-wise loader
    generic = []
    for la, lb in (("g", "n"), ("n", "g"), ("g", "g"), ("g", "t"), ("t", "g")):
        generic += [f"bwd:70,41,33,{la},{lb},0,5,fold_reduce=1", f"bwd:132,260,48,{la},{lb},3,1,fold_reduce=1", f"bwd:100,68,20,{la},{lb},1,4,fold_reduce=0"]
    run(exe, generic, cus=8)


def test_linear_backward_with_the_bias_gradient_in_the_weight_gradient_launch(exe):
    """tenmo_hip_linear_backward: the B fragments of the weight-gradient product X^T . dY added up beside the MFMAs
    (gemm_mfma_bsum_kernel, gemm_streamk_bsum_kernel): every tile, K slices (their sums added by the slice reduction),
    stream-K (whole tiles onto the result, pieces through the fix-up), whole and ragged tiles, a batched input folded into
    the reduction; `fused=1` makes the driver check that the call takes no launch more than without the bias gradient.
    What the fused sum does not take — a transposed-view input, a batch whose rows do not stack — streams dY once more
    (`fused=0`) and is still right."""
    cases = []
    for tile in (0, 1, 2, 3, 4):
        cases.append(f"lin:300,130,70,n,n,0,0,fused=1,gemm_tile={tile}")
        cases.append(f"lin:64,256,128,n,n,3,0,fused=1,gemm_tile={tile}")
    for tile, sk in ((0, 2), (1, 1), (1, 2), (2, 1), (3, 2)):
        cases.append(f"lin:1000,260,200,n,n,0,0,fused=1,gemm_tile={tile},gemm_streamk={sk}")
        cases.append(f"lin:2100,132,68,n,n,0,0,fused=1,gemm_tile={tile},gemm_streamk={sk}")
    for tile, splits in ((0, 3), (1, 4), (2, 2), (3, 8), (4, 5)):
        cases.append(f"lin:1000,200,260,n,n,0,0,fused=1,gemm_tile={tile},gemm_splitk={splits}")
    cases += ["lin:515,100,36,n,n,0,0,fused=1", "lin:40,12,4,n,n,0,0", "lin:300,130,70,t,n,0,0,fused=0", "lin:1,70,33,n,n,0,0,fused=1"]
    run(exe, cases, cus=8)
    run(exe, ["lin:2048,768,256,n,n,0,0,fused=1", "lin:512,768,768,n,n,4,0,fused=1"], cus=256, modes=("late",), timeout=1200)


def test_matrix_vector_kernels(exe):
    """mv and vm (tenmo_amd/csrc/gemv.hpp: the row kernel, the column kernels with aligned, shifted and element loads, their K
    slices and the slice reduction, the allocation-free entry) on matrices that END with their last element: row pitches that
    are and are not multiples of four floats, row counts and widths around the kernels' vector and unroll widths, batches, a
    matrix shared by the batches, accumulate."""
    cases = []
    for m, k in [(1, 1), (7, 5), (64, 1024), (515, 1030), (130, 4097), (1000, 33), (33, 6000)]:
        for layout in ("n", "t"):
            for pad in (0, 1, 4):
                cases.append(f"mv:{m},{k},{layout},0,{pad},0")
    cases += ["mv:70,300,n,3,0,1", "mv:70,300,t,3,2,1", "mv:65,257,n,-4,0,0", "mv:2048,768,n,0,0,0"]
    for k, n in [(1, 1), (5, 7), (1024, 64), (1030, 515), (300, 4099), (33, 1000), (2000, 50257 // 8)]:
        for layout in ("n", "t"):
            for pad in (0, 1, 4):
                cases.append(f"vm:{k},{n},{layout},0,{pad},0")
    cases += ["vm:300,70,n,3,0,1", "vm:300,1027,n,3,1,1", "vm:257,65,t,-4,0,0", "vm:4096,1500,n,0,0,1,entry=noalloc", "vm:700,260,n,2,0,1,entry=noalloc",
              "vm:768,4096,n,0,0,0", "vm:100,50000,n,0,0,0"]
    # the K slices added by the last workgroup of the streaming launch (join=1: the driver also requires the bits of the
    # two-launch result and one launch less), on few and on many modelled CUs (other slice counts)
    joined = ["vm:1024,64,n,0,0,0,join=1", "vm:1030,515,n,0,1,0,join=1", "vm:1030,515,n,0,0,1,join=1", "vm:300,4099,n,0,0,0,join=1",
              "vm:2000,6282,n,0,0,1,join=1", "vm:2000,6282,n,3,1,0,join=1", "vm:257,65,n,-4,0,0,join=1", "mv:515,1030,t,0,1,0,join=1",
              "mv:64,1024,t,2,0,1,join=1", "vm:4096,1500,n,0,0,1,entry=noalloc,join=1", "vm:100,50000,n,0,0,0,join=1", "vm:5000,9,n,0,0,0,join=1",
              "4,6282,768,n,n,0,0,1,cols_join=1", "8,1000,300,n,n,3,0,0,cols_join=1", "2,4099,515,n,n,0,0,0,cols_join=1"]
    run(exe, cases + joined, cus=16, modes=("early",))
    run(exe, cases[::5] + joined, cus=256, modes=("early",))


def test_adjacent_operators(exe):
    """Cross-entropy (forward with and without the softmax written, backward mean / sum), the convolution (forward and the
    three gradients: gathered operands, dilated and strided phases), dot, SGD and the column sum on exactly-sized operands:
    addresses only (their numbers are the parity tests' business)."""
    cases = ["ce:1,1,0,0", "ce:7,10,0,0", "ce:64,10,1,10", "ce:33,1000,0,0", "ce:5,50257,1,10", "ce:300,4099,0,0", "ce:2,100003,0,5",
             "conv:1,1,5,5,1,3,3,1,1", "conv:2,3,12,11,8,3,3,1,1", "conv:2,4,15,14,6,3,2,2,1", "conv:1,5,17,17,7,3,3,1,2", "conv:3,16,10,10,32,3,3,1,1",
             "conv:2,3,9,9,4,1,1,1,1", "conv:1,8,20,20,16,5,5,3,1",
             "misc:1", "misc:63", "misc:1000", "misc:300001",
             # the MLP training step op by op and with its last two layers fused into one launch: the MNIST shape, the largest
             # widths the fused launch takes, ragged ones, and a batch of one
             "mlp:64,784,128,32,10,0", "mlp:64,784,128,32,10,1", "mlp:64,300,128,64,32,1", "mlp:37,50,77,33,7,1", "mlp:1,9,5,3,2,1",
             "mlp:64,784,128,32,10,2", "mlp:37,50,77,33,7,2", "mlp:1,9,5,3,2,2", "mlp:64,17,128,64,32,2", "mlp:5,33,1,1,1,2",
             # ... and the first layer's forward as one launch (inputs of 256 and more; K tails of every kind, ragged blocks)
             "mlp:64,784,128,32,10,3", "mlp:37,257,77,33,7,3", "mlp:1,1001,5,3,2,3", "mlp:64,300,128,64,32,3", "mlp:100,518,130,40,9,3"]
    run(exe, cases, cus=16, modes=("early",))


def test_randomized_products(exe):
    """Seeded random shapes (small extents, the tile widths and their neighbours, anything up to 400), layouts including
    generic strides, batches with and without a shared B, accumulate, and kernel choices (every tile, K slices, stream-K, the
    short-reduction and the K-stream kernel in its variants forced on): whatever the dispatch makes of them must stay in bounds and be right.
    (TENMO_REPLAY_FUZZ=<n> runs n cases instead of 150.)"""
    import random

    rnd = random.Random(20240611)

    def extent(limit):
        r = rnd.random()
        if r < 0.15:
            return rnd.choice([1, 2, 3, 4, 5, 7, 8])
        if r < 0.5:
            return rnd.choice([16, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 130, 132, 255, 256, 257, 260])
        return rnd.randint(1, limit)

    cases = []
    for _ in range(int(os.environ.get("TENMO_REPLAY_FUZZ", "150"))):
        batch = rnd.choice([0, 0, 0, 1, 2, 3, 5, 9])
        knobs = {}
        r = rnd.random()
        if r < 0.2:
            knobs["gemm_tile"] = rnd.randint(0, 4)
        elif r < 0.3:
            knobs["gemm_splitk"] = rnd.choice([2, 3, 5, 8])
        elif r < 0.45:
            knobs["gemm_streamk"], knobs["gemm_tile"] = rnd.choice([1, 2]), rnd.randint(0, 3)
        elif r < 0.6:
            knobs["gemm_smallk"] = 1
        elif r < 0.75:
            knobs["gemm_panel"] = rnd.choice([1, 1, 3, 4, 5])
        cases.append(case(extent(400), extent(400), extent(300), rnd.choice("nntg"), rnd.choice("nntg"), batch,
                          rnd.choice([0, 0, 1]) if batch else 0, rnd.choice([0, 0, 1]), **knobs))
    for start in range(0, len(cases), 75):
        run(exe, cases[start:start + 75], cus=3)


def test_one_step_reduction_into_a_large_result(exe):
    """[8192,16].[16,8192] with B a transposed view, at full size and on the real 256 CUs: the launch after which a GPU run
    once ended in a memory fault.  The source was right (this replay was clean for all three kernels that ran then); the
    cause was an undeclared SCC clobber in an inline-assembly block, which only the generated ISA shows
    (tests/test_asm_clobbers.py).  K <= 16 currently takes the ordinary 64x64 kernel, which is what this replays."""
    run(exe, [case(8192, 8192, 16, "n", "t")], modes=("early",), timeout=1200)


def test_short_reduction_kernel_on_one_step_reductions(exe):
    """K <= 16 through the persistent short-reduction kernel (gemm_smallk = 3; the automatic choice keeps such products on the
    ordinary kernel): one K step per tile, so a workgroup's loop is all tile turnover — several tiles per workgroup (few
    modelled CUs), ragged last tile rows and columns, K tails (the masked direct load on every tile), every operand layout,
    plain and accumulating stores, batches with and without a shared B; and the product that once faulted on a GPU,
    [8192,16].[16,8192] with B a transposed view, at full size on the real 256 CUs through this kernel."""
    cases = []
    for la, lb in LAYOUTS:
        for (M, N, K) in [(300, 520, 16), (260, 132, 12), (320, 448, 8), (132, 68, 4)]:
            for acc in (0, 1):
                cases.append(case(M, N, K, la, lb, acc=acc, gemm_smallk=3, ran="gemm_smallk_kernel"))
        cases.append(case(200, 264, 16, la, lb, batch=5, gemm_smallk=3, ran="gemm_smallk_kernel"))
        cases.append(case(200, 264, 12, la, lb, batch=3, b_shared=1, acc=1, gemm_smallk=3, ran="gemm_smallk_kernel"))
    run(exe, cases, cus=2)
    run(exe, [case(8192, 8192, 16, "n", "t", gemm_smallk=3, ran="gemm_smallk_kernel", check=0)], modes=("late",), timeout=1800)


@pytest.mark.skipif(os.environ.get("TENMO_REPLAY_FULL") != "1", reason="a quarter of an hour of CPU time: set TENMO_REPLAY_FULL=1")
def test_benchmark_shapes_at_full_size_under_the_default_dispatch(exe):
    """The benchmark's own shapes, whole, at 256 CUs, through whatever kernel the library picks by itself: two GPT-2 Linear products,
    the up-projection's Linear backward with the bias gradient in the weight-gradient launch, the attention Q.K^T backward (8 of its
    96 batches), the broadcast-batched backward A[32,512,768].B[1,768,768], both CBOW products and the skinny product."""
    cases = ["8192,2304,768,n,n,0,0,0", "8192,768,3072,n,n,0,0,0", "lin:8192,3072,768,n,n,0,0,fused=1", "bwd:1024,1024,64,n,t,8,8",
             "bwd:512,768,768,n,n,32,1", "256,50000,100,n,n,0,0,0", "100,50000,256,t,n,0,0,0", "4,50257,768,n,n,0,0,0"]
    run(exe, cases, cus=256, modes=("late",), timeout=3000)
