"""The interpreter of tests/isa/gfx950.py against hand-made instruction sequences: the semantics that generated code leans on most and
that are easiest to get wrong (carries through SCC and VCC, execution-mask bookkeeping with source and destination in one register pair,
32-bit LDS addresses, the lane layout of the matrix instruction, loads that return late, bounds)."""
import os
import struct
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "isa"))
import gfx950  # noqa: E402

OUT = 0x1000_0000


def run(body: str, lds=1024, late=True, data=None, threads=64):
    """A one-workgroup kernel made of `body`; s[0:1] holds the address of the (empty) argument block, s2 the workgroup id; memory: 4 KiB
    at OUT (zeros, or `data`).  Returns that buffer as uint32."""
    text = "k:\n" + "\n".join("\t" + line.strip() for line in body.strip().split("\n")) + "\n\ts_endpgm\n.Lfunc_end0:\n" \
        "\t.amdhsa_kernel k\n\t\t.amdhsa_group_segment_fixed_size %d\n\t\t.amdhsa_private_segment_fixed_size 0\n\t\t.amdhsa_kernarg_size 0\n" \
        "\t\t.amdhsa_user_sgpr_count 2\n\t\t.amdhsa_user_sgpr_kernarg_segment_ptr 1\n\t\t.amdhsa_system_sgpr_workgroup_id_x 1\n\t.end_amdhsa_kernel\n" % lds
    program = gfx950.parse_program(text)
    mem = gfx950.Memory()
    buf = np.zeros(4096, dtype=np.uint8) if data is None else np.asarray(data).view(np.uint8).copy()
    mem.map(OUT, buf)
    gfx950.Emulator(program, mem, late=late).launch("k", (1, 1, 1), (threads, 1, 1), b"")
    return buf.view(np.uint32)


STORE_V1 = """
    v_lshlrev_b32_e32 v10, 2, v0
    s_mov_b32 s10, 0x10000000
    s_mov_b32 s11, 0
    s_nop 4
    global_store_dword v10, v1, s[10:11]
"""


def test_scalar_carry_chain_and_its_flags():
    out = run("""
        s_mov_b32 s4, 0xfffffff0
        s_add_u32 s5, s4, 0x20
        s_addc_u32 s6, 7, 0
        s_sub_u32 s7, 5, 9
        s_subb_u32 s8, 10, 0
        v_mov_b32_e32 v1, s5
        v_mov_b32_e32 v2, s6
        v_mov_b32_e32 v3, s7
        v_mov_b32_e32 v4, s8
        v_cmp_eq_u32_e32 vcc, 1, v0
        v_cndmask_b32_e32 v1, v1, v2, vcc
        v_cmp_eq_u32_e32 vcc, 2, v0
        v_cndmask_b32_e32 v1, v1, v3, vcc
        v_cmp_eq_u32_e32 vcc, 3, v0
        v_cndmask_b32_e32 v1, v1, v4, vcc
    """ + STORE_V1)
    assert list(out[:4]) == [0x10, 8, 0xFFFFFFFC, 9]


def test_vector_borrow_with_the_destination_among_the_sources():
    """v_sub_co_u32 v8, vcc, v8, v11: the borrow is that of the operands, not of the result written over one of them."""
    out = run("""
        v_mov_b32_e32 v8, 0x100
        v_mov_b32_e32 v11, 0x100
        v_mov_b32_e32 v9, 0
        v_mov_b32_e32 v12, 0
        v_sub_co_u32_e32 v8, vcc, v8, v11
        v_subb_co_u32_e32 v9, vcc, v9, v12, vcc
        v_mov_b32_e32 v1, v9
    """ + STORE_V1)
    assert np.all(out[:64] == 0)
    out = run("""
        v_mov_b32_e32 v8, 5
        v_mov_b32_e32 v9, 0
        v_sub_co_u32_e32 v8, vcc, v8, v0
        v_subbrev_co_u32_e32 v1, vcc, 0, v9, vcc
    """ + STORE_V1)
    assert list(out[:8]) == [0, 0, 0, 0, 0, 0, 0xFFFFFFFF, 0xFFFFFFFF]


def test_saveexec_with_one_register_pair_as_source_and_destination():
    """The else branch of generated code: s_andn2_saveexec_b64 s[6:7], s[6:7] leaves the lanes of the mask that are not running."""
    out = run("""
        v_mov_b32_e32 v1, 0
        v_cmp_gt_u32_e32 vcc, 16, v0
        s_and_saveexec_b64 s[6:7], vcc
        s_xor_b64 s[6:7], exec, s[6:7]
        v_mov_b32_e32 v1, 1
        s_andn2_saveexec_b64 s[6:7], s[6:7]
        v_mov_b32_e32 v1, 2
        s_or_b64 exec, exec, s[6:7]
    """ + STORE_V1)
    assert list(out[:64]) == [1] * 16 + [2] * 48


def test_lds_addresses_wrap_at_32_bits_and_are_bounded():
    out = run("""
        v_lshlrev_b32_e32 v2, 2, v0
        ds_write_b32 v2, v0
        v_add_u32_e32 v3, -12, v2
        s_waitcnt lgkmcnt(0)
        ds_read2_b32 v[4:5], v3 offset0:3 offset1:4
        s_waitcnt lgkmcnt(0)
        v_mov_b32_e32 v1, v4
    """ + STORE_V1)
    assert list(out[:64]) == list(range(64))
    with pytest.raises(gfx950.EmulationError, match="LDS read"):
        run("v_mov_b32_e32 v2, 1024\nds_read_b32 v1, v2\ns_waitcnt lgkmcnt(0)")


def test_a_result_read_before_its_wait_is_stale():
    data = np.arange(1024, dtype=np.uint32) + 100
    body = """
        v_lshlrev_b32_e32 v10, 2, v0
        s_mov_b32 s10, 0x10000000
        s_mov_b32 s11, 0
        v_mov_b32_e32 v1, 7
        s_nop 4
        global_load_dword v1, v10, s[10:11] offset:256
        %s
        v_mov_b32_e32 v2, v1
        s_waitcnt vmcnt(0)
        global_store_dword v10, v2, s[10:11]
    """
    assert list(run(body % "s_waitcnt vmcnt(0)", data=data)[:4]) == [164, 165, 166, 167]
    assert list(run(body % "s_nop 0", data=data)[:4]) == [7, 7, 7, 7]
    assert list(run(body % "s_nop 0", data=data, late=False)[:4]) == [164, 165, 166, 167]


def test_global_access_outside_every_buffer_names_the_instruction():
    with pytest.raises(gfx950.EmulationError, match=r"global store \(lane 0\) of 4 bytes at 0x110000000 lies outside every buffer(.|\n)*global_store_dword"):
        run("""
            v_lshlrev_b32_e32 v10, 2, v0
            s_mov_b32 s10, 0x10000000
            s_mov_b32 s11, 1
            s_nop 4
            global_store_dword v10, v0, s[10:11]
        """)


def test_matrix_instruction_lane_layout():
    """v_mfma_f32_32x32x2_f32: lane l supplies A[l % 32][l / 32] and B[l / 32][l % 32]; register e of the 16 holds element
    [8 (e / 4) + 4 (l / 32) + e % 4][l % 32].  With A[i][k] = i + 100 k and B[k][j] = (k + 1) (j + 1): D[i][j] = i (j + 1) + (i + 100) 2 (j + 1)."""
    stores = "\n".join(f"v_mov_b32_e32 v1, v{20 + e}\nglobal_store_dword v10, v1, s[10:11] offset:{256 * e}" for e in range(16))
    out = run("""
        v_and_b32_e32 v2, 31, v0
        v_lshrrev_b32_e32 v3, 5, v0
        v_mul_u32_u24_e32 v4, 0x64, v3
        v_add_u32_e32 v4, v4, v2
        v_cvt_f32_u32_e32 v4, v4
        v_add_u32_e32 v5, 1, v3
        v_add_u32_e32 v6, 1, v2
        v_mul_lo_u32 v5, v5, v6
        v_cvt_f32_u32_e32 v5, v5
        s_nop 1
        v_mfma_f32_32x32x2_f32 v[20:35], v4, v5, 0
        s_nop 15
        s_nop 3
        v_lshlrev_b32_e32 v10, 2, v0
        s_mov_b32 s10, 0x10000000
        s_mov_b32 s11, 0
    """ + stores).view(np.float32)
    for e in range(16):
        for lane in range(64):
            i, j = 8 * (e // 4) + 4 * (lane // 32) + e % 4, lane % 32
            assert out[64 * e + lane] == i * (j + 1) + (i + 100) * 2 * (j + 1), (e, lane)


def test_wait_states_before_a_vector_memory_instruction_reading_a_fresh_scalar():
    body = """
        v_lshlrev_b32_e32 v10, 2, v0
        v_mov_b32_e32 v3, 0x10000000
        s_mov_b32 s11, 0
        v_readfirstlane_b32 s10, v3
        %s
        global_store_dword v10, v0, s[10:11]
    """
    assert list(run(body % "s_nop 4")[:3]) == [0, 1, 2]
    with pytest.raises(gfx950.EmulationError, match="3 wait states after a vector instruction wrote it"):
        run(body % "s_nop 2")


def test_an_unknown_instruction_stops_the_run():
    with pytest.raises(gfx950.EmulationError, match="no model of instruction v_frobnicate_b32"):
        run("v_frobnicate_b32 v1, v2")


def test_relocation_across_4gib_moves_the_pointers_along():
    import harness

    buffers = [(0x5000_1230, np.zeros(100_000, np.uint8)), (0x7F00_0000_0100, np.zeros(64, np.uint8))]
    args = struct.pack("<QqQQ", 0x5000_1230 + 4000, 12345, 0x7F00_0000_0100, 0x5000_1230 + 100_000)   # a pointer, a number, a pointer, one past the end
    placed, moved = harness.across_4gib(buffers, args)
    p0, number, p1, end = struct.unpack("<QqQQ", moved)
    assert number == 12345 and p0 == placed[0] + 4000 and p1 == placed[1] and end == placed[0] + 100_000
    assert placed[0] % 4096 == 0x230 and placed[0] >> 32 != (placed[0] + 100_000) >> 32   # same alignment within a page; the boundary lies inside
    assert placed[1] % 4096 == 0x100
