"""An interpreter for the gfx950 code the GPU compiler generates for this library's kernels.  Test infrastructure.

The CPU replay (tests/replay/) runs the kernels' C++ source; what it cannot see is the instruction sequence that hipcc
makes of it — where the one GPU fault of this code base lived (an inline-assembly block that overwrote SCC without
saying so, and a carry the compiler had parked there).  This module closes that gap as far as a CPU can: it reads the
assembly text hipcc emits for a translation unit (`--cuda-device-only -S`), and executes a kernel launch wavefront by
wavefront: 64 lanes, scalar and vector registers, EXEC / VCC / SCC / M0, LDS, the workgroup barrier, global memory as a
set of bounded buffers.  Every global access is checked against those bounds (an address 4 GiB off is an error with the
instruction that made it), LDS accesses against the kernel's LDS size.

Memory returns late on purpose: a load's destination (registers, or LDS for the direct loads) changes only when an
s_waitcnt lets it, in the order the hardware guarantees (vector-memory operations in issue order; LDS operations in
issue order; scalar loads only at lgkmcnt(0)), so code that reads a result before waiting for it computes with stale
data, as it may on the chip.  Wait states that the compiler cannot see into an asm block for are checked as well: a
vector-memory instruction that reads a scalar register fewer than 5 wait states after a vector instruction wrote it,
and a load into LDS issued less than 1 wait state after M0 was written.

What is not modelled: timing, caches, other hazards than the two named, denormal flushing and the exact rounding of the
transcendental instructions (the GEMM kernels use none), instructions the library's kernels do not contain (an unknown
opcode stops the run with its name).
"""
from __future__ import annotations

import re
import struct

import numpy as np

MASK32 = 0xFFFFFFFF
MASK64 = 0xFFFFFFFFFFFFFFFF
LANES = np.arange(64, dtype=np.uint32)
AGPR_BASE = 256

INLINE_FLOATS = {"0.5": 0.5, "-0.5": -0.5, "1.0": 1.0, "-1.0": -1.0, "2.0": 2.0, "-2.0": -2.0, "4.0": 4.0, "-4.0": -4.0, "0.15915494": 0.15915494}


class EmulationError(RuntimeError):
    pass


def f32_bits(x: float) -> int:
    return struct.unpack("<I", struct.pack("<f", x))[0]


# ---- parsing ---------------------------------------------------------------------------------------------------------

class Operand:
    __slots__ = ("kind", "index", "count", "value", "neg", "abs")

    def __init__(self, kind, index=0, count=1, value=0, neg=False, abs_=False):
        self.kind, self.index, self.count, self.value, self.neg, self.abs = kind, index, count, value, neg, abs_

    def __repr__(self):
        return f"Operand({self.kind},{self.index},{self.count},{self.value})"


REG = re.compile(r"^([vsa])(\d+)$")
REG_RANGE = re.compile(r"^([vsa])\[(\d+):(\d+)\]$")


def parse_operand(text: str) -> Operand:
    t = text.strip()
    neg = abs_ = False
    if t.startswith("-") and len(t) > 1 and (t[1] in "vs|a" ):
        neg, t = True, t[1:]
    if t.startswith("|") and t.endswith("|"):
        abs_, t = True, t[1:-1]
    m = REG.match(t)
    if m:
        return Operand(m.group(1), int(m.group(2)), 1, 0, neg, abs_)
    m = REG_RANGE.match(t)
    if m:
        lo, hi = int(m.group(2)), int(m.group(3))
        return Operand(m.group(1), lo, hi - lo + 1, 0, neg, abs_)
    if t in ("vcc", "exec"):
        return Operand(t, 0, 2)
    if t in ("vcc_lo", "vcc_hi", "exec_lo", "exec_hi", "m0", "scc", "off", "null"):
        return Operand(t)
    if t in INLINE_FLOATS:
        return Operand("imm", value=f32_bits(INLINE_FLOATS[t]))
    try:
        v = int(t, 0)
    except ValueError:
        try:
            return Operand("imm", value=f32_bits(float(t)))
        except ValueError:
            return Operand("label", value=t)
    return Operand("imm", value=v & MASK64 if v < 0 else v)


class Instruction:
    __slots__ = ("op", "ops", "mods", "text", "line", "asm")

    def __init__(self, op, ops, mods, text, line, asm):
        self.op, self.ops, self.mods, self.text, self.line, self.asm = op, ops, mods, text, line, asm


def split_operands(rest: str):
    """Operands (comma separated) and the modifiers that trail the last one (space separated)."""
    parts = [p.strip() for p in rest.split(",")] if rest.strip() else []
    mods = {}
    if parts:
        words = parts[-1].split()
        keep = []
        for w in words:
            if ":" in w and not w.startswith(("v[", "s[", "a[")):
                k, v = w.split(":", 1)
                mods[k] = v
            elif w in ("glc", "slc", "sc0", "sc1", "nt", "gds", "clamp", "lds", "nv"):
                mods[w] = "1"
            else:
                keep.append(w)
        parts[-1] = " ".join(keep)
        if not parts[-1]:
            parts.pop()
    return parts, mods


class Kernel:
    def __init__(self, name):
        self.name = name
        self.instructions = []
        self.labels = {}
        self.desc = {}
        self.args = []


def parse_waitcnt(ins: Instruction):
    vm = lgkm = None
    for m in re.finditer(r"(vmcnt|lgkmcnt|expcnt)\((\d+)\)", ins.text):
        if m.group(1) == "vmcnt":
            vm = int(m.group(2))
        elif m.group(1) == "lgkmcnt":
            lgkm = int(m.group(2))
    if vm is None and lgkm is None and "(" not in ins.text:  # a raw immediate
        raw = int(ins.text.split()[1], 0)
        vm = (raw & 0xF) | ((raw >> 14) & 0x3) << 4
        lgkm = (raw >> 8) & 0xF
    return vm, lgkm


def parse_program(text: str):
    """name -> Kernel for every kernel of an assembly file."""
    kernels = {}
    cur = None
    in_asm = False
    lines = text.split("\n")
    for n, raw in enumerate(lines, 1):
        if "ASMSTART" in raw:
            in_asm = True
            continue
        if "ASMEND" in raw:
            in_asm = False
            continue
        line = raw.split(";")[0].rstrip()
        if not line.strip():
            continue
        m = re.match(r"^(_Z[\w$.]+|[A-Za-z_][\w$.]*):\s*$", line)
        if m and not line.startswith(".L"):
            cur = Kernel(m.group(1))
            kernels[cur.name] = cur
            continue
        m = re.match(r"^(\.L[\w$.]+):\s*$", line)
        if m:
            if cur is not None:
                cur.labels[m.group(1)] = len(cur.instructions)
            continue
        s = line.strip()
        if s.startswith(".amdhsa_kernel "):
            cur_desc = kernels.get(s.split()[1])
            continue
        if s.startswith(".amdhsa_") and "cur_desc" in locals() and cur_desc is not None:
            k, v = s.split()[:2]
            try:
                cur_desc.desc[k[len(".amdhsa_"):]] = int(v, 0)
            except ValueError:
                pass
            continue
        if s.startswith(".end_amdhsa_kernel"):
            cur_desc = None
            continue
        if s.startswith("."):
            if s.startswith(".Lfunc_end"):
                cur = None
            continue
        if cur is None:
            continue
        op, _, rest = s.partition(" ")
        if op == "s_waitcnt":
            ins = Instruction(op, [], {}, s, n, in_asm)
            ins.mods["vm"], ins.mods["lgkm"] = parse_waitcnt(ins)
        else:
            parts, mods = split_operands(rest)
            ins = Instruction(op, [parse_operand(p) for p in parts], mods, s, n, in_asm)
        cur.instructions.append(ins)
    # the argument lists of the metadata
    meta = re.search(r"\.amdgpu_metadata\n---\n(.*?)\n\.\.\.", text, re.S)
    if meta:
        import yaml

        doc = yaml.safe_load(meta.group(1))
        for k in doc.get("amdhsa.kernels", []):
            name = k[".name"]
            if name in kernels:
                kernels[name].args = k.get(".args", [])
                kernels[name].desc["kernarg_segment_size"] = k.get(".kernarg_segment_size", 0)
    return {k: v for k, v in kernels.items() if v.instructions and "group_segment_fixed_size" in v.desc}


# ---- memory ----------------------------------------------------------------------------------------------------------

class Memory:
    """Global memory: disjoint buffers at their own addresses; nothing else is mapped."""

    def __init__(self):
        self.bases = []
        self.buffers = []

    def map(self, base: int, data: np.ndarray):
        assert data.dtype == np.uint8
        self.bases.append(base)
        self.buffers.append(data)

    def find(self, addr: int, size: int, what: str):
        for base, buf in zip(self.bases, self.buffers):
            if base <= addr and addr + size <= base + len(buf):
                return buf, addr - base
        raise EmulationError(f"{what} of {size} bytes at 0x{addr:x} lies outside every buffer")

    def read(self, addr: int, size: int, what="read") -> bytes:
        buf, off = self.find(addr, size, what)
        return buf[off:off + size].tobytes()

    def write(self, addr: int, data: bytes, what="write"):
        buf, off = self.find(addr, len(data), what)
        buf[off:off + len(data)] = np.frombuffer(data, dtype=np.uint8)

    def gather_dwords(self, addrs: np.ndarray, active: np.ndarray, n: int, what: str) -> np.ndarray:
        """n dwords per active lane from per-lane byte addresses: uint32 [n, 64]."""
        out = np.zeros((n, 64), dtype=np.uint32)
        idx = np.nonzero(active)[0]
        if len(idx) == 0:
            return out
        a = addrs[idx].astype(np.uint64)
        lo, hi = int(a.min()), int(a.max()) + 4 * n
        try:
            buf, off = self.find(lo, hi - lo, what)
        except EmulationError:
            buf = None
        if buf is not None and np.all(a % 4 == 0) and (lo - off) % 4 == 0:
            words = buf.view(np.uint32) if (len(buf) % 4 == 0) else None
            if words is not None:
                base_word = (a - np.uint64(lo - off)) // np.uint64(4)
                for j in range(n):
                    out[j, idx] = words[(base_word + np.uint64(j)).astype(np.int64)]
                return out
        for lane, address in zip(idx, a):
            data = self.read(int(address), 4 * n, f"{what} (lane {lane})")
            out[:, lane] = np.frombuffer(data, dtype=np.uint32)
        return out

    def scatter_dwords(self, addrs: np.ndarray, active: np.ndarray, values: np.ndarray, what: str):
        n = values.shape[0]
        for lane in np.nonzero(active)[0]:
            self.write(int(addrs[lane]), values[:, lane].astype(np.uint32).tobytes(), f"{what} (lane {lane})")


# ---- a wavefront -----------------------------------------------------------------------------------------------------

SCALAR_WRITERS_BY_VALU = ("v_readfirstlane_b32", "v_readlane_b32")


class Wave:
    def __init__(self, emu, kernel: Kernel, wg, wave_index: int, lanes_alive: int):
        self.emu, self.k, self.wg, self.index = emu, kernel, wg, wave_index
        # nothing is zero that the hardware does not promise to be: registers, LDS and scratch start with a pattern that is a NaN as a
        # float and far outside every buffer as an address, so that a value used before it is written cannot pass for a right one
        self.s = [0xDEADBEEF] * 128
        self.v = np.full((512, 64), 0xFFFFDEAD, dtype=np.uint32)
        self.vcc = 0xAAAAAAAAAAAAAAAA
        self.exec = (1 << lanes_alive) - 1 if lanes_alive < 64 else MASK64
        self.em = self._mask_array(self.exec)
        self.m0 = 0xDEADBEEF
        self.scc = 1
        self.pc = 0
        self.done = False
        self.vm_queue = []      # vector memory operations in flight: callables that complete them (None: nothing to do)
        self.lgkm_queue = []    # (is_scalar_load, completion)
        self.scratch = np.full((64, max(4, kernel.desc.get("private_segment_fixed_size", 0) + 64)), 0xFF, dtype=np.uint8)
        self.steps = 0
        self.clock = 0                       # issue slots, counting the wait states of s_nop
        self.sgpr_written_by_valu = {}       # sgpr index -> clock of the vector instruction that wrote it
        self.m0_written = -100

    @staticmethod
    def _mask_array(mask: int) -> np.ndarray:
        return ((np.uint64(mask) >> LANES.astype(np.uint64)) & np.uint64(1)).astype(bool)

    def set_exec(self, value: int):
        self.exec = value & MASK64
        self.em = self._mask_array(self.exec)

    # -- scalar operand access --
    def sread(self, o: Operand, bits=32) -> int:
        k = o.kind
        if k == "s":
            if bits == 64:
                return self.s[o.index] | (self.s[o.index + 1] << 32)
            return self.s[o.index]
        if k == "imm":
            if bits == 64:
                v = o.value
                return v & MASK64
            return o.value & MASK32
        if k == "vcc":
            return self.vcc if bits == 64 else self.vcc & MASK32
        if k == "exec":
            return self.exec if bits == 64 else self.exec & MASK32
        if k == "vcc_lo":
            return self.vcc & MASK32
        if k == "vcc_hi":
            return self.vcc >> 32
        if k == "exec_lo":
            return self.exec & MASK32
        if k == "exec_hi":
            return self.exec >> 32
        if k == "m0":
            return self.m0
        if k == "scc":
            return self.scc
        if k == "null":
            return 0
        if k == "label" and o.value in ("src_shared_base", "src_private_base"):
            # the aperture of LDS / scratch in the flat address space: high half of a 64-bit flat address
            hi = 0x00010000 if o.value == "src_shared_base" else 0x00020000
            return (hi << 32) if bits == 64 else hi
        raise EmulationError(f"scalar read of {o}")

    def swrite(self, o: Operand, value: int, bits=32):
        k = o.kind
        if k == "s":
            if bits == 64:
                self.s[o.index] = value & MASK32
                self.s[o.index + 1] = (value >> 32) & MASK32
            else:
                self.s[o.index] = value & MASK32
        elif k == "vcc":
            self.vcc = value & MASK64
        elif k == "exec":
            self.set_exec(value)
        elif k == "vcc_lo":
            self.vcc = (self.vcc & ~MASK32) | (value & MASK32)
        elif k == "vcc_hi":
            self.vcc = (self.vcc & MASK32) | ((value & MASK32) << 32)
        elif k == "exec_lo":
            self.set_exec((self.exec & ~MASK32) | (value & MASK32))
        elif k == "exec_hi":
            self.set_exec((self.exec & MASK32) | ((value & MASK32) << 32))
        elif k == "m0":
            self.m0 = value & MASK32
            self.m0_written = self.clock
        elif k == "null":
            pass
        else:
            raise EmulationError(f"scalar write of {o}")

    # -- vector operand access --
    def vindex(self, o: Operand) -> int:
        return o.index + (AGPR_BASE if o.kind == "a" else 0)

    def vread(self, o: Operand) -> np.ndarray:
        """32-bit source of a vector instruction as uint32[64]."""
        if o.kind in ("v", "a"):
            return self.v[self.vindex(o)].copy()   # (a copy: the destination may be the same register)
        return np.full(64, self.sread(o) & MASK32, dtype=np.uint32)

    def vread64(self, o: Operand) -> np.ndarray:
        if o.kind in ("v", "a"):
            i = self.vindex(o)
            return self.v[i].astype(np.uint64) | (self.v[i + 1].astype(np.uint64) << np.uint64(32))
        if o.kind == "imm":
            return np.full(64, o.value & MASK64, dtype=np.uint64)
        return np.full(64, self.sread(o, 64), dtype=np.uint64)

    def fread(self, o: Operand) -> np.ndarray:
        x = self.vread(o).view(np.float32)
        if o.abs:
            x = np.abs(x)
        if o.neg:
            x = -x
        return x

    def vwrite(self, o: Operand, value: np.ndarray, offset=0):
        np.copyto(self.v[self.vindex(o) + offset], value.astype(np.uint32, copy=False), where=self.em)

    def vwrite64(self, o: Operand, value: np.ndarray):
        value = value.astype(np.uint64, copy=False)
        self.vwrite(o, (value & np.uint64(MASK32)).astype(np.uint32))
        self.vwrite(o, (value >> np.uint64(32)).astype(np.uint32), 1)

    def fwrite(self, o: Operand, value: np.ndarray):
        self.vwrite(o, np.asarray(value, dtype=np.float32).view(np.uint32))

    def mask_write(self, o: Operand, lanes_true: np.ndarray):
        """A per-lane condition into VCC or an SGPR pair: bits of inactive lanes become 0."""
        bits = lanes_true & self.em
        value = int(np.bitwise_or.reduce(np.left_shift(bits.astype(np.uint64), LANES.astype(np.uint64))))
        self.swrite(o, value, 64)
        if o.kind == "s":
            self.sgpr_written_by_valu[o.index] = self.clock
            self.sgpr_written_by_valu[o.index + 1] = self.clock

    def mask_read(self, o: Operand) -> np.ndarray:
        return self._mask_array(self.sread(o, 64))

    # -- outstanding memory operations --
    def wait(self, vm, lgkm):
        if vm is not None:
            while len(self.vm_queue) > vm:
                done = self.vm_queue.pop(0)
                if done:
                    done()
        if lgkm is not None:
            if lgkm == 0:
                for _scalar, done in self.lgkm_queue:
                    if done:
                        done()
                self.lgkm_queue = []
            else:
                # LDS operations return in order; a scalar load may return at any time, so it is complete only at lgkmcnt(0)
                while len(self.lgkm_queue) > lgkm and not any(sc for sc, _ in self.lgkm_queue):
                    _sc, done = self.lgkm_queue.pop(0)
                    if done:
                        done()

    def issue_vm(self, completion):
        if self.emu.late:
            self.vm_queue.append(completion)
            if len(self.vm_queue) > 63:   # the counter holds 63: the hardware issues no further one before the oldest has returned
                done = self.vm_queue.pop(0)
                if done:
                    done()
        elif completion:
            completion()

    def issue_lgkm(self, scalar, completion):
        if self.emu.late:
            self.lgkm_queue.append((scalar, completion))
        elif completion:
            completion()

    def where(self):
        ins = self.k.instructions[self.pc] if self.pc < len(self.k.instructions) else None
        return f"{self.k.name} workgroup {self.wg.bid} wave {self.index}, line {ins.line if ins else '?'}: {ins.text if ins else ''}"


class Workgroup:
    def __init__(self, bid, lds_bytes):
        self.bid = bid
        self.lds = np.full(max(lds_bytes, 4), 0xFF, dtype=np.uint8)   # (LDS is not cleared between workgroups on the chip)
        self.lds32 = self.lds.view(np.uint32)
        self.lds_bytes = lds_bytes


# ---- the instruction set ---------------------------------------------------------------------------------------------

def _s32(x: int) -> int:
    x &= MASK32
    return x - (1 << 32) if x & 0x80000000 else x


def _s64(x: int) -> int:
    x &= MASK64
    return x - (1 << 64) if x & (1 << 63) else x


class Emulator:
    def __init__(self, program: dict, memory: Memory, late=True, check_hazards=True, reverse=False):
        """reverse: workgroups of the grid and the wavefronts of a workgroup take their turns in descending instead of ascending order
        (a result must not depend on either: what one wavefront hands to another goes through a barrier)."""
        self.program, self.mem, self.late, self.check_hazards, self.reverse = program, memory, late, check_hazards, reverse
        self.kernarg_base = 0x7F00_0000_0000
        self.instruction_count = 0
        self.opcode_counts = {}
        self.handlers = {}
        for name in dir(self):
            if name.startswith("op_"):
                self.handlers[name[3:]] = getattr(self, name)

    # -- launching --
    def launch(self, kernel_name: str, grid, block, kernarg: bytes, max_steps=50_000_000):
        k = self.program[kernel_name]
        d = k.desc
        size = max(d.get("kernarg_size", 0), d.get("kernarg_segment_size", 0), len(kernarg))
        karg = bytearray(size + 64)
        karg[:len(kernarg)] = kernarg
        for a in k.args:
            kind, off, sz = a.get(".value_kind"), a[".offset"], a[".size"]
            value = None
            if kind in ("hidden_block_count_x", "hidden_block_count_y", "hidden_block_count_z"):
                value = grid["xyz".index(kind[-1])]
            elif kind in ("hidden_group_size_x", "hidden_group_size_y", "hidden_group_size_z"):
                value = block["xyz".index(kind[-1])]
            elif kind.startswith("hidden_remainder") or kind.startswith("hidden_global_offset"):
                value = 0
            elif kind == "hidden_grid_dims":
                value = 1 + (grid[1] * block[1] > 1) + (grid[2] * block[2] > 1)
            if value is not None:
                karg[off:off + sz] = int(value).to_bytes(sz, "little")
        explicit = [a for a in k.args if a.get(".value_kind") in ("by_value", "global_buffer")]
        if explicit:
            end = explicit[-1][".offset"] + explicit[-1][".size"]
            if not (end - 8 < len(kernarg) <= end + 8):
                raise EmulationError(f"{kernel_name}: {len(kernarg)} bytes of arguments given, the kernel takes {end}")
        kbuf = np.frombuffer(bytes(karg), dtype=np.uint8).copy()
        self.mem.map(self.kernarg_base, kbuf)
        try:
            threads = block[0] * block[1] * block[2]
            ids = [(bx, by, bz) for bz in range(grid[2]) for by in range(grid[1]) for bx in range(grid[0])]
            for bid in (reversed(ids) if self.reverse else ids):
                self.run_workgroup(k, bid, block, threads, max_steps)
        finally:
            self.mem.bases.pop()
            self.mem.buffers.pop()

    def run_workgroup(self, k: Kernel, bid, block, threads, max_steps):
        d = k.desc
        wg = Workgroup(bid, d["group_segment_fixed_size"])
        waves = []
        for w in range((threads + 63) // 64):
            alive = min(64, threads - 64 * w)
            wave = Wave(self, k, wg, w, alive)
            # user SGPRs, then the system ones
            i = 0
            for flag, n in (("user_sgpr_private_segment_buffer", 4), ("user_sgpr_dispatch_ptr", 2), ("user_sgpr_queue_ptr", 2),
                            ("user_sgpr_kernarg_segment_ptr", 2), ("user_sgpr_dispatch_id", 2), ("user_sgpr_flat_scratch_init", 2),
                            ("user_sgpr_private_segment_size", 1)):
                if d.get(flag, 0):
                    if flag == "user_sgpr_kernarg_segment_ptr":
                        wave.s[i] = self.kernarg_base & MASK32
                        wave.s[i + 1] = self.kernarg_base >> 32
                    i += n
            i += d.get("user_sgpr_kernarg_preload_length", 0)
            if i != d.get("user_sgpr_count", i):
                raise EmulationError(f"{k.name}: {d.get('user_sgpr_count')} user SGPRs, {i} accounted for")
            for flag, value in (("system_sgpr_workgroup_id_x", bid[0]), ("system_sgpr_workgroup_id_y", bid[1]), ("system_sgpr_workgroup_id_z", bid[2]),
                                ("system_sgpr_workgroup_info", 0)):
                if d.get(flag, 0):
                    wave.s[i] = value
                    i += 1
            if d.get("enable_private_segment", 0):
                wave.s[i] = 0  # (the wave's scratch offset: scratch is private to each emulated wave already)
                i += 1
            tid = 64 * w + LANES
            tx = tid % block[0]
            ty = (tid // block[0]) % block[1]
            tz = tid // (block[0] * block[1])
            wave.v[0] = (tx | (ty << 10) | (tz << 20)).astype(np.uint32)
            waves.append(wave)
        # run: each wave until it ends or meets the barrier; the barrier opens when every wave that is still running has arrived
        while True:
            running = [w for w in waves if not w.done]
            if not running:
                break
            for w in (reversed(running) if self.reverse else running):
                self.run_until_barrier(w, max_steps)
            # (a wave that ended no longer takes part)

    def run_until_barrier(self, w: Wave, max_steps):
        ins_list = w.k.instructions
        handlers = self.handlers
        while True:
            if w.pc >= len(ins_list):
                raise EmulationError(f"ran off the end of {w.k.name}")
            ins = ins_list[w.pc]
            w.steps += 1
            if w.steps > max_steps:
                raise EmulationError(f"more than {max_steps} instructions in one wave: {w.where()}")
            op = ins.op
            self.opcode_counts[op] = self.opcode_counts.get(op, 0) + 1
            if op == "s_barrier":
                w.pc += 1
                w.clock += 1
                return
            if op == "s_endpgm":
                w.wait(0, 0)
                w.done = True
                return
            h = handlers.get(op)
            if h is None:
                base = re.sub(r"_(e32|e64|sdwa|dpp)$", "", op)
                h = handlers.get(base)
                if h is None:
                    raise EmulationError(f"no model of instruction {op}: {w.where()}")
                handlers[op] = h
            if self.check_hazards:
                self.hazards(w, ins)
            try:
                jumped = h(w, ins)
            except EmulationError as e:
                raise EmulationError(f"{e}\n  at {w.where()}") from None
            w.clock += 1
            if not jumped:
                w.pc += 1

    # -- wait-state checks the compiler cannot make inside an asm block --
    def hazards(self, w: Wave, ins: Instruction):
        op = ins.op
        if op.startswith(("global_", "buffer_", "scratch_", "flat_")):
            for o in ins.ops:
                if o.kind == "s":
                    for i in range(o.index, o.index + o.count):
                        t = w.sgpr_written_by_valu.get(i)
                        if t is not None and w.clock - t - 1 < 5:
                            raise EmulationError(f"vector memory instruction reads s{i} {w.clock - t - 1} wait states after a vector instruction wrote it (5 needed): {w.where()}")
            if "_lds_" in op and w.clock - w.m0_written - 1 < 1:
                raise EmulationError(f"load into LDS {w.clock - w.m0_written - 1} wait states after M0 was written (1 needed): {w.where()}")

    # ---- scalar ALU ----
    def op_s_nop(self, w, i):
        w.clock += i.ops[0].value

    def op_s_mov_b32(self, w, i):
        w.swrite(i.ops[0], w.sread(i.ops[1]))

    def op_s_mov_b64(self, w, i):
        w.swrite(i.ops[0], _sext64(i.ops[1], w), 64)

    def op_s_movk_i32(self, w, i):
        v = i.ops[1].value & 0xFFFF
        w.swrite(i.ops[0], (v - 0x10000 if v & 0x8000 else v) & MASK32)

    def op_s_add_u32(self, w, i):
        r = w.sread(i.ops[1]) + w.sread(i.ops[2])
        w.scc = int(r > MASK32)
        w.swrite(i.ops[0], r)

    def op_s_addc_u32(self, w, i):
        r = w.sread(i.ops[1]) + w.sread(i.ops[2]) + w.scc
        w.scc = int(r > MASK32)
        w.swrite(i.ops[0], r)

    def op_s_sub_u32(self, w, i):
        a, b = w.sread(i.ops[1]), w.sread(i.ops[2])
        w.scc = int(b > a)
        w.swrite(i.ops[0], a - b)

    def op_s_subb_u32(self, w, i):
        a, b = w.sread(i.ops[1]), w.sread(i.ops[2])
        borrow = int(b + w.scc > a)
        w.swrite(i.ops[0], a - b - w.scc)
        w.scc = borrow

    def op_s_add_i32(self, w, i):
        a, b = _s32(w.sread(i.ops[1])), _s32(w.sread(i.ops[2]))
        r = a + b
        w.scc = int(r != _s32(r))
        w.swrite(i.ops[0], r)

    def op_s_sub_i32(self, w, i):
        a, b = _s32(w.sread(i.ops[1])), _s32(w.sread(i.ops[2]))
        r = a - b
        w.scc = int(r != _s32(r))
        w.swrite(i.ops[0], r)

    def op_s_addk_i32(self, w, i):
        k = i.ops[1].value & 0xFFFF
        k = k - 0x10000 if k & 0x8000 else k
        a = _s32(w.sread(i.ops[0]))
        r = a + k
        w.scc = int(r != _s32(r))
        w.swrite(i.ops[0], r)

    def op_s_mulk_i32(self, w, i):
        k = i.ops[1].value & 0xFFFF
        k = k - 0x10000 if k & 0x8000 else k
        w.swrite(i.ops[0], _s32(w.sread(i.ops[0])) * k)

    def op_s_mul_i32(self, w, i):
        w.swrite(i.ops[0], _s32(w.sread(i.ops[1])) * _s32(w.sread(i.ops[2])))

    def op_s_mul_hi_u32(self, w, i):
        w.swrite(i.ops[0], (w.sread(i.ops[1]) * w.sread(i.ops[2])) >> 32)

    def op_s_mul_hi_i32(self, w, i):
        w.swrite(i.ops[0], (_s32(w.sread(i.ops[1])) * _s32(w.sread(i.ops[2]))) >> 32)

    def _logic(self, w, i, bits, f):
        r = f(w.sread(i.ops[1], bits), w.sread(i.ops[2], bits)) & (MASK64 if bits == 64 else MASK32)
        w.swrite(i.ops[0], r, bits)
        w.scc = int(r != 0)

    def op_s_and_b32(self, w, i):
        self._logic(w, i, 32, lambda a, b: a & b)

    def op_s_and_b64(self, w, i):
        self._logic(w, i, 64, lambda a, b: a & b)

    def op_s_or_b32(self, w, i):
        self._logic(w, i, 32, lambda a, b: a | b)

    def op_s_or_b64(self, w, i):
        self._logic(w, i, 64, lambda a, b: a | b)

    def op_s_xor_b32(self, w, i):
        self._logic(w, i, 32, lambda a, b: a ^ b)

    def op_s_xor_b64(self, w, i):
        self._logic(w, i, 64, lambda a, b: a ^ b)

    def op_s_andn2_b64(self, w, i):
        self._logic(w, i, 64, lambda a, b: a & ~b)

    def op_s_andn2_b32(self, w, i):
        self._logic(w, i, 32, lambda a, b: a & ~b)

    def op_s_orn2_b64(self, w, i):
        self._logic(w, i, 64, lambda a, b: a | ~b)

    def op_s_not_b32(self, w, i):
        r = ~w.sread(i.ops[1]) & MASK32
        w.swrite(i.ops[0], r)
        w.scc = int(r != 0)

    def op_s_not_b64(self, w, i):
        r = ~w.sread(i.ops[1], 64) & MASK64
        w.swrite(i.ops[0], r, 64)
        w.scc = int(r != 0)

    def op_s_lshl_b32(self, w, i):
        r = (w.sread(i.ops[1]) << (w.sread(i.ops[2]) & 31)) & MASK32
        w.swrite(i.ops[0], r)
        w.scc = int(r != 0)

    def op_s_lshl_b64(self, w, i):
        r = (w.sread(i.ops[1], 64) << (w.sread(i.ops[2]) & 63)) & MASK64
        w.swrite(i.ops[0], r, 64)
        w.scc = int(r != 0)

    def op_s_lshr_b32(self, w, i):
        r = w.sread(i.ops[1]) >> (w.sread(i.ops[2]) & 31)
        w.swrite(i.ops[0], r)
        w.scc = int(r != 0)

    def op_s_lshr_b64(self, w, i):
        r = w.sread(i.ops[1], 64) >> (w.sread(i.ops[2]) & 63)
        w.swrite(i.ops[0], r, 64)
        w.scc = int(r != 0)

    def op_s_ashr_i32(self, w, i):
        r = (_s32(w.sread(i.ops[1])) >> (w.sread(i.ops[2]) & 31)) & MASK32
        w.swrite(i.ops[0], r)
        w.scc = int(r != 0)

    def op_s_ashr_i64(self, w, i):
        r = (_s64(_sext64(i.ops[1], w)) >> (w.sread(i.ops[2]) & 63)) & MASK64
        w.swrite(i.ops[0], r, 64)
        w.scc = int(r != 0)

    def op_s_bfe_u32(self, w, i):
        src, spec = w.sread(i.ops[1]), w.sread(i.ops[2])
        off, width = spec & 31, (spec >> 16) & 0x7F
        r = (src >> off) & ((1 << width) - 1) if width else 0
        w.swrite(i.ops[0], r)
        w.scc = int(r != 0)

    def op_s_bfe_i32(self, w, i):
        src, spec = w.sread(i.ops[1]), w.sread(i.ops[2])
        off, width = spec & 31, (spec >> 16) & 0x7F
        r = (src >> off) & ((1 << width) - 1) if width else 0
        if width and r & (1 << (width - 1)):
            r -= 1 << width
        w.swrite(i.ops[0], r)
        w.scc = int(r & MASK32 != 0)

    def op_s_bfe_i64(self, w, i):
        src, spec = _sext64(i.ops[1], w), w.sread(i.ops[2])
        off, width = spec & 63, (spec >> 16) & 0x7F
        r = (src >> off) & ((1 << width) - 1) if width else 0
        if width and r & (1 << (width - 1)):
            r -= 1 << width
        w.swrite(i.ops[0], r & MASK64, 64)
        w.scc = int(r & MASK64 != 0)

    def op_s_min_i32(self, w, i):
        a, b = _s32(w.sread(i.ops[1])), _s32(w.sread(i.ops[2]))
        w.scc = int(a < b)
        w.swrite(i.ops[0], min(a, b))

    def op_s_max_i32(self, w, i):
        a, b = _s32(w.sread(i.ops[1])), _s32(w.sread(i.ops[2]))
        w.scc = int(a > b)
        w.swrite(i.ops[0], max(a, b))

    def op_s_min_u32(self, w, i):
        a, b = w.sread(i.ops[1]), w.sread(i.ops[2])
        w.scc = int(a < b)
        w.swrite(i.ops[0], min(a, b))

    def op_s_max_u32(self, w, i):
        a, b = w.sread(i.ops[1]), w.sread(i.ops[2])
        w.scc = int(a > b)
        w.swrite(i.ops[0], max(a, b))

    def op_s_abs_i32(self, w, i):
        r = abs(_s32(w.sread(i.ops[1]))) & MASK32
        w.swrite(i.ops[0], r)
        w.scc = int(r != 0)

    def op_s_cselect_b32(self, w, i):
        w.swrite(i.ops[0], w.sread(i.ops[1]) if w.scc else w.sread(i.ops[2]))

    def op_s_cselect_b64(self, w, i):
        w.swrite(i.ops[0], _sext64(i.ops[1], w) if w.scc else _sext64(i.ops[2], w), 64)

    def op_s_bitset1_b32(self, w, i):
        w.swrite(i.ops[0], w.sread(i.ops[0]) | (1 << (w.sread(i.ops[1]) & 31)))

    def op_s_bitset0_b32(self, w, i):
        w.swrite(i.ops[0], w.sread(i.ops[0]) & ~(1 << (w.sread(i.ops[1]) & 31)))

    def op_s_bcnt1_i32_b64(self, w, i):
        r = bin(w.sread(i.ops[1], 64)).count("1")
        w.swrite(i.ops[0], r)
        w.scc = int(r != 0)

    def op_s_bcnt1_i32_b32(self, w, i):
        r = bin(w.sread(i.ops[1])).count("1")
        w.swrite(i.ops[0], r)
        w.scc = int(r != 0)

    def op_s_flbit_i32_b32(self, w, i):
        x = w.sread(i.ops[1])
        w.swrite(i.ops[0], (32 - x.bit_length()) if x else MASK32)

    def op_s_flbit_i32(self, w, i):
        x = w.sread(i.ops[1])
        if x in (0, MASK32):
            w.swrite(i.ops[0], MASK32)
        else:
            sign = x >> 31
            n = 0
            for b in range(31, -1, -1):
                if (x >> b) & 1 != sign:
                    break
                n += 1
            w.swrite(i.ops[0], n)

    def op_s_ff1_i32_b32(self, w, i):
        x = w.sread(i.ops[1])
        w.swrite(i.ops[0], (x & -x).bit_length() - 1 if x else MASK32)

    def op_s_ff1_i32_b64(self, w, i):
        x = w.sread(i.ops[1], 64)
        w.swrite(i.ops[0], (x & -x).bit_length() - 1 if x else MASK32)

    def _saveexec(self, w, i, f):
        old, src = w.exec, w.sread(i.ops[1], 64)   # (source and destination may be the same register pair)
        w.swrite(i.ops[0], old, 64)
        w.set_exec(f(src, old))
        w.scc = int(w.exec != 0)

    def op_s_and_saveexec_b64(self, w, i):
        self._saveexec(w, i, lambda s, e: s & e)

    def op_s_or_saveexec_b64(self, w, i):
        self._saveexec(w, i, lambda s, e: s | e)

    def op_s_xor_saveexec_b64(self, w, i):
        self._saveexec(w, i, lambda s, e: s ^ e)

    def op_s_andn2_saveexec_b64(self, w, i):
        self._saveexec(w, i, lambda s, e: s & ~e)

    def op_s_andn1_saveexec_b64(self, w, i):
        self._saveexec(w, i, lambda s, e: ~s & e)

    def _scmp(self, w, i, signed, f, bits=32):
        a, b = w.sread(i.ops[0], bits), w.sread(i.ops[1], bits)
        if signed:
            a, b = _s32(a), _s32(b)
        w.scc = int(f(a, b))

    def op_s_cmp_eq_u32(self, w, i):
        self._scmp(w, i, False, lambda a, b: a == b)

    def op_s_cmp_eq_i32(self, w, i):
        self._scmp(w, i, False, lambda a, b: a == b)

    def op_s_cmp_lg_u32(self, w, i):
        self._scmp(w, i, False, lambda a, b: a != b)

    def op_s_cmp_lg_i32(self, w, i):
        self._scmp(w, i, False, lambda a, b: a != b)

    def op_s_cmp_eq_u64(self, w, i):
        self._scmp(w, i, False, lambda a, b: a == b, 64)

    def op_s_cmp_lg_u64(self, w, i):
        self._scmp(w, i, False, lambda a, b: a != b, 64)

    def op_s_cmp_gt_u32(self, w, i):
        self._scmp(w, i, False, lambda a, b: a > b)

    def op_s_cmp_ge_u32(self, w, i):
        self._scmp(w, i, False, lambda a, b: a >= b)

    def op_s_cmp_lt_u32(self, w, i):
        self._scmp(w, i, False, lambda a, b: a < b)

    def op_s_cmp_le_u32(self, w, i):
        self._scmp(w, i, False, lambda a, b: a <= b)

    def op_s_cmp_gt_i32(self, w, i):
        self._scmp(w, i, True, lambda a, b: a > b)

    def op_s_cmp_ge_i32(self, w, i):
        self._scmp(w, i, True, lambda a, b: a >= b)

    def op_s_cmp_lt_i32(self, w, i):
        self._scmp(w, i, True, lambda a, b: a < b)

    def op_s_cmp_le_i32(self, w, i):
        self._scmp(w, i, True, lambda a, b: a <= b)

    def _scmpk(self, w, i, signed, f):
        a = w.sread(i.ops[0])
        k = i.ops[1].value & 0xFFFF
        if signed:
            a = _s32(a)
            k = k - 0x10000 if k & 0x8000 else k
        w.scc = int(f(a, k))

    def op_s_cmpk_eq_i32(self, w, i):
        self._scmpk(w, i, True, lambda a, b: a == b)

    def op_s_cmpk_lg_i32(self, w, i):
        self._scmpk(w, i, True, lambda a, b: a != b)

    def op_s_cmpk_gt_i32(self, w, i):
        self._scmpk(w, i, True, lambda a, b: a > b)

    def op_s_cmpk_ge_i32(self, w, i):
        self._scmpk(w, i, True, lambda a, b: a >= b)

    def op_s_cmpk_lt_i32(self, w, i):
        self._scmpk(w, i, True, lambda a, b: a < b)

    def op_s_cmpk_le_i32(self, w, i):
        self._scmpk(w, i, True, lambda a, b: a <= b)

    def op_s_cmpk_eq_u32(self, w, i):
        self._scmpk(w, i, False, lambda a, b: a == b)

    def op_s_cmpk_lg_u32(self, w, i):
        self._scmpk(w, i, False, lambda a, b: a != b)

    def op_s_cmpk_gt_u32(self, w, i):
        self._scmpk(w, i, False, lambda a, b: a > b)

    def op_s_cmpk_ge_u32(self, w, i):
        self._scmpk(w, i, False, lambda a, b: a >= b)

    def op_s_cmpk_lt_u32(self, w, i):
        self._scmpk(w, i, False, lambda a, b: a < b)

    def op_s_cmpk_le_u32(self, w, i):
        self._scmpk(w, i, False, lambda a, b: a <= b)

    # ---- branches ----
    def _jump(self, w, i, taken):
        if taken:
            label = i.ops[0].value
            if label not in w.k.labels:
                raise EmulationError(f"branch to unknown label {label}")
            w.pc = w.k.labels[label]
            return True
        return False

    def op_s_branch(self, w, i):
        return self._jump(w, i, True)

    def op_s_cbranch_scc0(self, w, i):
        return self._jump(w, i, w.scc == 0)

    def op_s_cbranch_scc1(self, w, i):
        return self._jump(w, i, w.scc == 1)

    def op_s_cbranch_vccz(self, w, i):
        return self._jump(w, i, w.vcc == 0)

    def op_s_cbranch_vccnz(self, w, i):
        return self._jump(w, i, w.vcc != 0)

    def op_s_cbranch_execz(self, w, i):
        return self._jump(w, i, w.exec == 0)

    def op_s_cbranch_execnz(self, w, i):
        return self._jump(w, i, w.exec != 0)

    def op_s_waitcnt(self, w, i):
        w.wait(i.mods["vm"], i.mods["lgkm"])

    def op_s_sleep(self, w, i):
        pass

    def op_s_setprio(self, w, i):
        pass

    def op_buffer_wbl2(self, w, i):
        w.issue_vm(None)

    def op_buffer_inv(self, w, i):
        w.issue_vm(None)

    # ---- scalar memory ----
    def _s_load(self, w, i, n):
        base = w.sread(i.ops[1], 64)
        off = w.sread(i.ops[2]) if i.ops[2].kind != "imm" else i.ops[2].value
        if "offset" in i.mods:
            off += int(i.mods["offset"], 0)
        data = np.frombuffer(self.mem.read(base + off, 4 * n, "scalar load"), dtype=np.uint32)
        dst = i.ops[0]

        def done():
            for j in range(n):
                w.s[dst.index + j] = int(data[j])

        w.issue_lgkm(True, done)

    def op_s_load_dword(self, w, i):
        self._s_load(w, i, 1)

    def op_s_load_dwordx2(self, w, i):
        self._s_load(w, i, 2)

    def op_s_load_dwordx4(self, w, i):
        self._s_load(w, i, 4)

    def op_s_load_dwordx8(self, w, i):
        self._s_load(w, i, 8)

    def op_s_load_dwordx16(self, w, i):
        self._s_load(w, i, 16)

    # ---- vector ALU: moves and integers ----
    def op_v_mov_b32(self, w, i):
        w.vwrite(i.ops[0], w.vread(i.ops[1]))

    def op_v_mov_b64(self, w, i):
        w.vwrite64(i.ops[0], w.vread64(i.ops[1]))

    def op_v_accvgpr_read_b32(self, w, i):
        w.vwrite(i.ops[0], w.vread(i.ops[1]))

    def op_v_accvgpr_write_b32(self, w, i):
        w.vwrite(i.ops[0], w.vread(i.ops[1]))

    def op_v_accvgpr_mov_b32(self, w, i):
        w.vwrite(i.ops[0], w.vread(i.ops[1]))

    def op_v_readfirstlane_b32(self, w, i):
        first = (w.exec & -w.exec).bit_length() - 1 if w.exec else 0
        w.swrite(i.ops[0], int(w.vread(i.ops[1])[first]))
        if i.ops[0].kind == "s":
            w.sgpr_written_by_valu[i.ops[0].index] = w.clock

    def op_v_readlane_b32(self, w, i):
        lane = w.sread(i.ops[2]) & 63
        w.swrite(i.ops[0], int(w.vread(i.ops[1])[lane]))
        if i.ops[0].kind == "s":
            w.sgpr_written_by_valu[i.ops[0].index] = w.clock

    def op_v_writelane_b32(self, w, i):
        lane = w.sread(i.ops[2]) & 63
        w.v[w.vindex(i.ops[0])][lane] = w.sread(i.ops[1]) & MASK32

    def op_v_mbcnt_lo_u32_b32(self, w, i):
        mask = w.vread(i.ops[1])
        below = ((np.uint64(1) << np.minimum(LANES, 32).astype(np.uint64)) - np.uint64(1)).astype(np.uint32)
        w.vwrite(i.ops[0], _popcount32(mask & below) + w.vread(i.ops[2]))

    def op_v_mbcnt_hi_u32_b32(self, w, i):
        mask = w.vread(i.ops[1])
        shift = np.where(LANES > 32, LANES - 32, 0).astype(np.uint64)
        below = ((np.uint64(1) << shift) - np.uint64(1)).astype(np.uint32)
        w.vwrite(i.ops[0], _popcount32(mask & below) + w.vread(i.ops[2]))

    def _v2(self, w, i, f):
        w.vwrite(i.ops[0], f(w.vread(i.ops[1]), w.vread(i.ops[2])))

    def _v3(self, w, i, f):
        w.vwrite(i.ops[0], f(w.vread(i.ops[1]), w.vread(i.ops[2]), w.vread(i.ops[3])))

    def op_v_add_u32(self, w, i):
        self._v2(w, i, lambda a, b: a + b)

    def op_v_sub_u32(self, w, i):
        self._v2(w, i, lambda a, b: a - b)

    def op_v_subrev_u32(self, w, i):
        self._v2(w, i, lambda a, b: b - a)

    def op_v_add_u16(self, w, i):
        self._v2(w, i, lambda a, b: (a + b) & np.uint32(0xFFFF))

    def op_v_and_b32(self, w, i):
        self._v2(w, i, lambda a, b: a & b)

    def op_v_or_b32(self, w, i):
        self._v2(w, i, lambda a, b: a | b)

    def op_v_xor_b32(self, w, i):
        self._v2(w, i, lambda a, b: a ^ b)

    def op_v_not_b32(self, w, i):
        w.vwrite(i.ops[0], ~w.vread(i.ops[1]))

    def op_v_lshlrev_b32(self, w, i):
        self._v2(w, i, lambda a, b: b << (a & np.uint32(31)))

    def op_v_lshrrev_b32(self, w, i):
        self._v2(w, i, lambda a, b: b >> (a & np.uint32(31)))

    def op_v_ashrrev_i32(self, w, i):
        self._v2(w, i, lambda a, b: (b.view(np.int32) >> (a & np.uint32(31)).astype(np.int32)).view(np.uint32))

    def op_v_lshlrev_b64(self, w, i):
        w.vwrite64(i.ops[0], w.vread64(i.ops[2]) << (w.vread(i.ops[1]) & np.uint32(63)).astype(np.uint64))

    def op_v_lshrrev_b64(self, w, i):
        w.vwrite64(i.ops[0], w.vread64(i.ops[2]) >> (w.vread(i.ops[1]) & np.uint32(63)).astype(np.uint64))

    def op_v_ashrrev_i64(self, w, i):
        w.vwrite64(i.ops[0], (w.vread64(i.ops[2]).view(np.int64) >> (w.vread(i.ops[1]) & np.uint32(63)).astype(np.int64)).view(np.uint64))

    def op_v_add3_u32(self, w, i):
        self._v3(w, i, lambda a, b, c: a + b + c)

    def op_v_add_lshl_u32(self, w, i):
        self._v3(w, i, lambda a, b, c: (a + b) << (c & np.uint32(31)))

    def op_v_lshl_add_u32(self, w, i):
        self._v3(w, i, lambda a, b, c: (a << (b & np.uint32(31))) + c)

    def op_v_lshl_or_b32(self, w, i):
        self._v3(w, i, lambda a, b, c: (a << (b & np.uint32(31))) | c)

    def op_v_and_or_b32(self, w, i):
        self._v3(w, i, lambda a, b, c: (a & b) | c)

    def op_v_or3_b32(self, w, i):
        self._v3(w, i, lambda a, b, c: a | b | c)

    def op_v_xad_u32(self, w, i):
        self._v3(w, i, lambda a, b, c: (a ^ b) + c)

    def op_v_bitop3_b32(self, w, i):
        table = int(i.mods["bitop3"], 0)
        a, b, c = w.vread(i.ops[1]), w.vread(i.ops[2]), w.vread(i.ops[3])
        out = np.zeros(64, dtype=np.uint32)
        for idx in range(8):
            if (table >> idx) & 1:
                ta = a if idx & 4 else ~a
                tb = b if idx & 2 else ~b
                tc = c if idx & 1 else ~c
                out |= ta & tb & tc
        w.vwrite(i.ops[0], out)

    def op_v_lshl_add_u64(self, w, i):
        w.vwrite64(i.ops[0], (w.vread64(i.ops[1]) << (w.vread(i.ops[2]) & np.uint32(7)).astype(np.uint64)) + w.vread64(i.ops[3]))

    def op_v_bfe_u32(self, w, i):
        def f(a, off, width):
            off, width = off & np.uint32(31), width & np.uint32(31)
            return (a >> off) & ((np.uint64(1) << width.astype(np.uint64)) - np.uint64(1)).astype(np.uint32)
        self._v3(w, i, f)

    def op_v_bfe_i32(self, w, i):
        def f(a, off, width):
            off, width = (off & np.uint32(31)).astype(np.int64), (width & np.uint32(31)).astype(np.int64)
            x = (a.astype(np.int64) >> off) & ((np.int64(1) << width) - 1)
            sign = (width > 0) & ((x >> np.maximum(width - 1, 0)) & 1 == 1)
            x = np.where(sign, x - (np.int64(1) << width), x)
            return (x & MASK32).astype(np.uint32)
        self._v3(w, i, f)

    def op_v_mul_lo_u32(self, w, i):
        self._v2(w, i, lambda a, b: a * b)

    def op_v_mul_hi_u32(self, w, i):
        self._v2(w, i, lambda a, b: ((a.astype(np.uint64) * b.astype(np.uint64)) >> np.uint64(32)).astype(np.uint32))

    def op_v_mul_hi_i32(self, w, i):
        self._v2(w, i, lambda a, b: ((a.view(np.int32).astype(np.int64) * b.view(np.int32).astype(np.int64)) >> 32).astype(np.int32).view(np.uint32))

    def op_v_mul_u32_u24(self, w, i):
        self._v2(w, i, lambda a, b: (a & np.uint32(0xFFFFFF)) * (b & np.uint32(0xFFFFFF)))

    def op_v_mul_i32_i24(self, w, i):
        self._v2(w, i, lambda a, b: (_i24(a) * _i24(b)).astype(np.uint32))

    def op_v_mad_u32_u24(self, w, i):
        self._v3(w, i, lambda a, b, c: (a & np.uint32(0xFFFFFF)) * (b & np.uint32(0xFFFFFF)) + c)

    def op_v_mad_i32_i24(self, w, i):
        self._v3(w, i, lambda a, b, c: ((_i24(a) * _i24(b)) & MASK32).astype(np.uint32) + c)

    def op_v_mad_u64_u32(self, w, i):
        # vdst[2], sdst (carry), a, b, c[2]
        a, b = w.vread(i.ops[2]).astype(np.uint64), w.vread(i.ops[3]).astype(np.uint64)
        c = w.vread64(i.ops[4])
        r = a * b + c
        w.vwrite64(i.ops[0], r)
        w.mask_write(i.ops[1], r < c)

    def op_v_mad_i64_i32(self, w, i):
        a, b = w.vread(i.ops[2]).view(np.int32).astype(np.int64), w.vread(i.ops[3]).view(np.int32).astype(np.int64)
        c = w.vread64(i.ops[4]).view(np.int64)
        with np.errstate(over="ignore"):
            r = a * b + c
        w.vwrite64(i.ops[0], r.view(np.uint64))
        w.mask_write(i.ops[1], np.zeros(64, dtype=bool))

    def op_v_min_u32(self, w, i):
        self._v2(w, i, np.minimum)

    def op_v_max_u32(self, w, i):
        self._v2(w, i, np.maximum)

    def op_v_min_i32(self, w, i):
        self._v2(w, i, lambda a, b: np.minimum(a.view(np.int32), b.view(np.int32)).view(np.uint32))

    def op_v_max_i32(self, w, i):
        self._v2(w, i, lambda a, b: np.maximum(a.view(np.int32), b.view(np.int32)).view(np.uint32))

    def op_v_cndmask_b32(self, w, i):
        sel = w.mask_read(i.ops[3]) if len(i.ops) > 3 else w._mask_array(w.vcc)
        a, b = w.vread(i.ops[1]), w.vread(i.ops[2])
        if i.ops[1].neg or i.ops[1].abs or i.ops[2].neg or i.ops[2].abs:
            a, b = w.fread(i.ops[1]).view(np.uint32), w.fread(i.ops[2]).view(np.uint32)
        w.vwrite(i.ops[0], np.where(sel, b, a))

    # carries (vdst, carry-out, a, b[, carry-in])
    def op_v_add_co_u32(self, w, i):
        a, b = w.vread(i.ops[2]).astype(np.uint64), w.vread(i.ops[3]).astype(np.uint64)
        r = a + b
        w.vwrite(i.ops[0], (r & np.uint64(MASK32)).astype(np.uint32))
        w.mask_write(i.ops[1], r > np.uint64(MASK32))

    def op_v_addc_co_u32(self, w, i):
        cin = w.mask_read(i.ops[4]).astype(np.uint64)
        r = w.vread(i.ops[2]).astype(np.uint64) + w.vread(i.ops[3]).astype(np.uint64) + cin
        w.vwrite(i.ops[0], (r & np.uint64(MASK32)).astype(np.uint32))
        w.mask_write(i.ops[1], r > np.uint64(MASK32))

    def op_v_sub_co_u32(self, w, i):
        a, b = w.vread(i.ops[2]), w.vread(i.ops[3])
        w.vwrite(i.ops[0], a - b)
        w.mask_write(i.ops[1], b > a)

    def op_v_subrev_co_u32(self, w, i):
        a, b = w.vread(i.ops[2]), w.vread(i.ops[3])
        w.vwrite(i.ops[0], b - a)
        w.mask_write(i.ops[1], a > b)

    def op_v_subb_co_u32(self, w, i):
        cin = w.mask_read(i.ops[4]).astype(np.uint64)
        a, b = w.vread(i.ops[2]).astype(np.uint64), w.vread(i.ops[3]).astype(np.uint64)
        w.vwrite(i.ops[0], ((a - b - cin) & np.uint64(MASK32)).astype(np.uint32))
        w.mask_write(i.ops[1], b + cin > a)

    def op_v_subbrev_co_u32(self, w, i):
        cin = w.mask_read(i.ops[4]).astype(np.uint64)
        a, b = w.vread(i.ops[2]).astype(np.uint64), w.vread(i.ops[3]).astype(np.uint64)
        w.vwrite(i.ops[0], ((b - a - cin) & np.uint64(MASK32)).astype(np.uint32))
        w.mask_write(i.ops[1], a + cin > b)

    # compares: e32 writes VCC, e64 names its destination
    def _vcmp(self, w, i, kind, f):
        if i.op.endswith("_e64") or len(i.ops) == 3:
            dst, a, b = i.ops[0], i.ops[1], i.ops[2]
        else:
            dst, a, b = Operand("vcc", 0, 2), i.ops[-2], i.ops[-1]
        if kind == "u32":
            x, y = w.vread(a), w.vread(b)
        elif kind == "i32":
            x, y = w.vread(a).view(np.int32), w.vread(b).view(np.int32)
        elif kind == "u64":
            x, y = w.vread64(a), w.vread64(b)
        elif kind == "i64":
            x, y = w.vread64(a).view(np.int64), w.vread64(b).view(np.int64)
        else:
            x, y = w.fread(a), w.fread(b)
        with np.errstate(invalid="ignore"):
            w.mask_write(dst, f(x, y))


def _sext64(o: Operand, w: Wave) -> int:
    """A 64-bit scalar source: registers as they are, an inline integer sign-extended, a 32-bit literal zero-extended."""
    if o.kind == "imm":
        v = o.value
        return v & MASK64
    return w.sread(o, 64)


def _popcount32(x: np.ndarray) -> np.ndarray:
    x = x.astype(np.uint32)
    x = x - ((x >> np.uint32(1)) & np.uint32(0x55555555))
    x = (x & np.uint32(0x33333333)) + ((x >> np.uint32(2)) & np.uint32(0x33333333))
    x = (x + (x >> np.uint32(4))) & np.uint32(0x0F0F0F0F)
    return ((x * np.uint32(0x01010101)) >> np.uint32(24)).astype(np.uint32)


def _i24(x: np.ndarray) -> np.ndarray:
    v = (x & np.uint32(0xFFFFFF)).astype(np.int64)
    return np.where(v & 0x800000, v - 0x1000000, v)


def _add_compares():
    table = {"eq": lambda a, b: a == b, "ne": lambda a, b: a != b, "lg": lambda a, b: a != b, "gt": lambda a, b: a > b, "ge": lambda a, b: a >= b,
             "lt": lambda a, b: a < b, "le": lambda a, b: a <= b,
             "ngt": lambda a, b: ~(a > b), "nlt": lambda a, b: ~(a < b), "nge": lambda a, b: ~(a >= b), "nle": lambda a, b: ~(a <= b),
             "neq": lambda a, b: ~(a == b), "nlg": lambda a, b: ~(a != b), "o": lambda a, b: ~(np.isnan(a) | np.isnan(b)), "u": lambda a, b: np.isnan(a) | np.isnan(b)}
    for kind in ("u32", "i32", "u64", "i64", "f32"):
        for name, f in table.items():
            if kind != "f32" and name in ("ngt", "nlt", "nge", "nle", "neq", "nlg", "o", "u", "lg"):
                continue
            def handler(self, w, i, kind=kind, f=f):
                self._vcmp(w, i, kind, f)
            setattr(Emulator, f"op_v_cmp_{name}_{kind}", handler)


_add_compares()


# ---- vector ALU: fp32 ------------------------------------------------------------------------------------------------

def _fma(a, b, c):
    """Fused multiply-add in fp32: the product of two floats is exact in float64; one rounding to float64 of the sum, then one to fp32."""
    return (a.astype(np.float64) * b.astype(np.float64) + c.astype(np.float64)).astype(np.float32)


def op_v_add_f32(self, w, i):
    with np.errstate(all="ignore"):
        w.fwrite(i.ops[0], w.fread(i.ops[1]) + w.fread(i.ops[2]))


def op_v_sub_f32(self, w, i):
    with np.errstate(all="ignore"):
        w.fwrite(i.ops[0], w.fread(i.ops[1]) - w.fread(i.ops[2]))


def op_v_subrev_f32(self, w, i):
    with np.errstate(all="ignore"):
        w.fwrite(i.ops[0], w.fread(i.ops[2]) - w.fread(i.ops[1]))


def op_v_mul_f32(self, w, i):
    with np.errstate(all="ignore"):
        w.fwrite(i.ops[0], w.fread(i.ops[1]) * w.fread(i.ops[2]))


def op_v_fma_f32(self, w, i):
    with np.errstate(all="ignore"):
        w.fwrite(i.ops[0], _fma(w.fread(i.ops[1]), w.fread(i.ops[2]), w.fread(i.ops[3])))


def op_v_fmac_f32(self, w, i):
    with np.errstate(all="ignore"):
        w.fwrite(i.ops[0], _fma(w.fread(i.ops[1]), w.fread(i.ops[2]), w.fread(i.ops[0])))


def op_v_fmamk_f32(self, w, i):  # d = a * K + b
    with np.errstate(all="ignore"):
        w.fwrite(i.ops[0], _fma(w.fread(i.ops[1]), w.fread(i.ops[2]), w.fread(i.ops[3])))


def op_v_fmaak_f32(self, w, i):  # d = a * b + K
    with np.errstate(all="ignore"):
        w.fwrite(i.ops[0], _fma(w.fread(i.ops[1]), w.fread(i.ops[2]), w.fread(i.ops[3])))


def op_v_max_f32(self, w, i):
    w.fwrite(i.ops[0], np.fmax(w.fread(i.ops[1]), w.fread(i.ops[2])))


def op_v_min_f32(self, w, i):
    w.fwrite(i.ops[0], np.fmin(w.fread(i.ops[1]), w.fread(i.ops[2])))


def op_v_max3_f32(self, w, i):
    w.fwrite(i.ops[0], np.fmax(np.fmax(w.fread(i.ops[1]), w.fread(i.ops[2])), w.fread(i.ops[3])))


def op_v_cvt_f32_u32(self, w, i):
    w.fwrite(i.ops[0], w.vread(i.ops[1]).astype(np.float32))


def op_v_cvt_f32_i32(self, w, i):
    w.fwrite(i.ops[0], w.vread(i.ops[1]).view(np.int32).astype(np.float32))


def op_v_cvt_f32_ubyte0(self, w, i):
    w.fwrite(i.ops[0], (w.vread(i.ops[1]) & np.uint32(0xFF)).astype(np.float32))


def op_v_cvt_u32_f32(self, w, i):
    x = w.fread(i.ops[1]).astype(np.float64)
    x = np.where(np.isnan(x), 0.0, np.clip(np.trunc(x), 0.0, float(MASK32)))
    w.vwrite(i.ops[0], x.astype(np.uint64).astype(np.uint32))


def op_v_cvt_i32_f32(self, w, i):
    x = w.fread(i.ops[1]).astype(np.float64)
    x = np.where(np.isnan(x), 0.0, np.clip(np.trunc(x), -2147483648.0, 2147483647.0))
    w.vwrite(i.ops[0], x.astype(np.int64).astype(np.int32).view(np.uint32))


def op_v_rcp_f32(self, w, i):
    with np.errstate(all="ignore"):
        w.fwrite(i.ops[0], np.float32(1.0) / w.fread(i.ops[1]))


op_v_rcp_iflag_f32 = op_v_rcp_f32


def op_v_trunc_f32(self, w, i):
    w.fwrite(i.ops[0], np.trunc(w.fread(i.ops[1])))


def op_v_rndne_f32(self, w, i):
    w.fwrite(i.ops[0], np.rint(w.fread(i.ops[1])))


def op_v_floor_f32(self, w, i):
    w.fwrite(i.ops[0], np.floor(w.fread(i.ops[1])))


def op_v_exp_f32(self, w, i):  # 2^x (approximate on the chip: 1 ulp)
    with np.errstate(all="ignore"):
        w.fwrite(i.ops[0], np.exp2(w.fread(i.ops[1]).astype(np.float64)).astype(np.float32))


def op_v_log_f32(self, w, i):  # log2
    with np.errstate(all="ignore"):
        w.fwrite(i.ops[0], np.log2(w.fread(i.ops[1]).astype(np.float64)).astype(np.float32))


def op_v_sqrt_f32(self, w, i):
    with np.errstate(all="ignore"):
        w.fwrite(i.ops[0], np.sqrt(w.fread(i.ops[1])))


def op_v_ldexp_f32(self, w, i):
    with np.errstate(all="ignore"):
        w.fwrite(i.ops[0], np.ldexp(w.fread(i.ops[1]).astype(np.float64), w.vread(i.ops[2]).view(np.int32)).astype(np.float32))


def op_v_div_scale_f32(self, w, i):
    # vdst, sdst(vcc), s0, s1, s2: scaling is only needed for operands near the ends of the exponent range; none is modelled
    w.fwrite(i.ops[0], w.fread(i.ops[2]))
    w.mask_write(i.ops[1], np.zeros(64, dtype=bool))


def op_v_div_fmas_f32(self, w, i):
    with np.errstate(all="ignore"):
        w.fwrite(i.ops[0], _fma(w.fread(i.ops[1]), w.fread(i.ops[2]), w.fread(i.ops[3])))


def op_v_div_fixup_f32(self, w, i):
    # (quotient, denominator, numerator): the special cases of IEEE division restored
    q, d, n = w.fread(i.ops[1]), w.fread(i.ops[2]), w.fread(i.ops[3])
    with np.errstate(all="ignore"):
        exact = n / d
    special = ~np.isfinite(exact) | (exact == 0) | ~np.isfinite(q)
    w.fwrite(i.ops[0], np.where(special, exact, q))


# ---- matrix cores ----------------------------------------------------------------------------------------------------

def op_v_mfma_f32_32x32x2_f32(self, w, i):
    """D[32x32] = A[32x2] . B[2x32] + C: lane l supplies A[l % 32][l / 32] and B[l / 32][l % 32] and holds, in register e of 16,
    element [8 (e / 4) + 4 (l / 32) + e % 4][l % 32] of C and D.  Both products are added in fp32 one after the other."""
    if w.exec != MASK64:
        raise EmulationError("MFMA issued with lanes switched off")
    a = w.fread(i.ops[1]).reshape(2, 32)           # [k][i]
    b = w.fread(i.ops[2]).reshape(2, 32)           # [k][j]
    c_op, d_op = i.ops[3], i.ops[0]
    if c_op.kind == "imm":
        c = np.zeros((16, 64), dtype=np.float32) + np.float32(struct.unpack("<f", struct.pack("<I", c_op.value & MASK32))[0])
    else:
        ci = w.vindex(c_op)
        c = w.v[ci:ci + 16].view(np.float32).copy()
    rows = (8 * (np.arange(16) // 4) + np.arange(16) % 4)[:, None] + 4 * (LANES // 32)[None, :].astype(np.int64)   # [e][lane]
    cols = np.broadcast_to((LANES % 32).astype(np.int64)[None, :], (16, 64))
    with np.errstate(all="ignore"):
        acc = c
        for k in range(2):
            acc = _fma(a[k][rows], b[k][cols], acc)
    di = w.vindex(d_op)
    w.v[di:di + 16] = acc.view(np.uint32)


# ---- LDS -------------------------------------------------------------------------------------------------------------

def _lds_check(w, addr, nbytes, active, what):
    if not active.any():
        return
    a = addr[active].astype(np.int64)
    if int(a.max()) + nbytes > w.wg.lds_bytes or int(a.min()) < 0:
        raise EmulationError(f"LDS {what} of {nbytes} bytes at 0x{int(a.max()):x}: the workgroup has {w.wg.lds_bytes} bytes")
    if np.any(a % 4):
        raise EmulationError(f"LDS {what} at an address that is no multiple of 4")


def _ds_read(self, w, i, ndw, offsets):
    """offsets: byte offsets of the pieces (one for a plain read, two for the read2 forms), ndw dwords each."""
    base = w.vread(i.ops[1]).astype(np.int64)
    active = w.em.copy()
    values = []
    for off in offsets:
        addr = (base + off) & MASK32   # (32-bit address arithmetic: a negative base with a positive offset is in use)
        _lds_check(w, addr, 4 * ndw, active, "read")
        word = np.where(active, addr // 4, 0)
        for j in range(ndw):
            values.append(w.wg.lds32[word + j].copy())
    dst, vi = i.ops[0], w.vindex(i.ops[0])

    def done():
        for j, val in enumerate(values):
            np.copyto(w.v[vi + j], val, where=active)

    w.issue_lgkm(False, done)


def _off(i, name="offset"):
    return int(i.mods.get(name, "0"), 0)


def op_ds_read_b32(self, w, i):
    _ds_read(self, w, i, 1, [_off(i)])


def op_ds_read_b64(self, w, i):
    _ds_read(self, w, i, 2, [_off(i)])


def op_ds_read_b96(self, w, i):
    _ds_read(self, w, i, 3, [_off(i)])


def op_ds_read_b128(self, w, i):
    _ds_read(self, w, i, 4, [_off(i)])


def op_ds_read2_b32(self, w, i):
    _ds_read(self, w, i, 1, [4 * _off(i, "offset0"), 4 * _off(i, "offset1")])


def op_ds_read2_b64(self, w, i):
    _ds_read(self, w, i, 2, [8 * _off(i, "offset0"), 8 * _off(i, "offset1")])


def op_ds_read2st64_b32(self, w, i):
    _ds_read(self, w, i, 1, [4 * 64 * _off(i, "offset0"), 4 * 64 * _off(i, "offset1")])


def op_ds_read2st64_b64(self, w, i):
    _ds_read(self, w, i, 2, [8 * 64 * _off(i, "offset0"), 8 * 64 * _off(i, "offset1")])


def _ds_write(self, w, i, pieces):
    """pieces: (byte offset, data operand, dwords)"""
    base = w.vread(i.ops[0]).astype(np.int64)
    active = w.em
    for off, op, ndw in pieces:
        addr = (base + off) & MASK32
        _lds_check(w, addr, 4 * ndw, active, "write")
        word = (addr // 4)[active]
        vi = w.vindex(op)
        for j in range(ndw):
            w.wg.lds32[word + j] = w.v[vi + j][active]
    w.issue_lgkm(False, None)


def op_ds_write_b32(self, w, i):
    _ds_write(self, w, i, [(_off(i), i.ops[1], 1)])


def op_ds_write_b64(self, w, i):
    _ds_write(self, w, i, [(_off(i), i.ops[1], 2)])


def op_ds_write_b96(self, w, i):
    _ds_write(self, w, i, [(_off(i), i.ops[1], 3)])


def op_ds_write_b128(self, w, i):
    _ds_write(self, w, i, [(_off(i), i.ops[1], 4)])


def op_ds_write2_b32(self, w, i):
    _ds_write(self, w, i, [(4 * _off(i, "offset0"), i.ops[1], 1), (4 * _off(i, "offset1"), i.ops[2], 1)])


def op_ds_write2_b64(self, w, i):
    _ds_write(self, w, i, [(8 * _off(i, "offset0"), i.ops[1], 2), (8 * _off(i, "offset1"), i.ops[2], 2)])


def op_ds_write2st64_b32(self, w, i):
    _ds_write(self, w, i, [(4 * 64 * _off(i, "offset0"), i.ops[1], 1), (4 * 64 * _off(i, "offset1"), i.ops[2], 1)])


def op_ds_write2st64_b64(self, w, i):
    _ds_write(self, w, i, [(8 * 64 * _off(i, "offset0"), i.ops[1], 2), (8 * 64 * _off(i, "offset1"), i.ops[2], 2)])


def op_ds_bpermute_b32(self, w, i):
    """dst[lane] = data[(addr[lane] / 4) % 64]; a lane that is switched off supplies 0."""
    src_lane = ((w.vread(i.ops[1]) + np.uint32(_off(i))) >> np.uint32(2)) & np.uint32(63)
    data = np.where(w.em, w.vread(i.ops[2]), 0).astype(np.uint32)
    values = data[src_lane]
    active = w.em.copy()
    vi = w.vindex(i.ops[0])

    def done():
        np.copyto(w.v[vi], values, where=active)

    w.issue_lgkm(False, done)


def op_ds_swizzle_b32(self, w, i):
    raise EmulationError("ds_swizzle_b32 is not modelled")


# ---- global memory ---------------------------------------------------------------------------------------------------

def _global_address(w, vaddr: Operand, saddr: Operand, i) -> np.ndarray:
    off = int(i.mods.get("offset", "0"), 0)
    if saddr.kind == "off":
        a = w.vread64(vaddr).astype(np.int64)
    else:
        a = w.vread(vaddr).astype(np.int64) + np.int64(_s64(w.sread(saddr, 64)))
    return a + off


def _global_load(self, w, i, ndw, sub=None):
    addr = _global_address(w, i.ops[1], i.ops[2], i)
    active = w.em.copy()
    if sub == "ushort":
        vals = np.zeros((1, 64), dtype=np.uint32)
        for lane in np.nonzero(active)[0]:
            vals[0, lane] = int.from_bytes(self.mem.read(int(addr[lane]), 2, f"global load (lane {lane})"), "little")
    else:
        vals = self.mem.gather_dwords(addr, active, ndw, "global load")
    vi = w.vindex(i.ops[0])

    def done():
        for j in range(vals.shape[0]):
            np.copyto(w.v[vi + j], vals[j], where=active)

    w.issue_vm(done)


def op_global_load_dword(self, w, i):
    _global_load(self, w, i, 1)


def op_global_load_dwordx2(self, w, i):
    _global_load(self, w, i, 2)


def op_global_load_dwordx3(self, w, i):
    _global_load(self, w, i, 3)


def op_global_load_dwordx4(self, w, i):
    _global_load(self, w, i, 4)


def op_global_load_ushort(self, w, i):
    _global_load(self, w, i, 1, "ushort")


def _global_store(self, w, i, ndw):
    addr = _global_address(w, i.ops[0], i.ops[2], i)
    vi = w.vindex(i.ops[1])
    self.mem.scatter_dwords(addr, w.em, w.v[vi:vi + ndw], "global store")
    w.issue_vm(None)


def op_global_store_dword(self, w, i):
    _global_store(self, w, i, 1)


def op_global_store_dwordx2(self, w, i):
    _global_store(self, w, i, 2)


def op_global_store_dwordx3(self, w, i):
    _global_store(self, w, i, 3)


def op_global_store_dwordx4(self, w, i):
    _global_store(self, w, i, 4)


def _global_atomic(self, w, i, f):
    """With a destination (glc / sc0): vdst, vaddr, vdata, saddr; without: vaddr, vdata, saddr."""
    returns = i.ops[0].kind in ("v", "a") and len(i.ops) == 4
    ops = i.ops[1:] if returns else i.ops
    addr = _global_address(w, ops[0], ops[2], i)
    data = w.vread(ops[1])
    old = np.zeros(64, dtype=np.uint32)
    for lane in np.nonzero(w.em)[0]:   # (lane after lane: lanes may name the same address)
        cur = np.frombuffer(self.mem.read(int(addr[lane]), 4, f"global atomic (lane {lane})"), dtype=np.uint32)[0]
        old[lane] = cur
        self.mem.write(int(addr[lane]), np.uint32(f(cur, data[lane])).tobytes())
    active = w.em.copy()
    if returns:
        vi = w.vindex(i.ops[0])

        def done():
            np.copyto(w.v[vi], old, where=active)

        w.issue_vm(done)
    else:
        w.issue_vm(None)


def op_global_atomic_add(self, w, i):
    _global_atomic(self, w, i, lambda cur, d: np.uint32((int(cur) + int(d)) & MASK32))


def op_global_atomic_add_f32(self, w, i):
    def add(cur, d):
        s = np.float32(np.array([cur], dtype=np.uint32).view(np.float32)[0] + np.array([d], dtype=np.uint32).view(np.float32)[0])
        return np.array([s], dtype=np.float32).view(np.uint32)[0]
    _global_atomic(self, w, i, add)


def op_global_load_lds_dwordx4(self, w, i):
    """vaddr, saddr: lane L copies 16 bytes from global memory to LDS at M0 + instruction offset + 16 L."""
    addr = _global_address(w, i.ops[0], i.ops[1], i)
    active = w.em.copy()
    vals = self.mem.gather_dwords(addr, active, 4, "direct load to LDS")
    if "offset" in i.mods:
        raise EmulationError("a direct load to LDS with an instruction offset is not modelled")
    lds_addr = np.int64(w.m0 & 0xFFFFFF) + 16 * LANES.astype(np.int64)
    _lds_check(w, lds_addr, 16, active, "write by a direct load")
    word = (lds_addr // 4)[active]
    wg = w.wg

    def done():
        for j in range(4):
            wg.lds32[word + j] = vals[j][active]

    w.issue_vm(done)


# ---- scratch (spilled registers): private to a lane -------------------------------------------------------------------

def _scratch_address(w, vaddr: Operand, saddr: Operand, i):
    off = int(i.mods.get("offset", "0"), 0)
    base = 0 if saddr.kind == "off" else w.sread(saddr)
    lanes = np.zeros(64, dtype=np.int64) if vaddr.kind == "off" else w.vread(vaddr).astype(np.int64)
    return lanes + base + off


def _scratch_load(self, w, i, ndw):
    addr = _scratch_address(w, i.ops[1], i.ops[2], i)
    vi = w.vindex(i.ops[0])
    limit = w.scratch.shape[1]
    vals = np.zeros((ndw, 64), dtype=np.uint32)
    for lane in np.nonzero(w.em)[0]:
        a = int(addr[lane])
        if a < 0 or a + 4 * ndw > limit:
            raise EmulationError(f"scratch load at {a}: the kernel has {limit - 64} bytes per lane")
        vals[:, lane] = w.scratch[lane, a:a + 4 * ndw].view(np.uint32)
    active = w.em.copy()

    def done():
        for j in range(ndw):
            np.copyto(w.v[vi + j], vals[j], where=active)

    w.issue_vm(done)


def _scratch_store(self, w, i, ndw):
    addr = _scratch_address(w, i.ops[0], i.ops[2], i)
    vi = w.vindex(i.ops[1])
    limit = w.scratch.shape[1]
    for lane in np.nonzero(w.em)[0]:
        a = int(addr[lane])
        if a < 0 or a + 4 * ndw > limit:
            raise EmulationError(f"scratch store at {a}: the kernel has {limit - 64} bytes per lane")
        w.scratch[lane, a:a + 4 * ndw] = w.v[vi:vi + ndw, lane].copy().view(np.uint8)
    w.issue_vm(None)


def op_scratch_load_dword(self, w, i):
    _scratch_load(self, w, i, 1)


def op_scratch_load_dwordx2(self, w, i):
    _scratch_load(self, w, i, 2)


def op_scratch_load_dwordx3(self, w, i):
    _scratch_load(self, w, i, 3)


def op_scratch_load_dwordx4(self, w, i):
    _scratch_load(self, w, i, 4)


def op_scratch_store_dword(self, w, i):
    _scratch_store(self, w, i, 1)


def op_scratch_store_dwordx2(self, w, i):
    _scratch_store(self, w, i, 2)


def op_scratch_store_dwordx3(self, w, i):
    _scratch_store(self, w, i, 3)


def op_scratch_store_dwordx4(self, w, i):
    _scratch_store(self, w, i, 4)


for _name, _f in list(globals().items()):
    if _name.startswith("op_") and callable(_f):
        setattr(Emulator, _name, _f)
