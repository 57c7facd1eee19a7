"""Runs launches that the CPU replay recorded (REPLAY_DUMP_DIR, tests/replay/replay_runtime.cpp) through the interpreter of the
generated gfx950 code (gfx950.py) and compares what the kernel leaves in memory.  Test infrastructure."""
from __future__ import annotations

import os
import re
import subprocess
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
CSRC = os.path.join(ROOT, "tenmo_amd", "csrc")
OUT = os.path.join(ROOT, "tests", "_build", "isa")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
sys.path.insert(0, HERE)
import gfx950  # noqa: E402


def device_units():
    """name -> (extra flags, source file) of the library's translation units, as tenmo_amd/build.py compiles them."""
    sys.path.insert(0, ROOT)
    import importlib

    b = importlib.import_module("tenmo_amd.build")
    units = {"tenmo_hip": ([], "tenmo_hip.hip")}
    for bm, bn, sk in b.TILES:
        units[f"gemm_{bm}x{bn}_{sk}"] = ([f"-DTENMO_TILE_BM={bm}", f"-DTENMO_TILE_BN={bn}", f"-DTENMO_TILE_STREAMK={sk}"], "gemm_tiles.hip")
    for extra in sorted(f for f in os.listdir(CSRC) if f.endswith(".hip") and f not in ("tenmo_hip.hip", "gemm_tiles.hip")):
        units[extra[:-4]] = ([], extra)
    return b.FLAGS, units


def compile_unit(name: str, csrc: str = CSRC, out_dir: str = OUT) -> str:
    """Path of the gfx950 assembly of one unit (compiled when a source is newer)."""
    flags, units = device_units()
    extra, source = units[name]
    os.makedirs(out_dir, exist_ok=True)
    target = os.path.join(out_dir, name + ".s")
    newest = max(os.path.getmtime(os.path.join(csrc, f)) for f in os.listdir(csrc))
    if os.path.exists(target) and os.path.getmtime(target) >= newest:
        return target
    cmd = [HIPCC] + list(flags) + ["-I", os.path.join(ROOT, "include")] + extra + ["--cuda-device-only", "-S", os.path.join(csrc, source), "-o", target]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("device compile failed: " + " ".join(cmd) + "\n" + res.stderr[-3000:])
    return target


_programs = {}


def program_of(unit: str, **kw):
    key = (unit, tuple(sorted(kw.items())))
    if key not in _programs:
        _programs[key] = gfx950.parse_program(open(compile_unit(unit, **kw)).read())
    return _programs[key]


def unit_of_symbol(symbol: str) -> str:
    m = re.search(r"gemm_(smallk|panel|resident)_kernel", symbol)
    if m:
        return "gemm_" + m.group(1)
    m = re.search(r"(gemm_mfma_kernel|gemm_mfma_bsum_kernel|gemm_reduce_kernel|gemm_pair_kernel|gemm_streamk_kernel|gemm_streamk_bsum_kernel|streamk_fixup_kernel)ILi(\d+)ELi(\d+)E", symbol)
    if m:
        streamk = 1 if "streamk" in m.group(1) else 0
        return f"gemm_{m.group(2)}x{m.group(3)}_{streamk}"
    return "tenmo_hip"


_symbols = {}


def symbol_at(path: str, offset: int) -> str:
    """The function whose code starts `offset` bytes into the loaded image of `path` (offset as dladdr counts it)."""
    if path not in _symbols:
        loads = subprocess.run(["readelf", "-lW", path], capture_output=True, text=True, check=True).stdout
        first = min(int(m.group(1), 16) for m in re.finditer(r"^\s*LOAD\s+0x[0-9a-f]+\s+0x([0-9a-f]+)", loads, re.M))
        table = {}
        for line in subprocess.run(["readelf", "-sW", path], capture_output=True, text=True, check=True).stdout.splitlines():
            parts = line.split()   # Num: Value Size Type Bind Vis Ndx Name
            if len(parts) == 8 and parts[3] == "FUNC" and parts[6] != "UND":
                table[int(parts[1], 16) - first] = parts[7]
        _symbols[path] = table
    return _symbols[path][offset]


def read_memory(path: str):
    out = []
    data = open(path, "rb").read()
    at = 0
    while at < len(data):   # per allocation: address, size, number of pages written out, the byte every other page is full of; then (offset, page) each
        addr, size, pages, background = (int(x) for x in np.frombuffer(data[at:at + 32], dtype=np.uint64))
        at += 32
        buf = np.full(size, background, dtype=np.uint8)
        for _ in range(pages):
            off = int(np.frombuffer(data[at:at + 8], dtype=np.uint64)[0])
            n = min(4096, size - off)
            buf[off:off + n] = np.frombuffer(data[at + 8:at + 8 + n], dtype=np.uint8)
            at += 8 + n
        out.append((addr, buf))
    return out


def load_dump(stem: str) -> dict:
    d = {}
    for line in open(stem + ".txt"):
        key, _, value = line.rstrip("\n").partition(" ")
        d[key] = value
    d["grid"] = tuple(int(x) for x in d["grid"].split())
    d["block"] = tuple(int(x) for x in d["block"].split())
    d["args"] = bytes.fromhex(d["args"])
    d["offset"] = int(d["offset"])
    d["before"] = read_memory(stem + ".before")
    d["after"] = read_memory(stem + ".after")
    d["symbol"] = symbol_at(d["file"], d["offset"])
    return d


def launches(dump_dir: str):
    return [load_dump(os.path.join(dump_dir, f[:-4])) for f in sorted(os.listdir(dump_dir)) if f.endswith(".txt")]


def differences(got: np.ndarray, want: np.ndarray, rtol=2e-6):
    """Indices (in dwords) where two buffers differ: bit patterns that are no ordinary floats must be equal, floats agree to rtol
    of the buffer's largest magnitude (the replay and the matrix cores may add the same products in different orders)."""
    n = len(want) // 4 * 4
    g32, w32 = got[:n].view(np.uint32), want[:n].view(np.uint32)
    bad = np.nonzero(g32 != w32)[0]
    if len(bad) == 0:
        return bad
    gf, wf = g32.view(np.float32), w32.view(np.float32)
    ordinary = np.isfinite(wf) & ((w32 & 0x7F800000) != 0) | (w32 == 0) | (w32 == 0x80000000)
    scale = float(np.max(np.abs(wf[ordinary]))) if ordinary.any() else 1.0
    with np.errstate(all="ignore"):
        close = ordinary[bad] & np.isfinite(gf[bad]) & (np.abs(gf[bad].astype(np.float64) - wf[bad].astype(np.float64)) <= rtol * max(scale, 1e-30))
    return bad[~close]


def across_4gib(buffers, args: bytes):
    """New addresses for the buffers, each placed so that a multiple of 4 GiB falls into its middle (keeping its alignment within a page),
    and the argument block with every pointer into a buffer moved along.  Host allocations never lie like that; device allocations can,
    and then every 64-bit address computation of the kernel has to carry."""
    placed, moved = [], bytearray(args)
    for n, (addr, data) in enumerate(buffers):
        half = (len(data) // 2) // 4096 * 4096
        placed.append(((n + 2) << 34) + (1 << 32) - half - (4096 if len(data) > 4096 and half == 0 else 0) + addr % 4096)
    for off in range(0, len(args) - 7, 8):
        value = int.from_bytes(args[off:off + 8], "little")
        for (addr, data), new in zip(buffers, placed):
            if addr <= value <= addr + len(data) and value > 0xFFFF:
                moved[off:off + 8] = (value - addr + new).to_bytes(8, "little")
                break
    return placed, bytes(moved)


def run_launch(d: dict, late=True, program=None, max_steps=50_000_000, reverse=False, relocate=False):
    """Executes the recorded launch on the generated code; returns (emulator, list of (address, differing dword indices)).
    relocate: with the buffers moved across 4 GiB boundaries (see across_4gib)."""
    prog = program or program_of(unit_of_symbol(d["symbol"]))
    if d["symbol"] not in prog:
        raise KeyError(f"{d['symbol']} is not in the unit {unit_of_symbol(d['symbol'])}")
    mem = gfx950.Memory()
    bases, args = ([addr for addr, _ in d["before"]], d["args"]) if not relocate else across_4gib(d["before"], d["args"])
    for base, (_addr, data) in zip(bases, d["before"]):
        mem.map(base, data.copy())
    emu = gfx950.Emulator(prog, mem, late=late, reverse=reverse)
    emu.launch(d["symbol"], d["grid"], d["block"], args, max_steps=max_steps)
    wrong = []
    for (addr, want), got in zip(d["after"], mem.buffers):
        bad = differences(got, want)
        if len(bad):
            wrong.append((addr, bad))
    return emu, wrong


def compile_all(names=None):
    """Every unit (or the named ones) compiled in parallel; name -> path of its assembly."""
    from concurrent.futures import ThreadPoolExecutor

    _flags, units = device_units()
    names = list(names or units)
    with ThreadPoolExecutor(max_workers=min(len(names), int(os.environ.get("MAX_JOBS", os.cpu_count() or 1)))) as pool:
        return dict(zip(names, pool.map(compile_unit, names)))


def replay_and_emulate(job):
    """(index, CUs, case of tests/replay/replay_gemm_main.cpp, dump directory) -> (case, [(kernel symbol, instructions, verdict)]):
    the case runs on the CPU replay, which records its launches, and every launch then runs on the generated code; 'ok' means
    that every device allocation holds what the replay left there."""
    import shutil

    index, cus, case, root, exe = job[:5]
    reverse = bool(job[5]) if len(job) > 5 else False
    relocate = bool(job[6]) if len(job) > 6 else False
    d = os.path.join(root, str(index))
    shutil.rmtree(d, ignore_errors=True)
    os.makedirs(d)
    r = subprocess.run([exe, "early", case], env=dict(os.environ, REPLAY_CUS=str(cus), REPLAY_DUMP_DIR=d), capture_output=True, text=True)
    if r.returncode != 0:
        return case, [("-", 0, "the replay failed: " + (r.stdout[-500:] + r.stderr[-500:]))]
    out = []
    for launch in launches(d):
        try:
            emu, wrong = run_launch(launch, reverse=reverse, relocate=relocate)
            verdict = "ok" if not wrong else "wrong values in " + ", ".join(f"{len(b)} dwords of the buffer at 0x{a:x}" for a, b in wrong)
            out.append((launch["symbol"], sum(emu.opcode_counts.values()), verdict))
        except (gfx950.EmulationError, KeyError) as e:
            out.append((launch["symbol"], 0, "error: " + str(e)[:1500]))
    shutil.rmtree(d, ignore_errors=True)
    return case, out
