"""The in-launch K-slice reduction of the column kernels (tenmo_amd/csrc/gemv.hpp, cols_join_slices) depends on memory
ordering between workgroups that no CPU run can show: a workgroup's partial sums must have left its caches before it
counts itself in, and the workgroup that arrives last must not be served stale lines when it reads the others' sums.
The source says so with __threadfence(); this test checks what the compiler made of it in the gfx950 ISA of a joined
instantiation, in program order:

    global stores (the partial sums) ... buffer_wbl2 sc1 + s_waitcnt vmcnt(0) ... s_barrier ... global_atomic_add (the arrival)
    ... s_barrier ... buffer_inv sc1 ... global loads (the slices) ... global stores (the result)

and that the instantiations without the join contain none of it.
"""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "tenmo_amd", "csrc")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

UNIT = """
#include <hip/hip_runtime.h>
#include "gemm_index.hpp"
#include "gemv.hpp"
namespace tenmo {
template __global__ void cols_kernel<4, true, true>(const ColsArgs);
template __global__ void cols_kernel<4, true, false>(const ColsArgs);
template __global__ void cols_shift_kernel<4, true>(const ColsArgs);
}
"""


def kernel_bodies(text):
    return {m.group(1): m.group(2).splitlines() for m in re.finditer(r"^(_Z\w+):\s*; @\1\n(.*?)\n\s*s_endpgm", text, re.S | re.M)}


def first(lines, pattern, start=0):
    rx = re.compile(pattern)
    for i in range(start, len(lines)):
        if rx.search(lines[i]):
            return i
    return -1


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="no hipcc")
def test_fences_stand_where_the_join_needs_them(tmp_path):
    src, out = tmp_path / "join_unit.hip", tmp_path / "join_unit.s"
    src.write_text(UNIT)
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-Wno-unused-result", "-I", os.path.join(ROOT, "include"), "-I", CSRC, "--cuda-device-only", "-S", str(src), "-o", str(out)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-3000:]
    bodies = kernel_bodies(out.read_text())
    joined = [n for n in bodies if n.endswith("Lb1EEEvNS_8ColsArgsE")]  # last template argument true
    plain = [n for n in bodies if n.endswith("Lb0EEEvNS_8ColsArgsE")]
    assert len(joined) == 2 and len(plain) == 1, sorted(bodies)
    for name in plain:
        assert not [l for l in bodies[name] if re.search(r"buffer_wbl2|buffer_inv|global_atomic", l)], name
    for name in joined:
        lines = bodies[name]
        arrive = first(lines, r"\bglobal_atomic_add\b")
        assert arrive > 0 and first(lines, r"\bglobal_atomic", arrive + 1) < 0, name  # one arrival
        # release: the last write-back before the arrival follows every store of partial sums, is waited for, and a
        # workgroup barrier stands between it and the arrival
        release = max(i for i in range(arrive) if re.search(r"\bbuffer_wbl2 sc1", lines[i]))
        assert not [i for i in range(release, arrive) if re.search(r"\bglobal_store", lines[i])], name
        assert first(lines, r"\bglobal_store", 0) < release, name
        assert re.search(r"s_waitcnt.*vmcnt\(0\)", lines[release + 1]), lines[release:release + 3]
        assert 0 < first(lines, r"\bs_barrier\b", release) < arrive, name
        # acquire: behind the arrival a barrier, then an invalidate, before the first load of a slice
        barrier = first(lines, r"\bs_barrier\b", arrive)
        acquire = first(lines, r"\bbuffer_inv sc1", barrier)
        load = first(lines, r"\bglobal_load_dword", acquire)
        assert arrive < barrier < acquire < load, (name, arrive, barrier, acquire, load)
        assert not [i for i in range(arrive, acquire) if re.search(r"\bglobal_load_dword", lines[i])], name
        assert first(lines, r"\bglobal_store", load) > load, name  # the joined result is stored
