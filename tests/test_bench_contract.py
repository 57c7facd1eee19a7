"""bench.py's one JSON line and __graft_entry__.smoke(), checked without a GPU: both run end to end against the CPU replay
of the library (tests/replay: the timings mean nothing there, the code path, the fields and the parity checks do)."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests", "replay"))
import build as replay_build  # noqa: E402

pytestmark = pytest.mark.skipif(not replay_build.available(), reason="no host clang++ at " + replay_build.CXX)

RUNNER = """
import runpy, sys
import torch_on_host  # torch's cuda allocations on the host (tests/replay)
sys.argv = ["bench.py"] + sys.argv[1:]
runpy.run_path("bench.py", run_name="__main__")
"""


def run_bench(*flags):
    env = dict(os.environ, TENMO_HIP_LIBRARY=replay_build.build_library(), REPLAY_STRICT="0",
               PYTHONPATH=os.path.join(ROOT, "tests", "replay") + os.pathsep + os.environ.get("PYTHONPATH", ""))
    return subprocess.run([sys.executable, "-c", RUNNER] + list(flags), cwd=ROOT, env=env, capture_output=True, text=True, timeout=900)


@pytest.mark.parametrize("mode", ["children", "single-process"])
def test_one_json_line_with_every_field(mode):
    """Both ways of running it: the default (a coordinating process and one child per phase; here the children are started
    through the same wrapper that puts torch's device on the host) and everything in one process."""
    import shlex

    how = ["--single-process"] if mode == "single-process" else ["--worker-launcher", " ".join(shlex.quote(a) for a in [sys.executable, "-c", RUNNER])]
    res = run_bench("--size", "256", "--steps", "2", "--warmup", "1", "--rows", "no-such-row", "--mlp-fused-tail", "--clock-probe-rounds", "4",
                    "--sweep", "gemm_panel=0;gemm_panel=1,gemm_smallk=0", *how)
    lines = [l for l in res.stdout.splitlines() if l.strip()]
    assert res.returncode == 0 and len(lines) == 1, res.stdout[-2000:] + res.stderr[-2000:]
    out = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline", "dtype",
                "data", "config", "roofline", "cpu_baseline"):
        assert key in out, key
    assert out["n_gpus"] == 1 and out["steps"] == 2 and out["warmup"] == 1 and out["dtype"] == "f32" and out["vs_baseline"] is None
    assert out["unit"] == "TFLOP/s" and out["higher_is_better"] is True and "workload" in out["config"] and "model" not in out["config"]
    roof = out["roofline"]
    assert roof["bound"] == "mfma" and roof["unit"] == "TFLOP/s" and roof["peak"] == 157.3 and abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert "traffic" in roof and "effective_mhz" in roof
    cpu = out["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["unit"] == "TFLOP/s" and cpu["cores"] >= 1 and cpu["value"] > 0 and cpu["sample"]
    extra = out["extra"]
    assert extra["rows"] == [] and "mlp_step_ms_gpu" in extra and "mlp_step_ms_gpu_fused_tail" in extra and "mlp_step_ms_gpu_fused_tail_and_first" in extra and "mlp_step_ms_cpu" in extra
    assert extra["mlp_max_abs_loss_diff"] <= 1e-4 and extra["mlp_parity_steps"] >= 20 and out["gates"]["mlp_loss_ok"] and out["gates"]["rel_err_ok"]
    assert extra["sweep"] == [{"tune": {"gemm_panel": 0}, "rows": []}, {"tune": {"gemm_panel": 1, "gemm_smallk": 0}, "rows": []}]
    assert not [k for k in extra if k.endswith("_error")], extra


def test_more_than_one_gpu_is_refused():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert res.returncode != 0 and "ONE GPU" in (res.stdout + res.stderr)


def test_smoke_entry_runs_on_the_replay():
    env = dict(os.environ, TENMO_HIP_LIBRARY=replay_build.build_library(), REPLAY_STRICT="0",
               PYTHONPATH=os.path.join(ROOT, "tests", "replay") + os.pathsep + os.environ.get("PYTHONPATH", ""))
    res = subprocess.run([sys.executable, "-c", "import torch_on_host, __graft_entry__ as g; g.smoke()"], cwd=ROOT, env=env, capture_output=True, text=True,
                         timeout=900)
    assert res.returncode == 0 and "smoke ok" in res.stdout, res.stdout[-2000:] + res.stderr[-2000:]


def test_a_dying_row_does_not_take_the_headline_with_it():
    """The phase that measures the rows dies of a signal after one row (here: a wrapper that kills itself): the line still
    carries the headline, the row that was finished and where it stopped; the CPU baseline is still measured, but
    nothing more is started on the GPU (no MLP step), and the exit status says that something went wrong."""
    import shlex

    dying = ("import sys, os, json, signal\n"
             "if sys.argv[sys.argv.index('--phase') + 1] == 'rows':\n"
             "    print(json.dumps({'row_done': {'name': 'only_row', 'us': 1.0, 'frac': 0.5, 'rel_err_vs_fp64': 1e-7}}), flush=True)\n"
             "    os.kill(os.getpid(), signal.SIGSEGV)\n") + RUNNER
    res = run_bench("--size", "256", "--steps", "2", "--warmup", "1", "--clock-probe-rounds", "4",
                    "--worker-launcher", " ".join(shlex.quote(a) for a in [sys.executable, "-c", dying]))
    lines = [l for l in res.stdout.splitlines() if l.strip()]
    assert res.returncode != 0 and len(lines) == 1, res.stdout[-2000:] + res.stderr[-2000:]
    out = json.loads(lines[0])
    assert out["value"] > 0 and out["roofline"]["frac"] > 0 and out["cpu_baseline"]["value"] > 0
    assert [r["name"] for r in out["extra"]["rows"]] == ["only_row"] and "status -11" in out["extra"]["rows_error"]
    assert "mlp_step_ms_gpu" not in out["extra"] and out["gates"]["measurements_ok"] is False
