"""bench.py's refusals, which need no GPU: more than one GPU, and a profiled run whose graphs would hold more kernel
nodes than any profiled run has survived."""
import os
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parents[1]


def run_bench(*flags, env=None):
    full = dict(os.environ)
    full.update(env or {})
    return subprocess.run([sys.executable, str(ROOT / "bench.py"), *flags], capture_output=True, text=True, env=full, timeout=120)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = run_bench("--gpus", "2")
    assert r.returncode != 0 and "one GPU" in r.stderr


def test_profiled_runs_keep_their_graphs_small():
    """Under a profiler's tracer (recognised by its environment) a run that would instantiate graphs of more than 512
    kernel nodes exits before it touches the GPU, and says what to change; the profile commands' own settings pass
    this check (they then fail further on for want of a GPU here, which is not what is tested)."""
    tracer = {"ROCPROFILER_REGISTER_FORCE_LOAD": "1"}
    r = run_bench("--workload", "q4k_decode", "--steps", "2000", env=tracer)
    assert r.returncode != 0 and "kernel nodes" in r.stderr and "--skip-stages" in r.stderr
    r = run_bench("--workload", "q4k_verify4", "--steps", "256", env=tracer)          # four kernels a forward and their stage plans
    assert r.returncode != 0 and "kernel nodes" in r.stderr
    for workload, steps in (("q4k_verify4", "256"), ("q4k_decode", "256"), ("q4k_prefill1024", "20")):
        r = run_bench("--workload", workload, "--steps", steps, "--skip-stages", env=tracer)
        assert "kernel nodes" not in r.stderr
    # the 48-layer stack replays a token and two 2048-token chunks through every layer: never under a tracer as it is
    r = run_bench("--workload", "q4k_stack48", "--steps", "3", "--skip-stages", env=tracer)
    assert r.returncode != 0 and "kernel nodes" in r.stderr
    r = run_bench("--workload", "q4k_stack48", "--steps", "3", "--layers", "8", "--skip-stages", env=tracer)
    assert "kernel nodes" not in r.stderr
