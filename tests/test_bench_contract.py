"""What bench.py promises without needing a GPU: one GPU only (a request for more exits with a
message instead of a number), no CPU fallback when no MI355X is present, and a JSON line that
carries the agreed keys (checked on the source, since the line itself needs the GPU; the GPU
run is checked by tests/test_gpu_full_size.py's neighbours and by the driver). CPU only."""
import os
import re
import subprocess
import sys

import pytest

import kvt_amd

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def _run(*args, env=None):
    return subprocess.run([sys.executable, BENCH, *args], capture_output=True, text=True,
                          timeout=300, env=env)


def test_more_than_one_gpu_is_refused_with_a_message():
    res = _run("--gpus", "2")
    assert res.returncode != 0
    assert "ONE MI355X" in res.stderr and res.stdout.strip() == ""
    env = dict(os.environ, WORLD_SIZE="2")
    res = _run(env=env)
    assert res.returncode != 0 and "ONE MI355X" in res.stderr


@pytest.mark.skipif(kvt_amd.device_count() > 0, reason="this check is for machines without a GPU")
def test_no_device_means_no_number():
    res = _run("--steps", "1", "--warmup", "0")
    assert res.returncode != 0
    assert "no CPU fallback" in res.stderr and res.stdout.strip() == ""


def test_the_json_line_names_every_agreed_key():
    src = open(BENCH).read()
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step",
                "higher_is_better", "scaling", "vs_baseline", "dtype", "data", "config",
                "roofline", "cpu_baseline"):
        assert re.search(r'"%s"\s*:' % key, src) or re.search(r'out\["%s"\]' % key, src), key
    for key in ("bound", "achieved", "peak", "frac", "traffic"):          # roofline
        assert re.search(r'"%s"\s*:' % key, src), key
    for key in ("cores", "kind", "sample"):                                # cpu_baseline
        assert re.search(r'"%s"\s*:' % key, src), key
    assert '"workload"' in src and '"model"' not in src
    # nothing under _work/ and no reference checkout at run time
    assert "_work/" not in src and "/root/reference" not in src


def test_the_measured_hbm_traffic_belongs_to_the_kernels_as_they_are_now():
    """roofline.traffic comes from profiler counter runs and is kept in bench.py next to the
    SHA-256 of the kernel source it was measured with. A kernel change without a new counter
    run must not go unnoticed: the figures would be quoted for code they were not taken from."""
    import hashlib
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench_module", BENCH)
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    kernels = os.path.join(ROOT, "llumnix-kv_amd", "csrc", "kvt_kernels.hip")
    sha = hashlib.sha256(open(kernels, "rb").read()).hexdigest()
    if not bench.MEASURED_TRAFFIC:
        assert bench.KERNELS_SHA256 == "unmeasured"
        return
    assert bench.KERNELS_SHA256 == sha, (
        "llumnix-kv_amd/csrc/kvt_kernels.hip has changed since the FETCH_SIZE / WRITE_SIZE runs "
        "behind bench.MEASURED_TRAFFIC: take the counter runs again (profiles/*_hbm_traffic.md "
        "give the commands), or empty the table")
    for (cfg, plan), row in bench.MEASURED_TRAFFIC.items():
        assert set(row) == {"pack", "unpack"} and all(v > 0 for v in row.values()), (cfg, plan)
