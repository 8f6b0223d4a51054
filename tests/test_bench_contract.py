"""bench.py's command-line contract: one GPU only, one JSON line with the agreed keys."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def _run(*args, env=None):
    return subprocess.run([sys.executable, BENCH, *args], capture_output=True, text=True, cwd=ROOT,
                          env={**os.environ, **(env or {})}, timeout=600)


def test_more_than_one_gpu_is_refused():
    proc = _run("--gpus", "2")
    assert proc.returncode != 0
    assert "one GPU" in proc.stderr


def test_world_size_above_one_is_refused():
    proc = _run(env={"WORLD_SIZE": "2"})
    assert proc.returncode != 0
    assert "one GPU" in proc.stderr


@pytest.mark.gpu
def test_json_line_has_the_contract_keys():
    proc = _run("--workload", "qwen2.5-0.5b", "--steps", "2", "--warmup", "1", "--cpu-sample-tokens", "64",
                "--no-hbm-kernels")
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = [l for l in proc.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
                "scaling", "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 2 and d["warmup"] == 1
    assert d["unit"] == "tokens/s" and d["higher_is_better"] is True and d["vs_baseline"] is None
    assert d["dtype"] == "bf16" and d["data"] == "synthetic" and "workload" in d["config"]
    r = d["roofline"]
    assert r["bound"] == "mfma" and r["unit"] == "TFLOP/s" and r["peak"] == 2500.0
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-12 and 0.0 < r["frac"] < 1.0
    c = d["cpu_baseline"]
    assert c["kind"] == "port" and c["unit"] == "tokens/s" and c["cores"] >= 1 and c["value"] > 0
    assert d["value"] > 0 and d["ms_per_step"] > 0


def test_kernel_names_quoted_by_the_bench_exist_in_the_library():
    # the roofline object names its kernels; a renamed kernel must not leave a stale label behind
    sys.path.insert(0, ROOT)
    import bench
    from areal_amd import _lib

    for name in (bench.KERNEL_FWD_SAVE, bench.KERNEL_FWD, bench.KERNEL_RECOMPUTE, bench.KERNEL_DHIDDEN,
                 bench.KERNEL_DWEIGHT):
        assert _lib.has_kernel(name), name
    assert not _lib.has_kernel("gemm16_sweep<9, Store16<false, 0> >")
    for name in ("gae_owned_kernel", "gae_tile_kernel", "loss_token_kernel", "loss_finalize_kernel", "rows_fwd_kernel",
                 "saved_prep_kernel", "lmhead_merge_kernel", "lmhead_rowref_kernel"):
        assert _lib.has_kernel(name), name
