"""The one JSON line ``bench.py`` prints: keys, types and internal consistency of
the headline record, the ``roofline`` and ``cpu_baseline`` objects, and the refusal
of more than one GPU."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*flags, timeout=300):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *flags], capture_output=True, text=True, timeout=timeout,
                          cwd=ROOT)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _run("--gpus", "2")
    assert r.returncode != 0 and "one GPU" in (r.stderr + r.stdout) and not r.stdout.strip().startswith("{")


def test_offline_counter_rows_belong_to_the_kernels_in_this_tree():
    """The traffic / MFMA-busy figures bench.py quotes were measured offline; each row carries the kernel name and the
    hash of the kernel source it was taken on, and bench.py withholds a row that no longer matches.  The committed
    tree must not be in that state (on a 256-CU device, which is also what the host-only plan query assumes here)."""
    sys.path.insert(0, ROOT)
    import bench
    from dmf_amd import _lib
    for (kind, wname), row in bench.OFFLINE_COUNTERS.items():
        B, H, N, D, _ = bench.WORKLOADS[wname]
        assert row["kernel"] == _lib.plan(kind, B, H, N, N, D), (kind, wname)
        assert row["src"][1] == bench.source_hash(row["src"][0]), f"{kind} {wname}: counters were measured on an older {row['src'][0]}"
        text = open(os.path.join(ROOT, bench.PROFILE_FILES[(kind, wname)])).read()
        assert all(k in text for k in row["kernel"].split(" + ")), bench.PROFILE_FILES[(kind, wname)]


@pytest.mark.gpu
def test_json_line_contract():
    r = _run("--steps", "6", "--warmup", "2", "--no-extra")
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1, "stdout must carry exactly one line"
    rec = json.loads(lines[0])
    assert rec["metric"] == "attn_fwd_jvp_tflops" and rec["unit"] == "TFLOP/s" and rec["higher_is_better"] is True
    assert (rec["n_gpus"], rec["steps"], rec["warmup"]) == (1, 6, 2)
    assert rec["dtype"] == "bf16" and rec["data"] == "synthetic" and rec["scaling"] == "weak" and rec["vs_baseline"] is None
    cfg = rec["config"]
    assert "workload" in cfg and "model" not in cfg and "N=1024" in cfg["workload"] and "D=72" in cfg["workload"]
    # value = algorithmic FLOPs per step / measured time per step
    assert abs(rec["value"] - cfg["flops_per_step"] / (rec["ms_per_step"] * 1e-3) / 1e12) <= 1e-6 * rec["value"]
    assert cfg["flops_per_step"] == 12 * 64 * 16 * 1024 * 1024 * 72
    roof = rec["roofline"]
    assert roof["bound"] == "mfma" and roof["unit"] == "TFLOP/s" and roof["peak"] == 2500.0
    assert abs(roof["achieved"] - rec["value"]) <= 1e-9 * rec["value"] and abs(roof["frac"] - roof["achieved"] / roof["peak"]) <= 1e-12
    assert 0.9 <= roof["traffic"] / cfg["hbm_bytes_per_step"] <= 1.1          # measured HBM bytes vs algorithmic bytes
    assert 0.2 < roof["frac"] < 1.0
    cpu = rec["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["unit"] == "TFLOP/s" and cpu["cores"] >= 1 and cpu["value"] > 0 and "sample" in cpu
