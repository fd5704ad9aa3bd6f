"""The command-line contract of bench.py: one JSON line with the agreed keys, one GPU only."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr
    assert r.stdout.strip() == ""


@pytest.mark.gpu
def test_one_json_line_with_the_agreed_keys():
    r = subprocess.run([sys.executable, BENCH, "--gpus", "1", "--steps", "10", "--warmup", "2", "--cpu-budget", "1",
                        "--backward"], capture_output=True, text=True, timeout=280)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [ln for ln in r.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 10 and d["warmup"] == 2
    assert d["vs_baseline"] is None and d["dtype"] == "f32" and d["data"] == "synthetic"
    assert set(d["config"]) >= {"workload"} and "model" not in d["config"]
    roof = d["roofline"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in roof, key
    assert roof["bound"] == "mfma" and roof["peak"] == 157.3 and roof["unit"] == "TFLOP/s"
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    cpu = d["cpu_baseline"]
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert key in cpu, key
    assert cpu["kind"] == "port" and cpu["cores"] >= 1
    # the parity gate ran on the timed buffers
    assert d["parity"]["imtrans_bit_exact"] and d["parity"]["relu_zero_mask_equal"]
    assert d["parity"]["conv_max_rel_err"] <= 1e-4
    assert d["backward"]["ms_conv_grad"] > 0 and d["backward"]["ms_imtrans_grad"] > 0


def _profile_traffic_tables():
    """(workload, precision, op) -> (kernel variant or None, FETCH_SIZE KiB, WRITE_SIZE KiB) from the committed
    rocprofv3 summaries: every table row of profiles/conv_imtrans_*.md that carries both counters."""
    import glob
    import re

    variants = {"wide48x64": "wide48x64", "wide48": "wide48", "tall16": "tall16", "short16": "short16", "ring32": "ring32", "ring16": "ring16",
                "3-ring": "stored-ring3", "4-ring": "stored-ring4", "stored-spread": "stored-spread", "stored-split4": "stored-split4",
                "stored-split`": "stored-split", "stored-tall": "stored-tall"}
    out = {}
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "conv_imtrans_*.md"))):
        file_workload = re.search(r"conv_imtrans_(cfg\w+?)_kernel_trace", os.path.basename(path))
        workload = file_workload.group(1) if file_workload else None
        precision = None
        for line in open(path, encoding="utf-8"):
            if line.startswith("## "):
                head = line[3:].strip()
                m = re.match(r"(cfg\w+)\s+(.*)", head)
                if m:
                    workload, head = m.group(1), m.group(2)
                precision = "bf16_stored" if head.startswith("bf16-stored") else "fp32" if head.startswith("fp32") else None
                continue
            cells = [c.strip() for c in line.split("|")[1:-1]]
            if len(cells) != 10 or precision is None or workload is None:
                continue
            name = cells[0]
            if name.startswith("imtrans_direct_kernel"):
                op = "imtrans"
            elif name.startswith("conv_"):
                op = "conv"
            else:
                continue
            try:
                fetch_kib, write_kib = float(cells[4]), float(cells[6])
            except ValueError:
                continue
            variant = next((v for tag, v in variants.items() if tag in name), None) if op == "conv" else None
            assert (workload, precision, op) not in out, (path, name)
            out[(workload, precision, op)] = (variant, fetch_kib, write_kib)
    return out


def test_traffic_literals_are_the_committed_profiles_figures():
    """roofline.traffic comes from literals in bench.py; each must be the FETCH_SIZE x 2.00 + WRITE_SIZE x 1.00 of
    the profile table row for the same workload, precision and kernel variant."""
    sys.path.insert(0, ROOT)
    import bench

    tables = _profile_traffic_tables()
    assert len(tables) >= 16
    for key, (variant, nbytes) in bench.MEASURED_TRAFFIC.items():
        assert key in tables, key
        t_variant, fetch_kib, write_kib = tables[key]
        assert variant == t_variant, (key, variant, t_variant)
        assert abs(nbytes - (fetch_kib * 2.00 + write_kib * 1.00) * 1024) < 1.0, key
    # and no conv row of the profiles is missing from the table in bench.py
    for key in tables:
        assert key in bench.MEASURED_TRAFFIC, key
