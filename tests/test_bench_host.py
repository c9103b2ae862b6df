"""Host-side logic of bench.py (no GPU): the byte model of a layer step, the one-GPU rule, the
counter reduction that writes profiles/traffic.json, and the guard that keeps child processes away from
a process that already holds the device."""
import csv
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import bench  # noqa: E402
from dejavu_amd.workloads import CONFIGS  # noqa: E402


def test_algorithmic_bytes_of_a_layer_step():
    """OPT-175B layer, batch 1: 785.2 MB per step (4 K d = 201.33 MB for the MLP pair, 301.99 MB QKV,
    33.55 MB KV of the selected heads, 100.66 MB out_proj, 122.88 + 24.77 MB predictors)."""
    cfg = CONFIGS["opt-175b"]
    b = bench.algorithmic_bytes(cfg, 1)
    assert b["fc1_gather"] + b["fc2_gather"] == 4 * cfg["K"] * cfg["d"] == 201_326_592
    assert b["qkv_sparse"] == 3 * 32 * 128 * 12288 * 2 == 301_989_888
    assert b["decode_attn"] == 2 * 32 * 2048 * 128 * 2 == 33_554_432
    assert b["out_proj_sparse"] == 12288 * 32 * 128 * 2
    assert b["mlp_predictor"] == (12288 * 1000 + 1000 * 49152) * 2
    assert b["head_predictor"] == (12288 * 1000 + 1000 * 96) * 2
    assert round(sum(b.values()) / 1e6, 1) == 785.2
    # the KV read scales with the batch, the weights do not
    b8 = bench.algorithmic_bytes(cfg, 8)
    assert b8["decode_attn"] == 8 * b["decode_attn"]
    assert {k: v for k, v in b8.items() if k != "decode_attn"} == {k: v for k, v in b.items() if k != "decode_attn"}
    # flush step: QKV, KV and out_proj of all 96 heads
    assert round(bench.flush_step_bytes(cfg, 1) / 1e6, 1) == 1657.6


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2
    assert "ONE GPU" in r.stderr and r.stdout.strip() == ""


def test_no_device_held_here():
    assert bench.holds_gpu() is False


def test_traffic_reduction_scales_by_the_calibration_copy(tmp_path, monkeypatch):
    """--traffic-from: per-kernel averages of FETCH_SIZE / WRITE_SIZE, each scaled by what the same counter
    reads for the largest buffer-copy dispatch (1 GiB), in bytes per launch."""

    def write(path, counter, rows):
        with open(path, "w", newline="") as f:
            w = csv.DictWriter(f, fieldnames=["Kernel_Name", "Counter_Name", "Counter_Value"])
            w.writeheader()
            for name, value in rows:
                w.writerow({"Kernel_Name": name, "Counter_Name": counter, "Counter_Value": value})

    fetch, wr = tmp_path / "f.csv", tmp_path / "w.csv"
    qkv = "_ZN2dv17qkv_sparse_kernelILi1ELi2ELi4EEEvPKDF16_"
    # the fetch counter reads half the KiB of the copy (factor 2), the write counter reads them all
    write(fetch, "FETCH_SIZE", [("__amd_rocclr_copyBuffer", 524288.0), ("__amd_rocclr_copyBuffer", 12.0),
                                (qkv, 100.0), (qkv, 300.0)])
    write(wr, "WRITE_SIZE", [("__amd_rocclr_copyBuffer", 1048576.0), (qkv, 10.0), (qkv, 30.0)])
    out = tmp_path / "traffic.json"
    monkeypatch.setattr(bench, "TRAFFIC_JSON", str(out))
    bench.write_traffic(str(fetch), str(wr))
    doc = json.loads(out.read_text())
    assert doc["scale"]["FETCH_SIZE"] == 2.0 and doc["scale"]["WRITE_SIZE"] == 1.0
    assert doc["bytes_per_launch"] == {"opt-175b/batch1/qkv_sparse": round((200.0 * 2.0 + 20.0) * 1024)}
    assert doc["csrc_sha256"] == bench.csrc_digest()
    # a measurement is only used while the kernels' sources are the ones it was taken on
    assert bench.measured_traffic("opt-175b", 1, "qkv_sparse") == 430080
    doc["csrc_sha256"] = "0" * 64
    out.write_text(json.dumps(doc))
    assert bench.measured_traffic("opt-175b", 1, "qkv_sparse") is None


def test_committed_traffic_file_is_close_to_the_algorithmic_bytes():
    with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
        doc = json.load(f)
    want = {"qkv_sparse": 301_989_888, "qkv_window_mfma": 301_989_888, "qkv_flush_mfma": 905_969_664,
            "qkv_l2_one_token": 301_989_888, "qkv_l2_mfma": 301_989_888, "qkv_l2_flush": 905_969_664}
    for key, nbytes in want.items():
        got = doc["bytes_per_launch"][f"opt-175b/batch1/{key}"]
        assert nbytes <= got <= 1.02 * nbytes, (key, got, nbytes)
