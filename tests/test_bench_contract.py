"""bench.py's command-line contract, as far as it can be checked without a GPU."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert p.returncode != 0
    assert "one GPU" in p.stderr


def test_traffic_records_are_consistent_and_say_what_they_were_taken_for():
    recs = json.load(open(os.path.join(ROOT, "profiles", "traffic.json")))
    assert "opt30b_ffn1_n16_s70" in recs
    for name, rec in recs.items():
        assert rec["bytes_per_launch"] == int((rec["fetch_size_kib"] * rec["fetch_scale"]
                                               + rec["write_size_kib"] * rec["write_scale"]) * 1024), name
        assert os.path.exists(os.path.join(ROOT, rec["source"])), name
        # bench.py quotes a record only for the kernel and Split_K it names
        assert rec["kernel"].startswith("spmm::spmm_bitmap_rows<") and rec["split_k"] >= 1, name


@pytest.mark.gpu
def test_bench_line_has_the_contract_fields():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--steps", "10", "--warmup", "2",
                        "--workload", "opt13b_out", "--cpu-seconds", "1", "--no-chain", "--no-qkv", "--no-sweep"],
                       capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    lines = [l for l in p.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
              "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert k in d, k
    assert d["n_gpus"] == 1 and d["steps"] == 10 and d["vs_baseline"] is None and "workload" in d["config"]
    r = d["roofline"]
    assert r["bound"] == "hbm" and r["peak"] == 8000.0 and abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-9
    # the headline fraction is the whole call's; the main kernel alone can only be faster
    assert r["main_kernel"]["frac"] >= r["frac"] * 0.98 and r["main_kernel"]["name"].startswith("spmm::spmm_bitmap_rows<")
    assert r["stream_ceiling_gbs"] is not None and 3000 < r["stream_ceiling_gbs"] < 8000
    assert r["traffic"] is None or isinstance(r["traffic"], int)
    assert d["decode_chain_opt13b"]["check"]["rel_l2"] <= 1e-3 if "decode_chain_opt13b" in d else True
    c = d["cpu_baseline"]
    assert c["kind"] == "port" and c["cores"] >= 1 and c["value"] > 0 and c["sample"]
    assert d["check"]["rel_l2"] <= 1e-3 and d["device_encoder"]["identical_to_host_encoder"]
