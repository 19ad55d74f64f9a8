"""CPU tests of bench.py's command-line contract (no GPU work is started)."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2", "--steps", "1", "--warmup", "0"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in (r.stdout + r.stderr) or "1 GPU" in (r.stdout + r.stderr) or "single" in (r.stdout + r.stderr).lower()


def test_algorithmic_bytes_of_the_headline_launch():
    sys.path.insert(0, ROOT)
    import bench

    # 16 B per (token, KV head) code + block table + query codes + one score per (block, head)
    codes = 32 * 32768 * 8 * 16
    assert bench.algorithmic_bytes() == codes + 4 * 32 * 256 + 4 * 32 * 32 * 4 + 4 * 32 * 8 * 256
    assert bench.HBM_PEAK_GBPS == 8000.0
    # the traffic figure comes from the committed counter summary and stays within 5 % of the
    # algorithmic bytes
    traffic = bench.measured_traffic()
    assert traffic is not None, "profiles/decode_step_config2_hbm_traffic_pmc.txt lacks traffic_bytes_per_launch"
    assert 1.0 <= traffic / bench.algorithmic_bytes() < 1.05
