"""bench.py without a GPU: the parts of its contract that need none."""
import importlib.util
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2 and "one GPU" in r.stderr and r.stdout.strip() == ""


def test_traffic_figure_comes_from_the_tracked_profile_summary():
    b = _bench()
    traffic = b.measured_traffic()
    algorithmic = b.anyprec_bytes(4096, 14336)
    assert algorithmic == 22286336                       # 3 planes + LUT + activations + outputs of the roofline shape
    assert traffic is not None and algorithmic <= traffic <= 1.2 * algorithmic
    text = open(os.path.join(ROOT, "profiles", "anyprec_gemv_4096x14336_pmc.md")).read()
    assert f"traffic_bytes_per_launch: {traffic}" in text


def test_layer_set_is_the_llama3_8b_decoder():
    b = _bench()
    assert [(n, k, m) for n, k, m in b.LLAMA3_8B] == [("q", 4096, 4096), ("k", 4096, 1024), ("v", 4096, 1024), ("o", 4096, 4096),
                                                       ("gate", 4096, 14336), ("up", 4096, 14336), ("down", 14336, 4096)]
    per_token = 32 * sum(b.anyprec_bytes(k, m) for _, k, m in b.LLAMA3_8B)
    assert abs(per_token - 2.64e9) < 0.02e9              # the base bytes per token the measurement plan states
