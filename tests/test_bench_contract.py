"""The command line of bench.py that needs no GPU: more than one GPU is refused with a message (this build runs one model on
one device), and the workload table names the five configurations the published figures are quoted on."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "ONE GPU" in r.stderr and "--gpus 2" in r.stderr
    assert r.stdout.strip() == ""            # no JSON line that could be mistaken for a measurement


def test_workload_table():
    sys.path.insert(0, ROOT)
    import bench
    assert set(bench.CONFIGS) >= {"c0", "c1", "c2", "c3", "c4"}
    dim, layers, heads, ffn, vocab, n_prompt, steps = bench.CONFIGS["c1"]
    assert (dim, layers, heads, ffn, vocab, n_prompt, steps) == (4096, 32, 32, 11008, 32000, 128, 256)
    assert bench.CONFIGS["c2"][:4] == (5120, 40, 40, 13824) and bench.CONFIGS["c2"][5:] == (2048, 128)
    assert bench.CONFIGS["c0"][:4] == (1024, 8, 16, 2816) and bench.CONFIGS["c0"][5:] == (16, 64)
    assert bench.CONFIGS["c4"][:4] == (8192, 80, 64, 22016)
    # the recorded traffic figures name the summaries they come from, and those exist
    for cfg, path in bench.TRAFFIC_SOURCE.items():
        assert os.path.exists(os.path.join(ROOT, path)), path
        assert f"{bench.MEASURED_TRAFFIC[cfg]:,}" in open(os.path.join(ROOT, path)).read(), (cfg, bench.MEASURED_TRAFFIC[cfg])
