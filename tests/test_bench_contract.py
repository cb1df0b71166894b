"""The benchmark's command line where it can be checked without a GPU: more than
one GPU is refused with one line and exit code 2, and its byte and flop counts
are those of the configuration it names."""
import os
import subprocess
import sys

from conftest import ROOT


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2
    lines = [ln for ln in r.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]


def test_bytes_and_flops_of_the_headline_configuration():
    sys.path.insert(0, ROOT)
    import bench
    from lyapunov_engine_amd.config import LlamaConfig

    cfg = LlamaConfig.from_dict(bench.MODEL)
    # 16 layers of q/k/v (3072 x 2048), o (2048 x 2048), gate, up and down (3 x 8192 x 2048), two norms;
    # the tied head once; the final norm
    per_layer = 3072 * 2048 + 2048 * 2048 + 3 * 8192 * 2048 + 2 * 2048
    assert bench.weight_bytes(cfg, 2) == (16 * per_layer + 128256 * 2048 + 2048) * 2
    assert bench.kv_bytes_per_token(cfg, 2) == 2 * 16 * 8 * 64 * 2
    T = 2048
    linear = 2 * T * (3072 * 2048 + 2048 * 2048 + 3 * 8192 * 2048)
    attention = 2 * 32 * 64 * T * T
    assert bench.prefill_flops(cfg, T) == 16 * (linear + attention) + 2 * 128256 * 2048
    assert set(bench.SHAPES) == {"1b", "3b", "8b"} and bench.SHAPES["1b"] is bench.MODEL
    for shape in bench.SHAPES.values():
        LlamaConfig.from_dict(shape)    # every shape is a valid configuration
