"""What the driver relies on in bench.py without running a model: more than one GPU is
refused with one line and exit status 2, and the byte and flop counts that price the step."""

import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_one_line():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2", "--steps", "1", "--warmup", "0"],
                          capture_output=True, text=True, timeout=120)
    assert proc.returncode == 2
    assert len(proc.stdout.strip().splitlines()) == 1 and "one GPU" in proc.stdout


def test_bytes_and_flops_of_the_headline_shape():
    sys.path.insert(0, ROOT)
    import bench

    class Spec:
        run_order = range(16)

    class Model:
        spec = Spec()

    cfg = bench.LLAMA_1B
    # weights 2.47 GB (16 layers of 60.8 M parameters and the tied table of 262.7 M, bfloat16) and
    # 32 KiB of cache a token: batch 8 at 8,192 tokens reads 4.62 GB a step
    total = bench.decode_bytes(Model(), cfg, 8, 8192, 2)
    assert abs(total - (2.4715e9 + 8 * 8192 * 32768)) < 2e6
    # a 2,048-token prompt: 3.99 TFLOP in the layers' products, 0.28 in causal attention, and the head on one row
    flops = bench.prefill_flops(cfg, 16, 2048)
    assert abs(flops - (2 * 2048 * 16 * 60.817e6 + 16 * 4 * 32 * 64 * 2048 * 2049 / 2 + 2 * 128256 * 2048)) < 2e9
    assert len(bench.SHAPES) == 3 and bench.SHAPES["1b"][1] is cfg
