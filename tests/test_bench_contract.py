"""bench.py's host side without a GPU: the workloads are the configurations BASELINE.json names,
the algorithmic bytes are what the kernel's streams add up to, and a request for more than one
GPU ends with a message."""
import math
import os
import subprocess
import sys

import bench

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _count(shapes):
    return sum(math.prod(s) for _, s in shapes)


def test_workloads_are_the_named_parameter_sets():
    l3 = bench.llama3_8b_shapes()
    assert len(l3) == 291 and _count(l3) == 8030261248          # Llama-3-8B
    assert sum(math.prod(s) for _, s in l3 if math.prod(s) > 4096) == 8029995008   # the quantized ones
    l2 = bench.llama2_13b_shapes()
    assert len(l2) == 362 and _count(l2) == 13015859200          # Llama-2-13B shapes without the final norm
    g2 = bench.gpt2_small_shapes()
    assert len(g2) == 148 and _count(g2) == 124439808            # GPT-2-small, tied head not repeated
    assert bench.WORKLOADS["single-4096"][0]() == [("w", (4096, 4096))]
    for name, (_, p, g, dist, desc) in bench.WORKLOADS.items():
        assert p in bench.DTYPE_NAMES and g in bench.DTYPE_NAMES and dist in ("student_t", "normal_outliers")
        assert ("BASELINE.json configs[" in desc) == (name != "single-2p30")
    assert bench.HP == dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)


def test_algorithmic_bytes_per_parameter():
    # p read + write, g read, a nibble of each moment read + write, two fp32 scales per 128 read + write
    assert bench.bytes_per_param("float32", "bfloat16") == 12.125
    assert bench.bytes_per_param("float32", "float32") == 14.125
    assert bench.bytes_per_param("bfloat16", "bfloat16") == 8.125
    assert bench.bytes_per_param("bfloat16", "float32") == 10.125
    assert bench.bytes_per_param("float16", "float16") == 8.125
    assert bench.HBM_PEAK_GBS == 8000.0


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0 and "ONE GPU" in r.stderr and r.stdout.strip() == ""
