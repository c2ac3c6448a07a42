"""bench.py on the CPU: the work formulas it prices the kernels with, its workload table and its
refusal to run on more than one GPU (no GPU is touched)."""
import os
import subprocess
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402


def test_prefill_flops_is_the_causal_exact_count():
    # brute force: token t of the chunk sees n_past + t + 1 keys; 2 products of d MACs per (query head, key)
    for H, d, P, B in [(12, 128, 0, 512), (32, 128, 4096, 512), (3, 64, 7, 5)]:
        brute = sum(4 * d * H * (P + t + 1) for t in range(B))
        assert bench.prefill_flops(H, d, P, B) == brute
    # the per-launch figures of the named configurations (Llama-3-8B at depth 4096, Qwen2.5-1.5B at depth 3584)
    assert abs(bench.prefill_flops(32, 128, 4096, 512) / 1e9 - 36.51) < 0.01
    assert abs(bench.prefill_flops(12, 128, 3584, 512) / 1e9 - 12.08) < 0.01


def test_decode_bytes_counts_k_and_v_once_plus_q_and_out():
    for H, G, d, L in [(12, 2, 128, 32768), (28, 4, 128, 32767), (32, 8, 128, 8192)]:
        assert bench.decode_bytes(H, G, d, L) == 2 * (G * L * d * 2) + 2 * H * d * 4
    assert abs(bench.decode_bytes(12, 2, 128, 32768) / 1e6 - 33.57) < 0.01


def test_workload_table_is_consistent():
    assert bench.WORKLOADS["qwen1.5b-prefill512"][3] == [(0, 512), (3584, 512)]   # the configuration the metric is quoted on
    for name, (shape, kind, n_ctx, spec) in bench.WORKLOADS.items():
        assert kind in ("prefill", "decode", "decode_store", "decode_rope_store", "copy", "read", "patterns", "logits", "handoff", "timeline", "cutoffs", "kv_store", "kv_shift", "rope", "decode_layer"), name
        if kind == "prefill":
            assert all(P + B <= n_ctx for P, B in spec), name
        if kind in ("decode", "decode_store"):
            assert 1 <= spec <= n_ctx, name
        if shape is not None:
            s = bench.SHAPES[shape]
            assert s["H"] % s["G"] == 0 and s["d"] in (64, 128), name
    assert set(bench.ALSO) <= set(bench.WORKLOADS) and set(bench.TRAFFIC) <= set(bench.WORKLOADS)
    # the cases the targets are stated on close the line, and the recorded traffic names its commit
    assert bench.ALSO[-3:] == ["llama8b-prefill512-d4096", "qwen1.5b-decode-32k", "qwen7b-decode-32k"]
    assert set(bench.TARGETS) <= set(bench.ALSO) and bench.ALSO_CPU <= set(bench.ALSO)
    assert bench.TRAFFIC and bench.TRAFFIC_COMMIT
    assert bench.PEAK_FLOPS == 2.5e15 and bench.PEAK_BYTES == 8.0e12


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0
    assert "one GPU" in (r.stderr + r.stdout)
