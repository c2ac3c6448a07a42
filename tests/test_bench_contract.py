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
    assert set(bench.ALSO) | set(bench.ALSO_FULL) <= set(bench.WORKLOADS) and set(bench.TRAFFIC) <= set(bench.WORKLOADS)
    # the default run: the cases the targets are stated on, the decode layer and the plain-read yardsticks -- and no
    # measurement aid (timelines, cut-off builds, stand-ins run only when named)
    assert bench.ALSO[-3:] == ["llama8b-prefill512-d4096", "qwen1.5b-decode-32k", "qwen7b-decode-32k"]
    assert set(bench.TARGETS) <= set(bench.ALSO) and bench.ALSO_CPU <= set(bench.ALSO)
    for name in bench.ALSO + bench.ALSO_FULL:
        assert bench.WORKLOADS[name][1] not in ("patterns", "handoff", "timeline", "cutoffs"), name
    assert bench.TRAFFIC and bench.TRAFFIC_COMMIT
    assert bench.PEAK_FLOPS == 2.5e15 and bench.PEAK_BYTES == 8.0e12


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0
    assert "one GPU" in (r.stderr + r.stdout)


def _stub_results():
    """Results shaped like the workloads' own (long notes and tables included), with made-up figures."""
    note = "launch_us: median of event pairs around single launches; " * 4
    prefill = dict(
        value=412.285851390437, unit="TFLOP/s", ms_per_step=0.8752794500004768,
        config=dict(workload="qwen1.5b-prefill512", shape="H12 G2 d128", layers=28, n_ctx=4096, chunks=[[0, 512], [3584, 512]],
                    flops_per_step=360865333248.0, launch="graph"),
        roofline=dict(bound="mfma", achieved=480.6225248967953, peak=2500.0, unit="TFLOP/s", frac=0.19224900995871813,
                      traffic=23301120, kernel="fa_prefill_kernel<128, ...> at P=3584 B=512", launch_us=25.136500597000122,
                      launch_us_back_to_back=24.247728713921138, flops_per_launch=12081168384.0, note=note,
                      traffic_measured_at_commit="77b7d84"),
        per_chunk=[dict(P=0, B=512, launch_us=8.07, tflops=99.9, frac=0.0399), dict(P=3584, B=512, launch_us=24.2, tflops=498.2, frac=0.199)],
        eager=dict(ms_per_step=0.91), graph=dict(ms_per_step=0.87),
        parity=dict(err_row=0.00045254957090506975, err_floor1pct=0.025632332290051376, rel_l2=0.00030701345331727545, rows="worst over ... " * 10),
        cpu_baseline=dict(value=0.0035616134711669617, unit="TFLOP/s", cores=1, kind="port", sample="2265 query tokens x 12 heads ... " * 8,
                          all_cores=dict(value=0.013, unit="TFLOP/s", cores=16, sample="every row ... " * 8)))
    also = []
    for name in bench.ALSO:
        kind = bench.WORKLOADS[name][1]
        rf = dict(bound="hbm", achieved=3050.123456789, peak=8000.0, unit="GB/s", frac=0.38126543209, traffic=35370000,
                  kernel="some kernel<128> + another kernel<128> (one layer)", launch_us=10.98765, bytes_per_launch=33566720.0, note=note)
        par = dict(err_row=3.1234567e-05, err_floor1pct=0.00054321, rel_l2=1e-5, rows="all heads of all layers " * 5)
        r = dict(value=3021.5, unit="GB/s", ms_per_step=0.31, config=dict(workload=name, shape="H12 G2 d128", layers=28),
                 roofline=rf, parity=par, eager=dict(ms_per_step=0.4, device_ms_per_step=0.39), graph=dict(ms_per_step=0.31, device_ms_per_step=0.30))
        if kind == "decode":
            r["cpu_baseline"] = dict(value=0.57, unit="GB/s", cores=1, kind="port", sample="64 decode steps " * 6)
        if kind == "decode_layer":
            rf.update(layer_us=34.554907, layer_frac=0.2297968, layer_us_reference_call_sequence=61.0123,
                      launches={f"launch {i}": dict(us=5.0, MB=3.2, GBps=1000.0) for i in range(6)})
        if kind == "read":
            rf.update(launch_us_by_shape={"16_loads_per_thread": 6.4, "4_loads_per_thread": 6.5}, tiny_kernel_launch_to_launch_us=1.65)
            r["parity"] = None
        also.append(r)
    return prefill, also


def test_the_last_line_is_compact_and_carries_the_measurement():
    """The driver parses the last stdout line: it has to stay small whatever the workloads put into their results."""
    import json

    main, also = _stub_results()
    line = bench.compact_line(main, also, 20, 5)
    text = json.dumps(line)
    assert len(text) < 4096, len(text)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "parity", "targets"):
        assert key in line, key
    assert line["config"]["workload"] == "qwen1.5b-prefill512" and "model" not in line["config"]
    assert line["roofline"]["frac"] == 0.1922 and line["roofline"]["bound"] == "mfma" and "note" not in line["roofline"]
    assert line["roofline"]["traffic"] == 23301120
    assert line["cpu_baseline"]["cores"] == 1 and line["cpu_baseline"]["kind"] == "port" and len(line["cpu_baseline"]["sample"]) <= 160
    assert set(line["targets"]) == set(bench.TARGETS)
    assert line["targets"]["qwen1.5b-decode-32k"]["frac"] == 0.3813 and line["targets"]["qwen1.5b-decode-32k"]["cpu_1core"] == 0.57
    assert line["targets"]["qwen1.5b-decode-layer-32k"]["layer_us"] == 34.55
    assert json.loads(text) == line
    # without the other workloads (--no-also) the line is still whole
    assert "targets" not in bench.compact_line(main, [], 20, 5)
