#!/usr/bin/env python3
"""Measurement aids behind bench.py: workloads that are not the operator and never run by default.

    python bench.py --workload weights-read-patterns | decode-handoff-mock | *-timeline | *-cutoffs

They time read-only stand-ins (load patterns of a matrix-vector kernel, a split + combine hand-off), read the
wall-clock stage marks of the timeline build of the library, and time the cut-off builds of the attention kernels
(kernels with parts taken out at compile time, results wrong by design; built on request by
orin_llm_amd.build.build(probes=True)).  bench.py dispatches here by workload kind.
"""
import time

import numpy as np

from bench import PEAK_BYTES, PEAK_FLOPS, SHAPES, WORKLOADS, decode_bytes, make_layer, prefill_flops

def run_patterns(torch, kernels, name, steps, warmup, with_cpu):
    """What the load pattern of a matrix-vector kernel costs by itself: a pair of Q4_K-shaped matrices read by
    kernels that compute nothing, launched back to back in a graph over buffers that rotate through more memory than
    the last-level cache holds.  One step = 16 launches; value and roofline are the best pattern's."""
    n_rows, n_blocks = WORKLOADS[name][3]
    mat = n_rows * n_blocks * 144
    nbytes = 2 * mat
    launches = 16
    n_buf = max(launches, int(np.ceil(1.2e9 / nbytes)))
    pool = torch.empty(n_buf * nbytes, dtype=torch.uint8, device="cuda").fill_(1)
    sink = torch.zeros(128, dtype=torch.int32, device="cuda")  # (a word the kernels never write)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    names = {0: "64 B of each of 16 rows per instruction", 1: "runs of 144 B", 2: "runs of 288 B", 4: "runs of 576 B"}
    out, wall_best, best_us = {}, None, None
    for pattern, label in names.items():
        for wgs_per_cu in (2, 3):
            g = torch.cuda.CUDAGraph()
            try:
                with torch.cuda.graph(g):
                    kernels.set_stream(torch.cuda.current_stream().cuda_stream)
                    for k in range(launches):
                        kernels.bench_read_pattern(pool[(k % n_buf) * nbytes:], mat, n_rows, n_blocks, pattern, wgs_per_cu * kernels.cu_count(), sink)
            finally:
                kernels.set_stream(torch.cuda.current_stream().cuda_stream)
            for _ in range(max(1, warmup)):
                g.replay()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            e0.record()
            for _ in range(steps):
                g.replay()
            e1.record()
            torch.cuda.synchronize()
            wall = time.perf_counter() - t0
            us = e0.elapsed_time(e1) * 1e3 / (steps * launches)
            del g
            out[f"{label}, {wgs_per_cu} workgroups per CU"] = dict(us=round(us, 2), GBps=round(nbytes / (us * 1e-6) / 1e9, 1))
            if best_us is None or us < best_us:
                best_us, wall_best, best = us, wall, f"{label}, {wgs_per_cu} workgroups per CU"
    del pool
    torch.cuda.empty_cache()
    return dict(value=nbytes * launches * steps / wall_best / 1e9, unit="GB/s", ms_per_step=wall_best / steps * 1e3,
                config=dict(workload=name, shape=f"2 x {n_rows} rows x {n_blocks} blocks of 144 B", bytes_per_launch=nbytes,
                            launches_per_step=launches, buffers_rotated=n_buf),
                roofline=dict(bound="hbm", achieved=nbytes / (best_us * 1e-6) / 1e9, peak=PEAK_BYTES / 1e9, unit="GB/s",
                              frac=nbytes / (best_us * 1e-6) / PEAK_BYTES, traffic=float(nbytes),
                              kernel=f"read_pattern_kernel ({best}; reads only, not part of the path)", launch_us=best_us,
                              launch_us_by_pattern=out, bytes_per_launch=nbytes),
                parity=None)


# Stage marks of the kernels (slot, what has happened by then), in the order a wave passes them.
PREFILL_STAGES = [(0, "entry"), (9, "queries and first K tile requested"), (11, "output accumulators cleared"), (12, "first V buffer cleared"),
                  (13, "first V tile requested"), (10, "second K tile requested"),
                  (1, "queries in registers"), (2, "first two score tiles"), (3, "first weights"), (4, "main loop done"),
                  (5, "last products done, accumulators in LDS"), (7, "barrier passed"), (8, "output stored")]
GEMV_STAGES = [(0, "entry"), (1, "first two items of weights requested"), (2, "digits of the wave's part of the activation done"),
               (3, "item 0 in LDS"), (4, "item 1 in LDS"), (5, "item 2 in LDS"), (6, "item 3 in LDS"), (7, "item 4 in LDS"),
               (10, "item 7 in LDS"), (13, "tile's sums out"), (14, "exit")]
DECODE_STAGES = [(0, "entry"), (1, "position known, query pieces met, tile requests issued"), (2, "query converted"),
                 (3, "K arrived, scores of the last tile done"), (4, "V arrived, last products done"), (5, "partials in LDS"),
                 (6, "barrier passed"), (7, "partial written")]


def run_timeline(torch, kernels, name, steps, warmup, with_cpu):
    """Not a timed workload: launches the kernel from the timeline build over a few cold layers and reports, for the
    last launch, when the waves pass each stage mark (microseconds after the first wave's entry: median, earliest,
    latest).  The stamps cost a little time themselves; durations come from the ordinary library's workloads."""
    import ctypes

    shape, _, n_ctx, (what, a, batch) = WORKLOADS[name]
    if what in ("gateup", "down"):
        return run_gemv_timeline(torch, kernels, name, steps)
    sh = SHAPES[shape]
    H, G, d = sh["H"], sh["G"], sh["d"]
    L = kernels.stamps_lib()
    rc = L.orin_fa_init(0)
    assert rc == 0, rc
    L.orin_fa_set_stream(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    scale = 1.0 / float(np.sqrt(d))
    n_layers = 10  # > 256 MB of K/V at every shape: nothing is left in a cache from the launch before
    n_filled = a + batch if what == "prefill" else a
    layers = [make_layer(torch, 900 + i, H, G, d, n_ctx, min(n_filled, n_ctx), batch, sh["outliers"]) for i in range(n_layers)]
    outs = [torch.empty((batch, H, d), dtype=torch.float32, device="cuda") for _ in range(n_layers)]
    dpos = torch.tensor([a - 1], dtype=torch.int32, device="cuda")
    waves = 4 if what == "prefill" else 8
    stages = PREFILL_STAGES if what == "prefill" else DECODE_STAGES

    def launch(i):
        q, k, v = layers[i]
        if what == "prefill":
            rc = L.orin_fa_prefill(q.data_ptr(), k.data_ptr(), v.data_ptr(), outs[i].data_ptr(), H, G, d, n_ctx, a, batch, scale)
        else:
            rc = L.orin_fa_decode_ind(q.data_ptr(), k.data_ptr(), v.data_ptr(), outs[i].data_ptr(), H, G, d, n_ctx,
                                      dpos.data_ptr(), scale)
        assert rc == 0, rc

    rows = []
    host = np.zeros(1024 * waves * 16, np.int64)
    for rep in range(1 + max(1, min(steps, 5))):
        for i in range(n_layers - rep % 3):  # (the last launch of a pass is a different layer from pass to pass)
            launch(i)
        torch.cuda.synchronize()
        rc = L.orin_fa_bench_stamps(0 if what == "prefill" else 1, host.ctypes.data, host.size)
        assert rc == 0, rc
        # (the library hands the table over and clears it, so a mark that a wave did not pass reads zero: workgroups
        # beyond the launch's grid, decode workgroups the position leaves without a tile, prefill waves without one)
        t = host.reshape(1024, waves, 16)[:, :, [slot for slot, _ in stages]].astype(np.float64) * 0.01  # 100 MHz -> us
        passed = t > 0
        passed &= passed[:, :, -1:]       # waves that went all the way
        t0 = t[:, :, 0][passed[:, :, 0]].min()
        if rep > 0:                       # (the first pass only clears what earlier launches left)
            rows.append([(float(np.median(t[:, :, j][passed[:, :, j]] - t0)), float((t[:, :, j][passed[:, :, j]] - t0).min()),
                          float((t[:, :, j][passed[:, :, j]] - t0).max())) for j in range(len(stages))])
    med = np.median(np.array(rows), axis=0)
    timeline = {label: dict(median=round(float(m[0]), 2), earliest=round(float(m[1]), 2), latest=round(float(m[2]), 2))
                for (_, label), m in zip(stages, med)}
    span = float(med[-1][2])
    if what == "prefill":
        work, peak, unit, bound = prefill_flops(H, d, a, batch), PEAK_FLOPS, "TFLOP/s", "mfma"
        kern = "fa_prefill_kernel (timeline build)"
    else:
        work, peak, unit, bound = decode_bytes(H, G, d, a), PEAK_BYTES, "GB/s", "hbm"
        kern = "fa_decode_split_kernel (timeline build; the combine kernel follows it)"
    scale_u = 1e12 if what == "prefill" else 1e9
    del layers, outs
    torch.cuda.empty_cache()
    return dict(value=work / (span * 1e-6) / scale_u, unit=unit, ms_per_step=span * 1e-3,
                config=dict(workload=name, shape=f"H{H} G{G} d{d}", n_ctx=n_ctx, what=what, depth_or_length=a, batch=batch),
                roofline=dict(bound=bound, achieved=work / (span * 1e-6) / scale_u, peak=peak / scale_u, unit=unit,
                              frac=work / (span * 1e-6) / peak, traffic=None, kernel=kern, launch_us=span,
                              note="launch_us: first wave's entry to last wave's last mark in the timeline build, stamps included"),
                parity=None, timeline_us=timeline)


def run_gemv_timeline(torch, kernels, name, steps):
    """run_timeline for the matrix-vector kernel: one big product of a decode layer over cold copies of its matrices
    (random block bytes with sane scales: the kernel's time does not depend on the values)."""
    import ctypes

    _, _, _, (what, n_in, n_out) = WORKLOADS[name]
    L = kernels.stamps_lib()
    rc = L.orin_fa_init(0)
    assert rc == 0, rc
    L.orin_fa_set_stream(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    wtype, blk, d_at = (12, 144, 0) if what == "gateup" else (14, 210, 208)   # Q4_K / Q6_K: where a block keeps its fp16 scale
    n_mat = 2 if what == "gateup" else 1
    row = n_in // 256 * blk
    per = n_mat * n_out * row
    copies = max(3, int(600e6 // per))  # more than the memory-side cache holds
    g = torch.Generator(device="cuda").manual_seed(77)
    W = torch.randint(0, 255, (copies, n_mat, n_out * row), dtype=torch.uint8, device="cuda", generator=g)
    Wb = W.view(copies, n_mat, -1, blk)
    Wb[..., d_at] = 0x00
    Wb[..., d_at + 1] = 0x2c
    if what == "gateup":
        Wb[..., 2] = 0x00
        Wb[..., 3] = 0x2c
    x = torch.randn(n_in, device="cuda", generator=g)
    nw = torch.ones(n_in, device="cuda")
    y = torch.zeros(n_out, device="cuda")
    vp, ci = ctypes.c_void_p, ctypes.c_int
    L.orin_gemv_norm_gate_up_swiglu.argtypes = [ci, vp, vp, vp, vp, ctypes.c_float, vp, ci, ci]
    L.orin_gemv_multi.argtypes = [ci, ci, vp, vp, vp, vp, vp, vp, ctypes.c_float, ci, ci]

    def launch(c):
        if what == "gateup":
            rc = L.orin_gemv_norm_gate_up_swiglu(wtype, W[c, 0].data_ptr(), W[c, 1].data_ptr(), x.data_ptr(), nw.data_ptr(), 1e-5,
                                                 y.data_ptr(), n_in, n_out)
        else:
            ws, ys, ns = (vp * 1)(W[c, 0].data_ptr()), (vp * 1)(y.data_ptr()), (ci * 1)(n_out)
            rc = L.orin_gemv_multi(wtype, 1, ws, None, ys, ns, x.data_ptr(), None, 0.0, n_in, 1)
        assert rc == 0, rc

    stages = GEMV_STAGES
    rows = []
    host = np.zeros(1024 * 4 * 16, np.int64)
    for rep_ in range(1 + max(1, min(steps, 5))):
        n_run = copies - rep_ % 2
        for c in range(n_run):            # (the earlier ones push the last launch's matrices out of every cache)
            launch(c)
            torch.cuda.synchronize()      # (every launch starts on an idle chip: behind another it shares the memory with its tail)
        rc = L.orin_fa_bench_stamps(2, host.ctypes.data, host.size)
        assert rc == 0, rc
        t = host.reshape(1024, 4, 16)[:, :, [slot for slot, _ in stages]].astype(np.float64) * 0.01  # 100 MHz -> us
        passed = t > 0                    # (a wave with fewer items leaves the later item marks at zero)
        passed &= passed[:, :, -1:]
        t0 = t[:, :, 0][passed[:, :, 0]].min()
        if rep_ > 0:
            rows.append([(float(np.median(t[:, :, j][passed[:, :, j]] - t0)), float((t[:, :, j][passed[:, :, j]] - t0).min()),
                          float((t[:, :, j][passed[:, :, j]] - t0).max())) if passed[:, :, j].any() else (0.0, 0.0, 0.0)
                         for j in range(len(stages))])
    med = np.median(np.array(rows), axis=0)
    timeline = {label: dict(median=round(float(m[0]), 2), earliest=round(float(m[1]), 2), latest=round(float(m[2]), 2))
                for (_, label), m in zip(stages, med) if m[2] > 0}
    span = float(med[-1][2])
    del W, Wb
    torch.cuda.empty_cache()
    return dict(value=per / (span * 1e-6) / 1e9, unit="GB/s", ms_per_step=span * 1e-3,
                config=dict(workload=name, what=what, n_in=n_in, n_out=n_out, weights="Q4_K" if wtype == 12 else "Q6_K", bytes=per),
                roofline=dict(bound="hbm", achieved=per / (span * 1e-6) / 1e9, peak=PEAK_BYTES / 1e9, unit="GB/s",
                              frac=per / (span * 1e-6) / PEAK_BYTES, traffic=None, kernel="gemv_rows_kernel (timeline build)", launch_us=span,
                              note="launch_us: first wave's entry to last wave's last mark in the timeline build, stamps included; "
                                   "one launch on an idle chip, its matrices cold"),
                parity=None, timeline_us=timeline)


CUTOFFS = [(None, "whole layer (split + combine kernels)"), (1, "split kernel alone"),
           (3, "... leaving once its first tile has arrived (no products, no merge, no partial)"),
           (7, "... with a constant position"), (15, "... and no query loads"), (31, "... and K fetched whole lines at a time")]


PREFILL_CUTOFFS = [(None, "whole kernel"), (16, "leaving once the accumulators are handed over (no barrier, merge, store)"),
                   (8, "leaving behind the main loop (no last products either)"),
                   (1, "whole, main loop without its vector work"), (2, "whole, main loop without its LDS operand reads"),
                   (4, "whole, main loop without its copies"), (32, "whole, main loop's copies all of one tile (no trip beyond the nearest cache)"),
                   (64, "whole, main loop's copies of the head's first 32 tiles over and over (no trip beyond the L2)"),
                   (7, "whole, main loop of matrix instructions only")]


def _need_cut_off_builds():
    from orin_llm_amd import build as fa_build

    if not fa_build.probes_built():  # not part of the default build: this workload is the request
        fa_build.build(probes=True)


def run_prefill_cutoffs(torch, kernels, name, steps, warmup):
    """The prefill layer stack timed with the ordinary library and with each cut-off build of the prefill kernel."""
    import ctypes

    _need_cut_off_builds()

    shape, _, n_ctx, (P, B) = WORKLOADS[name]
    sh = SHAPES[shape]
    H, G, d, n_layers = sh["H"], sh["G"], sh["d"], sh["layers"]
    scale = 1.0 / float(np.sqrt(d))
    layers = [make_layer(torch, 800 + i, H, G, d, n_ctx, P + B, B, sh["outliers"]) for i in range(n_layers)]
    outs = [torch.empty((B, H, d), dtype=torch.float32, device="cuda") for _ in range(n_layers)]
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    us = {}
    for flags, label in PREFILL_CUTOFFS:
        if flags is None:
            lib = kernels.lib()
        else:
            lib = kernels.probe_lib(flags, prefill=True)
            rc = lib.orin_fa_init(0)
            assert rc == 0, rc
            lib.orin_fa_set_stream(stream)

        def stack():
            for (q, k, v), o in zip(layers, outs):
                rc = lib.orin_fa_prefill(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), H, G, d, n_ctx, P, B, scale)
                assert rc == 0, rc

        for _ in range(max(1, warmup)):
            stack()
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(max(3, min(steps, 6))):
            e0.record()
            stack()
            e1.record()
            torch.cuda.synchronize()
            best = min(best, e0.elapsed_time(e1) * 1e3 / n_layers)
        us[label] = round(best, 2)
    f = prefill_flops(H, d, P, B)
    whole = us[PREFILL_CUTOFFS[0][1]]
    del layers, outs
    torch.cuda.empty_cache()
    return dict(value=f / (whole * 1e-6) / 1e12, unit="TFLOP/s", ms_per_step=whole * n_layers * 1e-3,
                config=dict(workload=name, shape=f"H{H} G{G} d{d}", layers=n_layers, n_ctx=n_ctx, n_past=P, batch=B, launch="eager"),
                roofline=dict(bound="mfma", achieved=f / (whole * 1e-6) / 1e12, peak=PEAK_FLOPS / 1e12, unit="TFLOP/s",
                              frac=f / (whole * 1e-6) / PEAK_FLOPS, traffic=None,
                              kernel="fa_prefill_kernel, whole and with parts taken out", launch_us=whole, flops_per_launch=f),
                parity=None, cutoffs_us_per_layer=us)


def run_cutoffs(torch, kernels, name, steps, warmup, with_cpu):
    """Not the operator: the decode layer stack timed with the ordinary library and with each cut-off build (the split
    kernel with parts taken out; their results are wrong by design), microseconds per layer, launches back to back."""
    import ctypes

    if isinstance(WORKLOADS[name][3], tuple):
        return run_prefill_cutoffs(torch, kernels, name, steps, warmup)
    _need_cut_off_builds()
    shape, _, n_ctx, L = WORKLOADS[name]
    sh = SHAPES[shape]
    H, G, d, n_layers = sh["H"], sh["G"], sh["d"], sh["layers"]
    scale = 1.0 / float(np.sqrt(d))
    layers = [make_layer(torch, 700 + i, H, G, d, n_ctx, L, 1, sh["outliers"]) for i in range(n_layers)]
    out = torch.empty((H, d), dtype=torch.float32, device="cuda")
    dpos = torch.tensor([L - 1], dtype=torch.int32, device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    us = {}
    for flags, label in CUTOFFS:
        if flags is None:
            lib = kernels.lib()
        else:
            lib = kernels.probe_lib(flags)
            rc = lib.orin_fa_init(0)
            assert rc == 0, rc
            lib.orin_fa_set_stream(stream)

        def stack():
            for q, k, v in layers:
                rc = lib.orin_fa_decode_ind(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), H, G, d, n_ctx, dpos.data_ptr(), scale)
                assert rc == 0, rc

        for _ in range(max(1, warmup)):
            stack()
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(max(3, min(steps, 8))):
            e0.record()
            stack()
            e1.record()
            torch.cuda.synchronize()
            best = min(best, e0.elapsed_time(e1) * 1e3 / n_layers)
        us[label] = round(best, 2)
    by = decode_bytes(H, G, d, L)
    whole = us[CUTOFFS[0][1]]
    del layers
    torch.cuda.empty_cache()
    return dict(value=by / (whole * 1e-6) / 1e9, unit="GB/s", ms_per_step=whole * n_layers * 1e-3,
                config=dict(workload=name, shape=f"H{H} G{G} d{d}", layers=n_layers, n_ctx=n_ctx, L=L, launch="eager"),
                roofline=dict(bound="hbm", achieved=by / (whole * 1e-6) / 1e9, peak=PEAK_BYTES / 1e9, unit="GB/s",
                              frac=by / (whole * 1e-6) / PEAK_BYTES, traffic=None,
                              kernel="fa_decode_split_kernel<128, 0>, whole and with parts taken out", launch_us=whole,
                              bytes_per_launch=by),
                parity=None, cutoffs_us_per_layer=us)


def run_handoff(torch, kernels, name, steps, warmup, with_cpu):
    """One step = 28 launches of the stand-in over rotating cold buffers; value = the two-launch form's rate."""
    nbytes, scratch_bytes = kernels.bench_handoff_sizes()
    launches = 28
    n_buf = max(launches, int(np.ceil(1.2e9 / nbytes)))
    pool = torch.empty(n_buf * nbytes, dtype=torch.uint8, device="cuda").fill_(1)
    scratch = torch.zeros(scratch_bytes, dtype=torch.uint8, device="cuda")
    outs = {f: torch.zeros(784, device="cuda") for f in (False, True)}
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    us, walls = {}, {}
    for fused in (False, True):
        k = 0

        def one_step():
            nonlocal k
            for _ in range(launches):
                kernels.bench_handoff(pool[(k % n_buf) * nbytes:], fused, scratch, outs[fused])
                k += 1

        for _ in range(warmup):
            one_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record()
        for _ in range(steps):
            one_step()
        e1.record()
        torch.cuda.synchronize()
        walls[fused] = time.perf_counter() - t0
        us[fused] = e0.elapsed_time(e1) * 1e3 / (steps * launches)
    want = np.tile(np.array([32896.0, 0.0, 256.0, 384.0], np.float32), 196)
    want[1::4] = 256.0 * (np.arange(196) & 7)
    same = bool(np.array_equal(outs[False].cpu().numpy(), want) and np.array_equal(outs[True].cpu().numpy(), want))
    del pool
    torch.cuda.empty_cache()
    return dict(value=nbytes * launches * steps / walls[False] / 1e9, unit="GB/s", ms_per_step=walls[False] / steps * 1e3,
                config=dict(workload=name, bytes_per_launch=nbytes, launches_per_step=launches, workgroups=256,
                            partial_floats=784),
                roofline=dict(bound="hbm", achieved=nbytes / (us[False] * 1e-6) / 1e9, peak=PEAK_BYTES / 1e9, unit="GB/s",
                              frac=nbytes / (us[False] * 1e-6) / PEAK_BYTES, traffic=None,
                              kernel="handoff_split_kernel<false> + handoff_combine_kernel (stand-in, not part of the path)",
                              launch_us=us[False], two_launch_us=us[False], fused_two_level_us=us[True],
                              bytes_per_launch=nbytes),
                parity=dict(both_forms_give_the_known_sum=same))

