#!/usr/bin/env python3
"""Benchmark of the MI355X GQA flash-attention path (one GPU).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-also] [--no-cpu] [--full]

The LAST line of stdout is one compact JSON object (under 4 KB: metric, value, roofline, cpu_baseline, parity and
the few figures of the target workloads under "targets"); every workload's full result goes to
the file --full-record names.  --full also runs the neighbouring operators' workloads (rope, kv_store, kv_shift,
fused decode entry points, long-context prefill, logits); measurement aids (timelines, cut-off builds, read-pattern
and hand-off stand-ins: bench_aids.py) run only when named with --workload.  A "step" is one pass of the attention operator over a whole layer
stack of synthetic inputs already resident in HBM (independent seeds and buffers per layer):

  qwen1.5b-prefill512   (default; the configuration the headline metric is quoted on) 28 layers x two 512-token causal chunks,
                        at cache depth 0 and 3584, 12 Q heads / 2 KV heads, d=128, K with 4
                        outlier channels x8.  value = causal-exact TFLOP/s (step launched eagerly and as
                        one HIP graph; the faster counts, both are reported).
  llama8b-prefill512-d4096, qwen7b-prefill512-d32256, qwen1.5b-decode-32k, llama8b-decode-8k,
  qwen7b-decode-32k     the other benchmark shapes; the target cases are also run after the
                        default workload and reported under "also".

FLOPs per prefill launch (causal-exact): 4*d*H*(B*P + B*(B+1)/2).  Bytes per decode launch:
4*G*L*d (fp16 K and V read once) + 2*H*d*4 (q in, out).  Peaks: 2.5e15 FLOP/s dense fp16
MFMA, 8.0e12 B/s HBM3E.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

PEAK_FLOPS = 2.5e15
PEAK_BYTES = 8.0e12

SHAPES = {
    "qwen1.5b": dict(H=12, G=2, d=128, layers=28, outliers=4, n_embd=1536, n_ff=8960, bias=True, neox=1, theta=1.0e6),
    "llama8b": dict(H=32, G=8, d=128, layers=32, outliers=0, n_embd=4096, n_ff=14336, bias=False, neox=0, theta=5.0e5),
    "qwen7b": dict(H=28, G=4, d=128, layers=28, outliers=4, n_embd=3584, n_ff=18944, bias=True, neox=1, theta=1.0e6),
}

WORKLOADS = {
    # name: (shape, kind, n_ctx, list of (P, B) for prefill | L for decode)
    "qwen1.5b-prefill512": ("qwen1.5b", "prefill", 4096, [(0, 512), (3584, 512)]),
    "qwen1.5b-prefill512-d3584": ("qwen1.5b", "prefill", 4096, [(3584, 512)]),  # the default workload's second chunk alone
    "qwen1.5b-prefill512-d32256": ("qwen1.5b", "prefill", 32768, [(32256, 512)]),  # the last chunk of a full 32k context
    "qwen1.5b-prefill45-d32000": ("qwen1.5b", "prefill", 32768, [(32000, 45)]),    # a short last piece of a long prompt
    "llama8b-prefill512-d4096": ("llama8b", "prefill", 8192, [(4096, 512)]),
    "llama8b-prefill512-d0": ("llama8b", "prefill", 8192, [(0, 512)]),
    "llama8b-prefill512-d7680": ("llama8b", "prefill", 8192, [(7680, 512)]),
    "qwen7b-prefill512-d32256": ("qwen7b", "prefill", 32768, [(32256, 512)]),
    "qwen1.5b-decode-1k": ("qwen1.5b", "decode", 32768, 1024),     # earlier positions of the same 32k cache
    "qwen1.5b-decode-8k": ("qwen1.5b", "decode", 32768, 8192),
    "qwen1.5b-decode-32k": ("qwen1.5b", "decode", 32768, 32768),
    "llama8b-decode-8k": ("llama8b", "decode", 8192, 8192),
    "qwen7b-decode-32k": ("qwen7b", "decode", 32768, 32767),
    # the decode layer's call pair (store the token's K/V rows, then attend; reference src/model_gpu.cu:281-282)
    # through the entry point that does both in the attention launches; the two calls are timed beside it
    "qwen1.5b-decode-store-32k": ("qwen1.5b", "decode_store", 32768, 32768),
    "qwen1.5b-decode-rope-store-32k": ("qwen1.5b", "decode_rope_store", 32768, 32768),
    # the two mutators of the cache (byte movers; value = bytes read + written per second)
    "llama8b-kv-store-512": ("llama8b", "kv_store", 8192, (4096, 512)),
    "qwen1.5b-kv-shift-32k": ("qwen1.5b", "kv_shift", 32768, (4, 16382)),
    # rotary embedding of a 512-token chunk's Q and K rows (value = bytes read + written per second)
    "llama8b-rope-512": ("llama8b", "rope", 8192, (4096, 512)),
    # not part of the path: a plain device copy of known size, the yardstick that the HBM
    # counters (FETCH_SIZE / WRITE_SIZE) and the achievable streaming rate are scaled by
    "hbm-copy-256MiB": (None, "copy", 0, 256 << 20),
    # not part of the path either: a kernel that only reads, as many bytes per launch as one decode layer's
    # cache (32 MiB: Qwen2.5-1.5B at 32k and Llama-3-8B at 8k; 64 MiB: Qwen2.5-7B at 32k), launched back to
    # back over rotating buffers that no cache holds -- what such a launch costs when nothing is computed
    "hbm-read-32MiB": (None, "read", 0, 32 << 20),
    "hbm-read-64MiB": (None, "read", 0, 64 << 20),
    # not part of the path: a stand-in for one split-KV decode step (256 workgroups stream 32 MiB and leave 3 KB
    # partials), its partials merged by a second kernel, as the library does, or inside the launch by a two-level
    # last-arriver reduction over write-through stores and relaxed atomics -- what fusing the combine would cost
    "decode-handoff-mock": (None, "handoff", 0, 32 << 20),
    # not part of the path: read-only stand-ins for the loads of a matrix-vector kernel over a Q4_K gate/up pair of
    # Llama-3-8B's shape (2 x 14336 rows x 16 blocks, 66 MB), by load pattern -- 64 bytes of each of 16 rows per
    # instruction, or lane-linear runs of one, two or four whole blocks of a row
    "weights-read-patterns": (None, "patterns", 0, (14336, 16)),
    # The whole decode layer around the path (norms, quantised projections, rotary embedding, cache store,
    # attention, feed-forward block): one token through every layer of the model, replayed as one graph.
    # Weights are random blocks in the mix of a Q4_K_M file (Q4_K; attn_v and ffn_down Q6_K).
    "qwen1.5b-decode-layer-32k": ("qwen1.5b", "decode_layer", 32768, 32768),
    "llama8b-decode-layer-8k": ("llama8b", "decode_layer", 8192, 8192),
    "qwen7b-decode-layer-32k": ("qwen7b", "decode_layer", 32768, 32767),
    # The end of a decode step (reference: src/model_gpu.cu:303-306): the last norm and the output matrix over the
    # residual stream, one token.  Output matrix Q6_K, as a Q4_K_M file keeps it; (vocabulary size)
    "llama8b-logits": ("llama8b", "logits", 0, 128256),
    "qwen1.5b-logits": ("qwen1.5b", "logits", 0, 151936),
    # not timed: where a kernel's microseconds go, from the timeline build of the library (the attention kernels'
    # stage marks store the wall clock there; medians over the waves of one launch, cold inputs)
    "llama8b-prefill512-d4096-timeline": ("llama8b", "timeline", 8192, ("prefill", 4096, 512)),
    "qwen1.5b-prefill512-d3584-timeline": ("qwen1.5b", "timeline", 4096, ("prefill", 3584, 512)),
    "qwen1.5b-prefill512-d0-timeline": ("qwen1.5b", "timeline", 4096, ("prefill", 0, 512)),
    # not part of the path: the decode split kernel with parts taken out (cut-off builds of the library, results
    # wrong by design), timed like the decode workloads: what the combine launch, the products and the merge,
    # the trip for the position, the query and the operand-order K loads each cost on top of a plain read
    "llama8b-prefill512-d4096-cutoffs": ("llama8b", "cutoffs", 8192, (4096, 512)),   # ... and of the prefill kernel
    "qwen1.5b-prefill512-d3584-cutoffs": ("qwen1.5b", "cutoffs", 4096, (3584, 512)),
    "qwen1.5b-decode-32k-cutoffs": ("qwen1.5b", "cutoffs", 32768, 32768),
    "llama8b-decode-8k-cutoffs": ("llama8b", "cutoffs", 8192, 8192),   # (shapes where a wave has one tile: the cut-off kernel leaves after its first)
    "qwen1.5b-decode-32k-timeline": ("qwen1.5b", "timeline", 32768, ("decode", 32768, 1)),
    "qwen7b-decode-32k-timeline": ("qwen7b", "timeline", 32768, ("decode", 32767, 1)),
    # ... and of the matrix-vector kernel that reads rows in long runs, on the two big products of a Llama-3-8B layer
    # (Q4_K gate/up pair with the norm folded in; Q6_K down projection adding into the residual stream): (what, n_in, n_out)
    "llama8b-gateup-timeline": ("llama8b", "timeline", 0, ("gateup", 4096, 14336)),
    "llama8b-down-timeline": ("llama8b", "timeline", 0, ("down", 14336, 4096)),
    # ... and of a Qwen2.5-1.5B layer, whose launches leave resident places empty
    "qwen1.5b-gateup-timeline": ("qwen1.5b", "timeline", 0, ("gateup", 1536, 8960)),
    "qwen1.5b-down-timeline": ("qwen1.5b", "timeline", 0, ("down", 8960, 1536)),
}
# HBM bytes per launch of the dominant kernel (decode: per layer, both kernels), from the FETCH_SIZE and
# WRITE_SIZE counter passes of rocprofv3 scaled by the same counters on a plain 256 MiB copy: recorded
# measurements (a counter pass cannot run inside the timed benchmark), kept with the commit they were
# taken at in profiles/traffic.json; None where not taken.
def _load_traffic():
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            doc = json.load(f)
        return {k: v["bytes_per_launch"] for k, v in doc["workloads"].items()}, doc.get("measured_at_commit")
    except (OSError, ValueError, KeyError):
        return {}, None


TRAFFIC, TRAFFIC_COMMIT = _load_traffic()
# Run after the default workload: the two plain-read yardsticks, the decode layer around the path on two models,
# and the three cases the targets are stated on.  Their few figures close the line under "targets".
ALSO = ["hbm-read-32MiB", "hbm-read-64MiB", "qwen1.5b-decode-layer-32k", "llama8b-decode-layer-8k",
        "llama8b-prefill512-d4096", "qwen1.5b-decode-32k", "qwen7b-decode-32k"]
# --full: the neighbouring operators and the other shapes, ahead of the above
ALSO_FULL = ["llama8b-rope-512", "llama8b-kv-store-512", "qwen1.5b-kv-shift-32k", "qwen1.5b-decode-store-32k",
             "qwen1.5b-decode-rope-store-32k", "qwen1.5b-prefill512-d32256", "llama8b-decode-8k", "llama8b-logits",
             "qwen7b-decode-layer-32k"]
TARGETS = list(ALSO)
ALSO_CPU = {"qwen1.5b-decode-32k"}  # the decode half of the metric gets its CPU baseline in the default run too


def prefill_flops(H, d, P, B):
    return 4.0 * d * H * (B * P + B * (B + 1) / 2.0)


def decode_bytes(H, G, d, L):
    return 4.0 * G * L * d + 2.0 * H * d * 4.0


def make_layer(torch, seed, H, G, d, n_ctx, n_filled, batch, outliers):
    """Seeded N(0,1) values rounded to fp16; K gets `outliers` channels per KV head scaled by 8."""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    q = torch.randn((batch, H, d), generator=g, device="cuda", dtype=torch.float32).half().float()
    k = torch.randn((G, n_ctx, d), generator=g, device="cuda", dtype=torch.float32).half()
    v = torch.randn((G, n_ctx, d), generator=g, device="cuda", dtype=torch.float32).half()
    if outliers:
        for kvh in range(G):
            ch = torch.randperm(d, generator=g, device="cuda")[:outliers]
            k[kvh, :, ch] *= 8.0
    if n_filled < n_ctx:  # the engine never zero-fills the cache: poison what must not be read
        k[:, n_filled:] = float("nan")
        v[:, n_filled:] = float("nan")
    return q, k.view(torch.int16), v.view(torch.int16)


def parity_rows(torch, ref, rel_err, q, k, v, out, H, G, d, n_ctx, n_past, batch, scale, n_rows=48, seed=0):
    rng = np.random.default_rng(seed)
    n_tok = max(1, min(8, n_rows // 4))
    toks = sorted({0, batch - 1, *(int(x) for x in rng.integers(0, batch, size=max(0, n_tok - 2)))})
    rows = np.array([(t, h) for t in toks for h in rng.choice(H, size=min(H, max(1, n_rows // len(toks))),
                                                              replace=False)], np.int32)
    want = ref.flash_attention_rows(q.cpu().numpy(), k.view(torch.uint16).cpu().numpy(),
                                    v.view(torch.uint16).cpu().numpy(), rows, H, G, d, n_ctx, n_past,
                                    np.float32(scale), threads=ref.max_threads())
    got = out.cpu().numpy()[rows[:, 0], rows[:, 1]]
    return rel_err(got, want)


def parity_stack(torch, ref, rel_err, stack, H, G, d, n_ctx, n_past, batch, scale, rows_first=48, rows_other=12):
    """Sampled (token, head) rows of EVERY layer of a timed stack against the CPU oracle (layer 0 more
    densely); returns the worst figures over the layers."""
    worst = [0.0, 0.0, 0.0]
    for l, (q, k, v, out) in enumerate(stack):
        e = parity_rows(torch, ref, rel_err, q, k, v, out, H, G, d, n_ctx, n_past, batch, scale,
                        n_rows=rows_first if l == 0 else rows_other, seed=l)
        worst = [max(a, b) for a, b in zip(worst, e)]
    return worst


def cpu_baseline_prefill(ref, layers_qkv, H, G, d, n_ctx, P, B, scale, budget_s=15.0):
    """The oracle's reference-order loop (fp32 cache, one thread) on a bounded sample of the same
    workload: the query tokens of the first layers' chunk, in a fixed shuffled order, until the
    time budget is used."""
    done, flops, dt, used = 0, 0.0, 0.0, 0
    for q, k, v in layers_qkv:
        kf = ref.fp16_to_fp32(k)  # (the conversion of the cache is not timed: the CPU backend stores fp32)
        vf = ref.fp16_to_fp32(v)
        used += 1
        t0 = time.perf_counter()
        for t in (int(t) for t in np.random.default_rng(1).permutation(B)):
            ref.attention_token_f32(q[t], kf, vf, H, G, d, n_ctx, P + t + 1, np.float32(scale))
            flops += 4.0 * d * H * (P + t + 1)
            done += 1
            if dt + time.perf_counter() - t0 > budget_s:
                break
        dt += time.perf_counter() - t0
        if dt > budget_s:
            break
    # Beside it, separately labelled: the same restatement spread over the host's cores (the
    # reference's CPU backend has no threading), one (token, head) row per task, fp16 cache.
    threads = ref.max_threads()
    rows = np.array([(t, h) for t in range(B) for h in range(H)], np.int32)
    mt_flops, mt_dt, mt_layers = 0.0, 0.0, 0
    for q, k, v in layers_qkv:
        t0 = time.perf_counter()
        ref.flash_attention_rows(q, k, v, rows, H, G, d, n_ctx, P, np.float32(scale), threads=threads)
        mt_dt += time.perf_counter() - t0
        mt_flops += prefill_flops(H, d, P, B)
        mt_layers += 1
        if mt_dt > budget_s / 3:
            break
    return dict(value=flops / dt / 1e12, unit="TFLOP/s", cores=1, kind="port",
                sample=f"{done} query tokens x {H} heads at depth {P} from the first {used} layer(s) "
                       f"({flops / 1e9:.2f} GFLOP in {dt:.1f} s), reference loop order, fp32 cache",
                all_cores=dict(value=mt_flops / mt_dt / 1e12, unit="TFLOP/s", cores=threads,
                               sample=f"every (token, head) row of {mt_layers} layer(s) at depth {P} in {mt_dt:.1f} s, "
                                      f"rows spread over {threads} OpenMP threads, fp16 cache"))


def cpu_baseline_decode(ref, q, k, v, H, G, d, n_ctx, L, scale):
    kf = ref.fp16_to_fp32(k)
    vf = ref.fp16_to_fp32(v)
    reps, t0 = 0, time.perf_counter()
    while True:
        ref.attention_token_f32(q, kf, vf, H, G, d, n_ctx, L, np.float32(scale))
        reps += 1
        if time.perf_counter() - t0 > 10.0 or reps >= 64:
            break
    dt = time.perf_counter() - t0
    # the CPU backend keeps an fp32 cache; the bytes counted are the fp16 bytes of the same positions
    threads = min(ref.max_threads(), H)
    rows = np.array([(0, h) for h in range(H)], np.int32)
    mt_reps, t0 = 0, time.perf_counter()
    while True:
        ref.flash_attention_rows(q[None], k, v, rows, H, G, d, n_ctx, L - 1, np.float32(scale), threads=threads)
        mt_reps += 1
        if time.perf_counter() - t0 > 3.0 or mt_reps >= 64:
            break
    mt_dt = time.perf_counter() - t0
    # the CPU backend keeps an fp32 cache; the bytes counted are the fp16 bytes of the same positions
    return dict(value=decode_bytes(H, G, d, L) * reps / dt / 1e9, unit="GB/s", cores=1, kind="port",
                sample=f"{reps} decode steps of layer 0 at L={L} in {dt:.1f} s, reference loop order, fp32 cache",
                all_cores=dict(value=decode_bytes(H, G, d, L) * mt_reps / mt_dt / 1e9, unit="GB/s", cores=threads,
                               sample=f"{mt_reps} decode steps of layer 0 at L={L} in {mt_dt:.1f} s, one head per "
                                      f"OpenMP thread, fp16 cache"))


def run_prefill(torch, kernels, name, steps, warmup, with_cpu):
    from oracle import ref
    from util import rel_err

    shape_name, _, n_ctx, chunks = WORKLOADS[name]
    s = SHAPES[shape_name]
    H, G, d, layers = s["H"], s["G"], s["d"], s["layers"]
    scale = float(1.0 / np.sqrt(d))
    stacks = []
    for ci, (P, B) in enumerate(chunks):
        stack = []
        for l in range(layers):
            q, k, v = make_layer(torch, 1000 * ci + l, H, G, d, n_ctx, P + B, B, s["outliers"])
            stack.append((q, k, v, torch.empty((B, H, d), dtype=torch.float32, device="cuda")))
        stacks.append(stack)

    def one_step(events=None):
        for ci, (P, B) in enumerate(chunks):
            if events is not None:
                events[ci][0].record()
            for q, k, v, out in stacks[ci]:
                kernels.flash_attention(q, k, v, out, H, G, d, n_ctx, P, B, scale)
            if events is not None:
                events[ci][1].record()

    for _ in range(warmup):
        one_step()
    torch.cuda.synchronize()
    evs = [[(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in chunks]
           for _ in range(steps)]
    t0 = time.perf_counter()
    for i in range(steps):
        one_step(evs[i])
    torch.cuda.synchronize()
    wall_eager = time.perf_counter() - t0

    # The same step captured once as a HIP graph and replayed (the operator is capture-safe: no
    # allocation, no synchronisation); the host may launch it either way, the faster one counts.
    g = torch.cuda.CUDAGraph()
    try:
        with torch.cuda.graph(g):
            kernels.set_stream(torch.cuda.current_stream().cuda_stream)
            one_step()
    finally:
        kernels.set_stream(torch.cuda.current_stream().cuda_stream)
    for _ in range(warmup):
        g.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        g.replay()
    torch.cuda.synchronize()
    wall_graph = time.perf_counter() - t0
    wall = min(wall_eager, wall_graph)

    # Per-launch duration of the dominant kernel: one event pair around every single launch of
    # one pass over the stack (the events sit on the stream the kernels are launched on).
    dom = max(range(len(chunks)), key=lambda ci: prefill_flops(H, d, *chunks[ci]))
    P, B = chunks[dom]
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in stacks[dom]]
    for (q, k, v, out), (a0, a1) in zip(stacks[dom], pairs):
        a0.record()
        kernels.flash_attention(q, k, v, out, H, G, d, n_ctx, P, B, scale)
        a1.record()
    torch.cuda.synchronize()
    single_us = float(np.median([a0.elapsed_time(a1) for a0, a1 in pairs])) * 1e3

    flops_step = sum(prefill_flops(H, d, P, B) for P, B in chunks) * layers
    per_chunk = []
    for ci, (P, B) in enumerate(chunks):
        ms = sum(evs[i][ci][0].elapsed_time(evs[i][ci][1]) for i in range(steps)) / (steps * layers)
        f = prefill_flops(H, d, P, B)
        per_chunk.append(dict(P=P, B=B, launch_us=ms * 1e3, tflops=f / (ms * 1e-3) / 1e12,
                              frac=f / (ms * 1e-3) / PEAK_FLOPS))
    errs = [parity_stack(torch, ref, rel_err, stacks[ci], H, G, d, n_ctx, Pc, Bc, scale) for ci, (Pc, Bc) in enumerate(chunks)]
    err = [max(e[i] for e in errs) for i in range(3)]
    res = dict(
        value=flops_step * steps / wall / 1e12, unit="TFLOP/s", ms_per_step=wall / steps * 1e3,
        config=dict(workload=name, shape=f"H{H} G{G} d{d}", layers=layers, n_ctx=n_ctx,
                    chunks=[list(c) for c in chunks], flops_per_step=flops_step),
        roofline=dict(bound="mfma", achieved=prefill_flops(H, d, P, B) / (single_us * 1e-6) / 1e12,
                      peak=PEAK_FLOPS / 1e12, unit="TFLOP/s",
                      frac=prefill_flops(H, d, P, B) / (single_us * 1e-6) / PEAK_FLOPS, traffic=TRAFFIC.get(name),
                      kernel=f"fa_prefill_kernel<{d}, ...> at P={P} B={B}", launch_us=single_us,
                      launch_us_back_to_back=per_chunk[dom]["launch_us"],
                      flops_per_launch=prefill_flops(H, d, P, B),
                      note="launch_us: median of event pairs around single launches; "
                           "launch_us_back_to_back: stack average including launch gaps"),
        per_chunk=per_chunk,
        eager=dict(ms_per_step=wall_eager / steps * 1e3), graph=dict(ms_per_step=wall_graph / steps * 1e3),
        parity=dict(err_row=err[0], err_floor1pct=err[1], rel_l2=err[2],
                    rows=f"worst over sampled rows of all {layers} layers of every chunk, vs CPU oracle"),
    )
    res["config"]["launch"] = "graph" if wall_graph <= wall_eager else "eager"
    if with_cpu:
        sample = [(ql.cpu().numpy(), kl.view(torch.uint16).cpu().numpy(), vl.view(torch.uint16).cpu().numpy())
                  for ql, kl, vl, _ in stacks[dom][:6]]
        res["cpu_baseline"] = cpu_baseline_prefill(ref, sample, H, G, d, n_ctx, P, B, scale)
    return res


def run_decode(torch, kernels, name, steps, warmup, with_cpu):
    from oracle import ref
    from util import rel_err

    shape_name, _, n_ctx, L = WORKLOADS[name]
    s = SHAPES[shape_name]
    H, G, d, layers = s["H"], s["G"], s["d"], s["layers"]
    scale = float(1.0 / np.sqrt(d))
    bytes_layer = decode_bytes(H, G, d, L)
    # The chip has 256 MB of last-level (Infinity) cache: rotate enough independent stacks that
    # a sweep exceeds it, so the timed loop streams from HBM.
    n_stacks = max(1, int(np.ceil(600e6 / (bytes_layer * layers))))
    stacks = []
    for si in range(n_stacks):
        stack = []
        for l in range(layers):
            q, k, v = make_layer(torch, 5000 + 100 * si + l, H, G, d, n_ctx, L, 1, s["outliers"])
            stack.append((q[0].contiguous(), k, v, torch.empty((H, d), dtype=torch.float32, device="cuda")))
        stacks.append(stack)
    dpos = torch.tensor([L - 1], dtype=torch.int32, device="cuda")
    rope = WORKLOADS[name][1] == "decode_rope_store"
    store = rope or WORKLOADS[name][1] == "decode_store"
    theta = 1.0e6  # Qwen2.5's rope base; "neox" pairing over the whole head
    gen = torch.Generator(device="cuda")
    gen.manual_seed(99)
    k_new = torch.randn((G, d), generator=gen, device="cuda", dtype=torch.float32)
    v_new = torch.randn((G, d), generator=gen, device="cuda", dtype=torch.float32)

    angles = torch.zeros((d // 2, 2), device="cuda")

    def one_stack(si):
        if rope:  # the token's angles once, then every layer
            kernels.rope_angles_ind(angles, d, theta, dpos)
        for q, k, v, out in stacks[si]:
            if rope:
                kernels.flash_attention_decode_rope_store_ind(q, k_new, v_new, k, v, out, H, G, d, n_ctx, dpos, scale,
                                                              d, theta, None, True, angles)
            elif store:
                kernels.flash_attention_decode_store_ind(q, k_new, v_new, k, v, out, H, G, d, n_ctx, dpos, scale)
            else:
                kernels.flash_attention_decode_ind(q, k, v, out, H, G, d, n_ctx, dpos, scale)

    q_sep, k_sep = stacks[0][0][0].clone(), k_new.clone()  # rotated in place over and over by the separate calls

    def one_stack_two_calls(si):
        for q, k, v, out in stacks[si]:
            if rope:
                kernels.rope_neox_ind(q_sep, H, d, d, theta, dpos)
                kernels.rope_neox_ind(k_sep, G, d, d, theta, dpos)
                kernels.kv_store_ind(k, v, k_sep, v_new, G, d, n_ctx, dpos)
                kernels.flash_attention_decode_ind(q_sep, k, v, out, H, G, d, n_ctx, dpos, scale)
            else:
                kernels.kv_store_ind(k, v, k_new, v_new, G, d, n_ctx, dpos)
                kernels.flash_attention_decode_ind(q, k, v, out, H, G, d, n_ctx, dpos, scale)

    # eager
    for i in range(warmup):
        one_stack(i % n_stacks)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        one_stack(i % n_stacks)
    e1.record()
    torch.cuda.synchronize()
    wall_eager = time.perf_counter() - t0
    dev_eager_ms = e0.elapsed_time(e1)

    # one HIP graph per stack, as the engine replays its decode step (reference src/model_gpu.cu:295-344)
    graphs = []
    for si in range(n_stacks):
        g = torch.cuda.CUDAGraph()
        try:
            with torch.cuda.graph(g):
                kernels.set_stream(torch.cuda.current_stream().cuda_stream)
                one_stack(si)
        finally:
            kernels.set_stream(torch.cuda.current_stream().cuda_stream)
        graphs.append(g)
    for i in range(warmup):
        graphs[i % n_stacks].replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        graphs[i % n_stacks].replay()
    e1.record()
    torch.cuda.synchronize()
    wall_graph = time.perf_counter() - t0
    dev_graph_ms = e0.elapsed_time(e1)

    two_calls_us = two_calls_graph_us = None
    if store:  # the same step as the reference makes it: two (with the rotary embedding four) calls per layer
        for i in range(warmup):
            one_stack_two_calls(i % n_stacks)
        torch.cuda.synchronize()
        e0.record()
        for i in range(steps):
            one_stack_two_calls(i % n_stacks)
        e1.record()
        torch.cuda.synchronize()
        two_calls_us = e0.elapsed_time(e1) * 1e3 / (steps * layers)
        sep_graphs = []
        for si in range(n_stacks):
            g = torch.cuda.CUDAGraph()
            try:
                with torch.cuda.graph(g):
                    kernels.set_stream(torch.cuda.current_stream().cuda_stream)
                    one_stack_two_calls(si)
            finally:
                kernels.set_stream(torch.cuda.current_stream().cuda_stream)
            sep_graphs.append(g)
        for i in range(warmup):
            sep_graphs[i % n_stacks].replay()
        torch.cuda.synchronize()
        e0.record()
        for i in range(steps):
            sep_graphs[i % n_stacks].replay()
        e1.record()
        torch.cuda.synchronize()
        two_calls_graph_us = e0.elapsed_time(e1) * 1e3 / (steps * layers)
        del sep_graphs

    if store:  # the check below is of the entry point this workload names, not of the last writer of `out`
        one_stack((steps - 1) % n_stacks)
        torch.cuda.synchronize()
    q, k, v, out = stacks[(steps - 1) % n_stacks][0]
    rows = np.array([(0, h) for h in range(H)], np.int32)
    q_rot = q  # layer 0's query as the oracle wants it
    err = [0.0, 0.0, 0.0]
    for ql, kl, vl, outl in stacks[(steps - 1) % n_stacks]:  # every head of every layer of the stack that ran last
        if rope:
            ql = ql.clone()
            kernels.rope_neox_ind(ql, H, d, d, theta, dpos)
            torch.cuda.synchronize()
        want = ref.flash_attention_rows(ql.cpu().numpy()[None], kl.view(torch.uint16).cpu().numpy(),
                                        vl.view(torch.uint16).cpu().numpy(), rows, H, G, d, n_ctx, L - 1,
                                        np.float32(scale), threads=ref.max_threads())
        err = [max(a, b) for a, b in zip(err, rel_err(outl.cpu().numpy(), want))]
    wall = min(wall_graph, wall_eager)
    launch_us = min(dev_graph_ms, dev_eager_ms) * 1e3 / (steps * layers)
    res = dict(
        value=bytes_layer * layers * steps / wall / 1e9, unit="GB/s", ms_per_step=wall / steps * 1e3,
        config=dict(workload=name, shape=f"H{H} G{G} d{d}", layers=layers, n_ctx=n_ctx, L=L,
                    bytes_per_step=bytes_layer * layers, stacks_rotated=n_stacks,
                    splits=kernels.decode_splits(H, G, d, n_ctx)),
        roofline=dict(bound="hbm", achieved=bytes_layer / (launch_us * 1e-6) / 1e9, peak=PEAK_BYTES / 1e9,
                      unit="GB/s", frac=bytes_layer / (launch_us * 1e-6) / PEAK_BYTES, traffic=TRAFFIC.get(name),
                      kernel=f"fa_decode_split_kernel<{d}> + fa_decode_combine_kernel<{d}> (one layer)",
                      launch_us=launch_us, bytes_per_launch=bytes_layer,
                      note="launch_us: both kernels of a layer, back to back in the timed loop, launch gaps "
                           "included; each kernel's own duration is in profiles/ (rocprofv3 kernel trace)"),
        eager=dict(ms_per_step=wall_eager / steps * 1e3, device_ms_per_step=dev_eager_ms / steps),
        graph=dict(ms_per_step=wall_graph / steps * 1e3, device_ms_per_step=dev_graph_ms / steps),
        parity=dict(err_row=err[0], err_floor1pct=err[1], rel_l2=err[2], rows=f"all heads of all {layers} layers, vs CPU oracle"),
    )
    if store:
        mode = "rotate + store" if rope else "store"
        res["roofline"]["kernel"] = f"fa_decode_split_kernel<{d}, {mode}> + fa_decode_combine_kernel<{d}> (one layer)"
        res["roofline"]["launch_us_eager"] = dev_eager_ms * 1e3 / (steps * layers)
        res["roofline"]["launch_us_graph"] = dev_graph_ms * 1e3 / (steps * layers)
        res["roofline"]["launch_us_separate_calls"] = two_calls_us
        res["roofline"]["launch_us_separate_calls_graph"] = two_calls_graph_us
        sep = ("rope_neox_ind on q, rope_neox_ind on the new K row, kv_store_ind, flash_attention_decode_ind" if rope
               else "kv_store_ind + flash_attention_decode_ind")
        res["roofline"]["note"] += f"; launch_us_separate_calls: {sep} per layer, back to back, eager and replayed from a graph"
    if with_cpu:
        if rope:  # the oracle attends with the rotated query; the cache already holds the rotated row
            q = q.clone()
            kernels.rope_neox_ind(q, H, d, d, theta, dpos)
            torch.cuda.synchronize()
        res["cpu_baseline"] = cpu_baseline_decode(ref, q.cpu().numpy(), k.view(torch.uint16).cpu().numpy(),
                                                  v.view(torch.uint16).cpu().numpy(), H, G, d, n_ctx, L, scale)
    del stacks, graphs
    torch.cuda.empty_cache()
    return res


def time_eager_and_graph(torch, kernels, one_step, steps, warmup):
    """Times `steps` passes of one_step launched eagerly and again replayed as one HIP graph
    (small launches are otherwise priced by the host's launch rate, not by the GPU).  Returns
    (wall seconds, device milliseconds) of the faster form and both forms' ms per step."""
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def timed(fn):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return time.perf_counter() - t0, e0.elapsed_time(e1)

    wall_e, dev_e = timed(one_step)
    g = torch.cuda.CUDAGraph()
    try:
        with torch.cuda.graph(g):
            kernels.set_stream(torch.cuda.current_stream().cuda_stream)
            one_step()
    finally:
        kernels.set_stream(torch.cuda.current_stream().cuda_stream)
    wall_g, dev_g = timed(g.replay)
    forms = dict(eager=dict(ms_per_step=wall_e / steps * 1e3, device_ms_per_step=dev_e / steps),
                 graph=dict(ms_per_step=wall_g / steps * 1e3, device_ms_per_step=dev_g / steps))
    return min(wall_e, wall_g), min(dev_e, dev_g), forms


def run_kv_store(torch, kernels, name, steps, warmup, with_cpu):
    """One step = kv_store_batch of a 512-token chunk into every layer's cache (fp32 in, fp16 out)."""
    from oracle import ref
    shape_name, _, n_ctx, (P, B) = WORKLOADS[name]
    s = SHAPES[shape_name]
    G, d, layers = s["G"], s["d"], s["layers"]
    g = torch.Generator(device="cuda")
    g.manual_seed(77)
    stack = [(torch.zeros((G, n_ctx, d), dtype=torch.int16, device="cuda"),
              torch.zeros((G, n_ctx, d), dtype=torch.int16, device="cuda"),
              torch.randn((B, G, d), generator=g, device="cuda"), torch.randn((B, G, d), generator=g, device="cuda"))
             for _ in range(layers)]

    def one_step():
        for kc, vc, k, v in stack:
            kernels.kv_store_batch(kc, vc, k, v, G, d, n_ctx, P, B)

    wall, dev_ms, forms = time_eager_and_graph(torch, kernels, one_step, steps, warmup)
    us = dev_ms * 1e3 / (steps * layers)
    nbytes = 2.0 * B * G * d * (4 + 2)  # K and V: fp32 read, fp16 written
    kc, vc, k, v = stack[0]
    wk = np.zeros((G, n_ctx, d), np.uint16)
    wv = np.zeros((G, n_ctx, d), np.uint16)
    ref.kv_store_f16(wk, wv, k.cpu().numpy(), v.cpu().numpy(), G, d, n_ctx, P, B)
    exact = bool(np.array_equal(kc.cpu().numpy().view(np.uint16), wk) and np.array_equal(vc.cpu().numpy().view(np.uint16), wv))
    return dict(value=nbytes * layers * steps / wall / 1e9, unit="GB/s", ms_per_step=wall / steps * 1e3,
                config=dict(workload=name, shape=f"G{G} d{d}", layers=layers, n_ctx=n_ctx, pos_base=P, batch=B,
                            bytes_per_step=nbytes * layers),
                roofline=dict(bound="hbm", achieved=nbytes / (us * 1e-6) / 1e9, peak=PEAK_BYTES / 1e9, unit="GB/s",
                              frac=nbytes / (us * 1e-6) / PEAK_BYTES, traffic=None, kernel="kv_store_kernel<8, false>",
                              launch_us=us, bytes_per_launch=nbytes,
                              note="3 MB per launch: bound by the launch, not by HBM"),
                parity=dict(bit_exact=exact, rows="layer 0, whole cache, vs CPU oracle"), **forms)


def run_rope(torch, kernels, name, steps, warmup, with_cpu):
    """One step = rope_normal_batch on the Q rows and on the K rows of a 512-token chunk, per layer."""
    from oracle import ref
    shape_name, _, n_ctx, (P, B) = WORKLOADS[name]
    s = SHAPES[shape_name]
    H, G, d, layers = s["H"], s["G"], s["d"], s["layers"]
    theta = 500000.0
    g = torch.Generator(device="cuda")
    g.manual_seed(79)
    q0 = torch.randn((B * H, d), generator=g, device="cuda")
    k0 = torch.randn((B * G, d), generator=g, device="cuda")
    stack = [(q0.clone(), k0.clone()) for _ in range(layers)]
    kernels.rope_normal_batch(stack[0][0], B * H, d, d, theta, P, H)
    kernels.rope_normal_batch(stack[0][1], B * G, d, d, theta, P, G)
    torch.cuda.synchronize()
    wq = ref.rope_batch(q0.cpu().numpy(), d, d, theta, P, H, None, False)
    wk = ref.rope_batch(k0.cpu().numpy(), d, d, theta, P, G, None, False)
    err = max(float(np.abs(stack[0][0].cpu().numpy() - wq).max() / np.abs(wq).max()),
              float(np.abs(stack[0][1].cpu().numpy() - wk).max() / np.abs(wk).max()))

    def one_step():
        for q, k in stack:
            kernels.rope_normal_batch(q, B * H, d, d, theta, P, H)
            kernels.rope_normal_batch(k, B * G, d, d, theta, P, G)

    wall, dev_ms, forms = time_eager_and_graph(torch, kernels, one_step, steps, warmup)
    us = dev_ms * 1e3 / (steps * layers)
    # beside it: the chunk's whole way into the cache -- rope on Q, rope on K, kv_store_batch -- as the three
    # calls of the reference and as the one call that stands for them
    vv = torch.randn((B * G, d), generator=g, device="cuda")
    caches = [(torch.zeros((G, n_ctx, d), dtype=torch.int16, device="cuda"),
               torch.zeros((G, n_ctx, d), dtype=torch.int16, device="cuda")) for _ in range(layers)]

    def three_calls():
        for (q, k), (kc, vc) in zip(stack, caches):
            kernels.rope_normal_batch(q, B * H, d, d, theta, P, H)
            kernels.rope_normal_batch(k, B * G, d, d, theta, P, G)
            kernels.kv_store_batch(kc, vc, k, vv, G, d, n_ctx, P, B)

    def one_call():
        for (q, k), (kc, vc) in zip(stack, caches):
            kernels.rope_store_batch(q, k, vv, kc, vc, B, H, G, d, n_ctx, P, d, theta, None, False)

    _, dev3, _ = time_eager_and_graph(torch, kernels, three_calls, steps, warmup)
    _, dev1, _ = time_eager_and_graph(torch, kernels, one_call, steps, warmup)
    forms["into_the_cache"] = dict(three_calls_us=dev3 * 1e3 / (steps * layers), one_call_us=dev1 * 1e3 / (steps * layers),
                                   note="rope on Q + rope on K + kv_store_batch per layer; one_call: orin_fa_rope_store_batch")
    nbytes = 2.0 * B * (H + G) * d * 4
    return dict(value=nbytes * layers * steps / wall / 1e9, unit="GB/s", ms_per_step=wall / steps * 1e3,
                config=dict(workload=name, shape=f"H{H} G{G} d{d}", layers=layers, n_past=P, batch=B, n_rot=d,
                            bytes_per_step=nbytes * layers),
                roofline=dict(bound="hbm", achieved=nbytes / (us * 1e-6) / 1e9, peak=PEAK_BYTES / 1e9, unit="GB/s",
                              frac=nbytes / (us * 1e-6) / PEAK_BYTES, traffic=None,
                              kernel="rope4_kernel<false, false>, Q rows then K rows", launch_us=us,
                              bytes_per_launch=nbytes, note="launch_us and bytes cover the two launches of a layer"),
                parity=dict(max_rel_to_tensor_max=err, rows="layer 0, all rows, vs CPU oracle"), **forms)


def run_kv_shift(torch, kernels, name, steps, warmup, with_cpu):
    """One step = kv_shift over the whole cache (all layers, K and V), in place."""
    from oracle import ref
    shape_name, _, n_ctx, (n_keep, shift) = WORKLOADS[name]
    s = SHAPES[shape_name]
    G, d, layers = s["G"], s["d"], s["layers"]
    g = torch.Generator(device="cuda")
    g.manual_seed(78)
    kc = torch.randint(1, 30000, (layers, G, n_ctx, d), generator=g, device="cuda", dtype=torch.int16)
    vc = torch.randint(1, 30000, (layers, G, n_ctx, d), generator=g, device="cuda", dtype=torch.int16)
    # parity on the first launch, against the oracle on two layers' worth of the same data
    hk, hv = kc[:2].cpu().numpy().view(np.uint16).copy(), vc[:2].cpu().numpy().view(np.uint16).copy()
    ref.kv_shift_u16(hk, hv, 2, G, d, n_ctx, n_keep, shift)
    kernels.kv_shift(kc, vc, layers, G, d, n_ctx, n_keep, shift)
    torch.cuda.synchronize()
    exact = bool(np.array_equal(kc[:2].cpu().numpy().view(np.uint16), hk) and
                 np.array_equal(vc[:2].cpu().numpy().view(np.uint16), hv))
    for _ in range(warmup):
        kernels.kv_shift(kc, vc, layers, G, d, n_ctx, n_keep, shift)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        kernels.kv_shift(kc, vc, layers, G, d, n_ctx, n_keep, shift)
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    us = e0.elapsed_time(e1) * 1e3 / steps
    moved = n_ctx - n_keep - shift
    nbytes = 2.0 * layers * G * d * 2 * (moved + moved + shift)  # rows read + rows written + rows cleared, K and V
    return dict(value=nbytes * steps / wall / 1e9, unit="GB/s", ms_per_step=wall / steps * 1e3,
                config=dict(workload=name, shape=f"G{G} d{d}", layers=layers, n_ctx=n_ctx, n_keep=n_keep, shift=shift,
                            bytes_per_step=nbytes),
                roofline=dict(bound="hbm", achieved=nbytes / (us * 1e-6) / 1e9, peak=PEAK_BYTES / 1e9, unit="GB/s",
                              frac=nbytes / (us * 1e-6) / PEAK_BYTES, traffic=None, kernel="kv_shift_kernel<16>",
                              launch_us=us, bytes_per_launch=nbytes),
                parity=dict(bit_exact=exact, rows="layers 0-1, whole strips, vs CPU oracle"))


def run_copy(torch, kernels, name, steps, warmup, with_cpu):
    """dst.copy_(src) over rotating buffer pairs larger than the last-level cache."""
    nbytes = WORKLOADS[name][3]
    pairs = [(torch.empty(nbytes, dtype=torch.uint8, device="cuda").fill_(i + 1),
              torch.empty(nbytes, dtype=torch.uint8, device="cuda")) for i in range(3)]
    for i in range(warmup):
        pairs[i % 3][1].copy_(pairs[i % 3][0])
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        pairs[i % 3][1].copy_(pairs[i % 3][0])
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    us = e0.elapsed_time(e1) * 1e3 / steps
    return dict(value=2.0 * nbytes * steps / wall / 1e9, unit="GB/s", ms_per_step=wall / steps * 1e3,
                config=dict(workload=name, bytes_read_per_step=nbytes, bytes_written_per_step=nbytes),
                roofline=dict(bound="hbm", achieved=2.0 * nbytes / (us * 1e-6) / 1e9, peak=PEAK_BYTES / 1e9, unit="GB/s",
                              frac=2.0 * nbytes / (us * 1e-6) / PEAK_BYTES, traffic=2.0 * nbytes,
                              kernel="torch copy kernel (read + write)", launch_us=us),
                parity=None)


def run_read(torch, kernels, name, steps, warmup, with_cpu):
    """A kernel that only reads: `nbytes` per launch, launched back to back over buffers that rotate through
    more memory than the last-level cache holds; the best of three load shapes is reported, all are listed.
    One step = 28 launches (a decode stack's worth).  Beside it, the launch-to-launch time of a one-wave kernel."""
    nbytes = WORKLOADS[name][3]
    launches = 28
    n_buf = max(launches, int(np.ceil(1.2e9 / nbytes)))
    pool = torch.empty(n_buf * nbytes, dtype=torch.uint8, device="cuda").fill_(1)
    bufs = [pool[i * nbytes:(i + 1) * nbytes] for i in range(n_buf)]
    sink = torch.zeros(128, dtype=torch.int32, device="cuda")  # (words the kernels never write)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    shapes, wall_best = {}, None
    for per in (16, 4, 2):
        k = 0

        def one_step():
            nonlocal k
            for _ in range(launches):
                kernels.bench_hbm_read(bufs[k % n_buf], nbytes, sink, per)
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
        wall = time.perf_counter() - t0
        us = e0.elapsed_time(e1) * 1e3 / (steps * launches)
        shapes[f"{per}_loads_per_thread"] = us
        if wall_best is None or us < best_us:
            best_us, wall_best = us, wall
    # launch-to-launch time of a one-wave kernel, replayed from a graph so that the host's own pace does not count
    g = torch.cuda.CUDAGraph()
    try:
        with torch.cuda.graph(g):
            kernels.set_stream(torch.cuda.current_stream().cuda_stream)
            for _ in range(200):
                kernels.bench_tiny_launch(sink, sink[64:])
    finally:
        kernels.set_stream(torch.cuda.current_stream().cuda_stream)
    g.replay()
    torch.cuda.synchronize()
    e0.record()
    for _ in range(5):
        g.replay()
    e1.record()
    torch.cuda.synchronize()
    tiny_us = e0.elapsed_time(e1) * 1e3 / 1000
    del g
    del bufs, pool
    torch.cuda.empty_cache()
    return dict(value=nbytes * launches * steps / wall_best / 1e9, unit="GB/s", ms_per_step=wall_best / steps * 1e3,
                config=dict(workload=name, bytes_per_launch=nbytes, launches_per_step=launches, buffers_rotated=n_buf),
                roofline=dict(bound="hbm", achieved=nbytes / (best_us * 1e-6) / 1e9, peak=PEAK_BYTES / 1e9, unit="GB/s",
                              frac=nbytes / (best_us * 1e-6) / PEAK_BYTES, traffic=float(nbytes),
                              kernel="hbm_read_kernel (plain streaming read, not part of the path)", launch_us=best_us,
                              launch_us_by_shape=shapes, tiny_kernel_launch_to_launch_us=tiny_us,
                              bytes_per_launch=nbytes),
                parity=None)


def random_weight(torch, gen, wtype, n_in, n_out, std=0.03):
    """Random blocks of a weight type with sane fp16 scales (every other byte random), on the device."""
    per, nbytes = {0: (1, 4), 1: (1, 2), 8: (32, 34), 12: (256, 144), 13: (256, 176), 14: (256, 210)}[wtype]
    nb = n_in // per * n_out
    if wtype in (0, 1):
        w = torch.randn((n_out, n_in), generator=gen, device="cuda") * std
        return (w if wtype == 0 else w.half()).contiguous().view(torch.uint8).reshape(-1)
    raw = torch.randint(0, 256, (nb, nbytes), generator=gen, device="cuda", dtype=torch.uint8)
    halves = raw.view(torch.float16)  # [nb][nbytes / 2]
    u = torch.rand(nb, generator=gen, device="cuda") + 0.5
    if wtype == 8:
        halves[:, 0] = (std / 74.0 * u).half()
    elif wtype == 12:
        halves[:, 0] = (std / 166.0 * u).half()
        halves[:, 1] = (std / 166.0 * 7.5 * u).half()
    elif wtype == 13:
        halves[:, 0] = (std / 340.0 * u).half()
        halves[:, 1] = (std / 340.0 * 15.5 * u).half()
    else:
        halves[:, 104] = (std / 1369.0 * u).half()
    return raw.reshape(-1)


def run_decode_layer(torch, kernels, name, steps, warmup, with_cpu):
    """One step = one token through every layer of the model: orin_decode_layer per layer (six launches:
    norm + q/k/v projections, rotary embedding + cache store + attention, output projection,
    norm + gate/up + SwiGLU, down projection), replayed as one HIP graph as the reference replays its decode
    step (src/model_gpu.cu:295-344).  value = HBM bytes the layer must read (its weights once, its cache
    once) per second."""
    from oracle import ref
    from orin_llm_amd import layer as ly

    shape_name, _, n_ctx, L = WORKLOADS[name]
    s = SHAPES[shape_name]
    H, G, d, layers, ne, nff = s["H"], s["G"], s["d"], s["layers"], s["n_embd"], s["n_ff"]
    Q4, Q6 = ly.Q4_K, ly.Q6_K
    types = dict(wq=Q4, wk=Q4, wv=Q6, wo=Q4, ffn_gate=Q4, ffn_up=Q4, ffn_down=Q6)
    dims = dict(wq=(ne, H * d), wk=(ne, G * d), wv=(ne, G * d), wo=(H * d, ne), ffn_gate=(ne, nff), ffn_up=(ne, nff),
                ffn_down=(nff, ne))
    hp = dict(n_embd=ne, n_head=H, n_kv=G, head_dim=d, n_ff=nff, n_rot=d, neox=s["neox"], rms_eps=1e-6, rope_theta=s["theta"],
              freq_factors_dev=None)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(4242)
    weight_bytes = sum(ly.row_bytes(types[k], dims[k][0]) * dims[k][1] for k in types)
    kv_bytes = 4.0 * G * L * d
    bytes_layer = weight_bytes + kv_bytes
    model = []
    for l in range(layers):
        Lw = {k: (types[k], random_weight(torch, gen, types[k], *dims[k])) for k in types}
        Lw["attn_norm"] = 1.0 + 0.1 * torch.randn(ne, generator=gen, device="cuda")
        Lw["ffn_norm"] = 1.0 + 0.1 * torch.randn(ne, generator=gen, device="cuda")
        if s["bias"]:
            Lw["bq"], Lw["bk"], Lw["bv"] = (0.1 * torch.randn(n, generator=gen, device="cuda") for n in (H * d, G * d, G * d))
        k = torch.randn((G, n_ctx, d), generator=gen, device="cuda", dtype=torch.float32).half().view(torch.int16)
        v = torch.randn((G, n_ctx, d), generator=gen, device="cuda", dtype=torch.float32).half().view(torch.int16)
        model.append((Lw, k, v))
    z = lambda n: torch.zeros(n, dtype=torch.float32, device="cuda")  # noqa: E731
    bufs = dict(x=z(ne), q=z(H * d), k=z(G * d), v=z(G * d), attn=z(H * d), act=z(nff), up_tmp=z(nff), xn=z(ne), xn2=z(ne))
    x0 = torch.randn(ne, generator=gen, device="cuda")
    dpos = torch.tensor([L - 1], dtype=torch.int32, device="cuda")
    angles = torch.zeros((d // 2, 2), device="cuda")
    descs = [ly.make_desc(hp, Lw, bufs, k, v, dpos, n_ctx, rope_angles=angles) for Lw, k, v in model]

    def one_step():
        bufs["x"].copy_(x0)
        kernels.rope_angles_ind(angles, d, s["theta"], dpos)
        for dsc in descs:
            ly.decode_layer(dsc)

    def one_step_calls():  # the reference's own sequence of operator calls (src/model_gpu.cu:251-293)
        bufs["x"].copy_(x0)
        for Lw, k, v in model:
            ly.decode_layer_calls(hp, Lw, bufs, k, v, dpos, n_ctx)

    wall, dev_ms, forms = time_eager_and_graph(torch, kernels, one_step, steps, warmup)
    us_layer = dev_ms * 1e3 / (steps * layers)
    _, dev_calls_ms, forms_calls = time_eager_and_graph(torch, kernels, one_step_calls, max(3, steps // 2), min(warmup, 2))
    us_layer_calls = dev_calls_ms * 1e3 / (max(3, steps // 2) * layers)

    # Each kind of launch by itself: the same launch of every layer back to back between one pair of events (every
    # layer has its own weights and cache, so the bytes come from HBM), per launch; a few ten nanoseconds of launch
    # gap included.
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    scale_f = float(1.0 / np.sqrt(d))
    launches = {
        "norm + q,k,v (one launch)": lambda Lw, k, v: ly.gemv_multi_types(
            [Q4, Q4, Q6], [Lw["wq"][1], Lw["wk"][1], Lw["wv"][1]], [Lw.get("bq"), Lw.get("bk"), Lw.get("bv")],
            [bufs["q"], bufs["k"], bufs["v"]], [H * d, G * d, G * d], bufs["x"], Lw["attn_norm"], 1e-6, ne),
        "rope + store + attention (two launches)": lambda Lw, k, v: kernels.flash_attention_decode_rope_store_ind(
            bufs["q"], bufs["k"], bufs["v"], k, v, bufs["attn"], H, G, d, n_ctx, dpos, scale_f, d, s["theta"], None, bool(s["neox"]), angles),
        "output projection (+=)": lambda Lw, k, v: ly.gemv_multi(Q4, [Lw["wo"][1]], None, [bufs["x"]], [ne], bufs["attn"], None, 0.0, H * d, True),
        "norm + gate/up + SwiGLU": lambda Lw, k, v: ly.gemv_norm_gate_up_swiglu(Q4, Lw["ffn_gate"][1], Lw["ffn_up"][1], bufs["x"], Lw["ffn_norm"],
                                                                               1e-6, bufs["act"], ne, nff),
        "down projection (+=)": lambda Lw, k, v: ly.gemv_multi(Q6, [Lw["ffn_down"][1]], None, [bufs["x"]], [ne], bufs["act"], None, 0.0, nff, True),
    }
    launch_bytes = {"norm + q,k,v (one launch)": ly.row_bytes(Q4, ne) * (H + G) * d + ly.row_bytes(Q6, ne) * G * d,
                    "rope + store + attention (two launches)": kv_bytes, "output projection (+=)": ly.row_bytes(Q4, H * d) * ne,
                    "norm + gate/up + SwiGLU": 2 * ly.row_bytes(Q4, ne) * nff, "down projection (+=)": ly.row_bytes(Q6, nff) * ne}
    launch_us = {}
    bufs["x"].copy_(x0)
    for what, fn in launches.items():
        g = torch.cuda.CUDAGraph()  # (a graph, so that the host's launch rate does not price the short ones)
        try:
            with torch.cuda.graph(g):
                kernels.set_stream(torch.cuda.current_stream().cuda_stream)
                for Lw, k, v in model:
                    fn(Lw, k, v)
        finally:
            kernels.set_stream(torch.cuda.current_stream().cuda_stream)
        ts = []
        for rep in range(6):
            torch.cuda.synchronize()
            ev[0].record()
            g.replay()
            ev[1].record()
            torch.cuda.synchronize()
            ts.append(ev[0].elapsed_time(ev[1]) * 1e3 / layers)
        del g
        bufs["x"].copy_(x0)  # (the accumulating launches have moved it)
        launch_us[what] = dict(us=round(float(np.median(ts)), 2), MB=round(launch_bytes[what] / 1e6, 2),
                               GBps=round(launch_bytes[what] / (float(np.median(ts)) * 1e-6) / 1e9, 1))
    Lw, k0, v0 = model[0]

    # Parity: layer 0 from x0, against the oracle's operators in the reference's order (fp16 cache).
    bufs["x"].copy_(x0)
    kernels.rope_angles_ind(angles, d, s["theta"], dpos)
    kc_before, vc_before = k0.clone(), v0.clone()
    ly.decode_layer(descs[0])
    torch.cuda.synchronize()
    got = bufs["x"].cpu().numpy()
    t0 = time.perf_counter()
    host = {k: (v[0], v[1].cpu().numpy()) if isinstance(v, tuple) else v.cpu().numpy() for k, v in Lw.items()}
    mv = lambda key, x: ref.gemv(host[key][0], host[key][1], x, dims[key][0], dims[key][1])  # noqa: E731
    xh = x0.cpu().numpy()
    t_cpu0 = time.perf_counter()
    xn = ref.rms_norm(xh, host["attn_norm"], 1e-6)
    qh, kh, vh = mv("wq", xn), mv("wk", xn), mv("wv", xn)
    if s["bias"]:
        qh, kh, vh = qh + host["bq"], kh + host["bk"], vh + host["bv"]
    qh = ref.rope_batch(qh.reshape(H, d), d, d, s["theta"], L - 1, H, None, bool(s["neox"]))
    kh = ref.rope_batch(kh.reshape(G, d), d, d, s["theta"], L - 1, G, None, bool(s["neox"]))
    kc_h, vc_h = kc_before.cpu().numpy().view(np.uint16).copy(), vc_before.cpu().numpy().view(np.uint16).copy()
    ref.kv_store_f16(kc_h, vc_h, kh.reshape(1, G, d), vh.reshape(1, G, d), G, d, n_ctx, L - 1, 1)
    attn = ref.flash_attention_decode_ind(qh, kc_h, vc_h, H, G, d, n_ctx, L - 1, float(1.0 / np.sqrt(d))).reshape(-1)
    x1 = xh + mv("wo", attn)
    act = ref.swiglu(mv("ffn_gate", ref.rms_norm(x1, host["ffn_norm"], 1e-6)), mv("ffn_up", ref.rms_norm(x1, host["ffn_norm"], 1e-6)))
    want = x1 + mv("ffn_down", act)
    cpu_s = time.perf_counter() - t_cpu0
    err = float(np.abs(got.astype(np.float64) - want).max() / np.abs(want).max())
    # the token's cache rows: fp16 roundings of projections that differ in the last bits of their fp32 sums
    row_k = ref.fp16_to_fp32(k0.cpu().numpy().view(np.uint16)[:, L - 1]) - ref.fp16_to_fp32(kc_h[:, L - 1])
    row_v = ref.fp16_to_fp32(v0.cpu().numpy().view(np.uint16)[:, L - 1]) - ref.fp16_to_fp32(vc_h[:, L - 1])
    cache_err = float(max(np.abs(row_k).max() / np.abs(ref.fp16_to_fp32(kc_h[:, L - 1])).max(),
                          np.abs(row_v).max() / np.abs(ref.fp16_to_fp32(vc_h[:, L - 1])).max()))
    main_key = "norm + gate/up + SwiGLU"
    res = dict(value=bytes_layer * layers * steps / (dev_ms * 1e-3) / 1e9, unit="GB/s", ms_per_step=wall / steps * 1e3,
               config=dict(workload=name, shape=f"H{H} G{G} d{d} n_embd {ne} n_ff {nff}", layers=layers, n_ctx=n_ctx, L=L,
                           weights="Q4_K, attn_v and ffn_down Q6_K", weight_MB_per_layer=round(weight_bytes / 1e6, 2),
                           cache_MB_per_layer=round(kv_bytes / 1e6, 2), launch="graph" if forms["graph"]["device_ms_per_step"] <= forms["eager"]["device_ms_per_step"] else "eager"),
               roofline=dict(bound="hbm", achieved=launch_bytes[main_key] / (launch_us[main_key]["us"] * 1e-6) / 1e9, peak=PEAK_BYTES / 1e9,
                             unit="GB/s", frac=launch_bytes[main_key] / (launch_us[main_key]["us"] * 1e-6) / PEAK_BYTES, traffic=None,
                             kernel="gemv_rows_kernel<Q4_K, two matrices> (norm + gate/up + SwiGLU)", launch_us=launch_us[main_key]["us"],
                             bytes_per_launch=launch_bytes[main_key], layer_us=us_layer, layer_frac=bytes_layer / (us_layer * 1e-6) / PEAK_BYTES,
                             layer_us_reference_call_sequence=us_layer_calls, launches=launch_us),
               parity=dict(err_row=err, err_floor1pct=err, cache_row_err=cache_err,
                           rows="layer 0's output vector, max |got - want| / max |want|, vs the CPU oracle's operators in the reference's order"),
               **forms)
    if with_cpu:
        res["cpu_baseline"] = dict(value=bytes_layer / cpu_s / 1e9, unit="GB/s", cores=1, kind="port",
                                   sample=f"layer 0 of {layers}, every operator, {cpu_s:.1f} s")
    return res


def run_logits(torch, kernels, name, steps, warmup, with_cpu):
    """One step = the last RMS norm and the output matrix (Q6_K, vocabulary x n_embd) over one token's residual
    stream: orin_rms_norm + orin_gemv, as the reference ends a decode step (src/model_gpu.cu:303-306); replayed
    from a graph over copies of the matrix that rotate through more memory than the last-level cache holds.
    value = bytes of the matrix per second."""
    from oracle import ref
    from orin_llm_amd import layer as ly

    shape_name, _, _, n_vocab = WORKLOADS[name]
    ne = SHAPES[shape_name]["n_embd"]
    wt = ly.Q6_K
    nbytes = ly.row_bytes(wt, ne) * n_vocab
    n_copies = max(2, int(np.ceil(0.6e9 / nbytes)))
    gen = torch.Generator(device="cuda")
    gen.manual_seed(777)
    ws = [random_weight(torch, gen, wt, ne, n_vocab) for _ in range(n_copies)]
    x = torch.randn(ne, generator=gen, device="cuda")
    nw = 1.0 + 0.1 * torch.randn(ne, generator=gen, device="cuda")
    xn, y = torch.zeros(ne, device="cuda"), torch.zeros(n_vocab, device="cuda")
    k = 0

    def one_step():
        nonlocal k
        ly.rms_norm(x, nw, ne, 1e-6, xn)
        ly.gemv(wt, ws[k % n_copies], xn, y, ne, n_vocab)
        k += 1

    g = torch.cuda.CUDAGraph()
    try:
        with torch.cuda.graph(g):
            kernels.set_stream(torch.cuda.current_stream().cuda_stream)
            for _ in range(n_copies):
                one_step()
    finally:
        kernels.set_stream(torch.cuda.current_stream().cuda_stream)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
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
    us = e0.elapsed_time(e1) * 1e3 / (steps * n_copies)
    del g
    # parity: a sample of rows of the last matrix used, against the oracle's product over the oracle's norm
    k = 0
    one_step()
    torch.cuda.synchronize()
    got = y.cpu().numpy()
    rb = ly.row_bytes(wt, ne)
    xh, nwh = x.cpu().numpy(), nw.cpu().numpy()
    t_cpu = time.perf_counter()
    xnh = ref.rms_norm(xh, nwh, 1e-6)
    rows = sorted(set([0, 1, 15, 16, n_vocab // 2, n_vocab - 17, n_vocab - 1]) | set(int(r) for r in np.random.default_rng(5).integers(0, n_vocab - 256, 41)))
    err, n_rows = 0.0, 0
    for r in rows:
        m = min(256, n_vocab - r)
        want = ref.gemv(wt, ws[0][r * rb:(r + m) * rb].cpu().numpy(), xnh, ne, m).astype(np.float64)
        err = max(err, float(np.abs(got[r:r + m] - want).max() / max(np.abs(want).max(), 1e-30)))
        n_rows += m
    cpu_s = time.perf_counter() - t_cpu
    res = dict(value=nbytes * n_copies * steps / wall / 1e9, unit="GB/s", ms_per_step=wall / steps * 1e3 / n_copies,
               config=dict(workload=name, shape=f"n_embd {ne}, vocabulary {n_vocab}", weights="Q6_K", MB=round(nbytes / 1e6, 1),
                           copies_rotated=n_copies, launch="graph"),
               roofline=dict(bound="hbm", achieved=nbytes / (us * 1e-6) / 1e9, peak=PEAK_BYTES / 1e9, unit="GB/s",
                             frac=nbytes / (us * 1e-6) / PEAK_BYTES, traffic=None,
                             kernel="rms_norm_kernel + gemv_rows_kernel<Q6_K> (last norm + output matrix)", launch_us=us,
                             bytes_per_launch=nbytes),
               parity=dict(err_row=err, err_floor1pct=err, rows=f"{n_rows} logits in runs of 256 (first, last, middle, random), max |got - want| / max |want| per run, vs the CPU oracle"))
    if with_cpu:
        res["cpu_baseline"] = dict(value=n_rows * rb / cpu_s / 1e9, unit="GB/s", cores=1, kind="port", sample=f"{n_rows} of {n_vocab} rows, {cpu_s:.1f} s")
    del ws
    torch.cuda.empty_cache()
    return res


def run(torch, kernels, name, steps, warmup, with_cpu):
    kind = WORKLOADS[name][1]
    if kind in ("patterns", "handoff", "timeline", "cutoffs"):  # measurement aids, not the operator
        import bench_aids

        fn = dict(patterns=bench_aids.run_patterns, handoff=bench_aids.run_handoff, timeline=bench_aids.run_timeline,
                  cutoffs=bench_aids.run_cutoffs)[kind]
    else:
        fn = dict(decode_layer=run_decode_layer, prefill=run_prefill, decode=run_decode, decode_store=run_decode,
                  decode_rope_store=run_decode, logits=run_logits, copy=run_copy, read=run_read, kv_store=run_kv_store,
                  kv_shift=run_kv_shift, rope=run_rope)[kind]
    return fn(torch, kernels, name, steps, warmup, with_cpu)


def _sig(x, digits=4):
    return None if x is None else float(f"{float(x):.{digits}g}")


def target_summary(res):
    """The few figures of one workload's result that the compact line carries under "targets"."""
    rf, par = res["roofline"], res.get("parity") or {}
    if "layer_us" in rf:  # the decode layer around the path
        t = dict(layer_us=round(rf["layer_us"], 2), layer_frac=round(rf["layer_frac"], 4),
                 ref_calls_us=round(rf["layer_us_reference_call_sequence"], 2),
                 gate_up_us=round(rf["launch_us"], 2), gate_up_frac=round(rf["frac"], 4))
    else:
        t = dict(frac=round(rf["frac"], 4), achieved=round(rf["achieved"], 1), unit=rf["unit"],
                 launch_us=round(rf["launch_us"], 2))
        if "tiny_kernel_launch_to_launch_us" in rf:
            t["tiny_launch_us"] = round(rf["tiny_kernel_launch_to_launch_us"], 2)
    if "err_row" in par:
        t["err_row"] = _sig(par["err_row"], 3)
        if "layer_us" not in rf:
            t["err_floor1pct"] = _sig(par["err_floor1pct"], 3)
    if "cpu_baseline" in res:
        t["cpu_1core"] = _sig(res["cpu_baseline"]["value"])
    return t


def compact_line(main_res, also, steps, warmup):
    """The line the driver parses: the contract's keys, the headline's roofline, cpu_baseline and parity, and
    "targets" (target_summary of the other workloads of the run).  Everything long (notes, per-launch tables,
    eager/graph forms, samples' prose) stays in the full record."""
    rf = main_res["roofline"]
    cfg = main_res["config"]
    line = dict(
        metric="prefill attn TFLOP/s + decode attn HBM GB/s (% of peak), Qwen2.5-1.5B GQA",
        value=_sig(main_res["value"], 6), unit=main_res["unit"], n_gpus=1, steps=steps, warmup=warmup,
        ms_per_step=_sig(main_res["ms_per_step"], 6), higher_is_better=True, scaling="weak", vs_baseline=None,
        dtype="f16", data="synthetic",
        config={k: cfg[k] for k in ("workload", "shape", "layers", "n_ctx", "chunks", "L", "launch") if k in cfg},
        roofline=dict(bound=rf["bound"], achieved=_sig(rf["achieved"], 6), peak=rf["peak"], unit=rf["unit"],
                      frac=_sig(rf["frac"], 4), traffic=rf.get("traffic"), kernel=rf.get("kernel"),
                      launch_us=_sig(rf.get("launch_us"))),
    )
    for k in ("flops_per_launch", "bytes_per_launch", "launch_us_back_to_back"):
        if k in rf:
            line["roofline"][k] = _sig(rf[k], 6)
    if "per_chunk" in main_res:
        line["per_chunk"] = [dict(P=c["P"], B=c["B"], launch_us=round(c["launch_us"], 2), frac=round(c["frac"], 4))
                             for c in main_res["per_chunk"]]
    cb = main_res.get("cpu_baseline")
    if cb:
        line["cpu_baseline"] = dict(value=_sig(cb["value"]), unit=cb["unit"], cores=cb["cores"], kind=cb["kind"],
                                    sample=cb["sample"][:160])
        if "all_cores" in cb:
            line["cpu_baseline"]["all_cores"] = dict(value=_sig(cb["all_cores"]["value"]), cores=cb["all_cores"]["cores"])
    par = main_res.get("parity")
    if par:
        line["parity"] = {k: (_sig(v, 3) if isinstance(v, float) else v) for k, v in par.items() if k != "rows"}
    if also:
        line["targets"] = {a["config"]["workload"]: target_summary(a) for a in also if a["config"]["workload"] in TARGETS}
    return line


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="qwen1.5b-prefill512", choices=sorted(WORKLOADS))
    ap.add_argument("--no-also", action="store_true", help="skip the other target workloads")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--full", action="store_true", help="also run the neighbouring operators' workloads (minutes)")
    ap.add_argument("--full-record", default=os.path.join(ROOT, "gpurun_out", "bench_full.json"),
                    help="where every workload's full result is written ('' = nowhere)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (the path has no cross-GPU part); use --gpus 1")

    import torch

    from orin_llm_amd import kernels

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    kernels.init(0)
    kernels.set_stream(torch.cuda.current_stream().cuda_stream)

    main_res = run(torch, kernels, args.workload, args.steps, args.warmup, not args.no_cpu)
    if TRAFFIC_COMMIT:
        main_res["roofline"]["traffic_measured_at_commit"] = TRAFFIC_COMMIT
    also = []
    if not args.no_also:
        for name in (ALSO_FULL if args.full else []) + ALSO:
            if name == args.workload:
                continue
            also.append(run(torch, kernels, name, max(3, min(args.steps, 10)), min(args.warmup, 2),
                            name in ALSO_CPU and not args.no_cpu))
    if args.full_record:
        try:
            os.makedirs(os.path.dirname(args.full_record), exist_ok=True)
            with open(args.full_record, "w") as f:
                json.dump(dict(steps=args.steps, warmup=args.warmup, main=main_res, also=also), f, indent=1)
        except OSError as e:
            print(f"bench.py: full record not written ({e})", file=sys.stderr)
    print(json.dumps(compact_line(main_res, also, args.steps, args.warmup)), flush=True)


if __name__ == "__main__":
    main()
