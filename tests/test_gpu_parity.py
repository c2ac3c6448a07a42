"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle.

Tolerance (written once, in util.py, used everywhere): TOL = 2e-3 on rel_err()[0], the maximum
error of any fp32 output element relative to the largest magnitude in its own (token, head)
row; and on rel_err()[1], the element-wise error with a floor of 1 % of the row maximum,
FLOOR_DECODE = 2e-3 for decode and the bound FLOOR_PREFILL = 4e-2 for prefill.
"""
import numpy as np
import pytest

from oracle import ref
from util import FLOOR_DECODE, FLOOR_FP32_KV, FLOOR_PREFILL, TOL, make_case, rel_err

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fa():
    torch = pytest.importorskip("torch")
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from orin_llm_amd import kernels

    kernels.init(0)
    kernels.set_stream(torch.cuda.current_stream().cuda_stream)
    return kernels


def _dev(a):
    import torch

    t = torch.from_numpy(np.ascontiguousarray(a))
    if t.dtype == torch.uint16:
        t = t.view(torch.int16)
    return t.cuda()


def gpu_prefill(fa, q, kc, vc, n_head, n_kv, d, n_ctx, n_past, batch, scale, pad_rows=2):
    """Runs the prefill operator; the output buffer carries sentinel rows past `batch`."""
    import torch

    dq, dk, dv = _dev(q), _dev(kc), _dev(vc)
    out = torch.full((batch + pad_rows, n_head, d), 12345.0, dtype=torch.float32, device="cuda")
    fa.flash_attention(dq, dk, dv, out, n_head, n_kv, d, n_ctx, n_past, batch, float(scale))
    torch.cuda.synchronize()
    o = out.cpu().numpy()
    assert (o[batch:] == 12345.0).all(), "rows past batch were written"
    return o[:batch]


def gpu_decode(fa, q, kc, vc, n_head, n_kv, d, n_ctx, pos, scale, dk=None, dv=None):
    import torch

    dq = _dev(q)
    dk = _dev(kc) if dk is None else dk
    dv = _dev(vc) if dv is None else dv
    dpos = torch.tensor([pos], dtype=torch.int32, device="cuda")
    out = torch.full((n_head + 1, d), 12345.0, dtype=torch.float32, device="cuda")
    fa.flash_attention_decode_ind(dq, dk, dv, out, n_head, n_kv, d, n_ctx, dpos, float(scale))
    torch.cuda.synchronize()
    o = out.cpu().numpy()
    assert (o[n_head:] == 12345.0).all()
    return o[:n_head]


def check(got, want, what, tol=TOL, floor=FLOOR_PREFILL):
    row, floor1pct, l2 = rel_err(got, want)
    print(f"{what}: err_row {row:.3e} (gate {tol:g})  floor1pct {floor1pct:.3e} (gate {floor:g})  l2 {l2:.3e}", flush=True)
    assert np.isfinite(got).all(), what
    assert row < tol, (what, row, floor1pct, l2)
    assert floor1pct < floor, (what, row, floor1pct, l2)


# ---------------------------------------------------------------- config 1 (golden)

def test_cfg1_golden_prefill_then_decode(fa, cfg1):
    """45-token prefill into an empty cache, then 128 decode steps, against the attention
    outputs recovered from the unmodified reference CPU build's logits."""
    c = cfg1
    H, G, d = c["n_head"], c["n_kv"], c["d"]
    n_pre, n_dec = c["n_prefill"], c["n_decode"]
    n_tok = n_pre + n_dec
    n_ctx = 4096
    scale = 1.0 / np.sqrt(np.float32(d))
    kc = np.zeros((G, n_ctx, d), np.uint16)
    vc = np.zeros((G, n_ctx, d), np.uint16)
    ref.kv_store_f16(kc, vc, c["k"].reshape(n_tok, G, d), c["v"].reshape(n_tok, G, d), G, d, n_ctx, 0, n_tok)
    q = c["q"].reshape(n_tok, H, d)
    for variant in ("a", "b"):
        lg = c["logits_" + variant]
        want = (lg[:, :-1] / lg[:, -1:]).reshape(n_tok, H, d)
        got = gpu_prefill(fa, q[:n_pre], kc, vc, H, G, d, n_ctx, 0, n_pre, scale)
        check(got, want[:n_pre], f"cfg1{variant} prefill", floor=FLOOR_FP32_KV if variant == "a" else FLOOR_PREFILL)
        import torch

        dk, dv = _dev(kc), _dev(vc)
        dec = np.stack([gpu_decode(fa, q[t], None, None, H, G, d, n_ctx, t, scale, dk=dk, dv=dv)
                        for t in range(n_pre, n_tok)])
        check(dec, want[n_pre:], f"cfg1{variant} decode", floor=FLOOR_FP32_KV if variant == "a" else FLOOR_DECODE)
        del torch


# ---------------------------------------------------------------- brute force, small shapes

@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("r", [1, 2, 3, 4, 5, 6, 7, 8, 12, 20])
def test_decode_small(fa, d, r):
    G = 2
    H = G * r
    n_ctx = 384
    scale = 1.0 / np.sqrt(d)
    q, kc, vc = make_case(100 + r, H, G, d, n_ctx, n_ctx, 1, outliers=4)
    import torch

    dk, dv = _dev(kc), _dev(vc)
    for npos in (1, 2, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 260, 384):
        want = ref.flash_attention_decode_ind(q[0], kc, vc, H, G, d, n_ctx, npos - 1, np.float32(scale))
        got = gpu_decode(fa, q[0], None, None, H, G, d, n_ctx, npos - 1, scale, dk=dk, dv=dv)
        check(got, want, f"decode d{d} r{r} npos{npos}", floor=FLOOR_DECODE)
    del torch


@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("r", [1, 2, 3, 4, 5, 6, 7, 8, 11])
def test_prefill_small(fa, d, r):
    G = 2
    H = G * r
    n_ctx = 600
    scale = 1.0 / np.sqrt(d)
    cases = [(0, 1), (0, 2), (0, 17), (1, 16), (63, 9), (64, 8), (65, 7), (0, 45), (100, 33), (31, 130)]
    for n_past, batch in cases:
        q, kc, vc = make_case(200 + r + n_past, H, G, d, n_ctx, n_past + batch, batch, outliers=4, poison_tail=True)
        want = ref.flash_attention(q, kc, vc, H, G, d, n_ctx, n_past, batch, np.float32(scale))
        got = gpu_prefill(fa, q, kc, vc, H, G, d, n_ctx, n_past, batch, scale)
        check(got, want, f"prefill d{d} r{r} P{n_past} B{batch}")


def test_prefill_chunk_edges(fa):
    """batch 511..513 and a last chunk that ends exactly at n_ctx."""
    H, G, d = 12, 2, 128
    scale = 1.0 / np.sqrt(d)
    for n_ctx, n_past, batch in [(1024, 0, 511), (1024, 0, 512), (1024, 5, 513), (1024, 512, 512)]:
        q, kc, vc = make_case(300 + batch, H, G, d, n_ctx, n_past + batch, batch, outliers=4, poison_tail=True)
        rows = np.array([(t, h) for t in (0, 1, 7, 8, 15, 16, 255, batch - 2, batch - 1) for h in range(H)], np.int32)
        want = ref.flash_attention_rows(q, kc, vc, rows, H, G, d, n_ctx, n_past, np.float32(scale))
        got = gpu_prefill(fa, q, kc, vc, H, G, d, n_ctx, n_past, batch, scale)
        check(got[rows[:, 0], rows[:, 1]], want, f"prefill edges ctx{n_ctx} P{n_past} B{batch}")


@pytest.mark.parametrize("d,r", [(64, 1), (64, 4), (64, 7), (128, 1), (128, 2), (128, 3), (128, 5), (128, 8), (128, 12)])
def test_prefill_wide_blocks(fa, d, r):
    """Grids with more workgroups than half the CUs take the 64-column packing: every ratio's
    column -> (token, head) map, padded columns and the second head group (r = 12)."""
    G = 8
    H = G * r
    n_ctx = 1536
    scale = 1.0 / np.sqrt(d)
    n_past, batch = 200, 1100
    q, kc, vc = make_case(500 + r + d, H, G, d, n_ctx, n_past + batch, batch, outliers=2, poison_tail=True)
    toks = sorted({0, 1, 8, 9, 20, 21, 31, 32, 63, 64, 65, 500, batch - 2, batch - 1})
    rows = np.array([(t, h) for t in toks for h in range(H)], np.int32)
    want = ref.flash_attention_rows(q, kc, vc, rows, H, G, d, n_ctx, n_past, np.float32(scale))
    got = gpu_prefill(fa, q, kc, vc, H, G, d, n_ctx, n_past, batch, scale)
    check(got[rows[:, 0], rows[:, 1]], want, f"prefill wide d{d} r{r}")


@pytest.mark.parametrize("H,G,d,n_past,batch,scale", [
    (12, 2, 128, 4608, 512, 0.0883883),   # Qwen2.5-1.5B heads: two workgroups share a token tile's rows
    (12, 2, 128, 7680, 512, 0.0883883),
    (2, 1, 128, 4100, 1100, 0.0883883),   # four workgroups per token tile
    (1, 1, 64, 0, 5200, 0.125),           # from an empty cache: early token tiles leave splits without a row
    (8, 1, 64, 4900, 300, -0.3),          # a ragged end, negative scale (the rescaling path on most tiles)
    (3, 1, 128, 5200, 1, 0.0883883),      # one token: sixteen workgroups share its rows
    (12, 2, 128, 9000, 45, 0.0883883),    # a short last chunk of a long prompt: sixteen workgroups per token tile
    (12, 2, 128, 3100, 200, 0.0883883),   # four workgroups per token tile, from 3072 rows
])
def test_prefill_kv_splits(fa, H, G, d, n_past, batch, scale):
    """Few query columns on a long context: the launcher cuts a token tile's KV rows among 2 to
    16 workgroups and a second kernel merges their results.  Same oracle, same tolerance; every
    element of out is written (the buffer starts as a sentinel value)."""
    n_ctx = n_past + batch + 7
    q, kc, vc = make_case(900 + H + n_past, H, G, d, n_ctx, n_past + batch, batch, outliers=2, poison_tail=True)
    toks = sorted({0, 1, 4, 5, 9, 10, 31, 32, 63, 64, 127, 128, 129, 255, 256, 511, batch // 2, batch - 2, batch - 1}
                  & set(range(batch)))
    rows = np.array([(t, h) for t in toks for h in range(H)], np.int32)
    want = ref.flash_attention_rows(q, kc, vc, rows, H, G, d, n_ctx, n_past, np.float32(scale))
    got = gpu_prefill(fa, q, kc, vc, H, G, d, n_ctx, n_past, batch, scale)
    assert np.isfinite(got).all() and (got != 12345.0).all()
    check(got[rows[:, 0], rows[:, 1]], want, f"prefill kv splits H{H} G{G} d{d} P{n_past} B{batch}")


@pytest.mark.parametrize("scale", [1.0, 0.35, -0.0883883])
@pytest.mark.parametrize("H,G,batch", [(4, 2, 96), (32, 8, 600)])
def test_prefill_moving_reference(fa, scale, H, G, batch):
    """Large and negative scales: the scores of early tiles exceed the reference taken from the
    tiles next to the diagonal by far more than the fp16 range of the weights allows, so the
    rescaling path runs on most tiles (both column packings)."""
    d, n_ctx, n_past = 128, 1024, 300
    q, kc, vc = make_case(77 + batch, H, G, d, n_ctx, n_past + batch, batch, outliers=4, poison_tail=True)
    toks = sorted({0, 1, 31, 32, 33, batch // 2, batch - 1})
    rows = np.array([(t, h) for t in toks for h in range(H)], np.int32)
    want = ref.flash_attention_rows(q, kc, vc, rows, H, G, d, n_ctx, n_past, np.float32(scale))
    got = gpu_prefill(fa, q, kc, vc, H, G, d, n_ctx, n_past, batch, scale)
    check(got[rows[:, 0], rows[:, 1]], want, f"prefill scale {scale} H{H} B{batch}")


# ---------------------------------------------------------------- invariants on the GPU path

def test_prefill_row_equals_decode_and_chunk_split(fa):
    H, G, d, n_ctx = 28, 4, 128, 2048
    scale = 1.0 / np.sqrt(d)
    n_past, batch = 700, 200
    q, kc, vc = make_case(41, H, G, d, n_ctx, n_past + batch, batch, outliers=4, poison_tail=True)
    whole = gpu_prefill(fa, q, kc, vc, H, G, d, n_ctx, n_past, batch, scale)
    a = gpu_prefill(fa, q[:77], kc, vc, H, G, d, n_ctx, n_past, 77, scale)
    b = gpu_prefill(fa, q[77:], kc, vc, H, G, d, n_ctx, n_past + 77, batch - 77, scale)
    # (the weights are rounded to fp16 relative to a reference that depends on how the rows fall
    # into tiles, so two chunkings agree to the size of that rounding, not bit for bit)
    check(np.concatenate([a, b]), whole, "chunk split", tol=1e-3)
    for t in (0, 76, 199):
        dec = gpu_decode(fa, q[t], kc, vc, H, G, d, n_ctx, n_past + t, scale)
        check(dec, whole[t], f"prefill row {t} vs decode", tol=1e-3)  # (prefill against decode: the prefill bound)


def test_decode_ignores_cache_tail_and_position_is_read_on_device(fa):
    import torch

    H, G, d, n_ctx = 32, 8, 128, 8192
    scale = 1.0 / np.sqrt(d)
    L = 5000
    q, kc, vc = make_case(51, H, G, d, n_ctx, L, 1, poison_tail=True)
    dq, dk, dv = _dev(q), _dev(kc), _dev(vc)
    dpos = torch.zeros(1, dtype=torch.int32, device="cuda")
    out = torch.empty((H, d), dtype=torch.float32, device="cuda")
    rows = np.array([(0, h) for h in range(H)], np.int32)
    for pos in (L - 1, 17, 4095, 4096):
        dpos.fill_(pos)  # same launch arguments every time: only device memory changes
        fa.flash_attention_decode_ind(dq, dk, dv, out, H, G, d, n_ctx, dpos, float(scale))
        torch.cuda.synchronize()
        want = ref.flash_attention_rows(q, kc, vc, rows, H, G, d, n_ctx, pos, np.float32(scale))
        check(out.cpu().numpy(), want, f"decode pos {pos}", floor=FLOOR_DECODE)


def test_decode_graph_capture_replay(fa):
    """The decode call is captured once and replayed with the position changed in between
    (the reference's use: src/model_gpu.cu:295-316)."""
    import torch

    H, G, d, n_ctx = 12, 2, 128, 4096
    n_layer = 4
    scale = 1.0 / np.sqrt(d)
    cases = [make_case(60 + l, H, G, d, n_ctx, n_ctx, 1) for l in range(n_layer)]
    dq = [_dev(c[0]) for c in cases]
    dk = [_dev(c[1]) for c in cases]
    dv = [_dev(c[2]) for c in cases]
    outs = [torch.zeros((H, d), dtype=torch.float32, device="cuda") for _ in range(n_layer)]
    dpos = torch.zeros(1, dtype=torch.int32, device="cuda")
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    try:
        with torch.cuda.graph(graph):
            fa.set_stream(torch.cuda.current_stream().cuda_stream)
            for l in range(n_layer):
                fa.flash_attention_decode_ind(dq[l], dk[l], dv[l], outs[l], H, G, d, n_ctx, dpos, float(scale))
    finally:
        fa.set_stream(torch.cuda.current_stream().cuda_stream)
    rows = np.array([(0, h) for h in range(H)], np.int32)
    for pos in (0, 100, 4095, 1234, 31):
        dpos.fill_(pos)
        for o in outs:
            o.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for l in range(n_layer):
            want = ref.flash_attention_rows(cases[l][0], cases[l][1], cases[l][2], rows, H, G, d, n_ctx, pos,
                                            np.float32(scale))
            check(outs[l].cpu().numpy(), want, f"graph replay pos {pos} layer {l}", floor=FLOOR_DECODE)


# ---------------------------------------------------------------- the benchmark configurations at full size (row-sampled oracle)

def _sample_rows(rng, batch, H, r, extra_tokens=()):
    toks = {0, 1, 7, 8, 15, 16, 31, 32, 255, 256, batch - 2, batch - 1, *extra_tokens}
    toks = sorted(t for t in toks if 0 <= t < batch)
    rows = [(t, h) for t in (toks[0], toks[-1]) for h in range(H)]           # every head on first/last token
    rows += [(t, h) for t in toks for h in range(r)]                          # one whole GQA group on edge tokens
    rows += [(int(rng.integers(batch)), int(rng.integers(H))) for _ in range(64)]
    return np.array(sorted(set(rows)), np.int32)


@pytest.mark.parametrize("name,H,G,n_ctx,n_past,batch,outliers", [
    ("cfg2 qwen1.5b P0", 12, 2, 4096, 0, 512, 4),
    ("cfg2 qwen1.5b P3584", 12, 2, 4096, 3584, 512, 4),
    ("cfg4 llama8b P0", 32, 8, 8192, 0, 512, 0),
    ("cfg4 llama8b P4096", 32, 8, 8192, 4096, 512, 0),
    ("cfg4 llama8b P7680", 32, 8, 8192, 7680, 512, 0),
    ("cfg5 qwen7b P32256", 28, 4, 32768, 32256, 512, 4),
])
def test_prefill_full_configs(fa, name, H, G, n_ctx, n_past, batch, outliers):
    d = 128
    scale = 1.0 / np.sqrt(d)
    rng = np.random.default_rng(7)
    for layer in range(2):  # independent seeds per layer
        q, kc, vc = make_case(1000 + 17 * layer + n_past, H, G, d, n_ctx, n_past + batch, batch,
                              outliers=outliers, poison_tail=True)
        rows = _sample_rows(rng, batch, H, H // G)
        want = ref.flash_attention_rows(q, kc, vc, rows, H, G, d, n_ctx, n_past, np.float32(scale))
        got = gpu_prefill(fa, q, kc, vc, H, G, d, n_ctx, n_past, batch, scale)
        check(got[rows[:, 0], rows[:, 1]], want, f"{name} layer {layer}")


@pytest.mark.parametrize("name,H,G,n_ctx,L,outliers", [
    ("cfg3 qwen1.5b L1024", 12, 2, 32768, 1024, 0),
    ("cfg3 qwen1.5b L8192", 12, 2, 32768, 8192, 0),
    ("cfg3 qwen1.5b L32768", 12, 2, 32768, 32768, 0),
    ("cfg4 llama8b L8192", 32, 8, 8192, 8192, 0),
    ("cfg5 qwen7b L32767", 28, 4, 32768, 32767, 4),
])
def test_decode_full_configs(fa, name, H, G, n_ctx, L, outliers):
    d = 128
    scale = 1.0 / np.sqrt(d)
    rows = np.array([(0, h) for h in range(H)], np.int32)
    for layer in range(2):
        q, kc, vc = make_case(2000 + 13 * layer + L, H, G, d, n_ctx, L, 1, outliers=outliers, poison_tail=True)
        want = ref.flash_attention_rows(q, kc, vc, rows, H, G, d, n_ctx, L - 1, np.float32(scale))
        got = gpu_decode(fa, q[0], kc, vc, H, G, d, n_ctx, L - 1, scale)
        check(got, want, f"{name} layer {layer}", floor=FLOOR_DECODE)


def test_cfg2_full_stack_28_layers(fa):
    """Config 2 as written: the full 28-layer stack with independent seeds per layer, both chunks
    (cache start positions 0 and 3584), sampled rows of every layer against the oracle."""
    H, G, d, n_ctx, batch, layers = 12, 2, 128, 4096, 512, 28
    scale = 1.0 / np.sqrt(d)
    worst = 0.0
    for n_past in (0, 3584):
        for layer in range(layers):
            q, kc, vc = make_case(50000 + 100 * layer + (n_past > 0), H, G, d, n_ctx, n_past + batch, batch,
                                  outliers=4, poison_tail=True)
            rng = np.random.default_rng(layer)
            toks = sorted({0, batch - 1, *(int(t) for t in rng.integers(0, batch, size=10))})
            rows = np.array([(t, int(h)) for t in toks for h in rng.choice(H, size=4, replace=False)], np.int32)
            want = ref.flash_attention_rows(q, kc, vc, rows, H, G, d, n_ctx, n_past, np.float32(scale), threads=ref.max_threads())
            got = gpu_prefill(fa, q, kc, vc, H, G, d, n_ctx, n_past, batch, scale)
            check(got[rows[:, 0], rows[:, 1]], want, f"cfg2 P{n_past} layer {layer}")
            worst = max(worst, rel_err(got[rows[:, 0], rows[:, 1]], want)[0])
    print(f"cfg2 28 layers x 2 chunks: worst err_row {worst:.3e}", flush=True)


# ---------------------------------------------------------------- error behaviour

def test_rejects_bad_arguments(fa):
    import torch

    from orin_llm_amd.kernels import OrinFaError

    t = torch.zeros(4096, dtype=torch.float32, device="cuda")
    with pytest.raises(OrinFaError) as e:
        fa.flash_attention(t, t, t, t, 8, 2, 96, 16, 0, 1, 0.1)  # reference: assert(false) on head_dim
    assert e.value.code == -2
    with pytest.raises(OrinFaError) as e:
        fa.flash_attention(t, t, t, t, 7, 2, 128, 16, 0, 1, 0.1)  # n_head % n_kv != 0
    assert e.value.code == -1
    with pytest.raises(OrinFaError):
        fa.flash_attention(t, t, t, t, 8, 2, 128, 16, 10, 7, 0.1)  # n_past + batch > n_ctx
    with pytest.raises(OrinFaError):
        fa.flash_attention_decode_ind(t, t, t, t, 8, 2, 128, 16, None, 0.1)
    fa.flash_attention(t, t, t, t, 8, 2, 128, 16, 0, 0, 0.1)  # empty chunk: nothing to do
    torch.cuda.synchronize()
