"""orin_decode_layer at the benchmark's model shapes, against the CPU oracle's operators in the reference's order
(src/model_gpu.cu:251-293): one Llama-3-8B-shaped layer at cache length 8192, one Qwen2.5-1.5B-shaped and one
Qwen2.5-7B-shaped layer (with q/k/v biases; seven query heads per KV head in the latter) at 32768, and one
Llama-3.2-1B-shaped layer (head_dim 64, rotary frequencies divided by per-pair factors) at 8192, weights in the mix
of a Q4_K_M file (Q4_K; attn_v and ffn_down Q6_K).  These are the shapes
at which the layer's launches take the forms the small whole-model fixtures never reach: q, k, v of two types in one
launch with eight waves a workgroup, accumulating projections whose rows are shared among workgroups, the kernel for
launches that leave resident places empty, 32-128 KV splits.

Three ways through the layer -- the reference's own call sequence, orin_decode_layer, orin_decode_layer captured in
a graph and replayed -- each against the oracle (fp16 cache, as the GPU keeps it) at TOL_OP * 10 of the output
vector's largest element (measured: a few 1e-6), and the token's cache rows against the oracle's to one fp16 step.
"""
import os
import sys

import numpy as np
import pytest

from oracle import ref
from test_gpu_layer import TOL_OP, _dev, dev_bytes, fa, ly, vec_err  # noqa: F401  (fa, ly: fixtures)

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import layer_model as lm  # noqa: E402

pytestmark = pytest.mark.gpu

MODELS = {
    "llama8b": dict(n_embd=4096, n_head=32, n_kv=8, head_dim=128, n_ff=14336, n_ctx=8192, L=8192, bias=False, neox=0, theta=5.0e5,
                    eps=1.0e-5),
    "qwen1.5b": dict(n_embd=1536, n_head=12, n_kv=2, head_dim=128, n_ff=8960, n_ctx=32768, L=32768, bias=True, neox=1, theta=1.0e6,
                     eps=1.0e-6),
    "qwen7b": dict(n_embd=3584, n_head=28, n_kv=4, head_dim=128, n_ff=18944, n_ctx=32768, L=32767, bias=True, neox=1, theta=1.0e6,
                   eps=1.0e-6),
    "llama1b": dict(n_embd=2048, n_head=32, n_kv=8, head_dim=64, n_ff=8192, n_ctx=8192, L=8192, bias=False, neox=0, theta=5.0e5,
                    eps=1.0e-5, freq_factors=True),
}
TYPES = dict(wq=lm.Q4_K, wk=lm.Q4_K, wv=lm.Q6_K, wo=lm.Q4_K, ffn_gate=lm.Q4_K, ffn_up=lm.Q4_K, ffn_down=lm.Q6_K)


def make_layer(name):
    c = MODELS[name]
    rs = lm.Stream(9000 + len(name))
    ne, nq, nkv, nff = c["n_embd"], c["n_head"] * c["head_dim"], c["n_kv"] * c["head_dim"], c["n_ff"]
    dims = dict(wq=(ne, nq), wk=(ne, nkv), wv=(ne, nkv), wo=(nq, ne), ffn_gate=(ne, nff), ffn_up=(ne, nff), ffn_down=(nff, ne))
    L = {k: lm.make_tensor(rs, TYPES[k], *dims[k], std=0.03) for k in TYPES}
    L["attn_norm"] = (1.0 + rs.sym(ne, 0.2)).astype(np.float32)
    L["ffn_norm"] = (1.0 + rs.sym(ne, 0.2)).astype(np.float32)
    if c["bias"]:
        L["bq"], L["bk"], L["bv"] = rs.sym(nq, 0.3), rs.sym(nkv, 0.3), rs.sym(nkv, 0.3)
    if c.get("freq_factors"):   # (the long-context scaling of the Llama-3 family: low frequencies slowed down)
        L["freq_factors"] = np.linspace(1.0, 8.0, c["head_dim"] // 2).astype(np.float32)
    x0 = rs.sym(ne, 1.0)
    rng = np.random.default_rng(77)
    kc = rng.standard_normal((c["n_kv"], c["n_ctx"], c["head_dim"]), dtype=np.float32).astype(np.float16).view(np.uint16)
    vc = rng.standard_normal((c["n_kv"], c["n_ctx"], c["head_dim"]), dtype=np.float32).astype(np.float16).view(np.uint16)
    return c, L, dims, x0, kc, vc


def oracle_layer(c, L, dims, x0, kc, vc):
    """The reference's decode_layer in the oracle's operators; returns x after the layer and the caches it wrote."""
    H, G, d, pos = c["n_head"], c["n_kv"], c["head_dim"], c["L"] - 1
    mv = lambda key, x: ref.gemv(L[key][0], L[key][1], x, dims[key][0], dims[key][1])  # noqa: E731
    xn = ref.rms_norm(x0, L["attn_norm"], c["eps"])
    q, k, v = mv("wq", xn), mv("wk", xn), mv("wv", xn)
    if c["bias"]:
        q, k, v = q + L["bq"], k + L["bk"], v + L["bv"]
    q = ref.rope_batch(q.reshape(H, d), d, d, c["theta"], pos, H, L.get("freq_factors"), bool(c["neox"]))
    k = ref.rope_batch(k.reshape(G, d), d, d, c["theta"], pos, G, L.get("freq_factors"), bool(c["neox"]))
    kc, vc = kc.copy(), vc.copy()
    ref.kv_store_f16(kc, vc, k.reshape(1, G, d), v.reshape(1, G, d), G, d, c["n_ctx"], pos, 1)
    attn = ref.flash_attention_decode_ind(q, kc, vc, H, G, d, c["n_ctx"], pos, float(1.0 / np.sqrt(d))).reshape(-1)
    x1 = x0 + mv("wo", attn)
    xn2 = ref.rms_norm(x1, L["ffn_norm"], c["eps"])
    act = ref.swiglu(mv("ffn_gate", xn2), mv("ffn_up", xn2))
    return (x1 + mv("ffn_down", act)).astype(np.float64), kc, vc


@pytest.fixture(scope="module", params=list(MODELS))
def case(request):
    c, L, dims, x0, kc, vc = make_layer(request.param)
    want, kc_want, vc_want = oracle_layer(c, L, dims, x0, kc, vc)
    return request.param, c, L, x0, kc, vc, want, kc_want, vc_want


@pytest.mark.parametrize("how", ["calls", "fused", "fused_graph"])
def test_decode_layer_at_model_shape(fa, ly, case, how):
    import torch

    name, c, L, x0, kc, vc, want, kc_want, vc_want = case
    H, G, d, ne, nff, n_ctx = c["n_head"], c["n_kv"], c["head_dim"], c["n_embd"], c["n_ff"], c["n_ctx"]
    D = {k: ((v[0], dev_bytes(v[1], offset=2 if v[0] == lm.Q6_K else 0)) if isinstance(v, tuple) else _dev(v)) for k, v in L.items()}
    hp = dict(n_embd=ne, n_head=H, n_kv=G, head_dim=d, n_ff=nff, n_rot=d, neox=c["neox"], rms_eps=c["eps"], rope_theta=c["theta"],
              freq_factors_dev=D.get("freq_factors"))
    z = lambda n: torch.zeros(n, dtype=torch.float32, device="cuda")  # noqa: E731
    bufs = dict(x=z(ne), xn=z(ne), xn2=z(ne), q=z(H * d), k=z(G * d), v=z(G * d), attn=z(max(H * d, ne)), act=z(nff), up_tmp=z(nff))
    dkc, dvc = torch.from_numpy(kc.view(np.int16)).cuda(), torch.from_numpy(vc.view(np.int16)).cuda()
    d_pos = torch.tensor([c["L"] - 1], dtype=torch.int32, device="cuda")
    angles = torch.zeros((d // 2, 2), device="cuda")
    desc = ly.make_desc(hp, D, bufs, dkc, dvc, d_pos, n_ctx, rope_angles=angles)

    def step():
        if how == "calls":
            ly.decode_layer_calls(hp, D, bufs, dkc, dvc, d_pos, n_ctx)
        else:
            fa.rope_angles_ind(angles, d, c["theta"], d_pos, D.get("freq_factors"))
            ly.decode_layer(desc)

    bufs["x"].copy_(_dev(x0))
    if how == "fused_graph":
        stream = torch.cuda.Stream()
        torch.cuda.synchronize()
        fa.set_stream(stream.cuda_stream)
        graph = torch.cuda.CUDAGraph()
        try:
            with torch.cuda.graph(graph, stream=stream):
                step()
        finally:
            fa.set_stream(torch.cuda.current_stream().cuda_stream)
        errs = []
        for _ in range(3):   # every replay from the same input: the same layer, three times
            bufs["x"].copy_(_dev(x0))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            errs.append(vec_err(bufs["x"].cpu().numpy(), want))
        err = max(errs)
    else:
        step()
        torch.cuda.synchronize()
        err = vec_err(bufs["x"].cpu().numpy(), want)
    pos = c["L"] - 1
    got_k, got_v = dkc.cpu().numpy().view(np.uint16), dvc.cpu().numpy().view(np.uint16)
    row_k = np.abs(ref.fp16_to_fp32(got_k[:, pos]) - ref.fp16_to_fp32(kc_want[:, pos])).max() / np.abs(ref.fp16_to_fp32(kc_want[:, pos])).max()
    row_v = np.abs(ref.fp16_to_fp32(got_v[:, pos]) - ref.fp16_to_fp32(vc_want[:, pos])).max() / np.abs(ref.fp16_to_fp32(vc_want[:, pos])).max()
    print(f"{name} {how}: layer output vs oracle {err:.2e}, the token's cache rows {row_k:.1e} / {row_v:.1e}", flush=True)
    assert err < TOL_OP * 10
    assert row_k < 1e-3 and row_v < 1e-3          # (one fp16 step of a projection that differs in the last bits of its fp32 sum)
    untouched = np.ones(n_ctx, bool)
    untouched[pos] = False
    assert np.array_equal(got_k[:, untouched], kc[:, untouched]) and np.array_equal(got_v[:, untouched], vc[:, untouched])


def test_decode_layer_replays_bit_for_bit_with_one_share(fa, ly, case):
    """With orin_gemv_row_shares(1) set before the capture, twenty replays of one captured layer give the same bits;
    with the default (rows of the output and down projections shared among workgroups that add atomically) they
    agree to the order of an fp32 sum."""
    import torch

    name, c, L, x0, kc, vc, want, _, _ = case
    H, G, d, ne, nff, n_ctx = c["n_head"], c["n_kv"], c["head_dim"], c["n_embd"], c["n_ff"], c["n_ctx"]
    D = {k: ((v[0], dev_bytes(v[1], offset=2 if v[0] == lm.Q6_K else 0)) if isinstance(v, tuple) else _dev(v)) for k, v in L.items()}
    hp = dict(n_embd=ne, n_head=H, n_kv=G, head_dim=d, n_ff=nff, n_rot=d, neox=c["neox"], rms_eps=c["eps"], rope_theta=c["theta"],
              freq_factors_dev=D.get("freq_factors"))
    z = lambda n: torch.zeros(n, dtype=torch.float32, device="cuda")  # noqa: E731
    bufs = dict(x=z(ne), q=z(H * d), k=z(G * d), v=z(G * d), attn=z(max(H * d, ne)), act=z(nff), up_tmp=z(nff))
    dkc, dvc = torch.from_numpy(kc.view(np.int16)).cuda(), torch.from_numpy(vc.view(np.int16)).cuda()
    d_pos = torch.tensor([c["L"] - 1], dtype=torch.int32, device="cuda")
    desc = ly.make_desc(hp, D, bufs, dkc, dvc, d_pos, n_ctx)
    dx0 = _dev(x0)
    stream = torch.cuda.Stream()
    results = {}
    try:
        for shares in (0, 1):
            ly.gemv_row_shares(shares)
            torch.cuda.synchronize()
            fa.set_stream(stream.cuda_stream)
            graph = torch.cuda.CUDAGraph()
            try:
                with torch.cuda.graph(graph, stream=stream):
                    ly.decode_layer(desc)
            finally:
                fa.set_stream(torch.cuda.current_stream().cuda_stream)
            outs = []
            for _ in range(20):
                bufs["x"].copy_(dx0)
                torch.cuda.synchronize()
                graph.replay()
                torch.cuda.synchronize()
                outs.append(bufs["x"].cpu().numpy())
            results[shares] = outs
            del graph
    finally:
        ly.gemv_row_shares(0)
    for outs in results.values():
        assert max(vec_err(o, want) for o in outs) < TOL_OP * 10
    assert all(np.array_equal(results[1][0].view(np.uint32), o.view(np.uint32)) for o in results[1][1:])
    spread = max(float(np.abs(o.astype(np.float64) - results[0][0]).max() / np.abs(want).max()) for o in results[0][1:])
    print(f"{name}: spread of 20 replays with shared rows {spread:.1e}; with one share bit-identical", flush=True)
    assert spread < 1e-5
