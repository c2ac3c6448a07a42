"""The attention path of an engine layer, driven through the C++ shim's own symbols.

The library exports the reference's operator functions under their C++ names (llm::cuda::...,
reference: src/kernels.h:8-12, 55-81), so an engine compiled against the reference header links
to them unchanged.  These tests call them by their mangled names in the order the reference's
layer code does -- rotary embedding of Q and K, store into the cache, attention -- for a
prefill chunk (reference: src/model_gpu.cu:378-384) and for a decode step captured once in a
graph and replayed while the position moves (src/model_gpu.cu:277-282, 295-316), and compare
with the CPU oracle doing the same three steps.
"""
import ctypes

import numpy as np
import pytest

from oracle import ref
from util import FLOOR_PREFILL, TOL, rel_err

pytestmark = pytest.mark.gpu

vp, ci, cf = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
SHIM = {  # name -> (mangled symbol, argument types)
    "init": ("_ZN3llm4cuda4initEv", []),
    "set_stream": ("_ZN3llm4cuda10set_streamEPv", [vp]),
    "rope_neox_batch": ("_ZN3llm4cuda15rope_neox_batchEPfiiifiiPKf", [vp, ci, ci, ci, cf, ci, ci, vp]),
    "rope_neox_ind": ("_ZN3llm4cuda13rope_neox_indEPfiiifPKiPKf", [vp, ci, ci, ci, cf, vp, vp]),
    "kv_store_batch": ("_ZN3llm4cuda14kv_store_batchEPtS1_PKfS3_iiiii", [vp, vp, vp, vp, ci, ci, ci, ci, ci]),
    "kv_store_ind": ("_ZN3llm4cuda12kv_store_indEPtS1_PKfS3_iiiPKi", [vp, vp, vp, vp, ci, ci, ci, vp]),
    "flash_attention": ("_ZN3llm4cuda15flash_attentionEPKfPKtS4_Pfiiiiiif", [vp] * 4 + [ci] * 6 + [cf]),
    "flash_attention_decode_ind": ("_ZN3llm4cuda26flash_attention_decode_indEPKfPKtS4_PfiiiiPKif",
                                   [vp] * 4 + [ci] * 4 + [vp, cf]),
}


@pytest.fixture(scope="module")
def shim():
    torch = pytest.importorskip("torch")
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from orin_llm_amd import kernels

    lib = ctypes.CDLL(kernels.LIB_PATH)

    class Shim:
        pass

    s = Shim()
    for name, (sym, argtypes) in SHIM.items():
        f = getattr(lib, sym)
        f.argtypes = argtypes
        f.restype = ci if name == "init" else None
        setattr(s, name, f)
    assert s.init() == 0
    s.set_stream(torch.cuda.current_stream().cuda_stream)
    return s


H, G, D, THETA = 12, 2, 128, 1.0e6   # Qwen2.5-1.5B heads
SCALE = float(1.0 / np.sqrt(D))


def _layer_inputs(seed, tokens):
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((tokens, H, D)).astype(np.float32)
    k = rng.standard_normal((tokens, G, D)).astype(np.float32)
    v = rng.standard_normal((tokens, G, D)).astype(np.float32)
    return q, k, v


def test_prefill_layer_through_the_shim(shim):
    import torch

    n_ctx, n_past, batch = 1024, 300, 200
    rng = np.random.default_rng(5)
    kc = rng.standard_normal((G, n_ctx, D)).astype(np.float16).view(np.uint16)
    vc = rng.standard_normal((G, n_ctx, D)).astype(np.float16).view(np.uint16)
    q, k, v = _layer_inputs(6, batch)
    # the oracle's layer: rotate, store, attend
    q_ref = ref.rope_batch(q.reshape(-1, D), D, D, THETA, n_past, H, None, True).reshape(batch, H, D)
    k_ref = ref.rope_batch(k.reshape(-1, D), D, D, THETA, n_past, G, None, True).reshape(batch, G, D)
    kc_ref, vc_ref = kc.copy(), vc.copy()
    ref.kv_store_f16(kc_ref, vc_ref, k_ref, v, G, D, n_ctx, n_past, batch)
    rows = np.array([(t, h) for t in (0, 1, 63, 64, batch - 1) for h in range(H)], np.int32)
    want = ref.flash_attention_rows(q_ref, kc_ref, vc_ref, rows, H, G, D, n_ctx, n_past, np.float32(SCALE))
    # the same through the shim
    dq, dk, dv = (torch.from_numpy(x).cuda() for x in (q, k, v))
    dkc = torch.from_numpy(kc.view(np.int16)).cuda()
    dvc = torch.from_numpy(vc.view(np.int16)).cuda()
    out = torch.empty((batch, H, D), device="cuda")
    shim.rope_neox_batch(dq.data_ptr(), batch * H, D, D, THETA, n_past, H, None)
    shim.rope_neox_batch(dk.data_ptr(), batch * G, D, D, THETA, n_past, G, None)
    shim.kv_store_batch(dkc.data_ptr(), dvc.data_ptr(), dk.data_ptr(), dv.data_ptr(), G, D, n_ctx, n_past, batch)
    shim.flash_attention(dq.data_ptr(), dkc.data_ptr(), dvc.data_ptr(), out.data_ptr(), H, G, D, n_ctx, n_past, batch, SCALE)
    torch.cuda.synchronize()
    assert np.array_equal(dkc.cpu().numpy().view(np.uint16)[:, :n_past], kc[:, :n_past])   # older rows untouched
    stored = dkc.cpu().numpy().view(np.uint16)[:, n_past:n_past + batch]
    # the rotated rows as fp16: equal to the oracle's except where the last bit of a sine moved a rounding
    assert (stored != kc_ref[:, n_past:n_past + batch]).mean() < 1e-3
    assert np.array_equal(dvc.cpu().numpy().view(np.uint16), vc_ref)
    got = out.cpu().numpy()[rows[:, 0], rows[:, 1]]
    e = rel_err(got, want)
    assert e[0] < TOL and e[1] < FLOOR_PREFILL, e


def test_decode_steps_through_the_shim_replayed_from_a_graph(shim):
    import torch

    n_ctx, n_layer, first = 2048, 28, 700
    rng = np.random.default_rng(7)
    kcs = [rng.standard_normal((G, n_ctx, D)).astype(np.float16).view(np.uint16) for _ in range(n_layer)]
    vcs = [rng.standard_normal((G, n_ctx, D)).astype(np.float16).view(np.uint16) for _ in range(n_layer)]
    dkc = [torch.from_numpy(a.view(np.int16)).cuda() for a in kcs]
    dvc = [torch.from_numpy(a.view(np.int16)).cuda() for a in vcs]
    # the engine's activation buffers: one q / k / v / out per step, refilled by the layers before the attention
    dq = torch.empty((n_layer, H, D), device="cuda")
    dk = torch.empty((n_layer, G, D), device="cuda")
    dv = torch.empty((n_layer, G, D), device="cuda")
    dout = torch.zeros((n_layer, H, D), device="cuda")
    dpos = torch.zeros(1, dtype=torch.int32, device="cuda")
    stage_q, stage_k = torch.empty_like(dq), torch.empty_like(dk)

    def layers():
        dq.copy_(stage_q)   # (stands for the projections that produce q and k; the rotation is in place)
        dk.copy_(stage_k)
        for l in range(n_layer):
            shim.rope_neox_ind(dq[l].data_ptr(), H, D, D, THETA, dpos.data_ptr(), None)
            shim.rope_neox_ind(dk[l].data_ptr(), G, D, D, THETA, dpos.data_ptr(), None)
            shim.kv_store_ind(dkc[l].data_ptr(), dvc[l].data_ptr(), dk[l].data_ptr(), dv[l].data_ptr(), G, D, n_ctx,
                              dpos.data_ptr())
            shim.flash_attention_decode_ind(dq[l].data_ptr(), dkc[l].data_ptr(), dvc[l].data_ptr(), dout[l].data_ptr(),
                                            H, G, D, n_ctx, dpos.data_ptr(), SCALE)

    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    try:
        with torch.cuda.graph(graph):
            shim.set_stream(torch.cuda.current_stream().cuda_stream)
            layers()
    finally:
        shim.set_stream(torch.cuda.current_stream().cuda_stream)
    rows = np.array([(0, h) for h in range(H)], np.int32)
    for step, pos in enumerate((first, first + 1, first + 2, n_ctx - 1)):
        q, k, v = _layer_inputs(100 + step, n_layer)     # [layer][heads][D]
        stage_q.copy_(torch.from_numpy(q))
        stage_k.copy_(torch.from_numpy(k))
        dv.copy_(torch.from_numpy(v))
        dpos.fill_(pos)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = dout.cpu().numpy()
        for l in (0, 13, n_layer - 1):
            q_ref = ref.rope_batch(q[l], D, D, THETA, pos, H, None, True)
            k_ref = ref.rope_batch(k[l], D, D, THETA, pos, G, None, True)
            ref.kv_store_f16(kcs[l], vcs[l], k_ref[None], v[l][None], G, D, n_ctx, pos, 1)
            want = ref.flash_attention_rows(q_ref[None], kcs[l], vcs[l], rows, H, G, D, n_ctx, pos, np.float32(SCALE))
            e = rel_err(got[l], want)  # (the rotated K row may differ from the oracle's in a last bit: the prefill bound)
            assert e[0] < TOL and e[1] < FLOOR_PREFILL, (pos, l, e)
        for l in range(n_layer):   # the oracle's caches follow every layer, checked or not
            if l not in (0, 13, n_layer - 1):
                k_ref = ref.rope_batch(k[l], D, D, THETA, pos, G, None, True)
                ref.kv_store_f16(kcs[l], vcs[l], k_ref[None], v[l][None], G, D, n_ctx, pos, 1)


# ---------------------------------------------------------------- the whole decode step

LAYER_SHIM = {  # the rest of what decode_layer calls (reference: src/model_gpu.cu:251-293, 303-306)
    "rope_normal_ind": ("_ZN3llm4cuda15rope_normal_indEPfiiifPKiPKf", [vp, ci, ci, ci, cf, vp, vp]),
    "quantize_activation": ("_ZN3llm4cuda19quantize_activationEPKfi", [vp, ci]),
    "gemv": ("_ZN3llm4cuda4gemvENS_5DTypeEPKvPKfPfii", [ci, vp, vp, vp, ci, ci]),
    "gemv_q8": ("_ZN3llm4cuda7gemv_q8ENS_5DTypeEPKvPfii", [ci, vp, vp, ci, ci]),
    "gemv_q8_bias": ("_ZN3llm4cuda12gemv_q8_biasENS_5DTypeEPKvPKfPfii", [ci, vp, vp, vp, ci, ci]),
    "gemv_q8_add": ("_ZN3llm4cuda11gemv_q8_addENS_5DTypeEPKvPfii", [ci, vp, vp, ci, ci]),
    "gemv_fused_gate_up_swiglu": ("_ZN3llm4cuda25gemv_fused_gate_up_swigluENS_5DTypeEPKvS3_Pfii", [ci, vp, vp, vp, ci, ci]),
    "dequant_row": ("_ZN3llm4cuda11dequant_rowENS_5DTypeEPKvPfi", [ci, vp, vp, ci]),
    "rms_norm": ("_ZN3llm4cuda8rms_normEPKfS2_ifPf", [vp, vp, ci, cf, vp]),
    "rms_norm_rows": ("_ZN3llm4cuda13rms_norm_rowsEPKfS2_iifPf", [vp, vp, ci, ci, cf, vp]),
    "swiglu": ("_ZN3llm4cuda6swigluEPfPKfS3_i", [vp, vp, vp, ci]),
}


@pytest.mark.parametrize("name", ["qwen2", "llama", "qwen2p", "narrow"])
def test_whole_decode_step_through_the_shim_replayed_from_a_graph(shim, name):
    """The reference's forward_capture (src/model_gpu.cu:295-316) over a small quantised model: embedding
    row, every layer call for call, last norm, output matrix -- through the llm::cuda symbols, captured once
    and replayed per token with the embedding row and the position updated in place -- against the logits of
    the unmodified reference CPU build."""
    import os
    import sys

    import torch

    here = os.path.dirname(os.path.abspath(__file__))
    sys.path.insert(0, os.path.join(here, "golden"))
    import layer_model as lm
    from orin_llm_amd import kernels, layer as ly
    from test_gpu_layer import make_bufs, upload, vec_err

    lib = ctypes.CDLL(kernels.LIB_PATH)

    class Ops:  # the operators under the reference's names, taking tensors
        pass

    ops = Ops()
    table = dict(SHIM)
    table.update(LAYER_SHIM)
    for fname, (sym, argtypes) in table.items():
        f = getattr(lib, sym)
        f.argtypes, f.restype = argtypes, (ci if fname == "init" else None)

        def call(*args, _f=f):
            _f(*[a.data_ptr() if hasattr(a, "data_ptr") else a for a in args])
        setattr(ops, fname, call)

    golden = np.load(os.path.join(here, "golden", "layer_reference.npz"))
    n_tok, n_ctx = (int(v) for v in golden["meta"])
    model = lm.build(name)
    hp, layers, top = upload(model)
    bufs = make_bufs(hp)
    ne, nv, nl = hp["n_embd"], hp["n_vocab"], hp["n_layer"]
    kc = torch.zeros((nl, hp["n_kv"], n_ctx, hp["head_dim"]), dtype=torch.int16, device="cuda")
    vc = torch.zeros_like(kc)
    d_pos = torch.zeros(1, dtype=torch.int32, device="cuda")
    et, eraw = top["token_embd"]
    rb = ref.row_bytes(et, ne)
    emb_row = torch.zeros(rb + 16, dtype=torch.uint8, device="cuda")[:rb]

    def step():
        ops.dequant_row(et, emb_row, bufs["x"], ne)
        for l in range(nl):
            ly.decode_layer_calls(hp, layers[l], bufs, kc[l], vc[l], d_pos, n_ctx, ops=ops)
        ops.rms_norm(bufs["x"], top["output_norm"], ne, hp["rms_eps"], bufs["xn"])
        ops.gemv(top["output"][0], top["output"][1], bufs["xn"], bufs["logits"], ne, nv)

    stream, graph, worst = torch.cuda.Stream(), None, 0.0
    for t in range(n_tok):
        emb_row.copy_(eraw[t * rb:(t + 1) * rb])
        d_pos.fill_(t)
        torch.cuda.synchronize()
        if graph is None:
            shim.set_stream(stream.cuda_stream)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                step()
            shim.set_stream(torch.cuda.current_stream().cuda_stream)
        graph.replay()
        torch.cuda.synchronize()
        worst = max(worst, vec_err(bufs["logits"].cpu().numpy(), golden["logits_" + name][t].astype(np.float64)))
    print(f"{name} through the shim, graph replay: vs reference logits {worst:.2e}", flush=True)
    assert worst < 1e-2
