#!/usr/bin/env python3
"""Produce tests/golden/layer_reference.npz from the UNMODIFIED reference CPU backend.

Run in the build container only (needs /root/reference and `make -C oracle ref`):

    python tests/golden/make_layer_fixture.py

Each model of layer_model.py (two layers; matrices of every weight type the reference reads,
src/common.h:47-54; projections with bias, per-head q/k norms, frequency factors, tied and untied
output matrix) is written as a GGUF file in /tmp (never committed) and walked by
oracle/_ref/ref_driver: token t at position t for t < N_TOKENS, i.e. the whole forward pass of
src/model_cpu.cpp:241-312 -- embedding row, norms, quantised matrix-vector products, rotary
embedding, cache write, attention, feed-forward block, output matrix.  Only the logits are stored;
the weights are rebuilt from their seeds by whoever checks against them.
"""
import os
import struct
import subprocess
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import layer_model as lm  # noqa: E402
from make_cfg1_fixture import DRIVER, GGUF_F32, GGUF_STR, GGUF_U32, _s  # noqa: E402

N_CTX = 32


def write_gguf(path, meta, tensors, align=32):
    """tensors: (name, type, n_in, n_out, uint8 array); a vector is a tensor with n_out = 1."""
    head = b"GGUF" + struct.pack("<IQQ", 3, len(tensors), len(meta))
    for key, typ, val in meta:
        head += _s(key) + struct.pack("<I", typ)
        head += struct.pack("<I", val) if typ == GGUF_U32 else struct.pack("<f", val) if typ == GGUF_F32 else _s(val)
    off, offsets = 0, []
    for name, typ, n_in, n_out, raw in tensors:
        per, nbytes = lm.BLOCK[typ]
        assert raw.dtype == np.uint8 and raw.size == n_in // per * nbytes * n_out, name
        head += _s(name) + struct.pack("<I", 2) + struct.pack("<QQ", n_in, n_out) + struct.pack("<I", typ) + struct.pack("<Q", off)
        offsets.append(off)
        off += (raw.size + align - 1) // align * align
    with open(path, "wb") as f:
        f.write(head + b"\0" * ((-len(head)) % align))
        for (_, _, _, _, raw) in tensors:
            f.write(raw.tobytes() + b"\0" * ((-raw.size) % align))


def to_gguf(model):
    hp = model["hp"]
    a = hp["arch"]
    meta = [("general.architecture", GGUF_STR, a), (a + ".block_count", GGUF_U32, hp["n_layer"]),
            (a + ".context_length", GGUF_U32, N_CTX), (a + ".attention.head_count", GGUF_U32, hp["n_head"]),
            (a + ".attention.head_count_kv", GGUF_U32, hp["n_kv"]), (a + ".attention.key_length", GGUF_U32, hp["head_dim"]),
            (a + ".rope.dimension_count", GGUF_U32, hp["n_rot"]), (a + ".rope.freq_base", GGUF_F32, hp["rope_theta"]),
            (a + ".attention.layer_norm_rms_epsilon", GGUF_F32, hp["rms_eps"])]

    def vec(name, x):
        return (name, lm.F32, x.size, 1, np.ascontiguousarray(x, np.float32).view(np.uint8))

    def mat(name, t):
        return (name, t[0], t[2], t[3], t[1])

    tensors = [mat("token_embd.weight", model["token_embd"]), vec("output_norm.weight", model["output_norm"])]
    if not model["tied_output"]:
        tensors.append(mat("output.weight", model["output"]))
    if hp["freq_factors"] is not None:
        tensors.append(vec("rope_freqs.weight", hp["freq_factors"]))
    for i, L in enumerate(model["layers"]):
        p = f"blk.{i}."
        for key, gname in (("wq", "attn_q"), ("wk", "attn_k"), ("wv", "attn_v"), ("wo", "attn_output"),
                           ("ffn_gate", "ffn_gate"), ("ffn_up", "ffn_up"), ("ffn_down", "ffn_down")):
            tensors.append(mat(p + gname + ".weight", L[key]))
        tensors += [vec(p + "attn_norm.weight", L["attn_norm"]), vec(p + "ffn_norm.weight", L["ffn_norm"])]
        for key, gname in (("bq", "attn_q.bias"), ("bk", "attn_k.bias"), ("bv", "attn_v.bias"),
                           ("q_norm", "attn_q_norm.weight"), ("k_norm", "attn_k_norm.weight")):
            if key in L:
                tensors.append(vec(p + gname, L[key]))
    return meta, tensors


def main():
    if not os.path.exists(DRIVER):
        sys.exit("build the driver first: make -C oracle ref")
    store = {}
    with tempfile.TemporaryDirectory(dir="/tmp") as tmp:
        for name in lm.VARIANTS:
            model = lm.build(name)
            gguf, out = os.path.join(tmp, name + ".gguf"), os.path.join(tmp, name + ".bin")
            write_gguf(gguf, *to_gguf(model))
            nv = model["hp"]["n_vocab"]
            subprocess.run([DRIVER, gguf, str(lm.N_TOKENS), str(N_CTX), str(nv), out], check=True)
            store["logits_" + name] = np.fromfile(out, dtype="<f4").reshape(lm.N_TOKENS, nv)
            assert np.isfinite(store["logits_" + name]).all()
    store["meta"] = np.array([lm.N_TOKENS, N_CTX], np.int32)
    dst = os.path.join(HERE, "layer_reference.npz")
    np.savez(dst, **store)
    print("wrote", dst, os.path.getsize(dst), "bytes")


if __name__ == "__main__":
    main()
