#!/usr/bin/env python3
"""Produce tests/golden/cfg1_reference.npz from the UNMODIFIED reference CPU backend.

Run in the build container only (needs /root/reference and `make -C oracle ref`):

    python tests/golden/make_cfg1_fixture.py

The reference's CPU attention (src/model_cpu.cpp:281-295) is inlined in
Model::forward and reachable only through a GGUF model, so this script writes a
synthetic one-layer F32 GGUF (in /tmp, never committed) whose weights make the
layer's projections return chosen q/k/v vectors EXACTLY and route the attention
output, unchanged, into the logits:

  * arch "llama", 12 heads, 2 KV heads, key_length 128, rope.dimension_count 0
    (both RoPE loops empty, src/model_cpu.cpp:179-203), rms epsilon 0.
  * n_embd 4096, token_embd[t] = e_t  =>  rms_norm gives exactly 64*e_t
    (ss/n = 2^-12, src/model_cpu.cpp:13-18).
  * Wq[:, t] = q_t/64, Wk[:, t] = k_t/64, Wv[:, t] = v_t/64  =>  the sequential fp32
    dot (src/model_cpu.cpp:32-36) has one non-zero, power-of-two-scaled product.
  * Wo copies attention element i to residual dim 2048+i; the FFN is all zeros.
  * output.weight row i<1536 = e_{2048+i}; row 1536 = ones over dims < N_TOKENS, so
    logits[i] = fl32(attn_i * r) and logits[1536] = fl32(r), r = 1/rms(x) in double.

Step t feeds token t at position t: 45 prefill tokens then 128 decode steps, which on
the CPU backend are the same call (src/model_cpu.cpp:314-319).

Two runs are stored: "A" with raw fp32 K/V (faithful: the CPU cache is fp32,
src/model_cpu.cpp:217) and "B" with K/V pre-rounded to fp16 values (isolates kernel
error from cache rounding).
"""
import os
import struct
import subprocess
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.dirname(os.path.dirname(HERE))
DRIVER = os.path.join(REPO, "oracle", "_ref", "ref_driver")

N_HEAD, N_KV, D = 12, 2, 128
N_PREFILL, N_DECODE = 45, 128
N_TOK = N_PREFILL + N_DECODE
N_EMBD, N_VOCAB = 4096, 2048
ATT = N_HEAD * D  # 1536
OUT_BASE = 2048
N_LOGITS = ATT + 1
SEED = 20250117

GGUF_U32, GGUF_F32, GGUF_STR = 4, 6, 8


def _s(b):
    b = b.encode()
    return struct.pack("<Q", len(b)) + b


def write_gguf(path, meta, tensors, align=32):
    """meta: list of (key, type, value); tensors: list of (name, 2-D float32 array [ne1][ne0])."""
    head = b"GGUF" + struct.pack("<IQQ", 3, len(tensors), len(meta))
    for key, typ, val in meta:
        head += _s(key) + struct.pack("<I", typ)
        if typ == GGUF_U32:
            head += struct.pack("<I", val)
        elif typ == GGUF_F32:
            head += struct.pack("<f", val)
        elif typ == GGUF_STR:
            head += _s(val)
        else:
            raise ValueError(typ)
    off = 0
    offsets = []
    for name, arr in tensors:
        assert arr.dtype == np.float32 and arr.ndim == 2
        ne1, ne0 = arr.shape
        head += _s(name) + struct.pack("<I", 2) + struct.pack("<QQ", ne0, ne1)
        head += struct.pack("<I", 0) + struct.pack("<Q", off)  # type F32
        offsets.append(off)
        off += (arr.nbytes + align - 1) // align * align
    pad = (-len(head)) % align
    with open(path, "wb") as f:
        f.write(head + b"\0" * pad)
        for (name, arr), o in zip(tensors, offsets):
            f.write(arr.tobytes())
            f.write(b"\0" * ((-arr.nbytes) % align))


def build_model(q, k, v):
    """q [N_TOK][ATT], k/v [N_TOK][N_KV*D] fp32."""
    def proj(x):
        w = np.zeros((x.shape[1], N_EMBD), np.float32)
        w[:, :N_TOK] = (x / np.float32(64.0)).T
        assert np.array_equal(w[:, :N_TOK] * np.float32(64.0), x.T)  # exact scaling
        return w

    emb = np.zeros((N_VOCAB, N_EMBD), np.float32)
    emb[np.arange(N_VOCAB), np.arange(N_VOCAB)] = 1.0
    wo = np.zeros((N_EMBD, N_EMBD), np.float32)
    wo[OUT_BASE + np.arange(ATT), np.arange(ATT)] = 1.0
    outw = np.zeros((N_LOGITS, N_EMBD), np.float32)
    outw[np.arange(ATT), OUT_BASE + np.arange(ATT)] = 1.0
    outw[ATT, :N_TOK] = 1.0
    ones = np.ones((1, N_EMBD), np.float32)
    tensors = [
        ("token_embd.weight", emb),
        ("output.weight", outw),
        ("output_norm.weight", ones),
        ("blk.0.attn_norm.weight", ones),
        ("blk.0.ffn_norm.weight", ones),
        ("blk.0.attn_q.weight", proj(q)),
        ("blk.0.attn_k.weight", proj(k)),
        ("blk.0.attn_v.weight", proj(v)),
        ("blk.0.attn_output.weight", wo),
        ("blk.0.ffn_gate.weight", np.zeros((1, N_EMBD), np.float32)),
        ("blk.0.ffn_up.weight", np.zeros((1, N_EMBD), np.float32)),
        ("blk.0.ffn_down.weight", np.zeros((N_EMBD, 1), np.float32)),
    ]
    meta = [
        ("general.architecture", GGUF_STR, "llama"),
        ("llama.block_count", GGUF_U32, 1),
        ("llama.context_length", GGUF_U32, 256),
        ("llama.attention.head_count", GGUF_U32, N_HEAD),
        ("llama.attention.head_count_kv", GGUF_U32, N_KV),
        ("llama.attention.key_length", GGUF_U32, D),
        ("llama.rope.dimension_count", GGUF_U32, 0),
        ("llama.attention.layer_norm_rms_epsilon", GGUF_F32, 0.0),
    ]
    return meta, tensors


def run_reference(q, k, v, tmp):
    meta, tensors = build_model(q, k, v)
    gguf = os.path.join(tmp, "cfg1.gguf")
    out = os.path.join(tmp, "logits.bin")
    write_gguf(gguf, meta, tensors)
    subprocess.run([DRIVER, gguf, str(N_TOK), "256", str(N_LOGITS), out], check=True)
    logits = np.fromfile(out, dtype="<f4").reshape(N_TOK, N_LOGITS)
    os.remove(gguf)
    return logits


def main():
    if not os.path.exists(DRIVER):
        sys.exit("build the driver first: make -C oracle ref")
    rng = np.random.default_rng(SEED)
    q = rng.standard_normal((N_TOK, ATT)).astype(np.float32)
    k = rng.standard_normal((N_TOK, N_KV * D)).astype(np.float32)
    v = rng.standard_normal((N_TOK, N_KV * D)).astype(np.float32)
    with tempfile.TemporaryDirectory(dir="/tmp") as tmp:
        logits_a = run_reference(q, k, v, tmp)
        k16 = k.astype(np.float16).astype(np.float32)
        v16 = v.astype(np.float16).astype(np.float32)
        logits_b = run_reference(q, k16, v16, tmp)
    dst = os.path.join(HERE, "cfg1_reference.npz")
    np.savez(dst, q=q, k=k, v=v, logits_a=logits_a, logits_b=logits_b,
             meta=np.array([N_HEAD, N_KV, D, N_PREFILL, N_DECODE, OUT_BASE, N_EMBD], np.int32))
    print("wrote", dst, os.path.getsize(dst), "bytes")


if __name__ == "__main__":
    main()
