#!/usr/bin/env python3
"""Produce tests/golden/rope_reference.npz from the UNMODIFIED reference CPU backend.

Run in the build container only (needs /root/reference and `make -C oracle ref`):

    python tests/golden/make_rope_fixture.py

Same synthetic one-layer model as make_cfg1_fixture.py (the projections return chosen q/k/v
rows exactly and the attention output reaches the logits unchanged), but with the rotary
embedding switched on, so that the reference's own rope_neox / rope_normal
(src/model_cpu.cpp:179-203, call site :264-275, selection src/model_common.cpp:24-41) run on the
way: what comes out is rope -> cache write -> attention of the reference, in its arithmetic.

Cases (each at positions [0, N) and again at [POS_HI, POS_HI + N), where the angles are large
and one ulp of a frequency shows):
  neox     arch "qwen2" (=> NeoX pairing), rope.dimension_count 128, freq_base 1e6
  normal   arch "llama" (=> adjacent pairs), rope.dimension_count 128, freq_base 5e5,
           with a rope_freqs.weight tensor (frequency factors, Llama-3 style)
  partial  arch "llama", rope.dimension_count 64 (< head_dim: the upper half is untouched),
           default freq_base 10000

Only numbers are stored: q, k, v, the factors and the logits of every run.
"""
import os
import subprocess
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import make_cfg1_fixture as base  # noqa: E402  (GGUF writer and the synthetic model)

N_TOK = 24
POS_HI = 32700
N_CTX_HI = 32768
SEED = 20250211

CASES = [
    # name, arch, n_rot, freq_base (None: the reference's default), with frequency factors
    ("neox", "qwen2", 128, 1.0e6, False),
    ("normal", "llama", 128, 5.0e5, True),
    ("partial", "llama", 64, None, False),
]


def build_model(q, k, v, arch, n_rot, freq_base, factors):
    meta, tensors = base.build_model(q, k, v)
    meta = [(key.replace("llama.", arch + "."), typ, arch if key == "general.architecture" else val)
            for key, typ, val in meta if not key.endswith("rope.dimension_count")]
    meta.append((arch + ".rope.dimension_count", base.GGUF_U32, n_rot))
    if freq_base is not None:
        meta.append((arch + ".rope.freq_base", base.GGUF_F32, float(freq_base)))
    if factors is not None:
        tensors = tensors + [("rope_freqs.weight", factors.reshape(1, -1).astype(np.float32))]
    return meta, tensors


def run_reference(meta, tensors, tmp, n_ctx, pos0):
    gguf = os.path.join(tmp, "rope.gguf")
    out = os.path.join(tmp, "logits.bin")
    base.write_gguf(gguf, meta, tensors)
    subprocess.run([base.DRIVER, gguf, str(N_TOK), str(n_ctx), str(base.N_LOGITS), out, str(pos0)], check=True)
    logits = np.fromfile(out, dtype="<f4").reshape(N_TOK, base.N_LOGITS)
    os.remove(gguf)
    return logits


def main():
    if not os.path.exists(base.DRIVER):
        sys.exit("build the driver first: make -C oracle ref")
    base.N_TOK = N_TOK  # the synthetic model's token count (columns of the projections, row of ones)
    rng = np.random.default_rng(SEED)
    q = rng.standard_normal((N_TOK, base.ATT)).astype(np.float32)
    k = rng.standard_normal((N_TOK, base.N_KV * base.D)).astype(np.float32)
    v = rng.standard_normal((N_TOK, base.N_KV * base.D)).astype(np.float32)
    # frequency factors in the style of Llama-3's long-context scaling: 1 for the fast pairs, 8 for the
    # slow ones, a ramp between
    i = np.arange(64)
    factors = np.clip(1.0 + 7.0 * (i - 20) / 24.0, 1.0, 8.0).astype(np.float32)
    store = dict(q=q, k=k, v=v, factors=factors,
                 meta=np.array([base.N_HEAD, base.N_KV, base.D, N_TOK, POS_HI, N_CTX_HI, base.OUT_BASE, base.N_EMBD], np.int32))
    with tempfile.TemporaryDirectory(dir="/tmp") as tmp:
        for name, arch, n_rot, freq_base, with_ff in CASES:
            meta, tensors = build_model(q, k, v, arch, n_rot, freq_base, factors if with_ff else None)
            store[f"logits_{name}_lo"] = run_reference(meta, tensors, tmp, 256, 0)
            store[f"logits_{name}_hi"] = run_reference(meta, tensors, tmp, N_CTX_HI, POS_HI)
    dst = os.path.join(HERE, "rope_reference.npz")
    np.savez(dst, **store)
    print("wrote", dst, os.path.getsize(dst), "bytes")


if __name__ == "__main__":
    main()
