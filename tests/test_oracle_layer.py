"""The decode-layer oracle (oracle/layer_ref.c, oracle/ref.py decode_forward) against what pins it:
the logits of the unmodified reference CPU build over small quantised models
(tests/golden/layer_reference.npz, written by tests/golden/make_layer_fixture.py), an independent
whole-array numpy decoding of the block formats, and facts of the operators that need no second
implementation.  CPU only.
"""
import os
import sys

import numpy as np
import pytest

from oracle import ref

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import layer_model as lm  # noqa: E402


@pytest.fixture(scope="module")
def golden():
    return np.load(os.path.join(HERE, "golden", "layer_reference.npz"))


@pytest.mark.parametrize("name", list(lm.VARIANTS))
def test_decode_forward_reproduces_the_reference_logits_bit_for_bit(golden, name):
    """Every operator of the layer sits between the token and the logits: a wrong nibble, pair,
    fifth bit, scale sign, norm or activation anywhere changes them."""
    model = lm.build(name)
    n_tok, n_ctx = (int(v) for v in golden["meta"])
    state = ref.RefState(model, n_ctx)
    for t in range(n_tok):
        got = ref.decode_forward(model, state, t, t)
        want = golden["logits_" + name][t]
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (name, t, float(np.abs(got - want).max()))


# ---- the block formats once more, written as whole-array numpy expressions ----

def _pairs(s):
    """s: uint8 [nb][12] -> (scale, min) uint8 [nb][8] each."""
    s = s.astype(np.uint16)
    sc = np.empty((s.shape[0], 8), np.uint16)
    mn = np.empty_like(sc)
    sc[:, :4], mn[:, :4] = s[:, 0:4] & 63, s[:, 4:8] & 63
    sc[:, 4:] = (s[:, 8:12] & 15) | ((s[:, 0:4] >> 6) << 4)
    mn[:, 4:] = (s[:, 8:12] >> 4) | ((s[:, 4:8] >> 6) << 4)
    return sc, mn


def _f16(b):
    return np.ascontiguousarray(b).view(np.float16).astype(np.float32).reshape(-1)


def numpy_decode(wtype, raw, n):
    per, nbytes = lm.BLOCK[wtype]
    b = raw.reshape(-1, nbytes)
    if wtype == lm.F32:
        return raw.view(np.float32).copy()
    if wtype == lm.F16:
        return raw.view(np.float16).astype(np.float32)
    if wtype == lm.Q8_0:
        return (_f16(b[:, 0:2])[:, None] * b[:, 2:].view(np.int8).astype(np.float32)).reshape(-1)
    if wtype in (lm.Q4_K, lm.Q5_K):
        d, dmin = _f16(b[:, 0:2]), _f16(b[:, 2:4])
        sc, mn = _pairs(b[:, 4:16])
        qs = b[:, 48:176] if wtype == lm.Q5_K else b[:, 16:144]
        qs = qs.reshape(-1, 4, 32)
        q = np.stack([qs & 15, qs >> 4], axis=2).reshape(-1, 8, 32).astype(np.int32)  # [nb][pair][32]
        if wtype == lm.Q5_K:
            hb = (b[:, 16:48][:, None, :] >> np.arange(8, dtype=np.uint8)[None, :, None]) & 1
            q = q + 16 * hb
        dp = d[:, None] * sc.astype(np.float32)
        mp = dmin[:, None] * mn.astype(np.float32)
        return (dp[:, :, None] * q.astype(np.float32) - mp[:, :, None]).reshape(-1)
    if wtype == lm.Q6_K:
        ql, qh = b[:, 0:128].reshape(-1, 2, 2, 32), b[:, 128:192].reshape(-1, 2, 32)
        sc = b[:, 192:208].view(np.int8).reshape(-1, 2, 4, 2).astype(np.float32)  # [nb][half][strip][l / 16]
        d = _f16(b[:, 208:210])
        out = np.empty((b.shape[0], 2, 4, 32), np.float32)
        for c in range(4):
            nib = (ql[:, :, c & 1, :] & 15) if c < 2 else (ql[:, :, c & 1, :] >> 4)
            q = (nib | (((qh >> (2 * c)) & 3) << 4)).astype(np.int32) - 32
            s = np.repeat(sc[:, :, c, :], 16, axis=2)
            out[:, :, c, :] = d[:, None, None] * s * q.astype(np.float32)
        return out.reshape(-1)
    raise ValueError(wtype)


@pytest.mark.parametrize("wtype", [lm.F32, lm.F16, lm.Q8_0, lm.Q4_K, lm.Q5_K, lm.Q6_K])
def test_dequantize_row_matches_whole_array_numpy_decoding(wtype):
    n = 1024
    t = lm.make_tensor(lm.Stream(900 + wtype), wtype, n, 3)
    rb = ref.row_bytes(wtype, n)
    assert rb == n // lm.BLOCK[wtype][0] * lm.BLOCK[wtype][1]
    for r in range(3):
        raw = t[1][r * rb:(r + 1) * rb]
        got = ref.dequantize_row(wtype, raw, n)
        want = numpy_decode(wtype, raw, n)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), lm.TYPE_NAME[wtype]


def test_row_bytes_rejects_partial_blocks_and_unknown_types():
    assert ref.row_bytes(lm.Q4_K, 300) == 0 and ref.row_bytes(lm.Q8_0, 48) == 0 and ref.row_bytes(7, 256) == 0
    assert ref.row_bytes(lm.Q4_K, 512) == 288 and ref.row_bytes(lm.Q5_K, 256) == 176
    assert ref.row_bytes(lm.Q6_K, 256) == 210 and ref.row_bytes(lm.Q8_0, 64) == 68


def test_gemv_is_the_sequential_fp32_dot_of_the_decoded_rows():
    n_in, n_out = 512, 5
    rs = lm.Stream(77)
    t = lm.make_tensor(rs, lm.Q4_K, n_in, n_out)
    x = rs.sym(n_in, 1.0)
    y = ref.gemv(lm.Q4_K, t[1], x, n_in, n_out)
    rb = ref.row_bytes(lm.Q4_K, n_in)
    for j in range(n_out):
        row = ref.dequantize_row(lm.Q4_K, t[1][j * rb:(j + 1) * rb], n_in)
        s = np.float32(0.0)
        for a, b in zip(row, x):
            s = np.float32(s + np.float32(a * b))
        assert s == y[j]
    # and, loosely, the float64 product
    w = np.stack([numpy_decode(lm.Q4_K, t[1][j * rb:(j + 1) * rb], n_in) for j in range(n_out)]).astype(np.float64)
    assert np.allclose(y, w @ x.astype(np.float64), rtol=0, atol=1e-5 * np.abs(w).sum(axis=1).max())


def test_rms_norm_and_swiglu_special_cases():
    x = np.full(64, 3.0, np.float32)
    w = np.arange(64, dtype=np.float32)
    assert np.allclose(ref.rms_norm(x, w, 0.0), w, rtol=1e-7)          # a constant vector normalises to ones
    assert np.array_equal(ref.rms_norm(-x, w, 0.0), -ref.rms_norm(x, w, 0.0))
    y = ref.rms_norm(np.array([3.0, 4.0], np.float32), np.ones(2, np.float32), 0.0)
    assert np.allclose(y, np.array([3.0, 4.0]) / np.sqrt(12.5), rtol=1e-7)
    g = np.array([0.0, 1.0, -1.0, 30.0, -30.0], np.float32)
    u = np.array([2.0, 2.0, 2.0, 1.0, 1.0], np.float32)
    want = g.astype(np.float64) / (1.0 + np.exp(-g.astype(np.float64))) * u
    assert np.allclose(ref.swiglu(g, u), want, rtol=2e-7, atol=1e-12)


def test_fp16_cache_moves_the_logits_only_a_little():
    """The GPU path keeps K and V in fp16; the reference CPU build in fp32.  The difference at the
    logits, for the checks of the GPU path that compare against the stored reference logits."""
    model = lm.build("llama")
    a, b = ref.RefState(model, 32), ref.RefState(model, 32, fp16_cache=True)
    worst = 0.0
    for t in range(lm.N_TOKENS):
        la, lb = ref.decode_forward(model, a, t, t), ref.decode_forward(model, b, t, t)
        worst = max(worst, float(np.abs(la - lb).max() / np.abs(la).max()))
    print("fp16 cache vs fp32 cache at the logits:", worst)
    assert 0.0 < worst < 5e-3
