"""ctypes binding of the CPU oracle (oracle/liborin_oracle.so) -- TEST INFRASTRUCTURE.

Importable only from tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg.
The product package never imports this module.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liborin_oracle.so")

_f32p = ctypes.POINTER(ctypes.c_float)
_u16p = ctypes.POINTER(ctypes.c_uint16)
_i32p = ctypes.POINTER(ctypes.c_int)
_int = ctypes.c_int
_flt = ctypes.c_float


def build():
    """Compile the C restatement (gcc, a few seconds)."""
    subprocess.run(["make", "-C", _HERE, "liborin_oracle.so"], check=True, capture_output=True)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    lib = ctypes.CDLL(_LIB_PATH)
    lib.orc_fp16_to_fp32_n.argtypes = [_u16p, _f32p, ctypes.c_size_t]
    lib.orc_fp32_to_fp16_n.argtypes = [_f32p, _u16p, ctypes.c_size_t]
    lib.orc_kv_store_f32.argtypes = [_f32p, _f32p, _f32p, _f32p, _int, _int, _int, _int, _int]
    lib.orc_kv_store_f16.argtypes = [_u16p, _u16p, _f32p, _f32p, _int, _int, _int, _int, _int]
    lib.orc_rope_batch.argtypes = [_f32p, _int, _int, _int, _flt, _int, _int, _f32p, _int]
    lib.orc_kv_shift_u16.argtypes = [_u16p, _u16p, _int, _int, _int, _int, _int, _int]
    lib.orc_attention_token_f32.argtypes = [_f32p, _f32p, _f32p, _f32p, _int, _int, _int, _int, _int, _flt, _f32p]
    lib.orc_attention_token_f16.argtypes = [_f32p, _u16p, _u16p, _f32p, _int, _int, _int, _int, _int, _flt, _f32p]
    lib.orc_attention_row_f16.argtypes = [_f32p, _u16p, _u16p, _f32p, _int, _int, _int, _int, _flt, _f32p]
    lib.orc_flash_attention.argtypes = [_f32p, _u16p, _u16p, _f32p, _int, _int, _int, _int, _int, _int, _flt]
    lib.orc_flash_attention_decode_ind.argtypes = [_f32p, _u16p, _u16p, _f32p, _int, _int, _int, _int, _i32p, _flt]
    lib.orc_flash_attention_rows.argtypes = [_f32p, _u16p, _u16p, _f32p, _i32p, _int,
                                             _int, _int, _int, _int, _int, _flt, _int]
    lib.orc_max_threads.restype = _int
    for name in ("orc_fp16_to_fp32_n", "orc_fp32_to_fp16_n", "orc_kv_store_f32", "orc_kv_store_f16",
                 "orc_attention_token_f32", "orc_attention_token_f16", "orc_attention_row_f16",
                 "orc_flash_attention", "orc_flash_attention_decode_ind", "orc_flash_attention_rows"):
        getattr(lib, name).restype = None
    return lib


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = _load()
    return _lib


def _p(a, typ):
    return a.ctypes.data_as(typ)


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


def fp16_to_fp32(bits):
    bits = _c(bits, np.uint16)
    out = np.empty(bits.shape, np.float32)
    lib().orc_fp16_to_fp32_n(_p(bits, _u16p), _p(out, _f32p), bits.size)
    return out


def fp32_to_fp16(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().orc_fp32_to_fp16_n(_p(x, _f32p), _p(out, _u16p), x.size)
    return out


def kv_store_f16(kc, vc, k, v, n_kv, d, n_ctx, pos_base, batch):
    """kc, vc: uint16 arrays [n_kv][n_ctx][d], modified in place; k, v: fp32 [batch][n_kv][d]."""
    k, v = _c(k, np.float32), _c(v, np.float32)
    assert kc.dtype == np.uint16 and kc.flags.c_contiguous and kc.size == n_kv * n_ctx * d
    lib().orc_kv_store_f16(_p(kc, _u16p), _p(vc, _u16p), _p(k, _f32p), _p(v, _f32p), n_kv, d, n_ctx, pos_base, batch)


def rope_batch(x, head_dim, n_rot, theta, n_past, heads, freq_factors=None, neox=True):
    """x: fp32 [rows][head_dim] (row = token * heads + head); returns the rotated copy."""
    x = np.array(x, dtype=np.float32, order="C", copy=True)
    rows = x.size // head_dim
    ff = None if freq_factors is None else _c(freq_factors, np.float32)
    lib().orc_rope_batch(_p(x, _f32p), rows, head_dim, n_rot, np.float32(theta), n_past, heads,
                         None if ff is None else _p(ff, _f32p), 1 if neox else 0)
    return x


def kv_shift_u16(kc, vc, n_layer, n_kv, d, n_ctx, n_keep, shift):
    """kc, vc: uint16 arrays [n_layer][n_kv][n_ctx][d], modified in place."""
    assert kc.dtype == np.uint16 and kc.flags.c_contiguous and kc.size == n_layer * n_kv * n_ctx * d
    assert vc.dtype == np.uint16 and vc.flags.c_contiguous and vc.size == kc.size
    assert 0 <= n_keep and 0 <= shift and n_keep + shift <= n_ctx
    lib().orc_kv_shift_u16(_p(kc, _u16p), _p(vc, _u16p), n_layer, n_kv, d, n_ctx, n_keep, shift)


def kv_store_f32(kc, vc, k, v, n_kv, d, n_ctx, pos_base, batch):
    k, v = _c(k, np.float32), _c(v, np.float32)
    assert kc.dtype == np.float32 and kc.flags.c_contiguous and kc.size == n_kv * n_ctx * d
    lib().orc_kv_store_f32(_p(kc, _f32p), _p(vc, _f32p), _p(k, _f32p), _p(v, _f32p), n_kv, d, n_ctx, pos_base, batch)


def attention_token_f32(q, kc, vc, n_head, n_kv, d, n_ctx, npos, scale):
    q, kc, vc = _c(q, np.float32), _c(kc, np.float32), _c(vc, np.float32)
    out = np.empty((n_head, d), np.float32)
    score = np.empty(max(npos, 1), np.float32)
    lib().orc_attention_token_f32(_p(q, _f32p), _p(kc, _f32p), _p(vc, _f32p), _p(out, _f32p),
                                  n_head, n_kv, d, n_ctx, npos, scale, _p(score, _f32p))
    return out


def attention_token_f16(q, kc, vc, n_head, n_kv, d, n_ctx, npos, scale):
    q, kc, vc = _c(q, np.float32), _c(kc, np.uint16), _c(vc, np.uint16)
    out = np.empty((n_head, d), np.float32)
    score = np.empty(max(npos, 1), np.float32)
    lib().orc_attention_token_f16(_p(q, _f32p), _p(kc, _u16p), _p(vc, _u16p), _p(out, _f32p),
                                  n_head, n_kv, d, n_ctx, npos, scale, _p(score, _f32p))
    return out


def flash_attention(q, kc, vc, n_head, n_kv, d, n_ctx, n_past, batch, scale):
    """Same call shape as the operator API: q fp32 [batch][n_head][d]; caches uint16 [n_kv][n_ctx][d]."""
    q, kc, vc = _c(q, np.float32), _c(kc, np.uint16), _c(vc, np.uint16)
    assert q.size == batch * n_head * d and kc.size == n_kv * n_ctx * d == vc.size
    out = np.empty((batch, n_head, d), np.float32)
    lib().orc_flash_attention(_p(q, _f32p), _p(kc, _u16p), _p(vc, _u16p), _p(out, _f32p),
                              n_head, n_kv, d, n_ctx, n_past, batch, scale)
    return out


def flash_attention_decode_ind(q, kc, vc, n_head, n_kv, d, n_ctx, pos, scale):
    q, kc, vc = _c(q, np.float32), _c(kc, np.uint16), _c(vc, np.uint16)
    assert q.size == n_head * d and kc.size == n_kv * n_ctx * d == vc.size
    out = np.empty((n_head, d), np.float32)
    p = ctypes.c_int(int(pos))
    lib().orc_flash_attention_decode_ind(_p(q, _f32p), _p(kc, _u16p), _p(vc, _u16p), _p(out, _f32p),
                                         n_head, n_kv, d, n_ctx, ctypes.byref(p), scale)
    return out


def flash_attention_rows(q, kc, vc, rows, n_head, n_kv, d, n_ctx, n_past, scale, threads=0):
    """rows: int array [n_rows][2] of (token, head).  Returns fp32 [n_rows][d]."""
    q, kc, vc = _c(q, np.float32), _c(kc, np.uint16), _c(vc, np.uint16)
    rows = _c(rows, np.int32).reshape(-1, 2)
    out = np.empty((rows.shape[0], d), np.float32)
    if threads <= 0:
        threads = max_threads()
    lib().orc_flash_attention_rows(_p(q, _f32p), _p(kc, _u16p), _p(vc, _u16p), _p(out, _f32p),
                                   _p(rows, _i32p), rows.shape[0], n_head, n_kv, d, n_ctx, n_past,
                                   scale, threads)
    return out


def max_threads():
    return min(int(lib().orc_max_threads()), 16)


def attention_f64(q, k, v, n_past, scale):
    """Textbook closed form in float64, independent of the C code.

    q [batch][n_head][d]; k, v [n_kv][L][d] (any float dtype, L >= n_past + batch);
    token b sees positions [0, n_past + b + 1).  Returns float64 [batch][n_head][d].
    """
    q = np.asarray(q, np.float64)
    k = np.asarray(k, np.float64)
    v = np.asarray(v, np.float64)
    batch, n_head, d = q.shape
    n_kv = k.shape[0]
    out = np.empty((batch, n_head, d), np.float64)
    L = n_past + batch
    for h in range(n_head):
        g = h * n_kv // n_head
        s = (q[:, h, :] @ k[g, :L, :].T) * float(scale)  # [batch][L]
        mask = np.arange(L)[None, :] > (n_past + np.arange(batch))[:, None]
        s = np.where(mask, -np.inf, s)
        s = s - s.max(axis=1, keepdims=True)
        p = np.exp(s)
        p /= p.sum(axis=1, keepdims=True)
        out[:, h, :] = p @ v[g, :L, :]
    return out


# ---- the decode layer around attention (layer_ref.h) ----

F32, F16, Q8_0, Q4_K, Q5_K, Q6_K = 0, 1, 8, 12, 13, 14
_vp = ctypes.c_void_p


def _layer_lib():
    l = lib()
    if not getattr(l, "_layer_ready", False):
        l.orc_row_bytes.argtypes = [_int, ctypes.c_int64]
        l.orc_row_bytes.restype = ctypes.c_size_t
        l.orc_dequantize_row.argtypes = [_int, _vp, _f32p, ctypes.c_int64]
        l.orc_dequantize_row.restype = _int
        l.orc_gemv.argtypes = [_int, _vp, _f32p, _f32p, _int, _int, _f32p]
        l.orc_gemv.restype = _int
        l.orc_rms_norm.argtypes = [_f32p, _f32p, _int, _flt, _f32p]
        l.orc_rms_norm.restype = None
        l.orc_swiglu.argtypes = [_f32p, _f32p, _f32p, _int]
        l.orc_swiglu.restype = None
        l._layer_ready = True
    return l


def row_bytes(wtype, n):
    return int(_layer_lib().orc_row_bytes(wtype, n))


def dequantize_row(wtype, raw, k):
    """raw: the row's bytes (uint8 array); returns fp32 [k]."""
    raw = _c(raw, np.uint8)
    assert raw.size >= row_bytes(wtype, k) > 0
    y = np.empty(k, np.float32)
    assert _layer_lib().orc_dequantize_row(wtype, raw.ctypes.data, _p(y, _f32p), k) == 0
    return y


def gemv(wtype, raw, x, n_in, n_out):
    """raw: n_out rows of n_in elements of type wtype (uint8 array); x fp32 [n_in]; returns fp32 [n_out]."""
    raw, x = _c(raw, np.uint8), _c(x, np.float32)
    assert raw.size >= row_bytes(wtype, n_in) * n_out > 0 and x.size == n_in
    y = np.empty(n_out, np.float32)
    row = np.empty(n_in, np.float32)
    assert _layer_lib().orc_gemv(wtype, raw.ctypes.data, _p(x, _f32p), _p(y, _f32p), n_in, n_out, _p(row, _f32p)) == 0
    return y


def rms_norm(x, w, eps):
    x, w = _c(x, np.float32), _c(w, np.float32)
    y = np.empty(x.size, np.float32)
    _layer_lib().orc_rms_norm(_p(x, _f32p), _p(w, _f32p), x.size, np.float32(eps), _p(y, _f32p))
    return y


def swiglu(gate, up):
    gate, up = _c(gate, np.float32), _c(up, np.float32)
    act = np.empty(gate.size, np.float32)
    _layer_lib().orc_swiglu(_p(act, _f32p), _p(gate, _f32p), _p(up, _f32p), gate.size)
    return act


class RefState:
    """The caches of one sequence: fp32 as the reference's CPU backend keeps them
    (src/model_cpu.cpp:217,226-231), or, with fp16_cache, rounded to fp16 on the way in as the
    GPU backend's cache is (src/kernels.cu:1675-1677)."""

    def __init__(self, model, n_ctx, fp16_cache=False):
        hp = model["hp"]
        shape = (hp["n_layer"], hp["n_kv"], n_ctx, hp["head_dim"])
        self.n_ctx, self.fp16_cache = n_ctx, fp16_cache
        self.kc = np.zeros(shape, np.float32)
        self.vc = np.zeros(shape, np.float32)


def decode_forward(model, state, token, n_past, trace=None):
    """One token through the whole model, as src/model_cpu.cpp:241-312 walks it; returns the logits.

    model: {"hp": {n_vocab, n_embd, n_layer, n_head, n_kv, head_dim, n_ff, n_rot, rms_eps,
    rope_theta, neox, freq_factors}, "token_embd": T, "output": T, "output_norm": fp32 array,
    "layers": [{"wq", "wk", "wv", "wo", "ffn_gate", "ffn_up", "ffn_down": T, "attn_norm", "ffn_norm":
    fp32 arrays, optional "bq", "bk", "bv", "q_norm", "k_norm": fp32 arrays}]} with
    T = (type, uint8 array of the tensor's bytes, n_in, n_out).
    trace: optional dict that receives the intermediate vectors of every layer.
    """
    hp = model["hp"]
    ne, nh, nkv, d, nff = hp["n_embd"], hp["n_head"], hp["n_kv"], hp["head_dim"], hp["n_ff"]
    eps, n_ctx = hp["rms_eps"], state.n_ctx
    scale = np.float32(1.0) / np.sqrt(np.float32(d))

    def mv(t, x):
        return gemv(t[0], t[1], x, t[2], t[3])

    def rope(x, heads):
        return rope_batch(x.reshape(heads, d), d, hp["n_rot"], hp["rope_theta"], n_past, heads,
                          hp.get("freq_factors"), bool(hp["neox"])).reshape(-1)

    et, eraw, e_in, _ = model["token_embd"]
    rb = row_bytes(et, e_in)
    x = dequantize_row(et, eraw[token * rb:(token + 1) * rb], ne)
    for li, L in enumerate(model["layers"]):
        xn = rms_norm(x, L["attn_norm"], eps)
        q, k, v = mv(L["wq"], xn), mv(L["wk"], xn), mv(L["wv"], xn)
        if L.get("bq") is not None:
            q = q + L["bq"]
        if L.get("bk") is not None:
            k = k + L["bk"]
        if L.get("bv") is not None:
            v = v + L["bv"]
        if L.get("q_norm") is not None:
            q = np.concatenate([rms_norm(q[h * d:(h + 1) * d], L["q_norm"], eps) for h in range(nh)])
        if L.get("k_norm") is not None:
            k = np.concatenate([rms_norm(k[h * d:(h + 1) * d], L["k_norm"], eps) for h in range(nkv)])
        q, k = rope(q, nh), rope(k, nkv)
        if state.fp16_cache:
            k_in, v_in = fp16_to_fp32(fp32_to_fp16(k)), fp16_to_fp32(fp32_to_fp16(v))
        else:
            k_in, v_in = k, v
        state.kc[li, :, n_past, :] = k_in.reshape(nkv, d)
        state.vc[li, :, n_past, :] = v_in.reshape(nkv, d)
        attn = attention_token_f32(q.reshape(nh, d), state.kc[li], state.vc[li], nh, nkv, d, n_ctx, n_past + 1,
                                   scale).reshape(-1)
        x1 = x + mv(L["wo"], attn)
        xn2 = rms_norm(x1, L["ffn_norm"], eps)
        act = swiglu(mv(L["ffn_gate"], xn2), mv(L["ffn_up"], xn2))
        x2 = x1 + mv(L["ffn_down"], act)
        if trace is not None:
            trace[li] = dict(x_in=x, xn=xn, q=q, k=k, v=v, attn=attn, x_mid=x1, xn2=xn2, act=act, x_out=x2)
        x = x2
    xn = rms_norm(x, model["output_norm"], eps)
    return mv(model["output"], xn)
