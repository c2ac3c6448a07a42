"""ctypes mirror of the decode-layer operators around attention, same names and argument order as
the reference's src/kernels.h:15-47, plus the fused forms of include/orin_layer.h.  Pointer
arguments accept torch tensors (device memory) or raw integer addresses; a non-zero return code
raises.  `decode_layer_calls` is the reference's decode_layer (src/model_gpu.cu:251-293) call for
call; `decode_layer` is the same layer through the library's one entry point.
"""
import ctypes

from . import kernels as _k

F32, F16, Q8_0, Q4_K, Q5_K, Q6_K = 0, 1, 8, 12, 13, 14

_vp, _int, _flt = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
_ready = False


class DecodeLayerDesc(ctypes.Structure):
    """struct orin_decode_layer_desc of include/orin_layer.h."""
    _fields_ = ([(n, _int) for n in ("n_embd", "n_head", "n_kv", "head_dim", "n_ff", "n_ctx", "n_rot", "neox")]
                + [(n, _flt) for n in ("rms_eps", "rope_theta", "scale")]
                + [(n, _int) for n in ("wq_type", "wk_type", "wv_type", "wo_type", "gate_type", "up_type", "down_type")]
                + [(n, _vp) for n in ("wq", "wk", "wv", "wo", "ffn_gate", "ffn_up", "ffn_down", "attn_norm", "ffn_norm",
                                      "q_norm", "k_norm", "bq", "bk", "bv", "freq_factors", "rope_angles", "kc", "vc",
                                      "x", "q", "k", "v", "attn", "act", "up_tmp", "d_pos")])


def _lib():
    global _ready
    L = _k.lib()
    if not _ready:
        L.orin_gemv_use_matrix_cores.argtypes = [_int]
        L.orin_gemv_use_matrix_cores.restype = None
        L.orin_gemv_row_shares.argtypes = [_int]
        L.orin_gemv_row_shares.restype = None
        L.orin_row_bytes.argtypes = [_int, _int]
        L.orin_row_bytes.restype = ctypes.c_size_t
        L.orin_rms_norm.argtypes = [_vp, _vp, _int, _flt, _vp]
        L.orin_rms_norm_rows.argtypes = [_vp, _vp, _int, _int, _flt, _vp]
        L.orin_quantize_activation.argtypes = [_vp, _int]
        L.orin_gemv_q8.argtypes = [_int, _vp, _vp, _int, _int]
        L.orin_gemv_q8_bias.argtypes = [_int, _vp, _vp, _vp, _int, _int]
        L.orin_gemv_q8_add.argtypes = [_int, _vp, _vp, _int, _int]
        L.orin_gemv_fused_gate_up_swiglu.argtypes = [_int, _vp, _vp, _vp, _int, _int]
        L.orin_gemv.argtypes = [_int, _vp, _vp, _vp, _int, _int]
        L.orin_dequant_row.argtypes = [_int, _vp, _vp, _int]
        L.orin_swiglu.argtypes = [_vp, _vp, _vp, _int]
        L.orin_gemv_multi.argtypes = [_int, _int, ctypes.POINTER(_vp), ctypes.POINTER(_vp), ctypes.POINTER(_vp),
                                      ctypes.POINTER(_int), _vp, _vp, _flt, _int, _int]
        L.orin_gemv_multi_types.argtypes = [ctypes.POINTER(_int), _int, ctypes.POINTER(_vp), ctypes.POINTER(_vp), ctypes.POINTER(_vp),
                                            ctypes.POINTER(_int), _vp, _vp, _flt, _int]
        L.orin_gemv_norm_gate_up_swiglu.argtypes = [_int, _vp, _vp, _vp, _vp, _flt, _vp, _int, _int]
        L.orin_decode_layer.argtypes = [ctypes.POINTER(DecodeLayerDesc)]
        for n in ("orin_rms_norm", "orin_rms_norm_rows", "orin_quantize_activation", "orin_gemv_q8", "orin_gemv_q8_bias",
                  "orin_gemv_q8_add", "orin_gemv_fused_gate_up_swiglu", "orin_gemv", "orin_dequant_row", "orin_swiglu",
                  "orin_gemv_multi", "orin_gemv_multi_types", "orin_gemv_norm_gate_up_swiglu", "orin_decode_layer"):
            getattr(L, n).restype = _int
        _ready = True
    return L


_p = _k._ptr


def _check(what, rc):
    if rc != 0:
        raise _k.OrinFaError(what, rc)


def use_matrix_cores(on):
    """Block types on the matrix cores (default) or on the vector ALU (for comparisons and tests)."""
    _lib().orin_gemv_use_matrix_cores(1 if on else 0)


def gemv_row_shares(shares):
    """Shares an accumulating projection may cut a row into: 0 = chosen by shape (default), 1 = never cut (every
    result bit for bit reproducible)."""
    _lib().orin_gemv_row_shares(int(shares))


def row_bytes(wtype, n):
    return int(_lib().orin_row_bytes(wtype, n))


def rms_norm(x, w, n, eps, y):
    _check("rms_norm", _lib().orin_rms_norm(_p(x), _p(w), n, eps, _p(y)))


def rms_norm_rows(x, w, rows, cols, eps, y):
    _check("rms_norm_rows", _lib().orin_rms_norm_rows(_p(x), _p(w), rows, cols, eps, _p(y)))


def quantize_activation(x, n_in):
    _check("quantize_activation", _lib().orin_quantize_activation(_p(x), n_in))


def gemv(wtype, W, x, y, n_in, n_out):
    _check("gemv", _lib().orin_gemv(wtype, _p(W), _p(x), _p(y), n_in, n_out))


def gemv_q8(wtype, W, y, n_in, n_out):
    _check("gemv_q8", _lib().orin_gemv_q8(wtype, _p(W), _p(y), n_in, n_out))


def gemv_q8_bias(wtype, W, bias, y, n_in, n_out):
    _check("gemv_q8_bias", _lib().orin_gemv_q8_bias(wtype, _p(W), _p(bias), _p(y), n_in, n_out))


def gemv_q8_add(wtype, W, y, n_in, n_out):
    _check("gemv_q8_add", _lib().orin_gemv_q8_add(wtype, _p(W), _p(y), n_in, n_out))


def gemv_fused_gate_up_swiglu(wtype, Wg, Wu, out, n_in, n_out):
    _check("gemv_fused_gate_up_swiglu", _lib().orin_gemv_fused_gate_up_swiglu(wtype, _p(Wg), _p(Wu), _p(out), n_in, n_out))


def dequant_row(wtype, src, y, n):
    _check("dequant_row", _lib().orin_dequant_row(wtype, _p(src), _p(y), n))


def swiglu(act, gate, up, n):
    _check("swiglu", _lib().orin_swiglu(_p(act), _p(gate), _p(up), n))


def gemv_multi(wtype, Ws, biases, ys, n_outs, x, norm_w, eps, n_in, accumulate=False):
    """Up to three matrices of one type over x in one launch, the RMS norm (norm_w, or None) folded in."""
    m = len(Ws)
    arr = lambda xs: (_vp * m)(*[_p(v) for v in xs])  # noqa: E731
    _check("gemv_multi", _lib().orin_gemv_multi(wtype, m, arr(Ws), arr(biases) if biases is not None else None, arr(ys),
                                                (_int * m)(*n_outs), _p(x), _p(norm_w), eps, n_in, 1 if accumulate else 0))


def gemv_multi_types(wtypes, Ws, biases, ys, n_outs, x, norm_w, eps, n_in):
    """gemv_multi with a type per matrix."""
    m = len(Ws)
    arr = lambda xs: (_vp * m)(*[_p(v) for v in xs])  # noqa: E731
    _check("gemv_multi_types", _lib().orin_gemv_multi_types((_int * m)(*wtypes), m, arr(Ws), arr(biases) if biases is not None else None,
                                                            arr(ys), (_int * m)(*n_outs), _p(x), _p(norm_w), eps, n_in))


def gemv_norm_gate_up_swiglu(wtype, Wg, Wu, x, norm_w, eps, out, n_in, n_out):
    _check("gemv_norm_gate_up_swiglu",
           _lib().orin_gemv_norm_gate_up_swiglu(wtype, _p(Wg), _p(Wu), _p(x), _p(norm_w), eps, _p(out), n_in, n_out))


def make_desc(hp, L, bufs, kc, vc, d_pos, n_ctx, rope_angles=None):
    """hp: the model's shape parameters; L: one layer's device tensors {name: (type, tensor) or tensor};
    bufs: {x, q, k, v, attn, act, up_tmp}."""
    d = DecodeLayerDesc()
    d.n_embd, d.n_head, d.n_kv, d.head_dim, d.n_ff = hp["n_embd"], hp["n_head"], hp["n_kv"], hp["head_dim"], hp["n_ff"]
    d.n_ctx, d.n_rot, d.neox = n_ctx, hp["n_rot"], hp["neox"]
    d.rms_eps, d.rope_theta, d.scale = hp["rms_eps"], hp["rope_theta"], 1.0 / float(hp["head_dim"]) ** 0.5
    for name, field in (("wq", "wq"), ("wk", "wk"), ("wv", "wv"), ("wo", "wo"), ("ffn_gate", "gate"), ("ffn_up", "up"),
                        ("ffn_down", "down")):
        setattr(d, field + "_type", L[name][0])
        setattr(d, name, _p(L[name][1]))
    for name in ("attn_norm", "ffn_norm", "q_norm", "k_norm", "bq", "bk", "bv"):
        setattr(d, name, _p(L.get(name)))
    d.freq_factors, d.rope_angles = _p(hp.get("freq_factors_dev")), _p(rope_angles)
    d.kc, d.vc, d.d_pos = _p(kc), _p(vc), _p(d_pos)
    for name in ("x", "q", "k", "v", "attn", "act", "up_tmp"):
        setattr(d, name, _p(bufs.get(name)))
    return d


def decode_layer(desc):
    _check("decode_layer", _lib().orin_decode_layer(ctypes.byref(desc)))


def decode_layer_calls(hp, L, bufs, kc, vc, d_pos, n_ctx, ops=None):
    """The reference's decode_layer, call for call (src/model_gpu.cu:251-293).  bufs additionally holds xn, xn2.
    ops: an object with the operators under the reference's names (default: this module and kernels)."""
    if ops is not None:
        return _decode_layer_calls(ops, ops, hp, L, bufs, kc, vc, d_pos, n_ctx)
    import sys
    return _decode_layer_calls(sys.modules[__name__], _k, hp, L, bufs, kc, vc, d_pos, n_ctx)


def _decode_layer_calls(o, ka, hp, L, bufs, kc, vc, d_pos, n_ctx):
    rms_norm, rms_norm_rows, quantize_activation, swiglu = o.rms_norm, o.rms_norm_rows, o.quantize_activation, o.swiglu
    gemv_q8, gemv_q8_bias, gemv_q8_add, gemv_fused_gate_up_swiglu = o.gemv_q8, o.gemv_q8_bias, o.gemv_q8_add, o.gemv_fused_gate_up_swiglu
    ne, nh, nkv, hd, nff = hp["n_embd"], hp["n_head"], hp["n_kv"], hp["head_dim"], hp["n_ff"]
    eps, scale = hp["rms_eps"], 1.0 / float(hd) ** 0.5
    x, xn, xn2, q, k, v, attn, act = (bufs[n] for n in ("x", "xn", "xn2", "q", "k", "v", "attn", "act"))
    rms_norm(x, L["attn_norm"], ne, eps, xn)
    quantize_activation(xn, ne)
    if L.get("bq") is not None:
        gemv_q8_bias(L["wq"][0], L["wq"][1], L["bq"], q, ne, nh * hd)
        gemv_q8_bias(L["wk"][0], L["wk"][1], L["bk"], k, ne, nkv * hd)
        gemv_q8_bias(L["wv"][0], L["wv"][1], L["bv"], v, ne, nkv * hd)
    else:
        gemv_q8(L["wq"][0], L["wq"][1], q, ne, nh * hd)
        gemv_q8(L["wk"][0], L["wk"][1], k, ne, nkv * hd)
        gemv_q8(L["wv"][0], L["wv"][1], v, ne, nkv * hd)
    if L.get("q_norm") is not None:
        rms_norm_rows(q, L["q_norm"], nh, hd, eps, q)
    if L.get("k_norm") is not None:
        rms_norm_rows(k, L["k_norm"], nkv, hd, eps, k)
    rope_ind = ka.rope_neox_ind if hp["neox"] else ka.rope_normal_ind
    rope_ind(q, nh, hd, hp["n_rot"], hp["rope_theta"], d_pos, hp.get("freq_factors_dev"))
    rope_ind(k, nkv, hd, hp["n_rot"], hp["rope_theta"], d_pos, hp.get("freq_factors_dev"))
    ka.kv_store_ind(kc, vc, k, v, nkv, hd, n_ctx, d_pos)
    ka.flash_attention_decode_ind(q, kc, vc, attn, nh, nkv, hd, n_ctx, d_pos, scale)
    quantize_activation(attn, ne)  # (as the reference: n_embd elements staged, the product reads the first n_head * head_dim)
    gemv_q8_add(L["wo"][0], L["wo"][1], x, nh * hd, ne)
    rms_norm(x, L["ffn_norm"], ne, eps, xn2)
    quantize_activation(xn2, ne)
    if L["ffn_gate"][0] == L["ffn_up"][0]:
        gemv_fused_gate_up_swiglu(L["ffn_gate"][0], L["ffn_gate"][1], L["ffn_up"][1], act, ne, nff)
    else:  # (the reference's fused kernel takes one type for both; mixed pairs go through the plain products)
        gemv_q8(L["ffn_gate"][0], L["ffn_gate"][1], act, ne, nff)
        gemv_q8(L["ffn_up"][0], L["ffn_up"][1], bufs["up_tmp"], ne, nff)
        swiglu(act, act, bufs["up_tmp"], nff)
    quantize_activation(act, nff)
    gemv_q8_add(L["ffn_down"][0], L["ffn_down"][1], x, nff, ne)
