"""ctypes mirror of the operator API, same names and argument order as the reference's
src/kernels.h:8-12,77-81.  Pointer arguments accept torch tensors (device memory) or raw
integer addresses.  A non-zero return code from the library raises, the Python analogue of
the reference's print-and-abort (src/common.h:14-22).  There is no fallback: a missing
library is an ImportError.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liborin_fa.so")

_vp = ctypes.c_void_p
_int = ctypes.c_int
_flt = ctypes.c_float

STAMPS_LIB_PATH = os.path.join(_HERE, "liborin_fa_stamps.so")
BENCH_LIB_PATH = os.path.join(_HERE, "liborin_fa_bench.so")

_lib = None
_stamps_lib = None
_bench_lib = None
_stream = None  # what set_stream was last given: the measurement aids launch on it too


class OrinFaError(RuntimeError):
    def __init__(self, what, code):
        self.code = code
        super().__init__(f"{what}: orin_fa error {code} ({error_string(code)})")


def lib():
    """The loaded C-ABI library.  Raises if it has not been built (python -m orin_llm_amd.build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} is missing: build it with __graft_entry__.build() "
                              "(hipcc --offload-arch=gfx950); there is no CPU fallback")
        L = ctypes.CDLL(LIB_PATH)
        L.orin_fa_init.argtypes = [_int]
        L.orin_fa_init.restype = _int
        L.orin_fa_set_stream.argtypes = [_vp]
        L.orin_fa_set_stream.restype = None
        L.orin_fa_workspace_bytes.argtypes = []
        L.orin_fa_workspace_bytes.restype = ctypes.c_size_t
        L.orin_fa_set_workspace.argtypes = [_vp, ctypes.c_size_t]
        L.orin_fa_set_workspace.restype = _int
        L.orin_fa_prefill.argtypes = [_vp, _vp, _vp, _vp, _int, _int, _int, _int, _int, _int, _flt]
        L.orin_fa_prefill.restype = _int
        L.orin_fa_decode_ind.argtypes = [_vp, _vp, _vp, _vp, _int, _int, _int, _int, _vp, _flt]
        L.orin_fa_decode_ind.restype = _int
        L.orin_fa_decode_ind_static.argtypes = [_vp, _vp, _vp, _vp, _int, _int, _int, _int, _vp, _flt]
        L.orin_fa_decode_ind_static.restype = _int
        L.orin_fa_static_scratch_bytes.argtypes = []
        L.orin_fa_static_scratch_bytes.restype = ctypes.c_size_t
        L.orin_fa_decode_store_ind.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _int, _vp, _flt]
        L.orin_fa_decode_store_ind.restype = _int
        L.orin_fa_decode_rope_store_ind.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _int, _vp, _flt,
                                                    _int, _flt, _vp, _int, _vp]
        L.orin_fa_rope_store_batch.argtypes = [_vp, _vp, _vp, _vp, _vp, _int, _int, _int, _int, _int, _int, _int, _flt, _vp, _int]
        L.orin_fa_rope_store_batch.restype = _int
        L.orin_fa_rope_angles_ind.argtypes = [_vp, _int, _flt, _vp, _vp]
        L.orin_fa_rope_angles_ind.restype = _int
        L.orin_fa_decode_rope_store_ind.restype = _int
        L.orin_fa_rope_batch.argtypes = [_vp, _int, _int, _int, _flt, _int, _int, _vp, _int]
        L.orin_fa_rope_batch.restype = _int
        L.orin_fa_rope_ind.argtypes = [_vp, _int, _int, _int, _flt, _vp, _vp, _int]
        L.orin_fa_rope_ind.restype = _int
        L.orin_fa_kv_store_batch.argtypes = [_vp, _vp, _vp, _vp, _int, _int, _int, _int, _int]
        L.orin_fa_kv_store_batch.restype = _int
        L.orin_fa_kv_store_ind.argtypes = [_vp, _vp, _vp, _vp, _int, _int, _int, _vp]
        L.orin_fa_kv_store_ind.restype = _int
        L.orin_fa_kv_shift.argtypes = [_vp, _vp, _int, _int, _int, _int, _int, _int]
        L.orin_fa_kv_shift.restype = _int
        L.orin_fa_decode_splits.argtypes = [_int, _int, _int, _int]
        L.orin_fa_decode_splits.restype = _int
        L.orin_fa_cu_count.argtypes = []
        L.orin_fa_cu_count.restype = _int
        L.orin_fa_error_string.argtypes = [_int]
        L.orin_fa_error_string.restype = ctypes.c_char_p
        _lib = L
    return _lib


def _ptr(x):
    if x is None:
        return None
    if isinstance(x, int):
        return x
    return x.data_ptr()


def error_string(code):
    return lib().orin_fa_error_string(int(code)).decode()


def init(device=0):
    rc = lib().orin_fa_init(int(device))
    if rc != 0:
        raise OrinFaError("init", rc)
    return 0


def set_stream(stream):
    """stream: a hipStream_t address (e.g. torch.cuda.Stream.cuda_stream), or None/0 for the null stream."""
    global _stream
    _stream = _ptr(stream) or None
    lib().orin_fa_set_stream(_stream)


def workspace_bytes():
    return int(lib().orin_fa_workspace_bytes())


def set_workspace(dev_ptr, nbytes):
    rc = lib().orin_fa_set_workspace(_ptr(dev_ptr), int(nbytes))
    if rc != 0:
        raise OrinFaError("set_workspace", rc)


def flash_attention(q, kc, vc, out, n_head, n_kv, head_dim, n_ctx, n_past, batch, scale):
    rc = lib().orin_fa_prefill(_ptr(q), _ptr(kc), _ptr(vc), _ptr(out), n_head, n_kv, head_dim, n_ctx,
                               n_past, batch, scale)
    if rc != 0:
        raise OrinFaError("flash_attention", rc)


def flash_attention_decode_ind(q, kc, vc, out, n_head, n_kv, head_dim, n_ctx, d_pos, scale):
    rc = lib().orin_fa_decode_ind(_ptr(q), _ptr(kc), _ptr(vc), _ptr(out), n_head, n_kv, head_dim, n_ctx,
                                  _ptr(d_pos), scale)
    if rc != 0:
        raise OrinFaError("flash_attention_decode_ind", rc)


def flash_attention_decode_ind_static(q, kc, vc, out, n_head, n_kv, head_dim, n_ctx, d_pos, scale):
    """flash_attention_decode_ind with its partial results in the library's fixed device block: allocates
    nothing and needs no workspace (no counterpart in the reference)."""
    rc = lib().orin_fa_decode_ind_static(_ptr(q), _ptr(kc), _ptr(vc), _ptr(out), n_head, n_kv, head_dim, n_ctx,
                                         _ptr(d_pos), scale)
    if rc != 0:
        raise OrinFaError("flash_attention_decode_ind_static", rc)


def static_scratch_bytes():
    return int(lib().orin_fa_static_scratch_bytes())


def flash_attention_decode_store_ind(q, k_new, v_new, kc, vc, out, n_head, n_kv, head_dim, n_ctx, d_pos, scale):
    """kv_store_ind(kc, vc, k_new, v_new, n_kv, ...) followed by flash_attention_decode_ind(...), in the
    launches of the latter alone (no counterpart in the reference; the results are identical)."""
    rc = lib().orin_fa_decode_store_ind(_ptr(q), _ptr(k_new), _ptr(v_new), _ptr(kc), _ptr(vc), _ptr(out),
                                        n_head, n_kv, head_dim, n_ctx, _ptr(d_pos), scale)
    if rc != 0:
        raise OrinFaError("flash_attention_decode_store_ind", rc)


def flash_attention_decode_rope_store_ind(q, k_new, v_new, kc, vc, out, n_head, n_kv, head_dim, n_ctx, d_pos, scale,
                                          n_rot, theta, freq_factors=None, neox=True, angles=None):
    """rope_*_ind on q and on k_new, kv_store_ind and flash_attention_decode_ind in the launches of the last
    (no counterpart in the reference; q and k_new are taken before the rotation and left as they are).
    angles: optionally the table rope_angles_ind wrote for this token."""
    rc = lib().orin_fa_decode_rope_store_ind(_ptr(q), _ptr(k_new), _ptr(v_new), _ptr(kc), _ptr(vc), _ptr(out),
                                             n_head, n_kv, head_dim, n_ctx, _ptr(d_pos), scale,
                                             n_rot, theta, _ptr(freq_factors), 1 if neox else 0, _ptr(angles))
    if rc != 0:
        raise OrinFaError("flash_attention_decode_rope_store_ind", rc)


def rope_store_batch(q, k, v, kc, vc, batch, n_head, n_kv, head_dim, n_ctx, n_past, n_rot, theta, freq_factors=None,
                     neox=True):
    """rope_*_batch on the Q rows and on the K rows, then kv_store_batch, as one call (no counterpart in the reference)."""
    rc = lib().orin_fa_rope_store_batch(_ptr(q), _ptr(k), _ptr(v), _ptr(kc), _ptr(vc), batch, n_head, n_kv, head_dim,
                                        n_ctx, n_past, n_rot, theta, _ptr(freq_factors), 1 if neox else 0)
    if rc != 0:
        raise OrinFaError("rope_store_batch", rc)


def rope_angles_ind(angles, n_rot, theta, d_pos, freq_factors=None):
    """(cos, sin) of the n_rot/2 pairs at *d_pos into angles [n_rot/2][2] (no counterpart in the reference)."""
    rc = lib().orin_fa_rope_angles_ind(_ptr(angles), n_rot, theta, _ptr(freq_factors), _ptr(d_pos))
    if rc != 0:
        raise OrinFaError("rope_angles_ind", rc)


def rope_neox_batch(x, rows, head_dim, n_rot, theta, n_past, heads, freq_factors=None):
    rc = lib().orin_fa_rope_batch(_ptr(x), rows, head_dim, n_rot, theta, n_past, heads, _ptr(freq_factors), 1)
    if rc != 0:
        raise OrinFaError("rope_neox_batch", rc)


def rope_normal_batch(x, rows, head_dim, n_rot, theta, n_past, heads, freq_factors=None):
    rc = lib().orin_fa_rope_batch(_ptr(x), rows, head_dim, n_rot, theta, n_past, heads, _ptr(freq_factors), 0)
    if rc != 0:
        raise OrinFaError("rope_normal_batch", rc)


def rope_neox_ind(x, rows, head_dim, n_rot, theta, d_pos, freq_factors=None):
    rc = lib().orin_fa_rope_ind(_ptr(x), rows, head_dim, n_rot, theta, _ptr(d_pos), _ptr(freq_factors), 1)
    if rc != 0:
        raise OrinFaError("rope_neox_ind", rc)


def rope_normal_ind(x, rows, head_dim, n_rot, theta, d_pos, freq_factors=None):
    rc = lib().orin_fa_rope_ind(_ptr(x), rows, head_dim, n_rot, theta, _ptr(d_pos), _ptr(freq_factors), 0)
    if rc != 0:
        raise OrinFaError("rope_normal_ind", rc)


def kv_store_batch(kc, vc, k, v, heads, head_dim, n_ctx, pos_base, batch):
    rc = lib().orin_fa_kv_store_batch(_ptr(kc), _ptr(vc), _ptr(k), _ptr(v), heads, head_dim, n_ctx, pos_base, batch)
    if rc != 0:
        raise OrinFaError("kv_store_batch", rc)


def kv_store_ind(kc, vc, k, v, heads, head_dim, n_ctx, d_pos):
    rc = lib().orin_fa_kv_store_ind(_ptr(kc), _ptr(vc), _ptr(k), _ptr(v), heads, head_dim, n_ctx, _ptr(d_pos))
    if rc != 0:
        raise OrinFaError("kv_store_ind", rc)


def kv_shift(kc, vc, n_layer, n_kv, head_dim, n_ctx, n_keep, shift):
    rc = lib().orin_fa_kv_shift(_ptr(kc), _ptr(vc), n_layer, n_kv, head_dim, n_ctx, n_keep, shift)
    if rc != 0:
        raise OrinFaError("kv_shift", rc)


def decode_splits(n_head, n_kv, head_dim, n_ctx):
    return int(lib().orin_fa_decode_splits(n_head, n_kv, head_dim, n_ctx))


def cu_count():
    return int(lib().orin_fa_cu_count())


def bench_lib():
    """The measurement aids' own library (include/orin_fa_bench.h): read-only stand-ins and a do-nothing kernel."""
    global _bench_lib
    if _bench_lib is None:
        if not os.path.exists(BENCH_LIB_PATH):
            raise ImportError(f"{BENCH_LIB_PATH} is missing: build it with __graft_entry__.build()")
        L = ctypes.CDLL(BENCH_LIB_PATH)
        L.orin_fa_bench_hbm_read.argtypes = [_vp, ctypes.c_size_t, _int, _vp, _vp]
        L.orin_fa_bench_read_pattern.argtypes = [_vp, ctypes.c_size_t, _int, _int, _int, _int, _vp, _vp]
        L.orin_fa_bench_handoff.argtypes = [_vp, _int, _vp, _vp, _vp]
        L.orin_fa_bench_tiny_launch.argtypes = [_vp, _vp, _vp]
        for n in ("orin_fa_bench_hbm_read", "orin_fa_bench_read_pattern", "orin_fa_bench_handoff", "orin_fa_bench_tiny_launch"):
            getattr(L, n).restype = _int
        L.orin_fa_bench_handoff_scratch_bytes.argtypes = []
        L.orin_fa_bench_handoff_scratch_bytes.restype = ctypes.c_size_t
        L.orin_fa_bench_handoff_stream_bytes.argtypes = []
        L.orin_fa_bench_handoff_stream_bytes.restype = ctypes.c_size_t
        _bench_lib = L
    return _bench_lib


def _bench_check(what, rc):
    if rc != 0:
        raise RuntimeError(f"{what}: measurement aid returned {rc}")


def bench_hbm_read(src, nbytes, sink, loads_per_thread=16):
    """Measurement aid: one launch (on the stream of set_stream) of a plain streaming read of nbytes at src;
    sink: a device word."""
    _bench_check("bench_hbm_read", bench_lib().orin_fa_bench_hbm_read(_ptr(src), int(nbytes), int(loads_per_thread), _ptr(sink), _stream))


def bench_read_pattern(w, mat_bytes, n_rows, n_blocks, pattern, workgroups, sink):
    """Measurement aid: one launch of a read-only stand-in for a matrix-vector kernel's loads over a pair of Q4_K-shaped matrices."""
    _bench_check("bench_read_pattern", bench_lib().orin_fa_bench_read_pattern(_ptr(w), int(mat_bytes), int(n_rows), int(n_blocks),
                                                                              int(pattern), int(workgroups), _ptr(sink), _stream))


def bench_tiny_launch(src, sink):
    """Measurement aid: one launch of a one-wave kernel that reads the word at src."""
    _bench_check("bench_tiny_launch", bench_lib().orin_fa_bench_tiny_launch(_ptr(src), _ptr(sink), _stream))


def bench_handoff(src, fused, scratch, out):
    """Measurement aid: a stand-in for a split-KV decode step, partial results merged by a second
    kernel (fused=False) or inside the launch (fused=True)."""
    _bench_check("bench_handoff", bench_lib().orin_fa_bench_handoff(_ptr(src), int(fused), _ptr(scratch), _ptr(out), _stream))


def probe_lib(flags, prefill=False):
    """A cut-off build of the library (liborin_fa_probe_<flags>.so: the decode split kernel with parts taken
    out; liborin_fa_pprobe_<flags>.so: the prefill kernel; results wrong by design; see fa_decode.hip and
    fa_prefill.hip) as an independent ctypes handle.  A measurement aid of bench.py."""
    path = os.path.join(_HERE, f"liborin_fa_{'pprobe' if prefill else 'probe'}_{int(flags)}.so")
    if not os.path.exists(path):
        raise ImportError(f"{path} is missing: build the cut-off libraries with `python -m orin_llm_amd.build --probes`")
    L = ctypes.CDLL(path)
    L.orin_fa_init.argtypes = [_int]
    L.orin_fa_init.restype = _int
    L.orin_fa_set_stream.argtypes = [_vp]
    L.orin_fa_set_stream.restype = None
    L.orin_fa_decode_ind.argtypes = [_vp, _vp, _vp, _vp, _int, _int, _int, _int, _vp, _flt]
    L.orin_fa_decode_ind.restype = _int
    L.orin_fa_prefill.argtypes = [_vp, _vp, _vp, _vp, _int, _int, _int, _int, _int, _int, _flt]
    L.orin_fa_prefill.restype = _int
    return L


def stamps_lib():
    """The timeline build of the library (stage marks of the attention kernels store the wall clock), as a
    second, independent ctypes handle with its own state: init, set_stream, the two attention entry points
    and orin_fa_bench_stamps.  A measurement aid of bench.py."""
    global _stamps_lib
    if _stamps_lib is None:
        if not os.path.exists(STAMPS_LIB_PATH):
            raise ImportError(f"{STAMPS_LIB_PATH} is missing: build it with __graft_entry__.build()")
        L = ctypes.CDLL(STAMPS_LIB_PATH)
        L.orin_fa_init.argtypes = [_int]
        L.orin_fa_init.restype = _int
        L.orin_fa_set_stream.argtypes = [_vp]
        L.orin_fa_set_stream.restype = None
        L.orin_fa_prefill.argtypes = [_vp, _vp, _vp, _vp, _int, _int, _int, _int, _int, _int, _flt]
        L.orin_fa_prefill.restype = _int
        L.orin_fa_decode_ind.argtypes = [_vp, _vp, _vp, _vp, _int, _int, _int, _int, _vp, _flt]
        L.orin_fa_decode_ind.restype = _int
        L.orin_fa_decode_splits.argtypes = [_int, _int, _int, _int]
        L.orin_fa_decode_splits.restype = _int
        L.orin_fa_bench_stamps.argtypes = [_int, _vp, ctypes.c_size_t]
        L.orin_fa_bench_stamps.restype = _int
        _stamps_lib = L
    return _stamps_lib


def bench_handoff_sizes():
    return int(bench_lib().orin_fa_bench_handoff_stream_bytes()), int(bench_lib().orin_fa_bench_handoff_scratch_bytes())
