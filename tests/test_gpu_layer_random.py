"""A seeded sweep of matrix-vector products nobody picked by hand: weight type, row length (whole 256s up to
24576, and for Q8_0 / F16 / F32 also lengths that are only whole 32s), row count, bias, accumulation, the norm
folded in, a gate/up pair, one to three matrices per launch, on the matrix cores and on the vector ALU --
against the CPU oracle's sequential fp32 products.  Tolerance as in test_gpu_layer.py (1e-4 of the output
vector's largest element; measured a few 1e-6).
"""
import os
import sys

import numpy as np
import pytest

from oracle import ref
from test_gpu_layer import TOL_OP, dev_bytes, ly, out_buf, vec_err  # noqa: F401  (ly: fixture)
from test_gpu_parity import _dev, fa  # noqa: F401  (fa: fixture)

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import layer_model as lm  # noqa: E402

pytestmark = pytest.mark.gpu
BLOCK_TYPES = (lm.Q8_0, lm.Q4_K, lm.Q5_K, lm.Q6_K)


def draw(seed, whole_tiles=False):
    """whole_tiles: heights that are whole 16-row tiles of a K-quant type on the matrix cores, i.e. the kernel that
    reads rows in long runs (the other draws mostly miss it)."""
    rng = np.random.default_rng(seed)
    wtype = int(rng.choice([lm.F32, lm.F16, lm.Q8_0, lm.Q4_K, lm.Q5_K, lm.Q6_K], p=[0.05, 0.1, 0.15, 0.3, 0.15, 0.25]))
    if wtype in (lm.F32, lm.F16, lm.Q8_0) and rng.random() < 0.4:
        n_in = 32 * int(rng.integers(1, 300))           # whole 32s only: the vector-ALU kernel
    else:
        n_in = 256 * int(rng.choice([1, 2, 3, 5, 6, 7, 8, 11, 14, 16, 24, 35, 37, 56, 74, 96], p=None))
    kind = str(rng.choice(["plain", "bias", "accumulate", "norm", "gate_up", "norm_gate_up", "multi"]))
    n_mat = int(rng.integers(2, 4)) if kind == "multi" else 1
    n_outs = [int(rng.integers(1, 140)) for _ in range(n_mat)]
    mfma = bool(rng.random() < 0.6)
    if whole_tiles:
        wtype = int(rng.choice([lm.Q4_K, lm.Q5_K, lm.Q6_K]))
        n_in = 256 * int(rng.choice([1, 2, 3, 5, 6, 7, 8, 11, 14, 16, 24, 35, 37, 56, 74]))
        n_outs = [16 * int(rng.choice([1, 2, 3, 7, 16, 40, 97])) for _ in range(n_mat)]
        mfma = True
    return dict(wtype=wtype, n_in=n_in, kind=kind, n_outs=n_outs, mfma=mfma, seed=seed)


@pytest.mark.parametrize("seed", list(range(7000, 7070)) + list(range(7100, 7150)))
def test_random_product(ly, seed):
    import torch

    c = draw(seed, whole_tiles=seed >= 7100)
    wtype, n_in, kind, n_outs = c["wtype"], c["n_in"], c["kind"], c["n_outs"]
    print(c, flush=True)
    rs = lm.Stream(seed)
    off = 2 if wtype in (lm.Q8_0, lm.Q6_K) else 0
    ts = [lm.make_tensor(rs, wtype, n_in, n) for n in n_outs]
    x = rs.sym(n_in, 2.0)
    nw = (1.0 + rs.sym(n_in, 0.3)).astype(np.float32)
    ly.use_matrix_cores(c["mfma"])
    try:
        ws = [dev_bytes(t[1], offset=off) for t in ts]
        ys = [out_buf(n) for n in n_outs]
        mv = lambda t, v: ref.gemv(wtype, t[1], v, n_in, t[3])  # noqa: E731
        if kind in ("plain", "bias", "accumulate"):
            bias = rs.sym(n_outs[0], 0.5) if kind == "bias" else None
            y0 = rs.sym(n_outs[0], 1.0)
            ys[0][:n_outs[0]].copy_(torch.from_numpy(y0))
            ly.gemv_multi(wtype, ws, [_dev(bias)] if bias is not None else None, ys, n_outs, _dev(x), None, 0.0, n_in,
                          accumulate=kind == "accumulate")
            want = [mv(ts[0], x) + (bias if bias is not None else 0.0) + (y0 if kind == "accumulate" else 0.0)]
        elif kind == "norm":
            ly.gemv_multi(wtype, ws, None, ys, n_outs, _dev(x), _dev(nw), 1e-6, n_in)
            want = [mv(ts[0], ref.rms_norm(x, nw, 1e-6))]
        elif kind in ("gate_up", "norm_gate_up"):
            up = lm.make_tensor(rs, wtype, n_in, n_outs[0])
            xin = ref.rms_norm(x, nw, 1e-6) if kind == "norm_gate_up" else x
            ly.gemv_norm_gate_up_swiglu(wtype, ws[0], dev_bytes(up[1], offset=off), _dev(x), _dev(nw) if kind == "norm_gate_up" else None,
                                        1e-6, ys[0], n_in, n_outs[0])
            want = [ref.swiglu(mv(ts[0], xin), mv(up, xin))]
        else:
            bs = [rs.sym(n, 0.5) for n in n_outs]
            ly.gemv_multi(wtype, ws, [_dev(b) for b in bs], ys, n_outs, _dev(x), _dev(nw), 1e-5, n_in)
            xn = ref.rms_norm(x, nw, 1e-5)
            want = [mv(t, xn) + b for t, b in zip(ts, bs)]
        torch.cuda.synchronize()
    finally:
        ly.use_matrix_cores(True)
    for y, w_, n in zip(ys, want, n_outs):
        got = y.cpu().numpy()
        assert (got[n:] == 12345.0).all(), "rows past n_out were written"
        assert vec_err(got[:n], np.asarray(w_, np.float64)) < TOL_OP, c
