"""GPU parity of the decode-layer operators (include/orin_layer.h), called through the C ABI, against
the CPU oracle and against the logits of the unmodified reference CPU build.

Tolerances.  The products keep the activation in fp32 and decode the weights to the oracle's exact
values, so only the order of the fp32 sum differs: TOL_OP = 1e-4 on max |got - want| / max |want| per
output vector (measured: a few 1e-6), far inside the 2e-3 the attention path is held to.
dequant_row is bit-exact.  Whole models: TOL_OP * 50 against the oracle run with an fp16 cache (what
the GPU keeps), TOL_MODEL = 1e-2 on the same figure against the stored reference logits, whose
run kept K and V in fp32 (tests/test_oracle_layer.py prints what that alone moves).
"""
import os
import sys

import numpy as np
import pytest

from oracle import ref
from test_gpu_parity import _dev, fa  # noqa: F401  (fa: fixture)

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import layer_model as lm  # noqa: E402

pytestmark = pytest.mark.gpu
TOL_OP = 1e-4
TOL_MODEL = 1e-2
TYPES = [lm.F32, lm.F16, lm.Q8_0, lm.Q4_K, lm.Q5_K, lm.Q6_K]


@pytest.fixture(scope="module")
def ly(fa):
    from orin_llm_amd import layer
    return layer


def vec_err(got, want):
    return float(np.abs(np.asarray(got, np.float64) - want).max() / max(np.abs(want).max(), 1e-30))


def dev_bytes(raw, offset=0):
    """Device copy of a byte array at `offset` bytes past a 256-byte boundary."""
    import torch

    t = torch.zeros(raw.size + 256 + offset, dtype=torch.uint8, device="cuda")
    base = (-t.data_ptr()) % 256 + offset
    view = t[base:base + raw.size]
    view.copy_(torch.from_numpy(raw))
    return view


def out_buf(n, fill=12345.0, pad=4):
    import torch

    return torch.full((n + pad,), fill, dtype=torch.float32, device="cuda")


# rows that exercise every team shape of the vector-ALU kernel: (n_in, waves per row, slots per lane); on the
# matrix cores the same lengths are 1 ... 74 blocks per row, shared among four waves
SHAPES = [(256, 1, 1), (1536, 1, 1), (2048, 1, 1), (4096, 1, 2), (6144, 1, 3), (8960, 2, 3), (14336, 4, 2), (18944, 4, 3),
          (28672, 4, 4), (32768, 4, 4)]


@pytest.fixture(params=["matrix cores", "vector ALU"])
def unit(request, ly):
    ly.use_matrix_cores(request.param == "matrix cores")
    yield request.param
    ly.use_matrix_cores(True)


# (F32 and F16 rows are always on the vector ALU)
TYPE_UNITS = [(t, "vector ALU") for t in TYPES] + [(t, "matrix cores") for t in (lm.Q8_0, lm.Q4_K, lm.Q5_K, lm.Q6_K)]


@pytest.mark.parametrize("wtype,where", TYPE_UNITS)
@pytest.mark.parametrize("n_in,kw,slots", SHAPES)
def test_gemv_against_the_oracle(ly, wtype, where, n_in, kw, slots):
    import torch

    unit = where
    ly.use_matrix_cores(where == "matrix cores")
    n_out = 37 if n_in > 4096 else 131
    rs = lm.Stream(1000 + wtype * 31 + n_in)
    t = lm.make_tensor(rs, wtype, n_in, n_out)
    x = rs.sym(n_in, 1.0)
    want = ref.gemv(wtype, t[1], x, n_in, n_out).astype(np.float64)
    w = dev_bytes(t[1], offset=2 if wtype in (lm.Q8_0, lm.Q6_K) else 0)  # (the 2-byte-aligned types at an odd spot)
    dx, y = _dev(x), out_buf(n_out)
    ly.gemv(wtype, w, dx, y, n_in, n_out)
    torch.cuda.synchronize()
    got = y.cpu().numpy()
    assert (got[n_out:] == 12345.0).all(), "rows past n_out were written"
    e = vec_err(got[:n_out], want)
    ly.use_matrix_cores(True)
    print(f"gemv {lm.TYPE_NAME[wtype]} n_in {n_in} on the {unit}: err {e:.2e}", flush=True)
    assert e < TOL_OP


@pytest.mark.parametrize("where", ["matrix cores", "vector ALU"])
@pytest.mark.parametrize("wtype,n_in", [(lm.Q4_K, 28672), (lm.Q6_K, 29696), (lm.Q5_K, 32768), (lm.Q8_0, 32768)])
def test_rows_past_24576_elements(ly, wtype, n_in, where):
    """Rows longer than four waves cover at three slots a lane (the feed-forward width of a 70B-class model is
    28672), up to the staged activation's 32768: the accumulating down projection and the gate/up pair
    with the norm folded in, on either unit, and the next multiple of 256 refused."""
    import torch
    from orin_llm_amd.kernels import OrinFaError

    n_out = 48
    rs = lm.Stream(8800 + wtype + n_in)
    t, tu = lm.make_tensor(rs, wtype, n_in, n_out), lm.make_tensor(rs, wtype, n_in, n_out)
    x, y0 = rs.sym(n_in, 1.0), rs.sym(n_out, 2.0)
    nw = (1.0 + rs.sym(n_in, 0.3)).astype(np.float32)
    off = 2 if wtype in (lm.Q8_0, lm.Q6_K) else 0
    w, wu, dx = dev_bytes(t[1], offset=off), dev_bytes(tu[1], offset=off), _dev(x)
    ly.use_matrix_cores(where == "matrix cores")
    try:
        y = _dev(y0)
        ly.gemv_multi(wtype, [w], None, [y], [n_out], dx, None, 0.0, n_in, True)
        act = out_buf(n_out)
        ly.gemv_norm_gate_up_swiglu(wtype, w, wu, dx, _dev(nw), 1e-6, act, n_in, n_out)
        torch.cuda.synchronize()
        e_add = vec_err(y.cpu().numpy(), (y0 + ref.gemv(wtype, t[1], x, n_in, n_out)).astype(np.float64))
        xn = ref.rms_norm(x, nw, 1e-6)
        want = ref.swiglu(ref.gemv(wtype, t[1], xn, n_in, n_out), ref.gemv(wtype, tu[1], xn, n_in, n_out)).astype(np.float64)
        got = act.cpu().numpy()
        e_ffn = vec_err(got[:n_out], want)
        print(f"type {lm.TYPE_NAME[wtype]} n_in {n_in} on the {where}: += {e_add:.2e}, norm + gate/up {e_ffn:.2e}", flush=True)
        assert (got[n_out:] == 12345.0).all()
        assert e_add < TOL_OP and e_ffn < TOL_OP
        with pytest.raises(OrinFaError):
            ly.gemv(wtype, w, dx, out_buf(n_out), 32768 + 256, n_out)
    finally:
        ly.use_matrix_cores(True)


@pytest.mark.parametrize("wtype", [lm.Q4_K, lm.Q6_K, lm.F16])
def test_staged_products_bias_add_and_snapshot(ly, wtype):
    """quantize_activation + gemv_q8 / _bias / _add (reference call order, src/model_gpu.cu:262-286):
    the product sees the activation as it was when it was staged."""
    import torch

    n_in, n_out = 1536, 70
    rs = lm.Stream(2000 + wtype)
    t = lm.make_tensor(rs, wtype, n_in, n_out)
    x, bias, y0 = rs.sym(n_in, 1.0), rs.sym(n_out, 0.5), rs.sym(n_out, 2.0)
    base = ref.gemv(wtype, t[1], x, n_in, n_out)
    w, dx = dev_bytes(t[1]), _dev(x)
    ly.quantize_activation(dx, n_in)
    dx.fill_(7.0)  # after staging: must not reach the products
    y = out_buf(n_out)
    ly.gemv_q8(wtype, w, y, n_in, n_out)
    yb = out_buf(n_out)
    ly.gemv_q8_bias(wtype, w, _dev(bias), yb, n_in, n_out)
    ya = _dev(np.concatenate([y0, np.full(4, 12345.0, np.float32)]))
    ly.gemv_q8_add(wtype, w, ya, n_in, n_out)
    torch.cuda.synchronize()
    assert vec_err(y.cpu().numpy()[:n_out], base.astype(np.float64)) < TOL_OP
    assert vec_err(yb.cpu().numpy()[:n_out], (base + bias).astype(np.float64)) < TOL_OP
    assert vec_err(ya.cpu().numpy()[:n_out], (y0 + base).astype(np.float64)) < TOL_OP
    assert (ya.cpu().numpy()[n_out:] == 12345.0).all() and (yb.cpu().numpy()[n_out:] == 12345.0).all()
    # a shorter product reads the first elements of what was staged, as the reference's do (its decode_layer stages
    # n_embd elements ahead of the output projection, whose rows have n_head * head_dim: src/model_gpu.cu:284-285) ...
    n_short = n_in // 2 if wtype == lm.F16 else 1280
    rb, rb_short = ref.row_bytes(wtype, n_in), ref.row_bytes(wtype, n_short)
    t_short = np.concatenate([t[1][r * rb:r * rb + rb_short] for r in range(n_out)])
    ys = out_buf(n_out)
    ly.gemv_q8(wtype, dev_bytes(t_short), ys, n_short, n_out)
    torch.cuda.synchronize()
    assert vec_err(ys.cpu().numpy()[:n_out], ref.gemv(wtype, t_short, x[:n_short], n_short, n_out).astype(np.float64)) < TOL_OP
    # ... and a longer one, which would read what nobody staged, is refused
    from orin_llm_amd.kernels import OrinFaError
    ly.quantize_activation(dx, n_short)
    with pytest.raises(OrinFaError):
        ly.gemv_q8(wtype, w, y, n_in, n_out)


@pytest.mark.parametrize("wtype,n_in,n_out", [(lm.Q4_K, 4096, 1536), (lm.Q6_K, 8960, 1536), (lm.Q6_K, 14336, 4096)])
def test_accumulating_projection_is_bit_stable_with_one_share(ly, wtype, n_in, n_out):
    """y += W x over long rows of a matrix with few rows (the output and down projections): by default a row is cut
    into shares that meet by atomic adds in no fixed order, so repeated runs agree to the order of an fp32 sum only;
    with orin_gemv_row_shares(1) every run gives the same bits (the reference's gemv_q8_add is a plain sum,
    src/kernels.cu:350-374)."""
    import torch

    rs = lm.Stream(7000 + wtype + n_in)
    t = lm.make_tensor(rs, wtype, n_in, n_out)
    x, y0 = rs.sym(n_in, 1.0), rs.sym(n_out, 2.0)
    want = (y0 + ref.gemv(wtype, t[1], x, n_in, n_out)).astype(np.float64)
    w, dx = dev_bytes(t[1], offset=2 if wtype == lm.Q6_K else 0), _dev(x)

    def runs(n):
        out = []
        for _ in range(n):
            y = _dev(y0)
            ly.gemv_multi(wtype, [w], None, [y], [n_out], dx, None, 0.0, n_in, True)
            torch.cuda.synchronize()
            out.append(y.cpu().numpy())
        return out

    try:
        ly.gemv_row_shares(0)
        shared = runs(20)
        ly.gemv_row_shares(1)
        single = runs(20)
    finally:
        ly.gemv_row_shares(0)
    for y in shared + single:
        assert vec_err(y, want) < TOL_OP
    assert all(np.array_equal(single[0].view(np.uint32), y.view(np.uint32)) for y in single[1:])
    spread = max(float(np.abs(y.astype(np.float64) - shared[0]).max() / np.abs(want).max()) for y in shared[1:])
    print(f"type {wtype} {n_in} x {n_out}: spread over 20 runs with shares {spread:.1e}", flush=True)
    assert spread < 1e-6   # (a few units in the last place of the largest element)


@pytest.mark.parametrize("wtype", [lm.Q4_K, lm.Q6_K, lm.Q8_0])
@pytest.mark.parametrize("bad", [float("nan"), float("inf"), float("-inf")])
def test_a_non_finite_activation_is_not_laundered(ly, wtype, bad):
    """An infinity or a NaN in the activation makes every row's sum non-finite on the matrix cores as on the vector
    ALU (the int8 digits of the matrix-core path cannot carry it: its sub-block's scale does)."""
    import torch

    n_in, n_out = 1536, 48
    rs = lm.Stream(8100 + wtype)
    t = lm.make_tensor(rs, wtype, n_in, n_out)
    x = rs.sym(n_in, 1.0)
    x[777] = bad
    w = dev_bytes(t[1], offset=2 if wtype in (lm.Q6_K, lm.Q8_0) else 0)
    got = {}
    for unit in (1, 0):
        ly.use_matrix_cores(unit)
        try:
            y = out_buf(n_out)
            ly.gemv(wtype, w, _dev(x), y, n_in, n_out)
            torch.cuda.synchronize()
            got[unit] = y.cpu().numpy()[:n_out]
        finally:
            ly.use_matrix_cores(1)
    assert not np.isfinite(got[1]).any() and not np.isfinite(got[0]).any()
    # the same rows over a finite activation stay finite (the flag is per sub-block and per launch)
    x[777] = 0.5
    y = out_buf(n_out)
    ly.gemv(wtype, w, _dev(x), y, n_in, n_out)
    torch.cuda.synchronize()
    assert vec_err(y.cpu().numpy()[:n_out], ref.gemv(wtype, t[1], x, n_in, n_out).astype(np.float64)) < TOL_OP


def test_q8_0_rows_that_are_not_whole_256s_stay_on_the_vector_alu(ly):
    """Q8_0 blocks are 32 elements: a row of 1568 is legal and does not fit the matrix-core kernel's 256-element steps."""
    import torch

    n_in, n_out = 1568, 50
    rs = lm.Stream(1234)
    t = lm.make_tensor(rs, lm.Q8_0, n_in, n_out)
    x = rs.sym(n_in, 1.0)
    y = out_buf(n_out)
    ly.gemv(lm.Q8_0, dev_bytes(t[1], offset=2), _dev(x), y, n_in, n_out)
    torch.cuda.synchronize()
    assert vec_err(y.cpu().numpy()[:n_out], ref.gemv(lm.Q8_0, t[1], x, n_in, n_out).astype(np.float64)) < TOL_OP


@pytest.mark.parametrize("wtype", [lm.Q8_0, lm.Q4_K, lm.Q5_K, lm.Q6_K])
@pytest.mark.parametrize("n_in", [1536, 8960])
def test_gate_up_swiglu_staged_and_with_the_norm_folded_in(ly, unit, wtype, n_in):
    import torch

    n_out = 90
    rs = lm.Stream(3000 + wtype + n_in)
    g, u = lm.make_tensor(rs, wtype, n_in, n_out), lm.make_tensor(rs, wtype, n_in, n_out)
    x, nw = rs.sym(n_in, 2.0), (1.0 + rs.sym(n_in, 0.3)).astype(np.float32)
    wg, wu = dev_bytes(g[1]), dev_bytes(u[1])
    # staged, as the reference calls it
    want = ref.swiglu(ref.gemv(wtype, g[1], x, n_in, n_out), ref.gemv(wtype, u[1], x, n_in, n_out)).astype(np.float64)
    out = out_buf(n_out)
    ly.quantize_activation(_dev(x), n_in)
    ly.gemv_fused_gate_up_swiglu(wtype, wg, wu, out, n_in, n_out)
    # with the norm in the same launch
    xn = ref.rms_norm(x, nw, 1e-6)
    want_n = ref.swiglu(ref.gemv(wtype, g[1], xn, n_in, n_out), ref.gemv(wtype, u[1], xn, n_in, n_out)).astype(np.float64)
    out_n = out_buf(n_out)
    ly.gemv_norm_gate_up_swiglu(wtype, wg, wu, _dev(x), _dev(nw), 1e-6, out_n, n_in, n_out)
    torch.cuda.synchronize()
    e, en = vec_err(out.cpu().numpy()[:n_out], want), vec_err(out_n.cpu().numpy()[:n_out], want_n)
    print(f"gate/up {lm.TYPE_NAME[wtype]} n_in {n_in}: err {e:.2e}, with norm {en:.2e}", flush=True)
    assert e < TOL_OP and en < TOL_OP
    assert (out.cpu().numpy()[n_out:] == 12345.0).all() and (out_n.cpu().numpy()[n_out:] == 12345.0).all()


@pytest.mark.parametrize("wtype", [lm.Q4_K, lm.Q6_K])
def test_three_projections_in_one_launch(ly, unit, wtype):
    """q, k, v of different heights over one normalised activation, with biases; and accumulated."""
    import torch

    n_in, n_outs = 1536, [1536, 256, 200]
    rs = lm.Stream(4000 + wtype)
    ts = [lm.make_tensor(rs, wtype, n_in, n) for n in n_outs]
    bs = [rs.sym(n, 0.5) for n in n_outs]
    x, nw = rs.sym(n_in, 3.0), (1.0 + rs.sym(n_in, 0.3)).astype(np.float32)
    xn = ref.rms_norm(x, nw, 1e-5)
    want = [ref.gemv(wtype, t[1], xn, n_in, n) + b for t, b, n in zip(ts, bs, n_outs)]
    ws, dbs, ys = [dev_bytes(t[1]) for t in ts], [_dev(b) for b in bs], [out_buf(n) for n in n_outs]
    ly.gemv_multi(wtype, ws, dbs, ys, n_outs, _dev(x), _dev(nw), 1e-5, n_in)
    torch.cuda.synchronize()
    for y, w_, n in zip(ys, want, n_outs):
        got = y.cpu().numpy()
        assert vec_err(got[:n], w_.astype(np.float64)) < TOL_OP and (got[n:] == 12345.0).all()
    ly.gemv_multi(wtype, ws[:2], None, ys[:2], n_outs[:2], _dev(x), None, 0.0, n_in, accumulate=True)
    torch.cuda.synchronize()
    for y, w_, t, n in zip(ys[:2], want[:2], ts[:2], n_outs[:2]):
        assert vec_err(y.cpu().numpy()[:n], (w_ + ref.gemv(wtype, t[1], x, n_in, n)).astype(np.float64)) < TOL_OP


@pytest.mark.parametrize("wtypes", [(lm.Q4_K, lm.Q4_K, lm.Q6_K), (lm.Q6_K, lm.Q4_K, lm.Q6_K), (lm.Q4_K, lm.Q5_K, lm.Q6_K), (lm.Q8_0, lm.F16)])
@pytest.mark.parametrize("n_in", [256, 1536, 4096])
@pytest.mark.parametrize("heights", [(520, 130, 96), (512, 128, 96), (4096, 1024, 1024)])
def test_projections_of_different_types(ly, unit, wtypes, n_in, heights):
    """One launch where every type is a block type and the matrix cores are in use, one per matrix otherwise; same
    results either way.  (Heights that are whole 16-row tiles go to the kernel that reads rows in long runs.)"""
    import torch

    n_outs = list(heights)[:len(wtypes)]
    rs = lm.Stream(4500 + sum(wtypes) + n_in)
    ts = [lm.make_tensor(rs, t, n_in, n) for t, n in zip(wtypes, n_outs)]
    bs = [rs.sym(n, 0.5) for n in n_outs]
    x, nw = rs.sym(n_in, 3.0), (1.0 + rs.sym(n_in, 0.3)).astype(np.float32)
    xn = ref.rms_norm(x, nw, 1e-6)
    want = [ref.gemv(t[0], t[1], xn, n_in, n) + b for t, b, n in zip(ts, bs, n_outs)]
    ws = [dev_bytes(t[1], offset=2 if t[0] in (lm.Q8_0, lm.Q6_K) else 0) for t in ts]
    ys = [out_buf(n) for n in n_outs]
    ly.gemv_multi_types(list(wtypes), ws, [_dev(b) for b in bs], ys, n_outs, _dev(x), _dev(nw), 1e-6, n_in)
    torch.cuda.synchronize()
    for y, w_, n in zip(ys, want, n_outs):
        got = y.cpu().numpy()
        assert vec_err(got[:n], w_.astype(np.float64)) < TOL_OP and (got[n:] == 12345.0).all()


# Q4_K / Q5_K / Q6_K matrices made of whole 16-row tiles go to the kernel that reads rows in long runs: 1 ... 74 blocks
# per row (one or two blocks per item, chunks shared among four or eight waves, ragged last chunks), few and many
# tiles (one per workgroup, several per workgroup), every epilogue.
LONG_RUN_SHAPES = [(256, 48), (512, 16), (1536, 12800), (1792, 64), (3584, 512), (4096, 4096), (8960, 96), (14336, 256), (18944, 32)]


@pytest.mark.parametrize("wtype", [lm.Q4_K, lm.Q5_K, lm.Q6_K])
@pytest.mark.parametrize("n_in,n_out", LONG_RUN_SHAPES)
def test_whole_tiles_in_long_runs(ly, wtype, n_in, n_out):
    import torch

    ly.use_matrix_cores(True)
    rs = lm.Stream(7000 + wtype * 131 + n_in + n_out)
    t = lm.make_tensor(rs, wtype, n_in, n_out)
    x = rs.sym(n_in, 1.0)
    nw = (1.0 + rs.sym(n_in, 0.3)).astype(np.float32)
    bias, y0 = rs.sym(n_out, 0.5), rs.sym(n_out, 1.0)
    odd = 2 if wtype == lm.Q6_K else 0   # (the 2-byte-aligned type at an odd spot)
    w, dx = dev_bytes(t[1], offset=odd), _dev(x)
    plain = ref.gemv(wtype, t[1], x, n_in, n_out).astype(np.float64)
    normed = ref.gemv(wtype, t[1], ref.rms_norm(x, nw, 1e-5), n_in, n_out).astype(np.float64)
    errs = {}
    y = out_buf(n_out)
    ly.gemv(wtype, w, dx, y, n_in, n_out)
    errs["plain"] = (y, plain)
    yb = out_buf(n_out)
    ly.gemv_multi(wtype, [w], [_dev(bias)], [yb], [n_out], dx, _dev(nw), 1e-5, n_in)
    errs["norm + bias"] = (yb, normed + bias)
    ya = _dev(np.concatenate([y0, np.full(4, 12345.0, np.float32)]))
    ly.gemv_multi(wtype, [w], None, [ya], [n_out], dx, None, 0.0, n_in, True)   # (few tiles and long rows: shares of a row)
    errs["accumulate"] = (ya, plain + y0)
    if n_out <= 4096:
        up = lm.make_tensor(rs, wtype, n_in, n_out)
        yg = out_buf(n_out)
        ly.gemv_norm_gate_up_swiglu(wtype, w, dev_bytes(up[1], offset=odd), dx, _dev(nw), 1e-5, yg, n_in, n_out)
        u = ref.gemv(wtype, up[1], ref.rms_norm(x, nw, 1e-5), n_in, n_out)
        errs["gate/up"] = (yg, ref.swiglu(normed.astype(np.float32), u).astype(np.float64))
    torch.cuda.synchronize()
    for what, (got_t, want) in errs.items():
        got = got_t.cpu().numpy()
        assert (got[n_out:] == 12345.0).all(), f"{what}: rows past n_out were written"
        e = vec_err(got[:n_out], want)
        print(f"{lm.TYPE_NAME[wtype]} {n_in} x {n_out} {what}: err {e:.2e}", flush=True)
        assert e < TOL_OP, what


def test_rms_norm_rows_swiglu_and_in_place(ly):
    import torch

    rs = lm.Stream(5000)
    for rows, cols in ((1, 1536), (1, 8960), (12, 128), (7, 64), (3, 100)):
        x, w = rs.sym(rows * cols, 4.0), (1.0 + rs.sym(cols, 0.3)).astype(np.float32)
        want = np.concatenate([ref.rms_norm(x[r * cols:(r + 1) * cols], w, 1e-6) for r in range(rows)]).astype(np.float64)
        dx, y = _dev(x), out_buf(rows * cols)
        ly.rms_norm_rows(dx, _dev(w), rows, cols, 1e-6, y)
        ly.rms_norm_rows(dx, _dev(w), rows, cols, 1e-6, dx)  # in place, as the per-head q/k norms run
        torch.cuda.synchronize()
        got = y.cpu().numpy()
        assert vec_err(got[:rows * cols], want) < 1e-6 and (got[rows * cols:] == 12345.0).all()
        assert np.array_equal(dx.cpu().numpy(), got[:rows * cols])
    g, u = rs.sym(1000, 8.0), rs.sym(1000, 2.0)
    act = out_buf(1000)
    ly.swiglu(act, _dev(g), _dev(u), 1000)
    torch.cuda.synchronize()
    assert vec_err(act.cpu().numpy()[:1000], ref.swiglu(g, u).astype(np.float64)) < 1e-6


@pytest.mark.parametrize("wtype", TYPES)
def test_dequant_row_bit_exact(ly, wtype):
    import torch

    n = 1536
    t = lm.make_tensor(lm.Stream(6000 + wtype), wtype, n, 4, std=1.0)
    rb = ref.row_bytes(wtype, n)
    w = dev_bytes(t[1])
    for r in (0, 3):
        y = out_buf(n)
        ly.dequant_row(wtype, w[r * rb:], y, n)
        torch.cuda.synchronize()
        got = y.cpu().numpy()
        want = ref.dequantize_row(wtype, t[1][r * rb:(r + 1) * rb], n)
        assert np.array_equal(got[:n].view(np.uint32), want.view(np.uint32)) and (got[n:] == 12345.0).all()


def test_rejects_bad_arguments(ly):
    import torch

    from orin_llm_amd.kernels import OrinFaError

    w = dev_bytes(np.zeros(144 * 8, np.uint8))
    x, y = out_buf(512), out_buf(8)
    for call in (lambda: ly.gemv(lm.Q4_K, w, x, y, 300, 2),            # not whole blocks
                 lambda: ly.gemv(7, w, x, y, 256, 2),                  # unknown type
                 lambda: ly.gemv(lm.Q4_K, w[4:], x, y, 256, 2),        # misaligned matrix
                 lambda: ly.gemv(lm.Q4_K, w, x[1:], y, 256, 2),        # misaligned activation
                 lambda: ly.gemv(lm.Q4_K, w, x, y.view(torch.uint8)[2:10].view(torch.int16), 256, 2),  # output not on a float boundary
                 lambda: ly.gemv(lm.F16, w, x, y, 32768 + 32, 1),      # longer than a workgroup covers
                 lambda: ly.gemv(lm.Q4_K, None, x, y, 256, 2),
                 lambda: ly.quantize_activation(x, 40000)):
        with pytest.raises(OrinFaError):
            call()


def test_decode_layer_rejects_what_it_cannot_run(ly):
    """Missing buffers, and gate/up of different types without the scratch vector for the up product."""
    import torch

    from orin_llm_amd.kernels import OrinFaError

    model = lm.build("qwen2")   # layer 0: ffn_gate Q4_K, ffn_up Q5_K
    hp, layers, _ = upload(model)
    bufs = make_bufs(hp)
    kc = torch.zeros((hp["n_kv"], 32, hp["head_dim"]), dtype=torch.int16, device="cuda")
    vc, d_pos = torch.zeros_like(kc), torch.zeros(1, dtype=torch.int32, device="cuda")
    bufs["x"].copy_(_dev(np.linspace(-1.0, 1.0, hp["n_embd"], dtype=np.float32)))
    x_before = bufs["x"].clone()
    for drop in ("x", "attn", "act", "up_tmp"):
        b = dict(bufs)
        b[drop] = None
        with pytest.raises(OrinFaError):
            ly.decode_layer(ly.make_desc(hp, layers[0], b, kc, vc, d_pos, 32))
    with pytest.raises(OrinFaError):
        ly.decode_layer(ly.make_desc(hp, layers[0], bufs, kc, vc, None, 32))
    with pytest.raises(OrinFaError):
        ly.decode_layer(ly.make_desc(hp, layers[0], bufs, kc, None, d_pos, 32))
    no_down = dict(layers[0])
    no_down["ffn_down"] = (lm.Q6_K, None)
    with pytest.raises(OrinFaError):
        ly.decode_layer(ly.make_desc(hp, no_down, bufs, kc, vc, d_pos, 32))
    desc = ly.make_desc(hp, layers[0], bufs, kc, vc, d_pos, 32)
    desc.n_ff = 0
    with pytest.raises(OrinFaError):
        ly.decode_layer(desc)
    torch.cuda.synchronize()
    assert torch.equal(bufs["x"], x_before)   # every one of them is refused before anything is launched


# ---------------------------------------------------------------- whole models

def upload(model):
    """Device copies: per layer {name: (type, bytes) or fp32 tensor}."""
    hp = dict(model["hp"])
    hp["freq_factors_dev"] = _dev(hp["freq_factors"]) if hp["freq_factors"] is not None else None
    layers = []
    for L in model["layers"]:
        D = {}
        for k, v in L.items():
            D[k] = (v[0], dev_bytes(v[1], offset=2 if v[0] in (lm.Q8_0, lm.Q6_K) else 0)) if isinstance(v, tuple) else _dev(v)
        layers.append(D)
    top = dict(token_embd=(model["token_embd"][0], dev_bytes(model["token_embd"][1])),
               output=(model["output"][0], dev_bytes(model["output"][1])), output_norm=_dev(model["output_norm"]))
    return hp, layers, top


def make_bufs(hp):
    import torch

    z = lambda n: torch.zeros(n, dtype=torch.float32, device="cuda")  # noqa: E731
    nq, nkv = hp["n_head"] * hp["head_dim"], hp["n_kv"] * hp["head_dim"]
    # (attn as large as the reference's: its decode_layer stages n_embd elements of it, src/model_gpu.cu:284)
    return dict(x=z(hp["n_embd"]), xn=z(hp["n_embd"]), xn2=z(hp["n_embd"]), q=z(nq), k=z(nkv), v=z(nkv), attn=z(max(nq, hp["n_embd"])),
                act=z(hp["n_ff"]), up_tmp=z(hp["n_ff"]), logits=z(hp["n_vocab"]))


@pytest.mark.parametrize("name", list(lm.VARIANTS))
@pytest.mark.parametrize("how", ["calls", "fused", "fused_graph"])
def test_whole_model_against_reference_logits(fa, ly, name, how):
    """Token t at position t through embedding row, every layer, the last norm and the output matrix:
    `calls` issues the reference's own sequence of operator calls (src/model_gpu.cu:251-293, 303-306),
    `fused` the library's one call per layer, `fused_graph` captures that step once and replays it with
    the token's embedding row and the position updated in place, as the reference's graph is replayed
    (src/model_gpu.cu:318-344)."""
    import torch

    golden = np.load(os.path.join(HERE, "golden", "layer_reference.npz"))
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
    descs = [ly.make_desc(hp, layers[l], bufs, kc[l], vc[l], d_pos, n_ctx) for l in range(nl)]

    def step():
        ly.dequant_row(et, emb_row, bufs["x"], ne)
        for l in range(nl):
            if how == "calls":
                ly.decode_layer_calls(hp, layers[l], bufs, kc[l], vc[l], d_pos, n_ctx)
            else:
                ly.decode_layer(descs[l])
        ly.rms_norm(bufs["x"], top["output_norm"], ne, hp["rms_eps"], bufs["xn"])
        ly.gemv(top["output"][0], top["output"][1], bufs["xn"], bufs["logits"], ne, nv)

    graph = None
    stream = torch.cuda.Stream()
    oracle_state = ref.RefState(model, n_ctx, fp16_cache=True)
    worst_o = worst_g = 0.0
    for t in range(n_tok):
        emb_row.copy_(eraw[t * rb:(t + 1) * rb])
        d_pos.fill_(t)
        torch.cuda.synchronize()
        if how == "fused_graph":
            if graph is None:
                fa.set_stream(stream.cuda_stream)
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=stream):
                    step()
                fa.set_stream(torch.cuda.current_stream().cuda_stream)
            graph.replay()
        else:
            step()
        torch.cuda.synchronize()
        got = bufs["logits"].cpu().numpy()
        want_o = ref.decode_forward(model, oracle_state, t, t).astype(np.float64)
        worst_o = max(worst_o, vec_err(got, want_o))
        worst_g = max(worst_g, vec_err(got, golden["logits_" + name][t].astype(np.float64)))
    print(f"{name} {how}: vs oracle (fp16 cache) {worst_o:.2e}, vs reference logits (fp32 cache) {worst_g:.2e}", flush=True)
    assert worst_o < TOL_OP * 50 and worst_g < TOL_MODEL
