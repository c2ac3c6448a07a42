"""Properties of attention that do not depend on the size, checked at the benchmark's full sizes.

The oracle checks sampled rows there (test_gpu_parity.py); these tests cover every output row
with facts that need no second implementation: a constant V gives that constant back, a
prefill row is the decode of the same position, a chunk may be cut anywhere, the order of the
visible cache rows does not matter to a decode, rows past the position are never used, and
the operator is linear in V.  Tolerances: TOL on the row figure; where both sides are decodes
(fp32-accurate) a hundredth of it; the floor figure's bound counts the prefill results compared.
"""
import numpy as np
import pytest

from test_gpu_parity import _dev, check, fa, gpu_decode, gpu_prefill  # noqa: F401  (fa: fixture)
from util import FLOOR_DECODE, FLOOR_PREFILL, TOL, make_case

pytestmark = pytest.mark.gpu

SCALE = 1.0 / np.sqrt(128.0)
# (name, H, G, n_ctx, n_past, batch): the 512-token chunks the benchmark times
PREFILL = [
    ("llama8b-d4096", 32, 8, 8192, 4096, 512),
    ("qwen1.5b-d3584", 12, 2, 4096, 3584, 512),
    ("qwen7b-d32256", 28, 4, 32768, 32256, 512),   # ends exactly at n_ctx
    ("qwen1.5b-d32256", 12, 2, 32768, 32256, 512), # KV rows split among workgroups + combine kernel
]
# (name, H, G, n_ctx, L): the decode steps the benchmark times
DECODE = [
    ("qwen1.5b-32k", 12, 2, 32768, 32768),
    ("qwen7b-32k", 28, 4, 32768, 32767),
    ("llama8b-8k", 32, 8, 8192, 8192),
]


def _const_v(vc, n_filled, values):
    """V rows [0, n_filled) of KV head g all equal to the vector values[g] (fp16 bit patterns)."""
    vb = np.asarray(values, np.float16).view(np.uint16)  # [G][d]
    vc = vc.copy()
    vc[:, :n_filled] = vb[:, None, :]
    return vc


@pytest.mark.parametrize("name,H,G,n_ctx,n_past,batch", PREFILL)
def test_prefill_constant_v_returns_the_constant(fa, name, H, G, n_ctx, n_past, batch):
    """Softmax weights sum to one: with every visible V row of a KV head equal to c, every
    output row of its heads is c, whatever Q and K are.  A dropped or doubled tile, a wrong
    row sum or a wrong merge of the waves' or splits' partial results shows up here."""
    d = 128
    q, kc, vc = make_case(301, H, G, d, n_ctx, n_past + batch, batch, outliers=4)
    c = np.random.default_rng(302).standard_normal((G, d)).astype(np.float16)
    got = gpu_prefill(fa, q, kc, _const_v(vc, n_past + batch, c), H, G, d, n_ctx, n_past, batch, SCALE)
    want = np.broadcast_to(np.repeat(c.astype(np.float32), H // G, axis=0)[None], got.shape)
    check(got, want, f"{name} constant V")


@pytest.mark.parametrize("name,H,G,n_ctx,L", DECODE)
def test_decode_constant_v_returns_the_constant(fa, name, H, G, n_ctx, L):
    d = 128
    q, kc, vc = make_case(311, H, G, d, n_ctx, L, 1, outliers=4)
    c = np.random.default_rng(312).standard_normal((G, d)).astype(np.float16)
    got = gpu_decode(fa, q[0], kc, _const_v(vc, L, c), H, G, d, n_ctx, L - 1, SCALE)
    check(got, np.repeat(c.astype(np.float32), H // G, axis=0), f"{name} constant V", tol=TOL / 100, floor=FLOOR_DECODE)


@pytest.mark.parametrize("name,H,G,n_ctx,n_past,batch", PREFILL[:3])
def test_prefill_rows_equal_decode_and_chunk_cut(fa, name, H, G, n_ctx, n_past, batch):
    """Row t of a chunk at depth P is the decode at position P + t, and a chunk cut in two
    gives the rows of the whole (the two halves fall into different token tiles and walks)."""
    d = 128
    q, kc, vc = make_case(321, H, G, d, n_ctx, n_past + batch, batch, outliers=4, poison_tail=True)
    whole = gpu_prefill(fa, q, kc, vc, H, G, d, n_ctx, n_past, batch, SCALE)
    cut = 203
    a = gpu_prefill(fa, q[:cut], kc, vc, H, G, d, n_ctx, n_past, cut, SCALE)
    b = gpu_prefill(fa, q[cut:], kc, vc, H, G, d, n_ctx, n_past + cut, batch - cut, SCALE)
    # (both sides are prefill results, each within FLOOR_PREFILL of the exact rows on the floor figure)
    check(np.concatenate([a, b]), whole, f"{name} chunk cut at {cut}", floor=2 * FLOOR_PREFILL)
    dk, dv = _dev(kc), _dev(vc)
    for t in (0, cut - 1, cut, batch - 1):
        dec = gpu_decode(fa, q[t], kc, vc, H, G, d, n_ctx, n_past + t, SCALE, dk=dk, dv=dv)
        check(whole[t], dec, f"{name} prefill row {t} vs decode")


@pytest.mark.parametrize("name,H,G,n_ctx,L", DECODE)
def test_decode_is_invariant_under_a_permutation_of_the_visible_rows(fa, name, H, G, n_ctx, L):
    """Attention is a sum over the visible (K row, V row) pairs: shuffling them moves every
    pair to another tile, wave and split, and must change nothing but rounding."""
    d = 128
    q, kc, vc = make_case(331, H, G, d, n_ctx, L, 1, outliers=4)
    base = gpu_decode(fa, q[0], kc, vc, H, G, d, n_ctx, L - 1, SCALE)
    perm = np.random.default_rng(332).permutation(L)
    kp, vp = kc.copy(), vc.copy()
    kp[:, :L] = kc[:, perm]
    vp[:, :L] = vc[:, perm]
    got = gpu_decode(fa, q[0], kp, vp, H, G, d, n_ctx, L - 1, SCALE)
    check(got, base, f"{name} permuted rows", tol=TOL / 100, floor=FLOOR_DECODE)


@pytest.mark.parametrize("name,H,G,n_ctx,L", DECODE[:2])
def test_decode_short_position_in_the_full_cache_ignores_the_rest(fa, name, H, G, n_ctx, L):
    """A position far below the cache's length: the rows past it hold NaN patterns in one run
    and other finite data in the other; the outputs are identical bit for bit."""
    d = 128
    pos = 20011
    q, kc, vc = make_case(341, H, G, d, n_ctx, n_ctx, 1, outliers=4)
    a = gpu_decode(fa, q[0], kc, vc, H, G, d, n_ctx, pos, SCALE)
    kn, vn = kc.copy(), vc.copy()
    kn[:, pos + 1:] = 0x7E00
    vn[:, pos + 1:] = 0x7E00
    b = gpu_decode(fa, q[0], kn, vn, H, G, d, n_ctx, pos, SCALE)
    assert np.isfinite(b).all()
    assert np.array_equal(a, b), f"{name}: rows past the position reached the result"


def test_prefill_is_linear_in_v(fa):
    """out(V1 + V2) = out(V1) + out(V2) with K and Q fixed (the weights depend on neither):
    Llama-3-8B's chunk at depth 4096, every row."""
    name, H, G, n_ctx, n_past, batch = PREFILL[0]
    d = 128
    q, kc, _ = make_case(351, H, G, d, n_ctx, n_past + batch, batch, outliers=0)
    rng = np.random.default_rng(352)

    def grid_v():  # multiples of 2^-7 below 4 in magnitude: the sum of two is still an exact fp16 value
        x = np.clip(rng.standard_normal((G, n_ctx, d), dtype=np.float32), -4.0, 4.0)
        return (np.round(x * 64.0) / 128.0).astype(np.float16)

    f1, f2 = grid_v(), grid_v()
    fs = f1.astype(np.float32) + f2.astype(np.float32)
    assert np.array_equal(fs.astype(np.float16).astype(np.float32), fs)
    o1 = gpu_prefill(fa, q, kc, f1.view(np.uint16), H, G, d, n_ctx, n_past, batch, SCALE)
    o2 = gpu_prefill(fa, q, kc, f2.view(np.uint16), H, G, d, n_ctx, n_past, batch, SCALE)
    os_ = gpu_prefill(fa, q, kc, fs.astype(np.float16).view(np.uint16), H, G, d, n_ctx, n_past, batch, SCALE)
    check(os_, o1 + o2, f"{name} linear in V", floor=3 * FLOOR_PREFILL)  # (three prefill results meet here)
