"""Seeded sweep over shapes nobody picked by hand: head_dim, GQA ratio (beyond 8 too), KV heads,
cache length (not a multiple of the tile), depth, chunk length (ragged, 1, ending at n_ctx), sign
and size of the scale, K outliers, NaN patterns past the filled rows -- prefill and decode through
the C ABI against the oracle on sampled rows, gates as everywhere (tests/util.py)."""
import numpy as np
import pytest

from oracle import ref
from test_gpu_parity import check, fa, gpu_decode, gpu_prefill  # noqa: F401  (fa: fixture)
from util import FLOOR_DECODE, make_case

pytestmark = pytest.mark.gpu


def _cases(seed, n):
    rng = np.random.default_rng(seed)
    out = []
    for it in range(n):
        d = int(rng.choice([64, 128]))
        G = int(rng.choice([1, 2, 3, 4, 8]))
        r = int(rng.choice([1, 2, 3, 4, 5, 6, 7, 8, 9, 12, 16, 17]))
        n_ctx = int(rng.choice([64, 100, 256, 1000, 2048, 4096, 8192, 16384]))
        scale = float(rng.choice([1.0 / np.sqrt(d), 0.3, -0.1, 1.0]))
        outliers = int(rng.choice([0, 4]))
        if rng.random() < 0.6:
            batch = int(min(n_ctx, rng.choice([1, 2, 5, 16, 31, 33, 64, 100, 257, 512])))
            n_past = n_ctx - batch if rng.random() < 0.3 else int(rng.integers(0, n_ctx - batch + 1))
            picks = [int(x) for x in rng.integers(0, batch, 3)]
            out.append(("prefill", it, d, G, r, n_ctx, n_past, batch, scale, outliers, picks))
        else:
            L = n_ctx if rng.random() < 0.3 else int(rng.integers(1, n_ctx + 1))
            out.append(("decode", it, d, G, r, n_ctx, L, 1, scale, outliers, []))
    return out


@pytest.mark.parametrize("case", _cases(20250, 90), ids=lambda c: f"{c[0]}{c[1]}-d{c[2]}-G{c[3]}-r{c[4]}-ctx{c[5]}-{c[6]}-{c[7]}")
def test_random_shape(fa, case):
    kind, it, d, G, r, n_ctx, a, batch, scale, outliers, picks = case
    H = G * r
    print(case, flush=True)
    if kind == "prefill":
        n_past = a
        q, kc, vc = make_case(5000 + it, H, G, d, n_ctx, n_past + batch, batch, outliers=outliers, poison_tail=True)
        got = gpu_prefill(fa, q, kc, vc, H, G, d, n_ctx, n_past, batch, scale)
        toks = sorted(set([0, batch - 1] + picks))
        rows = np.array([(t, h) for t in toks for h in range(H)], np.int32)
        want = ref.flash_attention_rows(q, kc, vc, rows, H, G, d, n_ctx, n_past, np.float32(scale))
        check(got[rows[:, 0], rows[:, 1]], want, str(case))
    else:
        L = a
        q, kc, vc = make_case(5000 + it, H, G, d, n_ctx, L, 1, outliers=outliers, poison_tail=True)
        got = gpu_decode(fa, q[0], kc, vc, H, G, d, n_ctx, L - 1, scale)
        rows = np.array([(0, h) for h in range(H)], np.int32)
        want = ref.flash_attention_rows(q, kc, vc, rows, H, G, d, n_ctx, L - 1, np.float32(scale))
        check(got, want, str(case), floor=FLOOR_DECODE)
