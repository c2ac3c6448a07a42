"""Shared helpers for the parity tests: input generators and the error metric."""
import numpy as np

# Gate for GPU-vs-oracle comparisons: max relative error on fp32 outputs.
TOL = 2e-3


def rel_err(got, ref):
    """Relative error with a per-row floor.

    err = max_i |got_i - ref_i| / max(|ref_i|, tau), tau = 1e-2 * max_j |ref_j| over the
    output row (one token, one head).  Plain element-wise relative error is undefined
    where the reference crosses zero; the floor is 1% of the row's largest magnitude.
    Returns (gated error, max|diff|/max|ref|, relative L2).
    """
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    assert got.shape == ref.shape
    g = got.reshape(-1, got.shape[-1])
    r = ref.reshape(-1, ref.shape[-1])
    tau = 1e-2 * np.abs(r).max(axis=1, keepdims=True)
    tau = np.maximum(tau, 1e-30)
    gated = float((np.abs(g - r) / np.maximum(np.abs(r), tau)).max())
    glob = float(np.abs(g - r).max() / max(np.abs(r).max(), 1e-30))
    l2 = float(np.linalg.norm(g - r) / max(np.linalg.norm(r), 1e-30))
    return gated, glob, l2


def normal_f16(rng, shape):
    """N(0,1) draws rounded to fp16; returns (fp32 values, uint16 bit patterns)."""
    h = rng.standard_normal(shape, dtype=np.float32).astype(np.float16)
    return h.astype(np.float32), h.view(np.uint16)


def make_case(seed, n_head, n_kv, d, n_ctx, n_filled, batch, outliers=0, poison_tail=False):
    """Seeded inputs in the operator API's layout.

    q fp32 [batch][n_head][d] with fp16-representable values; caches uint16
    [n_kv][n_ctx][d] filled on [0, n_filled); K gets `outliers` channels per KV head
    scaled by 8.  With poison_tail the unfilled rows hold NaN bit patterns instead of zeros.
    """
    rng = np.random.default_rng(seed)
    q, _ = normal_f16(rng, (batch, n_head, d))
    kf, _ = normal_f16(rng, (n_kv, n_filled, d))
    vf, vb = normal_f16(rng, (n_kv, n_filled, d))
    if outliers:
        for g in range(n_kv):
            ch = rng.choice(d, size=outliers, replace=False)
            kf[g, :, ch] *= 8.0
    kb = kf.astype(np.float16).view(np.uint16)
    fill = 0x7E00 if poison_tail else 0
    kc = np.full((n_kv, n_ctx, d), fill, np.uint16)
    vc = np.full((n_kv, n_ctx, d), fill, np.uint16)
    kc[:, :n_filled] = kb
    vc[:, :n_filled] = vb
    return q, kc, vc
