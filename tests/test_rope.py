"""Rotary position embedding: the oracle pinned on the CPU, the HIP path against it on the GPU
(reference: src/model_cpu.cpp:179-203; src/kernels.cu:1619-1657, 2059-2075)."""
import numpy as np
import pytest

from oracle import ref

# The GPU follows the CPU statement operation by operation; what may differ is the last bit of
# the library sine/cosine (and, rarely, of the frequency), so the gate is relative to the pair.
ROPE_TOL = 2e-6


def _closed_form(x, head_dim, n_rot, theta, n_past, heads, ff, neox):
    """float64 rotation by the angle the reference forms in fp32."""
    x = np.asarray(x, np.float64).reshape(-1, head_dim).copy()
    half = n_rot // 2
    i = np.arange(half, dtype=np.float32)
    expo = (np.float32(-2.0) * i) / np.float32(n_rot)
    freq = np.power(np.float64(np.float32(theta)), expo.astype(np.float64)).astype(np.float32)  # = correctly rounded powf
    if ff is not None:
        freq = freq / np.asarray(ff, np.float32)
    for r in range(x.shape[0]):
        pos = np.float32(n_past + r // heads)
        ang = (pos * freq).astype(np.float32).astype(np.float64)
        c, s = np.cos(ang), np.sin(ang)
        i0 = np.arange(half) if neox else 2 * np.arange(half)
        i1 = i0 + half if neox else i0 + 1
        x0, x1 = x[r, i0].copy(), x[r, i1].copy()
        x[r, i0] = x0 * c - x1 * s
        x[r, i1] = x0 * s + x1 * c
    return x


CASES = [  # head_dim, n_rot, theta, n_past, heads, tokens, with freq_factors
    (128, 128, 10000.0, 0, 12, 45, False),
    (128, 128, 1000000.0, 3584, 2, 64, False),
    (128, 64, 500000.0, 32000, 8, 9, True),
    (64, 64, 10000.0, 7, 3, 5, False),
    (96, 32, 10000.0, 1000, 4, 3, True),
]


@pytest.mark.parametrize("neox", [True, False])
@pytest.mark.parametrize("case", CASES)
def test_oracle_rope_is_the_float64_rotation(case, neox):
    head_dim, n_rot, theta, n_past, heads, tokens, with_ff = case
    rng = np.random.default_rng(11)
    x = rng.standard_normal((tokens * heads, head_dim)).astype(np.float32)
    ff = (1.0 + rng.random(n_rot // 2) * 7).astype(np.float32) if with_ff else None
    got = ref.rope_batch(x, head_dim, n_rot, theta, n_past, heads, ff, neox)
    want = _closed_form(x, head_dim, n_rot, theta, n_past, heads, ff, neox)
    assert np.abs(got - want).max() < 1e-6 * np.abs(x).max()
    assert np.array_equal(got[:, n_rot:], x[:, n_rot:])                      # past n_rot: untouched
    pair = np.hypot(got[:, :n_rot // 2], got[:, n_rot // 2:n_rot]) if neox else np.hypot(got[:, 0:n_rot:2], got[:, 1:n_rot:2])
    pair0 = np.hypot(x[:, :n_rot // 2], x[:, n_rot // 2:n_rot]) if neox else np.hypot(x[:, 0:n_rot:2], x[:, 1:n_rot:2])
    assert np.allclose(pair, pair0, rtol=1e-6, atol=1e-6)                     # a rotation keeps each pair's length


def test_oracle_rope_neox_is_normal_on_permuted_elements_and_pos0_is_identity():
    head_dim, n_rot, theta, heads, tokens = 128, 96, 10000.0, 5, 7
    rng = np.random.default_rng(12)
    x = rng.standard_normal((tokens * heads, head_dim)).astype(np.float32)
    half = n_rot // 2
    perm = np.arange(head_dim)
    perm[0:n_rot:2] = np.arange(half)            # normal's pair (2i, 2i+1) <- neox's pair (i, i + half)
    perm[1:n_rot:2] = np.arange(half) + half
    a = ref.rope_batch(x, head_dim, n_rot, theta, 123, heads, None, True)
    b = ref.rope_batch(x[:, perm], head_dim, n_rot, theta, 123, heads, None, False)
    assert np.array_equal(a[:, perm], b)
    one = ref.rope_batch(x[:heads], head_dim, n_rot, theta, 0, heads, None, True)
    assert np.array_equal(one, x[:heads])


# ---------------------------------------------------------------------------------------- GPU

@pytest.fixture(scope="module")
def fa():
    import torch
    from orin_llm_amd import kernels
    assert torch.cuda.is_available()
    kernels.init(0)
    kernels.set_stream(torch.cuda.current_stream().cuda_stream)
    return kernels


def _check(got, want, x, n_rot, what):
    scale = np.maximum(np.abs(x).max(axis=1, keepdims=True), 1e-30)
    err = (np.abs(got - want) / scale).max()
    print(f"{what}: max |d| / max|row| = {err:.3e} (gate {ROPE_TOL:g})", flush=True)
    assert np.isfinite(got).all() and err < ROPE_TOL, (what, err)
    assert np.array_equal(got[:, n_rot:], x[:, n_rot:])


@pytest.mark.gpu
@pytest.mark.parametrize("neox", [True, False])
@pytest.mark.parametrize("case", CASES + [(128, 128, 1000000.0, 32256, 28, 512, False), (128, 128, 500000.0, 7680, 8, 512, True)])
def test_rope_batch(fa, case, neox):
    import torch
    head_dim, n_rot, theta, n_past, heads, tokens, with_ff = case
    rng = np.random.default_rng(tokens + n_rot)
    x = rng.standard_normal((tokens * heads, head_dim)).astype(np.float32)
    ff = (1.0 + rng.random(n_rot // 2) * 7).astype(np.float32) if with_ff else None
    want = ref.rope_batch(x, head_dim, n_rot, theta, n_past, heads, ff, neox)
    dx = torch.from_numpy(x).cuda()
    dff = None if ff is None else torch.from_numpy(ff).cuda()
    (fa.rope_neox_batch if neox else fa.rope_normal_batch)(dx, tokens * heads, head_dim, n_rot, theta, n_past, heads, dff)
    torch.cuda.synchronize()
    _check(dx.cpu().numpy(), want, x, n_rot, f"rope batch neox={neox} {case}")


@pytest.mark.gpu
@pytest.mark.parametrize("neox", [True, False])
def test_rope_ind_reads_the_position_on_the_device_and_replays(fa, neox):
    import torch
    heads, head_dim, n_rot, theta = 12, 128, 128, 1000000.0
    rng = np.random.default_rng(13)
    x = rng.standard_normal((heads, head_dim)).astype(np.float32)
    dx = torch.empty((heads, head_dim), device="cuda")
    dpos = torch.zeros(1, dtype=torch.int32, device="cuda")
    fn = fa.rope_neox_ind if neox else fa.rope_normal_ind
    g = torch.cuda.CUDAGraph()
    try:
        with torch.cuda.graph(g):
            fa.set_stream(torch.cuda.current_stream().cuda_stream)
            fn(dx, heads, head_dim, n_rot, theta, dpos)
    finally:
        fa.set_stream(torch.cuda.current_stream().cuda_stream)
    for pos in (0, 1, 4095, 32767):
        dx.copy_(torch.from_numpy(x))
        dpos.fill_(pos)
        g.replay()
        torch.cuda.synchronize()
        want = ref.rope_batch(x, head_dim, n_rot, theta, pos, heads, None, neox)   # one token: every row at n_past
        _check(dx.cpu().numpy(), want, x, n_rot, f"rope ind neox={neox} pos={pos}")


@pytest.mark.gpu
def test_rope_rejects_bad_arguments(fa):
    import torch
    from orin_llm_amd.kernels import OrinFaError
    x = torch.zeros((8, 128), device="cuda")
    with pytest.raises(OrinFaError):
        fa.rope_neox_batch(x, 8, 128, 130, 10000.0, 0, 2)     # n_rot > head_dim
    with pytest.raises(OrinFaError):
        fa.rope_neox_batch(x, 8, 128, 63, 10000.0, 0, 2)      # odd n_rot
    with pytest.raises(OrinFaError):
        fa.rope_normal_batch(x, 7, 128, 64, 10000.0, 0, 2)    # rows not a multiple of heads
    with pytest.raises(OrinFaError):
        fa.rope_neox_ind(x, 8, 128, 64, 10000.0, None)
