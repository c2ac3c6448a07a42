"""KV-cache mutators: the oracle pinned on the CPU, the HIP path bit-exact against it on the GPU
(reference: src/kernels.cu:1659-1700, 2079-2093; src/model_cpu.cpp:276-279, 321-338)."""
import numpy as np
import pytest

from oracle import ref


def _cache(rng, n_layer, n_kv, n_ctx, d):
    return (rng.integers(1, 65535, size=(n_layer, n_kv, n_ctx, d), dtype=np.uint16),
            rng.integers(1, 65535, size=(n_layer, n_kv, n_ctx, d), dtype=np.uint16))


SHIFT_CASES = [  # n_layer, n_kv, d, n_ctx, n_keep, shift
    (2, 2, 128, 64, 4, 30),      # the engine's policy: half of what lies past n_keep
    (1, 3, 128, 97, 0, 1),       # one row, long chains
    (2, 1, 64, 50, 7, 43),       # shift == n_ctx - n_keep: everything past n_keep is cleared
    (1, 2, 128, 40, 40, 0),      # nothing to do
    (1, 2, 128, 33, 5, 5),
    (3, 2, 72, 31, 3, 9),        # 144-byte rows
    (1, 1, 20, 17, 2, 6),        # rows that are no multiple of 16 bytes
]


@pytest.mark.parametrize("case", SHIFT_CASES)
def test_oracle_kv_shift_is_the_slice_statement(case):
    n_layer, n_kv, d, n_ctx, n_keep, shift = case
    rng = np.random.default_rng(5)
    kc, vc = _cache(rng, n_layer, n_kv, n_ctx, d)
    k2, v2 = kc.copy(), vc.copy()
    ref.kv_shift_u16(k2, v2, n_layer, n_kv, d, n_ctx, n_keep, shift)
    for new, old in ((k2, kc), (v2, vc)):
        want = old.copy()
        want[:, :, n_keep:n_ctx - shift] = old[:, :, n_keep + shift:]
        want[:, :, n_ctx - shift:] = 0
        assert np.array_equal(new, want)


def test_oracle_kv_store_matches_numpy_float16():
    rng = np.random.default_rng(6)
    n_kv, d, n_ctx, pos_base, batch = 3, 128, 40, 11, 7
    k = rng.standard_normal((batch, n_kv, d)).astype(np.float32) * np.float32(100.0)
    v = rng.standard_normal((batch, n_kv, d)).astype(np.float32) * np.float32(1e-6)  # subnormal halves
    k[0, 0, :6] = [65504.0, 65519.99, 65520.0, 1e9, -np.inf, 2.0 ** -25]
    kc = np.full((n_kv, n_ctx, d), 0x1234, np.uint16)
    vc = np.full((n_kv, n_ctx, d), 0x4321, np.uint16)
    ref.kv_store_f16(kc, vc, k, v, n_kv, d, n_ctx, pos_base, batch)
    with np.errstate(over="ignore"):
        wk = k.astype(np.float16).view(np.uint16).transpose(1, 0, 2)
        wv = v.astype(np.float16).view(np.uint16).transpose(1, 0, 2)
    assert np.array_equal(kc[:, pos_base:pos_base + batch], wk)
    assert np.array_equal(vc[:, pos_base:pos_base + batch], wv)
    assert (kc[:, :pos_base] == 0x1234).all() and (kc[:, pos_base + batch:] == 0x1234).all()
    assert (vc[:, :pos_base] == 0x4321).all() and (vc[:, pos_base + batch:] == 0x4321).all()


# ---------------------------------------------------------------------------------------- GPU

@pytest.fixture(scope="module")
def fa():
    import torch
    from orin_llm_amd import kernels
    assert torch.cuda.is_available()
    kernels.init(0)
    kernels.set_stream(torch.cuda.current_stream().cuda_stream)
    return kernels


def _dev_u16(torch, a):
    return torch.from_numpy(a.view(np.int16).copy()).cuda()


def _host_u16(t):
    return t.cpu().numpy().view(np.uint16)


@pytest.mark.gpu
@pytest.mark.parametrize("n_kv,d,n_ctx,pos_base,batch", [
    (2, 128, 4096, 0, 512), (8, 128, 600, 88, 512), (4, 128, 300, 299, 1), (2, 64, 100, 3, 45),
    (3, 72, 50, 1, 9), (1, 20, 17, 5, 12)])
def test_kv_store_batch_bit_exact(fa, n_kv, d, n_ctx, pos_base, batch):
    import torch
    rng = np.random.default_rng(batch + d)
    k = (rng.standard_normal((batch, n_kv, d)) * 30).astype(np.float32)
    v = (rng.standard_normal((batch, n_kv, d)) * 3e-6).astype(np.float32)   # many subnormal halves
    k.reshape(-1)[:8] = [65504.0, 65519.99, 65520.0, 1e9, -np.inf, 2.0 ** -25, -0.0, 6.1e-5]
    kc0, vc0 = _cache(rng, 1, n_kv, n_ctx, d)
    kc0, vc0 = kc0[0], vc0[0]
    wk, wv = kc0.copy(), vc0.copy()
    ref.kv_store_f16(wk, wv, k, v, n_kv, d, n_ctx, pos_base, batch)
    dk, dv = _dev_u16(torch, kc0), _dev_u16(torch, vc0)
    fa.kv_store_batch(dk, dv, torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(), n_kv, d, n_ctx, pos_base, batch)
    torch.cuda.synchronize()
    assert np.array_equal(_host_u16(dk), wk)   # rows outside [pos_base, pos_base + batch) untouched as well
    assert np.array_equal(_host_u16(dv), wv)


@pytest.mark.gpu
def test_kv_store_ind_reads_the_position_on_the_device_and_replays(fa):
    import torch
    n_kv, d, n_ctx = 4, 128, 256
    rng = np.random.default_rng(9)
    kc0, vc0 = _cache(rng, 1, n_kv, n_ctx, d)
    dk, dv = _dev_u16(torch, kc0[0]), _dev_u16(torch, vc0[0])
    wk, wv = kc0[0].copy(), vc0[0].copy()
    k = torch.zeros((n_kv, d), device="cuda")
    v = torch.zeros((n_kv, d), device="cuda")
    dpos = torch.zeros(1, dtype=torch.int32, device="cuda")
    g = torch.cuda.CUDAGraph()
    try:
        with torch.cuda.graph(g):
            fa.set_stream(torch.cuda.current_stream().cuda_stream)
            fa.kv_store_ind(dk, dv, k, v, n_kv, d, n_ctx, dpos)
    finally:
        fa.set_stream(torch.cuda.current_stream().cuda_stream)
    for pos in (0, 17, 255, 256, -1):     # the last two are out of range: nothing may be written
        hk = rng.standard_normal((1, n_kv, d)).astype(np.float32)
        hv = rng.standard_normal((1, n_kv, d)).astype(np.float32)
        k.copy_(torch.from_numpy(hk[0]))
        v.copy_(torch.from_numpy(hv[0]))
        dpos.fill_(pos)
        g.replay()
        torch.cuda.synchronize()
        if 0 <= pos < n_ctx:
            ref.kv_store_f16(wk, wv, hk, hv, n_kv, d, n_ctx, pos, 1)
        assert np.array_equal(_host_u16(dk), wk), pos
        assert np.array_equal(_host_u16(dv), wv), pos


@pytest.mark.gpu
@pytest.mark.parametrize("case", SHIFT_CASES + [(4, 2, 128, 4096, 16, 2040), (2, 8, 128, 1024, 0, 512)])
def test_kv_shift_bit_exact(fa, case):
    import torch
    n_layer, n_kv, d, n_ctx, n_keep, shift = case
    rng = np.random.default_rng(n_ctx + shift)
    kc, vc = _cache(rng, n_layer, n_kv, n_ctx, d)
    dk, dv = _dev_u16(torch, kc), _dev_u16(torch, vc)
    ref.kv_shift_u16(kc, vc, n_layer, n_kv, d, n_ctx, n_keep, shift)
    fa.kv_shift(dk, dv, n_layer, n_kv, d, n_ctx, n_keep, shift)
    torch.cuda.synchronize()
    assert np.array_equal(_host_u16(dk), kc)
    assert np.array_equal(_host_u16(dv), vc)


@pytest.mark.gpu
def test_store_then_attend_equals_attending_a_prebuilt_cache(fa):
    """The call-site order (reference: src/model_gpu.cu:378-384): append the chunk's K/V, then attend."""
    import torch
    H, G, d, n_ctx, n_past, batch = 12, 2, 128, 512, 100, 77
    scale = float(1.0 / np.sqrt(d))
    rng = np.random.default_rng(3)
    k_all = rng.standard_normal((n_past + batch, G, d)).astype(np.float32)
    v_all = rng.standard_normal((n_past + batch, G, d)).astype(np.float32)
    q = rng.standard_normal((batch, H, d)).astype(np.float32)
    kc = np.zeros((G, n_ctx, d), np.uint16)
    vc = np.zeros((G, n_ctx, d), np.uint16)
    ref.kv_store_f16(kc, vc, k_all, v_all, G, d, n_ctx, 0, n_past + batch)
    want = ref.flash_attention(q, kc, vc, H, G, d, n_ctx, n_past, batch, np.float32(scale))
    dk = torch.full((G, n_ctx, d), 0x7e00, dtype=torch.int16, device="cuda")   # NaN everywhere
    dv = torch.full((G, n_ctx, d), 0x7e00, dtype=torch.int16, device="cuda")
    fa.kv_store_batch(dk, dv, torch.from_numpy(k_all[:n_past]).cuda(), torch.from_numpy(v_all[:n_past]).cuda(),
                      G, d, n_ctx, 0, n_past)
    fa.kv_store_batch(dk, dv, torch.from_numpy(k_all[n_past:]).cuda(), torch.from_numpy(v_all[n_past:]).cuda(),
                      G, d, n_ctx, n_past, batch)
    out = torch.empty((batch, H, d), device="cuda")
    fa.flash_attention(torch.from_numpy(q).cuda(), dk, dv, out, H, G, d, n_ctx, n_past, batch, scale)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    err = np.max(np.abs(got - want).max(axis=2) / np.abs(want).max(axis=2))
    assert np.isfinite(got).all() and err < 2e-3, err


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,d,n_ctx", [(12, 2, 128, 4096), (28, 4, 128, 32768), (8, 8, 64, 600), (40, 2, 128, 1024)])
def test_decode_store_equals_store_then_decode(fa, H, G, d, n_ctx):
    """The fused entry point against the two calls it stands for (reference call site:
    src/model_gpu.cu:281-282): same cache bytes and same output, bit for bit, at positions on
    both sides of tile and split edges, at the last row of the cache, out of range, and replayed
    from a graph with the position changed on the device."""
    import torch
    scale = float(1.0 / np.sqrt(d))
    rng = np.random.default_rng(H + n_ctx)
    base_k = rng.standard_normal((G, n_ctx, d)).astype(np.float16).view(np.int16)
    base_v = rng.standard_normal((G, n_ctx, d)).astype(np.float16).view(np.int16)
    q = torch.from_numpy(rng.standard_normal((H, d)).astype(np.float32)).cuda()
    k_new = torch.zeros((G, d), device="cuda")
    v_new = torch.zeros((G, d), device="cuda")
    dpos = torch.zeros(1, dtype=torch.int32, device="cuda")
    ka, va = torch.from_numpy(base_k).cuda(), torch.from_numpy(base_v).cuda()   # two calls
    kb, vb = ka.clone(), va.clone()                                             # fused
    out_a = torch.empty((H, d), device="cuda")
    out_b = torch.empty((H, d), device="cuda")
    g = torch.cuda.CUDAGraph()
    try:
        with torch.cuda.graph(g):
            fa.set_stream(torch.cuda.current_stream().cuda_stream)
            fa.flash_attention_decode_store_ind(q, k_new, v_new, kb, vb, out_b, H, G, d, n_ctx, dpos, scale)
    finally:
        fa.set_stream(torch.cuda.current_stream().cuda_stream)
    positions = [0, 1, 30, 31, 32, 33, 255, 256, 257, n_ctx // 2 - 1, n_ctx // 2, n_ctx - 2, n_ctx - 1, n_ctx, -1]
    for i, pos in enumerate(positions):
        k_new.copy_(torch.from_numpy(rng.standard_normal((G, d)).astype(np.float32) * 3.0))
        v_new.copy_(torch.from_numpy(rng.standard_normal((G, d)).astype(np.float32) * 3.0))
        dpos.fill_(pos)
        fa.kv_store_ind(ka, va, k_new, v_new, G, d, n_ctx, dpos)
        fa.flash_attention_decode_ind(q, ka, va, out_a, H, G, d, n_ctx, dpos, scale)
        if i % 2 == 0:
            g.replay()
        else:
            fa.flash_attention_decode_store_ind(q, k_new, v_new, kb, vb, out_b, H, G, d, n_ctx, dpos, scale)
        torch.cuda.synchronize()
        assert torch.equal(ka, kb) and torch.equal(va, vb), pos
        assert torch.equal(out_a.view(torch.int32), out_b.view(torch.int32)), pos


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,d,n_ctx,n_rot,neox,ff", [
    (12, 2, 128, 4096, 128, True, False),     # Qwen2.5-1.5B
    (28, 4, 128, 32768, 128, True, True),
    (32, 8, 128, 2048, 128, False, True),     # Llama-3 ("normal" pairing, frequency factors)
    (8, 8, 64, 600, 64, True, False),
    (8, 8, 64, 600, 32, False, False),        # partial rotation
    (40, 2, 128, 1024, 96, False, True),
    (12, 2, 128, 512, 0, True, False),        # no rotation: the store + attend pair
])
def test_decode_rope_store_equals_the_four_calls(fa, H, G, d, n_ctx, n_rot, neox, ff):
    """rope on q, rope on the new K row, kv_store_ind, flash_attention_decode_ind (reference
    call sites: src/model_gpu.cu:277-282) against the one call that stands for them: same cache
    bytes and same output bit for bit, q and k_new untouched, eager and replayed from a graph."""
    import torch
    scale = float(1.0 / np.sqrt(d))
    theta = 1.0e6 if neox else 5.0e5
    rng = np.random.default_rng(H * 7 + n_ctx + n_rot)
    base_k = rng.standard_normal((G, n_ctx, d)).astype(np.float16).view(np.int16)
    base_v = rng.standard_normal((G, n_ctx, d)).astype(np.float16).view(np.int16)
    freq = torch.from_numpy(rng.uniform(0.5, 8.0, max(n_rot // 2, 1)).astype(np.float32)).cuda() if ff else None
    q = torch.zeros((H, d), device="cuda")
    k_new = torch.zeros((G, d), device="cuda")
    v_new = torch.zeros((G, d), device="cuda")
    dpos = torch.zeros(1, dtype=torch.int32, device="cuda")
    ka, va = torch.from_numpy(base_k).cuda(), torch.from_numpy(base_v).cuda()   # four calls
    kb, vb = ka.clone(), va.clone()                                             # one call
    out_a = torch.empty((H, d), device="cuda")
    out_b = torch.empty((H, d), device="cuda")
    rope_ind = fa.rope_neox_ind if neox else fa.rope_normal_ind

    angles = torch.zeros((max(n_rot // 2, 1), 2), device="cuda")

    def fused(with_table=False):
        if with_table and n_rot:   # the angles once per token, as a decode step over many layers would
            fa.rope_angles_ind(angles, n_rot, theta, dpos, freq)
        fa.flash_attention_decode_rope_store_ind(q, k_new, v_new, kb, vb, out_b, H, G, d, n_ctx, dpos, scale,
                                                 n_rot, theta, freq, neox, angles if with_table and n_rot else None)
    g = torch.cuda.CUDAGraph()
    try:
        with torch.cuda.graph(g):
            fa.set_stream(torch.cuda.current_stream().cuda_stream)
            fused()
    finally:
        fa.set_stream(torch.cuda.current_stream().cuda_stream)
    positions = [0, 1, 31, 32, 33, 255, 256, 257, n_ctx // 2 - 1, n_ctx // 2, n_ctx - 2, n_ctx - 1, n_ctx, -1]
    for i, pos in enumerate(positions):
        q.copy_(torch.from_numpy(rng.standard_normal((H, d)).astype(np.float32)))
        k_new.copy_(torch.from_numpy(rng.standard_normal((G, d)).astype(np.float32) * 3.0))
        v_new.copy_(torch.from_numpy(rng.standard_normal((G, d)).astype(np.float32) * 3.0))
        dpos.fill_(pos)
        q_rot, k_rot = q.clone(), k_new.clone()
        q_before, k_before = q.clone(), k_new.clone()
        if n_rot:
            rope_ind(q_rot, H, d, n_rot, theta, dpos, freq)
            rope_ind(k_rot, G, d, n_rot, theta, dpos, freq)
        fa.kv_store_ind(ka, va, k_rot, v_new, G, d, n_ctx, dpos)
        fa.flash_attention_decode_ind(q_rot, ka, va, out_a, H, G, d, n_ctx, dpos, scale)
        if i % 2 == 0:
            g.replay()
        else:
            fused(with_table=(i % 4 == 1))
        torch.cuda.synchronize()
        assert torch.equal(q, q_before) and torch.equal(k_new, k_before), pos
        assert torch.equal(ka, kb) and torch.equal(va, vb), pos
        assert torch.equal(out_a.view(torch.int32), out_b.view(torch.int32)), pos
    if n_rot:   # the rotation did something: the rotated row differs from the raw one
        assert not torch.equal(k_rot, k_new)


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,d,n_ctx,neox", [(12, 2, 128, 32768, True), (32, 8, 64, 8192, False)])
def test_decode_rope_store_over_a_sweep_of_positions(fa, H, G, d, n_ctx, neox):
    """The one call against the four it stands for at every position 2^e - 1, 2^e, 2^e + 1 and at a handful in
    between: the wave that owns the new row's tile, the number of tiles a split takes and the number of splits
    with any tile all change with the position, which the captured launch reads on the device.  Same cache bytes
    and same output, bit for bit, from one graph replayed throughout."""
    import torch
    scale, theta = float(1.0 / np.sqrt(d)), (1.0e6 if neox else 5.0e5)
    rng = np.random.default_rng(n_ctx + H)
    base_k = rng.standard_normal((G, n_ctx, d)).astype(np.float16).view(np.int16)
    base_v = rng.standard_normal((G, n_ctx, d)).astype(np.float16).view(np.int16)
    q, k_new, v_new = torch.zeros((H, d), device="cuda"), torch.zeros((G, d), device="cuda"), torch.zeros((G, d), device="cuda")
    dpos = torch.zeros(1, dtype=torch.int32, device="cuda")
    ka, va = torch.from_numpy(base_k).cuda(), torch.from_numpy(base_v).cuda()
    kb, vb = ka.clone(), va.clone()
    out_a, out_b = torch.empty((H, d), device="cuda"), torch.empty((H, d), device="cuda")
    rope_ind = fa.rope_neox_ind if neox else fa.rope_normal_ind
    g = torch.cuda.CUDAGraph()
    try:
        with torch.cuda.graph(g):
            fa.set_stream(torch.cuda.current_stream().cuda_stream)
            fa.flash_attention_decode_rope_store_ind(q, k_new, v_new, kb, vb, out_b, H, G, d, n_ctx, dpos, scale, d, theta, None, neox, None)
    finally:
        fa.set_stream(torch.cuda.current_stream().cuda_stream)
    positions = sorted({p for e in range(0, 16) for p in (2 ** e - 1, 2 ** e, 2 ** e + 1) if 0 <= p < n_ctx}
                       | {int(x) for x in rng.integers(0, n_ctx, 24)} | {n_ctx - 1, n_ctx - 33, n_ctx - 257})
    for pos in positions:
        q.copy_(torch.from_numpy(rng.standard_normal((H, d)).astype(np.float32)))
        k_new.copy_(torch.from_numpy(rng.standard_normal((G, d)).astype(np.float32) * 3.0))
        v_new.copy_(torch.from_numpy(rng.standard_normal((G, d)).astype(np.float32) * 3.0))
        dpos.fill_(pos)
        q_rot, k_rot = q.clone(), k_new.clone()
        rope_ind(q_rot, H, d, d, theta, dpos, None)
        rope_ind(k_rot, G, d, d, theta, dpos, None)
        fa.kv_store_ind(ka, va, k_rot, v_new, G, d, n_ctx, dpos)
        fa.flash_attention_decode_ind(q_rot, ka, va, out_a, H, G, d, n_ctx, dpos, scale)
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(ka, kb) and torch.equal(va, vb), pos
        assert torch.equal(out_a.view(torch.int32), out_b.view(torch.int32)), pos
    print(f"{len(positions)} positions of a {n_ctx}-row cache", flush=True)


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,d,n_ctx,n_past,batch,n_rot,neox,ff", [
    (12, 2, 128, 4096, 3584, 512, 128, True, False),   # Qwen2.5-1.5B chunk
    (32, 8, 128, 1024, 100, 300, 128, False, True),    # Llama-3 ("normal" pairing, frequency factors)
    (6, 3, 64, 300, 0, 37, 64, True, True),            # ragged head groups (6 and 3 heads by fours)
    (5, 1, 128, 64, 63, 1, 128, False, False),         # one token at the last position
    (8, 2, 128, 512, 7, 45, 64, True, False),          # partial rotation: the three launches
    (4, 4, 96, 200, 10, 20, 32, False, True),          # head_dim 96
    (4, 2, 128, 256, 0, 16, 0, True, False),           # no rotation
])
def test_rope_store_batch_equals_the_three_calls(fa, H, G, d, n_ctx, n_past, batch, n_rot, neox, ff):
    """rope on the Q rows, rope on the K rows, kv_store_batch (reference call sites:
    src/model_gpu.cu:378-382) against the one call that stands for them: q, k and both caches
    bit for bit."""
    import torch
    theta = 1.0e6 if neox else 5.0e5
    rng = np.random.default_rng(H + d + batch)
    q = torch.from_numpy(rng.standard_normal((batch, H, d)).astype(np.float32) * 2.0).cuda()
    k = torch.from_numpy(rng.standard_normal((batch, G, d)).astype(np.float32) * 2.0).cuda()
    v = torch.from_numpy(rng.standard_normal((batch, G, d)).astype(np.float32) * 2.0).cuda()
    freq = torch.from_numpy(rng.uniform(0.5, 8.0, max(n_rot // 2, 1)).astype(np.float32)).cuda() if ff else None
    base = torch.from_numpy(rng.integers(0, 30000, (G, n_ctx, d)).astype(np.int16)).cuda()
    ka, va, kb, vb = base.clone(), base.clone(), base.clone(), base.clone()
    qa, kra, qb, krb = q.clone(), k.clone(), q.clone(), k.clone()
    rope = fa.rope_neox_batch if neox else fa.rope_normal_batch
    if n_rot:
        rope(qa, batch * H, d, n_rot, theta, n_past, H, freq)
        rope(kra, batch * G, d, n_rot, theta, n_past, G, freq)
    fa.kv_store_batch(ka, va, kra, v, G, d, n_ctx, n_past, batch)
    fa.rope_store_batch(qb, krb, v, kb, vb, batch, H, G, d, n_ctx, n_past, n_rot, theta, freq, neox)
    torch.cuda.synchronize()
    assert torch.equal(qa.view(torch.int32), qb.view(torch.int32))
    assert torch.equal(kra.view(torch.int32), krb.view(torch.int32))
    assert torch.equal(ka, kb) and torch.equal(va, vb)
    if n_rot and n_past + batch > 1:
        assert not torch.equal(qb, q)
    assert torch.equal(kb[:, :n_past], base[:, :n_past]) and torch.equal(kb[:, n_past + batch:], base[:, n_past + batch:])


@pytest.mark.gpu
def test_decode_rope_store_rejects_what_it_does_not_cover(fa):
    import torch
    from orin_llm_amd.kernels import OrinFaError
    H, G, d, n_ctx = 4, 2, 128, 256
    q = torch.zeros((H, d), device="cuda")
    kn = torch.zeros((G, d), device="cuda")
    kc = torch.zeros((G, n_ctx, d), dtype=torch.int16, device="cuda")
    out = torch.empty((H, d), device="cuda")
    dpos = torch.zeros(1, dtype=torch.int32, device="cuda")
    for n_rot, neox in [(64, True), (130, False), (63, False), (-2, False)]:
        with pytest.raises(OrinFaError):
            fa.flash_attention_decode_rope_store_ind(q, kn, kn, kc, kc.clone(), out, H, G, d, n_ctx, dpos, 0.1,
                                                     n_rot, 1.0e4, None, neox)
    with pytest.raises(OrinFaError):
        fa.rope_angles_ind(q, 63, 1.0e4, dpos)
    with pytest.raises(OrinFaError):
        fa.flash_attention_decode_rope_store_ind(q, None, kn, kc, kc.clone(), out, H, G, d, n_ctx, dpos, 0.1,
                                                 128, 1.0e4, None, True)


@pytest.mark.gpu
def test_rope_store_batch_rejects_bad_arguments(fa):
    import torch
    from orin_llm_amd.kernels import OrinFaError
    H, G, d, n_ctx = 4, 2, 128, 64
    q = torch.zeros((8, H, d), device="cuda")
    k = torch.zeros((8, G, d), device="cuda")
    kc = torch.zeros((G, n_ctx, d), dtype=torch.int16, device="cuda")
    vc = kc.clone()
    for n_past, batch, n_rot in [(60, 8, 128), (-1, 8, 128), (0, 8, 130), (0, 8, 63)]:   # past n_ctx, negative, n_rot > d, odd
        with pytest.raises(OrinFaError):
            fa.rope_store_batch(q, k, k, kc, vc, batch, H, G, d, n_ctx, n_past, n_rot, 1.0e4, None, True)
    with pytest.raises(OrinFaError):
        fa.rope_store_batch(q, None, k, kc, vc, 8, H, G, d, n_ctx, 0, 128, 1.0e4, None, True)
    fa.rope_store_batch(q, k, k, kc, vc, 0, H, G, d, n_ctx, 0, 128, 1.0e4, None, True)        # an empty chunk is a no-op
    torch.cuda.synchronize()
    assert not kc.any()


@pytest.mark.gpu
def test_kv_mutators_reject_bad_arguments(fa):
    import torch
    from orin_llm_amd.kernels import OrinFaError
    t16 = torch.zeros(2 * 64 * 128, dtype=torch.int16, device="cuda")
    t32 = torch.zeros(8 * 2 * 128, device="cuda")
    with pytest.raises(OrinFaError):
        fa.kv_store_batch(t16, t16, t32, t32, 2, 128, 64, 60, 8)      # runs past n_ctx
    with pytest.raises(OrinFaError):
        fa.kv_store_batch(t16, t16, t32, t32, 2, 128, 64, -1, 8)
    with pytest.raises(OrinFaError):
        fa.kv_shift(t16, t16, 1, 2, 128, 64, 40, 30)                  # n_keep + shift > n_ctx
    with pytest.raises(OrinFaError):
        fa.kv_store_ind(t16, t16, t32, t32, 2, 128, 64, None)
