"""The decode entry point that allocates nothing (partial results in the library's fixed device
block) against the ordinary one, through the C ABI: two calls in a row, the second smaller."""
import numpy as np
import pytest

from util import make_case

pytestmark = pytest.mark.gpu


def _setup():
    import torch

    from orin_llm_amd import kernels

    torch.cuda.set_device(0)
    kernels.init(0)
    kernels.set_stream(torch.cuda.current_stream().cuda_stream)
    return torch, kernels


def _both(torch, kernels, seed, H, G, d, n_ctx, pos):
    q, kc, vc = make_case(seed, H, G, d, n_ctx, pos + 1, 1, outliers=4, poison_tail=True)
    dq = torch.from_numpy(q[0]).cuda()
    dk = torch.from_numpy(kc).view(torch.int16).cuda()
    dv = torch.from_numpy(vc).view(torch.int16).cuda()
    dpos = torch.tensor([pos], dtype=torch.int32, device="cuda")
    scale = float(1.0 / np.sqrt(d))
    want = torch.full((H, d), float("nan"), device="cuda")
    got = torch.full((H, d), float("nan"), device="cuda")
    kernels.flash_attention_decode_ind(dq, dk, dv, want, H, G, d, n_ctx, dpos, scale)
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    kernels.flash_attention_decode_ind_static(dq, dk, dv, got, H, G, d, n_ctx, dpos, scale)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0  # nothing was allocated on the device
    return want.cpu().numpy(), got.cpu().numpy()


def test_static_scratch_decode_matches_workspace_decode_twice():
    torch, kernels = _setup()
    assert kernels.static_scratch_bytes() == 2 << 20
    # a long position (every split active), then a smaller call: fewer heads, a short position
    # in a shorter cache (most splits inactive, fewer splits), which finds the first call's partials
    # still in the block
    for seed, (H, G, d, n_ctx, pos) in enumerate([(28, 4, 128, 8192, 8000), (12, 2, 128, 2048, 77), (8, 8, 64, 4096, 4095)]):
        want, got = _both(torch, kernels, 40 + seed, H, G, d, n_ctx, pos)
        assert np.isfinite(got).all()
        assert np.array_equal(want.view(np.uint32), got.view(np.uint32)), (H, G, d, n_ctx, pos)


def test_static_scratch_rejects_what_does_not_fit():
    torch, kernels = _setup()
    # 64 KV heads x 4 query heads each: 256 heads x 4 splits... the block holds 2 MiB of partials
    H, G, d, n_ctx = 1024, 1, 128, 65536
    need = kernels.decode_splits(H, G, d, n_ctx) * H * (d + 2) * 4
    assert need > kernels.static_scratch_bytes()
    q = torch.zeros((H, d), device="cuda")
    kc = torch.zeros((G, n_ctx, d), dtype=torch.int16, device="cuda")
    out = torch.zeros((H, d), device="cuda")
    dpos = torch.tensor([5], dtype=torch.int32, device="cuda")
    with pytest.raises(kernels.OrinFaError) as e:
        kernels.flash_attention_decode_ind_static(q, kc, kc, out, H, G, d, n_ctx, dpos, 0.1)
    assert e.value.code == -3
