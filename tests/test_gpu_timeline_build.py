"""The timeline build (liborin_fa_stamps.so: the attention kernels' stage marks store the wall clock) is a
measurement aid, but it runs the same kernels: its outputs must equal the ordinary library's bit for bit, and
the marks of a wave must come in the order the wave passes them."""
import ctypes

import numpy as np
import pytest

from util import make_case

pytestmark = pytest.mark.gpu


def _dev(torch, a):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if t.dtype == torch.uint16:
        t = t.view(torch.int16)
    return t.cuda()


def test_timeline_build_gives_the_same_results_and_ordered_marks():
    torch = pytest.importorskip("torch")
    from orin_llm_amd import kernels

    kernels.init(0)
    kernels.set_stream(torch.cuda.current_stream().cuda_stream)
    L = kernels.stamps_lib()
    assert L.orin_fa_init(0) == 0
    L.orin_fa_set_stream(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    H, G, d, n_ctx, n_past, batch = 12, 2, 128, 4096, 1500, 200
    scale = 1.0 / np.sqrt(d)
    q, kc, vc = make_case(77, H, G, d, n_ctx, n_past + batch, batch, outliers=4)
    dq, dk, dv = _dev(torch, q), _dev(torch, kc), _dev(torch, vc)

    # prefill
    a = torch.empty((batch, H, d), dtype=torch.float32, device="cuda")
    b = torch.empty_like(a)
    kernels.flash_attention(dq, dk, dv, a, H, G, d, n_ctx, n_past, batch, float(scale))
    host = np.zeros(1024 * 4 * 16, np.int64)
    assert L.orin_fa_bench_stamps(0, host.ctypes.data, host.size) == 0  # (clears the table)
    assert L.orin_fa_prefill(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), b.data_ptr(), H, G, d, n_ctx, n_past, batch, scale) == 0
    torch.cuda.synchronize()
    assert torch.equal(a, b)
    assert L.orin_fa_bench_stamps(0, host.ctypes.data, host.size) == 0
    st = host.reshape(1024, 4, 16)
    order = [0, 9, 10, 1, 2, 3, 4, 5, 7, 8]
    full = st[:, :, 8] > 0
    assert full.any()
    marks = st[full][:, order]
    assert (np.diff(marks, axis=1) >= 0).all(), "a wave's marks are out of order"
    assert (marks[:, -1] - marks[:, 0]).max() < 100 * 1000  # below a millisecond at 100 MHz

    # decode
    pos = torch.tensor([n_past + batch - 1], dtype=torch.int32, device="cuda")
    oa = torch.empty((H, d), dtype=torch.float32, device="cuda")
    ob = torch.empty_like(oa)
    kernels.flash_attention_decode_ind(dq[-1], dk, dv, oa, H, G, d, n_ctx, pos, float(scale))
    host8 = np.zeros(1024 * 8 * 16, np.int64)
    assert L.orin_fa_bench_stamps(1, host8.ctypes.data, host8.size) == 0
    assert L.orin_fa_decode_ind(dq[-1].data_ptr(), dk.data_ptr(), dv.data_ptr(), ob.data_ptr(), H, G, d, n_ctx, pos.data_ptr(), scale) == 0
    torch.cuda.synchronize()
    assert torch.equal(oa, ob)
    assert L.orin_fa_bench_stamps(1, host8.ctypes.data, host8.size) == 0
    st8 = host8.reshape(1024, 8, 16)
    full8 = st8[:, :, 7] > 0
    assert full8.any()
    m8 = st8[full8][:, [0, 1, 2, 4, 5, 6, 7]]  # (mark 3 sits inside the tile loop: waves without a tile skip it)
    assert (np.diff(m8, axis=1) >= 0).all()


def test_ordinary_library_has_no_stamps():
    """The stage marks and their reader exist in the timeline build only: the product library does not export them."""
    from orin_llm_amd import kernels

    assert not hasattr(kernels.lib(), "orin_fa_bench_stamps")
    assert hasattr(kernels.stamps_lib(), "orin_fa_bench_stamps")
