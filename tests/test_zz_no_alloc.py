"""sz_matvec_cols_static, the entry point that allocates nothing: its workspace is a device array inside the library.
Through the C ABI, against sz_matvec_cols with a workspace of the caller's, bit for bit, on two calls in a row of which
the second is smaller (the array keeps the first call's contents), then a call too large for the array."""
import numpy as np
import pytest

import shadow_engine_amd as sz
from shadow_engine_amd import synth

pytestmark = pytest.mark.gpu


def test_static_workspace_entry_point_matches_matvec_cols_on_two_calls_in_a_row():
    import torch
    assert torch.cuda.is_available(), "no GPU visible"
    sz.init(0)
    rng = np.random.default_rng(77)
    # (type, cols = in, rows = out, inputs): a large call first, then a smaller one of another rate and shape
    calls = [(sz.EXL3(4), 2048, 1024, 8), (sz.EXL3(3), 512, 256, 3), (sz.EXL3(2), 1024, 128, 1), (sz.Q8_0, 2048, 96, 5)]
    stream = sz.Stream()
    prepared = []
    for ty, cols, rows, m in calls:
        w = synth.exl3_blob(rng, cols, rows, ty - 1020) if ty >= 1000 else synth.q8_0_matrix(rng, rows, cols)
        dw = torch.from_numpy(w).cuda()
        xs, ys = cols + 32, rows + 16
        dx = torch.from_numpy(rng.normal(size=(m, xs)).astype(np.float32)).cuda()
        nsb = sz.matvec_cols_scratch(ty, cols, rows, m)
        assert nsb <= sz.STATIC_WORKSPACE_BYTES
        scratch = torch.empty(max(nsb, 16), dtype=torch.uint8, device="cuda")
        want = torch.zeros((m, ys), dtype=torch.float32, device="cuda")
        sz.matvec_cols(ty, dw.data_ptr(), cols, rows, dx.data_ptr(), xs, want.data_ptr(), ys, m, scratch.data_ptr(), nsb, stream.handle)
        got = torch.full((m, ys), 7.0, dtype=torch.float32, device="cuda")
        prepared.append((ty, cols, rows, m, dw, dx, xs, ys, want, got))
    stream.synchronize()
    # all the calls back to back on one stream, nothing allocated or synchronized in between
    for ty, cols, rows, m, dw, dx, xs, ys, want, got in prepared:
        print("static call", ty, cols, rows, m, flush=True)
        sz.matvec_cols_static(ty, dw.data_ptr(), cols, rows, dx.data_ptr(), xs, got.data_ptr(), ys, m, stream.handle)
    stream.synchronize()
    for ty, cols, rows, m, dw, dx, xs, ys, want, got in prepared:
        g, w_ = got.cpu().numpy(), want.cpu().numpy()
        assert np.array_equal(g[:, :rows].view(np.uint32), w_[:, :rows].view(np.uint32)), (ty, cols, rows, m)
        assert np.all(g[:, rows:] == 7.0)          # nothing written past the rows
        assert np.any(w_[:, :rows] != 0.0)
    # the same first call again after the smaller ones: the array holds their leftovers now
    ty, cols, rows, m, dw, dx, xs, ys, want, got = prepared[0]
    got.fill_(0.0)
    sz.matvec_cols_static(ty, dw.data_ptr(), cols, rows, dx.data_ptr(), xs, got.data_ptr(), ys, m, stream.handle)
    stream.synchronize()
    assert np.array_equal(got.cpu().numpy()[:, :rows].view(np.uint32), want.cpu().numpy()[:, :rows].view(np.uint32))


def test_static_workspace_refuses_what_does_not_fit():
    import torch
    assert torch.cuda.is_available(), "no GPU visible"
    sz.init(0)
    ty, cols, rows, m = sz.EXL3(3), 2048, 151936 // 128 * 128, 8     # a head-sized product: 19 MB of partial sums
    assert sz.matvec_cols_scratch(ty, cols, rows, m) > sz.STATIC_WORKSPACE_BYTES
    with pytest.raises(sz.SzError, match="static one holds"):
        sz.matvec_cols_static(ty, 256, cols, rows, 256, cols, 256, rows, m)   # refused before any address is used
