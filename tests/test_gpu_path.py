"""GPU parity tests: every kernel of the verify path, called through the C ABI, against the CPU oracle on the same seeded
inputs.  Bars: dequantized values, routing ids, arg-max ids and accepted counts bit-exact; f32 outputs within 1e-3
relative L2 (the reference's own tighter bounds are asserted where it states one: 1e-4 * sum|w x| for GGUF products,
crates/shadowzero-cuda/tests/matvec.rs:95; 2e-4 * max|y| for EXL3, tests/exl3.rs:45)."""
import numpy as np
import pytest

import golden_io
import oracle_lib as O
import shadow_engine_amd as sz
from shadow_engine_amd import synth

pytestmark = pytest.mark.gpu

REL_L2 = 1e-3


@pytest.fixture(scope="module")
def gpu():
    import torch
    assert torch.cuda.is_available(), "no GPU visible"
    sz.init(0)
    return torch


def dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def rel_l2(got, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return float(np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-30))


def bits(a):
    return np.asarray(a, np.float32).view(np.uint32)


def test_device_and_registry(gpu):
    print("device:", sz.device_name(), flush=True)
    assert sz.device_count() >= 1
    assert len(sz.kernels()) > 30


# ------------------------------------------------------------------------------------------------------------ dequant
@pytest.mark.parametrize("ty", [sz.Q8_0, sz.IQ3_S])
def test_gguf_dequant_is_bit_exact(gpu, ty):
    rng = np.random.default_rng(ty)
    rows, cols = 24, 1024
    w = synth.q8_0_matrix(rng, rows, cols) if ty == sz.Q8_0 else synth.iq3_s_matrix(rng, rows, cols)
    if ty == sz.IQ3_S:   # the real blocks too
        w = np.concatenate([w] + [r[2] for r in golden_io.iq3s_records()])
        rows, cols = w.size // 110, 256
    dw = dev(gpu, w)
    out = gpu.empty(rows * cols, dtype=gpu.float32, device="cuda")
    sz.dequantize(ty, dw.data_ptr(), out.data_ptr(), cols, rows)
    gpu.cuda.synchronize()
    got = out.cpu().numpy()
    want = O.dequantize(ty, w)
    assert np.array_equal(bits(got), bits(want))
    if ty == sz.IQ3_S:
        for i, rec in enumerate(golden_io.iq3s_records()):
            assert np.array_equal(bits(got[(rows - 8 + i) * 256:(rows - 7 + i) * 256]), rec[3])


def test_exl3_codebook_is_bit_exact(gpu):
    out = gpu.empty(65536, dtype=gpu.float32, device="cuda")
    sz.exl3_codebook(out.data_ptr())
    gpu.cuda.synchronize()
    assert np.array_equal(bits(out.cpu().numpy()), bits(O.exl3_codebook_all(2)))


@pytest.mark.parametrize("bits_k", range(1, 9))
def test_exl3_decode_is_bit_exact(gpu, bits_k):
    rng = np.random.default_rng(40 + bits_k)
    inf, outf = 256, 384
    blob = synth.exl3_blob(rng, inf, outf, bits_k)
    db = dev(gpu, blob)
    out = gpu.empty(inf * outf, dtype=gpu.float32, device="cuda")
    sz.dequantize(sz.EXL3(bits_k), db.data_ptr(), out.data_ptr(), inf, outf)
    gpu.cuda.synchronize()
    want = O.exl3_reconstruct(inf, outf, bits_k, blob, inner=True)
    assert np.array_equal(bits(out.cpu().numpy()), bits(want.ravel()))


@pytest.mark.parametrize("bits_k", [1, 2, 3])
def test_exl3_half_rates_decode_bit_exact_and_multiply(gpu, bits_k):
    """K + 1/2 bits a weight (positions alternate K and K + 1 bits, exl3.rs:164; type ids 1030 + K): every decoded weight
    bit-exact, the product through Backend::matvec and matvec_cols within the reference's 2e-4 max|y|, a batch bit-equal to
    single-input launches.  (The fused layer at these rates is among the cases of test_moe_layer_verify_matches_the_oracle.)"""
    rng = np.random.default_rng(70 + bits_k)
    inf, outf = 384, 256
    ty = sz.EXL3_HALF(bits_k)
    blob = synth.exl3_blob(rng, inf, outf, bits_k, half=True)
    db = dev(gpu, blob)
    out = gpu.empty(inf * outf, dtype=gpu.float32, device="cuda")
    sz.dequantize(ty, db.data_ptr(), out.data_ptr(), inf, outf)
    gpu.cuda.synchronize()
    assert np.array_equal(bits(out.cpu().numpy()), bits(O.exl3_reconstruct(inf, outf, bits_k, blob, half=True, inner=True).ravel()))
    x = rng.uniform(-1, 1, (5, inf)).astype(np.float32)
    want = np.stack([O.exl3_matvec(inf, outf, bits_k, blob, x[j], half=True) for j in range(5)])
    be = sz.GpuBackend()
    got = be.matvec(ty, inf, outf, blob, None, x[0])
    assert np.max(np.abs(got - want[0])) <= 2e-4 * np.max(np.abs(want[0])) and rel_l2(got, want[0]) <= REL_L2
    dx = dev(gpu, x)
    nsb = sz.matvec_cols_scratch(ty, inf, outf, 5)
    scratch = gpu.empty(max(nsb, 16), dtype=gpu.uint8, device="cuda")
    y = gpu.zeros((5, outf), dtype=gpu.float32, device="cuda")
    sz.matvec_cols(ty, db.data_ptr(), inf, outf, dx.data_ptr(), inf, y.data_ptr(), outf, 5, scratch.data_ptr(), nsb)
    gpu.cuda.synchronize()
    ys = y.cpu().numpy()
    assert np.array_equal(bits(ys[0]), bits(got))
    for j in range(5):
        assert np.max(np.abs(ys[j] - want[j])) <= 2e-4 * np.max(np.abs(want[j]))


def test_exl3_decode_of_the_real_tensors_is_bit_exact(gpu):
    for inf, outf, k, blob, _, _ in golden_io.exl3_real_tensors():      # K = 2 and K = 4
        db = dev(gpu, blob)
        out = gpu.empty(inf * outf, dtype=gpu.float32, device="cuda")
        sz.dequantize(sz.EXL3(k), db.data_ptr(), out.data_ptr(), inf, outf)
        gpu.cuda.synchronize()
        assert np.array_equal(bits(out.cpu().numpy()), bits(O.exl3_reconstruct(inf, outf, k, blob, inner=True).ravel()))


# ---------------------------------------------------------------------------------------------- Backend::matvec (B1)
def gguf_bound(ty, cols, rows, w, x):
    dense = O.dequantize(ty, w).reshape(rows, cols).astype(np.float64)
    return 1e-4 * (np.abs(dense) * np.abs(x.astype(np.float64))[None, :]).sum(axis=1) + 1e-6


@pytest.mark.parametrize("ty,rows,cols", [(sz.Q8_0, 1024, 2048), (sz.IQ3_S, 1024, 2048), (sz.IQ3_S, 2048, 512), (sz.Q8_0, 100, 96),
                                          (sz.IQ3_S, 7, 768), (sz.Q8_0, 33, 4096)])
def test_backend_matvec_gguf(gpu, ty, rows, cols):
    rng = np.random.default_rng(rows * 7 + cols)
    w = synth.q8_0_matrix(rng, rows, cols) if ty == sz.Q8_0 else synth.iq3_s_matrix(rng, rows, cols)
    x = rng.normal(size=cols).astype(np.float32)
    be = sz.GpuBackend()
    got = be.matvec(ty, cols, rows, w, None, x)
    want = O.matvec(ty, cols, rows, w, x)
    assert np.all(np.abs(got - want) <= gguf_bound(ty, cols, rows, w, x))
    assert rel_l2(got, want) <= REL_L2
    # a keyed tensor is uploaded once (backend.rs:63-75)
    be.matvec(ty, cols, rows, w, "t", x)
    n = be.uploads
    got2 = be.matvec(ty, cols, rows, w, "t", x)
    assert be.uploads == n and be.resident_bytes == w.size and np.array_equal(got2, got)


@pytest.mark.parametrize("bits_k,inf,outf", [(2, 2048, 512), (3, 2048, 512), (4, 512, 2048), (3, 512, 2048), (1, 256, 128), (5, 640, 256),
                                             (6, 384, 384), (7, 128, 128), (8, 256, 256)])
def test_backend_matvec_exl3(gpu, bits_k, inf, outf):
    rng = np.random.default_rng(bits_k * 1000 + inf)
    blob = synth.exl3_blob(rng, inf, outf, bits_k)
    x = rng.uniform(-1, 1, inf).astype(np.float32)
    be = sz.GpuBackend()
    got = be.matvec(sz.EXL3(bits_k), inf, outf, blob, None, x)
    want = O.exl3_matvec(inf, outf, bits_k, blob, x)
    assert np.abs(got - want).max() <= 2e-4 * max(np.abs(want).max(), 1e-6)
    assert rel_l2(got, want) <= REL_L2


def test_backend_matvec_on_the_real_exl3_tensors(gpu):
    for inf, outf, k, blob, _, _ in golden_io.exl3_real_tensors():
        x = np.random.default_rng(5).normal(size=inf).astype(np.float32)
        got = sz.GpuBackend().matvec(sz.EXL3(k), inf, outf, blob, "gate%d" % k, x)
        want = O.exl3_matvec(inf, outf, k, blob, x)
        assert np.abs(got - want).max() <= 2e-4 * np.abs(want).max() and rel_l2(got, want) <= REL_L2


def test_backend_refuses_what_it_cannot_run(gpu):
    be = sz.GpuBackend()
    with pytest.raises(sz.SzError, match="no matvec kernel"):
        be.matvec(12, 256, 4, np.zeros(4 * 144, np.uint8), None, np.zeros(256, np.float32))      # Q4_K
    with pytest.raises(sz.SzError, match="bytes for"):
        be.matvec(sz.Q8_0, 64, 4, np.zeros(100, np.uint8), None, np.zeros(64, np.float32))
    with pytest.raises(sz.SzError, match="multiples of 128"):
        be.matvec(sz.EXL3(3), 100, 128, np.zeros(10, np.uint8), None, np.zeros(100, np.float32))


# ----------------------------------------------------------------------------------------------------- matvec_cols
@pytest.mark.parametrize("ty", [sz.Q8_0, sz.IQ3_S, sz.EXL3(3)])
def test_cols_matches_single_inputs_bitwise_and_the_oracle(gpu, ty):
    # crates/shadowzero-cuda/tests/matvec.rs:237: every input of a cols launch gives the bits a single-input launch gives
    rng = np.random.default_rng(ty)
    cols, rows = 2048, 512
    if ty >= 1000:
        w = synth.exl3_blob(rng, cols, rows, ty - 1020)
    else:
        w = synth.q8_0_matrix(rng, rows, cols) if ty == sz.Q8_0 else synth.iq3_s_matrix(rng, rows, cols)
    dw = dev(gpu, w)
    xs, ys = cols + 64, rows + 32                       # padded strides
    x = rng.normal(size=(8, xs)).astype(np.float32)
    dx = dev(gpu, x)
    nsb = sz.matvec_cols_scratch(ty, cols, rows, 8)
    scratch = gpu.empty(max(nsb, 16), dtype=gpu.uint8, device="cuda")
    singles = []
    for j in range(8):
        y1 = gpu.zeros(ys, dtype=gpu.float32, device="cuda")
        sz.matvec_cols(ty, dw.data_ptr(), cols, rows, dx[j].data_ptr(), xs, y1.data_ptr(), ys, 1, scratch.data_ptr(), nsb)
        gpu.cuda.synchronize()
        singles.append(y1.cpu().numpy()[:rows])
    for m in range(1, 9):
        y = gpu.zeros((8, ys), dtype=gpu.float32, device="cuda")
        sz.matvec_cols(ty, dw.data_ptr(), cols, rows, dx.data_ptr(), xs, y.data_ptr(), ys, m, scratch.data_ptr(), nsb)
        gpu.cuda.synchronize()
        got = y.cpu().numpy()
        for j in range(m):
            assert np.array_equal(bits(got[j, :rows]), bits(singles[j])), f"m={m} input {j}"
        assert not got[m:].any() and not got[:, rows:].any()
    for j in range(8):
        want = O.matvec(ty if ty < 1000 else O.exl3_type(ty - 1020), cols, rows, w, x[j, :cols])
        assert rel_l2(singles[j], want) <= REL_L2


@pytest.mark.parametrize("ty,rows,cols", [(sz.Q8_0, 100, 96), (sz.IQ3_S, 50, 768), (sz.Q8_0, 41, 3072), (sz.IQ3_S, 9, 4352), (sz.Q8_0, 70, 1280)])
def test_cols_on_rows_of_any_number_of_units(gpu, ty, rows, cols):
    """Rows whose 32-weight units neither divide a wave's 64 lanes nor fill whole waves: every input gives the bits of a
    single-input launch, and the oracle's values."""
    rng = np.random.default_rng(rows + cols)
    w = synth.q8_0_matrix(rng, rows, cols) if ty == sz.Q8_0 else synth.iq3_s_matrix(rng, rows, cols)
    dw = dev(gpu, w)
    x = rng.normal(size=(5, cols)).astype(np.float32)
    dx = dev(gpu, x)
    singles = gpu.zeros((5, rows), dtype=gpu.float32, device="cuda")
    for j in range(5):
        sz.matvec_cols(ty, dw.data_ptr(), cols, rows, dx[j].data_ptr(), cols, singles[j].data_ptr(), rows, 1)
    y = gpu.zeros((5, rows), dtype=gpu.float32, device="cuda")
    sz.matvec_cols(ty, dw.data_ptr(), cols, rows, dx.data_ptr(), cols, y.data_ptr(), rows, 5)
    gpu.cuda.synchronize()
    assert np.array_equal(bits(y.cpu().numpy()), bits(singles.cpu().numpy()))
    for j in range(5):
        assert rel_l2(y[j].cpu().numpy(), O.matvec(ty, cols, rows, w, x[j])) <= REL_L2


def dense_matrix(rng, ty, rows, cols):
    """An unquantized matrix as stored bytes (F32, F16 or BF16 = the upper half of the f32, rounded to nearest even)."""
    w = (rng.normal(size=(rows, cols)) * 0.05).astype(np.float32)
    if ty == sz.F32:
        return w.view(np.uint8).ravel()
    if ty == sz.F16:
        return w.astype(np.float16).view(np.uint8).ravel()
    b = w.view(np.uint32)
    return ((b + 0x7fff + ((b >> 16) & 1)) >> 16).astype(np.uint16).view(np.uint8).ravel()


@pytest.mark.parametrize("ty", [sz.F32, sz.F16, sz.BF16])
@pytest.mark.parametrize("rows,cols", [(513, 2048), (1, 2048), (7, 260), (130, 4)])
def test_unquantized_products_match_the_oracle(gpu, ty, rows, cols):
    """The router's and the shared gate's kind of matrix (quant.rs:237-239) through matvec_cols and Backend::matvec: within
    1e-4 * sum|w x| of the oracle's f64 row dots, every input of a batch bit-equal to a single-input launch, ragged shapes."""
    rng = np.random.default_rng(ty * 97 + rows + cols)
    w = dense_matrix(rng, ty, rows, cols)
    dw = dev(gpu, w)
    xs, ys = cols + 8, rows + 3
    x = rng.normal(size=(8, xs)).astype(np.float32)
    dx = dev(gpu, x)
    singles = []
    for j in range(8):
        y1 = gpu.zeros(ys, dtype=gpu.float32, device="cuda")
        sz.matvec_cols(ty, dw.data_ptr(), cols, rows, dx[j].data_ptr(), xs, y1.data_ptr(), ys, 1, 0, 0)
        gpu.cuda.synchronize()
        singles.append(y1.cpu().numpy())
        assert not singles[-1][rows:].any()
        want = O.matvec(ty, cols, rows, w, x[j, :cols])
        assert np.all(np.abs(singles[-1][:rows] - want) <= gguf_bound(ty, cols, rows, w, x[j, :cols]))
    for m in (2, 5, 8):
        y = gpu.zeros((8, ys), dtype=gpu.float32, device="cuda")
        sz.matvec_cols(ty, dw.data_ptr(), cols, rows, dx.data_ptr(), xs, y.data_ptr(), ys, m, 0, 0)
        gpu.cuda.synchronize()
        got = y.cpu().numpy()
        for j in range(m):
            assert np.array_equal(bits(got[j]), bits(singles[j])), f"m={m} input {j}"
        assert not got[m:].any()
    be = sz.GpuBackend()
    assert np.array_equal(bits(be.matvec(ty, cols, rows, w, "router", x[0, :cols])), bits(singles[0][:rows]))


# --------------------------------------------------------------------------------------------------- the MoE layer
def build_layer(torch, rng, ty, hidden, ff, ne, with_shared=True, lead=0, gap=0):
    """ne experts + one shared expert as one device buffer; returns (device tensor, stride, host blobs, shared blob).  The
    first expert starts `lead` bytes into the buffer and an expert's projections lie `gap` bytes apart (0, 0: contiguous
    [gate|up|down] blobs from the buffer's start); the bytes in between are 0xEE."""
    blobs = [synth.expert_blob(rng, ty, hidden, ff) for _ in range(ne)]
    gb, ub, _ = synth.expert_bytes(ty, hidden, ff)
    stride = (blobs[0].size + 2 * gap + 255) // 256 * 256
    buf = np.full(lead + (ne + 1) * stride, 0xEE, np.uint8)
    shared = synth.expert_blob(rng, ty, hidden, ff) if with_shared else None
    for e, b in enumerate(blobs + ([shared] if with_shared else [])):
        at = lead + e * stride
        for lo, hi, shift in ((0, gb, 0), (gb, gb + ub, gap), (gb + ub, b.size, 2 * gap)):
            buf[at + lo + shift:at + hi + shift] = b[lo:hi]
    return dev(torch, buf), stride, blobs, shared


def oracle_layer(ty, hidden, ff, k, blobs, shared, logits, sgl, u):
    oty = ty if ty < 1000 else O.exl3_type(ty - 1030, half=True) if ty > 1030 else O.exl3_type(ty - 1020)
    shape = O.expert_shape(oty, oty, hidden, ff)
    ys, idxs, ws = [], [], []
    for j in range(u.shape[0]):
        y, idx, w = O.moe_token(shape, blobs, k, logits[j], u[j], shape if shared is not None else None, shared,
                                float(sgl[j]) if shared is not None else 0.0)
        ys.append(y), idxs.append(idx), ws.append(w)
    return np.stack(ys), np.stack(idxs), np.stack(ws)


@pytest.mark.parametrize("ty,hidden,ff,ne,k,m,shared", [
    (sz.IQ3_S, 2048, 512, 64, 10, 1, True),        # the decode shape of one layer (batch 1), fewer experts
    (sz.IQ3_S, 2048, 512, 32, 10, 4, True),        # a verify batch; 32 experts so that tokens share experts
    (sz.Q8_0, 512, 256, 16, 4, 8, False),          # no shared expert, eight rows, many shared experts
    (sz.EXL3(3), 2048, 512, 48, 10, 4, True),
    (sz.EXL3(2), 2048, 512, 24, 10, 3, True),
    (sz.EXL3(4), 512, 256, 8, 4, 8, True),         # every expert used by several tokens (groups of up to 4, split groups)
    (sz.EXL3(3), 256, 256, 6, 6, 2, False),        # k = ne: every expert chosen
    (sz.EXL3(3), 512, 1024, 12, 4, 3, True),       # ff > 512: the down product's inputs are split, launch 3 sums the partials
    (sz.EXL3(2), 256, 256, 20, 16, 2, True),       # k = 16, the most the session takes: the shared expert shares a wave
    (sz.EXL3(4), 3072, 768, 8, 3, 5, True),        # hidden not a multiple of 1024: a launch-1 workgroup with idle waves
    (sz.IQ3_S, 1024, 1024, 24, 16, 2, True),
    (sz.EXL3(1), 512, 256, 8, 3, 2, True),         # the other bit rates of the fused layer kernels
    (sz.EXL3(5), 512, 256, 8, 3, 4, True),
    (sz.EXL3(6), 256, 512, 6, 2, 3, False),
    (sz.EXL3(7), 256, 256, 6, 2, 1, True),
    (sz.EXL3(8), 1024, 256, 6, 3, 4, True),
    (sz.EXL3_HALF(1), 512, 256, 8, 3, 2, True),    # K + 1/2 bits a weight
    (sz.EXL3_HALF(2), 2048, 512, 12, 4, 4, True),
    (sz.EXL3_HALF(3), 256, 512, 6, 2, 3, False),
    (sz.EXL3(3), 2048, 512, 512, 10, 8, True),     # the benchmark's layer at the most rows a verify batch takes (MAX_VERIFY)
    (sz.EXL3(4), 2048, 512, 512, 10, 5, True),
    (sz.Q8_0, 3072, 768, 8, 3, 5, True),           # rows of 96 and 24 units: a wave's lanes do not divide into whole rows
    (sz.IQ3_S, 3072, 1280, 8, 3, 2, True),
    (sz.IQ3_S, 768, 2304, 6, 2, 3, False),
    (sz.Q8_0, 4096, 1024, 6, 2, 2, True),          # rows of 128 units: the inputs come in two column chunks
])
def test_moe_layer_verify_matches_the_oracle(gpu, ty, hidden, ff, ne, k, m, shared):
    run_moe_layer_case(gpu, ty, hidden, ff, ne, k, m, shared)


@pytest.mark.parametrize("ty,hidden,ff,ne,k,m,shared", [
    (sz.IQ3_S, 2048, 512, 32, 10, 4, True),        # tokens share experts: groups of several inputs
    (sz.Q8_0, 512, 256, 16, 4, 8, False),
    (sz.IQ3_S, 768, 1280, 6, 3, 4, True),
])
def test_moe_layer_verify_planned_form_matches_the_oracle(gpu, monkeypatch, ty, hidden, ff, ne, k, m, shared):
    """The GGUF layer through the device planner and the grouped products (route_plan_res_small, matvec_grouped_*, swiglu),
    the form that shares one weight decode between the tokens of an expert."""
    monkeypatch.setenv("SHADOWZERO_GGUF_PLANNED", "1")
    run_moe_layer_case(gpu, ty, hidden, ff, ne, k, m, shared)


@pytest.mark.parametrize("ty,hidden,ff,ne,k,shared", [
    (sz.IQ3_S, 2048, 512, 96, 10, True),           # the decode shape
    (sz.IQ3_S, 1024, 256, 24, 16, True),           # k = 16, the most the session takes; 8 units a down row
    (sz.IQ3_S, 512, 1024, 8, 3, True),             # 32 units a down row
    (sz.IQ3_S, 512, 256, 8, 3, False),             # no shared expert: rank 0's workgroup computes the weights; 8 units a down row
    (sz.Q8_0, 1024, 512, 12, 4, True),
    (sz.Q8_0, 512, 256, 16, 4, False),
    (sz.Q8_0, 2048, 2048, 6, 2, True),             # too large for launch 2's staging: the call falls back to three launches
])
def test_one_token_layer_in_two_launches(gpu, monkeypatch, ty, hidden, ff, ne, k, shared):
    """A single token takes the two-launch form (act and the routing weights out of launch 1, the down rows of all experts and
    the rank-order sum in launch 2): against the oracle, with masked experts (fewer finite logits than k, and none but one),
    and against the three-launch form of the same call (the same sums; the weights may differ in the last bit, launch 1 sums
    only the chosen experts' exponentials)."""
    rng = np.random.default_rng(ty * 7 + hidden + k)
    dbuf, stride, blobs, sh = build_layer(gpu, rng, ty, hidden, ff, ne, shared)
    s = sz.Session(hidden, ff, ne, k, 1, 0, 8)
    s.set_layer(0, ty, dbuf.data_ptr(), stride, ty if shared else 0, dbuf.data_ptr() + ne * stride if shared else 0)
    for finite in (ne, max(1, k - 1), 1):
        u = rng.normal(size=(1, hidden)).astype(np.float32)
        logits = rng.normal(size=(1, ne)).astype(np.float32)
        if finite < ne:
            row = np.full(ne, -np.inf, np.float32)
            keep = rng.choice(ne, finite, replace=False)
            row[keep] = logits[0, keep]
            logits[0] = row
        sgl = rng.normal(size=1).astype(np.float32)
        du, dl, dg = dev(gpu, u), dev(gpu, logits), dev(gpu, sgl)
        dy = gpu.full((1, hidden), 7.0, dtype=gpu.float32, device="cuda")
        s.moe_layer_verify(0, 1, du.data_ptr(), dl.data_ptr(), dg.data_ptr(), dy.data_ptr())
        gpu.cuda.synchronize()
        got = dy.cpu().numpy()
        idx, w = s.last_route(1)
        want, widx, ww = oracle_layer(ty, hidden, ff, k, blobs, sh, logits, sgl, u)
        assert np.array_equal(idx, widx), f"{finite} finite logits"
        assert np.allclose(w, ww, rtol=2e-6, atol=0)
        assert rel_l2(got[0], want[0]) <= REL_L2, f"{finite} finite logits: {rel_l2(got[0], want[0])}"
        monkeypatch.setenv("SHADOWZERO_GGUF_THREE_LAUNCH", "1")
        dy3 = gpu.zeros((1, hidden), dtype=gpu.float32, device="cuda")
        s.moe_layer_verify(0, 1, du.data_ptr(), dl.data_ptr(), dg.data_ptr(), dy3.data_ptr())
        gpu.cuda.synchronize()
        monkeypatch.delenv("SHADOWZERO_GGUF_THREE_LAUNCH")
        assert rel_l2(dy3.cpu().numpy()[0], got[0]) <= 2e-7, f"{finite} finite logits: the two forms differ"
        idx3, w3 = s.last_route(1)
        assert np.array_equal(idx3, idx) and np.allclose(w3, w, rtol=2e-7, atol=0)


@pytest.mark.parametrize("ty", [sz.EXL3(3), sz.IQ3_S])
def test_moe_layer_with_masked_experts_matches_the_oracle(gpu, ty):
    """Logits of -inf (the reference masks the experts it skips that way, session.rs:6205): a row with fewer finite logits than
    k, a row with exactly k, a row with one; the chosen ids, their weights (0 for a masked expert) and y against the oracle."""
    rng = np.random.default_rng(77)
    hidden, ff, ne, k, m = 256, 256, 24, 4, 4
    dbuf, stride, blobs, sh = build_layer(gpu, rng, ty, hidden, ff, ne, True)
    s = sz.Session(hidden, ff, ne, k, 1, 0, 8)
    s.set_layer(0, ty, dbuf.data_ptr(), stride, ty, dbuf.data_ptr() + ne * stride)
    u = rng.normal(size=(m, hidden)).astype(np.float32)
    logits = rng.normal(size=(m, ne)).astype(np.float32)
    for j, finite in ((0, 2), (1, k), (2, 1)):
        keep = rng.choice(ne, finite, replace=False)
        row = np.full(ne, -np.inf, np.float32)
        row[keep] = logits[j, keep]
        logits[j] = row
    sgl = rng.normal(size=m).astype(np.float32)
    du, dl, dg = dev(gpu, u), dev(gpu, logits), dev(gpu, sgl)
    dy = gpu.zeros((m, hidden), dtype=gpu.float32, device="cuda")
    s.moe_layer_verify(0, m, du.data_ptr(), dl.data_ptr(), dg.data_ptr(), dy.data_ptr())
    gpu.cuda.synchronize()
    got = dy.cpu().numpy()
    idx, w = s.last_route(m)
    want, widx, ww = oracle_layer(ty, hidden, ff, k, blobs, sh, logits, sgl, u)
    assert np.array_equal(idx, widx)
    assert np.allclose(w, ww, rtol=2e-6, atol=0)
    assert np.all(np.isfinite(got))
    for j in range(m):
        assert rel_l2(got[j], want[j]) <= REL_L2, f"row {j}: {rel_l2(got[j], want[j])}"


# What the matrix-core forms of the EXL3 layer are held to (sz_session_set_expert_mode): mode 1 multiplies the codebook's own
# f16 values and differs from the exact kernels in the order of the f32 additions and in the 22 bits kept of an input; mode 2
# leaves out every weight's rounding to f16 (half a unit in its last place) and is held to the path's 1e-3.  Measured worst
# cases over the cases below: mode 1 3.4e-7 relative L2 and 4.2e-7 of the largest output; mode 2 4.2e-4 and 5.5e-4 (the
# reference holds its own tensor-core EXL3 kernels to 3e-3 of the largest output, crates/shadowzero-cuda/tests/exl3.rs:201).
# Mode 3 keeps the exact decode and the exact launches but rounds every rotated input to f16 (11 bits) so that two products
# go into one instruction: held to the path's 1e-3 as well.
MODE_BOUND = {0: REL_L2, 1: 2e-6, 2: REL_L2, 3: REL_L2}


@pytest.mark.parametrize("mode", [1, 2, 3])
@pytest.mark.parametrize("ty,hidden,ff,ne,k,m,shared", [
    (sz.EXL3(3), 2048, 512, 48, 10, 4, True),
    (sz.EXL3(2), 2048, 512, 24, 10, 3, True),
    (sz.EXL3(4), 512, 256, 8, 4, 8, True),         # every expert used by several tokens: items of up to 8 rows
    (sz.EXL3(3), 256, 256, 6, 6, 2, False),        # k = ne: every expert chosen; no shared expert
    (sz.EXL3(3), 512, 1024, 12, 4, 3, True),       # ff > 512: the down product's inputs are split, launch 3 sums the partials
    (sz.EXL3(2), 256, 256, 20, 16, 2, True),       # k = 16
    (sz.EXL3(4), 3072, 768, 8, 3, 5, True),        # hidden not a multiple of 1024, ff not of 512: workgroups with idle waves; items of 5 rows
    (sz.EXL3(1), 512, 256, 8, 3, 2, True),         # the other bit rates
    (sz.EXL3(5), 512, 256, 8, 3, 4, True),
    (sz.EXL3(6), 256, 512, 6, 2, 3, False),        # K > 5: a tile's windows need two funnel shifts
    (sz.EXL3(7), 256, 256, 6, 2, 1, True),
    (sz.EXL3(8), 1024, 256, 6, 3, 4, True),
    (sz.EXL3(3), 2048, 512, 512, 10, 8, True),     # the benchmark's layer at the most rows a verify batch takes
    (sz.EXL3(4), 2048, 512, 512, 10, 4, True),     # and at the rows the configurations name
])
def test_moe_layer_on_the_matrix_cores(gpu, mode, ty, hidden, ff, ne, k, m, shared):
    worst = run_moe_layer_case(gpu, ty, hidden, ff, ne, k, m, shared, mode)
    print(f"mode {mode}: worst relative L2 {worst[0]:.3g}, worst max|dy| / max|y| {worst[1]:.3g}", flush=True)


def run_moe_layer_case(gpu, ty, hidden, ff, ne, k, m, shared, mode=0):
    rng = np.random.default_rng(ty * 31 + ne + m)
    dbuf, stride, blobs, sh = build_layer(gpu, rng, ty, hidden, ff, ne, shared)
    s = sz.Session(hidden, ff, ne, k, 1, 0, 8)
    s.set_expert_mode(mode)
    s.set_layer(0, ty, dbuf.data_ptr(), stride, ty if shared else 0, dbuf.data_ptr() + ne * stride if shared else 0)
    u = rng.normal(size=(m, hidden)).astype(np.float32)
    logits = rng.normal(size=(m, ne)).astype(np.float32)
    sgl = rng.normal(size=m).astype(np.float32)
    du, dl, dg = dev(gpu, u), dev(gpu, logits), dev(gpu, sgl)
    dy = gpu.zeros((m, hidden), dtype=gpu.float32, device="cuda")
    s.moe_layer_verify(0, m, du.data_ptr(), dl.data_ptr(), dg.data_ptr(), dy.data_ptr())
    gpu.cuda.synchronize()
    got = dy.cpu().numpy()
    idx, w = s.last_route(m)
    want, widx, ww = oracle_layer(ty, hidden, ff, k, blobs, sh, logits, sgl, u)
    assert np.array_equal(idx, widx), "expert routing must be bit-exact (ids and order)"
    assert np.allclose(w, ww, rtol=2e-6, atol=0)
    for j in range(m):
        assert rel_l2(got[j], want[j]) <= MODE_BOUND[mode], f"row {j}: {rel_l2(got[j], want[j])}"
    # twice the same bits (deterministic reductions)
    dy2 = gpu.zeros((m, hidden), dtype=gpu.float32, device="cuda")
    s.moe_layer_verify(0, m, du.data_ptr(), dl.data_ptr(), dg.data_ptr(), dy2.data_ptr())
    gpu.cuda.synchronize()
    assert np.array_equal(bits(dy2.cpu().numpy()), bits(got))
    return (max(rel_l2(got[j], want[j]) for j in range(m)), max(float(np.abs(got[j] - want[j]).max() / np.abs(want[j]).max()) for j in range(m)))


@pytest.mark.parametrize("ty,hidden,ff,ne,k,m,mode", [
    (sz.EXL3(3), 2048, 512, 24, 10, 4, 0), (sz.EXL3(2), 512, 256, 8, 3, 8, 0), (sz.EXL3(4), 512, 1024, 8, 3, 3, 0), (sz.EXL3_HALF(2), 512, 256, 8, 3, 2, 0),
    (sz.EXL3(3), 512, 256, 8, 3, 5, 1), (sz.EXL3(4), 512, 256, 8, 3, 4, 2), (sz.EXL3(3), 512, 256, 8, 3, 4, 3),
    (sz.IQ3_S, 2048, 512, 16, 10, 1, 0), (sz.IQ3_S, 512, 256, 8, 3, 4, 0), (sz.Q8_0, 512, 256, 8, 3, 1, 0), (sz.Q8_0, 512, 256, 8, 3, 6, 0),
])
def test_a_layer_with_spaced_projections_gives_the_bits_of_the_contiguous_one(gpu, ty, hidden, ff, ne, k, m, mode):
    """sz_session_set_layer_spaced: the same experts with a gap between their projections and the first one off the buffer's
    start (for an EXL3 layer the spacing that puts every trellis on a 128-byte line, for a GGUF layer an arbitrary one) go
    through the same kernels in the same order: layer outputs, routing and a prefill chunk equal the contiguous layout's bit
    for bit.  The layouts are also told apart: a stride too small for the gaps is refused."""
    lead, gap = sz.layer_spacing(ty, hidden, ff) if ty >= 1000 else (36, 60)
    assert (lead, gap) == ((124, 124) if ty >= 1000 else (36, 60))
    outs = []
    for ld, gp in ((0, 0), (lead, gap)):
        rng = np.random.default_rng(ty + 7 * m)
        dbuf, stride, blobs, sh = build_layer(gpu, rng, ty, hidden, ff, ne, True, ld, gp)
        if ty >= 1000 and gp:   # where the trellises lie: 2 (in + out) + 4 bytes into each blob
            gb = synth.expert_bytes(ty, hidden, ff)[0]
            assert all((dbuf.data_ptr() + ld + e * stride + i * (gb + gp) + 2 * (hidden + ff) + 4) % 128 == 0 for e in (0, ne) for i in range(3))
        s = sz.Session(hidden, ff, ne, k, 1, 0, 8)
        s.set_expert_mode(mode)
        base = dbuf.data_ptr() + ld
        if gp:
            with pytest.raises(sz.SzError, match="stride is smaller"):
                s.set_layer(0, ty, base, blobs[0].size, ty, base + ne * stride, gap=gp)
        s.set_layer(0, ty, base, stride, ty, base + ne * stride, gap=gp)
        u = rng.normal(size=(m, hidden)).astype(np.float32)
        logits = rng.normal(size=(m, ne)).astype(np.float32)
        sgl = rng.normal(size=m).astype(np.float32)
        du, dl, dg = dev(gpu, u), dev(gpu, logits), dev(gpu, sgl)
        dy = gpu.zeros((m, hidden), dtype=gpu.float32, device="cuda")
        s.moe_layer_verify(0, m, du.data_ptr(), dl.data_ptr(), dg.data_ptr(), dy.data_ptr())
        gpu.cuda.synchronize()
        got = [bits(dy.cpu().numpy()), *s.last_route(m)]
        if mode == 0 and (ty == sz.IQ3_S or (1020 < ty < 1030)) and hidden % 256 == 0 and ff % 256 == 0 and ff <= 512:
            tokens = 40
            x = rng.normal(size=(tokens, hidden)).astype(np.float32)
            pl = rng.normal(size=(tokens, ne)).astype(np.float32)
            pg = rng.normal(size=tokens).astype(np.float32)
            dx, dpl, dpg = dev(gpu, x), dev(gpu, pl), dev(gpu, pg)
            py = gpu.zeros((tokens, hidden), dtype=gpu.float32, device="cuda")
            s.moe_prefill_chunk(0, tokens, dx.data_ptr(), dpl.data_ptr(), dpg.data_ptr(), py.data_ptr())
            gpu.cuda.synchronize()
            got.append(bits(py.cpu().numpy()))
        outs.append(got)
        if (ld, gp) == (0, 0):   # the contiguous run is also right: against the oracle
            want, widx, ww = oracle_layer(ty, hidden, ff, k, blobs, sh, logits, sgl, u)
            assert np.array_equal(got[1], widx) and all(rel_l2(dy.cpu().numpy()[j], want[j]) <= MODE_BOUND[mode] for j in range(m))
    assert len(outs[0]) == len(outs[1]) and all(np.array_equal(a, b) for a, b in zip(outs[0], outs[1]))


@pytest.mark.parametrize("ty,hidden,ff,ne,k,m", [
    (sz.EXL3(3), 2048, 512, 40, 10, 4),
    (sz.EXL3(2), 1024, 512, 16, 6, 8),
    (sz.EXL3_HALF(2), 512, 256, 12, 4, 4),
    (sz.IQ3_S, 2048, 512, 24, 10, 4),
    (sz.Q8_0, 1024, 512, 12, 4, 8),
    (sz.IQ3_S, 2048, 512, 24, 10, 1),              # one token: the two-launch form, whose first launch also selects all k on a wave of its own
    (sz.Q8_0, 1024, 512, 12, 4, 1),
])
def test_moe_layer_over_seeds_and_logit_kinds(gpu, ty, hidden, ff, ne, k, m):
    """One set of experts, then several batches against the oracle: normal logits, coarse logits (exact ties, the lower index
    must win) and near-ties a few units in the last place apart among the chosen experts, so that every path of the
    selection inside the layer's first launch feeds real expert products."""
    for seed in range(2):
        rng = np.random.default_rng(1000 * seed + ty + m)
        dbuf, stride, blobs, sh = build_layer(gpu, rng, ty, hidden, ff, ne, True)
        s = sz.Session(hidden, ff, ne, k, 1, 0, 8)
        s.set_layer(0, ty, dbuf.data_ptr(), stride, ty, dbuf.data_ptr() + ne * stride)
        for kind in range(3):
            u = rng.normal(size=(m, hidden)).astype(np.float32)
            logits = rng.normal(size=(m, ne)).astype(np.float32)
            if kind == 1:
                logits = (rng.integers(0, 8, (m, ne)) * 0.5).astype(np.float32)
            elif kind == 2:
                for j in range(m):
                    top = np.argsort(-logits[j])[:k + 2]
                    for a, b in zip(top[0::2], top[1::2]):
                        step = np.int32(rng.integers(1, 400))
                        v = logits[j, a].view(np.int32) + (step if logits[j, a] < 0 else -step)
                        logits[j, b] = np.int32(v).view(np.float32)
            sgl = rng.normal(size=m).astype(np.float32)
            du, dl, dg = dev(gpu, u), dev(gpu, logits), dev(gpu, sgl)
            dy = gpu.zeros((m, hidden), dtype=gpu.float32, device="cuda")
            s.moe_layer_verify(0, m, du.data_ptr(), dl.data_ptr(), dg.data_ptr(), dy.data_ptr())
            gpu.cuda.synchronize()
            got = dy.cpu().numpy()
            idx, w = s.last_route(m)
            want, widx, ww = oracle_layer(ty, hidden, ff, k, blobs, sh, logits, sgl, u)
            assert np.array_equal(idx, widx), f"seed {seed} kind {kind}"
            assert np.allclose(w, ww, rtol=2e-6, atol=0)
            for j in range(m):
                assert rel_l2(got[j], want[j]) <= REL_L2, f"seed {seed} kind {kind} row {j}: {rel_l2(got[j], want[j])}"


@pytest.mark.parametrize("ty,rty,hidden,ff,ne,k,m", [
    (sz.EXL3(3), sz.F32, 2048, 512, 48, 10, 4),
    (sz.IQ3_S, sz.BF16, 2048, 512, 32, 10, 3),
    (sz.EXL3(4), sz.F16, 512, 256, 10, 4, 8),
    (sz.IQ3_S, sz.F32, 2048, 512, 32, 10, 1),      # one token: the router's launch, then the two-launch layer
])
def test_moe_block_with_its_router_matches_the_oracle(gpu, ty, rty, hidden, ff, ne, k, m):
    """Session::moe (forward.rs:1009-1034) from the activations alone: the router and the shared expert's gate product
    (moe_router_batch, session.rs:7868), then the layer.  The router's outputs are checked against the oracle's f64 row
    dots; ids, weights and y against the oracle fed with the logits the GPU produced (a logit that differs in its last
    bit may legitimately swap two near-equal experts, as it may between the reference's own CPU and GPU paths)."""
    rng = np.random.default_rng(ty + rty + m)
    dbuf, stride, blobs, sh = build_layer(gpu, rng, ty, hidden, ff, ne, True)
    rw, gw = dense_matrix(rng, rty, ne, hidden), dense_matrix(rng, rty, 1, hidden)
    drw, dgw = dev(gpu, rw), dev(gpu, gw)
    s = sz.Session(hidden, ff, ne, k, 1, 0, 8)
    s.set_layer(0, ty, dbuf.data_ptr(), stride, ty, dbuf.data_ptr() + ne * stride)
    with pytest.raises(sz.SzError):
        s.moe_router_verify(0, m, 0)                      # no router yet
    with pytest.raises(sz.SzError):
        s.set_router(0, sz.Q8_0, drw.data_ptr(), rty, dgw.data_ptr())   # a quantized router has no kernel here
    s.set_router(0, rty, drw.data_ptr(), rty, dgw.data_ptr())
    u = rng.normal(size=(m, hidden)).astype(np.float32)
    du = dev(gpu, u)
    dy = gpu.zeros((m, hidden), dtype=gpu.float32, device="cuda")
    s.moe_block_verify(0, m, du.data_ptr(), dy.data_ptr())
    gpu.cuda.synchronize()
    rl_ptr, sgl_ptr = s.router_outputs()
    rl, sgl = np.empty((m, ne), np.float32), np.empty(m, np.float32)
    sz.download(rl, rl_ptr)
    sz.download(sgl, sgl_ptr)
    for j in range(m):
        want = O.matvec(rty, hidden, ne, rw, u[j])
        assert np.all(np.abs(rl[j] - want) <= gguf_bound(rty, hidden, ne, rw, u[j]))
        wg = O.matvec(rty, hidden, 1, gw, u[j])
        assert abs(sgl[j] - wg[0]) <= gguf_bound(rty, hidden, 1, gw, u[j])[0]
    got = dy.cpu().numpy()
    idx, w = s.last_route(m)
    want, widx, ww = oracle_layer(ty, hidden, ff, k, blobs, sh, rl, sgl, u)
    assert np.array_equal(idx, widx)
    assert np.allclose(w, ww, rtol=2e-6, atol=0)
    for j in range(m):
        assert rel_l2(got[j], want[j]) <= REL_L2
    # the two halves on their own give the same bits
    dy2 = gpu.zeros((m, hidden), dtype=gpu.float32, device="cuda")
    s.moe_router_verify(0, m, du.data_ptr())
    s.moe_layer_verify(0, m, du.data_ptr(), rl_ptr, sgl_ptr, dy2.data_ptr())
    gpu.cuda.synchronize()
    assert np.array_equal(bits(dy2.cpu().numpy()), bits(got))


@pytest.mark.parametrize("ty,h,cs,rank,m,inject", [(sz.BF16, 2048, 4, 320, 4, True), (sz.F32, 256, 2, 24, 8, True), (sz.F16, 512, 4, 64, 1, False)])
def test_hyper_connection_read_and_write_match_the_oracle(gpu, ty, h, cs, rank, m, inject):
    """hc_read on the residual streams of a verify batch (norm, down + inject, up, mix: session.rs:7432) and the hc_write that
    follows the sublayer, against forward.rs:797-817 / 1078-1084 restated in the oracle."""
    rng = np.random.default_rng(h + cs + m)
    ch, eps = h * cs, 1e-6
    r = rng.normal(size=(m, ch)).astype(np.float32)
    nw = (1 + 0.1 * rng.normal(size=ch)).astype(np.float32)
    wd, wu, wi = dense_matrix(rng, ty, rank, ch), dense_matrix(rng, ty, ch, rank), dense_matrix(rng, ty, cs, ch)
    dr, dnw, dwd, dwu, dwi = dev(gpu, r), dev(gpu, nw), dev(gpu, wd), dev(gpu, wu), dev(gpu, wi)
    hc = sz.HyperConnection(h, cs, rank, eps, dnw.data_ptr(), ty, dwd.data_ptr(), ty, dwu.data_ptr(), ty, dwi.data_ptr() if inject else 0)
    du = gpu.zeros((m, h), dtype=gpu.float32, device="cuda")
    hc.read(m, dr.data_ptr(), du.data_ptr())
    gpu.cuda.synchronize()
    u = du.cpu().numpy()
    g = np.empty((m, cs), np.float32)
    sz.download(g, hc.gains)
    y = rng.normal(size=(m, h)).astype(np.float32)
    dy = dev(gpu, y)
    for j in range(m):
        wu_, wg_ = O.hc_read(r[j], h, cs, rank, eps, nw, (ty, wd), (ty, wu), (ty, wi) if inject else None)
        assert rel_l2(u[j], wu_) <= 1e-5, rel_l2(u[j], wu_)
        if inject:
            assert np.allclose(g[j], wg_, rtol=1e-5, atol=1e-6)
    if inject:
        sz.hc_write(dr.data_ptr(), hc.gains, dy.data_ptr(), m, h, cs)
        gpu.cuda.synchronize()
        got = dr.cpu().numpy()
        for j in range(m):
            assert np.array_equal(bits(got[j]), bits(O.hc_write(r[j], g[j], y[j], h, cs)))   # given the same gains: one multiply-add an element
    with pytest.raises(sz.SzError):
        hc.read(9, dr.data_ptr(), du.data_ptr())
    with pytest.raises(sz.SzError):
        sz.HyperConnection(h, cs, rank, eps, dnw.data_ptr(), sz.Q8_0, dwd.data_ptr(), ty, dwu.data_ptr())


@pytest.mark.parametrize("ty", [sz.Q8_0, sz.EXL3(3)])
def test_routing_ties_and_order_are_bit_exact(gpu, ty):
    # coarse logits so that ties are common (forward.rs:1276-1303), through the routing inside the layer's first launch
    # (the GGUF kernels' and the EXL3 kernels' own call sites of the selection, each with its own fallback scratch)
    rng = np.random.default_rng(99)
    hidden, ff, ne, k, m = 256, 256, 512, 10, 8
    # the experts are never run to completion here on the oracle side; only the routing is compared
    one = synth.expert_blob(rng, ty, hidden, ff)
    stride = one.size
    s = sz.Session(hidden, ff, ne, k, 1, 0, 8)
    big = dev(gpu, np.tile(one, ne))            # 512 copies of one expert: only the routing is compared here
    s.set_layer(0, ty, big.data_ptr(), stride, 0, 0)
    du = dev(gpu, rng.normal(size=(m, hidden)).astype(np.float32))
    dg = dev(gpu, np.zeros(m, np.float32))
    dy = gpu.zeros((m, hidden), dtype=gpu.float32, device="cuda")
    for trial in range(9):
        if trial % 3 == 0:
            logits = (rng.integers(0, 16, (m, ne)) * 0.5).astype(np.float32)
        elif trial % 3 == 1:
            logits = (rng.integers(0, 100000, (m, ne)) / 7919.0 - 6.0).astype(np.float32)
        else:
            # near-ties: among the largest logits, pairs that differ by one to a few hundred units in the last place (below
            # what the 32-bit selection keys resolve), the larger one at the higher index half of the time; a row whose
            # second logit is within 2^-26 of the maximum; a row with a chosen expert more than 700 below the maximum
            logits = rng.normal(size=(m, ne)).astype(np.float32)
            for j in range(m):
                top = np.argsort(-logits[j])[:14]
                for a, b in zip(top[0::2], top[1::2]):
                    step = np.int32(rng.integers(1, 400))
                    v = logits[j, a].view(np.int32) + (step if logits[j, a] < 0 else -step)
                    logits[j, b] = np.int32(v).view(np.float32)
            logits[1, 7] = logits[1].max() * (1 - 2.0 ** -25) if logits[1].max() > 0 else logits[1].max() * (1 + 2.0 ** -25)
            logits[2] = -800.0
            logits[2, rng.integers(0, ne, 5)] = rng.normal(size=5).astype(np.float32)
            # masked experts (the reference sets the logits of skipped experts to -inf, session.rs:6205): fewer finite logits
            # than k in one row, exactly k in another
            logits[3] = -np.inf
            logits[3, rng.choice(ne, 6, replace=False)] = rng.normal(size=6).astype(np.float32)
            logits[4] = -np.inf
            logits[4, rng.choice(ne, k, replace=False)] = rng.normal(size=k).astype(np.float32)
        dl = dev(gpu, logits)
        s.moe_layer_verify(0, m, du.data_ptr(), dl.data_ptr(), dg.data_ptr(), dy.data_ptr())
        idx, w = s.last_route(m)
        for j in range(m):
            oi, ow = O.route(logits[j], k)
            assert np.array_equal(idx[j], oi), f"trial {trial} row {j}"
            assert np.allclose(w[j], ow.astype(np.float32), rtol=2e-6)


# ------------------------------------------------------------------------------------------------------------ the head
def planted_head(rng, vocab, hidden, m, winners=None):
    """A Q8_0 head and m inputs such that input j's largest logit is row winners[j] by a wide margin: that row is the
    input itself quantized (codes round(127 u / amax) a block, scale amax / 127 / 40), a logit of about |u|^2 / 40 = 51
    among logits of about +-0.5, so the arg-max does not hang on the last bits of an f32 sum."""
    w = synth.q8_0_matrix(rng, vocab, hidden)
    u = rng.normal(size=(m, hidden)).astype(np.float32)
    if winners is None:
        winners = [int(r) for r in rng.choice(vocab, size=m, replace=vocab < m)]
    rows = w.reshape(vocab, hidden // 32, 34)
    for j, r in enumerate(winners):
        if r in winners[:j]:
            continue                                   # a row already planted for an earlier input stays that input's
        blk = u[j].reshape(-1, 32)
        amax = np.abs(blk).max(axis=1, keepdims=True)
        rows[r, :, 2:] = np.round(blk / amax * 127.0).astype(np.int8).view(np.uint8)
        rows[r, :, :2] = (amax / 127.0 / 40.0).astype(np.float16).view(np.uint8).reshape(-1, 2)
    return w, u


@pytest.mark.parametrize("vocab,m,hidden", [(151936, 4, 2048), (1000, 1, 2048), (4099, 8, 2048), (8, 3, 2048),
                                            (3001, 5, 3072), (517, 2, 768), (2048, 3, 4096),    # rows that are not a power of two of 32-weight units
                                            (3000, 4, 1024), (40000, 8, 1536),                   # four waves a workgroup (2048 columns have a kernel of their own)
                                            (20000, 8, 4096), (20000, 7, 3072), (5000, 2, 2304), (5000, 3, 2560)])   # six and eight waves a workgroup
def test_head_argmax_and_logits_match_the_oracle(gpu, vocab, m, hidden):
    rng = np.random.default_rng(vocab + m)
    w, u = planted_head(rng, vocab, hidden, m, winners=[3] + [int(r) for r in rng.choice(vocab, size=m - 1)] if vocab == 4099 else None)
    if vocab == 4099:
        # exact ties: rows 7 and 4000 are copies of row 3, the planted maximum of input 0: the lowest id must win
        wb = w.reshape(vocab, -1)
        wb[7] = wb[3]
        wb[4000] = wb[3]
    dw = dev(gpu, w)
    du = dev(gpu, u)
    s = sz.Session(hidden, 512, 8, 2, 0, vocab, 8)
    s.set_head(sz.Q8_0, dw.data_ptr())
    ids = gpu.zeros(8, dtype=gpu.int32, device="cuda")
    s.head_argmax(m, du.data_ptr(), ids.data_ptr())
    logits = gpu.zeros((m, vocab), dtype=gpu.float32, device="cuda")
    s.head_logits(m, du.data_ptr(), logits.data_ptr())
    gpu.cuda.synchronize()
    got_ids = ids.cpu().numpy().astype(np.uint32)[:m]
    got_logits = logits.cpu().numpy()
    for j in range(m):
        want = O.matvec(O.Q8_0, hidden, vocab, w, u[j])
        assert rel_l2(got_logits[j], want) <= REL_L2
        # the planted maximum stands far above the f32 summation noise: the fused arg-max must be the oracle's, always
        top2 = np.sort(want)[-2:]
        assert top2[1] - top2[0] > 1e-2 * abs(top2[1]) or vocab == 4099
        assert got_ids[j] == O.argmax(want), (j, got_ids[j], O.argmax(want))
        assert got_ids[j] == O.argmax(got_logits[j])


@pytest.mark.parametrize("scale", [1.0e5, 3.0e-6, 6.0e4, 1.0])
def test_head_on_very_large_and_very_small_activations(gpu, scale):
    """The matrix-core head splits every input into f16 high and low parts: activations beyond f16's range (65504) or deep in
    its subnormals must give the oracle's ids and logits all the same (the rows are scaled by a power of two first)."""
    rng = np.random.default_rng(17)
    vocab, hidden, m = 4096, 2048, 4
    w, u = planted_head(rng, vocab, hidden, m)
    u = (u * np.float32(scale)).astype(np.float32)
    u[1, 5] *= 300.0                                          # one outlier far above the row's other elements
    dw, du = dev(gpu, w), dev(gpu, u)
    s = sz.Session(hidden, 512, 8, 2, 0, vocab, 8)
    s.set_head(sz.Q8_0, dw.data_ptr())
    ids = gpu.zeros(8, dtype=gpu.int32, device="cuda")
    s.head_argmax(m, du.data_ptr(), ids.data_ptr())
    top = s.head_top(m, du.data_ptr())
    gpu.cuda.synchronize()
    got_ids = ids.cpu().numpy().astype(np.uint32)[:m]
    for j in range(m):
        want = O.matvec(O.Q8_0, hidden, vocab, w, u[j])
        assert np.all(np.isfinite(want))
        assert got_ids[j] == O.argmax(want), (scale, j)
        vals, tids = top[j]
        wv, wi = O.topk(want)
        assert np.array_equal(tids[:8], wi[:8]) and rel_l2(vals, wv) <= REL_L2


def exl3_head_reference(blob, hidden, vocab, kb, u):
    """The oracle's logits of an EXL3 head for every input row (exl3.rs:528-599 matvec_blob)."""
    return [O.exl3_matvec(hidden, vocab, kb, blob, u[j]) for j in range(u.shape[0])]


def clear_gap(v, rank=1):
    """True when the `rank` largest values of v are further apart (relatively) than f32 summation noise can move them."""
    top = np.sort(v)[-(rank + 1):][::-1]
    return bool(np.all(top[:-1] - top[1:] > 1e-5 * np.abs(top[:-1])))


@pytest.mark.parametrize("kb,m,hidden,vocab", [(1, 2, 256, 512), (2, 3, 512, 1024), (3, 1, 512, 1024), (3, 8, 512, 1024), (4, 5, 768, 640),
                                              (5, 4, 512, 1024), (6, 7, 256, 512), (7, 2, 256, 256), (8, 8, 512, 1024), (4, 4, 2560, 1280),
                                              (4, 8, 4096, 512), (8, 8, 4096, 256)])   # 144 and 160 KiB of LDS a workgroup: the most a call may take
def test_exl3_head_argmax_logits_and_top_64_match_the_oracle(gpu, kb, m, hidden, vocab):
    """The lm_head of an EXL3 checkpoint (session.rs:7179-7187): fused arg-max ids bit-exact with the oracle's arg-max, logits
    within the reference's 2e-4 max|y| (tests/exl3.rs:45), the top 64 in the oracle's order; any whole rate, 1..8 rows."""
    rng = np.random.default_rng(1000 * kb + m)
    blob = synth.exl3_blob(rng, hidden, vocab, kb)
    u = rng.normal(size=(m, hidden)).astype(np.float32)
    u[0] *= 1.0e5                                            # a row far beyond f16's range, and a tiny one
    if m > 1:
        u[1] *= 3.0e-6
    db, du = dev(gpu, blob), dev(gpu, u)
    s = sz.Session(hidden, 512, 8, 2, 0, vocab, 8)
    s.set_head(sz.EXL3(kb), db.data_ptr())
    ids = gpu.zeros(8, dtype=gpu.int32, device="cuda")
    s.head_argmax(m, du.data_ptr(), ids.data_ptr())
    logits = gpu.zeros((m, vocab), dtype=gpu.float32, device="cuda")
    s.head_logits(m, du.data_ptr(), logits.data_ptr())
    top = s.head_top(m, du.data_ptr())
    gpu.cuda.synchronize()
    got_ids, got = ids.cpu().numpy().astype(np.uint32)[:m], logits.cpu().numpy()
    want = exl3_head_reference(blob, hidden, vocab, kb, u)
    for j in range(m):
        assert np.abs(got[j] - want[j]).max() <= 2e-4 * np.abs(want[j]).max() and rel_l2(got[j], want[j]) <= REL_L2
        assert clear_gap(want[j]), "pick another seed: the oracle's two largest logits are within f32 noise"
        assert got_ids[j] == O.argmax(want[j]) == O.argmax(got[j])
        vals, tids = top[j]
        wv, wi = O.topk(want[j])
        assert np.array_equal(tids, O.topk(got[j])[1])      # the exact top 64 of the GPU's own logits, ties to the lower id
        n_clear = 0
        while n_clear < 64 and clear_gap(want[j], n_clear + 1):
            n_clear += 1
        assert n_clear >= 4 and np.array_equal(tids[:n_clear], wi[:n_clear]) and rel_l2(vals, wv) <= REL_L2


def test_exl3_head_prefers_the_lowest_id_on_exact_ties(gpu):
    """Two 128-column blocks of the head with the same tiles and output scales give the same logits column by column: the
    lower column must win, also across the blocks' workgroups."""
    rng = np.random.default_rng(9)
    kb, hidden, vocab, m = 3, 512, 1024, 3
    blob = synth.exl3_blob(rng, hidden, vocab, kb).copy()
    svh = blob[2 * hidden:2 * hidden + 2 * vocab].view(np.float16)
    tr = blob[2 * hidden + 2 * vocab + 4:].view(np.uint16).reshape(hidden // 16, vocab // 16, 16 * kb)
    src, dst = 2, 5                                          # block 5 becomes a copy of block 2; both are made the loudest
    tr[:, 8 * dst:8 * dst + 8] = tr[:, 8 * src:8 * src + 8]
    svh[128 * src:128 * src + 128] *= np.float16(8.0)
    svh[128 * dst:128 * dst + 128] = svh[128 * src:128 * src + 128]
    u = rng.normal(size=(m, hidden)).astype(np.float32)
    db, du = dev(gpu, blob), dev(gpu, u)
    s = sz.Session(hidden, 512, 8, 2, 0, vocab, 8)
    s.set_head(sz.EXL3(kb), db.data_ptr())
    ids = gpu.zeros(8, dtype=gpu.int32, device="cuda")
    s.head_argmax(m, du.data_ptr(), ids.data_ptr())
    top = s.head_top(m, du.data_ptr())
    gpu.cuda.synchronize()
    got_ids = ids.cpu().numpy().astype(np.uint32)[:m]
    for j in range(m):
        want = O.exl3_matvec(hidden, vocab, kb, blob, u[j])
        best = O.argmax(want)
        assert 128 * src <= best < 128 * src + 128 and want[best] == want[best + 128 * (dst - src)]
        assert got_ids[j] == best
        assert top[j][1][0] == best and top[j][1][1] == best + 128 * (dst - src)


@pytest.mark.parametrize("kb,m", [(3, 1), (4, 4), (5, 8)])
def test_exl3_head_full_size(gpu, kb, m):
    """151 936 x 2048 at K = 3, 4, 5 for 1, 4 and 8 rows: ids equal to the oracle's arg-max, the top 64 in its order."""
    rng = np.random.default_rng(50 + kb)
    hidden, vocab = 2048, 151936
    blob = synth.exl3_blob(rng, hidden, vocab, kb)
    u = rng.normal(size=(m, hidden)).astype(np.float32)
    db, du = dev(gpu, blob), dev(gpu, u)
    s = sz.Session(hidden, 512, 8, 2, 0, vocab, 8)
    s.set_head(sz.EXL3(kb), db.data_ptr())
    ids = gpu.zeros(8, dtype=gpu.int32, device="cuda")
    print("exl3 head", kb, m, flush=True)
    s.head_argmax(m, du.data_ptr(), ids.data_ptr())
    gpu.cuda.synchronize()
    top = s.head_top(m, du.data_ptr())
    got_ids = ids.cpu().numpy().astype(np.uint32)[:m]
    for j in range(m):
        want = O.exl3_matvec(hidden, vocab, kb, blob, u[j])
        assert clear_gap(want), "pick another seed: the oracle's two largest logits are within f32 noise"
        assert got_ids[j] == O.argmax(want)
        vals, tids = top[j]
        wv, wi = O.topk(want)
        # the order must be the oracle's as far down as its neighbours are further apart than f32 summation noise; the ids
        # behind that prefix may swap places with a neighbour, so as a set all but the last few are the oracle's
        n_clear = 0
        while n_clear < 64 and clear_gap(want, n_clear + 1):
            n_clear += 1
        print(f"row {j}: the first {n_clear} ranks are clear of noise", flush=True)
        assert n_clear >= 1 and np.array_equal(tids[:n_clear], wi[:n_clear]) and rel_l2(vals, wv) <= REL_L2
        assert len(set(tids.tolist()) & set(wi.tolist())) >= 62


def test_verify_round_with_an_exl3_head(gpu):
    """A round of a model whose head is EXL3 too (the mixed-rate checkpoint's own): ids, accepted count and the graph replays."""
    rng = np.random.default_rng(31)
    hidden, ff, ne, k, vocab, m, kb = 512, 256, 8, 3, 1024, 4, 4
    s = sz.Session(hidden, ff, ne, k, 1, vocab, 8)
    dbuf, stride, blobs, sh = build_layer(gpu, rng, sz.EXL3(3), hidden, ff, ne, True)
    s.set_layer(0, sz.EXL3(3), dbuf.data_ptr(), stride, sz.EXL3(3), dbuf.data_ptr() + ne * stride)
    head = synth.exl3_blob(rng, hidden, vocab, kb)
    dh = dev(gpu, head)
    s.set_head(sz.EXL3(kb), dh.data_ptr())
    u = rng.normal(size=(1, m, hidden)).astype(np.float32)
    rl = rng.normal(size=(1, m, ne)).astype(np.float32)
    sgl = rng.normal(size=(1, m)).astype(np.float32)
    hu = rng.normal(size=(m, hidden)).astype(np.float32)
    du, drl, dsgl, dhu = dev(gpu, u), dev(gpu, rl), dev(gpu, sgl), dev(gpu, hu)
    want = [O.exl3_matvec(hidden, vocab, kb, head, hu[j]) for j in range(m)]
    assert all(clear_gap(w) for w in want)
    want_ids = np.array([O.argmax(w) for w in want], np.uint32)
    drafts = want_ids[:m - 1].copy()
    drafts[2] = (drafts[2] + 1) % vocab                      # two of the three drafts are accepted
    dd = dev(gpu, drafts.astype(np.int32))
    out = gpu.zeros(2 + 8, dtype=gpu.int32, device="cuda")
    y = gpu.zeros((1, m, hidden), dtype=gpu.float32, device="cuda")
    stream = sz.Stream()
    for replay in range(3):
        out.zero_()
        gpu.cuda.synchronize()
        s.verify_round(m, du.data_ptr(), drl.data_ptr(), dsgl.data_ptr(), y.data_ptr(), dhu.data_ptr(), dd.data_ptr(), out.data_ptr(), stream.handle)
        stream.synchronize()
        o = out.cpu().numpy().view(np.uint32)
        assert np.array_equal(o[2:2 + m], want_ids) and o[0] == 3 and o[1] == want_ids[2]
    # a head whose product has no arg-max fused in goes through its logits (the reference's mv_cols + topk_rows_at,
    # session.rs:7034-7052): the same round, captured anew for the new head
    wq = synth.iq3_s_matrix(rng, vocab, hidden)
    dq = dev(gpu, wq)
    s.set_head(sz.IQ3_S, dq.data_ptr())
    want = [O.matvec(sz.IQ3_S, hidden, vocab, wq, hu[j]) for j in range(m)]
    assert all(clear_gap(w) for w in want)
    want_ids = np.array([O.argmax(w) for w in want], np.uint32)
    drafts = want_ids[:m - 1].copy()
    drafts[1] = (drafts[1] + 1) % vocab                      # one of the three drafts is accepted
    dd2 = dev(gpu, drafts.astype(np.int32))
    for replay in range(3):
        out.zero_()
        gpu.cuda.synchronize()
        s.verify_round(m, du.data_ptr(), drl.data_ptr(), dsgl.data_ptr(), y.data_ptr(), dhu.data_ptr(), dd2.data_ptr(), out.data_ptr(), stream.handle)
        stream.synchronize()
        o = out.cpu().numpy().view(np.uint32)
        assert np.array_equal(o[2:2 + m], want_ids) and o[0] == 2 and o[1] == want_ids[1]


@pytest.mark.parametrize("ty", ["iq3_s", "f32", "f16", "bf16"])
def test_head_argmax_of_a_type_without_a_fused_kernel(gpu, ty):
    """sz_head_argmax for heads that are neither Q8_0 nor EXL3 (session.rs:7034-7052 takes any type): the oracle's arg-max of
    the oracle's logits on rows with a clear gap, the lowest id on exact ties (equal rows of the matrix in different slices of
    4096), a vocabulary that is no multiple of the slice, 1 to 8 rows."""
    t = {"iq3_s": sz.IQ3_S, "f32": sz.F32, "f16": sz.F16, "bf16": sz.BF16}[ty]
    rng = np.random.default_rng(77 + t)
    vocab, hidden = 9001, 512
    if t == sz.IQ3_S:
        w = synth.iq3_s_matrix(rng, vocab, hidden).reshape(vocab, -1)
    else:
        w = dense_matrix(rng, t, vocab, hidden).reshape(vocab, -1)
    u = rng.normal(size=(8, hidden)).astype(np.float32)
    base = O.matvec(t, hidden, vocab, w.reshape(-1), u[0])
    best = int(np.argmax(base))
    twins = [i for i in (17, 4100, 9000) if i != best]
    for i in twins:
        w[i] = w[best]                                       # row 0's largest logit now occurs at several ids
    dw, du = dev(gpu, w.reshape(-1)), dev(gpu, u)
    s = sz.Session(hidden, 512, 8, 2, 0, vocab, 8)
    s.set_head(t, dw.data_ptr())
    want = [O.matvec(t, hidden, vocab, w.reshape(-1), u[j]) for j in range(8)]
    for m in (1, 3, 8):
        ids = gpu.zeros(8, dtype=gpu.int32, device="cuda")
        s.head_argmax(m, du.data_ptr(), ids.data_ptr())
        gpu.cuda.synchronize()
        got = ids.cpu().numpy().view(np.uint32)
        assert got[0] == min([best] + twins)
        for j in range(1, m):
            if clear_gap(want[j]):
                assert got[j] == O.argmax(want[j]), (m, j)
        assert not got[m:].any()


def test_head_argmax_prefers_the_lowest_id_on_exact_ties(gpu):
    rng = np.random.default_rng(3)
    vocab, hidden = 640, 2048
    w = synth.q8_0_matrix(rng, vocab, hidden).reshape(vocab, -1)
    u = rng.normal(size=(2, hidden)).astype(np.float32)
    base = O.matvec(O.Q8_0, hidden, vocab, w.reshape(-1), u[0])
    best = int(np.argmax(base))
    others = [i for i in (5, 333, 639) if i != best]
    for i in others:
        w[i] = w[best]
    dw, du = dev(gpu, w.reshape(-1)), dev(gpu, u)
    s = sz.Session(hidden, 512, 8, 2, 0, vocab, 8)
    s.set_head(sz.Q8_0, dw.data_ptr())
    ids = gpu.zeros(8, dtype=gpu.int32, device="cuda")
    s.head_argmax(1, du.data_ptr(), ids.data_ptr())
    gpu.cuda.synchronize()
    assert int(ids[0]) == min([best] + others)


@pytest.mark.parametrize("block", [256, 1024])
def test_top64_on_adversarial_rows(gpu, block):
    # crates/shadowzero-cuda/tests/topk.rs: ties, all equal, -inf and NaN, winners in the ragged last slice; and zeros of both signs
    rng = np.random.default_rng(14)
    vocab = 151936
    u = rng.random((5, vocab)).astype(np.float32)
    rows = np.empty((5, vocab), np.float32)
    rows[0] = u[0] * 20 - 10
    rows[1] = rng.integers(0, 40, vocab) * 0.5
    rows[2] = 1.25
    rows[3] = -np.inf
    rows[3, 7::5000] = u[3, 7::5000]
    rows[3, 12345] = np.nan
    rows[4] = u[4]
    rows[4, vocab - 100:] += 50
    rows[2, 5::7] = -1.25                                     # two values only, so the 64 are the lowest ids of the larger
    rows[1] -= 19.5                                           # steps of 0.5 up to zero, and zeros of both signs at the top:
    rows[1, 3::11] = -0.0                                     # -0 equals +0, the order among them is by id, the sign comes back as it was
    nb = (vocab + 4095) // 4096
    dl = dev(gpu, rows)
    sv = gpu.empty(5 * nb * 64, dtype=gpu.float32, device="cuda")
    si = gpu.empty(5 * nb * 64, dtype=gpu.int32, device="cuda")
    out = gpu.empty(5 * 128, dtype=gpu.int32, device="cuda")
    A = sz.Arg
    sz.launch("topk_slices", (5 * nb, 1, 1), (block, 1, 1), 0, 0,
              [A.ptr(dl.data_ptr()), A.u32(vocab), A.u32(vocab), A.u32(nb), A.ptr(sv.data_ptr()), A.ptr(si.data_ptr())])
    sz.launch("topk_merge", (5, 1, 1), (block, 1, 1), 0, 0, [A.ptr(sv.data_ptr()), A.ptr(si.data_ptr()), A.u32(nb), A.ptr(out.data_ptr())])
    gpu.cuda.synchronize()
    words = out.cpu().numpy().view(np.uint32).reshape(5, 128)
    for r in range(5):
        vals, ids = O.topk(rows[r], 64)
        assert np.array_equal(words[r, 64:], ids), f"row {r}"
        assert np.array_equal(words[r, :64], bits(vals)), f"row {r}"


def test_top64_over_sizes_and_value_kinds(gpu):
    """Vocabularies of fewer than 64 words, around a chunk, a slice and several slices; normal values, heavy ties, a mix of NaN,
    both infinities and zeros of both signs, and a row of -inf only; both workgroup sizes: values and ids as the oracle's sort
    gives them, unused places (-inf, 0xffffffff)."""
    rng = np.random.default_rng(123)
    A = sz.Arg
    for vocab in (1, 63, 65, 4095, 4097, 12289):
        for block in (256, 1024):
            for kind in range(4):
                rows = 2
                x = rng.normal(size=(rows, vocab)).astype(np.float32)
                if kind == 1:
                    x = rng.integers(-3, 4, (rows, vocab)).astype(np.float32)
                elif kind == 2:
                    m = rng.random((rows, vocab))
                    for lo, hi, v in ((0, 0.05, np.nan), (0.05, 0.1, -np.inf), (0.1, 0.12, np.inf), (0.12, 0.2, -0.0), (0.2, 0.28, 0.0)):
                        x[(m >= lo) & (m < hi)] = v
                elif kind == 3:
                    x[:] = -np.inf
                nb = (vocab + 4095) // 4096
                dl = dev(gpu, x)
                sv = gpu.empty(rows * nb * 64, dtype=gpu.float32, device="cuda")
                si = gpu.empty(rows * nb * 64, dtype=gpu.int32, device="cuda")
                out = gpu.empty(rows * 128, dtype=gpu.int32, device="cuda")
                sz.launch("topk_slices", (rows * nb, 1, 1), (block, 1, 1), 0, 0,
                          [A.ptr(dl.data_ptr()), A.u32(vocab), A.u32(vocab), A.u32(nb), A.ptr(sv.data_ptr()), A.ptr(si.data_ptr())])
                sz.launch("topk_merge", (rows, 1, 1), (block, 1, 1), 0, 0, [A.ptr(sv.data_ptr()), A.ptr(si.data_ptr()), A.u32(nb), A.ptr(out.data_ptr())])
                gpu.cuda.synchronize()
                w = out.cpu().numpy().view(np.uint32).reshape(rows, 128)
                k = min(64, vocab)
                for r in range(rows):
                    vals, ids = O.topk(x[r], k)
                    assert np.array_equal(w[r, 64:64 + k], ids) and np.array_equal(w[r, :k], bits(vals)), (vocab, block, kind, r)
                    assert np.all(w[r, 64 + k:] == 0xffffffff) and np.all(w[r, k:64] == bits(np.float32(-np.inf))), (vocab, block, kind, r)


def test_head_top_hands_over_the_sorted_top_64(gpu):
    rng = np.random.default_rng(21)
    vocab, hidden, m = 9000, 2048, 3
    w, u = planted_head(rng, vocab, hidden, m)
    dw, du = dev(gpu, w), dev(gpu, u)
    s = sz.Session(hidden, 512, 8, 2, 0, vocab, 8)
    s.set_head(sz.Q8_0, dw.data_ptr())
    top = s.head_top(m, du.data_ptr())
    logits = gpu.zeros((m, vocab), dtype=gpu.float32, device="cuda")
    s.head_logits(m, du.data_ptr(), logits.data_ptr())
    gpu.cuda.synchronize()
    lg = logits.cpu().numpy()
    for j in range(m):
        vals, ids = O.topk(lg[j], 64)
        assert np.array_equal(top[j][1], ids) and np.array_equal(bits(top[j][0]), bits(vals))


# ------------------------------------------------------------------------------------------------- the verify round
@pytest.mark.parametrize("m,mode,layers", [(4, 0, 3), (1, 0, 3), (2, 0, 3), (8, 0, 3), (4, 1, 3), (4, 2, 3), (1, 2, 3), (8, 2, 3), (5, 1, 3),
                                           (4, 0, 12), (1, 0, 12), (8, 0, 12), (3, 2, 12), (3, 0, 13), (4, 3, 3), (4, 3, 12), (7, 3, 12)])   # 13 x 3: the routing launch's last workgroup has an idle wave
def test_verify_round_small_with_planted_drafts(gpu, m, mode, layers):
    """Three EXL3 layers of mixed bit rates, a Q8_0 head, and the m - 1 drafts planted so that 0, 1, .. and all of them are
    accepted; the round replayed as a graph gives the bits of the layer-by-layer calls every time (inside a round of a dozen
    layers or more all layers are routed by one launch up front and the exact launches read a plan a layer, in a shorter one they
    select for themselves; a layer's rank-order sum rides the next layer's first launch; a single call selects inside its first
    launch and sums in a launch of its own).  Token 0 of layer 1
    has fewer finite logits than k (masked experts, session.rs:6205: unused ranks in the plan).  In every mode of the expert
    products: the exact kernels (0) and the two matrix-core forms."""
    rng = np.random.default_rng(77 + m)
    hidden, ff, ne, k, vocab = 512, 256, 12, 4, 3000
    rates = [2, 3, 4] * (layers // 3)
    s = sz.Session(hidden, ff, ne, k, len(rates), vocab, 8)
    s.set_expert_mode(mode)
    keep_alive, host = [], []
    for l, kb in enumerate(rates):
        dbuf, stride, blobs, sh = build_layer(gpu, rng, sz.EXL3(kb), hidden, ff, ne, True)
        keep_alive.append(dbuf)
        host.append((blobs, sh))
        s.set_layer(l, sz.EXL3(kb), dbuf.data_ptr(), stride, sz.EXL3(kb), dbuf.data_ptr() + ne * stride)
    w = synth.q8_0_matrix(rng, vocab, hidden)
    dw = dev(gpu, w)
    s.set_head(sz.Q8_0, dw.data_ptr())
    L = len(rates)
    u = rng.normal(size=(L, m, hidden)).astype(np.float32)
    rl = rng.normal(size=(L, m, ne)).astype(np.float32)
    masked = np.full(ne, -np.inf, np.float32)
    masked[[3, 7]] = rl[1, 0, [3, 7]]
    rl[1, 0] = masked                                        # two finite logits, k = 4
    sgl = rng.normal(size=(L, m)).astype(np.float32)
    hu = rng.normal(size=(m, hidden)).astype(np.float32)
    du, drl, dsgl, dhu = dev(gpu, u), dev(gpu, rl), dev(gpu, sgl), dev(gpu, hu)
    want_ids = np.array([O.argmax(O.matvec(O.Q8_0, hidden, vocab, w, hu[j])) for j in range(m)], np.uint32)
    # layer by layer first
    y_ref = gpu.zeros((L, m, hidden), dtype=gpu.float32, device="cuda")
    for l in range(L):
        s.moe_layer_verify(l, m, du[l].data_ptr(), drl[l].data_ptr(), dsgl[l].data_ptr(), y_ref[l].data_ptr())
    gpu.cuda.synchronize()
    y_ref = y_ref.cpu().numpy()
    for l, kb in enumerate(rates):
        want, _, _ = oracle_layer(sz.EXL3(kb), hidden, ff, k, host[l][0], host[l][1], rl[l], sgl[l], u[l])
        for j in range(m):
            assert rel_l2(y_ref[l, j], want[j]) <= REL_L2
    stream = sz.Stream()
    for accepted in range(m):
        drafts = want_ids[:m - 1].copy()
        if accepted < m - 1:
            drafts[accepted] = (drafts[accepted] + 1) % vocab
        dd = dev(gpu, np.concatenate([drafts, [0]]).astype(np.int32))       # one spare word: no drafts at m = 1
        out = gpu.zeros(2 + 8, dtype=gpu.int32, device="cuda")
        y = gpu.zeros((L, m, hidden), dtype=gpu.float32, device="cuda")
        gpu.cuda.synchronize()
        for replay in range(3):
            y.zero_()
            gpu.cuda.synchronize()
            s.verify_round(m, du.data_ptr(), drl.data_ptr(), dsgl.data_ptr(), y.data_ptr(), dhu.data_ptr(), dd.data_ptr(), out.data_ptr(),
                           stream.handle)
            stream.synchronize()
            o = out.cpu().numpy().view(np.uint32)
            assert np.array_equal(o[2:2 + m], want_ids), "arg-max token ids must be bit-exact"
            assert o[0] == 1 + accepted == O.accept(want_ids[:m - 1], drafts), "accepted-draft count must be bit-exact"
            assert o[1] == want_ids[accepted]
            assert np.array_equal(bits(y.cpu().numpy()), bits(y_ref)), f"replay {replay}"
    idx, _ = s.last_route(m, stream.handle)                  # the round's last layer, whichever plan buffer it took
    assert np.array_equal(idx, oracle_layer(sz.EXL3(rates[-1]), hidden, ff, k, host[-1][0], host[-1][1], rl[-1], sgl[-1], u[-1])[1])


# ------------------------------------------------------------------------------------------------ run-time compile
def test_memset_is_a_launch_of_its_own_and_replays_in_a_graph(gpu):
    """sz_memset (driver.rs:419, cuMemsetD8) at ragged starts and lengths, the bytes either side untouched; then recorded into
    a graph (two fills, the second over a part of the first), every replay checked with eager work in between."""
    import ctypes as C
    lib = sz.lib()
    n = 1 << 16
    buf = sz.DeviceBuffer(n)
    for off, cnt, byte in ((0, n, 0x11), (1, 0, 0x22), (3, 5, 0x33), (13, 4099, 0x44), (16, 32, 0x55), (17, 15, 0x66), (4081, 61455, 0x77)):
        buf.upload(np.full(n, 0xee, np.uint8))
        buf.fill(byte, 0, off, cnt)
        sz.check(lib.sz_stream_synchronize(0))
        want = np.full(n, 0xee, np.uint8)
        want[off:off + cnt] = byte
        assert np.array_equal(buf.download(np.uint8), want), (off, cnt)
    stream = sz.Stream()
    src = sz.DeviceBuffer(4096)
    sz.check(lib.sz_capture_begin(stream.handle))
    src.fill(0xa5, stream.handle, 7, 4000)
    src.fill(0x5a, stream.handle, 100, 33)                 # ordered after the first on the stream: it wins where they overlap
    g = C.c_uint64()
    sz.check(lib.sz_capture_end(stream.handle, C.byref(g)))
    for replay in range(4):
        src.upload(np.full(4096, replay, np.uint8))        # eager work and a synchronisation between the replays
        sz.check(lib.sz_graph_launch(g.value, stream.handle))
        stream.synchronize()
        want = np.full(4096, replay, np.uint8)
        want[7:4007] = 0xa5
        want[100:133] = 0x5a
        assert np.array_equal(src.download(np.uint8), want), replay
    sz.check(lib.sz_graph_destroy(g.value))


def test_hiprtc_compiles_a_kernel_with_the_library_options(gpu):
    import ctypes as C
    src = b"""
    #if !defined(__HIPCC_RTC__)
    #include <hip/hip_runtime.h>
    #endif
    extern "C" __global__ void vector_add(const float* a, const float* b, float* c, unsigned int n) {
        unsigned int i = blockIdx.x * blockDim.x + threadIdx.x;
        if (i < n) c[i] = a[i] + b[i];
    }"""
    n, log = C.c_uint64(), C.c_char_p()
    r = sz.lib().sz_rtc_compile(b"vector_add.hip", src, C.byref(n), C.byref(log))
    assert r == 0, sz.last_error()
    assert n.value > 1000
    r = sz.lib().sz_rtc_compile(b"broken.hip", b"extern \"C\" __global__ void f( { }", C.byref(n), C.byref(log))
    assert r != 0 and "error" in sz.last_error()          # the compile log comes back whole (nvrtc.rs:225-227)


def test_the_library_compiles_its_own_kernel_files_at_run_time_in_a_fresh_process(gpu, tmp_path):
    """kernels.rs:532-545, nvrtc.rs:180-256: with an empty code-object cache sz_init compiles all four kernel files with hiprtc
    (global-to-LDS loads and wait counts in inline assembly, permlane swaps, matrix instructions), fills the cache under the
    run-time keys, which are not the keys of the objects built ahead of time, and the smoke round (EXL3 layer, Q8_0 head,
    arg-max, acceptance, against the oracle) passes on those objects."""
    import os
    import subprocess
    import sys
    import time
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, SHADOWZERO_KERNEL_CACHE=str(tmp_path))
    t0 = time.time()
    p = subprocess.Popen([sys.executable, "-u", "-c", "import __graft_entry__ as g; g.smoke()"], cwd=root, env=env,
                         stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out, limit = "", 900.0
    while True:
        # the pipe is drained while the child runs (a child that prints more than a pipe holds would otherwise never end) and
        # a child that does not end is killed, with what it printed in the failure
        try:
            out += p.communicate(timeout=5)[0]
            break
        except subprocess.TimeoutExpired as e:
            print("run-time compile: %.0f s" % (time.time() - t0), flush=True)
            if time.time() - t0 > limit:
                p.kill()
                out += p.communicate()[0] or ""
                pytest.fail("the child did not end within %.0f s; it printed:\n%s" % (limit, out[-3000:]))
    assert p.returncode == 0 and "smoke ok" in out, out[-3000:]
    import ctypes as C
    lib = sz.lib()
    made = sorted(f for f in os.listdir(tmp_path) if f.endswith(".hsaco"))
    rtc, aot = [], []
    for i in range(lib.sz_program_file_count()):
        name = lib.sz_program_file_name(i)
        k1, k2 = C.create_string_buffer(65), C.create_string_buffer(65)
        assert lib.sz_program_cache_key_rtc(name, k1) == 0 and lib.sz_program_cache_key(name, k2) == 0
        rtc.append(k1.value.decode() + ".hsaco")
        aot.append(k2.value.decode() + ".hsaco")
    assert made == sorted(rtc) and not set(rtc) & set(aot)
    print("run-time compile of %d kernel files + smoke: %.0f s" % (len(made), time.time() - t0), flush=True)


# ------------------------------------------------------------------------------------------- the int8 prefill chunk
def test_activation_quantization_on_the_gpu_is_bit_exact(gpu):
    rng = np.random.default_rng(31)
    x = rng.normal(size=(37, 2048)).astype(np.float32)
    x[3, 64:96] = 0.0                      # an all-zero block
    x[5, :32] = np.arange(32) - 15.5       # exact halves after scaling
    dx = dev(gpu, x)
    q = gpu.zeros(x.size, dtype=gpu.int8, device="cuda")
    d = gpu.zeros(x.size // 32, dtype=gpu.float32, device="cuda")
    sz.quantize_act(dx.data_ptr(), x.size, q.data_ptr(), d.data_ptr())
    gpu.cuda.synchronize()
    wq, wd, _ = O.quantize_act(x, 32)
    assert np.array_equal(q.cpu().numpy(), wq) and np.array_equal(bits(d.cpu().numpy()), bits(wd))


@pytest.mark.parametrize("tokens,hidden,ff,ne,k,shared,skew", [(48, 512, 256, 16, 4, True, True), (130, 256, 256, 8, 3, False, True),
                                                                 (5, 2048, 512, 40, 10, True, False)])
def test_prefill_chunk_matches_the_int8_oracle(gpu, tokens, hidden, ff, ne, k, shared, skew):
    """Routing ids and the int8 codes of the input activations bit-exact; the layer output within 1e-3 relative L2 of the oracle
    that runs the same int8 arithmetic (cpu_expert.rs:243-339 with per-32 activation blocks).  The codes of H = silu(gate) * up,
    quantized again between the two products, are held to a relaxed bar on purpose: at most 1e-3 of them may differ from the
    oracle's (by one step each), because the device's expf and the fused multiply-add that folds a sub-block's int32 sum into
    the f32 total leave H a last bit or two away from the oracle's, which now and then crosses a rounding boundary."""
    rng = np.random.default_rng(tokens * 3 + ne)
    ty = sz.IQ3_S
    dbuf, stride, blobs, sh = build_layer(gpu, rng, ty, hidden, ff, ne, shared)
    s = sz.Session(hidden, ff, ne, k, 1, 0, 8)
    s.set_layer(0, ty, dbuf.data_ptr(), stride, ty if shared else 0, dbuf.data_ptr() + ne * stride if shared else 0)
    x = rng.normal(size=(tokens, hidden)).astype(np.float32)
    logits = synth.zipf_router_logits(rng, tokens, ne) if skew else rng.normal(size=(tokens, ne)).astype(np.float32)
    sgl = rng.normal(size=tokens).astype(np.float32)
    dxx, dl, dg = dev(gpu, x), dev(gpu, logits), dev(gpu, sgl)
    y = gpu.zeros((tokens, hidden), dtype=gpu.float32, device="cuda")
    s.moe_prefill_chunk(0, tokens, dxx.data_ptr(), dl.data_ptr(), dg.data_ptr(), y.data_ptr())
    gpu.cuda.synchronize()
    got = y.cpu().numpy()

    def fetch(which, dtype, count):
        out = np.empty(count, dtype)
        sz.check(sz.lib().sz_download(out.ctypes.data, s.prefill_buffer(which), out.nbytes))
        return out

    tidx = fetch(2, np.uint32, tokens * k).reshape(tokens, k)
    xq = fetch(0, np.int8, tokens * hidden).reshape(tokens, hidden)
    xd = fetch(1, np.float32, tokens * hidden // 32).reshape(tokens, hidden // 32)
    hq = fetch(4, np.int8, tokens * k * ff).reshape(tokens, k, ff)
    code_total = code_diff = 0
    for j in range(tokens):
        oi, ow = O.route(logits[j], k)
        assert np.array_equal(tidx[j], oi), f"token {j}"
        wq, wd, _ = O.quantize_act(x[j], 32)
        assert np.array_equal(xq[j], wq) and np.array_equal(bits(xd[j]), bits(wd))
        acc = np.zeros(hidden, np.float32)
        for t, (e, w) in enumerate(zip(oi, ow)):
            out, act = O.expert_int8(blobs[e], hidden, ff, wq, wd)
            aq, _, _ = O.quantize_act(act, 32)
            code_total += ff
            code_diff += int((hq[j, t] != aq).sum())
            acc = acc + np.float32(w) * out
        if shared:
            out, _ = O.expert_int8(sh, hidden, ff, wq, wd)
            acc = acc + np.float32(1.0 / (1.0 + np.exp(-np.float64(sgl[j])))) * out
        assert rel_l2(got[j], acc) <= REL_L2, f"token {j}: {rel_l2(got[j], acc)}"
    # H codes: the same rounding rule on values that agree to the last bit or two of f32 (device expf against libm's, fused fold)
    print(f"H codes: {code_diff} of {code_total} differ from the oracle's ({code_diff / code_total:.2e} of the places)", flush=True)
    assert code_diff <= 1e-3 * code_total, f"{code_diff} of {code_total} H codes differ"


# ------------------------------------------------------------------------------------- the configurations at full size
def test_config2_iq3s_decode_layer_full_size(gpu):
    """One MoE layer, batch 1: hidden 2048, 512 IQ3_S experts of intermediate 512 plus the shared expert, top-10."""
    rng = np.random.default_rng(2)
    hidden, ff, ne, k = 2048, 512, 512, 10
    dbuf, stride, blobs, sh = build_layer(gpu, rng, sz.IQ3_S, hidden, ff, ne, True)
    s = sz.Session(hidden, ff, ne, k, 1, 0, 8)
    s.set_layer(0, sz.IQ3_S, dbuf.data_ptr(), stride, sz.IQ3_S, dbuf.data_ptr() + ne * stride)
    u = rng.normal(size=(1, hidden)).astype(np.float32)
    logits = rng.normal(size=(1, ne)).astype(np.float32)
    sgl = rng.normal(size=1).astype(np.float32)
    dy = gpu.zeros((1, hidden), dtype=gpu.float32, device="cuda")
    du, dl, dg = dev(gpu, u), dev(gpu, logits), dev(gpu, sgl)      # named: a temporary's memory would be reused by the next
    s.moe_layer_verify(0, 1, du.data_ptr(), dl.data_ptr(), dg.data_ptr(), dy.data_ptr())
    gpu.cuda.synchronize()
    idx, w = s.last_route(1)
    want, widx, ww = oracle_layer(sz.IQ3_S, hidden, ff, k, blobs, sh, logits, sgl, u)
    assert np.array_equal(idx, widx) and np.allclose(w, ww, rtol=2e-6)
    assert rel_l2(dy.cpu().numpy()[0], want[0]) <= REL_L2


def test_config4_prefill_chunk_full_size(gpu):
    """512 tokens x hidden 2048 through 512 IQ3_S experts with Zipf-skewed routing: routing and activation codes of every
    token bit-exact, the layer output of a sample of tokens against the int8 oracle, and every row finite and non-zero."""
    rng = np.random.default_rng(4)
    tokens, hidden, ff, ne, k = 512, 2048, 512, 512, 10
    dbuf, stride, blobs, _ = build_layer(gpu, rng, sz.IQ3_S, hidden, ff, ne, False)
    s = sz.Session(hidden, ff, ne, k, 1, 0, 8)
    s.set_layer(0, sz.IQ3_S, dbuf.data_ptr(), stride, 0, 0)
    x = rng.normal(size=(tokens, hidden)).astype(np.float32)
    logits = synth.zipf_router_logits(rng, tokens, ne)
    y = gpu.zeros((tokens, hidden), dtype=gpu.float32, device="cuda")
    dx, dl, dg = dev(gpu, x), dev(gpu, logits), dev(gpu, np.zeros(tokens, np.float32))
    s.moe_prefill_chunk(0, tokens, dx.data_ptr(), dl.data_ptr(), dg.data_ptr(), y.data_ptr())
    gpu.cuda.synchronize()
    got = y.cpu().numpy()
    tidx = np.empty((tokens, k), np.uint32)
    sz.check(sz.lib().sz_download(tidx.ctypes.data, s.prefill_buffer(2), tidx.nbytes))
    xq = np.empty((tokens, hidden), np.int8)
    sz.check(sz.lib().sz_download(xq.ctypes.data, s.prefill_buffer(0), xq.nbytes))
    wq_all, wd_all, _ = O.quantize_act(x, 32)
    assert np.array_equal(xq.ravel(), wq_all)
    wts = np.empty((tokens, k), np.float32)
    sz.check(sz.lib().sz_download(wts.ctypes.data, s.prefill_buffer(3), wts.nbytes))
    for j in range(tokens):
        oi, ow = O.route(logits[j], k)
        assert np.array_equal(tidx[j], oi), f"token {j}"
        # the chunk's weights are ex_t over the sum of the chosen ex (the reference divides every ex by the sum over all experts
        # first, forward.rs:1143-1147): the same value before rounding, within a unit in the last place of f32 after it
        assert np.allclose(wts[j], ow, rtol=2e-6, atol=0), f"token {j}"
    counts = np.bincount(tidx.ravel(), minlength=ne)
    print("distinct experts hit:", int((counts > 0).sum()), "largest group:", int(counts.max()), flush=True)
    assert counts.max() > 64, "the skew must give an expert more than one pass of 64 tokens"
    assert np.all(np.isfinite(got)) and np.all(np.abs(got).max(axis=1) > 0)
    for j in list(range(0, tokens, 61)) + [tokens - 1]:
        oi, ow = O.route(logits[j], k)
        wq = wq_all[j * hidden:(j + 1) * hidden]
        wd = wd_all[j * hidden // 32:(j + 1) * hidden // 32]
        acc = np.zeros(hidden, np.float32)
        for e, w in zip(oi, ow):
            acc = acc + np.float32(w) * O.expert_int8(blobs[e], hidden, ff, wq, wd)[0]
        assert rel_l2(got[j], acc) <= REL_L2, f"token {j}: {rel_l2(got[j], acc)}"


@pytest.mark.parametrize("kb,tokens,hidden,ff,ne,k,shared", [
    (3, 70, 512, 256, 8, 3, True),                 # experts with more than two items of 32, the last one ragged
    (4, 33, 256, 512, 6, 2, False),                # an item of one token beside a full one; no shared expert
    (2, 200, 1024, 512, 16, 4, True),
    (5, 40, 256, 256, 6, 2, True),                 # the other rates' lane maps
    (6, 24, 512, 256, 6, 3, True),
    (8, 17, 256, 512, 4, 2, False),
    (1, 50, 3072, 512, 8, 3, True),                # six workgroups over the inputs, 24 column blocks of the down projection
    (3, 40, 768, 256, 6, 2, True),                 # hidden not a multiple of 512: the last workgroup over the inputs (and over down's columns) has idle waves
])
def test_exl3_prefill_chunk_matches_the_oracle(gpu, kb, tokens, hidden, ff, ne, k, shared):
    """A prefill chunk through a layer of EXL3 experts (f16 activations on the rows of the matrix instruction, the rotations on
    the matrix cores, items of up to 32 tokens of one expert): routing ids and order bit-exact, weights within a unit in the
    last place, every token's output within 1e-3 relative L2 of the exact oracle (forward.rs:1009-1034 a token at a time)."""
    ty = sz.EXL3(kb)
    rng = np.random.default_rng(kb * 1000 + tokens)
    dbuf, stride, blobs, sh = build_layer(gpu, rng, ty, hidden, ff, ne, shared)
    s = sz.Session(hidden, ff, ne, k, 1, 0, 8)
    s.set_layer(0, ty, dbuf.data_ptr(), stride, ty if shared else 0, dbuf.data_ptr() + ne * stride if shared else 0)
    x = rng.normal(size=(tokens, hidden)).astype(np.float32)
    x[3] *= 300.0                                            # rows of very different sizes: the per-token power of two
    x[5] *= 1e-4
    logits = rng.normal(size=(tokens, ne)).astype(np.float32)
    sgl = rng.normal(size=tokens).astype(np.float32)
    dx, dl, dg = dev(gpu, x), dev(gpu, logits), dev(gpu, sgl)
    y = gpu.zeros((tokens, hidden), dtype=gpu.float32, device="cuda")
    print("exl3 prefill", kb, tokens, hidden, ff, flush=True)
    s.moe_prefill_chunk(0, tokens, dx.data_ptr(), dl.data_ptr(), dg.data_ptr(), y.data_ptr())
    gpu.cuda.synchronize()
    got = y.cpu().numpy()
    tidx = np.empty((tokens, k), np.uint32)
    sz.check(sz.lib().sz_download(tidx.ctypes.data, s.prefill_buffer(2), tidx.nbytes))
    wts = np.empty((tokens, k), np.float32)
    sz.check(sz.lib().sz_download(wts.ctypes.data, s.prefill_buffer(3), wts.nbytes))
    want, widx, ww = oracle_layer(ty, hidden, ff, k, blobs, sh, logits, sgl, x)
    assert np.array_equal(tidx, widx), "expert routing must be bit-exact (ids and order)"
    assert np.allclose(wts, ww, rtol=2e-6, atol=0)
    assert np.all(np.isfinite(got))
    errs = np.array([rel_l2(got[j], want[j]) for j in range(tokens)])
    print(f"relative L2 of a token: median {np.median(errs):.3g}, worst {errs.max():.3g} (token {int(errs.argmax())})", flush=True)
    assert errs.max() <= REL_L2
    # twice the same bits, and a token's row does not depend on the other tokens of its chunk
    y2 = gpu.zeros((tokens, hidden), dtype=gpu.float32, device="cuda")
    s.moe_prefill_chunk(0, tokens, dx.data_ptr(), dl.data_ptr(), dg.data_ptr(), y2.data_ptr())
    gpu.cuda.synchronize()
    assert np.array_equal(bits(y2.cpu().numpy()), bits(got))


def test_exl3_prefill_chunk_full_size(gpu):
    """512 tokens x hidden 2048 through 512 EXL3 K = 3 experts plus the shared one, top-10 with Zipf-skewed routing (the int8
    chunk's configuration with the verify round's experts): routing of every token bit-exact, a sample of tokens against the
    exact oracle, every row finite and non-zero."""
    from shadow_engine_amd import synth_device
    torch = gpu
    rng = np.random.default_rng(45)
    tokens, hidden, ff, ne, k, kb = 512, 2048, 512, 512, 10, 3
    buf, stride = synth_device.exl3_layer(torch, 4321, hidden, ff, ne, kb)
    s = sz.Session(hidden, ff, ne, k, 1, 0, 8)
    s.set_layer(0, sz.EXL3(kb), buf.data_ptr(), stride, sz.EXL3(kb), buf.data_ptr() + ne * stride)
    x = rng.normal(size=(tokens, hidden)).astype(np.float32)
    logits = synth.zipf_router_logits(rng, tokens, ne)
    sgl = rng.normal(size=tokens).astype(np.float32)
    dx, dl, dg = dev(gpu, x), dev(gpu, logits), dev(gpu, sgl)
    y = gpu.zeros((tokens, hidden), dtype=gpu.float32, device="cuda")
    s.moe_prefill_chunk(0, tokens, dx.data_ptr(), dl.data_ptr(), dg.data_ptr(), y.data_ptr())
    gpu.cuda.synchronize()
    got = y.cpu().numpy()
    tidx = np.empty((tokens, k), np.uint32)
    sz.check(sz.lib().sz_download(tidx.ctypes.data, s.prefill_buffer(2), tidx.nbytes))
    for j in range(tokens):
        assert np.array_equal(tidx[j], O.route(logits[j], k)[0]), f"token {j}"
    counts = np.bincount(tidx.ravel(), minlength=ne)
    print("distinct experts hit:", int((counts > 0).sum()), "largest group:", int(counts.max()), flush=True)
    assert counts.max() > 64 and np.all(np.isfinite(got)) and np.all(np.abs(got).max(axis=1) > 0)
    oty = O.exl3_type(kb)
    shape = O.expert_shape(oty, oty, hidden, ff)
    nb = shape.gate_bytes + shape.up_bytes + shape.down_bytes
    worst = 0.0
    for j in list(range(0, tokens, 47)) + [tokens - 1]:
        ids = tidx[j]
        host = {int(e): buf[int(e) * stride:int(e) * stride + nb].cpu().numpy() for e in list(ids) + [ne]}
        experts = [host.get(e, host[int(ids[0])]) for e in range(ne)]
        want, widx, _ = O.moe_token(shape, experts, k, logits[j], x[j], shape, host[ne], float(sgl[j]))
        assert np.array_equal(widx, ids)
        worst = max(worst, rel_l2(got[j], want))
    print(f"worst relative L2 of a sampled token: {worst:.3g}", flush=True)
    assert worst <= REL_L2


def test_prefill_chunk_of_the_largest_size_equals_its_parts(gpu):
    """16384 tokens (the reference's largest staged pass, session.rs:191) in one chunk against the same tokens in chunks of
    2048 and 512: a token's result does not depend on which other tokens share its chunk (every pair owns its output row and
    the combine adds in rank order), so the rows must be bit-identical however the chunk is cut."""
    rng = np.random.default_rng(44)
    tokens, hidden, ff, ne, k = 16384, 512, 256, 64, 6
    dbuf, stride, blobs, sh = build_layer(gpu, rng, sz.IQ3_S, hidden, ff, ne, True)
    s = sz.Session(hidden, ff, ne, k, 1, 0, 8)
    s.set_layer(0, sz.IQ3_S, dbuf.data_ptr(), stride, sz.IQ3_S, dbuf.data_ptr() + ne * stride)
    g = gpu.Generator(device="cuda")
    g.manual_seed(3)
    x = gpu.randn((tokens, hidden), device="cuda", generator=g)
    dl = dev(gpu, synth.zipf_router_logits(rng, tokens, ne))
    dg = gpu.randn(tokens, device="cuda", generator=g)
    whole = gpu.zeros((tokens, hidden), dtype=gpu.float32, device="cuda")
    s.moe_prefill_chunk(0, tokens, x.data_ptr(), dl.data_ptr(), dg.data_ptr(), whole.data_ptr())
    gpu.cuda.synchronize()
    want = whole.cpu().numpy()
    assert np.all(np.isfinite(want)) and np.all(np.abs(want).max(axis=1) > 0)
    for part in (2048, 512):
        cut = gpu.zeros((tokens, hidden), dtype=gpu.float32, device="cuda")
        for t0 in range(0, tokens, part):
            s.moe_prefill_chunk(0, part, x[t0:].data_ptr(), dl[t0:].data_ptr(), dg[t0:].data_ptr(), cut[t0:].data_ptr())
        gpu.cuda.synchronize()
        assert np.array_equal(bits(cut.cpu().numpy()), bits(want)), f"chunks of {part}"
    # and a sample of rows against the int8 oracle
    xh = x.cpu().numpy()
    lg, sg = dl.cpu().numpy(), dg.cpu().numpy()
    wq_all, wd_all, _ = O.quantize_act(xh, 32)
    for j in (0, 777, 9000, tokens - 1):
        oi, ow = O.route(lg[j], k)
        wq, wd = wq_all[j * hidden:(j + 1) * hidden], wd_all[j * hidden // 32:(j + 1) * hidden // 32]
        acc = np.zeros(hidden, np.float32)
        for e, w in zip(oi, ow):
            acc = acc + np.float32(w) * O.expert_int8(blobs[e], hidden, ff, wq, wd)[0]
        acc = acc + O.lib().orc_sigmoid(float(sg[j])) * O.expert_int8(sh, hidden, ff, wq, wd)[0]
        assert rel_l2(want[j], acc) <= REL_L2, f"token {j}: {rel_l2(want[j], acc)}"
    with pytest.raises(sz.SzError):
        s.moe_prefill_chunk(0, 16385, x.data_ptr(), dl.data_ptr(), dg.data_ptr(), whole.data_ptr())


def test_exl3_prefill_chunk_of_the_largest_size_equals_its_parts(gpu):
    """The same for EXL3 experts: 16384 tokens in one chunk against chunks of 4096 and 512 (a token's power of two, its
    rotations and its column of every matrix product do not depend on which other tokens share its work item), and a sample of
    rows against the exact oracle."""
    rng = np.random.default_rng(46)
    tokens, hidden, ff, ne, k, kb = 16384, 512, 256, 48, 6, 3
    ty = sz.EXL3(kb)
    dbuf, stride, blobs, sh = build_layer(gpu, rng, ty, hidden, ff, ne, True)
    s = sz.Session(hidden, ff, ne, k, 1, 0, 8)
    s.set_layer(0, ty, dbuf.data_ptr(), stride, ty, dbuf.data_ptr() + ne * stride)
    g = gpu.Generator(device="cuda")
    g.manual_seed(5)
    x = gpu.randn((tokens, hidden), device="cuda", generator=g)
    dl = dev(gpu, synth.zipf_router_logits(rng, tokens, ne))
    dg = gpu.randn(tokens, device="cuda", generator=g)
    whole = gpu.zeros((tokens, hidden), dtype=gpu.float32, device="cuda")
    s.moe_prefill_chunk(0, tokens, x.data_ptr(), dl.data_ptr(), dg.data_ptr(), whole.data_ptr())
    gpu.cuda.synchronize()
    want = whole.cpu().numpy()
    assert np.all(np.isfinite(want)) and np.all(np.abs(want).max(axis=1) > 0)
    for part in (4096, 512):
        cut = gpu.zeros((tokens, hidden), dtype=gpu.float32, device="cuda")
        for t0 in range(0, tokens, part):
            s.moe_prefill_chunk(0, part, x[t0:].data_ptr(), dl[t0:].data_ptr(), dg[t0:].data_ptr(), cut[t0:].data_ptr())
        gpu.cuda.synchronize()
        assert np.array_equal(bits(cut.cpu().numpy()), bits(want)), f"chunks of {part}"
    xh, lg, sg = x.cpu().numpy(), dl.cpu().numpy(), dg.cpu().numpy()
    rows = [0, 4097, 9000, tokens - 1]
    ref, _, _ = oracle_layer(ty, hidden, ff, k, blobs, sh, lg[rows], sg[rows], xh[rows])
    for i, j in enumerate(rows):
        assert rel_l2(want[j], ref[i]) <= REL_L2, f"token {j}: {rel_l2(want[j], ref[i])}"


def test_config5_full_depth_verify_round(gpu):
    """48 layers of 512 + 1 EXL3 experts at mixed rates (about 29 GB generated in HBM), a 4-token batch, the 151,936-row Q8_0
    head, arg-max and acceptance: token ids and the accepted count exact against the oracle, every layer's output of two
    tokens (all four for the first layer of each rate) within 1e-3."""
    from shadow_engine_amd import synth_device
    torch = gpu
    free, _total = torch.cuda.mem_get_info()
    if free < 40e9:
        pytest.skip("needs about 31 GB of free HBM")
    hidden, ff, ne, k, vocab, m, L = 2048, 512, 512, 10, 151936, 4, 48
    rates = synth_device.layer_rates(2026, L)
    s = sz.Session(hidden, ff, ne, k, L, vocab, 8)
    layers = []
    for l, kb in enumerate(rates):
        buf, stride = synth_device.exl3_layer(torch, 1000 + l, hidden, ff, ne, kb)
        layers.append((buf, stride))
        s.set_layer(l, sz.EXL3(kb), buf.data_ptr(), stride, sz.EXL3(kb), buf.data_ptr() + ne * stride)
    head = synth_device.q8_0_head(torch, 7, vocab, hidden)
    s.set_head(sz.Q8_0, head.data_ptr())
    g = torch.Generator(device="cuda")
    g.manual_seed(11)
    u = torch.randn((L, m, hidden), device="cuda", generator=g)
    rl = torch.randn((L, m, ne), device="cuda", generator=g)
    sgl = torch.randn((L, m), device="cuda", generator=g)
    hu = torch.randn((m, hidden), device="cuda", generator=g)
    y = torch.zeros((L, m, hidden), device="cuda")
    out = torch.zeros(10, dtype=torch.int32, device="cuda")
    head_h = head.cpu().numpy()
    hu_h = hu.cpu().numpy()
    want_ids = np.array([O.argmax(O.matvec(O.Q8_0, hidden, vocab, head_h, hu_h[j])) for j in range(m)], np.uint32)
    drafts = want_ids[:3].copy()
    drafts[1] = (drafts[1] + 7) % vocab                       # one draft is accepted
    dd = dev(gpu, drafts.astype(np.int32))
    stream = sz.Stream()
    for replay in range(2):
        s.verify_round(m, u.data_ptr(), rl.data_ptr(), sgl.data_ptr(), y.data_ptr(), hu.data_ptr(), dd.data_ptr(), out.data_ptr(), stream.handle)
        stream.synchronize()
        o = out.cpu().numpy().view(np.uint32)
        assert np.array_equal(o[2:2 + m], want_ids)
        assert o[0] == 2 == O.accept(want_ids[:3], drafts) and o[1] == want_ids[1]
    got = y.cpu().numpy()
    u_h, rl_h, sgl_h = u.cpu().numpy(), rl.cpu().numpy(), sgl.cpu().numpy()
    seen_rates = set()
    for l, kb in enumerate(rates):
        buf, stride = layers[l]
        oty = O.exl3_type(kb)
        shape = O.expert_shape(oty, oty, hidden, ff)
        nb = shape.gate_bytes + shape.up_bytes + shape.down_bytes
        toks = range(m) if kb not in seen_rates else [l % m, (l + 1) % m]
        seen_rates.add(kb)
        for j in toks:
            ids = synth_device.route_ids(rl_h[l, j:j + 1], k)[0]
            host = {int(e): buf[int(e) * stride:int(e) * stride + nb].cpu().numpy() for e in list(ids) + [ne]}
            experts = [host.get(e, host[int(ids[0])]) for e in range(ne)]
            want, widx, _ = O.moe_token(shape, experts, k, rl_h[l, j], u_h[l, j], shape, host[ne], float(sgl_h[l, j]))
            assert np.array_equal(widx, ids.astype(np.uint32))
            assert rel_l2(got[l, j], want) <= REL_L2, f"layer {l} (K={kb}) token {j}: {rel_l2(got[l, j], want)}"
