"""The optional, inexact 2-bit screen of an EXL3 head (HeadProxy: crates/shadowzero-cuda/src/session.rs:428-441, 2631-2674,
5952-6022; kernels/exl3.cu:916-996; kernels/forward.cu:4371-4660).  The reference holds this path as CUDA kernels and one GPU
test (crates/shadowzero-cuda/tests/head_proxy.rs); there is no CPU statement of it.  The oracle restates the kernels'
arithmetic; the CPU tests here pin that restatement against things it does not share code with — the exact product, a
float64 statement from the levels' values, the textbook distortion of the quantizer, a brute-force choice of blocks, and the
gates of the reference's own test on its shape and generator — and the GPU tests then hold the library to the oracle bit
for bit, stage by stage, and to the properties the reference asserts (chosen blocks bitwise equal to the full head, the top
64 exact among them, the best row never lost)."""
import numpy as np
import pytest
from scipy.linalg import hadamard

import oracle_lib as O
import shadow_engine_amd as sz
from shadow_engine_amd import synth

H128 = hadamard(128).astype(np.float64)      # Sylvester order = the butterfly's h = 1, 2, .. 64 stages


def head_blob(rng, hidden, vocab, kb):
    """A random EXL3 head with input and output scales around one, as the reference's test makes them (head_proxy.rs:58-84)."""
    blob = synth.exl3_blob(rng, hidden, vocab, kb).copy()
    sign = np.where(rng.integers(0, 2, hidden) == 0, 1.0, -1.0)
    blob[:2 * hidden] = (sign * (0.8 + 0.4 * rng.random(hidden))).astype(np.float16).view(np.uint8)
    blob[2 * hidden:2 * hidden + 2 * vocab] = (0.8 + 0.4 * rng.random(vocab)).astype(np.float16).view(np.uint8)
    return blob


def scales_of(blob, hidden, vocab):
    return (blob[:2 * hidden].view(np.float16).astype(np.float64), blob[2 * hidden:2 * hidden + 2 * vocab].view(np.float16).astype(np.float64))


def rotated_matrix(blob, hidden, vocab, kb):
    """W_rot[in][out] in float64, from the decoded trellis: every input row transformed over each 128-output block, / 128, * svh."""
    w = O.exl3_reconstruct(hidden, vocab, kb, blob, inner=True).astype(np.float64).reshape(hidden, vocab // 128, 128)
    _, svh = scales_of(blob, hidden, vocab)
    return (w @ H128).reshape(hidden, vocab) / 128.0 * svh[None, :]


def rotated_rows(blob, x, hidden):
    """(x * suh) transformed block by block without the 1/sqrt(128) factor, float64."""
    suh = blob[:2 * hidden].view(np.float16).astype(np.float64)
    return ((x.astype(np.float64) * suh[None, :]).reshape(x.shape[0], hidden // 128, 128) @ H128).reshape(x.shape[0], hidden)


def levels_of(wq, ws):
    """The screen as a float64 matrix [out][in]: level (2 u - 3) * sh, unpacked from the stated layout."""
    n_ob, n_b = ws.shape[0], ws.shape[1]
    out = np.zeros((n_ob, 128, n_b, 128))
    sh = ws.view(np.float16).astype(np.float64)                 # [ob][b][r]
    for hb in range(2):
        for wi in range(4):
            for sl in range(4):
                for bi in range(4):
                    u = (wq[:, :, hb, :, wi] >> np.uint32(8 * bi + 2 * sl)) & np.uint32(3)      # [ob][b][r]
                    out[:, :, :, hb * 64 + wi * 16 + sl * 4 + bi] = ((2.0 * u - 3.0) * sh).transpose(0, 2, 1)
    return out.reshape(n_ob * 128, n_b * 128)


def codes_of(xq):
    """int8 codes [m][in] from the packed words."""
    return xq.view(np.int8).reshape(xq.shape[0], -1).astype(np.float64)


def exact_logits(blob, hidden, vocab, kb, x):
    return np.stack([O.exl3_matvec(hidden, vocab, kb, blob, x[j]) for j in range(x.shape[0])])


# ------------------------------------------------------------------------------------------------- the oracle, pinned (CPU)
@pytest.mark.parametrize("kb", [2, 4, 5])
def test_the_screen_follows_the_exact_product(kb):
    """Scores from the levels' values against the exact logits: a 2-bit uniform quantizer keeps 1 - 0.119 of the variance, so
    the correlation is about 0.94 and the slope about one; a transposed operand, a wrong sign or a lost scale gives neither."""
    rng = np.random.default_rng(kb)
    hidden, vocab, m = 512, 1024, 6
    blob = head_blob(rng, hidden, vocab, kb)
    x = rng.normal(size=(m, hidden)).astype(np.float32)
    wq, ws = O.q2_proxy_build(hidden, vocab, kb, blob)
    score = rotated_rows(blob, x, hidden) @ levels_of(wq, ws).T
    want = exact_logits(blob, hidden, vocab, kb, x)
    for j in range(m):
        assert np.corrcoef(score[j], want[j])[0, 1] > 0.9
        assert 0.9 < float(score[j] @ want[j] / (score[j] @ score[j])) < 1.12
    # and the matrix the builder rotates is the exact head's: (x * suh) H W_rot = the logits
    full = rotated_rows(blob, x, hidden) @ rotated_matrix(blob, hidden, vocab, kb)
    assert np.abs(full - want).max() <= 2e-4 * np.abs(want).max()


def test_the_quantizer_is_the_optimal_uniform_four_level_one():
    """Step 0.9957 sigma, levels +-0.5 and +-1.5 steps, threshold one step: a Gaussian loses 0.1188 of its variance (Max 1960)."""
    rng = np.random.default_rng(7)
    hidden, vocab, kb = 512, 1024, 4
    blob = head_blob(rng, hidden, vocab, kb)
    wq, ws = O.q2_proxy_build(hidden, vocab, kb, blob)
    wrot = rotated_matrix(blob, hidden, vocab, kb).T                      # [out][in]
    lv = levels_of(wq, ws)
    assert 0.108 < float(((lv - wrot) ** 2).sum() / (wrot ** 2).sum()) < 0.130
    rms = np.sqrt((wrot.reshape(vocab, hidden // 128, 128) ** 2).mean(2))  # [out][b]
    sh = ws.view(np.float16).astype(np.float64).transpose(0, 2, 1).reshape(vocab, hidden // 128)
    assert np.abs(sh / (0.5 * 0.9957 * rms) - 1).max() < 2e-3           # f16 roundings of the values and of the scale
    u = ((lv / np.repeat(sh, 128, axis=1)) + 3) / 2                       # the stored level of every weight
    inner = np.abs(wrot) < np.repeat(2 * sh, 128, axis=1) * 0.999
    outer = np.abs(wrot) > np.repeat(2 * sh, 128, axis=1) * 1.001
    assert np.all(np.isin(u[inner], [1, 2])) and np.all(np.isin(u[outer], [0, 3])) and np.all((u >= 1.5) == (wrot >= 0) | (np.abs(wrot) < 1e-7))


def test_input_codes_scale_and_correction():
    rng = np.random.default_rng(8)
    hidden, vocab, kb, m = 768, 256, 3, 5
    blob = head_blob(rng, hidden, vocab, kb)
    x = rng.normal(size=(m, hidden)).astype(np.float32)
    x[1] *= 1e-6
    x[2, 128:256] = 0.0                                                   # a block of zeros: scale 0, codes 0
    xq, sc, corr = O.q2_proxy_quant_x(blob, x, hidden)
    xr = rotated_rows(blob, x, hidden).reshape(m, hidden // 128, 128)
    amax = np.abs(xr).max(2)
    assert np.allclose(sc, amax / 127.0, rtol=1e-5) and np.all(sc[2, 1] == 0)
    q = codes_of(xq).reshape(m, hidden // 128, 128)
    want = np.rint(xr / np.where(amax > 0, amax / 127.0, 1.0)[:, :, None])
    assert np.abs(q - want).max() <= 1 and (q != want).mean() < 5e-3 and np.abs(q).max() == 127
    assert np.allclose(corr, -3.0 * q.sum(2) * sc, rtol=1e-6, atol=0)


def test_block_maxima_equal_the_float_statement():
    """sum_b sh * (2 x_sc * sum(code * u) + x_corr) = sum over the inputs of level value * code * scale."""
    rng = np.random.default_rng(9)
    hidden, vocab, kb, m = 512, 2048, 4, 3
    blob = head_blob(rng, hidden, vocab, kb)
    x = rng.normal(size=(m, hidden)).astype(np.float32)
    wq, ws = O.q2_proxy_build(hidden, vocab, kb, blob)
    xq, sc, corr = O.q2_proxy_quant_x(blob, x, hidden)
    got = O.q2_proxy_bmax(wq, ws, xq, sc, corr)
    xdeq = codes_of(xq) * np.repeat(sc.astype(np.float64), 128, axis=1)
    want = (xdeq @ levels_of(wq, ws).T).reshape(m, vocab // 128, 128).max(2)
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()


def plain_top(row, k):
    v = np.where(np.isnan(row), np.float32(-3.0e38), row)
    return sorted(np.lexsort((np.arange(v.size), -v.astype(np.float64)))[:k].tolist())


def test_choice_of_blocks_against_brute_force():
    rng = np.random.default_rng(10)
    n_ob, k = 1187, 128
    for trial in range(20):
        bm = rng.normal(size=(1, n_ob)).astype(np.float32)
        if trial % 4 == 1:
            bm[0, rng.integers(0, n_ob, 300)] = 1.5                       # many exact ties: the lower blocks win
        if trial % 4 == 2:
            bm[0, rng.integers(0, n_ob, 50)] = np.nan
        best = plain_top(bm[0], k)
        per_class = np.bincount(np.array(best) % 256, minlength=256).max()
        sel, n = O.q2_proxy_pick(bm, k, k)
        if per_class <= 4:
            assert sel.tolist() == best and n == k
    # a thread's fifth: blocks 3, 259, 515, 771, 1027 all among the best eight -> the smallest of them is lost, the ninth comes in
    bm = rng.normal(size=(1, n_ob)).astype(np.float32)
    bm[0, [3, 259, 515, 771, 1027]] = [10, 9, 8, 7, 6]
    bm[0, [100, 200, 300]] = [5.5, 5.25, 5.0]
    bm[0, 400] = 4.75
    sel, n = O.q2_proxy_pick(bm, 8, 8)
    assert sel.tolist() == [3, 100, 200, 259, 300, 400, 515, 771] and n == 8
    # several rows: the union, ascending, cut to the bound
    bm = rng.normal(size=(3, 64)).astype(np.float32)
    sel, n = O.q2_proxy_pick(bm, 16, 40)
    union = sorted(set(plain_top(bm[0], 16)) | set(plain_top(bm[1], 16)) | set(plain_top(bm[2], 16)))
    assert n == len(union) and sel.tolist() == union[:40]


class RefRng:
    """The generator of the reference's test (head_proxy.rs:7-18): xorshift64, unit() in [-1, 1] in steps of 1e-4."""

    def __init__(self, seed):
        self.s = seed

    def next(self):
        s = self.s
        s ^= (s << 13) & 0xFFFFFFFFFFFFFFFF
        s ^= s >> 7
        s ^= (s << 17) & 0xFFFFFFFFFFFFFFFF
        self.s = s
        return s

    def unit(self):
        return np.float32(np.float32(self.next() % 20001) / np.float32(10000.0) - np.float32(1.0))


def reference_test_case():
    """make_exl3_k5_blob and the inputs of test_q2_proxy_and_sparse_topk_exactness (head_proxy.rs:58-117): 4096 x 2560, K = 5."""
    rng = RefRng(0xabcdef0123456789)
    rows, cols, m = 4096, 2560, 4
    suh = np.array([np.float32(0.8) + np.float32(0.4) * abs(rng.unit()) for _ in range(cols)], np.float32).astype(np.float16)
    svh = np.array([np.float32(0.8) + np.float32(0.4) * abs(rng.unit()) for _ in range(rows)], np.float32).astype(np.float16)
    n_words = rows * cols * 5 // 32
    tr = np.empty(n_words, np.uint32)
    nxt = rng.next
    for i in range(n_words):
        tr[i] = nxt() & 0xFFFFFFFF
    blob = np.concatenate([suh.view(np.uint8), svh.view(np.uint8), np.zeros(4, np.uint8), tr.view(np.uint8)])
    x = np.array([rng.unit() for _ in range(m * cols)], np.float32).reshape(m, cols)
    return blob, x, rows, cols, m


_case = {}


def the_case():
    if not _case:
        blob, x, rows, cols, m = reference_test_case()
        _case.update(blob=blob, x=x, rows=rows, cols=cols, m=m, want=exact_logits(blob, cols, rows, 5, x))
    return _case


def test_the_gates_of_the_reference_test_hold_for_the_oracle():
    """head_proxy.rs:176-232 on its own blob, inputs and k_blk = 12: cosine of the block maxima with the exact ones above 0.85,
    between k_blk and m k_blk blocks chosen, the best row's block among them."""
    c = the_case()
    blob, x, rows, cols, m, want = c["blob"], c["x"], c["rows"], c["cols"], c["m"], c["want"]
    k_blk, n_ob = 12, rows // 128
    wq, ws = O.q2_proxy_build(cols, rows, 5, blob)
    xq, sc, corr = O.q2_proxy_quant_x(blob, x, cols)
    bm = O.q2_proxy_bmax(wq, ws, xq, sc, corr)
    true = want.reshape(m, n_ob, 128).max(2)
    for j in range(m):
        cos = float(bm[j] @ true[j] / np.linalg.norm(bm[j]) / np.linalg.norm(true[j]))
        assert cos > 0.85
        assert np.corrcoef(bm[j], true[j])[0, 1] > 0.5                 # the cosine of two positive vectors says little; this says more
    sel, n = O.q2_proxy_pick(bm, k_blk, min(m * k_blk, n_ob))
    assert k_blk <= sel.size <= m * k_blk and n == sel.size
    for j in range(m):
        assert O.argmax(want[j]) // 128 in sel.tolist()


# ------------------------------------------------------------------------------------------------ the library against it (GPU)
@pytest.fixture(scope="module")
def gpu():
    import torch
    assert torch.cuda.is_available(), "no GPU visible"
    sz.init(0)
    return torch


def dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def fetch(torch, addr, dtype, n):
    out = np.empty(n, dtype)
    sz.download(out, addr)
    return out


def run_screened_head(gpu, blob, x, hidden, vocab, kb, k_blk):
    """head_top with the screen on; returns everything the stages left behind, the full head's logits and the top 64."""
    m = x.shape[0]
    db, du = dev(gpu, blob), dev(gpu, x)
    s = sz.Session(hidden, 512, 8, 2, 0, vocab, 8)
    s.set_head(sz.EXL3(kb), db.data_ptr())
    logits = gpu.zeros((m, vocab), dtype=gpu.float32, device="cuda")
    s.head_logits(m, du.data_ptr(), logits.data_ptr())
    exact_top = s.head_top(m, du.data_ptr())
    s.set_head_proxy(k_blk)
    top = s.head_top(m, du.data_ptr())
    top2 = s.head_top(m, du.data_ptr())                                   # the bit map is left clean: a second call gives the same
    gpu.cuda.synchronize()
    n_ob, n_b = vocab // 128, hidden // 128
    k_use = min(max(k_blk, 16), n_ob)
    max_sel = min(m * k_use, n_ob)
    st = dict(
        wq=fetch(gpu, s.buffer(5), np.uint32, vocab * hidden // 16).reshape(n_ob, n_b, 2, 128, 4),
        ws=fetch(gpu, s.buffer(6), np.uint16, vocab * n_b).reshape(n_ob, n_b, 128),
        xq=fetch(gpu, s.buffer(7), np.uint32, m * hidden // 4).reshape(m, hidden // 4),
        sc=fetch(gpu, s.buffer(8), np.float32, m * n_b).reshape(m, n_b),
        corr=fetch(gpu, s.buffer(9), np.float32, m * n_b).reshape(m, n_b),
        bmax=fetch(gpu, s.buffer(10), np.float32, m * n_ob).reshape(m, n_ob),
        sel=fetch(gpu, s.buffer(11), np.uint32, 1 + max_sel),
        sparse=fetch(gpu, s.buffer(12), np.float32, m * max_sel * 128).reshape(m, max_sel * 128),
        dense=logits.cpu().numpy(), top=top, top2=top2, exact_top=exact_top, max_sel=max_sel, k_use=k_use)
    s.set_head_proxy(0)
    off = s.head_top(m, du.data_ptr())
    for j in range(m):                                                    # switched off again: the exact path, bit for bit
        assert np.array_equal(off[j][1], exact_top[j][1]) and np.array_equal(off[j][0].view(np.uint32), exact_top[j][0].view(np.uint32))
    return st


def check_against_the_oracle(st, blob, x, hidden, vocab, kb):
    m = x.shape[0]
    wq, ws = O.q2_proxy_build(hidden, vocab, kb, blob)
    assert np.array_equal(st["ws"], ws), "scales of the 2-bit copy"
    assert np.array_equal(st["wq"], wq), "levels of the 2-bit copy"
    xq, sc, corr = O.q2_proxy_quant_x(blob, x, hidden)
    assert np.array_equal(st["xq"], xq) and np.array_equal(st["sc"].view(np.uint32), sc.view(np.uint32))
    assert np.array_equal(st["corr"].view(np.uint32), corr.view(np.uint32))
    bm = O.q2_proxy_bmax(wq, ws, xq, sc, corr)
    assert np.array_equal(st["bmax"].view(np.uint32), bm.view(np.uint32)), "block maxima"
    sel, _ = O.q2_proxy_pick(bm, st["k_use"], st["max_sel"])
    n = int(st["sel"][0])
    assert n == sel.size and np.array_equal(st["sel"][1:1 + n], sel), "chosen blocks"
    return sel


def check_exact_among_the_chosen(st, sel, m):
    """head_proxy.rs:196-227: chosen blocks bit-identical to the full head, the top 64 exact among them."""
    dense = st["dense"]
    ids = (sel[:, None].astype(np.int64) * 128 + np.arange(128)[None, :]).reshape(-1)
    for j in range(m):
        assert np.array_equal(st["sparse"][j, :ids.size].view(np.uint32), dense[j, ids].view(np.uint32))
        vals = np.where(np.isnan(dense[j, ids]), -np.inf, dense[j, ids])
        order = np.lexsort((ids, -vals.astype(np.float64)))[:64]
        got_v, got_i = st["top"][j]
        assert np.array_equal(got_i, ids[order].astype(np.uint32)) and np.array_equal(got_v.view(np.uint32), vals[order].astype(np.float32).view(np.uint32))
        assert np.array_equal(st["top2"][j][1], got_i) and np.array_equal(st["top2"][j][0].view(np.uint32), got_v.view(np.uint32))


@pytest.mark.gpu
@pytest.mark.parametrize("kb,hidden,vocab,m,k_blk", [(5, 2560, 4096, 4, 16), (4, 2048, 8192, 8, 16), (3, 512, 4096, 1, 16), (2, 1024, 4096, 3, 20),
                                                    (8, 256, 2048, 5, 16), (1, 512, 2048, 2, 16), (6, 768, 4096, 7, 24), (7, 256, 2048, 2, 16),
                                                    (4, 4096, 2048, 4, 16)])
def test_every_stage_of_the_screen_is_bit_exact(gpu, kb, hidden, vocab, m, k_blk):
    rng = np.random.default_rng(100 * kb + m)
    blob = head_blob(rng, hidden, vocab, kb)
    x = rng.normal(size=(m, hidden)).astype(np.float32)
    if m > 2:
        x[1] *= 1e-5
        x[2, :128] = 0.0
    print("screen", kb, hidden, vocab, m, k_blk, flush=True)
    st = run_screened_head(gpu, blob, x, hidden, vocab, kb, k_blk)
    sel = check_against_the_oracle(st, blob, x, hidden, vocab, kb)
    check_exact_among_the_chosen(st, sel, m)


@pytest.mark.gpu
def test_the_reference_test_through_the_kernels(gpu):
    """test_q2_proxy_and_sparse_topk_exactness (head_proxy.rs:87-233), kernel by kernel through the checked launch as there,
    with its blob, inputs and k_blk = 12."""
    c = the_case()
    blob, x, rows, cols, m, want = c["blob"], c["x"], c["rows"], c["cols"], c["m"], c["want"]
    k_blk, n_ob, n_b = 12, rows // 128, cols // 128
    max_sel = min(m * k_blk, n_ob)
    A = sz.Arg
    t = gpu
    db, dx = dev(t, blob), dev(t, x)
    z = lambda n, dt: t.zeros(n, dtype=dt, device="cuda")
    wq, ws = z(rows * cols // 16, t.int32), z(rows * n_b, t.int16)
    xa, inv = z(n_b * 16 * 128, t.int16), z(16, t.float32)
    xq, xsc, xcorr = z(m * n_b * 32, t.int32), z(m * n_b, t.float32), z(m * n_b, t.float32)
    bmax, seen, sel = z(m * n_ob, t.float32), z((n_ob + 31) // 32, t.int32), z(1 + max_sel, t.int32)
    dense, sparse, part = z(m * rows, t.float32), z(m * max_sel * 128, t.float32), z(n_ob * 16, t.int32)
    nbs = (max_sel * 128 + 4095) // 4096
    sv, si, fin = z(m * nbs * 64, t.float32), z(m * nbs * 64, t.int32), z(m * 128, t.int32)
    P = lambda a: A.ptr(a.data_ptr())
    lds = 4 * ((n_b + 3) // 4) * ((m + 1) // 2) * 1024
    sz.launch("exl3_build_q2_proxy_5", (n_ob, n_b, 1), (256, 1, 1), 0, 0, [P(db), P(wq), P(ws), A.u32(cols), A.u32(rows)])
    sz.launch("exl3_head_rotate", (m, 1, 1), (64 * min(16, n_b), 1, 1), 0, 0, [P(db), P(dx), A.u32(cols), P(xa), P(inv), A.u32(cols)])
    sz.launch("head_exl3_5", (n_ob, 1, 1), (256, 1, 1), lds, 0, [P(db), P(xa), P(inv), P(dense), A.u32(rows), P(part), A.u32(cols), A.u32(rows), A.u32(m), A.ptr(0)])
    sz.launch("proxy_q2_quant_x", (n_b, m, 1), (64, 1, 1), 0, 0, [P(db), P(dx), A.u32(cols), P(xq), P(xsc), P(xcorr), A.u32(cols)])
    sz.launch("proxy_q2_bmax_m4", (n_ob, 1, 1), (128, 1, 1), 0, 0, [P(wq), P(ws), P(xq), P(xsc), P(xcorr), P(bmax), A.u32(n_ob), A.u32(cols), A.u32(m)])
    sz.launch("proxy_pick_rows", (m, 1, 1), (1024, 1, 1), 0, 0, [P(bmax), A.u32(n_ob), A.u32(k_blk), P(seen)])
    sz.launch("proxy_compact_seen", (1, 1, 1), (64, 1, 1), 0, 0, [P(seen), A.u32(n_ob), A.u32(max_sel), P(sel)])
    sz.launch("head_exl3_5", (max_sel, 1, 1), (256, 1, 1), lds, 0, [P(db), P(xa), P(inv), P(sparse), A.u32(max_sel * 128), P(part), A.u32(cols), A.u32(rows), A.u32(m), P(sel)])
    sz.launch("topk_slices_blks", (m * nbs, 1, 1), (256, 1, 1), 0, 0, [P(sparse), A.u32(max_sel * 128), P(sel), A.u32(nbs), P(sv), P(si)])
    sz.launch("topk_merge", (m, 1, 1), (256, 1, 1), 0, 0, [P(sv), P(si), A.u32(nbs), P(fin)])
    t.cuda.synchronize()
    assert int(seen.cpu().numpy().view(np.uint32).sum()) == 0            # the compaction clears the bit map
    sel_h = sel.cpu().numpy().view(np.uint32)
    n_sel = int(sel_h[0])
    assert k_blk <= n_sel <= max_sel
    chosen = sel_h[1:1 + n_sel]
    d = dense.cpu().numpy().reshape(m, rows)
    assert np.abs(d - want).max() <= 2e-4 * np.abs(want).max()
    bm = bmax.cpu().numpy().reshape(m, n_ob)
    true = d.reshape(m, n_ob, 128).max(2)
    fin_h = fin.cpu().numpy().view(np.uint32).reshape(m, 128)
    st = dict(dense=d, sparse=sparse.cpu().numpy().reshape(m, max_sel * 128), top=[(fin_h[j, :64].view(np.float32), fin_h[j, 64:]) for j in range(m)])
    st["top2"] = st["top"]
    for j in range(m):
        assert float(bm[j] @ true[j] / np.linalg.norm(bm[j]) / np.linalg.norm(true[j])) > 0.85
        assert int(np.argmax(d[j])) // 128 in chosen.tolist()
    check_exact_among_the_chosen(st, chosen, m)
    # and the oracle, stage by stage, on the same case
    owq, ows = O.q2_proxy_build(cols, rows, 5, blob)
    assert np.array_equal(wq.cpu().numpy().view(np.uint32).reshape(owq.shape), owq) and np.array_equal(ws.cpu().numpy().view(np.uint16).reshape(ows.shape), ows)
    oxq, osc, ocorr = O.q2_proxy_quant_x(blob, x, cols)
    obm = O.q2_proxy_bmax(owq, ows, oxq, osc, ocorr)
    assert np.array_equal(bm.view(np.uint32), obm.view(np.uint32))
    assert np.array_equal(chosen, O.q2_proxy_pick(obm, k_blk, max_sel)[0])


@pytest.mark.gpu
def test_the_screen_at_the_full_vocabulary(gpu):
    """151 936 x 2048 at K = 4, 4 rows, 128 blocks a row (the reference's default): every stage equal to the oracle, the chosen
    blocks equal to the full head, the exact arg-max of every row among them (its logit stands out by far more than the
    screen's noise), and most of the exact top 64 too."""
    rng = np.random.default_rng(77)
    hidden, vocab, kb, m = 2048, 151936, 4, 4
    blob = head_blob(rng, hidden, vocab, kb)
    x = rng.normal(size=(m, hidden)).astype(np.float32)
    print("screen, full vocabulary", flush=True)
    st = run_screened_head(gpu, blob, x, hidden, vocab, kb, 128)
    sel = check_against_the_oracle(st, blob, x, hidden, vocab, kb)
    check_exact_among_the_chosen(st, sel, m)
    assert 128 <= sel.size <= 512
    for j in range(m):
        assert st["top"][j][1][0] == st["exact_top"][j][1][0] == int(np.argmax(st["dense"][j]))
        found = len(set(st["top"][j][1].tolist()) & set(st["exact_top"][j][1].tolist()))
        print("row", j, "of the exact top 64 found:", found, flush=True)
        assert found >= 32


@pytest.mark.gpu
def test_the_screen_is_refused_where_it_cannot_be_built(gpu):
    rng = np.random.default_rng(3)
    s = sz.Session(512, 512, 8, 2, 0, 1024, 8)
    with pytest.raises(sz.SzError, match="EXL3 head"):
        s.set_head_proxy(16)
    w = dev(gpu, synth.q8_0_matrix(rng, 1024, 512))
    s.set_head(sz.Q8_0, w.data_ptr())
    with pytest.raises(sz.SzError, match="EXL3 head"):
        s.set_head_proxy(16)
    s.set_head_proxy(0)                                                   # off is always accepted
    big = sz.Session(8192, 512, 8, 2, 0, 256, 8)
    blob = dev(gpu, synth.exl3_blob(rng, 8192, 256, 2))
    big.set_head(sz.EXL3(2), blob.data_ptr())
    with pytest.raises(sz.SzError, match="4096"):
        big.set_head_proxy(16)
