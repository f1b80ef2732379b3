"""ctypes access to the CPU oracle (oracle/libshadow_oracle.so) for the tests, the smoke check and the benchmark's
cpu_baseline leg.  Test infrastructure: nothing under shadow_engine_amd/ imports this."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
LIB_PATH = os.path.join(ORACLE_DIR, "libshadow_oracle.so")

Q8_0, IQ3_S, F32 = 8, 21, 0


def lib_types():
    """ggml ids of the unquantized types (gguf.rs:100-130)."""
    return {"F32": 0, "F16": 1, "BF16": 30}


def exl3_type(bits, cb=2, half=False):
    return 1030 + bits if half else 1000 + 10 * cb + bits


def build():
    subprocess.run(["make", "-C", ORACLE_DIR, "libshadow_oracle.so"], check=True, capture_output=True)


class Tensor(C.Structure):
    _fields_ = [("ggml_type", C.c_int32), ("cols", C.c_uint64), ("rows", C.c_uint64), ("bytes", C.c_void_p),
                ("nbytes", C.c_uint64)]


class ExpertShape(C.Structure):
    _fields_ = [("gate_up_type", C.c_int32), ("down_type", C.c_int32), ("hidden", C.c_uint64), ("ff", C.c_uint64),
                ("gate_bytes", C.c_uint64), ("up_bytes", C.c_uint64), ("down_bytes", C.c_uint64)]


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        build()
    L = C.CDLL(LIB_PATH)
    vp, u8p, f32p = C.c_void_p, C.c_void_p, C.c_void_p
    sig = {
        "orc_f16_to_f32": (C.c_float, [C.c_uint16]),
        "orc_f32_to_f16": (C.c_uint16, [C.c_float]),
        "orc_f64_to_f16_bits": (C.c_uint16, [C.c_double]),
        "orc_round_f16": (C.c_float, [C.c_double]),
        "orc_block_layout": (C.c_int, [C.c_int, vp, vp]),
        "orc_dequantize": (C.c_int, [C.c_int, u8p, C.c_size_t, f32p, C.c_size_t]),
        "orc_backend_matvec": (C.c_int, [C.POINTER(Tensor), f32p, f32p, C.c_int]),
        "orc_exl3_codebook": (C.c_float, [C.c_int, C.c_uint32]),
        "orc_exl3_tile_pos": (None, [C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
        "orc_exl3_state": (C.c_uint32, [vp, C.c_int, C.c_int, C.c_int]),
        "orc_exl3_decode_tile": (None, [vp, C.c_int, C.c_int, C.c_int, f32p]),
        "orc_exl3_decode_tile_fast": (None, [vp, C.c_int, C.c_int, C.c_int, f32p]),
        "orc_exl3_blob_len": (C.c_uint64, [C.c_uint64, C.c_uint64, C.c_int, C.c_int]),
        "orc_wht128": (None, [f32p]),
        "orc_exl3_reconstruct": (C.c_int, [C.c_uint64, C.c_uint64, C.c_int, C.c_int, C.c_int, u8p, C.c_uint64, C.c_int, f32p]),
        "orc_exl3_matvec_blob": (C.c_int, [C.c_uint64, C.c_uint64, C.c_int, C.c_int, C.c_int, u8p, C.c_uint64, f32p, f32p, C.c_int]),
        "orc_route": (C.c_int, [f32p, C.c_int, C.c_int, vp, vp]),
        "orc_silu": (C.c_float, [C.c_float]),
        "orc_sigmoid": (C.c_float, [C.c_float]),
        "orc_rmsnorm_groups": (None, [f32p, f32p, C.c_size_t, C.c_size_t, C.c_float, f32p]),
        "orc_hc_read": (C.c_int, [f32p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_float, f32p, C.POINTER(Tensor), C.POINTER(Tensor),
                                  C.POINTER(Tensor), f32p, f32p, C.c_int]),
        "orc_hc_write": (None, [f32p, f32p, f32p, C.c_size_t, C.c_size_t]),
        "orc_moe_token": (C.c_int, [C.POINTER(ExpertShape), vp, C.c_int, C.c_int, f32p, C.POINTER(ExpertShape), u8p, C.c_float,
                                    f32p, f32p, vp, vp, C.c_int]),
        "orc_quantize_act": (None, [f32p, C.c_size_t, C.c_size_t, vp, f32p, vp]),
        "orc_iq3s_int8": (None, [u8p, vp, f32p]),
        "orc_iq3s_row_dot_q8": (C.c_float, [u8p, C.c_size_t, vp, f32p, vp]),
        "orc_expert_int8": (C.c_int, [u8p, C.c_uint64, C.c_uint64, vp, f32p, f32p, f32p]),
        "orc_argmax": (C.c_uint32, [f32p, C.c_size_t]),
        "orc_topk": (None, [f32p, C.c_size_t, C.c_int, f32p, vp]),
        "orc_accept": (C.c_int, [vp, vp, C.c_int]),
        "orc_hardware_threads": (C.c_int, []),
        "orc_q2_proxy_build": (C.c_int, [C.c_uint64, C.c_uint64, C.c_int, u8p, C.c_uint64, vp, vp]),
        "orc_q2_proxy_quant_x": (None, [u8p, f32p, C.c_uint64, vp, f32p, f32p]),
        "orc_q2_proxy_bmax": (None, [vp, vp, vp, f32p, f32p, C.c_uint64, C.c_uint64, f32p]),
        "orc_q2_proxy_pick": (C.c_uint32, [f32p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    _lib = L
    return L


def _p(a):
    return a.ctypes.data


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def dequantize(ty, data):
    data = _c(data, np.uint8)
    e, b = C.c_uint64(), C.c_uint64()
    assert lib().orc_block_layout(ty, C.byref(e), C.byref(b)) == 0
    out = np.empty(data.size // b.value * e.value, np.float32)
    r = lib().orc_dequantize(ty, _p(data), data.size, _p(out), out.size)
    assert r == 0, r
    return out


def matvec(ty, cols, rows, data, x, threads=0):
    data, x = _c(data, np.uint8), _c(x, np.float32)
    t = Tensor(ty, cols, rows, _p(data), data.size)
    y = np.empty(rows, np.float32)
    r = lib().orc_backend_matvec(C.byref(t), _p(x), _p(y), threads)
    assert r == 0, r
    return y


def exl3_blob_len(inf, outf, bits, half=False):
    return lib().orc_exl3_blob_len(inf, outf, bits, int(half))


def exl3_codebook_all(cb=2):
    return np.array([lib().orc_exl3_codebook(cb, s) for s in range(65536)], np.float32)


def exl3_decode_tile(tile_u16, bits, half=False, cb=2, fast=False):
    tile = _c(tile_u16, np.uint16)
    out = np.empty(256, np.float32)
    (lib().orc_exl3_decode_tile_fast if fast else lib().orc_exl3_decode_tile)(_p(tile), bits, int(half), cb, _p(out))
    return out


def exl3_reconstruct(inf, outf, bits, blob, half=False, cb=2, inner=False):
    blob = _c(blob, np.uint8)
    w = np.empty((inf, outf), np.float32)
    r = lib().orc_exl3_reconstruct(inf, outf, bits, int(half), cb, _p(blob), blob.size, int(inner), _p(w))
    assert r == 0, r
    return w


def exl3_matvec(inf, outf, bits, blob, x, half=False, cb=2, threads=0):
    blob, x = _c(blob, np.uint8), _c(x, np.float32)
    y = np.empty(outf, np.float32)
    r = lib().orc_exl3_matvec_blob(inf, outf, bits, int(half), cb, _p(blob), blob.size, _p(x), _p(y),
                                   threads or lib().orc_hardware_threads())
    assert r == 0, r
    return y


def wht128(v):
    v = _c(v, np.float32).copy()
    lib().orc_wht128(_p(v))
    return v


def rmsnorm_groups(x, w, group, eps):
    x, w = _c(x, np.float32), _c(w, np.float32)
    out = np.empty_like(x)
    lib().orc_rmsnorm_groups(_p(x), _p(w), x.size, group, eps, _p(out))
    return out


def hc_read(r, hidden, streams, rank, eps, norm_w, down, up, inject=None):
    """down / up / inject: (ggml type, bytes) of [rank][streams*hidden], [streams*hidden][rank], [streams][streams*hidden].
    Returns (u[hidden], g[streams] or None)."""
    r, norm_w = _c(r, np.float32), _c(norm_w, np.float32)
    ch = hidden * streams
    keep = [_c(down[1], np.uint8), _c(up[1], np.uint8)]
    td = Tensor(down[0], ch, rank, _p(keep[0]), keep[0].size)
    tu = Tensor(up[0], rank, ch, _p(keep[1]), keep[1].size)
    ti = None
    if inject is not None:
        keep.append(_c(inject[1], np.uint8))
        ti = Tensor(inject[0], ch, streams, _p(keep[2]), keep[2].size)
    u, g = np.empty(hidden, np.float32), np.empty(streams, np.float32)
    rc = lib().orc_hc_read(_p(r), hidden, streams, rank, eps, _p(norm_w), C.byref(td), C.byref(tu), C.byref(ti) if ti else None,
                           _p(u), _p(g), 0)
    assert rc == 0, rc
    return u, (g if inject is not None else None)


def hc_write(r, g, y, hidden, streams):
    r = np.array(r, np.float32)
    g, y = _c(g, np.float32), _c(y, np.float32)
    lib().orc_hc_write(_p(r), _p(g), _p(y), hidden, streams)
    return r


def route(logits, k):
    logits = _c(logits, np.float32)
    idx = np.zeros(k, np.uint32)
    w = np.zeros(k, np.float64)
    n = lib().orc_route(_p(logits), logits.size, k, _p(idx), _p(w))
    return idx[:n], w[:n]


def expert_shape(gu_type, down_type, hidden, ff):
    def nbytes(ty, cols, rows):
        if ty >= 1000:
            half = ty >= 1030
            bits = ty - 1030 if half else ty % 10
            return exl3_blob_len(cols, rows, bits, half)
        e, b = C.c_uint64(), C.c_uint64()
        assert lib().orc_block_layout(ty, C.byref(e), C.byref(b)) == 0
        return rows * (cols // e.value) * b.value
    g = nbytes(gu_type, hidden, ff)
    return ExpertShape(gu_type, down_type, hidden, ff, g, g, nbytes(down_type, ff, hidden))


def moe_token(shape, experts, k, logits, u, shared_shape=None, shared=None, shared_gate_logit=0.0, threads=0):
    """experts: list of contiguous uint8 arrays [gate|up|down], one per expert.  Returns (y, route_idx, route_w)."""
    logits, u = _c(logits, np.float32), _c(u, np.float32)
    ne = len(experts)
    ptrs = (C.c_void_p * ne)(*[_p(e) for e in experts])
    y = np.empty(shape.hidden, np.float32)
    ridx = np.zeros(k, np.uint32)
    rw = np.zeros(k, np.float32)
    sh_ptr = _p(shared) if shared is not None else None
    r = lib().orc_moe_token(C.byref(shape), ptrs, ne, k, _p(logits), C.byref(shared_shape) if shared_shape is not None else None,
                            sh_ptr, shared_gate_logit, _p(u), _p(y), _p(ridx), _p(rw), threads)
    assert r == 0, r
    return y, ridx, rw


def quantize_act(x, blk=32):
    x = _c(x, np.float32).ravel()
    q = np.empty(x.size, np.int8)
    d = np.empty(x.size // blk, np.float32)
    s = np.empty(x.size // blk, np.int32)
    lib().orc_quantize_act(_p(x), x.size, blk, _p(q), _p(d), _p(s))
    return q, d, s


def iq3s_int8(block):
    block = _c(block, np.uint8)
    q = np.empty(256, np.int8)
    s = np.empty(8, np.float32)
    lib().orc_iq3s_int8(_p(block), _p(q), _p(s))
    return q, s


def iq3s_row_dot_q8(row, cols, q, d):
    row, q, d = _c(row, np.uint8), _c(q, np.int8), _c(d, np.float32)
    isums = np.empty(cols // 32, np.int32)
    v = lib().orc_iq3s_row_dot_q8(_p(row), cols, _p(q), _p(d), _p(isums))
    return v, isums


def expert_int8(expert, hidden, ff, xq, xd):
    expert, xq, xd = _c(expert, np.uint8), _c(xq, np.int8), _c(xd, np.float32)
    out = np.empty(hidden, np.float32)
    act = np.empty(ff, np.float32)
    r = lib().orc_expert_int8(_p(expert), hidden, ff, _p(xq), _p(xd), _p(out), _p(act))
    assert r == 0, r
    return out, act


def argmax(v):
    v = _c(v, np.float32)
    return lib().orc_argmax(_p(v), v.size)


def topk(row, k=64):
    row = _c(row, np.float32)
    vals = np.empty(k, np.float32)
    ids = np.empty(k, np.uint32)
    lib().orc_topk(_p(row), row.size, k, _p(vals), _p(ids))
    return vals, ids


def accept(want, drafts):
    want, drafts = _c(want, np.uint32), _c(drafts, np.uint32)
    return lib().orc_accept(_p(want), _p(drafts), drafts.size)


def lookup_draft(hist, k, lens=(3, 2)):
    hist, lens = _c(hist, np.uint32), _c(lens, np.uint32)
    out = np.zeros(max(k, 1), np.uint32)
    L = lib()
    L.orc_lookup_draft.restype = C.c_int
    L.orc_lookup_draft.argtypes = [C.c_void_p, C.c_size_t, C.c_int, C.c_void_p, C.c_int, C.c_void_p]
    n = L.orc_lookup_draft(_p(hist), hist.size, k, _p(lens), lens.size, _p(out))
    return out[:n].tolist()


def q2_proxy_build(inf, outf, bits, blob):
    """The 2-bit screen of an EXL3 head: (w_q2 u32[outf/128][inf/128][2][128][4], w_sc u16[outf/128][inf/128][128])."""
    blob = _c(blob, np.uint8)
    wq = np.zeros((outf // 128, inf // 128, 2, 128, 4), np.uint32)
    ws = np.zeros((outf // 128, inf // 128, 128), np.uint16)
    r = lib().orc_q2_proxy_build(inf, outf, bits, _p(blob), blob.size, _p(wq), _p(ws))
    assert r == 0, r
    return wq, ws


def q2_proxy_quant_x(blob, x, inf):
    """Rows x[m][inf] -> (xq u32[m][inf/4], x_sc f32[m][inf/128], x_corr f32[m][inf/128])."""
    blob = _c(blob, np.uint8)
    x = _c(x, np.float32).reshape(-1, inf)
    m = x.shape[0]
    xq = np.zeros((m, inf // 4), np.uint32)
    sc = np.zeros((m, inf // 128), np.float32)
    corr = np.zeros((m, inf // 128), np.float32)
    for j in range(m):
        lib().orc_q2_proxy_quant_x(_p(blob), _p(x[j]), inf, _p(xq[j]), _p(sc[j]), _p(corr[j]))
    return xq, sc, corr


def q2_proxy_bmax(wq, ws, xq, sc, corr):
    """bmax f32[m][outf/128] from the screen and the rows' codes."""
    n_ob, n_b = ws.shape[0], ws.shape[1]
    m = xq.shape[0]
    out = np.zeros((m, n_ob), np.float32)
    for j in range(m):
        lib().orc_q2_proxy_bmax(_p(wq), _p(ws), _p(xq[j]), _p(sc[j]), _p(corr[j]), n_ob, n_b * 128, _p(out[j]))
    return out


def q2_proxy_pick(bmax, k_blk, max_sel):
    """The chosen blocks (ascending) of all rows of bmax together, cut to max_sel, and the number marked before the cut."""
    bmax = _c(bmax, np.float32)
    m, n_ob = bmax.shape
    sel = np.zeros(1 + max_sel, np.uint32)
    n = lib().orc_q2_proxy_pick(_p(bmax), m, n_ob, k_blk, max_sel, _p(sel))
    return sel[1:1 + int(sel[0])].copy(), int(n)
