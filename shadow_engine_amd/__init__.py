"""shadow_engine_amd: the speculative-verify hot path of ShadowZero (quantized MoE expert products over Q8_0 / IQ3_S / EXL3,
routing + SwiGLU + combine, lm_head arg-max and greedy draft acceptance) on AMD MI355X.

This module is the thin Python face of libshadowzero_hip.so (the C ABI of include/shadowzero_hip.h), shaped after the
reference's own operator surface: `GpuBackend.matvec` (crates/shadowzero-cuda/src/backend.rs:57), the `Program.launch`
registry check (kernels.rs:546) and the `GpuSession` verify operations (session.rs:6076, 8222, 7034).  There is no CPU
fallback: without the built library, or without a GPU, the calls raise.
"""
import ctypes as C
import os

import numpy as np

PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG, "libshadowzero_hip.so")

Q8_0, IQ3_S = 8, 21
F32, F16, BF16 = 0, 1, 30


def EXL3_HALF(bits):
    """Type id of an EXL3 projection at bits + 1/2 bits a weight (bits = 1..3)."""
    return 1030 + bits


def EXL3(bits):
    """ggml-style type id of an EXL3 projection with the "mul1" codebook at `bits` bits a weight."""
    return 1020 + bits


class SzError(RuntimeError):
    pass


class Arg(C.Structure):
    _fields_ = [("kind", C.c_int32), ("pad", C.c_int32), ("value", C.c_uint64)]

    @staticmethod
    def ptr(p):
        return Arg(0, 0, int(p))

    @staticmethod
    def u32(v):
        return Arg(1, 0, int(v) & 0xffffffff)

    @staticmethod
    def i32(v):
        return Arg(2, 0, int(v) & 0xffffffff)

    @staticmethod
    def u64(v):
        return Arg(3, 0, int(v))

    @staticmethod
    def f32(v):
        return Arg(4, 0, int(np.array([v], np.float32).view(np.uint32)[0]))


class HcConfig(C.Structure):
    _fields_ = [("hidden", C.c_uint32), ("streams", C.c_uint32), ("rank", C.c_uint32), ("max_rows", C.c_uint32), ("eps", C.c_float),
                ("down_type", C.c_int32), ("up_type", C.c_int32), ("inject_type", C.c_int32), ("norm_w", C.c_uint64),
                ("down_w", C.c_uint64), ("up_w", C.c_uint64), ("inject_w", C.c_uint64)]


class SessionConfig(C.Structure):
    _fields_ = [("hidden", C.c_uint32), ("ff", C.c_uint32), ("n_expert", C.c_uint32), ("top_k", C.c_uint32), ("n_layers", C.c_uint32),
                ("vocab", C.c_uint32), ("max_rows", C.c_uint32), ("reserved", C.c_uint32)]


class TensorInfo(C.Structure):
    """sz_tensor_info: one tensor of a GGUF (TensorInfo, crates/shadowzero-model/src/gguf.rs:224)."""
    _fields_ = [("type", C.c_uint32), ("n_dims", C.c_uint32), ("shard", C.c_uint32), ("has_layout", C.c_uint32), ("dims", C.c_uint64 * 8),
                ("offset", C.c_uint64), ("nbytes_layout", C.c_uint64), ("nbytes_span", C.c_uint64), ("nbytes", C.c_uint64)]


class StInfo(C.Structure):
    """sz_st_info: one tensor of a safetensors file (StTensor, safetensors.rs:11)."""
    _fields_ = [("dtype", C.c_char * 8), ("n_dims", C.c_uint32), ("file", C.c_uint32), ("shape", C.c_uint64 * 8), ("start", C.c_uint64),
                ("end", C.c_uint64)]


class LayerLayout(C.Structure):
    """sz_layer_layout: where the parts of a staged MoE layer lie in its device buffer."""
    _fields_ = [("type", C.c_int32), ("shared_type", C.c_int32), ("router_type", C.c_int32), ("gate_type", C.c_int32), ("n_expert", C.c_uint32),
                ("gap", C.c_uint32), ("hidden", C.c_uint64), ("ff", C.c_uint64), ("gate_up_bytes", C.c_uint64), ("down_bytes", C.c_uint64),
                ("shared_gate_up_bytes", C.c_uint64), ("stride", C.c_uint64), ("shared_offset", C.c_uint64), ("router_offset", C.c_uint64),
                ("gate_offset", C.c_uint64), ("bytes", C.c_uint64), ("experts_offset", C.c_uint64)]


_u64, _u32, _i32, _vp = C.c_uint64, C.c_uint32, C.c_int32, C.c_void_p
_SIGNATURES = {
    "sz_last_error": (C.c_char_p, []),
    "sz_init": (_i32, [_i32]),
    "sz_device_count": (_i32, [C.POINTER(_i32)]),
    "sz_device_name": (_i32, [C.c_char_p, _u64]),
    "sz_mem_info": (_i32, [C.POINTER(_u64), C.POINTER(_u64)]),
    "sz_malloc": (_i32, [C.POINTER(_u64), _u64]),
    "sz_free": (_i32, [_u64]),
    "sz_upload": (_i32, [_u64, _vp, _u64]),
    "sz_download": (_i32, [_vp, _u64, _u64]),
    "sz_memset": (_i32, [_u64, _i32, _u64, _u64]),
    "sz_stream_create": (_i32, [C.POINTER(_u64)]),
    "sz_stream_destroy": (_i32, [_u64]),
    "sz_stream_synchronize": (_i32, [_u64]),
    "sz_synchronize": (_i32, []),
    "sz_event_create": (_i32, [C.POINTER(_u64)]),
    "sz_event_destroy": (_i32, [_u64]),
    "sz_event_record": (_i32, [_u64, _u64]),
    "sz_stream_wait_event": (_i32, [_u64, _u64]),
    "sz_event_synchronize": (_i32, [_u64]),
    "sz_event_elapsed_ms": (_i32, [_u64, _u64, C.POINTER(C.c_float)]),
    "sz_capture_begin": (_i32, [_u64]),
    "sz_capture_end": (_i32, [_u64, C.POINTER(_u64)]),
    "sz_graph_launch": (_i32, [_u64, _u64]),
    "sz_graph_destroy": (_i32, [_u64]),
    "sz_launch": (_i32, [C.c_char_p, _u32, _u32, _u32, _u32, _u32, _u32, _u32, _u64, C.POINTER(Arg), _i32]),
    "sz_kernel_count": (_i32, []),
    "sz_kernel_info": (_i32, [_i32, C.POINTER(C.c_char_p), C.POINTER(C.c_char_p), C.POINTER(_i32), C.POINTER(_i32), _i32]),
    "sz_launch_count": (_u64, []),
    "sz_ktime_begin": (_i32, [C.c_char_p]),
    "sz_ktime_entry": (_i32, [_i32, C.POINTER(C.c_char_p), C.POINTER(_u64), C.POINTER(C.c_double)]),
    "sz_ktime_end": (_i32, []),
    "sz_program_cache_key": (_i32, [C.c_char_p, C.c_char_p]),
    "sz_program_cache_key_rtc": (_i32, [C.c_char_p, C.c_char_p]),
    "sz_program_aot_options": (C.c_char_p, [C.c_char_p]),
    "sz_program_file_count": (_i32, []),
    "sz_program_file_name": (C.c_char_p, [_i32]),
    "sz_cache_dir": (C.c_char_p, []),
    "sz_compile_options": (C.c_char_p, []),
    "sz_program_write_source": (_i32, [C.c_char_p, C.c_char_p]),
    "sz_rtc_compile": (_i32, [C.c_char_p, C.c_char_p, C.POINTER(_u64), C.POINTER(C.c_char_p)]),
    "sz_backend_new": (_vp, [_u64]),
    "sz_backend_free": (None, [_vp]),
    "sz_matvec": (_i32, [_vp, _i32, _u64, _u64, _vp, _u64, C.c_char_p, _vp, _vp]),
    "sz_backend_resident_bytes": (_u64, [_vp]),
    "sz_backend_uploads": (_u64, [_vp]),
    "sz_dequantize": (_i32, [_i32, _u64, _u64, _u64, _u64, _u64]),
    "sz_exl3_codebook": (_i32, [_u64, _u64]),
    "sz_matvec_cols_scratch": (_u64, [_i32, _u64, _u64, _u32]),
    "sz_matvec_cols": (_i32, [_i32, _u64, _u64, _u64, _u64, _u32, _u64, _u32, _u32, _u64, _u64, _u64]),
    "sz_session_buffer": (_u64, [_vp, _i32]),
    "sz_matvec_cols_static": (_i32, [_i32, _u64, _u64, _u64, _u64, _u32, _u64, _u32, _u32, _u64]),
    "sz_session_new": (_vp, [C.POINTER(SessionConfig)]),
    "sz_session_free": (None, [_vp]),
    "sz_session_set_layer": (_i32, [_vp, _u32, _i32, _u64, _u64, _i32, _u64]),
    "sz_session_set_layer_spaced": (_i32, [_vp, _u32, _i32, _u64, _u64, _u64, _i32, _u64]),
    "sz_layer_spacing": (None, [_i32, _u64, _u64, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]),
    "sz_session_set_head": (_i32, [_vp, _i32, _u64]),
    "sz_session_set_head_proxy": (_i32, [_vp, _u32]),
    "sz_session_set_graph": (_i32, [_vp, _i32]),
    "sz_session_set_expert_mode": (_i32, [_vp, _i32]),
    "sz_exl3_head_lds_bytes": (_u32, [_i32, _u32, _u32]),
    "sz_moe_layer_verify": (_i32, [_vp, _u32, _u32, _u64, _u64, _u64, _u64, _u64]),
    "sz_session_set_router": (_i32, [_vp, _u32, _i32, _u64, _i32, _u64]),
    "sz_moe_router_verify": (_i32, [_vp, _u32, _u32, _u64, _u64]),
    "sz_session_router_outputs": (_i32, [_vp, _vp, _vp]),
    "sz_moe_block_verify": (_i32, [_vp, _u32, _u32, _u64, _u64, _u64]),
    "sz_session_last_route": (_i32, [_vp, _u32, _vp, _vp, _u64]),
    "sz_hc_new": (_vp, [_vp]),
    "sz_hc_free": (None, [_vp]),
    "sz_hc_read": (_i32, [_vp, _u32, _u64, _u64, _u64]),
    "sz_hc_gains": (_u64, [_vp]),
    "sz_hc_write": (_i32, [_u64, _u64, _u64, _u32, _u32, _u32, _u64]),
    "sz_head_argmax": (_i32, [_vp, _u32, _u64, _u64, _u64]),
    "sz_head_top": (_i32, [_vp, _u32, _u64, _vp, _u64]),
    "sz_head_logits": (_i32, [_vp, _u32, _u64, _u64, _u64]),
    "sz_verify_accept": (_i32, [_vp, _vp, _u32, C.POINTER(_u32)]),
    "sz_verify_round": (_i32, [_vp, _u32, _u64, _u64, _u64, _u64, _u64, _u64, _u64, _u64]),
    "sz_lookup_draft": (_i32, [_vp, _u64, _u32, _vp, _u32, _vp, C.POINTER(_u32)]),
    "sz_snapshot_new": (_i32, [_vp, _vp, _u32, C.POINTER(_vp)]),
    "sz_snapshot_free": (None, [_vp]),
    "sz_snapshot_bytes": (_u64, [_vp]),
    "sz_snapshot_take": (_i32, [_vp, _u64]),
    "sz_snapshot_restore": (_i32, [_vp, _u64]),
    "sz_snapshot_download": (_i32, [_vp, _u32, _vp, _u64]),
    "sz_copy_ranges": (_i32, [_vp, _u32, _u64]),
    "sz_quantize_act": (_i32, [_u64, _u64, _u64, _u64, _u64]),
    "sz_moe_prefill_chunk": (_i32, [_vp, _u32, _u32, _u64, _u64, _u64, _u64, _u64]),
    "sz_prefill_buffer": (_u64, [_vp, _i32]),
    "sz_type_info": (_i32, [_u32, C.c_char_p, _u64, C.POINTER(_u64), C.POINTER(_u64)]),
    "sz_gguf_shard_paths": (_i32, [C.c_char_p, _u32, C.c_char_p, _u64, C.POINTER(_u32)]),
    "sz_gguf_open": (_i32, [C.c_char_p, C.POINTER(_vp)]),
    "sz_gguf_close": (None, [_vp]),
    "sz_gguf_tensor_count": (_u64, [_vp]),
    "sz_gguf_tensor_at": (_i32, [_vp, _u64, C.c_char_p, _u64, C.POINTER(TensorInfo)]),
    "sz_gguf_tensor": (_i32, [_vp, C.c_char_p, C.POINTER(TensorInfo)]),
    "sz_gguf_tensor_bytes": (_u64, [_vp]),
    "sz_gguf_shard_count": (_u32, [_vp]),
    "sz_gguf_shard": (_i32, [_vp, _u32, C.c_char_p, _u64, C.POINTER(_u32), C.POINTER(_u64), C.POINTER(_u64), C.POINTER(_u64)]),
    "sz_gguf_kv_count": (_u64, [_vp]),
    "sz_gguf_kv_key": (_i32, [_vp, _u64, C.c_char_p, _u64]),
    "sz_gguf_kv_type": (_i32, [_vp, C.c_char_p, C.POINTER(_u32), C.POINTER(_u32), C.POINTER(_u64)]),
    "sz_gguf_kv_u64": (_i32, [_vp, C.c_char_p, C.POINTER(_u64)]),
    "sz_gguf_arch_u64": (_i32, [_vp, C.c_char_p, C.POINTER(_u64)]),
    "sz_gguf_kv_f64": (_i32, [_vp, C.c_char_p, C.POINTER(C.c_double)]),
    "sz_gguf_kv_str": (_i32, [_vp, C.c_char_p, C.c_char_p, _u64]),
    "sz_gguf_kv_array_u64": (_i32, [_vp, C.c_char_p, _u64, C.POINTER(_u64)]),
    "sz_gguf_kv_array_f64": (_i32, [_vp, C.c_char_p, _u64, C.POINTER(C.c_double)]),
    "sz_gguf_kv_array_str": (_i32, [_vp, C.c_char_p, _u64, C.c_char_p, _u64]),
    "sz_gguf_block_index": (C.c_int64, [C.c_char_p]),
    "sz_gguf_read_tensor": (_i32, [_vp, C.c_char_p, _vp, _u64]),
    "sz_gguf_expert_range": (_i32, [_vp, C.c_char_p, _u64, C.POINTER(_u32), C.POINTER(_u64), C.POINTER(_u64)]),
    "sz_st_open": (_i32, [C.POINTER(C.c_char_p), _u32, C.POINTER(_vp)]),
    "sz_st_open_dir": (_i32, [C.c_char_p, C.POINTER(_vp)]),
    "sz_st_close": (None, [_vp]),
    "sz_st_tensor_count": (_u64, [_vp]),
    "sz_st_file_count": (_u32, [_vp]),
    "sz_st_file": (_i32, [_vp, _u32, C.c_char_p, _u64]),
    "sz_st_tensor_at": (_i32, [_vp, _u64, C.c_char_p, _u64, C.POINTER(StInfo)]),
    "sz_st_tensor": (_i32, [_vp, C.c_char_p, C.POINTER(StInfo)]),
    "sz_st_read": (_i32, [_vp, C.c_char_p, _u64, _u64, _vp]),
    "sz_exl3_shape": (_i32, [_vp, C.c_char_p, C.POINTER(_u64), C.POINTER(_u64), C.POINTER(_i32)]),
    "sz_exl3_contiguous": (_i32, [_vp, C.c_char_p, C.POINTER(_u32), C.POINTER(_u64), C.POINTER(_u64)]),
    "sz_exl3_blob_len": (_u64, [_u64, _u64, _i32]),
    "sz_exl3_read_blob": (_i32, [_vp, C.c_char_p, _vp, _u64]),
    "sz_gguf_layer_layout": (_i32, [_vp, _u32, C.POINTER(LayerLayout)]),
    "sz_exl3_layer_layout": (_i32, [_vp, _u32, _u32, C.POINTER(LayerLayout)]),
    "sz_gguf_stage_layer": (_i32, [_vp, _u32, _u64, _u64, _u64]),
    "sz_exl3_stage_layer": (_i32, [_vp, _u32, _u32, _u64, _u64, _u64]),
    "sz_gguf_stage_tensor": (_i32, [_vp, C.c_char_p, _u64, _u64, _u64]),
    "sz_st_stage_tensor": (_i32, [_vp, C.c_char_p, _u64, _u64, _u64]),
    "sz_exl3_stage_blob": (_i32, [_vp, C.c_char_p, _u64, _u64, _u64]),
}

_lib = None


def lib():
    """The loaded C ABI library; raises if it has not been built (python -m shadow_engine_amd.build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise SzError(f"{LIB_PATH} is not built: run `python -m shadow_engine_amd.build`")
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def exported_symbols():
    return sorted(_SIGNATURES)


def last_error():
    return lib().sz_last_error().decode(errors="replace")


def check(status):
    if status != 0:
        raise SzError(last_error())


def init(device=0):
    check(lib().sz_init(device))


def device_count():
    n = _i32()
    check(lib().sz_device_count(C.byref(n)))
    return n.value


def device_name():
    buf = C.create_string_buffer(256)
    check(lib().sz_device_name(buf, 256))
    return buf.value.decode()


def kernels():
    """The registry: [(name, file, [parameter kinds])] (kernels.rs FILES)."""
    L = lib()
    out = []
    for i in range(L.sz_kernel_count()):
        name, file, n = C.c_char_p(), C.c_char_p(), _i32()
        kinds = (_i32 * 24)()
        check(L.sz_kernel_info(i, C.byref(name), C.byref(file), C.byref(n), kinds, 24))
        out.append((name.value.decode(), file.value.decode(), list(kinds[:n.value])))
    return out


def launch(name, grid, block, shared, stream, args):
    """Program::launch (kernels.rs:546): checked against the registry before anything reaches the driver."""
    arr = (Arg * max(len(args), 1))(*args)
    check(lib().sz_launch(name.encode(), grid[0], grid[1], grid[2], block[0], block[1], block[2], shared, stream, arr, len(args)))


def ktime_begin(prefix=""):
    """Time every launch whose kernel name starts with `prefix` between two events (SHADOWZERO_KTIME, kernels.rs:570)."""
    check(lib().sz_ktime_begin(prefix.encode()))


def ktime_end():
    """{kernel: (launches, total milliseconds)} since ktime_begin; stops timing."""
    out, i = {}, 0
    while True:
        name, n, ms = C.c_char_p(), _u64(), C.c_double()
        if lib().sz_ktime_entry(i, C.byref(name), C.byref(n), C.byref(ms)) != 0:
            break
        out[name.value.decode()] = (n.value, ms.value)
        i += 1
    check(lib().sz_ktime_end())
    return out


def download(out, dev_ptr):
    """Device memory at dev_ptr into the numpy array `out` (synchronous)."""
    check(lib().sz_download(out.ctypes.data, dev_ptr, out.nbytes))
    return out


class DeviceBuffer:
    """driver.rs DeviceBuffer: device memory owned by this object."""

    def __init__(self, nbytes):
        p = _u64()
        check(lib().sz_malloc(C.byref(p), nbytes))
        self.ptr, self.nbytes = p.value, nbytes

    @staticmethod
    def from_numpy(a):
        a = np.ascontiguousarray(a)
        b = DeviceBuffer(max(a.nbytes, 1))
        b.upload(a)
        return b

    def upload(self, a):
        a = np.ascontiguousarray(a)
        assert a.nbytes <= self.nbytes
        check(lib().sz_upload(self.ptr, a.ctypes.data, a.nbytes))

    def download(self, dtype, count=None):
        dtype = np.dtype(dtype)
        n = self.nbytes // dtype.itemsize if count is None else count
        out = np.empty(n, dtype)
        check(lib().sz_download(out.ctypes.data, self.ptr, out.nbytes))
        return out

    def fill(self, byte=0, stream=0, offset=0, nbytes=None):
        """driver.rs:419 DeviceBuffer::zero, for any byte and range; asynchronous on the stream."""
        n = self.nbytes - offset if nbytes is None else nbytes
        assert 0 <= offset and offset + n <= self.nbytes
        check(lib().sz_memset(self.ptr + offset, byte, n, stream))

    def free(self):
        if self.ptr:
            lib().sz_free(self.ptr)
            self.ptr = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Stream:
    def __init__(self):
        s = _u64()
        check(lib().sz_stream_create(C.byref(s)))
        self.handle = s.value

    def synchronize(self):
        check(lib().sz_stream_synchronize(self.handle))

    def wait_event(self, event):
        check(lib().sz_stream_wait_event(self.handle, event.handle))

    def __del__(self):
        try:
            if self.handle:
                lib().sz_stream_destroy(self.handle)
        except Exception:
            pass


class Event:
    def __init__(self):
        e = _u64()
        check(lib().sz_event_create(C.byref(e)))
        self.handle = e.value

    def record(self, stream=0):
        check(lib().sz_event_record(self.handle, stream))

    def synchronize(self):
        check(lib().sz_event_synchronize(self.handle))

    def since(self, start):
        ms = C.c_float()
        check(lib().sz_event_elapsed_ms(start.handle, self.handle, C.byref(ms)))
        return ms.value

    def __del__(self):
        try:
            if self.handle:
                lib().sz_event_destroy(self.handle)
        except Exception:
            pass


class GpuBackend:
    """forward::Backend on the GPU (backend.rs): y = W x from host bytes, resident by key within a budget."""

    def __init__(self, budget=1 << 30):
        self._h = lib().sz_backend_new(budget)
        if not self._h:
            raise SzError(last_error())

    def matvec(self, ggml_type, cols, rows, data, key, x):
        data = np.ascontiguousarray(data, np.uint8)
        x = np.ascontiguousarray(x, np.float32)
        y = np.empty(rows, np.float32)
        k = key.encode() if key is not None else None
        check(lib().sz_matvec(self._h, ggml_type, cols, rows, data.ctypes.data, data.size, k, x.ctypes.data, y.ctypes.data))
        return y

    @property
    def resident_bytes(self):
        return lib().sz_backend_resident_bytes(self._h)

    @property
    def uploads(self):
        return lib().sz_backend_uploads(self._h)

    def __del__(self):
        try:
            if self._h:
                lib().sz_backend_free(self._h)
                self._h = None
        except Exception:
            pass


def dequantize(ggml_type, w_dev, out_dev, cols, rows, stream=0):
    check(lib().sz_dequantize(ggml_type, w_dev, out_dev, cols, rows, stream))


def exl3_codebook(out_dev, stream=0):
    check(lib().sz_exl3_codebook(out_dev, stream))


def matvec_cols_scratch(ggml_type, cols, rows, m):
    return lib().sz_matvec_cols_scratch(ggml_type, cols, rows, m)


def matvec_cols(ggml_type, w_dev, cols, rows, x_dev, xs, y_dev, ys, m, scratch=0, scratch_bytes=0, stream=0):
    check(lib().sz_matvec_cols(ggml_type, w_dev, cols, rows, x_dev, xs, y_dev, ys, m, scratch, scratch_bytes, stream))


STATIC_WORKSPACE_BYTES = 4 << 20


def matvec_cols_static(ggml_type, w_dev, cols, rows, x_dev, xs, y_dev, ys, m, stream=0):
    """sz_matvec_cols on the library's own static device workspace: allocates nothing."""
    check(lib().sz_matvec_cols_static(ggml_type, w_dev, cols, rows, x_dev, xs, y_dev, ys, m, stream))


def program_keys():
    """{kernel file: cache key of the code object built ahead of time from its current source}."""
    out = {}
    L = lib()
    for i in range(L.sz_program_file_count()):
        name = L.sz_program_file_name(i)
        key = C.create_string_buffer(65)
        if L.sz_program_cache_key(name, key) == 0:
            out[name.decode()] = key.value.decode()
    return out


def verify_accept(ids, drafts):
    """engine.rs:2377-2408: keep = 1 + the leading drafts that equal the model's choices."""
    ids = np.ascontiguousarray(ids, np.uint32)
    drafts = np.ascontiguousarray(drafts, np.uint32)
    keep = _u32()
    check(lib().sz_verify_accept(ids.ctypes.data, drafts.ctypes.data, drafts.size, C.byref(keep)))
    return keep.value


def quantize_act(x_dev, n, q_dev, d_dev, stream=0):
    check(lib().sz_quantize_act(x_dev, n, q_dev, d_dev, stream))


class Session:
    """The verify-path subset of GpuSession (session.rs): resident experts per layer, the MoE block for a verify batch, the
    head with arg-max / top-64, and a whole verify round replayed as a HIP graph."""

    def __init__(self, hidden, ff, n_expert, top_k, n_layers, vocab, max_rows=8):
        self.cfg = SessionConfig(hidden, ff, n_expert, top_k, n_layers, vocab, max_rows, 0)
        self._h = lib().sz_session_new(C.byref(self.cfg))
        if not self._h:
            raise SzError(last_error())

    def set_layer(self, layer, expert_type, experts_dev, stride, shared_type=0, shared_dev=0, gap=0):
        """gap: bytes between an expert's projections (0: contiguous [gate|up|down]; layer_spacing() gives the one that puts
        an EXL3 layer's trellises on 128-byte lines)."""
        check(lib().sz_session_set_layer_spaced(self._h, layer, expert_type, experts_dev, stride, gap, shared_type, shared_dev))

    def set_head(self, ggml_type, w_dev):
        check(lib().sz_session_set_head(self._h, ggml_type, w_dev))

    def set_head_proxy(self, k_blk):
        """Build (k_blk > 0) or drop (0) the inexact 2-bit screen of the EXL3 head that head_top then uses."""
        check(lib().sz_session_set_head_proxy(self._h, k_blk))

    def set_graph(self, enabled):
        check(lib().sz_session_set_graph(self._h, int(enabled)))

    def set_expert_mode(self, mode):
        """0 (default): the exact EXL3 layer kernels, 1: the matrix cores on the codebook's f16 values, 2: on the linearised codebook."""
        check(lib().sz_session_set_expert_mode(self._h, int(mode)))

    def buffer(self, which):
        """Device address of a batch buffer: 0 plan, 1 gate/up partial sums, 2 down products, 3/4 GGUF rows, 5..12 the head screen's."""
        return lib().sz_session_buffer(self._h, which)

    def moe_layer_verify(self, layer, m, u_dev, rl_dev, sgl_dev, y_dev, stream=0):
        check(lib().sz_moe_layer_verify(self._h, layer, m, u_dev, rl_dev, sgl_dev, y_dev, stream))

    def set_router(self, layer, router_type, router_dev, gate_type=0, gate_dev=0):
        check(lib().sz_session_set_router(self._h, layer, router_type, router_dev, gate_type, gate_dev))

    def moe_router_verify(self, layer, m, u_dev, stream=0):
        check(lib().sz_moe_router_verify(self._h, layer, m, u_dev, stream))

    def router_outputs(self):
        """Device addresses of the router's outputs: (rl[max_rows][n_expert], sgl[max_rows])."""
        rl, sgl = _u64(), _u64()
        check(lib().sz_session_router_outputs(self._h, C.byref(rl), C.byref(sgl)))
        return rl.value, sgl.value

    def moe_block_verify(self, layer, m, u_dev, y_dev, stream=0):
        check(lib().sz_moe_block_verify(self._h, layer, m, u_dev, y_dev, stream))

    def last_route(self, m, stream=0):
        k = self.cfg.top_k
        idx = np.empty((m, k), np.uint32)
        w = np.empty((m, k), np.float32)
        check(lib().sz_session_last_route(self._h, m, idx.ctypes.data, w.ctypes.data, stream))
        return idx, w

    def head_argmax(self, m, u_dev, ids_dev, stream=0):
        check(lib().sz_head_argmax(self._h, m, u_dev, ids_dev, stream))

    def head_logits(self, m, u_dev, logits_dev, stream=0):
        check(lib().sz_head_logits(self._h, m, u_dev, logits_dev, stream))

    def head_top(self, m, u_dev, stream=0):
        """[(values[64], ids[64])] per row, as step_batch_verify_top hands the sampler (session.rs:6061)."""
        top = np.empty((m, 128), np.uint32)
        check(lib().sz_head_top(self._h, m, u_dev, top.ctypes.data, stream))
        return [(top[r, :64].view(np.float32).copy(), top[r, 64:].copy()) for r in range(m)]

    def verify_round(self, m, u_dev, rl_dev, sgl_dev, y_dev, head_u_dev, drafts_dev, out_dev, stream=0):
        check(lib().sz_verify_round(self._h, m, u_dev, rl_dev, sgl_dev, y_dev, head_u_dev, drafts_dev, out_dev, stream))

    def moe_prefill_chunk(self, layer, tokens, x_dev, rl_dev, sgl_dev, y_dev, stream=0):
        check(lib().sz_moe_prefill_chunk(self._h, layer, tokens, x_dev, rl_dev, sgl_dev, y_dev, stream))

    def prefill_buffer(self, which):
        return lib().sz_prefill_buffer(self._h, which)

    def __del__(self):
        try:
            if self._h:
                lib().sz_session_free(self._h)
                self._h = None
        except Exception:
            pass


class HyperConnection:
    """hc_read / hc_write around a sublayer (forward.rs:797-817, 1078-1084) on resident weights, for up to max_rows rows."""

    def __init__(self, hidden, streams, rank, eps, norm_dev, down_type, down_dev, up_type, up_dev, inject_type=0, inject_dev=0, max_rows=8):
        self.cfg = HcConfig(hidden, streams, rank, max_rows, eps, down_type, up_type, inject_type, norm_dev, down_dev, up_dev, inject_dev)
        self._h = lib().sz_hc_new(C.byref(self.cfg))
        if not self._h:
            raise SzError(last_error())

    def read(self, m, r_dev, u_dev, stream=0):
        check(lib().sz_hc_read(self._h, m, r_dev, u_dev, stream))

    @property
    def gains(self):
        """Device address of g[max_rows][streams], written by the last read (when the read has an inject matrix)."""
        return lib().sz_hc_gains(self._h)

    def __del__(self):
        try:
            if self._h:
                lib().sz_hc_free(self._h)
                self._h = None
        except Exception:
            pass


def hc_write(r_dev, g_dev, y_dev, m, hidden, streams, stream=0):
    check(lib().sz_hc_write(r_dev, g_dev, y_dev, m, hidden, streams, stream))


def lookup_draft(hist, k, lens=(3, 2)):
    """The lookup drafter (engine.rs:823-839): up to k tokens that followed the last earlier occurrence of the history's tail."""
    h = np.ascontiguousarray(hist, np.uint32)
    ln = np.ascontiguousarray(lens, np.uint32)
    out, n = np.zeros(max(k, 1), np.uint32), _u32()
    check(lib().sz_lookup_draft(h.ctypes.data, h.size, k, ln.ctypes.data, ln.size, out.ctypes.data, C.byref(n)))
    return out[:n.value].tolist()


class Snapshot:
    """A speculative pass's rollback point on the device (GpuSession::snapshot_again / restore_local, session.rs:3407-3510):
    `ranges` = [(device address, bytes), ...] of the state; take() saves it, restore() puts it back, one launch each."""

    def __init__(self, ranges):
        a = np.ascontiguousarray([r[0] for r in ranges], np.uint64)
        b = np.ascontiguousarray([r[1] for r in ranges], np.uint64)
        h = _vp()
        check(lib().sz_snapshot_new(a.ctypes.data, b.ctypes.data, len(ranges), C.byref(h)))
        self._h, self._sizes = h, [int(x) for x in b]

    @property
    def bytes(self):
        return lib().sz_snapshot_bytes(self._h)

    def take(self, stream=0):
        check(lib().sz_snapshot_take(self._h, stream))

    def restore(self, stream=0):
        check(lib().sz_snapshot_restore(self._h, stream))

    def saved(self, i):
        """The saved copy of range i as bytes (synchronizes with the device)."""
        if not 0 <= i < len(self._sizes):
            raise SzError(f"no range {i}")
        out = np.empty(self._sizes[i], np.uint8)
        check(lib().sz_snapshot_download(self._h, i, out.ctypes.data, out.size))
        return out

    def close(self):
        if self._h and _lib is not None:
            lib().sz_snapshot_free(self._h)
        self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def copy_ranges(ranges, stream=0):
    """[(dst, src, bytes), ...] device ranges copied by one launch (copy_many_with, session.rs:3385-3404); waits for it."""
    t = np.ascontiguousarray(ranges, np.uint64).reshape(-1, 3)
    check(lib().sz_copy_ranges(t.ctypes.data, t.shape[0], stream))


# ---- the checkpoint formats either side of the path --------------------------------------------------------------------
def type_info(type_id):
    """(name, block elements, block bytes) of a ggml type id; (name, 0, 0) when it has no block (GgmlType, gguf.rs:152-178)."""
    buf, be, bb = C.create_string_buffer(32), _u64(), _u64()
    check(lib().sz_type_info(type_id, buf, 32, C.byref(be), C.byref(bb)))
    return buf.value.decode(), be.value, bb.value


def gguf_shard_paths(path):
    """The file names of a model opened by any of its shards (shard_paths, gguf.rs:442)."""
    n = _u32()
    check(lib().sz_gguf_shard_paths(os.fsencode(path), 0, None, 0, C.byref(n)))
    out = []
    for i in range(n.value):
        buf = C.create_string_buffer(len(os.fsencode(path)) + 64)
        check(lib().sz_gguf_shard_paths(os.fsencode(path), i, buf, len(buf), None))
        out.append(os.fsdecode(buf.value))
    return out


def gguf_block_index(name):
    """N of a `blk.N.` tensor name, or None (block_index, gguf.rs:534)."""
    v = lib().sz_gguf_block_index(name.encode())
    return None if v < 0 else v


def _info_dict(name, t):
    return {"name": name, "dims": [t.dims[i] for i in range(t.n_dims)], "type": t.type, "shard": t.shard, "offset": t.offset,
            "nbytes_layout": t.nbytes_layout if t.has_layout else None, "nbytes_span": t.nbytes_span, "nbytes": t.nbytes}


class Gguf:
    """A GGUF model's header: key-values and tensor table of every shard (Gguf, gguf.rs:260, 459-531)."""

    def __init__(self, path):
        self._h = None
        h = _vp()
        check(lib().sz_gguf_open(os.fsencode(path), C.byref(h)))
        self._h = h

    def close(self):
        if self._h and _lib is not None:      # at interpreter exit the module may be gone before the object
            _lib.sz_gguf_close(self._h)
        self._h = None

    __del__ = close

    def tensors(self):
        out, buf, t = [], C.create_string_buffer(1024), TensorInfo()
        for i in range(lib().sz_gguf_tensor_count(self._h)):
            check(lib().sz_gguf_tensor_at(self._h, i, buf, 1024, C.byref(t)))
            out.append(_info_dict(buf.value.decode(errors="replace"), t))
        return out

    def tensor(self, name):
        t = TensorInfo()
        if lib().sz_gguf_tensor(self._h, name.encode(), C.byref(t)) != 0:
            return None
        return _info_dict(name, t)

    def tensor_bytes(self):
        return lib().sz_gguf_tensor_bytes(self._h)

    def shards(self):
        out = []
        for i in range(lib().sz_gguf_shard_count(self._h)):
            buf, v, fl, ds, al = C.create_string_buffer(4096), _u32(), _u64(), _u64(), _u64()
            check(lib().sz_gguf_shard(self._h, i, buf, 4096, C.byref(v), C.byref(fl), C.byref(ds), C.byref(al)))
            out.append({"path": os.fsdecode(buf.value), "version": v.value, "file_len": fl.value, "data_start": ds.value, "alignment": al.value})
        return out

    def keys(self):
        out, buf = [], C.create_string_buffer(1024)
        for i in range(lib().sz_gguf_kv_count(self._h)):
            check(lib().sz_gguf_kv_key(self._h, i, buf, 1024))
            out.append(buf.value.decode(errors="replace"))
        return out

    def kv_type(self, key):
        """(value type id, element type id of an array, count) or None."""
        t, e, n = _u32(), _u32(), _u64()
        if lib().sz_gguf_kv_type(self._h, key.encode(), C.byref(t), C.byref(e), C.byref(n)) != 0:
            return None
        return t.value, e.value, n.value

    def u64(self, key):
        v = _u64()
        return v.value if lib().sz_gguf_kv_u64(self._h, key.encode(), C.byref(v)) == 0 else None

    def arch_u64(self, key):
        v = _u64()
        return v.value if lib().sz_gguf_arch_u64(self._h, key.encode(), C.byref(v)) == 0 else None

    def f64(self, key):
        v = C.c_double()
        return v.value if lib().sz_gguf_kv_f64(self._h, key.encode(), C.byref(v)) == 0 else None

    def str(self, key):
        ty = self.kv_type(key)
        if ty is None or ty[0] != 8:
            return None
        buf = C.create_string_buffer(ty[2] + 1)
        check(lib().sz_gguf_kv_str(self._h, key.encode(), buf, len(buf)))
        return buf.raw[:ty[2]]

    def array(self, key):
        """An array's items: ints (flags as 0 / 1), floats or byte strings; None when the key is no array."""
        ty = self.kv_type(key)
        if ty is None or ty[0] != 9:
            return None
        _, et, n = ty
        out = []
        if et == 8:
            buf = C.create_string_buffer(1 << 16)
            for i in range(n):
                check(lib().sz_gguf_kv_array_str(self._h, key.encode(), i, buf, len(buf)))
                out.append(buf.value)
        elif et in (6, 12):
            v = C.c_double()
            for i in range(n):
                check(lib().sz_gguf_kv_array_f64(self._h, key.encode(), i, C.byref(v)))
                out.append(v.value)
        else:
            v = _u64()
            for i in range(n):
                check(lib().sz_gguf_kv_array_u64(self._h, key.encode(), i, C.byref(v)))
                out.append(v.value)
        return out

    def read_tensor(self, name):
        t = self.tensor(name)
        if t is None:
            raise SzError("no tensor " + name)
        out = np.empty(t["nbytes"], np.uint8)
        check(lib().sz_gguf_read_tensor(self._h, name.encode(), out.ctypes.data, out.size))
        return out

    def expert_range(self, name, e):
        """(shard, byte offset in the file, length) of expert e's slice (Model::expert_file_range, forward.rs:477)."""
        s, o, n = _u32(), _u64(), _u64()
        check(lib().sz_gguf_expert_range(self._h, name.encode(), e, C.byref(s), C.byref(o), C.byref(n)))
        return s.value, o.value, n.value

    def layer_layout(self, layer):
        L = LayerLayout()
        check(lib().sz_gguf_layer_layout(self._h, layer, C.byref(L)))
        return L

    def stage_layer(self, layer, dev, cap, stream=0):
        check(lib().sz_gguf_stage_layer(self._h, layer, dev, cap, stream))

    def stage_tensor(self, name, dev, cap, stream=0):
        check(lib().sz_gguf_stage_tensor(self._h, name.encode(), dev, cap, stream))


class SafeTensors:
    """Every tensor of one or more safetensors files, or of a directory's, by name (SafeTensors, safetensors.rs:29)."""

    def __init__(self, paths):
        self._h = None
        h = _vp()
        if isinstance(paths, (str, bytes, os.PathLike)) and os.path.isdir(paths):
            check(lib().sz_st_open_dir(os.fsencode(paths), C.byref(h)))
        else:
            if isinstance(paths, (str, bytes, os.PathLike)):
                paths = [paths]
            arr = (C.c_char_p * len(paths))(*[os.fsencode(p) for p in paths])
            check(lib().sz_st_open(arr, len(paths), C.byref(h)))
        self._h = h

    def close(self):
        if self._h and _lib is not None:
            _lib.sz_st_close(self._h)
        self._h = None

    __del__ = close

    @staticmethod
    def _dict(name, t):
        return {"name": name, "dtype": t.dtype.decode(), "shape": [t.shape[i] for i in range(t.n_dims)], "file": t.file, "start": t.start, "end": t.end}

    def files(self):
        out, buf = [], C.create_string_buffer(4096)
        for i in range(lib().sz_st_file_count(self._h)):
            check(lib().sz_st_file(self._h, i, buf, 4096))
            out.append(os.fsdecode(buf.value))
        return out

    def tensors(self):
        out, buf, t = [], C.create_string_buffer(1024), StInfo()
        for i in range(lib().sz_st_tensor_count(self._h)):
            check(lib().sz_st_tensor_at(self._h, i, buf, 1024, C.byref(t)))
            out.append(self._dict(buf.value.decode(errors="replace"), t))
        return out

    def get(self, name):
        t = StInfo()
        if lib().sz_st_tensor(self._h, name.encode(), C.byref(t)) != 0:
            return None
        return self._dict(name, t)

    def read(self, name, off=0, length=None):
        t = self.get(name)
        if t is None:
            raise SzError("no tensor " + name)
        n = t["end"] - t["start"] - off if length is None else length
        out = np.empty(max(n, 0), np.uint8)
        check(lib().sz_st_read(self._h, name.encode(), off, n, out.ctypes.data))
        return out

    def exl3_shape(self, prefix):
        """(in_features, out_features, ggml type id) of the projection `prefix` (linear_shape, exl3_model.rs:98)."""
        i, o, ty = _u64(), _u64(), _i32()
        check(lib().sz_exl3_shape(self._h, prefix.encode(), C.byref(i), C.byref(o), C.byref(ty)))
        return i.value, o.value, ty.value

    def exl3_contiguous(self, prefix):
        """(file, offset, length) when the projection's tensors are one range of a file in blob order, else None."""
        f, o, n = _u32(), _u64(), _u64()
        if lib().sz_exl3_contiguous(self._h, prefix.encode(), C.byref(f), C.byref(o), C.byref(n)) != 0:
            return None
        return f.value, o.value, n.value

    def exl3_blob(self, prefix):
        i, o, ty = self.exl3_shape(prefix)
        out = np.empty(lib().sz_exl3_blob_len(i, o, ty), np.uint8)
        check(lib().sz_exl3_read_blob(self._h, prefix.encode(), out.ctypes.data, out.size))
        return out

    def layer_layout(self, layer, n_expert=0):
        L = LayerLayout()
        check(lib().sz_exl3_layer_layout(self._h, layer, n_expert, C.byref(L)))
        return L

    def stage_layer(self, layer, dev, cap, n_expert=0, stream=0):
        check(lib().sz_exl3_stage_layer(self._h, layer, n_expert, dev, cap, stream))

    def stage_tensor(self, name, dev, cap, stream=0):
        check(lib().sz_st_stage_tensor(self._h, name.encode(), dev, cap, stream))

    def stage_exl3_blob(self, prefix, dev, cap, stream=0):
        check(lib().sz_exl3_stage_blob(self._h, prefix.encode(), dev, cap, stream))


def layer_spacing(expert_type, hidden, ff):
    """(lead, gap) of sz_layer_spacing: where a layer's first expert should start past a 128-byte boundary and how far apart an
    expert's projections should lie for every EXL3 trellis to start on a 128-byte line (0, 0 for GGUF types)."""
    lead, gap = C.c_uint32(0), C.c_uint32(0)
    lib().sz_layer_spacing(expert_type, hidden, ff, C.byref(lead), C.byref(gap))
    return lead.value, gap.value


def exl3_blob_len(in_features, out_features, type_id):
    return lib().sz_exl3_blob_len(in_features, out_features, type_id)
