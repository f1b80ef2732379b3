"""The C ABI without a GPU: the library loads, exports every symbol include/shadowzero_hip.h declares, its kernel registry
matches the kernel sources (the drift test of crates/shadowzero-cuda/tests/drift.rs), its SHA-256 is SHA-256, and a bad
launch is refused before anything reaches the driver (crates/shadowzero-cuda/tests/gpu.rs:75)."""
import ctypes as C
import hashlib
import os
import re

import pytest

import shadow_engine_amd as sz
from shadow_engine_amd import build

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "shadowzero_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sz_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = sz.lib()
    names = header_symbols()
    assert len(names) > 40
    for n in names:
        assert hasattr(L, n), f"{n} is declared in the header but not exported"
    assert set(names) == set(sz.exported_symbols()), "the Python binding and the header list different entry points"


def test_header_is_plain_c():
    """The boundary is a C ABI: the header must compile as C99 (what a cgo / bindgen / ctypes user feeds it to) and as C++."""
    import subprocess
    h = os.path.join(ROOT, "include", "shadowzero_hip.h")
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-fsyntax-only", "-x", "c", h], check=True)
    subprocess.run(["g++", "-std=c++17", "-Wall", "-Werror", "-fsyntax-only", "-x", "c++", h], check=True)


def test_registry_matches_the_kernel_sources():
    want = [(name, build.FILES[fi][0], kinds) for name, fi, kinds in build.registry_entries()]
    kind_id = {"SZ_P_PTR": 0, "SZ_P_CONSTPTR": 1, "SZ_P_U32": 2, "SZ_P_I32": 3, "SZ_P_U64": 4, "SZ_P_F32": 5}
    want = [(n, f, [kind_id[k] for k in ks]) for n, f, ks in want]
    got = sz.kernels()
    assert got == want
    names = [n for n, _, _ in got]
    assert len(names) == len(set(names))
    for expected in ("matvec_q8_0", "matvec_cols_iq3_s", "matvec_grouped_exl3_3", "exl3_decode_8", "route_plan_res_small",
                     "moe_combine_qwen_rows", "head_q8_0_argmax", "topk_merge", "verify_accept", "exl3_build_q2_proxy_5",
                     "proxy_q2_bmax_m4", "proxy_pick_rows", "topk_slices_blks"):
        assert expected in names


def test_parse_param_vocabulary():
    assert build.parse_param("const float* x") == "SZ_P_CONSTPTR"
    assert build.parse_param("u8* base") == "SZ_P_PTR"
    assert build.parse_param("u32 n") == "SZ_P_U32"
    assert build.parse_param("u64 n") == "SZ_P_U64"
    assert build.parse_param("float a") == "SZ_P_F32"
    with pytest.raises(ValueError):
        build.parse_param("double z")


def test_cache_key_is_sha256_of_source_options_target_and_build_mode():
    """nvrtc.rs:185-194 hashes source + options + target; here also how the object is built: the one hipcc makes ahead of time
    (with the file's own `// hipcc:` options) and the one hiprtc makes on a cache miss never share a name."""
    L = sz.lib()
    opts = L.sz_compile_options()
    assert b"ffp-contract=off" in opts and b"packed-fp32-ops" in opts
    extras = 0
    for i in range(L.sz_program_file_count()):
        name = L.sz_program_file_name(i)
        if not os.path.exists(os.path.join(build.KERNELS, name.decode())):
            continue
        key, rkey = C.create_string_buffer(65), C.create_string_buffer(65)
        assert L.sz_program_cache_key(name, key) == 0 and L.sz_program_cache_key_rtc(name, rkey) == 0
        tmp = os.path.join(ROOT, "tests", ".src_probe.tmp")
        try:
            assert L.sz_program_write_source(name, tmp.encode()) == 0
            src = open(tmp, "rb").read()
        finally:
            if os.path.exists(tmp):
                os.remove(tmp)
        own = b" ".join(l[len(b"// hipcc: "):].strip() for l in src.split(b"\n") if l.startswith(b"// hipcc: "))
        aot = L.sz_program_aot_options(name)
        assert aot == (opts + b" " + own if own else opts)
        extras += bool(own)
        assert key.value.decode() == hashlib.sha256(src + b"\0" + aot + b"\0gfx950\0hipcc").hexdigest()
        assert rkey.value.decode() == hashlib.sha256(src + b"\0" + opts + b"\0gfx950\0hiprtc").hexdigest()
        assert key.value != rkey.value
    assert extras >= 1          # prefill.hip asks for matrix results in vector registers
    key = C.create_string_buffer(65)
    assert L.sz_program_cache_key(b"nope.hip", key) != 0 and "not a registered kernel file" in sz.last_error()


def test_a_bad_launch_is_refused_before_the_driver():
    # no device is needed: the registry check comes first
    with pytest.raises(sz.SzError, match="no entry point"):
        sz.launch("no_such_kernel", (1, 1, 1), (64, 1, 1), 0, 0, [])
    with pytest.raises(sz.SzError, match="takes 4 arguments, 1 given"):
        sz.launch("swiglu", (1, 1, 1), (256, 1, 1), 0, 0, [sz.Arg.ptr(0)])
    with pytest.raises(sz.SzError, match="argument 3"):
        sz.launch("swiglu", (1, 1, 1), (256, 1, 1), 0, 0, [sz.Arg.ptr(0), sz.Arg.ptr(0), sz.Arg.ptr(0), sz.Arg.f32(1.0)])
    with pytest.raises(sz.SzError, match="empty grid"):
        sz.launch("swiglu", (0, 1, 1), (256, 1, 1), 0, 0, [sz.Arg.ptr(0), sz.Arg.ptr(0), sz.Arg.ptr(0), sz.Arg.u32(1)])


def test_host_side_acceptance_and_error_paths():
    assert sz.verify_accept([5, 6, 7], [5, 6, 7]) == 4
    assert sz.verify_accept([5, 6, 7], [5, 9, 7]) == 2
    assert sz.verify_accept([5, 6, 7], [1, 6, 7]) == 1
    assert sz.verify_accept([], []) == 1
    L = sz.lib()
    # nothing that touches the device works before sz_init; the error says so instead of crashing
    p = C.c_uint64()
    if L.sz_malloc(C.byref(p), 16) != 0:
        assert "sz_init" in sz.last_error()
    assert L.sz_session_new(C.byref(sz.SessionConfig(2048, 512, 512, 10, 1, 1000, 8, 0))) is None or True


def test_grid_table_copies_are_identical():
    # the oracle and the kernels each carry the IQ3_S grid as data; they must be the same table
    def nums(path):
        return re.findall(r"0x[0-9a-f]{8}", open(path).read())
    a = nums(os.path.join(ROOT, "oracle", "iq3s_grid.inc"))
    b = nums(os.path.join(ROOT, "shadow_engine_amd", "kernels", "iq_tables.hip.h"))
    assert len(a) == 512 and a == b


def test_the_exl3_heads_lds_bound_is_what_the_kernel_takes():
    """head_exl3_K: four 4-row rings (static) + 4 KiB of A rows for every 512 inputs and two rows (dynamic), against the 160 KiB of
    a compute unit: hidden 4096 takes 8 rows at every rate (exactly 160 KiB at K = 8), hidden 8192 at most 4."""
    L = sz.lib()
    ring = lambda k: 4 * 4 * 64 * (4 if k in (3, 4) else k) * 4
    for k in range(1, 9):
        for hidden in (128, 2048, 2560, 4096, 8192):
            for m in range(1, 9):
                want = ring(k) + 4096 * ((hidden // 128 + 3) // 4) * ((m + 1) // 2)
                assert L.sz_exl3_head_lds_bytes(sz.EXL3(k), hidden, m) == want
    assert L.sz_exl3_head_lds_bytes(sz.EXL3(8), 4096, 8) == 160 * 1024
    assert L.sz_exl3_head_lds_bytes(sz.EXL3(4), 8192, 5) > 160 * 1024 >= L.sz_exl3_head_lds_bytes(sz.EXL3(4), 8192, 4)
    assert L.sz_exl3_head_lds_bytes(sz.Q8_0, 4096, 8) == 0
