"""The tracked counters the benchmark quotes: profiles/counters.json names real kernels and real kernel files, and bench.py
stops quoting a kernel's counters as soon as the file that holds the kernel differs from the one they were measured on."""
import importlib.util
import json
import os

import shadow_engine_amd as sz

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def bench_module():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    m = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(m)
    return m


def test_counters_file_names_kernels_of_the_registry():
    c = json.load(open(os.path.join(ROOT, "profiles", "counters.json")))
    files = {f for _, f, _ in sz.kernels()}
    names = {n for n, _, _ in sz.kernels()}
    assert set(c["kernel_keys"]) == files
    assert all(len(k) == 64 for k in c["kernel_keys"].values())
    assert "config5" in c["workloads"]
    for wl, entry in c["workloads"].items():
        for k, v in entry["kernels"].items():
            assert k in names, (wl, k)
            if "SQ_INSTS_VALU" in v:
                # busy cycles are averaged over the 32 shader engines: a launch of fewer waves than the chip has SIMDs leaves
                # engines idle and reads a low clock, so only launches that fill the chip are held to a plausible one
                assert v["busy_cycles"] > 0 and 0.5 < v["clock_ghz"] < 3.0 or v["SQ_WAVES"] < 1024, (wl, k, v)


class FakeLibrary:
    def __init__(self, keys):
        self.keys = keys

    def kernels(self):
        return sz.kernels()

    def program_keys(self):
        return dict(self.keys)


def test_bench_quotes_counters_only_for_unchanged_kernel_files(tmp_path, monkeypatch):
    b = bench_module()
    keys = sz.program_keys()
    path = tmp_path / "counters.json"
    path.write_text(json.dumps({"kernel_keys": keys, "workloads": {}}))
    monkeypatch.setattr(b, "COUNTERS", str(path))
    c, stale = b.load_counters(FakeLibrary(keys))
    assert c is not None and stale == {}
    edited = dict(keys)
    edited["exl3.hip"] = "0" * 64
    c, stale = b.load_counters(FakeLibrary(edited))
    file_of = {n: f for n, f, _ in sz.kernels()}
    assert c is not None and set(stale) == {n for n, f in file_of.items() if f == "exl3.hip"}
    assert "verify_gate_up_exl3_3" in stale and "head_q8_0_argmax_mfma" not in stale
    monkeypatch.setattr(b, "COUNTERS", str(tmp_path / "missing.json"))
    c, stale = b.load_counters(FakeLibrary(keys))
    assert c is None and set(stale) == set(file_of)


def test_roofline_names_the_nearer_roof(monkeypatch):
    b = bench_module()

    class W:
        counters_key = "config5"
    per_kernel = {"verify_gate_up_exl3_3": {"launches_per_step": 16, "avg_us": 20.0, "bytes_per_launch": 32_000_000, "GBps": 1600.0},
                  "verify_combine_exl3": {"launches_per_step": 48, "avg_us": 4.0}}
    counters = {"workloads": {"config5": {"kernels": {"verify_gate_up_exl3_3": {"SQ_INSTS_VALU": 8_000_000, "clock_ghz": 2.0, "valu_busy_frac": 0.73,
                                                                               "traffic_bytes": 40_000_000}}}}}
    r = b.roofline_of(W(), per_kernel, counters, {})
    assert r["kernel"] == "verify_gate_up_exl3_3" and r["traffic"] == 40_000_000
    assert r["frac"] == 0.2 and r["vector_alu"]["peak"] == 512.0 and r["vector_alu"]["achieved"] == 400.0
    assert r["bound"] == "valu"
    stale = b.roofline_of(W(), per_kernel, counters, {"verify_gate_up_exl3_3": "measured on another exl3.hip"})
    assert stale["traffic"] is None and "vector_alu" not in stale and stale["bound"] == "hbm" and "another" in stale["counters"]
