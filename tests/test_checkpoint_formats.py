"""The checkpoint formats either side of the hot path: the library's GGUF and safetensors readers, the EXL3 projection blob and
the staging of a layer into device memory, against the oracle (oracle/checkpoint_formats.py) and against what pins the oracle:
the reference's own reader tests (crates/shadowzero-model/src/gguf.rs:551-624, safetensors.rs:346-360) restated on files written
here by hand, Python's json module, numpy's float16 rounding, and the golden EXL3 tensor of tests/golden."""
import json
import os
import struct
import sys

import numpy as np
import pytest

import oracle_lib as O
import shadow_engine_amd as sz
from shadow_engine_amd import synth
from shadow_engine_amd.synth import exl3_checkpoint, fused_experts_gguf, gguf_file, st_file

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import checkpoint_formats as F   # noqa: E402

REFERENCE = "/root/reference"


def tiny(path):
    """The two-tensor file of the reference's reader test (gguf.rs:551-583)."""
    kv = [("general.architecture", 8, "toy"), ("toy.block_count", 4, 2), ("tokenizer.ggml.tokens", 9, (8, ["a", "bc"]))]
    gguf_file(path, kv, [("blk.0.w", [32, 2], 0, b"\x07" * 256), ("blk.1.q", [256], 21, b"\x07" * 110)])


def same_tensor(a, b):
    return all(a[k] == b[k] for k in ("name", "dims", "type", "shard", "offset", "nbytes_layout", "nbytes_span", "nbytes"))


# ---- GGUF ---------------------------------------------------------------------------------------------------------------
def test_reads_the_hand_written_file_of_the_reference_test(tmp_path):
    p = str(tmp_path / "toy.gguf")
    tiny(p)
    o = F.gguf_open(p)
    assert o["kv"][b"general.architecture"] == (8, b"toy") and F.as_u64(o["kv"][b"toy.block_count"]) == 2
    assert len(o["kv"][b"tokenizer.ggml.tokens"][2]) == 2
    w, q = F.gguf_tensor(o, "blk.0.w"), F.gguf_tensor(o, "blk.1.q")
    assert (w["dims"], F.type_name(w["type"]), w["nbytes"]) == ([32, 2], "F32", 256)
    assert (F.type_name(q["type"]), q["nbytes_layout"], q["nbytes_span"]) == ("IQ3_S", 110, 110)
    assert sum(t["nbytes"] for t in o["tensors"]) == 366 and F.block_index("blk.1.q") == 1

    g = sz.Gguf(p)
    assert g.str("general.architecture") == b"toy" and g.arch_u64("block_count") == 2
    assert g.array("tokenizer.ggml.tokens") == [b"a", b"bc"]
    w, q = g.tensor("blk.0.w"), g.tensor("blk.1.q")
    assert (w["dims"], sz.type_info(w["type"])[0], w["nbytes"]) == ([32, 2], "F32", 256)
    assert (sz.type_info(q["type"])[0], q["nbytes_layout"], q["nbytes_span"]) == ("IQ3_S", 110, 110)
    assert g.tensor_bytes() == 366
    assert g.read_tensor("blk.1.q").tolist() == [7] * 110
    assert sz.gguf_block_index("blk.1.q") == 1 and sz.gguf_block_index("output.weight") is None and sz.gguf_block_index("blk.x.q") is None
    assert g.tensor("nope") is None and g.u64("nope") is None and g.u64("general.architecture") is None
    assert all(same_tensor(a, b) for a, b in zip(g.tensors(), o["tensors"]))
    assert g.shards() == [dict(o["shards"][0])]


def test_rejects_a_truncated_file(tmp_path):
    p = str(tmp_path / "cut.gguf")
    tiny(p)
    full = open(p, "rb").read()
    open(p, "wb").write(full[:-200])
    with pytest.raises(F.FormatError):
        F.gguf_open(p)
    with pytest.raises(sz.SzError, match="outside the file|needs 110 bytes"):
        sz.Gguf(p)


def test_finds_the_other_shards_by_name():
    for f in (F.shard_paths, sz.gguf_shard_paths):
        assert f("m/x-IQ3_S-00002-of-00002.gguf") == ["m/x-IQ3_S-00001-of-00002.gguf", "m/x-IQ3_S-00002-of-00002.gguf"]
        assert f("m/single.gguf") == ["m/single.gguf"]
        assert f("a-b-7-of-003.gguf") == ["a-b-001-of-003.gguf", "a-b-002-of-003.gguf", "a-b-003-of-003.gguf"]
        assert f("x-1-of-0.gguf") == ["x-1-of-0.gguf"] and f("x-of-2.gguf") == ["x-of-2.gguf"] and f("x-1-of-2.bin") == ["x-1-of-2.bin"]


def test_every_value_type_alignment_and_unknown_tensor_types(tmp_path):
    p = str(tmp_path / "v.gguf")
    kv = [("u8", 0, 200), ("i8", 1, -3), ("u16", 2, 65535), ("i16", 3, -2), ("u32", 4, 4000000000), ("i32", 5, 17), ("f32", 6, 0.1),
          ("flag", 7, 1), ("s", 8, "h\xe9llo"), ("u64", 10, 1 << 63), ("i64", 11, -1), ("f64", 12, 1e300), ("general.alignment", 4, 64),
          ("arr.f", 9, (6, [1.5, -2.25])), ("arr.i", 9, (5, [3, 4, 5])), ("arr.b", 9, (7, [1, 0, 1])), ("arr.nested", 9, (9, [(4, [1, 2]), (4, [])])),
          ("arr.empty", 9, (8, []))]
    # type 77 is unknown: its size is its span; an IQ3_S row of 100 is no whole block: no layout either
    gguf_file(p, kv, [("a", [3], 77, b"\x01" * 10), ("b", [100], 21, b"\x02" * 50), ("c", [64, 3], 8, b"\x03" * 204)], alignment=64, pad_tail=5)
    o, g = F.gguf_open(p), sz.Gguf(p)
    assert g.shards()[0]["alignment"] == 64 and g.shards()[0]["data_start"] % 64 == 0 and g.shards() == o["shards"]
    assert [g.u64(k) for k in ("u8", "i8", "u16", "i16", "u32", "i32", "u64", "i64", "flag", "f32")] == [200, None, 65535, None, 4000000000, 17, 1 << 63, None, None, None]
    assert [F.as_u64(o["kv"][k.encode()]) for k in ("u8", "i8", "u16", "i16", "u32", "i32", "u64", "i64", "flag", "f32")] == [200, None, 65535, None, 4000000000, 17, 1 << 63, None, None, None]
    assert g.f64("f32") == float(np.float32(0.1)) and g.f64("f64") == 1e300 and g.f64("u16") == 65535.0 and g.f64("i8") is None and g.f64("s") is None
    assert g.str("s") == "h\xe9llo".encode() and g.str("u8") is None
    assert g.array("arr.f") == [1.5, -2.25] and g.array("arr.i") == [3, 4, 5] and g.array("arr.b") == [1, 0, 1] and g.array("arr.empty") == []
    assert g.kv_type("arr.nested") == (9, 9, 2) and g.kv_type("s") == (8, 0, 6) and g.kv_type("nope") is None
    assert g.keys() == sorted(k for k, _, _ in kv)                 # byte order, as a BTreeMap iterates
    a, b, c = g.tensor("a"), g.tensor("b"), g.tensor("c")
    assert (a["nbytes_layout"], a["nbytes_span"], a["nbytes"]) == (None, 64, 64) and sz.type_info(77) == ("type77", 0, 0)
    assert (b["nbytes_layout"], b["nbytes"]) == (None, 64)
    assert (c["nbytes_layout"], c["nbytes_span"]) == (204, 209)     # the last tensor's span runs to the end of the file
    assert all(same_tensor(x, y) for x, y in zip(g.tensors(), o["tensors"]))


@pytest.mark.parametrize("what", ["magic", "version", "alignment", "depth", "value type", "dims", "string", "short"])
def test_refuses_what_the_reference_refuses(tmp_path, what):
    p = str(tmp_path / "bad.gguf")
    kv, tensors, kw = [("k", 4, 1)], [("t", [32], 0, b"\0" * 128)], {}
    if what == "magic":
        kw["magic"] = b"GGML"
    elif what == "version":
        kw["version"] = 1
    elif what == "alignment":
        kv = [("general.alignment", 4, 48)]
    elif what == "depth":
        kv = [("deep", 9, (9, [(9, [(9, [(9, [(4, [1])])])])]))]
    elif what == "dims":
        tensors = [("t", [1] * 9, 0, b"\0" * 4)]
    gguf_file(p, kv, tensors, **kw)
    if what == "value type":
        b = bytearray(open(p, "rb").read())
        i = b.index(b"k") + 1
        b[i:i + 4] = struct.pack("<I", 13)
        open(p, "wb").write(bytes(b))
    elif what == "string":
        b = bytearray(open(p, "rb").read())
        b[24:32] = struct.pack("<Q", 1 << 40)      # the first key's length
        open(p, "wb").write(bytes(b))
    elif what == "short":
        open(p, "wb").write(open(p, "rb").read()[:30])
    with pytest.raises(F.FormatError):
        F.gguf_open(p)
    with pytest.raises(sz.SzError):
        sz.Gguf(p)


def test_a_split_model_is_one_tensor_table(tmp_path):
    p1, p2 = str(tmp_path / "m-00001-of-00002.gguf"), str(tmp_path / "m-00002-of-00002.gguf")
    gguf_file(p1, [("general.architecture", 8, "toy"), ("split.count", 2, 2), ("split.tensors.count", 5, 3), ("who", 4, 1)],
              [("blk.0.a", [32], 0, b"\x01" * 128)])
    gguf_file(p2, [("who", 4, 2), ("only.second", 4, 9), ("general.alignment", 4, 128)], [("blk.1.a", [32], 0, b"\x02" * 128), ("blk.1.b", [32, 2], 8, b"\x03" * 68)],
              alignment=128)
    o, g = F.gguf_open(p2), sz.Gguf(p2)                             # opened from the second shard
    assert [s["path"] for s in g.shards()] == [p1, p2] and g.shards() == o["shards"]
    assert g.u64("who") == 1 and g.u64("only.second") == 9          # shard 0's key-values are the model's
    assert [t["shard"] for t in g.tensors()] == [0, 1, 1] and all(same_tensor(x, y) for x, y in zip(g.tensors(), o["tensors"]))
    assert g.read_tensor("blk.1.b").tolist() == [3] * 68
    gguf_file(p1, [("split.count", 2, 3)], [("blk.0.a", [32], 0, b"\x01" * 128)])
    with pytest.raises(sz.SzError, match="split.count 3, found 2 shards"):
        sz.Gguf(p1)
    with pytest.raises(F.FormatError):
        F.gguf_open(p1)
    os.remove(p2)
    with pytest.raises(sz.SzError):
        sz.Gguf(p1)


@pytest.mark.parametrize("name", ["models/bge-small-en-v1.5-q8_0.gguf", "models/embed-minilm/all-MiniLM-L6-v2-Q8_0.gguf"])
def test_the_reference_checkouts_own_gguf_models(name):
    """Real files a third party wrote: the spans must tile the data section, a layout never exceeds its span by the file's own
    rule, and the library and the oracle read the same table."""
    p = os.path.join(REFERENCE, name)
    if not os.path.exists(p):
        pytest.skip("the reference checkout is not here")
    o, g = F.gguf_open(p), sz.Gguf(p)
    ts, sh = g.tensors(), g.shards()[0]
    assert len(ts) == len(o["tensors"]) > 50 and all(same_tensor(x, y) for x, y in zip(ts, o["tensors"])) and g.shards() == o["shards"]
    by_off = sorted(ts, key=lambda t: t["offset"])
    assert by_off[0]["offset"] == sh["data_start"] and by_off[-1]["offset"] + by_off[-1]["nbytes_span"] == sh["file_len"]
    for a, b in zip(by_off, by_off[1:]):
        assert a["offset"] + a["nbytes_span"] == b["offset"]
    for t in ts:
        assert t["nbytes_layout"] is not None and 0 <= t["nbytes_span"] - t["nbytes_layout"] < sh["alignment"] and t["offset"] % sh["alignment"] == 0
    arch = g.str("general.architecture").decode()
    hidden, blocks = g.u64(arch + ".embedding_length"), g.arch_u64("block_count")
    emb = g.tensor("token_embd.weight")
    assert emb["dims"][0] == hidden and emb["type"] == sz.Q8_0 and max(sz.gguf_block_index(t["name"]) or 0 for t in ts) == blocks - 1
    assert len(g.array("tokenizer.ggml.tokens")) == emb["dims"][1]
    # its bytes are Q8_0 blocks of sane scale: the reader points at the right place
    rows = O.dequantize(sz.Q8_0, g.read_tensor("token_embd.weight")[:hidden // 32 * 34 * 8]).reshape(8, hidden)
    assert np.all(np.isfinite(rows)) and 1e-3 < float(np.abs(rows).mean()) < 1.0


def test_expert_ranges_and_the_layer_layout_of_a_gguf(tmp_path):
    rng = np.random.default_rng(5)
    p = str(tmp_path / "moe.gguf")
    hidden, ff, ne = 256, 512, 6
    blobs, sh, rw, gw = fused_experts_gguf(p, rng, sz.IQ3_S, hidden, ff, ne)
    o, g = F.gguf_open(p), sz.Gguf(p)
    data = np.fromfile(p, np.uint8)
    gu = synth.expert_bytes(sz.IQ3_S, hidden, ff)[0]
    for name, lo, hi in (("blk.0.ffn_gate_exps.weight", 0, gu), ("blk.0.ffn_up_exps.weight", gu, 2 * gu), ("blk.0.ffn_down_exps.weight", 2 * gu, 3 * gu)):
        for e in (0, 3, ne - 1):
            shard, off, n = g.expert_range(name, e)
            assert (shard, off, n) == F.expert_file_range(o, name, e)
            assert np.array_equal(data[off:off + n], blobs[e][lo:hi])             # the slice is that expert's projection
        with pytest.raises(sz.SzError):
            g.expert_range(name, ne)
    with pytest.raises(sz.SzError):
        g.expert_range("blk.0.ffn_gate_shexp.weight", 0)                           # not a fused tensor
    L = g.layer_layout(0)
    img, mask, stride, so, ro, go = F.layer_image([(b[:gu], b[gu:2 * gu], b[2 * gu:]) for b in blobs], [sh[:gu], sh[gu:2 * gu], sh[2 * gu:]],
                                                  rw.view(np.uint8).reshape(-1), gw.view(np.uint8).reshape(-1))
    assert (L.type, L.shared_type, L.router_type, L.gate_type, L.n_expert, L.hidden, L.ff) == (sz.IQ3_S, sz.IQ3_S, sz.F32, sz.F32, ne, hidden, ff)
    assert (L.gate_up_bytes, L.down_bytes, L.shared_gate_up_bytes) == (gu, gu, gu)
    assert (L.gap, L.experts_offset) == (0, 0)                     # a GGUF layer: contiguous, as the reference keeps it
    assert (L.stride, L.shared_offset, L.router_offset, L.gate_offset, L.bytes) == (stride, so, ro, go, img.size)
    with pytest.raises(sz.SzError, match="no tensor blk.1.ffn_gate_exps.weight"):
        g.layer_layout(1)
    p2 = str(tmp_path / "mixed.gguf")
    fused_experts_gguf(p2, rng, sz.Q8_0, 256, 256, 2, shared=False, down_ty=sz.F32 + 9)   # a Q8_1 down beside Q8_0 gate and up
    with pytest.raises(sz.SzError):
        sz.Gguf(p2)                                                                # and its bytes do not fit that type either


# ---- safetensors ------------------------------------------------------------------------------------------------------
HEADER_1 = r'''{"__metadata__":{"format":"pt"},"a.b":{"dtype":"I16","shape":[2,3],"data_offsets":[0,12]},"s\"x":{"dtype":"I32","shape":[],"data_offsets":[12,16]}}'''


def test_header_with_metadata_scalars_and_escapes(tmp_path):
    want = [("a.b", "I16", [2, 3], 0, 12), ('s"x', "I32", [], 12, 16)]          # safetensors.rs:349-352
    assert F.st_parse_header(HEADER_1) == want
    j = json.loads(HEADER_1)
    assert [(k, v["dtype"], v["shape"], *v["data_offsets"]) for k, v in j.items() if k != "__metadata__"] == want
    p = str(tmp_path / "h.safetensors")
    open(p, "wb").write(struct.pack("<Q", len(HEADER_1)) + HEADER_1.encode() + bytes(range(16)))
    st = sz.SafeTensors(p)
    d0 = 8 + len(HEADER_1)
    assert st.tensors() == [{"name": "a.b", "dtype": "I16", "shape": [2, 3], "file": 0, "start": d0, "end": d0 + 12},
                            {"name": 's"x', "dtype": "I32", "shape": [], "file": 0, "start": d0 + 12, "end": d0 + 16}]
    assert st.read('s"x').tolist() == [12, 13, 14, 15] and st.read("a.b", 2, 3).tolist() == [2, 3, 4] and st.get("zz") is None
    with pytest.raises(sz.SzError, match="outside a tensor"):
        st.read("a.b", 8, 5)


@pytest.mark.parametrize("text", ['{"a":{"dtype":"F16"}}', '{"a":', "", '{"a":{"dtype":"F16","shape":[1],"data_offsets":[4,2]}}',
                                  '{"a":{"dtype":"F16","shape":[1],"data_offsets":[0,2,4]}}', '{"a":{"dtype":"F16","shape":[1],"data_offsets":[0,2]}',
                                  '{"a":{"dtype":"F16","shape":[-1],"data_offsets":[0,2]}}', '{"a\\q":{"dtype":"F16","shape":[1],"data_offsets":[0,2]}}',
                                  '{"a":{"dtype":"F16","shape":[99999999999999999999],"data_offsets":[0,2]}}'])
def test_a_broken_header_is_an_error_not_a_crash(tmp_path, text):
    with pytest.raises(F.FormatError):                                            # safetensors.rs:355-360 and neighbours
        F.st_parse_header(text)
    p = str(tmp_path / "b.safetensors")
    open(p, "wb").write(struct.pack("<Q", len(text)) + text.encode() + b"\0" * 8)
    with pytest.raises(sz.SzError):
        sz.SafeTensors(p)


def test_unusual_but_valid_headers_read_like_json(tmp_path):
    text = ('{ "t\\u00e9\\n\\/" : { "extra" : [1, {"x": null}, "s,]}"], "shape" : [ ] , "dtype":"BF16",\n "data_offsets":[0 , 4], "more": true } ,\r\n'
            ' "__metadata__" : {"a":{"b":["}", 2.5e3, false]}}, "z": {"dtype":"F32","shape":[1],"data_offsets":[4,8]} }')
    j = json.loads(text)
    want = [(k, v["dtype"], v["shape"], *v["data_offsets"]) for k, v in j.items() if k != "__metadata__"]
    assert F.st_parse_header(text) == want
    p = str(tmp_path / "u.safetensors")
    open(p, "wb").write(struct.pack("<Q", len(text)) + text.encode() + b"\1" * 8)
    st = sz.SafeTensors(p)
    assert sorted((t["name"], t["dtype"], t["shape"], t["end"] - t["start"]) for t in st.tensors()) == sorted((n, d, s, e - b) for n, d, s, b, e in want)


def test_file_level_checks(tmp_path):
    a, b = str(tmp_path / "model-00001.safetensors"), str(tmp_path / "model-00002.safetensors")
    st_file(a, [("x", "F16", [2], b"\1\2\3\4")], metadata={"format": "pt"})
    st_file(b, [("y", "I32", [1], b"\5\6\7\x08")])
    open(str(tmp_path / "notes.txt"), "w").write("not a tensor file")
    st = sz.SafeTensors(str(tmp_path))                                          # open_dir: name order, only *.safetensors
    assert st.files() == [a, b] and [t["name"] for t in st.tensors()] == ["x", "y"] and st.get("y")["file"] == 1
    o = F.st_open([a, b])
    for t in st.tensors():
        assert {k: t[k] for k in ("dtype", "shape", "file", "start", "end")} == o["tensors"][t["name"]]
    with pytest.raises(sz.SzError, match="appears twice"):
        sz.SafeTensors([a, a])
    with pytest.raises(F.FormatError):
        F.st_open([a, a])
    cut = str(tmp_path / "cut.safetensors")
    open(cut, "wb").write(open(a, "rb").read()[:-1])
    with pytest.raises(sz.SzError, match="but the file has"):
        sz.SafeTensors(cut)
    with pytest.raises(F.FormatError):
        F.st_open([cut])
    huge = str(tmp_path / "huge.safetensors")
    open(huge, "wb").write(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(sz.SzError, match="not a safetensors header"):
        sz.SafeTensors(huge)
    with pytest.raises(sz.SzError):
        sz.SafeTensors(str(tmp_path / "absent.safetensors"))


def test_the_header_of_the_reference_fixture():
    """eval/fixtures/exl3_sample.safetensors: its header is whole (the data after it lost bytes to a line-ending conversion in
    this checkout, which the readers refuse as they must)."""
    p = os.path.join(REFERENCE, "eval/fixtures/exl3_sample.safetensors")
    if not os.path.exists(p):
        pytest.skip("the reference checkout is not here")
    raw = open(p, "rb").read()
    n = struct.unpack("<Q", raw[:8])[0]
    j = json.loads(raw[8:8 + n])
    got = F.st_parse_header(raw[8:8 + n])
    assert got == [(k, v["dtype"], v["shape"], *v["data_offsets"]) for k, v in j.items() if k != "__metadata__"] and len(got) == 8
    assert 8 + n + max(t[4] for t in got) == len(raw) + 12
    with pytest.raises(sz.SzError, match="ends at 1242600 but the file has 1242588 bytes"):
        sz.SafeTensors(p)
    with pytest.raises(F.FormatError):
        F.st_open([p])


# ---- the EXL3 projection --------------------------------------------------------------------------------------------------
def golden_parts():
    blob = np.fromfile(os.path.join(ROOT, "tests", "golden", "exl3_k2_gate_proj.blob"), np.uint8)
    inf, outf = 2560, 640
    return blob, blob[:2 * inf], blob[2 * inf:2 * inf + 2 * outf], blob[2 * inf + 2 * outf + 4:], inf, outf


MUL1 = struct.pack("<I", 0x83DCD12D)


def test_the_golden_tensor_as_a_checkpoint_gives_the_golden_blob(tmp_path):
    blob, suh, svh, tr, inf, outf = golden_parts()
    pre = "model.language_model.layers.0.mlp.experts.0.gate_proj"
    # the order of the reference's fixture (mul1 first): not one range in blob order, so the blob is put together, marker 1
    p = str(tmp_path / "a.safetensors")
    st_file(p, [(pre + ".mul1", "I32", [], MUL1), (pre + ".suh", "F16", [inf], suh), (pre + ".svh", "F16", [outf], svh),
                (pre + ".trellis", "I16", [inf // 16, outf // 16, 32], tr)])
    st, o = sz.SafeTensors(p), F.st_open([p])
    assert st.exl3_shape(pre) == (inf, outf, sz.EXL3(2)) and F.exl3_shape(o, pre) == (inf, outf, 2, False, 2, sz.EXL3(2))
    assert st.exl3_contiguous(pre) is None and F.exl3_contiguous(o, pre) is None
    assert sz.exl3_blob_len(inf, outf, sz.EXL3(2)) == blob.size == F.blob_len(inf, outf, 2, False)
    assert np.array_equal(st.exl3_blob(pre), blob) and np.array_equal(F.exl3_blob(o, pre), blob)
    # blob order in the file: one range, read as stored (the repo's own marker, not 1)
    p2 = str(tmp_path / "b.safetensors")
    st_file(p2, [("first", "F32", [1], b"\0\0\0\0"), (pre + ".suh", "F16", [inf], suh), (pre + ".svh", "F16", [outf], svh), (pre + ".mul1", "I32", [], MUL1),
                 (pre + ".trellis", "I16", [inf // 16, outf // 16, 32], tr)])
    st2, o2 = sz.SafeTensors(p2), F.st_open([p2])
    c = st2.exl3_contiguous(pre)
    assert c == F.exl3_contiguous(o2, pre) and c[0] == 0 and c[2] == blob.size and c[1] == st2.get(pre + ".suh")["start"]
    want = blob.copy()
    want[2 * inf + 2 * outf:2 * inf + 2 * outf + 4] = np.frombuffer(MUL1, np.uint8)
    assert np.array_equal(st2.exl3_blob(pre), want) and np.array_equal(F.exl3_blob(o2, pre), want)
    # the blob decodes to the tensor the reference recorded (sum of squares 287.702278, tests/exl3_vs_gguf.rs:133)
    w = O.exl3_reconstruct(inf, outf, 2, st.exl3_blob(pre))
    assert abs(float(np.sum(w.astype(np.float64) ** 2)) - 287.702278) < 1e-3 * 287.7


def test_bit_rates_codebooks_and_scale_types(tmp_path):
    rng = np.random.default_rng(11)
    inf, outf = 128, 256
    cases = {16: sz.EXL3(1), 48: sz.EXL3(3), 128: sz.EXL3(8), 24: sz.EXL3_HALF(1), 40: sz.EXL3_HALF(2), 56: sz.EXL3_HALF(3)}
    assert [F.bits_from_last_dim(n) for n in (16, 48, 128, 24, 40, 56, 72, 144, 8, 20)] == [(1, False), (3, False), (8, False), (1, True), (2, True), (3, True), None, None, None, None]
    tensors = []
    hard = np.array([0.0, -0.0, 1.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001, 2.0 ** -26, 6.1e-5, 6.0975e-5, 1.0 + 2.0 ** -11,
                     1.0 + 2.0 ** -11 + 2.0 ** -20, 1.0 + 3 * 2.0 ** -11, -3.14159, 0.33333334, 2047.5, 2049.0, np.inf, -np.inf], np.float32)
    for last in cases:
        pre = "p%d" % last
        suh32 = np.resize(np.concatenate([hard, rng.normal(size=64).astype(np.float32)]), inf).astype(np.float32)
        svh_bf = (rng.normal(size=outf).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
        tr = rng.integers(0, 65536, (inf // 16) * (outf // 16) * last, dtype=np.uint16)
        tensors += [(pre + ".trellis", "I16", [inf // 16, outf // 16, last], tr.tobytes()), (pre + ".svh", "BF16", [outf], svh_bf.tobytes()),
                    (pre + ".mul1", "I32", [], MUL1), (pre + ".suh", "F32", [inf], suh32.tobytes())]
    tensors += [("bad72.trellis", "I16", [8, 16, 72], b"\0" * (8 * 16 * 72 * 2)), ("bad72.mul1", "I32", [], MUL1),
                ("mcg.trellis", "I16", [8, 16, 32], b"\0" * (8 * 16 * 32 * 2)), ("mcg.mcg", "I32", [], MUL1),
                ("plain.trellis", "I16", [8, 16, 32], b"\0" * (8 * 16 * 32 * 2)),
                ("halfmcg.trellis", "I16", [8, 16, 40], b"\0" * (8 * 16 * 40 * 2)), ("halfmcg.mcg", "I32", [], MUL1),
                ("flat.trellis", "I16", [128, 32], b"\0" * (128 * 32 * 2)), ("short.trellis", "I16", [8, 16, 32], b"\0" * (8 * 16 * 32 * 2)),
                ("short.mul1", "I32", [], MUL1), ("short.suh", "F16", [100], b"\0" * 200), ("short.svh", "F16", [256], b"\0" * 512)]
    p = str(tmp_path / "r.safetensors")
    st_file(p, tensors)
    st, o = sz.SafeTensors(p), F.st_open([p])
    for last, ty in cases.items():
        pre = "p%d" % last
        assert st.exl3_shape(pre) == (inf, outf, ty) and F.exl3_shape(o, pre)[5] == ty
        got, want = st.exl3_blob(pre), F.exl3_blob(o, pre)
        assert got.size == sz.exl3_blob_len(inf, outf, ty) and np.array_equal(got, want)        # F32 and BF16 scales rounded as numpy rounds to f16
    assert st.exl3_shape("mcg")[2] == 1012 and st.exl3_shape("plain")[2] == 1002                # codebooks 1 and 0 (exl3_model.rs:105)
    for bad in ("bad72", "halfmcg", "flat", "nothing"):
        with pytest.raises(sz.SzError):
            st.exl3_shape(bad)
        with pytest.raises((F.FormatError, KeyError)):
            F.exl3_shape(o, bad)
    with pytest.raises(sz.SzError, match="suh/svh lengths"):
        st.exl3_blob("short")
    with pytest.raises(sz.SzError, match="no tensor plain.suh"):
        st.exl3_blob("plain")


def test_the_layer_layout_of_an_exl3_checkpoint(tmp_path):
    rng = np.random.default_rng(3)
    d = str(tmp_path / "ckpt")
    hidden, ff, ne = 256, 128, 5
    experts, shared, rw, gw = exl3_checkpoint(d, rng, sz.EXL3_HALF(2), hidden, ff, ne, sz.EXL3(4))
    st = sz.SafeTensors(d)
    o = F.st_open(st.files())
    L = st.layer_layout(3)
    lead, gap = F.exl3_spacing(hidden, ff, experts[0][0].size)
    assert (lead, gap) == (124, 124) == sz.layer_spacing(sz.EXL3_HALF(2), hidden, ff) and sz.layer_spacing(sz.IQ3_S, hidden, ff) == (0, 0)
    img, mask, stride, so, ro, go = F.layer_image(experts, shared, rw.view(np.uint8).reshape(-1), gw.view(np.uint8).reshape(-1), lead, gap)
    assert (L.gap, L.experts_offset) == (gap, lead)
    # every projection's trellis, 2 (in + out) + 4 bytes into its blob, starts on a 128-byte line of a 256-byte aligned buffer
    for base, gu in ((L.experts_offset + 2 * L.stride, L.gate_up_bytes), (L.shared_offset, L.shared_gate_up_bytes)):
        assert all((base + i * (gu + L.gap) + 2 * (hidden + ff) + 4) % 128 == 0 for i in range(3))
    assert (L.type, L.shared_type, L.router_type, L.gate_type, L.n_expert, L.hidden, L.ff) == (sz.EXL3_HALF(2), sz.EXL3(4), sz.BF16, sz.BF16, ne, hidden, ff)
    assert (L.gate_up_bytes, L.down_bytes) == (experts[0][0].size, experts[0][2].size) and L.shared_gate_up_bytes == shared[0].size
    assert (L.stride, L.shared_offset, L.router_offset, L.gate_offset, L.bytes) == (stride, so, ro, go, img.size)
    assert st.layer_layout(3, ne).n_expert == ne
    with pytest.raises(sz.SzError, match="not \\[n_expert, hidden\\]"):
        st.layer_layout(3, ne - 1)                       # the router is of another expert count
    with pytest.raises(sz.SzError):
        st.layer_layout(3, ne + 1)                       # the checkpoint has no such expert
    with pytest.raises(sz.SzError):
        st.layer_layout(2)
    for e in range(ne):                                  # each projection, both ways of reading it, is the blob that was written
        for i, name in enumerate(("gate_proj", "up_proj", "down_proj")):
            pre = "model.language_model.layers.3.mlp.experts.%d.%s" % (e, name)
            assert (st.exl3_contiguous(pre) is not None) == ((e + i) % 3 != 0) == (F.exl3_contiguous(o, pre) is not None)
            assert np.array_equal(st.exl3_blob(pre), experts[e][i]) and np.array_equal(F.exl3_blob(o, pre), experts[e][i])


# ---- staging into device memory ---------------------------------------------------------------------------------------------
@pytest.fixture(scope="module")
def gpu():
    import torch
    assert torch.cuda.is_available(), "no GPU visible"
    sz.init(0)
    return torch


def staged(torch, src, layer, **kw):
    L = src.layer_layout(layer, **kw) if kw else src.layer_layout(layer)
    buf = torch.full((L.bytes,), 0xA5, dtype=torch.uint8, device="cuda")
    assert buf.data_ptr() % 256 == 0
    with pytest.raises(sz.SzError, match="bytes into"):
        src.stage_layer(layer, buf.data_ptr(), L.bytes - 1, **kw)
    src.stage_layer(layer, buf.data_ptr(), L.bytes, **kw)
    return L, buf


def run_staged_layer(torch, L, buf, k, m, rng):
    """The MoE block on a staged layer: session, experts, router and gate all from the layout."""
    s = sz.Session(L.hidden, L.ff, L.n_expert, k, 1, 0, 8)
    base = buf.data_ptr()
    s.set_layer(0, L.type, base + L.experts_offset, L.stride, L.shared_type if L.shared_type >= 0 else 0,
                base + L.shared_offset if L.shared_type >= 0 else 0, gap=L.gap)
    s.set_router(0, L.router_type, base + L.router_offset, L.gate_type, base + L.gate_offset)
    u = rng.normal(size=(m, L.hidden)).astype(np.float32)
    du = torch.from_numpy(u).cuda()
    dy = torch.zeros((m, L.hidden), dtype=torch.float32, device="cuda")
    s.moe_block_verify(0, m, du.data_ptr(), dy.data_ptr())
    torch.cuda.synchronize()
    rl_ptr, sgl_ptr = s.router_outputs()
    rl, sgl = np.empty((m, L.n_expert), np.float32), np.empty(m, np.float32)
    sz.download(rl, rl_ptr)
    sz.download(sgl, sgl_ptr)
    idx, w = s.last_route(m)
    return u, rl, sgl, dy.cpu().numpy(), idx, w


@pytest.mark.gpu
@pytest.mark.parametrize("ty,rty", [(sz.IQ3_S, sz.F32), (sz.Q8_0, sz.BF16)])
def test_a_layer_staged_from_a_gguf_is_the_files_bytes_and_runs(gpu, tmp_path, ty, rty):
    from test_gpu_path import oracle_layer, rel_l2, gguf_bound
    rng = np.random.default_rng(ty)
    hidden, ff, ne, k, m = 512, 256, 12, 4, 3
    p = str(tmp_path / "moe.gguf")
    blobs, sh, rw, gw = fused_experts_gguf(p, rng, ty, hidden, ff, ne, router_ty=rty)
    g = sz.Gguf(p)
    L, buf = staged(gpu, g, 0)
    gu = L.gate_up_bytes
    img, mask, *_ = F.layer_image([(b[:gu], b[gu:2 * gu], b[2 * gu:]) for b in blobs], [sh[:gu], sh[gu:2 * gu], sh[2 * gu:]], rw.view(np.uint8).reshape(-1),
                                  gw.view(np.uint8).reshape(-1))
    got = buf.cpu().numpy()
    assert np.array_equal(got[mask], img[mask]) and np.all(got[~mask] == 0xA5)      # every byte in its place, nothing beside them touched
    u, rl, sgl, y, idx, w = run_staged_layer(gpu, L, buf, k, m, rng)
    for j in range(m):
        assert np.all(np.abs(rl[j] - O.matvec(rty, hidden, ne, rw, u[j])) <= gguf_bound(rty, hidden, ne, rw, u[j]))
    want, widx, ww = oracle_layer(ty, hidden, ff, k, blobs, sh, rl, sgl, u)
    assert np.array_equal(idx, widx) and np.allclose(w, ww, rtol=2e-6, atol=0)
    assert all(rel_l2(y[j], want[j]) <= 1e-3 for j in range(m))


@pytest.mark.gpu
@pytest.mark.parametrize("ty,shared_ty,scatter", [(sz.EXL3(3), sz.EXL3(3), True), (sz.EXL3_HALF(2), sz.EXL3_HALF(2), False)])
def test_a_layer_staged_from_an_exl3_checkpoint_is_its_blobs_and_runs(gpu, tmp_path, ty, shared_ty, scatter):
    from test_gpu_path import oracle_layer, rel_l2
    rng = np.random.default_rng(ty)
    hidden, ff, ne, k, m = 512, 256, 10, 4, 4
    d = str(tmp_path / "ckpt")
    experts, shared, rw, gw = exl3_checkpoint(d, rng, ty, hidden, ff, ne, shared_ty, scatter=scatter)
    st = sz.SafeTensors(d)
    L, buf = staged(gpu, st, 3)
    img, mask, *_ = F.layer_image(experts, shared, rw.view(np.uint8).reshape(-1), gw.view(np.uint8).reshape(-1), *F.exl3_spacing(hidden, ff, experts[0][0].size))
    got = buf.cpu().numpy()
    assert np.array_equal(got[mask], img[mask]) and np.all(got[~mask] == 0xA5)
    u, rl, sgl, y, idx, w = run_staged_layer(gpu, L, buf, k, m, rng)
    want, widx, ww = oracle_layer(ty, hidden, ff, k, [np.concatenate(e) for e in experts], np.concatenate(shared), rl, sgl, u)
    assert np.array_equal(idx, widx) and np.allclose(w, ww, rtol=2e-6, atol=0)
    assert all(rel_l2(y[j], want[j]) <= 1e-3 for j in range(m))


@pytest.mark.gpu
def test_staging_more_than_the_pinned_buffers_hold(gpu, tmp_path):
    """Five 64 MiB rounds through the two pinned buffers (each reused after its copies have left it), one tensor larger than a
    buffer: the device holds the file's bytes."""
    rng = np.random.default_rng(9)
    hidden, ff, ne = 2048, 1024, 40                     # 40 experts x 3 x 2.2 MB = 267 MB
    per = hidden * ff // 32 * 34
    p = str(tmp_path / "big.gguf")
    parts = [rng.integers(0, 256, ne * per, dtype=np.uint8) for _ in range(3)]
    gguf_file(p, [], [("blk.7.ffn_gate_exps.weight", [hidden, ff, ne], sz.Q8_0, parts[0]), ("blk.7.ffn_up_exps.weight", [hidden, ff, ne], sz.Q8_0, parts[1]),
                      ("blk.7.ffn_down_exps.weight", [ff, hidden, ne], sz.Q8_0, parts[2])])
    g = sz.Gguf(p)
    L, buf = staged(gpu, g, 7)
    assert (L.shared_type, L.router_type, L.gate_type) == (-1, -1, -1) and L.stride == 3 * per and L.bytes == ne * L.stride
    got = buf.cpu().numpy().reshape(ne, 3, per)
    for i in range(3):
        assert np.array_equal(got[:, i, :], parts[i].reshape(ne, per))


# ---- differential fuzzing: the library and the oracle accept, refuse and read the same on damaged files ----------------------
def mutate(rng, base, limit):
    """One to three random edits (byte, bit, insertion; or a truncation) in the first `limit` bytes."""
    b = bytearray(base)
    for _ in range(int(rng.integers(1, 4))):
        kind, i = int(rng.integers(0, 4)), int(rng.integers(0, limit))
        if kind == 0:
            b[i] = int(rng.integers(0, 256))
        elif kind == 1:
            b[i] ^= 1 << int(rng.integers(0, 8))
        elif kind == 2:
            return bytes(b[:int(rng.integers(9, len(b) + 1))])
        else:
            b[i:i] = bytes([int(rng.integers(0, 256))])
    return bytes(b)


def test_damaged_gguf_headers_read_the_same_or_are_refused_by_both(tmp_path):
    p, q = str(tmp_path / "v.gguf"), str(tmp_path / "m.gguf")
    kv = [("u8", 0, 200), ("i8", 1, -3), ("s", 8, "hello"), ("general.alignment", 4, 64), ("arr.f", 9, (6, [1.5, -2.25])),
          ("arr.nested", 9, (9, [(4, [1, 2]), (4, [])])), ("arr.s", 9, (8, ["a", "bc"]))]
    gguf_file(p, kv, [("a", [3], 77, b"\x01" * 10), ("b", [100], 21, b"\x02" * 50), ("c", [64, 3], 8, b"\x03" * 204)], alignment=64, pad_tail=5)
    base = open(p, "rb").read()
    rng = np.random.default_rng(0)
    view = lambda ts: [(t["name"], t["dims"], t["type"], t["offset"], t["nbytes_layout"], t["nbytes_span"]) for t in ts]
    accepted = 0
    for it in range(1500):
        open(q, "wb").write(mutate(rng, base, len(base) - 400))
        try:
            g = sz.Gguf(q)
            got = (view(g.tensors()), g.shards()[0]["data_start"], g.keys())
        except sz.SzError:
            got = None
        try:
            o = F.gguf_open(q)
            want = (view(o["tensors"]), o["shards"][0]["data_start"], sorted(k.decode(errors="replace") for k in o["kv"]))
        except F.FormatError:
            want = None
        assert got == want, "mutation %d" % it
        accepted += got is not None
    assert 50 < accepted < 1400          # the edits land in both classes


def test_damaged_safetensors_headers_read_the_same_or_are_refused_by_both(tmp_path):
    q = str(tmp_path / "m.safetensors")
    base = (b'{"__metadata__":{"format":"pt","n":[1,{"a":null}]},"a.b":{"dtype":"I16","shape":[2,3],"data_offsets":[0,12]},'
            b'"s\\"x\\u00e9":{"dtype":"I32","shape":[],"data_offsets":[12,16], "extra": "}"}, "w" : {"shape":[4],"data_offsets":[16,24],"dtype":"F16"}}')
    rng = np.random.default_rng(1)
    accepted = 0
    for it in range(1500):
        text = mutate(rng, base, len(base))
        open(q, "wb").write(struct.pack("<Q", len(text)) + text + b"\0" * 24)
        try:
            got = sorted((t["name"].encode(), t["dtype"], t["shape"], t["start"] - 8 - len(text), t["end"] - 8 - len(text)) for t in sz.SafeTensors(q).tensors())
        except sz.SzError:
            got = None
        try:
            o = F.st_open([q])
            want = sorted((n.encode(), t["dtype"], t["shape"], t["start"] - 8 - len(text), t["end"] - 8 - len(text)) for n, t in o["tensors"].items())
        except F.FormatError:
            want = None
        if got is not None and want is not None and any(len(t[1]) > 7 or len(t[2]) > 8 or b"\0" in t[0] or b"\0" in t[1].encode() for t in want):
            continue                                                   # what the C structure cannot carry: a long dtype, a name with a NUL
        assert got == want, "mutation %d: %r" % (it, text)
        accepted += got is not None
    assert 20 < accepted < 1400


def test_the_readers_under_the_address_and_undefined_behaviour_sanitizers(tmp_path):
    """The readers parse files they did not write: formats.cpp, compiled on its own with -fsanitize=address,undefined (host code
    only), reads a thousand damaged GGUF and safetensors files without a report."""
    import subprocess
    csrc = os.path.join(ROOT, "shadow_engine_amd", "csrc")
    exe = str(tmp_path / "driver")
    subprocess.run(["g++", "-O1", "-g", "-std=c++17", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-I", os.path.join(ROOT, "include"),
                    "-I", csrc, os.path.join(ROOT, "tests", "formats_sanitizer_driver.cpp"), os.path.join(csrc, "formats.cpp"), os.path.join(csrc, "hipbind.cpp"),
                    "-ldl", "-pthread", "-o", exe], check=True)
    rng = np.random.default_rng(5)
    g = str(tmp_path / "base.gguf")
    kv = [("u8", 0, 200), ("s", 8, "hello"), ("general.alignment", 4, 64), ("arr.nested", 9, (9, [(4, [1, 2]), (4, [])])), ("arr.s", 9, (8, ["a", "bc"])),
          ("general.architecture", 8, "toy"), ("toy.block_count", 4, 3)]
    gguf_file(g, kv, [("a", [3], 77, b"\x01" * 10), ("b", [100], 21, b"\x02" * 50), ("blk.0.ffn_gate_exps.weight", [32, 32, 2], 8, b"\4" * (2 * 32 * 34))], alignment=64)
    base = open(g, "rb").read()
    gfiles = []
    for i in range(500):
        gfiles.append(str(tmp_path / ("g%03d.gguf" % i)))
        open(gfiles[-1], "wb").write(mutate(rng, base, len(base) - 300))
    sb = str(tmp_path / "base.safetensors")
    st_file(sb, [("p.suh", "F16", [128], b"\0" * 256), ("p.svh", "F16", [256], b"\1" * 512), ("p.mul1", "I32", [], MUL1),
                 ("p.trellis", "I16", [8, 16, 32], np.arange(8 * 16 * 32, dtype=np.uint16).tobytes()), ("q.trellis", "I16", [8, 16, 40], b"\2" * (8 * 16 * 40 * 2)),
                 ("q.mul1", "I32", [], MUL1), ("q.suh", "F32", [128], b"\0" * 512), ("q.svh", "BF16", [256], b"\1" * 512)], metadata={"format": "pt"})
    base = open(sb, "rb").read()
    n = struct.unpack("<Q", base[:8])[0]
    sfiles = [sb]
    for i in range(500):
        sfiles.append(str(tmp_path / ("s%03d.safetensors" % i)))
        open(sfiles[-1], "wb").write(mutate(rng, base, 8 + n))
    env = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=1")
    for kind, files in (("g", gfiles), ("s", sfiles)):
        r = subprocess.run([exe, kind] + files, env=env, capture_output=True, text=True)
        assert r.returncode == 0 and r.stdout.startswith("ok "), r.stderr[-2000:]
        ok, refused = int(r.stdout.split()[1]), int(r.stdout.split()[3])
        assert ok > 10 and refused > 10 and ok + refused == len(files)



@pytest.mark.gpu
def test_single_tensors_and_blobs_staged_to_any_address(gpu, tmp_path):
    """The head's matrix (larger than a staging buffer), a plain safetensors tensor and an EXL3 projection both ways, each to a
    device address that is not 16-byte aligned: the device holds the file's bytes and nothing beside them is touched."""
    rng = np.random.default_rng(21)
    big = rng.integers(0, 256, 4096 * 512 * 34 + 0, dtype=np.uint8)        # a 71 MB Q8_0 matrix: 4096 x 16384
    small = rng.normal(size=300).astype(np.float32)
    p = str(tmp_path / "t.gguf")
    gguf_file(p, [], [("token_embd_norm.weight", [300], 0, small.tobytes()), ("output.weight", [16384, 4096], sz.Q8_0, big)])
    g = sz.Gguf(p)
    buf = gpu.full((big.size + 64,), 0x5A, dtype=gpu.uint8, device="cuda")
    with pytest.raises(sz.SzError, match="bytes into"):
        g.stage_tensor("output.weight", buf.data_ptr() + 4, big.size - 1)
    with pytest.raises(sz.SzError, match="no tensor"):
        g.stage_tensor("nope", buf.data_ptr(), big.size)
    g.stage_tensor("output.weight", buf.data_ptr() + 4, big.size)
    got = buf.cpu().numpy()
    assert np.array_equal(got[4:4 + big.size], big) and np.all(got[:4] == 0x5A) and np.all(got[4 + big.size:] == 0x5A)
    g.stage_tensor("token_embd_norm.weight", buf.data_ptr() + 1, 1200)           # byte-aligned only
    assert np.array_equal(buf[1:1201].cpu().numpy(), small.view(np.uint8)) and int(buf[0]) == 0x5A

    blob, suh, svh, tr, inf, outf = golden_parts()
    pre = "lm_head"
    a, b = str(tmp_path / "a.safetensors"), str(tmp_path / "b.safetensors")
    st_file(a, [(pre + ".mul1", "I32", [], MUL1), (pre + ".suh", "F16", [inf], suh), (pre + ".svh", "F16", [outf], svh), (pre + ".trellis", "I16", [inf // 16, outf // 16, 32], tr),
                ("norm.weight", "BF16", [7], b"\x01\x02" * 7)])
    st_file(b, [(pre + ".suh", "F16", [inf], suh), (pre + ".svh", "F16", [outf], svh), (pre + ".mul1", "I32", [], struct.pack("<i", 1)), (pre + ".trellis", "I16", [inf // 16, outf // 16, 32], tr)])
    for path in (a, b):                                                           # put together; one range of the file
        st = sz.SafeTensors(path)
        d = gpu.full((blob.size + 32,), 0x33, dtype=gpu.uint8, device="cuda")
        st.stage_exl3_blob(pre, d.data_ptr() + 8, blob.size)
        got = d.cpu().numpy()
        assert np.array_equal(got[8:8 + blob.size], blob) and np.all(got[:8] == 0x33) and np.all(got[8 + blob.size:] == 0x33)
        with pytest.raises(sz.SzError):
            st.stage_exl3_blob(pre, d.data_ptr(), blob.size - 1)
    st = sz.SafeTensors(a)
    d = gpu.zeros(32, dtype=gpu.uint8, device="cuda")
    st.stage_tensor("norm.weight", d.data_ptr() + 2, 14)
    assert d.cpu().numpy().tolist() == [0, 0] + [1, 2] * 7 + [0] * 16
