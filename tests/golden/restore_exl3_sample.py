"""Writes tests/golden/exl3_k2_gate_proj.blob and tests/golden/exl3_k4_shared_gate_proj.blob from the reference's fixture
eval/fixtures/exl3_sample.safetensors.

The copy of that fixture in the reference checkout this build sees went through a CRLF -> LF text normalisation: the
file holds no 0D 0A pair at all (about 19 are expected in 1.2 MB of trellis words) and is 12 bytes shorter than its
own header says.  Five of the lost 0D bytes fall inside the trellis of `layers.0.mlp.experts.0.gate_proj` (K = 2), seven
inside the trellis of `layers.0.mlp.shared_expert.gate_proj` (K = 4) that follows.

The five positions were located by (1) decoding every tile at byte shifts 0..5 and finding the monotone shift path of
least energy (a misaligned tile decodes to unit-variance noise, an aligned K = 2 tile to about 0.96), then (2) choosing,
among the 0A bytes near each change point, the combination whose reconstructed matrix reproduces the reference's
recorded sum of squares 287.702278 (crates/shadowzero-model/tests/exl3_vs_gguf.rs:133) to all printed digits.  The
energy statistic alone leaves each position uncertain by about +-16 tiles (0.3 % of the tensor), so the restored
tensor is checked at the reference's own tolerance (1e-3 of the sum of squares, 1e-6 on the first four values), which
a decoder that mis-addresses tiles misses by 4 %.

The K = 4 tensor the same way: an aligned K = 4 tile decodes to a mean square of about 0.81, a misaligned one to about
0.93, which places each of the seven change points to within a few tiles; among the 0A bytes within 8 tiles of each, 52
combinations reproduce the recorded sum of squares 161.198363 (exl3_vs_gguf.rs:134) to its last printed digit, and one
of them is at the same time the choice of least decoded energy at every one of the seven change points (its total decoded
energy is lower than that of the next best by the equivalent of five misaligned tiles): that one is used.  Two of the
change points lie in the same 128 x 128 block, where the sum of squares of the rotated-back weights is not additive over
tiles, so those two were searched jointly.

Run from the repository root in a container that has /root/reference; the output is a blob in the engine's layout
[suh f16 | svh f16 | 4-byte marker | trellis] (exl3.rs:388-398).
"""
import json
import struct
import sys

import numpy as np

SRC = "/root/reference/eval/fixtures/exl3_sample.safetensors"
PREFIX = "model.language_model.layers.0.mlp.experts.0.gate_proj"
# offsets inside the damaged trellis bytes: a 0D is put back before the 0A found at each
INSERT_BEFORE = [88577, 229059, 330937, 344788, 349453]
PREFIX_K4 = "model.language_model.layers.0.mlp.shared_expert.gate_proj"
INSERT_BEFORE_K4 = [275384, 285425, 557712, 604135, 628469, 803168, 811523]


def restore(damaged, positions, size):
    parts, last = [], 0
    for p in positions:
        assert damaged[p] == 0x0A
        parts += [damaged[last:p], np.array([0x0D], np.uint8)]
        last = p
    parts.append(damaged[last:])
    out = np.concatenate(parts)
    assert out.size == size
    return out


def main(out="tests/golden/exl3_k2_gate_proj.blob", out4="tests/golden/exl3_k4_shared_gate_proj.blob"):
    b = open(SRC, "rb").read()
    n = struct.unpack("<Q", b[:8])[0]
    header = json.loads(b[8:8 + n])
    data = b[8 + n:]
    lo_s, hi_s = header[PREFIX + ".suh"]["data_offsets"]
    lo_v, hi_v = header[PREFIX + ".svh"]["data_offsets"]
    lo_t, hi_t = header[PREFIX + ".trellis"]["data_offsets"]
    assert header[PREFIX + ".trellis"]["shape"] == [160, 40, 32]
    damaged = np.frombuffer(data[lo_t:hi_t - len(INSERT_BEFORE)], np.uint8)
    parts, last = [], 0
    for p in INSERT_BEFORE:
        assert damaged[p] == 0x0A
        parts += [damaged[last:p], np.array([0x0D], np.uint8)]
        last = p
    parts.append(damaged[last:])
    trellis = np.concatenate(parts)
    assert trellis.size == hi_t - lo_t == 409600
    # the tensor that follows must now start where the header says: its `mul1` scalar is the codebook multiplier
    nxt = header["model.language_model.layers.0.mlp.shared_expert.gate_proj.mul1"]["data_offsets"][0]
    assert data[nxt - len(INSERT_BEFORE):nxt - len(INSERT_BEFORE) + 4] == struct.pack("<I", 0x83DCD12D)
    blob = data[lo_s:hi_s] + data[lo_v:hi_v] + struct.pack("<i", 1) + trellis.tobytes()
    assert len(blob) == 2 * 2560 + 2 * 640 + 4 + 409600
    open(out, "wb").write(blob)
    print(f"wrote {out}: {len(blob)} bytes")
    # the K = 4 tensor: everything of it lies 5 bytes early in the damaged file, and its trellis has lost 7 more
    lost = len(INSERT_BEFORE)
    lo_s, hi_s = (o - lost for o in header[PREFIX_K4 + ".suh"]["data_offsets"])
    lo_v, hi_v = (o - lost for o in header[PREFIX_K4 + ".svh"]["data_offsets"])
    lo_t, hi_t = header[PREFIX_K4 + ".trellis"]["data_offsets"]
    assert header[PREFIX_K4 + ".trellis"]["shape"] == [160, 40, 64] and hi_t - lost - len(INSERT_BEFORE_K4) == len(data)
    trellis4 = restore(np.frombuffer(data[lo_t - lost:], np.uint8), INSERT_BEFORE_K4, 819200)
    blob4 = data[lo_s:hi_s] + data[lo_v:hi_v] + struct.pack("<i", 1) + trellis4.tobytes()
    assert len(blob4) == 2 * 2560 + 2 * 640 + 4 + 819200
    open(out4, "wb").write(blob4)
    print(f"wrote {out4}: {len(blob4)} bytes")


if __name__ == "__main__":
    main(*sys.argv[1:])
