"""Readers for the committed golden fixtures (plain data; nothing is executed from the files)."""
import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def iq3s_records():
    """[(tensor, block index, 110 block bytes, 256 expected f32 bit patterns)] from iq3_s_blocks.txt."""
    lines = [l.strip() for l in open(os.path.join(GOLDEN, "iq3_s_blocks.txt")) if l.strip() and not l.startswith("#")]
    assert len(lines) % 3 == 0
    out = []
    for i in range(0, len(lines), 3):
        ty, tensor, block = lines[i].split()
        assert ty == "IQ3_S"
        raw = np.frombuffer(bytes.fromhex(lines[i + 1]), np.uint8)
        want = np.frombuffer(bytes.fromhex(lines[i + 2]), ">u4").astype(np.uint32)
        out.append((tensor, int(block), raw, want))
    return out


def exl3_k2_gate_proj():
    """(in, out, K, blob) of the real K = 2 projection `layers.0.mlp.experts.0.gate_proj` of the reference's EXL3
    sample fixture, in the engine's blob layout (see golden/restore_exl3_sample.py for how it was recovered)."""
    blob = np.fromfile(os.path.join(GOLDEN, "exl3_k2_gate_proj.blob"), np.uint8)
    assert blob.size == 2 * 2560 + 2 * 640 + 4 + 2560 * 640 * 2 // 8
    return 2560, 640, 2, blob


def exl3_k4_shared_gate_proj():
    """(in, out, K, blob) of the real K = 4 projection `layers.0.mlp.shared_expert.gate_proj` of the same fixture."""
    blob = np.fromfile(os.path.join(GOLDEN, "exl3_k4_shared_gate_proj.blob"), np.uint8)
    assert blob.size == 2 * 2560 + 2 * 640 + 4 + 2560 * 640 * 4 // 8
    return 2560, 640, 4, blob


def exl3_real_tensors():
    """Both real tensors with what the reference recorded for them (crates/shadowzero-model/tests/exl3_vs_gguf.rs:133-134):
    (in, out, K, blob, sum of squares, first four weights)."""
    return [exl3_k2_gate_proj() + (287.702278, [-0.042833105, -0.0065446747, 0.029719023, -0.030945573]),
            exl3_k4_shared_gate_proj() + (161.198363, [-0.0071623405, 0.00092289475, -0.0021615676, -0.0026322217])]
