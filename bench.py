#!/usr/bin/env python3
"""Benchmark of the speculative-verify hot path on one MI355X.  Prints ONE JSON line.

Default workload (config 5, the one the headline metric is quoted on): a step is one full-depth verify round: 48 MoE
layers (hidden 2048, 512 EXL3 experts + a shared expert, top-10, per-layer bit rates 2/3/4 from a seeded assignment, about
29 GB resident) on a 4-token batch (1 accepted + 3 drafts), then the 151,936 x 2048 Q8_0 lm_head, arg-max and greedy
acceptance of the 3 drafts.  Only the MoE and head portion exists here, so only it is timed; inputs are resident in HBM
before the timed region.

The other configurations of the path can be timed the same way with --workload (they are parity-test cases first; their
lines carry the same fields):
    config1  one Q8_0 1024 x 2048 matrix-vector product
    config2  one IQ3_S MoE layer for one token (512 experts + shared, top-10); a step walks through 8 different layers
    config3  one EXL3 K=3 MoE layer for 4 tokens + head + acceptance (weights of the one layer stay warm in cache)
    config4  one prefill chunk: 512 tokens through the 512 IQ3_S experts of a layer on int8 activations (int8 MFMA)
    exl3head the 151,936 x 2048 lm_head of an EXL3 checkpoint (--bits K, default 4) for the batch, arg-max fused in
    exl3top  the same head's top-64 hand-off to the host; --screen N goes through the inexact 2-bit screen, N blocks a row
    stage    one EXL3 layer of a safetensors checkpoint staged into HBM (the loader beside the path; PCIe-inclusive)
    snapshot the rollback point of a pass: 73 device ranges (79 MB of recurrent state) saved and put back, a launch each

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload config5] [--layers 48]

The default run then times configurations 1-4 once each (`other_configs`).  `roofline` sets the dominant kernel against the
HBM roof and, from the hardware counters in profiles/counters.json (quoted only while the kernel file they were measured on is
unchanged), against the vector-ALU roof; `bound` names the nearer one.  `cpu_baseline` times the CPU oracle on one thread
and on all hardware threads, best of 20 runs.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
INT8_MFMA_PEAK_TOPS = 5000.0
HIDDEN, FF, NE, TOPK, VOCAB, ROWS = 2048, 512, 512, 10, 151936, 4
COUNTERS = os.path.join(ROOT, "profiles", "counters.json")
SIMDS = 256 * 4                                  # 256 compute units x 4 SIMDs; a wave64 vector instruction takes one for 4 cycles


def load_counters(sz):
    """profiles/counters.json (written by `python3 profile_counters.py` from rocprofv3 databases): per-kernel
    hardware counters of the benchmark's workloads, stamped with the cache keys of the kernel files they were measured on.
    Returns (counters or None, stale): stale maps every kernel whose file has changed since (or every kernel, when the
    file is missing) to the reason its counters are not quoted."""
    file_of = {name: f for name, f, _ in sz.kernels()}
    try:
        c = json.load(open(COUNTERS))
    except (OSError, ValueError) as e:
        return None, {k: "no usable profiles/counters.json (%s)" % type(e).__name__ for k in file_of}
    now, then = sz.program_keys(), c.get("kernel_keys", {})
    changed = sorted(f for f in now if then.get(f) != now[f])
    return c, {k: "profiles/counters.json was measured on another %s" % f for k, f in file_of.items() if f in changed}


class Workload:
    """step(): one pass, launched on `stream`; set_eager(bool): graph replay off/on where the workload has one;
    step_bytes: algorithmic bytes of a step; kernel_bytes: {kernel: algorithmic bytes per launch}; check(): raises if the
    pass went wrong; describe: the config object of the JSON line."""
    extra = {}
    kernel_ops = {}
    cold_variant = False

    def set_eager(self, eager):
        pass

    def check(self):
        pass


SPACED = True   # --contiguous-experts: the reference's layout, an expert's three blobs back to back


def exl3_experts(torch, synth_device, seed, kb):
    """A layer of EXL3 experts in the layout the stager writes (every trellis on a 128-byte line: sz_layer_spacing), or
    contiguous: (buffer from the first expert on, stride, gap between an expert's projections)."""
    if SPACED:
        return synth_device.exl3_layer(torch, seed, HIDDEN, FF, NE, kb, spaced=True)
    return (*synth_device.exl3_layer(torch, seed, HIDDEN, FF, NE, kb), 0)


def exl3_round(torch, sz, synth, synth_device, stream, L, rates, tag, mode=0):
    w = Workload()
    sess = sz.Session(HIDDEN, FF, NE, TOPK, L, VOCAB, 8)
    sess.set_expert_mode(mode)   # 0: the exact kernels (the default); 1, 2: the matrix-core launches
    layers = []
    for l, kb in enumerate(rates):
        buf, stride, gap = exl3_experts(torch, synth_device, 1000 + l, kb)
        layers.append((buf, stride, gap))
        sess.set_layer(l, sz.EXL3(kb), buf.data_ptr(), stride, sz.EXL3(kb), buf.data_ptr() + NE * stride, gap=gap)
    head = synth_device.q8_0_head(torch, 7, VOCAB, HIDDEN)
    sess.set_head(sz.Q8_0, head.data_ptr())
    g = torch.Generator(device="cuda")
    g.manual_seed(11)
    u = torch.randn((L, ROWS, HIDDEN), device="cuda", generator=g)
    rl = torch.randn((L, ROWS, NE), device="cuda", generator=g)
    sgl = torch.randn((L, ROWS), device="cuda", generator=g)
    hu = torch.randn((ROWS, HIDDEN), device="cuda", generator=g)
    y = torch.zeros((L, ROWS, HIDDEN), device="cuda")
    out = torch.zeros(2 + 8, dtype=torch.int32, device="cuda")
    drafts = torch.zeros(ROWS - 1, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()

    def step():
        sess.verify_round(ROWS, u.data_ptr(), rl.data_ptr(), sgl.data_ptr(), y.data_ptr(), hu.data_ptr(), drafts.data_ptr(),
                          out.data_ptr(), stream.handle)

    # a first round finds the model's tokens; the drafts are then planted so that 2 of the 3 are accepted
    step()
    stream.synchronize()
    ids = out.cpu().numpy().view(np.uint32)[2:2 + ROWS].copy()
    planted = ids[:ROWS - 1].astype(np.int64)
    wrong = min(2, ROWS - 2)                       # the first draft that is not the model's token: drafts before it are accepted
    planted[wrong] = (planted[wrong] + 1) % VOCAB
    drafts.copy_(torch.from_numpy(planted.astype(np.int32)))
    torch.cuda.synchronize()

    def check():
        o = out.cpu().numpy().view(np.uint32)
        assert o[0] == wrong + 1 and o[1] == ids[wrong], "acceptance of the planted drafts went wrong: %r" % (o[:6],)

    # algorithmic bytes of a round: every distinct expert touched (+ the shared one) once, the head once, activations
    rl_h = rl.cpu().numpy()
    sel = [np.unique(synth_device.route_ids(rl_h[l], TOPK)) for l in range(L)]
    ebytes = {kb: sum(synth.expert_bytes(synth.exl3_type(kb), HIDDEN, FF)) for kb in (2, 3, 4)}
    gu_bytes = {kb: 2 * synth.exl3_blob_len(HIDDEN, FF, kb) for kb in (2, 3, 4)}
    dn_bytes = {kb: synth.exl3_blob_len(FF, HIDDEN, kb) for kb in (2, 3, 4)}
    head_bytes = VOCAB * HIDDEN // 32 * 34
    act_bytes = L * ROWS * (2 * HIDDEN + NE + 1) * 4 + ROWS * HIDDEN * 4 + 64
    moe_bytes = sum((len(sel[l]) + 1) * ebytes[rates[l]] for l in range(L))
    n_sel = {kb: float(np.mean([len(sel[l]) + 1 for l in range(L) if rates[l] == kb])) if kb in rates else 0.0 for kb in (2, 3, 4)}
    pairs = ROWS * (TOPK + 1)                                       # (token, expert) work items, the shared expert included
    act_gu = ROWS * (HIDDEN + NE) * 4 + pairs * 2 * FF * 2 * 4     # u and logits in; two split-K partials of gate and up out
    act_dn = pairs * 2 * FF * 2 * 4 + pairs * HIDDEN * 4           # those partials in; one down output per pair out
    w.kernel_bytes = {n: head_bytes + ROWS * HIDDEN * 4 for n in ("head_q8_0_argmax", "head_q8_0_argmax_mfma", "head_q8_0_argmax_mfma_n8")}
    for kb in (2, 3, 4):
        for form in ("exl3", "mma_exl3", "mmaw_exl3", "lin_exl3", "linw_exl3", "exl3f"):      # the exact launches, the matrix-core ones and the f16-input ones (sz_session_set_expert_mode)
            w.kernel_bytes["verify_gate_up_%s_%d" % (form, kb)] = n_sel[kb] * gu_bytes[kb] + act_gu
            w.kernel_bytes["verify_down_%s_%d" % (form, kb)] = n_sel[kb] * dn_bytes[kb] + act_dn
    w.step, w.check, w.set_eager = step, check, (lambda eager: sess.set_graph(not eager))
    w.step_bytes = moe_bytes + head_bytes + act_bytes
    w.counters_key = "config5" if (L == 48 and tag == "config 5" and ROWS == 4) else ("config3" if (tag == "config 3" and ROWS == 4) else None)
    if mode:
        w.counters_key = "config5_mode%d" % mode if w.counters_key == "config5" else None
    w.cold_variant = tag == "config 3"
    w.dtype = "f32 accumulate over EXL3 f16 codebook weights / Q8_0 int8"
    w.describe = {"workload": "%s: verify round, %d MoE layer%s (hidden 2048, 512 experts + shared, top-10, EXL3 K in %s), %d-token batch, "
                              "Q8_0 lm_head 151936x2048, arg-max, greedy acceptance of %d drafts" % (tag, L, "s" if L > 1 else "", sorted(set(rates)), ROWS, ROWS - 1),
                  "layers": L, "rows": ROWS, "resident_GB": round(sum(b.numel() for b, _, _ in layers) / 1e9 + head.numel() / 1e9, 2)}
    w.describe["expert_layout"] = "every trellis on a 128-byte line (sz_layer_spacing)" if SPACED else "contiguous [gate|up|down]"
    if mode:
        w.describe["expert_mode"] = {1: "matrix cores, the codebook's f16 values", 2: "matrix cores, the linearised codebook",
                                     3: "the exact decode, inputs rounded to f16, two products an instruction"}[mode]
    w.extra = {"accepted_drafts": wrong}
    w.cpu = ("exl3_token", (layers[0], rates[0], rl_h[0], u[0].cpu().numpy(), sgl[0].cpu().numpy()))
    w.keep = (sess, layers, head, u, rl, sgl, hu, y, out, drafts)
    return w


def q8_matvec(torch, sz, synth, synth_device, stream):
    w = Workload()
    rows, cols = 1024, 2048
    mat = synth_device.q8_0_head(torch, 3, rows, cols)
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    x = torch.randn(cols, device="cuda", generator=g)
    y = torch.zeros(rows, device="cuda")
    w.step = lambda: sz.matvec_cols(sz.Q8_0, mat.data_ptr(), cols, rows, x.data_ptr(), cols, y.data_ptr(), rows, 1, 0, 0, stream.handle)
    w.step_bytes = mat.numel() + cols * 4 + rows * 4
    w.kernel_bytes = {"matvec_cols_q8_0": w.step_bytes}
    w.dtype = "f32 accumulate over Q8_0 int8"
    w.cold_variant = True
    w.describe = {"workload": "config 1: Q8_0 1024x2048 matrix-vector product, one input (the matrix stays warm in cache between steps)"}
    w.cpu = ("q8_0_matvec", (mat.cpu().numpy(), x.cpu().numpy(), rows, cols))
    w.keep = (mat, x, y)
    return w


def iq3s_decode(torch, sz, synth, synth_device, stream, L=8):
    w = Workload()
    sess = sz.Session(HIDDEN, FF, NE, TOPK, L, 0, 8)
    layers = []
    for l in range(L):
        buf, stride = synth_device.iq3_s_layer(torch, 300 + l, HIDDEN, FF, NE)
        layers.append(buf)
        sess.set_layer(l, sz.IQ3_S, buf.data_ptr(), stride, sz.IQ3_S, buf.data_ptr() + NE * stride)
    g = torch.Generator(device="cuda")
    g.manual_seed(12)
    u = torch.randn((L, 1, HIDDEN), device="cuda", generator=g)
    rl = torch.randn((L, 1, NE), device="cuda", generator=g)
    sgl = torch.randn((L, 1), device="cuda", generator=g)
    y = torch.zeros((L, 1, HIDDEN), device="cuda")

    def step():
        for l in range(L):
            sess.moe_layer_verify(l, 1, u[l].data_ptr(), rl[l].data_ptr(), sgl[l].data_ptr(), y[l].data_ptr(), stream.handle)

    expert = sum(synth.expert_bytes(sz.IQ3_S, HIDDEN, FF))
    w.step = step
    w.step_bytes = L * ((TOPK + 1) * expert + (2 * HIDDEN + NE + 1) * 4)
    gu, _, dn = synth.expert_bytes(sz.IQ3_S, HIDDEN, FF)
    w.kernel_bytes = {"decode_gate_up_iq3_s": (TOPK + 1) * 2 * gu + (HIDDEN + NE) * 4 + (TOPK + 1) * FF * 4,      # one token: two launches
                      "decode_down_combine_iq3_s": (TOPK + 1) * dn + (TOPK + 1) * FF * 4 + HIDDEN * 4,
                      "verify_gate_up_iq3_s": (TOPK + 1) * 2 * gu + (HIDDEN + NE) * 4 + (TOPK + 1) * 2 * FF * 4,   # the three-launch form
                      "verify_down_iq3_s": (TOPK + 1) * dn + (TOPK + 1) * (2 * FF + HIDDEN) * 4,
                      "matvec_grouped_iq3_s": (TOPK + 1) * expert / 2.0}      # the planned form: gate+up in one launch, down in the other: the mean
    w.dtype = "f32 accumulate over IQ3_S grid weights"
    w.cold_variant = True
    w.describe = {"workload": "config 2: IQ3_S MoE layer for one token (hidden 2048, 512 experts + shared, top-10); a step is %d "
                              "different layers one after the other" % L, "layers": L, "rows": 1,
                  "resident_GB": round(sum(b.numel() for b in layers) / 1e9, 2)}
    w.counters_key = "config2" if L == 8 else None
    w.cpu = ("iq3_s_token", (layers[0], stride, rl[0].cpu().numpy(), u[0].cpu().numpy(), sgl[0].cpu().numpy()))
    w.keep = (sess, layers, u, rl, sgl, y)
    return w


def iq3s_prefill(torch, sz, synth, synth_device, stream, tokens=512):
    w = Workload()
    sess = sz.Session(HIDDEN, FF, NE, TOPK, 1, 0, 8)
    buf, stride = synth_device.iq3_s_layer(torch, 400, HIDDEN, FF, NE)
    sess.set_layer(0, sz.IQ3_S, buf.data_ptr(), stride, 0, 0)
    rng = np.random.default_rng(4)
    logits = synth.zipf_router_logits(rng, tokens, NE)
    g = torch.Generator(device="cuda")
    g.manual_seed(13)
    x = torch.randn((tokens, HIDDEN), device="cuda", generator=g)
    rl = torch.from_numpy(logits).cuda()
    sgl = torch.zeros(tokens, device="cuda")
    y = torch.zeros((tokens, HIDDEN), device="cuda")
    w.step = lambda: sess.moe_prefill_chunk(0, tokens, x.data_ptr(), rl.data_ptr(), sgl.data_ptr(), y.data_ptr(), stream.handle)
    ids = synth_device.route_ids(logits, TOPK)
    distinct = int(np.unique(ids).size)
    gu, _, dn = synth.expert_bytes(sz.IQ3_S, HIDDEN, FF)
    w.step_bytes = distinct * (2 * gu + dn) + tokens * (2 * HIDDEN + NE) * 4
    # gate/up: the experts' two matrices, the tokens' int8 codes and scales in, H's codes and scales out; down: the experts' third
    # matrix, H in, the pairs' rows of the result out (f32, summed by the combine launch: counted as the EXL3 launches' are)
    w.kernel_bytes = {"prefill_gate_up_iq3_s": distinct * 2 * gu + tokens * HIDDEN * 9 // 8 + tokens * TOPK * FF * 9 // 8,
                      "prefill_down_iq3_s": distinct * dn + tokens * TOPK * FF * 9 // 8 + tokens * TOPK * HIDDEN * 4}
    w.kernel_ops = {"prefill_gate_up_iq3_s": 2.0 * tokens * TOPK * 2 * FF * HIDDEN, "prefill_down_iq3_s": 2.0 * tokens * TOPK * FF * HIDDEN}
    w.dtype = "int8 x int8 -> int32 MFMA, f32 scales"
    w.describe = {"workload": "config 4: prefill chunk, %d tokens x hidden 2048 through 512 IQ3_S experts (top-10, Zipf-skewed routing, "
                              "%d distinct experts hit) on per-32 int8 activations" % (tokens, distinct), "rows": tokens,
                  "resident_GB": round(buf.numel() / 1e9, 2)}
    w.counters_key = "config4" if tokens == 512 else None
    w.cpu = ("iq3_s_int8_pairs", (buf, stride, ids, x[:8].cpu().numpy()))
    w.keep = (sess, buf, x, rl, sgl, y)
    return w


def exl3_prefill(torch, sz, synth, synth_device, stream, tokens=512, bits=3):
    """The prefill chunk of config 4 through the verify round's kind of experts: EXL3 at `bits` bits a weight, f16 activations on the
    rows of the matrix instruction (no int8 quantization), the shared expert included."""
    w = Workload()
    sess = sz.Session(HIDDEN, FF, NE, TOPK, 1, 0, 8)
    buf, stride, gap = exl3_experts(torch, synth_device, 4400, bits)
    sess.set_layer(0, sz.EXL3(bits), buf.data_ptr(), stride, sz.EXL3(bits), buf.data_ptr() + NE * stride, gap=gap)
    rng = np.random.default_rng(4)
    logits = synth.zipf_router_logits(rng, tokens, NE)
    g = torch.Generator(device="cuda")
    g.manual_seed(13)
    x = torch.randn((tokens, HIDDEN), device="cuda", generator=g)
    rl = torch.from_numpy(logits).cuda()
    sgl = torch.randn(tokens, device="cuda", generator=g)
    y = torch.zeros((tokens, HIDDEN), device="cuda")
    w.step = lambda: sess.moe_prefill_chunk(0, tokens, x.data_ptr(), rl.data_ptr(), sgl.data_ptr(), y.data_ptr(), stream.handle)
    ids = synth_device.route_ids(logits, TOPK)
    distinct = int(np.unique(ids).size) + 1
    pairs = tokens * (TOPK + 1)
    zs = HIDDEN // 512
    gu, dn = 2 * synth.exl3_blob_len(HIDDEN, FF, bits), synth.exl3_blob_len(FF, HIDDEN, bits)
    w.step_bytes = distinct * (gu + dn) + tokens * (2 * HIDDEN + NE) * 4
    # gate/up: the experts' two matrices, the rows of x, the raw partial sums; act: the partial sums in, f16 operand rows out;
    # down: the experts' third matrix, the operand rows, the pairs' rows of the result
    w.kernel_bytes = {"prefill_gate_up_exl3_%d" % bits: distinct * gu + tokens * HIDDEN * 4 + pairs * 2 * zs * FF * 4,
                      "prefill_act_exl3": pairs * 2 * zs * FF * 4 + pairs * FF * 2,
                      "prefill_down_exl3_%d" % bits: distinct * dn + pairs * FF * 2 + pairs * HIDDEN * 4}
    w.dtype = "f32 accumulate over EXL3 f16 codebook weights x f16 activations (matrix cores)"
    w.describe = {"workload": "prefill chunk, %d tokens x hidden 2048 through 512 EXL3 K=%d experts + the shared one (top-10, Zipf-skewed routing, "
                              "%d distinct experts hit), f16 activations" % (tokens, bits, distinct), "rows": tokens, "resident_GB": round(buf.numel() / 1e9, 2)}
    w.describe["expert_layout"] = "every trellis on a 128-byte line (sz_layer_spacing)" if SPACED else "contiguous [gate|up|down]"
    w.counters_key = "exl3prefill" if (tokens == 512 and bits == 3) else None
    rl_h = logits[:1]
    w.cpu = ("exl3_token", ((buf, stride, gap), bits, rl_h, x[:1].cpu().numpy(), sgl[:1].cpu().numpy()))
    w.keep = (sess, buf, x, rl, sgl, y)
    return w


def exl3_head(torch, sz, synth, synth_device, stream, bits):
    """The lm_head of an EXL3 checkpoint: 151936 x 2048 at `bits` bits a weight for a verify batch, arg-max fused in."""
    w = Workload()
    sess = sz.Session(HIDDEN, FF, 8, 2, 0, VOCAB, 8)
    blob = synth_device.exl3_matrix(torch, 21, HIDDEN, VOCAB, bits)
    sess.set_head(sz.EXL3(bits), blob.data_ptr())
    g = torch.Generator(device="cuda")
    g.manual_seed(14)
    u = torch.randn((ROWS, HIDDEN), device="cuda", generator=g)
    ids = torch.zeros(8, dtype=torch.int32, device="cuda")
    w.step = lambda: sess.head_argmax(ROWS, u.data_ptr(), ids.data_ptr(), stream.handle)
    w.step_bytes = blob.numel() + ROWS * HIDDEN * 4 + ROWS * 4
    w.kernel_bytes = {"head_exl3_%d" % bits: blob.numel() + HIDDEN // 128 * 16 * 256}
    w.dtype = "f32 accumulate over EXL3 f16 codebook weights (f16 matrix cores, inputs as f16 high + low parts)"
    w.cold_variant = True
    w.describe = {"workload": "EXL3 lm_head 151936 x 2048 at K = %d for a %d-row verify batch, arg-max fused in (three launches: rotate, "
                              "product + per-block arg-max, merge)" % (bits, ROWS), "rows": ROWS, "resident_GB": round(blob.numel() / 1e9, 2)}
    w.counters_key = "exl3head" if (bits == 4 and ROWS == 4) else None
    w.cpu = ("exl3_matvec", (blob, bits, u[0].cpu().numpy()))
    w.keep = (sess, blob, u, ids)
    return w


def exl3_head_top(torch, sz, synth, synth_device, stream, bits, k_blk):
    """The top-64 hand-off of an EXL3 head (151936 x 2048): logits, slice sorts and merge, the 2 KiB a row brought to the host;
    with k_blk > 0 through the inexact 2-bit screen (the k_blk best 128-output blocks a row computed exactly)."""
    w = Workload()
    sess = sz.Session(HIDDEN, FF, 8, 2, 0, VOCAB, 8)
    blob = synth_device.exl3_matrix(torch, 21, HIDDEN, VOCAB, bits)
    sess.set_head(sz.EXL3(bits), blob.data_ptr())
    if k_blk:
        sess.set_head_proxy(k_blk)
    g = torch.Generator(device="cuda")
    g.manual_seed(14)
    u = torch.randn((ROWS, HIDDEN), device="cuda", generator=g)
    w.step = lambda: sess.head_top(ROWS, u.data_ptr(), stream.handle)
    screen = VOCAB * HIDDEN // 4 + VOCAB * (HIDDEN // 128) * 2
    if k_blk:
        chosen = min(ROWS * min(max(k_blk, 16), VOCAB // 128), VOCAB // 128)
        w.step_bytes = screen + chosen * 128 * HIDDEN * bits // 8 + ROWS * HIDDEN * 4
        w.kernel_bytes = {"proxy_q2_bmax_m%d" % (1 if ROWS == 1 else 4 if ROWS <= 4 else 8): screen}
    else:
        w.step_bytes = blob.numel() + ROWS * HIDDEN * 4 + 2 * ROWS * VOCAB * 4
        w.kernel_bytes = {"head_exl3_%d" % bits: blob.numel() + HIDDEN // 128 * 16 * 256 + ROWS * VOCAB * 4}
    w.dtype = ("int8 x 2-bit dot products (screen), then " if k_blk else "") + "f32 accumulate over EXL3 f16 codebook weights (f16 matrix cores)"
    w.describe = {"workload": "top-64 hand-off of the EXL3 lm_head 151936 x 2048 at K = %d for %d rows, to the host%s" % (
        bits, ROWS, " through the inexact 2-bit screen, %d blocks a row (at most %d of %d blocks computed exactly)" % (k_blk, chosen, VOCAB // 128)
        if k_blk else " (exact: full logits, slice sorts, merge)"), "rows": ROWS, "resident_GB": round((blob.numel() + (screen if k_blk else 0)) / 1e9, 2)}
    w.counters_key = {0: "exl3top", 128: "exl3top_screen"}.get(k_blk) if (bits == 4 and ROWS == 4) else None
    w.cpu = ("exl3_matvec", (blob, bits, u[0].cpu().numpy()))
    w.keep = (sess, blob, u)
    return w


def snapshot_states(torch, sz, stream):
    """The rollback point of a pass at the 35B model's sizes: 36 recurrent layers' states (2 MiB) and convolution windows
    (96 KiB) and one small buffer; a step takes the snapshot and restores it (two launches)."""
    w = Workload()
    bufs = []
    for _ in range(36):
        bufs += [torch.randn(32 * 128 * 128, device="cuda"), torch.randn(3 * 8192, device="cuda")]
    bufs.append(torch.randn(2048, device="cuda"))
    total = sum(b.numel() * 4 for b in bufs)
    snap = sz.Snapshot([(b.data_ptr(), b.numel() * 4) for b in bufs])
    before = [b.clone() for b in bufs]

    def step():
        snap.take(stream.handle)
        snap.restore(stream.handle)

    w.step = step
    w.step_bytes = 4 * total                                     # each direction reads and writes every byte
    w.kernel_bytes = {"copy_ranges": 2.0 * total}
    w.dtype = "u8"
    w.describe = {"workload": "snapshot + restore of %d device ranges (36 recurrent states of 2 MiB, 36 windows of 96 KiB, one of 8 KiB): "
                              "%.1f MB each way, a launch each" % (len(bufs), total / 1e6), "rows": 0, "resident_GB": round(2 * total / 1e9, 2)}
    w.extra = {"metric": "device bytes read + written a second by the snapshot's two launches"}

    def check():
        torch.cuda.synchronize()
        if not all(torch.equal(a, b) for a, b in zip(before, bufs)):
            raise RuntimeError("the restored state is not the state that was saved")

    w.check = check
    w.keep = (snap, bufs, before)
    return w


def stage_exl3_layer(torch, sz, synth, stream):
    """A config-5 layer as an EXL3 safetensors checkpoint over two files in a temporary directory (the page cache holds it); a
    step stages it into HBM in the layout the session takes."""
    import atexit
    import shutil
    import tempfile
    w = Workload()
    d = tempfile.mkdtemp(prefix="shadowzero_stage_")
    atexit.register(shutil.rmtree, d, ignore_errors=True)
    rng = np.random.default_rng(77)
    synth.exl3_checkpoint(d, rng, sz.EXL3(3), HIDDEN, FF, NE, sz.EXL3(3), scatter=False)
    st = sz.SafeTensors(d)
    L = st.layer_layout(3)
    buf = torch.empty(L.bytes, dtype=torch.uint8, device="cuda")
    file_bytes = NE * (2 * L.gate_up_bytes + L.down_bytes) + 2 * L.shared_gate_up_bytes + L.down_bytes + (NE + 1) * HIDDEN * 2
    w.step = lambda: st.stage_layer(3, buf.data_ptr(), L.bytes, stream=stream.handle)
    w.step_bytes = file_bytes
    w.kernel_bytes = {"scatter_pieces": 2.0 * (16 << 20)}       # a round of about 16 MiB read and written on the device
    w.dtype = "u8"
    w.describe = {"workload": "staging one EXL3 K=3 MoE layer (512 experts + shared, router, gate: %d projections) from a two-file safetensors "
                              "checkpoint in the page cache into HBM" % (3 * NE + 3), "rows": 0, "resident_GB": round(L.bytes / 1e9, 2)}
    w.extra = {"metric": "checkpoint layer staged into HBM, file bytes a second (reads, pinned buffers, PCIe and the scatter included)", "pcie_inclusive": True}

    def check():
        got = buf[L.experts_offset:L.experts_offset + L.gate_up_bytes].cpu().numpy()
        want = st.exl3_blob("model.language_model.layers.3.mlp.experts.0.gate_proj")
        if not np.array_equal(got, want):
            raise RuntimeError("the staged layer's first projection is not the checkpoint's")

    w.check = check
    w.keep = (st, buf)
    return w



def time_steps(w, stream, sz, torch, steps, warmup):
    """ms per step of `steps` steps after `warmup` untimed ones, events on the launch stream either side of the timed region."""
    for _ in range(warmup):
        w.step()
    stream.synchronize()
    torch.cuda.synchronize()
    e0, e1 = sz.Event(), sz.Event()
    t0 = time.perf_counter()
    e0.record(stream.handle)
    for _ in range(steps):
        w.step()
    e1.record(stream.handle)
    stream.synchronize()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return max(e1.since(e0), 0.0) / steps, wall_ms / steps


def kernel_times(w, stream, sz, reps):
    """Every kernel of the step, launch by launch, each between a start and a stop event on the launch stream that carry the
    dispatch's own begin and end time stamps (eager steps, same buffers)."""
    w.set_eager(True)
    sz.ktime_begin("")
    for _ in range(reps):
        w.step()
    stream.synchronize()
    kt = sz.ktime_end()
    w.set_eager(False)
    per_kernel = {}
    for name, (n, ms) in kt.items():
        us = ms / n * 1e3
        per_kernel[name] = {"launches_per_step": n // reps, "avg_us": us}
        if name in w.kernel_bytes:
            per_kernel[name]["bytes_per_launch"] = int(w.kernel_bytes[name])
            per_kernel[name]["GBps"] = w.kernel_bytes[name] / (us * 1e-6) / 1e9
        if name in w.kernel_ops:
            per_kernel[name]["int8_TOPs"] = w.kernel_ops[name] / (us * 1e-6) / 1e12
    return per_kernel


def roofline_of(w, per_kernel, counters, stale):
    """The dominant kernel (largest total time among those with known algorithmic bytes) against the HBM roof the metric is
    defined on and, where hardware counters of this very build are on file, against the vector-ALU roof: a SIMD issues one
    wave64 vector instruction in 4 cycles, at the shader clock the counters' run measured.  `bound` names the roof that
    the kernel is nearer to."""
    known = [k for k in per_kernel if "GBps" in per_kernel[k]]
    if not known:
        return None
    dom = max(known, key=lambda k: per_kernel[k]["avg_us"] * per_kernel[k]["launches_per_step"])
    a = per_kernel[dom]["GBps"]
    r = {"bound": "hbm", "kernel": dom, "achieved": round(a, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(a / HBM_PEAK_GBPS, 4),
         "traffic": None, "avg_launch_us": round(per_kernel[dom]["avg_us"], 2),
         "algorithmic_bytes_per_launch": int(per_kernel[dom]["bytes_per_launch"])}
    key = getattr(w, "counters_key", None)
    c = counters["workloads"].get(key, {}).get("kernels", {}).get(dom) if (counters and key and dom not in stale) else None
    if c:
        r["traffic"] = c.get("traffic_bytes")
        if c.get("SQ_INSTS_VALU") and c.get("clock_ghz"):
            peak = SIMDS * c["clock_ghz"] / 4.0                       # G wave64 vector instructions a second
            g = c["SQ_INSTS_VALU"] / (per_kernel[dom]["avg_us"] * 1e-6) / 1e9
            r["vector_alu"] = {"instructions_per_launch": int(c["SQ_INSTS_VALU"]), "achieved": round(g, 1), "peak": round(peak, 1),
                               "unit": "G wave64 instructions/s", "frac": round(g / peak, 4), "clock_ghz": c["clock_ghz"],
                               "busy_frac_in_counter_run": c.get("valu_busy_frac")}
            if g / peak > r["frac"]:
                r["bound"] = "valu"
        r["counters"] = "profiles/counters.json"
    else:
        r["counters"] = stale.get(dom, "none on file for this workload") if key else "none on file for this workload"
    if "int8_TOPs" in per_kernel[dom]:
        t = per_kernel[dom]["int8_TOPs"]
        r["mfma"] = {"achieved": round(t, 2), "peak": INT8_MFMA_PEAK_TOPS, "unit": "TOP/s", "frac": round(t / INT8_MFMA_PEAK_TOPS, 5)}
    return r


def vector_floor(w, per_kernel, counters, stale, ms_per_step):
    """The time a step's counted vector instructions would take if every one of the 1024 SIMDs issued one every 4 cycles for
    the whole step (no launch boundaries, no waits, perfectly even work): a floor for this instruction count, from the
    counters on file; None unless every kernel of the step that has algorithmic bytes has current counters."""
    key = getattr(w, "counters_key", None)
    ks = counters["workloads"].get(key, {}).get("kernels", {}) if (counters and key) else {}
    cycles, clocks, n = 0.0, [], 0
    for name, v in per_kernel.items():
        c = ks.get(name)
        if name in stale or not c or not c.get("SQ_INSTS_VALU"):
            if "bytes_per_launch" in v:
                return None
            continue
        cycles += c["SQ_INSTS_VALU"] * v["launches_per_step"] * 4.0 / SIMDS
        n += c["SQ_INSTS_VALU"] * v["launches_per_step"]
        if c.get("clock_ghz", 0) > 1.0:
            clocks.append(c["clock_ghz"])
    if not clocks:
        return None
    ghz = sum(clocks) / len(clocks)
    us = cycles / ghz / 1e3
    return {"us_per_step": round(us, 1), "frac_of_measured_step": round(us / (ms_per_step * 1e3), 4), "vector_instructions_per_step": int(n),
            "clock_ghz": round(ghz, 3), "means": "counted wave64 vector instructions of a step x 4 cycles / 1024 SIMDs / clock: the step cannot be "
            "shorter than this without issuing fewer instructions"}


def cold_run(w, stream, sz, torch, reps=15):
    """The median single-step time with 1 GiB of copy traffic on the same stream before every step (the workloads that fit
    the 256 MB Infinity Cache + L2 between steps)."""
    nwords = (512 << 20) // 16
    fsrc = torch.empty(nwords * 16, dtype=torch.uint8, device="cuda").fill_(1)
    fdst = torch.empty(nwords * 16, dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    times = []
    c0, c1 = sz.Event(), sz.Event()
    for _ in range(reps):
        sz.launch("copy_words16", (8192, 1, 1), (256, 1, 1), 0, stream.handle,
                  [sz.Arg.ptr(fsrc.data_ptr()), sz.Arg.ptr(fdst.data_ptr()), sz.Arg.u64(nwords)])
        c0.record(stream.handle)
        w.step()
        c1.record(stream.handle)
        stream.synchronize()
        times.append(c1.since(c0))
    med = float(np.median(times))
    del fsrc, fdst
    return {"median_us": round(med * 1e3, 2), "GBps": round(w.step_bytes / (med * 1e-3) / 1e9, 1), "reps": len(times),
            "flush": "1 GiB of copy traffic (512 MiB read + 512 MiB written) on the same stream before every step"}


def best_of(fn, min_reps, budget_s):
    """Best and mean seconds of fn() over at least min_reps runs after one warm-up run (crates/shadowzero-model/examples/
    cpu_expert_bench.rs:34-41 reports the best of its repeats), stopping early only when the budget is spent and 3 runs are in."""
    fn()
    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < min_reps or (len(times) < 3):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
        if time.perf_counter() > t_end and len(times) >= 3:
            break
    return min(times), sum(times) / len(times), len(times)


def cpu_baseline(kind, args, budget_s=8.0):
    """The CPU oracle (a restatement of the reference's scalar path, forward.rs:205-249 / exl3.rs:528-599 / cpu_expert.rs) on the
    host's cores, on a bounded sample of the workload: one thread and all hardware threads, best of >= 20 runs after a warm-up
    where the budget allows.  It is a baseline only."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_lib as O
    hw = int(O.lib().orc_hardware_threads())
    if kind == "exl3_token":
        (buf, stride, gap), kb, rl0, u0, sgl0 = args
        ty = O.exl3_type(kb)
        shape = O.expert_shape(ty, ty, HIDDEN, FF)
        per_expert = shape.gate_bytes + shape.up_bytes + shape.down_bytes
        ids = np.argsort(-rl0[0].astype(np.float64), kind="stable")[:TOPK]
        from shadow_engine_amd import synth_device
        host = {int(e): synth_device.expert_host(buf, stride, gap, int(e), (shape.gate_bytes, shape.up_bytes, shape.down_bytes)) for e in list(ids) + [NE]}
        experts = [host.get(e, host[int(ids[0])]) for e in range(NE)]      # only the routed ones are read
        nbytes = (TOPK + 1) * per_expert
        run = lambda t: O.moe_token(shape, experts, TOPK, rl0[0], u0[0], shape, host[NE], float(sgl0[0]), t)
        what = "one token through one layer's MoE block (top-10 + shared EXL3 K=%d experts, %d bytes each)" % (kb, per_expert)
        # exl3.rs:569-578 splits a projection over its 128-output blocks: 4 threads for gate and up (512 outputs), 16 for down
        used = min(hw, HIDDEN // 128)
        note = "a projection is split over its 128-output blocks (exl3.rs:569-578): gate and up run on 4 threads, down on %d" % used
    elif kind == "iq3_s_token":
        buf, stride, rl0, u0, sgl0 = args
        shape = O.expert_shape(O.IQ3_S, O.IQ3_S, HIDDEN, FF)
        per_expert = shape.gate_bytes + shape.up_bytes + shape.down_bytes
        ids = np.argsort(-rl0[0].astype(np.float64), kind="stable")[:TOPK]
        host = {int(e): buf[int(e) * stride:int(e) * stride + per_expert].cpu().numpy() for e in list(ids) + [NE]}
        experts = [host.get(e, host[int(ids[0])]) for e in range(NE)]
        nbytes = (TOPK + 1) * per_expert
        run = lambda t: O.moe_token(shape, experts, TOPK, rl0[0], u0[0], shape, host[NE], float(sgl0[0]), t)
        what = "one token through one layer's MoE block (top-10 + shared IQ3_S experts, %d bytes each)" % per_expert
        used, note = hw, "rows split over the threads as forward.rs:205-227"
    elif kind == "q8_0_matvec":
        mat, x, rows, cols = args
        nbytes = mat.size
        run = lambda t: O.matvec(O.Q8_0, cols, rows, mat, x, t)
        what = "the Q8_0 %d x %d matrix-vector product of the configuration (CpuBackend::matvec, forward.rs:239-249)" % (rows, cols)
        used, note = hw, "rows split over the threads as forward.rs:205-227"
    elif kind == "exl3_matvec":
        blob, bits, u0 = args
        rows = 128 * 64                                              # a bounded sample: the first 8192 rows of the vocabulary
        host = blob[:2 * HIDDEN].cpu().numpy()
        svh = blob[2 * HIDDEN:2 * HIDDEN + 2 * rows].cpu().numpy()
        tr = blob[2 * HIDDEN + 2 * VOCAB + 4:].view(HIDDEN // 16, VOCAB // 16, 32 * bits)[:, :rows // 16].contiguous().cpu().numpy()
        sample = np.concatenate([host, svh, np.array([1, 0, 0, 0], np.uint8), tr.reshape(-1)])
        nbytes = sample.size
        run = lambda t: O.exl3_matvec(HIDDEN, rows, bits, sample, u0, threads=t)
        what = "the head's first %d of %d rows for one input (exl3.rs:528-599 matvec_blob)" % (rows, VOCAB)
        used, note = min(hw, rows // 128), "one thread a 128-output block (exl3.rs:569-578)"
    elif kind == "iq3_s_int8_pairs":
        buf, stride, ids, x8 = args
        shape = O.expert_shape(O.IQ3_S, O.IQ3_S, HIDDEN, FF)
        per_expert = shape.gate_bytes + shape.up_bytes + shape.down_bytes
        pairs = [(t, int(e)) for t in range(x8.shape[0]) for e in ids[t][:2]]          # 16 (token, expert) pairs of the chunk
        host = {e: buf[e * stride:e * stride + per_expert].cpu().numpy() for _, e in pairs}
        xq = [O.quantize_act(x8[t], 32) for t in range(x8.shape[0])]
        nbytes = len(pairs) * per_expert
        run = lambda t: [O.expert_int8(host[e], HIDDEN, FF, xq[tok][0], xq[tok][1]) for tok, e in pairs]
        what = "%d (token, expert) pairs of the chunk through the int8-activation expert (cpu_expert.rs:243-339), one after the other" % len(pairs)
        used, note = 1, "the scalar int8 expert of the oracle runs on one thread"
    else:
        return None
    out = {"unit": "GB/s", "kind": "port", "bytes_per_run": int(nbytes)}
    modes = [("one_thread", 1)] + ([("all_threads", 0)] if used > 1 else [])
    for label, t in modes:
        best, mean, n = best_of(lambda: run(t), 20, budget_s / len(modes))
        out[label] = {"value": round(nbytes / best / 1e9, 3), "best_us": round(best * 1e6, 1), "mean_us": round(mean * 1e6, 1), "runs": n,
                      "threads": 1 if t == 1 else used}
    top = out.get("all_threads", out["one_thread"])
    out["value"], out["cores"] = top["value"], top["threads"]
    out["sample"] = "%s with the C++ oracle, best of %d runs after a warm-up; %s (%d hardware threads on the box)" % (what, top["runs"], note, hw)
    return out


def build_workload(name, torch, sz, synth, synth_device, stream, args):
    if name == "config5":
        return exl3_round(torch, sz, synth, synth_device, stream, args.layers, synth_device.layer_rates(2026, args.layers), "config 5", args.expert_mode)
    if name == "config3":
        return exl3_round(torch, sz, synth, synth_device, stream, 1, [3], "config 3", args.expert_mode)
    if name == "config1":
        return q8_matvec(torch, sz, synth, synth_device, stream)
    if name == "config2":
        return iq3s_decode(torch, sz, synth, synth_device, stream)
    if name == "config4":
        return iq3s_prefill(torch, sz, synth, synth_device, stream, args.tokens)
    if name == "exl3prefill":
        return exl3_prefill(torch, sz, synth, synth_device, stream, args.tokens, args.bits or 3)
    if name == "exl3head":
        return exl3_head(torch, sz, synth, synth_device, stream, args.bits or 4)
    if name == "exl3top":
        return exl3_head_top(torch, sz, synth, synth_device, stream, args.bits or 4, args.screen)
    if name == "stage":
        return stage_exl3_layer(torch, sz, synth, stream)
    return snapshot_states(torch, sz, stream)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--layers", type=int, default=48)
    ap.add_argument("--workload", default="config5", choices=["config1", "config2", "config3", "config4", "config5", "exl3prefill", "exl3head", "exl3top", "stage", "snapshot"])
    ap.add_argument("--rows", type=int, default=4, help="rows of the verify batch (config3, config5, exl3head; the configurations name 4; 1..8)")
    ap.add_argument("--tokens", type=int, default=512, help="tokens of the prefill chunk (config4, exl3prefill; the configuration names 512)")
    ap.add_argument("--bits", type=int, default=0, help="bits a weight of the EXL3 head (exl3head, exl3top: 4 unless given) or of the chunk's experts (exl3prefill: 3)")
    ap.add_argument("--expert-mode", type=int, default=0, choices=[0, 1, 2, 3],
                    help="config3, config5: 0 the exact EXL3 expert kernels (the library's default), 1 the matrix-core launches with the codebook's f16 values, "
                         "2 with the linearised codebook, 3 the exact launches with their inputs rounded to f16 (two products an instruction)")
    ap.add_argument("--screen", type=int, default=0, help="exl3top: blocks a row of the inexact 2-bit screen (0: the exact hand-off)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true", help="default workload only: do not time configurations 1-4 after it")
    ap.add_argument("--contiguous-experts", action="store_true",
                    help="EXL3 experts as the reference keeps them, [gate|up|down] back to back, instead of the stager's layout with every "
                         "trellis on a 128-byte line (config3, config5, exl3prefill)")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="BYTES",
                    help="also launch one plain copy of BYTES bytes, for scaling a profile's memory counters")
    args = ap.parse_args()
    global SPACED
    SPACED = not args.contiguous_experts
    if args.gpus != 1:
        print("bench.py: this build runs the verify path on ONE GPU (all experts resident in one MI355X's HBM); "
              "--gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    global ROWS
    if not 1 <= args.rows <= 8 or (args.rows == 1 and args.workload in ("config3", "config5")):
        print("bench.py: --rows takes 2..8 (1..8 for exl3head)", file=sys.stderr)
        sys.exit(2)
    ROWS = args.rows

    import torch

    import shadow_engine_amd as sz
    from shadow_engine_amd import synth, synth_device

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    sz.init(0)
    stream = sz.Stream()
    w = build_workload(args.workload, torch, sz, synth, synth_device, stream, args)
    torch.cuda.synchronize()

    ms_per_step, wall_ms = time_steps(w, stream, sz, torch, args.steps, args.warmup)
    w.check()
    gbps = w.step_bytes / (ms_per_step * 1e-3) / 1e9
    per_kernel = kernel_times(w, stream, sz, max(2, min(args.steps, 5)))
    counters, stale = load_counters(sz)
    roofline = roofline_of(w, per_kernel, counters, stale)
    cold = cold_run(w, stream, sz, torch) if w.cold_variant else None

    if args.copy_calibration:
        nwords = args.copy_calibration // 16
        src = torch.empty(nwords * 16, dtype=torch.uint8, device="cuda").fill_(3)
        dst = torch.empty(nwords * 16, dtype=torch.uint8, device="cuda")
        torch.cuda.synchronize()
        sz.launch("copy_words16", (8192, 1, 1), (256, 1, 1), 0, stream.handle,
                  [sz.Arg.ptr(src.data_ptr()), sz.Arg.ptr(dst.data_ptr()), sz.Arg.u64(nwords)])
        stream.synchronize()
        del src, dst

    cpu = None
    if not args.no_cpu_baseline and hasattr(w, "cpu"):
        cpu = cpu_baseline(*w.cpu)

    # the other configurations of the path, once each after the timed region of the default one (they are parity-test cases
    # first): time, algorithmic GB/s against 8 TB/s, warm and cold, their dominant kernel, and the CPU oracle beside each
    others = None
    if args.workload == "config5" and args.layers == 48 and ROWS == 4 and not args.no_other_configs:
        others = {}
        for name in ("config1", "config2", "config3", "config4", "exl3prefill"):   # the last: config 4's chunk through the round's kind of experts
            ow = build_workload(name, torch, sz, synth, synth_device, stream, args)
            torch.cuda.synchronize()
            oms, _ = time_steps(ow, stream, sz, torch, 30, 3)
            ow.check()
            opk = kernel_times(ow, stream, sz, 3)
            og = ow.step_bytes / (oms * 1e-3) / 1e9
            entry = {"workload": ow.describe["workload"], "us_per_step": round(oms * 1e3, 2), "GBps": round(og, 1),
                     "frac_of_8TBps": round(og / HBM_PEAK_GBPS, 4), "algorithmic_bytes_per_step": int(ow.step_bytes),
                     "roofline": roofline_of(ow, opk, counters, stale),
                     "cold_cache": cold_run(ow, stream, sz, torch, 9) if ow.cold_variant else None}
            if name == "config2":
                entry["us_per_layer"] = round(oms * 1e3 / ow.describe["layers"], 2)
            if not args.no_cpu_baseline and hasattr(ow, "cpu"):
                entry["cpu_baseline"] = cpu_baseline(*ow.cpu, budget_s=2.0)
            others[name] = entry
            del ow
            torch.cuda.empty_cache()

    line = {
        "metric": "MoE quant-matvec HBM GB/s (% of 8 TB/s); K=3 spec-verify round µs",
        "value": round(gbps, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": w.dtype, "data": "synthetic", "config": w.describe,
        "round_us": round(ms_per_step * 1e3, 1), "pct_of_8TBps": round(100 * gbps / HBM_PEAK_GBPS, 2),
        "algorithmic_bytes_per_step": int(w.step_bytes), "host_wall_ms_per_step": round(wall_ms, 4),
        "roofline": roofline, "vector_alu_floor": vector_floor(w, per_kernel, counters, stale, ms_per_step), "kernels": {k: {kk: (round(vv, 2) if isinstance(vv, float) else vv) for kk, vv in v.items()} for k, v in per_kernel.items()},
        "cpu_baseline": cpu, "cold_cache": cold,
    }
    if others is not None:
        line["other_configs"] = others
    line.update(w.extra)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
