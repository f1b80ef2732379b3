"""Device-side synthetic weights at the full shapes of the verify round: layers of 512 EXL3 experts plus a shared expert,
generated with torch straight into HBM (29 GB does not go through the host), and a Q8_0 head.  torch is plumbing here:
it owns the device memory and makes the random bytes; nothing in the timed path touches it.

The byte distributions are those of shadow_engine_amd.synth (random trellis words, suh = +-1, svh = 0.3 + U[0,1) as f16,
Q8_0 codes uniform in [-127, 127] with f16 scales |N(0, 0.02)| / 127), seeded per layer.
"""
import numpy as np

from . import synth


def exl3_layer(torch, seed, hidden, ff, ne, bits, spaced=False):
    """(buffer uint8[(ne + 1) * stride], stride): experts 0..ne-1 and the shared expert as [gate|up|down] blobs.
    spaced: the layout sz_layer_spacing describes instead, every projection's trellis on a 128-byte line of memory - the
    buffer returned starts at the first expert, an expert's projections lie `gap` bytes apart: (buffer, stride, gap)."""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    gb, ub, db = synth.expert_bytes(synth.exl3_type(bits), hidden, ff)
    lead = gap = 0
    if spaced:
        import shadow_engine_amd as sz
        lead, gap = sz.layer_spacing(sz.EXL3(bits), hidden, ff)
    stride = (gb + ub + db + 2 * gap + 255) // 256 * 256
    n = ne + 1
    if spaced:
        full = torch.randint(0, 256, (lead + n * stride,), dtype=torch.uint8, device="cuda", generator=g)
        assert full.data_ptr() % 256 == 0
        buf = full[lead:].view(n, stride)
    else:
        buf = torch.randint(0, 256, (n, stride), dtype=torch.uint8, device="cuda", generator=g)
    off = 0
    for inf, outf, nbytes in ((hidden, ff, gb), (hidden, ff, ub), (ff, hidden, db)):
        sign = torch.randint(0, 2, (n, inf), device="cuda", generator=g)
        suh = torch.where(sign == 0, 0x3C00, 0xBC00).to(torch.int16)                       # +1.0 / -1.0 as f16 bits
        svh = (0.3 + torch.randint(0, 100, (n, outf), device="cuda", generator=g).float() / 100.0).half()
        buf[:, off:off + 2 * inf] = suh.view(torch.uint8).reshape(n, 2 * inf)
        buf[:, off + 2 * inf:off + 2 * inf + 2 * outf] = svh.view(torch.uint8).reshape(n, 2 * outf)
        buf[:, off + 2 * inf + 2 * outf:off + 2 * inf + 2 * outf + 4] = torch.tensor([1, 0, 0, 0], dtype=torch.uint8, device="cuda")
        off += nbytes + gap
    return (buf.reshape(-1), stride, gap) if spaced else (buf.reshape(-1), stride)


def expert_host(buf, stride, gap, e, sizes):
    """Expert e of a layer buffer as the contiguous [gate|up|down] bytes on the host (sizes: the three projections' bytes)."""
    import numpy as np
    at, parts = e * stride, []
    for n in sizes:
        parts.append(buf[at:at + n].cpu().numpy())
        at += n + gap
    return np.concatenate(parts)


def exl3_matrix(torch, seed, inf, outf, bits):
    """uint8[exl3_blob_len]: one EXL3 projection (the lm_head's shape when outf is the vocabulary): random trellis words,
    suh = +-1, svh = 0.3 + U[0,1)."""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    n = synth.exl3_blob_len(inf, outf, bits)
    buf = torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda", generator=g)
    sign = torch.randint(0, 2, (inf,), device="cuda", generator=g)
    suh = torch.where(sign == 0, 0x3C00, 0xBC00).to(torch.int16)
    svh = (0.3 + torch.randint(0, 100, (outf,), device="cuda", generator=g).float() / 100.0).half()
    buf[:2 * inf] = suh.view(torch.uint8)
    buf[2 * inf:2 * inf + 2 * outf] = svh.view(torch.uint8)
    buf[2 * inf + 2 * outf:2 * inf + 2 * outf + 4] = torch.tensor([1, 0, 0, 0], dtype=torch.uint8, device="cuda")
    return buf


def q8_0_head(torch, seed, vocab, hidden):
    """uint8[vocab * hidden / 32 * 34]: the head as Q8_0 rows."""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    nb = vocab * hidden // 32
    buf = torch.empty((nb, 34), dtype=torch.uint8, device="cuda")
    d = (torch.randn(nb, device="cuda", generator=g).abs() * (0.02 / 127.0)).half()
    buf[:, 0:2] = d.view(torch.uint8).reshape(nb, 2)
    q = torch.randint(-127, 128, (nb, 32), dtype=torch.int8, device="cuda", generator=g)
    buf[:, 2:] = q.view(torch.uint8)
    return buf.reshape(-1)


def layer_rates(seed, n_layers, choices=(2, 3, 4)):
    """The seeded per-layer bit rates of the mixed-rate model: as many layers of each rate as divide evenly, shuffled."""
    rng = np.random.default_rng(seed)
    rates = [choices[i % len(choices)] for i in range(n_layers)]
    return [int(r) for r in rng.permutation(rates)]


def route_ids(logits, k):
    """Top-k expert ids per row by (logit descending, index ascending): the router's selection (forward.rs:1088) whenever
    the f64 exponentials of distinct logits are distinct."""
    order = np.lexsort((np.broadcast_to(np.arange(logits.shape[1]), logits.shape), -logits.astype(np.float64)), axis=1)
    return order[:, :k]


def iq3_s_layer(torch, seed, hidden, ff, ne):
    """(buffer uint8[(ne + 1) * stride], stride): experts 0..ne-1 and the shared expert as [gate|up|down] IQ3_S rows: random
    grid indices, signs and sub-block scales, block scale d a small positive normal f16 (as synth.iq3_s_matrix)."""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    gb, ub, db = synth.expert_bytes(21, hidden, ff)
    per = gb + ub + db
    stride = (per + 255) // 256 * 256
    n = ne + 1
    buf = torch.zeros((n, stride), dtype=torch.uint8, device="cuda")
    nb = per // 110
    blocks = torch.randint(0, 256, (n, nb, 110), dtype=torch.uint8, device="cuda", generator=g)
    d = (torch.randn((n, nb), device="cuda", generator=g).abs() * 2e-4 + 1e-4).half()
    blocks[:, :, 0:2] = d.view(torch.uint8).reshape(n, nb, 2)
    buf[:, :per] = blocks.reshape(n, per)
    return buf.reshape(-1), stride
