"""Seeded synthetic MoE layers for the parity tests and the benchmark: weights N(0, sigma) quantised by the oracle's
encoders into GGUF blocks, router weights and activations as the benchmark's five configurations describe them. numpy only."""
import numpy as np

import oracle

CONFIGS = {
    # name: hidden, ff, experts, topk, shared_ff, bank format, router / activation storage
    "c1": dict(hidden=2048, ff=768, experts=64, topk=8, shared_ff=0, wtype=oracle.Q4_K, rtype="f32", xtype="f32"),
    "c2": dict(hidden=2048, ff=512, experts=512, topk=10, shared_ff=512, wtype=oracle.IQ4_XS, rtype="bf16", xtype="bf16"),
    "c4": dict(hidden=2048, ff=768, experts=256, topk=8, shared_ff=0, wtype=oracle.IQ3_S, rtype="bf16", xtype="bf16"),
    "c5": dict(hidden=3072, ff=1536, experts=256, topk=8, shared_ff=1536, wtype=oracle.NVFP4G, rtype="bf16", xtype="bf16"),
}


# formats the oracle has no encoder for: offset of the fp16 block scale and the range it is drawn from (weights of about 0.02)
RANDOM_BLOCKS = {oracle.IQ3_XXS: [(0, 1.5e-4, 4e-4)], oracle.IQ2_S: [(0, 4e-4, 1e-3)], oracle.Q4_0: [(0, 2e-3, 6e-3)], oracle.Q3_K: [(108, 3e-4, 7e-4)],
                 oracle.IQ2_XXS: [(0, 2e-4, 5e-4)], oracle.IQ2_XS: [(0, 2e-4, 5e-4)], oracle.Q2_K: [(80, 1e-3, 3e-3), (82, 1.5e-3, 4.5e-3)],
                 oracle.IQ1_S: [(0, 2e-3, 4e-3)]}
# byte offset of the fp16 block scale where it is not the block's first field
SCALE_OFFSET = {oracle.Q6_K: 208, oracle.Q3_K: 108, oracle.Q2_K: 80}


def bank_blocks(wtype, rows, cols, rng, sigma=0.02):
    """GGUF blocks of a [rows][cols] matrix with weights of about `sigma`: encoded N(0, sigma) values, or, for a format the
    oracle has no encoder for, random valid blocks with block scales that give weights of that size."""
    if wtype in RANDOM_BLOCKS:
        el, nbytes = oracle.BLOCK[wtype]
        blocks = rng.integers(0, 256, (rows * cols // el, nbytes), dtype=np.uint8)
        for off, lo, hi in RANDOM_BLOCKS[wtype]:
            dd = np.float16(rng.uniform(lo, hi, len(blocks)) * (sigma / 0.02) * rng.choice([-1, 1], len(blocks)))
            blocks[:, off:off + 2] = dd.view(np.uint8).reshape(-1, 2)
        return blocks.reshape(-1)
    return oracle.quantize(wtype, (rng.standard_normal((rows, cols)) * sigma).astype(np.float32))


def small(cfg, hidden, ff, experts, topk=None):
    c = dict(cfg)
    c.update(hidden=hidden, ff=ff, experts=experts, topk=min(topk or cfg["topk"], experts))
    if c["shared_ff"]:
        c["shared_ff"] = ff
    return c


def _scale_field(raw, wtype, per_expert_blocks, factors):
    """Multiplies the block scale of every block of expert e by factors[e] so that tiled experts differ."""
    elems, nbytes = oracle.BLOCK[wtype]
    blocks = raw.reshape(len(factors), per_expert_blocks, nbytes)
    if wtype == oracle.NVFP4G:
        g = blocks[:, :, 0:4].copy().view(np.float32)
        blocks[:, :, 0:4] = (g * factors[:, None, None].astype(np.float32)).view(np.uint8)
    else:
        o = SCALE_OFFSET.get(wtype, 0)
        d = blocks[:, :, o:o + 2].copy().view(np.float16).astype(np.float32)
        blocks[:, :, o:o + 2] = (d * factors[:, None, None]).astype(np.float16).view(np.uint8)
        if wtype in (oracle.Q4_K, oracle.Q5_K, oracle.Q2_K):       # the minimums' scale follows the block scale
            m = blocks[:, :, o + 2:o + 4].copy().view(np.float16).astype(np.float32)
            blocks[:, :, o + 2:o + 4] = (m * factors[:, None, None]).astype(np.float16).view(np.uint8)
    return blocks.reshape(-1)


def make_banks(cfg, seed, distinct=None, sigma=0.02):
    """gate, up, down GGUF block streams (uint8) of experts (+1 shared) stacked matrices. `distinct` experts are really
    quantised; the rest repeat them with an expert-specific factor on the block scales (cheap, still all different)."""
    h, f, e = cfg["hidden"], cfg["ff"], cfg["experts"] + (1 if cfg["shared_ff"] else 0)
    d = min(distinct or e, e)
    rng = np.random.default_rng(seed)
    banks = []
    for rows, cols in ((f, h), (f, h), (h, f)):
        raw = bank_blocks(cfg["wtype"], d * rows, cols, rng, sigma)
        per = raw.size // d
        if d < e:
            raw = np.tile(raw, (e + d - 1) // d)[: per * e].copy()
            factors = 1.0 + 0.25 * (np.arange(e) // d) / max(1, (e - 1) // d)       # up to 1.25: all different, magnitudes as configured
            raw = _scale_field(raw, cfg["wtype"], per // oracle.BLOCK[cfg["wtype"]][1], factors)
        banks.append(raw)
    return banks


def make_inputs(cfg, n, seed, zipf=None):
    """router [E][H], shared gate [H], x [n][H] as (storage array, fp32 values).
    zipf: router logits become N(0, 1) plus a per-expert bias ln p_e of a Zipf(s = zipf) popularity over a seeded
    permutation of the experts (skewed expert load): router rows are N(0, 1 / H), their last column holds the bias and
    the last activation of every token is 1."""
    h, e = cfg["hidden"], cfg["experts"]
    rng = np.random.default_rng(seed)
    router = (rng.standard_normal((e, h)) * (0.02 if not zipf else h ** -0.5)).astype(np.float32)
    gate = (rng.standard_normal(h) * 0.02).astype(np.float32)
    x = rng.standard_normal((n, h)).astype(np.float32)
    if zipf:
        p = 1.0 / np.arange(1, e + 1) ** zipf
        p /= p.sum()
        router[:, -1] = np.log(p[rng.permutation(e)])
        x[:, -1] = 1.0
    out = {}
    for name, a, kind in (("router", router, cfg["rtype"]), ("shared_gate", gate, cfg["rtype"]), ("x", x, cfg["xtype"])):
        if kind == "bf16":
            bits, vals = oracle.to_bf16(a)
            out[name] = (bits, vals)
        else:
            out[name] = (a, a)
    return out


def errors(got, want):
    """(max abs error, rms error / rms of the reference) over the whole output."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return float(np.abs(got - want).max()), float(np.sqrt(np.mean((got - want) ** 2) / np.mean(want ** 2)))
