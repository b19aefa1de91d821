"""GPU parity, through the C ABI: bank decode bit-exact against the oracle's decoders; grouped expert products against
float64 on the decoded weights; the whole layer against the oracle's fp32 layer at the tolerance the target states
(max-abs 1e-2, rel-RMS 1e-3), with routing ids bit-exact on the device's own logits."""
import numpy as np
import pytest
import torch

import synth
from gpu_util import banks_on_device, clear_tokens, clear_tokens_gated, dev, oracle_mode

pytestmark = pytest.mark.gpu

MAX_ABS, REL_RMS = 1e-2, 1e-3


@pytest.fixture(scope="module")
def tq():
    import tqllm_amd
    return tqllm_amd


@pytest.mark.parametrize("wtype", [12, 21, 23, 323, 20, 8, 13, 14, 18, 22, 2, 11, 16, 17, 10, 19])
def test_bank_decode_bit_exact(tq, oracle, wtype):
    rng = np.random.default_rng(wtype)
    experts, rows, cols = 3, (64 if wtype == 23 else 40), 1024      # IQ4_XS banks are tiled by 32 rows
    el, bb = oracle.BLOCK[wtype]
    nb = experts * rows * cols // el
    # random block bytes with sane scale fields, as the reference's device tests make them (tests/moe_device.cu:121-138)
    raw = rng.integers(0, 256, (nb, bb), dtype=np.uint8)
    for off in {12: [0, 2], 21: [0], 23: [0], 20: [0], 8: [0], 13: [0, 2], 14: [208], 18: [0], 22: [0], 2: [0], 11: [108], 16: [0], 17: [0], 10: [80, 82], 19: [0]}.get(wtype, []):
        raw[:, off:off + 2] = np.float16(rng.uniform(1e-3, 5e-2, nb) * rng.choice([-1, 1], nb)).view(np.uint8).reshape(nb, 2)
    if wtype == 323:
        g = rng.uniform(1e-3, 2e-2, experts * rows).astype(np.float32)
        raw[:, 0:4] = np.repeat(g, cols // 128).view(np.uint8).reshape(nb, 4)
        raw[:, 4:12] &= 0x7E
    bank = tq.ExpertBank(wtype, raw.reshape(-1), experts, rows, cols)
    got = bank.dequant().cpu().numpy()
    want = oracle.dequantize(wtype, raw, experts * rows * cols).reshape(experts * rows, cols)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    part = bank.dequant(37, 11).cpu().numpy()
    assert np.array_equal(part, want[37:48])


def test_nvfp4_rows_with_two_globals_are_rejected(tq, oracle):
    rng = np.random.default_rng(1)
    raw = rng.integers(0, 256, (8, 76), dtype=np.uint8)
    raw[:, 4:12] &= 0x7E
    raw[:, 0:4] = np.float32(0.01).reshape(1).view(np.uint8)
    raw[3, 0:4] = np.float32(0.02).reshape(1).view(np.uint8)
    with pytest.raises(tq.TqmoeError):
        tq.ExpertBank(323, raw.reshape(-1), 1, 4, 256)       # row 1 (blocks 2, 3) disagrees


@pytest.mark.parametrize("name,rows,cols", [("c2", 512, 2048), ("c2", 2048, 512), ("c1", 768, 2048), ("c1", 2048, 768),
                                             ("c4", 768, 2048), ("c4", 2048, 768), ("c5", 1536, 3072), ("c5", 3072, 1536)])
def test_expert_matvec_against_float64(tq, oracle, name, rows, cols):
    cfg = synth.CONFIGS[name]
    wtype = cfg["wtype"]
    rng = np.random.default_rng(rows + cols)
    experts, n, k = 6, 3, 2
    w = (rng.standard_normal((experts * rows, cols)) * 0.02).astype(np.float32)
    raw = oracle.quantize(wtype, w)
    bank = tq.ExpertBank(wtype, raw, experts, rows, cols)
    dec = oracle.dequantize(wtype, raw, w.size).reshape(experts, rows, cols).astype(np.float64)
    xb, xv = oracle.to_bf16(rng.standard_normal((n, cols)).astype(np.float32))
    x = torch.from_numpy(xb.view(np.int16)).cuda().view(torch.bfloat16)
    ids = rng.integers(0, experts, (n, k)).astype(np.int32)
    ids[1, 1] = -1                                   # skipped: row stays as allocated
    y = tq.expert_matvec(bank, tq.quant_act(x), dev(ids)).cpu().numpy()
    for a in range(n * k):
        e = ids.reshape(-1)[a]
        if e < 0:
            assert not y[a].any()
            continue
        want = dec[e] @ xv[a // k].astype(np.float64)
        mx, rel = synth.errors(y[a], want)
        assert rel < 2e-4 and mx < 1e-3, (a, mx, rel)
    # per-expert input rows, bf16 output
    xe_b, xe_v = oracle.to_bf16(rng.standard_normal((n * k, cols)).astype(np.float32))
    xe = torch.from_numpy(xe_b.view(np.int16)).cuda().view(torch.bfloat16)
    y = tq.expert_matvec(bank, tq.quant_act(xe), dev(ids), per_expert_input=True, out_type=tq.BF16).float().cpu().numpy()
    for a in range(n * k):
        e = ids.reshape(-1)[a]
        if e >= 0:
            want = dec[e] @ xe_v[a].astype(np.float64)
            assert synth.errors(y[a], want)[1] < 4e-3      # bf16 output rounding


def test_matvec2_swiglu_combine_modular_path(tq, oracle):
    """The reference's step-by-step sequence (qwen35_forward.cpp:1229-1248) through the modular entry points equals the
    fused layer call."""
    cfg = synth.small(synth.CONFIGS["c2"], 512, 256, 12, 3)
    raws = synth.make_banks(cfg, seed=3)
    gate, up, down = banks_on_device(cfg, raws)
    n = 5
    inp = synth.make_inputs(cfg, n, seed=4)
    x = dev(inp["x"])
    logits = tq.moe_router(dev(inp["router"]), dev(inp["shared_gate"]), x)
    ids, w, sw = tq.moe_topk(logits, cfg["experts"], cfg["topk"])
    img = tq.quant_act(x)
    g, u = tq.expert_matvec2(gate, up, img, ids)
    g1 = tq.expert_matvec(gate, img, ids)
    assert torch.equal(g, g1)                                  # paired == two calls (tests/moe_device.cu:222-268)
    act = tq.moe_swiglu(g, u)
    routed = tq.expert_matvec(down, tq.quant_act(act), ids, per_expert_input=True)
    sid = torch.full((n, 1), cfg["experts"], dtype=torch.int32, device="cuda")
    sg, su = tq.expert_matvec2(gate, up, img, sid)
    shared = tq.expert_matvec(down, tq.quant_act(tq.moe_swiglu(sg, su)), sid, per_expert_input=True)
    out = tq.moe_combine(routed, shared, w, sw)
    layer = tq.MoeLayer(dev(inp["router"]), dev(inp["shared_gate"]), gate, up, down, cfg["topk"], shared_ff=cfg["shared_ff"])
    fused, fids, fw, flog = layer.forward(x, return_routing=True)
    assert torch.equal(fids, ids) and torch.equal(fw, w) and torch.equal(flog, logits)
    # the fused call quantises the intermediate rows per 32 values, the step-by-step one per row: both 2^-14 of a maximum
    assert torch.allclose(fused, out, rtol=0, atol=5e-5)
    gref = g.double().cpu().numpy()
    want = gref / (1 + np.exp(-gref)) * u.double().cpu().numpy()
    assert np.abs(act.cpu().numpy() - want).max() < 1e-5


def run_layer(tq, oracle, cfg, n, seed, distinct=None):
    raws = synth.make_banks(cfg, seed=seed, distinct=distinct)
    gate, up, down = banks_on_device(cfg, raws)
    inp = synth.make_inputs(cfg, n, seed=seed + 1)
    layer = tq.MoeLayer(dev(inp["router"]), dev(inp["shared_gate"]) if cfg["shared_ff"] else None, gate, up, down, cfg["topk"],
                        shared_ff=cfg["shared_ff"])
    out, ids, w, logits = (t.cpu().numpy() for t in layer.forward(dev(inp["x"]), return_routing=True))
    want, want_ids, want_w = oracle.layer_forward(inp["x"][1], logits, *raws, cfg["wtype"], cfg["hidden"], cfg["ff"], cfg["experts"],
                                                  cfg["topk"], shared_ff=cfg["shared_ff"], act_mode=oracle_mode(layer, n), threads=16)
    clear = clear_tokens(oracle, logits, cfg["experts"], cfg["topk"], ids, want_ids)
    return out, ids, w, want, want_ids, want_w, clear


def check_layer(out, ids, w, want, want_ids, want_w, clear):
    out, ids, w, want, want_ids, want_w = out[clear], ids[clear], w[clear], want[clear], want_ids[clear], want_w[clear]
    assert np.array_equal(ids, want_ids)
    assert np.abs(w - want_w).max() < 3e-6
    mx, rel = synth.errors(out, want)
    # max-abs 1e-2 where the outputs are of order one, as the configurations' are; relative to the largest value beyond that
    # (banks of random valid blocks can give larger outputs, and on the 8-bit grouped products one act value that rounds the
    # other way is a step of 1 / 127 of its row's largest)
    top = float(np.abs(want).max())
    print("layer, %d tokens: max-abs %.3g (largest value %.3g, bar %.3g) rel-rms %.3g" % (len(out), mx, top, MAX_ABS * max(1.0, top), rel))
    assert mx < MAX_ABS * max(1.0, top) and rel < REL_RMS, (mx, rel, top)
    return mx, rel


@pytest.mark.parametrize("name", ["c1", "c2", "c4", "c5"])
@pytest.mark.parametrize("n", [1, 5])
def test_layer_small_shapes(tq, oracle, name, n):
    base = synth.CONFIGS[name]
    cfg = synth.small(base, 768 if name != "c5" else 384, 512 if name != "c5" else 256, 10, 3)
    check_layer(*run_layer(tq, oracle, cfg, n, seed=50 + n))


@pytest.mark.parametrize("wtype", [20, 8, 13, 14, 18, 22, 2, 11, 16, 17, 10, 19])
@pytest.mark.parametrize("n", [1, 5, 300])
def test_layer_further_bank_formats(tq, oracle, wtype, n):
    """IQ4_NL (the CPU bench's format), Q8_0, Q5_K, Q6_K, IQ3_XXS and IQ2_S through the same decode kernels and grouped
    GEMM as the others, with a shared expert."""
    cfg = dict(hidden=768, ff=512, experts=10, topk=3, shared_ff=256, wtype=wtype, rtype="bf16", xtype="bf16")
    check_layer(*run_layer(tq, oracle, cfg, n, seed=90 + n + wtype))


@pytest.mark.parametrize("gu_type,down_type", [(12, 14), (23, 14), (13, 8)])
@pytest.mark.parametrize("n", [4, 300])
def test_layer_down_bank_of_another_format(tq, oracle, gu_type, down_type, n):
    """Mixed checkpoints (the K-quant mixes keep ffn_down_exps in a wider format than gate / up): the down bank may have a
    format of its own, on the decode kernels and on the grouped GEMM."""
    cfg = dict(hidden=768, ff=512, experts=10, topk=3, shared_ff=256, wtype=gu_type, rtype="bf16", xtype="bf16")
    raws = synth.make_banks(cfg, seed=120 + n)
    raws[2] = synth.make_banks(dict(cfg, wtype=down_type), seed=121 + n)[2]
    e = cfg["experts"] + 1
    gate, up = (tq.ExpertBank(gu_type, r, e, cfg["ff"], cfg["hidden"]) for r in raws[:2])
    down = tq.ExpertBank(down_type, raws[2], e, cfg["hidden"], cfg["ff"])
    inp = synth.make_inputs(cfg, n, seed=122 + n)
    layer = tq.MoeLayer(dev(inp["router"]), dev(inp["shared_gate"]), gate, up, down, cfg["topk"], shared_ff=cfg["shared_ff"])
    out, ids, w, logits = (t.cpu().numpy() for t in layer.forward(dev(inp["x"]), return_routing=True))
    want, want_ids, want_w = oracle.layer_forward(inp["x"][1], logits, *raws, gu_type, cfg["hidden"], cfg["ff"], cfg["experts"], cfg["topk"],
                                                  shared_ff=cfg["shared_ff"], act_mode=oracle_mode(layer, n), threads=16, wtype_down=down_type)
    check_layer(out, ids, w, want, want_ids, want_w, clear_tokens(oracle, logits, cfg["experts"], cfg["topk"], ids, want_ids))


@pytest.mark.parametrize("n", [1, 4, 16])
def test_layer_config2_full_shape(tq, oracle, n):
    """Flash-Next-shaped decode layer at its real shape: 512 IQ4_XS experts + shared, top-10, bf16 router and inputs."""
    check_layer(*run_layer(tq, oracle, synth.CONFIGS["c2"], n, seed=200 + n, distinct=20))


@pytest.mark.parametrize("n", [1, 16])
def test_layer_config1_full_shape(tq, oracle, n):
    """CPU-reference config: 64 Q4_K experts, top-8, fp32 router and activations."""
    check_layer(*run_layer(tq, oracle, synth.CONFIGS["c1"], n, seed=300 + n, distinct=16))


def test_layer_config4_and_5_full_shape_one_token(tq, oracle):
    check_layer(*run_layer(tq, oracle, synth.CONFIGS["c4"], 1, seed=400, distinct=8))
    check_layer(*run_layer(tq, oracle, synth.CONFIGS["c5"], 2, seed=500, distinct=4))


@pytest.mark.parametrize("n", [64, 512])
def test_layer_config4_crossover_token_counts(tq, oracle, n):
    """IQ3_S bank at 64 and 512 tokens (more assignments than the per-expert de-duplication handles at 512)."""
    check_layer(*run_layer(tq, oracle, synth.CONFIGS["c4"], n, seed=430 + n, distinct=8))


@pytest.mark.parametrize("gating,norm,biased,scale", [(2, True, True, 2.5), (2, False, False, 1.0), (4, True, True, 1.0), (3, False, True, 1.0), (1, False, True, 0.5)])
@pytest.mark.parametrize("n", [5, 800])
def test_layer_other_routing_modes(tq, oracle, gating, norm, biased, scale, n):
    """Sigmoid / sqrt-softplus / selected-softmax gating, a selection bias, raw weights and a weight scale through the
    whole layer (moe_route's modes, src/experts/moe.cpp:22-113), on the decode kernels (5 tokens) and the grouped GEMM."""
    cfg = synth.small(synth.CONFIGS["c1"], 768, 512, 10, 3)
    raws = synth.make_banks(cfg, seed=61)
    gate, up, down = banks_on_device(cfg, raws)
    inp = synth.make_inputs(cfg, n, seed=62)
    e, k = cfg["experts"], cfg["topk"]
    bias = np.random.default_rng(63).uniform(-0.5, 0.5, e).astype(np.float32) if biased else None
    layer = tq.MoeLayer(dev(inp["router"]), None, gate, up, down, k, shared_ff=0, weight_scale=scale,
                        gating=gating, probs_bias=dev(bias) if biased else None, norm_weights=norm)
    out, ids, w, logits = (t.cpu().numpy() for t in layer.forward(dev(inp["x"]), return_routing=True))
    want, want_ids, want_w = oracle.layer_forward(inp["x"][1], logits, *raws, cfg["wtype"], cfg["hidden"], cfg["ff"], e, k, shared_ff=cfg["shared_ff"],
                                                  act_mode=oracle_mode(layer, n), threads=16, gating=gating, norm=norm, scale=scale, bias=bias)
    # ids bit-exact on every token whose selection values are not within fp32 rounding of each other (counted and printed)
    clear = clear_tokens_gated(logits, e, k, gating, bias, ids, want_ids, "%d tokens" % n)
    assert np.array_equal(ids[clear], want_ids[clear])
    same = (ids == want_ids).all(axis=1)
    assert np.abs(w[same] - want_w[same]).max() < 4e-6 * max(1.0, float(np.abs(want_w).max()))
    mx, rel = synth.errors(out[same], want[same])
    assert mx < MAX_ABS * max(1.0, float(np.abs(want_w).sum(axis=1).max())) and rel < REL_RMS, (mx, rel)


def test_layer_linearity_and_bf16_output(tq, oracle):
    """One expert, normalised weight 1: the layer equals that expert's FFN (tests/moe.cpp:354-392); bf16 output is the
    rounded fp32 output."""
    cfg = synth.small(synth.CONFIGS["c1"], 512, 256, 4, 1)
    raws = synth.make_banks(cfg, seed=7)
    gate, up, down = banks_on_device(cfg, raws)
    inp = synth.make_inputs(cfg, 3, seed=8)
    layer = tq.MoeLayer(dev(inp["router"]), None, gate, up, down, 1)
    out, ids, w, _ = layer.forward(dev(inp["x"]), return_routing=True)
    assert torch.equal(w, torch.ones_like(w))
    img = tq.quant_act(dev(inp["x"]))
    g, u = tq.expert_matvec2(gate, up, img, ids)
    direct = tq.expert_matvec(down, tq.quant_act(tq.moe_swiglu(g, u)), ids, per_expert_input=True)
    assert torch.allclose(out, direct, rtol=0, atol=5e-5)      # intermediate rows quantised per 32 values (fused) or per row (here)
    out16 = layer.forward(dev(inp["x"]), out_type=tq.BF16)
    assert torch.equal(out16, out.to(torch.bfloat16))


@pytest.mark.parametrize("n", [3, 200])
def test_layer_shared_expert_without_a_gate_row(tq, oracle, n):
    """An always-on shared expert with no gate row (shared_gate NULL) is weighted by 1, on the decode kernels and on the
    grouped products: the oracle gets there through a shared-gate logit whose sigmoid is exactly 1."""
    cfg = synth.small(synth.CONFIGS["c2"], 512, 256, 12, 3)
    raws = synth.make_banks(cfg, seed=140 + n)
    gate, up, down = banks_on_device(cfg, raws)
    inp = synth.make_inputs(cfg, n, seed=141 + n)
    layer = tq.MoeLayer(dev(inp["router"]), None, gate, up, down, cfg["topk"], shared_ff=cfg["shared_ff"])
    out, ids, w, logits = (t.cpu().numpy() for t in layer.forward(dev(inp["x"]), return_routing=True))
    assert not logits[:, cfg["experts"]].any()
    logits[:, cfg["experts"]] = 100.0
    mode = oracle_mode(layer, n)
    want, want_ids, want_w = oracle.layer_forward(inp["x"][1], logits, *raws, cfg["wtype"], cfg["hidden"], cfg["ff"], cfg["experts"], cfg["topk"],
                                                  shared_ff=cfg["shared_ff"], act_mode=mode, threads=8)
    check_layer(out, ids, w, want, want_ids, want_w, clear_tokens(oracle, logits, cfg["experts"], cfg["topk"], ids, want_ids))
