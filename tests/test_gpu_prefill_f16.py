"""GPU parity of the fp16 grouped products (every bank format) and of the layer at prefill sizes for the formats that
take them, through the C ABI. The operands are rounded to fp16 (2^-11 relative), sums are fp32: the layer stays within
the stated bars of the fp32 oracle directly (max-abs 1e-2, rel-RMS 1e-3)."""
import numpy as np
import pytest
import torch

import synth
from gpu_util import banks_on_device, clear_tokens, dev, oracle_mode

pytestmark = pytest.mark.gpu

MAX_ABS, REL_RMS = 1e-2, 1e-3


@pytest.fixture(scope="module")
def tq():
    import tqllm_amd
    return tqllm_amd


@pytest.mark.parametrize("wtype", [12, 21, 23, 323, 20, 8, 13, 14, 11, 17, 10, 19])
@pytest.mark.parametrize("n,shared_ff", [(70, 0), (200, 128)])
def test_grouped_f16_products_against_float64(tq, oracle, wtype, n, shared_ff):
    rng = np.random.default_rng(wtype + n)
    experts, ff, hidden, k = 6, 256, 512, 3
    banks = experts + (1 if shared_ff else 0)
    decs, devb = [], []
    for rows, cols in ((ff, hidden), (ff, hidden), (hidden, ff)):
        raw = synth.bank_blocks(wtype, banks * rows, cols, rng)
        decs.append(oracle.dequantize(wtype, raw, banks * rows * cols).reshape(banks, rows, cols).astype(np.float64))
        devb.append(tq.ExpertBank(wtype, raw, banks, rows, cols))
    gate, up, down = devb
    slots = k + (1 if shared_ff else 0)
    ids = np.stack([rng.permutation(experts)[:k] for _ in range(n)]).astype(np.int32)
    ids[:, 0] = np.where(rng.random(n) < 0.6, 2, ids[:, 0])
    for t in range(n):
        if (ids[t, 1:] == ids[t, 0]).any():
            ids[t, 0] = [e for e in range(experts) if e not in ids[t, 1:]][0]
    if shared_ff:
        ids = np.concatenate([ids, np.full((n, 1), experts, np.int32)], axis=1)
    ids[3, 1] = -1                                         # skipped: rows stay as allocated
    xb, xv = oracle.to_bf16(rng.standard_normal((n, hidden)).astype(np.float32))
    x = torch.from_numpy(xb.view(np.int16)).cuda().view(torch.bfloat16)
    counts, offsets, perm, _ = tq.moe_dispatch(dev(ids), banks)
    lists = (counts, offsets, perm)
    act = tq.expert_gemm_gateup(gate, up, x, lists, n, slots, k, shared_ff)
    got = act.float().cpu().numpy()
    flat = ids.reshape(-1)
    for a in range(n * slots):
        e = flat[a]
        if e < 0:
            assert not got[a].any()
            continue
        lim = shared_ff if (shared_ff and e == experts) else ff
        g = decs[0][e][:lim] @ xv[a // slots].astype(np.float64)
        u = decs[1][e][:lim] @ xv[a // slots].astype(np.float64)
        want = g / (1 + np.exp(-g)) * u
        assert synth.errors(got[a, :lim], want)[1] < 1.5e-3, a       # fp16 weights and fp16 store
        assert not got[a, lim:].any()
    y = tq.expert_gemm(down, act, lists, n, slots, k, shared_ff, per_expert_input=True, out_type=tq.F32 if n > 100 else tq.F16).float().cpu().numpy()
    av = act.double().cpu().numpy()
    for a in range(n * slots):
        e = flat[a]
        if e < 0:
            continue
        lim = shared_ff if (shared_ff and e == experts) else ff
        want = decs[2][e][:, :lim] @ av[a, :lim]
        assert synth.errors(y[a], want)[1] < 1.5e-3, a


@pytest.mark.parametrize("rows", [40, 200, 333])
@pytest.mark.parametrize("n,xdtype", [(50, "f32"), (900, "f16"), (900, "bf16")])
def test_grouped_f16_product_ragged_rows_and_input_types(tq, oracle, rows, n, xdtype):
    """Weight-row counts that fill the kernel's 128-row blocks only partly, each input type, lists short (64-row blocks) and long
    (128-row blocks), one input row per token shared by its assignments."""
    rng = np.random.default_rng(rows + n)
    experts, cols, k = 5, 512, 2
    raw = synth.bank_blocks(12, experts * rows, cols, rng)
    dec = oracle.dequantize(12, raw, experts * rows * cols).reshape(experts, rows, cols).astype(np.float64)
    bank = tq.ExpertBank(12, raw, experts, rows, cols)
    ids = np.stack([rng.permutation(experts)[:k] for _ in range(n)]).astype(np.int32)
    x32 = rng.standard_normal((n, cols)).astype(np.float32)
    if xdtype == "f32":
        x, xv = torch.from_numpy(x32).cuda(), x32
    elif xdtype == "f16":
        x = torch.from_numpy(x32).cuda().half()
        xv = x.float().cpu().numpy()
    else:
        xb, xv = oracle.to_bf16(x32)
        x = torch.from_numpy(xb.view(np.int16)).cuda().view(torch.bfloat16)
    counts, offsets, perm, _ = tq.moe_dispatch(dev(ids), experts)
    y = tq.expert_gemm(bank, x, (counts, offsets, perm), n, k, k, out_type=tq.F32).cpu().numpy()
    flat = ids.reshape(-1)
    for a in range(0, n * k, 7):
        want = dec[flat[a]] @ xv[a // k].astype(np.float64)
        assert synth.errors(y[a], want)[1] < 1.5e-3, a


def run_layer(tq, oracle, cfg, n, seed, distinct=None, zipf=None, head=None):
    raws = synth.make_banks(cfg, seed=seed, distinct=distinct)
    gate, up, down = banks_on_device(cfg, raws)
    inp = synth.make_inputs(cfg, n, seed=seed + 1, zipf=zipf)
    layer = tq.MoeLayer(dev(inp["router"]), dev(inp["shared_gate"]) if cfg["shared_ff"] else None, gate, up, down, cfg["topk"],
                        shared_ff=cfg["shared_ff"])
    out, ids, w, logits = (t.cpu().numpy() for t in layer.forward(dev(inp["x"]), return_routing=True))
    sel = slice(None) if head is None else slice(0, head)
    want, want_ids, want_w = oracle.layer_forward(inp["x"][1][sel], logits[sel], *raws, cfg["wtype"], cfg["hidden"], cfg["ff"], cfg["experts"],
                                                  cfg["topk"], shared_ff=cfg["shared_ff"], act_mode=oracle_mode(layer, n), threads=16)
    clear = clear_tokens(oracle, logits[sel], cfg["experts"], cfg["topk"], ids[sel], want_ids)
    assert np.array_equal(ids[sel][clear], want_ids[clear])
    assert np.abs(w[sel][clear] - want_w[clear]).max() < 3e-6
    mx, rel = synth.errors(out[sel][clear], want[clear])
    top = float(np.abs(want[clear]).max())
    print("%s, %d tokens, %s: max-abs %.3g (largest value %.3g) rel-rms %.3g" % (cfg.get("name", cfg["wtype"]), n, layer.path(n), mx, top, rel))
    # the fp8 layer against its oracle: E4M3's coarse steps amplify last-bit differences of the act rows (one act value that
    # lands on the other side of a step moves by up to 12 %), so its gates are 3e-3 and 1e-2 of the largest value
    if layer.path(n) == "grouped_fp8":
        assert mx < MAX_ABS * max(1.0, top) and rel < 3e-3, (mx, top, rel)
    else:
        assert mx < MAX_ABS and rel < REL_RMS, (mx, rel)
    return out, ids, layer, inp


@pytest.mark.parametrize("name", ["c1", "c4", "c5"])
def test_layer_grouped_f16_small_shapes(tq, oracle, name):
    base = synth.CONFIGS[name]
    cfg = synth.small(base, 768 if name != "c5" else 384, 512 if name != "c5" else 256, 10, 3)
    run_layer(tq, oracle, cfg, 800, seed=80)      # 2400+ assignments: past what the decode kernels group per launch


def test_layer_config1_512_tokens(tq, oracle):
    run_layer(tq, oracle, synth.CONFIGS["c1"], 512, seed=310, distinct=16, head=96)


def test_layer_config5_full_size_properties(tq, oracle):
    """NVFP4 layer at 8192 tokens: the first 48 rows against the oracle, and a sub-batch in another order gives the same
    rows bit for bit (600 tokens: large enough for the same router and product kernels as the full batch)."""
    cfg = synth.CONFIGS["c5"]
    out, ids, layer, inp = run_layer(tq, oracle, cfg, 8192, seed=510, distinct=3, head=48)
    assert len(np.unique(ids)) == cfg["experts"]
    pick = torch.from_numpy(np.random.default_rng(2).permutation(8192)[:600].copy()).cuda()
    sub = layer.forward(dev(inp["x"])[pick].contiguous())
    assert torch.equal(sub.cpu(), torch.from_numpy(out)[pick.cpu()])
