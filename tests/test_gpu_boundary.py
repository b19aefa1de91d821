"""GPU parity of the entry points that take the reference's own operands, through the C ABI: the decode grouping maps
(moe_dedup_maps) and the routing histogram (moe_count) bit for bit against the oracle's restatements, moe_group with the
reference's arguments, the clamp of the SwiGLU inputs (MoeConfig::swiglu_clamp) on every path of the layer against the
oracle, and the int8 grouped product on natural-order rows (WeightFormat::expert_gemm_i8's operands)."""
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


@pytest.mark.parametrize("experts,n,topk,skew", [(512, 16, 10, False), (512, 1, 10, False), (64, 128, 8, True), (8, 100, 4, False), (300, 102, 10, True), (16, 5, 3, False)])
def test_dedup_maps_bit_exact(tq, oracle, experts, n, topk, skew):
    rng = np.random.default_rng(experts + n)
    p = 1.0 / np.arange(1, experts + 1) ** 1.2 if skew else np.ones(experts)
    ids = np.stack([rng.choice(experts, size=topk, replace=False, p=p / p.sum()) for _ in range(n)]).astype(np.int32).reshape(-1)
    ids[rng.random(len(ids)) < 0.05] = -1                          # skipped assignments
    slot_of = rng.permutation(experts * 3)[:experts].astype(np.int32)   # the bank slots need not be a permutation of the experts
    for groups in (len(ids), len(ids) + 7):
        slots, gu, dn = (t.cpu().numpy() for t in tq.moe_dedup_maps(dev(ids), dev(slot_of), topk, groups))
        ws, wgu, wdn = oracle.dedup_maps(ids, slot_of, topk, groups)
        assert np.array_equal(slots, ws) and np.array_equal(gu, wgu) and np.array_equal(dn, wdn)
    # every listed assignment appears exactly once as an output row, runs never mix slots
    used = gu[gu[:, 0] >= 0]
    rows = np.concatenate([g[10:10 + g[1]] for g in used])
    assert np.array_equal(np.sort(rows), np.flatnonzero(ids >= 0))
    with pytest.raises(tq.TqmoeError):
        tq.moe_dedup_maps(dev(ids), dev(slot_of), topk, len(ids) - 1)


@pytest.mark.parametrize("wtype_name", ["IQ4_XS", "IQ3_S"])
def test_matvec_over_dedup_maps(tq, oracle, wtype_name):
    """The products over the maps of moe_dedup_maps (gate / up from the token rows, down from a row per assignment) equal the
    products over the ids (to fp32 rounding: the waves may split a row's sum differently for another number of assignments),
    with bank slots that are not the experts' numbers and skipped assignments."""
    wtype = getattr(oracle, wtype_name)
    rng = np.random.default_rng(5)
    experts, rows, cols, n, topk = 12, 128, 512, 9, 4
    slot_of = rng.permutation(experts).astype(np.int32)
    ids = np.stack([rng.permutation(experts)[:topk] for _ in range(n)]).astype(np.int32)
    ids[2, 1] = -1
    banks = [tq.ExpertBank(wtype, synth.bank_blocks(wtype, experts * rows, cols, rng), experts, rows, cols) for _ in range(2)]
    x = torch.randn(n, cols, device="cuda", dtype=torch.float16)
    slots, gu, dn = tq.moe_dedup_maps(dev(ids.reshape(-1)), dev(slot_of), topk)
    slot_ids = slots.view(n, topk)
    img = tq.quant_act(x)
    want_g, want_u = tq.expert_matvec2(banks[0], banks[1], img, slot_ids)
    got_g, got_u = tq.expert_matvec_dedup(banks[0], x, gu, n * topk, bank2=banks[1])
    for got, want in ((got_g, want_g), (got_u, want_u)):
        assert (got - want).abs().max().item() <= 2e-6 * want.abs().max().item()
    xa = torch.randn(n * topk, cols, device="cuda", dtype=torch.float16)          # a row per assignment: the down product's input
    want_d = tq.expert_matvec(banks[0], tq.quant_act(xa), slot_ids, per_expert_input=True, out_type=tq.BF16)
    got_d = tq.expert_matvec_dedup(banks[0], xa, dn, n * topk, out_type=tq.BF16)
    assert (got_d.float() - want_d.float()).abs().max().item() <= 2.0 ** -7 * want_d.float().abs().max().item() and not got_d[2 * topk + 1].any()


def test_count_and_group(tq, oracle):
    rng = np.random.default_rng(4)
    experts, n, topk = 96, 700, 6
    ids = rng.integers(-1, experts, (n, topk)).astype(np.int32)
    counts = torch.zeros(experts, dtype=torch.int64, device="cuda")
    counts[5] = 1 << 40                                             # 64-bit counters that run on
    for _ in range(3):
        tq.moe_count(dev(ids), counts)
    want = np.zeros(experts, np.int64)
    want[5] = 1 << 40
    for _ in range(3):
        oracle.count(ids, want)
    assert np.array_equal(counts.cpu().numpy(), want)
    # moe_group with the reference's arguments: counts and ascending lists [experts][n], from the built-in scratch
    # (one chunk of assignments; several chunks; more than 1024 experts, where the placement reads offsets that the caller
    # did not ask for from the built-in scratch)
    for sub, ne in ((ids, experts), (ids[:3], experts), (rng.integers(0, 1500, (900, 2)).astype(np.int32), 1500)):
        c, g = (t.cpu().numpy() for t in tq.moe_group(dev(sub), ne))
        wc, wo, wp = oracle.dispatch(sub, ne)
        assert np.array_equal(c, wc)
        for e in range(ne):
            assert np.array_equal(g[e, : wc[e]], wp[wo[e]:wo[e + 1]]) and (g[e, wc[e]:] == -1).all()


@pytest.mark.parametrize("clamp_gate", [False, True])
def test_swiglu_clamped(tq, clamp_gate):
    rng = np.random.default_rng(12)
    g = (rng.standard_normal(5000) * 3).astype(np.float32)
    u = (rng.standard_normal(5000) * 3).astype(np.float32)
    limit = 1.25
    got = tq.moe_swiglu(dev(g), dev(u), limit, clamp_gate).cpu().numpy()
    g64, u64 = g.astype(np.float64), np.clip(u.astype(np.float64), -limit, limit)
    if clamp_gate:
        g64 = np.minimum(g64, limit)
    s = g64 / (1 + np.exp(-g64))
    if not clamp_gate:
        s = np.minimum(s, limit)
    assert np.abs(got - s * u64).max() < 2e-6 * np.abs(s * u64).max()
    plain = tq.moe_swiglu(dev(g), dev(u)).cpu().numpy()
    assert np.abs(plain - got).max() > 0.5                          # the limit really bites on these values
    assert np.array_equal(tq.moe_swiglu(dev(g), dev(u), 1e-6, clamp_gate).cpu().numpy(), plain)     # at or below 1e-6: no clamp


@pytest.mark.parametrize("name,n,path", [("c2", 5, "decode"), ("c2", 200, "grouped_i8"), ("c1", 5, "decode"), ("c1", 300, "grouped_i8"), ("c5", 300, "grouped_fp8")])
@pytest.mark.parametrize("clamp_gate", [False, True])
def test_layer_swiglu_clamp(tq, oracle, name, n, path, clamp_gate):
    """swiglu_clamp / clamp_gate of the layer descriptor on the decode kernels and the 8-bit grouped products against the oracle
    with the same clamp; the limit is set where it cuts a fair share of the values, so that the unclamped layer is far away."""
    base = synth.CONFIGS[name]
    cfg = synth.small(base, 768, 512, 10, 3)
    raws = synth.make_banks(cfg, seed=700, sigma=0.06)
    gate, up, down = banks_on_device(cfg, raws)
    inp = synth.make_inputs(cfg, n, seed=701)
    limit = 0.5
    mk = lambda c: tq.MoeLayer(dev(inp["router"]), dev(inp["shared_gate"]) if cfg["shared_ff"] else None, gate, up, down, cfg["topk"], shared_ff=cfg["shared_ff"],
                               swiglu_clamp=c, clamp_gate=clamp_gate, act_blocks=2 if path == "grouped_i8" else 0)
    layer = mk(limit)
    assert layer.path(n) == path
    out, ids, w, logits = (t.cpu().numpy() for t in layer.forward(dev(inp["x"]), return_routing=True))
    want, want_ids, want_w = oracle.layer_forward(inp["x"][1], logits, *raws, cfg["wtype"], cfg["hidden"], cfg["ff"], cfg["experts"], cfg["topk"],
                                                  shared_ff=cfg["shared_ff"], act_mode=oracle_mode(layer, n), threads=16, swiglu_clamp=limit, clamp_gate=clamp_gate)
    clear = clear_tokens(oracle, logits, cfg["experts"], cfg["topk"], ids, want_ids)
    assert np.array_equal(ids[clear], want_ids[clear])
    mx, rel = synth.errors(out[clear], want[clear])
    top = float(np.abs(want[clear]).max())
    fp8 = path == "grouped_fp8"
    print("%s, %d tokens, %s, clamp %.2f gate-first %s: max-abs %.3g (largest value %.3g) rel-rms %.3g" % (name, n, path, limit, clamp_gate, mx, top, rel))
    assert mx < MAX_ABS * max(1.0, top) and rel < (3e-3 if fp8 else REL_RMS), (mx, rel)
    plain = mk(0.0).forward(dev(inp["x"])).cpu().numpy()
    assert synth.errors(plain[clear], want[clear])[1] > 0.05       # without the clamp: another result
    # a descriptor that ends before the clamp fields does not clamp
    full = layer.desc

    def short():
        d = full()
        d.struct_size = tq.api._Layer.swiglu_clamp.offset
        return d
    layer.desc = short
    assert np.array_equal(layer.forward(dev(inp["x"])).cpu().numpy(), plain)


def test_layer_swiglu_clamp_f16_path(tq, oracle):
    """the same on the fp16 grouped products (a format with no 8-bit product)"""
    cfg = dict(hidden=768, ff=512, experts=10, topk=3, shared_ff=256, wtype=oracle.Q6_K, rtype="bf16", xtype="bf16")
    raws = synth.make_banks(cfg, seed=710, sigma=0.06)
    gate, up, down = banks_on_device(cfg, raws)
    n = 300
    inp = synth.make_inputs(cfg, n, seed=711)
    layer = tq.MoeLayer(dev(inp["router"]), dev(inp["shared_gate"]), gate, up, down, cfg["topk"], shared_ff=cfg["shared_ff"], swiglu_clamp=0.5, clamp_gate=True)
    assert layer.path(n) == "grouped_f16"
    out, ids, w, logits = (t.cpu().numpy() for t in layer.forward(dev(inp["x"]), return_routing=True))
    want, want_ids, _ = oracle.layer_forward(inp["x"][1], logits, *raws, cfg["wtype"], cfg["hidden"], cfg["ff"], cfg["experts"], cfg["topk"], shared_ff=cfg["shared_ff"],
                                             act_mode=0, threads=16, swiglu_clamp=0.5, clamp_gate=True)
    clear = clear_tokens(oracle, logits, cfg["experts"], cfg["topk"], ids, want_ids)
    mx, rel = synth.errors(out[clear], want[clear])
    assert mx < MAX_ABS * max(1.0, float(np.abs(want).max())) and rel < REL_RMS, (mx, rel)


def natural_rows(q):
    """int8 rows in the library's byte order -> natural element order (see tests/test_gpu_prefill.py::natural_order)"""
    rows, cols = q.shape
    pos = [2 * d if d < 4 else 2 * (d - 4) + 1 for d in range(8)]
    return np.ascontiguousarray(q.reshape(rows, cols // 32, 8, 4)[:, :, pos, :].reshape(rows, cols))


@pytest.mark.parametrize("wtype_name", ["IQ4_XS", "Q4_K", "IQ3_S"])
@pytest.mark.parametrize("per_expert_input", [False, True])
def test_expert_gemm_i8_reference_operands(tq, oracle, wtype_name, per_expert_input):
    """tqmoe_expert_gemm_i8_ref (natural-order int8 rows, scales [rows][cols / 32], counts + groups [E][capacity]) gives the
    rows of the library's own int8 product on the same quantised values bit for bit, in both activation modes (compared as
    fp16 rows); its bf16 rows (the reference's output type) are the same values rounded to bf16."""
    wtype = getattr(oracle, wtype_name)
    rng = np.random.default_rng(77)
    experts, rows, cols, n, topk = 6, 128, 512, 90, 3
    raw = synth.bank_blocks(wtype, experts * rows, cols, rng)
    bank = tq.ExpertBank(wtype, raw, experts, rows, cols)
    ids = np.stack([rng.permutation(experts)[:topk] for _ in range(n)]).astype(np.int32)
    ids[4, 2] = -1
    A = n * topk
    xdiv = 1 if per_expert_input else topk
    x = torch.randn(A if per_expert_input else n, cols, device="cuda", dtype=torch.float16)
    counts, offsets, perm, groups = tq.moe_dispatch(dev(ids), experts, capacity=int(np.bincount(ids[ids >= 0]).max()) + 3)
    lists = (counts, offsets, perm)
    # mode 2: one scale per token
    rq, rs = tq.quant_rows_i8(x)
    xq, xs = tq.gather_rows_i8(rq, rs, lists, A, xdiv)
    y_lib = tq.expert_gemm_i8(bank, xq, xs, lists, n, topk, topk)
    xq_nat = dev(natural_rows(rq.cpu().numpy()))
    xs_ref = rs[:, None].repeat(1, cols // 32).contiguous()
    y_ref = tq.expert_gemm_i8_ref(bank, xq_nat, xs_ref, counts, groups, topk, A, per_expert_input, mode=2, out_dtype=torch.float16)
    assert torch.equal(y_ref, y_lib)
    y_bf = tq.expert_gemm_i8_ref(bank, xq_nat, xs_ref, counts, groups, topk, A, per_expert_input, mode=2)
    assert y_bf.dtype == torch.bfloat16 and (y_bf.float() - y_lib.float()).abs().max().item() <= 2.0 ** -8 * y_lib.float().abs().max().item()
    assert not y_bf.float().cpu().numpy()[ids.reshape(-1) < 0].any()                       # unlisted rows untouched
    # mode 1: a scale per 32 values
    bq, bs, _ = tq.quant_rows_i8_blocks(x)
    xq1, xs1, xb1 = tq.gather_rows_i8_blocks(bq, bs, lists, A, xdiv)
    y_lib1 = tq.expert_gemm_i8_blocks(bank, xq1, xs1, xb1, lists, n, topk, topk)
    y_ref1 = tq.expert_gemm_i8_ref(bank, dev(natural_rows(bq.cpu().numpy())), bs, counts, groups, topk, A, per_expert_input, mode=1, out_dtype=torch.float16)
    assert torch.equal(y_ref1, y_lib1)
    # a capacity below the largest count: the lists are cut there, no row is written twice or from another expert's list
    cap = 4
    cut = groups[:, :cap].contiguous()
    y_cut = tq.expert_gemm_i8_ref(bank, xq_nat, xs_ref, counts, cut, topk, A, per_expert_input, mode=2, out_dtype=torch.float16)
    kept = np.zeros(A, bool)
    kept[cut.cpu().numpy()[cut.cpu().numpy() >= 0]] = True
    assert counts.max().item() > cap and torch.equal(y_cut[dev(kept)], y_lib[dev(kept)]) and not y_cut[dev(~kept)].any()
    # formats without an int8 product answer `unsupported` (the base class's false)
    if wtype_name == "IQ4_XS":
        q6 = tq.ExpertBank(oracle.Q6_K, synth.bank_blocks(oracle.Q6_K, experts * rows, cols, rng), experts, rows, cols)
        with pytest.raises(tq.TqmoeError) as ex:
            tq.expert_gemm_i8_ref(q6, xq_nat, xs_ref, counts, groups, topk, A, per_expert_input)
        assert ex.value.code == -2
