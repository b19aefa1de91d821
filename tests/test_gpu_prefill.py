"""GPU parity of the prefill-sized path (grouped int8 products on the matrix cores), through the C ABI.

The activations of this path are int8 per row, as in the reference's expert_gemm_i8 (weight_format.hpp:54-59, per-token
mode): a lossy operand format, so two oracles are used. Oracle B (oracle.layer_forward act_mode=5: the same per-row
int8 quantiser on both product inputs, fp16 storage of the intermediate rows) is the gate; the distance to oracle A
(fp32 activations) is reported and bounded loosely. Routing ids, counts and the dispatch lists stay bit-exact."""
import numpy as np
import pytest
import torch

import synth
from gpu_util import banks_on_device, clear_tokens, dev

pytestmark = pytest.mark.gpu

MAX_ABS, REL_RMS = 1e-2, 1e-3


@pytest.fixture(scope="module")
def tq():
    import tqllm_amd
    return tqllm_amd


def natural_order(q):
    """int8 rows as the library stores them -> natural element order. Every 32 values are kept as 8 dwords with natural
    dword d (values 4d .. 4d + 3) at position 2d (d < 4) or 2 (d - 4) + 1."""
    rows, cols = q.shape
    pos = [2 * d if d < 4 else 2 * (d - 4) + 1 for d in range(8)]
    return q.reshape(rows, cols // 32, 8, 4)[:, :, pos, :].reshape(rows, cols)


def ungroup(q, scale, counts, perm, assignments):
    """Grouped operand-major row tiles -> (int8 [assignments][cols] in natural order, scale [assignments]); rows of
    assignments that are in no list stay zero. A tile is [sub-block][lane half g][row r][16 bytes]; the two 16-byte halves
    of (row, sub-block) are the 32-byte block that natural_order() understands."""
    cols = q.shape[1]
    tiles = q.reshape(-1, cols // 32, 2, 32, 16)
    rows = tiles.transpose(0, 3, 1, 2, 4).reshape(-1, cols)          # [tile * 32 + r][cols], blocks of 32 bytes
    rows = natural_order(np.ascontiguousarray(rows))
    out = np.zeros((assignments, cols), np.int8)
    out_s = np.zeros(assignments, np.float32)
    base, at = 0, 0
    for c in counts:
        for i in range(c):
            out[perm[at + i]] = rows[base * 32 + i]
            out_s[perm[at + i]] = scale[base * 32 + i]
        at += c
        base += (c + 31) // 32
    return out, out_s


@pytest.mark.parametrize("kind", ["f32", "bf16", "f16"])
def test_quant_rows_i8_bit_exact(tq, oracle, kind):
    rng = np.random.default_rng(5)
    rows, cols = 37, 768
    x = rng.standard_normal((rows, cols)).astype(np.float32) * rng.uniform(0.01, 30, (rows, 1)).astype(np.float32)
    x[7] = 0
    t = torch.from_numpy(x).cuda().to({"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}[kind])
    xv = t.float().cpu().numpy()
    q, s = tq.quant_rows_i8(t)
    q, s = natural_order(q.cpu().numpy()), s.cpu().numpy()
    for r in range(rows):
        wq, ws = oracle.quant_act_row_i8(xv[r])
        assert np.array_equal(q[r], wq), r
        assert s[r] == np.float32(ws)


def grouped_setup(tq, oracle, seed, experts, ff, hidden, n, k, shared, wtype=None, widened=False):
    """widened: the decoded weights as the fp8 products take them (NVFP4G)"""
    wtype = oracle.IQ4_XS if wtype is None else wtype
    rng = np.random.default_rng(seed)
    banks = experts + (1 if shared else 0)
    raws, decs, devb = [], [], []
    for rows, cols in ((ff, hidden), (ff, hidden), (hidden, ff)):
        raw = synth.bank_blocks(wtype, banks * rows, cols, rng)     # encoded N(0, 0.02) weights, or random valid blocks of that size
        raws.append(raw)
        size = banks * rows * cols
        dec = oracle.dequantize_nvfp4_widened(raw, size) if widened else oracle.dequantize(wtype, raw, size)
        decs.append(dec.reshape(banks, rows, cols).astype(np.float64))
        devb.append(tq.ExpertBank(wtype, raw, banks, rows, cols))
    slots = k + (1 if shared else 0)
    ids = np.stack([rng.permutation(experts)[:k] for _ in range(n)]).astype(np.int32)
    ids[:, 0] = np.where(rng.random(n) < 0.7, 1, ids[:, 0])            # a crowded expert (several 128-chunks when n is large)
    for t in range(n):                                                  # keep ids distinct per token
        if (ids[t, 1:] == ids[t, 0]).any():
            ids[t, 0] = [e for e in range(experts) if e not in ids[t, 1:]][0]
    if shared:
        ids = np.concatenate([ids, np.full((n, 1), experts, np.int32)], axis=1)
    return decs, devb, ids, slots, banks


def e4m3_values(oracle, q):
    table = np.array([oracle.e4m3_to_float(c) for c in range(256)], np.float64)
    return table[q.view(np.uint8)]


@pytest.mark.parametrize("kind", ["f32", "bf16", "f16"])
def test_quant_rows_fp8_bit_exact(tq, oracle, kind):
    """Per-row E4M3 (scale amax / 448, nearest even) against the oracle's quantiser, byte for byte."""
    rng = np.random.default_rng(6)
    rows, cols = 41, 768
    x = rng.standard_normal((rows, cols)).astype(np.float32) * rng.uniform(1e-3, 300, (rows, 1)).astype(np.float32)
    x[7] = 0
    x[9, :200] *= 1e-4          # values far below the row's maximum: E4M3 subnormals and zeros
    t = torch.from_numpy(x).cuda().to({"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}[kind])
    xv = t.float().cpu().numpy()
    q, s = tq.quant_rows_fp8(t)
    q, s = natural_order(q.cpu().numpy()).view(np.uint8), s.cpu().numpy()
    for r in range(rows):
        wq, ws = oracle.quant_act_row_e4m3(xv[r])
        same = q[r] == wq
        assert (same | ((q[r] & 0x7F) == 0) & ((wq & 0x7F) == 0)).all(), r      # a zero's sign is free
        assert s[r] == np.float32(ws)


PLANE_FORMATS = ["IQ4_XS", "IQ3_S", "Q4_K", "NVFP4G", "IQ3_XXS", "IQ2_XXS", "IQ2_XS", "IQ2_S", "IQ1_S", "IQ4_NL", "Q5_K", "Q4_0", "Q8_0"]


@pytest.mark.parametrize("wtype", PLANE_FORMATS)
@pytest.mark.parametrize("n,shared_ff", [(3, 0), (70, 256), (300, 512), (900, 0)])
def test_grouped_products_against_float64(tq, oracle, n, shared_ff, wtype):
    """gate/up + SwiGLU and down products over the dispatch lists against float64 on the decoded weights and the
    dequantised 8-bit rows (the integer products are exact, so only fp32 accumulation of 256-blocks and the fp16 store
    separate the two; the fp8 products accumulate in fp32 on the decoded E4M3 operands)."""
    experts, ff, hidden, k = 7, 512, 768, 3
    fp8 = wtype == "NVFP4G"
    wtype = getattr(oracle, wtype)
    decs, (gate, up, down), ids, slots, banks = grouped_setup(tq, oracle, 11 + n, experts, ff, hidden, n, k, shared_ff > 0, wtype, widened=fp8)
    if fp8:
        return grouped_products_fp8(tq, oracle, decs, gate, up, down, ids, slots, banks, n, k, shared_ff, experts, ff, hidden)
    rng = np.random.default_rng(n)
    xb, xv = oracle.to_bf16(rng.standard_normal((n, hidden)).astype(np.float32))
    x = torch.from_numpy(xb.view(np.int16)).cuda().view(torch.bfloat16)
    counts, offsets, perm, _ = tq.moe_dispatch(dev(ids), banks)
    want_counts = np.bincount(ids.reshape(-1), minlength=banks)
    assert np.array_equal(counts.cpu().numpy(), want_counts)
    lists = (counts, offsets, perm)
    xq, xs = tq.group_rows_i8(x, lists, n * slots, slots)
    # the grouped rows are the plain per-row quantiser's rows, gathered
    pq, ps = tq.quant_rows_i8(x)
    uq, us = ungroup(xq.cpu().numpy(), xs.cpu().numpy(), want_counts, perm.cpu().numpy(), n * slots)
    assert np.array_equal(uq, natural_order(pq.cpu().numpy())[np.arange(n * slots) // slots])
    assert np.array_equal(us, ps.cpu().numpy()[np.arange(n * slots) // slots])
    act = tq.expert_gemm_gateup_i8(gate, up, xq, xs, lists, n, slots, k, shared_ff)
    xd = natural_order(pq.cpu().numpy()).astype(np.float64) * ps.cpu().numpy().astype(np.float64)[:, None]
    got = act.float().cpu().numpy()
    for a in range(n * slots):
        e = ids.reshape(-1)[a]
        lim = shared_ff if (shared_ff and e == experts) else ff
        g = decs[0][e][:lim] @ xd[a // slots]
        u = decs[1][e][:lim] @ xd[a // slots]
        want = g / (1 + np.exp(-g)) * u
        assert np.abs(got[a, :lim] - want).max() < 2e-3 * max(1.0, np.abs(want).max()), a
        assert not got[a, lim:].any()
    aq, a_s = tq.group_rows_i8(act, lists, n * slots, 1)
    y = tq.expert_gemm_i8(down, aq, a_s, lists, n, slots, k, shared_ff).float().cpu().numpy()
    pq, ps = tq.quant_rows_i8(act)
    ad = natural_order(pq.cpu().numpy()).astype(np.float64) * ps.cpu().numpy().astype(np.float64)[:, None]
    for a in range(n * slots):
        e = ids.reshape(-1)[a]
        lim = shared_ff if (shared_ff and e == experts) else ff
        want = decs[2][e][:, :lim] @ ad[a, :lim]
        assert np.abs(y[a] - want).max() < 2e-3 * max(1e-3, np.abs(want).max()), a


def ungroup_block_scales(bs, counts, perm, assignments, blocks):
    """block scales [row tile][block][32 rows] -> [assignments][blocks]"""
    t = bs.reshape(-1, blocks, 32).transpose(0, 2, 1).reshape(-1, blocks)     # [tile * 32 + r][blocks]
    out = np.zeros((assignments, blocks), np.float32)
    base, at = 0, 0
    for c in counts:
        for i in range(c):
            out[perm[at + i]] = t[base * 32 + i]
        at += c
        base += (c + 31) // 32
    return out


@pytest.mark.parametrize("kind", ["f32", "bf16", "f16"])
def test_quant_rows_i8_blocks_bit_exact(tq, oracle, kind):
    """A scale per 32 values and the sums per 16 (the reference's k_quant_act_rows mode 1) against the oracle's
    quantiser, bit for bit; blocks whose magnitudes differ a thousandfold, a zero block and a zero row among them."""
    rng = np.random.default_rng(8)
    rows, cols = 37, 768
    x = rng.standard_normal((rows, cols)).astype(np.float32) * np.repeat(rng.uniform(0.01, 30, (rows, cols // 32)), 32, axis=1).astype(np.float32)
    x[7] = 0
    x[9, 64:96] = 0
    t = torch.from_numpy(x).cuda().to({"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}[kind])
    xv = t.float().cpu().numpy()
    qd, sd, qsum = tq.quant_rows_i8_blocks(t)
    q, s, qsum = natural_order(qd.cpu().numpy()), sd.cpu().numpy(), qsum.cpu().numpy()
    for r in range(rows):
        wq, ws, wsum = oracle.quant_act_blocks_i8(xv[r])
        assert np.array_equal(q[r], wq), r
        assert np.array_equal(s[r], ws), r
        assert np.array_equal(qsum[r], wsum), r
    q2, s2, none = tq.quant_rows_i8_blocks(t, sums=False)
    assert none is None and torch.equal(q2, qd) and torch.equal(s2, sd)


BLOCK_FORMATS = [f for f in PLANE_FORMATS if f != "NVFP4G"]


@pytest.mark.parametrize("wtype", BLOCK_FORMATS)
@pytest.mark.parametrize("n,shared_ff", [(3, 0), (70, 256), (300, 512)])
def test_grouped_products_block_scales_against_float64(tq, oracle, n, shared_ff, wtype):
    """The two products on rows with a scale per 32 values against float64 on the decoded weights and the dequantised rows
    (the integer sum of a block is exact; fp32 scaling and accumulation over the blocks and the fp16 store separate the
    two). The inputs have blocks of very different magnitude, where the per-row quantiser loses the small blocks: its
    products must be measurably farther from the fp32 activations than these."""
    experts, ff, hidden, k = 7, 512, 768, 3
    wt = getattr(oracle, wtype)
    decs, (gate, up, down), ids, slots, banks = grouped_setup(tq, oracle, 31 + n, experts, ff, hidden, n, k, shared_ff > 0, wt)
    rng = np.random.default_rng(100 + n)
    xf = rng.standard_normal((n, hidden)).astype(np.float32) * np.repeat(10.0 ** rng.uniform(-2, 1, (n, hidden // 32)), 32, axis=1).astype(np.float32)
    xb, xv = oracle.to_bf16(xf)
    x = torch.from_numpy(xb.view(np.int16)).cuda().view(torch.bfloat16)
    counts, offsets, perm, _ = tq.moe_dispatch(dev(ids), banks)
    want_counts = np.bincount(ids.reshape(-1), minlength=banks)
    lists = (counts, offsets, perm)
    xq, xs, xbs = tq.group_rows_i8_blocks(x, lists, n * slots, slots)
    # the grouped rows are the plain block quantiser's rows, gathered, and so are the gathered quantised rows
    pq, ps, _ = tq.quant_rows_i8_blocks(x, sums=False)
    uq, us = ungroup(xq.cpu().numpy(), xs.cpu().numpy(), want_counts, perm.cpu().numpy(), n * slots)
    ub = ungroup_block_scales(xbs.cpu().numpy(), want_counts, perm.cpu().numpy(), n * slots, hidden // 32)
    tok = np.arange(n * slots) // slots
    assert np.array_equal(uq, natural_order(pq.cpu().numpy())[tok])
    assert np.array_equal(ub, ps.cpu().numpy()[tok]) and (us == 1).all()
    gq, gs, gbs = tq.gather_rows_i8_blocks(pq, ps, lists, n * slots, slots)
    live = np.zeros(xq.shape[0], bool)
    base = 0
    for c in want_counts:
        live[base * 32:base * 32 + c] = True
        base += (c + 31) // 32
    assert np.array_equal(gq.cpu().numpy()[live], xq.cpu().numpy()[live])
    assert np.array_equal(ungroup_block_scales(gbs.cpu().numpy(), want_counts, perm.cpu().numpy(), n * slots, hidden // 32), ub)
    act = tq.expert_gemm_gateup_i8_blocks(gate, up, xq, xs, xbs, lists, n, slots, k, shared_ff)
    xd = natural_order(pq.cpu().numpy()).astype(np.float64) * np.repeat(ps.cpu().numpy().astype(np.float64), 32, axis=1)
    got = act.float().cpu().numpy()
    act_rows = tq.expert_gemm_gateup_i8(gate, up, *tq.group_rows_i8(x, lists, n * slots, slots), lists, n, slots, k, shared_ff).float().cpu().numpy()
    err_blocks = err_rows = 0.0
    for a in range(n * slots):
        e = ids.reshape(-1)[a]
        lim = shared_ff if (shared_ff and e == experts) else ff
        g = decs[0][e][:lim] @ xd[a // slots]
        u = decs[1][e][:lim] @ xd[a // slots]
        want = g / (1 + np.exp(-g)) * u
        assert np.abs(got[a, :lim] - want).max() < 2e-3 * max(1.0, np.abs(want).max()), a
        assert not got[a, lim:].any()
        g, u = decs[0][e][:lim] @ xv[a // slots].astype(np.float64), decs[1][e][:lim] @ xv[a // slots].astype(np.float64)
        exact = g / (1 + np.exp(-g)) * u
        err_blocks += np.square(got[a, :lim] - exact).sum()
        err_rows += np.square(act_rows[a, :lim] - exact).sum()
    assert err_blocks < 0.5 * err_rows, (err_blocks, err_rows)
    aq, a_s, abs_ = tq.group_rows_i8_blocks(act, lists, n * slots, 1)
    y = tq.expert_gemm_i8_blocks(down, aq, a_s, abs_, lists, n, slots, k, shared_ff).float().cpu().numpy()
    pq, ps, _ = tq.quant_rows_i8_blocks(act, sums=False)
    ad = natural_order(pq.cpu().numpy()).astype(np.float64) * np.repeat(ps.cpu().numpy().astype(np.float64), 32, axis=1)
    for a in range(n * slots):
        e = ids.reshape(-1)[a]
        lim = shared_ff if (shared_ff and e == experts) else ff
        want = decs[2][e][:, :lim] @ ad[a, :lim]
        assert np.abs(y[a] - want).max() < 2e-3 * max(1e-3, np.abs(want).max()), a


@pytest.mark.parametrize("cols", [2304, 4096])
def test_group_rows_blocks_long_rows(tq, cols):
    """Rows longer than 2048 values take the grouping kernel that works row by row: the same bytes and block scales as the
    plain block quantiser's rows, gathered."""
    rng = np.random.default_rng(cols)
    n, experts, k = 45, 5, 2
    ids = np.stack([rng.permutation(experts)[:k] for _ in range(n)]).astype(np.int32)
    x = torch.from_numpy(rng.standard_normal((n, cols)).astype(np.float32) * np.repeat(10.0 ** rng.uniform(-2, 1, (n, cols // 32)), 32, axis=1).astype(np.float32))
    x = x.cuda().to(torch.float16)
    counts, offsets, perm, _ = tq.moe_dispatch(dev(ids), experts)
    lists = (counts, offsets, perm)
    want_counts = np.bincount(ids.reshape(-1), minlength=experts)
    xq, xs, xbs = tq.group_rows_i8_blocks(x, lists, n * k, k)
    pq, ps, _ = tq.quant_rows_i8_blocks(x, sums=False)
    uq, us = ungroup(xq.cpu().numpy(), xs.cpu().numpy(), want_counts, perm.cpu().numpy(), n * k)
    ub = ungroup_block_scales(xbs.cpu().numpy(), want_counts, perm.cpu().numpy(), n * k, cols // 32)
    tok = np.arange(n * k) // k
    assert np.array_equal(uq, natural_order(pq.cpu().numpy())[tok])
    assert np.array_equal(ub, ps.cpu().numpy()[tok]) and (us == 1).all()
    gq, gs, gbs = tq.gather_rows_i8_blocks(pq, ps, lists, n * k, k)
    assert np.array_equal(ungroup(gq.cpu().numpy(), gs.cpu().numpy(), want_counts, perm.cpu().numpy(), n * k)[0], uq)
    assert np.array_equal(ungroup_block_scales(gbs.cpu().numpy(), want_counts, perm.cpu().numpy(), n * k, cols // 32), ub)


def test_block_scale_products_refuse_fp8_banks_and_missing_scales(tq, oracle):
    decs, (gate, up, down), ids, slots, banks = grouped_setup(tq, oracle, 3, 4, 256, 256, 8, 2, False, oracle.NVFP4G)
    counts, offsets, perm, _ = tq.moe_dispatch(dev(ids), banks)
    lists = (counts, offsets, perm)
    x = torch.randn(8, 256, device="cuda", dtype=torch.bfloat16)
    xq, xs, xbs = tq.group_rows_i8_blocks(x, lists, 8 * slots, slots)
    with pytest.raises(Exception, match="int8"):
        tq.expert_gemm_gateup_i8_blocks(gate, up, xq, xs, xbs, lists, 8, slots, 2, 0)
    decs, (gate, up, down), ids, slots, banks = grouped_setup(tq, oracle, 3, 4, 256, 256, 8, 2, False, oracle.IQ4_XS)
    with pytest.raises(Exception, match="block scales"):
        tq.expert_gemm_i8_blocks(down, xq, xs, None, lists, 8, slots, 2, 0)


def grouped_products_fp8(tq, oracle, decs, gate, up, down, ids, slots, banks, n, k, shared_ff, experts, ff, hidden):
    rng = np.random.default_rng(n)
    xb, xv = oracle.to_bf16(rng.standard_normal((n, hidden)).astype(np.float32))
    x = torch.from_numpy(xb.view(np.int16)).cuda().view(torch.bfloat16)
    counts, offsets, perm, _ = tq.moe_dispatch(dev(ids), banks)
    lists = (counts, offsets, perm)
    xq, xs = tq.group_rows_fp8(x, lists, n * slots, slots)
    pq, ps = tq.quant_rows_fp8(x)
    uq, us = ungroup(xq.cpu().numpy(), xs.cpu().numpy(), np.bincount(ids.reshape(-1), minlength=banks), perm.cpu().numpy(), n * slots)
    assert np.array_equal(uq, natural_order(pq.cpu().numpy())[np.arange(n * slots) // slots])
    assert np.array_equal(us, ps.cpu().numpy()[np.arange(n * slots) // slots])
    act = tq.expert_gemm_gateup_fp8(gate, up, xq, xs, lists, n, slots, k, shared_ff)
    xd = e4m3_values(oracle, natural_order(pq.cpu().numpy())) * ps.cpu().numpy().astype(np.float64)[:, None]
    got = act.float().cpu().numpy()
    for a in range(n * slots):
        e = ids.reshape(-1)[a]
        lim = shared_ff if (shared_ff and e == experts) else ff
        g = decs[0][e][:lim] @ xd[a // slots]
        u = decs[1][e][:lim] @ xd[a // slots]
        want = g / (1 + np.exp(-g)) * u
        assert np.abs(got[a, :lim] - want).max() < 2e-3 * max(1.0, np.abs(want).max()), a
        assert not got[a, lim:].any()
    aq, a_s = tq.group_rows_fp8(act, lists, n * slots, 1)
    y = tq.expert_gemm_fp8(down, aq, a_s, lists, n, slots, k, shared_ff).float().cpu().numpy()
    pq, ps = tq.quant_rows_fp8(act)
    ad = e4m3_values(oracle, natural_order(pq.cpu().numpy())) * ps.cpu().numpy().astype(np.float64)[:, None]
    for a in range(n * slots):
        e = ids.reshape(-1)[a]
        lim = shared_ff if (shared_ff and e == experts) else ff
        want = decs[2][e][:, :lim] @ ad[a, :lim]
        assert np.abs(y[a] - want).max() < 2e-3 * max(1e-3, np.abs(want).max()), a


def test_grouped_products_refuse_the_wrong_operand_type(tq, oracle):
    """int8 rows for an NVFP4G bank, E4M3 rows for an int8 format, a format with neither: refused, nothing enqueued."""
    rng = np.random.default_rng(1)
    mk = lambda t: tq.ExpertBank(t, oracle.quantize(t, (rng.standard_normal((2 * 64, 256)) * 0.02).astype(np.float32)), 2, 64, 256)
    ids = np.zeros((4, 1), np.int32)
    counts, offsets, perm, _ = tq.moe_dispatch(dev(ids), 2)
    x = torch.randn(4, 256, device="cuda", dtype=torch.float16)
    xq, xs = tq.group_rows_i8(x, (counts, offsets, perm), 4, 1)
    for bank, fn in ((mk(oracle.NVFP4G), tq.expert_gemm_i8), (mk(oracle.IQ4_XS), tq.expert_gemm_fp8), (mk(oracle.Q6_K), tq.expert_gemm_i8)):
        with pytest.raises(tq.TqmoeError):
            fn(bank, xq, xs, (counts, offsets, perm), 4, 1, 1)


@pytest.mark.parametrize("wtype", PLANE_FORMATS)
@pytest.mark.parametrize("rows,experts", [(96, 5), (160, 5), (128, 5), (256, 5), (64, 1100)])
def test_gemm_i8_bank_shapes(tq, oracle, rows, experts, wtype):
    """tqmoe_expert_gemm_i8 over banks whose row count changes the kernel's arrangement (one or two operand slots per block,
    unit counts that do or do not allow the single-tile path) and over more experts than a block keeps an index of, against
    float64 on the decoded weights and the dequantised int8 rows. One expert gets several row tiles, the others one."""
    cols, n, k = 256, 150, 1
    fp8 = wtype == "NVFP4G"
    wtype = getattr(oracle, wtype)
    rng = np.random.default_rng(rows + experts)
    raw = synth.bank_blocks(wtype, experts * rows, cols, rng)
    size = experts * rows * cols
    dec = (oracle.dequantize_nvfp4_widened(raw, size) if fp8 else oracle.dequantize(wtype, raw, size)).reshape(experts, rows, cols).astype(np.float64)
    bank = tq.ExpertBank(wtype, raw, experts, rows, cols)
    ids = rng.integers(0, experts, size=(n, k)).astype(np.int32)
    ids[: n // 2, 0] = 2
    x = torch.randn(n, cols, device="cuda", dtype=torch.float16)
    counts, offsets, perm, _ = tq.moe_dispatch(dev(ids), experts)
    lists = (counts, offsets, perm)
    xq, xs = tq.group_rows_i8(x, lists, n * k, 1, fp8=fp8)
    y = tq.expert_gemm_i8(bank, xq, xs, lists, n, k, k, fp8=fp8).float().cpu().numpy()
    pq, ps = tq.quant_rows_i8(x, fp8=fp8)
    rows_q = natural_order(pq.cpu().numpy())
    xd = (e4m3_values(oracle, rows_q) if fp8 else rows_q.astype(np.float64)) * ps.cpu().numpy().astype(np.float64)[:, None]
    for a in range(n):
        want = dec[ids[a, 0]] @ xd[a]
        assert np.abs(y[a] - want).max() < 2e-3 * max(1e-3, np.abs(want).max()), a


def test_grouped_products_skip_negative_ids(tq, oracle):
    experts, ff, hidden, k, n = 4, 256, 512, 2, 40
    decs, (gate, up, down), ids, slots, banks = grouped_setup(tq, oracle, 3, experts, ff, hidden, n, k, False)
    ids[5, 1] = -1
    ids[17, 0] = -1
    x = torch.randn(n, hidden, device="cuda", dtype=torch.bfloat16)
    counts, offsets, perm, _ = tq.moe_dispatch(dev(ids), banks)
    xq, xs = tq.group_rows_i8(x, (counts, offsets, perm), n * slots, slots)
    act = tq.expert_gemm_gateup_i8(gate, up, xq, xs, (counts, offsets, perm), n, slots, k).cpu().numpy()
    flat = ids.reshape(-1)
    assert not act[flat < 0].any()
    assert act[flat >= 0].any(axis=1).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_gather_of_quantised_rows_equals_group_rows(tq, dtype):
    """Quantising every input row once and gathering gives the grouped operand of the one-step kernel bit for bit (rows of
    the padding are left as allocated by both: zeros here), with skipped assignments and a ragged expert."""
    experts, hidden, n, slots = 9, 768, 75, 3
    rng = np.random.default_rng(11)
    ids = rng.integers(0, experts, size=(n, slots)).astype(np.int32)
    ids[rng.random((n, slots)) < 0.1] = -1
    x = torch.randn(n, hidden, device="cuda", dtype=dtype)
    x[7] = 0          # a zero row: scale 0
    counts, offsets, perm, _ = tq.moe_dispatch(dev(ids), experts)
    lists = (counts, offsets, perm)
    q1, s1 = tq.group_rows_i8(x, lists, n * slots, slots)
    rq, rs = tq.quant_rows_i8(x)
    q2, s2 = tq.gather_rows_i8(rq, rs, lists, n * slots, slots)
    assert torch.equal(q1, q2)
    rows = q1.shape[0]
    assert torch.equal(s1[:rows], s2[:rows])
    assert torch.equal(s1[rows:].view(torch.int32), s2[rows:].view(torch.int32))      # the tile index behind the scales


def run_layer(tq, oracle, cfg, n, seed, distinct=None, zipf=None, modes=(5, 0), path="grouped_i8", act_blocks=False, request=True):
    raws = synth.make_banks(cfg, seed=seed, distinct=distinct)
    gate, up, down = banks_on_device(cfg, raws)
    inp = synth.make_inputs(cfg, n, seed=seed + 1, zipf=zipf)
    # the int8 products are asked for (a scale per token unless act_blocks): left alone the library picks the faster products
    layer = tq.MoeLayer(dev(inp["router"]), dev(inp["shared_gate"]) if cfg["shared_ff"] else None, gate, up, down, cfg["topk"],
                        shared_ff=cfg["shared_ff"], act_blocks=1 if act_blocks else 2 if path == "grouped_i8" and request else 0)
    assert layer.path(n) == path
    out, ids, w, logits = (t.cpu().numpy() for t in layer.forward(dev(inp["x"]), return_routing=True))
    wants = {}
    for mode in modes:
        wants[mode] = oracle.layer_forward(inp["x"][1], logits, *raws, cfg["wtype"], cfg["hidden"], cfg["ff"], cfg["experts"], cfg["topk"],
                                           shared_ff=cfg["shared_ff"], act_mode=mode, threads=16)
    clear = clear_tokens(oracle, logits, cfg["experts"], cfg["topk"], ids, wants[modes[0]][1])
    return out, ids, w, wants, clear


def check_layer(out, ids, w, wants, clear):
    fp8 = 2 in wants
    want, want_ids, want_w = wants[2] if fp8 else wants[5] if 5 in wants else wants[6] if 6 in wants else wants[0]
    assert np.array_equal(ids[clear], want_ids[clear])
    assert np.abs(w[clear] - want_w[clear]).max() < 3e-6
    mx, rel = synth.errors(out[clear], want[clear])
    # E4M3 keeps four significant bits: where the two sides' act values differ in their last fp16 bit (fp32 sums in another
    # order) and straddle an E4M3 step, the quantised value moves by 6 to 12 %. About 1e-4 of the act values do, which alone
    # is a relative RMS of about 1e-3 on the output, so the fp8 layer is gated at 3e-3 and at 1e-2 of the largest value; the
    # products on given operands are held to float64 in test_grouped_products_against_float64.
    top = float(np.abs(want[clear]).max())
    print("grouped layer, %d tokens: max-abs %.3g (largest value %.3g) rel-rms %.3g" % (int(clear.sum()), mx, top, rel))
    assert mx < MAX_ABS * (max(1.0, top) if fp8 else 1.0) and rel < (3e-3 if fp8 else REL_RMS), (mx, rel)
    if 0 in wants:                       # distance to the fp32-activation result: the price of the 8-bit operand format
        mxa, rela = synth.errors(out[clear], wants[0][0][clear])
        print("vs fp32 activations: max-abs %.3g rel-rms %.3g; vs the %s-operand oracle: max-abs %.3g rel-rms %.3g" % (mxa, rela, "E4M3" if fp8 else "int8", mx, rel))
        assert rela < (1e-1 if fp8 else 3e-2)
    return mx, rel


@pytest.mark.parametrize("n", [64, 150])
def test_layer_grouped_small_shapes(tq, oracle, n):
    cfg = synth.small(synth.CONFIGS["c2"], 768, 512, 10, 3)
    check_layer(*run_layer(tq, oracle, cfg, n, seed=60 + n))


@pytest.mark.parametrize("name,fmt,path,mode", [("c1", "Q4_K", "grouped_i8", 5), ("c4", "IQ3_S", "grouped_i8", 5), ("c5", "NVFP4G", "grouped_fp8", 2),
                                                ("c4", "IQ3_XXS", "grouped_i8", 5), ("c4", "IQ2_XXS", "grouped_i8", 5), ("c4", "IQ2_XS", "grouped_i8", 5),
                                                ("c4", "IQ2_S", "grouped_i8", 5), ("c4", "IQ1_S", "grouped_i8", 5), ("c4", "IQ4_NL", "grouped_i8", 5),
                                                ("c4", "Q5_K", "grouped_i8", 5), ("c4", "Q4_0", "grouped_i8", 5), ("c4", "Q8_0", "grouped_i8", 5)])
@pytest.mark.parametrize("n", [64, 300])
def test_layer_grouped_other_formats(tq, oracle, name, fmt, path, mode, n):
    """Q4_K and the lattice formats on the int8 products, NVFP4G banks on the fp8 products, against the oracle with the same
    declared operand quantisers (the distance to the fp32-activation oracle printed beside it)."""
    base = dict(synth.CONFIGS[name], wtype=getattr(oracle, fmt))
    cfg = synth.small(base, 768, 512, 10, 3)
    check_layer(*run_layer(tq, oracle, cfg, n, seed=160 + n, modes=(mode, 0), path=path))


@pytest.mark.parametrize("fmt,name,n,path", [("IQ4_XS", "c2", 8, "decode"), ("IQ4_XS", "c2", 300, "grouped_f16"), ("IQ4_XS", "c2", 1024, "grouped_i8"),
                                             ("Q4_K", "c1", 1024, "grouped_f16"), ("IQ3_S", "c4", 300, "grouped_f16"), ("Q8_0", "c4", 300, "grouped_f16"),
                                             ("IQ2_S", "c4", 300, "grouped_i8"), ("IQ1_S", "c4", 300, "grouped_i8"), ("NVFP4G", "c5", 300, "grouped_fp8"),
                                             ("Q6_K", "c4", 300, "grouped_f16")])
def test_layer_products_left_to_the_library(tq, oracle, fmt, name, n, path):
    """With nothing asked for (act_blocks 0) the layer takes the products measured faster for the formats and the batch: the
    decode kernels for few tokens, then the fp16 grouped products, the int8 ones for IQ4_XS from 1024 tokens and for the
    lattice formats, the fp8 ones for NVFP4G; each against the oracle of its operand format."""
    base = dict(synth.CONFIGS[name], wtype=getattr(oracle, fmt))
    cfg = synth.small(base, 768, 512, 10, 3)
    mode = {"decode": 0, "grouped_f16": 0, "grouped_i8": 5, "grouped_fp8": 2}[path]
    check_layer(*run_layer(tq, oracle, cfg, n, seed=860 + n, modes=(mode,), path=path, request=False))


@pytest.mark.parametrize("fmt,n", [("IQ4_XS", 64), ("IQ4_XS", 300), ("Q4_K", 300), ("IQ3_S", 300), ("IQ4_NL", 300), ("IQ2_S", 64), ("Q5_K", 300), ("Q4_0", 64), ("Q8_0", 300)])
def test_layer_block_scales(tq, oracle, fmt, n):
    """The layer with act_blocks set (a scale per 32 activations on both products' inputs, the reference's
    TQFN_PREFILL_INT8=1) against the oracle's mode of the same quantiser; the per-token oracle must be farther away."""
    base = dict(synth.CONFIGS["c2" if fmt == "IQ4_XS" else "c4"], wtype=getattr(oracle, fmt))
    cfg = synth.small(base, 768, 512, 10, 3)
    out, ids, w, wants, clear = run_layer(tq, oracle, cfg, n, seed=260 + n, modes=(6, 0, 5), act_blocks=True)
    wants6 = {6: wants[6], 0: wants[0]}
    mx, rel = check_layer(out, ids, w, wants6, clear)
    mx5, rel5 = synth.errors(out[clear], wants[5][0][clear])
    assert rel5 > 3 * rel, (rel, rel5)


def test_layer_descriptor_without_the_block_field(tq, oracle):
    """A descriptor that ends before act_blocks (an older caller) runs with a scale per token."""
    import ctypes as C
    cfg = synth.small(synth.CONFIGS["c2"], 512, 256, 6, 2)
    raws = synth.make_banks(cfg, seed=5)
    gate, up, down = banks_on_device(cfg, raws)
    inp = synth.make_inputs(cfg, 96, seed=6)
    outs = []
    for blocks, size in ((False, None), (True, tq.api._Layer.act_blocks.offset), (True, None)):
        layer = tq.MoeLayer(dev(inp["router"]), dev(inp["shared_gate"]), gate, up, down, cfg["topk"], shared_ff=cfg["shared_ff"], act_blocks=blocks)
        if size is not None:
            full = layer.desc

            def short(full=full, size=size):
                d = full()
                d.struct_size = size
                return d
            layer.desc = short
        outs.append(layer.forward(dev(inp["x"])).float().cpu())
    assert torch.equal(outs[0], outs[1]) and not torch.equal(outs[0], outs[2])


def test_layer_grouped_small_skewed(tq, oracle):
    cfg = synth.small(synth.CONFIGS["c2"], 512, 256, 12, 3)
    out, ids, w, wants, clear = run_layer(tq, oracle, cfg, 600, seed=71, zipf=1.1)
    check_layer(out, ids, w, wants, clear)
    counts = np.bincount(ids.reshape(-1), minlength=12)
    assert counts.max() > 4 * max(1, counts.min())            # the load really is skewed (several 128-chunks for the top expert)


def test_layer_config3_shape_256_tokens(tq, oracle):
    """Flash-Next-shaped layer, Zipf-skewed routing, 256 tokens against the oracle."""
    check_layer(*run_layer(tq, oracle, synth.CONFIGS["c2"], 256, seed=250, distinct=20, zipf=1.1, modes=(5,)))


def test_layer_config3_full_size_properties(tq, oracle):
    """4096 tokens, Zipf-skewed: too large for the oracle, so checked through what does not depend on size: the same rows
    pushed through in a different batch composition give the same output rows (every row's result depends only on the row
    and its routing), the routing of a row equals the oracle's on the device logits, and the dispatch lists are the
    stable counting sort of the ids."""
    cfg = synth.CONFIGS["c2"]
    n = 4096
    raws = synth.make_banks(cfg, seed=900, distinct=12)
    gate, up, down = banks_on_device(cfg, raws)
    inp = synth.make_inputs(cfg, n, seed=901, zipf=1.1)
    layer = tq.MoeLayer(dev(inp["router"]), dev(inp["shared_gate"]), gate, up, down, cfg["topk"], shared_ff=cfg["shared_ff"])
    x = dev(inp["x"])
    out, ids, w, logits = layer.forward(x, return_routing=True)
    # routing against the oracle on the device's logits
    lg = logits.cpu().numpy()
    want_ids, want_w = oracle.route(lg[:, :cfg["experts"]], cfg["topk"])
    clear = clear_tokens(oracle, lg, cfg["experts"], cfg["topk"], ids.cpu().numpy(), want_ids, "config 3, 4096 tokens")
    assert np.array_equal(ids.cpu().numpy()[clear], want_ids[clear])
    # dispatch lists: stable counting sort
    counts, offsets, perm, _ = tq.moe_dispatch(ids, cfg["experts"])
    flat = ids.cpu().numpy().reshape(-1)
    assert np.array_equal(counts.cpu().numpy(), np.bincount(flat, minlength=cfg["experts"]))
    assert np.array_equal(perm.cpu().numpy(), np.argsort(flat, kind="stable"))
    assert counts.max().item() > 128 * 3                      # the crowded experts span several chunks
    # a sub-batch taken in another order gives bit-identical rows (1100 tokens: on the same products as the full batch)
    assert layer.path(n) == layer.path(1100) == "grouped_i8"
    pick = torch.from_numpy(np.random.default_rng(1).permutation(n)[:1100].copy()).cuda()
    sub = layer.forward(x[pick].contiguous())
    assert torch.equal(sub, out[pick])
    # and 128 of them against the oracle: the first 96 tokens and 32 spread over the rows of the most crowded expert
    ids_np = ids.cpu().numpy()
    crowded = np.flatnonzero((ids_np == int(counts.argmax().item())).any(axis=1))
    head = np.unique(np.concatenate([np.arange(96), crowded[:: max(1, len(crowded) // 32)][:32]]))
    assert len(crowded) > 128 * 3
    want = oracle.layer_forward(inp["x"][1][head], lg[head], *raws, cfg["wtype"], cfg["hidden"], cfg["ff"], cfg["experts"], cfg["topk"],
                                shared_ff=cfg["shared_ff"], act_mode=5, threads=16)[0]
    ok = clear[head]
    mx, rel = synth.errors(out.cpu().numpy()[head][ok], want[ok])
    assert mx < MAX_ABS and rel < REL_RMS, (mx, rel)
