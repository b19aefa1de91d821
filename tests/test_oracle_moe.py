"""Pins the oracle's routing, dispatch, FFN, combine and whole-layer functions against checks the mathematics fixes
(independent max-scan selection, scipy softmax, closed forms and invariants of the reference's tests/moe.cpp, brute
force sorts, float64 numpy) and, where built, the reference's own objects."""
import ctypes as C

import numpy as np
import pytest
from scipy.special import softmax


def max_scan_route(logits, k, gating, norm, scale, bias):
    """Independent reference: repeated strict-greater max scan with a taken mask (the scheme of the reference's
    tests/moe.cpp:36-89), float32 arithmetic through numpy scalars."""
    lg = logits.astype(np.float32)
    if gating == 1:
        mx = lg.max()
        p = np.exp(lg - mx, dtype=np.float32)
        s = np.float32(0)
        for v in p:
            s = np.float32(s + v)
        p = (p / s).astype(np.float32)
    elif gating == 2:
        p = (np.float32(1) / (np.float32(1) + np.exp(-lg, dtype=np.float32))).astype(np.float32)
    elif gating == 3:
        p = lg
    else:
        p = np.sqrt(np.logaddexp(np.float64(0), lg.astype(np.float64))).astype(np.float32)   # log(1 + e^x), stable
    sel = p + bias.astype(np.float32) if bias is not None else p
    taken = np.zeros(len(lg), bool)
    ids, w = [], []
    for _ in range(k):
        best, bv = -1, -np.inf
        for i, v in enumerate(sel):
            if not taken[i] and v > bv:
                best, bv = i, v
        taken[best] = True
        ids.append(best)
        w.append(p[best])
    w = np.array(w, np.float32)
    if gating == 3:                      # softmax over the selected logits only
        w = softmax(w.astype(np.float64)).astype(np.float32)
    if norm:
        s = np.float32(0)
        for v in w:
            s = np.float32(s + v)
        w = (w / max(s, np.float32(6.103515625e-5))).astype(np.float32)
    if scale not in (0.0, 1.0):
        w = (w * np.float32(scale)).astype(np.float32)
    return np.array(ids, np.int32), w


def test_route_matches_independent_max_scan(oracle):
    rng = np.random.default_rng(11)
    for gating in (1, 2, 3, 4):
        for norm in (False, True):
            for biased in (False, True):
                for _ in range(60):
                    e = int(rng.integers(2, 62))
                    k = int(rng.integers(1, e + 1))
                    scale = float(np.float32(rng.uniform(0.01, 4)))
                    lg = rng.uniform(-8, 8, e).astype(np.float32)
                    bias = rng.uniform(-1, 1, e).astype(np.float32) if biased else None
                    ids, w = oracle.route(lg, k, gating, norm, scale, bias)
                    wi, ww = max_scan_route(lg, k, gating, norm, scale, bias)
                    assert np.array_equal(ids[0], wi)
                    assert np.abs(w[0] - ww).max() <= 1e-6


def test_route_softmax_against_scipy(oracle):
    rng = np.random.default_rng(12)
    for e, k in ((64, 8), (512, 10), (256, 8)):
        lg = rng.standard_normal((20, e)).astype(np.float32)
        ids, w = oracle.route(lg, k)
        p = softmax(lg.astype(np.float64), axis=1)
        for t in range(20):
            order = np.lexsort((np.arange(e), -p[t]))[:k]
            assert np.array_equal(ids[t], order)
            want = p[t, order] / p[t, order].sum()
            assert np.abs(w[t] - want).max() < 3e-7
            assert abs(float(w[t].sum()) - 1) < 1e-6
            assert (np.diff(w[t]) <= 0).all()          # descending probability order


def test_route_closed_forms(oracle):
    # all-equal logits: lowest indices win (tests/moe.cpp:183-194)
    ids, w = oracle.route(np.full(8, 0.5, np.float32), 3, gating=2, norm=False)
    assert ids[0].tolist() == [0, 1, 2]
    ids, w = oracle.route(np.full(512, -3.25, np.float32), 10)
    assert ids[0].tolist() == list(range(10)) and np.allclose(w[0], 0.1, atol=1e-7)
    # underflow: every sigmoid exactly 0, weights stay finite (tests/moe.cpp:196-210)
    ids, w = oracle.route(np.array([-200, -300, -400, -500], np.float32), 4, gating=2, norm=True)
    assert np.isfinite(w).all() and not w.any()
    # scale 0 and 1 both mean no scaling; 2.5 multiplies (tests/moe.cpp:212-236)
    lg = np.array([3, 1, -1, -3], np.float32)
    i0, w0 = oracle.route(lg, 2, gating=2, norm=True, scale=0.0)
    i1, w1 = oracle.route(lg, 2, gating=2, norm=True, scale=1.0)
    i2, w2 = oracle.route(lg, 2, gating=2, norm=True, scale=2.5)
    assert np.array_equal(w0, w1) and abs(w1.sum() - 1) < 1e-6 and abs(w2.sum() - 2.5) < 1e-6
    assert np.abs(w2 - 2.5 * w1).max() < 1e-6
    # selection bias moves the choice, not the weight (tests/moe.cpp:149-176)
    ids, w = oracle.route(np.array([2, 1, 0, -1], np.float32), 2, gating=2, norm=False, bias=np.array([0, 0, 0, 100], np.float32))
    assert ids[0, 0] == 3 and abs(w[0, 0] - 1 / (1 + np.exp(1.0))) < 1e-6
    # softmax with far-apart logits: exp underflows to exact zeros, ties among zeros go to the lower index
    ids, w = oracle.route(np.array([0, -200, 50, -300, -250], np.float32), 3)
    assert ids[0].tolist() == [2, 0, 1] and w[0, 0] == 1.0 and w[0, 2] == 0.0
    # softmax over the selected logits: the choice is by logit, the weights a softmax of the chosen ones (moe.cpp:88-97)
    ids, w = oracle.route(np.array([1.0, 3.0, 2.0, -5.0], np.float32), 2, gating=3, norm=False)
    assert ids[0].tolist() == [1, 2] and np.abs(w[0] - np.array([np.e, 1]) / (np.e + 1)).max() < 1e-6
    # sqrt(softplus): at 0 it is sqrt(ln 2); for large x it tends to sqrt(x); for very negative x to exp(x / 2)
    ids, w = oracle.route(np.array([0.0, 40.0, -30.0], np.float32), 3, gating=4, norm=False)
    assert ids[0].tolist() == [1, 0, 2]
    assert np.abs(w[0] - np.array([np.sqrt(40.0), np.sqrt(np.log(2.0)), np.exp(-15.0)])).max() < 1e-6
    assert oracle.shared_weight(0.0) == 0.5 and oracle.shared_weight(-1e30) == 0.0
    assert abs(oracle.shared_weight(1.25) - 1 / (1 + np.exp(-1.25))) < 1e-7


def test_route_matches_reference_objects(oracle, ref):
    rng = np.random.default_rng(13)
    for gating in (1, 2, 3, 4):
        for _ in range(200):
            e = int(rng.integers(2, 600))
            k = int(rng.integers(1, min(e, 16) + 1))
            lg = (rng.standard_normal(e) * rng.uniform(0.1, 6)).astype(np.float32)
            bias = rng.uniform(-1, 1, e).astype(np.float32) if rng.random() < 0.5 else None
            scale = float(np.float32(rng.choice([0.0, 1.0, 2.5])))
            norm = bool(rng.random() < 0.7)
            ids, w = oracle.route(lg, k, gating, norm, scale, bias)
            ri = np.empty(k, np.int32)
            rw = np.empty(k, np.float32)
            bp = bias.ctypes.data_as(C.c_void_p) if bias is not None else None
            assert ref.ref_route(gating, e, k, int(norm), scale, lg.ctypes.data_as(C.c_void_p), bp, ri.ctypes.data_as(C.c_void_p),
                                 rw.ctypes.data_as(C.c_void_p)) == 0
            assert np.array_equal(ids[0], ri)
            assert np.array_equal(w[0].view(np.uint32), rw.view(np.uint32))   # same libm, same order: bit for bit


def softmax_probs_f32(lg):
    """the reference's fp32 softmax, step by step (src/experts/moe.cpp:36-47): exp(l - max), a sequential sum, a division"""
    e = np.exp((lg - lg.max()).astype(np.float32)).astype(np.float32)
    s = np.float32(0)
    for v in e:
        s = np.float32(s + v)
    return (e / s).astype(np.float32)


def test_softmax_collision_flags_exactly_the_unreproducible_rows(oracle):
    """tqo_route_softmax_collision decides which tokens the GPU routing checks may exempt: rows where two *different* logits
    have one fp32 probability at the selection boundary (a selection by logit and the reference's by rounded probability
    can then differ), or where a boundary probability is subnormal. Everything else must not be flagged."""
    lg = np.full(12, -9.0, np.float32)
    near = np.float32(-1e-4)                                  # a ulp of this logit moves exp() by 7e-12, far below a ulp of the result
    lg[:3] = [0.0, near, np.nextafter(near, np.float32(-1))]
    p = softmax_probs_f32(lg)
    assert lg[1] != lg[2] and p[1] == p[2] and p[1] > 0       # the pair really collides in probability
    assert oracle.route_softmax_collision(lg, 2)[0]           # boundary between slots 1 and 2: flagged
    assert oracle.route_softmax_collision(lg, 3)[0]           # the pair inside the selection decides the order of the ids: flagged
    assert not oracle.route_softmax_collision(lg, 1)[0]       # boundary between 0.0 and the pair: clear
    moved = lg.copy()
    moved[[1, 2]] = moved[[2, 1]]                             # the same pair in the other index order: still a collision
    assert oracle.route_softmax_collision(moved, 2)[0]
    # the reference's own choice on that row is by probability, ties to the lower index: id 1 before id 2 both ways
    assert oracle.route(lg, 2)[0][0].tolist() == [0, 1] and oracle.route(moved, 2)[0][0].tolist() == [0, 1]
    # exact ties of equal logits are ordered by index on both sides: not flagged
    tie = lg.copy()
    tie[2] = tie[1]
    assert not oracle.route_softmax_collision(tie, 2)[0]
    # wide gaps: not flagged, whatever k
    wide = np.arange(12, dtype=np.float32) * 0.75
    assert not oracle.route_softmax_collision(wide, 1)[0] and not oracle.route_softmax_collision(wide, 8)[0]
    # a subnormal probability at the boundary (exp(-90) ~ 8e-40): flagged; the same row cut before it: clear
    sub = np.array([0.0, -1.0, -90.0, -200.0, -300.0], np.float32)
    ps = softmax_probs_f32(sub)
    assert 0 < ps[2] < np.finfo(np.float32).tiny and ps[3] == 0
    assert oracle.route_softmax_collision(sub, 2)[0] and oracle.route_softmax_collision(sub, 3)[0]
    assert not oracle.route_softmax_collision(sub, 1)[0]
    # probabilities that underflowed to exact zero are ordered by index: no collision although the logits differ
    zeros = np.array([0.0, -1.0, -200.0, -300.0, -250.0], np.float32)
    assert not oracle.route_softmax_collision(zeros, 4)[0]
    # random rows: collisions are rare (the tests allow one exempt token in 500)
    rng = np.random.default_rng(3)
    assert oracle.route_softmax_collision(rng.standard_normal((2000, 512)).astype(np.float32), 10).sum() <= 4


def test_dispatch_brute_force(oracle):
    rng = np.random.default_rng(14)
    for e, a in ((4, 0), (4, 1), (64, 128), (512, 40960), (7, 1000)):
        ids = rng.integers(-1 if a > 10 else 0, e, a).astype(np.int32)
        counts, offsets, perm = oracle.dispatch(ids, e)
        kept = np.flatnonzero(ids >= 0)
        assert np.array_equal(counts, np.bincount(ids[kept], minlength=e))
        assert offsets[0] == 0 and np.array_equal(np.diff(offsets), counts) and offsets[-1] == len(kept)
        want = kept[np.argsort(ids[kept], kind="stable")]
        assert np.array_equal(perm[:len(kept)], want)
        assert (perm[len(kept):] == -1).all()
        for x in range(e):  # ascending assignment order inside each expert (prefill_plan.hpp:69-73)
            seg = perm[offsets[x]:offsets[x + 1]]
            assert (np.diff(seg) > 0).all() and (ids[seg] == x).all()
    with pytest.raises(ValueError):
        oracle.dispatch(np.array([0, 9], np.int32), 4)


def test_expert_ffn_against_float64(oracle, ref):
    rng = np.random.default_rng(15)
    h, f = 96, 40
    x = rng.standard_normal(h).astype(np.float32)
    wg, wu = (rng.standard_normal((f, h)).astype(np.float32) * 0.2 for _ in range(2))
    wd = rng.standard_normal((h, f)).astype(np.float32) * 0.2
    g, u = wg.astype(np.float64) @ x, wu.astype(np.float64) @ x
    want = wd.astype(np.float64) @ (g / (1 + np.exp(-g)) * u)
    got = oracle.expert_ffn(x, wg, wu, wd)
    assert np.abs(got - want).max() < 1e-5
    # clamp branches (moe.cpp:133-143): GLM clamps gate, generic clamps silu(gate); both clamp up
    xc = x * 40
    g, u = wg.astype(np.float64) @ xc, np.clip(wu.astype(np.float64) @ xc, -7, 7)
    gl = np.minimum(g, 7)
    want_glm = wd.astype(np.float64) @ (gl / (1 + np.exp(-gl)) * u)
    want_gen = wd.astype(np.float64) @ (np.minimum(g / (1 + np.exp(-g)), 7) * u)
    assert np.abs(oracle.expert_ffn(xc, wg, wu, wd, 7.0, True) - want_glm).max() < 1e-3
    assert np.abs(oracle.expert_ffn(xc, wg, wu, wd, 7.0, False) - want_gen).max() < 1e-3
    out = np.empty(h, np.float32)
    p = lambda a: a.ctypes.data_as(C.c_void_p)
    for clamp, cg in ((0.0, 0), (7.0, 1), (7.0, 0)):
        ref.ref_expert_ffn(p(xc), h, p(wg), p(wu), p(wd), f, clamp, cg, p(out))
        assert np.array_equal(oracle.expert_ffn(xc, wg, wu, wd, clamp, bool(cg)), out)


def test_combine_closed_form(oracle):
    outs = np.stack([np.arange(1, 5), np.arange(10, 14)]).astype(np.float32)
    got = oracle.combine(np.array([0.75, 0.25], np.float32), outs)
    assert np.allclose(got, 0.75 * outs[0] + 0.25 * outs[1], atol=1e-6)


def test_router_logits_against_float64(oracle):
    rng = np.random.default_rng(16)
    h, e, n = 256, 24, 3
    w = rng.standard_normal((e, h)).astype(np.float32) * 0.02
    sg = rng.standard_normal(h).astype(np.float32) * 0.02
    x = rng.standard_normal((n, h)).astype(np.float32)
    got = oracle.router_logits(w, oracle.F32, sg, x, oracle.F32, h, e, n)
    want = x.astype(np.float64) @ np.vstack([w, sg]).astype(np.float64).T
    assert np.abs(got - want).max() < 3e-6
    wb, wbf = oracle.to_bf16(w)
    sb, sbf = oracle.to_bf16(sg)
    xb, xbf = oracle.to_bf16(x)
    got = oracle.router_logits(wb, oracle.BF16, sb, xb, oracle.BF16, h, e, n)
    want = xbf.astype(np.float64) @ np.vstack([wbf, sbf]).astype(np.float64).T
    assert np.abs(got - want).max() < 3e-6
    got = oracle.router_logits(w, oracle.F32, None, x, oracle.F32, h, e, n)
    assert not got[:, e].any()


def test_layer_forward_against_float64(oracle):
    """Whole layer vs float64 numpy on the decoded weights, routing taken from the oracle (ids are pinned above)."""
    rng = np.random.default_rng(17)
    h, f, e, k, sf, n = 256, 256, 6, 2, 256, 5
    for wtype in (oracle.IQ4_XS, oracle.Q4_K):
        banks = [oracle.quantize(wtype, (rng.standard_normal(((e + 1) * r, c)) * 0.05).astype(np.float32))
                 for r, c in ((f, h), (f, h), (h, f))]
        dec = [oracle.dequantize(wtype, b, (e + 1) * f * h).astype(np.float64) for b in banks]
        wg, wu = dec[0].reshape(e + 1, f, h), dec[1].reshape(e + 1, f, h)
        wd = dec[2].reshape(e + 1, h, f)
        x = rng.standard_normal((n, h)).astype(np.float32)
        logits = rng.standard_normal((n, e + 1)).astype(np.float32)
        out, ids, w = oracle.layer_forward(x, logits, *banks, wtype, h, f, e, k, shared_ff=sf, threads=3)
        ri, rw = oracle.route(logits[:, :e], k)
        assert np.array_equal(ids, ri) and np.array_equal(w, rw)

        def ffn(j, xv, ff):
            g, u = wg[j, :ff] @ xv, wu[j, :ff] @ xv
            return wd[j, :, :ff] @ (g / (1 + np.exp(-g)) * u)

        for t in range(n):
            want = sum(float(w[t, s]) * ffn(ids[t, s], x[t].astype(np.float64), f) for s in range(k))
            want = want + 1 / (1 + np.exp(-float(logits[t, e]))) * ffn(e, x[t].astype(np.float64), sf)
            assert np.abs(out[t] - want).max() < 2e-5 * max(1.0, np.abs(want).max())
        # no shared expert: that term disappears; linearity in the routed weights
        out2, _, _ = oracle.layer_forward(x, logits, *banks, wtype, h, f, e, k, shared_ff=0, threads=1)
        t = 0
        want = sum(float(w[t, s]) * ffn(ids[t, s], x[t].astype(np.float64), f) for s in range(k))
        assert np.abs(out2[t] - want).max() < 2e-5 * max(1.0, np.abs(want).max())
        # the other routing modes change the ids and weights (pinned above), nothing else
        bias = rng.uniform(-1, 1, e).astype(np.float32)
        out3, ids3, w3 = oracle.layer_forward(x, logits, *banks, wtype, h, f, e, k, shared_ff=0, threads=2, gating=2, norm=False, scale=2.5, bias=bias)
        ri, rw = oracle.route(logits[:, :e], k, 2, False, 2.5, bias)
        assert np.array_equal(ids3, ri) and np.array_equal(w3, rw) and not np.array_equal(ids3, ids)
        for t in range(n):
            want = sum(float(w3[t, s]) * ffn(ids3[t, s], x[t].astype(np.float64), f) for s in range(k))
            assert np.abs(out3[t] - want).max() < 2e-5 * max(1.0, np.abs(want).max())


def test_declared_quantisers(oracle):
    rng = np.random.default_rng(18)
    x = rng.standard_normal(512).astype(np.float32)
    q, s = oracle.quant_act_row_i8(x)
    m = np.abs(x).max()
    assert s == np.float32(m / np.float32(127)) and np.abs(q).max() == 127
    assert np.array_equal(q, np.rint(x * (np.float32(127) / m)).astype(np.int8))
    q0, s0 = oracle.quant_act_row_i8(np.zeros(64, np.float32))
    assert s0 == 0 and not q0.any()
    # E4M3 rows: scale amax / 448, every code the nearest E4M3 value of x * (448 / amax), found here by brute force over
    # the 254 finite codes (ties to the even mantissa), so a truncating or biased conversion fails
    q8, s8 = oracle.quant_act_row_e4m3(x)
    assert s8 == np.float32(m / np.float32(448))
    codes = np.array([b for b in range(256) if (b & 0x7F) != 0x7F], np.uint8)
    vals = np.array([oracle.e4m3_to_float(b) for b in codes], np.float64)
    scaled = (x * (np.float32(448) / m)).astype(np.float32).astype(np.float64)
    for v, got in zip(scaled, q8):
        d = np.abs(vals - v)
        best = codes[np.flatnonzero(d == d.min())]
        best = [b for b in best if (v < 0) == bool(b & 0x80) or v == 0]
        want = [b for b in best if not b & 1] if len(best) > 1 else best
        assert got in want, (v, got, best)
    assert max(oracle.e4m3_to_float(b & 0x7F) for b in q8) == 448.0
    q0, s0 = oracle.quant_act_row_e4m3(np.zeros(64, np.float32))
    assert s0 == 0 and not (q0 & 0x7F).any()


def _half(a):
    return np.asarray(a, np.float64).astype(np.float16).astype(np.float64)


def _requant_i8(v):
    """float64 restatement of the per-row int8 quantiser: fp32 scale amax / 127, q = rint(v * (127 / amax)), value q * scale"""
    v32 = np.asarray(v, np.float64).astype(np.float32)
    m = np.abs(v32).max()
    if m == 0:
        return np.zeros_like(v, np.float64)
    q = np.rint(v32 * (np.float32(127) / m))
    return q.astype(np.float64) * np.float64(np.float32(m / np.float32(127)))


def test_nvfp4_widened_weights_closed_form(oracle):
    """tqo_dequantize_nvfp4_widened against the closed form on every (scale byte, code) pair: the E4M3 value nearest to
    e2m1 * scale / 8 (found by brute force over the 256 codes, ties to the even code), times 8 * the global."""
    codes = np.arange(256, dtype=np.uint8)
    vals = np.array([oracle.e4m3_to_float(c) for c in codes], np.float64)
    finite = ~np.isnan(vals)
    e2m1 = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, -0., -.5, -1, -1.5, -2, -3, -4, -6])

    def nearest(v):   # the value only (the sign of a zero is not observable in a product)
        v = float(np.clip(v, -448, 448))
        d = np.abs(vals[finite] - v)
        best = np.flatnonzero(d == d.min())
        cands = codes[finite][best]
        return vals[finite][best][np.argmin(cands & 1)] if len(set(vals[finite][best])) > 1 else vals[finite][best][0]

    scales = [s for s in range(256) if not np.isnan(oracle.e4m3_to_float(s))]
    g = np.float32(0.37)
    for s0 in range(0, len(scales), 8):
        blk = np.zeros(76, np.uint8)
        blk[:4] = np.frombuffer(g.tobytes(), np.uint8)
        blk[4:12] = scales[s0:s0 + 8] + [0] * (8 - len(scales[s0:s0 + 8]))
        blk[12:76] = np.tile(np.array([0x10, 0x32, 0x54, 0x76, 0x98, 0xBA, 0xDC, 0xFE], np.uint8), 8)   # codes 0..15 in every group
        got = oracle.dequantize_nvfp4_widened(blk, 128).reshape(8, 16)
        for grp in range(8):
            sc = oracle.e4m3_to_float(int(blk[4 + grp]))
            want = np.array([nearest(e2m1[c] * sc / 8) for c in range(16)]) * np.float64(np.float32(8) * g)
            assert np.array_equal(got[grp].astype(np.float64), np.float32(want).astype(np.float64)), (grp, int(blk[4 + grp]))
    # where the product needs no rounding the widened bank is the plain one
    rng = np.random.default_rng(2)
    raw = oracle.quantize(oracle.NVFP4G, (rng.standard_normal((4, 256)) * 0.02).astype(np.float32))
    plain, wide = oracle.dequantize(oracle.NVFP4G, raw, 1024), oracle.dequantize_nvfp4_widened(raw, 1024)
    assert (np.abs(wide - plain) <= np.abs(plain) * 2.0 ** -4 + 1e-7).all()   # four significant bits kept
    assert (wide != plain).mean() > 0.05   # and it is lossy


def _requant_e4m3(oracle, v):
    v = np.asarray(v, np.float32)
    m = np.float32(np.abs(v).max())
    if m == 0:
        return v.astype(np.float64)
    mul = np.float32(448) / m
    q = np.array([oracle.e4m3_to_float(oracle.float_to_e4m3(np.float32(t * mul))) for t in v], np.float64)
    return q * np.float64(np.float32(m / np.float32(448)))


def test_layer_forward_fp8_mode_against_float64(oracle):
    """act_mode 2 (the gate of the grouped fp8 products) rebuilt in float64 numpy from the pinned pieces: widened weights,
    per-row E4M3 on the token row, fp16 rounding of silu(g) * u, per-row E4M3 on the act row, the down product rounded to
    fp16. Leaving any one step out must land far from the oracle."""
    rng = np.random.default_rng(29)
    h, f, e, k, n, sf = 256, 256, 5, 2, 5, 128
    wtype = oracle.NVFP4G
    banks = [oracle.quantize(wtype, (rng.standard_normal(((e + 1) * r, c)) * 0.05).astype(np.float32)) for r, c in ((f, h), (f, h), (h, f))]
    wide = [oracle.dequantize_nvfp4_widened(b, (e + 1) * f * h).astype(np.float64) for b in banks]
    plain = [oracle.dequantize(wtype, b, (e + 1) * f * h).astype(np.float64) for b in banks]
    x = rng.standard_normal((n, h)).astype(np.float32)
    logits = rng.standard_normal((n, e + 1)).astype(np.float32)
    got, ids, w = oracle.layer_forward(x, logits, *banks, wtype, h, f, e, k, shared_ff=sf, act_mode=2, threads=3)

    def rebuild(skip=None):
        dec = plain if skip == "w" else wide
        wg, wu, wd = dec[0].reshape(e + 1, f, h), dec[1].reshape(e + 1, f, h), dec[2].reshape(e + 1, h, f)
        out = np.zeros((n, h))
        for t in range(n):
            xq = _requant_e4m3(oracle, x[t]) if skip != "x" else x[t].astype(np.float64)

            def ffn(j, ff):
                g, u = wg[j, :ff] @ xq, wu[j, :ff] @ xq
                act = g / (1 + np.exp(-g)) * u
                if skip != "act16":
                    act = _half(act)
                if skip != "act":
                    act = _requant_e4m3(oracle, act)
                y = wd[j, :, :ff] @ act
                return _half(y) if skip != "y16" else y

            out[t] = sum(float(w[t, s]) * ffn(ids[t, s], f) for s in range(k)) + 1 / (1 + np.exp(-float(logits[t, e]))) * ffn(e, sf)
        return out

    want = rebuild()
    tol = 2e-5 * max(1.0, np.abs(want).max())
    off = np.abs(got - want) > tol
    assert off.mean() < 0.02, off.mean()
    assert np.abs(got - want).max() < 2e-3 * np.abs(want).max()
    for skip in ("w", "x", "act", "act16", "y16"):
        assert (np.abs(got - rebuild(skip)) > tol).mean() > 0.3, skip
    # the act rows the layer can hand back: row (t, s) = fp16(silu(g) * u) of the slot's expert on the quantised token row, the
    # shared expert in the last slot with its first shared_ff values; same output as without them
    got2, ids2, w2, act = oracle.layer_forward(x, logits, *banks, wtype, h, f, e, k, shared_ff=sf, act_mode=2, threads=2, return_act=True)
    assert np.array_equal(got2, got) and act.shape == (n, k + 1, f)
    wg, wu = wide[0].reshape(e + 1, f, h), wide[1].reshape(e + 1, f, h)
    for t in range(n):
        xq = _requant_e4m3(oracle, x[t])
        for s in range(k + 1):
            j, ff = (ids[t, s], f) if s < k else (e, sf)
            g, u = wg[j, :ff] @ xq, wu[j, :ff] @ xq
            want_act = _half(g / (1 + np.exp(-g)) * u)
            step = np.maximum(np.abs(want_act) * 2.0 ** -10, 2.0 ** -24)        # one fp16 step: fp32 sums against float64 here
            assert (np.abs(act[t, s, :ff] - want_act) <= step).all() and (act[t, s, :ff] != want_act).mean() < 0.02
            assert not act[t, s, ff:].any()
    # banks of another format have no such mode
    with pytest.raises(Exception):
        oracle.layer_forward(x, logits, *banks, oracle.IQ4_XS, h, f, e, k, act_mode=2)


def test_layer_forward_lossy_operand_modes_against_float64(oracle):
    """act_mode 1 and 5 of tqo_layer_forward (the gates of the grouped int8 products) rebuilt step by step in float64
    numpy: per-row int8 on the token row, [mode 5: fp16 rounding of silu(g) * u], per-row int8 on the act row, the down
    product [mode 5: rounded to fp16], the weighted sum in fp32. The same rebuild with any one of those steps left out
    must be far from the oracle, so an oracle that skipped a step would fail."""
    rng = np.random.default_rng(23)
    h, f, e, k, n = 256, 256, 6, 2, 6
    for wtype, sf in ((oracle.IQ4_XS, 256), (oracle.Q4_K, 0), (oracle.IQ3_S, 256)):
        banks = [oracle.quantize(wtype, (rng.standard_normal(((e + 1) * r, c)) * 0.05).astype(np.float32))
                 for r, c in ((f, h), (f, h), (h, f))]
        dec = [oracle.dequantize(wtype, b, (e + 1) * f * h).astype(np.float64) for b in banks]
        wg, wu, wd = dec[0].reshape(e + 1, f, h), dec[1].reshape(e + 1, f, h), dec[2].reshape(e + 1, h, f)
        x = rng.standard_normal((n, h)).astype(np.float32)
        logits = rng.standard_normal((n, e + 1)).astype(np.float32)

        def rebuild(ids, w, mode, skip=None):
            out = np.zeros((n, h))
            for t in range(n):
                xq = _requant_i8(x[t]) if skip != "x" else x[t].astype(np.float64)

                def ffn(j, ff):
                    g, u = wg[j, :ff] @ xq, wu[j, :ff] @ xq
                    act = g / (1 + np.exp(-g)) * u
                    if mode == 5 and skip != "act16":
                        act = _half(act)
                    if skip != "act":
                        act = _requant_i8(act)
                    y = wd[j, :, :ff] @ act
                    return _half(y) if mode == 5 and skip != "y16" else y

                out[t] = sum(float(w[t, s]) * ffn(ids[t, s], f) for s in range(k))
                if sf:
                    out[t] += 1 / (1 + np.exp(-float(logits[t, e]))) * ffn(e, sf)
            return out

        for mode in (1, 5):
            got, ids, w = oracle.layer_forward(x, logits, *banks, wtype, h, f, e, k, shared_ff=sf, act_mode=mode, threads=3)
            ri, rw = oracle.route(logits[:, :e], k)
            assert np.array_equal(ids, ri) and np.array_equal(w, rw)
            want = rebuild(ids, w, mode)
            tol = 2e-5 * max(1.0, np.abs(want).max())
            # fp32 sums in the oracle against float64 here: a value on a rounding boundary of the int8 or fp16 steps may
            # fall the other way, so a few elements may be off by one such step; everything else agrees to fp32 accuracy
            off = np.abs(got - want) > tol
            assert off.mean() < 0.01, (wtype, mode, off.mean())
            assert np.abs(got - want).max() < 5e-4 * np.abs(want).max(), (wtype, mode)
            for skip in ("x", "act") + (("act16", "y16") if mode == 5 else ()):
                other = rebuild(ids, w, mode, skip)
                assert (np.abs(got - other) > tol).mean() > 0.3, (wtype, mode, skip)
        # the fp32 oracle is none of them either
        a, _, _ = oracle.layer_forward(x, logits, *banks, wtype, h, f, e, k, shared_ff=sf, act_mode=0, threads=1)
        assert (np.abs(a - want) > tol).mean() > 0.5


def test_layer_forward_swiglu_clamp_against_float64(oracle):
    """The swiglu_clamp / clamp_gate fields of tqo_layer_forward (MoeConfig::swiglu_clamp, moe_expert_ffn's switch:
    src/experts/moe.cpp:128-143) in the fp32 mode and in the int8 mode the grouped products are gated by, rebuilt in float64:
    up clamped to [-c, c]; clamp_gate: gate clamped to at most c before the activation; else silu(gate) clamped to at most c
    after it. The limit is set where it really bites; without the clamp, or with the other branch, the rebuild is far off."""
    rng = np.random.default_rng(29)
    h, f, e, k, n, sf = 256, 256, 5, 2, 5, 256
    wtype = oracle.IQ4_XS
    banks = [oracle.quantize(wtype, (rng.standard_normal(((e + 1) * r, c)) * 0.08).astype(np.float32)) for r, c in ((f, h), (f, h), (h, f))]
    dec = [oracle.dequantize(wtype, b, (e + 1) * f * h).astype(np.float64) for b in banks]
    wg, wu, wd = dec[0].reshape(e + 1, f, h), dec[1].reshape(e + 1, f, h), dec[2].reshape(e + 1, h, f)
    x = rng.standard_normal((n, h)).astype(np.float32)
    logits = rng.standard_normal((n, e + 1)).astype(np.float32)
    limit = 0.6
    g_all = np.abs(wg[0] @ x[0].astype(np.float64))
    assert (g_all > limit).mean() > 0.2                       # the limit cuts a fair share of the values

    def rebuild(ids, w, mode, clamp, gate_first):
        out = np.zeros((n, h))
        for t in range(n):
            xq = _requant_i8(x[t]) if mode == 5 else x[t].astype(np.float64)

            def ffn(j, ff):
                g, u = wg[j, :ff] @ xq, wu[j, :ff] @ xq
                if clamp:
                    u = np.clip(u, -limit, limit)
                    if gate_first:
                        g = np.minimum(g, limit)
                sl = g / (1 + np.exp(-g))
                if clamp and not gate_first:
                    sl = np.minimum(sl, limit)
                act = sl * u
                if mode == 5:
                    act = _requant_i8(_half(act))
                y = wd[j, :, :ff] @ act
                return _half(y) if mode == 5 else y

            out[t] = sum(float(w[t, s]) * ffn(ids[t, s], f) for s in range(k)) + 1 / (1 + np.exp(-float(logits[t, e]))) * ffn(e, sf)
        return out

    for mode in (0, 5):
        for gate_first in (False, True):
            got, ids, w = oracle.layer_forward(x, logits, *banks, wtype, h, f, e, k, shared_ff=sf, act_mode=mode, threads=2, swiglu_clamp=limit,
                                               clamp_gate=gate_first)
            want = rebuild(ids, w, mode, True, gate_first)
            tol = (2e-5 if mode == 0 else 5e-4) * max(1.0, np.abs(want).max())
            assert (np.abs(got - want) > tol).mean() < 0.01, (mode, gate_first)
            for other in (rebuild(ids, w, mode, False, gate_first), rebuild(ids, w, mode, True, not gate_first)):
                assert (np.abs(got - other) > tol).mean() > 0.3, (mode, gate_first)
    # a limit at or below 1e-6 is no clamp (the reference's `limit > eps` test)
    a, _, _ = oracle.layer_forward(x, logits, *banks, wtype, h, f, e, k, shared_ff=sf, threads=2, swiglu_clamp=1e-6, clamp_gate=True)
    b, _, _ = oracle.layer_forward(x, logits, *banks, wtype, h, f, e, k, shared_ff=sf, threads=2)
    assert np.array_equal(a, b)


def _requant_blocks_i8(v):
    """float64 restatement of the per-32-block int8 quantiser: _requant_i8 on every 32 values"""
    v = np.asarray(v, np.float64)
    return np.concatenate([_requant_i8(v[i:i + 32]) for i in range(0, v.size, 32)])


def test_block_quantiser_and_layer_mode(oracle):
    """tqo_quant_act_blocks_i8: every 32 values are the per-row quantiser's result on those 32 alone (pinned above), the
    sums are the integer sums of each half; an input that is a multiple of its block's scale survives exactly. act_mode 6
    of tqo_layer_forward rebuilt in float64 numpy as mode 5 with that quantiser; the rebuild with per-row scales, or with a
    step left out, must be far from it."""
    rng = np.random.default_rng(41)
    x = (rng.standard_normal(256) * np.repeat(rng.uniform(0.01, 50, 8), 32)).astype(np.float32)
    x[64:96] = 0
    q, s, qsum = oracle.quant_act_blocks_i8(x)
    for b in range(8):
        wq, ws = oracle.quant_act_row_i8(x[32 * b:32 * b + 32])
        assert np.array_equal(q[32 * b:32 * b + 32], wq) and s[b] == np.float32(ws)
        assert qsum[b, 0] == int(wq[:16].astype(np.int32).sum()) and qsum[b, 1] == int(wq[16:].astype(np.int32).sum())
    assert s[2] == 0 and not q[64:96].any()
    # the extreme sums fit int16 (16 * 127), and integers times a power of two come back exactly
    q1, s1, qs1 = oracle.quant_act_blocks_i8(np.full(32, -3.0, np.float32))
    assert (q1 == -127).all() and qs1[0, 0] == -2032 and qs1[0, 1] == -2032
    ints = rng.integers(-127, 128, 64).astype(np.float32)
    ints[0], ints[32] = 127, -127
    q2, s2, _ = oracle.quant_act_blocks_i8(ints * np.float32(0.25))
    assert np.array_equal(q2.astype(np.float32), ints) and (s2 == np.float32(0.25)).all()

    h, f, e, k, n = 256, 256, 6, 2, 6
    for wtype, sf in ((oracle.IQ4_XS, 256), (oracle.Q4_K, 0)):
        banks = [oracle.quantize(wtype, (rng.standard_normal(((e + 1) * r, c)) * 0.05).astype(np.float32))
                 for r, c in ((f, h), (f, h), (h, f))]
        dec = [oracle.dequantize(wtype, b, (e + 1) * f * h).astype(np.float64) for b in banks]
        wg, wu, wd = dec[0].reshape(e + 1, f, h), dec[1].reshape(e + 1, f, h), dec[2].reshape(e + 1, h, f)
        xs = (rng.standard_normal((n, h)) * np.repeat(rng.uniform(0.05, 4, (n, h // 32)), 32, axis=1)).astype(np.float32)
        logits = rng.standard_normal((n, e + 1)).astype(np.float32)
        got, ids, w = oracle.layer_forward(xs, logits, *banks, wtype, h, f, e, k, shared_ff=sf, act_mode=6, threads=3)

        def rebuild(skip=None):
            out = np.zeros((n, h))
            rq = _requant_i8 if skip == "rows" else _requant_blocks_i8
            for t in range(n):
                xq = rq(xs[t]) if skip != "x" else xs[t].astype(np.float64)

                def ffn(j, ff):
                    g, u = wg[j, :ff] @ xq, wu[j, :ff] @ xq
                    act = g / (1 + np.exp(-g)) * u
                    if skip != "act16":
                        act = _half(act)
                    if skip != "act":
                        act = rq(act)
                    y = wd[j, :, :ff] @ act
                    return _half(y) if skip != "y16" else y

                out[t] = sum(float(w[t, s]) * ffn(ids[t, s], f) for s in range(k))
                if sf:
                    out[t] += 1 / (1 + np.exp(-float(logits[t, e]))) * ffn(e, sf)
            return out

        want = rebuild()
        tol = 2e-5 * max(1.0, np.abs(want).max())
        off = np.abs(got - want) > tol
        # (eight times the quantiser's roundings per row: more values on a rounding boundary fall the other way in fp32)
        assert off.mean() < 0.08, (wtype, off.mean())
        assert np.abs(got - want).max() < 5e-4 * np.abs(want).max(), wtype
        for skip in ("rows", "x", "act", "act16", "y16"):
            assert (np.abs(got - rebuild(skip)) > tol).mean() > 0.3, (wtype, skip)


def test_cpu_baseline_kernels_agree_with_decode(oracle, ref):
    """The CPU-baseline matvecs, row by row, with the gates of the reference's tests/test_cpu_expert_matvec.cpp:117-118, 178-195:
    fp32 variant vs decode + float64 dot rms-rel <= 1e-5; int8 variant <= 1e-2; and the AVX2 integer dots against the scalar
    ones (the integer sums are exact on both sides, so they agree to fp32 rounding of the scale products). Then the two bench
    schemes' checksums against float64; the reference's own IQ4_NL kernels agree likewise."""
    rng = np.random.default_rng(19)
    rel = lambda y, want: np.sqrt(np.mean((y - want) ** 2) / np.mean(want ** 2))
    for wtype in (oracle.IQ4_XS, oracle.Q4_K, oracle.IQ3_S, oracle.IQ4_NL, oracle.NVFP4G):
        rows, cols = 96, 768 if wtype != oracle.NVFP4G else 640
        for raw in (oracle.random_blocks(wtype, rows, cols, rng),
                    oracle.quantize(wtype, (rng.standard_normal((rows, cols)) * 0.02).astype(np.float32))):
            x = rng.standard_normal(cols).astype(np.float32)
            want = oracle.dequantize(wtype, raw, rows * cols).reshape(rows, cols).astype(np.float64) @ x.astype(np.float64)
            y32, y8, y8s = (oracle.cpu_matvec(wtype, raw, rows, cols, x, mode) for mode in (0, 1, 2))
            assert rel(y32, want) < 1e-5, (wtype, rel(y32, want))
            assert rel(y8, want) < 1e-2, (wtype, rel(y8, want))
            assert np.abs(y8 - y8s).max() < 2e-6 * np.abs(want).max(), wtype
    h, f, ne = 512, 256, 2
    for wtype in (oracle.IQ4_XS, oracle.Q4_K, oracle.IQ3_S, oracle.IQ4_NL, oracle.NVFP4G):
        if wtype == oracle.NVFP4G:
            h, f = 640, 256
        banks = [oracle.quantize(wtype, (rng.standard_normal((ne * r, c)) * 0.02).astype(np.float32))
                 for r, c in ((f, h), (f, h), (h, f))]
        t0, c0 = oracle.cpu_expert_bench(wtype, *banks, h, f, ne, 2, False, reps=1)
        t1, c1 = oracle.cpu_expert_bench(wtype, *banks, h, f, ne, 2, True, reps=1)
        dec = [oracle.dequantize(wtype, b, ne * f * h).astype(np.float64) for b in banks]
        want, first = 0.0, None
        for e in range(ne):
            x = 0.5 + 0.001 * ((np.arange(h) + e) & 15)
            g, u = dec[0].reshape(ne, f, h)[e] @ x, dec[1].reshape(ne, f, h)[e] @ x
            y = (dec[2].reshape(ne, h, f)[e] @ (g / (1 + np.exp(-g)) * u)).sum()
            first = y if first is None else first
            want += y
        assert abs(c0 - want) < 1e-4 * max(1.0, abs(want)), (wtype, c0, want)
        assert abs(c1 - want) < 3e-2 * max(1.0, abs(want)), (wtype, c1, want)
        assert t0 > 0 and t1 > 0
        # one expert with its rows split over persistent workers: the same result whatever the number of workers
        one = [b[: b.size // ne] for b in banks]
        lat = [oracle.cpu_expert_latency(wtype, *one, h, f, nt, reps=2) for nt in (1, 3)]
        assert lat[0][1] == lat[1][1] and abs(lat[0][1] - first) < 3e-2 * max(1.0, abs(first)), (wtype, lat, first)
    # the reference's IQ4_NL kernels on the same blocks
    rows, cols = 64, 512
    raw = oracle.quantize(oracle.IQ4_NL, (rng.standard_normal((rows, cols)) * 0.02).astype(np.float32))
    x = np.float16(rng.standard_normal(cols)).astype(np.float32)
    wd = oracle.dequantize(oracle.IQ4_NL, raw, rows * cols).reshape(rows, cols).astype(np.float64)
    want = wd @ x.astype(np.float64)
    y = np.empty(rows, np.float32)
    p = lambda a: a.ctypes.data_as(C.c_void_p)
    ref.ref_iq4nl_matvec(1, p(raw), rows, cols, p(x), 1, p(y))
    assert np.array_equal(y, want.astype(np.float32))
    ref.ref_iq4nl_matvec(0, p(raw), rows, cols, p(x), 1, p(y))
    assert np.sqrt(np.mean((y - want) ** 2) / np.mean(want ** 2)) < 1e-5
    ref.ref_iq4nl_matvec(2, p(raw), rows, cols, p(x), 1, p(y))
    assert np.sqrt(np.mean((y - want) ** 2) / np.mean(want ** 2)) < 1e-2


def sequential_dedup_maps(ids, slot_of, topk, groups):
    """An independent build of the decode grouping maps: walk the assignments in order and keep, per bank slot, the group that
    is open and how many columns it has; a full group (8 columns) is closed and the next assignment of that slot opens a new
    one with the next free group number."""
    gu = np.full((groups, 18), -1, np.int32)
    dn = np.full((groups, 18), -1, np.int32)
    slots = np.array([slot_of[e] if e >= 0 else -1 for e in ids], np.int32)
    open_group, ng = {}, 0
    for a, s in enumerate(slots):
        if s < 0:
            continue
        g, used = open_group.get(int(s), (-1, 8))
        if used == 8:
            g, used = ng, 0
            ng += 1
            gu[g, 0] = dn[g, 0] = s
        gu[g, 1] = dn[g, 1] = used + 1
        gu[g, 2 + used], gu[g, 10 + used] = a // topk, a
        dn[g, 2 + used], dn[g, 10 + used] = a, a
        open_group[int(s)] = (g, used + 1)
    return slots, gu, dn


def test_dedup_maps_against_a_sequential_build_and_by_hand(oracle):
    """oracle.dedup_maps follows the reference's kernel (every assignment finds its group by itself); it must equal the
    sequential walk on random inputs (skipped assignments, crowded slots that fill several groups, slots that are not the
    expert numbers), and a case worked by hand."""
    # by hand: topk 2, tokens 0..4; expert 7 appears 9 times (a full group and a second one), expert 2 twice, one skipped
    ids = np.array([7, 2, 7, -1, 7, 7, 7, 2, 7, 7, 7, 7], np.int32)
    slot_of = np.arange(10, dtype=np.int32) + 100
    slots, gu, dn = oracle.dedup_maps(ids, slot_of, 2, len(ids))
    assert slots.tolist() == [107, 102, 107, -1, 107, 107, 107, 102, 107, 107, 107, 107]
    # groups in order of opening: slot 107 (assignments 0 2 4 5 6 8 9 10), slot 102 (1 7), slot 107 again (11)
    assert gu[0].tolist() == [107, 8, 0, 1, 2, 2, 3, 4, 4, 5, 0, 2, 4, 5, 6, 8, 9, 10]
    assert gu[1].tolist() == [102, 2, 0, 3, -1, -1, -1, -1, -1, -1, 1, 7, -1, -1, -1, -1, -1, -1]
    assert gu[2].tolist() == [107, 1, 5] + [-1] * 7 + [11] + [-1] * 7
    assert dn[0].tolist() == [107, 8, 0, 2, 4, 5, 6, 8, 9, 10, 0, 2, 4, 5, 6, 8, 9, 10]
    assert (gu[3:] == -1).all() and (dn[3:] == -1).all()
    rng = np.random.default_rng(3)
    for experts, n, topk in ((6, 40, 3), (64, 30, 8), (3, 100, 2), (500, 16, 10)):
        ids = rng.integers(-1, experts, n * topk).astype(np.int32)
        slot_of = rng.permutation(experts * 2)[:experts].astype(np.int32)
        got = oracle.dedup_maps(ids, slot_of, topk, len(ids) + 3)
        want = sequential_dedup_maps(ids, slot_of, topk, len(ids) + 3)
        for g, w in zip(got, want):
            assert np.array_equal(g, w)
    counts = np.array([5, 0, 1 << 40], np.int64)
    assert oracle.count(np.array([[0, 2, -1], [2, 2, 0]]), counts).tolist() == [7, 0, (1 << 40) + 3]
