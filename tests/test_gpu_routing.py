"""GPU parity, through the C ABI: router logits, softmax top-k and the dispatch permutation against the CPU oracle.
Bars: logits within 3e-6 (the reference's own gate, tests/moe_device.cu:45-72); ids bit-exact and weights within 3e-6
against the oracle's routing of the device's own logits; counts, offsets and permutation bit-exact."""
import numpy as np
import pytest
import torch

import synth
from gpu_util import clear_tokens, clear_tokens_gated, dev, oracle_type

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tq():
    import tqllm_amd
    return tqllm_amd


@pytest.mark.parametrize("name,n", [("c1", 1), ("c1", 16), ("c2", 1), ("c2", 4), ("c2", 16), ("c4", 64), ("c5", 33)])
def test_router_logits(tq, oracle, name, n):
    cfg = synth.CONFIGS[name]
    inp = synth.make_inputs(cfg, n, seed=1000 + n)
    logits = tq.moe_router(dev(inp["router"]), dev(inp["shared_gate"]), dev(inp["x"])).cpu().numpy()
    want = oracle.router_logits(inp["router"][0], oracle_type(cfg["rtype"]), inp["shared_gate"][0], inp["x"][0], oracle_type(cfg["xtype"]),
                                cfg["hidden"], cfg["experts"], n)
    assert logits.shape == (n, cfg["experts"] + 1)
    # against the exact (float64) product of the stored values: the reference's 3e-6 gate; against the oracle's
    # column-order fp32 sum the distance is that sum's own rounding (a few 1e-6 at 2048 terms)
    exact = inp["x"][1].astype(np.float64) @ np.vstack([inp["router"][1], inp["shared_gate"][1]]).astype(np.float64).T
    assert np.abs(logits - exact).max() < 3e-6
    assert np.abs(logits - want).max() < 2e-5


@pytest.mark.parametrize("n,e,h,shared", [(32, 512, 2048, True), (100, 33, 512, False), (4096, 512, 2048, True), (77, 64, 192, True),
                                          (250, 600, 512, False), (1000, 130, 192, True), (9000, 1100, 256, True),
                                          (2100, 64, 320, True), (4096, 100, 2048, False)])   # few router rows: eight waves a block
def test_router_gemm_path(tq, oracle, n, e, h, shared):
    """bf16 router rows and bf16 inputs take the matrix-pipe kernel from about 120,000 tokens x rows (64-token blocks, 128-token
    blocks for the largest grids), the wave-per-row kernel below: same logits to the same bar, ragged token and row counts,
    with and without the shared-gate row; on the matrix-pipe kernel the rows of a large batch equal those of a smaller one."""
    rng = np.random.default_rng(n + e)
    wb, wv = oracle.to_bf16((rng.standard_normal((e, h)) * 0.02).astype(np.float32))
    gb, gv = oracle.to_bf16((rng.standard_normal(h) * 0.02).astype(np.float32))
    xb, xv = oracle.to_bf16(rng.standard_normal((n, h)).astype(np.float32))
    x = dev((xb, xv))
    logits = tq.moe_router(dev((wb, wv)), dev((gb, gv)) if shared else None, x)
    got = logits.cpu().numpy()
    exact = xv.astype(np.float64) @ np.vstack([wv, gv if shared else np.zeros_like(gv)]).astype(np.float64).T
    assert got.shape == (n, e + 1)
    # fp32 accumulation of up to 2048 exact products: a few ulps of the largest logits (|logit| up to ~5) over 2 million samples
    assert np.abs(got - exact).max() < 3e-6 * max(1.0, np.abs(exact).max() / 2)
    if not shared:
        assert not got[:, e].any()
    m = -(-130000 // (e + 1))
    if n >= m + 5:     # both calls on the matrix-pipe kernel: a row's sum does not depend on the batch around it
        part = tq.moe_router(dev((wb, wv)), dev((gb, gv)) if shared else None, x[5:5 + m].contiguous())
        assert torch.equal(part, logits[5:5 + m])


@pytest.mark.parametrize("n,e,h,shared", [(4096, 64, 2048, False), (3000, 130, 192, True), (2100, 64, 320, True), (1000, 64, 2048, False)])
def test_router_gemm_path_f32(tq, oracle, n, e, h, shared):
    """fp32 router rows and fp32 inputs take the matrix-pipe kernel from the same size on (the last case stays on the
    wave-per-row kernel): fp32 products and sums, ragged shapes, with and without the shared-gate row."""
    rng = np.random.default_rng(n + e + h)
    w = (rng.standard_normal((e, h)) * 0.02).astype(np.float32)
    gate = (rng.standard_normal(h) * 0.02).astype(np.float32)
    xv = rng.standard_normal((n, h)).astype(np.float32)
    x = dev(xv)
    logits = tq.moe_router(dev(w), dev(gate) if shared else None, x)
    got = logits.cpu().numpy()
    exact = xv.astype(np.float64) @ np.vstack([w, gate if shared else np.zeros_like(gate)]).astype(np.float64).T
    assert got.shape == (n, e + 1)
    assert np.abs(got - exact).max() < 3e-6 * max(1.0, np.abs(exact).max() / 2)
    if not shared:
        assert not got[:, e].any()
    m = -(-130000 // (e + 1))
    if n >= m + 5:
        part = tq.moe_router(dev(w), dev(gate) if shared else None, x[5:5 + m].contiguous())
        assert torch.equal(part, logits[5:5 + m])


def test_router_without_shared_gate_and_f16(tq, oracle):
    rng = np.random.default_rng(5)
    h, e, n = 512, 33, 7
    w = (rng.standard_normal((e, h)) * 0.02).astype(np.float32)
    x = rng.standard_normal((n, h)).astype(np.float16)
    logits = tq.moe_router(dev(w), None, dev(x)).cpu().numpy()
    want = oracle.router_logits(w, oracle.F32, None, x.view(np.uint16), oracle.F16, h, e, n)
    assert np.abs(logits - want).max() < 3e-6 and not logits[:, e].any()


@pytest.mark.parametrize("e,k,n", [(64, 8, 16), (512, 10, 16), (512, 10, 4096), (256, 8, 512), (4096, 6, 3), (5, 5, 2), (1000, 1, 9)])
def test_topk_matches_oracle_on_device_logits(tq, oracle, e, k, n):
    rng = np.random.default_rng(e * 7 + k)
    logits = rng.standard_normal((n, e + 1)).astype(np.float32)
    ids, w, sw = (t.cpu().numpy() for t in tq.moe_topk(dev(logits), e, k))
    want_ids, want_w = oracle.route(logits[:, :e], k)
    clear = clear_tokens(oracle, logits, e, k, ids, want_ids)
    assert np.array_equal(ids[clear], want_ids[clear])
    same = (ids == want_ids).all(axis=1)
    assert np.abs(w[same] - want_w[same]).max() < 3e-6
    assert np.abs(w.sum(axis=1) - 1).max() < 1e-5
    want_sw = np.array([oracle.shared_weight(v) for v in logits[:, e]], np.float32)
    assert np.abs(sw - want_sw).max() < 3e-6


@pytest.mark.parametrize("e,k,n", [(64, 8, 16), (512, 10, 300), (1000, 6, 9)])
def test_topk2_equals_two_calls(tq, oracle, e, k, n):
    """The reference's moe_topk2 (moe_kernels.cuh:24-25): two routings in one launch, the same bits as two launches; more
    than 1024 experts are refused as there."""
    rng = np.random.default_rng(e + k + n)
    a, b = (dev(rng.standard_normal((n, e + 1)).astype(np.float32)) for _ in range(2))
    first, second = tq.moe_topk2(a, b, e, k, scale=1.5)
    for got, logits in ((first, a), (second, b)):
        want = tq.moe_topk(logits, e, k, scale=1.5)
        for g, w in zip(got, want):
            assert torch.equal(g, w)
    with pytest.raises(tq.TqmoeError):
        big = dev(np.zeros((2, 1026), np.float32))
        tq.moe_topk2(big, big, 1025, 2)


def test_topk_ties_extremes_and_scale(tq, oracle):
    e, k = 96, 6
    rows = [np.full(e, 0.5, np.float32),                                   # all equal: lowest indices
            np.where(np.arange(e) % 7 == 0, 3.0, -2.0).astype(np.float32),  # many exact ties at the top
            np.linspace(-300, 80, e).astype(np.float32),                    # exp underflow to exact zeros
            np.full(e, -1e4, np.float32)]
    rows[3][10] = 5.0
    logits = np.concatenate([np.stack(rows), np.zeros((4, 1), np.float32)], axis=1)
    for scale in (1.0, 0.0, 2.5):
        ids, w, _ = (t.cpu().numpy() for t in tq.moe_topk(dev(logits), e, k, scale))
        want_ids, want_w = oracle.route(logits[:, :e], k, scale=scale)
        assert np.array_equal(ids, want_ids)
        assert np.abs(w - want_w).max() < 3e-6 * max(1.0, scale)
    assert ids[0].tolist() == list(range(k)) and ids[3][0] == 10


@pytest.mark.parametrize("gating", [1, 2, 3, 4])
@pytest.mark.parametrize("e,k,n", [(256, 8, 64), (512, 10, 16), (64, 6, 33), (1500, 4, 20), (160, 70, 24), (5, 5, 12)])
def test_topk_gated_matches_oracle(tq, oracle, gating, e, k, n):
    rng = np.random.default_rng(e * 11 + k + gating)
    logits = (rng.standard_normal((n, e + 1)) * 2).astype(np.float32)
    for biased in (False, True):
        for norm in (True, False):
            for scale in (1.0, 2.5):
                if gating == 1 and not biased and norm:
                    continue                 # the plain entry point's case, tested above
                bias = rng.uniform(-0.5, 0.5, e).astype(np.float32) if biased else None
                ids, w, sw = (t.cpu().numpy() for t in tq.moe_topk(dev(logits), e, k, scale, gating=gating, bias=dev(bias) if biased else None,
                                                                   norm=norm))
                want_ids, want_w = oracle.route(logits[:, :e], k, gating, norm, scale, bias)
                # exempt: at most one token per case (18 of the 5070 tokens of all the cases here); no other token may differ
                clear = clear_tokens_gated(logits, e, k, gating, bias, ids, want_ids, "%d experts top-%d, bias %s norm %s" % (e, k, biased, norm), most=1)
                same = (ids == want_ids).all(axis=1)
                assert np.array_equal(ids[clear], want_ids[clear])
                assert np.abs(w[same] - want_w[same]).max() < 4e-6 * max(1.0, float(np.abs(want_w).max()))
                want_sw = np.array([oracle.shared_weight(x) for x in logits[:, e]], np.float32)
                assert np.abs(sw - want_sw).max() < 3e-6


def test_topk_gated_closed_forms(tq, oracle):
    """The cases of the reference's tests/moe.cpp:149-236 on the device: a bias moves the choice and not the weight, equal
    values go to the lower index, underflowing sigmoids stay finite, scale 0 and 1 mean none."""
    lg = np.array([[2, 1, 0, -1, 0.0]], np.float32)
    ids, w, _ = (t.cpu().numpy() for t in tq.moe_topk(dev(lg), 4, 2, gating=2, bias=dev(np.array([0, 0, 0, 100], np.float32)), norm=False))
    assert ids[0].tolist() == [3, 0] and abs(w[0, 0] - 1 / (1 + np.exp(1.0))) < 1e-6
    ids, w, _ = (t.cpu().numpy() for t in tq.moe_topk(dev(np.full((1, 9), 0.5, np.float32)), 8, 3, gating=2, norm=False))
    assert ids[0].tolist() == [0, 1, 2] and np.abs(w - 1 / (1 + np.exp(-0.5))).max() < 1e-6
    ids, w, _ = (t.cpu().numpy() for t in tq.moe_topk(dev(np.array([[-200, -300, -400, -500, 0]], np.float32)), 4, 4, gating=2, norm=True))
    assert np.isfinite(w).all() and not w.any() and ids[0].tolist() == [0, 1, 2, 3]
    lg = np.array([[3, 1, -1, -3, 0]], np.float32)
    w0, w1, w2 = (tq.moe_topk(dev(lg), 4, 2, s, gating=2)[1].cpu().numpy() for s in (0.0, 1.0, 2.5))
    assert np.array_equal(w0, w1) and abs(w1.sum() - 1) < 1e-6 and np.abs(w2 - 2.5 * w1).max() < 1e-6
    # selected-softmax: chosen by logit, weighted by a softmax over the chosen ones
    ids, w, _ = (t.cpu().numpy() for t in tq.moe_topk(dev(np.array([[1, 3, 2, -5, 0]], np.float32)), 4, 2, gating=3, norm=False))
    assert ids[0].tolist() == [1, 2] and np.abs(w[0] - np.array([np.e, 1]) / (np.e + 1)).max() < 1e-6
    with pytest.raises(tq.TqmoeError):
        tq.moe_topk(dev(lg), 4, 2, gating=7)


@pytest.mark.parametrize("e,n,k", [(64, 1, 8), (512, 16, 10), (512, 4096, 10), (256, 8192, 9), (7, 300, 3), (4096, 700, 2), (512, 102, 10)])
def test_dispatch_bit_exact(tq, oracle, e, n, k):
    rng = np.random.default_rng(n + e)
    if e == 512 and n == 4096:   # skewed load: Zipf(1.1) popularity, as the prefill config
        p = 1.0 / np.arange(1, e + 1) ** 1.1
        ids = rng.choice(e, size=(n, k), p=p / p.sum()).astype(np.int32)
    else:
        ids = rng.integers(0, e, (n, k)).astype(np.int32)
    if n == 300:
        ids[rng.random((n, k)) < 0.2] = -1          # skipped assignments
    want_c, want_o, want_p = oracle.dispatch(ids, e)
    cap = int(want_c.max()) if want_c.max() else 1
    counts, offsets, perm, groups = (t.cpu().numpy() for t in tq.moe_dispatch(dev(ids), e, capacity=cap))
    assert np.array_equal(counts, want_c) and np.array_equal(offsets, want_o) and np.array_equal(perm, want_p)
    for x in range(e):
        assert np.array_equal(groups[x, :counts[x]], want_p[want_o[x]:want_o[x + 1]])
        assert (groups[x, counts[x]:] == -1).all()
    assert counts.sum() == (ids >= 0).sum()


def test_dispatch_is_deterministic_and_truncates_groups(tq, oracle):
    rng = np.random.default_rng(9)
    ids = rng.integers(0, 32, (2000, 4)).astype(np.int32)
    a = [t.cpu().numpy() for t in tq.moe_dispatch(dev(ids), 32, capacity=16)]
    b = [t.cpu().numpy() for t in tq.moe_dispatch(dev(ids), 32, capacity=16)]
    for u, v in zip(a, b):
        assert np.array_equal(u, v)
    want_c, want_o, want_p = oracle.dispatch(ids, 32)
    assert np.array_equal(a[0], want_c)
    for x in range(32):
        assert np.array_equal(a[3][x], want_p[want_o[x]:want_o[x] + 16])


def test_errors_are_reported(tq):
    with pytest.raises(tq.TqmoeError):
        tq.moe_topk(torch.zeros((2, 9), device="cuda"), 8, 9)
    with pytest.raises(tq.TqmoeError):
        tq.moe_router(torch.zeros((4, 12), device="cuda"), None, torch.zeros((1, 12), device="cuda"))
    with pytest.raises(tq.TqmoeError):
        tq.moe_router(torch.zeros((4, 16)), None, torch.zeros((1, 16)))      # host tensors: no CPU path
