"""The step either side of the layer: residual add + RMS norm in front (the reference's add_sumsq + norm_h,
qwen35_forward.cpp:1114-1115) and the residual add behind the combine (qwen35_forward.cpp:1248-1250). CPU tests pin the
oracle against float64 numpy and closed forms; GPU tests compare the library with the oracle."""
import numpy as np
import pytest


def bf16(a):
    import oracle
    return oracle.to_bf16(np.asarray(a, np.float32))


def test_oracle_add_rmsnorm_against_float64(oracle):
    rng = np.random.default_rng(31)
    for h, n in ((256, 3), (2048, 5), (4096, 2)):
        mb, mv = oracle.to_bf16(rng.standard_normal((n, h)).astype(np.float32) * 3)
        rb, rv = oracle.to_bf16(rng.standard_normal((n, h)).astype(np.float32))
        w = rng.uniform(0.5, 1.5, h).astype(np.float32)
        rows, normed = oracle.add_rmsnorm(mb, rb, w, 1e-6)
        sb, sv = oracle.to_bf16(mv + rv)                       # one fp32 add of two bf16 values, rounded once
        assert np.array_equal(rows, sb)
        s64 = sv.astype(np.float64)
        want = s64 / np.sqrt((s64 ** 2).mean(axis=1, keepdims=True) + 1e-6) * w
        got = oracle.from_bf16(normed).astype(np.float64)
        assert np.abs(got - want).max() <= np.abs(want).max() * 2.0 ** -8     # half a bf16 step plus the fp32 sum's error
        assert (np.abs(got - want) <= np.abs(want) * 2.0 ** -8 + 1e-30).all()
        # without a residual the rows stay as they are
        rows2, normed2 = oracle.add_rmsnorm(sb, None, w, 1e-6)
        assert np.array_equal(rows2, sb) and np.array_equal(normed2, normed)


def test_oracle_add_rmsnorm_closed_forms(oracle):
    h = 512
    w = np.full(h, 2.0, np.float32)
    # a constant row c: normed = c / sqrt(c^2 + eps) * w, here exactly representable
    cb, _ = oracle.to_bf16(np.full((1, h), 4.0, np.float32))
    _, normed = oracle.add_rmsnorm(cb, None, w, 0.0)
    assert (oracle.from_bf16(normed) == 2.0).all()
    # zero rows: 0 * (1 / sqrt(eps)) = 0, no NaN
    zb, _ = oracle.to_bf16(np.zeros((2, h), np.float32))
    rows, normed = oracle.add_rmsnorm(zb, zb, w, 1e-6)
    assert not rows.any() and not normed.any()
    # eps far above the mean square: normed = x / sqrt(eps) * w
    xb, xv = oracle.to_bf16(np.linspace(-1, 1, h, dtype=np.float32).reshape(1, h) * 1e-3)
    _, normed = oracle.add_rmsnorm(xb, None, np.ones(h, np.float32), 1e4)
    want = xv.astype(np.float64) / np.sqrt((xv.astype(np.float64) ** 2).mean() + 1e4)
    assert np.abs(oracle.from_bf16(normed) - want).max() <= np.abs(want).max() * 2.0 ** -8
    # residual that cancels the row
    ab, av = oracle.to_bf16(np.arange(h, dtype=np.float32).reshape(1, h))
    nb, _ = oracle.to_bf16(-av)
    rows, normed = oracle.add_rmsnorm(ab, nb, w, 1e-6)
    assert not rows.any() and not (normed & 0x7FFF).any()
    with pytest.raises(ValueError):
        oracle.add_rmsnorm(np.zeros((1, 100), np.uint16), None, np.ones(100, np.float32), 1e-6)


@pytest.fixture(scope="module")
def tq():
    import tqllm_amd
    return tqllm_amd


def _dev_bf16(bits):
    import torch
    return torch.from_numpy(bits.view(np.int16).copy()).cuda().view(torch.bfloat16)


def _bits(t):
    import torch
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


@pytest.mark.gpu
@pytest.mark.parametrize("h,n", [(2048, 4096), (512, 7), (1024, 33), (4096, 5), (768, 9), (256, 1)])
@pytest.mark.parametrize("with_residual", [True, False])
def test_add_rmsnorm_matches_oracle(tq, oracle, h, n, with_residual):
    import torch
    rng = np.random.default_rng(h + n)
    mb, _ = oracle.to_bf16(rng.standard_normal((n, h)).astype(np.float32) * rng.uniform(0.1, 8, (n, 1)).astype(np.float32))
    rb, _ = oracle.to_bf16(rng.standard_normal((n, h)).astype(np.float32))
    w = rng.uniform(0.5, 1.5, h).astype(np.float32)
    want_rows, want = oracle.add_rmsnorm(mb, rb if with_residual else None, w, 1e-6)
    for out_dtype in (torch.bfloat16, torch.float16):
        rows = _dev_bf16(mb)
        normed = tq.add_rmsnorm(rows, _dev_bf16(rb) if with_residual else None, torch.from_numpy(w).cuda(), 1e-6, out_dtype)
        assert np.array_equal(_bits(rows), want_rows)                    # the residual stream: bit for bit
        got = normed.float().cpu().numpy()
        ref = oracle.from_bf16(want)
        if out_dtype == torch.bfloat16:
            # the sum of squares is taken in another order and the reciprocal root is the device's: a value on a rounding
            # boundary may land one bf16 step away
            gb = _bits(normed).astype(np.int32)
            step = np.abs(gb - want.astype(np.int32))
            assert step.max() <= 1 and (step == 0).mean() > 0.995, (int(step.max()), float((step == 0).mean()))
        else:
            assert np.abs(got - ref).max() <= np.abs(ref).max() * 2.0 ** -7   # fp16 holds the bf16-rounded value exactly in this range


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_combine_residual_bit_exact(tq, oracle, dtype):
    import torch
    rng = np.random.default_rng(41)
    n, k, h = 37, 6, 512
    routed = rng.standard_normal((n, k, h)).astype(np.float32)
    shared = rng.standard_normal((n, h)).astype(np.float32)
    if dtype == "f16":
        routed, shared = routed.astype(np.float16).astype(np.float32), shared.astype(np.float16).astype(np.float32)
    w = rng.uniform(0, 1, (n, k)).astype(np.float32)
    sw = rng.uniform(0, 1, n).astype(np.float32)
    rb, rv = oracle.to_bf16(rng.standard_normal((n, h)).astype(np.float32) * 4)
    td = torch.float16 if dtype == "f16" else torch.float32
    plain = tq.moe_combine(torch.from_numpy(routed).cuda().to(td).float().reshape(n * k, h), torch.from_numpy(shared).cuda().to(td).float(), torch.from_numpy(w).cuda(),
                           torch.from_numpy(sw).cuda()).cpu().numpy()
    got = tq.moe_combine_residual(torch.from_numpy(routed).cuda().to(td), torch.from_numpy(shared).cuda().to(td), torch.from_numpy(w).cuda(),
                                  torch.from_numpy(sw).cuda(), _dev_bf16(rb))
    _, sum_bf16 = oracle.to_bf16(plain)                  # the library's own fp32 sum (checked against the oracle elsewhere), rounded as moe_sum stores it
    want, _ = oracle.to_bf16(sum_bf16 + rv)              # then the residual, rounded again
    assert np.array_equal(_bits(got), want)
    # in place: the residual buffer is the output
    buf = _dev_bf16(rb)
    tq.moe_combine_residual(torch.from_numpy(routed).cuda().to(td), torch.from_numpy(shared).cuda().to(td), torch.from_numpy(w).cuda(),
                            torch.from_numpy(sw).cuda(), buf, out=buf)
    assert np.array_equal(_bits(buf), want)


@pytest.mark.gpu
@pytest.mark.parametrize("n", [3, 200])
def test_layer_with_residual_equals_layer_plus_add(tq, oracle, n):
    import torch
    import synth
    from gpu_util import banks_on_device, dev
    cfg = synth.small(synth.CONFIGS["c2"], 512, 256, 12, 4)
    raws = synth.make_banks(cfg, seed=71)
    gate, up, down = banks_on_device(cfg, raws)
    inp = synth.make_inputs(cfg, n, seed=72)
    layer = tq.MoeLayer(dev(inp["router"]), dev(inp["shared_gate"]), gate, up, down, cfg["topk"], shared_ff=cfg["shared_ff"])
    rb, rv = oracle.to_bf16(np.random.default_rng(73).standard_normal((n, cfg["hidden"])).astype(np.float32))
    plain = layer.forward(dev(inp["x"])).cpu().numpy()                                   # fp32 sums
    got = layer.forward(dev(inp["x"]), residual=_dev_bf16(rb))
    assert got.dtype == torch.bfloat16
    _, s = oracle.to_bf16(plain)
    want, _ = oracle.to_bf16(s + rv)
    assert np.array_equal(_bits(got), want)
