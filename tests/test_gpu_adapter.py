"""The C++ adapter (include/tqmoe_adapter.hpp) as a drop-in behind the reference's WeightFormat interface: a C++ program
(tests/adapter_check.cpp) derives from a base class with the reference's expert virtuals, calls them by base pointer with
the reference's operands (fp16 rows, bf16 results, counts / groups / capacity lists) and this test compares what it
computed with float64 products of the oracle's decoded weights, at the bar of the reference's own test
(tests/nvfp4_expert.cu:108-118: error below 1 % of sum |w x|, i.e. bf16 output rounding plus accumulation)."""
import os
import subprocess

import numpy as np
import pytest
import torch

import build_adapter_check

pytestmark = pytest.mark.gpu


def bf16_to_f64(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)


@pytest.mark.parametrize("wtype_name", ["IQ4_XS", "Q4_K", "NVFP4G"])
def test_adapter_through_reference_signatures(oracle, tmp_path, wtype_name):
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    exe = build_adapter_check.EXE
    if not os.path.exists(exe):
        build_adapter_check.build()
    wtype = getattr(oracle, wtype_name)
    rng = np.random.default_rng(31)
    experts, rows, cols, n, topk = 5, 256, 512 if wtype != oracle.NVFP4G else 640, 70, 3
    A = n * topk
    banks = [oracle.quantize(wtype, (rng.standard_normal((experts * rows, cols)) * 0.02).astype(np.float32)) for _ in range(2)]
    x = rng.standard_normal((n, cols)).astype(np.float16)
    ids = np.stack([rng.permutation(experts)[:topk] for _ in range(n)]).astype(np.int32)
    ids[3, 1] = -1                                       # a skipped assignment: its rows stay untouched (zero here)
    # the reference's lists: counts and groups [experts][capacity], here in descending order inside each expert (the
    # device version of moe_group leaves them in no particular order)
    flat = ids.reshape(-1)
    counts = np.array([(flat == e).sum() for e in range(experts)], np.int32)
    capacity = int(counts.max()) + 2
    groups = np.full((experts, capacity), -1, np.int32)
    for e in range(experts):
        groups[e, : counts[e]] = np.flatnonzero(flat == e)[::-1]
    # the reference's activation quantiser (quant_act_rows_k, quant_u4h.inc:790-822) on the host: natural order, scales
    # [n][cols / 32], sums of q per 16 values; mode 1 a scale per block, mode 2 the token's scale in every entry
    xf32 = x.astype(np.float32)
    blocks = xf32.reshape(n, cols // 32, 32)
    m1 = np.abs(blocks).max(axis=2)
    xs1 = (m1 / np.float32(127)).astype(np.float32)
    inv1 = np.where(m1 > 0, np.float32(127) / np.where(m1 > 0, m1, 1), 0).astype(np.float32)
    xq1 = np.rint(blocks * inv1[:, :, None]).astype(np.int8)
    m2 = np.abs(xf32).max(axis=1)
    xs2 = np.repeat((m2 / np.float32(127)).astype(np.float32)[:, None], cols // 32, axis=1)
    xq2 = np.rint(xf32 * (np.float32(127) / m2)[:, None]).astype(np.int8)
    xsum = xq1.reshape(n, cols // 32, 2, 16).sum(axis=3).astype(np.int16)
    d = str(tmp_path)
    open(os.path.join(d, "meta.txt"), "w").write("%d %d %d %d %d %d %d\n" % (wtype, experts, rows, cols, n, topk, capacity))
    for name, arr in (("gate", banks[0]), ("up", banks[1]), ("x", x), ("ids", ids), ("counts", counts), ("groups", groups), ("xq1", xq1.reshape(n, cols)),
                      ("xq2", xq2), ("xs1", xs1), ("xs2", xs2), ("xsum", xsum)):
        np.ascontiguousarray(arr).tofile(os.path.join(d, name + ".bin"))
    run = subprocess.run([exe, d], capture_output=True, text=True, timeout=100)
    assert run.returncode == 0, (run.returncode, run.stdout, run.stderr)

    w = [oracle.dequantize(wtype, b, experts * rows * cols).reshape(experts, rows, cols).astype(np.float64) for b in banks]
    xf = x.astype(np.float64)
    want = [np.zeros((A, rows)) for _ in range(2)]
    mag = [np.zeros((A, rows)) for _ in range(2)]
    for a in range(A):
        if flat[a] < 0:
            continue
        for i in range(2):
            want[i][a] = w[i][flat[a]] @ xf[a // topk]
            mag[i][a] = np.abs(w[i][flat[a]]) @ np.abs(xf[a // topk])
    read = lambda name, dt: np.fromfile(os.path.join(d, name + ".bin"), dt).reshape(A, rows)
    yg, yu, y1, yd = (bf16_to_f64(read(name, np.uint16)) for name in ("yg", "yu", "y1", "yd"))
    act = read("act", np.float16).astype(np.float64)
    worst = lambda got, i: float((np.abs(got - want[i]) / (mag[i] + 1e-9)).max())
    listed = flat >= 0
    assert not yg[~listed].any() and not yd[~listed].any() and not act[~listed].any()      # untouched rows
    assert worst(yg, 0) < 1e-2 and worst(yu, 1) < 1e-2 and worst(y1, 0) < 1e-2, (worst(yg, 0), worst(yu, 1), worst(y1, 0))
    assert worst(yd, 1) < 1e-2, worst(yd, 1)                                               # expert_gemm on the up bank
    g, u = want
    want_act = g / (1 + np.exp(-g)) * u
    err = np.abs(act - want_act)[listed]
    assert err.max() < 1e-2 * max(1.0, np.abs(want_act).max()) and np.sqrt(np.mean(err ** 2) / np.mean(want_act[listed] ** 2)) < 5e-3
    # the products over the decode grouping maps give the rows of the products over the ids (the same kernels; the waves may
    # split a row's sum differently for another number of assignments, so to fp32 rounding: at most one bf16 step)
    dg, du, dg1 = (bf16_to_f64(read(name, np.uint16)) for name in ("dg", "du", "dg1"))
    for got, ref in ((dg, yg), (du, yu), (dg1, yg)):
        assert np.abs(got - ref).max() <= 2.0 ** -7 * np.abs(ref).max() and (got != ref).mean() < 0.01 and not got[~listed].any()
    # moe_group with the reference's seven arguments: counts and ascending lists [experts][n]
    mc = np.fromfile(os.path.join(d, "mg_counts.bin"), np.int32)
    mg = np.fromfile(os.path.join(d, "mg_groups.bin"), np.int32).reshape(experts, n)
    assert np.array_equal(mc, counts)
    for e in range(experts):
        assert np.array_equal(mg[e, : counts[e]], np.flatnonzero(flat == e)) and (mg[e, counts[e]:] == -1).all()
    # a capacity of 3 below the counts: exactly the first three listed assignments of every expert have rows, equal to the full run's
    ycap = bf16_to_f64(read("ycap", np.uint16))
    kept = np.zeros(A, bool)
    for e in range(experts):
        kept[groups[e, :3]] = True
    assert counts.max() > 3 and np.array_equal(ycap[kept], yd[kept]) and not ycap[~kept].any()
    # the int8 grouped product on the reference's operands, against float64 on the decoded weights and the dequantised rows
    if os.path.exists(os.path.join(d, "yi1.bin")):
        assert wtype != oracle.NVFP4G
        yi1, yi2 = bf16_to_f64(read("yi1", np.uint16)), bf16_to_f64(read("yi2", np.uint16))
        deq1 = (xq1.astype(np.float64) * xs1.astype(np.float64)[:, :, None]).reshape(n, cols)
        deq2 = xq2.astype(np.float64) * xs2[:, :1].astype(np.float64)
        for got, deq, label in ((yi1, deq1, "mode 1"), (yi2, deq2, "mode 2")):
            want_i = np.zeros((A, rows))
            mag_i = np.zeros((A, rows))
            for a in range(A):
                if flat[a] >= 0:
                    want_i[a] = w[1][flat[a]] @ deq[a // topk]
                    mag_i[a] = np.abs(w[1][flat[a]]) @ np.abs(deq[a // topk])
            wi = float((np.abs(got - want_i) / (mag_i + 1e-9)).max())
            assert not got[~listed].any() and wi < 1e-2, (label, wi)
            print("adapter %s: expert_gemm_i8 %s worst %.2e of sum |w x| (bf16 rows)" % (wtype_name, label, wi))
    else:
        assert wtype == oracle.NVFP4G          # `false`: no int8 kernel for this format, the engine falls back
    print("adapter %s: decode worst %.2e, grouped worst %.2e of sum |w x|; fused act max-abs %.2e" % (wtype_name, max(worst(yg, 0), worst(yu, 1)), worst(yd, 1), err.max()))
