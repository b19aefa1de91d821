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
    d = str(tmp_path)
    open(os.path.join(d, "meta.txt"), "w").write("%d %d %d %d %d %d %d\n" % (wtype, experts, rows, cols, n, topk, capacity))
    for name, arr in (("gate", banks[0]), ("up", banks[1]), ("x", x), ("ids", ids), ("counts", counts), ("groups", groups)):
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
    print("adapter %s: decode worst %.2e, grouped worst %.2e of sum |w x|; fused act max-abs %.2e" % (wtype_name, max(worst(yg, 0), worst(yu, 1)), worst(yd, 1), err.max()))
