"""GPU parity of the NVFP4 layer (fp8 grouped products) at the stated tolerance, stage by stage, at configuration 5's shape.

The whole fp8 layer is gated at rel-RMS 3e-3 against its own-operand oracle (tests/test_gpu_prefill.py) because E4M3 keeps
four significant bits: an act value that the device and the oracle compute one fp16 step apart can land on two different
E4M3 codes, 6 to 12 % apart. These tests show that this is the whole excess over the 1e-3 bar:
  * the down product and the combine, fed the device's own fp16 act rows, equal oracle mode 2 on those rows at
    max-abs 1e-2 / rel-RMS 1e-3 (nothing but the straddling act values separates the two sides behind the act rows);
  * end to end, the act values whose two sides fall on different E4M3 codes are counted, and the output difference they
    account for (float64, from the pinned decoders) is taken out: what is left is below 1e-3.
The oracle pieces used (tqo_quant_act_row_e4m3, tqo_dequantize_nvfp4_widened, mode 2 and its act rows) are pinned on the CPU
by tests/test_oracle_moe.py::test_layer_forward_fp8_mode_against_float64 and ::test_declared_quantisers."""
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


def half(a):
    return np.asarray(a, np.float64).astype(np.float16).astype(np.float64)


def e4m3_rows(oracle, rows):
    """per-row E4M3 codes, scales and dequantised values (float64) of fp32 rows, by the oracle's pinned quantiser"""
    table = np.array([oracle.e4m3_to_float(c) for c in range(256)], np.float64)
    codes = np.empty(rows.shape, np.uint8)
    scales = np.empty(len(rows), np.float32)
    for i, r in enumerate(rows):
        codes[i], scales[i] = oracle.quant_act_row_e4m3(np.ascontiguousarray(r, np.float32))
    return codes, scales, table[codes] * scales.astype(np.float64)[:, None]


def setup(tq, oracle, n, seed):
    cfg = synth.CONFIGS["c5"]
    raws = synth.make_banks(cfg, seed=seed, distinct=3)
    gate, up, down = banks_on_device(cfg, raws)
    inp = synth.make_inputs(cfg, n, seed=seed + 1)
    layer = tq.MoeLayer(dev(inp["router"]), dev(inp["shared_gate"]), gate, up, down, cfg["topk"], shared_ff=cfg["shared_ff"])
    assert layer.path(n) == "grouped_fp8"
    return cfg, raws, (gate, up, down), inp, layer


def widened_down(oracle, cfg, raw_down, ids):
    """(expert, its down matrix as the fp8 product reads it: widened to E4M3, times 8 x global; its (token, slot) pairs) for
    every expert of ids [tokens][slots], one matrix in memory at a time"""
    h, f = cfg["hidden"], cfg["ff"]
    elems, nbytes = oracle.BLOCK[cfg["wtype"]]
    per = h * f // elems * nbytes
    for e in np.unique(ids):
        wd = oracle.dequantize_nvfp4_widened(raw_down[int(e) * per:(int(e) + 1) * per], h * f).reshape(h, f).astype(np.float64)
        yield int(e), wd, np.argwhere(ids == e)


def modular_forward(tq, cfg, banks, x, ids_ext, weights, shared_w):
    """The layer's fp8 stages through the modular entry points on the device's routing: (act fp16 [n * slots][ff], out fp32
    [n][hidden])."""
    gate, up, down = banks
    n, slots = ids_ext.shape
    k = cfg["topk"]
    counts, offsets, perm, _ = tq.moe_dispatch(ids_ext, cfg["experts"] + 1)
    lists = (counts, offsets, perm)
    rq, rs = tq.quant_rows_fp8(x)
    xq, xs = tq.gather_rows_i8(rq, rs, lists, n * slots, slots)
    act = tq.expert_gemm_gateup_fp8(gate, up, xq, xs, lists, n, slots, k, cfg["shared_ff"])
    aq, a_s = tq.group_rows_fp8(act, lists, n * slots, 1)
    y = tq.expert_gemm_fp8(down, aq, a_s, lists, n, slots, k, cfg["shared_ff"])
    out = tq.moe_combine_strided(y.view(n, slots, cfg["hidden"]), slots, weights, shared_w)
    return act, out


def test_fp8_down_and_combine_on_the_device_act_rows(tq, oracle):
    """Configuration 5's shape, 320 tokens: the device's own fp16 act rows (gate / up product with SwiGLU through the modular
    entry points) go through oracle mode 2's second half on the host (per-row E4M3 of the act row, widened down weights,
    fp16 result rows, slot-ordered weighted sum with the shared row) and must equal the device's down + combine at
    max-abs 1e-2 / rel-RMS 1e-3; the fused layer gives the same rows as the modular sequence."""
    n, head = 320, 40
    cfg, raws, banks, inp, layer = setup(tq, oracle, n, seed=520)
    x = dev(inp["x"])
    out_layer, ids, w, logits = layer.forward(x, return_routing=True)
    k, e, h, f = cfg["topk"], cfg["experts"], cfg["hidden"], cfg["ff"]
    ids_ext = tq.moe_extend_ids(ids, e)
    shared_w = torch.sigmoid(logits[:, e].double()).float()      # the weight itself is checked by the routing tests
    act, out = modular_forward(tq, cfg, banks, x, ids_ext, w, shared_w)
    assert (out_layer - out).abs().max().item() < 5e-5 * max(1.0, out.abs().max().item())
    act_np = act.float().cpu().numpy().reshape(n, k + 1, f)[:head]
    ids_np, w_np, sw_np = ids_ext.cpu().numpy()[:head], w.cpu().numpy()[:head], shared_w.cpu().numpy()[:head]
    deq = np.stack([e4m3_rows(oracle, act_np[t])[2] for t in range(head)])
    rows = np.zeros((head, k + 1, h))
    for _, wd, pairs in widened_down(oracle, cfg, raws[2], ids_np):
        for t, s in pairs:
            ff = f if s < k else cfg["shared_ff"]
            rows[t, s] = half(wd[:, :ff] @ deq[t, s, :ff])
    want = np.zeros((head, h))
    for t in range(head):
        for s in range(k + 1):            # slot order, then the shared row
            want[t] += (float(w_np[t, s]) if s < k else float(sw_np[t])) * rows[t, s]
    mx, rel = synth.errors(out.cpu().numpy()[:head], want)
    top = float(np.abs(want).max())
    print("fp8 down + combine on the device's act rows, config 5 shape: max-abs %.3g (largest value %.3g) rel-rms %.3g" % (mx, top, rel))
    assert mx < MAX_ABS * max(1.0, top) and rel < REL_RMS, (mx, top, rel)


def test_fp8_layer_excess_is_the_straddling_act_values(tq, oracle):
    """End to end against oracle mode 2 at configuration 5's shape: the act values that the device and the oracle put on
    different E4M3 codes are counted, and the difference they make to the output (their dequantised difference through
    the widened down weights and the combine, float64) is taken out: the rest is inside rel-RMS 1e-3 / max-abs 1e-2,
    while the all-token figure beside it may reach 3e-3."""
    n, head = 320, 40
    cfg, raws, banks, inp, layer = setup(tq, oracle, n, seed=530)
    x = dev(inp["x"])
    out, ids, w, logits = layer.forward(x, return_routing=True)
    k, e, h, f, sf = cfg["topk"], cfg["experts"], cfg["hidden"], cfg["ff"], cfg["shared_ff"]
    lg = logits.cpu().numpy()
    want, want_ids, want_w, want_act = oracle.layer_forward(inp["x"][1][:head], lg[:head], *raws, cfg["wtype"], h, f, e, k, shared_ff=sf, act_mode=2,
                                                           threads=16, return_act=True)
    clear = clear_tokens(oracle, lg[:head], e, k, ids.cpu().numpy()[:head], want_ids)
    assert clear.all() and np.array_equal(ids.cpu().numpy()[:head], want_ids)
    ids_ext = tq.moe_extend_ids(ids, e)
    shared_w = torch.sigmoid(logits[:, e].double()).float()
    act, out_mod = modular_forward(tq, cfg, banks, x, ids_ext, w, shared_w)
    assert (out - out_mod).abs().max().item() < 5e-5 * max(1.0, out.abs().max().item())
    act_np = act.float().cpu().numpy().reshape(n, k + 1, f)[:head]
    ids_np, sw_np = ids_ext.cpu().numpy()[:head], shared_w.cpu().numpy()[:head]
    got = out.cpu().numpy()[:head].astype(np.float64)
    dev_q = [e4m3_rows(oracle, act_np[t]) for t in range(head)]
    ora_q = [e4m3_rows(oracle, want_act[t]) for t in range(head)]
    explained = np.zeros((head, h))
    straddle = values = last_bit = 0
    for _, wd, pairs in widened_down(oracle, cfg, raws[2], ids_np):
        for t, s in pairs:
            ff = f if s < k else sf
            cd, co = dev_q[t][0][s, :ff], ora_q[t][0][s, :ff]
            differ = ((cd & 0x7F) != (co & 0x7F)) | (((cd ^ co) & 0x80).astype(bool) & ((cd & 0x7F) != 0))
            straddle += int(differ.sum())
            values += ff
            last_bit += int((act_np[t, s, :ff] != want_act[t, s, :ff]).sum())
            delta = np.where(differ, dev_q[t][2][s, :ff] - ora_q[t][2][s, :ff], 0.0)
            explained[t] += (float(want_w[t, s]) if s < k else float(sw_np[t])) * (wd[:, :ff] @ delta)
    mx_all, rel_all = synth.errors(got, want)
    mx, rel = synth.errors(got - explained, want)
    top = float(np.abs(want).max())
    print("fp8 layer, config 5 shape, %d tokens: %d of %d act values differ in their last fp16 bits, %d of them (%.1e) land on another E4M3 code; "
          "all tokens: max-abs %.3g rel-rms %.3g (largest value %.3g); with the straddling values' share taken out: max-abs %.3g rel-rms %.3g"
          % (head, last_bit, values, straddle, straddle / values, mx_all, rel_all, top, mx, rel))
    assert 0 < straddle < 5e-3 * values                           # they exist and are rare (about one act value in a thousand)
    assert mx_all < MAX_ABS * max(1.0, top) and rel_all < 3e-3, (mx_all, rel_all)
    assert mx < MAX_ABS * max(1.0, top) and rel < REL_RMS, (mx, rel)
