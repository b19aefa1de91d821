"""ctypes binding of the CPU oracle (libtqmoe_oracle.so) and, where it was built, of the reference's own host objects
(oracle/_ref/libtqref.so). TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the cpu_baseline
leg of bench.py, never by the tqllm_amd package.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libtqmoe_oracle.so")
REF_PATH = os.path.join(HERE, "_ref", "libtqref.so")

F32, F16, Q4_K, IQ4_NL, IQ3_S, IQ4_XS, BF16, NVFP4G = 0, 1, 12, 20, 21, 23, 30, 323
Q8_0, Q5_K, Q6_K, IQ3_XXS, IQ2_S = 8, 13, 14, 18, 22
Q4_0, Q3_K, IQ2_XXS, IQ2_XS = 2, 11, 16, 17
Q2_K, IQ1_S = 10, 19
GATE_SOFTMAX, GATE_SIGMOID, GATE_SOFTMAX_WEIGHT, GATE_SQRT_SOFTPLUS = 1, 2, 3, 4
BLOCK = {Q4_K: (256, 144), Q5_K: (256, 176), Q6_K: (256, 210), IQ3_XXS: (256, 98), IQ2_S: (256, 82), Q4_0: (32, 18), Q3_K: (256, 110), IQ2_XXS: (256, 66), IQ2_XS: (256, 74), Q2_K: (256, 84), IQ1_S: (256, 50), Q8_0: (32, 34), IQ4_NL: (32, 18), IQ3_S: (256, 110), IQ4_XS: (256, 136), NVFP4G: (128, 76)}


def build(ref=True):
    """Compile the oracle (and the reference objects when the reference tree is present)."""
    targets = ["all"] + (["ref"] if ref and os.path.isdir("/root/reference/src") else [])
    subprocess.run(["make", "-s", "-C", HERE] + targets, check=True)


def _load():
    if not os.path.exists(LIB_PATH):
        build(ref=False)
    return C.CDLL(LIB_PATH)


_lib = _load()
_p = C.c_void_p
_lib.tqo_half_to_float.restype = C.c_float
_lib.tqo_half_to_float.argtypes = [C.c_uint16]
_lib.tqo_float_to_half.restype = C.c_uint16
_lib.tqo_float_to_half.argtypes = [C.c_float]
_lib.tqo_bf16_to_float.restype = C.c_float
_lib.tqo_bf16_to_float.argtypes = [C.c_uint16]
_lib.tqo_float_to_bf16.restype = C.c_uint16
_lib.tqo_float_to_bf16.argtypes = [C.c_float]
_lib.tqo_e4m3_to_float.restype = C.c_float
_lib.tqo_e4m3_to_float.argtypes = [C.c_uint8]
_lib.tqo_float_to_e4m3.restype = C.c_uint8
_lib.tqo_float_to_e4m3.argtypes = [C.c_float]
_lib.tqo_dequantize.argtypes = [C.c_uint32, _p, _p, C.c_int64]
_lib.tqo_quantize.argtypes = [C.c_uint32, _p, _p, C.c_int64, C.c_int64]
_lib.tqo_route.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, _p, _p, _p, _p]
_lib.tqo_route_softmax_collision.argtypes = [C.c_int, C.c_int, _p]
_lib.tqo_shared_weight.restype = C.c_float
_lib.tqo_shared_weight.argtypes = [C.c_float]
_lib.tqo_dispatch.argtypes = [_p, C.c_int, C.c_int, _p, _p, _p]
_lib.tqo_add_rmsnorm.argtypes = [_p, _p, _p, C.c_float, C.c_int, C.c_int, _p]
_lib.tqo_expert_ffn.restype = None
_lib.tqo_expert_ffn.argtypes = [_p, C.c_int, _p, _p, _p, C.c_int, C.c_float, C.c_int, _p]
_lib.tqo_combine.restype = None
_lib.tqo_combine.argtypes = [C.c_int, _p, _p, C.c_int, _p]
_lib.tqo_router_logits.argtypes = [_p, C.c_uint32, _p, _p, C.c_uint32, C.c_int, C.c_int, C.c_int, _p]
_lib.tqo_quant_act_row_i8.restype = None
_lib.tqo_quant_act_row_i8.argtypes = [_p, C.c_int, _p, _p]
_lib.tqo_quant_act_blocks_i8.restype = None
_lib.tqo_quant_act_blocks_i8.argtypes = [_p, C.c_int, _p, _p, _p]
_lib.tqo_dequantize_nvfp4_widened.restype = C.c_int
_lib.tqo_dequantize_nvfp4_widened.argtypes = [_p, _p, C.c_int64]
_lib.tqo_quant_act_row_e4m3.restype = None
_lib.tqo_quant_act_row_e4m3.argtypes = [_p, C.c_int, _p, _p]
_lib.tqo_cpu_expert_bench.restype = C.c_double
_lib.tqo_cpu_expert_bench.argtypes = [C.c_uint32, _p, _p, _p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _p]
_lib.tqo_cpu_expert_latency.restype = C.c_double
_lib.tqo_cpu_expert_latency.argtypes = [C.c_uint32, _p, _p, _p, C.c_int, C.c_int, C.c_int, C.c_int, _p]
_lib.tqo_cpu_matvec.argtypes = [C.c_uint32, _p, C.c_int, C.c_int, _p, C.c_int, _p]
_lib.tqo_hardware_threads.restype = C.c_int


class _Layer(C.Structure):
    _fields_ = [("hidden", C.c_int), ("ff", C.c_int), ("n_expert", C.c_int), ("k", C.c_int), ("has_shared", C.c_int),
                ("shared_ff", C.c_int), ("wtype", C.c_uint32), ("gate", _p), ("up", _p), ("down", _p),
                ("act_mode", C.c_int), ("threads", C.c_int), ("gating", C.c_int), ("raw_weights", C.c_int),
                ("weight_scale", C.c_float), ("bias", _p), ("wtype_down", C.c_uint32), ("swiglu_clamp", C.c_float), ("clamp_gate", C.c_int), ("act_out", _p)]


_lib.tqo_layer_forward.argtypes = [C.POINTER(_Layer), _p, _p, C.c_int, _p, _p, _p]


def _ptr(a):
    return a.ctypes.data_as(_p) if a is not None else None


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def half_to_float(h):
    return _lib.tqo_half_to_float(int(h))


def float_to_half(f):
    return _lib.tqo_float_to_half(float(f))


def e4m3_to_float(b):
    return _lib.tqo_e4m3_to_float(int(b))


def float_to_e4m3(f):
    return _lib.tqo_float_to_e4m3(float(f))


def to_bf16(a):
    """fp32 array -> (uint16 bf16 bits, fp32 values after rounding), round to nearest even."""
    a = _c(a, np.float32)
    u = a.view(np.uint32)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    return r, (r.astype(np.uint32) << 16).view(np.float32).reshape(a.shape)


def from_bf16(bits):
    """uint16 bf16 bits -> fp32 values."""
    return (np.asarray(bits, np.uint16).astype(np.uint32) << 16).view(np.float32)


def dequantize(wtype, raw, n):
    raw = _c(raw, np.uint8)
    out = np.empty(int(n), np.float32)
    if _lib.tqo_dequantize(wtype, _ptr(raw), _ptr(out), int(n)):
        raise ValueError("tqo_dequantize: bad type or size")
    return out


def dequantize_nvfp4_widened(raw, n):
    """NVFP4G blocks with e2m1 * scale rounded to E4M3 before the global multiplies it (the fp8 products' weights)."""
    raw = _c(raw, np.uint8)
    out = np.empty(int(n), np.float32)
    if _lib.tqo_dequantize_nvfp4_widened(_ptr(raw), _ptr(out), int(n)):
        raise ValueError("tqo_dequantize_nvfp4_widened: bad size")
    return out


def quantize(wtype, w, row=None):
    w = _c(w, np.float32)
    elems, nbytes = BLOCK[wtype]
    out = np.zeros(w.size // elems * nbytes, np.uint8)
    if _lib.tqo_quantize(wtype, _ptr(w), _ptr(out), w.size, int(row if row is not None else w.shape[-1])):
        raise ValueError("tqo_quantize: bad type or size")
    return out


def route(logits, k, gating=GATE_SOFTMAX, norm=True, scale=1.0, bias=None):
    """logits [n][E] (or [E]) -> ids [n][k] int32, weights [n][k] fp32."""
    lg = np.atleast_2d(_c(logits, np.float32))
    n, e = lg.shape
    ids = np.empty((n, k), np.int32)
    w = np.empty((n, k), np.float32)
    b = _c(bias, np.float32) if bias is not None else None
    for t in range(n):
        if _lib.tqo_route(gating, e, k, int(norm), float(scale), _ptr(lg[t]), _ptr(b), _ptr(ids[t]), _ptr(w[t])):
            raise ValueError("tqo_route: bad shape")
    return ids, w


def route_softmax_collision(logits, k):
    """bool per token: the reference's choice rests on a tie of rounded probabilities between different logits"""
    lg = np.atleast_2d(_c(logits, np.float32))
    return np.array([bool(_lib.tqo_route_softmax_collision(lg.shape[1], k, _ptr(lg[t]))) for t in range(lg.shape[0])])


def shared_weight(logit):
    return _lib.tqo_shared_weight(float(logit))


def dispatch(ids, n_expert):
    ids = _c(ids, np.int32).reshape(-1)
    counts = np.empty(n_expert, np.int32)
    offsets = np.empty(n_expert + 1, np.int32)
    perm = np.full(ids.size, -1, np.int32)
    if _lib.tqo_dispatch(_ptr(ids), ids.size, n_expert, _ptr(counts), _ptr(offsets), _ptr(perm)):
        raise ValueError("tqo_dispatch: id out of range")
    return counts, offsets, perm


DEDUP_COLS, DEDUP_STRIDE = 8, 18    # kDedupCols, kDedupStride (src/experts/moe_kernels.cuh:33-38)


def dedup_maps(ids, slot_of, topk, groups):
    """The decode grouping maps of moe_dedup_maps, one assignment at a time as the reference's kernel computes them
    (src/experts/moe.cu:452-483): slots[a] = slot_of[ids[a]] (-1 for a skipped assignment); an assignment's rank among the
    assignments of its slot gives its chunk (rank / 8) and column (rank % 8); its group is the number of groups opened by
    earlier assignments than its chunk's opener; a group's record is [slot, columns, 8 inputs, 8 outputs] with the token
    (gu) or the assignment (dn) as input and the assignment as output, unused entries -1. Pure Python: small inputs only.
    Returns (slots [count], gu [groups][18], dn [groups][18])."""
    ids = np.asarray(ids, np.int32).reshape(-1)
    count = ids.size
    slot = np.array([slot_of[e] if e >= 0 else -1 for e in ids], np.int32)
    gu = np.full((groups, DEDUP_STRIDE), -1, np.int32)
    dn = np.full((groups, DEDUP_STRIDE), -1, np.int32)
    rank = np.array([int((slot[:a] == slot[a]).sum()) for a in range(count)])
    total = np.array([int((slot == slot[a]).sum()) for a in range(count)])
    opens = (slot >= 0) & (rank % DEDUP_COLS == 0)
    for a in range(count):
        if slot[a] < 0:
            continue
        chunk, col = divmod(int(rank[a]), DEDUP_COLS)
        same = np.flatnonzero(slot[:a + 1] == slot[a])
        opener = int(same[chunk * DEDUP_COLS])
        g = int(opens[:opener].sum())
        cols = min(DEDUP_COLS, int(total[a]) - chunk * DEDUP_COLS)
        for part, e in ((0, gu), (1, dn)):
            if col == 0:
                e[g, 0], e[g, 1] = slot[a], cols
            e[g, 2 + col] = a if part else a // topk
            e[g, 2 + DEDUP_COLS + col] = a
    return slot, gu, dn


def count(ids, counts):
    """moe_count (src/experts/moe.cu:183-186, 279-282): counts[ids[i]] += 1 on 64-bit running counters; negative ids are
    skipped here as everywhere in this library (the reference's callers never pass them to this function)."""
    ids = np.asarray(ids).reshape(-1)
    np.add.at(counts, ids[ids >= 0], 1)
    return counts


def expert_ffn(x, w_gate, w_up, w_down, clamp=0.0, clamp_gate=False):
    x, w_gate, w_up, w_down = (_c(a, np.float32) for a in (x, w_gate, w_up, w_down))
    ff, hidden = w_gate.shape
    out = np.empty(hidden, np.float32)
    _lib.tqo_expert_ffn(_ptr(x), hidden, _ptr(w_gate), _ptr(w_up), _ptr(w_down), ff, float(clamp), int(clamp_gate), _ptr(out))
    return out


def combine(weights, expert_outs, out=None):
    weights, expert_outs = _c(weights, np.float32), _c(expert_outs, np.float32)
    k, hidden = expert_outs.shape
    out = np.zeros(hidden, np.float32) if out is None else out
    _lib.tqo_combine(k, _ptr(weights), _ptr(expert_outs), hidden, _ptr(out))
    return out


def router_logits(w, wtype, shared_gate, x, xtype, hidden, n_expert, n):
    out = np.empty((n, n_expert + 1), np.float32)
    if _lib.tqo_router_logits(_ptr(w), wtype, _ptr(shared_gate), _ptr(x), xtype, hidden, n_expert, n, _ptr(out)):
        raise ValueError("tqo_router_logits: bad shape or type")
    return out


def quant_act_row_i8(x):
    x = _c(x, np.float32)
    q = np.empty(x.size, np.int8)
    s = np.empty(1, np.float32)
    _lib.tqo_quant_act_row_i8(_ptr(x), x.size, _ptr(q), _ptr(s))
    return q, float(s[0])


def quant_act_blocks_i8(x):
    """(q int8 [cols], scales fp32 [cols / 32], sums of q per 16 int16 [cols / 32][2])"""
    x = _c(x, np.float32)
    q = np.empty(x.size, np.int8)
    s = np.empty(x.size // 32, np.float32)
    qsum = np.empty((x.size // 32, 2), np.int16)
    _lib.tqo_quant_act_blocks_i8(_ptr(x), x.size, _ptr(q), _ptr(s), _ptr(qsum))
    return q, s, qsum


def quant_act_row_e4m3(x):
    x = _c(x, np.float32)
    q = np.empty(x.size, np.uint8)
    s = np.empty(1, np.float32)
    _lib.tqo_quant_act_row_e4m3(_ptr(x), x.size, _ptr(q), _ptr(s))
    return q, float(s[0])


def add_rmsnorm(rows_bits, residual_bits, weight, eps):
    """rows_bits, residual_bits: uint16 bf16 [n][H] (residual may be None); returns (updated rows bits, normed bf16 bits)."""
    rows = np.array(rows_bits, dtype=np.uint16, order="C", copy=True)
    res = _c(residual_bits, np.uint16) if residual_bits is not None else None
    w = _c(weight, np.float32)
    n, h = rows.shape
    out = np.empty((n, h), np.uint16)
    if _lib.tqo_add_rmsnorm(_ptr(rows), _ptr(res), _ptr(w), float(eps), h, n, _ptr(out)):
        raise ValueError("tqo_add_rmsnorm: hidden must be a positive multiple of 256")
    return rows, out


def layer_forward(x, logits, gate, up, down, wtype, hidden, ff, n_expert, k, shared_ff=0, act_mode=0, threads=8, gating=GATE_SOFTMAX,
                  norm=True, scale=1.0, bias=None, wtype_down=0, swiglu_clamp=0.0, clamp_gate=False, return_act=False):
    """Whole layer on the host; returns (out [n][H] fp32, ids [n][k], weights [n][k]); with return_act (act modes other than 0)
    also the rows silu(gate) * up that the down product's quantiser receives, [n][slots][ff] (zero beyond a shared row's shared_ff)."""
    bias = _c(bias, np.float32) if bias is not None else None
    x, logits = _c(x, np.float32), _c(logits, np.float32)
    gate, up, down = (_c(a, np.uint8) for a in (gate, up, down))
    n = x.shape[0]
    L = _Layer(hidden, ff, n_expert, k, int(shared_ff > 0), shared_ff, wtype, _ptr(gate), _ptr(up), _ptr(down), act_mode, threads,
               int(gating), int(not norm), float(scale), _ptr(bias), int(wtype_down), float(swiglu_clamp), int(bool(clamp_gate)), None)
    act = None
    if return_act:
        if act_mode == 0:
            raise ValueError("tqo_layer_forward: act rows are returned by the act modes other than 0")
        act = np.zeros((n, k + int(shared_ff > 0), ff), np.float32)
        L.act_out = _ptr(act)
    out = np.empty((n, hidden), np.float32)
    ids = np.empty((n, k), np.int32)
    w = np.empty((n, k), np.float32)
    if _lib.tqo_layer_forward(C.byref(L), _ptr(x), _ptr(logits), n, _ptr(out), _ptr(ids), _ptr(w)):
        raise ValueError("tqo_layer_forward: bad configuration")
    return (out, ids, w, act) if return_act else (out, ids, w)


def cpu_expert_bench(wtype, gate, up, down, hidden, ff, n_expert, threads, int8_act, reps=3):
    gate, up, down = (_c(a, np.uint8) for a in (gate, up, down))
    chk = np.zeros(1, np.float32)
    t = _lib.tqo_cpu_expert_bench(wtype, _ptr(gate), _ptr(up), _ptr(down), hidden, ff, n_expert, threads, int(int8_act), reps, _ptr(chk))
    if t < 0:
        raise ValueError("tqo_cpu_expert_bench: bad configuration")
    return t, float(chk[0])


def cpu_expert_latency(wtype, gate, up, down, hidden, ff, threads, reps=20):
    """seconds per expert with the rows of one expert split over persistent workers (int8 activations)"""
    gate, up, down = (_c(a, np.uint8) for a in (gate, up, down))
    chk = np.zeros(1, np.float32)
    t = _lib.tqo_cpu_expert_latency(wtype, _ptr(gate), _ptr(up), _ptr(down), hidden, ff, threads, reps, _ptr(chk))
    if t < 0:
        raise ValueError("tqo_cpu_expert_latency: bad configuration")
    return t, float(chk[0])


def cpu_matvec(wtype, w, rows, cols, x, mode):
    """y [rows] = W x with the baseline's kernels: mode 0 fp32, 1 int8 activations (AVX2), 2 int8 activations (scalar)"""
    w, x = _c(w, np.uint8), _c(x, np.float32)
    y = np.empty(rows, np.float32)
    if _lib.tqo_cpu_matvec(wtype, _ptr(w), rows, cols, _ptr(x), mode, _ptr(y)):
        raise ValueError("tqo_cpu_matvec: bad configuration")
    return y


def hardware_threads():
    return _lib.tqo_hardware_threads()


def random_blocks(wtype, rows, cols, rng):
    """GGUF blocks of a [rows][cols] matrix: random codes and sub-scales, block scales sized for weights of about 0.02"""
    elems, nbytes = BLOCK[wtype]
    nb = rows * cols // elems
    raw = rng.integers(0, 256, (nb, nbytes), dtype=np.uint8)
    if wtype == NVFP4G:
        g = np.repeat(rng.uniform(5e-4, 2.5e-3, rows).astype(np.float32), cols // elems)
        raw[:, 0:4] = g.view(np.uint8).reshape(nb, 4)
        raw[:, 4:12] = 0x28 + rng.integers(0, 0x30, (nb, 8), dtype=np.uint8)
    else:
        lo, hi = {IQ4_XS: (4e-5, 8e-5), IQ4_NL: (1.5e-4, 3e-4), Q4_K: (1e-4, 2e-4), IQ3_S: (1.5e-4, 3e-4)}[wtype]
        raw[:, 0:2] = np.float16(rng.uniform(lo, hi, nb)).view(np.uint8).reshape(nb, 2)
        if wtype == Q4_K:
            raw[:, 2:4] = np.float16(rng.uniform(lo, hi, nb)).view(np.uint8).reshape(nb, 2)
    return raw.reshape(-1)


def cpu_baseline_sweep(wtype, hidden, ff, experts_per_token, cores, budget_s=12.0, sample_experts=24):
    """The CPU expert path on this machine's cores, as the reference's tests/bench_cpu_expert_mt.cpp runs it: thread counts
    1, 2, 4, ... up to `cores`, fp32 and int8-activation variants over `sample_experts` experts of the layer's shape pulled
    from an atomic queue; then the rows of one expert split over persistent workers. Returns the benchmark's cpu_baseline
    record: value = MoE-layer tokens/s of the best (threads, variant) = 1 / (experts_per_token x its mean time per expert)."""
    import time
    rng = np.random.default_rng(7)
    banks = [random_blocks(wtype, sample_experts * rows, cols, rng) for rows, cols in ((ff, hidden), (ff, hidden), (hidden, ff))]
    expert_bytes = sum(b.size for b in banks) / sample_experts
    t_start = time.time()
    counts = sorted({min(cores, 1 << i) for i in range(cores.bit_length() + 1)} | {cores})
    sweep, best = [], None
    for nt in counts:
        for int8 in (False, True):
            t_pass, _ = cpu_expert_bench(wtype, *banks, hidden, ff, sample_experts, nt, int8, reps=2)
            row = {"threads": nt, "variant": "int8" if int8 else "fp32", "ms_per_expert": round(t_pass / sample_experts * 1e3, 4),
                   "gb_per_s": round(expert_bytes * sample_experts / t_pass / 1e9, 2)}
            sweep.append(row)
            if best is None or t_pass < best[0]:
                best = (t_pass, nt, int8)
    # the best setting again, for what is left of the budget
    spent = time.time() - t_start
    reps = int(max(3, min(4000, (budget_s - spent) / max(best[0], 1e-4))))
    t_pass, _ = cpu_expert_bench(wtype, *banks, hidden, ff, sample_experts, best[1], best[2], reps=reps)
    per_expert = t_pass / sample_experts
    one = [b[: b.size // sample_experts] for b in banks]
    latency = {}
    for nt in counts:
        t_one, _ = cpu_expert_latency(wtype, *one, hidden, ff, nt, reps=30)
        latency[str(nt)] = round(t_one * 1e3, 4)
    name = {IQ4_XS: "IQ4_XS", IQ4_NL: "IQ4_NL", Q4_K: "Q4_K", IQ3_S: "IQ3_S", NVFP4G: "NVFP4G"}[wtype]
    return {"value": round(1.0 / (per_expert * experts_per_token), 2), "unit": "tokens/s", "cores": best[1], "kind": "port",
            "variant": "int8" if best[2] else "fp32", "ms_per_expert": round(per_expert * 1e3, 4),
            "gb_per_s": round(expert_bytes / per_expert / 1e9, 2), "cores_available": cores,
            "sample": "%d %s experts (gate/up %dx%d, down %dx%d), one token each, workers on an atomic expert queue, thread counts %s x {fp32, "
                      "int8 activations per 32-block with AVX2 integer dots}; value = best setting (%d threads, %s) re-timed over %d passes: "
                      "tokens/s = 1 / (%d experts x mean time per expert); %.1f s of CPU work"
                      % (sample_experts, name, ff, hidden, hidden, ff, counts, best[1], "int8" if best[2] else "fp32", reps, experts_per_token,
                         time.time() - t_start),
            "sweep": sweep, "row_split_ms_per_expert": latency}


def cpu_reference_shape(cores, sample_experts=24):
    """The shape the reference's own program runs (tests/bench_cpu_expert_mt.cpp:26-61: 24 experts of IQ4_NL gate / up 640 x 2560
    and down 2560 x 640, one token), on one thread and on all cores, fp32 and int8 activations: ms per expert and GB/s of
    packed weights, for continuity with the figures that program prints."""
    rng = np.random.default_rng(8)
    hidden, ff = 2560, 640
    banks = [random_blocks(IQ4_NL, sample_experts * rows, cols, rng) for rows, cols in ((ff, hidden), (ff, hidden), (hidden, ff))]
    expert_bytes = sum(b.size for b in banks) / sample_experts
    rows = []
    for nt in sorted({1, cores}):
        for int8 in (False, True):
            t_pass, _ = cpu_expert_bench(IQ4_NL, *banks, hidden, ff, sample_experts, nt, int8, reps=2)
            rows.append({"threads": nt, "variant": "int8" if int8 else "fp32", "ms_per_expert": round(t_pass / sample_experts * 1e3, 4),
                         "gb_per_s": round(expert_bytes * sample_experts / t_pass / 1e9, 2)})
    return {"shape": "IQ4_NL, %d experts, gate/up %dx%d, down %dx%d (tests/bench_cpu_expert_mt.cpp)" % (sample_experts, ff, hidden, hidden, ff), "rows": rows}


def cpu_config1_layer(cores, tokens=(1, 16)):
    """Configuration 1 whole on the host ("CPU reference, one MoE layer": hidden 2048, 64 Q4_K experts, softmax top-8
    renormalised, ff 768, fp32 router and activations): router logits, routing, the selected experts' FFN from the decoded
    weights in fp32, combine, on all cores. This is the correctness path timed as it is (it decodes every selected expert to
    fp32 first), not a tuned kernel: tokens/s per batch size."""
    import time
    rng = np.random.default_rng(9)
    h, f, e, k = 2048, 768, 64, 8
    banks = [random_blocks(Q4_K, e * rows, cols, rng) for rows, cols in ((f, h), (f, h), (h, f))]
    router = (rng.standard_normal((e, h)) * 0.02).astype(np.float32)
    out = []
    for n in tokens:
        x = rng.standard_normal((n, h)).astype(np.float32)
        best = None
        for _ in range(2):
            t0 = time.time()
            logits = router_logits(router, F32, None, x, F32, h, e, n)
            layer_forward(x, logits, *banks, Q4_K, h, f, e, k, threads=cores)
            dt = time.time() - t0
            best = dt if best is None else min(best, dt)
        out.append({"tokens": n, "ms": round(best * 1e3, 2), "tokens_per_s": round(n / best, 1), "threads": cores})
    return out


def ref_lib():
    """The reference's own host objects, or None where they were not built (no reference tree)."""
    if not os.path.exists(REF_PATH):
        return None
    r = C.CDLL(REF_PATH)
    r.ref_half_to_float.restype = C.c_float
    r.ref_half_to_float.argtypes = [C.c_uint16]
    r.ref_float_to_half.restype = C.c_uint16
    r.ref_float_to_half.argtypes = [C.c_float]
    r.ref_e4m3_to_float.restype = C.c_float
    r.ref_e4m3_to_float.argtypes = [C.c_uint8]
    r.ref_dequantize.argtypes = [C.c_uint32, _p, _p, C.c_int64]
    r.ref_route.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, _p, _p, _p, _p]
    r.ref_expert_ffn.restype = None
    r.ref_expert_ffn.argtypes = [_p, C.c_int, _p, _p, _p, C.c_int, C.c_float, C.c_int, _p]
    r.ref_combine.restype = None
    r.ref_combine.argtypes = [C.c_int, _p, _p, C.c_int, _p]
    r.ref_iq4nl_matvec.restype = None
    r.ref_iq4nl_matvec.argtypes = [C.c_int, _p, C.c_int, C.c_int, _p, C.c_int, _p]
    return r
