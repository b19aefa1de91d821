#!/usr/bin/env python3
"""MoE-layer benchmark on one MI355X.

The default run measures the metric of the benchmark definition, "MoE-layer tokens/s at 1 and 4096 tokens", on the
Flash-Next-shaped IQ4_XS layer: decode batches of 1, 4 and 16 tokens (configuration 2) and the 4096-token prefill with
Zipf-skewed routing (configuration 3). The headline fields of the JSON line are the 4096-token point; `points` carries
every measured point with its own step time, tokens/s, roofline and layer figures. `--config 1|4|5` measures the other
configurations at their own token counts, `--tokens T` one point only (what the profiling commands use).

A step is one pass of the whole layer (router, top-k, gate/up + SwiGLU, down, combine, shared expert) over one batch of
T tokens with every input already resident in HBM. Steps rotate over several independent expert banks (and, for short
batches, over several input batches per bank) so that a step's weights stream from HBM, not from the 256 MB last-level
cache. Per point:
  tokens_per_s  T / mean step time over exactly --steps steps, captured into one HIP graph, after --warmup untimed steps
  roofline      the dominant kernel (gate + up + SwiGLU) over its mean duration, measured with events on the launching
                stream around back-to-back launches of that kernel alone. Decode kernels: the bytes of the distinct
                experts the launch must read against 8 TB/s. Grouped products: 2 operations per multiply-add of their
                assignments against the dense matrix peak of the operand type
  layer         the whole step's algorithmic bytes and operations against the same peaks
cpu_baseline: the CPU expert path (the scheme of the reference's tests/bench_cpu_expert_mt.cpp at this layer's shape)
timed on this box's host cores on a bounded sample.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")   # measured with rocprofv3 --pmc (see the file)
HBM_PEAK = 8.0e12  # bytes/s, MI355X published
PEAK = {"int8": 5.0e15, "fp8": 5.0e15, "fp16": 2.5e15}   # dense matrix operations/s, MI355X published
ZIPF_S = 1.1
DISTINCT_MB = 640  # distinct weight bytes the steps of a point cycle through at least (the last-level cache holds 256 MB)

# GGUF type ids and block sizes (weights, bytes)
Q4_K, IQ3_S, IQ4_XS, NVFP4G = 12, 21, 23, 323
BLOCK = {Q4_K: (256, 144), IQ3_S: (256, 110), IQ4_XS: (256, 136), NVFP4G: (128, 76)}
CONFIGS = {
    "2": dict(label="config 2 / 3: Flash-Next-shaped layer, hidden 2048, 512 IQ4_XS experts top-10 + shared (ff 512), bf16 router and activations",
              hidden=2048, ff=512, experts=512, topk=10, shared_ff=512, wtype=IQ4_XS, fmt="IQ4_XS", rtype="bf16", xtype="bf16",
              points=(1, 4, 16, 4096), zipf_from=64),
    "1": dict(label="config 1: hidden 2048, 64 Q4_K experts top-8 (ff 768), fp32 router and activations",
              hidden=2048, ff=768, experts=64, topk=8, shared_ff=0, wtype=Q4_K, fmt="Q4_K", rtype="f32", xtype="f32", points=(1, 16, 4096), zipf_from=None),
    "4": dict(label="config 4: hidden 2048, 256 IQ3_S experts top-8 (ff 768), bf16 router and activations",
              hidden=2048, ff=768, experts=256, topk=8, shared_ff=0, wtype=IQ3_S, fmt="IQ3_S", rtype="bf16", xtype="bf16", points=(1, 64, 512),
              zipf_from=None),
    "5": dict(label="config 5: hidden 3072, 256 NVFP4 experts top-8 + shared (ff 1536), bf16 router and activations, router logits N(0,1)",
              hidden=3072, ff=1536, experts=256, topk=8, shared_ff=1536, wtype=NVFP4G, fmt="NVFP4G", rtype="bf16", xtype="bf16", points=(8192,),
              zipf_from=None, unit_logits=True),
}


def random_bank(torch, wtype, experts, rows, cols, gen):
    """GGUF block stream of random valid blocks on the device, block scales sized for weights of about 0.02 (random
    codes and sub-scales, small finite super-scales, as the reference's device tests make their banks:
    tests/moe_device.cu:121-138, tests/nvfp4_expert.cu:34-50)."""
    elems, nbytes = BLOCK[wtype]
    nb = experts * rows * cols // elems
    raw = torch.randint(0, 256, (nb, nbytes), dtype=torch.uint8, device="cuda", generator=gen)

    def half_field(lo, hi, signed):
        d = (torch.rand(nb, device="cuda", generator=gen) * (hi - lo) + lo).to(torch.float16)
        if signed:
            d = d * (torch.randint(0, 2, (nb,), device="cuda", generator=gen) * 2 - 1).to(torch.float16)
        return d.view(torch.uint8).reshape(nb, 2)

    if wtype == IQ4_XS:
        raw[:, 0:2] = half_field(4e-5, 8e-5, True)
    elif wtype == Q4_K:
        raw[:, 0:2] = half_field(1e-4, 2e-4, False)
        raw[:, 2:4] = half_field(1e-4, 2e-4, False)
    elif wtype == IQ3_S:
        raw[:, 0:2] = half_field(1.5e-4, 3e-4, True)
    elif wtype == NVFP4G:
        per_row = cols // elems
        g = (torch.rand(experts * rows, device="cuda", generator=gen) * 2e-3 + 5e-4).float()      # one global per row
        raw[:, 0:4] = g.repeat_interleave(per_row).view(torch.uint8).reshape(nb, 4)
        raw[:, 4:12] = (0x28 + torch.randint(0, 0x30, (nb, 8), device="cuda", generator=gen)).to(torch.uint8)   # E4M3 0.125 .. 16
    return raw.reshape(-1)


def build_banks(torch, tq, cfg, banks, seed):
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    h, f, e = cfg["hidden"], cfg["ff"], cfg["experts"] + (1 if cfg["shared_ff"] else 0)
    out = []
    for _ in range(banks):
        trio = []
        for rows, cols in ((f, h), (f, h), (h, f)):
            raw = random_bank(torch, cfg["wtype"], e, rows, cols, gen)
            trio.append(tq.ExpertBank(cfg["wtype"], raw, e, rows, cols))
            del raw
        out.append(trio)
    torch.cuda.synchronize()
    return out, gen


def build_point(torch, tq, cfg, trios, gen, tokens, act_blocks=False, batches=1):
    """One layer per bank and `batches` input batches per layer for a point of `tokens` tokens (a short batch reads few experts:
    with several batches per bank the steps cycle through more distinct weights than the last-level cache holds)."""
    h = cfg["hidden"]
    skew = cfg["zipf_from"] is not None and tokens >= cfg["zipf_from"]
    unit = skew or cfg.get("unit_logits")
    rdt = torch.bfloat16 if cfg["rtype"] == "bf16" else torch.float32
    xdt = torch.bfloat16 if cfg["xtype"] == "bf16" else torch.float32
    layers, xs = [], []
    for trio in trios:
        router = torch.randn((cfg["experts"], h), device="cuda", generator=gen) * (h ** -0.5 if unit else 0.02)
        x = torch.randn((batches, tokens, h), device="cuda", generator=gen)
        if skew:
            # logits = N(0, 1) + ln p_e, p_e ~ rank^-1.1 over a random permutation of the experts: the bias rides in the
            # last router column against a constant 1 in the last activation
            p = 1.0 / torch.arange(1, cfg["experts"] + 1, device="cuda", dtype=torch.float64) ** ZIPF_S
            p = (p / p.sum())[torch.randperm(cfg["experts"], device="cuda", generator=gen)]
            router[:, -1] = torch.log(p).float()
            x[:, :, -1] = 1.0
        sgate = (torch.randn((h,), device="cuda", generator=gen) * 0.02).to(rdt) if cfg["shared_ff"] else None
        layers.append(tq.MoeLayer(router.to(rdt), sgate, *trio, cfg["topk"], shared_ff=cfg["shared_ff"], act_blocks=act_blocks))
        xs.append([b.contiguous() for b in x.to(xdt)])
    torch.cuda.synchronize()
    return layers, xs, skew


def time_calls(torch, fn, calls, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(calls):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / calls  # ms per call


def measure_point(torch, tq, cfg, key, trios, gen, T, args, traffic):
    R = len(trios)
    h, f, k = cfg["hidden"], cfg["ff"], cfg["topk"]
    slots = k + (1 if cfg["shared_ff"] else 0)
    bpw = BLOCK[cfg["wtype"]][1] / BLOCK[cfg["wtype"]][0]
    # input batches per bank: enough distinct (bank, batch) steps that a cycle through them reads more weights than the
    # last-level cache holds (a one-token step reads eleven experts, 20 MB)
    step_mb = min(T * slots, cfg["experts"]) * 3 * f * h * bpw / 1e6
    X = max(1, min(8, math.ceil(DISTINCT_MB / (R * step_mb))))
    layers, xs, skew = build_point(torch, tq, cfg, trios, gen, T, act_blocks=args.act_blocks, batches=X)
    outs = [torch.empty((T, h), dtype=torch.float32, device="cuda") for _ in range(R)]
    for l in layers:
        l.workspace(T)
    path = layers[0].path(T)
    cycle = [(b, j) for j in range(X) for b in range(R)]      # the steps' order: every bank in turn, then the next batch

    # ---- whole layer: exactly `steps` steps, one after the other on the stream, timed with events around them. They are
    # captured into one HIP graph so that the host's launch rate is not what is measured; the warm-up is `warmup` steps of the
    # same cycle, untimed.
    def run_steps(first, count):
        for i in range(first, first + count):
            b, j = cycle[i % len(cycle)]
            layers[b].forward(xs[b][j], out=outs[b])

    K, W = args.steps, max(args.warmup, 1)
    launch = "eager"
    timed = lambda: run_steps(W, K)
    if not args.no_graph:
        try:
            run_steps(0, len(cycle))
            torch.cuda.synchronize()
            ref = [o.clone() for o in outs]
            check = torch.cuda.CUDAGraph()
            with torch.cuda.graph(check):
                run_steps(0, len(cycle))
            for _ in range(3):          # replays must reproduce the eager result
                for o in outs:
                    o.zero_()
                check.replay()
                torch.cuda.synchronize()
                assert all(torch.equal(a, c) for a, c in zip(ref, outs)), "graph replay differs from the eager result"
            del check
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                run_steps(W, K)
            timed, launch = g.replay, "hipgraph(%d steps)" % K
        except Exception as ex:  # noqa: BLE001
            print("bench.py: HIP graph path unavailable (%s); timing eager launches" % ex, file=sys.stderr)
    run_steps(0, W)                     # warm-up: W untimed steps
    torch.cuda.synchronize()
    t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0.record()
    timed()                             # exactly K steps
    t1.record()
    torch.cuda.synchronize()
    ms_step = t0.elapsed_time(t1) / K
    rounds = max(4, math.ceil(K / len(cycle)))   # passes over the cycle for the per-kernel timings below

    # ---- routing statistics of the steps (distinct experts a step must read)
    uniq, routing = [], []
    for b, j in cycle:
        _, ids, _, _ = layers[b].forward(xs[b][j], return_routing=True)
        uniq.append(int(torch.unique(ids).numel()))
        routing.append(ids)
    u_mean = sum(uniq) / len(uniq)
    shared = 1 if cfg["shared_ff"] else 0
    rbytes = 2 if cfg["rtype"] == "bf16" else 4
    xbytes = 2 if cfg["xtype"] == "bf16" else 4
    layer_bytes = (u_mean + shared) * 3 * f * h * bpw + (cfg["experts"] + shared) * h * rbytes + T * h * xbytes * 2
    gu_bytes = (u_mean + shared) * 2 * f * h * bpw
    dn_bytes = (u_mean + shared) * f * h * bpw
    gu_ops = T * slots * 2 * f * h * 2.0      # multiply-adds of gate and up, 2 operations each
    dn_ops = T * slots * f * h * 2.0

    # ---- dominant kernels alone: back-to-back launches over the rotating banks, inputs prepared once
    prep = []
    fp8 = path == "grouped_fp8"
    for (b, j), ids in zip(cycle, routing):
        l, x = layers[b], xs[b][j]
        ext = tq.moe_extend_ids(ids, cfg["experts"]) if shared else ids
        if path == "decode":
            img = tq.quant_act(x)
            act = tq.expert_gateup(l.gate, l.up, img, ext, k, shared_ff=cfg["shared_ff"])
            y = tq.expert_down(l.down, act, ext, k, shared_ff=cfg["shared_ff"])
            prep.append((l, ext, img, act, y))
        else:
            counts, offsets, perm, _ = tq.moe_dispatch(ext, cfg["experts"] + shared)
            lists = (counts, offsets, perm)
            if path == "grouped_i8" and args.act_blocks:   # a scale per 32 activations: the block scales ride along
                xq, xsc, xbs = tq.group_rows_i8_blocks(x, lists, T * slots, slots)
                act = tq.expert_gemm_gateup_i8_blocks(l.gate, l.up, xq, xsc, xbs, lists, T, slots, k, cfg["shared_ff"])
                aq, asc, abs_ = tq.group_rows_i8_blocks(act, lists, T * slots, 1)
                y = tq.expert_gemm_i8_blocks(l.down, aq, asc, abs_, lists, T, slots, k, cfg["shared_ff"])
                prep.append((l, lists, xq, (xsc, xbs), aq, (asc, abs_), act, y))
            elif path in ("grouped_i8", "grouped_fp8"):
                xq, xsc = tq.group_rows_i8(x, lists, T * slots, slots, fp8=fp8)
                act = tq.expert_gemm_gateup_i8(l.gate, l.up, xq, xsc, lists, T, slots, k, cfg["shared_ff"], fp8=fp8)
                aq, asc = tq.group_rows_i8(act, lists, T * slots, 1, fp8=fp8)
                y = tq.expert_gemm_i8(l.down, aq, asc, lists, T, slots, k, cfg["shared_ff"], fp8=fp8)
                prep.append((l, lists, xq, xsc, aq, asc, act, y))
            else:
                act = tq.expert_gemm_gateup(l.gate, l.up, x, lists, T, slots, k, cfg["shared_ff"])
                y = tq.expert_gemm(l.down, act, lists, T, slots, k, cfg["shared_ff"], per_expert_input=True, out_type=tq.F32)
                prep.append((l, lists, x, act, y))

    # (every launch writes into the rows its first run allocated: nothing but the kernel is on the stream between the events)
    def gateup_round():
        for item in prep:
            if path == "decode":
                l, ext, img, act, y = item
                tq.expert_gateup(l.gate, l.up, img, ext, k, shared_ff=cfg["shared_ff"], act_image=act)
            elif path in ("grouped_i8", "grouped_fp8"):
                l, lists, xq, xsc, aq, asc, act, y = item
                if isinstance(xsc, tuple):
                    tq.expert_gemm_gateup_i8_blocks(l.gate, l.up, xq, xsc[0], xsc[1], lists, T, slots, k, cfg["shared_ff"], act=act)
                else:
                    tq.expert_gemm_gateup_i8(l.gate, l.up, xq, xsc, lists, T, slots, k, cfg["shared_ff"], fp8=fp8, act=act)
            else:
                l, lists, x, act, y = item
                tq.expert_gemm_gateup(l.gate, l.up, x, lists, T, slots, k, cfg["shared_ff"], act=act)

    def down_round():
        for item in prep:
            if path == "decode":
                l, ext, img, act, y = item
                tq.expert_down(l.down, act, ext, k, shared_ff=cfg["shared_ff"], y=y)
            elif path in ("grouped_i8", "grouped_fp8"):
                l, lists, xq, xsc, aq, asc, act, y = item
                if isinstance(asc, tuple):
                    tq.expert_gemm_i8_blocks(l.down, aq, asc[0], asc[1], lists, T, slots, k, cfg["shared_ff"], y=y)
                else:
                    tq.expert_gemm_i8(l.down, aq, asc, lists, T, slots, k, cfg["shared_ff"], fp8=fp8, y=y)
            else:
                l, lists, x, act, y = item
                tq.expert_gemm(l.down, act, lists, T, slots, k, cfg["shared_ff"], per_expert_input=True, out_type=tq.F32, y=y)

    kernels = {}
    small = path == "decode"
    reps = 4 if small else 1
    for name, fn in (("gateup", gateup_round), ("down", down_round)):
        fn()
        torch.cuda.synchronize()
        timed = fn
        if small and not args.no_graph:   # microsecond kernels: replay a graph of them so that the host is not the bound
            gk = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gk):
                for _ in range(reps):
                    fn()
            timed = gk.replay
        n_calls = max(4, rounds // reps) if small else max(4, min(rounds, 20))
        kernels[name] = time_calls(torch, timed, n_calls, 2) / ((reps if timed is not fn else 1) * len(cycle))  # ms per launch

    gu_s, dn_s, step_s = kernels["gateup"] * 1e-3, kernels["down"] * 1e-3, ms_step * 1e-3
    if path == "decode":
        kname = "iq4xs_mfma_k<2> (gate + up + SwiGLU)" if cfg["wtype"] == IQ4_XS else "gateup_k<%s> (gate + up + SwiGLU)" % cfg["fmt"]
        roofline = {"bound": "hbm", "kernel": kname, "achieved": round(gu_bytes / gu_s / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                    "frac": round(gu_bytes / gu_s / HBM_PEAK, 4), "traffic": None, "algorithmic_bytes_per_launch": int(gu_bytes),
                    "us_per_launch": round(gu_s * 1e6, 2)}
        layer = {"algorithmic_bytes_per_step": int(layer_bytes), "hbm_frac": round(layer_bytes / step_s / HBM_PEAK, 4),
                 "down_us": round(dn_s * 1e6, 2), "down_hbm_frac": round(dn_bytes / dn_s / HBM_PEAK, 4)}
        dtype = "int8 x int8 -> int32 (weights exact, activations as two int8 planes), fp32 scales"
    else:
        op = {"grouped_i8": "int8", "grouped_f16": "fp16", "grouped_fp8": "fp8"}[path]
        kname = {"grouped_i8": "plane_gemm_k<2, %s> (grouped gate + up int8 MFMA product + SwiGLU)" % cfg["fmt"],
                 "grouped_f16": "expert_gemm_f16_k<%s,2> (grouped gate + up fp16 MFMA product + SwiGLU)" % cfg["fmt"],
                 "grouped_fp8": "plane_gemm_k<2, %s> (grouped gate + up fp8 MFMA product + SwiGLU)" % cfg["fmt"]}[path]
        roofline = {"bound": "mfma", "kernel": kname, "achieved": round(gu_ops / gu_s / 1e12, 2), "peak": PEAK[op] / 1e12, "unit": "TFLOP/s",
                    "frac": round(gu_ops / gu_s / PEAK[op], 4), "traffic": None,
                    "ops": "multiply-add = 2 operations; peak = dense %s %.1f POP/s" % (op, PEAK[op] / 1e15),
                    "algorithmic_ops_per_launch": int(gu_ops), "us_per_launch": round(gu_s * 1e6, 2),
                    "hbm_frac": round(gu_bytes / gu_s / HBM_PEAK, 4)}
        layer = {"algorithmic_ops_per_step": int(gu_ops + dn_ops), "mfma_frac": round((gu_ops + dn_ops) / step_s / PEAK[op], 4),
                 "algorithmic_bytes_per_step": int(layer_bytes), "hbm_frac": round(layer_bytes / step_s / HBM_PEAK, 4),
                 "down_us": round(dn_s * 1e6, 2), "down_mfma_frac": round(dn_ops / dn_s / PEAK[op], 4)}
        dtype = {"int8": "int8 x int8 -> int32 MFMA (weights exact, per-row int8 activations), fp32 scales",
                 "fp16": "fp16 x fp16 -> fp32 MFMA (weights and activations rounded to fp16)",
                 "fp8": "E4M3 x E4M3 -> fp32 MFMA (weights and activations rounded to E4M3), fp32 scales"}[op]
    # HBM bytes per launch of the roofline kernel as the counters saw them (a committed measurement of this same point)
    roofline["traffic"] = traffic.get("config%s_tokens_%d" % (key, T), {}).get("bytes_per_launch")
    del layers, xs, outs, prep
    torch.cuda.empty_cache()
    return {"tokens": T, "tokens_per_s": round(T / step_s, 1), "ms_per_step": round(ms_step, 5), "steps": K, "warmup": W,
            "path": path, "launch": launch, "distinct_steps": len(cycle), "routing": "N(0,1) logits + Zipf(%.1f) popularity bias" % ZIPF_S if skew else "random router",
            "distinct_experts_per_step": round(u_mean, 1), "dtype": dtype, "roofline": roofline, "layer": layer}


def cpu_baseline(cfg, budget_s=12.0):
    """CPU expert path on this box's cores at the layer's shape and format (see oracle.cpu_baseline_sweep); beside it the
    reference program's own shape (IQ4_NL 640 x 2560, 24 experts) and configuration 1 as a whole layer on the host."""
    import oracle
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else oracle.hardware_threads()
    cores = max(1, min(cores, 64))
    rec = oracle.cpu_baseline_sweep(cfg["wtype"], cfg["hidden"], cfg["ff"], cfg["topk"] + (1 if cfg["shared_ff"] else 0), cores, budget_s)
    rec["reference_shape"] = oracle.cpu_reference_shape(cores)
    rec["config1_layer"] = oracle.cpu_config1_layer(cores)
    return rec


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400, help="timed steps per point: exactly this many, one after the other")
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--config", default="2", choices=sorted(CONFIGS), help="benchmark configuration (2 covers configurations 2 and 3)")
    ap.add_argument("--tokens", type=int, default=None, help="measure this one point instead of the configuration's list")
    ap.add_argument("--banks", type=int, default=8, help="independent expert banks the steps rotate over")
    ap.add_argument("--no-graph", action="store_true", help="launch every step from the host instead of replaying a HIP graph")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--act-blocks", action="store_true", help="int8 grouped products with a scale per 32 activations in place of one per token "
                    "(the reference's TQFN_PREFILL_INT8=1); the headline numbers are measured without it")
    ap.add_argument("--copy-mb", type=int, default=0, help="also run one plain device copy of this many MiB (a kernel of known "
                    "traffic that calibrates the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run of this command)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus %d is not supported (nothing here uses a second GPU)" % args.gpus)

    import torch

    import tqllm_amd as tq
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the library has no CPU path")
    torch.cuda.set_device(0)
    if args.copy_mb > 0:
        src = torch.empty(args.copy_mb << 20, dtype=torch.uint8, device="cuda").random_(0, 255)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    cfg = CONFIGS[args.config]
    try:
        with open(TRAFFIC_FILE) as f:
            traffic = json.load(f)
    except (OSError, ValueError):
        traffic = {}
    trios, gen = build_banks(torch, tq, cfg, args.banks, seed=1234)
    tokens = (args.tokens,) if args.tokens else cfg["points"]
    points = [measure_point(torch, tq, cfg, args.config, trios, gen, T, args, traffic) for T in tokens]
    head = points[-1]   # the largest point: 4096 tokens in the default run
    line = {
        "metric": "MoE-layer tokens/s", "value": head["tokens_per_s"], "unit": "tokens/s", "n_gpus": 1,
        "steps": head["steps"], "warmup": head["warmup"], "ms_per_step": head["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": head["dtype"],
        "data": "synthetic: banks of random valid %s blocks with block scales sized for weights of about 0.02 (not N(0, 0.02) values run through an "
                "encoder: the time does not depend on the codes), N(0,1) activations; %d rotating banks, %d distinct steps per cycle"
                % (cfg["fmt"], args.banks, head["distinct_steps"]),
        "config": {"workload": "%s; T=%d, %s" % (cfg["label"], head["tokens"], head["routing"]), "tokens": head["tokens"], "launch": head["launch"],
                   "path": head["path"], "distinct_experts_per_step": head["distinct_experts_per_step"],
                   "points": "tokens " + ", ".join(str(p["tokens"]) for p in points),
                   "activation_scales": "per 32 values" if args.act_blocks else "per token"},
        "roofline": head["roofline"], "layer": head["layer"], "points": points,
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(cfg)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
