#!/usr/bin/env python3
"""MoE-layer benchmark on one MI355X: the Flash-Next-shaped IQ4_XS layer, as decode (configuration 2 of the benchmark definition, the default:
--tokens 16, also 1 and 4) or as prefill (config 3: --tokens 4096, Zipf-skewed routing, int8 MFMA grouped products).

A step is one pass of the whole layer (router, top-k, gate/up + SwiGLU, down + combine, shared expert) over one batch of
T tokens, with every input already resident in HBM. Steps rotate over several independent expert banks so that the
weights of a step stream from HBM, not from the 256 MB last-level cache. One JSON line is printed:
  value     MoE-layer tokens/s (T / mean step time), whole job = this one GPU
  roofline  the dominant kernel (fused gate/up + SwiGLU) over its mean duration, measured with HIP events around
            back-to-back launches of that kernel alone: decode = algorithmic bytes of the distinct experts it must read
            against 8 TB/s; prefill = int8 operations (2 per multiply-add) of its assignments against 5.0 POP/s
  cpu_baseline  the CPU expert path (port of the reference's tests/bench_cpu_expert_mt.cpp scheme to IQ4_XS at this
            layer's shape) timed on this box's host cores on a bounded sample
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")   # measured with rocprofv3 --pmc (see the file)
HBM_PEAK = 8.0e12  # bytes/s, MI355X published
INT8_PEAK = 5.0e15  # dense int8 operations/s, MI355X published
PREFILL_MIN = 64   # token counts from here up take the grouped int8 products inside the library
ZIPF_S = 1.1
CFG = dict(hidden=2048, ff=512, experts=512, topk=10, shared_ff=512)
IQ4_XS_BYTES_PER_WEIGHT = 136.0 / 256.0


def random_iq4xs_bank(torch, experts, rows, cols, gen):
    """GGUF IQ4_XS block stream of random valid blocks on the device (random codes and sub-scales, small finite fp16
    super-scales, as the reference's device tests make their banks: tests/moe_device.cu:121-138)."""
    nb = experts * rows * cols // 256
    raw = torch.randint(0, 256, (nb, 136), dtype=torch.uint8, device="cuda", generator=gen)
    d = (torch.rand(nb, device="cuda", generator=gen) * 4e-5 + 4e-5).to(torch.float16)
    d = d * (torch.randint(0, 2, (nb,), device="cuda", generator=gen) * 2 - 1).to(torch.float16)
    raw[:, 0:2] = d.view(torch.uint8).reshape(nb, 2)
    return raw.reshape(-1)


def build_layers(torch, tq, banks, tokens, seed):
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    h, f, e = CFG["hidden"], CFG["ff"], CFG["experts"] + 1
    layers, xs = [], []
    for _ in range(banks):
        trio = []
        for rows, cols in ((f, h), (f, h), (h, f)):
            raw = random_iq4xs_bank(torch, e, rows, cols, gen)
            trio.append(tq.ExpertBank(tq.IQ4_XS, raw, e, rows, cols))
            del raw
        skew = tokens >= PREFILL_MIN
        router = torch.randn((CFG["experts"], h), device="cuda", generator=gen) * (h ** -0.5 if skew else 0.02)
        x = torch.randn((tokens, h), device="cuda", generator=gen)
        if skew:
            # logits = N(0, 1) + ln p_e, p_e ~ rank^-1.1 over a random permutation of the experts: the bias rides in the
            # last router column against a constant 1 in the last activation
            p = 1.0 / torch.arange(1, CFG["experts"] + 1, device="cuda", dtype=torch.float64) ** ZIPF_S
            p = (p / p.sum())[torch.randperm(CFG["experts"], device="cuda", generator=gen)]
            router[:, -1] = torch.log(p).float()
            x[:, -1] = 1.0
        sgate = (torch.randn((h,), device="cuda", generator=gen) * 0.02).to(torch.bfloat16)
        layers.append(tq.MoeLayer(router.to(torch.bfloat16), sgate, *trio, CFG["topk"], shared_ff=CFG["shared_ff"]))
        xs.append(x.to(torch.bfloat16))
    torch.cuda.synchronize()
    return layers, xs


def time_steps(torch, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(steps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / steps  # ms per call


def cpu_baseline(sample_experts=24, budget_s=12.0):
    """CPU expert path on this box's cores: `sample_experts` IQ4_XS experts (gate, up 512x2048; down 2048x512), one token
    each, int8 activations per 32-block, all hardware threads pulling experts from a shared counter."""
    import numpy as np

    import oracle
    rng = np.random.default_rng(7)
    h, f = CFG["hidden"], CFG["ff"]
    banks = []
    for rows, cols in ((f, h), (f, h), (h, f)):
        nb = sample_experts * rows * cols // 256
        raw = rng.integers(0, 256, (nb, 136), dtype=np.uint8)
        raw[:, 0:2] = np.float16(rng.uniform(4e-5, 8e-5, nb)).view(np.uint8).reshape(nb, 2)
        banks.append(raw.reshape(-1))
    # the GPU box reports every core of its host; a job's share is what the affinity mask allows
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else oracle.hardware_threads()
    cores = max(1, min(cores, 64))
    t0 = time.time()
    t_pass, _ = oracle.cpu_expert_bench(oracle.IQ4_XS, *banks, h, f, sample_experts, cores, True, reps=1)
    reps = int(max(1, min(4000, budget_s / max(t_pass, 1e-4) - 2)))   # about budget_s seconds of CPU work
    t_pass, _ = oracle.cpu_expert_bench(oracle.IQ4_XS, *banks, h, f, sample_experts, cores, True, reps=reps)
    per_layer_token = t_pass / sample_experts * (CFG["topk"] + 1)
    return {"value": round(1.0 / per_layer_token, 2), "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": "%d IQ4_XS experts (gate/up 512x2048, down 2048x512), one token, int8 activations per 32-block, %d threads on an "
                      "atomic expert queue, %d timed passes of %.1f ms; tokens/s = 1 / (11 experts x mean time per expert); %.1f s of CPU work"
                      % (sample_experts, cores, reps, t_pass * 1e3, time.time() - t0)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed steps (default 400; 80 at prefill sizes)")
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--tokens", type=int, default=16, help="decode batch of the step (configuration 2 names 1, 4 and 16)")
    ap.add_argument("--banks", type=int, default=8, help="independent expert banks the steps rotate over")
    ap.add_argument("--no-graph", action="store_true", help="launch every step from the host instead of replaying a HIP graph")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
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
    T, R = args.tokens, args.banks
    if args.copy_mb > 0:
        src = torch.empty(args.copy_mb << 20, dtype=torch.uint8, device="cuda").random_(0, 255)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if args.steps is None:
        args.steps = 400 if T < PREFILL_MIN else 80
    if args.warmup is None:
        args.warmup = 40 if T < PREFILL_MIN else 8
    layers, xs = build_layers(torch, tq, R, T, seed=1234)
    outs = [torch.empty((T, CFG["hidden"]), dtype=torch.float32, device="cuda") for _ in range(R)]
    for l in layers:
        l.workspace(T)

    # ---- whole layer: K steps, rotating banks; a HIP graph of R steps is replayed so that the host is not the bound
    def eager_round():
        for l, x, o in zip(layers, xs, outs):
            l.forward(x, out=o)

    steps = max(R, args.steps // R * R)
    warm = max(R, args.warmup // R * R)
    launch = "eager"
    round_fn = eager_round
    if not args.no_graph:
        try:
            eager_round()
            torch.cuda.synchronize()
            ref = [o.clone() for o in outs]
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                eager_round()
            for _ in range(3):          # replays must reproduce the eager result
                for o in outs:
                    o.zero_()
                g.replay()
                torch.cuda.synchronize()
                assert all(torch.equal(a, b) for a, b in zip(ref, outs)), "graph replay differs from the eager result"
            round_fn, launch = g.replay, "hipgraph(%d steps)" % R
        except Exception as ex:  # noqa: BLE001
            print("bench.py: HIP graph path unavailable (%s); timing eager launches" % ex, file=sys.stderr)
    ms_round = time_steps(torch, round_fn, steps // R, warm // R)
    ms_step = ms_round / R

    # ---- routing statistics of the steps (distinct experts a step must read)
    uniq, routing = [], []
    for l, x in zip(layers, xs):
        _, ids, _, _ = l.forward(x, return_routing=True)
        uniq.append(int(torch.unique(ids).numel()))
        routing.append(ids)
    u_mean = sum(uniq) / len(uniq)
    per_expert = 3 * CFG["ff"] * CFG["hidden"] * IQ4_XS_BYTES_PER_WEIGHT
    layer_bytes = (u_mean + 1) * per_expert + (CFG["experts"] + 1) * CFG["hidden"] * 2 + T * CFG["hidden"] * 2 * 2
    slots = CFG["topk"] + 1
    prefill = T >= PREFILL_MIN

    # ---- dominant kernels alone: back-to-back launches over the rotating banks, inputs prepared once
    prep = []
    for l, x, ids in zip(layers, xs, routing):
        ext = tq.moe_extend_ids(ids, CFG["experts"])
        if prefill:
            counts, offsets, perm, _ = tq.moe_dispatch(ext, CFG["experts"] + 1)
            lists = (counts, offsets, perm)
            xq, xsc = tq.group_rows_i8(x, lists, T * slots, slots)
            act = tq.expert_gemm_gateup_i8(l.gate, l.up, xq, xsc, lists, T, slots, CFG["topk"], CFG["shared_ff"])
            aq, asc = tq.group_rows_i8(act, lists, T * slots, 1)
            prep.append((l, lists, xq, xsc, aq, asc))
        else:
            img = tq.quant_act(x)
            act = tq.expert_gateup(l.gate, l.up, img, ext, CFG["topk"], shared_ff=CFG["shared_ff"])
            y = tq.expert_down(l.down, act, ext, CFG["topk"], shared_ff=CFG["shared_ff"])
            prep.append((l, ext, img, act, y))

    def gateup_round():
        for item in prep:
            if prefill:
                l, lists, xq, xsc, aq, asc = item
                tq.expert_gemm_gateup_i8(l.gate, l.up, xq, xsc, lists, T, slots, CFG["topk"], CFG["shared_ff"])
            else:
                l, ext, img, act, y = item
                tq.expert_gateup(l.gate, l.up, img, ext, CFG["topk"], shared_ff=CFG["shared_ff"], act_image=act)

    def down_round():
        for item in prep:
            if prefill:
                l, lists, xq, xsc, aq, asc = item
                tq.expert_gemm_i8(l.down, aq, asc, lists, T, slots, CFG["topk"], CFG["shared_ff"])
            else:
                l, ext, img, act, y = item
                tq.expert_down(l.down, act, ext, CFG["topk"], shared_ff=CFG["shared_ff"], y=y)

    kernels = {}
    reps = 1 if prefill else 4
    for name, fn in (("gateup", gateup_round), ("down", down_round)):
        fn()
        torch.cuda.synchronize()
        timed = fn
        if not prefill:   # microsecond kernels: replay a graph of them so that the host is not the bound
            gk = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gk):
                for _ in range(reps):
                    fn()
            timed = gk.replay
        kernels[name] = time_steps(torch, timed, max(4, steps // (reps * R)), 2) / (reps * R)  # ms per launch
    gu_bytes = (u_mean + 1) * 2 * CFG["ff"] * CFG["hidden"] * IQ4_XS_BYTES_PER_WEIGHT
    dn_bytes = (u_mean + 1) * CFG["ff"] * CFG["hidden"] * IQ4_XS_BYTES_PER_WEIGHT
    gu_ops = T * slots * 2 * CFG["ff"] * CFG["hidden"] * 2.0      # int8 multiply-adds of gate and up, 2 operations each
    dn_ops = T * slots * CFG["ff"] * CFG["hidden"] * 2.0

    if prefill:
        achieved = gu_ops / (kernels["gateup"] * 1e-3)
        roofline = {"bound": "mfma", "kernel": "iq4xs_gemm_k<2> (grouped gate + up int8 MFMA product + SwiGLU)", "achieved": round(achieved / 1e12, 2),
                    "peak": INT8_PEAK / 1e12, "unit": "TFLOP/s", "frac": round(achieved / INT8_PEAK, 4), "traffic": None,
                    "ops": "int8 multiply-add = 2 operations; peak = dense int8 5.0 POP/s",
                    "algorithmic_ops_per_launch": int(gu_ops), "us_per_launch": round(kernels["gateup"] * 1e3, 2)}
        layer = {"algorithmic_ops_per_step": int(gu_ops + dn_ops), "mfma_frac": round((gu_ops + dn_ops) / (ms_step * 1e-3) / INT8_PEAK, 4),
                 "algorithmic_bytes_per_step": int(layer_bytes), "hbm_frac": round(layer_bytes / (ms_step * 1e-3) / HBM_PEAK, 4),
                 "down_us": round(kernels["down"] * 1e3, 2), "down_mfma_frac": round(dn_ops / (kernels["down"] * 1e-3) / INT8_PEAK, 4)}
        workload = ("config 3: Flash-Next-shaped prefill layer, hidden 2048, 512 IQ4_XS experts top-10 + shared (ff 512), T=%d, router logits N(0,1) + "
                    "Zipf(%.1f) popularity bias, per-row int8 activations" % (T, ZIPF_S))
        dtype = "int8 x int8 -> int32 MFMA, fp32 scales (IQ4_XS weights exact, per-row int8 activations)"
    else:
        achieved = gu_bytes / (kernels["gateup"] * 1e-3)
        roofline = {"bound": "hbm", "kernel": "iq4xs_mfma_k<2> (gate + up + SwiGLU)", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9,
                    "unit": "GB/s", "frac": round(achieved / HBM_PEAK, 4), "traffic": None,
                    "algorithmic_bytes_per_launch": int(gu_bytes), "us_per_launch": round(kernels["gateup"] * 1e3, 2)}
        layer = {"algorithmic_bytes_per_step": int(layer_bytes), "hbm_frac": round(layer_bytes / (ms_step * 1e-3) / HBM_PEAK, 4),
                 "down_us": round(kernels["down"] * 1e3, 2), "down_hbm_frac": round(dn_bytes / (kernels["down"] * 1e-3) / HBM_PEAK, 4)}
        workload = "config 2: Flash-Next-shaped decode layer, hidden 2048, 512 IQ4_XS experts top-10 + shared (ff 512), T=%d" % T
        dtype = "int8 x int8 -> int32 MFMA, fp32 scales (IQ4_XS weights exact, bf16 activations as 2 x int8 planes)"

    # HBM bytes per launch of the roofline kernel as the counters saw them (a committed measurement of this same command)
    try:
        with open(TRAFFIC_FILE) as f:
            roofline["traffic"] = json.load(f).get("tokens_%d" % T, {}).get("bytes_per_launch")
    except (OSError, ValueError):
        pass

    line = {
        "metric": "MoE-layer tokens/s", "value": round(T / (ms_step * 1e-3), 1), "unit": "tokens/s", "n_gpus": 1,
        "steps": steps, "warmup": warm, "ms_per_step": round(ms_step, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dtype,
        "data": "synthetic: random valid IQ4_XS blocks, bf16 router, bf16 N(0,1) activations; %d rotating banks" % R,
        "config": {"workload": workload, "tokens": T, "launch": launch, "distinct_experts_per_step": round(u_mean, 1)},
        "roofline": roofline, "layer": layer,
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
