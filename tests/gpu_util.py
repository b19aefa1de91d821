"""Helpers shared by the GPU parity tests: numpy <-> device tensors in the storage types the configs name."""
import numpy as np
import torch

import oracle
import tqllm_amd as tq


def dev(pair_or_array, kind=None):
    """(storage, values) pair from synth.make_inputs, or a plain array, as a cuda tensor of the storage type."""
    if isinstance(pair_or_array, tuple):
        storage = pair_or_array[0]
        if storage.dtype == np.uint16:
            return torch.from_numpy(storage.view(np.int16)).cuda().view(torch.bfloat16)
        return torch.from_numpy(storage).cuda()
    return torch.from_numpy(np.ascontiguousarray(pair_or_array)).cuda()


def banks_on_device(cfg, raws):
    h, f = cfg["hidden"], cfg["ff"]
    e = cfg["experts"] + (1 if cfg["shared_ff"] else 0)
    return [tq.ExpertBank(cfg["wtype"], raw, e, rows, cols) for raw, (rows, cols) in zip(raws, ((f, h), (f, h), (h, f)))]


def oracle_type(kind):
    return {"f32": oracle.F32, "bf16": oracle.BF16, "f16": oracle.F16}[kind]


def clear_tokens(oracle, logits, experts, k, ids=None, want_ids=None, label=""):
    """Tokens on which the routing ids must equal the reference's bit for bit: all but those where the reference's own
    choice rests on two different logits rounding to one fp32 probability (or on subnormal probabilities), which no
    other exp() implementation can be asked to reproduce. Prints how many tokens are exempt and, when the ids are given,
    how many of the exempt ones actually differ; at most one token in 500 may be exempt."""
    import numpy as np
    tie = oracle.route_softmax_collision(logits[:, :experts], k)
    differ = int((ids[tie] != want_ids[tie]).any(axis=1).sum()) if ids is not None and tie.any() else 0
    print("%srouting: %d of %d tokens exempt (probability ties between different logits), %d of them differ" % (label and label + ": ", int(tie.sum()), len(tie), differ))
    assert tie.sum() <= max(1, len(tie) // 500), "too many exempt tokens: pick another seed"
    return ~tie


def selection_values(logits, gating, bias):
    """float64 selection values of moe_route (src/experts/moe.cpp:33-65) per token and expert"""
    lg = logits.astype(np.float64)
    if gating == 1:
        p = np.exp(lg - lg.max(axis=1, keepdims=True))
        p /= p.sum(axis=1, keepdims=True)
    elif gating == 2:
        p = 1 / (1 + np.exp(-lg))
    elif gating == 3:
        p = lg
    else:
        p = np.sqrt(np.logaddexp(0, lg))
    return p + bias.astype(np.float64) if bias is not None else p


def clear_tokens_gated(logits, experts, k, gating, bias, ids=None, want_ids=None, label="", most=None):
    """The other gating functions have no collision rule an oracle could state exactly (sigmoid, softplus and their sums with a
    bias round differently in every libm), so a token is exempt from the bit-exact id check when two of its k + 1 largest
    selection values, computed in float64 here, lie within the fp32 rounding of the value (2e-6 relative, plus the bias'
    magnitude). Prints how many tokens are exempt and how many differ; at most `most` (default one in 250, at least one)
    may be exempt, and the caller asserts that no other token differs."""
    v = -np.sort(-selection_values(logits[:, :experts], gating, bias), axis=1)[:, :k + 1]
    room = 2e-6 * (np.abs(v[:, :-1]) + (float(np.abs(bias).max()) if bias is not None else 0.0))
    clear = (v[:, :-1] - v[:, 1:] > room).all(axis=1)
    exempt = int((~clear).sum())
    differ = int((ids != want_ids).any(axis=1).sum()) if ids is not None else 0
    if exempt or differ:
        print("%srouting (gating %d): %d of %d tokens exempt (selection values within fp32 rounding), %d tokens differ" % (label and label + ": ", gating, exempt, len(clear), differ))
    assert exempt <= (max(1, len(clear) // 250) if most is None else most), "too many exempt tokens: pick another seed"
    return clear


def oracle_mode(layer, n):
    """the oracle's operand mode for the products a batch of n tokens takes: fp32 activations for the decode kernels and
    the fp16 grouped products, the declared 8-bit quantisers for the int8 and fp8 grouped products"""
    return {"decode": 0, "grouped_f16": 0, "grouped_i8": 5, "grouped_fp8": 2}[layer.path(n)]
