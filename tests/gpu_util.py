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


def oracle_mode(layer, n):
    """the oracle's operand mode for the products a batch of n tokens takes: fp32 activations for the decode kernels and
    the fp16 grouped products, the declared 8-bit quantisers for the int8 and fp8 grouped products"""
    return {"decode": 0, "grouped_f16": 0, "grouped_i8": 5, "grouped_fp8": 2}[layer.path(n)]
