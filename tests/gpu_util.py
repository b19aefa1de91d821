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
