"""ctypes binding of libtqmoe.so and the host-side mirror of the reference's MoE operator interface.

Names follow the reference: moe_router / moe_topk / moe_group (here moe_dispatch, the deterministic form) / moe_swiglu /
moe_sum (here moe_combine) of src/experts/moe_kernels.cuh, and expert_matvec / expert_matvec2 of tqllm::WeightFormat
(src/formats/weight/weight_format.hpp:62-73). Every function enqueues on torch's current stream of the tensors' device
and raises TqmoeError with the library's message on failure. There is no fallback path: a missing library or a missing
GPU is an error.
"""
import ctypes as C
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libtqmoe.so")

F32, F16, BF16 = 0, 1, 30
Q4_K, IQ3_S, IQ4_XS, NVFP4G = 12, 21, 23, 323
Q8_0, IQ4_NL, Q5_K, Q6_K, IQ3_XXS, IQ2_S = 8, 20, 13, 14, 18, 22
Q4_0, Q3_K, IQ2_XXS, IQ2_XS = 2, 11, 16, 17
Q2_K, IQ1_S = 10, 19
GATE_SOFTMAX, GATE_SIGMOID, GATE_SOFTMAX_WEIGHT, GATE_SQRT_SOFTPLUS = 1, 2, 3, 4   # MoeGating, src/experts/moe.hpp:20-26
BLOCK = {Q4_K: (256, 144), IQ3_S: (256, 110), IQ4_XS: (256, 136), NVFP4G: (128, 76), IQ4_NL: (32, 18), Q8_0: (32, 34), Q5_K: (256, 176), Q6_K: (256, 210), IQ3_XXS: (256, 98), IQ2_S: (256, 82), Q4_0: (32, 18), Q3_K: (256, 110), IQ2_XXS: (256, 66), IQ2_XS: (256, 74), Q2_K: (256, 84), IQ1_S: (256, 50)}
_TORCH_TYPE = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}
_OUT_TYPE = {F32: torch.float32, BF16: torch.bfloat16}


class TqmoeError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("tqmoe error %d: %s" % (code, message))
        self.code = code


class _Error(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("code", C.c_int32), ("message", C.c_char * 256)]


class _Bank(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("type", C.c_uint32), ("experts", C.c_int32), ("rows", C.c_int32),
                ("cols", C.c_int32), ("codes", C.c_void_p), ("aux", C.c_void_p)]


class _Layer(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("hidden", C.c_int32), ("ff", C.c_int32), ("n_expert", C.c_int32),
                ("topk", C.c_int32), ("has_shared", C.c_int32), ("shared_ff", C.c_int32), ("weight_scale", C.c_float),
                ("router", C.c_void_p), ("shared_gate", C.c_void_p), ("router_type", C.c_uint32),
                ("gate", _Bank), ("up", _Bank), ("down", _Bank),
                ("gating", C.c_int32), ("raw_weights", C.c_int32), ("probs_bias", C.c_void_p), ("act_blocks", C.c_int32),
                ("swiglu_clamp", C.c_float), ("clamp_gate", C.c_int32)]


_lib = None


def lib():
    """The loaded library; raises when it has not been built (python -m tqllm_amd.build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise TqmoeError(-3, "libtqmoe.so is not built: run `python -m tqllm_amd.build` (there is no fallback path)")
        l = C.CDLL(LIB_PATH)
        p, i32, i64, u32, f32, sz = C.c_void_p, C.c_int32, C.c_int64, C.c_uint32, C.c_float, C.c_size_t
        e = C.POINTER(_Error)
        l.tqmoe_abi_version.restype = u32
        l.tqmoe_router.argtypes = [p, u32, p, p, u32, p, i32, i32, i32, p, e]
        l.tqmoe_topk.argtypes = [p, p, p, p, i32, i32, i32, f32, p, e]
        l.tqmoe_topk2.argtypes = [p, p, p, p, p, p, p, p, i32, i32, i32, f32, p, e]
        l.tqmoe_topk_gated.argtypes = [p, p, i32, i32, p, p, p, i32, i32, i32, f32, p, e]
        l.tqmoe_dispatch_workspace_bytes.restype = sz
        l.tqmoe_dispatch_workspace_bytes.argtypes = [i32, i32, i32]
        l.tqmoe_dispatch.argtypes = [p, p, p, p, p, i32, i32, i32, i32, p, sz, p, e]
        l.tqmoe_dispatch_static.argtypes = [p, p, p, p, p, i32, i32, i32, i32, p, e]
        l.tqmoe_static_scratch_init.argtypes = [e]
        l.tqmoe_count.argtypes = [p, p, i32, p, e]
        l.tqmoe_dedup_maps.argtypes = [p, p, i32, i32, p, p, p, i32, p, e]
        l.tqmoe_lists_from_groups_clamped.argtypes = [p, p, i32, i32, p, p, p, p, e]
        l.tqmoe_expert_gemm_i8_ref_scratch_bytes.restype = sz
        l.tqmoe_expert_gemm_i8_ref_scratch_bytes.argtypes = [i32, i64, i32, i32]
        l.tqmoe_expert_gemm_i8_ref.argtypes = [C.POINTER(_Bank), p, p, p, p, u32, p, p, i32, i32, i32, i32, i32, i64, p, sz, p, e]
        l.tqmoe_swiglu_clamped.argtypes = [p, p, p, i64, f32, i32, p, e]
        l.tqmoe_expert_matvec_dedup_scratch_bytes.restype = sz
        l.tqmoe_expert_matvec_dedup_scratch_bytes.argtypes = [i32, i32, i32, u32, i32]
        l.tqmoe_expert_matvec_dedup.argtypes = [C.POINTER(_Bank), C.POINTER(_Bank), p, u32, p, p, u32, p, i32, p, sz, p, e]
        l.tqmoe_bank_layout.argtypes = [u32, i64, i32, C.POINTER(sz), C.POINTER(sz), e]
        l.tqmoe_bank_load.argtypes = [u32, p, i64, i32, p, p, p, p, e]
        l.tqmoe_bank_dequant.argtypes = [C.POINTER(_Bank), i64, i64, p, p, e]
        l.tqmoe_act_image_bytes.restype = sz
        l.tqmoe_act_image_bytes.argtypes = [i32, i32]
        l.tqmoe_quant_act.argtypes = [p, u32, i32, i32, p, p, e]
        l.tqmoe_expert_matvec.argtypes = [C.POINTER(_Bank), p, p, u32, p, i32, i32, i32, p, e]
        l.tqmoe_expert_matvec2.argtypes = [C.POINTER(_Bank), C.POINTER(_Bank), p, p, p, u32, p, i32, i32, p, e]
        l.tqmoe_expert_matvec_rows.argtypes = [C.POINTER(_Bank), p, u32, p, u32, p, i32, i32, i32, p, sz, p, e]
        l.tqmoe_expert_matvec2_rows.argtypes = [C.POINTER(_Bank), C.POINTER(_Bank), p, u32, p, p, u32, p, i32, i32, p, sz, p, e]
        l.tqmoe_lists_from_groups.argtypes = [p, p, i32, i32, p, p, p, e]
        l.tqmoe_extend_ids.argtypes = [p, p, i32, i32, i32, p, e]
        l.tqmoe_expert_gateup.argtypes = [C.POINTER(_Bank), C.POINTER(_Bank), p, p, p, i32, i32, i32, i32, p, e]
        l.tqmoe_expert_down.argtypes = [C.POINTER(_Bank), p, p, p, i32, i32, i32, i32, p, e]
        l.tqmoe_combine_strided.argtypes = [p, i32, p, i64, p, p, p, u32, i32, i32, i32, p, e]
        l.tqmoe_combine_strided_f16.argtypes = [p, i32, p, i64, p, p, p, u32, i32, i32, i32, p, e]
        l.tqmoe_combine_residual.argtypes = [p, u32, i32, p, i64, p, p, p, p, i32, i32, i32, p, e]
        l.tqmoe_add_rmsnorm.argtypes = [p, p, p, f32, p, u32, i32, i32, p, e]
        l.tqmoe_layer_forward_residual.argtypes = [C.POINTER(_Layer), p, u32, p, i32, p, p, p, p, p, sz, p, e]
        l.tqmoe_quant_rows_i8.argtypes = [p, u32, i64, i32, p, p, p, e]
        l.tqmoe_grouped_rows.restype = i64
        l.tqmoe_grouped_rows.argtypes = [i64, i32]
        l.tqmoe_grouped_scale_words.restype = i64
        l.tqmoe_grouped_scale_words.argtypes = [i64, i32]
        l.tqmoe_group_rows_i8.argtypes = [p, u32, i32, p, p, p, i32, i64, i32, p, p, p, e]
        l.tqmoe_gather_rows_i8.argtypes = [p, p, i32, p, p, p, i32, i64, i32, p, p, p, e]
        l.tqmoe_expert_gemm_gateup_i8.argtypes = [C.POINTER(_Bank), C.POINTER(_Bank), p, p, p, p, p, i32, i32, i32, i32, p, p, e]
        l.tqmoe_expert_gemm_i8.argtypes = [C.POINTER(_Bank), p, p, p, p, p, i32, i32, i32, i32, p, p, e]
        l.tqmoe_quant_rows_i8_blocks.argtypes = [p, u32, i64, i32, p, p, p, p, e]
        l.tqmoe_grouped_block_scale_words.restype = i64
        l.tqmoe_grouped_block_scale_words.argtypes = [i64, i32, i32]
        l.tqmoe_group_rows_i8_blocks.argtypes = [p, u32, i32, p, p, p, i32, i64, i32, p, p, p, p, e]
        l.tqmoe_gather_rows_i8_blocks.argtypes = [p, p, i32, p, p, p, i32, i64, i32, p, p, p, p, e]
        l.tqmoe_expert_gemm_gateup_i8_blocks.argtypes = [C.POINTER(_Bank), C.POINTER(_Bank), p, p, p, p, p, p, i32, i32, i32, i32, p, p, e]
        l.tqmoe_expert_gemm_i8_blocks.argtypes = [C.POINTER(_Bank), p, p, p, p, p, p, i32, i32, i32, i32, p, p, e]
        l.tqmoe_quant_rows_fp8.argtypes = l.tqmoe_quant_rows_i8.argtypes
        l.tqmoe_group_rows_fp8.argtypes = l.tqmoe_group_rows_i8.argtypes
        l.tqmoe_expert_gemm_gateup_fp8.argtypes = l.tqmoe_expert_gemm_gateup_i8.argtypes
        l.tqmoe_expert_gemm_fp8.argtypes = l.tqmoe_expert_gemm_i8.argtypes
        l.tqmoe_expert_gemm_gateup.argtypes = [C.POINTER(_Bank), C.POINTER(_Bank), p, u32, p, p, p, i32, i32, i32, i32, p, p, e]
        l.tqmoe_expert_gemm.argtypes = [C.POINTER(_Bank), p, u32, p, p, p, i32, i32, i32, i32, i32, p, u32, p, e]
        l.tqmoe_swiglu.argtypes = [p, p, p, i64, p, e]
        l.tqmoe_combine.argtypes = [p, p, p, p, p, u32, i32, i32, i32, p, e]
        l.tqmoe_layer_workspace_bytes.restype = sz
        l.tqmoe_layer_workspace_bytes.argtypes = [C.POINTER(_Layer), i32]
        l.tqmoe_layer_forward.argtypes = [C.POINTER(_Layer), p, u32, i32, p, u32, p, p, p, p, sz, p, e]
        l.tqmoe_layer_path.argtypes = [C.POINTER(_Layer), i32]
        for name in ("tqmoe_router", "tqmoe_topk", "tqmoe_topk2", "tqmoe_dispatch", "tqmoe_bank_layout", "tqmoe_bank_load", "tqmoe_bank_dequant",
                     "tqmoe_quant_act", "tqmoe_expert_matvec", "tqmoe_expert_matvec2", "tqmoe_extend_ids", "tqmoe_expert_gateup", "tqmoe_expert_down", "tqmoe_combine_strided", "tqmoe_swiglu", "tqmoe_combine",
                     "tqmoe_layer_forward"):
            getattr(l, name).restype = i32
        _lib = l
    return _lib


def abi_version():
    return lib().tqmoe_abi_version()


def _err():
    return _Error(C.sizeof(_Error), 0, b"")


def _check(rc, err):
    if rc:
        raise TqmoeError(rc, err.message.decode("utf-8", "replace"))


def _ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else None


def _stream(t):
    if not t.is_cuda:
        raise TqmoeError(-3, "tensors must live on the GPU (there is no CPU path)")
    return C.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _ttype(t):
    try:
        return _TORCH_TYPE[t.dtype]
    except KeyError:
        raise TqmoeError(-2, "unsupported tensor dtype %s" % t.dtype)


def moe_router(router, shared_gate, x, experts=None):
    """logits [n][E + 1] fp32 = x @ [router; shared_gate]^T (moe_kernels.cuh:7-10)."""
    n, hidden = x.shape
    e = router.shape[0] if experts is None else experts
    logits = torch.empty((n, e + 1), dtype=torch.float32, device=x.device)
    err = _err()
    _check(lib().tqmoe_router(_ptr(router), _ttype(router), _ptr(shared_gate), _ptr(x), _ttype(x), _ptr(logits), hidden, e, n,
                              _stream(x), C.byref(err)), err)
    return logits


def moe_topk(logits, experts, topk, scale=1.0, gating=GATE_SOFTMAX, bias=None, norm=True):
    """ids [n][k] int32, weights [n][k] fp32, shared_weights [n] fp32 (moe_kernels.cuh:19-20). gating, bias (fp32 [experts],
    added for the choice only) and norm are moe_route's gating, probs_bias and norm_weights (src/experts/moe.cpp:22-113)."""
    n = logits.shape[0]
    ids = torch.empty((n, topk), dtype=torch.int32, device=logits.device)
    weights = torch.empty((n, topk), dtype=torch.float32, device=logits.device)
    shared = torch.empty((n,), dtype=torch.float32, device=logits.device)
    err = _err()
    if gating == GATE_SOFTMAX and bias is None and norm:
        _check(lib().tqmoe_topk(_ptr(logits), _ptr(ids), _ptr(weights), _ptr(shared), experts, topk, n, float(scale), _stream(logits),
                                C.byref(err)), err)
    else:
        _check(lib().tqmoe_topk_gated(_ptr(logits), _ptr(bias), int(gating), int(bool(norm)), _ptr(ids), _ptr(weights), _ptr(shared), experts, topk,
                                      n, float(scale), _stream(logits), C.byref(err)), err)
    return ids, weights, shared


def moe_topk2(logits, logits2, experts, topk, scale=1.0):
    """moe_topk of two routings of one shape in one launch (moe_kernels.cuh:24-25): (ids, weights, shared) of each."""
    n = logits.shape[0]
    if logits2.shape != logits.shape:
        raise ValueError("moe_topk2: the two logit arrays differ in shape")
    out = []
    for _ in range(2):
        out.append((torch.empty((n, topk), dtype=torch.int32, device=logits.device), torch.empty((n, topk), dtype=torch.float32, device=logits.device),
                    torch.empty((n,), dtype=torch.float32, device=logits.device)))
    err = _err()
    _check(lib().tqmoe_topk2(_ptr(logits), _ptr(out[0][0]), _ptr(out[0][1]), _ptr(out[0][2]), _ptr(logits2), _ptr(out[1][0]), _ptr(out[1][1]),
                             _ptr(out[1][2]), experts, topk, n, float(scale), _stream(logits), C.byref(err)), err)
    return out[0], out[1]


def moe_dispatch(ids, experts, capacity=0):
    """counts [E], offsets [E + 1], perm [A] (entries past offsets[E] are -1) and, with capacity > 0, the reference's
    groups [E][capacity] view (moe_kernels.cuh:29; deterministic, ascending inside each expert)."""
    n, topk = ids.shape
    dev = ids.device
    counts = torch.empty(experts, dtype=torch.int32, device=dev)
    offsets = torch.empty(experts + 1, dtype=torch.int32, device=dev)
    perm = torch.full((n * topk,), -1, dtype=torch.int32, device=dev)
    groups = torch.full((experts, capacity), -1, dtype=torch.int32, device=dev) if capacity > 0 else None
    wsb = lib().tqmoe_dispatch_workspace_bytes(experts, n, topk)
    ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device=dev)
    err = _err()
    _check(lib().tqmoe_dispatch(_ptr(ids), _ptr(counts), _ptr(offsets), _ptr(perm), _ptr(groups), capacity, experts, n, topk, _ptr(ws),
                                wsb, _stream(ids), C.byref(err)), err)
    return counts, offsets, perm, groups


def moe_group(ids, experts):
    """tqllm_cuda::moe_group (moe_kernels.cuh:29): (counts [E], groups [E][n]) of ids [n][topk], ascending inside each expert;
    entries of groups past an expert's count are -1 here (the library leaves them untouched)."""
    n, topk = ids.shape
    counts = torch.empty(experts, dtype=torch.int32, device=ids.device)
    groups = torch.full((experts, n), -1, dtype=torch.int32, device=ids.device)
    moe_dispatch_into(ids, experts, counts, None, None, groups, n)
    return counts, groups


def moe_count(ids, counts):
    """counts[ids[i]] += 1 into the caller's uint64-sized counters (int64 tensor), tqllm_cuda::moe_count (moe.cu:183-186)."""
    err = _err()
    _check(lib().tqmoe_count(_ptr(ids), _ptr(counts), ids.numel(), _stream(ids), C.byref(err)), err)
    return counts


DEDUP_COLS, DEDUP_STRIDE = 8, 18     # kDedupCols, kDedupStride (src/formats/weight/quant_kernels.cuh:26-27)


def moe_dedup_maps(ids, slot_of, topk, groups=None):
    """tqllm_cuda::moe_dedup_maps (moe_kernels.cuh:34-39): (slots [count], gu [groups][18], dn [groups][18]) of the flat ids."""
    count = ids.numel()
    groups = count if groups is None else groups
    dev = ids.device
    slots = torch.empty(count, dtype=torch.int32, device=dev)
    gu = torch.empty((groups, DEDUP_STRIDE), dtype=torch.int32, device=dev)
    dn = torch.empty((groups, DEDUP_STRIDE), dtype=torch.int32, device=dev)
    err = _err()
    _check(lib().tqmoe_dedup_maps(_ptr(ids), _ptr(slot_of), count, topk, _ptr(slots), _ptr(gu), _ptr(dn), groups, _stream(ids), C.byref(err)), err)
    return slots, gu, dn


def expert_matvec_dedup(bank, x, dmap, out_rows, bank2=None, out_type=F32):
    """WeightFormat::expert_matvec_dedup / _dedup2 (weight_format.hpp:66-69) over a map of moe_dedup_maps: y [out_rows][rows]
    (and a second one for bank2); rows no column names stay zero here."""
    groups = dmap.shape[0]
    y = torch.zeros((out_rows, bank.rows), dtype=_OUT_TYPE[out_type], device=x.device)
    y2 = torch.zeros_like(y) if bank2 is not None else None
    need = lib().tqmoe_expert_matvec_dedup_scratch_bytes(groups, bank.rows, bank.cols, out_type, int(bank2 is not None))
    scratch = torch.empty(max(need, 16), dtype=torch.uint8, device=x.device)
    err = _err()
    b = bank.view()
    b2 = bank2.view() if bank2 is not None else None
    _check(lib().tqmoe_expert_matvec_dedup(C.byref(b), C.byref(b2) if b2 is not None else None, _ptr(x), _ttype(x), _ptr(y), _ptr(y2), out_type, _ptr(dmap), groups,
                                           _ptr(scratch), scratch.numel(), _stream(x), C.byref(err)), err)
    return (y, y2) if bank2 is not None else y


def lists_from_groups(counts, groups, bound=None):
    """The reference's counts / groups [E][capacity] as (counts clamped to the capacity, offsets, perm) for the grouped products."""
    experts, capacity = groups.shape
    dev = groups.device
    cc = torch.empty(experts, dtype=torch.int32, device=dev)
    offsets = torch.empty(experts + 1, dtype=torch.int32, device=dev)
    perm = torch.full((bound or experts * capacity,), -1, dtype=torch.int32, device=dev)
    err = _err()
    _check(lib().tqmoe_lists_from_groups_clamped(_ptr(counts), _ptr(groups), capacity, experts, _ptr(cc), _ptr(offsets), _ptr(perm), _stream(groups),
                                                 C.byref(err)), err)
    return cc, offsets, perm


def expert_gemm_i8_ref(bank, xq, xs, counts, groups, topk, assignments, per_expert_input=False, mode=2, out_dtype=torch.bfloat16, y=None):
    """WeightFormat::expert_gemm_i8 with the reference's own operands (weight_format.hpp:54-56): xq int8 [rows][cols] in natural
    order, xs fp32 [rows][cols / 32] (mode 1: per block; mode 2: the token's scale, [row][0] read), counts [E],
    groups [E][capacity]; y [assignments][bank rows], bf16 as the reference (or fp16)."""
    experts, capacity = groups.shape
    if y is None:
        y = torch.zeros((assignments, bank.rows), dtype=out_dtype, device=xq.device)
    need = lib().tqmoe_expert_gemm_i8_ref_scratch_bytes(experts, assignments, bank.cols, mode)
    scratch = torch.zeros(max(need, 16), dtype=torch.uint8, device=xq.device)
    err = _err()
    b = bank.view()
    _check(lib().tqmoe_expert_gemm_i8_ref(C.byref(b), _ptr(xq), _ptr(xs), None, _ptr(y), _ttype(y), _ptr(counts), _ptr(groups), capacity, experts, topk,
                                          int(per_expert_input), mode, assignments, _ptr(scratch), scratch.numel(), _stream(xq), C.byref(err)), err)
    return y


def moe_dispatch_into(ids, experts, counts, offsets, perm, groups=None, capacity=0):
    """tqmoe_dispatch_static into tensors the caller already holds: the library's built-in scratch, nothing allocated.
    offsets and perm may be None when groups is given (counts + groups: moe_group)."""
    n, topk = ids.shape
    err = _err()
    _check(lib().tqmoe_dispatch_static(_ptr(ids), _ptr(counts), _ptr(offsets), _ptr(perm), _ptr(groups), capacity, experts, n, topk,
                                       _stream(ids), C.byref(err)), err)


class ExpertBank:
    """One projection of every expert in the library's device layout: the counterpart of tqllm::Mat for stacked experts
    (weight_format.hpp:22-28, 61). Built from the raw GGUF block stream of [experts * rows][cols]."""

    def __init__(self, wtype, gguf_blocks, experts, rows, cols, device="cuda"):
        self.type, self.experts, self.rows, self.cols = wtype, experts, rows, cols
        cb, ab = C.c_size_t(0), C.c_size_t(0)
        err = _err()
        _check(lib().tqmoe_bank_layout(wtype, experts * rows, cols, C.byref(cb), C.byref(ab), C.byref(err)), err)
        raw = gguf_blocks if isinstance(gguf_blocks, torch.Tensor) else torch.from_numpy(gguf_blocks)
        elems, nbytes = BLOCK[wtype]
        if raw.numel() != experts * rows * (cols // elems) * nbytes:
            raise TqmoeError(-1, "GGUF block stream has %d bytes, %d expected" % (raw.numel(), experts * rows * (cols // elems) * nbytes))
        raw = raw.to(device=device, dtype=torch.uint8).contiguous()
        self.codes = torch.empty(cb.value, dtype=torch.uint8, device=raw.device)
        self.aux = torch.empty(ab.value, dtype=torch.uint8, device=raw.device)
        status = torch.zeros(1, dtype=torch.int32, device=raw.device)
        _check(lib().tqmoe_bank_load(wtype, _ptr(raw), experts * rows, cols, _ptr(self.codes), _ptr(self.aux), _ptr(status), _stream(raw),
                                     C.byref(err)), err)
        if int(status.item()):
            raise TqmoeError(-1, "NVFP4G rows whose blocks carry different global scales are not loadable")

    @classmethod
    def from_gguf(cls, path, name, device="cuda"):
        """The bank of a 3-D expert tensor [cols, rows, n_experts] of a GGUF file (ffn_{gate,up,down}_exps.weight): its
        bytes are the stacked block stream as they lie (gguf_expert_slice, src/core/gguf.hpp:77-91)."""
        from .gguf import GgufFile
        wtype, experts, rows, cols, raw = GgufFile(path).expert_bank(name)
        if wtype not in BLOCK:
            raise TqmoeError(-1, "%s: no expert kernels for GGUF type %d" % (name, wtype))
        return cls(wtype, torch.from_numpy(np.array(raw)), experts, rows, cols, device=device)

    def view(self):
        return _Bank(C.sizeof(_Bank), self.type, self.experts, self.rows, self.cols, self.codes.data_ptr(), self.aux.data_ptr())

    def dequant(self, row0=0, nrows=None):
        """fp32 [nrows][cols] decoded values (WeightFormat::dequant_rows_h, weight_format.hpp:84-86)."""
        nrows = self.experts * self.rows - row0 if nrows is None else nrows
        out = torch.empty((nrows, self.cols), dtype=torch.float32, device=self.codes.device)
        err = _err()
        b = self.view()
        _check(lib().tqmoe_bank_dequant(C.byref(b), row0, nrows, _ptr(out), _stream(out), C.byref(err)), err)
        return out


def quant_act(x):
    """Activation image of x [n][cols] (see include/tqmoe.h): uint8 tensor."""
    n, cols = x.shape
    image = torch.empty(lib().tqmoe_act_image_bytes(n, cols), dtype=torch.uint8, device=x.device)
    err = _err()
    _check(lib().tqmoe_quant_act(_ptr(x), _ttype(x), n, cols, _ptr(image), _stream(x), C.byref(err)), err)
    return image


def expert_matvec(bank, image, ids, per_expert_input=False, out_type=F32):
    """y [n * topk][rows] (WeightFormat::expert_matvec, weight_format.hpp:62-64). Rows of assignments with id < 0 stay as
    allocated (zero here)."""
    n, topk = ids.shape
    y = torch.zeros((n * topk, bank.rows), dtype=_OUT_TYPE[out_type], device=ids.device)
    err = _err()
    b = bank.view()
    _check(lib().tqmoe_expert_matvec(C.byref(b), _ptr(image), _ptr(y), out_type, _ptr(ids), n, topk, int(per_expert_input), _stream(ids),
                                     C.byref(err)), err)
    return y


def expert_matvec2(gate, up, image, ids, out_type=F32):
    """gate and up over the same ids in one launch (WeightFormat::expert_matvec2, weight_format.hpp:70-73)."""
    n, topk = ids.shape
    yg = torch.zeros((n * topk, gate.rows), dtype=_OUT_TYPE[out_type], device=ids.device)
    yu = torch.zeros_like(yg)
    err = _err()
    g, u = gate.view(), up.view()
    _check(lib().tqmoe_expert_matvec2(C.byref(g), C.byref(u), _ptr(image), _ptr(yg), _ptr(yu), out_type, _ptr(ids), n, topk, _stream(ids),
                                      C.byref(err)), err)
    return yg, yu


def moe_extend_ids(ids, extra):
    """[n][topk + 1]: the routed ids with the shared expert's bank index as the last slot (moe_kernels.cuh:77-78)."""
    n, topk = ids.shape
    out = torch.empty((n, topk + 1), dtype=torch.int32, device=ids.device)
    err = _err()
    _check(lib().tqmoe_extend_ids(_ptr(ids), _ptr(out), topk, n, extra, _stream(ids), C.byref(err)), err)
    return out


def expert_gateup(gate, up, x_image, ids, topk, shared_ff=0, act_image=None):
    """Activation image of silu(gate x) * (up x) for every (token, slot) of ids [n][slots]; slots past topk are the shared
    expert (WeightFormat::expert_gemm_gateup, weight_format.hpp:57-59, at decode sizes)."""
    n, slots = ids.shape
    if act_image is None:
        act_image = torch.zeros(lib().tqmoe_act_image_bytes(n * slots, gate.rows), dtype=torch.uint8, device=ids.device)
    err = _err()
    g, u = gate.view(), up.view()
    _check(lib().tqmoe_expert_gateup(C.byref(g), C.byref(u), _ptr(x_image), _ptr(act_image), _ptr(ids), n, slots, topk, shared_ff, _stream(ids),
                                     C.byref(err)), err)
    return act_image


def expert_down(down, act_image, ids, topk, shared_ff=0, y=None):
    """y [n * slots][hidden] fp32: the down product of every (token, slot) from its row of the activation image."""
    n, slots = ids.shape
    if y is None:
        y = torch.zeros((n * slots, down.rows), dtype=torch.float32, device=ids.device)
    err = _err()
    d = down.view()
    _check(lib().tqmoe_expert_down(C.byref(d), _ptr(act_image), _ptr(y), _ptr(ids), n, slots, topk, shared_ff, _stream(ids), C.byref(err)), err)
    return y


def moe_combine_strided(y, slots, weights, shared_weights=None, out_type=F32, out=None):
    """moe_sum_strided (moe_kernels.cuh:80-81): y [n][slots][hidden], the first topk slots weighted, slot topk the shared row."""
    n, topk = weights.shape
    hidden = y.shape[-1]
    if out is None:
        out = torch.empty((n, hidden), dtype=_OUT_TYPE[out_type], device=y.device)
    shared = y.view(-1)[topk * hidden:] if shared_weights is not None else None
    err = _err()
    fn = lib().tqmoe_combine_strided_f16 if y.dtype == torch.float16 else lib().tqmoe_combine_strided
    _check(fn(_ptr(y), slots, _ptr(shared), slots * hidden, _ptr(weights), _ptr(shared_weights), _ptr(out), out_type, hidden, topk, n, _stream(y),
              C.byref(err)), err)
    return out


def quant_rows_i8(x, fp8=False):
    """Per-row int8 activations (k_quant_act_rows mode 2, quant_kernels.cuh:17-19): (q int8 [rows][cols] in the library's
    byte order, scale fp32 [rows]). fp8: E4M3 bytes with scale amax / 448 (fp8_quant_rows, fp8_gemm.cuh:19-31)."""
    rows, cols = x.shape
    q = torch.empty((rows, cols), dtype=torch.int8, device=x.device)
    scale = torch.empty(rows, dtype=torch.float32, device=x.device)
    err = _err()
    fn = lib().tqmoe_quant_rows_fp8 if fp8 else lib().tqmoe_quant_rows_i8
    _check(fn(_ptr(x), _ttype(x), rows, cols, _ptr(q), _ptr(scale), _stream(x), C.byref(err)), err)
    return q, scale


def quant_rows_fp8(x):
    return quant_rows_i8(x, fp8=True)


def quant_rows_i8_blocks(x, sums=True):
    """Int8 activations with a scale per 32 values (k_quant_act_rows mode 1, quant_kernels.cuh:17-19; quant_u4h.inc:790-822):
    (q int8 [rows][cols] in the library's byte order, scales fp32 [rows][cols / 32], sums of q per 16 values int16
    [rows][cols / 32][2] or None)."""
    rows, cols = x.shape
    q = torch.empty((rows, cols), dtype=torch.int8, device=x.device)
    scales = torch.empty((rows, cols // 32), dtype=torch.float32, device=x.device)
    qsum = torch.empty((rows, cols // 32, 2), dtype=torch.int16, device=x.device) if sums else None
    err = _err()
    _check(lib().tqmoe_quant_rows_i8_blocks(_ptr(x), _ttype(x), rows, cols, _ptr(q), _ptr(scales), _ptr(qsum) if sums else None, _stream(x), C.byref(err)), err)
    return q, scales, qsum


def _block_scales(assignments, experts, cols, device):
    return torch.zeros(lib().tqmoe_grouped_block_scale_words(assignments, experts, cols), dtype=torch.float32, device=device)


def group_rows_i8_blocks(x, lists, assignments, xdiv):
    """group_rows_i8 with a scale per row and 32 values: (q, scale, block_scale); block_scale is fp32
    [row tiles][cols / 32][32 rows], the rows' own scales in `scale` are 1."""
    counts, offsets, perm = lists
    cols = x.shape[1]
    rows = lib().tqmoe_grouped_rows(assignments, counts.numel())
    q = torch.zeros((rows, cols), dtype=torch.int8, device=x.device)
    scale = torch.zeros(lib().tqmoe_grouped_scale_words(assignments, counts.numel()), dtype=torch.float32, device=x.device)
    bs = _block_scales(assignments, counts.numel(), cols, x.device)
    err = _err()
    _check(lib().tqmoe_group_rows_i8_blocks(_ptr(x), _ttype(x), cols, _ptr(counts), _ptr(offsets), _ptr(perm), counts.numel(), assignments, xdiv, _ptr(q),
                                            _ptr(scale), _ptr(bs), _stream(x), C.byref(err)), err)
    return q, scale, bs


def gather_rows_i8_blocks(rows_q, rows_scales, lists, assignments, xdiv):
    """The arranging step of group_rows_i8_blocks alone, from rows quant_rows_i8_blocks has quantised."""
    counts, offsets, perm = lists
    cols = rows_q.shape[1]
    rows = lib().tqmoe_grouped_rows(assignments, counts.numel())
    q = torch.zeros((rows, cols), dtype=torch.int8, device=rows_q.device)
    scale = torch.zeros(lib().tqmoe_grouped_scale_words(assignments, counts.numel()), dtype=torch.float32, device=rows_q.device)
    bs = _block_scales(assignments, counts.numel(), cols, rows_q.device)
    err = _err()
    _check(lib().tqmoe_gather_rows_i8_blocks(_ptr(rows_q), _ptr(rows_scales), cols, _ptr(counts), _ptr(offsets), _ptr(perm), counts.numel(), assignments, xdiv,
                                             _ptr(q), _ptr(scale), _ptr(bs), _stream(rows_q), C.byref(err)), err)
    return q, scale, bs


def group_rows_i8(x, lists, assignments, xdiv, fp8=False):
    """Per-row int8 quantisation of the input row (a // xdiv) of every listed assignment a, gathered expert by expert into
    the operand-major row tiles the grouped products read (mmq_quantize_act_rows, mmq_experts.cu:79-95, in role):
    (q int8 [grouped rows][cols], scale fp32 [grouped rows]); rows of the padding hold zeros here."""
    counts, offsets, perm = lists
    cols = x.shape[1]
    rows = lib().tqmoe_grouped_rows(assignments, counts.numel())
    q = torch.zeros((rows, cols), dtype=torch.int8, device=x.device)
    scale = torch.zeros(lib().tqmoe_grouped_scale_words(assignments, counts.numel()), dtype=torch.float32, device=x.device)
    err = _err()
    fn = lib().tqmoe_group_rows_fp8 if fp8 else lib().tqmoe_group_rows_i8
    _check(fn(_ptr(x), _ttype(x), cols, _ptr(counts), _ptr(offsets), _ptr(perm), counts.numel(), assignments, xdiv, _ptr(q), _ptr(scale), _stream(x),
              C.byref(err)), err)
    return q, scale


def group_rows_fp8(x, lists, assignments, xdiv):
    """group_rows_i8 with E4M3 bytes (scale amax / 448): the operand of the NVFP4G grouped products."""
    return group_rows_i8(x, lists, assignments, xdiv, fp8=True)


def gather_rows_i8(rows_q, rows_scale, lists, assignments, xdiv):
    """The arranging step of group_rows_i8 alone, from rows quant_rows_i8 has quantised: the same (q, scale), every input row
    quantised once however many assignments read it."""
    counts, offsets, perm = lists
    cols = rows_q.shape[1]
    rows = lib().tqmoe_grouped_rows(assignments, counts.numel())
    q = torch.zeros((rows, cols), dtype=torch.int8, device=rows_q.device)
    scale = torch.zeros(lib().tqmoe_grouped_scale_words(assignments, counts.numel()), dtype=torch.float32, device=rows_q.device)
    err = _err()
    _check(lib().tqmoe_gather_rows_i8(_ptr(rows_q), _ptr(rows_scale), cols, _ptr(counts), _ptr(offsets), _ptr(perm), counts.numel(), assignments, xdiv,
                                      _ptr(q), _ptr(scale), _stream(rows_q), C.byref(err)), err)
    return q, scale


def expert_gemm_gateup(gate, up, x, lists, n, slots, topk, shared_ff=0, act=None):
    """WeightFormat::expert_gemm_gateup (weight_format.hpp:57-59), any bank format, fp16 operands: fp16 act [n * slots][ff];
    rows of assignments that are in no list are zero here (the library leaves them untouched)."""
    counts, offsets, perm = lists
    if act is None:
        act = torch.zeros((n * slots, gate.rows), dtype=torch.float16, device=x.device)
    err = _err()
    g, u = gate.view(), up.view()
    _check(lib().tqmoe_expert_gemm_gateup(C.byref(g), C.byref(u), _ptr(x), _ttype(x), _ptr(counts), _ptr(offsets), _ptr(perm), n, slots, topk, shared_ff,
                                          _ptr(act), _stream(x), C.byref(err)), err)
    return act


def expert_gemm(bank, x, lists, n, slots, topk, shared_ff=0, per_expert_input=False, out_type=F16, y=None):
    """WeightFormat::expert_gemm (weight_format.hpp:51-53), any bank format, fp16 operands: y [n * slots][rows], fp16 or fp32."""
    counts, offsets, perm = lists
    if y is None:
        y = torch.zeros((n * slots, bank.rows), dtype=torch.float16 if out_type == F16 else torch.float32, device=x.device)
    err = _err()
    b = bank.view()
    _check(lib().tqmoe_expert_gemm(C.byref(b), _ptr(x), _ttype(x), _ptr(counts), _ptr(offsets), _ptr(perm), n, slots, topk, shared_ff, int(per_expert_input),
                                   _ptr(y), out_type, _stream(x), C.byref(err)), err)
    return y


def expert_gemm_gateup_i8(gate, up, xq, xs, lists, n, slots, topk, shared_ff=0, fp8=False, act=None):
    """WeightFormat::expert_gemm_gateup (weight_format.hpp:57-59) on int8 rows: fp16 act [n * slots][ff]; rows of
    assignments that are in no list are zero here (the library leaves them untouched)."""
    counts, offsets, perm = lists
    if act is None:
        act = torch.zeros((n * slots, gate.rows), dtype=torch.float16, device=xq.device)
    err = _err()
    g, u = gate.view(), up.view()
    fn = lib().tqmoe_expert_gemm_gateup_fp8 if fp8 else lib().tqmoe_expert_gemm_gateup_i8
    _check(fn(C.byref(g), C.byref(u), _ptr(xq), _ptr(xs), _ptr(counts), _ptr(offsets), _ptr(perm), n, slots, topk, shared_ff, _ptr(act), _stream(xq),
              C.byref(err)), err)
    return act


def expert_gemm_gateup_fp8(gate, up, xq, xs, lists, n, slots, topk, shared_ff=0):
    """The gate / up product with SwiGLU on E4M3 rows (NVFP4G banks, weights widened to E4M3)."""
    return expert_gemm_gateup_i8(gate, up, xq, xs, lists, n, slots, topk, shared_ff, fp8=True)


def expert_gemm_i8(bank, xq, xs, lists, n, slots, topk, shared_ff=0, fp8=False, y=None):
    """WeightFormat::expert_gemm_i8 (weight_format.hpp:54-56), per-token scales, one input row per assignment: fp16
    y [n * slots][rows]."""
    counts, offsets, perm = lists
    if y is None:
        y = torch.zeros((n * slots, bank.rows), dtype=torch.float16, device=xq.device)
    err = _err()
    b = bank.view()
    fn = lib().tqmoe_expert_gemm_fp8 if fp8 else lib().tqmoe_expert_gemm_i8
    _check(fn(C.byref(b), _ptr(xq), _ptr(xs), _ptr(counts), _ptr(offsets), _ptr(perm), n, slots, topk, shared_ff, _ptr(y), _stream(xq), C.byref(err)), err)
    return y


def expert_gemm_fp8(bank, xq, xs, lists, n, slots, topk, shared_ff=0):
    return expert_gemm_i8(bank, xq, xs, lists, n, slots, topk, shared_ff, fp8=True)


def expert_gemm_gateup_i8_blocks(gate, up, xq, xs, block_scale, lists, n, slots, topk, shared_ff=0, act=None):
    """expert_gemm_gateup_i8 on rows with a scale per 32 values (expert_gemm_i8's mode 1, quant_kernels.cuh:13-16)."""
    counts, offsets, perm = lists
    if act is None:
        act = torch.zeros((n * slots, gate.rows), dtype=torch.float16, device=xq.device)
    err = _err()
    g, u = gate.view(), up.view()
    _check(lib().tqmoe_expert_gemm_gateup_i8_blocks(C.byref(g), C.byref(u), _ptr(xq), _ptr(xs), _ptr(block_scale), _ptr(counts), _ptr(offsets), _ptr(perm), n, slots,
                                                    topk, shared_ff, _ptr(act), _stream(xq), C.byref(err)), err)
    return act


def expert_gemm_i8_blocks(bank, xq, xs, block_scale, lists, n, slots, topk, shared_ff=0, y=None):
    """WeightFormat::expert_gemm_i8 (weight_format.hpp:54-56) with a scale per 32 values of the input rows (mode 1)."""
    counts, offsets, perm = lists
    if y is None:
        y = torch.zeros((n * slots, bank.rows), dtype=torch.float16, device=xq.device)
    err = _err()
    b = bank.view()
    _check(lib().tqmoe_expert_gemm_i8_blocks(C.byref(b), _ptr(xq), _ptr(xs), _ptr(block_scale), _ptr(counts), _ptr(offsets), _ptr(perm), n, slots, topk, shared_ff,
                                             _ptr(y), _stream(xq), C.byref(err)), err)
    return y


def moe_swiglu(gate, up, swiglu_clamp=0.0, clamp_gate=False):
    """silu(gate) * up in fp32 (moe_kernels.cuh:71-72) with the optional clamp of moe_expert_ffn (src/experts/moe.cpp:128-143)."""
    act = torch.empty_like(gate)
    err = _err()
    _check(lib().tqmoe_swiglu_clamped(_ptr(gate), _ptr(up), _ptr(act), gate.numel(), float(swiglu_clamp), int(bool(clamp_gate)), _stream(gate),
                                      C.byref(err)), err)
    return act


def moe_combine(routed, shared, weights, shared_weights, out_type=F32):
    """out [n][hidden] = sum_s weights[t][s] * routed[t * k + s] + shared_weights[t] * shared[t] (moe_kernels.cuh:73-74)."""
    n, topk = weights.shape
    hidden = routed.shape[1]
    out = torch.empty((n, hidden), dtype=_OUT_TYPE[out_type], device=routed.device)
    err = _err()
    _check(lib().tqmoe_combine(_ptr(routed), _ptr(shared), _ptr(weights), _ptr(shared_weights), _ptr(out), out_type, hidden, topk, n,
                               _stream(routed), C.byref(err)), err)
    return out


def add_rmsnorm(rows, residual, weight, eps, out_dtype=torch.bfloat16):
    """rows (bf16 [n][H], updated in place: += residual when given) -> normed rows of out_dtype (bf16 or fp16): the
    reference's add_sumsq + norm_h in front of the layer (qwen35_forward.cpp:1114-1115)."""
    n, h = rows.shape
    normed = torch.empty((n, h), dtype=out_dtype, device=rows.device)
    err = _err()
    _check(lib().tqmoe_add_rmsnorm(_ptr(rows), _ptr(residual), _ptr(weight), float(eps), _ptr(normed), _ttype(normed), h, n, _stream(rows), C.byref(err)), err)
    return normed


def moe_combine_residual(routed, shared, weights, shared_weights, residual, out=None):
    """out = bf16(bf16(weighted sum) + residual) (moe_sum then add_sumsq, qwen35_forward.cpp:1248-1250). routed: fp32 or fp16
    [n][topk][H]; shared: [n][H] of the same type or None."""
    n, topk, h = routed.shape
    if out is None:
        out = torch.empty((n, h), dtype=torch.bfloat16, device=routed.device)
    err = _err()
    _check(lib().tqmoe_combine_residual(_ptr(routed), _ttype(routed), topk, _ptr(shared), h, _ptr(weights), _ptr(shared_weights), _ptr(residual), _ptr(out),
                                        h, topk, n, _stream(routed), C.byref(err)), err)
    return out


class MoeLayer:
    """hidden states + router weights + expert banks in, combined hidden states out, in one library call."""

    def __init__(self, router, shared_gate, gate, up, down, topk, shared_ff=0, weight_scale=1.0, gating=GATE_SOFTMAX, probs_bias=None,
                 norm_weights=True, act_blocks=False, swiglu_clamp=0.0, clamp_gate=False):
        self.swiglu_clamp, self.clamp_gate = swiglu_clamp, clamp_gate   # MoeConfig::swiglu_clamp, moe_expert_ffn's clamp_gate
        self.router, self.shared_gate, self.gate, self.up, self.down = router, shared_gate, gate, up, down
        self.act_blocks = act_blocks   # 0 / False: the library picks the grouped products; 1 / True: int8 with a scale per 32 activations; 2: int8 with a scale per token
        self.n_expert, self.hidden = router.shape
        self.ff, self.topk, self.shared_ff, self.weight_scale = gate.rows, topk, shared_ff, weight_scale
        self.gating, self.probs_bias, self.norm_weights = gating, probs_bias, norm_weights
        self._ws = None

    def desc(self):
        return _Layer(C.sizeof(_Layer), self.hidden, self.ff, self.n_expert, self.topk, int(self.shared_ff > 0), self.shared_ff,
                      float(self.weight_scale), self.router.data_ptr(), self.shared_gate.data_ptr() if self.shared_gate is not None else None,
                      _ttype(self.router), self.gate.view(), self.up.view(), self.down.view(), int(self.gating), int(not self.norm_weights),
                      self.probs_bias.data_ptr() if self.probs_bias is not None else None, int(self.act_blocks), float(self.swiglu_clamp),
                      int(bool(self.clamp_gate)))

    def path(self, n):
        """'decode', 'grouped_i8', 'grouped_f16' or 'grouped_fp8': the expert products a batch of n tokens takes"""
        d = self.desc()
        rc = lib().tqmoe_layer_path(C.byref(d), n)
        if rc < 0:
            raise TqmoeError(rc, "layer descriptor rejected")
        return ("decode", "grouped_i8", "grouped_f16", "grouped_fp8")[rc]

    def workspace(self, n):
        d = self.desc()
        need = lib().tqmoe_layer_workspace_bytes(C.byref(d), n)
        if need == 0:
            raise TqmoeError(-1, "layer descriptor rejected (shapes of the banks do not match the layer)")
        if self._ws is None or self._ws.numel() < need:
            self._ws = torch.empty(need, dtype=torch.uint8, device=self.router.device)
        return self._ws

    def forward(self, x, out_type=F32, return_routing=False, out=None, residual=None):
        """residual (bf16 [n][H]): added to the result, which is then bf16: bf16(bf16(layer(x)) + residual)."""
        n = x.shape[0]
        ws = self.workspace(n)
        if residual is not None:
            out_type = BF16
        if out is None:
            out = torch.empty((n, self.hidden), dtype=_OUT_TYPE[out_type], device=x.device)
        ids = weights = logits = None
        if return_routing:
            ids = torch.empty((n, self.topk), dtype=torch.int32, device=x.device)
            weights = torch.empty((n, self.topk), dtype=torch.float32, device=x.device)
            logits = torch.empty((n, self.n_expert + 1), dtype=torch.float32, device=x.device)
        d = self.desc()
        err = _err()
        if residual is not None:
            _check(lib().tqmoe_layer_forward_residual(C.byref(d), _ptr(x), _ttype(x), _ptr(residual), n, _ptr(out), _ptr(ids), _ptr(weights), _ptr(logits),
                                                      _ptr(ws), ws.numel(), _stream(x), C.byref(err)), err)
        else:
            _check(lib().tqmoe_layer_forward(C.byref(d), _ptr(x), _ttype(x), n, _ptr(out), out_type, _ptr(ids), _ptr(weights), _ptr(logits),
                                             _ptr(ws), ws.numel(), _stream(x), C.byref(err)), err)
        return (out, ids, weights, logits) if return_routing else out
