"""Host-side checks that need no GPU: the C-ABI library loads and exports every entry point include/tqmoe.h declares, the
pure-host entry points (sizes, layouts) answer, bad arguments and a missing device are reported through the error
record (there is no CPU path to fall back to), the C++ adapter header compiles, and the product never touches the oracle."""
import ctypes as C
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "tqmoe.h")


@pytest.fixture(scope="module")
def tq():
    import tqllm_amd
    return tqllm_amd


def declared_functions():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    return sorted(set(re.findall(r"\b(tqmoe_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_entry_point_is_exported(tq):
    names = declared_functions()
    assert len(names) >= 24 and "tqmoe_layer_forward" in names and "tqmoe_expert_gemm_i8" in names
    lib = tq.lib()
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing
    assert tq.abi_version() == 1


def test_host_only_entry_points(tq):
    lib = tq.lib()
    code, aux = C.c_size_t(), C.c_size_t()
    err = tq.api._err()
    # IQ4_XS: 16 B of codes per 32 weights, 8 B per 256; rows in tiles of 32
    assert lib.tqmoe_bank_layout(tq.IQ4_XS, 64, 2048, C.byref(code), C.byref(aux), C.byref(err)) == 0
    assert (code.value, aux.value) == (64 * 2048 // 2, 64 * 2048 // 256 * 8)
    assert lib.tqmoe_bank_layout(tq.IQ3_S, 10, 512, C.byref(code), C.byref(aux), C.byref(err)) == 0
    assert (code.value, aux.value) == (10 * 16 * 12, 10 * 2 * 16)
    assert lib.tqmoe_bank_layout(tq.NVFP4G, 10, 256, C.byref(code), C.byref(aux), C.byref(err)) == 0
    assert code.value == 10 * 128 and aux.value == 160 + 40
    assert lib.tqmoe_bank_layout(tq.Q4_K, 10, 100, C.byref(code), C.byref(aux), C.byref(err)) == -1   # cols not a multiple of 256
    assert b"tqmoe_bank_layout" in err.message
    assert lib.tqmoe_bank_layout(7, 10, 256, C.byref(code), C.byref(aux), C.byref(err)) == -2         # unknown format
    assert lib.tqmoe_act_image_bytes(3, 2048) == 3 * 64 * 72
    assert lib.tqmoe_act_image_bytes(3, 100) == 0
    assert lib.tqmoe_dispatch_workspace_bytes(512, 4096, 10) > 0


def test_errors_are_reported_not_swallowed(tq):
    lib = tq.lib()
    err = tq.api._err()
    # bad shape: reported before any device work
    assert lib.tqmoe_topk(None, None, None, None, 8, 2, 1, 1.0, None, C.byref(err)) == -1
    assert err.code == -1 and err.message
    # err may be NULL
    assert lib.tqmoe_topk(None, None, None, None, 8, 2, 1, 1.0, None, None) == -1
    # a short error struct is left alone
    short = tq.api._Error(8, 0, b"")
    assert lib.tqmoe_topk(None, None, None, None, 8, 2, 1, 1.0, None, C.byref(short)) == -1 and short.code == 0


def test_no_device_is_an_error_not_a_fallback(tq):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    lib = tq.lib()
    err = tq.api._err()
    buf = (C.c_float * 64)()
    ids = (C.c_int32 * 4)()
    rc = lib.tqmoe_topk(buf, ids, buf, None, 8, 2, 1, 1.0, None, C.byref(err))
    assert rc == -3 and b"no CPU path" in err.message


def test_adapter_header_compiles(tmp_path):
    src = tmp_path / "use.cpp"
    src.write_text('#include "tqmoe_adapter.hpp"\n'
                   "int main() { tqmoe_error e = tqmoe_hip::fresh(); (void)e; return tqmoe_hip::ExpertFormat::has_expert_matvec() ? 0 : 1; }\n")
    subprocess.check_call(["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-I", os.path.join(ROOT, "include"), str(src)])
    # the C header alone is plain C
    csrc = tmp_path / "use.c"
    csrc.write_text('#include "tqmoe.h"\nint main(void) { return (int)sizeof(tqmoe_layer) == 0; }\n')
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-I", os.path.join(ROOT, "include"), str(csrc)])


def test_product_does_not_use_the_oracle():
    pkg = os.path.join(ROOT, "tqllm_amd")
    for base, _, files in os.walk(pkg):
        if os.path.basename(base) == "build":
            continue
        for f in files:
            if f.endswith((".py", ".hip", ".cuh", ".h", ".hpp")):
                text = open(os.path.join(base, f), errors="replace").read()
                assert "oracle" not in text.lower(), os.path.join(base, f)
