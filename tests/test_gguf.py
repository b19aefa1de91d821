"""GGUF expert-bank ingestion: the 3-D expert tensor reader and slicer (include/tqmoe_gguf.hpp and its Python mirror)
against a synthetic GGUF file whose experts carry distinguishable values, after the reference's own gate for this
(tests/moe_experts.cpp): every slice must read ITS OWN expert, and every inconsistency must raise."""
import os
import struct
import subprocess

import numpy as np
import pytest

import synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
COLS, ROWS, N_EXP = 256, 8, 5      # rows of one Q2_K block: rows must end on block boundaries


def put_str(b, s):
    b += struct.pack("<Q", len(s)) + s.encode()


def write_gguf(path, tensors, alignment=32, extra_kv=True):
    """tensors: list of (name, ne, type, bytes). GGUF v3 with a few metadata values of different types in front."""
    b = bytearray(b"GGUF")
    b += struct.pack("<IQQ", 3, len(tensors), 4 if extra_kv else 1)
    put_str(b, "general.alignment"); b += struct.pack("<II", 4, alignment)
    if extra_kv:
        put_str(b, "general.name"); b += struct.pack("<I", 8); put_str(b, "synthetic experts")
        put_str(b, "some.floats"); b += struct.pack("<IIQ", 9, 6, 3) + struct.pack("<3f", 1.0, 2.0, 3.0)
        put_str(b, "some.strings"); b += struct.pack("<IIQ", 9, 8, 2); put_str(b, "a"); put_str(b, "bc")
    at = 0
    for name, ne, type, data in tensors:
        put_str(b, name)
        b += struct.pack("<I", len(ne)) + struct.pack("<%dQ" % len(ne), *ne) + struct.pack("<IQ", type, at)
        at += (len(data) + alignment - 1) // alignment * alignment
    while len(b) % alignment:
        b.append(0)
    for name, ne, type, data in tensors:
        b += bytes(data)
        while len(b) % alignment:
            b.append(0)
    with open(path, "wb") as f:
        f.write(b)


@pytest.fixture(scope="module")
def synthetic(tmp_path_factory):
    path = str(tmp_path_factory.mktemp("gguf") / "experts.gguf")
    e, r, c = np.meshgrid(np.arange(N_EXP), np.arange(ROWS), np.arange(COLS), indexing="ij")
    f32 = (e * 10000 + r * 100 + c).astype(np.float32)
    q2k = np.concatenate([np.full(COLS * ROWS // 256 * 84, 0xE0 + i, np.uint8) for i in range(N_EXP)])
    write_gguf(path, [("experts.f32", (COLS, ROWS, N_EXP), 0, f32.tobytes()), ("experts.q2k", (COLS, ROWS, N_EXP), 10, q2k.tobytes()),
                      ("plain.f16", (16, 4), 1, np.zeros(64, np.float16).tobytes())])
    return path


def test_python_reader_slices_its_own_expert(synthetic):
    from tqllm_amd.gguf import GgufFile, gguf_expert_count, gguf_expert_slice
    f = GgufFile(synthetic)
    t = f.tensors["experts.f32"]
    assert gguf_expert_count(t) == N_EXP and t.ne == [COLS, ROWS, N_EXP]
    assert gguf_expert_count(f.tensors["plain.f16"]) == 0
    whole = np.array(f.read(t))
    assert whole.size == COLS * ROWS * N_EXP * 4
    for e in range(N_EXP):
        s = gguf_expert_slice(t, e, "experts.f32")
        assert s.ne == [COLS, ROWS] and s.bytes == COLS * ROWS * 4
        got = np.array(f.read(s))
        assert np.array_equal(got, whole[e * s.bytes:(e + 1) * s.bytes])
        v = got.view(np.float32)
        assert v[0] == e * 10000 and v[-1] == e * 10000 + (ROWS - 1) * 100 + (COLS - 1)
    q = f.tensors["experts.q2k"]
    for e in range(N_EXP):
        got = np.array(f.read(gguf_expert_slice(q, e, "experts.q2k")))
        assert got.size == COLS * ROWS // 256 * 84 and (got == 0xE0 + e).all()
    assert f.expert_bank("experts.q2k")[:4] == (10, N_EXP, ROWS, COLS)


def test_python_slicer_fails_closed():
    from tqllm_amd.gguf import GgufError, GgufTensor, gguf_expert_slice
    good = GgufTensor(0, [COLS, ROWS, N_EXP], 0, COLS * ROWS * N_EXP * 4)
    gguf_expert_slice(good, N_EXP - 1, "t")
    cases = [(good, N_EXP), (good, N_EXP + 100), (GgufTensor(0, [COLS, ROWS], 0, good.bytes), 0), (GgufTensor(0, [COLS, ROWS, 0], 0, good.bytes), 0),
             (GgufTensor(0, [COLS, ROWS, N_EXP], 0, good.bytes + 4), 0), (GgufTensor(10, [100, 7, N_EXP], 0, 100 * 7 * N_EXP), 0),
             (GgufTensor(0, [COLS, ROWS, N_EXP, 2], 0, good.bytes), 0), (GgufTensor(9999, [COLS, ROWS, N_EXP], 0, good.bytes), 0),
             (GgufTensor(10, [128, 2, N_EXP], 0, 84 * N_EXP), 0),                       # whole blocks per expert, but not per row
             (GgufTensor(0, [1 << 40, 1 << 30, 4], 0, 0), 0), (good, -1)]               # a byte count past 64 bits; a negative index
    for t, idx in cases:
        with pytest.raises(GgufError):
            gguf_expert_slice(t, idx, "t")


def test_reader_rejects_broken_files(tmp_path):
    from tqllm_amd.gguf import GgufError, GgufFile
    p = str(tmp_path / "x.gguf")
    open(p, "wb").write(b"GGML" + bytes(32))
    with pytest.raises(GgufError):
        GgufFile(p)
    write_gguf(p, [("t", (32, 8, 5), 0, bytes(100))])       # data shorter than the table says
    with pytest.raises(GgufError):
        GgufFile(p)
    write_gguf(p, [("t", (100, 7, 5), 10, bytes(4096))])     # not a whole number of blocks
    with pytest.raises(GgufError):
        GgufFile(p)


def test_cpp_header_against_the_same_file(synthetic, tmp_path):
    exe = str(tmp_path / "gguf_check")
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-Wextra", "-I", os.path.join(ROOT, "include"), os.path.join(ROOT, "tests", "gguf_check.cpp"), "-o", exe],
                   check=True)
    r = subprocess.run([exe, synthetic, str(COLS), str(ROWS), str(N_EXP)], stdout=subprocess.PIPE, text=True)
    assert r.returncode == 0, r.stdout
    assert "FAIL" not in r.stdout and r.stdout.count("ok  ") >= 16


@pytest.mark.gpu
def test_bank_from_gguf_decodes_like_the_oracle(tmp_path):
    """An IQ4_XS and a Q4_K expert tensor written as 3-D GGUF tensors load into banks whose decoded values are the
    oracle's, expert by expert (a wrong stride would decode a neighbour)."""
    import oracle
    import tqllm_amd as tq
    from tqllm_amd.gguf import GgufFile, gguf_expert_slice
    experts, rows, cols = 6, 64, 512
    rng = np.random.default_rng(5)
    tensors, raws = [], {}
    for name, wtype in (("blk.0.ffn_gate_exps.weight", oracle.IQ4_XS), ("blk.0.ffn_down_exps.weight", oracle.Q4_K)):
        w = (rng.standard_normal((experts * rows, cols)) * 0.02 * (1 + np.arange(experts * rows)[:, None] // rows)).astype(np.float32)
        raws[name] = (wtype, oracle.quantize(wtype, w))
        tensors.append((name, (cols, rows, experts), wtype, raws[name][1].tobytes()))
    path = str(tmp_path / "moe.gguf")
    write_gguf(path, tensors)
    f = GgufFile(path)
    for name, (wtype, raw) in raws.items():
        bank = tq.ExpertBank.from_gguf(path, name)
        assert (bank.type, bank.experts, bank.rows, bank.cols) == (wtype, experts, rows, cols)
        got = bank.dequant().cpu().numpy()
        for e in range(experts):
            s = gguf_expert_slice(f.tensors[name], e, name)
            want = oracle.dequantize(wtype, np.array(f.read(s)), rows * cols).reshape(rows, cols)
            assert np.array_equal(got[e * rows:(e + 1) * rows], want), (name, e)
