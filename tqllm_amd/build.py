"""Builds libtqmoe.so (the C-ABI HIP library) for gfx950 in-tree with hipcc."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libtqmoe.so")
SOURCES = ["routing.hip", "bank.hip", "decode.hip", "decode_iq4xs.hip", "decode_q4k.hip", "decode_iq3s.hip", "decode_nvfp4.hip", "decode_iq4nl.hip", "decode_q8_0.hip", "decode_q5k.hip", "decode_q6k.hip", "decode_iq3xxs.hip", "decode_iq2s.hip", "decode_q2k.hip", "decode_iq1s.hip", "decode_q4_0.hip", "decode_q3k.hip", "decode_iq2xxs.hip", "decode_iq2xs.hip", "prefill_planes.hip", "prefill_planes_blocks.hip", "prefill_planes_legacy.hip", "prefill_f16.hip", "norm.hip", "layer.hip"]
FLAGS = ["-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-Wall", "-Wextra", "-Wno-unused-parameter",
         # packed FP32 VALU forms are kept out of every kernel
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def build(verbose=False, jobs=None):
    """Compiles every source to an object (in parallel) and links the shared library. Always recompiles."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    procs = []
    for src in SOURCES:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [hipcc] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, obj, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    objs = []
    for src, obj, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l and l.strip())
        if p.returncode:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
        if verbose and out:
            print(out, flush=True)
        objs.append(obj)
    link = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    r = subprocess.run(link, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode:
        raise RuntimeError("link failed:\n" + r.stdout)
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
