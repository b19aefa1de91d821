"""Builds tests/_build/adapter_check (tests/adapter_check.cpp: the C++ adapter driven through a base class with the
reference's virtual signatures) against the in-tree libtqmoe.so. Host code only; needs the HIP runtime headers."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
EXE = os.path.join(HERE, "_build", "adapter_check")


def build():
    os.makedirs(os.path.dirname(EXE), exist_ok=True)
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = ["g++", "-std=c++17", "-O1", "-Wall", "-Wextra", "-Werror", "-D__HIP_PLATFORM_AMD__", "-I", os.path.join(rocm, "include"),
           "-I", os.path.join(ROOT, "include"), os.path.join(HERE, "adapter_check.cpp"), "-o", EXE,
           "-L", os.path.join(ROOT, "tqllm_amd"), "-ltqmoe", "-L", os.path.join(rocm, "lib"), "-lamdhip64",
           "-Wl,-rpath,$ORIGIN/../../tqllm_amd", "-Wl,-rpath," + os.path.join(rocm, "lib")]
    subprocess.run(cmd, check=True)
    return EXE


if __name__ == "__main__":
    print(build())
