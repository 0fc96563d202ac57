"""Compiles the gfx950 kernels and the C ABI into libyahkv.so next to this file."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
LIB = os.path.join(HERE, "libyahkv.so")
SOURCES = ["host.cpp", "append.hip", "decode.hip", "prefill.hip", "slots.hip", "f16kv.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",   # no packed-FP32 VALU forms
         "-mllvm", "--disable-promote-alloca-to-lds",                   # small private arrays stay out of LDS
         "-x", "hip"]


def build(verbose=False):
    srcs = [os.path.join(HERE, "csrc", s) for s in SOURCES]
    cmd = [HIPCC] + FLAGS + ["-I", os.path.join(ROOT, "include"), "-I", os.path.join(HERE, "csrc")] + srcs + ["-o", LIB]
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in r.stderr.splitlines() if noise not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + err)
    if verbose and err.strip():
        print(err)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
