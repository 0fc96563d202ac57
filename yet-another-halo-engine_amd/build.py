"""Compiles the gfx950 kernels and the C ABI into libyahkv.so next to this file."""
import os
import subprocess
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
LIB = os.path.join(HERE, "libyahkv.so")
SOURCES = ["host.cpp", "append.hip", "decode.hip", "prefill.hip", "slots.hip", "f16kv.hip", "kv8_append.hip",
           "kv8_decode.hip", "refslot.cpp"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wextra",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",   # no packed-FP32 VALU forms
         "-mllvm", "--disable-promote-alloca-to-lds",                   # small private arrays stay out of LDS
         "-x", "hip"]
NOISE = "is not a recognized feature for this target"


def _run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if NOISE not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + err)
    return err


EXTRA = os.environ.get("YAHKV_EXTRA_FLAGS", "").split()   # e.g. -DYAHKV_PREFILL_WIDE=1 for the alternative prefill kernel


def build(verbose=False, only=None):
    """Every source is compiled (one hipcc per file, side by side) and the objects are linked. `only`: names of the
    sources to compile again, the other objects are taken as they are (for work on one kernel file)."""
    obj_dir = os.path.join(HERE, "build")
    os.makedirs(obj_dir, exist_ok=True)
    inc = ["-I", os.path.join(ROOT, "include"), "-I", os.path.join(HERE, "csrc")]
    objs = {s: os.path.join(obj_dir, os.path.splitext(s)[0] + ".o") for s in SOURCES}
    todo = [s for s in SOURCES if only is None or s in only or not os.path.exists(objs[s])]
    with ThreadPoolExecutor(max_workers=min(8, len(todo) or 1)) as ex:
        errs = list(ex.map(lambda s: _run([HIPCC] + FLAGS + EXTRA + inc + ["-c", os.path.join(HERE, "csrc", s), "-o", objs[s]]),
                           todo))
    errs.append(_run([HIPCC, "--offload-arch=gfx950", "-fPIC", "-shared"] + [objs[s] for s in SOURCES] + ["-o", LIB]))
    if verbose and any(e.strip() for e in errs):
        print("\n".join(e for e in errs if e.strip()))
    return LIB


if __name__ == "__main__":
    import sys
    print(build(verbose=True, only=sys.argv[1:] or None))
