"""The C++ host classes of csrc/kv_cache.hpp (KvDecoder / KvPrefill / PagePool, the reference's LoomDecoder surface)
run as a standalone program against the CPU oracle. The program is compiled by __graft_entry__.build()."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "kv_cache_test")


@pytest.mark.gpu
def test_kv_cache_cpp_program():
    assert os.path.exists(BIN), "tests/cpp/kv_cache_test is not built: run `python __graft_entry__.py build`"
    r = subprocess.run([BIN], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "kv_cache_test: ok" in r.stdout


def test_kv_cache_header_is_host_only_cxx():
    """The header compiles as plain host C++ against the C ABI (no device code, no torch)."""
    src = '#include "kv_cache.hpp"\nint main() { return sizeof(yahkv_host::KvDecoder) > 0 ? 0 : 1; }\n'
    r = subprocess.run(["/opt/rocm/bin/hipcc", "-std=c++17", "-fsyntax-only", "-x", "c++", "-D__HIP_PLATFORM_AMD__",
                        "-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROOT, "yet-another-halo-engine_amd", "csrc"),
                        "-I", "/opt/rocm/include", "-"], input=src, capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
