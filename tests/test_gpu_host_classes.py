"""The C++ host classes of csrc/kv_cache.hpp (KvDecoder / KvPrefill / PagePool, the reference's LoomDecoder surface)
and the continuous-batching driver of csrc/kv_batcher.hpp run as standalone programs against the CPU oracle. The
programs are compiled by __graft_entry__.build()."""
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


@pytest.mark.gpu
def test_kv8_cache_cpp_program():
    """Kv8Decoder / Kv8Prefill (the reference's own KV format): chunks, steps across tiles and a page, a sequence that
    starts with steps, the contiguity rule of the open V tile; buffers bit for bit against the oracle of that format."""
    exe = os.path.join(ROOT, "tests", "cpp", "kv8_cache_test")
    assert os.path.exists(exe), "tests/cpp/kv8_cache_test is not built: run `python __graft_entry__.py build`"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "kv8_cache_test: ok" in r.stdout


@pytest.mark.gpu
def test_kv_batcher_cpp_program():
    """Twelve requests through a pool too small for them: waiting, side by side, put back and started again; every
    attention row against the oracle, every finished request's blocks bit-exact, no page lost."""
    exe = os.path.join(ROOT, "tests", "cpp", "kv_batcher_test")
    assert os.path.exists(exe), "tests/cpp/kv_batcher_test is not built: run `python __graft_entry__.py build`"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "kv_batcher_test: ok" in r.stdout


def test_kv_cache_header_is_host_only_cxx():
    """The headers compile as plain host C++ against the C ABI (no device code, no torch)."""
    src = ('#include "kv_batcher.hpp"\n'
           'int main() { return sizeof(yahkv_host::KvDecoder) + sizeof(yahkv_host::KvBatcher) > 0 ? 0 : 1; }\n')
    r = subprocess.run(["/opt/rocm/bin/hipcc", "-std=c++17", "-fsyntax-only", "-x", "c++", "-D__HIP_PLATFORM_AMD__",
                        "-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROOT, "yet-another-halo-engine_amd", "csrc"),
                        "-I", "/opt/rocm/include", "-"], input=src, capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr


@pytest.mark.gpu
def test_kv8_batcher_cpp_program():
    """The same driver over pools in the reference's own formats (kv8a16, then kv4a16): ten requests through five
    pages, chunks that start inside tiles and pages, first and later chunks in one step; all six buffers of both layers
    bit for bit against the oracle after every step, attention rows against the closed form."""
    exe = os.path.join(ROOT, "tests", "cpp", "kv8_batcher_test")
    assert os.path.exists(exe), "tests/cpp/kv8_batcher_test is not built: run `python __graft_entry__.py build`"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=200)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.count("kv8_batcher_test: ok") == 2
