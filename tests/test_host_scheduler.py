"""BatchScheduler (csrc/kv_batcher.hpp), the bookkeeping of the continuous-batching driver: a C++ program without any
GPU call runs random workloads and checks the page and queue invariants after every step (tests/cpp/
kv_scheduler_test.cc). The program is compiled by __graft_entry__.build(); it is built here if it is missing."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "kv_scheduler_test")


def test_scheduler_invariants_over_random_workloads():
    if not os.path.exists(BIN):
        sys.path.insert(0, ROOT)
        import __graft_entry__
        __graft_entry__.build_host_test()
    r = subprocess.run([BIN, "300"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "kv_scheduler_test: ok" in r.stdout
