"""Host-side checks that need no GPU: the C ABI library loads and exports every entry point include/yahkv.h declares,
geometry and size functions, page-table validation (the reference throws on an out-of-range entry,
engine/model/loom_prefill.hpp:1314-1316) and the page allocator's invariants."""
import ctypes as C
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "yahkv.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(yahkv_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_entry_point(yahkv):
    names = declared_functions()
    assert len(names) >= 20 and "yahkv_append" in names and "yahkv_prefill_attend" in names
    for n in names:
        assert hasattr(yahkv.lib, n), f"{n} is declared in include/yahkv.h but not exported by libyahkv.so"
    assert yahkv.lib.yahkv_version().startswith(b"yahkv")
    assert yahkv.status_text(0) == "ok" and "geometry" in yahkv.status_text(-2)


def test_geometry_and_pool_sizes(yahkv):
    g = yahkv.geometry(yahkv.Q8_0, 24, 4, 256, 64, 1024)
    b = yahkv.pool_bytes(g)
    assert b == {"kq": 1024 * 4 * 256 * 64, "ks": 1024 * 4 * 64 * 8 * 2, "vq": 1024 * 4 * 256 * 64, "vs": 1024 * 4 * 64 * 8 * 2}
    assert yahkv.lib.yahkv_bytes_per_token(C.byref(g)) == 2176           # 2 x 4 heads x 8 blocks x 34 B
    g4 = yahkv.geometry(yahkv.Q4_0, 24, 4, 256, 64, 1024)
    assert yahkv.lib.yahkv_bytes_per_token(C.byref(g4)) == 1152          # 18-byte blocks
    assert yahkv.pool_bytes(g4)["kq"] == b["kq"] // 2 and yahkv.pool_bytes(g4)["ks"] == b["ks"]
    assert sum(b.values()) == 1024 * 64 * 2176
    for bad in [(8, 24, 4, 192, 64, 8), (8, 24, 5, 256, 64, 8), (8, 36, 4, 256, 64, 8), (8, 24, 4, 256, 48, 8), (5, 24, 4, 256, 64, 8)]:
        with pytest.raises(yahkv.YahkvError) as e:
            yahkv.geometry(*bad)
        assert e.value.status == -2
    with pytest.raises(yahkv.YahkvError) as e:
        yahkv.geometry(8, 24, 4, 256, 64, 0)
    assert e.value.status == -1
    assert yahkv.decode_workspace_bytes(g, 64, 65536) > 0
    assert yahkv.decode_workspace_bytes(g, 64, 65536) >= yahkv.decode_workspace_bytes(g, 1, 1024)
    assert yahkv.decode_workspace_bytes(g, 0, 10) == 0


def test_validate_page_table(yahkv):
    g = yahkv.geometry(yahkv.Q8_0, 8, 2, 128, 16, 10)
    table = np.array([[0, 1, 2, 9], [3, 4, 5, 6]], np.int32)
    yahkv.validate_page_table(g, table, [64, 33])
    for bad, lens in [(np.array([[0, 1, 2, 10], [3, 4, 5, 6]]), [64, 33]),      # out of range
                      (np.array([[0, 1, 2, -1], [3, 4, 5, 6]]), [64, 33]),      # negative
                      (np.array([[0, 1, 2, 3], [3, 4, 5, 6]]), [64, 33]),       # page 3 used twice
                      (table, [65, 33])]:                                       # longer than the table's extent
        with pytest.raises(yahkv.YahkvError) as e:
            yahkv.validate_page_table(g, bad, lens)
        assert e.value.status == -3
    yahkv.validate_page_table(g, np.array([[0, 1, 2, 77], [3, 4, 5, 6]], np.int32), [48, 33])   # unused entries are free
    with pytest.raises(yahkv.YahkvError):
        yahkv.validate_page_table(g, table, [-1, 3])


def test_page_allocator_invariants(yahkv):
    n = 97
    pool = yahkv.PagePool(n)
    assert pool.free_count == n
    a = pool.alloc(10)
    assert a == list(range(10))                                 # lowest id first
    b = pool.alloc(n - 10)
    assert sorted(a + b) == list(range(n)) and pool.free_count == 0       # no page handed out twice, pool used up
    with pytest.raises(yahkv.YahkvError) as e:
        pool.alloc(1)
    assert e.value.status == -5 and pool.free_count == 0
    pool.free([5, 50, 7])
    assert pool.free_count == 3
    assert pool.alloc(2) == [5, 7]                              # freed pages are handed out again
    for bad in ([50], [n], [-1], [60, 60], [61, 50]):           # already free / out of range / listed twice
        before = pool.free_count
        with pytest.raises(yahkv.YahkvError) as e:
            pool.free(bad)
        assert e.value.status == -3 and pool.free_count == before      # and nothing was freed
    pool.close()
    # a shuffled pool still hands out every page exactly once ("pool sized to fit exactly")
    pool = yahkv.PagePool(1000)
    pool.shuffle(12345)
    got = pool.alloc(1000)
    assert sorted(got) == list(range(1000)) and got != list(range(1000))
    other = yahkv.PagePool(1000)
    other.shuffle(12345)
    assert other.alloc(1000) == got                             # seeded: reproducible
    rng = np.random.default_rng(0)                              # random alloc / free: allocated + free == pool
    pool = yahkv.PagePool(64)
    held = []
    for _ in range(300):
        if held and rng.random() < 0.5:
            k = int(rng.integers(1, len(held) + 1))
            idx = rng.permutation(len(held))[:k]
            pool.free([held[i] for i in idx])
            held = [p for i, p in enumerate(held) if i not in set(idx.tolist())]
        else:
            k = int(rng.integers(0, 9))
            if k <= pool.free_count:
                held += pool.alloc(k)
        assert len(set(held)) == len(held) and len(held) + pool.free_count == 64 and all(0 <= p < 64 for p in held)


def test_page_owner_counts(yahkv):
    """retain / free: a page returns to the free list only when its last owner lets go."""
    pool = yahkv.PagePool(8)
    a = pool.alloc(3)
    assert [pool.refcount(p) for p in a] == [1, 1, 1] and pool.refcount(7) == 0 and pool.refcount(8) == -1
    pool.retain(a[:2])                                   # a fork shares the first two pages
    assert [pool.refcount(p) for p in a] == [2, 2, 1]
    pool.free(a)                                         # the parent lets go: only the unshared page is free again
    assert pool.free_count == 6 and [pool.refcount(p) for p in a] == [1, 1, 0]
    with pytest.raises(yahkv.YahkvError) as e:
        pool.retain([a[2]])                              # a free page cannot gain an owner
    assert e.value.status == -3
    with pytest.raises(yahkv.YahkvError) as e:
        pool.free([a[0], a[0]])                          # the same page twice in one call
    assert e.value.status == -3
    pool.free(a[:2])
    assert pool.free_count == 8
    assert pool.alloc(8) == list(range(8))               # lowest id first again
    assert yahkv.lib.yahkv_slot_bytes(__import__("ctypes").byref(yahkv.geometry(8, 24, 4, 256, 64, 4)), 3) == \
        64 + 3 * sum(yahkv.pool_bytes(yahkv.geometry(8, 24, 4, 256, 64, 1)).values())


def test_undersized_pools_are_refused_before_any_launch(yahkv):
    """Every entry point that takes pools refuses a buffer shorter than the geometry needs (the reference refuses an
    undersized binding: engine/run/hal_run.cc:110-114, loom_decoder.hpp:186-203). The refusal comes before anything
    is launched, so the addresses here need not exist (and no GPU is needed)."""
    lib = yahkv.lib
    g = yahkv.geometry(yahkv.Q8_0, 24, 4, 256, 64, 8)
    need = yahkv.pool_bytes(g)
    fake = 0x10000                                        # a 16-byte aligned address nothing dereferences
    ok = dict(kq=need["kq"], ks=need["ks"], vq=need["vq"], vs=need["vs"])
    for short in ("kq", "ks", "vq", "vs"):
        n = dict(ok)
        n[short] -= 1
        p = yahkv.Pools(fake, fake, fake, fake, n["kq"], n["ks"], n["vq"], n["vs"])
        r, pr = C.byref(g), C.byref(p)
        ws = 1 << 30
        assert lib.yahkv_append(r, pr, fake, 4, fake, None, 1, 1, fake, fake, 0, None) == -1, short
        rope = yahkv.Rope(1e6, 1e-6, 64, None, None)
        assert lib.yahkv_append_rope(r, pr, fake, 4, fake, None, 1, 1, fake, fake, 0, C.byref(rope), None, None, 0, None,
                                     None) == -1
        assert lib.yahkv_decode_part(r, pr, fake, 4, fake, 1, 100, fake, 2, 0.1, fake, ws, None, None) == -1
        assert lib.yahkv_decode_attend(r, pr, fake, 4, fake, 1, 100, fake, 2, 0.1, None, fake, fake, ws, None, None) == -1
        assert lib.yahkv_decode_attend_static(r, pr, fake, 4, fake, 1, 100, fake, 2, 0.1, None, fake, None) == -1
        assert lib.yahkv_decode_step(r, pr, fake, 4, fake, 1, 100, fake, fake, 2, fake, 2, 0.1, None, fake, fake, ws, None,
                                     None) == -1
        assert lib.yahkv_prefill_attend(r, pr, fake, 4, fake, 1, 64, 64, fake, 0.1, None, fake, 0, fake, ws, None) == -1
        assert lib.yahkv_prefill_decode_tiles(r, pr, fake, 4, fake, 1, 64, 64, fake, ws, None) == -1
        assert lib.yahkv_gather_blocks(r, pr, fake, 10, fake, fake, None) == -1
        assert lib.yahkv_copy_pages(r, pr, fake, fake, 1, None) == -1
        assert lib.yahkv_slot_pack(r, pr, fake, 1, 10, fake, None) == -1
        assert lib.yahkv_slot_unpack(r, pr, fake, 1, fake, None) == -1
    # a misaligned or missing pool is refused the same way
    for kq in (fake + 8, 0):
        p = yahkv.Pools(kq, fake, fake, fake, ok["kq"], ok["ks"], ok["vq"], ok["vs"])
        assert lib.yahkv_append(C.byref(g), C.byref(p), fake, 4, fake, None, 1, 1, fake, fake, 0, None) == -1
    # the f16 twins
    g16 = yahkv.f16_geometry(24, 4, 256, 64, 8)
    n16 = lib.yahkv_f16_pool_bytes(C.byref(g16))
    for kb, vb in ((n16 - 1, n16), (n16, n16 - 1)):
        p = yahkv.F16PoolsStruct(fake, fake, kb, vb)
        assert lib.yahkv_f16_append(C.byref(g16), C.byref(p), fake, 4, fake, None, 1, 1, fake, fake, 0, None) == -1
        assert lib.yahkv_f16_decode_attend(C.byref(g16), C.byref(p), fake, 4, fake, 1, 100, fake, 2, 0.1, None, fake, fake,
                                           1 << 30, None, None) == -1
        assert lib.yahkv_f16_prefill_attend(C.byref(g16), C.byref(p), fake, 4, fake, 1, 64, 64, fake, 0.1, None, fake, 0,
                                            fake, 1 << 30, None) == -1


def test_slot_header_must_name_exactly_the_pages_its_tokens_fill(yahkv):
    """A loader scatters as many pages as the header names: a header with more pages than ceil(tokens / page_tokens),
    or with no tokens, is refused (the reference's LoadState checks its sizes exactly, loom_prefill.hpp:976-1024)."""
    g = yahkv.geometry(yahkv.Q8_0, 8, 2, 128, 16, 16)

    def header(pages, tokens):
        n = yahkv.lib.yahkv_slot_bytes(C.byref(g), pages)
        buf = np.zeros(n, np.uint8)
        buf[:64].view(np.uint64)[:] = [int.from_bytes(b"YKVSLOT1", "little"), 8, 2, 128, 16, pages, tokens, 4]
        return buf

    assert yahkv.slot_check(g, header(3, 33)) == (3, 33)
    assert yahkv.slot_check(g, header(3, 48)) == (3, 48)
    for pages, tokens in ((3, 32), (3, 0), (2, 33), (5, 17)):
        with pytest.raises(yahkv.YahkvError) as e:
            yahkv.slot_check(g, header(pages, tokens))
        assert e.value.status == -1, (pages, tokens)


def test_decode_options_change_only_what_they_name(yahkv):
    g = yahkv.geometry(yahkv.Q8_0, 24, 4, 256, 64, 1024)
    base = yahkv.decode_workspace_bytes(g, 64, 65536)
    assert yahkv.decode_workspace_bytes(g, 64, 65536, yahkv.decode_options()) == base          # zero fields: defaults
    assert yahkv.decode_workspace_bytes(g, 64, 65536, yahkv.decode_options(deterministic=True, pair_cost=-1,
                                                                           xcd_weight=[3, 1, 4, 1, 5, 9, 2, 6])) == base
    assert yahkv.decode_workspace_bytes(g, 64, 65536, yahkv.decode_options(n_chunks=512)) > base


def test_header_is_plain_c(tmp_path):
    """include/yahkv.h is the boundary a C, cgo or JNI binding includes: it must compile as C99 without warnings, and a C
    program must link against the library with nothing but the header."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = tmp_path / "t.c"
    src.write_text('#include <stdio.h>\n#include "yahkv.h"\n'
                   "int main(void) {\n"
                   "  yahkv_geometry g = {YAHKV_Q8_0, 24, 4, 256, 64, 8};\n"
                   "  yahkv_decode_options o = {0};\n"
                   '  printf("%zu %zu %d\\n", yahkv_kq_bytes(&g), yahkv_decode_workspace_bytes(&g, 2, 1000, &o),\n'
                   "         yahkv_check_geometry(&g));\n"
                   "  return 0;\n}\n")
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", os.path.join(root, "include"),
                    "-fsyntax-only", str(src)], check=True)
    pkg = os.path.join(root, "yet-another-halo-engine_amd")
    exe = tmp_path / "t"
    r = subprocess.run(["gcc", "-std=c99", "-I", os.path.join(root, "include"), str(src), "-L", pkg, "-lyahkv",
                        "-Wl,-rpath," + pkg, "-Wl,-rpath,/opt/rocm/lib", "-L/opt/rocm/lib", "-o", str(exe)],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    out = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stderr[-2000:]
    kq, ws, ok = out.stdout.split()
    assert int(kq) == 8 * 4 * 8 * 64 * 32 and int(ws) > 0 and int(ok) == 0
