"""The HBM pool through the C ABI (paras_alloc / paras_free / paras_empty_cache / paras_memory_stats):
reuse by size class, what `allocated` and `cached` count, and the order in which idle blocks go
back to the driver when hipMalloc runs out (contract: csrc/core/allocator.cpp:53-122 of the
reference, with the out-of-memory behaviour this build adds)."""
import ctypes as C

import pytest

import capi

pytestmark = pytest.mark.gpu
MiB = 1 << 20


def stats(L):
    a, c = C.c_uint64(), C.c_uint64()
    assert L.paras_memory_stats(0, C.byref(a), C.byref(c)) == 0
    return a.value, c.value


def alloc(L, n):
    p = C.c_void_p()
    rc = L.paras_alloc(0, n, C.byref(p))
    return rc, p


def test_blocks_are_reused_by_size_class_and_counted():
    L = capi.lib()
    assert L.paras_empty_cache(0) == 0
    a0, c0 = stats(L)
    assert c0 == 0
    rc, p = alloc(L, 3 * MiB)                     # rounds to 4 MiB
    assert rc == 0 and stats(L) == (a0 + 4 * MiB, 0)
    assert L.paras_free(0, p) == 0
    assert stats(L) == (a0 + 4 * MiB, 4 * MiB)    # idle, still held
    rc, q = alloc(L, 4 * MiB)                     # same class: the same block comes back
    assert rc == 0 and q.value == p.value and stats(L) == (a0 + 4 * MiB, 0)
    rc, r = alloc(L, 5 * MiB)                     # another class: a new block
    assert rc == 0 and r.value != q.value and stats(L) == (a0 + 12 * MiB, 0)
    assert L.paras_free(0, q) == 0 and L.paras_free(0, r) == 0
    assert L.paras_free(0, r) != 0                # a pointer the pool does not hold as in use
    assert b"unknown pointer" in L.paras_last_error()
    assert L.paras_empty_cache(0) == 0
    assert stats(L) == (a0, 0)


def test_sizes_above_one_gib_share_a_bin_but_not_blocks():
    L = capi.lib()
    assert L.paras_empty_cache(0) == 0
    a0, _ = stats(L)
    big, bigger = (1 << 30) + 1, (1 << 30) + 300 * MiB          # 1.25 GiB and 1.5 GiB classes
    rc, p = alloc(L, big)
    rc2, q = alloc(L, bigger)
    assert rc == 0 and rc2 == 0 and stats(L)[0] == a0 + 1280 * MiB + 1536 * MiB
    assert L.paras_free(0, p) == 0 and L.paras_free(0, q) == 0
    rc, r = alloc(L, big)                                       # the 1.25 GiB block, not the 1.5 GiB one
    assert rc == 0 and r.value == p.value
    assert L.paras_free(0, r) == 0 and L.paras_empty_cache(0) == 0
    assert stats(L) == (a0, 0)


def test_out_of_memory_gives_idle_blocks_back_and_reports():
    """A request the device cannot hold: every idle block has gone back to the driver by the time
    the call gives up, the call fails with an out-of-memory status, and the pool still works."""
    L = capi.lib()
    assert L.paras_empty_cache(0) == 0
    a0, _ = stats(L)
    held = [alloc(L, n)[1] for n in (64 * MiB, 512 * MiB, 2 * MiB)]
    for p in held:
        assert L.paras_free(0, p) == 0
    assert stats(L) == (a0 + 578 * MiB, 578 * MiB)
    rc, _ = alloc(L, 1 << 46)                                   # 64 TiB
    assert rc != 0 and b"hipMalloc" in L.paras_last_error()
    assert stats(L) == (a0, 0)
    rc, p = alloc(L, MiB)
    assert rc == 0 and L.paras_free(0, p) == 0 and L.paras_empty_cache(0) == 0
