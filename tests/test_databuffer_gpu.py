"""DataBuffer entry points of the C ABI (reference: legacy/NativeOps.h:464-482, array/cuda/DataBuffer.cu:367-413) on
buffers below and above the size from which the library page-locks the host side it allocates."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

FLOAT32 = 5
SIZES = [1000, 200_000, 300_000, 3_000_000]   # 4 KB, 0.8 MB (pageable) / 1.2 MB, 12 MB (page-locked)


def host(L, db, n):
    p = L.dbPrimaryBuffer(db)
    assert p
    return np.frombuffer((ctypes.c_char * (4 * n)).from_address(p), dtype=np.float32, count=n)


@pytest.mark.parametrize("n", SIZES)
def test_round_trip_through_the_device_copy(ex, n):
    from deeplearning4j_amd import nativeops as N
    L = ex.L
    db = L.dbAllocateDataBuffer(n, FLOAT32, True)
    N.check("dbAllocateDataBuffer")
    h = host(L, db, n)
    assert not h.any()                      # fresh buffers are zero-filled
    want = np.random.default_rng(n).standard_normal(n).astype(np.float32)
    h[:] = want
    L.dbTickHostWrite(db)
    L.dbSyncToSpecial(db)
    N.check("dbSyncToSpecial")
    h[:] = -1.0                             # the host side may be rewritten as soon as the sync returns
    L.dbTickDeviceWrite(db)                 # ... and the device side counts as the newer one
    L.dbSyncToPrimary(db)
    N.check("dbSyncToPrimary")
    assert np.array_equal(host(L, db, n), want)
    L.deleteDataBuffer(db)


@pytest.mark.parametrize("n", SIZES)
def test_expand_keeps_both_sides_and_zero_fills_the_rest(ex, n):
    from deeplearning4j_amd import nativeops as N
    L = ex.L
    db = L.dbAllocateDataBuffer(n, FLOAT32, True)
    want = np.arange(n, dtype=np.float32)
    host(L, db, n)[:] = want
    L.dbTickHostWrite(db)
    L.dbSyncToSpecial(db)
    L.dbExpand(db, 2 * n)                   # crosses the page-locking size for the third case
    N.check("dbExpand")
    assert L.dbBufferLength(db) == 2 * n
    h = host(L, db, 2 * n)
    assert np.array_equal(h[:n], want) and not h[n:].any()
    h[:] = 7.0
    L.dbTickDeviceWrite(db)
    L.dbSyncToPrimary(db)
    h = host(L, db, 2 * n)
    assert np.array_equal(h[:n], want) and not h[n:].any()
    L.deleteDataBuffer(db)


def test_caller_memory_replaces_an_owned_host_side(ex):
    from deeplearning4j_amd import nativeops as N
    L = ex.L
    n = 1_000_000                           # the owned host side is page-locked and must be released as such
    db = L.dbAllocateDataBuffer(n, FLOAT32, True)
    mine = np.linspace(0, 1, n, dtype=np.float32)
    L.dbSetPrimaryBuffer(db, mine.ctypes.data, 4 * n)
    N.check("dbSetPrimaryBuffer")
    assert L.dbPrimaryBuffer(db) == mine.ctypes.data
    L.dbSyncToSpecial(db)
    keep = mine.copy()
    mine[:] = 0
    L.dbTickDeviceWrite(db)
    L.dbSyncToPrimary(db)
    assert np.array_equal(mine, keep)
    L.deleteDataBuffer(db)                  # must not free the caller's memory
    assert np.array_equal(mine, keep)
